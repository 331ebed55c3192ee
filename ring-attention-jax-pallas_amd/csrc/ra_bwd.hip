// Backward ring step for gfx950, recomputing the probabilities from the saved logsumexp.
//
// Two kernels per step, both deterministic (no atomics):
//  * dkdv_kernel: a workgroup owns a slab of keys (its K/V operands live in registers, its
//    dK/dV accumulators too) and streams 32-query tiles of Q and dO through LDS.  Scores
//    are produced as S = Q K^T so that an accumulator lane owns one key and 16 queries:
//    P and dS are then directly the A operands of dV = P^T dO and dK = dS^T Q, whose B
//    operands come from the Q / dO tiles through the transposing LDS read.
//  * dq_kernel: a wave owns 32 queries (Q and dO operands in registers) and streams
//    32-key tiles of K and V through four LDS buffers.  Scores are produced transposed (S^T = K Q^T),
//    exactly as in the forward kernel, so dS^T is the B operand of dQ^T = K^T dS^T.
// Plus the elementwise delta = rowsum(out * dout) and the fp32 -> bf16 gradient cast.
#include <type_traits>

#include "ra_launch.h"

namespace ra {

constexpr int kBwdMaxListTiles = 2048;

// ------------------------------------------------------------------------------------------------
// delta
// ------------------------------------------------------------------------------------------------
// n_pass shards per launch: shard p reads out + p * sp and dout.ptr + p * dsp and writes the p-th
// [B, H, Lq] block of delta.
template <typename OutT, int D>
__global__ void bwd_delta_kernel(const OutT* out, long long sp, long long sb, long long sh, long long sl,
                                 TensorArg dout, long long dsp, float* delta, int n_pass, int B, int H, int Lq) {
  constexpr int CPR = D / 8;           // lanes per row
  constexpr int RPB = 256 / CPR;       // rows per block
  const int tid = threadIdx.x;
  const long long row = (long long)blockIdx.x * RPB + tid / CPR;
  const int c = tid % CPR;
  const long long rows = (long long)n_pass * B * H * Lq;
  float acc = 0.f;
  if (row < rows) {
    const int li = (int)(row % Lq);
    const int h = (int)((row / Lq) % H);
    const long long bp = row / ((long long)Lq * H);
    const int b = (int)(bp % B);
    const long long ps = bp / B;
    const OutT* op = out + ps * sp + b * sb + h * sh + (long long)li * sl + 8 * c;
    const bf16_t* dp = dout.ptr + ps * dsp + b * dout.sb + h * dout.sh + (long long)li * dout.sl + 8 * c;
    bf16x8 dv = *(const bf16x8*)dp;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc += (float)op[e] * (float)dv[e];
  }
#pragma unroll
  for (int o = CPR / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
  if (row < rows && c == 0) delta[row] = acc;
}

// ------------------------------------------------------------------------------------------------
// dK / dV
// ------------------------------------------------------------------------------------------------
constexpr int kQTile = 32;  // queries per LDS tile in dkdv_kernel

// s_waitcnt with only the vector-memory counter set (expcnt, lgkmcnt left at their maxima)
#define RA_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(0x0f70 | ((n) & 15) | (((n) >> 4) << 14))

// One workgroup = 4 waves = 128 keys; every wave owns 32 keys for the whole kernel: their K
// and V rows sit in registers as MFMA B operands (K already multiplied by sm_scale * log2(e))
// and the 32 x D dK and dV accumulators in accumulation registers (one wave per SIMD, 512
// registers).  32-query tiles of Q and dO stream through six LDS buffers with direct-to-LDS loads
// requested three tiles ahead; a tile's per-row statistics (-lse * log2(e), -delta) travel next
// to it and enter the score and dP accumulators as the MFMA chains' initial C operand.
// Iteration i, after its barrier, first runs the 16 MFMAs of dV += P(i-1)^T dO, dK += dS(i-1)^T Q
// (operands visible before the barrier, so their fetch straddles it; the next tile's loads and
// the hand-over of S(i), dP(i) to the vector ALU issue in their shadow), then the 16 MFMAs of
// S(i+1) = Q K^T and dP(i+1) = dO V^T with the exp2 / dS arithmetic of tile i in theirs.
// MULTI: grid dimension y is a ring pass, one key/value shard with its dk / dv.  The launch walks
// the query shards that `ring` lists for the pass one after another (the query side of the ring
// steps that this key/value shard takes part in); dK / dV stay in registers between them.
template <int D, int MODE, bool MULTI>
__global__ __launch_bounds__(256) void dkdv_kernel(
    const BwdArgs a, const std::conditional_t<MULTI, QRing, NoShardList> ring) {
  constexpr bool GENERAL = MODE != 0;  // bias terms beyond causal / window
  constexpr bool DENSE = MODE == 2;    // ... including a materialised bias block
  constexpr int NT = 256;
  constexpr int KS = D / 16;
  constexpr int DB = D / 32;
  constexpr int KEYS_WG = 128;
  constexpr int ROWB = D * 2;
  constexpr int TILE_BYTES = kQTile * ROWB;
  constexpr int NB = 6;                    // LDS tile buffers; tile j lives in buffer j % NB
  constexpr int NSTAT = GENERAL ? 4 : 2;   // per-row words that travel with a tile
  constexpr int STAT_BYTES = 4 * kQTile * 4;

  __shared__ __attribute__((aligned(16))) char s_q[NB][TILE_BYTES];
  __shared__ __attribute__((aligned(16))) char s_do[NB][TILE_BYTES];
  // per tile and row: -lse * log2(e) / scale_res (-inf for a fully masked row), -delta, segment id, prefix flag
  __shared__ __attribute__((aligned(16))) char s_stat[NB][STAT_BYTES];
  // the same words as they arrive from memory, one per lane and tile (see store_stat)
  __shared__ __attribute__((aligned(16))) unsigned s_raw[NB][NT];
  __shared__ unsigned short s_list[GENERAL ? kBwdMaxListTiles : 1];
  __shared__ unsigned char s_flag[GENERAL ? kBwdMaxListTiles : 1];
  __shared__ int s_red[20];
  // GENERAL: per wave and stretch of straight-line iterations: first tile ordinal, end, tile base
  __shared__ int s_st[GENERAL ? 4 : 1][12];
  // A operand of the matrix instruction that adds the ALiBi term to a fresh score tile
  __shared__ __attribute__((aligned(16))) bf16x8 s_ramp[GENERAL ? 64 : 1];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);  // same value in a scalar register
  const int l32 = lane & 31, g = lane >> 5;
  const int nkt = (a.Lk + KEYS_WG - 1) / KEYS_WG;
  int hh, kt;
  decode_block(blockIdx.x, a.B * a.H, nkt, hh, kt);
  kt = nkt - 1 - kt;  // under a causal mask the FIRST key slab has the most work
  const int b = hh / a.H, h = hh % a.H;
  const int k0 = kt * KEYS_WG;
  const int kw = k0 + wave * 32;
  const BiasArgs& bs = a.bias;
  const int flags = bs.flags;
  const bool wave_on = kw < a.Lk;
  // the key/value side of this workgroup's pass
  auto pass_kv_off = [&]() -> int { if constexpr (MULTI) return ring.kv_off[blockIdx.y]; else return bs.kv_off; };

  // ---- resident key-side operands ----------------------------------------------------------
  // K is multiplied once, here, by the power of two below sm_scale * log2(e) - exact in bf16 - so
  // that the score MFMAs deliver S * sm_scale * log2(e) / scale_res; the residual factor
  // scale_res in [1, 2) is applied to the fp32 score in front of exp2, and everything that is
  // added to a score tile (the row statistics, bias terms) is divided by it.  Folding the whole
  // scale into the bf16 operand would perturb every probability by ~1e-3 relative (more with a
  // wider score spread) and break the agreement with the forward pass's logsumexp.
  // They live in accumulation registers (the matrix unit reads its B operand from either file),
  // which leaves the vector registers to the score pipeline.
  u32x4 kfa[KS], vfa[KS];
  int k_seg = 0, k_pre = 0;
  {
    bf16x8 kf[KS], vf[KS];
    const int ki = min(kw + l32, a.Lk - 1);
    const bf16_t* k_res = a.k.ptr;
    const bf16_t* v_res = a.v.ptr;
    const int* kv_seg_res = bs.kv_seg;
    const int* kv_pre_res = bs.kv_pre;
    if constexpr (MULTI) {
      k_res = ring.k[blockIdx.y];
      v_res = ring.v[blockIdx.y];
      kv_seg_res = ring.kv_seg[blockIdx.y];
      kv_pre_res = ring.kv_pre[blockIdx.y];
    }
    const bf16_t* kp = k_res + b * a.k.sb + h * a.k.sh + (long long)ki * a.k.sl + 8 * g;
    const bf16_t* vp = v_res + b * a.v.sb + h * a.v.sh + (long long)ki * a.v.sl + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const bf16x8 kr = *(const bf16x8*)(kp + 16 * s);
#pragma unroll
      for (int e = 0; e < 8; ++e) kf[s][e] = (bf16_t)((float)kr[e] * a.scale_p2);
      vf[s] = *(const bf16x8*)(vp + 16 * s);
    }
    if (GENERAL && (flags & RA_BIAS_SEGMENT)) k_seg = kv_seg_res[b * bs.kv_seg_sb + ki];
    if (GENERAL && (flags & RA_BIAS_PREFIX)) k_pre = kv_pre_res[b * bs.kv_pre_sb + ki];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      // an empty statement whose result is bound to accumulation registers: the compiler
      // copies the four words there, and the fragment stays one aligned register tuple
      asm volatile("" : "=a"(kfa[s]) : "0"(__builtin_bit_cast(u32x4, kf[s])));
      asm volatile("" : "=a"(vfa[s]) : "0"(__builtin_bit_cast(u32x4, vf[s])));
    }
  }
  // acc += A x B with the accumulator in VECTOR registers and B in accumulation registers.  The
  // compiler gives every matrix instruction of a kernel the same register class for its result;
  // this kernel wants dK / dV in accumulation registers for the whole loop and the score tiles in
  // vector registers, where the vector ALU reads them without a copy, hence the assembly.  No
  // instruction depends on the result for hundreds of cycles (the next use of a score tile is
  // one iteration away; chained accumulations alternate between two tiles).
  auto mfma_scores = [&](f32x16& acc, const bf16x8& av, const u32x4& b_acc) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(av), "a"(b_acc));
  };
  // the same with B in vector registers
  auto mfma_scores_v = [&](f32x16& acc, const bf16x8& av, const bf16x8& bv) {
    // (the B operand was assembled by vector instructions just before: two wait states, which
    // the compiler would see to for one of its own matrix instructions)
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(av), "v"(bv));
  };
  if (GENERAL && tid < 64) {
    // row l32 of the 32 x 16 operand is [i, i, 1, 1, 1, 0 ...] with i = l32 the query's index in the
    // tile (exact in bf16); lanes 32..63 hold the other eight columns, all zero
    bf16x8 rf;
#pragma unroll
    for (int e = 0; e < 8; ++e) rf[e] = (bf16_t)0.f;
    if (g == 0) {
      rf[0] = rf[1] = (bf16_t)(float)l32;
      rf[2] = rf[3] = rf[4] = (bf16_t)1.0f;
    }
    s_ramp[tid] = rf;
  }
  float slope2 = 0.f;
  const float res = a.scale_res, inv_res = 1.0f / a.scale_res;
  if (GENERAL && (flags & RA_BIAS_ALIBI)) slope2 = bs.slopes[h] * kLog2e * inv_res;

  f32x16 dk[DB], dv[DB];
  {
    // zero the accumulators THROUGH the matrix unit so that they are born in accumulation
    // registers and stay there for the whole loop
    bf16x8 z8;
    f32x16 z16;
#pragma unroll
    for (int e = 0; e < 8; ++e) z8[e] = (bf16_t)0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) z16[r] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      dk[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(z8, z8, z16, 0, 0, 0);
      dv[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(z8, z8, z16, 0, 0, 0);
    }
  }
  // ---- one pass of everything below per query shard ------------------------------------------
  int q_off = bs.q_off;
  const bf16_t* q_ptr = a.q.ptr;
  const bf16_t* do_ptr = a.dout.ptr;
  const float* lse_ptr = a.lse;
  const float* delta_ptr = a.delta;
  const int* q_seg_ptr = bs.q_seg;
  const int* q_pre_ptr = bs.q_pre;
  const float* dense_ptr = bs.dense;
  int n_shards = 1;
  int tiles_listed = 0;  // over all shards of the pass: none, and the workgroup leaves its carry / gradients as they are
  if constexpr (MULTI) n_shards = ring.count[blockIdx.y];
  for (int shard = 0; shard < n_shards; ++shard) {
  if constexpr (MULTI) {
    const int si = ring.order[blockIdx.y][shard];
    q_off = ring.q.q_off[si];
    q_ptr = ring.q.q[si];
    do_ptr = ring.q.dout[si];
    lse_ptr = ring.q.lse[si];
    delta_ptr = ring.q.delta[si];
    q_seg_ptr = ring.q.q_seg[si];
    q_pre_ptr = ring.q.q_pre[si];
    dense_ptr = ring.q.dense[si];
    // other waves may still be reading the last tile of the previous shard
    if (shard > 0) __syncthreads();
  }
  const int* q_seg = (GENERAL && (flags & RA_BIAS_SEGMENT)) ? q_seg_ptr + b * bs.q_seg_sb : nullptr;
  const int* q_pre = (GENERAL && (flags & RA_BIAS_PREFIX)) ? q_pre_ptr + b * bs.q_pre_sb : nullptr;
  // ---- which query tiles does this workgroup visit -------------------------------------------
  const int ntiles = (a.Lq + kQTile - 1) / kQTile;
  const int k_hi = min(k0 + KEYS_WG, a.Lk) - 1;
  int i_lo, i_hi;
  const int kv_off = pass_kv_off();
  query_tile_range(flags, bs.window, kv_off + k0, kv_off + k_hi, q_off, ntiles, kQTile, i_lo, i_hi);
  int n_act = i_hi - i_lo;
  bool use_list = false;
  // Ordinals [run_lo, run_hi) are consecutive tiles `tile_base + ordinal` with one segment id
  // each: inside a straight-line stretch a lane decides per tile whether its key belongs to the
  // tile's document.  [run2_lo, run2_hi): a second such run behind the first one (a workgroup
  // that straddles a document boundary has one per document).  wg_one_doc: all keys of the
  // workgroup carry one id, so one-id tiles need no test in the generic iterations either.
  int run_lo = 0, run_hi = n_act, tile_base = i_lo;
  int run2_lo = 0, run2_hi = 0, tile_base2 = 0;
  // the listed tiles count up without a gap from the start of a run to ordinal cons_hi / cons2_hi
  int cons_hi = n_act, cons2_hi = 0;
  bool wg_one_doc = true;
  const bool seg_on = GENERAL && (flags & RA_BIAS_SEGMENT);
  const bool alibi_on = GENERAL && (flags & RA_BIAS_ALIBI);
  // A dense block that comes with its summary is listed the same way: tiles in which the
  // workgroup's keys meet nothing but -inf are left out, tiles of zeros have no term to evaluate,
  // the rest is evaluated element by element.  (Single-step launches only.)
  const unsigned char* dmap = nullptr;
  if constexpr (DENSE && !MULTI) {
    if (bs.dense_map) dmap = dense_map_of(bs, b, h, a.H, a.Lq, a.Lk);
  }
  if ((GENERAL && (flags & RA_BIAS_SEGMENT)) || (DENSE && dmap != nullptr)) {
    use_list = true;
    int kmin = 0, kmax = 0;
    if (seg_on) {
      int smin = 0x7fffffff, smax = (int)0x80000000;
      if (kw + l32 < a.Lk) {
        smin = k_seg;
        smax = k_seg;
      }
      smin = wave_min(smin);
      smax = wave_max(smax);
      if (lane == 0) {
        s_red[wave] = smin;
        s_red[4 + wave] = smax;
      }
      __syncthreads();
      kmin = s_red[0];
      kmax = s_red[4];
#pragma unroll
      for (int w = 1; w < 4; ++w) {
        kmin = min(kmin, s_red[w]);
        kmax = max(kmax, s_red[4 + w]);
      }
    }
    for (int i = i_lo + tid; i < i_hi; i += NT) {
      int f = 1;
      if (seg_on) {
        int qmin, qmax;
        tile_id_range<kQTile>(q_seg, i, a.Lq, qmin, qmax);
        const bool act = !(qmax < kmin || qmin > kmax);
        f = act ? ((qmin == qmax) ? 1 : 3) : 0;
      }
      if constexpr (DENSE) {
        if (dmap != nullptr && f != 0) {
          const int bits = dense_map_or(dmap, a.Lk, i * kQTile, min((i + 1) * kQTile, a.Lq) - 1, k0, k_hi);
          f = (bits & kMapLive) ? ((bits & kMapNonZero) ? 3 : f) : 0;
        }
      }
      s_flag[i - i_lo] = f;
    }
    wg_one_doc = kmin == kmax;
    __syncthreads();
    if (wave == 0) {
      int cnt = 0;
      for (int base = 0; base < n_act; base += 64) {
        const int i = base + lane;
        const int f = (i < n_act) ? s_flag[i] : 0;
        const unsigned long long mask = __ballot(f != 0);
        if (f) s_list[cnt + __popcll(mask & ((1ull << lane) - 1ull))] = (unsigned short)((i_lo + i) | ((f & 2) << 14));
        cnt += __popcll(mask);
      }
      int u_lo, u_hi, u_base, w_lo, w_hi, w_base;
      uniform_run(s_list, cnt, lane, 0, u_lo, u_hi, u_base);
      uniform_run(s_list, cnt, lane, u_hi, w_lo, w_hi, w_base);
      const int c_hi = consecutive_end(s_list, cnt, lane, u_lo);
      const int c2_hi = consecutive_end(s_list, cnt, lane, w_lo);
      if (lane == 0) {
        s_red[15] = c_hi;
        s_red[16] = c2_hi;
        s_red[8] = cnt;
        s_red[9] = u_lo;
        s_red[10] = u_hi;
        s_red[11] = u_base;
        s_red[12] = w_lo;
        s_red[13] = w_hi;
        s_red[14] = w_base;
      }
    }
    __syncthreads();
    n_act = s_red[8];
    run_lo = s_red[9];
    run_hi = s_red[10];
    tile_base = s_red[11];
    run2_lo = s_red[12];
    run2_hi = s_red[13];
    tile_base2 = s_red[14];
    cons_hi = s_red[15];
    cons2_hi = s_red[16];
  }
  const int n = __builtin_amdgcn_readfirstlane(n_act);
  tiles_listed += n;
  run_lo = __builtin_amdgcn_readfirstlane(run_lo);
  run_hi = __builtin_amdgcn_readfirstlane(min(run_hi, n));
  tile_base = __builtin_amdgcn_readfirstlane(tile_base);

  auto tile_at = [&](int i, int& segbit) -> int {
    if (GENERAL && use_list) {
      int e = s_list[i];
      segbit = (e >> 15) | (wg_one_doc ? 0 : 1);  // a tile of several ids, or keys of several
      return e & 0x7fff;
    }
    segbit = 0;
    return i_lo + i;
  };

  // ---- global -> LDS ---------------------------------------------------------------------------
  // every wave moves 8 of a tile's 32 rows of Q and of dO; lane l of a load instruction fills
  // physical chunk l % CPR of row l / CPR and fetches the logical chunk the XOR layout puts there
  const bf16_t* qbase = q_ptr + b * a.q.sb + h * a.q.sh;
  const bf16_t* dobase = do_ptr + b * a.dout.sb + h * a.dout.sh;
  constexpr int CPR = D / 8;
  constexpr int RPI = 64 / CPR;
  constexpr int NLD = 8 / RPI;
  constexpr int LPT = 2 * NLD + 1;  // vector-memory instructions per wave and tile
  int ld_row[NLD], ld_off[NLD];
  // per-lane byte offsets from the wave's first row; the second group of RPI rows (D = 128) rides
  // on the same scalar base through its distance, less the 1 KiB instruction offset of the paired load
  unsigned q_voff[NLD], do_voff[NLD];
#pragma unroll
  for (int t = 0; t < NLD; ++t) {
    const int rrow = 8 * wave + RPI * t + lane / CPR;
    const int pc = lane % CPR;
    ld_row[t] = rrow;
    ld_off[t] = ((tile_off<D>(rrow, pc) - rrow * ROWB) >> 4) * 8;
    q_voff[t] = (unsigned)(((long long)(lane / CPR + RPI * t) * a.q.sl + ld_off[t]) * 2 - 1024 * t);
    do_voff[t] = (unsigned)(((long long)(lane / CPR + RPI * t) * a.dout.sl + ld_off[t]) * 2 - 1024 * t);
  }
  // The per-row words of a tile: lane l of every wave fetches word class (l / 8) % NSTAT of row
  // 8 * wave + l % 8 (lanes 32..63 repeat lanes 0..31) straight into LDS, like the tile itself and
  // counted with the tile's loads, and moves it, converted, to s_stat when the tile is awaited (a
  // lane reads only what it fetched itself, so its own load counter is all it needs to watch).
  const int st_class = (lane >> 3) & (NSTAT - 1);
  const int st_row = 8 * wave + (lane & 7);
  const char* st_src;
  {
    const long long rowbase = ((long long)b * a.H + h) * a.Lq;
    const char* c0 = (const char*)(lse_ptr + rowbase);
    const char* c1 = (const char*)(delta_ptr + rowbase);
    const char* c2 = GENERAL && q_seg ? (const char*)q_seg : c0;
    const char* c3 = GENERAL && q_pre ? (const char*)q_pre : c0;
    st_src = st_class == 0 ? c0 : (st_class == 1 ? c1 : (st_class == 2 ? c2 : c3));
  }
  const unsigned st_dst = (unsigned)(st_class * (kQTile * 4) + st_row * 4);
  const float st_mul = st_class == 0 ? -kLog2e * inv_res : -1.0f;
  const float st_fix = st_class == 0 ? RA_NEG_INF : 0.f;
  auto load_stat = [&](const char* p, int buf) {
    global_to_lds4(p, RA_LDS_ADDR(&s_raw[0][0]) + buf * (NT * 4) + wave_u * 256);
  };
  auto issue_tile = [&](int it, int buf) {
    const int q0 = it * kQTile;
    const unsigned q_dst = RA_LDS_ADDR(&s_q[0][0]) + buf * TILE_BYTES + wave_u * 8 * ROWB;
    const unsigned do_dst = RA_LDS_ADDR(&s_do[0][0]) + buf * TILE_BYTES + wave_u * 8 * ROWB;
    load_stat(st_src + 4ll * min(q0 + st_row, a.Lq - 1), buf);
    if (q0 + kQTile <= a.Lq) {
      // wave-uniform row addresses in scalar registers, per-lane part in one VGPR
      const bf16_t* qs = qbase + (long long)(q0 + 8 * wave_u) * a.q.sl;
      const bf16_t* ds = dobase + (long long)(q0 + 8 * wave_u) * a.dout.sl;
      if (NLD == 2) {
        global_to_lds16_s_x2(qs, q_voff[0], q_voff[NLD - 1], q_dst);
        global_to_lds16_s_x2(ds, do_voff[0], do_voff[NLD - 1], do_dst);
      } else {
        global_to_lds16_s(qs, q_voff[0], q_dst);
        global_to_lds16_s(ds, do_voff[0], do_dst);
      }
    } else {  // last, partial tile: rows past the end repeat the last row (masked later)
#pragma unroll
      for (int t = 0; t < NLD; ++t) {
        const int gr = min(q0 + ld_row[t], a.Lq - 1);
        global_to_lds16(qbase + (long long)gr * a.q.sl + ld_off[t], q_dst + RPI * t * ROWB);
        global_to_lds16(dobase + (long long)gr * a.dout.sl + ld_off[t], do_dst + RPI * t * ROWB);
      }
    }
  };
  // The awaited tile's per-row word (the caller has waited for its load) is fetched, converted and
  // published.  In two steps where operand fetches are in flight: LDS answers a wave in order, so
  // using the word right behind its fetch would wait for every fetch issued before it.
  auto fetch_stat = [&](int buf) -> unsigned {
    asm volatile("" ::: "memory");  // the read below stays behind the wait for the load
    return s_raw[buf][tid];
  };
  auto publish_stat = [&](unsigned x, int buf) {
    // lse -> -lse * log2(e), but -inf for a fully masked row (lse = -inf) so that its P is 0;
    // delta -> -delta, but 0 for the NaN that a fully masked output row produces
    float v = __uint_as_float(x) * st_mul;
    v = (v < __builtin_inff()) ? v : st_fix;
    unsigned o = __float_as_uint(v);
    if (GENERAL) o = st_class >= 2 ? x : o;
    *(unsigned*)(&s_stat[0][0] + buf * STAT_BYTES + st_dst) = o;
  };
  auto store_stat = [&](int buf) { publish_stat(fetch_stat(buf), buf); };

  // per-lane LDS offsets of the operand fetches (the tile buffer and the 16-row step fold into
  // the instructions' immediate offsets)
  int noff[KS];
#pragma unroll
  for (int ss = 0; ss < KS; ++ss) noff[ss] = tile_off<D>(l32, 2 * ss + g);
  int toff[DB][2];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
      const int j = lane & 15;
      const int trow = 4 * g + (j >> 2) + 8 * h2;
      const int tcol = 32 * db + 16 * ((lane >> 4) & 1) + 4 * (j & 3);
      toff[db][h2] = tile_off<D>(trow, tcol >> 3) + ((tcol & 4) << 1);
    }
  auto nat_frag = [&](const char* tile, int ss) { return *(const bf16x8*)(tile + noff[ss]); };
  auto tr_frag = [&](const char* tile, int ks, int db) {
    const lds_char* p0 = (const lds_char*)(tile + 16 * ks * ROWB + toff[db][0]);
    const lds_char* p1 = (const lds_char*)(tile + 16 * ks * ROWB + toff[db][1]);
    bf16x4 x0 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) bf16x4*)p0);
    bf16x4 x1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) bf16x4*)p1);
    return __builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  // the statistics of the 16 queries an accumulator lane holds: rows 8 * bb + 4 * g + {0..3}
  const char* stat_rd = &s_stat[0][0] + 16 * g;
  auto stat_chunk = [&](int buf, int which, int bb) {
    return *(const f32x4*)(stat_rd + buf * STAT_BYTES + which * (kQTile * 4) + 32 * bb);
  };

  // positional class of this wave's 32 keys against query tile index i
  auto tile_class = [&](int i, int& qt0, int& segbit) -> int {
    qt0 = tile_at(i, segbit) * kQTile;
    if (flags & RA_BIAS_PREFIX) return 2;
    return classify_pos(flags, bs.window, q_off + qt0, q_off + qt0 + kQTile - 1, kv_off + kw,
                        kv_off + kw + 31);
  };
  // terms that every tile must evaluate; a dense block with a summary is read only in the tiles
  // that the list marks (segbit)
  int tile_terms = RA_BIAS_ALIBI | RA_BIAS_PREFIX | RA_BIAS_DENSE;
  if constexpr (DENSE) {
    if (dmap != nullptr) tile_terms &= ~RA_BIAS_DENSE;
  }
  auto needs_bias = [&](int qt0, int segbit, int cls) -> bool {
    bool nb = (cls & 2) || (qt0 + kQTile > a.Lq);
    if (GENERAL) nb = nb || (flags & tile_terms) || segbit;
    return nb;
  };
  constexpr int PFN = 4;  // operand fetches kept in flight ahead of the MFMA that uses them
  constexpr int PFT = 4;
  // S * scale2 - lse2 = Q K'^T and dP - delta = dO V^T of one tile, nothing interleaved
  auto compute_s_dp = [&](f32x16& S, f32x16& P, const char* qt, const char* dot, int buf) {
    bf16x8 fr[2 * KS];
#pragma unroll
    for (int bb = 0; bb < 4; ++bb) {
      const f32x4 t0 = stat_chunk(buf, 0, bb), t1 = stat_chunk(buf, 1, bb);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        S[4 * bb + c] = t0[c];
        P[4 * bb + c] = t1[c];
      }
    }
#pragma unroll
    for (int op = 0; op < PFN; ++op) fr[op] = nat_frag((op & 1) ? dot : qt, op >> 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int op = 0; op < 2 * KS; ++op) {
      if (op + PFN < 2 * KS) fr[op + PFN] = nat_frag(((op + PFN) & 1) ? dot : qt, (op + PFN) >> 1);
      if (op & 1) mfma_scores(P, fr[op], vfa[op >> 1]);
      else mfma_scores(S, fr[op], kfa[op >> 1]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // dV += P^T dO and dK += dS^T Q of one tile
  auto compute_dkdv = [&](const bf16x8 (&pf)[2], const bf16x8 (&dsf)[2], const char* qt, const char* dot) {
    bf16x8 fr[4 * DB];
#pragma unroll
    for (int op = 0; op < PFT; ++op) fr[op] = tr_frag((op & 1) ? qt : dot, op / (2 * DB), (op >> 1) % DB);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int op = 0; op < 4 * DB; ++op) {
      if (op + PFT < 4 * DB) {
        const int o2 = op + PFT;
        fr[o2] = tr_frag((o2 & 1) ? qt : dot, o2 / (2 * DB), (o2 >> 1) % DB);
      }
      const int ks = op / (2 * DB), db = (op >> 1) % DB;
      if (op & 1) dk[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dsf[ks], fr[op], dk[db], 0, 0, 0);
      else dv[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pf[ks], fr[op], dv[db], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // bias of a fresh S in place (rows of the accumulator are queries; S is in log2 units already)
  auto prepare = [&](f32x16& S, int qt0, int segbit, int cls, int ids_buf) {
    TileBias tb;
    tb.flags = (cls & 2) ? (flags & (RA_BIAS_CAUSAL | RA_BIAS_WINDOW)) : 0;
    if (GENERAL) {
      tb.flags |= flags & tile_terms;
      if (segbit) tb.flags |= DENSE ? (flags & (RA_BIAS_SEGMENT | RA_BIAS_DENSE)) : RA_BIAS_SEGMENT;
    }
    tb.window = bs.window;
    tb.slope2 = slope2;
    tb.dense_mul = kLog2e * inv_res;
    tb.dense = nullptr;
    tb.dense_vs = 1;
    tb.dense_vec = 0;
    tb.var_limit = a.Lq - (qt0 + 4 * g);
    const int rel0 = (q_off + qt0 + 4 * g) - (kv_off + kw + l32);
    const int* ids = (const int*)(stat_rd + ids_buf * STAT_BYTES);
    if (DENSE) {
      tb.dense = dense_ptr + b * bs.dense_sb + h * bs.dense_sh + (long long)(qt0 + 4 * g) * bs.dense_sq +
                 min(kw + l32, a.Lk - 1);
      tb.dense_vs = bs.dense_sq;
    }
    apply_bias<false, DENSE, GENERAL>(S, tb, rel0, k_seg, k_pre, ids + 2 * kQTile, ids + 3 * kQTile);
  };

  // ---- prologue: tiles 0, 1, 2 requested, S(0) and dP(0) computed ------------------------------
  {
    int sbu;
    if (n > 0) issue_tile(tile_at(0, sbu), 0);
    if (n > 1) issue_tile(tile_at(1, sbu), 1);
    if (n > 2) issue_tile(tile_at(2, sbu), 2);  // its statistics are stored in iteration 0
    __builtin_amdgcn_s_waitcnt(0);
    if (n > 0) store_stat(0);
    if (n > 1) store_stat(1);
  }
  __syncthreads();

  // Ordinals [plain_lo, plain_hi) of the query tiles this wave's keys see completely, unmasked
  // and in range: they take the fused path without any per-tile classification.
  // The per-tile-term variants have up to four such stretches (their bounds wait in LDS): under
  // ALiBi a stretch must lie on one side of the diagonal, where -slope |q_pos - kv_pos| is linear
  // in both positions (stretches 0 and 2: queries before the workgroup's keys, 1 and 3: queries
  // after them); stretches 0 and 1 lie in the first run of one-id tiles, 2 and 3 in the second.
  int plain_lo = 0, plain_hi = 0;
  if constexpr (GENERAL) {
    int st_lo[4] = {0, 0, 0, 0}, st_hi[4] = {0, 0, 0, 0};
    if (wave_on && !(flags & tile_terms & (RA_BIAS_PREFIX | RA_BIAS_DENSE))) {
      int lo, hi;
      query_tile_plain_range(flags, bs.window, kv_off + kw, kv_off + kw + 31, q_off, a.Lq / kQTile,
                             kQTile, lo, hi);
      int lo2 = hi, hi1 = hi;
      if (alibi_on) {
        // the same bounds for all waves (the workgroup's first and last key): the waves meet at a
        // barrier per tile, so a generic iteration in one of them holds up all
        hi1 = min(hi, floor_div(kv_off + k0 - q_off - (kQTile - 1), kQTile) + 1);     // last query <= first key
        lo2 = max(lo, ceil_div(kv_off + k0 + KEYS_WG - 1 - q_off, kQTile));          // first query >= last key
      }
      const int r2_hi = min(run2_hi, n);
      st_lo[0] = max(lo - tile_base, run_lo);
      st_hi[0] = max(min(hi1 - tile_base, run_hi), st_lo[0]);
      st_lo[1] = max(max(lo2 - tile_base, run_lo), st_hi[0]);
      st_hi[1] = max(min(hi - tile_base, run_hi), st_lo[1]);
      st_lo[2] = max(max(lo - tile_base2, run2_lo), st_hi[1]);
      st_hi[2] = max(min(hi1 - tile_base2, r2_hi), st_lo[2]);
      st_lo[3] = max(max(lo2 - tile_base2, run2_lo), st_hi[2]);
      st_hi[3] = max(min(hi - tile_base2, r2_hi), st_lo[3]);
    }
    if (lane == 0) {
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        const int base = st < 2 ? tile_base : tile_base2, c_hi = st < 2 ? cons_hi : cons2_hi;
        // iteration i is plain for first < i < end.  It requests tile i + 3 by running addresses:
        // where the list goes on that must be the listed tile, behind the list's end it only has
        // to lie inside the shard (nobody reads it).
        const int list_end = c_hi >= n ? 0x3fffffff : c_hi - 3;
        s_st[wave][3 * st] = st_lo[st];
        s_st[wave][3 * st + 1] = min(min(st_hi[st] - 1, list_end), a.Lq / kQTile - base - 3);
        s_st[wave][3 * st + 2] = base;
      }
    }
  } else if (wave_on) {
    int lo, hi;
    query_tile_plain_range(flags, bs.window, kv_off + kw, kv_off + kw + 31, q_off, a.Lq / kQTile,
                           kQTile, lo, hi);
    plain_lo = max(lo - tile_base, run_lo);
    plain_hi = max(min(hi - tile_base, run_hi), plain_lo);
  }
  plain_lo = __builtin_amdgcn_readfirstlane(plain_lo);
  plain_hi = __builtin_amdgcn_readfirstlane(plain_hi);

  // S(i) * scale2 - lse2 and dP(i) - delta of the current tile, in vector registers: the pair
  // (s_a, p_a) for even i, (s_b, p_b) for odd i; an iteration consumes one pair while the matrix
  // unit fills the other
  f32x16 s_a, p_a, s_b, p_b;
  bool cur_valid = false;
  if (n > 0 && wave_on) {
    int qt0, segbit;
    const int cls = tile_class(0, qt0, segbit);
    if (!(cls & 1)) {
      cur_valid = true;
      compute_s_dp(s_a, p_a, s_q[0], s_do[0], 0);
      if (needs_bias(qt0, segbit, cls)) prepare(s_a, qt0, segbit, cls, 0);
    }
  }
  // P(i-1) and dS(i-1), packed in pairs, waiting for their dV / dK products
  u32x4 pfw[2], dsw[2];
#pragma unroll
  for (int e = 0; e < 4; ++e) pfw[0][e] = pfw[1][e] = dsw[0][e] = dsw[1][e] = 0u;
  bool pend_valid = false;
  auto pack2 = [&](float x0, float x1) -> unsigned {
    bf16x2 t;
    t[0] = (bf16_t)x0;
    t[1] = (bf16_t)x1;
    return __builtin_bit_cast(unsigned, t);
  };

  // Generic iteration.  Tile j lives in LDS buffer j % NB = PH for j = i.
  auto iteration = [&](auto phase, int i, f32x16& SC, f32x16& PC, f32x16& SN, f32x16& PN) {
    constexpr int PH = decltype(phase)::value;
    constexpr int PHP = (PH + NB - 1) % NB, PH1 = (PH + 1) % NB, PH2 = (PH + 2) % NB, PH3 = (PH + 3) % NB;
    // this wave's share of tile i+1 is in LDS once at most the loads of tile i+2 are in flight;
    // the per-row word of tile i+2 (the first load of its group) is published one iteration
    // before the tile is read
    if (i + 2 < n) {
      RA_WAIT_VMCNT(LPT - 1);
      store_stat(PH2);
    } else {
      RA_WAIT_VMCNT(0);
    }
    __syncthreads();
    if (i + 3 < n) {
      int sbu;
      issue_tile(tile_at(i + 3, sbu), PH3);
    }
    if (pend_valid) {
      bf16x8 pf[2], dsf[2];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        pf[ks] = __builtin_bit_cast(bf16x8, pfw[ks]);
        dsf[ks] = __builtin_bit_cast(bf16x8, dsw[ks]);
      }
      compute_dkdv(pf, dsf, s_q[PHP], s_do[PHP]);
    }
    if (cur_valid) {
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        float p[2], ds[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          p[e] = fast_exp2(SC[r + e] * res);
          ds[e] = p[e] * PC[r + e];
        }
        pfw[r >> 3][(r & 7) >> 1] = pack2(p[0], p[1]);
        dsw[r >> 3][(r & 7) >> 1] = pack2(ds[0], ds[1]);
      }
    }
    pend_valid = cur_valid;
    int nqt0 = 0, nsegbit = 0, ncls = 1;
    bool nxt_valid = false;
    if (i + 1 >= plain_lo && i + 1 < plain_hi) {
      nxt_valid = true;
      ncls = 0;
    } else if (i + 1 < n && wave_on) {
      ncls = tile_class(i + 1, nqt0, nsegbit);
      nxt_valid = !(ncls & 1);
    }
    if (nxt_valid) {
      compute_s_dp(SN, PN, s_q[PH1], s_do[PH1], PH1);
      if (!(i + 1 >= plain_lo && i + 1 < plain_hi) && needs_bias(nqt0, nsegbit, ncls))
        prepare(SN, nqt0, nsegbit, ncls, PH1);
    }
    cur_valid = nxt_valid;
  };

  // Loads of the plain stretch: consecutive full tiles, so the wave-uniform global addresses
  // advance by a constant and stay in scalar registers.
  const bf16_t* q_run = qbase;
  const bf16_t* do_run = dobase;
  const char* st_run = st_src;
  const unsigned q_dst0 = RA_LDS_ADDR(&s_q[0][0]) + wave_u * 8 * ROWB;
  const unsigned do_dst0 = RA_LDS_ADDR(&s_do[0][0]) + wave_u * 8 * ROWB;
  // The first PFT operand fragments of an iteration's dV / dK products, fetched in the tail of the
  // iteration before (the tile they come from has been visible for two barriers by then): the
  // fetch pipeline does not start from empty behind every barrier.
  bf16x8 frc[PFT];
  auto seek_plain = [&](int tile) {
    q_run = qbase + (long long)(tile * kQTile + 8 * wave_u) * a.q.sl;
    do_run = dobase + (long long)(tile * kQTile + 8 * wave_u) * a.dout.sl;
    st_run = st_src + 4ll * (tile * kQTile + st_row);
    // a stretch begins with phase 0: its first products take tile i - 1 from buffer NB - 1
#pragma unroll
    for (int op = 0; op < PFT; ++op)
      frc[op] = tr_frag((op & 1) ? s_q[NB - 1] : s_do[NB - 1], op / (2 * DB), (op >> 1) % DB);
  };

  // The same iteration for a stretch of plain tiles: tiles i-1, i and i+1 are plain and tile i+3
  // exists and is complete, so there is nothing to classify and no flag to consult.
  // The segment ids of a stretch's tiles (one id per tile) travel in scalar registers, fetched
  // ahead through the constant address space: the compiler uses the scalar cache and tracks the
  // load in flight itself (the array is not written while the kernel runs).
  typedef const __attribute__((address_space(4))) int* const_ids;
  const const_ids doc_ids = (const_ids)(uintptr_t)q_seg;
  int doc_cur = 0, doc_nxt = 0, doc_far = 0;  // segment ids of tiles i, i + 1, i + 2 of a stretch
  float ali_s = 0.f;                          // +-slope in score units, set where a stretch begins
  bf16_t ali_s_hi = (bf16_t)0.f, ali_s_lo = (bf16_t)0.f;
  auto plain_iteration = [&](auto phase, int i, f32x16& SC, f32x16& PC, f32x16& SN, f32x16& PN) {
    constexpr int PH = decltype(phase)::value;
    constexpr int PHP = (PH + NB - 1) % NB, PH1 = (PH + 1) % NB, PH2 = (PH + 2) % NB, PH3 = (PH + 3) % NB;
    // documents: a lane whose key carries another id than tile i takes no part in it - its
    // probabilities are exp2(-inf) = 0
    float gate = 0.f;
    if (GENERAL && seg_on) {
      gate = (k_seg == doc_cur) ? 0.f : RA_NEG_INF;
      doc_cur = doc_nxt;
      doc_nxt = doc_far;                                                  // requested one iteration ago
      doc_far = doc_ids[(long long)(tile_base + i + 3) * kQTile];        // tile i + 3 exists
    }
    const char* qp = s_q[PHP];
    const char* dop = s_do[PHP];
    const char* qn = s_q[PH1];
    const char* don = s_do[PH1];
    // operands of the dV / dK products come from tile i-1, visible since two barriers ago; the
    // first PFT of them were requested by the previous iteration (or by seek_plain)
    bf16x8 frb[4 * DB];
#pragma unroll
    for (int op = 0; op < PFT; ++op) frb[op] = frc[op];
    // all but the loads of tile i+2 have landed: this wave's share of tile i+1 is in LDS.  The
    // barrier is issued without a fence: the only LDS operations in flight are the PFT operand
    // fetches above, and what other waves need (the statistics stored half an iteration ago) is
    // older than those.
    RA_WAIT_VMCNT(LPT);
    asm volatile("s_waitcnt lgkmcnt(%0)\n\ts_barrier" : : "n"(2 * PFT) : "memory");
    bf16x8 pf[2], dsf[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      pf[ks] = __builtin_bit_cast(bf16x8, pfw[ks]);
      dsf[ks] = __builtin_bit_cast(bf16x8, dsw[ks]);
    }
    bf16x8 fra[2 * KS];
    constexpr int NOPS = 4 * DB;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int op = 0; op < NOPS; ++op) {
      if (op + PFT < NOPS) {
        const int o2 = op + PFT;
        frb[o2] = tr_frag((o2 & 1) ? qp : dop, o2 / (2 * DB), (o2 >> 1) % DB);
      } else {
        // the first operands of the S / dP products ride behind the last dV / dK MFMAs
        const int o2 = op + PFT - NOPS;
        if (o2 < PFN) fra[o2] = nat_frag((o2 & 1) ? don : qn, o2 >> 1);
      }
      const int ks = op / (2 * DB), db = (op >> 1) % DB;
      if (op & 1) dk[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dsf[ks], frb[op], dk[db], 0, 0, 0);
      else dv[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pf[ks], frb[op], dv[db], 0, 0, 0);
      // next tile's loads, one instruction group per MFMA: their issue hides behind the MFMAs
      if (op == 0) {
        load_stat(st_run, PH3);
        st_run += kQTile * 4;
      }
      if (op == 1) {
        if (NLD == 2) global_to_lds16_s_x2(q_run, q_voff[0], q_voff[NLD - 1], q_dst0 + PH3 * TILE_BYTES);
        else global_to_lds16_s(q_run, q_voff[0], q_dst0 + PH3 * TILE_BYTES);
        q_run += (long long)kQTile * a.q.sl;
      }
      if (op == 2) {
        if (NLD == 2) global_to_lds16_s_x2(do_run, do_voff[0], do_voff[NLD - 1], do_dst0 + PH3 * TILE_BYTES);
        else global_to_lds16_s(do_run, do_voff[0], do_dst0 + PH3 * TILE_BYTES);
        do_run += (long long)kQTile * a.dout.sl;
      }
      // the statistics of tile i+1 are the initial values of S(i+1), dP(i+1)
      {
        const int j = op - (NOPS - 8);
        if (j >= 0) {
          const f32x4 t = stat_chunk(PH1, j >> 2, j & 3);
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            if (j >> 2) PN[4 * (j & 3) + c] = t[c];
            else SN[4 * (j & 3) + c] = t[c];
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // S(i+1), dP(i+1) with P(i), dS(i) in their shadow: one score element per MFMA, the chain of
    // an element (exp2, product, packing) spread over consecutive slots.  (Spreading the chain over
    // the dV / dK slots as well - they carry two operand fetches each but no arithmetic - made the
    // kernel 2 % slower: those slots are bound by their fetches, and vector instructions between
    // them delay the fetches.)
    float pe[16], de[16];
    constexpr int EPO = 16 / (2 * KS) > 0 ? 16 / (2 * KS) : 1;
    unsigned raw_word = 0;
    if (GENERAL && alibi_on) {
      // ALiBi of tile i+1 through the matrix unit: the score accumulators receive
      //   [r, r, 1, 1, 1] x [s_hi, s_lo, c_hi, c_mid, c_lo] = s r + c = -slope |q_pos - kv_pos| (score units)
      // with s = +-slope (the sign of the stretch), r the query's index in the tile and
      // c = s (position of the tile's first query - kv_pos); s is split into two bf16 words
      // and c into three (c grows with the distance between the shards: three words carry it to
      // fp32 accuracy, what an addition in the score chain would give), so that the chain below
      // needs no instruction for the bias.
      const int rel_t = q_off + (tile_base + i + 1) * kQTile - (kv_off + kw + l32);
      const float ali_c = ali_s * (float)rel_t;
      const bf16_t c_hi = (bf16_t)ali_c;
      const bf16_t c_mid = (bf16_t)(ali_c - (float)c_hi);
      const bf16_t c_lo = (bf16_t)((ali_c - (float)c_hi) - (float)c_mid);
      bf16x8 bq;
      bq[0] = ali_s_hi;
      bq[1] = ali_s_lo;
      bq[2] = c_hi;
      bq[3] = c_mid;
      bq[4] = c_lo;
      bq[5] = bq[6] = bq[7] = (bf16_t)0.f;
      mfma_scores_v(SN, s_ramp[lane], bq);
    }
    fra[PFN] = nat_frag((PFN & 1) ? don : qn, PFN >> 1);
#pragma unroll
    for (int op = 0; op < 2 * KS; ++op) {
      if (op & 1) mfma_scores(PN, fra[op], vfa[op >> 1]);
      else mfma_scores(SN, fra[op], kfa[op >> 1]);
      // The wait for the next MFMA's operand goes right behind this MFMA, in front of the slot's operand
      // fetch and vector work (the compiler waits in front of whatever reads a fetched register): a
      // lone wave issues MFMA, s_waitcnt, ds_read, 4 vector instructions in 36 cycles, and the same
      // instructions with the wait behind them, in front of the next MFMA, in 40 to 48.
      if (op + 1 < 2 * KS) asm volatile("" : : "v"(fra[op + 1]));
      if (op + 1 + PFN < 2 * KS) fra[op + 1 + PFN] = nat_frag(((op + 1 + PFN) & 1) ? don : qn, (op + 1 + PFN) >> 1);
      if (op == 2) {
        // the per-row word of tile i+2 is the oldest load but those of its tile and of tile i+3
        RA_WAIT_VMCNT(2 * LPT - 1);
        raw_word = fetch_stat(PH2);
      }
      if (op == 2 + PFN) publish_stat(raw_word, PH2);  // behind as many fetches as are kept in flight
      // the next iteration's first dV / dK operands: tile i, which it finds in buffer PH
      if (op >= 2 * KS - PFT) {
        const int o2 = op - (2 * KS - PFT);
        frc[o2] = tr_frag((o2 & 1) ? s_q[PH] : s_do[PH], o2 / (2 * DB), (o2 >> 1) % DB);
      }
#pragma unroll
      for (int e = 0; e < EPO; ++e) {
        const int r = op * EPO + e;
        if (r < 16) {
          if (GENERAL) pe[r] = fast_exp2(fmaf(SC[r], res, gate));
          else pe[r] = fast_exp2(SC[r] * res);
          asm volatile("" : "+v"(pe[r]));
        }
        if (r >= 1 && r <= 16) {
          de[r - 1] = pe[r - 1] * PC[r - 1];
          asm volatile("" : "+v"(de[r - 1]));
        }
        if (r >= 2 && r <= 16 && !(r & 1)) {
          unsigned pw = pack2(pe[r - 2], pe[r - 1]), dw = pack2(de[r - 2], de[r - 1]);
          asm volatile("" : "+v"(pw), "+v"(dw));
          pfw[(r - 2) >> 3][((r - 2) & 7) >> 1] = pw;
          dsw[(r - 2) >> 3][((r - 2) & 7) >> 1] = dw;
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    de[15] = pe[15] * PC[15];
    pfw[1][3] = pack2(pe[14], pe[15]);
    dsw[1][3] = pack2(de[14], de[15]);
  };

  // Three loops over the same sequence of tiles: generic iterations up to the plain stretch, the
  // plain stretch in whole groups of six, generic iterations for the rest.  Every wave runs n
  // iterations in total, so the barrier counts agree.
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  using P2 = std::integral_constant<int, 2>;
  using P3 = std::integral_constant<int, 3>;
  using P4 = std::integral_constant<int, 4>;
  using P5 = std::integral_constant<int, 5>;
  int i = 0;
  if constexpr (!GENERAL) {
  // iteration i is plain for plain_lo < i < plain_end (tile i+3 must exist and be complete)
  const int plain_end = __builtin_amdgcn_readfirstlane(
      min(min(plain_hi - 1, run_hi - 3), a.Lq / kQTile - tile_base - 3));
  for (; i < n && !(i > plain_lo && i + NB <= plain_end); i += NB) {
    iteration(P0{}, i, s_a, p_a, s_b, p_b);
    if (i + 1 < n) iteration(P1{}, i + 1, s_b, p_b, s_a, p_a);
    if (i + 2 < n) iteration(P2{}, i + 2, s_a, p_a, s_b, p_b);
    if (i + 3 < n) iteration(P3{}, i + 3, s_b, p_b, s_a, p_a);
    if (i + 4 < n) iteration(P4{}, i + 4, s_a, p_a, s_b, p_b);
    if (i + 5 < n) iteration(P5{}, i + 5, s_b, p_b, s_a, p_a);
  }
  if (i + NB <= plain_end) seek_plain(tile_base + i + 3);
  for (; i + NB <= plain_end; i += NB) {
    plain_iteration(P0{}, i, s_a, p_a, s_b, p_b);
    plain_iteration(P1{}, i + 1, s_b, p_b, s_a, p_a);
    plain_iteration(P2{}, i + 2, s_a, p_a, s_b, p_b);
    plain_iteration(P3{}, i + 3, s_b, p_b, s_a, p_a);
    plain_iteration(P4{}, i + 4, s_a, p_a, s_b, p_b);
    plain_iteration(P5{}, i + 5, s_b, p_b, s_a, p_a);
  }
  } else {
#pragma unroll 1
  for (int st = 0; st < 4; ++st) {
    // iteration i is plain for p_lo < i < p_end
    const int p_lo = __builtin_amdgcn_readfirstlane(s_st[wave_u][3 * st]);
    const int p_end = __builtin_amdgcn_readfirstlane(s_st[wave_u][3 * st + 1]);
    const int start = max(i, ((p_lo + NB) / NB) * NB);  // i is a multiple of six here
    if (start + NB > p_end) continue;
    tile_base = __builtin_amdgcn_readfirstlane(s_st[wave_u][3 * st + 2]);
    for (; i < start; i += NB) {
      iteration(P0{}, i, s_a, p_a, s_b, p_b);
      iteration(P1{}, i + 1, s_b, p_b, s_a, p_a);
      iteration(P2{}, i + 2, s_a, p_a, s_b, p_b);
      iteration(P3{}, i + 3, s_b, p_b, s_a, p_a);
      iteration(P4{}, i + 4, s_a, p_a, s_b, p_b);
      iteration(P5{}, i + 5, s_b, p_b, s_a, p_a);
    }
    seek_plain(tile_base + i + 3);
    if (seg_on) {
      doc_cur = doc_ids[(long long)(tile_base + i) * kQTile];
      doc_nxt = doc_ids[(long long)(tile_base + i + 1) * kQTile];
      doc_far = doc_ids[(long long)(tile_base + i + 2) * kQTile];
    }
    if (alibi_on) {
      // queries before the keys (even stretches): bias = slope (q_pos - kv_pos), rising with the
      // query's index; queries after them: falling
      ali_s = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(
          __builtin_bit_cast(int, (st & 1) ? -slope2 : slope2)));  // one slope per head
      ali_s_hi = (bf16_t)ali_s;
      ali_s_lo = (bf16_t)(ali_s - (float)ali_s_hi);
    }
    for (; i + NB <= p_end; i += NB) {
      plain_iteration(P0{}, i, s_a, p_a, s_b, p_b);
      plain_iteration(P1{}, i + 1, s_b, p_b, s_a, p_a);
      plain_iteration(P2{}, i + 2, s_a, p_a, s_b, p_b);
      plain_iteration(P3{}, i + 3, s_b, p_b, s_a, p_a);
      plain_iteration(P4{}, i + 4, s_a, p_a, s_b, p_b);
      plain_iteration(P5{}, i + 5, s_b, p_b, s_a, p_a);
    }
    if (seg_on && k_seg != doc_cur) {
      // the scores of tile i, which the next generic iteration turns into probabilities, came
      // out of the stretch without a mask: keys of another document drop out here
#pragma unroll
      for (int r = 0; r < 16; ++r) s_a[r] = RA_NEG_INF;
    }
  }
  }
  for (; i < n; i += NB) {
    iteration(P0{}, i, s_a, p_a, s_b, p_b);
    if (i + 1 < n) iteration(P1{}, i + 1, s_b, p_b, s_a, p_a);
    if (i + 2 < n) iteration(P2{}, i + 2, s_a, p_a, s_b, p_b);
    if (i + 3 < n) iteration(P3{}, i + 3, s_b, p_b, s_a, p_a);
    if (i + 4 < n) iteration(P4{}, i + 4, s_a, p_a, s_b, p_b);
    if (i + 5 < n) iteration(P5{}, i + 5, s_b, p_b, s_a, p_a);
  }
  if (pend_valid) {  // products of the last tile
    bf16x8 pf[2], dsf[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      pf[ks] = __builtin_bit_cast(bf16x8, pfw[ks]);
      dsf[ks] = __builtin_bit_cast(bf16x8, dsw[ks]);
    }
    const int last = (n - 1) % NB;
    compute_dkdv(pf, dsf, s_q[0] + last * TILE_BYTES, s_do[0] + last * TILE_BYTES);
  }
  }  // query shards
  const bool whole_ring = MULTI && (flags & kFlagWhole);
  if (!whole_ring && tiles_listed == 0) return;  // nothing to add
  if constexpr (MULTI) {
    if (whole_ring) {
      // the gradients of this key slab are complete: bf16, in the caller's layout
      const long long at = b * a.out_sb + h * a.out_sh + (long long)(kw + 4 * g) * a.out_sl + l32;
      bf16_t* const dkp = (bf16_t*)ring.dk[blockIdx.y] + at;
      bf16_t* const dvp = (bf16_t*)ring.dv[blockIdx.y] + at;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int kr = 8 * (r / 4) + (r % 4);
        if (kw + 4 * g + kr < a.Lk) {
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            dkp[kr * a.out_sl + 32 * db] = (bf16_t)(dk[db][r] * a.sm_scale);
            dvp[kr * a.out_sl + 32 * db] = (bf16_t)dv[db][r];
          }
        }
      }
      return;
    }
  }
  // ---- accumulate into the fp32 gradients owned by this key slab ------------------------------
  // All loads of an array are issued before the first value is needed: a load - add - store chain
  // per element would cost one memory round trip each, a hundred in a row with nothing to hide them.
  {
    float* dk_res = a.dk;
    float* dv_res = a.dv;
    if constexpr (MULTI) {
      dk_res = ring.dk[blockIdx.y];
      dv_res = ring.dv[blockIdx.y];
    }
    float* const dkp = dk_res + (((long long)b * a.H + h) * a.Lk + kw + 4 * g) * D + l32;
    float* const dvp = dv_res + (((long long)b * a.H + h) * a.Lk + kw + 4 * g) * D + l32;
    const int key0 = kw + 4 * g;
    auto add_to = [&](float* p, const f32x16 (&acc)[DB], float mul) {
      float old[DB][16];
      if (kw + 32 <= a.Lk) {  // the whole wave is in range (wave-uniform): straight-line code
#pragma unroll
        for (int r = 0; r < 16; ++r)
#pragma unroll
          for (int db = 0; db < DB; ++db) old[db][r] = p[(8 * (r / 4) + (r % 4)) * D + 32 * db];
#pragma unroll
        for (int r = 0; r < 16; ++r)
#pragma unroll
          for (int db = 0; db < DB; ++db)
            p[(8 * (r / 4) + (r % 4)) * D + 32 * db] = fmaf(acc[db][r], mul, old[db][r]);
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int kr = 8 * (r / 4) + (r % 4);
          if (key0 + kr < a.Lk) {
#pragma unroll
            for (int db = 0; db < DB; ++db) p[kr * D + 32 * db] += acc[db][r] * mul;
          }
        }
      }
    };
    add_to(dkp, dk, a.sm_scale);
    add_to(dvp, dv, 1.0f);
  }
}

// ------------------------------------------------------------------------------------------------
// dQ
// ------------------------------------------------------------------------------------------------
constexpr int kDqThreads = 512;
constexpr int kDqRows = 256;   // query rows per workgroup
constexpr int kDqKeyTile = 32; // keys per LDS tile

// One workgroup = 8 waves = 256 query rows; wave w owns 32 rows: their Q and dO rows sit in
// registers as MFMA B operands, dQ^T accumulates in registers.  32-key tiles of K and V stream
// through six LDS buffers with direct-to-LDS loads issued three tiles ahead.  Scores are
// transposed (S^T = K Q^T, dP^T = V dO^T) exactly as in the forward kernel, so dS^T is the B
// operand of dQ^T += K^T dS^T whose A operand is the K tile read through the transposing LDS
// fetch.  Iteration i, after its barrier, first runs the 8 MFMAs of dQ^T for tile i-1 (operands
// visible before the barrier, so their fetch straddles it), then the 16 MFMAs of S^T(i+1),
// dP^T(i+1) with the exp2 / dS arithmetic of tile i in their shadow.
// MULTI: grid dimension y is a ring pass, one query shard with its dq accumulator.  The launch
// walks the key/value shards that `ring` lists for the pass one after another (consecutive ring
// steps of that query shard); dQ stays in registers between them.
template <int D, int MODE, bool MULTI>
__global__ __launch_bounds__(kDqThreads) void dq_kernel(
    const BwdArgs a, const std::conditional_t<MULTI, KvRing, NoShardList> ring) {
  constexpr bool GENERAL = MODE != 0;  // bias terms beyond causal / window
  constexpr bool DENSE = MODE == 2;    // ... including a materialised bias block
  constexpr int KS = D / 16;
  constexpr int DB = D / 32;
  constexpr int ROWB = D * 2;
  constexpr int TILE_BYTES = kDqKeyTile * ROWB;
  constexpr int NBUF = 6;
  __shared__ __attribute__((aligned(16))) char s_k[NBUF][TILE_BYTES];
  __shared__ __attribute__((aligned(16))) char s_v[NBUF][TILE_BYTES];
  __shared__ __attribute__((aligned(16))) int s_seg[NBUF][kDqKeyTile];
  __shared__ __attribute__((aligned(16))) int s_pre[NBUF][kDqKeyTile];
  __shared__ unsigned short s_list[GENERAL ? kBwdMaxListTiles : 1];
  __shared__ unsigned char s_flag[GENERAL ? kBwdMaxListTiles : 1];
  __shared__ int s_red[28];
  __shared__ float s_rowc[2][kDqThreads];
  // GENERAL: per wave and stretch of straight-line iterations: first tile ordinal, end, tile base
  __shared__ int s_st[GENERAL ? 8 : 1][12];
  // per-lane values that only the generic iterations use wait here while a stretch runs
  __shared__ int s_stash[GENERAL ? 3 : 1][GENERAL ? kDqThreads : 1];
  // A operand of the matrix instruction that writes the ALiBi term into a fresh score tile
  __shared__ __attribute__((aligned(16))) bf16x8 s_ramp[GENERAL ? 64 : 1];
  // The GENERAL variants are a few registers short in their straight-line loop: the first operand
  // fragments of Q and dO and the per-lane load offsets wait here and are fetched once per
  // iteration instead (a spill to scratch memory would make every iteration wait for all loads).
  constexpr bool TIGHT = GENERAL || MULTI;
  __shared__ __attribute__((aligned(16))) bf16x8 s_q0[TIGHT ? kDqThreads : 1];
  __shared__ __attribute__((aligned(16))) bf16x8 s_do0[TIGHT ? kDqThreads : 1];
  __shared__ __attribute__((aligned(16))) bf16x8 s_q1[GENERAL ? kDqThreads : 1];
  __shared__ __attribute__((aligned(8))) unsigned s_voff[TIGHT ? kDqThreads : 1][2];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);  // same value in a scalar register
  const int l32 = lane & 31, g = lane >> 5;
  const int nqt = (a.Lq + kDqRows - 1) / kDqRows;
  int hh, qt;
  decode_block(blockIdx.x, a.B * a.H, nqt, hh, qt);
  const int b = hh / a.H, h = hh % a.H;
  const int q0 = qt * kDqRows;
  const int qw = q0 + wave * 32;
  const int qi = qw + l32;
  const bool q_valid = qi < a.Lq;
  const int qi_c = min(qi, a.Lq - 1);
  const BiasArgs& bs = a.bias;
  const int flags = bs.flags;
  const bool wave_on = qw < a.Lq;

  bf16x8 qf[KS], dof[KS];
  {
    const bf16_t* q_res = a.q.ptr;
    const bf16_t* do_res = a.dout.ptr;
    if constexpr (MULTI) {
      q_res = ring.q[blockIdx.y];
      do_res = ring.dout[blockIdx.y];
    }
    const bf16_t* qp = q_res + b * a.q.sb + h * a.q.sh + (long long)qi_c * a.q.sl + 8 * g;
    const bf16_t* dp = do_res + b * a.dout.sb + h * a.dout.sh + (long long)qi_c * a.dout.sl + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      // Q is multiplied once, here, by the power of two below sm_scale * log2(e) (exact in bf16);
      // the residual factor scale_res in [1, 2) is applied to the fp32 score in front of exp2, as
      // in the dK/dV kernel (dQ itself is built from the unscaled K)
      const bf16x8 qr = *(const bf16x8*)(qp + 16 * s);
#pragma unroll
      for (int e = 0; e < 8; ++e) qf[s][e] = (bf16_t)((float)qr[e] * a.scale_p2);
      dof[s] = *(const bf16x8*)(dp + 16 * s);
    }
    if (TIGHT) {
      s_q0[tid] = qf[0];
      s_do0[tid] = dof[0];
    }
    if (GENERAL) s_q1[tid] = qf[1];
    if (GENERAL && tid < 64) {
      // row l32 of the 32 x 16 operand is [j, j, 1, 1, 1, 0 ...] with j = l32 the key's index in the
      // tile (exact in bf16); lanes 32..63 hold the other eight columns, all zero
      bf16x8 rf;
#pragma unroll
      for (int e = 0; e < 8; ++e) rf[e] = (bf16_t)0.f;
      if (g == 0) {
        rf[0] = rf[1] = (bf16_t)(float)l32;
        rf[2] = rf[3] = rf[4] = (bf16_t)1.0f;
      }
      s_ramp[tid] = rf;
    }
  }
  const long long row = ((long long)b * a.H + h) * a.Lq + qi_c;
  const float* lse_res = a.lse;
  const float* delta_res = a.delta;
  if constexpr (MULTI) {
    lse_res = ring.x1[blockIdx.y];
    delta_res = ring.x2[blockIdx.y];
  }
  const float Lraw = lse_res[row];
  float neg_lse2 = (Lraw == RA_NEG_INF) ? RA_NEG_INF : -Lraw * kLog2e;  // fully masked row: P = 0
  float delta = delta_res[row];
  // exp2(S - lse2) (dP - delta) = exp2(S) (c dP - c delta) with c = exp2(-lse2): one vector
  // instruction less per score.  Only where no row's logsumexp is so large that exp2(S) or c
  // could leave the fp32 range (S <= lse2 always); other waves have no straight-line stretch.
  const bool lse_in_range = __all(fabsf(neg_lse2) <= 100.0f);
  float c_row = 0.f, cd_row = 0.f;
  f32x16 acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[db][r] = 0.f;

  int q_seg = 0, q_pre = 0;
  float slope2 = 0.f;
  if (GENERAL) {
    const int* q_seg_res = bs.q_seg;
    const int* q_pre_res = bs.q_pre;
    if constexpr (MULTI) {
      q_seg_res = ring.q_seg[blockIdx.y];
      q_pre_res = ring.q_pre[blockIdx.y];
    }
    if (flags & RA_BIAS_SEGMENT) q_seg = q_seg_res[b * bs.q_seg_sb + qi_c];
    if (flags & RA_BIAS_PREFIX) q_pre = q_pre_res[b * bs.q_pre_sb + qi_c];
    if (flags & RA_BIAS_ALIBI) slope2 = bs.slopes[h] * kLog2e / a.scale_res;
  }
  // ---- one pass of everything below per key/value shard ------------------------------------
  int kv_off = bs.kv_off;
  const bf16_t* k_ptr = a.k.ptr;
  const bf16_t* v_ptr = a.v.ptr;
  const int* kv_seg_ptr = bs.kv_seg;
  const int* kv_pre_ptr = bs.kv_pre;
  const float* dense_ptr = bs.dense;
  int n_shards = 1;
  int tiles_listed = 0;  // over all shards of the pass: none, and the workgroup leaves its carry / gradients as they are
  if constexpr (MULTI) n_shards = ring.count[blockIdx.y];
  for (int shard = 0; shard < n_shards; ++shard) {
  if constexpr (MULTI) {
    const int si = ring.order[blockIdx.y][shard];
    kv_off = ring.kv.kv_off[si];
    k_ptr = ring.kv.k[si];
    v_ptr = ring.kv.v[si];
    kv_seg_ptr = ring.kv.kv_seg[si];
    kv_pre_ptr = ring.kv.kv_pre[si];
    dense_ptr = ring.kv.dense[si];
    // other waves may still be reading the last K tile of the previous shard
    if (shard > 0) __syncthreads();
  }
  // Everything derived from the lane number is rebuilt per shard from an opaque copy of the
  // thread id: hoisted out of this loop it would occupy registers across the tile loops, which
  // have none to spare.
  int tid_shard = threadIdx.x;
  if constexpr (MULTI) asm volatile("" : "+v"(tid_shard));
  const int tid = tid_shard, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, g = lane >> 5;
  const int qw = q0 + wave * 32;
  const int qi = qw + l32;
  const bool q_valid = qi < a.Lq;
  const bool wave_on = qw < a.Lq;
  const int* kv_seg = (GENERAL && (flags & RA_BIAS_SEGMENT)) ? kv_seg_ptr + b * bs.kv_seg_sb : nullptr;
  const int* kv_pre = (GENERAL && (flags & RA_BIAS_PREFIX)) ? kv_pre_ptr + b * bs.kv_pre_sb : nullptr;

  // ---- which key tiles does this workgroup visit ------------------------------------------------
  const int ntiles = (a.Lk + kDqKeyTile - 1) / kDqKeyTile;
  const int q_rows_hi = min(q0 + kDqRows, a.Lq) - 1;
  int j_lo, j_hi;
  int q_off = bs.q_off;
  if constexpr (MULTI) q_off = ring.q_off[blockIdx.y];
  key_tile_range(flags, bs.window, q_off + q0, q_off + q_rows_hi, kv_off, ntiles, kDqKeyTile,
                 j_lo, j_hi);
  int n_act = j_hi - j_lo;
  bool use_list = false;
  // Ordinals [run_lo, run_hi) are consecutive tiles `run_base + ordinal` with one segment id
  // each: inside a straight-line stretch a lane decides per tile whether its query row belongs to
  // the tile's document.  [run2_lo, run2_hi): a second such run behind the first one (a workgroup
  // that straddles a document boundary has one per document).  wg_one_doc: all queries of the
  // workgroup carry one id, so one-id tiles need no test in the generic iterations either.
  int run_lo = 0, run_hi = n_act, run_base = j_lo;
  int run2_lo = 0, run2_hi = 0, run2_base = 0;
  // the listed tiles count up without a gap from the start of a run to ordinal cons_hi / cons2_hi
  int cons_hi = n_act, cons2_hi = 0;
  bool wg_one_doc = true;
  const bool seg_on = GENERAL && (flags & RA_BIAS_SEGMENT);
  // A dense block that comes with its summary is listed the same way: tiles in which the
  // workgroup's rows hold nothing but -inf are left out, tiles of zeros have no term to evaluate,
  // the rest is evaluated element by element.  (Single-step launches only.)
  const unsigned char* dmap = nullptr;
  if constexpr (DENSE && !MULTI) {
    if (bs.dense_map) dmap = dense_map_of(bs, b, h, a.H, a.Lq, a.Lk);
  }
  if ((GENERAL && (flags & RA_BIAS_SEGMENT)) || (DENSE && dmap != nullptr)) {
    use_list = true;
    int qmin = 0, qmax = 0;
    if (seg_on) {
      int smin = q_valid ? q_seg : 0x7fffffff, smax = q_valid ? q_seg : (int)0x80000000;
      smin = wave_min(smin);
      smax = wave_max(smax);
      if (lane == 0) {
        s_red[wave] = smin;
        s_red[8 + wave] = smax;
      }
      __syncthreads();
      qmin = s_red[0];
      qmax = s_red[8];
#pragma unroll
      for (int w = 1; w < 8; ++w) {
        qmin = min(qmin, s_red[w]);
        qmax = max(qmax, s_red[8 + w]);
      }
    }
    for (int j = j_lo + tid; j < j_hi; j += kDqThreads) {
      int f = 1;
      if (seg_on) {
        int kmin, kmax;
        tile_id_range<kDqKeyTile>(kv_seg, j, a.Lk, kmin, kmax);
        const bool act = !(kmax < qmin || kmin > qmax);
        f = act ? ((kmin == kmax) ? 1 : 3) : 0;
      }
      if constexpr (DENSE) {
        if (dmap != nullptr && f != 0) {
          const int bits = dense_map_or(dmap, a.Lk, q0, q_rows_hi, j * kDqKeyTile, min((j + 1) * kDqKeyTile, a.Lk) - 1);
          f = (bits & kMapLive) ? ((bits & kMapNonZero) ? 3 : f) : 0;
        }
      }
      s_flag[j - j_lo] = f;
    }
    wg_one_doc = qmin == qmax;
    __syncthreads();
    if (wave == 0) {
      int cnt = 0;
      for (int base = 0; base < n_act; base += 64) {
        const int i = base + lane;
        const int f = (i < n_act) ? s_flag[i] : 0;
        const unsigned long long mask = __ballot(f != 0);
        if (f) s_list[cnt + __popcll(mask & ((1ull << lane) - 1ull))] = (unsigned short)((j_lo + i) | ((f & 2) << 14));
        cnt += __popcll(mask);
      }
      int u_lo, u_hi, u_base, w_lo, w_hi, w_base;
      uniform_run(s_list, cnt, lane, 0, u_lo, u_hi, u_base);
      uniform_run(s_list, cnt, lane, u_hi, w_lo, w_hi, w_base);
      const int c_hi = consecutive_end(s_list, cnt, lane, u_lo);
      const int c2_hi = consecutive_end(s_list, cnt, lane, w_lo);
      if (lane == 0) {
        s_red[23] = c_hi;
        s_red[24] = c2_hi;
        s_red[16] = cnt;
        s_red[17] = u_lo;
        s_red[18] = u_hi;
        s_red[19] = u_base;
        s_red[20] = w_lo;
        s_red[21] = w_hi;
        s_red[22] = w_base;
      }
    }
    __syncthreads();
    n_act = s_red[16];
    run_lo = s_red[17];
    run_hi = s_red[18];
    run_base = s_red[19];
    run2_lo = s_red[20];
    run2_hi = s_red[21];
    run2_base = s_red[22];
    cons_hi = s_red[23];
    cons2_hi = s_red[24];
  }
  const int n = __builtin_amdgcn_readfirstlane(n_act);
  tiles_listed += n;
  run_lo = __builtin_amdgcn_readfirstlane(run_lo);
  run_hi = __builtin_amdgcn_readfirstlane(min(run_hi, n));
  run_base = __builtin_amdgcn_readfirstlane(run_base);

  auto tile_at = [&](int i, int& segbit) -> int {
    if (GENERAL && use_list) {
      int e = s_list[i];
      segbit = (e >> 15) | (wg_one_doc ? 0 : 1);  // a tile of several ids, or queries of several
      return e & 0x7fff;
    }
    segbit = 0;
    return j_lo + i;
  };

  // ---- global -> LDS: every wave moves 4 of a tile's 32 rows of K and of V ---------------------
  const bf16_t* kbase = k_ptr + b * a.k.sb + h * a.k.sh;
  const bf16_t* vbase = v_ptr + b * a.v.sb + h * a.v.sh;
  constexpr int CPR = D / 8;   // 16-byte chunks per row
  constexpr int RPW = 4;       // rows per wave per tile
  // D = 128: one load instruction = 4 rows; D = 64: lanes 0..31 cover the wave's 4 rows
  // (with D = 128 every lane takes part, and the compiler need not mask anything)
  const bool ld_lane_on = (64 / CPR <= RPW) || (lane / CPR) < RPW;
  const int ld_row = RPW * wave + (lane / CPR) % RPW;
  const int ld_chunk = ((tile_off<D>(ld_row, lane % CPR) - ld_row * ROWB) >> 4) * 8;
  const unsigned k_voff = (unsigned)(((long long)((lane / CPR) % RPW) * a.k.sl + ld_chunk) * 2);
  const unsigned v_voff = (unsigned)(((long long)((lane / CPR) % RPW) * a.v.sl + ld_chunk) * 2);
  if (TIGHT) {
    s_voff[tid][0] = k_voff;
    s_voff[tid][1] = v_voff;
  }
  int seg_r = 0, pre_r = 0;
  auto issue_tile = [&](int j, int buf, bool with_ids = true) {
    const int k0 = j * kDqKeyTile;
    unsigned kvo = k_voff, vvo = v_voff;
    if (TIGHT && !with_ids) {  // called from the straight-line loop
      kvo = s_voff[tid][0];
      vvo = s_voff[tid][1];
    }
    const unsigned k_dst = RA_LDS_ADDR(&s_k[0][0]) + buf * TILE_BYTES + wave_u * RPW * ROWB;
    const unsigned v_dst = RA_LDS_ADDR(&s_v[0][0]) + buf * TILE_BYTES + wave_u * RPW * ROWB;
    if (ld_lane_on) {
      if (k0 + kDqKeyTile <= a.Lk) {
        global_to_lds16_s(kbase + (long long)(k0 + RPW * wave_u) * a.k.sl, kvo, k_dst);
        global_to_lds16_s(vbase + (long long)(k0 + RPW * wave_u) * a.v.sl, vvo, v_dst);
      } else {  // last, partial tile: rows past the end repeat the last row (masked later)
        const int gr = min(k0 + ld_row, a.Lk - 1);
        global_to_lds16(kbase + (long long)gr * a.k.sl + ld_chunk, k_dst);
        global_to_lds16(vbase + (long long)gr * a.v.sl + ld_chunk, v_dst);
      }
    }
    if (GENERAL && with_ids && lane < kDqKeyTile) {
      int kk = min(k0 + lane, a.Lk - 1);
      if (kv_seg) seg_r = kv_seg[kk];
      if (kv_pre) pre_r = kv_pre[kk];
    }
  };
  auto store_ids = [&](int buf) {
    if (GENERAL && lane < kDqKeyTile) {
      s_seg[buf][lane] = seg_r;
      s_pre[buf][lane] = pre_r;
    }
  };

  // per-lane LDS offsets of the operand fetches
  int noff[KS];
#pragma unroll
  for (int ss = 0; ss < KS; ++ss) noff[ss] = tile_off<D>(l32, 2 * ss + g);
  int toff[DB][2];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2) {
      const int j = lane & 15;
      const int trow = 4 * g + (j >> 2) + 8 * h2;
      const int tcol = 32 * db + 16 * ((lane >> 4) & 1) + 4 * (j & 3);
      toff[db][h2] = tile_off<D>(trow, tcol >> 3) + ((tcol & 4) << 1);
    }
  auto nat_frag = [&](const char* tile, int ss) { return *(const bf16x8*)(tile + noff[ss]); };
  auto tr_frag = [&](const char* tile, int ks, int db) {
    const lds_char* p0 = (const lds_char*)(tile + 16 * ks * ROWB + toff[db][0]);
    const lds_char* p1 = (const lds_char*)(tile + 16 * ks * ROWB + toff[db][1]);
    bf16x4 x0 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) bf16x4*)p0);
    bf16x4 x1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) bf16x4*)p1);
    return __builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  auto tile_class = [&](int i, int& kt0, int& segbit) -> int {
    kt0 = tile_at(i, segbit) * kDqKeyTile;
    if (flags & RA_BIAS_PREFIX) return 2;
    return classify_pos(flags, bs.window, q_off + qw, q_off + qw + 31, kv_off + kt0,
                        kv_off + kt0 + kDqKeyTile - 1);
  };
  // terms that every tile must evaluate; a dense block with a summary is read only in the tiles
  // that the list marks (segbit)
  int tile_terms = RA_BIAS_ALIBI | RA_BIAS_PREFIX | RA_BIAS_DENSE;
  if constexpr (DENSE) {
    if (dmap != nullptr) tile_terms &= ~RA_BIAS_DENSE;
  }
  auto needs_bias = [&](int kt0, int segbit, int cls) -> bool {
    bool nb = (cls & 2) || (kt0 + kDqKeyTile > a.Lk);
    if (GENERAL) nb = nb || (flags & tile_terms) || segbit;
    return nb;
  };
  constexpr int PF = 2;
  auto compute_s_dp = [&](f32x16& S, f32x16& P, const char* kt, const char* vt) {
    bf16x8 fr[2 * KS];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      S[r] = 0.f;
      P[r] = 0.f;
    }
#pragma unroll
    for (int op = 0; op < PF; ++op) fr[op] = nat_frag((op & 1) ? vt : kt, op >> 1);
    // the fragments that the per-tile-term variants park in LDS are fetched from there here too:
    // they occupy no register outside the prologue
    bf16x8 qp0 = qf[0], qp1 = qf[1], dp0 = dof[0];
    if constexpr (GENERAL) {
      qp0 = s_q0[tid];
      qp1 = s_q1[tid];
      dp0 = s_do0[tid];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int op = 0; op < 2 * KS; ++op) {
      if (op + PF < 2 * KS) fr[op + PF] = nat_frag(((op + PF) & 1) ? vt : kt, (op + PF) >> 1);
      if (op & 1) P = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[op], op == 1 ? dp0 : dof[op >> 1], P, 0, 0, 0);
      else S = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[op], op == 0 ? qp0 : (op == 2 ? qp1 : qf[op >> 1]), S, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto compute_dq = [&](const bf16x8 (&dsf)[2], const char* kt) {
    bf16x8 fr[2 * DB];
#pragma unroll
    for (int op = 0; op < PF; ++op) fr[op] = tr_frag(kt, op / DB, op % DB);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int op = 0; op < 2 * DB; ++op) {
      if (op + PF < 2 * DB) fr[op + PF] = tr_frag(kt, (op + PF) / DB, (op + PF) % DB);
      acc[op % DB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[op], dsf[op / DB], acc[op % DB], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto prepare = [&](f32x16& S, int kt0, int segbit, int cls, int ids_buf) {
    TileBias tb;
    tb.flags = (cls & 2) ? (flags & (RA_BIAS_CAUSAL | RA_BIAS_WINDOW)) : 0;
    if (GENERAL) {
      tb.flags |= flags & tile_terms;
      if (segbit) tb.flags |= DENSE ? (flags & (RA_BIAS_SEGMENT | RA_BIAS_DENSE)) : RA_BIAS_SEGMENT;
    }
    tb.window = bs.window;
    tb.slope2 = slope2;
    tb.dense_mul = kLog2e / a.scale_res;
    tb.dense = nullptr;
    tb.dense_vs = 1;
    tb.dense_vec = 0;
    if (DENSE) {
      const float* head = dense_ptr + b * bs.dense_sb + h * bs.dense_sh;
      tb.dense_vec = kt0 + kDqKeyTile <= a.Lk && ((((uintptr_t)head) | ((uintptr_t)bs.dense_sq << 2)) & 15) == 0;
    }
    const int var0 = kt0 + 4 * g;
    tb.var_limit = a.Lk - var0;
    const int rel0 = (q_off + qi) - (kv_off + var0);
    if (DENSE)
      tb.dense = dense_ptr + b * bs.dense_sb + h * bs.dense_sh + (long long)min(qi, a.Lq - 1) * bs.dense_sq + var0;
    apply_bias<true, DENSE, GENERAL>(S, tb, rel0, q_seg, q_pre, &s_seg[ids_buf][4 * g], &s_pre[ids_buf][4 * g]);
  };

  // ---- prologue: tiles 0, 1, 2 in flight; S^T(0), dP^T(0) computed ------------------------------
  {
    int sbu;
    if (n > 0) {
      issue_tile(tile_at(0, sbu), 0);
      store_ids(0);
    }
    if (n > 1) {
      issue_tile(tile_at(1, sbu), 1);
      store_ids(1);
    }
    if (n > 2) issue_tile(tile_at(2, sbu), 2);  // its ids are stored at the top of iteration 0
  }
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();

  // Ordinals [plain_lo, plain_hi) of the tiles this wave sees completely, unmasked and in
  // range: they take the fused path without any per-tile classification.
  // The per-tile-term variants have up to four such stretches (their bounds wait in LDS): under
  // ALiBi a stretch must lie on one side of the diagonal, where -slope |q_pos - kv_pos| is linear
  // in both positions (stretches 0 and 2: keys before the workgroup's queries, 1 and 3: keys
  // after them); stretches 0 and 1 lie in the first run of one-id tiles, 2 and 3 in the second.
  int plain_lo = 0, plain_hi = 0;
  // ordinal of tile t inside the run: t - run_tile0
  int run_tile0 = run_base;
  const bool alibi_on = GENERAL && (flags & RA_BIAS_ALIBI);
  if constexpr (GENERAL) {
    int st_lo[4] = {0, 0, 0, 0}, st_hi[4] = {0, 0, 0, 0};
    if (wave_on && lse_in_range && !(flags & tile_terms & (RA_BIAS_PREFIX | RA_BIAS_DENSE))) {
      int lo, hi;
      key_tile_plain_range(flags, bs.window, q_off + qw, q_off + qw + 31, kv_off, a.Lk / kDqKeyTile,
                           kDqKeyTile, lo, hi);
      int lo2 = hi, hi1 = hi;
      if (alibi_on) {
        // the same bounds for all waves (the workgroup's first and last query): the waves meet at
        // a barrier per tile, so a generic iteration in one of them holds up all
        hi1 = min(hi, floor_div(q_off + q0 - kv_off - (kDqKeyTile - 1), kDqKeyTile) + 1);   // last key <= first query
        lo2 = max(lo, ceil_div(q_off + q0 + kDqRows - 1 - kv_off, kDqKeyTile));            // first key >= last query
      }
      st_lo[0] = max(lo - run_base, run_lo);
      st_hi[0] = max(min(hi1 - run_base, run_hi), st_lo[0]);
      st_lo[1] = max(max(lo2 - run_base, run_lo), st_hi[0]);
      st_hi[1] = max(min(hi - run_base, run_hi), st_lo[1]);
      const int r2_hi = min(run2_hi, n);
      st_lo[2] = max(max(lo - run2_base, run2_lo), st_hi[1]);
      st_hi[2] = max(min(hi1 - run2_base, r2_hi), st_lo[2]);
      st_lo[3] = max(max(lo2 - run2_base, run2_lo), st_hi[2]);
      st_hi[3] = max(min(hi - run2_base, r2_hi), st_lo[3]);
    }
    if (lane == 0) {
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        const int base = st < 2 ? run_base : run2_base, c_hi = st < 2 ? cons_hi : cons2_hi;
        // iteration i is plain for first < i < end.  It requests tile i + 3 by running addresses:
        // where the list goes on that must be the listed tile, behind the list's end it only has
        // to lie inside the shard (nobody reads it).
        const int list_end = c_hi >= n ? 0x3fffffff : c_hi - 3;
        s_st[wave][3 * st] = st_lo[st];
        s_st[wave][3 * st + 1] = min(min(st_hi[st] - 1, list_end), a.Lk / kDqKeyTile - base - 3);
        s_st[wave][3 * st + 2] = base;
      }
    }
  } else if (wave_on && lse_in_range) {
    int lo, hi;
    key_tile_plain_range(flags, bs.window, q_off + qw, q_off + qw + 31, kv_off, a.Lk / kDqKeyTile,
                         kDqKeyTile, lo, hi);
    plain_lo = max(lo - run_tile0, run_lo);
    plain_hi = max(min(hi - run_tile0, run_hi), plain_lo);
  }

  plain_lo = __builtin_amdgcn_readfirstlane(plain_lo);
  plain_hi = __builtin_amdgcn_readfirstlane(plain_hi);

  f32x16 s_a, p_a, s_b, p_b;
  bool cur_valid = false;
  if (n > 0 && wave_on) {
    int kt0, segbit;
    const int cls = tile_class(0, kt0, segbit);
    if (!(cls & 1)) {
      cur_valid = true;
      compute_s_dp(s_a, p_a, s_k[0], s_v[0]);
      if (needs_bias(kt0, segbit, cls)) prepare(s_a, kt0, segbit, cls, 0);
    }
  }
  // dS^T(i-1), packed in pairs, waiting for its dQ^T product
  u32x4 dsw[2];
#pragma unroll
  for (int e = 0; e < 4; ++e) dsw[0][e] = dsw[1][e] = 0u;
  bool pend_valid = false;
  auto pack2 = [&](float x0, float x1) -> unsigned {
    bf16x2 t;
    t[0] = (bf16_t)x0;
    t[1] = (bf16_t)x1;
    return __builtin_bit_cast(unsigned, t);
  };

  // Generic iteration; (SC, PC) hold S^T(i), dP^T(i); (SN, PN) receive tile i+1.  Tile j lives in
  // LDS buffer j % 6; iteration i reads tiles i-1 (transposed) and i+1, tile i stays for the next
  // iteration, tile i+2 is landing, tile i+3 is issued.
  auto iteration = [&](auto phase, int i, f32x16& SC, f32x16& PC, f32x16& SN, f32x16& PN) {
    constexpr int PH = decltype(phase)::value;
    constexpr int PHP = (PH + NBUF - 1) % NBUF, PH1 = (PH + 1) % NBUF, PH2 = (PH + 2) % NBUF, PH3 = (PH + 3) % NBUF;
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's share of tile i+2 is in LDS
    if (i + 2 < n) store_ids(PH2);       // ids of tile i+2 arrived with it
    __syncthreads();
    if (i + 3 < n) {
      int sbu;
      issue_tile(tile_at(i + 3, sbu), PH3);
    }
    if (pend_valid) {
      bf16x8 dsf[2];
      dsf[0] = __builtin_bit_cast(bf16x8, dsw[0]);
      dsf[1] = __builtin_bit_cast(bf16x8, dsw[1]);
      compute_dq(dsf, s_k[PHP]);
    }
    int nkt0 = 0, nsegbit = 0, ncls = 1;
    bool nxt_valid = false, nxt_bias = false;
    if (i + 1 >= plain_lo && i + 1 < plain_hi) {
      nxt_valid = true;
    } else if (i + 1 < n && wave_on) {
      ncls = tile_class(i + 1, nkt0, nsegbit);
      nxt_valid = !(ncls & 1);
      nxt_bias = nxt_valid && needs_bias(nkt0, nsegbit, ncls);
    }
    if (nxt_valid) compute_s_dp(SN, PN, s_k[PH1], s_v[PH1]);
    if (cur_valid) {
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        float ds[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          ds[e] = fast_exp2(fmaf(SC[r + e], a.scale_res, neg_lse2)) * (PC[r + e] - delta);
        }
        dsw[r >> 3][(r & 7) >> 1] = pack2(ds[0], ds[1]);
      }
    }
    pend_valid = cur_valid;
    if (nxt_bias) prepare(SN, nkt0, nsegbit, ncls, PH1);
    cur_valid = nxt_valid;
  };

  // Loads of the plain stretch: consecutive complete tiles, so the wave-uniform global addresses
  // advance by a constant and stay in scalar registers; nobody reads the ids of plain tiles.
  const bf16_t* k_run = kbase;
  const bf16_t* v_run = vbase;
  auto seek_plain = [&](int tile) {
    k_run = kbase + (long long)(tile * kDqKeyTile + RPW * wave_u) * a.k.sl;
    v_run = vbase + (long long)(tile * kDqKeyTile + RPW * wave_u) * a.v.sl;
  };
  auto issue_run = [&](int buf, int tid) {
    unsigned kvo = k_voff, vvo = v_voff;
    if (TIGHT) {
      kvo = s_voff[tid][0];
      vvo = s_voff[tid][1];
    }
    if (ld_lane_on) {
      global_to_lds16_s(k_run, kvo, RA_LDS_ADDR(&s_k[0][0]) + buf * TILE_BYTES + wave_u * RPW * ROWB);
      global_to_lds16_s(v_run, vvo, RA_LDS_ADDR(&s_v[0][0]) + buf * TILE_BYTES + wave_u * RPW * ROWB);
    }
    k_run += (long long)kDqKeyTile * a.k.sl;
    v_run += (long long)kDqKeyTile * a.v.sl;
  };

  // The same iteration for a stretch of plain tiles: tiles i-1, i and i+1 are plain and tile i+3
  // exists and is complete, so there is nothing to classify and no flag to consult.  Waves 4..7 take the
  // iteration's barrier between the two MFMA blocks instead of before them (see below).
  const bool late_half = wave_u >= 4;
  // The segment ids of a stretch's tiles (one id per tile) travel in scalar registers, fetched
  // ahead through the constant address space: the compiler uses the scalar cache and tracks the
  // load in flight itself (the array is not written while the kernel runs).
  typedef const __attribute__((address_space(4))) int* const_ids;
  const const_ids doc_ids = (const_ids)(uintptr_t)kv_seg;
  int doc_cur = 0, doc_nxt = 0, doc_far = 0;  // segment ids of tiles i, i + 1, i + 2 of a stretch
  float ali_s = 0.f;                          // +-slope in score units, set where a stretch begins
  const int q_first = q0;                     // the workgroup's first query row
  bf16_t ali_s_hi = (bf16_t)0.f, ali_s_lo = (bf16_t)0.f;
  auto plain_iteration = [&](auto phase, int i, f32x16& SC, f32x16& PC, f32x16& SN, f32x16& PN) {
    constexpr int PH = decltype(phase)::value;
    constexpr int PHP = (PH + NBUF - 1) % NBUF, PH1 = (PH + 1) % NBUF, PH3 = (PH + 3) % NBUF;
    const char* kp = s_k[PHP];
    const char* kn = s_k[PH1];
    const char* vn = s_v[PH1];
    // The per-tile-term variants rebuild the thread id per iteration (two instructions) instead
    // of carrying it, or the LDS addresses derived from it, through the loop.
    int tid_now = tid;
    if (GENERAL) {
      int ln;
      asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
      tid_now = wave_u * 64 + ln;
    }
    const int tid = tid_now;
    // documents: a lane whose query row carries another id than tile i takes no part in it - its
    // probabilities are exp2(-inf) = 0
    float gate = 0.f;
    if (GENERAL && seg_on) {
      gate = (s_stash[0][tid] == doc_cur) ? 0.f : RA_NEG_INF;
      doc_cur = doc_nxt;
      doc_nxt = doc_far;                                                      // requested one iteration ago
      doc_far = doc_ids[(long long)(run_tile0 + i + 3) * kDqKeyTile];        // tile i + 3 exists
    }
    // operands of the dQ^T product come from tile i-1, visible since two barriers ago
    bf16x8 frb[2 * DB];
#pragma unroll
    for (int op = 0; op < PF; ++op) frb[op] = tr_frag(kp, op / DB, op % DB);
    if (!late_half) {
      // all loads but the two of tile i+2 have landed: this wave's share of tile i+1 is in LDS.
      // The barrier is issued without a fence: a stretch writes nothing to LDS but through the
      // tile loads, which the counter above covers, and the operand fetches just issued (two LDS
      // instructions each) may stay in flight across it instead of being drained.
      __builtin_amdgcn_s_waitcnt(0x0f72);
      asm volatile("s_waitcnt lgkmcnt(%0)\n\ts_barrier" : : "n"(2 * PF) : "memory");
    }
    bf16x8 dsf[2];
    dsf[0] = __builtin_bit_cast(bf16x8, dsw[0]);
    dsf[1] = __builtin_bit_cast(bf16x8, dsw[1]);
    bf16x8 fra[2 * KS];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int op = 0; op < 2 * DB; ++op) {
      if (op + PF < 2 * DB) {
        frb[op + PF] = tr_frag(kp, (op + PF) / DB, (op + PF) % DB);
      } else if (!late_half) {
        // the first operands of the S^T / dP^T products ride behind the last dQ^T MFMAs
        const int o2 = op + PF - 2 * DB;
        fra[o2] = nat_frag((o2 & 1) ? vn : kn, o2 >> 1);
      }
      acc[op % DB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frb[op], dsf[op / DB], acc[op % DB], 0, 0, 0);
      if (op == 0) issue_run(PH3, tid);  // next loads: their issue hides behind the MFMAs
      __builtin_amdgcn_sched_barrier(0);
    }
    if (late_half) {
      // this half of the workgroup meets the barrier here, so that on every SIMD one wave runs
      // its dQ^T block while the other runs its S^T / dP^T block.  Tiles i+2 and i+3 may still
      // be in flight (two loads each).
      __builtin_amdgcn_s_waitcnt(0x0f74);
      barrier_bare();
#pragma unroll
      for (int op = 0; op < PF; ++op) fra[op] = nat_frag((op & 1) ? vn : kn, op >> 1);
    }
    bf16x8 q0 = qf[0], do0 = dof[0], q1 = qf[1];
    if (TIGHT) {
      q0 = s_q0[tid];
      do0 = s_do0[tid];
    }
    if (GENERAL) q1 = s_q1[tid];
    // The chain of a score element (exp2 and the scaled dP, their product, the packing of a
    // pair) is spread over three consecutive MFMA slots, one link per slot, so that no vector
    // instruction waits for the result of the one before it.
    constexpr int EPO = 16 / (2 * KS) > 0 ? 16 / (2 * KS) : 1;
    float ev[16], uv[16], dsv[16];
    auto chain_links = [&](int slot) {
#pragma unroll
      for (int e = 0; e < EPO; ++e) {
        const int r = slot * EPO + e;
        if (r >= 0 && r < 16) {
          if (GENERAL) ev[r] = fast_exp2(fmaf(SC[r], a.scale_res, gate));
          else ev[r] = fast_exp2(SC[r] * a.scale_res);
          uv[r] = fmaf(PC[r], c_row, cd_row);
          asm volatile("" : "+v"(ev[r]), "+v"(uv[r]));  // pins the arithmetic between two MFMAs
        }
      }
#pragma unroll
      for (int e = 0; e < EPO; ++e) {
        const int r = (slot - 1) * EPO + e;
        if (r >= 0 && r < 16) {
          dsv[r] = ev[r] * uv[r];
          asm volatile("" : "+v"(dsv[r]));
        }
      }
#pragma unroll
      for (int e = 0; e < EPO; ++e) {
        const int r = (slot - 2) * EPO + e;
        if (r >= 0 && r < 16 && (r & 1)) {
          unsigned dw = pack2(dsv[r - 1], dsv[r]);
          asm volatile("" : "+v"(dw));
          dsw[r >> 3][(r & 7) >> 1] = dw;
        }
      }
    };
    if (GENERAL && alibi_on) {
      // ALiBi of tile i+1 through the matrix unit: the accumulators start from
      //   [j, j, 1, 1, 1] x [s_hi, s_lo, c_hi, c_mid, c_lo] = s j + c = -slope |q_pos - kv_pos| (score units)
      // with s = +-slope (the sign of the stretch), j the key's index in the tile and
      // c = -s (q_pos - position of the tile's first key); s is split into two bf16 words and c
      // into three (c grows with the distance between the shards: three words carry it to fp32
      // accuracy, what an addition in the score chain would give), so that the chain below needs
      // no instruction for the bias.
      // (recomputed per tile from the lane number: the loop has no register to carry it in)
      const int ramp_lane = tid & 63;
      const int rel_i = q_off + q_first + (tid >> 6) * 32 + (ramp_lane & 31) - (kv_off + (run_tile0 + i + 1) * kDqKeyTile);
      const float ali_c = -ali_s * (float)rel_i;
      const bf16_t c_hi = (bf16_t)ali_c;
      const bf16_t c_mid = (bf16_t)(ali_c - (float)c_hi);
      const bf16_t c_lo = (bf16_t)((ali_c - (float)c_hi) - (float)c_mid);
      bf16x8 bq;
      bq[0] = ali_s_hi;
      bq[1] = ali_s_lo;
      bq[2] = c_hi;
      bq[3] = c_mid;
      bq[4] = c_lo;
      bq[5] = bq[6] = bq[7] = (bf16_t)0.f;
      f32x16 z;
#pragma unroll
      for (int r = 0; r < 16; ++r) z[r] = 0.f;
      SN = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s_ramp[ramp_lane], bq, z, 0, 0, 0);
    } else if (GENERAL) {
#pragma unroll
      for (int r = 0; r < 16; ++r) SN[r] = 0.f;
    }
#pragma unroll
    for (int op = 0; op < 2 * KS; ++op) {
      if (op + PF < 2 * KS) fra[op + PF] = nat_frag(((op + PF) & 1) ? vn : kn, (op + PF) >> 1);
      if (op < 2) {
        f32x16 z;
#pragma unroll
        for (int r = 0; r < 16; ++r) z[r] = 0.f;
        if (op & 1) PN = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fra[op], do0, z, 0, 0, 0);
        else if (GENERAL) SN = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fra[op], q0, SN, 0, 0, 0);
        else SN = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fra[op], q0, z, 0, 0, 0);
      } else {
        if (op & 1) PN = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fra[op], dof[op >> 1], PN, 0, 0, 0);
        else SN = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fra[op], op == 2 ? q1 : qf[op >> 1], SN, 0, 0, 0);
      }
      chain_links(op);
      __builtin_amdgcn_sched_barrier(0);
    }
    chain_links(2 * KS);      // the links that the last slots left over
    chain_links(2 * KS + 1);
  };

  // Three loops over the same sequence of tiles: generic iterations up to the plain stretch, the
  // plain stretch in whole groups of six, generic iterations for the rest.  Every wave runs n
  // iterations in total, so the barrier counts agree.
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  using P2 = std::integral_constant<int, 2>;
  using P3 = std::integral_constant<int, 3>;
  using P4 = std::integral_constant<int, 4>;
  using P5 = std::integral_constant<int, 5>;
  int i = 0;
  if constexpr (!GENERAL) {
  // iteration i is plain for plain_lo < i < plain_end
  // (tile i+3 must exist, belong to the run and be complete)
  const int plain_end = __builtin_amdgcn_readfirstlane(
      min(min(plain_hi - 1, min(run_hi, n) - 3), a.Lk / kDqKeyTile - run_tile0 - 3));
  for (; i < n && !(i > plain_lo && i + 6 <= plain_end); i += 6) {
    iteration(P0{}, i, s_a, p_a, s_b, p_b);
    if (i + 1 < n) iteration(P1{}, i + 1, s_b, p_b, s_a, p_a);
    if (i + 2 < n) iteration(P2{}, i + 2, s_a, p_a, s_b, p_b);
    if (i + 3 < n) iteration(P3{}, i + 3, s_b, p_b, s_a, p_a);
    if (i + 4 < n) iteration(P4{}, i + 4, s_a, p_a, s_b, p_b);
    if (i + 5 < n) iteration(P5{}, i + 5, s_b, p_b, s_a, p_a);
  }
  {
    const bool stretch = i + 6 <= plain_end;
    if (stretch) seek_plain(run_tile0 + i + 3);
    if (stretch) {
      // the two row constants of the stretch replace the two of the generic iterations, which
      // wait in LDS meanwhile (the kernel has no register to spare)
      c_row = fast_exp2(neg_lse2);
      cd_row = -c_row * delta;
      s_rowc[0][tid] = neg_lse2;
      s_rowc[1][tid] = delta;
      neg_lse2 = delta = 0.f;
    }
    for (; i + 6 <= plain_end; i += 6) {
      plain_iteration(P0{}, i, s_a, p_a, s_b, p_b);
      plain_iteration(P1{}, i + 1, s_b, p_b, s_a, p_a);
      plain_iteration(P2{}, i + 2, s_a, p_a, s_b, p_b);
      plain_iteration(P3{}, i + 3, s_b, p_b, s_a, p_a);
      plain_iteration(P4{}, i + 4, s_a, p_a, s_b, p_b);
      plain_iteration(P5{}, i + 5, s_b, p_b, s_a, p_a);
    }
    if (stretch) {
      neg_lse2 = s_rowc[0][tid];
      delta = s_rowc[1][tid];
    }
  }
  } else {
#pragma unroll 1
  for (int st = 0; st < 4; ++st) {
    // iteration i is plain for p_lo < i < p_end
    const int p_lo = __builtin_amdgcn_readfirstlane(s_st[wave_u][3 * st]);
    const int p_end = __builtin_amdgcn_readfirstlane(s_st[wave_u][3 * st + 1]);
    const int start = max(i, ((p_lo + 6) / 6) * 6);  // i is a multiple of six here
    if (start + 6 > p_end) continue;
    run_tile0 = __builtin_amdgcn_readfirstlane(s_st[wave_u][3 * st + 2]);
    for (; i < start; i += 6) {
      iteration(P0{}, i, s_a, p_a, s_b, p_b);
      iteration(P1{}, i + 1, s_b, p_b, s_a, p_a);
      iteration(P2{}, i + 2, s_a, p_a, s_b, p_b);
      iteration(P3{}, i + 3, s_b, p_b, s_a, p_a);
      iteration(P4{}, i + 4, s_a, p_a, s_b, p_b);
      iteration(P5{}, i + 5, s_b, p_b, s_a, p_a);
    }
    seek_plain(run_tile0 + i + 3);
    if (seg_on) {
      doc_cur = doc_ids[(long long)(run_tile0 + i) * kDqKeyTile];
      doc_nxt = doc_ids[(long long)(run_tile0 + i + 1) * kDqKeyTile];
      doc_far = doc_ids[(long long)(run_tile0 + i + 2) * kDqKeyTile];
    }
    if (alibi_on) {
      // keys before the queries (even stretches): bias = -slope (q_pos - kv_pos), rising with the
      // key's index; keys after them: falling
      ali_s = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(
          __builtin_bit_cast(int, (st & 1) ? -slope2 : slope2)));  // one slope per head
      ali_s_hi = (bf16_t)ali_s;
      ali_s_lo = (bf16_t)(ali_s - (float)ali_s_hi);
    }
    seg_r = pre_r = 0;  // stored already; not carried through the stretch
    // the two row constants of the stretch replace the two of the generic iterations, which wait
    // in LDS meanwhile with everything else only the generic iterations use
    c_row = fast_exp2(neg_lse2);
    cd_row = -c_row * delta;
    s_rowc[0][tid] = neg_lse2;
    s_rowc[1][tid] = delta;
    neg_lse2 = delta = 0.f;
    s_stash[0][tid] = q_seg;
    s_stash[1][tid] = q_pre;
    s_stash[2][tid] = __float_as_int(slope2);
    for (; i + 6 <= p_end; i += 6) {
      plain_iteration(P0{}, i, s_a, p_a, s_b, p_b);
      plain_iteration(P1{}, i + 1, s_b, p_b, s_a, p_a);
      plain_iteration(P2{}, i + 2, s_a, p_a, s_b, p_b);
      plain_iteration(P3{}, i + 3, s_b, p_b, s_a, p_a);
      plain_iteration(P4{}, i + 4, s_a, p_a, s_b, p_b);
      plain_iteration(P5{}, i + 5, s_b, p_b, s_a, p_a);
    }
    neg_lse2 = s_rowc[0][tid];
    delta = s_rowc[1][tid];
    q_seg = s_stash[0][tid];
    q_pre = s_stash[1][tid];
    slope2 = __int_as_float(s_stash[2][tid]);
    if (seg_on && q_seg != doc_cur) {
      // the scores of tile i, which the next generic iteration turns into probabilities, came
      // out of the stretch without a mask: rows of another document drop out here
#pragma unroll
      for (int r = 0; r < 16; ++r) s_a[r] = RA_NEG_INF;
    }
    if (lane < kDqKeyTile) {
      // the stretch moved no ids: those of the two tiles in flight are fetched now (i is a
      // multiple of 6 here: tile i+1 lives in buffer 1, the ids of tile i+2 wait in registers
      // for the top of the next iteration, as after a generic iteration).  Every wave does this for
      // itself, as it fetches and stores the ids in its generic iterations: the waves enter and
      // leave their stretches at different tiles and must not depend on one another for the ids.
      int sbu;
      if (i + 1 < n) {
        const int kk = min(tile_at(i + 1, sbu) * kDqKeyTile + lane, a.Lk - 1);
        s_seg[1][lane] = kv_seg ? kv_seg[kk] : 0;
        s_pre[1][lane] = kv_pre ? kv_pre[kk] : 0;
      }
      if (i + 2 < n) {
        const int kk = min(tile_at(i + 2, sbu) * kDqKeyTile + lane, a.Lk - 1);
        if (kv_seg) seg_r = kv_seg[kk];
        if (kv_pre) pre_r = kv_pre[kk];
      }
    }
  }
  }
  for (; i < n; i += 6) {
    iteration(P0{}, i, s_a, p_a, s_b, p_b);
    if (i + 1 < n) iteration(P1{}, i + 1, s_b, p_b, s_a, p_a);
    if (i + 2 < n) iteration(P2{}, i + 2, s_a, p_a, s_b, p_b);
    if (i + 3 < n) iteration(P3{}, i + 3, s_b, p_b, s_a, p_a);
    if (i + 4 < n) iteration(P4{}, i + 4, s_a, p_a, s_b, p_b);
    if (i + 5 < n) iteration(P5{}, i + 5, s_b, p_b, s_a, p_a);
  }
  if (pend_valid) {  // product of the last tile
    bf16x8 dsf[2];
    dsf[0] = __builtin_bit_cast(bf16x8, dsw[0]);
    dsf[1] = __builtin_bit_cast(bf16x8, dsw[1]);
    compute_dq(dsf, s_k[0] + ((n - 1) % NBUF) * TILE_BYTES);
  }
  }  // key/value shards
  const bool whole_ring = MULTI && (flags & kFlagWhole);
  if (!whole_ring && tiles_listed == 0) return;  // nothing to add
  if constexpr (MULTI) {
    if (whole_ring) {
      // dQ of these rows is complete: bf16, in the caller's layout
      if (q_valid) {
        bf16_t* dq = (bf16_t*)ring.x0[blockIdx.y] + b * a.out_sb + h * a.out_sh + (long long)qi * a.out_sl + 4 * g;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int bb = 0; bb < 4; ++bb) {
            bf16x4 t;
#pragma unroll
            for (int c = 0; c < 4; ++c) t[c] = (bf16_t)(acc[db][4 * bb + c] * a.sm_scale);
            *(bf16x4*)(dq + 32 * db + 8 * bb) = t;
          }
      }
      return;
    }
  }
  if (q_valid) {
    float* dq_res = a.dq;
    if constexpr (MULTI) dq_res = ring.x0[blockIdx.y];
    float* dq = dq_res + row * D + 4 * g;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) {
        f32x4 t = *(f32x4*)(dq + 32 * db + 8 * bb);
#pragma unroll
        for (int c = 0; c < 4; ++c) t[c] += acc[db][4 * bb + c] * a.sm_scale;
        *(f32x4*)(dq + 32 * db + 8 * bb) = t;
      }
  }
}

// ------------------------------------------------------------------------------------------------
// ------------------------------------------------------------------------------------------------
// fp32 accumulator -> bf16 gradient in the caller's layout
// ------------------------------------------------------------------------------------------------
// The accumulators of n_pass shards lie one after another; shard p is written to out + p * sp.
__global__ void bwd_finalize_kernel(const float* acc, bf16_t* out, long long sp, long long sb, long long sh,
                                    long long sl, int n_pass, int B, int H, int L, int D) {
  const int cpr = D / 4;
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long rows = (long long)n_pass * B * H * L;
  if (i >= rows * cpr) return;
  const long long row = i / cpr;
  const int c = (int)(i % cpr);
  const int li = (int)(row % L);
  const int h = (int)((row / L) % H);
  const long long bp = row / ((long long)L * H);
  const int b = (int)(bp % B);
  out += (bp / B) * sp;
  f32x4 x = *(const f32x4*)(acc + row * D + 4 * c);
  bf16x4 y;
#pragma unroll
  for (int e = 0; e < 4; ++e) y[e] = (bf16_t)x[e];
  *(bf16x4*)(out + b * sb + h * sh + (long long)li * sl + 4 * c) = y;
}

// ------------------------------------------------------------------------------------------------
// launchers
// ------------------------------------------------------------------------------------------------
hipError_t launch_bwd_delta(const void* out, int out_f32, long long sp, long long sb, long long sh, long long sl,
                            TensorArg dout, long long dsp, float* delta, int n_pass, int B, int H, int Lq, int D,
                            hipStream_t stream) {
  const long long rows = (long long)n_pass * B * H * Lq;
  const int rpb = 256 / (D / 8);
  dim3 grid((unsigned)((rows + rpb - 1) / rpb)), block(256);
  if (D == 128) {
    if (out_f32) hipLaunchKernelGGL((bwd_delta_kernel<float, 128>), grid, block, 0, stream, (const float*)out, sp, sb, sh, sl, dout, dsp, delta, n_pass, B, H, Lq);
    else hipLaunchKernelGGL((bwd_delta_kernel<bf16_t, 128>), grid, block, 0, stream, (const bf16_t*)out, sp, sb, sh, sl, dout, dsp, delta, n_pass, B, H, Lq);
  } else {
    if (out_f32) hipLaunchKernelGGL((bwd_delta_kernel<float, 64>), grid, block, 0, stream, (const float*)out, sp, sb, sh, sl, dout, dsp, delta, n_pass, B, H, Lq);
    else hipLaunchKernelGGL((bwd_delta_kernel<bf16_t, 64>), grid, block, 0, stream, (const bf16_t*)out, sp, sb, sh, sl, dout, dsp, delta, n_pass, B, H, Lq);
  }
  return hipGetLastError();
}

// mode: as for launch_fwd_step
hipError_t launch_bwd_step(const BwdArgs& a, int D, int mode, int parts, hipStream_t stream) {
  if (parts & 1) {
    const int keys_wg = 128;
    const int nkt = (a.Lk + keys_wg - 1) / keys_wg;
    dim3 grid((unsigned)(a.B * a.H * nkt)), block(256);
    if (D == 128) {
      if (mode == 2) hipLaunchKernelGGL((dkdv_kernel<128, 2, false>), grid, block, 0, stream, a, NoShardList{});
      else if (mode == 1) hipLaunchKernelGGL((dkdv_kernel<128, 1, false>), grid, block, 0, stream, a, NoShardList{});
      else hipLaunchKernelGGL((dkdv_kernel<128, 0, false>), grid, block, 0, stream, a, NoShardList{});
    } else {
      if (mode == 2) hipLaunchKernelGGL((dkdv_kernel<64, 2, false>), grid, block, 0, stream, a, NoShardList{});
      else if (mode == 1) hipLaunchKernelGGL((dkdv_kernel<64, 1, false>), grid, block, 0, stream, a, NoShardList{});
      else hipLaunchKernelGGL((dkdv_kernel<64, 0, false>), grid, block, 0, stream, a, NoShardList{});
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  if (parts & 2) {
    const int nqt = (a.Lq + kDqRows - 1) / kDqRows;
    dim3 grid((unsigned)(a.B * a.H * nqt)), block(kDqThreads);
    if (D == 128) {
      if (mode == 2) hipLaunchKernelGGL((dq_kernel<128, 2, false>), grid, block, 0, stream, a, NoShardList{});
      else if (mode == 1) hipLaunchKernelGGL((dq_kernel<128, 1, false>), grid, block, 0, stream, a, NoShardList{});
      else hipLaunchKernelGGL((dq_kernel<128, 0, false>), grid, block, 0, stream, a, NoShardList{});
    } else {
      if (mode == 2) hipLaunchKernelGGL((dq_kernel<64, 2, false>), grid, block, 0, stream, a, NoShardList{});
      else if (mode == 1) hipLaunchKernelGGL((dq_kernel<64, 1, false>), grid, block, 0, stream, a, NoShardList{});
      else hipLaunchKernelGGL((dq_kernel<64, 0, false>), grid, block, 0, stream, a, NoShardList{});
    }
  }
  return hipGetLastError();
}

hipError_t launch_bwd_dkdv_steps(const BwdArgs& a, const QRing& shards, int D, int mode, hipStream_t stream) {
  const int keys_wg = 128;
  const int nkt = (a.Lk + keys_wg - 1) / keys_wg;
  dim3 grid((unsigned)(a.B * a.H * nkt), (unsigned)shards.n_pass), block(256);
  if (D == 128) {
    if (mode == 2) hipLaunchKernelGGL((dkdv_kernel<128, 2, true>), grid, block, 0, stream, a, shards);
    else if (mode == 1) hipLaunchKernelGGL((dkdv_kernel<128, 1, true>), grid, block, 0, stream, a, shards);
    else hipLaunchKernelGGL((dkdv_kernel<128, 0, true>), grid, block, 0, stream, a, shards);
  } else {
    if (mode == 2) hipLaunchKernelGGL((dkdv_kernel<64, 2, true>), grid, block, 0, stream, a, shards);
    else if (mode == 1) hipLaunchKernelGGL((dkdv_kernel<64, 1, true>), grid, block, 0, stream, a, shards);
    else hipLaunchKernelGGL((dkdv_kernel<64, 0, true>), grid, block, 0, stream, a, shards);
  }
  return hipGetLastError();
}

hipError_t launch_bwd_dq_steps(const BwdArgs& a, const KvRing& shards, int D, int mode, hipStream_t stream) {
  const int nqt = (a.Lq + kDqRows - 1) / kDqRows;
  dim3 grid((unsigned)(a.B * a.H * nqt), (unsigned)shards.n_pass), block(kDqThreads);
  if (D == 128) {
    if (mode == 2) hipLaunchKernelGGL((dq_kernel<128, 2, true>), grid, block, 0, stream, a, shards);
    else if (mode == 1) hipLaunchKernelGGL((dq_kernel<128, 1, true>), grid, block, 0, stream, a, shards);
    else hipLaunchKernelGGL((dq_kernel<128, 0, true>), grid, block, 0, stream, a, shards);
  } else {
    if (mode == 2) hipLaunchKernelGGL((dq_kernel<64, 2, true>), grid, block, 0, stream, a, shards);
    else if (mode == 1) hipLaunchKernelGGL((dq_kernel<64, 1, true>), grid, block, 0, stream, a, shards);
    else hipLaunchKernelGGL((dq_kernel<64, 0, true>), grid, block, 0, stream, a, shards);
  }
  return hipGetLastError();
}

hipError_t launch_bwd_finalize(const float* acc, void* out, long long sp, long long sb, long long sh, long long sl,
                               int n_pass, int B, int H, int L, int D, hipStream_t stream) {
  const long long n = (long long)n_pass * B * H * L * (D / 4);
  hipLaunchKernelGGL(bwd_finalize_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, acc,
                     (bf16_t*)out, sp, sb, sh, sl, n_pass, B, H, L, D);
  return hipGetLastError();
}

}  // namespace ra

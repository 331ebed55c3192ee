// Forward ring step for gfx950: (o, m, l) <- online-softmax update with one K/V shard.
//
// Work split: one workgroup = 8 waves = 256 query rows of one (batch, head); wave w owns 32
// rows.  K/V are streamed in 64-key tiles through LDS (double buffered).  Scores are
// produced TRANSPOSED, S^T = K Q^T, so that in the 32x32 MFMA accumulator a lane owns one
// query row (lane%32) and 16 keys: row max / row sum are in-register reductions plus one
// exchange with lane^32, the rescale of the running output is a per-lane scalar, and the
// bf16 probabilities are already laid out as the B operand of O^T = V^T P^T, whose A
// operand comes from the V tile through the transposing LDS read.
#include <type_traits>

#include "ra_launch.h"

namespace ra {

constexpr int kFwdThreads = 512;
constexpr int kFwdRows = 256;   // query rows per workgroup
constexpr int kKeyTile = 64;    // keys per LDS tile
constexpr int kMaxListTiles = 1024;

// MULTI: grid dimension y is a ring pass, the trip of one query shard around the ring.  The launch
// walks the key/value shards that `ring` lists for the pass one after another (the arguments of
// consecutive ring steps of that query shard); the step's contribution stays in registers between
// them and meets the carry of the pass once, at the end.
// WHOLE: a whole-ring launch (see kFlagWhole) - its own instantiation: the variants that merge a
// carry keep the register allocation they have without the extra exit path.
template <int D, int MODE, bool MULTI, bool WHOLE = false>
__global__ __launch_bounds__(kFwdThreads) void fwd_step_kernel(
    const FwdArgs a, const std::conditional_t<MULTI, KvRing, NoShardList> ring) {
  static_assert(MULTI || !WHOLE, "a whole-ring launch walks the shards of its passes itself");
  constexpr bool GENERAL = MODE != 0;  // bias terms beyond causal / window
  constexpr bool DENSE = MODE == 2;    // ... including a materialised bias block
  constexpr int KS = D / 16;  // k-steps of the QK^T contraction
  constexpr int DB = D / 32;  // 32-wide blocks of the head dim
  constexpr int TILE_BYTES = kKeyTile * D * 2;

  __shared__ __attribute__((aligned(16))) char s_k[4][TILE_BYTES];
  __shared__ __attribute__((aligned(16))) char s_v[4][TILE_BYTES];
  __shared__ __attribute__((aligned(16))) int s_seg[4][kKeyTile];
  __shared__ __attribute__((aligned(16))) int s_pre[4][kKeyTile];
  __shared__ unsigned short s_list[GENERAL ? kMaxListTiles : 1];
  // The several-shard variants with per-tile terms park a third Q fragment in LDS (s_q2); the
  // room comes from a one-word stash, from the tile flags sharing the stash's memory (they are
  // used before a shard's loops, the stash inside them, a barrier separates two shards) and
  // from a ramp table without its all-zero half.
  constexpr bool PARK2 = GENERAL;
  // generic iterations issue their tile requests last (see the end of `iteration`): all variants
  // but the single-shard causal one
  constexpr bool DEFER = GENERAL || MULTI;
  __shared__ unsigned char s_flag_own[(GENERAL && !PARK2) ? kMaxListTiles : 1];
  __shared__ int s_red[28];
  __shared__ int s_st[GENERAL ? 8 : 1][12];  // per wave and stretch: first iteration, end, tile_base
  __shared__ int s_stash[GENERAL ? (PARK2 ? 1 : 3) : 1][GENERAL ? kFwdThreads : 1];
  static_assert(!PARK2 || kMaxListTiles <= kFwdThreads * 4, "the tile flags fit the stash");
  unsigned char* const s_flag = PARK2 ? (unsigned char*)&s_stash[0][0] : s_flag_own;
  // The GENERAL and MULTI variants are a few registers short in their straight-line loop: the
  // first operand fragment of Q waits here and is fetched once per iteration instead.
  constexpr bool TIGHT = GENERAL || MULTI;
  __shared__ __attribute__((aligned(16))) bf16x8 s_q0[TIGHT ? kFwdThreads : 1];
  __shared__ __attribute__((aligned(16))) bf16x8 s_q1[GENERAL ? kFwdThreads : 1];  // the second one too
  __shared__ __attribute__((aligned(16))) bf16x8 s_q2[PARK2 ? kFwdThreads : 1];    // ... and the third
  // ALiBi inside the straight-line loop (see plain_iteration): the key-side operand of the extra
  // matrix instruction, one fragment per 32-key block and lane
  // (lanes 32..63 hold the zero half of the operand: PARK2 gives them one shared zero entry, the last)
  __shared__ __attribute__((aligned(16))) bf16x8 s_ramp[GENERAL ? (PARK2 ? 65 : 128) : 1];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);  // same value in a scalar register
  const int l32 = lane & 31, g = lane >> 5;
  const int nqt = (a.Lq + kFwdRows - 1) / kFwdRows;
  int hh, qt;
  decode_block(blockIdx.x, a.B * a.H, nqt, hh, qt);
  const int b = hh / a.H, h = hh % a.H;
  const int q0 = qt * kFwdRows;
  const int qw = q0 + wave * 32;
  const int qi = qw + l32;
  const bool q_valid = qi < a.Lq;
  const int qi_c = min(qi, a.Lq - 1);
  const BiasArgs& bs = a.bias;
  const int flags = bs.flags;
  // the query side of this workgroup's pass (read from the argument block where it is needed:
  // nothing of it is carried through the loops)
  auto pass_q_off = [&]() -> int { if constexpr (MULTI) return ring.q_off[blockIdx.y]; else return bs.q_off; };
  auto pass_o = [&]() -> float* { if constexpr (MULTI) return ring.x0[blockIdx.y]; else return a.o; };
  auto pass_m = [&]() -> float* { if constexpr (MULTI) return ring.x1[blockIdx.y]; else return a.m; };
  auto pass_l = [&]() -> float* { if constexpr (MULTI) return ring.x2[blockIdx.y]; else return a.l; };

  // ---- per-lane query state ------------------------------------------------------------
  bf16x8 qf[KS];
  {
    const bf16_t* q_ptr = a.q.ptr;
    if constexpr (MULTI) q_ptr = ring.q[blockIdx.y];
    const bf16_t* qp = q_ptr + b * a.q.sb + h * a.q.sh + (long long)qi_c * a.q.sl + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; ++s) qf[s] = *(const bf16x8*)(qp + 16 * s);
    if (TIGHT) s_q0[tid] = qf[0];
    if (GENERAL) s_q1[tid] = qf[1];
    if (PARK2) s_q2[tid] = qf[2];
    if (GENERAL && tid < 64) {
      // row (32 kb + l32) of the 32 x 16 operand is [j, j, 1, 1, 1, 0 ...] with j the key's index in
      // the tile (exact in bf16); lanes 32..63 hold the other eight columns, all zero
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        bf16x8 rf;
#pragma unroll
        for (int e = 0; e < 8; ++e) rf[e] = (bf16_t)0.f;
        if (g == 0) {
          rf[0] = rf[1] = (bf16_t)(float)(32 * kb + l32);
          rf[2] = rf[3] = rf[4] = (bf16_t)1.0f;
        }
        if (!PARK2) s_ramp[64 * kb + tid] = rf;
        else if (tid < 32) s_ramp[32 * kb + tid] = rf;
        else if (tid == 32 && kb == 0) s_ramp[64] = rf;  // all zero
      }
    }
  }
  long long row = ((long long)b * a.H + h) * a.Lq + qi_c;
  // This step accumulates its own contribution from zero and is merged with the incoming carry
  // at the end.  Two row sums are kept: l_run adds the fp32 probabilities (it becomes the
  // carry's l and the logsumexp), lr_run adds the SAME probabilities after their rounding to
  // bf16, i.e. the weights that actually multiply V.  Scaling the step's output by
  // l_run / lr_run makes it a properly normalised average of V times the exact row sum, so
  // the rounding of P cancels in o / l instead of showing up as an error of order 2^-9 |v|
  // on rows that see only a few keys.
  // whole-ring launch: no carry comes in, the finished output goes out
  float m_run = WHOLE ? RA_NEG_INF : pass_m()[row] * kLog2e;  // exponent reference (log2 domain), moves lazily
  float l_run = 0.f, lr_run = 0.f;  // per-lane partial sums (this lane's keys only)
  // (Both sums in every loop: where a row's weight sits on one or two keys, the rounded sum
  // alone carries the rounding error of those few weights, up to 2^-8 relative, into the
  // logsumexp.)
  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
  bf16x2 ones2;
  ones2[0] = (bf16_t)1.0f;
  ones2[1] = (bf16_t)1.0f;
  int q_seg = 0, q_pre = 0;
  float slope2 = 0.f;
  if (GENERAL) {
    const int* q_seg_ptr = bs.q_seg;
    const int* q_pre_ptr = bs.q_pre;
    if constexpr (MULTI) {
      q_seg_ptr = ring.q_seg[blockIdx.y];
      q_pre_ptr = ring.q_pre[blockIdx.y];
    }
    if (flags & RA_BIAS_SEGMENT) q_seg = q_seg_ptr[b * bs.q_seg_sb + qi_c];
    if (flags & RA_BIAS_PREFIX) q_pre = q_pre_ptr[b * bs.q_pre_sb + qi_c];
    if (flags & RA_BIAS_ALIBI) slope2 = bs.slopes[h] * kLog2e;
  }
  float m_true = m_run;  // exact running maximum; m_run is the (possibly stale) exponent reference

  // ---- one pass of everything below per key/value shard ------------------------------------
  int kv_off = bs.kv_off;
  const bf16_t* k_ptr = a.k.ptr;
  const bf16_t* v_ptr = a.v.ptr;
  const int* kv_seg_ptr = bs.kv_seg;
  const int* kv_pre_ptr = bs.kv_pre;
  const float* dense_ptr = bs.dense;
  int n_shards = 1;
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
    // the late waves may still be reading the last V tile of the previous shard
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
  const int* kv_seg = (GENERAL && (flags & RA_BIAS_SEGMENT)) ? kv_seg_ptr + b * bs.kv_seg_sb : nullptr;
  const int* kv_pre = (GENERAL && (flags & RA_BIAS_PREFIX)) ? kv_pre_ptr + b * bs.kv_pre_sb : nullptr;
  // ---- which key tiles does this workgroup visit ------------------------------------------
  const int ntiles = (a.Lk + kKeyTile - 1) / kKeyTile;
  const int q_rows_hi = min(q0 + kFwdRows, a.Lq) - 1;
  int j_lo, j_hi;
  const int q_off = pass_q_off();
  key_tile_range(flags, bs.window, q_off + q0, q_off + q_rows_hi, kv_off, ntiles, kKeyTile,
                 j_lo, j_hi);
  int n_act = j_hi - j_lo;
  bool use_list = false;
  // Ordinals [run_lo, run_hi) are consecutive tiles `tile_base + ordinal` whose 64 keys share one
  // segment id each (not necessarily the same one, nor that of every query of the workgroup): the
  // straight-line loop walks them with one comparison per lane and tile - the lane's query row
  // belongs to the tile's document or it does not.  wg_one_doc: all queries of the workgroup
  // share one id, so that a listed tile with one id needs no test at all.
  int run_lo = 0, run_hi = n_act, tile_base = j_lo;
  // ... and a second such run further on (a workgroup whose queries straddle a document boundary
  // lists the tiles of both documents, with the tile that holds the boundary between them)
  int run2_lo = 0, run2_hi = 0, tile_base2 = 0;
  // the listed tiles count up without a gap from the start of a run to ordinal cons_hi / cons2_hi
  int cons_hi = n_act, cons2_hi = 0;
  bool wg_one_doc = true;
  // A dense block that comes with its summary is listed the same way: tiles in which the
  // workgroup's rows hold nothing but -inf are left out, tiles of zeros count as tiles of one
  // id (no term to evaluate: they may join a straight-line stretch), the rest is evaluated
  // element by element.  (Single-step launches only.)
  const unsigned char* dmap = nullptr;
  if constexpr (DENSE && !MULTI) {
    if (bs.dense_map) dmap = dense_map_of(bs, b, h, a.H, a.Lq, a.Lk);
  }
  const bool seg_list = GENERAL && (flags & RA_BIAS_SEGMENT);
  if (seg_list || (DENSE && dmap != nullptr)) {
    // segment-id range of the workgroup's queries, then one thread per key tile decides
    // whether the id ranges can intersect (skip otherwise) and whether the tile has one id
    use_list = true;
    int qmin = 0, qmax = 0;
    if (seg_list) {
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
    for (int j = j_lo + tid; j < j_hi; j += kFwdThreads) {
      int f = 1;
      if (seg_list) {
        int kmin, kmax;
        tile_id_range<kKeyTile>(kv_seg, j, a.Lk, kmin, kmax);
        const bool act = !(kmax < qmin || kmin > qmax);
        f = act ? ((kmin == kmax) ? 1 : 3) : 0;
      }
      if constexpr (DENSE) {
        if (dmap != nullptr && f != 0) {
          const int bits = dense_map_or(dmap, a.Lk, q0, q_rows_hi, j * kKeyTile, min((j + 1) * kKeyTile, a.Lk) - 1);
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
        s_red[16] = cnt;
        s_red[17] = u_lo;
        s_red[18] = u_hi;
        s_red[19] = u_base;
        s_red[20] = w_lo;
        s_red[21] = w_hi;
        s_red[22] = w_base;
        s_red[23] = c_hi;
        s_red[24] = c2_hi;
      }
    }
    __syncthreads();
    n_act = s_red[16];
    run_lo = s_red[17];
    run_hi = s_red[18];
    tile_base = s_red[19];
    run2_lo = s_red[20];
    run2_hi = s_red[21];
    tile_base2 = s_red[22];
    cons_hi = s_red[23];
    cons2_hi = s_red[24];
  }

  const bf16_t* kbase = k_ptr + b * a.k.sb + h * a.k.sh;
  const bf16_t* vbase = v_ptr + b * a.v.sb + h * a.v.sh;
  int seg_r = 0, pre_r = 0;

  auto tile_at = [&](int i, int& segbit) -> int {
    if (GENERAL && use_list) {
      int e = s_list[i];
      segbit = (e >> 15) | (wg_one_doc ? 0 : 1);  // a tile of several ids, or queries of several
      return e & 0x7fff;
    }
    segbit = 0;
    return j_lo + i;
  };

  // ---- global -> LDS: every wave moves 8 of a tile's 64 rows with two direct-to-LDS loads.
  // A load instruction writes 64 lanes x 16 bytes to CONSECUTIVE LDS addresses, i.e. lane l
  // fills physical chunk l%CPR of row l/CPR; the XOR layout is obtained by letting that lane
  // fetch logical chunk (l%CPR) ^ f(row) from global memory instead.
  constexpr int CPR = D / 8;            // 16-byte chunks per row
  constexpr int RPI = 64 / CPR;         // rows per load instruction
  constexpr int NLD = 8 / RPI;          // load instructions per wave per tile
  unsigned k_voff[NLD], v_voff[NLD];  // per-lane byte offsets inside a group of RPI rows
  // row inside the tile and element offset of the chunk that a lane moves with instruction t
  // (recomputed where the rare partial-tile path needs them: registers are scarce here)
  auto ld_row = [&](int t) { return 8 * wave + RPI * t + lane / CPR; };
  auto ld_koff = [&](int t) {
    const int rrow = 8 * wave + RPI * t + lane / CPR;
    return ((tile_off<D>(rrow, lane % CPR) - rrow * (D * 2)) >> 4) * 8;
  };
#pragma unroll
  for (int t = 0; t < NLD; ++t) {
    const int rrow = 8 * wave + RPI * t + lane / CPR;
    const int pc = lane % CPR;
    const int lc = (tile_off<D>(rrow, pc) - rrow * (D * 2)) >> 4;  // logical chunk stored at pc
    // from the wave's first row: the second group of RPI rows (D = 128) rides on the same scalar base
    k_voff[t] = (unsigned)(((long long)(lane / CPR + RPI * t) * a.k.sl + lc * 8) * 2);
    v_voff[t] = (unsigned)(((long long)(lane / CPR + RPI * t) * a.v.sl + lc * 8) * 2);
  }
  auto issue_rows = [&](const bf16_t* base, const unsigned (&voff)[NLD], long long sl, int k0, unsigned dst) {
    if (k0 + kKeyTile <= a.Lk) {
      const bf16_t* sb = base + (long long)(k0 + 8 * wave_u) * sl;  // wave-uniform: scalar registers
      global_to_lds16_s(sb, voff[0], dst);
      if (NLD == 2) global_to_lds16_s(sb, voff[NLD - 1], dst + RPI * (D * 2));
    } else {  // last, partial tile: rows past the end repeat the last row (masked later)
#pragma unroll
      for (int t = 0; t < NLD; ++t) {
        const int gr = min(k0 + ld_row(t), a.Lk - 1);
        global_to_lds16(base + (long long)gr * sl + ld_koff(t), dst + RPI * t * (D * 2));
      }
    }
  };
  // one load instruction (RPI rows) of a tile: the loop spreads a tile's instructions over its
  // MFMA blocks, a burst of them would queue up in the CU's one vector-memory pipe and stall
  // the issuing waves
  auto issue_part = [&](const bf16_t* base, const unsigned (&voff)[NLD], long long sl, int k0, unsigned dst, int t) {
    if (k0 + kKeyTile <= a.Lk) {
      global_to_lds16_s(base + (long long)(k0 + 8 * wave_u) * sl, voff[t], dst + RPI * t * (D * 2));
    } else {
      const int gr = min(k0 + ld_row(t), a.Lk - 1);
      global_to_lds16(base + (long long)gr * sl + ld_koff(t), dst + RPI * t * (D * 2));
    }
  };
  auto issue_k = [&](int j, int buf) {
    const int k0 = j * kKeyTile;
    issue_rows(kbase, k_voff, a.k.sl, k0, RA_LDS_ADDR(&s_k[0][0]) + buf * TILE_BYTES + wave_u * 8 * (D * 2));
    if (GENERAL && lane < kKeyTile) {
      int kk = min(k0 + lane, a.Lk - 1);
      if (kv_seg) seg_r = kv_seg[kk];
      if (kv_pre) pre_r = kv_pre[kk];
    }
  };
  auto issue_v = [&](int j, int buf) {
    issue_rows(vbase, v_voff, a.v.sl, j * kKeyTile, RA_LDS_ADDR(&s_v[0][0]) + buf * TILE_BYTES + wave_u * 8 * (D * 2));
  };
  const int n = __builtin_amdgcn_readfirstlane(n_act);  // the same in every lane; now the compiler knows
  j_lo = __builtin_amdgcn_readfirstlane(j_lo);
  run_lo = __builtin_amdgcn_readfirstlane(run_lo);
  run_hi = __builtin_amdgcn_readfirstlane(min(run_hi, n));
  tile_base = __builtin_amdgcn_readfirstlane(tile_base);
  run2_lo = __builtin_amdgcn_readfirstlane(run2_lo);
  run2_hi = __builtin_amdgcn_readfirstlane(min(run2_hi, n));
  tile_base2 = __builtin_amdgcn_readfirstlane(tile_base2);
  int sb_unused;
  // part t of the request for K tile ordinal j / V tile ordinal j (nothing if the tile does not exist)
  auto request_k = [&](int j, int t) {
    if (j < n && t < NLD) {
      const int k0 = tile_at(j, sb_unused) * kKeyTile;
      issue_part(kbase, k_voff, a.k.sl, k0, RA_LDS_ADDR(&s_k[0][0]) + (j & 3) * TILE_BYTES + wave_u * 8 * (D * 2), t);
      if (GENERAL && !DEFER && t == 0 && lane < kKeyTile) {
        int kk = min(k0 + lane, a.Lk - 1);
        if (kv_seg) seg_r = kv_seg[kk];
        if (kv_pre) pre_r = kv_pre[kk];
      }
    }
  };
  // The segment ids / prefix flags of a key tile.  EVERY wave fetches and stores them (the same
  // values to the same LDS words): the waves of a workgroup enter and leave their straight-line
  // stretches at different tiles (a window's lower edge, the diagonal), a stretch moves no ids,
  // and a wave in a generic iteration must not depend on another wave being in one too.
  // the ids of K tile ordinal j, into registers (store_ids publishes them), where they do not
  // travel with the request
  auto fetch_ids = [&](int j) {
    if (j < n && lane < kKeyTile) {
      const int kk = min(tile_at(j, sb_unused) * kKeyTile + lane, a.Lk - 1);
      if (kv_seg) seg_r = kv_seg[kk];
      if (kv_pre) pre_r = kv_pre[kk];
    }
  };
  auto request_v = [&](int j, int t) {
    if (j < n && t < NLD) {
      const int k0 = tile_at(j, sb_unused) * kKeyTile;
      issue_part(vbase, v_voff, a.v.sl, k0, RA_LDS_ADDR(&s_v[0][0]) + (j & 3) * TILE_BYTES + wave_u * 8 * (D * 2), t);
    }
  };
  auto store_ids = [&](int buf) {
    if (GENERAL && lane < kKeyTile) {
      s_seg[buf][lane] = seg_r;
      s_pre[buf][lane] = pre_r;
      seg_r = pre_r = 0;  // dead until the next request: not carried around the loops
    }
  };

  // ---- main loop ----------------------------------------------------------------------------------
  // The matrix unit runs ahead of the vector ALU inside every wave: while the 16 MFMAs of
  // S(i+1) = K_{i+1} Q^T are in flight, the same wave turns S(i) into probabilities (exp2, row
  // sum, bf16 packing), and while the 16 MFMAs of O += P(i) V_i run it takes the row maximum of
  // S(i+1).  Vector instructions issued by the wave that owns the MFMA in flight slip into its
  // shadow; the second wave of the SIMD covers LDS and barrier latency.
  // LDS: K tile j, V tile j and the ids of tile j live in slot j & 3 of their four buffers.
  // Iteration i reads K_{i+1} (first half: scores of the next tile, probabilities of this one) and
  // V_i (second half: output update).  Barrier number k publishes K_{k+1} and V_k; right after it
  // every wave may request its share of K_{k+3} and V_{k+2} (it does so inside its MFMA blocks, one
  // load instruction at a time): a tile has two iterations to arrive.  Before a barrier a wave
  // waits until only the requests that follow the previous barrier are in flight.
  // Waves 0..3 take barrier i at the top of iteration i, waves 4..7 take barrier i+1 BETWEEN the
  // two halves of iteration i, so that on every SIMD one wave runs its first half (vector-ALU
  // heavy) and its bookkeeping while the other runs its second half (matrix-unit only).  After
  // barrier k the tiles K_{k+1}, V_{k-1} (late waves) and V_k are read while K_{k+2}, K_{k+3},
  // V_{k+1}, V_{k+2} land: three K and four V tiles are live.
  const bool wave_on = qw < a.Lq;
  // what barriers -3, -2, -1 would have requested
  if (n > 0) {
    issue_k(tile_at(0, sb_unused), 0);
    store_ids(0);
    issue_v(tile_at(0, sb_unused), 0);
  }
  if (n > 1) {
    issue_k(tile_at(1, sb_unused), 1);
    store_ids(1);
    issue_v(tile_at(1, sb_unused), 1);
  }
  if (n > 2) {
    issue_k(tile_at(2, sb_unused), 2);
    store_ids(2);
  }
  __builtin_amdgcn_s_waitcnt(0);  // tiles, carry and Q operands have landed
  __syncthreads();

  constexpr int PF = 3;  // LDS operand fetches kept in flight ahead of the MFMA that uses them

  // positional class of this wave's 32 x 64 rectangle of tile index i
  auto tile_class = [&](int i, int& kt0, int& segbit) -> int {
    kt0 = tile_at(i, segbit) * kKeyTile;
    if (flags & RA_BIAS_PREFIX) return 2;
    return classify_pos(flags, bs.window, q_off + qw, q_off + qw + 31, kv_off + kt0,
                        kv_off + kt0 + kKeyTile - 1);
  };
  // Per-lane LDS byte offsets of the operand fetches.  Everything that changes from one MFMA
  // to the next (tile buffer, 32-key block, 16-key step) is a multiple of 16 rows, which the
  // XOR layout leaves alone, so it folds into the instruction's immediate offset field.
  int koff[KS];
#pragma unroll
  for (int ss = 0; ss < KS; ++ss) koff[ss] = tile_off<D>(l32, 2 * ss + g);
  int voff[DB][2];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int hh2 = 0; hh2 < 2; ++hh2) {
      const int j = lane & 15;
      const int vrow = 4 * g + (j >> 2) + 8 * hh2;
      const int vcol = 32 * db + 16 * ((lane >> 4) & 1) + 4 * (j & 3);
      // The V buffers start beyond the 64 KiB that an LDS instruction's immediate offset can span:
      // their base is part of the per-lane address (made opaque, so that the compiler does not
      // fold it back into the immediate and re-add it with a vector instruction per fetch).
      unsigned va = RA_LDS_ADDR(&s_v[0][0]) + tile_off<D>(vrow, vcol >> 3) + ((vcol & 4) << 1);
      asm volatile("" : "+v"(va));
      voff[db][hh2] = (int)va;
    }
  constexpr int ROWB = D * 2;
  auto s_op_frag = [&](const char* kt, int op) {
    return *(const bf16x8*)(kt + (32 * (op & 1)) * ROWB + koff[op >> 1]);
  };
  auto pv_op_frag = [&](unsigned vt, int op) {  // vt: byte offset of the tile buffer inside s_v
    const unsigned cofs = (32 * (op / (2 * DB)) + 16 * ((op / DB) & 1)) * ROWB;
    const lds_char* p0 = (const lds_char*)(uintptr_t)((unsigned)voff[op % DB][0] + (vt + cofs));
    const lds_char* p1 = (const lds_char*)(uintptr_t)((unsigned)voff[op % DB][1] + (vt + cofs));
    bf16x4 x0 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) bf16x4*)p0);
    bf16x4 x1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) bf16x4*)p1);
    return __builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  // S = K Q^T for one tile, nothing interleaved
  auto compute_s = [&](f32x16 (&S)[2], const char* kt) {
    bf16x8 fr[2 * KS];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      S[0][r] = 0.f;
      S[1][r] = 0.f;
    }
#pragma unroll
    for (int op = 0; op < PF; ++op) fr[op] = s_op_frag(kt, op);
    // the fragments that the per-tile-term variants park in LDS are fetched from there here too:
    // they occupy no register outside the prologue
    bf16x8 qp0 = qf[0], qp1 = qf[1], qp2 = qf[2];
    if constexpr (TIGHT) qp0 = s_q0[tid];
    if constexpr (GENERAL) qp1 = s_q1[tid];
    if constexpr (PARK2) qp2 = s_q2[tid];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int op = 0; op < 2 * KS; ++op) {
      if (op + PF < 2 * KS) fr[op + PF] = s_op_frag(kt, op + PF);
      S[op & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[op], op < 2 ? qp0 : (op < 4 ? qp1 : (op < 6 ? qp2 : qf[op >> 1])), S[op & 1], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto compute_pv = [&](const bf16x8 (&pf)[4], unsigned vt) {
    bf16x8 fr[4 * DB];
#pragma unroll
    for (int op = 0; op < PF; ++op) fr[op] = pv_op_frag(vt, op);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int op = 0; op < 4 * DB; ++op) {
      if (op + PF < 4 * DB) fr[op + PF] = pv_op_frag(vt, op + PF);
      oacc[op % DB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[op], pf[op / DB], oacc[op % DB], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto raw_rowmax = [&](const f32x16 (&S)[2]) -> float {
    float mx = RA_NEG_INF;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, S[kb][r]);
    return half_max(mx) * a.scale2;  // scale2 > 0: the maximum commutes with the scaling
  };
  // terms that every tile must evaluate; a dense block with a summary is read only in the tiles
  // that the list marks (segbit)
  int tile_terms = RA_BIAS_ALIBI | RA_BIAS_PREFIX | RA_BIAS_DENSE;
  if constexpr (DENSE) {
    if (dmap != nullptr) tile_terms &= ~RA_BIAS_DENSE;
  }
  auto needs_bias = [&](int kt0, int segbit, int cls) -> bool {
    bool nb = (cls & 2) || (kt0 + kKeyTile > a.Lk);
    if (GENERAL) nb = nb || (flags & tile_terms) || segbit;
    return nb;
  };
  // Bias of a fresh tile with the id arrays of LDS slot `ids_buf`; returns the row maximum (log2
  // units).  The tile keeps the units of the matrix product: a bias value enters divided by
  // scale2, so that biased and unbiased tiles go through the same exp2(S * scale2 - m) chain.
  auto prepare = [&](f32x16 (&S)[2], int kt0, int segbit, int cls, int ids_buf) -> float {
    TileBias tb;
    tb.flags = (cls & 2) ? (flags & (RA_BIAS_CAUSAL | RA_BIAS_WINDOW)) : 0;
    if (GENERAL) {
      tb.flags |= flags & tile_terms;
      if (segbit) tb.flags |= DENSE ? (flags & (RA_BIAS_SEGMENT | RA_BIAS_DENSE)) : RA_BIAS_SEGMENT;
    }
    tb.window = bs.window;
    const float inv_scale2 = 1.0f / a.scale2;
    tb.slope2 = slope2 * inv_scale2;
    tb.dense_mul = kLog2e * inv_scale2;
    tb.dense = nullptr;
    tb.dense_vs = 1;
    tb.dense_vec = 0;
    if (DENSE) {
      const float* head = dense_ptr + b * bs.dense_sb + h * bs.dense_sh;
      tb.dense_vec = kt0 + kKeyTile <= a.Lk && ((((uintptr_t)head) | ((uintptr_t)bs.dense_sq << 2)) & 15) == 0;
    }
    float mx = RA_NEG_INF;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      const int var0 = kt0 + 32 * kb + 4 * g;
      tb.var_limit = a.Lk - var0;
      const int rel0 = (q_off + qi) - (kv_off + var0);
      if (DENSE)
        tb.dense = dense_ptr + b * bs.dense_sb + h * bs.dense_sh + (long long)min(qi, a.Lq - 1) * bs.dense_sq + var0;
      apply_bias<true, DENSE, GENERAL>(S[kb], tb, rel0, q_seg, q_pre, &s_seg[ids_buf][32 * kb + 4 * g],
                       &s_pre[ids_buf][32 * kb + 4 * g]);
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, S[kb][r]);
    }
    return half_max(mx) * a.scale2;
  };
  // move the exponent reference if some row's maximum outgrew it by more than 2^8; until then
  // probabilities are taken relative to the old reference (they stay below 256, harmless in
  // fp32 / bf16) and the 64-register rescale of O is skipped
  auto update_reference = [&](float mx) {
    m_true = fmaxf(m_true, mx);
    if (__any(mx > m_run + 8.0f)) {
      const float m_new = fmaxf(m_run, mx);
      const float m_safe_new = (m_new == RA_NEG_INF) ? 0.f : m_new;
      const float corr = fast_exp2(m_run - m_safe_new);
      m_run = m_new;
      l_run *= corr;
      lr_run *= corr;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] *= corr;
    }
  };

  // Ordinals [st_lo[s], st_hi[s]) of the tiles this wave sees completely, unmasked and in range:
  // they take the straight-line path without any per-tile classification.  Under ALiBi a stretch
  // must also lie on one side of the diagonal, where -slope |q_pos - kv_pos| is linear in both
  // positions (stretch 0: keys before the wave's queries, stretch 1: keys after them).
  // Stretches 0 and 1 lie in the first run of tiles, 2 and 3 in the second one.
  constexpr int NST = 4;
  const bool alibi_on = GENERAL && (flags & RA_BIAS_ALIBI);
  int st_lo[NST] = {0, 0, 0, 0}, st_hi[NST] = {0, 0, 0, 0};
  if (wave_on && !(GENERAL && (flags & tile_terms & (RA_BIAS_PREFIX | RA_BIAS_DENSE)))) {
    int lo, hi;  // tile indices
    key_tile_plain_range(flags, bs.window, q_off + qw, q_off + qw + 31, kv_off, a.Lk / kKeyTile,
                         kKeyTile, lo, hi);
    int lo2 = hi, hi1 = hi;
    if (alibi_on) {
      // the same bounds for all waves (the workgroup's first and last query): the waves meet at a
      // barrier per tile, so a generic iteration in one of them holds up all
      hi1 = min(hi, floor_div(q_off + q0 - kv_off - (kKeyTile - 1), kKeyTile) + 1);       // last key <= first query
      lo2 = max(lo, ceil_div(q_off + q0 + kFwdRows - 1 - kv_off, kKeyTile));              // first key >= last query
    }
    st_lo[0] = max(lo - tile_base, run_lo);
    st_hi[0] = max(min(hi1 - tile_base, run_hi), st_lo[0]);
    st_lo[1] = max(max(lo2 - tile_base, run_lo), st_hi[0]);
    st_hi[1] = max(min(hi - tile_base, run_hi), st_lo[1]);
    if (GENERAL) {
      st_lo[2] = max(max(lo - tile_base2, run2_lo), st_hi[1]);
      st_hi[2] = max(min(hi1 - tile_base2, run2_hi), st_lo[2]);
      st_lo[3] = max(max(lo2 - tile_base2, run2_lo), st_hi[2]);
      st_hi[3] = max(min(hi - tile_base2, run2_hi), st_lo[3]);
    }
  }
  if constexpr (GENERAL) {
    // The stretches of this wave wait in LDS (the loops have no scalar register to spare):
    // iteration i is plain for p_lo <= i < p_end; exact row sums, so no minimum length.
    // Iteration i requests tiles up to i + 3 by running addresses: where the list goes on they
    // must be the listed ones, behind the list's end they only have to lie inside the shard
    // (nobody reads them).
    if (lane == 0) {
#pragma unroll
      for (int st = 0; st < NST; ++st) {
        const int base = st < 2 ? tile_base : tile_base2, c_hi = st < 2 ? cons_hi : cons2_hi;
        const int list_end = c_hi >= n ? 0x3fffffff : c_hi - 3;
        s_st[wave][3 * st] = st_lo[st];
        s_st[wave][3 * st + 1] = min(min(st_hi[st] - 1, list_end), a.Lk / kKeyTile - base - 3);
        s_st[wave][3 * st + 2] = base;
      }
    }
  }
  st_lo[0] = __builtin_amdgcn_readfirstlane(st_lo[0]);  // wave-uniform; now the compiler knows
  st_hi[0] = __builtin_amdgcn_readfirstlane(st_hi[0]);

  // Barrier number k and the requests that follow it (see the loop description above).
  const bool late_half = wave_u >= 4;
  // second half of iteration i: early waves are between barriers i and i+1 and request V_{i+2},
  // late waves are between barriers i+1 and i+2 and request V_{i+3}
  const int v_ahead = late_half ? 3 : 2;
  auto sync = [&](int k) {
    // this wave's share of K_{k+1}, V_k is in LDS once only the requests of barrier k-1 (K_{k+2},
    // V_{k+1}, NLD load instructions each, where they exist) are in flight
    const int pending = (k + 2 < n ? NLD : 0) + (k + 1 < n ? NLD : 0);
    // The variants whose generic iterations issue their requests last (DEFER): an early wave
    // has, as in the plain case, those of K_{k+2} and V_{k+1} as its most recent loads (the ids of
    // the per-tile-term variants, ordinary loads, are stored before the requests go out); a late
    // wave meets this barrier in the middle of an iteration, before its requests, so its most
    // recent loads are a tile older than the count assumes: it waits for everything.
    const bool counted = !DEFER || !late_half;
    if (!counted || k == 0 || pending == 0) __builtin_amdgcn_s_waitcnt(0x0f70);
    else if (pending == NLD) __builtin_amdgcn_s_waitcnt(0x0f70 | NLD);
    else __builtin_amdgcn_s_waitcnt(0x0f70 | (2 * NLD));
    __syncthreads();
  };

  // per-tile state handed from one iteration to the next
  f32x16 sa[2], sb[2];
  bool cur_valid = false;
  float cur_mx = RA_NEG_INF;
  if (n > 0 && wave_on) {
    int kt0, segbit;
    const int cls = tile_class(0, kt0, segbit);
    if (!(cls & 1)) {
      cur_valid = true;
      compute_s(sa, s_k[0]);
      cur_mx = needs_bias(kt0, segbit, cls) ? prepare(sa, kt0, segbit, cls, 0) : raw_rowmax(sa);
    }
  }

  // one iteration; SC holds S(i) on entry, SN receives S(i+1)
  auto iteration = [&](auto parity, int i, f32x16 (&SC)[2], f32x16 (&SN)[2]) {
    constexpr int PAR = decltype(parity)::value;  // i & 3, known at compile time
    if (!late_half) sync(i);
    const char* kt = s_k[(PAR + 1) & 3];
    const unsigned vt = PAR * TILE_BYTES;
    int nkt0 = 0, nsegbit = 0, ncls = 1;
    bool nxt_valid = false, nxt_biased = false;
    if (!alibi_on && wg_one_doc && i + 1 >= st_lo[0] && i + 1 < st_hi[0]) {
      nxt_valid = true;  // inside a stretch of plain tiles (without ALiBi there is one stretch)
    } else if (i + 1 < n && wave_on) {
      ncls = tile_class(i + 1, nkt0, nsegbit);
      nxt_valid = !(ncls & 1);
      nxt_biased = nxt_valid && needs_bias(nkt0, nsegbit, ncls);
    }
    float nxt_mx = RA_NEG_INF;
    bf16x8 pfrag[4];
    const bool fused = cur_valid && nxt_valid;
    if (cur_valid) update_reference(cur_mx);
    const float neg_m = (m_run == RA_NEG_INF) ? 0.f : -m_run;
    if (fused) {
      // ---- fused path: S(i+1) MFMAs with the exp2 / sum / pack of tile i in their shadow -------
      float rs0 = 0.f, rs1 = 0.f;
      {
        bf16x8 fr[2 * KS];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          SN[0][r] = 0.f;
          SN[1][r] = 0.f;
        }
#pragma unroll
        for (int op = 0; op < PF; ++op) fr[op] = s_op_frag(kt, op);
        bf16x8 qp0 = qf[0], qp1 = qf[1], qp2 = qf[2];  // from LDS where they are parked there
        if constexpr (TIGHT) qp0 = s_q0[tid];
        if constexpr (GENERAL) qp1 = s_q1[tid];
        if constexpr (PARK2) qp2 = s_q2[tid];
        __builtin_amdgcn_sched_barrier(0);
        constexpr int EPO = 32 / (2 * KS);  // score elements converted per MFMA
#pragma unroll
        for (int op = 0; op < 2 * KS; ++op) {
          if (op + PF < 2 * KS) fr[op + PF] = s_op_frag(kt, op + PF);
          SN[op & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[op], op < 2 ? qp0 : (op < 4 ? qp1 : (op < 6 ? qp2 : qf[op >> 1])), SN[op & 1], 0, 0, 0);
          if constexpr (!DEFER) {
            if (op == (2 * KS) / 4) request_k(i + 3, 0);
            if (op == (2 * KS) * 3 / 4) request_k(i + 3, 1);
          }
#pragma unroll
          for (int e = 0; e < EPO; e += 2) {
            const int el = op * EPO + e;  // 0..31 over (kb, r)
            const int kb = el >> 4, r = el & 15;
            const float p0 = fast_exp2(fmaf(SC[kb][r], a.scale2, neg_m));
            const float p1 = fast_exp2(fmaf(SC[kb][r + 1], a.scale2, neg_m));
            rs0 += p0;
            rs1 += p1;
            bf16x2 pr;
            pr[0] = (bf16_t)p0;
            pr[1] = (bf16_t)p1;
            // pinned between the two MFMAs: without it the compiler sinks the arithmetic to the
            // first use of the packed probabilities, behind the MFMA block it is meant to hide in
            unsigned pw = __builtin_bit_cast(unsigned, pr);
            asm volatile("" : "+v"(pw));
            pr = __builtin_bit_cast(bf16x2, pw);
            lr_run = __builtin_amdgcn_fdot2_f32_bf16(pr, ones2, lr_run, false);
            asm volatile("" : "+v"(lr_run));
            pfrag[2 * kb + (r >> 3)][r & 7] = pr[0];
            pfrag[2 * kb + (r >> 3)][(r & 7) + 1] = pr[1];
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      l_run += rs0 + rs1;
      if (late_half) sync(i + 1);
      // ---- O += P(i) V_i with the row maximum of S(i+1) in the shadow ---------------------------
      {
        bf16x8 fr[4 * DB];
        float mx0 = RA_NEG_INF, mx1 = RA_NEG_INF;
#pragma unroll
        for (int op = 0; op < PF; ++op) fr[op] = pv_op_frag(vt, op);
        __builtin_amdgcn_sched_barrier(0);
        constexpr int EPO = 32 / (4 * DB);
#pragma unroll
        for (int op = 0; op < 4 * DB; ++op) {
          if (op + PF < 4 * DB) fr[op + PF] = pv_op_frag(vt, op + PF);
          oacc[op % DB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[op], pfrag[op / DB], oacc[op % DB], 0, 0, 0);
          if constexpr (!DEFER) {
            if (op == (4 * DB) / 4) request_v(i + v_ahead, 0);
            if (op == (4 * DB) * 3 / 4) request_v(i + v_ahead, 1);
          }
#pragma unroll
          for (int e = 0; e < EPO; e += 2) {
            const int el = op * EPO + e;  // one three-operand maximum per pair of scores
            float& mx = (op & 1) ? mx1 : mx0;
            mx = fmaxf(fmaxf(mx, SN[el >> 4][el & 15]), SN[el >> 4][(el & 15) + 1]);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        nxt_mx = half_max(fmaxf(mx0, mx1)) * a.scale2;
      }
    } else {
      // ---- generic path (first / last / masked / biased tiles): same work, not interleaved -----
      if constexpr (!DEFER) {
        request_k(i + 3, 0);
        request_k(i + 3, 1);
      }
      if (nxt_valid) compute_s(SN, kt);
      if (cur_valid) {
        float rs = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float p = fast_exp2(fmaf(SC[kb][r], a.scale2, neg_m));
            SC[kb][r] = p;
            rs += p;
          }
        l_run += rs;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int ks = 0; ks < 2; ++ks) {
            pfrag[2 * kb + ks] = pack8(SC[kb], 8 * ks);
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
              bf16x2 pr;
              pr[0] = pfrag[2 * kb + ks][e];
              pr[1] = pfrag[2 * kb + ks][e + 1];
              lr_run = __builtin_amdgcn_fdot2_f32_bf16(pr, ones2, lr_run, false);
            }
          }
      }
      if (late_half) sync(i + 1);
      if constexpr (!DEFER) {
        request_v(i + v_ahead, 0);
        request_v(i + v_ahead, 1);
      }
      if (cur_valid) compute_pv(pfrag, vt);
      if (nxt_valid && !nxt_biased) nxt_mx = raw_rowmax(SN);
    }
    if (nxt_biased) nxt_mx = prepare(SN, nkt0, nsegbit, ncls, (i + 1) & 3);
    if constexpr (DEFER) {
      // These variants hold part of their state in scratch memory, and a reload waits for every
      // load issued before it: a generic iteration's requests go out last, behind the ids (plain
      // loads, awaited by the store), so that nothing in it waits for them.
      fetch_ids(i + 3);
      if (i + 3 < n) store_ids((i + 3) & 3);
      request_k(i + 3, 0);
      request_k(i + 3, 1);
      request_v(i + v_ahead, 0);
      request_v(i + v_ahead, 1);
    } else {
      if (i + 3 < n) store_ids((i + 3) & 3);
    }
    cur_valid = nxt_valid;
    cur_mx = nxt_mx;
  };

  // ---- the same iteration for a stretch of plain tiles ---------------------------------------------
  // Tiles i and i+1 are seen completely, unmasked and in range by this wave, and the tiles that the
  // iteration requests (K_{i+3}; V_{i+2} for the early waves, V_{i+3} for the late ones) exist and
  // are complete: straight-line code, no classification, no flags, scalar running addresses.
  const bf16_t* k_run = kbase;
  const bf16_t* v_run = vbase;
  const unsigned k_dst0 = RA_LDS_ADDR(&s_k[0][0]) + wave_u * 8 * (D * 2);
  const unsigned v_dst0 = RA_LDS_ADDR(&s_v[0][0]) + wave_u * 8 * (D * 2);
  auto seek_plain = [&](int ordinal) {  // the iteration with this ordinal is the next to run
    k_run = kbase + (long long)((tile_base + ordinal + 3) * kKeyTile + 8 * wave_u) * a.k.sl;
    v_run = vbase + (long long)((tile_base + ordinal + v_ahead) * kKeyTile + 8 * wave_u) * a.v.sl;
  };
  auto sync_plain = [&]() {
    __builtin_amdgcn_s_waitcnt(0x0f70 | (2 * NLD));  // only the previous barrier's requests are in flight
    barrier_bare();
  };
  const bool seg_on = GENERAL && (flags & RA_BIAS_SEGMENT);
  // The key-side ids seen through the constant address space: with a wave-uniform index the
  // compiler fetches them through the scalar cache and tracks the load in flight itself (the
  // array is not written while the kernel runs).
  typedef const __attribute__((address_space(4))) int* const_ids;
  const const_ids doc_ids = (const_ids)(uintptr_t)kv_seg;
  int doc_cur = 0, doc_nxt = 0, doc_far = 0;  // segment ids of tiles i, i + 1, i + 2 of a stretch
  float ali_s = 0.f;  // see plain_iteration; set where a stretch begins (wave-uniform)
  bf16_t ali_s_hi = (bf16_t)0.f, ali_s_lo = (bf16_t)0.f;
  auto plain_iteration = [&](auto parity, int i, f32x16 (&SC)[2], f32x16 (&SN)[2]) {
    constexpr int PAR = decltype(parity)::value;
    constexpr int PF = TIGHT ? 2 : 4;  // operand fetches in flight; the TIGHT variants have no registers for more
    if (!late_half) sync_plain();
    const char* kt = s_k[(PAR + 1) & 3];
    const unsigned vt = PAR * TILE_BYTES;
    update_reference(cur_mx);
    float neg_m = -m_run;  // finite: the current tile has unmasked scores
    bool gate_nxt = true;
    if (GENERAL && seg_on) {
      // documents: tile i and tile i + 1 have one segment id each; a lane whose query row carries
      // another id takes no part in the tile - its probabilities are exp2(-inf) = 0 and its row
      // maximum is -inf.  The ids travel in scalar registers, fetched one tile ahead.
      const int my_id = s_stash[0][tid];
      neg_m = (my_id == doc_cur) ? -m_run : RA_NEG_INF;
      gate_nxt = my_id == doc_nxt;
      doc_cur = doc_nxt;
      doc_nxt = doc_far;                                                // requested one iteration ago
      doc_far = doc_ids[(long long)(tile_base + i + 3) * kKeyTile];    // tile i + 3 exists
    }
    const unsigned v_dst = v_dst0 + (late_half ? ((PAR + 3) & 3) : ((PAR + 2) & 3)) * TILE_BYTES;
    // ---- S(i+1) MFMAs, then O += P(i) V_i, with the softmax arithmetic of tile i and the row
    // maximum of S(i+1) in their shadow.  The chain of a pair of scores (scale and shift, exp2,
    // pack, exact row sum) is spread over consecutive MFMA slots, one link per slot, so that no
    // vector instruction waits for the result of the one before it and no slot carries both the
    // exp2 pair of one chain and the sum instructions of another (1.8 % of the kernel); the
    // rounded row sums wait for the end of their block (see links_of_slot); the sixteen pairs of a lane
    // are spread over both MFMA blocks so that every slot carries about the same vector work:
    // half of them (the first two operand fragments of P) in the score block, the other half in
    // the first three quarters of the output block, the row maxima in the slots that remain.
    constexpr int NOPA = 2 * KS, NOPB = 4 * DB;
    auto slot_of = [](int w) constexpr -> int {  // global slot (score block first) of pair w's exp2
      if (D == 128) return w < 8 ? 2 * w : 16 + (3 * (w - 8)) / 2;
      return w < 8 ? w : 8 + (w - 8) / 2;
    };
    auto maxima_in = [](int sb) constexpr -> int {  // row-maximum instructions in slot sb of the output block
      if (D == 128) return (sb >= 12 || sb % 3 == 2) ? 2 : 0;
      return 2;
    };
    float t[16][2], e[16][2];
    unsigned pk[16];
    u32x4 pw[4];
    auto link1 = [&](int w) {  // pair w = elements 2w, 2w+1 of the 32 scores of this lane
      const int kb = (2 * w) >> 4, r = (2 * w) & 15;
      t[w][0] = fmaf(SC[kb][r], a.scale2, neg_m);
      t[w][1] = fmaf(SC[kb][r + 1], a.scale2, neg_m);
      asm volatile("" : "+v"(t[w][0]), "+v"(t[w][1]));
    };
    auto link2 = [&](int w) {
      e[w][0] = fast_exp2(t[w][0]);
      e[w][1] = fast_exp2(t[w][1]);
      asm volatile("" : "+v"(e[w][0]), "+v"(e[w][1]));
    };
    auto link3 = [&](int w) {
      bf16x2 pr;
      pr[0] = (bf16_t)e[w][0];
      pr[1] = (bf16_t)e[w][1];
      pk[w] = __builtin_bit_cast(unsigned, pr);
      asm volatile("" : "+v"(pk[w]));
      pw[w >> 2][w & 3] = pk[w];
    };
    auto link4 = [&](int w) {
      lr_run = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pk[w]), ones2, lr_run, false);
      asm volatile("" : "+v"(lr_run));
    };
    auto link5 = [&](int w) {
      l_run += e[w][0] + e[w][1];
      asm volatile("" : "+v"(l_run));
    };
    auto links_of_slot = [&](int gs) {
#pragma unroll
      for (int w = 0; w < 16; ++w) {
        if (slot_of(w) - 1 == gs) link1(w);
        if (slot_of(w) == gs) link2(w);
        if (slot_of(w) + 1 == gs) link3(w);
        if (slot_of(w) + 3 == gs) link5(w);
      }
      // The rounded row sums go in two bursts, behind the last MFMA of either block: a dot-product
      // instruction between two MFMAs holds the matrix pipe up for 17-19 cycles, one of a burst for
      // 5-9 (a v_fma_f32 in its place: 1).
      if (gs == NOPA - 1) {
#pragma unroll
        for (int w = 0; w < 16; ++w)
          if (slot_of(w) + 1 <= NOPA - 1) link4(w);
      }
      if (gs == NOPA + NOPB - 1) {
#pragma unroll
        for (int w = 0; w < 16; ++w)
          if (slot_of(w) + 1 > NOPA - 1) link4(w);
      }
    };
    {
      bf16x8 fr[NOPA];
      if (GENERAL && alibi_on) {
        // ALiBi of tile i+1 through the matrix unit: the accumulators start from
        //   [j, j, 1, 1, 1] x [s_hi, s_lo, c_hi, c_mid, c_lo] = s j + c = -slope |q_pos - kv_pos| / scale2
        // with s = +-slope / scale2 (the sign of the stretch), j the key's index in the tile and
        // c = -s (q_pos - position of the tile's first key); s is split into two bf16 words and c
        // into three (c grows with the distance between the shards: three words carry it to fp32
        // accuracy, what an addition in the score chain would give), so that the score chain
        // below needs no instruction for the bias.
        // (recomputed per tile from the lane number: the loop has no register to carry it in)
        const int ramp_lane = tid & 63;
        const int rel_i = q_off + q0 + (tid >> 6) * 32 + (ramp_lane & 31) - (kv_off + (tile_base + i + 1) * kKeyTile);
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
        const int r0 = PARK2 ? (ramp_lane < 32 ? ramp_lane : 64) : ramp_lane;
        const int r1 = PARK2 ? (ramp_lane < 32 ? 32 + ramp_lane : 64) : 64 + ramp_lane;
        SN[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s_ramp[r0], bq, z, 0, 0, 0);
        SN[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(s_ramp[r1], bq, z, 0, 0, 0);
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          SN[0][r] = 0.f;
          SN[1][r] = 0.f;
        }
      }
#pragma unroll
      for (int op = 0; op < PF; ++op) fr[op] = s_op_frag(kt, op);
      bf16x8 q0 = qf[0];
      if (TIGHT) q0 = s_q0[tid];
      bf16x8 q1 = qf[1];
      if (GENERAL) q1 = s_q1[tid];
      bf16x8 q2 = qf[2];
      if (PARK2) q2 = s_q2[tid];
      links_of_slot(-1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int op = 0; op < NOPA; ++op) {
        if (op + PF < NOPA) fr[op + PF] = s_op_frag(kt, op + PF);
        SN[op & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[op], op < 2 ? q0 : (op < 4 ? q1 : (op < 6 ? q2 : qf[op >> 1])), SN[op & 1], 0, 0, 0);
        if (op == NOPA / 4) global_to_lds16_s(k_run, k_voff[0], k_dst0 + ((PAR + 3) & 3) * TILE_BYTES);
        if (NLD == 2 && op == NOPA * 3 / 4)
          global_to_lds16_s(k_run, k_voff[NLD - 1], k_dst0 + ((PAR + 3) & 3) * TILE_BYTES + RPI * (D * 2));
        links_of_slot(op);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    k_run += (long long)kKeyTile * a.k.sl;
    if (late_half) sync_plain();
    {
      bf16x8 fr[NOPB];
      float mx0 = RA_NEG_INF, mx1 = RA_NEG_INF;
#pragma unroll
      for (int op = 0; op < PF; ++op) fr[op] = pv_op_frag(vt, op);
      __builtin_amdgcn_sched_barrier(0);
      int el = 0;  // next pair of S(i+1) elements to enter the row maximum
#pragma unroll
      for (int op = 0; op < NOPB; ++op) {
        if (op + PF < NOPB) fr[op + PF] = pv_op_frag(vt, op + PF);
        oacc[op % DB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            fr[op], __builtin_bit_cast(bf16x8, pw[op / DB]), oacc[op % DB], 0, 0, 0);
        if (op == NOPB / 4) global_to_lds16_s(v_run, v_voff[0], v_dst);
        if (NLD == 2 && op == NOPB * 3 / 4) global_to_lds16_s(v_run, v_voff[NLD - 1], v_dst + RPI * (D * 2));
        links_of_slot(NOPA + op);
#pragma unroll
        for (int x = 0; x < maxima_in(op); ++x) {
          float& mx = (x & 1) ? mx1 : mx0;  // one three-operand maximum per pair of scores
          mx = fmaxf(fmaxf(mx, SN[el >> 4][el & 15]), SN[el >> 4][(el & 15) + 1]);
          asm volatile("" : "+v"(mx));
          el += 2;
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      cur_mx = half_max(fmaxf(mx0, mx1)) * a.scale2;
      if (GENERAL && seg_on) cur_mx = gate_nxt ? cur_mx : RA_NEG_INF;
    }
    v_run += (long long)kKeyTile * a.v.sl;
  };

  if (late_half) {
    sync(0);
    request_v(2, 0);  // what the second half of iteration -1 would have requested
    request_v(2, 1);
  }
  // The same sequence of tiles in pieces: generic iterations up to a plain stretch, the stretch in
  // whole groups of four, ... , generic iterations for the rest.  Every wave runs n iterations in
  // total, so the barrier counts agree.
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  using P2 = std::integral_constant<int, 2>;
  using P3 = std::integral_constant<int, 3>;
  int i = 0;
  if constexpr (!GENERAL) {
    // one stretch; iteration i is plain for st_lo[0] <= i < plain_end
    const int plain_end =
        __builtin_amdgcn_readfirstlane(min(min(st_hi[0] - 1, run_hi - 3), a.Lk / kKeyTile - tile_base - 3));
    for (; i < n && !(i >= st_lo[0] && i + 4 <= plain_end); i += 4) {
      iteration(P0{}, i, sa, sb);
      if (i + 1 < n) iteration(P1{}, i + 1, sb, sa);
      if (i + 2 < n) iteration(P2{}, i + 2, sa, sb);
      if (i + 3 < n) iteration(P3{}, i + 3, sb, sa);
    }
    if (i + 4 <= plain_end) {
      seek_plain(i);
      for (; i + 4 <= plain_end; i += 4) {
        plain_iteration(P0{}, i, sa, sb);
        plain_iteration(P1{}, i + 1, sb, sa);
        plain_iteration(P2{}, i + 2, sa, sb);
        plain_iteration(P3{}, i + 3, sb, sa);
      }
    }
  } else {
#pragma unroll 1
  for (int st = 0; st < NST; ++st) {
    // iteration i is plain for p_lo <= i < p_end
    const int p_lo = __builtin_amdgcn_readfirstlane(s_st[wave_u][3 * st]);
    const int p_end = __builtin_amdgcn_readfirstlane(s_st[wave_u][3 * st + 1]);
    tile_base = __builtin_amdgcn_readfirstlane(s_st[wave_u][3 * st + 2]);
    const int start = max(i, (p_lo + 3) & ~3);  // i is a multiple of four here
    if (start + 4 > p_end) continue;
    for (; i < start; i += 4) {
      iteration(P0{}, i, sa, sb);
      iteration(P1{}, i + 1, sb, sa);
      iteration(P2{}, i + 2, sa, sb);
      iteration(P3{}, i + 3, sb, sa);
    }
    seek_plain(i);
    if (GENERAL && seg_on) {
      doc_cur = doc_ids[(long long)(tile_base + i) * kKeyTile];
      doc_nxt = doc_ids[(long long)(tile_base + i + 1) * kKeyTile];
      doc_far = doc_ids[(long long)(tile_base + i + 2) * kKeyTile];
    }
    if (GENERAL && alibi_on) {
      // the first iteration of the stretch computes the scores of tile i + 1
      ali_s = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(
          __builtin_bit_cast(int, ((st & 1) ? -slope2 : slope2) / a.scale2)));  // one slope per head
      ali_s_hi = (bf16_t)ali_s;
      ali_s_lo = (bf16_t)(ali_s - (float)ali_s_hi);
    }
    // per-lane values that only the generic iterations use wait in LDS while the plain loop runs:
    // it has no register to spare
    if (GENERAL) {
      s_stash[0][tid] = q_seg;
      if (!PARK2) {
        s_stash[1][tid] = q_pre;
        s_stash[2][tid] = __float_as_int(slope2);
      }
      seg_r = pre_r = 0;  // already stored
    }
    for (; i + 4 <= p_end; i += 4) {
      plain_iteration(P0{}, i, sa, sb);
      plain_iteration(P1{}, i + 1, sb, sa);
      plain_iteration(P2{}, i + 2, sa, sb);
      plain_iteration(P3{}, i + 3, sb, sa);
    }
    if (GENERAL) {
      q_seg = s_stash[0][tid];
      if (!PARK2) {
        q_pre = s_stash[1][tid];
        slope2 = __int_as_float(s_stash[2][tid]);
      } else {
        q_pre = 0;  // a stretch implies that there is no prefix term: the flag was never loaded
        slope2 = (flags & RA_BIAS_ALIBI) ? bs.slopes[h] * kLog2e : 0.f;
      }
    }
    if (GENERAL && seg_on) {
      // the scores of tile i, which the next generic iteration turns into probabilities, came
      // out of the stretch without a mask: rows of another document drop out here
      if (q_seg != doc_cur) {
#pragma unroll
        for (int r = 0; r < 16; ++r) sa[0][r] = sa[1][r] = RA_NEG_INF;
      }
    }
    // the plain iterations requested K tiles i .. i+2 without their ids: this wave fetches them
    // for its own iterations that follow
    if (GENERAL && lane < kKeyTile) {
#pragma unroll
      for (int t = 0; t < 3; ++t) {
        if (i + t < n) {
          const int kk = min(tile_at(i + t, sb_unused) * kKeyTile + lane, a.Lk - 1);
          if (kv_seg) s_seg[(i + t) & 3][lane] = kv_seg[kk];
          if (kv_pre) s_pre[(i + t) & 3][lane] = kv_pre[kk];
        }
      }
    }
  }
  }
  for (; i < n; i += 4) {
    iteration(P0{}, i, sa, sb);
    if (i + 1 < n) iteration(P1{}, i + 1, sb, sa);
    if (i + 2 < n) iteration(P2{}, i + 2, sa, sb);
    if (i + 3 < n) iteration(P3{}, i + 3, sb, sa);
  }
  if (!late_half) sync(n);  // both halves pass the same number of barriers
  }  // key/value shards
  // A wave that gathered no probability mass (no tile listed for its workgroup, or every score
  // masked) has nothing to merge: with l_step = 0 and an unchanged maximum the merge below is the
  // identity, so the carry's 32 rows stay where they are, unread.
  if (!WHOLE && __all(l_run == 0.f && lr_run == 0.f)) return;
  if constexpr (WHOLE) {
    {
      // out = o_step / (sum of the rounded weights): the normalised average of V;
      // lse = ln 2 (m_run + log2 l_step) with the exact sum.  A row that saw no key: 0 / 0 and -inf.
      const int qi_out = q0 + wave * 32 + l32;
      row = ((long long)b * a.H + h) * a.Lq + min(qi_out, a.Lq - 1);
      const float l_step = half_sum(l_run), lr_step = half_sum(lr_run);
      const float inv = 1.0f / lr_step;
      if (q_valid) {
        const long long at = b * a.out_sb + h * a.out_sh + (long long)qi_out * a.out_sl + 4 * g;
        if (flags & kFlagWholeBf16) {
          bf16_t* op = (bf16_t*)ring.x0[blockIdx.y] + at;
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) {
              bf16x4 t;
#pragma unroll
              for (int c = 0; c < 4; ++c) t[c] = (bf16_t)(oacc[db][4 * bb + c] * inv);
              *(bf16x4*)(op + 32 * db + 8 * bb) = t;
            }
        } else {
          float* op = ring.x0[blockIdx.y] + at;
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) {
              f32x4 t;
#pragma unroll
              for (int c = 0; c < 4; ++c) t[c] = oacc[db][4 * bb + c] * inv;
              *(f32x4*)(op + 32 * db + 8 * bb) = t;
            }
        }
        if (g == 0) ring.x1[blockIdx.y][row] = (l_step > 0.f) ? (m_run + __log2f(l_step)) * kLn2 : RA_NEG_INF;
      }
      return;
    }
  }
  // ---- merge this step into the carry ---------------------------------------------------------
  // o = o_in 2^(m_in - m_out) + o_step 2^(m_run - m_out) l_step / lr_step,  l likewise with the
  // exact sum, m_out = exact maximum over carry and step.
  {
    // the row index and the incoming maximum are recomputed / reloaded: not worth two registers
    // over the whole loop
    row = ((long long)b * a.H + h) * a.Lq + min(q0 + wave * 32 + l32, a.Lq - 1);
    const float m_in = pass_m()[row] * kLog2e;
    const float l_step = half_sum(l_run), lr_step = half_sum(lr_run);
    const float m_out = m_true;  // started from m_in, so it already covers the carry
    const float m_safe = (m_out == RA_NEG_INF) ? 0.f : m_out;
    const float f_in = fast_exp2(m_in - m_safe);   // 0 for an empty carry
    float f_step = fast_exp2(m_run - m_safe);      // 1 where the reference is exact
    const float ratio = (lr_step > 0.f) ? l_step / lr_step : 1.f;
    const float l_out = pass_l()[row] * f_in + l_step * f_step;
    f_step *= ratio;
    if (q_valid) {
      float* op = pass_o() + row * D + 4 * g;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) {
          f32x4 t = *(const f32x4*)(op + 32 * db + 8 * bb);
#pragma unroll
          for (int c = 0; c < 4; ++c) t[c] = t[c] * f_in + oacc[db][4 * bb + c] * f_step;
          *(f32x4*)(op + 32 * db + 8 * bb) = t;
        }
      if (g == 0) {
        pass_m()[row] = m_out * kLn2;
        pass_l()[row] = l_out;
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// carry init and finalisation (elementwise, HBM bound)
// ------------------------------------------------------------------------------------------------
__global__ void fwd_init_kernel(float* o, float* m, float* l, long long rows, int D) {
  const long long n4 = rows * (D / 4);
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n4) ((f32x4*)o)[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
  if (i < rows) {
    m[i] = RA_NEG_INF;
    l[i] = 0.f;
  }
}

// Summary of a dense bias block [nb, nh, Lq, Lk] (the strides say where a batch / head starts):
// one byte per cell of 32 queries x 32 keys, bit 0 = some value of the cell is not -inf, bit 1 =
// some value is not 0 (elements beyond Lq / Lk count for nothing).  A wave takes 32 rows x 256
// keys, eight cells: lane l reads keys 4l .. 4l+3 of every row.  HBM bound: the block is read once.
__global__ __launch_bounds__(256) void dense_map_kernel(const float* dense, long long sb, long long sh,
                                                        long long sq, int nh, int Lq, int Lk, unsigned char* map) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ncols = (Lk + kMapCell - 1) / kMapCell, nrows = (Lq + kMapCell - 1) / kMapCell;
  const int cg = blockIdx.x * 4 + wave;  // group of eight cell columns
  const int rb = blockIdx.y, bh = blockIdx.z;
  if (cg * 8 >= ncols) return;
  const float* base = dense + (bh / nh) * sb + (bh % nh) * sh;
  const int k0 = cg * 256 + 4 * lane;
  const bool vec = k0 + 3 < Lk && ((((uintptr_t)base) | ((uintptr_t)sq << 2)) & 15) == 0;
  const int rows = min(kMapCell, Lq - rb * kMapCell);
  bool live = false, nonzero = false;
#pragma unroll 4
  for (int r = 0; r < rows; ++r) {
    const float* p = base + (long long)(rb * kMapCell + r) * sq + k0;
    float x[4] = {RA_NEG_INF, RA_NEG_INF, RA_NEG_INF, RA_NEG_INF};
    if (vec) {
      const f32x4 v = *(const f32x4*)p;
#pragma unroll
      for (int c = 0; c < 4; ++c) x[c] = v[c];
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c)
        if (k0 + c < Lk) x[c] = p[c];
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const bool in = vec || k0 + c < Lk;
      live |= in && !(x[c] == RA_NEG_INF);
      nonzero |= in && x[c] != 0.f;
    }
  }
  const unsigned long long ml = __ballot(live), mn = __ballot(nonzero);
  if (lane < 8 && cg * 8 + lane < ncols) {
    const int bits = (((ml >> (8 * lane)) & 0xffull) ? kMapLive : 0) | (((mn >> (8 * lane)) & 0xffull) ? kMapNonZero : 0);
    map[((long long)bh * nrows + rb) * ncols + cg * 8 + lane] = (unsigned char)bits;
  }
}

// The carries of n_pass query shards lie one after another ([n_pass, B, H, Lq, D]); shard p is
// written to out + p * sp.
template <typename OutT>
__global__ void fwd_finalize_kernel(const float* o, const float* m, const float* l, OutT* out, long long sp,
                                    long long sb, long long sh, long long sl, float* lse, int n_pass, int B,
                                    int H, int Lq, int D) {
  const int cpr = D / 4;
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long rows = (long long)n_pass * B * H * Lq;
  if (i >= rows * cpr) return;
  const long long row = i / cpr;
  const int c = (int)(i % cpr);
  const int li = (int)(row % Lq);
  const int h = (int)((row / Lq) % H);
  const long long bp = row / ((long long)Lq * H);
  const int b = (int)(bp % B);
  out += (bp / B) * sp;
  const float lv = l[row];
  f32x4 x = *(const f32x4*)(o + row * D + 4 * c);
  typedef __attribute__((ext_vector_type(4))) OutT out4;
  out4 y;
#pragma unroll
  for (int e = 0; e < 4; ++e) y[e] = (OutT)(x[e] / lv);
  *(out4*)(out + b * sb + h * sh + (long long)li * sl + 4 * c) = y;
  if (c == 0) lse[row] = m[row] + logf(lv);
}

}  // namespace ra

// ------------------------------------------------------------------------------------------------
// launchers (called from the C ABI translation unit)
// ------------------------------------------------------------------------------------------------
namespace ra {

// mode: 0 = causal / window terms only, 1 = any of the per-tile terms, 2 = a dense bias block too
template <bool MULTI, bool WHOLE, typename Shards>
static hipError_t launch_fwd(const FwdArgs& a, const Shards& sl, int n_pass, int D, int mode, hipStream_t stream) {
  const int nqt = (a.Lq + kFwdRows - 1) / kFwdRows;
  dim3 grid((unsigned)(a.B * a.H * nqt), (unsigned)n_pass), block(kFwdThreads);
  if (D == 128) {
    if (mode == 2) hipLaunchKernelGGL((fwd_step_kernel<128, 2, MULTI, WHOLE>), grid, block, 0, stream, a, sl);
    else if (mode == 1) hipLaunchKernelGGL((fwd_step_kernel<128, 1, MULTI, WHOLE>), grid, block, 0, stream, a, sl);
    else hipLaunchKernelGGL((fwd_step_kernel<128, 0, MULTI, WHOLE>), grid, block, 0, stream, a, sl);
  } else {
    if (mode == 2) hipLaunchKernelGGL((fwd_step_kernel<64, 2, MULTI, WHOLE>), grid, block, 0, stream, a, sl);
    else if (mode == 1) hipLaunchKernelGGL((fwd_step_kernel<64, 1, MULTI, WHOLE>), grid, block, 0, stream, a, sl);
    else hipLaunchKernelGGL((fwd_step_kernel<64, 0, MULTI, WHOLE>), grid, block, 0, stream, a, sl);
  }
  return hipGetLastError();
}

hipError_t launch_fwd_step(const FwdArgs& a, int D, int mode, hipStream_t stream) {
  return launch_fwd<false, false>(a, NoShardList{}, 1, D, mode, stream);
}

hipError_t launch_fwd_steps(const FwdArgs& a, const KvRing& ring, int D, int mode, hipStream_t stream) {
  if (a.bias.flags & kFlagWhole) return launch_fwd<true, true>(a, ring, ring.n_pass, D, mode, stream);
  return launch_fwd<true, false>(a, ring, ring.n_pass, D, mode, stream);
}

hipError_t launch_fwd_init(float* o, float* m, float* l, long long rows, int D, hipStream_t stream) {
  const long long n = rows * (D / 4);
  hipLaunchKernelGGL(fwd_init_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, o, m, l,
                     rows, D);
  return hipGetLastError();
}

hipError_t launch_dense_map(const float* dense, long long sb, long long sh, long long sq, int nb, int nh, int Lq,
                            int Lk, unsigned char* map, hipStream_t stream) {
  const int ncols = (Lk + kMapCell - 1) / kMapCell, nrows = (Lq + kMapCell - 1) / kMapCell;
  dim3 grid((unsigned)((ncols + 31) / 32), (unsigned)nrows, (unsigned)(nb * nh));
  hipLaunchKernelGGL(dense_map_kernel, grid, dim3(256), 0, stream, dense, sb, sh, sq, nh, Lq, Lk, map);
  return hipGetLastError();
}

hipError_t launch_fwd_finalize(const float* o, const float* m, const float* l, void* out, int out_f32,
                               long long sp, long long sb, long long sh, long long sl, float* lse, int n_pass,
                               int B, int H, int Lq, int D, hipStream_t stream) {
  const long long n = (long long)n_pass * B * H * Lq * (D / 4);
  dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (out_f32)
    hipLaunchKernelGGL((fwd_finalize_kernel<float>), grid, block, 0, stream, o, m, l, (float*)out, sp, sb,
                       sh, sl, lse, n_pass, B, H, Lq, D);
  else
    hipLaunchKernelGGL((fwd_finalize_kernel<bf16_t>), grid, block, 0, stream, o, m, l, (bf16_t*)out, sp,
                       sb, sh, sl, lse, n_pass, B, H, Lq, D);
  return hipGetLastError();
}

}  // namespace ra

// Backward ring step for gfx950, recomputing the probabilities from the saved logsumexp.
//
// Two kernels per step, both deterministic (no atomics):
//  * dkdv_kernel: a workgroup owns a slab of keys (its K/V operands live in registers, its
//    dK/dV accumulators too) and streams 32-query tiles of Q and dO through LDS.  Scores
//    are produced as S = Q K^T so that an accumulator lane owns one key and 16 queries:
//    P and dS are then directly the A operands of dV = P^T dO and dK = dS^T Q, whose B
//    operands come from the Q / dO tiles through the transposing LDS read.
//  * dq_kernel: a wave owns 32 queries (Q and dO operands in registers) and streams
//    64-key tiles of K and V through LDS.  Scores are produced transposed (S^T = K Q^T),
//    exactly as in the forward kernel, so dS^T is the B operand of dQ^T = K^T dS^T.
// Plus the elementwise delta = rowsum(out * dout) and the fp32 -> bf16 gradient cast.
#include "ra_launch.h"

namespace ra {

constexpr int kBwdMaxListTiles = 2048;

// ------------------------------------------------------------------------------------------------
// delta
// ------------------------------------------------------------------------------------------------
template <typename OutT, int D>
__global__ void bwd_delta_kernel(const OutT* out, long long sb, long long sh, long long sl, TensorArg dout,
                                 float* delta, int B, int H, int Lq) {
  constexpr int CPR = D / 8;           // lanes per row
  constexpr int RPB = 256 / CPR;       // rows per block
  const int tid = threadIdx.x;
  const long long row = (long long)blockIdx.x * RPB + tid / CPR;
  const int c = tid % CPR;
  const long long rows = (long long)B * H * Lq;
  float acc = 0.f;
  if (row < rows) {
    const int li = (int)(row % Lq);
    const int h = (int)((row / Lq) % H);
    const int b = (int)(row / ((long long)Lq * H));
    const OutT* op = out + b * sb + h * sh + (long long)li * sl + 8 * c;
    const bf16_t* dp = dout.ptr + b * dout.sb + h * dout.sh + (long long)li * dout.sl + 8 * c;
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

template <int D, int NKB, bool GENERAL>
__global__ __launch_bounds__(256) void dkdv_kernel(const BwdArgs a) {
  constexpr int NT = 256;
  constexpr int KS = D / 16;
  constexpr int DB = D / 32;
  constexpr int KEYS_WG = 4 * 32 * NKB;
  constexpr int TILE_BYTES = kQTile * D * 2;

  __shared__ __attribute__((aligned(16))) char s_q[2][TILE_BYTES];
  __shared__ __attribute__((aligned(16))) char s_do[2][TILE_BYTES];
  __shared__ __attribute__((aligned(16))) float s_lse[2][kQTile];
  __shared__ __attribute__((aligned(16))) float s_delta[2][kQTile];
  __shared__ __attribute__((aligned(16))) int s_seg[2][kQTile];
  __shared__ __attribute__((aligned(16))) int s_pre[2][kQTile];
  __shared__ unsigned short s_list[GENERAL ? kBwdMaxListTiles : 1];
  __shared__ unsigned char s_flag[GENERAL ? kBwdMaxListTiles : 1];
  __shared__ int s_red[12];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const int nkt = (a.Lk + KEYS_WG - 1) / KEYS_WG;
  int hh, kt;
  decode_block(blockIdx.x, a.B * a.H, nkt, hh, kt);
  kt = nkt - 1 - kt;  // under a causal mask the FIRST key slab has the most work
  const int b = hh / a.H, h = hh % a.H;
  const int k0 = kt * KEYS_WG;
  const int kw = k0 + wave * 32 * NKB;
  const BiasArgs& bs = a.bias;
  const int flags = bs.flags;

  // ---- resident key-side operands ----------------------------------------------------------
  bf16x8 kf[NKB][KS], vf[NKB][KS];
  int k_seg[NKB], k_pre[NKB];
#pragma unroll
  for (int kb = 0; kb < NKB; ++kb) {
    const int ki = min(kw + 32 * kb + l32, a.Lk - 1);
    const bf16_t* kp = a.k.ptr + b * a.k.sb + h * a.k.sh + (long long)ki * a.k.sl + 8 * g;
    const bf16_t* vp = a.v.ptr + b * a.v.sb + h * a.v.sh + (long long)ki * a.v.sl + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      kf[kb][s] = *(const bf16x8*)(kp + 16 * s);
      vf[kb][s] = *(const bf16x8*)(vp + 16 * s);
    }
    k_seg[kb] = (GENERAL && (flags & RA_BIAS_SEGMENT)) ? bs.kv_seg[b * bs.kv_seg_sb + ki] : 0;
    k_pre[kb] = (GENERAL && (flags & RA_BIAS_PREFIX)) ? bs.kv_pre[b * bs.kv_pre_sb + ki] : 0;
  }
  float slope2 = 0.f;
  if (GENERAL && (flags & RA_BIAS_ALIBI)) slope2 = bs.slopes[h] * kLog2e;
  const int* q_seg = (GENERAL && (flags & RA_BIAS_SEGMENT)) ? bs.q_seg + b * bs.q_seg_sb : nullptr;
  const int* q_pre = (GENERAL && (flags & RA_BIAS_PREFIX)) ? bs.q_pre + b * bs.q_pre_sb : nullptr;

  f32x16 dk[NKB][DB], dv[NKB][DB];
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
    for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        dk[kb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(z8, z8, z16, 0, 0, 0);
        dv[kb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(z8, z8, z16, 0, 0, 0);
      }
  }

  // ---- which query tiles does this workgroup visit -------------------------------------------
  const int ntiles = (a.Lq + kQTile - 1) / kQTile;
  const int k_hi = min(k0 + KEYS_WG, a.Lk) - 1;
  int i_lo, i_hi;
  query_tile_range(flags, bs.window, bs.kv_off + k0, bs.kv_off + k_hi, bs.q_off, ntiles, kQTile, i_lo, i_hi);
  int n_act = i_hi - i_lo;
  bool use_list = false;
  if (GENERAL && (flags & RA_BIAS_SEGMENT)) {
    use_list = true;
    int smin = 0x7fffffff, smax = (int)0x80000000;
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb)
      if (kw + 32 * kb + l32 < a.Lk) {
        smin = min(smin, k_seg[kb]);
        smax = max(smax, k_seg[kb]);
      }
    smin = wave_min(smin);
    smax = wave_max(smax);
    if (lane == 0) {
      s_red[wave] = smin;
      s_red[4 + wave] = smax;
    }
    __syncthreads();
    int kmin = s_red[0], kmax = s_red[4];
#pragma unroll
    for (int w = 1; w < 4; ++w) {
      kmin = min(kmin, s_red[w]);
      kmax = max(kmax, s_red[4 + w]);
    }
    for (int i = i_lo + tid; i < i_hi; i += NT) {
      int qmin = 0x7fffffff, qmax = (int)0x80000000;
      const int qend = min((i + 1) * kQTile, a.Lq);
      for (int qq = i * kQTile; qq < qend; ++qq) {
        int sid = q_seg[qq];
        qmin = min(qmin, sid);
        qmax = max(qmax, sid);
      }
      const bool act = !(qmax < kmin || qmin > kmax);
      const bool uniform = (kmin == kmax) && (qmin == qmax) && (kmin == qmin);
      s_flag[i - i_lo] = act ? (uniform ? 1 : 3) : 0;
    }
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
      if (lane == 0) s_red[8] = cnt;
    }
    __syncthreads();
    n_act = s_red[8];
  }

  const bf16_t* qbase = a.q.ptr + b * a.q.sb + h * a.q.sh;
  const bf16_t* dobase = a.dout.ptr + b * a.dout.sb + h * a.dout.sh;
  const float* lse_row = a.lse + ((long long)b * a.H + h) * a.Lq;
  const float* delta_row = a.delta + ((long long)b * a.H + h) * a.Lq;
  TileStage<D, kQTile, NT> qst, dost;
  float lse_r = 0.f, delta_r = 0.f;
  int seg_r = 0, pre_r = 0;

  auto tile_at = [&](int i, int& segbit) -> int {
    if (GENERAL && use_list) {
      int e = s_list[i];
      segbit = e >> 15;
      return e & 0x7fff;
    }
    segbit = 0;
    return i_lo + i;
  };
  auto issue_loads = [&](int it) {
    qst.load(qbase, a.q.sl, it * kQTile, a.Lq, tid);
    dost.load(dobase, a.dout.sl, it * kQTile, a.Lq, tid);
    if (tid < kQTile) {
      const int qq = min(it * kQTile + tid, a.Lq - 1);
      const float L = lse_row[qq];
      lse_r = (L == RA_NEG_INF) ? __builtin_inff() : L * kLog2e;  // fully masked row: P = 0
      delta_r = delta_row[qq];
      if (GENERAL && q_seg) seg_r = q_seg[qq];
      if (GENERAL && q_pre) pre_r = q_pre[qq];
    }
  };

  int sb0 = 0;
  if (n_act > 0) issue_loads(tile_at(0, sb0));

  for (int i = 0; i < n_act; ++i) {
    const int buf = i & 1;
    qst.store(s_q[buf], tid);
    dost.store(s_do[buf], tid);
    if (tid < kQTile) {
      s_lse[buf][tid] = lse_r;
      s_delta[buf][tid] = delta_r;
      if (GENERAL) {
        s_seg[buf][tid] = seg_r;
        s_pre[buf][tid] = pre_r;
      }
    }
    __syncthreads();
    int cur_segbit;
    const int it = tile_at(i, cur_segbit);
    if (i + 1 < n_act) {
      int nb;
      issue_loads(tile_at(i + 1, nb));
    }
    const int qt0 = it * kQTile;
    const int qlo = bs.q_off + qt0, qhi = qlo + kQTile - 1;
    const bool ragged = qt0 + kQTile > a.Lq;

#pragma unroll
    for (int kb = 0; kb < NKB; ++kb) {
      const int kb0 = kw + 32 * kb;
      if (kb0 >= a.Lk) continue;
      const int klo = bs.kv_off + kb0, khi = klo + 31;
      const int cls = (flags & RA_BIAS_PREFIX) ? 2 : classify_pos(flags, bs.window, qlo, qhi, klo, khi);
      if (cls & 1) continue;
      TileBias tb;
      tb.flags = (cls & 2) ? (flags & (RA_BIAS_CAUSAL | RA_BIAS_WINDOW)) : 0;
      if (GENERAL) {
        tb.flags |= flags & (RA_BIAS_ALIBI | RA_BIAS_PREFIX);
        if (cur_segbit) tb.flags |= RA_BIAS_SEGMENT;
      }
      tb.window = bs.window;
      tb.slope2 = slope2;
      tb.var_limit = a.Lq - (qt0 + 4 * g);

      // S = Q K^T and dP = dO V^T for 32 queries x 32 keys
      f32x16 sacc, pacc;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        sacc[r] = 0.f;
        pacc[r] = 0.f;
      }
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        bf16x8 qa = frag_nat<D>(s_q[buf], l32, s, g);
        sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa, kf[kb][s], sacc, 0, 0, 0);
      }
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        bf16x8 da = frag_nat<D>(s_do[buf], l32, s, g);
        pacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(da, vf[kb][s], pacc, 0, 0, 0);
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[r] *= a.scale2;
      if (tb.flags != 0 || ragged) {
        const int rel0 = (bs.q_off + qt0 + 4 * g) - (bs.kv_off + kb0 + l32);
        apply_bias<false>(sacc, tb, rel0, k_seg[kb], k_pre[kb], &s_seg[buf][4 * g], &s_pre[buf][4 * g]);
      }
      // P = exp2(t - lse2), dS = P * (dP - delta); rows of the accumulator are queries
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) {
        const f32x4 L4 = *(const f32x4*)&s_lse[buf][8 * bb + 4 * g];
        const f32x4 d4 = *(const f32x4*)&s_delta[buf][8 * bb + 4 * g];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const int r = 4 * bb + c;
          const float p = fast_exp2(sacc[r] - L4[c]);
          sacc[r] = p;
          pacc[r] = p * (pacc[r] - d4[c]);
        }
      }
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const bf16x8 pf = pack8(sacc, 8 * ks);
        const bf16x8 dsf = pack8(pacc, 8 * ks);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          bf16x8 dob = frag_tr<D>(s_do[buf], 16 * ks, 32 * db, lane);
          dv[kb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pf, dob, dv[kb][db], 0, 0, 0);
          bf16x8 qb = frag_tr<D>(s_q[buf], 16 * ks, 32 * db, lane);
          dk[kb][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(dsf, qb, dk[kb][db], 0, 0, 0);
        }
      }
    }
  }

  // ---- accumulate into the fp32 gradients owned by this key slab ------------------------------
#pragma unroll
  for (int kb = 0; kb < NKB; ++kb) {
    const int kb0 = kw + 32 * kb;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int key = kb0 + 8 * (r / 4) + 4 * g + (r % 4);
      if (key < a.Lk) {
        const long long off = (((long long)b * a.H + h) * a.Lk + key) * D + l32;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          a.dk[off + 32 * db] += dk[kb][db][r] * a.sm_scale;
          a.dv[off + 32 * db] += dv[kb][db][r];
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------
// dQ
// ------------------------------------------------------------------------------------------------
constexpr int kDqThreads = 512;
constexpr int kDqRows = 256;
constexpr int kDqKeyTile = 64;

template <int D, bool GENERAL>
__global__ __launch_bounds__(kDqThreads) void dq_kernel(const BwdArgs a) {
  constexpr int KS = D / 16;
  constexpr int DB = D / 32;
  constexpr int TILE_BYTES = kDqKeyTile * D * 2;

  __shared__ __attribute__((aligned(16))) char s_k[2][TILE_BYTES];
  __shared__ __attribute__((aligned(16))) char s_v[2][TILE_BYTES];
  __shared__ __attribute__((aligned(16))) int s_seg[2][kDqKeyTile];
  __shared__ __attribute__((aligned(16))) int s_pre[2][kDqKeyTile];
  __shared__ unsigned short s_list[GENERAL ? kBwdMaxListTiles : 1];
  __shared__ unsigned char s_flag[GENERAL ? kBwdMaxListTiles : 1];
  __shared__ int s_red[20];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
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

  bf16x8 qf[KS], dof[KS];
  {
    const bf16_t* qp = a.q.ptr + b * a.q.sb + h * a.q.sh + (long long)qi_c * a.q.sl + 8 * g;
    const bf16_t* dp = a.dout.ptr + b * a.dout.sb + h * a.dout.sh + (long long)qi_c * a.dout.sl + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      qf[s] = *(const bf16x8*)(qp + 16 * s);
      dof[s] = *(const bf16x8*)(dp + 16 * s);
    }
  }
  const long long row = ((long long)b * a.H + h) * a.Lq + qi_c;
  const float Lraw = a.lse[row];
  const float lse2 = (Lraw == RA_NEG_INF) ? __builtin_inff() : Lraw * kLog2e;
  const float delta = a.delta[row];
  f32x16 acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[db][r] = 0.f;

  int q_seg = 0, q_pre = 0;
  float slope2 = 0.f;
  if (GENERAL) {
    if (flags & RA_BIAS_SEGMENT) q_seg = bs.q_seg[b * bs.q_seg_sb + qi_c];
    if (flags & RA_BIAS_PREFIX) q_pre = bs.q_pre[b * bs.q_pre_sb + qi_c];
    if (flags & RA_BIAS_ALIBI) slope2 = bs.slopes[h] * kLog2e;
  }
  const int* kv_seg = (GENERAL && (flags & RA_BIAS_SEGMENT)) ? bs.kv_seg + b * bs.kv_seg_sb : nullptr;
  const int* kv_pre = (GENERAL && (flags & RA_BIAS_PREFIX)) ? bs.kv_pre + b * bs.kv_pre_sb : nullptr;

  const int ntiles = (a.Lk + kDqKeyTile - 1) / kDqKeyTile;
  const int q_rows_hi = min(q0 + kDqRows, a.Lq) - 1;
  int j_lo, j_hi;
  key_tile_range(flags, bs.window, bs.q_off + q0, bs.q_off + q_rows_hi, bs.kv_off, ntiles, kDqKeyTile,
                 j_lo, j_hi);
  int n_act = j_hi - j_lo;
  bool use_list = false;
  if (GENERAL && (flags & RA_BIAS_SEGMENT)) {
    use_list = true;
    int smin = q_valid ? q_seg : 0x7fffffff, smax = q_valid ? q_seg : (int)0x80000000;
    smin = wave_min(smin);
    smax = wave_max(smax);
    if (lane == 0) {
      s_red[wave] = smin;
      s_red[8 + wave] = smax;
    }
    __syncthreads();
    int qmin = s_red[0], qmax = s_red[8];
#pragma unroll
    for (int w = 1; w < 8; ++w) {
      qmin = min(qmin, s_red[w]);
      qmax = max(qmax, s_red[8 + w]);
    }
    for (int j = j_lo + tid; j < j_hi; j += kDqThreads) {
      int kmin = 0x7fffffff, kmax = (int)0x80000000;
      const int kend = min((j + 1) * kDqKeyTile, a.Lk);
      for (int kk = j * kDqKeyTile; kk < kend; ++kk) {
        int sid = kv_seg[kk];
        kmin = min(kmin, sid);
        kmax = max(kmax, sid);
      }
      const bool act = !(kmax < qmin || kmin > qmax);
      const bool uniform = (kmin == kmax) && (qmin == qmax) && (kmin == qmin);
      s_flag[j - j_lo] = act ? (uniform ? 1 : 3) : 0;
    }
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
      if (lane == 0) s_red[16] = cnt;
    }
    __syncthreads();
    n_act = s_red[16];
  }

  const bf16_t* kbase = a.k.ptr + b * a.k.sb + h * a.k.sh;
  const bf16_t* vbase = a.v.ptr + b * a.v.sb + h * a.v.sh;
  TileStage<D, kDqKeyTile, kDqThreads> kst, vst;
  int seg_r = 0, pre_r = 0;

  auto tile_at = [&](int i, int& segbit) -> int {
    if (GENERAL && use_list) {
      int e = s_list[i];
      segbit = e >> 15;
      return e & 0x7fff;
    }
    segbit = 0;
    return j_lo + i;
  };
  auto issue_loads = [&](int j) {
    kst.load(kbase, a.k.sl, j * kDqKeyTile, a.Lk, tid);
    vst.load(vbase, a.v.sl, j * kDqKeyTile, a.Lk, tid);
    if (GENERAL && tid < kDqKeyTile) {
      int kk = min(j * kDqKeyTile + tid, a.Lk - 1);
      if (kv_seg) seg_r = kv_seg[kk];
      if (kv_pre) pre_r = kv_pre[kk];
    }
  };

  int sb0 = 0;
  if (n_act > 0) issue_loads(tile_at(0, sb0));

  for (int i = 0; i < n_act; ++i) {
    const int buf = i & 1;
    kst.store(s_k[buf], tid);
    vst.store(s_v[buf], tid);
    if (GENERAL && tid < kDqKeyTile) {
      s_seg[buf][tid] = seg_r;
      s_pre[buf][tid] = pre_r;
    }
    __syncthreads();
    int cur_segbit;
    const int j = tile_at(i, cur_segbit);
    if (i + 1 < n_act) {
      int nb;
      issue_loads(tile_at(i + 1, nb));
    }
    if (qw >= a.Lq) continue;
    const int kt0 = j * kDqKeyTile;
    const int qlo = bs.q_off + qw, qhi = qlo + 31;

#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      const int kb0 = kt0 + 32 * kb;
      if (kb0 >= a.Lk) continue;
      const int klo = bs.kv_off + kb0, khi = klo + 31;
      const int cls = (flags & RA_BIAS_PREFIX) ? 2 : classify_pos(flags, bs.window, qlo, qhi, klo, khi);
      if (cls & 1) continue;
      TileBias tb;
      tb.flags = (cls & 2) ? (flags & (RA_BIAS_CAUSAL | RA_BIAS_WINDOW)) : 0;
      if (GENERAL) {
        tb.flags |= flags & (RA_BIAS_ALIBI | RA_BIAS_PREFIX);
        if (cur_segbit) tb.flags |= RA_BIAS_SEGMENT;
      }
      tb.window = bs.window;
      tb.slope2 = slope2;
      const int var0 = kb0 + 4 * g;
      tb.var_limit = a.Lk - var0;
      const bool ragged = kb0 + 32 > a.Lk;

      f32x16 sacc, pacc;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        sacc[r] = 0.f;
        pacc[r] = 0.f;
      }
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        bf16x8 ka = frag_nat<D>(s_k[buf], 32 * kb + l32, s, g);
        sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qf[s], sacc, 0, 0, 0);
      }
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        bf16x8 va = frag_nat<D>(s_v[buf], 32 * kb + l32, s, g);
        pacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, dof[s], pacc, 0, 0, 0);
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[r] *= a.scale2;
      if (tb.flags != 0 || ragged) {
        const int rel0 = (bs.q_off + qi) - (bs.kv_off + var0);
        apply_bias<true>(sacc, tb, rel0, q_seg, q_pre, &s_seg[buf][32 * kb + 4 * g],
                         &s_pre[buf][32 * kb + 4 * g]);
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float p = fast_exp2(sacc[r] - lse2);
        pacc[r] = p * (pacc[r] - delta);
      }
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const bf16x8 dsf = pack8(pacc, 8 * ks);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          bf16x8 kt = frag_tr<D>(s_k[buf], 32 * kb + 16 * ks, 32 * db, lane);
          acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kt, dsf, acc[db], 0, 0, 0);
        }
      }
    }
  }

  if (q_valid) {
    float* dq = a.dq + row * D + 4 * g;
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
// fp32 accumulator -> bf16 gradient in the caller's layout
// ------------------------------------------------------------------------------------------------
__global__ void bwd_finalize_kernel(const float* acc, bf16_t* out, long long sb, long long sh, long long sl,
                                    int B, int H, int L, int D) {
  const int cpr = D / 4;
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long rows = (long long)B * H * L;
  if (i >= rows * cpr) return;
  const long long row = i / cpr;
  const int c = (int)(i % cpr);
  const int li = (int)(row % L);
  const int h = (int)((row / L) % H);
  const int b = (int)(row / ((long long)L * H));
  f32x4 x = *(const f32x4*)(acc + row * D + 4 * c);
  bf16x4 y;
#pragma unroll
  for (int e = 0; e < 4; ++e) y[e] = (bf16_t)x[e];
  *(bf16x4*)(out + b * sb + h * sh + (long long)li * sl + 4 * c) = y;
}

// ------------------------------------------------------------------------------------------------
// launchers
// ------------------------------------------------------------------------------------------------
hipError_t launch_bwd_delta(const void* out, int out_f32, long long sb, long long sh, long long sl,
                            TensorArg dout, float* delta, int B, int H, int Lq, int D, hipStream_t stream) {
  const long long rows = (long long)B * H * Lq;
  const int rpb = 256 / (D / 8);
  dim3 grid((unsigned)((rows + rpb - 1) / rpb)), block(256);
  if (D == 128) {
    if (out_f32) hipLaunchKernelGGL((bwd_delta_kernel<float, 128>), grid, block, 0, stream, (const float*)out, sb, sh, sl, dout, delta, B, H, Lq);
    else hipLaunchKernelGGL((bwd_delta_kernel<bf16_t, 128>), grid, block, 0, stream, (const bf16_t*)out, sb, sh, sl, dout, delta, B, H, Lq);
  } else {
    if (out_f32) hipLaunchKernelGGL((bwd_delta_kernel<float, 64>), grid, block, 0, stream, (const float*)out, sb, sh, sl, dout, delta, B, H, Lq);
    else hipLaunchKernelGGL((bwd_delta_kernel<bf16_t, 64>), grid, block, 0, stream, (const bf16_t*)out, sb, sh, sl, dout, delta, B, H, Lq);
  }
  return hipGetLastError();
}

constexpr int kNkb = 1;  // 32-key blocks per wave in dkdv_kernel

hipError_t launch_bwd_step(const BwdArgs& a, int D, bool general, int parts, hipStream_t stream) {
  if (parts & 1) {
    const int keys_wg = 4 * 32 * kNkb;
    const int nkt = (a.Lk + keys_wg - 1) / keys_wg;
    dim3 grid((unsigned)(a.B * a.H * nkt)), block(256);
    if (D == 128) {
      if (general) hipLaunchKernelGGL((dkdv_kernel<128, kNkb, true>), grid, block, 0, stream, a);
      else hipLaunchKernelGGL((dkdv_kernel<128, kNkb, false>), grid, block, 0, stream, a);
    } else {
      if (general) hipLaunchKernelGGL((dkdv_kernel<64, kNkb, true>), grid, block, 0, stream, a);
      else hipLaunchKernelGGL((dkdv_kernel<64, kNkb, false>), grid, block, 0, stream, a);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  if (parts & 2) {
    const int nqt = (a.Lq + kDqRows - 1) / kDqRows;
    dim3 grid((unsigned)(a.B * a.H * nqt)), block(kDqThreads);
    if (D == 128) {
      if (general) hipLaunchKernelGGL((dq_kernel<128, true>), grid, block, 0, stream, a);
      else hipLaunchKernelGGL((dq_kernel<128, false>), grid, block, 0, stream, a);
    } else {
      if (general) hipLaunchKernelGGL((dq_kernel<64, true>), grid, block, 0, stream, a);
      else hipLaunchKernelGGL((dq_kernel<64, false>), grid, block, 0, stream, a);
    }
  }
  return hipGetLastError();
}

hipError_t launch_bwd_finalize(const float* acc, void* out, long long sb, long long sh, long long sl, int B,
                               int H, int L, int D, hipStream_t stream) {
  const long long n = (long long)B * H * L * (D / 4);
  hipLaunchKernelGGL(bwd_finalize_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, acc,
                     (bf16_t*)out, sb, sh, sl, B, H, L, D);
  return hipGetLastError();
}

}  // namespace ra

// Forward ring step for gfx950: (o, m, l) <- online-softmax update with one K/V shard.
//
// Work split: one workgroup = 8 waves = 256 query rows of one (batch, head); wave w owns 32
// rows.  K/V are streamed in 64-key tiles through LDS (double buffered).  Scores are
// produced TRANSPOSED, S^T = K Q^T, so that in the 32x32 MFMA accumulator a lane owns one
// query row (lane%32) and 16 keys: row max / row sum are in-register reductions plus one
// exchange with lane^32, the rescale of the running output is a per-lane scalar, and the
// bf16 probabilities are already laid out as the B operand of O^T = V^T P^T, whose A
// operand comes from the V tile through the transposing LDS read.
#include "ra_launch.h"

namespace ra {


constexpr int kFwdThreads = 512;
constexpr int kFwdRows = 256;   // query rows per workgroup
constexpr int kKeyTile = 64;    // keys per LDS tile
constexpr int kMaxListTiles = 1024;

template <int D, bool GENERAL>
__global__ __launch_bounds__(kFwdThreads) void fwd_step_kernel(const FwdArgs a) {
  constexpr int KS = D / 16;  // k-steps of the QK^T contraction
  constexpr int DB = D / 32;  // 32-wide blocks of the head dim
  constexpr int TILE_BYTES = kKeyTile * D * 2;

  __shared__ __attribute__((aligned(16))) char s_k[2][TILE_BYTES];
  __shared__ __attribute__((aligned(16))) char s_v[2][TILE_BYTES];
  __shared__ __attribute__((aligned(16))) int s_seg[2][kKeyTile];
  __shared__ __attribute__((aligned(16))) int s_pre[2][kKeyTile];
  __shared__ unsigned short s_list[GENERAL ? kMaxListTiles : 1];
  __shared__ unsigned char s_flag[GENERAL ? kMaxListTiles : 1];
  __shared__ int s_red[20];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
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

  // ---- per-lane query state ------------------------------------------------------------
  bf16x8 qf[KS];
  {
    const bf16_t* qp = a.q.ptr + b * a.q.sb + h * a.q.sh + (long long)qi_c * a.q.sl + 8 * g;
#pragma unroll
    for (int s = 0; s < KS; ++s) qf[s] = *(const bf16x8*)(qp + 16 * s);
  }
  const long long row = ((long long)b * a.H + h) * a.Lq + qi_c;
  float m_run = a.m[row] * kLog2e;
  float l_run = (g == 0) ? a.l[row] : 0.f;
  f32x16 oacc[DB];
  {
    const float* op = a.o + row * D + 4 * g;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) {
        f32x4 t = *(const f32x4*)(op + 32 * db + 8 * bb);
#pragma unroll
        for (int c = 0; c < 4; ++c) oacc[db][4 * bb + c] = t[c];
      }
  }
  int q_seg = 0, q_pre = 0;
  float slope2 = 0.f;
  if (GENERAL) {
    if (flags & RA_BIAS_SEGMENT) q_seg = bs.q_seg[b * bs.q_seg_sb + qi_c];
    if (flags & RA_BIAS_PREFIX) q_pre = bs.q_pre[b * bs.q_pre_sb + qi_c];
    if (flags & RA_BIAS_ALIBI) slope2 = bs.slopes[h] * kLog2e;
  }
  const int* kv_seg = (GENERAL && (flags & RA_BIAS_SEGMENT)) ? bs.kv_seg + b * bs.kv_seg_sb : nullptr;
  const int* kv_pre = (GENERAL && (flags & RA_BIAS_PREFIX)) ? bs.kv_pre + b * bs.kv_pre_sb : nullptr;

  // ---- which key tiles does this workgroup visit ------------------------------------------
  const int ntiles = (a.Lk + kKeyTile - 1) / kKeyTile;
  const int q_rows_hi = min(q0 + kFwdRows, a.Lq) - 1;
  int j_lo, j_hi;
  key_tile_range(flags, bs.window, bs.q_off + q0, bs.q_off + q_rows_hi, bs.kv_off, ntiles, kKeyTile,
                 j_lo, j_hi);
  int n_act = j_hi - j_lo;
  bool use_list = false;
  if (GENERAL && (flags & RA_BIAS_SEGMENT)) {
    // segment-id range of the workgroup's queries, then one thread per key tile decides
    // whether the id ranges can intersect (skip otherwise) and whether the tile is uniform
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
    for (int j = j_lo + tid; j < j_hi; j += kFwdThreads) {
      int kmin = 0x7fffffff, kmax = (int)0x80000000;
      const int kend = min((j + 1) * kKeyTile, a.Lk);
      for (int kk = j * kKeyTile; kk < kend; ++kk) {
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
  TileStage<D, kKeyTile, kFwdThreads> kst, vst;
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
    kst.load(kbase, a.k.sl, j * kKeyTile, a.Lk, tid);
    vst.load(vbase, a.v.sl, j * kKeyTile, a.Lk, tid);
    if (GENERAL && tid < kKeyTile) {
      int kk = min(j * kKeyTile + tid, a.Lk - 1);
      if (kv_seg) seg_r = kv_seg[kk];
      if (kv_pre) pre_r = kv_pre[kk];
    }
  };

  int segbit = 0;
  if (n_act > 0) issue_loads(tile_at(0, segbit));

  for (int i = 0; i < n_act; ++i) {
    const int buf = i & 1;
    kst.store(s_k[buf], tid);
    vst.store(s_v[buf], tid);
    if (GENERAL && tid < kKeyTile) {
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

    // ---- classify this wave's 32 x 64 rectangle ------------------------------------------
    const int kt0 = j * kKeyTile;
    const int qlo = bs.q_off + qw, qhi = qlo + 31;
    const int klo = bs.kv_off + kt0, khi = klo + kKeyTile - 1;
    const int cls = (flags & RA_BIAS_PREFIX) ? 2 : classify_pos(flags, bs.window, qlo, qhi, klo, khi);
    if ((cls & 1) || qw >= a.Lq) continue;
    TileBias tb;
    tb.flags = (cls & 2) ? (flags & (RA_BIAS_CAUSAL | RA_BIAS_WINDOW)) : 0;
    if (GENERAL) {
      tb.flags |= flags & (RA_BIAS_ALIBI | RA_BIAS_PREFIX);
      if (cur_segbit) tb.flags |= RA_BIAS_SEGMENT;
    }
    tb.window = bs.window;
    tb.slope2 = slope2;
    const bool ragged = kt0 + kKeyTile > a.Lk;
    const bool need_bias = tb.flags != 0 || ragged;

    // ---- S^T = K Q^T ---------------------------------------------------------------------
    f32x16 sacc[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[kb][r] = 0.f;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        bf16x8 kf = frag_nat<D>(s_k[buf], 32 * kb + l32, s, g);
        sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[s], sacc[kb], 0, 0, 0);
      }
    }
    // ---- scale, bias, row statistics -------------------------------------------------------
    float mx = RA_NEG_INF;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[kb][r] *= a.scale2;
      if (need_bias) {
        const int var0 = kt0 + 32 * kb + 4 * g;
        tb.var_limit = a.Lk - var0;
        const int rel0 = (bs.q_off + qi) - (bs.kv_off + var0);
        apply_bias<true>(sacc[kb], tb, rel0, q_seg, q_pre, &s_seg[buf][32 * kb + 4 * g],
                         &s_pre[buf][32 * kb + 4 * g]);
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sacc[kb][r]);
    }
    mx = half_max(mx);
    const float m_new = fmaxf(m_run, mx);
    const float m_safe = (m_new == RA_NEG_INF) ? 0.f : m_new;
    const float corr = fast_exp2(m_run - m_safe);
    m_run = m_new;
    float rs = 0.f;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float p = fast_exp2(sacc[kb][r] - m_safe);
        sacc[kb][r] = p;
        rs += p;
      }
    l_run = l_run * corr + rs;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[db][r] *= corr;
    // ---- O^T += V^T P^T -----------------------------------------------------------------
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const bf16x8 pf = pack8(sacc[kb], 8 * ks);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          bf16x8 vf = frag_tr<D>(s_v[buf], 32 * kb + 16 * ks, 32 * db, lane);
          oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf, oacc[db], 0, 0, 0);
        }
      }
  }

  // ---- write the carry back ------------------------------------------------------------------
  const float l_tot = half_sum(l_run);
  if (q_valid) {
    float* op = a.o + row * D + 4 * g;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) {
        f32x4 t;
#pragma unroll
        for (int c = 0; c < 4; ++c) t[c] = oacc[db][4 * bb + c];
        *(f32x4*)(op + 32 * db + 8 * bb) = t;
      }
    if (g == 0) {
      a.m[row] = m_run * kLn2;
      a.l[row] = l_tot;
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

template <typename OutT>
__global__ void fwd_finalize_kernel(const float* o, const float* m, const float* l, OutT* out,
                                    long long sb, long long sh, long long sl, float* lse, int B,
                                    int H, int Lq, int D) {
  const int cpr = D / 4;
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  const long long rows = (long long)B * H * Lq;
  if (i >= rows * cpr) return;
  const long long row = i / cpr;
  const int c = (int)(i % cpr);
  const int li = (int)(row % Lq);
  const int h = (int)((row / Lq) % H);
  const int b = (int)(row / ((long long)Lq * H));
  const float lv = l[row];
  f32x4 x = *(const f32x4*)(o + row * D + 4 * c);
  OutT* dst = out + b * sb + h * sh + (long long)li * sl + 4 * c;
#pragma unroll
  for (int e = 0; e < 4; ++e) dst[e] = (OutT)(x[e] / lv);
  if (c == 0) lse[row] = m[row] + logf(lv);
}

}  // namespace ra

// ------------------------------------------------------------------------------------------------
// launchers (called from the C ABI translation unit)
// ------------------------------------------------------------------------------------------------
namespace ra {

hipError_t launch_fwd_step(const FwdArgs& a, int D, bool general, hipStream_t stream) {
  const int nqt = (a.Lq + kFwdRows - 1) / kFwdRows;
  dim3 grid((unsigned)(a.B * a.H * nqt)), block(kFwdThreads);
  if (D == 128) {
    if (general) hipLaunchKernelGGL((fwd_step_kernel<128, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((fwd_step_kernel<128, false>), grid, block, 0, stream, a);
  } else {
    if (general) hipLaunchKernelGGL((fwd_step_kernel<64, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((fwd_step_kernel<64, false>), grid, block, 0, stream, a);
  }
  return hipGetLastError();
}

hipError_t launch_fwd_init(float* o, float* m, float* l, long long rows, int D, hipStream_t stream) {
  const long long n = rows * (D / 4);
  hipLaunchKernelGGL(fwd_init_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, o, m, l,
                     rows, D);
  return hipGetLastError();
}

hipError_t launch_fwd_finalize(const float* o, const float* m, const float* l, void* out, int out_f32,
                               long long sb, long long sh, long long sl, float* lse, int B, int H,
                               int Lq, int D, hipStream_t stream) {
  const long long n = (long long)B * H * Lq * (D / 4);
  dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (out_f32)
    hipLaunchKernelGGL((fwd_finalize_kernel<float>), grid, block, 0, stream, o, m, l, (float*)out, sb,
                       sh, sl, lse, B, H, Lq, D);
  else
    hipLaunchKernelGGL((fwd_finalize_kernel<bf16_t>), grid, block, 0, stream, o, m, l, (bf16_t*)out,
                       sb, sh, sl, lse, B, H, Lq, D);
  return hipGetLastError();
}

}  // namespace ra

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

  // ---- global -> LDS: every wave moves 8 of a tile's 64 rows with two direct-to-LDS loads.
  // A load instruction writes 64 lanes x 16 bytes to CONSECUTIVE LDS addresses, i.e. lane l
  // fills physical chunk l%CPR of row l/CPR; the XOR layout is obtained by letting that lane
  // fetch logical chunk (l%CPR) ^ f(row) from global memory instead.
  constexpr int CPR = D / 8;            // 16-byte chunks per row
  constexpr int RPI = 64 / CPR;         // rows per load instruction
  constexpr int NLD = 8 / RPI;          // load instructions per wave per tile
  int ld_row[NLD];
  long long ld_koff[NLD], ld_voff[NLD];
#pragma unroll
  for (int t = 0; t < NLD; ++t) {
    const int rrow = 8 * wave + RPI * t + lane / CPR;
    const int pc = lane % CPR;
    const int lc = (tile_off<D>(rrow, pc) - rrow * (D * 2)) >> 4;  // logical chunk stored at pc
    ld_row[t] = rrow;
    ld_koff[t] = lc * 8;
    ld_voff[t] = lc * 8;
  }
  auto issue_k = [&](int j, int buf) {
    const int k0 = j * kKeyTile;
#pragma unroll
    for (int t = 0; t < NLD; ++t) {
      const int gr = min(k0 + ld_row[t], a.Lk - 1);
      const bf16_t* src = kbase + (long long)gr * a.k.sl + ld_koff[t];
      global_to_lds16(src, s_k[buf] + (8 * wave + RPI * t) * (D * 2));
    }
    if (GENERAL && tid < kKeyTile) {
      int kk = min(k0 + tid, a.Lk - 1);
      if (kv_seg) seg_r = kv_seg[kk];
      if (kv_pre) pre_r = kv_pre[kk];
    }
  };
  auto issue_v = [&](int j, int buf) {
    const int k0 = j * kKeyTile;
#pragma unroll
    for (int t = 0; t < NLD; ++t) {
      const int gr = min(k0 + ld_row[t], a.Lk - 1);
      const bf16_t* src = vbase + (long long)gr * a.v.sl + ld_voff[t];
      global_to_lds16(src, s_v[buf] + (8 * wave + RPI * t) * (D * 2));
    }
  };
  // pair p = (K tile p, V tile p-1) -> LDS buffer p & 1
  const int n = n_act;
  int sb_unused;
  auto issue_pair = [&](int pidx) {
    if (pidx < n) issue_k(tile_at(pidx, sb_unused), pidx & 1);
    if (pidx >= 1 && pidx - 1 < n) issue_v(tile_at(pidx - 1, sb_unused), pidx & 1);
  };
  auto store_ids = [&](int buf) {
    if (GENERAL && tid < kKeyTile) {
      s_seg[buf][tid] = seg_r;
      s_pre[buf][tid] = pre_r;
    }
  };

  // ---- main loop: two wave groups in opposite phases -------------------------------------------
  // Waves 0-3 (group 0) and 4-7 (group 1) share the four SIMDs pairwise.  Time is cut into
  // slots separated by workgroup barriers.  In every slot one group runs a MATRIX phase (PV of
  // the previous tile, then S of the next one: 32 MFMAs fed by software-pipelined LDS reads)
  // while the other runs the VECTOR phase of the tile in between (bias, row statistics, exp2,
  // bf16 packing), so the matrix unit and the vector ALU of a SIMD work at the same time.
  // Group 0 runs matrix phase i in slot 2i and vector phase i in slot 2i+1; group 1 is one slot
  // behind.  Pair p is fetched during slots 2p-2 and 2p-1 and consumed in slots 2p and 2p+1.
  const int grp = wave >> 2;
  issue_pair(0);
  store_ids(0);
  __builtin_amdgcn_s_waitcnt(0);  // also: carry and Q operand loads have landed
  __syncthreads();

  f32x16 sacc[2];
  bf16x8 pfrag[4];
  bool s_valid = false, p_valid = false;
  float m_true = m_run;  // exact running maximum; m_run is the (possibly stale) exponent reference
  const bool wave_on = qw < a.Lq;

  constexpr int PF = 6;  // LDS operand fetches kept in flight ahead of the MFMA that uses them
  auto matrix_phase = [&](int i, int buf) {
    __builtin_amdgcn_s_setprio(2);
    const char* vt = s_v[buf];
    const char* kt = s_k[buf];
    if (p_valid) {
      // O^T += V^T P^T : op = (kb, ks, db)
      bf16x8 fr[16];
#pragma unroll
      for (int op = 0; op < PF; ++op)
        fr[op] = frag_tr<D>(vt, 32 * (op / (2 * DB)) + 16 * ((op / DB) & 1), 32 * (op % DB), lane);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int op = 0; op < 4 * DB; ++op) {
        if (op + PF < 4 * DB) {
          const int o2 = op + PF;
          fr[o2] = frag_tr<D>(vt, 32 * (o2 / (2 * DB)) + 16 * ((o2 / DB) & 1), 32 * (o2 % DB), lane);
          __builtin_amdgcn_sched_barrier(0);
        }
        oacc[op % DB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[op], pfrag[op / DB], oacc[op % DB], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      p_valid = false;
    }
    s_valid = false;
    if (i < n && wave_on) {
      int segbit_i;
      const int kt0 = tile_at(i, segbit_i) * kKeyTile;
      const int cls = (flags & RA_BIAS_PREFIX)
                          ? 2
                          : classify_pos(flags, bs.window, bs.q_off + qw, bs.q_off + qw + 31,
                                         bs.kv_off + kt0, bs.kv_off + kt0 + kKeyTile - 1);
      if (!(cls & 1)) {
        s_valid = true;
        // S^T = K Q^T : op = (ks, kb)
        bf16x8 fr[2 * KS];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          sacc[0][r] = 0.f;
          sacc[1][r] = 0.f;
        }
#pragma unroll
        for (int op = 0; op < PF; ++op) fr[op] = frag_nat<D>(kt, 32 * (op & 1) + l32, op >> 1, g);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int op = 0; op < 2 * KS; ++op) {
          if (op + PF < 2 * KS) {
            const int o2 = op + PF;
            fr[o2] = frag_nat<D>(kt, 32 * (o2 & 1) + l32, o2 >> 1, g);
            __builtin_amdgcn_sched_barrier(0);
          }
          sacc[op & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr[op], qf[op >> 1], sacc[op & 1], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    __builtin_amdgcn_s_setprio(0);
  };

  auto vector_phase = [&](int i, int buf) {
    if (!s_valid) return;
    int cur_segbit;
    const int kt0 = tile_at(i, cur_segbit) * kKeyTile;
    const int qlo = bs.q_off + qw, qhi = qlo + 31;
    const int klo = bs.kv_off + kt0, khi = klo + kKeyTile - 1;
    const int cls = (flags & RA_BIAS_PREFIX) ? 2 : classify_pos(flags, bs.window, qlo, qhi, klo, khi);
    TileBias tb;
    tb.flags = (cls & 2) ? (flags & (RA_BIAS_CAUSAL | RA_BIAS_WINDOW)) : 0;
    if (GENERAL) {
      tb.flags |= flags & (RA_BIAS_ALIBI | RA_BIAS_PREFIX);
      if (cur_segbit) tb.flags |= RA_BIAS_SEGMENT;
    }
    tb.window = bs.window;
    tb.slope2 = slope2;
    const bool need_bias = tb.flags != 0 || (kt0 + kKeyTile > a.Lk);
    float mx = RA_NEG_INF;
    if (need_bias) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[kb][r] *= a.scale2;
        const int var0 = kt0 + 32 * kb + 4 * g;
        tb.var_limit = a.Lk - var0;
        const int rel0 = (bs.q_off + qi) - (bs.kv_off + var0);
        apply_bias<true>(sacc[kb], tb, rel0, q_seg, q_pre, &s_seg[buf][32 * kb + 4 * g],
                         &s_pre[buf][32 * kb + 4 * g]);
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sacc[kb][r]);
      }
      mx = half_max(mx);
    } else {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sacc[kb][r]);
      mx = half_max(mx) * a.scale2;  // scale2 > 0: the maximum commutes with the scaling
    }
    m_true = fmaxf(m_true, mx);
    // The exponent reference only moves when some row's maximum grew by more than 2^8; until
    // then probabilities are taken relative to the old reference (they stay below 256,
    // harmless in fp32 / bf16) and the 64-register rescale of O is skipped.
    if (__any(mx > m_run + 8.0f)) {
      const float m_new = fmaxf(m_run, mx);
      const float m_safe_new = (m_new == RA_NEG_INF) ? 0.f : m_new;
      const float corr = fast_exp2(m_run - m_safe_new);
      m_run = m_new;
      l_run *= corr;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] *= corr;
    }
    const float neg_m = (m_run == RA_NEG_INF) ? 0.f : -m_run;
    float rs = 0.f;
    if (need_bias) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float p = fast_exp2(sacc[kb][r] + neg_m);
          sacc[kb][r] = p;
          rs += p;
        }
    } else {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float p = fast_exp2(fmaf(sacc[kb][r], a.scale2, neg_m));
          sacc[kb][r] = p;
          rs += p;
        }
    }
    l_run += rs;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) pfrag[2 * kb + ks] = pack8(sacc[kb], 8 * ks);
    p_valid = true;
    s_valid = false;
  };

  if (grp == 1) {  // slot 0 of group 1: nothing to compute yet, but its share of pair 1 is due
    issue_pair(1);
    __syncthreads();
  }
  for (int i = 0; i <= n; ++i) {
    const int buf = i & 1;
    // matrix phase i  (group 0: slot 2i, group 1: slot 2i+1)
    if (grp == 0) issue_pair(i + 1);
    matrix_phase(i, buf);
    if (grp == 1) __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): pair i+1 complete
    __syncthreads();
    // vector phase i  (group 0: slot 2i+1, group 1: slot 2i+2)
    if (grp == 1) issue_pair(i + 2);
    vector_phase(i, buf);
    if (grp == 0) {
      store_ids((i + 1) & 1);
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): pair i+1 complete
    }
    if (i < n || grp == 0) __syncthreads();
  }

  // bring the carry back to the exact maximum
  {
    const float m_safe = (m_true == RA_NEG_INF) ? 0.f : m_true;
    const float f = fast_exp2(m_run - m_safe);  // 1 where the reference is exact, 0 for empty rows
    if (__any(m_run != m_true)) {
      l_run *= f;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] *= f;
    }
    m_run = m_true;
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

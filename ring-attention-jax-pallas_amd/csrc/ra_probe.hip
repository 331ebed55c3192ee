// Benchmark-only library (libringattn_probe.so), not part of the block-step ABI.
// Diagnostic: the bf16 MFMA rate this GPU sustains with nothing but matrix instructions in flight.
// The published dense peak assumes the maximum clock; under a full matrix load with operands
// that toggle like real data the clock settles lower, so the rate measured here is the ceiling
// any kernel made of v_mfma_f32_32x32x16_bf16 can approach on this board.
#include "ra_common.h"

namespace ra {

__device__ __forceinline__ unsigned probe_hash(unsigned x) {
  x ^= x >> 16;
  x *= 0x85ebca6bu;
  x ^= x >> 13;
  x *= 0xc2b2ae35u;
  x ^= x >> 16;
  return x;
}

// One wave per SIMD, eight independent accumulator chains, operands fixed in registers.
// RANDOM = 1: operands uniform in [-2, 2) (different in every lane); 0: nearly constant operands.
template <int RANDOM>
__global__ __launch_bounds__(256) void mfma_rate_kernel(float* sink, int iters) {
  bf16x8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const unsigned h1 = probe_hash((threadIdx.x + blockIdx.x * 256u) * 64u + i * 8u + e), h2 = probe_hash(h1 + 12345u);
      a[i][e] = (bf16_t)(RANDOM ? ((int)(h1 & 0xffff) - 32768) / 16384.0f : 0.001f * threadIdx.x);
      b[i][e] = (bf16_t)(RANDOM ? ((int)(h2 & 0xffff) - 32768) / 16384.0f : 0.5f * e);
    }
  f32x16 acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  for (int it = 0; it < iters; it += 4) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 8; ++i)
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(i + j) & 3], b[i & 3], acc[i], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  sink[blockIdx.x * 256 + threadIdx.x] = s;
}

// ---------------------------------------------------------------------------------------------
// What fits in the shadow of an MFMA.  Every wave runs a loop of eight v_mfma_f32_32x32x16_bf16 on
// eight independent accumulators, each followed by a fixed group of other instructions (written in
// assembly, so that the sequence is exactly the one named), and reports the shader-clock cycles
// the loop took.  32 cycles per MFMA and SIMD keep the matrix pipe busy; anything above is what
// the group costs.  The operands are zero: this measures issue, not arithmetic.
#define RA_MF(n) "v_mfma_f32_32x32x16_bf16 a[" #n "], v[0:3], v[4:7], a[" #n "]\n"
#define RA_SLOTS8(X) RA_MF(0:15) X RA_MF(16:31) X RA_MF(32:47) X RA_MF(48:63) X RA_MF(64:79) X RA_MF(80:95) X RA_MF(96:111) X RA_MF(112:127) X
#define RA_F1 "v_fma_f32 v16, v24, v25, v16\n"
#define RA_F2 RA_F1 "v_fma_f32 v17, v24, v25, v17\n"
#define RA_F4 RA_F2 "v_fma_f32 v18, v24, v25, v18\nv_fma_f32 v19, v24, v25, v19\n"
#define RA_F6 RA_F4 "v_fma_f32 v20, v24, v25, v20\nv_fma_f32 v21, v24, v25, v21\n"
#define RA_F8 RA_F6 "v_fma_f32 v22, v24, v25, v22\nv_fma_f32 v23, v24, v25, v23\n"
#define RA_E2 "v_exp_f32 v32, v24\nv_exp_f32 v33, v24\n"
#define RA_E4 RA_E2 "v_exp_f32 v34, v24\nv_exp_f32 v35, v24\n"
#define RA_DOT "v_dot2c_f32_bf16 v36, v24, v25\n"
#define RA_DOT8 "v_dot2c_f32_bf16 v36, v24, v25\nv_dot2c_f32_bf16 v37, v24, v25\nv_dot2c_f32_bf16 v38, v24, v25\nv_dot2c_f32_bf16 v39, v24, v25\n" \
                "v_dot2c_f32_bf16 v40, v24, v25\nv_dot2c_f32_bf16 v41, v24, v25\nv_dot2c_f32_bf16 v42, v24, v25\nv_dot2c_f32_bf16 v43, v24, v25\n"
#define RA_R1 "ds_read_b128 v[44:47], v26\n"
#define RA_R2 RA_R1 "ds_read_b128 v[48:51], v26 offset:4096\n"
#define RA_R3 RA_R2 "ds_read_b128 v[52:55], v26 offset:8192\n"
#define RA_T2 "ds_read_b64_tr_b16 v[44:45], v26\nds_read_b64_tr_b16 v[46:47], v26 offset:4096\n"
#define RA_T3 RA_T2 "ds_read_b64_tr_b16 v[48:49], v26 offset:8192\n"
#define RA_CHAIN "v_mul_f32 v56, v24, v25\nv_exp_f32 v57, v24\nv_mul_f32 v58, v24, v25\nv_cvt_pk_bf16_f32 v59, v24, v25\n"
#define RA_WAIT "s_waitcnt lgkmcnt(4)\n"
#define RA_LOAD "s_mov_b32 m0, %5\ns_nop 0\nglobal_load_lds_dwordx4 v27, %6\n"

struct CoissueCase {
  const char* what;
};
__device__ __host__ constexpr int kCoissueCases = 19;
static const CoissueCase kCoissue[kCoissueCases] = {
    {"nothing"},
    {"4 v_fma_f32"},
    {"6 v_fma_f32"},
    {"8 v_fma_f32"},
    {"2 v_exp_f32"},
    {"4 v_exp_f32"},
    {"1 v_fma_f32"},
    {"1 v_dot2c_f32_bf16"},
    {"nothing; 8 v_dot2c_f32_bf16 in one burst behind the 8th MFMA"},
    {"2 ds_read_b128"},
    {"3 ds_read_b128"},
    {"2 ds_read_b64_tr_b16"},
    {"3 ds_read_b64_tr_b16"},
    {"s_waitcnt lgkmcnt(4), ds_read_b128, v_mul v_exp v_mul v_cvt_pk"},
    {"ds_read_b128, v_mul v_exp v_mul v_cvt_pk, s_waitcnt lgkmcnt(4)"},
    {"v_mul v_exp v_mul v_cvt_pk, ds_read_b128, s_waitcnt lgkmcnt(4)"},
    {"2 ds_read_b64_tr_b16, s_waitcnt lgkmcnt(6)"},
    {"one global_load_lds_dwordx4 (tile load of 1 KiB)"},
    {"2 ds_read_b64_tr_b16, s_waitcnt lgkmcnt(6); one tile load behind every 4th MFMA"},
};

template <int CASE>
__global__ __launch_bounds__(512) void coissue_kernel(long long* cycles, int iters, const char* src) {
  extern __shared__ char probe_lds[];
  const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const unsigned addr = (unsigned)(uintptr_t)(lds_char*)probe_lds + threadIdx.x % 64 * 16 + wave * 1024;
  const unsigned voff = threadIdx.x % 64 * 16;
  const unsigned dst = (unsigned)(uintptr_t)(lds_char*)probe_lds + 32768 + wave * 1024;
  const char* base = src + (size_t)blockIdx.x * 16384 + wave * 1024;
  long long t0, t1;
#define RA_PROBE_BEGIN                                                                               \
  "v_mov_b32 v26, %2\nv_mov_b32 v27, %4\nv_mov_b32 v24, 1.0\nv_mov_b32 v25, 0.5\n"                   \
  "v_mov_b32 v0, 0\nv_mov_b32 v1, 0\nv_mov_b32 v2, 0\nv_mov_b32 v3, 0\n"                             \
  "v_mov_b32 v4, 0\nv_mov_b32 v5, 0\nv_mov_b32 v6, 0\nv_mov_b32 v7, 0\n"                             \
  "s_mov_b32 s20, %3\ns_waitcnt vmcnt(0) lgkmcnt(0)\ns_barrier\ns_memtime %0\ns_waitcnt lgkmcnt(0)\n1:\n"
#define RA_PROBE_END                                                                                 \
  "s_sub_u32 s20, s20, 1\ns_cmp_lg_u32 s20, 0\ns_cbranch_scc1 1b\ns_nop 7\n"                         \
  "s_waitcnt vmcnt(0) lgkmcnt(0)\ns_memtime %1\ns_waitcnt lgkmcnt(0)\n"
#define RA_PROBE(BODY)                                                                               \
  asm volatile(RA_PROBE_BEGIN BODY RA_PROBE_END                                                      \
               : "=&s"(t0), "=&s"(t1) /* written while the inputs are still in use */                \
               : "v"(addr), "s"(iters), "v"(voff), "s"(dst), "s"(base)                               \
               : "memory", "s20", "m0", "v0", "v1", "v2", "v3", "v4", "v5", "v6", "v7", "v16", "v17", "v18", \
                 "v19", "v20", "v21", "v22", "v23", "v24", "v25", "v26", "v27", "v32", "v33", "v34", "v35",   \
                 "v36", "v37", "v38", "v39", "v40", "v41", "v42", "v43", "v44", "v45", "v46", "v47", "v48",   \
                 "v49", "v50", "v51", "v52", "v53", "v54", "v55", "v56", "v57", "v58", "v59", \
                 "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", "a10", "a11", "a12", \
                 "a13", "a14", "a15", "a16", "a17", "a18", "a19", "a20", "a21", "a22", "a23", "a24", \
                 "a25", "a26", "a27", "a28", "a29", "a30", "a31", "a32", "a33", "a34", "a35", "a36", \
                 "a37", "a38", "a39", "a40", "a41", "a42", "a43", "a44", "a45", "a46", "a47", "a48", \
                 "a49", "a50", "a51", "a52", "a53", "a54", "a55", "a56", "a57", "a58", "a59", "a60", \
                 "a61", "a62", "a63", "a64", "a65", "a66", "a67", "a68", "a69", "a70", "a71", "a72", \
                 "a73", "a74", "a75", "a76", "a77", "a78", "a79", "a80", "a81", "a82", "a83", "a84", \
                 "a85", "a86", "a87", "a88", "a89", "a90", "a91", "a92", "a93", "a94", "a95", "a96", \
                 "a97", "a98", "a99", "a100", "a101", "a102", "a103", "a104", "a105", "a106", "a107", \
                 "a108", "a109", "a110", "a111", "a112", "a113", "a114", "a115", "a116", "a117", \
                 "a118", "a119", "a120", "a121", "a122", "a123", "a124", "a125", "a126", "a127")
  if constexpr (CASE == 0) RA_PROBE(RA_SLOTS8(""));
  if constexpr (CASE == 1) RA_PROBE(RA_SLOTS8(RA_F4));
  if constexpr (CASE == 2) RA_PROBE(RA_SLOTS8(RA_F6));
  if constexpr (CASE == 3) RA_PROBE(RA_SLOTS8(RA_F8));
  if constexpr (CASE == 4) RA_PROBE(RA_SLOTS8(RA_E2));
  if constexpr (CASE == 5) RA_PROBE(RA_SLOTS8(RA_E4));
  if constexpr (CASE == 6) RA_PROBE(RA_SLOTS8(RA_F1));
  if constexpr (CASE == 7) RA_PROBE(RA_SLOTS8(RA_DOT));
  if constexpr (CASE == 8) RA_PROBE(RA_SLOTS8("") RA_DOT8);
  if constexpr (CASE == 9) RA_PROBE(RA_SLOTS8(RA_R2));
  if constexpr (CASE == 10) RA_PROBE(RA_SLOTS8(RA_R3));
  if constexpr (CASE == 11) RA_PROBE(RA_SLOTS8(RA_T2));
  if constexpr (CASE == 12) RA_PROBE(RA_SLOTS8(RA_T3));
  if constexpr (CASE == 13) RA_PROBE(RA_SLOTS8(RA_WAIT RA_R1 RA_CHAIN));
  if constexpr (CASE == 14) RA_PROBE(RA_SLOTS8(RA_R1 RA_CHAIN RA_WAIT));
  if constexpr (CASE == 15) RA_PROBE(RA_SLOTS8(RA_CHAIN RA_R1 RA_WAIT));
  if constexpr (CASE == 16) RA_PROBE(RA_SLOTS8(RA_T2 "s_waitcnt lgkmcnt(6)\n"));
  if constexpr (CASE == 17) RA_PROBE(RA_SLOTS8(RA_LOAD));
  if constexpr (CASE == 18)
    RA_PROBE(RA_MF(0:15) RA_T2 "s_waitcnt lgkmcnt(6)\n" RA_LOAD RA_MF(16:31) RA_T2 "s_waitcnt lgkmcnt(6)\n"
             RA_MF(32:47) RA_T2 "s_waitcnt lgkmcnt(6)\n" RA_MF(48:63) RA_T2 "s_waitcnt lgkmcnt(6)\n"
             RA_MF(64:79) RA_T2 "s_waitcnt lgkmcnt(6)\n" RA_LOAD RA_MF(80:95) RA_T2 "s_waitcnt lgkmcnt(6)\n"
             RA_MF(96:111) RA_T2 "s_waitcnt lgkmcnt(6)\n" RA_MF(112:127) RA_T2 "s_waitcnt lgkmcnt(6)\n");
  if (threadIdx.x % 64 == 0) cycles[blockIdx.x * (blockDim.x / 64) + wave] = t1 - t0;
}

template <int CASE>
hipError_t launch_coissue(long long* cycles, int blocks, int waves, int iters, const char* src, hipStream_t st) {
  constexpr int kLds = 96 * 1024;  // more than half of a compute unit's LDS: one workgroup per compute unit
  hipError_t e = hipFuncSetAttribute((const void*)coissue_kernel<CASE>, hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL((coissue_kernel<CASE>), dim3(blocks), dim3(64 * waves), kLds, st, cycles, iters, src);
  return hipGetLastError();
}

}  // namespace ra

// Launches `blocks` workgroups of four waves (one per SIMD) that each issue iters x 8 independent
// v_mfma_f32_32x32x16_bf16 and nothing else; the caller times the launch and divides
// blocks * 4 * iters * 8 * 32768 FLOP by it.  `sink` receives blocks * 256 floats.  Returns 0, -1
// for bad arguments or the HIP error code of the launch.
extern "C" int ra_probe_mfma_rate(float* sink, int blocks, int iters, int random_operands, void* stream) {
  if (!sink || blocks <= 0 || blocks > 65536 || iters <= 0 || (iters % 4)) return -1;
  hipStream_t st = (hipStream_t)stream;
  if (random_operands) hipLaunchKernelGGL((ra::mfma_rate_kernel<1>), dim3(blocks), dim3(256), 0, st, sink, iters);
  else hipLaunchKernelGGL((ra::mfma_rate_kernel<0>), dim3(blocks), dim3(256), 0, st, sink, iters);
  return (int)hipGetLastError();
}

// The co-issue probe.  ra_probe_coissue_cases() = number of cases, ra_probe_coissue_what(c) = the
// instructions that case c puts behind every MFMA.  ra_probe_coissue launches `blocks` workgroups of
// 4 (one wave per SIMD) or 8 waves (two per SIMD); every wave runs `iters` trips of eight MFMAs and
// writes the shader-clock cycles it took to cycles[block * waves + wave].  `src` is any readable
// device buffer of blocks * 16 KiB (the tile-load cases read it).  Returns 0, -1 for bad
// arguments or the HIP error code of the launch.
extern "C" int ra_probe_coissue_cases(void) { return ra::kCoissueCases; }
extern "C" const char* ra_probe_coissue_what(int c) { return (c >= 0 && c < ra::kCoissueCases) ? ra::kCoissue[c].what : ""; }
extern "C" int ra_probe_coissue(long long* cycles, int c, int waves, int blocks, int iters, const void* src, void* stream) {
  if (!cycles || !src || c < 0 || c >= ra::kCoissueCases || (waves != 4 && waves != 8) || blocks <= 0 || blocks > 65536 || iters <= 0)
    return -1;
  hipStream_t st = (hipStream_t)stream;
  const char* s = (const char*)src;
  switch (c) {
#define RA_CASE(n) case n: return (int)ra::launch_coissue<n>(cycles, blocks, waves, iters, s, st);
    RA_CASE(0) RA_CASE(1) RA_CASE(2) RA_CASE(3) RA_CASE(4) RA_CASE(5) RA_CASE(6) RA_CASE(7) RA_CASE(8) RA_CASE(9)
    RA_CASE(10) RA_CASE(11) RA_CASE(12) RA_CASE(13) RA_CASE(14) RA_CASE(15) RA_CASE(16) RA_CASE(17) RA_CASE(18)
#undef RA_CASE
  }
  return -1;
}

// Kernel argument blocks and host launchers shared between the kernel translation units
// and the C ABI.
#pragma once
#include "ra_common.h"

namespace ra {

// Whole-ring launches (every step of a pass in one launch, several-shard kernels only) are marked
// by one of these bits in BiasArgs::flags, next to the RA_BIAS_* bits.  Forward: the carry starts
// empty and never touches memory; the pass's x0 / x1 table entries are its slice of the attention
// output (bf16 or fp32) and its logsumexp rows.  Backward: the gradient of the resident shard is
// complete when its workgroup ends and is stored as bf16 where the pass's accumulator entries
// point, instead of being added to fp32 accumulators.  The strides of those results (in
// elements) travel in the argument slots of the pointers that such a launch does not use, so
// that the argument block does not grow: the kernels' scalar registers are all taken.
constexpr int kFlagWholeBf16 = 1 << 24;
constexpr int kFlagWholeF32 = 1 << 25;
constexpr int kFlagWhole = kFlagWholeBf16 | kFlagWholeF32;

struct FwdArgs {
  TensorArg q, k, v;
  union { float* o; long long out_sb; };
  union { float* m; long long out_sh; };
  union { float* l; long long out_sl; };
  int B, H, Lq, Lk;
  float scale2;  // sm_scale * log2(e)
  BiasArgs bias;
};

struct BwdArgs {
  TensorArg q, k, v, dout;
  const float* lse;
  const float* delta;
  union { float* dq; long long out_sb; };
  union { float* dk; long long out_sh; };
  union { float* dv; long long out_sl; };
  int B, H, Lq, Lk;
  float scale2;    // sm_scale * log2(e) = scale_p2 * scale_res
  float scale_p2;  // the power of two below scale2: folded into a bf16 operand without rounding
  float scale_res; // scale2 / scale_p2 in [1, 2): applied to the fp32 scores
  float sm_scale;
  BiasArgs bias;
};

// Per-shard arguments of a launch that walks several shards: the key/value side of consecutive
// ring steps of one query shard (forward, dQ) ...
constexpr int kMaxShards = 16;
struct KvShardList {
  int n;
  int kv_off[kMaxShards];
  const bf16_t* k[kMaxShards];
  const bf16_t* v[kMaxShards];
  const int* kv_seg[kMaxShards];
  const int* kv_pre[kMaxShards];
  const float* dense[kMaxShards];
};
// ... or the query side of the steps that one key/value shard takes part in (dK/dV).
struct QShardList {
  int n;
  int q_off[kMaxShards];
  const bf16_t* q[kMaxShards];
  const bf16_t* dout[kMaxShards];
  const float* lse[kMaxShards];
  const float* delta[kMaxShards];
  const int* q_seg[kMaxShards];
  const int* q_pre[kMaxShards];
  const float* dense[kMaxShards];
};
struct NoShardList {};

// A launch that covers several ring PASSES at once (grid dimension y = pass): every pass is the
// trip of one resident shard around the ring, i.e. what one multi-step launch walks.  The
// travelling shards come from one shared table; a pass lists the entries it meets, in ring order
// (steps that are masked entirely are left out by the host).  The resident side of a pass - for
// the forward and dQ kernels a query shard with its carry or dq accumulator, for the dK/dV kernel
// a key/value shard with its dk / dv - replaces the corresponding fields of FwdArgs / BwdArgs.
constexpr int kMaxPasses = 16;
struct KvRing {
  KvShardList kv;  // the key/value shards the passes draw from
  int n_pass;
  unsigned char count[kMaxPasses];              // live steps of pass p
  unsigned char order[kMaxPasses][kMaxShards];  // their entries of `kv`, in ring order
  int q_off[kMaxPasses];
  const bf16_t* q[kMaxPasses];
  const bf16_t* dout[kMaxPasses];  // dQ only
  float* x0[kMaxPasses];           // forward: o carry;  dQ: dq accumulator
  float* x1[kMaxPasses];           // forward: m;        dQ: lse
  float* x2[kMaxPasses];           // forward: l;        dQ: delta
  const int* q_seg[kMaxPasses];
  const int* q_pre[kMaxPasses];
};
struct QRing {
  QShardList q;  // the query shards the passes draw from
  int n_pass;
  unsigned char count[kMaxPasses];
  unsigned char order[kMaxPasses][kMaxShards];
  int kv_off[kMaxPasses];
  const bf16_t* k[kMaxPasses];
  const bf16_t* v[kMaxPasses];
  float* dk[kMaxPasses];
  float* dv[kMaxPasses];
  const int* kv_seg[kMaxPasses];
  const int* kv_pre[kMaxPasses];
};

hipError_t launch_fwd_step(const FwdArgs& a, int D, int mode, hipStream_t stream);
hipError_t launch_fwd_steps(const FwdArgs& a, const KvRing& ring, int D, int mode, hipStream_t stream);
hipError_t launch_fwd_init(float* o, float* m, float* l, long long rows, int D, hipStream_t stream);
hipError_t launch_dense_map(const float* dense, long long sb, long long sh, long long sq, int nb, int nh, int Lq,
                            int Lk, unsigned char* map, hipStream_t stream);
hipError_t launch_fwd_finalize(const float* o, const float* m, const float* l, void* out, int out_f32,
                               long long sp, long long sb, long long sh, long long sl, float* lse, int n_pass,
                               int B, int H, int Lq, int D, hipStream_t stream);
hipError_t launch_bwd_delta(const void* out, int out_f32, long long sp, long long sb, long long sh, long long sl,
                            TensorArg dout, long long dsp, float* delta, int n_pass, int B, int H, int Lq, int D,
                            hipStream_t stream);
hipError_t launch_bwd_step(const BwdArgs& a, int D, int mode, int parts, hipStream_t stream);
hipError_t launch_bwd_dq_steps(const BwdArgs& a, const KvRing& ring, int D, int mode, hipStream_t stream);
hipError_t launch_bwd_dkdv_steps(const BwdArgs& a, const QRing& ring, int D, int mode, hipStream_t stream);
hipError_t launch_bwd_finalize(const float* acc, void* out, long long sp, long long sb, long long sh, long long sl,
                               int n_pass, int B, int H, int L, int D, hipStream_t stream);

}  // namespace ra

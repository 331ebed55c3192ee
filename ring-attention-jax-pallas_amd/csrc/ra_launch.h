// Kernel argument blocks and host launchers shared between the kernel translation units
// and the C ABI.
#pragma once
#include "ra_common.h"

namespace ra {

struct FwdArgs {
  TensorArg q, k, v;
  float* o;
  float* m;
  float* l;
  int B, H, Lq, Lk;
  float scale2;  // sm_scale * log2(e)
  BiasArgs bias;
};

struct BwdArgs {
  TensorArg q, k, v, dout;
  const float* lse;
  const float* delta;
  float* dq;
  float* dk;
  float* dv;
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

hipError_t launch_fwd_step(const FwdArgs& a, int D, int mode, hipStream_t stream);
hipError_t launch_fwd_steps(const FwdArgs& a, const KvShardList& shards, int D, int mode, hipStream_t stream);
hipError_t launch_fwd_init(float* o, float* m, float* l, long long rows, int D, hipStream_t stream);
hipError_t launch_fwd_finalize(const float* o, const float* m, const float* l, void* out, int out_f32,
                               long long sb, long long sh, long long sl, float* lse, int B, int H,
                               int Lq, int D, hipStream_t stream);
hipError_t launch_bwd_delta(const void* out, int out_f32, long long sb, long long sh, long long sl,
                            TensorArg dout, float* delta, int B, int H, int Lq, int D,
                            hipStream_t stream);
hipError_t launch_bwd_step(const BwdArgs& a, int D, int mode, int parts, hipStream_t stream);
hipError_t launch_bwd_dq_steps(const BwdArgs& a, const KvShardList& shards, int D, int mode, hipStream_t stream);
hipError_t launch_bwd_dkdv_steps(const BwdArgs& a, const QShardList& shards, int D, int mode, hipStream_t stream);
hipError_t launch_bwd_finalize(const float* acc, void* out, long long sb, long long sh, long long sl,
                               int B, int H, int L, int D, hipStream_t stream);

}  // namespace ra

/*
 * ring_attention_hip.h - C ABI of the MI355X (gfx950) ring-attention block-step library.
 *
 * The library replaces the per-device block step that the reference's ring_attention runs
 * at every ring rotation, plus the carry initialisation / finalisation around it.  Every
 * entry point below names the reference interface it stands in for (paths are relative to
 * the reference checkout, package ring_attention/).  The reference has no C/FFI layer of
 * its own: its plug point is the pair of Python callables selected by `block_impl`
 * (ring.py:296-312), so these are the functions an FFI binding for that plug point binds.
 *
 * Conventions
 *  - plain C types only; all pointers are DEVICE pointers unless stated otherwise;
 *  - the caller owns every buffer; no entry point allocates or frees device memory;
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream); work is
 *    enqueued asynchronously on it and the call returns without synchronising;
 *  - return value: RA_OK (0) or a negative RA_ERR_* code; argument validation happens
 *    before any HIP call, so invalid arguments are rejected without touching a GPU;
 *    ra_last_error() returns a thread-local description of the last failure;
 *  - q/k/v/do/out tensors are bf16 with the head dimension contiguous; the batch, head and
 *    length strides are given in ELEMENTS, so both the public [b, l, h, d] layout
 *    (ring.py:80-82) and the internal [b, h, l, d] layout (ring.py:96-98) are accepted
 *    without a transpose;
 *  - carries and accumulators are fp32 and contiguous: o/dq/dk/dv [B, H, L, D],
 *    m/l/lse/delta [B, H, L];
 *  - prefix masks are read as booleans: any non-zero value marks a prefix token;
 *  - D must be 64 or 128 and equal for q, k and v; lengths may be any positive number.
 *
 * Limits against the reference's call surface (RA_ERR_HEAD_DIM / RA_ERR_SHAPE / RA_ERR_BIAS):
 *  - one head dim for q, k and v: dk != dv is not supported.  The reference's fused kernels assume
 *    dk == dv as well (ring_kernel.py:170,175 index o with dim_k); only its "jax" block functions
 *    (ring.py:58-76,140-157) take a different dv.
 *  - D in {64, 128} at this boundary; a host pads smaller head dims with zero columns (exact: zero
 *    columns add nothing to a dot product).  Head dims above 128 are not supported.
 *  - operands are bf16 (fp32 accumulation, fp32 carries, statistics and accumulators): a host
 *    holding fp32 or fp16 arrays rounds them on entry.  The reference computes in the dtype of
 *    its inputs (fp32 in its tests, ring_test.py:70-72).
 *  - token positions (q_offset / kv_offset + index) lie in [0, RA_MAX_POSITION); shards hold at
 *    most 2^24 tokens, RA_MAX_SEGMENT_SHARD under a segment bias.
 *  - row strides (ra_tensor.stride_l) lie in [D, RA_MAX_ROW_STRIDE] elements: rows do not overlap, and the
 *    rows one wavefront moves stay within a 32-bit byte offset of each other.
 */
#ifndef RING_ATTENTION_HIP_H
#define RING_ATTENTION_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RA_OK 0
#define RA_ERR_NULL (-1)        /* a required pointer is NULL                       */
#define RA_ERR_SHAPE (-2)       /* a dimension is not positive / too large          */
#define RA_ERR_HEAD_DIM (-3)    /* D is not 64 or 128                               */
#define RA_ERR_ALIGN (-4)       /* pointer or stride breaks the 16-byte row rule    */
#define RA_ERR_BIAS (-5)        /* inconsistent bias description                    */
#define RA_ERR_HIP (-6)         /* a HIP runtime call failed (see ra_last_error)    */
#define RA_ERR_DTYPE (-7)       /* unknown output dtype code                        */
#define RA_ERR_TOO_LARGE (-8)   /* a whole-ring launch cannot hold these passes     */

/* Bias terms, OR-ed into ra_bias.flags.  They are the device-side form of the reference's
 * bias_fn (ring.py:107,186): each term is evaluated per score tile from token positions
 * and per-token ids instead of being materialised as a dense [b, h, lq, lk] block. */
#define RA_BIAS_CAUSAL 1   /* kv_pos <= q_pos                  (ring.py:393-397)            */
#define RA_BIAS_WINDOW 2   /* |q_pos - kv_pos| < window (one-sided when CAUSAL is set)    */
#define RA_BIAS_SEGMENT 4  /* q_segment_id == kv_segment_id    (ring.py:388-391)            */
#define RA_BIAS_PREFIX 8   /* (q_prefix & kv_prefix) | kv_pos <= q_pos (ring.py:399-406)    */
#define RA_BIAS_ALIBI 16   /* additive -slope[h] * |q_pos - kv_pos|                       */
#define RA_BIAS_DENSE 32   /* additive fp32 block, the array a bias_fn returns (ring.py:107) */
/* With RA_BIAS_SEGMENT one call takes shards of at most this many tokens (the kernels sort a
 * shard's tiles by id range into a list of that capacity); RA_ERR_SHAPE beyond.  A longer shard
 * is walked as several shorter ones: the block step is associative over key/value shards and
 * independent over query rows (ring.py:58-76). */
#define RA_MAX_SEGMENT_SHARD 65536
/* Token positions (offset + index) must stay below this; RA_ERR_BIAS beyond.  A window wider than
 * any position difference (>= 2^30) masks nothing and is treated as 2^30. */
#define RA_MAX_POSITION ((1 << 30) - (1 << 16))
/* ra_tensor.stride_l lies in [D, RA_MAX_ROW_STRIDE] elements; RA_ERR_SHAPE beyond. */
#define RA_MAX_ROW_STRIDE (1 << 27)

#define RA_DTYPE_BF16 0
#define RA_DTYPE_F32 1

/* bf16 tensor view [B, H, L, D] with explicit element strides (D contiguous; strides multiples of 8,
 * D <= stride_l <= 2^27). */
typedef struct ra_tensor {
  const void* ptr;
  int64_t stride_b;
  int64_t stride_h;
  int64_t stride_l;
} ra_tensor;

/* Bias description for one (query shard, key/value shard) pair.
 * Positions are implicit: token i of the query shard has position q_offset + i, token j
 * of the key/value shard has position kv_offset + j (the shard's place in the ring).
 * Per-token arrays are int32 [B, L] with a batch stride in elements; the kv-side arrays
 * travel with the key/value shard, the q-side arrays with the query shard, exactly as
 * bias_kv_kwargs / bias_q_kwargs rotate in the reference (ring.py:120,195). */
typedef struct ra_bias {
  int32_t flags;
  int32_t window;
  int64_t q_offset;
  int64_t kv_offset;
  const int32_t* q_segment_ids;
  const int32_t* kv_segment_ids;
  int64_t q_segment_stride_b;
  int64_t kv_segment_stride_b;
  const int32_t* q_prefix;
  const int32_t* kv_prefix;
  int64_t q_prefix_stride_b;
  int64_t kv_prefix_stride_b;
  const float* alibi_slopes; /* [H] */
  /* RA_BIAS_DENSE: the materialised bias of this (query shard, key/value shard) pair, exactly
   * the `bias` argument of the reference's fwd_block / bwd_block (ring_kernel.py:127,206):
   * fp32, element [b, h, i, j] at dense_bias[b*stride_b + h*stride_h + i*stride_q + j], added to
   * the scaled scores (-inf masks).  stride_b / stride_h may be 0: that broadcasts the block
   * over the batch / the heads, the reference's [b, 1, lq, lk] form.  It combines with the
   * other terms by addition.  No gradient is produced for it (ring.py:243 returns None). */
  const float* dense_bias;
  int64_t dense_stride_b, dense_stride_h, dense_stride_q;
  /* Optional (NULL: none) with RA_BIAS_DENSE: the block's summary as written by ra_dense_map().
   * The reference hands its kernels the whole block and they read all of it
   * (ring_kernel.py:75-85); the blocks a bias_fn returns are mostly masks (ring_test.py:226-246:
   * 0 or -inf), so ra_fwd_step / ra_bwd_step take the summary to leave out the tiles whose part of
   * the block is -inf throughout (they contribute exp(-inf) = 0, exactly) and to read the block
   * only in tiles that hold a value other than 0.  Results are those without a summary.  It must
   * describe this block (same strides and shape); the several-step entry points evaluate the
   * whole block and do not read it.  Shards of at most RA_MAX_SEGMENT_SHARD tokens. */
  const uint8_t* dense_map;
} ra_bias;

/* One ring step of the forward pass. */
typedef struct ra_fwd_step_params {
  int32_t B, H, Lq, Lk, D;
  float sm_scale;
  ra_tensor q, k, v;
  float* o; /* [B,H,Lq,D] unnormalised output carry, updated in place */
  float* m; /* [B,H,Lq]   running row maximum of the biased, scaled scores */
  float* l; /* [B,H,Lq]   running row sum of exp(score - m) */
  ra_bias bias;
} ra_fwd_step_params;

/* One ring step of the backward pass. */
typedef struct ra_bwd_step_params {
  int32_t B, H, Lq, Lk, D;
  float sm_scale;
  ra_tensor q, k, v, dout;
  const float* lse;   /* [B,H,Lq] m + log(l) of the whole forward pass */
  const float* delta; /* [B,H,Lq] from ra_bwd_delta */
  float* dq;          /* [B,H,Lq,D] accumulated in place (owned by the query shard)    */
  float* dk;          /* [B,H,Lk,D] accumulated in place (owned by the key/value shard) */
  float* dv;          /* [B,H,Lk,D] accumulated in place */
  ra_bias bias;
} ra_bwd_step_params;

/* Version of this ABI (major * 1000 + minor). */
int ra_version(void);
/* Thread-local text for the last error returned on this thread ("" if none). */
const char* ra_last_error(void);

/* Carry initialisation o = 0, l = 0, m = -inf.          Replaces ring.py:124-126. */
int ra_fwd_init(float* o, float* m, float* l, int32_t B, int32_t H, int32_t Lq, int32_t D,
                void* stream);

/* (o, m, l) <- online-softmax update with one key/value shard.
 * Replaces fwd_block (ring_kernel.py:123-199) / _fwd_block (ring.py:58-76) together with
 * the bias_fn call in front of it (ring.py:107).  Fully masked score tiles are skipped. */
int ra_fwd_step(const ra_fwd_step_params* p, void* stream);

/* out = o / l (bf16 or fp32, strided like q), lse = m + log(l).   Replaces ring.py:134-135
 * and the output transpose ring.py:137.  out_dtype is RA_DTYPE_BF16 or RA_DTYPE_F32. */
int ra_fwd_finalize(const float* o, const float* m, const float* l, void* out,
                    int32_t out_dtype, int64_t out_stride_b, int64_t out_stride_h,
                    int64_t out_stride_l, float* lse, int32_t B, int32_t H, int32_t Lq,
                    int32_t D, void* stream);

/* delta = rowsum(out * dout) in fp32.   Replaces _precompute_delta (ring_kernel.py:387-409)
 * / the inline form ring.py:151.  `out` may be bf16 or fp32 (out_dtype), dout is bf16. */
int ra_bwd_delta(const void* out, int32_t out_dtype, int64_t out_stride_b,
                 int64_t out_stride_h, int64_t out_stride_l, const ra_tensor* dout,
                 float* delta, int32_t B, int32_t H, int32_t Lq, int32_t D, void* stream);

/* dq, dk, dv += gradients of one (query shard, key/value shard) pair, recomputed from the
 * saved logsumexp.  Replaces bwd_block (ring_kernel.py:202-297) / _bwd_block
 * (ring.py:140-157) and the accumulation ring.py:191-193. */
int ra_bwd_step(const ra_bwd_step_params* p, void* stream);

/* ra_bwd_step restricted to a subset of its kernels: parts is a bit mask, 1 = the dK/dV
 * kernel (the q-loop of ring_kernel.py:343-367), 2 = the dQ kernel (the dq product that the
 * reference adds atomically, ring_kernel.py:369-374).  parts = 3 is ra_bwd_step.  Lets a
 * caller time or schedule the two halves separately. */
int ra_bwd_step_parts(const ra_bwd_step_params* p, int32_t parts, void* stream);

/* Cast an fp32 accumulator [B,H,L,D] to a strided bf16 tensor (the final dq/dk/dv in the
 * caller's layout).   Replaces the output transposes ring.py:208-210. */
int ra_bwd_finalize(const float* acc, void* out, int64_t out_stride_b, int64_t out_stride_h,
                    int64_t out_stride_l, int32_t B, int32_t H, int32_t L, int32_t D,
                    void* stream);

/* Several ring steps in ONE launch.  steps[0 .. n_steps) are the parameter blocks that the
 * caller would hand to ra_fwd_step / ra_bwd_step one after another, in that order; the result
 * is the same up to the rounding of fp32 sums.  What runs differently: the kernel walks the
 * shards itself and keeps its running state (the forward step's output and softmax statistics,
 * dQ, or dK and dV) in registers between them, so the carry or gradient accumulator is read and
 * written once per launch instead of once per step, and small shards cost one launch instead
 * of one per step.  It is the loop of the reference around its block functions
 * (ring.py:104-132 forward, ring.py:183-206 backward) for callers that hold several shards in
 * memory at once - an emulated ring on one GPU, or a ring whose next shards have already
 * arrived.  Steps whose scores are all masked (ra_step_is_skippable) are dropped; more than 16
 * remaining steps are split into several launches.
 *  - ra_fwd_steps and ra_bwd_dq_steps: one query shard against several key/value shards.  The
 *    blocks must agree in everything but k.ptr, v.ptr, bias.kv_offset, bias.kv_segment_ids,
 *    bias.kv_prefix and bias.dense_bias (and, for the backward, dk and dv, which are not
 *    touched): RA_ERR_SHAPE otherwise.  ra_bwd_dq_steps accumulates dq only.
 *  - ra_bwd_dkdv_steps: one key/value shard against several query shards (the query side is
 *    what travels in the reference's backward ring, ring.py:195).  The blocks must agree in
 *    everything but q.ptr, dout.ptr, lse, delta, dq (not touched), bias.q_offset,
 *    bias.q_segment_ids, bias.q_prefix and bias.dense_bias.  Accumulates dk and dv only. */
int ra_fwd_steps(const ra_fwd_step_params* steps, int32_t n_steps, void* stream);
int ra_bwd_dq_steps(const ra_bwd_step_params* steps, int32_t n_steps, void* stream);
int ra_bwd_dkdv_steps(const ra_bwd_step_params* steps, int32_t n_steps, void* stream);

/* Several ring PASSES in one launch.  A pass is what ra_fwd_steps / ra_bwd_dq_steps /
 * ra_bwd_dkdv_steps take: the steps of one resident shard's whole trip around the ring.  `steps`
 * holds the passes one after another, pass p being the next steps_per_pass[p] blocks; the result
 * is that of calling the *_steps entry point once per pass.  Passes are independent of each other
 * (different query shards with their own carries or dq accumulators, or different key/value
 * shards with their own dk / dv), so one grid runs them side by side: this is the loop nest of an
 * emulated ring - all devices of ring.py:104-132 (forward) or ring.py:183-206 (backward) at once -
 * for shards so small that one pass cannot fill the GPU.  Within a pass the blocks must agree as
 * for *_steps; across passes they must share shape, strides, sm_scale and the bias terms (flags,
 * window, id strides, slopes).  One launch covers at most 16 passes that draw from at most 16
 * distinct travelling shards with at most 16 live steps each and no dense bias block; anything
 * beyond that is issued pass by pass, with the same result. */
int ra_fwd_passes(const ra_fwd_step_params* steps, const int32_t* steps_per_pass, int32_t n_passes,
                  void* stream);
int ra_bwd_dq_passes(const ra_bwd_step_params* steps, const int32_t* steps_per_pass, int32_t n_passes,
                     void* stream);
int ra_bwd_dkdv_passes(const ra_bwd_step_params* steps, const int32_t* steps_per_pass, int32_t n_passes,
                       void* stream);

/* The WHOLE ring in one launch with nothing in between.  `steps` / `steps_per_pass` as for the
 * *_passes entry points, but every pass holds ALL the blocks of its resident shard (at least one;
 * blocks that a positional mask rules out may be listed, they are skipped), so a workgroup
 * finishes its rows inside the launch and no intermediate state goes through memory:
 *  - ra_fwd_ring = zero carry (ra_fwd_init) + ra_fwd_passes + ra_fwd_finalize_passes: the carry
 *    (ring.py:104-132) stays in registers, `out` (bf16 or fp32, pass p at p * out_stride_pass
 *    elements, strides in elements) and `lse` ([n_passes, B, H, Lq] fp32) receive what
 *    ring.py:134-137 returns.  The o / m / l fields of the blocks are not used.
 *  - ra_bwd_dq_ring / ra_bwd_dkdv_ring = zeroed accumulators + ra_bwd_*_passes +
 *    ra_bwd_finalize_passes: dq (per query shard), dk and dv (per key/value shard, same strides)
 *    are stored as bf16 (ring.py:208-210).  The dq / dk / dv fields of the blocks are not used.
 * Result pointers must be aligned to four elements and the strides multiples of four.  Results
 * agree with the split entry points to rounding (the final division is folded differently), not
 * bit for bit.  RA_ERR_TOO_LARGE, with nothing launched, when one launch cannot hold the passes
 * (more than 16 passes, more than 16 distinct travelling shards): use the split entry points. */
int ra_fwd_ring(const ra_fwd_step_params* steps, const int32_t* steps_per_pass, int32_t n_passes, void* out,
                int32_t out_dtype, int64_t out_stride_pass, int64_t out_stride_b, int64_t out_stride_h,
                int64_t out_stride_l, float* lse, void* stream);
int ra_bwd_dq_ring(const ra_bwd_step_params* steps, const int32_t* steps_per_pass, int32_t n_passes, void* dq,
                   int64_t stride_pass, int64_t stride_b, int64_t stride_h, int64_t stride_l, void* stream);
int ra_bwd_dkdv_ring(const ra_bwd_step_params* steps, const int32_t* steps_per_pass, int32_t n_passes, void* dk,
                     void* dv, int64_t stride_pass, int64_t stride_b, int64_t stride_h, int64_t stride_l,
                     void* stream);

/* The elementwise entry points for the shards of n_passes passes in one launch: the fp32 arrays of
 * the passes (carries, accumulators, lse, delta) lie one after another ([n_passes, B, H, L, ...]),
 * pass p reads / writes its strided tensor at an offset of p * stride_pass elements.  With
 * n_passes = 1 they are ra_fwd_finalize (ring.py:134-135,137), ra_bwd_delta
 * (ring_kernel.py:387-409) and ra_bwd_finalize (ring.py:208-210). */
int ra_fwd_finalize_passes(const float* o, const float* m, const float* l, void* out, int32_t out_dtype,
                           int64_t out_stride_pass, int64_t out_stride_b, int64_t out_stride_h,
                           int64_t out_stride_l, float* lse, int32_t n_passes, int32_t B, int32_t H,
                           int32_t Lq, int32_t D, void* stream);
int ra_bwd_delta_passes(const void* out, int32_t out_dtype, int64_t out_stride_pass, int64_t out_stride_b,
                        int64_t out_stride_h, int64_t out_stride_l, const ra_tensor* dout,
                        int64_t dout_stride_pass, float* delta, int32_t n_passes, int32_t B, int32_t H,
                        int32_t Lq, int32_t D, void* stream);
int ra_bwd_finalize_passes(const float* acc, void* out, int64_t out_stride_pass, int64_t out_stride_b,
                           int64_t out_stride_h, int64_t out_stride_l, int32_t n_passes, int32_t B,
                           int32_t H, int32_t L, int32_t D, void* stream);

/* Summary of a dense bias block for ra_bias.dense_map: one byte per cell of 32 queries x 32 keys,
 * bit 0 = the cell holds a value other than -inf, bit 1 = it holds a value other than 0;
 * map[nb, nh, ceil(Lq/32), ceil(Lk/32)] with nb = B (1 if stride_b is 0) and nh = H (1 if
 * stride_h is 0), ra_dense_map_bytes() bytes.  One pass over the block (HBM bound), to be run
 * once per block that a bias_fn returns (ring.py:107,186: the reference calls bias_fn once per
 * ring step in the forward and once more in the backward loop); the forward step and both halves
 * of the backward step of the pair then share it.  B, H, Lq, Lk and the strides are those of the
 * step the block belongs to. */
int64_t ra_dense_map_bytes(int64_t stride_b, int64_t stride_h, int32_t B, int32_t H, int32_t Lq, int32_t Lk);
int ra_dense_map(const float* dense_bias, int64_t stride_b, int64_t stride_h, int64_t stride_q, int32_t B,
                 int32_t H, int32_t Lq, int32_t Lk, uint8_t* map, void* stream);

/* Host-only, pure: 1 if every score of the (query shard, key/value shard) pair is masked
 * by the positional terms of `bias` (CAUSAL / WINDOW), so that the whole ring step is an
 * identity on the carry and may be skipped; 0 otherwise.  The reference runs such steps and
 * lets its -inf guards nullify them (ring.py:66,69). */
int ra_step_is_skippable(const ra_bias* bias, int32_t Lq, int32_t Lk);

/* Argument checks of ra_fwd_step / ra_bwd_step without launching anything (host only). */
int ra_fwd_step_check(const ra_fwd_step_params* p);
int ra_bwd_step_check(const ra_bwd_step_params* p);

#ifdef __cplusplus
}
#endif
#endif /* RING_ATTENTION_HIP_H */

// XLA FFI handlers over the C ABI of libringattn_hip.so (include/ring_attention_hip.h): the
// translation unit that lets the reference's Python keep its own call surface under JAX.  The plug
// point is the pair of block functions that ring_attention selects by `block_impl`
// (reference ring.py:296-312): fwd_block_fn(q, k, v, bias, o, m, l, sm_scale) -> (o, m, l)
// (ring.py:109-118) and bwd_block_fn(q, k, v, bias, o, L, do, sm_scale) -> (dq, dk, dv)
// (ring.py:190).  A `block_impl == "hip"` branch binds them to the handlers below through
// jax.ffi.ffi_call; the scan, the ppermute rotation and the custom_vjp of the reference stay as
// they are.
//
// Compiled only where the XLA FFI headers exist (they ship inside jaxlib: jax.ffi.include_dir());
// build.py skips this file otherwise and says so.  Nothing else in the library depends on it.
//
// Conventions of every handler
//  - arrays arrive in XLA's dense row-major layout with the reference's internal axis order
//    [b, h, l, d] (ring.py:96-98): strides are derived from the dimensions;
//  - an optional array (segment ids, prefix masks, ALiBi slopes, a dense bias block) is absent when
//    its buffer has zero elements, and its flag in `bias_flags` must then be clear;
//  - the carries (o, m, l) and the gradient accumulators (dq, dk, dv) are operands AND results: the
//    caller aliases them (input_output_aliases in ffi_call) and the kernels update them in place; if
//    XLA hands over distinct buffers the operand is copied into the result first, on the same stream;
//  - errors of the C ABI come back as ffi::Error with the library's own text (ra_last_error).
#include <cstdint>
#include <string>

#include <hip/hip_runtime.h>

#include "xla/ffi/api/ffi.h"

#include "../../include/ring_attention_hip.h"

namespace ffi = xla::ffi;

namespace {

using Bf16Buf = ffi::Buffer<ffi::BF16>;
using F32Buf = ffi::Buffer<ffi::F32>;
using S32Buf = ffi::Buffer<ffi::S32>;
using F32Res = ffi::Result<ffi::Buffer<ffi::F32>>;

ffi::Error Fail(const char* fn, int code) {
  return ffi::Error::InvalidArgument(std::string(fn) + " failed with code " + std::to_string(code) + ": " +
                                     ra_last_error());
}

// [b, h, l, d] dense row-major -> ra_tensor (element strides)
template <typename Buf>
bool View4(const Buf& t, ra_tensor* out, int64_t dims[4]) {
  auto d = t.dimensions();
  if (d.size() != 4) return false;
  for (int i = 0; i < 4; ++i) dims[i] = d[i];
  out->ptr = t.untyped_data();
  out->stride_l = d[3];
  out->stride_h = d[2] * d[3];
  out->stride_b = d[1] * d[2] * d[3];
  return true;
}

// In-place contract: result buffers alias their operands; a distinct buffer gets a copy first.
ffi::Error Carry(hipStream_t stream, const void* operand, void* result, size_t bytes) {
  if (operand == result || bytes == 0) return ffi::Error::Success();
  if (hipMemcpyAsync(result, operand, bytes, hipMemcpyDeviceToDevice, stream) != hipSuccess)
    return ffi::Error::Internal("hipMemcpyAsync of a carry operand into its result buffer failed");
  return ffi::Error::Success();
}

// The bias description of one (query shard, key/value shard) pair: the device-side form of the
// bias_fn call in front of each block step (ring.py:107,186).
ffi::Error FillBias(ra_bias* b, int32_t flags, int32_t window, int64_t q_offset, int64_t kv_offset,
                    const S32Buf& q_seg, const S32Buf& kv_seg, const S32Buf& q_prefix, const S32Buf& kv_prefix,
                    const F32Buf& slopes, const F32Buf& dense, int64_t B, int64_t H, int64_t Lq, int64_t Lk) {
  *b = ra_bias{};
  b->flags = flags;
  b->window = window;
  b->q_offset = q_offset;
  b->kv_offset = kv_offset;
  auto ids = [&](const S32Buf& t, int64_t L, const int32_t** p, int64_t* sb, int bit, const char* name) -> ffi::Error {
    if (t.element_count() == 0) {
      if (flags & bit) return ffi::Error::InvalidArgument(std::string(name) + " is empty but its bias term is set");
      return ffi::Error::Success();
    }
    auto d = t.dimensions();
    if (d.size() != 2 || d[0] != B || d[1] != L)
      return ffi::Error::InvalidArgument(std::string(name) + " must be int32 [b, l]");
    *p = t.typed_data();
    *sb = d[1];
    return ffi::Error::Success();
  };
  if (auto e = ids(q_seg, Lq, &b->q_segment_ids, &b->q_segment_stride_b, RA_BIAS_SEGMENT, "q_segment_ids"); e.failure()) return e;
  if (auto e = ids(kv_seg, Lk, &b->kv_segment_ids, &b->kv_segment_stride_b, RA_BIAS_SEGMENT, "kv_segment_ids"); e.failure()) return e;
  if (auto e = ids(q_prefix, Lq, &b->q_prefix, &b->q_prefix_stride_b, RA_BIAS_PREFIX, "q_prefix_mask"); e.failure()) return e;
  if (auto e = ids(kv_prefix, Lk, &b->kv_prefix, &b->kv_prefix_stride_b, RA_BIAS_PREFIX, "kv_prefix_mask"); e.failure()) return e;
  if (slopes.element_count() != 0) {
    if (slopes.element_count() != (size_t)H) return ffi::Error::InvalidArgument("alibi_slopes must be float32 [h]");
    b->alibi_slopes = slopes.typed_data();
  } else if (flags & RA_BIAS_ALIBI) {
    return ffi::Error::InvalidArgument("alibi_slopes is empty but RA_BIAS_ALIBI is set");
  }
  if (dense.element_count() != 0) {
    // the array a bias_fn returns: [b, h | 1, lq, lk] (ring.py:107; head broadcast as in ring.py:409)
    auto d = dense.dimensions();
    if (d.size() != 4 || (d[0] != B && d[0] != 1) || (d[1] != H && d[1] != 1) || d[2] != Lq || d[3] != Lk)
      return ffi::Error::InvalidArgument("the dense bias must be float32 [b | 1, h | 1, lq, lk]");
    b->flags |= RA_BIAS_DENSE;
    b->dense_bias = dense.typed_data();
    b->dense_stride_q = Lk;
    b->dense_stride_h = d[1] == 1 ? 0 : Lq * Lk;
    b->dense_stride_b = d[0] == 1 ? 0 : d[1] * Lq * Lk;
  } else if (flags & RA_BIAS_DENSE) {
    return ffi::Error::InvalidArgument("the dense bias is empty but RA_BIAS_DENSE is set");
  }
  return ffi::Error::Success();
}

// ---- fwd_block (ring_kernel.py:123-199 / ring.py:58-76): (o, m, l) <- one ring step -------------
ffi::Error FwdStepImpl(hipStream_t stream, Bf16Buf q, Bf16Buf k, Bf16Buf v, F32Buf o_in, F32Buf m_in, F32Buf l_in,
                       S32Buf q_seg, S32Buf kv_seg, S32Buf q_prefix, S32Buf kv_prefix, F32Buf slopes, F32Buf dense,
                       F32Res o, F32Res m, F32Res l, float sm_scale, int32_t bias_flags, int32_t window,
                       int64_t q_offset, int64_t kv_offset) {
  ra_fwd_step_params p{};
  int64_t dq[4], dk[4], dv[4];
  if (!View4(q, &p.q, dq) || !View4(k, &p.k, dk) || !View4(v, &p.v, dv))
    return ffi::Error::InvalidArgument("q, k, v must be [b, h, l, d]");
  if (dk[0] != dq[0] || dk[1] != dq[1] || dk[3] != dq[3] || dv[0] != dk[0] || dv[1] != dk[1] || dv[2] != dk[2] ||
      dv[3] != dk[3])
    return ffi::Error::InvalidArgument("q, k, v disagree in batch, heads or head dim (dk must equal dv)");
  p.B = (int32_t)dq[0];
  p.H = (int32_t)dq[1];
  p.Lq = (int32_t)dq[2];
  p.Lk = (int32_t)dk[2];
  p.D = (int32_t)dq[3];
  p.sm_scale = sm_scale;
  const size_t rows = (size_t)dq[0] * dq[1] * dq[2];
  if (o_in.element_count() != rows * (size_t)dq[3] || m_in.element_count() != rows || l_in.element_count() != rows ||
      o->element_count() != o_in.element_count() || m->element_count() != rows || l->element_count() != rows)
    return ffi::Error::InvalidArgument("carry shapes must be o [b, h, lq, d], m and l [b, h, lq]");
  if (auto e = Carry(stream, o_in.typed_data(), o->typed_data(), o_in.size_bytes()); e.failure()) return e;
  if (auto e = Carry(stream, m_in.typed_data(), m->typed_data(), m_in.size_bytes()); e.failure()) return e;
  if (auto e = Carry(stream, l_in.typed_data(), l->typed_data(), l_in.size_bytes()); e.failure()) return e;
  p.o = o->typed_data();
  p.m = m->typed_data();
  p.l = l->typed_data();
  if (auto e = FillBias(&p.bias, bias_flags, window, q_offset, kv_offset, q_seg, kv_seg, q_prefix, kv_prefix, slopes,
                        dense, dq[0], dq[1], dq[2], dk[2]);
      e.failure())
    return e;
  const int rc = ra_fwd_step(&p, stream);
  return rc == RA_OK ? ffi::Error::Success() : Fail("ra_fwd_step", rc);
}

// ---- o / l and m + log l after the scan (ring.py:134-135) ------------------------------------
ffi::Error FwdFinalizeImpl(hipStream_t stream, F32Buf o, F32Buf m, F32Buf l, ffi::Result<ffi::AnyBuffer> out,
                           F32Res lse) {
  auto d = o.dimensions();
  if (d.size() != 4) return ffi::Error::InvalidArgument("o must be [b, h, lq, d]");
  int32_t dt;
  if (out->element_type() == ffi::BF16) dt = RA_DTYPE_BF16;
  else if (out->element_type() == ffi::F32) dt = RA_DTYPE_F32;
  else return ffi::Error::InvalidArgument("out must be bfloat16 or float32");
  if (out->element_count() != o.element_count() || lse->element_count() != m.element_count())
    return ffi::Error::InvalidArgument("out must have the shape of o, lse the shape of m");
  const int rc = ra_fwd_finalize(o.typed_data(), m.typed_data(), l.typed_data(), out->untyped_data(), dt,
                                 d[1] * d[2] * d[3], d[2] * d[3], d[3], lse->typed_data(), (int32_t)d[0],
                                 (int32_t)d[1], (int32_t)d[2], (int32_t)d[3], stream);
  return rc == RA_OK ? ffi::Error::Success() : Fail("ra_fwd_finalize", rc);
}

// ---- _precompute_delta (ring_kernel.py:387-409): delta = rowsum(out * dout) -------------------
ffi::Error BwdDeltaImpl(hipStream_t stream, ffi::AnyBuffer out, Bf16Buf dout, F32Res delta) {
  ra_tensor dt_view;
  int64_t d[4];
  if (!View4(dout, &dt_view, d)) return ffi::Error::InvalidArgument("dout must be [b, h, lq, d]");
  int32_t dt;
  if (out.element_type() == ffi::BF16) dt = RA_DTYPE_BF16;
  else if (out.element_type() == ffi::F32) dt = RA_DTYPE_F32;
  else return ffi::Error::InvalidArgument("out must be bfloat16 or float32");
  if (out.element_count() != dout.element_count() || delta->element_count() != (size_t)(d[0] * d[1] * d[2]))
    return ffi::Error::InvalidArgument("out must have the shape of dout, delta must be [b, h, lq]");
  const int rc = ra_bwd_delta(out.untyped_data(), dt, d[1] * d[2] * d[3], d[2] * d[3], d[3], &dt_view,
                              delta->typed_data(), (int32_t)d[0], (int32_t)d[1], (int32_t)d[2], (int32_t)d[3], stream);
  return rc == RA_OK ? ffi::Error::Success() : Fail("ra_bwd_delta", rc);
}

// ---- bwd_block (ring_kernel.py:202-297 / ring.py:140-157) with the accumulation ring.py:191-193 -
ffi::Error BwdStepImpl(hipStream_t stream, Bf16Buf q, Bf16Buf k, Bf16Buf v, Bf16Buf dout, F32Buf lse, F32Buf delta,
                       F32Buf dq_in, F32Buf dk_in, F32Buf dv_in, S32Buf q_seg, S32Buf kv_seg, S32Buf q_prefix,
                       S32Buf kv_prefix, F32Buf slopes, F32Buf dense, F32Res dq, F32Res dk, F32Res dv, float sm_scale,
                       int32_t bias_flags, int32_t window, int64_t q_offset, int64_t kv_offset) {
  ra_bwd_step_params p{};
  int64_t sq[4], sk[4], sv[4], sd[4];
  if (!View4(q, &p.q, sq) || !View4(k, &p.k, sk) || !View4(v, &p.v, sv) || !View4(dout, &p.dout, sd))
    return ffi::Error::InvalidArgument("q, k, v, dout must be [b, h, l, d]");
  if (sk[0] != sq[0] || sk[1] != sq[1] || sk[3] != sq[3] || sv[0] != sk[0] || sv[1] != sk[1] || sv[2] != sk[2] ||
      sv[3] != sk[3] || sd[0] != sq[0] || sd[1] != sq[1] || sd[2] != sq[2] || sd[3] != sq[3])
    return ffi::Error::InvalidArgument("q, k, v, dout disagree in batch, heads, length or head dim");
  p.B = (int32_t)sq[0];
  p.H = (int32_t)sq[1];
  p.Lq = (int32_t)sq[2];
  p.Lk = (int32_t)sk[2];
  p.D = (int32_t)sq[3];
  p.sm_scale = sm_scale;
  const size_t rows_q = (size_t)sq[0] * sq[1] * sq[2], rows_k = (size_t)sk[0] * sk[1] * sk[2];
  if (lse.element_count() != rows_q || delta.element_count() != rows_q ||
      dq_in.element_count() != rows_q * (size_t)sq[3] || dk_in.element_count() != rows_k * (size_t)sq[3] ||
      dv_in.element_count() != rows_k * (size_t)sq[3] || dq->element_count() != dq_in.element_count() ||
      dk->element_count() != dk_in.element_count() || dv->element_count() != dv_in.element_count())
    return ffi::Error::InvalidArgument("lse, delta must be [b, h, lq]; dq [b, h, lq, d]; dk, dv [b, h, lk, d]");
  p.lse = lse.typed_data();
  p.delta = delta.typed_data();
  if (auto e = Carry(stream, dq_in.typed_data(), dq->typed_data(), dq_in.size_bytes()); e.failure()) return e;
  if (auto e = Carry(stream, dk_in.typed_data(), dk->typed_data(), dk_in.size_bytes()); e.failure()) return e;
  if (auto e = Carry(stream, dv_in.typed_data(), dv->typed_data(), dv_in.size_bytes()); e.failure()) return e;
  p.dq = dq->typed_data();
  p.dk = dk->typed_data();
  p.dv = dv->typed_data();
  if (auto e = FillBias(&p.bias, bias_flags, window, q_offset, kv_offset, q_seg, kv_seg, q_prefix, kv_prefix, slopes,
                        dense, sq[0], sq[1], sq[2], sk[2]);
      e.failure())
    return e;
  const int rc = ra_bwd_step(&p, stream);
  return rc == RA_OK ? ffi::Error::Success() : Fail("ra_bwd_step", rc);
}

// ---- fp32 accumulator -> bf16 gradient (the casts behind ring.py:208-210) ----------------------
ffi::Error BwdFinalizeImpl(hipStream_t stream, F32Buf acc, ffi::Result<Bf16Buf> out) {
  auto d = acc.dimensions();
  if (d.size() != 4 || out->element_count() != acc.element_count())
    return ffi::Error::InvalidArgument("acc must be [b, h, l, d] and out must have its shape");
  const int rc = ra_bwd_finalize(acc.typed_data(), out->untyped_data(), d[1] * d[2] * d[3], d[2] * d[3], d[3],
                                 (int32_t)d[0], (int32_t)d[1], (int32_t)d[2], (int32_t)d[3], stream);
  return rc == RA_OK ? ffi::Error::Success() : Fail("ra_bwd_finalize", rc);
}

}  // namespace

// Operand / result / attribute order below is the order ffi_call passes them in.
XLA_FFI_DEFINE_HANDLER_SYMBOL(
    RaFwdStep, FwdStepImpl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<Bf16Buf>()  // q  [b, h, lq, d]
        .Arg<Bf16Buf>()  // k  [b, h, lk, d]
        .Arg<Bf16Buf>()  // v  [b, h, lk, d]
        .Arg<F32Buf>()   // o  [b, h, lq, d]  carry, aliased to result 0
        .Arg<F32Buf>()   // m  [b, h, lq]     carry, aliased to result 1
        .Arg<F32Buf>()   // l  [b, h, lq]     carry, aliased to result 2
        .Arg<S32Buf>()   // q_segment_ids  [b, lq] or empty
        .Arg<S32Buf>()   // kv_segment_ids [b, lk] or empty
        .Arg<S32Buf>()   // q_prefix_mask  [b, lq] or empty
        .Arg<S32Buf>()   // kv_prefix_mask [b, lk] or empty
        .Arg<F32Buf>()   // alibi_slopes   [h] or empty
        .Arg<F32Buf>()   // dense bias     [b | 1, h | 1, lq, lk] or empty
        .Ret<F32Buf>()   // o
        .Ret<F32Buf>()   // m
        .Ret<F32Buf>()   // l
        .Attr<float>("sm_scale")
        .Attr<int32_t>("bias_flags")
        .Attr<int32_t>("window")
        .Attr<int64_t>("q_offset")
        .Attr<int64_t>("kv_offset"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(RaFwdFinalize, FwdFinalizeImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<F32Buf>()          // o
                                  .Arg<F32Buf>()          // m
                                  .Arg<F32Buf>()          // l
                                  .Ret<ffi::AnyBuffer>()  // out (bf16 or fp32) [b, h, lq, d]
                                  .Ret<F32Buf>());        // lse [b, h, lq]

XLA_FFI_DEFINE_HANDLER_SYMBOL(RaBwdDelta, BwdDeltaImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<ffi::AnyBuffer>()  // out (bf16 or fp32) [b, h, lq, d]
                                  .Arg<Bf16Buf>()         // dout
                                  .Ret<F32Buf>());        // delta [b, h, lq]

XLA_FFI_DEFINE_HANDLER_SYMBOL(
    RaBwdStep, BwdStepImpl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<Bf16Buf>()  // q
        .Arg<Bf16Buf>()  // k
        .Arg<Bf16Buf>()  // v
        .Arg<Bf16Buf>()  // dout
        .Arg<F32Buf>()   // lse   [b, h, lq]
        .Arg<F32Buf>()   // delta [b, h, lq]
        .Arg<F32Buf>()   // dq accumulator [b, h, lq, d], aliased to result 0
        .Arg<F32Buf>()   // dk accumulator [b, h, lk, d], aliased to result 1
        .Arg<F32Buf>()   // dv accumulator [b, h, lk, d], aliased to result 2
        .Arg<S32Buf>()   // q_segment_ids
        .Arg<S32Buf>()   // kv_segment_ids
        .Arg<S32Buf>()   // q_prefix_mask
        .Arg<S32Buf>()   // kv_prefix_mask
        .Arg<F32Buf>()   // alibi_slopes
        .Arg<F32Buf>()   // dense bias
        .Ret<F32Buf>()   // dq
        .Ret<F32Buf>()   // dk
        .Ret<F32Buf>()   // dv
        .Attr<float>("sm_scale")
        .Attr<int32_t>("bias_flags")
        .Attr<int32_t>("window")
        .Attr<int64_t>("q_offset")
        .Attr<int64_t>("kv_offset"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(RaBwdFinalize, BwdFinalizeImpl,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Arg<F32Buf>()     // fp32 accumulator [b, h, l, d]
                                  .Ret<Bf16Buf>());  // bf16 gradient

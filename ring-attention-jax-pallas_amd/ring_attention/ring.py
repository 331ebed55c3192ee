"""Ring attention on one MI355X: the reference's call surface over the HIP block-step kernels.

Public names follow the reference (``ring.py:246`` ``ring_attention``, ``ring.py:328``
``ring_self_attention``; block functions ``ring_kernel.py:123`` ``fwd_block`` and
``ring_kernel.py:202`` ``bwd_block``).  What differs, and why:

* There is one GPU and no mesh.  ``q, k, v`` are the GLOBAL ``[b, S, h, d]`` arrays and
  ``axis_name`` carries the ring size (``RingAxis("sp", 8)`` or just ``8``).  The ring is
  emulated: the arrays are cut into ``size`` shards along the sequence; "device" r keeps
  query shard r and its fp32 ``(o, m, l)`` carry, and at step t meets the key/value shard
  that started on device ``(r - t) mod size`` - the order ``ppermute`` produces in
  ``ring.py:51-55,120``.  In the backward pass the query side travels instead
  (``ring.py:195``).  The result is what ``shard_map(ring_attention)`` returns for the
  global arrays.
* ``bias_fn`` is either a declarative ``BiasFn`` (see ``bias.py``), evaluated inside the
  kernels so that ring steps and score tiles that are entirely masked are skipped, or any
  Python callable with the reference's contract ``bias_fn(**q_kwargs, **kv_kwargs) ->
  [b, h | 1, lq, lk]`` (ring.py:107), whose dense block is materialised per ring step and
  streamed by the kernels.
* Compute is bf16 on the matrix cores with fp32 carries; other input dtypes are cast on
  entry and the result is cast back.  Head dims other than 64/128 are zero-padded.

Everything runs through ``libringattn_hip.so``; if it is missing the import of this module
succeeds but every call raises.
"""
from __future__ import annotations

import collections
import ctypes as C
import math
from dataclasses import dataclass
from typing import Callable, Optional, Union

import torch

from . import _lib
from .bias import BiasFn, BlockBias

# The reference's two values (ring.py:255,296-312) plus the two launch schemes by name:
#   "pallas"    its default, "fused kernels": the library picks the launch scheme - the whole ring
#               per launch (below) wherever that applies, a launch per step otherwise;
#   "jax"       its plain per-block loop: one launch per ring step (the same as "hip");
#   "hip"       one launch per ring step, the reference's loop (ring.py:104-132) as it stands;
#   "hip_fused" one launch for ALL ring passes - the kernels walk the shards of a query (or
#               key/value) shard's whole trip around the ring themselves, one grid row per
#               resident shard.
_IMPLS = ("pallas", "jax", "hip", "hip_fused")


def _launch_whole_ring(block_impl: str, plan: "_RingPlan") -> bool:
    """Which launch scheme a call takes.  On one GPU every shard of the emulated ring is resident,
    so nothing has to wait for a transfer and the whole ring can go into one launch: never slower
    than a launch per step, and up to twice as fast where one step cannot fill the chip (shards of
    a few thousand tokens) or where a positional mask leaves a step work for only some of its
    workgroups.  A callable ``bias_fn`` keeps the launch per step: its dense block is built per
    (query shard, key/value shard) pair and only one is alive at a time that way."""
    if block_impl == "hip_fused":
        return True
    if block_impl in ("hip", "jax"):
        return False
    return plan.callable is None


@dataclass(frozen=True)
class RingAxis:
    """Stands in for the mesh axis the reference shards sequences over."""
    name: str
    size: int


def _axis_size(axis_name) -> int:
    if isinstance(axis_name, RingAxis):
        return axis_name.size
    if isinstance(axis_name, int):
        return axis_name
    if isinstance(axis_name, (tuple, list)) and len(axis_name) == 2:
        return int(axis_name[1])
    raise TypeError("axis_name must be a RingAxis, an int ring size or a (name, size) pair")


def _walked_ring_size(n: int, Sq: int, Sk: int, bias_fn) -> int:
    """Ring size that the emulation walks.  Under a segment bias one call of the library takes
    shards of at most ``RA_MAX_SEGMENT_SHARD`` tokens; a ring whose shards are longer is walked as
    a finer ring (every shard cut into f equal pieces).  The online softmax is associative over
    key/value shards and independent over query rows (ring.py:58-76), so the result is the same
    up to the rounding of a different summation order.  Lengths that no f <= 4096 divides keep
    ``n`` (and the library reports the limit)."""
    if not (isinstance(bias_fn, BiasFn) and bias_fn.segments) or Sq % n or Sk % n:
        return n
    longest = max(Sq // n, Sk // n)
    if longest <= _lib.RA_MAX_SEGMENT_SHARD:
        return n
    for f in range(-(-longest // _lib.RA_MAX_SEGMENT_SHARD), 4097):
        if (Sq // n) % f == 0 and (Sk // n) % f == 0:
            return n * f
    return n


def _stream() -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _require_gpu(t: torch.Tensor) -> None:
    if not t.is_cuda:
        raise RuntimeError("ring_attention runs on the GPU only: tensors must live on a HIP device "
                           "(there is no CPU fallback)")


def _view_bhld(t: torch.Tensor) -> _lib.RaTensor:
    """RaTensor for a tensor indexed [b, h, l, d] (any strides, d contiguous)."""
    return _lib.RaTensor(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))


def _kernel_ready(t: torch.Tensor) -> torch.Tensor:
    """[b, l, h, d] as the kernels take it: bf16, unit inner stride, 16-byte aligned rows that do not
    overlap and lie within the row stride the C ABI admits; anything else is copied."""
    if t.dtype != torch.bfloat16:
        t = t.to(torch.bfloat16)
    ok = (t.stride(-1) == 1 and all(s % 8 == 0 for s in t.stride()[:-1]) and t.data_ptr() % 16 == 0
          and t.shape[-1] <= t.stride(1) <= _lib.RA_MAX_ROW_STRIDE)
    return t if ok else t.contiguous()


# --------------------------------------------------------------------------------------
# block-level API (one ring step)
# --------------------------------------------------------------------------------------
def _bias_struct(bias, device, shape=None, summary=True) -> _lib.RaBias:
    """``bias`` is None, a ``BlockBias`` or a dense additive array ``[b, h | 1, lq, lk]`` - the
    form the reference's block functions take (ring_kernel.py:127,206).  ``summary``: a dense
    block travels with its summary (``ra_dense_map``); the single-step launches read it, the
    several-step launches do not, so their callers pass False."""
    if bias is None:
        return _lib.RaBias()
    if isinstance(bias, torch.Tensor):
        bias = BlockBias(dense=bias)
    if shape is not None:
        bias.check_dense_shape(*shape)
    return bias.to_struct(device, summary=summary)


def fwd_block(q, k, v, bias: Union[BlockBias, torch.Tensor, None], o, m, l, sm_scale: float):
    """One ring step of the forward pass, in place on the fp32 carry.

    Same contract as the reference's ``fwd_block`` (ring_kernel.py:123-199): ``q`` is
    ``[b, h, lq, d]``, ``k``/``v`` are ``[b, h, lk, d]`` (bf16, any batch/head/length strides),
    ``o`` ``[b, h, lq, d]`` is the unnormalised output and ``m``/``l`` ``[b, h, lq]`` the
    running max / sum (fp32, contiguous).  ``bias`` is the block's additive bias: a dense
    ``[b, h | 1, lq, lk]`` array as in the reference, or a ``BlockBias`` description.
    Returns ``(o, m, l)`` (the same tensors, updated)."""
    _require_gpu(q)
    lib = _lib.load()
    B, H, Lq, D = q.shape
    p = _lib.RaFwdStepParams()
    p.B, p.H, p.Lq, p.Lk, p.D = B, H, Lq, k.shape[2], D
    p.sm_scale = float(sm_scale)
    p.q, p.k, p.v = _view_bhld(q), _view_bhld(k), _view_bhld(v)
    for t_ in (o, m, l):
        if t_.dtype != torch.float32 or not t_.is_contiguous():
            raise ValueError("o, m, l carries must be contiguous float32 tensors")
    p.o, p.m, p.l = o.data_ptr(), m.data_ptr(), l.data_ptr()
    p.bias = _bias_struct(bias, q.device, (B, H, Lq, k.shape[2]))
    _lib.check("ra_fwd_step", lib.ra_fwd_step(C.byref(p), _stream()))
    return o, m, l


def _fwd_params(q, k, v, bias, o, m, l, sm_scale, summary=False) -> _lib.RaFwdStepParams:
    B, H, Lq, D = q.shape
    p = _lib.RaFwdStepParams()
    p.B, p.H, p.Lq, p.Lk, p.D = B, H, Lq, k.shape[2], D
    p.sm_scale = float(sm_scale)
    p.q, p.k, p.v = _view_bhld(q), _view_bhld(k), _view_bhld(v)
    if o is not None:  # None: the caller fills the carry pointers in later, or has no carry
        for t_ in (o, m, l):
            if t_.dtype != torch.float32 or not t_.is_contiguous():
                raise ValueError("o, m, l carries must be contiguous float32 tensors")
        p.o, p.m, p.l = o.data_ptr(), m.data_ptr(), l.data_ptr()
    p.bias = _bias_struct(bias, q.device, (B, H, Lq, k.shape[2]), summary=summary)
    return p


def fwd_blocks(q, kvs, biases, o, m, l, sm_scale: float):
    """Several consecutive ring steps of one query shard in ONE launch: equivalent to
    ``fwd_block(q, k, v, bias, o, m, l, sm_scale)`` for every ``(k, v)`` of ``kvs`` with the bias
    of the same index, in that order (the loop ring.py:104-132), with the step's running state
    kept in registers between the shards.  The shards share their shape and strides."""
    _require_gpu(q)
    lib = _lib.load()
    steps = (_lib.RaFwdStepParams * len(kvs))()
    keep = []  # the bias structs point into tensors that must outlive the call
    for i, ((k, v), bias) in enumerate(zip(kvs, biases)):
        if isinstance(bias, torch.Tensor):
            bias = BlockBias(dense=bias)
        keep.append(bias)
        steps[i] = _fwd_params(q, k, v, bias, o, m, l, sm_scale)
    _lib.check("ra_fwd_steps", lib.ra_fwd_steps(steps, len(kvs), _stream()))
    return o, m, l


def init_carry(batch, heads, q_len, dim, device):
    """Fresh carry o = 0, l = 0, m = -inf (ring.py:124-126), fp32."""
    lib = _lib.load()
    o = torch.empty((batch, heads, q_len, dim), dtype=torch.float32, device=device)
    m = torch.empty((batch, heads, q_len), dtype=torch.float32, device=device)
    l = torch.empty((batch, heads, q_len), dtype=torch.float32, device=device)
    reset_carry(o, m, l)
    return o, m, l


def reset_carry(o, m, l):
    lib = _lib.load()
    B, H, Lq, D = o.shape
    _lib.check("ra_fwd_init", lib.ra_fwd_init(o.data_ptr(), m.data_ptr(), l.data_ptr(), B, H, Lq, D,
                                              _stream()))


def finalize_carry(o, m, l, out, lse):
    """out = o / l written into ``out`` ([b, h, lq, d] view, bf16 or fp32), lse = m + log l
    (ring.py:134-135)."""
    lib = _lib.load()
    B, H, Lq, D = o.shape
    dt = {torch.bfloat16: _lib.RA_DTYPE_BF16, torch.float32: _lib.RA_DTYPE_F32}[out.dtype]
    _lib.check("ra_fwd_finalize", lib.ra_fwd_finalize(
        o.data_ptr(), m.data_ptr(), l.data_ptr(), out.data_ptr(), dt, out.stride(0), out.stride(1),
        out.stride(2), lse.data_ptr(), B, H, Lq, D, _stream()))


def precompute_delta(out, do, delta=None):
    """delta = rowsum(out * do) in fp32 (ring_kernel.py:387-409).  ``out`` (bf16 or fp32) and
    ``do`` (bf16) are ``[b, h, l, d]`` views; returns ``[b, h, l]``."""
    _require_gpu(out)
    lib = _lib.load()
    B, H, L, D = out.shape
    if delta is None:
        delta = torch.empty((B, H, L), dtype=torch.float32, device=out.device)
    dt = {torch.bfloat16: _lib.RA_DTYPE_BF16, torch.float32: _lib.RA_DTYPE_F32}[out.dtype]
    do_t = _view_bhld(do)
    _lib.check("ra_bwd_delta", lib.ra_bwd_delta(out.data_ptr(), dt, out.stride(0), out.stride(1),
                                                out.stride(2), C.byref(do_t), delta.data_ptr(), B, H,
                                                L, D, _stream()))
    return delta


def _bwd_params(q, k, v, do, lse, delta, dq, dk, dv, bias, sm_scale, summary=False) -> _lib.RaBwdStepParams:
    B, H, Lq, D = q.shape
    p = _lib.RaBwdStepParams()
    p.B, p.H, p.Lq, p.Lk, p.D = B, H, Lq, k.shape[2], D
    p.sm_scale = float(sm_scale)
    p.q, p.k, p.v, p.dout = _view_bhld(q), _view_bhld(k), _view_bhld(v), _view_bhld(do)
    p.lse, p.delta = lse.data_ptr(), delta.data_ptr()
    if dq is not None:  # None: the caller fills the accumulator pointers in later, or has none
        p.dq, p.dk, p.dv = dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    p.bias = _bias_struct(bias, q.device, (B, H, Lq, k.shape[2]), summary=summary)
    return p


def _bwd_step(q, k, v, do, lse, delta, dq, dk, dv, bias, sm_scale, parts=3):
    lib = _lib.load()
    p = _bwd_params(q, k, v, do, lse, delta, dq, dk, dv, bias, sm_scale, summary=True)
    _lib.check("ra_bwd_step", lib.ra_bwd_step_parts(C.byref(p), parts, _stream()))


def _bwd_steps(which: str, step_args, sm_scale):
    """``step_args``: one ``(q, k, v, do, lse, delta, dq, dk, dv, bias)`` tuple per ring step, as
    for ``_bwd_step``; ``which`` is ``"dq"`` (one query shard, several key/value shards) or
    ``"dkdv"`` (one key/value shard, several query shards).  One launch for all of them."""
    lib = _lib.load()
    steps = (_lib.RaBwdStepParams * len(step_args))()
    keep = []  # the bias structs point into tensors that must outlive the call
    for i, args in enumerate(step_args):
        bias = args[9]
        if isinstance(bias, torch.Tensor):
            bias = BlockBias(dense=bias)
        keep.append(bias)
        steps[i] = _bwd_params(*args[:9], bias, sm_scale)
    fn = {"dq": "ra_bwd_dq_steps", "dkdv": "ra_bwd_dkdv_steps"}[which]
    _lib.check(fn, getattr(lib, fn)(steps, len(step_args), _stream()))


def bwd_block(q, k, v, bias: Union[BlockBias, torch.Tensor, None], o, L, do, sm_scale: float):
    """Gradients of one (query block, key/value block) pair, as the reference's
    ``bwd_block`` (ring_kernel.py:202-297): all tensors ``[b, h, l, d]``, ``o`` the normalised
    forward output, ``L`` the logsumexp ``[b, h, lq]``.  Returns fp32 ``(dq, dk, dv)``."""
    _require_gpu(q)
    delta = precompute_delta(o, do)
    dq = torch.zeros(q.shape, dtype=torch.float32, device=q.device)
    dk = torch.zeros(k.shape, dtype=torch.float32, device=q.device)
    dv = torch.zeros(v.shape, dtype=torch.float32, device=q.device)
    _bwd_step(q, k, v, do, L.contiguous(), delta, dq, dk, dv, bias, sm_scale)
    return dq, dk, dv


def _finalize_grad(acc, out):
    lib = _lib.load()
    B, H, L, D = acc.shape
    _lib.check("ra_bwd_finalize", lib.ra_bwd_finalize(acc.data_ptr(), out.data_ptr(), out.stride(0),
                                                      out.stride(1), out.stride(2), B, H, L, D,
                                                      _stream()))


# --------------------------------------------------------------------------------------
# emulated ring
# --------------------------------------------------------------------------------------
class _RingPlan:
    """Shard bookkeeping shared by the forward and backward loops."""

    def __init__(self, q, k, n, fn: Optional[BiasFn], q_kwargs, kv_kwargs):
        self.n = n
        self.B, Sq, self.H, self.D = q.shape
        Sk = k.shape[1]
        if Sq % n or Sk % n:
            raise ValueError(f"sequence lengths ({Sq}, {Sk}) must be divisible by the ring size {n}")
        self.Lq, self.Lk = Sq // n, Sk // n
        self.fn = fn
        self.callable = None
        dev = q.device
        q_kwargs = dict(q_kwargs or {})
        kv_kwargs = dict(kv_kwargs or {})
        self.q_off = [r * self.Lq for r in range(n)]
        self.kv_off = [r * self.Lk for r in range(n)]
        if fn is not None and not isinstance(fn, BiasFn):
            # The reference's general form (ring.py:107,186): any callable of per-token arrays.
            # Every kwarg is an array whose axis 1 is the sequence; its shards travel with the
            # query / key-value shards exactly as bias_q_kwargs / bias_kv_kwargs do there.
            for name, t in list(q_kwargs.items()) + list(kv_kwargs.items()):
                S = Sq if name in q_kwargs else Sk
                if not isinstance(t, torch.Tensor) or t.dim() < 2 or t.shape[1] != S:
                    raise ValueError(f"bias kwarg {name!r} must be a tensor [b, {S}, ...]")
            self.callable = fn
            self.fn = None
            self.q_kw = {a: t.to(dev) for a, t in q_kwargs.items()}
            self.kv_kw = {a: t.to(dev) for a, t in kv_kwargs.items()}
            return
        known_q = {"q_segment_ids", "q_positions", "q_prefix_mask"}
        known_kv = {"kv_segment_ids", "kv_positions", "kv_prefix_mask"}
        for name in list(q_kwargs) + list(kv_kwargs):
            if name not in known_q | known_kv:
                raise ValueError(f"unknown bias kwarg {name!r}; expected one of "
                                 f"{sorted(known_q | known_kv)}")
        if fn is None and any(v is not None for v in list(q_kwargs.values()) + list(kv_kwargs.values())):
            raise ValueError("bias kwargs were given without a bias_fn")

        def ids(t, S, name):
            if t is None:
                return None
            if tuple(t.shape) != (self.B, S):
                raise ValueError(f"{name} must have shape {(self.B, S)}, got {tuple(t.shape)}")
            return t.to(device=dev, dtype=torch.int32).contiguous()

        self.q_seg = self.kv_seg = self.q_pre = self.kv_pre = None
        if fn is not None:
            fn.validate()
            if fn.segments:
                self.q_seg = ids(q_kwargs.get("q_segment_ids"), Sq, "q_segment_ids")
                self.kv_seg = ids(kv_kwargs.get("kv_segment_ids"), Sk, "kv_segment_ids")
                if self.q_seg is None or self.kv_seg is None:
                    raise ValueError("segment bias needs q_segment_ids and kv_segment_ids")
            if fn.prefix:
                self.q_pre = ids(q_kwargs.get("q_prefix_mask"), Sq, "q_prefix_mask")
                self.kv_pre = ids(kv_kwargs.get("kv_prefix_mask"), Sk, "kv_prefix_mask")
                if self.q_pre is None or self.kv_pre is None:
                    raise ValueError("prefix bias needs q_prefix_mask and kv_prefix_mask")
            if fn.alibi_slopes is not None:
                if fn.alibi_slopes.numel() != self.H:
                    raise ValueError("alibi slopes must have one entry per head")
                self.fn = fn = BiasFn(fn.causal, fn.window, fn.segments, fn.prefix,
                                      fn.alibi_slopes.to(device=dev, dtype=torch.float32).contiguous())
            if fn.needs_positions:
                qp, kp = q_kwargs.get("q_positions"), kv_kwargs.get("kv_positions")
                q_off = self.q_off if qp is None else self._offsets(qp, Sq, self.Lq, "q_positions")
                kv_off = self.kv_off if kp is None else self._offsets(kp, Sk, self.Lk, "kv_positions")
                if q_off is None or kv_off is None:
                    # Arbitrary positions (the reference compares kv_positions <= q_positions element
                    # by element, ring.py:396): the kernels take one offset per shard, so the terms
                    # are materialised per ring step from the position arrays and streamed as a
                    # dense block, like a callable bias_fn.
                    def full(t, S):
                        if t is None:
                            t = torch.arange(S, device=dev)[None].expand(self.B, S)
                        return t.to(device=dev, dtype=torch.int64)
                    self.callable = _positional_bias_callable(fn)
                    self.fn = None
                    self.q_kw = {"q_positions": full(qp, Sq)}
                    self.kv_kw = {"kv_positions": full(kp, Sk)}
                    for kw, name, t in ((self.q_kw, "q_segment_ids", self.q_seg), (self.kv_kw, "kv_segment_ids", self.kv_seg),
                                        (self.q_kw, "q_prefix_mask", self.q_pre), (self.kv_kw, "kv_prefix_mask", self.kv_pre)):
                        if t is not None:
                            kw[name] = t
                    return
                self.q_off, self.kv_off = q_off, kv_off

    def _offsets(self, pos, S, L, name):
        """One position offset per shard if the positions are consecutive inside every shard and
        equal across the batch (what the in-kernel terms take); None otherwise."""
        if tuple(pos.shape) != (self.B, S):
            raise ValueError(f"{name} must have shape {(self.B, S)}, got {tuple(pos.shape)}")
        pos = pos.to(torch.int64)
        starts = pos[:, ::L]
        expect = (starts[:, :, None] + torch.arange(L, device=pos.device)[None, None, :]).reshape(self.B, S)
        if not torch.equal(expect, pos) or not bool((starts == starts[:1]).all()):
            return None
        if int(starts.min()) < 0 or int(starts.max()) + L > _lib.RA_MAX_POSITION:
            return None  # outside the position range of the C ABI
        return [int(x) for x in starts[0].tolist()]

    def live_steps(self, qs: Optional[int], ks: Optional[int]) -> int:
        """How many ring steps of query shard ``qs`` (or key/value shard ``ks``) are not masked
        entirely by the positional terms - the steps that cost something."""
        fn = self.fn
        if fn is None or not (fn.causal or fn.window):
            return self.n
        cnt = 0
        for other in range(self.n):
            q_lo = self.q_off[qs if qs is not None else other]
            k_lo = self.kv_off[ks if ks is not None else other]
            q_hi, k_hi = q_lo + self.Lq - 1, k_lo + self.Lk - 1
            dead = fn.causal and k_lo > q_hi
            if fn.window:
                dead = dead or q_lo - k_hi >= fn.window or (not fn.causal and k_lo - q_hi >= fn.window)
            cnt += not dead
        return cnt

    def block_bias(self, qs: int, ks: int) -> Optional[BlockBias]:
        """Bias of (query shard qs, key/value shard ks)."""
        sl_q = slice(qs * self.Lq, (qs + 1) * self.Lq)
        sl_k = slice(ks * self.Lk, (ks + 1) * self.Lk)
        if self.callable is not None:
            dense = self.callable(**{a: t[:, sl_q] for a, t in self.q_kw.items()},
                                  **{a: t[:, sl_k] for a, t in self.kv_kw.items()})
            if not isinstance(dense, torch.Tensor):
                raise TypeError("a callable bias_fn must return a torch.Tensor [b, h | 1, lq, lk]")
            return BlockBias(dense=dense)
        if self.fn is None:
            return None
        return BlockBias(
            self.fn, self.q_off[qs], self.kv_off[ks],
            None if self.q_seg is None else self.q_seg[:, sl_q],
            None if self.kv_seg is None else self.kv_seg[:, sl_k],
            None if self.q_pre is None else self.q_pre[:, sl_q],
            None if self.kv_pre is None else self.kv_pre[:, sl_k])


def _positional_bias_callable(fn: BiasFn):
    """The terms of ``fn`` as a dense-bias callable of explicit per-token positions: the mask
    builder of the reference (ring.py:376-409: segments ``:388-391``, causal ``kv_pos <= q_pos``
    ``:393-397``, prefix-LM ``:399-406``, ``where(mask, 0, -inf)[:, None]`` ``:408-409``) plus the
    window and ALiBi terms, for positions that one offset per shard cannot express."""
    def bias_fn(q_positions, kv_positions, q_segment_ids=None, kv_segment_ids=None, q_prefix_mask=None,
                kv_prefix_mask=None):
        rel = q_positions[:, :, None] - kv_positions[:, None, :]  # [b, lq, lk]
        mask = torch.ones_like(rel, dtype=torch.bool)
        if fn.segments:
            mask &= q_segment_ids[:, :, None] == kv_segment_ids[:, None, :]
        if fn.causal:
            mask &= rel >= 0
        if fn.window is not None:
            mask &= (rel < fn.window) if fn.causal else (rel.abs() < fn.window)
        if fn.prefix:
            mask &= ((q_prefix_mask[:, :, None] != 0) & (kv_prefix_mask[:, None, :] != 0)) | (rel >= 0)
        bias = torch.zeros(mask.shape, dtype=torch.float32, device=mask.device)
        bias.masked_fill_(~mask, float("-inf"))
        bias = bias[:, None]
        if fn.alibi_slopes is not None:
            bias = bias - fn.alibi_slopes.to(bias.device)[None, :, None, None] * rel.abs()[:, None].to(torch.float32)
        return bias
    return bias_fn


def _shard_bhld(x, s, L):
    """Shard s of a [b, S, h, d] array, viewed as [b, h, L, d] (no copy)."""
    return x[:, s * L:(s + 1) * L].permute(0, 2, 1, 3)


class _NoTimer:
    """Default launch observer: does nothing.  A benchmark passes an object whose
    ``span(kind, qs, ks)`` context manager brackets one kernel launch with stream events."""

    class _Span:
        def __enter__(self):
            return self

        def __exit__(self, *exc):
            return False

    _span = _Span()
    split_bwd = False

    def span(self, kind, qs, ks):
        return self._span


_NO_TIMER = _NoTimer()


def _ring_forward(q, k, v, plan: _RingPlan, sm_scale, out_dtype, carries_out=None, timer=_NO_TIMER):
    n, B, H, D, Lq, Lk = plan.n, plan.B, plan.H, plan.D, plan.Lq, plan.Lk
    dev = q.device
    out = torch.empty((B, n * Lq, H, D), dtype=out_dtype, device=dev)
    lse = torch.empty((n, B, H, Lq), dtype=torch.float32, device=dev)
    o, m, l = init_carry(B, H, Lq, D, dev)
    for r in range(n):
        if r:
            reset_carry(o, m, l)
        qr = _shard_bhld(q, r, Lq)
        for t in range(n):
            src = (r - t) % n  # ring.py:51-55: after t rotations device r holds shard r - t
            bias = plan.block_bias(r, src)  # ring.py:107 (a callable's dense block is built here)
            with timer.span("fwd", r, src):
                fwd_block(qr, _shard_bhld(k, src, Lk), _shard_bhld(v, src, Lk), bias, o, m, l, sm_scale)
            if carries_out is not None:
                carries_out.append((r, t, o.clone(), m.clone(), l.clone()))
        finalize_carry(o, m, l, _shard_bhld(out, r, Lq), lse[r])
    return out, lse


_PLAN_CACHE: "collections.OrderedDict" = collections.OrderedDict()
_PLAN_CACHE_SIZE = 8


def clear_plan_cache() -> None:
    """Drop the cached ring plans (and the references to bias arrays that they hold)."""
    _PLAN_CACHE.clear()


def _plan_for(q, k, n, bias_fn, q_kwargs, kv_kwargs) -> "_RingPlan":
    """The ``_RingPlan`` of a call, from a small cache: a plan (shard offsets read back from the
    position arrays, id arrays converted to int32, the parameter blocks of the whole-ring
    launches) depends on shapes, the ring size and the bias arrays only, so a caller who repeats a
    call - a training loop - pays for it once.  A bias array is identified by the tensor object and
    its version counter; the cache entry keeps the object alive, so its identity cannot be taken
    over by another tensor, and an in-place change gives a new version and a new plan."""
    def ident(t):
        return (id(t), t._version) if isinstance(t, torch.Tensor) else ("v", t)

    fn_key = bias_fn
    if isinstance(bias_fn, BiasFn):
        fn_key = (bias_fn.causal, bias_fn.window, bias_fn.segments, bias_fn.prefix,
                  None if bias_fn.alibi_slopes is None else ident(bias_fn.alibi_slopes))
    elif bias_fn is not None:
        fn_key = ("callable", id(bias_fn))
    kw_key = tuple(tuple(sorted((a, ident(t)) for a, t in (kw or {}).items())) for kw in (q_kwargs, kv_kwargs))
    key = (tuple(q.shape), tuple(k.shape), str(q.device), n, fn_key, kw_key)
    hit = _PLAN_CACHE.get(key)
    if hit is not None:
        _PLAN_CACHE.move_to_end(key)
        return hit[0]
    plan = _RingPlan(q, k, n, bias_fn, q_kwargs, kv_kwargs)
    _PLAN_CACHE[key] = (plan, bias_fn, dict(q_kwargs or {}), dict(kv_kwargs or {}))
    while len(_PLAN_CACHE) > _PLAN_CACHE_SIZE:
        _PLAN_CACHE.popitem(last=False)
    return plan


# A callable's dense blocks are [b, h | 1, lq, lk] fp32 each: the several-step launches below take
# as many of them per launch as fit this many bytes (and at most 16, what one launch walks).
_DENSE_BLOCKS_BYTES = 1 << 30


def _row_chunks(plan: "_RingPlan", r: int):
    """The ring steps of query shard r in ring order, in chunks whose dense blocks are alive
    together: lists of (key/value shard, BlockBias)."""
    n = plan.n
    chunk, used = [], 0
    for t in range(n):
        src = (r - t) % n  # ring.py:51-55
        bias = plan.block_bias(r, src)
        size = bias.dense.numel() * 4 if bias is not None and bias.dense is not None else 0
        if chunk and (len(chunk) == 16 or used + size > _DENSE_BLOCKS_BYTES):
            yield chunk
            chunk, used = [], 0
        chunk.append((src, bias))
        used += size
    if chunk:
        yield chunk


def _ring_forward_rows(q, k, v, plan: "_RingPlan", sm_scale, out_dtype, timer=_NO_TIMER):
    """The several-step launch scheme for a callable ``bias_fn``: one query shard at a time, its
    ring steps in launches of up to 16 (``ra_fwd_steps``, the step's running state in registers
    between the shards), so that only the dense blocks of one launch are alive."""
    n, B, H, D, Lq, Lk = plan.n, plan.B, plan.H, plan.D, plan.Lq, plan.Lk
    dev = q.device
    out = torch.empty((B, n * Lq, H, D), dtype=out_dtype, device=dev)
    lse = torch.empty((n, B, H, Lq), dtype=torch.float32, device=dev)
    o, m, l = init_carry(B, H, Lq, D, dev)
    for r in range(n):
        if r:
            reset_carry(o, m, l)
        qr = _shard_bhld(q, r, Lq)
        for chunk in _row_chunks(plan, r):
            with timer.span("fwd_ring", r, -1):
                fwd_blocks(qr, [(_shard_bhld(k, s, Lk), _shard_bhld(v, s, Lk)) for s, _ in chunk],
                           [b for _, b in chunk], o, m, l, sm_scale)
        finalize_carry(o, m, l, _shard_bhld(out, r, Lq), lse[r])
    return out, lse


def _ring_backward_rows(q, k, v, out, lse, do, plan: "_RingPlan", sm_scale, timer=_NO_TIMER):
    """Backward twin of ``_ring_forward_rows``: every dense block is built ONCE and serves both
    halves of its step - the dQ product of its query shard (one launch per chunk of blocks,
    ``ra_bwd_dq_steps``) and the dK / dV products of its key/value shard (one launch per block,
    into that shard's fp32 accumulators)."""
    n, B, H, D, Lq, Lk = plan.n, plan.B, plan.H, plan.D, plan.Lq, plan.Lk
    dev = q.device
    delta = torch.empty((n, B, H, Lq), dtype=torch.float32, device=dev)
    for s in range(n):
        precompute_delta(_shard_bhld(out, s, Lq), _shard_bhld(do, s, Lq), delta[s])
    dq_acc = torch.empty((B, H, Lq, D), dtype=torch.float32, device=dev)
    dkv_acc = torch.zeros((2, n, B, H, Lk, D), dtype=torch.float32, device=dev)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    for r in range(n):
        dq_acc.zero_()
        qr, dor = _shard_bhld(q, r, Lq), _shard_bhld(do, r, Lq)
        for chunk in _row_chunks(plan, r):
            args = [(qr, _shard_bhld(k, s, Lk), _shard_bhld(v, s, Lk), dor, lse[r], delta[r], dq_acc,
                     dkv_acc[0, s], dkv_acc[1, s], b) for s, b in chunk]
            with timer.span("bwd_dq_ring", r, -1):
                _bwd_steps("dq", args, sm_scale)
            for a in args:
                with timer.span("bwd_dkdv", r, -1):
                    _bwd_step(*a, sm_scale, parts=1)
        _finalize_grad(dq_acc, _shard_bhld(dq, r, Lq))
    for s in range(n):
        _finalize_grad(dkv_acc[0, s], _shard_bhld(dk, s, Lk))
        _finalize_grad(dkv_acc[1, s], _shard_bhld(dv, s, Lk))
    return dq, dk, dv


def _pass_steps(plan: "_RingPlan", cache_key, key, build):
    """The parameter blocks of all ring passes of one kind, built once per plan and set of input
    tensors: only the pointers of buffers allocated per call are patched afterwards."""
    cache = plan.__dict__.setdefault("_step_cache", {})
    hit = cache.get(cache_key)
    if hit is None or hit[0] != key:
        hit = (key,) + build()
        cache[cache_key] = hit
    return hit[1:]


def _ring_forward_fused(q, k, v, plan: _RingPlan, sm_scale, out_dtype, timer=_NO_TIMER, whole=True):
    """``_ring_forward`` with ALL ring passes in one launch: grid dimension y is the query shard,
    and the kernel visits that shard's key/value shards in ring order itself.  ``whole``: the one
    launch is everything (ra_fwd_ring: the carry of ring.py:104-132 stays in registers, output and
    logsumexp come out finished); a ring too large for that, or ``whole=False``, takes three
    launches: carry reset, the ring (ra_fwd_passes), finalisation."""
    if plan.callable is not None:
        return _ring_forward_rows(q, k, v, plan, sm_scale, out_dtype, timer)
    n, B, H, D, Lq, Lk = plan.n, plan.B, plan.H, plan.D, plan.Lq, plan.Lk
    dev = q.device
    lib = _lib.load()
    out = torch.empty((B, n * Lq, H, D), dtype=out_dtype, device=dev)
    lse = torch.empty((n, B, H, Lq), dtype=torch.float32, device=dev)
    dt = {torch.bfloat16: _lib.RA_DTYPE_BF16, torch.float32: _lib.RA_DTYPE_F32}[out.dtype]
    ov = out.permute(0, 2, 1, 3)  # [b, h, S, d] view; shard r starts r * Lq rows further

    def build():
        steps = (_lib.RaFwdStepParams * (n * n))()
        keep = []  # the bias structs point into tensors that must outlive the calls
        for r in range(n):
            for t in range(n):
                src = (r - t) % n  # ring.py:51-55
                bias = plan.block_bias(r, src)
                keep.append(bias)
                steps[r * n + t] = _fwd_params(_shard_bhld(q, r, Lq), _shard_bhld(k, src, Lk), _shard_bhld(v, src, Lk),
                                               bias, None, None, None, sm_scale)  # carry pointers: set per call
        return steps, (C.c_int32 * n)(*([n] * n)), keep

    key = (q.data_ptr(), k.data_ptr(), v.data_ptr(), q.stride(), k.stride(), v.stride(), sm_scale)
    steps, counts, _keep = _pass_steps(plan, "fwd", key, build)
    if whole:
        with timer.span("fwd_ring", -1, -1):
            rc = lib.ra_fwd_ring(steps, counts, n, out.data_ptr(), dt, Lq * ov.stride(2), ov.stride(0), ov.stride(1),
                                 ov.stride(2), lse.data_ptr(), _stream())
        if rc != _lib.RA_ERR_TOO_LARGE:
            _lib.check("ra_fwd_ring", rc)
            return out, lse
    o = torch.empty((n, B, H, Lq, D), dtype=torch.float32, device=dev)
    m = torch.empty((n, B, H, Lq), dtype=torch.float32, device=dev)
    l = torch.empty((n, B, H, Lq), dtype=torch.float32, device=dev)
    _lib.check("ra_fwd_init", lib.ra_fwd_init(o.data_ptr(), m.data_ptr(), l.data_ptr(), n * B, H, Lq, D, _stream()))
    so, sm = o[0].numel() * 4, m[0].numel() * 4
    for r in range(n):
        for t in range(n):
            st = steps[r * n + t]
            st.o, st.m, st.l = o.data_ptr() + r * so, m.data_ptr() + r * sm, l.data_ptr() + r * sm
    with timer.span("fwd_ring", -1, -1):
        _lib.check("ra_fwd_passes", lib.ra_fwd_passes(steps, counts, n, _stream()))
    _lib.check("ra_fwd_finalize_passes", lib.ra_fwd_finalize_passes(
        o.data_ptr(), m.data_ptr(), l.data_ptr(), out.data_ptr(), dt, Lq * ov.stride(2), ov.stride(0), ov.stride(1),
        ov.stride(2), lse.data_ptr(), n, B, H, Lq, D, _stream()))
    return out, lse


def _ring_backward_fused(q, k, v, out, lse, do, plan: _RingPlan, sm_scale, timer=_NO_TIMER, whole=True):
    """``_ring_backward`` with all passes of a kind in one launch: one for dK / dV (grid dimension y
    is the key/value shard, the kernel visits the query shards in the order they arrive,
    ring.py:195), one for dQ (y is the query shard), behind one delta launch.  ``whole``: the two
    launches store the finished bf16 gradients themselves (ra_bwd_dkdv_ring, ra_bwd_dq_ring); a
    ring too large for that, or ``whole=False``, adds into zeroed fp32 accumulators
    (ra_bwd_*_passes) that three more launches cast."""
    if plan.callable is not None:
        return _ring_backward_rows(q, k, v, out, lse, do, plan, sm_scale, timer)
    n, B, H, D, Lq, Lk = plan.n, plan.B, plan.H, plan.D, plan.Lq, plan.Lk
    dev = q.device
    lib = _lib.load()
    delta = torch.empty((n, B, H, Lq), dtype=torch.float32, device=dev)
    ov, dov = out.permute(0, 2, 1, 3), do.permute(0, 2, 1, 3)
    dt = {torch.bfloat16: _lib.RA_DTYPE_BF16, torch.float32: _lib.RA_DTYPE_F32}[out.dtype]
    do_t = _view_bhld(dov)
    _lib.check("ra_bwd_delta_passes", lib.ra_bwd_delta_passes(
        out.data_ptr(), dt, Lq * ov.stride(2), ov.stride(0), ov.stride(1), ov.stride(2), C.byref(do_t),
        Lq * dov.stride(2), delta.data_ptr(), n, B, H, Lq, D, _stream()))
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)

    def build():
        by_kv = (_lib.RaBwdStepParams * (n * n))()
        by_q = (_lib.RaBwdStepParams * (n * n))()
        keep = []
        for r in range(n):
            for t in range(n):
                # dK / dV: key/value shard r meets query shard (r - t) mod n at step t (ring.py:195);
                # dQ: query shard r meets key/value shard (r + t) mod n at step t of that device
                for arr, qs, ks in ((by_kv, (r - t) % n, r), (by_q, r, (r + t) % n)):
                    bias = plan.block_bias(qs, ks)
                    keep.append(bias)
                    arr[r * n + t] = _bwd_params(_shard_bhld(q, qs, Lq), _shard_bhld(k, ks, Lk), _shard_bhld(v, ks, Lk),
                                                 _shard_bhld(do, qs, Lq), lse[qs], delta[qs], None, None, None,
                                                 bias, sm_scale)  # accumulator pointers: set per call
        pairs = [((r - t) % n, r) for r in range(n) for t in range(n)], [(r, (r + t) % n) for r in range(n) for t in range(n)]
        return by_kv, by_q, pairs, (C.c_int32 * n)(*([n] * n)), keep

    key = (q.data_ptr(), k.data_ptr(), v.data_ptr(), q.stride(), k.stride(), v.stride(), do.stride(), sm_scale)
    by_kv, by_q, pairs, counts, _keep = _pass_steps(plan, "bwd", key, build)
    s_row = lse[0].numel() * 4
    do_shard = Lq * do.stride(1) * do.element_size()
    for arr, pr in zip((by_kv, by_q), pairs):
        for i, (qs, ks) in enumerate(pr):
            st = arr[i]
            st.dout.ptr = do.data_ptr() + qs * do_shard
            st.dout.stride_b, st.dout.stride_h, st.dout.stride_l = do.stride(0), do.stride(2), do.stride(1)
            st.lse, st.delta = lse.data_ptr() + qs * s_row, delta.data_ptr() + qs * s_row
    if whole:
        gq, gk, gv = (g.permute(0, 2, 1, 3) for g in (dq, dk, dv))
        assert gk.stride() == gv.stride()
        with timer.span("bwd_dkdv_ring", -1, -1):
            rc = lib.ra_bwd_dkdv_ring(by_kv, counts, n, dk.data_ptr(), dv.data_ptr(), Lk * gk.stride(2), gk.stride(0),
                                      gk.stride(1), gk.stride(2), _stream())
        if rc != _lib.RA_ERR_TOO_LARGE:
            _lib.check("ra_bwd_dkdv_ring", rc)
            with timer.span("bwd_dq_ring", -1, -1):
                _lib.check("ra_bwd_dq_ring", lib.ra_bwd_dq_ring(by_q, counts, n, dq.data_ptr(), Lq * gq.stride(2),
                                                                gq.stride(0), gq.stride(1), gq.stride(2), _stream()))
            return dq, dk, dv
    dq_acc = torch.zeros((n, B, H, Lq, D), dtype=torch.float32, device=dev)
    dkv_acc = torch.zeros((2, n, B, H, Lk, D), dtype=torch.float32, device=dev)
    s_acc, s_kv = dq_acc[0].numel() * 4, dkv_acc[0, 0].numel() * 4
    for arr, pr in zip((by_kv, by_q), pairs):
        for i, (qs, ks) in enumerate(pr):
            st = arr[i]
            st.dq = dq_acc.data_ptr() + qs * s_acc
            st.dk = dkv_acc.data_ptr() + ks * s_kv
            st.dv = dkv_acc.data_ptr() + (n + ks) * s_kv
    with timer.span("bwd_dkdv_ring", -1, -1):
        _lib.check("ra_bwd_dkdv_passes", lib.ra_bwd_dkdv_passes(by_kv, counts, n, _stream()))
    with timer.span("bwd_dq_ring", -1, -1):
        _lib.check("ra_bwd_dq_passes", lib.ra_bwd_dq_passes(by_q, counts, n, _stream()))
    for acc, g, L in ((dq_acc, dq, Lq), (dkv_acc[0], dk, Lk), (dkv_acc[1], dv, Lk)):
        gv = g.permute(0, 2, 1, 3)
        _lib.check("ra_bwd_finalize_passes", lib.ra_bwd_finalize_passes(
            acc.data_ptr(), g.data_ptr(), L * gv.stride(2), gv.stride(0), gv.stride(1), gv.stride(2), n, B, H, L, D,
            _stream()))
    return dq, dk, dv


def _ring_backward(q, k, v, out, lse, do, plan: _RingPlan, sm_scale, timer=_NO_TIMER):
    n, B, H, D, Lq, Lk = plan.n, plan.B, plan.H, plan.D, plan.Lq, plan.Lk
    dev = q.device
    delta = torch.empty((n, B, H, Lq), dtype=torch.float32, device=dev)
    for s in range(n):
        precompute_delta(_shard_bhld(out, s, Lq), _shard_bhld(do, s, Lq), delta[s])
    dq_acc = torch.zeros((n, B, H, Lq, D), dtype=torch.float32, device=dev)
    dk_acc = torch.empty((B, H, Lk, D), dtype=torch.float32, device=dev)
    dv_acc = torch.empty((B, H, Lk, D), dtype=torch.float32, device=dev)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    for r in range(n):  # device r keeps its key/value shard and dk/dv (ring.py:183-200)
        dk_acc.zero_()
        dv_acc.zero_()
        kr, vr = _shard_bhld(k, r, Lk), _shard_bhld(v, r, Lk)
        for t in range(n):
            src = (r - t) % n  # the query-side shard visiting device r at step t (ring.py:195)
            args = (_shard_bhld(q, src, Lq), kr, vr, _shard_bhld(do, src, Lq), lse[src], delta[src],
                    dq_acc[src], dk_acc, dv_acc, plan.block_bias(src, r), sm_scale)
            if timer.split_bwd:
                with timer.span("bwd_dkdv", src, r):
                    _bwd_step(*args, parts=1)
                with timer.span("bwd_dq", src, r):
                    _bwd_step(*args, parts=2)
            else:
                _bwd_step(*args)
        _finalize_grad(dk_acc, _shard_bhld(dk, r, Lk))
        _finalize_grad(dv_acc, _shard_bhld(dv, r, Lk))
    for s in range(n):
        _finalize_grad(dq_acc[s], _shard_bhld(dq, s, Lq))
    return dq, dk, dv


class _RingAttentionFn(torch.autograd.Function):
    """custom_vjp of the reference (ring.py:214-243): forward saves (q, k, v, o, L)."""

    @staticmethod
    def forward(ctx, q, k, v, plan, sm_scale, out_dtype, fused):
        fwd = _ring_forward_fused if fused else _ring_forward
        out, lse = fwd(q, k, v, plan, sm_scale, out_dtype)
        ctx.save_for_backward(q, k, v, out, lse)
        ctx.plan, ctx.sm_scale, ctx.fused = plan, sm_scale, fused
        ctx.mark_non_differentiable(lse)
        return out, lse

    @staticmethod
    def backward(ctx, do, _dlse):
        q, k, v, out, lse = ctx.saved_tensors
        do = _kernel_ready(do)
        bwd = _ring_backward_fused if ctx.fused else _ring_backward
        dq, dk, dv = bwd(q, k, v, out, lse, do, ctx.plan, ctx.sm_scale)
        return dq, dk, dv, None, None, None, None


def ring_attention_with_lse(q, k, v, axis_name, bias_fn: Union[BiasFn, Callable, None] = None, bias_q_kwargs=None,
                            bias_kv_kwargs=None, sm_scale: Optional[float] = None,
                            block_impl: str = "pallas", out_dtype=None):
    """``ring_attention`` that also returns the logsumexp ``[b, h, S]`` (the ``L`` residual of
    ring.py:135)."""
    if block_impl not in _IMPLS:
        raise ValueError(block_impl)
    if bias_fn is not None and not isinstance(bias_fn, BiasFn) and not callable(bias_fn):
        raise TypeError("bias_fn must be a ring_attention.BiasFn or a callable returning the dense "
                        "[b, h | 1, lq, lk] bias of a block")
    _require_gpu(q)
    _lib.load()
    n = _axis_size(axis_name)
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("q, k, v must be [b, l, h, d]")
    d_true = q.shape[-1]
    if k.shape[-1] != d_true or v.shape[-1] != d_true:
        raise ValueError("q, k and v must share the head dim")
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(d_true)  # ring.py:287-288
    in_dtype = q.dtype
    if out_dtype is None:
        out_dtype = torch.float32 if in_dtype == torch.float32 else torch.bfloat16
    d_pad = 64 if d_true <= 64 else 128
    if d_true > 128:
        raise ValueError("head dims above 128 are not supported")
    if d_pad != d_true:
        pad = (0, d_pad - d_true)
        q, k, v = (torch.nn.functional.pad(x, pad) for x in (q, k, v))
    q, k, v = _kernel_ready(q), _kernel_ready(k), _kernel_ready(v)
    plan = _plan_for(q, k, _walked_ring_size(n, q.shape[1], k.shape[1], bias_fn), bias_fn, bias_q_kwargs,
                     bias_kv_kwargs)
    out, lse = _RingAttentionFn.apply(q, k, v, plan, float(sm_scale), out_dtype,
                                      _launch_whole_ring(block_impl, plan))
    if d_pad != d_true:
        out = out[..., :d_true]
    if in_dtype not in (torch.float32, torch.bfloat16):
        out = out.to(in_dtype)
    lse_full = lse.permute(1, 2, 0, 3).reshape(plan.B, plan.H, plan.n * plan.Lq)
    return out, lse_full


def ring_attention(q, k, v, axis_name, bias_fn: Union[BiasFn, Callable, None] = None, bias_q_kwargs=None,
                   bias_kv_kwargs=None, sm_scale: Optional[float] = None, block_impl: str = "pallas"):
    """Ring attention - general (reference ``ring_attention``, ring.py:246-325).

    Args:
        q, k, v: ``[b, S, h, d]`` global arrays on the GPU (see the module docstring).
        axis_name: ``RingAxis`` / int ring size: how many shards the sequence is cut into.
        bias_fn: optional block-wise attention bias: a ``BiasFn`` description (evaluated inside the
            kernels, masked tiles skipped) or, as in the reference, any callable
            ``bias_fn(**q_kwargs, **kv_kwargs)`` returning the additive ``[b, h | 1, lq, lk]`` block
            of one (query shard, key/value shard) pair; no gradient flows into it (ring.py:243).
        bias_q_kwargs / bias_kv_kwargs: query- / key-aligned ``[b, S, ...]`` arrays the bias needs;
            for a ``BiasFn``: ``q_segment_ids``, ``q_positions``, ``q_prefix_mask`` and their
            ``kv_`` twins.
        sm_scale: softmax scale, 1/sqrt(d) if unspecified.
        block_impl: the reference's ``"pallas"`` (its default, ring.py:255: the library picks the
            launch scheme - the whole ring per launch unless ``bias_fn`` is a callable) and
            ``"jax"`` (one kernel launch per ring step), or the launch schemes by name: ``"hip"``
            (launch per step) and ``"hip_fused"`` (one launch for all ring passes: the kernels walk
            the shards themselves); anything else raises ``ValueError`` as the reference does
            (ring.py:312).  Every value runs the same kernels on the same bf16 operands.
    Returns:
        attention output ``[b, S, h, d]``; differentiable w.r.t. q, k, v.
    """
    out, _ = ring_attention_with_lse(q, k, v, axis_name, bias_fn, bias_q_kwargs, bias_kv_kwargs,
                                     sm_scale, block_impl)
    return out


def ring_self_attention(q, k, v, mesh, pspec=None, sm_scale: Optional[float] = None,
                        causal: bool = False, segment_ids=None, positions=None, prefix_mask=None,
                        block_impl: str = "pallas"):
    """Ring attention for self-attention (reference ``ring_self_attention``, ring.py:328-449).

    Supports full bidirectional attention (default), block-sparse attention via
    ``segment_ids``, causal attention (requires ``positions``) and prefix-LM attention via
    ``prefix_mask`` (requires ``positions``), and their combinations.  ``mesh`` gives the
    ring size (``RingAxis`` or int); ``pspec`` is accepted for signature compatibility."""
    if causal:
        assert positions is not None, "positions are requried for causal attention"
        assert prefix_mask is None, "causal attention does not support prefix_mask"
    if prefix_mask is not None:
        assert positions is not None, "positions are requried for prefixlm attention"
        assert not causal
    fn = BiasFn(causal=causal, segments=segment_ids is not None, prefix=prefix_mask is not None)
    has_bias = causal or segment_ids is not None or prefix_mask is not None
    q_kw = {"q_segment_ids": segment_ids, "q_positions": positions, "q_prefix_mask": prefix_mask}
    kv_kw = {"kv_segment_ids": segment_ids, "kv_positions": positions, "kv_prefix_mask": prefix_mask}
    return ring_attention(q, k, v, mesh, bias_fn=fn if has_bias else None,
                          bias_q_kwargs=q_kw if has_bias else None,
                          bias_kv_kwargs=kv_kw if has_bias else None, sm_scale=sm_scale,
                          block_impl=block_impl)

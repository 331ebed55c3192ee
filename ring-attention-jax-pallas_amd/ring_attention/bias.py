"""Declarative attention-bias terms: the device-side form of the reference's ``bias_fn``.

The reference lets the user pass any ``bias_fn(**bias_q_kwargs, **bias_kv_kwargs)`` that
returns a dense additive ``[b, h, lq, lk]`` block per ring step (ring.py:107,186).  A dense
block is 1 GiB per head at 16k x 16k, so here a bias is DESCRIBED by a ``BiasFn`` object and
evaluated inside the kernels, tile by tile, from token positions and per-token id arrays.
Terms add up exactly as additive biases do (0 / -inf masks and finite ALiBi penalties):

    bias_fn = causal_bias() + segment_bias()              # ring.py:388-397
    bias_fn = prefix_lm_bias() + segment_bias()           # ring.py:399-406
    bias_fn = sliding_window_bias(4096)                   # causal window
    bias_fn = segment_bias() + alibi_bias(slopes)

The per-token arrays keep the reference's kwarg names (ring.py:411-420):
``q_segment_ids`` / ``kv_segment_ids``, ``q_positions`` / ``kv_positions``,
``q_prefix_mask`` / ``kv_prefix_mask``; the q-side ones go into ``bias_q_kwargs`` and the
kv-side ones into ``bias_kv_kwargs``.  Positions are optional: when absent a token's
position is its index in the global sequence.  Positions that are consecutive inside every
shard and equal across the batch cost nothing (the kernels take one offset per shard); any other
positions are honoured by materialising the terms per ring step as a dense block, the slow path
of a callable ``bias_fn``.
"""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Optional

import torch

from . import _lib

# A dense block is handed to the single-step launches together with its summary (one more pass
# over the block, shared by the three kernels of the pair); False: the kernels read all of it.
DENSE_SUMMARY = True


@dataclass(frozen=True)
class BiasFn:
    causal: bool = False
    window: Optional[int] = None
    segments: bool = False
    prefix: bool = False
    alibi_slopes: Optional[torch.Tensor] = None  # [H] float32

    def __add__(self, other: "BiasFn") -> "BiasFn":
        if not isinstance(other, BiasFn):
            return NotImplemented
        if self.window is not None and other.window is not None:
            window = min(self.window, other.window)
        else:
            window = self.window if self.window is not None else other.window
        if self.alibi_slopes is not None and other.alibi_slopes is not None:
            slopes = self.alibi_slopes + other.alibi_slopes
        else:
            slopes = self.alibi_slopes if self.alibi_slopes is not None else other.alibi_slopes
        out = BiasFn(self.causal or other.causal, window, self.segments or other.segments,
                     self.prefix or other.prefix, slopes)
        out.validate()
        return out

    def validate(self) -> None:
        # same rule as ring_self_attention's asserts (ring.py:368-374)
        if self.causal and self.prefix:
            raise ValueError("causal attention does not support prefix_mask")
        if self.window is not None and self.window <= 0:
            raise ValueError("window must be positive")

    @property
    def flags(self) -> int:
        f = 0
        if self.causal:
            f |= _lib.RA_BIAS_CAUSAL
        if self.window is not None:
            f |= _lib.RA_BIAS_WINDOW
        if self.segments:
            f |= _lib.RA_BIAS_SEGMENT
        if self.prefix:
            f |= _lib.RA_BIAS_PREFIX
        if self.alibi_slopes is not None:
            f |= _lib.RA_BIAS_ALIBI
        return f

    @property
    def needs_positions(self) -> bool:
        return self.causal or self.prefix or self.window is not None or self.alibi_slopes is not None


def causal_bias() -> BiasFn:
    """0 where kv_position <= q_position, -inf elsewhere (ring.py:393-397)."""
    return BiasFn(causal=True)


def sliding_window_bias(window: int, causal: bool = True) -> BiasFn:
    """0 where 0 <= q_pos - kv_pos < window (or |q_pos - kv_pos| < window if not causal)."""
    b = BiasFn(causal=causal, window=int(window))
    b.validate()
    return b


def segment_bias() -> BiasFn:
    """0 where q_segment_ids == kv_segment_ids, -inf elsewhere (ring.py:388-391)."""
    return BiasFn(segments=True)


def prefix_lm_bias() -> BiasFn:
    """0 where (q_prefix_mask & kv_prefix_mask) | kv_pos <= q_pos (ring.py:399-406)."""
    return BiasFn(prefix=True)


def alibi_bias(slopes) -> BiasFn:
    """-slopes[h] * |q_pos - kv_pos| added to the scaled scores of head h."""
    return BiasFn(alibi_slopes=torch.as_tensor(slopes, dtype=torch.float32))


def alibi_slopes(num_heads: int) -> torch.Tensor:
    """The geometric slope family 2^(-8 h / H), h = 1..H."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / num_heads) for h in range(num_heads)],
                        dtype=torch.float32)


@dataclass
class BlockBias:
    """A BiasFn bound to ONE (query shard, key/value shard) pair: what ``bias_fn(...)``
    returns for a ring step in the reference, in un-materialised form."""
    fn: BiasFn = BiasFn()
    q_offset: int = 0
    kv_offset: int = 0
    q_segment_ids: Optional[torch.Tensor] = None   # int32 [b, lq]
    kv_segment_ids: Optional[torch.Tensor] = None  # int32 [b, lk]
    q_prefix_mask: Optional[torch.Tensor] = None   # int32 [b, lq]
    kv_prefix_mask: Optional[torch.Tensor] = None  # int32 [b, lk]
    # materialised additive bias [b|1, h|1, lq, lk]: the array the reference's bias_fn returns and
    # its fwd_block / bwd_block take (ring.py:107, ring_kernel.py:127); added to the other terms
    dense: Optional[torch.Tensor] = None

    def to_struct(self, device, summary: bool = True) -> "_lib.RaBias":
        """``summary``: hand a dense block's summary along (built once per block and kept with
        it: the forward step and both halves of the backward step of a pair share it)."""
        s = _lib.RaBias()
        fn = self.fn
        s.flags = fn.flags
        s.window = fn.window or 0
        s.q_offset = int(self.q_offset)
        s.kv_offset = int(self.kv_offset)
        self._keep = []

        def ids(t, name):
            if t is None:
                raise ValueError(f"bias needs {name}")
            if t.dtype != torch.int32 or t.stride(-1) != 1 or t.device != device:
                raise ValueError(f"{name} must be an int32 tensor on {device} with unit inner stride")
            self._keep.append(t)
            return t.data_ptr(), t.stride(0)

        if fn.segments:
            s.q_segment_ids, s.q_segment_stride_b = ids(self.q_segment_ids, "q_segment_ids")
            s.kv_segment_ids, s.kv_segment_stride_b = ids(self.kv_segment_ids, "kv_segment_ids")
        if fn.prefix:
            s.q_prefix, s.q_prefix_stride_b = ids(self.q_prefix_mask, "q_prefix_mask")
            s.kv_prefix, s.kv_prefix_stride_b = ids(self.kv_prefix_mask, "kv_prefix_mask")
        if fn.alibi_slopes is not None:
            sl = fn.alibi_slopes
            if sl.device != device:
                raise ValueError("alibi slopes must be moved to the compute device first")
            self._keep.append(sl)
            s.alibi_slopes = sl.data_ptr()
        if self.dense is not None:
            d = self.dense
            if d.dim() != 4:
                raise ValueError(f"a dense bias must be [b, h, lq, lk], got shape {tuple(d.shape)}")
            if d.device != device:
                raise ValueError(f"the dense bias must live on {device}")
            if d.dtype != torch.float32:
                d = d.to(torch.float32)
            if d.stride(-1) != 1 or d.stride(2) < d.shape[3]:
                d = d.contiguous()
            self._keep.append(d)
            s.flags |= _lib.RA_BIAS_DENSE
            s.dense_bias = d.data_ptr()
            s.dense_stride_b = 0 if d.shape[0] == 1 else d.stride(0)
            s.dense_stride_h = 0 if d.shape[1] == 1 else d.stride(1)
            s.dense_stride_q = d.stride(2)
            if summary and DENSE_SUMMARY and d.is_cuda and max(d.shape[2], d.shape[3]) <= _lib.RA_MAX_SEGMENT_SHARD:
                s.dense_map = self._dense_summary(d, s).data_ptr()
        return s

    def _dense_summary(self, d: torch.Tensor, s: "_lib.RaBias") -> torch.Tensor:
        """One byte per 32 x 32 cell of the block (``ra_dense_map``): the step kernels leave out
        tiles that are -inf throughout and read the block only where it is not zero."""
        key = (d.data_ptr(), tuple(d.shape), tuple(d.stride()), d._version)
        hit = self.__dict__.get("_summary")
        if hit is None or hit[0] != key:
            lib = _lib.load()
            B, H, Lq, Lk = d.shape
            size = lib.ra_dense_map_bytes(s.dense_stride_b, s.dense_stride_h, B, H, Lq, Lk)
            m = torch.empty((size,), dtype=torch.uint8, device=d.device)
            stream = torch.cuda.current_stream(d.device).cuda_stream
            _lib.check("ra_dense_map", lib.ra_dense_map(d.data_ptr(), s.dense_stride_b, s.dense_stride_h,
                                                        s.dense_stride_q, B, H, Lq, Lk, m.data_ptr(), stream))
            hit = (key, m, d)
            self.__dict__["_summary"] = hit
        self._keep.append(hit[1])
        return hit[1]

    def check_dense_shape(self, B: int, H: int, Lq: int, Lk: int) -> None:
        """The broadcasting rule of the reference's block functions: [b, h | 1, lq, lk]
        (ring_kernel.py:136-141); a batch of 1 broadcasts too."""
        if self.dense is None:
            return
        sh = tuple(self.dense.shape)
        if len(sh) != 4 or sh[0] not in (1, B) or sh[1] not in (1, H) or sh[2:] != (Lq, Lk):
            raise ValueError(f"dense bias of shape {sh} does not broadcast to {(B, H, Lq, Lk)}")

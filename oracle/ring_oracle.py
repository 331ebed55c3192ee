"""CPU restatement (numpy) of the reference's ring-attention hot path.

TEST INFRASTRUCTURE ONLY: the shipped package never imports this module.  It is the
checker for the HIP kernels (tests, smoke check) and the timed CPU baseline of the
benchmark.  Every function cites the reference lines it restates
(paths relative to the reference checkout, package ``ring_attention/``).

Two independent statements of the same mathematics live here:

* ``mha_dense`` / ``mha_dense_grads`` - the closed form (dense softmax attention and its
  analytic gradients).  This is the reference's own test oracle (ring_test.py:26-42) and
  is what pins everything else.
* ``fwd_block`` / ``bwd_block`` / ``ring_attention`` / ``ring_attention_bwd`` - the
  blockwise ring algorithm with the (o, m, l) online-softmax carry, restating
  ring.py:58-76, :104-137, :140-157, :183-211 step for step, including the ring order
  (device r at step t holds the shard that started on device (r - t) mod n,
  ring.py:51-55) and the -inf guards.

How each function is pinned (tests/test_oracle.py):
  mha_dense            scipy.special.softmax / logsumexp; hand-computed 2x2 case
  mha_dense_grads      torch.autograd in fp64 on an independent dense formula;
                       central finite differences on tiny inputs
  fwd_block            prefix invariant against mha_dense restricted to the visited keys;
                       hand-built all-masked first block (guards ring.py:66,69)
  ring_attention       equals mha_dense for every ring size / odd cross-attention shape
                       of the reference's tests (ring_test.py:48-53)
  bwd_block, ring_attention_bwd   equal mha_dense_grads (ring_test.py:104-111 shapes)
  bias builders        brute-force per-element predicate loops on small inputs
The reference holds no golden vectors (its expected values are computed in-test by the
dense formula), and its random inputs come from jax.random which is absent here, so
"same seeded inputs" means this module's ``make_inputs`` fed to both sides.
"""
from __future__ import annotations

import math
from typing import Callable

import numpy as np

NEG_INF = -np.inf


# --------------------------------------------------------------------------------------
# inputs
# --------------------------------------------------------------------------------------
def bf16_round(x: np.ndarray) -> np.ndarray:
    """Round fp32 values to the nearest bfloat16 (ties to even); result stays fp32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    u = (u + 0x7FFF + lsb) & 0xFFFF0000
    out = u.astype(np.uint32).view(np.float32).reshape(x.shape)
    return np.where(np.isfinite(x), out, x)


def make_inputs(seed, batch, q_len, kv_len, heads, dim, std=1.0, with_do=True, bf16=True):
    """q, k, v (and dO) ~ N(0, std^2) in the public [b, l, h, d] layout
    (shapes as ring_test.py:70-72,133), optionally rounded to bf16-representable fp32."""
    rng = np.random.default_rng(seed)
    shp_q = (batch, q_len, heads, dim)
    shp_kv = (batch, kv_len, heads, dim)
    q = (rng.standard_normal(shp_q, dtype=np.float32) * np.float32(std))
    k = (rng.standard_normal(shp_kv, dtype=np.float32) * np.float32(std))
    v = (rng.standard_normal(shp_kv, dtype=np.float32) * np.float32(std))
    do = rng.standard_normal(shp_q, dtype=np.float32) if with_do else None
    if bf16:
        q, k, v = bf16_round(q), bf16_round(k), bf16_round(v)
        if do is not None:
            do = bf16_round(do)
    return q, k, v, do


def geometric_segment_ids(seed, batch, length, mean_len):
    """Packed-document segment ids: consecutive runs whose lengths are geometric with the
    given mean, truncated at ``length`` (ids are non-decreasing along the sequence)."""
    rng = np.random.default_rng(seed)
    out = np.zeros((batch, length), dtype=np.int32)
    for b in range(batch):
        pos, sid = 0, 0
        while pos < length:
            n = int(rng.geometric(1.0 / mean_len))
            out[b, pos:pos + n] = sid
            pos += n
            sid += 1
    return out


def alibi_slopes(heads):
    """Per-head ALiBi slopes 2^(-8 h / H), h = 1..H."""
    return np.array([2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)], dtype=np.float64)


# --------------------------------------------------------------------------------------
# bias builders  (dense materialisation, as the reference's bias_fn does per ring step)
# --------------------------------------------------------------------------------------
def make_bias_fn(causal=False, window=None, alibi=None, use_segments=False, use_prefix=False):
    """Returns bias_fn(**q_kwargs, **kv_kwargs) -> additive bias [b, h|1, lq, lk].

    Mask part restates ring.py:376-409: segment equality (:388-391), causal
    kv_pos <= q_pos (:393-397), prefix-LM (q_pref & kv_pref) | causal (:399-406),
    encoded as where(mask, 0, -inf)[:, None] (:408-409).  The sliding window
    (0 <= q_pos - kv_pos < window) and ALiBi (-slope_h * |q_pos - kv_pos|) terms are not in
    the reference; they enter through the same additive-bias contract.
    """
    slopes = None if alibi is None else np.asarray(alibi, dtype=np.float64)

    def bias_fn(q_segment_ids=None, kv_segment_ids=None, q_positions=None,
                kv_positions=None, q_prefix_mask=None, kv_prefix_mask=None):
        mask = None

        def _and(a, b):
            return b if a is None else (a & b)

        if use_segments:
            mask = _and(mask, q_segment_ids[:, :, None] == kv_segment_ids[:, None, :])
        if causal or window is not None or use_prefix or slopes is not None:
            qp = q_positions[:, :, None].astype(np.int64)
            kp = kv_positions[:, None, :].astype(np.int64)
        if causal:
            mask = _and(mask, kp <= qp)
        elif use_prefix:
            pm = q_prefix_mask[:, :, None].astype(bool) & kv_prefix_mask[:, None, :].astype(bool)
            mask = _and(mask, pm | (kp <= qp))
        if window is not None:
            w = (qp - kp < window)
            if not causal:
                w = w & (kp - qp < window)
            mask = _and(mask, w)
        if mask is None:
            b_, lq = q_positions.shape if q_positions is not None else q_segment_ids.shape
            lk = (kv_positions if kv_positions is not None else kv_segment_ids).shape[1]
            bias = np.zeros((b_, 1, lq, lk))
        else:
            bias = np.where(mask, 0.0, NEG_INF)[:, None, :, :]
        if slopes is not None:
            bias = bias - slopes[None, :, None, None] * np.abs(qp - kp)[:, None, :, :]
        return bias

    return bias_fn


# --------------------------------------------------------------------------------------
# closed form: dense attention and its gradients  (ring_test.py:26-42)
# --------------------------------------------------------------------------------------
def _heads(x):  # [b l h d] -> [b h l d]
    return np.transpose(x, (0, 2, 1, 3))


def mha_dense(q, k, v, bias=None, sm_scale=None, dtype=np.float64):
    """softmax(q k^T * sm_scale + bias) v.  Inputs [b, l, h, d]; bias [b, h|1, lq, lk].
    Returns (out [b, lq, h, d], lse [b, h, lq]).  Rows whose every score is -inf give NaN
    output and -inf lse, as the reference's softmax does."""
    q, k, v = (np.asarray(a, dtype=dtype) for a in (q, k, v))
    B, Lq, H, D = q.shape
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    out = np.empty((B, Lq, H, v.shape[-1]), dtype=dtype)
    lse = np.empty((B, H, Lq), dtype=dtype)
    for b in range(B):
        for h in range(H):
            s = (q[b, :, h] @ k[b, :, h].T) * sm_scale
            if bias is not None:
                s = s + bias[b, h if bias.shape[1] > 1 else 0]
            m = s.max(axis=-1, keepdims=True)
            with np.errstate(invalid="ignore", divide="ignore"):
                p = np.exp(s - m)
                l = p.sum(axis=-1, keepdims=True)
                out[b, :, h] = (p @ v[b, :, h]) / l
                # a row with no visible key: m = -inf, and ring.py:135 yields -inf + log(0) = -inf
                lse[b, h] = np.where(np.isneginf(m), NEG_INF, m + np.log(l))[:, 0]
    return out, lse


def mha_dense_grads(q, k, v, do, bias=None, sm_scale=None, dtype=np.float64):
    """Gradients of sum(do * mha_dense(q, k, v)) w.r.t. q, k, v (what jax.grad returns in
    ring_test.py:135-138), by the analytic softmax vjp."""
    q, k, v, do = (np.asarray(a, dtype=dtype) for a in (q, k, v, do))
    B, Lq, H, D = q.shape
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    dq, dk, dv = np.zeros_like(q), np.zeros_like(k), np.zeros_like(v)
    for b in range(B):
        for h in range(H):
            s = (q[b, :, h] @ k[b, :, h].T) * sm_scale
            if bias is not None:
                s = s + bias[b, h if bias.shape[1] > 1 else 0]
            p = np.exp(s - s.max(axis=-1, keepdims=True))
            p = p / p.sum(axis=-1, keepdims=True)
            g = do[b, :, h]
            dv[b, :, h] = p.T @ g
            dp = g @ v[b, :, h].T
            ds = p * (dp - (p * dp).sum(axis=-1, keepdims=True)) * sm_scale
            dq[b, :, h] = ds @ k[b, :, h]
            dk[b, :, h] = ds.T @ q[b, :, h]
    return dq, dk, dv


# --------------------------------------------------------------------------------------
# blockwise ring algorithm
# --------------------------------------------------------------------------------------
def fwd_block(q, k, v, bias, o, m_prev, l, sm_scale):
    """One ring step of the online softmax, restating ring.py:58-76.
    q [b h lq d], k/v [b h lk d], bias [b h|1 lq lk] or None, o [b h lq d], m_prev/l
    [b h lq].  Returns the unnormalised (o, m, l)."""
    s = np.matmul(q, np.swapaxes(k, -1, -2)) * sm_scale
    if bias is not None:
        s = s + bias
    m = np.maximum(m_prev, s.max(axis=-1))
    with np.errstate(invalid="ignore"):
        correction = np.exp(m_prev - m)
        correction = np.where(np.isneginf(m) & np.isneginf(m_prev), 0.0, correction)
        p = np.exp(s - m[..., None])
        p = np.where(np.isneginf(m)[..., None], 0.0, p)
    pv = np.matmul(p, v)
    o = o * correction[..., None] + pv
    l = correction * l + p.sum(axis=-1)
    return o, m, l


def bwd_block(q, k, v, bias, o, L, do, sm_scale):
    """One ring step of the backward pass, restating ring.py:140-157."""
    s = np.matmul(q, np.swapaxes(k, -1, -2)) * sm_scale
    if bias is not None:
        s = s + bias
    with np.errstate(invalid="ignore"):
        p = np.exp(s - L[..., None])
    dv = np.matmul(np.swapaxes(p, -1, -2), do)
    dp = np.matmul(do, np.swapaxes(v, -1, -2))
    delta = np.sum(do * o, axis=-1, keepdims=True)
    ds = p * (dp - delta) * sm_scale
    dq = np.matmul(ds, k)
    dk = np.matmul(np.swapaxes(ds, -1, -2), q)
    return dq, dk, dv


def _split(x, n, axis):
    return list(np.split(x, n, axis=axis))


def _split_kwargs(kw, n):
    """Shard every [b, l] array of a kwargs dict along l (None entries stay None)."""
    kw = kw or {}
    return [{key: (None if val is None else np.split(val, n, axis=1)[i]) for key, val in kw.items()}
            for i in range(n)]


def ring_attention(q, k, v, ring_size, bias_fn: Callable | None = None, bias_q_kwargs=None,
                   bias_kv_kwargs=None, sm_scale=None, dtype=np.float64, return_carries=False,
                   skip_masked_steps=False):
    """Forward ring attention over ``ring_size`` emulated devices, restating
    ring.py:79-137 (per-device function) under the shard_map of ring_test.py:82-94.

    q [b, Lq, h, d], k/v [b, Lk, h, d] are the GLOBAL arrays; they are cut into
    ``ring_size`` shards along the length axis.  Device r keeps q shard r; at step t it
    holds the kv shard (and kv-side bias kwargs) that started on device (r - t) mod n
    (ring.py:51-55,120).  Carry init ring.py:124-126, finalise ring.py:134-135.

    Returns (out [b, Lq, h, d], lse [b, h, Lq]) and, if asked, the list over devices of
    the per-step unnormalised carries [(o, m, l) after step t].  With
    ``skip_masked_steps`` a step whose bias block is entirely -inf is not executed (it is
    an identity on the carry), which the tests check changes nothing.
    """
    q, k, v = (np.asarray(a, dtype=dtype) for a in (q, k, v))
    n = ring_size
    B, Lq, H, D = q.shape
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)  # ring.py:287-288
    qs = [_heads(x) for x in _split(q, n, 1)]
    ks = [_heads(x) for x in _split(k, n, 1)]
    vs = [_heads(x) for x in _split(v, n, 1)]
    qkw, kvkw = _split_kwargs(bias_q_kwargs, n), _split_kwargs(bias_kv_kwargs, n)
    outs, lses, carries = [], [], []
    for r in range(n):
        lq = qs[r].shape[2]
        o = np.zeros((B, H, lq, vs[0].shape[-1]), dtype=dtype)
        l = np.zeros((B, H, lq), dtype=dtype)
        m = np.full((B, H, lq), NEG_INF, dtype=dtype)
        steps = []
        for t in range(n):
            src = (r - t) % n
            bias = bias_fn(**qkw[r], **kvkw[src]) if bias_fn is not None else None
            if not (skip_masked_steps and bias is not None and np.all(np.isneginf(bias))):
                o, m, l = fwd_block(qs[r], ks[src], vs[src], bias, o, m, l, sm_scale)
            if return_carries:
                steps.append((o.copy(), m.copy(), l.copy()))
        with np.errstate(invalid="ignore", divide="ignore"):
            outs.append(o / l[..., None])
            lses.append(m + np.log(l))
        carries.append(steps)
    out = np.concatenate([np.transpose(x, (0, 2, 1, 3)) for x in outs], axis=1)
    lse = np.concatenate(lses, axis=2)
    if return_carries:
        return out, lse, carries
    return out, lse


def ring_attention_bwd(q, k, v, out, lse, do, ring_size, bias_fn=None, bias_q_kwargs=None,
                       bias_kv_kwargs=None, sm_scale=None, dtype=np.float64):
    """Backward ring pass, restating ring.py:160-211: device r keeps kv shard r and its
    dk/dv accumulators; the query side (q, o, dq, do, L and the q-side bias kwargs)
    rotates, so at step t device r holds the query shard of device (r - t) mod n
    (ring.py:195).  ``out`` [b, Lq, h, d] and ``lse`` [b, h, Lq] are the forward results.
    Returns dq, dk, dv in the public [b, l, h, d] layout."""
    q, k, v, out, do = (np.asarray(a, dtype=dtype) for a in (q, k, v, out, do))
    lse = np.asarray(lse, dtype=dtype)
    n = ring_size
    D = q.shape[-1]
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(D)
    qs = [_heads(x) for x in _split(q, n, 1)]
    ks = [_heads(x) for x in _split(k, n, 1)]
    vs = [_heads(x) for x in _split(v, n, 1)]
    os_ = [_heads(x) for x in _split(out, n, 1)]
    dos = [_heads(x) for x in _split(do, n, 1)]
    Ls = _split(lse, n, 2)
    qkw, kvkw = _split_kwargs(bias_q_kwargs, n), _split_kwargs(bias_kv_kwargs, n)
    dqs = [np.zeros_like(x) for x in qs]
    dks = [np.zeros_like(x) for x in ks]
    dvs = [np.zeros_like(x) for x in vs]
    for r in range(n):
        for t in range(n):
            src = (r - t) % n
            bias = bias_fn(**qkw[src], **kvkw[r]) if bias_fn is not None else None
            dq_, dk_, dv_ = bwd_block(qs[src], ks[r], vs[r], bias, os_[src], Ls[src], dos[src], sm_scale)
            dqs[src] += dq_
            dks[r] += dk_
            dvs[r] += dv_
    cat = lambda xs: np.concatenate([np.transpose(x, (0, 2, 1, 3)) for x in xs], axis=1)
    return cat(dqs), cat(dks), cat(dvs)


def precompute_delta(out, do):
    """delta = rowsum(o * do) in the [b, h, l] layout (ring_kernel.py:387-394, ring.py:151)."""
    return np.transpose(np.sum(np.asarray(out, np.float64) * np.asarray(do, np.float64), axis=-1), (0, 2, 1))


# --------------------------------------------------------------------------------------
# work accounting (closed forms used by the benchmark's FLOP count)
# --------------------------------------------------------------------------------------
def count_unmasked_pairs(bias_fn, bias_q_kwargs, bias_kv_kwargs, heads):
    """Number of (query, key) pairs whose bias is finite, summed over batch and heads."""
    bias = bias_fn(**(bias_q_kwargs or {}), **(bias_kv_kwargs or {}))
    cnt = np.isfinite(bias).sum(axis=(0, 2, 3))
    return int(cnt.sum() * (heads if bias.shape[1] == 1 else 1))

"""Pins the CPU oracle (oracle/ring_oracle.py) without the reference (jax is absent):
library routines (scipy softmax/logsumexp, torch.autograd in fp64), finite differences,
hand-computed cases and invariants.  Shapes and tolerances follow the reference's tests
(ring_test.py:45-98, :101-171, :174-300, :320-378)."""
import glob
import os

import numpy as np
import pytest
import scipy.special
import torch

from oracle import ring_oracle as R

FWD_SHAPES = [(0, 24, 16, 1, 2), (1, 128, 64, 4, 64), (2, 64, 512, 4, 16), (3, 2048, 2048, 4, 128)]
BWD_SHAPES = [(0, 24, 16, 1, 2), (1, 128, 64, 4, 64), (2, 64, 512, 4, 16), (3, 128, 2048, 2, 128),
              (3, 2048, 128, 2, 128), (3, 512, 512, 4, 128)]


def _torch_mha(q, k, v, bias, sm_scale):
    s = torch.einsum("bihd,bjhd->bhij", q, k) * sm_scale
    if bias is not None:
        s = s + bias
    return torch.einsum("bhij,bjhd->bihd", torch.softmax(s, dim=-1), v)


def test_bf16_round_matches_torch():
    x = np.random.default_rng(0).standard_normal(10000).astype(np.float32) * 3
    x[:4] = [0.0, -0.0, 1.0039062, 65504.0]
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    np.testing.assert_array_equal(R.bf16_round(x), want)


def test_dense_hand_case():
    # one query, two keys, scores ln(1) and ln(3): weights 1/4, 3/4
    q = np.array([[[[1.0, 0.0]]]])
    k = np.array([[[[0.0, 0.0]], [[np.log(3.0), 5.0]]]])
    v = np.array([[[[4.0, 0.0]], [[0.0, 8.0]]]])
    out, lse = R.mha_dense(q, k, v, sm_scale=1.0)
    np.testing.assert_allclose(out[0, 0, 0], [1.0, 6.0], rtol=1e-12)
    np.testing.assert_allclose(lse[0, 0, 0], np.log(4.0), rtol=1e-12)


@pytest.mark.parametrize("seed,q_len,kv_len,h,d", FWD_SHAPES[:3])
def test_dense_against_scipy(seed, q_len, kv_len, h, d):
    q, k, v, _ = R.make_inputs(seed, 2, q_len, kv_len, h, d, bf16=False)
    out, lse = R.mha_dense(q, k, v)
    s = np.einsum("bihd,bjhd->bhij", q.astype(np.float64), k.astype(np.float64)) / np.sqrt(d)
    want = np.einsum("bhij,bjhd->bihd", scipy.special.softmax(s, axis=-1), v.astype(np.float64))
    np.testing.assert_allclose(out, want, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(lse, scipy.special.logsumexp(s, axis=-1), rtol=1e-10)


@pytest.mark.parametrize("seed,q_len,kv_len,h,d", BWD_SHAPES[:3])
def test_dense_grads_against_autograd(seed, q_len, kv_len, h, d):
    q, k, v, do = R.make_inputs(seed, 2, q_len, kv_len, h, d, bf16=False)
    seg_q = np.random.default_rng(seed).integers(0, 3, (2, q_len))
    seg_k = np.random.default_rng(seed + 1).integers(0, 3, (2, kv_len))
    seg_k[:, 0] = seg_q[:, 0]
    bias = np.where(seg_q[:, :, None] == seg_k[:, None, :], 0.0, -1e30)[:, None]  # finite: no NaN rows
    tq, tk, tv = (torch.tensor(x, dtype=torch.float64, requires_grad=True) for x in (q, k, v))
    (_torch_mha(tq, tk, tv, torch.tensor(bias), 1 / np.sqrt(d)) * torch.tensor(do, dtype=torch.float64)).sum().backward()
    dq, dk, dv = R.mha_dense_grads(q, k, v, do, bias)
    np.testing.assert_allclose(dq, tq.grad.numpy(), rtol=1e-8, atol=1e-10)
    np.testing.assert_allclose(dk, tk.grad.numpy(), rtol=1e-8, atol=1e-10)
    np.testing.assert_allclose(dv, tv.grad.numpy(), rtol=1e-8, atol=1e-10)


def test_dense_grads_finite_differences():
    q, k, v, do = R.make_inputs(5, 1, 3, 4, 1, 2, bf16=False)
    q, k, v, do = (x.astype(np.float64) for x in (q, k, v, do))
    dq, dk, dv = R.mha_dense_grads(q, k, v, do)
    f = lambda q_, k_, v_: float((R.mha_dense(q_, k_, v_)[0] * do).sum())
    eps = 1e-6
    for arr, grad, idx in ((q, dq, 0), (k, dk, 1), (v, dv, 2)):
        for pos in np.ndindex(arr.shape):
            args = [q.copy(), k.copy(), v.copy()]
            args[idx][pos] += eps
            up = f(*args)
            args[idx][pos] -= 2 * eps
            dn = f(*args)
            assert abs((up - dn) / (2 * eps) - grad[pos]) < 1e-6


@pytest.mark.parametrize("seed,q_len,kv_len,h,d", FWD_SHAPES)
def test_ring_forward_equals_dense(seed, q_len, kv_len, h, d):
    # ring_test.py:45-98: 8 devices, tolerance rtol=0.01 atol=0.001 (fp32 there; fp64 here is far tighter)
    q, k, v, _ = R.make_inputs(seed, 2, q_len, kv_len, h, d, bf16=False)
    want, want_lse = R.mha_dense(q, k, v)
    out, lse = R.ring_attention(q, k, v, 8)
    assert not np.isnan(out).any()
    np.testing.assert_allclose(out, want, rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(lse, want_lse, rtol=1e-9, atol=1e-12)
    out32, _ = R.ring_attention(q, k, v, 8, dtype=np.float32)
    np.testing.assert_allclose(out32, want, rtol=0.01, atol=0.001)


@pytest.mark.parametrize("seed,q_len,kv_len,h,d", BWD_SHAPES)
def test_ring_backward_equals_dense(seed, q_len, kv_len, h, d):
    # ring_test.py:101-171: atol=1e-4, rtol=0.01
    q, k, v, do = R.make_inputs(seed, 2, q_len, kv_len, h, d, bf16=False)
    want = R.mha_dense_grads(q, k, v, do)
    out, lse = R.ring_attention(q, k, v, 8)
    got = R.ring_attention_bwd(q, k, v, out, lse, do, 8)
    for g, w in zip(got, want):
        assert not np.isnan(g).any()
        np.testing.assert_allclose(g, w, rtol=1e-8, atol=1e-10)
    out32, lse32 = R.ring_attention(q, k, v, 8, dtype=np.float32)
    got32 = R.ring_attention_bwd(q, k, v, out32, lse32, do, 8, dtype=np.float32)
    for g, w in zip(got32, want):
        np.testing.assert_allclose(g, w, rtol=0.01, atol=1e-4)


@pytest.mark.parametrize("seed,q_len,kv_len,h,d", FWD_SHAPES[:3] + [(3, 512, 512, 4, 128)])
def test_ring_segment_bias(seed, q_len, kv_len, h, d):
    # ring_test.py:174-300: random segment ids in [0, q_len // 5); NaN pattern must match
    q, k, v, do = R.make_inputs(seed, 2, q_len, kv_len, h, d, bf16=False)
    rng = np.random.default_rng(seed)
    qs = rng.integers(0, q_len // 5, (2, q_len)).astype(np.int32)
    ks = rng.integers(0, q_len // 5, (2, kv_len)).astype(np.int32)
    fn = R.make_bias_fn(use_segments=True)
    bias = np.repeat(fn(q_segment_ids=qs, kv_segment_ids=ks), h, axis=1)
    want, _ = R.mha_dense(q, k, v, bias)
    out, lse = R.ring_attention(q, k, v, 8, fn, {"q_segment_ids": qs}, {"kv_segment_ids": ks})
    np.testing.assert_array_equal(np.isnan(out), np.isnan(want))
    np.testing.assert_allclose(out, want, rtol=1e-9, atol=1e-12)
    out_s, lse_s = R.ring_attention(q, k, v, 8, fn, {"q_segment_ids": qs}, {"kv_segment_ids": ks},
                                    skip_masked_steps=True)
    np.testing.assert_array_equal(out, out_s)  # skipping a fully masked step is an exact identity
    np.testing.assert_array_equal(lse, lse_s)
    rows_ok = ~np.isnan(want).any(axis=(2, 3))  # [b, lq] rows that see at least one key
    if rows_ok.all():
        got = R.ring_attention_bwd(q, k, v, out, lse, do, 8, fn, {"q_segment_ids": qs}, {"kv_segment_ids": ks})
        for g, w in zip(got, R.mha_dense_grads(q, k, v, do, bias)):
            np.testing.assert_allclose(g, w, rtol=1e-8, atol=1e-10)


@pytest.mark.parametrize("seed,length,h,d", [(0, 16, 1, 2), (1, 128, 4, 64), (2, 512, 4, 16), (4, 2048, 4, 64)])
def test_ring_self_attention_causal_segments(seed, length, h, d):
    # ring_test.py:320-378: segments in [0, 5), positions = arange, causal
    q, k, v, _ = R.make_inputs(seed, 2, length, length, h, d, bf16=False)
    seg = np.random.default_rng(seed).integers(0, 5, (2, length)).astype(np.int32)
    pos = np.broadcast_to(np.arange(length), (2, length))
    mask = (seg[:, :, None] == seg[:, None, :]) & (np.arange(length)[None, :] <= np.arange(length)[:, None])
    want, _ = R.mha_dense(q, k, v, np.where(mask, 0.0, -np.inf)[:, None])
    fn = R.make_bias_fn(causal=True, use_segments=True)
    out, _ = R.ring_attention(q, k, v, 8, fn, {"q_segment_ids": seg, "q_positions": pos},
                              {"kv_segment_ids": seg, "kv_positions": pos}, skip_masked_steps=True)
    np.testing.assert_allclose(out, want, rtol=1e-9, atol=1e-12)


def test_carry_prefix_invariant_and_ring_order():
    """After step t device r has seen kv shards r, r-1, ..., r-t (mod n): o/l is dense attention
    restricted to those keys, m their row max, m + log l their logsumexp."""
    n, B, L, H, D = 4, 1, 8, 2, 4
    q, k, v, _ = R.make_inputs(7, B, n * L, n * L, H, D, bf16=False)
    _, _, carries = R.ring_attention(q, k, v, n, return_carries=True)
    for r in range(n):
        seen = []
        for t in range(n):
            seen.append((r - t) % n)
            idx = np.concatenate([np.arange(s * L, (s + 1) * L) for s in seen])
            qs = q[:, r * L:(r + 1) * L]
            want, want_lse = R.mha_dense(qs, k[:, idx], v[:, idx])
            o, m, l = carries[r][t]
            np.testing.assert_allclose(np.transpose(o / l[..., None], (0, 2, 1, 3)), want, rtol=1e-10)
            np.testing.assert_allclose(m + np.log(l), want_lse, rtol=1e-10)
            s = np.einsum("bihd,bjhd->bhij", qs.astype(np.float64), k[:, idx].astype(np.float64)) / np.sqrt(D)
            np.testing.assert_allclose(m, s.max(axis=-1), rtol=1e-13)


def test_fwd_block_guards_all_masked_first_block():
    """ring.py:66,69: a block whose bias is all -inf on a fresh carry must leave (o, m, l) =
    (0, -inf, 0) without NaN, and the next block must behave as if it were the first."""
    q, k, v, _ = R.make_inputs(3, 1, 4, 6, 1, 2, bf16=False)
    qh, kh, vh = (np.transpose(x, (0, 2, 1, 3)).astype(np.float64) for x in (q, k, v))
    o = np.zeros((1, 1, 4, 2)); m = np.full((1, 1, 4), -np.inf); l = np.zeros((1, 1, 4))
    bias = np.full((1, 1, 4, 6), -np.inf)
    o1, m1, l1 = R.fwd_block(qh, kh, vh, bias, o, m, l, 0.5)
    assert not np.isnan(o1).any() and np.all(o1 == 0) and np.all(l1 == 0) and np.all(np.isneginf(m1))
    o2, m2, l2 = R.fwd_block(qh, kh, vh, None, o1, m1, l1, 0.5)
    o3, m3, l3 = R.fwd_block(qh, kh, vh, None, o, m, l, 0.5)
    np.testing.assert_array_equal(o2, o3); np.testing.assert_array_equal(m2, m3); np.testing.assert_array_equal(l2, l3)
    # partially masked rows: row 0 sees nothing in block 1, everything in block 2
    bias = np.zeros((1, 1, 4, 6)); bias[0, 0, 0, :] = -np.inf
    o4, m4, l4 = R.fwd_block(qh, kh, vh, bias, o, m, l, 0.5)
    assert np.isneginf(m4[0, 0, 0]) and l4[0, 0, 0] == 0 and not np.isnan(o4).any()
    o5, m5, l5 = R.fwd_block(qh, kh, vh, None, o4, m4, l4, 0.5)
    np.testing.assert_allclose((o5 / l5[..., None])[0, 0, 0], (o3 / l3[..., None])[0, 0, 0], rtol=1e-12)


def test_visiting_order_does_not_matter():
    q, k, v, _ = R.make_inputs(9, 1, 32, 32, 2, 8, bf16=False)
    a, la = R.ring_attention(q, k, v, 4)
    b, lb = R.ring_attention(q, k, v, 1)
    np.testing.assert_allclose(a, b, rtol=1e-12)
    np.testing.assert_allclose(la, lb, rtol=1e-12)


@pytest.mark.parametrize("causal,window,prefix,segments,alibi", [
    (True, None, False, False, False), (True, 5, False, True, False), (False, 4, False, False, True),
    (False, None, True, True, False), (True, None, False, False, True), (False, None, False, True, True)])
def test_bias_builders_brute_force(causal, window, prefix, segments, alibi):
    B, Lq, Lk, H = 2, 9, 11, 3
    rng = np.random.default_rng(1)
    qp = rng.integers(0, 12, (B, Lq)); kp = rng.integers(0, 12, (B, Lk))
    qs = rng.integers(0, 3, (B, Lq)); ks = rng.integers(0, 3, (B, Lk))
    qm = rng.integers(0, 2, (B, Lq)); km = rng.integers(0, 2, (B, Lk))
    slopes = R.alibi_slopes(H) if alibi else None
    fn = R.make_bias_fn(causal=causal, window=window, alibi=slopes, use_segments=segments, use_prefix=prefix)
    got = fn(q_segment_ids=qs, kv_segment_ids=ks, q_positions=qp, kv_positions=kp, q_prefix_mask=qm,
             kv_prefix_mask=km)
    got = np.broadcast_to(got, (B, H, Lq, Lk))
    for b in range(B):
        for h in range(H):
            for i in range(Lq):
                for j in range(Lk):
                    ok = True
                    if segments:
                        ok &= qs[b, i] == ks[b, j]
                    if causal:
                        ok &= kp[b, j] <= qp[b, i]
                    elif prefix:
                        ok &= bool(qm[b, i] and km[b, j]) or kp[b, j] <= qp[b, i]
                    if window is not None:
                        ok &= (qp[b, i] - kp[b, j] < window) and (causal or kp[b, j] - qp[b, i] < window)
                    want = 0.0 if ok else -np.inf
                    if alibi and ok:
                        want = -slopes[h] * abs(int(qp[b, i]) - int(kp[b, j]))
                    assert got[b, h, i, j] == want or (not ok and np.isneginf(got[b, h, i, j]))


def test_alibi_slopes_and_segments_generator():
    np.testing.assert_allclose(R.alibi_slopes(8), [2.0 ** -(i + 1) for i in range(8)])
    np.testing.assert_allclose(R.alibi_slopes(16)[[0, 15]], [2 ** -0.5, 2 ** -8])
    seg = R.geometric_segment_ids(0, 2, 4096, 64)
    assert seg.shape == (2, 4096) and (np.diff(seg, axis=1) >= 0).all() and (np.diff(seg, axis=1) <= 1).all()
    assert 30 < 4096 / (seg[0, -1] + 1) < 130


def test_precompute_delta():
    q, k, v, do = R.make_inputs(2, 1, 8, 8, 2, 4, bf16=False)
    out, _ = R.mha_dense(q, k, v)
    d = R.precompute_delta(out, do)
    assert d.shape == (1, 2, 8)
    np.testing.assert_allclose(d[0, 1, 3], float((out[0, 3, 1] * do[0, 3, 1]).sum()), rtol=1e-12)


def test_count_unmasked_pairs_closed_forms():
    S, W, H = 64, 10, 3
    pos = np.arange(S)[None]
    fn = R.make_bias_fn(causal=True)
    assert R.count_unmasked_pairs(fn, {"q_positions": pos}, {"kv_positions": pos}, H) == H * S * (S + 1) // 2
    fn = R.make_bias_fn(causal=True, window=W)
    assert R.count_unmasked_pairs(fn, {"q_positions": pos}, {"kv_positions": pos}, H) == H * (W * (W + 1) // 2 + (S - W) * W)


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz"))))
def test_oracle_against_golden_fixtures(path):
    """The blockwise ring restatement must reproduce the frozen fixtures."""
    z = np.load(path)
    name = os.path.basename(path)
    B, Lq = z["q"].shape[:2]
    Lk = z["k"].shape[1]
    qpos = np.broadcast_to(np.arange(Lq), (B, Lq)); kpos = np.broadcast_to(np.arange(Lk), (B, Lk))
    fn, qkw, kvkw = None, {}, {}
    if "causal_segments" in name:
        fn = R.make_bias_fn(causal=True, use_segments=True)
        qkw = {"q_positions": qpos, "q_segment_ids": z["seg"]}; kvkw = {"kv_positions": kpos, "kv_segment_ids": z["seg"]}
    elif "causal" in name:
        fn = R.make_bias_fn(causal=True); qkw = {"q_positions": qpos}; kvkw = {"kv_positions": kpos}
    elif "window_alibi" in name:
        fn = R.make_bias_fn(causal=True, window=40, alibi=z["slopes"]); qkw = {"q_positions": qpos}; kvkw = {"kv_positions": kpos}
    n = int(z["ring"])
    out, lse = R.ring_attention(z["q"], z["k"], z["v"], n, fn, qkw, kvkw)
    np.testing.assert_allclose(out, z["out"], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(lse, z["lse"], rtol=1e-5, atol=1e-6)
    got = R.ring_attention_bwd(z["q"], z["k"], z["v"], out, lse, z["do"], n, fn, qkw, kvkw)
    for g, key in zip(got, ("dq", "dk", "dv")):
        np.testing.assert_allclose(g, z[key], rtol=1e-4, atol=1e-5)

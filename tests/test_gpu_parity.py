"""GPU parity tests: the HIP kernels (through the C ABI) against the CPU oracle on the same
seeded inputs.  Tolerances: forward output max-abs error <= 1e-2 and
logsumexp <= 1e-3 for bf16 inputs against the fp64 oracle on the same bf16-rounded values,
dq/dk/dv relative error <= 2e-2 (max|diff| / max|ref| and Frobenius).  Where outputs are small
(long rows, N(0, 0.5^2) inputs) the absolute bound alone would let a large relative error
through, so the output also has to stay within OUT_REL of the largest reference value of its
(batch, head)."""
import glob
import math
import os

import numpy as np
import pytest
import torch

import ring_attention as ra
from oracle import ring_oracle as R
from ring_attention import ring as rr

pytestmark = pytest.mark.gpu

OUT_TOL, LSE_TOL, GRAD_TOL = 1e-2, 1e-3, 2e-2
OUT_REL = 1e-2  # max|out - ref| over a (batch, head) / max|ref| over the same (batch, head)


def _out_rel(out, want):
    """Largest max|diff| / max|ref| over the (batch, head) slices of [b, l, h, d] arrays (NaN rows
    of the reference, fully masked queries, left out)."""
    d = np.where(np.isnan(want), 0.0, np.abs(out - want))
    ref = np.where(np.isnan(want), 0.0, np.abs(want))
    return float((d.max(axis=(1, 3)) / np.maximum(ref.max(axis=(1, 3)), 1e-30)).max())


def _dev(x, device, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(x)).to(device)
    return t.to(dtype) if dtype is not None else t


def _rel(a, b):
    """max|diff| / max|ref| and the Frobenius ratio.  The denominators are floored at 0.05 (per
    element) so that a gradient that is exactly zero in real arithmetic (a window of one key:
    dq = dk = 0) is judged on its absolute size instead of on rounding noise."""
    return (np.abs(a - b).max() / max(np.abs(b).max(), 0.05),
            np.linalg.norm(a - b) / max(np.linalg.norm(b), 0.05 * np.sqrt(b.size)))


def _run_hip(device, q, k, v, do, n, fn, qkw, kvkw, sm_scale=None, impl="hip"):
    tq, tk, tv = (_dev(x, device, torch.bfloat16).requires_grad_(True) for x in (q, k, v))
    tqkw = {a: _dev(b, device) for a, b in (qkw or {}).items()} or None
    tkvkw = {a: _dev(b, device) for a, b in (kvkw or {}).items()} or None
    out, lse = ra.ring_attention_with_lse(tq, tk, tv, n, bias_fn=fn, bias_q_kwargs=tqkw,
                                          bias_kv_kwargs=tkvkw, sm_scale=sm_scale, out_dtype=torch.float32,
                                          block_impl=impl)
    grads = None
    if do is not None:
        out.backward(_dev(do, device, torch.float32))
        grads = tuple(t.grad.float().cpu().numpy() for t in (tq, tk, tv))
    torch.cuda.synchronize()
    return out.detach().cpu().numpy(), lse.cpu().numpy(), grads


def _check(device, name, B, Sq, Sk, H, D, n, fn=None, ofn=None, qkw=None, kvkw=None, std=1.0, seed=0,
           grads=True, impl="hip"):
    print(f"[parity] {name}: B={B} Sq={Sq} Sk={Sk} H={H} D={D} ring={n} seed={seed} impl={impl}", flush=True)
    q, k, v, do = R.make_inputs(seed, B, Sq, Sk, H, D, std=std)
    out, lse, g = _run_hip(device, q, k, v, do if grads else None, n, fn, qkw, kvkw, impl=impl)
    oq, okv = dict(qkw or {}), dict(kvkw or {})
    bias = None
    if ofn is not None:
        oq.setdefault("q_positions", np.broadcast_to(np.arange(Sq), (B, Sq)))
        okv.setdefault("kv_positions", np.broadcast_to(np.arange(Sk), (B, Sk)))
        bias = ofn(**oq, **okv)
    want, want_lse = R.mha_dense(q, k, v, bias)
    np.testing.assert_array_equal(np.isnan(out), np.isnan(want))
    ok = ~np.isnan(want)
    e_out, e_rel = np.abs(out - want)[ok].max(initial=0.0), _out_rel(out, want)
    okl = np.isfinite(want_lse)
    np.testing.assert_array_equal(np.isneginf(lse), np.isneginf(want_lse))
    e_lse = np.abs(lse[okl] - want_lse[okl]).max(initial=0.0)  # (no live query at all: nothing to compare)
    worst = {"out": e_out, "out_rel": e_rel, "lse": e_lse}
    assert e_out <= OUT_TOL and e_rel <= OUT_REL and e_lse <= LSE_TOL, worst
    if grads:
        # Queries that see no key (NaN output, ring.py:134-135) must contribute nothing to dk / dv;
        # the reference gradients are those of the attention over the live queries only (a dead
        # row with a zero bias row and a zero dO row adds exactly nothing), and dq is compared on
        # the live rows.
        live = ok.all(axis=(2, 3))  # [b, lq]
        if not live.all():
            do = np.where(live[:, :, None, None], do, 0.0)
            bias = np.where(live[:, None, :, None], bias, 0.0)
        for got, ref, nm in zip(g, R.mha_dense_grads(q, k, v, do, bias), ("dq", "dk", "dv")):
            if nm == "dq":
                got, ref = got[live], ref[live]
                if got.size == 0:
                    continue
            else:
                assert np.isfinite(got).all(), nm
            mx, fro = _rel(got, ref)
            worst[nm] = max(mx, fro)
            assert mx <= GRAD_TOL and fro <= GRAD_TOL, (nm, mx, fro)
    print("[parity]   worst: " + " ".join(f"{a} {b:.2e}" for a, b in worst.items()), flush=True)
    return worst


# ---- the reference's own test shapes (ring_test.py:48-53, :104-111), 8 shards, B=2 -------------
@pytest.mark.parametrize("seed,q_len,kv_len,h,d", [
    (0, 24, 16, 1, 2), (1, 128, 64, 4, 64), (2, 64, 512, 4, 16), (3, 128, 2048, 2, 128),
    (3, 2048, 128, 2, 128), (3, 2048, 2048, 4, 128)])
def test_reference_shapes_no_bias(device, seed, q_len, kv_len, h, d):
    _check(device, "ref-shape", 2, q_len, kv_len, h, d, 8, seed=seed)


@pytest.mark.parametrize("seed,q_len,kv_len,h,d", [
    (0, 24, 16, 1, 2), (1, 128, 64, 4, 64), (2, 64, 512, 4, 16), (3, 2048, 2048, 4, 128)])
def test_reference_shapes_segment_bias(device, seed, q_len, kv_len, h, d):
    # ring_test.py:174-300: random ids in [0, q_len // 5): rows without a matching key give NaN
    rng = np.random.default_rng(seed)
    qs = rng.integers(0, q_len // 5, (2, q_len)).astype(np.int32)
    ks = rng.integers(0, q_len // 5, (2, kv_len)).astype(np.int32)
    _check(device, "ref-shape-segments", 2, q_len, kv_len, h, d, 8, ra.segment_bias(),
           R.make_bias_fn(use_segments=True), {"q_segment_ids": qs}, {"kv_segment_ids": ks}, seed=seed)


@pytest.mark.parametrize("seed,length,h,d", [(0, 16, 1, 2), (1, 128, 4, 64), (2, 512, 4, 16), (4, 2048, 4, 64)])
def test_reference_shapes_self_attention(device, seed, length, h, d):
    # ring_test.py:320-378: ring_self_attention, causal + segments in [0, 5), positions = arange
    print(f"[parity] self-attention length={length} h={h} d={d}", flush=True)
    q, k, v, _ = R.make_inputs(seed, 2, length, length, h, d)
    seg = np.random.default_rng(seed).integers(0, 5, (2, length)).astype(np.int32)
    pos = np.broadcast_to(np.arange(length), (2, length)).copy()
    out = ra.ring_self_attention(_dev(q, device), _dev(k, device), _dev(v, device), ra.RingAxis("sp", 8), None,
                                 causal=True, segment_ids=_dev(seg, device), positions=_dev(pos, device))
    assert out.dtype == torch.float32 and out.shape == q.shape
    bias = R.make_bias_fn(causal=True, use_segments=True)(
        q_segment_ids=seg, kv_segment_ids=seg, q_positions=pos, kv_positions=pos)
    want, want_lse = R.mha_dense(q, k, v, bias)
    got = out.cpu().numpy()
    assert np.abs(got - want).max() <= OUT_TOL and _out_rel(got, want) <= OUT_REL
    # the logsumexp of the same call: ring_self_attention is ring_attention with this bias (ring.py:376-449)
    seg_t, pos_t = _dev(seg, device), _dev(pos, device)
    out2, lse = ra.ring_attention_with_lse(
        _dev(q, device), _dev(k, device), _dev(v, device), ra.RingAxis("sp", 8),
        bias_fn=ra.causal_bias() + ra.segment_bias(), bias_q_kwargs={"q_segment_ids": seg_t, "q_positions": pos_t},
        bias_kv_kwargs={"kv_segment_ids": seg_t, "kv_positions": pos_t})
    assert torch.equal(out2, out)
    assert np.abs(lse.cpu().numpy() - want_lse).max() <= LSE_TOL


# ---- bias functors --------------------------------------------------------------------------------
def test_causal_c1_config(device):
    # benchmark config 1: B=1 H=4 S=1024 D=64, ring of 4 shards of 256, causal
    _check(device, "C1", 1, 1024, 1024, 4, 64, 4, ra.causal_bias(), R.make_bias_fn(causal=True))


def test_ragged_lengths(device):
    _check(device, "ragged", 1, 200, 136, 2, 128, 1)
    _check(device, "ragged-causal", 2, 3 * 37, 3 * 37, 2, 64, 3, ra.causal_bias(), R.make_bias_fn(causal=True))


def test_causal_d128_ring8(device):
    _check(device, "causal-d128", 2, 2048, 2048, 4, 128, 8, ra.causal_bias(), R.make_bias_fn(causal=True))


@pytest.mark.parametrize("window,causal", [(300, True), (64, True), (1, True), (200, False)])
def test_sliding_window(device, window, causal):
    _check(device, f"window{window}", 1, 2048, 2048, 2, 128, 8, ra.sliding_window_bias(window, causal),
           R.make_bias_fn(causal=causal, window=window), std=0.5)


def test_sorted_segments_and_alibi(device):
    seg = R.geometric_segment_ids(0, 2, 2048, 300)
    _check(device, "segments-sorted", 2, 2048, 2048, 2, 128, 4, ra.segment_bias(),
           R.make_bias_fn(use_segments=True), {"q_segment_ids": seg}, {"kv_segment_ids": seg})
    sl = R.alibi_slopes(4)
    _check(device, "segments+alibi", 1, 2048, 2048, 4, 128, 4, ra.segment_bias() + ra.alibi_bias(sl),
           R.make_bias_fn(use_segments=True, alibi=sl), {"q_segment_ids": seg[:1]}, {"kv_segment_ids": seg[:1]})
    _check(device, "causal+alibi", 1, 1024, 1024, 4, 64, 4, ra.causal_bias() + ra.alibi_bias(sl),
           R.make_bias_fn(causal=True, alibi=sl))


@pytest.mark.parametrize("causal,ring", [(False, 1), (True, 1), (True, 2)])
def test_long_documents(device, causal, ring):
    # documents long enough (dozens of key tiles each, boundaries off the tile grid) for the
    # kernels to switch to their straight-line loops inside a document and back at its end
    S = 6144
    seg = np.zeros((1, S), np.int32)
    seg[0, 2900:5031] = 1
    seg[0, 5031:] = 2
    fn = ra.segment_bias() + ra.causal_bias() if causal else ra.segment_bias()
    _check(device, f"long-documents causal={causal}", 1, S, S, 2, 128, ring, fn,
           R.make_bias_fn(causal=causal, use_segments=True), {"q_segment_ids": seg}, {"kv_segment_ids": seg},
           std=0.7)


@pytest.mark.parametrize("impl", ["hip", "hip_fused"])
@pytest.mark.parametrize("causal,D", [(False, 128), (True, 128), (False, 64)])
def test_documents_and_alibi_inside_the_straight_line_loops(device, impl, causal, D):
    """Documents + ALiBi (C4's bias) on documents long enough for straight-line stretches in all
    three kernels: a document shorter than a workgroup's rows (100 tokens), a workgroup that
    straddles a boundary off the tile grid (two runs of one-id tiles: 1500 lies inside rows
    1280-1535), a document that crosses the shard boundary, ALiBi stretches on both sides of
    the diagonal (not causal) or one (causal), one slope per head."""
    S, H = 4096, 4
    seg = np.zeros((1, S), np.int32)
    seg[0, 100:1500] = 1
    seg[0, 1500:] = 2
    sl = R.alibi_slopes(H)
    fn = ra.segment_bias() + ra.alibi_bias(sl)
    if causal:
        fn = fn + ra.causal_bias()
    _check(device, f"documents+alibi causal={causal} D={D}", 1, S, S, H, D, 2, fn,
           R.make_bias_fn(causal=causal, use_segments=True, alibi=sl), {"q_segment_ids": seg},
           {"kv_segment_ids": seg}, impl=impl)
    # ALiBi alone: every tile off the diagonal band is inside a stretch
    fn = ra.alibi_bias(sl) + ra.causal_bias() if causal else ra.alibi_bias(sl)
    _check(device, f"alibi causal={causal} D={D}", 1, S, S, H, D, 2, fn, R.make_bias_fn(causal=causal, alibi=sl),
           impl=impl, seed=3)


def test_fully_masked_rows_do_not_poison_key_gradients(device):
    # queries whose segment id matches no key: o = NaN, lse = -inf like the reference
    # (ring.py:134-135); such rows must contribute nothing to dk / dv.  The expected gradients
    # are those of the attention restricted to the queries that do see a key.
    print("[parity] fully masked rows: dk / dv stay finite", flush=True)
    B, S, H, D, n = 1, 512, 2, 128, 4
    q, k, v, do = R.make_inputs(11, B, S, S, H, D)
    rng = np.random.default_rng(11)
    ks = rng.integers(0, 3, (B, S)).astype(np.int32)
    qs = rng.integers(0, 4, (B, S)).astype(np.int32)  # id 3 matches no key
    out, lse, g = _run_hip(device, q, k, v, do, n, ra.segment_bias(), {"q_segment_ids": qs},
                           {"kv_segment_ids": ks})
    dead = qs[0] == 3
    assert dead.any() and not dead.all()
    assert np.isnan(out[0, dead]).all() and np.isneginf(lse[0][:, dead]).all()
    live = ~dead
    bias = R.make_bias_fn(use_segments=True)(q_segment_ids=qs[:, live], kv_segment_ids=ks)
    wq, wk, wv = R.mha_dense_grads(q[:, live], k, v, do[:, live], bias)
    dq, dk, dv = g
    assert np.isfinite(dk).all() and np.isfinite(dv).all()
    for got, ref, nm in ((dq[:, live], wq, "dq"), (dk, wk, "dk"), (dv, wv, "dv")):
        mx, fro = _rel(got, ref)
        assert mx <= GRAD_TOL and fro <= GRAD_TOL, (nm, mx, fro)


def test_prefix_lm(device):
    pm = (np.arange(512)[None, :] < np.array([[100], [300]])).astype(np.int32)
    _check(device, "prefix", 2, 512, 512, 2, 64, 4, ra.prefix_lm_bias(), R.make_bias_fn(use_prefix=True),
           {"q_prefix_mask": pm}, {"kv_prefix_mask": pm})
    seg = np.sort(np.random.default_rng(3).integers(0, 3, (2, 512)), axis=1).astype(np.int32)
    _check(device, "prefix+segments", 2, 512, 512, 2, 128, 4, ra.prefix_lm_bias() + ra.segment_bias(),
           R.make_bias_fn(use_prefix=True, use_segments=True),
           {"q_prefix_mask": pm, "q_segment_ids": seg}, {"kv_prefix_mask": pm, "kv_segment_ids": seg})


@pytest.mark.parametrize("impl", ["hip", "hip_fused"])
def test_ring_self_attention_prefix_lm(device, impl):
    """ring_self_attention(prefix_mask=..., positions=...) (ring.py:399-406): bidirectional inside
    the prefix, causal after it, with document ids on top; forward and gradients."""
    B, S, H, D, n = 2, 1024, 2, 128, 4
    q, k, v, do = R.make_inputs(31, B, S, S, H, D)
    pos = np.broadcast_to(np.arange(S), (B, S)).copy()
    pm = (np.arange(S)[None, :] < np.array([[333], [700]])).astype(np.int32) * 7  # any non-zero value marks the prefix
    seg = np.sort(np.random.default_rng(31).integers(0, 3, (B, S)), axis=1).astype(np.int32)
    print(f"[parity] ring_self_attention prefix-LM impl={impl}", flush=True)
    tq, tk, tv = (_dev(x, device, torch.bfloat16).requires_grad_(True) for x in (q, k, v))
    out = ra.ring_self_attention(tq, tk, tv, ra.RingAxis("sp", n), None, segment_ids=_dev(seg, device),
                                 positions=_dev(pos, device), prefix_mask=_dev(pm, device), block_impl=impl)
    out.float().backward(_dev(do, device, torch.float32))
    torch.cuda.synchronize()
    bias = R.make_bias_fn(use_prefix=True, use_segments=True)(
        q_segment_ids=seg, kv_segment_ids=seg, q_positions=pos, kv_positions=pos,
        q_prefix_mask=(pm != 0).astype(np.int32), kv_prefix_mask=(pm != 0).astype(np.int32))
    want, _ = R.mha_dense(q, k, v, bias)
    # the public entry point returns bf16 for bf16 inputs: its rounding (2^-9 relative) comes on top
    assert np.abs(out.detach().float().cpu().numpy() - want).max() <= OUT_TOL + 2.0 ** -9 * np.abs(want).max()
    for t, ref, nm in zip((tq, tk, tv), R.mha_dense_grads(q, k, v, do, bias), ("dq", "dk", "dv")):
        mx, fro = _rel(t.grad.float().cpu().numpy(), ref)
        assert mx <= GRAD_TOL and fro <= GRAD_TOL, (nm, mx, fro)


def test_arbitrary_positions(device):
    """Positions that no per-shard offset can express (strided, shuffled inside a shard, different
    in every batch row) follow the reference's element-wise rule kv_positions <= q_positions
    (ring.py:393-397) through the dense-block path."""
    B, S, n = 2, 512, 4
    rng = np.random.default_rng(17)
    pos = np.stack([rng.permutation(S) * 3, np.arange(S)[::-1].copy()]).astype(np.int64)
    seg = rng.integers(0, 2, (B, S)).astype(np.int32)
    _check(device, "arbitrary-positions causal+segments", B, S, S, 2, 64, n, ra.causal_bias() + ra.segment_bias(),
           R.make_bias_fn(causal=True, use_segments=True), {"q_positions": pos, "q_segment_ids": seg},
           {"kv_positions": pos, "kv_segment_ids": seg})
    sl = R.alibi_slopes(2)
    _check(device, "arbitrary-positions window+alibi", B, S, S, 2, 128, n, ra.sliding_window_bias(200) + ra.alibi_bias(sl),
           R.make_bias_fn(causal=True, window=200, alibi=sl), {"q_positions": pos}, {"kv_positions": pos})


def test_shard_positions_with_offsets(device):
    # positions restart from an arbitrary offset in every shard
    B, S, n = 1, 512, 4
    starts = np.array([1000, 0, 5000, 128])
    pos = (starts[:, None] + np.arange(S // n)[None, :]).reshape(1, S)
    _check(device, "offsets", B, S, S, 2, 64, n, ra.causal_bias(), R.make_bias_fn(causal=True),
           {"q_positions": pos}, {"kv_positions": pos})


# ---- golden fixtures ----------------------------------------------------------------------------------
@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz"))))
def test_golden_fixtures(device, path):
    z = np.load(path)
    name = os.path.basename(path)
    print(f"[parity] golden {name}", flush=True)
    fn, qkw, kvkw = None, None, None
    if "causal_segments" in name:
        fn = ra.causal_bias() + ra.segment_bias()
        qkw, kvkw = {"q_segment_ids": z["seg"]}, {"kv_segment_ids": z["seg"]}
    elif "causal" in name:
        fn = ra.causal_bias()
    elif "window_alibi" in name:
        fn = ra.sliding_window_bias(40) + ra.alibi_bias(z["slopes"])
    out, lse, g = _run_hip(device, z["q"], z["k"], z["v"], z["do"], int(z["ring"]), fn, qkw, kvkw)
    assert np.abs(out - z["out"]).max() <= OUT_TOL
    assert np.abs(lse - z["lse"]).max() <= LSE_TOL
    for got, key in zip(g, ("dq", "dk", "dv")):
        mx, fro = _rel(got, z[key])
        assert mx <= GRAD_TOL and fro <= GRAD_TOL, (key, mx, fro)


# ---- per-step carry semantics ----------------------------------------------------------------------------
def test_per_step_carries_match_oracle(device):
    """(o, m, l) after every ring step equals the oracle's blockwise carry (ring.py:104-132)."""
    B, S, H, D, n = 1, 1024, 2, 64, 4
    q, k, v, _ = R.make_inputs(21, B, S, S, H, D)
    pos = np.broadcast_to(np.arange(S), (B, S))
    _, _, want = R.ring_attention(q, k, v, n, R.make_bias_fn(causal=True), {"q_positions": pos},
                                  {"kv_positions": pos}, return_carries=True)
    tq, tk, tv = (_dev(x, device, torch.bfloat16) for x in (q, k, v))
    plan = rr._RingPlan(tq, tk, n, ra.causal_bias(), None, None)
    got = []
    rr._ring_forward(tq, tk, tv, plan, 1 / math.sqrt(D), torch.float32, carries_out=got)
    torch.cuda.synchronize()
    for r, t, o, m, l in got:
        wo, wm, wl = want[r][t]
        m_, l_, o_ = m.cpu().numpy(), l.cpu().numpy(), o.cpu().numpy()
        np.testing.assert_array_equal(np.isneginf(m_), np.isneginf(wm))
        fin = np.isfinite(wm)
        assert np.abs(m_ - wm)[fin].max() <= 1e-4
        np.testing.assert_allclose(l_, wl, rtol=5e-3, atol=1e-6)
        assert np.abs(o_ - wo).max() <= 1e-2 * max(1.0, np.abs(wo).max())


def test_block_api_matches_reference_contract(device):
    """fwd_block / bwd_block on [b, h, l, d] tensors (ring_kernel.py:123-131, :202-211)."""
    B, H, Lq, Lk, D = 2, 2, 256, 128, 128
    q, k, v, do = R.make_inputs(5, B, Lq, Lk, H, D)
    hq, hk, hv, hdo = (np.ascontiguousarray(np.transpose(x, (0, 2, 1, 3))) for x in (q, k, v, do))
    tq, tk, tv, tdo = (_dev(x, device, torch.bfloat16) for x in (hq, hk, hv, hdo))
    o, m, l = rr.init_carry(B, H, Lq, D, device)
    assert torch.all(o == 0) and torch.all(l == 0) and torch.all(torch.isneginf(m))
    scale = 1 / math.sqrt(D)
    o, m, l = ra.fwd_block(tq, tk, tv, None, o, m, l, scale)
    wo, wm, wl = R.fwd_block(hq.astype(np.float64), hk.astype(np.float64), hv.astype(np.float64), None,
                             np.zeros((B, H, Lq, D)), np.full((B, H, Lq), -np.inf), np.zeros((B, H, Lq)), scale)
    assert np.abs(m.cpu().numpy() - wm).max() <= 1e-4
    np.testing.assert_allclose(l.cpu().numpy(), wl, rtol=5e-3)
    out = (o / l[..., None])
    L = m + torch.log(l)
    dq, dk, dv = ra.bwd_block(tq, tk, tv, None, out, L, tdo, scale)
    wdq, wdk, wdv = R.bwd_block(hq.astype(np.float64), hk.astype(np.float64), hv.astype(np.float64), None,
                                wo / wl[..., None], wm + np.log(wl), hdo.astype(np.float64), scale)
    for got, ref in ((dq, wdq), (dk, wdk), (dv, wdv)):
        mx, fro = _rel(got.cpu().numpy(), ref)
        assert mx <= GRAD_TOL and fro <= GRAD_TOL


def _block_step_against_oracle(device, fn, ofn, q_off, kv_off, Lq, Lk, D, qkw=None, kvkw=None, seed=3, check_m=True):
    """One block step (fwd_block, then bwd_block on its own normalised output) at the given shard
    positions against the oracle's block functions fed the dense bias of explicit positions."""
    B, H = 1, 2
    q, k, v, do = R.make_inputs(seed, B, Lq, Lk, H, D)
    hq, hk, hv, hdo = (np.ascontiguousarray(np.transpose(x, (0, 2, 1, 3))) for x in (q, k, v, do))
    tq, tk, tv, tdo = (_dev(x, device, torch.bfloat16) for x in (hq, hk, hv, hdo))
    qpos = np.broadcast_to(q_off + np.arange(Lq, dtype=np.int64), (B, Lq))
    kpos = np.broadcast_to(kv_off + np.arange(Lk, dtype=np.int64), (B, Lk))
    dense = ofn(**dict(qkw or {}, q_positions=qpos), **dict(kvkw or {}, kv_positions=kpos))  # [b, h | 1, lq, lk]
    dense = np.broadcast_to(dense, (B, H, Lq, Lk)).astype(np.float64)
    if fn.alibi_slopes is not None:
        fn = ra.BiasFn(fn.causal, fn.window, fn.segments, fn.prefix, fn.alibi_slopes.to(device))
    bb = ra.BlockBias(fn, q_off, kv_off, *(None if x is None else _dev(x, device) for x in (
        (qkw or {}).get("q_segment_ids"), (kvkw or {}).get("kv_segment_ids"),
        (qkw or {}).get("q_prefix_mask"), (kvkw or {}).get("kv_prefix_mask"))))
    scale = 1 / math.sqrt(D)
    o, m, l = rr.init_carry(B, H, Lq, D, device)
    o, m, l = ra.fwd_block(tq, tk, tv, bb, o, m, l, scale)
    wo, wm, wl = R.fwd_block(hq.astype(np.float64), hk.astype(np.float64), hv.astype(np.float64), dense,
                             np.zeros((B, H, Lq, D)), np.full((B, H, Lq), -np.inf), np.zeros((B, H, Lq)), scale)
    live = np.isfinite(wm)
    assert live.any()
    np.testing.assert_array_equal(np.isneginf(m.cpu().numpy()), ~live)
    got_out = (o / l[..., None]).cpu().numpy()[live]
    got_lse = (m + torch.log(l)).cpu().numpy()[live]
    want_out, want_lse = (wo / wl[..., None])[live], (wm + np.log(wl))[live]
    e_out, e_lse = np.abs(got_out - want_out).max(), np.abs(got_lse - want_lse).max()
    # |lse| grows with the bias: hold it to the fp32 resolution of its own size on top of the bound
    assert e_out <= OUT_TOL and e_lse <= LSE_TOL + 4e-7 * np.abs(want_lse).max(), (e_out, e_lse)
    if check_m:
        assert np.abs(m.cpu().numpy()[live] - wm[live]).max() <= 1e-4 + 4e-7 * np.abs(wm[live]).max()
    out = torch.nan_to_num(o / l[..., None])
    L = m + torch.log(l)
    dq, dk, dv = ra.bwd_block(tq, tk, tv, bb, out, L, tdo, scale)
    w_out = np.where(live[..., None], wo / np.where(wl == 0, 1, wl)[..., None], 0.0)
    w_do = np.where(live[..., None], hdo.astype(np.float64), 0.0)       # dead rows contribute nothing
    w_L = np.where(live, wm + np.log(np.where(wl == 0, 1, wl)), 0.0)
    w_dense = np.where(live[..., None], dense, 0.0)
    wdq, wdk, wdv = R.bwd_block(hq.astype(np.float64), hk.astype(np.float64), hv.astype(np.float64), w_dense,
                                w_out, w_L, w_do, scale)
    for nm, got, ref in (("dq", dq.cpu().numpy()[live], wdq[live]), ("dk", dk.cpu().numpy(), wdk),
                         ("dv", dv.cpu().numpy(), wdv)):
        mx, fro = _rel(got, ref)
        assert mx <= GRAD_TOL and fro <= GRAD_TOL, (nm, mx, fro)
    return e_out, e_lse


@pytest.mark.parametrize("q_off,kv_off", [(0, rr._lib.RA_MAX_POSITION - 384), (rr._lib.RA_MAX_POSITION - 256, 0),
                                          (1000, 1000 + (1 << 29) + 5), (0, 64)])
def test_prefix_block_step_far_from_the_diagonal(device, q_off, kv_off):
    """A lone block step whose key/value shard lies up to 2^30 positions before or behind the query
    shard (the widest the C ABI takes): behind it only prefix & prefix pairs are unmasked, before
    it every pair is."""
    Lq, Lk = 256, 384
    rng = np.random.default_rng(1)
    qpm = (rng.random((1, Lq)) < 0.5).astype(np.int32)
    kpm = (rng.random((1, Lk)) < 0.5).astype(np.int32)
    _block_step_against_oracle(device, ra.prefix_lm_bias(), R.make_bias_fn(use_prefix=True), q_off, kv_off, Lq, Lk, 64,
                               {"q_prefix_mask": qpm}, {"kv_prefix_mask": kpm})


@pytest.mark.parametrize("q_off,kv_off,causal", [(100000, 0, True), (0, 300000, False), (5000, 4000, False),
                                                 (200000, 0, True)])
def test_alibi_block_step_far_from_the_diagonal(device, q_off, kv_off, causal):
    """ALiBi on a lone block step far from the diagonal: slope x distance reaches 6000 - 19000 (the
    largest slope is 1/16 here), and the weights inside the block must still follow the bias of
    the oracle - the kernels add the term through the matrix unit, the distance-dependent constant
    split into three bf16 words.  (Beyond a few hundred thousand positions fp32 itself - the
    reference's bias dtype - no longer resolves the bias to 1e-3.)"""
    H = 2
    sl = R.alibi_slopes(H)
    fn = ra.alibi_bias(sl) + (ra.causal_bias() if causal else ra.BiasFn())
    _block_step_against_oracle(device, fn, R.make_bias_fn(causal=causal, alibi=sl), q_off, kv_off, 1024, 1024, 128)


# ---- arbitrary bias_fn callables: the dense additive block of ring.py:107 ---------------------------
def _callable_check(device, name, B, Sq, Sk, H, D, n, torch_fn, numpy_fn, qkw, kvkw, seed=0):
    """ring_attention with a Python callable as bias_fn against the dense closed form with the
    same function evaluated by numpy on the whole sequence."""
    print(f"[parity] {name}: B={B} Sq={Sq} Sk={Sk} H={H} D={D} ring={n}", flush=True)
    q, k, v, do = R.make_inputs(seed, B, Sq, Sk, H, D)
    out, lse, g = _run_hip(device, q, k, v, do, n, torch_fn, qkw, kvkw)
    bias = numpy_fn(**qkw, **kvkw)
    want, want_lse = R.mha_dense(q, k, v, bias)
    np.testing.assert_array_equal(np.isnan(out), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.abs(out - want)[ok].max() <= OUT_TOL
    okl = np.isfinite(want_lse)
    assert np.abs(lse[okl] - want_lse[okl]).max() <= LSE_TOL
    if ok.all():
        for got, ref, nm in zip(g, R.mha_dense_grads(q, k, v, do, bias), ("dq", "dk", "dv")):
            mx, fro = _rel(got, ref)
            assert mx <= GRAD_TOL and fro <= GRAD_TOL, (nm, mx, fro)


@pytest.mark.parametrize("seed,q_len,kv_len,h,d", [(1, 128, 64, 4, 64), (2, 64, 512, 4, 16), (3, 2048, 2048, 4, 128)])
def test_callable_segment_bias_fn(device, seed, q_len, kv_len, h, d):
    # the bias_fn of the reference's own test (ring_test.py:226-246): a callable that builds the
    # [b, 1, lq, lk] mask block from the two id arrays
    rng = np.random.default_rng(seed)
    qs = rng.integers(0, 5, (2, q_len)).astype(np.int32)
    ks = rng.integers(0, 5, (2, kv_len)).astype(np.int32)

    def torch_fn(q_segment_ids, kv_segment_ids):
        same = q_segment_ids[:, None, :, None] == kv_segment_ids[:, None, None, :]
        return torch.where(same, 0.0, -torch.inf)

    def numpy_fn(q_segment_ids, kv_segment_ids):
        same = q_segment_ids[:, None, :, None] == kv_segment_ids[:, None, None, :]
        return np.where(same, 0.0, -np.inf)

    _callable_check(device, "callable-segments", 2, q_len, kv_len, h, d, 8, torch_fn, numpy_fn,
                    {"q_segment_ids": qs}, {"kv_segment_ids": ks}, seed=seed)


def test_callable_per_head_finite_bias_fn(device):
    # a finite per-head bias of arbitrary per-token features (not expressible by the built-in
    # terms), ragged shard length, plus a causal mask folded into the same callable
    B, S, H, D, n = 2, 3 * 200, 3, 64, 3
    rng = np.random.default_rng(7)
    qf = rng.standard_normal((B, S, H)).astype(np.float32)
    kf = rng.standard_normal((B, S, H)).astype(np.float32)
    pos = np.broadcast_to(np.arange(S, dtype=np.int32), (B, S)).copy()

    def torch_fn(q_feat, q_pos, kv_feat, kv_pos):
        bias = torch.einsum("bqh,bkh->bhqk", q_feat, kv_feat)
        return bias.masked_fill(kv_pos[:, None, None, :] > q_pos[:, None, :, None], -torch.inf)

    def numpy_fn(q_feat, q_pos, kv_feat, kv_pos):
        bias = np.einsum("bqh,bkh->bhqk", q_feat.astype(np.float64), kv_feat.astype(np.float64))
        return np.where(kv_pos[:, None, None, :] > q_pos[:, None, :, None], -np.inf, bias)

    _callable_check(device, "callable-per-head", B, S, S, H, D, n, torch_fn, numpy_fn,
                    {"q_feat": qf, "q_pos": pos}, {"kv_feat": kf, "kv_pos": pos})


def test_block_api_dense_bias(device):
    """fwd_block / bwd_block with the dense [b, 1, lq, lk] bias array the reference's block
    functions take (ring_kernel.py:127,136-141), broadcast over the heads, rows fully masked."""
    B, H, Lq, Lk, D = 2, 3, 200, 333, 128
    q, k, v, do = R.make_inputs(11, B, Lq, Lk, H, D)
    rng = np.random.default_rng(11)
    bias = rng.standard_normal((B, 1, Lq, Lk)).astype(np.float32)
    bias[rng.random((B, 1, Lq, Lk)) < 0.3] = -np.inf
    bias[:, :, 17, :] = -np.inf  # a query without any key: carry untouched, l stays 0
    hq, hk, hv, hdo = (np.ascontiguousarray(np.transpose(x, (0, 2, 1, 3))) for x in (q, k, v, do))
    tq, tk, tv, tdo = (_dev(x, device, torch.bfloat16) for x in (hq, hk, hv, hdo))
    tb = _dev(bias, device)
    o, m, l = rr.init_carry(B, H, Lq, D, device)
    scale = 1 / math.sqrt(D)
    o, m, l = ra.fwd_block(tq, tk, tv, tb, o, m, l, scale)
    f64 = lambda x: x.astype(np.float64)
    wo, wm, wl = R.fwd_block(f64(hq), f64(hk), f64(hv), f64(bias), np.zeros((B, H, Lq, D)),
                             np.full((B, H, Lq), -np.inf), np.zeros((B, H, Lq)), scale)
    assert torch.all(l[:, :, 17] == 0) and torch.all(torch.isneginf(m[:, :, 17]))
    live = np.ones(Lq, bool)
    live[17] = False
    assert np.abs(m.cpu().numpy()[:, :, live] - wm[:, :, live]).max() <= 1e-4
    np.testing.assert_allclose(l.cpu().numpy()[:, :, live], wl[:, :, live], rtol=5e-3)
    got_out = (o / l[..., None]).cpu().numpy()[:, :, live]
    assert np.abs(got_out - wo[:, :, live] / wl[:, :, live, None]).max() <= OUT_TOL
    # backward on the live rows (the reference's block would divide by zero on row 17)
    out = torch.where(l[..., None] > 0, o / l[..., None], torch.zeros_like(o))
    L = m + torch.log(l)
    dq, dk, dv = ra.bwd_block(tq, tk, tv, tb, out, L, tdo, scale)
    wout = np.where(wl[..., None] > 0, wo / np.where(wl > 0, wl, 1)[..., None], 0.0)
    wL = np.where(wl > 0, wm + np.log(np.where(wl > 0, wl, 1)), -np.inf)
    sel = np.ix_(range(B), range(H), np.nonzero(live)[0])
    wdq, wdk, wdv = R.bwd_block(f64(hq)[sel], f64(hk), f64(hv), f64(bias)[:, :, live], wout[sel], wL[sel],
                                f64(hdo)[sel], scale)
    assert torch.all(dq[:, :, 17] == 0)
    for got, ref in ((dq.cpu().numpy()[sel], wdq), (dk.cpu().numpy(), wdk), (dv.cpu().numpy(), wdv)):
        mx, fro = _rel(got, ref)
        assert mx <= GRAD_TOL and fro <= GRAD_TOL
    with pytest.raises(ValueError):
        ra.fwd_block(tq, tk, tv, tb[:, :, :, :-1], o, m, l, scale)


def test_dense_bias_adds_to_declarative_terms(device):
    """A dense block and the in-kernel terms add up (here: a finite dense bias over a causal mask
    with shard offsets), forward and backward, through the block API."""
    B, H, Lq, Lk, D = 1, 2, 384, 256, 128
    q, k, v, do = R.make_inputs(13, B, Lq, Lk, H, D)
    rng = np.random.default_rng(13)
    dense = rng.standard_normal((B, H, Lq, Lk)).astype(np.float32)
    q_off, kv_off = 200, 100
    causal = np.where((kv_off + np.arange(Lk))[None, :] <= (q_off + np.arange(Lq))[:, None], 0.0, -np.inf)
    total = dense.astype(np.float64) + causal[None, None]
    hq, hk, hv, hdo = (np.ascontiguousarray(np.transpose(x, (0, 2, 1, 3))) for x in (q, k, v, do))
    tq, tk, tv, tdo = (_dev(x, device, torch.bfloat16) for x in (hq, hk, hv, hdo))
    bias = ra.BlockBias(ra.causal_bias(), q_offset=q_off, kv_offset=kv_off, dense=_dev(dense, device))
    o, m, l = rr.init_carry(B, H, Lq, D, device)
    scale = 1 / math.sqrt(D)
    o, m, l = ra.fwd_block(tq, tk, tv, bias, o, m, l, scale)
    f64 = lambda x: x.astype(np.float64)
    wo, wm, wl = R.fwd_block(f64(hq), f64(hk), f64(hv), total, np.zeros((B, H, Lq, D)),
                             np.full((B, H, Lq), -np.inf), np.zeros((B, H, Lq)), scale)
    assert np.abs(m.cpu().numpy() - wm).max() <= 1e-4
    assert np.abs((o / l[..., None]).cpu().numpy() - wo / wl[..., None]).max() <= OUT_TOL
    dq, dk, dv = ra.bwd_block(tq, tk, tv, bias, o / l[..., None], m + torch.log(l), tdo, scale)
    wdq, wdk, wdv = R.bwd_block(f64(hq), f64(hk), f64(hv), total, wo / wl[..., None], wm + np.log(wl),
                                f64(hdo), scale)
    for got, ref in ((dq, wdq), (dk, wdk), (dv, wdv)):
        mx, fro = _rel(got.cpu().numpy(), ref)
        assert mx <= GRAD_TOL and fro <= GRAD_TOL


# ---- several ring steps per launch (ra_fwd_steps, ra_bwd_dq_steps, ra_bwd_dkdv_steps) -----------
def _fused_cases():
    seg = R.geometric_segment_ids(0, 2, 2048, 300)
    rng = np.random.default_rng(5)
    segr = rng.integers(0, 5, (2, 512)).astype(np.int32)
    sl = R.alibi_slopes(4)
    pm = (np.arange(512)[None, :] < np.array([[100], [300]])).astype(np.int32)
    docs = (np.arange(6144)[None, :] >= 2900).astype(np.int32)
    return {
        "no_bias_cross": dict(B=2, Sq=128, Sk=64, H=4, D=64, n=8),
        "no_bias_ragged_shards": dict(B=1, Sq=600, Sk=408, H=2, D=128, n=3),
        "causal_c1": dict(B=1, Sq=1024, Sk=1024, H=4, D=64, n=4, fn=ra.causal_bias(), ofn=R.make_bias_fn(causal=True)),
        "causal_d128_ring8": dict(B=2, Sq=2048, Sk=2048, H=4, D=128, n=8, fn=ra.causal_bias(),
                                  ofn=R.make_bias_fn(causal=True)),
        "causal_long_shards": dict(B=1, Sq=6144, Sk=6144, H=2, D=128, n=3, fn=ra.causal_bias(),
                                   ofn=R.make_bias_fn(causal=True)),
        "more_steps_than_one_launch_takes": dict(B=1, Sq=2560, Sk=2560, H=2, D=64, n=20),
        "window": dict(B=1, Sq=2048, Sk=2048, H=2, D=128, n=8, fn=ra.sliding_window_bias(300),
                       ofn=R.make_bias_fn(causal=True, window=300), std=0.5),
        "window_two_sided": dict(B=1, Sq=2048, Sk=2048, H=2, D=64, n=8, fn=ra.sliding_window_bias(200, causal=False),
                                 ofn=R.make_bias_fn(window=200), std=0.5),
        "segments_sorted": dict(B=2, Sq=2048, Sk=2048, H=2, D=128, n=4, fn=ra.segment_bias(),
                                ofn=R.make_bias_fn(use_segments=True), qkw={"q_segment_ids": seg},
                                kvkw={"kv_segment_ids": seg}),
        "segments_random_causal": dict(B=2, Sq=512, Sk=512, H=4, D=64, n=8, fn=ra.causal_bias() + ra.segment_bias(),
                                       ofn=R.make_bias_fn(causal=True, use_segments=True),
                                       qkw={"q_segment_ids": segr}, kvkw={"kv_segment_ids": segr}),
        "long_documents_causal": dict(B=1, Sq=6144, Sk=6144, H=2, D=128, n=2, std=0.7, fn=ra.causal_bias() + ra.segment_bias(),
                                      ofn=R.make_bias_fn(causal=True, use_segments=True),
                                      qkw={"q_segment_ids": docs}, kvkw={"kv_segment_ids": docs}),
        "alibi_segments": dict(B=1, Sq=2048, Sk=2048, H=4, D=128, n=4, fn=ra.segment_bias() + ra.alibi_bias(sl),
                               ofn=R.make_bias_fn(use_segments=True, alibi=sl), qkw={"q_segment_ids": seg[:1]},
                               kvkw={"kv_segment_ids": seg[:1]}),
        "prefix_lm": dict(B=2, Sq=512, Sk=512, H=2, D=64, n=4, fn=ra.prefix_lm_bias(),
                          ofn=R.make_bias_fn(use_prefix=True), qkw={"q_prefix_mask": pm}, kvkw={"kv_prefix_mask": pm}),
    }


@pytest.mark.parametrize("name", sorted(_fused_cases()))
def test_fused_ring_pass(device, name):
    """block_impl="hip_fused": all ring passes in one launch, the kernels walk the shards
    themselves.  Same oracle, same tolerances as the launch-per-step path."""
    _check(device, "fused " + name, impl="hip_fused", **_fused_cases()[name])


def test_pass_entry_points_equal_launches_per_pass(device):
    """ra_fwd_passes / ra_bwd_dq_passes / ra_bwd_dkdv_passes (all ring passes in one grid) give what
    one ra_*_steps launch per pass gives, bit for bit: the same workgroups do the same arithmetic."""
    B, H, D, n, L = 2, 2, 128, 4, 384
    S = n * L
    q, k, v, do = (_dev(x, device, torch.bfloat16) for x in R.make_inputs(19, B, S, S, H, D))
    seg = _dev(R.geometric_segment_ids(2, B, S, 300), device)
    plan = rr._RingPlan(q, k, n, ra.causal_bias() + ra.segment_bias(), {"q_segment_ids": seg}, {"kv_segment_ids": seg})
    sc = 1 / math.sqrt(D)
    sh = lambda x, s_: rr._shard_bhld(x, s_, L)
    out, lse = rr._ring_forward_fused(q, k, v, plan, sc, torch.float32, whole=False)
    dq, dk, dv = rr._ring_backward_fused(q, k, v, out, lse, do, plan, sc, whole=False)
    # the same passes, one launch each
    out1 = torch.empty_like(out)
    lse1 = torch.empty_like(lse)
    for r in range(n):
        o, m, l = rr.init_carry(B, H, L, D, device)
        order = [(r - t) % n for t in range(n)]
        rr.fwd_blocks(sh(q, r), [(sh(k, s_), sh(v, s_)) for s_ in order], [plan.block_bias(r, s_) for s_ in order], o, m, l, sc)
        rr.finalize_carry(o, m, l, sh(out1, r), lse1[r])
    assert torch.equal(out, out1) and torch.equal(lse, lse1)
    delta = torch.stack([rr.precompute_delta(sh(out, s_), sh(do, s_)) for s_ in range(n)])
    z = lambda: torch.zeros((B, H, L, D), dtype=torch.float32, device=device)
    dq1, dk1, dv1 = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    for r in range(n):
        dqa, dka, dva = z(), z(), z()
        rr._bwd_steps("dkdv", [(sh(q, (r - t) % n), sh(k, r), sh(v, r), sh(do, (r - t) % n), lse[(r - t) % n],
                                delta[(r - t) % n], dqa, dka, dva, plan.block_bias((r - t) % n, r)) for t in range(n)], sc)
        rr._finalize_grad(dka, sh(dk1, r))
        rr._finalize_grad(dva, sh(dv1, r))
        dqa = z()
        rr._bwd_steps("dq", [(sh(q, r), sh(k, (r + t) % n), sh(v, (r + t) % n), sh(do, r), lse[r], delta[r], dqa, dka, dva,
                              plan.block_bias(r, (r + t) % n)) for t in range(n)], sc)
        rr._finalize_grad(dqa, sh(dq1, r))
    torch.cuda.synchronize()
    assert torch.equal(dq, dq1) and torch.equal(dk, dk1) and torch.equal(dv, dv1)
    # a second call reuses the cached parameter blocks of the plan with fresh buffers
    out2, lse2 = rr._ring_forward_fused(q, k, v, plan, sc, torch.float32, whole=False)
    g2 = rr._ring_backward_fused(q, k, v, out2, lse2, do, plan, sc, whole=False)
    assert torch.equal(out2, out) and all(torch.equal(a, b_) for a, b_ in zip(g2, (dq, dk, dv)))


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_whole_ring_entry_points_agree_with_the_split_ones(device, out_dtype):
    """ra_fwd_ring / ra_bwd_dq_ring / ra_bwd_dkdv_ring (nothing between the launches goes through
    memory) against init + ra_*_passes + finalize on the same inputs: the same sums, the final
    division and casts folded differently, so they agree to rounding - fp32 outputs to 1e-5 relative,
    bf16 results to one unit in the last place.  Cross attention with a window leaves query rows
    without any key (NaN output, -inf logsumexp, zero gradient) and a pass without a live step."""
    B, H, D, n, Lq, Lk = 2, 2, 128, 4, 320, 192
    q, k, v, do = R.make_inputs(23, B, n * Lq, n * Lk, H, D)
    q, k, v, do = (_dev(x, device, torch.bfloat16) for x in (q, k, v, do))
    sc = 1 / math.sqrt(D)
    for fn in (None, ra.causal_bias(), ra.sliding_window_bias(100)):
        plan = rr._RingPlan(q, k, n, fn, None, None)
        outs = [rr._ring_forward_fused(q, k, v, plan, sc, out_dtype, whole=w) for w in (True, False)]
        (o1, l1), (o0, l0) = outs
        assert torch.equal(torch.isnan(o1), torch.isnan(o0)) and torch.equal(torch.isinf(l1), torch.isinf(l0))
        fin = ~torch.isnan(o0)
        tol = 1e-5 if out_dtype == torch.float32 else 2.0 ** -7
        assert ((o1.float() - o0.float()).abs()[fin] <= tol * o0.float().abs()[fin] + 1e-6).all()
        lf = ~torch.isinf(l0)
        assert ((l1 - l0).abs()[lf] <= 1e-5).all()
        out_b = torch.nan_to_num(o0).to(torch.bfloat16)
        lse_b = l0
        g1 = rr._ring_backward_fused(q, k, v, out_b, lse_b, do, plan, sc, whole=True)
        g0 = rr._ring_backward_fused(q, k, v, out_b, lse_b, do, plan, sc, whole=False)
        torch.cuda.synchronize()
        for a, b_ in zip(g1, g0):
            assert torch.isfinite(a.float()).all()
            assert ((a.float() - b_.float()).abs() <= 2.0 ** -7 * b_.float().abs() + 1e-6).all()


def test_fused_ring_pass_with_a_callable_bias_fn(device):
    B, S, H, D, n = 2, 960, 2, 128, 3
    q, k, v, do = R.make_inputs(7, B, S, S, H, D)
    pos = np.broadcast_to(np.arange(S), (B, S))

    def torch_fn(q_pos, kv_pos):
        rel = q_pos[:, None, :, None] - kv_pos[:, None, None, :]
        return torch.where(rel >= 0, -0.01 * rel.float(), -torch.inf)

    bias = np.where(pos[:, None, :, None] >= pos[:, None, None, :],
                    -0.01 * (pos[:, None, :, None] - pos[:, None, None, :]).astype(np.float32), -np.inf)
    tq, tk, tv = (_dev(x, device, torch.bfloat16).requires_grad_(True) for x in (q, k, v))
    tpos = _dev(pos, device)
    out, lse = ra.ring_attention_with_lse(tq, tk, tv, n, bias_fn=torch_fn, bias_q_kwargs={"q_pos": tpos},
                                          bias_kv_kwargs={"kv_pos": tpos}, out_dtype=torch.float32,
                                          block_impl="hip_fused")
    out.backward(_dev(do, device, torch.float32))
    torch.cuda.synchronize()
    want, want_lse = R.mha_dense(q, k, v, bias)
    assert np.abs(out.detach().cpu().numpy() - want).max() <= OUT_TOL
    assert np.abs(lse.cpu().numpy() - want_lse).max() <= LSE_TOL
    for t, ref, nm in zip((tq, tk, tv), R.mha_dense_grads(q, k, v, do, bias), ("dq", "dk", "dv")):
        mx, fro = _rel(t.grad.float().cpu().numpy(), ref)
        assert mx <= GRAD_TOL and fro <= GRAD_TOL, (nm, mx, fro)


def test_multi_step_entry_points_equal_consecutive_steps(device):
    """ra_fwd_steps / ra_bwd_dq_steps / ra_bwd_dkdv_steps against the same steps issued one by one
    through ra_fwd_step / ra_bwd_step: the same sums in another rounding order."""
    B, H, D, n, L = 1, 3, 128, 4, 640
    S = n * L
    q, k, v, do = R.make_inputs(11, B, S, S, H, D)
    tq, tk, tv, tdo = (_dev(x, device, torch.bfloat16) for x in (q, k, v, do))
    fn = ra.causal_bias()
    sc = 1 / math.sqrt(D)
    sh = lambda x, s: rr._shard_bhld(x, s, L)
    bias = lambda qs, ks: rr.BlockBias(fn, qs * L, ks * L)
    r = 2
    order = [(r - t) % n for t in range(n)]  # the last one is fully masked
    o1, m1, l1 = rr.init_carry(B, H, L, D, device)
    for s in order:
        rr.fwd_block(sh(tq, r), sh(tk, s), sh(tv, s), bias(r, s), o1, m1, l1, sc)
    o2, m2, l2 = rr.init_carry(B, H, L, D, device)
    rr.fwd_blocks(sh(tq, r), [(sh(tk, s), sh(tv, s)) for s in order], [bias(r, s) for s in order], o2, m2, l2, sc)
    assert torch.equal(m1, m2)
    torch.testing.assert_close(l2, l1, rtol=2e-3, atol=0)
    torch.testing.assert_close(o2 / l2[..., None], o1 / l1[..., None], rtol=0, atol=4e-3)
    lse = (m1 + l1.log()).contiguous()
    out = (o1 / l1[..., None]).to(torch.bfloat16)
    delta = rr.precompute_delta(out, sh(tdo, r))
    z = lambda: torch.zeros((B, H, L, D), dtype=torch.float32, device=device)
    dq1, dq2, dk_, dv_ = z(), z(), z(), z()
    for s in order:
        rr._bwd_step(sh(tq, r), sh(tk, s), sh(tv, s), sh(tdo, r), lse, delta, dq1, dk_, dv_, bias(r, s), sc, parts=2)
    rr._bwd_steps("dq", [(sh(tq, r), sh(tk, s), sh(tv, s), sh(tdo, r), lse, delta, dq2, dk_, dv_, bias(r, s))
                         for s in order], sc)
    assert float(dk_.abs().max()) == 0.0 and float(dv_.abs().max()) == 0.0  # dq launches leave dk, dv alone
    torch.testing.assert_close(dq2, dq1, rtol=0, atol=5e-3 * float(dq1.abs().max()))
    # one key/value shard against all query shards (statistics of a plausible forward pass)
    ks = 1
    lse_all = torch.stack([lse + 0.1 * i for i in range(n)])
    dl_all = torch.stack([delta * (1 + 0.1 * i) for i in range(n)])
    dk1, dv1, dk2, dv2, dqx = z(), z(), z(), z(), z()
    for qs in range(n):
        rr._bwd_step(sh(tq, qs), sh(tk, ks), sh(tv, ks), sh(tdo, qs), lse_all[qs], dl_all[qs], dqx, dk1, dv1,
                     bias(qs, ks), sc, parts=1)
    rr._bwd_steps("dkdv", [(sh(tq, qs), sh(tk, ks), sh(tv, ks), sh(tdo, qs), lse_all[qs], dl_all[qs], dqx, dk2, dv2,
                            bias(qs, ks)) for qs in range(n)], sc)
    torch.cuda.synchronize()
    assert float(dqx.abs().max()) == 0.0
    torch.testing.assert_close(dk2, dk1, rtol=0, atol=5e-3 * float(dk1.abs().max()))
    torch.testing.assert_close(dv2, dv1, rtol=0, atol=5e-3 * float(dv1.abs().max()))


@pytest.mark.parametrize("impl", ["hip", "hip_fused"])
def test_ring_replays_from_a_captured_graph(device, impl):
    """Every launch of a forward + backward ring goes to the caller's stream (and, for the fused
    passes, to side streams forked from it and joined back), allocates through torch only and
    clears memory with fill kernels: the whole of it can be captured in a HIP graph.  Replays,
    with eager work and synchronisations between them, reproduce the eager result bit for bit."""
    B, S, H, D, n = 1, 2048, 4, 128, 4
    q, k, v, do = (_dev(x, device, torch.bfloat16) for x in R.make_inputs(3, B, S, S, H, D))
    seg = _dev(R.geometric_segment_ids(1, B, S, 500), device)
    plan = rr._RingPlan(q, k, n, ra.causal_bias() + ra.segment_bias(), {"q_segment_ids": seg},
                        {"kv_segment_ids": seg})
    sc = 1 / math.sqrt(D)
    fwd = rr._ring_forward_fused if impl == "hip_fused" else rr._ring_forward
    bwd = rr._ring_backward_fused if impl == "hip_fused" else rr._ring_backward

    def step():
        out, lse = fwd(q, k, v, plan, sc, torch.bfloat16)
        return (out, lse) + tuple(bwd(q, k, v, out, lse, do, plan, sc))

    eager = [t.clone() for t in step()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up off the default stream, as capture requires
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    torch.cuda.synchronize()
    for _ in range(3):
        for t in captured:
            t.fill_(0) if t.dtype != torch.bfloat16 else t.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(captured, eager):
            assert torch.equal(got, want)
        again = step()  # eager work between the replays
        torch.cuda.synchronize()
        for got, want in zip(again, eager):
            assert torch.equal(got, want)


def _random_cases(seed, count):
    """The seeded sweep generator: ragged shard lengths, cross attention, padded head dims, ring
    sizes 1..8 and nine bias combinations."""
    rng = np.random.default_rng(seed)
    for case in range(count):
        B, H = int(rng.integers(1, 3)), int(rng.choice([1, 2, 4]))
        D = int(rng.choice([64, 128, 32, 96]))
        n = int(rng.choice([1, 2, 3, 4, 8]))
        Lq = int(rng.choice([3, 17, 64, 100, 128, 200, 256, 300, 520]))
        cross = rng.random() < 0.3
        Lk = int(rng.choice([5, 64, 96, 128, 250, 400])) if cross else Lq
        Sq, Sk = n * Lq, n * Lk
        kind = str(rng.choice(["none", "causal", "window", "window2", "seg", "seg_causal", "alibi",
                               "alibi_causal_seg", "prefix"]))
        if cross and kind == "prefix":
            kind = "seg"
        if rng.random() < 0.6:
            segq = np.sort(rng.integers(0, max(2, Sq // 150), (B, Sq)).astype(np.int32), axis=1)
        else:
            segq = rng.integers(0, 3, (B, Sq)).astype(np.int32)
        segk = segq if not cross else np.sort(rng.integers(0, max(2, Sq // 150), (B, Sk)).astype(np.int32), axis=1)
        seg_kw = ({"q_segment_ids": segq}, {"kv_segment_ids": segk})
        sl = R.alibi_slopes(H)
        w = int(rng.integers(1, max(2, Sk)))
        pm = (np.arange(Sq)[None] < rng.integers(0, Sq, (B, 1))).astype(np.int32)
        fn, ofn, (qkw, kvkw) = {
            "none": (None, None, ({}, {})),
            "causal": (ra.causal_bias(), R.make_bias_fn(causal=True), ({}, {})),
            "window": (ra.sliding_window_bias(w), R.make_bias_fn(causal=True, window=w), ({}, {})),
            "window2": (ra.sliding_window_bias(w, causal=False), R.make_bias_fn(window=w), ({}, {})),
            "seg": (ra.segment_bias(), R.make_bias_fn(use_segments=True), seg_kw),
            "seg_causal": (ra.segment_bias() + ra.causal_bias(), R.make_bias_fn(causal=True, use_segments=True), seg_kw),
            "alibi": (ra.alibi_bias(sl), R.make_bias_fn(alibi=sl), ({}, {})),
            "alibi_causal_seg": (ra.alibi_bias(sl) + ra.causal_bias() + ra.segment_bias(),
                                 R.make_bias_fn(causal=True, use_segments=True, alibi=sl), seg_kw),
            "prefix": (ra.prefix_lm_bias(), R.make_bias_fn(use_prefix=True),
                       ({"q_prefix_mask": pm}, {"kv_prefix_mask": pm})),
        }[kind]
        std = float(rng.choice([0.5, 1.0]))
        data_seed = int(rng.integers(1 << 30))
        yield case, kind, dict(B=B, Sq=Sq, Sk=Sk, H=H, D=D, n=n, fn=fn, ofn=ofn, qkw=qkw, kvkw=kvkw, std=std,
                               seed=data_seed)


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_random_configurations(device, seed):
    """Seeded random shapes and bias combinations, each through both launch schemes and through the
    default block_impl (the reference's "pallas": the library picks the scheme), against the dense
    oracle."""
    for case, kind, kw in _random_cases(seed, 12):
        for impl in ("hip", "hip_fused", "pallas"):
            _check(device, f"random {seed}.{case} {kind}", impl=impl, **kw)


@pytest.mark.parametrize("impl", ["hip", "hip_fused"])
def test_random_configuration_in_which_no_query_sees_a_key(device, impl):
    """Case 3 of sweep seed 109: six queries against 800 keys under causal + segment + ALiBi
    biases, and every query row is fully masked.  All outputs are NaN and all logsumexps -inf
    (ring.py:134-135), dk and dv are zero, and there is no live row to compare dq on."""
    case, kind, kw = [c for c in _random_cases(109, 4)][3]
    assert (kw["Sq"], kw["Sk"], kind) == (6, 800, "alibi_causal_seg")
    _check(device, f"random 109.{case} {kind}", impl=impl, **kw)


# The cases of the seed-0 sweep with shard lengths off the tile grid (300, 520, 100 queries;
# 250, 400, 96 keys) that an earlier hand-run sweep reported above tolerance.  That run drew its
# inputs from N(0, 2^2): scores with a standard deviation of 4 and outputs up to 8.5, where the
# half-ulp of a bf16 probability (2^-9 relative) alone is worth 1e-2 on the output.  At the
# amplitudes of the benchmark configurations (N(0, 1) and N(0, 0.5^2)) every one of them is
# within tolerance; at N(0, 2^2) the output stays within 2.5e-3 of its largest value.
_SEED0_RAGGED = (9, 20, 21, 32, 55, 58, 67)


@pytest.mark.parametrize("impl", ["hip", "hip_fused"])
def test_seed0_ragged_sweep_cases(device, impl):
    worst = {}
    for case, kind, kw in _random_cases(0, max(_SEED0_RAGGED) + 1):
        if case not in _SEED0_RAGGED:
            continue
        for std in (0.5, 1.0):
            got = _check(device, f"seed-0 sweep case {case} {kind} std={std}", impl=impl, **{**kw, "std": std})
            for a, b in got.items():
                worst[a] = max(worst.get(a, 0.0), b)
    print("[parity] seed-0 ragged cases, worst over all: " + " ".join(f"{a} {b:.2e}" for a, b in worst.items()),
          flush=True)


@pytest.mark.parametrize("impl", ["hip", "hip_fused"])
def test_seed0_ragged_sweep_cases_at_four_times_the_score_spread(device, impl):
    """The same cases with N(0, 2^2) inputs (what the hand-run sweep used): outside the amplitude
    the absolute tolerances are stated for, so the output is held to a relative bound; the
    logsumexp and the gradients keep theirs (the backward kernels fold only a power of two of the
    softmax scale into their bf16 operands, so a wider score spread costs them nothing)."""
    for case, kind, kw in _random_cases(0, max(_SEED0_RAGGED) + 1):
        if case not in _SEED0_RAGGED:
            continue
        print(f"[parity] seed-0 sweep case {case} {kind} std=2.0 impl={impl}", flush=True)
        q, k, v, do = R.make_inputs(kw["seed"], kw["B"], kw["Sq"], kw["Sk"], kw["H"], kw["D"], std=2.0)
        out, lse, g = _run_hip(device, q, k, v, do, kw["n"], kw["fn"], kw["qkw"], kw["kvkw"], impl=impl)
        oq, okv = dict(kw["qkw"]), dict(kw["kvkw"])
        bias = None
        if kw["ofn"] is not None:
            oq.setdefault("q_positions", np.broadcast_to(np.arange(kw["Sq"]), (kw["B"], kw["Sq"])))
            okv.setdefault("kv_positions", np.broadcast_to(np.arange(kw["Sk"]), (kw["B"], kw["Sk"])))
            bias = kw["ofn"](**oq, **okv)
        want, want_lse = R.mha_dense(q, k, v, bias)
        assert not np.isnan(want).any()
        rel = np.abs(out - want).max() / np.abs(want).max()
        assert rel <= 2.5e-3, (case, rel)
        assert np.abs(lse - want_lse).max() <= LSE_TOL
        for got, ref, nm in zip(g, R.mha_dense_grads(q, k, v, do, bias), ("dq", "dk", "dv")):
            mx, fro = _rel(got, ref)
            assert mx <= GRAD_TOL and fro <= GRAD_TOL, (case, nm, mx, fro)


def test_delta_kernel(device):
    B, H, L, D = 2, 3, 100, 64
    rng = np.random.default_rng(0)
    out = R.bf16_round(rng.standard_normal((B, L, H, D)).astype(np.float32))
    do = R.bf16_round(rng.standard_normal((B, L, H, D)).astype(np.float32))
    want = R.precompute_delta(out, do)
    for dt in (torch.bfloat16, torch.float32):
        got = ra.precompute_delta(_dev(out, device, dt).permute(0, 2, 1, 3), _dev(do, device, torch.bfloat16).permute(0, 2, 1, 3))
        np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-5, atol=1e-5)


def test_deterministic_and_layout_independent(device):
    """No atomics: two runs agree bit for bit; [b,l,h,d] and [b,h,l,d] storage give the same bits."""
    B, S, H, D, n = 1, 1024, 4, 128, 4
    q, k, v, do = R.make_inputs(8, B, S, S, H, D)
    a = _run_hip(device, q, k, v, do, n, ra.causal_bias(), None, None)
    b = _run_hip(device, q, k, v, do, n, ra.causal_bias(), None, None)
    np.testing.assert_array_equal(a[0], b[0])
    for x, y in zip(a[2], b[2]):
        np.testing.assert_array_equal(x, y)
    # head-major storage viewed as [b, l, h, d]
    tq, tk, tv = (_dev(np.ascontiguousarray(np.transpose(x, (0, 2, 1, 3))), device, torch.bfloat16).permute(0, 2, 1, 3)
                  for x in (q, k, v))
    assert not tq.is_contiguous()
    out = ra.ring_attention(tq, tk, tv, n, bias_fn=ra.causal_bias())
    out_ref = ra.ring_attention(_dev(q, device, torch.bfloat16), _dev(k, device, torch.bfloat16),
                                _dev(v, device, torch.bfloat16), n, bias_fn=ra.causal_bias())
    assert torch.equal(out, out_ref)


def test_fp32_and_fp16_inputs_are_cast(device):
    q, k, v, _ = R.make_inputs(2, 1, 256, 256, 2, 64)
    want, _ = R.mha_dense(q, k, v)
    out = ra.ring_attention(_dev(q, device), _dev(k, device), _dev(v, device), 2)
    assert out.dtype == torch.float32 and np.abs(out.cpu().numpy() - want).max() <= OUT_TOL
    out16 = ra.ring_attention(_dev(q, device, torch.float16), _dev(k, device, torch.float16), _dev(v, device, torch.float16), 2)
    assert out16.dtype == torch.float16
    out_bf = ra.ring_attention(_dev(q, device, torch.bfloat16), _dev(k, device, torch.bfloat16), _dev(v, device, torch.bfloat16), 2)
    assert out_bf.dtype == torch.bfloat16
    assert np.abs(out_bf.float().cpu().numpy() - want).max() <= 2e-2  # bf16 output rounding on top


# ---- benchmark configs at full size -------------------------------------------------------------------------
def _dense_reference_on_device(Q, K, V, DO, scale, bias_rows, chunk=1024):
    """The dense closed form softmax(Q K^T * scale + bias) V and its analytic gradients
    (oracle mha_dense / mha_dense_grads, ring.py:142-155) for ONE (batch, head), evaluated in fp64
    with torch matrix products on the device, a chunk of query rows at a time.  ``bias_rows(i0, i1)``
    returns the additive bias rows [i1 - i0, Sk] (fp64, -inf masks).  Independent of the HIP
    kernels: nothing of their output enters.  Returns out, lse, dq, dk, dv."""
    Sq, Sk = Q.shape[0], K.shape[0]
    out, lse = torch.empty_like(Q), torch.empty(Sq, dtype=torch.float64, device=Q.device)
    dq, dk, dv = torch.empty_like(Q), torch.zeros_like(K), torch.zeros_like(V)
    for i0 in range(0, Sq, chunk):
        i1 = min(i0 + chunk, Sq)
        s = (Q[i0:i1] @ K.T) * scale + bias_rows(i0, i1)
        m = s.max(dim=1, keepdim=True).values
        p = torch.exp(s - m)
        l = p.sum(dim=1, keepdim=True)
        p /= l
        lse[i0:i1] = (m + torch.log(l))[:, 0]
        o = p @ V
        out[i0:i1] = o
        g = DO[i0:i1]
        dv += p.T @ g
        dp = g @ V.T
        ds = p * (dp - (o * g).sum(dim=1, keepdim=True)) * scale
        dq[i0:i1] = ds @ K
        dk += ds.T @ Q[i0:i1]
    return out, lse, dq, dk, dv


def _full_size_check(device, name, B, H, D, S, n, fn, std, bias_rows_t, bias_row_np, qkw=None, kvkw=None,
                     impl="hip", heads=None, n_rows=256):
    """One benchmark configuration at full size through the HIP path, inputs as bench.py makes them
    (the oracle's make_inputs stream, seed 0).  Checked, for every batch and the chosen heads:
      * EVERY row of out, lse, dq, dk, dv against the dense fp64 closed form evaluated on the
        device by torch (which never sees a kernel output);
      * that torch evaluation itself against the numpy oracle formulas on n_rows sampled query
        rows per head - row 0, every shard boundary -1 / +0 / +1, the last row, random rows -
        which ties the full-size reference to the oracle;
      * two invariants of softmax attention on all heads, with relative slack only."""
    print(f"[parity] {name}: B={B} H={H} D={D} S={S} ring={n} impl={impl}", flush=True)
    rng = np.random.default_rng(0)

    def mk(sd):
        t = torch.empty(B * S * H * D, device=device, dtype=torch.bfloat16)
        piece = 1 << 26
        for a0 in range(0, t.numel(), piece):
            x = rng.standard_normal(min(piece, t.numel() - a0), dtype=np.float32)
            if sd != 1.0:
                x *= np.float32(sd)
            t[a0:a0 + x.size] = torch.from_numpy(x).to(device).to(torch.bfloat16)
        return t.view(B, S, H, D)

    q, k, v, do = mk(std), mk(std), mk(std), mk(1.0)
    q.requires_grad_(True); k.requires_grad_(True); v.requires_grad_(True)
    out, lse = ra.ring_attention_with_lse(q, k, v, n, bias_fn=fn, bias_q_kwargs=qkw, bias_kv_kwargs=kvkw,
                                          out_dtype=torch.float32, block_impl=impl)
    out.backward(do.float())
    torch.cuda.synchronize()
    scale = 1 / math.sqrt(D)
    # invariants (exact in real arithmetic whenever every query sees at least one key):
    #   sum_j dv_j = sum_i do_i   (rows of P sum to one);   <q, dq> = <k, dk>   (both are sum_ij ds_ij s_ij / scale)
    dv_sum, do_sum = v.grad.double().sum(dim=1), do.double().sum(dim=1)
    inv1 = ((dv_sum - do_sum).abs().max() / do_sum.abs().max()).item()
    qdq = (q.detach().double() * q.grad.double()).sum(dim=(1, 3))
    kdk = (k.detach().double() * k.grad.double()).sum(dim=(1, 3))
    inv2 = ((qdq - kdk).abs().max() / qdq.abs().max()).item()
    assert inv1 <= GRAD_TOL and inv2 <= GRAD_TOL, (inv1, inv2)
    L = S // n
    edge = sorted({0, S - 1} | {min(max(c * L + d, 0), S - 1) for c in range(1, n) for d in (-1, 0, 1)})
    worst = {"out": 0.0, "out_rel": 0.0, "lse": 0.0, "dq": 0.0, "dk": 0.0, "dv": 0.0, "ref_vs_oracle": 0.0}
    for b in range(B):
        for h in (sorted(heads) if heads is not None else range(H)):
            Q, K, V, DO = (x.detach()[b, :, h].double() for x in (q, k, v, do))
            r_out, r_lse, r_dq, r_dk, r_dv = _dense_reference_on_device(Q, K, V, DO, scale,
                                                                       lambda i0, i1: bias_rows_t(b, h, i0, i1))
            g_out, g_lse = out.detach()[b, :, h].double(), lse[b, h].double()
            worst["out"] = max(worst["out"], (g_out - r_out).abs().max().item())
            worst["out_rel"] = max(worst["out_rel"], ((g_out - r_out).abs().max() / r_out.abs().max()).item())
            worst["lse"] = max(worst["lse"], (g_lse - r_lse).abs().max().item())
            for nm, got, ref in (("dq", q.grad, r_dq), ("dk", k.grad, r_dk), ("dv", v.grad, r_dv)):
                d = got[b, :, h].double() - ref
                worst[nm] = max(worst[nm], (d.abs().max() / ref.abs().max()).item(),
                                (d.norm() / ref.norm()).item())
            # the oracle's formulas in numpy on sampled rows
            rows = sorted(set(edge) | set(np.random.default_rng(1000 * b + h).integers(0, S, n_rows - len(edge)).tolist()))
            Kn, Vn = K.cpu().numpy(), V.cpu().numpy()
            Qn, DOn = Q[rows].cpu().numpy(), DO[rows].cpu().numpy()
            t_out, t_lse, t_dq = r_out[rows].cpu().numpy(), r_lse[rows].cpu().numpy(), r_dq[rows].cpu().numpy()
            sc_ = (Qn @ Kn.T) * scale + np.stack([bias_row_np(b, h, i) for i in rows])
            mx = sc_.max(axis=1, keepdims=True)
            pr = np.exp(sc_ - mx)
            l_ = pr.sum(axis=1, keepdims=True)
            pr /= l_
            dp = DOn @ Vn.T
            o_np = pr @ Vn
            dq_np = (pr * (dp - (pr * dp).sum(axis=1, keepdims=True)) * scale) @ Kn
            e = max(np.abs(t_out - o_np).max(), np.abs(t_lse - (mx + np.log(l_))[:, 0]).max(),
                    (np.abs(t_dq - dq_np).max(axis=1) / (np.abs(dq_np).max(axis=1) + 1e-6)).max())
            worst["ref_vs_oracle"] = max(worst["ref_vs_oracle"], float(e))
    print(f"[parity] {name}: " + " ".join(f"{a} {b_:.2e}" for a, b_ in worst.items()) +
          f" inv_dv {inv1:.2e} inv_qk {inv2:.2e}", flush=True)
    assert worst["ref_vs_oracle"] <= 1e-9
    assert worst["out"] <= OUT_TOL and worst["out_rel"] <= OUT_REL and worst["lse"] <= LSE_TOL, worst
    for nm in ("dq", "dk", "dv"):
        assert worst[nm] <= GRAD_TOL, worst


def _causal_rows_t(device, S, window=None):
    pos = torch.arange(S, device=device)

    def rows(b, h, i0, i1):
        rel = pos[i0:i1, None] - pos[None, :]
        ok = rel >= 0 if window is None else (rel >= 0) & (rel < window)
        return torch.where(ok, 0.0, -torch.inf).double()
    return rows


def _causal_row_np(S, window=None):
    pos = np.arange(S)
    if window is None:
        return lambda b, h, i: np.where(pos <= i, 0.0, -np.inf)
    return lambda b, h, i: np.where((pos <= i) & (i - pos < window), 0.0, -np.inf)


@pytest.mark.parametrize("impl", ["hip", "hip_fused"])
def test_config2_full_size(device, impl):
    # B=2 H=16 D=128 S=8192 in 8 shards of 1024, causal with fully masked steps skipped; every head,
    # launch per step and launch per ring pass (small shards are where the latter pays)
    B, H, D, S, n = 2, 16, 128, 8192, 8
    _full_size_check(device, "C2", B, H, D, S, n, ra.causal_bias(), 1.0, _causal_rows_t(device, S),
                     _causal_row_np(S), impl=impl, n_rows=64)


@pytest.mark.parametrize("impl", ["hip", "hip_fused"])
def test_config3_full_size(device, impl):
    # B=1 H=32 D=128 S=131072 in 8 shards of 16384, causal: the benchmark workload
    B, H, D, S, n = 1, 32, 128, 131072, 8
    _full_size_check(device, "C3", B, H, D, S, n, ra.causal_bias(), 1.0, _causal_rows_t(device, S),
                     _causal_row_np(S), impl=impl, heads={0, 13, H - 1})


@pytest.mark.parametrize("impl", ["hip", "hip_fused"])
def test_config4_full_size(device, impl):
    # B=1 H=16 D=128 S=32768 in 4 shards: geometric segments (mean 2048) + ALiBi 2^(-8h/H)
    B, H, D, S, n = 1, 16, 128, 32768, 4
    seg = R.geometric_segment_ids(0, B, S, 2048)
    slopes = R.alibi_slopes(H)
    pos = np.arange(S)
    tseg = torch.from_numpy(seg).to(device)
    tpos = torch.arange(S, device=device)

    def rows_t(b, h, i0, i1):
        same = tseg[b, i0:i1, None] == tseg[b, None, :]
        dist = (tpos[i0:i1, None] - tpos[None, :]).abs().double()
        return torch.where(same, 0.0, -torch.inf).double() - float(slopes[h]) * dist

    brow = lambda b, h, i: np.where(seg[b] == seg[b, i], 0.0, -np.inf) - slopes[h] * np.abs(i - pos)
    _full_size_check(device, "C4", B, H, D, S, n, ra.segment_bias() + ra.alibi_bias(slopes), 1.0, rows_t, brow,
                     {"q_segment_ids": tseg}, {"kv_segment_ids": tseg}, impl=impl, heads={0, 7, H - 1})


@pytest.mark.parametrize("impl", ["hip", "hip_fused"])
def test_config5_full_size(device, impl):
    # B=1 H=8 D=128 S=65536 in 8 shards of 8192, causal window 4096, N(0, 0.5^2)
    B, H, D, S, n, W = 1, 8, 128, 65536, 8, 4096
    _full_size_check(device, "C5", B, H, D, S, n, ra.sliding_window_bias(W), 0.5, _causal_rows_t(device, S, W),
                     _causal_row_np(S, W), impl=impl, heads={0, 3, H - 1})


@pytest.mark.parametrize("impl", ["hip", "hip_fused"])
def test_segment_shards_longer_than_one_call_takes(device, impl):
    # one "device" holding 98304 tokens of three documents, causal: above the 65536 tokens that a
    # call takes under a segment bias, so the ring is walked as two shards of 49152
    B, H, D, S, n = 1, 2, 64, 98304, 1
    seg = np.zeros((B, S), np.int32)
    seg[0, 30000:] += 1
    seg[0, 70001:] += 1
    tseg = torch.from_numpy(seg).to(device)
    tpos = torch.arange(S, device=device)
    pos = np.arange(S)

    def rows_t(b, h, i0, i1):
        ok = (tseg[b, i0:i1, None] == tseg[b, None, :]) & (tpos[None, :] <= tpos[i0:i1, None])
        return torch.where(ok, 0.0, -torch.inf).double()

    brow = lambda b, h, i: np.where((seg[b] == seg[b, i]) & (pos <= i), 0.0, -np.inf)
    _full_size_check(device, "long segment shard", B, H, D, S, n, ra.segment_bias() + ra.causal_bias(), 1.0, rows_t,
                     brow, {"q_segment_ids": tseg}, {"kv_segment_ids": tseg}, impl=impl, n_rows=64)


@pytest.mark.parametrize("impl", ["hip", "hip_fused"])
@pytest.mark.parametrize("std,D,kind", [(4.0, 128, "causal"), (8.0, 128, "causal"), (8.0, 64, "none"),
                                        (8.0, 128, "causal+alibi"), (0.05, 128, "causal"), (0.05, 64, "none")])
def test_extreme_score_spreads(device, impl, std, D, kind):
    """Inputs far outside the benchmark amplitudes.  N(0, 4^2) and N(0, 8^2) give scores with a
    standard deviation of 16..64 (times sqrt(d) * sm_scale = 1): every row's weight sits on one or
    two keys; N(0, 0.05^2) gives flat rows whose outputs are averages that nearly cancel.  Everything
    must stay finite, the output within 2^-8 of its largest value (half a unit in the last place
    of one bf16 probability), logsumexp and gradients within their usual bounds.  (A row sum
    taken over the bf16-rounded weights alone fails this: one dominant weight's rounding error,
    up to 2^-8 relative, lands in the logsumexp.  The kernels keep the exact sum beside it.)"""
    B, H, n, L = 1, 2, 3, 1536
    S = n * L
    sl = R.alibi_slopes(H)
    fn, ofn = {"causal": (ra.causal_bias(), R.make_bias_fn(causal=True)), "none": (None, None),
               "causal+alibi": (ra.alibi_bias(sl) + ra.causal_bias(), R.make_bias_fn(causal=True, alibi=sl))}[kind]
    print(f"[parity] extreme spread std={std} D={D} {kind} impl={impl}", flush=True)
    q, k, v, do = R.make_inputs(7, B, S, S, H, D, std=std)
    out, lse, g = _run_hip(device, q, k, v, do, n, fn, None, None, impl=impl)
    bias = None
    if ofn is not None:
        pos = np.broadcast_to(np.arange(S), (B, S))
        bias = ofn(q_positions=pos, kv_positions=pos)
    want, want_lse = R.mha_dense(q, k, v, bias)
    assert np.isfinite(out).all() and np.isfinite(lse).all()
    worst = {"out_rel": np.abs(out - want).max() / np.abs(want).max(), "lse": np.abs(lse - want_lse).max()}
    for got, ref, nm in zip(g, R.mha_dense_grads(q, k, v, do, bias), ("dq", "dk", "dv")):
        assert np.isfinite(got).all(), nm
        worst[nm] = np.abs(got - ref).max() / np.abs(ref).max()
    print("[parity]   worst: " + " ".join(f"{a} {b:.2e}" for a, b in worst.items()), flush=True)
    assert worst["out_rel"] <= 2.0 ** -8 and worst["lse"] <= LSE_TOL, worst
    assert max(worst["dq"], worst["dk"], worst["dv"]) <= GRAD_TOL, worst

"""The summary of a dense bias block (ra_dense_map) and the step kernels that take it: tiles whose
part of the block is -inf throughout are left out, the block is read only where it is not zero,
and the results are those of the kernels that read all of it (ring_kernel.py:75-85 adds the whole
block).  Checked against numpy (the summary itself), against the dense oracle, and against the
same call without a summary."""
import ctypes as C

import numpy as np
import pytest
import torch

import ring_attention as ra
from ring_attention import _lib, bias as rbias, ring as rr
from oracle import ring_oracle as R

from test_gpu_parity import GRAD_TOL, LSE_TOL, OUT_TOL, _dev, _rel, _run_hip

pytestmark = pytest.mark.gpu


def _numpy_summary(block, Lq, Lk):
    """bit 0: some value of the 32 x 32 cell is not -inf; bit 1: some value is not 0."""
    nb, nh = block.shape[:2]
    rows, cols = (Lq + 31) // 32, (Lk + 31) // 32
    out = np.zeros((nb, nh, rows, cols), dtype=np.uint8)
    for r in range(rows):
        for c in range(cols):
            cell = block[:, :, 32 * r:32 * r + 32, 32 * c:32 * c + 32]
            live = ~np.isneginf(cell)
            nonzero = cell != 0
            out[:, :, r, c] = live.any(axis=(2, 3)) * 1 + nonzero.any(axis=(2, 3)) * 2
    return out


def _patchwork(rng, nb, nh, Lq, Lk):
    """A block of rectangles that are -inf, zero, finite values, or one of the first two with a
    single odd element somewhere; cell boundaries fall on and off the rectangles' edges."""
    blk = np.zeros((nb, nh, Lq, Lk), dtype=np.float32)
    for b in range(nb):
        for h in range(nh):
            for r0 in range(0, Lq, 48):
                for c0 in range(0, Lk, 80):
                    kind = rng.integers(0, 6)
                    sl = (b, h, slice(r0, r0 + 48), slice(c0, c0 + 80))
                    shape = blk[sl].shape
                    if kind == 0:
                        blk[sl] = -np.inf
                    elif kind == 2:
                        blk[sl] = rng.standard_normal(shape)
                    elif kind in (3, 4):
                        blk[sl] = -np.inf if kind == 3 else 0.0
                        i, j = rng.integers(0, shape[0]), rng.integers(0, shape[1])
                        blk[b, h, r0 + i, c0 + j] = 0.0 if kind == 3 else (-np.inf if rng.random() < 0.5 else 1.5)
                    elif kind == 5:
                        blk[sl] = np.where(rng.random(shape) < 0.5, 0.0, -np.inf)
    return blk


@pytest.mark.parametrize("nb,nh,Lq,Lk,pad", [(1, 1, 64, 64, 0), (2, 3, 100, 250, 0), (2, 3, 100, 250, 6),
                                             (1, 2, 300, 520, 0), (1, 1, 33, 1031, 1), (2, 1, 512, 2048, 0)])
def test_summary_matches_numpy(device, nb, nh, Lq, Lk, pad):
    """Aligned rows (16-byte loads), rows off that alignment (Lk = 250, or a padded pitch), cells cut
    by the block's edges, batch and head strides."""
    lib = _lib.load()
    rng = np.random.default_rng(nb * 1000 + Lq + Lk + pad)
    blk = _patchwork(rng, nb, nh, Lq, Lk)
    store = torch.full((nb, nh, Lq, Lk + pad), float("nan"), device=device)  # the padding must not be read as data
    store[..., :Lk] = torch.from_numpy(blk).to(device)
    view = store[..., :Lk]
    B, H = (nb, nh)
    sb = 0 if nb == 1 else view.stride(0)
    sh = 0 if nh == 1 else view.stride(1)
    size = lib.ra_dense_map_bytes(sb, sh, B, H, Lq, Lk)
    assert size == nb * nh * ((Lq + 31) // 32) * ((Lk + 31) // 32)
    got = torch.full((size + 64,), 0xEE, dtype=torch.uint8, device=device)
    _lib.check("ra_dense_map", lib.ra_dense_map(view.data_ptr(), sb, sh, view.stride(2), B, H, Lq, Lk,
                                                got.data_ptr(), None))
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    assert (got[size:] == 0xEE).all(), "wrote past the summary"
    np.testing.assert_array_equal(got[:size].reshape(nb, nh, (Lq + 31) // 32, (Lk + 31) // 32),
                                  _numpy_summary(blk, Lq, Lk))


def test_summary_of_nan_and_positive_infinity(device):
    """NaN and +inf are values like any other: the cell is neither all -inf nor all zero."""
    lib = _lib.load()
    blk = torch.zeros((1, 1, 64, 64), device=device)
    blk[0, 0, :32, :32] = float("nan")
    blk[0, 0, 32:, :32] = float("inf")
    blk[0, 0, :32, 32:] = -float("inf")
    got = torch.zeros((4,), dtype=torch.uint8, device=device)
    _lib.check("ra_dense_map", lib.ra_dense_map(blk.data_ptr(), 0, 0, 64, 1, 1, 64, 64, got.data_ptr(), None))
    assert got.cpu().tolist() == [3, 2, 3, 1]


def _both_ways(device, monkeypatch, name, B, Sq, Sk, H, D, n, torch_fn, numpy_fn, qkw, kvkw, seed=0, tight=True):
    """The same call with and without the summary, each against the dense oracle, and the two
    against each other."""
    print(f"[parity] {name}: B={B} Sq={Sq} Sk={Sk} H={H} D={D} ring={n}", flush=True)
    q, k, v, do = R.make_inputs(seed, B, Sq, Sk, H, D)
    res = {}
    for on in (True, False):
        monkeypatch.setattr(rbias, "DENSE_SUMMARY", on)
        res[on] = _run_hip(device, q, k, v, do, n, torch_fn, qkw, kvkw)
    bias = numpy_fn(**qkw, **kvkw)
    want, want_lse = R.mha_dense(q, k, v, bias)
    ok = ~np.isnan(want)
    live = ok.all(axis=(2, 3))
    okl = np.isfinite(want_lse)
    ref_g = None
    if live.any():
        do_l = np.where(live[:, :, None, None], do, 0.0)
        bias_l = np.where(live[:, None, :, None], np.broadcast_to(bias, (B, bias.shape[1], Sq, Sk)), 0.0)
        ref_g = R.mha_dense_grads(q, k, v, do_l, bias_l)
    for on in (True, False):
        out, lse, g = res[on]
        np.testing.assert_array_equal(np.isnan(out), np.isnan(want))
        np.testing.assert_array_equal(np.isneginf(lse), np.isneginf(want_lse))
        assert np.abs(out - want)[ok].max(initial=0.0) <= OUT_TOL, on
        assert np.abs(lse[okl] - want_lse[okl]).max(initial=0.0) <= LSE_TOL, on
        if ref_g is not None:
            for got, ref, nm in zip(g, ref_g, ("dq", "dk", "dv")):
                if nm == "dq":
                    got, ref = got[live], ref[live]
                else:
                    assert np.isfinite(got).all(), (nm, on)
                mx, fro = _rel(got, ref)
                assert mx <= GRAD_TOL and fro <= GRAD_TOL, (nm, on, mx, fro)
    # with and without: the same tiles contribute the same numbers; only the order of fp32 sums
    # and the bf16 rounding points of a straight-line stretch differ from a generic iteration
    (o1, l1, g1), (o0, l0, g0) = res[True], res[False]
    assert np.abs(o1 - o0)[ok].max(initial=0.0) <= (2e-3 if tight else OUT_TOL)
    assert np.abs(l1[okl] - l0[okl]).max(initial=0.0) <= 2e-4
    for a, b_, nm in zip(g1, g0, ("dq", "dk", "dv")):
        if nm == "dq":
            a, b_ = a[live], b_[live]
        if a.size:
            assert _rel(a, b_)[0] <= 5e-3, nm


@pytest.mark.parametrize("seed,q_len,kv_len,h,d", [(1, 128, 64, 4, 64), (2, 64, 512, 4, 16), (3, 2048, 2048, 4, 128)])
def test_reference_segment_callable_with_and_without_summary(device, monkeypatch, seed, q_len, kv_len, h, d):
    """The bias_fn of the reference's own test (ring_test.py:226-246) with random ids: every cell
    of the mask is mixed, so the summary changes nothing but must not break anything."""
    rng = np.random.default_rng(seed)
    qs = rng.integers(0, 5, (2, q_len)).astype(np.int32)
    ks = rng.integers(0, 5, (2, kv_len)).astype(np.int32)

    def torch_fn(q_segment_ids, kv_segment_ids):
        return torch.where(q_segment_ids[:, None, :, None] == kv_segment_ids[:, None, None, :], 0.0, -torch.inf)

    def numpy_fn(q_segment_ids, kv_segment_ids):
        return np.where(q_segment_ids[:, None, :, None] == kv_segment_ids[:, None, None, :], 0.0, -np.inf)

    _both_ways(device, monkeypatch, "summary/reference-callable", 2, q_len, kv_len, h, d, 8, torch_fn, numpy_fn,
               {"q_segment_ids": qs}, {"kv_segment_ids": ks}, seed=seed)


@pytest.mark.parametrize("D,S,n,B,H", [(128, 4096, 4, 1, 2), (64, 3072, 3, 2, 2), (128, 2400, 3, 1, 2), (128, 1800, 1, 1, 1)])
def test_document_mask_callable_with_and_without_summary(device, monkeypatch, D, S, n, B, H):
    """Sorted documents as a callable's 0 / -inf block: whole tiles are -inf (left out), whole
    tiles are zero (straight-line stretches in the forward kernel), boundary tiles are mixed.
    Shard lengths on and off the tile grids (1024, 800, 1800)."""
    rng = np.random.default_rng(S + D)
    cuts = np.sort(rng.integers(1, S, (B, 5)), axis=1)
    seg = (np.arange(S)[None, :, None] >= cuts[:, None, :]).sum(-1).astype(np.int32)

    def torch_fn(q_segment_ids, kv_segment_ids):
        return torch.where(q_segment_ids[:, None, :, None] == kv_segment_ids[:, None, None, :], 0.0, -torch.inf)

    def numpy_fn(q_segment_ids, kv_segment_ids):
        return np.where(q_segment_ids[:, None, :, None] == kv_segment_ids[:, None, None, :], 0.0, -np.inf)

    _both_ways(device, monkeypatch, "summary/documents", B, S, S, H, D, n, torch_fn, numpy_fn,
               {"q_segment_ids": seg}, {"kv_segment_ids": seg}, seed=S)


def test_causal_document_mask_with_values_and_dead_rows(device, monkeypatch):
    """A per-head block that mixes everything: documents, a causal mask, finite values on part of
    the keys, zero elsewhere, and queries that see no key at all (their rows are -inf throughout:
    NaN output, -inf logsumexp, no gradient contribution, ring.py:134-135)."""
    B, S, H, D, n = 1, 4 * 640, 2, 128, 4
    rng = np.random.default_rng(11)
    cuts = np.sort(rng.integers(1, S, (B, 3)), axis=1)
    seg = (np.arange(S)[None, :, None] >= cuts[:, None, :]).sum(-1).astype(np.int32)
    pos = np.broadcast_to(np.arange(S, dtype=np.int32), (B, S)).copy()
    feat = (rng.standard_normal((B, S)) * (np.arange(S) % 700 < 200)).astype(np.float32)  # zero on most keys
    dead = np.zeros((B, S), dtype=np.int32)
    dead[:, 700:830] = 1

    def torch_fn(q_segment_ids, q_pos, q_dead, kv_segment_ids, kv_pos, kv_feat):
        ok = (q_segment_ids[:, None, :, None] == kv_segment_ids[:, None, None, :]) & \
             (kv_pos[:, None, None, :] <= q_pos[:, None, :, None]) & (q_dead[:, None, :, None] == 0)
        val = kv_feat[:, None, None, :] * torch.tensor([1.0, -0.5], device=kv_feat.device)[None, :, None, None]
        return torch.where(ok, val.expand(-1, -1, ok.shape[2], -1), -torch.inf)

    def numpy_fn(q_segment_ids, q_pos, q_dead, kv_segment_ids, kv_pos, kv_feat):
        ok = (q_segment_ids[:, None, :, None] == kv_segment_ids[:, None, None, :]) & \
             (kv_pos[:, None, None, :] <= q_pos[:, None, :, None]) & (q_dead[:, None, :, None] == 0)
        val = kv_feat[:, None, None, :].astype(np.float64) * np.array([1.0, -0.5])[None, :, None, None]
        return np.where(ok, np.broadcast_to(val, (B, 2, S, S)), -np.inf)

    _both_ways(device, monkeypatch, "summary/mixed", B, S, S, H, D, n, torch_fn, numpy_fn,
               {"q_segment_ids": seg, "q_pos": pos, "q_dead": dead},
               {"kv_segment_ids": seg, "kv_pos": pos, "kv_feat": feat}, seed=5)


def test_block_api_takes_a_summary_with_segment_ids(device, monkeypatch):
    """fwd_block / bwd_block with a BlockBias that carries segment ids AND a dense block: a tile is
    left out if either says so, and evaluated element by element if either needs it."""
    B, H, Lq, Lk, D = 1, 2, 768, 1024, 128
    rng = np.random.default_rng(3)
    q, k, v, do = R.make_inputs(9, B, Lq, Lk, H, D)
    qseg = (np.arange(Lq) >= 500).astype(np.int32)[None]
    kseg = (np.arange(Lk) >= 640).astype(np.int32)[None]
    dense = np.zeros((B, 1, Lq, Lk), dtype=np.float32)
    dense[..., :, 256:384] = -np.inf          # a band of keys nobody sees
    dense[..., 100:130, :64] = rng.standard_normal((30, 64))
    fn = ra.segment_bias()
    want_bias = R.make_bias_fn(use_segments=True)(q_segment_ids=qseg, kv_segment_ids=kseg,
                                                  q_positions=np.arange(Lq)[None], kv_positions=np.arange(Lk)[None])
    want_bias = want_bias + dense
    want, want_lse = R.mha_dense(q, k, v, want_bias)
    ref_g = R.mha_dense_grads(q, k, v, do, want_bias)
    hq, hk, hv, hdo = (np.ascontiguousarray(np.transpose(x, (0, 2, 1, 3))) for x in (q, k, v, do))
    tq, tk, tv, tdo = (_dev(x, device, torch.bfloat16) for x in (hq, hk, hv, hdo))
    for on in (True, False):
        monkeypatch.setattr(rbias, "DENSE_SUMMARY", on)
        bias = rr.BlockBias(fn, 0, 0, q_segment_ids=_dev(qseg, device), kv_segment_ids=_dev(kseg, device),
                            dense=_dev(dense, device))
        o, m, l = rr.init_carry(B, H, Lq, D, device)
        o, m, l = rr.fwd_block(tq, tk, tv, bias, o, m, l, D ** -0.5)
        out, lse = o / l[..., None], m + torch.log(l)
        dq, dk, dv = rr.bwd_block(tq, tk, tv, bias, out, lse, tdo, D ** -0.5)
        torch.cuda.synchronize()
        assert ("_summary" in bias.__dict__) == on
        assert np.abs(out.permute(0, 2, 1, 3).cpu().numpy() - want).max() <= OUT_TOL
        assert np.abs(lse.cpu().numpy() - want_lse).max() <= LSE_TOL
        for got, ref, nm in zip((dq, dk, dv), ref_g, ("dq", "dk", "dv")):
            mx, fro = _rel(got.permute(0, 2, 1, 3).cpu().numpy(), ref)
            assert mx <= GRAD_TOL and fro <= GRAD_TOL, (nm, on, mx, fro)

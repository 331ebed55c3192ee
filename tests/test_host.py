"""CPU-only checks of the host-side mirror of the reference interface (no kernels run)."""
import numpy as np
import pytest
import torch

import ring_attention as ra
from ring_attention import ring as rr
from ring_attention.bias import BiasFn


def test_public_names_match_reference_package():
    # reference __init__.py:3 re-exports exactly these two
    assert callable(ra.ring_attention) and callable(ra.ring_self_attention)


def test_bias_composition_and_flags():
    b = ra.causal_bias() + ra.segment_bias()
    assert b.causal and b.segments and b.flags == 1 | 4
    w = ra.sliding_window_bias(128) + ra.sliding_window_bias(64)
    assert w.window == 64 and w.flags == 1 | 2
    a = ra.alibi_bias([0.5, 0.25]) + ra.alibi_bias([0.5, 0.25])
    assert torch.allclose(a.alibi_slopes, torch.tensor([1.0, 0.5]))
    with pytest.raises(ValueError):
        ra.causal_bias() + ra.prefix_lm_bias()  # ring.py:368-374
    with pytest.raises(ValueError):
        ra.sliding_window_bias(0)
    np.testing.assert_allclose(ra.alibi_slopes(8).numpy(), [2.0 ** -(i + 1) for i in range(8)])


def test_cpu_tensors_fail_loudly():
    q = torch.zeros(1, 64, 1, 64)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ra.ring_attention(q, q, q, 2)


def test_block_impl_and_bias_type_errors():
    q = torch.zeros(1, 64, 1, 64)
    with pytest.raises(ValueError):
        ra.ring_attention(q, q, q, 2, block_impl="triton")  # ring.py:312 raises ValueError too
    # the reference's own two values are both accepted (ring.py:296-311): they get past the
    # block_impl check and fail on the CPU tensors like any other call
    for impl in ("jax", "pallas", "hip", "hip_fused"):
        with pytest.raises(RuntimeError, match="no CPU fallback"):
            ra.ring_attention(q, q, q, 2, block_impl=impl)
    with pytest.raises(TypeError):
        ra.ring_attention(q, q, q, 2, bias_fn="causal")  # neither a BiasFn nor a callable
    with pytest.raises(TypeError):
        rr._axis_size("sp")
    assert rr._axis_size(ra.RingAxis("sp", 8)) == 8 and rr._axis_size(("sp", 4)) == 4


def test_ring_self_attention_argument_rules():
    q = torch.zeros(1, 64, 1, 64)
    pos = torch.arange(64)[None]
    with pytest.raises(AssertionError):
        ra.ring_self_attention(q, q, q, 2, causal=True)  # positions required (ring.py:369)
    with pytest.raises(AssertionError):
        ra.ring_self_attention(q, q, q, 2, causal=True, positions=pos, prefix_mask=pos)  # ring.py:370
    with pytest.raises(AssertionError):
        ra.ring_self_attention(q, q, q, 2, prefix_mask=pos)  # ring.py:373


def test_long_segment_shards_are_walked_as_a_finer_ring():
    seg, causal = ra.segment_bias(), ra.causal_bias()
    cap = rr._lib.RA_MAX_SEGMENT_SHARD
    assert cap == 65536
    assert rr._walked_ring_size(1, 98304, 98304, seg + causal) == 2      # 2 x 49152
    assert rr._walked_ring_size(2, 4 * cap, 4 * cap, seg) == 4           # shards of 2 x cap -> cap
    assert rr._walked_ring_size(2, 4 * cap + 6, 4 * cap + 6, seg) == 10  # shards of 131075 = 5 x 26215
    assert rr._walked_ring_size(1, 98304, 1024, seg) == 2                # the longer side decides
    assert rr._walked_ring_size(1, 98304, 1023, seg) == 3                # ... and both must divide
    assert rr._walked_ring_size(8, 8 * cap, 8 * cap, seg) == 8           # at the limit: untouched
    assert rr._walked_ring_size(1, 98304, 98304, causal) == 1            # no segment term: no limit
    assert rr._walked_ring_size(1, 98304, 98304, None) == 1
    assert rr._walked_ring_size(1, 2 * 65537, 2 * 65537, seg) == 1       # 2 x a prime: left to the library's check


def test_ring_plan_shards_and_offsets():
    q = torch.zeros(2, 64, 2, 64, dtype=torch.bfloat16)
    k = torch.zeros(2, 32, 2, 64, dtype=torch.bfloat16)
    seg_q = torch.arange(64)[None].repeat(2, 1) // 10
    seg_k = torch.arange(32)[None].repeat(2, 1) // 10
    plan = rr._RingPlan(q, k, 4, ra.causal_bias() + ra.segment_bias(),
                        {"q_segment_ids": seg_q, "q_positions": torch.arange(64)[None].repeat(2, 1) + 100},
                        {"kv_segment_ids": seg_k})
    assert (plan.Lq, plan.Lk) == (16, 8)
    assert plan.q_off == [100, 116, 132, 148] and plan.kv_off == [0, 8, 16, 24]
    bb = plan.block_bias(2, 3)
    assert bb.q_offset == 132 and bb.kv_offset == 24
    assert torch.equal(bb.q_segment_ids, seg_q[:, 32:48].to(torch.int32))
    assert torch.equal(bb.kv_segment_ids, seg_k[:, 24:32].to(torch.int32))
    # shards may restart their positions, but must be consecutive inside
    pos = torch.cat([torch.arange(16) + 7 * i for i in range(4)])[None].repeat(2, 1)
    plan = rr._RingPlan(q, k, 4, ra.causal_bias(), {"q_positions": pos}, {})
    assert plan.q_off == [0, 7, 14, 21]
    # any other positions are honoured through a dense block per ring step, built from the
    # position arrays exactly like the reference's mask builder (ring.py:393-409)
    plan = rr._RingPlan(q, k, 4, ra.causal_bias() + ra.segment_bias(),
                        {"q_positions": pos * 2, "q_segment_ids": seg_q}, {"kv_segment_ids": seg_k})
    assert plan.callable is not None and plan.fn is None
    bb = plan.block_bias(1, 2)
    assert tuple(bb.dense.shape) == (2, 1, 16, 8)
    qp, kp = (pos * 2)[:, 16:32], torch.arange(32)[None].repeat(2, 1)[:, 16:24]
    want = (kp[:, None, :] <= qp[:, :, None]) & (seg_q[:, 16:32, None] == seg_k[:, None, 16:24])
    assert torch.equal(bb.dense[:, 0] == 0, want) and torch.equal(torch.isneginf(bb.dense[:, 0]), ~want)
    # positions that differ across the batch take the same path
    pos_b = torch.stack([torch.arange(64), torch.arange(64) + 3])
    assert rr._RingPlan(q, k, 4, ra.causal_bias(), {"q_positions": pos_b}, {}).callable is not None
    with pytest.raises(ValueError):
        rr._RingPlan(q, k, 3, None, None, None)  # 64 % 3 != 0
    with pytest.raises(ValueError):
        rr._RingPlan(q, k, 4, ra.segment_bias(), {"q_segment_ids": seg_q}, {})
    with pytest.raises(ValueError):
        rr._RingPlan(q, k, 4, ra.causal_bias(), {"bogus": seg_q}, {})
    with pytest.raises(ValueError):
        rr._RingPlan(q, k, 4, None, {"q_segment_ids": seg_q}, {})


def test_ring_plan_counts_the_steps_that_cost_something():
    q = torch.zeros(1, 64, 1, 64, dtype=torch.bfloat16)
    plan = rr._RingPlan(q, q, 4, ra.causal_bias(), None, None)
    assert [plan.live_steps(r, None) for r in range(4)] == [1, 2, 3, 4]
    assert [plan.live_steps(None, r) for r in range(4)] == [4, 3, 2, 1]
    plan = rr._RingPlan(q, q, 4, ra.sliding_window_bias(18), None, None)  # shards of 16 tokens
    assert [plan.live_steps(r, None) for r in range(4)] == [1, 2, 3, 3]
    plan = rr._RingPlan(q, q, 4, ra.sliding_window_bias(5, causal=False), None, None)
    assert [plan.live_steps(r, None) for r in range(4)] == [2, 3, 3, 2]
    assert rr._RingPlan(q, q, 4, None, None, None).live_steps(2, None) == 4
    # agrees with the library's own classification of a step
    lib = rr._lib.load()
    for fn in (ra.causal_bias(), ra.sliding_window_bias(17), ra.sliding_window_bias(18), ra.sliding_window_bias(5, causal=False)):
        plan = rr._RingPlan(q, q, 4, fn, None, None)
        for r in range(4):
            live = 0
            for s in range(4):
                st = plan.block_bias(r, s).to_struct(torch.device("cpu"))
                live += not lib.ra_step_is_skippable(st, 16, 16)
            assert plan.live_steps(r, None) == live


def test_ring_plan_with_a_callable_bias_fn():
    # the reference's general form: the callable sees the shards of its kwargs (ring.py:107,186)
    q = torch.zeros(2, 64, 2, 64, dtype=torch.bfloat16)
    k = torch.zeros(2, 32, 2, 64, dtype=torch.bfloat16)
    feat_q = torch.arange(2 * 64 * 3, dtype=torch.float32).reshape(2, 64, 3)
    ids_k = torch.arange(32)[None].repeat(2, 1)
    seen = {}

    def fn(q_feat, kv_ids):
        seen["q"], seen["k"] = q_feat, kv_ids
        return torch.zeros(2, 1, q_feat.shape[1], kv_ids.shape[1])

    plan = rr._RingPlan(q, k, 4, fn, {"q_feat": feat_q}, {"kv_ids": ids_k})
    bb = plan.block_bias(2, 3)
    assert torch.equal(seen["q"], feat_q[:, 32:48]) and torch.equal(seen["k"], ids_k[:, 24:32])
    assert bb.dense.shape == (2, 1, 16, 8) and bb.fn.flags == 0
    bb.check_dense_shape(2, 2, 16, 8)
    with pytest.raises(ValueError):
        bb.check_dense_shape(2, 2, 16, 9)
    s = bb.to_struct(torch.device("cpu"))
    assert s.flags == 32 and s.dense_stride_h == 0 and s.dense_stride_q == 8 and s.dense_stride_b == 128
    with pytest.raises(ValueError):
        rr._RingPlan(q, k, 4, fn, {"q_feat": feat_q[:, :10]}, {"kv_ids": ids_k})
    with pytest.raises(TypeError):
        rr._RingPlan(q, k, 4, lambda **kw: None, {}, {}).block_bias(0, 0)


def test_shard_view_is_zero_copy():
    x = torch.arange(2 * 8 * 3 * 4).reshape(2, 8, 3, 4)
    s = rr._shard_bhld(x, 1, 4)
    assert s.shape == (2, 3, 4, 4) and s.data_ptr() == x[:, 4:].data_ptr()
    assert torch.equal(s[1, 2, 3], x[1, 7, 2])


def test_launch_scheme_per_block_impl():
    q = torch.zeros(1, 64, 1, 64, dtype=torch.bfloat16)
    plain = rr._RingPlan(q, q, 4, ra.causal_bias(), None, None)
    dense = rr._RingPlan(q, q, 4, lambda q_ids, kv_ids: torch.zeros(1, 1, 16, 16),
                         {"q_ids": torch.zeros(1, 64)}, {"kv_ids": torch.zeros(1, 64)})
    # the reference's default spelling picks the scheme; its "jax" is the plain per-step loop
    assert rr._launch_whole_ring("pallas", plain) and not rr._launch_whole_ring("pallas", dense)
    assert not rr._launch_whole_ring("jax", plain) and not rr._launch_whole_ring("hip", plain)
    assert rr._launch_whole_ring("hip_fused", plain) and rr._launch_whole_ring("hip_fused", dense)
    import inspect
    for f in (ra.ring_attention, ra.ring_self_attention, ra.ring_attention_with_lse):
        assert inspect.signature(f).parameters["block_impl"].default == "pallas"  # ring.py:255


def test_plans_are_cached_per_bias_arrays():
    ra.clear_plan_cache()
    q = torch.zeros(2, 64, 2, 64, dtype=torch.bfloat16)
    seg = torch.arange(64)[None].repeat(2, 1) // 10
    fn = ra.causal_bias() + ra.segment_bias()
    a = rr._plan_for(q, q, 4, fn, {"q_segment_ids": seg}, {"kv_segment_ids": seg})
    assert rr._plan_for(q, q, 4, fn, {"q_segment_ids": seg}, {"kv_segment_ids": seg}) is a
    assert rr._plan_for(q, q, 4, ra.causal_bias() + ra.segment_bias(), {"q_segment_ids": seg},
                        {"kv_segment_ids": seg}) is a           # an equal description, not the same object
    assert rr._plan_for(q, q, 2, fn, {"q_segment_ids": seg}, {"kv_segment_ids": seg}) is not a
    seg2 = seg.clone()
    assert rr._plan_for(q, q, 4, fn, {"q_segment_ids": seg2}, {"kv_segment_ids": seg2}) is not a
    seg += 1                                                    # in place: a new version of the same tensor
    b = rr._plan_for(q, q, 4, fn, {"q_segment_ids": seg}, {"kv_segment_ids": seg})
    assert b is not a and torch.equal(b.q_seg, seg.to(torch.int32))
    # positions are read back on the host when a plan is made: the offsets follow the array
    pos = torch.arange(64)[None].repeat(2, 1)
    p1 = rr._plan_for(q, q, 4, ra.causal_bias(), {"q_positions": pos}, {})
    pos += 5
    p2 = rr._plan_for(q, q, 4, ra.causal_bias(), {"q_positions": pos}, {})
    assert p1.q_off == [0, 16, 32, 48] and p2.q_off == [5, 21, 37, 53]
    for i in range(20):                                         # bounded
        rr._plan_for(q, q, 4, ra.sliding_window_bias(i + 1), None, None)
    assert len(rr._PLAN_CACHE) <= rr._PLAN_CACHE_SIZE
    ra.clear_plan_cache()
    assert not rr._PLAN_CACHE


def test_a_callable_bias_is_built_in_bounded_chunks():
    q = torch.zeros(1, 256, 1, 64, dtype=torch.bfloat16)
    calls = []

    def fn(q_ids, kv_ids):
        calls.append((int(q_ids[0, 0]), int(kv_ids[0, 0])))
        return torch.zeros(1, 1, q_ids.shape[1], kv_ids.shape[1])

    ids = torch.arange(256)[None]
    plan = rr._RingPlan(q, q, 32, fn, {"q_ids": ids}, {"kv_ids": ids})
    chunks = list(rr._row_chunks(plan, 3))
    assert [len(c) for c in chunks] == [16, 16]                 # what one launch walks
    assert [s for c in chunks for s, _ in c] == [(3 - t) % 32 for t in range(32)]   # ring order, ring.py:51-55
    assert len(calls) == 32 and all(a == 24 for a, _ in calls)  # one block per pair, each built once
    old = rr._DENSE_BLOCKS_BYTES
    try:
        rr._DENSE_BLOCKS_BYTES = 3 * 8 * 8 * 4                  # three 8 x 8 blocks
        assert [len(c) for c in rr._row_chunks(plan, 0)] == [3] * 10 + [2]
    finally:
        rr._DENSE_BLOCKS_BYTES = old


def test_views_the_kernels_cannot_take_are_copied():
    # a view is passed through when its rows are 16-byte aligned, do not overlap and lie within the
    # row stride of the C ABI; otherwise the host makes a contiguous copy
    base = torch.zeros((2, 16, 4, 64 + 8), dtype=torch.bfloat16)
    padded = base[..., :64]                       # row stride 4 * 72, inner stride 1
    assert rr._kernel_ready(padded) is padded
    odd = torch.zeros((2, 16, 4, 65), dtype=torch.bfloat16)[..., :64]   # strides not multiples of 8
    assert rr._kernel_ready(odd).is_contiguous()
    same_row = torch.zeros((2, 1, 4, 64), dtype=torch.bfloat16).expand(2, 16, 4, 64)   # row stride 0
    got = rr._kernel_ready(same_row)
    assert got.is_contiguous() and got.shape == same_row.shape
    heads_interleaved = torch.zeros((2, 4, 16, 64), dtype=torch.bfloat16).permute(0, 2, 1, 3)  # [b, l, h, d] view, row stride 64
    assert rr._kernel_ready(heads_interleaved) is heads_interleaved
    assert rr._kernel_ready(torch.zeros((1, 8, 1, 64))).dtype == torch.bfloat16

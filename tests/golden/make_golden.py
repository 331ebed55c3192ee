"""Writes tests/golden/*.npz: small seeded inputs with expected outputs.

The reference ships no golden vectors (its tests compute every expected value in-test with a
dense softmax, ring_test.py:26-42) and cannot be imported here (jax is absent), so the
expected values are produced by the same closed form in fp64 (oracle.ring_oracle.mha_dense /
mha_dense_grads, themselves pinned against scipy and torch.autograd in tests/test_oracle.py).
The fixtures freeze inputs AND outputs, so a later change to the oracle or to the input
generator cannot silently move the target.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import ring_oracle as R  # noqa: E402

CASES = {
    # name: (seed, B, Lq, Lk, H, D, ring, bias kind)
    "fwd_bwd_nobias_d64": (11, 1, 64, 128, 2, 64, 2, None),
    "fwd_bwd_causal_d128": (12, 1, 128, 128, 1, 128, 4, "causal"),
    "fwd_bwd_causal_segments_d64": (13, 2, 128, 128, 2, 64, 4, "causal+segments"),
    "fwd_bwd_window_alibi_d64": (14, 1, 128, 128, 2, 64, 2, "window+alibi"),
}


def build(name):
    seed, B, Lq, Lk, H, D, n, kind = CASES[name]
    q, k, v, do = R.make_inputs(seed, B, Lq, Lk, H, D)
    rng = np.random.default_rng(seed + 1000)
    qpos = np.broadcast_to(np.arange(Lq), (B, Lq)).astype(np.int32)
    kpos = np.broadcast_to(np.arange(Lk), (B, Lk)).astype(np.int32)
    seg = np.sort(rng.integers(0, 4, (B, Lq)), axis=1).astype(np.int32)
    slopes = R.alibi_slopes(H)
    bias = None
    if kind == "causal":
        bias = R.make_bias_fn(causal=True)(q_positions=qpos, kv_positions=kpos)
    elif kind == "causal+segments":
        bias = R.make_bias_fn(causal=True, use_segments=True)(
            q_positions=qpos, kv_positions=kpos, q_segment_ids=seg, kv_segment_ids=seg)
    elif kind == "window+alibi":
        bias = R.make_bias_fn(causal=True, window=40, alibi=slopes)(q_positions=qpos, kv_positions=kpos)
    out, lse = R.mha_dense(q, k, v, bias)
    dq, dk, dv = R.mha_dense_grads(q, k, v, do, bias)
    np.savez_compressed(
        os.path.join(HERE, name + ".npz"), q=q, k=k, v=v, do=do, seg=seg, slopes=slopes,
        ring=np.int32(n), out=out.astype(np.float32), lse=lse.astype(np.float32),
        dq=dq.astype(np.float32), dk=dk.astype(np.float32), dv=dv.astype(np.float32))


if __name__ == "__main__":
    for name in CASES:
        build(name)
        print("wrote", name)

"""CPU-only checks of the C ABI: the library loads, exports what include/ring_attention_hip.h
declares, rejects bad arguments before touching a GPU, and classifies skippable ring steps
exactly like a brute-force evaluation of the bias."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from oracle import ring_oracle as R
from ring_attention import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ring_attention_hip.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ra_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(lib):
    names = _declared()
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), f"{n} declared in the header but not exported"
    assert sorted(_lib.EXPORTS) == names, "python binding table and header disagree"
    assert lib.ra_version() >= 1000


def test_struct_layout_matches_header():
    # sizes implied by the header with natural alignment on x86-64
    assert C.sizeof(_lib.RaTensor) == 32
    assert C.sizeof(_lib.RaBias) == 8 + 16 + 16 + 16 + 16 + 16 + 8 + 8 + 24 + 8
    assert C.sizeof(_lib.RaFwdStepParams) == 24 + 3 * 32 + 24 + C.sizeof(_lib.RaBias)
    assert C.sizeof(_lib.RaBwdStepParams) == 24 + 4 * 32 + 40 + C.sizeof(_lib.RaBias)


def _good_fwd():
    p = _lib.RaFwdStepParams()
    p.B, p.H, p.Lq, p.Lk, p.D = 1, 2, 64, 64, 128
    p.sm_scale = 0.1
    for t in (p.q, p.k, p.v):
        t.ptr, t.stride_b, t.stride_h, t.stride_l = 0x1000, 64 * 256, 128, 256
    p.o = p.m = p.l = 0x2000
    return p


def _good_bwd():
    p = _lib.RaBwdStepParams()
    p.B, p.H, p.Lq, p.Lk, p.D = 1, 2, 64, 64, 64
    p.sm_scale = 0.1
    for t in (p.q, p.k, p.v, p.dout):
        t.ptr, t.stride_b, t.stride_h, t.stride_l = 0x1000, 64 * 128, 64, 128
    p.lse = p.delta = p.dq = p.dk = p.dv = 0x2000
    return p


def test_check_accepts_good_params(lib):
    assert lib.ra_fwd_step_check(C.byref(_good_fwd())) == 0
    assert lib.ra_bwd_step_check(C.byref(_good_bwd())) == 0


@pytest.mark.parametrize("mutate,code", [
    (lambda p: setattr(p, "D", 96), -3),
    (lambda p: setattr(p, "D", 256), -3),
    (lambda p: setattr(p, "Lq", 0), -2),
    (lambda p: setattr(p, "B", -1), -2),
    (lambda p: setattr(p.q, "ptr", None), -1),
    (lambda p: setattr(p.k, "ptr", 0x1008), -4),
    (lambda p: setattr(p.v, "stride_l", 129), -4),
    (lambda p: setattr(p, "o", None), -1),
    (lambda p: setattr(p, "sm_scale", float("nan")), -2),
    (lambda p: setattr(p.bias, "flags", 64), -5),
    (lambda p: setattr(p.bias, "flags", _lib.RA_BIAS_WINDOW), -5),            # window == 0
    (lambda p: setattr(p.bias, "flags", _lib.RA_BIAS_CAUSAL | _lib.RA_BIAS_PREFIX), -5),
    (lambda p: setattr(p.bias, "flags", _lib.RA_BIAS_SEGMENT), -1),           # no id arrays
    (lambda p: setattr(p.bias, "flags", _lib.RA_BIAS_ALIBI), -1),             # no slopes
    (lambda p: setattr(p.bias, "flags", _lib.RA_BIAS_DENSE), -1),             # no dense block
    (lambda p: (setattr(p.bias, "flags", _lib.RA_BIAS_DENSE), setattr(p.bias, "dense_bias", 0x3000),
                setattr(p.bias, "dense_stride_q", 63)), -5),                  # rows overlap
    (lambda p: (setattr(p.bias, "flags", _lib.RA_BIAS_DENSE), setattr(p.bias, "dense_bias", 0x3002),
                setattr(p.bias, "dense_stride_q", 64)), -4),
    (lambda p: (setattr(p.bias, "flags", _lib.RA_BIAS_CAUSAL), setattr(p.bias, "q_offset", -5)), -5),
    # positions (offset + index) stay below RA_MAX_POSITION: the last token of the shard counts
    (lambda p: (setattr(p.bias, "flags", _lib.RA_BIAS_CAUSAL),
                setattr(p.bias, "q_offset", _lib.RA_MAX_POSITION - p.Lq + 1)), -5),
    (lambda p: (setattr(p.bias, "flags", _lib.RA_BIAS_CAUSAL),
                setattr(p.bias, "kv_offset", _lib.RA_MAX_POSITION - p.Lk + 1)), -5),
])
def test_fwd_step_rejects_bad_params_without_a_gpu(lib, mutate, code):
    p = _good_fwd()
    mutate(p)
    assert lib.ra_fwd_step_check(C.byref(p)) == code
    assert lib.ra_fwd_step(C.byref(p), None) == code  # validation comes before any HIP call
    assert lib.ra_last_error() != b""


def test_position_and_window_limits(lib):
    # the largest positions and any window width pass the checks (a window wider than every
    # position difference masks nothing and is clamped inside the library)
    p = _good_fwd()
    p.bias.flags = _lib.RA_BIAS_CAUSAL | _lib.RA_BIAS_WINDOW
    p.bias.window = 2 ** 31 - 1
    p.bias.q_offset = _lib.RA_MAX_POSITION - p.Lq
    p.bias.kv_offset = _lib.RA_MAX_POSITION - p.Lk
    assert lib.ra_fwd_step_check(C.byref(p)) == 0
    # a step against keys 2^30 positions behind a window of 2^31 - 1 still has work; one beyond a
    # small window has none
    p.bias.kv_offset = 0
    assert lib.ra_step_is_skippable(C.byref(p.bias), p.Lq, p.Lk) == 0
    p.bias.window = 1000
    assert lib.ra_step_is_skippable(C.byref(p.bias), p.Lq, p.Lk) == 1


def test_row_stride_limits(lib):
    # rows may not overlap (stride_l >= D) and the row stride stays within 2^27 elements: the kernels
    # reach the rows one wavefront moves through a 32-bit byte offset from the wavefront's first row
    for bad in (0, -128, 64, _lib.RA_MAX_ROW_STRIDE + 8):
        p = _good_fwd()
        p.k.stride_l = bad
        assert p.D == 128 and lib.ra_fwd_step_check(C.byref(p)) == -2, bad
        assert b"row stride" in lib.ra_last_error()
        p = _good_bwd()
        p.dout.stride_l = min(bad, 56)  # D = 64 there
        assert lib.ra_bwd_step_check(C.byref(p)) == -2, bad
    for good in (128, 136, _lib.RA_MAX_ROW_STRIDE):
        p = _good_fwd()
        p.v.stride_l = good
        assert lib.ra_fwd_step_check(C.byref(p)) == 0, good


def test_dense_map_arguments_are_checked_without_a_gpu(lib):
    """ra_dense_map_bytes is plain arithmetic; ra_dense_map and a step that carries a summary
    refuse bad arguments before anything is launched."""
    assert lib.ra_dense_map_bytes(0, 0, 2, 3, 64, 64) == 4
    assert lib.ra_dense_map_bytes(1 << 20, 0, 2, 3, 100, 250) == 2 * 4 * 8
    assert lib.ra_dense_map_bytes(1 << 20, 1 << 16, 2, 3, 33, 1031) == 2 * 3 * 2 * 33
    assert lib.ra_dense_map_bytes(0, 0, 0, 3, 64, 64) == 0
    good = dict(dense_bias=0x1000, stride_b=0, stride_h=0, stride_q=64, B=1, H=1, Lq=64, Lk=64, map=0x2000)

    def call(**kw):
        a = {**good, **kw}
        return lib.ra_dense_map(a["dense_bias"], a["stride_b"], a["stride_h"], a["stride_q"], a["B"], a["H"],
                                a["Lq"], a["Lk"], a["map"], None)

    assert call(dense_bias=None) == -1 and call(map=None) == -1          # RA_ERR_NULL
    assert call(Lq=0) == -2 and call(B=-1) == -2                          # RA_ERR_SHAPE
    assert call(Lk=_lib.RA_MAX_SEGMENT_SHARD + 1, stride_q=1 << 20) == -2
    assert call(dense_bias=0x1002) == -4                                  # RA_ERR_ALIGN
    assert call(stride_q=63) == -5 and call(stride_b=-8) == -5            # RA_ERR_BIAS
    # a step whose dense block comes with a summary: shards of at most RA_MAX_SEGMENT_SHARD tokens
    p = _good_fwd()
    p.bias.flags = _lib.RA_BIAS_DENSE
    p.bias.dense_bias, p.bias.dense_stride_q, p.bias.dense_map = 0x3000, 64, 0x4000
    assert lib.ra_fwd_step_check(C.byref(p)) == 0
    p.Lk = _lib.RA_MAX_SEGMENT_SHARD + 64
    p.bias.dense_stride_q = p.Lk
    assert lib.ra_fwd_step_check(C.byref(p)) == -2 and b"summary" in lib.ra_last_error()
    p.bias.dense_map = None
    assert lib.ra_fwd_step_check(C.byref(p)) == 0


def test_bwd_step_rejects_bad_params_without_a_gpu(lib):
    p = _good_bwd()
    p.dk = None
    assert lib.ra_bwd_step(C.byref(p), None) == -1
    p = _good_bwd()
    p.dout.stride_h = 3
    assert lib.ra_bwd_step(C.byref(p), None) == -4
    p = _good_bwd()
    assert lib.ra_bwd_step_parts(C.byref(p), 7, None) == -2
    assert lib.ra_fwd_step(None, None) == -1
    assert lib.ra_fwd_init(None, None, None, 1, 1, 1, 64, None) == -1
    assert lib.ra_fwd_finalize(0x10, 0x10, 0x10, 0x10, 5, 8, 8, 8, 0x10, 1, 1, 1, 64, None) == -7


def test_finalize_entry_points_check_alignment_without_a_gpu(lib):
    # ra_fwd_finalize stores four elements at a time: out must be aligned to 8 (bf16) / 16 (fp32) bytes
    ok = (0x1000, 0x1000, 0x1000)
    assert lib.ra_fwd_finalize(*ok, 0x2004, _lib.RA_DTYPE_BF16, 128, 128, 128, 0x3000, 1, 1, 4, 64, None) == -4
    assert b"aligned" in lib.ra_last_error()
    assert lib.ra_fwd_finalize(*ok, 0x2008, _lib.RA_DTYPE_F32, 128, 128, 128, 0x3000, 1, 1, 4, 64, None) == -4
    assert lib.ra_fwd_finalize(0x1004, 0x1000, 0x1000, 0x2000, _lib.RA_DTYPE_F32, 128, 128, 128, 0x3000,
                               1, 1, 4, 64, None) == -4
    assert lib.ra_fwd_finalize(*ok, 0x2000, _lib.RA_DTYPE_F32, 130, 128, 128, 0x3000, 1, 1, 4, 64, None) == -4
    # ra_bwd_finalize loads 16 bytes of fp32 and stores 8 bytes of bf16 at a time
    assert lib.ra_bwd_finalize(0x1000, 0x2004, 128, 128, 128, 1, 1, 4, 64, None) == -4
    assert b"8-byte" in lib.ra_last_error()
    assert lib.ra_bwd_finalize(0x1008, 0x2000, 128, 128, 128, 1, 1, 4, 64, None) == -4
    assert lib.ra_bwd_finalize(0x1000, 0x2000, 128, 126, 128, 1, 1, 4, 64, None) == -4


def test_grids_beyond_the_launch_limit_are_rejected(lib):
    # B*H*ceil(L/128) workgroups must fit a 31-bit grid dimension: a larger launch would be cut short
    p = _good_fwd()
    p.B, p.H, p.Lq = 1 << 10, 1 << 10, 1 << 22      # 2^20 heads x 2^15 tiles = 2^35 workgroups
    assert lib.ra_fwd_step_check(C.byref(p)) == -2 and b"grid" in lib.ra_last_error()
    p.Lq, p.Lk = 64, 1 << 22                          # the key side counts as well (dK/dV grid)
    assert lib.ra_fwd_step_check(C.byref(p)) == -2
    b = _good_bwd()
    b.B, b.H, b.Lk = 1 << 10, 1 << 10, 1 << 22
    assert lib.ra_bwd_step_check(C.byref(b)) == -2
    p = _good_fwd()
    p.B, p.H, p.Lq = 1 << 10, 1 << 10, 1 << 17      # 2^30 workgroups: still fine
    assert lib.ra_fwd_step_check(C.byref(p)) == 0


@pytest.mark.parametrize("flags,window", [(1, 0), (3, 7), (2, 7), (3, 64), (2, 1), (0, 0), (8, 0)])
def test_step_is_skippable_matches_brute_force(lib, flags, window):
    Lq, Lk = 16, 24
    for q_off in (0, 16, 40, 100):
        for kv_off in (0, 24, 48, 96):
            b = _lib.RaBias()
            b.flags, b.window, b.q_offset, b.kv_offset = flags, window, q_off, kv_off
            got = lib.ra_step_is_skippable(C.byref(b), Lq, Lk)
            qp = (q_off + np.arange(Lq))[None]
            kp = (kv_off + np.arange(Lk))[None]
            fn = R.make_bias_fn(causal=bool(flags & 1), window=window if flags & 2 else None,
                                use_prefix=bool(flags & 8))
            pm_q = np.ones((1, Lq), dtype=np.int32); pm_k = np.ones((1, Lk), dtype=np.int32)
            bias = fn(q_positions=qp, kv_positions=kp, q_prefix_mask=pm_q, kv_prefix_mask=pm_k)
            want = int(np.all(np.isneginf(bias)))
            if flags & 8:
                want = 0  # prefix masks are data dependent: never skipped on the host
            assert got == want, (flags, window, q_off, kv_off)


def _steps(make, n):
    arr = (type(make()) * n)()
    for i in range(n):
        arr[i] = make()
    return arr


def test_multi_step_entry_points_validate_before_any_gpu_call(lib):
    # nothing to do / bad counts
    assert lib.ra_fwd_steps(None, 0, None) == 0
    assert lib.ra_fwd_steps(None, 2, None) == -1
    assert lib.ra_bwd_dq_steps(None, -1, None) == -2
    assert lib.ra_bwd_dkdv_steps(None, 3, None) == -1
    # every block goes through the single-step checks
    f = _steps(_good_fwd, 3)
    f[2].D = 96
    assert lib.ra_fwd_steps(f, 3, None) == -3
    # the blocks of one launch may differ in the travelling shard only
    f = _steps(_good_fwd, 2)
    f[1].o = 0x3000
    assert lib.ra_fwd_steps(f, 2, None) == -2 and b"steps[1]" in lib.ra_last_error()
    f = _steps(_good_fwd, 2)
    f[1].k.stride_l = 512
    assert lib.ra_fwd_steps(f, 2, None) == -2
    f = _steps(_good_fwd, 2)
    f[1].bias.q_offset = 64
    assert lib.ra_fwd_steps(f, 2, None) == -2
    b = _steps(_good_bwd, 2)
    b[1].lse = 0x4000          # the query side is fixed in a dq launch ...
    assert lib.ra_bwd_dq_steps(b, 2, None) == -2
    b = _steps(_good_bwd, 2)
    b[1].dk = 0x4000           # ... and the key/value side in a dk/dv launch
    assert lib.ra_bwd_dkdv_steps(b, 2, None) == -2
    b = _steps(_good_bwd, 2)
    b[1].bias.kv_offset = 64
    assert lib.ra_bwd_dkdv_steps(b, 2, None) == -2
    # steps that are masked entirely are dropped on the host: nothing is launched for these
    for arr, fn in ((_steps(_good_fwd, 2), lib.ra_fwd_steps), (_steps(_good_bwd, 2), lib.ra_bwd_dq_steps),
                    (_steps(_good_bwd, 2), lib.ra_bwd_dkdv_steps)):
        for p in arr:
            p.bias.flags = _lib.RA_BIAS_CAUSAL
            p.bias.kv_offset = 1 << 20
        assert fn(arr, 2, None) == 0


def test_header_is_plain_c(tmp_path):
    """include/ring_attention_hip.h must compile as C99 on its own (no HIP, no C++)."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    src = tmp_path / "hdr.c"
    src.write_text('#include "ring_attention_hip.h"\n'
                   "int main(void) { ra_fwd_step_params p; (void)p; return RA_OK; }\n")
    res = subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only",
                          "-I", os.path.join(ROOT, "include"), str(src)], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr

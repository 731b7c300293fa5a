"""The int8 instructions the CPU backend keeps un-lowered besides Relu and the
ones a lowered FullyConnected leaves behind: Clip, LeakyRelu, CPUMaxSplat and
BatchedAdd (reference LLVMBackend.cpp:69-79, CPUBackend.cpp:71-84,
LLVMIRGen.cpp:1501-1590, 2322-2375, CPULLVMIRGen.cpp:135-167). The backend
derives their integer parameters from the tensors' float scales; the oracle
derives them again, by the reference's formulas, and runs libjit's arithmetic."""
import numpy as np
import pytest

from glow_amd import host as H
from oracle import glow_oracle as go

f32 = np.float32


def _s(ratio):
    return go.quantize_scale_offset_32to8(float(f32(ratio)), 0)[:3]


def _q8(x, scale, offset):
    return int(np.clip(go.quantize_value_i32(x, scale, offset), -128, 127))


def _module():
    """Relu6 behind an Add (a Clip no convolution can absorb), a LeakyRelu, a
    Max(x, Splat) and a MatMul + BatchedAdd pair, on one input."""
    rng = np.random.default_rng(31)
    n, k, cols = 96, 64, 48
    m = H.Module("element_kinds")
    x = m.placeholder("x", (n, k), H.INT8Q, np.int8, 0.05, -3)
    y = m.placeholder("y", (n, k), H.INT8Q, np.int8, 0.07, 4)
    clip_out = m.placeholder("clip_out", (n, k), H.INT8Q, np.int8, 0.03, -128)
    leaky_out = m.placeholder("leaky_out", (n, k), H.INT8Q, np.int8, 0.04, -10)
    max_out = m.placeholder("max_out", (n, k), H.INT8Q, np.int8, 0.05, -3)
    fc8_out = m.placeholder("fc8_out", (n, cols), H.INT8Q, np.int8, 0.9, 2)
    fc32_out = m.placeholder("fc32_out", (n, cols), H.INT8Q, np.int8, 0.8, -5)
    w = rng.integers(-128, 128, (k, cols)).astype(np.int8)
    b8 = rng.integers(-128, 128, cols).astype(np.int8)
    b32 = rng.integers(-30000, 30000, cols).astype(np.int32)
    wv = m.constant("w", w, H.INT8Q, 0.02, 1)
    b8v = m.constant("b8", b8, H.INT8Q, 0.5, -7)
    b32v = m.constant("b32", b32, H.INT32Q, 0.001, 0)
    f = m.function("main")
    s = m.activation(f, "sum", (n, k), H.INT8Q, 0.09, 5)
    mm = m.activation(f, "mm", (n, cols), H.INT8Q, 0.7, -1)
    m.instruction(f, H.ELEMENT_ADD, "add", [s, x, y])
    m.instruction(f, H.CLIP, "relu6", [clip_out, s], (), (0.0, 6.0))
    m.instruction(f, H.LEAKY_RELU, "leaky", [leaky_out, s], (), (0.1,))
    m.instruction(f, H.CPU_MAX_SPLAT, "max0", [max_out, x], (), (0.0,))
    m.instruction(f, H.MATMUL, "matmul", [mm, x, wv])
    m.instruction(f, H.BATCHED_ADD, "bias8", [fc8_out, mm, b8v])
    m.instruction(f, H.BATCHED_ADD, "bias32", [fc32_out, mm, b32v])
    return m, f, dict(w=w, b8=b8, b32=b32, n=n, k=k, cols=cols)


def _expected(c, x, y):
    s = go.add_i8(x, y, 5, -3, 4, _s(f32(0.05) / f32(0.09)), _s(f32(0.07) / f32(0.09)))
    clip = go.clip_elem_i8(s, _q8(0.0, 0.09, 5), _q8(6.0, 0.09, 5), 5, -128,
                           _s(f32(0.09) / f32(0.03)))
    leaky = go.leaky_relu_i8(s, 5, -10, _s(f32(0.09) / f32(0.04)),
                             _s(f32(0.09) * f32(0.1) / f32(0.04)))
    mx = go.max_splat_i8(x, _q8(0.0, 0.05, -3))
    mm = go.matmul_i8(x, c["w"], -1, -3, 1, _s(f32(0.05) * f32(0.02) / f32(0.7)))
    fc8 = go.batched_add_i8(mm, c["b8"], 2, -1, -7, _s(f32(0.7) / f32(0.9)),
                            _s(f32(0.5) / f32(0.9)))
    fc32 = go.batched_add_i8(mm, c["b32"], -5, -1, 0, _s(f32(0.7) / f32(0.8)),
                             _s(f32(0.001) / f32(0.8)))
    return dict(clip_out=clip, leaky_out=leaky, max_out=mx, fc8_out=fc8, fc32_out=fc32)


def test_kinds_compile_to_their_kernels():
    m, f, _ = _module()
    m.compile(f, fuse_add_relu=False)
    rows = [r for r in H.parse_listing(m.describe(f)) if r["phase"] == "launch"]
    k = [r["kernel"] for r in rows]
    assert k == ["mi355x_add_i8", "mi355x_clip_i8", "mi355x_leaky_relu_i8",
                 "mi355x_max_splat_i8", "mi355x_matmul_i8", "mi355x_batched_add_i8",
                 "mi355x_batched_add_i8"]
    clip = rows[1]
    lo, hi = _q8(0.0, 0.09, 5), _q8(6.0, 0.09, 5)
    pre, post, scale = _s(f32(0.09) / f32(0.03))
    assert (clip["clip_min"], clip["clip_max"], clip["src_offset"], clip["dest_offset"]) == \
        (lo, hi, 5, -128)
    assert (clip["pre"], clip["post"], clip["scale"]) == (pre, post, scale)
    leaky = rows[2]
    assert (leaky["neg_pre"], leaky["neg_post"], leaky["neg_scale"]) == \
        _s(f32(0.09) * f32(0.1) / f32(0.04))
    assert rows[3]["value"] == _q8(0.0, 0.05, -3)
    assert (rows[5]["slice_is_i32"], rows[6]["slice_is_i32"]) == (0, 1)
    assert (rows[6]["slice_pre"], rows[6]["slice_post"], rows[6]["slice_scale"]) == \
        _s(f32(0.001) / f32(0.8))


def test_type_legality():
    m = H.Module("bad")
    a = m.placeholder("a", (4, 8), H.INT8Q, np.int8, 0.1, 0)
    b = m.placeholder("b", (4, 8), H.INT8Q, np.int8, 0.2, 3)
    fl = m.placeholder("fl", (4, 8), H.FLOAT, np.float32)
    sl = m.placeholder("sl", (7,), H.INT8Q, np.int8, 0.1, 0)
    for kind, ops, fa, why in (
            (H.CLIP, [fl, a], (0.0, 6.0), "i8"),                # float result
            (H.CLIP, [b, a], (0.0,), "min, max"),              # one bound only
            (H.LEAKY_RELU, [b, a], (), "alpha"),
            (H.CPU_MAX_SPLAT, [b, a], (0.0,), "share scale"),  # changes the type
            (H.BATCHED_ADD, [b, a, sl], (), "slice")):          # 7 is no slice of 4 x 8
        ok, msg = m.is_op_supported(kind, ops, (), fa)
        assert not ok and why in msg, (kind, msg)
    assert m.is_op_supported(H.CLIP, [b, a], (), (0.0, 6.0))[0]
    assert m.is_op_supported(H.CPU_MAX_SPLAT, [a, a], (), (0.0,))[0]


@pytest.mark.gpu
def test_kinds_through_the_device_manager():
    m, f, c = _module()
    m.compile(f)
    dm = H.DeviceManager().init()
    try:
        dm.add_network(m)
        rng = np.random.default_rng(32)
        for _ in range(3):
            x = rng.integers(-128, 128, (c["n"], c["k"])).astype(np.int8)
            y = rng.integers(-128, 128, (c["n"], c["k"])).astype(np.int8)
            want = _expected(c, x, y)
            outs = {k: np.zeros(v.shape, np.int8) for k, v in want.items()}
            dm.run("main", dict(outs, x=x, y=y))
            for k in want:
                np.testing.assert_array_equal(outs[k], want[k], err_msg=k)
            assert len(np.unique(want["clip_out"])) > 10
    finally:
        dm.stop()

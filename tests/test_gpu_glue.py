"""int8 glue operators on the GPU through the C ABI: bit-exact against the
oracle and the golden vectors of the reference's compiled libjit; fp32 softmax
within 1e-5 relative."""
import numpy as np
import pytest

from glow_amd import capi
from oracle import glow_oracle as go
from tests import golden_io as gio

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _init():
    capi.init(0)


def _p(ratio):
    return go.quantize_scale_offset_32to8(float(np.float32(ratio)), 0)[:3]


def test_glue_golden():
    ops, logits, softmax = gio.glue()
    for name, call, want in ops:
        np.testing.assert_array_equal(call(capi), want, err_msg=name)
    np.testing.assert_allclose(capi.softmax_f32(logits), softmax, rtol=1e-5, atol=1e-30)


@pytest.mark.parametrize("shape", [(1,), (15,), (16,), (4099,), (3, 7, 11, 13), (64, 56, 56, 64)])
def test_add_and_relu(shape):
    rng = np.random.default_rng(sum(shape))
    a = rng.integers(-128, 128, shape).astype(np.int8)
    b = rng.integers(-128, 128, shape).astype(np.int8)
    for ls, rs, ds, lo, ro, do in [(0.05, 0.07, 0.11, 3, -4, 5), (0.3, 0.002, 0.1, -128, 0, -128),
                                   (0.9, 1.1, 0.25, 100, -100, 0)]:
        lp, rp = _p(np.float32(ls) / np.float32(ds)), _p(np.float32(rs) / np.float32(ds))
        want = go.add_i8(a, b, do, lo, ro, lp, rp)
        np.testing.assert_array_equal(capi.add_i8(a, b, do, lo, ro, lp, rp), want)
        dp = _p(np.float32(ds) / np.float32(0.2))
        want_r = go.relu_i8(want, do, -7, dp)
        np.testing.assert_array_equal(capi.relu_i8(want, do, -7, dp), want_r)
        # the fused pass gives what the two separate instructions give
        np.testing.assert_array_equal(
            capi.add_relu_i8(a, b, do, lo, ro, lp, rp, -7, dp), want_r)


def test_elementwise_unaligned_views():
    """Tensors that start at an odd device address take the scalar path."""
    rng = np.random.default_rng(5)
    n = 1000
    a = rng.integers(-128, 128, n + 1).astype(np.int8)
    b = rng.integers(-128, 128, n + 1).astype(np.int8)
    da, db = capi.to_device(a), capi.to_device(b)
    out = capi.DeviceBuffer.empty((n + 1,), np.int8)
    out.fill(0)
    lp, rp = _p(0.5), _p(0.7)
    capi.launch_add_i8(out.ptr + 1, da.ptr + 1, db.ptr + 1, n, 1, 2, 3, lp, rp)
    got = out.numpy()
    assert got[0] == 0
    np.testing.assert_array_equal(got[1:], go.add_i8(a[1:], b[1:], 1, 2, 3, lp, rp))


POOLS = [
    ((2, 9, 11, 20), (3, 3), (2, 2), (1, 1, 1, 1)),
    ((2, 9, 11, 32), (3, 3), (2, 2), (1, 1, 1, 1)),      # 16-byte channel groups
    ((1, 8, 8, 16), (2, 2), (2, 2), (0, 0, 0, 0)),
    ((3, 7, 7, 64), (7, 7), (1, 1), (0, 0, 0, 0)),       # global pooling
    ((1, 6, 5, 3), (3, 2), (1, 2), (2, 1, 2, 1)),
    ((1, 5, 5, 4), (3, 3), (3, 3), (2, 2, 2, 2)),        # windows that start in the padding
    ((2, 112, 112, 64), (3, 3), (2, 2), (1, 1, 1, 1)),   # the ResNet stem pool
]


@pytest.mark.parametrize("shape,k,st,pd", POOLS)
def test_max_pool(shape, k, st, pd):
    rng = np.random.default_rng(shape[1] * 31 + shape[3])
    x = rng.integers(-128, 128, shape).astype(np.int8)
    np.testing.assert_array_equal(capi.max_pool_i8(x, k, st, pd, -5),
                                  go.max_pool_i8(x, k, st, pd, -5))


@pytest.mark.parametrize("shape,k,st,pd", POOLS)
@pytest.mark.parametrize("cip", [0, 1])
def test_avg_pool(shape, k, st, pd, cip):
    rng = np.random.default_rng(shape[1] * 37 + shape[3] + cip)
    x = rng.integers(-128, 128, shape).astype(np.int8)
    sc = np.float32(0.06) / np.float32(0.05)
    if cip:
        sc = sc / np.float32(k[0] * k[1])
    op = _p(sc)
    np.testing.assert_array_equal(capi.avg_pool_i8(x, k, st, pd, cip, 4, -9, op),
                                  go.avg_pool_i8(x, k, st, pd, cip, 4, -9, op))


@pytest.mark.parametrize("rows,cols", [(1, 1), (3, 7), (64, 1000), (5, 5000)])
def test_softmax(rows, cols):
    rng = np.random.default_rng(rows + cols)
    x = rng.normal(0, 5, (rows, cols)).astype(np.float32)
    got = capi.softmax_f32(x)
    np.testing.assert_allclose(got, go.softmax_f32(x), rtol=1e-5, atol=1e-30)
    np.testing.assert_allclose(got.sum(axis=1), 1.0, rtol=1e-5)


@pytest.mark.parametrize("rows,cols", [(1, 1), (3, 7), (64, 1000), (5, 5000)])
def test_dequantize_and_softmax_in_one_pass(rows, cols):
    rng = np.random.default_rng(rows * 31 + cols)
    q = rng.integers(-128, 128, (rows, cols)).astype(np.int8)
    scale, offset = np.float32(0.0731), -17
    want = go.softmax_f32(go.dequantize_i8(q, scale, offset))
    got = capi.dequantize_softmax(q, scale, offset)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-30)
    # the two-launch path gives the same numbers
    np.testing.assert_allclose(got, capi.softmax_f32(capi.dequantize_i8(q, scale, offset)),
                               rtol=1e-6, atol=1e-30)


def test_argument_errors():
    with pytest.raises(capi.MI355XError):
        capi.add_i8(np.zeros(4, np.int8), np.zeros(4, np.int8), 0, 0, 0, (0, 40, 1), (0, 0, 1))
    x = np.zeros((1, 4, 4, 4), np.int8)
    d = capi.to_device(x)
    with pytest.raises(capi.MI355XError):   # output larger than the input allows
        capi.check(capi.lib().mi355x_max_pool_i8(
            capi._vp(d), capi._vp(d), *[capi._sz(v) for v in (1, 4, 4, 4, 9, 9, 2, 2, 1, 1, 0, 0)],
            capi._i32(0), capi._vp(None)))


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("shape", [(2, 14, 14, 64, 256, 1), (1, 9, 9, 16, 40, 3), (3, 7, 7, 32, 64, 3)])
def test_conv_with_fused_residual_add(shape, relu):
    """Convolution + ElementAdd (+ Relu) in one kernel equals the separate
    instructions executed by the oracle."""
    from tests import cases
    N, Hh, W, IC, OC, k = shape
    pad = 1 if k == 3 else 0
    c = cases.cwq_conv_case(91, N, Hh, W, IC, OC, kernel=(k, k), pads=(pad,) * 4,
                            act=cases._w.ACT_NONE, in_offset=-5, out_offset=6)
    conv = go.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    rng = np.random.default_rng(92)
    res = rng.integers(-128, 128, conv.shape).astype(np.int8)
    cs, rs, ss, ds = np.float32(c["out_scale_f"]), np.float32(0.09), np.float32(0.13), np.float32(0.2)
    cp, rp, dp = _p(cs / ss), _p(rs / ss), _p(ss / ds)
    want = go.add_i8(conv, res, 11, c["out_offset"], -20, cp, rp)
    if relu:
        want = go.relu_i8(want, 11, -128, dp)
    add = capi.fused_add(11, -20, cp, rp, relu, -128, dp)
    got = capi.cwq_conv2d_add_i8(*cases.cwq_conv_args(c), res, add)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("params", [
    # (conv, residual, relu) rescale triples (pre, post, scale)
    ((0, 9, 300), (0, 8, 411), (0, 9, 333)),         # no pre-shift, small scales: folded constants
    ((0, 0, 1), (0, 0, 1), (0, 0, 1)),               # identities
    ((1, 9, 300), (0, 8, 411), (0, 9, 333)),         # a pre-shift in the add
    ((0, 9, 300), (0, 8, 411), (2, 9, 333)),         # a pre-shift in the relu
    ((0, 20, 1 << 24), (0, 8, 411), (0, 9, 333)),    # a scale beyond the 24-bit multiplier
])
def test_fused_residual_add_parameter_paths(params, relu):
    """Every arithmetic path of the fused add (+ Relu) stage gives the bits of
    the separate instructions."""
    from tests import cases
    cp, rp, dp = params
    c = cases.cwq_conv_case(93, 2, 10, 10, 32, 64, kernel=(1, 1), pads=(0,) * 4,
                            act=cases._w.ACT_NONE, in_offset=3, out_offset=-7)
    conv = go.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    res = np.random.default_rng(94).integers(-128, 128, conv.shape).astype(np.int8)
    for sum_off, res_off, dest_off in ((11, -20, -128), (-128, 127, 127), (0, 0, 0)):
        want = go.add_i8(conv, res, sum_off, c["out_offset"], res_off, cp, rp)
        if relu:
            want = go.relu_i8(want, sum_off, dest_off, dp)
        add = capi.fused_add(sum_off, res_off, cp, rp, relu, dest_off, dp)
        got = capi.cwq_conv2d_add_i8(*cases.cwq_conv_args(c), res, add)
        np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("shape,pads", [((2, 16, 16, 3), (3, 3)), ((1, 9, 7, 4), (0, 1)), ((3, 8, 8, 1), (1, 0))])
def test_space_to_depth(shape, pads):
    rng = np.random.default_rng(shape[1])
    x = rng.integers(-128, 128, shape).astype(np.int8)
    n, ih, iw, c = shape
    bh, bw, cout, fill = (ih + pads[0] + 4) // 2, (iw + pads[1] + 4) // 2, 16, -9
    xp = np.full((n, 2 * bh, 2 * bw, c), fill, np.int8)
    hh, ww = min(ih, 2 * bh - pads[0]), min(iw, 2 * bw - pads[1])
    xp[:, pads[0]:pads[0] + hh, pads[1]:pads[1] + ww] = x[:, :hh, :ww]
    want = np.full((n, bh, bw, cout), fill, np.int8)
    for dh in range(2):
        for dw in range(2):
            q = dh * 2 + dw
            want[..., q * c:(q + 1) * c] = xp[:, dh::2, dw::2]
    np.testing.assert_array_equal(capi.space_to_depth2_i8(x, pads[0], pads[1], bh, bw, cout, fill), want)


@pytest.mark.parametrize("shape,pads", [((2, 16, 16, 3), (3, 3)), ((1, 9, 7, 4), (0, 1)), ((2, 224, 224, 3), (3, 3))])
def test_quantize_and_space_to_depth_in_one_pass(shape, pads):
    """The fused pass writes what Quantize (against the oracle) followed by the
    layout change writes."""
    rng = np.random.default_rng(shape[1] + 1)
    x = rng.normal(0.45, 0.25, shape).astype(np.float32)
    x.reshape(-1)[:8] = [0.0, -0.0, 1e9, -1e9, 0.0125, -0.0125, 0.0375, 3.175]   # ties and clips
    scale, offset = 0.025, -128
    q = go.quantize_i8(x, scale, offset)
    n, ih, iw, c = shape
    bh, bw, cout, fill = (ih + pads[0] + 4) // 2, (iw + pads[1] + 4) // 2, 16, offset
    want = capi.space_to_depth2_i8(q, pads[0], pads[1], bh, bw, cout, fill)
    got = capi.quantize_space_to_depth2_i8(x, pads[0], pads[1], bh, bw, cout, fill, scale, offset)
    np.testing.assert_array_equal(got, want)
    assert len(np.unique(got)) > 20


def test_add_with_scales_beyond_24_bits():
    """Parameters outside the 24-bit fast path take the 32-bit multiplier."""
    rng = np.random.default_rng(31)
    a = rng.integers(-128, 128, 5000).astype(np.int8)
    b = rng.integers(-128, 128, 5000).astype(np.int8)
    for lp, rp, lo, ro in [((0, 20, (1 << 23) + 5), (1, 3, 7), 3, -4),
                           ((0, 0, 1), (0, 25, -(1 << 24) - 1), 0, (1 << 22) + 9),
                           ((3, 9, (1 << 23) - 1), (0, 31, 1 << 30), -(1 << 22) + 1, 12)]:
        want = go.add_i8(a, b, 5, lo, ro, lp, rp)
        np.testing.assert_array_equal(capi.add_i8(a, b, 5, lo, ro, lp, rp), want)
        dp = (0, 22, (1 << 23) + 77)
        np.testing.assert_array_equal(capi.add_relu_i8(a, b, 5, lo, ro, lp, rp, -3, dp),
                                      go.relu_i8(want, 5, -3, dp))


def test_unlowered_element_ops_golden_and_oracle():
    """Clip, LeakyRelu, Max(x, Splat) and BatchedAdd (what the CPU backend keeps
    un-lowered besides Relu; libjit.cpp:1865-1892, 997-1015, libjit_cpu.cpp:45-46):
    the golden vectors of the compiled reference, then larger and unaligned
    tensors against the oracle."""
    for name, fn, args, want in gio.element_ops():
        np.testing.assert_array_equal(getattr(capi, fn)(*args), want, err_msg=name)
    rng = np.random.default_rng(77)
    p = lambda r: go.quantize_scale_offset_32to8(float(np.float32(r)), 0)[:3]
    for n in (1, 15, 16, 17, 4099, 1 << 20):
        a = rng.integers(-128, 128, n).astype(np.int8)
        np.testing.assert_array_equal(capi.clip_elem_i8(a, -30, 90, -5, 7, p(0.37)),
                                      go.clip_elem_i8(a, -30, 90, -5, 7, p(0.37)))
        np.testing.assert_array_equal(capi.leaky_relu_i8(a, 4, -9, p(1.9), p(0.19)),
                                      go.leaky_relu_i8(a, 4, -9, p(1.9), p(0.19)))
        np.testing.assert_array_equal(capi.max_splat_i8(a, -3), np.maximum(a, np.int8(-3)))
    for ns, ss in ((1, 1), (7, 5), (64, 1000), (300, 1024), (4096, 512)):
        b = rng.integers(-128, 128, (ns, ss)).astype(np.int8)
        for sl in (rng.integers(-128, 128, ss).astype(np.int8),
                   rng.integers(-100000, 100000, ss).astype(np.int32)):
            sp = p(0.9) if sl.dtype == np.int8 else p(0.0007)
            np.testing.assert_array_equal(capi.batched_add_i8(b, sl, -2, 3, -1, p(1.3), sp),
                                          go.batched_add_i8(b, sl, -2, 3, -1, p(1.3), sp))

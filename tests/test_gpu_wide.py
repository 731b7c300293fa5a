"""The 16/32-bit Quantize / Dequantize / RescaleQuantized, Transpose of up to
six dimensions and the 3-D channelwise quantized convolution against the
golden vectors (outputs of the reference's compiled libjit) and the oracle.

Run on the GPU box:  python -u -m pytest tests -m gpu -x -v --timeout 120
"""
import numpy as np
import pytest

from glow_amd import capi
from oracle import glow_oracle as go
from tests import cases
from tests import golden_io as gio

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _device():
    capi.init(0)
    yield
    capi.sync()


def say(*a):
    print(*a, flush=True)


@pytest.mark.parametrize("bits", [16, 32])
def test_wide_elementwise_golden_and_oracle(bits):
    d = gio.wide()
    q = d[f"q{bits}"]
    for i in range(3):
        s, o = d[f"quant{bits}_{i}_params"]
        np.testing.assert_array_equal(capi.quantize_wide(d["x"], float(s), int(o), bits),
                                      d[f"quant{bits}_{i}_out"])
        np.testing.assert_array_equal(capi.dequantize_wide(q, float(s), int(o)),
                                      d[f"dequant{bits}_{i}_out"])
    for i in range(4):
        oo, io, pre, post, sc = (int(v) for v in d[f"rescale{bits}_{i}_params"])
        np.testing.assert_array_equal(capi.rescale_wide(q, oo, io, pre, post, sc),
                                      d[f"rescale{bits}_{i}_out"])
    # a million elements (more than one pass of the grid), exact ties, huge values
    rng = np.random.default_rng(bits)
    dt = np.int16 if bits == 16 else np.int32
    lim = 2 ** (bits - 1)
    x = np.concatenate([rng.normal(0, 5000, 1_100_000), (np.arange(-300, 300) + 0.5),
                        [3e9, -3e9, 1e30, -1e30, 0.0, -0.0]]).astype(np.float32)
    big = rng.integers(-lim, lim, 1_100_003).astype(dt)
    for scale, off in [(0.37, -11), (2.5, 40000)]:
        np.testing.assert_array_equal(capi.quantize_wide(x, scale, off, bits),
                                      go.quantize_wide(x, scale, off, bits))
        np.testing.assert_array_equal(capi.dequantize_wide(big, scale, off),
                                      go.dequantize_wide(big, scale, off))
    for r, io, oo in [(0.0007, 5, -9), (0.9, -128, 127), (3.3, 1000, -1000)]:
        pre, post, sc, _ = go.quantize_scale_offset_32to8(r, 0)
        np.testing.assert_array_equal(capi.rescale_wide(big, oo, io, pre, post, sc),
                                      go.rescale_wide(big, oo, io, pre, post, sc))
    # empty tensors are no-ops; shifts outside [0, 31] are refused
    assert capi.rescale_wide(big[:0], 0, 0, 1, 1, 1).size == 0
    with pytest.raises(capi.MI355XError):
        capi.rescale_wide(big[:8], 0, 0, 32, 1, 1)


def test_transpose_nd_golden_and_oracle():
    d = gio.wide()
    i = 0
    while f"transpose{i}_in" in d:
        x, sh = d[f"transpose{i}_in"], [int(v) for v in d[f"transpose{i}_shuffle"]]
        got = capi.transpose_nd(x, sh)
        np.testing.assert_array_equal(got, d[f"transpose{i}_out"].reshape(got.shape))
        i += 1
    assert i == 6
    rng = np.random.default_rng(11)
    for nd in range(1, 7):
        for dt in (np.int8, np.int16, np.float32, np.int64):
            shape = tuple(int(v) for v in rng.integers(1, 9, nd))
            sh = [int(v) for v in rng.permutation(nd)]
            x = rng.integers(-100, 100, shape).astype(dt)
            say("transpose", shape, sh, np.dtype(dt).name)
            got = capi.transpose_nd(x, sh)
            np.testing.assert_array_equal(got, go.transpose(x, sh))
            np.testing.assert_array_equal(got, x.transpose(sh))
    # NCHW <-> NHWC of an image batch (more elements than one pass of the grid)
    x = rng.integers(-128, 128, (8, 64, 56, 56)).astype(np.int8)
    np.testing.assert_array_equal(capi.transpose_nd(x, [0, 2, 3, 1]), x.transpose(0, 2, 3, 1))
    for bad in ([0, 0, 1, 2], [0, 1, 2, 4]):
        with pytest.raises(capi.MI355XError):
            capi.transpose_nd(x, bad)


def test_cwq_conv3d_golden():
    n = 0
    for tag, args, want in gio.conv3d_cases():
        say("conv3d golden", tag)
        np.testing.assert_array_equal(capi.cwq_conv3d_i8(*args), want)
        n += 1
    assert n == 4


CONV3D = [
    dict(N=2, T=6, H=14, W=14, IC=16, OC=32),
    dict(N=1, T=4, H=9, W=7, IC=6, OC=9, kernel=(2, 3, 2), stride=(1, 2, 2),
         pads=(0, 1, 2, 0, 1, 1), group=3, symmetric=False, in_offset=-20, act=go.ACT_NONE),
    dict(N=3, T=3, H=5, W=5, IC=5, OC=7, kernel=(3, 1, 1), pads=(1, 1, 0, 0, 0, 0),
         act=go.ACT_CLIP, out_offset=-30, bias_i8=True),
    dict(N=1, T=2, H=6, W=6, IC=8, OC=8, kernel=(2, 2, 2), stride=(2, 2, 2),
         pads=(0, 0, 0, 0, 0, 0), act=go.ACT_LEAKY_RELU, out_offset=12, in_offset=7),
    dict(N=1, T=5, H=16, W=16, IC=32, OC=64, kernel=(3, 3, 3), symmetric=False, in_offset=-128),
]


@pytest.mark.parametrize("kw", CONV3D)
def test_cwq_conv3d_vs_oracle(kw):
    c = cases.cwq_conv3d_case(31, **kw)
    g = c["geom"]
    say("conv3d", kw, "output", g.OT, g.OH, g.OW)
    want = go.cwq_conv3d_i8(*cases.cwq_conv_args(c))
    got = capi.cwq_conv3d_i8(*cases.cwq_conv_args(c))
    np.testing.assert_array_equal(got, want)
    assert want.std() > 1


def test_cwq_conv3d_with_one_frame_is_the_2d_convolution():
    """T = KT = 1: the same numbers as the 2-D kernels on the same operands."""
    c3 = cases.cwq_conv3d_case(33, N=2, T=1, H=12, W=10, IC=16, OC=24, kernel=(1, 3, 3),
                               pads=(0, 0, 1, 1, 1, 1), in_offset=-3)
    got = capi.cwq_conv3d_i8(*cases.cwq_conv_args(c3))
    g2 = go.conv_geom(2, 12, 10, 16, 24, (3, 3), (1, 1), (1, 1, 1, 1))
    a = list(cases.cwq_conv_args(c3))
    a[0], a[1], a[3] = c3["x"][:, 0], c3["filt"][:, 0], g2
    np.testing.assert_array_equal(got[:, 0], capi.cwq_conv2d_i8(*a))


def test_cwq_conv3d_rejects_malformed_geometry():
    c = cases.cwq_conv3d_case(35, N=1, T=3, H=4, W=4, IC=4, OC=4)
    g = c["geom"]
    bad = go.Conv3dGeom(*[getattr(g, n) for n, _ in g._fields_])
    bad.OT = 40          # output frames that would start past the input
    a = list(cases.cwq_conv_args(c))
    a[3] = bad
    with pytest.raises(capi.MI355XError):
        capi.cwq_conv3d_i8(*a)
    a[3] = g
    a[14] = 3            # fused tanh is not defined for quantized convolutions
    with pytest.raises(capi.MI355XError):
        capi.cwq_conv3d_i8(*a)

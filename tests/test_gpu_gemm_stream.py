"""The streaming kernel for short K and many rows (tile 8): FullyConnected and
pointwise convolutions over 64, 128 or 256 inputs, against the oracle and the
tiled kernels, with column slices, row tails, strides, the fused residual add
and Relu, and the requantisation hints.

Run on the GPU box:  python -u -m pytest tests -m gpu -x -v --timeout 120
"""
import numpy as np
import pytest

from glow_amd import capi
from oracle import glow_oracle as go
from tests import cases, tiles

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _device():
    capi.init(0)
    yield
    capi.sync()


def say(*a):
    print(*a, flush=True)


class forced_tile:
    def __init__(self, tile):
        self.tile = tile

    def __enter__(self):
        capi.check(capi.lib().mi355x_gemm_tile_override(self.tile))

    def __exit__(self, *exc):
        capi.check(capi.lib().mi355x_gemm_tile_override(-1))
        return False


FC_SHAPES = [
    # M, K, N: row tails, one and several column slices, more tiles than waves
    (1, 64, 32), (33, 64, 64), (1000, 64, 256), (257, 128, 512), (4096, 256, 64),
    (70, 256, 384), (20000, 64, 96), (129, 128, 1024),
]


@pytest.mark.parametrize("shape", FC_SHAPES)
def test_stream_fc_vs_oracle(shape):
    M, K, N = shape
    c = cases.rwq_fc_case(800 + M + K, M, K, N)
    c["w_offsets"][:] = 0          # what the kernel takes: symmetric weights
    want = go.rwq_fc_i8(*cases.rwq_fc_args(c))
    say("stream fc", shape)
    with forced_tile(8):
        got = capi.rwq_fc_i8(*cases.rwq_fc_args(c))
    np.testing.assert_array_equal(got, want)
    assert want.std() > 5
    # with the requantisation hint the backend derives for these constants
    hint = capi.gemm_requant_hint_host(K, c["in_offset"], c["out_offset"], c["w_offsets"],
                                       c["bias"], c["bias_offset"], c["bias_pre"], c["bias_post"],
                                       c["bias_scale"], c["out_pre"], c["out_post"], c["out_scale"])
    with forced_tile(8), capi.requant_hint(hint):
        np.testing.assert_array_equal(capi.rwq_fc_i8(*cases.rwq_fc_args(c)), want)
    # no input offset (no use of the weight row sums), int8 bias
    c2 = cases.rwq_fc_case(801 + M, M, K, N, in_offset=0, bias_i8=True, bias_scale=0.01,
                           bias_offset=3)
    c2["w_offsets"][:] = 0
    with forced_tile(8):
        np.testing.assert_array_equal(capi.rwq_fc_i8(*cases.rwq_fc_args(c2)),
                                      go.rwq_fc_i8(*cases.rwq_fc_args(c2)))


def test_stream_refuses_what_it_cannot_run():
    """Weight offsets (row sums of A would be needed), other K, sums not
    precomputed: asked for by number (tile 8) the kernel refuses the launch,
    and the shape rule runs the tiled kernels."""
    for K, kw, sums in ((64, dict(symmetric=False), True), (192, dict(), True),
                        (64, dict(in_offset=5), False),   # an input offset needs the row sums
                        (320, dict(), True)):
        c = cases.rwq_fc_case(850 + K, 100, K, 64, **kw)
        if kw.get("symmetric", True):
            c["w_offsets"][:] = 0
        want = go.rwq_fc_i8(*cases.rwq_fc_args(c))
        assert tiles.refused(8, lambda: capi.rwq_fc_i8(*cases.rwq_fc_args(c),
                                                       precomputed_sums=sums))
        got = capi.rwq_fc_i8(*cases.rwq_fc_args(c), precomputed_sums=sums)
        np.testing.assert_array_equal(got, want)


CONV_CASES = [
    dict(N=2, H=56, W=56, IC=64, OC=256),                              # ResNet stage 1
    dict(N=1, H=28, W=28, IC=128, OC=512, in_offset=-128),
    dict(N=3, H=9, W=7, IC=256, OC=96, act=go.ACT_CLIP, in_offset=3),
    dict(N=2, H=56, W=56, IC=256, OC=512, stride=(2, 2)),              # strided shortcut
    dict(N=1, H=15, W=13, IC=64, OC=64, stride=(2, 3), act=go.ACT_LEAKY_RELU, out_offset=10),
    dict(N=1, H=5, W=5, IC=128, OC=32, bias_i8=True, act=go.ACT_NONE, in_offset=-5),
]


@pytest.mark.parametrize("kw", CONV_CASES)
def test_stream_pointwise_conv_vs_oracle(kw):
    kw = dict(kw)
    kw.setdefault("in_offset", -128)
    c = cases.cwq_conv_case(61, kernel=(1, 1), pads=(0, 0, 0, 0), **kw)
    g = c["geom"]
    say("stream conv", kw, "output", g.OH, "x", g.OW)
    want = go.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    with forced_tile(8):
        got = capi.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    np.testing.assert_array_equal(got, want)
    with forced_tile(1):
        np.testing.assert_array_equal(capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)), want)
    hint = capi.gemm_requant_hint_host(g.IC, c["in_offset"], c["out_offset"], c["f_offsets"],
                                       c["bias"], 0, c["bias_pre"], c["bias_post"], c["bias_scale"],
                                       c["out_pre"], c["out_post"], c["out_scale"],
                                       bias_offsets=c["b_offsets"])
    with forced_tile(8), capi.requant_hint(hint):
        np.testing.assert_array_equal(capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)), want)
    assert want.std() > 1


WINDOW_CASES = [
    # the stem of an image network after space-to-depth: 4x4 over 16 channels
    dict(N=2, H=115, W=115, IC=16, OC=64, kernel=(4, 4)),
    dict(N=1, H=9, W=11, IC=16, OC=32, kernel=(2, 2), act=go.ACT_CLIP),             # K 64
    dict(N=3, H=8, W=8, IC=32, OC=96, kernel=(2, 2), stride=(2, 2), in_offset=4),   # K 128
    dict(N=1, H=10, W=7, IC=64, OC=64, kernel=(2, 2), stride=(1, 2)),               # K 256
    dict(N=2, H=6, W=12, IC=16, OC=256, kernel=(2, 8), act=go.ACT_LEAKY_RELU),      # rows of 128 bytes
    dict(N=1, H=7, W=7, IC=32, OC=64, kernel=(4, 1), bias_i8=True),                 # rows of 32 bytes
]


@pytest.mark.parametrize("kw", WINDOW_CASES)
def test_stream_window_conv_vs_oracle(kw):
    """Windows without padding whose rows are whole 32-byte chunks run on the
    streaming kernel as rows of several segments."""
    kw = dict(kw)
    kw.setdefault("in_offset", -128)
    c = cases.cwq_conv_case(63, pads=(0, 0, 0, 0), **kw)
    g = c["geom"]
    say("stream window conv", kw, "output", g.OH, "x", g.OW)
    want = go.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    with forced_tile(8):
        got = capi.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    np.testing.assert_array_equal(got, want)
    with forced_tile(2):
        np.testing.assert_array_equal(capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)), want)
    assert want.std() > 1


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("IC,OC", [(64, 256), (128, 512), (256, 1024)])
def test_stream_conv_with_fused_residual_add(IC, OC, relu):
    c = cases.cwq_conv_case(71 + IC, 2, 14, 14, IC, OC, kernel=(1, 1), pads=(0, 0, 0, 0),
                            act=go.ACT_NONE, in_offset=-128, out_offset=6)
    conv = go.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    rng = np.random.default_rng(72)
    res = rng.integers(-128, 128, conv.shape).astype(np.int8)
    p = lambda r: go.quantize_scale_offset_32to8(float(np.float32(r)), 0)[:3]
    cs, rs, ss, ds = np.float32(c["out_scale_f"]), np.float32(0.09), np.float32(0.13), np.float32(0.2)
    cp, rp, dp = p(cs / ss), p(rs / ss), p(ss / ds)
    want = go.add_i8(conv, res, 11, c["out_offset"], -20, cp, rp)
    if relu:
        want = go.relu_i8(want, 11, -128, dp)
    add = capi.fused_add(11, -20, cp, rp, relu, -128, dp)
    with forced_tile(8):
        got = capi.cwq_conv2d_add_i8(*cases.cwq_conv_args(c), res, add)
    np.testing.assert_array_equal(got, want)


def test_stream_conv_full_batch():
    """The first ResNet stage's pointwise layer with the residual at batch 64:
    two images on the oracle, the rest through batch independence."""
    c = cases.cwq_conv_case(91, 64, 56, 56, 64, 256, kernel=(1, 1), pads=(0, 0, 0, 0),
                            in_offset=-128)
    c["x"][2::2] = c["x"][0]
    c["x"][3::2] = c["x"][1]
    with forced_tile(8):
        got = capi.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    c2 = dict(c, x=c["x"][:2], geom=go.conv_geom(2, 56, 56, 64, 256, (1, 1), (1, 1), (0, 0, 0, 0)))
    want = go.cwq_conv2d_i8(*cases.cwq_conv_args(c2))
    np.testing.assert_array_equal(got[:2], want)
    for i in range(2, 64):
        np.testing.assert_array_equal(got[i], want[i % 2])


@pytest.mark.parametrize("IC,OC,slow", [(64, 64, False), (128, 96, False), (64, 32, True),
                                        (128, 256, True), (64, 128, False)])
def test_stream_add_narrow_slices_and_general_scales(IC, OC, slow):
    """Slices of 32, 64 and 96 columns (two and four passes of the copy-out,
    lanes past the tile's rows) with the residual, and add parameters outside
    the short form (a pre-shift, a scale beyond 23 bits)."""
    c = cases.cwq_conv_case(75 + IC + OC, 3, 11, 13, IC, OC, kernel=(1, 1), pads=(0, 0, 0, 0),
                            act=go.ACT_NONE, in_offset=-128, out_offset=-3)
    conv = go.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    rng = np.random.default_rng(76)
    res = rng.integers(-128, 128, conv.shape).astype(np.int8)
    p = lambda r: go.quantize_scale_offset_32to8(float(np.float32(r)), 0)[:3]
    cp, rp, dp = p(0.8), p(0.61), p(0.7)
    if slow:
        cp = (1, cp[1], cp[2] * 2)                 # the same ratio through a pre-shift
        rp = (0, 24, int(round(0.61 * (1 << 24))))
    want = go.relu_i8(go.add_i8(conv, res, 7, c["out_offset"], -9, cp, rp), 7, -128, dp)
    add = capi.fused_add(7, -9, cp, rp, True, -128, dp)
    say("stream add", IC, OC, "slow" if slow else "short form", cp, rp)
    with forced_tile(8):
        got = capi.cwq_conv2d_add_i8(*cases.cwq_conv_args(c), res, add)
    np.testing.assert_array_equal(got, want)
    with forced_tile(2):
        np.testing.assert_array_equal(capi.cwq_conv2d_add_i8(*cases.cwq_conv_args(c), res, add), want)
    assert len(np.unique(want)) > 20


def test_stream_add_several_tiles_per_wave():
    """More 32-row tiles than the launch has waves, with the residual: a wave's
    next rows and residual bytes are asked for while it works on a tile. Two
    images and two residual images on the oracle, the rest through batch
    independence."""
    n = 44                                           # 137984 rows = 4312 tiles
    c = cases.cwq_conv_case(93, n, 56, 56, 64, 64, kernel=(1, 1), pads=(0, 0, 0, 0),
                            act=go.ACT_NONE, in_offset=-128)
    c["x"][2::2] = c["x"][0]
    c["x"][3::2] = c["x"][1]
    rng = np.random.default_rng(94)
    res = np.empty((n, 56, 56, 64), np.int8)
    res[0::2] = rng.integers(-128, 128, (56, 56, 64)).astype(np.int8)
    res[1::2] = rng.integers(-128, 128, (56, 56, 64)).astype(np.int8)
    p = lambda r: go.quantize_scale_offset_32to8(float(np.float32(r)), 0)[:3]
    cp, rp, dp = p(0.9), p(0.5), p(0.66)
    add = capi.fused_add(2, 5, cp, rp, True, -128, dp)
    with forced_tile(8):
        got = capi.cwq_conv2d_add_i8(*cases.cwq_conv_args(c), res, add)
    c2 = dict(c, x=c["x"][:2], geom=go.conv_geom(2, 56, 56, 64, 64, (1, 1), (1, 1), (0, 0, 0, 0)))
    conv = go.cwq_conv2d_i8(*cases.cwq_conv_args(c2))
    want = go.relu_i8(go.add_i8(conv, res[:2], 2, c["out_offset"], 5, cp, rp), 2, -128, dp)
    for i in range(n):
        np.testing.assert_array_equal(got[i], want[i % 2])
    assert len(np.unique(want)) > 20

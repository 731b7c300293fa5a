"""The 3x3, stride-1, 64-input-channel convolution with filter and input rows
resident in LDS (tile 7) against the oracle and against the implicit-GEMM
kernels, over image shapes, paddings, output-channel counts, offsets,
activations, the fused residual add and the requantisation hints.

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


HALO_CASES = [
    dict(N=2, H=56, W=56, OC=64),                               # the ResNet layer shape
    dict(N=3, H=13, W=9, OC=64),                                # tiles that end inside an image
    dict(N=1, H=5, W=130, OC=128, pads=(1, 1, 1, 1)),           # one row per tile, five waves
    dict(N=2, H=20, W=20, OC=192, pads=(0, 0, 0, 0)),           # no padding: output 18x18
    dict(N=2, H=11, W=12, OC=64, pads=(2, 0, 1, 3)),            # uneven padding
    dict(N=1, H=3, W=3, OC=64, pads=(1, 1, 1, 1)),              # a single small tile
    dict(N=1, H=4, W=256, OC=64),                               # the widest row the kernel takes
    dict(N=1, H=3, W=257, OC=64, served=False),                 # wider: refused, the implicit GEMM serves it
    dict(N=2, H=300, W=1, OC=64),                               # tall and thin: 256 rows per tile
    dict(N=300, H=9, W=9, OC=64),                               # more tiles than resident workgroups
    dict(N=5, H=7, W=7, OC=128, in_offset=0, act=go.ACT_NONE),  # no input offset, no row sums used
    dict(N=1, H=28, W=28, OC=64, in_offset=7, out_offset=5, act=go.ACT_CLIP),
    dict(N=1, H=16, W=16, OC=64, act=go.ACT_LEAKY_RELU, out_offset=10, bias_i8=True),
]


@pytest.mark.parametrize("kw", HALO_CASES)
def test_halo_conv_vs_oracle(kw):
    kw = dict(kw)
    kw.setdefault("in_offset", -128)
    served = kw.pop("served", True)
    c = cases.cwq_conv_case(17, IC=64, **kw)
    g = c["geom"]
    say("halo conv", kw, "output", g.OH, "x", g.OW)
    want = go.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    if not served:
        # the kernel refuses the shape; the shape rule runs the implicit GEMM
        assert tiles.refused(7, lambda: capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)))
        np.testing.assert_array_equal(capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)), want)
        return
    with forced_tile(7):
        got = capi.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    np.testing.assert_array_equal(got, want)
    # by the shape rule (no override) the same kernel serves the launch
    np.testing.assert_array_equal(capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)), want)
    # the implicit-GEMM path gives the same bytes
    with forced_tile(2):
        np.testing.assert_array_equal(capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)), want)
    # with the requantisation hint
    hint = capi.gemm_requant_hint_host(576, c["in_offset"], c["out_offset"], c["f_offsets"],
                                       c["bias"], 0, c["bias_pre"], c["bias_post"], c["bias_scale"],
                                       c["out_pre"], c["out_post"], c["out_scale"],
                                       bias_offsets=c["b_offsets"])
    with forced_tile(7), capi.requant_hint(hint):
        np.testing.assert_array_equal(capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)), want)
    assert want.std() > 1
    # uniform-parameter convolution through its own entry point
    args = (c["x"], c["filt"], c["bias"], c["geom"], c["out_offset"], c["in_offset"],
            int(c["f_offsets"][1]), int(c["b_offsets"][1]),
            (c["bias_pre"][1], c["bias_post"][1], c["bias_scale"][1]),
            (c["out_pre"][1], c["out_post"][1], c["out_scale"][1]), c["act"], c["act_args"])
    with forced_tile(7):
        np.testing.assert_array_equal(capi.conv2d_i8(*args, precomputed_sums=True),
                                      go.conv2d_i8(*args))


def test_halo_conv_refuses_what_it_cannot_run():
    """Filter offsets (the kernel would need input row sums), missing filter row
    sums, other channel counts, strides or dilations: asked for by number (tile
    7) the kernel refuses the launch, and the shape rule runs another one."""
    for kw, sums in ((dict(IC=64, symmetric=False), True), (dict(IC=64), False),
                     (dict(IC=32), True), (dict(IC=64, stride=(2, 2)), True),
                     (dict(IC=64, dilation=(2, 2), pads=(2, 2, 2, 2)), True),
                     (dict(IC=128, group=2), True)):
        c = cases.cwq_conv_case(19, 2, 12, 12, OC=64, in_offset=-9, **kw)
        want = go.cwq_conv2d_i8(*cases.cwq_conv_args(c))
        assert tiles.refused(7, lambda: capi.cwq_conv2d_i8(*cases.cwq_conv_args(c),
                                                           precomputed_sums=sums))
        got = capi.cwq_conv2d_i8(*cases.cwq_conv_args(c), precomputed_sums=sums)
        np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("relu", [False, True])
def test_halo_conv_with_fused_residual_add(relu):
    c = cases.cwq_conv_case(91, 2, 15, 14, 64, 128, act=go.ACT_NONE, in_offset=-5, out_offset=6)
    conv = go.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    rng = np.random.default_rng(92)
    res = rng.integers(-128, 128, conv.shape).astype(np.int8)
    p = lambda r: go.quantize_scale_offset_32to8(float(np.float32(r)), 0)[:3]
    cs, rs, ss, ds = np.float32(c["out_scale_f"]), np.float32(0.09), np.float32(0.13), np.float32(0.2)
    cp, rp, dp = p(cs / ss), p(rs / ss), p(ss / ds)
    want = go.add_i8(conv, res, 11, c["out_offset"], -20, cp, rp)
    if relu:
        want = go.relu_i8(want, 11, -128, dp)
    add = capi.fused_add(11, -20, cp, rp, relu, -128, dp)
    with forced_tile(7):
        got = capi.cwq_conv2d_add_i8(*cases.cwq_conv_args(c), res, add)
    np.testing.assert_array_equal(got, want)


def test_halo_conv_full_batch():
    """The ResNet layer at its batch of 32: two images on the oracle, the rest
    through batch independence."""
    c = cases.cwq_conv_case(41, 32, 56, 56, 64, 64, in_offset=-128)
    c["x"][2::2] = c["x"][0]
    c["x"][3::2] = c["x"][1]
    with forced_tile(7):
        got = capi.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    c2 = dict(c, x=c["x"][:2], geom=go.conv_geom(2, 56, 56, 64, 64, (3, 3), (1, 1), (1, 1, 1, 1)))
    want = go.cwq_conv2d_i8(*cases.cwq_conv_args(c2))
    np.testing.assert_array_equal(got[:2], want)
    for i in range(2, 32):
        np.testing.assert_array_equal(got[i], want[i % 2])

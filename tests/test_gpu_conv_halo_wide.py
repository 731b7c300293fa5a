"""The 3x3, stride-1 convolution over 128, 256 or 512 input channels with the
input patch resident in LDS and the filter slice streamed through it tap by
tap (tile 7 for these channel counts) against the oracle and against the
implicit-GEMM kernels: row tiles, several small images per tile, tiles that
end early, paddings, offsets, activations, the fused residual add and the
requantisation hints.

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


WIDE_CASES = [
    dict(IC=256, N=3, H=14, W=14, OC=128),                       # one image per tile, seven waves
    dict(IC=128, N=2, H=28, W=28, OC=128),                       # four tiles of seven rows per image
    dict(IC=512, N=5, H=7, W=7, OC=64),                          # two images per tile, the last tile one
    dict(IC=128, N=7, H=7, W=7, OC=192),                         # five images per tile, the last tile two
    dict(IC=256, N=2, H=13, W=9, OC=64, pads=(2, 0, 1, 3)),      # uneven padding
    dict(IC=128, N=1, H=20, W=20, OC=64, pads=(0, 0, 0, 0)),     # no padding: output 18 x 18, two tiles
    dict(IC=512, N=1, H=14, W=14, OC=64),                        # LDS allows nine rows: two tiles of seven
    dict(IC=128, N=1, H=4, W=256, OC=64),                        # the widest row the kernel takes
    dict(IC=256, N=1, H=3, W=40, OC=64),                         # 120 pixels: four waves, the fewest
    dict(IC=128, N=1, H=5, W=5, OC=64, served=False),            # too few pixels: refused, the implicit GEMM serves it
    dict(IC=256, N=2, H=14, W=14, OC=64, in_offset=0, act=go.ACT_NONE),
    dict(IC=128, N=1, H=28, W=28, OC=64, in_offset=7, out_offset=5, act=go.ACT_CLIP),
    dict(IC=256, N=1, H=14, W=14, OC=64, act=go.ACT_LEAKY_RELU, out_offset=10, bias_i8=True),
]


@pytest.mark.parametrize("kw", WIDE_CASES)
def test_wide_halo_conv_vs_oracle(kw):
    kw = dict(kw)
    kw.setdefault("in_offset", -128)
    served = kw.pop("served", True)
    c = cases.cwq_conv_case(23, **kw)
    g = c["geom"]
    say("wide halo conv", kw, "output", g.OH, "x", g.OW)
    want = go.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    if not served:
        assert tiles.refused(7, lambda: capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)))
        np.testing.assert_array_equal(capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)), want)
        return
    with forced_tile(7):
        got = capi.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    np.testing.assert_array_equal(got, want)
    # whatever the shape rule picks gives the same bytes, and so does the implicit GEMM
    np.testing.assert_array_equal(capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)), want)
    with forced_tile(2):
        np.testing.assert_array_equal(capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)), want)
    hint = capi.gemm_requant_hint_host(9 * g.IC, c["in_offset"], c["out_offset"], c["f_offsets"],
                                       c["bias"], 0, c["bias_pre"], c["bias_post"], c["bias_scale"],
                                       c["out_pre"], c["out_post"], c["out_scale"],
                                       bias_offsets=c["b_offsets"])
    with forced_tile(7), capi.requant_hint(hint):
        np.testing.assert_array_equal(capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)), want)
    assert want.std() > 1


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("IC", [128, 512])
def test_wide_halo_conv_with_fused_residual_add(IC, relu):
    c = cases.cwq_conv_case(93, 3, 7, 14, IC, 128, act=go.ACT_NONE, in_offset=-5, out_offset=6)
    conv = go.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    rng = np.random.default_rng(94)
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


@pytest.mark.parametrize("IC,H", [(128, 28), (256, 14), (512, 7)])
def test_wide_halo_conv_full_batch(IC, H):
    """The ResNet layers at their batch of 64: two images on the oracle, the
    rest through batch independence."""
    c = cases.cwq_conv_case(43, 64, H, H, IC, IC, in_offset=-128)
    c["x"][2::2] = c["x"][0]
    c["x"][3::2] = c["x"][1]
    with forced_tile(7):
        got = capi.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    c2 = dict(c, x=c["x"][:2], geom=go.conv_geom(2, H, H, IC, IC, (3, 3), (1, 1), (1, 1, 1, 1)))
    want = go.cwq_conv2d_i8(*cases.cwq_conv_args(c2))
    np.testing.assert_array_equal(got[:2], want)
    for i in range(2, 64):
        np.testing.assert_array_equal(got[i], want[i % 2])


@pytest.mark.parametrize("seed", range(16))
def test_wide_halo_conv_random_geometry(seed):
    """Seeded shapes around the tiling's corners: rows per tile, images per
    tile, the last tile of an image or of the batch, every padding."""
    rng = np.random.default_rng(500 + seed)
    IC = int(rng.choice([128, 256, 512]))
    H, W = int(rng.integers(3, 31)), int(rng.integers(3, 41))
    if IC == 512:
        H, W = min(H, 16), min(W, 16)
    N = int(rng.integers(1, 7))
    pads = tuple(int(v) for v in rng.integers(0, 3, 4))
    kw = dict(IC=IC, N=N, H=H, W=W, OC=64 * int(rng.integers(1, 3)), pads=pads,
              in_offset=int(rng.integers(-128, 128)), out_offset=int(rng.integers(-128, 128)),
              act=[go.ACT_NONE, go.ACT_RELU, go.ACT_CLIP][seed % 3])
    c = cases.cwq_conv_case(600 + seed, **kw)
    g = c["geom"]
    if g.OH <= 0 or g.OW <= 0:
        pytest.skip("empty output")
    say("wide halo conv", kw, "output", g.OH, "x", g.OW)
    want = go.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    got = tiles.forced_or_refused(7, lambda: capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)))
    if got is None:
        # the kernel refuses the shape (too few pixels for four waves, a patch
        # that does not fit LDS): what the shape rule picks must serve it
        say("  refused by the kernel; served by the shape rule's choice")
        got = capi.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    np.testing.assert_array_equal(got, want)

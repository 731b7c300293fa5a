"""Every workgroup tile of the int8 contraction on K loops longer than its ring
of load stages, compared with the CPU oracle.

The tile is forced with mi355x_gemm_tile_override, so the 256x256, 256x128 and
128x256 instantiations (which the shape rules pick only for large problems)
run their steady-state ring: wrap-around of the slots, the wait counts of the
split tile loads and the slotted fragment reads, for the dense-row operand
(RowwiseQuantizedFullyConnected, libjit_matmul.cpp:284-316) and the
convolution operand (ChannelwiseQuantizedConvolution, libjit_conv.cpp:151-239).
The two large FullyConnected shapes the benchmark times are checked at full
size: the oracle on a row sample, every other row through the repeated-rows
property (equal input rows give equal output rows).

Run on the GPU box:  python -u -m pytest tests -m gpu -x -v --timeout 120
"""
import numpy as np
import pytest

from glow_amd import capi
from oracle import glow_oracle as go
from tests import cases

pytestmark = pytest.mark.gpu

TILES = {0: "256x256", 1: "128x128", 2: "128x64", 3: "64x64", 4: "256x128", 5: "128x256"}


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


_FC_WANT = {}


def _fc_case(K, variant):
    """M and N are not multiples of 256 (or of 128 for the asymmetric case), so
    edge tiles with clamped rows are part of every run."""
    key = (K, variant)
    if key not in _FC_WANT:
        M, N = (512, 512) if variant == "symmetric" else (520, 392)
        c = cases.rwq_fc_case(500 + K + len(variant), M, K, N,
                              symmetric=(variant == "symmetric"),
                              in_offset=(0 if variant == "no_offsets" else None),
                              bias_i8=(variant == "asymmetric_bias8"),
                              bias_scale=(0.01 if variant == "asymmetric_bias8" else 5e-5),
                              bias_offset=(3 if variant == "asymmetric_bias8" else 0))
        if variant == "no_offsets":
            c["w_offsets"][:] = 0
        _FC_WANT[key] = (c, go.rwq_fc_i8(*cases.rwq_fc_args(c)))
    return _FC_WANT[key]


@pytest.mark.parametrize("K", [256, 1024, 4096])
@pytest.mark.parametrize("tile", list(TILES))
def test_rwq_fc_long_k_on_every_tile(tile, K):
    for variant in ("symmetric", "asymmetric", "asymmetric_bias8", "no_offsets"):
        c, want = _fc_case(K, variant)
        say("rwq_fc tile", TILES[tile], "K", K, variant, c["x"].shape, c["w"].shape)
        with forced_tile(tile):
            got = capi.rwq_fc_i8(*cases.rwq_fc_args(c))
            got_own_sums = capi.rwq_fc_i8(*cases.rwq_fc_args(c), precomputed_sums=False)
        np.testing.assert_array_equal(got, want)
        np.testing.assert_array_equal(got_own_sums, want)
        assert want.std() > 5


_CONV_WANT = {}


def _conv_case(IC, variant):
    key = (IC, variant)
    if key not in _CONV_WANT:
        if variant == "symmetric":      # ResNet stage-3/4 style 3x3, post-ReLU input
            c = cases.cwq_conv_case(700 + IC, 2, 14, 14, IC, 256, in_offset=-128)
        elif variant == "asymmetric":   # filter offsets: the kernel sums the input rows
            c = cases.cwq_conv_case(710 + IC, 1, 15, 13, IC, 136, in_offset=-7,
                                    symmetric=False, act=go.ACT_NONE)
        else:                           # strided, padded unevenly, two groups
            c = cases.cwq_conv_case(720 + IC, 2, 17, 15, IC, 192, stride=(2, 2),
                                    pads=(0, 1, 2, 1), group=2, in_offset=5)
        _CONV_WANT[key] = (c, go.cwq_conv2d_i8(*cases.cwq_conv_args(c)))
    return _CONV_WANT[key]


@pytest.mark.parametrize("IC", [256, 512])
@pytest.mark.parametrize("tile", list(TILES))
def test_cwq_conv_long_k_on_every_tile(tile, IC):
    for variant in ("symmetric", "asymmetric", "strided_groups"):
        c, want = _conv_case(IC, variant)
        g = c["geom"]
        say("cwq_conv tile", TILES[tile], "IC", IC, variant,
            "K", g.KH * g.KW * IC // g.group)
        with forced_tile(tile):
            got = capi.cwq_conv2d_i8(*cases.cwq_conv_args(c))
            got_own_sums = capi.cwq_conv2d_i8(*cases.cwq_conv_args(c), precomputed_sums=False)
        np.testing.assert_array_equal(got, want)
        np.testing.assert_array_equal(got_own_sums, want)
        assert want.std() > 1


def _check_large(M, K, N, seed, symmetric, distinct, sample, tile=None):
    """Rows [distinct, M) repeat rows [0, distinct); the oracle runs on
    `sample` of the distinct rows."""
    c = cases.rwq_fc_case(seed, M, K, N, symmetric=symmetric)
    for lo in range(distinct, M, distinct):
        c["x"][lo:lo + distinct] = c["x"][:min(distinct, M - lo)]
    if tile is None:
        got = capi.rwq_fc_i8(*cases.rwq_fc_args(c))
    else:
        with forced_tile(tile):
            got = capi.rwq_fc_i8(*cases.rwq_fc_args(c))
    for lo in range(distinct, M, distinct):
        np.testing.assert_array_equal(got[lo:lo + distinct], got[:min(distinct, M - lo)])
    cs = dict(c, x=c["x"][sample])
    np.testing.assert_array_equal(got[sample], go.rwq_fc_i8(*cases.rwq_fc_args(cs)))
    assert got.std() > 5


def test_rwq_fc_m8192_k4096_n4096():
    """The benchmark's large FullyConnected (256x256 tiles by the shape rule)."""
    say("rwq_fc M8192 K4096 N4096")
    rows = np.r_[0:24, 250:262, 500:512]
    _check_large(8192, 4096, 4096, 81, True, 512, rows)


def test_rwq_fc_m8192_k4096_n4096_asymmetric_weights():
    say("rwq_fc M8192 K4096 N4096, weight offsets")
    rows = np.r_[0:8, 255:259, 508:512]
    _check_large(8192, 4096, 4096, 82, False, 512, rows)


@pytest.mark.parametrize("tile", [None, 0, 4, 5])
def test_rwq_fc_m16384_k1024_n1024(tile):
    """The benchmark's M = 16384 variant of the single-FC shape (256x128 tiles by
    the shape rule; the other large tiles forced)."""
    say("rwq_fc M16384 K1024 N1024 tile", TILES.get(tile, "by shape"))
    rows = np.r_[0:40, 1000:1040, 2040:2048]
    _check_large(16384, 1024, 1024, 83 + (tile or 0), tile in (None, 4), 2048, rows, tile)


def test_rwq_fc_m4096_k1024_n1024_all_tiles_agree():
    """One mid-size product on all six tiles: identical bytes."""
    c = cases.rwq_fc_case(77, 4096, 1024, 1024, symmetric=False)
    c["x"][2048:] = c["x"][:2048]
    ref = None
    for tile in TILES:
        say("rwq_fc M4096 K1024 N1024 tile", TILES[tile])
        with forced_tile(tile):
            got = capi.rwq_fc_i8(*cases.rwq_fc_args(c))
        if ref is None:
            ref = got
            rows = np.r_[0:40, 1000:1040, 2040:2048]
            cs = dict(c, x=c["x"][rows])
            np.testing.assert_array_equal(got[rows], go.rwq_fc_i8(*cases.rwq_fc_args(cs)))
            np.testing.assert_array_equal(got[2048:], got[:2048])
        else:
            np.testing.assert_array_equal(got, ref)

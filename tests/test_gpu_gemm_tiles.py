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
from tests import cases, tiles

pytestmark = pytest.mark.gpu

TILES = {0: "256x256", 1: "128x128", 2: "128x64", 3: "64x64", 4: "256x128", 5: "128x256",
         6: "32x32 split-K", 9: "128x128, 8 waves", 10: "256x128, 8 waves",
         11: "256x256, 8 waves"}


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
        # the split-K kernel (tile 6) refuses weight offsets and missing row sums
        got = tiles.forced_or_refused(tile, lambda: capi.rwq_fc_i8(*cases.rwq_fc_args(c)))
        got_own_sums = tiles.forced_or_refused(
            tile, lambda: capi.rwq_fc_i8(*cases.rwq_fc_args(c), precomputed_sums=False))
        assert tile == 6 or (got is not None and got_own_sums is not None)
        if tile == 6:
            assert (got is not None) == (variant in ("symmetric", "no_offsets"))
            # without precomputed row sums it runs only where none are needed
            assert (got_own_sums is not None) == (variant == "no_offsets")
        if got is not None:
            np.testing.assert_array_equal(got, want)
        if got_own_sums is not None:
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
        if tile == 6:
            # the split-K kernel serves FullyConnected forms only
            assert tiles.refused(6, lambda: capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)))
            continue
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
    """The benchmark's large FullyConnected (256x256 tiles with eight waves by the
    shape rule)."""
    say("rwq_fc M8192 K4096 N4096")
    rows = np.r_[0:24, 250:262, 500:512]
    _check_large(8192, 4096, 4096, 81, True, 512, rows)


def test_rwq_fc_m8192_k4096_n4096_asymmetric_weights():
    say("rwq_fc M8192 K4096 N4096, weight offsets")
    rows = np.r_[0:8, 255:259, 508:512]
    _check_large(8192, 4096, 4096, 82, False, 512, rows)


@pytest.mark.parametrize("tile", [None, 0, 4, 5, 10])
def test_rwq_fc_m16384_k1024_n1024(tile):
    """The benchmark's M = 16384 variant of the single-FC shape (256x256 tiles
    with eight waves by the shape rule; the other large tiles forced)."""
    say("rwq_fc M16384 K1024 N1024 tile", TILES.get(tile, "by shape"))
    rows = np.r_[0:40, 1000:1040, 2040:2048]
    _check_large(16384, 1024, 1024, 83 + (tile or 0), tile in (None, 4, 10), 2048, rows, tile)


def test_rwq_fc_m4096_k1024_n1024_all_tiles_agree():
    """One mid-size product on every tile: identical bytes."""
    c = cases.rwq_fc_case(77, 4096, 1024, 1024, symmetric=False)
    c["x"][2048:] = c["x"][:2048]
    ref = None
    for tile in TILES:
        say("rwq_fc M4096 K1024 N1024 tile", TILES[tile])
        if tile == 6:   # weight offsets: refused by the split-K kernel
            assert tiles.refused(6, lambda: capi.rwq_fc_i8(*cases.rwq_fc_args(c)))
            continue
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


# ---- requantisation hints ---------------------------------------------------------

def _hint_for_fc(c, K):
    return capi.gemm_requant_hint_host(K, c["in_offset"], c["out_offset"], c["w_offsets"], c["bias"],
                                       c["bias_offset"], c["bias_pre"], c["bias_post"],
                                       c["bias_scale"], c["out_pre"], c["out_post"], c["out_scale"])


@pytest.mark.parametrize("tile", list(TILES))
def test_requant_hint_gives_the_same_bytes_on_every_tile(tile):
    """With the hint the host derives from a launch's parameters the epilogue
    runs its 24-bit multiply-add forms; the results are those of libjit_scale."""
    seen = set()
    for K, wr, sym in ((64, (0.0002, 0.002), True), (64, (0.02, 0.1), True),
                       (256, (0.0002, 0.002), False), (576, (0.0002, 0.001), True)):
        c = cases.rwq_fc_case(300 + K, 300, K, 200, w_scale_range=wr, symmetric=sym)
        hint = _hint_for_fc(c, K)
        seen.add(hint)
        want = go.rwq_fc_i8(*cases.rwq_fc_args(c))
        say("hint", hint, "tile", TILES[tile], "K", K, "pre", int(c["out_pre"].min()),
            int(c["out_pre"].max()))
        with capi.requant_hint(hint):
            got = tiles.forced_or_refused(tile, lambda: capi.rwq_fc_i8(*cases.rwq_fc_args(c)))
            got2 = tiles.forced_or_refused(
                tile, lambda: capi.rwq_fc_i8(*cases.rwq_fc_args(c), precomputed_sums=False))
        assert tile == 6 or (got is not None and got2 is not None)
        if tile == 6:   # split-K: symmetric weights with precomputed sums only
            assert (got is not None) == sym and (got2 is None or c["in_offset"] == 0)
        if got is not None:
            np.testing.assert_array_equal(got, want)
        if got2 is not None:
            np.testing.assert_array_equal(got2, want)
    assert {1, 3} <= seen          # both fast forms were exercised


def test_requant_hint_holds_for_the_largest_accumulators():
    """The hint is derived for worst-case operand bytes: operands that give the
    largest possible sums of either sign still requantise exactly."""
    K, M, N = 64, 96, 160
    c = cases.rwq_fc_case(7, M, K, N, w_scale_range=(0.02, 0.1), symmetric=False, in_offset=-128)
    c["x"][:] = 127
    c["x"][M // 2:] = -128
    c["w"][:] = -128
    c["w"][::2] = 127
    c["w_offsets"][:] = 20
    c["w_offsets"][::3] = -20
    c["bias"][:] = 1000
    c["bias"][::2] = -1000
    hint = _hint_for_fc(c, K)
    assert hint & 1, "this launch fits 24 bits by construction"
    want = go.rwq_fc_i8(*cases.rwq_fc_args(c))
    with capi.requant_hint(hint):
        np.testing.assert_array_equal(capi.rwq_fc_i8(*cases.rwq_fc_args(c)), want)
        np.testing.assert_array_equal(
            capi.rwq_fc_i8(*cases.rwq_fc_args(c), precomputed_sums=False), want)
    assert len(np.unique(want)) > 2


def test_requant_hint_with_convolutions_and_the_fused_add():
    for kw in (dict(N=2, H=20, W=20, IC=64, OC=96), dict(N=1, H=14, W=14, IC=128, OC=64, kernel=(1, 1),
                                                          pads=(0, 0, 0, 0)),
               dict(N=2, H=9, W=9, IC=32, OC=48, symmetric=False, act=go.ACT_CLIP)):
        c = cases.cwq_conv_case(55, in_offset=-128, **kw)
        g = c["geom"]
        K = g.KH * g.KW * g.IC // g.group
        hint = capi.gemm_requant_hint_host(K, c["in_offset"], c["out_offset"], c["f_offsets"],
                                           c["bias"], 0, c["bias_pre"], c["bias_post"],
                                           c["bias_scale"], c["out_pre"], c["out_post"],
                                           c["out_scale"], bias_offsets=c["b_offsets"])
        say("conv hint", hint, kw)
        assert hint & 1
        want = go.cwq_conv2d_i8(*cases.cwq_conv_args(c))
        with capi.requant_hint(hint):
            np.testing.assert_array_equal(capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)), want)


# ---- 32x32 tiles with the K loop split over the waves ------------------------------

SKINNY_SHAPES = [(128, 1024, 1024), (1, 128, 1), (7, 160, 33), (33, 96, 70), (64, 4096, 256),
                 (130, 32, 90), (16, 2048 + 32, 1000), (256, 512, 128)]


@pytest.mark.parametrize("shape", SKINNY_SHAPES)
def test_split_k_small_tiles_vs_oracle(shape):
    """Symmetric weights with precomputed row sums (what the kernel serves), both
    by the shape rule and forced; int32 and int8 bias, zero and non-zero input
    offset, with and without the requantisation hint, and the fused Relu."""
    M, K, N = shape
    for seed, b8, in_off in ((1, False, None), (2, True, None), (3, False, 0)):
        c = cases.rwq_fc_case(seed + M + K, M, K, N, symmetric=True, bias_i8=b8,
                              bias_scale=(0.01 if b8 else 5e-5), bias_offset=(3 if b8 else 0),
                              in_offset=in_off)
        args = cases.rwq_fc_args(c)
        want = go.rwq_fc_i8(*args)
        hint = _hint_for_fc(c, K)
        say("split-K", shape, "bias8" if b8 else "bias32", "in_offset", c["in_offset"], "hint", hint)
        for forced in (6, None):
            for h in sorted({0, hint}):
                with capi.requant_hint(h):
                    if forced is None:
                        got = capi.rwq_fc_i8(*args)
                    else:
                        with forced_tile(forced):
                            got = capi.rwq_fc_i8(*args)
                np.testing.assert_array_equal(got, want)
        fc = want
        for relu_offset, reluP in ((-128, (0, 8, 300)), (5, (1, 9, 1 << 24))):
            want_relu = go.relu_i8(fc, c["out_offset"], relu_offset, reluP)
            with forced_tile(6):
                got = capi.rwq_fc_relu_i8(*args[:10], c["out_offset"], c["in_offset"],
                                          c["bias_offset"], relu_offset, reluP)
            np.testing.assert_array_equal(got, want_relu)


def test_split_k_tile_refuses_what_it_cannot_run():
    """Weight offsets, missing row sums or a K that is no multiple of 32: asked
    for by number (tile 6) the kernel refuses the launch; the shape rule runs
    the tiled kernels, same results."""
    for kw, sums in ((dict(symmetric=False), True), (dict(symmetric=True), False)):
        c = cases.rwq_fc_case(9, 40, 256, 72, **kw)
        want = go.rwq_fc_i8(*cases.rwq_fc_args(c))
        assert tiles.refused(6, lambda: capi.rwq_fc_i8(*cases.rwq_fc_args(c),
                                                       precomputed_sums=sums))
        got = capi.rwq_fc_i8(*cases.rwq_fc_args(c), precomputed_sums=sums)
        np.testing.assert_array_equal(got, want)
    c = cases.rwq_fc_case(10, 40, 272, 72)           # K % 32 == 16
    assert tiles.refused(6, lambda: capi.rwq_fc_i8(*cases.rwq_fc_args(c)))
    np.testing.assert_array_equal(capi.rwq_fc_i8(*cases.rwq_fc_args(c)),
                                  go.rwq_fc_i8(*cases.rwq_fc_args(c)))

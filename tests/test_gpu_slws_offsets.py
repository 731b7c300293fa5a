"""mi355x_frwq_slws_offsets: the SparseLengths lookup with the bags given as
positions (the exclusive prefix sums a device manager makes of the lengths it
uploads) against the oracle and against the lengths entry point, bit for bit.

Run on the GPU box:  python -u -m pytest tests -m gpu -x -v --timeout 120
"""
import numpy as np
import pytest

from glow_amd import capi
from oracle import glow_oracle as go
from tests import cases

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _device():
    capi.init(0)
    yield
    capi.sync()


def say(*a):
    print(*a, flush=True)


SHAPES = [
    # rows, cols, bags, mean length
    (50, 8, 20, 3), (1000, 128, 64, 40), (300, 37, 10, 12), (500, 64, 33, 20),
    (200, 256, 9, 7), (4000, 128, 4096, 40), (999, 32, 100, 90), (64, 16, 5, 200),
    (5000, 64, 20000, 6),   # more bags than the lengths path sums in one launch
]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("idt", [np.int64, np.int32])
def test_offsets_u8_f32_bit_exact(shape, idt):
    rows, cols, bags, mean = shape
    say("slws offsets u8/f32", shape, idt.__name__)
    rng = np.random.default_rng(rows + cols)
    table = cases.random_fused_table(rng, rows, cols)
    lengths, idx, w = cases.slws_batch(bags, rows, bags, mean, 1.05, idt)
    lengths[bags // 2] = 0
    total = int(lengths.sum())
    idx, w = idx[:total], w[:total]
    want = go.frwq_slws_f32(table, w, idx, lengths)
    got = capi.frwq_slws(table, capi.FUSED_U8_F32, w, idx, lengths, bag_offsets=True)
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(got, capi.frwq_slws(table, capi.FUSED_U8_F32, w, idx, lengths))
    # unweighted
    np.testing.assert_array_equal(
        capi.frwq_slws(table, capi.FUSED_U8_F32, None, idx, lengths, bag_offsets=True),
        go.frwq_slws_f32(table, np.ones(total, np.float32), idx, lengths))


@pytest.mark.parametrize("kind", [capi.FUSED_U8_F16, capi.FUSED_U4_F16, capi.FUSED_U4_F32])
@pytest.mark.parametrize("cols", [64, 130, 6, 256])
def test_offsets_other_kinds_equal_the_lengths_path(kind, cols):
    say("slws offsets kind", kind, "cols", cols)
    rng = np.random.default_rng(kind * 100 + cols)
    rows, bags = 400, 37
    table = cases.random_fused_table(rng, rows, cols, kind)
    lengths, idx, w = cases.slws_batch(kind + cols, rows, bags, 9, 1.05, np.int64)
    f16 = kind in (capi.FUSED_U8_F16, capi.FUSED_U4_F16)
    wt = w.astype(np.float16) if f16 else w
    for acc16 in ((False, True) if f16 else (False,)):
        a = capi.frwq_slws(table, kind, wt, idx, lengths, f16, acc16)
        b = capi.frwq_slws(table, kind, wt, idx, lengths, f16, acc16, bag_offsets=True)
        np.testing.assert_array_equal(a.view(np.uint8), b.view(np.uint8))


def test_offsets_on_a_second_stream():
    rows, cols, bags = 3000, 128, 500
    rng = np.random.default_rng(77)
    table = cases.random_fused_table(rng, rows, cols)
    lengths, idx, w = cases.slws_batch(78, rows, bags, 30, 1.05, np.int64)
    want = go.frwq_slws_f32(table, w, idx, lengths)
    st = capi.Stream()
    np.testing.assert_array_equal(
        capi.frwq_slws(table, 0, w, idx, lengths, bag_offsets=True, stream=st), want)


@pytest.mark.fused_math
@pytest.mark.parametrize("cols", [32, 64, 128, 256])
def test_offsets_fused_arithmetic_equals_the_lengths_path(cols):
    """The regrouped sum (the library's default outside these tests): both entry
    points run the same kernel, so the bits agree; against the oracle to 1e-5 of
    the magnitude a bag adds up."""
    rows, bags = 3000, 700
    rng = np.random.default_rng(cols)
    table = cases.random_fused_table(rng, rows, cols)
    lengths, idx, w = cases.slws_batch(cols, rows, bags, 30, 1.05, np.int64)
    a = capi.frwq_slws(table, 0, w, idx, lengths)
    b = capi.frwq_slws(table, 0, w, idx, lengths, bag_offsets=True)
    np.testing.assert_array_equal(a, b)
    want = go.frwq_slws_f32(table, w, idx, lengths)
    assert cases.slws_error_ratio(b, want, table, w, idx, lengths) <= 1e-5


def test_offsets_that_make_no_sense_never_leave_the_index_list():
    rows, cols = 50, 16
    rng = np.random.default_rng(12)
    table = cases.random_fused_table(rng, rows, cols)
    idx = rng.integers(0, rows, 9).astype(np.int64)
    w = rng.random(9).astype(np.float32)
    lengths = np.array([3, 2, 4], np.int32)
    # negative lengths are empty bags, in both entry points
    neg = np.array([3, -5, 4, 2], np.int32)
    offs = capi.slws_bag_offsets_host(neg)
    np.testing.assert_array_equal(offs, [0, 3, 3, 7, 9])
    np.testing.assert_array_equal(
        capi.frwq_slws(table, 0, w, idx, neg, bag_offsets=True),
        capi.frwq_slws(table, 0, w, idx, neg))
    # an end past the list and a decreasing pair: bag 1 is empty (its end is
    # clamped up to its start), bag 2 runs from position 2 to the end of the list
    bad = np.array([0, 3, 2, 40], np.int32)
    got = capi.frwq_slws(table, 0, w, idx, lengths, bag_offsets=bad)
    want = go.frwq_slws_f32(table, np.r_[w[:3], w[2:]].astype(np.float32),
                            np.r_[idx[:3], idx[2:]], np.array([3, 0, 7], np.int32))
    np.testing.assert_array_equal(got, want)
    # a negative start counts as position 0
    bad = np.array([-4, 3, 5, 9], np.int32)
    np.testing.assert_array_equal(capi.frwq_slws(table, 0, w, idx, lengths, bag_offsets=bad),
                                  go.frwq_slws_f32(table, w, idx, lengths))


def test_offsets_full_size_config():
    """The benchmark configuration at full size through the offsets entry point."""
    rows, cols, bags = 4_000_000, 128, 4096
    say("slws offsets full size")
    rng = np.random.default_rng(2026)
    table = cases.random_fused_table(rng, rows, cols)
    lengths, idx, w = cases.slws_batch(2027, rows, bags, 40, 1.05, np.int64)
    got = capi.frwq_slws(table, capi.FUSED_U8_F32, w, idx, lengths, bag_offsets=True)
    np.testing.assert_array_equal(got, go.frwq_slws_f32(table, w, idx, lengths))

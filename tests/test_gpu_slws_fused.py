"""The SparseLengths kernels with their default (fused multiply-add)
arithmetic, against the CPU oracle's sequential loop. The default form
  v = fma(s_j, q_jk, o_j);  acc_k = fma(w_j, v, acc_k)
is the loop's own expression w_j (s_j q_jk + o_j) per element without the two
intermediate roundings (what the reference's libjit becomes on a host with
fused multiply-add), with the lookups of a bag summed in two interleaved
partial sums. The bar is the stated one for floating point, element by
element: |got - want| <= 1e-5 |want| for every output with
|want| >= max(1, B / 128), where B = sum_j |w_j| (|s_j| q_max + |o_j|) is the
magnitude of what the bag adds up. A result that has cancelled further than
that is held to 1e-5 max(1, B / 128) instead: a sum of L terms taken in another
order moves by about sqrt(L) units in the last place of its partial sums, which
no relative bar on a cancelled result can absorb (the reference's own builds
differ among themselves in the same way:
tests/test_oracle_vs_ref.py::test_slws_reference_builds_differ_by_rounding).
fp16 outputs get one extra fp16 unit in the last place for the final rounding.
Everything else about the operator (skipped lookups, empty bags, index types,
every output row written) is checked as in the bit-exact tests.
"""
import numpy as np
import pytest

from glow_amd import capi
from oracle import glow_oracle as go
from tests import cases

pytestmark = [pytest.mark.gpu, pytest.mark.fused_math]

RTOL = 1e-5
FLOOR = 1.0   # element-wise bar applies to outputs at least this large


@pytest.fixture(scope="module", autouse=True)
def _device():
    capi.init(0)
    yield
    capi.sync()


def say(*a):
    print(*a, flush=True)


def row_scale_offset(table, kind):
    """fp32 (scale, offset) of every fused row."""
    if kind in (capi.FUSED_U8_F32, capi.FUSED_U4_F32):
        so = np.ascontiguousarray(table[:, -8:]).view(np.float32)
    else:
        so = np.ascontiguousarray(table[:, -4:]).view(np.float16).astype(np.float32)
    return so[:, 0], so[:, 1]


def bag_magnitude(table, kind, w, idx, lengths, scales=None, offsets=None):
    """B per bag, float64."""
    s, o = (scales, offsets) if scales is not None else row_scale_offset(table, kind)
    qmax = 255.0 if kind in (capi.FUSED_U8_F32, capi.FUSED_U8_F16) else 15.0
    total = int(lengths.sum())
    idx = np.asarray(idx[:total])
    ok = (idx >= 0) & (idx < table.shape[0])
    r = np.where(ok, idx, 0)
    ww = np.ones(total) if w is None else np.abs(np.asarray(w[:total], np.float64))
    m = np.where(ok, ww * (np.abs(s[r].astype(np.float64)) * qmax +
                            np.abs(o[r].astype(np.float64))), 0.0)
    ends = np.cumsum(lengths)
    c = np.r_[0.0, np.cumsum(m)]
    return c[ends] - c[ends - lengths]


def check(got, want, mag, out16=False, what=""):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    tol = RTOL * mag[:, None]
    if out16:
        tol = tol + np.abs(want) * 2.0 ** -10
    err = np.abs(got - want)
    worst = float(np.max(err / np.maximum(mag[:, None], 1e-30))) if err.size else 0.0
    floor = np.maximum(FLOOR, mag[:, None] / 128.0) * np.ones_like(want)
    big = np.abs(want) >= floor
    etol = RTOL * np.maximum(np.abs(want), floor) + (np.abs(want) * 2.0 ** -10 if out16 else 0.0)
    worst_rel = float(np.max(err[big] / np.abs(want[big]))) if big.any() else 0.0
    say(f"  {what} max error / B = {worst:.2e}; max |got - want| / |want| over the "
        f"{big.mean():.0%} of outputs with |want| >= max({FLOOR:g}, B/128): {worst_rel:.2e}")
    assert np.all(err <= tol), (what, worst)
    assert np.all(err <= etol), (what, worst_rel)
    # empty bags are exact zeros
    empty = mag == 0
    assert np.all(got[empty] == 0)


# data bytes 32/64/128/256 take the fused kernels; the others in the list stay
# on the separately rounded ones and must agree exactly
SHAPES = [
    # rows, cols, bags, mean length
    (1000, 128, 64, 40), (500, 64, 33, 20), (200, 256, 9, 7), (4000, 128, 4096, 40),
    (999, 32, 100, 90), (700, 128, 50, 150), (300, 37, 10, 12), (64, 16, 5, 200),
]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("idt", [np.int64, np.int32])
def test_slws_u8_f32(shape, idt):
    rows, cols, bags, mean = shape
    say("fused slws u8/f32", shape, idt.__name__)
    rng = np.random.default_rng(rows + cols)
    table = cases.random_fused_table(rng, rows, cols)
    lengths, idx, w = cases.slws_batch(bags, rows, bags, mean, 1.05, idt)
    lengths[bags // 2] = 0
    total = int(lengths.sum())
    idx, w = idx[:total], w[:total]
    mag = bag_magnitude(table, capi.FUSED_U8_F32, w, idx, lengths)
    check(capi.frwq_slws(table, capi.FUSED_U8_F32, w, idx, lengths),
          go.frwq_slws_f32(table, w, idx, lengths), mag, what="weighted")
    mag1 = bag_magnitude(table, capi.FUSED_U8_F32, None, idx, lengths)
    check(capi.frwq_slws(table, capi.FUSED_U8_F32, None, idx, lengths),
          go.frwq_slws_f32(table, np.ones(total, np.float32), idx, lengths), mag1,
          what="sum")
    if cols not in (32, 64, 128, 256):
        np.testing.assert_array_equal(
            capi.frwq_slws(table, capi.FUSED_U8_F32, w, idx, lengths),
            go.frwq_slws_f32(table, w, idx, lengths))


@pytest.mark.parametrize("kind", [capi.FUSED_U8_F16, capi.FUSED_U4_F16, capi.FUSED_U4_F32])
@pytest.mark.parametrize("cols", [64, 128, 256, 512, 16])
def test_slws_other_kinds(kind, cols):
    say("fused slws kind", kind, "cols", cols)
    rng = np.random.default_rng(kind * 100 + cols)
    rows, bags = 700, 150
    table = cases.random_fused_table(rng, rows, cols, kind)
    lengths, idx, w = cases.slws_batch(cols, rows, bags, 20, 1.1, np.int64)
    lengths[7] = 0
    total = int(lengths.sum())
    idx, w = idx[:total], w[:total]
    f16 = kind in (capi.FUSED_U8_F16, capi.FUSED_U4_F16)
    combos = [(w, False, False), (None, False, False)]
    if f16:
        combos += [(w.astype(np.float16), True, False), (None, True, False),
                   (w.astype(np.float16), True, True)]
    for weights, out16, acc16 in combos:
        want = go.frwq_slws_generic(table, kind, weights, idx, lengths, out16, acc16)
        got = capi.frwq_slws(table, kind, weights, idx, lengths, out16, acc16)
        if acc16:
            # fp16 accumulation keeps the separately rounded kernels
            np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))
            continue
        mag = bag_magnitude(table, kind, weights, idx, lengths)
        check(got.astype(np.float32), want.astype(np.float32), mag, out16,
              what=f"w={'none' if weights is None else weights.dtype} out16={out16}")


@pytest.mark.parametrize("kind,cols,pitch", [
    (capi.FUSED_U4_F16, 64, 64),     # 36-byte rows, several bags per wavefront
    (capi.FUSED_U8_F32, 32, 64),     # 40-byte rows
    (capi.FUSED_U8_F16, 64, 128),    # 68-byte rows
    (capi.FUSED_U8_F32, 128, 192),   # 136-byte rows, one wavefront per bag
    (capi.FUSED_U8_F32, 256, 272),
    (capi.FUSED_U4_F32, 60, 40),     # 38-byte rows on the general kernel
    (capi.FUSED_U8_F16, 30, 35),     # odd pitch: byte loads
])
def test_rows_further_apart_than_their_size(kind, cols, pitch):
    """A table laid out with padded rows (in_line_size above the fused row's
    size) gives what the packed table gives: the same bits from the same
    kernel, and the oracle's values to the stated tolerance."""
    say("padded table kind", kind, "cols", cols, "pitch", pitch)
    rng = np.random.default_rng(kind * 1000 + cols)
    rows, bags = 900, 130
    table = cases.random_fused_table(rng, rows, cols, kind)
    assert table.shape[1] <= pitch
    lengths, idx, w = cases.slws_batch(cols + 1, rows, bags, 18, 1.1, np.int64)
    lengths[3] = 0
    total = int(lengths.sum())
    idx, w = idx[:total], w[:total]
    f16 = kind in (capi.FUSED_U8_F16, capi.FUSED_U4_F16)
    for weights in (w, None):
        want = go.frwq_slws_generic(table, kind, weights, idx, lengths, f16, False)
        packed = capi.frwq_slws(table, kind, weights, idx, lengths, f16)
        padded = capi.frwq_slws(table, kind, weights, idx, lengths, f16, row_pitch=pitch)
        assert np.array_equal(padded.view(np.uint8), packed.view(np.uint8))
        check(padded.astype(np.float32), want.astype(np.float32),
              bag_magnitude(table, kind, weights, idx, lengths), f16,
              what=f"w={'none' if weights is None else 'f32'}")


def test_invalid_lookups_are_skipped_and_rows_rezeroed():
    rows, cols = 50, 128
    rng = np.random.default_rng(12)
    table = cases.random_fused_table(rng, rows, cols)
    lengths = np.array([3, 2, 4], np.int32)
    idx = np.array([1, 99, 3, -1, 4, 5, 6, 7, 8], np.int64)  # 99 and -1 are out of range
    w = rng.random(9).astype(np.float32)
    keep = np.array([1, 0, 1, 0, 1, 1, 1, 1, 1], bool)
    want = go.frwq_slws_f32(table, np.where(keep, w, 0).astype(np.float32),
                            np.where(keep, idx, 0), lengths)
    mag = bag_magnitude(table, 0, w, idx, lengths)
    check(capi.frwq_slws(table, 0, w, idx, lengths), want, mag, what="skips")
    # lengths that run past the index list: the missing lookups are skipped
    got = capi.frwq_slws(table, 0, w[:7], idx[:7].clip(0, 49), lengths)
    want = go.frwq_slws_f32(table, np.r_[w[:7], [0, 0]].astype(np.float32),
                            np.r_[idx[:7].clip(0, 49), [0, 0]], lengths)
    check(got, want, bag_magnitude(table, 0, np.r_[w[:7], [0, 0]],
                                   np.r_[idx[:7].clip(0, 49), [0, 0]], lengths),
          what="short list")
    # a second call with emptied bags rewrites their rows with zeros
    l2 = np.array([3, 0, 4], np.int32)
    i2 = np.r_[idx[:3].clip(0, 49), idx[5:9]]
    w2 = np.r_[w[:3], w[5:9]].astype(np.float32)
    got = capi.frwq_slws(table, 0, w2, i2, l2)
    assert np.all(got[1] == 0)


def test_embedding_bag_offsets_mode():
    rows, cols, bags = 400, 128, 60
    rng = np.random.default_rng(21)
    for kind in (capi.FUSED_U8_F32, capi.FUSED_U4_F16):
        table = cases.random_fused_table(rng, rows, cols, kind)
        lengths, idx, w = cases.slws_batch(5, rows, bags, 9, 1.05, np.int32)
        total = int(lengths.sum())
        offs = np.r_[0, np.cumsum(lengths)].astype(np.int32)
        f16 = kind == capi.FUSED_U4_F16
        ww = w[:total].astype(np.float16) if f16 else w[:total]
        got = capi.embedding_bag_rowwise_offsets(table, kind, ww, idx[:total], offs,
                                                 True, f16, False)
        want = go.frwq_slws_generic(table, kind, ww, idx[:total], lengths, f16, False)
        check(got.astype(np.float32), want.astype(np.float32),
              bag_magnitude(table, kind, ww, idx, lengths), f16, what=f"kind {kind}")


def test_rowwise_tables_with_separate_scales():
    rows, cols, bags = 300, 64, 40
    rng = np.random.default_rng(33)
    data = rng.integers(0, 256, (rows, cols), dtype=np.uint8)
    scales = rng.uniform(0.01, 0.03, rows).astype(np.float32)
    offsets = rng.normal(-3, 0.5, rows).astype(np.float32)
    lengths, idx, w = cases.slws_batch(6, rows, bags, 11, 1.05, np.int64)
    total = int(lengths.sum())
    got = capi.rwq_slws(data, scales, offsets, w[:total], idx[:total], lengths)
    want = go.rwq_slws_f32(data, scales, offsets, w[:total], idx[:total], lengths)
    check(got, want, bag_magnitude(data, 0, w, idx, lengths, scales, offsets),
          what="rowwise")


def test_many_bags_and_full_size_config():
    """More than one chunk of bags, and the benchmark configuration at full
    size (4M x 128 table, 4096 bags Poisson(40), Zipf(1.05) int64 indices)."""
    rng = np.random.default_rng(8)
    table = cases.random_fused_table(rng, 5000, 64)
    lengths, idx, w = cases.slws_batch(9, 5000, 20000, 6, 1.05, np.int64)
    check(capi.frwq_slws(table, 0, w, idx, lengths),
          go.frwq_slws_f32(table, w, idx, lengths),
          bag_magnitude(table, 0, w, idx, lengths), what="20000 bags")
    rows, cols, bags = 4_000_000, 128, 4096
    rng = np.random.default_rng(2026)
    table = cases.random_fused_table(rng, rows, cols)
    lengths, idx, w = cases.slws_batch(2027, rows, bags, 40, 1.05, np.int64)
    got = capi.frwq_slws(table, 0, w, idx, lengths)
    want = go.frwq_slws_f32(table, w, idx, lengths)
    check(got, want, bag_magnitude(table, 0, w, idx, lengths), what="full size")
    # the strict arithmetic on the same inputs is bit-exact, and the two agree
    capi.slws_set_fused_math(False)
    try:
        strict = capi.frwq_slws(table, 0, w, idx, lengths)
    finally:
        capi.slws_set_fused_math(True)
    np.testing.assert_array_equal(strict, want)
    np.testing.assert_allclose(got, strict, rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("kind,cols", [(capi.FUSED_U4_F16, 64), (capi.FUSED_U8_F32, 32),
                                       (capi.FUSED_U8_F16, 64), (capi.FUSED_U4_F32, 128)])
def test_short_rows_with_uneven_bags(kind, cols):
    """Rows of 32 or 64 data bytes put 8 or 4 bags side by side in a wavefront:
    neighbours with very different lengths (empty, one lookup, several rounds
    of 32) must not disturb each other, for both index types."""
    rows = 900
    rng = np.random.default_rng(kind * 7 + cols)
    table = cases.random_fused_table(rng, rows, cols, kind)
    lengths = np.array([0, 1, 33, 0, 70, 2, 0, 0, 32, 31, 100, 0, 5, 64, 65, 1, 0, 3] * 3 + [0, 97],
                       np.int32)
    total = int(lengths.sum())
    f16 = kind in (capi.FUSED_U8_F16, capi.FUSED_U4_F16)
    for idt in (np.int64, np.int32):
        idx = rng.integers(0, rows, total).astype(idt)
        w = rng.random(total).astype(np.float16 if f16 else np.float32)
        for weights in (w, None):
            want = go.frwq_slws_generic(table, kind, weights, idx, lengths, f16, False)
            got = capi.frwq_slws(table, kind, weights, idx, lengths, f16, False)
            check(got.astype(np.float32), want.astype(np.float32),
                  bag_magnitude(table, kind, weights, idx, lengths), f16,
                  what=f"{idt.__name__} weights={'yes' if weights is not None else 'no'}")


def test_many_tables_in_one_launch_with_int8_store():
    """The multi-table launch with the fused ConvertTo + Quantize + InsertTensor
    store: dense outputs within the fp32 bar of the sequential loop, the int8
    concatenation within one quantization step of it (a value can land on the
    other side of a rounding boundary), and nearly everywhere equal."""
    kind, cols, rows, bags, n = capi.FUSED_U4_F16, 64, 3000, 500, 5
    rng = np.random.default_rng(77)
    tables = [cases.random_fused_table(rng, rows, cols, kind) for _ in range(n)]
    batches = [cases.slws_batch(80 + t, rows, bags, 20, 1.1, np.int64, weighted=False)
               for t in range(n)]
    lens = [b[0] for b in batches]
    idx = [b[1][:int(b[0].sum())] for b in batches]
    outs = capi.frwq_sls_multi(tables, kind, idx, lens, capi.SLS_OUT_F16)
    q = capi.frwq_sls_multi(tables, kind, idx, lens, capi.SLS_OUT_I8_VIA_F16, 0.05, -3)
    assert q.shape == (bags, n * cols)
    off = 0
    for t in range(n):
        want = go.frwq_slws_generic(tables[t], kind, None, idx[t], lens[t], True, False)
        check(outs[t].astype(np.float32), want.astype(np.float32),
              bag_magnitude(tables[t], kind, None, idx[t], lens[t]), True, what=f"table {t}")
        wq = go.quantize_i8(want.astype(np.float32), 0.05, -3)
        d = np.abs(q[:, off:off + cols].astype(np.int32) - wq.astype(np.int32))
        assert d.max() <= 1 and (d > 0).mean() < 0.01, (t, d.max(), (d > 0).mean())
        off += cols


import os  # noqa: E402

_MORE = max(1, int(os.environ.get("MI355X_TEST_SEEDS", "1")))


@pytest.mark.parametrize("seed", range(40 * _MORE))
def test_random_tables_and_batches(seed):
    """Seeded random kinds, row widths (those the fused kernels take and some
    they do not), table sizes, bag-length distributions, index and weight
    types, lengths and offsets mode."""
    rng = np.random.default_rng(9000 + seed)
    kind = int(rng.integers(0, 4))
    is4 = kind in (capi.FUSED_U4_F16, capi.FUSED_U4_F32)
    data_bytes = int(rng.choice([32, 64, 128, 256, 256, 128, 20, 96]))
    cols = data_bytes * (2 if is4 else 1)
    rows, bags = int(rng.integers(1, 3000)), int(rng.integers(1, 400))
    table = cases.random_fused_table(rng, rows, cols, kind)
    mean = float(rng.choice([0.3, 2, 20, 45, 90]))
    lengths, idx, w = cases.slws_batch(seed, rows, bags, mean, 1.05,
                                       rng.choice([np.int64, np.int32]))
    total = int(lengths.sum())
    idx, w = idx[:total], w[:total]
    f16 = kind in (capi.FUSED_U8_F16, capi.FUSED_U4_F16)
    out16 = f16 and bool(rng.integers(0, 2))
    weights = None if rng.random() < 0.3 else (w.astype(np.float16) if out16 else w)
    say("random", kind, cols, rows, bags, total, out16)
    want = go.frwq_slws_generic(table, kind, weights, idx, lengths, out16, False)
    mag = bag_magnitude(table, kind, weights, idx, lengths)
    got = capi.frwq_slws(table, kind, weights, idx, lengths, out16, False)
    check(got.astype(np.float32), want.astype(np.float32), mag, out16, what="lengths")
    if idx.dtype == np.int32:
        offs = np.r_[0, np.cumsum(lengths)].astype(np.int32)
        ww = weights if weights is not None else np.ones(total, np.float16 if out16 else np.float32)
        got = capi.embedding_bag_rowwise_offsets(table, kind, ww, idx, offs, True, out16, False)
        check(got.astype(np.float32), want.astype(np.float32), mag, out16, what="offsets")


@pytest.mark.parametrize("cols", [128, 256])
def test_bags_per_workgroup_do_not_change_a_bit(cols):
    """Whole rows of 128 and 256 bytes run sixteen bags per workgroup below
    16 384 bags per launch and eight from there on. The same bags must come
    out bit for bit the same whichever launch they are part of, on both sides
    of the boundary, through the lengths and through host-made positions, and
    within the element-wise bar of the oracle."""
    rows = 3000
    rng = np.random.default_rng(100 + cols)
    table = cases.random_fused_table(rng, rows, cols)
    lengths, idx, w = cases.slws_batch(41, rows, 20001, 5, 1.05, np.int64)
    outs = {}
    for bags in (4095, 16383, 16384, 20001):
        L = np.ascontiguousarray(lengths[:bags])
        total = int(L.sum())
        say(f"cols {cols} bags {bags} lookups {total}")
        got = capi.frwq_slws(table, 0, w[:total], idx[:total], L)
        outs[bags] = got
        off = capi.frwq_slws(table, 0, w[:total], idx[:total], L, bag_offsets=True)
        assert np.array_equal(got.view(np.uint32), off.view(np.uint32)), f"offsets, {bags} bags"
    for small in (4095, 16383, 16384):
        assert np.array_equal(outs[small].view(np.uint32),
                              outs[20001][:small].view(np.uint32)), f"{small} of 20001 bags"
    total = int(lengths.sum())
    check(outs[20001], go.frwq_slws_f32(table, w[:total], idx[:total], lengths),
          bag_magnitude(table, 0, w, idx, lengths), what=f"20001 bags of {cols} columns")

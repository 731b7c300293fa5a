"""Data movement and the small operators of ranking models on the GPU through
the C ABI, against the oracle (bit-exact; fp32 sigmoid within 1e-5)."""
import numpy as np
import pytest

from glow_amd import capi
from oracle import glow_oracle as go

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _init():
    capi.init(0)


def test_convert_f16_to_f32():
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.normal(0, 100, 4097), [0, -0.0, 65504, -65504, 6e-8, np.inf]]).astype(np.float16)
    np.testing.assert_array_equal(capi.convert_f16_to_f32(x), x.astype(np.float32))


@pytest.mark.parametrize("dtype,widths", [(np.int8, (64, 351)), (np.int8, (16, 32, 48)),
                                          (np.float32, (13, 64)), (np.int8, (3, 5, 7))])
def test_concat_through_insert(dtype, widths):
    rng = np.random.default_rng(2)
    parts = [rng.integers(-100, 100, (37, w)).astype(dtype) for w in widths]
    np.testing.assert_array_equal(capi.concat_rows(parts), np.concatenate(parts, axis=1))


def test_insert_rejects_overflowing_slice():
    d = capi.DeviceBuffer.empty((4, 8), np.int8)
    with pytest.raises(capi.MI355XError):
        capi.check(capi.lib().mi355x_insert_rows(capi._vp(d), capi._vp(d), capi._sz(4), capi._sz(6),
                                                 capi._sz(8), capi._sz(4), capi._vp(None)))


def test_batch_transpose():
    rng = np.random.default_rng(3)
    x = rng.integers(-128, 128, (50, 27, 64)).astype(np.int8)
    np.testing.assert_array_equal(capi.batch_transpose_i8(x), x.transpose(0, 2, 1))


@pytest.mark.parametrize("idt", [np.int32, np.int64])
def test_gather(idt):
    rng = np.random.default_rng(4)
    data = rng.integers(-128, 128, (33, 729)).astype(np.int8)
    iu = np.triu_indices(27, 1)
    idx = (iu[0] * 27 + iu[1]).astype(idt)
    np.testing.assert_array_equal(capi.gather(data, idx, 1), go.gather(data, idx, 1))
    table = rng.normal(0, 1, (100, 6, 4)).astype(np.float32)
    rows = rng.integers(0, 100, 17).astype(idt)
    np.testing.assert_array_equal(capi.gather(table, rows, 0), go.gather(table, rows, 0))


@pytest.mark.parametrize("b,m,k,n", [(64, 27, 64, 27), (3, 5, 7, 9), (1, 1, 1, 1), (10, 32, 16, 8)])
def test_batch_matmul(b, m, k, n):
    rng = np.random.default_rng(b + m)
    lhs = rng.integers(-128, 128, (b, m, k)).astype(np.int8)
    rhs = rng.integers(-128, 128, (b, k, n)).astype(np.int8)
    for oo, lo, ro, ratio in [(3, -4, 5, 0.004), (-128, 0, 0, 0.0007), (0, 127, -128, 0.02)]:
        p = go.quantize_scale_offset_32to8(ratio, 0)[:3]
        np.testing.assert_array_equal(capi.batch_matmul_i8(lhs, rhs, oo, lo, ro, p),
                                      go.batch_matmul_i8(lhs, rhs, oo, lo, ro, p))


def test_sigmoid():
    rng = np.random.default_rng(5)
    x = np.concatenate([rng.normal(0, 5, 10000), [0.0, 30.0, -30.0, 88.0, -88.0]]).astype(np.float32)
    np.testing.assert_allclose(capi.sigmoid_f32(x), go.sigmoid_f32(x), rtol=1e-5, atol=1e-37)


@pytest.mark.parametrize("kind,cols,idt", [(2, 64, np.int64), (0, 128, np.int32), (1, 40, np.int64),
                                           (3, 16, np.int32)])
def test_multi_table_sls(kind, cols, idt):
    """Several tables in one launch give what one launch per table gives; with
    the int8 output kinds, what ConvertTo + Quantize + InsertTensor behind each
    lookup give."""
    from tests import cases
    rng = np.random.default_rng(40 + kind)
    n, bags = 5, 300
    tables = [cases.random_fused_table(rng, 700 + 10 * t, cols, kind) for t in range(n)]
    lens, idx = [], []
    for t in range(n):
        ln, ix, _ = cases.slws_batch(50 + t, tables[t].shape[0], bags, 7, 1.1, idt, weighted=False)
        if t == 2:
            ln[:] = 0                       # a table whose bags are all empty
            ix = ix[:0]
        lens.append(ln)
        idx.append(ix)
    f16 = kind in (1, 2)
    want = [go.frwq_slws_generic(tables[t], kind, None, idx[t], lens[t], out_f16=f16) for t in range(n)]
    got = capi.frwq_sls_multi(tables, kind, idx, lens,
                              capi.SLS_OUT_F16 if f16 else capi.SLS_OUT_F32)
    for t in range(n):
        np.testing.assert_array_equal(got[t], want[t], err_msg=f"table {t}")
    scale, off = 0.37, -11
    wq = np.concatenate([go.quantize_i8(w.astype(np.float32), scale, off) for w in want], axis=1)
    gq = capi.frwq_sls_multi(tables, kind, idx, lens,
                             capi.SLS_OUT_I8_VIA_F16 if f16 else capi.SLS_OUT_I8, scale, off)
    np.testing.assert_array_equal(gq, wq)
    # the bags of every table as positions instead of lengths: the same bytes
    got = capi.frwq_sls_multi(tables, kind, idx, lens,
                              capi.SLS_OUT_F16 if f16 else capi.SLS_OUT_F32, bag_offsets=True)
    for t in range(n):
        np.testing.assert_array_equal(got[t], want[t], err_msg=f"table {t}, bag offsets")
    gq = capi.frwq_sls_multi(tables, kind, idx, lens,
                             capi.SLS_OUT_I8_VIA_F16 if f16 else capi.SLS_OUT_I8, scale, off,
                             bag_offsets=True)
    np.testing.assert_array_equal(gq, wq)


@pytest.mark.parametrize("cols,idt", [(128, np.int64), (37, np.int32), (64, np.int64), (16, np.int32)])
def test_rowwise_quantized_slws(cols, idt):
    """Separate per-row scales and offsets instead of fused rows (bit-exact)."""
    rng = np.random.default_rng(cols)
    rows, bags = 3000, 500
    data = rng.integers(0, 256, (rows, cols), dtype=np.uint8)
    scales = rng.uniform(0.001, 0.1, rows).astype(np.float32)
    offsets = rng.normal(0, 1, rows).astype(np.float32)
    lengths = rng.poisson(9, bags).astype(np.int32)
    lengths[7] = 0
    idx = rng.integers(0, rows, int(lengths.sum())).astype(idt)
    w = rng.random(idx.size).astype(np.float32)
    np.testing.assert_array_equal(capi.rwq_slws(data, scales, offsets, w, idx, lengths),
                                  go.rwq_slws_f32(data, scales, offsets, w, idx, lengths))
    ones = np.ones(idx.size, np.float32)
    np.testing.assert_array_equal(capi.rwq_slws(data, scales, offsets, None, idx, lengths),
                                  go.rwq_slws_f32(data, scales, offsets, ones, idx, lengths))


@pytest.mark.parametrize("shape", [(37, 27, 64, 27), (5, 32, 32, 32), (3, 40, 48, 70), (9, 1, 16, 5),
                                   (4, 64, 128, 33)])
def test_batch_matmul_with_k_contiguous_right_operand(shape):
    """lhs x transpose(rhs_nk) equals BatchMatMul(lhs, transposed copy), bit for bit."""
    b, m, k, n = shape
    rng = np.random.default_rng(sum(shape))
    lhs = rng.integers(-128, 128, (b, m, k)).astype(np.int8)
    rhs_nk = rng.integers(-128, 128, (b, n, k)).astype(np.int8)
    for (oo, lo, ro, outP) in ((3, -5, 7, (2, 9, 300)), (-128, 127, -128, (0, 14, 411)),
                               (0, 0, 0, (0, 0, 1))):
        want = go.batch_matmul_i8(lhs, np.ascontiguousarray(rhs_nk.transpose(0, 2, 1)), oo, lo, ro, outP)
        got = capi.batch_matmul_nt_i8(lhs, rhs_nk, oo, lo, ro, outP)
        np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("rows,cols,wide,col", [(33, 64, 200, 64), (7, 13, 29, 5), (1, 4, 4, 0),
                                                (300, 16, 48, 32)])
def test_rescale_written_as_a_slice(rows, cols, wide, col):
    """RescaleQuantized + InsertTensor in one pass: the slice holds the oracle's
    rescale, every other byte of the wide tensor is untouched."""
    rng = np.random.default_rng(rows + cols)
    q = rng.integers(-128, 128, (rows, cols)).astype(np.int8)
    into = rng.integers(-128, 128, (rows, wide)).astype(np.int8)
    for ratio, oo, io in [(1.7, 3, -4), (0.013, -128, 100), (300.0, 0, 0)]:
        pre, post, scale, _ = go.quantize_scale_offset_32to8(ratio, 0)
        want = into.copy()
        want[:, col:col + cols] = go.rescale_i8(q, oo, io, pre, post, scale)
        np.testing.assert_array_equal(capi.rescale_rows_i8(q, into, col, oo, io, pre, post, scale), want)


@pytest.mark.parametrize("idt", [np.int32, np.int64])
def test_gather_written_as_a_slice(idt):
    rng = np.random.default_rng(8)
    data = rng.integers(-128, 128, (33, 729)).astype(np.int8)
    iu = np.triu_indices(27, 1)
    idx = (iu[0] * 27 + iu[1]).astype(idt)
    into = rng.integers(-128, 128, (33, 64 + idx.size + 3)).astype(np.int8)
    want = into.copy()
    want[:, 64:64 + idx.size] = go.gather(data, idx, 1)
    np.testing.assert_array_equal(capi.gather_rows(data, idx, into, 64), want)
    # wider slices (fp32 rows of 4 values)
    table = rng.normal(0, 1, (20, 6, 4)).astype(np.float32)
    pick = np.array([5, 0, 5, 2], idt)
    into = np.zeros((20, 40), np.float32)
    want = into.copy()
    want[:, 8:24] = go.gather(table, pick, 1).reshape(20, 16)
    np.testing.assert_array_equal(capi.gather_rows(table, pick, into, 8), want)


def test_dequantize_then_sigmoid_in_one_pass():
    q = np.arange(-128, 128).astype(np.int8).reshape(16, 16)
    for scale, offset in [(0.05, 3), (0.7, -128), (1e-3, 127)]:
        want = go.sigmoid_f32(go.dequantize_i8(q, scale, offset))
        np.testing.assert_allclose(capi.dequantize_sigmoid(q, scale, offset), want, rtol=1e-5, atol=1e-37)


@pytest.mark.parametrize("b,m,k,n", [(64, 27, 64, 27), (5, 40, 32, 33), (3, 4, 16, 9)])
def test_product_of_which_only_picked_elements_are_written(b, m, k, n):
    """BatchMatMul + Gather of single elements + InsertTensor in one pass: the
    picked elements of the oracle's product land where the list says, the rest
    of the wide tensor is untouched."""
    rng = np.random.default_rng(b * m)
    lhs = rng.integers(-128, 128, (b, m, k)).astype(np.int8)
    rhs = rng.integers(-128, 128, (b, n, k)).astype(np.int8)
    pick = rng.permutation(m * n)[: max(1, (m * n) // 3)].astype(np.int64)
    dest_of = np.full(m * n, -1, np.int32)
    dest_of[pick] = np.arange(pick.size, dtype=np.int32)
    into = rng.integers(-128, 128, (b, pick.size + 11)).astype(np.int8)
    for oo, lo, ro, ratio in [(3, -4, 5, 0.004), (-128, 0, 0, 0.0007)]:
        p = go.quantize_scale_offset_32to8(ratio, 0)[:3]
        z = go.batch_matmul_i8(lhs, np.ascontiguousarray(rhs.transpose(0, 2, 1)), oo, lo, ro, p)
        want = into.copy()
        want[:, 7:7 + pick.size] = go.gather(z.reshape(b, m * n), pick, 1)
        got = capi.batch_matmul_nt_select_i8(lhs, rhs, oo, lo, ro, p, dest_of, into, 7)
        np.testing.assert_array_equal(got, want)

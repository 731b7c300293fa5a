"""Seeded random shapes through every contraction and lookup entry point,
against the oracle: odd sizes, unaligned K, few and many rows, every fused
kind. Fixed seeds; the cases differ from the hand-picked ones elsewhere only
in that nobody chose them."""
import os

import numpy as np
import pytest

from glow_amd import capi
from oracle import glow_oracle as go
from tests import cases

pytestmark = pytest.mark.gpu

# MI355X_TEST_SEEDS=10 runs ten times as many cases of each kind
_MORE = max(1, int(os.environ.get("MI355X_TEST_SEEDS", "1")))


@pytest.fixture(scope="module", autouse=True)
def _device():
    capi.init(0)
    yield
    capi.sync()


def _dim(rng, hi, mult_of=1):
    """A size in [1, hi], biased towards small values and the multiples of 16/64
    where the kernels change path."""
    r = rng.random()
    if r < 0.3:
        v = int(rng.integers(1, 20))
    elif r < 0.6:
        v = int(rng.choice([16, 32, 48, 64, 128, 192, 256])) + int(rng.integers(-1, 2))
    else:
        v = int(rng.integers(1, hi + 1))
    v = max(1, min(hi, v))
    return max(mult_of, v // mult_of * mult_of)


@pytest.mark.parametrize("seed", range(40 * _MORE))
def test_rowwise_fc(seed):
    rng = np.random.default_rng(1000 + seed)
    M, K, N = _dim(rng, 400), _dim(rng, 600), _dim(rng, 400)
    c = cases.rwq_fc_case(seed, M, K, N, symmetric=bool(rng.integers(0, 2)),
                          bias_i8=bool(rng.integers(0, 2)), out_offset=int(rng.integers(-128, 128)))
    print("rwq_fc", M, K, N, flush=True)
    want = go.rwq_fc_i8(*cases.rwq_fc_args(c))
    np.testing.assert_array_equal(capi.rwq_fc_i8(*cases.rwq_fc_args(c)), want)
    np.testing.assert_array_equal(
        capi.rwq_fc_i8(*cases.rwq_fc_args(c), precomputed_sums=False), want)


@pytest.mark.parametrize("seed", range(20 * _MORE))
def test_plain_fc(seed):
    rng = np.random.default_rng(2000 + seed)
    M, K, N = _dim(rng, 300), _dim(rng, 500), _dim(rng, 300)
    c = cases.fc_case(seed, M, K, N, bias_i8=bool(rng.integers(0, 2)))
    print("fc", M, K, N, flush=True)
    args = cases.fc_args(c)
    np.testing.assert_array_equal(capi.fc_i8(*args), go.fc_i8(*args))


@pytest.mark.parametrize("seed", range(40 * _MORE))
def test_convolution(seed):
    rng = np.random.default_rng(3000 + seed)
    group = int(rng.choice([1, 1, 1, 2, 4]))
    icg = int(rng.choice([1, 3, 4, 8, 16, 16, 32, 48, 64, 80]))
    ocg = int(rng.choice([1, 5, 8, 16, 24, 64]))
    kh, kw = int(rng.integers(1, 4)), int(rng.integers(1, 4))
    dil = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
    stride = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
    H = int(rng.integers((kh - 1) * dil[0] + 1, 14))
    W = int(rng.integers((kw - 1) * dil[1] + 1, 14))
    pads = tuple(int(v) for v in rng.integers(0, 3, 4))
    kw_ = dict(N=int(rng.integers(1, 4)), H=H, W=W, IC=icg * group, OC=ocg * group,
               kernel=(kh, kw), stride=stride, pads=pads, group=group, dilation=dil,
               act=int(rng.choice([go.ACT_NONE, go.ACT_RELU, go.ACT_CLIP, go.ACT_LEAKY_RELU])),
               in_offset=int(rng.integers(-128, 128)), out_offset=int(rng.integers(-128, 128)),
               symmetric=bool(rng.integers(0, 2)), bias_i8=bool(rng.integers(0, 2)))
    print("conv", kw_, flush=True)
    c = cases.cwq_conv_case(seed, **kw_)
    want = go.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    np.testing.assert_array_equal(capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)), want)
    np.testing.assert_array_equal(
        capi.cwq_conv2d_i8(*cases.cwq_conv_args(c), precomputed_sums=False), want)


@pytest.mark.parametrize("seed", range(30 * _MORE))
def test_lookups_strict_arithmetic(seed):
    rng = np.random.default_rng(4000 + seed)
    kind = int(rng.integers(0, 4))
    is4 = kind in (capi.FUSED_U4_F16, capi.FUSED_U4_F32)
    cols = _dim(rng, 300, 2 if is4 else 1)
    rows, bags = int(rng.integers(1, 2000)), int(rng.integers(1, 300))
    table = cases.random_fused_table(rng, rows, cols, kind)
    lengths, idx, w = cases.slws_batch(seed, rows, bags, float(rng.choice([0.5, 3, 20, 70])),
                                       1.05, rng.choice([np.int64, np.int32]))
    total = int(lengths.sum())
    idx, w = idx[:total], w[:total]
    f16 = kind in (capi.FUSED_U8_F16, capi.FUSED_U4_F16)
    out16 = f16 and bool(rng.integers(0, 2))
    acc16 = out16 and bool(rng.integers(0, 2))
    weights = None if rng.random() < 0.3 else (w.astype(np.float16) if out16 else w)
    print("slws", kind, cols, rows, bags, total, out16, acc16, flush=True)
    want = go.frwq_slws_generic(table, kind, weights, idx, lengths, out16, acc16)
    got = capi.frwq_slws(table, kind, weights, idx, lengths, out16, acc16)
    np.testing.assert_array_equal(got.view(np.uint16 if out16 else np.uint32),
                                  want.view(np.uint16 if out16 else np.uint32))


def _params(rng):
    """A plausible (pre, post, scale) triple: sometimes small, sometimes beyond
    the 24-bit multiplier, sometimes with a pre-shift."""
    r = rng.random()
    if r < 0.5:
        return (0, int(rng.integers(6, 12)), int(rng.integers(128, 600)))
    if r < 0.75:
        return (int(rng.integers(1, 4)), int(rng.integers(8, 16)), int(rng.integers(200, 520)))
    if r < 0.9:
        return (0, int(rng.integers(18, 26)), int(rng.integers(1 << 23, 1 << 26)))
    return (0, 0, 1)


@pytest.mark.parametrize("seed", range(30 * _MORE))
def test_pools(seed):
    rng = np.random.default_rng(5000 + seed)
    kh, kw = int(rng.integers(1, 5)), int(rng.integers(1, 5))
    stride = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
    pads = (int(rng.integers(0, kh)), int(rng.integers(0, kw)),
            int(rng.integers(0, kh)), int(rng.integers(0, kw)))
    H, W = int(rng.integers(kh, 16)), int(rng.integers(kw, 16))
    C = int(rng.choice([1, 3, 4, 7, 16, 20, 64]))
    x = rng.integers(-128, 128, (int(rng.integers(1, 4)), H, W, C)).astype(np.int8)
    print("pool", x.shape, (kh, kw), stride, pads, flush=True)
    off = int(rng.integers(-128, 128))
    np.testing.assert_array_equal(capi.max_pool_i8(x, (kh, kw), stride, pads, off),
                                  go.max_pool_i8(x, (kh, kw), stride, pads, off))
    P = _params(rng)
    for cip in (True, False):
        args = ((kh, kw), stride, pads, cip, int(rng.integers(-128, 128)),
                int(rng.integers(-128, 128)), P)
        np.testing.assert_array_equal(capi.avg_pool_i8(x, *args), go.avg_pool_i8(x, *args))


@pytest.mark.parametrize("seed", range(30 * _MORE))
def test_elementwise_and_glue(seed):
    rng = np.random.default_rng(6000 + seed)
    n = int(rng.choice([1, 3, 15, 16, 17, 255, 1000, 4099, 70001]))
    q = rng.integers(-128, 128, n).astype(np.int8)
    r = rng.integers(-128, 128, n).astype(np.int8)
    x = (rng.normal(0, 3, n) * rng.choice([1e-3, 1, 50])).astype(np.float32)
    s, o = float(rng.choice([0.003, 0.05, 1.7])), int(rng.integers(-128, 128))
    print("elementwise", n, s, o, flush=True)
    np.testing.assert_array_equal(capi.quantize_i8(x, s, o), go.quantize_i8(x, s, o))
    np.testing.assert_array_equal(capi.dequantize_i8(q, s, o).view(np.uint32),
                                  go.dequantize_i8(q, s, o).view(np.uint32))
    P, Q, R = _params(rng), _params(rng), _params(rng)
    oo, io = int(rng.integers(-128, 128)), int(rng.integers(-128, 128))
    np.testing.assert_array_equal(capi.rescale_i8(q, oo, io, *P), go.rescale_i8(q, oo, io, *P))
    lo, ro = int(rng.integers(-128, 128)), int(rng.integers(-128, 128))
    want = go.add_i8(q, r, oo, lo, ro, P, Q)
    np.testing.assert_array_equal(capi.add_i8(q, r, oo, lo, ro, P, Q), want)
    do = int(rng.integers(-128, 128))
    np.testing.assert_array_equal(capi.relu_i8(q, io, do, R), go.relu_i8(q, io, do, R))
    np.testing.assert_array_equal(capi.add_relu_i8(q, r, oo, lo, ro, P, Q, do, R),
                                  go.relu_i8(want, oo, do, R))


@pytest.mark.parametrize("seed", range(30 * _MORE))
def test_small_matrix_products(seed):
    rng = np.random.default_rng(7000 + seed)
    b, m, n = int(rng.integers(1, 40)), int(rng.integers(1, 70)), int(rng.integers(1, 70))
    k = int(rng.integers(1, 9)) * 16
    lhs = rng.integers(-128, 128, (b, m, k)).astype(np.int8)
    rhs_nk = rng.integers(-128, 128, (b, n, k)).astype(np.int8)
    rhs = np.ascontiguousarray(rhs_nk.transpose(0, 2, 1))
    oo, lo, ro = (int(v) for v in rng.integers(-128, 128, 3))
    P = _params(rng)
    print("bmm", b, m, k, n, P, flush=True)
    want = go.batch_matmul_i8(lhs, rhs, oo, lo, ro, P)
    np.testing.assert_array_equal(capi.batch_matmul_nt_i8(lhs, rhs_nk, oo, lo, ro, P), want)
    if (m + n) * k <= 64 * 1024:
        np.testing.assert_array_equal(capi.batch_matmul_i8(lhs, rhs, oo, lo, ro, P), want)
    # the single-matrix product, odd K included
    k2 = int(rng.integers(1, 200))
    a = rng.integers(-128, 128, (m, k2)).astype(np.int8)
    bb = rng.integers(-128, 128, (k2, n)).astype(np.int8)
    np.testing.assert_array_equal(capi.matmul_i8(a, bb, oo, lo, ro, P),
                                  go.matmul_i8(a, bb, oo, lo, ro, P))
    np.testing.assert_array_equal(capi.batch_transpose_i8(lhs), lhs.transpose(0, 2, 1))
    np.testing.assert_array_equal(capi.transpose2d_i8(a), a.T)


@pytest.mark.parametrize("seed", range(20 * _MORE))
def test_other_lookup_forms(seed):
    rng = np.random.default_rng(8000 + seed)
    rows, bags = int(rng.integers(1, 1500)), int(rng.integers(1, 200))
    cols = _dim(rng, 300)
    # byte rows with separate fp32 scales and offsets
    data = rng.integers(0, 256, (rows, cols), dtype=np.uint8)
    scales = rng.uniform(0.01, 0.03, rows).astype(np.float32)
    offsets = rng.normal(-3, 0.5, rows).astype(np.float32)
    lengths, idx, w = cases.slws_batch(seed, rows, bags, float(rng.choice([1, 8, 40])), 1.05,
                                       rng.choice([np.int64, np.int32]))
    total = int(lengths.sum())
    print("lookups", rows, bags, cols, total, flush=True)
    np.testing.assert_array_equal(
        capi.rwq_slws(data, scales, offsets, w[:total], idx[:total], lengths).view(np.uint32),
        go.rwq_slws_f32(data, scales, offsets, w[:total], idx[:total], lengths).view(np.uint32))
    # bags given by offsets
    table = cases.random_fused_table(rng, rows, cols)
    offs = np.r_[0, np.cumsum(lengths)].astype(np.int32)
    i32 = idx[:total].astype(np.int32)
    for has_end in (True, False):
        o = offs if has_end else offs[:-1]
        got = capi.embedding_bag_rowwise_offsets(table, capi.FUSED_U8_F32, w[:total], i32, o,
                                                 has_end, False, False)
        want = go.embedding_bag_byte_rowwise_offsets_f32(table, w[:total], i32, o, has_end)
        np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    # gather of rows and of per-sample slices
    d = rng.integers(-128, 128, (int(rng.integers(1, 30)), int(rng.integers(1, 50)),
                                 int(rng.integers(1, 9)))).astype(np.int8)
    gi = rng.integers(0, d.shape[1], int(rng.integers(1, 60))).astype(rng.choice([np.int64, np.int32]))
    np.testing.assert_array_equal(capi.gather(d, gi, 1), go.gather(d, gi, 1))
    g0 = rng.integers(0, d.shape[0], 17).astype(np.int64)
    np.testing.assert_array_equal(capi.gather(d, g0, 0), go.gather(d, g0, 0))


@pytest.mark.parametrize("seed", range(30 * _MORE))
def test_unlowered_element_operators(seed):
    """Clip, LeakyRelu, Max(x, Splat) and BatchedAdd over random sizes
    (aligned and not, below and above one 16-byte piece) and parameters."""
    rng = np.random.default_rng(9000 + seed)
    n = int(rng.choice([1, 5, 15, 16, 17, 63, 1000, 4099, 65537]))
    q = rng.integers(-128, 128, n).astype(np.int8)
    so, do = int(rng.integers(-128, 128)), int(rng.integers(-128, 128))
    lo, hi = sorted(int(v) for v in rng.integers(-128, 128, 2))
    P, Q = _params(rng), _params(rng)
    print("element operators", n, so, do, lo, hi, P, Q, flush=True)
    np.testing.assert_array_equal(capi.clip_elem_i8(q, lo, hi, so, do, P),
                                  go.clip_elem_i8(q, lo, hi, so, do, P))
    np.testing.assert_array_equal(capi.leaky_relu_i8(q, so, do, P, Q),
                                  go.leaky_relu_i8(q, so, do, P, Q))
    v = int(rng.integers(-128, 128))
    np.testing.assert_array_equal(capi.max_splat_i8(q, v), go.max_splat_i8(q, v))
    slices, size = int(rng.integers(1, 40)), int(rng.choice([1, 3, 4, 12, 64, 250, 1000]))
    batch = rng.integers(-128, 128, (slices, size)).astype(np.int8)
    sl = (rng.integers(-30000, 30000, size).astype(np.int32) if rng.integers(0, 2)
          else rng.integers(-128, 128, size).astype(np.int8))
    bo, slo = int(rng.integers(-128, 128)), int(rng.integers(-128, 128))
    np.testing.assert_array_equal(capi.batched_add_i8(batch, sl, do, bo, slo, P, Q),
                                  go.batched_add_i8(batch, sl, do, bo, slo, P, Q))


@pytest.mark.parametrize("seed", range(20 * _MORE))
def test_k_loop_split_over_workgroups(seed):
    """The named K-split tile on random products (K a multiple of 64 with at
    least two steps, symmetric weights): the oracle's bytes, and the workspace
    ready for the next launch."""
    rng = np.random.default_rng(9500 + seed)
    M, N = _dim(rng, 500), _dim(rng, 400)
    K = 64 * int(rng.integers(2, 40))
    c = cases.rwq_fc_case(seed, M, K, N, symmetric=True, bias_i8=bool(rng.integers(0, 2)),
                          out_offset=int(rng.integers(-128, 128)))
    print("rwq_fc, K split", M, K, N, flush=True)
    need = capi.gemm_splitk_workspace_bytes(M, N, K, named=True)
    ws = capi.DeviceBuffer(need)
    ws.fill(0)
    opts = capi.LaunchOpts(gemm_tile=capi.TILE_SPLIT_K, workspace=ws)
    want = go.rwq_fc_i8(*cases.rwq_fc_args(c))
    for _ in range(2):
        np.testing.assert_array_equal(capi.rwq_fc_i8(*cases.rwq_fc_args(c), opts=opts), want)

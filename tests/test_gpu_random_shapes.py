"""Seeded random shapes through every contraction and lookup entry point,
against the oracle: odd sizes, unaligned K, few and many rows, every fused
kind. Fixed seeds; the cases differ from the hand-picked ones elsewhere only
in that nobody chose them."""
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


@pytest.mark.parametrize("seed", range(40))
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


@pytest.mark.parametrize("seed", range(20))
def test_plain_fc(seed):
    rng = np.random.default_rng(2000 + seed)
    M, K, N = _dim(rng, 300), _dim(rng, 500), _dim(rng, 300)
    c = cases.fc_case(seed, M, K, N, bias_i8=bool(rng.integers(0, 2)))
    print("fc", M, K, N, flush=True)
    args = cases.fc_args(c)
    np.testing.assert_array_equal(capi.fc_i8(*args), go.fc_i8(*args))


@pytest.mark.parametrize("seed", range(40))
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


@pytest.mark.parametrize("seed", range(30))
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

"""GPU parity tests: every HIP entry point, called through the C ABI, against
the CPU oracle on identical seeded inputs and against the committed golden
vectors (outputs of the reference's compiled libjit). Integer outputs must be
bit-exact; fp32 / fp16 SLWS and dequantize outputs are also compared bit for
bit (the kernels round every multiply and add separately, in bag order, like
the oracle), which is inside the 1e-5 relative bar.

Run on the GPU box:  python -u -m pytest tests -m gpu -x -v --timeout 120
"""
import numpy as np
import pytest

from glow_amd import capi
from oracle import glow_oracle as go
from tests import cases
from tests import golden_io as gio

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _device():
    capi.init(0)
    info = capi.device_info()
    print("device:", info.name.decode(), info.arch.decode(),
          info.compute_units, "CUs", "LDS/block", info.lds_bytes_per_block,
          flush=True)
    yield
    capi.sync()


def say(*a):
    print(*a, flush=True)


# ---- elementwise -----------------------------------------------------------------

def test_elementwise_golden():
    d = gio.elementwise()
    for i in range(3):
        s, o = d[f"quant{i}_params"]
        np.testing.assert_array_equal(capi.quantize_i8(d["x"], float(s), int(o)),
                                      d[f"quant{i}_out"])
        np.testing.assert_array_equal(capi.dequantize_i8(d["q"], float(s), int(o)),
                                      d[f"dequant{i}_out"])
    for i in range(4):
        oo, io, pre, post, sc = (int(v) for v in d[f"rescale{i}_params"])
        np.testing.assert_array_equal(
            capi.rescale_i8(d["q"], oo, io, pre, post, sc), d[f"rescale{i}_out"])


@pytest.mark.parametrize("n", [0, 1, 15, 16, 17, 4097, 1 << 20, (1 << 22) + 5])
def test_elementwise_vs_oracle(n):
    say("elementwise n", n)
    rng = np.random.default_rng(n)
    x = (rng.normal(0, 4, n)).astype(np.float32)
    if n > 100:
        x[:64] = (np.arange(64) - 32 + 0.5) * 0.05  # exact rounding ties
        x[64:70] = [1e9, -1e9, 1e-30, -0.0, 6.35, -6.4]
    for scale, off in [(0.05, -3), (0.1, 0), (0.0173, 50)]:
        q = capi.quantize_i8(x, scale, off)
        np.testing.assert_array_equal(q, go.quantize_i8(x, scale, off))
        np.testing.assert_array_equal(capi.dequantize_i8(q, scale, off),
                                      go.dequantize_i8(q, scale, off))
    q = rng.integers(-128, 128, n).astype(np.int8)
    for ratio, io, oo in [(0.37, 4, -9), (1.0, 0, 0), (2.5, -100, 100), (0.0009, 3, 3)]:
        pre, post, sc, _ = go.quantize_scale_offset_32to8(ratio, 0)
        np.testing.assert_array_equal(capi.rescale_i8(q, oo, io, pre, post, sc),
                                      go.rescale_i8(q, oo, io, pre, post, sc))


def test_elementwise_unaligned_views():
    # a tensor view at an odd byte offset inside an allocation takes the
    # scalar path
    rng = np.random.default_rng(5)
    n = 1000
    q = rng.integers(-128, 128, n + 3).astype(np.int8)
    d_in = capi.to_device(q)
    d_out = capi.DeviceBuffer.empty((n + 3,), np.int8)
    d_out.fill(0)
    pre, post, sc, _ = go.quantize_scale_offset_32to8(0.4, 0)
    capi.launch_rescale_i8(d_out.ptr + 3, d_in.ptr + 3, n, -2, 5, pre, post, sc)
    got = d_out.numpy()
    np.testing.assert_array_equal(got[3:], go.rescale_i8(q[3:], -2, 5, pre, post, sc))
    np.testing.assert_array_equal(got[:3], 0)


# ---- RowwiseQuantizedFullyConnected ------------------------------------------------

def test_rwq_fc_golden():
    for tag, args, want in gio.rwq_fc_cases():
        say("rwq_fc golden", tag)
        np.testing.assert_array_equal(capi.rwq_fc_i8(*args), want)


RWQ_SHAPES = [
    (1, 16, 1), (2, 100, 5), (7, 37, 11), (33, 64, 65), (128, 1024, 1024),
    (130, 80, 257), (300, 256, 200), (64, 13, 512), (257, 415, 96),
    (1024, 512, 256), (4096, 64, 64),
]


@pytest.mark.parametrize("shape", RWQ_SHAPES)
def test_rwq_fc_vs_oracle(shape):
    M, K, N = shape
    for seed, sym, b8 in [(1, True, False), (2, False, False), (3, False, True)]:
        say("rwq_fc", shape, "symmetric" if sym else "asymmetric",
            "bias8" if b8 else "bias32")
        c = cases.rwq_fc_case(seed + M, M, K, N, symmetric=sym, bias_i8=b8,
                              bias_scale=(0.01 if b8 else 5e-5),
                              bias_offset=(3 if b8 else 0))
        want = go.rwq_fc_i8(*cases.rwq_fc_args(c))
        np.testing.assert_array_equal(capi.rwq_fc_i8(*cases.rwq_fc_args(c)), want)
        # without precomputed weight row sums the kernel forms them itself
        np.testing.assert_array_equal(
            capi.rwq_fc_i8(*cases.rwq_fc_args(c), precomputed_sums=False), want)
    # zero input offset and symmetric weights: the path without row sums
    c = cases.rwq_fc_case(9, M, K, N, in_offset=0)
    np.testing.assert_array_equal(capi.rwq_fc_i8(*cases.rwq_fc_args(c)),
                                  go.rwq_fc_i8(*cases.rwq_fc_args(c)))


@pytest.mark.parametrize("K", [64, 256, 448, 511, 512])
def test_rwq_fc_with_accumulators_and_constants_around_2_to_the_23(K):
    """Operands that give the largest possible sums (every product +16384),
    column constants that bring accumulator + constant to just below and just
    above 2^23, scales up to 2^23 - 1 (products that wrap around 32 bits):
    where a shortcut through a narrower multiplier would first go wrong."""
    M, N = 96, 128
    rng = np.random.default_rng(K)
    lim = (1 << 23) - min(K, 511) * 16384
    x = np.full((M, K), -128, np.int8)
    w = np.full((N, K), -128, np.int8)        # every product +16384: the largest sum
    x[M // 2:] = 127
    w[1::2, ::3] = 127
    bias = np.empty(N, np.int32)
    bias[0::4] = lim - 1
    bias[1::4] = -lim
    bias[2::4] = rng.integers(-1000, 1000, N // 4)
    bias[3::4] = lim - 1
    for outside in (False, True):
        b = bias.copy()
        if outside:
            b[3::4] = lim + 5                 # one column in four leaves the bound
        one = np.ones(N, np.int32)
        zero = np.zeros(N, np.int32)
        out_scale = rng.integers(256, 512, N).astype(np.int32)
        out_scale[::5] = (1 << 23) - 1
        out_pre = rng.integers(0, 9, N).astype(np.int32)
        out_post = rng.integers(8, 24, N).astype(np.int32)
        args = (x, w, b, zero, zero, zero, one, out_pre, out_post, out_scale, 3, 0, 0)
        want = go.rwq_fc_i8(*args)
        assert len(np.unique(want)) > 3
        np.testing.assert_array_equal(capi.rwq_fc_i8(*args), want)


def test_rwq_fc_every_row_length_up_to_three_chunks():
    """Rows that are not a whole number of 16-byte chunks: every remainder 1..15
    both for rows shorter than one chunk and for longer ones (the last chunk is
    read as the 16 bytes that end with the row and shifted down)."""
    for K in range(1, 50):
        for M, N in [(9, 5), (70, 66)]:
            c = cases.rwq_fc_case(1000 + K, M, K, N, symmetric=False)
            want = go.rwq_fc_i8(*cases.rwq_fc_args(c))
            got = capi.rwq_fc_i8(*cases.rwq_fc_args(c), precomputed_sums=False)
            assert np.array_equal(got, want), (M, K, N)


@pytest.mark.parametrize("shape", [(128, 1024, 1024), (300, 13, 512), (77, 415, 96), (4096, 512, 256)])
def test_rwq_fc_with_fused_relu(shape):
    """RowwiseQuantizedFullyConnected + Relu in one kernel equals the two
    instructions run one after the other, for both multiplier paths of the
    Relu rescale."""
    M, K, N = shape
    say("rwq_fc+relu", shape)
    c = cases.rwq_fc_case(M + K, M, K, N, symmetric=(K % 2 == 0))
    args = cases.rwq_fc_args(c)
    fc = go.rwq_fc_i8(*args)
    for relu_offset, reluP in ((-128, (0, 8, 300)), (5, (1, 9, 1 << 24)), (-3, (0, 0, 1))):
        want = go.relu_i8(fc, c["out_offset"], relu_offset, reluP)
        got = capi.rwq_fc_relu_i8(*args[:10], c["out_offset"], c["in_offset"], c["bias_offset"],
                                  relu_offset, reluP)
        np.testing.assert_array_equal(got, want)


def test_rwq_fc_large_tiles_properties():
    """A mid-size product with whatever tile the shape rules pick (the forced
    tiles on long K loops are in test_gpu_gemm_tiles.py). The oracle runs on a
    row sample; all rows are checked through independence in the batch
    dimension: identical input rows must give identical output rows."""
    M, K, N = 4096, 1024, 1024
    say("rwq_fc large", (M, K, N))
    c = cases.rwq_fc_case(77, M, K, N, symmetric=False)
    c["x"][2048:] = c["x"][:2048]          # second half repeats the first
    got = capi.rwq_fc_i8(*cases.rwq_fc_args(c))
    np.testing.assert_array_equal(got[2048:], got[:2048])
    rows = np.r_[0:40, 1000:1040, 2040:2048]
    cs = dict(c, x=c["x"][rows])
    np.testing.assert_array_equal(got[rows], go.rwq_fc_i8(*cases.rwq_fc_args(cs)))
    assert got.std() > 5


def test_rwq_fc_wraparound_matches():
    # accumulators pushed beyond int32 wrap identically on both sides
    rng = np.random.default_rng(4)
    M, K, N = 8, 4096, 16
    x = np.full((M, K), 127, np.int8)
    w = np.full((N, K), 127, np.int8)
    w[::2] = -128
    bias = np.full(N, 2 ** 29, np.int32)
    z = np.zeros(N, np.int32)
    woff = np.full(N, -128, np.int32)
    bp = (z, z, np.full(N, 7, np.int32))
    op = (np.full(N, 2, np.int32), np.full(N, 9, np.int32), np.full(N, 300, np.int32))
    args = (x, w, bias, woff, *bp, *op, 3, -128, 0)
    np.testing.assert_array_equal(capi.rwq_fc_i8(*args), go.rwq_fc_i8(*args))
    del rng


# ---- FullyConnected / MatMul / transpose --------------------------------------------

def test_fc_golden_and_matmul():
    for tag, args, want, mm in gio.fc_cases():
        say("fc golden", tag)
        np.testing.assert_array_equal(capi.fc_i8(*args), want)
        x, w, _, oo, io, wo, _, _, outP = args
        np.testing.assert_array_equal(capi.matmul_i8(x, w, oo, io, wo, outP), mm)


@pytest.mark.parametrize("shape", [(64, 2048, 1000), (5, 19, 9), (200, 128, 130)])
def test_fc_vs_oracle(shape):
    for b8 in (False, True):
        say("fc", shape, "bias8" if b8 else "bias32")
        c = cases.fc_case(shape[0], *shape, bias_i8=b8)
        want = go.fc_i8(*cases.fc_args(c))
        np.testing.assert_array_equal(capi.fc_i8(*cases.fc_args(c)), want)
        np.testing.assert_array_equal(
            capi.fc_i8(*cases.fc_args(c), precomputed_sums=True), want)
    np.testing.assert_array_equal(
        capi.matmul_i8(c["x"], c["w"], c["out_offset"], c["in_offset"],
                       c["w_offset"], c["outP"]),
        go.matmul_i8(c["x"], c["w"], c["out_offset"], c["in_offset"],
                     c["w_offset"], c["outP"]))


def test_rowsum():
    rng = np.random.default_rng(16)
    for shape in [(1, 1), (5, 100), (64, 1024), (300, 2048 + 37), (7, 3, 3, 64)]:
        a = rng.integers(-128, 128, shape).astype(np.int8)
        want = a.reshape(shape[0], -1).astype(np.int32).sum(1)
        np.testing.assert_array_equal(capi.rowsum_i8(a), want)


def test_transpose2d():
    rng = np.random.default_rng(6)
    for shape in [(1, 1), (3, 200), (64, 64), (100, 65), (1000, 2048)]:
        a = rng.integers(-128, 128, shape).astype(np.int8)
        np.testing.assert_array_equal(capi.transpose2d_i8(a), a.T)


# ---- convolutions ---------------------------------------------------------------------

def test_cwq_conv_golden():
    for tag, args, want in gio.cwq_conv_cases():
        say("cwq_conv golden", tag)
        np.testing.assert_array_equal(capi.cwq_conv2d_i8(*args), want)


def test_cwq_conv_exact_kat():  # reference OperatorTest.cpp:11407-11485
    x = np.arange(1, 13).astype(np.int8).reshape(1, 2, 3, 2)
    filt = np.zeros((4, 2, 1, 1), np.int8)
    filt[:, 0] = 1
    filt[:, 1] = 2
    g = go.conv_geom(1, 2, 3, 2, 4, (2, 1), (1, 1), (0, 0, 0, 0), group=2)
    z, one = np.zeros(4, np.int32), np.ones(4, np.int32)
    out = capi.cwq_conv2d_i8(x, filt, z, g, 0, 0, z, z, z, z, one, z, z, one)
    np.testing.assert_array_equal(
        out.reshape(-1), [15, 15, 18, 18, 21, 21, 24, 24, 27, 27, 30, 30])


CONV_CASES = [
    dict(N=2, H=56, W=56, IC=64, OC=64),                       # ResNet layer shape
    dict(N=1, H=14, W=14, IC=256, OC=256, act=go.ACT_NONE),
    dict(N=2, H=28, W=28, IC=128, OC=512, kernel=(1, 1), pads=(0, 0, 0, 0)),
    dict(N=2, H=56, W=56, IC=256, OC=128, kernel=(1, 1), stride=(2, 2), pads=(0, 0, 0, 0)),
    dict(N=1, H=15, W=15, IC=32, OC=48, stride=(2, 2), pads=(0, 1, 2, 1), symmetric=False),
    dict(N=2, H=9, W=8, IC=32, OC=32, group=2, dilation=(2, 1), kernel=(2, 3),
         in_offset=-9, out_offset=5, act=go.ACT_CLIP),
    dict(N=1, H=12, W=12, IC=16, OC=8, act=go.ACT_LEAKY_RELU, out_offset=10, bias_i8=True),
    dict(N=2, H=32, W=32, IC=3, OC=64, kernel=(7, 7), stride=(2, 2), pads=(3, 3, 3, 3)),
    dict(N=1, H=6, W=7, IC=4, OC=8, in_offset=7),
    dict(N=3, H=5, W=5, IC=6, OC=10, group=2, kernel=(5, 5), pads=(2, 2, 2, 2), symmetric=False),
    # 64 or more channels per group, not a multiple of the 64-byte K step: the
    # tap location advances across tap and filter-row boundaries mid-step
    dict(N=1, H=9, W=9, IC=80, OC=32, kernel=(3, 3), dilation=(2, 2), pads=(2, 2, 2, 2)),
    dict(N=2, H=7, W=6, IC=192, OC=64, group=2, kernel=(2, 3), stride=(1, 2), pads=(1, 1, 0, 1),
         in_offset=11),
    dict(N=1, H=8, W=8, IC=48, OC=16, kernel=(3, 2), pads=(1, 0, 1, 1)),   # fewer than 64
]


@pytest.mark.parametrize("kw", CONV_CASES)
def test_cwq_conv_vs_oracle(kw):
    say("cwq_conv", kw)
    kw = dict(kw)
    kw.setdefault("in_offset", -128)  # post-ReLU activations of the uint8-style schema
    c = cases.cwq_conv_case(31, **kw)
    want = go.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    np.testing.assert_array_equal(capi.cwq_conv2d_i8(*cases.cwq_conv_args(c)), want)
    np.testing.assert_array_equal(
        capi.cwq_conv2d_i8(*cases.cwq_conv_args(c), precomputed_sums=False), want)
    assert want.std() > 1
    # uniform-parameter convolution through its own entry point
    args = (c["x"], c["filt"], c["bias"], c["geom"], c["out_offset"],
            c["in_offset"], int(c["f_offsets"][1]), int(c["b_offsets"][1]),
            (c["bias_pre"][1], c["bias_post"][1], c["bias_scale"][1]),
            (c["out_pre"][1], c["out_post"][1], c["out_scale"][1]),
            c["act"], c["act_args"])
    np.testing.assert_array_equal(capi.conv2d_i8(*args), go.conv2d_i8(*args))


def test_cwq_conv_full_batch_properties():
    """The ResNet layer at its full batch of 32: images 0 and 1 are checked
    against the oracle, the rest through batch independence (an image repeated
    in the batch gives the same output slice)."""
    say("cwq_conv batch 32")
    c = cases.cwq_conv_case(41, 32, 56, 56, 64, 64, in_offset=-128)
    c["x"][2::2] = c["x"][0]
    c["x"][3::2] = c["x"][1]
    got = capi.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    c2 = dict(c, x=c["x"][:2], geom=go.conv_geom(2, 56, 56, 64, 64, (3, 3), (1, 1), (1, 1, 1, 1)))
    want = go.cwq_conv2d_i8(*cases.cwq_conv_args(c2))
    np.testing.assert_array_equal(got[:2], want)
    for i in range(2, 32):
        np.testing.assert_array_equal(got[i], want[i % 2])


# ---- fused-rowwise SLWS ------------------------------------------------------------------

def test_slws_golden():
    for tag, (table, w, idx, lens), want in gio.slws_cases():
        say("slws golden", tag)
        np.testing.assert_array_equal(
            capi.frwq_slws(table, capi.FUSED_U8_F32, w, idx, lens), want)


def test_slws_reference_kats():  # reference OperatorTest.cpp:16941-17040, 17314-17511
    data = np.array([[2.0], [-0.5], [13.0]], np.float32)
    w = np.array([3, 1, 0, 0, 0, 0, 2, -0.5], np.float32)
    idx = np.array([1, 0, 2, 0, 1, 2, 2, 0])
    lens = np.array([3, 0, 3, 2], np.int32)
    want = np.array([[0.5], [0], [0], [25]], np.float32)
    f = capi.fused_rowwise_quantize_host(data, capi.FUSED_U8_F32)
    for idt in (np.int64, np.int32):
        out = capi.frwq_slws(f, capi.FUSED_U8_F32, w, idx.astype(idt), lens)
        assert np.max(np.abs(out - want)) <= 1e-4
    two = np.array([[1.0, 1.2], [2.3, 3.4], [4.5, 5.7]], np.float32)
    idx2 = np.array([2, 0, 1, 2, 0, 0, 0, 0], np.int64)
    len2 = np.array([2, 0, 2, 1, 3], np.int32)
    w2 = np.array([1, -1, 1.5, 0.5, -1.5, 2, -2, -0.5], np.float32)
    sls = np.array([[5.5, 6.9], [0, 0], [6.8, 9.1], [1.0, 1.2], [3.0, 3.6]], np.float32)
    slws = np.array([[3.5, 4.5], [0, 0], [5.7, 7.95], [-1.5, -1.8], [-0.5, -0.6]], np.float32)
    f2 = capi.fused_rowwise_quantize_host(two, capi.FUSED_U8_F32)
    assert np.max(np.abs(capi.frwq_slws(f2, 0, None, idx2, len2) - sls)) <= 0.015
    assert np.max(np.abs(capi.frwq_slws(f2, 0, w2, idx2, len2) - slws)) <= 0.015
    f4 = capi.fused_rowwise_quantize_host(two, capi.FUSED_U4_F16)
    for acc in (False, True):
        o = capi.frwq_slws(f4, capi.FUSED_U4_F16, None, idx2, len2, True, acc)
        assert np.max(np.abs(o.astype(np.float32) - sls)) <= 0.15
        o = capi.frwq_slws(f4, capi.FUSED_U4_F16, w2.astype(np.float16), idx2,
                           len2, True, acc)
        assert np.max(np.abs(o.astype(np.float32) - slws)) <= 0.1


def test_slws_4bit_near_exact_kat():  # reference OperatorTest.cpp:16152-16295
    data = np.array([0, 1, 2, 3, 0, 1, 2, 3, 0, 1, 2, 3, -3, -2, -1, 0,
                     0, -1, -2, -3, 2, 2, 2, 2, 2, 2, 2, 2], np.float32).reshape(7, 4)
    w = np.array([1, 2, 3, 2, 0.5, -0.5, 2], np.float16)
    idx = np.array([0, 1, 2, 4, 3, 5, 6], np.int32)
    offs = np.array([0, 3, 5, 7], np.int32)
    want = np.array([[0, 6, 12, 18], [-1.5, -3, -4.5, -6], [3, 3, 3, 3],
                     [0, 0, 0, 0]], np.float32)
    f = capi.fused_rowwise_quantize_host(data, capi.FUSED_U4_F16)
    for acc in (False, True):
        o = capi.embedding_bag_rowwise_offsets(f, capi.FUSED_U4_F16, w, idx,
                                               offs, False, True, acc)
        assert np.max(np.abs(o.astype(np.float32) - want)) <= 0.005
        # with an end offset and junk behind it
        o = capi.embedding_bag_rowwise_offsets(
            f, capi.FUSED_U4_F16, np.r_[w, np.float16([-42, 42])],
            np.r_[idx, [100, 200]].astype(np.int32),
            np.r_[offs, [7]].astype(np.int32), True, True, acc)
        assert np.max(np.abs(o.astype(np.float32) - want)) <= 0.005


SLWS_SHAPES = [
    # rows, cols, bags, mean length
    (50, 8, 20, 3), (1000, 128, 64, 40), (300, 37, 10, 12), (500, 64, 33, 20),
    (200, 256, 9, 7), (4000, 128, 4096, 40), (999, 32, 100, 90), (64, 16, 5, 200),
    (300, 2, 7, 3),
]


@pytest.mark.parametrize("shape", SLWS_SHAPES)
@pytest.mark.parametrize("idt", [np.int64, np.int32])
def test_slws_u8_f32_bit_exact(shape, idt):
    rows, cols, bags, mean = shape
    say("slws u8/f32", shape, idt.__name__)
    rng = np.random.default_rng(rows + cols)
    table = cases.random_fused_table(rng, rows, cols)
    lengths, idx, w = cases.slws_batch(bags, rows, bags, mean, 1.05, idt)
    lengths[bags // 2] = 0
    total = int(lengths.sum())
    idx, w = idx[:total], w[:total]
    want = go.frwq_slws_f32(table, w, idx, lengths)
    got = capi.frwq_slws(table, capi.FUSED_U8_F32, w, idx, lengths)
    np.testing.assert_array_equal(got, want)
    # 1e-5 relative, the stated bar, holds a fortiori
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=0)
    # unweighted sum == all-ones weights
    ones = np.ones(total, np.float32)
    np.testing.assert_array_equal(
        capi.frwq_slws(table, capi.FUSED_U8_F32, None, idx, lengths),
        go.frwq_slws_f32(table, ones, idx, lengths))


@pytest.mark.parametrize("kind", [capi.FUSED_U8_F16, capi.FUSED_U4_F16, capi.FUSED_U4_F32])
@pytest.mark.parametrize("cols", [64, 16, 130, 6, 128, 256])
def test_slws_other_kinds_bit_exact(kind, cols):
    say("slws kind", kind, "cols", cols)
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
        combos += [(w.astype(np.float16), True, False),
                   (w.astype(np.float16), True, True), (None, True, True)]
    for weights, out16, acc16 in combos:
        want = go.frwq_slws_generic(table, kind, weights, idx, lengths, out16, acc16)
        got = capi.frwq_slws(table, kind, weights, idx, lengths, out16, acc16)
        np.testing.assert_array_equal(got.view(np.uint16 if out16 else np.uint32),
                                      want.view(np.uint16 if out16 else np.uint32))


@pytest.mark.parametrize("kind,cols,pitch", [
    (capi.FUSED_U4_F16, 64, 64), (capi.FUSED_U8_F32, 32, 64), (capi.FUSED_U8_F32, 128, 192),
    (capi.FUSED_U8_F16, 30, 35), (capi.FUSED_U4_F32, 130, 80),
])
def test_slws_padded_rows_bit_exact(kind, cols, pitch):
    """in_line_size above the fused row's own size: rows that far apart."""
    say("slws padded rows kind", kind, "cols", cols, "pitch", pitch)
    rng = np.random.default_rng(kind * 77 + cols)
    rows, bags = 600, 90
    table = cases.random_fused_table(rng, rows, cols, kind)
    lengths, idx, w = cases.slws_batch(cols + 2, rows, bags, 15, 1.1, np.int32)
    total = int(lengths.sum())
    idx, w = idx[:total], w[:total]
    f16 = kind in (capi.FUSED_U8_F16, capi.FUSED_U4_F16)
    combos = [(w, False, False), (None, False, False)]
    if f16:
        combos += [(w.astype(np.float16), True, True)]
    for weights, out16, acc16 in combos:
        want = go.frwq_slws_generic(table, kind, weights, idx, lengths, out16, acc16)
        got = capi.frwq_slws(table, kind, weights, idx, lengths, out16, acc16, row_pitch=pitch)
        np.testing.assert_array_equal(got.view(np.uint16 if out16 else np.uint32),
                                      want.view(np.uint16 if out16 else np.uint32))


def test_slws_fp16_accumulation_rounds_the_product_twice():
    """fp16 accumulation rounds w*(s*q+o) to binary32 and then to binary16, as
    the CPU does; a single rounding differs in the last place about once in
    ten thousand elements (seen with these seeds before the kernel kept the
    two roundings apart)."""
    for kind, cols in ((capi.FUSED_U8_F16, 64), (capi.FUSED_U8_F16, 256)):
        rng = np.random.default_rng(kind * 100 + cols)
        table = cases.random_fused_table(rng, 700, cols, kind)
        lengths, idx, w = cases.slws_batch(cols, 700, 150, 20, 1.1, np.int64)
        total = int(lengths.sum())
        w16 = w[:total].astype(np.float16)
        want = go.frwq_slws_generic(table, kind, w16, idx[:total], lengths, True, True)
        got = capi.frwq_slws(table, kind, w16, idx[:total], lengths, True, True)
        np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))


def test_slws_many_bags_uses_chunk_sums():
    rows, cols, bags = 5000, 64, 20000   # more than one chunk of 8192 bags
    say("slws many bags", bags)
    rng = np.random.default_rng(8)
    table = cases.random_fused_table(rng, rows, cols)
    lengths, idx, w = cases.slws_batch(9, rows, bags, 6, 1.05, np.int64)
    np.testing.assert_array_equal(
        capi.frwq_slws(table, capi.FUSED_U8_F32, w, idx, lengths),
        go.frwq_slws_f32(table, w, idx, lengths))


def test_slws_back_to_back_rezeroes_rows():  # reference OperatorTest.cpp:17242-17312
    rows, cols, bags = 300, 32, 40
    rng = np.random.default_rng(10)
    table = cases.random_fused_table(rng, rows, cols)
    d_table = capi.to_device(table)
    l1, i1, w1 = cases.slws_batch(1, rows, bags, 5, 1.05, np.int64)
    l2 = l1.copy()
    l2[::3] = 0
    i2, w2 = i1[:int(l2.sum())], w1[:int(l2.sum())]
    capi.frwq_slws(table, 0, w1, i1, l1, d_data=d_table)
    got = capi.frwq_slws(table, 0, w2, i2, l2, d_data=d_table)
    np.testing.assert_array_equal(got, go.frwq_slws_f32(table, w2, i2, l2))
    np.testing.assert_array_equal(got[::3], 0)


def test_slws_invalid_lookups_are_skipped():
    rows, cols = 50, 16
    rng = np.random.default_rng(12)
    table = cases.random_fused_table(rng, rows, cols)
    lengths = np.array([3, 2, 4], np.int32)
    idx = np.array([1, 99, 3, -1, 4, 5, 6, 7, 8], np.int64)  # 99 and -1 are out of range
    w = rng.random(9).astype(np.float32)
    got = capi.frwq_slws(table, 0, w, idx, lengths)
    keep = np.array([1, 0, 1, 0, 1, 1, 1, 1, 1], bool)
    want = go.frwq_slws_f32(table, np.where(keep, w, 0).astype(np.float32),
                            np.where(keep, idx, 0), lengths)
    np.testing.assert_array_equal(got, want)
    # lengths that run past the index list: the missing lookups are skipped
    got = capi.frwq_slws(table, 0, w[:7], idx[:7].clip(0, 49), np.array([3, 2, 4], np.int32))
    want = go.frwq_slws_f32(table, np.r_[w[:7], [0, 0]].astype(np.float32),
                            np.r_[idx[:7].clip(0, 49), [0, 0]], lengths)
    np.testing.assert_array_equal(got, want)


def test_slws_full_size_config():
    """The benchmark configuration at full size: 4M x 128 table (544 MB),
    4096 bags Poisson(40), Zipf(1.05) int64 indices. The oracle checks all of
    it (it needs about a second)."""
    rows, cols, bags = 4_000_000, 128, 4096
    say("slws full size")
    rng = np.random.default_rng(2026)
    table = cases.random_fused_table(rng, rows, cols)
    lengths, idx, w = cases.slws_batch(2027, rows, bags, 40, 1.05, np.int64)
    got = capi.frwq_slws(table, capi.FUSED_U8_F32, w, idx, lengths)
    want = go.frwq_slws_f32(table, w, idx, lengths)
    np.testing.assert_array_equal(got, want)
    assert np.unique(idx).size > 20000 and idx.max() > rows // 2


# ---- static memory plan -------------------------------------------------------------------

def test_arena_regions_and_bounds():
    a = capi.Arena(1000, 300, 5000)
    assert a.nbytes >= 6300
    x = np.arange(300, dtype=np.uint8)
    a.upload(capi.REGION_MUTABLE, 0, x)
    np.testing.assert_array_equal(a.download(capi.REGION_MUTABLE, 0, 300, np.uint8), x)
    assert a.ptr(capi.REGION_ACTIVATIONS, 64) % 64 == 0
    with pytest.raises(capi.MI355XError):
        a.upload(capi.REGION_MUTABLE, 200, x)  # runs past the region
    with pytest.raises(capi.MI355XError):
        a.ptr(7, 0)
    # kernels run on arena addresses: quantize from mutable into activations
    f = np.linspace(-3, 3, 64).astype(np.float32)
    a.upload(capi.REGION_MUTABLE, 0, f)
    capi.launch_quantize_i8(a.ptr(capi.REGION_ACTIVATIONS, 128),
                            a.ptr(capi.REGION_MUTABLE, 0), 64, 0.05, 1)
    np.testing.assert_array_equal(
        a.download(capi.REGION_ACTIVATIONS, 128, 64, np.int8),
        go.quantize_i8(f, 0.05, 1))
    a.destroy()


@pytest.mark.gpu
def test_rescale_both_multiplier_paths():
    """Scales below 2^23 take the 24-bit multiplier, others the 32-bit one:
    the results must not depend on which."""
    q = np.arange(-128, 128).astype(np.int8).repeat(20)
    for sc in (1, 255, (1 << 23) - 1, 1 << 23, (1 << 23) + 12345, -(1 << 23) + 1, -(1 << 23),
               (1 << 30) + 7, -5):
        for pre, post, io, oo in ((0, 0, 0, 0), (2, 15, -7, 9), (0, 31, 127, -128), (7, 3, -128, 127)):
            np.testing.assert_array_equal(capi.rescale_i8(q, oo, io, pre, post, sc),
                                          go.rescale_i8(q, oo, io, pre, post, sc),
                                          err_msg=f"scale {sc} pre {pre} post {post}")


@pytest.mark.gpu
@pytest.mark.parametrize("tile", list(range(6)))
@pytest.mark.parametrize("K", [64, 128, 192])
def test_short_k_loops_on_every_tile(tile, K):
    """K loops of one, two and three steps (shorter than, or as long as, the
    ring of load stages), symmetric weights with precomputed row sums: the
    128x128 tile has a variant of its own for these."""
    c = cases.rwq_fc_case(90 + tile + K, 390, K, 260, symmetric=True)
    cc = cases.cwq_conv_case(95 + tile + K, 2, 14, 14, K, 160, kernel=(1, 1), pads=(0, 0, 0, 0),
                             in_offset=-128)
    want_fc = go.rwq_fc_i8(*cases.rwq_fc_args(c))
    want_cv = go.cwq_conv2d_i8(*cases.cwq_conv_args(cc))
    capi.check(capi.lib().mi355x_gemm_tile_override(tile))
    try:
        got_fc = capi.rwq_fc_i8(*cases.rwq_fc_args(c))
        got_cv = capi.cwq_conv2d_i8(*cases.cwq_conv_args(cc))
    finally:
        capi.check(capi.lib().mi355x_gemm_tile_override(-1))
    np.testing.assert_array_equal(got_fc, want_fc)
    np.testing.assert_array_equal(got_cv, want_cv)


@pytest.mark.gpu
@pytest.mark.parametrize("tile", list(range(6)))
def test_every_gemm_tile_gives_the_same_result(tile):
    """Results do not depend on the workgroup tile."""
    c = cases.rwq_fc_case(60 + tile, 700, 192, 330, symmetric=False)
    cc = cases.cwq_conv_case(70 + tile, 3, 20, 20, 32, 96, in_offset=-4, symmetric=False)
    cg = cases.cwq_conv_case(80 + tile, 2, 12, 12, 64, 64, group=2, in_offset=3)
    want_fc = go.rwq_fc_i8(*cases.rwq_fc_args(c))
    want_cv = go.cwq_conv2d_i8(*cases.cwq_conv_args(cc))
    want_cg = go.cwq_conv2d_i8(*cases.cwq_conv_args(cg))
    capi.check(capi.lib().mi355x_gemm_tile_override(tile))
    try:
        got_fc = capi.rwq_fc_i8(*cases.rwq_fc_args(c))
        got_cv = capi.cwq_conv2d_i8(*cases.cwq_conv_args(cc))
        got_cg = capi.cwq_conv2d_i8(*cases.cwq_conv_args(cg))
    finally:
        capi.check(capi.lib().mi355x_gemm_tile_override(-1))
    np.testing.assert_array_equal(got_fc, want_fc)
    np.testing.assert_array_equal(got_cv, want_cv)
    np.testing.assert_array_equal(got_cg, want_cg)


@pytest.mark.gpu
def test_pinned_host_arrays_round_trip():
    a = capi.pinned_copy(np.arange(100000, dtype=np.float32).reshape(100, 1000))
    d = capi.to_device(a)
    b = capi.pinned_empty(a.shape, a.dtype)
    capi.check(capi.lib().mi355x_memcpy_d2h(capi._vp(b), capi._vp(d), capi._sz(a.nbytes), capi._vp(None)))
    capi.sync()
    np.testing.assert_array_equal(a, b)
    del a, b
    import gc
    gc.collect()


@pytest.mark.gpu
def test_embedding_bag_with_senseless_offsets_stays_in_bounds():
    """Negative, decreasing and oversized start offsets give short or empty
    bags; valid bags next to them are unaffected."""
    rng = np.random.default_rng(77)
    rows, cols = 500, 64
    table = cases.random_fused_table(rng, rows, cols)
    idx = rng.integers(0, rows, 200).astype(np.int32)
    w = rng.random(200).astype(np.float32)
    offs = np.array([0, 10, -50, 30, 25, 40, 100000, 60, 200], np.int32)
    got = capi.embedding_bag_rowwise_offsets(table, capi.FUSED_U8_F32, w, idx, offs, True)
    # bag 0 = [0,10) and bag 7 = [60,200) are well formed
    good = go.embedding_bag_byte_rowwise_offsets_f32(table, w, idx, np.array([0, 10], np.int32), True)
    np.testing.assert_array_equal(got[0], good[0])
    good7 = go.embedding_bag_byte_rowwise_offsets_f32(table, w, idx, np.array([60, 200], np.int32), True)
    np.testing.assert_array_equal(got[7], good7[0])
    assert np.all(np.isfinite(got))
    # [40, 100000) is cut at the end of the index list; [100000, 60) is empty
    cut = go.embedding_bag_byte_rowwise_offsets_f32(table, w, idx, np.array([40, 200], np.int32), True)
    np.testing.assert_array_equal(got[5], cut[0])
    assert not got[6].any()

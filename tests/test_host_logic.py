"""CPU-side checks of the product library: it loads, exports every symbol the
header declares, reports errors the documented way without a GPU, and its
host-side parameter math equals the oracle's. No kernel is launched here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from glow_amd import capi
from oracle import glow_oracle as go

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_loads_and_exports_every_declared_symbol():
    lib = capi.lib()
    header = open(os.path.join(ROOT, "include", "glow_mi355x.h")).read()
    declared = set(re.findall(r"\b(mi355x_[a-z0-9_]+)\s*\(", header))
    assert declared == set(capi.EXPORTS), declared ^ set(capi.EXPORTS)
    for name in declared:
        assert hasattr(lib, name), name


def test_product_does_not_link_the_oracle():
    import subprocess
    out = subprocess.run(["ldd", capi.LIB_PATH], capture_output=True, text=True).stdout
    assert "oracle" not in out
    src = os.path.join(ROOT, "glow_amd")
    for dirpath, _, files in os.walk(src):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "glow_oracle" not in text and "from oracle" not in text, f


def test_errors_without_gpu_are_reported_not_swallowed():
    if capi.num_devices() > 0:
        pytest.skip("a GPU is present")
    with pytest.raises(capi.MI355XError) as e:
        capi.init(0)
    assert e.value.code == -6  # RUNTIME_DEVICE_NOT_FOUND
    assert "not found" in str(e.value) or "hipGetDeviceCount" in str(e.value)


def test_argument_validation_needs_no_gpu():
    lib = capi.lib()
    # shift outside [0, 31]
    rc = lib.mi355x_rescale_i8(C.c_void_p(16), C.c_void_p(16), C.c_size_t(4),
                               0, 0, 40, 0, 1, None)
    assert rc == -1 and b"shift" in lib.mi355x_last_error()
    # rows too close together for out_line_size columns plus scale and offset
    rc = lib.mi355x_frwq_slws(C.c_void_p(16), 0, C.c_void_p(16), C.c_size_t(10),
                              0, None, 0, C.c_void_p(16), 1, C.c_size_t(4),
                              C.c_void_p(16), C.c_size_t(2), C.c_size_t(136),
                              C.c_size_t(130), 0, None)
    assert rc == -1 and b"in_line_size" in lib.mi355x_last_error()
    # an odd number of 4-bit columns
    rc = lib.mi355x_frwq_slws(C.c_void_p(16), 1, C.c_void_p(16), C.c_size_t(10),
                              2, None, 0, C.c_void_p(16), 1, C.c_size_t(4),
                              C.c_void_p(16), C.c_size_t(2), C.c_size_t(36),
                              C.c_size_t(63), 0, None)
    assert rc == -1 and b"out_line_size" in lib.mi355x_last_error()
    # unknown schema
    s, o = C.c_float(), C.c_int32()
    rc = lib.mi355x_choose_quantization_params(C.c_float(0), C.c_float(1), 9, 8,
                                               C.byref(s), C.byref(o))
    assert rc == -1
    # empty tensors are a no-op, not an error
    assert lib.mi355x_quantize_i8(None, None, C.c_size_t(0), C.c_float(1), 0, None) == 0


def test_quantize_scale_offset_equals_oracle():
    rng = np.random.default_rng(0)
    scales = np.concatenate([
        np.exp(rng.uniform(np.log(1e-8), np.log(300.0), 4000)),
        2.0 ** np.arange(-24, 9), [1.0, 0.5, 255.0, 256.0, 0.4999999, 3.0]
    ]).astype(np.float32)
    for s in scales:
        assert capi.quantize_scale_offset_32to8(float(s), 7) == \
            go.quantize_scale_offset_32to8(float(s), 7), s


def test_choose_quantization_params_equals_oracle():
    rng = np.random.default_rng(1)
    for _ in range(3000):
        a, b = np.sort(rng.normal(0, 2, 2) * 10.0 ** rng.integers(-3, 3)).astype(np.float32)
        if rng.random() < 0.1:
            b = a
        if rng.random() < 0.1:
            a = -b
            a, b = min(a, b), max(a, b)
        for schema in range(4):
            for qty in (8, 16, 32, 108):
                if qty == 108 and schema != 0:
                    continue  # symmetric schemas need a signed range
                got = capi.choose_quantization_params(float(a), float(b), schema, qty)
                want = go.choose_qparams(float(a), float(b), schema, qty)
                assert got == want, (a, b, schema, qty)


@pytest.mark.parametrize("kind", [0, 1, 2, 3])
def test_fused_rowwise_quantize_equals_oracle(kind):
    rng = np.random.default_rng(2)
    x = (rng.normal(0, 1, (40, 24)) * 10.0 ** rng.integers(-3, 3, (40, 1))).astype(np.float32)
    x[5] = 0.75
    x[6] = 0.0
    x[7, :] = np.float32(6.1e-5)  # fp16 subnormal range for the offset
    assert capi.fused_row_bytes(24, kind) == go.fused_row_bytes(24, kind)
    np.testing.assert_array_equal(capi.fused_rowwise_quantize_host(x, kind),
                                  go.fused_rowwise_quantize(x, kind))


def test_rowwise_quantize_equals_oracle():
    rng = np.random.default_rng(3)
    w = rng.normal(0, 0.2, (17, 33)).astype(np.float32)
    for schema in range(4):
        for got, want in zip(capi.rowwise_quantize_i8_host(w, schema),
                             go.rowwise_quantize_i8(w, schema)):
            np.testing.assert_array_equal(got, want)


def test_specialize_bias_weights_qparams_equals_oracle():
    rng = np.random.default_rng(12)
    for _ in range(200):
        bs = float(np.float32(10 ** rng.uniform(-8, 0)))
        ws = float(np.float32(10 ** rng.uniform(-4, 0)))
        ins = float(np.float32(10 ** rng.uniform(-3, 0)))
        bo = int(rng.integers(-5, 6))
        for i32 in (True, False):
            for zero in (False, True):
                assert capi.specialize_bias_weights_qparams(bs, bo, ins, ws, i32, zero) == \
                    go.specialize_bias_weights_qparams(bs, bo, ins, ws, i32, zero)


def test_channelwise_conv_constants_equal_the_oracle():
    """mi355x_channelwise_quantize_conv_host and mi355x_specialize_bias_qparams
    against the oracle's restatement of Graph.cpp:3576-3700 / Base.cpp:567-592."""
    from glow_amd import capi
    rng = np.random.default_rng(21)
    for trial in range(30):
        oc, per = int(rng.integers(1, 40)), int(rng.integers(1, 200))
        filt = (rng.standard_normal((oc, per)) * rng.uniform(1e-3, 5.0, (oc, 1))).astype(np.float32)
        bias = (rng.standard_normal(oc) * 10.0 ** rng.uniform(-3, 7, oc)).astype(np.float32)
        bias[rng.random(oc) < 0.2] = 0.0
        in_scale = float(np.float32(10.0 ** rng.uniform(-3, 0)))
        for schema in (go.SYMMETRIC, go.ASYMMETRIC, go.SYMMETRIC_WITH_UNSIGNED):
            got = capi.channelwise_quantize_conv_host(filt, bias, in_scale, schema)
            want = go.channelwise_quantize_conv(filt, bias, in_scale, schema)
            for g, w in zip(got, want):
                np.testing.assert_array_equal(g, w)
    for _ in range(2000):
        a = [float(np.float32(10.0 ** rng.uniform(-8, 2))) for _ in range(3)]
        off = int(rng.integers(-100, 100))
        for i32 in (True, False):
            for zero in (True, False):
                assert capi.specialize_bias_qparams(a[0], off, a[1], a[2], i32, zero) == \
                    go.specialize_bias_qparams(a[0], off, a[1], a[2], i32, zero)


def test_requant_hint_is_refused_when_24_bits_cannot_be_guaranteed():
    """Worst-case accumulators of a long contraction without a pre-shift do not
    fit 24 bits: no hint. With enough pre-shift they do."""
    N = 8
    one, zero = np.ones(N, np.int32), np.zeros(N, np.int32)
    sc = np.full(N, 300, np.int32)
    post = np.full(N, 15, np.int32)
    args = lambda K, pre: (K, -128, 0, None, None, 0, None, None, None, np.full(N, pre, np.int32), post, sc)
    assert capi.gemm_requant_hint_host(*args(64, 0)) == 3
    assert capi.gemm_requant_hint_host(*args(4096, 0)) == 0
    assert capi.gemm_requant_hint_host(*args(4096, 5)) == 1
    # a scale of 24 bits or more, or an offset that does not fit below the post-shift
    big = sc.copy()
    big[3] = 1 << 23
    assert capi.gemm_requant_hint_host(64, 0, 0, None, None, 0, None, None, None, zero, post, big) == 0
    assert capi.gemm_requant_hint_host(64, 0, 100, None, None, 0, None, None, None, zero,
                                       np.full(N, 25, np.int32), sc) == 0
    # a huge bias moves the bound too
    bias = np.full(N, 2 ** 30, np.int32)
    assert capi.gemm_requant_hint_host(64, 0, 0, None, bias, 0, zero, zero, one, zero, post, sc) == 0
    with pytest.raises(capi.MI355XError):
        capi.check(capi.lib().mi355x_gemm_requant_hint(2))


def test_slws_bag_offsets_host():
    """Exclusive prefix sums of the clamped lengths; sums past int32 are refused."""
    rng = np.random.default_rng(3)
    lengths = rng.integers(-3, 50, 5000).astype(np.int32)
    offs = capi.slws_bag_offsets_host(lengths)
    want = np.r_[0, np.cumsum(np.maximum(lengths, 0))]
    np.testing.assert_array_equal(offs, want)
    assert offs.dtype == np.int32 and offs.size == lengths.size + 1
    np.testing.assert_array_equal(capi.slws_bag_offsets_host(np.zeros(0, np.int32)), [0])
    big = np.full(3, 2**30, np.int32)
    with pytest.raises(capi.MI355XError):
        capi.slws_bag_offsets_host(big)
    np.testing.assert_array_equal(capi.slws_bag_offsets_host(big[:1]), [0, 2**30])

"""The CPU oracle reproduces every committed golden vector (outputs of the
reference's compiled libjit kernels) bit for bit. CPU only; runs where the
reference tree is absent."""
import numpy as np

from oracle import glow_oracle as go
from tests import golden_io as gio


def test_elementwise_golden():
    d = gio.elementwise()
    i = 0
    while f"quant{i}_params" in d:
        s, o = d[f"quant{i}_params"]
        np.testing.assert_array_equal(go.quantize_i8(d["x"], float(s), int(o)),
                                      d[f"quant{i}_out"])
        np.testing.assert_array_equal(go.dequantize_i8(d["q"], float(s), int(o)),
                                      d[f"dequant{i}_out"])
        i += 1
    assert i == 3
    i = 0
    while f"rescale{i}_params" in d:
        oo, io, pre, post, sc = (int(v) for v in d[f"rescale{i}_params"])
        np.testing.assert_array_equal(
            go.rescale_i8(d["q"], oo, io, pre, post, sc), d[f"rescale{i}_out"])
        i += 1
    assert i == 4


def test_rwq_fc_golden():
    n = 0
    for _, args, want in gio.rwq_fc_cases():
        np.testing.assert_array_equal(go.rwq_fc_i8(*args), want)
        n += 1
    assert n == 3


def test_fc_golden():
    n = 0
    for _, args, want, mm in gio.fc_cases():
        np.testing.assert_array_equal(go.fc_i8(*args), want)
        x, w, _, oo, io, wo, _, _, outP = args
        np.testing.assert_array_equal(go.matmul_i8(x, w, oo, io, wo, outP), mm)
        n += 1
    assert n == 2


def test_cwq_conv_golden():
    n = 0
    for _, args, want in gio.cwq_conv_cases():
        np.testing.assert_array_equal(go.cwq_conv2d_i8(*args), want)
        n += 1
    assert n == 5


def test_slws_golden():
    n = 0
    for _, (table, w, idx, lens), want in gio.slws_cases():
        np.testing.assert_array_equal(go.frwq_slws_f32(table, w, idx, lens), want)
        n += 1
    assert n == 2


def test_glue_golden():
    ops, logits, softmax = gio.glue()
    for name, call, want in ops:
        np.testing.assert_array_equal(call(go), want, err_msg=name)
    # libm's expf may differ by an ulp between hosts; the sums are sequential
    np.testing.assert_allclose(go.softmax_f32(logits), softmax, rtol=2e-6, atol=1e-30)


def test_wide_elementwise_golden():
    """int16 / int32 Quantize, Dequantize, RescaleQuantized as the reference's
    compiled libjit computes them (x reaches past the int16 range, so the int16
    clip and the unclipped int32 form both show)."""
    d = gio.wide()
    for bits in (16, 32):
        q = d[f"q{bits}"]
        for i in range(3):
            s, o = d[f"quant{bits}_{i}_params"]
            np.testing.assert_array_equal(go.quantize_wide(d["x"], float(s), int(o), bits),
                                          d[f"quant{bits}_{i}_out"])
            np.testing.assert_array_equal(go.dequantize_wide(q, float(s), int(o)),
                                          d[f"dequant{bits}_{i}_out"])
        for i in range(4):
            oo, io, pre, post, sc = (int(v) for v in d[f"rescale{bits}_{i}_params"])
            np.testing.assert_array_equal(go.rescale_wide(q, oo, io, pre, post, sc),
                                          d[f"rescale{bits}_{i}_out"])
    assert d["quant16_0_out"].min() == -32768 and d["quant16_0_out"].max() == 32767
    assert np.abs(d["quant32_0_out"].astype(np.int64)).max() > 2 ** 16


def test_transpose_golden():
    d = gio.wide()
    i = 0
    while f"transpose{i}_in" in d:
        x, sh = d[f"transpose{i}_in"], [int(v) for v in d[f"transpose{i}_shuffle"]]
        got = go.transpose(x, sh)
        np.testing.assert_array_equal(got, d[f"transpose{i}_out"].reshape(got.shape))
        np.testing.assert_array_equal(got, x.transpose(sh))      # the textbook routine
        i += 1
    assert i == 6


def test_cwq_conv3d_golden():
    n = 0
    for _, args, want in gio.conv3d_cases():
        np.testing.assert_array_equal(go.cwq_conv3d_i8(*args), want)
        n += 1
    assert n == 4


def test_element_ops_golden():
    """Clip, LeakyRelu, Max(x, Splat) and BatchedAdd against what the compiled
    reference produced (tests/golden/element_ops.npz)."""
    n = 0
    for name, fn, args, want in gio.element_ops():
        np.testing.assert_array_equal(getattr(go, fn)(*args), want, err_msg=name)
        n += 1
    assert n >= 19

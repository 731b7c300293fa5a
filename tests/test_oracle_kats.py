"""Pins the CPU oracle against the known answers the reference's own unit
tests hold (tests/unittests/QuantizationTest.cpp, OperatorTest.cpp) and
against what the mathematics fixes. CPU only."""
import numpy as np
import pytest

from oracle import glow_oracle as go


# ---- quantizeScaleOffset32To8 ------------------------------------------------

# QuantizationTest.cpp:223-247
SCALES = [
    0.0000001596, 0.00000025, 0.000000995, 0.0000035, 0.00000952,
    0.00000113, 0.000721, 0.0000721, 0.0000172, 0.0000951,
    0.0000721, 0.0000341, 0.0000222, 0.0000172, 0.000752,
    0.000371, 0.000321, 0.000223, 0.000112, 0.00852,
    0.00671, 0.00592, 0.00200, 0.00107, 0.0931,
    0.0721, 0.031, 0.014, 0.0132, 0.712,
    0.613, 0.412, 0.223, 0.134, 1.0,
    1.13, 1.612, 1.523, 2.0]


def _c_round(x):
    """C round(): half away from zero."""
    return int(np.sign(x) * np.floor(abs(x) + 0.5))


@pytest.mark.parametrize("scale", SCALES)
def test_quant_scale_offset_within_one(scale):
    s32 = np.float32(scale)
    pre, post, sc, off = go.quantize_scale_offset_32to8(float(s32), 0)
    assert off == 0
    for inp in range(-128, 127):
        # `input / scale` is an int8 promoted to float divided by a float
        sum32 = _c_round(float(np.float32(inp) / s32))
        got = go.scale_i32(sum32, pre, post, sc, 0)
        assert abs(got - inp) <= 1, (scale, inp, got, (pre, post, sc))


# QuantizationTest.cpp:249-275
@pytest.mark.parametrize("exp", range(-10, 2))
def test_quant_scale_offset_power_of_two(exp):
    scale = 2.0 ** exp
    pre, post, sc, off = go.quantize_scale_offset_32to8(scale, 7)
    assert pre == 0 and off == 7
    if exp > 0:
        assert (post, sc) == (0, int(scale))
    else:
        assert (post, sc) == (-exp, 1)
    for inp in range(-128, 127):
        sum32 = _c_round(inp / scale)
        assert abs(go.scale_i32(sum32, pre, post, sc, 0) - inp) <= 1


def test_quant_scale_offset_hand_derived():
    # 0.01: doubles 15 times -> 327.68 (>=256 stops the first loop at post 15),
    # 327.68 >= 255 so no pre-shift; round -> 328.
    assert go.quantize_scale_offset_32to8(0.01, 0) == (0, 15, 328, 0)
    # 0.0005: 15 doublings -> 16.384; pre-shift loop doubles while < 255 and
    # pre < 15 // 2 = 7: 32.768, 65.536, 131.07, 262.14 -> pre 4, scale 262.
    assert go.quantize_scale_offset_32to8(0.0005, 3) == (4, 15, 262, 3)
    # 3.0 (not a power of two): post runs to 15 while scale < 256:
    # 3*2^7 = 384 after 7 doublings -> post 7; 384 >= 255 -> pre 0.
    assert go.quantize_scale_offset_32to8(3.0, 0) == (0, 7, 384, 0)
    # a ratio of exactly 1.0 is the identity transform
    assert go.quantize_scale_offset_32to8(1.0, 0) == (0, 0, 1, 0)
    # very small scale: keeps doubling until >= 0.5, beyond post 15:
    # 1.5*2^-20 needs 19 doublings to reach 0.75; then pre < 19 // 2 = 9 allows
    # nine more doublings (0.75 * 512 = 384; every step was still < 255).
    assert go.quantize_scale_offset_32to8(2.0 ** -20 * 1.5, 0) == (9, 19, 384, 0)


def test_scale_i32_matches_python_big_ints():
    rng = np.random.default_rng(1)
    for _ in range(3000):
        x = int(rng.integers(-2 ** 31, 2 ** 31))
        pre = int(rng.integers(0, 12))
        post = int(rng.integers(0, 31))
        sc = int(rng.integers(-70000, 70000))
        off = int(rng.integers(-200, 200))
        rtn = (1 << (post - 1)) if post > 0 else 0
        m = ((x >> pre) * sc + rtn) & 0xFFFFFFFF
        if m >= 2 ** 31:
            m -= 2 ** 32
        want = ((m >> post) + off + 2 ** 31) % 2 ** 32 - 2 ** 31
        assert go.scale_i32(x, pre, post, sc, off) == want


def test_clip_and_activation():
    assert [go.clip_i8(v) for v in (-1000, -129, -128, 0, 127, 128, 99999)] == \
        [-128, -128, -128, 0, 127, 127, 127]
    # libjit_defs.h:206-233
    assert go.activation_i32(-7, -3, go.ACT_NONE) == -7
    assert go.activation_i32(-7, -3, go.ACT_RELU) == -3
    assert go.activation_i32(5, -3, go.ACT_RELU) == 5
    assert go.activation_i32(50, 0, go.ACT_CLIP, (-10, 20)) == 20
    assert go.activation_i32(-50, 0, go.ACT_CLIP, (-10, 20)) == -10
    # leaky relu with alpha 0.25 = {pre 0, post 2, scale 1}: x<off ->
    # ((x-off)+2)>>2 + off
    p = go.quantize_scale_offset_32to8(0.25, 0)
    assert p[:3] == (0, 2, 1)
    assert go.activation_i32(-37, 3, go.ACT_LEAKY_RELU, p[:3]) == ((-40 + 2) >> 2) + 3
    assert go.activation_i32(9, 3, go.ACT_LEAKY_RELU, p[:3]) == 9


# ---- chooseQuantizationParams -------------------------------------------------

def test_choose_qparams_asymmetric_int8():  # QuantizationTest.cpp:1751-1811
    s, o = go.choose_qparams(0.0, 6.0, go.ASYMMETRIC)
    assert o == -128 and abs(s - 6.0 / 255) < 1e-3
    s, o = go.choose_qparams(-3.0, 3.0, go.ASYMMETRIC)
    assert o == 0 and abs(s - 6.0 / 255) < 1e-3
    s, o = go.choose_qparams(-2.0, 5.0, go.ASYMMETRIC)
    assert o == int(2.0 * 255 / 7.0 - 128) and abs(s - 7.0 / 255) < 1e-3
    s, o = go.choose_qparams(2.0, 5.0, go.ASYMMETRIC)
    assert o == -128 and abs(s - 5.0 / 255) < 1e-3
    s, o = go.choose_qparams(-8.0, -2.0, go.ASYMMETRIC)
    assert o == 127 and abs(s - 8.0 / 255) < 1e-3


def test_choose_qparams_symmetric_int8():  # QuantizationTest.cpp:1815-1855
    for (mn, mx), want in [((0.0, 6.0), 12.0), ((-3.0, 3.0), 6.0),
                           ((-2.0, 5.0), 10.0), ((2.0, 5.0), 10.0),
                           ((-8.0, -2.0), 16.0)]:
        s, o = go.choose_qparams(mn, mx, go.SYMMETRIC)
        assert o == 0 and abs(s - want / 255) < 1e-3


def test_choose_qparams_symmetric_with_uint8():  # QuantizationTest.cpp:2069-2116
    cases = [((0.0, 6.0), -128, 6.0 / 255), ((-3.0, 3.0), 0, 6.0 / 255),
             ((-2.0, 5.0), 0, 10.0 / 255), ((0.0, 0.0), 0, 0.1),
             ((2.0, 5.0), -128, 5.0 / 255), ((-8.0, -2.0), 0, 16.0 / 255)]
    for (mn, mx), off, sc in cases:
        s, o = go.choose_qparams(mn, mx, go.SYMMETRIC_WITH_UNSIGNED)
        assert o == off and abs(s - sc) < 1e-3


def test_choose_qparams_closed_forms():
    # exact double arithmetic of Base.cpp:512-549 redone with Python floats
    rng = np.random.default_rng(5)
    for _ in range(500):
        a, b = np.sort(rng.normal(0, 3, 2)).astype(np.float32)
        mn, mx = min(float(a), 0.0), max(float(b), 0.0)
        s, o = go.choose_qparams(float(a), float(b), go.ASYMMETRIC)
        scale = (mx - mn) / 255.0
        if scale == 0:
            scale = 0.1
        assert s == np.float32(scale)
        e_min = 128 + abs(mn / scale)
        e_max = 127 + abs(mx / scale)
        zp = (-128 - mn / scale) if e_min < e_max else (127 - mx / scale)
        if abs(np.float32(mx) + np.float32(mn)) <= np.finfo(np.float32).eps:
            zp = 0
        assert o == min(127, max(-128, _c_round(zp)))
    # Int32QTy uses an int30 range [-2^29, 2^29-1] (Base.cpp:361-403)
    s, o = go.choose_qparams(-1.0, 1.0, go.SYMMETRIC, 32)
    assert o == 0
    assert abs(s - 2.0 / (2 ** 30 - 1)) / s < 1e-6
    # power-of-two schema rounds the scale up to a power of two
    s, o = go.choose_qparams(-1.0, 1.0, go.SYMMETRIC_POW2)
    assert o == 0 and s == 2.0 ** -6


def test_specialize_bias_qparams():  # Base.cpp:594-629; OperatorTest.cpp:11143-11332
    # bias scale below in*w: forced to the product, weights scale untouched
    bs, bo, ws = go.specialize_bias_weights_qparams(1e-6, 5, 0.05, 0.01)
    assert bo == 0 and ws == np.float32(0.01)
    assert bs == np.float32(0.05) * np.float32(0.01)
    # bias scale above in*w with int32 bias: weights scale is changed so that
    # the product equals the bias scale exactly
    bs, bo, ws = go.specialize_bias_weights_qparams(0.5, 0, 0.05, 0.01)
    assert bs == np.float32(0.05) * np.float32(ws)
    assert abs(ws - 10.0) < 1e-4


# ---- fp16 -----------------------------------------------------------------------

def test_fp16_conversion_matches_numpy():
    rng = np.random.default_rng(2)
    xs = np.concatenate([
        rng.normal(0, 1, 4000), rng.normal(0, 1e-5, 2000),
        rng.normal(0, 3e4, 2000), rng.uniform(-7e-8, 7e-8, 2000),
        [0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24,
         2.0 ** -25, 2.0 ** -25 * 1.0001, 2.0 ** -14, 6.1e-5, np.inf, -np.inf],
    ]).astype(np.float32)
    want = xs.astype(np.float16).view(np.uint16)
    got = np.array([go.f32_to_f16_bits(float(x)) for x in xs], np.uint16)
    np.testing.assert_array_equal(got, want)
    # every finite half converts back exactly
    allh = np.arange(0, 65536, dtype=np.uint32).astype(np.uint16)
    f = allh.view(np.float16).astype(np.float32)
    ok = np.isfinite(f)
    back = np.array([go.f16_bits_to_f32(int(h)) for h in allh[ok]], np.float32)
    np.testing.assert_array_equal(back, f[ok])
    # ties: exactly halfway between two halves goes to the even one
    h = np.float32(1.0 + 2.0 ** -11)  # between 1.0 and 1.0+2^-10
    assert go.f32_to_f16_bits(float(h)) == 0x3C00
    h = np.float32(1.0 + 3 * 2.0 ** -11)
    assert go.f32_to_f16_bits(float(h)) == 0x3C02


# ---- elementwise ------------------------------------------------------------------

def test_quantize_round_half_even_and_clip():
    # x/scale + offset landing exactly on .5 goes to the even integer
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, 3.49, 1000.0, -1000.0], np.float32)
    q = go.quantize_i8(x, 1.0, 0)
    np.testing.assert_array_equal(q, [0, 2, 2, 0, -2, 3, 127, -128])
    q = go.quantize_i8(np.array([5.25], np.float32), 0.25, 4)  # 21 + 4
    assert q[0] == 25


def test_quantize_rescale_dequantize_chain():  # OperatorTest.cpp:19246-19275
    q = go.quantize_i8(np.array([21.0], np.float32), 0.25, 4)
    pre, post, sc, _ = go.quantize_scale_offset_32to8(
        float(np.float32(0.25) / np.float32(0.5)), 4)
    r = go.rescale_i8(q, 11, 4, pre, post, sc)
    d = go.dequantize_i8(r, 0.5, 11)
    assert abs(d[0] - 21.0) < 1e-3


def test_rescale_node_chain():  # OperatorTest.cpp:8174-8204
    q = go.quantize_i8(np.full(16, 40.0, np.float32), 0.7, 5)
    chain = [((0.7, 5), (0.3, -4)), ((0.3, -4), (0.4, -4))]
    for (ss, so), (ds, do) in chain:
        pre, post, sc, _ = go.quantize_scale_offset_32to8(
            float(np.float32(ss) / np.float32(ds)), so)
        q = go.rescale_i8(q, do, so, pre, post, sc)
    d = go.dequantize_i8(q, 0.4, -4)
    assert np.all(np.abs(d - 40.0) <= 1.0)


def test_dequantize_closed_form():
    q = np.arange(-128, 128).astype(np.int8)
    d = go.dequantize_i8(q, 0.37, -11)
    want = np.float32(0.37) * (q.astype(np.int32) + 11).astype(np.float32)
    np.testing.assert_array_equal(d, want)


# ---- FC / conv brute force ----------------------------------------------------------

def _req(acc, pre, post, sc, off):
    """Vectorised libjit_scale on int64 -> wraps to int32."""
    def wrap(v):
        return ((v + 2 ** 31) % 2 ** 32) - 2 ** 31
    acc = np.asarray(acc, np.int64)
    pre = np.asarray(pre, np.int64)
    post = np.asarray(post, np.int64)
    rtn = np.where(post > 0, 1 << np.maximum(post - 1, 0), 0)
    m = wrap((acc >> pre) * np.asarray(sc, np.int64) + rtn)
    return wrap((m >> post) + off)


def test_rwq_fc_brute_force():
    rng = np.random.default_rng(3)
    M, K, N = 7, 37, 11
    x = rng.integers(-128, 128, (M, K)).astype(np.int8)
    w = rng.integers(-128, 128, (N, K)).astype(np.int8)
    bias = rng.integers(-1000, 1000, N).astype(np.int32)
    woff = rng.integers(-5, 6, N).astype(np.int32)
    in_off, out_off, b_off = -7, 3, 2
    bp = np.array([go.quantize_scale_offset_32to8(float(s), b_off)[:3]
                   for s in rng.uniform(0.2, 3.0, N)], np.int32)
    op = np.array([go.quantize_scale_offset_32to8(float(s), 0)[:3]
                   for s in rng.uniform(0.0005, 0.01, N)], np.int32)
    got = go.rwq_fc_i8(x, w, bias, woff, bp[:, 0], bp[:, 1], bp[:, 2],
                       op[:, 0], op[:, 1], op[:, 2], out_off, in_off, b_off)
    acc = (x.astype(np.int64) - in_off) @ (w.astype(np.int64) - woff[:, None]).T
    acc = acc + _req(bias.astype(np.int64) - b_off, bp[:, 0], bp[:, 1], bp[:, 2], 0)
    want = np.clip(_req(acc, op[:, 0], op[:, 1], op[:, 2], out_off), -128, 127)
    np.testing.assert_array_equal(got, want.astype(np.int8))


def test_fc_and_matmul_brute_force():
    rng = np.random.default_rng(4)
    M, K, N = 5, 19, 9
    x = rng.integers(-128, 128, (M, K)).astype(np.int8)
    w = rng.integers(-128, 128, (K, N)).astype(np.int8)
    bias8 = rng.integers(-128, 128, N).astype(np.int8)
    bP = go.quantize_scale_offset_32to8(1.7, 0)[:3]
    oP = go.quantize_scale_offset_32to8(0.003, 0)[:3]
    got = go.fc_i8(x, w, bias8, -2, 4, -3, 1, bP, oP)
    acc = (x.astype(np.int64) - 4) @ (w.astype(np.int64) + 3)
    acc = acc + _req(bias8.astype(np.int64) - 1, *bP, 0)
    want = np.clip(_req(acc, *oP, -2), -128, 127).astype(np.int8)
    np.testing.assert_array_equal(got, want)
    got = go.matmul_i8(x, w, 5, 4, -3, oP)
    acc = (x.astype(np.int64) - 4) @ (w.astype(np.int64) + 3)
    want = np.clip(_req(acc, *oP, 5), -128, 127).astype(np.int8)
    np.testing.assert_array_equal(got, want)


def test_cwq_conv2d_exact_kat():  # OperatorTest.cpp:11407-11485
    x = go.quantize_i8(np.arange(1, 13, dtype=np.float32), 1.0, 0).reshape(1, 2, 3, 2)
    filt = np.zeros((4, 2, 1, 1), np.int8)
    filt[:, 0] = 1
    filt[:, 1] = 2
    g = go.conv_geom(1, 2, 3, 2, 4, (2, 1), (1, 1), (0, 0, 0, 0), group=2)
    assert (g.OH, g.OW) == (1, 3)
    ident = go.quantize_scale_offset_32to8(1.0, 0)
    assert ident[:3] == (0, 0, 1)
    z = np.zeros(4, np.int32)
    one = np.ones(4, np.int32)
    out = go.cwq_conv2d_i8(x, filt, np.zeros(4, np.int32), g, 0, 0, z, z,
                           z, z, one, z, z, one)
    d = go.dequantize_i8(out, 1.0, 0).reshape(-1)
    np.testing.assert_array_equal(
        d, [15, 15, 18, 18, 21, 21, 24, 24, 27, 27, 30, 30])


def _conv_brute(x, filt, bias_scaled, g, in_off, f_off):
    """int64 accumulator of a grouped NHWC conv with skipped pad taps."""
    acc = np.zeros((g.N, g.OH, g.OW, g.OC), np.int64)
    icg, ocg = g.IC // g.group, g.OC // g.group
    for n in range(g.N):
        for d in range(g.OC):
            grp = d // ocg
            for ax in range(g.OH):
                for ay in range(g.OW):
                    s = int(bias_scaled[d])
                    for fx in range(g.KH):
                        for fy in range(g.KW):
                            ox = ax * g.strideH - g.padT + fx * g.dilH
                            oy = ay * g.strideW - g.padL + fy * g.dilW
                            if ox < 0 or oy < 0 or ox >= g.IH or oy >= g.IW:
                                continue
                            xi = x[n, ox, oy, grp * icg:(grp + 1) * icg].astype(np.int64)
                            fi = filt[d, fx, fy].astype(np.int64)
                            s += int(((xi - in_off) * (fi - f_off[d])).sum())
                    acc[n, ax, ay, d] = s
    return acc


@pytest.mark.parametrize("group,dil,stride,act", [
    (1, (1, 1), (1, 1), go.ACT_RELU), (2, (2, 1), (2, 1), go.ACT_NONE),
    (1, (1, 2), (1, 2), go.ACT_CLIP)])
def test_conv_brute_force(group, dil, stride, act):
    rng = np.random.default_rng(6)
    N, IH, IW, IC, OC = 2, 6, 5, 4, 6
    x = rng.integers(-128, 128, (N, IH, IW, IC)).astype(np.int8)
    filt = rng.integers(-128, 128, (OC, 3, 2, IC // group)).astype(np.int8)
    bias = rng.integers(-3000, 3000, OC).astype(np.int32)
    g = go.conv_geom(N, IH, IW, IC, OC, (3, 2), stride, (1, 1, 1, 0), group, dil)
    f_off = rng.integers(-4, 5, OC).astype(np.int32)
    b_off = rng.integers(-4, 5, OC).astype(np.int32)
    bp = np.array([go.quantize_scale_offset_32to8(float(s), 0)[:3]
                   for s in rng.uniform(0.3, 2.0, OC)], np.int32)
    op = np.array([go.quantize_scale_offset_32to8(float(s), 0)[:3]
                   for s in rng.uniform(0.001, 0.02, OC)], np.int32)
    in_off, out_off = 5, -20
    args = (-30, 40) if act == go.ACT_CLIP else ()
    got = go.cwq_conv2d_i8(x, filt, bias, g, out_off, in_off, f_off, b_off,
                           bp[:, 0], bp[:, 1], bp[:, 2], op[:, 0], op[:, 1],
                           op[:, 2], act, args)
    bs = _req(bias.astype(np.int64) - b_off, bp[:, 0], bp[:, 1], bp[:, 2], 0)
    acc = _conv_brute(x, filt, bs, g, in_off, f_off)
    y = _req(acc, op[:, 0], op[:, 1], op[:, 2], out_off)
    if act == go.ACT_RELU:
        y = np.maximum(y, out_off)
    elif act == go.ACT_CLIP:
        y = np.minimum(np.maximum(y, args[0]), args[1])
    np.testing.assert_array_equal(got, np.clip(y, -128, 127).astype(np.int8))
    # uniform-parameter convolution == channelwise with constant vectors
    got_u = go.conv2d_i8(x, filt, bias, g, out_off, in_off, 3, -2, bp[0], op[0],
                         act, args)
    c = lambda v: np.full(OC, v, np.int32)
    got_c = go.cwq_conv2d_i8(x, filt, bias, g, out_off, in_off, c(3), c(-2),
                             c(bp[0, 0]), c(bp[0, 1]), c(bp[0, 2]), c(op[0, 0]),
                             c(op[0, 1]), c(op[0, 2]), act, args)
    np.testing.assert_array_equal(got_u, got_c)


# ---- fused rowwise + SLWS ---------------------------------------------------------

def test_fused_rowwise_quantize_layout_and_closed_form():
    rng = np.random.default_rng(7)
    x = rng.normal(0, 1, (5, 12)).astype(np.float32)
    x[3] = 2.5  # constant row: range < 1e-10 -> scale 1.0, offset = value
    f = go.fused_rowwise_quantize(x, go.U8_F32)
    assert f.shape == (5, 20)
    sc = f[:, 12:16].copy().view(np.float32).ravel()
    of = f[:, 16:20].copy().view(np.float32).ravel()
    mn, mx = x.min(1), x.max(1)
    np.testing.assert_array_equal(of, mn)
    want_sc = ((mx.astype(np.float64) - mn.astype(np.float64)) / 255.0).astype(np.float32)
    want_sc[3] = 1.0
    np.testing.assert_array_equal(sc, want_sc)
    q = np.floor(np.abs((x - of[:, None]) / sc[:, None]) + np.float32(0.5))
    np.testing.assert_array_equal(f[:, :12], q.astype(np.uint8))
    # 4-bit: even column in the low nibble, fp16 scale/offset
    f4 = go.fused_rowwise_quantize(x, go.U4_F16)
    assert f4.shape == (5, 6 + 4)
    sc4 = ((mx.astype(np.float64) - mn.astype(np.float64)) / 15.0).astype(np.float32)
    sc4[3] = 1.0
    q4 = np.clip(np.floor((x - mn[:, None]) / sc4[:, None] + np.float32(0.5)), 0, 15).astype(np.uint8)
    np.testing.assert_array_equal(f4[:, :6], q4[:, 0::2] | (q4[:, 1::2] << 4))
    np.testing.assert_array_equal(f4[:, 6:8].copy().view(np.float16).ravel(),
                                  sc4.astype(np.float16))
    np.testing.assert_array_equal(f4[:, 8:10].copy().view(np.float16).ravel(),
                                  mn.astype(np.float16))


@pytest.mark.parametrize("kind", [go.U4_F32, go.U4_F16])
@pytest.mark.parametrize("delta", [-3, 0, 3, -7, 7])
def test_fused_4bit_round_trip(kind, delta):  # QuantizationTest.cpp:444-489
    x = np.array([[(i + j) * 1.0 + delta for j in range(6)] for i in range(2)],
                 np.float32)
    f = go.fused_rowwise_quantize(x, kind)
    assert f.shape == (2, 3 + (8 if kind == go.U4_F32 else 4))
    d = go.frwq_slws_generic(f, kind, None, np.arange(2, dtype=np.int64),
                             np.ones(2, np.int32))
    assert np.max(np.abs(d - x)) <= 0.02


def test_rowwise_quantize_equals_per_row_tensor_quantize():  # QuantizationTest.cpp:603-684
    rng = np.random.default_rng(8)
    w = rng.normal(0, 0.3, (6, 20)).astype(np.float32)
    for schema in (go.ASYMMETRIC, go.SYMMETRIC, go.SYMMETRIC_WITH_UNSIGNED,
                   go.SYMMETRIC_POW2):
        q, s, o = go.rowwise_quantize_i8(w, schema)
        for i in range(6):
            si, oi = go.choose_qparams(float(w[i].min()), float(w[i].max()), schema)
            assert (s[i], o[i]) == (np.float32(si), oi)
            np.testing.assert_array_equal(q[i], go.quantize_i8(w[i], si, oi))


def _slws_case_weighted():
    data = np.array([[2.0], [-0.5], [13.0]], np.float32)
    w = np.array([3, 1, 0, 0, 0, 0, 2, -0.5], np.float32)
    idx = np.array([1, 0, 2, 0, 1, 2, 2, 0])
    lens = np.array([3, 0, 3, 2], np.int32)
    return data, w, idx, lens, np.array([[0.5], [0], [0], [25]], np.float32)


@pytest.mark.parametrize("idt", [np.int64, np.int32])
def test_slws_float_kat(idt):  # OperatorTest.cpp:16941-17040
    data, w, idx, lens, want = _slws_case_weighted()
    f = go.fused_rowwise_quantize(data, go.U8_F32)
    out = go.frwq_slws_f32(f, w, idx.astype(idt), lens)
    assert np.max(np.abs(out - want)) <= 1e-4
    out = go.frwq_slws_generic(f, go.U8_F32, w, idx.astype(idt), lens)
    assert np.max(np.abs(out - want)) <= 1e-4
    # fp16 scale/offset kind, fp16 weights/out, both accumulation modes
    f16 = go.fused_rowwise_quantize(data, go.U8_F16)
    for acc in (False, True):
        out = go.frwq_slws_generic(f16, go.U8_F16, w.astype(np.float16),
                                   idx.astype(idt), lens, out_f16=True,
                                   fp16_accum=acc)
        assert out.dtype == np.float16
        assert np.max(np.abs(out.astype(np.float32) - want)) <= 1e-4


_TWO_COL = np.array([[1.0, 1.2], [2.3, 3.4], [4.5, 5.7]], np.float32)
_TC_IDX = np.array([2, 0, 1, 2, 0, 0, 0, 0], np.int64)
_TC_LEN = np.array([2, 0, 2, 1, 3], np.int32)


def test_sls_float_kat():  # OperatorTest.cpp:17314-17380
    want = np.array([[5.5, 6.9], [0, 0], [6.8, 9.1], [1.0, 1.2], [3.0, 3.6]], np.float32)
    f = go.fused_rowwise_quantize(_TWO_COL, go.U8_F32)
    out = go.frwq_slws_f32(f, np.ones(8, np.float32), _TC_IDX, _TC_LEN)
    assert np.max(np.abs(out - want)) <= 0.015
    out2 = go.frwq_slws_generic(f, go.U8_F32, None, _TC_IDX, _TC_LEN)
    np.testing.assert_array_equal(out, out2)
    # 4-bit fp16 SLS, tolerance of OperatorTest.cpp:17401-17407
    f4 = go.fused_rowwise_quantize(_TWO_COL, go.U4_F16)
    for acc in (False, True):
        o4 = go.frwq_slws_generic(f4, go.U4_F16, None, _TC_IDX, _TC_LEN,
                                  out_f16=True, fp16_accum=acc)
        assert np.max(np.abs(o4.astype(np.float32) - want)) <= 0.15


def test_slws_two_column_kat():  # OperatorTest.cpp:17411-17547
    w = np.array([1, -1, 1.5, 0.5, -1.5, 2, -2, -0.5], np.float32)
    want = np.array([[3.5, 4.5], [0, 0], [5.7, 7.95], [-1.5, -1.8], [-0.5, -0.6]], np.float32)
    f = go.fused_rowwise_quantize(_TWO_COL, go.U8_F32)
    out = go.frwq_slws_f32(f, w, _TC_IDX, _TC_LEN)
    assert np.max(np.abs(out - want)) <= 0.015
    f16 = go.fused_rowwise_quantize(_TWO_COL, go.U8_F16)
    for acc in (False, True):
        o = go.frwq_slws_generic(f16, go.U8_F16, w.astype(np.float16), _TC_IDX,
                                 _TC_LEN, out_f16=True, fp16_accum=acc)
        assert np.max(np.abs(o.astype(np.float32) - want)) <= 0.015
    f4 = go.fused_rowwise_quantize(_TWO_COL, go.U4_F16)
    o = go.frwq_slws_generic(f4, go.U4_F16, w.astype(np.float16), _TC_IDX,
                             _TC_LEN, out_f16=True, fp16_accum=True)
    assert np.max(np.abs(o.astype(np.float32) - want)) <= 0.1
    f4f = go.fused_rowwise_quantize(_TWO_COL, go.U4_F32)
    o = go.frwq_slws_generic(f4f, go.U4_F32, w, _TC_IDX, _TC_LEN)
    assert np.max(np.abs(o - want)) <= 0.1


def test_4bit_near_exact_kat():  # OperatorTest.cpp:16152-16295
    data = np.array([0, 1, 2, 3, 0, 1, 2, 3, 0, 1, 2, 3, -3, -2, -1, 0,
                     0, -1, -2, -3, 2, 2, 2, 2, 2, 2, 2, 2], np.float32).reshape(7, 4)
    w = np.array([1, 2, 3, 2, 0.5, -0.5, 2], np.float16)
    idx = np.array([0, 1, 2, 4, 3, 5, 6], np.int32)
    lens = np.array([3, 2, 2, 0], np.int32)  # offsets {0,3,5,7}
    want = np.array([[0, 6, 12, 18], [-1.5, -3, -4.5, -6], [3, 3, 3, 3],
                     [0, 0, 0, 0]], np.float32)
    f = go.fused_rowwise_quantize(data, go.U4_F16)
    for acc in (False, True):
        o = go.frwq_slws_generic(f, go.U4_F16, w, idx, lens, out_f16=True,
                                 fp16_accum=acc)
        assert np.max(np.abs(o.astype(np.float32) - want)) <= 0.005


def test_slws_generic_brute_force_numpy():
    rng = np.random.default_rng(9)
    rows, cols = 9, 6
    x = rng.normal(0, 1, (rows, cols)).astype(np.float32)
    lens = np.array([3, 0, 5, 1], np.int32)
    idx = rng.integers(0, rows, lens.sum()).astype(np.int64)
    w = rng.uniform(-1, 1, lens.sum()).astype(np.float32)
    for kind in (go.U8_F32, go.U8_F16, go.U4_F16, go.U4_F32):
        f = go.fused_rowwise_quantize(x, kind)
        so = 8 if kind in (go.U8_F32, go.U4_F32) else 4
        dt = np.float32 if so == 8 else np.float16
        half = so // 2
        sc = f[:, -so:-half].copy().view(dt).astype(np.float32).ravel()
        of = f[:, -half:].copy().view(dt).astype(np.float32).ravel()
        if kind in (go.U4_F16, go.U4_F32):
            b = f[:, :cols // 2]
            q = np.empty((rows, cols), np.float32)
            q[:, 0::2] = b & 15
            q[:, 1::2] = b >> 4
        else:
            q = f[:, :cols].astype(np.float32)
        deq = q * sc[:, None] + of[:, None]
        want = np.zeros((lens.size, cols), np.float32)
        cur = 0
        for i, L in enumerate(lens):
            for _ in range(L):
                want[i] = want[i] + deq[idx[cur]] * w[cur]
                cur += 1
        out16 = so == 4
        got = go.frwq_slws_generic(f, kind, w, idx, lens, out_f16=out16)
        if out16:
            np.testing.assert_array_equal(got, want.astype(np.float16))
        else:
            np.testing.assert_array_equal(got, want)


def test_slws_fp16_accumulation_brute_force_numpy():
    """The float16-accumulator branch (reference InterpreterNodes.cpp:5799-5836
    with AccumT = float16_t, Float16.h operator+=): every product is rounded to
    half on its own, and so is every partial sum. numpy's float16 is an
    independent implementation of the roundings; the inputs are not
    representable in half, so dropping either rounding changes bits."""
    rng = np.random.default_rng(2024)
    rows, cols = 40, 16
    x = rng.normal(0, 3, (rows, cols)).astype(np.float32)
    lens = np.array([7, 0, 12, 1, 30], np.int32)
    idx = rng.integers(0, rows, lens.sum()).astype(np.int64)
    w = rng.uniform(-2, 2, lens.sum()).astype(np.float16)
    differs_from_f32_accum = differs_from_unrounded_product = 0
    for kind in (go.U8_F16, go.U4_F16):
        f = go.fused_rowwise_quantize(x, kind)
        sc = f[:, -4:-2].copy().view(np.float16).astype(np.float32).ravel()
        of = f[:, -2:].copy().view(np.float16).astype(np.float32).ravel()
        if kind == go.U4_F16:
            b = f[:, :cols // 2]
            q = np.empty((rows, cols), np.float32)
            q[:, 0::2] = b & 15
            q[:, 1::2] = b >> 4
        else:
            q = f[:, :cols].astype(np.float32)
        deq = (q * sc[:, None]).astype(np.float32) + of[:, None]   # fp32, separately rounded
        want = np.zeros((lens.size, cols), np.float16)
        loose = np.zeros((lens.size, cols), np.float16)            # product left in fp32
        cur = 0
        for i, L in enumerate(lens):
            acc = np.zeros(cols, np.float16)
            acc2 = np.zeros(cols, np.float16)
            for _ in range(L):
                prod = deq[idx[cur]] * np.float32(w[cur])           # fp32
                term = prod.astype(np.float16)                      # rounded to half
                acc = (acc.astype(np.float32) + term.astype(np.float32)).astype(np.float16)
                acc2 = (acc2.astype(np.float32) + prod).astype(np.float16)
                cur += 1
            want[i], loose[i] = acc, acc2
        got = go.frwq_slws_generic(f, kind, w, idx, lens, out_f16=True, fp16_accum=True)
        np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))
        f32acc = go.frwq_slws_generic(f, kind, w, idx, lens, out_f16=True, fp16_accum=False)
        differs_from_f32_accum += int((f32acc.view(np.uint16) != want.view(np.uint16)).sum())
        differs_from_unrounded_product += int((loose.view(np.uint16) != want.view(np.uint16)).sum())
    # the check discriminates: both simplifications change bits on these inputs
    assert differs_from_f32_accum > 0 and differs_from_unrounded_product > 0


def test_slws_invariants():
    rng = np.random.default_rng(10)
    x = rng.normal(0, 1, (50, 16)).astype(np.float32)
    f = go.fused_rowwise_quantize(x, go.U8_F32)
    lens = rng.poisson(4, 20).astype(np.int32)
    idx = rng.integers(0, 50, lens.sum()).astype(np.int64)
    w = rng.uniform(0, 1, lens.sum()).astype(np.float32)
    a = go.frwq_slws_f32(f, w, idx, lens)
    np.testing.assert_array_equal(a[lens == 0], 0)  # empty bag -> zeros
    # linear in the weights (up to rounding)
    b = go.frwq_slws_f32(f, 2 * w, idx, lens)
    np.testing.assert_allclose(b, 2 * a, rtol=1e-6, atol=1e-6)
    # generic formula ((q*scale)+offset)*w agrees with libjit's w*((scale*q)+offset)
    c = go.frwq_slws_generic(f, go.U8_F32, w, idx, lens)
    np.testing.assert_array_equal(a, c)
    # int32 and int64 indices agree
    np.testing.assert_array_equal(a, go.frwq_slws_f32(f, w, idx.astype(np.int32), lens))


def test_embedding_bag_offsets_equals_lengths_form():
    rng = np.random.default_rng(11)
    x = rng.normal(0, 1, (30, 8)).astype(np.float32)
    f = go.fused_rowwise_quantize(x, go.U8_F32)
    lens = np.array([2, 0, 4, 3], np.int32)
    idx = rng.integers(0, 30, lens.sum()).astype(np.int32)
    w = rng.uniform(0, 1, lens.sum()).astype(np.float32)
    offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    a = go.frwq_slws_f32(f, w, idx, lens)
    b = go.embedding_bag_byte_rowwise_offsets_f32(f, w, idx, offs, True)
    np.testing.assert_array_equal(a, b)
    c = go.embedding_bag_byte_rowwise_offsets_f32(f, w, idx, offs[:-1], False)
    np.testing.assert_array_equal(a, c)


# ---- bias specialisation and channelwise convolution constants --------------------
# Base.cpp:567-629, Graph.cpp:3576-3700. The reference's tests hold no exact
# vectors for these (its operator tests compare against fp32 within a
# tolerance), so the restatement is pinned by what the algorithm fixes.

def test_specialize_bias_closed_forms():
    f = np.float32
    # the accumulator's scale is at least the bias's own: the bias takes it
    bs, bo = go.specialize_bias_qparams(1e-6, 7, 0.05, 0.01)
    assert f(bs) == f(0.05) * f(0.01) and bo == 0
    # the bias's own scale is larger: it is kept, the weights are untouched
    bs, bo = go.specialize_bias_qparams(1e-2, 7, 0.05, 0.01)
    assert f(bs) == f(1e-2) and bo == 0
    # ... unless the bias is all zero
    bs, bo = go.specialize_bias_qparams(1e-2, 7, 0.05, 0.01, bias_zero=True)
    assert f(bs) == f(0.05) * f(0.01)
    # an int8 bias keeps its offset
    assert go.specialize_bias_qparams(1e-6, 7, 0.05, 0.01, bias_is_i32=False)[1] == 7
    # bias-and-weights variant: the weights scale gives way, and the product is
    # re-formed so that it equals the bias scale bit for bit
    bs, bo, ws = go.specialize_bias_weights_qparams(1e-2, 3, 0.05, 0.01)
    assert f(ws) == f(1e-2) / f(0.05) and f(bs) == f(0.05) * f(ws) and bo == 0
    bs, bo, ws = go.specialize_bias_weights_qparams(1e-6, 3, 0.05, 0.01)
    assert f(ws) == f(0.01) and f(bs) == f(0.05) * f(0.01)


def test_channelwise_conv_constants_invariants():
    rng = np.random.default_rng(12)
    oc, per = 24, 3 * 3 * 16
    filt = (rng.standard_normal((oc, per)) * rng.uniform(0.01, 2.0, (oc, 1))).astype(np.float32)
    bias = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    bias[3] = 0.0
    bias[5] = 3.0e6        # so large that inScale * filterScale would saturate int32
    in_scale = np.float32(0.02)
    fq, bq, fs, fo, bs, bo = go.channelwise_quantize_conv(filt, bias, in_scale, go.SYMMETRIC)
    assert not fo.any() and not bo.any()                 # symmetric filter, int32 bias
    # the defining property (asserted by the reference itself): bit-exact product
    np.testing.assert_array_equal(bs, in_scale * fs)
    for c in range(oc):
        own_scale, own_off = go.choose_qparams(float(filt[c].min()), float(filt[c].max()),
                                               go.SYMMETRIC, 8)
        bias_own, _ = go.choose_qparams(float(bias[c]), float(bias[c]), go.SYMMETRIC, 32)
        if c == 5:
            # the filter scale gave way to keep the bias inside int32
            assert fs[c] > np.float32(own_scale) and fs[c] == np.float32(bias_own) / in_scale
        else:
            assert fs[c] == np.float32(own_scale)
        # each value is quantized by x / scale, round-half-even, clipped
        want = np.clip(np.rint(filt[c] / fs[c] + np.float32(fo[c])), -128, 127)
        np.testing.assert_array_equal(fq[c], want.astype(np.int8))
        wb = np.clip(np.rint(np.float64(np.float32(bias[c]) / bs[c])), -2 ** 31, 2 ** 31 - 1)
        assert bq[c] == int(wb)
        # round trip: within half a step where nothing was clipped
        assert np.abs(fq[c].astype(np.float32) * fs[c] - filt[c]).max() <= fs[c] * 0.5001
    # (the Int32QTy range the parameters are chosen for is 30 bits wide)
    assert bq[3] == 0 and abs(int(bq[5])) >= 2 ** 29 - 1

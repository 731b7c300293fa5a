"""Per-call options (mi355x_launch_opts): they are validated before anything
touches the device, they hold for the one call that names them whatever the
thread's or the process's defaults say, and two device managers in one process
run their SparseLengths launches each with its own arithmetic."""
import ctypes as C

import numpy as np
import pytest

from glow_amd import capi
from glow_amd import host as H
from tests import cases
from oracle import glow_oracle as go


def _slws_opts_call(opts):
    """mi355x_frwq_slws_opts on NULL tensors with zero bags: returns before any
    device work, after the options have been looked at."""
    z = C.c_void_p(0)
    return capi.lib().mi355x_frwq_slws_opts(
        z, 0, z, C.c_size_t(0), 0, z, 0, z, 1, C.c_size_t(0), z, C.c_size_t(0),
        C.c_size_t(136), C.c_size_t(128), 0, z, C.byref(opts))


def test_options_are_validated_on_the_host():
    assert _slws_opts_call(capi.LaunchOpts()) == 0
    bad = capi.LaunchOpts()
    bad.struct_size = 8
    assert _slws_opts_call(bad) == -1 and b"struct_size" in capi.lib().mi355x_last_error()
    # a caller built before the workspace fields existed passes the shorter struct
    short = capi.LaunchOpts()
    short.struct_size = 16
    assert _slws_opts_call(short) == 0
    for field, value in (("gemm_tile", 13), ("gemm_tile", -2), ("requant_hint", 2),
                         ("requant_hint", 4), ("slws_math", 3), ("slws_math", -2)):
        o = capi.LaunchOpts()
        setattr(o, field, value)
        assert _slws_opts_call(o) == -1, (field, value)
        assert field.encode() in capi.lib().mi355x_last_error()


def _emulate_element(table, w, idx, lengths, cols=128):
    """v = fma(s, q, o); acc = fma(w, v, acc), lookups of even and odd position
    in the bag summed apart (the two rows one load instruction fetches) and
    added at the end: the rows kernel's arithmetic, through float64 (exact
    products, one rounding)."""
    def fma32(a, b, c):
        return (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)).astype(np.float32)
    out = np.zeros((lengths.size, cols), np.float32)
    so = np.ascontiguousarray(table[:, cols:cols + 8]).view(np.float32)
    pos = 0
    for b, n in enumerate(lengths):
        acc = [np.zeros(cols, np.float32), np.zeros(cols, np.float32)]
        for j in range(n):
            r = idx[pos + j]
            v = fma32(np.full(cols, so[r, 0], np.float32), table[r, :cols].astype(np.float32),
                      np.full(cols, so[r, 1], np.float32))
            acc[j & 1] = fma32(np.full(cols, w[pos + j], np.float32), v, acc[j & 1])
        out[b] = acc[0] + acc[1]
        pos += n
    return out


@pytest.mark.gpu
def test_slws_arithmetic_named_by_the_call_wins_over_the_defaults():
    rng = np.random.default_rng(5)
    table = cases.random_fused_table(rng, 20000, 128)
    lengths, idx, w = cases.slws_batch(6, 20000, 200, 30, 1.05, np.int64)
    want = go.frwq_slws_f32(table, w, idx, lengths)
    emu = _emulate_element(table, w, idx, lengths)
    assert not np.array_equal(want, emu)   # the two arithmetics differ on this input
    for default in (capi.SLWS_MATH_STRICT, capi.SLWS_MATH_ELEMENT, capi.SLWS_MATH_REGROUPED):
        capi.slws_set_fused_math(default)
        strict = capi.frwq_slws(table, capi.FUSED_U8_F32, w, idx, lengths,
                                opts=capi.LaunchOpts(slws_math=capi.SLWS_MATH_STRICT))
        elem = capi.frwq_slws(table, capi.FUSED_U8_F32, w, idx, lengths,
                              opts=capi.LaunchOpts(slws_math=capi.SLWS_MATH_ELEMENT))
        np.testing.assert_array_equal(strict, want)
        np.testing.assert_array_equal(elem, emu)
        # the default is what a call without a named arithmetic gets
        plain = capi.frwq_slws(table, capi.FUSED_U8_F32, w, idx, lengths, opts=capi.LaunchOpts())
        np.testing.assert_array_equal(
            plain, capi.frwq_slws(table, capi.FUSED_U8_F32, w, idx, lengths))
        if default == capi.SLWS_MATH_STRICT:
            np.testing.assert_array_equal(plain, want)
        elif default == capi.SLWS_MATH_ELEMENT:
            np.testing.assert_array_equal(plain, emu)


@pytest.mark.gpu
def test_tile_named_by_the_call_and_a_tile_that_does_not_apply():
    c = cases.rwq_fc_case(21, 256, 512, 384)
    want = go.rwq_fc_i8(*cases.rwq_fc_args(c))
    d = {k: capi.to_device(np.ascontiguousarray(v)) for k, v in c.items()
         if isinstance(v, np.ndarray)}
    out = capi.DeviceBuffer.empty((256, 384), np.int8)

    def run(opts):
        out.fill(0x55)
        capi.launch_rwq_fc_i8(out, d["x"], d["w"], d["bias"], False, d["w_offsets"],
                              d["bias_pre"], d["bias_post"], d["bias_scale"], d["out_pre"],
                              d["out_post"], d["out_scale"], 256, 512, 384, c["out_offset"],
                              c["in_offset"], c["bias_offset"], True, opts=opts)
        capi.sync()
        return out.numpy()

    # a thread default that the calls below must not see, and must not disturb
    capi.check(capi.lib().mi355x_gemm_tile_override(3))
    try:
        for tile in (-1, 0, 1, 2, 3, 4, 5, 9, 10, 11):
            np.testing.assert_array_equal(run(capi.LaunchOpts(gemm_tile=tile)), want)
        # tile 8 (the streaming kernel) needs K of 64, 128 or 256: K = 512 is refused
        with pytest.raises(capi.MI355XError) as e:
            run(capi.LaunchOpts(gemm_tile=8))
        assert e.value.code == -4
        np.testing.assert_array_equal(run(None), want)   # the thread's default tile still works
    finally:
        capi.check(capi.lib().mi355x_gemm_tile_override(-1))


@pytest.mark.gpu
def test_two_device_managers_keep_their_own_lookup_arithmetic():
    rng = np.random.default_rng(18)
    rows, cols, bags = 5000, 128, 300
    table = cases.random_fused_table(rng, rows, cols)
    lengths, idx, w = cases.slws_batch(19, rows, bags, 12, 1.05, np.int64)
    want = go.frwq_slws_f32(table, w, idx, lengths)
    emu = _emulate_element(table, w, idx, lengths)
    assert not np.array_equal(want, emu)

    def module(name):
        m = H.Module(name)
        data = m.constant("data", table, H.UINT8_FUSED)
        wv = m.placeholder("weights", (idx.size,), H.FLOAT, np.float32)
        iv = m.placeholder("indices", (idx.size,), H.INT64I, np.int64)
        lv = m.placeholder("lengths", (bags,), H.INT32I, np.int32)
        out = m.placeholder("output", (bags, cols), H.FLOAT, np.float32)
        f = m.function("main")
        m.instruction(f, H.FRWQ_SLWS, "slws", [out, data, wv, iv, lv], [0])
        m.compile(f)
        return m

    strict_dm = H.DeviceManager(slws_math=capi.SLWS_MATH_STRICT).init()
    element_dm = H.DeviceManager(slws_math=capi.SLWS_MATH_ELEMENT).init()
    try:
        strict_dm.add_network(module("a"))
        element_dm.add_network(module("b"))
        # whatever the process default is, and in whichever order they run
        for default in (capi.SLWS_MATH_ELEMENT, capi.SLWS_MATH_STRICT):
            capi.slws_set_fused_math(default)
            for dm, expect in ((strict_dm, want), (element_dm, emu), (strict_dm, want)):
                res = np.zeros((bags, cols), np.float32)
                dm.run("main", {"weights": w, "indices": idx, "lengths": lengths, "output": res})
                np.testing.assert_array_equal(res, expect)
    finally:
        strict_dm.stop()
        element_dm.stop()

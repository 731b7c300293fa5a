"""Builds host-layer modules (glow_amd.host) from the seeded operator cases of
tests/cases.py, whose integer parameters come from the oracle's host math: the
backend under test has to derive the same ones from the float scales."""
import numpy as np

from glow_amd import host as H


def rwq_fc_module(c, name="main", bias_i8=False):
    M, K = c["x"].shape
    N = c["w"].shape[0]
    m = H.Module("rwqfc")
    x = m.placeholder("input", (M, K), H.INT8Q, np.int8, c["in_scale_f"], c["in_offset"])
    out = m.placeholder("output", (M, N), H.INT8Q, np.int8, c["out_scale_f"], c["out_offset"])
    w = m.constant("weights", c["w"], H.INT8Q)
    b = m.constant("bias", c["bias"], H.INT8Q if bias_i8 else H.INT32Q,
                   c["bias_scale_f"], c["bias_offset"])
    sc = m.constant("scales", c["w_scales"].astype(np.float32))
    of = m.constant("offsets", c["w_offsets"].astype(np.int32), H.INT32I)
    f = m.function(name)
    m.instruction(f, H.ROWWISE_QUANTIZED_FC, "rwqfc", [out, x, w, b, sc, of])
    return m, f


def fc_module(c, bias_i8=False, name="main"):
    M, K = c["x"].shape
    N = c["w"].shape[1]
    m = H.Module("fc")
    x = m.placeholder("input", (M, K), H.INT8Q, np.int8, c["in_scale_f"], c["in_offset"])
    out = m.placeholder("output", (M, N), H.INT8Q, np.int8, c["out_scale_f"], c["out_offset"])
    w = m.constant("weights", c["w"], H.INT8Q, c["w_scale_f"], c["w_offset"])
    b = m.constant("bias", c["bias"], H.INT8Q if bias_i8 else H.INT32Q,
                   c["bias_scale_f"], c["bias_offset"])
    f = m.function(name)
    m.instruction(f, H.FULLY_CONNECTED, "fc", [out, x, w, b])
    return m, f


def cwq_conv_module(c, kernel=(3, 3), stride=(1, 1), pads=(1, 1, 1, 1), group=1,
                    dilation=(1, 1), bias_i8=False, name="main"):
    g = c["geom"]
    m = H.Module("conv")
    x = m.placeholder("input", c["x"].shape, H.INT8Q, np.int8, c["in_scale_f"], c["in_offset"])
    out = m.placeholder("output", (g.N, g.OH, g.OW, g.OC), H.INT8Q, np.int8,
                        c["out_scale_f"], c["out_offset"])
    filt = m.constant("filter", c["filt"], H.INT8Q)
    b = m.constant("bias", c["bias"], H.INT8Q if bias_i8 else H.INT32Q)
    fs = m.constant("filterScales", c["f_scales"])
    fo = m.constant("filterOffsets", c["f_offsets"], H.INT32I)
    bs = m.constant("biasScales", c["b_scales"])
    bo = m.constant("biasOffsets", c["b_offsets"], H.INT32I)
    f = m.function(name)
    m.instruction(f, H.CHANNELWISE_QUANTIZED_CONV, "conv",
                  [out, x, filt, b, fs, fo, bs, bo],
                  H.conv_attrs(kernel, stride, pads, group, dilation, c["act"]),
                  c["act_fargs"])
    return m, f


def cwq_conv3d_module(c, kernel, stride, pads, group=1, bias_i8=False, name="main"):
    """ChannelwiseQuantizedConvolution over NTHWC tensors; pads are
    (near, far, top, bottom, left, right)."""
    g = c["geom"]
    m = H.Module("conv3d")
    x = m.placeholder("input", c["x"].shape, H.INT8Q, np.int8, c["in_scale_f"], c["in_offset"])
    out = m.placeholder("output", (g.N, g.OT, g.OH, g.OW, g.OC), H.INT8Q, np.int8,
                        c["out_scale_f"], c["out_offset"])
    filt = m.constant("filter", c["filt"], H.INT8Q)
    b = m.constant("bias", c["bias"], H.INT8Q if bias_i8 else H.INT32Q)
    fs = m.constant("filterScales", c["f_scales"])
    fo = m.constant("filterOffsets", c["f_offsets"], H.INT32I)
    bs = m.constant("biasScales", c["b_scales"])
    bo = m.constant("biasOffsets", c["b_offsets"], H.INT32I)
    f = m.function(name)
    m.instruction(f, H.CHANNELWISE_QUANTIZED_CONV, "conv3d", [out, x, filt, b, fs, fo, bs, bo],
                  [*kernel, *stride, *pads, group, c["act"]], c["act_fargs"])
    return m, f

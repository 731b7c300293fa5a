"""Seeded synthetic operator workloads (numpy) for the benchmark and the
tests. Integer parameters are derived the way Glow's CPU code generator
derives them (reference lib/LLVMIRCodeGen/LLVMIRGen.cpp:2222-2320, 2695-2798)
through a `Host` object that supplies quantizeScaleOffset32To8 and friends:
by default the library's own host math."""
import numpy as np

from glow_amd import capi

ACT_NONE, ACT_RELU, ACT_CLIP, ACT_TANH, ACT_SIGMOID, ACT_LEAKY_RELU = range(6)
U8_F32, U8_F16, U4_F16, U4_F32 = 0, 1, 2, 3


class Host:
    """Host-side parameter math used to build the cases."""

    def s32to8(self, scale, offset=0):
        return capi.quantize_scale_offset_32to8(scale, offset)

    def quantize_value_i32(self, x, scale, offset):
        r = np.float32(x) / np.float32(scale) + np.float32(offset)
        return int(np.clip(np.rint(r), -2 ** 31, 2 ** 31 - 1))

    def conv_geom(self, N, IH, IW, IC, OC, kernel, stride, pads, group=1,
                  dilation=(1, 1)):
        KH, KW = kernel
        sh, sw = stride
        pt, pl, pb, pr = pads
        dh, dw = dilation
        OH = (IH + pt + pb - (KH - 1) * dh - 1) // sh + 1
        OW = (IW + pl + pr - (KW - 1) * dw - 1) // sw + 1
        return capi.ConvGeom(N, IH, IW, IC, OH, OW, OC, KH, KW, sh, sw, pt, pl,
                             dh, dw, group)

    def conv3d_geom(self, *a, **kw):
        return capi.conv3d_geom(*a, **kw)

    def fused_row_bytes(self, cols, kind):
        return (cols // 2 if kind in (U4_F16, U4_F32) else cols) + \
            (8 if kind in (U8_F32, U4_F32) else 4)


_HOST = None


def default_host():
    global _HOST
    if _HOST is None:
        _HOST = Host()
    return _HOST



def s32to8_vec(ratios, host=None):
    """Per-element quantizeScaleOffset32To8 -> (pre, post, scale) int32 vectors."""
    host = host or default_host()
    p = np.array([host.s32to8(float(np.float32(r)), 0)[:3]
                  for r in np.asarray(ratios, np.float32)], np.int32)
    p = p.reshape(-1, 3)
    return (np.ascontiguousarray(p[:, 0]), np.ascontiguousarray(p[:, 1]),
            np.ascontiguousarray(p[:, 2]))


def rwq_fc_case(seed, M, K, N, in_scale=0.05, out_scale=0.1, out_offset=0,
                w_scale_range=(0.001, 0.02), symmetric=True, bias_i8=False,
                bias_scale=5e-5, bias_offset=0, in_offset=None, sigma=40.0, host=None):
    """RowwiseQuantizedFullyConnected operands and per-row parameters.

    The defaults are the single-FC configuration: int8 input clamp(N(0,40)),
    scale 0.05, offset ~ U{-10..10}; symmetric per-row weight scales
    ~ U[0.001, 0.02]; int32 bias ~ U{-1000..1000} at scale 5e-5 offset 0;
    output scale 0.1 offset 0."""
    rng = np.random.default_rng(seed)
    x = np.clip(np.rint(rng.normal(0, sigma, (M, K))), -128, 127).astype(np.int8)
    if in_offset is None:
        in_offset = int(rng.integers(-10, 11))
    w = rng.integers(-127, 128, (N, K)).astype(np.int8)
    w_scales = rng.uniform(*w_scale_range, N).astype(np.float32)
    w_offsets = (np.zeros(N, np.int32) if symmetric
                 else rng.integers(-20, 21, N).astype(np.int32))
    if bias_i8:
        bias = rng.integers(-128, 128, N).astype(np.int8)
    else:
        bias = rng.integers(-1000, 1001, N).astype(np.int32)
    mm = np.float32(in_scale) * w_scales              # matMulScale, fp32
    bpre, bpost, bscale = s32to8_vec(np.float32(bias_scale) / mm, host)
    opre, opost, oscale = s32to8_vec(mm / np.float32(out_scale), host)
    return dict(x=x, w=w, bias=bias, w_offsets=w_offsets, w_scales=w_scales,
                bias_pre=bpre, bias_post=bpost, bias_scale=bscale,
                out_pre=opre, out_post=opost, out_scale=oscale,
                out_offset=int(out_offset), in_offset=int(in_offset),
                bias_offset=int(bias_offset), in_scale_f=float(in_scale),
                out_scale_f=float(out_scale), bias_scale_f=float(bias_scale))


def rwq_fc_args(c):
    return (c["x"], c["w"], c["bias"], c["w_offsets"], c["bias_pre"],
            c["bias_post"], c["bias_scale"], c["out_pre"], c["out_post"],
            c["out_scale"], c["out_offset"], c["in_offset"], c["bias_offset"])


def fc_case(seed, M, K, N, bias_i8=False, host=None):
    """Uniform-parameter FullyConnected, weights [K x N]."""
    host = host or default_host()
    rng = np.random.default_rng(seed)
    x = rng.integers(-128, 128, (M, K)).astype(np.int8)
    w = rng.integers(-128, 128, (K, N)).astype(np.int8)
    bias = (rng.integers(-128, 128, N).astype(np.int8) if bias_i8
            else rng.integers(-5000, 5001, N).astype(np.int32))
    in_scale, w_scale, out_scale = np.float32(0.04), np.float32(0.007), np.float32(0.6)
    b_scale = np.float32(0.02) if bias_i8 else in_scale * w_scale
    mm = in_scale * w_scale
    biasP = host.s32to8(float(b_scale / mm), 0)[:3]
    outP = host.s32to8(float(mm / out_scale), 0)[:3]
    return dict(x=x, w=w, bias=bias, out_offset=int(rng.integers(-10, 11)),
                in_offset=int(rng.integers(-10, 11)),
                w_offset=int(rng.integers(-5, 6)),
                bias_offset=int(rng.integers(-3, 4)) if bias_i8 else 0,
                biasP=biasP, outP=outP, in_scale_f=float(in_scale),
                w_scale_f=float(w_scale), out_scale_f=float(out_scale),
                bias_scale_f=float(b_scale))


def fc_args(c):
    return (c["x"], c["w"], c["bias"], c["out_offset"], c["in_offset"],
            c["w_offset"], c["bias_offset"], c["biasP"], c["outP"])


def cwq_conv_case(seed, N, H, W, IC, OC, kernel=(3, 3), stride=(1, 1),
                  pads=(1, 1, 1, 1), group=1, dilation=(1, 1), act=ACT_RELU,
                  in_scale=0.05, in_offset=0, out_scale=None, out_offset=-128,
                  f_scale_range=(0.002, 0.02), symmetric=True, bias_i8=False,
                  host=None):
    """ChannelwiseQuantizedConvolution operands and per-channel parameters.
    Bias parameters follow Glow's specialisation for int32 bias: scale ==
    inScale * filterScale, offset 0 (Base.cpp:594-629)."""
    host = host or default_host()
    rng = np.random.default_rng(seed)
    x = rng.integers(-128, 128, (N, H, W, IC)).astype(np.int8)
    filt = rng.integers(-127, 128, (OC, kernel[0], kernel[1], IC // group)).astype(np.int8)
    f_scales = rng.uniform(*f_scale_range, OC).astype(np.float32)
    f_offsets = (np.zeros(OC, np.int32) if symmetric
                 else rng.integers(-10, 11, OC).astype(np.int32))
    mm = np.float32(in_scale) * f_scales
    if bias_i8:
        bias = rng.integers(-128, 128, OC).astype(np.int8)
        b_scales = mm * np.float32(37.0)
        b_offsets = rng.integers(-5, 6, OC).astype(np.int32)
    else:
        bias = rng.integers(-20000, 20001, OC).astype(np.int32)
        b_scales = mm
        b_offsets = np.zeros(OC, np.int32)
    if out_scale is None:
        # keep a good share of the outputs inside the int8 range
        k = kernel[0] * kernel[1] * (IC // group)
        out_scale = float(np.sqrt(k) * 74 * 74 * in_scale * f_scales.mean() / 40)
    bpre, bpost, bscale = s32to8_vec(b_scales / mm, host)
    opre, opost, oscale = s32to8_vec(mm / np.float32(out_scale), host)
    g = host.conv_geom(N, H, W, IC, OC, kernel, stride, pads, group, dilation)
    act_args, act_fargs = (), ()
    if act == ACT_CLIP:
        act_fargs = (0.0, float(np.float32(6.0 * out_scale * 20)))
        act_args = (host.quantize_value_i32(act_fargs[0], out_scale, out_offset),
                    host.quantize_value_i32(act_fargs[1], out_scale, out_offset))
    elif act == ACT_LEAKY_RELU:
        act_fargs = (0.1,)
        act_args = host.s32to8(0.1, 0)[:3]
    return dict(x=x, filt=filt, bias=bias, geom=g, out_offset=int(out_offset),
                in_offset=int(in_offset), f_offsets=f_offsets,
                b_offsets=b_offsets, bias_pre=bpre, bias_post=bpost,
                bias_scale=bscale, out_pre=opre, out_post=opost,
                out_scale=oscale, act=act, act_args=act_args,
                act_fargs=act_fargs, f_scales=f_scales, b_scales=np.asarray(b_scales, np.float32),
                in_scale_f=float(in_scale), out_scale_f=float(out_scale))


def cwq_conv_args(c):
    return (c["x"], c["filt"], c["bias"], c["geom"], c["out_offset"],
            c["in_offset"], c["f_offsets"], c["b_offsets"], c["bias_pre"],
            c["bias_post"], c["bias_scale"], c["out_pre"], c["out_post"],
            c["out_scale"], c["act"], c["act_args"])


def cwq_conv3d_case(seed, N, T, H, W, IC, OC, kernel=(3, 3, 3), stride=(1, 1, 1),
                    pads=(1, 1, 1, 1, 1, 1), group=1, act=ACT_RELU, in_scale=0.05,
                    in_offset=0, out_offset=-128, symmetric=True, bias_i8=False, host=None):
    """Operands and per-channel parameters of the channelwise quantized 3-D
    convolution (NTHWC), derived like cwq_conv_case."""
    host = host or default_host()
    rng = np.random.default_rng(seed)
    x = rng.integers(-128, 128, (N, T, H, W, IC)).astype(np.int8)
    filt = rng.integers(-127, 128, (OC, *kernel, IC // group)).astype(np.int8)
    f_scales = rng.uniform(0.002, 0.02, OC).astype(np.float32)
    f_offsets = (np.zeros(OC, np.int32) if symmetric
                 else rng.integers(-10, 11, OC).astype(np.int32))
    mm = np.float32(in_scale) * f_scales
    if bias_i8:
        bias = rng.integers(-128, 128, OC).astype(np.int8)
        b_scales = mm * np.float32(37.0)
        b_offsets = rng.integers(-5, 6, OC).astype(np.int32)
    else:
        bias = rng.integers(-20000, 20001, OC).astype(np.int32)
        b_scales = mm
        b_offsets = np.zeros(OC, np.int32)
    k = kernel[0] * kernel[1] * kernel[2] * (IC // group)
    out_scale = float(np.sqrt(k) * 74 * 74 * in_scale * f_scales.mean() / 40)
    bpre, bpost, bscale = s32to8_vec(b_scales / mm, host)
    opre, opost, oscale = s32to8_vec(mm / np.float32(out_scale), host)
    g = host.conv3d_geom(N, T, H, W, IC, OC, kernel, stride, pads, group)
    act_args, act_fargs = (), ()
    if act == ACT_CLIP:
        act_fargs = (0.0, float(np.float32(6.0 * out_scale * 20)))
        act_args = (host.quantize_value_i32(act_fargs[0], out_scale, out_offset),
                    host.quantize_value_i32(act_fargs[1], out_scale, out_offset))
    elif act == ACT_LEAKY_RELU:
        act_fargs = (0.1,)
        act_args = host.s32to8(0.1, 0)[:3]
    return dict(x=x, filt=filt, bias=bias, geom=g, out_offset=int(out_offset),
                in_offset=int(in_offset), f_offsets=f_offsets, b_offsets=b_offsets,
                bias_pre=bpre, bias_post=bpost, bias_scale=bscale, out_pre=opre,
                out_post=opost, out_scale=oscale, act=act, act_args=act_args,
                act_fargs=act_fargs, f_scales=f_scales,
                b_scales=np.asarray(b_scales, np.float32), in_scale_f=float(in_scale),
                out_scale_f=float(out_scale))


def zipf_indices(rng, n, rows, alpha):
    """n draws from a truncated Zipf(alpha) over `rows` ranks (inverse CDF of
    the continuous approximation), mapped to rows through a fixed odd-multiplier
    permutation so hot rows are scattered over the table."""
    u = rng.random(n)
    if abs(alpha - 1.0) < 1e-9:
        r = np.exp(u * np.log(rows + 1.0))
    else:
        a = 1.0 - alpha
        r = (u * ((rows + 1.0) ** a - 1.0) + 1.0) ** (1.0 / a)
    rank = np.minimum(np.floor(r).astype(np.int64) - 1, rows - 1)
    rank = np.maximum(rank, 0)
    return (rank * 2654435761 + 12345) % rows


def random_fused_table(rng, rows, cols, kind=U8_F32):
    """A fused-rowwise table filled directly with random codes and per-row
    (scale, offset), without materialising the fp32 source (which would be
    2.1 GB for 4M x 128)."""
    row_bytes = default_host().fused_row_bytes(cols, kind)
    data_bytes = cols if kind in (U8_F32, U8_F16) else cols // 2
    t = np.empty((rows, row_bytes), np.uint8)
    t[:, :data_bytes] = rng.integers(0, 256, (rows, data_bytes), dtype=np.uint8)
    div = 255.0 if kind in (U8_F32, U8_F16) else 15.0
    mn = rng.normal(-3.0, 0.5, rows).astype(np.float32)
    sc = (rng.uniform(4.0, 8.0, rows) / div).astype(np.float32)
    if kind in (U8_F32, U4_F32):
        t[:, data_bytes:data_bytes + 4] = sc.view(np.uint8).reshape(rows, 4)
        t[:, data_bytes + 4:] = mn.view(np.uint8).reshape(rows, 4)
    else:
        t[:, data_bytes:data_bytes + 2] = sc.astype(np.float16).view(np.uint8).reshape(rows, 2)
        t[:, data_bytes + 2:] = mn.astype(np.float16).view(np.uint8).reshape(rows, 2)
    return t


def slws_batch(seed, rows, bags, mean_len, alpha, idx_dtype=np.int64,
               weighted=True):
    rng = np.random.default_rng(seed)
    lengths = rng.poisson(mean_len, bags).astype(np.int32)
    total = int(lengths.sum())
    idx = zipf_indices(rng, total, rows, alpha).astype(idx_dtype)
    w = rng.random(total).astype(np.float32) if weighted else None
    return lengths, idx, w


def slws_error_ratio(got, want, table, w, idx, lengths):
    """max |got - want| / B over the output of a uint8/fp32 fused-rowwise SLWS,
    where B = sum_j |w_j| (|scale_j| 255 + |offset_j|) per bag is the magnitude
    of what the bag adds up (the result itself may cancel to nearly zero).
    Empty bags must be exact zeros (returns inf otherwise)."""
    total = int(lengths.sum())
    so = np.ascontiguousarray(table[:, -8:]).view(np.float32).astype(np.float64)
    r = np.asarray(idx[:total])
    ww = np.ones(total) if w is None else np.abs(np.asarray(w[:total], np.float64))
    m = ww * (np.abs(so[r, 0]) * 255.0 + np.abs(so[r, 1]))
    c = np.r_[0.0, np.cumsum(m)]
    ends = np.cumsum(lengths)
    mag = c[ends] - c[ends - lengths]
    err = np.abs(np.asarray(got, np.float64) - np.asarray(want, np.float64)).max(axis=1)
    if np.any(err[mag == 0] != 0):
        return float("inf")
    live = mag > 0
    return float(np.max(err[live] / mag[live])) if live.any() else 0.0

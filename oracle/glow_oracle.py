"""numpy-facing loader for ``libglow_oracle.so`` (the CPU restatement).

TEST INFRASTRUCTURE: the checker and the timed CPU baseline, never a product
code path. Every function forwards to the C function of the same name in
``glow_oracle.c``, which cites the reference lines it restates.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libglow_oracle.so")

ASYMMETRIC, SYMMETRIC, SYMMETRIC_WITH_UNSIGNED, SYMMETRIC_POW2 = 0, 1, 2, 3
U8_F32, U8_F16, U4_F16, U4_F32 = 0, 1, 2, 3
ACT_NONE, ACT_RELU, ACT_CLIP, ACT_TANH, ACT_SIGMOID, ACT_LEAKY_RELU = range(6)


def build(force=False):
    """Compile the restatement (and oracle/_ref when the reference is there)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "all"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


class ConvGeom(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "N", "IH", "IW", "IC", "OH", "OW", "OC", "KH", "KW", "strideH",
        "strideW", "padT", "padL", "dilH", "dilW", "group")]


def conv_geom(N, IH, IW, IC, OC, kernel, stride, pads, group=1, dilation=(1, 1)):
    """pads = (top, left, bottom, right). Output size as Glow computes it
    (calculateConvPoolOutputDims, include/glow/Graph/Nodes.h)."""
    KH, KW = kernel
    sh, sw = stride
    pt, pl, pb, pr = pads
    dh, dw = dilation
    OH = (IH + pt + pb - (KH - 1) * dh - 1) // sh + 1
    OW = (IW + pl + pr - (KW - 1) * dw - 1) // sw + 1
    return ConvGeom(N, IH, IW, IC, OH, OW, OC, KH, KW, sh, sw, pt, pl, dh, dw,
                    group)


_lib = None


def use_native_build():
    """Switches this module to a build of the same source for the host it runs
    on (-O3 -march=native, made here and now by the Makefile's `native`
    target): what the timed CPU baseline uses. Returns True when that build is
    in use, False when it could not be made (the portable build stays)."""
    global _lib, _LIB_PATH
    native = os.path.join(_HERE, "_native", "libglow_oracle_native.so")
    try:
        subprocess.check_call(["make", "-C", _HERE, "native"], stdout=subprocess.DEVNULL,
                              stderr=subprocess.DEVNULL)
    except (subprocess.CalledProcessError, OSError):
        return False
    if not os.path.exists(native):
        return False
    _LIB_PATH = native
    _lib = None
    return True


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.go_scale_i32.restype = C.c_int32
        _lib.go_scale_i32.argtypes = [C.c_int32] * 5
        _lib.go_clip_i8.restype = C.c_int8
        _lib.go_clip_i8.argtypes = [C.c_int32]
        _lib.go_f32_to_f16.restype = C.c_uint16
        _lib.go_f32_to_f16.argtypes = [C.c_float]
        _lib.go_f16_to_f32.restype = C.c_float
        _lib.go_f16_to_f32.argtypes = [C.c_uint16]
        _lib.go_quantize_value_i8.restype = C.c_int8
        _lib.go_quantize_value_i8.argtypes = [C.c_float, C.c_float, C.c_int32]
        _lib.go_quantize_value_i32.restype = C.c_int32
        _lib.go_quantize_value_i32.argtypes = [C.c_float, C.c_float, C.c_int32]
        _lib.go_fused_row_bytes.restype = C.c_size_t
        _lib.go_fused_row_bytes.argtypes = [C.c_size_t, C.c_int]
        _lib.go_activation_i32.restype = C.c_int32
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def _i32v(a):
    return _c(a, np.int32)


# ---- scalars ---------------------------------------------------------------

def scale_i32(x, pre, post, scale, offset):
    return lib().go_scale_i32(int(x), int(pre), int(post), int(scale), int(offset))


def clip_i8(v):
    return lib().go_clip_i8(int(v))


def activation_i32(x, offset, act, args=()):
    a = _i32v(list(args) + [0, 0, 0])
    return lib().go_activation_i32(C.c_int32(int(x)), C.c_int32(int(offset)),
                                   C.c_int32(int(act)), _p(a))


def f32_to_f16_bits(x):
    return lib().go_f32_to_f16(float(x))


def f16_bits_to_f32(h):
    return lib().go_f16_to_f32(int(h))


def quantize_scale_offset_32to8(scale, offset=0):
    """-> (pre, post, scale, offset)"""
    out = (C.c_int32 * 4)()
    lib().go_quantize_scale_offset_32to8(C.c_float(scale), C.c_int32(offset), out)
    return tuple(out)


def choose_qparams(mn, mx, schema=ASYMMETRIC, qty=8):
    s = C.c_float()
    o = C.c_int32()
    lib().go_choose_qparams(C.c_float(mn), C.c_float(mx), C.c_int(schema),
                            C.c_int(qty), C.byref(s), C.byref(o))
    return s.value, o.value


def specialize_bias_weights_qparams(bias_scale, bias_offset, input_scale,
                                    weights_scale, bias_is_i32=True,
                                    bias_zero=False):
    bs = C.c_float(bias_scale)
    bo = C.c_int32(bias_offset)
    ws = C.c_float(weights_scale)
    lib().go_specialize_bias_weights_qparams(
        C.byref(bs), C.byref(bo), C.c_float(input_scale), C.byref(ws),
        C.c_int(bias_is_i32), C.c_int(bias_zero))
    return bs.value, bo.value, ws.value


def specialize_bias_qparams(bias_scale, bias_offset, input_scale, weights_scale,
                            bias_is_i32=True, bias_zero=False):
    bs = C.c_float(bias_scale)
    bo = C.c_int32(bias_offset)
    lib().go_specialize_bias_qparams(C.byref(bs), C.byref(bo), C.c_float(input_scale),
                                     C.c_float(weights_scale), C.c_int(bias_is_i32),
                                     C.c_int(bias_zero))
    return bs.value, bo.value


def channelwise_quantize_conv(filter_f, bias_f, input_scale, schema=SYMMETRIC):
    f = _c(filter_f, np.float32)
    b = _c(bias_f, np.float32)
    oc = f.shape[0]
    per = f.size // max(oc, 1)
    fq = np.empty(f.shape, np.int8)
    bq = np.empty(oc, np.int32)
    fs, bs = np.empty(oc, np.float32), np.empty(oc, np.float32)
    fo, bo = np.empty(oc, np.int32), np.empty(oc, np.int32)
    lib().go_channelwise_quantize_conv(_p(f), _p(b), C.c_size_t(oc), C.c_size_t(per),
                                       C.c_float(input_scale), C.c_int(schema), _p(fq), _p(bq),
                                       _p(fs), _p(fo), _p(bs), _p(bo))
    return fq, bq, fs, fo, bs, bo


def quantize_value_i8(x, scale, offset):
    return lib().go_quantize_value_i8(x, scale, offset)


def quantize_value_i32(x, scale, offset):
    return lib().go_quantize_value_i32(x, scale, offset)


def rowwise_quantize_i8(w, schema=SYMMETRIC):
    w = _c(w, np.float32)
    rows, cols = w.shape
    q = np.empty((rows, cols), np.int8)
    s = np.empty(rows, np.float32)
    o = np.empty(rows, np.int32)
    lib().go_rowwise_quantize_i8(_p(w), C.c_size_t(rows), C.c_size_t(cols),
                                 C.c_int(schema), _p(q), _p(s), _p(o))
    return q, s, o


def fused_row_bytes(cols, kind):
    return lib().go_fused_row_bytes(cols, kind)


def fused_rowwise_quantize(x, kind):
    x = _c(x, np.float32)
    rows, cols = x.shape
    out = np.zeros((rows, fused_row_bytes(cols, kind)), np.uint8)
    lib().go_fused_rowwise_quantize(_p(x), C.c_size_t(rows), C.c_size_t(cols),
                                    C.c_int(kind), _p(out))
    return out


# ---- elementwise -----------------------------------------------------------

def quantize_i8(x, scale, offset):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.int8)
    lib().go_quantize_i8(_p(out), _p(x), C.c_size_t(x.size), C.c_float(scale),
                         C.c_int32(offset))
    return out


def dequantize_i8(q, scale, offset):
    q = _c(q, np.int8)
    out = np.empty(q.shape, np.float32)
    lib().go_dequantize_i8(_p(out), _p(q), C.c_size_t(q.size), C.c_float(scale),
                           C.c_int32(offset))
    return out


_WIDE = {16: np.int16, 32: np.int32}


def quantize_wide(x, scale, offset, bits):
    """Quantize to int16 (clipped) or int32 (not clipped)."""
    x = _c(x, np.float32)
    out = np.empty(x.shape, _WIDE[bits])
    getattr(lib(), f"go_quantize_i{bits}")(_p(out), _p(x), C.c_size_t(x.size), C.c_float(scale),
                                          C.c_int32(offset))
    return out


def dequantize_wide(q, scale, offset):
    q = np.ascontiguousarray(q)
    bits = {np.dtype(np.int16): 16, np.dtype(np.int32): 32}[q.dtype]
    out = np.empty(q.shape, np.float32)
    getattr(lib(), f"go_dequantize_i{bits}")(_p(out), _p(q), C.c_size_t(q.size), C.c_float(scale),
                                            C.c_int32(offset))
    return out


def rescale_wide(q, out_offset, in_offset, pre, post, scale):
    q = np.ascontiguousarray(q)
    bits = {np.dtype(np.int16): 16, np.dtype(np.int32): 32}[q.dtype]
    out = np.empty(q.shape, q.dtype)
    getattr(lib(), f"go_rescale_i{bits}")(_p(out), _p(q), C.c_size_t(q.size),
                                         C.c_int32(out_offset), C.c_int32(in_offset),
                                         C.c_int32(pre), C.c_int32(post), C.c_int32(scale))
    return out


def transpose(x, shuffle):
    """Transpose of up to six dimensions: output dimension d is input dimension
    shuffle[d] (numpy's x.transpose(shuffle))."""
    x = np.ascontiguousarray(x)
    nd = x.ndim
    assert nd <= 6 and sorted(shuffle) == list(range(nd))
    idim = (C.c_size_t * nd)(*x.shape)
    sh = (C.c_size_t * nd)(*shuffle)
    out = np.empty([x.shape[d] for d in shuffle], x.dtype)
    lib().go_transpose(_p(out), _p(x), idim, sh, C.c_size_t(nd), C.c_size_t(x.itemsize))
    return out


def rescale_i8(q, out_offset, in_offset, pre, post, scale):
    q = _c(q, np.int8)
    out = np.empty(q.shape, np.int8)
    lib().go_rescale_i8(_p(out), _p(q), C.c_size_t(q.size),
                        C.c_int32(out_offset), C.c_int32(in_offset),
                        C.c_int32(pre), C.c_int32(post), C.c_int32(scale))
    return out


# ---- FC / matmul -------------------------------------------------------------

def _bias(bias):
    bias = np.ascontiguousarray(bias)
    if bias.dtype == np.int8:
        return bias, 1
    return _c(bias, np.int32), 0


def fc_i8(x, w_kn, bias, out_offset, in_offset, w_offset, bias_offset, biasP,
          outP):
    """biasP/outP = (pre, post, scale)."""
    x = _c(x, np.int8)
    w_kn = _c(w_kn, np.int8)
    M, K = x.shape
    N = w_kn.shape[1]
    bias, b8 = _bias(bias)
    out = np.empty((M, N), np.int8)
    lib().go_fc_i8(_p(out), _p(x), _p(w_kn), _p(bias), C.c_int(b8),
                   C.c_size_t(M), C.c_size_t(K), C.c_size_t(N),
                   C.c_int32(out_offset), C.c_int32(in_offset),
                   C.c_int32(w_offset), C.c_int32(bias_offset),
                   *[C.c_int32(int(v)) for v in biasP],
                   *[C.c_int32(int(v)) for v in outP])
    return out


def rwq_fc_i8(x, w_nk, bias, w_offsets, bias_pre, bias_post, bias_scale,
              out_pre, out_post, out_scale, out_offset, in_offset, bias_offset):
    x = _c(x, np.int8)
    w_nk = _c(w_nk, np.int8)
    M, K = x.shape
    N = w_nk.shape[0]
    bias, b8 = _bias(bias)
    vs = [_i32v(v) for v in (w_offsets, bias_pre, bias_post, bias_scale,
                             out_pre, out_post, out_scale)]
    out = np.empty((M, N), np.int8)
    lib().go_rwq_fc_i8(_p(out), _p(x), _p(w_nk), _p(bias), C.c_int(b8),
                       *[_p(v) for v in vs], C.c_size_t(M), C.c_size_t(K),
                       C.c_size_t(N), C.c_int32(out_offset),
                       C.c_int32(in_offset), C.c_int32(bias_offset))
    return out


def matmul_i8(lhs, rhs, out_offset, lhs_offset, rhs_offset, outP):
    lhs = _c(lhs, np.int8)
    rhs = _c(rhs, np.int8)
    M, K = lhs.shape
    N = rhs.shape[1]
    out = np.empty((M, N), np.int8)
    lib().go_matmul_i8(_p(out), _p(lhs), _p(rhs), C.c_size_t(M), C.c_size_t(K),
                       C.c_size_t(N), C.c_int32(out_offset),
                       C.c_int32(lhs_offset), C.c_int32(rhs_offset),
                       *[C.c_int32(int(v)) for v in outP])
    return out


# ---- convolution -------------------------------------------------------------

def _act_args(args):
    return _i32v(list(args) + [0, 0, 0])


def conv2d_i8(x, filt, bias, geom, out_offset, in_offset, filter_offset,
              bias_offset, biasP, outP, act=ACT_NONE, act_args=()):
    x = _c(x, np.int8)
    filt = _c(filt, np.int8)
    bias, b8 = _bias(bias)
    out = np.empty((geom.N, geom.OH, geom.OW, geom.OC), np.int8)
    aa = _act_args(act_args)
    lib().go_conv2d_i8(_p(out), _p(x), _p(filt), _p(bias), C.c_int(b8),
                       C.byref(geom), C.c_int32(out_offset),
                       C.c_int32(in_offset), C.c_int32(filter_offset),
                       C.c_int32(bias_offset),
                       *[C.c_int32(int(v)) for v in biasP],
                       *[C.c_int32(int(v)) for v in outP], C.c_int32(act),
                       _p(aa))
    return out


def cwq_conv2d_i8(x, filt, bias, geom, out_offset, in_offset, filter_offsets,
                  bias_offsets, bias_pre, bias_post, bias_scale, out_pre,
                  out_post, out_scale, act=ACT_NONE, act_args=()):
    x = _c(x, np.int8)
    filt = _c(filt, np.int8)
    bias, b8 = _bias(bias)
    vs = [_i32v(v) for v in (filter_offsets, bias_offsets, bias_pre, bias_post,
                             bias_scale, out_pre, out_post, out_scale)]
    out = np.empty((geom.N, geom.OH, geom.OW, geom.OC), np.int8)
    aa = _act_args(act_args)
    lib().go_cwq_conv2d_i8(_p(out), _p(x), _p(filt), _p(bias), C.c_int(b8),
                           C.byref(geom), C.c_int32(out_offset),
                           C.c_int32(in_offset), *[_p(v) for v in vs],
                           C.c_int32(act), _p(aa))
    return out


class Conv3dGeom(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "N", "IT", "IH", "IW", "IC", "OT", "OH", "OW", "OC", "KT", "KH", "KW",
        "strideT", "strideH", "strideW", "padN", "padT", "padL", "group")]


def conv3d_geom(N, IT, IH, IW, IC, OC, kernel, stride, pads, group=1):
    """pads = (near, far, top, bottom, left, right). Output size as Glow computes
    it (calculate3DConvPoolOutputDims, include/glow/Graph/Nodes.h)."""
    KT, KH, KW = kernel
    st, sh, sw = stride
    pn, pf, pt, pb, pl, pr = pads
    OT = (IT + pn + pf - KT) // st + 1
    OH = (IH + pt + pb - KH) // sh + 1
    OW = (IW + pl + pr - KW) // sw + 1
    return Conv3dGeom(N, IT, IH, IW, IC, OT, OH, OW, OC, KT, KH, KW, st, sh, sw, pn, pt, pl,
                      group)


def cwq_conv3d_i8(x, filt, bias, geom, out_offset, in_offset, filter_offsets,
                  bias_offsets, bias_pre, bias_post, bias_scale, out_pre,
                  out_post, out_scale, act=ACT_NONE, act_args=()):
    x = _c(x, np.int8)
    filt = _c(filt, np.int8)
    bias, b8 = _bias(bias)
    vs = [_i32v(v) for v in (filter_offsets, bias_offsets, bias_pre, bias_post,
                             bias_scale, out_pre, out_post, out_scale)]
    out = np.empty((geom.N, geom.OT, geom.OH, geom.OW, geom.OC), np.int8)
    aa = _act_args(act_args)
    lib().go_cwq_conv3d_i8(_p(out), _p(x), _p(filt), _p(bias), C.c_int(b8),
                           C.byref(geom), C.c_int32(out_offset),
                           C.c_int32(in_offset), *[_p(v) for v in vs],
                           C.c_int32(act), _p(aa))
    return out


# ---- fused-rowwise SLWS ------------------------------------------------------

def _idx(indices):
    indices = np.ascontiguousarray(indices)
    if indices.dtype == np.int64:
        return indices, 1
    return _c(indices, np.int32), 0


def frwq_slws_f32(data, weights, indices, lengths, out_cols=None):
    data = _c(data, np.uint8)
    weights = _c(weights, np.float32)
    indices, i64 = _idx(indices)
    lengths = _i32v(lengths)
    in_line = data.shape[1]
    out_line = in_line - 8 if out_cols is None else out_cols
    out = np.empty((lengths.size, out_line), np.float32)
    lib().go_frwq_slws_f32(_p(out), _p(data), _p(weights), _p(indices),
                           C.c_int(i64), _p(lengths), C.c_size_t(lengths.size),
                           C.c_size_t(in_line), C.c_size_t(out_line))
    return out


def frwq_slws_generic(data, kind, weights, indices, lengths, out_f16=False,
                      fp16_accum=False):
    """weights: None (plain SLS), float32 array, or float16 array."""
    data = _c(data, np.uint8)
    indices, i64 = _idx(indices)
    lengths = _i32v(lengths)
    in_line = data.shape[1]
    so = 8 if kind in (U8_F32, U4_F32) else 4
    out_line = (in_line - so) * (2 if kind in (U4_F16, U4_F32) else 1)
    w16 = 0
    if weights is not None:
        weights = np.ascontiguousarray(weights)
        if weights.dtype == np.float16:
            w16 = 1
        else:
            weights = _c(weights, np.float32)
    out = np.empty((lengths.size, out_line),
                   np.float16 if out_f16 else np.float32)
    lib().go_frwq_slws_generic(_p(out), C.c_int(out_f16), _p(data),
                               C.c_int(kind), _p(weights), C.c_int(w16),
                               _p(indices), C.c_int(i64), _p(lengths),
                               C.c_size_t(lengths.size), C.c_size_t(in_line),
                               C.c_size_t(out_line), C.c_int(fp16_accum))
    return out


def embedding_bag_byte_rowwise_offsets_f32(data, weights, indices, offsets,
                                           has_end_offset):
    data = _c(data, np.uint8)
    weights = _c(weights, np.float32)
    indices = _i32v(indices)
    offsets = _i32v(offsets)
    in_line = data.shape[1]
    out_line = in_line - 8
    segs = offsets.size
    out = np.empty((segs - (1 if has_end_offset else 0), out_line), np.float32)
    lib().go_embedding_bag_byte_rowwise_offsets_f32(
        _p(out), _p(data), _p(weights), _p(indices), _p(offsets),
        C.c_size_t(segs), C.c_size_t(indices.size), C.c_size_t(in_line),
        C.c_size_t(out_line), C.c_int(has_end_offset))
    return out


# ---- int8 glue operators -----------------------------------------------------

def add_i8(lhs, rhs, dest_offset, lhs_offset, rhs_offset, lhsP, rhsP):
    """lhsP / rhsP = (pre, post, scale)."""
    lhs = _c(lhs, np.int8)
    rhs = _c(rhs, np.int8)
    out = np.empty(lhs.shape, np.int8)
    lib().go_add_i8(_p(out), _p(lhs), _p(rhs), C.c_size_t(lhs.size),
                    C.c_int32(dest_offset), C.c_int32(lhs_offset), C.c_int32(rhs_offset),
                    *[C.c_int32(int(v)) for v in lhsP], *[C.c_int32(int(v)) for v in rhsP])
    return out


def relu_i8(src, src_offset, dest_offset, destP):
    src = _c(src, np.int8)
    out = np.empty(src.shape, np.int8)
    lib().go_relu_i8(_p(out), _p(src), C.c_size_t(src.size), C.c_int8(src_offset),
                     C.c_int8(dest_offset), *[C.c_int32(int(v)) for v in destP])
    return out


def clip_elem_i8(src, clip_min, clip_max, src_offset, dest_offset, destP):
    """libjit_element_clip_i8 over a tensor."""
    src = _c(src, np.int8)
    out = np.empty(src.shape, np.int8)
    lib().go_clip_elem_i8(_p(out), _p(src), C.c_size_t(src.size), C.c_int8(clip_min),
                          C.c_int8(clip_max), C.c_int8(src_offset), C.c_int8(dest_offset),
                          *[C.c_int32(int(v)) for v in destP])
    return out


def leaky_relu_i8(src, src_offset, dest_offset, posP, negP):
    """libjit_element_leaky_relu_i8 over a tensor."""
    src = _c(src, np.int8)
    out = np.empty(src.shape, np.int8)
    lib().go_leaky_relu_i8(_p(out), _p(src), C.c_size_t(src.size), C.c_int8(src_offset),
                           C.c_int8(dest_offset), *[C.c_int32(int(v)) for v in posP],
                           *[C.c_int32(int(v)) for v in negP])
    return out


def max_splat_i8(src, value):
    """libjit_element_maxsplat_kernel_i8 over a tensor."""
    src = _c(src, np.int8)
    out = np.empty(src.shape, np.int8)
    lib().go_max_splat_i8(_p(out), _p(src), C.c_size_t(src.size), C.c_int8(value))
    return out


def batched_add_i8(batch, slice_, dest_offset, batch_offset, slice_offset, batchP, sliceP):
    """libjit_batchedadd_i8 (int8 slice) / libjit_batchedadd_i32_i8 (int32 slice):
    batch [numSlice x ...], slice [...]."""
    batch = _c(batch, np.int8)
    slice_ = np.ascontiguousarray(slice_)
    i32 = slice_.dtype == np.int32
    if not i32:
        slice_ = _c(slice_, np.int8)
    out = np.empty(batch.shape, np.int8)
    lib().go_batched_add_i8(_p(out), _p(batch), _p(slice_), C.c_int(int(i32)),
                            C.c_size_t(batch.shape[0]), C.c_size_t(slice_.size),
                            C.c_int32(dest_offset), C.c_int32(batch_offset),
                            C.c_int32(slice_offset), *[C.c_int32(int(v)) for v in batchP],
                            *[C.c_int32(int(v)) for v in sliceP])
    return out


def pool_out_dims(IH, IW, kernel, stride, pads):
    """pads = (top, left, bottom, right)."""
    OH = (IH + pads[0] + pads[2] - kernel[0]) // stride[0] + 1
    OW = (IW + pads[1] + pads[3] - kernel[1]) // stride[1] + 1
    return OH, OW


def _pool_args(x, kernel, stride, pads):
    N, IH, IW, Cn = x.shape
    OH, OW = pool_out_dims(IH, IW, kernel, stride, pads)
    out = np.empty((N, OH, OW, Cn), np.int8)
    sz = [C.c_size_t(int(v)) for v in (N, IH, IW, Cn, OH, OW, kernel[0], kernel[1],
                                       stride[0], stride[1], pads[0], pads[1])]
    return out, sz


def max_pool_i8(x, kernel, stride, pads, out_offset):
    x = _c(x, np.int8)
    out, sz = _pool_args(x, kernel, stride, pads)
    lib().go_max_pool_i8(_p(out), _p(x), *sz, C.c_int32(out_offset))
    return out


def avg_pool_i8(x, kernel, stride, pads, count_include_pads, out_offset, in_offset, outP):
    x = _c(x, np.int8)
    out, sz = _pool_args(x, kernel, stride, pads)
    lib().go_avg_pool_i8(_p(out), _p(x), *sz, C.c_int(int(count_include_pads)),
                         C.c_int32(out_offset), C.c_int32(in_offset),
                         *[C.c_int32(int(v)) for v in outP])
    return out


def softmax_f32(x):
    x = _c(x, np.float32)
    out = np.empty_like(x)
    lib().go_softmax_f32(_p(out), _p(x), C.c_size_t(x.shape[0]), C.c_size_t(x.shape[1]))
    return out


# ---- data movement and the small operators of ranking models -----------------

def sigmoid_f32(x):
    x = _c(x, np.float32)
    out = np.empty_like(x)
    lib().go_sigmoid_f32(_p(out), _p(x), C.c_size_t(x.size))
    return out


def gather(data, indices, batch_dims=0):
    data = np.ascontiguousarray(data)
    idx = _c(indices, np.int64)
    samples = data.shape[0] if batch_dims else 1
    inner = data.shape[batch_dims + 1:]
    slice_bytes = int(np.prod(inner, dtype=np.int64)) * data.dtype.itemsize
    sample_bytes = data.shape[batch_dims] * slice_bytes
    out = np.empty(data.shape[:batch_dims] + (idx.size,) + inner, data.dtype)
    lib().go_gather(_p(out), _p(data), _p(idx), C.c_size_t(idx.size), C.c_size_t(slice_bytes),
                    C.c_size_t(samples), C.c_size_t(sample_bytes))
    return out


def batch_matmul_i8(lhs, rhs, out_offset, lhs_offset, rhs_offset, outP):
    """BatchMatMul as it is lowered: libjit_matmul_i8 on every pair of the batch."""
    return np.stack([matmul_i8(lhs[b], rhs[b], out_offset, lhs_offset, rhs_offset, outP)
                     for b in range(lhs.shape[0])])


def rwq_slws_f32(data, scales, offsets, weights, indices, lengths):
    data = _c(data, np.uint8)
    scales, offsets, weights = _c(scales, np.float32), _c(offsets, np.float32), _c(weights, np.float32)
    indices, i64 = _idx(indices)
    lengths = _i32v(lengths)
    out = np.empty((lengths.size, data.shape[1]), np.float32)
    lib().go_rwq_slws_f32(_p(out), _p(data), _p(scales), _p(offsets), _p(weights), _p(indices),
                          C.c_int(i64), _p(lengths), C.c_size_t(lengths.size),
                          C.c_size_t(data.shape[1]))
    return out

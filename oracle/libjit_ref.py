"""ctypes access to oracle/_ref/libjit_ref*.so: the reference's own libjit
kernel sources compiled unmodified by oracle/Makefile (only where the
reference tree is mounted).

TEST INFRASTRUCTURE: used to validate the restatement in glow_oracle.c and to
write the golden vectors under tests/golden. Signatures follow
lib/LLVMIRCodeGen/libjit/libjit_matmul.cpp:395-450, libjit_conv.cpp:496-562,
libjit.cpp:2416-2481, 2998-3056 (dim_t is uint64_t, libjit_dim_t.h:37).
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))


def path(fastmath=False):
    """fastmath: False = plain build, True = the reference's default fast-math
    flags, "fma" = those flags on a host with fused multiply-add (-mfma)."""
    name = {False: "libjit_ref.so", True: "libjit_ref_fastmath.so",
            "fma": "libjit_ref_fma.so"}[fastmath]
    return os.path.join(_HERE, "_ref", name)


def available(fastmath=False):
    return os.path.exists(path(fastmath))


_libs = {}


def lib(fastmath=False):
    if fastmath not in _libs:
        l = C.CDLL(path(fastmath))
        l.libjit_element_quantize_kernel_i8.restype = C.c_int8
        l.libjit_element_quantize_kernel_i8.argtypes = [
            C.c_uint64, C.c_void_p, C.c_float, C.c_int32]
        l.libjit_element_dequantize_kernel_i8.restype = C.c_float
        l.libjit_element_dequantize_kernel_i8.argtypes = [
            C.c_uint64, C.c_void_p, C.c_float, C.c_int32]
        l.libjit_element_rescale_kernel_i8.restype = C.c_int8
        l.libjit_element_rescale_kernel_i8.argtypes = [
            C.c_uint64, C.c_void_p] + [C.c_int32] * 5
        for bits, ct in ((16, C.c_int16), (32, C.c_int32)):
            q = getattr(l, f"libjit_element_quantize_kernel_i{bits}")
            q.restype, q.argtypes = ct, [C.c_uint64, C.c_void_p, C.c_float, C.c_int32]
            d = getattr(l, f"libjit_element_dequantize_kernel_i{bits}")
            d.restype, d.argtypes = C.c_float, [C.c_uint64, C.c_void_p, C.c_float, C.c_int32]
            r = getattr(l, f"libjit_element_rescale_kernel_i{bits}")
            r.restype, r.argtypes = ct, [C.c_uint64, C.c_void_p] + [C.c_int32] * 5
        _libs[fastmath] = l
    return _libs[fastmath]


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def _dims(*d):
    return np.asarray(d, dtype=np.uint64)


def _i32v(a):
    return _c(a, np.int32)


def quantize_i8(x, scale, offset, fastmath=False):
    x = _c(x, np.float32).ravel()
    f = lib(fastmath).libjit_element_quantize_kernel_i8
    px = x.ctypes.data
    return np.array([f(i, px, scale, offset) for i in range(x.size)], np.int8)


def dequantize_i8(q, scale, offset, fastmath=False):
    q = _c(q, np.int8).ravel()
    f = lib(fastmath).libjit_element_dequantize_kernel_i8
    pq = q.ctypes.data
    return np.array([f(i, pq, scale, offset) for i in range(q.size)], np.float32)


def rescale_i8(q, out_offset, in_offset, pre, post, scale, fastmath=False):
    q = _c(q, np.int8).ravel()
    f = lib(fastmath).libjit_element_rescale_kernel_i8
    pq = q.ctypes.data
    return np.array([f(i, pq, out_offset, in_offset, pre, post, scale)
                     for i in range(q.size)], np.int8)


_WIDE = {16: np.int16, 32: np.int32}


def quantize_wide(x, scale, offset, bits, fastmath=False):
    x = _c(x, np.float32).ravel()
    f = getattr(lib(fastmath), f"libjit_element_quantize_kernel_i{bits}")
    px = x.ctypes.data
    return np.array([f(i, px, scale, offset) for i in range(x.size)], _WIDE[bits])


def dequantize_wide(q, scale, offset, fastmath=False):
    q = np.ascontiguousarray(q).ravel()
    f = getattr(lib(fastmath), f"libjit_element_dequantize_kernel_i{q.itemsize * 8}")
    pq = q.ctypes.data
    return np.array([f(i, pq, scale, offset) for i in range(q.size)], np.float32)


def rescale_wide(q, out_offset, in_offset, pre, post, scale, fastmath=False):
    q = np.ascontiguousarray(q).ravel()
    f = getattr(lib(fastmath), f"libjit_element_rescale_kernel_i{q.itemsize * 8}")
    pq = q.ctypes.data
    return np.array([f(i, pq, out_offset, in_offset, pre, post, scale)
                     for i in range(q.size)], q.dtype)


def transpose_i8(x, shuffle, fastmath=False):
    x = _c(x, np.int8)
    out = np.empty([x.shape[d] for d in shuffle], np.int8)
    lib(fastmath).libjit_transpose_i8(_p(x), _p(out), _p(_dims(*x.shape)), _p(_dims(*out.shape)),
                                      _p(_dims(*shuffle)), C.c_uint64(x.ndim))
    return out


def cwq_conv3d_i8(x, filt, bias, g, out_offset, in_offset, filter_offsets,
                  bias_offsets, bias_pre, bias_post, bias_scale, out_pre,
                  out_post, out_scale, act=0, act_args=(), fastmath=False):
    """g: the oracle's Conv3dGeom."""
    x = _c(x, np.int8)
    filt = _c(filt, np.int8)
    bias = np.ascontiguousarray(bias)
    out = np.empty((g.N, g.OT, g.OH, g.OW, g.OC), np.int8)
    od = _dims(g.N, g.OT, g.OH, g.OW, g.OC)
    idm = _dims(g.N, g.IT, g.IH, g.IW, g.IC)
    fd, bd = _dims(*filt.shape), _dims(g.OC)
    ks, st = _dims(g.KT, g.KH, g.KW), _dims(g.strideT, g.strideH, g.strideW)
    # the far / bottom / right pads are not read; the output dims carry them
    pd = _dims(g.padN, g.padN, g.padT, g.padT, g.padL, g.padL)
    dl = _dims(1, 1, 1)
    vs = [_i32v(v) for v in (filter_offsets, bias_offsets, bias_pre, bias_post,
                             bias_scale, out_pre, out_post, out_scale)]
    aa = _i32v(list(act_args) + [0, 0, 0])
    fn = (lib(fastmath).libjit_channelwise_quantized_conv3d_i8_i8
          if bias.dtype == np.int8
          else lib(fastmath).libjit_channelwise_quantized_conv3d_i8_i32)
    fn(_p(out), _p(x), _p(filt), _p(bias), _p(od), _p(idm), _p(fd), _p(bd),
       _p(ks), _p(st), _p(pd), C.c_uint64(g.group), _p(dl),
       C.c_int32(out_offset), C.c_int32(in_offset), *[_p(v) for v in vs],
       C.c_int32(act), _p(aa))
    return out


def fc_i8(x, w_kn, bias, out_offset, in_offset, w_offset, bias_offset, biasP,
          outP, fastmath=False):
    x = _c(x, np.int8)
    w_kn = _c(w_kn, np.int8)
    bias = np.ascontiguousarray(bias)
    M, K = x.shape
    N = w_kn.shape[1]
    out = np.empty((M, N), np.int8)
    fn = (lib(fastmath).libjit_fc_i8_i8 if bias.dtype == np.int8
          else lib(fastmath).libjit_fc_i8_i32)
    od, idm, wd, bd = _dims(M, N), _dims(M, K), _dims(K, N), _dims(N)
    fn(_p(out), _p(x), _p(w_kn), _p(bias), _p(od), _p(idm), _p(wd), _p(bd),
       C.c_int32(out_offset), C.c_int32(in_offset), C.c_int32(w_offset),
       C.c_int32(bias_offset), *[C.c_int32(int(v)) for v in biasP],
       *[C.c_int32(int(v)) for v in outP])
    return out


def rwq_fc_i8(x, w_nk, bias, w_offsets, bias_pre, bias_post, bias_scale,
              out_pre, out_post, out_scale, out_offset, in_offset, bias_offset,
              fastmath=False):
    x = _c(x, np.int8)
    w_nk = _c(w_nk, np.int8)
    bias = np.ascontiguousarray(bias)
    M, K = x.shape
    N = w_nk.shape[0]
    out = np.empty((M, N), np.int8)
    fn = (lib(fastmath).libjit_rowwise_quantized_fc_i8_i8
          if bias.dtype == np.int8
          else lib(fastmath).libjit_rowwise_quantized_fc_i8_i32)
    vs = [_i32v(v) for v in (w_offsets, bias_pre, bias_post, bias_scale,
                             out_pre, out_post, out_scale)]
    od, idm, wd, bd = _dims(M, N), _dims(M, K), _dims(N, K), _dims(N)
    fn(_p(out), _p(x), _p(w_nk), _p(bias), *[_p(v) for v in vs], _p(od),
       _p(idm), _p(wd), _p(bd), C.c_uint64(N), C.c_int32(out_offset),
       C.c_int32(in_offset), C.c_int32(bias_offset))
    return out


def matmul_i8(lhs, rhs, out_offset, lhs_offset, rhs_offset, outP,
              fastmath=False):
    lhs = _c(lhs, np.int8)
    rhs = _c(rhs, np.int8)
    M, K = lhs.shape
    N = rhs.shape[1]
    out = np.empty((M, N), np.int8)
    od, ld, rd = _dims(M, N), _dims(M, K), _dims(K, N)
    lib(fastmath).libjit_matmul_i8(
        _p(out), _p(lhs), _p(rhs), _p(od), _p(ld), _p(rd),
        C.c_int32(out_offset), C.c_int32(lhs_offset), C.c_int32(rhs_offset),
        *[C.c_int32(int(v)) for v in outP])
    return out


def _conv_dims(g, filt):
    od = _dims(g.N, g.OH, g.OW, g.OC)
    idm = _dims(g.N, g.IH, g.IW, g.IC)
    fd = _dims(*filt.shape)
    bd = _dims(g.OC)
    ks = _dims(g.KH, g.KW)
    st = _dims(g.strideH, g.strideW)
    # bottom / right pads are not read by the kernels; output dims carry them
    pd = _dims(g.padT, g.padL, g.padT, g.padL)
    dl = _dims(g.dilH, g.dilW)
    return od, idm, fd, bd, ks, st, pd, dl


def conv2d_i8(x, filt, bias, g, out_offset, in_offset, filter_offset,
              bias_offset, biasP, outP, act=0, act_args=(), depth_unroll=None,
              fastmath=False):
    x = _c(x, np.int8)
    filt = _c(filt, np.int8)
    bias = np.ascontiguousarray(bias)
    out = np.empty((g.N, g.OH, g.OW, g.OC), np.int8)
    od, idm, fd, bd, ks, st, pd, dl = _conv_dims(g, filt)
    if depth_unroll is None:  # LLVMIRGen.cpp:2527-2538
        depth_unroll = 8 if (g.OC // g.group) % 8 == 0 else 1
    aa = _i32v(list(act_args) + [0, 0, 0])
    fn = (lib(fastmath).libjit_conv2d_i8_i8 if bias.dtype == np.int8
          else lib(fastmath).libjit_conv2d_i8_i32)
    fn(_p(out), _p(x), _p(filt), _p(bias), _p(od), _p(idm), _p(fd), _p(bd),
       _p(ks), _p(st), _p(pd), C.c_uint64(g.group), C.c_int32(out_offset),
       C.c_int32(in_offset), C.c_int32(filter_offset), C.c_int32(bias_offset),
       *[C.c_int32(int(v)) for v in biasP], *[C.c_int32(int(v)) for v in outP],
       C.c_uint(depth_unroll), _p(dl), C.c_int32(act), _p(aa))
    return out


def cwq_conv2d_i8(x, filt, bias, g, out_offset, in_offset, filter_offsets,
                  bias_offsets, bias_pre, bias_post, bias_scale, out_pre,
                  out_post, out_scale, act=0, act_args=(), fastmath=False):
    x = _c(x, np.int8)
    filt = _c(filt, np.int8)
    bias = np.ascontiguousarray(bias)
    out = np.empty((g.N, g.OH, g.OW, g.OC), np.int8)
    od, idm, fd, bd, ks, st, pd, dl = _conv_dims(g, filt)
    vs = [_i32v(v) for v in (filter_offsets, bias_offsets, bias_pre, bias_post,
                             bias_scale, out_pre, out_post, out_scale)]
    aa = _i32v(list(act_args) + [0, 0, 0])
    fn = (lib(fastmath).libjit_channelwise_quantized_conv2d_i8_i8
          if bias.dtype == np.int8
          else lib(fastmath).libjit_channelwise_quantized_conv2d_i8_i32)
    fn(_p(out), _p(x), _p(filt), _p(bias), _p(od), _p(idm), _p(fd), _p(bd),
       _p(ks), _p(st), _p(pd), C.c_uint64(g.group), _p(dl),
       C.c_int32(out_offset), C.c_int32(in_offset), *[_p(v) for v in vs],
       C.c_int32(act), _p(aa))
    return out


def frwq_slws_f32(data, weights, indices, lengths, out_cols=None,
                  fastmath=False):
    data = _c(data, np.uint8)
    weights = _c(weights, np.float32)
    indices = np.ascontiguousarray(indices)
    lengths = _i32v(lengths)
    in_line = data.shape[1]
    out_line = in_line - 8 if out_cols is None else out_cols
    out = np.empty((lengths.size, out_line), np.float32)
    if indices.dtype == np.int64:
        fn = lib(fastmath).libjit_fused_rowwise_quantized_sparse_lengths_weighted_sum_f_u
    else:
        indices = _c(indices, np.int32)
        fn = lib(fastmath).libjit_fused_rowwise_quantized_sparse_lengths_weighted_sum_f_i32
    fn(_p(out), _p(data), _p(weights), _p(indices), _p(lengths),
       C.c_uint64(lengths.size), C.c_uint64(in_line), C.c_uint64(out_line))
    return out


def embedding_bag_byte_rowwise_offsets_f32(data, weights, indices, offsets,
                                           has_end_offset, fastmath=False):
    data = _c(data, np.uint8)
    weights = _c(weights, np.float32)
    indices = _i32v(indices)
    offsets = _i32v(offsets)
    in_line = data.shape[1]
    out_line = in_line - 8
    segs = offsets.size
    out = np.empty((segs - (1 if has_end_offset else 0), out_line), np.float32)
    lib(fastmath).libjit_embedding_bag_byte_rowwise_offsets_f(
        _p(out), _p(data), _p(weights), _p(indices), _p(offsets),
        C.c_uint64(segs), C.c_uint64(indices.size), C.c_uint64(in_line),
        C.c_uint64(out_line), C.c_bool(has_end_offset))
    return out


# ---- int8 glue operators (libjit.cpp:1593-1603, 1851-1858, 2592-2597, 2812-2880, 3058-3082) ----

def add_i8(lhs, rhs, dest_offset, lhs_offset, rhs_offset, lhsP, rhsP, fastmath=False):
    lhs = _c(lhs, np.int8).ravel()
    rhs = _c(rhs, np.int8).ravel()
    f = lib(fastmath).libjit_element_add_kernel_i8
    f.restype = C.c_int8
    f.argtypes = [C.c_uint64, C.c_void_p, C.c_void_p] + [C.c_int32] * 9
    pl, pr = lhs.ctypes.data, rhs.ctypes.data
    return np.array([f(i, pl, pr, dest_offset, lhs_offset, rhs_offset,
                       *[int(v) for v in lhsP], *[int(v) for v in rhsP])
                     for i in range(lhs.size)], np.int8)


def relu_i8(src, src_offset, dest_offset, destP, fastmath=False):
    src = _c(src, np.int8).ravel()
    f = lib(fastmath).libjit_element_relu_i8
    f.restype = C.c_int8
    f.argtypes = [C.c_uint64, C.c_void_p, C.c_int8, C.c_int8] + [C.c_int32] * 3
    ps = src.ctypes.data
    return np.array([f(i, ps, src_offset, dest_offset, *[int(v) for v in destP])
                     for i in range(src.size)], np.int8)


def clip_elem_i8(src, clip_min, clip_max, src_offset, dest_offset, destP, fastmath=False):
    src = _c(src, np.int8).ravel()
    f = lib(fastmath).libjit_element_clip_i8
    f.restype = C.c_int8
    f.argtypes = [C.c_uint64, C.c_void_p] + [C.c_int8] * 4 + [C.c_int32] * 3
    ps = src.ctypes.data
    return np.array([f(i, ps, clip_min, clip_max, src_offset, dest_offset,
                       *[int(v) for v in destP]) for i in range(src.size)], np.int8)


def leaky_relu_i8(src, src_offset, dest_offset, posP, negP, fastmath=False):
    src = _c(src, np.int8).ravel()
    f = lib(fastmath).libjit_element_leaky_relu_i8
    f.restype = C.c_int8
    f.argtypes = [C.c_uint64, C.c_void_p, C.c_int8, C.c_int8] + [C.c_int32] * 6
    ps = src.ctypes.data
    return np.array([f(i, ps, src_offset, dest_offset, *[int(v) for v in posP],
                       *[int(v) for v in negP]) for i in range(src.size)], np.int8)


def max_splat_i8(src, value, fastmath=False):
    """libjit_element_maxsplat_kernel_i8 of the CPU backend's own kernel file
    (lib/Backends/CPU/libjit_cpu/libjit_cpu.cpp)."""
    src = _c(src, np.int8).ravel()
    f = lib(fastmath).libjit_element_maxsplat_kernel_i8
    f.restype = C.c_int8
    f.argtypes = [C.c_uint64, C.c_int8, C.c_void_p, C.c_void_p]
    ps = src.ctypes.data
    return np.array([f(i, value, ps, None) for i in range(src.size)], np.int8)


def batched_add_i8(batch, slice_, dest_offset, batch_offset, slice_offset, batchP, sliceP,
                   fastmath=False):
    batch = _c(batch, np.int8)
    slice_ = np.ascontiguousarray(slice_)
    if slice_.dtype == np.int32:
        f = lib(fastmath).libjit_batchedadd_i32_i8
    else:
        slice_ = _c(slice_, np.int8)
        f = lib(fastmath).libjit_batchedadd_i8
    f.restype = None
    f.argtypes = [C.c_void_p] * 3 + [C.c_uint64] * 2 + [C.c_int32] * 9
    out = np.empty(batch.shape, np.int8)
    f(_p(out), _p(batch), _p(slice_), batch.shape[0], slice_.size, dest_offset, batch_offset,
      slice_offset, *[int(v) for v in batchP], *[int(v) for v in sliceP])
    return out


def _pool_dims(x, kernel, stride, pads):
    N, IH, IW, Cn = x.shape
    OH = (IH + pads[0] + pads[2] - kernel[0]) // stride[0] + 1
    OW = (IW + pads[1] + pads[3] - kernel[1]) // stride[1] + 1
    return (np.empty((N, OH, OW, Cn), np.int8), _dims(N, IH, IW, Cn), _dims(N, OH, OW, Cn),
            _dims(*kernel), _dims(*stride), _dims(*pads))


def max_pool_i8(x, kernel, stride, pads, out_offset, fastmath=False):
    x = _c(x, np.int8)
    out, idm, od, ks, st, pd = _pool_dims(x, kernel, stride, pads)
    lib(fastmath).libjit_max_pool_i8(_p(x), _p(out), _p(idm), _p(od), _p(ks), _p(st), _p(pd),
                                     C.c_int32(out_offset))
    return out


def avg_pool_i8(x, kernel, stride, pads, count_include_pads, out_offset, in_offset, outP,
                fastmath=False):
    x = _c(x, np.int8)
    out, idm, od, ks, st, pd = _pool_dims(x, kernel, stride, pads)
    lib(fastmath).libjit_avg_pool_i8(_p(x), _p(out), _p(idm), _p(od), _p(ks), _p(st), _p(pd),
                                     C.c_bool(bool(count_include_pads)), C.c_int32(out_offset),
                                     C.c_int32(in_offset), *[C.c_int32(int(v)) for v in outP])
    return out


def softmax_f32(x, fastmath=False):
    x = _c(x, np.float32)
    out = np.empty_like(x)
    d = _dims(*x.shape)
    lib(fastmath).libjit_softmax_f(_p(x), _p(out), _p(d), _p(d))
    return out


def sigmoid_f32(x, fastmath=False):
    x = _c(x, np.float32).ravel()
    f = lib(fastmath).libjit_sigmoid_kernel_f
    f.restype = C.c_float
    f.argtypes = [C.c_uint64, C.c_void_p, C.c_void_p, C.c_void_p]
    px = x.ctypes.data
    return np.array([f(i, px, None, None) for i in range(x.size)], np.float32)


def gather64_i8(data, indices, num_samples, sample_size, slice_size):
    data = _c(data, np.int8)
    idx = _c(indices, np.int64)
    out = np.empty(num_samples * idx.size * slice_size, np.int8)
    lib().libjit_gather64_i8(_p(out), _p(data), _p(idx), C.c_uint64(idx.size),
                             C.c_uint64(slice_size), C.c_uint64(num_samples),
                             C.c_uint64(sample_size))
    return out


def rwq_slws_f32(data, scales, offsets, weights, indices, lengths, fastmath=False):
    """libjit.cpp:2400-2414"""
    data = _c(data, np.uint8)
    scales, offsets, weights = _c(scales, np.float32), _c(offsets, np.float32), _c(weights, np.float32)
    indices = np.ascontiguousarray(indices)
    lengths = _i32v(lengths)
    out = np.empty((lengths.size, data.shape[1]), np.float32)
    fn = (lib(fastmath).libjit_rowwise_quantized_sparse_lengths_weighted_sum_f_u
          if indices.dtype == np.int64
          else lib(fastmath).libjit_rowwise_quantized_sparse_lengths_weighted_sum_f_i32)
    fn(_p(out), _p(data), _p(scales), _p(offsets), _p(weights), _p(indices), _p(lengths),
       C.c_uint64(lengths.size), C.c_uint64(data.shape[1]))
    return out

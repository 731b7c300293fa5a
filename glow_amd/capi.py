"""ctypes binding of libglow_mi355x.so (the C ABI in include/glow_mi355x.h)
plus thin numpy conveniences used by the tests, the smoke check and the
benchmark. There is no CPU fallback: if the library is missing or a call
fails, an exception is raised."""
import ctypes as C
import os

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libglow_mi355x.so")

FUSED_U8_F32, FUSED_U8_F16, FUSED_U4_F16, FUSED_U4_F32 = 0, 1, 2, 3
ACT_NONE, ACT_RELU, ACT_CLIP, ACT_TANH, ACT_SIGMOID, ACT_LEAKY_RELU = range(6)
SCHEMA_ASYMMETRIC, SCHEMA_SYMMETRIC, SCHEMA_SYMMETRIC_WITH_UNSIGNED, \
    SCHEMA_SYMMETRIC_POWER2 = range(4)
QTY_INT8, QTY_INT16, QTY_INT32, QTY_UINT8 = 8, 16, 32, 108
REGION_CONSTANTS, REGION_MUTABLE, REGION_ACTIVATIONS = 0, 1, 2

# Every symbol include/glow_mi355x.h declares (checked by the CPU test suite).
EXPORTS = [
    "mi355x_last_error", "mi355x_num_devices", "mi355x_init", "mi355x_rwq_fc_i8_opts", "mi355x_rwq_fc_relu_i8_opts", "mi355x_fc_i8_opts", "mi355x_matmul_i8_opts", "mi355x_cwq_conv2d_i8_opts", "mi355x_cwq_conv2d_add_i8_opts", "mi355x_conv2d_i8_opts", "mi355x_frwq_slws_opts", "mi355x_frwq_slws_offsets_opts", "mi355x_frwq_slws_noalloc_opts", "mi355x_frwq_sls_multi_opts", "mi355x_rwq_slws_opts", "mi355x_embedding_bag_rowwise_offsets_opts", "mi355x_frwq_slws_probe",
    "mi355x_device_info", "mi355x_malloc", "mi355x_free", "mi355x_host_alloc",
    "mi355x_host_free", "mi355x_memcpy_h2d", "mi355x_memcpy_d2h",
    "mi355x_memcpy_d2d", "mi355x_fill_u8", "mi355x_copy_u8", "mi355x_gemm_tile_override", "mi355x_gemm_splitk_workspace_bytes",
    "mi355x_cwq_conv2d_add_i8", "mi355x_frwq_sls_multi",
    "mi355x_specialize_bias_weights_qparams", "mi355x_rwq_slws", "mi355x_slws_set_fused_math", "mi355x_batch_matmul_nt_i8", "mi355x_batch_matmul_nt_select_i8", "mi355x_rwq_fc_relu_i8", "mi355x_add_i8", "mi355x_add_relu_i8",
    "mi355x_relu_i8", "mi355x_clip_i8", "mi355x_leaky_relu_i8", "mi355x_max_splat_i8", "mi355x_batched_add_i8", "mi355x_convert_f16_to_f32", "mi355x_insert_rows",
    "mi355x_batch_transpose_i8", "mi355x_space_to_depth2_i8", "mi355x_quantize_space_to_depth2_i8", "mi355x_gather", "mi355x_gather_rows", "mi355x_rescale_rows_i8",
    "mi355x_dequantize_sigmoid", "mi355x_batch_matmul_i8", "mi355x_sigmoid_f32",
    "mi355x_max_pool_i8", "mi355x_avg_pool_i8", "mi355x_softmax_f32", "mi355x_dequantize_softmax", "mi355x_stream_create",
    "mi355x_stream_destroy", "mi355x_stream_sync", "mi355x_device_sync",
    "mi355x_event_create", "mi355x_event_destroy", "mi355x_event_record", "mi355x_stream_wait_event",
    "mi355x_event_sync", "mi355x_event_elapsed_ms", "mi355x_arena_create",
    "mi355x_arena_destroy", "mi355x_arena_ptr", "mi355x_arena_upload",
    "mi355x_arena_download", "mi355x_arena_bytes",
    "mi355x_graph_begin_capture", "mi355x_graph_end_capture",
    "mi355x_graph_launch", "mi355x_graph_destroy",
    "mi355x_quantize_scale_offset_32to8", "mi355x_choose_quantization_params",
    "mi355x_fused_row_bytes", "mi355x_fused_rowwise_quantize_host",
    "mi355x_rowwise_quantize_i8_host", "mi355x_quantize_i8",
    "mi355x_dequantize_i8", "mi355x_rescale_i8", "mi355x_rowsum_i8",
    "mi355x_rwq_fc_i8",
    "mi355x_fc_i8", "mi355x_matmul_i8", "mi355x_transpose2d_i8",
    "mi355x_cwq_conv2d_i8", "mi355x_conv2d_i8", "mi355x_frwq_slws",
    "mi355x_embedding_bag_rowwise_offsets",
    "mi355x_slws_reserve_stream", "mi355x_frwq_slws_noalloc",
    "mi355x_frwq_slws_offsets", "mi355x_slws_bag_offsets_host",
    "mi355x_quantize_i16", "mi355x_quantize_i32", "mi355x_dequantize_i16",
    "mi355x_dequantize_i32", "mi355x_rescale_i16", "mi355x_rescale_i32",
    "mi355x_transpose_nd", "mi355x_cwq_conv3d_i8",
    "mi355x_shader_clock_probe", "mi355x_wall_clock_khz",
    "mi355x_specialize_bias_qparams", "mi355x_channelwise_quantize_conv_host",
    "mi355x_gemm_requant_hint", "mi355x_gemm_requant_hint_host",
]


class MI355XError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"mi355x status {code}: {msg}")
        self.code = code


class Info(C.Structure):
    _fields_ = [("name", C.c_char * 128), ("arch", C.c_char * 64),
                ("compute_units", C.c_int32), ("clock_khz", C.c_int32),
                ("total_memory", C.c_uint64), ("free_memory", C.c_uint64),
                ("device", C.c_int32), ("lds_bytes_per_block", C.c_int32)]


class ConvGeom(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "N", "IH", "IW", "IC", "OH", "OW", "OC", "KH", "KW", "strideH",
        "strideW", "padT", "padL", "dilH", "dilW", "group")]


class Conv3dGeom(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "N", "IT", "IH", "IW", "IC", "OT", "OH", "OW", "OC", "KT", "KH", "KW",
        "strideT", "strideH", "strideW", "padN", "padT", "padL", "group")]


def conv3d_geom(N, IT, IH, IW, IC, OC, kernel, stride, pads, group=1):
    """pads = (near, far, top, bottom, left, right); output extents as Glow
    computes them (include/glow/Graph/Nodes.h, calculate3DConvPoolOutputDims)."""
    KT, KH, KW = kernel
    st, sh, sw = stride
    pn, pf, pt, pb, pl, pr = pads
    return Conv3dGeom(N, IT, IH, IW, IC, (IT + pn + pf - KT) // st + 1,
                      (IH + pt + pb - KH) // sh + 1, (IW + pl + pr - KW) // sw + 1, OC,
                      KT, KH, KW, st, sh, sw, pn, pt, pl, group)


_lib = None


def lib():
    """The loaded library. Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise MI355XError(
                -4, f"{LIB_PATH} is not built (run __graft_entry__.build())")
        l = C.CDLL(LIB_PATH)
        l.mi355x_last_error.restype = C.c_char_p
        l.mi355x_fused_row_bytes.restype = C.c_size_t
        l.mi355x_fused_row_bytes.argtypes = [C.c_size_t, C.c_int]
        l.mi355x_arena_bytes.restype = C.c_uint64
        l.mi355x_arena_bytes.argtypes = [C.c_void_p]
        l.mi355x_quantize_scale_offset_32to8.restype = None
        _lib = l
    return _lib


def check(rc):
    if rc != 0:
        raise MI355XError(rc, lib().mi355x_last_error().decode())


def _vp(x):
    """void* from a DeviceBuffer / Stream / Event, an int address, a numpy
    array or None."""
    if x is None:
        return C.c_void_p(0)
    if isinstance(x, (DeviceBuffer, Stream, Event)):
        return C.c_void_p(x.ptr)
    if isinstance(x, np.ndarray):
        return C.c_void_p(x.ctypes.data)
    return C.c_void_p(int(x))


def _sz(v):
    return C.c_size_t(int(v))


def _i32(v):
    return C.c_int32(int(v))


# ---- device / memory ---------------------------------------------------------

_initialised = False


def init(device=0):
    global _initialised
    check(lib().mi355x_init(C.c_int(device)))
    _initialised = True


def num_devices():
    n = C.c_int(0)
    rc = lib().mi355x_num_devices(C.byref(n))
    return n.value if rc == 0 else 0


def device_info():
    info = Info()
    check(lib().mi355x_device_info(C.byref(info)))
    return info


def sync():
    check(lib().mi355x_device_sync())


class DeviceBuffer:
    """A device allocation that frees itself; `ptr` is the device address."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = C.c_void_p(0)
        check(lib().mi355x_malloc(C.byref(p), _sz(max(self.nbytes, 1))))
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a, stream=None):
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes)
        b.dtype, b.shape = a.dtype, a.shape
        if a.nbytes:
            check(lib().mi355x_memcpy_h2d(_vp(b.ptr), _vp(a), _sz(a.nbytes),
                                          _vp(stream)))
            check(lib().mi355x_stream_sync(_vp(stream)))
        return b

    @classmethod
    def empty(cls, shape, dtype):
        shape = tuple(int(s) for s in np.atleast_1d(shape))
        b = cls(int(np.prod(shape)) * np.dtype(dtype).itemsize)
        b.dtype, b.shape = np.dtype(dtype), shape
        return b

    def upload(self, a, stream=None):
        a = np.ascontiguousarray(a)
        assert a.nbytes <= self.nbytes
        check(lib().mi355x_memcpy_h2d(_vp(self.ptr), _vp(a), _sz(a.nbytes),
                                      _vp(stream)))
        check(lib().mi355x_stream_sync(_vp(stream)))

    def numpy(self, stream=None):
        out = np.empty(self.shape, self.dtype)
        if out.nbytes:
            check(lib().mi355x_memcpy_d2h(_vp(out), _vp(self.ptr),
                                          _sz(out.nbytes), _vp(stream)))
        check(lib().mi355x_stream_sync(_vp(stream)))
        return out

    def fill(self, value, stream=None):
        check(lib().mi355x_fill_u8(_vp(self.ptr), C.c_int(value),
                                   _sz(self.nbytes), _vp(stream)))

    def free(self):
        if self.ptr:
            lib().mi355x_free(_vp(self.ptr))
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def to_device(a):
    return DeviceBuffer.from_numpy(a)


class _Pinned:
    """Owner of one pinned host allocation (DeviceManager::allocateDeviceIOBuffer)."""

    def __init__(self, nbytes):
        p = C.c_void_p(0)
        check(lib().mi355x_host_alloc(C.byref(p), _sz(max(int(nbytes), 1))))
        self.ptr = p.value

    def __del__(self):
        try:
            if self.ptr:
                lib().mi355x_host_free(C.c_void_p(self.ptr))
                self.ptr = 0
        except Exception:
            pass


def pinned_empty(shape, dtype):
    """A numpy array in pinned host memory: copies to and from the device run at
    full PCIe rate and asynchronously. The memory lives as long as the array."""
    dtype = np.dtype(dtype)
    shape = tuple(int(s) for s in np.atleast_1d(shape))
    n = int(np.prod(shape, dtype=np.int64)) * dtype.itemsize
    owner = _Pinned(n)
    buf = (C.c_char * max(n, 1)).from_address(owner.ptr)
    arr = np.frombuffer(buf, dtype=dtype, count=n // dtype.itemsize).reshape(shape)
    _PINNED_OWNERS[id(buf)] = owner
    # the ctypes buffer is the array's base; tie the allocation's life to it
    import weakref
    weakref.finalize(buf, _PINNED_OWNERS.pop, id(buf), None)
    return arr


_PINNED_OWNERS = {}


def pinned_copy(a):
    out = pinned_empty(a.shape, a.dtype)
    out[...] = a
    return out


class Stream:
    def __init__(self):
        p = C.c_void_p(0)
        check(lib().mi355x_stream_create(C.byref(p)))
        self.ptr = p.value

    def sync(self):
        check(lib().mi355x_stream_sync(_vp(self.ptr)))

    def wait_event(self, event):
        """Work queued on this stream from here on starts after `event`."""
        check(lib().mi355x_stream_wait_event(_vp(self.ptr), _vp(event.ptr)))

    def __del__(self):
        try:
            if self.ptr:
                lib().mi355x_stream_destroy(_vp(self.ptr))
        except Exception:
            pass


class Event:
    def __init__(self):
        p = C.c_void_p(0)
        check(lib().mi355x_event_create(C.byref(p)))
        self.ptr = p.value

    def record(self, stream=None):
        check(lib().mi355x_event_record(_vp(self.ptr), _vp(stream)))

    def sync(self):
        check(lib().mi355x_event_sync(_vp(self.ptr)))

    def elapsed_ms(self, later):
        ms = C.c_float(0)
        check(lib().mi355x_event_elapsed_ms(_vp(self.ptr), _vp(later.ptr),
                                            C.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            if self.ptr:
                lib().mi355x_event_destroy(_vp(self.ptr))
        except Exception:
            pass


class Graph:
    """Records the launches issued on `stream` inside the `with` block and
    replays them with launch()."""

    def __init__(self, stream):
        self.stream = stream
        self.handle = 0

    def __enter__(self):
        check(lib().mi355x_graph_begin_capture(_vp(self.stream.ptr)))
        return self

    def __exit__(self, exc_type, exc, tb):
        p = C.c_void_p(0)
        rc = lib().mi355x_graph_end_capture(_vp(self.stream.ptr), C.byref(p))
        if exc_type is None:
            check(rc)
        self.handle = p.value or 0
        return False

    def launch(self, stream=None):
        s = stream if stream is not None else self.stream
        check(lib().mi355x_graph_launch(_vp(self.handle), _vp(s.ptr)))

    def destroy(self):
        if self.handle:
            check(lib().mi355x_graph_destroy(_vp(self.handle)))
            self.handle = 0

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class Arena:
    """constants | mutable | activations in one HBM allocation."""

    def __init__(self, const_bytes, mutable_bytes, activation_bytes):
        p = C.c_void_p(0)
        check(lib().mi355x_arena_create(_sz(const_bytes), _sz(mutable_bytes),
                                        _sz(activation_bytes), C.byref(p)))
        self.handle = p.value

    def ptr(self, region, offset):
        p = C.c_void_p(0)
        check(lib().mi355x_arena_ptr(_vp(self.handle), C.c_int(region),
                                     _sz(offset), C.byref(p)))
        return p.value

    def upload(self, region, offset, a, stream=None):
        a = np.ascontiguousarray(a)
        check(lib().mi355x_arena_upload(_vp(self.handle), C.c_int(region),
                                        _sz(offset), _vp(a), _sz(a.nbytes),
                                        _vp(stream)))
        check(lib().mi355x_stream_sync(_vp(stream)))

    def download(self, region, offset, shape, dtype, stream=None):
        out = np.empty(shape, dtype)
        check(lib().mi355x_arena_download(_vp(self.handle), C.c_int(region),
                                          _sz(offset), _vp(out),
                                          _sz(out.nbytes), _vp(stream)))
        check(lib().mi355x_stream_sync(_vp(stream)))
        return out

    @property
    def nbytes(self):
        return lib().mi355x_arena_bytes(_vp(self.handle))

    def destroy(self):
        if self.handle:
            check(lib().mi355x_arena_destroy(_vp(self.handle)))
            self.handle = 0

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


# ---- host-side parameter derivation ------------------------------------------

def quantize_scale_offset_32to8(scale, offset=0):
    out = (C.c_int32 * 4)()
    lib().mi355x_quantize_scale_offset_32to8(C.c_float(scale), _i32(offset), out)
    return tuple(out)


def choose_quantization_params(mn, mx, schema=SCHEMA_ASYMMETRIC, qty=QTY_INT8):
    s = C.c_float()
    o = C.c_int32()
    check(lib().mi355x_choose_quantization_params(
        C.c_float(mn), C.c_float(mx), C.c_int(schema), C.c_int(qty),
        C.byref(s), C.byref(o)))
    return s.value, o.value


def specialize_bias_weights_qparams(bias_scale, bias_offset, input_scale, weights_scale,
                                    bias_is_i32=True, bias_is_zero=False):
    """-> (bias_scale, bias_offset, weights_scale)."""
    bs, bo, ws = C.c_float(bias_scale), C.c_int32(bias_offset), C.c_float(weights_scale)
    check(lib().mi355x_specialize_bias_weights_qparams(
        C.byref(bs), C.byref(bo), C.c_float(input_scale), C.byref(ws),
        C.c_int(int(bias_is_i32)), C.c_int(int(bias_is_zero))))
    return bs.value, bo.value, ws.value


def specialize_bias_qparams(bias_scale, bias_offset, input_scale, weights_scale,
                            bias_is_i32=True, bias_is_zero=False):
    """specializeBiasQuantizationParams -> (bias_scale, bias_offset)."""
    bs, bo = C.c_float(bias_scale), C.c_int32(bias_offset)
    check(lib().mi355x_specialize_bias_qparams(
        C.byref(bs), C.byref(bo), C.c_float(input_scale), C.c_float(weights_scale),
        C.c_int(bool(bias_is_i32)), C.c_int(bool(bias_is_zero))))
    return bs.value, bo.value


def channelwise_quantize_conv_host(filter_f, bias_f, input_scale, schema=SCHEMA_SYMMETRIC):
    """createChannelwiseQuantizedConv's constants for a float filter [OC, ...] and
    float bias [OC] -> (filter_q int8, bias_q int32, filter_scales, filter_offsets,
    bias_scales, bias_offsets)."""
    f = np.ascontiguousarray(filter_f, np.float32)
    b = np.ascontiguousarray(bias_f, np.float32)
    oc = f.shape[0]
    per = f.size // max(oc, 1)
    fq = np.empty(f.shape, np.int8)
    bq = np.empty(oc, np.int32)
    fs, bs = np.empty(oc, np.float32), np.empty(oc, np.float32)
    fo, bo = np.empty(oc, np.int32), np.empty(oc, np.int32)
    check(lib().mi355x_channelwise_quantize_conv_host(
        _vp(f), _vp(b), _sz(oc), _sz(per), C.c_float(input_scale), C.c_int(schema),
        _vp(fq), _vp(bq), _vp(fs), _vp(fo), _vp(bs), _vp(bo)))
    return fq, bq, fs, fo, bs, bo


def gemm_requant_hint_host(K, in_offset, out_offset, w_offsets, bias, bias_offset, bias_pre,
                           bias_post, bias_scale, out_pre, out_post, out_scale,
                           bias_offsets=None):
    """Requantisation hint flags for a launch with these (host) parameter
    vectors; `bias_offset` scalar or `bias_offsets` per column."""
    N = len(out_pre)
    i32 = lambda v: None if v is None else np.ascontiguousarray(v, np.int32)
    vs = [i32(v) for v in (w_offsets, bias_offsets, bias_pre, bias_post, bias_scale,
                           out_pre, out_post, out_scale)]
    b8 = 0
    if bias is not None:
        bias = np.ascontiguousarray(bias)
        b8 = int(bias.dtype == np.int8)
        if not b8:
            bias = bias.astype(np.int32)
    flags = C.c_int(0)
    check(lib().mi355x_gemm_requant_hint_host(
        _sz(K), _sz(N), _i32(in_offset), _i32(out_offset), _vp(vs[0]), _vp(bias), C.c_int(b8),
        _vp(vs[1]), _i32(bias_offset), _vp(vs[2]), _vp(vs[3]), _vp(vs[4]), _vp(vs[5]),
        _vp(vs[6]), _vp(vs[7]), C.byref(flags)))
    return flags.value


class requant_hint:
    """with requant_hint(flags): ... applies the hint to the launches inside."""

    def __init__(self, flags):
        self.flags = int(flags)

    def __enter__(self):
        check(lib().mi355x_gemm_requant_hint(self.flags))

    def __exit__(self, *exc):
        check(lib().mi355x_gemm_requant_hint(0))
        return False


def fused_row_bytes(cols, kind):
    return lib().mi355x_fused_row_bytes(cols, kind)


def fused_rowwise_quantize_host(x, kind):
    x = np.ascontiguousarray(x, np.float32)
    rows, cols = x.shape
    out = np.zeros((rows, fused_row_bytes(cols, kind)), np.uint8)
    check(lib().mi355x_fused_rowwise_quantize_host(
        _vp(x), _sz(rows), _sz(cols), C.c_int(kind), _vp(out)))
    return out


def rowwise_quantize_i8_host(w, schema=SCHEMA_SYMMETRIC):
    w = np.ascontiguousarray(w, np.float32)
    rows, cols = w.shape
    q = np.empty((rows, cols), np.int8)
    s = np.empty(rows, np.float32)
    o = np.empty(rows, np.int32)
    check(lib().mi355x_rowwise_quantize_i8_host(
        _vp(w), _sz(rows), _sz(cols), C.c_int(schema), _vp(q), _vp(s), _vp(o)))
    return q, s, o


# ---- raw launches on device buffers (used by the benchmark) --------------------

def launch_quantize_i8(dst, src, n, scale, offset, stream=None):
    check(lib().mi355x_quantize_i8(_vp(dst), _vp(src), _sz(n), C.c_float(scale),
                                   _i32(offset), _vp(stream)))


def launch_dequantize_i8(dst, src, n, scale, offset, stream=None):
    check(lib().mi355x_dequantize_i8(_vp(dst), _vp(src), _sz(n),
                                     C.c_float(scale), _i32(offset),
                                     _vp(stream)))


def launch_rescale_i8(dst, src, n, out_offset, in_offset, pre, post, scale,
                      stream=None):
    check(lib().mi355x_rescale_i8(_vp(dst), _vp(src), _sz(n), _i32(out_offset),
                                  _i32(in_offset), _i32(pre), _i32(post),
                                  _i32(scale), _vp(stream)))


def launch_copy_u8(dst, src, nbytes, stream=None):
    check(lib().mi355x_copy_u8(_vp(dst), _vp(src), _sz(nbytes), _vp(stream)))


def launch_rowsum_i8(sums, rows, n_rows, K, stream=None):
    check(lib().mi355x_rowsum_i8(_vp(sums), _vp(rows), _sz(n_rows), _sz(K),
                                 _vp(stream)))


SLWS_MATH_STRICT, SLWS_MATH_ELEMENT, SLWS_MATH_REGROUPED = 0, 1, 2


class LaunchOpts(C.Structure):
    """mi355x_launch_opts: options that hold for one call of an <entry>_opts
    entry point (workgroup tile, requantisation hint, SparseLengths
    arithmetic)."""
    _fields_ = [("struct_size", C.c_uint32), ("gemm_tile", C.c_int32),
                ("requant_hint", C.c_int32), ("slws_math", C.c_int32),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_uint64)]

    def __init__(self, gemm_tile=-1, requant_hint=0, slws_math=-1, workspace=None):
        """workspace: a zero-filled DeviceBuffer for launches that split K over
        workgroups (gemm_splitk_workspace_bytes), or None."""
        super().__init__(C.sizeof(LaunchOpts), gemm_tile, requant_hint, slws_math,
                         workspace.ptr if workspace is not None else None,
                         workspace.nbytes if workspace is not None else 0)
        self._keep = workspace


TILE_SPLIT_K = 12


def gemm_splitk_workspace_bytes(M, N, K, groups=1, named=False):
    """Bytes of workspace a K-split launch of this product uses (0: none)."""
    n = C.c_size_t(0)
    check(lib().mi355x_gemm_splitk_workspace_bytes(_sz(M), _sz(N), _sz(K), _sz(groups),
                                                   C.c_int(int(named)), C.byref(n)))
    return n.value


def _entry(name, opts):
    """(function, trailing arguments) of entry point `name`: its _opts twin when
    options are given."""
    if opts is None:
        return getattr(lib(), name), ()
    return getattr(lib(), name + "_opts"), (C.byref(opts),)


def launch_rwq_fc_i8(out, x, w, bias, bias_is_i8, w_offsets, bias_pre,
                     bias_post, bias_scale, out_pre, out_post, out_scale, M, K,
                     N, out_offset, in_offset, bias_offset,
                     w_offsets_all_zero=False, w_row_sums=None, stream=None, opts=None):
    fn, tail = _entry("mi355x_rwq_fc_i8", opts)
    check(fn(
        _vp(out), _vp(x), _vp(w), _vp(bias), C.c_int(bias_is_i8),
        _vp(w_offsets), _vp(bias_pre), _vp(bias_post), _vp(bias_scale),
        _vp(out_pre), _vp(out_post), _vp(out_scale), _sz(M), _sz(K), _sz(N),
        _i32(out_offset), _i32(in_offset), _i32(bias_offset),
        C.c_int(bool(w_offsets_all_zero)), _vp(w_row_sums), _vp(stream), *tail))


def launch_cwq_conv2d_i8(out, x, filt, bias, bias_is_i8, geom, out_offset,
                         in_offset, f_offsets, b_offsets, bias_pre, bias_post,
                         bias_scale, out_pre, out_post, out_scale, act,
                         act_args, f_offsets_all_zero=False, f_row_sums=None,
                         stream=None, opts=None):
    aa = (C.c_int32 * 3)(*(list(act_args) + [0, 0, 0])[:3])
    fn, tail = _entry("mi355x_cwq_conv2d_i8", opts)
    check(fn(
        _vp(out), _vp(x), _vp(filt), _vp(bias), C.c_int(bias_is_i8),
        C.byref(geom), _i32(out_offset), _i32(in_offset), _vp(f_offsets),
        _vp(b_offsets), _vp(bias_pre), _vp(bias_post), _vp(bias_scale),
        _vp(out_pre), _vp(out_post), _vp(out_scale), _i32(act), aa,
        C.c_int(bool(f_offsets_all_zero)), _vp(f_row_sums), _vp(stream), *tail))


class FusedAdd(C.Structure):
    """mi355x_fused_add: the ElementAdd (+ Relu) behind a convolution."""
    _fields_ = [(n, C.c_int32) for n in (
        "sum_offset", "residual_offset", "conv_pre", "conv_post", "conv_scale",
        "residual_pre", "residual_post", "residual_scale", "relu", "dest_offset",
        "dest_pre", "dest_post", "dest_scale")]


def fused_add(sum_offset, residual_offset, convP, resP, relu=False, dest_offset=0,
              destP=(0, 0, 1)):
    return FusedAdd(sum_offset, residual_offset, *[int(v) for v in convP],
                    *[int(v) for v in resP], int(bool(relu)), dest_offset,
                    *[int(v) for v in destP])


def launch_cwq_conv2d_add_i8(out, x, filt, bias, bias_is_i8, geom, conv_offset,
                             in_offset, f_offsets, b_offsets, bias_pre, bias_post,
                             bias_scale, out_pre, out_post, out_scale, act,
                             act_args, f_offsets_all_zero, f_row_sums, residual,
                             add, stream=None):
    aa = (C.c_int32 * 3)(*(list(act_args) + [0, 0, 0])[:3])
    check(lib().mi355x_cwq_conv2d_add_i8(
        _vp(out), _vp(x), _vp(filt), _vp(bias), C.c_int(bias_is_i8),
        C.byref(geom), _i32(conv_offset), _i32(in_offset), _vp(f_offsets),
        _vp(b_offsets), _vp(bias_pre), _vp(bias_post), _vp(bias_scale),
        _vp(out_pre), _vp(out_post), _vp(out_scale), _i32(act), aa,
        C.c_int(bool(f_offsets_all_zero)), _vp(f_row_sums), _vp(residual),
        C.byref(add), _vp(stream)))


def launch_frwq_slws(dest, out_is_f16, data, data_rows, kind, weights,
                     weights_are_f16, indices, idx_is_64, num_indices, lengths,
                     segments, in_line, out_line, fp16_accum=False,
                     stream=None, noalloc=False, opts=None):
    """noalloc: through mi355x_frwq_slws_noalloc (scratch in the library's fixed
    device array) instead of mi355x_frwq_slws (per-stream scratch)."""
    fn, tail = _entry("mi355x_frwq_slws_noalloc" if noalloc else "mi355x_frwq_slws", opts)
    check(fn(
        _vp(dest), C.c_int(bool(out_is_f16)), _vp(data), _sz(data_rows),
        C.c_int(kind), _vp(weights), C.c_int(bool(weights_are_f16)),
        _vp(indices), C.c_int(bool(idx_is_64)), _sz(num_indices), _vp(lengths),
        _sz(segments), _sz(in_line), _sz(out_line), C.c_int(bool(fp16_accum)),
        _vp(stream), *tail))


def launch_frwq_slws_offsets(dest, out_is_f16, data, data_rows, kind, weights,
                             weights_are_f16, indices, idx_is_64, num_indices,
                             bag_offsets, segments, in_line, out_line, fp16_accum=False,
                             stream=None, opts=None):
    """mi355x_frwq_slws_offsets: bags by their segments + 1 positions."""
    fn, tail = _entry("mi355x_frwq_slws_offsets", opts)
    check(fn(
        _vp(dest), C.c_int(bool(out_is_f16)), _vp(data), _sz(data_rows),
        C.c_int(kind), _vp(weights), C.c_int(bool(weights_are_f16)),
        _vp(indices), C.c_int(bool(idx_is_64)), _sz(num_indices), _vp(bag_offsets),
        _sz(segments), _sz(in_line), _sz(out_line), C.c_int(bool(fp16_accum)),
        _vp(stream), *tail))


def slws_bag_offsets_host(lengths):
    """Exclusive prefix sums (segments + 1 int32) of the clamped lengths, made
    by the library on the host."""
    lengths = np.ascontiguousarray(lengths, np.int32)
    out = np.empty(lengths.size + 1, np.int32)
    check(lib().mi355x_slws_bag_offsets_host(_vp(lengths), _sz(lengths.size), _vp(out)))
    return out


# ---- numpy in / numpy out conveniences (tests, smoke) --------------------------

def _geom(g):
    """Accepts this module's ConvGeom or any ctypes struct with the same
    fields (the oracle's)."""
    if isinstance(g, ConvGeom):
        return g
    return ConvGeom(*[getattr(g, n) for n, _ in ConvGeom._fields_])


def quantize_i8(x, scale, offset):
    x = np.ascontiguousarray(x, np.float32)
    d_in = to_device(x)
    d_out = DeviceBuffer.empty(x.shape, np.int8)
    launch_quantize_i8(d_out, d_in, x.size, scale, offset)
    return d_out.numpy()


def dequantize_i8(q, scale, offset):
    q = np.ascontiguousarray(q, np.int8)
    d_in = to_device(q)
    d_out = DeviceBuffer.empty(q.shape, np.float32)
    launch_dequantize_i8(d_out, d_in, q.size, scale, offset)
    return d_out.numpy()


def rescale_i8(q, out_offset, in_offset, pre, post, scale):
    q = np.ascontiguousarray(q, np.int8)
    d_in = to_device(q)
    d_out = DeviceBuffer.empty(q.shape, np.int8)
    launch_rescale_i8(d_out, d_in, q.size, out_offset, in_offset, pre, post,
                      scale)
    return d_out.numpy()


def _dev_i32(v):
    return to_device(np.ascontiguousarray(v, np.int32))


def _bias_dev(bias):
    bias = np.ascontiguousarray(bias)
    if bias.dtype == np.int8:
        return to_device(bias), 1
    return to_device(bias.astype(np.int32)), 0


def rowsum_i8(rows):
    rows = np.ascontiguousarray(rows, np.int8)
    n, K = rows.shape[0], int(np.prod(rows.shape[1:]))
    d_rows = to_device(rows)
    d_sums = DeviceBuffer.empty((n,), np.int32)
    launch_rowsum_i8(d_sums, d_rows, n, K)
    return d_sums.numpy()


def _row_sums_dev(d_rows, n, K, wanted):
    """Device vector of weight row sums when `wanted`, else None (the kernel
    then forms them itself)."""
    if not wanted:
        return None
    d_sums = DeviceBuffer.empty((n,), np.int32)
    launch_rowsum_i8(d_sums, d_rows, n, K)
    return d_sums


def rwq_fc_i8(x, w_nk, bias, w_offsets, bias_pre, bias_post, bias_scale,
              out_pre, out_post, out_scale, out_offset, in_offset, bias_offset,
              w_offsets_all_zero=None, precomputed_sums=True, opts=None):
    x = np.ascontiguousarray(x, np.int8)
    w_nk = np.ascontiguousarray(w_nk, np.int8)
    M, K = x.shape
    N = w_nk.shape[0]
    if w_offsets_all_zero is None:
        w_offsets_all_zero = not np.any(w_offsets)
    d_x, d_w = to_device(x), to_device(w_nk)
    d_b, b8 = _bias_dev(bias)
    vs = [_dev_i32(v) for v in (w_offsets, bias_pre, bias_post, bias_scale,
                                out_pre, out_post, out_scale)]
    d_out = DeviceBuffer.empty((M, N), np.int8)
    d_sums = _row_sums_dev(d_w, N, K, precomputed_sums)
    launch_rwq_fc_i8(d_out, d_x, d_w, d_b, b8, *vs, M, K, N, out_offset,
                     in_offset, bias_offset, w_offsets_all_zero, d_sums, opts=opts)
    return d_out.numpy()


def rwq_fc_relu_i8(x, w_nk, bias, w_offsets, bias_pre, bias_post, bias_scale,
                   out_pre, out_post, out_scale, fc_offset, in_offset, bias_offset,
                   relu_offset, reluP, w_offsets_all_zero=None, precomputed_sums=True):
    """RowwiseQuantizedFullyConnected + Relu in one kernel; reluP = (pre, post, scale)."""
    x = np.ascontiguousarray(x, np.int8)
    w_nk = np.ascontiguousarray(w_nk, np.int8)
    M, K = x.shape
    N = w_nk.shape[0]
    if w_offsets_all_zero is None:
        w_offsets_all_zero = not np.any(w_offsets)
    d_x, d_w = to_device(x), to_device(w_nk)
    d_b, b8 = _bias_dev(bias)
    vs = [_dev_i32(v) for v in (w_offsets, bias_pre, bias_post, bias_scale,
                                out_pre, out_post, out_scale)]
    d_out = DeviceBuffer.empty((M, N), np.int8)
    d_sums = _row_sums_dev(d_w, N, K, precomputed_sums)
    check(lib().mi355x_rwq_fc_relu_i8(
        _vp(d_out), _vp(d_x), _vp(d_w), _vp(d_b), C.c_int(b8), *[_vp(v) for v in vs],
        _sz(M), _sz(K), _sz(N), _i32(fc_offset), _i32(in_offset), _i32(bias_offset),
        C.c_int(bool(w_offsets_all_zero)), _vp(d_sums), _i32(relu_offset), *_i32s(reluP),
        _vp(None)))
    return d_out.numpy()


def fc_i8(x, w_kn, bias, out_offset, in_offset, w_offset, bias_offset, biasP,
          outP, precomputed_sums=False):
    x = np.ascontiguousarray(x, np.int8)
    w_kn = np.ascontiguousarray(w_kn, np.int8)
    M, K = x.shape
    N = w_kn.shape[1]
    d_x, d_w = to_device(x), to_device(w_kn)
    d_ws = DeviceBuffer.empty((N, K), np.int8)
    d_b, b8 = _bias_dev(bias)
    d_out = DeviceBuffer.empty((M, N), np.int8)
    repack, d_sums = 1, None
    if precomputed_sums:  # what a backend does once at load time
        check(lib().mi355x_transpose2d_i8(_vp(d_ws), _vp(d_w), _sz(K), _sz(N),
                                          _vp(None)))
        d_sums = _row_sums_dev(d_ws, N, K, True)
        repack = 0
    check(lib().mi355x_fc_i8(
        _vp(d_out), _vp(d_x), _vp(d_w), _vp(d_ws), C.c_int(repack), _vp(d_b),
        C.c_int(b8), _sz(M), _sz(K), _sz(N), _i32(out_offset), _i32(in_offset),
        _i32(w_offset), _i32(bias_offset), *[_i32(v) for v in biasP],
        *[_i32(v) for v in outP], _vp(d_sums), _vp(None)))
    return d_out.numpy()


def matmul_i8(lhs, rhs_kn, out_offset, lhs_offset, rhs_offset, outP):
    lhs = np.ascontiguousarray(lhs, np.int8)
    rhs_kn = np.ascontiguousarray(rhs_kn, np.int8)
    M, K = lhs.shape
    N = rhs_kn.shape[1]
    d_l, d_r = to_device(lhs), to_device(rhs_kn)
    d_ws = DeviceBuffer.empty((N, K), np.int8)
    d_out = DeviceBuffer.empty((M, N), np.int8)
    check(lib().mi355x_matmul_i8(
        _vp(d_out), _vp(d_l), _vp(d_r), _vp(d_ws), C.c_int(1), _sz(M), _sz(K),
        _sz(N), _i32(out_offset), _i32(lhs_offset), _i32(rhs_offset),
        *[_i32(v) for v in outP], _vp(None)))
    return d_out.numpy()


def transpose2d_i8(a):
    a = np.ascontiguousarray(a, np.int8)
    d_a = to_device(a)
    d_o = DeviceBuffer.empty((a.shape[1], a.shape[0]), np.int8)
    check(lib().mi355x_transpose2d_i8(_vp(d_o), _vp(d_a), _sz(a.shape[0]),
                                      _sz(a.shape[1]), _vp(None)))
    return d_o.numpy()


def cwq_conv2d_i8(x, filt, bias, geom, out_offset, in_offset, f_offsets,
                  b_offsets, bias_pre, bias_post, bias_scale, out_pre, out_post,
                  out_scale, act=ACT_NONE, act_args=(), f_offsets_all_zero=None,
                  precomputed_sums=True, opts=None):
    g = _geom(geom)
    x = np.ascontiguousarray(x, np.int8)
    filt = np.ascontiguousarray(filt, np.int8)
    if f_offsets_all_zero is None:
        f_offsets_all_zero = not np.any(f_offsets)
    d_x, d_f = to_device(x), to_device(filt)
    d_b, b8 = _bias_dev(bias)
    vs = [_dev_i32(v) for v in (f_offsets, b_offsets, bias_pre, bias_post,
                                bias_scale, out_pre, out_post, out_scale)]
    d_out = DeviceBuffer.empty((g.N, g.OH, g.OW, g.OC), np.int8)
    d_sums = _row_sums_dev(d_f, g.OC, filt.size // g.OC, precomputed_sums)
    launch_cwq_conv2d_i8(d_out, d_x, d_f, d_b, b8, g, out_offset, in_offset,
                         *vs, act, act_args, f_offsets_all_zero, d_sums, opts=opts)
    return d_out.numpy()


def cwq_conv2d_add_i8(x, filt, bias, geom, out_offset, in_offset, f_offsets,
                      b_offsets, bias_pre, bias_post, bias_scale, out_pre, out_post,
                      out_scale, act, act_args, residual, add):
    """The convolution of cwq_conv2d_i8 followed by ElementAdd with `residual`
    (and Relu when add.relu) in one kernel."""
    g = _geom(geom)
    x = np.ascontiguousarray(x, np.int8)
    filt = np.ascontiguousarray(filt, np.int8)
    residual = np.ascontiguousarray(residual, np.int8)
    d_x, d_f, d_r = to_device(x), to_device(filt), to_device(residual)
    d_b, b8 = _bias_dev(bias)
    vs = [_dev_i32(v) for v in (f_offsets, b_offsets, bias_pre, bias_post,
                                bias_scale, out_pre, out_post, out_scale)]
    d_out = DeviceBuffer.empty((g.N, g.OH, g.OW, g.OC), np.int8)
    d_sums = _row_sums_dev(d_f, g.OC, filt.size // g.OC, True)
    launch_cwq_conv2d_add_i8(d_out, d_x, d_f, d_b, b8, g, out_offset, in_offset,
                             *vs, act, act_args, not np.any(f_offsets), d_sums, d_r, add)
    return d_out.numpy()


def conv2d_i8(x, filt, bias, geom, out_offset, in_offset, filter_offset,
              bias_offset, biasP, outP, act=ACT_NONE, act_args=(),
              precomputed_sums=False):
    g = _geom(geom)
    x = np.ascontiguousarray(x, np.int8)
    filt = np.ascontiguousarray(filt, np.int8)
    d_x, d_f = to_device(x), to_device(filt)
    d_b, b8 = _bias_dev(bias)
    d_out = DeviceBuffer.empty((g.N, g.OH, g.OW, g.OC), np.int8)
    aa = (C.c_int32 * 3)(*(list(act_args) + [0, 0, 0])[:3])
    d_sums = _row_sums_dev(d_f, g.OC, filt.size // g.OC, precomputed_sums)
    check(lib().mi355x_conv2d_i8(
        _vp(d_out), _vp(d_x), _vp(d_f), _vp(d_b), C.c_int(b8), C.byref(g),
        _i32(out_offset), _i32(in_offset), _i32(filter_offset),
        _i32(bias_offset), *[_i32(v) for v in biasP], *[_i32(v) for v in outP],
        _i32(act), aa, _vp(d_sums), _vp(None)))
    return d_out.numpy()


def _fused_cols(in_line, kind):
    so = 8 if kind in (FUSED_U8_F32, FUSED_U4_F32) else 4
    return (in_line - so) * (2 if kind in (FUSED_U4_F16, FUSED_U4_F32) else 1)


def frwq_slws(data, kind, weights, indices, lengths, out_f16=False,
              fp16_accum=False, d_data=None, row_pitch=None, stream=None,
              noalloc=False, bag_offsets=False, opts=None):
    """weights: None (plain SLS), float32 or float16 array. `d_data` lets a
    caller reuse a table already resident on the device. `row_pitch` lays the
    table out with its rows that many bytes apart (the gaps hold junk).
    `bag_offsets`: through mi355x_frwq_slws_offsets, with the positions that
    mi355x_slws_bag_offsets_host makes of the lengths (or the array given)."""
    data_shape = data.shape
    in_line = data_shape[1]
    out_line = _fused_cols(in_line, kind)
    if row_pitch is not None:
        wide = np.full((data_shape[0], row_pitch), 0xA5, np.uint8)
        wide[:, :in_line] = data
        d_data = to_device(wide)
        in_line = row_pitch
    if d_data is None:
        d_data = to_device(np.ascontiguousarray(data, np.uint8))
    indices = np.ascontiguousarray(indices)
    if indices.dtype != np.int64:
        indices = indices.astype(np.int32)
    lengths = np.ascontiguousarray(lengths, np.int32)
    d_w, w16 = None, 0
    if weights is not None:
        weights = np.ascontiguousarray(weights)
        if weights.dtype == np.float16:
            w16 = 1
        else:
            weights = weights.astype(np.float32)
        d_w = to_device(weights)
    d_idx, d_len = to_device(indices), to_device(lengths)
    d_out = DeviceBuffer.empty((lengths.size, out_line),
                               np.float16 if out_f16 else np.float32)
    d_out.fill(0xFF)  # poison: every row must be written by the kernel
    if stream is not None:
        sync()        # streams of this library do not wait for the default stream
    if bag_offsets is not False:
        offs = slws_bag_offsets_host(lengths) if bag_offsets is True else \
            np.ascontiguousarray(bag_offsets, np.int32)
        assert offs.size == lengths.size + 1
        launch_frwq_slws_offsets(d_out, out_f16, d_data, data_shape[0], kind, d_w, w16,
                                 d_idx, indices.dtype == np.int64, indices.size,
                                 to_device(offs), lengths.size, in_line, out_line,
                                 fp16_accum, stream=stream, opts=opts)
    else:
        launch_frwq_slws(d_out, out_f16, d_data, data_shape[0], kind, d_w, w16,
                         d_idx, indices.dtype == np.int64, indices.size, d_len,
                         lengths.size, in_line, out_line, fp16_accum, stream=stream,
                         noalloc=noalloc, opts=opts)
    if stream is not None:
        stream.sync()
    return d_out.numpy()


def embedding_bag_rowwise_offsets(data, kind, weights, indices, offsets,
                                  has_end_offset, out_f16=False,
                                  fp16_accum=False):
    data = np.ascontiguousarray(data, np.uint8)
    in_line = data.shape[1]
    out_line = _fused_cols(in_line, kind)
    indices = np.ascontiguousarray(indices, np.int32)
    offsets = np.ascontiguousarray(offsets, np.int32)
    d_w, w16 = None, 0
    if weights is not None:
        weights = np.ascontiguousarray(weights)
        if weights.dtype == np.float16:
            w16 = 1
        else:
            weights = weights.astype(np.float32)
        d_w = to_device(weights)
    d_data, d_idx, d_off = to_device(data), to_device(indices), to_device(offsets)
    rows = offsets.size - (1 if has_end_offset else 0)
    d_out = DeviceBuffer.empty((rows, out_line),
                               np.float16 if out_f16 else np.float32)
    d_out.fill(0xFF)
    check(lib().mi355x_embedding_bag_rowwise_offsets(
        _vp(d_out), C.c_int(bool(out_f16)), _vp(d_data), _sz(data.shape[0]),
        C.c_int(kind), _vp(d_w), C.c_int(w16), _vp(d_idx), _sz(indices.size),
        _vp(d_off), _sz(offsets.size), C.c_int(bool(has_end_offset)),
        _sz(in_line), _sz(out_line), C.c_int(bool(fp16_accum)), _vp(None)))
    return d_out.numpy()


# ---- 16/32-bit elementwise forms, N-D transpose, 3-D convolution ---------------

_WIDE = {16: np.int16, 32: np.int32}


def quantize_wide(x, scale, offset, bits):
    x = np.ascontiguousarray(x, np.float32)
    d_in, d_out = to_device(x), DeviceBuffer.empty(x.shape, _WIDE[bits])
    check(getattr(lib(), f"mi355x_quantize_i{bits}")(
        _vp(d_out), _vp(d_in), _sz(x.size), C.c_float(scale), _i32(offset), _vp(None)))
    return d_out.numpy()


def dequantize_wide(q, scale, offset):
    q = np.ascontiguousarray(q)
    d_in, d_out = to_device(q), DeviceBuffer.empty(q.shape, np.float32)
    check(getattr(lib(), f"mi355x_dequantize_i{q.itemsize * 8}")(
        _vp(d_out), _vp(d_in), _sz(q.size), C.c_float(scale), _i32(offset), _vp(None)))
    return d_out.numpy()


def rescale_wide(q, out_offset, in_offset, pre, post, scale):
    q = np.ascontiguousarray(q)
    d_in, d_out = to_device(q), DeviceBuffer.empty(q.shape, q.dtype)
    check(getattr(lib(), f"mi355x_rescale_i{q.itemsize * 8}")(
        _vp(d_out), _vp(d_in), _sz(q.size), _i32(out_offset), _i32(in_offset), _i32(pre),
        _i32(post), _i32(scale), _vp(None)))
    return d_out.numpy()


def transpose_nd(x, shuffle):
    """Output dimension d is input dimension shuffle[d] (numpy's transpose)."""
    x = np.ascontiguousarray(x)
    nd = x.ndim
    dims = (C.c_size_t * nd)(*x.shape)
    sh = (C.c_size_t * nd)(*shuffle)
    out_shape = [x.shape[d] for d in shuffle] if sorted(shuffle) == list(range(nd)) else x.shape
    d_in, d_out = to_device(x), DeviceBuffer.empty(out_shape, x.dtype)
    check(lib().mi355x_transpose_nd(_vp(d_out), _vp(d_in), dims, sh, _sz(nd), _sz(x.itemsize),
                                    _vp(None)))
    return d_out.numpy()


def cwq_conv3d_i8(x, filt, bias, geom, out_offset, in_offset, filter_offsets,
                  bias_offsets, bias_pre, bias_post, bias_scale, out_pre, out_post,
                  out_scale, act=0, act_args=()):
    g = geom if isinstance(geom, Conv3dGeom) else \
        Conv3dGeom(*[getattr(geom, n) for n, _ in Conv3dGeom._fields_])
    bias = np.ascontiguousarray(bias)
    b8 = int(bias.dtype == np.int8)
    if not b8:
        bias = bias.astype(np.int32)
    d = [to_device(np.ascontiguousarray(v, np.int8)) for v in (x, filt)]
    vs = [to_device(np.ascontiguousarray(v, np.int32)) for v in (
        filter_offsets, bias_offsets, bias_pre, bias_post, bias_scale, out_pre, out_post,
        out_scale)]
    d_bias = to_device(bias)
    d_out = DeviceBuffer.empty((g.N, g.OT, g.OH, g.OW, g.OC), np.int8)
    d_out.fill(0x55)
    aa = (C.c_int32 * 3)(*(list(act_args) + [0, 0, 0])[:3])
    check(lib().mi355x_cwq_conv3d_i8(
        _vp(d_out), _vp(d[0]), _vp(d[1]), _vp(d_bias), C.c_int(b8), C.byref(g),
        _i32(out_offset), _i32(in_offset), *[_vp(v) for v in vs], _i32(act), aa, _vp(None)))
    return d_out.numpy()


# ---- int8 glue operators ------------------------------------------------------

def _i32s(vals):
    return [_i32(int(v)) for v in vals]


def launch_add_i8(dst, lhs, rhs, n, dest_offset, lhs_offset, rhs_offset, lhsP, rhsP,
                  stream=None):
    check(lib().mi355x_add_i8(_vp(dst), _vp(lhs), _vp(rhs), _sz(n), _i32(dest_offset),
                              _i32(lhs_offset), _i32(rhs_offset), *_i32s(lhsP),
                              *_i32s(rhsP), _vp(stream)))


def launch_add_relu_i8(dst, lhs, rhs, n, sum_offset, lhs_offset, rhs_offset, lhsP, rhsP,
                       dest_offset, destP, stream=None):
    check(lib().mi355x_add_relu_i8(_vp(dst), _vp(lhs), _vp(rhs), _sz(n), _i32(sum_offset),
                                   _i32(lhs_offset), _i32(rhs_offset), *_i32s(lhsP),
                                   *_i32s(rhsP), _i32(dest_offset), *_i32s(destP),
                                   _vp(stream)))


def add_i8(lhs, rhs, dest_offset, lhs_offset, rhs_offset, lhsP, rhsP):
    lhs = np.ascontiguousarray(lhs, np.int8)
    rhs = np.ascontiguousarray(rhs, np.int8)
    dl, dr = to_device(lhs), to_device(rhs)
    out = DeviceBuffer.empty(lhs.shape, np.int8)
    launch_add_i8(out, dl, dr, lhs.size, dest_offset, lhs_offset, rhs_offset, lhsP, rhsP)
    return out.numpy()


def add_relu_i8(lhs, rhs, sum_offset, lhs_offset, rhs_offset, lhsP, rhsP, dest_offset, destP):
    lhs = np.ascontiguousarray(lhs, np.int8)
    rhs = np.ascontiguousarray(rhs, np.int8)
    dl, dr = to_device(lhs), to_device(rhs)
    out = DeviceBuffer.empty(lhs.shape, np.int8)
    launch_add_relu_i8(out, dl, dr, lhs.size, sum_offset, lhs_offset, rhs_offset, lhsP, rhsP,
                       dest_offset, destP)
    return out.numpy()


def relu_i8(src, src_offset, dest_offset, destP):
    src = np.ascontiguousarray(src, np.int8)
    ds = to_device(src)
    out = DeviceBuffer.empty(src.shape, np.int8)
    check(lib().mi355x_relu_i8(_vp(out), _vp(ds), _sz(src.size), _i32(src_offset),
                               _i32(dest_offset), *_i32s(destP), _vp(None)))
    return out.numpy()


def _pool_sizes(x, kernel, stride, pads):
    N, IH, IW, Cn = x.shape
    OH = (IH + pads[0] + pads[2] - kernel[0]) // stride[0] + 1
    OW = (IW + pads[1] + pads[3] - kernel[1]) // stride[1] + 1
    sz = [_sz(int(v)) for v in (N, IH, IW, Cn, OH, OW, kernel[0], kernel[1], stride[0],
                                stride[1], pads[0], pads[1])]
    return (N, OH, OW, Cn), sz


def clip_elem_i8(src, clip_min, clip_max, src_offset, dest_offset, destP):
    src = np.ascontiguousarray(src, np.int8)
    ds = to_device(src)
    out = DeviceBuffer.empty(src.shape, np.int8)
    check(lib().mi355x_clip_i8(_vp(out), _vp(ds), _sz(src.size), _i32(clip_min), _i32(clip_max),
                               _i32(src_offset), _i32(dest_offset),
                               *[_i32(int(v)) for v in destP], _vp(None)))
    return out.numpy()


def leaky_relu_i8(src, src_offset, dest_offset, posP, negP):
    src = np.ascontiguousarray(src, np.int8)
    ds = to_device(src)
    out = DeviceBuffer.empty(src.shape, np.int8)
    check(lib().mi355x_leaky_relu_i8(_vp(out), _vp(ds), _sz(src.size), _i32(src_offset),
                                     _i32(dest_offset), *[_i32(int(v)) for v in posP],
                                     *[_i32(int(v)) for v in negP], _vp(None)))
    return out.numpy()


def max_splat_i8(src, value):
    src = np.ascontiguousarray(src, np.int8)
    ds = to_device(src)
    out = DeviceBuffer.empty(src.shape, np.int8)
    check(lib().mi355x_max_splat_i8(_vp(out), _vp(ds), _sz(src.size), _i32(value), _vp(None)))
    return out.numpy()


def batched_add_i8(batch, slice_, dest_offset, batch_offset, slice_offset, batchP, sliceP):
    batch = np.ascontiguousarray(batch, np.int8)
    slice_ = np.ascontiguousarray(slice_)
    i32 = slice_.dtype == np.int32
    if not i32:
        slice_ = slice_.astype(np.int8)
    db, dsl = to_device(batch), to_device(slice_)
    out = DeviceBuffer.empty(batch.shape, np.int8)
    check(lib().mi355x_batched_add_i8(_vp(out), _vp(db), _vp(dsl), C.c_int(int(i32)),
                                      _sz(batch.shape[0]), _sz(slice_.size), _i32(dest_offset),
                                      _i32(batch_offset), _i32(slice_offset),
                                      *[_i32(int(v)) for v in batchP],
                                      *[_i32(int(v)) for v in sliceP], _vp(None)))
    return out.numpy()


def max_pool_i8(x, kernel, stride, pads, out_offset):
    """pads = (top, left, bottom, right)."""
    x = np.ascontiguousarray(x, np.int8)
    shape, sz = _pool_sizes(x, kernel, stride, pads)
    dx = to_device(x)
    out = DeviceBuffer.empty(shape, np.int8)
    check(lib().mi355x_max_pool_i8(_vp(out), _vp(dx), *sz, _i32(out_offset), _vp(None)))
    return out.numpy()


def avg_pool_i8(x, kernel, stride, pads, count_include_pads, out_offset, in_offset, outP):
    x = np.ascontiguousarray(x, np.int8)
    shape, sz = _pool_sizes(x, kernel, stride, pads)
    dx = to_device(x)
    out = DeviceBuffer.empty(shape, np.int8)
    check(lib().mi355x_avg_pool_i8(_vp(out), _vp(dx), *sz, C.c_int(int(count_include_pads)),
                                   _i32(out_offset), _i32(in_offset), *_i32s(outP), _vp(None)))
    return out.numpy()


def softmax_f32(x):
    x = np.ascontiguousarray(x, np.float32)
    dx = to_device(x)
    out = DeviceBuffer.empty(x.shape, np.float32)
    check(lib().mi355x_softmax_f32(_vp(out), _vp(dx), _sz(x.shape[0]), _sz(x.shape[1]),
                                   _vp(None)))
    return out.numpy()


def dequantize_softmax(q, scale, offset):
    q = np.ascontiguousarray(q, np.int8)
    dq = to_device(q)
    out = DeviceBuffer.empty(q.shape, np.float32)
    check(lib().mi355x_dequantize_softmax(_vp(out), _vp(dq), _sz(q.shape[0]), _sz(q.shape[1]),
                                          C.c_float(scale), _i32(offset), _vp(None)))
    return out.numpy()


# ---- data movement and the small operators of ranking models -------------------
# (device buffers are bound to names so they outlive the launch)

def convert_f16_to_f32(x):
    x = np.ascontiguousarray(x, np.float16)
    dx = to_device(x)
    out = DeviceBuffer.empty(x.shape, np.float32)
    check(lib().mi355x_convert_f16_to_f32(_vp(out), _vp(dx), _sz(x.size), _vp(None)))
    return out.numpy()


def concat_rows(parts):
    """Concat of 2-D arrays of one dtype along dimension 1 through InsertTensor."""
    parts = [np.ascontiguousarray(p) for p in parts]
    rows, item = parts[0].shape[0], parts[0].dtype.itemsize
    width = sum(p.shape[1] for p in parts)
    out = DeviceBuffer.empty((rows, width), parts[0].dtype)
    held, off = [], 0
    for p in parts:
        dp = to_device(p)
        held.append(dp)
        check(lib().mi355x_insert_rows(_vp(out), _vp(dp), _sz(rows), _sz(p.shape[1] * item),
                                       _sz(width * item), _sz(off * item), _vp(None)))
        off += p.shape[1]
    return out.numpy()


def batch_transpose_i8(x):
    x = np.ascontiguousarray(x, np.int8)
    b, r, c = x.shape
    dx = to_device(x)
    out = DeviceBuffer.empty((b, c, r), np.int8)
    check(lib().mi355x_batch_transpose_i8(_vp(out), _vp(dx), _sz(b), _sz(r), _sz(c), _vp(None)))
    return out.numpy()


def gather(data, indices, batch_dims=0):
    """Gather along the first non-batch dimension (batch_dims 0 or 1)."""
    data = np.ascontiguousarray(data)
    indices = np.ascontiguousarray(indices)
    assert indices.dtype in (np.int32, np.int64) and indices.ndim == 1
    samples = data.shape[0] if batch_dims else 1
    inner = data.shape[batch_dims + 1:]
    slice_bytes = int(np.prod(inner, dtype=np.int64)) * data.dtype.itemsize
    sample_bytes = data.shape[batch_dims] * slice_bytes
    shape = (data.shape[:batch_dims]) + (indices.size,) + inner
    dd, di = to_device(data), to_device(indices)
    out = DeviceBuffer.empty(shape, data.dtype)
    check(lib().mi355x_gather(_vp(out), _vp(dd), _vp(di), C.c_int(indices.dtype == np.int64),
                              _sz(indices.size), _sz(slice_bytes), _sz(samples),
                              _sz(sample_bytes), _vp(None)))
    return out.numpy()


def gather_rows(data, indices, into, col):
    """Gather with one batch dimension whose samples land in the 2-D array
    `into` starting at element column `col`; returns the updated array."""
    data = np.ascontiguousarray(data)
    indices = np.ascontiguousarray(indices)
    into = np.ascontiguousarray(into)
    assert into.dtype == data.dtype and into.ndim == 2 and into.shape[0] == data.shape[0]
    es = data.dtype.itemsize
    slice_bytes = int(np.prod(data.shape[2:], dtype=np.int64)) * es
    sample_bytes = data.shape[1] * slice_bytes
    dd, di, out = to_device(data), to_device(indices), to_device(into)
    check(lib().mi355x_gather_rows(_vp(out.ptr + col * es), _vp(dd), _vp(di),
                                   C.c_int(indices.dtype == np.int64), _sz(indices.size),
                                   _sz(slice_bytes), _sz(data.shape[0]), _sz(sample_bytes),
                                   _sz(into.shape[1] * es), _vp(None)))
    return out.numpy()


def rescale_rows_i8(q, into, col, out_offset, in_offset, pre, post, scale):
    """Rescale of the 2-D int8 array `q` written into `into` at column `col`."""
    q = np.ascontiguousarray(q, np.int8)
    into = np.ascontiguousarray(into, np.int8)
    d_in, out = to_device(q), to_device(into)
    check(lib().mi355x_rescale_rows_i8(_vp(out.ptr + col), _vp(d_in), _sz(q.shape[0]),
                                       _sz(q.shape[1]), _sz(into.shape[1]), _i32(out_offset),
                                       _i32(in_offset), _i32(pre), _i32(post), _i32(scale),
                                       _vp(None)))
    return out.numpy()


def dequantize_sigmoid(q, scale, offset):
    q = np.ascontiguousarray(q, np.int8)
    d_in = to_device(q)
    out = DeviceBuffer.empty(q.shape, np.float32)
    check(lib().mi355x_dequantize_sigmoid(_vp(out), _vp(d_in), _sz(q.size), C.c_float(scale),
                                          _i32(offset), _vp(None)))
    return out.numpy()


def batch_matmul_i8(lhs, rhs, out_offset, lhs_offset, rhs_offset, outP):
    lhs = np.ascontiguousarray(lhs, np.int8)
    rhs = np.ascontiguousarray(rhs, np.int8)
    b, m, k = lhs.shape
    n = rhs.shape[2]
    dl, dr = to_device(lhs), to_device(rhs)
    out = DeviceBuffer.empty((b, m, n), np.int8)
    check(lib().mi355x_batch_matmul_i8(_vp(out), _vp(dl), _vp(dr), _sz(b), _sz(m), _sz(k),
                                       _sz(n), _i32(out_offset), _i32(lhs_offset),
                                       _i32(rhs_offset), *_i32s(outP), _vp(None)))
    return out.numpy()


def batch_matmul_nt_i8(lhs, rhs_nk, out_offset, lhs_offset, rhs_offset, outP):
    """lhs [B, M, K] x transpose of rhs_nk [B, N, K]."""
    lhs = np.ascontiguousarray(lhs, np.int8)
    rhs_nk = np.ascontiguousarray(rhs_nk, np.int8)
    b, m, k = lhs.shape
    n = rhs_nk.shape[1]
    dl, dr = to_device(lhs), to_device(rhs_nk)
    out = DeviceBuffer.empty((b, m, n), np.int8)
    check(lib().mi355x_batch_matmul_nt_i8(_vp(out), _vp(dl), _vp(dr), _sz(b), _sz(m), _sz(k),
                                          _sz(n), _i32(out_offset), _i32(lhs_offset),
                                          _i32(rhs_offset), *_i32s(outP), _vp(None)))
    return out.numpy()


def batch_matmul_nt_select_i8(lhs, rhs_nk, out_offset, lhs_offset, rhs_offset, outP, dest_of,
                              into, col):
    """The product's elements e with dest_of[e] >= 0 written into the 2-D int8
    array `into` at column col + dest_of[e]; returns the updated array."""
    lhs = np.ascontiguousarray(lhs, np.int8)
    rhs_nk = np.ascontiguousarray(rhs_nk, np.int8)
    b, m, k = lhs.shape
    n = rhs_nk.shape[1]
    dest_of = np.ascontiguousarray(dest_of, np.int32)
    assert dest_of.size == m * n
    into = np.ascontiguousarray(into, np.int8)
    dl, dr, dd, out = to_device(lhs), to_device(rhs_nk), to_device(dest_of), to_device(into)
    check(lib().mi355x_batch_matmul_nt_select_i8(
        _vp(out.ptr + col), _vp(dl), _vp(dr), _sz(b), _sz(m), _sz(k), _sz(n), _i32(out_offset),
        _i32(lhs_offset), _i32(rhs_offset), *_i32s(outP), _vp(dd), _sz(into.shape[1]), _vp(None)))
    return out.numpy()


def sigmoid_f32(x):
    x = np.ascontiguousarray(x, np.float32)
    dx = to_device(x)
    out = DeviceBuffer.empty(x.shape, np.float32)
    check(lib().mi355x_sigmoid_f32(_vp(out), _vp(dx), _sz(x.size), _vp(None)))
    return out.numpy()


def space_to_depth2_i8(x, pad_t, pad_l, bh, bw, cout, fill):
    x = np.ascontiguousarray(x, np.int8)
    n, ih, iw, c = x.shape
    dx = to_device(x)
    out = DeviceBuffer.empty((n, bh, bw, cout), np.int8)
    check(lib().mi355x_space_to_depth2_i8(_vp(out), _vp(dx), _sz(n), _sz(ih), _sz(iw), _sz(c),
                                          _sz(pad_t), _sz(pad_l), _sz(bh), _sz(bw), _sz(cout),
                                          _i32(fill), _vp(None)))
    return out.numpy()


def quantize_space_to_depth2_i8(x, pad_t, pad_l, bh, bw, cout, fill, scale, offset):
    x = np.ascontiguousarray(x, np.float32)
    n, ih, iw, c = x.shape
    dx = to_device(x)
    out = DeviceBuffer.empty((n, bh, bw, cout), np.int8)
    check(lib().mi355x_quantize_space_to_depth2_i8(
        _vp(out), _vp(dx), _sz(n), _sz(ih), _sz(iw), _sz(c), _sz(pad_t), _sz(pad_l), _sz(bh),
        _sz(bw), _sz(cout), _i32(fill), C.c_float(scale), _i32(offset), _vp(None)))
    return out.numpy()


class SlsTable(C.Structure):
    """mi355x_sls_table: one table of a multi-table pooled lookup."""
    _fields_ = [("data", C.c_void_p), ("indices", C.c_void_p), ("lengths", C.c_void_p),
                ("dest", C.c_void_p), ("data_rows", C.c_uint64), ("num_indices", C.c_uint64),
                ("bag_offsets", C.c_void_p)]


SLS_OUT_F32, SLS_OUT_F16, SLS_OUT_I8, SLS_OUT_I8_VIA_F16 = range(4)


def frwq_sls_multi(tables, kind, indices, lengths, out_kind=SLS_OUT_F32, out_scale=1.0,
                   out_offset=0, fp16_accum=False, bag_offsets=False):
    """tables, indices, lengths: equally long lists (one entry per table; tables
    of one shape, indices of one dtype). Dense output kinds return a list of
    [bags x cols] arrays; the int8 kinds return the concatenation
    [bags x tables*cols] that the fused InsertTensors build."""
    n = len(tables)
    tabs = [np.ascontiguousarray(t, np.uint8) for t in tables]
    idx = [np.ascontiguousarray(i) for i in indices]
    lens = [np.ascontiguousarray(l, np.int32) for l in lengths]
    in_line = tabs[0].shape[1]
    cols = _fused_cols(in_line, kind)
    bags = lens[0].size
    d_t = [to_device(t) for t in tabs]
    d_i = [to_device(i if i.size else np.zeros(1, i.dtype)) for i in idx]
    d_l = [to_device(l) for l in lens]
    q8 = out_kind >= SLS_OUT_I8
    if q8:
        out = DeviceBuffer.empty((bags, n * cols), np.int8)
        dests = [out.ptr + t * cols for t in range(n)]
        stride = n * cols
    else:
        dt = np.float16 if out_kind == SLS_OUT_F16 else np.float32
        outs = [DeviceBuffer.empty((bags, cols), dt) for _ in range(n)]
        dests = [o.ptr for o in outs]
        stride = 0
    # bag_offsets: every table's bags as host-made positions instead of lengths
    d_o = [to_device(slws_bag_offsets_host(l)) for l in lengths] if bag_offsets else None
    arr = (SlsTable * n)()
    for t in range(n):
        arr[t] = SlsTable(d_t[t].ptr, d_i[t].ptr, d_l[t].ptr, dests[t], tabs[t].shape[0],
                          idx[t].size, d_o[t].ptr if bag_offsets else None)
    d_arr = DeviceBuffer(C.sizeof(arr))
    check(lib().mi355x_memcpy_h2d(_vp(d_arr), C.byref(arr), _sz(C.sizeof(arr)), _vp(None)))
    sync()
    check(lib().mi355x_frwq_sls_multi(
        _vp(d_arr), _sz(n), _sz(max(t.shape[0] for t in tabs)), C.c_int(kind),
        C.c_int(idx[0].dtype == np.int64), _sz(bags), _sz(in_line), _sz(cols),
        C.c_int(out_kind), C.c_float(out_scale), _i32(out_offset), _sz(stride),
        C.c_int(bool(fp16_accum)), _vp(None)))
    if q8:
        return out.numpy()
    return [o.numpy() for o in outs]


def slws_set_fused_math(on):
    """Process-wide: fused multiply-add arithmetic in the SparseLengths kernels
    (default) or the CPU loop's separately rounded operations."""
    check(lib().mi355x_slws_set_fused_math(C.c_int(int(on))))


def rwq_slws(data, scales, offsets, weights, indices, lengths):
    """RowwiseQuantizedSparseLengthsWeightedSum: uint8 rows, separate fp32
    scales and offsets per row."""
    data = np.ascontiguousarray(data, np.uint8)
    scales = np.ascontiguousarray(scales, np.float32)
    offsets = np.ascontiguousarray(offsets, np.float32)
    indices = np.ascontiguousarray(indices)
    lengths = np.ascontiguousarray(lengths, np.int32)
    d_d, d_s, d_o = to_device(data), to_device(scales), to_device(offsets)
    d_i = to_device(indices if indices.size else np.zeros(1, indices.dtype))
    d_l = to_device(lengths)
    d_w = None if weights is None else to_device(np.ascontiguousarray(weights, np.float32))
    out = DeviceBuffer.empty((lengths.size, data.shape[1]), np.float32)
    check(lib().mi355x_rwq_slws(_vp(out), _vp(d_d), _sz(data.shape[0]), _vp(d_s), _vp(d_o),
                                _vp(d_w), _vp(d_i), C.c_int(indices.dtype == np.int64),
                                _sz(indices.size), _vp(d_l), _sz(lengths.size),
                                _sz(data.shape[1]), _vp(None)))
    return out.numpy()

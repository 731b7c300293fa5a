"""ctypes view of the MI355X backend's host layer (glow_amd/host, C++):
Module -> MI355XBackend.compile -> MI355XDeviceManager add/run/evict, the way a
Glow runtime drives a backend (reference include/glow/Backend/Backend.h,
include/glow/Backends/DeviceManager.h). Used by the harnesses and tests."""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

(FLOAT, FLOAT16, INT8Q, INT32Q, INT32I, INT64I, UINT8_FUSED, UINT8_FUSED_FP16,
 UINT4_FUSED_FP16, UINT4_FUSED, BOOL, INT16Q) = range(12)
(QUANTIZE, DEQUANTIZE, RESCALE_QUANTIZED, FULLY_CONNECTED, ROWWISE_QUANTIZED_FC,
 MATMUL, CONVOLUTION, CHANNELWISE_QUANTIZED_CONV, FRWQ_SLWS, FRWQ_SLS, ELEMENT_ADD,
 RELU, MAX_POOL, AVG_POOL, SOFTMAX, CONVERT_TO, INSERT_TENSOR, TRANSPOSE, GATHER,
 BATCH_MATMUL, SIGMOID, RWQ_SLWS, EMBEDDING_BAG_BYTE_ROWWISE_OFFSETS, COPY, CLIP, LEAKY_RELU,
 CPU_MAX_SPLAT, BATCHED_ADD) = range(28)
ACT_NONE, ACT_RELU, ACT_CLIP, ACT_TANH, ACT_SIGMOID, ACT_LEAKY_RELU = range(6)

ERROR_NAMES = ["SUCCESS", "UNKNOWN", "RUNTIME_ERROR", "RUNTIME_OUT_OF_DEVICE_MEMORY",
               "RUNTIME_NET_NOT_FOUND", "RUNTIME_REQUEST_REFUSED",
               "RUNTIME_DEVICE_NOT_FOUND", "RUNTIME_DEVICE_NONRECOVERABLE",
               "RUNTIME_NET_BUSY", "DEVICE_FEATURE_NOT_SUPPORTED",
               "COMPILE_UNSUPPORTED_NODE_AFTER_OPTIMIZE", "COMPILE_CONTEXT_MALFORMED"]

EXPORTS = [
    "mi355x_host_last_error", "mi355x_host_error_name", "mi355x_host_module_create",
    "mi355x_host_module_destroy", "mi355x_host_add_constant", "mi355x_host_add_placeholder",
    "mi355x_host_create_function", "mi355x_host_add_activation", "mi355x_host_add_view", "mi355x_host_add_view_at",
    "mi355x_host_add_instruction", "mi355x_host_is_op_supported", "mi355x_host_compile",
    "mi355x_host_describe", "mi355x_host_bundle_sizes", "mi355x_host_dm_create", "mi355x_host_dm_create_opts",
    "mi355x_host_dm_destroy", "mi355x_host_dm_init", "mi355x_host_dm_stop",
    "mi355x_host_dm_add_network", "mi355x_host_dm_evict_network", "mi355x_host_dm_run",
    "mi355x_host_dm_time_function", "mi355x_host_dm_maximum_memory", "mi355x_host_dm_available_memory",
    "mi355x_host_dm_add_functions", "mi355x_host_dm_transfer_static_placeholder",
]


class HostError(RuntimeError):
    def __init__(self, code, msg):
        self.code = code
        self.code_name = ERROR_NAMES[code] if 0 <= code < len(ERROR_NAMES) else "UNKNOWN"
        super().__init__(f"{self.code_name}: {msg}")


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libglow_mi355x_host.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is not built: run __graft_entry__.build()")
        # the kernel library first, so the host layer binds to the same copy
        from glow_amd import capi
        capi.lib()
        L = C.CDLL(path)
        L.mi355x_host_last_error.restype = C.c_char_p
        L.mi355x_host_error_name.restype = C.c_char_p
        L.mi355x_host_module_create.restype = C.c_void_p
        L.mi355x_host_dm_create.restype = C.c_void_p
        L.mi355x_host_dm_create_opts.restype = C.c_void_p
        L.mi355x_host_dm_maximum_memory.restype = C.c_uint64
        L.mi355x_host_dm_available_memory.restype = C.c_uint64
        _LIB = L
    return _LIB


def _check(rc):
    if rc < 0:
        raise HostError(-rc, lib().mi355x_host_last_error().decode())
    return rc


def _dims(shape):
    shape = [int(s) for s in shape]
    return (C.c_int64 * len(shape))(*shape), len(shape)


_NP_KIND = {np.dtype(np.float32): FLOAT, np.dtype(np.float16): FLOAT16,
            np.dtype(np.int64): INT64I}


class Module:
    """Constants, placeholders, functions and their instructions."""

    def __init__(self, name="module"):
        self._h = C.c_void_p(lib().mi355x_host_module_create(name.encode()))
        self.placeholders = {}     # name -> (shape, numpy dtype)
        self.functions = {}        # name -> index

    def __del__(self):
        try:
            if self._h:
                lib().mi355x_host_module_destroy(self._h)
                self._h = None
        except Exception:
            pass

    def constant(self, name, array, kind=None, scale=1.0, offset=0):
        a = np.ascontiguousarray(array)
        if kind is None:
            kind = _NP_KIND.get(a.dtype)
            if kind is None:
                raise ValueError(f"give the element kind of a {a.dtype} constant")
        d, nd = _dims(a.shape)
        return _check(lib().mi355x_host_add_constant(
            self._h, name.encode(), kind, d, nd, C.c_float(scale), C.c_int32(offset),
            a.ctypes.data_as(C.c_void_p)))

    def placeholder(self, name, shape, kind, dtype, scale=1.0, offset=0):
        d, nd = _dims(shape)
        self.placeholders[name] = (tuple(int(s) for s in shape), np.dtype(dtype))
        return _check(lib().mi355x_host_add_placeholder(
            self._h, name.encode(), kind, d, nd, C.c_float(scale), C.c_int32(offset)))

    def function(self, name):
        idx = _check(lib().mi355x_host_create_function(self._h, name.encode()))
        self.functions[name] = idx
        return idx

    def activation(self, fn, name, shape, kind, scale=1.0, offset=0):
        d, nd = _dims(shape)
        return _check(lib().mi355x_host_add_activation(
            self._h, fn, name.encode(), kind, d, nd, C.c_float(scale), C.c_int32(offset)))

    def view(self, name, source, shape, kind, scale=1.0, offset=0, byte_offset=0):
        d, nd = _dims(shape)
        if byte_offset:
            return _check(lib().mi355x_host_add_view_at(
                self._h, name.encode(), source, kind, d, nd, C.c_float(scale), C.c_int32(offset),
                C.c_size_t(byte_offset)))
        return _check(lib().mi355x_host_add_view(
            self._h, name.encode(), source, kind, d, nd, C.c_float(scale), C.c_int32(offset)))

    @staticmethod
    def _inst_args(operands, iattrs, fattrs):
        ops = (C.c_int * len(operands))(*[int(o) for o in operands])
        ia = (C.c_int64 * max(len(iattrs), 1))(*[int(v) for v in iattrs])
        fa = (C.c_float * max(len(fattrs), 1))(*[float(v) for v in fattrs])
        return ops, len(operands), ia, len(iattrs), fa, len(fattrs)

    def instruction(self, fn, kind, name, operands, iattrs=(), fattrs=()):
        return _check(lib().mi355x_host_add_instruction(
            self._h, fn, kind, name.encode(), *self._inst_args(operands, iattrs, fattrs)))

    def is_op_supported(self, kind, operands, iattrs=(), fattrs=()):
        rc = _check(lib().mi355x_host_is_op_supported(
            self._h, kind, *self._inst_args(operands, iattrs, fattrs)))
        return bool(rc), (lib().mi355x_host_last_error().decode() if not rc else "")

    def compile(self, fn, precompute_weight_row_sums=True, fuse_add_relu=True,
                fuse_conv_add=True, space_to_depth_stem=True, fuse_sls_chains=True,
                fuse_transpose_matmul=True, fuse_fc_relu=True,
                pad_table_rows=True, fuse_insert=True, fuse_dequantize_sigmoid=True,
                derive_bag_offsets=True, reuse_activations=True,
                fuse_quantize_stem=True, split_k=True):
        opts = ((1 if precompute_weight_row_sums else 0) | (2 if fuse_add_relu else 0) |
                (4 if fuse_conv_add else 0) | (8 if space_to_depth_stem else 0) |
                (16 if fuse_sls_chains else 0) | (32 if fuse_transpose_matmul else 0) |
                (64 if fuse_fc_relu else 0) |
                (128 if pad_table_rows else 0) | (256 if fuse_insert else 0) |
                (512 if fuse_dequantize_sigmoid else 0) |
                (1024 if derive_bag_offsets else 0) | (2048 if reuse_activations else 0) |
                (4096 if fuse_quantize_stem else 0) | (8192 if split_k else 0))
        _check(lib().mi355x_host_compile(self._h, fn, opts))

    def describe(self, fn):
        n = _check(lib().mi355x_host_describe(self._h, fn, None, C.c_size_t(0)))
        buf = C.create_string_buffer(n)
        _check(lib().mi355x_host_describe(self._h, fn, buf, C.c_size_t(n)))
        return buf.value.decode()

    def bundle_sizes(self, fn):
        out = (C.c_uint64 * 4)()
        _check(lib().mi355x_host_bundle_sizes(self._h, fn, out))
        return dict(constants=out[0], generated=out[1], mutable=out[2], activations=out[3])


def conv_attrs(kernel, stride, pads, group=1, dilation=(1, 1), act=ACT_NONE):
    """The twelve integer attributes of the convolution kinds; pads are TLBR."""
    return [kernel[0], kernel[1], stride[0], stride[1], pads[0], pads[1], pads[2],
            pads[3], group, dilation[0], dilation[1], act]


def parse_listing(text):
    """describe() text -> list of dicts (one per setup/launch line)."""
    out = []
    for line in text.splitlines():
        parts = line.split()
        if not parts or parts[0] not in ("setup", "launch"):
            continue
        d = {"phase": parts[0], "kernel": parts[1]}
        for tok in parts[2:]:
            k, _, v = tok.partition("=")
            if v.startswith("["):
                d[k] = [int(x) for x in v.strip("[]").split(",") if x]
            else:
                try:
                    d[k] = int(v)
                except ValueError:
                    try:
                        d[k] = float(v)
                    except ValueError:
                        d[k] = v
        out.append(d)
    return out


def parse_activations(text):
    """describe() text -> {value id: dict(name, offset, bytes)} for the
    activations that have memory of their own."""
    out = {}
    for line in text.splitlines():
        parts = line.split()
        if not parts or parts[0] != "activation":
            continue
        d = dict(tok.partition("=")[::2] for tok in parts[1:])
        out[int(d["id"])] = dict(name=d["name"], offset=int(d["offset"]), bytes=int(d["bytes"]))
    return out


class DeviceManager:
    """use_launch_graphs: False = kernel by kernel; True = launch graphs with
    the default number of parallel branches; n > 1 = up to n branches (the first
    nine requests of a function compare its recordings with all branches, one
    chain and two branches; the fastest stays); -n = exactly n branches."""

    def __init__(self, device=0, memory_bytes=0, use_launch_graphs=True, slws_math=-1):
        """slws_math: arithmetic of this device manager's SparseLengths launches
        (capi.SLWS_MATH_*; -1 = the library's default), passed with every call."""
        self._h = C.c_void_p(lib().mi355x_host_dm_create_opts(
            device, C.c_uint64(memory_bytes), int(use_launch_graphs), int(slws_math)))
        self._modules = []

    def init(self):
        _check(lib().mi355x_host_dm_init(self._h))
        return self

    def stop(self):
        if self._h:
            _check(lib().mi355x_host_dm_stop(self._h))

    def __del__(self):
        try:
            if self._h:
                lib().mi355x_host_dm_destroy(self._h)
                self._h = None
        except Exception:
            pass

    def add_network(self, module, functions=None):
        """functions: indices of the compiled functions to load (default: all)."""
        if functions is None:
            _check(lib().mi355x_host_dm_add_network(self._h, module._h))
        else:
            fs = (C.c_int * len(functions))(*[int(f) for f in functions])
            _check(lib().mi355x_host_dm_add_functions(self._h, module._h, fs, len(functions)))
        self._modules.append(module)   # the device manager keeps pointers into it

    def transfer_static_placeholder(self, module, name, array):
        """transferStaticPlaceholderToDevice: host array -> the placeholder's
        device slot; later requests that do not bind it read this value."""
        assert array.flags["C_CONTIGUOUS"]
        _check(lib().mi355x_host_dm_transfer_static_placeholder(
            self._h, module._h, name.encode(), C.c_void_p(array.ctypes.data),
            C.c_size_t(array.nbytes)))

    def evict_network(self, name):
        _check(lib().mi355x_host_dm_evict_network(self._h, name.encode()))

    def run(self, name, bindings):
        """bindings: placeholder name -> numpy array (inputs read, outputs
        written in place)."""
        names = list(bindings)
        arrs = [bindings[n] for n in names]
        for a in arrs:
            assert a.flags["C_CONTIGUOUS"]
        cn = (C.c_char_p * len(names))(*[n.encode() for n in names])
        cb = (C.c_void_p * len(names))(*[a.ctypes.data for a in arrs])
        cs = (C.c_size_t * len(names))(*[a.nbytes for a in arrs])
        _check(lib().mi355x_host_dm_run(self._h, name.encode(), cn, cb, cs, len(names)))

    def time_function(self, name, iterations):
        """Average device milliseconds per replay, no host copies."""
        ms = C.c_float(0)
        _check(lib().mi355x_host_dm_time_function(self._h, name.encode(), int(iterations),
                                                  C.byref(ms)))
        return ms.value

    @property
    def maximum_memory(self):
        return lib().mi355x_host_dm_maximum_memory(self._h)

    @property
    def available_memory(self):
        return lib().mi355x_host_dm_available_memory(self._h)

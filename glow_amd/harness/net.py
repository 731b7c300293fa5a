"""A network as plain data: named tensors (type, role, payload) and a list of
lowered instructions over them. One description feeds both the host layer
(`to_module`) and, in the tests, a CPU executor built on the oracle."""
import numpy as np

from glow_amd import host as H

NP_DTYPE = {H.FLOAT: np.float32, H.FLOAT16: np.float16, H.INT8Q: np.int8, H.INT32Q: np.int32,
            H.INT32I: np.int32, H.INT64I: np.int64, H.UINT8_FUSED: np.uint8,
            H.UINT8_FUSED_FP16: np.uint8, H.UINT4_FUSED_FP16: np.uint8, H.UINT4_FUSED: np.uint8}


class Tensor:
    def __init__(self, name, kind, shape, role, scale=1.0, offset=0, data=None):
        self.name, self.kind, self.shape, self.role = name, kind, tuple(int(s) for s in shape), role
        self.scale, self.offset, self.data = float(np.float32(scale)), int(offset), data

    @property
    def dtype(self):
        return np.dtype(NP_DTYPE[self.kind])


class Op:
    def __init__(self, kind, name, operands, iattrs=(), fattrs=()):
        self.kind, self.name = kind, name
        self.operands = list(operands)          # tensor names, destination first
        self.iattrs, self.fattrs = list(iattrs), list(fattrs)


class Net:
    def __init__(self, name):
        self.name = name
        self.tensors = {}
        self.ops = []

    def _add(self, t):
        assert t.name not in self.tensors, t.name
        self.tensors[t.name] = t
        return t.name

    def constant(self, name, data, kind, scale=1.0, offset=0):
        data = np.ascontiguousarray(data, NP_DTYPE[kind])
        return self._add(Tensor(name, kind, data.shape, "constant", scale, offset, data))

    def placeholder(self, name, shape, kind, scale=1.0, offset=0):
        return self._add(Tensor(name, kind, shape, "placeholder", scale, offset))

    def activation(self, name, shape, kind, scale=1.0, offset=0):
        return self._add(Tensor(name, kind, shape, "activation", scale, offset))

    def view(self, name, source, shape, first=0):
        """The bytes of `source` under another shape (same kind and parameters),
        from element `first` of the source on (a slice of a placeholder's or
        constant's outermost dimension when not 0)."""
        s = self.tensors[source]
        t = Tensor(name, s.kind, shape, "view", s.scale, s.offset)
        t.source, t.first = source, int(first)
        assert t.first + int(np.prod(t.shape, dtype=np.int64)) <= int(np.prod(s.shape, dtype=np.int64))
        return self._add(t)

    def first_element(self, name):
        """Where `name` starts inside its root, in elements."""
        t = self.tensors[name]
        return t.first + self.first_element(t.source) if t.role == "view" else 0

    def root(self, name):
        t = self.tensors[name]
        return self.root(t.source) if t.role == "view" else name

    def op(self, kind, name, operands, iattrs=(), fattrs=()):
        for o in operands:
            assert o in self.tensors, o
        self.ops.append(Op(kind, name, operands, iattrs, fattrs))

    def ops_count(self):
        """2 x multiply-accumulates of the matrix-core instructions."""
        total = 0
        for o in self.ops:
            t = [self.tensors[n] for n in o.operands]
            if o.kind in (H.CONVOLUTION, H.CHANNELWISE_QUANTIZED_CONV):
                n, oh, ow, oc = t[0].shape
                _, kh, kw, icg = t[2].shape
                total += 2 * n * oh * ow * oc * kh * kw * icg
            elif o.kind in (H.FULLY_CONNECTED, H.ROWWISE_QUANTIZED_FC, H.MATMUL):
                m, k = t[1].shape
                total += 2 * m * k * t[0].shape[1]
        return total


def to_module(net, function="main"):
    """Net -> (host Module, function index)."""
    m = H.Module(net.name)
    ids = {}
    f = None
    for t in net.tensors.values():
        if t.role == "constant":
            ids[t.name] = m.constant(t.name, t.data, t.kind, t.scale, t.offset)
        elif t.role == "placeholder":
            ids[t.name] = m.placeholder(t.name, t.shape, t.kind, t.dtype, t.scale, t.offset)
    f = m.function(function)
    for t in net.tensors.values():
        if t.role == "activation":
            ids[t.name] = m.activation(f, t.name, t.shape, t.kind, t.scale, t.offset)
        elif t.role == "view":      # sources precede their views in insertion order
            if t.source not in ids:
                raise ValueError(f"view {t.name} precedes its source {t.source}")
            ids[t.name] = m.view(t.name, ids[t.source], t.shape, t.kind, t.scale, t.offset,
                                 byte_offset=t.first * t.dtype.itemsize)
    for o in net.ops:
        m.instruction(f, o.kind, o.name, [ids[n] for n in o.operands], o.iattrs, o.fattrs)
    return m, f

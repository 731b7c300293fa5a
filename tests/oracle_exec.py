"""Runs a glow_amd.harness.net.Net on the CPU with the oracle: every lowered
instruction is executed by the restated reference arithmetic, with the integer
parameters derived here (from the tensors' float scales, by the oracle's host
math, in the reference code generator's order, LLVMIRGen.cpp:1465-1499,
1670-1690, 1716-1771, 2222-2320, 2695-2798, 3003-3048) and not by the backend
under test."""
import numpy as np

from glow_amd import host as H
from oracle import glow_oracle as go


def _s(ratio):
    return go.quantize_scale_offset_32to8(float(np.float32(ratio)), 0)[:3]


def _f(x):
    return np.float32(x)


class _Values:
    """Tensor values by name; a view shares the storage of its source."""

    def __init__(self, net):
        self.net = net
        self.flat = {}

    def _storage(self, name):
        root = self.net.root(name)
        if root not in self.flat:
            t = self.net.tensors[root]
            self.flat[root] = np.zeros(int(np.prod(t.shape, dtype=np.int64)), t.dtype)
        return self.flat[root]

    def get(self, name):
        t = self.net.tensors[name]
        n = int(np.prod(t.shape, dtype=np.int64))
        at = self.net.first_element(name)
        return self._storage(name)[at:at + n].reshape(t.shape)

    def set(self, name, value):
        t = self.net.tensors[name]
        value = np.asarray(value)
        flat = self._storage(name)
        at = self.net.first_element(name)
        flat[at:at + value.size] = value.astype(t.dtype, copy=False).ravel()

    def __getitem__(self, name):
        return self.get(name)


def run(net, inputs):
    """inputs: placeholder name -> array (may be shorter than the placeholder).
    Returns the tensor values, indexable by name."""
    v = _Values(net)
    for t in net.tensors.values():
        if t.role == "constant":
            v.set(t.name, t.data)
    for k, x in inputs.items():
        v.set(k, x)
    T = net.tensors
    for o in net.ops:
        t = [T[n] for n in o.operands]
        a = [v.get(n) for n in o.operands]
        d = t[0]
        if o.kind == H.QUANTIZE:
            r = go.quantize_i8(a[1], d.scale, d.offset)
        elif o.kind == H.DEQUANTIZE:
            r = go.dequantize_i8(a[1], t[1].scale, t[1].offset)
        elif o.kind == H.RESCALE_QUANTIZED:
            r = go.rescale_i8(a[1], d.offset, t[1].offset, *_s(_f(t[1].scale) / _f(d.scale)))
        elif o.kind == H.ELEMENT_ADD:
            r = go.add_i8(a[1], a[2], d.offset, t[1].offset, t[2].offset,
                          _s(_f(t[1].scale) / _f(d.scale)), _s(_f(t[2].scale) / _f(d.scale)))
        elif o.kind == H.RELU:
            r = go.relu_i8(a[1], t[1].offset, d.offset, _s(_f(t[1].scale) / _f(d.scale)))
        elif o.kind == H.CLIP:
            # bounds quantized with the source tensor's parameters (LLVMIRGen.cpp:1515-1518)
            lo, hi = (int(np.clip(go.quantize_value_i32(x, t[1].scale, t[1].offset), -128, 127))
                      for x in o.fattrs)
            r = go.clip_elem_i8(a[1], lo, hi, t[1].offset, d.offset,
                                _s(_f(t[1].scale) / _f(d.scale)))
        elif o.kind == H.LEAKY_RELU:
            r = go.leaky_relu_i8(a[1], t[1].offset, d.offset, _s(_f(t[1].scale) / _f(d.scale)),
                                 _s(_f(t[1].scale) * _f(o.fattrs[0]) / _f(d.scale)))
        elif o.kind == H.CPU_MAX_SPLAT:
            val = int(np.clip(go.quantize_value_i32(o.fattrs[0], t[1].scale, t[1].offset),
                              -128, 127))
            r = go.max_splat_i8(a[1], val)
        elif o.kind == H.BATCHED_ADD:
            r = go.batched_add_i8(a[1], a[2], d.offset, t[1].offset, t[2].offset,
                                  _s(_f(t[1].scale) / _f(d.scale)),
                                  _s(_f(t[2].scale) / _f(d.scale)))
        elif o.kind == H.MAX_POOL:
            k = o.iattrs
            r = go.max_pool_i8(a[1], k[0:2], k[2:4], k[4:8], d.offset)
        elif o.kind == H.AVG_POOL:
            k = o.iattrs
            sc = _f(t[1].scale) / _f(d.scale)
            if k[8]:
                sc = sc / _f(k[0] * k[1])
            r = go.avg_pool_i8(a[1], k[0:2], k[2:4], k[4:8], k[8], d.offset, t[1].offset, _s(sc))
        elif o.kind == H.SOFTMAX:
            r = go.softmax_f32(a[1])
        elif o.kind == H.ROWWISE_QUANTIZED_FC:
            mm = _f(t[1].scale) * a[4].astype(np.float32)
            bp = np.array([_s(_f(t[3].scale) / m) for m in mm], np.int32)
            op = np.array([_s(m / _f(d.scale)) for m in mm], np.int32)
            r = go.rwq_fc_i8(a[1], a[2], a[3], a[5], bp[:, 0], bp[:, 1], bp[:, 2], op[:, 0],
                             op[:, 1], op[:, 2], d.offset, t[1].offset, t[3].offset)
        elif o.kind == H.CHANNELWISE_QUANTIZED_CONV:
            k = o.iattrs
            n, ih, iw, ic = t[1].shape
            oc = d.shape[3]
            g = go.conv_geom(n, ih, iw, ic, oc, (k[0], k[1]), (k[2], k[3]), tuple(k[4:8]),
                             k[8], (k[9], k[10]))
            mm = _f(t[1].scale) * a[4].astype(np.float32)
            bp = np.array([_s(b / m) for b, m in zip(a[6].astype(np.float32), mm)], np.int32)
            op = np.array([_s(m / _f(d.scale)) for m in mm], np.int32)
            act = k[11]
            args = ()
            if act == H.ACT_CLIP:
                args = tuple(go.quantize_value_i32(x, d.scale, d.offset) for x in o.fattrs)
            elif act == H.ACT_LEAKY_RELU:
                args = _s(o.fattrs[0])
            r = go.cwq_conv2d_i8(a[1], a[2], a[3], g, d.offset, t[1].offset, a[5], a[7],
                                 bp[:, 0], bp[:, 1], bp[:, 2], op[:, 0], op[:, 1], op[:, 2],
                                 act, args)
        elif o.kind in (H.FRWQ_SLS, H.FRWQ_SLWS):
            weighted = o.kind == H.FRWQ_SLWS
            data, w = a[1], (a[2] if weighted else None)
            idx, ln = (a[3], a[4]) if weighted else (a[2], a[3])
            kind = {H.UINT8_FUSED: go.U8_F32, H.UINT8_FUSED_FP16: go.U8_F16,
                    H.UINT4_FUSED_FP16: go.U4_F16, H.UINT4_FUSED: go.U4_F32}[t[1].kind]
            r = go.frwq_slws_generic(data, kind, w, idx, ln, out_f16=d.kind == H.FLOAT16,
                                     fp16_accum=bool(o.iattrs and o.iattrs[0]))
        elif o.kind == H.CONVERT_TO:
            r = a[1].astype(np.float32)
        elif o.kind == H.COPY:
            r = np.ascontiguousarray(a[1]).reshape(d.shape)
        elif o.kind == H.SIGMOID:
            r = go.sigmoid_f32(a[1])
        elif o.kind == H.INSERT_TENSOR:
            off = o.iattrs[0]
            a[0][:, off:off + a[1].shape[1]] = a[1]
            continue
        elif o.kind == H.TRANSPOSE:
            r = np.ascontiguousarray(np.transpose(a[1], o.iattrs))
        elif o.kind == H.GATHER:
            r = go.gather(a[1], a[2], o.iattrs[0])
        elif o.kind == H.BATCH_MATMUL:
            r = go.batch_matmul_i8(a[1], a[2], d.offset, t[1].offset, t[2].offset,
                                   _s(_f(t[1].scale) * _f(t[2].scale) / _f(d.scale)))
        else:
            raise NotImplementedError(f"instruction kind {o.kind}")
        v.set(d.name, r)
    return v

"""The workload generators of glow_amd.workloads with the integer parameters
derived by the ORACLE's restated host math instead of the library's own, so
that the parity tests do not depend on the code under test for their inputs."""
import numpy as np

from glow_amd import workloads as _w
from oracle import glow_oracle as go


class _OracleHost(_w.Host):
    def s32to8(self, scale, offset=0):
        return go.quantize_scale_offset_32to8(scale, offset)

    def quantize_value_i32(self, x, scale, offset):
        return go.quantize_value_i32(x, scale, offset)

    def conv_geom(self, *a, **kw):
        return go.conv_geom(*a, **kw)

    def conv3d_geom(self, *a, **kw):
        return go.conv3d_geom(*a, **kw)

    def fused_row_bytes(self, cols, kind):
        return go.fused_row_bytes(cols, kind)


_HOST = _OracleHost()


def s32to8_vec(ratios):
    return _w.s32to8_vec(ratios, _HOST)


def rwq_fc_case(*a, **kw):
    return _w.rwq_fc_case(*a, host=_HOST, **kw)


def fc_case(*a, **kw):
    return _w.fc_case(*a, host=_HOST, **kw)


def cwq_conv_case(*a, **kw):
    return _w.cwq_conv_case(*a, host=_HOST, **kw)


def cwq_conv3d_case(*a, **kw):
    return _w.cwq_conv3d_case(*a, host=_HOST, **kw)


rwq_fc_args = _w.rwq_fc_args
fc_args = _w.fc_args
cwq_conv_args = _w.cwq_conv_args
zipf_indices = _w.zipf_indices
random_fused_table = _w.random_fused_table
slws_batch = _w.slws_batch
slws_error_ratio = _w.slws_error_ratio


def element_op_cases(seed=700):
    """Parameter sets of the int8 element operators the CPU backend keeps
    un-lowered besides Relu: Clip, LeakyRelu, Max(x, Splat) and BatchedAdd. Each
    entry is (name, args) with args in the oracle wrappers' order; the scale
    parameters come from quantizeScaleOffset32To8 of the float ratios the
    reference's code generator forms (LLVMIRGen.cpp:1501-1590, 2322-2375)."""
    from oracle import glow_oracle as go
    rng = np.random.default_rng(seed)
    f32 = np.float32
    a = rng.integers(-128, 128, (3, 7, 5, 6)).astype(np.int8)
    a.ravel()[:256] = np.arange(-128, 128).astype(np.int8)     # every int8 value once
    out = []
    for i, (ss, ds, so, do, lo, hi) in enumerate([(0.1, 0.1, -20, -20, 0.0, 6.0),
                                                  (0.05, 0.2, 7, -128, -1.0, 1.0),
                                                  (0.4, 0.013, -128, -100, 0.0, 30.0),
                                                  (0.02, 0.02, 0, 0, -100.0, 100.0)]):
        dp = go.quantize_scale_offset_32to8(float(f32(ss) / f32(ds)), 0)[:3]
        # bounds quantized with the source tensor's parameters (Base.h:323-329)
        qlo = int(np.clip(np.rint(f32(lo) / f32(ss) + so), -128, 127))
        qhi = int(np.clip(np.rint(f32(hi) / f32(ss) + so), -128, 127))
        out.append((f"clip{i}", "clip_elem_i8", (a, qlo, qhi, so, do, dp)))
    for i, (ss, ds, so, do, alpha) in enumerate([(0.1, 0.1, -20, -20, 0.01), (0.05, 0.2, 7, -128, 0.2),
                                                 (0.4, 0.013, -128, -100, 0.5),
                                                 (0.03, 0.03, 0, 0, 1.0)]):
        pp = go.quantize_scale_offset_32to8(float(f32(ss) / f32(ds)), 0)[:3]
        npar = go.quantize_scale_offset_32to8(float(f32(ss) * f32(alpha) / f32(ds)), 0)[:3]
        out.append((f"leaky{i}", "leaky_relu_i8", (a, so, do, pp, npar)))
    for i, v in enumerate([-128, -20, 0, 57, 127]):
        out.append((f"maxsplat{i}", "max_splat_i8", (a, v)))
    batch = rng.integers(-128, 128, (9, 5, 12)).astype(np.int8)
    for i, (bs, sls, ds, bo, so, do, i32) in enumerate([(0.05, 0.07, 0.11, 3, -4, 5, False),
                                                        (0.3, 0.002, 0.1, -128, 0, -128, False),
                                                        (0.05, 0.0005, 0.06, 10, 0, -3, True),
                                                        (1.0, 1.0, 1.0, 0, 0, 0, True)]):
        bp = go.quantize_scale_offset_32to8(float(f32(bs) / f32(ds)), bo)[:3]
        sp = go.quantize_scale_offset_32to8(float(f32(sls) / f32(ds)), so)[:3]
        sl = (rng.integers(-20000, 20000, (5, 12)).astype(np.int32) if i32
              else rng.integers(-128, 128, (5, 12)).astype(np.int8))
        out.append((f"batchedadd{i}", "batched_add_i8", (batch, sl, do, bo, so, bp, sp)))
    # a slice that is not a multiple of four elements, and a single slice
    b2 = rng.integers(-128, 128, (4, 7)).astype(np.int8)
    out.append(("batchedadd_odd", "batched_add_i8",
                (b2, rng.integers(-128, 128, 7).astype(np.int8), 1, 2, 3, (0, 8, 300), (1, 9, 400))))
    out.append(("batchedadd_one", "batched_add_i8",
                (b2[:1], rng.integers(-999, 999, 7).astype(np.int32), 0, 0, 0, (0, 8, 256),
                 (0, 10, 700))))
    return out

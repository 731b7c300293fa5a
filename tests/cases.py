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

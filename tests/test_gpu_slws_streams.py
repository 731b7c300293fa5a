"""Lengths-mode SparseLengths launches with more than 4096 bags on two streams
at once: each stream has its own scratch for the bag-offset pre-pass, so
overlapping launches do not disturb each other's bag offsets.

Run on the GPU box:  python -u -m pytest tests -m gpu -x -v --timeout 120
"""
import numpy as np
import pytest

from glow_amd import capi
from oracle import glow_oracle as go
from tests import cases

pytestmark = pytest.mark.gpu


def _resident(batch, rows, bags, mean_len, seed):
    lengths, idx, w = cases.slws_batch(seed, rows, bags, mean_len, 1.05)
    return dict(lengths=lengths, idx=idx, w=w, d_len=capi.to_device(lengths),
                d_idx=capi.to_device(idx), d_w=capi.to_device(w),
                d_out=capi.DeviceBuffer.empty((bags, 128), np.float32))


def test_two_streams_with_20000_bags_each():
    capi.init(0)
    rng = np.random.default_rng(8)
    rows = 60_000
    table = cases.random_fused_table(rng, rows, 128)
    d_table = capi.to_device(table)
    # different lengths per stream: shared chunk sums would move bag offsets
    a = _resident(0, rows, 20_000, 7, 61)
    b = _resident(1, rows, 20_000, 3, 62)
    sa, sb = capi.Stream(), capi.Stream()
    for rep in range(20):
        for s, x in ((sa, a), (sb, b)):
            capi.launch_frwq_slws(x["d_out"], False, d_table, rows, capi.FUSED_U8_F32,
                                  x["d_w"], False, x["d_idx"], True, x["idx"].size,
                                  x["d_len"], x["lengths"].size, 136, 128, stream=s)
    sa.sync()
    sb.sync()
    for x in (a, b):
        want = go.frwq_slws_f32(table, x["w"], x["idx"], x["lengths"])
        np.testing.assert_array_equal(x["d_out"].numpy(), want)


def test_rowwise_table_lookup_on_two_streams():
    """RowwiseQuantizedSparseLengthsWeightedSum uses the same pre-pass."""
    capi.init(0)
    rng = np.random.default_rng(9)
    rows = 20_000
    data = rng.integers(0, 256, (rows, 64), dtype=np.uint8)
    scales = rng.uniform(0.01, 0.03, rows).astype(np.float32)
    offsets = rng.normal(-2, 0.3, rows).astype(np.float32)
    d = [capi.to_device(v) for v in (data, scales, offsets)]
    out = []
    streams = [capi.Stream(), capi.Stream()]
    import ctypes as C
    for k, st in enumerate(streams):
        lengths, idx, w = cases.slws_batch(70 + k, rows, 9000, 2 + 3 * k, 1.05)
        dl, di, dw = capi.to_device(lengths), capi.to_device(idx), capi.to_device(w)
        do = capi.DeviceBuffer.empty((9000, 64), np.float32)
        out.append((lengths, idx, w, dl, di, dw, do))
    for rep in range(10):
        for (lengths, idx, w, dl, di, dw, do), st in zip(out, streams):
            capi.check(capi.lib().mi355x_rwq_slws(
                capi._vp(do), capi._vp(d[0]), capi._sz(rows), capi._vp(d[1]), capi._vp(d[2]),
                capi._vp(dw), capi._vp(di), C.c_int(1), capi._sz(idx.size), capi._vp(dl),
                capi._sz(9000), capi._sz(64), capi._vp(st)))
    for st in streams:
        st.sync()
    for lengths, idx, w, dl, di, dw, do in out:
        want = go.rwq_slws_f32(data, scales, offsets, w, idx, lengths)
        np.testing.assert_array_equal(do.numpy(), want)

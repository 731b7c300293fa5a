"""mi355x_frwq_slws_noalloc: the SparseLengths entry point that allocates
nothing (the scratch of its bag-offset pre-pass is a fixed array inside the
library) against mi355x_frwq_slws on the same inputs, bit for bit, on calls in
a row that share the array: many bags, then fewer, then a batch that needs no
scratch at all, then many again.

Run on the GPU box:  python -u -m pytest tests -m gpu -x -v --timeout 120
"""
import ctypes as C

import numpy as np
import pytest

from glow_amd import capi
from oracle import glow_oracle as go
from tests import cases

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def _both(table, d_table, kind, lengths, idx, w, **kw):
    want = capi.frwq_slws(table, kind, w, idx, lengths, d_data=d_table, **kw)
    got = capi.frwq_slws(table, kind, w, idx, lengths, d_data=d_table, noalloc=True, **kw)
    return got, want


def _run_sequence():
    capi.init(0)
    rng = np.random.default_rng(5)
    rows = 50_000
    table = cases.random_fused_table(rng, rows, 128)
    d_table = capi.to_device(table)
    # calls in a row on one GPU: the second has fewer bags than the first
    for call, bags in enumerate((20_000, 9_000, 300, 20_001)):
        lengths, idx, w = cases.slws_batch(40 + call, rows, bags, 6, 1.05)
        say("noalloc call", call, "bags", bags, "lookups", int(lengths.sum()))
        got, want = _both(table, d_table, capi.FUSED_U8_F32, lengths, idx, w)
        np.testing.assert_array_equal(got, want)
        assert np.abs(got).max() > 0
        if call == 1:   # and the existing entry point is itself held to the oracle
            ref = go.frwq_slws_f32(table, w, idx, lengths)
            assert cases.slws_error_ratio(got, ref, table, w, idx, lengths) <= 1e-5
    capi.sync()


def test_noalloc_matches_the_allocating_entry_point_strict_arithmetic():
    _run_sequence()


@pytest.mark.fused_math
def test_noalloc_matches_the_allocating_entry_point_default_arithmetic():
    _run_sequence()


def test_noalloc_four_bit_fp16_rows_and_sum_without_weights():
    capi.init(0)
    rng = np.random.default_rng(6)
    rows = 30_000
    table = cases.random_fused_table(rng, rows, 64, capi.FUSED_U4_F16)
    d_table = capi.to_device(table)
    for call, bags in enumerate((12_000, 5_000)):
        lengths, idx, _ = cases.slws_batch(50 + call, rows, bags, 5, 1.1, np.int32, weighted=False)
        say("noalloc 4-bit call", call, "bags", bags)
        got, want = _both(table, d_table, capi.FUSED_U4_F16, lengths, idx, None, out_f16=True)
        np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))
        ref = go.frwq_slws_generic(table, go.U4_F16, None, idx, lengths, out_f16=True)
        np.testing.assert_array_equal(got.view(np.uint16), ref.view(np.uint16))


def test_noalloc_rejects_more_bags_than_its_scratch_holds():
    capi.init(0)
    too_many = 4096 * 4096 + 1
    one = capi.DeviceBuffer.empty((64,), np.uint8)
    with pytest.raises(capi.MI355XError) as e:
        capi.check(capi.lib().mi355x_frwq_slws_noalloc(
            capi._vp(one), C.c_int(0), capi._vp(one), capi._sz(1), C.c_int(capi.FUSED_U8_F32),
            capi._vp(None), C.c_int(0), capi._vp(one), C.c_int(1), capi._sz(0), capi._vp(one),
            capi._sz(too_many), capi._sz(136), capi._sz(128), C.c_int(0), capi._vp(None)))
    assert "at most" in str(e.value)

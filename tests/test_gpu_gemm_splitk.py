"""The matrix-core launch with its K loop split over workgroups (tile 12,
mi355x_launch_opts::workspace): every workgroup of an output tile leaves its
int32 sums in the caller's workspace and the last one to arrive adds them up
and requantises. Results are the oracle's bit for bit (the int32 sum wraps, so
the order of the partial sums does not matter: reference
lib/LLVMIRCodeGen/libjit/libjit_matmul.cpp:284-316, libjit_conv.cpp:151-239);
the workspace's counters are zero again after every launch."""
import numpy as np
import pytest

from glow_amd import capi
from oracle import glow_oracle as go
from tests import cases

pytestmark = pytest.mark.gpu

NOT_SUPPORTED = -4


def say(*a):
    print(*a, flush=True)


def _workspace(nbytes):
    ws = capi.DeviceBuffer(max(nbytes, 256))
    ws.fill(0)
    capi.sync()
    return ws


def _counters_are_zero(ws, M, N, groups=1):
    tiles = ((M + 127) // 128) * ((N + 127) // 128) * groups
    head = np.empty(ws.nbytes, np.uint8)
    capi.check(capi.lib().mi355x_memcpy_d2h(capi._vp(head), capi._vp(ws.ptr),
                                            capi._sz(min(ws.nbytes, 4 * tiles)), capi._vp(None)))
    capi.sync()
    return not head[:4 * tiles].any()


@pytest.mark.parametrize("shape", [(100, 128, 64), (256, 1024, 256), (300, 2048, 200),
                                   (129, 4096, 130), (1000, 704, 384)])
def test_named_tile_vs_oracle(shape):
    M, K, N = shape
    for seed, kw in ((1, {}), (2, dict(bias_i8=True, bias_scale=0.01, bias_offset=3)),
                     (3, dict(in_offset=0))):
        c = cases.rwq_fc_case(seed + M + K, M, K, N, symmetric=True, **kw)
        args = cases.rwq_fc_args(c)
        want = go.rwq_fc_i8(*args)
        need = capi.gemm_splitk_workspace_bytes(M, N, K, named=True)
        assert need > 0
        ws = _workspace(need)
        say("split K over workgroups", shape, kw, "workspace", need)
        opts = capi.LaunchOpts(gemm_tile=capi.TILE_SPLIT_K, workspace=ws)
        # twice on one workspace: the first launch leaves its counters zero
        for _ in range(2):
            got = capi.rwq_fc_i8(*args, opts=opts)
            np.testing.assert_array_equal(got, want)
            assert _counters_are_zero(ws, M, N)
        assert want.std() > 1


def test_convolution_on_the_named_tile():
    for IC, OC, hw in ((256, 256, 14), (512, 512, 7), (64, 128, 9)):
        c = cases.cwq_conv_case(5 + IC, 2, hw, hw, IC, OC)
        args = cases.cwq_conv_args(c)
        want = go.cwq_conv2d_i8(*args)
        g = c["geom"]
        M, K = g.N * g.OH * g.OW, g.KH * g.KW * IC
        ws = _workspace(capi.gemm_splitk_workspace_bytes(M, OC, K, named=True))
        say("split K over workgroups, convolution", IC, OC, hw)
        opts = capi.LaunchOpts(gemm_tile=capi.TILE_SPLIT_K, workspace=ws)
        for _ in range(2):
            np.testing.assert_array_equal(capi.cwq_conv2d_i8(*args, opts=opts), want)
        assert _counters_are_zero(ws, M, OC)


def test_the_library_splits_by_itself_when_given_a_workspace():
    """Few output tiles and a long K: the size query says a split would be used;
    with the workspace in the options (no tile named) the result is the oracle's,
    and the same launch without a workspace gives the same bytes."""
    M, K, N = 784, 4608, 256
    assert capi.gemm_splitk_workspace_bytes(M, N, K) > 0
    assert capi.gemm_splitk_workspace_bytes(16384, 1024, 1024) == 0    # the grid fills the chip
    assert capi.gemm_splitk_workspace_bytes(M, N, 256) == 0            # K too short to share
    c = cases.rwq_fc_case(77, M, K, N, symmetric=True)
    args = cases.rwq_fc_args(c)
    want = go.rwq_fc_i8(*args)
    ws = _workspace(capi.gemm_splitk_workspace_bytes(M, N, K))
    np.testing.assert_array_equal(capi.rwq_fc_i8(*args, opts=capi.LaunchOpts(workspace=ws)), want)
    np.testing.assert_array_equal(capi.rwq_fc_i8(*args), want)
    assert _counters_are_zero(ws, M, N)


def test_named_tile_refuses_what_it_cannot_run():
    c = cases.rwq_fc_case(9, 200, 1024, 256, symmetric=True)
    args = cases.rwq_fc_args(c)
    need = capi.gemm_splitk_workspace_bytes(200, 256, 1024, named=True)

    def refused(opts, a=args, **kw):
        with pytest.raises(capi.MI355XError) as e:
            capi.rwq_fc_i8(*a, opts=opts, **kw)
        assert e.value.code == NOT_SUPPORTED, e.value
        return True

    assert refused(capi.LaunchOpts(gemm_tile=capi.TILE_SPLIT_K))                       # no workspace
    assert refused(capi.LaunchOpts(gemm_tile=capi.TILE_SPLIT_K, workspace=_workspace(need // 2)))
    ws = _workspace(need)
    assert refused(capi.LaunchOpts(gemm_tile=capi.TILE_SPLIT_K, workspace=ws),
                   precomputed_sums=False)                                              # in-kernel sums
    c64 = cases.rwq_fc_case(10, 200, 64, 256, symmetric=True)                          # one K step
    assert capi.gemm_splitk_workspace_bytes(200, 256, 64, named=True) == 0
    assert refused(capi.LaunchOpts(gemm_tile=capi.TILE_SPLIT_K, workspace=ws),
                   a=cases.rwq_fc_args(c64))
    c72 = cases.rwq_fc_case(11, 200, 1000, 256, symmetric=True)                        # K % 64 != 0
    assert refused(capi.LaunchOpts(gemm_tile=capi.TILE_SPLIT_K, workspace=ws),
                   a=cases.rwq_fc_args(c72))
    # and the same options run where the kernel applies
    np.testing.assert_array_equal(
        capi.rwq_fc_i8(*args, opts=capi.LaunchOpts(gemm_tile=capi.TILE_SPLIT_K, workspace=ws)),
        go.rwq_fc_i8(*args))

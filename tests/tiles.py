"""Helpers of the tests that name a workgroup tile (a kernel) for a launch."""
import pytest

from glow_amd import capi

NOT_SUPPORTED = -4


class forced_tile:
    """The calling thread's default tile for the launches inside the block."""

    def __init__(self, tile):
        self.tile = tile

    def __enter__(self):
        capi.check(capi.lib().mi355x_gemm_tile_override(self.tile))

    def __exit__(self, *exc):
        capi.check(capi.lib().mi355x_gemm_tile_override(-1))
        return False


def refused(tile, launch):
    """A tile in 6..8 names one special kernel; a launch that kernel cannot
    serve must fail with MI355X_ERR_NOT_SUPPORTED rather than run another
    kernel under that number."""
    with forced_tile(tile), pytest.raises(capi.MI355XError) as e:
        launch()
    assert e.value.code == NOT_SUPPORTED, e.value
    return True


def forced_or_refused(tile, launch):
    """The launch's result under the named tile, or None when the kernel the
    tile names refuses it (any other failure is raised)."""
    with forced_tile(tile):
        try:
            return launch()
        except capi.MI355XError as e:
            if e.code != NOT_SUPPORTED:
                raise
            return None

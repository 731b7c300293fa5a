"""MI355X (gfx950) kernel library for Glow's quantized-inference hot path.

`glow_amd.capi` binds the C ABI declared in include/glow_mi355x.h; the HIP
sources are under glow_amd/csrc.
"""

"""Standalone model harnesses over the host layer, the counterpart of the
reference's tests/benchmark programs: they build a quantized network as a
module of lowered instructions, hand it to MI355XBackend / MI355XDeviceManager
and time it."""

"""CPU checker for the MI355X quantized-inference path (test infrastructure).

Only tests, the smoke check and the CPU-baseline leg of the benchmark import
this package; nothing in ``glow_amd`` does.
"""

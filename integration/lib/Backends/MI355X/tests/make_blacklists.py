#!/usr/bin/env python3
"""Writes the per-backend test lists of lib/Backends/MI355X/tests from a Glow
checkout, in the form Glow's backend-parameterised unittests expect
(`std::set<std::string> glow::backendTestBlacklist`, see
lib/Backends/CPU/tests/CPUOperatorTest.cpp and tests/unittests/BackendTestUtils.h).

The MI355X backend covers the quantized-inference path only, so the rule is the
reverse of the CPU backend's: every TEST_P of a suite is black-listed unless
its name is in ALLOW below. ALLOW holds tests whose graphs stay inside
MI355XBackend::isOpSupported (Quantize / Dequantize / Save around the int8
operators and the fused-rowwise lookups); it is to be widened as tests are
confirmed inside a Glow build with the backend linked in.

Test names that a suite generates through macros with token pasting are not
seen by the regular expression here; `<suite> --gtest_list_tests` in a Glow
build gives the authoritative list, and the script accepts such a listing with
--listing.

usage: make_blacklists.py <glow checkout> [--listing Suite=file ...]
"""
import os
import re
import sys

SUITES = {
    # output file                        unittest source                test class(es)
    "MI355XOperatorTest.cpp": ("OperatorTest.cpp", ("OperatorTest", "OperatorStatelessTest")),
    "MI355XDeviceManagerTest.cpp": ("DeviceManagerTest.cpp", ("DeviceManagerTest",)),
    "MI355XQuantizationTest.cpp": ("QuantizationTest.cpp", ("Operator", "InterpAndCPU", "Quantization")),
    "MI355XRecommendationSystemTest.cpp": ("RecommendationSystemTest.cpp", ("RecommendationSystemTest",)),
    "MI355XBackendCorrectnessTest.cpp": ("BackendCorrectnessTest.cpp", ("BackendCorrectnessTest",)),
    "MI355XHostManagerTest.cpp": ("HostManagerTest.cpp", ("HostManagerTest",)),
    # training, tracing and graph-optimizer suites: nothing applies
    "MI355XGradCheckTest.cpp": ("GradCheckTest.cpp", ("GradCheck",)),
    "MI355XOperatorGradTest.cpp": ("OperatorGradTest.cpp", ("OperatorGradTest",)),
    "MI355XMLTest.cpp": ("MLTest.cpp", ("MLTest",)),
    "MI355XTraceEventsTest.cpp": ("TraceEventsTest.cpp", ("TraceEventsTest",)),
}

ALLOW = {
    "MI355XOperatorTest.cpp": {
        # ChannelwiseQuantizedConvolution (reference libjit_conv.cpp:151-239)
        "ChannelwiseQuantizedConv2D", "ChannelwiseQuantizedConv2D_Int32Bias_SmallFilterData",
        "ChannelwiseQuantizedConv2D_Int32Bias_ZeroBiasData",
        "ChannelwiseQuantizedConv2D_NonZero_QuantizedBias",
        # ... and its NTHWC form (libjit_conv.cpp:244-349)
        "ChannelwiseQuantizedConv3D",
        # fused-rowwise pooled lookups (libjit.cpp:1253-1276, 2416-2481;
        # InterpreterNodes.cpp:5764-5889)
        "FusedRowwiseQuantizedSparseLengthsWeightedSum_Float",
        "FusedRowwiseQuantizedSparseLengthsWeightedSum_Float16_AccumFloat",
        "FusedRowwiseQuantizedSparseLengthsWeightedSum_Float16_AccumFloat16",
        "FusedRowwiseQuantizedSparseLengthsSum_Float",
        "FusedRowwiseQuantizedSparseLengthsSum_Float16_AccumFloat",
        "FusedRowwiseQuantizedSparseLengthsSum_Float16_AccumFloat16",
        "FusedRowwiseQuantizedSLWSTwoColumn_Float",
        "FusedRowwiseQuantizedSLWSTwoColumn_Float16_AccumFloat",
        "FusedRowwiseQuantizedSLWSTwoColumn_Float16_AccumFloat16",
        "FusedRowwiseQuantizedSLWSAllLengthsOne_Float",
        "EmbeddingBagByteRowwiseOffsets_Float", "EmbeddingBagByteRowwiseOffsets_Float_End_Offset",
        "EmbeddingBagByteRowwiseOffsets_Float_End_Offset_Partial",
        "RowwiseQuantizedSparseLengthsWeightedSum_Float",
        "RowwiseQuantizedSparseLengthsWeightedSum_Float_Int32",
        # int8 glue
        "Int8AvgPool", "Int8AvgPoolCountExcludePads", "Int8MaxPool", "Relu_Int8",
        "GatherDataInt8IdxInt32", "GatherDataInt8IdxInt64", "QuantizeSimpleInt8",
        "QuantizeSimpleInt16", "QuantizeSimpleInt32",
        "TestQuantizedRescaleSequence",
        # Transpose of 2 to 6 dimensions, any plain element kind (libjit.cpp:565-653)
        "Transpose2Dims", "FP16Transpose2Dims", "BoolTranspose2Dims", "Transpose6Dims",
        "Transpose3Dims_Float", "Transpose3Dims_Float16", "Transpose3Dims_Int8",
        # RowwiseQuantizedFullyConnected / FullyConnected
        "rowwiseQuantizedFCTest_Int8_BiasInt8", "rowwiseQuantizedFCTest_Int8_BiasInt32",
        "rowwiseQuantizedFCTestSymmetric",
        "Int8ConvolutionDepth10", "Int8ConvolutionDepth8",
    },
    # DeviceManagerTest builds a float Tanh graph, QuantizationTest and
    # RecommendationSystemTest mix float operators into their graphs: all
    # outside the path. The device-manager contract is covered on int8 graphs
    # by the kernel library's own tests (tests/test_gpu_device_manager.py).
    "MI355XDeviceManagerTest.cpp": set(),
    "MI355XQuantizationTest.cpp": set(),
    "MI355XRecommendationSystemTest.cpp": set(),
}

HEADER = '''/**
 * Tests of {source} the MI355X backend does not run: every test of the
 * suite except those whose graphs stay on the quantized-inference path.
 * GENERATED by lib/Backends/MI355X/tests/make_blacklists.py from the TEST_P
 * names of tests/unittests/{source}; NOT COMPILED in the repository this file
 * ships in.
 */
#include "tests/unittests/BackendTestUtils.h"

using namespace glow;

std::set<std::string> glow::backendTestBlacklist = {{
'''


def test_names(path, classes):
    text = open(path, errors="replace").read()
    names = []
    for cls, name in re.findall(r"TEST_P\(\s*(\w+)\s*,\s*(\w+)\s*\)", text):
        if cls in classes and "##" not in name and name not in names:
            names.append(name)
    return names


def main():
    if len(sys.argv) < 2:
        sys.exit(__doc__)
    glow = sys.argv[1]
    listings = dict(a.split("=", 1) for a in sys.argv[3:]) if "--listing" in sys.argv else {}
    here = os.path.dirname(os.path.abspath(__file__))
    for out, (source, classes) in SUITES.items():
        src = os.path.join(glow, "tests", "unittests", source)
        if not os.path.exists(src):
            print("skipped (no such file):", src)
            continue
        names = test_names(src, classes)
        if out in listings:
            for line in open(listings[out]):
                m = re.match(r"\s+(\w+)/0", line)
                if m and m.group(1) not in names:
                    names.append(m.group(1))
        allow = ALLOW.get(out, set())
        unknown = sorted(allow - set(names))
        if unknown:
            print(f"{out}: allow-listed names not found in {source}: {unknown}")
        with open(os.path.join(here, out), "w") as f:
            f.write(HEADER.format(source=source))
            for n in names:
                if n not in allow:
                    f.write(f'    "{n}/0",\n')
            f.write("};\n")
        print(f"{out}: {len(names)} tests, {len(set(names) & allow)} enabled")


if __name__ == "__main__":
    main()

"""The int8 ResNet-50 harness: the description builds and compiles on the CPU;
on the GPU the whole network, run through MI355XDeviceManager, gives the same
int8 logits as the oracle executing the same quantized graph instruction by
instruction (bit-exact), and the same fp32 probabilities within 1e-5."""
import numpy as np
import pytest

from glow_amd import host as H
from glow_amd.harness import net as netlib
from glow_amd.harness import resnet50
from tests import oracle_exec

SMALL = ((16, 2, 1), (32, 1, 2))     # two stages are enough to cover every block shape


def _small(batch=2, size=32, classes=10):
    return resnet50.make(batch=batch, size=size, profile_images=4, seed=3, layers=SMALL,
                         classes=classes)


def test_structure_of_the_full_network():
    steps = resnet50.build_fp32(0)
    convs = [s for s in steps if s[0] == "conv"]
    assert len(convs) == 53                      # 1 stem + 16 blocks x 3 + 4 shortcuts
    assert sum(1 for s in steps if s[0] == "add") == 16
    assert steps[-1][3][0].shape == (1000, 2048)


def test_small_network_compiles_and_fuses():
    net = _small()
    m, f = netlib.to_module(net)
    m.compile(f)
    rows = H.parse_listing(m.describe(f))
    kernels = [r["kernel"] for r in rows if r["phase"] == "launch"]
    # stem, 3 blocks x 3, 1 shortcut; the last convolution of each block takes
    # the residual add and the Relu with it
    assert kernels.count("mi355x_cwq_conv2d_i8") == 1 + 3 * 2 + 1
    assert kernels.count("mi355x_cwq_conv2d_add_i8") == 3
    assert "mi355x_add_relu_i8" not in kernels and "mi355x_add_i8" not in kernels
    m2, f2 = netlib.to_module(net)
    m2.compile(f2, fuse_conv_add=False, space_to_depth_stem=False)
    k2 = [r["kernel"] for r in H.parse_listing(m2.describe(f2)) if r["phase"] == "launch"]
    assert k2.count("mi355x_add_relu_i8") == 3 and k2.count("mi355x_cwq_conv2d_i8") == 11
    # the 7x7 stride-2 stem over 3 channels runs as a 4x4 stride-1 convolution
    # over a space-to-depth image of 16 channels, which is quantized from the
    # float input while it is re-laid
    # the int8 logits become probabilities in one launch
    assert kernels[-1] == "mi355x_dequantize_softmax" and "mi355x_dequantize_i8" not in kernels
    m4, f4 = netlib.to_module(net)
    m4.compile(f4, fuse_dequantize_sigmoid=False)
    k4 = [r["kernel"] for r in H.parse_listing(m4.describe(f4)) if r["phase"] == "launch"]
    assert k4[-2:] == ["mi355x_dequantize_i8", "mi355x_softmax_f32"] and k4[:-2] == kernels[:-1]
    assert kernels[0] == "mi355x_quantize_space_to_depth2_i8" and "mi355x_quantize_i8" not in kernels
    m3, f3 = netlib.to_module(net)
    m3.compile(f3, fuse_quantize_stem=False)
    k3 = [r["kernel"] for r in H.parse_listing(m3.describe(f3)) if r["phase"] == "launch"]
    assert k3[:2] == ["mi355x_quantize_i8", "mi355x_space_to_depth2_i8"] and k3[2:] == kernels[1:]
    assert k2[0] == "mi355x_quantize_i8" and "mi355x_space_to_depth2_i8" not in k2
    stem = [r for r in rows if r.get("space_to_depth") == 1][0]
    assert (stem["KH"], stem["KW"], stem["IC"], stem["IH"]) == (4, 4, 16, 16 + 3)
    # post-ReLU tensors use the unsigned range: offset -128
    assert net.tensors["stem"].offset == -128
    assert net.ops_count() > 0


def test_oracle_executes_the_small_network():
    net = _small(batch=1)
    x = resnet50.synthetic_images(9, 1, 32)
    v = oracle_exec.run(net, {"input": x})
    assert v["prob"].shape == (1, 10)
    np.testing.assert_allclose(v["prob"].sum(), 1.0, rtol=1e-5)
    assert len(np.unique(v["logits_q"])) > 1


@pytest.mark.gpu
@pytest.mark.parametrize("fuse", [(True, True, True), (True, False, False), (False, False, True),
                                  (True, True, True, False)])
def test_device_matches_oracle(fuse):
    net = resnet50.make(batch=2, size=64, profile_images=4, seed=5,
                        layers=((64, 2, 1), (128, 2, 2), (256, 1, 2)), classes=100)
    m, f = netlib.to_module(net)
    m.compile(f, fuse_conv_add=fuse[0], fuse_add_relu=fuse[1], space_to_depth_stem=fuse[2],
              fuse_quantize_stem=len(fuse) < 4)
    dm = H.DeviceManager().init()
    try:
        dm.add_network(m)
        x = resnet50.synthetic_images(11, 2, 64)
        logits = np.zeros((2, 100), np.int8)
        prob = np.zeros((2, 100), np.float32)
        dm.run("main", {"input": x, "logits_q": logits, "prob": prob})
        want = oracle_exec.run(net, {"input": x})
        np.testing.assert_array_equal(logits, want["logits_q"])
        np.testing.assert_allclose(prob, want["prob"], rtol=1e-5, atol=1e-30)
        # a second batch through the same resident network
        x2 = resnet50.synthetic_images(12, 2, 64)
        dm.run("main", {"input": x2, "logits_q": logits, "prob": prob})
        np.testing.assert_array_equal(logits, oracle_exec.run(net, {"input": x2})["logits_q"])
        assert dm.time_function("main", 3) > 0
    finally:
        dm.stop()


def test_batch_as_independent_chains_is_the_same_network_on_the_oracle():
    """The batch computed as chains over slices of the input and output
    placeholders (views that start inside their source, constants shared)
    gives the single chain's outputs; in the launch list no chain's launch
    depends on another chain's before the outputs."""
    steps = resnet50.build_fp32(3, SMALL, 10)
    ranges = resnet50.profile(steps, resnet50.synthetic_images(4, 4, 32))
    one = resnet50.build_int8(steps, ranges, 4, 32)
    two = resnet50.build_int8(steps, ranges, 4, 32, chains=2)
    assert len(two.ops) == 2 * len(one.ops)
    assert sum(t.role == "constant" for t in two.tensors.values()) == \
        sum(t.role == "constant" for t in one.tensors.values())
    x = resnet50.synthetic_images(9, 4, 32)
    a, b = oracle_exec.run(one, {"input": x}), oracle_exec.run(two, {"input": x})
    np.testing.assert_array_equal(a["logits_q"], b["logits_q"])
    np.testing.assert_array_equal(a["prob"], b["prob"])
    m, f = netlib.to_module(two)
    m.compile(f)
    rows = [r for r in H.parse_listing(m.describe(f)) if r["phase"] == "launch"]
    levels = {c: [r["level"] for r in rows if r["inst"].split("+")[0].endswith(f"@{c}")]
              for c in (0, 1)}
    # (the launches that write the shared output placeholders are ordered)
    assert levels[0][:-3] == levels[1][:-3] and levels[0][0] == 0


def test_views_that_start_inside_their_source():
    m = H.Module("views")
    p = m.placeholder("p", (4, 8), H.INT8Q, np.int8, 0.1, 0)
    f = m.function("main")
    act = m.activation(f, "a", (4, 8), H.INT8Q, 0.1, 0)
    assert m.view("rows23", p, (2, 8), H.INT8Q, 0.1, 0, byte_offset=16) >= 0
    with pytest.raises(H.HostError):
        m.view("past_the_end", p, (2, 8), H.INT8Q, 0.1, 0, byte_offset=24)
    with pytest.raises(H.HostError):        # activations are placed by the backend
        m.view("of_activation", act, (2, 8), H.INT8Q, 0.1, 0, byte_offset=16)


@pytest.mark.gpu
@pytest.mark.parametrize("chains", [2, 4])
def test_device_runs_the_batch_as_independent_chains(chains):
    steps = resnet50.build_fp32(5, ((64, 2, 1), (128, 1, 2)), 100)
    ranges = resnet50.profile(steps, resnet50.synthetic_images(6, 4, 64))
    net = resnet50.build_int8(steps, ranges, 4, 64, chains=chains)
    m, f = netlib.to_module(net)
    m.compile(f)
    dm = H.DeviceManager().init()
    try:
        dm.add_network(m)
        # more requests than the device manager spends on choosing a recording
        for seed in range(12):
            x = resnet50.synthetic_images(20 + seed, 4, 64)
            logits = np.zeros((4, 100), np.int8)
            prob = np.zeros((4, 100), np.float32)
            dm.run("main", {"input": x, "logits_q": logits, "prob": prob})
            want = oracle_exec.run(net, {"input": x})
            np.testing.assert_array_equal(logits, want["logits_q"])
            np.testing.assert_allclose(prob, want["prob"], rtol=1e-5, atol=1e-30)
    finally:
        dm.stop()

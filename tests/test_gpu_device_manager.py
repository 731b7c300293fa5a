"""MI355XDeviceManager on the GPU, in the shape of the reference's
DeviceManagerTest (tests/unittests/DeviceManagerTest.cpp:132-673): add a
network, run it, run it again, several functions and modules, eviction, memory
accounting and the error codes; every result is compared with the oracle."""
import numpy as np
import pytest

from glow_amd import host as H
from tests import cases, host_cases
from oracle import glow_oracle as go

pytestmark = pytest.mark.gpu


@pytest.fixture
def dm():
    d = H.DeviceManager().init()
    yield d
    d.stop()


def _rwq_expected(c, x=None):
    args = list(cases.rwq_fc_args(c))
    if x is not None:
        args[0] = x
    return go.rwq_fc_i8(*args)


def test_basic(dm):
    c = cases.rwq_fc_case(11, 32, 256, 192)
    m, f = host_cases.rwq_fc_module(c)
    m.compile(f)
    dm.add_network(m)
    out = np.zeros((32, 192), np.int8)
    dm.run("main", {"input": c["x"], "output": out})
    assert np.array_equal(out, _rwq_expected(c))


@pytest.mark.parametrize("graphs", [True, False])
def test_product_with_its_k_loop_split_over_workgroups(graphs):
    """Few output tiles and a long K: the compiled launch carries a workspace and
    the library splits its K loop; request after request gives the oracle's
    bytes (the workspace's counters are left zero by every launch), also while
    the device manager times the launch's candidate tiles."""
    d = H.DeviceManager(use_launch_graphs=graphs).init()
    try:
        c = cases.rwq_fc_case(31, 300, 4608, 256, symmetric=True)
        m, f = host_cases.rwq_fc_module(c)
        m.compile(f)
        assert "splitk_workspace" in [r for r in H.parse_listing(m.describe(f))
                                      if r["kernel"] == "mi355x_rwq_fc_i8"][0]
        d.add_network(m)
        rng = np.random.default_rng(1)
        for _ in range(12):
            x = rng.integers(-128, 128, c["x"].shape).astype(np.int8)
            out = np.zeros((300, 256), np.int8)
            d.run("main", {"input": x, "output": out})
            assert np.array_equal(out, _rwq_expected(c, x))
    finally:
        d.stop()


@pytest.mark.parametrize("graphs", [True, False])
def test_multi_run(graphs):
    d = H.DeviceManager(use_launch_graphs=graphs).init()
    try:
        c = cases.rwq_fc_case(12, 16, 128, 64, symmetric=False)
        m, f = host_cases.rwq_fc_module(c)
        m.compile(f)
        d.add_network(m)
        rng = np.random.default_rng(0)
        for _ in range(4):
            x = rng.integers(-128, 128, c["x"].shape).astype(np.int8)
            out = np.zeros((16, 64), np.int8)
            d.run("main", {"input": x, "output": out})
            assert np.array_equal(out, _rwq_expected(c, x))
    finally:
        d.stop()


def test_pipeline_quantize_fc_dequantize(dm):
    """Quantize -> RWQ-FC -> Rescale -> Dequantize through activations."""
    c = cases.rwq_fc_case(13, 8, 64, 48)
    M, K, N = 8, 64, 48
    m = H.Module("pipe")
    xin = m.placeholder("input", (M, K), H.FLOAT, np.float32)
    yout = m.placeholder("output", (M, N), H.FLOAT, np.float32)
    w = m.constant("weights", c["w"], H.INT8Q)
    b = m.constant("bias", c["bias"], H.INT32Q, c["bias_scale_f"], c["bias_offset"])
    sc = m.constant("scales", c["w_scales"])
    of = m.constant("offsets", c["w_offsets"], H.INT32I)
    f = m.function("main")
    q = m.activation(f, "q", (M, K), H.INT8Q, c["in_scale_f"], c["in_offset"])
    y = m.activation(f, "y", (M, N), H.INT8Q, c["out_scale_f"], c["out_offset"])
    z = m.activation(f, "z", (M, N), H.INT8Q, 0.23, 5)
    m.instruction(f, H.QUANTIZE, "quant", [q, xin])
    m.instruction(f, H.ROWWISE_QUANTIZED_FC, "fc", [y, q, w, b, sc, of])
    m.instruction(f, H.RESCALE_QUANTIZED, "rescale", [z, y])
    m.instruction(f, H.DEQUANTIZE, "dequant", [yout, z])
    m.compile(f)
    dm.add_network(m)
    rng = np.random.default_rng(1)
    x = rng.normal(0, 2.0, (M, K)).astype(np.float32)
    out = np.zeros((M, N), np.float32)
    dm.run("main", {"input": x, "output": out})
    xq = go.quantize_i8(x, c["in_scale_f"], c["in_offset"])
    yq = _rwq_expected(c, xq)
    pre, post, scale, _ = go.quantize_scale_offset_32to8(
        float(np.float32(c["out_scale_f"]) / np.float32(0.23)), 0)
    zq = go.rescale_i8(yq, 5, c["out_offset"], pre, post, scale)
    want = go.dequantize_i8(zq, 0.23, 5)
    assert np.array_equal(out, want)


def test_multi_function_and_eviction(dm):
    c1 = cases.rwq_fc_case(14, 8, 64, 32)
    c2 = cases.cwq_conv_case(15, 2, 10, 10, 16, 32, in_offset=-3)
    m1, f1 = host_cases.rwq_fc_module(c1, name="fc_net")
    m2, f2 = host_cases.cwq_conv_module(c2, name="conv_net")
    m1.compile(f1)
    m2.compile(f2)
    before = dm.available_memory
    dm.add_network(m1)
    dm.add_network(m2)
    assert dm.available_memory < before
    o1 = np.zeros((8, 32), np.int8)
    g = c2["geom"]
    o2 = np.zeros((g.N, g.OH, g.OW, g.OC), np.int8)
    dm.run("fc_net", {"input": c1["x"], "output": o1})
    dm.run("conv_net", {"input": c2["x"], "output": o2})
    assert np.array_equal(o1, _rwq_expected(c1))
    assert np.array_equal(o2, go.cwq_conv2d_i8(*cases.cwq_conv_args(c2)))
    dm.evict_network("fc_net")
    with pytest.raises(H.HostError) as e:
        dm.run("fc_net", {"input": c1["x"], "output": o1})
    assert e.value.code_name == "RUNTIME_NET_NOT_FOUND"
    with pytest.raises(H.HostError) as e:
        dm.evict_network("fc_net")
    assert e.value.code_name == "RUNTIME_NET_NOT_FOUND"
    # the other network is untouched, and the name can be used again
    o2[:] = 0
    dm.run("conv_net", {"input": c2["x"], "output": o2})
    assert np.array_equal(o2, go.cwq_conv2d_i8(*cases.cwq_conv_args(c2)))
    dm.add_network(m1)
    o1[:] = 0
    dm.run("fc_net", {"input": c1["x"], "output": o1})
    assert np.array_equal(o1, _rwq_expected(c1))
    dm.evict_network("fc_net")
    dm.evict_network("conv_net")
    assert dm.available_memory == before


def test_two_functions_of_one_module_share_its_constants(dm):
    c = cases.rwq_fc_case(16, 8, 64, 32)
    m, f = host_cases.rwq_fc_module(c, name="a")
    # second function of the same module: rescale of the same input
    g = m.function("b")
    vals = {n: i for i, n in enumerate(["input", "output", "weights", "bias", "scales", "offsets"])}
    r = m.placeholder("rescaled", (8, 64), H.INT8Q, np.int8, 0.11, -1)
    m.instruction(g, H.RESCALE_QUANTIZED, "r", [r, vals["input"]])
    m.compile(f)
    m.compile(g)
    dm.add_network(m)
    out = np.zeros((8, 32), np.int8)
    dm.run("a", {"input": c["x"], "output": out})
    assert np.array_equal(out, _rwq_expected(c))
    res = np.zeros((8, 64), np.int8)
    dm.run("b", {"input": c["x"], "rescaled": res})
    pre, post, scale, _ = go.quantize_scale_offset_32to8(
        float(np.float32(c["in_scale_f"]) / np.float32(0.11)), 0)
    assert np.array_equal(res, go.rescale_i8(c["x"], -1, c["in_offset"], pre, post, scale))


def test_duplicate_name_and_out_of_memory():
    c = cases.rwq_fc_case(17, 8, 64, 32)
    m, f = host_cases.rwq_fc_module(c)
    m.compile(f)
    small = H.DeviceManager(memory_bytes=1024).init()
    try:
        assert small.maximum_memory == 1024
        with pytest.raises(H.HostError) as e:
            small.add_network(m)
        assert e.value.code_name == "RUNTIME_OUT_OF_DEVICE_MEMORY"
        assert small.available_memory == 1024
    finally:
        small.stop()
    d = H.DeviceManager().init()
    try:
        d.add_network(m)
        with pytest.raises(H.HostError) as e:
            d.add_network(m)
        assert "already have a function called main" in str(e.value)
    finally:
        d.stop()


def test_partial_input_tensor(dm):
    """A bound tensor smaller than its placeholder fills the front of it
    (DeviceManagerTest PartialTensorCopy)."""
    m = H.Module()
    a = m.placeholder("a", (4, 16), H.INT8Q, np.int8, 0.5, 0)
    b = m.placeholder("b", (4, 16), H.FLOAT, np.float32)
    f = m.function("main")
    m.instruction(f, H.DEQUANTIZE, "d", [b, a])
    m.compile(f)
    dm.add_network(m)
    full = np.arange(64, dtype=np.int8).reshape(4, 16)
    out = np.zeros((4, 16), np.float32)
    dm.run("main", {"a": full, "b": out})
    assert np.array_equal(out, full.astype(np.float32) * 0.5)
    half = (np.arange(32, dtype=np.int8) - 7).reshape(2, 16)
    out2 = np.zeros((2, 16), np.float32)
    dm.run("main", {"a": half, "b": out2})
    assert np.array_equal(out2, half.astype(np.float32) * 0.5)
    too_big = np.zeros((5, 16), np.int8)
    with pytest.raises(H.HostError):
        dm.run("main", {"a": too_big, "b": out})


def test_slws_network(dm):
    rng = np.random.default_rng(18)
    rows, cols, bags = 5000, 128, 300
    table = cases.random_fused_table(rng, rows, cols)
    lengths, idx, w = cases.slws_batch(19, rows, bags, 12, 1.05, np.int64)
    n = idx.size + 50      # statically sized index/weight tensors, only sum(lengths) used
    m = H.Module("slws")
    data = m.constant("data", table, H.UINT8_FUSED)
    wv = m.placeholder("weights", (n,), H.FLOAT, np.float32)
    iv = m.placeholder("indices", (n,), H.INT64I, np.int64)
    lv = m.placeholder("lengths", (bags,), H.INT32I, np.int32)
    out = m.placeholder("output", (bags, cols), H.FLOAT, np.float32)
    f = m.function("main")
    m.instruction(f, H.FRWQ_SLWS, "slws", [out, data, wv, iv, lv], [0])
    m.compile(f)
    dm.add_network(m)
    res = np.zeros((bags, cols), np.float32)
    dm.run("main", {"weights": w, "indices": idx, "lengths": lengths, "output": res})
    assert np.array_equal(res, go.frwq_slws_f32(table, w, idx, lengths))


def test_slws_network_bag_positions_follow_every_upload(dm):
    """The lookup reads bag positions that the device manager derives from the
    lengths it uploads: per request, for a partial lengths tensor (the missing
    bags are empty), and after transferStaticPlaceholderToDevice."""
    rng = np.random.default_rng(28)
    rows, cols, bags = 3000, 64, 200
    table = cases.random_fused_table(rng, rows, cols)
    m = H.Module("slws_positions")
    data = m.constant("data", table, H.UINT8_FUSED)
    n = 4000
    wv = m.placeholder("weights", (n,), H.FLOAT, np.float32)
    iv = m.placeholder("indices", (n,), H.INT64I, np.int64)
    lv = m.placeholder("lengths", (bags,), H.INT32I, np.int32)
    out = m.placeholder("output", (bags, cols), H.FLOAT, np.float32)
    f = m.function("main")
    m.instruction(f, H.FRWQ_SLWS, "slws", [out, data, wv, iv, lv], [0])
    m.compile(f)
    assert "mi355x_frwq_slws_offsets" in m.describe(f)
    dm.add_network(m)
    res = np.zeros((bags, cols), np.float32)
    for seed, mean in ((1, 12), (2, 3), (3, 15)):
        lengths, idx, w = cases.slws_batch(seed, rows, bags, mean, 1.05, np.int64)
        lengths[seed] = -4     # a negative length is an empty bag
        dm.run("main", {"weights": w, "indices": idx, "lengths": lengths, "output": res})
        want = go.frwq_slws_f32(table, w, idx, np.maximum(lengths, 0))
        np.testing.assert_array_equal(res, want)
    # half the lengths: the other bags are empty
    lengths, idx, w = cases.slws_batch(4, rows, bags, 10, 1.05, np.int64)
    half = lengths[:bags // 2].copy()
    dm.run("main", {"weights": w, "indices": idx, "lengths": half, "output": res})
    padded = np.r_[half, np.zeros(bags - half.size, np.int32)].astype(np.int32)
    np.testing.assert_array_equal(res, go.frwq_slws_f32(table, w, idx, padded))
    # lengths sent on their own, then a request that does not bind them
    lengths, idx, w = cases.slws_batch(5, rows, bags, 8, 1.05, np.int64)
    dm.transfer_static_placeholder(m, "lengths", lengths)
    dm.run("main", {"weights": w, "indices": idx, "output": res})
    np.testing.assert_array_equal(res, go.frwq_slws_f32(table, w, idx, lengths))


def _two_lookup_functions(table, bags, cols, n, writer=False, derive_second=True):
    """One module, one lengths placeholder, two functions that each pool the
    same table over it (into outputs of their own); `writer` adds a third
    function that copies another placeholder into the lengths on the device."""
    m = H.Module("shared_lengths")
    data = m.constant("data", table, H.UINT8_FUSED)
    wv = m.placeholder("weights", (n,), H.FLOAT, np.float32)
    iv = m.placeholder("indices", (n,), H.INT64I, np.int64)
    lv = m.placeholder("lengths", (bags,), H.INT32I, np.int32)
    out_a = m.placeholder("out_a", (bags, cols), H.FLOAT, np.float32)
    out_b = m.placeholder("out_b", (bags, cols), H.FLOAT, np.float32)
    fw = None
    if writer:
        src = m.placeholder("new_lengths", (bags,), H.INT32I, np.int32)
        fw = m.function("set_lengths")
        m.instruction(fw, H.COPY, "store", [lv, src])
    fa = m.function("a")
    m.instruction(fa, H.FRWQ_SLWS, "slws_a", [out_a, data, wv, iv, lv], [0])
    fb = m.function("b")
    m.instruction(fb, H.FRWQ_SLS, "sls_b", [out_b, data, iv, lv], [0])
    return m, fa, fb, fw


def test_bag_positions_of_every_function_of_a_module_follow_an_upload(dm):
    """The lengths placeholder belongs to the module: a request to one function
    that binds new lengths must also refresh the bag positions of the module's
    other functions, which read the same slot without binding it."""
    rng = np.random.default_rng(41)
    rows, cols, bags, n = 2000, 64, 150, 3000
    table = cases.random_fused_table(rng, rows, cols)
    m, fa, fb, _ = _two_lookup_functions(table, bags, cols, n)
    m.compile(fa)
    m.compile(fb)
    assert "mi355x_frwq_slws_offsets" in m.describe(fa) and "_offsets" in m.describe(fb)
    dm.add_network(m)
    ra, rb = np.zeros((bags, cols), np.float32), np.zeros((bags, cols), np.float32)
    ones = np.ones(n, np.float32)
    for seed, mean in ((1, 12), (2, 4)):
        lengths, idx, w = cases.slws_batch(seed, rows, bags, mean, 1.05, np.int64)
        dm.run("a", {"weights": w, "indices": idx, "lengths": lengths, "out_a": ra})
        np.testing.assert_array_equal(ra, go.frwq_slws_f32(table, w, idx, lengths))
        # b reads the lengths a's request left in the module's slot
        dm.run("b", {"indices": idx, "out_b": rb})
        np.testing.assert_array_equal(rb, go.frwq_slws_f32(table, ones[:idx.size], idx, lengths))
    # a partial lengths tensor after longer ones: the rest of the slot is cleared,
    # so both functions see empty bags there
    lengths, idx, w = cases.slws_batch(3, rows, bags, 9, 1.05, np.int64)
    half = lengths[:bags // 3].copy()
    padded = np.r_[half, np.zeros(bags - half.size, np.int32)].astype(np.int32)
    dm.run("b", {"indices": idx, "lengths": half, "out_b": rb})
    np.testing.assert_array_equal(rb, go.frwq_slws_f32(table, ones[:idx.size], idx, padded))
    dm.run("a", {"weights": w, "indices": idx, "out_a": ra})
    np.testing.assert_array_equal(ra, go.frwq_slws_f32(table, w, idx, padded))


def test_lengths_written_on_the_device_are_not_summed_on_the_host(dm):
    """A function of the module that writes the lengths placeholder: the lookups
    compiled after it read the lengths themselves; one compiled before it (with
    positions from the host) cannot share a device with it."""
    rng = np.random.default_rng(42)
    rows, cols, bags, n = 1500, 64, 90, 2000
    table = cases.random_fused_table(rng, rows, cols)
    m, fa, fb, fw = _two_lookup_functions(table, bags, cols, n, writer=True)
    for f in (fw, fa, fb):
        m.compile(f)
    assert "_offsets" not in m.describe(fa) and "_offsets" not in m.describe(fb)
    dm.add_network(m)
    ra = np.zeros((bags, cols), np.float32)
    lengths, idx, w = cases.slws_batch(7, rows, bags, 10, 1.05, np.int64)
    dm.run("set_lengths", {"new_lengths": lengths})
    dm.run("a", {"weights": w, "indices": idx, "out_a": ra})
    np.testing.assert_array_equal(ra, go.frwq_slws_f32(table, w, idx, lengths))


def test_fc_and_conv_networks(dm):
    c = cases.fc_case(20, 24, 96, 80)
    m, f = host_cases.fc_module(c)
    m.compile(f)
    dm.add_network(m)
    out = np.zeros((24, 80), np.int8)
    dm.run("main", {"input": c["x"], "output": out})
    assert np.array_equal(out, go.fc_i8(*cases.fc_args(c)))
    dm.evict_network("main")
    for act in (cases._w.ACT_CLIP, cases._w.ACT_LEAKY_RELU):
        cc = cases.cwq_conv_case(21, 2, 12, 12, 32, 32, act=act, in_offset=4, symmetric=False)
        mc, fc = host_cases.cwq_conv_module(cc)
        mc.compile(fc)
        dm.add_network(mc)
        g = cc["geom"]
        o = np.zeros((g.N, g.OH, g.OW, g.OC), np.int8)
        dm.run("main", {"input": cc["x"], "output": o})
        assert np.array_equal(o, go.cwq_conv2d_i8(*cases.cwq_conv_args(cc)))
        dm.evict_network("main")


def test_wide_kinds_transposes_and_3d_convolution_networks(dm):
    """Quantize -> RescaleQuantized -> Dequantize through int16 and int32
    tensors, transposes beyond the two tiled shuffles, and the NTHWC
    convolution, each as a function on the device manager."""
    rng = np.random.default_rng(41)
    x = rng.normal(0, 40, (32, 50)).astype(np.float32)
    m = H.Module("wide")
    px = m.placeholder("x", x.shape, H.FLOAT, np.float32)
    f = m.function("main")
    outs = {}
    for kind, tag, bits in ((H.INT16Q, "i16", 16), (H.INT32Q, "i32", 32)):
        q = m.activation(f, f"q_{tag}", x.shape, kind, 0.01, 3)
        r = m.activation(f, f"r_{tag}", x.shape, kind, 0.02, -5)
        y = m.placeholder(f"y_{tag}", x.shape, H.FLOAT, np.float32)
        m.instruction(f, H.QUANTIZE, f"quant_{tag}", [q, px])
        m.instruction(f, H.RESCALE_QUANTIZED, f"rescale_{tag}", [r, q])
        m.instruction(f, H.DEQUANTIZE, f"dequant_{tag}", [y, r])
        pre, post, sc, _ = go.quantize_scale_offset_32to8(float(np.float32(0.01) / np.float32(0.02)), 0)
        want = go.dequantize_wide(
            go.rescale_wide(go.quantize_wide(x, 0.01, 3, bits), -5, 3, pre, post, sc), 0.02, -5)
        outs[f"y_{tag}"] = (np.zeros(x.shape, np.float32), want)
    t = rng.integers(-128, 128, (3, 16, 9, 11)).astype(np.int8)
    pt = m.placeholder("t_in", t.shape, H.INT8Q, np.int8, 0.1, 1)
    po = m.placeholder("t_out", (3, 9, 11, 16), H.INT8Q, np.int8, 0.1, 1)
    m.instruction(f, H.TRANSPOSE, "nchw2nhwc", [po, pt], [0, 2, 3, 1])
    ft = rng.normal(0, 1, (7, 5, 3)).astype(np.float32)
    pf = m.placeholder("f_in", ft.shape, H.FLOAT, np.float32)
    pfo = m.placeholder("f_out", (3, 7, 5), H.FLOAT, np.float32)
    m.instruction(f, H.TRANSPOSE, "float_t", [pfo, pf], [2, 0, 1])
    m.compile(f)
    dm.add_network(m)
    t_out, f_out = np.zeros((3, 9, 11, 16), np.int8), np.zeros((3, 7, 5), np.float32)
    bind = {"x": x, "t_in": t, "f_in": ft, "t_out": t_out, "f_out": f_out}
    bind.update({k: v[0] for k, v in outs.items()})
    dm.run("main", bind)
    for k, (got, want) in outs.items():
        np.testing.assert_array_equal(got, want, err_msg=k)
    np.testing.assert_array_equal(t_out, t.transpose(0, 2, 3, 1))
    np.testing.assert_array_equal(f_out, ft.transpose(2, 0, 1))
    dm.evict_network("main")

    kernel, stride, pads = (2, 3, 3), (1, 2, 1), (1, 0, 1, 1, 0, 2)
    c = cases.cwq_conv3d_case(43, N=2, T=4, H=9, W=8, IC=8, OC=12, kernel=kernel, stride=stride,
                              pads=pads, act=cases._w.ACT_CLIP, in_offset=6, symmetric=False)
    mc, fc = host_cases.cwq_conv3d_module(c, kernel, stride, pads)
    mc.compile(fc)
    dm.add_network(mc)
    g = c["geom"]
    o = np.zeros((g.N, g.OT, g.OH, g.OW, g.OC), np.int8)
    dm.run("main", {"input": c["x"], "output": o})
    np.testing.assert_array_equal(o, go.cwq_conv3d_i8(*cases.cwq_conv_args(c)))
    dm.evict_network("main")


def test_other_lookup_forms(dm):
    """RowwiseQuantizedSparseLengthsWeightedSum and EmbeddingBagByteRowwiseOffsets
    as instructions of one function."""
    rng = np.random.default_rng(23)
    rows, cols, bags = 800, 32, 60
    data = rng.integers(0, 256, (rows, cols), dtype=np.uint8)
    scales = rng.uniform(0.001, 0.1, rows).astype(np.float32)
    offs = rng.normal(0, 1, rows).astype(np.float32)
    fused = cases.random_fused_table(rng, rows, cols)
    lengths = rng.poisson(5, bags).astype(np.int32)
    n = int(lengths.sum())
    idx = rng.integers(0, rows, n).astype(np.int32)
    w = rng.random(n).astype(np.float32)
    starts = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)     # with the end offset
    m = H.Module("lookups")
    c_data = m.constant("data", data, H.INT8Q)
    c_sc = m.constant("scales", scales)
    c_of = m.constant("offsets", offs)
    c_fused = m.constant("fused", fused, H.UINT8_FUSED)
    p_w = m.placeholder("weights", (n,), H.FLOAT, np.float32)
    p_i = m.placeholder("indices", (n,), H.INT32I, np.int32)
    p_l = m.placeholder("lengths", (bags,), H.INT32I, np.int32)
    p_s = m.placeholder("starts", (bags + 1,), H.INT32I, np.int32)
    o1 = m.placeholder("out_rwq", (bags, cols), H.FLOAT, np.float32)
    o2 = m.placeholder("out_bag", (bags, cols), H.FLOAT, np.float32)
    f = m.function("main")
    m.instruction(f, H.RWQ_SLWS, "rwq", [o1, c_data, c_sc, c_of, p_w, p_i, p_l])
    m.instruction(f, H.EMBEDDING_BAG_BYTE_ROWWISE_OFFSETS, "bag", [o2, c_fused, p_w, p_i, p_s], [1])
    m.compile(f)
    dm.add_network(m)
    r1 = np.zeros((bags, cols), np.float32)
    r2 = np.zeros((bags, cols), np.float32)
    dm.run("main", {"weights": w, "indices": idx, "lengths": lengths, "starts": starts,
                    "out_rwq": r1, "out_bag": r2})
    np.testing.assert_array_equal(r1, go.rwq_slws_f32(data, scales, offs, w, idx, lengths))
    np.testing.assert_array_equal(
        r2, go.embedding_bag_byte_rowwise_offsets_f32(fused, w, idx, starts, True))


def test_multi_module(dm):
    """Two modules built the same way under different function names, both
    resident, both run (reference DeviceManagerTest.cpp:488 MultiModule)."""
    c = cases.rwq_fc_case(31, 8, 64, 32, symmetric=False)
    m1, f1 = host_cases.rwq_fc_module(c, name="func1")
    m2, f2 = host_cases.rwq_fc_module(c, name="func2")
    m1.compile(f1)
    m2.compile(f2)
    dm.add_network(m1)
    dm.add_network(m2)
    rng = np.random.default_rng(3)
    x1 = rng.integers(-128, 128, c["x"].shape).astype(np.int8)
    x2 = rng.integers(-128, 128, c["x"].shape).astype(np.int8)
    o1, o2 = np.zeros((8, 32), np.int8), np.zeros((8, 32), np.int8)
    dm.run("func1", {"input": x1, "output": o1})
    dm.run("func2", {"input": x2, "output": o2})
    # each module has its own placeholders: the second run did not disturb the first
    assert np.array_equal(o1, _rwq_expected(c, x1))
    assert np.array_equal(o2, _rwq_expected(c, x2))


def test_reuse_module(dm):
    """The functions of ONE module added by two addNetwork calls; both see the
    module's placeholders and constants (reference DeviceManagerTest.cpp:573
    ReuseModule)."""
    c = cases.rwq_fc_case(32, 8, 64, 32)
    m, f = host_cases.rwq_fc_module(c, name="func1")
    g = m.function("func2")
    r = m.placeholder("func2_output", (8, 64), H.INT8Q, np.int8, 0.07, 2)
    m.instruction(g, H.RESCALE_QUANTIZED, "r", [r, 0])      # value 0 is "input"
    m.compile(f)
    m.compile(g)
    before = dm.available_memory
    dm.add_network(m, functions=[f])
    after_first = dm.available_memory
    dm.add_network(m, functions=[g])
    # the module's constants and placeholders were made resident once
    assert before - after_first > after_first - dm.available_memory >= 0
    out = np.zeros((8, 32), np.int8)
    dm.run("func1", {"input": c["x"], "output": out})
    assert np.array_equal(out, _rwq_expected(c))
    res = np.zeros((8, 64), np.int8)
    dm.run("func2", {"input": c["x"], "func2_output": res})
    pre, post, scale, _ = go.quantize_scale_offset_32to8(
        float(np.float32(c["in_scale_f"]) / np.float32(0.07)), 0)
    assert np.array_equal(res, go.rescale_i8(c["x"], 2, c["in_offset"], pre, post, scale))
    # the same name cannot be added twice
    with pytest.raises(H.HostError):
        dm.add_network(m, functions=[g])
    dm.evict_network("func1")
    res[:] = 0
    dm.run("func2", {"input": c["x"], "func2_output": res})
    assert np.array_equal(res, go.rescale_i8(c["x"], 2, c["in_offset"], pre, post, scale))
    dm.evict_network("func2")
    assert dm.available_memory == before


def test_transfer_static_placeholder(dm):
    """transferStaticPlaceholderToDevice (reference DeviceManagerTest.cpp:239):
    a placeholder filled once on the device serves later requests that do not
    bind it."""
    c = cases.rwq_fc_case(33, 8, 64, 32, symmetric=False)
    m, f = host_cases.rwq_fc_module(c)
    m.compile(f)
    dm.add_network(m)
    rng = np.random.default_rng(5)
    static_x = rng.integers(-128, 128, c["x"].shape).astype(np.int8)
    dm.transfer_static_placeholder(m, "input", static_x)
    for _ in range(2):
        out = np.zeros((8, 32), np.int8)
        dm.run("main", {"output": out})            # "input" is not bound
        assert np.array_equal(out, _rwq_expected(c, static_x))
    # a bound tensor still replaces it for that and later requests
    out = np.zeros((8, 32), np.int8)
    dm.run("main", {"input": c["x"], "output": out})
    assert np.array_equal(out, _rwq_expected(c))
    with pytest.raises(H.HostError):
        dm.transfer_static_placeholder(m, "weights", static_x)       # a constant
    with pytest.raises(H.HostError):
        dm.transfer_static_placeholder(m, "nothing", static_x)
    with pytest.raises(H.HostError):
        dm.transfer_static_placeholder(m, "input", np.zeros(10_000, np.int8))   # too large
    other, f2 = host_cases.rwq_fc_module(c, name="elsewhere")
    with pytest.raises(H.HostError):
        dm.transfer_static_placeholder(other, "input", static_x)    # module not resident


def test_copy_into_an_output_placeholder(dm):
    """RWQ-FC into an activation, then a Copy into the output placeholder (the
    shape a Save node takes when the optimizer cannot write in place)."""
    c = cases.rwq_fc_case(34, 8, 64, 32)
    m = H.Module("copied")
    x = m.placeholder("input", (8, 64), H.INT8Q, np.int8, c["in_scale_f"], c["in_offset"])
    out = m.placeholder("output", (256,), H.INT8Q, np.int8, c["out_scale_f"], c["out_offset"])
    w = m.constant("weights", c["w"], H.INT8Q)
    b = m.constant("bias", c["bias"], H.INT32Q, c["bias_scale_f"], c["bias_offset"])
    sc = m.constant("scales", c["w_scales"].astype(np.float32))
    of = m.constant("offsets", c["w_offsets"].astype(np.int32), H.INT32I)
    f = m.function("main")
    y = m.activation(f, "y", (8, 32), H.INT8Q, c["out_scale_f"], c["out_offset"])
    m.instruction(f, H.ROWWISE_QUANTIZED_FC, "fc", [y, x, w, b, sc, of])
    m.instruction(f, H.COPY, "save", [out, y])
    m.compile(f)
    dm.add_network(m)
    got = np.zeros(256, np.int8)
    dm.run("main", {"input": c["x"], "output": got})
    assert np.array_equal(got.reshape(8, 32), _rwq_expected(c))


def test_chains_that_wait_for_each_other_in_a_ring():
    """Three chains of adds where the second waits for the first, the third for
    the second and the first, further on, for the third: recorded on one side
    stream per chain, the waits between the streams would run in a circle. The
    recording must come out (with fewer streams) and compute the same sums."""
    n, shape = 4, (64, 256)
    m = H.Module()
    ty = (H.INT8Q, np.int8, 0.1, 0)
    ins = [m.placeholder(f"in{i}", shape, *ty) for i in range(n)]
    outs = [m.placeholder(f"out{i}", shape, *ty) for i in range(n)]
    f = m.function("main")
    act = lambda name: m.activation(f, name, shape, H.INT8Q, 0.1, 0)
    ops = []                       # (dest, lhs, rhs) by name, for the restatement below

    def add(dest, lhs, rhs, names):
        m.instruction(f, H.ELEMENT_ADD, names[0], [dest, lhs, rhs])
        ops.append(names)

    v = {}
    for i in range(n):             # every chain starts on its own
        v[f"c{i}_0"] = act(f"c{i}_0")
        add(v[f"c{i}_0"], ins[i], ins[i], (f"c{i}_0", f"in{i}", f"in{i}"))
    # chain 0 is long (it keeps the capturing stream); 1 -> 2 -> 3 -> 1 cross over
    for k in range(1, 5):
        v[f"c0_{k}"] = act(f"c0_{k}")
        add(v[f"c0_{k}"], v[f"c0_{k-1}"], ins[0], (f"c0_{k}", f"c0_{k-1}", "in0"))
    v["c2_1"] = act("c2_1"); add(v["c2_1"], v["c2_0"], v["c1_0"], ("c2_1", "c2_0", "c1_0"))
    v["c3_1"] = act("c3_1"); add(v["c3_1"], v["c3_0"], v["c2_1"], ("c3_1", "c3_0", "c2_1"))
    v["c1_1"] = act("c1_1"); add(v["c1_1"], v["c1_0"], v["c3_1"], ("c1_1", "c1_0", "c3_1"))
    v["c2_2"] = act("c2_2"); add(v["c2_2"], v["c2_1"], v["c1_1"], ("c2_2", "c2_1", "c1_1"))
    for i, last in enumerate(["c0_4", "c1_1", "c2_2", "c3_1"]):
        add(outs[i], v[last], ins[i], (f"out{i}", last, f"in{i}"))
    m.compile(f)
    rng = np.random.default_rng(5)
    x = {f"in{i}": rng.integers(-20, 21, shape).astype(np.int8) for i in range(n)}
    one = go.quantize_scale_offset_32to8(1.0, 0)[:3]
    want = dict(x)
    for dest, lhs, rhs in ops:
        want[dest] = go.add_i8(want[lhs], want[rhs], 0, 0, 0, one, one)
    for graphs in (-4, True, False):
        dm = H.DeviceManager(use_launch_graphs=graphs).init()
        try:
            dm.add_network(m)
            for _ in range(2):
                got = {f"out{i}": np.zeros(shape, np.int8) for i in range(n)}
                dm.run("main", dict(x, **got))
                for i in range(n):
                    np.testing.assert_array_equal(got[f"out{i}"], want[f"out{i}"])
        finally:
            dm.stop()

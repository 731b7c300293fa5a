"""CPU tests of the backend's host layer: the flat C view exports what its
header declares; MI355XBackend::compile derives the same integer kernel
parameters from float scales as the oracle's restatement of the reference code
generator (LLVMIRGen.cpp:2161-2320, 2695-2798); unsupported instructions and a
missing device come back as the reference's error codes."""
import os
import re

import numpy as np
import pytest

from glow_amd import capi
from glow_amd import host as H
from tests import cases, host_cases
from oracle import glow_oracle as go

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_exports_match_header():
    text = open(os.path.join(ROOT, "include", "glow_mi355x_host.h")).read()
    declared = sorted(set(re.findall(r"\b(mi355x_host_[a-z0-9_]+)\s*\(", text)))
    assert declared == sorted(H.EXPORTS)
    L = H.lib()
    for name in declared:
        assert hasattr(L, name), name


def test_host_library_does_not_link_the_oracle():
    import subprocess
    out = subprocess.run(["ldd", os.path.join(ROOT, "glow_amd", "libglow_mi355x_host.so")],
                         capture_output=True, text=True).stdout
    assert "oracle" not in out and "libjit" not in out
    assert "libglow_mi355x.so" in out


def _launch(m, f, kernel):
    rows = [r for r in H.parse_listing(m.describe(f)) if r["kernel"] == kernel and r["phase"] == "launch"]
    assert len(rows) == 1
    return rows[0]


@pytest.mark.parametrize("seed,symmetric,bias_i8", [(1, True, False), (2, False, False), (3, True, True)])
def test_rwqfc_parameters(seed, symmetric, bias_i8):
    c = cases.rwq_fc_case(seed, 8, 64, 48, symmetric=symmetric, bias_i8=bias_i8,
                          bias_scale=0.01 if bias_i8 else 5e-5,
                          bias_offset=-2 if bias_i8 else 0)
    m, f = host_cases.rwq_fc_module(c, bias_i8=bias_i8)
    m.compile(f)
    r = _launch(m, f, "mi355x_rwq_fc_i8")
    for k in ("bias_pre", "bias_post", "bias_scale", "out_pre", "out_post", "out_scale"):
        assert r[k] == c[k].tolist(), k
    assert (r["M"], r["K"], r["N"]) == (8, 64, 48)
    assert r["out_offset"] == c["out_offset"] and r["in_offset"] == c["in_offset"]
    assert r["bias_offset"] == c["bias_offset"] and r["bias_is_i8"] == int(bias_i8)
    assert r["weights_offsets_all_zero"] == int(symmetric)
    # row sums are only worth forming when the input offset is non-zero
    setup = [x for x in H.parse_listing(m.describe(f)) if x["phase"] == "setup"]
    assert (len(setup) == 1) == (c["in_offset"] != 0)


def test_fc_parameters():
    c = cases.fc_case(4, 8, 32, 24)
    m, f = host_cases.fc_module(c)
    m.compile(f)
    r = _launch(m, f, "mi355x_fc_i8")
    assert (r["bias_pre"], r["bias_post"], r["bias_scale"]) == tuple(c["biasP"])
    assert (r["out_pre"], r["out_post"], r["out_scale"]) == tuple(c["outP"])
    assert r["weights_offset"] == c["w_offset"] and r["repack"] == 0
    kernels = [x["kernel"] for x in H.parse_listing(m.describe(f)) if x["phase"] == "setup"]
    assert kernels[0] == "mi355x_transpose2d_i8"     # [K x N] -> [N x K] once, at load


@pytest.mark.parametrize("act", [cases._w.ACT_NONE, cases._w.ACT_RELU, cases._w.ACT_CLIP,
                                 cases._w.ACT_LEAKY_RELU])
def test_cwq_conv_parameters(act):
    c = cases.cwq_conv_case(5, 2, 9, 9, 16, 32, act=act, in_offset=-7, symmetric=False)
    m, f = host_cases.cwq_conv_module(c)
    m.compile(f)
    r = _launch(m, f, "mi355x_cwq_conv2d_i8")
    for k in ("bias_pre", "bias_post", "bias_scale", "out_pre", "out_post", "out_scale"):
        assert r[k] == c[k].tolist(), k
    want = list(c["act_args"]) + [0] * (3 - len(c["act_args"]))
    assert r["act_args"] == want and r["act"] == act
    g = c["geom"]
    assert (r["OH"], r["OW"], r["OC"], r["KH"], r["KW"]) == (g.OH, g.OW, g.OC, g.KH, g.KW)
    assert r["filter_offsets_all_zero"] == 0


def test_rescale_parameters():
    m = H.Module()
    a = m.placeholder("a", (5, 7), H.INT8Q, np.int8, 0.37, -4)
    b = m.placeholder("b", (5, 7), H.INT8Q, np.int8, 0.05, 9)
    f = m.function("main")
    m.instruction(f, H.RESCALE_QUANTIZED, "r", [b, a])
    m.compile(f)
    r = _launch(m, f, "mi355x_rescale_i8")
    pre, post, scale, _ = go.quantize_scale_offset_32to8(float(np.float32(0.37) / np.float32(0.05)), 0)
    assert (r["pre"], r["post"], r["scale"]) == (pre, post, scale)
    assert (r["in_offset"], r["out_offset"], r["n"]) == (-4, 9, 35)


def test_memory_plan_is_aligned_and_disjoint():
    c = cases.rwq_fc_case(1, 8, 64, 48)
    m, f = host_cases.rwq_fc_module(c)
    m.compile(f)
    s = m.bundle_sizes(f)
    # weights 48*64, bias 48*4, scales 48*4, offsets 48*4, each rounded to 64
    assert s["constants"] == 3072 + 192 * 3
    assert s["mutable"] == 8 * 64 + 8 * 48 + (64 - (8 * 48) % 64) % 64
    assert s["generated"] >= 6 * 192 and s["generated"] % 64 == 0
    assert s["activations"] == 0


def _slws_module(data_kind, dest_kind, w_kind):
    m = H.Module()
    row = {H.UINT8_FUSED: 16 + 8, H.UINT8_FUSED_FP16: 16 + 4,
           H.UINT4_FUSED_FP16: 8 + 4, H.UINT4_FUSED: 8 + 8}[data_kind]
    data = m.placeholder("data", (10, row), data_kind, np.uint8)
    dest = m.placeholder("dest", (3, 16), dest_kind, np.float32)
    w = m.placeholder("w", (12,), w_kind, np.float32)
    idx = m.placeholder("idx", (12,), H.INT64I, np.int64)
    ln = m.placeholder("len", (3,), H.INT32I, np.int32)
    return m, [dest, data, w, idx, ln]


def test_slws_type_legality_follows_the_reference():
    # fp32-scale data: (float weights, float result) or (f16, f16) only;
    # fp16-scale data: float16 result, float or float16 weights.
    ok = [(H.UINT8_FUSED, H.FLOAT, H.FLOAT), (H.UINT8_FUSED, H.FLOAT16, H.FLOAT16),
          (H.UINT4_FUSED_FP16, H.FLOAT16, H.FLOAT), (H.UINT4_FUSED_FP16, H.FLOAT16, H.FLOAT16),
          (H.UINT8_FUSED_FP16, H.FLOAT16, H.FLOAT16), (H.UINT4_FUSED, H.FLOAT, H.FLOAT)]
    bad = [(H.UINT8_FUSED, H.FLOAT, H.FLOAT16), (H.UINT8_FUSED, H.FLOAT16, H.FLOAT),
           (H.UINT4_FUSED_FP16, H.FLOAT, H.FLOAT), (H.UINT8_FUSED_FP16, H.FLOAT, H.FLOAT16)]
    for d, r, w in ok:
        m, ops = _slws_module(d, r, w)
        assert m.is_op_supported(H.FRWQ_SLWS, ops, [0])[0], (d, r, w)
    for d, r, w in bad:
        m, ops = _slws_module(d, r, w)
        assert not m.is_op_supported(H.FRWQ_SLWS, ops, [0])[0], (d, r, w)


def test_unsupported_instructions_are_compile_errors():
    m = H.Module()
    a = m.placeholder("a", (4, 4), H.FLOAT, np.float32)
    b = m.placeholder("b", (4, 4), H.FLOAT, np.float32)
    f = m.function("main")
    m.instruction(f, H.QUANTIZE, "q", [b, a])          # float -> float
    with pytest.raises(H.HostError) as e:
        m.compile(f)
    assert e.value.code_name == "COMPILE_UNSUPPORTED_NODE_AFTER_OPTIMIZE"
    f2 = m.function("other")
    m.instruction(f2, 77, "mystery", [b, a])
    with pytest.raises(H.HostError) as e:
        m.compile(f2)
    assert e.value.code_name == "COMPILE_UNSUPPORTED_NODE_AFTER_OPTIMIZE"
    # fused Sigmoid/Tanh are rejected for quantized convolutions like on the CPU backend
    c = cases.cwq_conv_case(5, 1, 5, 5, 16, 16, act=cases._w.ACT_RELU)
    c["act"] = cases._w.ACT_SIGMOID
    m2, f3 = host_cases.cwq_conv_module(c)
    with pytest.raises(H.HostError):
        m2.compile(f3)


def test_shape_mismatch_is_reported_with_the_instruction_name():
    c = cases.rwq_fc_case(1, 8, 64, 48)
    c["bias"] = c["bias"][:-1]
    m, f = host_cases.rwq_fc_module(c)
    with pytest.raises(H.HostError) as e:
        m.compile(f)
    assert "rwqfc" in str(e.value) and "shape mismatch" in str(e.value)


def test_device_manager_without_a_device():
    from glow_amd import capi
    if capi.num_devices() > 0:
        pytest.skip("a GPU is present")
    dm = H.DeviceManager()
    with pytest.raises(H.HostError) as e:
        dm.init()
    assert e.value.code_name == "RUNTIME_DEVICE_NOT_FOUND"
    # requests to a manager that is not running are refused, not queued
    c = cases.rwq_fc_case(1, 8, 64, 48)
    m, f = host_cases.rwq_fc_module(c)
    m.compile(f)
    with pytest.raises(H.HostError) as e:
        dm.add_network(m)
    assert e.value.code_name == "RUNTIME_REQUEST_REFUSED"
    with pytest.raises(H.HostError) as e:
        dm.run("main", {})
    assert e.value.code_name == "RUNTIME_REQUEST_REFUSED"


def _resblock_tail(fuse):
    """conv output + residual -> ElementAdd -> Relu, the tail of a ResNet block."""
    m = H.Module()
    a = m.placeholder("a", (2, 4, 4, 16), H.INT8Q, np.int8, 0.05, 3)
    b = m.placeholder("b", (2, 4, 4, 16), H.INT8Q, np.int8, 0.07, -4)
    out = m.placeholder("out", (2, 4, 4, 16), H.INT8Q, np.int8, 0.2, -128)
    f = m.function("main")
    s = m.activation(f, "sum", (2, 4, 4, 16), H.INT8Q, 0.11, 5)
    m.instruction(f, H.ELEMENT_ADD, "add", [s, a, b])
    m.instruction(f, H.RELU, "relu", [out, s])
    m.compile(f, fuse_add_relu=fuse)
    return H.parse_listing(m.describe(f))


def test_add_relu_parameters_and_fusion():
    lp = go.quantize_scale_offset_32to8(float(np.float32(0.05) / np.float32(0.11)), 0)[:3]
    rp = go.quantize_scale_offset_32to8(float(np.float32(0.07) / np.float32(0.11)), 0)[:3]
    dp = go.quantize_scale_offset_32to8(float(np.float32(0.11) / np.float32(0.2)), 0)[:3]
    sep = _resblock_tail(False)
    assert [r["kernel"] for r in sep] == ["mi355x_add_i8", "mi355x_relu_i8"]
    assert (sep[0]["lhs_pre"], sep[0]["lhs_post"], sep[0]["lhs_scale"]) == lp
    assert (sep[0]["rhs_pre"], sep[0]["rhs_post"], sep[0]["rhs_scale"]) == rp
    assert (sep[0]["dest_offset"], sep[0]["lhs_offset"], sep[0]["rhs_offset"]) == (5, 3, -4)
    assert (sep[1]["pre"], sep[1]["post"], sep[1]["scale"]) == dp
    assert (sep[1]["src_offset"], sep[1]["dest_offset"]) == (5, -128)
    fused = _resblock_tail(True)
    assert [r["kernel"] for r in fused] == ["mi355x_add_relu_i8"]
    assert (fused[0]["relu_pre"], fused[0]["relu_post"], fused[0]["relu_scale"]) == dp
    assert fused[0]["relu_dest_offset"] == -128 and fused[0]["dest_offset"] == 5


def test_pool_parameters_and_checks():
    m = H.Module()
    x = m.placeholder("x", (2, 9, 9, 16), H.INT8Q, np.int8, 0.06, -9)
    mp = m.placeholder("mp", (2, 5, 5, 16), H.INT8Q, np.int8, 0.06, -9)
    ap = m.placeholder("ap", (2, 5, 5, 16), H.INT8Q, np.int8, 0.05, 4)
    f = m.function("main")
    attrs = [3, 3, 2, 2, 1, 1, 1, 1]
    m.instruction(f, H.MAX_POOL, "maxpool", [mp, x], attrs)
    m.instruction(f, H.AVG_POOL, "avgpool", [ap, x], attrs + [1])
    m.compile(f)
    rows = H.parse_listing(m.describe(f))
    assert rows[0]["kernel"] == "mi355x_max_pool_i8" and rows[0]["out_offset"] == -9
    sc = np.float32(0.06) / np.float32(0.05) / np.float32(9)
    assert (rows[1]["pre"], rows[1]["post"], rows[1]["scale"]) == \
        go.quantize_scale_offset_32to8(float(sc), 0)[:3]
    assert (rows[1]["in_offset"], rows[1]["out_offset"], rows[1]["count_include_pads"]) == (-9, 4, 1)
    # max pool passes values through: differing parameters are rejected
    bad = m.placeholder("bad", (2, 5, 5, 16), H.INT8Q, np.int8, 0.07, -9)
    assert not m.is_op_supported(H.MAX_POOL, [bad, x], attrs)[0]
    wrong = m.placeholder("wrong", (2, 4, 4, 16), H.INT8Q, np.int8, 0.06, -9)
    ok, why = m.is_op_supported(H.MAX_POOL, [wrong, x], attrs)
    assert not ok and "computed 5 x 5" in why


def _slice_module(between=None, second_reader=False, y_is_placeholder=False):
    """x --Rescale--> y --InsertTensor(cols 5..20)--> wide, optionally with
    another instruction between the two."""
    m = H.Module()
    x = m.placeholder("x", (8, 16), H.INT8Q, np.int8, 0.30, 2)
    x2 = m.placeholder("x2", (8, 5), H.INT8Q, np.int8, 0.11, -3)
    wide = m.placeholder("wide", (8, 40), H.INT8Q, np.int8, 0.11, -3)
    spare = m.placeholder("spare", (8, 40), H.INT8Q, np.int8, 0.2, 0)
    spare16 = m.placeholder("spare16", (8, 16), H.INT8Q, np.int8, 0.2, 0)
    f = m.function("main")
    y = (m.placeholder("y", (8, 16), H.INT8Q, np.int8, 0.11, -3) if y_is_placeholder
         else m.activation(f, "y", (8, 16), H.INT8Q, 0.11, -3))
    m.instruction(f, H.RESCALE_QUANTIZED, "r", [y, x])
    if between == "reads_wide":
        m.instruction(f, H.RESCALE_QUANTIZED, "peek", [spare, wide])
    elif between == "other_columns":
        m.instruction(f, H.INSERT_TENSOR, "left", [wide, x2], [0])
    elif between == "same_columns":
        m.instruction(f, H.INSERT_TENSOR, "clash", [wide, x2], [18])
    m.instruction(f, H.INSERT_TENSOR, "ins", [wide, y], [5])
    if second_reader:
        m.instruction(f, H.RESCALE_QUANTIZED, "again", [spare16, y])
    return m, f


def test_insert_is_folded_into_the_producer_only_when_nothing_can_tell():
    def kernels(**kw):
        m, f = _slice_module(**kw)
        m.compile(f)
        return [(r["kernel"], r["inst"]) for r in H.parse_listing(m.describe(f)) if r["phase"] == "launch"]
    assert kernels() == [("mi355x_rescale_rows_i8", "r+ins")]
    m, f = _slice_module()
    m.compile(f)
    r = _launch(m, f, "mi355x_rescale_rows_i8")
    assert (r["rows"], r["cols"], r["stride"], r["offset"]) == (8, 16, 40, 5)
    pre, post, scale, _ = go.quantize_scale_offset_32to8(float(np.float32(0.30) / np.float32(0.11)), 0)
    assert (r["pre"], r["post"], r["scale"], r["in_offset"], r["out_offset"]) == (pre, post, scale, 2, -3)
    # an insert of other columns in between does not stand in the way
    assert kernels(between="other_columns") == [("mi355x_rescale_rows_i8", "r+ins"),
                                                 ("mi355x_insert_rows", "left")]
    # a reader of the wide tensor, an insert overlapping the slice, a second
    # reader of the result, or a result the caller can see: two launches
    for kw in (dict(between="reads_wide"), dict(between="same_columns"), dict(second_reader=True),
               dict(y_is_placeholder=True)):
        k = [n for n, _ in kernels(**kw)]
        assert "mi355x_rescale_rows_i8" not in k and k.count("mi355x_rescale_i8") >= 1, kw
    m, f = _slice_module()
    m.compile(f, fuse_insert=False)
    assert [r["kernel"] for r in H.parse_listing(m.describe(f)) if r["phase"] == "launch"] == \
        ["mi355x_rescale_i8", "mi355x_insert_rows"]


def test_dequantize_and_sigmoid_become_one_launch():
    def build(extra_reader):
        m = H.Module()
        q = m.placeholder("q", (6, 3), H.INT8Q, np.int8, 0.04, 7)
        p = m.placeholder("p", (6, 3), H.FLOAT, np.float32)
        p2 = m.placeholder("p2", (6, 3), H.FLOAT, np.float32)
        f = m.function("main")
        x = m.activation(f, "x", (6, 3), H.FLOAT)
        m.instruction(f, H.DEQUANTIZE, "deq", [x, q])
        m.instruction(f, H.SIGMOID, "sig", [p, x])
        if extra_reader:
            m.instruction(f, H.SIGMOID, "sig2", [p2, x])
        return m, f
    m, f = build(False)
    m.compile(f)
    r = _launch(m, f, "mi355x_dequantize_sigmoid")
    assert (r["inst"], r["n"], r["offset"]) == ("deq+sig", 18, 7) and abs(r["scale"] - 0.04) < 1e-7
    m, f = build(True)
    m.compile(f)
    assert [r["kernel"] for r in H.parse_listing(m.describe(f))] == \
        ["mi355x_dequantize_i8", "mi355x_sigmoid_f32", "mi355x_sigmoid_f32"]
    m, f = build(False)
    m.compile(f, fuse_dequantize_sigmoid=False)
    assert [r["kernel"] for r in H.parse_listing(m.describe(f))] == \
        ["mi355x_dequantize_i8", "mi355x_sigmoid_f32"]


def _interaction_module(idx, peek=False):
    """x [B,4,16] -> Transpose -> BatchMatMul -> (flat view) Gather(idx) ->
    InsertTensor into the output at column 3."""
    m = H.Module()
    B = 6
    x = m.placeholder("x", (B, 4, 16), H.INT8Q, np.int8, 0.1, 2)
    wide = m.placeholder("wide", (B, 3 + len(idx)), H.INT8Q, np.int8, 0.3, -5)
    spare = m.placeholder("spare", (B, 16), H.INT8Q, np.int8, 0.3, -5)
    ix = m.constant("idx", np.asarray(idx, np.int64), H.INT64I)
    f = m.function("main")
    xt = m.activation(f, "xT", (B, 16, 4), H.INT8Q, 0.1, 2)
    z = m.activation(f, "z", (B, 4, 4), H.INT8Q, 0.3, -5)
    zf = m.view("z_flat", z, (B, 16), H.INT8Q, 0.3, -5)
    pairs = m.activation(f, "pairs", (B, len(idx)), H.INT8Q, 0.3, -5)
    m.instruction(f, H.TRANSPOSE, "t", [xt, x], [0, 2, 1])
    m.instruction(f, H.BATCH_MATMUL, "mm", [z, x, xt])
    if peek:
        m.instruction(f, H.RESCALE_QUANTIZED, "peek", [spare, zf])
    m.instruction(f, H.GATHER, "pick", [pairs, zf, ix], [1])
    m.instruction(f, H.INSERT_TENSOR, "ins", [wide, pairs], [3])
    m.compile(f)
    return [(r["kernel"], r["inst"]) for r in H.parse_listing(m.describe(f)) if r["phase"] == "launch"], m, f


def test_gather_of_product_elements_is_folded_into_the_product():
    k, m, f = _interaction_module([1, 2, 3, 6, 7, 11])
    assert k == [("mi355x_batch_matmul_nt_select_i8", "mm+pick+ins")]
    r = _launch(m, f, "mi355x_batch_matmul_nt_select_i8")
    assert (r["picked"], r["stride"], r["offset"], r["M"], r["N"], r["K"]) == (6, 9, 3, 4, 4, 16)
    # an index picked twice, an index outside the matrix, or a second reader of
    # the product: the product is written whole and gathered afterwards
    for idx, peek in (([1, 2, 2], False), ([1, 16], False), ([1, 2, 3], True)):
        k, _, _ = _interaction_module(idx, peek)
        names = [n for n, _ in k]
        assert "mi355x_batch_matmul_nt_select_i8" not in names and "mi355x_batch_matmul_nt_i8" in names
        assert "mi355x_gather_rows" in names


def test_per_row_and_per_channel_shifts_are_checked_at_compile_time():
    """A row scale so small that its rescale needs a shift beyond 31 bits is a
    compile error (the scalar parameters of every entry point are held to
    [0, 31]; the per-row vectors live in device memory, so the backend checks
    them where it makes them)."""
    c = cases.rwq_fc_case(1, 8, 64, 48)
    c["w_scales"] = c["w_scales"].copy()
    c["w_scales"][17] = 1e-22
    m, f = host_cases.rwq_fc_module(c)
    with pytest.raises(H.HostError) as e:
        m.compile(f)
    assert "row 17" in str(e.value) and "[0, 31]" in str(e.value)
    cc = cases.cwq_conv_case(2, 1, 6, 6, 16, 8)
    cc["f_scales"] = cc["f_scales"].copy()
    cc["b_scales"] = cc["b_scales"].copy()
    cc["f_scales"][5] = 1e-22
    cc["b_scales"][5] = 1e-22 * 0.05
    m, f = host_cases.cwq_conv_module(cc)
    with pytest.raises(H.HostError) as e:
        m.compile(f)
    assert "channel 5" in str(e.value)


def test_copy_instruction():
    """CopyInst (what Save and Reshape lower to): one device copy of the bytes;
    element kinds, sizes and quantization parameters must agree."""
    m = H.Module("copy")
    a = m.placeholder("a", (4, 48), H.INT8Q, np.int8, 0.1, 3)
    b = m.placeholder("b", (192,), H.INT8Q, np.int8, 0.1, 3)
    c = m.placeholder("c", (192,), H.INT8Q, np.int8, 0.2, 3)
    f = m.function("main")
    m.instruction(f, H.COPY, "save", [b, a])
    m.compile(f)
    r = _launch(m, f, "mi355x_copy_u8")
    assert r["bytes"] == 192 and r["inst"] == "save"
    g = m.function("bad")
    m.instruction(g, H.COPY, "rescaling_copy", [c, a])
    with pytest.raises(H.HostError):
        m.compile(g)


def test_lookups_with_input_lengths_read_host_made_bag_positions():
    """Lengths that are an input placeholder: the launch goes through
    mi355x_frwq_slws_offsets with positions the device manager sums on the host;
    lengths an instruction writes on the device, or the option off: through the
    lengths entry point."""
    m, ops = _slws_module(H.UINT8_FUSED, H.FLOAT, H.FLOAT)
    f = m.function("main")
    m.instruction(f, H.FRWQ_SLWS, "slws", ops, [0])
    m.compile(f)
    rows = [r for r in H.parse_listing(m.describe(f)) if r["phase"] == "launch"]
    assert [r["kernel"] for r in rows] == ["mi355x_frwq_slws_offsets"]
    assert rows[0]["bag_offsets"] == "host(len)" and rows[0]["segments"] == 3
    m.compile(f, derive_bag_offsets=False)
    rows = [r for r in H.parse_listing(m.describe(f)) if r["phase"] == "launch"]
    assert [r["kernel"] for r in rows] == ["mi355x_frwq_slws"]
    # lengths copied on the device from another placeholder
    m, ops = _slws_module(H.UINT8_FUSED, H.FLOAT, H.FLOAT)
    src = m.placeholder("len_src", (3,), H.INT32I, np.int32)
    f = m.function("main")
    m.instruction(f, H.COPY, "copy_len", [ops[4], src])
    m.instruction(f, H.FRWQ_SLWS, "slws", ops, [0])
    m.compile(f)
    rows = [r for r in H.parse_listing(m.describe(f)) if r["phase"] == "launch"]
    assert [r["kernel"] for r in rows] == ["mi355x_copy_u8", "mi355x_frwq_slws"]


def test_wide_kinds_transposes_and_3d_convolutions_compile():
    """int16 / int32 Quantize, RescaleQuantized, Dequantize; shuffles other than
    the two tiled ones; the NTHWC form of ChannelwiseQuantizedConvolution."""
    m = H.Module("wide")
    x = m.placeholder("x", (4, 6), H.FLOAT, np.float32)
    y = m.placeholder("y", (4, 6), H.FLOAT, np.float32)
    f = m.function("main")
    for kind, tag in ((H.INT16Q, "i16"), (H.INT32Q, "i32")):
        q = m.activation(f, f"q_{tag}", (4, 6), kind, 0.01, 3)
        r = m.activation(f, f"r_{tag}", (4, 6), kind, 0.02, -5)
        m.instruction(f, H.QUANTIZE, f"quant_{tag}", [q, x])
        m.instruction(f, H.RESCALE_QUANTIZED, f"rescale_{tag}", [r, q])
        m.instruction(f, H.DEQUANTIZE, f"dequant_{tag}", [y, r])
    t_in = m.placeholder("t_in", (2, 3, 4, 5), H.INT8Q, np.int8, 0.1, 1)
    t_out = m.placeholder("t_out", (2, 4, 5, 3), H.INT8Q, np.int8, 0.1, 1)
    m.instruction(f, H.TRANSPOSE, "nchw2nhwc", [t_out, t_in], [0, 2, 3, 1])
    f_in = m.placeholder("f_in", (3, 5), H.FLOAT, np.float32)
    f_out = m.placeholder("f_out", (5, 3), H.FLOAT, np.float32)
    m.instruction(f, H.TRANSPOSE, "float_t", [f_out, f_in], [1, 0])
    m.compile(f)
    k = [r["kernel"] for r in H.parse_listing(m.describe(f)) if r["phase"] == "launch"]
    assert k == ["mi355x_quantize_i16", "mi355x_rescale_i16", "mi355x_dequantize_i16",
                 "mi355x_quantize_i32", "mi355x_rescale_i32", "mi355x_dequantize_i32",
                 "mi355x_transpose_nd", "mi355x_transpose_nd"]
    # mismatched kinds and a shuffle that is no permutation are refused
    q16 = m.activation(f, "q16b", (4, 6), H.INT16Q, 0.01, 0)
    q32 = m.activation(f, "q32b", (4, 6), H.INT32Q, 0.01, 0)
    assert not m.is_op_supported(H.RESCALE_QUANTIZED, [q32, q16])[0]
    assert not m.is_op_supported(H.TRANSPOSE, [t_out, t_in], [0, 2, 2, 1])[0]
    assert not m.is_op_supported(H.TRANSPOSE, [t_out, t_in], [0, 3, 2, 1])[0]   # shape mismatch

    c = cases.cwq_conv3d_case(5, N=1, T=4, H=5, W=5, IC=4, OC=6, kernel=(2, 3, 3),
                              stride=(1, 2, 1), pads=(1, 0, 1, 1, 0, 2))
    mc, fc = host_cases.cwq_conv3d_module(c, (2, 3, 3), (1, 2, 1), (1, 0, 1, 1, 0, 2))
    mc.compile(fc)
    rows = [r for r in H.parse_listing(mc.describe(fc)) if r["phase"] == "launch"]
    assert [r["kernel"] for r in rows] == ["mi355x_cwq_conv3d_i8"]
    g = c["geom"]
    assert (rows[0]["OT"], rows[0]["OH"], rows[0]["OW"]) == (g.OT, g.OH, g.OW)
    # an output shape that the attributes do not give is refused
    bad, fb = host_cases.cwq_conv3d_module(c, (2, 3, 3), (1, 1, 1), (1, 0, 1, 1, 0, 2))
    with pytest.raises(H.HostError):
        bad.compile(fb)


def test_bag_positions_are_not_derived_from_lengths_some_function_writes():
    """Bag positions summed on the host need lengths only the host writes: a
    write through a view, or by another function of the module, switches the
    lookup back to reading the lengths on the device."""
    rng = np.random.default_rng(5)
    table = rng.integers(0, 256, (50, 72)).astype(np.uint8)

    def build(view_write, other_function):
        m = H.Module("w")
        data = m.constant("data", table, H.UINT8_FUSED)
        iv = m.placeholder("indices", (400,), H.INT64I, np.int64)
        lv = m.placeholder("lengths", (32,), H.INT32I, np.int32)
        src = m.placeholder("src", (32,), H.INT32I, np.int32)
        out = m.placeholder("out", (32, 64), H.FLOAT, np.float32)
        f = m.function("main")
        if other_function:
            g = m.function("writer")
            m.instruction(g, H.COPY, "store", [lv, src])
        if view_write:
            half = m.view("first_half", lv, (16,), H.INT32I)
            src_half = m.view("src_half", src, (16,), H.INT32I)
            m.instruction(f, H.COPY, "store_half", [half, src_half])
        m.instruction(f, H.FRWQ_SLS, "sls", [out, data, iv, lv], [0])
        m.compile(f)
        return m.describe(f)

    assert "mi355x_frwq_slws_offsets" in build(False, False)
    assert "mi355x_frwq_slws_offsets" not in build(True, False)
    assert "mi355x_frwq_slws_offsets" not in build(False, True)


def test_long_k_products_with_few_tiles_get_a_workspace():
    """A matrix-core launch whose 128x128 grid would leave half the chip idle and
    whose K loop is long gets a workspace in the generated region (zero-filled
    by a set-up launch), so that the kernel library may split K over workgroups;
    other launches get none, and the option switches it off."""
    c = cases.rwq_fc_case(21, 300, 4608, 256, symmetric=True)
    m, f = host_cases.rwq_fc_module(c)
    m.compile(f)
    r = _launch(m, f, "mi355x_rwq_fc_i8")
    want = capi.gemm_splitk_workspace_bytes(300, 256, 4608)
    assert want > 0 and r["splitk_workspace"] == want
    fills = [x for x in H.parse_listing(m.describe(f))
             if x["phase"] == "setup" and x["kernel"] == "mi355x_fill_u8"]
    assert len(fills) == 1 and fills[0]["bytes"] == want
    assert m.bundle_sizes(f)["generated"] >= want
    m2, f2 = host_cases.rwq_fc_module(c)
    m2.compile(f2, split_k=False)
    assert "splitk_workspace" not in _launch(m2, f2, "mi355x_rwq_fc_i8")
    small = cases.rwq_fc_case(22, 300, 512, 256, symmetric=True)     # K too short to share
    m3, f3 = host_cases.rwq_fc_module(small)
    m3.compile(f3)
    assert "splitk_workspace" not in _launch(m3, f3, "mi355x_rwq_fc_i8")

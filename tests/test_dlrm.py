"""The DLRM-style harness: builds and compiles on the CPU; on the GPU the whole
network through MI355XDeviceManager matches the oracle executing the same
quantized graph: bit-exact int8 logits (the fp16 pooled embeddings feeding them
included), sigmoid within 1e-5."""
import numpy as np
import pytest

from glow_amd import host as H
from glow_amd.harness import dlrm
from glow_amd.harness import net as netlib
from tests import oracle_exec

SMALL = dict(tables=3, rows=2000, dim=16, batch=64, mean_len=5, bottom=(32, 16), top=(32, 1))


def test_builds_and_compiles():
    net, max_idx = dlrm.make(seed=2, **SMALL)
    m, f = netlib.to_module(net)
    m.compile(f)
    rows = [r for r in H.parse_listing(m.describe(f)) if r["phase"] == "launch"]
    k = [r["kernel"] for r in rows]
    # the three lookups with their ConvertTo / Quantize / InsertTensor are one launch
    assert k.count("mi355x_frwq_sls_multi") == 1 and "mi355x_frwq_slws" not in k
    multi = rows[k.index("mi355x_frwq_sls_multi")]
    assert (multi["tables"], multi["out_kind"], multi["stride"]) == (3, 3, 4 * 16)
    # the lengths are inputs: every table's bags come as positions summed on the host
    assert multi["bag_offsets_from_host"] == 3
    assert k.count("mi355x_convert_f16_to_f32") == 0
    # no InsertTensor is left: the bottom MLP's rescaled output and the upper
    # triangle of the interaction are written where they are inserted
    assert k.count("mi355x_insert_rows") == 0 and k.count("mi355x_rescale_rows_i8") == 2
    # ... the interaction writes the picked pairs itself
    assert k.count("mi355x_gather_rows") == 0 and k.count("mi355x_gather") == 0
    sel = rows[k.index("mi355x_batch_matmul_nt_select_i8")]
    assert (sel["inst"], sel["picked"], sel["stride"], sel["offset"]) == \
        ("interact+upper_triangle+insert_pairs", 6, 22, 16)
    assert k[-1] == "mi355x_dequantize_sigmoid"
    # the interaction's Transpose + BatchMatMul read the features as they lie
    assert k.count("mi355x_batch_matmul_nt_select_i8") == 1 and k.count("mi355x_batch_transpose_i8") == 0
    assert k.count("mi355x_batch_matmul_i8") == 0
    # every hidden layer's Relu runs inside its FullyConnected
    assert k.count("mi355x_relu_i8") == 0 and k.count("mi355x_rwq_fc_relu_i8") >= 2
    m, f = netlib.to_module(net)
    m.compile(f, fuse_sls_chains=False, fuse_transpose_matmul=False, fuse_fc_relu=False,
              fuse_insert=False, fuse_dequantize_sigmoid=False)
    k = [r["kernel"] for r in H.parse_listing(m.describe(f)) if r["phase"] == "launch"]
    assert k.count("mi355x_frwq_slws_offsets") == 3 and k.count("mi355x_rwq_fc_i8") == 4
    assert k.count("mi355x_convert_f16_to_f32") == 3 and k.count("mi355x_insert_rows") == 6
    assert k.count("mi355x_batch_matmul_i8") == 1 and k.count("mi355x_gather") == 1
    assert k[-1] == "mi355x_sigmoid_f32"
    # 4 vectors of 16 -> 6 pairs + 16 dense outputs feed the top MLP
    assert net.tensors["top_in"].shape == (64, 22)


def test_small_table_rows_are_relaid_64_bytes_apart():
    """64 four-bit columns with fp16 scale/offset make 36-byte rows: each
    constant table gets one set-up copy to a 64-byte pitch and the lookups are
    told that pitch; switched off, they read the packed rows."""
    cfg = dict(tables=3, rows=300, dim=64, batch=32, mean_len=4, bottom=(32, 64), top=(32, 1))
    net, _ = dlrm.make(seed=4, **cfg)
    for fuse in (True, False):
        m, f = netlib.to_module(net)
        m.compile(f, fuse_sls_chains=fuse)
        rows = H.parse_listing(m.describe(f))
        pads = [r for r in rows if r["phase"] == "setup" and r["inst"].endswith(".pad_rows")]
        assert len(pads) == 3 and all((r["kernel"], r["row_bytes"], r["pitch"]) ==
                                      ("mi355x_insert_rows", 36, 64) for r in pads)
        look = [r for r in rows if r["phase"] == "launch" and "_sl" in r["kernel"]]
        assert len(look) == (1 if fuse else 3) and all(r["in_line"] == 64 for r in look)
        m, f = netlib.to_module(net)
        m.compile(f, fuse_sls_chains=fuse, pad_table_rows=False)
        rows = H.parse_listing(m.describe(f))
        assert not [r for r in rows if r["inst"].endswith(".pad_rows")]
        assert all(r["in_line"] == 36 for r in rows
                   if r["phase"] == "launch" and "_sl" in r["kernel"])


def test_oracle_executes_the_small_network():
    net, max_idx = dlrm.make(seed=2, **SMALL)
    inp = dlrm.Inputs(7, 3, 2000, 64, 5, 1.1, 13)
    v = oracle_exec.run(net, dlrm.bindings(net, inp, max_idx))
    p = v["prob"]
    assert p.shape == (64, 1) and np.all((p >= 0) & (p <= 1))
    assert len(np.unique(v["logit_q"])) > 1 and len(np.unique(v["pairs"])) > 1


@pytest.mark.gpu
@pytest.mark.parametrize("pad", [True, False])
@pytest.mark.parametrize("fuse", [True, False])
def test_device_matches_oracle(fuse, pad):
    cfg = dict(tables=4, rows=5000, dim=64, batch=256, mean_len=8, bottom=(64, 64), top=(128, 1))
    net, max_idx = dlrm.make(seed=3, **cfg)
    m, f = netlib.to_module(net)
    m.compile(f, fuse_sls_chains=fuse, fuse_transpose_matmul=fuse, fuse_fc_relu=fuse,
              pad_table_rows=pad, fuse_insert=fuse, fuse_dequantize_sigmoid=fuse)
    dm = H.DeviceManager().init()
    try:
        dm.add_network(m)
        for seed in (11, 12):
            inp = dlrm.Inputs(seed, 4, 5000, 256, 8, 1.1, 13)
            b = dlrm.bindings(net, inp, max_idx)
            logit = np.zeros((256, 1), np.int8)
            prob = np.zeros((256, 1), np.float32)
            dm.run("main", dict(b, logit_q=logit, prob=prob))
            want = oracle_exec.run(net, b)
            np.testing.assert_array_equal(logit, want["logit_q"])
            np.testing.assert_allclose(prob, want["prob"], rtol=1e-5, atol=1e-30)
    finally:
        dm.stop()


@pytest.mark.gpu
@pytest.mark.fused_math
def test_device_with_fused_lookup_arithmetic_stays_within_one_step():
    """The library's default lookup arithmetic (fused multiply-adds) moves a
    pooled embedding by rounding only, so behind the Quantize that follows at
    most a rare value lands on the other side of a rounding boundary: the
    network's int8 logit may differ from the sequential CPU arithmetic by one
    quantization step in a few samples, and nowhere by more."""
    cfg = dict(tables=4, rows=5000, dim=64, batch=256, mean_len=8, bottom=(64, 64), top=(128, 1))
    net, max_idx = dlrm.make(seed=3, **cfg)
    m, f = netlib.to_module(net)
    m.compile(f)
    dm = H.DeviceManager().init()
    try:
        dm.add_network(m)
        inp = dlrm.Inputs(11, 4, 5000, 256, 8, 1.1, 13)
        b = dlrm.bindings(net, inp, max_idx)
        logit = np.zeros((256, 1), np.int8)
        prob = np.zeros((256, 1), np.float32)
        dm.run("main", dict(b, logit_q=logit, prob=prob))
        want = oracle_exec.run(net, b)
        d = np.abs(logit.astype(np.int32) - want["logit_q"].astype(np.int32))
        print("logits off by one step:", int((d == 1).sum()), "of", d.size, flush=True)
        assert d.max() <= 1 and (d > 0).sum() <= 1
    finally:
        dm.stop()

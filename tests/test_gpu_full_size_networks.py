"""The two network configurations at their full sizes, through
MI355XDeviceManager, against the oracle executing the same quantized graph
instruction by instruction.

Int8 ResNet-50: batch 64 of 224x224x3 images, all 16 bottleneck blocks, 1000
classes. The batch holds two distinct images, each repeated 32 times; the
oracle runs the two (8 GMAC on one CPU thread) and every slot of the batch
must equal the oracle's logits for its image, bit for bit. This reaches the
real layer shapes and the per-layer tiles the device manager tunes at
addNetwork.

DLRM-style net: 26 four-bit tables of 1M rows x 64, batch 4096, Poisson(20)
bags of Zipf(1.1) int64 indices, MLPs 13-512-256-64 and 415-512-256-1: the
whole batch against the oracle (2 GMAC and 2.1M lookups).

Run on the GPU box:  python -u -m pytest tests -m gpu -x -v --timeout 120
"""
import numpy as np
import pytest

from glow_amd import host as H
from glow_amd.harness import dlrm
from glow_amd.harness import net as netlib
from glow_amd.harness import resnet50
from tests import oracle_exec

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def test_resnet50_batch_64_at_224():
    batch, size = 64, 224
    steps = resnet50.build_fp32(0)
    # the configuration's own profile: 100 synthetic images
    ranges = resnet50.profile(steps, resnet50.synthetic_images(1, 100, size))
    net = resnet50.build_int8(steps, ranges, batch, size)
    two = resnet50.build_int8(steps, ranges, 2, size)     # same constants and scales
    x2 = resnet50.synthetic_images(21, 2, size)
    x2[1] = 0.9 - x2[1]                                   # make the second image differ more
    say("resnet50 full size: oracle on two images")
    want = oracle_exec.run(two, {"input": x2})
    want_logits = np.array(want["logits_q"])
    want_prob = np.array(want["prob"])
    assert len(np.unique(want_logits)) > 20

    m, f = netlib.to_module(net)
    m.compile(f)
    launches = [r for r in H.parse_listing(m.describe(f)) if r["phase"] == "launch"]
    assert sum(1 for r in launches if "conv2d" in r["kernel"]) == 53
    x = np.ascontiguousarray(np.tile(x2, (batch // 2, 1, 1, 1)))
    logits = np.zeros((batch, 1000), np.int8)
    prob = np.zeros((batch, 1000), np.float32)
    say("resnet50 full size: addNetwork (tunes tiles per layer)")
    dm = H.DeviceManager().init()
    try:
        dm.add_network(m)
        # more requests than the device manager spends on choosing how to
        # record the function, so every recording it may settle on is checked
        for request in range(12):
            say("resnet50 full size: request", request)
            logits[:] = 0
            prob[:] = 0
            dm.run("main", {"input": x, "logits_q": logits, "prob": prob})
            for i in range(batch):
                assert np.array_equal(logits[i], want_logits[i % 2]), (request, i)
            np.testing.assert_allclose(prob, np.tile(want_prob, (batch // 2, 1)),
                                       rtol=1e-5, atol=1e-30)
    finally:
        dm.stop()


@pytest.fixture(scope="module")
def full_dlrm():
    say("dlrm full size: building 26 tables of 1M rows")
    net, max_idx = dlrm.make()
    inp = dlrm.Inputs(99, 26, 1_000_000, 4096, 20, 1.1, 13)
    b = dlrm.bindings(net, inp, max_idx)
    say("dlrm full size: oracle on the whole batch")
    want = oracle_exec.run(net, b)
    return net, b, np.array(want["logit_q"]), np.array(want["prob"])


def _run_dlrm(net, b, requests=12):
    m, f = netlib.to_module(net)
    m.compile(f)
    k = [r["kernel"] for r in H.parse_listing(m.describe(f)) if r["phase"] == "launch"]
    assert k.count("mi355x_frwq_sls_multi") == 1      # 26 tables x 4096 bags in one launch
    dm = H.DeviceManager().init()
    out = []
    try:
        dm.add_network(m)
        for request in range(requests):
            logit = np.zeros((4096, 1), np.int8)
            prob = np.zeros((4096, 1), np.float32)
            dm.run("main", dict(b, logit_q=logit, prob=prob))
            out.append((logit, prob))
    finally:
        dm.stop()
    return out


def test_dlrm_26_tables_of_1m_rows_batch_4096(full_dlrm):
    net, b, want_logit, want_prob = full_dlrm
    assert len(np.unique(want_logit)) > 20
    for request, (logit, prob) in enumerate(_run_dlrm(net, b)):
        say("dlrm full size: request", request)
        np.testing.assert_array_equal(logit, want_logit)
        np.testing.assert_allclose(prob, want_prob, rtol=1e-5, atol=1e-30)


@pytest.mark.fused_math
def test_dlrm_full_size_with_the_default_lookup_arithmetic(full_dlrm):
    """The library's default (fused multiply-add) lookup arithmetic moves a
    pooled value by rounding only; behind the Quantize that follows, a logit
    may land one quantization step away in a few samples, never further."""
    net, b, want_logit, _ = full_dlrm
    logit, _ = _run_dlrm(net, b, requests=2)[-1]
    d = np.abs(logit.astype(np.int32) - want_logit.astype(np.int32))
    say("dlrm full size, fused arithmetic: logits off by one step:", int((d == 1).sum()),
        "of", d.size)
    assert d.max() <= 1 and (d > 0).mean() <= 0.002

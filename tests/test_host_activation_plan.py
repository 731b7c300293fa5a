"""Where the compiler puts a function's activations
(AllocationsInfo::allocateActivations, AllocationsInfo.cpp:128-156: Glow gives
activations whose lives do not meet the same bytes; MemoryAllocator.cpp:58-91
is first fit by address).

The property that makes sharing safe is checked from the listing alone, with
the dependence graph rebuilt here: two values may overlap in memory only if
every launch touching one of them precedes every launch touching the other in
every order of execution the data flow allows (the device manager replays
launches as parallel branches of a graph, ordered by data flow only)."""
import itertools

import numpy as np
import pytest

from glow_amd import host as H
from glow_amd.harness import dlrm, resnet50, net as netlib
from tests import oracle_exec


def _accesses(row, which):
    return list(zip(row.get(which, []), row.get(which + "_lo", []), row.get(which + "_hi", [])))


def _overlap(a, b):
    if a[0] != b[0]:
        return False
    if a[2] < 0 or b[2] < 0:
        return True
    return a[1] < b[2] and b[1] < a[2]


def _conflict(early, late):
    ew, er = _accesses(early, "writes"), _accesses(early, "reads")
    lw, lr = _accesses(late, "writes"), _accesses(late, "reads")
    return (any(_overlap(w, x) for w in ew for x in lr + lw) or
            any(_overlap(r, w) for r in er for w in lw))


def _ancestors(launches):
    anc = []
    for i, li in enumerate(launches):
        s = set()
        for j in range(i):
            if _conflict(launches[j], li):
                s |= anc[j] | {j}
        anc.append(s)
    return anc


def _check_plan(text, expect_sharing):
    launches = [r for r in H.parse_listing(text) if r["phase"] == "launch"]
    acts = H.parse_activations(text)
    assert acts, "no activation was placed"
    anc = _ancestors(launches)
    touchers = {i: [] for i in acts}
    for k, l in enumerate(launches):
        for root, _, _ in _accesses(l, "reads") + _accesses(l, "writes"):
            if root in touchers and (not touchers[root] or touchers[root][-1] != k):
                touchers[root].append(k)
    size = int(text.split("activations=")[1].split()[0])
    shared = 0
    for a in acts.values():
        assert a["offset"] % 256 == 0 and a["offset"] + a["bytes"] <= size
    for p, q in itertools.combinations(acts, 2):
        a, b = acts[p], acts[q]
        if a["offset"] + a["bytes"] <= b["offset"] or b["offset"] + b["bytes"] <= a["offset"]:
            continue
        shared += 1
        p_first = all(tp in anc[tq] for tp in touchers[p] for tq in touchers[q])
        q_first = all(tq in anc[tp] for tp in touchers[p] for tq in touchers[q])
        assert p_first or q_first, (a, b)
    assert size == max(a["offset"] + a["bytes"] for a in acts.values())
    assert (shared > 0) == expect_sharing
    return size


def _small_resnet():
    return resnet50.make(batch=2, size=64, profile_images=4, seed=5,
                         layers=((64, 2, 1), (128, 2, 2), (256, 1, 2)), classes=100)


@pytest.mark.parametrize("fuse", [True, False])
def test_resnet_activations_share_memory_only_along_the_data_flow(fuse):
    net = _small_resnet()
    m, f = netlib.to_module(net)
    m.compile(f, fuse_conv_add=fuse, fuse_add_relu=fuse)
    with_sharing = _check_plan(m.describe(f), True)
    assert m.bundle_sizes(f)["activations"] == with_sharing
    m2, f2 = netlib.to_module(net)
    m2.compile(f2, fuse_conv_add=fuse, fuse_add_relu=fuse, reuse_activations=False)
    apart = _check_plan(m2.describe(f2), False)
    assert with_sharing < apart / 2


@pytest.mark.parametrize("fuse", [True, False])
def test_parallel_lookup_chains_keep_their_own_memory(fuse):
    """The chains of a ranking net's tables are independent of each other: none
    of them may wait for another because of a shared buffer."""
    cfg = dict(tables=4, rows=500, dim=64, batch=64, mean_len=4, bottom=(64, 64), top=(128, 1))
    net, _ = dlrm.make(seed=3, **cfg)
    m, f = netlib.to_module(net)
    m.compile(f, fuse_sls_chains=fuse, fuse_insert=fuse)
    text = m.describe(f)
    _check_plan(text, True)
    launches = [r for r in H.parse_listing(text) if r["phase"] == "launch"]
    # the dependence levels are those of the data flow alone
    m2, f2 = netlib.to_module(net)
    m2.compile(f2, fuse_sls_chains=fuse, fuse_insert=fuse, reuse_activations=False)
    apart = [r for r in H.parse_listing(m2.describe(f2)) if r["phase"] == "launch"]
    assert [l["level"] for l in launches] == [l["level"] for l in apart]


def test_results_inside_fused_launches_get_no_memory():
    net = _small_resnet()
    m, f = netlib.to_module(net)
    m.compile(f)
    text = m.describe(f)
    acts = H.parse_activations(text)
    fused = [r for r in H.parse_listing(text)
             if r["phase"] == "launch" and r["kernel"] == "mi355x_cwq_conv2d_add_i8"]
    assert fused
    for l in fused:
        # convolution result and sum are handed on inside the kernel
        inner = set(l["writes"]) & set(l["reads"])
        assert len(inner) == 2 and not inner & set(acts)
        assert set(l["writes"]) - inner <= set(acts)


@pytest.mark.gpu
@pytest.mark.parametrize("graphs", [False, True, -4])
def test_device_results_do_not_depend_on_the_plan(graphs):
    net = _small_resnet()
    x = resnet50.synthetic_images(11, 2, 64)
    want = oracle_exec.run(net, {"input": x})
    for reuse in (True, False):
        m, f = netlib.to_module(net)
        m.compile(f, reuse_activations=reuse)
        dm = H.DeviceManager(use_launch_graphs=graphs).init()
        try:
            dm.add_network(m)
            for _ in range(3):
                logits = np.zeros((2, 100), np.int8)
                prob = np.zeros((2, 100), np.float32)
                dm.run("main", {"input": x, "logits_q": logits, "prob": prob})
                np.testing.assert_array_equal(logits, want["logits_q"])
                np.testing.assert_allclose(prob, want["prob"], rtol=1e-5, atol=1e-30)
        finally:
            dm.stop()

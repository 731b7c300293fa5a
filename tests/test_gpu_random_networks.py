"""Seeded random variations of the two harness networks (stage widths, depths
and strides of the ResNet; table count, embedding width, batch and MLP sizes of
the ranking net) through MI355XBackend + MI355XDeviceManager with every rewrite
on, against the oracle executing the same lowered program instruction by
instruction: int8 results bit for bit, fp32 within 1e-5."""
import os

import numpy as np
import pytest

from glow_amd import host as H
from glow_amd.harness import dlrm, resnet50
from glow_amd.harness import net as netlib
from tests import oracle_exec

pytestmark = pytest.mark.gpu

_MORE = max(1, int(os.environ.get("MI355X_TEST_SEEDS", "1")))


@pytest.mark.parametrize("seed", range(6 * _MORE))
def test_random_resnet(seed):
    rng = np.random.default_rng(100 + seed)
    stages = int(rng.integers(1, 4))
    layers, planes = [], int(rng.choice([16, 32, 64]))
    for s in range(stages):
        layers.append((planes, int(rng.integers(1, 3)), 1 if s == 0 else int(rng.integers(1, 3))))
        planes *= 2
    batch, size = int(rng.integers(1, 4)), int(rng.choice([32, 48, 64]))
    classes = int(rng.choice([7, 10, 100]))
    print("resnet", layers, batch, size, classes, flush=True)
    net = resnet50.make(batch=batch, size=size, profile_images=3, seed=seed, layers=tuple(layers),
                        classes=classes)
    m, f = netlib.to_module(net)
    m.compile(f)
    dm = H.DeviceManager().init()
    try:
        dm.add_network(m)
        x = resnet50.synthetic_images(50 + seed, batch, size)
        logits = np.zeros((batch, classes), np.int8)
        prob = np.zeros((batch, classes), np.float32)
        dm.run("main", {"input": x, "logits_q": logits, "prob": prob})
        want = oracle_exec.run(net, {"input": x})
        np.testing.assert_array_equal(logits, want["logits_q"])
        np.testing.assert_allclose(prob, want["prob"], rtol=1e-5, atol=1e-30)
    finally:
        dm.stop()


@pytest.mark.parametrize("seed", range(6 * _MORE))
def test_random_ranking_net(seed):
    rng = np.random.default_rng(200 + seed)
    tables, dim = int(rng.integers(1, 7)), int(rng.choice([16, 32, 64, 128]))
    batch, rows = int(rng.choice([8, 64, 200, 512])), int(rng.integers(50, 4000))
    dense = int(rng.choice([3, 13, 16]))
    bottom = (int(rng.choice([16, 64, 96])), dim)
    top = (int(rng.choice([32, 128])), 1)
    mean_len = float(rng.choice([1, 6, 25]))
    print("ranking", tables, dim, batch, rows, dense, bottom, top, mean_len, flush=True)
    net, max_idx = dlrm.make(tables=tables, rows=rows, dim=dim, batch=batch, mean_len=mean_len,
                             dense_features=dense, bottom=bottom, top=top, seed=seed)
    m, f = netlib.to_module(net)
    m.compile(f)
    dm = H.DeviceManager().init()
    try:
        dm.add_network(m)
        inp = dlrm.Inputs(300 + seed, tables, rows, batch, mean_len, 1.1, dense)
        b = dlrm.bindings(net, inp, max_idx)
        logit = np.zeros((batch, 1), np.int8)
        prob = np.zeros((batch, 1), np.float32)
        dm.run("main", dict(b, logit_q=logit, prob=prob))
        want = oracle_exec.run(net, b)
        np.testing.assert_array_equal(logit, want["logit_q"])
        np.testing.assert_allclose(prob, want["prob"], rtol=1e-5, atol=1e-30)
    finally:
        dm.stop()


@pytest.mark.parametrize("graphs", [1, 2, -1, -3])
def test_every_recording_of_a_function_gives_the_same_results(graphs):
    """The first nine requests of a function go to its three recordings (all
    branches, one chain, two branches) in turn and later ones to the fastest:
    each request, with its own inputs, must match the oracle. Negative values
    fix the number of branches."""
    tables, dim, batch, rows, dense = 3, 32, 64, 500, 13
    net, max_idx = dlrm.make(tables=tables, rows=rows, dim=dim, batch=batch, mean_len=6.0,
                             dense_features=dense, bottom=(64, dim), top=(32, 1), seed=5)
    m, f = netlib.to_module(net)
    m.compile(f)
    dm = H.DeviceManager(use_launch_graphs=graphs).init()
    try:
        dm.add_network(m)
        for request in range(12):
            inp = dlrm.Inputs(400 + request, tables, rows, batch, 6.0, 1.1, dense)
            b = dlrm.bindings(net, inp, max_idx)
            logit = np.zeros((batch, 1), np.int8)
            prob = np.zeros((batch, 1), np.float32)
            dm.run("main", dict(b, logit_q=logit, prob=prob))
            want = oracle_exec.run(net, b)
            np.testing.assert_array_equal(logit, want["logit_q"], err_msg=f"request {request}")
            np.testing.assert_allclose(prob, want["prob"], rtol=1e-5, atol=1e-30)
    finally:
        dm.stop()

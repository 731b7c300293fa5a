"""Reads the committed golden vectors (tests/golden/*.npz, written by
tests/golden/make_golden.py from the reference's compiled libjit) back into
the argument tuples the oracle wrappers and the HIP wrappers share."""
import os

import numpy as np

from oracle import glow_oracle as go

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(name):
    with np.load(os.path.join(GOLDEN, name + ".npz")) as z:
        return {k: z[k] for k in z.files}


def _tags(d, suffix="_out"):
    return sorted({k[:-len(suffix)] for k in d if k.endswith(suffix)
                   and "matmul" not in k})


def elementwise():
    return _load("elementwise")


def rwq_fc_cases():
    d = _load("rwq_fc")
    for t in _tags(d):
        g = lambda k: d[f"{t}_{k}"]
        args = (g("x"), g("w"), g("bias"), g("w_offsets"), g("bias_pre"),
                g("bias_post"), g("bias_scale"), g("out_pre"), g("out_post"),
                g("out_scale"), int(g("out_offset")), int(g("in_offset")),
                int(g("bias_offset")))
        yield t, args, g("out")


def fc_cases():
    d = _load("fc")
    for t in _tags(d):
        g = lambda k: d[f"{t}_{k}"]
        args = (g("x"), g("w"), g("bias"), int(g("out_offset")),
                int(g("in_offset")), int(g("w_offset")), int(g("bias_offset")),
                tuple(int(v) for v in g("biasP")), tuple(int(v) for v in g("outP")))
        yield t, args, g("out"), g("matmul_out")


def cwq_conv_cases():
    d = _load("cwq_conv")
    for t in _tags(d):
        g = lambda k: d[f"{t}_{k}"]
        geom = go.ConvGeom(*[int(v) for v in g("geom")])
        args = (g("x"), g("filt"), g("bias"), geom, int(g("out_offset")),
                int(g("in_offset")), g("f_offsets"), g("b_offsets"),
                g("bias_pre"), g("bias_post"), g("bias_scale"), g("out_pre"),
                g("out_post"), g("out_scale"), int(g("act")),
                tuple(int(v) for v in g("act_args")))
        yield t, args, g("out")


def slws_cases():
    d = _load("frwq_slws")
    for t in _tags(d):
        g = lambda k: d[f"{t}_{k}"]
        yield t, (g("table"), g("weights"), g("indices"), g("lengths")), g("out")


def glue():
    """Golden int8 glue operators. Yields (name, callable(impl) -> got, want)
    where `impl` is a module with add_i8 / relu_i8 / max_pool_i8 / avg_pool_i8 /
    softmax_f32 in the oracle wrappers' signature."""
    d = _load("glue")
    a, b, x = d["a"], d["b"], d["x"]
    out = []
    for i in range(3):
        p = [int(v) for v in d[f"add{i}_params"]]
        out.append((f"add{i}", lambda m, p=p: m.add_i8(a, b, p[0], p[1], p[2], p[3:6], p[6:9]),
                    d[f"add{i}_out"]))
        p = [int(v) for v in d[f"relu{i}_params"]]
        out.append((f"relu{i}", lambda m, p=p: m.relu_i8(a, p[0], p[1], p[2:5]),
                    d[f"relu{i}_out"]))
    for i in range(4):
        g = [int(v) for v in d[f"pool{i}_geom"]]
        k, st, pd = g[0:2], g[2:4], g[4:8]
        out.append((f"maxpool{i}", lambda m, k=k, st=st, pd=pd: m.max_pool_i8(x, k, st, pd, -7),
                    d[f"maxpool{i}_out"]))
        for cip in (0, 1):
            p = [int(v) for v in d[f"avgpool{i}_{cip}_params"]]
            out.append((f"avgpool{i}_{cip}",
                        lambda m, k=k, st=st, pd=pd, p=p: m.avg_pool_i8(x, k, st, pd, p[0], p[1],
                                                                       p[2], p[3:6]),
                        d[f"avgpool{i}_{cip}_out"]))
    return out, d["logits"], d["softmax_out"]


def element_ops():
    """Golden Clip / LeakyRelu / Max(x, Splat) / BatchedAdd cases. Yields
    (name, function name in the oracle wrappers' naming, args, want)."""
    d = _load("element_ops")
    for entry in d["names"]:
        name, fn = str(entry).split(":")
        args = []
        k = 0
        while f"{name}_arg{k}" in d:
            v = d[f"{name}_arg{k}"]
            args.append(v if v.ndim and v.size > 3 else
                        (tuple(int(x) for x in v) if v.ndim else int(v)))
            k += 1
        yield name, fn, tuple(args), d[f"{name}_out"]


def wide():
    """The 16/32-bit elementwise vectors, transposes and 3-D convolutions."""
    return _load("wide")


def conv3d_cases():
    d = _load("wide")
    tags = sorted({k[len("conv3d_"):-len("_out")] for k in d
                   if k.startswith("conv3d_") and k.endswith("_out")})
    for t in tags:
        g = lambda k: d[f"conv3d_{t}_{k}"]
        geom = go.Conv3dGeom(*[int(v) for v in g("geom")])
        args = (g("x"), g("filt"), g("bias"), geom, int(g("out_offset")),
                int(g("in_offset")), g("f_offsets"), g("b_offsets"),
                g("bias_pre"), g("bias_post"), g("bias_scale"), g("out_pre"),
                g("out_post"), g("out_scale"), int(g("act")),
                tuple(int(v) for v in g("act_args")))
        yield t, args, g("out")

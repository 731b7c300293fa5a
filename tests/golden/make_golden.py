"""Writes the golden vectors under tests/golden/*.npz.

Run in the authoring container (where the reference tree is mounted and
oracle/Makefile has built oracle/_ref from the reference's unmodified libjit
sources):   python tests/golden/make_golden.py

Each file holds the seeded inputs, the derived integer parameters and the
outputs the REFERENCE's compiled kernels produced for them. The fixtures are
data only; they let the oracle and the HIP kernels be checked where the
reference is absent (the GPU box)."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import glow_oracle as go  # noqa: E402
from oracle import libjit_ref as ref  # noqa: E402
from tests import cases  # noqa: E402


def geom_vec(g):
    return np.array([getattr(g, n) for n, _ in g._fields_], np.int32)


def save(name, **kw):
    path = os.path.join(HERE, name + ".npz")
    np.savez_compressed(path, **kw)
    print(name, os.path.getsize(path), "bytes")


def glue():
    """int8 glue operators: add, relu, max pool, avg pool; fp32 softmax."""
    rng = np.random.default_rng(600)
    gl = {}
    a = rng.integers(-128, 128, (3, 7, 5, 6)).astype(np.int8)
    b = rng.integers(-128, 128, a.shape).astype(np.int8)
    gl["a"], gl["b"] = a, b
    for i, (ls, rs, ds, lo, ro, do) in enumerate([(0.05, 0.07, 0.11, 3, -4, 5),
                                                  (0.3, 0.002, 0.1, -128, 0, -128),
                                                  (1.0, 1.0, 1.0, 0, 0, 0)]):
        lp = go.quantize_scale_offset_32to8(float(np.float32(ls) / np.float32(ds)), lo)[:3]
        rp = go.quantize_scale_offset_32to8(float(np.float32(rs) / np.float32(ds)), ro)[:3]
        gl[f"add{i}_params"] = np.array([do, lo, ro, *lp, *rp], np.int32)
        gl[f"add{i}_out"] = ref.add_i8(a, b, do, lo, ro, lp, rp).reshape(a.shape)
    for i, (ss, ds, so, do) in enumerate([(0.1, 0.1, -20, -128), (0.05, 0.2, 7, 7),
                                          (0.4, 0.013, -128, -100)]):
        dp = go.quantize_scale_offset_32to8(float(np.float32(ss) / np.float32(ds)), 0)[:3]
        gl[f"relu{i}_params"] = np.array([so, do, *dp], np.int32)
        gl[f"relu{i}_out"] = ref.relu_i8(a, so, do, dp).reshape(a.shape)
    x = rng.integers(-128, 128, (2, 9, 11, 20)).astype(np.int8)
    gl["x"] = x
    pools = [((3, 3), (2, 2), (1, 1, 1, 1)), ((2, 3), (1, 2), (0, 1, 0, 1)),
             ((9, 11), (1, 1), (0, 0, 0, 0)), ((3, 3), (3, 3), (2, 2, 2, 2))]
    for i, (k, st, pd) in enumerate(pools):
        gl[f"pool{i}_geom"] = np.array([*k, *st, *pd], np.int32)
        gl[f"maxpool{i}_out"] = ref.max_pool_i8(x, k, st, pd, -7)
        for cip in (0, 1):
            sc = np.float32(0.06) / np.float32(0.05)
            if cip:
                sc = sc / np.float32(k[0] * k[1])
            op = go.quantize_scale_offset_32to8(float(sc), 0)[:3]
            gl[f"avgpool{i}_{cip}_params"] = np.array([cip, 4, -9, *op], np.int32)
            gl[f"avgpool{i}_{cip}_out"] = ref.avg_pool_i8(x, k, st, pd, cip, 4, -9, op)
    logits = rng.normal(0, 3, (5, 1000)).astype(np.float32)
    logits[1] *= 10
    gl["logits"] = logits
    gl["softmax_out"] = ref.softmax_f32(logits)
    save("glue", **gl)


def element_ops():
    """Clip, LeakyRelu, Max(x, Splat) and BatchedAdd on int8: inputs, integer
    parameters and what the compiled reference returns for them."""
    el = {}
    names = []
    for name, fn, args in cases.element_op_cases():
        names.append(f"{name}:{fn}")
        for k, v in enumerate(args):
            el[f"{name}_arg{k}"] = np.asarray(v)
        el[f"{name}_out"] = np.asarray(getattr(ref, fn)(*args)).reshape(np.asarray(args[0]).shape)
    el["names"] = np.array(names)
    save("element_ops", **el)


WIDE_CONV3D = [
    ("relu3", dict(N=2, T=4, H=5, W=6, IC=8, OC=8)),
    ("stride_group", dict(N=1, T=5, H=7, W=6, IC=8, OC=12, kernel=(2, 3, 1), stride=(2, 1, 2),
                          pads=(1, 0, 0, 2, 1, 1), group=2, act=go.ACT_NONE, symmetric=False,
                          in_offset=-9, out_offset=5)),
    ("clip_b8", dict(N=1, T=3, H=3, W=3, IC=3, OC=5, kernel=(3, 3, 3), act=go.ACT_CLIP,
                     bias_i8=True)),
    ("leaky", dict(N=1, T=2, H=4, W=4, IC=4, OC=4, kernel=(1, 2, 2), pads=(0, 0, 1, 0, 0, 1),
                   act=go.ACT_LEAKY_RELU, out_offset=10)),
]
WIDE_TRANSPOSES = [((5, 7), (1, 0)), ((3, 4, 5), (2, 0, 1)), ((2, 3, 4, 5), (0, 3, 1, 2)),
                   ((2, 3, 4, 5), (3, 2, 1, 0)), ((2, 3, 2, 3, 4), (4, 0, 3, 1, 2)),
                   ((2, 2, 3, 2, 3, 2), (5, 3, 1, 4, 2, 0))]


def wide():
    """The 16/32-bit elementwise forms, N-D transposes and the 3-D channelwise
    convolution, as the reference's compiled libjit computes them."""
    rng = np.random.default_rng(700)
    wd = {}
    x = np.concatenate([rng.normal(0, 300, 1500), rng.normal(0, 3e5, 500),
                        (np.arange(-100, 100) + 0.5) * 0.25]).astype(np.float32)
    wd["x"] = x
    for bits in (16, 32):
        dt = np.int16 if bits == 16 else np.int32
        lim = 2 ** (bits - 1)
        q = np.concatenate([rng.integers(-lim, lim, 1500), [-lim, lim - 1, 0, 1, -1]]).astype(dt)
        wd[f"q{bits}"] = q
        for i, (s, o) in enumerate([(0.25, 4), (0.05, -7), (17.3, 33)]):
            wd[f"quant{bits}_{i}_params"] = np.array([s, o], np.float64)
            wd[f"quant{bits}_{i}_out"] = ref.quantize_wide(x, s, o, bits)
            wd[f"dequant{bits}_{i}_out"] = ref.dequantize_wide(q, s, o)
        # rescale ratios whose 64-bit products stay well inside int64
        for i, (r, io, oo) in enumerate([(0.0123, -5, 7), (0.5, 0, -128), (1.7, 20, -3),
                                         (2.0, 1, 1)]):
            pre, post, sc, _ = go.quantize_scale_offset_32to8(r, 0)
            wd[f"rescale{bits}_{i}_params"] = np.array([oo, io, pre, post, sc], np.int32)
            wd[f"rescale{bits}_{i}_out"] = ref.rescale_wide(q, oo, io, pre, post, sc)
    for i, (shape, shuffle) in enumerate(WIDE_TRANSPOSES):
        t = rng.integers(-128, 128, shape).astype(np.int8)
        wd[f"transpose{i}_in"] = t
        wd[f"transpose{i}_shuffle"] = np.array(shuffle, np.int32)
        wd[f"transpose{i}_out"] = ref.transpose_i8(t, shuffle)
    for tag, kw in WIDE_CONV3D:
        c = cases.cwq_conv3d_case(800, **kw)
        for k, v in c.items():
            if k == "geom":
                wd[f"conv3d_{tag}_geom"] = geom_vec(v)
            elif k not in ("act_fargs", "f_scales", "b_scales", "in_scale_f", "out_scale_f"):
                wd[f"conv3d_{tag}_{k}"] = np.asarray(v, dtype=np.int32 if k == "act_args" else None)
        wd[f"conv3d_{tag}_out"] = ref.cwq_conv3d_i8(*cases.cwq_conv_args(c))
    save("wide", **wd)


def main():
    assert ref.available(), "build oracle/_ref first (make -C oracle)"
    if sys.argv[1:] == ["glue"]:
        glue()
        return
    if sys.argv[1:] == ["wide"]:
        wide()
        return

    # elementwise
    rng = np.random.default_rng(100)
    x = np.concatenate([rng.normal(0, 3, 2000),
                        (np.arange(-200, 200) + 0.5) * 0.25]).astype(np.float32)
    q = np.arange(-128, 128).astype(np.int8)
    el = dict(x=x, q=q)
    for i, (s, o) in enumerate([(0.25, 4), (0.05, -7), (0.0173, 33)]):
        el[f"quant{i}_params"] = np.array([s, o], np.float64)
        el[f"quant{i}_out"] = ref.quantize_i8(x, s, o)
        el[f"dequant{i}_out"] = ref.dequantize_i8(q, s, o)
    for i, (r, io, oo) in enumerate([(0.0123, -5, 7), (0.5, 0, -128), (1.7, 20, -3),
                                     (2.0, 1, 1)]):
        pre, post, sc, _ = go.quantize_scale_offset_32to8(r, 0)
        el[f"rescale{i}_params"] = np.array([oo, io, pre, post, sc], np.int32)
        el[f"rescale{i}_out"] = ref.rescale_i8(q, oo, io, pre, post, sc)
    save("elementwise", **el)

    # RowwiseQuantizedFullyConnected
    fc = {}
    for tag, (M, K, N), kw in [
            ("sym", (9, 70, 20), dict()),
            ("asym", (16, 128, 48), dict(symmetric=False)),
            ("bias8", (5, 33, 7), dict(symmetric=False, bias_i8=True,
                                       bias_scale=0.01, bias_offset=3))]:
        c = cases.rwq_fc_case(200, M, K, N, **kw)
        for k, v in c.items():
            fc[f"{tag}_{k}"] = np.asarray(v)
        fc[f"{tag}_out"] = ref.rwq_fc_i8(*cases.rwq_fc_args(c))
    save("rwq_fc", **fc)

    # plain FullyConnected + MatMul
    pf = {}
    for tag, shape, b8 in [("i32", (6, 50, 12), False), ("i8", (3, 21, 5), True)]:
        c = cases.fc_case(300, *shape, bias_i8=b8)
        for k, v in c.items():
            pf[f"{tag}_{k}"] = np.asarray(v)
        pf[f"{tag}_out"] = ref.fc_i8(*cases.fc_args(c))
        pf[f"{tag}_matmul_out"] = ref.matmul_i8(
            c["x"], c["w"], c["out_offset"], c["in_offset"], c["w_offset"], c["outP"])
    save("fc", **pf)

    # ChannelwiseQuantizedConvolution
    cv = {}
    for tag, kw in [
            ("relu3x3", dict(N=2, H=8, W=8, IC=16, OC=16)),
            ("stride2", dict(N=1, H=9, W=9, IC=8, OC=4, stride=(2, 2), pads=(0, 1, 2, 1))),
            ("group_dil", dict(N=1, H=8, W=6, IC=8, OC=8, group=2, dilation=(2, 1),
                               kernel=(2, 3), act=go.ACT_NONE, symmetric=False,
                               in_offset=-9, out_offset=5)),
            ("clip5x5", dict(N=1, H=5, W=5, IC=3, OC=5, kernel=(5, 5),
                             pads=(2, 2, 2, 2), act=go.ACT_CLIP)),
            ("leaky_b8", dict(N=1, H=6, W=7, IC=4, OC=8, act=go.ACT_LEAKY_RELU,
                              out_offset=10, bias_i8=True))]:
        c = cases.cwq_conv_case(400, **kw)
        for k, v in c.items():
            if k == "geom":
                cv[f"{tag}_geom"] = geom_vec(v)
            else:
                cv[f"{tag}_{k}"] = np.asarray(v, dtype=np.int32 if k == "act_args" else None)
        cv[f"{tag}_out"] = ref.cwq_conv2d_i8(*cases.cwq_conv_args(c))
    save("cwq_conv", **cv)

    # FusedRowwiseQuantizedSparseLengthsWeightedSum (8-bit, fp32)
    sl = {}
    rng = np.random.default_rng(500)
    for tag, (rows, cols, bags, mean), idt in [
            ("d128", (400, 128, 24, 40), np.int64),
            ("d37", (100, 37, 12, 6), np.int32)]:
        table = cases.random_fused_table(rng, rows, cols)
        lengths, idx, w = cases.slws_batch(501, rows, bags, mean, 1.05, idt)
        lengths[3] = 0  # an empty bag
        total = int(lengths.sum())
        idx, w = idx[:total], w[:total]
        sl[f"{tag}_table"] = table
        sl[f"{tag}_lengths"] = lengths
        sl[f"{tag}_indices"] = idx
        sl[f"{tag}_weights"] = w
        sl[f"{tag}_out"] = ref.frwq_slws_f32(table, w, idx, lengths)
    save("frwq_slws", **sl)
    glue()
    wide()


if __name__ == "__main__":
    if len(sys.argv) > 1:      # only the named files: python make_golden.py element_ops
        for what in sys.argv[1:]:
            globals()[what]()
    else:
        main()
        element_ops()

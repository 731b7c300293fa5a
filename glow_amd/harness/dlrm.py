"""DLRM-style ranking network on the quantized path: 4-bit fused-rowwise
embedding tables (fp16 scale and offset) pooled with
FusedRowwiseQuantizedSparseLengthsSum, a bottom int8 MLP over the dense
features, pairwise dot-product interaction of the 27 feature vectors
(BatchMatMul + Gather of the upper triangle), a top int8 MLP and a sigmoid.
Every FullyConnected is rowwise-quantized, like the reference's recommendation
system test builds them (tests/unittests/RecommendationSystemTest.cpp:913-932
uses the full n^2 interaction; the upper triangle gives the 351 + 64 = 415
inputs of the top MLP).

Scales come from one fp32 profiling batch evaluated in numpy on the host."""
import numpy as np

from glow_amd import capi
from glow_amd import host as H
from glow_amd import workloads
from glow_amd.harness import resnet50
from glow_amd.harness.net import Net


def _tqp(lo, hi):
    return capi.choose_quantization_params(float(lo), float(hi),
                                           capi.SCHEMA_SYMMETRIC_WITH_UNSIGNED, capi.QTY_INT8)


def _dequant_rows4(table, idx):
    """fp32 values of 4-bit fused rows (fp16 scale, offset) `idx`."""
    rows = table[idx]
    data = rows[:, :-4]
    so = np.ascontiguousarray(rows[:, -4:]).view(np.float16).astype(np.float32)
    q = np.empty((rows.shape[0], data.shape[1] * 2), np.float32)
    q[:, 0::2] = data & 15
    q[:, 1::2] = data >> 4
    return q * so[:, :1] + so[:, 1:2]


class Inputs:
    """One synthetic request batch."""

    def __init__(self, seed, tables, rows, batch, mean_len, alpha, dense_features):
        rng = np.random.default_rng(seed)
        self.dense = rng.normal(0, 1, (batch, dense_features)).astype(np.float32)
        self.lengths, self.indices = [], []
        for t in range(tables):
            ln, idx, _ = workloads.slws_batch(seed * 1000 + t, rows, batch, mean_len, alpha,
                                              np.int64, weighted=False)
            self.lengths.append(ln)
            self.indices.append(idx)


def make(tables=26, rows=1_000_000, dim=64, batch=4096, mean_len=20, alpha=1.1,
         dense_features=13, bottom=(512, 256, 64), top=(512, 256, 1), seed=0):
    """Returns (net, max_indices): index placeholders hold `max_indices` entries."""
    assert bottom[-1] == dim
    rng = np.random.default_rng(seed)
    emb = [workloads.random_fused_table(rng, rows, dim, workloads.U4_F16) for _ in range(tables)]

    def mlp(sizes, fan_in):
        layers = []
        for n in sizes:
            layers.append(((rng.standard_normal((n, fan_in)) * np.sqrt(2.0 / fan_in)).astype(np.float32),
                           (rng.standard_normal(n) * 0.05).astype(np.float32)))
            fan_in = n
        return layers

    nvec = tables + 1
    iu = np.triu_indices(nvec, 1)
    pair_idx = (iu[0] * nvec + iu[1]).astype(np.int64)
    bot = mlp(bottom, dense_features)
    topl = mlp(top, pair_idx.size + dim)

    # ---- fp32 profile on one batch -------------------------------------------
    prof = Inputs(seed + 1, tables, rows, batch, mean_len, alpha, dense_features)
    r = {"dense": (prof.dense.min(), prof.dense.max())}
    x = prof.dense
    for i, (w, b) in enumerate(bot):
        x = np.maximum(x @ w.T + b, 0)
        r[f"bot{i}"] = (x.min(), x.max())
    vecs = [x]
    lo, hi = x.min(), x.max()
    for t in range(tables):
        ends = np.cumsum(prof.lengths[t])
        vals = _dequant_rows4(emb[t], prof.indices[t])
        csum = np.concatenate([np.zeros((1, dim), np.float32), np.cumsum(vals, axis=0)])
        pooled = csum[ends] - csum[ends - prof.lengths[t]]
        vecs.append(pooled.astype(np.float32))
        lo, hi = min(lo, pooled.min()), max(hi, pooled.max())
    r["feat"] = (lo, hi)
    f3 = np.stack(vecs, axis=1)
    z = np.einsum("bik,bjk->bij", f3, f3)
    r["z"] = (min(z.min(), x.min()), max(z.max(), x.max()))
    x = np.concatenate([x, z.reshape(batch, -1)[:, pair_idx]], axis=1)
    for i, (w, b) in enumerate(topl):
        x = x @ w.T + b
        if i + 1 < len(topl):
            x = np.maximum(x, 0)
        r[f"top{i}"] = (x.min(), x.max())
    tq = {k: _tqp(*v) for k, v in r.items()}

    # ---- the quantized network -------------------------------------------------
    max_idx = int(max(i.size for i in prof.indices) * 1.25) + 64
    net = Net("dlrm_int8")
    net.placeholder("dense", (batch, dense_features), H.FLOAT)
    net.activation("dense_q", (batch, dense_features), H.INT8Q, *tq["dense"])
    net.op(H.QUANTIZE, "quantize_dense", ["dense_q", "dense"])

    def fc_stack(layers, src, src_tq, prefix, last_relu, out_placeholder=None):
        cur, cur_tq = src, src_tq
        for i, (w, b) in enumerate(layers):
            n, k = w.shape
            q, ws, wo = capi.rowwise_quantize_i8_host(w, capi.SCHEMA_SYMMETRIC)
            bq, bscale, boff = resnet50.quantize_fc_bias(b, w, cur_tq[0])
            name = f"{prefix}{i}"
            net.constant(name + "_w", q, H.INT8Q)
            net.constant(name + "_b", bq, H.INT32Q, bscale, boff)
            net.constant(name + "_s", ws, H.FLOAT)
            net.constant(name + "_o", wo, H.INT32I)
            relu = last_relu or i + 1 < len(layers)
            out_tq = tq[name]
            if relu:
                # the FC writes the pre-activation range, Relu narrows it
                pre_tq = _tqp(-r[name][1], r[name][1])
                net.activation(name + "_pre", (batch, n), H.INT8Q, *pre_tq)
                net.op(H.ROWWISE_QUANTIZED_FC, name, [name + "_pre", cur, name + "_w", name + "_b",
                                                      name + "_s", name + "_o"])
                net.activation(name, (batch, n), H.INT8Q, *out_tq)
                net.op(H.RELU, name + "_relu", [name, name + "_pre"])
            elif out_placeholder and i + 1 == len(layers):
                # an output of the network: the last FC writes it where it is saved
                net.placeholder(out_placeholder, (batch, n), H.INT8Q, *out_tq)
                net.op(H.ROWWISE_QUANTIZED_FC, name, [out_placeholder, cur, name + "_w", name + "_b",
                                                      name + "_s", name + "_o"])
                name = out_placeholder
            else:
                net.activation(name, (batch, n), H.INT8Q, *out_tq)
                net.op(H.ROWWISE_QUANTIZED_FC, name, [name, cur, name + "_w", name + "_b",
                                                      name + "_s", name + "_o"])
            cur, cur_tq = name, out_tq
        return cur, cur_tq

    bot_out, bot_tq = fc_stack(bot, "dense_q", tq["dense"], "bot", True)

    net.activation("feat", (batch, nvec * dim), H.INT8Q, *tq["feat"])
    net.activation("bot_f", (batch, dim), H.INT8Q, *tq["feat"])
    net.op(H.RESCALE_QUANTIZED, "bot_to_feat", ["bot_f", bot_out])
    net.op(H.INSERT_TENSOR, "insert_bot", ["feat", "bot_f"], [0])
    for t in range(tables):
        net.constant(f"table{t}", emb[t], H.UINT4_FUSED_FP16)
        net.placeholder(f"indices{t}", (max_idx,), H.INT64I)
        net.placeholder(f"lengths{t}", (batch,), H.INT32I)
        net.activation(f"emb{t}_h", (batch, dim), H.FLOAT16)
        net.op(H.FRWQ_SLS, f"sls{t}", [f"emb{t}_h", f"table{t}", f"indices{t}", f"lengths{t}"], [0])
        net.activation(f"emb{t}_f", (batch, dim), H.FLOAT)
        net.op(H.CONVERT_TO, f"convert{t}", [f"emb{t}_f", f"emb{t}_h"])
        net.activation(f"emb{t}_q", (batch, dim), H.INT8Q, *tq["feat"])
        net.op(H.QUANTIZE, f"quantize{t}", [f"emb{t}_q", f"emb{t}_f"])
        net.op(H.INSERT_TENSOR, f"insert{t}", ["feat", f"emb{t}_q"], [(t + 1) * dim])
    net.view("feat3", "feat", (batch, nvec, dim))
    net.activation("featT", (batch, dim, nvec), H.INT8Q, *tq["feat"])
    net.op(H.TRANSPOSE, "transpose", ["featT", "feat3"], [0, 2, 1])
    net.activation("z", (batch, nvec, nvec), H.INT8Q, *tq["z"])
    net.op(H.BATCH_MATMUL, "interact", ["z", "feat3", "featT"])
    net.view("z_flat", "z", (batch, nvec * nvec))
    net.constant("pair_idx", pair_idx, H.INT64I)
    net.activation("pairs", (batch, pair_idx.size), H.INT8Q, *tq["z"])
    net.op(H.GATHER, "upper_triangle", ["pairs", "z_flat", "pair_idx"], [1])
    net.activation("top_in", (batch, dim + pair_idx.size), H.INT8Q, *tq["z"])
    net.activation("bot_z", (batch, dim), H.INT8Q, *tq["z"])
    net.op(H.RESCALE_QUANTIZED, "bot_to_top", ["bot_z", bot_out])
    net.op(H.INSERT_TENSOR, "insert_dense", ["top_in", "bot_z"], [0])
    net.op(H.INSERT_TENSOR, "insert_pairs", ["top_in", "pairs"], [dim])
    top_out, _ = fc_stack(topl, "top_in", tq["z"], "top", False, "logit_q")
    net.activation("logit_f", (batch, top[-1]), H.FLOAT)
    net.op(H.DEQUANTIZE, "dequantize", ["logit_f", top_out])
    net.placeholder("prob", (batch, top[-1]), H.FLOAT)
    net.op(H.SIGMOID, "sigmoid", ["prob", "logit_f"])
    return net, max_idx


def bindings(net, inp, max_idx):
    """Host arrays for one request: name -> array (index tensors are statically
    sized; only the first sum(lengths) entries are used)."""
    b = {"dense": inp.dense}
    for t, (ln, idx) in enumerate(zip(inp.lengths, inp.indices)):
        assert idx.size <= max_idx
        b[f"lengths{t}"] = ln
        b[f"indices{t}"] = idx
    return b

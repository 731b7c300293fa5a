"""Int8 ResNet-50 (bottleneck {3,4,6,3}, stride on the 3x3 convolution, as
the reference's tests/benchmark/ResNetBench.cpp:138-385 builds it), quantized
from a profile the way Glow's profile-guided flow does: random He-normal fp32
weights (BatchNorm folded away), min/max of every activation over synthetic
N(0.45, 0.25) images, chooseQuantizationParams with the SymmetricWithUInt8
schema for activations; filters and biases of the convolutions through
createChannelwiseQuantizedConv's own preparation (per-channel parameters,
specializeBiasWeightsQuantizationParams, int32 biases at scale
inScale*filterScale); a RowwiseQuantizedFullyConnected classifier whose bias
is typed the way the quantizer types a FullyConnected bias; Dequantize and an
fp32 SoftMax. (The optimizer's rescale folding does not apply: this graph is
built without the Quantize/Dequantize pairs it removes.)

The fp32 profiling pass runs in numpy on the host; everything that is timed
runs on the GPU through the host layer."""
import numpy as np

from glow_amd import capi
from glow_amd import host as H
from glow_amd.harness.net import Net

LAYERS = ((64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2))   # planes, blocks, stride


class _Conv:
    def __init__(self, rng, ic, oc, k, stride, pad, relu):
        self.k, self.stride, self.pad, self.relu = k, stride, pad, relu
        self.w = (rng.standard_normal((oc, k, k, ic)) * np.sqrt(2.0 / (k * k * ic))).astype(np.float32)
        self.b = (rng.standard_normal(oc) * 0.05).astype(np.float32)


def build_fp32(seed=0, layers=LAYERS, classes=1000, stem=64):
    """The fp32 network as a list of steps over named values."""
    rng = np.random.default_rng(seed)
    steps = []      # (op, out, inputs, params)
    steps.append(("conv", "stem", ["input"], _Conv(rng, 3, stem, 7, 2, 3, True)))
    steps.append(("maxpool", "pool", ["stem"], (3, 2, 1)))
    cur, ch = "pool", stem
    for li, (planes, blocks, stride) in enumerate(layers):
        for b in range(blocks):
            s = stride if b == 0 else 1
            tag = f"l{li}b{b}"
            res = cur
            if b == 0 and (s != 1 or ch != planes * 4):
                steps.append(("conv", tag + "_sc", [cur], _Conv(rng, ch, planes * 4, 1, s, 0, False)))
                res = tag + "_sc"
            steps.append(("conv", tag + "_c1", [cur], _Conv(rng, ch, planes, 1, 1, 0, True)))
            steps.append(("conv", tag + "_c2", [tag + "_c1"], _Conv(rng, planes, planes, 3, s, 1, True)))
            steps.append(("conv", tag + "_c3", [tag + "_c2"], _Conv(rng, planes, planes * 4, 1, 1, 0, False)))
            steps.append(("add", tag + "_sum", [tag + "_c3", res], None))
            steps.append(("relu", tag + "_out", [tag + "_sum"], None))
            cur, ch = tag + "_out", planes * 4
    steps.append(("avgpool", "gap", [cur], None))
    fc_w = (rng.standard_normal((classes, ch)) * np.sqrt(1.0 / ch)).astype(np.float32)
    fc_b = (rng.standard_normal(classes) * 0.05).astype(np.float32)
    steps.append(("fc", "logits", ["gap"], (fc_w, fc_b)))
    return steps


def _conv_fp32(x, c):
    """NHWC fp32 convolution as k*k shifted matrix products."""
    n, h, w, ic = x.shape
    oc = c.w.shape[0]
    oh = (h + 2 * c.pad - c.k) // c.stride + 1
    ow = (w + 2 * c.pad - c.k) // c.stride + 1
    if c.pad:
        x = np.pad(x, ((0, 0), (c.pad, c.pad), (c.pad, c.pad), (0, 0)))
    out = np.zeros((n * oh * ow, oc), np.float32)
    for kh in range(c.k):
        for kw in range(c.k):
            v = x[:, kh:kh + (oh - 1) * c.stride + 1:c.stride,
                  kw:kw + (ow - 1) * c.stride + 1:c.stride, :]
            out += np.ascontiguousarray(v).reshape(-1, ic) @ c.w[:, kh, kw, :].T
    out += c.b
    if c.relu:
        np.maximum(out, 0, out=out)
    return out.reshape(n, oh, ow, oc)


def _maxpool_fp32(x, k, s, p):
    n, h, w, ch = x.shape
    oh, ow = (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1
    xp = np.pad(x, ((0, 0), (p, p), (p, p), (0, 0)), constant_values=-np.inf)
    out = np.full((n, oh, ow, ch), -np.inf, np.float32)
    for kh in range(k):
        for kw in range(k):
            np.maximum(out, xp[:, kh:kh + (oh - 1) * s + 1:s, kw:kw + (ow - 1) * s + 1:s, :], out=out)
    return out


def profile(steps, images):
    """min/max of every value over `images` [N,H,W,3] fp32 (processed in chunks)."""
    lo, hi = {}, {}

    def note(name, v):
        lo[name] = min(lo.get(name, np.inf), float(v.min()))
        hi[name] = max(hi.get(name, -np.inf), float(v.max()))

    for i in range(0, images.shape[0], 10):
        vals = {"input": images[i:i + 10]}
        note("input", vals["input"])
        for op, out, ins, prm in steps:
            a = vals[ins[0]]
            if op == "conv":
                v = _conv_fp32(a, prm)
            elif op == "maxpool":
                v = _maxpool_fp32(a, *prm)
            elif op == "add":
                v = a + vals[ins[1]]
            elif op == "relu":
                v = np.maximum(a, 0)
            elif op == "avgpool":
                v = a.mean(axis=(1, 2), keepdims=True)
            else:
                v = a.reshape(a.shape[0], -1) @ prm[0].T + prm[1]
            vals[out] = v
            note(out, v)
    return {k: (lo[k], hi[k]) for k in lo}


def _tqp(rng_):
    return capi.choose_quantization_params(rng_[0], rng_[1], capi.SCHEMA_SYMMETRIC_WITH_UNSIGNED,
                                           capi.QTY_INT8)


SCHEMA = capi.SCHEMA_SYMMETRIC_WITH_UNSIGNED


def _quantize_rows(w2d):
    q, scales, offsets = capi.rowwise_quantize_i8_host(w2d, capi.SCHEMA_SYMMETRIC)
    return q, scales, offsets


def quantize_fc_bias(bias, weights, in_scale):
    """The int32 bias of a FullyConnected as Glow's quantizer types it before the
    node becomes rowwise-quantized (reference lib/Quantization/Quantization.cpp:
    103-113, 142-152): its own range as an Int32QTy tensor, specialised against
    the input's scale and the scale of the WHOLE weight tensor
    (specializeBiasQuantizationParams). Returns (int32 values, scale, offset)."""
    w_scale, _ = capi.choose_quantization_params(float(weights.min()), float(weights.max()),
                                                 SCHEMA, capi.QTY_INT8)
    own_scale, own_off = capi.choose_quantization_params(float(bias.min()), float(bias.max()),
                                                         SCHEMA, capi.QTY_INT32)
    scale, off = capi.specialize_bias_qparams(own_scale, own_off, in_scale, w_scale,
                                              bias_is_i32=True, bias_is_zero=not bias.any())
    q = np.rint(bias.astype(np.float32) / np.float32(scale) + np.float32(off))
    return np.clip(q, -2 ** 31, 2 ** 31 - 1).astype(np.int32), scale, off


def build_int8(steps, ranges, batch, size, chains=1):
    """The quantized network as lowered instructions. chains > 1: the batch is
    computed as that many independent instruction chains over equal slices of
    the input and output placeholders, sharing every constant (the data-parallel
    split of Glow's parallelizeOps, reference
    include/glow/Optimizer/GraphOptimizer/GraphOptimizer.h:199-211): nothing
    orders one chain's launches against another's, so a device manager may run
    them side by side."""
    assert batch % chains == 0
    net = Net("resnet50_int8")
    tq = {k: _tqp(v) for k, v in ranges.items()}
    per = batch // chains
    net.placeholder("input", (batch, size, size, 3), H.FLOAT)
    classes = [prm[0].shape[0] for op, _, _, prm in steps if op == "fc"][0]
    out_q = None
    for c in range(chains):
        sfx = "" if chains == 1 else f"@{c}"
        first = c == 0
        shapes = {"input": (per, size, size, 3)}
        if chains == 1:
            x = "input"
        else:
            x = net.view("input" + sfx, "input", shapes["input"], first=c * per * size * size * 3)
        net.activation("input_q" + sfx, shapes["input"], H.INT8Q, *tq["input"])
        net.op(H.QUANTIZE, "quantize" + sfx, ["input_q" + sfx, x])
        name_of = {"input": "input_q" + sfx}
        for op, out, ins, prm in steps:
            src = name_of[ins[0]]
            ishape = shapes[ins[0]]
            o = out + sfx
            if op == "conv":
                n, h, w, ic = ishape
                oc = prm.w.shape[0]
                oh = (h + 2 * prm.pad - prm.k) // prm.stride + 1
                ow = (w + 2 * prm.pad - prm.k) // prm.stride + 1
                shapes[out] = (n, oh, ow, oc)
                if first:
                    # what Quantizer::enableChannelwise makes of a Convolution with
                    # constant fp32 filter and bias (createChannelwiseQuantizedConv)
                    q, bq, fs, fo, bs, bo = capi.channelwise_quantize_conv_host(
                        prm.w, prm.b, tq[ins[0]][0], SCHEMA)
                    net.constant(out + "_filter", q, H.INT8Q)
                    net.constant(out + "_bias", bq, H.INT32Q)
                    net.constant(out + "_fscales", fs, H.FLOAT)
                    net.constant(out + "_foffsets", fo, H.INT32I)
                    net.constant(out + "_bscales", bs, H.FLOAT)
                    net.constant(out + "_boffsets", bo, H.INT32I)
                net.activation(o, shapes[out], H.INT8Q, *tq[out])
                net.op(H.CHANNELWISE_QUANTIZED_CONV, o,
                       [o, src, out + "_filter", out + "_bias", out + "_fscales",
                        out + "_foffsets", out + "_bscales", out + "_boffsets"],
                       H.conv_attrs((prm.k, prm.k), (prm.stride, prm.stride), (prm.pad,) * 4,
                                    act=H.ACT_RELU if prm.relu else H.ACT_NONE))
            elif op == "maxpool":
                k, s, p = prm
                n, h, w, ch = ishape
                shapes[out] = (n, (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1, ch)
                # max pool passes values through: it keeps its input's parameters
                tq[out] = tq[ins[0]]
                net.activation(o, shapes[out], H.INT8Q, *tq[out])
                net.op(H.MAX_POOL, o, [o, src], [k, k, s, s, p, p, p, p])
            elif op == "add":
                shapes[out] = ishape
                net.activation(o, ishape, H.INT8Q, *tq[out])
                net.op(H.ELEMENT_ADD, o, [o, src, name_of[ins[1]]])
            elif op == "relu":
                shapes[out] = ishape
                net.activation(o, ishape, H.INT8Q, *tq[out])
                net.op(H.RELU, o, [o, src])
            elif op == "avgpool":
                n, h, w, ch = ishape
                shapes[out] = (n, 1, 1, ch)
                net.activation(o, shapes[out], H.INT8Q, *tq[out])
                net.op(H.AVG_POOL, o, [o, src], [h, w, 1, 1, 0, 0, 0, 0, 1])
            else:
                fw, fb = prm
                n = ishape[0]
                _, k = fw.shape
                shapes[out] = (n, classes)
                if first:
                    q, ws, wo = _quantize_rows(fw)
                    bq, bscale, boff = quantize_fc_bias(fb, fw, tq[ins[0]][0])
                    net.constant("fc_weights", q, H.INT8Q)
                    net.constant("fc_bias", bq, H.INT32Q, bscale, boff)
                    net.constant("fc_scales", ws, H.FLOAT)
                    net.constant("fc_offsets", wo, H.INT32I)
                    # the int8 logits are an output of the network: the FC writes
                    # them where they are saved
                    net.placeholder("logits_q", (batch, classes), H.INT8Q, *tq[out])
                # the pooled [N,1,1,C] tensor is read as [N,C]: the same bytes (a
                # Reshape is a TensorView in Glow's IR, no instruction)
                net.view("gap_2d" + sfx, src, (n, k))
                out_q = "logits_q"
                if chains > 1:
                    out_q = net.view("logits_q" + sfx, "logits_q", (n, classes),
                                     first=c * per * classes)
                net.op(H.ROWWISE_QUANTIZED_FC, "fc" + sfx,
                       [out_q, "gap_2d" + sfx, "fc_weights", "fc_bias", "fc_scales", "fc_offsets"])
                name_of[out] = out_q
                continue
            name_of[out] = o
        net.activation("logits_f" + sfx, (per, classes), H.FLOAT)
        net.op(H.DEQUANTIZE, "dequantize" + sfx, ["logits_f" + sfx, out_q])
        if first:
            net.placeholder("prob", (batch, classes), H.FLOAT)
        prob = "prob"
        if chains > 1:
            prob = net.view("prob" + sfx, "prob", (per, classes), first=c * per * classes)
        net.op(H.SOFTMAX, "softmax" + sfx, [prob, "logits_f" + sfx])
    if chains > 1:
        # step k of every chain before step k + 1 of any: a device manager that
        # records the list stream by stream then finds each chain's launches
        # behind one another on a stream of their own, not behind another chain's
        per_chain = len(net.ops) // chains
        net.ops = [net.ops[c * per_chain + k] for k in range(per_chain) for c in range(chains)]
    return net


def synthetic_images(seed, n, size):
    rng = np.random.default_rng(seed)
    return rng.normal(0.45, 0.25, (n, size, size, 3)).astype(np.float32)


def make(batch=64, size=224, profile_images=100, seed=0, layers=LAYERS, classes=1000, chains=1):
    steps = build_fp32(seed, layers, classes)
    ranges = profile(steps, synthetic_images(seed + 1, profile_images, size))
    return build_int8(steps, ranges, batch, size, chains)

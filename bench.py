"""Benchmark of the MI355X quantized-inference hot path on ONE GPU.

Headline workload (one step = one pass of the hot path over one batch):
FusedRowwiseQuantizedSparseLengthsWeightedSum over a uint8 fused-rowwise table
of 4M rows x 128 dims (fp32 scale and offset per row, 136-byte rows, 544 MB),
4096 bags with Poisson(40) lengths, Zipf(1.05) int64 indices, fp32 weights
U[0,1), fp32 output [4096 x 128]. Throughput is counted the way the
reference's SLS benchmark counts bytes (tests/benchmark/CommonSLSEB.h:120-176:
every lookup moves its row, scale and offset, index and weight; plus lengths
and output; no credit for cache hits).

Prints ONE JSON line. Besides the headline it reports, under "extra", the
int8 matrix-core kernels (RowwiseQuantizedFullyConnected at the single-FC
configuration and at a large shape, ChannelwiseQuantizedConvolution at the
ResNet-50 3x3x64 layer shape) and the elementwise kernels, each with its own
roofline fraction, and times the CPU oracle on this host's cores.

  python bench.py --gpus 1 --steps 200 --warmup 20
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# HBM bytes per launch of the default workloads (FETCH_SIZE + WRITE_SIZE of two
# counter runs, scaled by what the counters read for a plain copy of known
# size). They hold for the default sizes only; other sizes report null.
MEASURED_TRAFFIC = {"slws": 23.98e6, "fc_large": 236.3e6, "conv_c3": 13.40e6}

HBM_PEAK_GBPS = 8000.0       # MI355X HBM3E, published
INT8_PEAK_TOPS = 5000.0      # MI355X dense int8 MFMA, published (5.0 POP/s)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batches", type=int, default=8,
                    help="distinct index batches cycled through by the steps")
    ap.add_argument("--rows", type=int, default=4_000_000)
    ap.add_argument("--bags", type=int, default=4096,
                    help="bags per step (4096 is the headline configuration)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0,
                    help="wall-clock budget of the CPU baseline leg")
    ap.add_argument("--resnet-batch", type=int, default=64)
    ap.add_argument("--resnet-profile-images", type=int, default=100)
    ap.add_argument("--dlrm-rows", type=int, default=1_000_000)
    ap.add_argument("--no-extra", action="store_true",
                    help="headline workload only")
    ap.add_argument("--only", default="",
                    help="run a single extra kernel (profiling aid): "
                         "slws|fc_large|fc_large_zero|fc_c1|fc_m16384|fc_mid|conv_c3|quantize|dequantize|"
                         "rescale|copy|resnet50|dlrm")
    ap.add_argument("--tile", type=int, default=-1,
                    help="force a workgroup tile for the matrix-core legs of --only "
                         "(0..5, see mi355x_gemm_tile_override; default: chosen from the shape)")
    return ap.parse_args()


def timed_launches(capi, fn, steps, warmup):
    """Average seconds per launch. `fn(i, stream)` issues launch i. After
    `warmup` eager launches, the `steps` timed launches are recorded into one
    launch graph and replayed, so the figure is the device-side rate and not
    the host's enqueue rate (a Python -> ctypes -> HIP launch costs 4-6 us,
    more than some of these kernels take). HIP events bracket the replay on
    the stream it runs on, with the device idle before and after."""
    stream = capi.Stream()
    for i in range(warmup):
        fn(i, stream)
    stream.sync()
    with capi.Graph(stream) as graph:
        for i in range(steps):
            fn(warmup + i, stream)
    graph.launch()          # untimed first replay (uploads the graph)
    stream.sync()
    capi.sync()
    e0, e1 = capi.Event(), capi.Event()
    e0.record(stream)
    graph.launch()
    e1.record(stream)
    e1.sync()
    capi.sync()
    sec = e0.elapsed_ms(e1) * 1e-3 / steps
    graph.destroy()
    return sec


def slws_bytes(total_lookups, bags, cols, row_bytes):
    """Algorithmic bytes of one launch (reference CommonSLSEB.h:120-176)."""
    return total_lookups * (row_bytes + 8 + 4) + bags * 4 + bags * cols * 4


def bench_slws(capi, cases, args, table, d_table):
    rows, cols, bags = args.rows, 128, args.bags
    row_bytes = cols + 8
    batches = []
    for b in range(args.batches):
        lengths, idx, w = cases.slws_batch(1000 + b, rows, bags, 40, 1.05, np.int64)
        batches.append(dict(
            lengths=lengths, idx=idx, w=w, total=int(lengths.sum()),
            d_len=capi.to_device(lengths), d_idx=capi.to_device(idx),
            d_w=capi.to_device(w)))
    d_out = capi.DeviceBuffer.empty((bags, cols), np.float32)

    def step(i, stream):
        b = batches[i % len(batches)]
        capi.launch_frwq_slws(d_out, False, d_table, rows, capi.FUSED_U8_F32,
                              b["d_w"], False, b["d_idx"], True, b["total"],
                              b["d_len"], bags, row_bytes, cols, stream=stream)

    sec = timed_launches(capi, step, args.steps, args.warmup)
    mean_total = float(np.mean([batches[(args.warmup + i) % len(batches)]["total"]
                                for i in range(args.steps)]))
    nbytes = slws_bytes(mean_total, bags, cols, row_bytes)
    return dict(sec=sec, bytes=nbytes, batches=batches, mean_lookups=mean_total,
                d_out=d_out)


def bench_slws_with_h2d(capi, s, args, d_table):
    """Same launches, but every step first copies its indices, weights and
    lengths from pinned host memory: what a DeviceManager does per request."""
    import ctypes as C
    rows, cols, bags = args.rows, 128, args.bags
    pinned = []
    for b in s["batches"]:
        ent = {}
        for key, arr in (("idx", b["idx"]), ("w", b["w"]), ("lengths", b["lengths"])):
            hp = C.c_void_p(0)
            capi.check(capi.lib().mi355x_host_alloc(C.byref(hp), C.c_size_t(max(arr.nbytes, 1))))
            C.memmove(hp.value, arr.ctypes.data, arr.nbytes)
            ent[key] = (hp, arr.nbytes)
        pinned.append(ent)

    def step(i, stream):
        b = s["batches"][i % len(s["batches"])]
        h = pinned[i % len(pinned)]
        for key, dst in (("idx", b["d_idx"]), ("w", b["d_w"]), ("lengths", b["d_len"])):
            hp, n = h[key]
            capi.check(capi.lib().mi355x_memcpy_h2d(C.c_void_p(dst.ptr), hp, C.c_size_t(n),
                                                    C.c_void_p(stream.ptr)))
        capi.launch_frwq_slws(s["d_out"], False, d_table, rows, capi.FUSED_U8_F32,
                              b["d_w"], False, b["d_idx"], True, b["total"],
                              b["d_len"], bags, cols + 8, cols, stream=stream)

    sec = timed_launches(capi, step, args.steps, args.warmup)
    for h in pinned:
        for hp, _ in h.values():
            capi.lib().mi355x_host_free(hp)
    return dict(workload="SLWS headline step + H2D of indices, weights, lengths "
                         "from pinned host memory", ms=sec * 1e3,
                gbps=s["bytes"] / sec / 1e9,
                h2d_bytes_per_step=s["mean_lookups"] * 12 + bags * 4)


def bench_slws_more_bags(capi, cases, args, d_table, bags):
    """The headline lookup on the same table with a larger batch: the part of a
    launch that does not shrink with the batch (dispatch, bag offsets, the
    index -> row dependent round trips) is spread over more bytes."""
    rows, cols = args.rows, 128
    lengths, idx, w = cases.slws_batch(2000 + bags, rows, bags, 40, 1.05, np.int64)
    total = int(lengths.sum())
    d_len, d_idx, d_w = capi.to_device(lengths), capi.to_device(idx), capi.to_device(w)
    d_out = capi.DeviceBuffer.empty((bags, cols), np.float32)

    def step(_, stream):
        capi.launch_frwq_slws(d_out, False, d_table, rows, capi.FUSED_U8_F32, d_w, False, d_idx,
                              True, total, d_len, bags, cols + 8, cols, stream=stream)

    sec = timed_launches(capi, step, max(20, args.steps // 4), max(3, args.warmup // 4))
    nbytes = slws_bytes(total, bags, cols, cols + 8)
    return dict(workload=f"SLWS, same table, {bags} bags ({total} lookups)", ms=sec * 1e3,
                gbps=nbytes / sec / 1e9, frac_of_hbm_peak=nbytes / sec / 1e9 / HBM_PEAK_GBPS)


def cpu_all_cores_slws(table, batches, budget_s):
    """The oracle on every host core this process may use, one whole batch per
    thread at a time (the reference's CPU backend exposes one device per
    hardware thread, lib/Backends/CPU/CPUBackend.cpp:114-116)."""
    import threading
    from oracle import glow_oracle as go
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else os.cpu_count()
    cores = max(1, min(cores, 16))
    done = [0.0] * cores
    t0 = time.perf_counter()

    def work(t):
        n = t
        while time.perf_counter() - t0 < budget_s:
            b = batches[n % len(batches)]
            go.frwq_slws_f32(table, b["w"], b["idx"], b["lengths"])
            done[t] += slws_bytes(b["total"], b["lengths"].size, 128, 136)
            n += cores

    th = [threading.Thread(target=work, args=(t,)) for t in range(cores)]
    for t in th:
        t.start()
    for t in th:
        t.join()
    el = time.perf_counter() - t0
    return dict(value=sum(done) / el / 1e9, unit="GB/s", cores=cores, kind="port",
                sample=f"whole batches for {el:.1f} s, one batch per thread at a time")


def cpu_baseline_slws(table, batches, budget_s, gpu_out, gpu_batch):
    """The CPU leg: the oracle (the restated libjit loop, one thread) over
    whole batches of the same workload until the time budget is used. As the
    checker it also confirms the GPU output of the last timed step."""
    from oracle import glow_oracle as go
    want = go.frwq_slws_f32(table, gpu_batch["w"], gpu_batch["idx"],
                            gpu_batch["lengths"])
    # default (fused multiply-add) arithmetic: equal to the sequential CPU loop
    # to rounding; the bar is 1e-5 of the magnitude a bag adds up
    from glow_amd import workloads
    parity = workloads.slws_error_ratio(gpu_out, want, table, gpu_batch["w"],
                                        gpu_batch["idx"], gpu_batch["lengths"])
    done_bytes, n = 0.0, 0
    t0 = time.perf_counter()
    while True:
        b = batches[n % len(batches)]
        go.frwq_slws_f32(table, b["w"], b["idx"], b["lengths"])
        done_bytes += slws_bytes(b["total"], b["lengths"].size, 128, 136)
        n += 1
        el = time.perf_counter() - t0
        if el >= budget_s or n >= 4000:
            break
    return dict(value=done_bytes / el / 1e9, unit="GB/s", cores=1, kind="port",
                sample=f"{n} full batches of {batches[0]['lengths'].size} bags (single thread, "
                       f"{el:.1f} s) of the same table and index batches"), parity


def bench_fc(capi, cases, M, K, N, steps, warmup, seed=5, zero_leg=False):
    c = cases.rwq_fc_case(seed, M, K, N) if M * K <= (1 << 24) else None
    rng = np.random.default_rng(seed)
    if c is None:
        # large shape: same distributions, parameters from a small case
        small = cases.rwq_fc_case(seed, 8, 64, N)
        c = dict(small)
        c["x"] = np.clip(np.rint(rng.normal(0, 40, (M, K))), -128, 127).astype(np.int8)
        c["w"] = rng.integers(-127, 128, (N, K)).astype(np.int8)
    d = {k: capi.to_device(np.ascontiguousarray(v)) for k, v in c.items()
         if isinstance(v, np.ndarray)}
    d_out = capi.DeviceBuffer.empty((M, N), np.int8)
    # weights are constants: their row sums are formed once, outside the steps
    d_sums = capi.DeviceBuffer.empty((N,), np.int32)
    capi.launch_rowsum_i8(d_sums, d["w"], N, K)

    def step(_, stream):
        capi.launch_rwq_fc_i8(d_out, d["x"], d["w"], d["bias"], False,
                              d["w_offsets"], d["bias_pre"], d["bias_post"],
                              d["bias_scale"], d["out_pre"], d["out_post"],
                              d["out_scale"], M, K, N, c["out_offset"],
                              c["in_offset"], c["bias_offset"], True,
                              w_row_sums=d_sums, stream=stream)

    sec = timed_launches(capi, step, steps, warmup)
    ops = 2.0 * M * N * K
    zero = None
    if zero_leg:
        # The same launch on all-zero operands: identical instruction stream,
        # but the matrix cores toggle no data, so the part holds a higher clock
        # under its power limit. The ratio shows how much of the distance to
        # the published peak is clock, not kernel.
        d["x"].fill(0)
        d["w"].fill(0)
        capi.sync()
        zsec = timed_launches(capi, step, steps, warmup)
        zero = dict(ms=zsec * 1e3, tops=ops / zsec / 1e12)
    normal = None
    if zero_leg:
        # Weights as symmetric per-row quantization makes them from normally
        # distributed fp32 rows (q = rint(127 w / max|w|): mostly small
        # magnitudes) instead of uniform int8: same instruction stream again,
        # fewer bits toggling than with uniform weights.
        wf = rng.normal(0, 1, (N, K)).astype(np.float32)
        wq = np.rint(wf * (127.0 / np.abs(wf).max(axis=1, keepdims=True))).astype(np.int8)
        d["x"].upload(c["x"])
        d["w"].upload(wq)
        capi.sync()
        nsec = timed_launches(capi, step, steps, warmup)
        normal = dict(ms=nsec * 1e3, tops=ops / nsec / 1e12)
    return dict(workload=f"rwq_fc M{M} K{K} N{N}", ms=sec * 1e3,
                tops=ops / sec / 1e12, zero_operands=zero, normal_weights=normal,
                roofline=dict(bound="mfma", achieved=ops / sec / 1e12,
                              peak=INT8_PEAK_TOPS, unit="TOP/s",
                              frac=ops / sec / 1e12 / INT8_PEAK_TOPS,
                              traffic=(MEASURED_TRAFFIC["fc_large"]
                                       if (M, K, N) == (8192, 4096, 4096) else None)),
                gbps=(M * K + N * K + M * N + 8 * 4 * N) / sec / 1e9)


def bench_conv(capi, cases, steps, warmup):
    c = cases.cwq_conv_case(7, 32, 56, 56, 64, 64, in_offset=-128)
    g = capi._geom(c["geom"])
    d = {k: capi.to_device(np.ascontiguousarray(v)) for k, v in c.items()
         if isinstance(v, np.ndarray)}
    d_out = capi.DeviceBuffer.empty((g.N, g.OH, g.OW, g.OC), np.int8)
    d_sums = capi.DeviceBuffer.empty((g.OC,), np.int32)
    capi.launch_rowsum_i8(d_sums, d["filt"], g.OC, c["filt"].size // g.OC)

    def step(_, stream):
        capi.launch_cwq_conv2d_i8(d_out, d["x"], d["filt"], d["bias"], False, g,
                                  c["out_offset"], c["in_offset"],
                                  d["f_offsets"], d["b_offsets"], d["bias_pre"],
                                  d["bias_post"], d["bias_scale"], d["out_pre"],
                                  d["out_post"], d["out_scale"], c["act"],
                                  c["act_args"], True, f_row_sums=d_sums,
                                  stream=stream)

    sec = timed_launches(capi, step, steps, warmup)
    ops = 2.0 * g.N * g.OH * g.OW * g.OC * g.KH * g.KW * g.IC
    nbytes = c["x"].size + d_out.nbytes + c["filt"].size + 9 * 4 * g.OC
    return dict(workload="cwq_conv2d 32x56x56x64 3x3x64->64 s1 p1 relu",
                ms=sec * 1e3, tops=ops / sec / 1e12, gbps=nbytes / sec / 1e9,
                roofline=dict(bound="mfma", achieved=ops / sec / 1e12,
                              peak=INT8_PEAK_TOPS, unit="TOP/s",
                              frac=ops / sec / 1e12 / INT8_PEAK_TOPS,
                              traffic=MEASURED_TRAFFIC["conv_c3"]))


def bench_elementwise(capi, which, steps, warmup):
    n = 64 * 56 * 56 * 64 * 4  # four ResNet stem activations: 51.4M elements
    rng = np.random.default_rng(3)
    if which == "quantize":
        src = capi.to_device(rng.normal(0, 1, n).astype(np.float32))
        dst = capi.DeviceBuffer.empty((n,), np.int8)
        fn = lambda _, st: capi.launch_quantize_i8(dst, src, n, 0.02, -3, st)
        nbytes = n * 5
    elif which == "dequantize":
        src = capi.to_device(rng.integers(-128, 128, n).astype(np.int8))
        dst = capi.DeviceBuffer.empty((n,), np.float32)
        fn = lambda _, st: capi.launch_dequantize_i8(dst, src, n, 0.02, -3, st)
        nbytes = n * 5
    elif which == "copy":
        # plain copy of known size: what the HBM byte counters are scaled by
        n = 256 << 20
        src = capi.to_device(rng.integers(-128, 128, n).astype(np.int8))
        dst = capi.DeviceBuffer.empty((n,), np.int8)
        fn = lambda _, st: capi.launch_copy_u8(dst, src, n, st)
        nbytes = n * 2
    else:
        src = capi.to_device(rng.integers(-128, 128, n).astype(np.int8))
        dst = capi.DeviceBuffer.empty((n,), np.int8)
        fn = lambda _, st: capi.launch_rescale_i8(dst, src, n, 3, -5, 2, 15, 300, st)
        nbytes = n * 2
    sec = timed_launches(capi, fn, steps, warmup)
    return dict(workload=f"{which}_u8 n={n}" if which == "copy" else f"{which}_i8 n={n}", ms=sec * 1e3,
                gbps=nbytes / sec / 1e9,
                roofline=dict(bound="hbm", achieved=nbytes / sec / 1e9,
                              peak=HBM_PEAK_GBPS, unit="GB/s",
                              frac=nbytes / sec / 1e9 / HBM_PEAK_GBPS,
                              traffic=None))


def cpu_baseline_mfma_kernels(budget_s):
    """The oracle (the restated libjit loops, one thread) on the single-FC
    configuration and on a bounded slice of the ResNet 3x3 convolution: the
    reference's CPU path for the two matrix-core workloads."""
    from oracle import glow_oracle as go
    from tests import cases as ocases
    out = {}
    c = ocases.rwq_fc_case(5, 128, 1024, 1024)
    args_ = ocases.rwq_fc_args(c)
    n, t0 = 0, time.perf_counter()
    while True:
        go.rwq_fc_i8(*args_)
        n += 1
        el = time.perf_counter() - t0
        if el >= budget_s / 2 or n >= 200:
            break
    out["rwq_fc_c1"] = dict(value=2.0 * 128 * 1024 * 1024 * n / el / 1e9, unit="GOP/s", cores=1,
                            kind="port", sample=f"{n} full passes of M128 K1024 N1024 in {el:.1f} s")
    # two images of the 32-image batch (same layer shape), repeated
    cc = ocases.cwq_conv_case(7, 2, 56, 56, 64, 64, in_offset=-128)
    cargs = ocases.cwq_conv_args(cc)
    n, t0 = 0, time.perf_counter()
    while True:
        go.cwq_conv2d_i8(*cargs)
        n += 1
        el = time.perf_counter() - t0
        if el >= budget_s / 2 or n >= 200:
            break
    out["cwq_conv_c3"] = dict(value=2.0 * 2 * 56 * 56 * 64 * 576 * n / el / 1e9, unit="GOP/s",
                              cores=1, kind="port",
                              sample=f"{n} passes over 2 of the 32 images (56x56x64, 3x3x64->64) "
                                     f"in {el:.1f} s")
    return out


def bench_resnet50(args):
    """Int8 ResNet-50 at batch 64, 224x224 through MI355XDeviceManager:
    images/s of the resident network replayed on device-resident input
    (device time), and of whole requests including the fp32 input upload and
    the result download."""
    from glow_amd import host as H
    from glow_amd.harness import net as netlib
    from glow_amd.harness import resnet50
    batch, size = args.resnet_batch, 224
    t0 = time.perf_counter()
    net = resnet50.make(batch=batch, size=size, profile_images=args.resnet_profile_images)
    t_build = time.perf_counter() - t0
    m, f = netlib.to_module(net)
    m.compile(f)
    dm = H.DeviceManager().init()
    try:
        dm.add_network(m)
        # request buffers in pinned host memory (allocateDeviceIOBuffer)
        from glow_amd import capi
        x = capi.pinned_copy(resnet50.synthetic_images(77, batch, size))
        prob = capi.pinned_empty((batch, 1000), np.float32)
        logits = capi.pinned_empty((batch, 1000), np.int8)
        dm.run("main", {"input": x, "prob": prob, "logits_q": logits})
        reps = max(3, args.steps // 10)
        ms = dm.time_function("main", reps)
        t1 = time.perf_counter()
        for _ in range(3):
            dm.run("main", {"input": x, "prob": prob, "logits_q": logits})
        e2e = (time.perf_counter() - t1) / 3
    finally:
        dm.stop()
    ops = net.ops_count()
    return dict(workload=f"int8 ResNet-50, batch {batch}, {size}x{size}x3, channelwise-quantized "
                         f"convolutions, rowwise-quantized FC, fp32 softmax; "
                         f"{args.resnet_profile_images} profiling images",
                images_per_s=batch / (ms * 1e-3), ms_per_batch=ms,
                images_per_s_with_host_copies=batch / e2e,
                tops=ops / (ms * 1e-3) / 1e12, gop_per_image=ops / batch / 1e9,
                launches_per_batch=len([r for r in H.parse_listing(m.describe(f))
                                        if r["phase"] == "launch"]),
                prob_row_sum=float(prob[0].sum()), host_build_seconds=t_build)


def bench_dlrm(args):
    """DLRM-style ranking net, batch 4096: 26 tables of 1M x 64 (4-bit fused,
    fp16 scale/offset), Poisson(20) bags of Zipf(1.1) int64 indices, int8 MLPs
    13-512-256-64 and 415-512-256-1, dot interaction, sigmoid."""
    from glow_amd import host as H
    from glow_amd.harness import dlrm
    from glow_amd.harness import net as netlib
    batch, tables = 4096, 26
    t0 = time.perf_counter()
    net, max_idx = dlrm.make(tables=tables, rows=args.dlrm_rows, batch=batch)
    t_build = time.perf_counter() - t0
    m, f = netlib.to_module(net)
    m.compile(f)
    dm = H.DeviceManager().init()
    try:
        dm.add_network(m)
        inp = dlrm.Inputs(99, tables, args.dlrm_rows, batch, 20, 1.1, 13)
        from glow_amd import capi
        b = {k: capi.pinned_copy(v) for k, v in dlrm.bindings(net, inp, max_idx).items()}
        prob = capi.pinned_empty((batch, 1), np.float32)
        dm.run("main", dict(b, prob=prob))
        reps = max(5, args.steps // 4)
        ms = dm.time_function("main", reps)
        t1 = time.perf_counter()
        for _ in range(3):
            dm.run("main", dict(b, prob=prob))
        e2e = (time.perf_counter() - t1) / 3
    finally:
        dm.stop()
    lookups = int(sum(int(l.sum()) for l in inp.lengths))
    sls_bytes = lookups * (36 + 8) + tables * batch * (4 + 64 * 2)
    return dict(workload=f"DLRM-style net, batch {batch}, {tables} tables x {args.dlrm_rows} rows x 64 "
                         "(4-bit fused, fp16 scale/offset), Poisson(20) bags, Zipf(1.1) int64 indices",
                samples_per_s=batch / (ms * 1e-3), ms_per_batch=ms,
                samples_per_s_with_host_copies=batch / e2e,
                lookups_per_batch=lookups, sls_algorithmic_mb_per_batch=sls_bytes / 1e6,
                launches_per_batch=len([r for r in H.parse_listing(m.describe(f))
                                        if r["phase"] == "launch"]),
                prob_mean=float(prob.mean()), host_build_seconds=t_build)


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one MI355X; multi-GPU runs are not part of "
              "this build (the path shards by bags with no exchange). "
              "Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    from glow_amd import capi
    from glow_amd import workloads as cases

    if args.only == "resnet50":
        print(json.dumps(bench_resnet50(args)))
        return
    if args.only == "dlrm":
        print(json.dumps(bench_dlrm(args)))
        return

    capi.init(0)
    info = capi.device_info()
    extra = {}
    only = args.only
    if args.tile >= 0:
        capi.check(capi.lib().mi355x_gemm_tile_override(args.tile))

    if only in ("fc_large", "fc_large_zero", "fc_c1", "fc_m16384", "fc_mid", "conv_c3", "quantize",
                "dequantize", "rescale", "copy"):
        if only == "fc_large":
            r = bench_fc(capi, cases, 8192, 4096, 4096, args.steps, args.warmup)
        elif only == "fc_large_zero":
            r = bench_fc(capi, cases, 8192, 4096, 4096, args.steps, args.warmup, zero_leg=True)
        elif only == "fc_c1":
            r = bench_fc(capi, cases, 128, 1024, 1024, args.steps, args.warmup)
        elif only == "fc_m16384":
            r = bench_fc(capi, cases, 16384, 1024, 1024, args.steps, args.warmup)
        elif only == "fc_mid":
            # a 3x3 convolution of ResNet-50's 14x14 stage as a plain product:
            # 196 workgroups of 128x128, fewer than the part has CUs
            r = bench_fc(capi, cases, 12544, 2304, 256, args.steps, args.warmup)
        elif only == "conv_c3":
            r = bench_conv(capi, cases, args.steps, args.warmup)
        else:
            r = bench_elementwise(capi, only, args.steps, args.warmup)
        print(json.dumps(r))
        return

    rng = np.random.default_rng(42)
    table = cases.random_fused_table(rng, args.rows, 128)
    d_table = capi.to_device(table)
    s = bench_slws(capi, cases, args, table, d_table)
    gbps = s["bytes"] / s["sec"] / 1e9

    # CPU leg: baseline timing, and the check of the last timed step's output
    last = s["batches"][(args.warmup + args.steps - 1) % len(s["batches"])]
    cpu, parity = None, None
    if not only and args.cpu_seconds > 0:
        cpu, parity = cpu_baseline_slws(table, s["batches"], args.cpu_seconds,
                                        s["d_out"].numpy(), last)

    if not args.no_extra and not only:
        st, wu = max(20, args.steps // 4), max(3, args.warmup // 4)
        extra["slws_with_h2d"] = bench_slws_with_h2d(capi, s, args, d_table)
        extra["slws_more_bags"] = [bench_slws_more_bags(capi, cases, args, d_table, n)
                                   for n in (16384, 65536)]
        if args.cpu_seconds > 0:
            extra["cpu_all_cores"] = cpu_all_cores_slws(table, s["batches"],
                                                        args.cpu_seconds / 2)
            extra["cpu_mfma_kernels"] = cpu_baseline_mfma_kernels(args.cpu_seconds / 2)
        extra["rwq_fc_c1"] = bench_fc(capi, cases, 128, 1024, 1024, args.steps, args.warmup)
        # enough launches for the clock to settle under the power limit
        extra["rwq_fc_large"] = bench_fc(capi, cases, 8192, 4096, 4096, max(st, 300), max(wu, 30),
                                             zero_leg=True)
        # the single-FC configuration's own K and N at a large batch
        extra["rwq_fc_m16384"] = bench_fc(capi, cases, 16384, 1024, 1024, max(st, 300),
                                          max(wu, 30))
        extra["cwq_conv_c3"] = bench_conv(capi, cases, args.steps, args.warmup)
        for w in ("quantize", "dequantize", "rescale"):
            extra[w] = bench_elementwise(capi, w, st, wu)
        extra["resnet50_int8"] = bench_resnet50(args)
        extra["dlrm_int8"] = bench_dlrm(args)

    out = {
        "metric": "FusedRowwiseQuantizedSLWS algorithmic GB/s (1 GPU)",
        "value": gbps,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": s["sec"] * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8->f32",
        "data": "synthetic",
        "config": {
            "workload": "FusedRowwiseQuantizedSparseLengthsWeightedSum, uint8 "
                        f"fused-rowwise table {args.rows} x 128 (136-byte rows), "
                        f"{args.bags} bags Poisson(40), Zipf(1.05) int64 indices, fp32 "
                        "weights, fp32 out",
            "index_batches_cycled": args.batches,
            "mean_lookups_per_step": s["mean_lookups"],
            "bytes_per_step": s["bytes"],
            "device": info.name.decode() or "MI355X", "arch": info.arch.decode(),
            "compute_units": info.compute_units,
        },
        "parity_with_oracle": (None if parity is None else bool(parity <= 1e-5)),
        "max_error_over_bag_magnitude": parity,
        "roofline": {"bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS,
                     "traffic": (MEASURED_TRAFFIC["slws"]
                                 if (args.rows, args.bags, args.batches) ==
                                 (4_000_000, 4096, 8) else None),
                     "kernel": "slws_rows_kernel<false,false,32,true>"},
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(out))
    if parity is not None and not parity <= 1e-5:
        sys.exit(1)


if __name__ == "__main__":
    main()

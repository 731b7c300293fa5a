"""Benchmark of the MI355X quantized-inference hot path on ONE GPU.

Headline workload (one step = one pass of the hot path over one batch):
FusedRowwiseQuantizedSparseLengthsWeightedSum over a uint8 fused-rowwise table
of 4M rows x 128 dims (fp32 scale and offset per row, 136-byte rows, 544 MB),
4096 bags with Poisson(40) lengths, Zipf(1.05) int64 indices, fp32 weights
U[0,1), fp32 output [4096 x 128]. Throughput is counted the way the
reference's SLS benchmark counts bytes (tests/benchmark/CommonSLSEB.h:120-176:
every lookup moves its row, scale and offset, index and weight; plus lengths
and output; no credit for cache hits).

The timed steps cycle through 64 distinct index batches (about 22 MB of table
rows each, 1.4 GB in all) and the caches are flushed with a 1 GiB copy between
the untimed and the timed replay, so the rows a step reads come from HBM and
not from the 256 MB last-level cache; the rows that Zipf makes hot stay hot
across steps, as they would in service.

Prints ONE JSON line. Besides the headline it reports, under "extra", the
same lookup with a cache-resident working set and with the strict (bit-exact)
arithmetic, the int8 matrix-core kernels (RowwiseQuantizedFullyConnected at
the single-FC configuration and at a large shape,
ChannelwiseQuantizedConvolution at the ResNet-50 3x3x64 layer shape) and the
elementwise kernels, each with its own roofline fraction and a comparison of
a sample of its output with the CPU oracle, the two networks, and times the
CPU oracle on this host's cores.

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
MEASURED_TRAFFIC = {"slws": 24.00e6, "fc_large": 236.0e6, "conv_c3": 19.63e6}

HBM_PEAK_GBPS = 8000.0       # MI355X HBM3E, published
INT8_PEAK_TOPS = 5000.0      # MI355X dense int8 MFMA, published (5.0 POP/s)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batches", type=int, default=64,
                    help="distinct index batches cycled through by the steps")
    ap.add_argument("--rows", type=int, default=4_000_000)
    ap.add_argument("--bags", type=int, default=4096,
                    help="bags per step (4096 is the headline configuration)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0,
                    help="wall-clock budget of the CPU baseline leg")
    ap.add_argument("--cpu-threads", type=int, default=16,
                    help="threads of the all-cores CPU leg: the CPU share of a one-GPU job "
                         "on the benchmark host (capped by the cores this process may use)")
    ap.add_argument("--net-replays", type=int, default=30,
                    help="timed replays of the two networks (at least 20)")
    ap.add_argument("--resnet-batch", type=int, default=64)
    ap.add_argument("--resnet-profile-images", type=int, default=100)
    ap.add_argument("--resnet-chains", type=int, default=1,
                    help="compute the ResNet-50 batch as this many independent instruction "
                         "chains over equal slices of it (constants shared)")
    ap.add_argument("--dlrm-rows", type=int, default=1_000_000)
    ap.add_argument("--no-extra", action="store_true",
                    help="headline workload only")
    ap.add_argument("--only", default="",
                    help="run a single extra kernel (profiling aid): "
                         "slws|slws_warm|slws_strict|slws_probe|fc_large|fc_large_zero|fc_c1|fc_m16384|fc_mid|"
                         "fc_split_k|"
                         "fc|conv_c3|quantize|dequantize|rescale|copy|resnet50|dlrm")
    ap.add_argument("--shape", default="",
                    help="MxKxN of --only fc (a RowwiseQuantizedFullyConnected of that shape)")
    ap.add_argument("--hint", action="store_true",
                    help="--only fc: run with the requantisation hint the backend derives "
                         "from the launch's constants")
    ap.add_argument("--tile", type=int, default=-1,
                    help="force a workgroup tile for the matrix-core legs of --only "
                         "(0..5, see mi355x_gemm_tile_override; default: chosen from the shape)")
    return ap.parse_args()


DIRECT_MAX_STEPS = 64   # launches the host surely queues while a cache flush runs


def timed_launches(capi, fn, steps, warmup, flush=None, during=None, lanes=1):
    """Average seconds per launch. `fn(i, stream)` issues launch i. After
    `warmup` eager launches, the `steps` timed launches are recorded into one
    launch graph and replayed (or, behind a cache flush and up to
    DIRECT_MAX_STEPS of them, queued directly while the flush runs), so the
    figure is the device-side rate and not the host's enqueue rate (a Python ->
    ctypes -> HIP launch costs 4-6 us, more than some of these kernels take). HIP events bracket the replay on
    the stream it runs on, with the device idle before and after.
    `flush(stream)` runs between the untimed and the timed replay (cache
    flush, queued directly in front of the timed region); `during()` is called
    while the timed replay runs (it may queue work
    on other streams) and its result is returned beside the time.
    lanes > 1: the recorded launches are dealt round-robin onto that many
    streams that fork from and join the recording stream, so launch i need
    not wait for launch i - 1 (independent requests in flight together, what
    the reference's benchmarks call asyncLaunchSize); fn then gets the lane as
    a third argument and must keep the lanes' outputs apart."""
    stream = capi.Stream()
    for i in range(warmup):
        fn(i, stream) if lanes == 1 else fn(i, stream, 0)
    stream.sync()
    if flush is not None and lanes == 1 and during is None and steps <= DIRECT_MAX_STEPS:
        # Behind a flush a short run needs no graph: the flush keeps the stream
        # busy for several hundred microseconds, the host queues the K launches
        # behind it meanwhile (5 us each), and the device then finds them back
        # to back. A replay has a start-up of ~11 us of its own whatever it
        # holds, which at K = 20 would be 0.5 us on every step. (Without a
        # flush the replay stays: launches of a few microseconds queued one by
        # one leave wider gaps than the nodes of a graph, measured.)
        capi.sync()
        e0, e1 = capi.Event(), capi.Event()
        flush(stream)
        e0.record(stream)
        for i in range(steps):
            fn(warmup + i, stream)
        e1.record(stream)
        e1.sync()
        capi.sync()
        return e0.elapsed_ms(e1) * 1e-3 / steps
    side = [capi.Stream() for _ in range(lanes - 1)]
    with capi.Graph(stream) as graph:
        if lanes == 1:
            for i in range(steps):
                fn(warmup + i, stream)
        else:
            events = [capi.Event() for _ in range(lanes)]   # alive until the capture ends
            events[0].record(stream)
            for s in side:
                s.wait_event(events[0])
            for i in range(steps):
                fn(warmup + i, ([stream] + side)[i % lanes], i % lanes)
            for s, done in zip(side, events[1:]):
                done.record(s)
                stream.wait_event(done)
    graph.launch()          # untimed first replay (uploads the graph)
    stream.sync()
    capi.sync()
    e0, e1 = capi.Event(), capi.Event()
    # The flush (a 1 GiB copy, several hundred microseconds) is queued in front
    # of the first event and not waited for: while it runs the host submits the
    # events and the graph, so the timed region holds the K launches and not
    # the host's submission of them (some 30 us, 1.5 us per step at K = 20).
    if flush is not None:
        flush(stream)
    e0.record(stream)
    graph.launch()
    e1.record(stream)
    seen = during() if during is not None else None
    e1.sync()
    capi.sync()
    sec = e0.elapsed_ms(e1) * 1e-3 / steps
    graph.destroy()
    return (sec, seen) if during is not None else sec


class CacheFlush:
    """A 1 GiB device copy: four times the 256 MB last-level cache, so whatever
    earlier launches left in the caches is gone when it ends."""

    def __init__(self, capi, nbytes=1 << 30):
        self.capi, self.n = capi, nbytes
        self.src = capi.DeviceBuffer.empty((nbytes,), np.uint8)
        self.dst = capi.DeviceBuffer.empty((nbytes,), np.uint8)
        self.src.fill(1)
        capi.sync()

    def __call__(self, stream):
        self.capi.launch_copy_u8(self.dst, self.src, self.n, stream)


class ClockProbe:
    """`probes` clock probes of `micros` us each on a stream of their own:
    launch() queues them (nothing in it waits for the device, so it can be
    called while other work runs), result() gives the shader clock each saw."""

    def __init__(self, capi, micros=200, probes=24):
        import ctypes as C
        self.capi, self.micros, self.probes = capi, micros, probes
        self.stream = capi.Stream()
        self.out = capi.DeviceBuffer.empty((probes, 2), np.uint64)
        self.out.fill(0)
        khz = C.c_int(0)
        capi.check(capi.lib().mi355x_wall_clock_khz(C.byref(khz)))
        self.khz = khz.value
        capi.sync()

    def launch(self):
        import ctypes as C
        for i in range(self.probes):
            self.capi.check(self.capi.lib().mi355x_shader_clock_probe(
                C.c_void_p(self.out.ptr + 16 * i), C.c_uint32(self.micros),
                C.c_void_p(self.stream.ptr)))
        return self

    def result(self):
        self.stream.sync()
        v = self.out.numpy().astype(np.float64)
        ok = v[:, 1] > 0
        if not ok.any():
            return None
        mhz = v[ok, 0] / v[ok, 1] * self.khz / 1e3
        return dict(median=float(np.median(mhz)), min=float(mhz.min()), max=float(mhz.max()),
                    probes=int(ok.sum()), probe_us=self.micros)


def slws_bytes(total_lookups, bags, cols, row_bytes):
    """Algorithmic bytes of one launch (reference CommonSLSEB.h:120-176)."""
    return total_lookups * (row_bytes + 8 + 4) + bags * 4 + bags * cols * 4


def make_slws_batches(capi, cases, args, count):
    batches = []
    for b in range(count):
        lengths, idx, w = cases.slws_batch(1000 + b, args.rows, args.bags, 40, 1.05, np.int64)
        batches.append(dict(
            lengths=lengths, idx=idx, w=w, total=int(lengths.sum()),
            d_len=capi.to_device(lengths), d_idx=capi.to_device(idx),
            d_w=capi.to_device(w),
            d_off=capi.to_device(capi.slws_bag_offsets_host(lengths))))
    return batches


def bench_slws(capi, args, d_table, batches, flush, bag_offsets=False, probe_stage=None, lanes=1):
    """Times args.steps launches that cycle through `batches`; `flush` (or None)
    empties the caches before the timed replay. bag_offsets: the bags as the
    positions a device manager derives from the lengths on the host
    (mi355x_frwq_slws_offsets) instead of the lengths themselves. probe_stage:
    the launch cut off behind that stage (mi355x_frwq_slws_probe)."""
    import ctypes as C
    rows, cols, bags = args.rows, 128, args.bags
    row_bytes = cols + 8
    d_outs = [capi.DeviceBuffer.empty((bags, cols), np.float32) for _ in range(lanes)]

    def step(i, stream, lane=0):
        b = batches[i % len(batches)]
        d_out = d_outs[lane]
        if probe_stage is not None:
            capi.check(capi.lib().mi355x_frwq_slws_probe(
                C.c_int(probe_stage), C.c_void_p(d_out.ptr), C.c_void_p(d_table.ptr),
                C.c_size_t(rows), C.c_void_p(b["d_w"].ptr), C.c_void_p(b["d_idx"].ptr),
                C.c_size_t(b["total"]), C.c_void_p(b["d_len"].ptr), C.c_size_t(bags),
                C.c_size_t(row_bytes), C.c_void_p(stream.ptr)))
            return
        if bag_offsets:
            capi.launch_frwq_slws_offsets(d_out, False, d_table, rows, capi.FUSED_U8_F32,
                                          b["d_w"], False, b["d_idx"], True, b["total"],
                                          b["d_off"], bags, row_bytes, cols, stream=stream)
            return
        capi.launch_frwq_slws(d_out, False, d_table, rows, capi.FUSED_U8_F32,
                              b["d_w"], False, b["d_idx"], True, b["total"],
                              b["d_len"], bags, row_bytes, cols, stream=stream)

    sec = timed_launches(capi, step, args.steps, args.warmup, flush=flush, lanes=lanes)
    d_out = d_outs[(args.steps - 1) % lanes]    # the last timed step's output
    mean_total = float(np.mean([batches[(args.warmup + i) % len(batches)]["total"]
                                for i in range(args.steps)]))
    nbytes = slws_bytes(mean_total, bags, cols, row_bytes)
    last = batches[(args.warmup + args.steps - 1) % len(batches)]
    return dict(sec=sec, bytes=nbytes, batches=batches, mean_lookups=mean_total,
                d_out=d_out, last=last)


def slws_errors(got, want, table, b):
    """(max error over the magnitude a bag adds up, max element-wise relative
    error over the outputs with |want| >= 1, share of outputs above that floor)."""
    from glow_amd import workloads
    ratio = workloads.slws_error_ratio(got, want, table, b["w"], b["idx"], b["lengths"])
    big = np.abs(want) >= 1.0
    rel = float(np.max(np.abs(got[big].astype(np.float64) - want[big]) / np.abs(want[big]))) \
        if big.any() else 0.0
    return ratio, rel, float(big.mean())


def slws_stage_probe(capi, args, d_table, batches, flush, s):
    """The headline launch cut off behind each of its dependent stages, same
    grid, same batches, same flush: what the decomposition costs before any
    arithmetic. `s` is the headline's own bench_slws result."""
    stages = ("empty launch", "bag positions (prefix over the lengths)",
              "index and weight of every lookup", "scale and offset of every row",
              "every row read, no arithmetic")
    probe = [bench_slws(capi, args, d_table, batches, flush, probe_stage=k)["sec"] * 1e6
             for k in range(len(stages))]
    return dict(
        workload="headline launch cut off behind a stage (mi355x_frwq_slws_probe), "
                 "cumulative microseconds per launch",
        stages={name: round(us, 3) for name, us in zip(stages, probe)},
        floor_us=probe[-1],
        floor_frac_of_hbm_peak=s["bytes"] / (probe[-1] * 1e-6) / 1e9 / HBM_PEAK_GBPS,
        headline_us=s["sec"] * 1e6)


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


def bench_slws_more_bags(capi, cases, args, d_table, bags, flush):
    """The headline lookup on the same table with a larger batch: the part of a
    launch that does not shrink with the batch (dispatch, bag offsets, the
    index -> row dependent round trips) is spread over more bytes. Enough
    distinct batches are cycled that their rows exceed the last-level cache
    twice over, and the caches are flushed before the timed replay."""
    rows, cols = args.rows, 128
    count = max(2, int(np.ceil(600e6 / (bags * 40 * 136.0))))
    bs = []
    for k in range(count):
        lengths, idx, w = cases.slws_batch(2000 + bags + k, rows, bags, 40, 1.05, np.int64)
        bs.append((int(lengths.sum()), capi.to_device(lengths), capi.to_device(idx),
                   capi.to_device(w)))
    d_out = capi.DeviceBuffer.empty((bags, cols), np.float32)

    def step(i, stream):
        total, d_len, d_idx, d_w = bs[i % count]
        capi.launch_frwq_slws(d_out, False, d_table, rows, capi.FUSED_U8_F32, d_w, False, d_idx,
                              True, total, d_len, bags, cols + 8, cols, stream=stream)

    steps, warmup = max(20, args.steps // 4), max(3, args.warmup // 4)
    sec = timed_launches(capi, step, steps, warmup, flush=flush)
    total = float(np.mean([bs[(warmup + i) % count][0] for i in range(steps)]))
    nbytes = slws_bytes(total, bags, cols, cols + 8)
    return dict(workload=f"SLWS, same table, {bags} bags ({total:.0f} lookups), {count} batches cycled",
                ms=sec * 1e3, gbps=nbytes / sec / 1e9,
                frac_of_hbm_peak=nbytes / sec / 1e9 / HBM_PEAK_GBPS)


def cpu_all_cores_slws(table, batches, budget_s, threads):
    """The oracle on the host cores of this job, one whole batch per thread at a
    time (the reference's CPU backend exposes one device per hardware thread,
    lib/Backends/CPU/CPUBackend.cpp:114-116). `threads` is the job's CPU share
    (16 for a one-GPU job on the benchmark host, whatever the machine has),
    capped by the cores this process may run on."""
    import threading
    from oracle import glow_oracle as go
    avail = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else os.cpu_count()
    cores = max(1, min(avail, threads))
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
                cores_visible=avail,
                sample=f"whole batches for {el:.1f} s, one batch per thread at a time")


def cpu_baseline_slws(table, batches, budget_s, native):
    """The CPU leg: the oracle (the restated libjit loop, one thread) over
    whole batches of the same workload until the time budget is used."""
    from oracle import glow_oracle as go
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
    build = "-O3 -march=native, built on this host" if native else "-O3, portable build"
    return dict(value=done_bytes / el / 1e9, unit="GB/s", cores=1, kind="port",
                sample=f"{n} full batches of {batches[0]['lengths'].size} bags (single thread, "
                       f"{el:.1f} s) of the same table and index batches; oracle compiled {build}")


def cpu_reference_libjit_slws(table, batches, budget_s):
    """The reference's own libjit (its sources compiled unmodified, with the
    reference's default -ffast-math flags, -O2, portable code) on the same
    batches, one thread; None where that library has not been built."""
    from oracle import libjit_ref
    if not libjit_ref.available(fastmath=True):
        return None
    done_bytes, n = 0.0, 0
    t0 = time.perf_counter()
    while True:
        b = batches[n % len(batches)]
        libjit_ref.frwq_slws_f32(table, b["w"], b["idx"], b["lengths"], fastmath=True)
        done_bytes += slws_bytes(b["total"], b["lengths"].size, 128, 136)
        n += 1
        el = time.perf_counter() - t0
        if el >= budget_s or n >= 4000:
            break
    return dict(value=done_bytes / el / 1e9, unit="GB/s", cores=1, kind="reference",
                sample=f"{n} full batches (single thread, {el:.1f} s); libjit.cpp compiled "
                       "-O2 -ffast-math -fno-finite-math-only for generic x86-64")


def oracle_rows_check(capi, c, d_out, M, rows):
    """Rows `rows` of the device result against the oracle run on those rows."""
    from oracle import glow_oracle as go
    got = d_out.numpy()
    cs = dict(c, x=np.ascontiguousarray(c["x"][rows]))
    want = go.rwq_fc_i8(cs["x"], c["w"], c["bias"], c["w_offsets"], c["bias_pre"],
                        c["bias_post"], c["bias_scale"], c["out_pre"], c["out_post"],
                        c["out_scale"], c["out_offset"], c["in_offset"], c["bias_offset"])
    return bool(np.array_equal(got[rows], want)), int(len(rows))


def bench_fc(capi, cases, M, K, N, steps, warmup, seed=5, zero_leg=False, check=True,
             clock=False, use_hint=False, split_k=False):
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

    opts = None
    if split_k:
        # a zero-filled workspace with the call: the library may split the K loop
        # over workgroups (it does when the grid would leave half the CUs idle)
        ws = capi.DeviceBuffer(max(256, capi.gemm_splitk_workspace_bytes(M, N, K)))
        ws.fill(0)
        opts = capi.LaunchOpts(workspace=ws)

    def step(_, stream):
        capi.launch_rwq_fc_i8(d_out, d["x"], d["w"], d["bias"], False,
                              d["w_offsets"], d["bias_pre"], d["bias_post"],
                              d["bias_scale"], d["out_pre"], d["out_post"],
                              d["out_scale"], M, K, N, c["out_offset"],
                              c["in_offset"], c["bias_offset"], True,
                              w_row_sums=d_sums, stream=stream, opts=opts)

    hint = 0
    if use_hint:
        # as the backend compiles it: the requantisation hints derived from the
        # launch's constants (host-verified bounds)
        hint = capi.gemm_requant_hint_host(K, c["in_offset"], c["out_offset"], c["w_offsets"],
                                           c["bias"], c["bias_offset"], c["bias_pre"],
                                           c["bias_post"], c["bias_scale"], c["out_pre"],
                                           c["out_post"], c["out_scale"])
        capi.check(capi.lib().mi355x_gemm_requant_hint(hint))
    clocks = None
    if clock:
        # the shader clock the part holds while this kernel runs, sampled from
        # a second stream during the timed replay, and the clock of the idle part
        idle = ClockProbe(capi).launch().result()
        probe = ClockProbe(capi)
        sec, _ = timed_launches(capi, step, steps, warmup, during=probe.launch)
        clocks = dict(during_timed_launches_mhz=probe.result(), idle_mhz=idle)
    else:
        sec = timed_launches(capi, step, steps, warmup)
    ops = 2.0 * M * N * K
    parity = None
    if check:
        # the oracle on a row sample of what the timed launches left behind
        step_rows = max(1, M // 24)
        rows = np.unique(np.r_[0:min(M, 8), np.arange(0, M, step_rows), M - 1])[:40]
        parity = oracle_rows_check(capi, c, d_out, M, rows)
    zero = None
    if zero_leg:
        # The same launch on all-zero operands: identical instruction stream,
        # but the matrix cores toggle no data, so the part holds a higher clock
        # under its power limit. The ratio shows how much of the distance to
        # the published peak is clock, not kernel.
        d["x"].fill(0)
        d["w"].fill(0)
        capi.sync()
        if clock:
            probe = ClockProbe(capi)
            zsec, _ = timed_launches(capi, step, steps, warmup, during=probe.launch)
            clocks["zero_operands_mhz"] = probe.result()
        else:
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
    if use_hint:
        capi.check(capi.lib().mi355x_gemm_requant_hint(0))
    return dict(workload=f"rwq_fc M{M} K{K} N{N}", requant_hint=hint, ms=sec * 1e3,
                tops=ops / sec / 1e12, zero_operands=zero, normal_weights=normal,
                shader_clock=clocks,
                parity_with_oracle=(None if parity is None else parity[0]),
                rows_checked=(None if parity is None else parity[1]),
                roofline=dict(bound="mfma", achieved=ops / sec / 1e12,
                              peak=INT8_PEAK_TOPS, unit="TOP/s",
                              frac=ops / sec / 1e12 / INT8_PEAK_TOPS,
                              traffic=(MEASURED_TRAFFIC["fc_large"]
                                       if (M, K, N) == (8192, 4096, 4096) else None)),
                gbps=(M * K + N * K + M * N + 8 * 4 * N) / sec / 1e9)


def bench_conv(capi, cases, steps, warmup, check=True):
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

    sec_plain = timed_launches(capi, step, steps, warmup)
    # as the backend compiles it: the requantisation hints it derives for this
    # launch from the constants (host-verified bounds), in force while timed
    hint = capi.gemm_requant_hint_host(
        g.KH * g.KW * g.IC, c["in_offset"], c["out_offset"], c["f_offsets"], c["bias"], 0,
        c["bias_pre"], c["bias_post"], c["bias_scale"], c["out_pre"], c["out_post"],
        c["out_scale"], bias_offsets=c["b_offsets"])
    d_out.fill(0)
    with capi.requant_hint(hint):
        sec = timed_launches(capi, step, steps, warmup)
    parity = None
    if check:
        # images 0 and 31 of what the timed launches left behind, on the oracle
        from oracle import glow_oracle as go
        got = d_out.numpy()
        pick = [0, g.N - 1]
        c2 = dict(c, x=np.ascontiguousarray(c["x"][pick]),
                  geom=go.conv_geom(len(pick), g.IH, g.IW, g.IC, g.OC, (g.KH, g.KW),
                                    (g.strideH, g.strideW), (g.padT, g.padL, g.padT, g.padL)))
        want = go.cwq_conv2d_i8(*cases.cwq_conv_args(c2))
        parity = bool(np.array_equal(got[pick], want))
    ops = 2.0 * g.N * g.OH * g.OW * g.OC * g.KH * g.KW * g.IC
    nbytes = c["x"].size + d_out.nbytes + c["filt"].size + 9 * 4 * g.OC
    return dict(workload="cwq_conv2d 32x56x56x64 3x3x64->64 s1 p1 relu",
                ms=sec * 1e3, tops=ops / sec / 1e12, gbps=nbytes / sec / 1e9,
                requant_hint=int(hint), ms_without_hint=sec_plain * 1e3,
                parity_with_oracle=parity, images_checked=(2 if check else None),
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
        # the parameters of a rescale between scales 0.05 and 0.07
        # (quantizeScaleOffset32To8(0.714) = {pre 0, post 9, scale 366}; a
        # pre-shift only appears for ratios below 2^-7)
        fn = lambda _, st: capi.launch_rescale_i8(dst, src, n, 3, -5, 0, 9, 366, st)
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


def bench_resnet50(args, check=True):
    """Int8 ResNet-50 at batch 64, 224x224 through MI355XDeviceManager:
    images/s of the resident network replayed on device-resident input
    (device time), and of whole requests including the fp32 input upload and
    the result download. The first and the last image of the batch are run
    through the oracle executing the same quantized graph."""
    from glow_amd import host as H
    from glow_amd.harness import net as netlib
    from glow_amd.harness import resnet50
    batch, size = args.resnet_batch, 224
    t0 = time.perf_counter()
    steps = resnet50.build_fp32(0)
    ranges = resnet50.profile(steps, resnet50.synthetic_images(1, args.resnet_profile_images, size))
    net = resnet50.build_int8(steps, ranges, batch, size, chains=args.resnet_chains)
    t_build = time.perf_counter() - t0
    m, f = netlib.to_module(net)
    m.compile(f)
    dm = H.DeviceManager().init()
    reps = max(20, args.net_replays)
    try:
        dm.add_network(m)
        # request buffers in pinned host memory (allocateDeviceIOBuffer)
        from glow_amd import capi
        x = capi.pinned_copy(resnet50.synthetic_images(77, batch, size))
        prob = capi.pinned_empty((batch, 1000), np.float32)
        logits = capi.pinned_empty((batch, 1000), np.int8)
        dm.run("main", {"input": x, "prob": prob, "logits_q": logits})
        ms = dm.time_function("main", reps)
        t1 = time.perf_counter()
        for _ in range(3):
            dm.run("main", {"input": x, "prob": prob, "logits_q": logits})
        e2e = (time.perf_counter() - t1) / 3
    finally:
        dm.stop()
    parity = None
    if check:
        from tests import oracle_exec
        pick = [0, batch - 1]
        two = resnet50.build_int8(steps, ranges, len(pick), size)
        want = oracle_exec.run(two, {"input": np.ascontiguousarray(np.asarray(x)[pick])})
        parity = bool(np.array_equal(np.asarray(logits)[pick], want["logits_q"]) and
                      np.allclose(np.asarray(prob)[pick], want["prob"], rtol=1e-5, atol=1e-30))
    ops = net.ops_count()
    return dict(workload=f"int8 ResNet-50, batch {batch}, {size}x{size}x3, channelwise-quantized "
                         f"convolutions, rowwise-quantized FC, fp32 softmax; "
                         f"{args.resnet_profile_images} profiling images",
                images_per_s=batch / (ms * 1e-3), ms_per_batch=ms, timed_replays=reps,
                images_per_s_with_host_copies=batch / e2e,
                tops=ops / (ms * 1e-3) / 1e12, gop_per_image=ops / batch / 1e9,
                launches_per_batch=len([r for r in H.parse_listing(m.describe(f))
                                        if r["phase"] == "launch"]),
                parity_with_oracle=parity, images_checked=(2 if check else None),
                prob_row_sum=float(prob[0].sum()), host_build_seconds=t_build)


def bench_dlrm(args, check=True):
    """DLRM-style ranking net, batch 4096: 26 tables of 1M x 64 (4-bit fused,
    fp16 scale/offset), Poisson(20) bags of Zipf(1.1) int64 indices, int8 MLPs
    13-512-256-64 and 415-512-256-1, dot interaction, sigmoid. The whole batch
    is run through the oracle executing the same quantized graph; the lookups
    run the library's default (fused multiply-add) arithmetic, which may move
    an int8 logit by one quantization step against the sequential CPU sum."""
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
    reps = max(20, args.net_replays)
    try:
        dm.add_network(m)
        inp = dlrm.Inputs(99, tables, args.dlrm_rows, batch, 20, 1.1, 13)
        from glow_amd import capi
        hb = dlrm.bindings(net, inp, max_idx)
        b = {k: capi.pinned_copy(v) for k, v in hb.items()}
        prob = capi.pinned_empty((batch, 1), np.float32)
        logit = capi.pinned_empty((batch, 1), np.int8)
        dm.run("main", dict(b, prob=prob, logit_q=logit))
        ms = dm.time_function("main", reps)
        t1 = time.perf_counter()
        for _ in range(3):
            dm.run("main", dict(b, prob=prob, logit_q=logit))
        e2e = (time.perf_counter() - t1) / 3
    finally:
        dm.stop()
    parity, off_by_one = None, None
    if check:
        from tests import oracle_exec
        want = oracle_exec.run(net, hb)
        d = np.abs(np.asarray(logit).astype(np.int32) - want["logit_q"].astype(np.int32))
        off_by_one = int((d == 1).sum())
        parity = bool(d.max() <= 1 and (d > 0).mean() <= 0.002)
    lookups = int(sum(int(l.sum()) for l in inp.lengths))
    sls_bytes = lookups * (36 + 8) + tables * batch * (4 + 64 * 2)
    return dict(workload=f"DLRM-style net, batch {batch}, {tables} tables x {args.dlrm_rows} rows x 64 "
                         "(4-bit fused, fp16 scale/offset), Poisson(20) bags, Zipf(1.1) int64 indices",
                samples_per_s=batch / (ms * 1e-3), ms_per_batch=ms, timed_replays=reps,
                samples_per_s_with_host_copies=batch / e2e,
                lookups_per_batch=lookups, sls_algorithmic_mb_per_batch=sls_bytes / 1e6,
                launches_per_batch=len([r for r in H.parse_listing(m.describe(f))
                                        if r["phase"] == "launch"]),
                parity_with_oracle=parity, logits_one_step_off=off_by_one,
                samples_checked=(batch if check else None),
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

    if only and only not in ("slws", "slws_warm", "slws_strict", "slws_probe", "fc", "fc_large", "fc_large_zero",
                             "fc_c1", "fc_m16384", "fc_mid", "fc_split_k", "conv_c3", "quantize",
                             "dequantize", "rescale", "copy"):
        print(f"unknown --only {only}", file=sys.stderr)
        sys.exit(2)
    if only in ("fc", "fc_large", "fc_large_zero", "fc_c1", "fc_m16384", "fc_mid", "fc_split_k", "conv_c3",
                "quantize", "dequantize", "rescale", "copy"):
        if only == "fc":
            M, K, N = (int(v) for v in args.shape.split("x"))
            r = bench_fc(capi, cases, M, K, N, args.steps, args.warmup, use_hint=args.hint)
        elif only == "fc_large":
            r = bench_fc(capi, cases, 8192, 4096, 4096, args.steps, args.warmup)
        elif only == "fc_large_zero":
            r = bench_fc(capi, cases, 8192, 4096, 4096, args.steps, args.warmup, zero_leg=True,
                         clock=True)
        elif only == "fc_c1":
            r = bench_fc(capi, cases, 128, 1024, 1024, args.steps, args.warmup)
        elif only == "fc_m16384":
            r = bench_fc(capi, cases, 16384, 1024, 1024, args.steps, args.warmup)
        elif only == "fc_mid":
            # a 3x3 convolution of ResNet-50's 14x14 stage as a plain product:
            # 196 workgroups of 128x128, fewer than the part has CUs
            r = bench_fc(capi, cases, 12544, 2304, 256, args.steps, args.warmup)
        elif only == "fc_split_k":
            # few output tiles and a long K: the K loop split over workgroups
            # through a caller's workspace
            r = bench_fc(capi, cases, 3136, 4608, 512, args.steps, args.warmup, split_k=True)
        elif only == "conv_c3":
            r = bench_conv(capi, cases, args.steps, args.warmup)
        else:
            r = bench_elementwise(capi, only, args.steps, args.warmup)
        print(json.dumps(r))
        return

    rng = np.random.default_rng(42)
    table = cases.random_fused_table(rng, args.rows, 128)
    d_table = capi.to_device(table)
    flush = CacheFlush(capi)
    batches = make_slws_batches(capi, cases, args, args.batches)

    if only == "slws_warm":
        # the cache-resident variant: 8 batches, no flush
        s = bench_slws(capi, args, d_table, batches[:8], None)
    elif only == "slws_strict":
        capi.slws_set_fused_math(capi.SLWS_MATH_STRICT)
        s = bench_slws(capi, args, d_table, batches, flush)
        capi.slws_set_fused_math(capi.SLWS_MATH_ELEMENT)
    else:
        s = bench_slws(capi, args, d_table, batches, flush)
    if only == "slws_probe":
        extra["slws_stage_probe"] = slws_stage_probe(capi, args, d_table, batches, flush, s)
    gbps = s["bytes"] / s["sec"] / 1e9

    # the check of the last timed step's output (portable build of the oracle),
    # then the CPU leg on the build for this host
    cpu, parity, rel, share = None, None, None, None
    if not only and args.cpu_seconds > 0:
        from oracle import glow_oracle as go
        want = go.frwq_slws_f32(table, s["last"]["w"], s["last"]["idx"], s["last"]["lengths"])
        parity, rel, share = slws_errors(s["d_out"].numpy(), want, table, s["last"])
        native = go.use_native_build()
        cpu = cpu_baseline_slws(table, batches, args.cpu_seconds, native)

    if not args.no_extra and not only:
        st, wu = max(20, args.steps // 4), max(3, args.warmup // 4)
        # the same launches with a working set that stays in the last-level
        # cache: 8 batches (176 MB of rows), no flush
        w8 = bench_slws(capi, args, d_table, batches[:8], None)
        extra["slws_warm"] = dict(
            workload="headline lookup, 8 index batches cycled, caches not flushed "
                     "(working set inside the 256 MB last-level cache)",
            ms=w8["sec"] * 1e3, gbps=w8["bytes"] / w8["sec"] / 1e9,
            frac_of_hbm_peak=w8["bytes"] / w8["sec"] / 1e9 / HBM_PEAK_GBPS)
        # strict arithmetic: every multiply and add rounded on its own, in bag
        # order; bit for bit the CPU loop
        capi.slws_set_fused_math(capi.SLWS_MATH_STRICT)
        try:
            ss = bench_slws(capi, args, d_table, batches, flush)
            bit_exact = None
            if args.cpu_seconds > 0:
                from oracle import glow_oracle as go
                want = go.frwq_slws_f32(table, ss["last"]["w"], ss["last"]["idx"],
                                        ss["last"]["lengths"])
                bit_exact = bool(np.array_equal(ss["d_out"].numpy(), want))
        finally:
            capi.slws_set_fused_math(capi.SLWS_MATH_ELEMENT)
        extra["slws_strict"] = dict(
            workload="headline lookup with MI355X_SLWS_MATH_STRICT",
            ms=ss["sec"] * 1e3, gbps=ss["bytes"] / ss["sec"] / 1e9,
            frac_of_hbm_peak=ss["bytes"] / ss["sec"] / 1e9 / HBM_PEAK_GBPS,
            bit_exact_with_oracle=bit_exact)
        extra["slws_stage_probe"] = slws_stage_probe(capi, args, d_table, batches, flush, s)
        # Independent requests in flight together: the same launches dealt onto 2
        # and 4 streams (each with an output of its own), so one launch's
        # dependent trips run while another's rows stream. Throughput of the
        # job, not the duration of a launch.
        extra["slws_requests_in_flight"] = []
        for lanes in (2, 4):
            sl = bench_slws(capi, args, d_table, batches, flush, lanes=lanes)
            same = None
            if args.cpu_seconds > 0:
                want = go.frwq_slws_f32(table, sl["last"]["w"], sl["last"]["idx"],
                                        sl["last"]["lengths"])
                _, rel_l, _ = slws_errors(sl["d_out"].numpy(), want, table, sl["last"])
                same = bool(rel_l <= 1e-5)
            extra["slws_requests_in_flight"].append(dict(
                workload=f"headline launches on {lanes} streams that fork from and join the "
                         "timed stream (independent batches, one output each), caches flushed",
                streams=lanes, us_per_step=sl["sec"] * 1e6, gbps=sl["bytes"] / sl["sec"] / 1e9,
                frac_of_hbm_peak=sl["bytes"] / sl["sec"] / 1e9 / HBM_PEAK_GBPS,
                parity_with_oracle=same))
        # the bags as positions (what the device manager hands over for lengths it
        # uploads itself): no prefix sum in front of a bag's first index load
        so = bench_slws(capi, args, d_table, batches, flush, bag_offsets=True)
        same = None
        if args.cpu_seconds > 0:
            # against the lengths entry point on the same (last) batch, bit for bit
            ref = capi.DeviceBuffer.empty((args.bags, 128), np.float32)
            b = so["last"]
            capi.launch_frwq_slws(ref, False, d_table, args.rows, capi.FUSED_U8_F32, b["d_w"],
                                  False, b["d_idx"], True, b["total"], b["d_len"], args.bags,
                                  136, 128)
            capi.sync()
            same = bool(np.array_equal(so["d_out"].numpy(), ref.numpy()))
        extra["slws_bag_offsets"] = dict(
            workload="headline lookup through mi355x_frwq_slws_offsets (bag positions "
                     "precomputed on the host from the lengths), same batches, caches flushed",
            ms=so["sec"] * 1e3, gbps=so["bytes"] / so["sec"] / 1e9,
            frac_of_hbm_peak=so["bytes"] / so["sec"] / 1e9 / HBM_PEAK_GBPS,
            ms_lengths_entry_point=s["sec"] * 1e3, equal_to_lengths_entry_point=same)
        extra["slws_with_h2d"] = bench_slws_with_h2d(capi, s, args, d_table)
        extra["slws_more_bags"] = [bench_slws_more_bags(capi, cases, args, d_table, n, flush)
                                   for n in (16384, 65536)]
        if args.cpu_seconds > 0:
            extra["cpu_all_cores"] = cpu_all_cores_slws(table, batches, args.cpu_seconds / 2,
                                                        args.cpu_threads)
            extra["cpu_reference_libjit"] = cpu_reference_libjit_slws(table, batches,
                                                                      args.cpu_seconds / 2)
            extra["cpu_mfma_kernels"] = cpu_baseline_mfma_kernels(args.cpu_seconds / 2)
        extra["rwq_fc_c1"] = bench_fc(capi, cases, 128, 1024, 1024, args.steps, args.warmup)
        # enough launches for the clock to settle under the power limit
        extra["rwq_fc_large"] = bench_fc(capi, cases, 8192, 4096, 4096, max(st, 300), max(wu, 30),
                                         zero_leg=True, clock=True)
        # the single-FC configuration's own K and N at a large batch
        extra["rwq_fc_m16384"] = bench_fc(capi, cases, 16384, 1024, 1024, max(st, 300),
                                          max(wu, 30))
        # few output tiles and a long K (the product of ResNet-50's 7x7 stage
        # 3x3 convolutions): as it runs by itself, and with a workspace in the
        # call's options, which lets the library split K over workgroups
        plain = bench_fc(capi, cases, 3136, 4608, 512, max(st, 100), max(wu, 10))
        split = bench_fc(capi, cases, 3136, 4608, 512, max(st, 100), max(wu, 10), split_k=True)
        extra["rwq_fc_split_k"] = dict(
            workload="rwq_fc M3136 K4608 N512 (100 tiles of 128x128)",
            ms=plain["ms"], ms_with_workspace=split["ms"],
            workspace_bytes=capi.gemm_splitk_workspace_bytes(3136, 512, 4608),
            parity_with_oracle=bool(plain["parity_with_oracle"] and split["parity_with_oracle"]))
        extra["cwq_conv_c3"] = bench_conv(capi, cases, args.steps, args.warmup)
        for w in ("quantize", "dequantize", "rescale"):
            extra[w] = bench_elementwise(capi, w, st, wu)
        del flush
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
        # the stated bar, element by element: |got - oracle| <= 1e-5 |oracle| for
        # every output at or above the floor, and the outputs below it (sums that
        # have cancelled) within 1e-5 of the magnitude their bag adds up
        "parity_with_oracle": (None if parity is None
                               else bool(rel <= 1e-5 and parity <= 1e-5)),
        "max_rel_error_elementwise": rel,
        "rel_error_floor": "outputs with |oracle value| >= 1.0",
        "share_of_outputs_above_floor": share,
        "max_error_over_bag_magnitude": parity,
        "arithmetic": "v = fma(s, q, o); acc = fma(w, v, acc) per element in bag order "
                      "(MI355X_SLWS_MATH_ELEMENT, the library's default)",
        "cache_state": ("caches flushed before the timed launches; "
                        f"{args.batches} distinct index batches cycled"),
        "roofline": {"bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS,
                     "traffic": (MEASURED_TRAFFIC["slws"]
                                 if (args.rows, args.bags, args.batches) ==
                                 (4_000_000, 4096, 64) and not only else None),
                     "traffic_source": "profiles/slws_rows_kernel__slws_u8_4Mx128_4096bags.md "
                                       "(rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not "
                                       "measured in this run)",
                     "kernel": "slws_rows_kernel<false,false,32,true,1,%d>"
                               % (16 if args.bags < 16384 else 8)},
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(out))
    if parity is not None and not (rel <= 1e-5 and parity <= 1e-5):
        sys.exit(1)


if __name__ == "__main__":
    main()

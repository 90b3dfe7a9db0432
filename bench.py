#!/usr/bin/env python3
"""Headline benchmark of the block-quantized matmul path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras]
    python bench.py --read-sweep      (a table instead: a read-only kernel over the same weight in every launch shape)
    python bench.py --grid-barrier    (a table instead: a barrier over all workgroups of a launch through device-scope atomics)

A "step" is one Q4_K GEMV (decode-path quantized matmul), weight 14336 x 4096 drawn ~N(0, 0.02) with
1 % of entries at +-0.5, activation f32[4096] ~N(0, 1), batch 1: the bandwidth headline case.  Launch i
reads copy i mod R of the weight from a ring of R copies (> 700 MB, beyond the 256 MB last-level cache),
so that every step streams its 33 MB from HBM; inputs are resident in HBM before the timed region.

Prints ONE JSON line.  `value` is whole-job throughput in algorithmic GB/s (packed weight bytes + x + y
per step, divided by the median step time of 25 event-bracketed repeats on the kernel's stream).  `roofline`
prices the dominant kernel against the 8 TB/s HBM peak; `cpu_baseline` times the CPU oracle (a C
restatement of the reference composition dequantize -> transpose -> one-thread sgemm) on this box's host
cores on the same workload.  `extra` carries the other configurations (other block types, the 7B-shape
decode, the prefill GEMM) when their code paths are built.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published
N_HEAD, K_HEAD = 14336, 4096
RING_BYTES = 700e6


def log(*a):
    print(*a, file=sys.stderr, flush=True)


RING_SEED0 = 1234  # copy i of a ring is drawn with seed RING_SEED0 + i


def make_ring(ctx, qtype, n, k, copies, outlier_p, seed0=RING_SEED0):
    """`copies` device-resident weights, generated and quantised on the device."""
    from axonml_amd._lib import MEM_DEVICE

    lib = ctx.lib
    f = ctx.malloc(n * k * 4)
    ws = []
    for i in range(copies):
        ctx.check(lib.axq_fill_normal_f32(ctx.handle, f, n * k, 0.0, 0.02, outlier_p, 0.5, seed0 + i))
        h = C.c_void_p()
        ctx.check(lib.axq_weight_quantize(ctx.handle, int(qtype), n, k, f, MEM_DEVICE, C.byref(h)))
        ws.append(h)
    ctx.free(f)
    return ws


INTERNAL_WARMUP = 200  # untimed launches before any timed one, whatever --warmup says (clocks and caches settle)
MIN_PER_REPEAT = 200   # launches between one pair of events, at least
REPEATS = 25           # timed repeats, each between its own pair of events; the median repeat is reported


def time_ring(ctx, launch, ring_len, steps, warmup):
    """launch(first, count) enqueues `count` launches that walk the ring from position `first`.  Returns (median ms
    per launch, per-repeat ms per launch, launches per repeat, untimed launches).  The timed launches are split into
    REPEATS event-bracketed repeats of steps // REPEATS launches, and of MIN_PER_REPEAT at least: the queue is empty
    when a repeat starts, and the 20 us or so until launches overlap again would otherwise weigh on a short repeat as
    if it were the kernel's time.  The ring position runs on across repeats, so no repeat starts on a copy the caches
    still hold."""
    untimed = max(INTERNAL_WARMUP, warmup)
    per = max(MIN_PER_REPEAT, steps // REPEATS)
    pos = 0
    launch(pos, untimed)
    pos += untimed
    ctx.synchronize()
    times = []
    for _ in range(REPEATS):
        ctx.timer_start()
        launch(pos % ring_len, per)
        times.append(ctx.timer_stop() / per)
        pos += per
    return float(np.median(times)), times, per, untimed


def time_gemv(ctx, ws, x_dev, y_dev, batch, steps, warmup):
    lib = ctx.lib
    arr = (C.c_void_p * len(ws))(*[w.value for w in ws])
    return time_ring(ctx, lambda first, n: ctx.check(lib.axq_bench_gemv_ring(ctx.handle, arr, len(ws), first, x_dev, batch, y_dev, n)),
                     len(ws), steps, warmup)


def time_graph(ctx, ws, x_dev, y_dev, batch, warmup_replays=2, read_sink=None):
    """The ring recorded once as a HIP graph (a whole number of trips round the ring, MIN_PER_REPEAT launches at least) and
    replayed REPEATS times, each replay between its own pair of events: the same dependent launches as time_gemv's, handed
    to the GPU in one submission, the way a decode loop replays its step.  Returns (median ms per launch, per-replay ms
    per launch, launches per replay)."""
    lib = ctx.lib
    arr = (C.c_void_p * len(ws))(*[w.value for w in ws])
    per = len(ws) * -(-MIN_PER_REPEAT // len(ws))
    g = C.c_void_p()
    if read_sink is not None:  # the read-only kernel's launches instead of the GEMV's
        ctx.check(lib.axq_bench_graph_create_read(ctx.handle, arr, len(ws), 0, read_sink, per, C.byref(g)))
    else:
        ctx.check(lib.axq_bench_graph_create(ctx.handle, arr, len(ws), 0, x_dev, batch, y_dev, per, C.byref(g)))
    try:
        ctx.check(lib.axq_bench_graph_launch(ctx.handle, g, warmup_replays))
        ctx.synchronize()
        times = []
        for _ in range(REPEATS):
            ctx.timer_start()
            ctx.check(lib.axq_bench_graph_launch(ctx.handle, g, 1))
            times.append(ctx.timer_stop() / per)
    finally:
        lib.axq_bench_graph_destroy(ctx.handle, g)
    return float(np.median(times)), times, per


def time_read(ctx, ws, sink_dev, steps, warmup):
    """The same ring under a kernel that only reads each weight's device image, on the GEMV's grid."""
    lib = ctx.lib
    arr = (C.c_void_p * len(ws))(*[w.value for w in ws])
    return time_ring(ctx, lambda first, n: ctx.check(lib.axq_bench_read_ring(ctx.handle, arr, len(ws), first, sink_dev, n)),
                     len(ws), steps, warmup)


def gemv_case(ctx, qtype, n, k, batch, steps, warmup, outlier_p=0.0, ring=True, graph=True):
    from axonml_amd import quant as q

    lib = ctx.lib
    wbytes = lib.axq_packed_bytes(int(qtype), n * k)
    copies = max(2, int(RING_BYTES // wbytes) + 1) if ring else 1
    ws = make_ring(ctx, qtype, n, k, copies, outlier_p)
    rng = np.random.default_rng(0)
    x = rng.standard_normal((batch, k)).astype(np.float32)
    x_dev = ctx.to_device(x)
    y_dev = ctx.malloc(batch * n * 4)
    ms_s, times_s, per_s, untimed = time_gemv(ctx, ws, x_dev, y_dev, batch, steps, warmup)
    ms_g, times_g, per_g = time_graph(ctx, ws, x_dev, y_dev, batch) if graph and copies > 1 else (None, None, None)
    # the figure of the case: the recorded graph when it is the faster way to hand over the same launches
    use_graph = ms_g is not None and ms_g < ms_s
    ms, times, per = (ms_g, times_g, per_g) if use_graph else (ms_s, times_s, per_s)
    algo_bytes = wbytes + 4 * batch * (n + k)
    res = {"type": str(q.QuantType(qtype)), "n": n, "k": k, "batch": batch, "us_per_step": ms * 1e3,
           "us_per_step_min_max": [min(times) * 1e3, max(times) * 1e3], "launches_per_repeat": per, "untimed_launches": untimed,
           "submission": "hipGraph replay" if use_graph else "stream launches",
           "us_per_step_stream_launches": ms_s * 1e3, "us_per_step_graph_replay": ms_g * 1e3 if ms_g is not None else None,
           "algorithmic_bytes": algo_bytes, "gbps": algo_bytes / (ms * 1e-3) / 1e9, "ring_copies": copies}
    res["frac_of_hbm_peak"] = res["gbps"] / HBM_PEAK_GBPS
    return res, ws, x, x_dev, y_dev


def free_case(ctx, ws, x_dev, y_dev):
    for h in ws:
        ctx.lib.axq_weight_free(ctx.handle, h)
    ctx.free(x_dev)
    ctx.free(y_dev)


def check_against_oracle(ctx, w_handle, qtype, n, k, x, y_dev):
    """Same-run correctness gate: packed bytes come back from the device, the oracle does the rest."""
    import oracle as o
    from axonml_amd._lib import MEM_DEVICE, MEM_HOST

    lib = ctx.lib
    nbytes = lib.axq_packed_bytes(int(qtype), n * k)
    packed = np.empty(nbytes, dtype=np.uint8)
    ctx.check(lib.axq_weight_download(ctx.handle, w_handle, packed.ctypes.data, nbytes, MEM_HOST))
    x_dev = ctx.to_device(x)
    ctx.check(lib.axq_gemv_f32(ctx.handle, w_handle, x_dev, x.shape[0], None, y_dev, MEM_DEVICE))
    got = ctx.to_host(y_dev, (x.shape[0], n), np.float32)
    ctx.free(x_dev)
    want = o.matmul_ref(int(qtype), packed, x, n, k)
    denom = np.maximum(np.abs(want), 1e-2 * np.abs(want).max())
    return float((np.abs(got - want) / denom).max()), packed


def codes_bit_exact(ctx, packed, qtype, n, k, outlier_p, seed):
    """The other half of the same-run gate (quantize.rs:82-205 restated on the device): the f32 weight the device drew
    for ring copy 0 comes back to the host, the oracle quantises it there, and every packed byte -- codes and f16
    scales -- has to equal what the device quantiser left in the weight the benchmark multiplies with."""
    import oracle as o

    f = ctx.malloc(n * k * 4)
    ctx.check(ctx.lib.axq_fill_normal_f32(ctx.handle, f, n * k, 0.0, 0.02, outlier_p, 0.5, seed))
    w = ctx.to_host(f, (n * k,), np.float32)
    ctx.free(f)
    want = o.quantize(int(qtype), w)
    return bool(want.size == packed.size and np.array_equal(want, packed))


def cpu_baseline(packed, qtype, n, k, x, budget_s=12.0):
    """Times the oracle's faithful composition (per call: dequantise all blocks, transposed copy,
    one-thread sgemm) on the host, for about `budget_s` seconds."""
    import oracle as o

    L = o.lib()
    y = np.empty((x.shape[0], n), dtype=np.float32)
    scratch = np.empty(2 * n * k, dtype=np.float32)
    args = (int(qtype), packed.ctypes.data, x.ctypes.data, None, x.shape[0], n, k, y.ctypes.data, scratch.ctypes.data)
    L.axo_matmul_ref(*args)  # warm-up (page faults of the scratch)
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 400):
        t0 = time.perf_counter()
        L.axo_matmul_ref(*args)
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    wbytes = packed.size
    algo = wbytes + 4 * x.shape[0] * (n + k)
    return {"value": algo / med / 1e9, "unit": "GB/s", "cores": int(L.axo_num_threads()), "kind": "port",
            "sample": f"{len(times)} full calls of the same {n}x{k} GEMV (median {med * 1e3:.1f} ms per call: "
                      f"block-parallel dequantise on all threads + transposed copy + single-thread f32 sgemm)",
            "ms_per_step": med * 1e3}


COPY_PROBE_BYTES = 256 << 20
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "gemv_q4k_14336x4096_hbm_counters.txt")


def counter_probe(ctx, steps):
    """Work for a `rocprofv3 --pmc FETCH_SIZE` (or WRITE_SIZE) run: the copy kernel moves a known number of
    bytes each way, which gives the factor between the counter and bytes; the GEMV launches follow."""
    from axonml_amd import quant as q

    src = ctx.malloc(COPY_PROBE_BYTES)
    dst = ctx.malloc(COPY_PROBE_BYTES)
    ctx.check(ctx.lib.axq_fill_normal_f32(ctx.handle, src, COPY_PROBE_BYTES // 4, 0.0, 1.0, 0.0, 0.0, 5))
    ctx.check(ctx.lib.axq_bench_copy(ctx.handle, dst, src, COPY_PROBE_BYTES, 8))
    ctx.synchronize()
    ctx.free(src)
    ctx.free(dst)
    _, ws, _, x_dev, y_dev = gemv_case(ctx, q.QuantType.Q4_K, N_HEAD, K_HEAD, 1, steps, 20, outlier_p=0.01)
    free_case(ctx, ws, x_dev, y_dev)
    log(f"counter probe: 8 copies of {COPY_PROBE_BYTES} B, then {steps + 20} GEMV launches")


def measured_traffic():
    """HBM bytes per GEMV launch from the committed counter summary (a line `traffic_bytes_per_launch: N`),
    or None when no summary is there."""
    try:
        with open(TRAFFIC_FILE) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch:"):
                    return float(line.split(":", 1)[1])
    except OSError:
        pass
    return None


def cpu_decode_baseline(budget_tokens=8):
    """Same-run host figure for the 7B-shape decode: the CPU decode oracle (f32 weights dequantised once, all
    threads in the matrix-vector products) on a TWO-layer slice of the Mistral-7B shape plus the full lm_head,
    timed per token at a short context and EXTRAPOLATED to 32 layers by the f32 weight bytes a token streams
    (the host path is memory-bound): t_32 = t_2 * bytes_32 / bytes_2.  A full 32-layer f32 model (28 GB) is not
    practical to build and time inside the benchmark."""
    import oracle as o

    H, I, V, NH, NKV, D = 4096, 14336, 32000, 32, 8, 128
    rng = np.random.default_rng(7)

    def packed(n, k):
        nsb = n * k // 256
        b = rng.integers(0, 256, size=(nsb, 144), dtype=np.uint8)
        b[:, 0:2] = np.frombuffer(np.float16(8e-4).tobytes(), np.uint8)
        b[:, 2:4] = np.frombuffer(np.float16(6e-3).tobytes(), np.uint8)
        return b.reshape(-1)

    layers = 2
    m = o.DecodeModel(vocab_size=V, hidden_size=H, intermediate_size=I, num_layers=layers, num_heads=NH,
                      num_kv_heads=NKV, head_dim=D, max_seq_len=16, rms_norm_eps=1e-5, rope_theta=10000.0)
    m.set_embedding_f16((rng.standard_normal((V, H)) * 0.02).astype(np.float16).view(np.uint16))
    shapes = {"q": (H, H), "k": (NKV * D, H), "v": (NKV * D, H), "o": (H, H), "gate": (I, H), "up": (I, H), "down": (H, I)}
    for layer in range(layers):
        for name, (n, k) in shapes.items():
            m.set_linear(layer, o.DecodeModel.LIN[name], o.Q4_K, packed(n, k))
    m.set_linear(-1, 0, o.Q4_K, packed(V, H))
    m.forward(1, 0, want_logits=False)  # first touch
    times = []
    for pos in range(1, 1 + budget_tokens):
        t0 = time.perf_counter()
        m.forward(pos, pos, want_logits=False)
        times.append(time.perf_counter() - t0)
    m.close()
    t2 = float(np.median(times))
    per_layer = 2 * H * H + 2 * NKV * D * H + 3 * I * H
    scale = (32 * per_layer + V * H) / (layers * per_layer + V * H)
    t32 = t2 * scale
    return {"tokens_per_s": 1.0 / t32, "ms_per_token": t32 * 1e3, "kind": "port, extrapolated from a 2-layer slice",
            "cores": int(o.lib().axo_num_threads()), "ms_per_token_2_layers_plus_head": t2 * 1e3, "extrapolation_factor": scale,
            "sample": f"median of {budget_tokens} tokens on a 2-layer model of the Mistral-7B shape with the full lm_head, context < 16"}


def codec_rates(ctx, n=N_HEAD, k=K_HEAD, iters=20):
    """quantize_tensor / dequantize_tensor on the device for one weight of the headline shape, per type: time per call
    and the bytes it has to move (4 B per element on the f32 side, the packed image on the other)."""
    from axonml_amd import quant as q
    from axonml_amd._lib import MEM_DEVICE

    lib, numel = ctx.lib, n * k
    f = ctx.malloc(numel * 4)
    g = ctx.malloc(numel * 4)
    ctx.check(lib.axq_fill_normal_f32(ctx.handle, f, numel, 0.0, 0.02, 0.01, 0.5, 99))
    out = []
    for qt in (q.QuantType.Q8_0, q.QuantType.Q4_0, q.QuantType.Q4_1, q.QuantType.Q5_0, q.QuantType.Q5_1, q.QuantType.Q4_K, q.QuantType.F16):
        nbytes = lib.axq_packed_bytes(int(qt), numel)
        p = ctx.malloc(nbytes)
        r = {"type": str(qt), "numel": numel, "packed_bytes": nbytes}
        for name, call in (("quantize", lambda: lib.axq_quantize(ctx.handle, int(qt), f, numel, p, MEM_DEVICE)),
                           ("dequantize", lambda: lib.axq_dequantize(ctx.handle, int(qt), p, numel, g, MEM_DEVICE))):
            for _ in range(3):
                ctx.check(call())
            ctx.synchronize()
            ctx.timer_start()
            for _ in range(iters):
                ctx.check(call())
            t = ctx.timer_stop() / iters
            r[f"{name}_us"] = t * 1e3
            r[f"{name}_gbps"] = (numel * 4 + nbytes) / (t * 1e-3) / 1e9
        log(f"  codec {r['type']}: quantize {r['quantize_us']:.1f} us ({r['quantize_gbps']:.0f} GB/s), "
            f"dequantize {r['dequantize_us']:.1f} us ({r['dequantize_gbps']:.0f} GB/s)")
        out.append(r)
        ctx.free(p)
    ctx.free(f)
    ctx.free(g)
    return out


def read_sweep(ctx, steps, warmup):
    """Prints a table: a kernel that only READS a ring copy of the headline weight (no arithmetic, one sink store per
    workgroup), over workgroups per CU x threads x 16-byte loads in flight per thread x temporal / non-temporal loads,
    launches following one another on one stream; the same kernel over several streams; a row-walking pattern; and the
    GEMV itself on one and on several streams.  The best one-stream line is the ceiling the GEMV is held against."""
    from axonml_amd import quant as q

    lib, T = ctx.lib, q.QuantType
    wbytes = lib.axq_packed_bytes(int(T.Q4_K), N_HEAD * K_HEAD)
    ws = make_ring(ctx, T.Q4_K, N_HEAD, K_HEAD, int(RING_BYTES // wbytes) + 1, 0.01)
    arr = (C.c_void_p * len(ws))(*[w.value for w in ws])
    sink = ctx.malloc(256)
    x_dev = ctx.to_device(np.random.default_rng(0).standard_normal((1, K_HEAD)).astype(np.float32))
    y_dev = ctx.malloc(N_HEAD * 4)

    def t_read(wg, th, u, nt, pattern, streams):
        ms, _, _, _ = time_ring(ctx, lambda first, n: ctx.check(lib.axq_bench_read_ring_ex(ctx.handle, arr, len(ws), first, sink, n, wg, th, u,
                                                                                              nt, pattern, streams)), len(ws), steps, warmup)
        return ms * 1e3

    def line(what, us, nbytes=wbytes):
        print(f"{what:<72s} {us:7.2f} us  {nbytes / us / 1e3:7.1f} GB/s  {nbytes / us / 1e3 / HBM_PEAK_GBPS:5.3f} of peak", flush=True)

    print(f"# Q4_K {N_HEAD} x {K_HEAD}: {wbytes} bytes per launch, ring of {len(ws)} copies, {steps} launches per figure (median of {REPEATS})")
    line("GEMV, one stream", time_gemv(ctx, ws, x_dev, y_dev, 1, steps, warmup)[0] * 1e3)
    for st in (2, 3, 4):
        ms, _, _, _ = time_ring(ctx, lambda first, n: ctx.check(lib.axq_bench_gemv_ring_streams(ctx.handle, arr, len(ws), first, x_dev, 1, y_dev,
                                                                                                 n, st)), len(ws), steps, warmup)
        line(f"GEMV, launches dealt over {st} streams", ms * 1e3)
    best = None
    for wg in (1, 2, 4):
        for th in (256, 512, 1024):
            for u in (4, 8, 16, 32):
                if th == 1024 and u == 32:
                    continue
                for nt in (1, 0):
                    us = t_read(wg, th, u, nt, 0, 1)
                    line(f"read: {wg} wg/CU x {th:4d} threads x {u:2d} loads in flight, {'non-temporal' if nt else 'temporal'}", us)
                    if best is None or us < best[0]:
                        best = (us, wg, th, u, nt)
    # the code plane only (k / 2 bytes per row): in the order the one-vector GEMV asks for it (a wave's load takes 256 bytes
    # of each of four rows), and the same count of bytes per wave and step from one contiguous run (what a tiled layout
    # of the plane would give the GEMV), per wave or per workgroup
    for pattern, what in ((1, "the GEMV's row order"), (2, "contiguous per wave"), (3, "contiguous per workgroup")):
        for u in (4, 8, 14):
            line(f"read, code plane, {what}, {u:2d} loads in flight per lane", t_read(1, 512, u, 1, pattern, 1), N_HEAD * K_HEAD // 2)
    for st in (2, 4):
        line(f"read: 1 wg/CU x  512 threads x 16 loads, launches dealt over {st} streams", t_read(1, 512, 16, 1, 0, st))
        line(f"read: 2 wg/CU x  256 threads x 16 loads, launches dealt over {st} streams", t_read(2, 256, 16, 1, 0, st))
    line("GEMV, one stream (again)", time_gemv(ctx, ws, x_dev, y_dev, 1, steps, warmup)[0] * 1e3)
    print(f"# best read-only kernel on one stream: {best[1]} wg/CU x {best[2]} threads x {best[3]} loads in flight, "
          f"{'non-temporal' if best[4] else 'temporal'}: {best[0]:.2f} us = {wbytes / best[0] / 1e3 / HBM_PEAK_GBPS:.3f} of peak")
    for w in ws:
        lib.axq_weight_free(ctx.handle, w)
    ctx.free(sink)
    ctx.free(x_dev)
    ctx.free(y_dev)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-extras", action="store_true", help="headline case only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--ring-only", action="store_true",
                    help="for kernel-trace profiles: skip the cache-resident leg, so that every launch of the GEMV kernel "
                         "but the one oracle check streams a ring copy from HBM")
    ap.add_argument("--profile-graph", action="store_true", help="for kernel-trace profiles: one more pass of graph replays of the headline ring")
    ap.add_argument("--counter-probe", action="store_true",
                    help="for profiler counter runs: a few launches of a 256 MiB plain copy kernel, then the "
                         "headline GEMV ring; no oracle, no CPU leg, no JSON line")
    ap.add_argument("--read-sweep", action="store_true",
                    help="instead of the benchmark: time a read-only kernel over the headline weight in every launch shape, "
                         "and print the table")
    ap.add_argument("--gemv-table", action="store_true",
                    help="instead of the benchmark, for kernel-trace profiles: the one-vector and batch-8 GEMVs of every block "
                         "type at 14336x4096 and 4096x14336 as plain stream launches over their rings, one line each")
    ap.add_argument("--grid-barrier", action="store_true",
                    help="instead of the benchmark: time a barrier over all workgroups of one resident launch through device-scope "
                         "atomics (what a kernel that spans dependent steps would pay per step), and print the table")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus must be 1 (no multi-GPU path is built or measured)")

    from axonml_amd import quant as q

    ctx = q.default_context()
    lib = ctx.lib
    info = ctx.device_info()
    log(f"device: {info.name.decode()} {info.arch.decode()} CUs={info.compute_units}")
    T = q.QuantType

    if args.counter_probe:
        counter_probe(ctx, args.steps)
        return
    if args.read_sweep:
        read_sweep(ctx, args.steps, args.warmup)
        return
    if args.grid_barrier:
        out = (C.c_float * 3)()
        print(f"{info.compute_units} workgroups of 256 threads, one per compute unit; 256 rounds per line, medians over the last 192; us")
        print("counters  published bytes per workgroup   last arrival -> release seen by the median workgroup   by the slowest   publishing")
        for levels in (1, 2):
            for pub in (0, 1024, 4096, 16384):
                ctx.check(lib.axq_bench_grid_barrier(ctx.handle, levels, pub, 256, out))
                print(f"{'one' if levels == 1 else '16 + 1':8s}  {pub:8d}   {out[0]:6.2f}   {out[1]:6.2f}   {out[2]:6.2f}", flush=True)
        return
    if args.gemv_table:
        for qt in (T.Q4_K, T.Q5_K, T.Q6_K, T.Q4_0, T.Q4_1, T.Q5_0, T.Q5_1, T.Q8_0):
            for n, k in ((N_HEAD, K_HEAD), (K_HEAD, N_HEAD)):
                for b in (1, 8):
                    r, ws, _, xd, yd = gemv_case(ctx, qt, n, k, b, args.steps, 50, graph=False)
                    free_case(ctx, ws, xd, yd)
                    print(f"{r['type']} [{n},{k}] b={b}: {r['us_per_step']:.2f} us, {r['gbps']:.0f} GB/s, ring of {r['ring_copies']}", flush=True)
        return

    # ---- headline: Q4_K GEMV 14336 x 4096, batch 1
    head, ws, x, x_dev, y_dev = gemv_case(ctx, T.Q4_K, N_HEAD, K_HEAD, 1, args.steps, args.warmup, outlier_p=0.01)
    err, packed = check_against_oracle(ctx, ws[0], T.Q4_K, N_HEAD, K_HEAD, x, y_dev)
    log(f"headline: {head['us_per_step']:.2f} us/step, {head['gbps']:.0f} GB/s, max rel err vs oracle {err:.2e}")
    if err > 1e-3:
        sys.exit(f"bench.py: GPU result differs from the oracle (max rel err {err:.3e} > 1e-3)")
    exact = codes_bit_exact(ctx, packed, T.Q4_K, N_HEAD, K_HEAD, 0.01, RING_SEED0)
    log(f"headline weight: device-quantised codes and scales {'equal' if exact else 'DIFFER FROM'} the oracle's, byte for byte")
    if not exact:
        sys.exit("bench.py: the device quantiser's packed bytes differ from the oracle's on the headline weight")
    # the read ceiling of the same run: the same ring, the same grid, a kernel that only reads
    sink = ctx.malloc(256)
    ms_read_s, _, _, _ = time_read(ctx, ws, sink, args.steps, args.warmup)
    ms_read_g, _, _ = time_graph(ctx, ws, None, None, 1, read_sink=sink)
    ms_read = min(ms_read_s, ms_read_g)  # the ceiling is whichever way of handing over the launches is faster, as for the GEMV
    # launches that do not wait for each other: the same ring spread over three streams (a figure beside the reported one)
    arr = (C.c_void_p * len(ws))(*[w.value for w in ws])
    ms_streams, _, _, _ = time_ring(ctx, lambda first, n: ctx.check(lib.axq_bench_gemv_ring_streams(ctx.handle, arr, len(ws), first, x_dev, 1, y_dev, n, 3)),
                                    len(ws), args.steps, args.warmup)
    ms_read_streams, _, _, _ = time_ring(ctx, lambda first, n: ctx.check(lib.axq_bench_read_ring_ex(ctx.handle, arr, len(ws), first, sink, n, 1, 512, 16, 1, 0, 2)),
                                         len(ws), args.steps, args.warmup)
    ctx.free(sink)
    read_gbps = lib.axq_packed_bytes(int(T.Q4_K), N_HEAD * K_HEAD) / (ms_read * 1e-3) / 1e9
    log(f"read-only kernel over the same ring: {ms_read * 1e3:.2f} us/launch ({ms_read_s * 1e3:.2f} as stream launches, {ms_read_g * 1e3:.2f} "
        f"as a graph replay), {read_gbps:.0f} GB/s; the GEMV runs at {head['gbps'] / read_gbps:.2f} of it")
    log(f"launches that may overlap: GEMV over 3 streams {ms_streams * 1e3:.2f} us/launch, read-only kernel over 2 streams "
        f"{ms_read_streams * 1e3:.2f} us/launch")
    # cache-resident figure, labelled as such
    ms_hot = None if args.ring_only else time_gemv(ctx, ws[:1], x_dev, y_dev, 1, args.steps, args.warmup)[0]
    if args.profile_graph:  # for kernel-trace profiles of the reported submission: replays of the recorded ring, nothing else after them
        time_graph(ctx, ws, x_dev, y_dev, 1)
    free_case(ctx, ws, x_dev, y_dev)

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(packed, T.Q4_K, N_HEAD, K_HEAD, x)
        log(f"cpu baseline: {cpu['ms_per_step']:.1f} ms/step on {cpu['cores']} threads")

    wq4k = lib.axq_packed_bytes(int(T.Q4_K), N_HEAD * K_HEAD)
    extra = {"read_ceiling_gbps": read_gbps, "read_ceiling_us": ms_read * 1e3,
             "read_ceiling_us_stream_launches": ms_read_s * 1e3, "read_ceiling_us_graph_replay": ms_read_g * 1e3,
             "read_ceiling_note": "same run, same ring of weight copies, one 512-thread workgroup per compute unit reading each "
                                  "copy's packed image with non-temporal 16-byte loads and keeping nothing; the faster of stream "
                                  "launches and a graph replay, as for the GEMV (profiles/read_only_kernel_sweep.txt: no grid, "
                                  "workgroup size, depth or load type reads these 33 MB faster in launches that follow each other)",
             "frac_of_read_ceiling": head["gbps"] / read_gbps,
             "headline_us_per_step_stream_launches": head["us_per_step_stream_launches"],
             "headline_us_per_step_graph_replay": head["us_per_step_graph_replay"],
             "overlapped_launches": {
                 "note": "launches that do not wait for each other (ring spread over streams); beside the reported figure, which is "
                         "for launches that follow each other on one stream",
                 "gemv_3_streams_us_per_step": ms_streams * 1e3,
                 "gemv_3_streams_gbps": head["algorithmic_bytes"] / (ms_streams * 1e-3) / 1e9,
                 "gemv_3_streams_frac_of_hbm_peak": head["algorithmic_bytes"] / (ms_streams * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                 "read_only_2_streams_us_per_launch": ms_read_streams * 1e3,
                 "read_only_2_streams_gbps": wq4k / (ms_read_streams * 1e-3) / 1e9},
             "headline_us_per_step_min_max_over_repeats": head["us_per_step_min_max"],
             "headline_cache_resident_us": ms_hot * 1e3 if ms_hot else None,
             "headline_cache_resident_gbps": head["algorithmic_bytes"] / (ms_hot * 1e-3) / 1e9 if ms_hot else None,
             "max_rel_err_vs_oracle": err}
    gate = {"codes_bit_exact": exact, "max_rel_err_vs_oracle": err, "tolerance": 1e-3,
            "what": "ring copy 0 of the headline weight: the f32 the device drew, quantised by the oracle on the host, equals the "
                    "device quantiser's packed image byte for byte; the GEMV on it against the oracle's dequantise -> f32 sgemm"}
    if not args.no_extras:
        cases = [(T.Q4_K, 4096, 14336, 1, 0.01), (T.Q8_0, 4096, 4096, 1, 0.0), (T.Q4_0, 11008, 4096, 1, 0.0),
                 (T.Q4_0, 4096, 11008, 1, 0.0), (T.Q4_1, 11008, 4096, 1, 0.0), (T.Q4_1, 4096, 11008, 1, 0.0),
                 (T.Q4_0, 11008, 4096, 8, 0.0), (T.Q4_1, 11008, 4096, 8, 0.0), (T.Q4_0, 4096, 11008, 8, 0.0),
                 (T.Q4_1, 4096, 11008, 8, 0.0),
                 # the types a Q4_K_M or Q5_K_M GGUF file holds beside Q4_K
                 (T.Q6_K, 14336, 4096, 1, 0.0), (T.Q6_K, 4096, 14336, 1, 0.0), (T.Q5_K, 14336, 4096, 1, 0.0)]
        gem = []
        for qt, n, k, b, op in cases:
            r, ws2, _, xd, yd = gemv_case(ctx, qt, n, k, b, args.steps, 50, outlier_p=op)
            free_case(ctx, ws2, xd, yd)
            gem.append(r)
            log(f"  {r['type']} [{n},{k}] b={b}: {r['us_per_step']:.2f} us, {r['gbps']:.0f} GB/s")
        extra["gemv"] = gem
        extra["codecs"] = codec_rates(ctx)
        try:
            from axonml_amd import decode as d

            extra["decode"] = d.bench_7b(ctx, log)
            if not args.no_cpu:
                extra["decode"]["cpu_baseline"] = cpu_decode_baseline()
                log(f"  decode cpu baseline (extrapolated): {extra['decode']['cpu_baseline']['tokens_per_s']:.2f} tok/s")
        except ImportError:
            pass
        try:
            from axonml_amd import prefill as pf

            extra["prefill_gemm"] = pf.bench(ctx, log)
        except ImportError:
            pass
        try:
            from axonml_amd import gguf

            extra["gguf_convert"] = gguf.bench(ctx, log)
        except ImportError:
            pass

    out = {
        "metric": "q4k_gemv_effective_hbm_gbps",
        "value": head["gbps"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["us_per_step"] / 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "Q4_K GEMV 14336x4096, batch 1 (BASELINE config 3)", "quant_type": "Q4_K",
                   "n_rows": N_HEAD, "k": K_HEAD, "batch": 1, "ring_copies": head["ring_copies"],
                   "repeats": REPEATS, "launches_per_repeat": head["launches_per_repeat"],
                   "internal_warmup": head["untimed_launches"], "submission": head["submission"],
                   "timing": "median over `repeats` event-bracketed repeats of `launches_per_repeat` launches that follow each other "
                             "on one stream, after `internal_warmup` untimed launches; measured twice, as plain stream launches "
                             "(max(200, steps / repeats) per repeat) and as replays of one recorded hipGraph (a whole number of trips "
                             "round the ring), and the faster way of handing the same launches over is reported (`submission`)",
                   "algorithmic_bytes_per_step": head["algorithmic_bytes"],
                   "inputs": "W~N(0,0.02) with 1% at +-0.5, x~N(0,1), generated and quantised on the device"},
        "roofline": {"bound": "hbm", "achieved": head["gbps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": head["gbps"] / HBM_PEAK_GBPS, "traffic": measured_traffic(),
                     "traffic_source": "profiles/gemv_q4k_14336x4096_hbm_counters.txt (profiler counter runs of this "
                                       "kernel), not measured in this run"},
        "cpu_baseline": cpu,
        "codes_bit_exact": exact,
        "correctness_gate": gate,
        "extra": extra,
    }
    print(json.dumps(out), flush=True)
    ctx.close()  # device memory and the stream go now, not whenever the interpreter gets round to it


if __name__ == "__main__":
    main()

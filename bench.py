#!/usr/bin/env python3
"""Benchmark of the torch_webgpu op path on one MI355X: achieved HBM GB/s.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--log2n 28]

One "step" is one pass of the three ops the headline metric names, each on 2^28
fp32 elements already resident in HBM:
    add.Tensor   two contiguous vectors                      12 B/elem
    gelu         approximate='none' on [16384, 16384]          8 B/elem
    masked_select  Bernoulli(0.5) mask, count read back        5 B/elem + 4 B/selected
`value` is the algorithmic bytes of one step divided by the wall time of one step.
After the timed steps every other configuration (silu, relu, row-bias and
transposed add, eq / ne / bitwise_and, masked_select at p = 0.01 / 0.99 /
clustered) is timed per launch with HIP events and listed under "ops".

Kernels are launched through the C ABI of libtwg_hip.so (ctypes); durations come
from hipEvents recorded on the library's own stream.  The CPU baseline legs time
(a) the single-threaded C oracle and (b) PyTorch's CPU kernels on the box's cores,
on bounded samples.  Prints ONE JSON line on stdout; progress goes to stderr.
"""
import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "torch-webgpu_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published


# Every masked_select launch of the run, by mask, in launch order (run-length encoded in the JSON
# line as "masked_select_launch_order"): a kernel trace or counter run of this script shows one
# kernel name for all masks, and this is what tells its dispatches apart.
MS_LAUNCHES = []


def note_ms(name):
    if MS_LAUNCHES and MS_LAUNCHES[-1][0] == name:
        MS_LAUNCHES[-1][1] += 1
    else:
        MS_LAUNCHES.append([name, 1])


class Durations(list):
    """Per-launch durations with room for the back-to-back average."""
    batch_avg = None


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--log2n", type=int, default=28, help="log2 of the element count (28 = the named config)")
    ap.add_argument("--no-sweep", action="store_true", help="skip the per-op sweep of the other configs")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-dispatcher", action="store_true",
                    help="skip the lines timed through device=\"webgpu\" (torch dispatcher, result allocated per call)")
    ap.add_argument("--only", default="", help="comma list of op names to run in the sweep")
    ap.add_argument("--geometries", action="store_true",
                    help="instead of the benchmark: time add over families of broadcast and permuted "
                         "operands (~2^25 elements each) and print their spread as one JSON line")
    ap.add_argument("--first-launches", action="store_true",
                    help="instead of the benchmark: time 40 consecutive gelu launches one by one on buffers "
                         "in different states (fresh from hipMalloc, filled once, recycled by the pool, after "
                         "2 s of idle time) and print the series as one JSON line")
    ap.add_argument("--chain", action="store_true",
                    help="instead of the benchmark: time a chain of five dependent elementwise ops "
                         "(gelu, add, relu, mul, silu) on tensors of 8 to 256 MiB, the inputs taken in turn "
                         "from four sets and the intermediates recycled, and print one JSON line")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py: this op path is single-GPU (no collectives, nothing to shard in one "
            "process); run with --gpus 1.  Across GPUs every op would split along the flattened "
            "element axis with no exchange; masked_select adds one scan of the per-GPU counts.")
        sys.exit(2)

    import torch
    import twg_capi as capi
    import twg_workloads as W

    L = capi.load()
    capi.init()
    if args.geometries:
        print(json.dumps(geometry_families(capi, L)), flush=True)
        return
    if args.first_launches:
        print(json.dumps(first_launches(capi, L, torch, 1 << args.log2n)), flush=True)
        return
    if args.chain:
        print(json.dumps(op_chain(capi, L)), flush=True)
        return
    dev_name, cus, mem = capi.device_info()
    log(f"device: {dev_name}  CUs={cus}  mem={mem / 2**30:.0f} GiB")
    n = 1 << args.log2n
    K, Wm = args.steps, args.warmup

    def ev_pair():
        return capi.Event(), capi.Event()

    def time_launches(fn, warm, reps):
        """Durations (ms) of `reps` launches.  The list holds one figure per launch from an
        event pair around each call; its attribute `batch_avg` is (stop - start) / reps for
        the same number of launches issued back to back between ONE event pair, which leaves
        out the event packets and the host's gap between calls (5-10 us per launch: 7% of a
        0.13 ms kernel) and is what a kernel trace reports as the average duration."""
        for _ in range(warm):
            fn()
        capi.sync()
        evs = [ev_pair() for _ in range(reps)]
        for s, e in evs:
            s.record()
            fn()
            e.record()
        capi.sync()
        per_launch = Durations(s.elapsed_ms(e) for s, e in evs)
        s, e = ev_pair()
        s.record()
        for _ in range(reps):
            fn()
        e.record()
        capi.sync()
        per_launch.batch_avg = s.elapsed_ms(e) / reps
        return per_launch

    # HBM bytes per launch measured with rocprofv3 (FETCH_SIZE + WRITE_SIZE, each scaled by a
    # transfer of known size); recorded figures, not re-measured by this run
    traffic = {}
    traffic_source = None
    tr = os.path.join(ROOT, "profiles", "hbm_traffic.txt")
    if os.path.exists(tr):
        commit = "unknown commit"
        with open(tr) as f:
            for line in f:
                if line.startswith("# measured at commit"):
                    commit = line.split()[-1]
                elif "=" in line and not line.startswith("#"):
                    k, v = line.split("=")
                    traffic[k.strip()] = int(v)
        traffic_source = f"recorded: profiles/hbm_traffic.txt @ {commit} (not measured by this run)"

    def summarize(name, kernel, nbytes, ms_list, nelem, extra=None):
        avg = getattr(ms_list, "batch_avg", None) or sum(ms_list) / len(ms_list)
        med = statistics.median(ms_list)
        moved = traffic.get(f"{name}@2^{args.log2n}")
        d = {
            "op": name, "kernel": kernel, "elements": nelem, "bytes": nbytes,
            "avg_ms": round(avg, 5), "median_ms": round(med, 5), "min_ms": round(min(ms_list), 5),
            "avg_over": ("launches issued back to back between one event pair"
                         if getattr(ms_list, "batch_avg", None) else "one event pair per launch"),
            "per_launch_avg_ms": round(sum(ms_list) / len(ms_list), 5),
            "GBps": round(nbytes / avg / 1e6, 1),
            "GBps_median": round(nbytes / med / 1e6, 1),
            "Gelem_per_s": round(nelem / avg / 1e6, 2),
            "pct_hbm_peak": round(nbytes / avg / 1e6 / HBM_PEAK_GBS * 100, 2),
            # the same time against the bytes the kernel really moved over HBM (recorded
            # FETCH_SIZE + WRITE_SIZE): below the algorithmic figure where source lines
            # without a selected element are never fetched
            "traffic": moved,
            "traffic_source": traffic_source if moved else None,
            "pct_hbm_peak_on_traffic": (round(moved / avg / 1e6 / HBM_PEAK_GBS * 100, 2)
                                        if moved else None),
        }
        if extra:
            d.update(extra)
        on_traffic = (f"  ({d['pct_hbm_peak_on_traffic']:6.2f}% on measured traffic)"
                      if moved else "")
        if "pct_hbm_peak_rotating_outputs" in d:
            on_traffic += f"  ({d['pct_hbm_peak_rotating_outputs']:6.2f}% with rotating outputs)"
        log(f"  {name:28s} {d['avg_ms']:9.4f} ms  {d['GBps']:8.1f} GB/s  {d['pct_hbm_peak']:6.2f}% of peak{on_traffic}")
        return d

    f32 = ctypes.c_float

    # Two transfers of known size that are none of the measured kernels: a 1 GiB device-to-device
    # hipMemcpyAsync (the runtime's own blit kernel: 1 GiB read, 1 GiB written) and a 1 GiB fill
    # (1 GiB written, nothing read).  A counter run of this script (rocprofv3 --pmc FETCH_SIZE /
    # WRITE_SIZE) reads its scale factors off these two dispatches.
    cal = calibration_transfers(capi, L)

    # ------------------------------------------------------------ headline inputs
    t0 = time.time()
    log(f"generating inputs for n = 2^{args.log2n} ...")
    rows = 1 << (args.log2n // 2)
    cols = n // rows
    a_h, b_h = W.add_contiguous(n, seed=0)
    x_h = W.activation_input(rows, cols, seed=1).view(-1)
    src_h = W.select_source(n, seed=4)
    m50_h = W.bernoulli_mask(n, 0.5)
    k50 = int(m50_h.sum())
    d_a, d_b, d_x, d_src, d_m = (capi.to_device(t) for t in (a_h, b_h, x_h, src_h, m50_h))
    d_out = capi.DeviceBuffer(4 * n)
    d_cnt = capi.DeviceBuffer(8)
    scratch_bytes = L.twg_masked_select_scratch_bytes(n)
    d_scratch = capi.DeviceBuffer(scratch_bytes)
    it = capi.dense_iter(n)
    cnt_host = torch.zeros(1, dtype=torch.int64)
    capi.sync()
    log(f"  inputs ready in {time.time() - t0:.1f} s")

    def run_add():
        capi.check(L.twg_add_f32(d_out.ptr, d_a.ptr, d_b.ptr, f32(1.0), ctypes.byref(it), None))

    def run_gelu():
        capi.check(L.twg_unary_f32(capi.UNARY_GELU_ERF, d_out.ptr, d_x.ptr, ctypes.byref(it), None))

    k_host = ctypes.c_int64(0)

    def run_ms(mask_buf=None):
        """The op as the dispatcher runs it: compaction with the count handed to the host
        (the call returns once the count is known; the output is stream ordered), tickets
        and status words in the array the library keeps for this (no scratch passed)."""
        note_ms("masked_select_p0.50")
        capi.check(L.twg_masked_select_count(d_out.ptr, ctypes.byref(k_host), d_src.ptr, 4,
                                             (mask_buf or d_m).ptr, ctypes.byref(it),
                                             None, 0, None))
        return k_host.value

    bytes_add = W.BYTES_PER_ELEM["add"] * n
    bytes_gelu = W.BYTES_PER_ELEM["gelu"] * n
    bytes_ms = W.masked_select_bytes(n, k50)
    step_bytes = bytes_add + bytes_gelu + bytes_ms

    # ------------------------------------------------------------ timed steps
    # A GPU that has been idle (here: while the host generated and uploaded the inputs) runs
    # its first 2-3 ms of work at full rate, then 10-20% slower for about 4 ms, then settles
    # (profiles/first_launches_after_idle_gelu_2p28.md: the same on buffers that were never
    # touched, filled once, or recycled, and again after any 2 s pause).  Forty untimed gelu
    # launches (13 ms) put that transient behind the run before the W warm-up steps start.
    settle = 40
    for _ in range(settle):
        run_gelu()
    log(f"timing {K} steps after {settle} settling launches and {Wm} warm-up steps ...")
    for _ in range(Wm):
        run_add(); run_gelu(); assert run_ms() == k50
    capi.sync()
    ev = [[capi.Event() for _ in range(4)] for _ in range(K)]
    t_start = time.perf_counter()
    for i in range(K):
        e = ev[i]
        e[0].record(); run_add()
        e[1].record(); run_gelu()
        e[2].record(); got = run_ms()
        e[3].record()
        if got != k50:
            raise RuntimeError(f"masked_select count {got} != {k50}")
    capi.sync()
    t_stop = time.perf_counter()
    ms_per_step = (t_stop - t_start) * 1e3 / K
    value = step_bytes / (ms_per_step * 1e6)  # GB/s

    ops = []
    add_ms = [e[0].elapsed_ms(e[1]) for e in ev]
    gelu_ms = [e[1].elapsed_ms(e[2]) for e in ev]
    msk_ms = [e[2].elapsed_ms(e[3]) for e in ev]   # scratch clear + compaction kernel
    # the whole op as the host sees it: calls that each wait for their count, back to back
    mso_ms = time_launches(run_ms, 1, K).batch_avg
    head = [
        summarize("add", "ew_contig<AddOp>", bytes_add, add_ms, n),
        summarize("gelu", "ew_contig<GeluErfOp>", bytes_gelu, gelu_ms, n),
        summarize("masked_select_p0.50", "ms_compact_stream<16,4>", bytes_ms, msk_ms, n,
                  {"selected": k50, "op_ms_with_count_readback": round(mso_ms, 5)}),
    ]
    ops += head
    dominant = max(head, key=lambda d: d["avg_ms"])
    roofline = {
        "bound": "hbm", "kernel": dominant["kernel"], "op": dominant["op"],
        "achieved": dominant["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(dominant["GBps"] / HBM_PEAK_GBS, 4),
        "traffic": None,
        "algorithmic_bytes_per_launch": dominant["bytes"],
        "avg_launch_ms": dominant["avg_ms"],
    }
    roofline["traffic"] = dominant["traffic"]
    roofline["traffic_source"] = dominant["traffic_source"]
    roofline["frac_on_traffic"] = (round(dominant["pct_hbm_peak_on_traffic"] / 100, 4)
                                   if dominant["traffic"] else None)

    # ------------------------------------------------------------ sweep of the other configs
    del a_h, b_h
    only = set(filter(None, args.only.split(",")))

    def want(name):
        return not only or name in only

    result_sweep = []
    if not args.no_sweep:
        log("sweep of the remaining configurations ...")
        result_sweep = sweep(args, capi, W, L, torch, n, rows, cols, K, Wm, time_launches, summarize,
                             d_out, d_cnt, d_scratch, scratch_bytes, d_src, d_x, it, cnt_host, want)
    ops += result_sweep

    # ------------------------------------------------------------ the product path itself
    disp = None
    if not args.no_dispatcher and not only:
        # release what the C-ABI legs hold first; the dispatcher legs upload their own tensors
        by_name = {d["op"]: d for d in ops}
        disp = dispatcher_lines(args, capi, W, torch, n, rows, cols, K, Wm, time_launches, by_name,
                                x_h, src_h, m50_h, k50)

    # ------------------------------------------------------------ config 1: small add + transfers
    small = None
    if not args.no_sweep and want("config1"):
        small = config1(capi, W, L, torch, time_launches, Wm, K)

    # ------------------------------------------------------------ CPU baselines
    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(torch, W, n, x_h, src_h, m50_h, step_bytes, bytes_add, bytes_gelu, bytes_ms)

    out = {
        "metric": "HBM GB/s (% of peak) for add/gelu/masked_select at 2^28 fp32, 1 GPU",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": Wm,
        "settle_launches_before_warmup": settle,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"one step = add.Tensor + gelu(approximate='none') + masked_select"
                               f"(Bernoulli 0.5) on 2^{args.log2n} fp32 elements resident in HBM "
                               "(configs[1] shape [16384,16384] for gelu; configs[0]/[4] shapes for "
                               "add and masked_select at the same element count)",
                   "elements": n, "step_bytes": step_bytes},
        "pct_hbm_peak": round(value / HBM_PEAK_GBS * 100, 2),
        "roofline": roofline,
        "cpu_baseline": cpu,
        "config1_small_add_and_transfers": small,
        "dispatcher": disp,
        "ops": ops,
        "device": {"name": dev_name, "compute_units": cus},
        "counter_calibration_transfers": cal,
        "masked_select_launch_order": MS_LAUNCHES,
    }
    print(json.dumps(out), flush=True)


def calibration_transfers(capi, L):
    gib = 1 << 30
    a, b = capi.DeviceBuffer(gib), capi.DeviceBuffer(gib)
    capi.check(L.twg_fill_bytes(a.ptr, 0x5A, gib, None))
    capi.sync()
    res = {}
    # the runtime's own device-to-device copy, called directly: an anchor that is none of the
    # library's kernels (twg_memcpy_d2d uses the library's copy kernel at this size)
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipMemcpyAsync.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int,
                                   ctypes.c_void_p]
    hip.hipMemcpyAsync.restype = ctypes.c_int
    L.twg_default_stream.restype = ctypes.c_void_p
    stream = L.twg_default_stream()

    def runtime_copy():
        rc = hip.hipMemcpyAsync(b.ptr, a.ptr, gib, 3, stream)  # 3 = hipMemcpyDeviceToDevice
        if rc:
            raise RuntimeError(f"hipMemcpyAsync failed: {rc}")

    for name, fn in (("hipMemcpyAsync_d2d_1GiB", runtime_copy),
                     ("twg_fill_bytes_1GiB", lambda: capi.check(L.twg_fill_bytes(b.ptr, 0xA5, gib, None)))):
        fn()
        capi.sync()
        e0, e1 = capi.Event(), capi.Event()
        e0.record()
        for _ in range(3):
            fn()
        e1.record()
        capi.sync()
        res[name] = {"ms": round(e0.elapsed_ms(e1) / 3, 4), "dispatches": 4}
    return res


def dispatcher_lines(args, capi, W, torch, n, rows, cols, K, Wm, time_launches, by_name,
                     x_h, src_h, m_h, k50):
    """The same ops as a user runs them: `a + b`, `F.gelu(x)`, `torch.eq(p, q)`,
    `torch.masked_select(x, m)` on device="webgpu" tensors through the torch dispatcher, the
    result allocated by each call (caching allocator) and, for masked_select, the count
    waited for and the result shaped.  Timed with events on the library's stream, calls issued
    back to back; `vs_c_abi` is this time over the C-ABI line of the same op."""
    import torch.nn.functional as F
    import torch_webgpu  # noqa: F401
    res = []

    def line(name, fn, nbytes, ref_ms):
        # these legs upload their own operands, and after the idle time of an upload the GPU's
        # first 9 ms of work hold a slow stretch (see the note at the timed steps): keep it busy
        # for 25 ms before the warm-up launches
        t_busy = time.perf_counter()
        settled = 0
        while time.perf_counter() - t_busy < 0.025:
            for _ in range(10):
                fn()
            settled += 10
            capi.sync()
        ms = time_launches(fn, Wm, K)
        avg = ms.batch_avg
        d = {"op": name, "avg_ms": round(avg, 5), "GBps": round(nbytes / avg / 1e6, 1),
             "pct_hbm_peak": round(nbytes / avg / 1e6 / HBM_PEAK_GBS * 100, 2),
             "c_abi_ms": ref_ms, "vs_c_abi": round(avg / ref_ms, 4) if ref_ms else None,
             "settling_launches": settled}
        log(f"  {name:28s} {avg:9.4f} ms  {d['GBps']:8.1f} GB/s  {d['pct_hbm_peak']:6.2f}% of peak"
            f"  ({d['vs_c_abi']} x the C-ABI line)")
        res.append(d)

    def c_abi(name, key="avg_ms"):
        d = by_name.get(name)
        return d.get(key) if d else None

    log("through the dispatcher (device=\"webgpu\") ...")
    a_h, b_h = W.add_contiguous(n, seed=0)
    a, b = a_h.to("webgpu"), b_h.to("webgpu")
    del a_h, b_h
    line("add", lambda: a + b, 12 * n, c_abi("add"))
    line("eq", lambda: torch.eq(a, b), 9 * n, c_abi("eq"))
    del b
    x = x_h.view(rows, cols).to("webgpu")
    line("gelu", lambda: F.gelu(x), 8 * n, c_abi("gelu"))
    line("silu", lambda: F.silu(x), 8 * n, c_abi("silu"))
    del x
    # config 3b built on the device: as_strided view with transposed strides + contiguous tensor
    r3 = 1 << (args.log2n // 2 - 1)
    c3 = n // r3
    at = torch.as_strided(a.view(r3, c3), (c3, r3), (1, c3))
    c = src_h.view(c3, r3).to("webgpu")
    line("add_transposed", lambda: at + c, 12 * n, c_abi("add_transposed"))
    del at, a, c
    src, m = src_h.to("webgpu"), m_h.to("webgpu")
    note_ms("dispatcher masked_select_p0.50")
    got = torch.masked_select(src, m)
    if got.numel() != k50:
        raise RuntimeError(f"dispatcher masked_select: {got.numel()} != {k50}")
    del got
    def ms_call():
        note_ms("dispatcher masked_select_p0.50")
        return torch.masked_select(src, m)

    line("masked_select_p0.50", ms_call, W.masked_select_bytes(n, k50),
         c_abi("masked_select_p0.50", "op_ms_with_count_readback"))
    del src, m
    res.append(small_call_latency(torch, F))
    return res


def small_call_latency(torch, F):
    """What one call costs the host on tensors too small for the GPU to matter (1024 floats; 4 KiB
    for the upload): microseconds per call over 2000 calls issued back to back, and the same
    with the queue drained at the end (equal when the GPU keeps up with the host)."""
    a = torch.randn(1024).to("webgpu")
    b = torch.randn(1024).to("webgpu")
    o = torch.empty_like(a)
    m = (torch.randn(1024) > 0).to("webgpu")
    h = torch.randn(1024)
    one = a[:1]

    def drain():
        one.cpu()  # a read of four bytes is the sync point

    out = {}
    for name, fn, reps in (("add", lambda: a + b, 2000), ("add_out", lambda: torch.add(a, b, out=o), 2000),
                           ("gelu", lambda: F.gelu(a), 2000), ("eq", lambda: torch.eq(a, b), 2000),
                           ("empty", lambda: torch.empty(1024, device="webgpu"), 2000),
                           ("as_strided", lambda: a.as_strided((512,), (2,)), 2000),
                           ("masked_select_with_count", lambda: torch.masked_select(a, m), 500),
                           ("upload_4KiB", lambda: o.copy_(h), 2000),
                           ("read_4_bytes", lambda: one.cpu(), 1000), ("item", lambda: one.item(), 1000)):
        for _ in range(100):
            fn()
        drain()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        t1 = time.perf_counter()
        drain()
        t2 = time.perf_counter()
        out[name] = {"host_us": round((t1 - t0) / reps * 1e6, 2), "drained_us": round((t2 - t0) / reps * 1e6, 2)}
    log("  host microseconds per call on 1024-element tensors: " +
        ", ".join(f"{k} {v['host_us']}" for k, v in out.items()))
    return {"op": "small_call_latency", "elements": 1024, "us_per_call": out}


def first_launches(capi, L, torch, n, launches=40):
    """Is the first pass over freshly allocated device memory slower?  Times `launches`
    consecutive gelu launches on n floats, each between its own pair of events, with the output
    (and input) buffer in different states.  Microseconds per launch, in launch order."""
    it = capi.dense_iter(n)
    series = []

    def run(label, din, dout):
        evs = [capi.Event() for _ in range(launches + 1)]
        evs[0].record()
        for i in range(launches):
            capi.check(L.twg_unary_f32(capi.UNARY_GELU_ERF, dout.ptr, din.ptr, ctypes.byref(it), None))
            evs[i + 1].record()
        evs[-1].sync()
        us = [round(evs[i].elapsed_ms(evs[i + 1]) * 1000) for i in range(launches)]
        log(f"  {label:64s} " + " ".join(str(x) for x in us))
        series.append({"state": label, "us": us})

    for rep in range(2):
        capi.check(L.twg_empty_cache())
        din = capi.DeviceBuffer(4 * n)
        capi.check(L.twg_fill_bytes(din.ptr, 0x3c, 4 * n, None))
        dout = capi.DeviceBuffer(4 * n)
        capi.sync()
        run(f"pass {rep}: output fresh from hipMalloc, never touched", din, dout)
        run(f"pass {rep}: the same buffers, next {launches} launches", din, dout)
        dout.free(); din.free()
        capi.check(L.twg_empty_cache())
        din = capi.DeviceBuffer(4 * n)
        capi.check(L.twg_fill_bytes(din.ptr, 0x3c, 4 * n, None))
        dout = capi.DeviceBuffer(4 * n)
        capi.check(L.twg_fill_bytes(dout.ptr, 0, 4 * n, None))
        capi.sync()
        run(f"pass {rep}: output fresh from hipMalloc, filled once", din, dout)
        dout.free()
        dout = capi.DeviceBuffer(4 * n)  # the block just freed, from the pool
        run(f"pass {rep}: output recycled by the pool", din, dout)
        time.sleep(2.0)
        run(f"pass {rep}: the same buffers after 2 s without GPU work", din, dout)
        dout.free(); din.free()
        capi.check(L.twg_empty_cache())
        din = capi.DeviceBuffer(4 * n)
        din.upload(torch.full((n,), 1.0))  # 20 ms of DMA, no kernels
        dout = capi.DeviceBuffer(4 * n)
        run(f"pass {rep}: input written by an upload only, output fresh", din, dout)
        dout.free(); din.free()
        capi.check(L.twg_empty_cache())
        din, dout = capi.DeviceBuffer(4 * n), capi.DeviceBuffer(4 * n)
        run(f"pass {rep}: input and output fresh, right after the previous series", din, dout)
        dout.free(); din.free()
    return {"first_launches": series, "elements": n, "kernel": "ew_contig<GeluErfOp>", "unit": "us per launch"}


def op_chain(capi, L):
    """t1 = gelu(x); t2 = t1 + y; t3 = relu(t2); t1 = t3 * t2; t2 = silu(t1) on dense fp32 tensors of
    2^21 .. 2^26 elements: what an op's result being (or not being) in the last-level cache is worth
    to the op that consumes it.  x and y come in turn from four sets, so only the intermediates
    can be found cached.  Microseconds per chain over 40 chains between one pair of events."""
    rows = []
    for log2n in range(21, 27):
        n = 1 << log2n
        it = capi.dense_iter(n)
        pairs = [(capi.DeviceBuffer(4 * n), capi.DeviceBuffer(4 * n)) for _ in range(4)]
        for x, y in pairs:
            capi.check(L.twg_fill_bytes(x.ptr, 0x3c, 4 * n, None))
            capi.check(L.twg_fill_bytes(y.ptr, 0x3c, 4 * n, None))
        t1, t2, t3 = capi.DeviceBuffer(4 * n), capi.DeviceBuffer(4 * n), capi.DeviceBuffer(4 * n)
        one = ctypes.c_float(1.0)

        def chain(i):
            x, y = pairs[i % 4]
            capi.check(L.twg_unary_f32(capi.UNARY_GELU_ERF, t1.ptr, x.ptr, ctypes.byref(it), None))
            capi.check(L.twg_add_f32(t2.ptr, t1.ptr, y.ptr, one, ctypes.byref(it), None))
            capi.check(L.twg_unary_f32(capi.UNARY_RELU, t3.ptr, t2.ptr, ctypes.byref(it), None))
            capi.check(L.twg_mul_f32(t1.ptr, t3.ptr, t2.ptr, ctypes.byref(it), None))
            capi.check(L.twg_unary_f32(capi.UNARY_SILU, t2.ptr, t1.ptr, ctypes.byref(it), None))
        for i in range(4):
            chain(i)
        capi.sync()
        e0, e1 = capi.Event(), capi.Event()
        e0.record()
        for i in range(40):
            chain(i)
        e1.record()
        capi.sync()
        ms = e0.elapsed_ms(e1) / 40
        nbytes = (8 + 12 + 8 + 12 + 8) * n
        rows.append({"log2_elements": log2n, "tensor_MiB": 4 * n >> 20, "chain_us": round(ms * 1e3, 1),
                     "GBps": round(nbytes / ms / 1e6), "pct_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBS * 100, 1)})
        log(f"  2^{log2n}: {rows[-1]['chain_us']} us per chain, {rows[-1]['pct_hbm_peak']}% of HBM peak on algorithmic bytes")
        for x, y in pairs:
            x.free(); y.free()
        t1.free(); t2.free(); t3.free()
    return {"op_chain": rows, "ops": "gelu, add, relu, mul, silu", "bytes_per_element": 48}


def geometry_families(capi, L):
    """add.Tensor on ~2^25 fp32 elements with (a) the second operand broadcast in every possible
    way over a set of 2- to 4-dimensional shapes, (b) the first operand stored in every
    permutation of its dimensions and (c) one or both operands slices of a larger storage; and
    (d) copies of permuted tensors of 1-, 2- and 8-byte elements (twg_copy_strided).  Reports algorithmic bytes / time as % of the HBM peak: the
    slowest patterns and the median of each family.  Median of three batches of 12 launches,
    each batch between one pair of events on the library's stream, consecutive launches on
    three sets of operands in turn."""
    import itertools

    def contig(shape):
        st, acc = [], 1
        for s in reversed(shape):
            st.append(acc)
            acc *= s
        return list(reversed(st))

    # Consecutive launches go to three different sets of operands in turn: at this size one set
    # is 400 MB, and launched again and again on the same set, a kernel that reads an operand
    # with default caching finds a good part of it in the 256 MB last-level cache the launch
    # before left there (a reversed [128,56,56,96] operand: 83% of "HBM peak" on one set, 65%
    # in rotation; kernels whose loads carry the nontemporal hint read the same either way).
    kSets = 3

    launches = [0]  # patterns timed so far: a kernel trace of this sweep tells them apart by it

    def median_launch_seconds(run):
        launches[0] += 1
        for i in range(kSets):
            run(i)
        capi.sync()
        batches = []
        for _ in range(3):  # median of three batches of 12 launches between one event pair
            e0, e1 = capi.Event(), capi.Event()
            e0.record()
            for i in range(12):
                run(i % kSets)
            e1.record()
            capi.sync()
            batches.append(e0.elapsed_ms(e1) / 12)
        return statistics.median(batches) / 1e3

    def timed(shape, a_st, b_st, nb):
        n = 1
        for s in shape:
            n *= s
        sets = [(capi.DeviceBuffer(4 * n), capi.DeviceBuffer(4 * max(nb, 1)), capi.DeviceBuffer(4 * n))
                for _ in range(kSets)]
        it = capi.make_iter(shape, contig(shape), a_st, b_st)

        def run(i):
            da, db, do = sets[i]
            capi.check(L.twg_add_f32(do.ptr, da.ptr, db.ptr, ctypes.c_float(1.0), ctypes.byref(it), None))
        t = median_launch_seconds(run)
        return round((8 * n + 4 * nb) / t / 1e9 / HBM_PEAK_GBS * 100, 1), round(t * 1e3, 4)

    fam = {}
    rows_ = []
    for shape in ([2048, 256, 7, 7], [512, 256, 14, 14], [128, 64, 56, 56], [32, 16, 1024, 64],
                  [32, 16, 256, 256], [16, 2048, 1000], [256, 197, 768], [5792, 5792], [512, 768, 3, 27],
                  [256, 224, 224, 3]):
        for keep in itertools.product((True, False), repeat=len(shape)):
            if all(keep) or not any(keep):
                continue
            bshape = [s if k else 1 for s, k in zip(shape, keep)]
            b_st = [st if k else 0 for st, k in zip(contig(bshape), keep)]
            nb = 1
            for s in bshape:
                nb *= s
            pct, ms = timed(shape, contig(shape), b_st, nb)
            rows_.append({"pct_hbm_peak": pct, "ms": ms, "a": shape, "b": bshape, "launch_order": launches[0]})
    rows_.sort(key=lambda r: r["pct_hbm_peak"])
    fam["broadcast_second_operand"] = {"patterns": len(rows_), "median_pct": rows_[len(rows_) // 2]["pct_hbm_peak"],
                                       "slowest": rows_[:5], "all": rows_}
    log(f"broadcast family: {len(rows_)} patterns, median {rows_[len(rows_) // 2]['pct_hbm_peak']}%, "
        f"slowest {rows_[0]['pct_hbm_peak']}%")
    rows_ = []
    for shape in ([32, 16, 1024, 64], [64, 128, 64, 64], [256, 197, 768], [512, 3, 224, 96], [128, 56, 56, 96],
                  [256, 224, 224, 3]):
        nd = len(shape)
        n = 1
        for s in shape:
            n *= s
        for perm in itertools.permutations(range(nd)):
            if list(perm) == list(range(nd)):
                continue
            phys = contig([shape[p] for p in perm])
            a_st = [0] * nd
            for pos, p in enumerate(perm):
                a_st[p] = phys[pos]
            pct, ms = timed(shape, a_st, contig(shape), n)
            rows_.append({"pct_hbm_peak": pct, "ms": ms, "shape": shape, "a_memory_order": list(perm),
                          "launch_order": launches[0]})
    rows_.sort(key=lambda r: r["pct_hbm_peak"])
    fam["permuted_first_operand"] = {"patterns": len(rows_), "median_pct": rows_[len(rows_) // 2]["pct_hbm_peak"],
                                     "slowest": rows_[:5], "all": rows_}
    log(f"permutation family: {len(rows_)} patterns, median {rows_[len(rows_) // 2]['pct_hbm_peak']}%, "
        f"slowest {rows_[0]['pct_hbm_peak']}%")
    # (c) the first operand a slice of a larger storage: stepped, shifted or narrowed along one
    # dimension or all of them (x[:, ::2], x[1:], x[:, :, 3:-2] ...), the second operand and the
    # output contiguous; and both operands sliced alike
    def timed_view(shape, storage, starts, steps, both):
        n = 1
        for s_ in shape:
            n *= s_
        ns = 1
        for s_ in storage:
            ns *= s_
        st_storage = contig(storage)
        a_st = [st * k for st, k in zip(st_storage, steps)]
        off = sum(b0 * st for b0, st in zip(starts, st_storage))
        sets = [(capi.DeviceBuffer(4 * ns), capi.DeviceBuffer(4 * (ns if both else n)), capi.DeviceBuffer(4 * n))
                for _ in range(kSets)]
        b_st = a_st if both else contig(shape)
        it = capi.make_iter(shape, contig(shape), a_st, b_st)

        def run(i):
            da, db, do = sets[i]
            capi.check(L.twg_add_f32(do.ptr, da.ptr + 4 * off, db.ptr + (4 * off if both else 0),
                                     ctypes.c_float(1.0), ctypes.byref(it), None))
        t = median_launch_seconds(run)
        return round(12 * n / t / 1e9 / HBM_PEAK_GBS * 100, 1), round(t * 1e3, 4)

    rows_ = []
    for shape in ([4096, 8192], [64, 512, 1024], [32, 16, 256, 256], [8192, 4000]):
        nd = len(shape)
        variants = []
        for d in sorted({0, nd // 2, nd - 1}):
            for step in (2, 3):
                storage = list(shape)
                storage[d] *= step
                steps = [1] * nd
                steps[d] = step
                variants.append((f"dim {d} stepped by {step}", storage, [0] * nd, steps))
            for pad in (1, 5, 32):
                storage = list(shape)
                storage[d] += pad
                starts = [0] * nd
                starts[d] = pad if pad == 1 else 0
                variants.append((f"dim {d} of {storage[d]} " + ("from 1 on" if pad == 1 else f"narrowed by {pad}"),
                                 storage, starts, [1] * nd))
        variants.append(("every dim from 1 on, to the last but one", [s_ + 2 for s_ in shape], [1] * nd, [1] * nd))
        for what, storage, starts, steps in variants:
            for both in (False, True):
                pct, ms = timed_view(shape, storage, starts, steps, both)
                rows_.append({"pct_hbm_peak": pct, "ms": ms, "shape": shape, "slice": what,
                              "operands_sliced": "both" if both else "first", "launch_order": launches[0]})
    rows_.sort(key=lambda r: r["pct_hbm_peak"])
    fam["sliced_operands"] = {"patterns": len(rows_), "median_pct": rows_[len(rows_) // 2]["pct_hbm_peak"],
                              "slowest": rows_[:5], "all": rows_}
    log(f"slice family: {len(rows_)} patterns, median {rows_[len(rows_) // 2]['pct_hbm_peak']}%, "
        f"slowest {rows_[0]['pct_hbm_peak']}%")
    # (d) copies (what .contiguous() runs) of permuted tensors whose elements are not 4 bytes
    # wide: bool masks, half / bfloat16, int64 / float64.  Bytes: 2 x the element size per element.
    def timed_copy(shape, a_st, es):
        n = 1
        for s_ in shape:
            n *= s_
        sets = [(capi.DeviceBuffer(es * n), capi.DeviceBuffer(es * n)) for _ in range(kSets)]
        it = capi.make_iter(shape, contig(shape), a_st)

        def run(i):
            da, do = sets[i]
            capi.check(L.twg_copy_strided(do.ptr, da.ptr, es, ctypes.byref(it), None))
        t = median_launch_seconds(run)
        return round(2 * es * n / t / 1e9 / HBM_PEAK_GBS * 100, 1), round(t * 1e3, 4)

    rows_ = []
    for es in (1, 2, 8):
        for shape, perm in (([8192, 4096], [1, 0]), ([16384, 8192], [1, 0]), ([128, 56, 56, 96], [0, 3, 1, 2]),
                            ([256, 224, 224, 3], [0, 3, 1, 2]), ([256, 197, 768], [0, 2, 1]),
                            ([64, 128, 64, 64], [0, 2, 1, 3]), ([2048, 96, 192], [0, 2, 1])):
            nd = len(shape)
            phys = contig([shape[p_] for p_ in perm])
            a_st = [0] * nd
            for pos, p_ in enumerate(perm):
                a_st[p_] = phys[pos]
            pct, ms = timed_copy(shape, a_st, es)
            rows_.append({"pct_hbm_peak": pct, "ms": ms, "shape": shape, "a_memory_order": perm,
                          "element_bytes": es, "launch_order": launches[0]})
    rows_.sort(key=lambda r: r["pct_hbm_peak"])
    fam["permuted_copies_of_1_2_8_byte_elements"] = {
        "patterns": len(rows_), "median_pct": rows_[len(rows_) // 2]["pct_hbm_peak"], "slowest": rows_[:5],
        "all": rows_}
    log(f"copies of 1-, 2- and 8-byte elements: {len(rows_)} patterns, median "
        f"{rows_[len(rows_) // 2]['pct_hbm_peak']}%, slowest {rows_[0]['pct_hbm_peak']}%")
    return {"geometry_families": fam, "elements_per_pattern": "about 2^25", "op": "add.Tensor fp32",
            "operand_sets_in_rotation": kSets,
            "launches_per_pattern": kSets + 3 * 12,
            "bytes": "4 B per element read per full operand + 4 B written; a broadcast operand counts its own size; "
                     "a stepped operand counts the elements used, not the lines touched; the copies of the last family "
                     "(twg_copy_strided, not add) move 2 x their element size per element"}


def sweep(args, capi, W, L, torch, n, rows, cols, K, Wm, time_launches, summarize,
          d_out, d_cnt, d_scratch, scratch_bytes, d_src, d_x, it, cnt_host, want):
    f32 = ctypes.c_float
    res = []
    by = W.BYTES_PER_ELEM

    # config 2: silu, relu on the gelu input
    for name, op in (("copy", capi.UNARY_COPY), ("silu", capi.UNARY_SILU), ("relu", capi.UNARY_RELU),
                     ("gelu_tanh", capi.UNARY_GELU_TANH)):
        if want(name):
            ms = time_launches(lambda: capi.check(L.twg_unary_f32(op, d_out.ptr, d_x.ptr,
                                                                   ctypes.byref(it), None)), Wm, K)
            res.append(summarize(name, f"ew_contig<{name}>", 8 * n, ms, n))

    # config 3: row-bias add and transposed add
    if want("add_rowbias") or want("add_transposed"):
        r3, c3 = (1 << (args.log2n // 2 - 1)), 0
        c3 = n // r3  # 8192 x 32768 at 2^28
        a_h, bias_h, c_h = W.broadcast_add_inputs(r3, c3, seed=2)
        d_a3, d_bias, d_c3 = capi.to_device(a_h), capi.to_device(bias_h), capi.to_device(c_h)
        del a_h, c_h
        if want("add_rowbias"):
            it_rb = capi.make_iter((r3, c3), (c3, 1), (c3, 1), (0, 1))
            ms = time_launches(lambda: capi.check(L.twg_add_f32(d_out.ptr, d_a3.ptr, d_bias.ptr, f32(1.0),
                                                                ctypes.byref(it_rb), None)), Wm, K)
            res.append(summarize("add_rowbias", "ew_rows<AddOp>", by["add_rowbias"] * n + 4 * c3, ms, n,
                                 {"shape": [r3, c3]}))
        if want("add_transposed"):
            # A viewed as (c3, r3) with strides (1, c3) + contiguous C[c3, r3]; at::TensorIterator
            # gives the output the first input's layout, so dimension 0 of the iterator is the
            # logical dimension 0 (stride 1 for out and A, stride r3 for C).
            it_t = capi.Iter()
            it_t.ndim = 2
            it_t.numel = n
            it_t.shape[0], it_t.shape[1] = c3, r3
            for slot, st in ((capi.OUT, (1, c3)), (capi.A, (1, c3)), (capi.B, (r3, 1))):
                it_t.stride[slot][0], it_t.stride[slot][1] = st
            ms = time_launches(lambda: capi.check(L.twg_add_f32(d_out.ptr, d_a3.ptr, d_c3.ptr, f32(1.0),
                                                                ctypes.byref(it_t), None)), Wm, K)
            res.append(summarize("add_transposed", "ew_tile_vec<AddOp,256,32>", by["add_transposed"] * n, ms, n,
                                 {"logical_shape": [c3, r3], "out_strides": [1, c3]}))
        del d_a3, d_bias, d_c3

    # config 4: eq, ne.Scalar, bitwise_and
    if any(want(k) for k in ("eq", "ne_scalar", "bitwise_and", "cast_bool_f32", "cast_f32_f16")):
        p_h, q_h, z_h = W.mask_inputs(n, seed=3)
        d_p, d_q, d_z = capi.to_device(p_h), capi.to_device(q_h), capi.to_device(z_h)
        del p_h, q_h, z_h
        d_m1, d_m2, d_m3 = capi.DeviceBuffer(n), capi.DeviceBuffer(n), capi.DeviceBuffer(n)
        # A bool output of 2^28 elements is 256 MiB, the size of the last-level (Infinity)
        # cache: launched again and again into the same buffer, the kernel writes lines that
        # are still resident.  Each of these three is therefore also timed with its output
        # rotating over three buffers (`pct_hbm_peak_rotating_outputs`), which is what a call
        # whose result lands in memory not touched recently sees.
        spare = [capi.DeviceBuffer(n), capi.DeviceBuffer(n)]

        def rotating(call, first):
            outs = [first] + spare
            state = {"i": 0}

            def fn():
                o = outs[state["i"] % 3]
                state["i"] += 1
                call(o)
            ms_r = time_launches(fn, Wm + 3, K)
            return ms_r.batch_avg

        def mask_line(name, kernel, nbytes, call, first):
            ms = time_launches(lambda: call(first), Wm, K)
            t_rot = rotating(call, first)
            res.append(summarize(name, kernel, nbytes, ms, n, {
                "avg_ms_rotating_outputs": round(t_rot, 5),
                "pct_hbm_peak_rotating_outputs": round(nbytes / t_rot / 1e6 / HBM_PEAK_GBS * 100, 2)}))

        mask_line("eq", "ew_contig<EqOp>", by["eq"] * n,
                  lambda o: capi.check(L.twg_eq_f32(o.ptr, d_p.ptr, d_q.ptr, ctypes.byref(it), None)), d_m1)
        mask_line("ne_scalar", "ew_contig<NeScalarOp>", by["ne_scalar"] * n,
                  lambda o: capi.check(L.twg_ne_scalar_f32(o.ptr, d_z.ptr, f32(0.0), ctypes.byref(it), None)), d_m2)
        # leave the masks of the parity configuration in d_m1 / d_m2 for bitwise_and
        capi.check(L.twg_eq_f32(d_m1.ptr, d_p.ptr, d_q.ptr, ctypes.byref(it), None))
        capi.check(L.twg_ne_scalar_f32(d_m2.ptr, d_z.ptr, f32(0.0), ctypes.byref(it), None))
        mask_line("bitwise_and", "ew_contig<AndOp>", by["bitwise_and"] * n,
                  lambda o: capi.check(L.twg_and_u8(o.ptr, d_m1.ptr, d_m2.ptr, ctypes.byref(it), None)), d_m3)
        del spare
        # dtype conversion of a mask (mask.float()) and of fp32 data (x.half()): 5 and 6 B/element
        if want("cast_bool_f32"):
            ms = time_launches(lambda: capi.check(L.twg_cast(d_out.ptr, capi.DTYPES[torch.float32], d_m1.ptr,
                                                             capi.DTYPES[torch.bool], ctypes.byref(it), None)), Wm, K)
            res.append(summarize("cast_bool_f32", "ew_contig<CastOp<float,bool>>", 5 * n, ms, n))
        if want("cast_f32_f16"):
            ms = time_launches(lambda: capi.check(L.twg_cast(d_out.ptr, capi.DTYPES[torch.float16], d_z.ptr,
                                                             capi.DTYPES[torch.float32], ctypes.byref(it), None)), Wm, K)
            res.append(summarize("cast_f32_f16", "ew_contig<CastOp<half,float>>", 6 * n, ms, n))
        del d_p, d_q, d_z, d_m1, d_m2, d_m3

    # config 5: the other masks
    # (p = 0.05 / 0.1 / 0.25 sit around the density, one selected element in 16 per wavefront,
    # at which a wavefront switches from gathering to streaming; the alternating mask has
    # 8192-element spans at 1% and 90% in turn, so both kinds of wavefront share every tile)
    for name, make in (("masked_select_p0.01", lambda: W.bernoulli_mask(n, 0.01)),
                       ("masked_select_p0.05", lambda: W.bernoulli_mask(n, 0.05)),
                       ("masked_select_p0.10", lambda: W.bernoulli_mask(n, 0.10)),
                       ("masked_select_p0.25", lambda: W.bernoulli_mask(n, 0.25)),
                       ("masked_select_p0.99", lambda: W.bernoulli_mask(n, 0.99)),
                       ("masked_select_clustered", lambda: W.clustered_mask(n, 4096)),
                       ("masked_select_alternating", lambda: W.alternating_density_mask(n, 8192, 0.01, 0.9))):
        if not want(name):
            continue
        m_h = make()
        k = int(m_h.sum())
        d_mask = capi.to_device(m_h)
        del m_h

        def launch(name=name):
            note_ms(name)
            capi.check(L.twg_masked_select_f32(d_out.ptr, d_cnt.ptr, d_src.ptr, d_mask.ptr,
                                               ctypes.byref(it), d_scratch.ptr, scratch_bytes, None))

        k_host = ctypes.c_int64(-1)

        def full(name=name):
            note_ms(name)
            capi.check(L.twg_masked_select_count(d_out.ptr, ctypes.byref(k_host), d_src.ptr, 4,
                                                 d_mask.ptr, ctypes.byref(it), d_scratch.ptr,
                                                 scratch_bytes, None))

        ms_kernel = time_launches(launch, Wm, K)
        ms_full = time_launches(full, 1, K)
        if k_host.value != k:
            raise RuntimeError(f"{name}: count {k_host.value} != {k}")
        res.append(summarize(name, "ms_compact_stream<16,4>", W.masked_select_bytes(n, k), ms_kernel, n,
                             {"selected": k, "op_ms_with_count_readback": round(ms_full.batch_avg, 5)}))
        del d_mask
    return res


def config1(capi, W, L, torch, time_launches, Wm, K):
    """The 2^20-element add with its copies up and down: too small for an HBM figure (it
    fits the caches), so it is reported as launch latency and host-link rates."""
    n1 = 1 << 20
    a_h, b_h = W.add_contiguous(n1, seed=0)
    d_a, d_b, d_o = capi.to_device(a_h), capi.to_device(b_h), capi.DeviceBuffer(4 * n1)
    it1 = capi.dense_iter(n1)
    ms = time_launches(lambda: capi.check(L.twg_add_f32(d_o.ptr, d_a.ptr, d_b.ptr, ctypes.c_float(1.0),
                                                        ctypes.byref(it1), None)), Wm, K)
    back = torch.empty(n1)
    reps = 20

    def wall(fn):
        """Median wall time of one copy, device side finished (a mean over the repetitions
        would carry every scheduling hiccup of the host)."""
        ts = []
        for i in range(reps + 3):
            capi.sync()
            t = time.perf_counter()
            fn()
            capi.sync()
            if i >= 3:
                ts.append(time.perf_counter() - t)
        return statistics.median(ts)

    t_up = wall(lambda: d_a.upload(a_h))
    t_down = wall(lambda: capi.check(L.twg_memcpy_d2h(back.data_ptr(), d_o.ptr, 4 * n1, None)))
    if not torch.equal(back, a_h + b_h):
        raise RuntimeError("config 1: add result differs from the CPU sum")
    d = {"elements": n1, "add_kernel_us": round(statistics.median(ms) * 1e3, 2),
         "h2d_4MiB_us": round(t_up * 1e6, 1), "h2d_GBps": round(4 * n1 / t_up / 1e9, 2),
         "d2h_4MiB_us": round(t_down * 1e6, 1), "d2h_GBps": round(4 * n1 / t_down / 1e9, 2),
         "note": "pageable host memory through the pinned ring (up: DMA per piece, down: streamed by workgroups); median of single copies; result equals the CPU sum"}
    log(f"  config 1 (2^20): add {d['add_kernel_us']} us, H2D {d['h2d_GBps']} GB/s, D2H {d['d2h_GBps']} GB/s")
    return d


def cpu_baseline(torch, W, n, x_h, src_h, m_h, step_bytes, bytes_add, bytes_gelu, bytes_ms):
    """Times the same three ops on the host: (a) the C oracle, one thread, on samples;
    (b) PyTorch's CPU kernels on all cores at full size."""
    from oracle import oracle
    import torch.nn.functional as F

    OL = oracle.lib()
    # about 10 s of single-thread work in total (gelu through libm erfc dominates)
    ns_add = min(n, 1 << 27)
    ns_gelu = min(n, 1 << 27)
    ns_ms = min(n, 1 << 27)
    a = torch.rand(ns_add) * 8 - 4
    b = torch.rand(ns_add) * 8 - 4
    o = torch.empty(ns_add)

    def best(fn, reps=3):
        ts = []
        for _ in range(reps):
            t = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t)
        return statistics.median(ts)

    log("CPU baseline: C oracle, 1 thread ...")
    t_add = best(lambda: OL.oracle_dense_add_f32(o.data_ptr(), a.data_ptr(), b.data_ptr(), 1.0, ns_add))
    xs = x_h[:ns_gelu].contiguous()
    og = torch.empty(ns_gelu)
    t_gelu = best(lambda: OL.oracle_dense_unary_f32(oracle.GELU_ERF, og.data_ptr(), xs.data_ptr(), ns_gelu))
    ss, msk = src_h[:ns_ms].contiguous(), m_h[:ns_ms].contiguous()
    om = torch.empty(ns_ms)
    t_ms = best(lambda: OL.oracle_dense_masked_select_f32(om.data_ptr(), ss.data_ptr(), msk.data_ptr(), ns_ms))
    g_add = 12 * ns_add / t_add / 1e9
    g_gelu = 8 * ns_gelu / t_gelu / 1e9
    g_ms = (5 * ns_ms + 4 * int(msk.sum())) / t_ms / 1e9
    step_s = bytes_add / g_add / 1e9 + bytes_gelu / g_gelu / 1e9 + bytes_ms / g_ms / 1e9
    port = {"add_GBps": round(g_add, 2), "gelu_GBps": round(g_gelu, 3), "masked_select_GBps": round(g_ms, 2)}

    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    log(f"CPU baseline: PyTorch CPU kernels, {threads} threads ...")
    nt = n  # the full configuration
    a = torch.rand(nt) * 8 - 4
    b = torch.rand(nt) * 8 - 4
    o = torch.empty(nt)
    xt, st, mt = x_h[:nt], src_h[:nt], m_h[:nt]
    ta = best(lambda: torch.add(a, b, out=o), 5)
    tg = best(lambda: F.gelu(xt), 5)
    tm = best(lambda: torch.masked_select(st, mt), 5)
    kt = int(mt.sum())
    ga, gg, gm = 12 * nt / ta / 1e9, 8 * nt / tg / 1e9, (5 * nt + 4 * kt) / tm / 1e9
    # the other ops of the sweep, same inputs as the GPU side, same bytes-per-element figures
    others = {}
    others["silu_GBps"] = round(8 * nt / best(lambda: F.silu(xt)) / 1e9, 2)
    others["relu_GBps"] = round(8 * nt / best(lambda: torch.relu(xt)) / 1e9, 2)
    del a, b, o
    p_h, q_h, z_h = W.mask_inputs(nt, seed=3)
    others["eq_GBps"] = round(9 * nt / best(lambda: torch.eq(p_h, q_h)) / 1e9, 2)
    others["ne_scalar_GBps"] = round(5 * nt / best(lambda: z_h.ne(0.0)) / 1e9, 2)
    m1, m2 = torch.eq(p_h, q_h), z_h.ne(0.0)
    others["bitwise_and_GBps"] = round(3 * nt / best(lambda: torch.bitwise_and(m1, m2)) / 1e9, 2)
    del p_h, q_h, z_h, m1, m2
    step_t = bytes_add / ga / 1e9 + bytes_gelu / gg / 1e9 + bytes_ms / gm / 1e9
    try:
        with open("/proc/cpuinfo") as f:
            model = [l.split(":", 1)[1].strip() for l in f if l.startswith("model name")][0]
    except Exception:
        model = "unknown"
    # The reference's CPU path is ATen's CPU kernels: its boxed fallback runs them for eq, ne,
    # bitwise_and and masked_select (csrc/bindings.cpp:27-43), and they are the stated baseline
    # for every op here.  The single-threaded C restatement of the WGSL arithmetic is nested.
    return {
        "value": round(step_bytes / step_t / 1e9, 2), "unit": "GB/s", "cores": threads,
        "kind": "reference_cpu", "cpu_model": model,
        "sample": f"ATen CPU kernels (torch.add, F.gelu, torch.masked_select) on 2^{nt.bit_length() - 1} "
                  f"elements each, {threads} threads, median of 5; per-op GB/s combined into the "
                  "time of one step",
        "per_op": dict({"add_GBps": round(ga, 2), "gelu_GBps": round(gg, 2),
                        "masked_select_GBps": round(gm, 2)}, **others),
        "c_port": {
            "value": round(step_bytes / step_s / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"oracle/twg_oracle.c, 1 thread: add on 2^{ns_add.bit_length() - 1}, gelu on "
                      f"2^{ns_gelu.bit_length() - 1}, masked_select on 2^{ns_ms.bit_length() - 1} "
                      "elements, median of 3",
            "per_op": port,
        },
    }


if __name__ == "__main__":
    main()

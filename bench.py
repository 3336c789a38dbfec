#!/usr/bin/env python3
"""Headline benchmark: one rank's 8-partial reduce + residual + RMSNorm + per-token fp8 quant stage
at 2048 x 8192 bf16 (the headline configuration, here called c3) on ONE MI355X, through the C ABI (tde_reduce_rms).

A step is one launch of the fused row kernel over one batch of synthetic inputs that already sit
in HBM.  Inputs and outputs rotate over enough distinct sets (> 4 GiB of inputs, > 1 GiB of
outputs) that the 256 MB memory-side cache neither serves a launch's reads nor absorbs its writes.
The first set is drawn on the CPU from the configuration's seed (the same tensors the parity tests use); the
CPU-baseline leg runs the oracle on it and compares the kernel's outputs for that set bit for bit.
Before the W warm-up steps the same step runs untimed for about 20 ms (--settle-ms): a device that has been idle
runs its first 10-20 ms under load differently from everything after (c3 1 % slower, c5 up to 14 %).
Two clocks, both in the line: `value` / `ms_per_step` are the host's wall clock around the K launches and the
synchronization that ends them; `roofline.achieved` / `frac` / `kernel_avg_us` are HIP events recorded on the launch
stream around the same K launches.  Two states, both in the line: `roofline.cold_kernel_avg_us` is the same
measurement (W warm-up launches, K timed) taken before the settling phase, `kernel_avg_us` after it.
`roofline.fit` times the same kernel at three row counts and reports the straight line through them
(`fixed_us` + bytes / `bulk_GBs`); `roofline.device_rates_floor` is what the device's own plain read, write and copy
rates, measured in the same process, make of the launch's bytes.
Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c3] [--no-cpu-baseline] [--settle-ms 20]
    python bench.py --config custom --nranks 8 --tokens 2048 --hidden 4096 --dtype f32 --quant none
"""
import argparse
import ctypes
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E published peak

# HBM bytes per launch, measured with two rocprofv3 counter runs of this script per configuration (--pmc FETCH_SIZE,
# then --pmc WRITE_SIZE; KiB per dispatch of the row kernel), each scaled by what the same counter reads for the three
# 256 MiB calibration copies this script dispatches before its warm-up (FETCH_SIZE reads half the bytes on this part).
# They describe the kernels whose sources hash to `sources_sha256`; with any other kernel source the bench line reports
# traffic as null.
TRAFFIC = {
    "sources_sha256": "55bb90777cf227977d0f7689232b58b52ca6a471a27da75b4f630d2904ba9706",
    "bytes": {"c2": 11693631, "c3": 352653693, "c4": 765467842, "c5": 2181249484},
}

BENCH_CONFIGS = {
    # name: (N, T, H, dtype, sigma, eps, quant, seed, outlier_channels)
    "c2": (8, 128, 4096, "bf16", 0.5, 1e-5, "none", 2, 0),
    "c3": (8, 2048, 8192, "bf16", 0.5, 1e-5, "fp8_token", 3, 0),
    "c4": (4, 8192, 7168, "bf16", 1.0, 1e-6, "fp8_group", 4, 0),
    "c5": (4, 32768, 5120, "f16", 1.0, 1e-6, "int8_token", 5, 5),
}


def kernel_sources_sha256():
    """One hash over the kernel sources, so that figures measured with other kernels are not reported for these."""
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "torch_dist_ext_amd", "csrc")
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".hip", ".h")):
            with open(os.path.join(csrc, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()


TORCH_DTYPES = {"bf16": "bfloat16", "f16": "float16", "f32": "float32", "f64": "float64"}
ELEM_BYTES = {"bf16": 2, "f16": 2, "f32": 4, "f64": 8}


def torch_dtype(torch, dt):
    return getattr(torch, TORCH_DTYPES[dt])


def seeded_cpu_inputs(torch, cfg):
    """The configuration's inputs drawn on the CPU from its seed: partials ~ N(0, sigma), residual ~ N(0, 1),
    gamma ~ U(0.5, 1.5), an optional fixed seeded set of outlier channels multiplied by 100 in every partial."""
    N, T, H, dt, sigma, eps, quant, seed, outliers = cfg
    dtype = torch_dtype(torch, dt)
    wide = torch.float64 if dt == "f64" else torch.float32
    g = torch.Generator().manual_seed(seed)
    parts = torch.randn((N, T, H), generator=g, dtype=wide) * sigma
    if outliers:
        cols = torch.randperm(H, generator=g)[:outliers]
        parts[:, :, cols] *= 100.0
    residual = torch.randn((T, H), generator=g, dtype=wide)
    gamma = torch.rand((H,), generator=g, dtype=wide) + 0.5
    return parts.to(dtype), residual.to(dtype), gamma.to(dtype)


def make_sets(torch, cfg, nsets, dev, first, rows=None):
    """nsets sets of device buffers of `rows` rows each (the configuration's own count if None); set 0 holds the
    seeded CPU inputs `first` when given."""
    N, T, H, dt, sigma, eps, quant, seed, outliers = cfg
    T = rows or T
    dtype = torch_dtype(torch, dt)
    g = torch.Generator(device=dev).manual_seed(1234)
    sets = []
    for k in range(nsets):
        if k == 0 and first is not None:
            parts = [first[0][r].to(dev) for r in range(N)]
            residual = first[1].to(dev)
        else:
            parts = [(torch.randn((T, H), generator=g, device=dev, dtype=torch.float32) * sigma).to(dtype) for _ in range(N)]
            residual = torch.randn((T, H), generator=g, device=dev, dtype=torch.float32).to(dtype)
        res_out = torch.empty_like(residual)
        q = torch.empty((T, H), dtype=torch.uint8, device=dev) if quant != "none" else None
        nscale = T * (H // 128) if quant == "fp8_group" else T
        scale = torch.empty((nscale,), dtype=torch.float32, device=dev) if quant != "none" else None
        norm = torch.empty_like(residual) if quant == "none" else None
        sets.append(dict(parts=parts, residual=residual, res_out=res_out, q=q, scale=scale, norm=norm))
    return sets


def cpu_baseline(torch, cfg, first, kernel_out, budget_s=15.0):
    """The oracle's torch-eager composition timed on the host cores, on a bounded sample: as many full-size
    passes over the configuration's seeded inputs (at most 2048 rows of them) as fit in about budget_s (at least
    2 after one warm-up).  The warm-up pass doubles as the checker of the kernel's outputs for the same rows."""
    from oracle import eager
    N, T, H, dt, sigma, eps, quant, seed, outliers = cfg
    cores = os.cpu_count() or 1
    threads = min(cores, 16)
    torch.set_num_threads(threads)
    rows = min(T, 2048)
    parts, residual, gamma = first[0][:, :rows].contiguous(), first[1][:rows].contiguous(), first[2]
    want = eager.reduce_rms(parts, residual, gamma, eps, quant)  # warm-up, and the expected outputs
    checked = {}
    for key, got in kernel_out.items():
        ref = want[key].reshape(rows, -1)
        g = got.reshape(T, -1)[:rows]
        same = bool(torch.equal(g.contiguous().view(torch.uint8), ref.contiguous().view(torch.uint8)))
        checked[key] = same
    times = []
    t_begin = time.perf_counter()
    while len(times) < 2 or (time.perf_counter() - t_begin < budget_s and len(times) < 50):
        t0 = time.perf_counter()
        eager.reduce_rms(parts, residual, gamma, eps, quant)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {
        "value": rows / med, "unit": "tokens/s", "cores": torch.get_num_threads(), "host_cpu_count": cores, "kind": "port",
        "sample": "%d passes of %d rows x %d (%s, N=%d, %s), median; torch-eager oracle on host CPU" % (
            len(times), rows, H, dt, N, quant),
        "ms_per_pass": med * 1e3,
        "kernel_outputs_bit_identical_to_oracle": checked,
    }


def operator_path_cost(torch, cfg, first, dev, calls=2000):
    """Host-side cost of the torch operator path (the reference's call sequence get_workspace -> allreduce_rms,
    test/test_all_reduce_fusion.py:55-59) on ONE set of buffers: microseconds per call of the functional operator back
    to back (whichever of host and kernel is slower shows), of the operator the reference registers in C++
    (outputs given), and of 20 calls captured in a HIP graph and replayed (kernel-bound)."""
    import torch_dist_ext_amd as tde
    N, T, H, dt, sigma, eps, quant, seed, outliers = cfg
    e = ELEM_BYTES[dt]
    tde.setup_env(0, N, max_size_in_bytes=T * H * e)
    x = first[0][0].to(dev)
    for r in range(1, N):
        tde.set_peer_partial(r, first[0][r].to(dev))
    res, gamma = first[1].to(dev), first[2].to(dev)
    ws = tde.get_workspace(x)
    mode = tde.QUANT_MODES[quant]
    if quant == "none":
        def op():
            return torch.ops.torch_dist_ext.allreduce_rms(0, N, x, res, gamma, eps, ws)
    else:
        def op():
            return torch.ops.torch_dist_ext.allreduce_rms_quant(0, N, x, res, gamma, eps, ws, mode, False)

    def per_call(fn, n):
        for _ in range(50):
            fn()
        torch.cuda.synchronize(dev)
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize(dev)
        return (time.perf_counter() - t0) * 1e6 / n

    out = {"calls": calls, "functional_op_us_per_call": per_call(op, calls),
           "get_workspace_plus_functional_op_us_per_call": per_call(lambda: (tde.get_workspace(x), op()), calls)}
    if quant == "none":
        n_out, r_out = torch.empty_like(x), torch.empty_like(res)
        out["out_variant_op_us_per_call"] = per_call(
            lambda: tde.allreduce_rms_fusion_impl(0, N, x, res, gamma, r_out, n_out, eps, ws), calls)
    side = torch.cuda.Stream(dev)
    with torch.cuda.stream(side):
        op()
        torch.cuda.synchronize(dev)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            kept = [op() for _ in range(20)]
        out["graph_replay_us_per_call"] = per_call(graph.replay, max(calls // 20, 10)) / 20
        del kept, graph
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="c3", choices=sorted(BENCH_CONFIGS) + ["custom"])
    ap.add_argument("--tokens", type=int, default=0,
                    help="rows, if not the configuration's own (c5 is quoted at 1, 64, 512, 4096 and 32768 rows)")
    ap.add_argument("--nranks", type=int, default=8, help="--config custom: partial buffers (2, 4, 8)")
    ap.add_argument("--hidden", type=int, default=4096, help="--config custom: row length")
    ap.add_argument("--dtype", default="bf16", choices=sorted(TORCH_DTYPES), help="--config custom: element type")
    ap.add_argument("--quant", default="none", choices=["none", "fp8_token", "fp8_group", "int8_token"], help="--config custom")
    ap.add_argument("--sets", type=int, default=0, help="distinct input sets to rotate over (0 = enough for > 1 GiB)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-fit", action="store_true", help="skip roofline.fit (the same kernel at three row counts)")
    ap.add_argument("--operator-path", action="store_true",
                    help="also time the torch operator path on one set of buffers (done for c2 unless --no-operator-path)")
    ap.add_argument("--no-operator-path", action="store_true")
    ap.add_argument("--algo", default="auto", choices=["auto", "fused", "staged", "staged_owned"])
    ap.add_argument("--settle-ms", type=float, default=20.0,
                    help="before the warm-up steps, run the same step untimed for about this long (0 = not at all; steps shorter "
                         "than 20 us never): a device that has been idle takes 10-20 ms under load to reach the state it then keeps")
    ap.add_argument("--workgroups-per-cu", type=int, default=0,
                    help="limit on resident workgroups per compute unit: 0 = the library's choice, -1 = none, 1..8 = forced")
    ap.add_argument("--print-source-hash", action="store_true", help="print the kernel-source hash and exit")
    args = ap.parse_args()
    if args.print_source_hash:
        print(kernel_sources_sha256())
        return
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (one rank's stage with N local partial buffers); "
              "--gpus %d with WORLD_SIZE=%s is not supported" % (args.gpus, os.environ.get("WORLD_SIZE", "1")), file=sys.stderr)
        sys.exit(2)

    import torch
    from torch_dist_ext_amd import _capi

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.config == "custom":
        cfg = (args.nranks, args.tokens or 2048, args.hidden, args.dtype, 0.5, 1e-5, args.quant, 6, 0)
    else:
        cfg = BENCH_CONFIGS[args.config]
    N, T, H, dt, sigma, eps, quant, seed, outliers = cfg
    own_tokens = T
    if args.tokens > 0:
        T = args.tokens
        cfg = (N, T, H, dt, sigma, eps, quant, seed, outliers)
    qm = {"none": _capi.QUANT_NONE, "fp8_token": _capi.QUANT_FP8_TOKEN, "fp8_group": _capi.QUANT_FP8_GROUP,
          "int8_token": _capi.QUANT_INT8_TOKEN}[quant]
    algo = {"auto": _capi.ALGO_AUTO, "fused": _capi.ALGO_FUSED, "staged": _capi.ALGO_STAGED,
            "staged_owned": _capi.ALGO_STAGED_OWNED}[args.algo]
    dcode = {"bf16": _capi.BF16, "f16": _capi.F16, "f32": _capi.F32, "f64": _capi.F64}[dt]
    e = ELEM_BYTES[dt]
    dtype = torch_dtype(torch, dt)

    def problem(rows):
        return _capi.make_problem(dcode, N, rows, H, eps, quant=qm, algo=algo, write_norm=0, workgroups_per_cu=args.workgroups_per_cu)

    prob = problem(T)
    plan = _capi.plan(prob)
    bytes_per_launch = plan.algorithmic_bytes
    # Enough distinct sets that a buffer is touched again only after > 4 GiB of other inputs AND > 1 GiB of other
    # outputs have passed: the 256 MB memory-side cache then neither serves reads nor absorbs the writes
    # (c3 on one reused set measures 4 % faster than with this rotation, on three sets or more within 1 % of it).
    out_bytes = bytes_per_launch - (N + 1) * T * H * e - H * e
    nsets = args.sets or min(128, max(3, -(-(4 << 30) // bytes_per_launch), -(-(1 << 30) // max(out_bytes, 1))) + 1)
    first = seeded_cpu_inputs(torch, cfg)
    sets = make_sets(torch, cfg, nsets, dev, first)
    gamma = first[2].to(dev)
    staged = algo in (_capi.ALGO_STAGED, _capi.ALGO_STAGED_OWNED)
    # One stage buffer per input set, so that stage B reads it from HBM like everything else.
    stages = [torch.zeros((T, H), dtype=dtype, device=dev) for _ in range(nsets)] if staged else None
    if algo == _capi.ALGO_STAGED_OWNED:
        # One rank's local share of the two-shot: stage A touches T/N rows of the N partials, stage B all T rows
        # of the stage (the rows of the other ranks are taken as already delivered; they are zeros here).
        owned = -(-T // N)
        bytes_per_launch = (N + 1) * owned * H * e + 2 * T * H * e + H * e + T * H * e + out_bytes
    elif staged:
        bytes_per_launch += 2 * T * H * e      # the stage is written once and read once on top of the fused job
    stream = torch.cuda.current_stream(dev)
    lib = _capi.load()
    hip_stream = ctypes.c_void_p(stream.cuda_stream)

    def argument_blocks(buffer_sets, rows_total, rows, stage_list=None):
        """One tde_buffers per block of `rows` rows inside every set of `rows_total` rows."""
        blocks = []
        groups = H // 128 if quant == "fp8_group" else 1
        for k, s in enumerate(buffer_sets):
            for o in range(0, rows_total - rows + 1, rows):
                b = _capi.Buffers()
                for r, p in enumerate(s["parts"]):
                    b.partial[r] = p.data_ptr() + o * H * e
                b.residual_in, b.residual_out = s["residual"].data_ptr() + o * H * e, s["res_out"].data_ptr() + o * H * e
                b.gamma = gamma.data_ptr()
                b.norm_out = s["norm"].data_ptr() + o * H * e if s["norm"] is not None else None
                b.q_out = s["q"].data_ptr() + o * H if s["q"] is not None else None
                b.scale_out = s["scale"].data_ptr() + o * groups * 4 if s["scale"] is not None else None
                b.stage = stage_list[k].data_ptr() + o * H * e if stage_list else None
                blocks.append(b)
        return blocks

    # Argument blocks are built once per input set; a step is then a single C-ABI call.
    calls = argument_blocks(sets, T, T, stages)
    prob_ref = ctypes.byref(prob)
    call_refs = [ctypes.byref(b) for b in calls]

    def event_timed(fn, steps, warmup):
        """Average duration of `steps` back-to-back calls of fn(i) on the launch stream, by HIP events."""
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize(dev)
        ev0 = torch.cuda.Event(enable_timing=True)
        ev1 = torch.cuda.Event(enable_timing=True)
        ev0.record(stream)
        for i in range(steps):
            fn(i)
        ev1.record(stream)
        torch.cuda.synchronize(dev)
        return ev0.elapsed_time(ev1) * 1e3 / steps

    def settle(fn):
        """Runs fn(i) back to back, untimed, for about --settle-ms of device time; returns the number of calls.
        Measured on c3 from a cold process: launches run 57.7-57.9 us for the first 9 ms and 57.0-57.3 us from then
        on; c5's launches 5 to 50 (2-18 ms) run up to 14 % slow.  A serving process is never in that state."""
        if args.settle_ms <= 0:
            return 0
        per_call_ms = event_timed(fn, 3, 2) * 1e-3
        if per_call_ms < 0.02:
            # Launch-bound steps (c2: 5 us) do not load the device, and thousands of them back to back leave the next
            # 200 anywhere between 5.0 and 6.1 us from one run to the next (0, 1, 3, 8, 20, 60 ms tried): not settled
            return 0
        n = int(args.settle_ms / per_call_ms) + 1
        for i in range(n):
            fn(i)
        torch.cuda.synchronize(dev)
        return n + 5

    def timed(fn, steps, warmup):
        settle(fn)
        return event_timed(fn, steps, warmup)

    def launch(i):
        st = lib.tde_reduce_rms(prob_ref, call_refs[i % nsets], hip_stream)
        if st != 0:
            _capi.check(st)

    # Calibration dispatches for profiler runs: three plain copies of a known size (256 MiB read +
    # 256 MiB written each) ahead of the warm-up, outside the timed region.
    cal_bytes = 256 << 20
    cal_src = torch.empty(cal_bytes, dtype=torch.uint8, device=dev).random_(0, 255)
    cal_dst = torch.empty_like(cal_src)
    for _ in range(3):
        _capi.probe_copy(cal_dst.data_ptr(), cal_src.data_ptr(), cal_bytes, stream.cuda_stream)
    torch.cuda.synchronize(dev)
    del cal_src, cal_dst

    # The same measurement before the settling phase: what the first milliseconds of a process that has been idle see.
    cold_avg_us = event_timed(launch, args.steps, args.warmup)
    settle_steps = settle(launch)
    for i in range(args.warmup):
        launch(i)
    torch.cuda.synchronize(dev)

    # Timed region: exactly K steps between two synchronizations.  HIP events recorded on the launch
    # stream at both ends give the device-side span; its K-th part is the average launch duration
    # (back-to-back launches on one stream; the gap between them is part of it).
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    ev0.record(stream)      # torch creates the HIP event at its first record: not inside the timed region
    ev1.record(stream)
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    ev0.record(stream)
    for i in range(args.steps):
        launch(i)
    ev1.record(stream)
    torch.cuda.synchronize(dev)
    wall = time.perf_counter() - t0
    avg_ms = ev0.elapsed_time(ev1) / args.steps

    # The kernel's outputs for the seeded set, kept for the checker in the CPU-baseline leg (the probes below
    # overwrite the device copies).  Every timed launch of that set wrote the same values.
    launch(0)
    torch.cuda.synchronize(dev)
    s0 = sets[0]
    kernel_out = {"residual_out": s0["res_out"].cpu()}
    if s0["norm"] is not None:
        kernel_out["norm_out"] = s0["norm"].cpu()
    if s0["q"] is not None:
        kernel_out["q"] = s0["q"].cpu()
        kernel_out["scale"] = s0["scale"].cpu()

    # The same launches with the arithmetic removed (tde_probe_rows_parts): what the access pattern alone takes
    # on this box, in this process, over the same buffers -- all of it, its input streams alone, its output
    # streams alone.  They overwrite the outputs, hence after the timed run.
    pattern = {}
    if not staged and dt != "f64":
        for key, parts in (("traffic_only_us", 7), ("reads_only_us", 1), ("writes_only_us", 6)):
            if parts == 6 and out_bytes <= 0:
                continue

            def launch_parts(i, parts=parts):
                st = lib.tde_probe_rows_parts(prob_ref, call_refs[i % nsets], parts, hip_stream)
                if st != 0:
                    _capi.check(st)
            pattern[key] = timed(launch_parts, args.steps, args.warmup)
    if "reads_only_us" in pattern and "writes_only_us" in pattern:
        # The input streams and the output streams as two kernels at once, on two streams: different workgroups on
        # different compute units, the same memory system.  Against traffic_only_us (both in one kernel) this tells
        # whether mixing reads with writes costs on the compute units or behind them.  The span is taken on the launch
        # stream, which waits for both side streams; the cross-stream waits cost about a microsecond per step.
        side = [torch.cuda.Stream(dev), torch.cuda.Stream(dev)]
        side_h = [ctypes.c_void_p(x.cuda_stream) for x in side]

        def both_at_once(steps):
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            done = [torch.cuda.Event(), torch.cuda.Event()]
            begin.record(stream)
            for x in side:
                x.wait_event(begin)
            for i in range(steps):
                lib.tde_probe_rows_parts(prob_ref, call_refs[i % nsets], 1, side_h[0])
                lib.tde_probe_rows_parts(prob_ref, call_refs[i % nsets], 6, side_h[1])
            for x, ev in zip(side, done):
                ev.record(x)
                stream.wait_event(ev)
            end.record(stream)
            torch.cuda.synchronize(dev)
            return begin.elapsed_time(end) * 1e3 / steps
        if args.warmup > 0:
            both_at_once(args.warmup)
        pattern["reads_and_writes_as_two_concurrent_kernels_us"] = both_at_once(args.steps)
    floor_us = pattern.get("traffic_only_us")
    read_bytes = (N + 1) * T * H * e
    launch_floor_us = timed(lambda i: lib.tde_probe_launch(hip_stream), 500, 50)

    ms_per_step = wall * 1e3 / args.steps
    gbs_job = bytes_per_launch / (wall / args.steps) / 1e9
    achieved = bytes_per_launch / (avg_ms * 1e-3) / 1e9
    traffic = None
    if not staged and T == own_tokens and args.config != "custom" and TRAFFIC["sources_sha256"] == kernel_sources_sha256():
        traffic = TRAFFIC["bytes"].get(args.config)
    out = {
        "metric": ("achieved HBM GB/s, one rank's 8-partial reduce+residual+RMSNorm+per-token fp8 stage" if args.config == "c3"
                   else "achieved HBM GB/s, one rank's %d-partial reduce+residual+RMSNorm stage, quant=%s" % (N, quant)),
        "value": gbs_job, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        # value, ms_per_step, tokens_per_s and pct_of_hbm_peak are by the host's wall clock around the K launches and the
        # synchronization after them; roofline.achieved / frac / kernel_avg_us by HIP events on the launch stream
        "value_clock": "host wall clock, K launches + synchronize",
        "settle_ms": args.settle_ms, "settle_steps": settle_steps,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        # dtype is the arithmetic type (fp32 accumulate, norm and quant; double for double tensors); tensors are stored as storage_dtype
        "dtype": "f64" if dt == "f64" else "f32", "storage_dtype": dt, "data": "synthetic",
        "tokens_per_s": T / (wall / args.steps),
        "pct_of_hbm_peak": 100.0 * gbs_job / HBM_PEAK_GBS,
        "config": {"workload": "%s: N=%d partials [%d,%d] %s, residual add + RMSNorm + %s%s" % (
                       args.config, N, T, H, dt, quant,
                       {"staged": " (two launches through a stage buffer)",
                        "staged_owned": " (two launches; stage A over this rank's T/N rows only)"}.get(args.algo, "")),
                   "storage_dtype": dt, "output": quant, "algo": args.algo, "input_sets": nsets, "block_threads": plan.block_threads,
                   "workgroups_per_cu": plan.workgroups_per_cu, "grid_blocks": plan.grid_blocks, "algorithmic_bytes": bytes_per_launch,
                   "settle_steps": settle_steps},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                     "clock": "HIP events on the launch stream around the K launches",
                     "kernel_avg_us": avg_ms * 1e3,
                     # W warm-up + K launches timed the same way before the settling phase (a device that has just been idle)
                     "cold_kernel_avg_us": cold_avg_us,
                     "cold_frac": bytes_per_launch / (cold_avg_us * 1e-6) / 1e9 / HBM_PEAK_GBS,
                     "fit": None,   # filled in below
                     # the same launches without arithmetic (same bytes, same access pattern), and their share of the peak
                     "traffic_only_us": floor_us,
                     "traffic_only_frac": (bytes_per_launch / (floor_us * 1e-6) / 1e9 / HBM_PEAK_GBS) if floor_us else None,
                     # the pattern's input streams alone and output streams alone (same workgroups, no arithmetic)
                     "reads_only_us": pattern.get("reads_only_us"),
                     "reads_only_GBs": (read_bytes / (pattern["reads_only_us"] * 1e-6) / 1e9) if pattern.get("reads_only_us") else None,
                     "writes_only_us": pattern.get("writes_only_us"),
                     "writes_only_GBs": (out_bytes / (pattern["writes_only_us"] * 1e-6) / 1e9) if pattern.get("writes_only_us") else None,
                     "reads_and_writes_as_two_concurrent_kernels_us": pattern.get("reads_and_writes_as_two_concurrent_kernels_us"),
                     # one empty dispatch, back to back on the same stream: the floor under latency-bound sizes
                     "launch_floor_us": launch_floor_us},
    }
    # The device's practical streaming rates, measured now (tde_probe_stream: 1 GiB per launch, four buffers
    # in rotation): what reads alone, writes alone and a plain copy reach on this box.
    # Nothing has been given back to the driver so far, and nothing is until every rate is measured: after device
    # memory is freed (torch.cuda.empty_cache -> hipFree) memory-bound launches run about 1.4 % slower for some
    # hundred milliseconds (c3: kernel 57.2 -> 58.0 us, skeleton 55.8 -> 56.6, measured by freeing 7 GiB between two
    # timings), presumably the driver clearing the freed pages in the background.
    gib = 1 << 30
    bufs = [torch.empty(gib, dtype=torch.uint8, device=dev).random_(0, 255) for _ in range(4)]
    rates = {}
    for mode, name, moved in ((0, "read_only_GBs", gib), (1, "write_only_GBs", gib), (2, "copy_GBs", 2 * gib)):
        us = timed(lambda i, mode=mode: _capi.probe_stream(bufs[i % 4].data_ptr(), bufs[(i + 1) % 4].data_ptr(), gib, mode,
                                                           stream.cuda_stream), 12, 3)
        rates[name] = moved / (us * 1e-6) / 1e9
    del bufs
    # What the device's own plain-stream rates make of this launch's bytes: the reads at the read-only rate plus the writes
    # at the write-only rate, times what the plain copy pays for moving both together, plus one dispatch.  No kernel with
    # this traffic goes below it on this box; the skeleton (traffic_only_us) is the same thing measured on the real pattern.
    mixing = (2.0 / rates["copy_GBs"]) / (1.0 / rates["read_only_GBs"] + 1.0 / rates["write_only_GBs"])
    rates_us = (read_bytes / rates["read_only_GBs"] + max(out_bytes, 0) / rates["write_only_GBs"]) * 1e-3 * mixing + launch_floor_us
    out["roofline"]["device_rates_floor"] = {
        "us": rates_us, "frac": bytes_per_launch / (rates_us * 1e-6) / 1e9 / HBM_PEAK_GBS, "copy_mixing_factor": mixing,
        "what": "reads at device.read_only_GBs + writes at device.write_only_GBs, times the plain copy's cost of moving both together, plus launch_floor_us"}

    # The same kernel at three row counts, in blocks of the same rotating buffers (or of larger ones), and the
    # straight line through the three points: time = fixed_us + bytes / bulk_GBs.
    fit = None
    if not args.no_fit and not staged and T >= 4:
        grow = (N + 2) * 4 * T * H * e <= (2 << 30)     # sets of 4 T rows stay below 2 GiB each: fit at T, 2T, 4T
        rows_list = [T, 2 * T, 4 * T] if grow else [T // 4, T // 2, T]
        top = rows_list[-1]
        if grow:
            fit_sets = make_sets(torch, cfg, max(3, -(-(5 << 30) // ((N + 2) * top * H * e))), dev, None, rows=top)
        else:
            fit_sets = sets
        points = []
        for rows in rows_list:
            blocks = argument_blocks(fit_sets, top, rows)
            refs = [ctypes.byref(b) for b in blocks]
            p_rows = problem(rows)
            pr = ctypes.byref(p_rows)

            def launch_rows(i, pr=pr, refs=refs):
                st = lib.tde_reduce_rms(pr, refs[i % len(refs)], hip_stream)
                if st != 0:
                    _capi.check(st)
            steps = max(20, min(args.steps, int(args.steps * T / rows)))
            points.append((rows, _capi.plan(p_rows).algorithmic_bytes, timed(launch_rows, steps, args.warmup)))
        n = len(points)
        mx = sum(p[1] for p in points) / n
        my = sum(p[2] for p in points) / n
        slope = sum((p[1] - mx) * (p[2] - my) for p in points) / sum((p[1] - mx) ** 2 for p in points)   # us per byte
        fit = {"rows": [p[0] for p in points], "kernel_us": [p[2] for p in points],
               "frac_of_peak": [p[1] / (p[2] * 1e-6) / 1e9 / HBM_PEAK_GBS for p in points],
               "fixed_us": my - slope * mx,
               # launch-bound sizes do not grow with the bytes: no rate to quote
               "bulk_GBs": (1e-3 / slope) if slope > 0 else None}
        if grow:
            del fit_sets   # back to torch's allocator, not to the driver

    out["roofline"]["fit"] = fit
    if args.operator_path or (args.config == "c2" and not args.no_operator_path):
        out["operator_path"] = operator_path_cost(torch, cfg, first, dev)
    info = _capi.device_info()
    out["device"] = {"name": torch.cuda.get_device_properties(dev).name, "compute_units": info.compute_units,
                     "memory_clock_khz": info.memory_clock_khz, "memory_bus_bits": info.memory_bus_bits,
                     "hbm_bytes": info.total_memory_bytes, **rates,
                     # transfers per reported memory clock that the published 8 TB/s corresponds to
                     "peak_transfers_per_clock": (HBM_PEAK_GBS * 1e9 * 8 / (info.memory_bus_bits * info.memory_clock_khz * 1e3)
                                                  if info.memory_bus_bits and info.memory_clock_khz else None)}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch, cfg, first, kernel_out)
        bad = [k for k, same in out["cpu_baseline"]["kernel_outputs_bit_identical_to_oracle"].items() if not same]
        if bad:
            print(json.dumps(out))
            print("bench.py: kernel outputs differ from the oracle: %s" % ", ".join(bad), file=sys.stderr)
            sys.exit(3)
    print(json.dumps(out))


if __name__ == "__main__":
    main()

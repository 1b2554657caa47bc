"""Benchmark of the bf16 scan, forward + backward, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--case C3_4096] [--config V,S,W]

One "step" is one forward scan plus one backward scan over one batch of
synthetic input, launched through the C ABI on torch's current stream with all
tensors already resident in HBM.  Prints ONE JSON line:

  value            algorithmic GB/s of the whole step: 16 B per element (forward reads
                   alpha, beta and writes h = 6 B; backward reads alpha, h, dout and
                   writes grad_alpha, grad_beta = 10 B) divided by the wall time per step
  roofline         the dominant kernel (the backward scan, 10 of the 16 B): its
                   algorithmic bytes per launch over its launch duration.  The duration is
                   the kernel's share of the wall time per step of the timed region - the
                   step split in the ratio of the two launches as HIP events around sampled
                   steps see them - so forward and backward add up to `ms_per_step` and the
                   few microseconds between two launches are charged to the kernels, not
                   dropped (`avg_launch_ms`; a rocprofv3 kernel trace, which leaves those
                   gaps out, reads 0-3 % shorter).  Beside it: `avg_launch_ms_events_raw`
                   (events as read, at least 32 samples) and `avg_launch_ms_events_corrected`
                   (less what a pair of events adds to a kernel between them, calibrated in the
                   same run with the library's copy kernel: one launch between two events
                   against four).  `traffic` is the counter-measured HBM bytes per launch from
                   profiles/, when that summary covers the configuration; `frac_no_reuse` is
                   the same fraction with eight sets of tensors in rotation;
                   `frac_of_machine` the kernel's rate in that rotation over what the
                   library's plain streaming kernel reaches on the same buffers with the
                   same mix of reads and writes (`machine_stream`)
  machine_stream   fss_stream_mix over the same eight tensor sets in rotation: 3 reads, 2 reads +
                   1 non-temporal write (the forward's mix), 3 reads + 2 non-temporal writes
                   (the backward's): this machine's own streaming rates, GB/s, each the best
                   of eight launch shapes of that kernel (`*_shape` names the one that won);
                   `one_set_step_ms`: the forward's mix and the backward's alternating on one
                   set of tensors, the protocol of `value`; `step_frac_of_machine` (top level)
                   is that over `ms_per_step`
  workloads        all ten measured workloads, forward+backward on one set of tensors and over
                   sets in rotation (more than 1.5 GB, nothing reused): ms per step, the two
                   kernels' shares, fraction of 8 TB/s
  rotating_sets    the same step over eight sets of tensors in rotation, so that no step finds its
                   inputs in the memory-side cache (`value` reuses one set, as the reference's
                   benchmark does); `--rotate 8` makes that the timed region itself
  cpu_baseline     the reference's PyTorch sequential loop (oracle/torch_loop.py) on the
                   host cores, same inputs, fp32; also the parity check of this run
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
FWD_BYTES_PER_ELEM = 6
BWD_BYTES_PER_ELEM = 10


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=25)
    ap.add_argument("--case", default="C3_4096", help="workload name from fast_sequential_scan_amd.workloads")
    ap.add_argument("--dtype", default="bf16", choices=("bf16", "f32", "f16"),
                    help="storage type of the tensors (the headline metric is bf16; carries are fp32 either way)")
    ap.add_argument("--op", default="scan", choices=("scan", "gated", "cm"),
                    help="scan: the reference's operator (headline metric); gated: the scan with the sigmoid/"
                         "sqrt(1-alpha^2) gating computed inside the kernels (9 tensors of traffic per step); "
                         "cm: the scan on channel-major (bs, d, seq) tensors")
    ap.add_argument("--config", default=None, help="explicit vec,steps,waves for both kernels (tuning)")
    ap.add_argument("--fwd-config", default=None)
    ap.add_argument("--bwd-config", default=None)
    ap.add_argument("--event-stride", type=int, default=8,
                    help="record HIP events around the two launches of every N-th timed step")
    ap.add_argument("--rotate", type=int, default=1,
                    help="number of tensor sets the timed loop cycles through (1: every step reuses the same "
                         "tensors, as the reference's benchmark does, so part of them sits in the 256 MB "
                         "memory-side cache; 8: 3.2 GB in rotation at the headline shape, nothing reused)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline / parity leg")
    ap.add_argument("--no-autograd", action="store_true",
                    help="skip the timing of the public autograd path (profiler runs: its launches would be "
                         "averaged into the kernels' statistics)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline leg")
    ap.add_argument("--flush-mb", type=int, default=1024, help="size of the cache-flush read for the cold timings")
    ap.add_argument("--cache-policy", default="auto", choices=("auto", "streaming"),
                    help="fss_set_cache_policy for the run (streaming: assume nothing is found in the caches again)")
    ap.add_argument("--sweep", action="store_true",
                    help="the reference's benchmark sweep (benchmark.py:37-110): sequence lengths 128..32768 at "
                         "--sweep-bs x --sweep-d, forward and forward+backward through the public autograd API, "
                         "one cache-clearing write before every timed call as triton's do_bench does; one JSON line")
    ap.add_argument("--sweep-bs", type=int, default=8)
    ap.add_argument("--sweep-d", type=int, default=1024)
    ap.add_argument("--no-workloads", action="store_true",
                    help="skip the table of all ten workloads (profiler runs: its launches would be averaged "
                         "into the kernels' statistics)")
    ap.add_argument("--stream-one-set", action="store_true",
                    help="only the plain streaming kernel in the benchmark's protocol (one set of tensors of --case's "
                         "size, forward's mix then backward's, --steps steps in each launch shape); for profiling")
    ap.add_argument("--copy-mb", type=int, default=0,
                    help="run only the library's plain copy kernel on this many MiB, --steps times "
                         "(hardware counters of the scan kernels are scaled by what they read for it)")
    return ap.parse_args()


def quantile_pair(samples):
    """20th and 80th percentile, as the reference's benchmark reports them (benchmark.py:65)."""
    if len(samples) < 2:
        return [round(samples[0], 5)] * 2 if samples else None
    q = statistics.quantiles(samples, n=5, method="inclusive")
    return [round(q[0], 5), round(q[3], 5)]


def sweep(args, torch, scan_cu, dev) -> int:
    """Times what the reference's benchmark.py times for its "cuda-bf16" provider: `scan_cu(alpha, beta)`
    and `scan_cu(alpha, beta).backward(dy)` per sequence length, median and 20th/80th percentile of
    100 calls, each after a 256 MB write that clears the caches."""
    bs, d = args.sweep_bs, args.sweep_d
    flush = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
    rows = []
    for sq in (128, 256, 1024, 2048, 4096, 8192, 16384, 32768):
        gen = torch.Generator(device=dev).manual_seed(sq)
        alpha = torch.sigmoid(torch.randn(bs, sq, d, device=dev, generator=gen)).to(torch.bfloat16).requires_grad_(True)
        beta = torch.randn(bs, sq, d, device=dev, generator=gen).to(torch.bfloat16).requires_grad_(True)
        dy = (0.1 * torch.randn(bs, sq, d, device=dev, generator=gen)).to(torch.bfloat16)

        def fwd():
            with torch.no_grad():
                return scan_cu(alpha, beta)

        def fwd_bwd():
            alpha.grad = beta.grad = None
            scan_cu(alpha, beta).backward(dy)

        row = {"seq": sq, "elements": bs * sq * d}
        for name, fn, nbytes in (("fwd", fwd, 6), ("fwd_bwd", fwd_bwd, 16)):
            for _ in range(10):
                fn()
            times = []
            for _ in range(100):
                flush.zero_()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                fn()
                e1.record()
                e1.synchronize()
                times.append(e0.elapsed_time(e1))
            med = statistics.median(times)
            row[name + "_ms"] = round(med, 5)
            row[name + "_ms_p20_p80"] = quantile_pair(times)
            row[name + "_GBps"] = round(nbytes * bs * sq * d / (med * 1e-3) / 1e9, 1)
        rows.append(row)
        del alpha, beta, dy
    print(json.dumps({
        "metric": "scan_cu forward and forward+backward ms per sequence length (the reference's benchmark.py sweep)",
        "unit": "ms", "bs": bs, "d_model": d, "dtype": "bf16", "data": "synthetic",
        "protocol": "public autograd API, caches cleared by a 256 MB write before every timed call, median of 100",
        "sweep": rows,
    }))
    return 0


def frac_of_machine(machine, key, nbytes, kernel_ms):
    """The kernel's rate over tensor sets in rotation as a fraction of the plain streaming kernel's
    on the same buffers with the same mix of reads and writes."""
    if not machine or not kernel_ms:
        return None
    return round(nbytes / (kernel_ms * 1e-3) / 1e9 / machine[key], 4)


# Launch shapes the calibration tries: (workgroups, threads, vectors per lane and iteration,
# non-temporal loads).  Which one streams fastest depends on the mix; the best is what counts.
STREAM_SHAPES = ((2048, 256, 1, 0), (16384, 256, 1, 0), (1024, 1024, 1, 0), (8192, 512, 1, 0),
                 (512, 256, 2, 1), (1024, 512, 2, 1), (512, 256, 1, 1), (2048, 256, 2, 0))


def stream_one_set(_native, torch, p, tensor_bytes, sp, sink, warmup, steps):
    """The benchmark's own protocol for the plain streaming kernel: the forward's mix and the
    backward's alternating on ONE set of tensors (p: addresses of alpha, beta, dout, h, grad_alpha,
    grad_beta), where the 256 MB memory-side cache returns part of every stream; both launches of
    a step in the same launch shape.  Returns (best ms per step, its shape, ms per step by shape)."""
    by_shape = {}
    for shape in STREAM_SHAPES:
        def run(n):
            for _ in range(n):
                _native.stream_mix([p[0], p[1]], [p[3]], tensor_bytes, True, sp, sink.data_ptr(), shape)
                _native.stream_mix([p[0], p[3], p[2]], [p[4], p[5]], tensor_bytes, True, sp, sink.data_ptr(), shape)
        run(warmup)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run(steps)
        torch.cuda.synchronize()
        by_shape[shape] = (time.perf_counter() - t0) * 1e3 / steps
    best = min(by_shape, key=by_shape.get)
    return by_shape[best], best, by_shape


def machine_stream_leg(lib, _native, torch, pointer_sets, tensor_bytes, sp):
    """What this machine streams: the library's plain streaming kernel (fss_stream_mix) over the
    tensor sets of the rotation - every launch meets buffers that were last touched seven launches
    (several GB) ago - with the forward's mix of streams (reads alpha, beta; writes h), the
    backward's (reads alpha, h, dout; writes grad_alpha, grad_beta) and reads only.  Every mix is
    run in each of STREAM_SHAPES; the fastest shape's rate is the machine's for that mix."""
    sink = torch.zeros(16, dtype=torch.uint8, device="cuda")
    mixes = {
        "read_only_GBps": (lambda p: ([p[0], p[1], p[2]], [])),
        "fwd_mix_GBps": (lambda p: ([p[0], p[1]], [p[3]])),
        "bwd_mix_GBps": (lambda p: ([p[0], p[3], p[2]], [p[4], p[5]])),
    }
    out = {"tensor_sets": len(pointer_sets), "bytes_per_stream": tensor_bytes,
           "kernel": "fss::stream_mix_kernel<reads, writes, ...>, 16 B per lane and access, linear, non-temporal "
                     "writes; best of the launch shapes tried (workgroups, threads, vectors per lane and "
                     "iteration, non-temporal loads)"}
    n_launches = 4 * len(pointer_sets)
    for name, pick in mixes.items():
        def run(n, shape):
            for i in range(n):
                reads, writes = pick(pointer_sets[i % len(pointer_sets)])
                _native.stream_mix(reads, writes, tensor_bytes, True, sp, sink.data_ptr(), shape)
        best_ms, best_shape, default_ms = None, None, None
        for shape in STREAM_SHAPES:
            run(len(pointer_sets), shape)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            run(n_launches, shape)
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) * 1e3 / n_launches
            if default_ms is None:
                default_ms = ms
            if best_ms is None or ms < best_ms:
                best_ms, best_shape = ms, shape
        reads, writes = pick(pointer_sets[0])
        nbytes = (len(reads) + len(writes)) * tensor_bytes
        out[name] = round(nbytes / (best_ms * 1e-3) / 1e9, 1)
        out[name.replace("_GBps", "_ms_per_launch")] = round(best_ms, 5)
        out[name.replace("_GBps", "_shape")] = list(best_shape)
        out[name.replace("_GBps", "_first_shape_GBps")] = round(nbytes / (default_ms * 1e-3) / 1e9, 1)
    best_ms, best_shape, _ = stream_one_set(_native, torch, pointer_sets[0], tensor_bytes, sp, sink, 10, 50)
    out["one_set_step_ms"] = round(best_ms, 5)
    out["one_set_step_GBps"] = round(8 * tensor_bytes / (best_ms * 1e-3) / 1e9, 1)
    out["one_set_step_shape"] = list(best_shape)
    return out


def measure_workload(lib, _native, torch, dev, case):
    """One measured workload, briefly: forward+backward through the C ABI with the library's own
    choices, on one set of tensors (as the reference's benchmark loops) and over enough sets in
    rotation that nothing is found in a cache again (more than 1.5 GB).  Inputs are drawn on the
    device with the workload's recipe; their values only matter to the timing through the recipe.
    Kernel times are the kernels' shares of the wall time per step (split as HIP events around
    16 sampled steps see the two launches)."""
    from fast_sequential_scan_amd.workloads import BASELINE_CASES

    recipe, bs, seq, d = BASELINE_CASES[case]
    n = bs * seq * d
    gen = torch.Generator(device=dev).manual_seed(sum(case.encode()))
    x = torch.randn(bs, seq, d, device=dev, generator=gen)
    beta = torch.randn(bs, seq, d, device=dev, generator=gen)
    if recipe == "normal":
        alpha = x
    elif recipe == "sigmoid_plus2":
        alpha = torch.sigmoid(x + 2.0)
    else:
        alpha = torch.sigmoid(x)
    if recipe == "hawk":
        beta = beta * torch.sqrt(1.0 - alpha * alpha)
    alpha, beta = alpha.to(torch.bfloat16), beta.to(torch.bfloat16)
    dout = torch.randn(bs, seq, d, device=dev, generator=gen).to(torch.bfloat16)
    del x
    per_set = 6 * n * 2
    n_sets = min(64, max(3, -(-(3 << 29) // per_set)))
    sets = [(alpha, beta, dout, torch.empty_like(alpha), torch.empty_like(alpha), torch.empty_like(alpha))]
    for _ in range(n_sets - 1):
        sets.append((alpha.clone(), beta.clone(), dout.clone(), torch.empty_like(alpha), torch.empty_like(alpha),
                     torch.empty_like(alpha)))
    ptrs = [tuple(t.data_ptr() for t in ts) for ts in sets]
    stream = torch.cuda.current_stream()
    sp = stream.cuda_stream
    code = _native.FSS_BF16
    ws_bytes = max(lib.fss_workspace_bytes(bs, seq, d, code, _native.FSS_FWD, None),
                   lib.fss_workspace_bytes(bs, seq, d, code, _native.FSS_BWD, None))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    _native.check(lib.fss_workspace_init(ws.data_ptr(), ws.numel(), sp))
    pws = ws.data_ptr()

    def step(p):
        pa, pb, pd, ph, pga, pgb = p
        rc = lib.fss_scan_fwd_ex(code, pa, pb, ph, bs, seq, d, pws, ws_bytes, sp, None)
        if rc == 0:
            rc = lib.fss_scan_bwd_ex(code, pa, ph, pd, pga, pgb, bs, seq, d, pws, ws_bytes, sp, None)
        if rc:
            _native.check(rc)

    def timed(rotate, n_steps):
        k = len(ptrs) if rotate else 1
        for i in range(max(5, k)):
            step(ptrs[i % k])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n_steps):
            step(ptrs[i % k])
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / n_steps
        evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(16)]
        for i, e in enumerate(evs):
            pa, pb, pd, ph, pga, pgb = ptrs[i % k]
            e[0].record(stream)
            _native.check(lib.fss_scan_fwd_ex(code, pa, pb, ph, bs, seq, d, pws, ws_bytes, sp, None))
            e[1].record(stream)
            _native.check(lib.fss_scan_bwd_ex(code, pa, ph, pd, pga, pgb, bs, seq, d, pws, ws_bytes, sp, None))
            e[2].record(stream)
        torch.cuda.synchronize()
        f = statistics.fmean(e[0].elapsed_time(e[1]) for e in evs)
        b = statistics.fmean(e[1].elapsed_time(e[2]) for e in evs)
        return ms, ms * f / (f + b), ms * b / (f + b)

    step_bytes = 16 * n
    n_steps = int(max(30, min(300, 0.012 / (step_bytes / 5.5e12 + 15e-6))))  # about 12 ms of GPU time per leg
    ms, f_ms, b_ms = timed(False, n_steps)
    rms, rf_ms, rb_ms = timed(True, max(n_steps // 2, 2 * n_sets))
    _native.check(lib.fss_workspace_status(pws, sp))
    cf, cb = _native.FssConfig(), _native.FssConfig()
    lib.fss_choose_config(bs, seq, d, code, _native.FSS_FWD, 16, ctypes.byref(cf))
    lib.fss_choose_config(bs, seq, d, code, _native.FSS_BWD, 16, ctypes.byref(cb))

    def frac(nbytes, t_ms):
        return round(nbytes / (t_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)

    return {
        "case": case, "bs": bs, "seq": seq, "d_model": d, "recipe": recipe,
        "launch_config_fwd": [cf.vec, cf.steps, cf.waves, cf.cols], "launch_config_bwd": [cb.vec, cb.steps, cb.waves, cb.cols],
        "ms_per_step": round(ms, 5), "fwd_ms": round(f_ms, 5), "bwd_ms": round(b_ms, 5),
        "GBps": round(step_bytes / (ms * 1e-3) / 1e9, 1), "frac": frac(step_bytes, ms),
        "fwd_frac": frac(6 * n, f_ms), "bwd_frac": frac(10 * n, b_ms),
        "no_reuse": {"tensor_sets": n_sets, "ms_per_step": round(rms, 5), "fwd_ms": round(rf_ms, 5),
                     "bwd_ms": round(rb_ms, 5), "frac": frac(step_bytes, rms),
                     "fwd_frac": frac(6 * n, rf_ms), "bwd_frac": frac(10 * n, rb_ms)},
        "frac_no_reuse": frac(step_bytes, rms),
    }


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(
            "bench.py measures one GPU: channels are independent, so more GPUs would each run this "
            "same kernel on a slice of bs or d with no communication; run with --gpus 1",
            file=sys.stderr,
        )
        return 2

    import torch

    from fast_sequential_scan_amd import _native, scan_cm, scan_cu, scan_cu_fp16, scan_cu_single, scan_gated
    from fast_sequential_scan_amd import sequential_scan_cuda as ext
    from fast_sequential_scan_amd.workloads import BASELINE_CASES, make_inputs

    lib = _native.lib()  # no fallback: a missing HIP library is an error
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)

    if args.copy_mb > 0:
        n = args.copy_mb << 20
        src = torch.ones(n, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        sp = torch.cuda.current_stream().cuda_stream
        for _ in range(args.warmup):
            _native.check(lib.fss_copy_bytes(src.data_ptr(), dst.data_ptr(), n, sp))
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(args.steps):
            _native.check(lib.fss_copy_bytes(src.data_ptr(), dst.data_ptr(), n, sp))
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / args.steps
        print(json.dumps({"metric": "plain copy kernel", "read_bytes": n, "written_bytes": n, "steps": args.steps,
                          "ms_per_launch": round(ms, 5), "value": round(2 * n / (ms * 1e-3) / 1e9, 1),
                          "unit": "GB/s (read+write)"}))
        return 0

    if args.stream_one_set:
        _, bs, seq, d = BASELINE_CASES[args.case]
        esize = 4 if args.dtype == "f32" else 2
        nbytes = bs * seq * d * esize
        tensors = [torch.full((nbytes,), i + 1, dtype=torch.uint8, device=dev) for i in range(6)]
        sink = torch.zeros(16, dtype=torch.uint8, device=dev)
        sp = torch.cuda.current_stream().cuda_stream
        best_ms, best_shape, by_shape = stream_one_set(_native, torch, [t.data_ptr() for t in tensors], nbytes, sp, sink,
                                                       args.warmup, args.steps)
        print(json.dumps({"metric": "plain streaming kernel, forward's mix then backward's on one set of tensors",
                          "case": args.case, "dtype": args.dtype, "bytes_per_stream": nbytes, "steps": args.steps,
                          "ms_per_step": round(best_ms, 5), "launch_shape": list(best_shape),
                          "value": round(8 * nbytes / (best_ms * 1e-3) / 1e9, 1), "unit": "GB/s",
                          "ms_per_step_by_shape": {"x".join(map(str, k)): round(v, 5) for k, v in by_shape.items()}}))
        return 0

    ext.set_cache_policy(args.cache_policy)
    if args.sweep:
        return sweep(args, torch, scan_cu, dev)

    recipe, bs, seq, d = BASELINE_CASES[args.case]
    n_elem = bs * seq * d
    is_16bit = args.dtype != "f32"
    gated = args.op == "gated"
    cm = args.op == "cm"
    scan_fn = scan_gated if gated else scan_cm if cm else {"bf16": scan_cu, "f16": scan_cu_fp16, "f32": scan_cu_single}[args.dtype]
    tol = {"bf16": 1e-2, "f16": 2e-3, "f32": 1e-4}[args.dtype]  # bf16: the reference's test tolerance; fp32 differs by carry re-association only
    kname = args.dtype.upper()
    fss_dtype = {"bf16": _native.FSS_BF16, "f16": _native.FSS_F16, "f32": _native.FSS_F32}[args.dtype]
    esize = 2 if is_16bit else 4
    fwd_bytes_per_elem = FWD_BYTES_PER_ELEM * esize // 2
    # gated backward: reads gate, x, h, dout and writes grad_gate, grad_x = 6 tensors
    bwd_bytes_per_elem = (12 if gated else BWD_BYTES_PER_ELEM) * esize // 2
    tdtype = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[args.dtype]
    alpha_c, beta_c, dout_c = make_inputs(recipe, bs, seq, d, dtype=tdtype)
    if gated:
        # first input = the gate pre-activation, second = x; both N(0,1) (the "hawk" recipe before its gating)
        gen = torch.Generator().manual_seed(4242)
        alpha_c = torch.randn(bs, seq, d, generator=gen).to(tdtype)
        beta_c = torch.randn(bs, seq, d, generator=gen).to(tdtype)
    if cm:  # the same values, time contiguous on the device; the CPU loop keeps its (bs, seq, d) view
        alpha, beta, dout = (t.transpose(1, 2).contiguous().to(dev) for t in (alpha_c, beta_c, dout_c))
    else:
        alpha, beta, dout = alpha_c.to(dev), beta_c.to(dev), dout_c.to(dev)
    h = torch.empty_like(alpha)
    galpha = torch.empty_like(alpha)
    gbeta = torch.empty_like(alpha)

    def cfg_of(text):
        return tuple(int(x) for x in text.split(",")) if text else None

    fwd_cfg = cfg_of(args.fwd_config or args.config)
    bwd_cfg = cfg_of(args.bwd_config or args.config)
    fwd_cfg_p, bwd_cfg_p = _native.make_config(fwd_cfg), _native.make_config(bwd_cfg)

    stream = torch.cuda.current_stream()
    sp = stream.cuda_stream
    dir_fwd, dir_bwd = (_native.FSS_GATED_FWD, _native.FSS_GATED_BWD) if gated else (_native.FSS_FWD, _native.FSS_BWD)
    if cm:
        ws_bytes = max(
            lib.fss_cm_workspace_bytes(bs, d, seq, fss_dtype, dir_fwd, fwd_cfg_p),
            lib.fss_cm_workspace_bytes(bs, d, seq, fss_dtype, dir_bwd, bwd_cfg_p),
        )
    else:
        ws_bytes = max(
            lib.fss_workspace_bytes(bs, seq, d, fss_dtype, dir_fwd, fwd_cfg_p),
            lib.fss_workspace_bytes(bs, seq, d, fss_dtype, dir_bwd, bwd_cfg_p),
        )
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    _native.check(lib.fss_workspace_init(ws.data_ptr(), ws.numel(), sp))
    pws = ws.data_ptr()
    # set 0 is the one everything else in this file looks at; the others are copies of its inputs
    tensor_sets = [(alpha, beta, dout, h, galpha, gbeta)]
    for _ in range(max(1, args.rotate) - 1):
        tensor_sets.append((alpha.clone(), beta.clone(), dout.clone(), torch.empty_like(h),
                            torch.empty_like(h), torch.empty_like(h)))
    pointer_sets = [tuple(t.data_ptr() for t in ts) for ts in tensor_sets]
    pa, pb, pd, ph, pga, pgb = pointer_sets[0]
    turn = [0]

    def next_set():
        nonlocal pa, pb, pd, ph, pga, pgb
        turn[0] = (turn[0] + 1) % len(pointer_sets)
        pa, pb, pd, ph, pga, pgb = pointer_sets[turn[0]]

    def first_set():
        nonlocal pa, pb, pd, ph, pga, pgb
        turn[0] = 0
        pa, pb, pd, ph, pga, pgb = pointer_sets[0]

    def fwd():
        if gated:
            rc = lib.fss_gated_scan_fwd(fss_dtype, pa, pb, ph, bs, seq, d, pws, ws_bytes, sp, fwd_cfg_p)
        elif cm:
            rc = lib.fss_scan_fwd_cm(fss_dtype, pa, pb, ph, bs, d, seq, pws, ws_bytes, sp, fwd_cfg_p)
        else:
            rc = lib.fss_scan_fwd_ex(fss_dtype, pa, pb, ph, bs, seq, d, pws, ws_bytes, sp, fwd_cfg_p)
        if rc:
            _native.check(rc)

    def bwd():
        if gated:  # pga receives grad_gate, pgb grad_x
            rc = lib.fss_gated_scan_bwd(fss_dtype, pa, pb, ph, pd, pga, pgb, bs, seq, d, pws, ws_bytes, sp, bwd_cfg_p)
        elif cm:
            rc = lib.fss_scan_bwd_cm(fss_dtype, pa, ph, pd, pga, pgb, bs, d, seq, pws, ws_bytes, sp, bwd_cfg_p)
        else:
            rc = lib.fss_scan_bwd_ex(fss_dtype, pa, ph, pd, pga, pgb, bs, seq, d, pws, ws_bytes, sp, bwd_cfg_p)
        if rc:
            _native.check(rc)

    chosen = {}
    for name, direction, user in (("fwd", dir_fwd, fwd_cfg), ("bwd", dir_bwd, bwd_cfg)):
        c = _native.FssConfig()
        if cm:  # 16 bytes per lane; 8 waves, fewer when the sequence is shorter than their reach
            c.vec = 16 // esize
            c.waves = min(8, -(-seq // (64 * c.vec)))
        else:
            lib.fss_choose_config(bs, seq, d, fss_dtype, direction, 16, ctypes.byref(c))
        chosen[name] = list(user[:3]) if user else [c.vec, c.steps, c.waves]
        chosen[name + "_cols"] = (user[4] if user and len(user) > 4 and user[4] else 1) if (user or cm) else c.cols

    # ---- warm-up, then the timed region: exactly K steps between two synchronisations ----
    for _ in range(args.warmup):
        fwd()
        bwd()
        next_set()
    K = args.steps
    # HIP events around the launches of every `stride`-th step of the timed region (an event
    # between two kernels costs a few microseconds of GPU time, so not around every one)
    stride = max(1, args.event_stride)
    sampled = list(range(0, K, stride))
    ev = {k: [torch.cuda.Event(enable_timing=True) for _ in range(3)] for k in sampled}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(K):
        e = ev.get(k)
        if e is None:
            fwd()
            bwd()
        else:
            e[0].record(stream)
            fwd()
            e[1].record(stream)
            bwd()
            e[2].record(stream)
        next_set()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    first_set()
    _native.check(lib.fss_workspace_status(pws, sp))

    ms_per_step = wall * 1e3 / K

    def launch_pair_samples(n):
        """n more steps with events around both launches of each: [(fwd_ms, bwd_ms)] raw."""
        evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(n)]
        for e in evs:
            e[0].record(stream)
            fwd()
            e[1].record(stream)
            bwd()
            e[2].record(stream)
            next_set()
        torch.cuda.synchronize()
        return [(e[0].elapsed_time(e[1]), e[1].elapsed_time(e[2])) for e in evs]

    # What a pair of events adds to the kernel between them.  An empty pair overstates it (the
    # second event's packet is processed while a kernel runs, not after), so it is calibrated with
    # the library's copy kernel on a cache-resident buffer: events around one launch against
    # events around four launches back to back; a launch costs (t4 - t1)/3, the rest of t1 is the
    # events'.  What is left in the kernel times after subtracting it is the gap between two
    # launches, so they err on the long side.
    cal = torch.empty(4 << 20, dtype=torch.uint8, device=dev)
    cal2 = torch.empty_like(cal)

    def copy_between_events(n_launches):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(n_launches):
            lib.fss_copy_bytes(cal.data_ptr(), cal2.data_ptr(), cal.numel(), sp)
        e1.record(stream)
        return e0, e1

    for _ in range(10):
        copy_between_events(4)
    ones = [copy_between_events(1) for _ in range(60)]
    fours = [copy_between_events(4) for _ in range(60)]
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(60)]
    for e0, e1 in pairs:
        e0.record(stream)
        e1.record(stream)
    torch.cuda.synchronize()
    t1 = statistics.median(e0.elapsed_time(e1) for e0, e1 in ones)
    t4 = statistics.median(e0.elapsed_time(e1) for e0, e1 in fours)
    empty_pair = statistics.median(e0.elapsed_time(e1) for e0, e1 in pairs)
    event_overhead = min(max(t1 - (t4 - t1) / 3.0, 0.0), empty_pair)
    del cal, cal2

    fwd_raw = [ev[k][0].elapsed_time(ev[k][1]) for k in sampled]
    bwd_raw = [ev[k][1].elapsed_time(ev[k][2]) for k in sampled]
    in_region = len(sampled)
    if in_region < 32:  # the same loop goes on, untimed, until there are enough samples
        more = launch_pair_samples(32 - in_region)
        first_set()
        fwd_raw += [f for f, _ in more]
        bwd_raw += [b for _, b in more]
    fwd_ms = [max(t - event_overhead, 1e-6) for t in fwd_raw]
    bwd_ms = [max(t - event_overhead, 1e-6) for t in bwd_raw]
    fwd_corr, bwd_corr = statistics.fmean(fwd_ms), statistics.fmean(bwd_ms)
    # the kernels' shares of the wall time per step, split as the events see the two launches:
    # they add up to ms_per_step, launch gaps included
    raw_f, raw_b = statistics.fmean(fwd_raw), statistics.fmean(bwd_raw)
    fwd_mean = ms_per_step * raw_f / (raw_f + raw_b)
    bwd_mean = ms_per_step * raw_b / (raw_f + raw_b)
    step_bytes = (fwd_bytes_per_elem + bwd_bytes_per_elem) * n_elem
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    bwd_gbps = bwd_bytes_per_elem * n_elem / (bwd_mean * 1e-3) / 1e9
    fwd_gbps = fwd_bytes_per_elem * n_elem / (fwd_mean * 1e-3) / 1e9

    # ---- the same step over eight tensor sets in rotation (nothing reused between steps), unless
    # the timed region above already rotated; reported next to `value`, never as `value` ----
    rotating = {}
    machine = None
    if len(pointer_sets) == 1 and args.flush_mb > 0:
        extra = [(alpha.clone(), beta.clone(), dout.clone(), torch.empty_like(h), torch.empty_like(h),
                  torch.empty_like(h)) for _ in range(7)]
        pointer_sets.extend(tuple(t.data_ptr() for t in ts) for ts in extra)
        n_rot = max(16, K // 2)

        def rotating_leg():
            for _ in range(8):
                fwd()
                bwd()
                next_set()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(n_rot):
                fwd()
                bwd()
                next_set()
            torch.cuda.synchronize()
            rot_ms = (time.perf_counter() - t0) * 1e3 / n_rot
            rot = launch_pair_samples(32)
            rf, rb = statistics.fmean(f for f, _ in rot), statistics.fmean(b for _, b in rot)
            rot_fwd, rot_bwd = rot_ms * rf / (rf + rb), rot_ms * rb / (rf + rb)  # shares of the wall time, as above
            return {"tensor_sets": len(pointer_sets), "steps": n_rot, "ms_per_step": round(rot_ms, 5),
                    "GBps": round(step_bytes / (rot_ms * 1e-3) / 1e9, 1),
                    "pct_of_hbm_peak": round(100.0 * step_bytes / (rot_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2),
                    "fwd_ms": round(rot_fwd, 5), "bwd_ms": round(rot_bwd, 5),
                    "fwd_ms_events_corrected": round(max(rf - event_overhead, 1e-6), 5),
                    "bwd_ms_events_corrected": round(max(rb - event_overhead, 1e-6), 5),
                    "fwd_frac": round(fwd_bytes_per_elem * n_elem / (rot_fwd * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                    "bwd_frac": round(bwd_bytes_per_elem * n_elem / (rot_bwd * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}

        rotating = rotating_leg()
        if not gated and not cm:
            machine = machine_stream_leg(lib, _native, torch, pointer_sets, alpha.numel() * alpha.element_size(), sp)
        if args.cache_policy == "auto" and not cm:
            # the same rotation as a caller would run it who knows that nothing is reused
            # (fss_set_cache_policy(FSS_CACHE_STREAMING): other cache hints, same tiling, same bits)
            ext.set_cache_policy("streaming")
            try:
                rotating["streaming_policy"] = rotating_leg()
            finally:
                ext.set_cache_policy("auto")
        del pointer_sets[1:]
        del extra
        first_set()
    elif len(pointer_sets) > 1:
        rotating = {"tensor_sets": len(pointer_sets), "steps": K, "ms_per_step": round(ms_per_step, 5),
                    "GBps": round(value, 1), "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
                    "fwd_ms": round(fwd_mean, 5), "bwd_ms": round(bwd_mean, 5),
                    "fwd_frac": round(fwd_gbps / HBM_PEAK_GBPS, 4), "bwd_frac": round(bwd_gbps / HBM_PEAK_GBPS, 4)}

    # ---- cold timings: reading a large buffer between launches evicts L2 and the memory-side
    # cache and leaves them clean (a large write would leave dirty lines whose write-back is then
    # charged to the kernel under test) ----
    cold = {}
    if args.flush_mb > 0:
        junk = torch.zeros(args.flush_mb << 18, dtype=torch.int32, device=dev)
        torch.cuda.synchronize()
        e = [torch.cuda.Event(enable_timing=True) for _ in range(4)]

        def cold_leg():
            cf, cb = [], []
            for _ in range(10):
                junk.sum()
                e[0].record(stream)
                fwd()
                e[1].record(stream)
                junk.sum()
                e[2].record(stream)
                bwd()
                e[3].record(stream)
                torch.cuda.synchronize()
                cf.append(e[0].elapsed_time(e[1]))
                cb.append(e[2].elapsed_time(e[3]))
            return {
                "fwd_ms": round(statistics.median(cf), 5),
                "bwd_ms": round(statistics.median(cb), 5),
                # (a launch timed alone between two events: less what the pair of events adds, as calibrated above)
                "fwd_ms_events_corrected": round(max(statistics.median(cf) - event_overhead, 1e-6), 5),
                "bwd_ms_events_corrected": round(max(statistics.median(cb) - event_overhead, 1e-6), 5),
                "fwd_GBps": round(fwd_bytes_per_elem * n_elem / (statistics.median(cf) * 1e-3) / 1e9, 1),
                "bwd_GBps": round(bwd_bytes_per_elem * n_elem / (statistics.median(cb) * 1e-3) / 1e9, 1),
            }

        cold = cold_leg()
        cold["flush_MB"] = args.flush_mb
        if args.cache_policy == "auto" and not cm:
            ext.set_cache_policy("streaming")
            try:
                cold["streaming_policy"] = cold_leg()
            finally:
                ext.set_cache_policy("auto")
        del junk

    # ---- the public autograd path (allocates its outputs, goes through torch.autograd) ----
    autograd_ms = autograd_cpu_ms = autograd_inline_ms = autograd_inline_cpu_ms = None
    if not args.no_autograd:
        a_req = alpha.detach().clone().requires_grad_(True)
        b_req = beta.detach().clone().requires_grad_(True)
        # (the allocator and the autograd engine take a few dozen steps to settle: with ten timed steps
        # after five the figure read 25 % above what the same loop reaches from step 50 on)
        for _ in range(50):
            scan_fn(a_req, b_req).backward(dout)
            a_req.grad = b_req.grad = None
        torch.cuda.synchronize()
        n_auto = max(200, K)
        t0 = time.perf_counter()
        for _ in range(n_auto):
            scan_fn(a_req, b_req).backward(dout)
            a_req.grad = b_req.grad = None
        t_enqueued = time.perf_counter()
        torch.cuda.synchronize()
        autograd_ms = (time.perf_counter() - t0) * 1e3 / n_auto
        autograd_cpu_ms = (t_enqueued - t0) * 1e3 / n_auto  # host time to issue a step; the GPU may lag behind it
        # the same loop with torch's autograd engine running the backward on the calling thread instead of
        # handing it to its device thread (a caller's choice; the hand-over costs up to 30 us per step on some hosts)
        with torch.autograd.set_multithreading_enabled(False):
            for _ in range(20):
                scan_fn(a_req, b_req).backward(dout)
                a_req.grad = b_req.grad = None
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(n_auto):
                scan_fn(a_req, b_req).backward(dout)
                a_req.grad = b_req.grad = None
            t_enqueued = time.perf_counter()
            torch.cuda.synchronize()
            autograd_inline_ms = (time.perf_counter() - t0) * 1e3 / n_auto
            autograd_inline_cpu_ms = (t_enqueued - t0) * 1e3 / n_auto

    # ---- every measured workload, briefly (the headline run only) ----
    workloads = None
    if args.case == "C3_4096" and args.dtype == "bf16" and args.op == "scan" and not args.no_workloads \
            and args.rotate == 1 and fwd_cfg is None and bwd_cfg is None:
        del tensor_sets[1:]
        workloads = [measure_workload(lib, _native, torch, dev, case) for case in BASELINE_CASES]

    # ---- CPU baseline + parity of this very run ----
    cpu = None
    parity = None
    if not args.no_cpu:
        from oracle.torch_loop import torch_gated_bwd, torch_gated_fwd, torch_loop_bwd, torch_loop_fwd

        fwd()
        bwd()
        torch.cuda.synchronize()
        h_gpu, ga_gpu, gb_gpu = h.float().cpu(), galpha.float().cpu(), gbeta.float().cpu()
        if cm:
            h_gpu, ga_gpu, gb_gpu = (t.transpose(1, 2) for t in (h_gpu, ga_gpu, gb_gpu))
        reps, spent = 0, 0.0
        f_times, b_times = [], []
        while reps < 1 or (spent < args.cpu_seconds and reps < 20):
            t0 = time.perf_counter()
            if gated:
                a_ref, h_ref = torch_gated_fwd(alpha_c, beta_c)
                t1 = time.perf_counter()
                ga_ref, gb_ref = torch_gated_bwd(a_ref, beta_c, h_ref, dout_c)
            else:
                h_ref = torch_loop_fwd(alpha_c, beta_c)
                t1 = time.perf_counter()
                ga_ref, gb_ref = torch_loop_bwd(alpha_c, h_ref, dout_c)
            t2 = time.perf_counter()
            f_times.append(t1 - t0)
            b_times.append(t2 - t1)
            spent += t2 - t0
            reps += 1
        cpu_step = statistics.median(f_times) + statistics.median(b_times)

        # gated, 16-bit storage: where sigmoid(gate) sits on a rounding boundary of the storage type the
        # device's exp2/rcp and the CPU's may round alpha to different neighbours; the NumPy oracle is
        # therefore evaluated with both roundings and every element must lie within the tolerance of
        # the interval they span (identical to the plain tolerance wherever no such element matters)
        other = None
        if gated and is_16bit:
            import oracle

            rounding = "bf16" if args.dtype == "bf16" else "f16"
            g32, x32, d32 = alpha_c.float().numpy(), beta_c.float().numpy(), dout_c.float().numpy()
            h_dev = h_gpu.numpy()
            want = (oracle.gated_scan_fwd(g32, x32, rounding), *oracle.gated_scan_bwd(g32, x32, h_dev, d32, rounding))
            alt = (oracle.gated_scan_fwd(g32, x32, rounding, True), *oracle.gated_scan_bwd(g32, x32, h_dev, d32, rounding, True))
            other = {id(t): (w, a) for t, w, a in zip((h_ref, ga_ref, gb_ref), want, alt)}

        def ok(got, want):
            if other is not None:
                import oracle

                w, a = other[id(want)]
                return bool(oracle.within_rounding_envelope(got.numpy(), w, a, tol, tol).all())
            return bool(((got - want).abs() <= tol + tol * want.abs()).all().item())

        names = ("h", "grad_gate", "grad_x") if gated else ("h", "grad_alpha", "grad_beta")
        parity = {
            names[0]: ok(h_gpu, h_ref), names[1]: ok(ga_gpu, ga_ref), names[2]: ok(gb_gpu, gb_ref),
            "rtol": tol, "atol": tol, "outlier_fraction_allowed": 0.0,
            "against": (f"fp32 sequential loop on the CPU, same {args.dtype} inputs"
                        + (", alpha rounded either way where its rounding is ambiguous" if other is not None else "")),
        }
        cpu = {
            "value": round(step_bytes / cpu_step / 1e9, 3),
            "unit": "GB/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"the full workload ({args.case}: bs{bs} seq{seq} d{d}), fwd+bwd, median of {reps} run(s)",
            "ms_per_step": round(cpu_step * 1e3, 2),
            "fwd_ms": round(statistics.median(f_times) * 1e3, 2),
            "bwd_ms": round(statistics.median(b_times) * 1e3, 2),
            "host_cpus": os.cpu_count(),
            "impl": "oracle/torch_loop.py: PyTorch loop over seq on CPU tensors, fp32"
                    + (", gating as torch elementwise ops" if gated else ""),
        }

    # HBM bytes per launch from hardware counters: not measurable from inside this process, so
    # taken from the committed rocprofv3 counter summary when it covers this workload and these
    # launch configurations; each counter is scaled by what it read for a plain copy of known size.
    traffic = {"fwd": None, "bwd": None}
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic_bs8_seq4096_d1024.json")) as f:
            prof = json.load(f)
        if prof["case"] == args.case and args.dtype == "bf16":
            part = prof if args.op == "scan" else prof[args.op]
            scale_r = part["copy"]["bytes_read"] / (part["copy"]["fetch_kib"] * 1024.0)
            scale_w = part["copy"]["bytes_written"] / (part["copy"]["write_kib"] * 1024.0)
            for name in ("fwd", "bwd"):
                if part[name]["config"] == chosen[name] and part[name].get("cols", 1) == chosen[name + "_cols"]:
                    traffic[name] = int(part[name]["fetch_kib"] * 1024 * scale_r + part[name]["write_kib"] * 1024 * scale_w)
    except (OSError, KeyError, ValueError):
        pass

    out = {
        "metric": "fwd+bwd scan ms & achieved HBM GB/s (% peak), bf16 bs8 d1024 seq4096"
        if args.case == "C3_4096" and args.dtype == "bf16" and args.op == "scan"
        else f"fwd+bwd {'gated ' if gated else 'channel-major ' if cm else ''}scan ms & achieved HBM GB/s (% peak), {args.dtype} {args.case}",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic",
        "tensor_sets_in_rotation": len(pointer_sets),
        "cache_policy": args.cache_policy,
        "config": {
            "workload": f"{args.case}: bs{bs} seq{seq} d{d}, {'gated scan of N(0,1) gate and x' if gated else 'recipe ' + recipe}{', tensors (bs, d, seq)' if cm else ''}, {args.dtype} storage / fp32 carries, forward+backward",
            "bs": bs, "seq": seq, "d_model": d,
            "launch_config_fwd_vec_steps_waves": chosen["fwd"],
            "launch_config_bwd_vec_steps_waves": chosen["bwd"],
            "column_tiles_per_workgroup_fwd_bwd": [chosen["fwd_cols"], chosen["bwd_cols"]],
        },
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "pct_of_hbm_peak_no_reuse": rotating.get("pct_of_hbm_peak"),
        # this step against the library's plain streaming kernel moving the same streams in the
        # same protocol (one set of tensors, forward's mix then backward's): machine_stream.one_set_step_ms
        # (the calibration only runs when the timed region above used one set of tensors)
        "step_frac_of_machine": round(machine["one_set_step_ms"] / ms_per_step, 4) if machine else None,
        "fwd_ms": round(fwd_mean, 5),
        "bwd_ms": round(bwd_mean, 5),
        "fwd_ms_median": round(statistics.median(fwd_ms), 5),
        "bwd_ms_median": round(statistics.median(bwd_ms), 5),
        "fwd_ms_p20_p80": quantile_pair(fwd_ms),
        "bwd_ms_p20_p80": quantile_pair(bwd_ms),
        "algorithmic_bytes_per_step": step_bytes,
        "event_samples": len(fwd_ms),
        "event_samples_in_timed_region": in_region,
        "event_pair_overhead_ms": round(event_overhead, 5),
        "event_pair_empty_ms": round(empty_pair, 5),
        "fwd_ms_event_raw": round(raw_f, 5),
        "bwd_ms_event_raw": round(raw_b, 5),
        "fwd_ms_events_corrected": round(fwd_corr, 5),
        "bwd_ms_events_corrected": round(bwd_corr, 5),
        "roofline": {
            "bound": "hbm",
            "kernel": f"{'cm_' if cm else ''}scan_kernel<{kname},...,BWD=true{',GATED' if gated else ''}> (backward scan)",
            "achieved": round(bwd_gbps, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(bwd_gbps / HBM_PEAK_GBPS, 4),
            "frac_no_reuse": rotating.get("bwd_frac"),
            "frac_of_machine": frac_of_machine(machine, "bwd_mix_GBps", bwd_bytes_per_elem * n_elem, rotating.get("bwd_ms")),
            "traffic": traffic["bwd"],
            "bytes_per_launch": bwd_bytes_per_elem * n_elem,
            "avg_launch_ms": round(bwd_mean, 5),
            "avg_launch_ms_events_raw": round(raw_b, 5),
            "avg_launch_ms_events_corrected": round(bwd_corr, 5),
        },
        "roofline_fwd": {
            "bound": "hbm",
            "kernel": f"{'cm_' if cm else ''}scan_kernel<{kname},...,BWD=false{',GATED' if gated else ''}> (forward scan)",
            "achieved": round(fwd_gbps, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(fwd_gbps / HBM_PEAK_GBPS, 4),
            "frac_no_reuse": rotating.get("fwd_frac"),
            "frac_of_machine": frac_of_machine(machine, "fwd_mix_GBps", fwd_bytes_per_elem * n_elem, rotating.get("fwd_ms")),
            "traffic": traffic["fwd"],
            "bytes_per_launch": fwd_bytes_per_elem * n_elem,
            "avg_launch_ms": round(fwd_mean, 5),
            "avg_launch_ms_events_raw": round(raw_f, 5),
            "avg_launch_ms_events_corrected": round(fwd_corr, 5),
        },
        "machine_stream": machine,
        "workloads": workloads,
        "cold_cache": cold,
        "rotating_sets": rotating,
        "autograd_path_ms_per_step": None if autograd_ms is None else round(autograd_ms, 5),
        "autograd_path_host_ms_per_step": None if autograd_cpu_ms is None else round(autograd_cpu_ms, 5),
        "autograd_path_backward_on_calling_thread": None if autograd_inline_ms is None else {
            "ms_per_step": round(autograd_inline_ms, 5), "host_ms_per_step": round(autograd_inline_cpu_ms, 5),
            "how": "torch.autograd.set_multithreading_enabled(False)"},
        "parity": parity,
        "cpu_baseline": cpu,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())

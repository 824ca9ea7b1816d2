#!/usr/bin/env python3
"""Benchmark of the teacher-student step kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-eager] [--no-kernels]

One "step" is the MoCo-v3 ViT-Base teacher-student step of the kernel path:
the momentum EMA over the ViT-B/16 parameter list (152 fp32 tensors,
86,567,656 elements, m = 0.99) on one HIP stream, and the InfoNCE loss forward
+ backward on bf16 q, k of 4096 x 256 (tau = 0.2) on a second stream.  The two
streams carry no dependency on each other (the EMA chain is ordered by its own
stream), so steps overlap on the GPU the way TSPipe's pipeline overlaps teacher
and student work; the timed region ends with a device-wide synchronize.  All
inputs are resident in HBM before the timed region.

Prints ONE JSON line.  `value` is steps per second over exactly K timed steps;
`roofline` is for the dominant kernel (the multi-tensor EMA): algorithmic bytes
per launch (12 B per parameter) over its average duration, measured with HIP
events that the launch itself stamps with the kernel's begin and end, on the
kernel's own stream, inside the timed region;
`cpu_baseline` is the oracle's eager PyTorch restatement of the same step on
the host cores (bounded sample); `eager_gpu_baseline` is the same eager op
chain -- what the reference's plug-ins execute -- on this GPU through
PyTorch-ROCm; `kernels` holds stand-alone timings of every kernel at the other
configurations (informational), each with `cpu_ms` and `eager_gpu_ms` beside it.
"""
import argparse
import gc
import json
import os
import statistics
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

STEP_NCE_WORKGROUPS = 64   # InfoNCE workgroup target inside the step: two key splits, 64 long workgroups
TIMED_EVERY = 4  # one EMA launch in four carries kernel timing events
SETUP_STEPS = 12  # untimed calls before the warm-up steps (resource creation, see run_step_benchmark)
HBM_PEAK_GBS = 8000.0       # MI355X published HBM3E bandwidth
MFMA_BF16_PEAK_TFLOPS = 2500.0
MFMA_F32_PEAK_TFLOPS = 157.3
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "hbm_traffic_pmc_all_kernels.md")


def _ema_traffic():
    """(bytes, commit): HBM bytes one ViT-B EMA launch moves, read from the
    committed rocprofv3 --pmc summary (FETCH_SIZE and WRITE_SIZE runs scaled by
    the same counters on a copy of known size), and the commit those runs were
    made on; (None, None) when the summary is not in the tree.  The value is a
    record of those profiler runs, not a product of this run."""
    nbytes = commit = None
    try:
        for line in open(TRAFFIC_SUMMARY):
            if line.startswith("bench.py roofline.traffic"):
                nbytes = float(line.split("=")[1].split()[0])
            elif line.startswith("collected on commit"):
                commit = line.split()[3]
    except OSError:
        pass
    return nbytes, commit


def _shapes():
    from tspipe_amd.shapes import numel, resnet18_shapes, vit_base_shapes
    return numel, resnet18_shapes(), vit_base_shapes()


def _event_ms(pairs):
    return [a.elapsed_time(b) for a, b in pairs]


def _time_gpu(fn, iters, warmup=5):
    """Median / mean milliseconds of fn() over `iters` runs, HIP events on the current stream."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    pairs = []
    for _ in range(iters):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        pairs.append((a, b))
    torch.cuda.synchronize()
    ms = _event_ms(pairs)
    return statistics.median(ms), sum(ms) / len(ms), min(ms)


def run_step_benchmark(steps, warmup, dev):
    import torch
    import tspipe_amd as ta
    from tspipe_amd import _lib
    from tspipe_amd import ema as ema_mod
    numel, _, vit = _shapes()

    g = torch.Generator().manual_seed(3)
    teacher = [(torch.randn(s, generator=g) * 0.02).to(dev) for s in vit]
    student = [(torch.randn(s, generator=g) * 0.02).to(dev) for s in vit]
    q = torch.nn.functional.normalize(torch.randn(4096, 256, generator=g), dim=1).to(torch.bfloat16).to(dev)
    k = torch.nn.functional.normalize(torch.randn(4096, 256, generator=g), dim=1).to(torch.bfloat16).to(dev)
    q.requires_grad_()
    n_params = sum(numel(s) for s in vit)

    # Teacher and student work sit on their own HIP streams, as in TSPipe's
    # pipeline: the EMA of step i only depends on the EMA of step i-1 (same
    # stream, in order), the loss only on its own inputs, so no event ties the
    # two streams together inside the timed region; its closing
    # torch.cuda.synchronize() waits for both.
    s_ema, s_loss = torch.cuda.Stream(dev), torch.cuda.Stream(dev)
    s_ema.wait_stream(torch.cuda.current_stream(dev))
    s_loss.wait_stream(torch.cuda.current_stream(dev))
    state = {"teacher": teacher, "loss": None}

    # One host thread per stream, as TSPipe's workers are: the loss thread
    # spends most of a step waiting for autograd's device thread (GIL released),
    # and the EMA thread's launches fit into those waits.
    def ema_worker(n, events):
        with torch.cuda.stream(s_ema):
            state["ema_span"] = span = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
            span[0].record()
            for i in range(n):
                ema_mod.kernel_events = events if (events is not None and i % TIMED_EVERY == 0) else None
                state["teacher"] = ta.calculate_updated_momentum_encoder(0.99, student, state["teacher"])
            span[1].record()
        ema_mod.kernel_events = None
        state["ema_enqueued"] = time.perf_counter()

    def loss_worker(n, _events):
        with torch.cuda.stream(s_loss):
            state["loss_span"] = span = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
            span[0].record()
            for _ in range(n):
                q.grad = None
                loss = ta.infonce_loss(q, k, 0.2)
                loss.backward()
                state["loss"] = loss
            span[1].record()
        state["loss_enqueued"] = time.perf_counter()

    # The two host threads live for the whole benchmark, like TSPipe's worker
    # threads: what they keep per thread (pinned staging buffers, autograd's
    # hand-off state) is created once, in the set-up phase.  A phase starts
    # when main and both workers meet at `gate` and ends at `done`.
    gate, done = threading.Barrier(3), threading.Barrier(3)
    phase = {"n": 0, "events": None, "stop": False}
    failures = []

    def worker_loop(fn):
        while True:
            gate.wait()
            if phase["stop"]:
                return
            try:
                fn(phase["n"], phase["events"])
            except BaseException as exc:  # re-raised on the main thread below
                failures.append(exc)
            done.wait()

    workers = [threading.Thread(target=worker_loop, args=(f,), daemon=True) for f in (ema_worker, loss_worker)]
    for w in workers:
        w.start()

    def run_steps(n, events):
        """Runs n steps on the two worker threads; returns the start time and
        the wall time from the moment both are released to the end of a
        device-wide synchronize."""
        phase["n"], phase["events"] = n, events
        torch.cuda.synchronize()
        gate.wait()
        t0 = time.perf_counter()
        done.wait()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        if failures:
            raise failures[0]
        return t0, elapsed

    # Set-up, not steps: the first calls create the output arenas, the chunk
    # tables, autograd's device thread and the allocator's blocks on the two
    # streams.  The W warm-up steps the caller asked for follow.
    run_steps(SETUP_STEPS, None)
    run_steps(warmup, None)
    torch.cuda.synchronize()
    # Every TIMED_EVERY-th EMA launch of the timed region stamps its own begin
    # and end into a pair of HIP events (a timed launch costs the host ~25 us
    # more than a plain one, so timing all of them would slow the step).
    n_timed = (steps + TIMED_EVERY - 1) // TIMED_EVERY
    _lib.prepare_timing_events(dev, n_timed)
    torch.cuda.synchronize()
    events = []
    gc.collect()
    gc.disable()  # as timeit does: no collector pause inside the timed region
    t0, elapsed = run_steps(steps, events)
    gc.enable()
    phase["stop"] = True
    gate.wait()
    for w in workers:
        w.join()
    host_ms = {"ema_thread_enqueue_ms_per_step": round((state["ema_enqueued"] - t0) / steps * 1e3, 4),
               "loss_thread_enqueue_ms_per_step": round((state["loss_enqueued"] - t0) / steps * 1e3, 4),
               # first to last command of each stream, by HIP events on that stream
               "ema_stream_ms_per_step": round(state["ema_span"][0].elapsed_time(state["ema_span"][1]) / steps, 4),
               "loss_stream_ms_per_step": round(state["loss_span"][0].elapsed_time(state["loss_span"][1]) / steps, 4)}
    ema_ms = _event_ms(events)
    assert len(ema_ms) == n_timed
    avg_ema_ms = sum(ema_ms) / len(ema_ms)
    algo_bytes = 12 * n_params
    achieved = algo_bytes / (avg_ema_ms * 1e-3) / 1e9
    # the same launches with nothing else on the GPU (the figure above shares
    # HBM and the CUs with the loss kernels of the other stream)
    _lib.prepare_timing_events(dev, 30)
    torch.cuda.synchronize()
    ema_mod.kernel_events = alone = []
    with torch.cuda.stream(s_ema):
        for _ in range(30):
            state["teacher"] = ta.calculate_updated_momentum_encoder(0.99, student, state["teacher"])
    torch.cuda.synchronize()
    ema_mod.kernel_events = None
    alone_ms = sum(_event_ms(alone)) / len(alone)
    alone_gbs = algo_bytes / (alone_ms * 1e-3) / 1e9
    return {
        "elapsed": elapsed, "n_params": n_params, "loss": float(state["loss"].item()), "host": host_ms,
        "roofline": {"bound": "hbm", "kernel": "ema_multi_kernel", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": _ema_traffic()[0], "traffic_commit": _ema_traffic()[1],
                     "traffic_source": "profiles/hbm_traffic_pmc_all_kernels.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                                       "runs of this script, scaled by a copy of known size); not measured by this run",
                     "algorithmic_bytes_per_launch": algo_bytes,
                     "avg_kernel_ms": round(avg_ema_ms, 4), "launches_timed": len(ema_ms),
                     "note": "inside the timed region the kernel shares the GPU with the InfoNCE stream; 'alone' is "
                             "the same launch with the other stream idle",
                     "alone": {"achieved": round(alone_gbs, 1), "frac": round(alone_gbs / HBM_PEAK_GBS, 4),
                               "avg_kernel_ms": round(alone_ms, 4), "launches_timed": len(alone)}},
    }


def _time_stream(fn, iters=50, warmup=10, batch=4):
    """Median milliseconds per call of fn(): `warmup` untimed calls (at least
    10), then `iters` samples (at least 50), each sample being `batch`
    back-to-back calls between one pair of HIP events on the current stream
    (an event pair around every single call would add its own marker packets
    to a kernel of a few microseconds).  Callers that rotate through several
    buffer sets pass the number of sets as `batch`, so every sample touches
    each set once.  The calls go straight to the C ABI with preallocated
    buffers (about 10 us of host time each); for kernels longer than that the
    figure is device time.  Without rotation a sample is four calls on the same
    buffers."""
    import torch
    for _ in range(max(warmup, 10)):
        fn()
    torch.cuda.synchronize()
    pairs = []
    for _ in range(max(iters, 50)):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(batch):
            fn()
        b.record()
        pairs.append((a, b))
    torch.cuda.synchronize()
    return statistics.median(_event_ms(pairs)) / batch


TIMING_NOTE = ("ms: median over >=50 samples after >=10 warm-up calls; a sample is one HIP-event pair around "
               "`calls_per_sample` back-to-back calls, one per rotating buffer set (4 calls on the same buffers "
               "where the entry names no buffer sets)")
MALL_BYTES = 256 << 20  # Infinity Cache: a working set below this is not an HBM measurement
ONE_SET_NOTE = ("the same call looping on one set: the logits of its selected rows (75 MB) can stay in the Infinity "
                "Cache between calls")
KD_MASKED_LAUNCHES = 2   # row kernel (selected rows and the zero-fill of the others), final reduction


def _cpu_ms(fn, budget_s=1.2, max_iters=20):
    """Median milliseconds of fn() on the host cores: one untimed call, then
    calls until the budget is spent (at least one).  Returns (ms, calls)."""
    t0 = time.perf_counter()
    fn()
    first = time.perf_counter() - t0
    if first > budget_s:
        return first * 1e3, 1
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < max_iters and (not times or time.perf_counter() < t_end):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return statistics.median(times) * 1e3, len(times)


def _eager_gpu_ms(fn, budget_s=1.0, max_iters=30):
    """Wall milliseconds per call of fn(), an eager PyTorch op chain on the GPU:
    two untimed calls, then back-to-back calls until the budget is spent (at
    least three), closed by a device synchronize.  Wall time, because that is
    what such a chain costs its caller: many of them are bound by the host's
    launches rather than by the kernels.  Returns (ms, calls)."""
    import torch
    fn()
    fn()
    torch.cuda.synchronize()
    n, t0 = 0, time.perf_counter()
    while n < 3 or (n < max_iters and time.perf_counter() - t0 < budget_s):
        fn()
        n += 1
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / n * 1e3, n


def run_kernel_table(dev, with_cpu=True, with_eager=True):
    """Stand-alone device timings of each kernel at the other configurations,
    called through the C ABI with preallocated outputs and workspaces; beside
    each, `cpu_ms`: the oracle's eager PyTorch chain for the same operation on
    the same shape, on the host cores (bounded sample, see _cpu_ms)."""
    import torch
    import tspipe_amd as ta
    from oracle import ts_oracle
    from tspipe_amd import _lib, _tables
    from tspipe_amd import ema as ema_mod
    numel, r18, vit = _shapes()
    lib = _lib.lib()
    out = {}
    g = torch.Generator().manual_seed(0)
    stream = _lib.current_stream_ptr(dev)
    if with_cpu:
        cores = os.cpu_count() or 1
        torch.set_num_threads(min(cores, int(os.environ.get("OMP_NUM_THREADS", cores))))

    def cpu(name, fn):
        """Adds the host-side timing of the same operation to out[name]."""
        if not with_cpu:
            return
        ms, calls = _cpu_ms(fn)
        out[name]["cpu_ms"] = round(ms, 3)
        out[name]["cpu_calls"] = calls
        out[name]["gpu_over_cpu"] = round(ms / out[name]["ms"], 1)

    def eager(name, fn):
        """Adds the timing of the same operation as the reference's eager op
        chain on this GPU to out[name]."""
        if not with_eager:
            return
        ms, calls = _eager_gpu_ms(fn)
        out[name]["eager_gpu_ms"] = round(ms, 4)
        out[name]["eager_gpu_calls"] = calls
        out[name]["eager_gpu_over_this"] = round(ms / out[name]["ms"], 1)
        torch.cuda.empty_cache()  # the chain's temporaries go back before the next entry sizes its buffers

    def kd_cpu(s, t, T, mask=None, device="cpu"):
        s_c = s.detach().to(device).requires_grad_()
        t_c = t.detach().to(device)
        m_c = None if mask is None else mask.to(device)

        def f():
            s_c.grad = None
            if m_c is None:
                ts_oracle.kd_soft_target(s_c, t_c, T).backward()
            else:
                ts_oracle.distil_ce(s_c, t_c, m_c, T).backward()
        return f

    def entry(nbytes, ms, note=None, launches=None, working_set=None, sets=1, resident_ms=None, resident_note=None):
        """working_set: bytes the timed calls touch between two visits of the
        same address (all rotating sets together); sets: buffer sets rotated
        through; resident_ms: the same call looping on ONE set, when that set
        is smaller than the Infinity Cache."""
        gbs = nbytes / (ms * 1e-3) / 1e9
        e = {"ms": round(ms, 4), "GB/s": round(gbs, 1), "frac_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
             "algorithmic_bytes": nbytes}
        if launches:
            e["kernel_launches"] = launches
        if working_set is not None:
            e["working_set_bytes"] = int(working_set)
            e["calls_per_sample"] = sets
            if working_set < MALL_BYTES:
                e["cache_note"] = "working set below the 256 MB Infinity Cache: not an HBM figure"
        if resident_ms is not None:
            e["infinity_cache_resident"] = {"ms": round(resident_ms, 4),
                                            "GB/s": round(nbytes / (resident_ms * 1e-3) / 1e9, 1),
                                            "note": resident_note or "the same call looping on one buffer set that fits "
                                                                     "the Infinity Cache"}
        if note:
            e["note"] = note
        return e

    def rotate(fns):
        """One callable that runs fns[0], fns[1], ... in turn."""
        state = {"i": 0}

        def f():
            fns[state["i"] % len(fns)]()
            state["i"] += 1
        f.keep = fns
        return f

    # EMA, stand-alone (no concurrent loss), both parameter lists; kernel-only events
    for name, shapes, m in (("ema_vit_base", vit, 0.99), ("ema_resnet18", r18, 0.996)):
        teacher = [(torch.randn(s, generator=g) * 0.02).to(dev) for s in shapes]
        student = [(torch.randn(s, generator=g) * 0.02).to(dev) for s in shapes]
        st = {"t": teacher}

        def f():
            st["t"] = ta.calculate_target_network_parameters(m, student, st["t"])
        for _ in range(5):
            f()
        torch.cuda.synchronize()
        ema_mod.kernel_events = []
        for _ in range(30):
            f()
        torch.cuda.synchronize()
        ms = _event_ms(ema_mod.kernel_events)
        ema_mod.kernel_events = None
        nbytes = 12 * sum(numel(s) for s in shapes)
        note = "working set below the 256 MB Infinity Cache: not an HBM figure" if name == "ema_resnet18" else None
        out[name] = entry(nbytes, statistics.median(ms), note, 1)
        t_c, s_c = [t.cpu() for t in teacher], [s_.cpu() for s_ in student]
        cpu(name, lambda: ts_oracle.ema_update(m, s_c, t_c))
        eager(name, lambda: ts_oracle.ema_update(m, student, teacher))
        del teacher, student, st, t_c, s_c
    ema_mod.release_pool()

    # student clone fused into the EMA launch (16 B per parameter: read s, t; write s', t')
    teacher = [(torch.randn(s, generator=g) * 0.02).to(dev) for s in vit]
    student = [(torch.randn(s, generator=g) * 0.02).to(dev) for s in vit]
    keep = {}

    def fused():
        keep["c"], keep["t"] = ta.clone_and_update(0.99, student, teacher)
    for _ in range(5):
        fused()
    torch.cuda.synchronize()
    ema_mod.kernel_events = []
    for _ in range(30):
        fused()
    torch.cuda.synchronize()
    ms = _event_ms(ema_mod.kernel_events)
    ema_mod.kernel_events = None
    out["ema_clone_fused_vit_base"] = entry(16 * sum(numel(s) for s in vit), statistics.median(ms),
                                            "kernel-only events", 1)
    t_c, s_c = [t.cpu() for t in teacher], [s_.cpu() for s_ in student]
    cpu("ema_clone_fused_vit_base", lambda: ([p_.detach().clone() for p_ in s_c], ts_oracle.ema_update(0.99, s_c, t_c)))
    eager("ema_clone_fused_vit_base",
          lambda: ([p_.detach().clone() for p_ in student], ts_oracle.ema_update(0.99, student, teacher)))
    del teacher, student, keep, t_c, s_c
    ema_mod.release_pool()

    def kd_call(s, t, mask, T, grad):
        rows, V = s.shape[0] * (s.shape[1] if s.dim() == 3 else 1), s.shape[-1]
        code = _lib.dtype_code(s.dtype)
        ws = torch.empty(lib.ts_kd_workspace_bytes(rows, V, code), dtype=torch.uint8, device=dev)
        loss = torch.empty((), device=dev)
        mptr = None if mask is None else mask.view(torch.uint8).data_ptr()

        def f():
            _lib.check(lib.ts_kd_fwd_bwd(s.data_ptr(), t.data_ptr(), mptr, rows, V, V, V, 1.0 / T, T * T, ws.data_ptr(),
                                         loss.data_ptr(), grad.data_ptr(), V, code, stream), "ts_kd_fwd_bwd")
        f.keep = (ws, loss)
        return f

    # KD small (cfg2, latency) and the same row width at 65536 rows for a bandwidth figure: 8 buffer
    # sets of 78.6 MB each in turn, so that no call finds its operands in the Infinity Cache
    s = (torch.randn(256, 100, generator=g) * 3).to(dev)
    t = (torch.randn(256, 100, generator=g) * 3).to(dev)
    f = kd_call(s, t, None, 4.0, torch.empty_like(s))
    out["kd_256x100_f32"] = entry(3 * 256 * 100 * 4, _time_stream(f), "cfg2 itself; latency-bound: two launches (rows, final sum)", 2,
                                  working_set=3 * 256 * 100 * 4)
    cpu("kd_256x100_f32", kd_cpu(s, t, 4.0))
    eager("kd_256x100_f32", kd_cpu(s, t, 4.0, device=dev))

    # the soft-target benchmark's whole loss at the same shape: hard-label CE + lambda * KD in one pass
    y = torch.randint(0, 100, (256,), generator=g).to(dev)
    g_ce = torch.empty_like(s)
    ws_ce = torch.empty(lib.ts_kd_workspace_bytes(256, 100, _lib.TS_F32), dtype=torch.uint8, device=dev)
    loss_ce = torch.empty((), device=dev)

    def f_kdce():
        _lib.check(lib.ts_kdce_fwd_bwd(s.data_ptr(), t.data_ptr(), None, y.data_ptr(), -100, 256, 100, 100, 100, 0.25,
                                       16.0 * 0.7, 1.0, ws_ce.data_ptr(), loss_ce.data_ptr(), g_ce.data_ptr(), 100,
                                       _lib.TS_F32, stream), "ts_kdce_fwd_bwd")
    out["kdce_256x100_f32"] = entry(3 * 256 * 100 * 4, _time_stream(f_kdce),
                                    "cfg2's shape with the plug-in's hard-label term (train_kd.py:439-453): CE + 0.7 * KD in "
                                    "one pass; latency-bound: two launches, every workgroup counts the labels itself", 2,
                                    working_set=3 * 256 * 100 * 4)
    s_e = s.detach().clone().requires_grad_()

    def kdce_eager():
        s_e.grad = None
        ts_oracle.soft_target_tspipe_loss(s_e, t, y, 4.0, 0.7).backward()
    eager("kdce_256x100_f32", kdce_eager)
    if with_cpu:
        s_c, t_c, y_c = s.detach().cpu().requires_grad_(), t.cpu(), y.cpu()

        def kdce_cpu():
            s_c.grad = None
            ts_oracle.soft_target_tspipe_loss(s_c, t_c, y_c, 4.0, 0.7).backward()
        cpu("kdce_256x100_f32", kdce_cpu)

    def kd_sets(rows, V, n_sets):
        fns = []
        for _ in range(n_sets):
            s_ = (torch.randn(rows, V, generator=g) * 3).to(dev)
            t_ = (torch.randn(rows, V, generator=g) * 3).to(dev)
            fns.append(kd_call(s_, t_, None, 4.0, torch.empty_like(s_)))
            fns[-1].operands = (s_, t_)
        return fns
    fns = kd_sets(65536, 100, 8)
    one = 3 * 65536 * 100 * 4
    out["kd_65536x100_f32"] = entry(one, _time_stream(rotate(fns), batch=8), None, 2, working_set=8 * one, sets=8,
                                    resident_ms=_time_stream(fns[0]))
    cpu("kd_65536x100_f32", kd_cpu(*fns[0].operands, 4.0))
    eager("kd_65536x100_f32", kd_cpu(*fns[0].operands, 4.0, device=dev))
    del fns

    # an ImageNet-sized class count (not one of the benchmark configurations): rows long enough to stream
    fns = kd_sets(32768, 1000, 2)
    one = 3 * 32768 * 1000 * 4
    out["kd_32768x1000_f32"] = entry(one, _time_stream(rotate(fns), batch=2), "not one of the benchmark configurations", 2,
                                     working_set=2 * one, sets=2)
    cpu("kd_32768x1000_f32", kd_cpu(*fns[0].operands, 4.0))
    eager("kd_32768x1000_f32", kd_cpu(*fns[0].operands, 4.0, device=dev))
    del fns, s, t, f

    # DistilBERT-shaped masked KD (cfg3) after a gather of 4 micro-batches.  The selected rows of one
    # set of logits (75 MB) would survive in the Infinity Cache from call to call, so the loss entries
    # take two sets (their own logits, mask and gradient buffers) in turn.
    import ctypes
    row_b = 30522 * 2
    sets = []
    for _ in range(2):
        ps = [(torch.randn(8, 128, 30522, generator=g) * 2).to(torch.bfloat16).to(dev) for _ in range(4)]
        pt = [(torch.randn(8, 128, 30522, generator=g) * 2).to(torch.bfloat16).to(dev) for _ in range(4)]
        sets.append({"s": ps, "t": pt, "mask": (torch.rand(32, 128, generator=g) < 0.15).to(dev)})
    pieces_s, pieces_t, mask = sets[0]["s"], sets[0]["t"], sets[0]["mask"]
    n_sel = int(mask.sum().item())
    n_sel_avg = sum(int(d["mask"].sum().item()) for d in sets) / len(sets)
    s_full = torch.empty(32, 128, 30522, dtype=torch.bfloat16, device=dev)
    dsts = list(s_full.chunk(4))
    for i in range(25):
        if i == 5:
            torch.cuda.synchronize()
            _tables.kernel_events = []
        _tables.copy_segments(pieces_s, dsts)
    torch.cuda.synchronize()
    ms = _event_ms(_tables.kernel_events)
    _tables.kernel_events = None
    out["gather_4x62.5MB_bf16"] = entry(2 * 250036224, statistics.median(ms), "kernel-only events", 1)
    pieces_c = [p_.cpu() for p_ in pieces_s]
    cpu("gather_4x62.5MB_bf16", lambda: ts_oracle.gather(pieces_c))
    eager("gather_4x62.5MB_bf16", lambda: ts_oracle.gather(pieces_s))
    del pieces_c, s_full, dsts
    kd_bytes = int(3 * n_sel_avg * row_b + (4096 - n_sel_avg) * row_b)

    # the loss straight from the four micro-batch outputs (no gather of s or t)
    def pieces_call(d):
        flat_s = [p.view(-1, 30522) for p in d["s"]]
        flat_t = [p.view(-1, 30522) for p in d["t"]]
        grads = [torch.empty_like(p) for p in flat_s]
        ws_p = torch.empty(lib.ts_kd_workspace_bytes(4096, 30522, _lib.TS_BF16), dtype=torch.uint8, device=dev)
        loss_p = torch.empty((), device=dev)
        arr = lambda ts: (ctypes.c_void_p * 4)(*[t.data_ptr() for t in ts])
        a_s, a_t, a_g, a_r = arr(flat_s), arr(flat_t), arr(grads), (ctypes.c_int64 * 4)(1024, 1024, 1024, 1024)
        mptr = d["mask"].view(torch.uint8).data_ptr()

        def f():
            _lib.check(lib.ts_kdce_pieces_fwd_bwd(a_s, a_t, a_g, a_r, 4, mptr, None, 0, 30522, 0.5, 4.0, 0.0,
                                                  ws_p.data_ptr(), loss_p.data_ptr(), _lib.TS_BF16, stream),
                       "ts_kdce_pieces_fwd_bwd")
        f.keep = (flat_s, flat_t, grads, ws_p, loss_p, a_s, a_t, a_g, a_r)
        return f
    fns = [pieces_call(d) for d in sets]
    out["kd_masked_4_pieces_8x128x30522_bf16"] = entry(
        kd_bytes, _time_stream(rotate(fns), batch=2),
        "same loss read from the 4 micro-batch outputs in place: replaces 2 gathers (2 x ~78 us) + the call below",
        KD_MASKED_LAUNCHES, working_set=2 * 3 * 4096 * row_b, sets=2, resident_ms=_time_stream(fns[0]),
        resident_note=ONE_SET_NOTE)
    del fns
    # the gathered form: s, t of each set concatenated first (untimed), the pieces released
    for d in sets:
        d["s_full"] = ta.gather([ta.Batch(p) for p in d["s"]])
        d["t_full"] = ta.gather([ta.Batch(p) for p in d["t"]])
        d["s"] = d["t"] = None
    del pieces_s, pieces_t
    fns = [kd_call(d["s_full"], d["t_full"], d["mask"], 2.0, torch.empty_like(d["s_full"])) for d in sets]
    out["kd_masked_32x128x30522_bf16"] = entry(
        kd_bytes, _time_stream(rotate(fns), batch=2),
        f"n_sel={n_sel_avg:.0f} on average; bytes = read s,t + write grad for selected rows, zero-fill of the other rows",
        KD_MASKED_LAUNCHES, working_set=2 * 3 * 4096 * row_b, sets=2, resident_ms=_time_stream(fns[0]),
        resident_note=ONE_SET_NOTE)
    # the rest of TSPipeDistiller.loss_fn on the same two sets (not benchmark configurations of their own):
    # KD + masked-LM cross-entropy in one pass (alpha_mlm > 0, restrict_ce_to_mask), the squared-error term on
    # the logits, the cosine term on [32, 128, 768] hidden states
    def kdce_call(d, grad):
        labels = torch.full((4096,), -100, dtype=torch.long)
        m_host = d["mask"].reshape(-1).cpu()
        labels[m_host] = torch.randint(0, 30522, (int(m_host.sum()),), generator=g)
        labels = labels.to(dev)
        ws = torch.empty(lib.ts_kd_workspace_bytes(4096, 30522, _lib.TS_BF16), dtype=torch.uint8, device=dev)
        loss = torch.empty((), device=dev)
        mptr = d["mask"].view(torch.uint8).data_ptr()

        def f():
            _lib.check(lib.ts_kdce_fwd_bwd(d["s_full"].data_ptr(), d["t_full"].data_ptr(), mptr, labels.data_ptr(), -100,
                                           4096, 30522, 30522, 30522, 0.5, 4.0 * 0.5, 2.0, ws.data_ptr(), loss.data_ptr(),
                                           grad.data_ptr(), 30522, _lib.TS_BF16, stream), "ts_kdce_fwd_bwd")
        f.keep = (labels, ws, loss, grad)
        return f

    def mse_call(d, grad):
        ws = torch.empty(lib.ts_mse_workspace_bytes(4096, 30522), dtype=torch.uint8, device=dev)
        loss = torch.empty((), device=dev)
        mptr = d["mask"].view(torch.uint8).data_ptr()

        def f():
            _lib.check(lib.ts_mse_fwd_bwd(d["s_full"].data_ptr(), d["t_full"].data_ptr(), mptr, 4096, 30522, 30522, 30522,
                                          0.1, 0, 0, ws.data_ptr(), loss.data_ptr(), grad.data_ptr(), 30522, _lib.TS_BF16,
                                          stream), "ts_mse_fwd_bwd")
        f.keep = (ws, loss, grad)
        return f
    grads = [torch.empty_like(d["s_full"]) for d in sets]
    fns2 = [kdce_call(d, gr) for d, gr in zip(sets, grads)]
    out["kdce_masked_32x128x30522_bf16"] = entry(
        kd_bytes, _time_stream(rotate(fns2), batch=2),
        "KD + cross-entropy on the masked tokens in one pass (distiller.py:719-744), two sets of logits in turn", 2,
        working_set=2 * 3 * 4096 * row_b, sets=2)
    sg = sets[0]["s_full"].detach().requires_grad_()
    lab2d = fns2[0].keep[0].view(32, 128)

    def kdce_eager():  # distiller.py:719-744 with alpha_ce 0.5, alpha_mlm 2, temperature 2, CE restricted to the mask
        sg.grad = None
        ts_oracle.distil_loss(sg, sets[0]["t_full"], None, None, lab2d, sets[0]["mask"], 0.5, 2.0, 0.0, 2.0, True).backward()
    eager("kdce_masked_32x128x30522_bf16", kdce_eager)
    sg.grad = None
    del sg, lab2d
    fns2 = [mse_call(d, gr) for d, gr in zip(sets, grads)]
    out["mse_masked_32x128x30522_bf16"] = entry(
        kd_bytes, _time_stream(rotate(fns2), batch=2),
        "squared-error term on the masked tokens (distiller.py:751-755): a workgroup per row, final sum", 2,
        working_set=2 * 3 * 4096 * row_b, sets=2)
    del fns2, grads
    hid = [torch.randn(4096, 768, generator=g).to(dev) for _ in range(2)]
    ghid = torch.empty_like(hid[0])
    ws_c = torch.empty(lib.ts_cosine_workspace_bytes(4096), dtype=torch.uint8, device=dev)
    loss_c = torch.empty((), device=dev)

    def f_cos():
        _lib.check(lib.ts_cosine_fwd_bwd(hid[0].data_ptr(), hid[1].data_ptr(), sets[0]["mask"].view(torch.uint8).data_ptr(),
                                         4096, 768, 1.0, ws_c.data_ptr(), loss_c.data_ptr(), ghid.data_ptr(), _lib.TS_F32,
                                         stream), "ts_cosine_fwd_bwd")
    n0 = int(sets[0]["mask"].sum().item())
    out["cosine_masked_4096x768_f32"] = entry(
        (3 * n0 + (4096 - n0)) * 768 * 4, _time_stream(f_cos),
        "cosine term on the hidden states (distiller.py:756-770); latency-bound", 2, working_set=3 * 4096 * 768 * 4)
    del hid, ghid
    d = sets[0]
    eager("kd_masked_32x128x30522_bf16", kd_cpu(d["s_full"], d["t_full"], 2.0, d["mask"], device=dev))
    sp_g, tp_g = list(d["s_full"].chunk(4)), list(d["t_full"].chunk(4))

    def pieces_eager():  # the reference's order: gather both outputs, then the loss
        s_all = ts_oracle.gather(sp_g).requires_grad_()
        ts_oracle.distil_ce(s_all, ts_oracle.gather(tp_g), d["mask"], 2.0).backward()
    eager("kd_masked_4_pieces_8x128x30522_bf16", pieces_eager)
    del sp_g, tp_g
    if with_cpu:
        s_c, t_c, m_c = d["s_full"].cpu(), d["t_full"].cpu(), d["mask"].cpu()
        sp_c, tp_c = list(s_c.chunk(4)), list(t_c.chunk(4))
        cpu("kd_masked_32x128x30522_bf16", kd_cpu(s_c, t_c, 2.0, m_c))

        def pieces_cpu():  # the reference's order: gather both outputs, then the loss
            s_all = ts_oracle.gather(sp_c).requires_grad_()
            ts_oracle.distil_ce(s_all, ts_oracle.gather(tp_c), m_c, 2.0).backward()
        cpu("kd_masked_4_pieces_8x128x30522_bf16", pieces_cpu)
        del s_c, t_c, m_c, sp_c, tp_c
    del fns, sets

    # InfoNCE: cfg4 (single pair), the symmetric two-pair call of MoCo-v3's contrastive_loss, and a
    # batch four times as large, where the fixed costs of the three launches weigh less
    def nce_entry(name, n, pairs, note=None, dtype=torch.bfloat16):
        mk = lambda: torch.nn.functional.normalize(torch.randn(n, 256, generator=g), dim=1).to(dtype).to(dev)
        q1, k1 = mk(), mk()
        q2, k2 = (mk(), mk()) if pairs == 2 else (None, None)
        ws = torch.empty(lib.ts_infonce_workspace_bytes(n, 256, pairs), dtype=torch.uint8, device=dev)
        loss, d1 = torch.empty((), device=dev), torch.empty_like(q1)
        d2 = torch.empty_like(q1) if pairs == 2 else None
        ptr = lambda t: None if t is None else t.data_ptr()

        def f():
            _lib.check(lib.ts_infonce_fwd_bwd(ptr(q1), ptr(k1), ptr(q2), ptr(k2), n, 256, 0.2, ws.data_ptr(),
                                              loss.data_ptr(), ptr(d1), ptr(d2), _lib.dtype_code(dtype), stream),
                       "ts_infonce_fwd_bwd")
        ms = _time_stream(f)
        flops = pairs * 2 * 2 * n * n * 256
        peak_key, peak = (("frac_mfma_bf16_peak", MFMA_BF16_PEAK_TFLOPS) if dtype != torch.float32
                          else ("frac_mfma_f32_peak", MFMA_F32_PEAK_TFLOPS))
        e = {"ms": round(ms, 4), "TFLOP/s": round(flops / (ms * 1e-3) / 1e12, 1),
             peak_key: round(flops / (ms * 1e-3) / 1e12 / peak, 4),
             "algorithmic_flop": flops, "kernel_launches": 3 if dtype != torch.float32 else 4}
        if note:
            e["note"] = note
        out[name] = e
        qc = [t.cpu().requires_grad_() for t in ((q1, q2) if pairs == 2 else (q1,))]
        kc = [t.cpu() for t in ((k1, k2) if pairs == 2 else (k1,))]

        def f_cpu():
            for t in qc:
                t.grad = None
            sum(ts_oracle.infonce(a, b, 0.2) for a, b in zip(qc, kc)).backward()
        cpu(name, f_cpu)
        qg = [t.detach().clone().requires_grad_() for t in ((q1, q2) if pairs == 2 else (q1,))]
        kg = (k1, k2) if pairs == 2 else (k1,)

        def f_eager():
            for t in qg:
                t.grad = None
            sum(ts_oracle.infonce(a, b, 0.2) for a, b in zip(qg, kg)).backward()
        eager(name, f_eager)
    nce_entry("infonce_4096x256_bf16", 4096, 1)
    nce_entry("infonce_2_pairs_4096x256_bf16", 4096, 2, "both directions of the symmetric loss in one call")
    nce_entry("infonce_16384x256_bf16", 16384, 1,
              "not one of the benchmark configurations: the same kernels at 16x the work")
    nce_entry("infonce_4096x256_f32", 4096, 1,
              "fp32 embeddings (the reference's TSPipe MoCo run is fp32): fp32-MFMA kernels, every product and sum in "
              "fp32; not one of the benchmark configurations", dtype=torch.float32)

    # BYOL loss (latency only)
    loss = torch.empty((), device=dev)
    o = [torch.randn(256, 128, generator=g).to(dev) for _ in range(4)]
    g1, g2 = torch.empty_like(o[0]), torch.empty_like(o[1])
    wsb = torch.empty(512, device=dev)

    def f():
        _lib.check(lib.ts_byol_fwd_bwd(o[0].data_ptr(), o[3].data_ptr(), o[1].data_ptr(), o[2].data_ptr(), 256, 128,
                                       wsb.data_ptr(), loss.data_ptr(), g1.data_ptr(), g2.data_ptr(), _lib.TS_F32,
                                       stream), "ts_byol_fwd_bwd")
    out["byol_256x128_f32"] = {"ms": round(_time_stream(f), 4), "note": "latency-bound", "kernel_launches": 2}
    oc = [t.cpu() for t in o]
    oc[0].requires_grad_()
    oc[1].requires_grad_()

    def byol_cpu():
        oc[0].grad = oc[1].grad = None
        ts_oracle.byol_contrastive_loss(*oc).backward()
    cpu("byol_256x128_f32", byol_cpu)
    og = [t.detach().clone() for t in o]
    og[0].requires_grad_()
    og[1].requires_grad_()

    def byol_eager():
        og[0].grad = og[1].grad = None
        ts_oracle.byol_contrastive_loss(*og).backward()
    eager("byol_256x128_f32", byol_eager)

    # DeferredBatchNorm (cfg5): 8 different micro-batches of [32, 256, 56, 56] (822 MB of inputs, and as much
    # again of outputs) taken in turn, as the configuration has them: no call finds its micro-batch in the
    # Infinity Cache.  Statistics only, statistics + normalise, backward, and the configuration's whole sequence.
    MB = 8
    dgen = torch.Generator(device=dev).manual_seed(5)
    xs = [torch.randn(32, 256, 56, 56, generator=dgen, device=dev) * 1.5 + 0.5 for _ in range(MB)]
    ys = [torch.empty_like(xs[0]) for _ in range(MB)]
    x, y = xs[0], ys[0]
    z = lambda n: torch.zeros(n, device=dev)  # noqa: E731
    wsn, acc_s, acc_q, mean_b, inv_b = z(768), z(256), z(256), z(256), z(256)
    run_m, run_v, nbt = z(256), torch.ones(256, device=dev), torch.zeros((), dtype=torch.int64, device=dev)
    gamma, beta = torch.rand(256, generator=g).to(dev) + 0.5, (torch.randn(256, generator=g) * 0.1).to(dev)
    one_x = x.numel() * 4

    def stats_of(xi):
        def f():
            _lib.check(lib.ts_bn_stats(xi.data_ptr(), 32, 256, 3136, wsn.data_ptr(), acc_s.data_ptr(), acc_q.data_ptr(),
                                       mean_b.data_ptr(), inv_b.data_ptr(), 1e-5, stream), "ts_bn_stats")
        return f

    def apply_of(xi, yi):
        def f():
            _lib.check(lib.ts_bn_apply(xi.data_ptr(), yi.data_ptr(), mean_b.data_ptr(), inv_b.data_ptr(), gamma.data_ptr(),
                                       beta.data_ptr(), 32, 256, 3136, 0, 1e-5, stream), "ts_bn_apply")
        return f

    def both_of(xi, yi):
        st_, ap_ = stats_of(xi), apply_of(xi, yi)

        def f():
            st_()
            ap_()
        return f
    out["bn_stats_32x256x56x56_f32"] = entry(one_x, _time_stream(rotate([stats_of(xi) for xi in xs]), batch=MB), None, 1,
                                             working_set=MB * one_x, sets=MB, resident_ms=_time_stream(stats_of(x)))
    out["bn_stats_normalise_32x256x56x56_f32"] = entry(
        3 * one_x, _time_stream(rotate([both_of(xi, yi) for xi, yi in zip(xs, ys)]), batch=MB),
        "ts_bn_stats and ts_bn_apply as two separate calls: the stand-alone statistics pass streams x past the caches, "
        "so the second call reads it from HBM again; ts_bn_forward_train (next entry) is the call for this sequence", 2,
        working_set=2 * MB * one_x, sets=MB, resident_ms=_time_stream(both_of(x, y)))
    ws4, par = z(4 * 256), {"p": 0}

    def fused_of(xi, yi):
        def f():
            _lib.check(lib.ts_bn_forward_train(xi.data_ptr(), yi.data_ptr(), gamma.data_ptr(), beta.data_ptr(), 32, 256,
                                               3136, acc_s.data_ptr(), acc_q.data_ptr(), mean_b.data_ptr(),
                                               inv_b.data_ptr(), ws4.data_ptr(), par["p"], 1e-5, stream),
                       "ts_bn_forward_train")
            par["p"] ^= 1
        return f
    out["bn_forward_train_32x256x56x56_f32"] = entry(
        3 * one_x, _time_stream(rotate([fused_of(xi, yi) for xi, yi in zip(xs, ys)]), batch=MB),
        "the same work in 2 launches (what DeferredBatchNorm.forward runs)", 2,
        working_set=2 * MB * one_x, sets=MB, resident_ms=_time_stream(fused_of(x, y)))

    def commit():
        _lib.check(lib.ts_bn_commit(acc_s.data_ptr(), acc_q.data_ptr(), run_m.data_ptr(), run_v.data_ptr(), nbt.data_ptr(),
                                    256, float(MB * 32 * 3136), 0.1, stream), "ts_bn_commit")

    # the configuration's own sequence: 8 micro-batches tracked (and normalised), then one commit
    track8 = [stats_of(xi) for xi in xs]
    fwd8 = [fused_of(xi, yi) for xi, yi in zip(xs, ys)]

    def cfg5_track():
        for f_ in track8:
            f_()
        commit()

    def cfg5_forward():
        for f_ in fwd8:
            f_()
        commit()
    out["bn_cfg5_track_x8_commit"] = entry(MB * one_x, _time_stream(cfg5_track, batch=1), "8 x _track over 8 different "
                                           "micro-batches + _commit (momentum 0.1): one mini-batch of the configuration",
                                           MB + 1, working_set=MB * one_x, sets=1)
    out["bn_cfg5_forward_x8_commit"] = entry(3 * MB * one_x, _time_stream(cfg5_forward, batch=1), "8 x training forward "
                                             "(statistics + normalise with gamma, beta) + _commit: what DeferredBatchNorm "
                                             "runs for one mini-batch of the configuration", 2 * MB + 1,
                                             working_set=2 * MB * one_x, sets=1)
    del ys, y
    dys = [torch.randn(32, 256, 56, 56, generator=dgen, device=dev) for _ in range(4)]
    dxs = [torch.empty_like(xs[0]) for _ in range(4)]
    dy = dys[0]
    dgam, dbet = z(256), z(256)

    def bwd_of(xi, dyi, dxi):
        def f():
            _lib.check(lib.ts_bn_backward(xi.data_ptr(), dyi.data_ptr(), mean_b.data_ptr(), inv_b.data_ptr(),
                                          gamma.data_ptr(), dxi.data_ptr(), dgam.data_ptr(), dbet.data_ptr(), ws4.data_ptr(),
                                          par["p"], 32, 256, 3136, 1, stream), "ts_bn_backward")
            par["p"] ^= 1
        return f
    out["bn_backward_32x256x56x56_f32"] = entry(
        5 * one_x, _time_stream(rotate([bwd_of(xi, dyi, dxi) for xi, dyi, dxi in zip(xs, dys, dxs)]), batch=4),
        "bytes = read x,dy twice + write dx", 2, working_set=3 * 4 * one_x, sets=4)
    del dxs
    # the reference's module arithmetic on this GPU: its buffers moved to the device
    ora_g = ts_oracle.DeferredBNOracle(256, chunks=1 << 30, weight=gamma, bias=beta)
    for attr in ("running_mean", "running_var", "num_batches_tracked", "sum", "sum_squares"):
        setattr(ora_g, attr, getattr(ora_g, attr).to(dev))
    it = {"i": 0}

    def next_x():
        it["i"] += 1
        return xs[it["i"] % MB]
    eager("bn_stats_32x256x56x56_f32", lambda: ora_g.track(next_x()))
    eager("bn_stats_normalise_32x256x56x56_f32", lambda: ora_g.forward(next_x()))
    eager("bn_forward_train_32x256x56x56_f32", lambda: ora_g.forward(next_x()))

    def cfg5_track_eager():
        for xi in xs:
            ora_g.track(xi)
        ora_g.commit()

    def cfg5_forward_eager():
        for xi in xs:
            ora_g.forward(xi)
        ora_g.commit()
    eager("bn_cfg5_track_x8_commit", cfg5_track_eager)
    eager("bn_cfg5_forward_x8_commit", cfg5_forward_eager)
    if with_eager:  # four graphs over four micro-batches in turn, like the entry above
        we, be = gamma.clone().requires_grad_(), beta.clone().requires_grad_()
        xes = [xi.clone().requires_grad_() for xi in xs[:4]]
        yes = [torch.nn.functional.batch_norm(xe, None, None, we, be, True, 0.0, 1e-5) for xe in xes]

        def bn_bwd_eager():
            it["i"] += 1
            i = it["i"] % 4
            xes[i].grad = we.grad = be.grad = None
            yes[i].backward(dys[i], retain_graph=True)
        eager("bn_backward_32x256x56x56_f32", bn_bwd_eager)
        del xes, yes, we, be
    if with_cpu:
        x_c, dy_c, gamma_c, beta_c = x.cpu(), dy.cpu(), gamma.cpu(), beta.cpu()
        ora = ts_oracle.DeferredBNOracle(256, chunks=1 << 30, weight=gamma_c, bias=beta_c)
        cpu("bn_stats_32x256x56x56_f32", lambda: ora.track(x_c))
        cpu("bn_stats_normalise_32x256x56x56_f32", lambda: ora.forward(x_c))
        cpu("bn_forward_train_32x256x56x56_f32", lambda: ora.forward(x_c))
        xg, wg, bg = x_c.clone().requires_grad_(), gamma_c.clone().requires_grad_(), beta_c.clone().requires_grad_()
        y_c = torch.nn.functional.batch_norm(xg, None, None, wg, bg, True, 0.0, 1e-5)

        def bn_bwd_cpu():
            xg.grad = wg.grad = bg.grad = None
            y_c.backward(dy_c, retain_graph=True)
        cpu("bn_backward_32x256x56x56_f32", bn_bwd_cpu)
    del xs, dys

    # The late stages of a ResNet: many channels, planes of 7 x 7.  A plane is shorter than a wavefront's
    # round of loads, so these shapes take the flat-tile kernels; the whole activation (25.7 MB) stays in
    # the caches, and the call is a matter of launches and latency.
    xs7 = torch.randn(256, 512, 7, 7, generator=dgen, device=dev) * 1.5 + 0.5
    ys7, dy7, dx7 = torch.empty_like(xs7), torch.randn(256, 512, 7, 7, generator=dgen, device=dev), torch.empty_like(xs7)
    g7, b7 = torch.rand(512, generator=g).to(dev) + 0.5, (torch.randn(512, generator=g) * 0.1).to(dev)
    s7, q7, m7, i7, dg7, db7, ws7, par7 = z(512), z(512), z(512), z(512), z(512), z(512), z(4 * 512), {"p": 0}
    one7 = xs7.numel() * 4

    def fwd7():
        _lib.check(lib.ts_bn_forward_train(xs7.data_ptr(), ys7.data_ptr(), g7.data_ptr(), b7.data_ptr(), 256, 512, 49,
                                           s7.data_ptr(), q7.data_ptr(), m7.data_ptr(), i7.data_ptr(), ws7.data_ptr(),
                                           par7["p"], 1e-5, stream), "ts_bn_forward_train")
        par7["p"] ^= 1

    def bwd7():
        _lib.check(lib.ts_bn_backward(xs7.data_ptr(), dy7.data_ptr(), m7.data_ptr(), i7.data_ptr(), g7.data_ptr(),
                                      dx7.data_ptr(), dg7.data_ptr(), db7.data_ptr(), ws7.data_ptr(), par7["p"], 256, 512,
                                      49, 1, stream), "ts_bn_backward")
        par7["p"] ^= 1
    small_note = "planes of 49 values: the flat-tile kernels (a workgroup per 4 KB of the tensor as it lies in memory)"
    out["bn_forward_train_256x512x7x7_f32"] = entry(3 * one7, _time_stream(fwd7), small_note, 2, working_set=2 * one7)
    out["bn_backward_256x512x7x7_f32"] = entry(5 * one7, _time_stream(bwd7), small_note, 2, working_set=3 * one7)
    ora7 = ts_oracle.DeferredBNOracle(512, chunks=1 << 30, weight=g7, bias=b7)
    for attr in ("running_mean", "running_var", "num_batches_tracked", "sum", "sum_squares"):
        setattr(ora7, attr, getattr(ora7, attr).to(dev))
    eager("bn_forward_train_256x512x7x7_f32", lambda: ora7.forward(xs7))
    if with_eager:
        w7e, b7e, x7e = g7.clone().requires_grad_(), b7.clone().requires_grad_(), xs7.clone().requires_grad_()
        y7e = torch.nn.functional.batch_norm(x7e, None, None, w7e, b7e, True, 0.0, 1e-5)

        def bn7_bwd_eager():
            x7e.grad = w7e.grad = b7e.grad = None
            y7e.backward(dy7, retain_graph=True)
        eager("bn_backward_256x512x7x7_f32", bn7_bwd_eager)
        del w7e, b7e, x7e, y7e

    # A gather of a few small pieces (per-micro-batch outputs, labels, embeddings): segments in the kernel's
    # arguments, no table.  Host time is what such a call costs; the entry is the device side of it.
    small = [torch.randn(64, 256, generator=dgen, device=dev) for _ in range(4)]
    joined = torch.empty(256, 256, device=dev)
    src_arr = (ctypes.c_void_p * 4)(*[t_.data_ptr() for t_ in small])
    dst_arr = (ctypes.c_void_p * 4)(*[joined.data_ptr() + i * 65536 for i in range(4)])
    len_arr = (ctypes.c_int64 * 4)(*([65536] * 4))

    def few():
        _lib.check(lib.ts_copy_few(src_arr, dst_arr, len_arr, 4, stream), "ts_copy_few")
    out["gather_4x64KB_f32"] = entry(2 * 4 * 65536, _time_stream(few), "ts_copy_few: four segments in the kernel arguments",
                                     1, working_set=2 * 4 * 65536)
    eager("gather_4x64KB_f32", lambda: ts_oracle.gather(small))
    return out


def run_cpu_baseline(budget_s=12.0):
    """The oracle's eager-PyTorch step (reference arithmetic) on the host cores."""
    import torch
    from oracle import ts_oracle
    numel, _, vit = _shapes()
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(3)
    teacher = [torch.randn(s, generator=g) * 0.02 for s in vit]
    student = [torch.randn(s, generator=g) * 0.02 for s in vit]
    q = torch.nn.functional.normalize(torch.randn(4096, 256, generator=g), dim=1).to(torch.bfloat16).requires_grad_()
    k = torch.nn.functional.normalize(torch.randn(4096, 256, generator=g), dim=1).to(torch.bfloat16)

    def step(t):
        t = ts_oracle.ema_update(0.99, student, t, skip_none=True)
        q.grad = None
        ts_oracle.infonce(q, k, 0.2).backward()
        return t

    teacher = step(teacher)  # warm-up
    n, t0 = 0, time.perf_counter()
    while True:
        teacher = step(teacher)
        n += 1
        el = time.perf_counter() - t0
        if el > budget_s or n >= 2000:
            break
    return {"value": round(n / el, 4), "unit": "steps/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{n} full steps (EMA over 152 tensors / 86.6M params per-tensor loop + InfoNCE 4096x256 bf16 "
                      f"fwd+bwd, eager PyTorch on CPU) in {el:.1f} s"}


def run_eager_gpu_baseline(dev, budget_s=4.0):
    """The oracle's eager-PyTorch step on this GPU: the op chain the reference's
    plug-ins execute (per-tensor EMA loop, normalize / einsum / cross-entropy
    and its backward), issued from one host thread in the order TSPipe's compute
    thread runs them, through PyTorch-ROCm."""
    import torch
    from oracle import ts_oracle
    _, _, vit = _shapes()
    g = torch.Generator().manual_seed(3)
    teacher = [(torch.randn(s, generator=g) * 0.02).to(dev) for s in vit]
    student = [(torch.randn(s, generator=g) * 0.02).to(dev) for s in vit]
    q = torch.nn.functional.normalize(torch.randn(4096, 256, generator=g), dim=1).to(torch.bfloat16).to(dev).requires_grad_()
    k = torch.nn.functional.normalize(torch.randn(4096, 256, generator=g), dim=1).to(torch.bfloat16).to(dev)

    def step(t):
        t = ts_oracle.ema_update(0.99, student, t, skip_none=True)
        q.grad = None
        ts_oracle.infonce(q, k, 0.2).backward()
        return t

    for _ in range(5):
        teacher = step(teacher)
    torch.cuda.synchronize()
    n, t0 = 0, time.perf_counter()
    while n < 20 or (n < 2000 and time.perf_counter() - t0 < budget_s):
        teacher = step(teacher)
        n += 1
    torch.cuda.synchronize()
    el = time.perf_counter() - t0
    return {"value": round(n / el, 2), "unit": "steps/s", "kind": "port", "device": torch.cuda.get_device_name(dev),
            "sample": f"{n} full steps (the same eager PyTorch op chain as cpu_baseline, on the GPU through PyTorch-ROCm, "
                      f"one host thread, one stream) in {el:.1f} s"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel table")
    ap.add_argument("--no-eager", action="store_true",
                    help="skip the eager-PyTorch-on-GPU legs (thousands of small launches: leave them out under a profiler)")
    ap.add_argument("--nce-workgroups", type=int, default=STEP_NCE_WORKGROUPS,
                    help="workgroup target of the InfoNCE kernels inside the step (the kernel table uses the default, 256)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build measures one GPU only; the kernel path has no cross-GPU exchange "
                 "(each pipeline partition runs it on its own parameters). Run with --gpus 1.")

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    from tspipe_amd import _lib
    _lib.lib()  # fail loudly if the HIP library is missing

    # Inside the step the loss shares the GPU with the EMA stream: fewer, longer
    # InfoNCE workgroups (less partial-sum traffic, CUs left to the EMA) make
    # the step shorter although the loss kernel alone gets slower.
    from tspipe_amd import set_infonce_workgroup_target
    set_infonce_workgroup_target(args.nce_workgroups)
    res = run_step_benchmark(args.steps, args.warmup, dev)
    set_infonce_workgroup_target(0)
    line = {
        "metric": "TS-steps/sec at ViT-B momentum (EMA over 86.6M fp32 params || InfoNCE 4096x256 bf16 fwd+bwd)",
        "value": round(args.steps / res["elapsed"], 2),
        "unit": "steps/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(res["elapsed"] / args.steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "MoCo-v3 ViT-Base step: fp32 EMA over ViT-B/16 shapes (152 tensors, 86,567,656 params, "
                               "m=0.99) + InfoNCE fwd+bwd on bf16 q,k 4096x256, tau=0.2, two HIP streams",
                   "ema_tensors": 152, "ema_params": res["n_params"], "infonce_n": 4096, "infonce_c": 256,
                   "infonce_workgroup_target": args.nce_workgroups},
        "roofline": res["roofline"],
        "loss": res["loss"],
        "host": res["host"],
    }
    if not args.no_kernels:
        line["kernels"] = run_kernel_table(dev, with_cpu=not args.no_cpu, with_eager=not args.no_eager)
        line["kernels_timing_note"] = TIMING_NOTE
        line["kernels_cpu_note"] = ("cpu_ms: the oracle's eager PyTorch chain for the same operation and shape on "
                                    f"{min(os.cpu_count() or 1, int(os.environ.get('OMP_NUM_THREADS', os.cpu_count() or 1)))} "
                                    "host threads, median of up to 20 calls within ~1.2 s (a single call when one takes longer)")
        line["kernels_eager_gpu_note"] = ("eager_gpu_ms: the same eager PyTorch chain (the reference's arithmetic) on this GPU, "
                                          "wall time per call over up to 30 back-to-back calls within ~1 s, temporaries and "
                                          "launch overhead included as the reference's caller pays them")
    if not args.no_eager:
        line["eager_gpu_baseline"] = run_eager_gpu_baseline(dev)
        line["eager_gpu_baseline"]["this_over_eager_gpu"] = round(line["value"] / line["eager_gpu_baseline"]["value"], 1)
    else:
        line["eager_gpu_baseline"] = None
    if not args.no_cpu:
        line["cpu_baseline"] = run_cpu_baseline()
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))


if __name__ == "__main__":
    main()

"""Benchmark of the fused-region hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c5]

A step is one call of the hot path on one batch of synthetic, seeded input
already resident in HBM: plan lookup + argument marshalling + output allocation
+ kernel launches + the wait for the kept-row counts (what a caller of the
operator waits for; the counts arrive before the kernels end, so consecutive
calls overlap on the stream).  K steps are timed back to back between two device
synchronisations, the way the reference times a call (functs/utils/evaluate.py:179-190).
Prints ONE JSON line.  `value` is the per-call latency of the headline workload
(c5: ParallelMap over 16 YOLOv3-style images) through the TorchScript route, i.e.
the scripted program whose fused regions run as tssa::ParallelFunctor;
`drained_latency_us` is the same call with the device drained after every call
(`drain_floor_us`: a 256-byte copy kernel drained the same way);
`region_api_latency_us` is the same regions driven from Python through ctypes;
`compiled_kernels` says whether the regions ran ahead-of-time compiled kernels
(functs_amd.aot) or the bytecode interpreter (`--interpreter` forces the latter);
`per_config` repeats the measurement for every benchmark configuration that is
implemented, each with its CPU baseline, the library's copy kernel on the same
bytes, the operator's host time by section and, for row compactions (whose default
is the kernel generated from the region's programs, fx_rs_kernel), the figures of
the hand-written and the generic kernels and of the opt-in call forms (lazy_lists,
padded_outputs); `c5_batch64`: four times c5's batch, more chunks than the device holds
workgroups; `c5_batch128`: eight times, more per-task buffers than the kernel arguments hold
(the pointer table is uploaded ahead of the kernel); `head_variants`: other spellings of the detection head, each on its
own generated kernel; `c5_nms_tail`: the compaction followed by the detection tail,
also through the TorchScript route.  `roofline` prices the dominant kernel against the 8 TB/s
HBM peak with the algorithmic bytes of the call; its duration is measured with
HIP events on the launch stream around ten back-to-back launches of the kernel
(mean per launch, `kernel_ms`; the reading of a pair around a single launch,
which carries about 2 us of the pair itself, is `kernel_ms_single_launch`).
`cpu_baseline` times the unfused TorchScript CPU path (the oracle) on a bounded
sample (`cpu_baseline_one_thread`: the same on one thread).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
KERNEL_BATCH = 10   # launches of a kernel inside one event pair (see measure)


def build_workload(name, dev, fused=True):
    """`fused`: c3 as ONE region (decode + softmax inside the class map, run by the library's SSD
    head kernel), as the TorchScript route builds it; otherwise as the two regions of the
    reference's pipeline (dense decode + softmax, then the class map) on the generic kernels."""
    import torch
    from functs_amd import configs
    from functs_amd.benchmark.inputs import INPUTS

    def G(*xs):
        return [x.to(dev) if isinstance(x, torch.Tensor) else x for x in xs]

    if name not in ("c1", "c2", "c3", "c5"):
        raise SystemExit("unknown workload %s" % name)
    cpu_args = INPUTS[name](0)
    if name == "c1":
        a, b, n = cpu_args
        calls = [(configs.build_c1(), G(b, n))]
        desc = "c1 get_started loop [1024,1024] n=1024"
    elif name == "c2":
        calls = [(configs.build_c2(), G(*cpu_args))]
        desc = "c2 YOLOv3-style post-proc [1,10647,85]"
    elif name == "c5":
        calls = [(configs.build_c5(16), G(*cpu_args))]
        desc = "c5 ParallelMap x16 YOLOv3-style post-proc [16,10647,85]"
    elif name == "c3":
        if fused:
            calls = [(configs.build_c3_fused(80), G(*cpu_args))]
        else:
            calls = [(configs.build_c3_decode(), G(*cpu_args)), (configs.build_c3_classes(80), None)]
        desc = "c3 SSD300-style post-proc [1,8732,4]+[1,8732,81]"
    return desc, calls, cpu_args


COLD_BYTES = 640 << 20   # the buffer sets of a workload together: well above the 256 MB last-level cache
MAX_SETS = 64


class Workload:
    """Binds the regions of one config to resident inputs: `sets` independent copies of the
    inputs, outputs and scratch (set 0 is the one the latency loops use; the others exist so
    that timed kernels can be rotated over more memory than the caches hold)."""

    def __init__(self, name, dev, sets=1, fused=True):
        import torch
        self.name = name
        self.desc, calls, self.cpu_args = build_workload(name, dev, fused)
        self.calls = calls
        self.dev = dev
        self.sets = []
        self._bind_set([args for _, args in calls])
        self.bound = self.sets[0]
        self.launches = sum(bc.plan.launches for bc in self.bound)
        for _ in range(sets - 1):
            self.add_set()

    def _bind_set(self, args_per_call):
        bound, prev_out = [], None
        for (region, _), args in zip(self.calls, args_per_call):
            if args is None:  # consumes the previous region's outputs
                args = prev_out
            bc = region.bind(*args)
            bound.append(bc)
            bc.launch()
            prev_out = bc.results()
        self.sets.append(bound)

    def add_set(self):
        import torch
        clone = lambda a: a.clone() if isinstance(a, torch.Tensor) else a
        self._bind_set([None if args is None else [clone(a) for a in args] for _, args in self.calls])

    def touched_bytes(self):
        """Device memory one call of one set reads or writes (inputs, outputs at their
        allocated size, scratch)."""
        import torch
        n = 0
        for bc in self.bound:
            for a in bc.args:
                for t in (a if isinstance(a, (list, tuple)) else [a]):
                    if isinstance(t, torch.Tensor):
                        n += t.numel() * t.element_size()
            for row in bc.outs:
                n += sum(t.numel() * t.element_size() for t in row)
            if bc.scratch is not None:
                n += bc.scratch.numel()
        return n

    def grow_cold(self):
        want = min(MAX_SETS, max(4, -(-COLD_BYTES // max(self.touched_bytes(), 1))))
        while len(self.sets) < want:
            self.add_set()
        return len(self.sets)

    def step(self):
        out = None
        for bc in self.bound:
            bc.launch()
            out = bc.results()
        return out

    def kernel_times_ms(self, repeat=1):
        t = []
        for bc in self.bound:
            t += bc.launch_timed(repeat=repeat)
        return t

    def cold_times_ms(self, rounds):
        """Per kernel of the call, and per region (all its kernels in order), the mean duration
        when consecutive launches rotate over the buffer sets."""
        from functs_amd.region import timed_sets
        flush(self.dev)
        per_kernel, per_region = [], []
        for i in range(len(self.bound)):
            col = [s[i] for s in self.sets]
            # one untimed pass first: the first burst of launches behind the allocation of the
            # sets reads up to 2 us longer per launch than any later one (clocks coming up)
            timed_sets(col, which=-1, rounds=1)
            flush(self.dev)
            for k in range(col[0].plan.launches):
                per_kernel.append(timed_sets(col, which=k, rounds=rounds))
                flush(self.dev)
            per_region.append(timed_sets(col, which=-1, rounds=rounds))
            flush(self.dev)
        return per_kernel, per_region

    def algorithmic_bytes(self):
        """Inputs read once + outputs written once for the fused call
        (intermediates between two regions of one config count zero)."""
        import torch
        total = self.bound[0].plan.alg_bytes
        if self.name == "c3":   # loc, conf and priors read once, whichever way the regions are cut
            total = sum(a.numel() * a.element_size() for a in self.cpu_args)
        last = self.bound[-1]
        last.launch()
        outs = last.results()
        if last.plan.compact:
            for o in outs:
                for t in (o if isinstance(o, list) else [o]):
                    total += t.numel() * t.element_size()
        elif len(self.bound) > 1:
            total += last.plan.alg_bytes
        return total


_FLUSH = {}


def flush(dev):
    """Streams 1 GiB through the library's copy kernel: what the caches held before is gone."""
    import torch
    from functs_amd import _lib
    if dev not in _FLUSH:
        _FLUSH[dev] = (torch.ones(512 << 18, dtype=torch.float32, device=dev), torch.empty(512 << 18, dtype=torch.float32, device=dev))
    _lib.copy_bytes(*_FLUSH[dev])
    # drained before anything is timed: launches queued right behind the flush read up to 1.5 us
    # longer each over the first tens of launches (seen on the 4 us kernels of c1)
    torch.cuda.synchronize()


def drain_floor_us(dev, n=200):
    """One small library kernel and a device synchronisation, per round: what draining the device
    after a call costs whatever the call does (the part of every drained latency that no kernel
    of this library can take away)."""
    import torch
    from functs_amd import _lib
    x, y = torch.zeros(64, device=dev), torch.zeros(64, device=dev)
    for _ in range(20):
        _lib.copy_bytes(x, y)
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n):
        _lib.copy_bytes(x, y)
        torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e6 / n


def recorded_traffic(kernel, workload):
    """HBM bytes per launch from the committed FETCH_SIZE / WRITE_SIZE counter
    summary of this kernel and workload (counter runs are separate rocprofv3 runs, so the
    figure is read from the summary, not measured in this run), or None when none is recorded."""
    path = os.path.join(ROOT, "profiles", "%s_%s_hbm_traffic.md" % (kernel, workload))
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch %s:" % kernel):
                return int(line.split(":")[1]), os.path.relpath(path, ROOT)
    except OSError:
        pass
    return None, None


def head_kernel_in_use(plan):
    """Does a call of this plan run as ONE launch of a compaction kernel built for its shape of
    work?  The kernel's name or None: fx_rs_kernel is the row-stream kernel GENERATED from the
    region's own programs; fx_head_stream (YOLO-style heads) and fx_classmap_head (SSD-style
    heads) are the hand-written ones."""
    import ctypes
    from functs_amd import _lib
    out = (ctypes.c_int64 * 8)()
    _lib.check(_lib.lib.fx_plan_rowstream_info(plan.handle, out, 8))
    if out[1]:
        return "fx_rs_kernel"
    _lib.check(_lib.lib.fx_plan_head_info(plan.handle, out, 8))
    if not out[1]:
        return None
    return {1: "fx_head_stream", 2: "fx_classmap_head"}[int(out[0])]


def copy_reference_ms(dev, nbytes, rounds=4):
    """The library's plain copy kernel moving the same number of bytes (half read, half written)
    on cold lines: pairs of buffers that together exceed the last-level cache, in rotation, the
    caches flushed first.  What the memory system gives a kernel that does nothing else."""
    import torch
    from functs_amd import _lib
    half = max(nbytes // 2 // 16 * 16, 16)
    n_pairs = max(4, -(-COLD_BYTES // (2 * half)))
    pairs = [(torch.empty(half, dtype=torch.uint8, device=dev), torch.empty(half, dtype=torch.uint8, device=dev))
             for _ in range(n_pairs)]
    for a, b in pairs:
        a.zero_()
        _lib.copy_bytes(a, b)
    flush(dev)
    torch.cuda.synchronize()
    # launched back to back by the library, the way the regions' kernels are timed (a Python loop
    # issues a launch every 5 to 6 us, longer than a small copy runs)
    return _lib.copy_bytes_timed_sets(pairs, rounds)


def measure(w, steps, warmup):
    import torch
    for _ in range(warmup):
        w.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        w.step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    # Per-kernel durations with HIP events on the launch stream.  An event pair around one
    # launch reads about 2 us more than the kernel runs (an empty kernel reads 6 us that way),
    # so every kernel is launched KERNEL_BATCH times back to back inside its pair and the mean
    # is taken: that is the duration a kernel trace reports.  The single-launch reading is kept
    # beside it.
    def mean_of(repeat, n):
        acc = None
        for _ in range(n):
            k = w.kernel_times_ms(repeat)
            acc = k if acc is None else [a + b for a, b in zip(acc, k)]
        return [a / n for a in acc]
    kern = mean_of(KERNEL_BATCH, max(steps // KERNEL_BATCH, 5))
    single = mean_of(1, steps)
    return ms, kern, single


def torchscript_route(name, cpu_args, dev, steps, warmup, cold_bytes=0, **build_options):
    """Per-call wall time of the same config through functs_amd.jit: the scripted
    program, functionalized, with its regions run by tssa::ParallelFunctor
    (output allocation, launches and the kept-row synchronisation included).
    With cold_bytes, consecutive calls rotate over copies of the inputs and the outputs of
    the last calls are kept alive, so that the allocator hands out other blocks: the calls
    then work on memory that the caches do not hold (returned beside the warm figures).
    Every figure is the median over regions_for(steps) timed regions of exactly `steps` calls."""
    import collections
    import torch
    import functs_amd.jit as fj
    from functs_amd.benchmark import PROGRAMS
    import functs_amd.aot as aot
    fn = fj.build(fj.script(PROGRAMS[name]), list(cpu_args), **build_options)
    args = [a.to(dev) if isinstance(a, torch.Tensor) else a for a in cpu_args]
    n_regions = regions_for(steps)

    def regions(call, k, drained=False):
        """Median time per call over n_regions timed regions of exactly k calls each, every region
        between two device synchronisations (drained: a synchronisation after every call)."""
        per_call = []
        for _ in range(n_regions):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(k):
                call(i)
                if drained:
                    torch.cuda.synchronize()
            torch.cuda.synchronize()
            per_call.append((time.perf_counter() - t0) * 1e6 / k)
        per_call.sort()
        return per_call[len(per_call) // 2]

    # the calls that settle the process (first launches load the kernels' code, the allocators
    # grow their pools) are not part of the warm-up the caller asks for
    for _ in range(max(warmup, SETTLE_CALLS)):
        fn(*args)
    torch.cuda.synchronize()
    l0, s0 = aot.launch_stats()
    us = regions(lambda i: fn(*args), steps)
    l1, s1 = aot.launch_stats()
    # the same call with the device drained after every call: issue to completion of one call
    n_sync = max(steps // 4, 5)
    sync_us = regions(lambda i: fn(*args), n_sync, drained=True)
    n_functors = str(fn.graph).count("= tssa::ParallelFunctor")
    cold_us = cold_sync_us = None
    if cold_bytes:
        in_bytes = sum(a.numel() * a.element_size() for a in args if isinstance(a, torch.Tensor))
        n_sets = min(MAX_SETS, max(4, -(-cold_bytes // max(2 * in_bytes, 1))))
        sets = [[a.clone() if isinstance(a, torch.Tensor) else a for a in args] for _ in range(n_sets)]
        ring = collections.deque(maxlen=n_sets)
        # (the ring of kept results has to fill and the allocator to hand out a block for the call
        # after it before the calls run as they do in the long run)
        for i in range(max(warmup, n_sets + 2, SETTLE_CALLS)):
            ring.append(fn(*sets[i % n_sets]))
        torch.cuda.synchronize()
        flush(dev)
        torch.cuda.synchronize()
        cold_us = regions(lambda i: ring.append(fn(*sets[i % n_sets])), steps)
        cold_sync_us = regions(lambda i: ring.append(fn(*sets[i % n_sets])), n_sync, drained=True)
    # host time of the operator by section (mean microseconds per operator call), warm calls
    from functs_amd import _C
    _C._functor_host_timing(True)
    for _ in range(steps):
        fn(*args)
    torch.cuda.synchronize()
    host = {k: round(v, 2) for k, v in _C._functor_host_times().items()}
    _C._functor_host_timing(False)
    return us, n_functors, (s1 - s0) / max(l1 - l0, 1), sync_us, cold_us, cold_sync_us, host


SETTLE_CALLS = 24      # untimed calls of a freshly built function before its first timed region
TIMED_CALLS = 200      # calls a figure rests on: a region of K calls is repeated until about this many have run


def regions_for(steps):
    """How many timed regions of `steps` calls a figure is the median of (an odd number)."""
    n = max(1, -(-TIMED_CALLS // max(steps, 1)))
    return min(n | 1, 15)


def set_kernels(rowstream, head):
    """Which kernels a compacting region may run: the generated row-stream kernels, the
    hand-written head kernels; with both off, the generic count + scatter pair."""
    from functs_amd import _lib
    _lib.lib.fx_set_rowstream(1 if rowstream else 0)
    _lib.lib.fx_set_head_kernel(1 if head else 0)


def cpu_baseline(name, budget_s, threads=None):
    import torch
    from oracle import configs as oc
    fn = oc.scripted(name)
    cpu_args = getattr(oc, name + "_inputs")(0)
    before = torch.get_num_threads()
    if threads:
        torch.set_num_threads(threads)
    try:
        return _cpu_loop(fn, cpu_args, budget_s)
    finally:
        torch.set_num_threads(before)


def _cpu_loop(fn, cpu_args, budget_s):
    import torch
    for _ in range(2):
        fn(*cpu_args)
    n, t0 = 0, time.perf_counter()
    while True:
        fn(*cpu_args)
        n += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s or n >= 2000:
            break
    return dt / n * 1e6, n, torch.get_num_threads()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c5")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--no-per-config", action="store_true")
    ap.add_argument("--interpreter", action="store_true",
                    help="run every region with the bytecode interpreter (no ahead-of-time compiled kernels)")
    ap.add_argument("--no-rowstream", action="store_true",
                    help="run compacting regions without the generated row-stream kernels (fx_rs_kernel): the detection heads "
                         "(c2, c5) then run the hand-written fx_head_stream")
    ap.add_argument("--no-head-kernel", action="store_true",
                    help="run compacting regions with the generic row-compaction kernels (count + scatter): neither the "
                         "generated row-stream kernels nor the hand-written head kernels")
    ap.add_argument("--cpu-seconds-per-config", type=float, default=2.0,
                    help="CPU time spent on the baseline of each configuration other than the headline one")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="BYTES",
                    help="also launch the library's plain copy kernel on BYTES (3 times): the known-size reference "
                         "dispatch that FETCH_SIZE / WRITE_SIZE counter runs are scaled by")
    ap.add_argument("--cold-profile", type=int, default=0, metavar="ROUNDS",
                    help="profiling aid: nothing but ROUNDS rounds of the workload's kernels, every call on the next of the "
                         "rotated buffer sets (cold lines), the caches flushed first; what a kernel trace or a counter run of "
                         "this command sees of the region's kernels is all cold")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this path runs on ONE GPU. Its map tasks and row ranges are independent and "
                         "would shard over GPUs without exchange, but that is not built. Run with --gpus 1.")
    import torch
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs an MI355X (no CPU fallback exists)")
    dev = torch.device("cuda:0")
    import functs_amd.aot as aot
    if args.interpreter:
        aot.enable(False)
    use_rs, use_head = not (args.no_rowstream or args.no_head_kernel), not args.no_head_kernel
    set_kernels(use_rs, use_head)

    if args.copy_calibration:
        from functs_amd import _lib
        n = args.copy_calibration // 4
        src = torch.ones(n, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            _lib.copy_bytes(src, dst)
        torch.cuda.synchronize()
        assert torch.equal(src, dst)

    if args.cold_profile:
        from functs_amd.region import timed_sets
        w = Workload(args.workload, dev, fused=use_head)
        n_sets = w.grow_cold()
        flush(dev)
        call_ms = [timed_sets([s[i] for s in w.sets], which=-1, rounds=args.cold_profile) for i in range(len(w.bound))]
        print(json.dumps({"mode": "cold-profile", "workload": w.desc, "cold_sets": n_sets,
                          "cold_bytes": n_sets * w.touched_bytes(), "rounds": args.cold_profile,
                          "launches_per_call": w.launches, "call_kernels_ms": [round(m, 5) for m in call_ms],
                          "calls_of_every_kernel": n_sets * (args.cold_profile + 2)}))
        return

    def run_one(name, with_cpu):
        w = Workload(name, dev, fused=use_head)
        ms, kern, single = measure(w, args.steps, args.warmup)
        alg = w.algorithmic_bytes()
        # the same kernels with consecutive launches rotated over buffer sets that together
        # exceed the last-level cache: every launch reads and writes cold lines
        n_sets = w.grow_cold()
        rounds = max(4, min(10, -(-40 // n_sets)))
        cold, cold_regions = w.cold_times_ms(rounds)
        dom_i = max(range(len(cold)), key=lambda i: cold[i])
        dom = cold[dom_i]
        frac = lambda ms_: round(alg / (ms_ * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)
        rec = {
            "workload": w.desc,
            "latency_us": round(ms * 1e3, 2),
            "kernel_us": [round(k * 1e3, 2) for k in cold],
            "kernel_us_warm": [round(k * 1e3, 2) for k in kern],
            "kernel_us_single_launch": [round(k * 1e3, 2) for k in single],
            "call_kernels_us": round(sum(cold_regions) * 1e3, 2),
            "cold_sets": n_sets,
            "cold_bytes": n_sets * w.touched_bytes(),
            "launches_per_call": w.launches,
            "row_compaction": any(bc.plan.compact for bc in w.bound),
            "head_kernel": next((k for k in (head_kernel_in_use(bc.plan) for bc in w.bound) if k), None),
            "algorithmic_bytes": alg,
            "dominant_kernel_index": dom_i,
            "gbps_dominant_kernel": round(alg / (dom * 1e-3) / 1e9, 1),
            "gbps_all_kernels": round(alg / (sum(cold_regions) * 1e-3) / 1e9, 1),
            "frac_hbm_peak": frac(dom),
            "frac_hbm_peak_warm": frac(kern[dom_i]),
            "frac_hbm_peak_call": frac(sum(cold_regions)),
            "frac_hbm_peak_call_warm": frac(sum(kern)),
        }
        if name == "c3" and rec["head_kernel"]:
            # the two regions of the reference's pipeline on the generic kernels, for comparison
            del w
            w = Workload(name, dev, fused=False)
            measure(w, 5, 3)
            w.grow_cold()
            split_cold, split_regions = w.cold_times_ms(rounds)
            rec["split_regions_kernel_us"] = [round(k * 1e3, 2) for k in split_cold]
            rec["split_regions_call_kernels_us"] = round(sum(split_regions) * 1e3, 2)
            rec["split_regions_launches_per_call"] = w.launches
        if rec["row_compaction"] and rec["head_kernel"]:
            # the same call on the library's other kernels for it: with the generated row-stream
            # kernels off (the hand-written head kernel where one matches the region) and on the
            # generic pair (count + scatter), every launch on cold lines as above
            def other(rowstream, head, fused):
                set_kernels(rowstream, head)
                try:
                    w2 = Workload(name, dev, fused=fused)
                    measure(w2, 5, 3)
                    w2.grow_cold()
                    k, regions = w2.cold_times_ms(rounds)
                    which = next((x for x in (head_kernel_in_use(bc.plan) for bc in w2.bound) if x), None)
                    return which, [round(x * 1e3, 2) for x in k], sum(regions)
                finally:
                    set_kernels(use_rs, use_head)
            if rec["head_kernel"] == "fx_rs_kernel":
                which, k, tot = other(False, True, True)
                if which:
                    rec["handwritten_kernel"] = which
                    rec["handwritten_kernel_us"] = k
                    rec["handwritten_frac_call"] = frac(tot)
            which, k, tot = other(False, False, name != "c3")
            rec["generic_kernel_us"] = k
            rec["generic_call_kernels_us"] = round(tot * 1e3, 2)
            rec["generic_frac_call"] = frac(tot)
        copy_ms = copy_reference_ms(dev, alg)
        rec["copy_same_bytes_us"] = round(copy_ms * 1e3, 2)
        rec["copy_same_bytes_frac"] = frac(copy_ms)
        rec["compiled_kernels"] = rec["head_kernel"] is not None or all(bc.region.specialized(*bc.args) for bc in w.bound)
        if all(bc.region.specialized(*bc.args) for bc in w.bound):
            # the same launches through the bytecode interpreter (c3: of the two regions)
            aot.enable(False)
            _, ikern, _ = measure(w, max(args.steps // 4, 5), 3)
            aot.enable(True)
            rec["interpreter_kernel_us"] = [round(k * 1e3, 2) for k in ikern]
        ts_us, n_functors, spec_share, sync_us, cold_us, cold_sync_us, host = torchscript_route(
            name, w.cpu_args, dev, args.steps, args.warmup, COLD_BYTES)
        rec["torchscript_route_host_us"] = host
        rec["torchscript_route_direct_call"] = n_functors == 1   # one functor: called without the TorchScript interpreter
        if rec["row_compaction"]:
            # opt-in forms of the same call (functs_amd.jit.build): results that stay the operator's
            # lists, and results at full size with their counts as a tensor, which wait for nothing
            options = {"padded_outputs": dict(padded_outputs=True)}
            if name in ("c3", "c5"):
                options["lazy_lists"] = dict(lazy_lists=True)
            for label, kw in options.items():
                o_us, _, _, o_sync, o_cold, o_cold_sync, _ = torchscript_route(name, w.cpu_args, dev, args.steps, args.warmup, COLD_BYTES, **kw)
                rec["torchscript_route_latency_us_" + label] = round(o_cold, 2)
                rec["torchscript_route_drained_latency_us_" + label] = round(o_cold_sync, 2)
                rec["torchscript_route_latency_us_warm_" + label] = round(o_us, 2)
        rec["torchscript_route_latency_us"] = round(cold_us, 2)
        rec["torchscript_route_drained_latency_us"] = round(cold_sync_us, 2)
        rec["torchscript_route_latency_us_warm"] = round(ts_us, 2)
        rec["torchscript_route_drained_latency_us_warm"] = round(sync_us, 2)
        rec["torchscript_route_functors"] = n_functors
        rec["torchscript_route_compiled_share"] = round(spec_share, 3)
        us, n, cores = cpu_baseline(name, args.cpu_seconds if with_cpu else args.cpu_seconds_per_config)
        rec["cpu_baseline"] = {"value": round(us, 1), "unit": "us", "cores": cores, "kind": "port",
                               "sample": "%d calls of torch.jit.script(%s) on the same seeded CPU tensors" % (n, name)}
        if with_cpu:
            us1, n1, _ = cpu_baseline(name, min(args.cpu_seconds / 3, 4.0), threads=1)
            rec["cpu_baseline_one_thread"] = {"value": round(us1, 1), "unit": "us", "cores": 1, "kind": "port",
                                              "sample": "%d calls, torch.set_num_threads(1)" % n1}
        return rec

    def run_c4():
        """The stacked LSTM: its (time, layer) loops carry state, the reference runs them on the
        host.  Here the loop nest is collapsed into one node whose functor runs one persistent
        kernel per call (weights read once, 65 dependent steps that hand the h vectors from all
        workgroups to all workgroups), so the figure of merit is the latency of the call; the HBM
        fraction is reported for completeness, the kernel is bound by the latency of its steps."""
        from functs_amd.benchmark.inputs import INPUTS
        import functs_amd.aot as aot
        import functs_amd.jit as fj
        from functs_amd.benchmark import PROGRAMS
        cpu_args = INPUTS["c4"](0)
        n_rep = max(args.steps // 10, 5)
        us, n_functors, spec_share, sync_us, cold_us, cold_sync_us, _ = torchscript_route("c4", cpu_args, dev, n_rep, 2, COLD_BYTES)
        fn = fj.build(fj.script(PROGRAMS["c4"]), list(cpu_args))
        gargs = [a.to(dev) for a in cpu_args]
        fn(*gargs)
        torch.cuda.synchronize()
        # device time of a call: the functor launches on torch's current stream
        l0, _ = aot.launch_stats()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n_rep):
            fn(*gargs)
        e1.record()
        torch.cuda.synchronize()
        l1, _ = aot.launch_stats()
        dev_us = e0.elapsed_time(e1) * 1e3 / n_rep
        collapsed = "fx::lstm_stack" in str(fn.graph)
        # the same call replayed as one HIP graph (functs_amd.jit.build(..., hip_graph=True))
        gfn = fj.build(fj.script(PROGRAMS["c4"]), list(cpu_args), hip_graph=True)
        for _ in range(3):
            gfn(*gargs)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n_rep):
            gfn(*gargs)
        torch.cuda.synchronize()
        graph_us = (time.perf_counter() - t0) * 1e6 / n_rep
        seq_len, layers = cpu_args[0].size(0), cpu_args[1].size(0)
        alg = 17072128  # weights + biases + x + out, each once
        c_us, c_n, c_cores = cpu_baseline("c4", args.cpu_seconds_per_config)
        copy_ms = copy_reference_ms(dev, alg)
        return {"workload": "c4 stacked LSTM 2x512, T=64, B=1",
                "cpu_baseline": {"value": round(c_us, 1), "unit": "us", "cores": c_cores, "kind": "port",
                                 "sample": "%d calls of torch.jit.script(c4) on the same seeded CPU tensors" % c_n},
                "copy_same_bytes_us": round(copy_ms * 1e3, 2), "torchscript_route_latency_us": round(us, 1),
                "torchscript_route_latency_us_synced": round(sync_us, 1),
                "torchscript_route_latency_us_cold": round(cold_us, 1),
                "torchscript_route_latency_us_cold_synced": round(cold_sync_us, 1),
                "device_us_per_call": round(dev_us, 1),
                "hip_graph_latency_us": round(graph_us, 1),
                "torchscript_route_functors": n_functors, "torchscript_route_compiled_share": round(spec_share, 3),
                "loops_collapsed": collapsed,
                "launches_per_call": (l1 - l0) / n_rep,
                "dependent_steps": seq_len + layers - 1,
                "us_per_dependent_step": round(dev_us / (seq_len + layers - 1), 2),
                "algorithmic_bytes": alg, "gbps_call": round(alg / (cold_us * 1e-6) / 1e9, 1),
                "frac_hbm_peak": round(alg / (cold_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 5),
                "bound": "latency of %d dependent steps (each one hand-over of the h vectors between all workgroups through the "
                         "memory side of the caches), not HBM" % (seq_len + layers - 1)}

    def run_tail():
        """The step behind the hot path: c5's compaction followed by the detection tail
        (score threshold, sort, class-aware NMS, top-100: yolov3_bbox.py:104-179) for the 16
        images in ONE more launch that reads the kept-row counts from memory.  The class logits
        are shifted by -6 so that about 1e-3 of the class scores pass 0.05, as behind a trained
        head (with N(0,1) logits nearly all 850k (row, class) pairs of an image would be
        candidates, the case the reference hands to a per-class loop)."""
        from functs_amd import configs, detection
        from functs_amd.benchmark.inputs import INPUTS
        preds, anchors, strides = INPUTS["c5"](0)
        preds = preds.clone()
        preds[..., 5:] -= 6.0
        bc = configs.build_c5(16).bind(preds.to(dev), anchors.to(dev), strides.to(dev))

        def call():
            bc.launch()
            return detection.multiclass_nms_batched(bc.batched(0), bc.batched(1), bc.batched(2), counts=bc.totals)

        for _ in range(max(args.warmup // 4, 3)):
            res = call()
        torch.cuda.synchronize()
        n = max(args.steps // 4, 5)
        t0 = time.perf_counter()
        for _ in range(n):
            res = call()
        torch.cuda.synchronize()
        us = (time.perf_counter() - t0) * 1e6 / n
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        bc.launch()
        e0.record()
        for _ in range(n):
            res = detection.multiclass_nms_batched(bc.batched(0), bc.batched(1), bc.batched(2), counts=bc.totals)
        e1.record()
        torch.cuda.synchronize()
        # the same through the TorchScript route: the scripted loop with functs::multiclass_nms in it
        # (functs_amd/benchmark/programs.py yolov3_batched_nms), which the pipeline turns into the
        # functor with padded outputs, ONE batched tail launch and one wait at the end
        ts_args = INPUTS["c5_nms"](0)
        ts_us, ts_functors, _, ts_sync_us, ts_cold_us, ts_cold_sync_us, ts_host = torchscript_route(
            "c5_nms", ts_args, dev, n, max(args.warmup // 4, 3), COLD_BYTES)
        kept = [int(k) for k in res.n.cpu()]
        rows = bc.totals.tolist()
        cand = [int((bc.batched(1)[t, :rows[t]] > 0.05).sum()) for t in range(16)]
        read = sum(r * (80 + 4 + 1) * 4 for r in rows)
        return {"workload": "c5 compaction + multiclass NMS tail, 16 images (class logits shifted by -6)",
                "latency_us": round(us, 1), "launches_per_call": bc.plan.launches + 1,
                "torchscript_route_latency_us": round(ts_cold_us, 1), "torchscript_route_drained_latency_us": round(ts_cold_sync_us, 1),
                "torchscript_route_latency_us_warm": round(ts_us, 1), "torchscript_route_drained_latency_us_warm": round(ts_sync_us, 1),
                "torchscript_route_functors": ts_functors, "torchscript_route_host_us": ts_host,
                "nms_kernel_us": round(e0.elapsed_time(e1) * 1e3 / n, 1),
                "kept_rows_per_image": [min(rows), max(rows)], "candidates_per_image": [min(cand), max(cand)],
                "detections_per_image": [min(kept), max(kept)],
                "nms_bytes_read": read, "nms_gbps": round(read / (e0.elapsed_time(e1) * 1e-3 / n) / 1e9, 1),
                "bound": "the candidate scan reads the image's class scores once (a workgroup per CU, shared out over the images); "
                         "sort and the greedy walk are done by the last workgroup of an image (registers and LDS)"}

    def run_rows():
        """The stand-alone row compaction of the C ABI (fx_compact_rows: count and scatter; a scan
        launch between them above 2 097 152 rows) on 700 000 rows of 16 float32 with half of them
        kept, next to the library's plain copy kernel on the same number of bytes."""
        import ctypes
        from functs_amd import _lib
        n, w = 700000, 16
        g = torch.Generator().manual_seed(0)
        mask = (torch.rand(n, generator=g) < 0.5).to(dev)
        col = torch.rand(n, w, generator=g).to(dev)
        out = torch.empty_like(col)
        m8 = mask.view(torch.uint8)
        src, dst = (ctypes.c_void_p * 1)(col.data_ptr()), (ctypes.c_void_p * 1)(out.data_ptr())
        rowlen, elsize = (ctypes.c_int32 * 1)(w), (ctypes.c_int32 * 1)(4)
        sb = _lib.lib.fx_compact_rows_scratch_bytes(n)
        scratch = torch.empty(sb, dtype=torch.uint8, device=dev)
        total = torch.zeros(1, dtype=torch.int32).pin_memory()
        stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)

        def call():
            _lib.check(_lib.lib.fx_compact_rows(m8.data_ptr(), n, src, dst, rowlen, elsize, 1, scratch.data_ptr(), sb,
                                                total.data_ptr(), stream))

        for _ in range(3):
            call()
        torch.cuda.synchronize()
        kept = int(total[0])
        reps = max(args.steps // 5, 5)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            call()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / reps
        moved = 2 * n + n * w * 4 + kept * w * 4    # mask twice (count, scatter), rows in, kept rows out
        a, b = torch.empty(moved // 2 // 16 * 16, dtype=torch.uint8, device=dev), torch.empty(moved // 2 // 16 * 16, dtype=torch.uint8, device=dev)
        _lib.copy_bytes(a, b)
        e0.record()
        for _ in range(reps):
            _lib.copy_bytes(a, b)
        e1.record()
        torch.cuda.synchronize()
        copy_us = e0.elapsed_time(e1) * 1e3 / reps
        return {"workload": "fx_compact_rows, 700000 rows x 16 float32, half kept (warm)", "launches_per_call": 2,
                "call_us": round(us, 1), "bytes_moved": moved, "gbps": round(moved / (us * 1e-6) / 1e9, 1),
                "copy_kernel_same_bytes_us": round(copy_us, 1), "copy_kernel_gbps": round(2 * a.numel() / (copy_us * 1e-6) / 1e9, 1)}

    def run_variants():
        """Detection heads that are NOT the text of the benchmark's region (corners joined by stack
        or cat, a padded class matrix, objectness in another column, another size constant, rows
        kept on a class score, one joined output matrix) on c5's inputs: each runs as one launch of
        the row-stream kernel generated from its own programs; cold lines, as for the configs."""
        from functs_amd import configs
        from functs_amd.benchmark.inputs import INPUTS
        from functs_amd.region import timed_sets
        cpu_args = INPUTS["c5"](0)
        out = {}
        for vname, kw in configs.HEAD_VARIANTS.items():
            region = configs.build_head_variant(batch=16, **kw)
            bound = [region.bind(*[a.clone().to(dev) for a in cpu_args]) for _ in range(6)]
            for bc in bound:
                bc.launch()
            res = bound[0].results()
            torch.cuda.synchronize()
            alg = bound[0].plan.alg_bytes + sum(t.numel() * t.element_size() for o in res for t in (o if isinstance(o, list) else [o]))
            flush(dev)
            ms = timed_sets(bound, which=-1, rounds=8)
            out[vname] = {"kernel": head_kernel_in_use(bound[0].plan), "launches_per_call": bound[0].plan.launches,
                          "call_kernels_us": round(ms * 1e3, 2), "algorithmic_bytes": alg,
                          "frac_hbm_peak_call": round(alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
            del bound
        return out

    def run_big_batch(batch=64):
        """The benchmark's region and one of the variants on four times c5's batch: more chunks of
        256 rows than the device holds workgroups (2 688 against 1 536), so every workgroup of the
        row-stream kernel takes chunks in turn; the variant also on the generic two passes."""
        from functs_amd import configs, _lib
        from functs_amd.benchmark.inputs import INPUTS
        from functs_amd.region import timed_sets
        preds, anchors, strides = INPUTS["c5"](0)
        torch.manual_seed(1)
        preds = preds.repeat(batch // preds.size(0), 1, 1)
        preds = preds + 0.01 * torch.randn(preds.shape)
        out = {"batch": batch}
        for vname, region_of in (("benchmark", lambda: configs.build_c5(batch)),
                                 ("stack", lambda: configs.build_head_variant(batch=batch, **configs.HEAD_VARIANTS["stack"]))):
            for rowstream in ((True, False) if vname == "stack" else (True,)):
                _lib.lib.fx_set_rowstream(1 if rowstream else 0)
                _lib.lib.fx_set_head_kernel(1 if rowstream else 0)
                try:
                    region = region_of()
                    bound = [region.bind(preds.clone().to(dev), anchors.to(dev), strides.to(dev)) for _ in range(2)]
                    for bc in bound:
                        bc.launch()
                    res = bound[0].results()
                    torch.cuda.synchronize()
                    alg = bound[0].plan.alg_bytes + sum(t.numel() * t.element_size() for o in res for t in (o if isinstance(o, list) else [o]))
                    flush(dev)
                    ms = timed_sets(bound, which=-1, rounds=6 if batch <= 64 else 3)
                    out[vname if rowstream else vname + "_generic"] = {
                        "kernel": head_kernel_in_use(bound[0].plan), "launches_per_call": bound[0].plan.launches,
                        "call_kernels_us": round(ms * 1e3, 2), "algorithmic_bytes": alg,
                        "frac_hbm_peak_call": round(alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}
                    del bound
                finally:
                    _lib.lib.fx_set_rowstream(1)
                    _lib.lib.fx_set_head_kernel(1)
        return out

    def run_stream():
        """Not one of the five configurations: one big fused elementwise region (sigmoid(2x + 1) on
        [8192, 4096] fp32), the shape on which the dense kernel itself meets the HBM roofline."""
        from functs_amd import Region
        x = torch.rand(8192, 4096, device=dev)
        r = Region()
        xi = r.tensor_input(torch.float32, 2)
        r.output((xi * 2.0 + 1.0).sigmoid())
        bc = r.finalize().bind(x)
        compiled = bc.region.specialized(x)
        for _ in range(args.warmup):
            bc.launch()
        torch.cuda.synchronize()
        acc = 0.0
        n = max(args.steps // KERNEL_BATCH, 5)
        for _ in range(n):
            acc += sum(bc.launch_timed(repeat=KERNEL_BATCH))
        ms = acc / n
        alg = 2 * x.numel() * 4
        return {"workload": "fused elementwise region sigmoid(2x+1), [8192,4096] fp32", "kernel_us": [round(ms * 1e3, 2)],
                "compiled_kernels": compiled,
                "launches_per_call": 1, "algorithmic_bytes": alg,
                "gbps_dominant_kernel": round(alg / (ms * 1e-3) / 1e9, 1),
                "frac_hbm_peak": round(alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)}

    head = run_one(args.workload, True)
    per = {}
    if not args.no_per_config:
        for name in ("c1", "c2", "c3", "c5"):
            if name == args.workload:
                per[name] = dict(head)
                continue
            try:
                r = run_one(name, False)
                per[name] = r
            except Exception as e:  # a config that cannot run is reported, never faked
                per[name] = {"error": str(e)[:200]}
        try:
            per["elementwise_stream"] = run_stream()
        except Exception as e:
            per["elementwise_stream"] = {"error": str(e)[:200]}
        try:
            per["head_variants"] = run_variants()
        except Exception as e:
            per["head_variants"] = {"error": str(e)[:200]}
        for batch in (64, 128):
            try:
                per["c5_batch%d" % batch] = run_big_batch(batch)
            except Exception as e:
                per["c5_batch%d" % batch] = {"error": str(e)[:200]}
        try:
            per["c4"] = run_c4()
        except Exception as e:
            per["c4"] = {"error": str(e)[:200]}
        try:
            per["standalone_compact_rows"] = run_rows()
        except Exception as e:
            per["standalone_compact_rows"] = {"error": str(e)[:200]}
        try:
            per["c5_nms_tail"] = run_tail()
        except Exception as e:
            per["c5_nms_tail"] = {"error": str(e)[:200]}
    dom_ms = head["kernel_us"][head["dominant_kernel_index"]] / 1e3
    dom_kernel = head.get("head_kernel") or ("fx_compact_scatter" if head["row_compaction"] else "fx_region_dense")
    copy_ms = head["copy_same_bytes_us"] / 1e3
    traffic, traffic_src = recorded_traffic(dom_kernel, args.workload)
    out = {
        "metric": "per-call latency",
        "value": head["torchscript_route_latency_us"],
        "value_kind": "back-to-back: K calls between two device synchronisations, consecutive calls on rotated copies of the inputs and on fresh output blocks (cold caches); the median of timed_regions such regions of exactly K calls each (about 200 calls in all), after the W warm-up calls and the calls that settle a freshly built function (kernel code loaded, allocator pools grown); drained_latency_us: the device drained after every call; *_warm: every call on the same buffers",
        "unit": "us",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "timed_regions": regions_for(args.steps),
        "ms_per_step": round(head["torchscript_route_latency_us"] / 1e3, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic (torch.manual_seed(0), CPU generator, copied to HBM)",
        "config": {"workload": head["workload"],
                   "route": "functs_amd.jit.script -> build -> tssa::ParallelFunctor (C++ operator over the C ABI)",
                   "compiled_kernels": head["compiled_kernels"] and not args.interpreter,
                   "drained_latency_us": head["torchscript_route_drained_latency_us"],
                   "drain_floor_us": round(drain_floor_us(dev), 2),
                   "latency_us_warm": head["torchscript_route_latency_us_warm"],
                   "drained_latency_us_warm": head["torchscript_route_drained_latency_us_warm"],
                   "region_api_latency_us": head["latency_us"], "launches_per_call": head["launches_per_call"],
                   "kernel_us": head["kernel_us"], "kernel_us_warm": head["kernel_us_warm"],
                   "gbps_all_kernels": head["gbps_all_kernels"]},
        "roofline": {"bound": "hbm", "achieved": head["gbps_dominant_kernel"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": head["frac_hbm_peak"], "frac_warm": head["frac_hbm_peak_warm"],
                     "frac_call": head["frac_hbm_peak_call"], "frac_call_warm": head["frac_hbm_peak_call_warm"],
                     "traffic": traffic,
                     "traffic_source": ("%s (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, separate runs; not measured in this run)" % traffic_src)
                     if traffic_src else None,
                     "kernel": dom_kernel,
                     "algorithmic_bytes": head["algorithmic_bytes"], "kernel_ms": round(dom_ms, 5),
                     "kernel_ms_warm": round(head["kernel_us_warm"][head["dominant_kernel_index"]] / 1e3, 5),
                     "call_kernels_ms": round(head["call_kernels_us"] / 1e3, 5),
                     "kernel_ms_single_launch": round(head["kernel_us_single_launch"][head["dominant_kernel_index"]] / 1e3, 5),
                     "cold_sets": head["cold_sets"], "cold_bytes": head["cold_bytes"],
                     "copy_same_bytes_ms": round(copy_ms, 5),
                     "copy_same_bytes_frac": round(head["algorithmic_bytes"] / (copy_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                     "timing": "HIP events on the launch stream around back-to-back launches, mean per launch. frac / kernel_ms: "
                               "the dominant kernel rotated over cold_sets independent sets of inputs, outputs and scratch "
                               "(cold_bytes in total, above the 256 MB last-level cache), the caches flushed before; "
                               "frac_warm / kernel_ms_warm: %d launches on one set; frac_call / call_kernels_ms: every kernel of "
                               "the call in order, rotated the same way; frac_call_warm: sum of the warm kernels; "
                               "copy_same_bytes_ms / _frac: the library's plain copy kernel moving algorithmic_bytes (half read, "
                               "half written) on cold lines, the same way" % KERNEL_BATCH},
        "cpu_baseline": head["cpu_baseline"],
        "cpu_baseline_one_thread": head["cpu_baseline_one_thread"],
        "per_config": per,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Benchmark of the fused NHWC GroupNorm + activation forward / backward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload sd_unet|all|<config name>] [--all]

A "step" is one forward + backward call of the op, through the C ABI of libgnnhwc_hip.so, on each shape
of the workload (default: the latent-diffusion UNet sweep c3a, c3b, c3c in bf16 with fused SiLU), with
inputs, outputs and workspaces already resident in HBM.  The timed region is K steps between two
torch.cuda.synchronize() calls.  Prints ONE JSON line:

  value        algorithmic GB/s of the timed region: (2 S fwd + 3 S bwd per shape) / time
  roofline     the dominant kernel (the kernel kind and shape the step spends the largest share of its kernel time
               in: mean launch duration x launches per step): its algorithmic bytes / its mean duration, measured
               here with HIP events bound to every launch on the launch stream, against 8 TB/s; every kernel's share
               and fraction is listed under `kernels`; `traffic` is read from profiles/results_all_configs.txt
               (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of `bench.py --counter-workload`), null when absent
  copy_ceiling the library's plain copy kernel on tensors of each shape's size: what a kernel with no
               arithmetic and no cross-workgroup dependency reaches at that size on this GPU
  cpu_baseline torch.nn.functional.group_norm + SiLU + autograd on the host cores, same tensors (bounded sample)
  torch_gpu    the same torch expression on the same GPU and the same channels-last tensors, us per call (context only)
  shapes       per-shape us/call and GB/s, with warm (same buffers every call) and cold (rotating through
               > 512 MB of distinct buffers) figures
"""
import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "channels-last-groupnorm_amd"))

HBM_PEAK_GBPS = 8000.0
# algorithmic bytes of each kernel kind, in units of S = bytes of one activation-sized tensor
KERNEL_STREAMS = {"fwd_stats": 1, "fwd_stats_compact": 0, "fwd_apply": 2, "bwd_reduce": 2, "bwd_compact": 0, "bwd_dx": 3,
                  "fused_fwd": 2, "fused_bwd": 3}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="sd_unet")
    ap.add_argument("--all", action="store_true", help="also time every other configuration (reported under 'shapes')")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-torch-gpu", action="store_true", help="skip the torch-on-the-same-GPU context leg")
    ap.add_argument("--no-shapes", action="store_true", help="skip the per-shape warm / cold / copy-ceiling table")
    ap.add_argument("--graph", action="store_true", help="time the replay of a HIP graph of the K steps instead of eager launches")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline sample")
    ap.add_argument("--fused-add", action="store_true",
                    help="also time gnnhwc_fwd_add (residual + sum output fused into the forward) against an elementwise "
                         "addition followed by gnnhwc_fwd, per shape (reported under 'fused_add')")
    ap.add_argument("--cast", action="store_true",
                    help="also time gnnhwc_fwd_cast (float32 x, y written as bfloat16 by the kernel) against gnnhwc_fwd followed "
                         "by a cast kernel, on the float32 versions of the workload's shapes (reported under 'cast')")
    ap.add_argument("--nchw", action="store_true",
                    help="also time the channels-first entry points on the same shapes against torch's GroupNorm + activation "
                         "on channels-first tensors (reported under 'channels_first')")
    ap.add_argument("--timeline", action="store_true",
                    help="no headline: print the in-kernel timeline of the single-launch kernels (wall-clock stamps every workgroup "
                         "takes at its phase boundaries; min / median / max over the workgroups of one launch) for each shape of "
                         "the workload (default here: c3a c3b c3c c4a), forward and backward, in a loop over that shape alone; "
                         "for the default workload first the same inside the sweep itself")
    ap.add_argument("--switch-cost", action="store_true",
                    help="no headline: event-timed duration of each kernel of the workload when it follows itself and when it "
                         "follows a different kernel whose data is tiny (a 1 MB plain copy; a small GroupNorm forward)")
    ap.add_argument("--recovery-cost", action="store_true",
                    help="no headline: event-timed duration of each kernel of the workload on the fast path and with every wait "
                         "forced to expire (every workgroup recomputes the records it needs): the worst case of the recovery path")
    ap.add_argument("--load-ceiling", action="store_true",
                    help="no headline: the load phase of each single-launch kernel of the workload on its own (a kernel that only "
                         "requests the rows), beside the kernel itself, on cold tensors")
    ap.add_argument("--code-placement", action="store_true",
                    help="no headline: per-kernel times of the workload (event-timed inside the sweep) in four child processes that "
                         "first load 0, 1, 2, 3 copies of the library under other names, which moves the code of the library proper "
                         "by one 2 MB slot each: how much of a kernel's time depends on where the loader put its code")
    ap.add_argument("--code-placement-child", type=int, default=-1, help=argparse.SUPPRESS)
    ap.add_argument("--results-table", action="store_true",
                    help="no headline: print the per-configuration result table (timings measured now; counter traffic and parity "
                         "errors read from the files named by --pmc-plan, --pmc-fetch, --pmc-write and --parity-log)")
    ap.add_argument("--pmc-plan", help="stdout of a `--counter-workload` run (its JSON line says which dispatches belong to which configuration)")
    ap.add_argument("--pmc-fetch", help="counter_collection CSV of the rocprofv3 --pmc FETCH_SIZE run")
    ap.add_argument("--pmc-write", help="counter_collection CSV of the rocprofv3 --pmc WRITE_SIZE run")
    ap.add_argument("--parity-log", help="JSON lines written by tests/test_gpu_parity.py with GNNHWC_PARITY_LOG set")
    ap.add_argument("--counter-workload", action="store_true",
                    help="no timing: one 256 MiB plain copy (calibration) and a few fwd+bwd calls per shape, for a rocprofv3 --pmc run")
    return ap.parse_args()


class Problem:
    """Device buffers for one configuration: `nsets` independent sets of x, dy, y, dx (+ shared parameters)."""

    def __init__(self, cfg, device, nsets=1):
        import torch
        import workloads as configs
        from workloads import nrc_view

        self.cfg = cfg
        self.S = configs.tensor_bytes(cfg)
        inp = configs.make_inputs(cfg, device)
        x, dy = nrc_view(inp["x"]), nrc_view(inp["dy"])
        self.N, self.R, self.C = x.shape
        self.G = cfg.G
        from gnnhwc.custom_gn import ACTIVATION_CODES

        self.act = ACTIVATION_CODES[cfg.act]
        self.w, self.b = inp["w"], inp["b"]
        self.sets = []
        for i in range(nsets):
            xs = x if i == 0 else x.clone()
            dys = dy if i == 0 else dy.clone()
            self.sets.append(dict(x=xs, dy=dys, y=torch.empty_like(xs), dx=torch.empty_like(xs)))
        sd = torch.float32 if x.dtype in (torch.float16, torch.bfloat16) else x.dtype
        self.mean = torch.empty((self.N, self.G), dtype=sd, device=device)
        self.rstd = torch.empty((self.N, self.G), dtype=sd, device=device)
        self.dw = torch.empty((self.C,), dtype=self.w.dtype, device=device)
        self.db = torch.empty((self.C,), dtype=self.w.dtype, device=device)
        from gnnhwc import _cabi
        from workloads import DT_CODE

        self.lib = _cabi.lib
        self.dt = DT_CODE[x.dtype]
        self.sdt = DT_CODE[sd]
        fb = self.lib.gnnhwc_fwd_workspace_bytes(self.N, self.R, self.C, self.G, self.dt)
        bb = self.lib.gnnhwc_bwd_workspace_bytes(self.N, self.R, self.C, self.G, self.dt)
        self.ws_f = torch.empty((fb,), dtype=torch.uint8, device=device)
        self.ws_b = torch.empty((bb,), dtype=torch.uint8, device=device)
        self.bwd = cfg.passes != "fwd"

    def alg_bytes(self):
        return (5 if self.bwd else 2) * self.S

    def fwd(self, s, stream):
        b = self.sets[s]
        rc = self.lib.gnnhwc_fwd(b["x"].data_ptr(), self.w.data_ptr(), self.b.data_ptr(), b["y"].data_ptr(),
                                 self.mean.data_ptr(), self.rstd.data_ptr(), self.N, self.R, self.C, self.G, 1e-5, self.act,
                                 self.dt, self.dt, self.sdt, self.ws_f.data_ptr(), self.ws_f.numel(), stream)
        if rc != 0:
            raise RuntimeError(self.lib.gnnhwc_last_error().decode())

    def bwd_(self, s, stream):
        b = self.sets[s]
        rc = self.lib.gnnhwc_bwd(b["dy"].data_ptr(), b["x"].data_ptr(), self.w.data_ptr(), self.b.data_ptr(),
                                 self.mean.data_ptr(), self.rstd.data_ptr(), b["dx"].data_ptr(), self.dw.data_ptr(),
                                 self.db.data_ptr(), self.N, self.R, self.C, self.G, self.act, self.dt, self.dt, self.sdt,
                                 self.ws_b.data_ptr(), self.ws_b.numel(), stream)
        if rc != 0:
            raise RuntimeError(self.lib.gnnhwc_last_error().decode())

    def instance(self, which):
        """Name of the kernel instance the library launches for this problem's forward / backward, from a call made now:
        e.g. fused_bwd,rows=22,window=0,two_level=0,launches=1 or multi-launch."""
        import torch
        from gnnhwc import _cabi

        stream = torch.cuda.current_stream().cuda_stream
        (self.fwd if which == "fwd" else self.bwd_)(0, stream)
        return _cabi.last_launch().replace(" ", ",")

    def step(self, s, stream, which="both"):
        if which in ("both", "fwd"):
            self.fwd(s, stream)
        if self.bwd and which in ("both", "bwd"):
            self.bwd_(s, stream)


def time_region(fn_step, steps, warmup, use_graph, reps=1):
    """Time `steps` calls of fn_step() between two device synchronisations; returns seconds (median of reps).
    With use_graph the K calls are captured once into a HIP graph and the graph is replayed."""
    import torch

    if use_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(max(3, min(warmup, 5))):
                fn_step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(steps):
                fn_step()
        run = g.replay
        nwarm = max(1, warmup // max(1, steps) + 1)
    else:
        def run():
            for _ in range(steps):
                fn_step()
        nwarm = 1
        for _ in range(warmup):
            fn_step()
    for _ in range(nwarm):
        run()
    times = []
    for _ in range(reps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    return statistics.median(times)


def measure_shape(prob_warm, prob_cold, steps, warmup, use_graph):
    """us/call and GB/s for one configuration: fwd, bwd and fwd+bwd; warm and cold."""
    import torch

    out = {}
    for label, prob in (("warm", prob_warm), ("cold", prob_cold)):
        if prob is None:
            continue
        nsets = len(prob.sets)
        for which in (("fwd", "bwd", "both") if prob.bwd else ("fwd",)):
            ctr = [0]

            def one():
                stream = torch.cuda.current_stream().cuda_stream
                prob.step(ctr[0] % nsets, stream, which)
                ctr[0] += 1

            k = steps if label == "warm" else max(nsets, (steps // nsets) * nsets)
            ctr[0] = 0
            t = time_region(one, k, warmup, use_graph, reps=5)
            us = t / k * 1e6
            nbytes = {"fwd": 2, "bwd": 3, "both": 5 if prob.bwd else 2}[which] * prob.S
            key = {"fwd": "fwd", "bwd": "bwd", "both": "fwd_bwd"}[which] if prob.bwd else "fwd"
            out["%s_%s_us" % (label, key)] = round(us, 3)
            out["%s_%s_gbps" % (label, key)] = round(nbytes / (t / k) / 1e9, 1)
    return out


def kernel_profile(probs, steps):
    """{shape: {kind: (mean us per launch, launches per call)}} with a HIP event pair bound to every launch of one
    shape at a time on the launch stream (begin-to-end time of each dispatch), while the whole workload runs in the
    order of the timed region: every kernel is measured in the cache state and queue position it has there."""
    import torch
    from gnnhwc import _cabi

    stream = torch.cuda.current_stream().cuda_stream
    out = {}
    torch.cuda.synchronize()

    def sweeps(target, count):
        for _ in range(count):
            for p in probs:
                if p is target:
                    _cabi.profile_enable(True)
                    p.step(0, stream)
                    _cabi.profile_enable(False)
                else:
                    p.step(0, stream)

    try:
        for target in probs:
            sweeps(target, steps)  # untimed pass: creates the event pool, so that the host keeps ahead of the GPU below
            _cabi.profile_collect()
            best = {}
            for _ in range(3):  # three passes, the fastest mean of each kind: robust against a transient slow start
                sweeps(target, steps)
                res = _cabi.profile_collect()
                for k, (n, ms) in res.items():
                    if n and (k not in best or ms / n < best[k][0] / best[k][1]):
                        best[k] = (ms, n)
            # mean per launch, and launches per call (a call may run one kernel kind several times, over groups of samples)
            out[target.cfg.name] = {k: (ms / n * 1e3, n / steps) for k, (ms, n) in best.items()}
    finally:
        _cabi.profile_enable(False)
    return out


def copy_ceiling(nbytes, device, steps):
    """GB/s (read + write) of the library's plain copy kernel on a tensor of nbytes, warm, eager launches."""
    import torch
    from gnnhwc import _cabi

    n = (nbytes + 15) // 16 * 16
    src = torch.empty((n,), dtype=torch.uint8, device=device).random_(0, 255)
    dst = torch.empty_like(src)
    stream = torch.cuda.current_stream().cuda_stream

    def one():
        _cabi.check(_cabi.lib.gnnhwc_debug_copy(dst.data_ptr(), src.data_ptr(), n, stream), "gnnhwc_debug_copy")

    t = time_region(one, steps, 10, False, reps=5)
    return 2 * n / (t / steps) / 1e9


TRAFFIC_FILE = os.path.join(ROOT, "profiles", "results_all_configs.txt")


def kernel_sources_sha16():
    """First 16 hex digits of the SHA-256 over the kernel sources (csrc/*.h, *.hip, Makefile, in name order): what the
    counter summary was taken on, to be compared with what is in the tree now."""
    import glob
    import hashlib

    h = hashlib.sha256()
    csrc = os.path.join(os.path.dirname(os.path.abspath(__file__)), "channels-last-groupnorm_amd", "csrc")
    for path in sorted(glob.glob(os.path.join(csrc, "*.h")) + glob.glob(os.path.join(csrc, "*.hip")) + [os.path.join(csrc, "Makefile")]):
        with open(path, "rb") as fh:
            h.update(os.path.basename(path).encode() + b"\0" + fh.read())
    return h.hexdigest()[:16]


def recorded_traffic():
    """{(shape, kind): (fetch_bytes, write_bytes, instance)} from the lines `TRAFFIC <shape> <kind> <fetch> <write>
    <instance>` of the committed counter summary, or {} when there is none.  `instance` names the kernel the counters
    were taken on (rows per lane, window, exchange form: Problem.instance()); a figure whose instance is not the one
    this build launches for the shape is stale and is not reported."""
    out = {}
    try:
        with open(TRAFFIC_FILE) as f:
            for ln in f:
                w = ln.split()
                if len(w) >= 5 and w[0] == "TRAFFIC":
                    out[(w[1], w[2])] = (float(w[3]), float(w[4]), w[5] if len(w) > 5 else "")
                elif len(w) == 2 and w[0] == "SOURCES":
                    out[("", "sources")] = w[1]  # kernel_sources_sha16() of the tree the counters were taken on
    except OSError:
        pass
    return out


def traffic_of(traffic, prob, kind):
    """Recorded traffic (bytes per launch) of `kind` on prob's shape if it was taken on the kernel instance this build
    launches, else None and why."""
    rec = traffic.get((prob.cfg.name, kind))
    if rec is None:
        return None, "not recorded"
    now = prob.instance("bwd" if "bwd" in kind else "fwd")
    if rec[2] != now:
        return None, "stale: recorded on %s, this build launches %s" % (rec[2] or "an unnamed instance", now)
    return rec[0] + rec[1], None


def counter_workload(probs, device):
    """What `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` observe: a plain copy of known size first (its
    counter reading calibrates the unit), then every shape's forward and backward a few times."""
    import torch
    from gnnhwc import _cabi

    stream = torch.cuda.current_stream().cuda_stream
    n = 256 << 20
    src = torch.empty((n,), dtype=torch.uint8, device=device).random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(3):
        _cabi.check(_cabi.lib.gnnhwc_debug_copy(dst.data_ptr(), src.data_ptr(), n, stream), "gnnhwc_debug_copy")
    torch.cuda.synchronize()
    plan = []
    mark_src = torch.zeros((16,), dtype=torch.uint8, device=device)
    mark_dst = torch.zeros_like(mark_src)
    for p in probs:
        # a 16-byte plain copy (one workgroup) in front of every configuration: the marker that cuts the dispatch sequence
        _cabi.check(_cabi.lib.gnnhwc_debug_copy(mark_dst.data_ptr(), mark_src.data_ptr(), 16, stream), "gnnhwc_debug_copy")
        # one call first, with the library's own launch count: how many dispatches a forward and a backward of this shape are
        _cabi.profile_collect()
        _cabi.profile_enable(True)
        p.step(0, stream, "fwd")
        _cabi.profile_enable(False)
        nf = sum(v[0] for v in _cabi.profile_collect().values())
        fi = _cabi.last_launch().replace(" ", ",")
        nb, bi = 0, None
        if p.bwd:
            _cabi.profile_enable(True)
            p.step(0, stream, "bwd")
            _cabi.profile_enable(False)
            nb = sum(v[0] for v in _cabi.profile_collect().values())
            bi = _cabi.last_launch().replace(" ", ",")
        for _ in range(5):
            p.step(0, stream)
        torch.cuda.synchronize()
        plan.append({"name": p.cfg.name, "S": p.S, "fwd_dispatches": nf, "bwd_dispatches": nb, "fwd_instance": fi, "bwd_instance": bi})
    # dispatch order: 3 plain copies of copy_bytes, then per configuration a one-workgroup marker copy and several calls, each
    # `fwd_dispatches` forward launches followed by `bwd_dispatches` backward launches
    print(json.dumps({"counter_workload": plan, "copy_bytes": n, "copies": 3}))


FWD_STAMPS = ((0, "workgroup starts"), (1, "tile moments in registers (all rows arrived)"), (2, "tile reduced, records published"),
              (3, "other tiles' records seen, statistics merged"), (4, "rows normalised and stored"))
BWD_STAMPS = ((0, "workgroup starts"), (1, "mean / rstd staged"), (6, "tile sums in registers (all rows arrived)"),
              (2, "tile reduced, records published"), (3, "other tiles' records seen, coefficients merged"), (4, "dx stored"),
              (5, "dgamma / dbeta written (workgroups of sample 0)"))


ARRIVAL_STAMP = {"fwd": 1, "bwd": 6}  # the stamp taken when all rows of the tile are in registers


def arrival_by_dispatch_order(t, which, cus=256):
    """Median 'rows arrived' time of the workgroups of one traced launch (stamps `t`, one row per workgroup in the
    order of their linear block index, which is the order they are dispatched in), grouped by cus: the first `cus`
    workgroups are the first on their CU, the next `cus` the second, and so on."""
    import numpy as np

    pt = ARRIVAL_STAMP[which]
    rel = (t[:, pt] - t[:, 0].min()) / 100.0
    return [float(np.median(rel[i:i + cus])) for i in range(0, t.shape[0], cus)]


def print_arrival_by_dispatch_order(rows_by_rep):
    if not rows_by_rep or len(rows_by_rep[0]) < 2:
        return
    n = min(len(r) for r in rows_by_rep)
    med = [statistics.median(r[i] for r in rows_by_rep) for i in range(n)]
    print("    %-58s %s" % ("  all rows arrived, workgroups 0-255 / 256-511 / ... (median)", " / ".join("%7.2f" % m for m in med)))


def timeline(names, device, reps=5):
    """In-kernel timeline of the single-launch kernels.  Thread 0 of every workgroup stamps a 100 MHz wall clock at its
    phase boundaries (GNNHWC_TRACE=2: the stamps do not wait for outstanding memory operations, so the kernel overlaps
    as it does untraced); the stamps of the most recent launch are read back and reported relative to the earliest
    workgroup start of that launch, in microseconds, as min / median / max over its workgroups.  The event-timed
    duration of the same launch (begin to end of the dispatch) is printed beside it."""
    import numpy as np
    import torch
    from gnnhwc import _cabi
    import workloads as configs

    stream = torch.cuda.current_stream().cuda_stream
    words = np.zeros((1024, 8), dtype=np.uint64)
    print("# in-kernel timeline, microseconds after the first workgroup of the launch started: min / median / max over workgroups")
    for name in names:
        p = Problem(configs.CONFIGS[name], device)
        for which, stamps in (("fwd", FWD_STAMPS), ("bwd", BWD_STAMPS)):
            if which == "bwd" and not p.bwd:
                continue
            for _ in range(3):
                p.step(0, stream)
            torch.cuda.synchronize()
            time.sleep(0.002)  # stamps of earlier launches end up far behind those of the launches below
            t0 = time.perf_counter()
            while time.perf_counter() - t0 < 0.02:  # launches right after the pause run at idle clocks: not timed
                p.step(0, stream, which)
            _cabi.profile_enable(True)
            for _ in range(20):
                p.step(0, stream, which)
            _cabi.profile_enable(False)
            res = {k: v for k, v in _cabi.profile_collect().items() if v[0]}
            kinds = ", ".join("%s %.2f us x %d per call" % (k, ms / n * 1e3, n // 20) for k, (n, ms) in res.items())
            if not any(k.startswith("fused") for k in res):
                print("%s %s: multi-launch kernels (no in-kernel timeline); event-timed: %s" % (name, which, kinds))
                continue
            torch.cuda.synchronize()
            time.sleep(0.002)
            rows = []
            waves = []
            for _ in range(reps):
                p.step(0, stream, "both")  # the traced launch runs behind other kernels, as in the sweep: a backward behind its
                if which == "fwd":         # own forward, a forward behind the backward of the call before
                    p.step(0, stream, "fwd")
                torch.cuda.synchronize()
                _cabi.check(_cabi.lib.gnnhwc_debug_read_trace(words.ctypes.data, words.size), "gnnhwc_debug_read_trace")
                t = words.astype(np.int64)
                live = t[:, 0] >= t[:, 0].max() - 300  # started within 3 us of the latest start: the workgroups of this launch
                t = t[live]
                waves.append(arrival_by_dispatch_order(t, which))
                rel = (t - t[:, 0].min()) / 100.0
                taken = {}
                for pt, _ in stamps:  # a stamp older than the launch was not taken by this launch (stamp 5: sample 0 only)
                    v = rel[:, pt][t[:, pt] >= t[:, 0].min()]
                    if v.size:
                        taken[pt] = (float(v.min()), float(np.median(v)), float(v.max()))
                rows.append((int(live.sum()), taken))
                time.sleep(0.002)
            nwg = rows[-1][0]
            print("%s %s: %d workgroups in the traced launch; event-timed: %s" % (name, which, nwg, kinds))
            for pt, label in stamps:
                vals = [r[1][pt] for r in rows if pt in r[1]]
                if not vals:
                    continue
                med = [statistics.median(v[i] for v in vals) for i in range(3)]
                print("    %-58s %7.2f / %7.2f / %7.2f" % (label, med[0], med[1], med[2]))
                if pt == ARRIVAL_STAMP[which]:
                    print_arrival_by_dispatch_order(waves)
        del p
        torch.cuda.empty_cache()


def timeline_in_sweep(names, device, reps=5):
    """The same stamps for every single-launch kernel of a workload taken INSIDE the workload: a few full steps run, then
    the launches of one more step up to and including the traced one, so that the traced launch finds the caches and
    the queue as it does in the timed region (its tensors evicted by the other shapes, another kernel ahead of it)."""
    import numpy as np
    import torch
    from gnnhwc import _cabi
    import workloads as configs

    stream = torch.cuda.current_stream().cuda_stream
    words = np.zeros((1024, 8), dtype=np.uint64)
    probs = [Problem(configs.CONFIGS[n], device) for n in names]
    launches = [(p, w) for p in probs for w in (("fwd", "bwd") if p.bwd else ("fwd",))]
    ev = {n: {k: us for k, (us, _) in kinds.items()} for n, kinds in kernel_profile(probs, 50).items()}
    print("# in-kernel timeline inside the workload %s, microseconds after the first workgroup of the launch started: "
          "min / median / max over workgroups" % "+".join(names))
    for ti, (p, which) in enumerate(launches):
        stamps = FWD_STAMPS if which == "fwd" else BWD_STAMPS
        kind = "fused_fwd" if which == "fwd" else "fused_bwd"
        evs = ev.get(p.cfg.name, {})
        if kind not in evs:
            print("%s %s: multi-launch kernels (no in-kernel timeline); event-timed in the workload: %s"
                  % (p.cfg.name, which, ", ".join("%s %.2f us" % kv for kv in evs.items() if not kv[0].startswith("fused"))))
            continue
        rows = []
        waves = []
        for _ in range(reps):
            torch.cuda.synchronize()
            time.sleep(0.002)
            for _ in range(6):
                for q, w in launches:
                    q.step(0, stream, w)
            for q, w in launches[:ti + 1]:
                q.step(0, stream, w)
            torch.cuda.synchronize()
            _cabi.check(_cabi.lib.gnnhwc_debug_read_trace(words.ctypes.data, words.size), "gnnhwc_debug_read_trace")
            t = words.astype(np.int64)
            live = t[:, 0] >= t[:, 0].max() - 300
            t = t[live]
            waves.append(arrival_by_dispatch_order(t, which))
            rel = (t - t[:, 0].min()) / 100.0
            taken = {}
            for pt, _ in stamps:
                v = rel[:, pt][t[:, pt] >= t[:, 0].min()]
                if v.size:
                    taken[pt] = (float(v.min()), float(np.median(v)), float(v.max()))
            rows.append((int(live.sum()), taken))
        print("%s %s: %d workgroups in the traced launch; event-timed in the workload: %s %.2f us"
              % (p.cfg.name, which, rows[-1][0], kind, evs[kind]))
        for pt, label in stamps:
            vals = [r[1][pt] for r in rows if pt in r[1]]
            if not vals:
                continue
            med = [statistics.median(v[i] for v in vals) for i in range(3)]
            print("    %-58s %7.2f / %7.2f / %7.2f" % (label, med[0], med[1], med[2]))
            if pt == ARRIVAL_STAMP[which]:
                print_arrival_by_dispatch_order(waves)


def switch_cost(names, device):
    """What following a DIFFERENT kernel costs a launch.  Each kernel of the workload is timed (event pair bound to the
    dispatch) in three loops: relaunched back to back; alternating with the library's plain copy kernel on 1 MB; and
    alternating with a GroupNorm forward on a 1 MB tensor.  The other kernels touch too little data to evict the timed
    kernel's tensors from the caches, so the difference is what the switch itself costs (a new program on every CU)."""
    import torch
    from gnnhwc import _cabi
    import workloads as configs

    stream = torch.cuda.current_stream().cuda_stream
    src = torch.empty((1 << 20,), dtype=torch.uint8, device=device)
    dst = torch.empty_like(src)
    small = Problem(configs.CONFIGS["c5a_bf16_gelu"], device)

    def copy():
        _cabi.check(_cabi.lib.gnnhwc_debug_copy(dst.data_ptr(), src.data_ptr(), src.numel(), stream), "gnnhwc_debug_copy")

    others = (("after itself", None), ("after a 1 MB plain copy", copy),
              ("after a 1 MB GroupNorm forward", lambda: small.step(0, stream, "fwd")))
    print("# event-timed microseconds per launch; same buffers every launch")
    print("%-6s %-4s %-12s %14s %26s %32s" % ("shape", "pass", "kernel", others[0][0], others[1][0], others[2][0]))
    # the plain copy kernel (a few hundred bytes of code) on 10 MB, as the kernel that is timed: what a switch costs a
    # kernel whose code is negligible (its "different kernel" is the small GroupNorm forward in both columns)
    big_src = torch.empty((10 << 20,), dtype=torch.uint8, device=device)
    big_dst = torch.empty_like(big_src)

    def big_copy():
        _cabi.check(_cabi.lib.gnnhwc_debug_copy(big_dst.data_ptr(), big_src.data_ptr(), big_src.numel(), stream), "gnnhwc_debug_copy")

    row = []
    for other in (None, lambda: small.step(0, stream, "fwd"), lambda: small.step(0, stream, "fwd")):
        def it(profile):
            if other is not None:
                other()
            _cabi.profile_enable(profile)
            big_copy()
            _cabi.profile_enable(False)
        for _ in range(50):
            it(False)
        torch.cuda.synchronize()
        _cabi.profile_collect()
        best = None
        for _ in range(3):
            for _ in range(100):
                it(True)
            torch.cuda.synchronize()
            res = {k: ms / n * 1e3 for k, (n, ms) in _cabi.profile_collect().items() if n}
            best = res["copy"] if best is None else min(best, res["copy"])
        row.append(best)
    print("%-6s %-4s %-12s %14.2f %26.2f %32.2f" % ("10MB", "-", "copy", row[0], row[1], row[2]))
    for name in names:
        p = Problem(configs.CONFIGS[name], device)
        for which in (("fwd", "bwd") if p.bwd else ("fwd",)):
            row, kind = [], None
            for _, other in others:
                def it(profile):
                    if other is not None:
                        other()
                    _cabi.profile_enable(profile)
                    p.step(0, stream, which)
                    _cabi.profile_enable(False)
                for _ in range(50):
                    it(False)
                torch.cuda.synchronize()
                for _ in range(20):
                    it(True)
                _cabi.profile_collect()
                best = None
                for _ in range(3):
                    for _ in range(100):
                        it(True)
                    torch.cuda.synchronize()
                    res = {k: ms / n * 1e3 for k, (n, ms) in _cabi.profile_collect().items() if n}
                    kind = "+".join(sorted(res))
                    v = sum(res.values())
                    best = v if best is None else min(best, v)
                row.append(best)
            print("%-6s %-4s %-12s %14.2f %26.2f %32.2f" % (name, which, kind, row[0], row[1], row[2]))
        del p
        torch.cuda.empty_cache()


def recovery_cost(names, device):
    """What the recovery path of the single-launch kernels costs in the worst case: every wait of every workgroup is made to
    expire at its first poll (poll limit -2), so every workgroup recomputes every record it needs from the inputs and reads
    its rows again.  Event-timed microseconds per launch, next to the same launch on the fast path."""
    import torch
    from gnnhwc import _cabi
    import workloads as configs

    stream = torch.cuda.current_stream().cuda_stream
    lib = _cabi.lib
    print("# event-timed microseconds per launch: fast path | every workgroup on the recovery path (poll limit -2)")
    print("%-6s %-4s %12s %14s %8s" % ("shape", "pass", "fast path", "all recover", "x"))
    for name in names:
        p = Problem(configs.CONFIGS[name], device)
        for which in (("fwd", "bwd") if p.bwd else ("fwd",)):
            row = []
            for limit in (-1, -2):
                prev = lib.gnnhwc_debug_set_spin_limit(limit)
                try:
                    for _ in range(5):
                        p.step(0, stream, which)
                    torch.cuda.synchronize()
                    _cabi.profile_collect()
                    _cabi.profile_enable(True)
                    for _ in range(20):
                        p.step(0, stream, which)
                    _cabi.profile_enable(False)
                    torch.cuda.synchronize()
                    res = {k: ms / n * 1e3 for k, (n, ms) in _cabi.profile_collect().items() if n}
                    row.append(sum(res.values()))
                finally:
                    lib.gnnhwc_debug_set_spin_limit(prev)
            lib.gnnhwc_resident_status()
            print("%-6s %-4s %12.2f %14.1f %8.0f" % (name, which, row[0], row[1], row[1] / row[0]))
        del p
        torch.cuda.empty_cache()


def load_ceiling(names, device):
    """The load phase of the single-launch kernels on its own: a kernel with their grid and tile geometry whose lanes request
    all their rows up front and do nothing else (gnnhwc_debug_load_tile), on cold tensors (eight sets in rotation).  No
    single-launch kernel can have its rows sooner; next to it the library's kernels on the same rotation of cold tensors."""
    import re
    import torch
    from gnnhwc import _cabi
    import workloads as configs

    stream = torch.cuda.current_stream().cuda_stream
    lib = _cabi.lib
    print("# event-timed microseconds per launch on cold tensors (8 sets of buffers in rotation)")
    print("%-6s %-4s %-44s %10s %10s %12s" % ("shape", "pass", "kernel", "kernel us", "loads us", "loads GB/s"))
    for name in names:
        cfg = configs.CONFIGS[name]
        p = Problem(cfg, device, 8)
        row_bytes = p.C * (p.S // (p.N * p.R * p.C))
        for which in (("fwd", "bwd") if p.bwd else ("fwd",)):
            p.step(0, stream, which)
            inst = _cabi.last_launch()
            m = re.search(r"rows=(\d+)", inst)
            ctr = [0]

            def kernel():
                p.step(ctr[0] % 8, stream, which)
                ctr[0] += 1

            def loads():
                b = p.sets[ctr[0] % 8]
                ctr[0] += 1
                _cabi.check(lib.gnnhwc_debug_load_tile(b["x"].data_ptr(), b["dy"].data_ptr() if which == "bwd" else None, None, p.N, p.R,
                                                       row_bytes, int(m.group(1)), stream), "gnnhwc_debug_load_tile")

            row = []
            for fn in (kernel, loads):
                if fn is loads and (m is None or row_bytes % 128 != 0):
                    row.append(float("nan"))
                    continue
                blocks = []
                for _ in range(2):  # the smaller of two blocks of 48 launches (the first block after a reallocation can run slow)
                    for _ in range(16):
                        fn()
                    torch.cuda.synchronize()
                    _cabi.profile_collect()
                    _cabi.profile_enable(True)
                    for _ in range(48):
                        fn()
                    _cabi.profile_enable(False)
                    torch.cuda.synchronize()
                    res = {k: ms / n * 1e3 for k, (n, ms) in _cabi.profile_collect().items() if n}
                    blocks.append(sum(res.values()))
                row.append(min(blocks))
                if max(blocks) > 2 * min(blocks):
                    print("# %s %s %s: blocks of %.1f and %.1f us per launch" % (name, which, fn.__name__, blocks[0], blocks[1]))
                if lib.gnnhwc_resident_status() != 0:
                    raise RuntimeError("a single-launch kernel recomputed records during the probe: its time is not a load ceiling comparison")
            nbytes = (2 if which == "bwd" else 1) * p.S
            print("%-6s %-4s %-44s %10.2f %10.2f %12.0f" % (name, which, inst.replace(" ", ","), row[0], row[1], nbytes / (row[1] * 1e-6) / 1e9))
        del p
        torch.cuda.empty_cache()


def code_placement_child(names, device, copies):
    """One process of --code-placement: load `copies` copies of the library first (each one's first kernel launch makes the
    runtime load a code object, which takes the next 2 MB-aligned slot), then time the workload's kernels inside the sweep."""
    import ctypes
    import shutil
    import tempfile
    import torch
    from gnnhwc import _cabi
    import workloads as configs

    keep = []
    tmp = tempfile.mkdtemp(prefix="gnnhwc_copies_")
    a = torch.empty((1 << 16,), dtype=torch.uint8, device=device)
    b = torch.empty_like(a)
    for i in range(copies):
        dst = os.path.join(tmp, "libcopy%d.so" % i)
        shutil.copy(_cabi.LIB_PATH, dst)
        lib = ctypes.CDLL(dst)
        lib.gnnhwc_debug_copy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        lib.gnnhwc_debug_copy(b.data_ptr(), a.data_ptr(), a.numel(), None)
        torch.cuda.synchronize()
        keep.append(lib)
    probs = [Problem(configs.CONFIGS[n], device) for n in names]
    r = kernel_profile(probs, 100)
    cells = []
    for n in names:
        for kind, (us, per_call) in sorted(r[n].items()):
            cells.append("%s %s %.2f" % (n, kind, us))
    print("copies loaded first: %d | %s | sum %.2f" % (copies, " | ".join(cells),
                                                        sum(us * pc for k in r.values() for us, pc in k.values())))
    shutil.rmtree(tmp, ignore_errors=True)


def code_placement(workload):
    import subprocess
    print("# event-timed microseconds per launch inside the sweep; one child process per line")
    for copies in (0, 1, 2, 3, 0, 1):
        out = subprocess.run([sys.executable, os.path.abspath(__file__), "--workload", workload, "--code-placement-child", str(copies)],
                             capture_output=True, text=True)
        lines = [ln for ln in out.stdout.splitlines() if ln.startswith("copies loaded first")]
        print(lines[-1] if lines else "child failed: " + out.stderr.strip().splitlines()[-1])
        sys.stdout.flush()


def cpu_baseline(cfg_names, seconds):
    """torch's CPU GroupNorm + activation + autograd on the host cores, same seeded tensors and dtype."""
    import torch
    from oracle import gn_oracle as orc  # the checker's torch_reference: the CPU baseline leg
    import workloads as configs

    per = {}
    total_bytes, total_time = 0.0, 0.0
    budget = seconds / len(cfg_names)
    for name in cfg_names:
        cfg = configs.CONFIGS[name]
        inp = configs.make_inputs(cfg, "cpu")
        dy = inp["dy"] if cfg.passes != "fwd" else None
        ts = []
        t_begin = time.perf_counter()
        n = 0
        while n < 3 or (n < 13 and time.perf_counter() - t_begin < budget):
            t0 = time.perf_counter()
            orc.torch_reference(inp["x"], inp["w"], inp["b"], cfg.G, 1e-5, cfg.act, dy)
            ts.append(time.perf_counter() - t0)
            n += 1
        ts = ts[1:] if len(ts) > 3 else ts  # first call pays one-off set-up
        med = statistics.median(ts)
        per[name] = round(med * 1e6, 1)
        total_bytes += configs.algorithmic_bytes(cfg)
        total_time += med
    # second leg: the C restatement of the reference algorithm (float accumulation, OpenMP over its (n, g) slabs),
    # on float32 copies of the same tensors; its bytes are counted at float32 width
    oc_bytes, oc_time, oc_per = 0.0, 0.0, {}
    for name in cfg_names:
        cfg = configs.CONFIGS[name]
        inp = configs.make_inputs(cfg, "cpu")
        x = orc.to_nrc(inp["x"]).astype("float32")
        dy = orc.to_nrc(inp["dy"]).astype("float32")
        w, b = inp["w"].float().numpy(), inp["b"].float().numpy()
        act = orc.ACT_CODES[cfg.act]
        ts = []
        for _ in range(3):
            t0 = time.perf_counter()
            if cfg.passes == "fwd":
                orc.fwd(x, w, b, cfg.G, 1e-5, act, dtype="float32")
            else:
                orc.fwd_bwd(x, w, b, dy, cfg.G, 1e-5, act, dtype="float32")
            ts.append(time.perf_counter() - t0)
        med = statistics.median(ts)
        oc_per[name] = round(med * 1e6, 1)
        oc_bytes += (2 if cfg.passes == "fwd" else 5) * x.nbytes
        oc_time += med
    return {
        "oracle_c_f32": {"value": round(oc_bytes / oc_time / 1e9, 3), "unit": "GB/s (float32 tensors)", "us_per_call": oc_per,
                         "sample": "oracle/gn_oracle.c float path, median of 3 calls per shape"},
        "value": round(total_bytes / total_time / 1e9, 3),
        "unit": "GB/s",
        "cores": torch.get_num_threads(),
        "host_cpus": os.cpu_count(),
        "kind": "port",
        "sample": "torch.nn.functional.group_norm + activation + autograd.grad on CPU (the results contract), same seeded "
                  "tensors and dtype, median of up to 12 calls per shape after 1 discarded; us/call per shape: %s" % json.dumps(per),
        "us_per_call": per,
    }


def fused_add_table(names, device, steps, warmup):
    """Forward with the skip-connection addition fused in (reads x and the residual, writes their sum and y:
    4 S algorithmic bytes) against the unfused sequence a caller of the plain forward runs (torch.add into a sum
    buffer, then gnnhwc_fwd on it: 3 S + 2 S), and the channel-bias-only form (2 S) against its unfused sequence."""
    import torch
    import workloads as configs

    out = {}
    for n in names:
        cfg = configs.CONFIGS[n]
        p = Problem(cfg, device)
        b = p.sets[0]
        x = b["x"]
        res = (0.5 * torch.randn(x.shape, device=device)).to(x.dtype)
        cb = torch.randn((p.N, p.C), device=device).to(x.dtype)
        total = torch.empty_like(x)
        stream_of = lambda: torch.cuda.current_stream().cuda_stream  # noqa: E731

        def call_add(residual, channel_bias, sum_out):
            rc = p.lib.gnnhwc_fwd_add(x.data_ptr(), residual.data_ptr() if residual is not None else None,
                                      channel_bias.data_ptr() if channel_bias is not None else None,
                                      sum_out.data_ptr() if sum_out is not None else None, p.w.data_ptr(), p.b.data_ptr(),
                                      b["y"].data_ptr(), p.mean.data_ptr(), p.rstd.data_ptr(), p.N, p.R, p.C, p.G, 1e-5,
                                      p.act, p.dt, p.dt, p.sdt, p.dt, p.ws_f.data_ptr(), p.ws_f.numel(), stream_of())
            if rc != 0:
                raise RuntimeError(p.lib.gnnhwc_last_error().decode())

        def plain_on(t):
            rc = p.lib.gnnhwc_fwd(t.data_ptr(), p.w.data_ptr(), p.b.data_ptr(), b["y"].data_ptr(), p.mean.data_ptr(),
                                  p.rstd.data_ptr(), p.N, p.R, p.C, p.G, 1e-5, p.act, p.dt, p.dt, p.sdt,
                                  p.ws_f.data_ptr(), p.ws_f.numel(), stream_of())
            if rc != 0:
                raise RuntimeError(p.lib.gnnhwc_last_error().decode())

        def unfused_residual():
            torch.add(x, res, out=total)
            plain_on(total)

        def unfused_bias():
            torch.add(x, cb[:, None, :], out=total)
            plain_on(total)

        cases = {
            "residual_sum_fused": (lambda: call_add(res, None, total), 4),
            "residual_sum_unfused": (unfused_residual, 4),
            "channel_bias_fused": (lambda: call_add(None, cb, None), 2),
            "channel_bias_unfused": (unfused_bias, 2),
        }
        r = {}
        for key, (fn, streams) in cases.items():
            t = min(time_region(fn, steps, warmup, False) for _ in range(3)) / steps
            r[key + "_us"] = round(t * 1e6, 3)
            r[key + "_gbps"] = round(streams * p.S / t / 1e9, 1)  # algorithmic bytes of the FUSED form / time
        r["residual_sum_speedup"] = round(r["residual_sum_unfused_us"] / r["residual_sum_fused_us"], 3)
        r["channel_bias_speedup"] = round(r["channel_bias_unfused_us"] / r["channel_bias_fused_us"], 3)
        out[n] = r
        del p
        torch.cuda.empty_cache()
    return out


def cast_table(names, device, steps, warmup):
    """Forward of float32 data with y leaving as bfloat16 (reads S, writes S / 2) against the sequence a caller of the
    plain forward runs for a half-precision consumer: gnnhwc_fwd (2 S) and a cast kernel (1.5 S more)."""
    import torch
    import workloads as configs

    out = {}
    for n in names:
        cfg = configs.CONFIGS[n]._replace(dtype="fp32")
        p = Problem(cfg, device)
        b = p.sets[0]
        x = b["x"]
        y16 = torch.empty(x.shape, dtype=torch.bfloat16, device=device)
        stream_of = lambda: torch.cuda.current_stream().cuda_stream  # noqa: E731

        def fused():
            rc = p.lib.gnnhwc_fwd_cast(x.data_ptr(), p.w.data_ptr(), p.b.data_ptr(), y16.data_ptr(), p.mean.data_ptr(),
                                       p.rstd.data_ptr(), p.N, p.R, p.C, p.G, 1e-5, p.act, p.dt, p.dt, p.sdt, 3,
                                       p.ws_f.data_ptr(), p.ws_f.numel(), stream_of())
            if rc != 0:
                raise RuntimeError(p.lib.gnnhwc_last_error().decode())

        def unfused():
            rc = p.lib.gnnhwc_fwd(x.data_ptr(), p.w.data_ptr(), p.b.data_ptr(), b["y"].data_ptr(), p.mean.data_ptr(),
                                  p.rstd.data_ptr(), p.N, p.R, p.C, p.G, 1e-5, p.act, p.dt, p.dt, p.sdt,
                                  p.ws_f.data_ptr(), p.ws_f.numel(), stream_of())
            if rc != 0:
                raise RuntimeError(p.lib.gnnhwc_last_error().decode())
            y16.copy_(b["y"])

        r = {}
        for key, fn in (("fused", fused), ("unfused", unfused)):
            t = min(time_region(fn, steps, warmup, False) for _ in range(3)) / steps
            r[key + "_us"] = round(t * 1e6, 3)
            r[key + "_gbps"] = round(1.5 * p.S / t / 1e9, 1)  # algorithmic bytes of the FUSED form / time
        r["speedup"] = round(r["unfused_us"] / r["fused_us"], 3)
        # the backward that follows: the gradient of y arrives as bfloat16; read as it is (gnnhwc_bwd_cast: x S, dy S / 2,
        # dx S) against a widening pass (1.5 S more) followed by gnnhwc_bwd
        if p.bwd:
            dy16 = torch.randn(x.shape, device=device).to(torch.bfloat16)
            dyf = torch.empty_like(x)

            def bwd_fused():
                rc = p.lib.gnnhwc_bwd_cast(dy16.data_ptr(), x.data_ptr(), p.w.data_ptr(), p.b.data_ptr(), p.mean.data_ptr(),
                                           p.rstd.data_ptr(), b["dx"].data_ptr(), p.dw.data_ptr(), p.db.data_ptr(), p.N, p.R, p.C,
                                           p.G, p.act, p.dt, p.dt, p.sdt, 3, p.ws_b.data_ptr(), p.ws_b.numel(), stream_of())
                if rc != 0:
                    raise RuntimeError(p.lib.gnnhwc_last_error().decode())

            def bwd_unfused():
                dyf.copy_(dy16)
                rc = p.lib.gnnhwc_bwd(dyf.data_ptr(), x.data_ptr(), p.w.data_ptr(), p.b.data_ptr(), p.mean.data_ptr(),
                                      p.rstd.data_ptr(), b["dx"].data_ptr(), p.dw.data_ptr(), p.db.data_ptr(), p.N, p.R, p.C, p.G,
                                      p.act, p.dt, p.dt, p.sdt, p.ws_b.data_ptr(), p.ws_b.numel(), stream_of())
                if rc != 0:
                    raise RuntimeError(p.lib.gnnhwc_last_error().decode())

            fused()  # (mean / rstd of this x)
            for key, fn in (("bwd_fused", bwd_fused), ("bwd_unfused", bwd_unfused)):
                t = min(time_region(fn, steps, warmup, False) for _ in range(3)) / steps
                r[key + "_us"] = round(t * 1e6, 3)
                r[key + "_gbps"] = round(2.5 * p.S / t / 1e9, 1)  # algorithmic bytes of the FUSED form / time
            r["bwd_speedup"] = round(r["bwd_unfused_us"] / r["bwd_fused_us"], 3)
        out[n + "_fp32"] = r
        del p
        torch.cuda.empty_cache()
    return out


def nchw_table(names, device, steps, warmup):
    """gnnhwc_fwd_nchw / gnnhwc_bwd_nchw (two launches forward, three backward; algorithmic bytes 2 S / 3 S as for the
    channels-last path) against what the reference does with channels-first input: torch's GroupNorm followed by the
    activation, and their autograd backward."""
    import torch
    import torch.nn.functional as F
    import workloads as configs
    from workloads import DT_CODE

    acts = {"identity": lambda t: t, "relu": F.relu, "silu": F.silu, "gelu": F.gelu,
            "gelu_tanh": lambda t: F.gelu(t, approximate="tanh")}
    out = {}
    for n in list(names) + ["one_group"]:
        cfg = configs.CONFIGS.get(n) or configs.EXTRA[n]
        p = Problem(cfg, device)
        b = p.sets[0]
        x = b["x"].permute(0, 2, 1).contiguous()   # (N, C, R)
        dy = b["dy"].permute(0, 2, 1).contiguous()
        y, dx = torch.empty_like(x), torch.empty_like(x)
        lib = p.lib
        nb = max(lib.gnnhwc_nchw_workspace_bytes(p.N, p.C, p.R, p.G, p.dt, 0), lib.gnnhwc_nchw_workspace_bytes(p.N, p.C, p.R, p.G, p.dt, 1))
        ws = torch.empty((nb,), dtype=torch.uint8, device=device)
        stream_of = lambda: torch.cuda.current_stream().cuda_stream  # noqa: E731

        def fwd():
            rc = lib.gnnhwc_fwd_nchw(x.data_ptr(), p.w.data_ptr(), p.b.data_ptr(), y.data_ptr(), p.mean.data_ptr(), p.rstd.data_ptr(),
                                     p.N, p.C, p.R, p.G, 1e-5, p.act, p.dt, p.dt, p.sdt, ws.data_ptr(), nb, stream_of())
            if rc != 0:
                raise RuntimeError(lib.gnnhwc_last_error().decode())

        def bwd():
            rc = lib.gnnhwc_bwd_nchw(dy.data_ptr(), x.data_ptr(), p.w.data_ptr(), p.b.data_ptr(), p.mean.data_ptr(), p.rstd.data_ptr(),
                                     dx.data_ptr(), p.dw.data_ptr(), p.db.data_ptr(), p.N, p.C, p.R, p.G, p.act, p.dt, p.dt, p.sdt,
                                     ws.data_ptr(), nb, stream_of())
            if rc != 0:
                raise RuntimeError(lib.gnnhwc_last_error().decode())

        xt = x.view(p.N, p.C, p.R, 1).clone().requires_grad_()
        wt, bt = p.w.clone().requires_grad_(), p.b.clone().requires_grad_()
        act = acts[cfg.act]
        dyt = dy.view(p.N, p.C, p.R, 1)

        def torch_fwd():
            with torch.no_grad():
                act(F.group_norm(xt, p.G, wt, bt, 1e-5))

        def torch_fwd_bwd():
            yt = act(F.group_norm(xt, p.G, wt, bt, 1e-5))
            torch.autograd.grad(yt, (xt, wt, bt), dyt)

        def ours_fwd_bwd():
            fwd()
            bwd()

        r = {}
        for key, fn, streams in (("fwd", fwd, 2), ("fwd_bwd", ours_fwd_bwd, 5), ("torch_fwd", torch_fwd, 2), ("torch_fwd_bwd", torch_fwd_bwd, 5)):
            if key.endswith("bwd") and not p.bwd:
                continue
            t = min(time_region(fn, steps, warmup, False) for _ in range(3)) / steps
            r[key + "_us"] = round(t * 1e6, 3)
            r[key + "_gbps"] = round(streams * p.S / t / 1e9, 1)
        r["fwd_speedup_over_torch"] = round(r["torch_fwd_us"] / r["fwd_us"], 3)
        if p.bwd:
            r["fwd_bwd_speedup_over_torch"] = round(r["torch_fwd_bwd_us"] / r["fwd_bwd_us"], 3)
        out[n] = r
        del p
        torch.cuda.empty_cache()
    return out


def torch_gpu_leg(names, device, steps, warmup):
    """Context only, never a target: torch's own GroupNorm followed by the activation (and their autograd backward) on
    the same GPU and the same channels-last tensors -- the comparison the reference's benchmark makes
    (benchmark.py:48-49, 86-96).  us per call, forward and forward + backward."""
    import torch
    import torch.nn.functional as F
    import workloads as configs

    acts = {"identity": lambda t: t, "relu": F.relu, "silu": F.silu, "gelu": F.gelu,
            "gelu_tanh": lambda t: F.gelu(t, approximate="tanh")}
    out = {}
    for n in names:
        cfg = configs.CONFIGS[n]
        inp = configs.make_inputs(cfg, device)
        xt = inp["x"].detach().clone(memory_format=torch.preserve_format).requires_grad_()  # (N, C, *spatial), channels fastest
        wt, bt = inp["w"].clone().requires_grad_(), inp["b"].clone().requires_grad_()
        dyt = inp["dy"]
        act = acts[cfg.act]

        def fwd():
            with torch.no_grad():
                act(F.group_norm(xt, cfg.G, wt, bt, 1e-5))

        def fwd_bwd():
            yt = act(F.group_norm(xt, cfg.G, wt, bt, 1e-5))
            torch.autograd.grad(yt, (xt, wt, bt), dyt)

        r = {"fwd_us": round(min(time_region(fwd, steps, warmup, False) for _ in range(3)) / steps * 1e6, 2)}
        if cfg.passes != "fwd":
            r["fwd_bwd_us"] = round(min(time_region(fwd_bwd, steps, warmup, False) for _ in range(3)) / steps * 1e6, 2)
        out[n] = r
        del xt, dyt
        torch.cuda.empty_cache()
    return {"what": "torch.nn.functional.group_norm + activation (+ autograd.grad) on the same GPU, same channels-last "
                    "tensors, eager; context only", "us_per_call": out}


def counter_bytes_per_config(csv_path, plan, counter):
    """{config: {"fwd": bytes, "bwd": bytes}} (medians over the calls) from the counter_collection CSV of a
    `rocprofv3 --pmc <counter>` run of `bench.py --counter-workload`, whose JSON line (`plan`) says how many dispatches
    each configuration's forward and backward are.  The unit is calibrated on the plain copies the workload starts with."""
    import collections
    import csv

    per_dispatch = collections.OrderedDict()
    with open(csv_path) as f:
        for r in csv.DictReader(f):
            # (kernels on _Float16 come out of the profiler with their names still mangled: _ZN2gn...)
            if ("gn::" not in r["Kernel_Name"] and not r["Kernel_Name"].startswith("_ZN2gn")) or r["Counter_Name"] != counter:
                continue
            key = int(r["Dispatch_Id"])
            name, val = per_dispatch.get(key, (r["Kernel_Name"], 0.0))
            per_dispatch[key] = (name, val + float(r["Counter_Value"]))
    seq = [per_dispatch[k] for k in sorted(per_dispatch)]
    copies = [v for n, v in seq[:plan["copies"]]]
    assert all("copy_kernel" in n for n, _ in seq[:plan["copies"]]), "the workload does not start with its plain copies"
    unit = plan["copy_bytes"] / statistics.median(copies)  # bytes per counter unit
    segments = []  # one per configuration: the dispatches between two marker copies
    for name, val in seq[plan["copies"]:]:
        if "copy_kernel" in name:
            segments.append([])
        else:
            segments[-1].append(val)
    assert len(segments) == len(plan["counter_workload"]), "markers in the counter file do not match the workload's configurations"
    out = {}
    for c, seg in zip(plan["counter_workload"], segments):
        per_call = c["fwd_dispatches"] + c["bwd_dispatches"]
        assert len(seg) % per_call == 0 and len(seg) >= 3 * per_call, (c["name"], len(seg), per_call)
        fwd, bwd = [], []
        for pos in range(0, len(seg), per_call):
            fwd.append(sum(seg[pos:pos + c["fwd_dispatches"]]))
            if c["bwd_dispatches"]:
                bwd.append(sum(seg[pos + c["fwd_dispatches"]:pos + per_call]))
        out[c["name"]] = {"fwd": statistics.median(fwd) * unit, "bwd": statistics.median(bwd) * unit if bwd else None}
    return out, unit


def results_table(args, device):
    """The per-configuration result table: us per call, algorithmic GB/s and fraction of the 8 TB/s peak, counter
    traffic against the algorithmic bytes, the plain copy of the same size, torch's CPU time, and the parity errors
    observed by tests/test_gpu_parity.py::test_config_parity next to their bars."""
    import torch
    import workloads as configs

    names = list(configs.ALL_NAMES)
    plan = json.loads([ln for ln in open(args.pmc_plan).read().splitlines() if ln.startswith('{"counter_workload"')][-1])
    fetch, fu = counter_bytes_per_config(args.pmc_fetch, plan, "FETCH_SIZE")
    write, wu = counter_bytes_per_config(args.pmc_write, plan, "WRITE_SIZE")
    inst = {c["name"]: c for c in plan["counter_workload"]}
    errs = {}
    if args.parity_log:
        for ln in open(args.parity_log):
            r = json.loads(ln)
            if r["family"] == "resident":
                errs[r["config"]] = r["observed"]
    cpu = cpu_baseline(names, args.cpu_seconds)
    steps = max(20, args.steps // 2)
    print("Per-configuration results on one MI355X: every named configuration, forward and backward through the C ABI, eager launches,")
    print("each configuration alone in a loop on the same buffers (warm); inputs resident in HBM.")
    print()
    print("commands (each rocprofv3 run from /tmp with TMPDIR=/tmp; one counter per run):")
    print("  GNNHWC_PARITY_LOG=<errors.jsonl> python -m pytest tests/test_gpu_parity.py -m gpu -k test_config_parity")
    print("  rocprofv3 --pmc FETCH_SIZE --output-format csv -d <fetch> -o p -- python3 bench.py --counter-workload --workload all > <plan.log>")
    print("  rocprofv3 --pmc WRITE_SIZE --output-format csv -d <write> -o p -- python3 bench.py --counter-workload --workload all")
    print("  python3 bench.py --results-table --pmc-plan <plan.log> --pmc-fetch <fetch>/p_counter_collection.csv \\")
    print("          --pmc-write <write>/p_counter_collection.csv --parity-log <errors.jsonl>")
    print()
    print("columns: us per call (median of 5 timed loops of %d calls); GB/s = algorithmic bytes (2 S forward, 3 S backward) / time of forward + backward;" % steps)
    print("  %peak = that / 8000 GB/s; traffic = FETCH_SIZE + WRITE_SIZE of all launches of the call, calibrated on a 256 MiB plain copy")
    print("  (1 FETCH_SIZE unit = %.1f bytes, 1 WRITE_SIZE unit = %.1f bytes), ratio = traffic / algorithmic bytes; copy us = the library's plain" % (fu, wu))
    print("  copy kernel reading and writing one tensor of the same size (2 S); cpu us = torch.nn.functional.group_norm + activation (+ autograd)")
    print("  on %d host threads, same tensors; err = max |ours - truth| / (|truth| + rms(truth)) against the float64 oracle, observed / bar" % cpu["cores"])
    print("  (float32: bar 1e-5 and also the pure relative error over |truth| >= rms, in brackets; 16-bit: bar = torch's own error in that type + 2 %).")
    print("  kernel = what the library launched (rows per lane of the register tile, x window rows, rows of x parked in LDS, two-level exchange, launches per call).")
    print()
    hdr = "%-20s %-5s %-22s %7s %7s %8s %7s %6s | %7s %6s %7s %6s | %7s %9s | %-34s | %s" % (
        "config", "dtype", "shape (N,C,spatial) G", "fwd us", "bwd us", "f+b us", "GB/s", "%peak", "fwd MB", "ratio", "bwd MB", "ratio",
        "copy us", "cpu us", "err y / dx / dw / db (observed/bar)", "kernel fwd ; bwd")
    print(hdr)
    for n in names:
        cfg = configs.CONFIGS[n]
        S = configs.tensor_bytes(cfg)
        prob = Problem(cfg, device, 1)
        r = measure_shape(prob, None, steps, args.warmup, False)
        fwd_us = r["warm_fwd_us"]
        bwd_us = r.get("warm_bwd_us")
        both_us = r.get("warm_fwd_bwd_us", fwd_us)
        alg = (5 if prob.bwd else 2) * S
        gbps = alg / (both_us * 1e-6) / 1e9
        copy_us = 2 * S / copy_ceiling(S, device, steps) / 1e3
        ft = fetch[n]["fwd"] + write[n]["fwd"]
        bt = (fetch[n]["bwd"] + write[n]["bwd"]) if prob.bwd else None
        e = errs.get(n, {})

        def cell(k):
            if k not in e:
                return "-"
            v = e[k]
            extra = "[%.0e]" % v["rel"] if cfg.dtype in ("fp32", "fp64") else ""
            return "%.1e%s/%.1e" % (v["err"], extra, v["bar"])

        print("%-20s %-5s %-22s %7.2f %7s %8.2f %7.0f %6.1f | %7.1f %6.3f %7s %6s | %7.2f %9.0f | %-34s | %s ; %s" % (
            n, cfg.dtype, "%s G%d %s" % ("x".join(str(v) for v in cfg.shape), cfg.G, cfg.act), fwd_us,
            "%.2f" % bwd_us if bwd_us else "-", both_us, gbps, 100 * gbps / HBM_PEAK_GBPS, ft / 1e6, ft / (2 * S),
            "%.1f" % (bt / 1e6) if bt else "-", "%.3f" % (bt / (3 * S)) if bt else "-", copy_us, cpu["us_per_call"][n],
            " ".join(cell(k) for k in ("y", "dx", "dw", "db")), inst[n]["fwd_instance"], inst[n]["bwd_instance"] or "-"))
        sys.stdout.flush()
        del prob
        torch.cuda.empty_cache()
    print()
    print("machine-readable traffic per launch for bench.py (roofline.traffic), single-launch kernels only")
    print("(SOURCES: SHA-256, first 16 digits, of the kernel sources these counters were taken on):")
    print("SOURCES %s" % kernel_sources_sha16())
    for n in names:
        c = inst[n]
        if c["fwd_dispatches"] == 1 and c["fwd_instance"].startswith("fused"):
            print("TRAFFIC %s fused_fwd %.0f %.0f %s" % (n, fetch[n]["fwd"], write[n]["fwd"], c["fwd_instance"]))
        if c["bwd_dispatches"] == 1 and c["bwd_instance"] and c["bwd_instance"].startswith("fused"):
            print("TRAFFIC %s fused_bwd %.0f %.0f %s" % (n, fetch[n]["bwd"], write[n]["bwd"], c["bwd_instance"]))


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (GroupNorm statistics are per sample; nothing is exchanged "
              "between GPUs). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if args.code_placement:  # (the children touch the GPU; this process does not)
        code_placement(args.workload)
        return
    if args.timeline:
        os.environ["GNNHWC_TRACE"] = "2"  # read by the library at its first single-launch call
    import torch
    import workloads as configs

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    use_graph = args.graph
    if args.code_placement_child >= 0:
        code_placement_child(list(configs.SD_UNET_SWEEP) if args.workload == "sd_unet" else [args.workload], device,
                             args.code_placement_child)
        return
    if args.results_table:
        results_table(args, device)
        return
    if args.load_ceiling:
        load_ceiling(list(configs.SD_UNET_SWEEP) + ["c4a", "c4b", "c5b_bf16_silu"] if args.workload == "sd_unet" else [args.workload], device)
        return
    if args.recovery_cost:
        recovery_cost(list(configs.SD_UNET_SWEEP) + ["c4a", "c2"] if args.workload == "sd_unet" else [args.workload], device)
        return
    if args.switch_cost:
        switch_cost(list(configs.SD_UNET_SWEEP) if args.workload == "sd_unet" else
                    list(configs.ALL_NAMES) if args.workload == "all" else [args.workload], device)
        return
    if args.timeline:
        if args.workload == "sd_unet":
            timeline_in_sweep(list(configs.SD_UNET_SWEEP), device)
        timeline(["c3a", "c3b", "c3c", "c4a"] if args.workload == "sd_unet" else
                 list(configs.ALL_NAMES) if args.workload == "all" else [args.workload], device)
        return

    if args.workload == "sd_unet":
        head_names = list(configs.SD_UNET_SWEEP)
    elif args.workload == "all":
        head_names = list(configs.ALL_NAMES)
    else:
        head_names = [args.workload]
    probs = [Problem(configs.CONFIGS[n], device) for n in head_names]
    stream_of = lambda: torch.cuda.current_stream().cuda_stream  # noqa: E731

    def step():
        s = stream_of()
        for p in probs:
            p.step(0, s)

    if args.counter_workload:
        counter_workload(probs, device)
        return

    # ---- headline: K steps between synchronisations ----
    t = time_region(step, args.steps, args.warmup, use_graph, reps=1)
    alg = sum(p.alg_bytes() for p in probs)
    ms_per_step = t / args.steps * 1e3
    value = alg / (t / args.steps) / 1e9
    t_other = time_region(step, args.steps, args.warmup, not use_graph, reps=1)
    # the same K steps five more times (no further warm-up): spread of the headline figure
    repeats = [time_region(step, args.steps, 0, use_graph, reps=1) for _ in range(5)]

    # ---- per-kernel durations (HIP events on the launch stream) ----
    prof = kernel_profile(probs, max(20, args.steps // 4))
    S_of = {p.cfg.name: p.S for p in probs}

    def launch_bytes(name, kind):  # algorithmic bytes of ONE launch of this kind on this shape
        return KERNEL_STREAMS[kind] * S_of[name] / prof[name][kind][1]

    # time a kernel kind on a shape takes per step: mean launch duration x launches per call; the dominant kernel is
    # the one the step spends most of its time in
    step_us = {(n, k): prof[n][k][0] * prof[n][k][1] for n in prof for k in prof[n]}
    total_us = sum(step_us.values())
    dom_shape, dominant = max(step_us, key=step_us.get)
    dom_us = prof[dom_shape][dominant][0]
    dom_bytes = launch_bytes(dom_shape, dominant)
    achieved = dom_bytes / (dom_us * 1e-6) / 1e9
    traffic = recorded_traffic()
    by_name = {p.cfg.name: p for p in probs}
    tr, tr_why = traffic_of(traffic, by_name[dom_shape], dominant)
    roofline = {
        "bound": "hbm",
        "kernel": dominant,
        "shape": dom_shape,
        "achieved": round(achieved, 1),
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBPS, 4),
        "traffic": round(tr) if tr else None,
        "traffic_source": ("profiles/results_all_configs.txt (rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE, copy-calibrated; taken on "
                           "the kernel instance this run launches: %s)" % by_name[dom_shape].instance("bwd" if "bwd" in dominant else "fwd")
                           if tr else tr_why),
        "traffic_taken_on_sources": traffic.get(("", "sources")),
        "kernel_sources": kernel_sources_sha16(),
        "bytes_per_launch": dom_bytes,
        "mean_launch_us": round(dom_us, 3),
        "share_of_step": round(step_us[(dom_shape, dominant)] / total_us, 4),
        "selection": "largest share of the step's kernel time (mean launch duration x launches per step)",
        "kernels": {n: {k: {"us": round(us, 3), "launches_per_call": per_call, "alg_bytes": launch_bytes(n, k),
                            "frac": round(launch_bytes(n, k) / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                            "share_of_step": round(step_us[(n, k)] / total_us, 4),
                            "traffic": (lambda t: round(t) if t else None)(traffic_of(traffic, by_name[n], k)[0])}
                        for k, (us, per_call) in kinds.items()} for n, kinds in prof.items()},
    }

    # ---- per-shape table ----
    shapes = {}
    names = [] if args.no_shapes else list(configs.ALL_NAMES) if args.all else head_names
    for n in names:
        cfg = configs.CONFIGS[n]
        S = configs.tensor_bytes(cfg)
        nsets = max(2, int(600e6 // (4 * S)) + 1)
        warm = Problem(cfg, device, 1)
        cold = Problem(cfg, device, nsets)
        k = max(20, args.steps // 2)
        r = measure_shape(warm, cold, k, args.warmup, use_graph)
        r.update(dtype=cfg.dtype, shape=list(cfg.shape), G=cfg.G, act=cfg.act, S_bytes=S)
        key = "fwd_bwd" if cfg.passes != "fwd" else "fwd"
        r["warm_frac_of_peak"] = round(r["warm_%s_gbps" % key] / HBM_PEAK_GBPS, 4)
        r["cold_frac_of_peak"] = round(r["cold_%s_gbps" % key] / HBM_PEAK_GBPS, 4)
        r["copy_kernel_gbps"] = round(copy_ceiling(S, device, k), 1)
        shapes[n] = r
        del warm, cold
        torch.cuda.empty_cache()

    line = {
        "metric": ("fused GN+SiLU fwd+bwd achieved HBM GB/s (algorithmic bytes / time), SD-UNet shapes" if args.workload == "sd_unet"
                   else "fused GN+activation achieved HBM GB/s (algorithmic bytes / time), workload %s" % args.workload),
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "us_per_call": {p.cfg.name: shapes[p.cfg.name].get("warm_fwd_bwd_us", shapes[p.cfg.name].get("warm_fwd_us"))
                        for p in probs if p.cfg.name in shapes},
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": ({"bf16": "bf16 data, f32 arithmetic", "fp16": "f16 data, f32 arithmetic", "fp32": "f32", "fp64": "f64"}[probs[0].cfg.dtype]
                  if len({p.cfg.dtype for p in probs}) == 1 else "mixed (f32 arithmetic)"),
        "data": "synthetic (seeded)",
        "config": {"workload": "+".join(head_names) if len(head_names) <= 4 else "%s (%d configurations)" % (args.workload, len(head_names)),
                   "passes": "fwd+bwd" if all(p.bwd for p in probs) else "per configuration",
                   "activation": probs[0].cfg.act if len({p.cfg.act for p in probs}) == 1 else "per configuration",
                   "timing": "HIP graph replay of the K steps" if use_graph else "eager launches through the C ABI",
                   "algorithmic_bytes_per_step": alg},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
        # the reference's own benchmark counts 3 tensor sizes for a forward and 8 for forward + backward
        # (benchmark.py:101,107); the same time expressed in that accounting, for comparison with its CSVs
        "reference_accounting_gbps": round(sum((8 if p.bwd else 3) * p.S for p in probs) / (t / args.steps) / 1e9, 1),
        ("eager_ms_per_step" if use_graph else "graph_replay_ms_per_step"): round(t_other / args.steps * 1e3, 5),
        "repeat_ms_per_step": [round(r / args.steps * 1e3, 5) for r in repeats],
        "repeat_median_gbps": round(alg / (statistics.median(repeats) / args.steps) / 1e9, 1),
        "roofline": roofline,
        "shapes": shapes,
    }
    if args.nchw:
        line["channels_first"] = nchw_table(head_names, device, max(20, args.steps // 2), args.warmup)
    if args.cast:
        line["cast"] = cast_table(head_names, device, max(20, args.steps // 2), args.warmup)
    if args.fused_add:
        line["fused_add"] = fused_add_table(head_names, device, max(20, args.steps // 2), args.warmup)
    if not args.no_torch_gpu:
        line["torch_gpu"] = torch_gpu_leg(head_names, device, max(10, args.steps // 4), min(args.warmup, 5))
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(head_names, args.cpu_seconds)
    print(json.dumps(line))


if __name__ == "__main__":
    main()

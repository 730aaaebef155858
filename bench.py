"""Benchmark of the per-rank hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--skip-cpu] [--skip-layers] [--only NAMES | --all]

Headline workload (BASELINE.json configs[1]): Repartition pack + unpack of one
rank, bf16 global tensor [8,4096,8192] moved from P_x=[1,8,1] to P_y=[1,1,8].
One step = one pack launch (the [8,512,8192] shard into eight [8,512,1024]
boxes) + one unpack launch (eight seeded boxes into the [8,4096,1024] output
shard) = 268 435 456 algorithmic bytes.  The box lists come from the product's
own planner (distdl_amd.nn.Repartition's set-up on rank 0 of 8) and are
asserted equal to the oracle's before anything is timed.  Inputs are resident
in HBM before the timed region; a step rotates over several buffer sets so that
the 256 MB last-level cache cannot hold the working set.  The other hot-path
kernels (LayerNorm, Embedding, Linear GEMM, halo staging) are measured the same
way and reported under "workloads" of the same JSON line, and once more, one
short entry each, under roofline["configs"] and cpu_baseline["configs"].  A run
without --only / --all measures the five BASELINE configurations and the few
workloads read next to them (DEFAULT_WORKLOADS); --all adds the backward
kernels, fp32 GEMM, slab-only halo exchange, re-layouts and MFMA probes.  Each
workload carries

  roofline      algorithmic work / HIP-event time of the step's launches
  layer         microseconds per forward call of the distdl_amd.nn module that
                wraps the kernel (host path included), next to the kernel time
  cpu_baseline  the oracle's CPU restatement of the reference path, timed on a
                bounded sample in this same run

Timing: the launches of the timed region are captured once into a HIP graph
(no host work between kernels) and replayed; wall clock with a device
synchronisation on both sides gives ms_per_step, HIP events on the launch
stream give the per-launch kernel duration used for the roofline.  Workloads
whose step takes 20 us or more are timed a second time with the same launches
issued directly on the stream (no dependency edges between graph nodes, and
the host stays ahead of kernels that long); the record is the faster of the
two and names its mode.  If graph capture is unavailable only the stream mode
runs.
The headline runs exactly --steps steps; the other workloads run at least 100
steps after at least 20 warm-ups, whatever --steps says, because the GEMM's
clock needs that many samples to settle.
"""

import argparse
import ctypes
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published
MFMA_F32_PEAK_TFLOPS = 157.3    # MI355X dense fp32 matrix, published
MIN_SECONDARY_STEPS, MIN_SECONDARY_WARMUP = 100, 20


def profile_traffic(name, combine):
    """HBM bytes per launch of a workload, as measured with rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE (each counter scaled by what it reads for a plain
    copy of known size) and written down in profiles/<name>_hbm_traffic_pmc.txt:
    one "traffic (read + write) = N B" line per kernel of a step.  These are not
    measured by the run that prints them; None when there is no such summary."""
    path = os.path.join(ROOT, "profiles", f"{name}_hbm_traffic_pmc.txt")
    try:
        with open(path) as f:
            values = [int(v) for v in re.findall(r"traffic \(read \+ write\) = (\d+) B", f.read())]
    except OSError:
        return None
    if not values:
        return None
    return sum(values) / len(values) if combine == "mean" else sum(values)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--skip-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--skip-layers", action="store_true", help="skip the module-level (host path included) timings")
    ap.add_argument("--only", default=None, help="run only these workloads, comma-separated; see WORKLOADS")
    ap.add_argument("--all", action="store_true", help="every workload of WORKLOADS except the comparison figures "
                    "(backward kernels, fp32 GEMM, slab-only halo, MFMA probes, ...) instead of the default set")
    ap.add_argument("--no-graph", action="store_true", help="launch on the stream instead of replaying a HIP graph")
    ap.add_argument("--cpu-worker", default=None, help=argparse.SUPPRESS)
    return ap.parse_args()


# The stream every launch closure uses; rebound to the capture stream while a
# graph is being recorded.
STREAM = [ctypes.c_void_p(0)]


def bind_stream(torch):
    STREAM[0] = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


class Timed:
    """A list of zero-argument launch closures, run `steps` times."""

    def __init__(self, torch, launches_per_step, use_graph):
        self.torch = torch
        self.step_fns = launches_per_step      # list over buffer sets of [closures of one step]
        self.use_graph = use_graph
        self.graph = None
        self.rest_graphs = {}
        self.mode = "stream"

    def _run_sets(self):
        bind_stream(self.torch)
        for fns in self.step_fns:
            for fn in fns:
                fn()

    def prepare(self):
        torch = self.torch
        self._run_sets()
        torch.cuda.synchronize()
        if not self.use_graph:
            return
        try:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                self._run_sets()
            graph.replay()
            torch.cuda.synchronize()
            self.graph = graph
            self.mode = "graph"
        except Exception as exc:  # graph capture refused: keep the stream mode
            sys.stderr.write(f"[bench] HIP graph capture unavailable ({exc}); launching on the stream\n")
            self.graph = None
            torch.cuda.synchronize()

    def _rest_graph(self, rest):
        """A graph of the first `rest` buffer sets, for step counts that are no
        multiple of the number of sets; captured (and replayed once) outside the
        timed region.  None when capture is refused."""
        torch = self.torch
        if rest in self.rest_graphs:
            return self.rest_graphs[rest]
        graph = None
        try:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                bind_stream(torch)
                for fns in self.step_fns[:rest]:
                    for fn in fns:
                        fn()
            graph.replay()
            torch.cuda.synchronize()
        except Exception as exc:
            sys.stderr.write(f"[bench] capture of the {rest}-step remainder refused ({exc}); launching it on the stream\n")
            graph = None
            torch.cuda.synchronize()
        self.rest_graphs[rest] = graph
        return graph

    def run(self, steps):
        """Runs exactly `steps` steps: whole passes over the buffer sets (graph
        replays when a graph was captured) and the remaining steps from a
        second, shorter graph (or launched on the stream when nothing could be
        captured).  Returns (steps, wall seconds, event seconds)."""
        torch = self.torch
        nsets = len(self.step_fns)
        passes, rest = divmod(steps, nsets)
        rest_graph = self._rest_graph(rest) if self.graph is not None and rest else None
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        bind_stream(torch)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(passes):
            if self.graph is not None:
                self.graph.replay()
            else:
                self._run_sets()
        if rest_graph is not None:
            rest_graph.replay()
        else:
            for fns in self.step_fns[:rest]:
                for fn in fns:
                    fn()
        e1.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        return steps, t1 - t0, e0.elapsed_time(e1) * 1e-3


STREAM_MODE_MIN_STEP_US = 20.0


def measure(torch, name, step_fns, launches_per_step, steps, warmup, use_graph):
    """Times `steps` steps after `warmup` untimed ones.  The launches are replayed from a HIP graph; when a step is long
    enough for the host to stay ahead of the device (at least STREAM_MODE_MIN_STEP_US), the same launches are also
    issued directly on the stream, for another `warmup` + `steps` steps, and the record is that of the faster way of
    launching (a graph puts a dependency between consecutive kernel nodes, which costs long kernels a few tenths of a
    microsecond each; short kernels are host-bound on the stream).  `mode` says which; `us_per_step_by_mode` has both."""
    def run(graph):
        timed = Timed(torch, step_fns, graph)
        timed.prepare()
        if warmup > 0:
            timed.run(warmup)
        n, wall, ev = timed.run(steps)
        return {"name": name, "steps": n, "wall_s": wall, "event_s": ev, "mode": timed.mode,
                "launch_s": ev / (n * launches_per_step)}
    best = run(use_graph)
    by_mode = {best["mode"]: 1e6 * best["event_s"] / best["steps"]}
    if best["mode"] == "graph" and by_mode["graph"] >= STREAM_MODE_MIN_STEP_US:
        other = run(False)
        by_mode[other["mode"]] = 1e6 * other["event_s"] / other["steps"]
        if other["event_s"] < best["event_s"]:
            best = other
    best["us_per_step_by_mode"] = by_mode
    return best


def _call(lib, _lib, name, args):
    def fn(a=args, f=getattr(lib, name), n=name):
        rc = f(*a, STREAM[0])
        if rc:
            _lib.check(rc, n)
    return fn


def time_layer(torch, fn, inputs, calls=200, warm=10, grad=False):
    """Microseconds per call of a module's forward, `fn(x)` over the inputs in
    turn (enough of them that the last-level cache cannot hold what one round
    touches): the host loop alone, and with the device drained at the end (the
    larger of the two is what a caller sees per call in steady state).  With
    `grad` the calls record for autograd (the forward of a training step)."""
    n = len(inputs)
    with torch.enable_grad() if grad else torch.no_grad():
        for i in range(warm):
            fn(inputs[i % n])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(calls):
            fn(inputs[i % n])
        t1 = time.perf_counter()
        torch.cuda.synchronize()
        t2 = time.perf_counter()
    return {"host_us": 1e6 * (t1 - t0) / calls, "us": 1e6 * (t2 - t0) / calls, "calls": calls, "inputs": n}


def timed_cpu(fn, budget_s):
    """Runs fn() (one sample) until about budget_s seconds are spent; returns
    (runs, seconds), after one untimed run."""
    fn()
    n, t0 = 0, time.perf_counter()
    while True:
        fn()
        n += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s:
            return n, dt


# ----------------------------------------------------------------------------
# configuration 2: Repartition (headline)
# ----------------------------------------------------------------------------

def repartition_layer(torch):
    """The product's Repartition for configuration 2 on rank 0 of 8, set up
    for the [8,512,8192] bf16 shard: (layer, x)."""
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import Repartition
    world = SimWorld(8)
    base = world.partition(0).create_partition_inclusive(list(range(8)))
    P_x = base.create_cartesian_topology_partition([1, 8, 1])
    P_y = base.create_cartesian_topology_partition([1, 1, 8])
    layer = Repartition(P_x, P_y)
    gen = torch.Generator().manual_seed(1002)
    x = (2 * torch.rand(8, 512, 8192, generator=gen) - 1).to(torch.bfloat16).cuda()
    layer._distdl_forward_pre_hook(layer, (x,))       # what torch calls in front of forward
    return layer, x


def build_repartition(torch, lib, _lib, nsets):
    """Config 2.  Box lists from the product's planner, checked against the oracle's."""
    from oracle import repartition as o_rep
    layer, x0 = repartition_layer(torch)
    send0 = [tuple(sl) for sl, sh, p in layer.P_x_to_y_overlaps]
    recv0 = [tuple(sl) for sl, sh, p in layer.P_y_to_x_overlaps]
    o_send, o_recv, _, _ = o_rep.plan([8, 4096, 8192], [1, 8, 1], [1, 1, 8])

    def norm(slices):
        return [tuple((int(s.start), int(s.stop)) for s in sl) for sl in slices]
    assert norm(send0) == norm([sl for sl, sh, p in o_send[0]]), "planner and oracle disagree on the send boxes"
    assert norm(recv0) == norm([sl for sl, sh, p in o_recv[0]]), "planner and oracle disagree on the receive boxes"
    assert tuple(layer.output_tensor_structure.shape) == (8, 4096, 1024)
    del x0
    keep, steps = [], []
    for s in range(nsets):
        gen = torch.Generator().manual_seed(1002 + s)
        x = (2 * torch.rand(8, 512, 8192, generator=gen) - 1).to(torch.bfloat16).cuda()
        sbufs = [torch.empty(8, 512, 1024, dtype=torch.bfloat16, device="cuda") for _ in range(8)]
        gen = torch.Generator().manual_seed(1102 + s)
        rbufs = [(2 * torch.rand(8, 512, 1024, generator=gen) - 1).to(torch.bfloat16).cuda() for _ in range(8)]
        y = torch.empty(8, 4096, 1024, dtype=torch.bfloat16, device="cuda")
        pack_args = (x.data_ptr(), _lib.i64_array(x.shape), _lib.i64_array(x.stride()), 3, 2, 8,
                     _lib.i64_array([int(sl_d.start) for sl in send0 for sl_d in sl]),
                     _lib.i64_array([int(sl_d.stop - sl_d.start) for sl in send0 for sl_d in sl]),
                     _lib.ptr_array([b.data_ptr() for b in sbufs]))
        unpack_args = (y.data_ptr(), _lib.i64_array(y.shape), _lib.i64_array(y.stride()), 3, 2, 8,
                       _lib.i64_array([int(sl_d.start) for sl in recv0 for sl_d in sl]),
                       _lib.i64_array([int(sl_d.stop - sl_d.start) for sl in recv0 for sl_d in sl]),
                       _lib.ptr_array([b.data_ptr() for b in rbufs]), 0, 0)
        keep.append((x, sbufs, rbufs, y, pack_args, unpack_args))
        steps.append([_call(lib, _lib, "ddl_pack_boxes", pack_args), _call(lib, _lib, "ddl_unpack_boxes", unpack_args)])
    return steps, keep, 268435456


def _build_repartition_half(which):
    def build(torch, lib, _lib, nsets):
        """Config 2's pack (or unpack) alone, one launch per step: the two
        halves of the headline step timed separately."""
        steps, keep, _ = build_repartition(torch, lib, _lib, nsets)
        return [[fns[which]] for fns in steps], keep, 134217728
    return build


def layer_repartition(torch):
    layer, x = repartition_layer(torch)
    xs = [x] + [torch.empty_like(x).copy_(x) for _ in range(5)]      # 6 x 64 MiB in, as much out
    rec = time_layer(torch, layer, xs)
    rec["module"] = "Repartition([1,8,1]->[1,1,8]).forward, no_grad, rank 0 of 8, solo transport"
    return rec


def _cpu_repartition_rank(rank, budget_s):
    """(steps, seconds) of one rank's pack + unpack of config 2 with the
    oracle's NumPy code (np.copyto per box, zero-filled output), single thread,
    uint16 views of the bf16 payload."""
    import numpy as np
    from oracle import repartition as o_rep
    send, recv, _, _ = o_rep.plan([8, 4096, 8192], [1, 8, 1], [1, 1, 8])
    send_r = [(sl, sh, 99 if p == "self" else p) for sl, sh, p in send[rank]]
    recv_r = [(sl, sh, 99 if p == "self" else p) for sl, sh, p in recv[rank]]
    rng = np.random.default_rng(1002 + rank)
    x = rng.integers(0, 2 ** 16, size=(8, 512, 8192), dtype=np.uint16)
    rbufs = [rng.integers(0, 2 ** 16, size=(8, 512, 1024), dtype=np.uint16) for _ in range(8)]

    def step():
        o_rep.pack(x, send_r)
        o_rep.unpack(recv_r, rbufs, (8, 4096, 1024), np.uint16)
    return timed_cpu(step, budget_s)


def cpu_worker(spec):
    """`bench.py --cpu-worker repartition:RANK:SECONDS`: one rank of the CPU
    baseline as a process of its own (NumPy only, nothing touches the GPU);
    prints {"steps", "seconds"}."""
    what, rank, seconds = spec.split(":")
    if what != "repartition":
        raise SystemExit(f"bench.py: no CPU worker for {what!r}")
    n, dt = _cpu_repartition_rank(int(rank), float(seconds))
    print(json.dumps({"steps": n, "seconds": dt}))


def cpu_repartition_all_ranks(budget_s=6.0, ranks=8):
    """The eight ranks of config 2 at once, one process each, as `mpirun -np 8`
    would run the reference's CPU backend (without its messages): what the box's
    cores sustain together, next to the one rank the GPU's figure stands for."""
    import subprocess
    procs = [subprocess.Popen([sys.executable, os.path.abspath(__file__), "--cpu-worker", f"repartition:{r}:{budget_s}"],
                              stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True) for r in range(ranks)]
    rates = []
    for p in procs:
        out, _ = p.communicate(timeout=120 + 10 * budget_s)
        if p.returncode != 0:
            return None
        rec = json.loads(out.strip().splitlines()[-1])
        rates.append(268435456 * rec["steps"] / rec["seconds"] / 1e9)
    return {"processes": ranks, "value": sum(rates), "unit": "GB/s", "per_process": sum(rates) / len(rates),
            "what": f"{ranks} rank processes running config 2's pack + unpack at the same time, {budget_s:.0f} s each, summed"}


def cpu_repartition(budget_s=12.0):
    """One rank's pack + unpack of config 2 on one core, and all eight ranks at
    once on eight processes."""
    n, dt = _cpu_repartition_rank(0, budget_s)
    return {"all_ranks": cpu_repartition_all_ranks(),
            "value": 268435456 * n / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{n} full steps of config 2, np.copyto per box + zero-filled output, one process as rank 0, {dt:.1f} s"}


# ----------------------------------------------------------------------------
# configuration 1: LayerNorm
# ----------------------------------------------------------------------------

def _ln_steps(torch, lib, _lib, nsets, rows, cols, seed, peers_from_global):
    import numpy as np
    from oracle import layernorm as o_ln
    keep, steps = [], []
    part_cols = _lib.i64_array([cols] * 4)
    for s in range(nsets):
        if peers_from_global:
            gen = torch.Generator().manual_seed(seed + s)
            xg = torch.randn(16, 512, 4 * cols, generator=gen)
            gamma = (1 + 0.1 * torch.randn(4 * cols, generator=gen))[:cols].contiguous().cuda()
            beta = (0.1 * torch.randn(4 * cols, generator=gen))[:cols].contiguous().cuda()
            x = xg[..., :cols].contiguous().cuda().reshape(rows, cols)
            gathered = torch.empty(4, rows, 2, device="cuda")
            for p in range(1, 4):   # peers' partial statistics: seeded, computed on the CPU from the same global x
                gathered[p] = torch.from_numpy(o_ln.partial_stats(xg[..., cols * p:cols * (p + 1)].numpy()).astype(np.float32))
        else:
            gen = torch.Generator(device="cuda").manual_seed(seed + s)
            x = torch.randn(rows, cols, generator=gen, device="cuda")
            gamma = 1 + 0.1 * torch.randn(cols, generator=gen, device="cuda")
            beta = 0.1 * torch.randn(cols, generator=gen, device="cuda")
            gathered = torch.zeros(4, rows, 2, device="cuda")
            gathered[1:, :, 1] = float(cols)                             # peers: mean 0, M2 = n (unit variance)
        y = torch.empty_like(x)
        stats_args = (x.data_ptr(), rows, cols, cols, gathered.data_ptr())      # own partials land in slot 0
        norm_args = (x.data_ptr(), rows, cols, cols, gathered.data_ptr(), 4, part_cols, gamma.data_ptr(),
                     beta.data_ptr(), 1e-5, y.data_ptr(), cols, None, None)
        keep.append((x, gamma, beta, gathered, y, stats_args, norm_args))
        steps.append([_call(lib, _lib, "ddl_ln_partial_stats_f32", stats_args),
                      _call(lib, _lib, "ddl_ln_normalize_affine_f32", norm_args)])
    return steps, keep


def ln_bytes(rows, cols, nparts=4):
    # x read by both kernels, y written once, gamma and beta, own statistics written and all nparts read back
    return 3 * rows * cols * 4 + 2 * cols * 4 + rows * 8 + nparts * rows * 8


def build_layernorm(torch, lib, _lib, nsets):
    """Config 1: rank 0's [16,512,256] fp32 shard; stats + normalize."""
    steps, keep = _ln_steps(torch, lib, _lib, nsets, 16 * 512, 256, 1001, True)
    return steps, keep, 25298944


def build_layernorm_joined(torch, lib, _lib, nsets):
    """Config 1 in one launch (ddl_ln_stats_normalize): the peers' statistics are
    seeded, i.e. in memory before the launch, so the kernel that computes rank
    0's partial sums can go on to normalise with the row still in registers.
    `work` is what the kernel moves -- x read ONCE, y written, statistics and
    parameters -- not config 1's three passes; the two-launch form (workload
    `layernorm`) is what applies when peers compute at the same time."""
    rows, cols = 16 * 512, 256
    steps2, keep = _ln_steps(torch, lib, _lib, nsets, rows, cols, 1001, True)
    part_cols = _lib.i64_array([cols] * 4)
    steps = []
    for (x, gamma, beta, gathered, y, _, _) in keep:
        args = (x.data_ptr(), _lib.DDL_DT_F32, rows, cols, cols, gathered.data_ptr(), 4, 0, part_cols, gamma.data_ptr(),
                beta.data_ptr(), 1e-5, y.data_ptr(), cols, None, None)
        steps.append([_call(lib, _lib, "ddl_ln_stats_normalize", args)])
    keep.append(part_cols)
    return steps, keep, 2 * rows * cols * 4 + 2 * cols * 4 + 4 * rows * 8


def build_layernorm_long(torch, lib, _lib, nsets):
    """The kernels of config 1 on 32 times its rows ([262144, 256] fp32, 268 MB):
    the streaming rate of the same code once launch ramp and memory latency no
    longer dominate.  Not a BASELINE configuration; reported next to config 1."""
    steps, keep = _ln_steps(torch, lib, _lib, nsets, 32 * 16 * 512, 256, 2001, False)
    return steps, keep, 32 * 25298944 - 31 * 2 * 256 * 4


def build_layernorm_wide(torch, lib, _lib, nsets):
    """Rows longer than a wavefront keeps in registers: [4096, 8192] fp32
    (128 MiB), one workgroup per row.  Not a BASELINE configuration."""
    rows, cols = 4096, 8192
    steps, keep = _ln_steps(torch, lib, _lib, nsets, rows, cols, 2101, False)
    return steps, keep, ln_bytes(rows, cols)


def build_layernorm_local(torch, lib, _lib, nsets):
    """The single-launch kernel for rows one worker holds whole (the reference's
    F.layer_norm branch): the global rows of config 1, [8192, 1024] fp32."""
    rows, cols = 16 * 512, 1024
    keep, steps = [], []
    for s in range(nsets):
        gen = torch.Generator(device="cuda").manual_seed(2201 + s)
        x = torch.randn(rows, cols, generator=gen, device="cuda")
        gamma = 1 + 0.1 * torch.randn(cols, generator=gen, device="cuda")
        beta = 0.1 * torch.randn(cols, generator=gen, device="cuda")
        y = torch.empty_like(x)
        args = (x.data_ptr(), _lib.DDL_DT_F32, rows, cols, cols, gamma.data_ptr(), beta.data_ptr(), 1e-5, y.data_ptr(),
                cols, None, None)
        keep.append((x, gamma, beta, y, args))
        steps.append([_call(lib, _lib, "ddl_layer_norm", args)])
    return steps, keep, 2 * rows * cols * 4 + 2 * cols * 4


def layer_layernorm(torch):
    import numpy as np
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import DistributedLayerNorm
    from distdl_amd.nn.layernorm import STATS_TAG
    from oracle import layernorm as o_ln
    world = SimWorld(4)
    P_x = world.partition(0).create_partition_inclusive(list(range(4))).create_cartesian_topology_partition([1, 1, 4])
    layer = DistributedLayerNorm(P_x, [1024])
    gen = torch.Generator().manual_seed(1001)
    xg = torch.randn(16, 512, 1024, generator=gen)
    x = xg[..., :256].contiguous().cuda()
    peers = [None] + [torch.from_numpy(o_ln.partial_stats(xg[..., 256 * p:256 * (p + 1)].numpy()).astype(np.float32)).cuda()
                      for p in range(1, 4)]
    world.transport.set_gather_provider(STATS_TAG, lambda P, t: list(peers), constant=True)
    xs = [x] + [torch.empty_like(x).copy_(x) for _ in range(63)]     # 64 x 8 MiB in, as much out
    rec = time_layer(torch, layer, xs, calls=256)
    rec["module"] = "DistributedLayerNorm([1,1,4], 1024).forward, no_grad, rank 0 of 4, peers' statistics seeded"
    grad = time_layer(torch, layer, [t.requires_grad_(True) for t in xs], calls=256, grad=True)
    rec["host_us_grad_mode"], rec["us_grad_mode"] = grad["host_us"], grad["us"]
    return rec


def cpu_layernorm(budget_s=4.0):
    """Rank 0's share of the reference's op sequence (local mean, all-reduce,
    local mean of squared deviations, all-reduce, normalise, affine) in NumPy
    fp32, the all-reduces replaced by adding the seeded sums of ranks 1-3."""
    import numpy as np
    from oracle import layernorm as o_ln
    rng = np.random.default_rng(1001)
    xg = rng.standard_normal((16, 512, 1024), dtype=np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(256)).astype(np.float32)
    beta = (0.1 * rng.standard_normal(256)).astype(np.float32)
    x = np.ascontiguousarray(xg[..., :256])
    mean = xg.mean(axis=-1, keepdims=True)
    peer_mean = sum(xg[..., 256 * p:256 * (p + 1)].mean(axis=-1, keepdims=True) for p in range(1, 4))
    peer_var = sum(((xg[..., 256 * p:256 * (p + 1)] - mean) ** 2).mean(axis=-1, keepdims=True) for p in range(1, 4))
    n, dt = timed_cpu(lambda: o_ln.forward_rank(x, peer_mean, peer_var, 4, gamma, beta, 1e-5), budget_s)
    return {"value": 25298944 * n / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{n} full steps of config 1 on rank 0, the reference's op sequence in NumPy fp32, seeded peer sums, {dt:.1f} s"}


# ----------------------------------------------------------------------------
# configuration 3: Embedding
# ----------------------------------------------------------------------------

def build_embedding(torch, lib, _lib, nsets):
    """Config 3: rank-0 vocabulary shard [16032,4096] bf16, ids [32,4096] int64."""
    gen = torch.Generator().manual_seed(1003)
    table = (0.02 * torch.randn(16032, 4096, generator=gen)).to(torch.bfloat16).cuda()
    keep, steps, nbytes = [table], [], []
    for s in range(nsets):
        gen = torch.Generator().manual_seed(2003 + s)
        ids = torch.randint(0, 128256, (32, 4096), generator=gen)
        n_hit = int((ids < 16032).sum())
        nbytes.append(32 * 4096 * 4096 * 2 + ids.numel() * 8 + n_hit * 8192)
        ids = ids.cuda()
        out = torch.empty(32, 4096, 4096, dtype=torch.bfloat16, device="cuda")
        args = (table.data_ptr(), 4096, 4096, 2, ids.data_ptr(), 1, ids.numel(), 0, 16032, out.data_ptr())
        keep.append((ids, out, args))
        steps.append([_call(lib, _lib, "ddl_embedding_gather", args)])
    return steps, keep, sum(nbytes) / len(nbytes)


def layer_embedding(torch):
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import DistributedEmbedding
    world = SimWorld(1)
    P_x = world.partition(0).create_partition_inclusive([0]).create_cartesian_topology_partition([1, 1, 1])
    layer = DistributedEmbedding(P_x, 128256, 4096, dtype=torch.bfloat16, vocab_shard=(0, 16032))
    ids = [torch.randint(0, 128256, (32, 4096), generator=torch.Generator().manual_seed(2003 + s)).cuda() for s in range(4)]
    rec = time_layer(torch, layer, ids, calls=48, warm=4)            # every call writes a new 1 GiB
    rec["module"] = "DistributedEmbedding(128256, 4096, bf16, vocab_shard=(0,16032)).forward, no_grad, ids [32,4096]"
    return rec


def cpu_embedding(budget_s=4.0):
    """The oracle's gather (NumPy row indexing, zero rows outside the window) on
    the first 4096 tokens of config 3 against the full rank-0 shard."""
    import numpy as np
    from oracle import embedding as o_emb
    rng = np.random.default_rng(1003)
    table = rng.integers(0, 2 ** 16, size=(16032, 4096), dtype=np.uint16)
    ids = rng.integers(0, 128256, size=(4096,), dtype=np.int64)
    n_hit = int((ids < 16032).sum())
    nbytes = ids.size * 4096 * 2 + ids.size * 8 + n_hit * 8192
    n, dt = timed_cpu(lambda: o_emb.gather(table, ids, 0, 16032), budget_s)
    return {"value": nbytes * n / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{n} gathers of 4096 of config 3's 131072 tokens (1/32 step), NumPy indexing, {dt:.1f} s"}


# ----------------------------------------------------------------------------
# configuration 4: Linear
# ----------------------------------------------------------------------------

def _linear_operands(torch, nsets):
    gen = torch.Generator().manual_seed(1004)
    w = (0.02 * torch.randn(3584, 8192, generator=gen)).to(torch.bfloat16).cuda()
    b = (0.02 * torch.randn(3584, generator=gen)).to(torch.bfloat16).cuda()
    xs = []
    for s in range(nsets):
        gen = torch.Generator().manual_seed(3004 + s)
        xs.append(torch.randn(4, 2048, 8192, generator=gen).to(torch.bfloat16).cuda())
    return w, b, xs


def build_linear(torch, lib, _lib, nsets):
    """Config 4: M=8192 N=3584 K=8192 bf16, fp32 accumulate, bias."""
    w, b, xs = _linear_operands(torch, nsets)
    keep, steps = [w, b], []
    for x in xs:
        y = torch.empty(4, 2048, 3584, dtype=torch.bfloat16, device="cuda")
        args = (x.data_ptr(), w.data_ptr(), b.data_ptr(), y.data_ptr(), 8192, 3584, 8192, 8192, 8192, 3584)
        keep.append((x, y, args))
        steps.append([_call(lib, _lib, "ddl_linear_bf16", args)])
    return steps, keep, 2 * 8192 * 3584 * 8192


def _build_linear_f32(library):
    def build(torch, lib, _lib, nsets):
        M, N, K = 8192, 3584, 8192
        gen = torch.Generator(device="cuda").manual_seed(7004)
        w = 0.02 * torch.randn(N, K, generator=gen, device="cuda")
        b = 0.02 * torch.randn(N, generator=gen, device="cuda")
        keep, steps = [w, b], []
        for s in range(nsets):
            x = torch.randn(M, K, generator=gen, device="cuda")
            if library:
                keep.append(x)

                def gemm(x=x):
                    torch.nn.functional.linear(x, w, b)
                steps.append([gemm])
            else:
                y = torch.empty(M, N, device="cuda")
                keep.append((x, y))
                steps.append([_call(lib, _lib, "ddl_linear", (x.data_ptr(), w.data_ptr(), b.data_ptr(), y.data_ptr(), _lib.DDL_DT_F32,
                                                              M, N, K, K, K, N))])
        return steps, keep, 2 * M * N * K
    build.__doc__ = ("Config 4's shape in float32, the default dtype of the reference's layers: M=8192 N=3584 K=8192, bias, "
                     + ("through torch.nn.functional.linear (the vendor GEMM library), for comparison." if library else
                        "through ddl_linear (fp32 MFMA kernel)."))
    return build


def build_linear_f32_bwd(torch, lib, _lib, nsets):
    """Backward of the float32 shard of config 4's shape: dx = dy w and dw = dy^T x through ddl_gemm_f32 on the
    operands where they lie, db = column sums of dy.  Work: 2 x 2 M N K flop."""
    M, N, K = 8192, 3584, 8192
    gen = torch.Generator(device="cuda").manual_seed(7005)
    w = 0.02 * torch.randn(N, K, generator=gen, device="cuda")
    work = torch.empty(64 * N, device="cuda")
    keep, steps = [w, work], []
    f32 = _lib.DDL_DT_F32
    for s in range(nsets):
        x = torch.randn(M, K, generator=gen, device="cuda")
        dy = torch.randn(M, N, generator=gen, device="cuda")
        dx, dw, db = torch.empty(M, K, device="cuda"), torch.empty(N, K, device="cuda"), torch.empty(N, device="cuda")
        keep.append((x, dy, dx, dw, db))
        steps.append([
            _call(lib, _lib, "ddl_gemm_f32", (dy.data_ptr(), N, 1, w.data_ptr(), 1, K, None, dx.data_ptr(), K, M, K, N)),
            _call(lib, _lib, "ddl_gemm_f32", (dy.data_ptr(), 1, N, x.data_ptr(), 1, K, None, dw.data_ptr(), K, N, K, M)),
            _call(lib, _lib, "ddl_colsum", (dy.data_ptr(), f32, M, N, N, db.data_ptr(), work.data_ptr(), work.numel())),
        ])
    return steps, keep, 2 * 2 * M * N * K


def build_linear_library(torch, lib, _lib, nsets):
    """The same product on the same operands through torch.nn.functional.linear
    (the vendor GEMM library): the comparison figure for the hand-written
    kernel, not a product path."""
    w, b, xs = _linear_operands(torch, nsets)
    keep, steps = [w, b], []
    for x in xs:
        keep.append(x)

        def gemm(x=x):
            torch.nn.functional.linear(x, w, b)     # result dropped: its block is reused by the next call
        steps.append([gemm])
    return steps, keep, 2 * 8192 * 3584 * 8192


def layer_linear(torch):
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import DistributedLinearAllGather
    world = SimWorld(8)
    P_y = world.partition(0).create_partition_inclusive(list(range(8))).create_cartesian_topology_partition([1, 1, 8])
    layer = DistributedLinearAllGather(P_y, 8192, 28672, dtype=torch.bfloat16)
    xs = [torch.randn(4, 2048, 8192, generator=torch.Generator().manual_seed(3004 + s)).to(torch.bfloat16).cuda()
          for s in range(4)]                                         # 4 x 128 MiB
    rec = time_layer(torch, layer, xs, calls=120, warm=20)           # as many steps as the kernel's own timing: the clock settles
    rec["module"] = "DistributedLinearAllGather([1,1,8], 8192, 28672, bf16).forward, no_grad, rank 0 of 8, x whole"
    return rec


def cpu_linear(budget_s=4.0):
    """The oracle's product (NumPy matmul on fp32 operands converted from the
    same bf16 bits beforehand, bias added) on 256 of config 4's 8192 rows."""
    import numpy as np
    from oracle import linear as o_lin
    rng = np.random.default_rng(1004)
    m = 256
    x = o_lin.bf16_bits_to_f32(o_lin.f32_to_bf16_bits(rng.standard_normal((m, 8192), dtype=np.float32)))
    w = o_lin.bf16_bits_to_f32(o_lin.f32_to_bf16_bits(0.02 * rng.standard_normal((3584, 8192), dtype=np.float32)))
    b = o_lin.bf16_bits_to_f32(o_lin.f32_to_bf16_bits(0.02 * rng.standard_normal(3584, dtype=np.float32)))
    n, dt = timed_cpu(lambda: o_lin.linear_values(x, w, b), budget_s)
    threads = 1
    try:
        from threadpoolctl import threadpool_info
        threads = max([int(p.get("num_threads", 1)) for p in threadpool_info() if p.get("user_api") == "blas"] or [1])
    except Exception:
        pass
    return {"value": 2.0 * m * 3584 * 8192 * n / dt / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"{n} products of 256 of config 4's 8192 rows (1/32 step), NumPy fp32 matmul (BLAS, {threads} threads), {dt:.1f} s"}


# ----------------------------------------------------------------------------
# configuration 5: halo
# ----------------------------------------------------------------------------

RANK0 = [[0, 0], [0, 0], [0, 1], [0, 1], [0, 1]]        # corner rank of 2x2x2: right-hand neighbours only
INTERIOR = [[0, 0], [0, 0], [1, 1], [1, 1], [1, 1]]     # interior rank of a partition at least 3 wide
PAD5 = [[0, 0], [0, 0], [1, 1], [1, 1], [1, 1]]


def _halo_sets(torch, nsets, widths, seed, padded_input=False):
    from distdl_amd import hip_ops
    plan = hip_ops.HaloPadPlan((1, 32, 128, 128, 128), PAD5, widths, widths)
    sets = []
    for s in range(nsets):
        gen = torch.Generator(device="cuda").manual_seed(seed + s)
        shape = plan.padded_shape if padded_input else (1, 32, 128, 128, 128)
        x = torch.randn(shape, generator=gen, device="cuda")
        ghosts, bulks = [], []
        for d in range(5):
            grow, brow = [], []
            for side in range(2):
                gs, bs = plan.slab_shape(d, side, "ghost"), plan.slab_shape(d, side, "bulk")
                grow.append(None if gs is None else torch.randn(gs, generator=gen, device="cuda"))
                brow.append(None if bs is None else torch.empty(bs, device="cuda"))
            ghosts.append(grow)
            bulks.append(brow)
        sets.append((x, ghosts, bulks))
    return plan, sets


def _slab_bytes(plan, kind):
    total = 0
    for d in range(5):
        for side in range(2):
            shape = plan.slab_shape(d, side, kind)
            if shape is not None:
                n = 4
                for v in shape:
                    n *= v
                total += n
    return total


def _build_halo_fused(torch, lib, _lib, nsets, widths, seed):
    plan, sets = _halo_sets(torch, nsets, widths, seed)
    keep, steps = [], []
    for x, ghosts, bulks in sets:
        out = torch.empty(plan.padded_shape, device="cuda")
        gptr = [None if g is None else g.data_ptr() for row in ghosts for g in row]
        bptr = [None if b is None else b.data_ptr() for row in bulks for b in row]
        args = (x.data_ptr(), out.data_ptr(), plan.shape_arr, 5, 4, plan.pad_arr, plan.recv_arr, plan.send_arr,
                _lib.ptr_array(gptr), _lib.ptr_array(bptr), _lib.DDL_HALO_AUTO)
        keep.append((x, out, ghosts, bulks, args))
        steps.append([_call(lib, _lib, "ddl_halo_pad_exchange", args)])
    work = 268435456 + 281216000 + _slab_bytes(plan, "ghost") + _slab_bytes(plan, "bulk")
    return steps, keep, work


def build_halo(torch, lib, _lib, nsets):
    """Config 5 (fused): rank 0 of a 2x2x2 split, [1,32,128^3] fp32 -> [1,32,130^3], 3 + 3 slabs."""
    steps, keep, work = _build_halo_fused(torch, lib, _lib, nsets, RANK0, 1005)
    assert work == 562531072
    return steps, keep, work


def build_halo_interior(torch, lib, _lib, nsets):
    """The same shard as an interior rank: 6 ghost + 6 bulk slabs in the same single pass."""
    return _build_halo_fused(torch, lib, _lib, nsets, INTERIOR, 1205)


def _build_halo_slabs(torch, lib, _lib, nsets, widths, seed):
    """Slab-only exchange on an existing padded tensor, in the reference's
    order: per exchanged dimension one pack launch (bulk slabs of both sides)
    and one unpack launch (ghost slabs of both sides)."""
    from oracle import halo as o_halo
    plan, sets = _halo_sets(torch, nsets, widths, seed, padded_input=True)
    slices = o_halo.slab_slices(plan.padded_shape, widths, widths)
    keep, steps = [], []
    launches = 0
    for xp, ghosts, bulks in sets:
        fns = []
        shape_arr, stride_arr = _lib.i64_array(xp.shape), _lib.i64_array(xp.stride())
        for d in range(5):
            lbs, lgs, rbs, rgs = slices[d]
            packs = [(sl, bulks[d][side]) for side, sl in ((0, lbs), (1, rbs)) if bulks[d][side] is not None]
            unpacks = [(sl, ghosts[d][side]) for side, sl in ((0, lgs), (1, rgs)) if ghosts[d][side] is not None]
            for name, boxes, extra in (("ddl_pack_boxes", packs, ()), ("ddl_unpack_boxes", unpacks, (0, 0))):
                if not boxes:
                    continue
                starts = _lib.i64_array([int(s.start) for sl, _ in boxes for s in sl])
                shapes = _lib.i64_array([int(s.stop - s.start) for sl, _ in boxes for s in sl])
                ptrs = _lib.ptr_array([b.data_ptr() for _, b in boxes])
                args = (xp.data_ptr(), shape_arr, stride_arr, 5, 4, len(boxes), starts, shapes, ptrs) + extra
                keep.append(args)
                fns.append(_call(lib, _lib, name, args))
        keep.append((xp, ghosts, bulks))
        launches = len(fns)
        steps.append(fns)
    work = 2 * (_slab_bytes(plan, "ghost") + _slab_bytes(plan, "bulk"))
    return steps, keep, work, launches


def build_halo_slabs(torch, lib, _lib, nsets):
    """Config 5, slab-only part: 3 bulk slabs packed, 3 ghost slabs unpacked (25 759 232 B in six launches)."""
    steps, keep, work, launches = _build_halo_slabs(torch, lib, _lib, nsets, RANK0, 1305)
    assert work == 25759232 and launches == 6, (work, launches)
    return steps, keep, work


def build_halo_slabs_interior(torch, lib, _lib, nsets):
    """Slab-only exchange of an interior rank: 6 + 6 slabs (51 122 176 B in six launches)."""
    steps, keep, work, launches = _build_halo_slabs(torch, lib, _lib, nsets, INTERIOR, 1405)
    assert work == 51122176 and launches == 6, (work, launches)
    return steps, keep, work


def layer_halo(torch):
    from distdl_amd.backends.stub_hip import SimWorld
    from distdl_amd.nn import DistributedConv3d
    world = SimWorld(8)
    P_x = world.partition(0).create_partition_inclusive(list(range(8))).create_cartesian_topology_partition([1, 1, 2, 2, 2])
    layer = DistributedConv3d(P_x, in_channels=32, out_channels=4, kernel_size=3, padding=1, bias=False)
    gen = torch.Generator(device="cuda").manual_seed(1005)
    xs = [torch.randn(1, 32, 128, 128, 128, generator=gen, device="cuda") for _ in range(3)]     # 3 x 256 MiB
    layer._distdl_forward_pre_hook(layer, (xs[0],))
    rec = time_layer(torch, layer.stage_input, xs, calls=48, warm=6)
    rec["module"] = "DistributedConv3d([1,1,2,2,2], kernel 3, padding 1).stage_input (pad + exchange + crop), no_grad, rank 0 of 8"
    return rec


def cpu_halo(budget_s=4.0):
    """The oracle's np.pad + per-dimension slab pack / ghost unpack on the full
    rank-0 shard of config 5."""
    import numpy as np
    from oracle import halo as o_halo
    rng = np.random.default_rng(1005)
    x = rng.standard_normal((1, 32, 128, 128, 128), dtype=np.float32)
    shape = [1, 32, 130, 130, 130]
    slices = o_halo.slab_slices(shape, RANK0, RANK0)
    ghosts = []
    for d in range(5):
        lbs, lgs, rbs, rgs = slices[d]
        ghosts.append([None, rng.standard_normal([s.stop - s.start for s in rgs], dtype=np.float32) if RANK0[d][1] else None])
    n, dt = timed_cpu(lambda: o_halo.pad_exchange_single(x, PAD5, RANK0, RANK0, ghosts), budget_s)
    return {"value": 562531072 * n / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{n} full steps of config 5 on rank 0 (3 + 3 slabs): np.pad, per dimension pack bulk / unpack ghosts, {dt:.1f} s"}


# ----------------------------------------------------------------------------
# backward (adjoint) workloads: the same shapes as the forward configurations
# ----------------------------------------------------------------------------

def build_layernorm_bwd(torch, lib, _lib, nsets, rows=16 * 512, cols=256, nparts=4):
    """Backward of config 1 on rank 0 as the layer runs it when every gradient
    is wanted: row sums + partial column sums in one launch, then (after the
    gather of the row sums) input gradient + final parameter sums in one launch.
    Algorithmic bytes: dy and x are read twice (once per launch), dx is written
    once: 5 x 8 388 608 B, plus the small vectors and the partial column sums."""
    keep, steps = [], []
    for s in range(nsets):
        gen = torch.Generator(device="cuda").manual_seed(4001 + s)
        x = torch.randn(rows, cols, generator=gen, device="cuda")
        dy = torch.randn(rows, cols, generator=gen, device="cuda")
        gamma = 1 + 0.1 * torch.randn(cols, generator=gen, device="cuda")
        mean = 0.01 * torch.randn(rows, generator=gen, device="cuda")
        rstd = 1 + 0.01 * torch.randn(rows, generator=gen, device="cuda")
        sums = torch.zeros(nparts, rows, 2, device="cuda")                # slot 0 is written by the kernel, the others seeded
        dx = torch.empty_like(x)
        dg, db = torch.empty(cols, device="cuda"), torch.empty(cols, device="cuda")
        work = torch.empty(2 * 256 * cols, device="cuda")
        keep.append((x, dy, gamma, mean, rstd, sums, dx, dg, db, work))
        a1 = (dy.data_ptr(), x.data_ptr(), rows, cols, cols, cols, mean.data_ptr(), rstd.data_ptr(), gamma.data_ptr(),
              sums.data_ptr(), work.data_ptr(), work.numel())
        a2 = (dy.data_ptr(), x.data_ptr(), rows, cols, cols, cols, mean.data_ptr(), rstd.data_ptr(), gamma.data_ptr(),
              sums.data_ptr(), nparts, 1.0 / (nparts * cols), dx.data_ptr(), cols, work.data_ptr(), work.numel(), dg.data_ptr(),
              db.data_ptr())
        steps.append([_call(lib, _lib, "ddl_ln_bwd_partial_params_f32", a1),
                      _call(lib, _lib, "ddl_ln_bwd_input_params_f32", a2)])
    return steps, keep, 5 * rows * cols * 4 + 2 * (2 * rows * 4) + (nparts + 1) * rows * 2 * 4 + 3 * cols * 4 + 2 * (2 * 256 * cols * 4)


def build_layernorm_local_bwd_two_passes(torch, lib, _lib, nsets):
    """The two-launch backward on rows held whole ([8192, 1024] fp32), beside
    layernorm_local_bwd: dy and x read twice."""
    return build_layernorm_bwd(torch, lib, _lib, nsets, 16 * 512, 1024, 1)


def _build_layernorm_bwd_one_pass(rows, cols, nparts):
    def build(torch, lib, _lib, nsets):
        """LayerNorm backward with one pass over dy and x (ddl_ln_bwd_one_pass:
        row sums, dx and partial column sums in one launch, the final parameter
        sums in a second, small one): rows held whole (nparts 1) or the other
        workers' row sums seeded.  `work` is what is moved: dy and x read once,
        dx written, plus the small vectors and the partial column sums."""
        keep, steps = [], []
        for s in range(nsets):
            gen = torch.Generator(device="cuda").manual_seed(4101 + s)
            x = torch.randn(rows, cols, generator=gen, device="cuda")
            dy = torch.randn(rows, cols, generator=gen, device="cuda")
            gamma = 1 + 0.1 * torch.randn(cols, generator=gen, device="cuda")
            mean = 0.01 * torch.randn(rows, generator=gen, device="cuda")
            rstd = 1 + 0.01 * torch.randn(rows, generator=gen, device="cuda")
            sums = torch.zeros(nparts, rows, 2, device="cuda")
            dx = torch.empty_like(x)
            dg, db = torch.empty(cols, device="cuda"), torch.empty(cols, device="cuda")
            work = torch.empty(2 * 256 * cols, device="cuda")
            keep.append((x, dy, gamma, mean, rstd, sums, dx, dg, db, work))
            args = (dy.data_ptr(), x.data_ptr(), _lib.DDL_DT_F32, rows, cols, cols, cols, mean.data_ptr(), rstd.data_ptr(),
                    gamma.data_ptr(), sums.data_ptr(), nparts, 0, 1.0 / (nparts * cols), dx.data_ptr(), cols, work.data_ptr(),
                    work.numel(), dg.data_ptr(), db.data_ptr())
            steps.append([_call(lib, _lib, "ddl_ln_bwd_one_pass", args)])
        return steps, keep, 3 * rows * cols * 4 + 2 * rows * 4 + (nparts + 1) * rows * 2 * 4 + 3 * cols * 4 + 2 * (2 * 256 * cols * 4)
    return build


def build_embedding_bwd(torch, lib, _lib, nsets):
    """Backward of config 3 on rank 0: gradient of the [16032, 4096] bf16 shard
    from dy [32, 4096, 4096].  Algorithmic bytes: the dy rows of the hit tokens,
    the ids (read twice), the whole gradient written once."""
    keep, steps, nbytes = [], [], []
    gen = torch.Generator(device="cuda").manual_seed(5003)
    dy = torch.randn(32, 4096, 4096, generator=gen, device="cuda").to(torch.bfloat16)
    keep.append(dy)
    for s in range(nsets):
        g = torch.Generator().manual_seed(2003 + s)
        ids = torch.randint(0, 128256, (32, 4096), generator=g)
        n_hit = int((ids < 16032).sum())
        nbytes.append(n_hit * 8192 + 2 * ids.numel() * 8 + 16032 * 4096 * 2)
        ids = ids.cuda()
        dw = torch.empty(16032, 4096, dtype=torch.bfloat16, device="cuda")
        work = torch.empty(3 * 16032 + 1 + ids.numel(), dtype=torch.int32, device="cuda")
        keep.append((ids, dw, work))
        args = (dy.data_ptr(), _lib.DDL_DT_BF16, 4096, 4096, ids.data_ptr(), 1, ids.numel(), 0, 16032, -1, 0, dw.data_ptr(),
                4096, work.data_ptr(), work.numel())
        steps.append([_call(lib, _lib, "ddl_embedding_backward", args)])
    return steps, keep, sum(nbytes) / len(nbytes)


def _build_linear_bwd(in_place):
    def build(torch, lib, _lib, nsets):
        M, N, K = 8192, 3584, 8192
        gen = torch.Generator(device="cuda").manual_seed(6004)
        w = (0.02 * torch.randn(N, K, generator=gen, device="cuda")).to(torch.bfloat16)
        work = torch.empty(64 * N, device="cuda")
        keep, steps = [w, work], []
        if not in_place:
            w_t = torch.empty(K, N, dtype=torch.bfloat16, device="cuda")
            dy_t = torch.empty(N, M, dtype=torch.bfloat16, device="cuda")
            x_t = torch.empty(K, M, dtype=torch.bfloat16, device="cuda")
            keep += [w_t, dy_t, x_t]
        bf16 = _lib.DDL_DT_BF16
        for s in range(nsets):
            x = torch.randn(M, K, generator=gen, device="cuda").to(torch.bfloat16)
            dy = torch.randn(M, N, generator=gen, device="cuda").to(torch.bfloat16)
            dx = torch.empty(M, K, dtype=torch.bfloat16, device="cuda")
            dw = torch.empty(N, K, dtype=torch.bfloat16, device="cuda")
            db = torch.empty(N, dtype=torch.bfloat16, device="cuda")
            keep.append((x, dy, dx, dw, db))
            if in_place:
                products = [
                    _call(lib, _lib, "ddl_gemm", (dy.data_ptr(), N, 1, w.data_ptr(), 1, K, None, dx.data_ptr(), bf16, K, M, K, N)),
                    _call(lib, _lib, "ddl_gemm", (dy.data_ptr(), 1, N, x.data_ptr(), 1, K, None, dw.data_ptr(), bf16, K, N, K, M)),
                ]
            else:
                products = [
                    _call(lib, _lib, "ddl_transpose_2d", (w.data_ptr(), w_t.data_ptr(), N, K, K, N, 2)),
                    _call(lib, _lib, "ddl_linear_bf16", (dy.data_ptr(), w_t.data_ptr(), None, dx.data_ptr(), M, K, N, N, N, K)),
                    _call(lib, _lib, "ddl_transpose_2d", (dy.data_ptr(), dy_t.data_ptr(), M, N, N, M, 2)),
                    _call(lib, _lib, "ddl_transpose_2d", (x.data_ptr(), x_t.data_ptr(), M, K, K, M, 2)),
                    _call(lib, _lib, "ddl_linear_bf16", (dy_t.data_ptr(), x_t.data_ptr(), None, dw.data_ptr(), N, K, M, M, M, K)),
                ]
            steps.append(products + [
                _call(lib, _lib, "ddl_colsum_bf16", (dy.data_ptr(), M, N, N, db.data_ptr(), work.data_ptr(), work.numel())),
            ])
        return steps, keep, 2 * 2 * M * N * K
    build.__doc__ = ("Backward of config 4 on rank 0: dx = dy w and dw = dy^T x through the shard GEMM, "
                     + ("which reads w, dy and x where they lie (ddl_gemm)" if in_place else
                        "on transposed copies of w, dy and x (the three transposes are part of the step; what shapes "
                        "that ddl_gemm cannot read in place fall back to)")
                     + ", db = column sums of dy.  Work: 2 x 2 M N K flop.")
    return build


# ----------------------------------------------------------------------------
# local re-layouts of AllGather / ReduceScatter at configuration 4's activation
# ----------------------------------------------------------------------------

def build_all_gather_relayout(torch, lib, _lib, nsets):
    """The local half of the all-gather in front of configuration 4's GEMM
    (DistributedLinearAllGather with the features of x sharded over 8 workers):
    eight received pieces [4,2048,1024] bf16 unpacked into x [4,2048,8192], one
    launch.  Bytes: every element read once and written once."""
    keep, steps = [], []
    starts = _lib.i64_array([v for q in range(8) for v in (0, 0, 1024 * q)])
    shapes = _lib.i64_array([4, 2048, 1024] * 8)
    for s in range(nsets):
        gen = torch.Generator(device="cuda").manual_seed(8004 + s)
        parts = [torch.randn(4, 2048, 1024, generator=gen, device="cuda").to(torch.bfloat16) for _ in range(8)]
        x = torch.empty(4, 2048, 8192, dtype=torch.bfloat16, device="cuda")
        args = (x.data_ptr(), _lib.i64_array(x.shape), _lib.i64_array(x.stride()), 3, 2, 8, starts, shapes,
                _lib.ptr_array([p.data_ptr() for p in parts]), 0, 0)
        keep.append((parts, x, args))
        steps.append([_call(lib, _lib, "ddl_unpack_boxes", args)])
    keep.append((starts, shapes))
    return steps, keep, 2 * 4 * 2048 * 8192 * 2


def build_reduce_scatter_relayout(torch, lib, _lib, nsets):
    """The local half of a reduce-scatter over 8 workers at the same shape:
    worker 3's slab [4,2048,1024] of the sum of eight full tensors [4,2048,8192]
    bf16 (strided reads where the tensors lie), one launch of the sum kernel.
    Bytes: eight slabs read, one written."""
    keep, steps = [], []
    for s in range(nsets):
        gen = torch.Generator(device="cuda").manual_seed(8104 + s)
        fulls = [torch.randn(4, 2048, 8192, generator=gen, device="cuda").to(torch.bfloat16) for _ in range(8)]
        out = torch.empty(4, 2048, 1024, dtype=torch.bfloat16, device="cuda")
        box = _lib.ddl_box_t()
        box.ndim = 3
        for d, n in enumerate((4, 2048, 1024)):
            box.shape[d], box.src_stride[d], box.dst_stride[d] = n, fulls[0].stride(d), out.stride(d)
        box.dst = out.data_ptr()
        srcs = _lib.ptr_array([f.data_ptr() + 3 * 1024 * 2 for f in fulls])
        args = (ctypes.byref(box), srcs, 8, 2, _lib.DDL_DT_BF16, 1.0)
        keep.append((fulls, out, box, srcs, args))
        steps.append([_call(lib, _lib, "ddl_sum_boxes", args)])
    return steps, keep, 9 * 4 * 2048 * 1024 * 2


def cpu_all_gather_relayout(budget_s=3.0):
    """The oracle's restatement of the reference's gather + rearrange on the
    eight pieces of the workload, bf16 moved as int16 as the reference moves it."""
    import numpy as np
    from oracle import relayout as o_rl
    rng = np.random.default_rng(8004)
    parts = [rng.integers(-2 ** 15, 2 ** 15, size=(4, 2048, 1024), dtype=np.int16) for _ in range(8)]
    n, dt = timed_cpu(lambda: o_rl.all_gather(parts, 2), budget_s)
    return {"value": 2 * 4 * 2048 * 8192 * 2 * n / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{n} gathers of eight [4,2048,1024] int16 pieces into [4,2048,8192] (np.stack, np.concatenate), {dt:.1f} s"}


def cpu_reduce_scatter_relayout(budget_s=3.0):
    """The oracle's reduce-scatter over all eight workers on a sixteenth of the
    rows, in float32 (NumPy has no bfloat16; the reference would add the int16
    views): eight slabs of the sum of eight tensors, i.e. eight workers' shares
    per run, counted as such."""
    import numpy as np
    from oracle import relayout as o_rl
    rng = np.random.default_rng(8104)
    fulls = [rng.standard_normal((4, 128, 8192), dtype=np.float32) for _ in range(8)]
    n, dt = timed_cpu(lambda: o_rl.reduce_scatter(fulls, 2), budget_s)
    work = 8 * 9 * 4 * 128 * 1024 * 4            # per worker: eight slabs read, one written
    return {"value": work * n / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{n} reduce-scatters of eight [4,128,8192] float32 tensors over 8 simulated workers (split, pad-free "
                      f"flatten, rank-order sum), {dt:.1f} s"}


# ----------------------------------------------------------------------------
# measurement aids
# ----------------------------------------------------------------------------

def build_calib(torch, lib, _lib, nsets):
    """Counter calibration: a plain contiguous device-to-device copy of 64 MiB
    (torch's own copy kernel), so that FETCH_SIZE / WRITE_SIZE readings of the
    kernels above can be scaled by what the same counters read for a known
    amount of traffic."""
    keep, steps = [], []
    for s in range(nsets):
        a = torch.empty(64 << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
        b = torch.empty_like(a)
        keep.append((a, b))

        def copy(a=a, b=b):
            b.copy_(a)      # torch's current stream is the one STREAM[0] is bound to
        steps.append([copy])
    return steps, keep, 2 * (64 << 20)


_PROBES = [None]


def probes_lib():
    """The benchmark's own helper library (an empty kernel and an MFMA-only
    kernel; distdl_amd/csrc/bench_probes.hip), not part of the product library."""
    if _PROBES[0] is None:
        path = os.path.join(ROOT, "distdl_amd", "libdistdl_bench_probes.so")
        if not os.path.exists(path):
            raise SystemExit(f"bench.py: {path} is not built; run `make -C distdl_amd/csrc`")
        probes = ctypes.CDLL(path)
        probes.bench_probe_launch.restype = ctypes.c_int
        probes.bench_probe_launch.argtypes = [ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
        probes.bench_probe_mfma.restype = ctypes.c_int
        probes.bench_probe_mfma.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_int64,
                                            ctypes.POINTER(ctypes.c_int64), ctypes.c_void_p]
        _PROBES[0] = probes
    return _PROBES[0]


def _probe_call(name, args):
    def fn(a=args, f=getattr(probes_lib(), name), n=name):
        rc = f(*a, STREAM[0])
        if rc:
            raise RuntimeError(f"{n} failed with code {rc}")
    return fn


def build_launch_floor(torch, lib, _lib, nsets):
    """A kernel that does nothing, launched with the grid of config 1's
    LayerNorm kernels (2048 workgroups of 256 threads) and replayed from the
    same kind of graph: the time a launch costs on its own.  `work` is zero
    bytes; only the time per launch means anything."""
    steps = [[_probe_call("bench_probe_launch", (2048, 256)), _probe_call("bench_probe_launch", (2048, 256))]
             for _ in range(nsets)]
    return steps, [], 0


def _build_mfma_probe(instruction, random):
    def build(torch, lib, _lib, nsets):
        """Nothing but MFMAs on register operands (bench_probe_mfma): what the matrix
        cores of this machine sustain with this instruction on this kind of data,
        the ceiling the shard GEMM's figure is read against."""
        sink = torch.empty(512 * 256, device="cuda")
        flop = ctypes.c_int64(0)
        iters = 4000
        args = (instruction, random, iters, sink.data_ptr(), sink.numel(), ctypes.byref(flop))
        _probe_call("bench_probe_mfma", args)()
        torch.cuda.synchronize()
        return [[_probe_call("bench_probe_mfma", args)] for _ in range(nsets)], [sink, flop], int(flop.value)
    return build


# name -> (builder, buffer sets, launches per step, bound, rule for combining the traffic figures of a step's kernels,
#          layer timer, cpu baseline, BASELINE.json configuration number)
WORKLOADS = {
    "repartition": (build_repartition, 8, 2, "hbm", "mean", layer_repartition, cpu_repartition, 2),
    "repartition_pack": (_build_repartition_half(0), 8, 1, "hbm", None, None, None, None),
    "repartition_unpack": (_build_repartition_half(1), 8, 1, "hbm", None, None, None, None),
    "layernorm": (build_layernorm, 64, 2, "hbm", "mean", layer_layernorm, cpu_layernorm, 1),
    "layernorm_joined": (build_layernorm_joined, 64, 1, "hbm", None, None, None, None),
    "layernorm_long": (build_layernorm_long, 3, 2, "hbm", None, None, None, None),
    "layernorm_wide": (build_layernorm_wide, 4, 2, "hbm", None, None, None, None),
    "layernorm_local": (build_layernorm_local, 16, 1, "hbm", None, None, None, None),
    "embedding": (build_embedding, 4, 1, "hbm", "sum", layer_embedding, cpu_embedding, 3),
    "linear": (build_linear, 4, 1, "mfma", "sum", layer_linear, cpu_linear, 4),
    "halo": (build_halo, 4, 1, "hbm", "sum", layer_halo, cpu_halo, 5),
    "halo_interior": (build_halo_interior, 4, 1, "hbm", None, None, None, None),
    "halo_slabs": (build_halo_slabs, 8, 6, "hbm", None, None, None, None),
    "halo_slabs_interior": (build_halo_slabs_interior, 8, 6, "hbm", None, None, None, None),
    "all_gather_relayout": (build_all_gather_relayout, 3, 1, "hbm", "sum", None, cpu_all_gather_relayout, None),
    "reduce_scatter_relayout": (build_reduce_scatter_relayout, 2, 1, "hbm", "sum", None, cpu_reduce_scatter_relayout, None),
    "layernorm_bwd": (build_layernorm_bwd, 32, 2, "hbm", None, None, None, None),
    "layernorm_bwd_one_pass": (_build_layernorm_bwd_one_pass(16 * 512, 256, 4), 32, 2, "hbm", None, None, None, None),
    "layernorm_local_bwd": (_build_layernorm_bwd_one_pass(16 * 512, 1024, 1), 8, 2, "hbm", None, None, None, None),
    "embedding_bwd": (build_embedding_bwd, 4, 1, "hbm", None, None, None, None),
    "linear_bwd": (_build_linear_bwd(True), 2, 1, "mfma", None, None, None, None),
    "linear_f32": (_build_linear_f32(False), 2, 1, "mfma_f32", None, None, None, None),
    "linear_f32_bwd": (build_linear_f32_bwd, 2, 1, "mfma_f32", None, None, None, None),
    "launch_floor": (build_launch_floor, 8, 2, "hbm", None, None, None, None),
    "mfma_32x32x16_constant": (_build_mfma_probe(0, 0), 1, 1, "mfma", None, None, None, None),
    "mfma_32x32x16_random": (_build_mfma_probe(0, 1), 1, 1, "mfma", None, None, None, None),
    "mfma_16x16x32_constant": (_build_mfma_probe(1, 0), 1, 1, "mfma", None, None, None, None),
    "mfma_16x16x32_random": (_build_mfma_probe(1, 1), 1, 1, "mfma", None, None, None, None),
    # only with --only:
    "layernorm_local_bwd_two_passes": (build_layernorm_local_bwd_two_passes, 8, 2, "hbm", None, None, None, None),
    "linear_library": (build_linear_library, 4, 1, "mfma", None, None, None, None),
    "linear_bwd_transposed": (_build_linear_bwd(False), 2, 1, "mfma", None, None, None, None),
    "linear_f32_library": (_build_linear_f32(True), 2, 1, "mfma_f32", None, None, None, None),
    "calib": (build_calib, 4, 1, "hbm", None, None, None, None),
}
# What a run without --only / --all measures: the five BASELINE configurations and the secondaries read next to them.
DEFAULT_WORKLOADS = ("repartition", "layernorm", "layernorm_joined", "embedding", "linear", "halo", "halo_interior",
                     "all_gather_relayout", "reduce_scatter_relayout", "launch_floor")
# Never part of --all (comparison figures through other libraries, counter calibration): only with --only.
ONLY_ON_REQUEST = ("layernorm_local_bwd_two_passes", "linear_library", "linear_bwd_transposed", "linear_f32_library", "calib")


def cpu_host():
    import torch
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"nproc": os.cpu_count(), "affinity": len(os.sched_getaffinity(0)), "torch_threads": torch.get_num_threads(),
            "cpu_model": model, "launch": "one process standing in for rank 0 (no mpirun: mpi4py is not installed); "
                                          "cpu_baseline.all_ranks: the headline's eight ranks as eight processes at once"}


def main():
    args = parse_args()
    if args.cpu_worker:
        cpu_worker(args.cpu_worker)
        return
    if args.gpus != 1:
        sys.stderr.write("bench.py measures one rank's share on ONE GPU; --gpus N with N > 1 is not part of this build "
                         "(no collectives, no cross-GPU sharding).\n")
        sys.exit(2)

    import torch
    import distdl_amd  # noqa: F401
    from distdl_amd import _lib
    if not torch.cuda.is_available():
        sys.stderr.write("bench.py needs a GPU\n")
        sys.exit(2)
    torch.cuda.set_device(0)
    lib = _lib.load()
    use_graph = not args.no_graph

    if args.only:
        names = [n.strip() for n in args.only.split(",")]
    elif args.all:
        names = [n for n in WORKLOADS if n not in ONLY_ON_REQUEST]
    else:
        names = list(DEFAULT_WORKLOADS)
    for n in names:
        if n not in WORKLOADS:
            raise SystemExit(f"bench.py: unknown workload {n!r}; choose from {', '.join(WORKLOADS)}")
    head_name = "repartition" if "repartition" in names else names[0]
    results = {}
    for name in names:
        build, nsets, launches, bound, combine, layer_fn, cpu_fn, config = WORKLOADS[name]
        step_fns, keep, work = build(torch, lib, _lib, nsets)
        if name == head_name:
            steps, warm = args.steps, args.warmup
        else:
            steps, warm = max(args.steps, MIN_SECONDARY_STEPS), max(args.warmup, MIN_SECONDARY_WARMUP)
        m = measure(torch, name, step_fns, launches, steps, warm, use_graph)
        per_launch = work / launches
        if bound == "hbm":
            achieved, peak, unit = per_launch / m["launch_s"] / 1e9, HBM_PEAK_GBS, "GB/s"
            value = work * m["steps"] / m["wall_s"] / 1e9
        else:
            peak = MFMA_F32_PEAK_TFLOPS if bound == "mfma_f32" else MFMA_BF16_PEAK_TFLOPS
            achieved, unit, bound = per_launch / m["launch_s"] / 1e12, "TFLOP/s", "mfma"
            value = work * m["steps"] / m["wall_s"] / 1e12
        traffic = profile_traffic(name, combine) if combine else None
        results[name] = {
            "value": value, "unit": unit, "steps": m["steps"], "warmup": warm, "ms_per_step": 1e3 * m["wall_s"] / m["steps"],
            "mode": m["mode"], "us_per_step_by_mode": m["us_per_step_by_mode"], "work_per_step": work, "launches_per_step": launches, "us_per_launch": 1e6 * m["launch_s"],
            "baseline_config": config,
            "roofline": {"bound": bound, "achieved": achieved, "peak": peak, "unit": unit, "frac": achieved / peak,
                         "traffic": traffic},
        }
        del step_fns, keep
        torch.cuda.empty_cache()
        if layer_fn is not None and not args.skip_layers:
            rec = layer_fn(torch)
            rec["kernel_us"] = 1e6 * m["launch_s"] * launches
            results[name]["layer"] = rec
            torch.cuda.empty_cache()
        if cpu_fn is not None and not args.skip_cpu:
            results[name]["cpu_baseline"] = cpu_fn()

    # Config 1 is small enough that what a launch costs by itself is a large part of its time: next to the plain
    # fraction, the one computed on (time of the step's launches - time of as many empty launches of the same grid).
    if "launch_floor" in results:
        floor_us = results["launch_floor"]["us_per_launch"]
        for name in ("layernorm", "layernorm_joined"):
            if name in results:
                r = results[name]
                us = r["us_per_launch"] * r["launches_per_step"]
                above = us - floor_us * r["launches_per_step"]
                r["roofline"]["launch_floor_us"] = floor_us
                if above > 0:
                    r["roofline"]["frac_above_launch_floor"] = r["work_per_step"] / (above * 1e-6) / 1e9 / HBM_PEAK_GBS
    if "layernorm_joined" in results:
        # The same step counted with config 1's algorithmic bytes (x read by both halves): the path the layer takes for
        # config 1 under the solo transport, where the peers' statistics are in memory beforehand.
        r = results["layernorm_joined"]
        r["roofline"]["frac_of_config1_bytes"] = 25298944 / (r["us_per_launch"] * 1e-6) / 1e9 / HBM_PEAK_GBS

    head = results[head_name]
    # One entry per workload, small enough to survive in a truncated record: fraction of the roofline, time of one
    # step's launches by HIP events, throughput by wall clock.
    table = {}
    for name, r in results.items():
        key = f"cfg{r['baseline_config']}_{name}" if r["baseline_config"] else name
        table[key] = {"frac": r["roofline"]["frac"], "us": r["us_per_launch"] * r["launches_per_step"], "value": r["value"],
                      "unit": r["unit"], "ms_per_step": r["ms_per_step"]}
        for extra in ("frac_above_launch_floor", "frac_of_config1_bytes"):
            if extra in r["roofline"]:
                table[key][extra] = r["roofline"][extra]
        if "layer" in r:
            table[key]["layer_us"] = r["layer"]["us"]
    roofline = dict(head["roofline"])
    roofline["traffic_source"] = "profiles/<workload>_hbm_traffic_pmc.txt: rocprofv3 --pmc runs of the same workloads, not this run"
    roofline["configs"] = table
    line = {
        "metric": "Repartition pack+unpack GB/s (rank 0, bf16 [8,4096,8192], P_x=[1,8,1] -> P_y=[1,1,8])"
        if head_name == "repartition" else head_name,
        "value": head["value"], "unit": head["unit"], "n_gpus": 1, "steps": head["steps"], "warmup": head["warmup"],
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u16" if head_name == "repartition" else "mixed", "data": "synthetic",
        "config": {"workload": "BASELINE.json configs[1]: Repartition pack/unpack bf16, rank 0 of 8, "
                               "pack [8,512,8192] -> 8x[8,512,1024], unpack 8x[8,512,1024] -> [8,4096,1024]"
                   if head_name == "repartition" else head_name,
                   "launch_mode": head["mode"], "buffer_sets": WORKLOADS[head_name][1],
                   "box_lists": "distdl_amd.nn.Repartition set-up (rank 0 of 8), asserted equal to the oracle's plan"},
        "roofline": roofline,
    }
    if "cpu_baseline" in head:
        cpu = dict(head["cpu_baseline"])
        cpu["configs"] = {(f"cfg{r['baseline_config']}_{name}" if r["baseline_config"] else name):
                          {k: r["cpu_baseline"][k] for k in ("value", "unit", "cores")}
                          for name, r in results.items() if "cpu_baseline" in r}
        line["cpu_baseline"] = cpu
    if not args.skip_cpu:
        line["cpu_host"] = cpu_host()
    line["workloads"] = results
    print(json.dumps(compact(line)))


def compact(obj):
    """Floats to five significant digits: the line stays short enough to be kept whole."""
    if isinstance(obj, float):
        return float(f"{obj:.5g}")
    if isinstance(obj, dict):
        return {k: compact(v) for k, v in obj.items()}
    if isinstance(obj, (list, tuple)):
        return [compact(v) for v in obj]
    return obj


if __name__ == "__main__":
    main()

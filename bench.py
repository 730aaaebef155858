"""Benchmark of the per-rank hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--skip-cpu] [--only NAME]

Headline workload (BASELINE.json configs[1]): Repartition pack + unpack of one
rank, bf16 global tensor [8,4096,8192] moved from P_x=[1,8,1] to P_y=[1,1,8].
One step = one pack launch (the [8,512,8192] shard into eight [8,512,1024]
boxes) + one unpack launch (eight seeded boxes into the [8,4096,1024] output
shard) = 268 435 456 algorithmic bytes.  Inputs are resident in HBM before the
timed region; the step rotates over several buffer sets so that the 256 MB
last-level cache cannot hold the working set.  The other hot-path kernels
(LayerNorm, Embedding, Linear GEMM, fused halo staging) are measured the same
way and reported under "workloads" of the same JSON line.

Timing: the launches of the timed region are captured once into a HIP graph
(no host work between kernels) and replayed; wall clock with a device
synchronisation on both sides gives ms_per_step, HIP events on the launch
stream give the per-launch kernel duration used for the roofline.  If graph
capture is unavailable the same launches are issued directly on the stream.
"""

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published

# HBM bytes per launch (read + write) from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs of these same workloads, each counter scaled by what it reads
# for a plain 64 MiB device copy (FETCH_SIZE x1.9993, WRITE_SIZE x1.0000); the
# summaries are profiles/*_hbm_traffic_pmc.txt.  layernorm is the mean of its two
# kernels (stats 8 482 132 B, normalize 17 875 667 B), like its launch time;
# linear is the sum of the two launches of a step (256-wide tiles 436 344 160 B,
# 192-wide tiles 398 065 226 B).
MEASURED_TRAFFIC_BYTES = {
    "repartition": 134414634,
    "layernorm": 13178900,
    "embedding": 1210721771,
    "linear": 834409386,
    "halo": 568008812,
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--skip-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default=None, help="run only these workloads, comma-separated (repartition, layernorm, layernorm_long, embedding, linear, halo, layernorm_bwd, embedding_bwd, linear_bwd, calib)")
    ap.add_argument("--no-graph", action="store_true", help="launch on the stream instead of replaying a HIP graph")
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

    def run(self, steps):
        """Runs exactly `steps` steps: whole passes over the buffer sets (graph
        replays when a graph was captured) and the remaining steps launched on
        the stream.  Returns (steps, wall seconds, event seconds)."""
        torch = self.torch
        nsets = len(self.step_fns)
        passes, rest = divmod(steps, nsets)
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
        for fns in self.step_fns[:rest]:
            for fn in fns:
                fn()
        e1.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        return steps, t1 - t0, e0.elapsed_time(e1) * 1e-3


def measure(torch, name, step_fns, launches_per_step, steps, warmup, use_graph):
    timed = Timed(torch, step_fns, use_graph)
    timed.prepare()
    if warmup > 0:
        timed.run(warmup)
    n, wall, ev = timed.run(steps)
    return {"name": name, "steps": n, "wall_s": wall, "event_s": ev, "mode": timed.mode,
            "launch_s": ev / (n * launches_per_step)}


# ----------------------------------------------------------------------------
# workloads
# ----------------------------------------------------------------------------

def build_repartition(torch, lib, _lib, nsets):
    """Config 2.  Returns (step closures per set, bytes per step, description)."""
    from oracle import repartition as o_rep
    send, recv, _, _ = o_rep.plan([8, 4096, 8192], [1, 8, 1], [1, 1, 8])
    send0 = [sl for sl, sh, p in send[0]]
    recv0 = [sl for sl, sh, p in recv[0]]
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

        def pack(a=pack_args):
            rc = lib.ddl_pack_boxes(*a, STREAM[0])
            if rc:
                _lib.check(rc, "ddl_pack_boxes")

        def unpack(a=unpack_args):
            rc = lib.ddl_unpack_boxes(*a, STREAM[0])
            if rc:
                _lib.check(rc, "ddl_unpack_boxes")
        steps.append([pack, unpack])
    return steps, keep, 268435456


def build_layernorm(torch, lib, _lib, nsets):
    """Config 1: rank 0's [16,512,256] fp32 shard; stats + normalize."""
    import numpy as np
    from oracle import layernorm as o_ln
    rows, cols = 16 * 512, 256
    keep, steps = [], []
    part_cols = _lib.i64_array([256] * 4)
    for s in range(nsets):
        gen = torch.Generator().manual_seed(1001 + s)
        xg = torch.randn(16, 512, 1024, generator=gen)
        gamma = (1 + 0.1 * torch.randn(1024, generator=gen))[:256].contiguous().cuda()
        beta = (0.1 * torch.randn(1024, generator=gen))[:256].contiguous().cuda()
        x = xg[..., :256].contiguous().cuda()
        gathered = torch.empty(4, rows, 2, device="cuda")
        for p in range(1, 4):   # peers' partial statistics: seeded, computed on the CPU from the same global x
            gathered[p] = torch.from_numpy(o_ln.partial_stats(xg[..., 256 * p:256 * (p + 1)].numpy()).astype(np.float32))
        y = torch.empty_like(x)
        stats_args = (x.data_ptr(), rows, cols, cols, gathered.data_ptr())      # own partials land in slot 0
        norm_args = (x.data_ptr(), rows, cols, cols, gathered.data_ptr(), 4, part_cols, gamma.data_ptr(),
                     beta.data_ptr(), 1e-5, y.data_ptr(), cols, None, None)
        keep.append((x, gamma, beta, gathered, y, stats_args, norm_args))

        def stats(a=stats_args):
            rc = lib.ddl_ln_partial_stats_f32(*a, STREAM[0])
            if rc:
                _lib.check(rc, "ddl_ln_partial_stats_f32")

        def norm(a=norm_args):
            rc = lib.ddl_ln_normalize_affine_f32(*a, STREAM[0])
            if rc:
                _lib.check(rc, "ddl_ln_normalize_affine_f32")
        steps.append([stats, norm])
    return steps, keep, 25298944


def build_layernorm_long(torch, lib, _lib, nsets):
    """The kernels of config 1 on 32 times its rows ([262144, 256] fp32, 268 MB):
    the streaming rate of the same code once launch ramp and memory latency no
    longer dominate.  Not a BASELINE configuration; reported next to config 1."""
    rows, cols = 32 * 16 * 512, 256
    keep, steps = [], []
    part_cols = _lib.i64_array([256] * 4)
    for s in range(nsets):
        gen = torch.Generator(device="cuda").manual_seed(2001 + s)
        x = torch.randn(rows, cols, generator=gen, device="cuda")
        gamma = 1 + 0.1 * torch.randn(cols, generator=gen, device="cuda")
        beta = 0.1 * torch.randn(cols, generator=gen, device="cuda")
        gathered = torch.zeros(4, rows, 2, device="cuda")
        gathered[1:, :, 1] = 256.0                                   # peers: mean 0, M2 = n (unit variance)
        y = torch.empty_like(x)
        stats_args = (x.data_ptr(), rows, cols, cols, gathered.data_ptr())
        norm_args = (x.data_ptr(), rows, cols, cols, gathered.data_ptr(), 4, part_cols, gamma.data_ptr(),
                     beta.data_ptr(), 1e-5, y.data_ptr(), cols, None, None)
        keep.append((x, gamma, beta, gathered, y, stats_args, norm_args))

        def stats(a=stats_args):
            rc = lib.ddl_ln_partial_stats_f32(*a, STREAM[0])
            if rc:
                _lib.check(rc, "ddl_ln_partial_stats_f32")

        def norm(a=norm_args):
            rc = lib.ddl_ln_normalize_affine_f32(*a, STREAM[0])
            if rc:
                _lib.check(rc, "ddl_ln_normalize_affine_f32")
        steps.append([stats, norm])
    return steps, keep, 32 * 25298944 - 31 * 2 * 256 * 4


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

        def gather(a=args):
            rc = lib.ddl_embedding_gather(*a, STREAM[0])
            if rc:
                _lib.check(rc, "ddl_embedding_gather")
        steps.append([gather])
    return steps, keep, sum(nbytes) / len(nbytes)


def build_linear(torch, lib, _lib, nsets):
    """Config 4: M=8192 N=3584 K=8192 bf16, fp32 accumulate, bias."""
    gen = torch.Generator().manual_seed(1004)
    w = (0.02 * torch.randn(3584, 8192, generator=gen)).to(torch.bfloat16).cuda()
    b = (0.02 * torch.randn(3584, generator=gen)).to(torch.bfloat16).cuda()
    keep, steps = [w, b], []
    for s in range(nsets):
        gen = torch.Generator().manual_seed(3004 + s)
        x = torch.randn(4, 2048, 8192, generator=gen).to(torch.bfloat16).cuda()
        y = torch.empty(4, 2048, 3584, dtype=torch.bfloat16, device="cuda")
        args = (x.data_ptr(), w.data_ptr(), b.data_ptr(), y.data_ptr(), 8192, 3584, 8192, 8192, 8192, 3584)
        keep.append((x, y, args))

        def gemm(a=args):
            rc = lib.ddl_linear_bf16(*a, STREAM[0])
            if rc:
                _lib.check(rc, "ddl_linear_bf16")
        steps.append([gemm])
    return steps, keep, 2 * 8192 * 3584 * 8192


def build_halo(torch, lib, _lib, nsets):
    """Config 5 (fused): rank 0 of a 2x2x2 split, [1,32,128^3] fp32 -> [1,32,130^3]."""
    from distdl_amd import hip_ops
    pad = [[0, 0], [0, 0], [1, 1], [1, 1], [1, 1]]
    rs = [[0, 0], [0, 0], [0, 1], [0, 1], [0, 1]]
    plan = hip_ops.HaloPadPlan((1, 32, 128, 128, 128), pad, rs, rs)
    keep, steps = [], []
    for s in range(nsets):
        gen = torch.Generator().manual_seed(1005 + s)
        x = torch.randn(1, 32, 128, 128, 128, generator=gen).cuda()
        out = torch.empty(plan.padded_shape, device="cuda")
        gptr, bptr, bufs = [], [], []
        for d in range(5):
            for side in range(2):
                gs, bs = plan.slab_shape(d, side, "ghost"), plan.slab_shape(d, side, "bulk")
                g = None if gs is None else torch.randn(gs, generator=gen).cuda()
                b = None if bs is None else torch.empty(bs, device="cuda")
                bufs += [g, b]
                gptr.append(None if g is None else g.data_ptr())
                bptr.append(None if b is None else b.data_ptr())
        args = (x.data_ptr(), out.data_ptr(), plan.shape_arr, 5, 4, plan.pad_arr, plan.recv_arr, plan.send_arr,
                _lib.ptr_array(gptr), _lib.ptr_array(bptr), _lib.DDL_HALO_AUTO)
        keep.append((x, out, bufs, args))

        def fused(a=args):
            rc = lib.ddl_halo_pad_exchange(*a, STREAM[0])
            if rc:
                _lib.check(rc, "ddl_halo_pad_exchange")
        steps.append([fused])
    return steps, keep, 562531072


# ----------------------------------------------------------------------------
# backward (adjoint) workloads: the same shapes as the forward configurations
# ----------------------------------------------------------------------------

def _call(lib, _lib, name, args):
    def fn(a=args, f=getattr(lib, name), n=name):
        rc = f(*a, STREAM[0])
        if rc:
            _lib.check(rc, n)
    return fn


def build_layernorm_bwd(torch, lib, _lib, nsets):
    """Backward of config 1 on rank 0 as the layer runs it when every gradient
    is wanted: row sums + partial column sums in one launch, then (after the
    gather of the row sums) input gradient + final parameter sums in one launch.
    Algorithmic bytes: dy and x are read twice (once per launch), dx is written
    once: 5 x 8 388 608 B, plus the small vectors and the partial column sums."""
    rows, cols = 16 * 512, 256
    keep, steps = [], []
    for s in range(nsets):
        gen = torch.Generator(device="cuda").manual_seed(4001 + s)
        x = torch.randn(rows, cols, generator=gen, device="cuda")
        dy = torch.randn(rows, cols, generator=gen, device="cuda")
        gamma = 1 + 0.1 * torch.randn(cols, generator=gen, device="cuda")
        mean = 0.01 * torch.randn(rows, generator=gen, device="cuda")
        rstd = 1 + 0.01 * torch.randn(rows, generator=gen, device="cuda")
        sums = torch.zeros(4, rows, 2, device="cuda")                     # slot 0 is written by the kernel, 1..3 seeded
        dx = torch.empty_like(x)
        dg, db = torch.empty(cols, device="cuda"), torch.empty(cols, device="cuda")
        work = torch.empty(2 * 256 * cols, device="cuda")
        keep.append((x, dy, gamma, mean, rstd, sums, dx, dg, db, work))
        a1 = (dy.data_ptr(), x.data_ptr(), rows, cols, cols, cols, mean.data_ptr(), rstd.data_ptr(), gamma.data_ptr(),
              sums.data_ptr(), work.data_ptr(), work.numel())
        a2 = (dy.data_ptr(), x.data_ptr(), rows, cols, cols, cols, mean.data_ptr(), rstd.data_ptr(), gamma.data_ptr(),
              sums.data_ptr(), 4, 1.0 / (4 * cols), dx.data_ptr(), cols, work.data_ptr(), work.numel(), dg.data_ptr(),
              db.data_ptr())
        steps.append([_call(lib, _lib, "ddl_ln_bwd_partial_params_f32", a1),
                      _call(lib, _lib, "ddl_ln_bwd_input_params_f32", a2)])
    return steps, keep, 5 * rows * cols * 4 + 2 * (2 * rows * 4) + 5 * rows * 2 * 4 + 3 * cols * 4 + 2 * (2 * 256 * cols * 4)


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
        work = torch.empty(2 * 16032 + 1 + ids.numel(), dtype=torch.int32, device="cuda")
        keep.append((ids, dw, work))
        args = (dy.data_ptr(), _lib.DDL_DT_BF16, 4096, 4096, ids.data_ptr(), 1, ids.numel(), 0, 16032, -1, 0, dw.data_ptr(),
                4096, work.data_ptr(), work.numel())
        steps.append([_call(lib, _lib, "ddl_embedding_backward", args)])
    return steps, keep, sum(nbytes) / len(nbytes)


def build_linear_bwd(torch, lib, _lib, nsets):
    """Backward of config 4 on rank 0: dx = dy w and dw = dy^T x through the
    shard GEMM on transposed operands (the three transposes are part of the
    step), db = column sums of dy.  Work: 2 x 2 M N K flop."""
    M, N, K = 8192, 3584, 8192
    gen = torch.Generator(device="cuda").manual_seed(6004)
    w = (0.02 * torch.randn(N, K, generator=gen, device="cuda")).to(torch.bfloat16)
    w_t = torch.empty(K, N, dtype=torch.bfloat16, device="cuda")
    dy_t = torch.empty(N, M, dtype=torch.bfloat16, device="cuda")
    x_t = torch.empty(K, M, dtype=torch.bfloat16, device="cuda")
    work = torch.empty(64 * N, device="cuda")
    keep, steps = [w, w_t, dy_t, x_t, work], []
    for s in range(nsets):
        x = torch.randn(M, K, generator=gen, device="cuda").to(torch.bfloat16)
        dy = torch.randn(M, N, generator=gen, device="cuda").to(torch.bfloat16)
        dx = torch.empty(M, K, dtype=torch.bfloat16, device="cuda")
        dw = torch.empty(N, K, dtype=torch.bfloat16, device="cuda")
        db = torch.empty(N, dtype=torch.bfloat16, device="cuda")
        keep.append((x, dy, dx, dw, db))
        steps.append([
            _call(lib, _lib, "ddl_transpose_2d", (w.data_ptr(), w_t.data_ptr(), N, K, K, N, 2)),
            _call(lib, _lib, "ddl_linear_bf16", (dy.data_ptr(), w_t.data_ptr(), None, dx.data_ptr(), M, K, N, N, N, K)),
            _call(lib, _lib, "ddl_transpose_2d", (dy.data_ptr(), dy_t.data_ptr(), M, N, N, M, 2)),
            _call(lib, _lib, "ddl_transpose_2d", (x.data_ptr(), x_t.data_ptr(), M, K, K, M, 2)),
            _call(lib, _lib, "ddl_linear_bf16", (dy_t.data_ptr(), x_t.data_ptr(), None, dw.data_ptr(), N, K, M, M, M, K)),
            _call(lib, _lib, "ddl_colsum_bf16", (dy.data_ptr(), M, N, N, db.data_ptr(), work.data_ptr(), work.numel())),
        ])
    return steps, keep, 2 * 2 * M * N * K


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


# ----------------------------------------------------------------------------
# CPU baseline (the oracle, i.e. a port of the reference's mpi_numpy path)
# ----------------------------------------------------------------------------

def cpu_baseline_repartition(budget_s=12.0):
    """One rank's pack + unpack of config 2 with the oracle's NumPy code
    (np.copyto per box, zero-filled output), single thread, int16 views of the
    bf16 payload.  Runs whole steps until about `budget_s` seconds are spent."""
    import numpy as np
    from oracle import repartition as o_rep
    send, recv, _, _ = o_rep.plan([8, 4096, 8192], [1, 8, 1], [1, 1, 8])
    send0 = [(sl, sh, 99 if p == "self" else p) for sl, sh, p in send[0]]
    recv0 = [(sl, sh, 99 if p == "self" else p) for sl, sh, p in recv[0]]
    rng = np.random.default_rng(1002)
    x = rng.integers(0, 2 ** 16, size=(8, 512, 8192), dtype=np.uint16)
    rbufs = [rng.integers(0, 2 ** 16, size=(8, 512, 1024), dtype=np.uint16) for _ in range(8)]
    o_rep.pack(x, send0)
    o_rep.unpack(recv0, rbufs, (8, 4096, 1024), np.uint16)
    n, t0 = 0, time.perf_counter()
    while True:
        o_rep.pack(x, send0)
        o_rep.unpack(recv0, rbufs, (8, 4096, 1024), np.uint16)
        n += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s:
            break
    return {"value": 268435456 * n / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{n} full steps of config 2 (pack 8 boxes + zero-filled unpack of 8 boxes), "
                      f"NumPy np.copyto on uint16 views, one process standing in for rank 0, {dt:.1f} s"}


# ----------------------------------------------------------------------------

def main():
    args = parse_args()
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

    builders = {
        "repartition": (build_repartition, 8, 2, "hbm"),
        "layernorm": (build_layernorm, 64, 2, "hbm"),
        "layernorm_long": (build_layernorm_long, 3, 2, "hbm"),
        "embedding": (build_embedding, 4, 1, "hbm"),
        "linear": (build_linear, 4, 1, "mfma"),
        "halo": (build_halo, 4, 1, "hbm"),
        "layernorm_bwd": (build_layernorm_bwd, 32, 2, "hbm"),
        "embedding_bwd": (build_embedding_bwd, 4, 1, "hbm"),
        "linear_bwd": (build_linear_bwd, 2, 1, "mfma"),
        "calib": (build_calib, 4, 1, "hbm"),     # only with --only calib
    }
    names = [n.strip() for n in args.only.split(",")] if args.only else [n for n in builders if n != "calib"]
    for n in names:
        if n not in builders:
            raise SystemExit(f"bench.py: unknown workload {n!r}; choose from {', '.join(builders)}")
    results = {}
    for name in names:
        build, nsets, launches, bound = builders[name]
        step_fns, keep, work = build(torch, lib, _lib, nsets)
        steps = args.steps if name in ("repartition", "layernorm") else max(8, args.steps // 4)
        warm = args.warmup if name in ("repartition", "layernorm") else max(4, args.warmup // 4)
        m = measure(torch, name, step_fns, launches, steps, warm, use_graph)
        per_launch = work / launches
        if bound == "hbm":
            achieved, peak, unit = per_launch / m["launch_s"] / 1e9, HBM_PEAK_GBS, "GB/s"
            value = work * m["steps"] / m["wall_s"] / 1e9
        else:
            achieved, peak, unit = per_launch / m["launch_s"] / 1e12, MFMA_BF16_PEAK_TFLOPS, "TFLOP/s"
            value = work * m["steps"] / m["wall_s"] / 1e12
        results[name] = {
            "value": value, "unit": unit, "steps": m["steps"], "ms_per_step": 1e3 * m["wall_s"] / m["steps"],
            "mode": m["mode"], "work_per_step": work,
            "roofline": {"bound": bound, "achieved": achieved, "peak": peak, "unit": unit, "frac": achieved / peak,
                         "traffic": MEASURED_TRAFFIC_BYTES.get(name)},
        }
        del step_fns, keep
        torch.cuda.empty_cache()

    head_name = "repartition" if "repartition" in results else names[0]
    head = results[head_name]
    line = {
        "metric": "Repartition pack+unpack GB/s (rank 0, bf16 [8,4096,8192], P_x=[1,8,1] -> P_y=[1,1,8])"
        if head_name == "repartition" else head_name,
        "value": head["value"], "unit": head["unit"], "n_gpus": 1, "steps": head["steps"], "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u16" if head_name == "repartition" else "mixed", "data": "synthetic",
        "config": {"workload": "BASELINE.json configs[1]: Repartition pack/unpack bf16, rank 0 of 8, "
                               "pack [8,512,8192] -> 8x[8,512,1024], unpack 8x[8,512,1024] -> [8,4096,1024]"
                   if head_name == "repartition" else head_name,
                   "launch_mode": head["mode"], "buffer_sets": builders[head_name][1]},
        "roofline": head["roofline"],
        "workloads": results,
    }
    if not args.skip_cpu:
        line["cpu_baseline"] = cpu_baseline_repartition()
    print(json.dumps(line))


if __name__ == "__main__":
    main()

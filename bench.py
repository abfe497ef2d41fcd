#!/usr/bin/env python3
"""Benchmark of the MI355X DistConv hot path (one GPU).

One "step" is one pass of the path BASELINE.json's metric is quoted on:
  * 3-D batch-norm forward + backward on NCDHW 4 x 64 x 64^3 fp32 (config 3),
  * one full halo exchange (pack + unpack, 3 dimension phases, width 1) of a
    periodic 2 x 2 x 2 grid of virtual ranks, each N1 C32 128^3 fp32 (config 2).
`value` is the algorithmic bytes of a step divided by its wall time, inputs
resident in HBM.  Every BASELINE config, the exchange's phases and the
follow-on operators are timed separately under "breakdown" (GPU time through
HIP-graph replay, and the eager Python figure beside it where it differs).

Prints ONE JSON line.  `--gpus N` with N > 1 exits: this build runs on one GPU.
"""
from __future__ import annotations

import argparse
import hashlib
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth
SEED = 1234


def _gbs(nbytes: float, ms: float) -> float:
    return nbytes / (ms * 1e-3) / 1e9 if ms > 0 else 0.0


def _time_events(fn, iters: int, warmup: int, inner: int = 4):
    """Median and minimum milliseconds of one eager fn() measured with events on
    the current stream (the stream every kernel of fn is launched on).  `inner`
    calls are issued back to back between the two events so that the launch
    latency of a call is hidden behind the execution of the previous one -- the
    reference's harness hides it with a spin kernel
    (legacy/benchmarks/distconv_benchmark_bn.cpp:254-295).  Calls shorter than
    their own Python + launch cost (a few tens of microseconds) are bound by
    the host here; _time_graph gives their GPU time."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(iters):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(inner):
            fn()
        e1.record()
        e1.synchronize()
        times.append(e0.elapsed_time(e1) / inner)
    return statistics.median(times), min(times)


def _time_graph(fn, iters: int, warmup: int, inner: int = 4):
    """Median and minimum (of the per-iteration differences) milliseconds of one fn() on
    the GPU, free of host enqueue cost: `inner` calls are captured into one HIP graph and 2 x `inner`
    calls into another, both are replayed between two events, and the difference
    of the two replay times is divided by `inner`.  The difference removes what a
    replay costs besides its kernels (8-25 us between the first event and the
    first kernel on this stack: a 7 us call measured 9.5 us with 4 calls a replay
    and 8.1 us with 8)."""
    import torch
    for _ in range(max(warmup, 1)):
        fn()
    torch.cuda.synchronize()
    graphs = []
    for calls in (inner, 2 * inner):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(calls):
                fn()
        for _ in range(2):
            graph.replay()
        graphs.append(graph)
    torch.cuda.synchronize()
    times = ([], [])
    for _ in range(iters):
        for which, graph in enumerate(graphs):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            graph.replay()
            e1.record()
            e1.synchronize()
            times[which].append(e0.elapsed_time(e1))
    del graphs
    # one difference per iteration (the long and the short replay run back to back): their
    # median, and their minimum, which is the minimum of a difference and not a lower bound
    diffs = [(b - a) / inner for a, b in zip(*times)]
    return statistics.median(diffs), min(diffs)


def _time_graph_cold(fn, flush, iters: int, warmup: int, inner: int = 2):
    """GPU time of one fn() whose working set is in no cache when it starts: `flush` (a
    read-only pass over a buffer twice the size of the 256 MB memory-side cache, launched by
    the library's own sum kernel) runs before every call inside the graph.  One graph holds
    `inner` x (flush, fn), the other `inner` x flush; the difference of the two replay times
    divided by `inner` is the call, free of host enqueue cost and of the flush.  What the call
    leaves dirty in the caches is written back under the next flush, which both graphs pay
    alike only in part: the figure is an upper estimate of the cold call."""
    import torch
    for _ in range(max(warmup, 1)):
        flush()
        fn()
    torch.cuda.synchronize()
    graphs = []
    for with_fn in (False, True):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(inner):
                flush()
                if with_fn:
                    fn()
        for _ in range(2):
            graph.replay()
        graphs.append(graph)
    torch.cuda.synchronize()
    times = ([], [])
    for _ in range(iters):
        for which, graph in enumerate(graphs):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            graph.replay()
            e1.record()
            e1.synchronize()
            times[which].append(e0.elapsed_time(e1))
    del graphs
    diffs = [(b - a) / inner for a, b in zip(*times)]
    return statistics.median(diffs), min(diffs)


def _time_events_cold(fn, flush, iters: int, warmup: int):
    """As _time_events, but every timed call starts with caches that hold
    nothing of its working set: `flush` (a read of a buffer larger than the
    256 MB memory-side cache) runs before each one, outside the event pair."""
    import torch
    for _ in range(warmup):
        fn()
    times = []
    for _ in range(iters):
        flush()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        e1.synchronize()
        times.append(e0.elapsed_time(e1))
    return statistics.median(times), min(times)


class BatchNormWorkload:
    """BatchNormalization forward + backward on one rank.  `overlap` puts a
    halo of that width on every spatial dimension (the strided kernels)."""

    def __init__(self, shape_np, seed, overlap: int = 0, fuse_local: bool = True):
        import torch
        from dihydrogen_amd.layers import BatchNormalization
        from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
        g = torch.Generator(device="cuda").manual_seed(seed)
        nd = len(shape_np)
        c = shape_np[1]
        if overlap:
            # a distribution split over every spatial dimension gives the tensor its halos; one
            # virtual rank of it is enough to run the kernels on a haloed shard of this local size
            locale = [2] * (nd - 2) + [1, 1]
            dist = Distribution.make_overlapped_distribution(locale, [overlap] * (nd - 2) + [0, 0])
            gshape = [2 * e for e in shape_np[:1:-1]] + [shape_np[1], shape_np[0]]
            mk = lambda: Tensor(gshape, LocaleVirtual(0, 2 ** (nd - 2)), dist).allocate()
        else:
            dist = Distribution.make_localized_distribution(nd)
            mk = lambda: Tensor(list(shape_np[::-1]), LocaleVirtual(0, 1), dist).allocate()
        self.x, self.y, self.dy, self.dx = mk(), mk(), mk(), mk()
        self.x.data.normal_(0, 1, generator=g)
        self.dy.data.normal_(0, 1, generator=g)
        self.scale = torch.empty(c, device="cuda").uniform_(0.5, 1.5, generator=g)
        self.bias = torch.empty(c, device="cuda").normal_(0, 0.1, generator=g)
        self.mean, self.var = torch.empty(c, device="cuda"), torch.empty(c, device="cuda")
        self.rm, self.rv = torch.zeros(c, device="cuda"), torch.ones(c, device="cuda")
        self.grads = [torch.empty(c, device="cuda") for _ in range(4)]
        self.bn = BatchNormalization(nd, 0.9, 1e-5, fuse_local=fuse_local)
        self.elems = self.x.get_local_size()

    def forward(self):
        self.bn.forward(self.x, self.mean, self.var, self.rm, self.rv, self.scale, self.bias,
                        self.y, True)

    def backward(self):
        self.bn.backward(self.x, self.dy, self.mean, self.var, self.scale, *self.grads, self.dx)

    def backward_reduce(self):
        self.bn.backward_stage1(self.x, self.dy, self.mean, self.var, self.scale, *self.grads)
        self.bn.backward_allreduce(*self.grads)

    def backward_apply(self):
        self.bn.backward_stage2(self.x, self.dy, self.mean, self.var, self.scale, self.grads[2],
                                self.grads[3], self.dx)


class HaloWorkload:
    """Halo exchange of a 2 x 2 x 2 grid of virtual ranks (periodic unless said otherwise)."""

    def __init__(self, local_spatial, channels, seed, periodic=True):
        import torch
        from dihydrogen_amd.layers import HaloExchangeVirtual
        from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
        g = torch.Generator(device="cuda").manual_seed(seed)
        locale, overlap = (2, 2, 2, 1, 1), (1, 1, 1, 0, 0)
        gshape = [2 * local_spatial] * 3 + [channels, 1]
        dist = Distribution.make_overlapped_distribution(locale, overlap)
        self.ranks = [Tensor(gshape, LocaleVirtual(r, 8), dist).allocate() for r in range(8)]
        for t in self.ranks:
            t.interior_view().uniform_(-1, 1, generator=g)
        self.xch = HaloExchangeVirtual(self.ranks, periodic=periodic)
        face = (local_spatial + 2) ** 2 * channels
        # per rank: 3 dims x 2 sides x (pack: read+write, unpack: read+write) x 4 bytes
        self.bytes = 8 * 3 * 2 * 2 * 2 * face * 4
        self.elems = 8 * 12 * face

    def run(self):
        self.xch.exchange()


class SoftmaxWorkload:
    def __init__(self, shape_np, seed, instance: bool = False):
        import torch
        from dihydrogen_amd.layers import Softmax, SoftmaxMode
        from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
        g = torch.Generator(device="cuda").manual_seed(seed)
        dist = Distribution.make_localized_distribution(len(shape_np))
        mk = lambda: Tensor(list(shape_np[::-1]), LocaleVirtual(0, 1), dist).allocate()
        self.x, self.y, self.dy, self.dx = mk(), mk(), mk(), mk()
        self.x.data.normal_(0, 2, generator=g)  # sigma = 2
        self.dy.data.normal_(0, 1, generator=g)
        self.sm = Softmax()
        self.sm.setup(self.x, SoftmaxMode.INSTANCE if instance else SoftmaxMode.CHANNEL)
        self.elems = self.x.get_local_size()

    def forward(self):
        self.sm.forward(self.x, self.y)

    def backward(self):
        self.sm.backward(self.y, self.dy, self.dx)


class ShuffleWorkload:
    """Sample-parallel (N over `ranks` ranks) <-> spatial-parallel (H x W grid)."""

    def __init__(self, gshape, seed, ranks=4, grid=(2, 2), dst_overlap=0):
        import torch
        from dihydrogen_amd.layers import TensorShufflerVirtual
        from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
        g = torch.Generator(device="cuda").manual_seed(seed)
        sd = Distribution([1, 1, 1, ranks])
        dd = (Distribution.make_overlapped_distribution([grid[0], grid[1], 1, 1], [dst_overlap, dst_overlap, 0, 0])
              if dst_overlap else Distribution([grid[0], grid[1], 1, 1]))
        self.src = [Tensor(gshape, LocaleVirtual(r, ranks), sd).allocate() for r in range(ranks)]
        self.dst = [Tensor(gshape, LocaleVirtual(r, ranks), dd).allocate() for r in range(ranks)]
        for t in self.src:
            t.data.uniform_(-1, 1, generator=g)
        self.sh = TensorShufflerVirtual(self.src, self.dst)
        self.elems = 1
        for e in gshape:
            self.elems *= e

    def forward(self):
        self.sh.shuffle_forward()

    def backward(self):
        self.sh.shuffle_backward()


# ---------------------------------------------------------------------------------------------
# Parity gate: every timed configuration's outputs are checked on the GPU before its timing is
# taken, against the definition of the operation evaluated in float64 by library routines
# (batch-norm, softmax; bound 1e-5 of the terms of each expression, the bound an fp32 result
# can meet where terms cancel) or bit for bit against the closed form (halo: every cell of
# every rank equals the periodic global field; shuffle: every element sits at its global
# position, and the round trip restores the source).  The full comparison with the CPU oracle
# is in tests/; this gate keeps a wrong kernel from being timed.
# ---------------------------------------------------------------------------------------------
GATE_TOL = 1e-5


class ParityError(RuntimeError):
    pass


def _gate(ok: bool, what: str):
    if not ok:
        raise ParityError(f"parity gate failed: {what}")


def _within(got, want, terms, what):
    """|got - want| <= GATE_TOL * terms everywhere (terms: sum of the magnitudes of the
    addends of the expression, the conditioning of its fp32 evaluation)."""
    import torch
    err = (got.double() - want).abs()
    bound = GATE_TOL * terms + 1e-30
    bad = int((~(err <= bound)).sum())
    _gate(bad == 0, f"{what}: {bad} of {err.numel()} elements beyond {GATE_TOL:g} of their terms "
                    f"(largest error {float(err.max()):.3g})")
    return float((err / (terms + 1e-30)).max())


def gate_batchnorm(w: "BatchNormWorkload", backward: bool = True):
    """mean, var, y (and dscale, dbias, dmean, dvar, dx) of the last forward() / backward()."""
    import torch
    x = w.x.interior_view().double()
    dims = [0] + list(range(2, x.dim()))
    bshape = [1, -1] + [1] * (x.dim() - 2)
    n = x.numel() // x.shape[1]
    m64, v64 = x.mean(dims), x.var(dims, unbiased=True)
    q64 = (x * x).mean(dims)
    worst = {}
    worst["mean"] = _within(w.mean, m64, x.abs().mean(dims), "batch-norm mean")
    worst["var"] = _within(w.var, v64, q64 + m64 * m64, "batch-norm var")
    mean, var = w.mean.double(), w.var.double()
    r = torch.rsqrt(var + 1e-5)
    scale, bias = w.scale.double(), w.bias.double()
    xm = x - mean.view(bshape)
    a = xm * (r * scale).view(bshape)
    worst["y"] = _within(w.y.interior_view(), a + bias.view(bshape), a.abs() + bias.abs().view(bshape), "batch-norm y")
    del a
    if backward:
        dy = w.dy.interior_view().double()
        dscale, dbias, dmean, dvar = (g.double() for g in w.grads)
        t = dy * xm
        s_dyxm, a_dyxm = t.sum(dims), t.abs().sum(dims)
        del t
        s_dy, a_dy = dy.sum(dims), dy.abs().sum(dims)
        worst["dscale"] = _within(w.grads[0], s_dyxm * r, a_dyxm * r, "batch-norm dscale")
        worst["dbias"] = _within(w.grads[1], s_dy, a_dy, "batch-norm dbias")
        worst["dmean"] = _within(w.grads[2], -s_dy * scale * r, a_dy * scale * r, "batch-norm dmean")
        worst["dvar"] = _within(w.grads[3], -s_dyxm * scale * r ** 3 / 2, a_dyxm * scale * r ** 3 / 2,
                                "batch-norm dvar")
        t1 = dy * (scale * r).view(bshape)
        t2 = (dmean / n).view(bshape)
        t3 = xm * (dvar * 2 / (n - 1)).view(bshape)
        worst["dx"] = _within(w.dx.interior_view(), t1 + t2 + t3, t1.abs() + t2.abs() + t3.abs(), "batch-norm dx")
    return worst


def gate_halo(w: "HaloWorkload"):
    """After an exchange on the periodic grid every cell of every rank, halo cells included,
    holds the value of the global field at its wrapped global index
    (legacy/tests/tensor/test_halo_exchange_cuda.cu:104-233), bit for bit."""
    import torch
    ranks = w.ranks
    t0 = ranks[0]
    nd = len(t0.local_shape)
    gshape_np = [t0.shape[d] for d in range(nd - 1, -1, -1)]
    field = torch.empty(gshape_np, dtype=t0.data.dtype, device="cuda")
    for t in ranks:
        sl = tuple(slice(g, g + l) for g, l in zip(reversed(t.global_index), reversed(t.local_shape)))
        field[sl] = t.interior_view()
    ov = list(reversed(t0.overlap))            # numpy order
    pad = []
    for o in reversed(ov[2:]):                 # F.pad takes the last dimension first
        pad += [o, o]
    padded = torch.nn.functional.pad(field, pad, mode="circular")
    del field
    for r, t in enumerate(ranks):
        sl = tuple(slice(g, g + l + 2 * o)
                   for g, l, o in zip(reversed(t.global_index), reversed(t.local_shape), ov))
        _gate(torch.equal(t.real_view(), padded[sl]), f"halo exchange: rank {r} differs from the periodic field")
    return {"ranks": len(ranks), "cells_per_rank": int(ranks[0].real_view().numel())}


def gate_softmax(w: "SoftmaxWorkload", instance: bool = False):
    import torch
    x = w.x.interior_view().double()
    y = w.y.interior_view()
    if instance:
        want = torch.softmax(x.flatten(1), 1).view_as(x)
    else:
        want = torch.softmax(x, 1)
    # the reference clamps y to FLT_MIN from below (softmax.cu:565,590)
    want = want.clamp_min(1.1754943508222875e-38)
    worst = {"y": _within(y, want, want, "softmax y")}
    y64, dy = y.double(), w.dy.interior_view().double()
    ydy = y64 * dy
    if instance:
        dp = ydy.flatten(1).sum(1).view([-1] + [1] * (x.dim() - 1))
        adp = ydy.abs().flatten(1).sum(1).view([-1] + [1] * (x.dim() - 1))
    else:
        dp, adp = ydy.sum(1, keepdim=True), ydy.abs().sum(1, keepdim=True)
    want_dx = y64 * (dy - dp)
    terms = ydy.abs() + y64 * adp       # dp itself is a sum that cancels: its terms count, not its value
    # y at the clamp gives dx = 0 in the reference (softmax.cu:666); N(0, 2) logits never get there
    worst["dx"] = _within(w.dx.interior_view(), want_dx, terms, "softmax dx")
    return worst


def gate_shuffle(w: "ShuffleWorkload"):
    """forward: every destination rank holds its part of the global tensor; backward into
    cleared sources: the sources are back, bit for bit
    (legacy/tests/tensor/test_tensor_mpi_shuffle.cpp:26-154)."""
    import torch
    nd = len(w.src[0].local_shape)
    gshape_np = [w.src[0].shape[d] for d in range(nd - 1, -1, -1)]
    field = torch.empty(gshape_np, dtype=w.src[0].data.dtype, device="cuda")
    part = lambda t: tuple(slice(g, g + l) for g, l in zip(reversed(t.global_index), reversed(t.local_shape)))
    for t in w.src:
        field[part(t)] = t.interior_view()
    w.forward()
    for r, t in enumerate(w.dst):
        _gate(torch.equal(t.interior_view(), field[part(t)]), f"shuffle forward: destination rank {r}")
    for t in w.src:
        t.data.zero_()
    w.backward()
    for r, t in enumerate(w.src):
        _gate(torch.equal(t.interior_view(), field[part(t)]), f"shuffle backward: source rank {r}")
    return {"elements": int(field.numel())}


def _cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(repeats: int = 5):
    """The CPU oracle (this repository's restatement of the reference kernels:
    the reference has no CPU implementation of batch-norm, softmax or halo
    packing, and its CPU shuffler is restated too) timed on the host cores, per
    BASELINE config, on bounded samples that are stated with each figure."""
    import numpy as np
    import oracle
    from oracle import geometry as G
    lib = oracle.lib()
    lib.orc_num_threads.restype = __import__("ctypes").c_int
    threads = lib.orc_num_threads()
    rng = np.random.default_rng(SEED)

    def med(fn):
        """Median of at least `repeats` runs and at least two seconds of them
        (about 15 s of CPU work over all configs)."""
        fn()
        ts = []
        while len(ts) < repeats or (sum(ts) < 2.0 and len(ts) < 2000):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return statistics.median(ts)

    def entry(nbytes, elems, seconds, sample):
        return {"GB/s": nbytes / seconds / 1e9, "Gelem/s": elems / seconds / 1e9, "seconds": seconds,
                "bytes": nbytes, "sample": sample}

    configs = {}
    # C1: 2-D batch-norm forward, in full
    x1 = rng.standard_normal((8, 64, 56, 56), dtype=np.float32)
    sc, bi = rng.uniform(0.5, 1.5, 64).astype(np.float32), (0.1 * rng.standard_normal(64)).astype(np.float32)
    t = med(lambda: oracle.bn_forward(x1, sc, bi, np.zeros(64, np.float32), np.ones(64, np.float32)))
    configs["C1_bn2d_fwd"] = entry(3 * x1.size * 4, x1.size, t, "in full")
    # C3: 3-D batch-norm forward + backward, in full
    shp = (4, 64, 64, 64, 64)
    x3 = rng.standard_normal(shp, dtype=np.float32)
    dy3 = rng.standard_normal(shp, dtype=np.float32)

    def c3():
        y, mean, var = oracle.bn_forward(x3, sc, bi, np.zeros(64, np.float32), np.ones(64, np.float32))
        oracle.bn_backward(x3, dy3, mean, var, sc)

    t3 = med(c3)
    configs["C3_bn3d_fwd_bwd"] = entry(8 * x3.size * 4, x3.size, t3, "in full")
    del x3, dy3
    # C2: halo pack + unpack of all 6 faces, 2 of the 8 ranks
    halo_ranks = 2
    fields = [rng.uniform(-1, 1, (1, 32, 130, 130, 130)).astype(np.float32) for _ in range(halo_ranks)]
    bufs = {d: np.empty(oracle.halo_size((130, 130, 130, 32, 1), d, 1), np.float32) for d in range(3)}

    def c2():
        for f in fields:
            for d in range(3):
                for side in (0, 1):
                    oracle.halo_pack_or_unpack(f, d, side, 1, bufs[d], True)
                    oracle.halo_pack_or_unpack(f, d, side, 1, bufs[d], False)

    t2 = med(c2)
    halo_bytes = halo_ranks * 3 * 2 * 2 * 2 * bufs[0].size * 4
    configs["C2_halo"] = entry(halo_bytes, halo_ranks * 12 * bufs[0].size, t2,
                               f"{halo_ranks} of 8 ranks, all 6 faces each, pack + unpack")
    del fields
    # C4: channel softmax forward + backward, in full
    x4 = (2 * rng.standard_normal((16, 21, 256, 256), dtype=np.float32))
    dy4 = rng.standard_normal((16, 21, 256, 256), dtype=np.float32)

    def c4():
        y = oracle.softmax_channel_forward(x4)
        oracle.softmax_channel_backward(y, dy4)

    t4 = med(c4)
    configs["C4_softmax_fwd_bwd"] = entry(5 * x4.size * 4, x4.size, t4, "in full")
    del x4, dy4
    # C5: the shuffler's pack + unpack of one direction.  Generic per-element path (single-threaded,
    # as the reference's: shuffle_mpi.hpp:688-706,851-872) on one of the four ranks; OpenMP row-copy
    # path (shuffle_mpi.hpp:708-849,874-947) on all four.
    shape5, n5 = (128, 128, 64, 32), 4
    src_g = [G.TensorGeom(shape5, G.Dist((1, 1, 1, 4), (1, 1, 1, 4), [0] * 4), r) for r in range(n5)]
    dst_g = [G.TensorGeom(shape5, G.Dist((2, 2, 1, 1), (2, 2, 1, 1), [0] * 4), r) for r in range(n5)]
    # every rank has arrays of its own, as in a real job: nothing is shared through the caches
    fields5 = [rng.uniform(-1, 1, src_g[r].local_size).astype(np.float32) for r in range(n5)]
    bufs5 = [np.empty(src_g[r].local_size, np.float32) for r in range(n5)]
    outs5 = [np.empty(dst_g[r].local_size, np.float32) for r in range(n5)]
    field = fields5[0]
    tables = []
    for r in range(n5):
        _, sd, _, rd = G.counts_and_displs(src_g[r], dst_g[r])
        tables.append((G.rank_limits(src_g[r], dst_g[r]), sd, G.rank_limits(dst_g[r], src_g[r]), rd))

    def generic(r):
        lim, sd, lim_d, rd = tables[r]
        field, buf, out = fields5[r], bufs5[r], outs5[r]
        oracle.shuffle_pack_or_unpack(field, src_g[r].local_shape, src_g[r].strides(), (2, 2, 1, 1), lim, buf, sd, True)
        oracle.shuffle_pack_or_unpack(out, dst_g[r].local_shape, dst_g[r].strides(), (1, 1, 1, 4), lim_d, buf, rd, False)

    def rows():
        for r in range(n5):
            lim, sd, lim_d, rd = tables[r]
            field, buf, out = fields5[r], bufs5[r], outs5[r]
            oracle.shuffle_rows(field, src_g[r].local_shape, src_g[r].strides(), (2, 2, 1, 1), lim, buf, sd, True)
            oracle.shuffle_rows(out, dst_g[r].local_shape, dst_g[r].strides(), (1, 1, 1, 4), lim_d, buf, rd, False)

    t0 = time.perf_counter()
    generic(0)
    tg = time.perf_counter() - t0
    per_rank = 4 * field.size * 4  # pack read + write, unpack read + write
    configs["C5_shuffle_generic"] = entry(per_rank, field.size, tg,
                                          "1 of 4 ranks, forward direction, per-element path on one thread (one run)")
    tr = med(rows)
    configs["C5_shuffle_row_copy"] = entry(n5 * per_rank, n5 * field.size, tr,
                                           "all 4 ranks, forward direction, OpenMP row-copy path")
    # the step the headline value is quoted on: C3 in full + C2 scaled to its 2-rank sample
    step_bytes = 8 * 67108864 * 4 + halo_bytes
    return {
        "value": step_bytes / (t3 + t2) / 1e9,
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "cpu_model": _cpu_model(),
        "logical_cpus": os.cpu_count(),
        "sample": (f"config 3 batch-norm fwd+bwd in full + config 2 exchange of {halo_ranks} of 8 ranks; "
                   f"medians of at least {repeats} runs and 2 s each ({t3:.3f} s + {t2:.3f} s a run); gcc -O3 -fopenmp, "
                   f"OMP threads = {threads}"),
        "configs": configs,
    }


# Traffic between the L2 and the memory fabric per launch, measured with rocprofv3 --pmc
# (profiles/bench_pmc_traffic.txt): read bytes = 128 x TCC_EA0_RDREQ_128B + 64 x TCC_EA0_RDREQ_64B
# + 32 x TCC_EA0_RDREQ_32B, written bytes = 64 x TCC_EA0_WRREQ_64B + 32 x (TCC_EA0_WRREQ -
# TCC_EA0_WRREQ_64B), request counts summed over the L2 channels, per dispatch.
# label -> (bytes read, bytes written) per launch
PMC_TRAFFIC = {
    "bn_sums": (268455424, 131072),
    "bn_apply": (268462080, 268468224),
    "bn_backprop1": (536912576, 131104),
    "bn_backprop2": (536906240, 268435456),
    "halo_dim0_pack": (150615792, 8652800),    # 4 faces (2 ranks) a launch, four launches a step
    "halo_dim0_unpack": (9218176, 43264000),
    "halo_dim1_pack": (42624704, 34611200),
    "halo_dim1_unpack": (34630400, 36218592),
    "halo_dim2_pack": (34694400, 34611200),
    "halo_dim2_unpack": (34630400, 34619392),
}
# steps of the timed region whose dominant-kernel launches are bracketed by events: every EVENT_EVERY-th
EVENT_EVERY = 4

# sha256 (first 16 hex digits) of the kernel sources the table was measured with, see
# kernel_sources_sha(); with other sources the traffic fields are omitted
PMC_SOURCES_SHA = "3bcdabae02179b5c"
PMC_COMMIT = "3387492"

KERNEL_OF = {
    "bn_sums": "bn_sums_kernel<float,4> (+bn_finish_kernel<float,2>)",
    "bn_statistics": "bn_statistics_kernel<float>",
    "bn_apply": "bn_apply_kernel<float,4>",
    "bn_backprop1": "bn_backprop1_kernel<float,4> (+bn_finish_kernel<float,4>)",
    "bn_backprop2": "bn_backprop2_kernel<float,4>",
    "halo_dim0_pack": "box_copy_kernel<u32,1,OpId,sparse,pack>",
    "halo_dim0_unpack": "box_copy_kernel<u32,1,OpId,sparse,unpack>",
    "halo_dim1_pack": "box_copy_kernel<u32,4,OpId,dense,pack>",
    "halo_dim1_unpack": "box_copy_kernel<u32,4,OpId,dense,unpack>",
    "halo_dim2_pack": "box_copy_kernel<u32,4,OpId,dense,pack>",
    "halo_dim2_unpack": "box_copy_kernel<u32,4,OpId,dense,unpack>",
}


# the sources of the kernels of the step (batch-norm and box copy), whose traffic PMC_TRAFFIC holds
STEP_KERNEL_SOURCES = ("h2x_bn.hip", "h2x_bn_maps.hpp", "h2x_copy.hip", "h2x_copy_acc.hip", "h2x_copy_kernel.hpp", "h2x_device.hpp")


def kernel_sources_sha() -> str:
    """Hash of the HIP sources of the step's kernels: ties the measured-traffic
    constants to the kernels they were measured on."""
    h = hashlib.sha256()
    d = os.path.join(ROOT, "dihydrogen_amd", "csrc")
    for name in STEP_KERNEL_SOURCES:
        with open(os.path.join(d, name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


def dim0_study():
    """The dimension-0 phase of the config 2 exchange (one 4-byte element per
    520-byte row and side) as a rate of memory transactions: every packed
    element costs the fetch of a 128-byte line (two neighbouring rows' ends
    share one), every unpacked row seam an 8-byte partial write.  Timed for
    launch groups of 2, 4 and 8 ranks, pack and unpack alone and together, and
    for the tensor-to-tensor form."""
    import ctypes
    import torch
    from dihydrogen_amd import capi
    from dihydrogen_amd.layers import HaloExchangeAccumOp
    lib = capi.load()
    halo = HaloWorkload(128, 32, SEED + 2)
    xch, dt = halo.xch, halo.ranks[0].h2x_dtype
    rows = 130 * 130 * 32                      # rows of one rank
    lines_per_rank = rows * (1 + 12 / 128)     # one line per row pair end, 12 bytes apart: 9 % straddle
    seams_per_rank = rows
    ident = HaloExchangeAccumOp.ID

    def faces(group, is_pack):
        out = []
        for r in group:
            for side in (capi.LHS, capi.RHS):
                peer = xch.find_peer_rank(r, 0, side)
                buf = xch.recv_buffer(peer, 0, capi.LHS if side == capi.RHS else capi.RHS) if is_pack \
                    else xch.recv_buffer(r, 0, side)
                out.append(xch.make_face(r, 0, side, 1, buf, is_pack, False, ident))
        return (capi.HaloFace * len(out))(*out)

    def launch(arr):
        # on torch's current stream (the capture stream while a graph is recorded)
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        capi.check(lib.h2x_halo_pack_or_unpack_batched(dt, arr, len(arr), stream), "halo")

    result = {"rows_per_rank": rows, "lines_per_rank": int(lines_per_rank), "seam_writes_per_rank": seams_per_rank,
              "groups": {}}
    for size in (2, 4, 8):
        groups = [list(range(g, g + size)) for g in range(0, 8, size)]
        packs = [faces(g, True) for g in groups]
        unpacks = [faces(g, False) for g in groups]
        t_pack = _time_graph(lambda: [launch(a) for a in packs], 10, 3, inner=2)[0]
        t_unpack = _time_graph(lambda: [launch(a) for a in unpacks], 10, 3, inner=2)[0]
        t_both = _time_graph(lambda: [(launch(p), launch(u)) for p, u in zip(packs, unpacks)], 10, 3, inner=2)[0]
        result["groups"][str(size)] = {
            "pack_us": t_pack * 1e3, "unpack_us": t_unpack * 1e3, "pack_then_unpack_us": t_both * 1e3,
            "pack_Glines_per_s": 8 * lines_per_rank / (t_pack * 1e-3) / 1e9,
            "pack_line_traffic_GB/s": 8 * lines_per_rank * 128 / (t_pack * 1e-3) / 1e9,
            "unpack_Gseams_per_s": 8 * seams_per_rank / (t_unpack * 1e-3) / 1e9,
        }
    ov = [1, 0, 0, 0, 0]
    t_fused = _time_graph(lambda: xch.exchange(ov, ov, ov, ov, fused=True), 10, 3, inner=2)[0]
    result["fused_us"] = t_fused * 1e3
    return result


def halo_sweep():
    """How the rate of a dense halo phase grows with the bytes one launch moves:
    the dimension-1 and dimension-2 phases (one pack launch + one unpack launch,
    16 faces each) of the config 2 grid at 2 ... 128 channels, and beside each
    two plain device-to-device copies of the same bytes.  A phase that tracks
    the copies is bound by how fast a launch of that size fills and drains the
    chip, not by its access pattern."""
    import torch
    rows = []
    for channels in (2, 4, 8, 16, 32, 64, 128):
        halo = HaloWorkload(128, channels, SEED + 2)
        launch_bytes = halo.bytes // 6  # one launch: 16 faces read and written
        n = launch_bytes // 8           # floats one plain copy moves (read + write = launch_bytes)
        a = torch.empty(2, n, device="cuda").normal_()
        b = torch.empty(2, n, device="cuda")
        row = {"channels": channels, "bytes_per_launch": launch_bytes}
        t = _time_graph(lambda: (b[0].copy_(a[0]), b[1].copy_(a[1])), 20, 5)[0]
        row["copy_pair_us"], row["copy_pair_GB/s"] = t * 1e3, _gbs(2 * launch_bytes, t)
        for d, name in ((1, "dim1"), (2, "dim2")):
            ov = [1 if k == d else 0 for k in range(5)]
            t = _time_graph(lambda ov=ov: halo.xch.exchange(ov, ov, ov, ov), 20, 5)[0]
            row[f"{name}_us"], row[f"{name}_GB/s"] = t * 1e3, _gbs(2 * launch_bytes, t)
            row[f"{name}_vs_copy"] = row["copy_pair_us"] / (t * 1e3)
        rows.append(row)
        del halo, a, b
        torch.cuda.empty_cache()
    return {"peak_GB/s": HBM_PEAK_GBS, "rows": rows}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-breakdown", action="store_true")
    ap.add_argument("--dim0-study", action="store_true",
                    help="instead of the benchmark: the innermost-dimension halo phase alone, by number of "
                         "ranks per launch group, as cache lines and seam writes per second")
    ap.add_argument("--halo-sweep", action="store_true",
                    help="instead of the benchmark: the dimension-1 and -2 halo phases of the config 2 grid for "
                         "growing channel counts, beside plain copies of the same bytes per launch")
    ap.add_argument("--sources-sha", action="store_true", help="print the hash of the kernel sources and exit")
    args = ap.parse_args()
    if args.sources_sha:
        print(kernel_sources_sha())
        return 0
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (virtual ranks share it); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        return 2

    import torch
    from dihydrogen_amd import capi
    capi.load()  # raises if libh2x.so is missing: there is no fallback
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    torch.cuda.set_device(0)

    if args.dim0_study:
        print(json.dumps(dim0_study()))
        return 0

    if args.halo_sweep:
        print(json.dumps(halo_sweep()))
        return 0

    bn3 = BatchNormWorkload((4, 64, 64, 64, 64), SEED + 3)
    halo = HaloWorkload(128, 32, SEED + 2)
    S3 = bn3.elems
    bn_bytes = 8 * S3 * 4
    step_bytes = bn_bytes + halo.bytes
    step_elems = S3 + halo.elems
    face_bytes = halo.bytes // (6 * 16)  # one face of one rank, read + write (16 faces per dimension)
    algo_bytes = {"bn_sums": S3 * 4, "bn_statistics": 0, "bn_apply": 2 * S3 * 4, "bn_backprop1": 2 * S3 * 4,
                  "bn_backprop2": 3 * S3 * 4}
    faces_per_launch = {}  # halo label -> faces in one launch (the exchange may split a phase)

    # Every launch is bracketed by a pair of events on the stream it is launched on
    # (torch's current stream, whose handle the C ABI receives).
    events = {}
    recording = [False]
    only = [None]  # labels to instrument; None = all

    def timed(label, launch, num_faces=None):
        if num_faces is not None:
            faces_per_launch[label] = num_faces
            algo_bytes[label] = num_faces * face_bytes
        if not recording[0] or (only[0] is not None and label not in only[0]):
            launch()
            return
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        launch()
        e1.record()
        events.setdefault(label, []).append((e0, e1))

    halo.xch.launch_hook = timed
    b = bn3.bn
    nps = b._num_per_sum(bn3.x)

    def step():
        """The timed step: the layer's own forward() and backward() (two launches each: the
        second kernel of each finishes the first one's channel sums) and the exchange."""
        bn3.forward()
        bn3.backward()
        halo.run()

    def step_staged():
        """The same work with the staged batch-norm entry points (what a rank that all-reduces
        between the stages runs), every launch labelled: the per-launch table."""
        timed("bn_sums", lambda: b.forward_stage1(bn3.x, bn3.mean, bn3.var, True))
        timed("bn_statistics", lambda: b.sums_to_statistics(nps, bn3.mean, bn3.var, bn3.rm, bn3.rv))
        timed("bn_apply", lambda: b.batch_normalization(bn3.x, bn3.mean, bn3.var, bn3.scale, bn3.bias, bn3.y))
        timed("bn_backprop1", bn3.backward_reduce)
        timed("bn_backprop2", bn3.backward_apply)
        halo.run()

    def kernel_share(evs):
        """Milliseconds per step by kernel: median launch time x launches per step."""
        tot = {}
        for label, pairs in evs.items():
            per_step = 16 // faces_per_launch[label] if label in faces_per_launch else 1
            ms = statistics.median(e0.elapsed_time(e1) for e0, e1 in pairs) * per_step
            tot[KERNEL_OF[label]] = tot.get(KERNEL_OF[label], 0.0) + ms
        return tot

    # warm-up, with every launch bracketed by events: finds the dominant kernel
    recording[0] = True
    for _ in range(max(args.warmup, 3)):
        step_staged()
    torch.cuda.synchronize()
    share0 = kernel_share(events)
    dominant = max(share0, key=share0.get)
    events.clear()
    step()  # the fused entry points once, untimed (first-use allocations)
    torch.cuda.synchronize()
    events.clear()
    # parity gate of the step's two configurations, before the timed region
    parity = {"C3_bn3d_fwd_bwd": gate_batchnorm(bn3), "C2_halo_8ranks": gate_halo(halo)}
    torch.cuda.synchronize()

    # timed region: only the dominant kernel's launches carry events, and only in every
    # EVENT_EVERY-th step (a pair of timing events costs the stream 2-3 us: bracketing all four
    # launches of every step would take 3 % off the figure the events are there to explain)
    only[0] = {l for l, k in KERNEL_OF.items() if k == dominant}
    t0 = time.perf_counter()
    for i in range(args.steps):
        recording[0] = i % EVENT_EVERY == 0
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    recording[0] = True
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    value = _gbs(step_bytes, ms_per_step)
    dominant_events = dict(events)
    events.clear()

    # a second, fully instrumented pass for the per-launch table
    only[0] = None
    for _ in range(args.steps):
        step_staged()
    torch.cuda.synchronize()
    recording[0] = False
    halo.xch.launch_hook = None
    for label, pairs in dominant_events.items():
        events[label] = pairs  # the dominant kernel's figures come from the timed region

    sources_sha = kernel_sources_sha()
    traffic_valid = bool(PMC_TRAFFIC) and sources_sha == PMC_SOURCES_SHA
    launches = {}
    for label, pairs in events.items():
        samples = [e0.elapsed_time(e1) for e0, e1 in pairs]
        # the dominant kernel's figure is the average over the timed region; the other launches come
        # from the instrumented pass, where the median keeps a late host enqueue out of the figure
        ms = statistics.mean(samples) if label in dominant_events else statistics.median(samples)
        launches[label] = {
            "kernel": KERNEL_OF[label], "avg_launch_ms": ms, "algorithmic_bytes": algo_bytes[label],
            "GB/s": _gbs(algo_bytes[label], ms), "frac": _gbs(algo_bytes[label], ms) / HBM_PEAK_GBS,
            "traffic": sum(PMC_TRAFFIC[label]) if traffic_valid and label in PMC_TRAFFIC else None,
        }
        if label in faces_per_launch:
            launches[label]["faces"] = faces_per_launch[label]
            launches[label]["launches_per_step"] = 16 // faces_per_launch[label]
    # dominant kernel = the kernel with the largest share of the step's launch time
    share = {}
    for label, v in launches.items():
        share.setdefault(v["kernel"], []).append(label)
    dl = [l for l in share[dominant] if l in dominant_events] or share[dominant]
    d_ms = statistics.mean(launches[l]["avg_launch_ms"] for l in dl)
    d_bytes = statistics.mean(launches[l]["algorithmic_bytes"] for l in dl)
    d_traffic = (statistics.mean(launches[l]["traffic"] for l in dl)
                 if all(launches[l]["traffic"] is not None for l in dl) else None)
    roofline = {
        "kernel": dominant, "launches_per_step": dl, "bound": "hbm",
        "achieved": _gbs(d_bytes, d_ms), "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": _gbs(d_bytes, d_ms) / HBM_PEAK_GBS,
        "traffic": int(d_traffic) if d_traffic is not None else None,
        "avg_launch_ms": d_ms, "algorithmic_bytes": int(d_bytes),
        "avg_launch_samples": sum(len(dominant_events[l]) for l in dl if l in dominant_events),
        "avg_launch_source": f"HIP events around this kernel's launches in every {EVENT_EVERY}th step of "
                             "the timed region",
        # the same launch priced by the bytes the memory system moved for it
        "traffic_GB/s": _gbs(d_traffic, d_ms) if d_traffic is not None else None,
        "frac_of_peak_in_traffic": _gbs(d_traffic, d_ms) / HBM_PEAK_GBS if d_traffic is not None else None,
        "traffic_source": (f"rocprofv3 --pmc, profiles/bench_pmc_traffic.txt @ {PMC_COMMIT}, kernel sources "
                           f"{PMC_SOURCES_SHA}" if traffic_valid else
                           f"omitted: kernel sources {sources_sha} differ from the profiled {PMC_SOURCES_SHA or 'none'}"),
    }

    breakdown = {}
    if not args.no_breakdown:
        it, wu = 20, 5

        def entry(nbytes, elems, fn, inner=4, eager=True):
            med, mn = _time_graph(fn, it, wu, inner)
            e = {"bytes": nbytes, "ms_median": med, "ms_min": mn, "GB/s": _gbs(nbytes, med),
                 "frac_of_peak": _gbs(nbytes, med) / HBM_PEAK_GBS, "Gelem/s": elems / (med * 1e-3) / 1e9,
                 "timing": "HIP-graph replay, difference of two replay lengths (GPU time)"}
            if eager:
                e["ms_eager_median"] = _time_events(fn, it, wu, inner)[0]
            return e

        evict = torch.empty(1 << 27, device="cuda").fill_(1.0)   # 512 MB: twice the memory-side cache
        from dihydrogen_amd import layers as L
        from dihydrogen_amd.tensor import Distribution as _D, LocaleVirtual as _LV, Tensor as _T
        evict_t = _T([1 << 21, 1, 1, 64, 1], _LV(0, 1), _D.make_localized_distribution(5))
        evict_t.data = evict
        evict_stat = _T([1, 1, 1, 64, 1], _LV(0, 1), _D.make_localized_distribution(5)).allocate()
        flush_in_graph = lambda: L.reduce_sum(evict_t, evict_stat)   # a read-only pass, the library's own kernel

        def cold_entry(nbytes, elems, fn, inner=2):
            med, mn = _time_graph_cold(fn, flush_in_graph, it, wu, inner)
            return {"bytes": nbytes, "ms_median": med, "ms_min": mn, "GB/s": _gbs(nbytes, med),
                    "frac_of_peak": _gbs(nbytes, med) / HBM_PEAK_GBS, "Gelem/s": elems / (med * 1e-3) / 1e9,
                    "timing": "HIP-graph replay of (512 MB read-only flush, call) pairs minus the replay of the "
                              "flushes alone (GPU time, caches cold)"}

        breakdown["C3_bn3d_fwd"] = entry(3 * S3 * 4, S3, bn3.forward)
        breakdown["C3_bn3d_bwd"] = entry(5 * S3 * 4, S3, bn3.backward)
        breakdown["C3_bn3d_fwd_bwd"] = entry(8 * S3 * 4, S3, lambda: (bn3.forward(), bn3.backward()), inner=2)
        breakdown["C3_bn3d_fwd_bwd_cold"] = cold_entry(8 * S3 * 4, S3, lambda: (bn3.forward(), bn3.backward()), inner=1)
        bn3.bn.fuse_local = False
        bn3.forward(), bn3.backward()
        parity["C3_bn3d_fwd_bwd_staged"] = gate_batchnorm(bn3)
        breakdown["C3_bn3d_fwd_bwd_staged"] = entry(8 * S3 * 4, S3, lambda: (bn3.forward(), bn3.backward()), inner=2)
        bn3.bn.fuse_local = True
        breakdown["C2_halo_8ranks"] = entry(halo.bytes, halo.elems, halo.run, inner=2)
        for d, name in enumerate(("dim0_W", "dim1_H", "dim2_D")):
            ov = [1 if k == d else 0 for k in range(5)]
            fn = lambda ov=ov: halo.xch.exchange(ov, ov, ov, ov)
            breakdown[f"C2_halo_{name}"] = entry(halo.bytes // 3, halo.elems // 3, fn)
            breakdown[f"C2_halo_{name}_cold"] = cold_entry(halo.bytes // 3, halo.elems // 3, fn)
        breakdown["C2_halo_8ranks_cold"] = cold_entry(halo.bytes, halo.elems, halo.run, inner=1)
        # the same exchange as tensor-to-tensor transfers (no buffers): half the bytes per strip
        for t in halo.ranks:          # poison the halos: the fused exchange has to fill every cell again
            keep = t.interior_view().clone()
            t.real_view().fill_(float("nan"))
            t.interior_view().copy_(keep)
        del keep
        halo.xch.exchange(fused=True)
        parity["C2_halo_8ranks_fused"] = gate_halo(halo)
        breakdown["C2_halo_8ranks_fused"] = entry(halo.bytes // 2, halo.elems // 2,
                                                  lambda: halo.xch.exchange(fused=True), inner=2)
        for d, name in enumerate(("dim0_W", "dim1_H", "dim2_D")):
            ov = [1 if k == d else 0 for k in range(5)]
            fn = lambda ov=ov: halo.xch.exchange(ov, ov, ov, ov, fused=True)
            breakdown[f"C2_halo_{name}_fused"] = entry(halo.bytes // 6, halo.elems // 6, fn)
        # follow-on rows at the config 2 shape: clear_halo of all three dimensions on every rank
        # (writes only), and the reverse exchange that adds halo contributions onto the interiors
        from dihydrogen_amd.layers import HaloExchangeAccumOp

        def clear_all():
            for d in range(3):
                halo.xch.clear_halo(d)

        breakdown["C2_clear_halo_8ranks"] = entry(halo.bytes // 4, halo.elems // 2, clear_all, inner=2)
        # the same strips cleared by one batched call (3 launches instead of 24)
        breakdown["C2_clear_halos_batched_8ranks"] = entry(halo.bytes // 4, halo.elems // 2, halo.xch.clear_halos,
                                                          inner=2)
        # pack: read + write; accumulating unpack: read buffer, read + write tensor -> 5/4 of the forward bytes
        breakdown["C2_halo_reverse_sum_8ranks"] = entry(
            halo.bytes * 5 // 4, halo.elems,
            lambda: halo.xch.exchange(is_reverse=True, op=HaloExchangeAccumOp.SUM), inner=2)
        # tensor::Transform / ReduceSum at the config 3 shape: scale in place (read + write), copy into a
        # second tensor (read + write), per-channel sums and sums of squares (one read each)
        breakdown["C3_transform_scale"] = entry(2 * S3 * 4, S3, lambda: L.transform(capi.TRANSFORM_SCALE, [bn3.y], [1.0]))
        breakdown["C3_transform_copy"] = entry(2 * S3 * 4, S3, lambda: L.transform(capi.TRANSFORM_COPY, [bn3.x, bn3.y]))
        stat = _T([1, 1, 1, 64, 1], _LV(0, 1), _D.make_localized_distribution(5)).allocate()
        stat.data.zero_()
        L.reduce_sum(bn3.x, stat)
        want = bn3.x.interior_view().double().sum((0, 2, 3, 4))
        parity["C3_reduce_sum_per_channel"] = {"sum": _within(
            stat.data.view(-1), want, bn3.x.interior_view().double().abs().sum((0, 2, 3, 4)), "reduce_sum")}
        breakdown["C3_reduce_sum_per_channel"] = entry(S3 * 4, S3, lambda: L.reduce_sum(bn3.x, stat))
        breakdown["C3_reduce_sum_per_channel_cold"] = cold_entry(S3 * 4, S3, lambda: L.reduce_sum(bn3.x, stat))
        breakdown["C3_reduce_sqsum_per_channel"] = entry(S3 * 4, S3, lambda: L.reduce_sum(bn3.x, stat, square=True))
        # what a convolution does before it runs (convolution.hpp:400-411): clear the halos, exchange.
        # Bytes: the exchange's; the clearing is overhead.  On the periodic grid every strip is overwritten
        # by the exchange, on the open one half of them.
        breakdown["C2_clear_then_exchange"] = entry(halo.bytes, halo.elems,
                                                    lambda: (halo.xch.clear_halos(), halo.run()), inner=2)
        breakdown["C2_clear_unfilled_then_exchange"] = entry(
            halo.bytes, halo.elems, lambda: (halo.xch.clear_halos(only_unfilled=True), halo.run()), inner=2)
        yard_x, yard_y = bn3.x.data, bn3.y.data
        breakdown["yardstick_torch_copy_268MB"] = entry(2 * S3 * 4, S3, lambda: yard_y.copy_(yard_x), eager=False)
        del bn3, halo, b, yard_x, yard_y
        torch.cuda.empty_cache()
        # the same on an open (non-periodic) 2 x 2 x 2 grid: every rank has a neighbour on 3 of its 6 sides
        halo_open = HaloWorkload(128, 32, SEED + 2, periodic=False)
        breakdown["C2open_clear_then_exchange"] = entry(halo_open.bytes // 2, halo_open.elems // 2,
                                                        lambda: (halo_open.xch.clear_halos(), halo_open.run()), inner=2)
        breakdown["C2open_clear_unfilled_then_exchange"] = entry(
            halo_open.bytes // 2, halo_open.elems // 2,
            lambda: (halo_open.xch.clear_halos(only_unfilled=True), halo_open.run()), inner=2)
        del halo_open
        torch.cuda.empty_cache()
        # strided batch-norm: the config 3 shard with a halo of 1 on all three spatial dimensions
        bn3h = BatchNormWorkload((4, 64, 64, 64, 64), SEED + 6, overlap=1)
        bn3h.forward(), bn3h.backward()
        parity["C3_bn3d_haloed_fwd_bwd"] = gate_batchnorm(bn3h)
        breakdown["C3_bn3d_haloed_fwd_bwd"] = entry(8 * bn3h.elems * 4, bn3h.elems,
                                                    lambda: (bn3h.forward(), bn3h.backward()), inner=2)
        # the same shard with clear_output_halo: normalise and the input gradient walk the whole real
        # tensors in aligned vectors and leave the halos of y and dx cleared (what the convolution that
        # follows would do with a separate clear_halo per dimension); the gate also looks at the halos
        bn3h.bn.clear_output_halo = True
        for t in (bn3h.y, bn3h.dx):
            t.real_view().fill_(float("nan"))
        bn3h.forward(), bn3h.backward()
        parity["C3_bn3d_haloed_clearing_fwd_bwd"] = gate_batchnorm(bn3h)
        for t, what in ((bn3h.y, "y"), (bn3h.dx, "dx")):
            # as many non-zero cells in the real tensor as in its interior, none of them a NaN
            nonzero_real, nonzero_interior = int((t.real_view() != 0).sum()), int((t.interior_view() != 0).sum())
            _gate(nonzero_real == nonzero_interior and not bool(torch.isnan(t.real_view()).any()),
                  f"clearing batch-norm: halo of {what} is not zero")
        breakdown["C3_bn3d_haloed_clearing_fwd_bwd"] = entry(8 * bn3h.elems * 4, bn3h.elems,
                                                             lambda: (bn3h.forward(), bn3h.backward()), inner=2)
        del bn3h
        torch.cuda.empty_cache()
        # short segments (the last stage of a ResNet): a workgroup serves a window of whole channels
        bn7 = BatchNormWorkload((256, 2048, 7, 7), SEED + 7)
        bn7.forward(), bn7.backward()
        parity["bn2d_7x7_N256_C2048"] = gate_batchnorm(bn7)
        breakdown["bn2d_7x7_N256_C2048_fwd"] = entry(3 * bn7.elems * 4, bn7.elems, bn7.forward)
        breakdown["bn2d_7x7_N256_C2048_bwd"] = entry(5 * bn7.elems * 4, bn7.elems, bn7.backward)
        del bn7
        torch.cuda.empty_cache()
        # configs 1 and 4 fit in the memory-side cache: warm = back to back, cold = after a 512 MB read
        flush = lambda: evict.sum()
        bn1 = BatchNormWorkload((8, 64, 56, 56), SEED + 1)
        bn1.forward()
        parity["C1_bn2d_fwd"] = gate_batchnorm(bn1, backward=False)
        breakdown["C1_bn2d_fwd"] = entry(3 * bn1.elems * 4, bn1.elems, bn1.forward)
        med, mn = _time_events_cold(bn1.forward, flush, it, wu)
        breakdown["C1_bn2d_fwd_cold"] = {
            "bytes": 3 * bn1.elems * 4, "ms_median": med, "ms_min": mn, "GB/s": _gbs(3 * bn1.elems * 4, med),
            "frac_of_peak": _gbs(3 * bn1.elems * 4, med) / HBM_PEAK_GBS,
            "timing": "events around one eager call after a cache-evicting read (2 launches)"}
        bn1.bn.fuse_local = False
        bn1.forward()
        parity["C1_bn2d_fwd_staged"] = gate_batchnorm(bn1, backward=False)
        breakdown["C1_bn2d_fwd_staged"] = entry(3 * bn1.elems * 4, bn1.elems, bn1.forward)
        del bn1
        sm = SoftmaxWorkload((16, 21, 256, 256), SEED + 4)
        sm.forward(), sm.backward()
        parity["C4_softmax"] = gate_softmax(sm)
        breakdown["C4_softmax_fwd"] = entry(2 * sm.elems * 4, sm.elems, sm.forward)
        breakdown["C4_softmax_bwd"] = entry(3 * sm.elems * 4, sm.elems, sm.backward)
        for name, fn, nb in (("fwd", sm.forward, 2), ("bwd", sm.backward, 3)):
            med, mn = _time_events_cold(fn, flush, it, wu)
            breakdown[f"C4_softmax_{name}_cold"] = {
                "bytes": nb * sm.elems * 4, "ms_median": med, "ms_min": mn, "GB/s": _gbs(nb * sm.elems * 4, med),
                "frac_of_peak": _gbs(nb * sm.elems * 4, med) / HBM_PEAK_GBS,
                "timing": "events around one eager call after a cache-evicting read"}
        del sm
        # instance-mode softmax at the same shape, every sample whole on this rank: forward reads x three
        # times and writes y once (max, sum of exponentials, y from x), backward reads y and dy twice
        # and writes dx
        smi = SoftmaxWorkload((16, 21, 256, 256), SEED + 4, instance=True)
        smi.forward(), smi.backward()
        parity["C4_softmax_instance"] = gate_softmax(smi, instance=True)
        breakdown["C4_softmax_instance_fwd"] = entry(4 * smi.elems * 4, smi.elems, smi.forward)
        breakdown["C4_softmax_instance_bwd"] = entry(5 * smi.elems * 4, smi.elems, smi.backward)
        del smi
        torch.cuda.empty_cache()
        shf = ShuffleWorkload((128, 128, 64, 32), SEED + 5)
        parity["C5_shuffle"] = gate_shuffle(shf)
        breakdown["C5_shuffle_fwd"] = entry(4 * shf.elems * 4, shf.elems, shf.forward)
        breakdown["C5_shuffle_bwd"] = entry(4 * shf.elems * 4, shf.elems, shf.backward)
        breakdown["C5_shuffle_round_trip"] = entry(8 * shf.elems * 4, 2 * shf.elems,
                                                   lambda: (shf.forward(), shf.backward()), inner=2)
        breakdown["C5_shuffle_fwd_cold"] = cold_entry(4 * shf.elems * 4, shf.elems, shf.forward)
        breakdown["C5_shuffle_bwd_cold"] = cold_entry(4 * shf.elems * 4, shf.elems, shf.backward)
        breakdown["C5_shuffle_round_trip_cold"] = cold_entry(8 * shf.elems * 4, 2 * shf.elems,
                                                             lambda: (shf.forward(), shf.backward()), inner=1)
        del shf
        torch.cuda.empty_cache()
        # the spatial side with a halo of 1 (what a convolution behind the shuffle needs): the unpack
        # writes rows of 64 floats into rows of 66, the backward pack reads them
        shfh = ShuffleWorkload((128, 128, 64, 32), SEED + 5, dst_overlap=1)
        parity["C5_shuffle_haloed_dst"] = gate_shuffle(shfh)
        breakdown["C5_shuffle_haloed_dst_round_trip"] = entry(8 * shfh.elems * 4, 2 * shfh.elems,
                                                              lambda: (shfh.forward(), shfh.backward()), inner=2)
        del shfh
        torch.cuda.empty_cache()
        # the same tensor between 16 ranks: 256 boxes a direction, one launch each for pack and unpack
        shf16 = ShuffleWorkload((128, 128, 64, 32), SEED + 5, ranks=16, grid=(4, 4))
        parity["C5_shuffle_16ranks"] = gate_shuffle(shf16)
        breakdown["C5_shuffle_16ranks_round_trip"] = entry(8 * shf16.elems * 4, 2 * shf16.elems,
                                                           lambda: (shf16.forward(), shf16.backward()), inner=2)
        del shf16, evict, evict_t, evict_stat
        torch.cuda.empty_cache()

    out = {
        "metric": "achieved HBM GB/s (% of MI355X peak) for BN fwd+bwd and halo pack/unpack",
        "value": value,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": ("C3 batch-norm fwd+bwd NCDHW 4x64x64^3 + C2 halo exchange 3x3x3 "
                         "(8 virtual ranks 2x2x2 periodic, N1 C32 128^3, width 1)"),
            "step_bytes": step_bytes,
            "step_elements": step_elems,
            "seed": SEED,
        },
        "frac_of_hbm_peak": value / HBM_PEAK_GBS,
        "elements_per_s": step_elems / (ms_per_step * 1e-3),
        "kernel_sources": sources_sha,
        "parity_gate": "ok",
        "parity": parity,
        "roofline": roofline,
        "cpu_baseline": None if args.no_cpu_baseline else cpu_baseline(),
        "launches": launches,
        "breakdown": breakdown,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    try:
        sys.exit(main())
    except ParityError as e:
        print(f"bench.py: {e}", file=sys.stderr)
        sys.exit(1)

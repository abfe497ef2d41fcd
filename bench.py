#!/usr/bin/env python3
"""Benchmark of the MI355X DistConv hot path (one GPU).

One "step" is one pass of the path BASELINE.json's metric is quoted on:
  * 3-D batch-norm forward + backward on NCDHW 4 x 64 x 64^3 fp32 (config 3),
  * one full halo exchange (pack + unpack, 3 dimension phases, width 1) of a
    periodic 2 x 2 x 2 grid of virtual ranks, each N1 C32 128^3 fp32 (config 2).
`value` is the algorithmic bytes of a step divided by its wall time, inputs
resident in HBM.  The other BASELINE configs (2-D batch-norm forward, channel
softmax, shuffle) are timed once each and reported under "breakdown".

Prints ONE JSON line.  `--gpus N` with N > 1 exits: this build runs on one GPU.
"""
from __future__ import annotations

import argparse
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
    """Median and minimum milliseconds of one fn() measured with events on the
    current stream (the stream every kernel of fn is launched on).  `inner`
    calls are issued back to back between the two events so that the launch
    latency of a call is hidden behind the execution of the previous one -- the
    reference's harness hides it with a spin kernel
    (legacy/benchmarks/distconv_benchmark_bn.cpp:254-295)."""
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
    """BatchNormalization forward + backward on one rank."""

    def __init__(self, shape_np, seed):
        import torch
        from dihydrogen_amd.layers import BatchNormalization
        from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
        g = torch.Generator(device="cuda").manual_seed(seed)
        nd = len(shape_np)
        c = shape_np[1]
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
        self.bn = BatchNormalization(nd, 0.9, 1e-5)
        self.elems = self.x.get_local_size()

    def forward(self):
        self.bn.forward(self.x, self.mean, self.var, self.rm, self.rv, self.scale, self.bias,
                        self.y, True)

    def backward_reduce(self):
        self.bn.backward_stage1(self.x, self.dy, self.mean, self.var, self.scale, *self.grads)
        self.bn.backward_allreduce(*self.grads)

    def backward_apply(self):
        self.bn.backward_stage2(self.x, self.dy, self.mean, self.var, self.scale, self.grads[2],
                                self.grads[3], self.dx)

    def backward(self):
        self.backward_reduce()
        self.backward_apply()


class HaloWorkload:
    """Halo exchange of a periodic 2 x 2 x 2 grid of virtual ranks."""

    def __init__(self, local_spatial, channels, seed):
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
        self.xch = HaloExchangeVirtual(self.ranks, periodic=True)
        face = (local_spatial + 2) ** 2 * channels
        # per rank: 3 dims x 2 sides x (pack: read+write, unpack: read+write) x 4 bytes
        self.bytes = 8 * 3 * 2 * 2 * 2 * face * 4
        self.elems = 8 * 12 * face

    def run(self):
        self.xch.exchange()


class SoftmaxWorkload:
    def __init__(self, shape_np, seed):
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
        self.sm.setup(self.x, SoftmaxMode.CHANNEL)
        self.elems = self.x.get_local_size()

    def forward(self):
        self.sm.forward(self.x, self.y)

    def backward(self):
        self.sm.backward(self.y, self.dy, self.dx)


class ShuffleWorkload:
    """Sample-parallel (N over 4 ranks) <-> spatial-parallel (H/2 x W/2)."""

    def __init__(self, gshape, seed):
        import torch
        from dihydrogen_amd.layers import TensorShufflerVirtual
        from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
        g = torch.Generator(device="cuda").manual_seed(seed)
        sd, dd = Distribution([1, 1, 1, 4]), Distribution([2, 2, 1, 1])
        self.src = [Tensor(gshape, LocaleVirtual(r, 4), sd).allocate() for r in range(4)]
        self.dst = [Tensor(gshape, LocaleVirtual(r, 4), dd).allocate() for r in range(4)]
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


def cpu_baseline(repeats: int = 9):
    """The CPU oracle (this repository's restatement of the reference kernels;
    the reference has no CPU implementation of batch-norm, softmax or halo
    packing) on the same step: config 3 batch-norm forward+backward plus the
    config 2 exchange for 2 of the 8 virtual ranks' worth of faces."""
    import numpy as np
    import oracle
    lib = oracle.lib()
    lib.orc_num_threads.restype = __import__("ctypes").c_int
    threads = lib.orc_num_threads()
    rng = np.random.default_rng(SEED)
    shp = (4, 64, 64, 64, 64)
    x = rng.standard_normal(shp, dtype=np.float32)
    dy = rng.standard_normal(shp, dtype=np.float32)
    scale = rng.uniform(0.5, 1.5, 64).astype(np.float32)
    bias = (0.1 * rng.standard_normal(64)).astype(np.float32)
    halo_ranks = 2
    fields = [rng.uniform(-1, 1, (1, 32, 130, 130, 130)).astype(np.float32) for _ in range(halo_ranks)]
    bufs = {d: np.empty(oracle.halo_size((130, 130, 130, 32, 1), d, 1), np.float32) for d in range(3)}
    bn_bytes = 8 * x.size * 4
    halo_bytes = halo_ranks * 3 * 2 * 2 * 2 * bufs[0].size * 4

    def step():
        rm, rv = np.zeros(64, np.float32), np.ones(64, np.float32)
        y, mean, var = oracle.bn_forward(x, scale, bias, rm, rv)
        oracle.bn_backward(x, dy, mean, var, scale)
        for f in fields:
            for d in range(3):
                for side in (0, 1):
                    oracle.halo_pack_or_unpack(f, d, side, 1, bufs[d], True)
                    oracle.halo_pack_or_unpack(f, d, side, 1, bufs[d], False)

    step()
    times = []
    for _ in range(repeats):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    t = statistics.median(times)
    return {
        "value": (bn_bytes + halo_bytes) / t / 1e9,
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": (f"config 3 batch-norm fwd+bwd in full (67108864 elems) + config 2 exchange of "
                   f"{halo_ranks} of 8 ranks; median of {repeats} runs, {t:.3f} s each; "
                   f"gcc -O3 -fopenmp, OMP threads = {threads}"),
    }


# HBM traffic per launch measured with rocprofv3 --pmc (profiles/bench_pmc_traffic.txt):
# FETCH_SIZE and WRITE_SIZE in KiB per dispatch; FETCH_SIZE reads 0.5x for full-line
# streaming reads on this stack (calibrated there on a copy of known size), WRITE_SIZE 1.0x.
PMC_KIB = {  # label -> (FETCH_SIZE KiB, fetch scale, WRITE_SIZE KiB) per launch
    "bn_sums": (131095, 2.0, 128),
    "bn_apply": (131102, 2.0, 262162),
    "bn_backprop1": (262182, 2.0, 128),
    "bn_backprop2": (262178, 2.0, 262144),
    "halo_dim0_pack": (154900, 2.0, 16900),    # 8 faces per launch, two launches per step
    "halo_dim0_unpack": (8503, 2.0, 135200),
    "halo_dim1_pack": (21017, 2.0, 33800),
    "halo_dim1_unpack": (16954, 2.0, 37365),
    "halo_dim2_pack": (17048, 2.0, 33800),
    "halo_dim2_unpack": (16956, 2.0, 35112),
}

KERNEL_OF = {
    "bn_sums": "bn_sums_kernel<float,4> (+bn_finish_kernel<float,2>)",
    "bn_statistics": "bn_statistics_kernel<float>",
    "bn_apply": "bn_apply_kernel<float,4>",
    "bn_backprop1": "bn_backprop1_kernel<float,4> (+bn_finish_kernel<float,4>)",
    "bn_backprop2": "bn_backprop2_kernel<float,4>",
    "halo_dim0_pack": "box_copy_kernel<u32,1,OpId,sparse>",
    "halo_dim0_unpack": "box_copy_kernel<u32,1,OpId,sparse>",
    "halo_dim1_pack": "box_copy_kernel<u32,2,OpId>",
    "halo_dim1_unpack": "box_copy_kernel<u32,2,OpId>",
    "halo_dim2_pack": "box_copy_kernel<u32,4,OpId>",
    "halo_dim2_unpack": "box_copy_kernel<u32,4,OpId>",
}


def dim0_study():
    """The dimension-0 phase of the config 2 exchange (one 4-byte element per
    520-byte row and side) as a rate of memory transactions: every packed
    element costs the fetch of a 128-byte line (two neighbouring rows' ends
    share one), every unpacked element a 32-byte masked write.  Timed for
    launch groups of 2, 4 and 8 ranks, pack and unpack alone and together, and
    for the tensor-to-tensor form."""
    from dihydrogen_amd import capi
    from dihydrogen_amd.layers import HaloExchangeAccumOp
    lib = capi.load()
    halo = HaloWorkload(128, 32, SEED + 2)
    xch, dt = halo.xch, halo.ranks[0].h2x_dtype
    rows = 130 * 130 * 32                      # rows of one rank
    lines_per_rank = rows * (1 + 12 / 128)     # one line per row pair end, 12 bytes apart: 9 % straddle
    writes_per_rank = 2 * rows
    ident = HaloExchangeAccumOp.ID

    def faces(group, is_pack):
        out = []
        for r in group:
            for side in (capi.LHS, capi.RHS):
                peer = xch.find_peer_rank(r, 0, side)
                buf = xch._recv_buffer(peer, 0, capi.LHS if side == capi.RHS else capi.RHS) if is_pack \
                    else xch._recv_buffer(r, 0, side)
                out.append(xch._face(r, 0, side, 1, buf, is_pack, False, ident))
        return (capi.HaloFace * len(out))(*out)

    def launch(arr):
        capi.check(lib.h2x_halo_pack_or_unpack_batched(dt, arr, len(arr), None), "halo")

    result = {"rows_per_rank": rows, "lines_per_rank": int(lines_per_rank), "writes_per_rank": writes_per_rank,
              "groups": {}}
    for size in (2, 4, 8):
        groups = [list(range(g, g + size)) for g in range(0, 8, size)]
        packs = [faces(g, True) for g in groups]
        unpacks = [faces(g, False) for g in groups]
        t_pack = _time_events(lambda: [launch(a) for a in packs], 10, 3, inner=2)[0]
        t_unpack = _time_events(lambda: [launch(a) for a in unpacks], 10, 3, inner=2)[0]
        t_both = _time_events(lambda: [(launch(p), launch(u)) for p, u in zip(packs, unpacks)], 10, 3, inner=2)[0]
        result["groups"][str(size)] = {
            "pack_us": t_pack * 1e3, "unpack_us": t_unpack * 1e3, "pack_then_unpack_us": t_both * 1e3,
            "pack_Glines_per_s": 8 * lines_per_rank / (t_pack * 1e-3) / 1e9,
            "pack_line_traffic_GB/s": 8 * lines_per_rank * 128 / (t_pack * 1e-3) / 1e9,
            "unpack_Gwrites_per_s": 8 * writes_per_rank / (t_unpack * 1e-3) / 1e9,
        }
    ov = [1, 0, 0, 0, 0]
    t_fused = _time_events(lambda: xch.exchange(ov, ov, ov, ov, fused=True), 10, 3, inner=2)[0]
    result["fused_us"] = t_fused * 1e3
    result["fused_Gtransactions_per_s"] = 8 * (lines_per_rank + writes_per_rank) / (t_fused * 1e-3) / 1e9
    return result


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-breakdown", action="store_true")
    ap.add_argument("--dim0-study", action="store_true",
                    help="instead of the benchmark: the innermost-dimension halo phase alone, by number of "
                         "ranks per launch group, as cache lines and masked writes per second")
    args = ap.parse_args()
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

    # Every launch of the step is bracketed by a pair of events on the stream it is
    # launched on (torch's current stream, whose handle the C ABI receives).
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
        timed("bn_sums", lambda: b.forward_stage1(bn3.x, bn3.mean, bn3.var, True))
        b.forward_allreduce(bn3.mean, bn3.var, True)
        timed("bn_statistics", lambda: b.sums_to_statistics(nps, bn3.mean, bn3.var, bn3.rm, bn3.rv))
        timed("bn_apply", lambda: b.batch_normalization(bn3.x, bn3.mean, bn3.var, bn3.scale, bn3.bias, bn3.y))
        timed("bn_backprop1", bn3.backward_reduce)
        timed("bn_backprop2", bn3.backward_apply)
        halo.run()

    def kernel_share(evs, steps):
        tot = {}
        for label, pairs in evs.items():
            ms = sum(e0.elapsed_time(e1) for e0, e1 in pairs) / steps  # per step, all launches
            tot[KERNEL_OF[label]] = tot.get(KERNEL_OF[label], 0.0) + ms
        return tot

    # warm-up, with every launch bracketed by events: finds the dominant kernel
    recording[0] = True
    for _ in range(max(args.warmup, 1)):
        step()
    torch.cuda.synchronize()
    share0 = kernel_share(events, max(args.warmup, 1))
    dominant = max(share0, key=share0.get)
    events.clear()

    # timed region: only the dominant kernel's launches carry events
    only[0] = {l for l, k in KERNEL_OF.items() if k == dominant}
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    value = _gbs(step_bytes, ms_per_step)
    dominant_events = dict(events)
    events.clear()

    # a second, fully instrumented pass for the per-launch table
    only[0] = None
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    recording[0] = False
    halo.xch.launch_hook = None
    for label, pairs in dominant_events.items():
        events[label] = pairs  # the dominant kernel's figures come from the timed region

    launches = {}
    for label, pairs in events.items():
        samples = [e0.elapsed_time(e1) for e0, e1 in pairs]
        # the dominant kernel's figure is the average over the timed region; the other launches come
        # from the instrumented pass, where the median keeps a late host enqueue out of the figure
        ms = statistics.mean(samples) if label in dominant_events else statistics.median(samples)
        fetch_kib, scale, write_kib = PMC_KIB.get(label, (0, 0.0, 0))
        launches[label] = {
            "kernel": KERNEL_OF[label], "avg_launch_ms": ms, "algorithmic_bytes": algo_bytes[label],
            "GB/s": _gbs(algo_bytes[label], ms), "frac": _gbs(algo_bytes[label], ms) / HBM_PEAK_GBS,
            "traffic": int((fetch_kib * scale + write_kib) * 1024) if label in PMC_KIB else None,
        }
        if label in faces_per_launch:
            launches[label]["faces"] = faces_per_launch[label]
            launches[label]["launches_per_step"] = 16 // faces_per_launch[label]
    # dominant kernel = the kernel with the largest share of the step's launch time
    share = {}
    for label, v in launches.items():
        share.setdefault(v["kernel"], []).append(label)
    dl = share[dominant]
    d_ms = statistics.mean(launches[l]["avg_launch_ms"] for l in dl)
    d_bytes = statistics.mean(launches[l]["algorithmic_bytes"] for l in dl)
    d_traffic = statistics.mean(launches[l]["traffic"] for l in dl)
    roofline = {
        "kernel": dominant, "launches_per_step": dl, "bound": "hbm",
        "achieved": _gbs(d_bytes, d_ms), "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": _gbs(d_bytes, d_ms) / HBM_PEAK_GBS, "traffic": int(d_traffic),
        "avg_launch_ms": d_ms, "algorithmic_bytes": int(d_bytes),
        "traffic_GB/s": _gbs(d_traffic, d_ms),
    }

    breakdown = {}
    if not args.no_breakdown:
        it, wu = 20, 5

        def entry(nbytes, elems, med, mn):
            return {"bytes": nbytes, "ms_median": med, "ms_min": mn, "GB/s": _gbs(nbytes, med),
                    "frac_of_peak": _gbs(nbytes, med) / HBM_PEAK_GBS, "Gelem/s": elems / (med * 1e-3) / 1e9}

        breakdown["C3_bn3d_fwd"] = entry(3 * S3 * 4, S3, *_time_events(bn3.forward, it, wu))
        breakdown["C3_bn3d_bwd"] = entry(5 * S3 * 4, S3, *_time_events(bn3.backward, it, wu))
        breakdown["C3_bn3d_fwd_bwd"] = entry(
            8 * S3 * 4, S3, *_time_events(lambda: (bn3.forward(), bn3.backward()), it, wu))
        breakdown["C2_halo_8ranks"] = entry(halo.bytes, halo.elems, *_time_events(halo.run, it, wu))
        for d, name in enumerate(("dim0_W", "dim1_H", "dim2_D")):
            ov = [1 if k == d else 0 for k in range(5)]
            fn = lambda ov=ov: halo.xch.exchange(ov, ov, ov, ov)
            breakdown[f"C2_halo_{name}"] = entry(halo.bytes // 3, halo.elems // 3, *_time_events(fn, it, wu))
        # the same exchange as tensor-to-tensor transfers (no buffers): half the bytes per strip
        breakdown["C2_halo_8ranks_fused"] = entry(
            halo.bytes // 2, halo.elems // 2, *_time_events(lambda: halo.xch.exchange(fused=True), it, wu))
        for d, name in enumerate(("dim0_W", "dim1_H", "dim2_D")):
            ov = [1 if k == d else 0 for k in range(5)]
            fn = lambda ov=ov: halo.xch.exchange(ov, ov, ov, ov, fused=True)
            breakdown[f"C2_halo_{name}_fused"] = entry(halo.bytes // 6, halo.elems // 6,
                                                       *_time_events(fn, it, wu))
        yard_x, yard_y = bn3.x.data, bn3.y.data
        breakdown["yardstick_torch_copy_268MB"] = entry(
            2 * S3 * 4, S3, *_time_events(lambda: yard_y.copy_(yard_x), it, wu))
        del bn3, halo, b, yard_x, yard_y
        torch.cuda.empty_cache()
        # configs 1 and 4 fit in the memory-side cache: warm = back to back, cold = after a 512 MB read
        evict = torch.empty(1 << 27, device="cuda").fill_(1.0)
        flush = lambda: evict.sum()
        bn1 = BatchNormWorkload((8, 64, 56, 56), SEED + 1)
        breakdown["C1_bn2d_fwd_warm"] = entry(3 * bn1.elems * 4, bn1.elems, *_time_events(bn1.forward, it, wu))
        breakdown["C1_bn2d_fwd_cold"] = entry(3 * bn1.elems * 4, bn1.elems,
                                              *_time_events_cold(bn1.forward, flush, it, wu))
        del bn1
        sm = SoftmaxWorkload((16, 21, 256, 256), SEED + 4)
        sm.forward()
        breakdown["C4_softmax_fwd"] = entry(2 * sm.elems * 4, sm.elems, *_time_events(sm.forward, it, wu))
        breakdown["C4_softmax_bwd"] = entry(3 * sm.elems * 4, sm.elems, *_time_events(sm.backward, it, wu))
        breakdown["C4_softmax_fwd_cold"] = entry(2 * sm.elems * 4, sm.elems,
                                                 *_time_events_cold(sm.forward, flush, it, wu))
        breakdown["C4_softmax_bwd_cold"] = entry(3 * sm.elems * 4, sm.elems,
                                                 *_time_events_cold(sm.backward, flush, it, wu))
        del sm, evict
        shf = ShuffleWorkload((128, 128, 64, 32), SEED + 5)
        breakdown["C5_shuffle_fwd"] = entry(4 * shf.elems * 4, shf.elems, *_time_events(shf.forward, it, wu))
        breakdown["C5_shuffle_bwd"] = entry(4 * shf.elems * 4, shf.elems, *_time_events(shf.backward, it, wu))

        def round_trip():
            shf.forward()
            shf.backward()

        breakdown["C5_shuffle_round_trip"] = entry(8 * shf.elems * 4, 2 * shf.elems,
                                                   *_time_events(round_trip, it, wu))
        del shf
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
        "roofline": roofline,
        "cpu_baseline": None if args.no_cpu_baseline else cpu_baseline(),
        "launches": launches,
        "breakdown": breakdown,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())

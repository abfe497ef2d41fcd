"""Shared helpers of the test-suite (not collected by pytest)."""
from __future__ import annotations

import numpy as np


def rel_metric(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """The reference's comparison metric, max(|d/v1|, |d/v2|) elementwise
    (legacy/tests/compare_binary_files.cpp:47-49); 0 where both are equal."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    d = np.abs(a - b)
    with np.errstate(divide="ignore", invalid="ignore"):
        m = np.maximum(d / np.abs(a), d / np.abs(b))
    m[d == 0] = 0.0
    return m


def max_rel(a, b) -> float:
    m = rel_metric(a, b)
    return float(np.max(m)) if m.size else 0.0


def bn_inputs(shape_ncs, seed, dtype=np.float32):
    """x ~ N(0,1), dy ~ N(0,1), scale ~ U(0.5,1.5), bias ~ N(0,0.1); shape is
    numpy order (N, C, *spatial)."""
    rng = np.random.default_rng(seed)
    c = shape_ncs[1]
    x = rng.standard_normal(shape_ncs).astype(dtype)
    dy = rng.standard_normal(shape_ncs).astype(dtype)
    scale = rng.uniform(0.5, 1.5, c).astype(dtype)
    bias = (0.1 * rng.standard_normal(c)).astype(dtype)
    return x, dy, scale, bias


# ---------------------------------------------------------------------------
# virtual ranks on the CPU, driven through the oracle
# ---------------------------------------------------------------------------

def global_offset_field(geom, mod=None):
    """Interior of one rank initialised to the global linear offset of each
    element (legacy/tests/tensor/test_halo_exchange_cuda.cu:43-102); returns
    the interior array in numpy order.  With ``mod`` the offset is hashed into
    [0, mod) so that it stays exactly representable in float32."""
    nd = geom.nd
    idx = np.indices(geom.local_shape[::-1], dtype=np.int64)  # numpy order axes
    off = np.zeros(geom.local_shape[::-1], dtype=np.int64)
    stride = 1
    for d in range(nd):
        off += (idx[nd - 1 - d] + geom.global_index[d]) * stride
        stride *= geom.shape[d]
    if mod is not None:
        off = (off * 2654435761) % mod
    return off


def interior_slices(geom):
    return tuple(slice(o, o + l) for o, l in zip(geom.overlap[::-1], geom.local_shape[::-1]))


def oracle_halo_exchange(oracle, geoms, fields, periodic=False, widths=None, is_reverse=False,
                         op=0):
    """HaloExchange::exchange for all virtual ranks on the CPU
    (legacy/include/distconv/tensor/halo_exchange_cuda.hpp:56-106 with the
    message order of halo_exchange_cuda_mpi.hpp:25-100).  ``fields`` are the
    ranks' real (haloed) arrays, modified in place."""
    from oracle import geometry as G
    nd = geoms[0].nd
    for d in range(nd):
        w = geoms[0].overlap[d] if widths is None else widths[d]
        if w == 0 or geoms[0].dist.split_shape[d] <= 1:
            continue
        recv = {}
        for r, g in enumerate(geoms):
            if g.local_size == 0:
                continue
            for side in (0, 1):
                peer = G.halo_peer(g, d, side, periodic)
                if peer is None:
                    continue
                buf = np.zeros(oracle.halo_size(g.real_shape, d, w), fields[r].dtype)
                oracle.halo_pack_or_unpack(fields[r], d, side, w, buf, True, is_reverse, op)
                recv[(peer, 1 - side)] = buf
        for r, g in enumerate(geoms):
            if g.local_size == 0:
                continue
            for side in (0, 1):
                if G.halo_peer(g, d, side, periodic) is None:
                    continue
                oracle.halo_pack_or_unpack(fields[r], d, side, w, recv[(r, side)], False,
                                           is_reverse, op)

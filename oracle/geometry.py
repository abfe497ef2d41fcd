"""Oracle restatement of the reference's tensor geometry and shuffler tables.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  Pure Python integers;
all shapes and indices are innermost first, as in the reference.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Sequence


def rank_to_index(rank: int, locale_shape: Sequence[int]) -> List[int]:
    """Dimension 0 varies fastest.
    legacy/include/distconv/tensor/tensor_mpi.hpp:47-56."""
    idx = []
    for e in locale_shape:
        idx.append(rank % e)
        rank //= e
    return idx


def index_to_rank(idx: Sequence[int], locale_shape: Sequence[int]) -> int:
    """legacy/include/distconv/tensor/tensor_base.hpp:344-361 (get_offset)."""
    r, m = 0, 1
    for i, e in zip(idx, locale_shape):
        r += i * m
        m *= e
    return r


@dataclass
class Dist:
    """legacy/include/distconv/tensor/distribution.hpp:14-33; overlap is
    cleared on dimensions that are not split (:245-251)."""
    locale_shape: List[int]
    split_shape: List[int]
    overlap: List[int]

    def __post_init__(self):
        self.locale_shape = list(self.locale_shape)
        self.split_shape = list(self.split_shape)
        self.overlap = [o if s > 1 else 0 for o, s in zip(self.overlap, self.split_shape)]
        for l, s in zip(self.locale_shape, self.split_shape):
            assert l % s == 0

    def ranks_per_split(self, d: int) -> int:
        return self.locale_shape[d] // self.split_shape[d]

    def is_split_root_dim(self, d: int, rank_idx: int) -> bool:
        return rank_idx % self.ranks_per_split(d) == 0

    def is_split_root(self, idx: Sequence[int]) -> bool:
        return all(self.is_split_root_dim(d, i) for d, i in enumerate(idx))

    @property
    def num_ranks(self) -> int:
        n = 1
        for e in self.locale_shape:
            n *= e
        return n


def split_extent(extent: int, num_splits: int, split_idx: int) -> int:
    """Block partition: the first ``extent % num_splits`` parts get one more.
    legacy/include/distconv/tensor/tensor_mpi.hpp:458-488 (block size 1)."""
    base, rem = divmod(extent, num_splits)
    return base + (1 if split_idx < rem else 0)


class TensorGeom:
    """Geometry of one rank's local part of a distributed tensor
    (tensor_mpi.hpp:436-564: init_local_tensor, init_offsets)."""

    def __init__(self, shape: Sequence[int], dist: Dist, rank: int):
        self.shape = list(shape)
        self.dist = dist
        self.rank = rank
        self.nd = len(shape)
        self.proc_idx = rank_to_index(rank, dist.locale_shape)
        self.split_idx = [p // dist.ranks_per_split(d) for d, p in enumerate(self.proc_idx)]
        self.local_shape = [
            split_extent(self.shape[d], dist.split_shape[d], self.split_idx[d])
            if dist.split_shape[d] > 1 else self.shape[d] for d in range(self.nd)]
        self.overlap = list(dist.overlap)
        self.real_shape = [l + 2 * o for l, o in zip(self.local_shape, self.overlap)]
        # offsets of every rank index along every dimension (init_offsets)
        self.offset_all = []
        for d in range(self.nd):
            offs = []
            for j in range(dist.locale_shape[d]):
                sj = j // dist.ranks_per_split(d)
                if dist.split_shape[d] > 1:
                    offs.append(sum(split_extent(self.shape[d], dist.split_shape[d], k)
                                    for k in range(sj)))
                else:
                    offs.append(0)
            self.offset_all.append(offs)
        self.global_index = [self.offset_all[d][self.proc_idx[d]] for d in range(self.nd)]

    @property
    def is_split_root(self) -> bool:
        return self.dist.is_split_root(self.proc_idx)

    @property
    def local_size(self) -> int:
        n = 1
        for e in self.local_shape:
            n *= e
        return n

    @property
    def real_size(self) -> int:
        n = 1
        for e in self.real_shape:
            n *= e
        return n

    def strides(self) -> List[int]:
        """legacy/include/distconv/tensor/tensor.hpp:291-298."""
        s, out = 1, []
        for e in self.real_shape:
            out.append(s)
            s *= e
        return out

    def base_offset(self) -> int:
        """Offset of the first interior element (get_base_ptr)."""
        return sum(o * s for o, s in zip(self.overlap, self.strides()))

    def dimension_rank_offset(self, d: int, rank_idx: int) -> int:
        return self.offset_all[d][rank_idx]

    def remote_dimension(self, d: int, rank_idx: int) -> int:
        """tensor.hpp:322-335."""
        off = self.offset_all[d][rank_idx]
        nxt = self.shape[d]
        for k in range(rank_idx + 1, self.dist.locale_shape[d]):
            if self.dist.is_split_root_dim(d, k):
                nxt = self.offset_all[d][k]
                break
        return nxt - off


def _intersect(a0, ae, b0, be):
    """Region::intersect, legacy/include/distconv/tensor/tensor_base.hpp:515-567."""
    size = 1
    for x0, xe, y0, ye in zip(a0, ae, b0, be):
        lo = max(x0, y0)
        hi = min(x0 + xe, y0 + ye)
        size *= max(hi - lo, 0)
    return size


def rank_limits(src: TensorGeom, dst: TensorGeom, optimize: bool = False) -> List[int]:
    """setup_rank_limits (+ optimize_find_destination when ``optimize``),
    legacy/include/distconv/tensor/shuffle_mpi_cuda.hpp:129-213."""
    out: List[int] = []
    for d in range(src.nd):
        ld = dst.dist.locale_shape[d]
        start = len(out)
        for j in range(ld):
            nxt = dst.shape[d]
            for k in range(j + 1, ld):
                if dst.dist.is_split_root_dim(d, k):
                    nxt = dst.dimension_rank_offset(d, k)
                    break
            if nxt < src.global_index[d]:
                lim = 0
            else:
                lim = min(nxt - src.global_index[d], src.local_shape[d])
            out.append(lim)
        if optimize:
            ref = dst.local_shape[d]
            even = all(dst.remote_dimension(d, j) == ref for j in range(ld))
            if even and ld >= 16:
                out[start] = -1
                out[start + 1] = src.global_index[d]
                out[start + 2] = ref
    return out


def counts_and_displs(src: TensorGeom, dst: TensorGeom):
    """setup_displs, shuffle_mpi_cuda.hpp:215-287.  Returns
    (send_counts, send_displs, recv_counts, recv_displs) for ``src.rank``
    (== ``dst.rank``: one process holds one part of each tensor)."""
    assert src.rank == dst.rank
    nranks = src.dist.num_ranks
    sc, sd, rc, rd = [], [], [], []
    cs = cr = 0
    for pid in range(nranks):
        sd.append(cs)
        rd.append(cr)
        dpi = rank_to_index(pid, dst.dist.locale_shape)
        if src.is_split_root and dst.dist.is_split_root(dpi):
            r0 = [dst.dimension_rank_offset(d, dpi[d]) for d in range(dst.nd)]
            re = [dst.remote_dimension(d, dpi[d]) for d in range(dst.nd)]
            sc.append(_intersect(src.global_index, src.local_shape, r0, re))
        else:
            sc.append(0)
        cs += sc[-1]
        spi = rank_to_index(pid, src.dist.locale_shape)
        if dst.is_split_root and src.dist.is_split_root(spi):
            r0 = [src.dimension_rank_offset(d, spi[d]) for d in range(src.nd)]
            re = [src.remote_dimension(d, spi[d]) for d in range(src.nd)]
            rc.append(_intersect(dst.global_index, dst.local_shape, r0, re))
        else:
            rc.append(0)
        cr += rc[-1]
    return sc, sd, rc, rd


def halo_peer(t: TensorGeom, d: int, side: int, periodic: bool = False):
    """find_peer_rank, legacy/include/distconv/tensor/halo_exchange_cuda.hpp:322-357
    (side: 0 LHS, 1 RHS).  ``periodic`` wraps at the grid edge, which the
    reference never does (it returns MPI_PROC_NULL there)."""
    if not (t.dist.split_shape[d] > 1 and t.overlap[d] > 0 and t.local_size > 0):
        return None
    p = t.proc_idx[d] + (1 if side == 1 else -1)
    n = t.dist.locale_shape[d]
    if p < 0 or p >= n:
        if not periodic:
            return None
        p %= n
    idx = list(t.proc_idx)
    idx[d] = p
    if not periodic and t.dimension_rank_offset(d, p) == t.shape[d]:
        return None
    return index_to_rank(idx, t.dist.locale_shape)

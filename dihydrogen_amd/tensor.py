"""Host-side tensor model for the Python binding: distributions, virtual
locales and distributed tensors whose local parts live in torch device memory.

Mirrors the part of DistConv's tensor model the hot path is written against
(legacy/include/distconv/tensor/distribution.hpp, tensor.hpp, tensor_mpi.hpp)
with one change: the locale is *virtual* -- a (rank, size) pair without a
communicator -- so several ranks' local tensors can live on one GPU.  Shapes
and indices are innermost first, as in the reference; torch views use the
reversed (outermost first) order.
"""
from __future__ import annotations

import math
from typing import Iterable, List, Optional, Sequence

import torch

from . import capi


def _prod(values: Iterable[int]) -> int:
    return math.prod(int(v) for v in values)


class Distribution:
    """legacy/include/distconv/tensor/distribution.hpp:14-275."""

    def __init__(self, locale_shape: Sequence[int], split_shape: Optional[Sequence[int]] = None,
                 overlap: Optional[Sequence[int]] = None):
        self.locale_shape = [int(v) for v in locale_shape]
        self.split_shape = list(self.locale_shape) if split_shape is None else [int(v) for v in split_shape]
        nd = len(self.locale_shape)
        ov = [0] * nd if overlap is None else [int(v) for v in overlap]
        if len(self.split_shape) != nd or len(ov) != nd:
            raise ValueError("locale shape, split shape and overlap must have the same length")
        for l, s in zip(self.locale_shape, self.split_shape):
            if s < 1 or l % s != 0:
                raise ValueError(f"locale extent {l} is not divisible by split extent {s}")
        # halo only where the dimension is actually split (distribution.hpp:245-251)
        self.overlap = [o if s > 1 else 0 for o, s in zip(ov, self.split_shape)]

    # factories, named as in the reference (distribution.hpp:54-95)
    @staticmethod
    def make_localized_distribution(num_dims: int) -> "Distribution":
        return Distribution([1] * num_dims)

    @staticmethod
    def make_distribution(locale_shape: Sequence[int]) -> "Distribution":
        return Distribution(locale_shape)

    @staticmethod
    def make_overlapped_distribution(locale_shape, overlap) -> "Distribution":
        return Distribution(locale_shape, locale_shape, overlap)

    @staticmethod
    def make_shared_distribution(locale_shape, split_shape=None) -> "Distribution":
        return Distribution(locale_shape, [1] * len(locale_shape) if split_shape is None else split_shape)

    @property
    def num_dims(self) -> int:
        return len(self.locale_shape)

    @property
    def num_ranks(self) -> int:
        return _prod(self.locale_shape)

    def get_num_ranks_per_split(self, dim: int) -> int:
        return self.locale_shape[dim] // self.split_shape[dim]

    def is_distributed(self, dim: int) -> bool:
        return self.split_shape[dim] > 1

    def is_split_root_index(self, rank_index: Sequence[int]) -> bool:
        return all(r % self.get_num_ranks_per_split(d) == 0 for d, r in enumerate(rank_index))

    def rank_index(self, rank: int) -> List[int]:
        """rank -> grid index, dimension 0 fastest (tensor_mpi.hpp:47-56)."""
        out = []
        for extent in self.locale_shape:
            rank, r = divmod(rank, extent)
            out.append(r)
        return out

    def rank_of(self, rank_index: Sequence[int]) -> int:
        rank = 0
        for extent, r in zip(reversed(self.locale_shape), reversed(list(rank_index))):
            rank = rank * extent + r
        return rank

    def __eq__(self, other):
        return (isinstance(other, Distribution) and self.locale_shape == other.locale_shape
                and self.split_shape == other.split_shape and self.overlap == other.overlap)


class LocaleVirtual:
    """Stands in for LocaleMPI (tensor_mpi.hpp:16-90): a rank among `size`
    ranks that all live in this process."""

    def __init__(self, rank: int, size: int):
        if not 0 <= rank < size:
            raise ValueError("rank out of range")
        self.rank, self.size = rank, size

    def get_rank(self) -> int:
        return self.rank

    def get_size(self) -> int:
        return self.size


def _block_start(extent: int, parts: int, index: int) -> int:
    """First element of part `index` when `extent` is cut into `parts` blocks,
    the first extent % parts of which are one longer (tensor_mpi.hpp:458-488)."""
    base, rem = divmod(extent, parts)
    return index * base + min(index, rem)


_TORCH_DTYPES = {torch.float32: capi.F32, torch.float64: capi.F64}


class Tensor:
    """Tensor<DataType, LocaleVirtual, device allocator>: global shape plus
    distribution; `allocate()` creates the local real (haloed) buffer."""

    def __init__(self, shape: Sequence[int], locale: LocaleVirtual, dist: Distribution,
                 dtype: torch.dtype = torch.float32, device: str = "cuda"):
        self.shape = [int(v) for v in shape]
        if len(self.shape) != dist.num_dims:
            raise ValueError("shape and distribution disagree on the number of dimensions")
        if dist.num_ranks != locale.size:
            raise ValueError("distribution does not cover the locale")
        self.locale, self.dist, self.dtype, self.device = locale, dist, dtype, device
        self.proc_index = dist.rank_index(locale.rank)
        self.split_index = [p // dist.get_num_ranks_per_split(d) for d, p in enumerate(self.proc_index)]
        self.global_index, self.local_shape = [], []
        for d, extent in enumerate(self.shape):
            parts = dist.split_shape[d]
            if parts > 1:
                lo = _block_start(extent, parts, self.split_index[d])
                hi = _block_start(extent, parts, self.split_index[d] + 1)
            else:
                lo, hi = 0, extent
            self.global_index.append(lo)
            self.local_shape.append(hi - lo)
        self.overlap = list(dist.overlap)
        self.local_real_shape = [l + 2 * o for l, o in zip(self.local_shape, self.overlap)]
        self.data: Optional[torch.Tensor] = None

    # -- geometry ------------------------------------------------------------
    def get_num_dims(self) -> int:
        return len(self.shape)

    def get_local_size(self) -> int:
        return _prod(self.local_shape)

    def get_local_real_size(self) -> int:
        return _prod(self.local_real_shape)

    def is_split_root(self) -> bool:
        return self.dist.is_split_root_index(self.proc_index)

    def get_strides(self) -> List[int]:
        """tensor.hpp:291-298."""
        out, s = [], 1
        for extent in self.local_real_shape:
            out.append(s)
            s *= extent
        return out

    def get_dimension_rank_offset(self, dim: int, rank_index: int) -> int:
        parts = self.dist.split_shape[dim]
        if parts == 1:
            return 0
        return _block_start(self.shape[dim], parts, rank_index // self.dist.get_num_ranks_per_split(dim))

    def get_remote_dimension(self, dim: int, rank_index: int) -> int:
        parts = self.dist.split_shape[dim]
        if parts == 1:
            return self.shape[dim]
        si = rank_index // self.dist.get_num_ranks_per_split(dim)
        return _block_start(self.shape[dim], parts, si + 1) - _block_start(self.shape[dim], parts, si)

    def base_offset(self) -> int:
        return sum(o * s for o, s in zip(self.overlap, self.get_strides()))

    @property
    def h2x_dtype(self) -> int:
        return _TORCH_DTYPES[self.dtype]

    # -- storage -------------------------------------------------------------
    def allocate(self) -> "Tensor":
        self.data = torch.zeros(max(self.get_local_real_size(), 1), dtype=self.dtype, device=self.device)
        return self

    def get_buffer(self) -> int:
        """Device address of the real allocation (tensor.hpp:449-460)."""
        return self.data.data_ptr()

    def get_base_ptr(self) -> int:
        """Device address of the first interior element (tensor.hpp:462-481)."""
        return self.data.data_ptr() + self.base_offset() * self.data.element_size()

    def real_view(self) -> torch.Tensor:
        """The real local tensor as a torch view, outermost dimension first."""
        n = self.get_local_real_size()
        return self.data[:n].view(*reversed(self.local_real_shape))

    def interior_view(self) -> torch.Tensor:
        v = self.real_view()
        for axis, (o, l) in enumerate(zip(reversed(self.overlap), reversed(self.local_shape))):
            v = v.narrow(axis, o, l)
        return v

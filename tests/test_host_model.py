"""Host-side tensor model and shuffler tables of the Python binding against
the oracle's independent restatement, on CPU (no buffers are allocated)."""
import itertools

import numpy as np
import pytest

from oracle import geometry as G
from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor

CASES = [
    ((8, 8, 2, 4), (2, 2, 1, 1), None, (1, 1, 0, 0)),
    ((11, 7, 3, 5), (2, 2, 1, 1), None, None),
    ((13, 9, 5, 3, 6), (3, 1, 2, 1, 2), None, (2, 1, 1, 0, 0)),
    ((8, 8, 2, 4), (2, 2, 1, 1), (2, 1, 1, 1), None),
    ((8, 8, 2, 8), (4, 2, 1, 2), (2, 2, 1, 1), (1, 0, 0, 0)),
    ((2, 8, 2, 4), (4, 1, 1, 1), None, None),
]


@pytest.mark.parametrize("shape,locale,split,overlap", CASES)
def test_partition_matches_oracle(shape, locale, split, overlap):
    nd, n = len(shape), int(np.prod(locale))
    dist = Distribution(locale, split, overlap)
    od = G.Dist(locale, split or locale, overlap or [0] * nd)
    for r in range(n):
        t = Tensor(shape, LocaleVirtual(r, n), dist)
        g = G.TensorGeom(shape, od, r)
        assert t.proc_index == g.proc_idx and t.split_index == g.split_idx
        assert t.local_shape == g.local_shape and t.local_real_shape == g.real_shape
        assert t.global_index == g.global_index and t.get_strides() == g.strides()
        assert t.base_offset() == g.base_offset() and t.is_split_root() == g.is_split_root
        for d in range(nd):
            for j in range(locale[d]):
                assert t.get_dimension_rank_offset(d, j) == g.dimension_rank_offset(d, j)
                assert t.get_remote_dimension(d, j) == g.remote_dimension(d, j)
        assert dist.rank_of(t.proc_index) == r == G.index_to_rank(g.proc_idx, locale)


def test_block_partition_rule():
    """extent 11 over 4 parts: 3 3 3 2 (tensor_mpi.hpp:468-482)."""
    dist = Distribution([4, 1, 1, 1])
    sizes = [Tensor([11, 2, 2, 2], LocaleVirtual(r, 4), dist).local_shape[0] for r in range(4)]
    starts = [Tensor([11, 2, 2, 2], LocaleVirtual(r, 4), dist).global_index[0] for r in range(4)]
    assert sizes == [3, 3, 3, 2] and starts == [0, 3, 6, 9]


def test_overlap_only_on_split_dimensions():
    d = Distribution.make_overlapped_distribution([2, 1, 1, 1], [1, 1, 0, 0])
    assert d.overlap == [1, 0, 0, 0]  # distribution.hpp:245-251
    with pytest.raises(ValueError):
        Distribution([4, 1], [3, 1])


@pytest.mark.parametrize("src,dst", list(itertools.permutations(range(len(CASES) - 2), 2))[:6])
def test_shuffler_tables_match_oracle(src, dst):
    from dihydrogen_amd.layers import TensorShufflerVirtual as S
    shape = (8, 8, 2, 4)
    specs = [((2, 2, 1, 1), None, (1, 1, 0, 0)), ((1, 1, 1, 4), None, None), ((4, 1, 1, 1), None, None),
             ((2, 2, 1, 1), (2, 1, 1, 1), None)]
    (sl, ss, so), (dl, ds, do) = specs[src % 4], specs[dst % 4]
    n = int(np.prod(sl))
    if int(np.prod(dl)) != n:
        pytest.skip("rank counts differ")
    sd, dd = Distribution(sl, ss, so), Distribution(dl, ds, do)
    for r in range(n):
        a, b = Tensor(shape, LocaleVirtual(r, n), sd), Tensor(shape, LocaleVirtual(r, n), dd)
        ga = G.TensorGeom(shape, G.Dist(sl, ss or sl, so or [0] * 4), r)
        gb = G.TensorGeom(shape, G.Dist(dl, ds or dl, do or [0] * 4), r)
        assert S.rank_limits(a, b) == G.rank_limits(ga, gb)
        assert S.rank_limits(b, a) == G.rank_limits(gb, ga)
        sc, _, rc, _ = G.counts_and_displs(ga, gb)
        shuffler = S.__new__(S)
        shuffler.num_ranks = n
        assert shuffler._counts(a, b) == sc and shuffler._counts(b, a) == rc


def test_halo_exchange_rank_groups():
    """The innermost-dimension phase of a large exchange is split into groups
    of ranks: every group is closed under the neighbour relation along that
    dimension, the groups partition the ranks, and small or dense phases stay
    one group."""
    from dihydrogen_amd.layers import HaloExchangeVirtual as H

    def make(gshape, locale, overlap):
        dist = Distribution.make_overlapped_distribution(locale, overlap)
        n = int(np.prod(locale))
        x = H.__new__(H)
        x.tensors = [Tensor(gshape, LocaleVirtual(r, n), dist) for r in range(n)]
        x.dist, x.periodic = dist, True
        return x

    big = make((256, 256, 256, 32, 1), (2, 2, 2, 1, 1), (1, 1, 1, 0, 0))
    groups = big._rank_groups(0, 1)
    assert sorted(sum(groups, [])) == list(range(8)) and len(groups) == 4  # 138 MB of lines per pair
    for g in groups:
        for r in g:
            idx = list(big.tensors[r].proc_index)
            for p in range(2):  # every rank of the line along dimension 0 is in the group
                idx[0] = p
                assert big.dist.rank_of(idx) in g
    assert big._rank_groups(1, 1) == [list(range(8))]
    assert big._rank_groups(2, 1) == [list(range(8))]
    assert big._rank_groups(0, 32) == [list(range(8))]  # 128-byte runs are not sparse
    small = make((16, 16, 16, 4, 1), (2, 2, 2, 1, 1), (1, 1, 1, 0, 0))
    assert small._rank_groups(0, 1) == [list(range(8))]
    # a line of four ranks along dimension 0 is never split, whatever its size
    line = make((1024, 512, 256, 32, 1), (4, 1, 1, 1, 1), (1, 0, 0, 0, 0))
    assert line._rank_groups(0, 1) == [list(range(4))]

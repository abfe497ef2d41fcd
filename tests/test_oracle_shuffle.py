"""Pins the shuffler functions and tables of the CPU oracle with the closed
form of the reference's own tests (legacy/tests/tensor/test_tensor_mpi_shuffle.cpp:26-154):
every element carries its global offset, after shuffle_forward every element
of every destination rank holds its own global offset, and shuffle_backward
restores the source.  The all-to-all between the per-rank buffers is done here
in numpy with the reference's counts and displacements (MPI_Alltoallv,
legacy/include/distconv/tensor/shuffle_mpi.hpp:595-608)."""
import numpy as np
import pytest

import oracle
from oracle import geometry as G
from helpers import global_offset_field, interior_slices

CASES = {
    "same_distribution": ((8, 8, 2, 4), ((2, 2, 1, 1), None, None), ((2, 2, 1, 1), None, None)),
    "sample_to_spatial": ((8, 8, 2, 4), ((1, 1, 1, 4), None, None), ((2, 2, 1, 1), None, None)),
    "sample_to_spatial_halo": ((8, 8, 2, 4), ((1, 1, 1, 4), None, None), ((2, 2, 1, 1), None, (1, 1, 0, 0))),
    "overlap_to_nonoverlap": ((8, 8, 2, 4), ((2, 2, 1, 1), None, (1, 2, 0, 0)), ((2, 2, 1, 1), None, None)),
    "uneven": ((11, 7, 3, 5), ((1, 1, 1, 4), None, None), ((2, 2, 1, 1), None, None)),
    "shrink_split_shared": ((8, 8, 2, 4), ((2, 2, 1, 1), None, None), ((2, 2, 1, 1), (2, 1, 1, 1), None)),
    "five_d": ((6, 8, 4, 2, 4), ((1, 1, 1, 1, 4), None, None), ((1, 2, 2, 1, 1), None, (0, 1, 1, 0, 0))),
    "sixteen_ranks_even": ((32, 4, 2, 16), ((1, 1, 1, 16), None, None), ((16, 1, 1, 1), None, None)),
    "empty_ranks": ((2, 8, 2, 4), ((1, 1, 1, 4), None, None), ((4, 1, 1, 1), None, None)),
}


def _geoms(case):
    shape, (sl, ss, so), (dl, ds, do) = CASES[case]
    nd, n = len(shape), int(np.prod(sl))
    src = [G.TensorGeom(shape, G.Dist(sl, ss or sl, so or [0] * nd), r) for r in range(n)]
    dst = [G.TensorGeom(shape, G.Dist(dl, ds or dl, do or [0] * nd), r) for r in range(n)]
    return src, dst


def _shuffle(src_g, dst_g, src_fields, dst_fields, optimize=False):
    """shuffle() of legacy/src/tensor/shuffle_mpi_cuda.cu:378-476 for all ranks."""
    n = len(src_g)
    tables = [G.counts_and_displs(src_g[r], dst_g[r]) for r in range(n)]
    send = []
    for r in range(n):
        buf = np.zeros(max(src_g[r].local_size, 1), src_fields[r].dtype)
        if src_g[r].is_split_root and src_g[r].local_size:
            flat = src_fields[r].reshape(-1)[src_g[r].base_offset():]
            oracle.shuffle_pack_or_unpack(flat, src_g[r].local_shape, src_g[r].strides(),
                                          dst_g[r].dist.locale_shape,
                                          G.rank_limits(src_g[r], dst_g[r], optimize), buf,
                                          tables[r][1], True)
        send.append(buf)
    for r in range(n):
        sc_r, sd_r, rc_r, rd_r = tables[r]
        recv = np.zeros(max(dst_g[r].local_size, 1), dst_fields[r].dtype)
        for p in range(n):
            cnt = rc_r[p]
            assert cnt == tables[p][0][r]
            recv[rd_r[p]:rd_r[p] + cnt] = send[p][tables[p][1][r]:tables[p][1][r] + cnt]
        if dst_g[r].is_split_root and dst_g[r].local_size:
            flat = dst_fields[r].reshape(-1)[dst_g[r].base_offset():]
            oracle.shuffle_pack_or_unpack(flat, dst_g[r].local_shape, dst_g[r].strides(),
                                          src_g[r].dist.locale_shape,
                                          G.rank_limits(dst_g[r], src_g[r], optimize), recv, rd_r, False)


@pytest.mark.parametrize("optimize", [False, True])
@pytest.mark.parametrize("case", list(CASES))
def test_closed_form_round_trip(case, optimize):
    src_g, dst_g = _geoms(case)
    src_f = []
    for g in src_g:
        f = np.full(g.real_shape[::-1], -1, np.float32)
        f[interior_slices(g)] = global_offset_field(g)
        src_f.append(f)
    dst_f = [np.full(g.real_shape[::-1], -7, np.float32) for g in dst_g]
    _shuffle(src_g, dst_g, src_f, dst_f, optimize)
    for g, f in zip(dst_g, dst_f):
        if g.is_split_root and g.local_size:
            assert np.array_equal(f[interior_slices(g)], global_offset_field(g).astype(np.float32))
    back = [np.full(g.real_shape[::-1], -1, np.float32) for g in src_g]
    _shuffle(dst_g, src_g, dst_f, back, optimize)
    for g, a, b in zip(src_g, src_f, back):
        if g.is_split_root:
            assert np.array_equal(a, b)


def test_tables_match_hand_computation():
    """N split over 4 -> H/2 x W/2 on an 8 x 8 x 2 x 4 tensor, rank 1."""
    src_g, dst_g = _geoms("sample_to_spatial")
    s, d = src_g[1], dst_g[1]
    assert s.local_shape == [8, 8, 2, 1] and s.global_index == [0, 0, 0, 1]
    assert d.local_shape == [4, 4, 2, 4] and d.global_index == [4, 0, 0, 0]   # rank 1 = (pw 1, ph 0)
    assert G.rank_limits(s, d) == [4, 8, 4, 8, 2, 1]  # W | H | C | N
    sc, sd, rc, rd = G.counts_and_displs(s, d)
    assert sc == [32, 32, 32, 32] and sd == [0, 32, 64, 96]
    assert rc == [32, 32, 32, 32] and rd == [0, 32, 64, 96]
    # uneven: 11 = 6 + 5 (first rem ranks get one more, tensor_mpi.hpp:468-482)
    _, dst_u = _geoms("uneven")
    assert [g.local_shape[0] for g in dst_u] == [6, 5, 6, 5]
    assert [g.local_shape[1] for g in dst_u] == [4, 4, 3, 3]


def test_find_destination_brute_force():
    """Per-element destination of the oracle vs. a direct search of which
    destination rank owns the element's global index."""
    src_g, dst_g = _geoms("uneven")
    for r in (0, 3):
        s = src_g[r]
        field = np.arange(s.local_size, dtype=np.float32)
        sc, sd, _, _ = G.counts_and_displs(s, dst_g[r])
        buf = np.full(s.local_size, -1, np.float32)
        oracle.shuffle_pack_or_unpack(field, s.local_shape, s.strides(), dst_g[r].dist.locale_shape,
                                      G.rank_limits(s, dst_g[r]), buf, sd, True)
        # walk destination ranks and their intersections in natural order
        pos = 0
        for p, d in enumerate(dst_g):
            lo = [max(a, b) for a, b in zip(s.global_index, d.global_index)]
            hi = [min(a + la, b + lb) for a, la, b, lb in zip(s.global_index, s.local_shape, d.global_index, d.local_shape)]
            ext = [max(h - l, 0) for l, h in zip(lo, hi)]
            assert int(np.prod(ext)) == sc[p] and pos == sd[p]
            for i3 in range(ext[3]):
                for i2 in range(ext[2]):
                    for i1 in range(ext[1]):
                        for i0 in range(ext[0]):
                            gi = [lo[0] + i0, lo[1] + i1, lo[2] + i2, lo[3] + i3]
                            li = [a - b for a, b in zip(gi, s.global_index)]
                            off = sum(x * st for x, st in zip(li, s.strides()))
                            assert buf[pos] == field[off]
                            pos += 1
        assert pos == s.local_size


def test_row_copy_pack_equals_generic_pack():
    for case in ("sample_to_spatial", "uneven", "spatial"):
        if case == "spatial":
            shape, sl, dl = (12, 8, 3, 4), (2, 1, 1, 2), (1, 2, 2, 1)
            src_g = [G.TensorGeom(shape, G.Dist(sl, sl, [0] * 4), r) for r in range(4)]
            dst_g = [G.TensorGeom(shape, G.Dist(dl, dl, [0] * 4), r) for r in range(4)]
        else:
            src_g, dst_g = _geoms(case)
        for r, s in enumerate(src_g):
            rng = np.random.default_rng(r)
            field = rng.standard_normal(s.local_size).astype(np.float32)
            lim = G.rank_limits(s, dst_g[r])
            _, sd, _, _ = G.counts_and_displs(s, dst_g[r])
            a = np.zeros(s.local_size, np.float32)
            b = np.zeros(s.local_size, np.float32)
            oracle.shuffle_pack_or_unpack(field, s.local_shape, s.strides(), dst_g[r].dist.locale_shape, lim, a, sd, True)
            oracle.shuffle_pack_rows4(field, s.local_shape, dst_g[r].dist.locale_shape, lim, b, sd)
            assert np.array_equal(a, b)
            c = np.zeros(s.local_size, np.float32)
            oracle.shuffle_pack_or_unpack(field, s.local_shape, s.strides(), dst_g[r].dist.locale_shape, lim, c, sd, True, parallel=True)
            assert np.array_equal(a, c)


def test_row_copy_of_any_rank_equals_the_generic_path():
    """orc_shuffle_rows (the structure of pack_sample_to_spatial4/5 and
    unpack_sample_to_spatial[_halo4/5], shuffle_mpi.hpp:708-849,874-947) against
    the per-element pack / unpack on the same tables: 4-D and 5-D, uneven splits,
    and a haloed destination for the unpack (rows land inside the halo frame,
    the frame itself is not touched)."""
    cases = [
        ((8, 8, 2, 4), (1, 1, 1, 4), (2, 2, 1, 1), None),
        ((11, 7, 3, 5), (1, 1, 1, 4), (2, 2, 1, 1), None),
        ((8, 8, 2, 4), (1, 1, 1, 4), (2, 2, 1, 1), (1, 1, 0, 0)),
        ((6, 8, 4, 2, 4), (1, 1, 1, 1, 4), (1, 2, 2, 1, 1), (0, 1, 1, 0, 0)),
        ((7, 5, 6, 3, 8), (1, 1, 1, 1, 8), (2, 2, 2, 1, 1), None),
    ]
    for shape, sl, dl, halo in cases:
        nd, n = len(shape), int(np.prod(sl))
        src_g = [G.TensorGeom(shape, G.Dist(sl, sl, [0] * nd), r) for r in range(n)]
        dst_g = [G.TensorGeom(shape, G.Dist(dl, dl, list(halo) if halo else [0] * nd), r) for r in range(n)]
        for r in range(n):
            s, d = src_g[r], dst_g[r]
            rng = np.random.default_rng(100 + r)
            # pack on the source side
            field = rng.standard_normal(s.real_size).astype(np.float32)
            lim = G.rank_limits(s, d)
            _, sd, _, rd = G.counts_and_displs(s, d)
            a, b = np.zeros(s.local_size, np.float32), np.zeros(s.local_size, np.float32)
            base = s.base_offset()
            oracle.shuffle_pack_or_unpack(field[base:], s.local_shape, s.strides(), d.dist.locale_shape, lim, a, sd, True)
            oracle.shuffle_rows(field[base:], s.local_shape, s.strides(), d.dist.locale_shape, lim, b, sd, True)
            assert np.array_equal(a, b)
            # unpack on the destination side (haloed or not)
            lim_d = G.rank_limits(d, s)
            buf = rng.standard_normal(d.local_size).astype(np.float32)
            t1 = np.full(d.real_size, -5.0, np.float32)
            t2 = t1.copy()
            base = d.base_offset()
            oracle.shuffle_pack_or_unpack(t1[base:], d.local_shape, d.strides(), s.dist.locale_shape, lim_d, buf, rd, False)
            oracle.shuffle_rows(t2[base:], d.local_shape, d.strides(), s.dist.locale_shape, lim_d, buf, rd, False)
            assert np.array_equal(t1, t2)
            assert (t2 == -5.0).sum() == d.real_size - d.local_size   # only the interior was written

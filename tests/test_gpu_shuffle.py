"""GPU parity: tensor-shuffler pack/unpack, bit-exact.

Follows legacy/tests/tensor/test_tensor_mpi_shuffle.cpp and
test_tensor_mpi_cuda_shuffle.cu: every element is initialised to its global
linear offset, the tensor is shuffled to another distribution and every local
element of every destination rank must hold its own global offset; shuffling
back must restore the source.  Single-rank pack/unpack calls are additionally
compared with the oracle's per-element restatement on the reference's own
buffer layout.
"""
import ctypes

import numpy as np
import pytest

from helpers import global_offset_field, interior_slices

pytestmark = pytest.mark.gpu

# (shape, src (locale, split, overlap), dst (locale, split, overlap)); innermost first
CASES = {
    "same_distribution": ((8, 8, 2, 4), ((2, 2, 1, 1), None, None), ((2, 2, 1, 1), None, None)),
    "sample_to_spatial": ((8, 8, 2, 4), ((1, 1, 1, 4), None, None), ((2, 2, 1, 1), None, None)),
    "sample_to_spatial_halo": ((8, 8, 2, 4), ((1, 1, 1, 4), None, None), ((2, 2, 1, 1), None, (1, 1, 0, 0))),
    "overlap_to_nonoverlap": ((8, 8, 2, 4), ((2, 2, 1, 1), None, (1, 2, 0, 0)), ((2, 2, 1, 1), None, None)),
    "spatial_to_other_spatial": ((12, 8, 2, 4), ((4, 1, 1, 1), None, None), ((1, 2, 1, 2), None, None)),
    "uneven": ((11, 7, 3, 5), ((1, 1, 1, 4), None, None), ((2, 2, 1, 1), None, None)),
    "shrink_split_shared": ((8, 8, 2, 4), ((2, 2, 1, 1), None, None), ((2, 2, 1, 1), (2, 1, 1, 1), None)),
    "five_d": ((6, 8, 4, 2, 4), ((1, 1, 1, 1, 4), None, None), ((1, 2, 2, 1, 1), None, (0, 1, 1, 0, 0))),
    "sixteen_ranks_even": ((32, 4, 2, 16), ((1, 1, 1, 16), None, None), ((16, 1, 1, 1), None, None)),
    "empty_ranks": ((2, 8, 2, 4), ((1, 1, 1, 4), None, None), ((4, 1, 1, 1), None, None)),
    # runs of 19 and 18 elements (and 37 when rows are whole): 16-byte vectors with straddlers
    "odd_runs": ((37, 6, 3, 4), ((1, 1, 1, 4), None, None), ((2, 2, 1, 1), None, None)),
    "odd_runs_halo": ((37, 5, 2, 4), ((1, 1, 1, 4), None, None), ((2, 2, 1, 1), None, (1, 1, 0, 0))),
}


def _build(case, torch_dtype, np_dtype, mod=None):
    import torch
    from oracle import geometry as G
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    shape, (sl, ss, so), (dl, ds, do) = CASES[case]
    nd = len(shape)
    n = int(np.prod(sl))
    sdist = Distribution(sl, ss, so)
    ddist = Distribution(dl, ds, do)
    src = [Tensor(shape, LocaleVirtual(r, n), sdist, torch_dtype).allocate() for r in range(n)]
    dst = [Tensor(shape, LocaleVirtual(r, n), ddist, torch_dtype).allocate() for r in range(n)]
    og_s = [G.TensorGeom(shape, G.Dist(sl, ss or sl, so or [0] * nd), r) for r in range(n)]
    og_d = [G.TensorGeom(shape, G.Dist(dl, ds or dl, do or [0] * nd), r) for r in range(n)]
    for t, g in zip(src + dst, og_s + og_d):
        assert t.local_shape == g.local_shape and t.global_index == g.global_index
        assert t.local_real_shape == g.real_shape and t.is_split_root() == g.is_split_root
    for t, g in zip(src, og_s):
        f = np.full(g.real_shape[::-1], -1, np_dtype)
        f[interior_slices(g)] = global_offset_field(g, mod).astype(np_dtype)
        t.real_view().copy_(torch.from_numpy(f))
    return src, dst, og_s, og_d


@pytest.mark.parametrize("case", list(CASES))
def test_forward_backward_closed_form(case):
    import torch
    from dihydrogen_amd.layers import TensorShufflerVirtual
    src, dst, og_s, og_d = _build(case, torch.float32, np.float32)
    for t in dst:
        t.data.fill_(-7.0)
    sh = TensorShufflerVirtual(src, dst)
    sh.shuffle_forward()
    torch.cuda.synchronize()
    for t, g in zip(dst, og_d):
        f = t.real_view().cpu().numpy()
        if g.is_split_root and g.local_size:
            assert np.array_equal(f[interior_slices(g)], global_offset_field(g).astype(np.float32))
            halo = np.ones(f.shape, bool)
            halo[interior_slices(g)] = False
            assert (f[halo] == -7.0).all()  # halo cells are not written by unpack
        else:
            assert (f == -7.0).all()        # non-root ranks of a shared split receive nothing
    keep = [t.real_view().cpu().numpy().copy() for t in src]
    for t in src:
        t.real_view()[tuple(interior_slices_of(t))] = -3.0
    sh.shuffle_backward()
    torch.cuda.synchronize()
    for t, k, g in zip(src, keep, og_s):
        if g.is_split_root:
            assert np.array_equal(t.real_view().cpu().numpy(), k)


def interior_slices_of(t):
    return [slice(o, o + l) for o, l in zip(t.overlap[::-1], t.local_shape[::-1])]


@pytest.mark.parametrize("case", ["sample_to_spatial", "uneven", "overlap_to_nonoverlap",
                                  "sample_to_spatial_halo", "five_d", "sixteen_ranks_even", "odd_runs",
                                  "odd_runs_halo"])
@pytest.mark.parametrize("np_dtype", [np.float32, np.int16, np.float64])
def test_single_rank_pack_unpack_vs_oracle(case, np_dtype, oracle_mod):
    """h2x_shuffle_pack / h2x_shuffle_unpack with the reference's own table
    layout (displacements in rank order inside one rank's buffer) against the
    oracle's per-element pack / unpack, for 2-, 4- and 8-byte elements."""
    import torch
    from oracle import geometry as G
    from dihydrogen_amd import capi
    lib = capi.load()
    tdt = {np.float32: torch.float32, np.int16: torch.int16, np.float64: torch.float64}[np_dtype]
    mod = 30000 if np_dtype == np.int16 else None
    shape, (sl, ss, so), (dl, ds, do) = CASES[case]
    nd = len(shape)
    n = int(np.prod(sl))
    og_s = [G.TensorGeom(shape, G.Dist(sl, ss or sl, so or [0] * nd), r) for r in range(n)]
    og_d = [G.TensorGeom(shape, G.Dist(dl, ds or dl, do or [0] * nd), r) for r in range(n)]
    rng = np.random.default_rng(1)
    for r in range(n):
        for mine, other, direction in ((og_s[r], og_d[r], "fwd"), (og_d[r], og_s[r], "bwd")):
            if not mine.is_split_root or mine.local_size == 0:
                continue
            limits = G.rank_limits(mine, other)
            if direction == "fwd":
                counts, displs, _, _ = G.counts_and_displs(og_s[r], og_d[r])
            else:
                _, _, counts, displs = G.counts_and_displs(og_s[r], og_d[r])
            assert sum(counts) == mine.local_size
            field = rng.integers(-20000, 20000, mine.real_size).astype(np_dtype)
            base = mine.base_offset()
            # ---- pack
            buf_o = np.zeros(mine.local_size, np_dtype)
            oracle_mod.shuffle_pack_or_unpack(field[base:], mine.local_shape, mine.strides(),
                                              other.dist.locale_shape, limits, buf_o, displs, True)
            g = capi.ShuffleGeometry()
            g.num_dims, g.elem_size = nd, np.dtype(np_dtype).itemsize
            for i in range(nd):
                g.local_shape[i], g.strides[i] = mine.local_shape[i], mine.strides()[i]
                g.peer_locale_shape[i] = other.dist.locale_shape[i]
            rl = (ctypes.c_int32 * len(limits))(*limits)
            dp = (ctypes.c_int32 * len(displs))(*displs)
            g.rank_limits, g.displs = rl, dp
            plan = ctypes.c_void_p()
            capi.check(lib.h2x_shuffle_plan_create(ctypes.byref(g), ctypes.byref(plan)))
            td = torch.from_numpy(field).cuda()
            bd = torch.zeros(mine.local_size, dtype=tdt, device="cuda")
            esz = np.dtype(np_dtype).itemsize
            capi.check(lib.h2x_shuffle_pack(plan, td.data_ptr() + base * esz, bd.data_ptr(), None))
            torch.cuda.synchronize()
            assert np.array_equal(bd.cpu().numpy(), buf_o)
            # ---- unpack of a fresh buffer
            buf2 = rng.integers(-20000, 20000, mine.local_size).astype(np_dtype)
            field_o = field.copy()
            oracle_mod.shuffle_pack_or_unpack(field_o[base:], mine.local_shape, mine.strides(),
                                              other.dist.locale_shape, limits, buf2, displs, False)
            b2 = torch.from_numpy(buf2).cuda()
            capi.check(lib.h2x_shuffle_unpack(plan, td.data_ptr() + base * esz, b2.data_ptr(), None))
            torch.cuda.synchronize()
            assert np.array_equal(td.cpu().numpy(), field_o)
            lib.h2x_shuffle_plan_destroy(plan)


@pytest.mark.parametrize("shift", [1, 2, 3])
def test_pack_unpack_with_a_buffer_that_is_not_16_byte_aligned(shift, oracle_mod):
    """Plans keep their boxes in a device table made for 16-byte aligned staging
    buffers; a buffer that starts `shift` elements later goes through the
    launch-argument path with narrower vectors.  Same bits either way."""
    import torch
    from oracle import geometry as G
    from dihydrogen_amd import capi
    lib = capi.load()
    shape, (sl, ss, so), (dl, ds, do) = CASES["odd_runs"]
    nd, n = len(shape), int(np.prod(sl))
    mine = G.TensorGeom(shape, G.Dist(sl, sl, [0] * nd), 1)
    other = G.TensorGeom(shape, G.Dist(dl, dl, [0] * nd), 1)
    limits = G.rank_limits(mine, other)
    counts, displs, _, _ = G.counts_and_displs(mine, other)
    rng = np.random.default_rng(5)
    field = rng.integers(-20000, 20000, mine.real_size).astype(np.float32)
    buf_o = np.zeros(mine.local_size, np.float32)
    oracle_mod.shuffle_pack_or_unpack(field, mine.local_shape, mine.strides(), other.dist.locale_shape,
                                      limits, buf_o, displs, True)
    g = capi.ShuffleGeometry()
    g.num_dims, g.elem_size = nd, 4
    for i in range(nd):
        g.local_shape[i], g.strides[i] = mine.local_shape[i], mine.strides()[i]
        g.peer_locale_shape[i] = other.dist.locale_shape[i]
    rl = (ctypes.c_int32 * len(limits))(*limits)
    dp = (ctypes.c_int32 * len(displs))(*displs)
    g.rank_limits, g.displs = rl, dp
    plan = ctypes.c_void_p()
    capi.check(lib.h2x_shuffle_plan_create(ctypes.byref(g), ctypes.byref(plan)))
    td = torch.from_numpy(field).cuda()
    bd = torch.full((mine.local_size + 8,), -1.0, device="cuda")
    capi.check(lib.h2x_shuffle_pack(plan, td.data_ptr(), bd.data_ptr() + 4 * shift, None))
    torch.cuda.synchronize()
    got = bd.cpu().numpy()
    assert np.array_equal(got[shift:shift + mine.local_size], buf_o)
    assert (got[:shift] == -1).all() and (got[shift + mine.local_size:] == -1).all()
    t2 = torch.zeros_like(td)
    capi.check(lib.h2x_shuffle_unpack(plan, t2.data_ptr(), bd.data_ptr() + 4 * shift, None))
    torch.cuda.synchronize()
    assert np.array_equal(t2.cpu().numpy(), field)  # the rank's boxes tile its whole local tensor
    lib.h2x_shuffle_plan_destroy(plan)


def test_plan_rejects_bad_tables():
    from dihydrogen_amd import capi
    lib = capi.load()
    g = capi.ShuffleGeometry()
    g.num_dims, g.elem_size = 2, 4
    g.local_shape[0], g.local_shape[1] = 8, 4
    g.strides[0], g.strides[1] = 1, 8
    g.peer_locale_shape[0], g.peer_locale_shape[1] = 2, 1
    rl = (ctypes.c_int32 * 3)(6, 4, 4)  # decreasing limits
    dp = (ctypes.c_int32 * 2)(0, 16)
    g.rank_limits, g.displs = rl, dp
    plan = ctypes.c_void_p()
    assert lib.h2x_shuffle_plan_create(ctypes.byref(g), ctypes.byref(plan)) == -1
    g.elem_size = 3
    assert lib.h2x_shuffle_plan_create(ctypes.byref(g), ctypes.byref(plan)) != 0

"""GPU parity: halo pack/unpack/clear against the CPU oracle, bit-exact.

Structure follows legacy/tests/tensor/test_halo_exchange_cuda.cu: interiors are
initialised to the global linear offset, halos are exchanged, and every halo
cell whose source exists must hold the offset of its source.  On top of that
closed form, whole real tensors (corners included) are compared with the
oracle's exchange of the same virtual ranks.
"""
import itertools

import numpy as np
import pytest

from helpers import global_offset_field, interior_slices, oracle_halo_exchange

pytestmark = pytest.mark.gpu


def _single_face(real_shape_np, dim, side, width, is_pack, is_reverse, op, dtype, oracle_mod):
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    rng = np.random.default_rng(hash((real_shape_np, dim, side, width, is_pack, is_reverse, op)) % 2**32)
    t = rng.uniform(-1, 1, real_shape_np).astype(dtype)
    shape = real_shape_np[::-1]
    n = oracle_mod.halo_size(shape, dim, width)
    b = rng.uniform(-1, 1, n).astype(dtype)
    t_o, b_o = t.copy(), b.copy()
    oracle_mod.halo_pack_or_unpack(t_o, dim, side, width, b_o, is_pack, is_reverse, op)
    td, bd = torch.from_numpy(t).cuda(), torch.from_numpy(b).cuda()
    shp = capi.i64_array(shape)
    h2x_dt = capi.F32 if dtype == np.float32 else capi.F64
    capi.check(lib.h2x_halo_pack_or_unpack(h2x_dt, td.data_ptr(), len(shape), shp, dim, side, width,
                                           bd.data_ptr(), int(is_pack), int(is_reverse), op, None))
    torch.cuda.synchronize()
    assert np.array_equal(td.cpu().numpy(), t_o, equal_nan=True)
    assert np.array_equal(bd.cpu().numpy(), b_o, equal_nan=True)


@pytest.mark.parametrize("real_shape_np", [(2, 3, 6, 8), (2, 3, 5, 6, 7), (1, 2, 9, 10, 12)])
def test_every_face_every_width(real_shape_np, oracle_mod):
    """All (dim, side, width, pack/unpack, forward/reverse) of 4-D and 5-D
    tensors, including 5-D dimension 0, which the reference's optimised
    traversal leaves empty (halo_cuda.hpp:220-235)."""
    nd = len(real_shape_np)
    shape = real_shape_np[::-1]
    for dim, side, is_pack, is_reverse in itertools.product(range(nd), (0, 1), (True, False), (False, True)):
        for width in (1, 2, 3, 4):
            if 2 * width > shape[dim]:
                continue
            _single_face(real_shape_np, dim, side, width, is_pack, is_reverse, 0, np.float32, oracle_mod)


@pytest.mark.parametrize("op", [1, 2, 3])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_accumulate_ops(op, dtype, oracle_mod):
    """SUM / MAX / MIN unpack (halo_packing_cuda.hpp:36-58)."""
    for dim in range(4):
        for side in (0, 1):
            _single_face((4, 4, 8, 12), dim, side, 2, False, True, op, dtype, oracle_mod)
            _single_face((4, 4, 8, 12), dim, side, 1, False, False, op, dtype, oracle_mod)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("real_shape_np", [(2, 3, 5, 21), (1, 2, 4, 6, 19), (1, 2, 3, 130), (2, 2, 3, 3, 34)])
def test_rows_that_are_no_multiple_of_the_vector(real_shape_np, dtype, oracle_mod):
    """Runs of 17..130 elements move in 16-byte vectors indexed from the buffer
    side; the vectors that straddle a row end, and the last one of a strip whose
    size is no multiple of 4, go element by element.  Every dimension whose strip
    has such runs, both sides, widths 1-3, pack, unpack and an accumulating unpack."""
    nd = len(real_shape_np)
    shape = real_shape_np[::-1]
    for dim, side in itertools.product(range(1, nd), (0, 1)):
        for width in (1, 2, 3):
            if 2 * width > shape[dim]:
                continue
            _single_face(real_shape_np, dim, side, width, True, False, 0, dtype, oracle_mod)
            _single_face(real_shape_np, dim, side, width, False, False, 0, dtype, oracle_mod)
            _single_face(real_shape_np, dim, side, width, False, True, 1, dtype, oracle_mod)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("op", [0, 1, 2])
def test_both_faces_of_the_innermost_dimension_in_one_call(op, dtype, oracle_mod):
    """LHS and RHS face of dimension 0, width 1, unpacked by one batched call: the
    RHS halo cell of a row and the LHS halo cell of the next row are neighbours in
    memory and are written together.  Identity and accumulating ops, against
    the oracle's two separate unpacks; then the same pair packed."""
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    real_np = (2, 3, 7, 9)
    shape = real_np[::-1]
    rng = np.random.default_rng(17 + op)
    t = rng.uniform(-1, 1, real_np).astype(dtype)
    n = oracle_mod.halo_size(shape, 0, 1)
    bufs = [rng.uniform(-1, 1, n).astype(dtype) for _ in range(2)]
    h2x_dt = capi.F32 if dtype == np.float32 else capi.F64
    for is_pack in (False, True):
        t_o, b_o = t.copy(), [b.copy() for b in bufs]
        for side in (0, 1):
            oracle_mod.halo_pack_or_unpack(t_o, 0, side, 1, b_o[side], is_pack, False, op)
        td = torch.from_numpy(t).cuda()
        bd = [torch.from_numpy(b).cuda() for b in bufs]
        faces = (capi.HaloFace * 2)()
        for side in (0, 1):
            f = faces[side]
            f.tensor, f.buffer = td.data_ptr(), bd[side].data_ptr()
            for i, e in enumerate(shape):
                f.real_shape[i] = e
            f.num_dims, f.dim, f.side, f.width = len(shape), 0, side, 1
            f.inner, f.is_pack, f.op = int(is_pack), int(is_pack), op
        capi.check(lib.h2x_halo_pack_or_unpack_batched(h2x_dt, faces, 2, None))
        torch.cuda.synchronize()
        assert np.array_equal(td.cpu().numpy(), t_o)
        for side in (0, 1):
            assert np.array_equal(bd[side].cpu().numpy(), b_o[side])


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("op", [1, 2, 3])
@pytest.mark.parametrize("real_np,width", [((2, 3, 7, 9), 1), ((2, 3, 7, 3), 1), ((2, 2, 5, 6), 2),
                                           ((2, 2, 5, 7), 2), ((1, 2, 3, 130), 1)])
def test_reverse_accumulation_of_both_faces_in_one_call(real_np, width, op, dtype, oracle_mod):
    """Reverse unpack (halo contributions folded into the interior strips) of
    the LHS and RHS face of dimension 0 by one batched call.  With an interior
    as narrow as the strip the two strips are the same cells, with one cell
    more they overlap in part: every cell must then receive both contributions,
    as the oracle's two unpacks one after the other give them."""
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    shape = real_np[::-1]
    rng = np.random.default_rng(29 + op + width)
    t = rng.uniform(-1, 1, real_np).astype(dtype)
    n = oracle_mod.halo_size(shape, 0, width)
    bufs = [rng.uniform(-1, 1, n).astype(dtype) for _ in range(2)]
    h2x_dt = capi.F32 if dtype == np.float32 else capi.F64
    t_o = t.copy()
    for side in (0, 1):
        oracle_mod.halo_pack_or_unpack(t_o, 0, side, width, bufs[side], False, True, op)
    td = torch.from_numpy(t).cuda()
    bd = [torch.from_numpy(b).cuda() for b in bufs]
    faces = (capi.HaloFace * 2)()
    for side in (0, 1):
        f = faces[side]
        f.tensor, f.buffer = td.data_ptr(), bd[side].data_ptr()
        for i, e in enumerate(shape):
            f.real_shape[i] = e
        f.num_dims, f.dim, f.side, f.width = len(shape), 0, side, width
        f.inner, f.is_pack, f.op = 1, 0, op
    capi.check(lib.h2x_halo_pack_or_unpack_batched(h2x_dt, faces, 2, None))
    torch.cuda.synchronize()
    assert np.array_equal(td.cpu().numpy(), t_o)


def _exchange_case(shape, locale, overlap, periodic, oracle_mod, widths=None, dtype=np.float32,
                   fused=False):
    """Runs the exchange on the GPU and on the CPU oracle; returns both."""
    import torch
    from oracle import geometry as G
    from dihydrogen_amd.layers import HaloExchangeVirtual
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor

    nranks = int(np.prod(locale))
    odist = G.Dist(locale, locale, overlap)
    geoms = [G.TensorGeom(shape, odist, r) for r in range(nranks)]
    fields = []
    for g in geoms:
        f = np.full(g.real_shape[::-1], np.nan, dtype)
        f[interior_slices(g)] = global_offset_field(g)
        fields.append(f)
    dist = Distribution.make_overlapped_distribution(locale, overlap)
    tensors = []
    for r in range(nranks):
        t = Tensor(shape, LocaleVirtual(r, nranks), dist, torch.float32 if dtype == np.float32 else torch.float64).allocate()
        assert t.local_real_shape == geoms[r].real_shape and t.global_index == geoms[r].global_index
        t.real_view().copy_(torch.from_numpy(fields[r]))
        tensors.append(t)
    xch = HaloExchangeVirtual(tensors, periodic=periodic)
    if widths is None:
        xch.exchange(fused=fused)
    else:
        xch.exchange(widths, widths, widths, widths, fused=fused)
    torch.cuda.synchronize()
    oracle_halo_exchange(oracle_mod, geoms, fields, periodic, widths)
    return geoms, fields, [t.real_view().cpu().numpy() for t in tensors]


def _closed_form_check(geoms, got, periodic, widths=None):
    """check_tensor of the reference test (test_halo_exchange_cuda.cu:104-233):
    walk both outer strips of each dimension; wherever the source coordinate
    exists (or wraps, for periodic grids) the stored value is its global offset."""
    for g, f in zip(geoms, got):
        nd = g.nd
        for d in range(nd):
            w = g.overlap[d] if widths is None else widths[d]
            if w == 0 or g.dist.split_shape[d] <= 1:
                continue
            for side in (0, 1):
                lo = 0 if side == 0 else g.real_shape[d] - w
                sl = [slice(None)] * nd
                sl[nd - 1 - d] = slice(lo, lo + w)
                strip = f[tuple(sl)]
                idx = np.indices(strip.shape, dtype=np.int64)
                ok = np.ones(strip.shape, bool)
                off = np.zeros(strip.shape, np.int64)
                stride = 1
                for k in range(nd):
                    local = idx[nd - 1 - k] + (lo if k == d else 0)
                    glob = local + g.global_index[k] - g.overlap[k]
                    if periodic:
                        glob %= g.shape[k]
                    else:
                        ok &= (glob >= 0) & (glob < g.shape[k])
                    off += np.clip(glob, 0, g.shape[k] - 1) * stride
                    stride *= g.shape[k]
                assert np.array_equal(strip[ok], off[ok].astype(f.dtype))


EXCHANGE_CASES = [
    # shape (innermost first), locale, overlap
    ((12, 10, 3, 2), (2, 2, 1, 1), (1, 1, 0, 0)),
    ((12, 10, 3, 2), (2, 2, 1, 1), (2, 2, 0, 0)),
    ((13, 11, 3, 2), (3, 2, 1, 1), (1, 2, 0, 0)),          # uneven partition
    ((8, 10, 12, 3, 2), (2, 2, 2, 1, 1), (1, 1, 1, 0, 0)),  # 3-D decomposition incl. dimension 0
    ((8, 9, 10, 2, 1), (1, 2, 2, 1, 1), (0, 2, 1, 0, 0)),   # the reference's default 3-D driver keeps W whole
    ((16, 8, 2, 2), (4, 1, 1, 1), (3, 0, 0, 0)),
]


@pytest.mark.parametrize("periodic", [False, True])
@pytest.mark.parametrize("case", EXCHANGE_CASES)
def test_exchange_closed_form_and_oracle(case, periodic, oracle_mod):
    shape, locale, overlap = case
    geoms, want, got = _exchange_case(shape, locale, overlap, periodic, oracle_mod)
    _closed_form_check(geoms, got, periodic)
    for w, g in zip(want, got):
        assert np.array_equal(w, g, equal_nan=True)


@pytest.mark.parametrize("periodic", [False, True])
@pytest.mark.parametrize("case", EXCHANGE_CASES)
def test_fused_exchange_closed_form_and_oracle(case, periodic, oracle_mod):
    """Tensor-to-tensor transfers leave what pack + unpack through buffers leave."""
    shape, locale, overlap = case
    geoms, want, got = _exchange_case(shape, locale, overlap, periodic, oracle_mod, fused=True)
    _closed_form_check(geoms, got, periodic)
    for w, g in zip(want, got):
        assert np.array_equal(w, g, equal_nan=True)


def test_fused_exchange_narrower_than_halo_f64(oracle_mod):
    shape, locale, overlap = (12, 10, 3, 2), (2, 2, 1, 1), (2, 2, 0, 0)
    geoms, want, got = _exchange_case(shape, locale, overlap, True, oracle_mod, widths=[1, 1, 0, 0],
                                      dtype=np.float64, fused=True)
    for w, g in zip(want, got):
        assert np.array_equal(w, g, equal_nan=True)


@pytest.mark.parametrize("op", [1, 2, 3])
def test_fused_reverse_exchange_ops(op, oracle_mod):
    """Reverse transfers combine the neighbour's halo into the boundary cells
    with SUM / MAX / MIN, as the unpack of halo_packing_cuda.hpp:36-58 does."""
    import torch
    from oracle import geometry as G
    from dihydrogen_amd.layers import HaloExchangeAccumOp, HaloExchangeVirtual
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    shape, locale, overlap = (10, 12, 6, 2, 1), (2, 3, 2, 1, 1), (1, 2, 1, 0, 0)
    nranks = 12
    rng = np.random.default_rng(80 + op)
    geoms = [G.TensorGeom(shape, G.Dist(locale, locale, overlap), r) for r in range(nranks)]
    fields = [rng.integers(-8, 8, g.real_shape[::-1]).astype(np.float32) for g in geoms]
    dist = Distribution.make_overlapped_distribution(locale, overlap)
    tensors = []
    for r in range(nranks):
        t = Tensor(shape, LocaleVirtual(r, nranks), dist).allocate()
        t.real_view().copy_(torch.from_numpy(fields[r]))
        tensors.append(t)
    HaloExchangeVirtual(tensors, periodic=True).exchange(is_reverse=True, op=HaloExchangeAccumOp(op),
                                                         fused=True)
    torch.cuda.synchronize()
    oracle_halo_exchange(oracle_mod, geoms, fields, True, None, True, op)
    for f, t in zip(fields, tensors):
        assert np.array_equal(f, t.real_view().cpu().numpy())


def test_fused_transfer_rejects_mismatched_shapes():
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    a, b = torch.zeros(4 * 6 * 8, device="cuda"), torch.ones(4 * 6 * 8, device="cuda")
    m = capi.HaloTransfer()
    m.src, m.dst = a.data_ptr(), b.data_ptr()
    for i, (x, y) in enumerate(zip((8, 6, 4), (8, 5, 4))):
        m.src_real_shape[i], m.dst_real_shape[i] = x, y
    m.num_dims, m.dim, m.src_side, m.width, m.is_reverse, m.op = 3, 0, capi.RHS, 1, 0, 0
    assert lib.h2x_halo_exchange_fused(capi.F32, m, 1, None) == -1  # extents differ off the exchanged dimension
    m.dst_real_shape[1] = 6
    m.width = 5  # two strips of 5 do not fit in 8
    assert lib.h2x_halo_exchange_fused(capi.F32, m, 1, None) == -1
    m.width = 0
    assert lib.h2x_halo_exchange_fused(capi.F32, m, 1, None) == 0
    torch.cuda.synchronize()
    assert (b == 1).all()


def test_exchange_narrower_than_halo(oracle_mod):
    """Width 1 in a halo of 2: strips are positioned by the width passed in,
    not by the halo width (halo_cuda.hpp:59-81)."""
    shape, locale, overlap = (12, 10, 3, 2), (2, 2, 1, 1), (2, 2, 0, 0)
    geoms, want, got = _exchange_case(shape, locale, overlap, False, oracle_mod, widths=[1, 1, 0, 0])
    for w, g in zip(want, got):
        assert np.array_equal(w, g, equal_nan=True)


def test_exchange_wider_than_halo_is_rejected_and_reallocation_is_seen(oracle_mod):
    """Strips wider than the halo would run past the receive buffers: the layer
    refuses them.  Face tables are cached per tensor address: an exchange after
    a tensor was reallocated works on the new allocation."""
    import torch
    from dihydrogen_amd.layers import HaloExchangeVirtual
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    shape, locale, overlap = (12, 10, 3, 2), (2, 2, 1, 1), (1, 1, 0, 0)
    dist = Distribution.make_overlapped_distribution(locale, overlap)
    tensors = [Tensor(shape, LocaleVirtual(r, 4), dist).allocate() for r in range(4)]
    xch = HaloExchangeVirtual(tensors, periodic=True)
    for fused in (False, True):
        with pytest.raises(ValueError):
            xch.exchange([2, 1, 0, 0], [2, 1, 0, 0], [2, 1, 0, 0], [2, 1, 0, 0], fused=fused)
    for fused in (False, True):
        for t in tensors:
            t.real_view().fill_(float("nan"))
            t.interior_view().fill_(1.0)
        xch.exchange(fused=fused)
        torch.cuda.synchronize()
        keep = [t.data for t in tensors]          # old allocations stay alive, so the new ones differ
        for t in tensors:
            t.data = torch.full_like(t.data, float("nan"))
            t.interior_view().fill_(2.0)
        xch.exchange(fused=fused)
        torch.cuda.synchronize()
        for t in tensors:
            assert (t.real_view() == 2.0).all()   # periodic: every halo cell has a source
        del keep


def test_reverse_sum_exchange(oracle_mod):
    """Reverse exchange with SUM: halo contributions are added onto the
    neighbour's boundary cells (used by backward-data and pooling)."""
    import torch
    from oracle import geometry as G
    from dihydrogen_amd.layers import HaloExchangeAccumOp, HaloExchangeVirtual
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    shape, locale, overlap = (10, 8, 2, 2), (2, 2, 1, 1), (1, 2, 0, 0)
    nranks = 4
    rng = np.random.default_rng(8)
    geoms = [G.TensorGeom(shape, G.Dist(locale, locale, overlap), r) for r in range(nranks)]
    fields = [rng.integers(-8, 8, g.real_shape[::-1]).astype(np.float32) for g in geoms]
    dist = Distribution.make_overlapped_distribution(locale, overlap)
    tensors = []
    for r in range(nranks):
        t = Tensor(shape, LocaleVirtual(r, nranks), dist).allocate()
        t.real_view().copy_(torch.from_numpy(fields[r]))
        tensors.append(t)
    HaloExchangeVirtual(tensors).exchange(is_reverse=True, op=HaloExchangeAccumOp.SUM)
    torch.cuda.synchronize()
    oracle_halo_exchange(oracle_mod, geoms, fields, False, None, True, 1)
    for f, t in zip(fields, tensors):
        assert np.array_equal(f, t.real_view().cpu().numpy())


def test_clear_halo(oracle_mod):
    import torch
    from dihydrogen_amd.layers import HaloExchangeVirtual
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    shape, locale, overlap = (10, 8, 6, 2, 1), (2, 2, 2, 1, 1), (1, 2, 1, 0, 0)
    dist = Distribution.make_overlapped_distribution(locale, overlap)
    tensors = [Tensor(shape, LocaleVirtual(r, 8), dist).allocate() for r in range(8)]
    for t in tensors:
        t.data.fill_(5.0)
    xch = HaloExchangeVirtual(tensors)
    for d in range(3):
        xch.clear_halo(d)
    torch.cuda.synchronize()
    for t in tensors:
        f = t.real_view().cpu().numpy()
        want = np.zeros_like(f)
        want[tuple(slice(o, o + l) for o, l in zip(t.overlap[::-1], t.local_shape[::-1]))] = 5.0
        assert np.array_equal(f, want)


@pytest.mark.parametrize("shape,locale,overlap", [((32, 31, 4, 8), (2, 2, 1, 1), (1, 2, 0, 0)),
                                                  ((12, 9, 10, 3, 2), (2, 1, 2, 1, 1), (2, 0, 1, 0, 0))])
def test_clear_halo_one_dimension_at_a_time(shape, locale, overlap):
    """The reference's own check (legacy/tests/tensor/test_tensor_mpi_cuda.cu:162-231): fill
    with 1, clear the halo of ONE dimension, and every cell whose index along that
    dimension lies in the halo is 0, every other cell - the halos of the other
    dimensions included - still 1."""
    import torch
    from dihydrogen_amd.layers import HaloExchangeVirtual
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    n = int(np.prod(locale))
    dist = Distribution.make_overlapped_distribution(locale, overlap)
    tensors = [Tensor(shape, LocaleVirtual(r, n), dist).allocate() for r in range(n)]
    xch = HaloExchangeVirtual(tensors)
    for d in range(len(shape)):
        for t in tensors:
            t.data.fill_(1.0)
        xch.clear_halo(d)
        torch.cuda.synchronize()
        for t in tensors:
            f = t.real_view().cpu().numpy()
            want = np.ones_like(f)
            ov = t.overlap[d]
            if ov:
                axis = len(shape) - 1 - d
                idx = [slice(None)] * len(shape)
                idx[axis] = slice(0, ov)
                want[tuple(idx)] = 0
                idx[axis] = slice(f.shape[axis] - ov, None)
                want[tuple(idx)] = 0
            assert np.array_equal(f, want), (d, t.locale.get_rank() if hasattr(t, "locale") else None)


def test_zero_width_is_noop():
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    t = torch.ones(64, device="cuda")
    shp = capi.i64_array((4, 4, 2, 2))
    assert lib.h2x_halo_pack_or_unpack(capi.F32, t.data_ptr(), 4, shp, 0, 0, 0, None, 1, 0, 0, None) == 0
    # a dimension that does not exist is rejected, nothing is launched
    assert lib.h2x_halo_pack_or_unpack(capi.F32, t.data_ptr(), 4, shp, 9, 0, 1, t.data_ptr(), 1, 0, 0,
                                       None) == -1
    torch.cuda.synchronize()
    assert (t == 1).all()


@pytest.mark.parametrize("periodic", [False, True])
@pytest.mark.parametrize("shape,locale,overlap", [((10, 8, 6, 2, 1), (2, 2, 2, 1, 1), (1, 2, 1, 0, 0)),
                                                  ((12, 9, 4, 3), (3, 2, 1, 1), (2, 1, 0, 0)),
                                                  ((130, 6, 5, 2), (2, 1, 1, 1), (1, 0, 0, 0))])
def test_batched_clear_and_clearing_only_what_the_exchange_leaves(shape, locale, overlap, periodic):
    """clear_halos() (one batched call for all ranks, dimensions and sides) equals
    clear_halo(dim) rank by rank; and clear_halos(only_unfilled=True) followed by a
    full-width exchange leaves every tensor - corners and the halos at the edge of a
    non-periodic grid included - bit for bit as clearing everything and then
    exchanging, from halos poisoned with different values on every rank."""
    import torch
    from dihydrogen_amd.layers import HaloExchangeVirtual
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    n = int(np.prod(locale))
    dist = Distribution.make_overlapped_distribution(locale, overlap)
    rng = np.random.default_rng(3)

    def make():
        ts = [Tensor(shape, LocaleVirtual(r, n), dist).allocate() for r in range(n)]
        g = np.random.default_rng(11)
        for t in ts:
            t.real_view().copy_(torch.from_numpy(g.uniform(1, 2, tuple(t.real_view().shape)).astype(np.float32)))
        return ts

    a, b = make(), make()
    xa, xb = HaloExchangeVirtual(a, periodic=periodic), HaloExchangeVirtual(b, periodic=periodic)
    for d in range(len(shape)):
        xa.clear_halo(d)
    xb.clear_halos()
    torch.cuda.synchronize()
    for ta, tb in zip(a, b):
        assert torch.equal(ta.real_view(), tb.real_view())
    # the reference's sequence against the shortened one
    c, d_ = make(), make()
    xc, xd = HaloExchangeVirtual(c, periodic=periodic), HaloExchangeVirtual(d_, periodic=periodic)
    xc.clear_halos()
    xc.exchange()
    xd.clear_halos(only_unfilled=True)
    xd.exchange()
    torch.cuda.synchronize()
    for tc, td in zip(c, d_):
        assert torch.equal(tc.real_view(), td.real_view())
    del rng

"""Pins the halo functions of the CPU oracle: strip position and packed order
by brute force, the exchange by the reference test's closed form
(legacy/tests/tensor/test_halo_exchange_cuda.cu:43-233), and the accumulate
ops by conservation."""
import itertools

import numpy as np
import pytest

import oracle
from oracle import geometry as G
from helpers import global_offset_field, interior_slices, oracle_halo_exchange


def _brute_strip(real_shape, dim, side, inner, width):
    """Tensor offsets of the strip in natural packed order, plain loops
    (legacy/include/distconv/tensor/halo_cuda.hpp:47-81)."""
    nd = len(real_shape)
    ext = [width if i == dim else real_shape[i] for i in range(nd)]
    if side == 1:
        start = real_shape[dim] - (2 * width if inner else width)
    else:
        start = width if inner else 0
    offs = []
    for idx in itertools.product(*[range(e) for e in reversed(ext)]):  # outermost first
        idx = idx[::-1]
        off, stride = 0, 1
        for i in range(nd):
            off += (idx[i] + (start if i == dim else 0)) * stride
            stride *= real_shape[i]
        offs.append(off)
    return offs


@pytest.mark.parametrize("real_shape", [(6, 5, 3, 2), (5, 6, 4, 3, 2), (9, 8, 2, 1)])
def test_strip_position_and_order(real_shape):
    nd = len(real_shape)
    n = int(np.prod(real_shape))
    for dim, side, inner, width in itertools.product(range(nd), (0, 1), (0, 1), (1, 2, 3, 4)):
        if (2 if inner else 1) * width > real_shape[dim]:
            continue
        t = np.arange(n, dtype=np.float32).reshape(real_shape[::-1])
        buf = np.zeros(oracle.halo_size(real_shape, dim, width), np.float32)
        oracle.halo_pack_or_unpack(t, dim, side, width, buf, True, is_reverse=not inner)
        assert buf.tolist() == [float(o) for o in _brute_strip(real_shape, dim, side, inner, width)]
        # unpack writes exactly those cells, in that order
        t2 = np.zeros(n, np.float32).reshape(real_shape[::-1])
        vals = np.arange(1, buf.size + 1, dtype=np.float32)
        oracle.halo_pack_or_unpack(t2, dim, side, width, vals, False, is_reverse=bool(inner))
        want = np.zeros(n, np.float32)
        want[_brute_strip(real_shape, dim, side, inner, width)] = vals
        assert np.array_equal(t2.ravel(), want)


@pytest.mark.parametrize("periodic", [False, True])
@pytest.mark.parametrize("case", [
    ((12, 10, 3, 2), (2, 2, 1, 1), (1, 1, 0, 0)),
    ((13, 11, 3, 2), (3, 2, 1, 1), (1, 2, 0, 0)),
    ((8, 10, 12, 3, 2), (2, 2, 2, 1, 1), (1, 1, 1, 0, 0)),
])
def test_exchange_closed_form(case, periodic):
    shape, locale, overlap = case
    nranks = int(np.prod(locale))
    geoms = [G.TensorGeom(shape, G.Dist(locale, locale, overlap), r) for r in range(nranks)]
    fields = []
    for g in geoms:
        f = np.full(g.real_shape[::-1], np.nan, np.float32)
        f[interior_slices(g)] = global_offset_field(g)
        fields.append(f)
    oracle_halo_exchange(oracle, geoms, fields, periodic)
    nd = len(shape)
    for g, f in zip(geoms, fields):
        idx = np.indices(f.shape, dtype=np.int64)
        off, stride = np.zeros(f.shape, np.int64), 1
        ok = np.ones(f.shape, bool)
        for k in range(nd):
            glob = idx[nd - 1 - k] + g.global_index[k] - g.overlap[k]
            if periodic and g.dist.split_shape[k] > 1:
                glob %= g.shape[k]
            ok &= (glob >= 0) & (glob < g.shape[k])
            off += np.clip(glob, 0, g.shape[k] - 1) * stride
            stride *= g.shape[k]
        # every cell whose source exists holds the source's global offset: faces, edges and corners
        assert np.array_equal(f[ok], off[ok].astype(np.float32))
        assert np.isnan(f[~ok]).all()


def test_reverse_sum_conserves_and_adds():
    """Reverse exchange with SUM adds each halo cell onto the neighbour's
    boundary cell it mirrors: the total over interiors grows by exactly the
    sum of the halo cells that have a neighbour (cf. check_tensor_reverse,
    test_halo_exchange_cuda.cu:235-432)."""
    shape, locale, overlap = (8, 6, 2, 1), (2, 1, 1, 1), (2, 0, 0, 0)
    geoms = [G.TensorGeom(shape, G.Dist(locale, locale, overlap), r) for r in range(2)]
    rng = np.random.default_rng(3)
    fields = [rng.integers(-5, 5, g.real_shape[::-1]).astype(np.float32) for g in geoms]
    before = [f.copy() for f in fields]
    oracle_halo_exchange(oracle, geoms, fields, False, None, True, oracle.OP_SUM)
    # rank 0's RHS halo (last 2 columns) is added onto rank 1's first 2 interior columns, and vice versa
    assert np.array_equal(fields[1][..., 2:4], before[1][..., 2:4] + before[0][..., -2:])
    assert np.array_equal(fields[0][..., -4:-2], before[0][..., -4:-2] + before[1][..., :2])
    assert np.array_equal(fields[0][..., :-4], before[0][..., :-4])


@pytest.mark.parametrize("op,fn", [(oracle.OP_MAX, np.maximum), (oracle.OP_MIN, np.minimum)])
def test_max_min(op, fn):
    rng = np.random.default_rng(4)
    t = rng.standard_normal((2, 3, 4, 6)).astype(np.float32)
    buf = rng.standard_normal(oracle.halo_size((6, 4, 3, 2), 1, 1)).astype(np.float32)
    t0 = t.copy()
    oracle.halo_pack_or_unpack(t, 1, 0, 1, buf, False, False, op)
    assert np.array_equal(t[:, :, 0, :], fn(t0[:, :, 0, :], buf.reshape(2, 3, 6)))
    assert np.array_equal(t[:, :, 1:, :], t0[:, :, 1:, :])

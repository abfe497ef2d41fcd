"""GPU parity: elementwise transforms and sums over dimensions through the C ABI
(h2x_tensor_transform, h2x_tensor_reduce_sum) against the oracle.

Transforms: bit-exact (one rounding per operation, same operations).  Sums:
within 1e-5 relative of the float64 sum (both sides accumulate in float64 and
round once; the orders of addition differ), identical from run to run, and the reference test's closed forms hold
(legacy/tests/tensor/test_tensor_mpi_cuda_algorithms.cu:100-300)."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
TOL = 1e-5


def _haloed(rng, local_np, halo_np, dtype):
    """A real (haloed) array in numpy order, its interior view, and its geometry."""
    from dihydrogen_amd import capi
    real = tuple(l + 2 * h for l, h in zip(local_np, halo_np))
    a = rng.standard_normal(real).astype(dtype)
    sl = tuple(slice(h, h + l) for l, h in zip(local_np, halo_np))
    g = capi.TensorGeometry()
    nd = len(local_np)
    g.num_dims = nd
    strides = [1] * nd
    for i in range(1, nd):
        strides[i] = strides[i - 1] * real[nd - i]          # innermost first
    for i in range(nd):
        g.local_shape[i] = local_np[nd - 1 - i]
        g.strides[i] = strides[i]
    base = sum(h * s for h, s in zip(reversed(halo_np), strides))
    return a, sl, g, base


def _transform(op, arrays, geoms, bases, params, dtype):
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    dev = [torch.from_numpy(a).cuda() for a in arrays]
    es = np.dtype(dtype).itemsize
    n = len(arrays)
    gp = (ctypes.POINTER(capi.TensorGeometry) * n)(*[ctypes.pointer(g) for g in geoms])
    tp = (ctypes.c_void_p * n)(*[d.data_ptr() + b * es for d, b in zip(dev, bases)])
    pp = (ctypes.c_double * 4)(*(list(params) + [0.0] * (4 - len(params))))
    capi.check(lib.h2x_tensor_transform(op, capi.F32 if dtype == np.float32 else capi.F64, n, gp, tp, pp, None),
               "transform")
    torch.cuda.synchronize()
    return [d.cpu().numpy() for d in dev]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("local,halos", [((2, 3, 5, 7), ((0, 0, 0, 0), (0, 0, 1, 2))),
                                         ((1, 4, 3, 6, 8), ((0, 0, 1, 1, 1), (0, 0, 0, 0, 0))),
                                         ((5, 1, 1, 9), ((0, 0, 0, 3), (0, 0, 0, 0))),
                                         ((64, 33), ((0, 0), (1, 0))),
                                         ((2, 3, 4, 8), ((0, 0, 1, 1), (0, 0, 0, 2))),
                                         ((3, 2, 5, 64), ((0, 0, 0, 0), (0, 0, 1, 0)))])
def test_transforms_match_oracle(local, halos, dtype, oracle_mod):
    from dihydrogen_amd import capi
    rng = np.random.default_rng(11)
    a, sa, ga, ba = _haloed(rng, local, halos[0], dtype)
    b, sb, gb, bb = _haloed(rng, local, halos[1], dtype)
    # scale: one tensor, halo untouched
    want = a.copy()
    oracle_mod.tensor_transform(oracle_mod.TRANSFORM_SCALE, [want[sa]], [1.75])
    got, = _transform(capi.TRANSFORM_SCALE, [a], [ga], [ba], [1.75], dtype)
    assert np.array_equal(got, want)
    # copy and scale-bias between two tensors with different halos
    for op, oop, params in ((capi.TRANSFORM_COPY, oracle_mod.TRANSFORM_COPY, []),
                            (capi.TRANSFORM_SCALE_BIAS, oracle_mod.TRANSFORM_SCALE_BIAS, [-0.5, 0.125])):
        wa, wb = a.copy(), b.copy()
        oracle_mod.tensor_transform(oop, [wa[sa], wb[sb]], params)
        ga_, gb_ = _transform(op, [a, b], [ga, gb], [ba, bb], params, dtype)
        assert np.array_equal(ga_, wa) and np.array_equal(gb_, wb)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n", [0, 1, 25088])
def test_sums_to_statistics_as_a_four_tensor_transform(n, dtype, oracle_mod):
    """The reference's sums_to_statistics is a Transform over four {1,1,C,1} tensors
    (batchnorm.cu:317-346).  Same bits as h2x_bn_sums_to_statistics and as the oracle."""
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    rng = np.random.default_rng(5)
    c = 19
    vals = [rng.uniform(1, 2, (1, c, 1, 1)).astype(dtype) * (n if i < 2 else 1) for i in range(4)]
    geoms, bases = [], []
    for v in vals:
        _, _, g, _ = _haloed(rng, v.shape, (0, 0, 0, 0), dtype)
        geoms.append(g)
        bases.append(0)
    want = [v.copy() for v in vals]
    oracle_mod.tensor_transform(oracle_mod.TRANSFORM_SUMS_TO_STATISTICS, want, [n, 0.9])
    got = _transform(capi.TRANSFORM_SUMS_TO_STATISTICS, vals, geoms, bases, [n, 0.9], dtype)
    dev = [torch.from_numpy(v.copy()).cuda() for v in vals]
    capi.check(lib.h2x_bn_sums_to_statistics(capi.F32 if dtype == np.float32 else capi.F64, c, n, 0.9,
                                             *[d.data_ptr() for d in dev], None))
    torch.cuda.synchronize()
    for g, w, d in zip(got, want, dev):
        assert np.array_equal(g, w, equal_nan=True)
        assert np.array_equal(g, d.cpu().numpy(), equal_nan=True)


def _reduce(src, ssl, gs, bs, dst, gd, square, dtype):
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    es = np.dtype(dtype).itemsize
    sd, dd = torch.from_numpy(src).cuda(), torch.from_numpy(dst).cuda()
    nbytes = lib.h2x_tensor_reduce_sum_workspace_bytes(ctypes.byref(gs), ctypes.byref(gd))
    assert nbytes > 0 and nbytes % 256 == 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    capi.check(lib.h2x_tensor_reduce_sum(capi.F32 if dtype == np.float32 else capi.F64, ctypes.byref(gs),
                                         sd.data_ptr() + bs * es, ctypes.byref(gd), dd.data_ptr(), int(square),
                                         ws.data_ptr(), None), "reduce_sum")
    torch.cuda.synchronize()
    return dd.cpu().numpy()


REDUCE_CASES = [
    # local shape (numpy order), halo, which axes are reduced
    ((3, 4, 5, 6), (0, 0, 1, 2), (0, 2, 3)),       # per channel, as batch-norm
    ((3, 4, 5, 6), (0, 0, 0, 0), (0,)),            # over samples only: innermost kept
    ((3, 4, 5, 6), (0, 0, 1, 1), (3,)),            # innermost only
    ((3, 4, 5, 6), (0, 0, 0, 0), (0, 1, 2, 3)),    # to one cell
    ((3, 4, 5, 6), (0, 0, 2, 0), ()),              # nothing reduced: dst += src
    ((8, 64, 56, 56), (0, 0, 0, 0), (0, 2, 3)),    # config 1's shape
    ((2, 3, 4, 40, 50), (0, 0, 1, 1, 1), (0, 2, 3, 4)),
    ((6, 5, 2000), (0, 0, 0), (0,)),
    ((6, 5, 2000), (0, 0, 3), (1, 2)),
    ((2, 3, 4, 6, 8), (0, 0, 1, 1, 1), (0, 2, 3, 4)),   # rows of whole 16-byte vectors that start on any element
    ((2, 3, 1100, 4), (0, 0, 1, 1), (0, 2, 3)),         # more than one group per output, groups of whole vectors
    ((3, 5, 6, 64), (0, 0, 0, 0), (3,)),                # few addends per output: lanes of a wave share an output
    ((3, 5, 6, 64), (0, 0, 1, 2), (3,)),
    ((2, 3, 7, 9), (0, 0, 0, 1), (2, 3)),               # 63 addends in two reduced dimensions, no vectors
    ((4, 3, 5, 1), (0, 0, 0, 0), (3,)),                 # a single addend
    ((6, 4, 5, 64), (0, 0, 0, 0), (0,)),                # innermost kept: vectors of neighbouring outputs
    ((6, 4, 5, 64), (0, 0, 1, 1), (0, 1)),
    ((40, 3, 5, 8), (0, 0, 0, 2), (0, 2)),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("square", [False, True])
@pytest.mark.parametrize("local,halo,axes", REDUCE_CASES)
def test_reduce_sum_matches_oracle_and_is_deterministic(local, halo, axes, square, dtype, oracle_mod):
    rng = np.random.default_rng(21)
    src, ssl, gs, bs = _haloed(rng, local, halo, dtype)
    dshape = tuple(1 if i in axes else e for i, e in enumerate(local))
    dst, _, gd, _ = _haloed(rng, dshape, (0,) * len(local), dtype)
    want = dst.copy()
    oracle_mod.tensor_reduce_sum(src[ssl], want, square)
    got = _reduce(src, ssl, gs, bs, dst, gd, square, dtype)
    again = _reduce(src, ssl, gs, bs, dst, gd, square, dtype)
    assert np.array_equal(got, again)                       # fixed order of additions
    x = src[ssl].astype(np.float64)
    scale = np.abs(x * x if square else x).sum(axis=axes, keepdims=True) + np.abs(dst)
    tol = TOL if dtype == np.float32 else 1e-12
    assert (np.abs(got.astype(np.float64) - want) <= tol * scale).all()


def test_reduce_sum_reference_closed_form(oracle_mod):
    """test_reduce of the reference: offsets in, plain sums out, then one cell =
    (size - 1) * size / 2 (test_tensor_mpi_cuda_algorithms.cu:218-300); float64 keeps it exact."""
    local = (4, 6, 10, 12)
    rng = np.random.default_rng(0)
    src, ssl, gs, bs = _haloed(rng, local, (0, 0, 1, 1), np.float64)
    src[ssl] = np.arange(int(np.prod(local)), dtype=np.float64).reshape(local)
    mid, _, gm, _ = _haloed(rng, (1, 6, 1, 1), (0, 0, 0, 0), np.float64)
    mid[...] = 0
    got = _reduce(src, ssl, gs, bs, mid, gm, False, np.float64)
    assert np.array_equal(got.ravel(), src[ssl].sum(axis=(0, 2, 3)))
    one, _, go, _ = _haloed(rng, (1, 1, 1, 1), (0, 0, 0, 0), np.float64)
    one[...] = 0
    total = _reduce(got, tuple(slice(None) for _ in range(4)), gm, 0, one, go, False, np.float64)
    size = int(np.prod(local))
    assert total.item() == (size - 1) * size / 2


def test_transform_and_reduce_reject_bad_calls():
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    rng = np.random.default_rng(1)
    a, _, ga, _ = _haloed(rng, (2, 3, 4), (0, 0, 0), np.float32)
    b, _, gb, _ = _haloed(rng, (2, 4, 3), (0, 0, 0), np.float32)
    da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    gp = (ctypes.POINTER(capi.TensorGeometry) * 2)(ctypes.pointer(ga), ctypes.pointer(gb))
    tp = (ctypes.c_void_p * 2)(da.data_ptr(), db.data_ptr())
    pp = (ctypes.c_double * 4)(1, 0, 0, 0)
    assert lib.h2x_tensor_transform(capi.TRANSFORM_COPY, capi.F32, 2, gp, tp, pp, None) == -1   # shapes differ
    assert lib.h2x_tensor_transform(capi.TRANSFORM_COPY, capi.F32, 1, gp, tp, pp, None) == -1   # wrong count
    assert lib.h2x_tensor_transform(17, capi.F32, 1, gp, tp, pp, None) == -2
    assert lib.h2x_tensor_transform(capi.TRANSFORM_SCALE, 5, 1, gp, tp, pp, None) == -2
    ws = torch.empty(1 << 16, dtype=torch.uint8, device="cuda")
    assert lib.h2x_tensor_reduce_sum(capi.F32, ctypes.byref(ga), da.data_ptr(), ctypes.byref(gb), db.data_ptr(),
                                     0, ws.data_ptr(), None) == -1                               # extent 4 -> 3
    torch.cuda.synchronize()
    assert np.array_equal(da.cpu().numpy(), a) and np.array_equal(db.cpu().numpy(), b)

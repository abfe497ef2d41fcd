"""GPU parity at the edges of the C ABI: base pointers that are not 16-byte
aligned, real (haloed) sizes larger than the local ones, and the status codes
of rejected calls (nothing may be launched or written by a rejected call).

The dense geometry is the one the reference's optimised kernels accept
(legacy/src/dnn_backend/batchnorm.cu:134-190, 210-230): a halo only on the
outermost spatial dimension makes spatial_real > spatial and moves the base
pointer off the start of the allocation."""
import ctypes

import numpy as np
import pytest

from helpers import max_rel

pytestmark = pytest.mark.gpu
TOL = 1e-5
POISON = -777.0


def _ptr(t, offset_elems=0):
    return ctypes.c_void_p(t.data_ptr() + offset_elems * t.element_size())


@pytest.mark.parametrize("offset", [0, 1, 2, 3])
@pytest.mark.parametrize("spatial,real", [(37, 41), (64, 64), (64, 68), (5, 9),
                                          # long segments that are no multiple of 4 long or start off a 16-byte
                                          # boundary: unaligned vectors, single elements at the end of a segment
                                          (1027, 1031), (1028, 1028), (1030, 1040), (1025, 1025)])
def test_bn_dense_unaligned_padded(offset, spatial, real, oracle_mod):
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    n, c = 3, 5
    rng = np.random.default_rng(100 * offset + spatial)
    x = rng.standard_normal((n, c, spatial)).astype(np.float32)
    dy = rng.standard_normal((n, c, spatial)).astype(np.float32)
    scale = rng.uniform(0.5, 1.5, c).astype(np.float32)
    bias = (0.1 * rng.standard_normal(c)).astype(np.float32)

    def padded(a):  # [n][c][real] with poison in the padding, `offset` elements in front
        full = np.full(offset + n * c * real, POISON, np.float32)
        view = full[offset:].reshape(n, c, real)
        if a is not None:
            view[:, :, :spatial] = a
        return torch.from_numpy(full).cuda()

    xd, dyd, yd, dxd = padded(x), padded(dy), padded(None), padded(None)
    dev = lambda a: torch.from_numpy(a.copy()).cuda()
    mean, var = torch.empty(c, device="cuda"), torch.empty(c, device="cuda")
    rm, rv = torch.zeros(c, device="cuda"), torch.ones(c, device="cuda")
    sc, bi = dev(scale), dev(bias)
    grads = [torch.empty(c, device="cuda") for _ in range(4)]
    ws = torch.empty(lib.h2x_bn_workspace_bytes(c), dtype=torch.uint8, device="cuda")
    nps = n * spatial
    F = capi.F32
    capi.check(lib.h2x_bn_channel_sums_and_sqsums(F, n, c, spatial, real, _ptr(xd, offset), _ptr(mean),
                                                  _ptr(var), _ptr(ws), None))
    capi.check(lib.h2x_bn_sums_to_statistics(F, c, nps, 0.9, _ptr(mean), _ptr(var), _ptr(rm), _ptr(rv),
                                             None))
    capi.check(lib.h2x_bn_batch_normalization(F, n, c, spatial, real, real, _ptr(xd, offset), _ptr(mean),
                                              _ptr(var), _ptr(sc), _ptr(bi), _ptr(yd, offset), 1e-5, None))
    capi.check(lib.h2x_bn_backprop1(F, n, c, spatial, real, real, _ptr(xd, offset), _ptr(dyd, offset),
                                    _ptr(mean), _ptr(var), _ptr(sc), *[_ptr(g) for g in grads], 1e-5,
                                    _ptr(ws), None))
    capi.check(lib.h2x_bn_backprop2(F, n, c, spatial, real, real, real, nps, _ptr(xd, offset),
                                    _ptr(dyd, offset), _ptr(mean), _ptr(var), _ptr(sc), _ptr(grads[2]),
                                    _ptr(grads[3]), _ptr(dxd, offset), 1e-5, None))
    torch.cuda.synchronize()

    x4, dy4 = x.reshape(n, c, spatial, 1), dy.reshape(n, c, spatial, 1)
    rm_o, rv_o = np.zeros(c, np.float32), np.ones(c, np.float32)
    y_o, mean_o, var_o = oracle_mod.bn_forward(x4, scale, bias, rm_o, rv_o, 1e-5, 0.9)
    dx_o, ds_o, db_o, dm_o, dv_o = oracle_mod.bn_backward(x4, dy4, mean_o, var_o, scale, 1e-5)
    assert max_rel(mean.cpu().numpy(), mean_o) <= TOL and max_rel(var.cpu().numpy(), var_o) <= TOL
    for got, want in zip(grads, (ds_o, db_o, dm_o, dv_o)):
        assert max_rel(got.cpu().numpy(), want) <= TOL
    for got, want in ((yd, y_o), (dxd, dx_o)):
        full = got.cpu().numpy()
        view = full[offset:].reshape(n, c, real)
        assert max_rel(view[:, :, :spatial], want.reshape(n, c, spatial)) <= TOL
        assert (view[:, :, spatial:] == POISON).all(), "padding between segments was written"
        assert (full[:offset] == POISON).all()


def test_softmax_unaligned(oracle_mod):
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    n, c, s = 2, 21, 77
    rng = np.random.default_rng(5)
    x = (2 * rng.standard_normal((n, c, s))).astype(np.float32)
    dy = rng.standard_normal((n, c, s)).astype(np.float32)
    for offset in (1, 2, 3):
        mk = lambda a: torch.from_numpy(np.concatenate([np.full(offset, POISON, np.float32),
                                                         a.ravel()])).cuda()
        xd, dyd = mk(x), mk(dy)
        yd, dxd = mk(np.zeros_like(x)), mk(np.zeros_like(x))
        capi.check(lib.h2x_softmax_channel_forward(capi.F32, n, c, s, _ptr(xd, offset), _ptr(yd, offset),
                                                   None))
        capi.check(lib.h2x_softmax_channel_backward(capi.F32, n, c, s, _ptr(yd, offset), _ptr(dyd, offset),
                                                    _ptr(dxd, offset), None))
        torch.cuda.synchronize()
        y_o = oracle_mod.softmax_channel_forward(x.reshape(n, c, s, 1))
        y_g = yd.cpu().numpy()[offset:]
        assert max_rel(y_g, y_o.ravel()) <= TOL
        # the backward pass is compared on the same y (dx = y * (dy - dp) cancels)
        dx_o = oracle_mod.softmax_channel_backward(y_g.reshape(n, c, s, 1).copy(), dy.reshape(n, c, s, 1))
        assert max_rel(dxd.cpu().numpy()[offset:], dx_o.ravel()) <= TOL
        assert (yd.cpu().numpy()[:offset] == POISON).all()


def test_rejected_calls_return_status_and_write_nothing():
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    c = 4
    x = torch.ones(2 * c * 8, device="cuda")
    out = [torch.full((c,), POISON, device="cuda") for _ in range(4)]
    ws = torch.empty(lib.h2x_bn_workspace_bytes(c), dtype=torch.uint8, device="cuda")
    INVALID, UNSUPPORTED = -1, -2
    p = _ptr
    # unknown dtype
    assert lib.h2x_bn_channel_sums_and_sqsums(7, 2, c, 8, 8, p(x), p(out[0]), p(out[1]), p(ws), None) == UNSUPPORTED
    # negative sizes, real < local, null outputs / workspace
    assert lib.h2x_bn_channel_sums_and_sqsums(capi.F32, -1, c, 8, 8, p(x), p(out[0]), p(out[1]), p(ws), None) == INVALID
    assert lib.h2x_bn_channel_sums_and_sqsums(capi.F32, 2, c, 8, 7, p(x), p(out[0]), p(out[1]), p(ws), None) == INVALID
    assert lib.h2x_bn_channel_sums_and_sqsums(capi.F32, 2, c, 8, 8, p(x), None, p(out[1]), p(ws), None) == INVALID
    assert lib.h2x_bn_channel_sums_and_sqsums(capi.F32, 2, c, 8, 8, p(x), p(out[0]), p(out[1]), None, None) == INVALID
    assert lib.h2x_bn_channel_sums_and_sqsums(capi.F32, 2, c, 8, 8, None, p(out[0]), p(out[1]), p(ws), None) == INVALID
    assert lib.h2x_bn_batch_normalization(capi.F32, 2, c, 8, 8, 4, p(x), p(out[0]), p(out[1]), p(out[2]),
                                          p(out[3]), p(x), 1e-5, None) == INVALID
    assert lib.h2x_bn_backprop1(capi.F32, 2, c, 8, 8, 8, p(x), p(x), p(out[0]), p(out[1]), p(out[2]),
                                p(out[0]), p(out[1]), p(out[2]), None, 1e-5, p(ws), None) == INVALID
    assert lib.h2x_softmax_channel_forward(capi.F32, -2, c, 8, p(x), p(x), None) == INVALID
    assert lib.h2x_softmax_channel_forward(9, 2, c, 8, p(x), p(x), None) == UNSUPPORTED
    # strided geometry: more than three spatial dimensions, or an innermost stride other than 1
    g = capi.TensorGeometry()
    g.num_dims = 6
    assert lib.h2x_bn_channel_sums_and_sqsums_strided(capi.F32, 2, ctypes.byref(g), p(x), p(out[0]),
                                                      p(out[1]), p(ws), None) == INVALID
    g.num_dims = 4
    for i, (e, s) in enumerate(zip((4, 2, c, 2), (2, 8, 16, 64))):
        g.local_shape[i], g.strides[i] = e, s
    assert lib.h2x_bn_channel_sums_and_sqsums_strided(capi.F32, 2, ctypes.byref(g), p(x), p(out[0]),
                                                      p(out[1]), p(ws), None) == UNSUPPORTED
    # two geometries with equal channel count and equal spatial size but other extents
    # (4 x 2 against 2 x 4) would pair different elements: rejected
    ga, gb = capi.TensorGeometry(), capi.TensorGeometry()
    ga.num_dims = gb.num_dims = 4
    for i, (e, s) in enumerate(zip((4, 2, c, 2), (1, 4, 8, 8 * c))):
        ga.local_shape[i], ga.strides[i] = e, s
    for i, (e, s) in enumerate(zip((2, 4, c, 2), (1, 2, 8, 8 * c))):
        gb.local_shape[i], gb.strides[i] = e, s
    y = torch.full_like(x, POISON)
    assert lib.h2x_bn_batch_normalization_strided(
        capi.F32, 2, ctypes.byref(ga), ctypes.byref(gb), p(x), p(out[0]), p(out[1]), p(out[2]), p(out[3]),
        p(y), 1e-5, None) == INVALID
    assert lib.h2x_bn_backprop1_strided(
        capi.F32, 2, ctypes.byref(ga), ctypes.byref(gb), p(x), p(x), p(x), p(x), p(x), p(out[0]), p(out[1]),
        p(out[2]), p(out[3]), 1e-5, p(ws), None) == INVALID
    assert lib.h2x_bn_backprop2_strided(
        capi.F32, 2, 16, ctypes.byref(ga), ctypes.byref(ga), ctypes.byref(gb), p(x), p(x), p(x), p(x), p(x),
        p(x), p(x), p(y), 1e-5, None) == INVALID
    torch.cuda.synchronize()
    assert (y == POISON).all()
    for o in out:
        assert (o == POISON).all()
    assert (x == 1).all()
    for status in (0, INVALID, UNSUPPORTED, -3, 1):
        assert lib.h2x_status_string(status)  # every status has a text


def test_zero_sized_calls_are_noops_or_zero_fill():
    """Empty local tensors: the reductions zero their outputs, the elementwise
    passes do nothing (batchnorm.cu:145-146, 207-208, 470-471)."""
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    c = 6
    out = [torch.full((c,), POISON, device="cuda") for _ in range(4)]
    vec = torch.ones(c, device="cuda")
    ws = torch.empty(lib.h2x_bn_workspace_bytes(c), dtype=torch.uint8, device="cuda")
    p = _ptr
    capi.check(lib.h2x_bn_channel_sums_and_sqsums(capi.F32, 0, c, 16, 16, None, p(out[0]), p(out[1]), p(ws), None))
    capi.check(lib.h2x_bn_backprop1(capi.F32, 4, c, 0, 0, 0, None, None, p(vec), p(vec), p(vec), p(out[0]),
                                    p(out[1]), p(out[2]), p(out[3]), 1e-5, p(ws), None))
    capi.check(lib.h2x_bn_batch_normalization(capi.F32, 0, c, 16, 16, 16, None, p(vec), p(vec), p(vec),
                                              p(vec), None, 1e-5, None))
    capi.check(lib.h2x_softmax_channel_forward(capi.F32, 0, c, 16, None, None, None))
    torch.cuda.synchronize()
    for o in out:
        assert (o == 0).all()


def test_guard_zones_of_the_test_tensors_detect_a_stray_store(guarded_tensor_allocations):
    """The guard zones every GPU test's tensors lie between: a store one element in front of or
    behind the allocation is reported, a store inside it (halo cells included) is not."""
    import helpers
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    dist = Distribution.make_overlapped_distribution([2, 2, 1, 1], [1, 1, 0, 0])
    t = Tensor([12, 10, 3, 2], LocaleVirtual(0, 4), dist).allocate()
    mine = [a for a in guarded_tensor_allocations if a[2] == tuple(t.local_real_shape)]
    assert len(mine) == 1 and t.data.data_ptr() % 16 == 0
    raw, guard_bytes, _ = mine[0]
    t.real_view().fill_(1.0)   # the whole allocation, halo included
    helpers.check_guards(mine)
    elem = t.data.element_size()
    for at in (guard_bytes - elem, raw.numel() - guard_bytes):   # last element in front, first behind
        saved = raw[at:at + elem].clone()
        raw[at:at + elem] = 0
        with pytest.raises(AssertionError, match="wrote outside a tensor"):
            helpers.check_guards(mine)
        raw[at:at + elem] = saved
    helpers.check_guards(mine)

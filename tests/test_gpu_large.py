"""Tensors with more than 2^31 elements: the dense batch-norm kernels index with
64-bit offsets, and the result is checked through closed forms that are exact
in fp32 (a constant channel has sum = n * value, variance 0 and y = bias)."""
import ctypes

import pytest

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def test_batchnorm_beyond_2_31_elements():
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    n, c = 1, 2
    spatial = (1 << 30) + (1 << 20)  # exactly representable in fp32, and c * spatial > 2^31
    free, _ = torch.cuda.mem_get_info()
    if free < 3 * c * spatial * 4:
        pytest.skip("not enough device memory")
    x = torch.empty(n * c * spatial, device="cuda")
    x[:spatial].fill_(1.0)
    x[spatial:].fill_(2.0)
    sums, sqsums = torch.empty(c, device="cuda"), torch.empty(c, device="cuda")
    ws = torch.empty(lib.h2x_bn_workspace_bytes(c), dtype=torch.uint8, device="cuda")
    capi.check(lib.h2x_bn_channel_sums_and_sqsums(capi.F32, n, c, spatial, spatial, _ptr(x), _ptr(sums),
                                                  _ptr(sqsums), _ptr(ws), None))
    torch.cuda.synchronize()
    assert sums.tolist() == [float(spatial), 2.0 * spatial]
    assert sqsums.tolist() == [float(spatial), 4.0 * spatial]
    # statistics: mean 1 and 2, variance 0; y = bias everywhere, dx through backprop2 = dy * scale * r
    rm, rv = torch.zeros(c, device="cuda"), torch.ones(c, device="cuda")
    capi.check(lib.h2x_bn_sums_to_statistics(capi.F32, c, n * spatial, 0.9, _ptr(sums), _ptr(sqsums), _ptr(rm),
                                             _ptr(rv), None))
    torch.cuda.synchronize()
    assert sums.tolist() == [1.0, 2.0] and sqsums.tolist() == [0.0, 0.0]
    scale = torch.tensor([3.0, 5.0], device="cuda")
    bias = torch.tensor([0.25, -0.5], device="cuda")
    y = torch.empty_like(x)
    capi.check(lib.h2x_bn_batch_normalization(capi.F32, n, c, spatial, spatial, spatial, _ptr(x), _ptr(sums),
                                              _ptr(sqsums), _ptr(scale), _ptr(bias), _ptr(y), 1e-5, None))
    torch.cuda.synchronize()
    assert bool((y[:spatial] == 0.25).all()) and bool((y[spatial:] == -0.5).all())
    # backward reductions with dy = x: dbias = sum dy, dscale = 0 (x - mean = 0)
    grads = [torch.empty(c, device="cuda") for _ in range(4)]
    capi.check(lib.h2x_bn_backprop1(capi.F32, n, c, spatial, spatial, spatial, _ptr(x), _ptr(x), _ptr(sums),
                                    _ptr(sqsums), _ptr(scale), *[_ptr(g) for g in grads], 1e-5, _ptr(ws), None))
    torch.cuda.synchronize()
    assert grads[0].tolist() == [0.0, 0.0]
    assert grads[1].tolist() == [float(spatial), 2.0 * spatial]


def test_halo_faces_beyond_2_31_elements():
    """Strips that start more than 2^31 elements into the tensor (64-bit offsets
    in the copy kernel), dense and sparse faces, pack and unpack, bit-exact."""
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    w, h, c = 1024, 1024, 2100  # 2.2e9 elements
    free, _ = torch.cuda.mem_get_info()
    if free < 2 * w * h * c * 4:
        pytest.skip("not enough device memory")
    t = torch.empty((1, c, h, w), device="cuda")
    t.view(-1)[: 1 << 20].uniform_(-1, 1)
    t.view(-1).copy_(t.view(-1)[: 1 << 20].repeat(c * h * w >> 20)[: c * h * w])  # cheap non-constant fill
    t[0, :, :, :] += torch.arange(c, device="cuda", dtype=torch.float32).view(c, 1, 1)
    shape = capi.i64_array((w, h, c, 1))
    for dim, expect in ((1, lambda: t[0, :, h - 2, :]), (0, lambda: t[0, :, :, w - 2])):
        n = lib.h2x_halo_size(4, shape, dim, 1)
        buf = torch.full((n,), float("nan"), device="cuda")
        capi.check(lib.h2x_halo_pack_or_unpack(capi.F32, _ptr(t), 4, shape, dim, capi.RHS, 1, _ptr(buf), 1, 0, 0,
                                               None))
        torch.cuda.synchronize()
        assert torch.equal(buf, expect().reshape(-1))
        # unpack the negated strip into the outer halo cells of the same side
        buf.neg_()
        capi.check(lib.h2x_halo_pack_or_unpack(capi.F32, _ptr(t), 4, shape, dim, capi.RHS, 1, _ptr(buf), 0, 0, 0,
                                               None))
        torch.cuda.synchronize()
        outer = t[0, :, h - 1, :] if dim == 1 else t[0, :, :, w - 1]
        assert torch.equal(outer.reshape(-1), buf)

"""h2x_bn_channel_sums_and_sqsums_static (the entry point that allocates
nothing: partial sums in an array inside the library's device image) against
h2x_bn_channel_sums_and_sqsums with a caller-provided workspace, through the C
ABI.  Same kernels and order of additions, so the results must be identical
bit for bit; two calls in a row, the second on a smaller input, so that what the
first call left in the shared array would show."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _sums(lib, capi, torch, x, static):
    n, c = x.shape[0], x.shape[1]
    spatial = int(np.prod(x.shape[2:]))
    sums = torch.full((c,), float("nan"), device="cuda")
    sqsums = torch.full((c,), float("nan"), device="cuda")
    if static:
        capi.check(lib.h2x_bn_channel_sums_and_sqsums_static(
            capi.F32, n, c, spatial, spatial, x.data_ptr(), sums.data_ptr(), sqsums.data_ptr(), None),
            "static sums")
    else:
        ws = torch.empty(lib.h2x_bn_workspace_bytes(c), dtype=torch.uint8, device="cuda")
        capi.check(lib.h2x_bn_channel_sums_and_sqsums(
            capi.F32, n, c, spatial, spatial, x.data_ptr(), sums.data_ptr(), sqsums.data_ptr(),
            ws.data_ptr(), None), "sums")
    torch.cuda.synchronize()
    return sums.cpu().numpy(), sqsums.cpu().numpy()


def test_static_scratch_entry_point_matches_workspace_entry_point():
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    g = torch.Generator(device="cuda").manual_seed(99)
    # first a large input (many workgroups per channel), then a smaller one with
    # fewer channels and fewer partial sums per channel, then short segments (another
    # family of kernels, which lays its partial sums out range by range)
    for shape in ((4, 64, 32, 32, 32), (2, 5, 7, 9, 11), (300, 40, 7, 7), (3, 70, 14, 14)):
        x = torch.empty(shape, device="cuda").normal_(0, 1, generator=g)
        want = _sums(lib, capi, torch, x, static=False)
        got = _sums(lib, capi, torch, x, static=True)
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1]), shape
        assert np.isfinite(got[0]).all() and np.isfinite(got[1]).all()
        # and against float64 arithmetic on the host (fp64 accumulation on the device, one rounding)
        xh = x.cpu().numpy().astype(np.float64)
        axes = (0,) + tuple(range(2, xh.ndim))
        np.testing.assert_allclose(got[0], xh.sum(axis=axes), rtol=1e-6, atol=1e-4)
        np.testing.assert_allclose(got[1], (xh * xh).sum(axis=axes), rtol=1e-6)


def test_static_scratch_entry_point_rejects_too_many_channels():
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    limit = lib.h2x_bn_static_max_channels()
    assert limit >= 2048
    out = torch.zeros(2 * (limit + 1), device="cuda")
    x = torch.zeros(limit + 1, device="cuda")
    status = lib.h2x_bn_channel_sums_and_sqsums_static(
        capi.F32, 1, limit + 1, 1, 1, x.data_ptr(), out.data_ptr(), out.data_ptr() + 4 * (limit + 1), None)
    assert status == -4  # H2X_ERR_SCRATCH_LIMIT
    assert b"static scratch" in lib.h2x_status_string(status)
    torch.cuda.synchronize()
    assert (out == 0).all()  # nothing was launched

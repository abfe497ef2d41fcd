"""GPU parity: channel softmax entry points against the CPU oracle.

Tolerance 1e-5 relative, metric max(|d/v1|, |d/v2|).  The reference holds no
softmax test; the oracle is pinned by torch.softmax and its autograd in fp64
(tests/test_oracle_softmax.py).
"""
import numpy as np
import pytest

from helpers import max_rel

pytestmark = pytest.mark.gpu
TOL = 1e-5

CASES = [
    (16, 21, 64, 64),     # BASELINE config 4 at reduced spatial size (full size in test_gpu_full_size.py)
    (2, 21, 7, 9),        # scalar path
    (3, 4, 8, 8),
    (2, 1, 4, 4),         # one channel
    (1, 33, 6, 10),       # more than 32 channels: the waves of a workgroup share the channels, two pixels a lane
    (2, 70, 3, 5),        # the same, one pixel a lane
    (2, 64, 8, 16),       # 16 channels a wave exactly
    (1, 200, 4, 4),       # 50 of 64 channels a wave
    (1, 384, 3, 3),       # 96 channels a wave
    (2, 150, 9, 7),
    (3, 300, 16, 16),
    (4, 1000, 1, 1),      # one pixel per sample: a wave per sample, lanes over the channels
    (70, 10, 1, 1),       # the same with fewer channels than lanes
    (3, 2048, 1, 1),      # 32 channels a lane, the most
    (2, 2100, 1, 1),      # beyond that: a workgroup per sample
    (3, 40000, 1, 1),     # a large vocabulary
    (2, 19, 4, 6, 10),    # 5-D
    (2, 256, 6, 10),      # 64 channels a wave in registers, two pixels a lane
    (2, 257, 3, 5),       # 65 of 128 channels a wave, one pixel a lane
    (1, 512, 4, 4),       # the most four waves hold
    (1, 513, 2, 2),       # eight waves share the channels
    (2, 768, 2, 3),       # the most eight waves hold backward
    (1, 800, 3, 2),       # forward in registers, backward the re-reading kernel
    (2, 1024, 3, 3),      # the most eight waves hold forward
    (1, 1025, 2, 2),      # beyond that: the re-reading kernel
    (3, 150, 40, 40),     # several workgroups a sample, the last one partly filled
    # fewer than 128 pixels a sample: the pixels are counted through all samples, a tile holds several samples
    (37, 5, 3, 5),
    (130, 40, 7, 7),
    (9, 600, 7, 7),
    (11, 1100, 3, 3),
]


def _tensors(shape, dtype="float32"):
    import torch
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    dist = Distribution.make_localized_distribution(len(shape))
    mk = lambda: Tensor(list(shape[::-1]), LocaleVirtual(0, 1), dist, getattr(torch, dtype)).allocate()
    return mk


@pytest.mark.parametrize("shape", CASES)
def test_forward_backward(shape, oracle_mod):
    import torch
    from dihydrogen_amd.layers import Softmax, SoftmaxMode
    rng = np.random.default_rng(99)
    x = (2.0 * rng.standard_normal(shape)).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    mk = _tensors(shape)
    xt, yt, dyt, dxt = mk(), mk(), mk(), mk()
    xt.real_view().copy_(torch.from_numpy(x))
    dyt.real_view().copy_(torch.from_numpy(dy))
    sm = Softmax()
    sm.setup(xt, SoftmaxMode.CHANNEL)
    assert sm.forward(xt, yt) == 0
    torch.cuda.synchronize()
    y = yt.real_view().cpu().numpy()
    y_o = oracle_mod.softmax_channel_forward(x)
    assert max_rel(y, y_o) <= TOL
    assert np.abs(y.sum(axis=1) - 1).max() < 1e-5
    # backward from the GPU's own y, compared with the oracle on the same y
    assert sm.backward(yt, dyt, dxt) == 0
    torch.cuda.synchronize()
    dx = dxt.real_view().cpu().numpy()
    dx_o = oracle_mod.softmax_channel_backward(y, dy)
    if shape[1] <= 32 and int(np.prod(shape[2:])) > 1:
        assert np.array_equal(dx, dx_o) or max_rel(dx, dx_o) <= TOL
    else:
        # above 32 channels dp = sum_c y * dy is formed from four partial sums (one pixel per
        # sample: from the lanes' partial sums), the oracle's from one running sum:
        # dx = y * (dy - dp) then agrees to the tolerance in units of
        # the terms that are added up (|dy| and sum_c |y * dy|), not of their difference
        terms = np.abs(dy) + (y.astype(np.float64) * np.abs(dy)).sum(axis=1, keepdims=True)
        bound = TOL * y * terms
        assert (np.abs(dx.astype(np.float64) - dx_o) <= bound + 1e-45).all()


def test_underflow_clamp_and_guard(oracle_mod):
    """A logit gap > 104 underflows exp: y is clamped to FLT_MIN and the
    backward guard y > FLT_MIN zeroes the gradient
    (legacy/src/dnn_backend/softmax.cu:557,590,634,666)."""
    import torch
    from dihydrogen_amd.layers import Softmax, SoftmaxMode
    shape = (1, 4, 2, 4)
    x = np.zeros(shape, np.float32)
    x[:, 0] = 120.0
    x[:, 3] = -50.0
    dy = np.ones(shape, np.float32)
    dy[:, 1] = 2.0
    mk = _tensors(shape)
    xt, yt, dyt, dxt = mk(), mk(), mk(), mk()
    xt.real_view().copy_(torch.from_numpy(x))
    dyt.real_view().copy_(torch.from_numpy(dy))
    sm = Softmax()
    sm.setup(xt, SoftmaxMode.CHANNEL)
    sm.forward(xt, yt)
    sm.backward(yt, dyt, dxt)
    torch.cuda.synchronize()
    y = yt.real_view().cpu().numpy()
    dx = dxt.real_view().cpu().numpy()
    flt_min = np.finfo(np.float32).tiny
    assert (y[:, 1:] == flt_min).all() and (y[:, 0] == 1.0).all()
    assert (dx[:, 1:] == 0).all()
    assert np.array_equal(y, oracle_mod.softmax_channel_forward(x))
    assert np.array_equal(dx, oracle_mod.softmax_channel_backward(y, dy))


def test_all_negative_logits_keep_reference_maximum(oracle_mod):
    """The running maximum starts at FLT_MIN, so all-negative logits are
    shifted by ~0, not by their maximum (softmax.cu:565)."""
    import torch
    from dihydrogen_amd.layers import Softmax, SoftmaxMode
    shape = (1, 5, 2, 4)
    rng = np.random.default_rng(5)
    x = (-1.0 - rng.uniform(0, 3, shape)).astype(np.float32)
    mk = _tensors(shape)
    xt, yt = mk(), mk()
    xt.real_view().copy_(torch.from_numpy(x))
    sm = Softmax()
    sm.setup(xt, SoftmaxMode.CHANNEL)
    sm.forward(xt, yt)
    torch.cuda.synchronize()
    assert max_rel(yt.real_view().cpu().numpy(), oracle_mod.softmax_channel_forward(x)) <= TOL


@pytest.mark.parametrize("shape", [(2, 9, 4, 6), (2, 100, 4, 6), (1, 200, 3, 3), (1, 300, 2, 2), (3, 130, 1, 1)])
def test_float64(shape, oracle_mod):
    import torch
    from dihydrogen_amd.layers import Softmax, SoftmaxMode
    rng = np.random.default_rng(17)
    x = 2.0 * rng.standard_normal(shape)
    dy = rng.standard_normal(shape)
    mk = _tensors(shape, "float64")
    xt, yt, dyt, dxt = mk(), mk(), mk(), mk()
    xt.real_view().copy_(torch.from_numpy(x))
    dyt.real_view().copy_(torch.from_numpy(dy))
    sm = Softmax()
    sm.setup(xt, SoftmaxMode.CHANNEL)
    sm.forward(xt, yt)
    sm.backward(yt, dyt, dxt)
    torch.cuda.synchronize()
    y = yt.real_view().cpu().numpy()
    assert max_rel(y, oracle_mod.softmax_channel_forward(x)) <= 1e-12
    assert max_rel(dxt.real_view().cpu().numpy(), oracle_mod.softmax_channel_backward(y, dy)) <= 1e-12


INSTANCE_CASES = [(16, 21, 64, 64), (3, 4, 5, 6), (2, 7, 9), (1, 2, 3, 4, 5), (5, 1, 1, 1), (2, 64, 128, 128),
                  # samples of at most 2048 elements: a wave per sample
                  (300, 10, 1, 1), (7, 1000, 1, 1), (3, 2048, 1, 1), (130, 5, 13, 1),
                  # to 8192 elements: a workgroup per sample
                  (2, 2049, 1, 1), (5, 4096), (3, 4097), (4, 8192), (2, 8193)]


@pytest.mark.parametrize("shape", INSTANCE_CASES)
def test_instance_mode(shape, oracle_mod):
    """SoftmaxMode::INSTANCE (legacy/src/dnn_backend/softmax.cu:705-784) against the oracle."""
    import torch
    from dihydrogen_amd.layers import Softmax, SoftmaxMode
    rng = np.random.default_rng(123)
    x = (2.0 * rng.standard_normal(shape)).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    mk = _tensors(shape)
    xt, yt, dyt, dxt = mk(), mk(), mk(), mk()
    xt.real_view().copy_(torch.from_numpy(x))
    dyt.real_view().copy_(torch.from_numpy(dy))
    sm = Softmax()
    sm.setup(xt, SoftmaxMode.INSTANCE)
    assert sm.forward(xt, yt) == 0
    torch.cuda.synchronize()
    y = yt.real_view().cpu().numpy()
    assert max_rel(y, oracle_mod.softmax_instance_forward(x)) <= TOL
    assert sm.backward(yt, dyt, dxt) == 0
    torch.cuda.synchronize()
    # dp is a sum of signed terms; dx = y * (dy - dp): compare relative to the operands
    dx, dx_o = dxt.real_view().cpu().numpy(), oracle_mod.softmax_instance_backward(y, dy)
    n = shape[0]
    bound = 1e-5 * np.abs(y) * (np.abs(dy) + np.abs(y * dy).reshape(n, -1).sum(axis=1).reshape((n,) + (1,) * (len(shape) - 1)))
    assert (np.abs(dx - dx_o) <= bound + 1e-30).all()


def test_instance_mode_split_sample_allreduce(oracle_mod):
    """Two virtual ranks each hold half of every sample; the per-sample scalars
    are combined through the allreduce hook (softmax.hpp:52-62)."""
    import torch
    from dihydrogen_amd.layers import Softmax, SoftmaxMode
    rng = np.random.default_rng(77)
    full = (2.0 * rng.standard_normal((4, 6, 8, 16))).astype(np.float32)
    halves = [np.ascontiguousarray(full[:, :, :4]), np.ascontiguousarray(full[:, :, 4:])]
    want = oracle_mod.softmax_instance_forward(full)
    shape = halves[0].shape
    mk = _tensors(shape)
    xs, ys = [mk(), mk()], [mk(), mk()]
    for t, h in zip(xs, halves):
        t.real_view().copy_(torch.from_numpy(h))
    # lock-step emulation: run rank 0's stage, then rank 1's, exchanging scalars in between
    lib = __import__("dihydrogen_amd.capi", fromlist=["x"]).load()
    from dihydrogen_amd import capi
    n, size = shape[0], int(np.prod(shape[1:]))
    ws = torch.empty(lib.h2x_softmax_instance_workspace_bytes(n), dtype=torch.uint8, device="cuda")
    mx = [torch.empty(n, device="cuda") for _ in range(2)]
    ex = [torch.empty(n, device="cuda") for _ in range(2)]
    for r in range(2):
        capi.check(lib.h2x_softmax_instance_max(capi.F32, n, size, xs[r].get_base_ptr(), mx[r].data_ptr(), ws.data_ptr(), None))
    m = torch.maximum(mx[0], mx[1])
    for r in range(2):
        capi.check(lib.h2x_softmax_instance_exp(capi.F32, n, size, xs[r].get_base_ptr(), m.data_ptr(),
                                                ys[r].get_base_ptr(), ex[r].data_ptr(), ws.data_ptr(), None))
    e = ex[0] + ex[1]
    for r in range(2):
        capi.check(lib.h2x_softmax_instance_normalize(capi.F32, n, size, e.data_ptr(), ys[r].get_base_ptr(), None))
    torch.cuda.synchronize()
    got = np.concatenate([ys[0].real_view().cpu().numpy(), ys[1].real_view().cpu().numpy()], axis=2)
    assert max_rel(got, want) <= TOL


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("shape", INSTANCE_CASES + [(3, 1031)])
def test_instance_forward_in_four_passes_equals_the_staged_calls(shape, dtype):
    """h2x_softmax_instance_forward_local (whole samples on this rank: the exponentials are
    summed without being stored and made again from x) against the three staged calls:
    y, the per-sample maxima and the per-sample sums must agree bit for bit."""
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    rng = np.random.default_rng(5)
    x = (2.0 * rng.standard_normal(shape)).astype(dtype)
    n, size = shape[0], int(np.prod(shape[1:]))
    dt = capi.F32 if dtype == np.float32 else capi.F64
    xd = torch.from_numpy(x).cuda()
    ws = torch.empty(lib.h2x_softmax_instance_workspace_bytes(n), dtype=torch.uint8, device="cuda")
    tdt = torch.float32 if dtype == np.float32 else torch.float64
    outs = []
    for local in (True, False):
        y = torch.full(shape, float("nan"), dtype=tdt, device="cuda")
        mx = torch.full((n,), float("nan"), dtype=tdt, device="cuda")
        ex = torch.full((n,), float("nan"), dtype=tdt, device="cuda")
        if local:
            capi.check(lib.h2x_softmax_instance_forward_local(dt, n, size, xd.data_ptr(), y.data_ptr(), mx.data_ptr(),
                                                              ex.data_ptr(), ws.data_ptr(), None))
        else:
            capi.check(lib.h2x_softmax_instance_max(dt, n, size, xd.data_ptr(), mx.data_ptr(), ws.data_ptr(), None))
            capi.check(lib.h2x_softmax_instance_exp(dt, n, size, xd.data_ptr(), mx.data_ptr(), y.data_ptr(),
                                                    ex.data_ptr(), ws.data_ptr(), None))
            capi.check(lib.h2x_softmax_instance_normalize(dt, n, size, ex.data_ptr(), y.data_ptr(), None))
        torch.cuda.synchronize()
        outs.append([t.cpu().numpy() for t in (y, mx, ex)])
    for name, a, b in zip(("y", "sample_max", "sample_exp"), *outs):
        assert np.array_equal(a, b), name


@pytest.mark.parametrize("shape", [(2, 21, 8, 8), (1, 200, 4, 4)])
def test_non_finite_logits_propagate_as_in_the_oracle(shape, oracle_mod):
    """A NaN, +inf and -inf logit, each at a pixel of its own, in the register kernel and
    in the kernel that shares channels between waves: NaNs at the same positions as the
    oracle's, the finite outputs within the tolerance, the other pixels unaffected."""
    import torch
    from dihydrogen_amd.layers import Softmax, SoftmaxMode
    rng = np.random.default_rng(41)
    x = (2.0 * rng.standard_normal(shape)).astype(np.float32)
    x[0, 3, 1, 1] = np.nan
    x[0, 5, 2, 2] = np.inf
    x[0, 7, 3, 3] = -np.inf
    mk = _tensors(shape)
    xt, yt = mk(), mk()
    xt.real_view().copy_(torch.from_numpy(x))
    sm = Softmax()
    sm.setup(xt, SoftmaxMode.CHANNEL)
    assert sm.forward(xt, yt) == 0
    torch.cuda.synchronize()
    y = yt.real_view().cpu().numpy()
    with np.errstate(all="ignore"):
        y_o = oracle_mod.softmax_channel_forward(x)
    assert np.array_equal(np.isnan(y), np.isnan(y_o))
    ok = np.isfinite(y_o)
    assert ok.sum() > y.size // 2 and max_rel(y[ok], y_o[ok]) <= TOL

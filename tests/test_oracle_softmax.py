"""Pins the channel-softmax functions of the CPU oracle.

The reference has no softmax test at all, so outside of the library routine
the behaviour is pinned only by reading softmax.cu; what the mathematics fixes
is checked here: torch.softmax and its autograd in float64, the invariants
sum_c y = 1 and sum_c dx = 0, shift invariance, and the FLT_MIN clamp / guard /
initial-maximum quirks of legacy/src/dnn_backend/softmax.cu:557-590,634-666.
"""
import glob
import os

import numpy as np
import pytest

import oracle
from helpers import max_rel

FLT_MIN = np.finfo(np.float32).tiny


def test_golden():
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "softmax_2x21x5x7.npz"))
    y = oracle.softmax_channel_forward(g["x"])
    assert max_rel(y, g["y"]) < 1e-6
    dx = oracle.softmax_channel_backward(g["y"].astype(np.float32), g["dy"])
    y32 = g["y"].astype(np.float32).astype(np.float64)
    cond = np.abs(y32) * (np.abs(g["dy"]) + np.abs(y32 * g["dy"]).sum(axis=1, keepdims=True))
    assert (np.abs(dx - g["dx"]) <= 1e-6 * cond + 1e-12).all()


@pytest.mark.parametrize("shape", [(2, 21, 8, 8), (3, 4, 5), (1, 7, 2, 3, 4)])
def test_against_torch(shape):
    import torch
    rng = np.random.default_rng(5)
    x = (2 * rng.standard_normal(shape)).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    yt = torch.softmax(xt, dim=1)
    yt.backward(torch.tensor(dy, dtype=torch.float64))
    y = oracle.softmax_channel_forward(x)
    assert max_rel(y, yt.detach().numpy()) < 1e-6
    dx = oracle.softmax_channel_backward(y, dy)
    assert np.abs(dx - xt.grad.numpy()).max() < 2e-6
    assert np.abs(y.astype(np.float64).sum(axis=1) - 1).max() < 1e-6
    assert np.abs(dx.astype(np.float64).sum(axis=1)).max() < 1e-6
    # shift invariance (logits with a positive maximum)
    y2 = oracle.softmax_channel_forward(x + np.float32(3.0))
    assert max_rel(y, y2) < 1e-5


def test_clamp_guard_and_initial_maximum():
    x = np.zeros((1, 3, 1, 2), np.float32)
    x[0, 0] = 200.0
    y = oracle.softmax_channel_forward(x)
    assert (y[0, 0] == 1).all() and (y[0, 1:] == FLT_MIN).all()        # clamp
    dy = np.ones_like(x)
    dy[0, 1] = 5
    dx = oracle.softmax_channel_backward(y, dy)
    assert (dx[0, 1:] == 0).all()                                       # guard y > FLT_MIN
    # the maximum starts at FLT_MIN (> 0): all-negative logits are shifted by ~0
    xn = np.array([-1.0, -2.0, -3.0], np.float32).reshape(1, 3, 1)
    e = np.exp(xn.astype(np.float64))
    assert max_rel(oracle.softmax_channel_forward(xn), e / e.sum()) < 1e-6
    xv = np.array([-200.0, -201.0], np.float32).reshape(1, 2, 1)        # exp underflows: 0 * inf
    with np.errstate(all="ignore"):
        yv = oracle.softmax_channel_forward(xv)
    assert np.isnan(yv).all() or (yv == FLT_MIN).all()


def test_float64_variant():
    rng = np.random.default_rng(6)
    x = rng.standard_normal((2, 5, 3, 3))
    e = np.exp(x - x.max(axis=1, keepdims=True))
    assert max_rel(oracle.softmax_channel_forward(x), e / e.sum(axis=1, keepdims=True)) < 1e-13


@pytest.mark.parametrize("shape", [(3, 4, 5, 6), (2, 21, 8), (1, 2, 3, 4, 5)])
def test_instance_mode_against_torch(shape):
    """Instance mode = softmax over all elements of a sample: torch.softmax on the
    flattened sample and its autograd in float64."""
    import torch
    rng = np.random.default_rng(8)
    x = (2 * rng.standard_normal(shape)).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    yt = torch.softmax(xt.reshape(shape[0], -1), dim=1).reshape(shape)
    yt.backward(torch.tensor(dy, dtype=torch.float64))
    y = oracle.softmax_instance_forward(x)
    assert max_rel(y, yt.detach().numpy()) < 2e-6
    dx = oracle.softmax_instance_backward(y, dy)
    assert np.abs(dx - xt.grad.numpy()).max() < 2e-6
    assert np.abs(y.reshape(shape[0], -1).astype(np.float64).sum(axis=1) - 1).max() < 1e-6
    assert np.abs(dx.reshape(shape[0], -1).astype(np.float64).sum(axis=1)).max() < 1e-6


def test_instance_mode_clamp_and_split_sample():
    """Clamp and guard at sqrt(FLT_MIN) (softmax.cu:156-160); a sample split over
    two ranks with the per-sample scalars all-reduced gives the unsplit result."""
    x = np.zeros((1, 2, 2, 2), np.float32)
    x[0, 0, 0, 0] = 100.0
    y = oracle.softmax_instance_forward(x)
    lim = np.float32(np.sqrt(np.float32(FLT_MIN)))
    assert y[0, 0, 0, 0] == 1 and (y.reshape(-1)[1:] == lim).all()
    assert (oracle.softmax_instance_backward(y, np.ones_like(x)).reshape(-1)[1:] == 0).all()
    # split every sample's elements over two "ranks": record each rank's local
    # scalars, combine them as the all-reduce would, then rerun with the combined values
    rng = np.random.default_rng(9)
    full = (2 * rng.standard_normal((3, 4, 6, 8))).astype(np.float32)
    halves = [np.ascontiguousarray(full[:, :, :3]), np.ascontiguousarray(full[:, :, 3:])]

    def staged(inject=None):
        """Runs both ranks stage by stage; returns y of both."""
        import ctypes
        lib = oracle.lib()
        n, size = 3, halves[0].size // 3
        mx = [np.empty(n, np.float32) for _ in range(2)]
        ex = [np.empty(n, np.float32) for _ in range(2)]
        ys = [np.empty_like(h) for h in halves]
        P = lambda a: ctypes.c_void_p(a.ctypes.data)
        for r in range(2):
            lib.orc_softmax_instance_max_f32(ctypes.c_int(n), ctypes.c_size_t(size), P(halves[r]), P(mx[r]))
        m = np.maximum(mx[0], mx[1])                      # allreduce(max)
        for r in range(2):
            lib.orc_softmax_instance_exp_f32(ctypes.c_int(n), ctypes.c_size_t(size), P(halves[r]), P(m), P(ys[r]), P(ex[r]))
        e = ex[0] + ex[1]                                 # allreduce(sum)
        for r in range(2):
            lib.orc_softmax_instance_normalize_f32(ctypes.c_int(n), ctypes.c_size_t(size), P(e), P(ys[r]))
        return ys

    y0, y1 = staged()
    want = oracle.softmax_instance_forward(full)
    assert max_rel(np.concatenate([y0, y1], axis=2), want) < 1e-6

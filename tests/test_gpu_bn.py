"""GPU parity: batch-norm entry points of libh2x.so against the CPU oracle.

Tolerance: 1e-5 relative with the reference's metric max(|d/v1|, |d/v2|)
(legacy/tests/compare_binary_files.cpp:47-49, legacy/tests/dnn_backend/
test_cudnn_util.sh.in:64-72 uses 1.5e-5).  The oracle performs the same fp32
operations in the same order with fp64 accumulation, so the match is in fact
much tighter; the asserted bound is the contract.
"""
import numpy as np
import pytest

from helpers import bn_inputs, max_rel

pytestmark = pytest.mark.gpu
TOL = 1e-5

CASES = [
    # (N, C, spatial dims...) numpy order
    (8, 64, 56, 56),        # BASELINE config 1
    (2, 3, 4, 5),           # tiny, spatial % 4 == 0
    (2, 3, 5, 7),           # scalar path (spatial % 4 != 0)
    (3, 5, 3, 4, 5),        # 5-D
    (1, 1, 1, 1),           # n == 1: unbiased variance is 0 * inf = NaN in the reference too
    (64, 16, 7, 7),         # more samples than chunks
    (2, 130, 33, 31),       # many channels, odd sizes
    (4, 8, 16, 16, 16),     # 5-D vector path
    (16, 24, 1, 1),         # one element per segment: samples folded into the spatial index
    (32, 8, 3, 3),          # short odd segments, folded, scalar
    (48, 40, 4, 4),         # short segments, folded, vector width 4
    (6, 5, 2, 7, 9),        # 5-D, 126 elements per segment
    (3, 20, 37, 37),        # long odd segments (1369 = 4 * 342 + 1): unaligned vectors and single elements at the end
    (1, 6, 19, 19),         # one sample, 361 elements
    (2, 5, 11, 11, 11),     # 1331 = 4 * 332 + 3
    (2, 4, 33, 34),         # 1122 = 4 * 280 + 2
    (5, 6, 27, 27),         # folded rows of 729: vectors that cross a row end are split
    (6, 3, 13, 13),         # folded rows of 169
    (3, 4, 5, 13),          # folded rows of 65, just above the limit for split vectors
    # short segments: a workgroup serves a window of whole channels
    (5, 300, 7, 7),         # 19 channels a window, the last window partly filled, last slot of 1 element
    (3, 70, 14, 14),        # 196 elements: whole vectors only
    (7, 33, 16, 16),        # 256 elements, the longest short segment: 4 channels a window
    (9, 260, 1, 1),         # one element per segment, two windows
    (130, 12, 2, 1),        # two elements per segment
    (2, 9, 3, 5, 17),       # 255 elements: last slot of 3
    (512, 600, 1, 1),       # few windows, many samples: four rows of lanes share a workgroup's samples
    (300, 500, 3, 3),       # the same with three slots a segment
    (37, 2, 3, 3, 3),       # 27 elements, two channels, one workgroup a range of samples
]


def _run_forward(x, scale, bias, eps=1e-5, decay=0.9, dtype="float32"):
    import torch
    from dihydrogen_amd.layers import BatchNormalization
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor

    nd = x.ndim
    shape = list(x.shape[::-1])
    tdt = getattr(torch, dtype)
    dist = Distribution.make_localized_distribution(nd)
    loc = LocaleVirtual(0, 1)
    xin = Tensor(shape, loc, dist, tdt).allocate()
    yout = Tensor(shape, loc, dist, tdt).allocate()
    xin.real_view().copy_(torch.from_numpy(x))
    c = x.shape[1]
    dev = lambda a: torch.from_numpy(a.copy()).cuda()
    mean = torch.empty(c, dtype=tdt, device="cuda")
    var = torch.empty(c, dtype=tdt, device="cuda")
    rm = torch.zeros(c, dtype=tdt, device="cuda")
    rv = torch.ones(c, dtype=tdt, device="cuda")
    bn = BatchNormalization(nd, decay, eps)
    assert bn.forward(xin, mean, var, rm, rv, dev(scale), dev(bias), yout, True) == 0
    torch.cuda.synchronize()
    return bn, xin, yout, mean, var, rm, rv


def assert_nan_parity(got, want, name):
    """NaNs and infinities in the same places (same sign), the finite elements within TOL."""
    got, want = np.asarray(got), np.asarray(want)
    assert np.array_equal(np.isnan(got), np.isnan(want)), name
    inf = np.isinf(want)
    assert np.array_equal(np.isinf(got), inf) and np.array_equal(got[inf], want[inf]), name
    ok = np.isfinite(want)
    assert max_rel(got[ok], want[ok]) <= TOL, name


@pytest.mark.parametrize("shape", CASES)
def test_forward_matches_oracle(shape, oracle_mod):
    x, dy, scale, bias = bn_inputs(shape, seed=1234)
    bn, xin, yout, mean, var, rm, rv = _run_forward(x, scale, bias)
    rm_o = np.zeros(shape[1], np.float32)
    rv_o = np.ones(shape[1], np.float32)
    y_o, mean_o, var_o = oracle_mod.bn_forward(x, scale, bias, rm_o, rv_o, 1e-5, 0.9)
    got = lambda t: t.cpu().numpy()
    if int(np.prod(shape)) // shape[1] == 1:
        # n == 1: var = max(E[x^2] - mean^2, 0) * (1 / 0) is NaN or +inf, depending on the
        # rounding of x * x (batchnorm.cu:304-306); the kernel must give what the oracle gives
        assert not np.isfinite(var_o).any()
        assert_nan_parity(got(var), var_o, "var")
        assert max_rel(got(mean), mean_o) <= TOL
        return
    assert max_rel(got(mean), mean_o) <= TOL
    assert max_rel(got(var), var_o) <= TOL
    assert max_rel(got(rm), rm_o) <= TOL
    assert max_rel(got(rv), rv_o) <= TOL
    assert max_rel(got(yout.real_view()), y_o) <= TOL


@pytest.mark.parametrize("shape", CASES)
def test_backward_matches_oracle(shape, oracle_mod):
    import torch
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor

    x, dy, scale, bias = bn_inputs(shape, seed=4321)
    bn, xin, yout, mean, var, rm, rv = _run_forward(x, scale, bias)
    c = shape[1]
    dist = Distribution.make_localized_distribution(x.ndim)
    loc = LocaleVirtual(0, 1)
    dyt = Tensor(list(x.shape[::-1]), loc, dist).allocate()
    dxt = Tensor(list(x.shape[::-1]), loc, dist).allocate()
    dyt.real_view().copy_(torch.from_numpy(dy))
    outs = [torch.empty(c, device="cuda") for _ in range(4)]
    sc = torch.from_numpy(scale).cuda()
    assert bn.backward(xin, dyt, mean, var, sc, outs[0], outs[1], outs[2], outs[3], dxt) == 0
    torch.cuda.synchronize()
    mean_h, var_h = mean.cpu().numpy(), var.cpu().numpy()
    dx_o, dscale_o, dbias_o, dmean_o, dvar_o = oracle_mod.bn_backward(x, dy, mean_h, var_h, scale, 1e-5)
    if int(np.prod(shape)) // shape[1] == 1:
        # n == 1: the unbiased variance is 0 * inf = NaN (batchnorm.cu:304-306) and
        # everything derived from it; the finite outputs (dbias) still have to agree
        assert not np.isfinite(var_h).any()
        for got, want, name in zip(outs, (dscale_o, dbias_o, dmean_o, dvar_o),
                                   ("dscale", "dbias", "dmean", "dvar")):
            assert_nan_parity(got.cpu().numpy(), want, name)
        assert_nan_parity(dxt.real_view().cpu().numpy(), dx_o, "dx")
        return
    for got, want, name in zip(outs, (dscale_o, dbias_o, dmean_o, dvar_o),
                               ("dscale", "dbias", "dmean", "dvar")):
        assert max_rel(got.cpu().numpy(), want) <= TOL, name
    assert max_rel(dxt.real_view().cpu().numpy(), dx_o) <= TOL


@pytest.mark.parametrize("dtype", ["float32", "float64"])
@pytest.mark.parametrize("shape", [(8, 64, 56, 56), (2, 3, 4, 5), (3, 5, 7, 9, 11), (64, 32, 7, 7), (1, 1, 1, 1),
                                   (2, 4, 40, 40, 40), (1, 300, 3, 3), (3, 20, 37, 37), (2, 16, 8, 16, 16), (1, 24, 2, 1024),
                                   (40, 300, 7, 7), (512, 600, 1, 1), (6, 9, 3, 5, 17), (33, 70, 14, 14)])
def test_two_launch_forward_and_backward_equal_the_staged_calls(shape, dtype):
    """forward()/backward() of a single rank finish the channel sums inside the
    normalising / input-gradient kernel (h2x_bn_forward_local, _backward_local);
    the staged methods launch the finishing kernels.  Same additions in the same
    order: every output must agree bit for bit (NaNs included)."""
    import torch
    from dihydrogen_amd.layers import BatchNormalization
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    np_dt = np.float32 if dtype == "float32" else np.float64
    tdt = getattr(torch, dtype)
    x, dy, scale, bias = bn_inputs(shape, seed=99, dtype=np_dt)
    nd, c = x.ndim, shape[1]
    dist = Distribution.make_localized_distribution(nd)
    loc = LocaleVirtual(0, 1)
    results = []
    for fuse in (True, False):
        mk = lambda: Tensor(list(x.shape[::-1]), loc, dist, tdt).allocate()
        xt, yt, dyt, dxt = mk(), mk(), mk(), mk()
        xt.real_view().copy_(torch.from_numpy(x))
        dyt.real_view().copy_(torch.from_numpy(dy))
        vec = lambda v: torch.full((c,), v, dtype=tdt, device="cuda")
        mean, var, rm, rv = vec(float("nan")), vec(float("nan")), vec(0.25), vec(0.75)
        grads = [vec(float("nan")) for _ in range(4)]
        sc, bi = torch.from_numpy(scale).cuda(), torch.from_numpy(bias).cuda()
        bn = BatchNormalization(nd, 0.9, 1e-5, fuse_local=fuse)
        if fuse:
            assert bn.forward(xt, mean, var, rm, rv, sc, bi, yt, True) == 0
            assert bn.backward(xt, dyt, mean, var, sc, *grads, dxt) == 0
        else:
            bn.forward_stage1(xt, mean, var, True)
            bn.forward_stage2(xt, mean, var, rm, rv, sc, bi, yt, True)
            bn.backward_stage1(xt, dyt, mean, var, sc, *grads)
            bn.backward_stage2(xt, dyt, mean, var, sc, grads[2], grads[3], dxt)
        torch.cuda.synchronize()
        results.append([t.cpu().numpy() for t in (mean, var, rm, rv, yt.real_view(), *grads, dxt.real_view())])
    names = ("mean", "var", "running_mean", "running_var", "y", "dscale", "dbias", "dmean", "dvar", "dx")
    for name, a, b in zip(names, *results):
        assert np.array_equal(a, b, equal_nan=True), name


@pytest.mark.parametrize("shape", [(2, 6, 8, 12), (9, 45, 7, 7)])
def test_backprop2_in_place(shape, oracle_mod):
    """dx may alias x (legacy/src/dnn_backend/batchnorm.cu:1303-1314)."""
    import torch
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor

    x, dy, scale, bias = bn_inputs(shape, seed=7)
    bn, xin, yout, mean, var, rm, rv = _run_forward(x, scale, bias)
    dist = Distribution.make_localized_distribution(4)
    dyt = Tensor(list(shape[::-1]), LocaleVirtual(0, 1), dist).allocate()
    dyt.real_view().copy_(torch.from_numpy(dy))
    outs = [torch.empty(shape[1], device="cuda") for _ in range(4)]
    sc = torch.from_numpy(scale).cuda()
    bn.backward(xin, dyt, mean, var, sc, *outs, xin)  # d_input aliases input
    torch.cuda.synchronize()
    dx_o = oracle_mod.bn_backward(x, dy, mean.cpu().numpy(), var.cpu().numpy(), scale, 1e-5)[0]
    assert max_rel(xin.real_view().cpu().numpy(), dx_o) <= TOL


@pytest.mark.parametrize("fuse", [True, False])
@pytest.mark.parametrize("shape", [(3, 5, 57, 57), (2, 3, 1027, 1031), (4, 6, 19, 19), (2, 4, 9, 11, 13)])
def test_backprop2_in_place_on_segments_that_end_in_an_overlapping_vector(shape, fuse, oracle_mod):
    """Dense segments that are no multiple of the vector long go through the padded-row
    kernels, whose last vector of a row overlaps the one before it; with dx == x the
    shared elements must be stored by their owner only.  Both the two-launch
    backward() and the staged calls."""
    import torch
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor

    x, dy, scale, bias = bn_inputs(shape, seed=17)
    bn, xin, yout, mean, var, rm, rv = _run_forward(x, scale, bias)
    bn.fuse_local = fuse
    dist = Distribution.make_localized_distribution(len(shape))
    dyt = Tensor(list(shape[::-1]), LocaleVirtual(0, 1), dist).allocate()
    dyt.real_view().copy_(torch.from_numpy(dy))
    outs = [torch.empty(shape[1], device="cuda") for _ in range(4)]
    sc = torch.from_numpy(scale).cuda()
    assert bn.backward(xin, dyt, mean, var, sc, *outs, xin) == 0  # d_input aliases input
    torch.cuda.synchronize()
    dx_o, dscale_o, dbias_o, dmean_o, dvar_o = oracle_mod.bn_backward(
        x, dy, mean.cpu().numpy(), var.cpu().numpy(), scale, 1e-5)
    assert max_rel(xin.real_view().cpu().numpy(), dx_o) <= TOL
    for got, want in zip(outs, (dscale_o, dbias_o, dmean_o, dvar_o)):
        assert max_rel(got.cpu().numpy(), want) <= TOL


@pytest.mark.parametrize("case", [
    ((134, 6, 3, 2), (2, 2, 1, 1), (1, 1, 0, 0)),          # haloed rows of 67 elements
    ((130, 4, 6, 2, 2), (2, 1, 2, 1, 1), (2, 0, 1, 0, 0)),  # 5-D, rows of 65
    ((14, 14, 70, 5), (2, 2, 1, 1), (1, 1, 0, 0)),          # 7 x 7 tiles in 9 x 9: short-segment kernels
    ((18, 10, 14, 3, 2), (2, 2, 2, 1, 1), (1, 1, 1, 0, 0)),  # 9 x 5 x 7 tiles in 11 x 7 x 9
])
def test_backprop2_in_place_on_haloed_tensors(case, oracle_mod):
    """dx == x on every rank of a decomposition whose local parts carry halos: interior
    equal to the oracle's, halo cells untouched (they keep the input's halo values)."""
    import torch
    from dihydrogen_amd.layers import BatchNormalization
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    gshape, locale, overlap = case
    nd = len(gshape)
    nranks = int(np.prod(locale))
    dist = Distribution.make_overlapped_distribution(locale, overlap)
    c = gshape[nd - 2]
    rng = np.random.default_rng(23)
    scale = rng.uniform(0.5, 1.5, c).astype(np.float32)
    bias = (0.1 * rng.standard_normal(c)).astype(np.float32)
    for r in range(nranks):
        loc = LocaleVirtual(r, nranks)
        x, y, dy = (Tensor(gshape, loc, dist).allocate() for _ in range(3))
        for t in (x, y, dy):
            t.real_view().fill_(float("nan"))
        xi = rng.standard_normal(x.local_shape[::-1]).astype(np.float32)
        di = rng.standard_normal(x.local_shape[::-1]).astype(np.float32)
        x.interior_view().copy_(torch.from_numpy(xi))
        dy.interior_view().copy_(torch.from_numpy(di))
        dev = lambda a: torch.from_numpy(a.copy()).cuda()
        mean, var = torch.empty(c, device="cuda"), torch.empty(c, device="cuda")
        rm, rv = torch.zeros(c, device="cuda"), torch.ones(c, device="cuda")
        grads = [torch.empty(c, device="cuda") for _ in range(4)]
        bn = BatchNormalization(nd, 0.9, 1e-5)
        assert bn.forward(x, mean, var, rm, rv, dev(scale), dev(bias), y, True) == 0
        assert bn.backward(x, dy, mean, var, dev(scale), *grads, x) == 0  # d_input aliases input
        torch.cuda.synchronize()
        dx_o = oracle_mod.bn_backward(xi, di, mean.cpu().numpy(), var.cpu().numpy(), scale)[0]
        assert max_rel(x.interior_view().cpu().numpy(), dx_o) <= TOL
        assert int(torch.isnan(x.real_view()).sum()) == x.get_local_real_size() - x.get_local_size()


def test_inference_uses_running_statistics(oracle_mod):
    import torch
    shape = (2, 4, 6, 6)
    x, dy, scale, bias = bn_inputs(shape, seed=11)
    bn, xin, yout, mean, var, rm, rv = _run_forward(x, scale, bias)
    sc, bi = torch.from_numpy(scale).cuda(), torch.from_numpy(bias).cuda()
    bn.forward(xin, mean, var, rm, rv, sc, bi, yout, False)
    torch.cuda.synchronize()
    y_o = oracle_mod.bn_batch_normalization(x, rm.cpu().numpy(), rv.cpu().numpy(), scale, bias, 1e-5)
    assert max_rel(yout.real_view().cpu().numpy(), y_o) <= TOL


def test_deterministic_and_workspace_reuse():
    """Same input several times through one workspace: bit-identical sums (the
    reference's atomics are not, legacy/src/dnn_backend/batchnorm.cu:127-131)."""
    import torch
    shape = (4, 32, 24, 24, 24)
    x, dy, scale, bias = bn_inputs(shape, seed=3)
    bn, xin, yout, mean, var, rm, rv = _run_forward(x, scale, bias)
    results = []
    for _ in range(4):
        bn.forward_stage1(xin, mean, var, True)
        torch.cuda.synchronize()
        results.append((mean.cpu().numpy().copy(), var.cpu().numpy().copy()))
    for m, v in results[1:]:
        assert np.array_equal(m, results[0][0]) and np.array_equal(v, results[0][1])
    s64 = x.astype(np.float64).sum(axis=(0, 2, 3, 4))
    assert max_rel(results[0][0], s64.astype(np.float32)) <= 1e-6


@pytest.mark.parametrize("shape", [(2, 5, 6, 10), (12, 50, 7, 7), (6, 7, 3, 5, 17)])
def test_float64(shape, oracle_mod):
    x, dy, scale, bias = bn_inputs(shape, seed=5, dtype=np.float64)
    bn, xin, yout, mean, var, rm, rv = _run_forward(x, scale, bias, dtype="float64")
    rm_o, rv_o = np.zeros(shape[1]), np.ones(shape[1])
    y_o, mean_o, var_o = oracle_mod.bn_forward(x, scale, bias, rm_o, rv_o, 1e-5, 0.9)
    assert max_rel(mean.cpu().numpy(), mean_o) <= 1e-10
    assert max_rel(var.cpu().numpy(), var_o) <= 1e-10
    assert max_rel(yout.real_view().cpu().numpy(), y_o) <= 1e-10


def test_empty_tensor_zeroes_sums():
    """No samples: outputs are zeroed, nothing else happens
    (legacy/src/dnn_backend/batchnorm.cu:201-208)."""
    import ctypes
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    c = 7
    ws = torch.empty(lib.h2x_bn_workspace_bytes(c), dtype=torch.uint8, device="cuda")
    s = torch.full((c,), 3.0, device="cuda")
    q = torch.full((c,), 3.0, device="cuda")
    capi.check(lib.h2x_bn_channel_sums_and_sqsums(capi.F32, 0, c, 16, 16, None, s.data_ptr(),
                                                  q.data_ptr(), ws.data_ptr(), None))
    torch.cuda.synchronize()
    assert (s == 0).all() and (q == 0).all()


def test_golden_fixtures():
    """The committed float64 fixtures (tests/golden) through the GPU library."""
    import glob
    import os
    import torch
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    for path in sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "bn_*.npz"))):
        g = np.load(path)
        x, dy, scale, bias = g["x"], g["dy"], g["scale"], g["bias"]
        bn, xin, yout, mean, var, rm, rv = _run_forward(x, scale, bias)
        assert max_rel(var.cpu().numpy(), g["var"]) < 2e-6
        assert np.abs(mean.cpu().numpy() - g["mean"]).max() < 1e-6
        assert np.abs(yout.real_view().cpu().numpy() - g["y"]).max() < 5e-6
        dist = Distribution.make_localized_distribution(x.ndim)
        dyt = Tensor(list(x.shape[::-1]), LocaleVirtual(0, 1), dist).allocate()
        dxt = Tensor(list(x.shape[::-1]), LocaleVirtual(0, 1), dist).allocate()
        dyt.real_view().copy_(torch.from_numpy(dy))
        outs = [torch.empty(x.shape[1], device="cuda") for _ in range(4)]
        bn.backward(xin, dyt, mean, var, torch.from_numpy(scale).cuda(), *outs, dxt)
        torch.cuda.synchronize()
        assert np.abs(dxt.real_view().cpu().numpy() - g["dx"]).max() < 2e-5
        assert np.abs(outs[0].cpu().numpy() - g["dscale"]).max() < 2e-5
        assert np.abs(outs[1].cpu().numpy() - g["dbias"]).max() < 2e-5


HALO_CASES = [
    # global shape (innermost first), locale, overlap: tensors with halos on inner spatial dimensions
    ((16, 12, 5, 3), (2, 2, 1, 1), (1, 1, 0, 0)),       # W % 4 == 0 locally (8), unaligned rows
    ((14, 12, 5, 3), (2, 2, 1, 1), (2, 1, 0, 0)),       # W = 7: scalar rows
    ((16, 8, 12, 4, 2), (2, 1, 2, 1, 1), (1, 0, 2, 0, 0)),
    ((8, 8, 8, 3, 2), (2, 2, 2, 1, 1), (1, 1, 1, 0, 0)),
    ((16, 8, 6, 2), (1, 2, 1, 1), (0, 3, 0, 0)),        # halo only on the outermost spatial dimension: dense path
    ((134, 6, 3, 2), (2, 2, 1, 1), (1, 1, 0, 0)),       # haloed rows of 67 elements: vectors split at row ends
    ((130, 4, 6, 2, 2), (2, 1, 2, 1, 1), (2, 0, 1, 0, 0)),  # 5-D, rows of 65
    # small haloed tiles: the short-segment kernels with each lane's place in the tile worked out once
    ((28, 28, 40, 3), (2, 2, 1, 1), (1, 1, 0, 0)),      # 14 x 14 in 16 x 16: one vector in seven crosses a row end
    ((14, 14, 70, 5), (2, 2, 1, 1), (1, 1, 0, 0)),      # 7 x 7 in 9 x 9, odd segment length
    ((12, 12, 12, 9, 2), (2, 2, 2, 1, 1), (1, 1, 1, 0, 0)),  # 6 x 6 x 6 in 8 x 8 x 8
    ((16, 16, 30, 4), (2, 2, 1, 1), (2, 2, 0, 0)),      # 8 x 8 with a halo of 2
    ((6, 6, 300, 33), (2, 3, 1, 1), (1, 1, 0, 0)),      # 3 x 2: shorter than a vector times two, many channels and samples
]


@pytest.mark.parametrize("case", HALO_CASES)
def test_haloed_tensors_match_oracle(case, oracle_mod):
    """Forward + backward on every rank of a spatially decomposed tensor whose
    local parts carry halos (the reference's generic kernels,
    legacy/src/dnn_backend/batchnorm.cu:39-90,369-418,899-980,1303-1369)."""
    import torch
    from dihydrogen_amd.layers import BatchNormalization
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    gshape, locale, overlap = case
    nd = len(gshape)
    nranks = int(np.prod(locale))
    dist = Distribution.make_overlapped_distribution(locale, overlap)
    dist_dy = Distribution.make_distribution(locale)   # gradient tensor without halo, as after a conv
    c = gshape[nd - 2]
    rng = np.random.default_rng(5)
    scale = rng.uniform(0.5, 1.5, c).astype(np.float32)
    bias = (0.1 * rng.standard_normal(c)).astype(np.float32)
    for r in range(nranks):
        loc = LocaleVirtual(r, nranks)
        x, y, dx = (Tensor(gshape, loc, dist).allocate() for _ in range(3))
        dy = Tensor(gshape, loc, dist_dy).allocate()
        x.real_view().fill_(float("nan"))
        y.real_view().fill_(float("nan"))
        dx.real_view().fill_(float("nan"))
        xi = rng.standard_normal(x.local_shape[::-1]).astype(np.float32)
        di = rng.standard_normal(x.local_shape[::-1]).astype(np.float32)
        x.interior_view().copy_(torch.from_numpy(xi))
        dy.interior_view().copy_(torch.from_numpy(di))
        dev = lambda a: torch.from_numpy(a.copy()).cuda()
        mean, var = torch.empty(c, device="cuda"), torch.empty(c, device="cuda")
        rm, rv = torch.zeros(c, device="cuda"), torch.ones(c, device="cuda")
        grads = [torch.empty(c, device="cuda") for _ in range(4)]
        bn = BatchNormalization(nd, 0.9, 1e-5)
        assert bn.forward(x, mean, var, rm, rv, dev(scale), dev(bias), y, True) == 0
        assert bn.backward(x, dy, mean, var, dev(scale), *grads, dx) == 0
        torch.cuda.synchronize()
        rm_o, rv_o = np.zeros(c, np.float32), np.ones(c, np.float32)
        y_o, mean_o, var_o = oracle_mod.bn_forward(xi, scale, bias, rm_o, rv_o)
        dx_o, dscale_o, dbias_o, dmean_o, dvar_o = oracle_mod.bn_backward(xi, di, mean_o, var_o, scale)
        assert max_rel(mean.cpu().numpy(), mean_o) <= TOL and max_rel(var.cpu().numpy(), var_o) <= TOL
        assert max_rel(y.interior_view().cpu().numpy(), y_o) <= TOL
        for got, want in zip(grads, (dscale_o, dbias_o, dmean_o, dvar_o)):
            assert max_rel(got.cpu().numpy(), want) <= TOL
        assert max_rel(dx.interior_view().cpu().numpy(), dx_o) <= TOL
        # halo cells are never written
        for t in (y, dx):
            assert int(torch.isnan(t.real_view()).sum()) == t.get_local_real_size() - t.get_local_size()


CLEARING_CASES = HALO_CASES + [
    ((16, 8, 6, 2), (1, 2, 1, 1), (0, 3, 0, 0)),          # halo on the outermost spatial dimension only
    ((10, 6, 6, 3, 2), (2, 1, 2, 1, 1), (1, 0, 2, 0, 0)),  # real segment of 7 x 6 x 7 elements: no whole vectors
    ((128, 128, 8, 2), (2, 2, 1, 1), (1, 1, 0, 0)),        # 66 x 66 real: rows 8 bytes off every other time    # real planes of 18 and 15 cells with no halo on dimension 1: vectors that begin in the last row of a
    # plane and end in the first, interior, row of the next
    ((8, 3, 4, 3, 2), (2, 1, 2, 1, 1), (1, 0, 1, 0, 0)),
    ((6, 3, 4, 3, 2), (2, 1, 2, 1, 1), (1, 0, 1, 0, 0)),
]


@pytest.mark.parametrize("dtype", ["float32", "float64"])
@pytest.mark.parametrize("case", CLEARING_CASES)
def test_clearing_variants_equal_the_strided_calls_followed_by_clear_halo(case, dtype):
    """clear_output_halo: normalise and the input gradient leave the halo of their output
    cleared.  Bit for bit what the reference's sequence leaves: the kernel on the interior,
    then Tensor::clear_halo on every spatial dimension of the output
    (legacy/src/tensor/tensor_mpi_cuda.cu:14-84); the halos of the inputs hold NaNs and stay."""
    import ctypes
    import torch
    from dihydrogen_amd import capi
    from dihydrogen_amd.layers import BatchNormalization
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    lib = capi.load()
    gshape, locale, overlap = case
    nd = len(gshape)
    nranks = int(np.prod(locale))
    tdt = getattr(torch, dtype)
    dist = Distribution.make_overlapped_distribution(locale, overlap)
    c = gshape[nd - 2]
    g = torch.Generator(device="cuda").manual_seed(31)
    scale = torch.empty(c, dtype=tdt, device="cuda").uniform_(0.5, 1.5, generator=g)
    bias = torch.empty(c, dtype=tdt, device="cuda").normal_(0, 0.1, generator=g)
    for r in range(nranks):
        loc = LocaleVirtual(r, nranks)
        results = []
        xi = di = None
        for clearing in (False, True):
            x, y, dy, dx = (Tensor(gshape, loc, dist, tdt).allocate() for _ in range(4))
            for t in (x, y, dy, dx):
                t.real_view().fill_(float("nan"))
            if xi is None:
                xi = torch.empty_like(x.interior_view()).normal_(0, 1, generator=g)
                di = torch.empty_like(x.interior_view()).normal_(0, 1, generator=g)
            x.interior_view().copy_(xi)
            dy.interior_view().copy_(di)
            vec = lambda: torch.empty(c, dtype=tdt, device="cuda")
            mean, var, rm, rv = vec(), vec(), torch.zeros(c, dtype=tdt, device="cuda"), torch.ones(c, dtype=tdt, device="cuda")
            grads = [vec() for _ in range(4)]
            bn = BatchNormalization(nd, 0.9, 1e-5, clear_output_halo=clearing)
            assert bn.forward(x, mean, var, rm, rv, scale, bias, y, True) == 0
            assert bn.backward(x, dy, mean, var, scale, *grads, dx) == 0
            if not clearing:
                for t in (y, dx):
                    for d in range(nd - 2):
                        if t.overlap[d]:
                            capi.check(lib.h2x_halo_clear(t.h2x_dtype, ctypes.c_void_p(t.get_buffer()), nd,
                                                          capi.i64_array(t.local_real_shape), d, t.overlap[d], None))
            torch.cuda.synchronize()
            results.append([t.real_view().cpu().numpy() for t in (y, dx)] + [v.cpu().numpy() for v in (mean, var, *grads)])
            # the inputs are untouched: their halos still hold NaNs
            for t in (x, dy):
                assert int(torch.isnan(t.real_view()).sum()) == t.get_local_real_size() - t.get_local_size()
        for a, b in zip(*results):
            assert np.array_equal(a, b)
        assert not np.isnan(results[1][0]).any() and not np.isnan(results[1][1]).any()


def test_clearing_input_gradient_in_place():
    """dx == x with clear_output_halo: the interior holds the gradient, the halo zeros."""
    import torch
    from dihydrogen_amd.layers import BatchNormalization
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    gshape, locale, overlap = (60, 12, 10, 3, 2), (2, 1, 2, 1, 1), (1, 0, 1, 0, 0)
    dist = Distribution.make_overlapped_distribution(locale, overlap)
    loc = LocaleVirtual(1, 4)
    g = torch.Generator(device="cuda").manual_seed(37)
    c = gshape[3]
    outs = []
    for alias in (False, True):
        x, y, dy, dx = (Tensor(gshape, loc, dist).allocate() for _ in range(4))
        torch.manual_seed(5)
        for t in (x, dy):
            t.real_view().copy_(torch.randn(t.real_view().shape, device="cuda"))
        scale, bias = torch.ones(c, device="cuda") * 1.25, torch.zeros(c, device="cuda")
        mean, var, rm, rv = (torch.zeros(c, device="cuda") for _ in range(4))
        grads = [torch.empty(c, device="cuda") for _ in range(4)]
        bn = BatchNormalization(5, 0.9, 1e-5, clear_output_halo=True)
        bn.forward(x, mean, var, rm, rv, scale, bias, y, True)
        target = x if alias else dx
        bn.backward(x, dy, mean, var, scale, *grads, target)
        torch.cuda.synchronize()
        outs.append(target.real_view().cpu().numpy())
    assert np.array_equal(outs[0], outs[1])


@pytest.mark.parametrize("case", HALO_CASES)
def test_two_launch_calls_on_haloed_tensors_equal_the_staged_calls(case):
    """forward()/backward() on tensors with halos on inner dimensions take
    h2x_bn_forward_local_strided / _backward_local_strided (two launches each): every
    output equals the staged calls' bit for bit, halo cells stay untouched."""
    import torch
    from dihydrogen_amd.layers import BatchNormalization
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    gshape, locale, overlap = case
    nd = len(gshape)
    nranks = int(np.prod(locale))
    dist = Distribution.make_overlapped_distribution(locale, overlap)
    dist_dy = Distribution.make_distribution(locale)
    c = gshape[nd - 2]
    g = torch.Generator(device="cuda").manual_seed(41)
    scale = torch.empty(c, device="cuda").uniform_(0.5, 1.5, generator=g)
    bias = torch.empty(c, device="cuda").normal_(0, 0.1, generator=g)
    for r in range(nranks):
        loc = LocaleVirtual(r, nranks)
        xi = di = None
        results = []
        for fuse in (True, False):
            x, y, dx = (Tensor(gshape, loc, dist).allocate() for _ in range(3))
            dy = Tensor(gshape, loc, dist_dy).allocate()
            for t in (x, y, dx):
                t.real_view().fill_(float("nan"))
            if xi is None:
                xi = torch.empty_like(x.interior_view()).normal_(0, 1, generator=g)
                di = torch.empty_like(dy.interior_view()).normal_(0, 1, generator=g)
            x.interior_view().copy_(xi)
            dy.interior_view().copy_(di)
            vec = lambda v: torch.full((c,), v, device="cuda")
            mean, var, rm, rv = vec(float("nan")), vec(float("nan")), vec(0.25), vec(0.75)
            grads = [vec(float("nan")) for _ in range(4)]
            bn = BatchNormalization(nd, 0.9, 1e-5, fuse_local=fuse)
            assert bn.forward(x, mean, var, rm, rv, scale, bias, y, True) == 0
            assert bn.backward(x, dy, mean, var, scale, *grads, dx) == 0
            torch.cuda.synchronize()
            results.append([t.cpu().numpy() for t in (mean, var, rm, rv, y.real_view(), *grads, dx.real_view())])
        for a, b in zip(*results):
            assert np.array_equal(a, b, equal_nan=True)


def test_non_finite_inputs_propagate_as_in_the_oracle(oracle_mod):
    """A NaN, an infinity, values near the float32 maximum (whose squares overflow
    float32 but not the float64 accumulators) and denormals, each in a channel of
    its own: NaNs and infinities come out in the same places as the oracle's, the
    finite outputs within the tolerance; the untouched channels are unaffected."""
    shape = (3, 6, 10, 12)
    x, dy, scale, bias = bn_inputs(shape, seed=77)
    x[1, 0, 3, 4] = np.nan
    x[2, 1, 0, 0] = np.inf
    x[:, 2] *= np.float32(1e38)          # sums of squares beyond the float32 range
    x[:, 3] *= np.float32(1e-42)         # denormal inputs
    x[0, 4, 5, 5] = -np.inf
    bn, xin, yout, mean, var, rm, rv = _run_forward(x, scale, bias)
    with np.errstate(all="ignore"):
        y_o, mean_o, var_o = oracle_mod.bn_forward(x, scale, bias, np.zeros(6, np.float32), np.ones(6, np.float32),
                                                   1e-5, 0.9)
    assert_nan_parity(mean.cpu().numpy(), mean_o, "mean")
    assert_nan_parity(var.cpu().numpy(), var_o, "var")
    assert_nan_parity(yout.real_view().cpu().numpy(), y_o, "y")
    assert np.isfinite(y_o[:, 5]).all() and np.isfinite(y_o[:, 3]).all()   # the test has teeth: finite channels exist

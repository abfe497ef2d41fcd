"""GPU parity of batch-norm on the inputs the reference validates with.

The reference's benchmark fills x and d_output with its Initializer (seeds 0 and 2): averages
of two table entries of rand() / RAND_MAX, i.e. values in [0, 1) with mean 1/2, and sets
scale = 1, bias = 0, running_mean = 0, running_var = 1
(legacy/benchmarks/distconv_benchmark_bn.cpp:200-213, benchmark_common.hpp:43-79); its test
script compares every dumped tensor at 1.5e-5, d_bias at 5e-5
(legacy/tests/dnn_backend/test_cudnn_util.sh.in:50-84).  On such data the variance
q/n - mean^2 cancels (4x here, 100x in the offset case below), so a one-ulp difference in a
rounded channel sum that zero-mean data would hide shows up in var, y, dscale, dvar and dx.
Every output is compared with the oracle at 1e-5 in the reference's metric
max(|d/v1|, |d/v2|) (legacy/tests/compare_binary_files.cpp:47-49).
"""
import numpy as np
import pytest

from helpers import max_rel, reference_initializer

pytestmark = pytest.mark.gpu
TOL = 1e-5
NAMES = ("mean", "var", "running_mean", "running_var", "y", "dscale", "dbias", "dmean", "dvar", "dx")


def _forward_backward(x, dy, scale, bias, dist_x=None, dist_dy=None, gshape=None, rank=0, nranks=1):
    """forward() + backward() of the layer on one rank; x and dy are the rank's interiors."""
    import torch
    from dihydrogen_amd.layers import BatchNormalization
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    nd, c = x.ndim, x.shape[1]
    gshape = list(x.shape[::-1]) if gshape is None else list(gshape)
    dist_x = dist_x or Distribution.make_localized_distribution(nd)
    dist_dy = dist_dy or dist_x
    loc = LocaleVirtual(rank, nranks)
    xt, yt, dxt = (Tensor(gshape, loc, dist_x).allocate() for _ in range(3))
    dyt = Tensor(gshape, loc, dist_dy).allocate()
    for t in (xt, yt, dxt, dyt):
        t.real_view().fill_(float("nan"))       # halo cells must be neither read nor written
    xt.interior_view().copy_(torch.from_numpy(x))
    dyt.interior_view().copy_(torch.from_numpy(dy))
    dev = lambda a: torch.from_numpy(a.copy()).cuda()
    mean, var = torch.empty(c, device="cuda"), torch.empty(c, device="cuda")
    rm, rv = torch.zeros(c, device="cuda"), torch.ones(c, device="cuda")
    grads = [torch.empty(c, device="cuda") for _ in range(4)]
    bn = BatchNormalization(nd, 0.9, 1e-5)
    assert bn.forward(xt, mean, var, rm, rv, dev(scale), dev(bias), yt, True) == 0
    assert bn.backward(xt, dyt, mean, var, dev(scale), *grads, dxt) == 0
    torch.cuda.synchronize()
    for t in (yt, dxt):
        assert int(torch.isnan(t.real_view()).sum()) == t.get_local_real_size() - t.get_local_size()
    host = lambda t: t.cpu().numpy()
    return (host(mean), host(var), host(rm), host(rv), host(yt.interior_view()), *map(host, grads),
            host(dxt.interior_view()))


def _oracle(oracle_mod, x, dy, scale, bias):
    c = x.shape[1]
    rm, rv = np.zeros(c, np.float32), np.ones(c, np.float32)
    y, mean, var = oracle_mod.bn_forward(x, scale, bias, rm, rv, 1e-5, 0.9)
    dx, dscale, dbias, dmean, dvar = oracle_mod.bn_backward(x, dy, mean, var, scale, 1e-5)
    return mean, var, rm, rv, y, dscale, dbias, dmean, dvar, dx


def _compare(got, want):
    for name, g, w in zip(NAMES, got, want):
        assert np.isfinite(w).all(), name
        assert max_rel(g, w) <= TOL, f"{name}: {max_rel(g, w):.3g}"


@pytest.mark.parametrize("shape,seeds", [
    ((8, 64, 56, 56), (0, 2)),          # config 1 with the reference's own seeds
    ((8, 64, 56, 56), (1, 0)),
    ((8, 64, 56, 56), (2, 1)),
    ((4, 64, 64, 64, 64), (0, 2)),      # config 3
    ((16, 32, 7, 7), (0, 2)),           # short segments
    ((3, 20, 37, 37), (0, 2)),          # odd segments: padded rows
])
def test_reference_validation_inputs(shape, seeds, oracle_mod):
    x = reference_initializer(shape, seeds[0])
    dy = reference_initializer(shape, seeds[1])
    assert 0.0 <= x.min() and x.max() < 1.0 and abs(float(x.mean()) - 0.5) < 0.1
    c = shape[1]
    scale, bias = np.ones(c, np.float32), np.zeros(c, np.float32)
    _compare(_forward_backward(x, dy, scale, bias), _oracle(oracle_mod, x, dy, scale, bias))


@pytest.mark.parametrize("rank", [0, 5])
def test_reference_validation_inputs_on_a_haloed_shard(rank, oracle_mod):
    """One rank of a 2 x 2 x 2 decomposition with a halo of 1: values by global index, as
    the reference initialises a distributed tensor (distconv_benchmark_common.hpp:65-92)."""
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    gshape, locale, overlap = (64, 64, 64, 16, 2), (2, 2, 2, 1, 1), (1, 1, 1, 0, 0)
    dist = Distribution.make_overlapped_distribution(locale, overlap)
    dist_dy = Distribution.make_distribution(locale)
    probe = Tensor(gshape, LocaleVirtual(rank, 8), dist)
    local, gidx = probe.local_shape[::-1], probe.global_index[::-1]
    x = reference_initializer(local, 0, global_shape=gshape[::-1], global_index=gidx)
    dy = reference_initializer(local, 2, global_shape=gshape[::-1], global_index=gidx)
    scale, bias = np.ones(16, np.float32), np.zeros(16, np.float32)
    got = _forward_backward(x, dy, scale, bias, dist, dist_dy, gshape, rank, 8)
    _compare(got, _oracle(oracle_mod, x, dy, scale, bias))


@pytest.mark.parametrize("shape", [(8, 64, 56, 56), (4, 16, 32, 32, 32), (64, 48, 7, 7)])
def test_offset_inputs_where_the_variance_cancels_a_hundredfold(shape, oracle_mod):
    """x ~ N(10, 1): q/n = 101 against mean^2 = 100."""
    rng = np.random.default_rng(2024)
    x = (10.0 + rng.standard_normal(shape)).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    c = shape[1]
    scale, bias = np.ones(c, np.float32), np.zeros(c, np.float32)
    want = _oracle(oracle_mod, x, dy, scale, bias)
    assert abs(float(want[1].mean()) - 1.0) < 0.05       # the variance is about 1
    _compare(_forward_backward(x, dy, scale, bias), want)

"""GPU parity at the full sizes of BASELINE.json's configurations.

Batch-norm (configs 1 and 3) and softmax (config 4) are compared with the
oracle in full (it finishes in seconds); halo (config 2) and shuffle (config 5)
are checked through size-independent properties: the closed form of the
reference tests (every halo cell holds the value of its periodic source;
every shuffled element sits at its global position) and a bit-exact round trip.
"""
import numpy as np
import pytest

from helpers import max_rel

pytestmark = pytest.mark.gpu
TOL = 1e-5


def _bn_full(shape, seed, oracle_mod):
    import torch
    from dihydrogen_amd.layers import BatchNormalization
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    rng = np.random.default_rng(seed)
    c = shape[1]
    x = rng.standard_normal(shape, dtype=np.float32)
    dy = rng.standard_normal(shape, dtype=np.float32)
    scale = rng.uniform(0.5, 1.5, c).astype(np.float32)
    bias = (0.1 * rng.standard_normal(c)).astype(np.float32)
    dist = Distribution.make_localized_distribution(len(shape))
    mk = lambda: Tensor(list(shape[::-1]), LocaleVirtual(0, 1), dist).allocate()
    xt, yt, dyt, dxt = mk(), mk(), mk(), mk()
    xt.real_view().copy_(torch.from_numpy(x))
    dyt.real_view().copy_(torch.from_numpy(dy))
    dev = lambda a: torch.from_numpy(a.copy()).cuda()
    mean, var = torch.empty(c, device="cuda"), torch.empty(c, device="cuda")
    rm, rv = torch.zeros(c, device="cuda"), torch.ones(c, device="cuda")
    grads = [torch.empty(c, device="cuda") for _ in range(4)]
    bn = BatchNormalization(len(shape), 0.9, 1e-5)
    bn.forward(xt, mean, var, rm, rv, dev(scale), dev(bias), yt, True)
    bn.backward(xt, dyt, mean, var, dev(scale), *grads, dxt)
    torch.cuda.synchronize()
    rm_o, rv_o = np.zeros(c, np.float32), np.ones(c, np.float32)
    y_o, mean_o, var_o = oracle_mod.bn_forward(x, scale, bias, rm_o, rv_o)
    assert max_rel(mean.cpu().numpy(), mean_o) <= TOL
    assert max_rel(var.cpu().numpy(), var_o) <= TOL
    assert max_rel(rm.cpu().numpy(), rm_o) <= TOL and max_rel(rv.cpu().numpy(), rv_o) <= TOL
    assert max_rel(yt.real_view().cpu().numpy(), y_o) <= TOL
    del y_o
    dx_o, dscale_o, dbias_o, dmean_o, dvar_o = oracle_mod.bn_backward(x, dy, mean_o, var_o, scale)
    for got, want in zip(grads, (dscale_o, dbias_o, dmean_o, dvar_o)):
        assert max_rel(got.cpu().numpy(), want) <= TOL
    assert max_rel(dxt.real_view().cpu().numpy(), dx_o) <= TOL


def test_config1_bn2d(oracle_mod):
    _bn_full((8, 64, 56, 56), 1235, oracle_mod)


def test_config3_bn3d(oracle_mod):
    _bn_full((4, 64, 64, 64, 64), 1237, oracle_mod)


@pytest.mark.parametrize("clearing", [False, True])
def test_config3_bn3d_on_a_haloed_shard(oracle_mod, clearing):
    """Config 3's local size with a halo of one cell on every spatial dimension (the shard of
    a 2 x 2 x 2 decomposition): the interior equals the oracle on the interior alone; the halo
    cells of y and dx keep what they held, or are zero with clear_output_halo."""
    import torch
    from dihydrogen_amd.layers import BatchNormalization
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    shape = (4, 64, 64, 64, 64)
    rng = np.random.default_rng(1239)
    c = shape[1]
    x = rng.standard_normal(shape, dtype=np.float32)
    dy = rng.standard_normal(shape, dtype=np.float32)
    scale = rng.uniform(0.5, 1.5, c).astype(np.float32)
    bias = (0.1 * rng.standard_normal(c)).astype(np.float32)
    dist = Distribution.make_overlapped_distribution([2, 2, 2, 1, 1], [1, 1, 1, 0, 0])
    mk = lambda: Tensor([128, 128, 128, c, shape[0]], LocaleVirtual(0, 8), dist).allocate()
    xt, yt, dyt, dxt = mk(), mk(), mk(), mk()
    sentinel = 7.25
    for t in (xt, dyt):
        t.real_view().fill_(1e30)  # the halo of an input is never read
    for t in (yt, dxt):
        t.real_view().fill_(sentinel)
    xt.interior_view().copy_(torch.from_numpy(x))
    dyt.interior_view().copy_(torch.from_numpy(dy))
    dev = lambda a: torch.from_numpy(a.copy()).cuda()
    mean, var = torch.empty(c, device="cuda"), torch.empty(c, device="cuda")
    rm, rv = torch.zeros(c, device="cuda"), torch.ones(c, device="cuda")
    grads = [torch.empty(c, device="cuda") for _ in range(4)]
    bn = BatchNormalization(len(shape), 0.9, 1e-5, clear_output_halo=clearing)
    bn.forward(xt, mean, var, rm, rv, dev(scale), dev(bias), yt, True)
    bn.backward(xt, dyt, mean, var, dev(scale), *grads, dxt)
    torch.cuda.synchronize()
    rm_o, rv_o = np.zeros(c, np.float32), np.ones(c, np.float32)
    y_o, mean_o, var_o = oracle_mod.bn_forward(x, scale, bias, rm_o, rv_o)
    assert max_rel(mean.cpu().numpy(), mean_o) <= TOL
    assert max_rel(var.cpu().numpy(), var_o) <= TOL
    assert max_rel(rm.cpu().numpy(), rm_o) <= TOL and max_rel(rv.cpu().numpy(), rv_o) <= TOL
    assert max_rel(yt.interior_view().cpu().numpy(), y_o) <= TOL
    del y_o
    dx_o, dscale_o, dbias_o, dmean_o, dvar_o = oracle_mod.bn_backward(x, dy, mean_o, var_o, scale)
    for got, want in zip(grads, (dscale_o, dbias_o, dmean_o, dvar_o)):
        assert max_rel(got.cpu().numpy(), want) <= TOL
    assert max_rel(dxt.interior_view().cpu().numpy(), dx_o) <= TOL
    del dx_o
    # the halo: what is left of the whole allocation once the interior is taken out
    expect = 0.0 if clearing else sentinel
    for t in (yt, dxt):
        whole = t.real_view()
        halo_cells = whole.numel() - t.interior_view().numel()
        t.interior_view().fill_(expect)
        assert int((whole == expect).sum().item()) == whole.numel() and halo_cells > 0


def test_config4_softmax(oracle_mod):
    import torch
    from dihydrogen_amd.layers import Softmax, SoftmaxMode
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    shape = (16, 21, 256, 256)
    rng = np.random.default_rng(1238)
    x = 2.0 * rng.standard_normal(shape, dtype=np.float32)
    dy = rng.standard_normal(shape, dtype=np.float32)
    dist = Distribution.make_localized_distribution(4)
    mk = lambda: Tensor(list(shape[::-1]), LocaleVirtual(0, 1), dist).allocate()
    xt, yt, dyt, dxt = mk(), mk(), mk(), mk()
    xt.real_view().copy_(torch.from_numpy(x))
    dyt.real_view().copy_(torch.from_numpy(dy))
    sm = Softmax()
    sm.setup(xt, SoftmaxMode.CHANNEL)
    sm.forward(xt, yt)
    sm.backward(yt, dyt, dxt)
    torch.cuda.synchronize()
    y = yt.real_view().cpu().numpy()
    assert max_rel(y, oracle_mod.softmax_channel_forward(x)) <= TOL
    assert max_rel(dxt.real_view().cpu().numpy(), oracle_mod.softmax_channel_backward(y, dy)) <= TOL


@pytest.mark.parametrize("fused", [False, True])
def test_config2_halo_closed_form(fused):
    """8 virtual ranks, N1 C32 128^3 each, periodic 2x2x2, width 1: after the
    exchange every cell of every real tensor, halo faces, edges and corners
    included, equals the value of its periodic source coordinate.  Once through
    pack + unpack, once as tensor-to-tensor transfers."""
    import torch
    from dihydrogen_amd.layers import HaloExchangeVirtual
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    L, C = 128, 32
    gshape = (2 * L, 2 * L, 2 * L, C, 1)
    dist = Distribution.make_overlapped_distribution((2, 2, 2, 1, 1), (1, 1, 1, 0, 0))
    ranks = [Tensor(gshape, LocaleVirtual(r, 8), dist).allocate() for r in range(8)]

    def field(t, with_halo):
        # value = hash of the global coordinate, exact in float32
        axes = []
        for d in range(5):
            n = t.local_real_shape[d] if with_halo else t.local_shape[d]
            g = torch.arange(n, device="cuda", dtype=torch.int64) + t.global_index[d]
            if with_halo:
                g = (g - t.overlap[d]) % gshape[d]
            axes.append(g)
        w, h, dd, c, n = axes
        off = (w.view(1, 1, 1, 1, -1) + gshape[0] * (h.view(1, 1, 1, -1, 1) + gshape[1] * (
            dd.view(1, 1, -1, 1, 1) + gshape[2] * c.view(1, -1, 1, 1, 1))))
        return ((off * 2654435761) % 16777213).float()

    for t in ranks:
        t.real_view().fill_(float("nan"))
        t.interior_view().copy_(field(t, False))
    HaloExchangeVirtual(ranks, periodic=True).exchange(fused=fused)
    torch.cuda.synchronize()
    for t in ranks:
        assert torch.equal(t.real_view(), field(t, True))


def test_config5_shuffle_round_trip():
    import torch
    from dihydrogen_amd.layers import TensorShufflerVirtual
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    gshape = (128, 128, 64, 32)
    sd, dd = Distribution([1, 1, 1, 4]), Distribution([2, 2, 1, 1])
    src = [Tensor(gshape, LocaleVirtual(r, 4), sd).allocate() for r in range(4)]
    dst = [Tensor(gshape, LocaleVirtual(r, 4), dd).allocate() for r in range(4)]
    g = torch.Generator(device="cuda").manual_seed(1239)
    full = torch.empty(*reversed(gshape), device="cuda").uniform_(-1, 1, generator=g)
    box = lambda t: tuple(slice(a, a + l) for a, l in zip(reversed(t.global_index), reversed(t.local_shape)))
    for t in src:
        t.real_view().copy_(full[box(t)])
    sh = TensorShufflerVirtual(src, dst)
    sh.shuffle_forward()
    torch.cuda.synchronize()
    for t in dst:
        assert torch.equal(t.real_view(), full[box(t)])
    for t in src:
        t.data.zero_()
    sh.shuffle_backward()
    torch.cuda.synchronize()
    for t in src:
        assert torch.equal(t.real_view(), full[box(t)])

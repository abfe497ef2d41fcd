"""The entry points can be captured into a HIP graph: they allocate nothing,
never synchronise and clear memory with kernels only.  A graph holding batch
norm forward+backward (dense, on a haloed shard, and with the halo cleared),
channel softmax, a halo exchange and a shuffle is
replayed several times on fresh inputs, with eager work and synchronisation
between the replays, and every replay must reproduce the eager results bit for
bit (all kernels are deterministic)."""
import pytest

pytestmark = pytest.mark.gpu


def test_graph_replays_match_eager():
    import torch
    from dihydrogen_amd.layers import (BatchNormalization, HaloExchangeVirtual, Softmax, SoftmaxMode,
                                       TensorShufflerVirtual)
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor

    gen = torch.Generator(device="cuda").manual_seed(7)
    # batch norm, 5-D
    shape = [16, 12, 10, 8, 2]
    dist = Distribution.make_localized_distribution(5)
    mk = lambda: Tensor(shape, LocaleVirtual(0, 1), dist).allocate()
    x, y, dy, dx = mk(), mk(), mk(), mk()
    c = 8
    vec = lambda v: torch.full((c,), v, device="cuda")
    mean, var, rm, rv = vec(0.0), vec(0.0), vec(0.0), vec(1.0)
    scale, bias = vec(0.75), vec(0.25)
    grads = [vec(0.0) for _ in range(4)]
    bn = BatchNormalization(5, 0.9, 1e-5)
    # softmax
    sshape = [16, 16, 21, 2]
    sdist = Distribution.make_localized_distribution(4)
    smk = lambda: Tensor(sshape, LocaleVirtual(0, 1), sdist).allocate()
    lx, ly, ldy, ldx = smk(), smk(), smk(), smk()
    sm = Softmax()
    sm.setup(lx, SoftmaxMode.CHANNEL)
    # halo exchange
    hdist = Distribution.make_overlapped_distribution((2, 2, 1, 1), (1, 1, 0, 0))
    ranks = [Tensor((12, 10, 3, 2), LocaleVirtual(r, 4), hdist).allocate() for r in range(4)]
    xch = HaloExchangeVirtual(ranks, periodic=True)
    # shuffle
    sd, dd = Distribution([1, 1, 1, 4]), Distribution([2, 2, 1, 1])
    src = [Tensor((8, 8, 2, 4), LocaleVirtual(r, 4), sd).allocate() for r in range(4)]
    dst = [Tensor((8, 8, 2, 4), LocaleVirtual(r, 4), dd).allocate() for r in range(4)]
    sh = TensorShufflerVirtual(src, dst)

    # batch norm on a haloed shard: the two-launch calls on strided tensors, and the halo-clearing kernels
    bdist = Distribution.make_overlapped_distribution((2, 2, 1, 1), (1, 1, 0, 0))
    bmk = lambda: Tensor((36, 28, c, 3), LocaleVirtual(0, 4), bdist).allocate()
    hx, hy, hdy, hdx, hy2, hdx2 = (bmk() for _ in range(6))
    hstats = [vec(0.0) for _ in range(4)]
    hgrads = [vec(0.0) for _ in range(4)]
    bn_haloed = BatchNormalization(4, 0.9, 1e-5)
    bn_clearing = BatchNormalization(4, 0.9, 1e-5, clear_output_halo=True)

    inputs = [x.data, dy.data, lx.data, ldy.data, hx.data, hdy.data] + [t.data for t in ranks] + [t.data for t in src]
    outputs = [y.data, dx.data, mean, var, rm, rv, ly.data, ldx.data] + grads \
        + [t.data for t in ranks] + [t.data for t in dst] \
        + [hy.data, hdx.data, hy2.data, hdx2.data] + hstats + hgrads

    def new_inputs():
        for t in inputs:
            t.normal_(0, 1, generator=gen)
        rm.zero_()
        rv.fill_(1.0)
        for t in (hy, hdx, hy2, hdx2):
            t.data.fill_(3.0)  # halo cells: kept by the plain calls, zeroed by the clearing ones

    def step():
        bn.forward(x, mean, var, rm, rv, scale, bias, y, True)
        bn.backward(x, dy, mean, var, scale, *grads, dx)
        sm.forward(lx, ly)
        sm.backward(ly, ldy, ldx)
        xch.exchange()
        sh.shuffle_forward()
        for layer, out, din in ((bn_haloed, hy, hdx), (bn_clearing, hy2, hdx2)):
            hstats[2].zero_()
            hstats[3].fill_(1.0)
            layer.forward(hx, hstats[0], hstats[1], hstats[2], hstats[3], scale, bias, out, True)
            layer.backward(hx, hdy, hstats[0], hstats[1], scale, *hgrads, din)

    new_inputs()
    step()  # eager warm-up: workspaces and receive buffers are allocated here, not under capture
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    capture_stream = torch.cuda.Stream()
    capture_stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph, stream=capture_stream):
        step()
    torch.cuda.synchronize()

    for _ in range(4):
        new_inputs()
        saved = [t.clone() for t in inputs]
        graph.replay()
        torch.cuda.synchronize()
        replayed = [t.clone() for t in outputs]
        # the same inputs, eagerly
        for t, s in zip(inputs, saved):
            t.copy_(s)
        rm.zero_()
        rv.fill_(1.0)
        for t in (hy, hdx, hy2, hdx2):
            t.data.fill_(3.0)
        step()
        torch.cuda.synchronize()
        for a, b in zip(replayed, outputs):
            assert torch.equal(a, b)
        # the two haloed passes agree on the interior and differ in the halo only
        assert torch.equal(hy.interior_view(), hy2.interior_view())
        assert torch.equal(hdx.interior_view(), hdx2.interior_view())
        assert int((hy.real_view() == 3.0).sum()) >= hy.get_local_real_size() - hy.get_local_size()
        assert int((hy2.real_view() == 0.0).sum()) >= hy2.get_local_real_size() - hy2.get_local_size()

"""Every entry point launches on the stream it is given and nowhere else: the
layers run on a user-created stream (default priority) while the default
stream is kept busy with unrelated work, and the results must equal those of a
run on the default stream.  The reference's layers are asynchronous on the
caller's stream in the same way (legacy/include/distconv/dnn_backend/batchnorm.hpp:171-260)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _run_all(stream):
    """Batch norm forward+backward, channel softmax, halo exchange (both forms)
    and a shuffle round trip, all on `stream` (None = torch's current stream)."""
    import torch
    from dihydrogen_amd.layers import (BatchNormalization, HaloExchangeVirtual, Softmax, SoftmaxMode,
                                       TensorShufflerVirtual)
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor

    out = {}
    g = torch.Generator(device="cuda").manual_seed(99)
    ctx = torch.cuda.stream(stream) if stream is not None else torch.cuda.stream(torch.cuda.current_stream())
    with ctx:
        # batch norm
        shape = [24, 20, 12, 16, 3]
        dist = Distribution.make_localized_distribution(5)
        mk = lambda: Tensor(shape, LocaleVirtual(0, 1), dist).allocate()
        x, y, dy, dx = mk(), mk(), mk(), mk()
        x.data.normal_(0, 1, generator=g)
        dy.data.normal_(0, 1, generator=g)
        c = 16
        vec = lambda v: torch.full((c,), v, device="cuda")
        mean, var, rm, rv = vec(0.0), vec(0.0), vec(0.0), vec(1.0)
        scale, bias = vec(1.25), vec(-0.5)
        grads = [vec(0.0) for _ in range(4)]
        bn = BatchNormalization(5, 0.9, 1e-5, stream=stream)
        bn.forward(x, mean, var, rm, rv, scale, bias, y, True)
        bn.backward(x, dy, mean, var, scale, *grads, dx)
        out["bn"] = [y.data, dx.data, mean, var, rm, rv] + grads
        # softmax
        sshape = [32, 16, 21, 2]
        sdist = Distribution.make_localized_distribution(4)
        smk = lambda: Tensor(sshape, LocaleVirtual(0, 1), sdist).allocate()
        lx, ly, ldy, ldx = smk(), smk(), smk(), smk()
        lx.data.normal_(0, 2, generator=g)
        ldy.data.normal_(0, 1, generator=g)
        sm = Softmax(stream=stream)
        sm.setup(lx, SoftmaxMode.CHANNEL)
        sm.forward(lx, ly)
        sm.backward(ly, ldy, ldx)
        out["softmax"] = [ly.data, ldx.data]
        # halo exchange, through buffers and fused
        hshape, locale, overlap = (12, 10, 8, 3, 1), (2, 2, 2, 1, 1), (1, 2, 1, 0, 0)
        hdist = Distribution.make_overlapped_distribution(locale, overlap)
        for fused in (False, True):
            ranks = [Tensor(hshape, LocaleVirtual(r, 8), hdist).allocate() for r in range(8)]
            for t in ranks:
                t.data.uniform_(-1, 1, generator=g)
            HaloExchangeVirtual(ranks, periodic=True, stream=stream).exchange(fused=fused)
            out[f"halo{int(fused)}"] = [t.data for t in ranks]
        # shuffle round trip
        tshape = (16, 12, 3, 8)
        sd, dd = Distribution([1, 1, 1, 4]), Distribution([2, 2, 1, 1])
        src = [Tensor(tshape, LocaleVirtual(r, 4), sd).allocate() for r in range(4)]
        dst = [Tensor(tshape, LocaleVirtual(r, 4), dd).allocate() for r in range(4)]
        for t in src:
            t.data.uniform_(-1, 1, generator=g)
        keep = [t.data.clone() for t in src]
        sh = TensorShufflerVirtual(src, dst, stream=stream)
        sh.shuffle_forward()
        for t in src:
            t.data.zero_()
        sh.shuffle_backward()
        out["shuffle"] = [t.data for t in dst] + [t.data for t in src]
        out["shuffle_keep"] = keep
    return out


def test_user_stream_matches_default_stream():
    import torch
    ref = _run_all(None)
    torch.cuda.synchronize()
    ref = {k: [t.clone() for t in v] for k, v in ref.items()}

    side = torch.cuda.Stream()  # default priority
    busy = torch.empty(1 << 26, device="cuda")
    side.wait_stream(torch.cuda.current_stream())
    for _ in range(8):  # unrelated work on the default stream while the side stream runs
        busy.normal_()
    got = _run_all(side)
    for _ in range(8):
        busy.normal_()
    side.synchronize()
    torch.cuda.synchronize()
    for key, tensors in ref.items():
        for a, b in zip(tensors, got[key]):
            assert torch.equal(a, b) or (torch.isnan(a) == torch.isnan(b)).all() and \
                torch.equal(torch.nan_to_num(a), torch.nan_to_num(b)), key
    for kept, back in zip(got["shuffle_keep"], got["shuffle"][4:]):
        assert torch.equal(kept, back)

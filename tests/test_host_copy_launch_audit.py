"""What the halo and shuffle launches touch - on the CPU, through the launch audit of the copy
entry points (h2x_copy_audit_begin / _end; no GPU call).

The host layer runs unchanged on CPU tensors; the library plans every launch as usual and plays
each workgroup and lane through the code of the kernel itself, counting per byte what would be
loaded and stored.  The expectations are stated independently of that code, from the definition
of the strips and boxes: an exchange loads each rank's inner strips and stores its outer strips
(a strip spans the whole real extent of the other dimensions), a shuffle loads every interior
element of the source once and stores every interior element of the destination once, packed
buffers are written once and read once, and nothing else is touched."""
import itertools

import numpy as np
import pytest

from helpers import CopyAudit


def _tensors(shape, locale, overlap, dtype, audit):
    import torch
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    dist = Distribution.make_overlapped_distribution(locale, overlap)
    n = int(np.prod(locale))
    ts = [Tensor(shape, LocaleVirtual(r, n), dist, dtype, device="cpu").allocate() for r in range(n)]
    for t in ts:
        audit.register(t.data)
    return ts


def _strip(t, dim, side, width, inner):
    """Boolean mask (outermost dimension first) of a halo strip of a local tensor."""
    real = t.local_real_shape
    m = np.zeros(real[::-1], bool)
    start = {(0, 0): 0, (0, 1): width, (1, 0): real[dim] - width, (1, 1): real[dim] - 2 * width}[(side, int(inner))]
    index = [slice(None)] * len(real)
    index[len(real) - 1 - dim] = slice(start, start + width)
    m[tuple(index)] = True
    return m


def _expected_exchange(xch, reverse):
    """Per rank: how often each cell is loaded by the packs and stored by the unpacks of one
    full-width exchange (forward: inner strips -> outer strips; reverse: the other way round)."""
    from dihydrogen_amd import capi
    packed, unpacked = [], []
    for r, t in enumerate(xch.tensors):
        p, u = np.zeros(t.local_real_shape[::-1], np.int64), np.zeros(t.local_real_shape[::-1], np.int64)
        for d in range(xch.nd):
            w = t.overlap[d]
            if w == 0:
                continue
            for side in (capi.LHS, capi.RHS):
                if xch.find_peer_rank(r, d, side) is None:
                    continue
                p += _strip(t, d, side, w, inner=not reverse)
                u += _strip(t, d, side, w, inner=reverse)
        packed.append(p.ravel())
        unpacked.append(u.ravel())
    return packed, unpacked


def _clean(report):
    assert report.launches > 0
    assert (report.outside_loads, report.outside_stores, report.misaligned) == (0, 0, 0), \
        (report.outside_loads, report.outside_stores, report.misaligned)


# global shape (innermost first), locale, overlap
HALO_CASES = [
    ((16, 12, 3, 2), (2, 2, 1, 1), (1, 1, 0, 0)),
    ((14, 10, 3, 2), (2, 2, 1, 1), (2, 1, 0, 0)),          # rows of 7 + 4: no whole vectors
    ((38, 8, 2, 1), (2, 1, 1, 1), (3, 0, 0, 0)),           # innermost dimension only, width 3
    ((40, 6, 6, 2, 1), (2, 1, 2, 1, 1), (1, 0, 2, 0, 0)),  # 5-D; rows of 22 elements: vectors that straddle rows
    ((8, 8, 8, 3, 2), (2, 2, 2, 1, 1), (1, 1, 1, 0, 0)),
    ((12, 20, 2, 1), (1, 4, 1, 1), (0, 2, 0, 0)),          # four ranks in a line
    ((66, 4, 2, 1), (2, 2, 1, 1), (1, 1, 0, 0)),           # rows of 35 elements
]


@pytest.mark.parametrize("dtype", ["float32", "float64"])
@pytest.mark.parametrize("periodic", [False, True])
@pytest.mark.parametrize("fused", [False, True])
def test_forward_exchange_loads_inner_strips_and_stores_outer_strips(fused, periodic, dtype):
    import torch
    from dihydrogen_amd.layers import HaloExchangeVirtual
    for shape, locale, overlap in HALO_CASES:
        with CopyAudit() as audit:
            ts = _tensors(shape, locale, overlap, getattr(torch, dtype), audit)
            xch = HaloExchangeVirtual(ts, periodic=periodic)
            xch.exchange(fused=fused)
            want_loads, want_stores = _expected_exchange(xch, reverse=False)
        what = f"{shape} {locale} {overlap} periodic {periodic} fused {fused} {dtype}"
        if any(w.any() for w in want_loads):
            _clean(audit.report)
        for t, wl, ws in zip(ts, want_loads, want_stores):
            loads, stores = audit.counts(t.data)
            assert np.array_equal(loads, wl), what
            assert np.array_equal(stores, ws), what
        assert bool(audit.buffers) == (not fused and any(w.any() for w in want_loads)), what
        for b in audit.buffers:   # every packed strip is written once and read once
            loads, stores = audit.counts(b)
            assert (loads == 1).all() and (stores == 1).all(), what


@pytest.mark.parametrize("op", ["SUM", "MAX"])
@pytest.mark.parametrize("fused", [False, True])
def test_reverse_exchange_accumulates_into_inner_strips(fused, op):
    import torch
    from dihydrogen_amd.layers import HaloExchangeAccumOp, HaloExchangeVirtual
    for (shape, locale, overlap), dtype in itertools.product(HALO_CASES, (torch.float32, torch.float64)):
        with CopyAudit() as audit:
            ts = _tensors(shape, locale, overlap, dtype, audit)
            xch = HaloExchangeVirtual(ts, periodic=True)
            xch.exchange(is_reverse=True, op=HaloExchangeAccumOp[op], fused=fused)
            halo, boundary = _expected_exchange(xch, reverse=True)
        _clean(audit.report)
        for t, h, b in zip(ts, halo, boundary):
            loads, stores = audit.counts(t.data)
            # the halo strips are read, the boundary strips are read, combined and written
            assert np.array_equal(loads, h + b), (shape, locale, overlap, fused, op)
            assert np.array_equal(stores, b), (shape, locale, overlap, fused, op)


@pytest.mark.parametrize("only_unfilled", [False, True])
def test_clear_halos_stores_the_outer_strips_only(only_unfilled):
    import torch
    from dihydrogen_amd import capi
    from dihydrogen_amd.layers import HaloExchangeVirtual
    for (shape, locale, overlap), dtype in itertools.product(HALO_CASES, (torch.float32, torch.float64)):
        with CopyAudit() as audit:
            ts = _tensors(shape, locale, overlap, dtype, audit)
            xch = HaloExchangeVirtual(ts, periodic=False)
            xch.clear_halos(only_unfilled=only_unfilled)
        touched = False
        for r, t in enumerate(ts):
            want = np.zeros(t.local_real_shape[::-1], np.int64)
            for d in range(xch.nd):
                for side in (capi.LHS, capi.RHS):
                    if t.overlap[d] and not (only_unfilled and xch.find_peer_rank(r, d, side) is not None):
                        want += _strip(t, d, side, t.overlap[d], inner=False)
            loads, stores = audit.counts(t.data)
            assert not loads.any()
            assert np.array_equal(stores, want.ravel()), (shape, locale, overlap, only_unfilled)
            touched = touched or want.any()
        if touched:
            _clean(audit.report)


def test_single_strips_with_unaligned_buffers_and_every_width():
    """h2x_halo_pack_or_unpack on one tensor: every dimension, side and width up to the halo, the
    buffer on and off a 16-byte boundary."""
    import ctypes
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    for real, dtype in itertools.product(((22, 9, 5, 2), (13, 6, 4, 3, 2), (64, 6, 2, 1)), (torch.float32, torch.float64)):
        nd = len(real)
        for dim, side, width, is_pack, shift in itertools.product(range(nd - 2), (0, 1), (1, 2, 3), (1, 0), (0, 1)):
            if 2 * width > real[dim]:
                continue  # the boundary strip would leave the tensor: rejected by the library
            tensor = torch.zeros(int(np.prod(real)), dtype=dtype)
            n = lib.h2x_halo_size(nd, capi.i64_array(real), dim, width)
            assert n == width * int(np.prod(real)) // real[dim]
            whole = torch.zeros(n + 8, dtype=dtype)
            buffer = whole[shift:shift + n]
            with CopyAudit() as audit:
                audit.register(tensor)
                audit.register(whole)
                h2x_dtype = capi.F32 if dtype == torch.float32 else capi.F64
                capi.check(lib.h2x_halo_pack_or_unpack(
                    h2x_dtype, ctypes.c_void_p(tensor.data_ptr()), nd, capi.i64_array(real), dim, side, width,
                    ctypes.c_void_p(buffer.data_ptr()), is_pack, 0, 0, ctypes.c_void_p(0)), "pack_or_unpack")
            _clean(audit.report)

            class Shape:
                local_real_shape = list(real)
            strip = _strip(Shape, dim, side, width, inner=bool(is_pack)).ravel().astype(np.int64)
            t_loads, t_stores = audit.counts(tensor)
            b_loads, b_stores = audit.counts(whole)
            used = np.zeros(n + 8, np.int64)
            used[shift:shift + n] = 1
            what = (real, dim, side, width, is_pack, shift)
            assert np.array_equal(t_loads if is_pack else t_stores, strip), what
            assert not (t_stores if is_pack else t_loads).any(), what
            assert np.array_equal(b_stores if is_pack else b_loads, used), what
            assert not (b_loads if is_pack else b_stores).any(), what


def test_shuffles_load_every_source_element_and_store_every_destination_element_once():
    import torch
    import test_gpu_shuffle as cases
    from dihydrogen_amd.layers import TensorShufflerVirtual
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    for (name, (shape, (sl, ss, so), (dl, ds, do))), dtype in itertools.product(
            cases.CASES.items(), (torch.float32, torch.int16, torch.float64)):
        if ss is not None or ds is not None:
            continue  # shared distributions: ranks that are no split roots move nothing
        n = int(np.prod(sl))
        for forward in (True, False):
            with CopyAudit() as audit:
                src = [Tensor(shape, LocaleVirtual(r, n), Distribution(sl, ss, so), dtype, device="cpu").allocate()
                       for r in range(n)]
                dst = [Tensor(shape, LocaleVirtual(r, n), Distribution(dl, ds, do), dtype, device="cpu").allocate()
                       for r in range(n)]
                for t in src + dst:
                    audit.register(t.data)
                sh = TensorShufflerVirtual(src, dst)
                (sh.shuffle_forward if forward else sh.shuffle_backward)()
                del sh
            _clean(audit.report)
            read, written = (src, dst) if forward else (dst, src)
            for t in read + written:
                interior = np.zeros(t.local_real_shape[::-1], np.int64)
                index = tuple(slice(o, o + l) for o, l in zip(reversed(t.overlap), reversed(t.local_shape)))
                interior[index] = 1
                loads, stores = audit.counts(t.data)
                if interior.size == 0:      # a rank without data (one padding element is allocated)
                    assert not loads.any() and not stores.any(), (name, forward, dtype)
                    continue
                if any(t is r for r in read):
                    assert np.array_equal(loads, interior.ravel()) and not stores.any(), (name, forward, dtype)
                else:
                    assert np.array_equal(stores, interior.ravel()) and not loads.any(), (name, forward, dtype)
            used = 0
            for b in audit.buffers:   # one arena per direction: the one in use is written once and read once
                loads, stores = audit.counts(b)
                if loads.any() or stores.any():
                    assert (loads == 1).all() and (stores == 1).all(), (name, forward, dtype)
                    used += 1
            assert used == 1, (name, forward, dtype)


def test_an_access_outside_the_registered_ranges_is_reported():
    """The audit itself: a tensor registered one element short shows up as bytes outside."""
    import ctypes
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    real = (10, 6, 3, 1)
    tensor = torch.zeros(int(np.prod(real)), dtype=torch.float32)
    n = lib.h2x_halo_size(4, capi.i64_array(real), 1, 1)
    buffer = torch.zeros(n, dtype=torch.float32)
    with CopyAudit() as audit:
        audit.register(tensor[:-1])     # the last element of the RHS strip of dimension 1 is missing
        audit.register(buffer)
        capi.check(lib.h2x_halo_pack_or_unpack(capi.F32, ctypes.c_void_p(tensor.data_ptr()), 4, capi.i64_array(real),
                                               1, 1, 1, ctypes.c_void_p(buffer.data_ptr()), 0, 0, 0,
                                               ctypes.c_void_p(0)), "unpack")
    assert audit.report.outside_stores > 0 and audit.report.outside_loads == 0
    # calls outside an audit are not affected: without a GPU they fail with HIP's error, with one they run
    assert lib.h2x_copy_audit_end(None) == -1


def test_random_halo_and_shuffle_geometries():
    """Seeded random decompositions (the generators of the GPU suite, other seeds): forward and reverse
    exchanges and shuffles in both directions touch what their definition says, and nothing else."""
    import torch
    import test_gpu_random_shapes as shapes
    from dihydrogen_amd.layers import HaloExchangeAccumOp, HaloExchangeVirtual, TensorShufflerVirtual
    from dihydrogen_amd.tensor import Distribution, LocaleVirtual, Tensor
    for (shape, locale, overlap, periodic, fused), reverse in itertools.product(shapes._halo_cases(60, 731), (False, True)):
        with CopyAudit() as audit:
            ts = _tensors(shape, locale, overlap, torch.float32, audit)
            xch = HaloExchangeVirtual(ts, periodic=periodic)
            xch.exchange(is_reverse=reverse, op=HaloExchangeAccumOp.SUM if reverse else HaloExchangeAccumOp.ID,
                         fused=fused)
            packed, unpacked = _expected_exchange(xch, reverse=reverse)
        what = (shape, locale, overlap, periodic, fused, reverse)
        assert (audit.report.outside_loads, audit.report.outside_stores, audit.report.misaligned) == (0, 0, 0), what
        for t, p, u in zip(ts, packed, unpacked):
            loads, stores = audit.counts(t.data)
            assert np.array_equal(loads, p + u if reverse else p) and np.array_equal(stores, u), what
    for (shape, (sl, ss, so), (dl, ds, do)), forward in itertools.product(shapes._shuffle_cases(40, 732), (True, False)):
        if ss is not None or ds is not None:
            continue
        n = int(np.prod(sl))
        with CopyAudit() as audit:
            src = [Tensor(shape, LocaleVirtual(r, n), Distribution(sl, ss, so), device="cpu").allocate() for r in range(n)]
            dst = [Tensor(shape, LocaleVirtual(r, n), Distribution(dl, ds, do), device="cpu").allocate() for r in range(n)]
            for t in src + dst:
                audit.register(t.data)
            sh = TensorShufflerVirtual(src, dst)
            (sh.shuffle_forward if forward else sh.shuffle_backward)()
            del sh
        what = (shape, sl, so, dl, do, forward)
        assert (audit.report.outside_loads, audit.report.outside_stores, audit.report.misaligned) == (0, 0, 0), what
        read = src if forward else dst
        for t in src + dst:
            interior = np.zeros(t.local_real_shape[::-1], np.int64)
            interior[tuple(slice(o, o + l) for o, l in zip(reversed(t.overlap), reversed(t.local_shape)))] = 1
            loads, stores = audit.counts(t.data)
            moved, other = (loads, stores) if any(t is r for r in read) else (stores, loads)
            assert not other.any() and (np.array_equal(moved, interior.ravel()) if interior.size else not moved.any()), what


def test_strips_of_a_tensor_beyond_2_to_the_32_elements():
    """Offsets that need 64 bits: the far strips of an (imaginary) tensor of 4.85 billion elements.  The
    outermost strip is contiguous, so its own byte range is registered with counters and everything else
    counts as outside; the strided strip of dimension 1 is checked against the bounds of the tensor."""
    import ctypes
    import torch
    from dihydrogen_amd import capi
    lib = capi.load()
    real = (2100, 2100, 1100, 1, 1)
    total = int(np.prod(real))
    assert total > 2 ** 32
    base = 1 << 44                     # never followed
    for dim, is_pack in itertools.product((2, 1), (1, 0)):
        n = lib.h2x_halo_size(5, capi.i64_array(real), dim, 1)
        buffer = torch.zeros(n, dtype=torch.float32)
        with CopyAudit() as audit:
            audit.register(buffer)
            region = capi.CopyAuditRegion()
            if dim == 2:
                # RHS strip, inner when packing: plane 1098 (1099 is the halo), outer when unpacking: plane 1099
                plane = 1098 if is_pack else 1099
                loads = np.zeros(n * 4, np.uint8)
                stores = np.zeros(n * 4, np.uint8)
                region.base, region.bytes = base + plane * 2100 * 2100 * 4, n * 4
                region.loads = loads.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8))
                region.stores = stores.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8))
            else:
                region.base, region.bytes = base, total * 4      # bounds only
            capi.check(lib.h2x_copy_audit_add_region(ctypes.byref(region)), "region")
            capi.check(lib.h2x_halo_pack_or_unpack(capi.F32, ctypes.c_void_p(base), 5, capi.i64_array(real), dim, 1, 1,
                                                   ctypes.c_void_p(buffer.data_ptr()), is_pack, 0, 0,
                                                   ctypes.c_void_p(0)), "pack_or_unpack")
        _clean(audit.report)
        b_loads, b_stores = audit.counts(buffer)
        assert ((b_stores if is_pack else b_loads) == 1).all() and not (b_loads if is_pack else b_stores).any()
        if dim == 2:
            assert ((loads if is_pack else stores) == 1).all() and not (stores if is_pack else loads).any()

"""Which kernels a batch-normalisation call launches, with what geometry, and
what those launches touch - on the CPU, through h2x_bn_audit (no GPU call).

The library plans the launches of an entry point and plays every workgroup and
lane through the index maps of its kernels.  The checks here are stated
independently of that code: the set of interior elements comes from shape and
strides, and the expected family of kernels comes from the rule below.

Dispatch rule (shape -> family), as documented for the library:
  1. a (sample, channel) segment of at most 256 elements      -> short segments
  2. else a tensor with halos inside its segments             -> strided (rows padded to vectors)
  3. else segments of 257..1023 elements and several samples  -> strided, samples folded into rows
  4. else every tensor 16-byte aligned, segment a multiple of
     the vector                                                -> dense, full vectors
  5. else                                                      -> strided, one row per segment
Every shape lands in exactly one of them.
"""
import ctypes
import itertools

import pytest

from dihydrogen_amd import capi

SHORT, DENSE, STRIDED = 2, 0, 1
MAIN = (0, 1, 2, 3)  # kernels that walk tensors
REDUCTIONS = (0, 2)


def dense_geometry(n, c, s, real=None):
    real = s if real is None else real
    g = capi.TensorGeometry()
    g.num_dims = 3
    for i, (e, st) in enumerate(zip((s, c, n), (1, real, real * c))):
        g.local_shape[i], g.strides[i] = e, st
    return g


def haloed_geometry(spatial, c, n, halo):
    """Local shape `spatial` (innermost first) with `halo[d]` cells on both sides of dimension d."""
    g = capi.TensorGeometry()
    shape = list(spatial) + [c, n]
    real = [e + 2 * h for e, h in zip(spatial, halo)] + [c, n]
    g.num_dims = len(shape)
    stride = 1
    for i, e in enumerate(shape):
        g.local_shape[i], g.strides[i] = e, stride
        stride *= real[i]
    return g


def audit(stage, dtype, n, geometries, addresses):
    lib = capi.load()
    arr = (ctypes.POINTER(capi.TensorGeometry) * 3)(*[ctypes.pointer(g) for g in geometries])
    adr = (ctypes.c_uint64 * 3)(*(list(addresses) + [0] * (3 - len(addresses))))
    rep = capi.BnAuditReport()
    err = lib.h2x_bn_audit(stage, dtype, n, arr, adr, ctypes.byref(rep))
    return err, rep


def tensors_of(stage):
    return {capi.BN_STAGE_SUMS: 1, capi.BN_STAGE_NORMALIZE: 2, capi.BN_STAGE_BACKPROP1: 2,
            capi.BN_STAGE_BACKPROP2: 3, capi.BN_STAGE_FORWARD_LOCAL: 2, capi.BN_STAGE_BACKWARD_LOCAL: 3}[stage]


def check_report(rep, what):
    assert 1 <= rep.num_launches <= capi.BN_AUDIT_MAX_LAUNCHES, what
    mains = []
    for i in range(rep.num_launches):
        l = rep.launch[i]
        assert 1 <= l.grid_x <= 0x7FFFFFFF and 1 <= l.grid_y <= 65535, (what, l.grid_x, l.grid_y)
        if l.kernel not in MAIN:
            continue
        mains.append(l)
        assert l.family in (SHORT, DENSE, STRIDED), what
        if l.kernel in REDUCTIONS:
            assert l.partials_bytes <= l.partials_capacity <= rep.workspace_bytes, (what, l.partials_bytes)
        for t in range(l.num_tensors):
            c = l.tensor[t]
            assert (c.outside, c.missed, c.owned_twice) == (0, 0, 0), \
                (what, "kernel", l.kernel, "family", l.family, "tensor", t, c.outside, c.missed, c.owned_twice)
            assert c.loads + c.stores > 0, what
    return mains


def expected_family(dtype, n, spatial_elems, haloed_inside, aligned):
    vec = 4 if dtype == capi.F32 else 2
    if spatial_elems <= 256:
        return SHORT, False
    if haloed_inside:
        return STRIDED, False
    if spatial_elems < 1024 and n > 1:
        return STRIDED, True
    if aligned and spatial_elems % vec == 0:
        return DENSE, False
    return STRIDED, False


STAGES = (capi.BN_STAGE_SUMS, capi.BN_STAGE_NORMALIZE, capi.BN_STAGE_BACKPROP1, capi.BN_STAGE_BACKPROP2,
          capi.BN_STAGE_FORWARD_LOCAL, capi.BN_STAGE_BACKWARD_LOCAL)
SPATIAL = (1, 2, 3, 4, 5, 49, 196, 255, 256, 257, 361, 1023, 1024, 1027, 3249, 4096, 4100, 9000)


@pytest.mark.parametrize("dtype", (capi.F32, capi.F64))
@pytest.mark.parametrize("stage", STAGES)
def test_dense_tensors_land_in_one_family_and_touch_only_their_interior(stage, dtype):
    elem = 4 if dtype == capi.F32 else 8
    vec = 16 // elem
    for s, (n, c), pad, shift in itertools.product(SPATIAL, ((1, 3), (2, 1), (5, 3), (3, 70)), (0, 3), (0, 1)):
        if c == 70 and s > 1100:
            continue  # keeps the walk short; the large channel count is covered at the small segments
        k = tensors_of(stage)
        geometries = [dense_geometry(n, c, s, s + pad) for _ in range(k)]
        base = 1 << 20
        addresses = [base + t * (1 << 30) + shift * elem for t in range(k)]
        err, rep = audit(stage, dtype, n, geometries, addresses)
        what = f"stage {stage} dtype {dtype} N {n} C {c} S {s} pad {pad} shift {shift}"
        assert err == 0, what
        mains = check_report(rep, what)
        aligned = shift == 0 and (s + pad) % vec == 0
        family, folded = expected_family(dtype, n, s, False, aligned)
        for l in mains:
            assert (l.family, bool(l.folded)) == (family, folded), (what, l.kernel, l.family, l.folded)
            if family == DENSE:
                assert l.vector_width == vec
        # the two-launch entry points: a reduction that leaves partial sums and a consumer that adds them
        if stage in (capi.BN_STAGE_FORWARD_LOCAL, capi.BN_STAGE_BACKWARD_LOCAL):
            assert [l.kernel for l in mains] == ([0, 1] if stage == capi.BN_STAGE_FORWARD_LOCAL else [2, 3]), what
            assert rep.num_launches == 2 and mains[1].fused == 1, what


HALOED_4D = [((7, 7), (1, 1)), ((14, 14), (1, 1)), ((16, 16), (2, 1)), ((5, 51), (1, 0)), ((30, 30), (1, 1)),
             ((57, 57), (1, 1)), ((64, 40), (0, 1)), ((130, 3), (1, 1)), ((3, 100), (1, 1)), ((1, 300), (1, 1))]
HALOED_5D = [((4, 4, 4), (1, 1, 1)), ((8, 8, 8), (1, 1, 1)), ((30, 6, 5), (1, 0, 1)), ((64, 8, 8), (0, 0, 1)),
             ((33, 9, 3), (1, 1, 0)), ((6, 6, 40), (0, 1, 1))]


@pytest.mark.parametrize("dtype", (capi.F32, capi.F64))
@pytest.mark.parametrize("stage", STAGES)
def test_haloed_tensors_land_in_one_family_and_touch_only_their_interior(stage, dtype):
    elem = 4 if dtype == capi.F32 else 8
    vec = 16 // elem
    k = tensors_of(stage)
    for (spatial, halo), (n, c) in itertools.product(HALOED_4D + HALOED_5D, ((1, 2), (3, 5))):
        s = 1
        for e in spatial:
            s *= e
        # every tensor haloed, and each tensor in turn dense beside haloed ones
        layouts = [[True] * k] + [[i != j for i in range(k)] for j in range(k) if k > 1]
        for haloed in layouts:
            geometries = [haloed_geometry(spatial, c, n, halo if h else [0] * len(halo)) for h in haloed]
            addresses = [(1 << 20) + t * (1 << 30) + (elem if t == 1 else 0) for t in range(k)]
            err, rep = audit(stage, dtype, n, geometries, addresses)
            what = f"stage {stage} dtype {dtype} N {n} C {c} spatial {spatial} halo {halo} haloed {haloed}"
            assert err == 0, what
            mains = check_report(rep, what)
            for l in mains:
                # the tensors this launch addresses: a reduction of a two-launch stage sees x (and dy) only
                seen = haloed[:l.num_tensors]
                # a halo on the outermost spatial dimension only leaves the segments dense inside
                inside = any(h and any(halo[:-1]) for h in seen)
                aligned = False  # the second tensor starts one element off a 16-byte boundary
                if l.num_tensors == 1:
                    real_c = 1
                    for e, h in zip(spatial, halo if seen[0] else [0] * len(halo)):
                        real_c *= e + 2 * h
                    aligned = real_c % vec == 0
                family, folded = expected_family(dtype, n, s, inside, aligned)
                assert (l.family, bool(l.folded)) == (family, folded), (what, l.kernel, l.family, l.folded)


@pytest.mark.parametrize("dtype", (capi.F32, capi.F64))
def test_input_gradient_in_place_stores_every_element_once(dtype):
    """dx may be x itself: the elements two overlapping vectors share are then stored by
    their owner only, so stores = interior elements; with disjoint tensors both lanes store them."""
    for geometry, n, c in ((dense_geometry(2, 3, 3249), 2, 3), (dense_geometry(4, 6, 49), 4, 6),
                           (haloed_geometry((57, 57), 3, 2, (1, 1)), 2, 3),
                           (haloed_geometry((7, 7), 6, 4, (1, 1)), 4, 6),
                           (haloed_geometry((31, 6, 5), 2, 2, (1, 1, 1)), 2, 2)):
        elems = n * c
        for d in range(geometry.num_dims - 2):
            elems *= geometry.local_shape[d]
        stores = {}
        for alias in (True, False):
            x = 1 << 20
            err, rep = audit(capi.BN_STAGE_BACKPROP2, dtype, n, [geometry] * 3,
                             [x, x + (1 << 30), x if alias else x + (2 << 30)])
            assert err == 0
            (l,) = check_report(rep, f"in place {alias}")
            stores[alias] = l.tensor[2].stores
        assert stores[True] == elems
        assert stores[False] > elems  # rows of 57, 49 or 31 elements end in an overlapping vector


def test_rejected_and_empty_calls():
    # more channels than a grid dimension holds: the long-segment reductions refuse, nothing is planned
    err, _ = audit(capi.BN_STAGE_SUMS, capi.F32, 1, [dense_geometry(1, 70000, 300)], [1 << 20])
    assert err == -3
    err, _ = audit(capi.BN_STAGE_FORWARD_LOCAL, capi.F32, 1, [dense_geometry(1, 70000, 300)] * 2, [1 << 20, 1 << 30])
    assert err == -3
    # the short-segment kernels take any channel count
    err, rep = audit(capi.BN_STAGE_SUMS, capi.F32, 2, [dense_geometry(2, 70000, 4)], [1 << 20])
    assert err == 0
    check_report(rep, "70000 channels of 4 elements")
    # no samples: the per-channel outputs are zeroed, no tensor is touched
    err, rep = audit(capi.BN_STAGE_SUMS, capi.F32, 0, [dense_geometry(0, 8, 64)], [1 << 20])
    assert err == 0 and [rep.launch[i].kernel for i in range(rep.num_launches)] == [6, 6]
    # geometries of unequal local shape
    err, _ = audit(capi.BN_STAGE_NORMALIZE, capi.F32, 2,
                   [haloed_geometry((8, 4), 3, 2, (1, 1)), haloed_geometry((4, 8), 3, 2, (1, 1))], [1 << 20, 1 << 30])
    assert err == -1


def clearing_geometry(spatial, c, n, lower, upper):
    g = capi.HaloedGeometry()
    shape = list(spatial) + [c, n]
    g.num_dims = len(shape)
    for i, e in enumerate(shape):
        lo = lower[i] if i < len(spatial) else 0
        hi = upper[i] if i < len(spatial) else 0
        g.local_shape[i], g.real_shape[i], g.lower_halo[i] = e, e + lo + hi, lo
    return g


def audit_clearing(backward, dtype, geometry, addresses):
    lib = capi.load()
    adr = (ctypes.c_uint64 * 3)(*(list(addresses) + [0] * (3 - len(addresses))))
    rep = capi.BnAuditReport()
    err = lib.h2x_bn_audit_clearing(int(backward), dtype, ctypes.byref(geometry), adr, ctypes.byref(rep))
    return err, rep


CLEARING = [((64, 64, 64), (1, 1, 1), (1, 1, 1)), ((14, 14), (1, 1), (1, 1)), ((7, 7), (1, 1), (1, 1)),
            ((30, 6, 5), (1, 0, 1), (1, 0, 1)), ((8, 8, 8), (2, 1, 0), (0, 1, 2)), ((33, 9), (3, 2), (0, 1)),
            ((5, 51), (0, 1), (0, 1)), ((1, 300), (1, 1), (1, 1)), ((130, 3), (1, 1), (2, 2)), ((6, 6, 40), (0, 1, 1), (0, 1, 1)),
            ((12, 3, 4), (0, 0, 0), (0, 0, 0)),
            # real planes of 15 and 18 cells, no halo on dimension 1: vectors that begin in the last row
            # of one plane and end in the first, interior, row of the next
            ((4, 3, 2), (1, 0, 1), (0, 0, 1)), ((5, 3, 2), (1, 0, 1), (0, 0, 1))]


@pytest.mark.parametrize("dtype", (capi.F32, capi.F64))
@pytest.mark.parametrize("backward", (False, True))
def test_halo_clearing_kernels_store_every_real_cell_once_and_zero_exactly_the_halo(backward, dtype):
    elem = 4 if dtype == capi.F32 else 8
    vec = 16 // elem
    for (spatial, lower, upper), (n, c), shift in itertools.product(CLEARING, ((1, 2), (3, 5)), (0, 1)):
        if spatial[0] == 64 and (n, c) != (1, 2):
            continue  # the large box once: enough to cross several chunks
        g = clearing_geometry(spatial, c, n, lower, upper)
        real = 1
        for e, lo, hi in zip(spatial, lower, upper):
            real *= e + lo + hi
        k = 3 if backward else 2
        x = (1 << 20) + shift * elem
        # out of place, and in place (the output is x itself)
        for out in (x + (2 << 30), x):
            addresses = [x, x + (1 << 30), out][:k - 1] + [out]
            err, rep = audit_clearing(backward, dtype, g, addresses)
            what = f"backward {backward} dtype {dtype} spatial {spatial} halo {lower}/{upper} N {n} C {c} shift {shift}"
            assert err == 0 and rep.num_launches == 1, what
            l = rep.launch[0]
            assert l.kernel == 7 and l.num_tensors == k and 1 <= l.grid_x <= 0x7FFFFFFF, what
            assert l.vector_width == (vec if real % vec == 0 and shift == 0 else 1), what
            for t in range(k):
                c_ = l.tensor[t]
                assert (c_.outside, c_.missed, c_.owned_twice) == (0, 0, 0), (what, t, c_.outside, c_.missed, c_.owned_twice)
            assert l.tensor[k - 1].stores == n * c * real, what
            assert all(l.tensor[t].loads == n * c * real for t in range(k - 1)), what


def test_halo_clearing_audit_rejects_what_the_entry_points_reject():
    g = clearing_geometry((8, 8), 3, 2, (1, 1), (1, 1))
    g.lower_halo[2] = 1          # a halo on the channel dimension
    g.real_shape[2] += 1
    err, _ = audit_clearing(False, capi.F32, g, [1 << 20, 1 << 30])
    assert err == -2
    g = clearing_geometry((8, 8), 3, 2, (1, 1), (1, 1))
    g.real_shape[0] = 8          # real extent smaller than halo + local
    err, _ = audit_clearing(False, capi.F32, g, [1 << 20, 1 << 30])
    assert err == -1
    # nothing to do: no launch is planned
    err, rep = audit_clearing(True, capi.F32, clearing_geometry((8, 8), 0, 2, (1, 1), (1, 1)), [1 << 20, 1 << 30, 1 << 31])
    assert err == 0 and rep.num_launches == 0

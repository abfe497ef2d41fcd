"""GPU parity on seeded random shapes.

The kernels are chosen from the geometry (segment length, channel count, samples,
vector alignment); the hand-picked cases of the other files sit on the borders
that were known when they were written.  These draws cover the space between:
every shape runs the same checks as the hand-picked ones (against the CPU oracle,
and the two-launch paths against the staged calls bit for bit).
"""
import numpy as np
import pytest

import test_gpu_bn as bn_tests
import test_gpu_softmax as softmax_tests

pytestmark = pytest.mark.gpu


def _spatial(rng, lo, hi, nd):
    """nd extents whose product lies in [lo, hi]."""
    for _ in range(1000):
        target = int(np.exp(rng.uniform(np.log(lo), np.log(hi))))
        dims = []
        rest = target
        for i in range(nd - 1):
            d = int(rng.integers(1, max(2, int(round(rest ** (1.0 / (nd - i)) * 2)))))
            d = max(1, min(d, rest))
            dims.append(d)
            rest = max(1, rest // d)
        dims.append(rest)
        p = int(np.prod(dims))
        if lo <= p <= hi:
            return tuple(int(d) for d in dims)
    return (lo,) + (1,) * (nd - 1)


def _bn_shapes(count=36, seed=20240607, max_elems=400_000):
    rng = np.random.default_rng(seed)
    shapes = []
    regimes = [(1, 256), (1, 256), (257, 1023), (1024, 6000)]   # short segments twice as often
    while len(shapes) < count:
        lo, hi = regimes[len(shapes) % len(regimes)]
        sp = _spatial(rng, lo, hi, int(rng.integers(2, 4)))
        s = int(np.prod(sp))
        c = int(np.exp(rng.uniform(0, np.log(700))))
        n_max = max(1, max_elems // (s * c))
        n = int(np.exp(rng.uniform(0, np.log(min(n_max, 700)))))
        shapes.append((n, c) + sp)
    return shapes


def _bn_long_shapes(count=12, seed=20240613, max_elems=6_000_000):
    """Segments of 6 000 to 1.5 million elements: the chunking of the long-segment kernels
    (chunks of whole tiles, last chunks, odd lengths that end in an overlapping vector)."""
    rng = np.random.default_rng(seed)
    shapes = []
    while len(shapes) < count:
        sp = _spatial(rng, 6000, 1_500_000, int(rng.integers(2, 4)))
        s = int(np.prod(sp))
        c = int(np.exp(rng.uniform(0, np.log(max(1, min(40, max_elems // s))))))
        n = int(np.exp(rng.uniform(0, np.log(max(1, min(8, max_elems // (s * c)))))))
        shapes.append((n, c) + sp)
    return shapes


def _softmax_shapes(count=30, seed=20240608, max_elems=300_000):
    rng = np.random.default_rng(seed)
    shapes = []
    while len(shapes) < count:
        c = int(np.exp(rng.uniform(0, np.log(560))))          # past the largest register tile (512)
        kind = len(shapes) % 3
        sp = (1, 1) if kind == 0 else _spatial(rng, 2, max(2, min(5000, max_elems // c)), int(rng.integers(2, 4)))
        s = int(np.prod(sp))
        n = int(np.exp(rng.uniform(0, np.log(max(1, min(300, max_elems // (s * c)))))))
        shapes.append((n, c) + sp)
    return shapes


def _instance_shapes(count=16, seed=20240609):
    rng = np.random.default_rng(seed)
    shapes = []
    while len(shapes) < count:
        size = int(np.exp(rng.uniform(0, np.log(9000))))      # around the wave-per-sample limit (2048)
        n = int(np.exp(rng.uniform(0, np.log(max(1, min(400, 300_000 // size))))))
        shapes.append((n, size))
    return shapes


@pytest.mark.parametrize("shape", _bn_shapes())
def test_batch_norm(shape, oracle_mod):
    if shape[0] * int(np.prod(shape[2:])) > 1:
        bn_tests.test_forward_matches_oracle(shape, oracle_mod)
        bn_tests.test_backward_matches_oracle(shape, oracle_mod)
    for dtype in ("float32", "float64"):
        bn_tests.test_two_launch_forward_and_backward_equal_the_staged_calls(shape, dtype)


@pytest.mark.parametrize("shape", _bn_long_shapes())
def test_batch_norm_on_long_segments(shape, oracle_mod):
    test_batch_norm(shape, oracle_mod)


@pytest.mark.parametrize("shape", _softmax_shapes())
def test_channel_softmax(shape, oracle_mod):
    softmax_tests.test_forward_backward(shape, oracle_mod)


@pytest.mark.parametrize("shape", _instance_shapes())
def test_instance_softmax(shape, oracle_mod):
    softmax_tests.test_instance_mode(shape, oracle_mod)
    for dtype in (np.float32, np.float64):
        softmax_tests.test_instance_forward_in_four_passes_equals_the_staged_calls(shape, dtype)


def _factor(rng, n, slots):
    """n as a product over `slots` positions (random assignment of its prime factors)."""
    out = [1] * slots
    p = 2
    while n > 1:
        while n % p == 0:
            out[int(rng.integers(0, slots))] *= p
            n //= p
        p += 1
    return out


def _halo_cases(count=24, seed=20240610):
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        nd = int(rng.integers(4, 6))
        ns = nd - 2
        locale = _factor(rng, int(rng.choice([2, 3, 4, 6, 8, 12])), ns) + [1, 1]
        overlap = [int(rng.integers(0, 4)) if locale[d] > 1 or rng.random() < 0.3 else 0 for d in range(ns)] + [0, 0]
        if not any(overlap[d] and locale[d] > 1 for d in range(ns)):
            continue
        shape = [int(locale[d] * max(overlap[d], 1) + rng.integers(0, 24)) for d in range(ns)]
        shape += [int(rng.integers(1, 6)), int(rng.integers(1, 4))]
        if int(np.prod(shape)) > 200_000:
            continue
        cases.append((tuple(shape), tuple(locale), tuple(overlap), bool(rng.integers(0, 2)), bool(rng.integers(0, 2))))
    return cases


def _shuffle_cases(count=24, seed=20240611):
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        nd = int(rng.integers(4, 6))
        ns = nd - 2
        n = int(rng.choice([2, 3, 4, 6, 8, 16]))
        def locale(kind):
            if kind == 0:                                    # sample-distributed
                return [1] * (nd - 1) + [n]
            if kind == 1:                                    # spatially distributed
                return _factor(rng, n, ns) + [1, 1]
            f = _factor(rng, n, ns + 1)                      # spatial dimensions and samples
            return f[:ns] + [1] + f[ns:]
        sl, dl = locale(int(rng.integers(0, 3))), locale(int(rng.integers(1, 3)))
        shape = [int(rng.integers(1, 3) * max(sl[d], dl[d]) + rng.integers(0, 20)) for d in range(ns)]
        shape += [int(rng.integers(1, 5)), int(max(sl[-1], dl[-1]) * rng.integers(1, 3) + rng.integers(0, 3))]
        if int(np.prod(shape)) > 150_000:
            continue
        def overlap(loc):
            if rng.random() < 0.5:
                return None
            ov = [int(rng.integers(0, 3)) if loc[d] > 1 and shape[d] // loc[d] >= 2 else 0 for d in range(ns)] + [0, 0]
            return tuple(ov) if any(ov) else None
        cases.append((tuple(shape), (tuple(sl), None, overlap(sl)), (tuple(dl), None, overlap(dl))))
    return cases


def _bn_halo_cases(count=16, seed=20240612):
    """Spatially decomposed tensors with halos, for batch-norm on every rank: local tiles from a
    few elements (the short-segment kernels, slots by rows) to a few thousand (padded rows)."""
    rng = np.random.default_rng(seed)
    cases = []
    while len(cases) < count:
        nd = int(rng.integers(4, 6))
        ns = nd - 2
        locale = _factor(rng, int(rng.choice([2, 4, 8])), ns) + [1, 1]
        overlap = [int(rng.integers(0, 3)) for _ in range(ns)] + [0, 0]
        if not any(overlap[:ns - 1]):            # a halo on an inner dimension: the strided layout
            continue
        small = len(cases) % 2 == 0
        shape = [int(locale[d] * rng.integers(max(overlap[d], 1), 9 if small else 40)) for d in range(ns)]
        shape += [int(np.exp(rng.uniform(0, np.log(40)))), int(rng.integers(1, 6))]
        if int(np.prod(shape)) > 150_000:
            continue
        cases.append((tuple(shape), tuple(locale), tuple(overlap)))
    return cases


@pytest.mark.parametrize("case", _bn_halo_cases())
def test_batch_norm_on_haloed_tensors(case, oracle_mod):
    bn_tests.test_haloed_tensors_match_oracle(case, oracle_mod)


@pytest.mark.parametrize("case", _halo_cases())
def test_halo_exchange(case, oracle_mod):
    import test_gpu_halo as halo_tests
    shape, locale, overlap, periodic, fused = case
    geoms, want, got = halo_tests._exchange_case(shape, locale, overlap, periodic, oracle_mod, fused=fused)
    halo_tests._closed_form_check(geoms, got, periodic)
    for w, g in zip(want, got):
        assert np.array_equal(w, g, equal_nan=True)


@pytest.mark.parametrize("index", range(24))
def test_shuffle(index):
    import test_gpu_shuffle as shuffle_tests
    name = f"random_{index}"
    shuffle_tests.CASES[name] = _shuffle_cases()[index]
    try:
        shuffle_tests.test_forward_backward_closed_form(name)
    finally:
        del shuffle_tests.CASES[name]

"""On a machine without a GPU: calls the library must reject are rejected with its own (negative)
status before any HIP call is made, and a valid call fails loudly with HIP's own (positive) error:
there is no CPU path behind the C ABI.

Pointers are imaginary (never followed: nothing is launched).  The whole file is skipped where a GPU is
visible, because a valid call would then launch on those pointers; the GPU twin of these checks, with
real buffers, is tests/test_gpu_abi_edges.py."""
import ctypes

import pytest

from dihydrogen_amd import capi

INVALID, UNSUPPORTED, TOO_LARGE = -1, -2, -3
P = ctypes.c_void_p(1 << 20)


@pytest.fixture(autouse=True)
def no_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is visible: these calls would launch on imaginary pointers")


def test_batch_norm_and_softmax_rejections():
    lib = capi.load()
    c = 4
    assert lib.h2x_bn_channel_sums_and_sqsums(7, 2, c, 8, 8, P, P, P, P, None) == UNSUPPORTED
    assert lib.h2x_bn_channel_sums_and_sqsums(capi.F32, -1, c, 8, 8, P, P, P, P, None) == INVALID
    assert lib.h2x_bn_channel_sums_and_sqsums(capi.F32, 2, c, 8, 7, P, P, P, P, None) == INVALID
    assert lib.h2x_bn_channel_sums_and_sqsums(capi.F32, 2, c, 8, 8, P, None, P, P, None) == INVALID
    assert lib.h2x_bn_channel_sums_and_sqsums(capi.F32, 2, c, 8, 8, P, P, P, None, None) == INVALID
    assert lib.h2x_bn_channel_sums_and_sqsums(capi.F32, 2, c, 8, 8, None, P, P, P, None) == INVALID
    assert lib.h2x_bn_batch_normalization(capi.F32, 2, c, 8, 8, 4, P, P, P, P, P, P, 1e-5, None) == INVALID
    assert lib.h2x_bn_backprop1(capi.F32, 2, c, 8, 8, 8, P, P, P, P, P, P, P, P, None, 1e-5, P, None) == INVALID
    assert lib.h2x_bn_channel_sums_and_sqsums_static(capi.F32, 2, lib.h2x_bn_static_max_channels() + 1, 8, 8, P, P,
                                                     P, None) == -4
    assert lib.h2x_softmax_channel_forward(capi.F32, -2, c, 8, P, P, None) == INVALID
    assert lib.h2x_softmax_channel_forward(9, 2, c, 8, P, P, None) == UNSUPPORTED
    g = capi.TensorGeometry()
    g.num_dims = 6
    assert lib.h2x_bn_channel_sums_and_sqsums_strided(capi.F32, 2, ctypes.byref(g), P, P, P, P, None) == INVALID
    g.num_dims = 4
    for i, (e, s) in enumerate(zip((4, 2, c, 2), (2, 8, 16, 64))):     # innermost stride 2
        g.local_shape[i], g.strides[i] = e, s
    assert lib.h2x_bn_channel_sums_and_sqsums_strided(capi.F32, 2, ctypes.byref(g), P, P, P, P, None) == UNSUPPORTED
    # more channels than a grid dimension holds, long segments
    assert lib.h2x_bn_channel_sums_and_sqsums(capi.F32, 1, 70000, 300, 300, P, P, P, P, None) == TOO_LARGE
    assert lib.h2x_bn_forward_local(capi.F32, 1, 70000, 300, 300, 300, P, P, P, 300, 0.9, 1e-5, P, P, P, P, P, P,
                                    None) == TOO_LARGE


def test_halo_and_shuffle_rejections():
    lib = capi.load()
    real = capi.i64_array((10, 8, 3, 2))
    # dimension or side out of range, a width whose boundary strip leaves the tensor, unknown op, null tensor
    assert lib.h2x_halo_pack_or_unpack(capi.F32, P, 4, real, 4, 0, 1, P, 1, 0, 0, None) == INVALID
    assert lib.h2x_halo_pack_or_unpack(capi.F32, P, 4, real, 0, 2, 1, P, 1, 0, 0, None) == INVALID
    assert lib.h2x_halo_pack_or_unpack(capi.F32, P, 4, real, 1, 0, 5, P, 1, 0, 0, None) == INVALID
    assert lib.h2x_halo_pack_or_unpack(capi.F32, P, 4, real, 0, 0, 1, P, 0, 0, 9, None) in (INVALID, UNSUPPORTED)
    assert lib.h2x_halo_pack_or_unpack(capi.F32, None, 4, real, 0, 0, 1, P, 1, 0, 0, None) == INVALID
    assert lib.h2x_halo_pack_or_unpack(7, P, 4, real, 0, 0, 1, P, 1, 0, 0, None) == UNSUPPORTED
    assert lib.h2x_halo_pack_or_unpack(capi.F32, P, 9, real, 0, 0, 1, P, 1, 0, 0, None) == INVALID
    # width 0 is a no-op, not an error
    assert lib.h2x_halo_pack_or_unpack(capi.F32, P, 4, real, 0, 0, 0, P, 1, 0, 0, None) == 0
    assert lib.h2x_halo_clear(capi.F32, P, 4, real, 5, 1, None) == INVALID
    # shuffle geometry: element size, limits that decrease or do not end at the local extent
    g = capi.ShuffleGeometry()
    g.num_dims = 2
    limits = (ctypes.c_int32 * 3)(4, 8, 3)
    displs = (ctypes.c_int32 * 2)(0, 12)
    for i, (e, s, p) in enumerate(zip((8, 3), (1, 8), (2, 1))):
        g.local_shape[i], g.strides[i], g.peer_locale_shape[i] = e, s, p
    g.rank_limits, g.displs = limits, displs
    plan = ctypes.c_void_p()
    g.elem_size = 3
    assert lib.h2x_shuffle_plan_create(ctypes.byref(g), ctypes.byref(plan)) == UNSUPPORTED
    g.elem_size = 4
    limits[0], limits[1] = 6, 4
    assert lib.h2x_shuffle_plan_create(ctypes.byref(g), ctypes.byref(plan)) == INVALID
    limits[0], limits[1] = 4, 7
    assert lib.h2x_shuffle_plan_create(ctypes.byref(g), ctypes.byref(plan)) == INVALID
    assert not plan.value


def test_a_valid_call_fails_with_the_runtime_error_of_a_machine_without_a_gpu():
    """Nothing computes on the CPU: what is not rejected goes to the GPU, and without one the HIP
    runtime's error comes back (a positive hipError_t), from every family of entry points."""
    lib = capi.load()
    c = 4
    assert lib.h2x_bn_channel_sums_and_sqsums(capi.F32, 2, c, 8, 8, P, P, P, P, None) > 0
    assert lib.h2x_bn_batch_normalization(capi.F32, 2, c, 8, 8, 8, P, P, P, P, P, P, 1e-5, None) > 0
    assert lib.h2x_softmax_channel_forward(capi.F32, 2, c, 8, P, P, None) > 0
    real = capi.i64_array((10, 8, 3, 2))
    assert lib.h2x_halo_pack_or_unpack(capi.F32, P, 4, real, 0, 0, 1, P, 1, 0, 0, None) > 0
    assert lib.h2x_halo_clear(capi.F32, P, 4, real, 1, 1, None) > 0
    assert "h2x" in lib.h2x_status_string(-1).decode() or lib.h2x_status_string(-1)

"""ctypes binding of ``libh2x.so`` (the C ABI declared in ``include/h2x.h``).

The library is loaded from this package directory.  There is no fallback: if
the shared object is missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_double, c_int, c_int32, c_int64, c_size_t, c_uint32, c_uint64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libh2x.so")

H2X_MAX_DIMS = 6
F32, F64 = 0, 1
LHS, RHS = 0, 1
HALO_ID, HALO_SUM, HALO_MAX, HALO_MIN = 0, 1, 2, 3
TRANSFORM_SCALE, TRANSFORM_COPY, TRANSFORM_SCALE_BIAS, TRANSFORM_SUMS_TO_STATISTICS = 0, 1, 2, 3

ABI_VERSION = 1


class H2XError(RuntimeError):
    pass


class HaloFace(ctypes.Structure):
    """struct h2x_halo_face"""
    _fields_ = [
        ("tensor", c_void_p),
        ("buffer", c_void_p),
        ("real_shape", c_int64 * H2X_MAX_DIMS),
        ("num_dims", c_int32),
        ("dim", c_int32),
        ("side", c_int32),
        ("width", c_int32),
        ("inner", c_int32),
        ("is_pack", c_int32),
        ("op", c_int32),
        ("reserved", c_int32),
    ]


class HaloTransfer(ctypes.Structure):
    """struct h2x_halo_transfer"""
    _fields_ = [
        ("src", c_void_p),
        ("dst", c_void_p),
        ("src_real_shape", c_int64 * H2X_MAX_DIMS),
        ("dst_real_shape", c_int64 * H2X_MAX_DIMS),
        ("num_dims", c_int32),
        ("dim", c_int32),
        ("src_side", c_int32),
        ("width", c_int32),
        ("is_reverse", c_int32),
        ("op", c_int32),
    ]


class TensorGeometry(ctypes.Structure):
    """struct h2x_tensor_geometry"""
    _fields_ = [
        ("num_dims", c_int32),
        ("reserved", c_int32),
        ("local_shape", c_int64 * H2X_MAX_DIMS),
        ("strides", c_int64 * H2X_MAX_DIMS),
    ]


class HaloedGeometry(ctypes.Structure):
    """struct h2x_haloed_geometry"""
    _fields_ = [
        ("num_dims", c_int32),
        ("reserved", c_int32),
        ("local_shape", c_int64 * H2X_MAX_DIMS),
        ("real_shape", c_int64 * H2X_MAX_DIMS),
        ("lower_halo", c_int64 * H2X_MAX_DIMS),
    ]


BN_STAGE_SUMS, BN_STAGE_NORMALIZE, BN_STAGE_BACKPROP1, BN_STAGE_BACKPROP2 = 0, 1, 2, 3
BN_STAGE_FORWARD_LOCAL, BN_STAGE_BACKWARD_LOCAL = 4, 5
BN_AUDIT_MAX_LAUNCHES = 8


class BnAuditTensor(ctypes.Structure):
    """struct h2x_bn_audit_tensor"""
    _fields_ = [("loads", c_uint64), ("stores", c_uint64), ("outside", c_uint64), ("missed", c_uint64),
                ("owned_twice", c_uint64)]


class BnAuditLaunch(ctypes.Structure):
    """struct h2x_bn_audit_launch"""
    _fields_ = [
        ("kernel", c_int32), ("family", c_int32), ("vector_width", c_int32), ("tail", c_int32),
        ("folded", c_int32), ("fused", c_int32), ("grid_x", c_uint32), ("grid_y", c_uint32),
        ("partials_bytes", c_uint64), ("partials_capacity", c_uint64),
        ("num_tensors", c_int32), ("reserved", c_int32),
        ("tensor", BnAuditTensor * 3),
    ]


class BnAuditReport(ctypes.Structure):
    """struct h2x_bn_audit_report"""
    _fields_ = [("num_launches", c_int32), ("reserved", c_int32), ("workspace_bytes", c_uint64),
                ("launch", BnAuditLaunch * BN_AUDIT_MAX_LAUNCHES)]


class ShuffleGeometry(ctypes.Structure):
    """struct h2x_shuffle_geometry"""
    _fields_ = [
        ("num_dims", c_int32),
        ("elem_size", c_int32),
        ("local_shape", c_int64 * H2X_MAX_DIMS),
        ("strides", c_int64 * H2X_MAX_DIMS),
        ("peer_locale_shape", c_int64 * H2X_MAX_DIMS),
        ("rank_limits", POINTER(c_int32)),
        ("displs", POINTER(c_int32)),
    ]


class CopyAuditRegion(ctypes.Structure):
    """struct h2x_copy_audit_region"""
    _fields_ = [
        ("base", c_uint64),
        ("bytes", c_uint64),
        ("loads", POINTER(ctypes.c_uint8)),
        ("stores", POINTER(ctypes.c_uint8)),
    ]


class CopyAuditReport(ctypes.Structure):
    """struct h2x_copy_audit_report"""
    _fields_ = [
        ("launches", c_uint64),
        ("workgroups", c_uint64),
        ("outside_loads", c_uint64),
        ("outside_stores", c_uint64),
        ("misaligned", c_uint64),
    ]


# name -> (restype, argtypes); every symbol include/h2x.h declares.
SIGNATURES = {
    "h2x_abi_version": (c_int, []),
    "h2x_status_string": (ctypes.c_char_p, [c_int]),
    "h2x_bn_workspace_bytes": (c_size_t, [c_int]),
    "h2x_bn_channel_sums_and_sqsums": (c_int, [c_int, c_int, c_int, c_size_t, c_size_t, c_void_p,
                                               c_void_p, c_void_p, c_void_p, c_void_p]),
    "h2x_bn_channel_sums_and_sqsums_static": (c_int, [c_int, c_int, c_int, c_size_t, c_size_t, c_void_p,
                                                      c_void_p, c_void_p, c_void_p]),
    "h2x_bn_static_max_channels": (c_size_t, []),
    "h2x_bn_sums_to_statistics": (c_int, [c_int, c_int, c_size_t, c_double, c_void_p, c_void_p,
                                          c_void_p, c_void_p, c_void_p]),
    "h2x_bn_batch_normalization": (c_int, [c_int, c_int, c_int, c_size_t, c_size_t, c_size_t,
                                           c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                           c_void_p, c_double, c_void_p]),
    "h2x_bn_backprop1": (c_int, [c_int, c_int, c_int, c_size_t, c_size_t, c_size_t, c_void_p,
                                 c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_void_p, c_void_p, c_double, c_void_p, c_void_p]),
    "h2x_bn_backprop2": (c_int, [c_int, c_int, c_int, c_size_t, c_size_t, c_size_t, c_size_t,
                                 c_size_t, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_void_p, c_void_p, c_void_p, c_double, c_void_p]),
    "h2x_bn_forward_local": (c_int, [c_int, c_int, c_int, c_size_t, c_size_t, c_size_t, c_void_p, c_void_p,
                                     c_void_p, c_size_t, c_double, c_double, c_void_p, c_void_p, c_void_p,
                                     c_void_p, c_void_p, c_void_p, c_void_p]),
    "h2x_bn_backward_local": (c_int, [c_int, c_int, c_int, c_size_t, c_size_t, c_size_t, c_size_t, c_size_t,
                                      c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_void_p, c_void_p, c_void_p, c_double, c_void_p, c_void_p]),
    "h2x_bn_channel_sums_and_sqsums_strided": (c_int, [c_int, c_int, POINTER(TensorGeometry), c_void_p,
                                                       c_void_p, c_void_p, c_void_p, c_void_p]),
    "h2x_bn_batch_normalization_strided": (c_int, [c_int, c_int, POINTER(TensorGeometry),
                                                   POINTER(TensorGeometry), c_void_p, c_void_p,
                                                   c_void_p, c_void_p, c_void_p, c_void_p, c_double,
                                                   c_void_p]),
    "h2x_bn_backprop1_strided": (c_int, [c_int, c_int, POINTER(TensorGeometry), POINTER(TensorGeometry),
                                         c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                         c_void_p, c_void_p, c_void_p, c_double, c_void_p, c_void_p]),
    "h2x_bn_backprop2_strided": (c_int, [c_int, c_int, c_size_t, POINTER(TensorGeometry),
                                         POINTER(TensorGeometry), POINTER(TensorGeometry), c_void_p,
                                         c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                         c_void_p, c_double, c_void_p]),
    "h2x_bn_forward_local_strided": (c_int, [c_int, c_int, POINTER(TensorGeometry), POINTER(TensorGeometry), c_void_p,
                                             c_void_p, c_void_p, c_size_t, c_double, c_double, c_void_p, c_void_p,
                                             c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "h2x_bn_backward_local_strided": (c_int, [c_int, c_int, c_size_t, POINTER(TensorGeometry), POINTER(TensorGeometry),
                                              POINTER(TensorGeometry), c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                              c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_double, c_void_p,
                                              c_void_p]),
    "h2x_bn_batch_normalization_clearing": (c_int, [c_int, POINTER(HaloedGeometry), c_void_p, c_void_p, c_void_p,
                                                    c_void_p, c_void_p, c_void_p, c_double, c_void_p]),
    "h2x_bn_backprop2_clearing": (c_int, [c_int, c_size_t, POINTER(HaloedGeometry), c_void_p, c_void_p, c_void_p,
                                          c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_double, c_void_p]),
    "h2x_bn_audit": (c_int, [c_int, c_int, c_int, POINTER(POINTER(TensorGeometry)), POINTER(c_uint64),
                             POINTER(BnAuditReport)]),
    "h2x_copy_audit_begin": (c_int, []),
    "h2x_copy_audit_add_region": (c_int, [POINTER(CopyAuditRegion)]),
    "h2x_copy_audit_end": (c_int, [POINTER(CopyAuditReport)]),
    "h2x_bn_audit_clearing": (c_int, [c_int, c_int, POINTER(HaloedGeometry), POINTER(c_uint64),
                                      POINTER(BnAuditReport)]),
    "h2x_tensor_transform": (c_int, [c_int, c_int, c_int, POINTER(POINTER(TensorGeometry)), POINTER(c_void_p),
                                     POINTER(c_double), c_void_p]),
    "h2x_tensor_reduce_sum_workspace_bytes": (c_size_t, [POINTER(TensorGeometry), POINTER(TensorGeometry)]),
    "h2x_tensor_reduce_sum": (c_int, [c_int, POINTER(TensorGeometry), c_void_p, POINTER(TensorGeometry), c_void_p,
                                      c_int, c_void_p, c_void_p]),
    "h2x_softmax_channel_forward": (c_int, [c_int, c_int, c_int, c_size_t, c_void_p, c_void_p,
                                            c_void_p]),
    "h2x_softmax_channel_backward": (c_int, [c_int, c_int, c_int, c_size_t, c_void_p, c_void_p,
                                             c_void_p, c_void_p]),
    "h2x_softmax_instance_workspace_bytes": (c_size_t, [c_int]),
    "h2x_softmax_instance_max": (c_int, [c_int, c_int, c_size_t, c_void_p, c_void_p, c_void_p, c_void_p]),
    "h2x_softmax_instance_exp": (c_int, [c_int, c_int, c_size_t, c_void_p, c_void_p, c_void_p, c_void_p,
                                         c_void_p, c_void_p]),
    "h2x_softmax_instance_normalize": (c_int, [c_int, c_int, c_size_t, c_void_p, c_void_p, c_void_p]),
    "h2x_softmax_instance_forward_local": (c_int, [c_int, c_int, c_size_t, c_void_p, c_void_p, c_void_p, c_void_p,
                                                   c_void_p, c_void_p]),
    "h2x_softmax_instance_dot": (c_int, [c_int, c_int, c_size_t, c_void_p, c_void_p, c_void_p, c_void_p,
                                         c_void_p]),
    "h2x_softmax_instance_gradient": (c_int, [c_int, c_int, c_size_t, c_void_p, c_void_p, c_void_p,
                                              c_void_p, c_void_p]),
    "h2x_halo_size": (c_size_t, [c_int, POINTER(c_int64), c_int, c_int]),
    "h2x_halo_pack_or_unpack": (c_int, [c_int, c_void_p, c_int, POINTER(c_int64), c_int, c_int,
                                        c_int, c_void_p, c_int, c_int, c_int, c_void_p]),
    "h2x_halo_pack_or_unpack_batched": (c_int, [c_int, POINTER(HaloFace), c_int, c_void_p]),
    "h2x_halo_clear": (c_int, [c_int, c_void_p, c_int, POINTER(c_int64), c_int, c_int, c_void_p]),
    "h2x_halo_clear_batched": (c_int, [c_int, POINTER(HaloFace), c_int, c_void_p]),
    "h2x_halo_exchange_fused": (c_int, [c_int, POINTER(HaloTransfer), c_int, c_void_p]),
    "h2x_shuffle_plan_create": (c_int, [POINTER(ShuffleGeometry), POINTER(c_void_p)]),
    "h2x_shuffle_plan_destroy": (c_int, [c_void_p]),
    "h2x_shuffle_pack": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p]),
    "h2x_shuffle_unpack": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p]),
    "h2x_shuffle_pack_batched": (c_int, [POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p),
                                         c_int, c_void_p]),
    "h2x_shuffle_unpack_batched": (c_int, [POINTER(c_void_p), POINTER(c_void_p),
                                           POINTER(c_void_p), c_int, c_void_p]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Loads libh2x.so and checks its ABI version.  Raises if it is absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise H2XError(
            f"{LIB_PATH} is missing: build it with `make -C dihydrogen_amd/csrc` "
            "(or __graft_entry__.build()); there is no fallback path")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.h2x_abi_version() != ABI_VERSION:
        raise H2XError(f"libh2x.so has ABI {lib.h2x_abi_version()}, binding expects {ABI_VERSION}")
    _lib = lib
    return lib


def check(status: int, what: str = "") -> None:
    if status != 0:
        msg = load().h2x_status_string(status).decode()
        raise H2XError(f"{what or 'h2x call'} failed: {msg} ({status})")


def i64_array(values):
    arr = (c_int64 * H2X_MAX_DIMS)()
    for i, v in enumerate(values):
        arr[i] = int(v)
    return arr

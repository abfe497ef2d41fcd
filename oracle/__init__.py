"""CPU oracle: numpy front-end of ``libh2x_oracle.so``.

TEST INFRASTRUCTURE ONLY.  May be imported by ``tests/``, by
``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py``;
the product package never imports it.

Every function takes and returns numpy arrays laid out as the reference lays
out its local tensors: C-contiguous ``[N][C][spatial_real]`` (numpy shape
order is outermost first, i.e. the reverse of the reference's innermost-first
``Shape``).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libh2x_oracle.so")
_lib = None

_c_i64p = ctypes.POINTER(ctypes.c_int64)
_c_i32p = ctypes.POINTER(ctypes.c_int32)


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (oracle/Makefile)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _sfx(dtype) -> str:
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32"
    if dtype == np.float64:
        return "f64"
    raise TypeError(f"oracle supports float32/float64, got {dtype}")


def _ptr(a: np.ndarray):
    return ctypes.c_void_p(a.ctypes.data)


def _i64(seq):
    return (ctypes.c_int64 * len(seq))(*[int(v) for v in seq])


def _scalar(dtype, v):
    return ctypes.c_float(v) if np.dtype(dtype) == np.float32 else ctypes.c_double(v)


def _ncs(x: np.ndarray):
    """(N, C, spatial_real) of a C-contiguous [N][C][...] array."""
    assert x.flags.c_contiguous and x.ndim >= 3
    n, c = x.shape[0], x.shape[1]
    return n, c, int(np.prod(x.shape[2:], dtype=np.int64))


# --------------------------------------------------------------------------
# Batch normalisation
# --------------------------------------------------------------------------

def bn_channel_sums_and_sqsums(x: np.ndarray, spatial: int | None = None):
    n, c, real = _ncs(x)
    spatial = real if spatial is None else spatial
    sums = np.empty(c, x.dtype)
    sqsums = np.empty(c, x.dtype)
    fn = getattr(lib(), "orc_bn_channel_sums_and_sqsums_" + _sfx(x.dtype))
    fn(ctypes.c_int(n), ctypes.c_int(c), ctypes.c_size_t(spatial), ctypes.c_size_t(real),
       _ptr(x), _ptr(sums), _ptr(sqsums))
    return sums, sqsums


def bn_sums_to_statistics(num_per_sum: int, decay: float, mean, var, running_mean, running_var):
    """In place on all four arrays, like the reference."""
    c = mean.shape[0]
    fn = getattr(lib(), "orc_bn_sums_to_statistics_" + _sfx(mean.dtype))
    fn(ctypes.c_int(c), ctypes.c_size_t(num_per_sum), _scalar(mean.dtype, decay),
       _ptr(mean), _ptr(var), _ptr(running_mean), _ptr(running_var))


def bn_batch_normalization(x, mean, var, scale, bias, eps: float, spatial: int | None = None):
    n, c, real = _ncs(x)
    spatial = real if spatial is None else spatial
    y = np.zeros_like(x)
    fn = getattr(lib(), "orc_bn_batch_normalization_" + _sfx(x.dtype))
    fn(ctypes.c_int(n), ctypes.c_int(c), ctypes.c_size_t(spatial), ctypes.c_size_t(real),
       ctypes.c_size_t(real), _ptr(x), _ptr(mean), _ptr(var), _ptr(scale), _ptr(bias), _ptr(y),
       _scalar(x.dtype, eps))
    return y


def bn_backprop1(x, dy, mean, var, scale, eps: float, spatial: int | None = None):
    n, c, real = _ncs(x)
    spatial = real if spatial is None else spatial
    outs = [np.empty(c, x.dtype) for _ in range(4)]
    fn = getattr(lib(), "orc_bn_backprop1_" + _sfx(x.dtype))
    fn(ctypes.c_int(n), ctypes.c_int(c), ctypes.c_size_t(spatial), ctypes.c_size_t(real),
       ctypes.c_size_t(real), _ptr(x), _ptr(dy), _ptr(mean), _ptr(var), _ptr(scale),
       _ptr(outs[0]), _ptr(outs[1]), _ptr(outs[2]), _ptr(outs[3]), _scalar(x.dtype, eps))
    return tuple(outs)  # dscale, dbias, dmean, dvar


def bn_backprop2(x, dy, mean, var, scale, dmean, dvar, eps: float, num_per_sum: int,
                 spatial: int | None = None, out: np.ndarray | None = None):
    n, c, real = _ncs(x)
    spatial = real if spatial is None else spatial
    dx = np.zeros_like(x) if out is None else out
    fn = getattr(lib(), "orc_bn_backprop2_" + _sfx(x.dtype))
    fn(ctypes.c_int(n), ctypes.c_int(c), ctypes.c_size_t(spatial), ctypes.c_size_t(real),
       ctypes.c_size_t(real), ctypes.c_size_t(real), ctypes.c_size_t(num_per_sum), _ptr(x),
       _ptr(dy), _ptr(mean), _ptr(var), _ptr(scale), _ptr(dmean), _ptr(dvar), _ptr(dx),
       _scalar(x.dtype, eps))
    return dx


def bn_forward(x, scale, bias, running_mean, running_var, eps=1e-5, decay=0.9):
    """BatchNormalization::forward with local statistics on one rank
    (legacy/include/distconv/dnn_backend/batchnorm.hpp:293-333): returns
    y, mean, var; the running statistics are updated in place."""
    n, c, real = _ncs(x)
    mean, var = bn_channel_sums_and_sqsums(x)
    bn_sums_to_statistics(n * real, decay, mean, var, running_mean, running_var)
    y = bn_batch_normalization(x, mean, var, scale, bias, eps)
    return y, mean, var


def bn_backward(x, dy, mean, var, scale, eps=1e-5):
    """BatchNormalization::backward on one rank (batchnorm.hpp:432-464):
    returns dx, dscale, dbias, dmean, dvar."""
    n, c, real = _ncs(x)
    dscale, dbias, dmean, dvar = bn_backprop1(x, dy, mean, var, scale, eps)
    dx = bn_backprop2(x, dy, mean, var, scale, dmean, dvar, eps, n * real)
    return dx, dscale, dbias, dmean, dvar


# -- strided variants: `x` is the flat real buffer starting at the first interior
#    element, shape/strides innermost first (channel = nd-2, sample = nd-1)

def _geom(shape, *strides_list):
    nd = len(shape)
    return [ctypes.c_int(nd), _i64(shape)] + [_i64(st) for st in strides_list]


def bn_channel_sums_and_sqsums_strided(x, shape, strides):
    c = int(shape[-2])
    sums, sqsums = np.empty(c, x.dtype), np.empty(c, x.dtype)
    fn = getattr(lib(), "orc_bn_channel_sums_and_sqsums_strided_" + _sfx(x.dtype))
    fn(*_geom(shape, strides), _ptr(x), _ptr(sums), _ptr(sqsums))
    return sums, sqsums


def bn_batch_normalization_strided(x, shape, x_strides, y, y_strides, mean, var, scale, bias, eps):
    fn = getattr(lib(), "orc_bn_batch_normalization_strided_" + _sfx(x.dtype))
    fn(*_geom(shape, x_strides, y_strides), _ptr(x), _ptr(mean), _ptr(var), _ptr(scale), _ptr(bias),
       _ptr(y), _scalar(x.dtype, eps))


def bn_backprop1_strided(x, shape, x_strides, dy, dy_strides, mean, var, scale, eps):
    c = int(shape[-2])
    outs = [np.empty(c, x.dtype) for _ in range(4)]
    fn = getattr(lib(), "orc_bn_backprop1_strided_" + _sfx(x.dtype))
    fn(*_geom(shape, x_strides, dy_strides), _ptr(x), _ptr(dy), _ptr(mean), _ptr(var), _ptr(scale),
       _ptr(outs[0]), _ptr(outs[1]), _ptr(outs[2]), _ptr(outs[3]), _scalar(x.dtype, eps))
    return tuple(outs)


def bn_backprop2_strided(x, shape, x_strides, dy, dy_strides, dx, dx_strides, num_per_sum, mean, var,
                         scale, dmean, dvar, eps):
    fn = getattr(lib(), "orc_bn_backprop2_strided_" + _sfx(x.dtype))
    fn(*_geom(shape, x_strides, dy_strides, dx_strides), ctypes.c_size_t(num_per_sum), _ptr(x),
       _ptr(dy), _ptr(mean), _ptr(var), _ptr(scale), _ptr(dmean), _ptr(dvar), _ptr(dx),
       _scalar(x.dtype, eps))


# --------------------------------------------------------------------------
# Channel softmax
# --------------------------------------------------------------------------

def softmax_channel_forward(x: np.ndarray) -> np.ndarray:
    n, c, s = _ncs(x)
    y = np.empty_like(x)
    fn = getattr(lib(), "orc_softmax_channel_forward_" + _sfx(x.dtype))
    fn(ctypes.c_int(n), ctypes.c_int(c), ctypes.c_size_t(s), _ptr(x), _ptr(y))
    return y


def softmax_channel_backward(y: np.ndarray, dy: np.ndarray) -> np.ndarray:
    n, c, s = _ncs(y)
    dx = np.empty_like(y)
    fn = getattr(lib(), "orc_softmax_channel_backward_" + _sfx(y.dtype))
    fn(ctypes.c_int(n), ctypes.c_int(c), ctypes.c_size_t(s), _ptr(y), _ptr(dy), _ptr(dx))
    return dx


def softmax_instance_forward(x: np.ndarray, allreduce=None):
    """Softmax::forward in instance mode (legacy/src/dnn_backend/softmax.cu:705-747):
    returns y.  `allreduce(values, is_max)` stands where the reference all-reduces
    the per-sample scalars over the ranks that share a sample."""
    n = x.shape[0]
    size = x.size // n if n else 0
    sfx = _sfx(x.dtype)
    mx, ex, y = np.empty(n, x.dtype), np.empty(n, x.dtype), np.empty_like(x)
    getattr(lib(), "orc_softmax_instance_max_" + sfx)(ctypes.c_int(n), ctypes.c_size_t(size), _ptr(x), _ptr(mx))
    if allreduce:
        allreduce(mx, True)
    getattr(lib(), "orc_softmax_instance_exp_" + sfx)(ctypes.c_int(n), ctypes.c_size_t(size), _ptr(x), _ptr(mx),
                                                      _ptr(y), _ptr(ex))
    if allreduce:
        allreduce(ex, False)
    getattr(lib(), "orc_softmax_instance_normalize_" + sfx)(ctypes.c_int(n), ctypes.c_size_t(size), _ptr(ex), _ptr(y))
    return y


def softmax_instance_backward(y: np.ndarray, dy: np.ndarray, allreduce=None):
    """Softmax::backward in instance mode (softmax.cu:749-784)."""
    n = y.shape[0]
    size = y.size // n if n else 0
    sfx = _sfx(y.dtype)
    dp, dx = np.empty(n, y.dtype), np.empty_like(y)
    getattr(lib(), "orc_softmax_instance_dot_" + sfx)(ctypes.c_int(n), ctypes.c_size_t(size), _ptr(y), _ptr(dy), _ptr(dp))
    if allreduce:
        allreduce(dp, False)
    getattr(lib(), "orc_softmax_instance_gradient_" + sfx)(ctypes.c_int(n), ctypes.c_size_t(size), _ptr(y), _ptr(dy),
                                                           _ptr(dp), _ptr(dx))
    return dx


# --------------------------------------------------------------------------
# Halo pack / unpack
# --------------------------------------------------------------------------

LHS, RHS = 0, 1
OP_ID, OP_SUM, OP_MAX, OP_MIN = 0, 1, 2, 3


def halo_size(real_shape, dim: int, width: int) -> int:
    """real_shape is innermost first, as in the reference."""
    s = 1
    for i, e in enumerate(real_shape):
        s *= width if i == dim else int(e)
    return s


def halo_pack_or_unpack(tensor: np.ndarray, dim: int, side: int, width: int, buf: np.ndarray,
                        is_pack: bool, is_reverse: bool = False, op: int = OP_ID) -> None:
    """``tensor`` is the real (haloed) local tensor, numpy shape outermost first;
    ``dim`` counts innermost first.  Follows pack_or_unpack,
    legacy/include/distconv/tensor/halo_packing_cuda.hpp:85-167."""
    assert tensor.flags.c_contiguous
    if width == 0:
        return
    shape = (ctypes.c_int64 * tensor.ndim)(*tensor.shape[::-1])
    inner = (is_pack and not is_reverse) or ((not is_pack) and is_reverse)
    extent = tensor.shape[::-1][dim]
    if (2 if inner else 1) * width > extent:
        raise ValueError("halo strip does not fit the tensor")  # TraverseHalo asserts, halo_cuda.hpp:911-916
    assert buf.dtype == tensor.dtype and buf.size >= halo_size(tensor.shape[::-1], dim, width)
    fn = getattr(lib(), "orc_halo_pack_or_unpack_" + _sfx(tensor.dtype))
    fn(_ptr(tensor), ctypes.c_int(tensor.ndim), shape, ctypes.c_int(dim), ctypes.c_int(side),
       ctypes.c_int(int(inner)), ctypes.c_int(width), _ptr(buf), ctypes.c_int(int(is_pack)),
       ctypes.c_int(op))


# --------------------------------------------------------------------------
# Shuffler pack / unpack
# --------------------------------------------------------------------------

def _i32arr(a):
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a, a.ctypes.data_as(_c_i32p)


def shuffle_pack_or_unpack(tensor: np.ndarray, local_shape, strides, peer_locale_shape,
                           rank_limits, buf: np.ndarray, displs, is_pack: bool,
                           parallel: bool = False) -> None:
    """local_shape / strides / peer_locale_shape innermost first.  ``tensor``
    is a flat view starting at the first interior element."""
    nd = len(local_shape)
    rl, rlp = _i32arr(rank_limits)
    dp, dpp = _i32arr(displs)
    lib().orc_shuffle_pack_or_unpack(
        _ptr(tensor), ctypes.c_int(nd), ctypes.c_int(tensor.dtype.itemsize), _i64(local_shape),
        _i64(strides), _i64(peer_locale_shape), rlp, _ptr(buf), dpp, ctypes.c_int(int(is_pack)),
        ctypes.c_int(int(parallel)))


def shuffle_pack_rows4(tensor: np.ndarray, local_shape, peer_locale_shape, rank_limits,
                       buf: np.ndarray, displs) -> None:
    assert len(local_shape) == 4
    rl, rlp = _i32arr(rank_limits)
    dp, dpp = _i32arr(displs)
    lib().orc_shuffle_pack_rows4(
        _ptr(tensor), ctypes.c_int(tensor.dtype.itemsize), _i64(local_shape),
        _i64(peer_locale_shape), rlp, _ptr(buf), dpp)


# --------------------------------------------------------------------------
# Elementwise transforms and sums over dimensions
# (legacy/include/distconv/tensor/algorithms/transform_cuda.hpp:359-693,
#  reduce_sum_cuda.hpp:56-113,388-439)
# --------------------------------------------------------------------------

TRANSFORM_SCALE, TRANSFORM_COPY, TRANSFORM_SCALE_BIAS, TRANSFORM_SUMS_TO_STATISTICS = 0, 1, 2, 3


def tensor_transform(op: int, tensors, params=()):
    """tensor::Transform over the interiors of 1-4 tensors (numpy views of equal
    shape, e.g. interiors of haloed arrays), in place, for the named functors:
    ScaleFunctor (legacy/src/tensor/tensor_mpi_cuda.cu:86-98), copy,
    CastScaleBias with equal types (tensor_mpi_cuda.cu:113-135) and the
    sums-to-statistics functor (legacy/src/dnn_backend/batchnorm.cu:297-346).
    Arithmetic is done in the tensors' own type, one rounding per operation."""
    t = list(tensors)
    dt = t[0].dtype.type
    if op == TRANSFORM_SCALE:
        t[0][...] = t[0] * dt(params[0])
    elif op == TRANSFORM_COPY:
        t[1][...] = t[0]
    elif op == TRANSFORM_SCALE_BIAS:
        t[1][...] = dt(params[0]) * t[0] + dt(params[1])
    elif op == TRANSFORM_SUMS_TO_STATISTICS:
        mean, var, rmean, rvar = t
        shape = mean.shape
        m, v = np.ascontiguousarray(mean).ravel(), np.ascontiguousarray(var).ravel()
        rm, rv = np.ascontiguousarray(rmean).ravel(), np.ascontiguousarray(rvar).ravel()
        bn_sums_to_statistics(int(params[0]), float(params[1]), m, v, rm, rv)
        mean[...], var[...] = m.reshape(shape), v.reshape(shape)
        rmean[...], rvar[...] = rm.reshape(shape), rv.reshape(shape)
    else:
        raise ValueError(op)


def tensor_reduce_sum(src: np.ndarray, dst: np.ndarray, square: bool = False) -> None:
    """tensor::ReduceSum / TransformReduceSum: ``dst += sum(src)`` over every
    axis where dst has extent 1 (reduce_sum_cuda.hpp:69-113: each element is
    added onto its destination cell; the destination is not cleared).  The sum
    is taken in float64 and rounded once, the arithmetic the device path
    uses; the reference accumulates floats with atomics in arrival order."""
    assert src.ndim == dst.ndim
    axes = tuple(i for i in range(src.ndim) if dst.shape[i] == 1 and src.shape[i] != 1)
    for i in range(src.ndim):
        assert dst.shape[i] in (1, src.shape[i])
    x = src.astype(np.float64)
    if square:
        x = x * x
    total = x.sum(axis=axes, keepdims=True) if axes else x
    dst[...] = dst + total.astype(dst.dtype)


def shuffle_rows(tensor: np.ndarray, local_shape, strides, peer_locale_shape, rank_limits,
                 buf: np.ndarray, displs, is_pack: bool) -> None:
    """Row-copy pack / unpack of any rank (the reference's OpenMP memcpy paths,
    legacy/include/distconv/tensor/shuffle_mpi.hpp:708-849,874-947); plain
    rank limits only; requires strides[0] == 1."""
    nd = len(local_shape)
    assert strides[0] == 1
    rl, rlp = _i32arr(rank_limits)
    dp, dpp = _i32arr(displs)
    lib().orc_shuffle_rows(
        _ptr(tensor), ctypes.c_int(nd), ctypes.c_int(tensor.dtype.itemsize), _i64(local_shape),
        _i64(strides), _i64(peer_locale_shape), rlp, _ptr(buf), dpp, ctypes.c_int(int(is_pack)))

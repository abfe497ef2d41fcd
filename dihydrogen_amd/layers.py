"""Python mirror of the DistConv layer API for the non-convolution hot path,
on top of the C ABI (``include/h2x.h``).  Method names, argument order and
return values follow the reference classes; MPI ranks are replaced by virtual
ranks whose local tensors live on one GPU, and every "transfer" between ranks
is pointer wiring between device buffers.
"""
from __future__ import annotations

import ctypes
from enum import Enum
from typing import Callable, List, Optional, Sequence

import torch

from . import capi
from .tensor import Tensor, _prod


def _device_buffer(count: int, dtype, device="cuda", zero: bool = False) -> torch.Tensor:
    """Every device buffer the layers own (workspaces, receive buffers, the shuffler's arena)
    comes from here, so that a test can put guard zones around them."""
    return (torch.zeros if zero else torch.empty)(count, dtype=dtype, device=device)



_has_gpu: Optional[bool] = None


def _stream_handle(stream: Optional[torch.cuda.Stream]) -> ctypes.c_void_p:
    global _has_gpu
    if stream is None:
        if _has_gpu is None:
            _has_gpu = torch.cuda.is_available()  # asked once: the answer does not change
        if not _has_gpu:
            # no GPU: the null stream; every launch then fails with HIP's own error.  (Launch
            # audits, which play the kernels' indexing on the CPU, ignore the stream.)
            return ctypes.c_void_p(0)
        stream = torch.cuda.current_stream()
    return ctypes.c_void_p(stream.cuda_stream)


def _ptr(t) -> ctypes.c_void_p:
    if t is None:
        return ctypes.c_void_p(0)
    if isinstance(t, torch.Tensor):
        return ctypes.c_void_p(t.data_ptr())
    return ctypes.c_void_p(int(t))


def _is_dense(t: Tensor) -> bool:
    """No halo on the inner spatial dimensions: the layout the dense entry points
    take (legacy/src/dnn_backend/batchnorm.cu:210-219)."""
    nd = t.get_num_dims()
    return all(t.overlap[d] == 0 for d in range(nd - 3))


def _channel_geometry(t: Tensor):
    """(num_samples, num_channels, spatial, spatial_real) of a dense local tensor."""
    nd = t.get_num_dims()
    if t.overlap[nd - 2] != 0 or t.overlap[nd - 1] != 0:
        raise NotImplementedError("halo on the channel or sample dimension is not supported")
    n, c = t.local_shape[nd - 1], t.local_shape[nd - 2]
    return n, c, _prod(t.local_shape[: nd - 2]), _prod(t.local_real_shape[: nd - 2])


def _tensor_geometry(t: Tensor, num_samples: int) -> capi.TensorGeometry:
    """h2x_tensor_geometry of a local tensor (local shape + get_strides())."""
    nd = t.get_num_dims()
    if t.overlap[nd - 2] != 0 or t.overlap[nd - 1] != 0:
        raise NotImplementedError("halo on the channel or sample dimension is not supported")
    g = capi.TensorGeometry()
    g.num_dims = nd
    strides = t.get_strides()
    for i in range(nd):
        g.local_shape[i] = t.local_shape[i]
        g.strides[i] = strides[i]
    g.local_shape[nd - 1] = num_samples
    return g


def _haloed_geometry(t: Tensor) -> capi.HaloedGeometry:
    """h2x_haloed_geometry of a local tensor: local and real extents, halo widths."""
    g = capi.HaloedGeometry()
    g.num_dims = t.get_num_dims()
    for i in range(g.num_dims):
        g.local_shape[i] = t.local_shape[i]
        g.real_shape[i] = t.local_real_shape[i]
        g.lower_halo[i] = t.overlap[i]
    return g


def _share_a_haloed_geometry(*tensors: Tensor) -> bool:
    """Tensors with a halo on a spatial dimension whose local parts lie in memory alike."""
    t0 = tensors[0]
    nd = t0.get_num_dims()
    return (any(t0.overlap[: nd - 2]) and t0.overlap[nd - 2] == 0 and t0.overlap[nd - 1] == 0
            and all(t.local_shape == t0.local_shape and t.local_real_shape == t0.local_real_shape
                    and t.overlap == t0.overlap and t.h2x_dtype == t0.h2x_dtype for t in tensors))


class BatchNormalization:
    """BatchNormalization<Backend, DataType>
    (legacy/include/distconv/dnn_backend/batchnorm.hpp:100-581).

    ``allreduce``, if given, is called as ``allreduce(list_of_per_channel_tensors)``
    where the reference sums over ranks (batchnorm.hpp:185-214,360-400); with the
    default ``None`` the layer is a single rank and the step is the identity.
    """

    def __init__(self, num_dims: int, decay: float, epsilon: float, global_stats: bool = False,
                 allreduce: Optional[Callable[[List[torch.Tensor]], None]] = None,
                 stream: Optional[torch.cuda.Stream] = None, fuse_local: bool = True,
                 clear_output_halo: bool = False):
        if num_dims not in (4, 5):
            raise ValueError("4-D (NCHW) or 5-D (NCDHW) tensors only")  # batchnorm.cu:259-270
        self.num_dims, self.decay, self.epsilon = num_dims, float(decay), float(epsilon)
        self.global_stats, self.allreduce, self.stream = global_stats, allreduce, stream
        # forward()/backward() of a rank that all-reduces nothing between its two
        # stages run as two launches each (h2x_bn_forward_local / _backward_local);
        # the staged methods always use the staged entry points
        self.fuse_local = fuse_local
        # Haloed tensors of one geometry: normalise and the input gradient also clear
        # the halo of their output (what Convolution::forward does to its input before
        # every exchange, convolution.hpp:400-411), in one pass over the real tensors
        # (h2x_bn_batch_normalization_clearing / h2x_bn_backprop2_clearing).  Off by
        # default: the reference's kernels leave halo cells alone.
        self.clear_output_halo = clear_output_halo
        self.num_current_samples = 0
        self._lib = capi.load()
        self._workspace: Optional[torch.Tensor] = None
        self._workspace_channels = -1

    # batchnorm.hpp:467-475
    def set_num_samples(self, n: int) -> None:
        self.num_current_samples = int(n)

    def _ws(self, num_channels: int) -> torch.Tensor:
        if self._workspace is None or self._workspace_channels != num_channels:
            nbytes = self._lib.h2x_bn_workspace_bytes(num_channels)
            self._workspace = _device_buffer(nbytes, torch.uint8)
            self._workspace_channels = num_channels
        return self._workspace

    def _num_per_sum(self, t: Tensor) -> int:
        """Elements per channel of the global (global_stats) or local shape
        (batchnorm.hpp:232-236,414-418)."""
        nd = t.get_num_dims()
        shape = t.shape if self.global_stats else t.local_shape
        return _prod(shape) // shape[nd - 2] if shape[nd - 2] else 0

    # ---- forward -----------------------------------------------------------
    def forward_stage1(self, input: Tensor, mean: torch.Tensor, var: torch.Tensor,
                       is_training: bool = True) -> int:
        self.set_num_samples(input.local_shape[-1])
        if not is_training:
            return 0
        n, c, s, sr = _channel_geometry(input)
        active = input.is_split_root() and input.get_local_size() > 0
        ns = self.num_current_samples if active else 0
        if _is_dense(input):
            capi.check(self._lib.h2x_bn_channel_sums_and_sqsums(
                input.h2x_dtype, ns, c, s, sr, _ptr(input.get_base_ptr()), _ptr(mean), _ptr(var),
                _ptr(self._ws(c)), _stream_handle(self.stream)), "channel_sums_and_sqsums")
        else:  # halo on an inner spatial dimension: the generic path of batchnorm.cu:232-248
            g = _tensor_geometry(input, ns)
            capi.check(self._lib.h2x_bn_channel_sums_and_sqsums_strided(
                input.h2x_dtype, ns, ctypes.byref(g), _ptr(input.get_base_ptr()), _ptr(mean),
                _ptr(var), _ptr(self._ws(c)), _stream_handle(self.stream)),
                "channel_sums_and_sqsums (strided)")
        return 0

    def forward_allreduce(self, mean: torch.Tensor, var: torch.Tensor, is_training: bool = True) -> int:
        if is_training and self.global_stats and self.allreduce is not None:
            self.allreduce([mean, var])
        return 0

    def sums_to_statistics(self, num_per_sum: int, mean, var, running_mean, running_var,
                           dtype: int = capi.F32) -> None:
        """batchnorm.hpp:494-503."""
        capi.check(self._lib.h2x_bn_sums_to_statistics(
            dtype, mean.numel(), num_per_sum, self.decay, _ptr(mean), _ptr(var), _ptr(running_mean),
            _ptr(running_var), _stream_handle(self.stream)), "sums_to_statistics")

    def batch_normalization(self, input: Tensor, mean, var, scale, bias, output: Tensor) -> None:
        """batchnorm.hpp:505-517."""
        n, c, s, sr = _channel_geometry(input)
        _, _, so, sro = _channel_geometry(output)
        ns = self.num_current_samples
        if self.clear_output_halo and ns == n and _share_a_haloed_geometry(input, output):
            g = _haloed_geometry(output)
            capi.check(self._lib.h2x_bn_batch_normalization_clearing(
                input.h2x_dtype, ctypes.byref(g), _ptr(input.get_buffer()), _ptr(mean), _ptr(var), _ptr(scale),
                _ptr(bias), _ptr(output.get_buffer()), self.epsilon, _stream_handle(self.stream)),
                "batch_normalization (clearing)")
        elif _is_dense(input) and _is_dense(output):
            capi.check(self._lib.h2x_bn_batch_normalization(
                input.h2x_dtype, ns, c, s, sr, sro, _ptr(input.get_base_ptr()), _ptr(mean), _ptr(var),
                _ptr(scale), _ptr(bias), _ptr(output.get_base_ptr()), self.epsilon,
                _stream_handle(self.stream)), "batch_normalization")
        else:
            gx, gy = _tensor_geometry(input, ns), _tensor_geometry(output, ns)
            capi.check(self._lib.h2x_bn_batch_normalization_strided(
                input.h2x_dtype, ns, ctypes.byref(gx), ctypes.byref(gy), _ptr(input.get_base_ptr()),
                _ptr(mean), _ptr(var), _ptr(scale), _ptr(bias), _ptr(output.get_base_ptr()),
                self.epsilon, _stream_handle(self.stream)), "batch_normalization (strided)")

    def forward_stage2(self, input: Tensor, mean, var, running_mean, running_var, scale, bias,
                       output: Tensor, is_training: bool = True) -> int:
        if is_training:
            self.sums_to_statistics(self._num_per_sum(input), mean, var, running_mean, running_var,
                                    input.h2x_dtype)
            self.batch_normalization(input, mean, var, scale, bias, output)
        else:
            self.batch_normalization(input, running_mean, running_var, scale, bias, output)  # :243-247
        return 0

    def _runs_local(self, *tensors: Tensor) -> bool:
        """No all-reduce between the stages, a rank that owns elements (and no halo to clear)."""
        t0 = tensors[0]
        return (self.fuse_local and not (self.global_stats and self.allreduce is not None)
                and t0.is_split_root() and t0.get_local_size() > 0
                and not (self.clear_output_halo and any(any(t.overlap) for t in tensors)))

    def forward(self, input, mean, var, running_mean, running_var, scale, bias, output,
                is_training: bool = True) -> int:
        if is_training and self._runs_local(input, output):
            self.set_num_samples(input.local_shape[-1])
            n, c, s, sr = _channel_geometry(input)
            _, _, _, sro = _channel_geometry(output)
            if _is_dense(input) and _is_dense(output):
                capi.check(self._lib.h2x_bn_forward_local(
                    input.h2x_dtype, self.num_current_samples, c, s, sr, sro, _ptr(input.get_base_ptr()),
                    _ptr(scale), _ptr(bias), self._num_per_sum(input), self.decay, self.epsilon, _ptr(mean),
                    _ptr(var), _ptr(running_mean), _ptr(running_var), _ptr(output.get_base_ptr()),
                    _ptr(self._ws(c)), _stream_handle(self.stream)), "bn forward (local)")
            else:
                ns = self.num_current_samples
                gx, gy = _tensor_geometry(input, ns), _tensor_geometry(output, ns)
                capi.check(self._lib.h2x_bn_forward_local_strided(
                    input.h2x_dtype, ns, ctypes.byref(gx), ctypes.byref(gy), _ptr(input.get_base_ptr()),
                    _ptr(scale), _ptr(bias), self._num_per_sum(input), self.decay, self.epsilon, _ptr(mean),
                    _ptr(var), _ptr(running_mean), _ptr(running_var), _ptr(output.get_base_ptr()),
                    _ptr(self._ws(c)), _stream_handle(self.stream)), "bn forward (local, strided)")
            return 0
        self.forward_stage1(input, mean, var, is_training)
        self.forward_allreduce(mean, var, is_training)
        return self.forward_stage2(input, mean, var, running_mean, running_var, scale, bias, output,
                                   is_training)

    # ---- backward ----------------------------------------------------------
    def backward_stage1(self, input: Tensor, d_output: Tensor, mean, var, scale, scale_gradient,
                        bias_gradient, mean_gradient, var_gradient) -> int:
        self.set_num_samples(input.local_shape[-1])
        n, c, s, sr = _channel_geometry(input)
        _, _, _, sro = _channel_geometry(d_output)
        active = input.is_split_root() and input.get_local_size() > 0
        ns = self.num_current_samples if active else 0
        tail = (_ptr(mean), _ptr(var), _ptr(scale), _ptr(scale_gradient), _ptr(bias_gradient),
                _ptr(mean_gradient), _ptr(var_gradient), self.epsilon, _ptr(self._ws(c)),
                _stream_handle(self.stream))
        if _is_dense(input) and _is_dense(d_output):
            capi.check(self._lib.h2x_bn_backprop1(
                input.h2x_dtype, ns, c, s, sr, sro, _ptr(input.get_base_ptr()),
                _ptr(d_output.get_base_ptr()), *tail), "backprop1")
        else:
            gx, gd = _tensor_geometry(input, ns), _tensor_geometry(d_output, ns)
            capi.check(self._lib.h2x_bn_backprop1_strided(
                input.h2x_dtype, ns, ctypes.byref(gx), ctypes.byref(gd), _ptr(input.get_base_ptr()),
                _ptr(d_output.get_base_ptr()), *tail), "backprop1 (strided)")
        return 0

    def backward_allreduce(self, scale_gradient, bias_gradient, mean_gradient, var_gradient,
                           skip_weights: bool = False) -> int:
        if not self.global_stats or self.allreduce is None:  # batchnorm.hpp:367-368
            return 0
        self.allreduce([mean_gradient, var_gradient])
        if not skip_weights:
            self.allreduce([scale_gradient])
            self.allreduce([bias_gradient])
        return 0

    def backward_stage2(self, input: Tensor, d_output: Tensor, mean, var, scale, mean_gradient,
                        var_gradient, d_input: Tensor) -> int:
        n, c, s, sr = _channel_geometry(input)
        _, _, _, sro = _channel_geometry(d_output)
        _, _, _, sri = _channel_geometry(d_input)
        ns = self.num_current_samples
        tail = (_ptr(input.get_base_ptr()), _ptr(d_output.get_base_ptr()), _ptr(mean), _ptr(var),
                _ptr(scale), _ptr(mean_gradient), _ptr(var_gradient), _ptr(d_input.get_base_ptr()),
                self.epsilon, _stream_handle(self.stream))
        if self.clear_output_halo and ns == n and _share_a_haloed_geometry(input, d_output, d_input):
            g = _haloed_geometry(d_input)
            capi.check(self._lib.h2x_bn_backprop2_clearing(
                input.h2x_dtype, self._num_per_sum(input), ctypes.byref(g), _ptr(input.get_buffer()),
                _ptr(d_output.get_buffer()), _ptr(mean), _ptr(var), _ptr(scale), _ptr(mean_gradient),
                _ptr(var_gradient), _ptr(d_input.get_buffer()), self.epsilon, _stream_handle(self.stream)),
                "backprop2 (clearing)")
        # the reference takes its fast path only for halo-free tensors (batchnorm.cu:1503-1506)
        elif _is_dense(input) and _is_dense(d_output) and _is_dense(d_input):
            capi.check(self._lib.h2x_bn_backprop2(
                input.h2x_dtype, ns, c, s, sr, sro, sri, self._num_per_sum(input), *tail), "backprop2")
        else:
            gx, gd, gi = (_tensor_geometry(t, ns) for t in (input, d_output, d_input))
            capi.check(self._lib.h2x_bn_backprop2_strided(
                input.h2x_dtype, ns, self._num_per_sum(input), ctypes.byref(gx), ctypes.byref(gd),
                ctypes.byref(gi), *tail), "backprop2 (strided)")
        return 0

    def backward(self, input, d_output, mean, var, scale, scale_gradient, bias_gradient,
                 mean_gradient, var_gradient, d_input) -> int:
        if self._runs_local(input, d_output, d_input):
            self.set_num_samples(input.local_shape[-1])
            n, c, s, sr = _channel_geometry(input)
            _, _, _, sro = _channel_geometry(d_output)
            _, _, _, sri = _channel_geometry(d_input)
            tail = (_ptr(input.get_base_ptr()), _ptr(d_output.get_base_ptr()), _ptr(mean), _ptr(var),
                    _ptr(scale), _ptr(scale_gradient), _ptr(bias_gradient), _ptr(mean_gradient),
                    _ptr(var_gradient), _ptr(d_input.get_base_ptr()), self.epsilon, _ptr(self._ws(c)),
                    _stream_handle(self.stream))
            if _is_dense(input) and _is_dense(d_output) and _is_dense(d_input):
                capi.check(self._lib.h2x_bn_backward_local(
                    input.h2x_dtype, self.num_current_samples, c, s, sr, sro, sri, self._num_per_sum(input),
                    *tail), "bn backward (local)")
            else:
                ns = self.num_current_samples
                gx, gd, gi = (_tensor_geometry(t, ns) for t in (input, d_output, d_input))
                capi.check(self._lib.h2x_bn_backward_local_strided(
                    input.h2x_dtype, ns, self._num_per_sum(input), ctypes.byref(gx), ctypes.byref(gd),
                    ctypes.byref(gi), *tail), "bn backward (local, strided)")
            return 0
        self.backward_stage1(input, d_output, mean, var, scale, scale_gradient, bias_gradient,
                             mean_gradient, var_gradient)
        self.backward_allreduce(scale_gradient, bias_gradient, mean_gradient, var_gradient)
        return self.backward_stage2(input, d_output, mean, var, scale, mean_gradient, var_gradient,
                                    d_input)


def _local_geometry(t: Tensor, region: Optional[Sequence[int]] = None) -> capi.TensorGeometry:
    """Local shape (or a region of it that starts at the first interior element)
    and the strides of the real allocation."""
    g = capi.TensorGeometry()
    nd = t.get_num_dims()
    g.num_dims = nd
    strides = t.get_strides()
    for i in range(nd):
        g.local_shape[i] = t.local_shape[i] if region is None else region[i]
        g.strides[i] = strides[i]
    return g


def transform(op: int, tensors: Sequence[Tensor], params: Sequence[float] = (),
              stream: Optional[torch.cuda.Stream] = None) -> None:
    """tensor::Transform over the interiors of 1-4 tensors of equal local shape
    (legacy/include/distconv/tensor/algorithms/transform_cuda.hpp:359-693) for the
    functors the library names: capi.TRANSFORM_SCALE (t *= p0), TRANSFORM_COPY
    (t1 = t0), TRANSFORM_SCALE_BIAS (t1 = p0 * t0 + p1), TRANSFORM_SUMS_TO_STATISTICS
    (mean, var, running_mean, running_var; p0 = count, p1 = decay)."""
    n = len(tensors)
    for t in tensors:
        if list(t.local_shape) != list(tensors[0].local_shape):
            raise ValueError("tensors of a transform must have the same local shape")  # :383-390
    if tensors[0].get_local_size() == 0:
        return
    geoms = [_local_geometry(t) for t in tensors]
    gp = (ctypes.POINTER(capi.TensorGeometry) * n)(*[ctypes.pointer(g) for g in geoms])
    tp = (ctypes.c_void_p * n)(*[t.get_base_ptr() for t in tensors])
    pp = (ctypes.c_double * 4)(*(list(params) + [0.0] * (4 - len(params))))
    capi.check(capi.load().h2x_tensor_transform(op, tensors[0].h2x_dtype, n, gp, tp, pp, _stream_handle(stream)),
               "tensor transform")


_reduce_workspaces = {}


def reduce_sum(src: Tensor, dst: Tensor, square: bool = False, region: Optional[Sequence[int]] = None,
               stream: Optional[torch.cuda.Stream] = None) -> None:
    """tensor::ReduceSum / TransformReduceSum (reduce_sum_cuda.hpp:388-439,
    transform_reduce_sum_cuda.hpp:17-87): dst += sum of src (of its squares) over
    every dimension along which dst's local extent is 1.  The sum over ranks that
    the reference ends with (reduce_sum_cuda.hpp:186-192) is the caller's."""
    lib = capi.load()
    gs, gd = _local_geometry(src, region), _local_geometry(dst)
    need = lib.h2x_tensor_reduce_sum_workspace_bytes(ctypes.byref(gs), ctypes.byref(gd))
    key = torch.cuda.current_stream().cuda_stream if stream is None else stream.cuda_stream
    ws = _reduce_workspaces.get(key)
    if ws is None or ws.numel() < need:
        ws = _reduce_workspaces[key] = _device_buffer(max(need, 256), torch.uint8)
    capi.check(lib.h2x_tensor_reduce_sum(src.h2x_dtype, ctypes.byref(gs), ctypes.c_void_p(src.get_base_ptr()),
                                         ctypes.byref(gd), ctypes.c_void_p(dst.get_base_ptr()), int(square),
                                         ctypes.c_void_p(ws.data_ptr()), _stream_handle(stream)), "tensor reduce_sum")


class SoftmaxMode(Enum):
    """legacy/include/distconv/base.hpp (SoftmaxMode)."""
    INSTANCE = 0
    CHANNEL = 1


class Softmax:
    """Softmax<Backend> (legacy/include/distconv/dnn_backend/softmax.hpp:14-63).

    ``allreduce(values, is_max)``, if given, is called on the per-sample scalars of
    instance mode where the reference all-reduces them over the ranks that share
    a sample (softmax.hpp:52-62); ``None`` means every sample is whole on this rank.
    """

    def __init__(self, stream: Optional[torch.cuda.Stream] = None,
                 allreduce: Optional[Callable[[torch.Tensor, bool], None]] = None):
        self.stream, self.allreduce = stream, allreduce
        self.mode = SoftmaxMode.CHANNEL
        self._lib = capi.load()
        self._ws: Optional[torch.Tensor] = None

    def setup(self, input: Tensor, mode: SoftmaxMode) -> None:
        self.mode = mode

    @staticmethod
    def _geometry(t: Tensor):
        if any(t.overlap):
            raise NotImplementedError("softmax assumes a dense local tensor")  # softmax.cu:562-563
        nd = t.get_num_dims()
        return t.local_shape[nd - 1], t.local_shape[nd - 2], _prod(t.local_shape[: nd - 2])

    def _workspace(self, n: int) -> torch.Tensor:
        need = self._lib.h2x_softmax_instance_workspace_bytes(n)
        if self._ws is None or self._ws.numel() < need:
            self._ws = _device_buffer(need, torch.uint8)
        return self._ws

    def forward(self, x: Tensor, y: Tensor) -> int:
        n, c, s = self._geometry(x)
        if n == 0:
            return 0
        st = _stream_handle(self.stream)
        if self.mode == SoftmaxMode.CHANNEL:
            capi.check(self._lib.h2x_softmax_channel_forward(
                x.h2x_dtype, n, c, s, _ptr(x.get_base_ptr()), _ptr(y.get_base_ptr()), st), "softmax forward")
            return 0
        # instance mode: softmax.cu:723-746
        dt, size, ws = x.h2x_dtype, c * s, self._workspace(n)
        smax = torch.empty(n, dtype=x.dtype, device=x.device)
        sexp = torch.empty(n, dtype=x.dtype, device=x.device)
        if self.allreduce is None:
            # every sample is whole on this rank: the stages need not be separate calls
            capi.check(self._lib.h2x_softmax_instance_forward_local(
                dt, n, size, _ptr(x.get_base_ptr()), _ptr(y.get_base_ptr()), _ptr(smax), _ptr(sexp), _ptr(ws), st),
                "softmax instance forward")
            return 0
        capi.check(self._lib.h2x_softmax_instance_max(dt, n, size, _ptr(x.get_base_ptr()), _ptr(smax),
                                                      _ptr(ws), st), "softmax instance max")
        if self.allreduce:
            self.allreduce(smax, True)
        capi.check(self._lib.h2x_softmax_instance_exp(dt, n, size, _ptr(x.get_base_ptr()), _ptr(smax),
                                                      _ptr(y.get_base_ptr()), _ptr(sexp), _ptr(ws), st),
                   "softmax instance exp")
        if self.allreduce:
            self.allreduce(sexp, False)
        capi.check(self._lib.h2x_softmax_instance_normalize(dt, n, size, _ptr(sexp), _ptr(y.get_base_ptr()), st),
                   "softmax instance normalize")
        return 0

    def backward(self, y: Tensor, dy: Tensor, dx: Tensor) -> int:
        n, c, s = self._geometry(dx)
        if n == 0:
            return 0
        st = _stream_handle(self.stream)
        if self.mode == SoftmaxMode.CHANNEL:
            capi.check(self._lib.h2x_softmax_channel_backward(
                y.h2x_dtype, n, c, s, _ptr(y.get_base_ptr()), _ptr(dy.get_base_ptr()),
                _ptr(dx.get_base_ptr()), st), "softmax backward")
            return 0
        # instance mode: softmax.cu:770-783
        dt, size, ws = y.h2x_dtype, c * s, self._workspace(n)
        sdp = torch.empty(n, dtype=y.dtype, device=y.device)
        capi.check(self._lib.h2x_softmax_instance_dot(dt, n, size, _ptr(y.get_base_ptr()),
                                                      _ptr(dy.get_base_ptr()), _ptr(sdp), _ptr(ws), st),
                   "softmax instance dot")
        if self.allreduce:
            self.allreduce(sdp, False)
        capi.check(self._lib.h2x_softmax_instance_gradient(dt, n, size, _ptr(y.get_base_ptr()),
                                                           _ptr(dy.get_base_ptr()), _ptr(sdp),
                                                           _ptr(dx.get_base_ptr()), st),
                   "softmax instance gradient")
        return 0


class HaloExchangeAccumOp(Enum):
    """legacy/include/distconv/tensor/halo_exchange.hpp:8-9."""
    ID = capi.HALO_ID
    SUM = capi.HALO_SUM
    MAX = capi.HALO_MAX
    MIN = capi.HALO_MIN


class HaloExchangeVirtual:
    """HaloExchange for all virtual ranks of one distributed tensor
    (legacy/include/distconv/tensor/halo_exchange_cuda.hpp:18-423).

    The reference object belongs to one rank and hands packed strips to a
    transport.  Here the object holds every rank's local tensor; rank r's send
    buffer for (dim, side) *is* the receive buffer of its neighbour on that
    side for the opposite side, so the transfer is free, and each dimension
    phase is two launches (pack all ranks and sides, unpack all ranks and
    sides).  ``periodic`` wraps neighbours at the grid edge; the reference
    never does (MPI_PROC_NULL, halo_exchange_cuda.hpp:343-345).
    """

    def __init__(self, tensors: Sequence[Tensor], periodic: bool = False,
                 stream: Optional[torch.cuda.Stream] = None):
        self.tensors = list(tensors)
        self.periodic, self.stream = periodic, stream
        self._lib = capi.load()
        t0 = self.tensors[0]
        self.dist = t0.dist
        if len(self.tensors) != self.dist.num_ranks:
            raise ValueError("one local tensor per rank of the distribution is required")
        if t0.dist.num_ranks != _prod(t0.dist.split_shape):
            raise NotImplementedError("shared (replicated) distributions are not exchanged")  # :30-31
        self.nd = t0.get_num_dims()
        self._recv = {}  # (rank, dim, side) -> torch buffer the rank unpacks from
        self._faces = {}  # exchange arguments -> (pack faces, unpack faces)
        # optional callable(label, launch, num_faces): wraps every launch, for per-kernel timing
        self.launch_hook = None

    def get_halo_size(self, rank: int, dim: int, width: int) -> int:
        """halo_exchange_cuda.hpp:267-271."""
        shape = list(self.tensors[rank].local_real_shape)
        shape[dim] = width
        return _prod(shape)

    def is_exchange_required(self, rank: int, dim: int, widths=None) -> bool:
        """halo_exchange_cuda.hpp:305-320."""
        t = self.tensors[rank]
        w = t.overlap[dim] if widths is None else max(widths)
        return self.dist.is_distributed(dim) and self.dist.split_shape[dim] > 1 and w > 0 \
            and t.get_local_size() > 0

    def find_peer_rank(self, rank: int, dim: int, side: int) -> Optional[int]:
        """halo_exchange_cuda.hpp:322-357; None stands for MPI_PROC_NULL."""
        t = self.tensors[rank]
        if not self.is_exchange_required(rank, dim):
            return None
        extent = self.dist.locale_shape[dim]
        p = t.proc_index[dim] + (1 if side == capi.RHS else -1)
        if p < 0 or p >= extent:
            if not self.periodic:
                return None
            p %= extent
        idx = list(t.proc_index)
        idx[dim] = p
        peer = self.dist.rank_of(idx)
        if self.tensors[peer].get_local_size() == 0:
            return None
        return peer

    def _check_widths(self, dim: int, widths) -> None:
        """The receive buffers hold `overlap[dim]` cells per row and the strips lie
        inside the halo: TraverseHalo's precondition, halo_cuda.hpp:909-916."""
        for t in self.tensors:
            if max(widths) > t.overlap[dim]:
                raise ValueError(f"halo width {max(widths)} exceeds the overlap {t.overlap[dim]} of "
                                 f"dimension {dim}")

    def _addresses(self):
        """Device addresses the cached face tables were built for; a tensor that
        was reallocated gets new tables."""
        return tuple(t.get_buffer() if t.data is not None else 0 for t in self.tensors)

    def recv_buffer(self, rank: int, dim: int, side: int) -> torch.Tensor:
        """The buffer rank `rank` unpacks its (dim, side) halo from -- and its
        neighbour on that side packs into (get_recv_buffer, halo_exchange_cuda.hpp:277-283)."""
        key = (rank, dim, side)
        if key not in self._recv:
            t = self.tensors[rank]
            n = self.get_halo_size(rank, dim, t.overlap[dim])  # sized for the full halo (:285-303)
            self._recv[key] = _device_buffer(max(n, 1), t.dtype, t.device, zero=True)
        return self._recv[key]

    def make_face(self, rank, dim, side, width, buf, is_pack, is_reverse, op) -> capi.HaloFace:
        """One h2x_halo_face of rank `rank`: what pack_dim / unpack_dim pass down
        (halo_exchange_cuda.hpp:365-393)."""
        t = self.tensors[rank]
        f = capi.HaloFace()
        f.tensor = t.get_buffer()
        f.buffer = buf.data_ptr()
        for i, e in enumerate(t.local_real_shape):
            f.real_shape[i] = e
        f.num_dims, f.dim, f.side, f.width = self.nd, dim, side, width
        f.inner = int((is_pack and not is_reverse) or ((not is_pack) and is_reverse))
        f.is_pack, f.op = int(is_pack), op.value
        return f

    def exchange_dim(self, dim: int, width_rhs_send: int, width_rhs_recv: int, width_lhs_send: int,
                     width_lhs_recv: int, is_reverse: bool = False, skip_unpack: bool = False,
                     op: HaloExchangeAccumOp = HaloExchangeAccumOp.ID, fused: bool = False) -> None:
        """One dimension for all ranks; the order pack -> (transfer) -> unpack of
        halo_exchange_cuda_mpi.hpp:25-100.  A rank's RHS strip goes to its RHS
        neighbour's LHS receive buffer and vice versa.  With ``fused`` the strips
        move straight from tensor to tensor in one launch per group of ranks;
        the result is the same."""
        dtype = self.tensors[0].h2x_dtype
        self._check_widths(dim, (width_rhs_send, width_rhs_recv, width_lhs_send, width_lhs_recv))
        if fused:
            if skip_unpack:
                raise ValueError("a fused exchange has no separate unpack to skip")
            self._exchange_dim_fused(dim, width_rhs_send, width_rhs_recv, width_lhs_send,
                                     width_lhs_recv, is_reverse, op)
            return
        key = (dim, width_rhs_send, width_rhs_recv, width_lhs_send, width_lhs_recv, is_reverse,
               skip_unpack, op, self._addresses())
        cached = self._faces.get(key)
        if cached is None:
            widths = (width_rhs_send, width_rhs_recv, width_lhs_send, width_lhs_recv)
            cached = []
            for group in self._rank_groups(dim, max(widths)):
                packs, unpacks = [], []
                for r in group:
                    if not self.is_exchange_required(r, dim, widths):
                        continue
                    for side in (capi.LHS, capi.RHS):
                        peer = self.find_peer_rank(r, dim, side)
                        if peer is None:
                            continue
                        w_send = width_rhs_send if side == capi.RHS else width_lhs_send
                        w_recv = width_rhs_recv if side == capi.RHS else width_lhs_recv
                        if w_send > 0:
                            dst = self.recv_buffer(peer, dim, capi.LHS if side == capi.RHS else capi.RHS)
                            packs.append(self.make_face(r, dim, side, w_send, dst, True, is_reverse, op))
                        if w_recv > 0 and not skip_unpack:
                            src = self.recv_buffer(r, dim, side)
                            unpacks.append(self.make_face(r, dim, side, w_recv, src, False, is_reverse, op))
                # the face tables depend only on the arguments and on the tensors'
                # addresses (part of the key): build them once
                cached.append(tuple((capi.HaloFace * len(f))(*f) if f else None for f in (packs, unpacks)))
            self._faces[key] = cached
        st = _stream_handle(self.stream)
        for group in cached:
            for what, arr in zip(("pack", "unpack"), group):
                if arr is None:
                    continue
                launch = lambda arr=arr: capi.check(
                    self._lib.h2x_halo_pack_or_unpack_batched(dtype, arr, len(arr), st), "halo pack/unpack")
                if self.launch_hook is None:
                    launch()
                else:
                    self.launch_hook(f"halo_dim{dim}_{what}", launch, len(arr))

    def _exchange_dim_fused(self, dim, width_rhs_send, width_rhs_recv, width_lhs_send,
                            width_lhs_recv, is_reverse, op) -> None:
        dtype = self.tensors[0].h2x_dtype
        widths = (width_rhs_send, width_rhs_recv, width_lhs_send, width_lhs_recv)
        key = ("fused", dim) + widths + (is_reverse, op, self._addresses())
        cached = self._faces.get(key)
        if cached is None:
            cached = []
            # one launch for all ranks: nothing is read back between two launches
            # here, so groups would only add launches (measured: 289 us against 301 us)
            for group in [range(len(self.tensors))]:
                moves = []
                for r in group:  # r receives; both of its halos are neighbours in the table
                    if not self.is_exchange_required(r, dim, widths):
                        continue
                    for side in (capi.LHS, capi.RHS):
                        peer = self.find_peer_rank(r, dim, side)
                        if peer is None:
                            continue
                        # what the peer sends towards r leaves the peer on the opposite side
                        w_send = width_lhs_send if side == capi.RHS else width_rhs_send
                        w_recv = width_rhs_recv if side == capi.RHS else width_lhs_recv
                        if w_send != w_recv:
                            raise ValueError("a fused exchange needs equal send and receive widths")
                        if w_recv == 0:
                            continue
                        src, dst = self.tensors[peer], self.tensors[r]
                        m = capi.HaloTransfer()
                        m.src, m.dst = src.get_buffer(), dst.get_buffer()
                        for i in range(self.nd):
                            m.src_real_shape[i] = src.local_real_shape[i]
                            m.dst_real_shape[i] = dst.local_real_shape[i]
                        m.num_dims, m.dim, m.width = self.nd, dim, w_recv
                        m.src_side = capi.LHS if side == capi.RHS else capi.RHS
                        m.is_reverse, m.op = int(is_reverse), op.value
                        moves.append(m)
                cached.append((capi.HaloTransfer * len(moves))(*moves) if moves else None)
            self._faces[key] = cached
        st = _stream_handle(self.stream)
        for arr in cached:
            if arr is None:
                continue
            launch = lambda arr=arr: capi.check(
                self._lib.h2x_halo_exchange_fused(dtype, arr, len(arr), st), "fused halo exchange")
            if self.launch_hook is None:
                launch()
            else:
                self.launch_hook(f"halo_dim{dim}_fused", launch, len(arr))

    # Faces of the innermost dimension touch one short run per row, and every
    # run costs a whole 128-byte line of memory traffic; the unpack writes into
    # the lines its rank's pack has just read.  Exchanging a few ranks at a time
    # keeps those lines in the 256 MB memory-side cache between the two launches,
    # where the unpack's partial writes merge into whole lines (measured on the
    # 8-rank, 130^3 x 32 case: groups of two ranks, 138 MB of lines, take 275 us,
    # groups of four 290 us, all eight at once more than 300 us).
    _SPARSE_GROUP_BYTES = 160 << 20
    _LINE_BYTES = 128

    def _rank_groups(self, dim: int, width: int) -> List[List[int]]:
        """Partition of the ranks into groups that exchange dimension `dim`
        one after the other.  Neighbours along `dim` always share a group."""
        ranks = list(range(len(self.tensors)))
        t0 = self.tensors[0]
        elem = torch.empty(0, dtype=t0.dtype).element_size()
        if dim != 0 or width * elem >= self._LINE_BYTES:
            return [ranks]
        lines = {}
        for r in ranks:
            idx = list(self.tensors[r].proc_index)
            idx[dim] = 0
            lines.setdefault(tuple(idx), []).append(r)
        groups, current, current_bytes = [], [], 0
        for members in lines.values():
            nbytes = sum(_prod(self.tensors[r].local_real_shape[1:]) * self._LINE_BYTES for r in members)
            if current and current_bytes + nbytes > self._SPARSE_GROUP_BYTES:
                groups.append(current)
                current, current_bytes = [], 0
            current += members
            current_bytes += nbytes
        if current:
            groups.append(current)
        return groups

    def exchange(self, widths_rhs_send=None, widths_rhs_recv=None, widths_lhs_send=None,
                 widths_lhs_recv=None, is_reverse: bool = False, skip_unpack: bool = False,
                 op: HaloExchangeAccumOp = HaloExchangeAccumOp.ID, fused: bool = False) -> None:
        """All dimensions, innermost first, each seeing the halo cells the previous
        ones filled (halo_exchange_cuda.hpp:56-106)."""
        ov = self.tensors[0].overlap
        wrs = ov if widths_rhs_send is None else widths_rhs_send
        wrr = ov if widths_rhs_recv is None else widths_rhs_recv
        wls = ov if widths_lhs_send is None else widths_lhs_send
        wlr = ov if widths_lhs_recv is None else widths_lhs_recv
        for d in range(self.nd):
            self.exchange_dim(d, wrs[d], wrr[d], wls[d], wlr[d], is_reverse, skip_unpack, op, fused)

    def clear_halo(self, dim: int) -> None:
        """Tensor::clear_halo (legacy/src/tensor/tensor_mpi_cuda.cu:14-84) on every rank."""
        for t in self.tensors:
            if t.overlap[dim] == 0 or t.get_local_size() == 0:
                continue
            shape = capi.i64_array(t.local_real_shape)
            capi.check(self._lib.h2x_halo_clear(t.h2x_dtype, _ptr(t.get_buffer()), self.nd, shape,
                                                dim, t.overlap[dim], _stream_handle(self.stream)),
                       "clear_halo")


    def clear_halos(self, only_unfilled: bool = False) -> None:
        """clear_halo of every dimension that has a halo, on every rank, in batched
        launches: the loop that precedes the forward exchange in Convolution::forward
        (legacy/include/distconv/dnn_backend/convolution.hpp:400-411).

        ``only_unfilled``: only the sides without a neighbour are cleared.  A
        full-width ``exchange()`` that follows overwrites every other halo strip
        completely (a strip spans the whole real extent of the other dimensions);
        the stale values it moves into corner cells on the way are overwritten by a
        later dimension's phase, and a corner that no later phase fills receives
        cleared cells, because neighbours along one dimension sit at the same
        position of every other dimension.  The tensors end up exactly as after
        clearing everything first."""
        key = ("clear", only_unfilled, self._addresses())
        if key not in self._faces:
            faces = []
            for r, t in enumerate(self.tensors):
                if t.get_local_size() == 0:
                    continue
                for d in range(self.nd):
                    if t.overlap[d] == 0:
                        continue
                    for side in (capi.LHS, capi.RHS):
                        if only_unfilled and self.find_peer_rank(r, d, side) is not None:
                            continue
                        f = capi.HaloFace()
                        f.tensor = t.get_buffer()
                        for i, e in enumerate(t.local_real_shape):
                            f.real_shape[i] = e
                        f.num_dims, f.dim, f.side, f.width, f.inner = self.nd, d, side, t.overlap[d], 0
                        faces.append(f)
            self._faces[key] = (capi.HaloFace * len(faces))(*faces)
        arr = self._faces[key]
        if len(arr):
            capi.check(self._lib.h2x_halo_clear_batched(self.tensors[0].h2x_dtype, arr, len(arr),
                                                        _stream_handle(self.stream)), "clear_halos")


class TensorShufflerVirtual:
    """TensorMPICUDAShuffler for all virtual ranks of a (src, dst) pair of
    distributed tensors (legacy/include/distconv/tensor/shuffle_mpi_cuda.hpp:14-512,
    legacy/src/tensor/shuffle_mpi_cuda.cu:378-476).

    The tables are the reference constructor's (rank_limits per dimension,
    counts and displacements in rank order).  All ranks' receive buffers live in
    one arena and every rank packs straight into its peers' chunks of it -- the
    all-to-all of the reference's ``transfer`` is therefore free -- and each
    direction is two launches: pack for all ranks, unpack for all ranks.
    """

    def __init__(self, src_tensors: Sequence[Tensor], dst_tensors: Sequence[Tensor],
                 stream: Optional[torch.cuda.Stream] = None):
        self.src, self.dst, self.stream = list(src_tensors), list(dst_tensors), stream
        self._lib = capi.load()
        if len(self.src) != len(self.dst):
            raise ValueError("source and destination must have the same number of ranks")
        self.num_ranks = len(self.src)
        self.elem_size = torch.empty(0, dtype=self.src[0].dtype).element_size()
        self._keep = []  # ctypes arrays referenced by geometries
        self._fwd = self._direction(self.src, self.dst)
        self._bwd = self._direction(self.dst, self.src)

    @staticmethod
    def get_buf_size(t: Tensor) -> int:
        """shuffle_mpi_cuda.hpp:83-90 (bytes)."""
        return t.get_local_size() * torch.empty(0, dtype=t.dtype).element_size()

    # -- tables (shuffle_mpi_cuda.hpp:129-287) --------------------------------
    @staticmethod
    def rank_limits(a: Tensor, b: Tensor) -> List[int]:
        """End, in a's local coordinates, of each slab of b's process grid."""
        out = []
        for d in range(a.get_num_dims()):
            extent = b.dist.locale_shape[d]
            per = b.dist.get_num_ranks_per_split(d)
            for j in range(extent):
                nxt_root = (j // per + 1) * per  # next split root after j
                nxt = b.get_dimension_rank_offset(d, nxt_root) if nxt_root < extent else b.shape[d]
                lim = 0 if nxt < a.global_index[d] else min(nxt - a.global_index[d], a.local_shape[d])
                out.append(lim)
        return out

    @staticmethod
    def _overlap_size(a: Tensor, b: Tensor, b_index: Sequence[int]) -> int:
        size = 1
        for d in range(a.get_num_dims()):
            b0 = b.get_dimension_rank_offset(d, b_index[d])
            b1 = b0 + b.get_remote_dimension(d, b_index[d])
            lo, hi = max(a.global_index[d], b0), min(a.global_index[d] + a.local_shape[d], b1)
            size *= max(hi - lo, 0)
        return size

    def _counts(self, a: Tensor, b: Tensor) -> List[int]:
        """Elements rank a exchanges with every rank of b's grid, in rank order."""
        counts = []
        for pid in range(self.num_ranks):
            idx = b.dist.rank_index(pid)
            ok = a.is_split_root() and b.dist.is_split_root_index(idx)
            counts.append(self._overlap_size(a, b, idx) if ok else 0)
        return counts

    def _direction(self, src: List[Tensor], dst: List[Tensor]):
        """Plans and buffers for src -> dst."""
        n = self.num_ranks
        send_counts = [self._counts(src[r], dst[r]) for r in range(n)]
        recv_counts = [self._counts(dst[r], src[r]) for r in range(n)]
        for r in range(n):
            for p in range(n):
                assert send_counts[r][p] == recv_counts[p][r]
        recv_displs = [[sum(recv_counts[r][:p]) for p in range(n)] for r in range(n)]
        recv_sizes = [sum(recv_counts[r]) for r in range(n)]
        arena_offsets = [sum(recv_sizes[:r]) for r in range(n)]
        arena = _device_buffer(max(sum(recv_sizes), 1), src[0].dtype, src[0].device, zero=True)
        if sum(recv_sizes) >= 2 ** 31:
            raise ValueError("arena exceeds the 32-bit displacements of the shuffler tables")
        pack_plans, unpack_plans = [], []
        for r in range(n):
            # pack: chunk for peer p lands in p's receive buffer at the slot reserved for r
            displs = [arena_offsets[p] + recv_displs[p][r] for p in range(n)]
            pack_plans.append(self._plan(src[r], dst[r], self.rank_limits(src[r], dst[r]), displs)
                              if src[r].is_split_root() and src[r].get_local_size() > 0 else None)
            displs = [arena_offsets[r] + recv_displs[r][p] for p in range(n)]
            unpack_plans.append(self._plan(dst[r], src[r], self.rank_limits(dst[r], src[r]), displs)
                                if dst[r].is_split_root() and dst[r].get_local_size() > 0 else None)
        return dict(arena=arena, pack=pack_plans, unpack=unpack_plans,
                    send_counts=send_counts, recv_counts=recv_counts, recv_displs=recv_displs)

    def _plan(self, mine: Tensor, other: Tensor, limits: List[int], displs: List[int]):
        g = capi.ShuffleGeometry()
        g.num_dims, g.elem_size = mine.get_num_dims(), self.elem_size
        for i in range(mine.get_num_dims()):
            g.local_shape[i] = mine.local_shape[i]
            g.strides[i] = mine.get_strides()[i]
            g.peer_locale_shape[i] = other.dist.locale_shape[i]
        rl = (ctypes.c_int32 * len(limits))(*limits)
        dp = (ctypes.c_int32 * len(displs))(*displs)
        g.rank_limits, g.displs = rl, dp
        plan = ctypes.c_void_p()
        capi.check(self._lib.h2x_shuffle_plan_create(ctypes.byref(g), ctypes.byref(plan)),
                   "shuffle plan")
        return plan

    def _launch(self, fn, plans, tensors: List[Tensor], arena: torch.Tensor) -> None:
        live = [(p, t) for p, t in zip(plans, tensors) if p is not None]
        if not live:
            return
        n = len(live)
        pa = (ctypes.c_void_p * n)(*[p for p, _ in live])
        ta = (ctypes.c_void_p * n)(*[t.get_base_ptr() for _, t in live])
        ba = (ctypes.c_void_p * n)(*[arena.data_ptr()] * n)
        capi.check(fn(pa, ta, ba, n, _stream_handle(self.stream)), "shuffle")

    def shuffle_forward(self) -> None:
        """src tensors -> dst tensors (shuffle_mpi_cuda.cu:478-484)."""
        d = self._fwd
        self._launch(self._lib.h2x_shuffle_pack_batched, d["pack"], self.src, d["arena"])
        self._launch(self._lib.h2x_shuffle_unpack_batched, d["unpack"], self.dst, d["arena"])

    def shuffle_backward(self) -> None:
        """dst tensors -> src tensors (shuffle_mpi_cuda.cu:485-490)."""
        d = self._bwd
        self._launch(self._lib.h2x_shuffle_pack_batched, d["pack"], self.dst, d["arena"])
        self._launch(self._lib.h2x_shuffle_unpack_batched, d["unpack"], self.src, d["arena"])

    def __del__(self):
        try:
            for d in (self._fwd, self._bwd):
                for p in d["pack"] + d["unpack"]:
                    if p is not None:
                        self._lib.h2x_shuffle_plan_destroy(p)
        except Exception:
            pass

"""MI355X (gfx950) implementation of DistConv's data-parallel non-convolution
hot path: batch-norm statistics, halo pack/unpack, channel softmax and the
tensor shuffler, as hand-written HIP kernels behind a C ABI (include/h2x.h).

``capi``     ctypes binding of libh2x.so (raises if the library is missing)
``tensor``   distributions, virtual locales, distributed tensors on torch memory
``layers``   BatchNormalization, Softmax, HaloExchangeVirtual, TensorShufflerVirtual
"""
from . import capi  # noqa: F401

__all__ = ["capi", "tensor", "layers"]

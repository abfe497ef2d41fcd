#!/usr/bin/env python3
"""Writes the small golden fixtures of this directory.

The reference ships no stored vectors for this path (its tests use closed
forms and self-comparison), so these are computed here from the mathematics in
float64 numpy -- independently of the oracle's C code -- for seeded inputs.
They pin the oracle (CPU tests) and the GPU library (GPU tests) to the same
numbers.  Run:  python tests/golden/make_golden.py
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def bn_case(shape, seed):
    rng = np.random.default_rng(seed)
    c = shape[1]
    x = rng.standard_normal(shape).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    scale = rng.uniform(0.5, 1.5, c).astype(np.float32)
    bias = (0.1 * rng.standard_normal(c)).astype(np.float32)
    eps, decay = 1e-5, 0.9
    axes = (0,) + tuple(range(2, len(shape)))
    bshape = (1, c) + (1,) * (len(shape) - 2)
    x64, dy64 = x.astype(np.float64), dy.astype(np.float64)
    n = x64.size // c
    mean = x64.mean(axis=axes)
    var = np.maximum((x64 ** 2).mean(axis=axes) - mean ** 2, 0) * n / (n - 1)  # unbiased
    r = 1.0 / np.sqrt(var + eps)
    xm = x64 - mean.reshape(bshape)
    y = xm * r.reshape(bshape) * scale.reshape(bshape) + bias.reshape(bshape)
    dscale = (dy64 * xm * r.reshape(bshape)).sum(axis=axes)
    dbias = dy64.sum(axis=axes)
    dmean = -(dy64 * (scale * r).reshape(bshape)).sum(axis=axes)
    dvar = -(dy64 * scale.reshape(bshape) * xm * (r ** 3 / 2).reshape(bshape)).sum(axis=axes)
    dx = (dy64 * (scale * r).reshape(bshape) + (dmean / n).reshape(bshape)
          + (dvar * 2 / (n - 1)).reshape(bshape) * xm)
    return dict(x=x, dy=dy, scale=scale, bias=bias, mean=mean, var=var,
                running_mean=(1 - decay) * mean, running_var=decay * 1.0 + (1 - decay) * var,
                y=y, dscale=dscale, dbias=dbias, dmean=dmean, dvar=dvar, dx=dx)


def softmax_case(shape, seed):
    rng = np.random.default_rng(seed)
    x = (2.0 * rng.standard_normal(shape)).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(axis=1, keepdims=True))
    y = e / e.sum(axis=1, keepdims=True)
    dx = y * (dy - (y * dy).sum(axis=1, keepdims=True))
    return dict(x=x, dy=dy, y=y, dx=dx)


if __name__ == "__main__":
    np.savez_compressed(os.path.join(HERE, "bn_nchw_2x3x4x5.npz"), **bn_case((2, 3, 4, 5), 101))
    np.savez_compressed(os.path.join(HERE, "bn_ncdhw_2x4x3x5x6.npz"), **bn_case((2, 4, 3, 5, 6), 102))
    np.savez_compressed(os.path.join(HERE, "softmax_2x21x5x7.npz"), **softmax_case((2, 21, 5, 7), 103))
    print("golden fixtures written to", HERE)

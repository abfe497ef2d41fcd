"""Shared helpers of the test-suite (not collected by pytest)."""
from __future__ import annotations

import contextlib

import numpy as np


def rel_metric(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """The reference's comparison metric, max(|d/v1|, |d/v2|) elementwise
    (legacy/tests/compare_binary_files.cpp:47-49); 0 where both are equal."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    d = np.abs(a - b)
    with np.errstate(divide="ignore", invalid="ignore"):
        m = np.maximum(d / np.abs(a), d / np.abs(b))
    m[d == 0] = 0.0
    return m


def max_rel(a, b) -> float:
    m = rel_metric(a, b)
    return float(np.max(m)) if m.size else 0.0


def bn_inputs(shape_ncs, seed, dtype=np.float32):
    """x ~ N(0,1), dy ~ N(0,1), scale ~ U(0.5,1.5), bias ~ N(0,0.1); shape is
    numpy order (N, C, *spatial)."""
    rng = np.random.default_rng(seed)
    c = shape_ncs[1]
    x = rng.standard_normal(shape_ncs).astype(dtype)
    dy = rng.standard_normal(shape_ncs).astype(dtype)
    scale = rng.uniform(0.5, 1.5, c).astype(dtype)
    bias = (0.1 * rng.standard_normal(c)).astype(dtype)
    return x, dy, scale, bias


def glibc_rand(seed: int, count: int) -> np.ndarray:
    """The first ``count`` values of ``srand(seed); rand()`` of the GNU C library (its
    additive-feedback generator of degree 31; ``RAND_MAX`` = 2**31 - 1), restated here so
    that the values do not depend on the C library of the machine and drawing them leaves
    the process's own generator alone.  tests/test_oracle_bn.py pins it on the C library."""
    seed = seed or 1                     # srand(0) seeds with 1
    r = [0] * (344 + count)
    r[0] = seed
    for i in range(1, 31):
        # 16807 * r[i-1] mod (2**31 - 1) on the signed 32-bit value, by Schrage's method
        prev = _to_signed(r[i - 1])
        hi = int(prev / 127773)          # C division: towards zero
        lo = prev - hi * 127773
        word = 16807 * lo - 2836 * hi
        r[i] = (word + 2147483647 if word < 0 else word) & 0xffffffff
    for i in range(31, 34):
        r[i] = r[i - 31]
    for i in range(34, 344 + count):
        r[i] = (r[i - 31] + r[i - 3]) & 0xffffffff
    return np.array([v >> 1 for v in r[344:]], dtype=np.int64)


def _to_signed(v: int) -> int:
    return v - (1 << 32) if v & 0x80000000 else v


def reference_initializer(shape_ncs, seed, num_rands=100, global_shape=None, global_index=None,
                          dtype=np.float32):
    """The input generator of the reference's benchmarks and validation runs
    (legacy/benchmarks/benchmark_common.hpp:46-79, used by distconv_benchmark_bn.cpp:200-213
    with seeds 0 for the input and 2 for d_output): a table of ``num_rands`` values of
    ``rand()``; the element at global index i gets
    (table[sum(i) % num_rands] + table[offset(i) % num_rands]) / 2 / RAND_MAX, its offset taken
    in the global tensor, innermost dimension fastest.  Values lie in [0, 1) with mean 1/2.
    ``shape_ncs``, ``global_shape`` and ``global_index`` are in numpy order (N, C, *spatial)."""
    table = glibc_rand(seed, num_rands).astype(np.float64) / 2147483647.0
    nd = len(shape_ncs)
    gshape = tuple(global_shape) if global_shape is not None else tuple(shape_ncs)
    gidx = tuple(global_index) if global_index is not None else (0,) * nd
    # both table indices are sums of per-axis terms taken modulo num_rands: small integers
    total = np.zeros((1,) * nd, np.int16)
    offset = np.zeros((1,) * nd, np.int16)
    stride = 1
    for axis in range(nd - 1, -1, -1):
        view = [1] * nd
        view[axis] = shape_ncs[axis]
        i = np.arange(shape_ncs[axis], dtype=np.int64) + gidx[axis]
        total = total + (i % num_rands).astype(np.int16).reshape(view)
        offset = offset + ((i * stride) % num_rands).astype(np.int16).reshape(view)
        stride *= gshape[axis]
    # one gather from the table of all pairs, each pair averaged in double and rounded once
    pairs = ((table[:, None] + table[None, :]) / 2).astype(dtype).ravel()
    total %= num_rands
    offset %= num_rands
    index = total.astype(np.int32)
    index *= num_rands
    index += offset
    return pairs[index]


# ---------------------------------------------------------------------------
# virtual ranks on the CPU, driven through the oracle
# ---------------------------------------------------------------------------

def global_offset_field(geom, mod=None):
    """Interior of one rank initialised to the global linear offset of each
    element (legacy/tests/tensor/test_halo_exchange_cuda.cu:43-102); returns
    the interior array in numpy order.  With ``mod`` the offset is hashed into
    [0, mod) so that it stays exactly representable in float32."""
    nd = geom.nd
    idx = np.indices(geom.local_shape[::-1], dtype=np.int64)  # numpy order axes
    off = np.zeros(geom.local_shape[::-1], dtype=np.int64)
    stride = 1
    for d in range(nd):
        off += (idx[nd - 1 - d] + geom.global_index[d]) * stride
        stride *= geom.shape[d]
    if mod is not None:
        off = (off * 2654435761) % mod
    return off


def interior_slices(geom):
    return tuple(slice(o, o + l) for o, l in zip(geom.overlap[::-1], geom.local_shape[::-1]))


def oracle_halo_exchange(oracle, geoms, fields, periodic=False, widths=None, is_reverse=False,
                         op=0):
    """HaloExchange::exchange for all virtual ranks on the CPU
    (legacy/include/distconv/tensor/halo_exchange_cuda.hpp:56-106 with the
    message order of halo_exchange_cuda_mpi.hpp:25-100).  ``fields`` are the
    ranks' real (haloed) arrays, modified in place."""
    from oracle import geometry as G
    nd = geoms[0].nd
    for d in range(nd):
        w = geoms[0].overlap[d] if widths is None else widths[d]
        if w == 0 or geoms[0].dist.split_shape[d] <= 1:
            continue
        recv = {}
        for r, g in enumerate(geoms):
            if g.local_size == 0:
                continue
            for side in (0, 1):
                peer = G.halo_peer(g, d, side, periodic)
                if peer is None:
                    continue
                buf = np.zeros(oracle.halo_size(g.real_shape, d, w), fields[r].dtype)
                oracle.halo_pack_or_unpack(fields[r], d, side, w, buf, True, is_reverse, op)
                recv[(peer, 1 - side)] = buf
        for r, g in enumerate(geoms):
            if g.local_size == 0:
                continue
            for side in (0, 1):
                if G.halo_peer(g, d, side, periodic) is None:
                    continue
                oracle.halo_pack_or_unpack(fields[r], d, side, w, recv[(r, side)], False,
                                           is_reverse, op)


GUARD_ELEMS = 1024   # on either side of a tensor; keeps the tensor's 16-byte alignment
GUARD_BYTE = 0xA5


@contextlib.contextmanager
def guarded_allocations():
    """While active, Tensor.allocate and the buffers the layers own (workspaces, receive buffers,
    the shuffler's arena) lie between two guard zones of GUARD_BYTE each; the allocations are
    recorded in the list this yields (for check_guards)."""
    import torch
    from dihydrogen_amd import tensor as tensor_mod
    allocated = []

    def allocate(self):
        n = max(self.get_local_real_size(), 1)
        whole = torch.zeros(n + 2 * GUARD_ELEMS, dtype=self.dtype, device=self.device)
        raw = whole.view(torch.uint8)
        guard_bytes = GUARD_ELEMS * whole.element_size()
        raw[:guard_bytes] = GUARD_BYTE
        raw[-guard_bytes:] = GUARD_BYTE
        self.data = whole[GUARD_ELEMS:GUARD_ELEMS + n]
        allocated.append((raw, guard_bytes, tuple(self.local_real_shape)))
        return self

    def device_buffer(count, dtype, device="cuda", zero=False):
        whole = torch.zeros(count + 2 * GUARD_ELEMS, dtype=dtype, device=device)
        raw = whole.view(torch.uint8)
        guard_bytes = GUARD_ELEMS * whole.element_size()
        raw[:guard_bytes] = GUARD_BYTE
        raw[-guard_bytes:] = GUARD_BYTE
        allocated.append((raw, guard_bytes, ("buffer", count)))
        return whole[GUARD_ELEMS:GUARD_ELEMS + count]

    from dihydrogen_amd import layers as layers_mod
    original, original_buffer = tensor_mod.Tensor.allocate, layers_mod._device_buffer
    tensor_mod.Tensor.allocate, layers_mod._device_buffer = allocate, device_buffer
    try:
        yield allocated
    finally:
        tensor_mod.Tensor.allocate, layers_mod._device_buffer = original, original_buffer


def check_guards(allocated):
    import torch
    torch.cuda.synchronize()
    for raw, guard_bytes, shape in allocated:
        front = int((raw[:guard_bytes] != GUARD_BYTE).sum())
        back = int((raw[-guard_bytes:] != GUARD_BYTE).sum())
        assert front == 0 and back == 0, \
            f"a kernel wrote outside a tensor of real shape (or a buffer of size) {shape}: {front} bytes in front, {back} behind"


class CopyAudit:
    """A launch audit of the copy entry points (h2x_copy_audit_begin ... _end) around host-layer
    code that runs on CPU tensors: every tensor registered here, and every buffer the layers
    allocate while the audit is open, gets one load and one store counter per byte."""

    def __init__(self):
        self.entries = []     # (torch tensor, loads, stores, region struct): kept alive until the end
        self.report = None

    def __enter__(self):
        from dihydrogen_amd import capi, layers
        self._lib = capi.load()
        capi.check(self._lib.h2x_copy_audit_begin(), "audit begin")
        self._layers, self._original = layers, layers._device_buffer

        def device_buffer(count, dtype, device="cuda", zero=False):
            import torch
            t = torch.zeros(count, dtype=dtype, device="cpu")
            self.register(t)
            self.buffers.append(t)
            return t

        self.buffers = []
        layers._device_buffer = device_buffer
        return self

    def register(self, t):
        import ctypes
        from dihydrogen_amd import capi
        nbytes = t.numel() * t.element_size()
        loads, stores = np.zeros(nbytes, np.uint8), np.zeros(nbytes, np.uint8)
        region = capi.CopyAuditRegion()
        region.base, region.bytes = t.data_ptr(), nbytes
        region.loads = loads.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8))
        region.stores = stores.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8))
        capi.check(self._lib.h2x_copy_audit_add_region(ctypes.byref(region)), "audit region")
        self.entries.append((t, loads, stores, region))

    def counts(self, t):
        """(loads, stores) per element of a registered tensor; all bytes of an element move together."""
        for u, loads, stores, _ in self.entries:
            if u.data_ptr() == t.data_ptr():
                e = u.element_size()
                out = []
                for c in (loads, stores):
                    per = c.reshape(-1, e)
                    assert (per == per[:, :1]).all(), "bytes of one element were moved separately"
                    out.append(per[:, 0].astype(np.int64))
                return out
        raise KeyError("tensor not registered")

    def __exit__(self, *exc):
        import ctypes
        from dihydrogen_amd import capi
        self._layers._device_buffer = self._original
        self.report = capi.CopyAuditReport()
        capi.check(self._lib.h2x_copy_audit_end(ctypes.byref(self.report)), "audit end")
        return False

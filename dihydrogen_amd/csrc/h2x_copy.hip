// Box copy engine for gfx950: halo pack/unpack/clear and tensor-shuffler
// pack/unpack, with the C entry points of both.
//
// Both operations move a rectangular sub-box of a strided tensor to or from a
// contiguous buffer that holds the box in natural (innermost-first) order of
// the box's own extents:
//   - a halo strip is the box {shape[0..dim-1], width, shape[dim+1..]} at the
//     strip's start along `dim` (legacy/include/distconv/tensor/halo_cuda.hpp:34-88);
//   - the part of a local tensor that goes to one peer rank of a shuffle is
//     the intersection box of the two ranks' regions, and the order
//     find_destination produces inside a peer's chunk is the natural order of
//     that box (legacy/src/tensor/shuffle_mpi_cuda.cu:42-98).
// The host reduces every box to as few dimensions as possible (extent-1
// dimensions vanish, dimensions that are contiguous in the tensor merge), so a
// halo strip becomes "outer runs of `run` contiguous elements" and the device
// index arithmetic is one or two multiply-high divisions per 16 bytes moved,
// instead of a division chain per element (halo_cuda.hpp:47-81) or a search
// per element (shuffle_mpi_cuda.cu:70-84).  Up to kMaxBoxes boxes -- both
// sides of a dimension, all peers of a rank, several virtual ranks -- share a
// launch; their descriptors travel in the kernel arguments, so nothing is
// allocated or copied to set a launch up.
//
// A fourth mode moves a strip straight from one tensor into another (the
// neighbour's interior strip into this rank's halo) when both live on the same
// device: pack and unpack of a halo exchange without the buffer in between.
#include "h2x_device.hpp"

#include <algorithm>
#include <cstring>
#include <new>
#include <type_traits>
#include <vector>

namespace h2x
{
namespace
{

constexpr int kMaxBoxes = 16;
constexpr int kMaxBoxDims = H2X_MAX_DIMS;
constexpr int kCopyUnroll = 4;

enum Mode : int
{
    kPack = 0,    // buffer <- tensor
    kUnpack = 1,  // tensor <- op(tensor, buffer)
    kClear = 2,   // tensor <- 0
    kTransfer = 3 // tensor <- op(tensor, source tensor)
};

// One reduced box.  Packed element g (natural order of extent[]) lives at
// tensor[tensor_offset + sum idx[i] * stride[i]].
struct Box
{
    char* tensor;            // base the strides are relative to
    char* buffer;            // start of this box's contiguous image (kTransfer: source box origin)
    char* tensor2;           // second box of identical geometry (sparse pairs), or null
    char* buffer2;
    int64_t stride[kMaxBoxDims]; // elements
    int64_t stride_src[kMaxBoxDims]; // kTransfer: strides of the source tensor
    FastDiv div[kMaxBoxDims];    // by extent[i]; the last used one is never divided by
    uint32_t count;          // elements in the box (< 2^31)
    uint32_t first_block;    // first workgroup of this box in the launch
    int32_t num_dims;
    int32_t mode;            // Mode
};

struct BoxBatch
{
    Box box[kMaxBoxes];
    int32_t num_boxes;
    uint32_t num_blocks;
    uint32_t blocks_per_box; // > 0: the boxes take turns, each for this many workgroups
};

template <typename W, int VEC>
struct Words
{
    typedef W aligned_t __attribute__((ext_vector_type(VEC)));
    typedef W unaligned_t __attribute__((ext_vector_type(VEC), aligned(sizeof(W))));
};

struct OpId
{
    template <typename T>
    __device__ __forceinline__ T operator()(T, T b) const { return b; }
};
struct OpSum
{
    template <typename T>
    __device__ __forceinline__ T operator()(T a, T b) const { return a + b; }
};
struct OpMax
{
    template <typename T>
    __device__ __forceinline__ T operator()(T a, T b) const { return a > b ? a : b; }
};
struct OpMin
{
    template <typename T>
    __device__ __forceinline__ T operator()(T a, T b) const { return a < b ? a : b; }
};

// Loads and stores of "sparse" boxes: runs shorter than a cache line that are
// a row apart (a halo face of the innermost dimension).  Every element costs a
// whole 128-byte line of HBM traffic; stores are write-through so that the
// line is not allocated for a 4-byte write.
template <typename T>
__device__ __forceinline__ void sparse_store_scalar(T* p, T v)
{
    if constexpr (sizeof(T) >= 4)
        __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
        *p = v;
}

// T: element type the op sees (an unsigned integer of the element's size for
// plain copies).  VEC elements of one run move per thread and step; the buffer
// side is VEC-aligned, the tensor side may start on any element.  SPARSE boxes
// come in pairs of identical geometry (the LHS and RHS face of one tensor):
// one thread serves the same index of both, so that neighbouring rows' ends,
// which share a cache line, are touched by neighbouring lanes of one wave.
template <typename T, int VEC, typename Op, bool SPARSE>
__global__ __launch_bounds__(kBlockSize) void box_copy_kernel(const BoxBatch batch, Op op)
{
    // which box does this workgroup belong to?
    // The boxes take turns workgroup by workgroup.  Workgroups go to the eight
    // XCDs round-robin, so with 8 or 16 boxes in a launch every box is served
    // by one XCD, whose L2 then streams one contiguous region (measured: C2
    // exchange 425 -> 403 us, C5 round trip 191 -> 180 us against box after
    // box; rotating the turns so that a box wanders over the XCDs loses the
    // gain again).  A turn beyond the end of a smaller box finds every index
    // out of range and does nothing.  With very unequal boxes they follow one
    // another.
    int b = 0;
    uint32_t local_block;
    if (batch.blocks_per_box != 0)
    {
        b = blockIdx.x % batch.num_boxes;
        local_block = blockIdx.x / batch.num_boxes;
    }
    else
    {
#pragma unroll 1
        for (int i = 1; i < batch.num_boxes; ++i)
            if (blockIdx.x >= batch.box[i].first_block)
                b = i;
        local_block = blockIdx.x - batch.box[b].first_block;
    }
    const Box& box = batch.box[b];
    const uint32_t count = box.count;
    const int nd = box.num_dims;
    const int mode = box.mode;
    using WA = typename Words<T, VEC>::aligned_t;
    using WU = typename Words<T, VEC>::unaligned_t;

    constexpr uint32_t kStride = kBlockSize * VEC;
    const uint32_t block_base = local_block * (kStride * kCopyUnroll);

    int64_t toff[kCopyUnroll];
    int64_t soff[kCopyUnroll]; // kTransfer only: offset in the source tensor
    uint32_t g[kCopyUnroll];
#pragma unroll
    for (int u = 0; u < kCopyUnroll; ++u)
    {
        g[u] = block_base + u * kStride + threadIdx.x * VEC;
        uint32_t rem = g[u];
        int64_t off = 0, src = 0;
#pragma unroll
        for (int i = 0; i < kMaxBoxDims - 1; ++i)
        {
            if (i < nd - 1)
            {
                const uint32_t q = fastdiv(rem, box.div[i]);
                const int64_t idx = rem - q * box.div[i].divisor;
                off += idx * box.stride[i];
                if (mode == kTransfer)
                    src += idx * box.stride_src[i];
                rem = q;
            }
        }
        off += static_cast<int64_t>(rem) * box.stride[nd - 1];
        if (mode == kTransfer)
            src += static_cast<int64_t>(rem) * box.stride_src[nd - 1];
        toff[u] = off;
        soff[u] = src;
    }

    constexpr int kSides = SPARSE ? 2 : 1;
#pragma unroll
    for (int side = 0; side < kSides; ++side)
    {
        T* const tensor = reinterpret_cast<T*>(side == 0 ? box.tensor : box.tensor2);
        T* const buffer = reinterpret_cast<T*>(side == 0 ? box.buffer : box.buffer2);
        if (side == 1 && tensor == nullptr)
            break;
        if (mode == kPack)
        {
            if constexpr (SPARSE)
            {
                // both faces' loads are issued before any store, so that the
                // two touches of a shared line meet in the cache
                if (side == 1)
                    break;
                T* const tensor_b = reinterpret_cast<T*>(box.tensor2);
                T* const buffer_b = reinterpret_cast<T*>(box.buffer2);
                WU va[kCopyUnroll], vb[kCopyUnroll];
#pragma unroll
                for (int u = 0; u < kCopyUnroll; ++u)
                    if (g[u] < count)
                    {
                        va[u] = *reinterpret_cast<const WU*>(tensor + toff[u]);
                        if (tensor_b != nullptr)
                            vb[u] = *reinterpret_cast<const WU*>(tensor_b + toff[u]);
                    }
#pragma unroll
                for (int u = 0; u < kCopyUnroll; ++u)
                    if (g[u] < count)
                    {
                        *reinterpret_cast<WA*>(buffer + g[u]) = va[u];
                        if (tensor_b != nullptr)
                            *reinterpret_cast<WA*>(buffer_b + g[u]) = vb[u];
                    }
            }
            else
            {
                // The tensor is read once and streams past the memory-side
                // cache; the packed image is stored normally so that it is
                // still there when the matching unpack reads it.
                WU v[kCopyUnroll];
#pragma unroll
                for (int u = 0; u < kCopyUnroll; ++u)
                    if (g[u] < count)
                        v[u] = __builtin_nontemporal_load(
                            reinterpret_cast<const WU*>(tensor + toff[u]));
#pragma unroll
                for (int u = 0; u < kCopyUnroll; ++u)
                    if (g[u] < count)
                        *reinterpret_cast<WA*>(buffer + g[u]) = v[u];
            }
        }
        else if (mode == kUnpack)
        {
            WA v[kCopyUnroll];
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u)
                if (g[u] < count)
                    v[u] = __builtin_nontemporal_load(
                        reinterpret_cast<const WA*>(buffer + g[u])); // last use of the image
            if constexpr (std::is_same<Op, OpId>::value)
            {
#pragma unroll
                for (int u = 0; u < kCopyUnroll; ++u)
                    if (g[u] < count)
                    {
                        if constexpr (SPARSE && VEC == 1)
                            sparse_store_scalar(tensor + toff[u], v[u][0]);
                        else
                            __builtin_nontemporal_store(
                                static_cast<WU>(v[u]), reinterpret_cast<WU*>(tensor + toff[u]));
                    }
            }
            else
            {
#pragma unroll
                for (int u = 0; u < kCopyUnroll; ++u)
                    if (g[u] < count)
                    {
                        WU t = *reinterpret_cast<const WU*>(tensor + toff[u]);
#pragma unroll
                        for (int j = 0; j < VEC; ++j)
                            t[j] = op(t[j], v[u][j]);
                        *reinterpret_cast<WU*>(tensor + toff[u]) = t;
                    }
            }
        }
        else if (mode == kTransfer)
        {
            // `buffer` is the origin of the source box in the other tensor
            WU v[kCopyUnroll];
            if constexpr (SPARSE)
            {
                // both faces' loads before any store, as for sparse packs
                if (side == 1)
                    break;
                T* const tensor_b = reinterpret_cast<T*>(box.tensor2);
                const T* const source_b = reinterpret_cast<const T*>(box.buffer2);
                WU w[kCopyUnroll];
#pragma unroll
                for (int u = 0; u < kCopyUnroll; ++u)
                    if (g[u] < count)
                    {
                        v[u] = *reinterpret_cast<const WU*>(buffer + soff[u]);
                        if (tensor_b != nullptr)
                            w[u] = *reinterpret_cast<const WU*>(source_b + soff[u]);
                    }
#pragma unroll
                for (int u = 0; u < kCopyUnroll; ++u)
                    if (g[u] < count)
                    {
                        if constexpr (std::is_same<Op, OpId>::value && VEC == 1)
                        {
                            sparse_store_scalar(tensor + toff[u], v[u][0]);
                            if (tensor_b != nullptr)
                                sparse_store_scalar(tensor_b + toff[u], w[u][0]);
                        }
                        else
                        {
                            WU t = *reinterpret_cast<const WU*>(tensor + toff[u]);
#pragma unroll
                            for (int j = 0; j < VEC; ++j)
                                t[j] = op(t[j], v[u][j]);
                            *reinterpret_cast<WU*>(tensor + toff[u]) = t;
                            if (tensor_b != nullptr)
                            {
                                WU tb = *reinterpret_cast<const WU*>(tensor_b + toff[u]);
#pragma unroll
                                for (int j = 0; j < VEC; ++j)
                                    tb[j] = op(tb[j], w[u][j]);
                                *reinterpret_cast<WU*>(tensor_b + toff[u]) = tb;
                            }
                        }
                    }
            }
            else
            {
#pragma unroll
                for (int u = 0; u < kCopyUnroll; ++u)
                    if (g[u] < count)
                        v[u] = __builtin_nontemporal_load(
                            reinterpret_cast<const WU*>(buffer + soff[u]));
#pragma unroll
                for (int u = 0; u < kCopyUnroll; ++u)
                    if (g[u] < count)
                    {
                        if constexpr (std::is_same<Op, OpId>::value)
                        {
                            __builtin_nontemporal_store(
                                v[u], reinterpret_cast<WU*>(tensor + toff[u]));
                        }
                        else
                        {
                            WU t = *reinterpret_cast<const WU*>(tensor + toff[u]);
#pragma unroll
                            for (int j = 0; j < VEC; ++j)
                                t[j] = op(t[j], v[u][j]);
                            *reinterpret_cast<WU*>(tensor + toff[u]) = t;
                        }
                    }
            }
        }
        else
        {
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u)
                if (g[u] < count)
                {
                    if constexpr (SPARSE && VEC == 1)
                    {
                        sparse_store_scalar(tensor + toff[u], T(0));
                    }
                    else
                    {
                        WU z;
#pragma unroll
                        for (int j = 0; j < VEC; ++j)
                            z[j] = T(0);
                        *reinterpret_cast<WU*>(tensor + toff[u]) = z;
                    }
                }
        }
    }
}

// ---- host: box reduction ------------------------------------------------------

struct HostBox
{
    int nd = 0;
    int64_t extent[kMaxBoxDims];
    int64_t stride[kMaxBoxDims];
    int64_t stride_src[kMaxBoxDims] = {}; // transfers: strides of the source tensor
    int64_t tensor_offset = 0; // elements from the tensor pointer to the box origin
    int64_t buffer_offset = 0; // elements from the buffer (transfers: source tensor) pointer
    int64_t count = 1;
    bool transfer = false;
};

// Drops extent-1 dimensions and merges neighbours that are contiguous in the
// tensor (for a transfer: in both tensors); the natural order of the reduced
// box is the natural order of the original one.
HostBox reduce_box(int nd, const int64_t* extent, const int64_t* stride, int64_t tensor_offset,
                   int64_t buffer_offset, const int64_t* stride_src = nullptr)
{
    HostBox h;
    h.tensor_offset = tensor_offset;
    h.buffer_offset = buffer_offset;
    h.transfer = stride_src != nullptr;
    for (int i = 0; i < nd; ++i)
    {
        h.count *= extent[i];
        if (extent[i] == 1)
            continue;
        const bool merge =
            h.nd > 0 && stride[i] == h.stride[h.nd - 1] * h.extent[h.nd - 1]
            && (!stride_src || stride_src[i] == h.stride_src[h.nd - 1] * h.extent[h.nd - 1]);
        if (merge)
        {
            h.extent[h.nd - 1] *= extent[i];
        }
        else
        {
            h.extent[h.nd] = extent[i];
            h.stride[h.nd] = stride[i];
            h.stride_src[h.nd] = stride_src ? stride_src[i] : 0;
            ++h.nd;
        }
    }
    if (h.nd == 0)
    {
        h.nd = 1;
        h.extent[0] = 1;
        h.stride[0] = 1;
        h.stride_src[0] = 1;
    }
    return h;
}

// Largest power-of-two vector (elements, at most 16 bytes) that never crosses a
// run of the box and keeps the buffer side aligned.
int box_vector(const HostBox& h, int elem_size, const void* buffer)
{
    int v = 16 / elem_size;
    if (h.stride[0] != 1 || (h.transfer && h.stride_src[0] != 1))
        return 1;
    while (v > 1)
    {
        // a transfer has no buffer side: both tensors take unaligned vectors
        const bool ok = h.extent[0] % v == 0
                        && (h.transfer
                            || (h.buffer_offset % v == 0
                                && reinterpret_cast<uintptr_t>(buffer)
                                           % (static_cast<size_t>(v) * elem_size)
                                       == 0));
        if (ok)
            break;
        v /= 2;
    }
    return v;
}

bool same_geometry(const HostBox& a, const HostBox& b)
{
    if (a.nd != b.nd || a.count != b.count)
        return false;
    for (int i = 0; i < a.nd; ++i)
        if (a.extent[i] != b.extent[i] || a.stride[i] != b.stride[i]
            || a.stride_src[i] != b.stride_src[i])
            return false;
    return true;
}

struct Launcher
{
    hipStream_t stream;
    int elem_size;
    h2x_dtype dtype; // meaningful for accumulate ops only
    int op;          // h2x_halo_op
    int vec = 0;
    bool sparse = false;
    HostBox last;         // geometry of the most recently queued box
    int last_mode = -1;
    uint32_t launch_blocks = 0; // workgroups of the launch being issued
    BoxBatch batch;

    Launcher(hipStream_t s, int es, h2x_dtype dt, int o) : stream(s), elem_size(es), dtype(dt), op(o)
    {
        batch.num_boxes = 0;
        batch.num_blocks = 0;
    }

    template <typename T, int VEC>
    int launch_typed()
    {
        const dim3 grid(launch_blocks);
        switch (op)
        {
        case H2X_HALO_ID:
            if (sparse)
                box_copy_kernel<T, VEC, OpId, true><<<grid, kBlockSize, 0, stream>>>(batch, OpId());
            else
                box_copy_kernel<T, VEC, OpId, false><<<grid, kBlockSize, 0, stream>>>(batch, OpId());
            break;
        default: return H2X_ERR_UNSUPPORTED;
        }
        return launch_status();
    }

    template <typename T, int VEC>
    int launch_accumulate()
    {
        const dim3 grid(launch_blocks);
        switch (op)
        {
        case H2X_HALO_SUM:
            if (sparse)
                box_copy_kernel<T, VEC, OpSum, true><<<grid, kBlockSize, 0, stream>>>(batch, OpSum());
            else
                box_copy_kernel<T, VEC, OpSum, false><<<grid, kBlockSize, 0, stream>>>(batch, OpSum());
            break;
        case H2X_HALO_MAX:
            if (sparse)
                box_copy_kernel<T, VEC, OpMax, true><<<grid, kBlockSize, 0, stream>>>(batch, OpMax());
            else
                box_copy_kernel<T, VEC, OpMax, false><<<grid, kBlockSize, 0, stream>>>(batch, OpMax());
            break;
        case H2X_HALO_MIN:
            if (sparse)
                box_copy_kernel<T, VEC, OpMin, true><<<grid, kBlockSize, 0, stream>>>(batch, OpMin());
            else
                box_copy_kernel<T, VEC, OpMin, false><<<grid, kBlockSize, 0, stream>>>(batch, OpMin());
            break;
        default: return H2X_ERR_UNSUPPORTED;
        }
        return launch_status();
    }

    template <typename U, typename F, int V>
    int launch_width()
    {
        if constexpr (!std::is_void<F>::value)
            if (op != H2X_HALO_ID)
                return launch_accumulate<F, V>();
        return launch_typed<U, V>();
    }

    template <typename U, typename F>
    int launch_vec()
    {
        constexpr int kFull = 16 / sizeof(U);
        switch (vec)
        {
        case 8:
            if constexpr (kFull >= 8)
                return launch_width<U, F, 8>();
            break;
        case 4:
            if constexpr (kFull >= 4)
                return launch_width<U, F, 4>();
            break;
        case 2: return launch_width<U, F, 2>();
        case 1: return launch_width<U, F, 1>();
        }
        return H2X_ERR_UNSUPPORTED;
    }

    int flush()
    {
        if (batch.num_boxes == 0)
            return H2X_SUCCESS;
        // Taking turns needs one workgroup count for all boxes: the largest.  The
        // surplus workgroups of smaller boxes find nothing to do; if they would
        // more than double the grid, the boxes follow one another instead.
        batch.blocks_per_box = 0;
        uint32_t grid_blocks = batch.num_blocks;
        if (batch.num_boxes > 1)
        {
            uint32_t most = 0;
            for (int i = 0; i < batch.num_boxes; ++i)
            {
                const uint32_t end = i + 1 < batch.num_boxes ? batch.box[i + 1].first_block
                                                             : batch.num_blocks;
                most = std::max(most, end - batch.box[i].first_block);
            }
            const uint64_t turns = static_cast<uint64_t>(most) * batch.num_boxes;
            if (turns <= 2ull * batch.num_blocks && turns <= 0x7fffffffull)
            {
                batch.blocks_per_box = most;
                grid_blocks = static_cast<uint32_t>(turns);
            }
        }
        launch_blocks = grid_blocks;
        int err;
        switch (elem_size)
        {
        case 2: err = op == H2X_HALO_ID ? launch_vec<uint16_t, void>() : H2X_ERR_UNSUPPORTED; break;
        case 4: err = launch_vec<uint32_t, float>(); break;
        case 8: err = launch_vec<uint64_t, double>(); break;
        default: err = H2X_ERR_UNSUPPORTED;
        }
        batch.num_boxes = 0;
        batch.num_blocks = 0;
        vec = 0;
        last_mode = -1;
        return err;
    }

    // Queues one box; launches what is queued when the batch is full or the
    // new box needs another vector width.
    int add(const HostBox& h, void* tensor, void* buffer, int mode)
    {
        if (h.count == 0)
            return H2X_SUCCESS;
        if (h.count >= (1ll << 31))
            return H2X_ERR_TOO_LARGE;
        const int v = mode == kClear ? box_vector(h, elem_size, nullptr) : box_vector(h, elem_size, buffer);
        // sparse: every run is shorter than a cache line and the runs are apart
        const bool sp = h.nd > 1 ? h.extent[0] * h.stride[0] * elem_size < 128
                                 : (h.stride[0] != 1 && h.extent[0] > 1);
        char* const tptr = static_cast<char*>(tensor) + h.tensor_offset * elem_size;
        char* const bptr = static_cast<char*>(buffer) + h.buffer_offset * elem_size;
        // second box of a sparse pair: same geometry and mode as the box queued last
        if (sp && batch.num_boxes > 0 && sparse && v == vec && last_mode == mode
            && batch.box[batch.num_boxes - 1].tensor2 == nullptr && same_geometry(h, last))
        {
            batch.box[batch.num_boxes - 1].tensor2 = tptr;
            batch.box[batch.num_boxes - 1].buffer2 = bptr;
            return H2X_SUCCESS;
        }
        if (batch.num_boxes == kMaxBoxes || (batch.num_boxes > 0 && (v != vec || sp != sparse)))
        {
            const int err = flush();
            if (err != 0)
                return err;
        }
        vec = v;
        sparse = sp;
        last = h;
        last_mode = mode;
        Box& b = batch.box[batch.num_boxes];
        b.tensor = tptr;
        b.buffer = bptr;
        b.tensor2 = nullptr;
        b.buffer2 = nullptr;
        for (int i = 0; i < kMaxBoxDims; ++i)
        {
            b.stride[i] = i < h.nd ? h.stride[i] : 0;
            b.stride_src[i] = i < h.nd ? h.stride_src[i] : 0;
            b.div[i] = make_fastdiv(i < h.nd ? static_cast<uint32_t>(h.extent[i]) : 1u);
        }
        b.count = static_cast<uint32_t>(h.count);
        b.first_block = batch.num_blocks;
        b.num_dims = h.nd;
        b.mode = mode;
        const uint64_t per_block = static_cast<uint64_t>(kBlockSize) * v * kCopyUnroll;
        const uint64_t blocks = (static_cast<uint64_t>(h.count) + per_block - 1) / per_block;
        if (batch.num_blocks + blocks > 0x7fffffffull)
            return H2X_ERR_TOO_LARGE;
        batch.num_blocks += static_cast<uint32_t>(blocks);
        ++batch.num_boxes;
        return H2X_SUCCESS;
    }
};

int elem_size_of(h2x_dtype dtype)
{
    return dtype == H2X_F32 ? 4 : dtype == H2X_F64 ? 8 : 0;
}

// The strip of a halo face as a box over the real tensor.
int halo_box(const h2x_halo_face& f, HostBox* out, bool origin_only = false)
{
    const int nd = f.num_dims;
    if (nd < 1 || nd > H2X_MAX_DIMS || f.dim < 0 || f.dim >= nd || f.width < 0
        || (f.side != H2X_LHS && f.side != H2X_RHS))
        return H2X_ERR_INVALID_ARGUMENT;
    int64_t extent[kMaxBoxDims], stride[kMaxBoxDims];
    int64_t s = 1;
    for (int i = 0; i < nd; ++i)
    {
        if (f.real_shape[i] < 0)
            return H2X_ERR_INVALID_ARGUMENT;
        extent[i] = f.real_shape[i];
        stride[i] = s;
        s *= f.real_shape[i];
    }
    const int64_t len = f.real_shape[f.dim];
    const int64_t w = f.width;
    int64_t start;
    if (f.side == H2X_RHS)
        start = f.inner ? len - 2 * w : len - w;
    else
        start = f.inner ? w : 0;
    if (w > 0 && (start < 0 || start + w > len))
        return H2X_ERR_INVALID_ARGUMENT;
    extent[f.dim] = w;
    if (origin_only)
    {
        *out = HostBox();
        out->tensor_offset = start * stride[f.dim];
        return H2X_SUCCESS;
    }
    *out = reduce_box(nd, extent, stride, start * stride[f.dim], 0);
    return H2X_SUCCESS;
}

} // namespace
} // namespace h2x

using namespace h2x;

// ---- halo ----------------------------------------------------------------------

extern "C" size_t h2x_halo_size(int num_dims, const int64_t* real_shape, int dim, int width)
{
    size_t s = 1;
    for (int i = 0; i < num_dims; ++i)
        s *= static_cast<size_t>(i == dim ? width : real_shape[i]);
    return s;
}

extern "C" int h2x_halo_pack_or_unpack_batched(h2x_dtype dtype, const h2x_halo_face* faces,
                                               int num_faces, h2x_stream_t stream)
{
    const int es = elem_size_of(dtype);
    if (es == 0)
        return H2X_ERR_UNSUPPORTED;
    if (num_faces < 0 || (num_faces > 0 && !faces))
        return H2X_ERR_INVALID_ARGUMENT;
    // validate everything before anything is launched
    std::vector<HostBox> boxes(num_faces);
    for (int i = 0; i < num_faces; ++i)
    {
        const int err = halo_box(faces[i], &boxes[i]);
        if (err != 0)
            return err;
        if (boxes[i].count > 0 && (!faces[i].tensor || !faces[i].buffer))
            return H2X_ERR_INVALID_ARGUMENT;
        if (boxes[i].count >= (1ll << 31))
            return H2X_ERR_TOO_LARGE;
        if (faces[i].op < H2X_HALO_ID || faces[i].op > H2X_HALO_MIN)
            return H2X_ERR_INVALID_ARGUMENT;
    }
    // faces with the same effective op share launches
    for (int op = H2X_HALO_ID; op <= H2X_HALO_MIN; ++op)
    {
        Launcher l(as_stream(stream), es, dtype, op);
        for (int i = 0; i < num_faces; ++i)
        {
            const int eff = faces[i].is_pack ? H2X_HALO_ID : faces[i].op;
            if (eff != op)
                continue;
            const int err = l.add(boxes[i], faces[i].tensor, faces[i].buffer,
                                  faces[i].is_pack ? kPack : kUnpack);
            if (err != 0)
                return err;
        }
        const int err = l.flush();
        if (err != 0)
            return err;
    }
    return H2X_SUCCESS;
}

extern "C" int h2x_halo_pack_or_unpack(h2x_dtype dtype, void* tensor, int num_dims,
                                       const int64_t* real_shape, int dim, int side, int width,
                                       void* buffer, int is_pack, int is_reverse, int op,
                                       h2x_stream_t stream)
{
    if (width == 0)
        return H2X_SUCCESS; // halo_packing_cuda.hpp:153-154
    if (!real_shape || num_dims < 1 || num_dims > H2X_MAX_DIMS)
        return H2X_ERR_INVALID_ARGUMENT;
    h2x_halo_face f;
    std::memset(&f, 0, sizeof(f));
    f.tensor = tensor;
    f.buffer = buffer;
    for (int i = 0; i < num_dims; ++i)
        f.real_shape[i] = real_shape[i];
    f.num_dims = num_dims;
    f.dim = dim;
    f.side = side;
    f.width = width;
    f.inner = ((is_pack && !is_reverse) || (!is_pack && is_reverse)) ? 1 : 0;
    f.is_pack = is_pack ? 1 : 0;
    f.op = op;
    return h2x_halo_pack_or_unpack_batched(dtype, &f, 1, stream);
}

extern "C" int h2x_halo_clear(h2x_dtype dtype, void* tensor, int num_dims,
                              const int64_t* real_shape, int dim, int width, h2x_stream_t stream)
{
    const int es = elem_size_of(dtype);
    if (es == 0)
        return H2X_ERR_UNSUPPORTED;
    if (width == 0)
        return H2X_SUCCESS;
    if (!tensor || !real_shape || num_dims < 1 || num_dims > H2X_MAX_DIMS)
        return H2X_ERR_INVALID_ARGUMENT;
    Launcher l(as_stream(stream), es, dtype, H2X_HALO_ID);
    for (int side = 0; side < 2; ++side)
    {
        h2x_halo_face f;
        std::memset(&f, 0, sizeof(f));
        for (int i = 0; i < num_dims; ++i)
            f.real_shape[i] = real_shape[i];
        f.num_dims = num_dims;
        f.dim = dim;
        f.side = side;
        f.width = width;
        f.inner = 0;
        HostBox h;
        int err = halo_box(f, &h);
        if (err != 0)
            return err;
        err = l.add(h, tensor, nullptr, kClear);
        if (err != 0)
            return err;
    }
    return l.flush();
}

extern "C" int h2x_halo_exchange_fused(h2x_dtype dtype, const h2x_halo_transfer* transfers,
                                       int num_transfers, h2x_stream_t stream)
{
    const int es = elem_size_of(dtype);
    if (es == 0)
        return H2X_ERR_UNSUPPORTED;
    if (num_transfers < 0 || (num_transfers > 0 && !transfers))
        return H2X_ERR_INVALID_ARGUMENT;
    // validate everything before anything is launched
    std::vector<HostBox> boxes(num_transfers);
    for (int i = 0; i < num_transfers; ++i)
    {
        const h2x_halo_transfer& t = transfers[i];
        if (t.op < H2X_HALO_ID || t.op > H2X_HALO_MIN
            || (t.src_side != H2X_LHS && t.src_side != H2X_RHS))
            return H2X_ERR_INVALID_ARGUMENT;
        // the strip as pack sees it in src and as unpack sees it in dst
        h2x_halo_face from, to;
        std::memset(&from, 0, sizeof(from));
        std::memset(&to, 0, sizeof(to));
        from.num_dims = to.num_dims = t.num_dims;
        from.dim = to.dim = t.dim;
        from.width = to.width = t.width;
        from.side = t.src_side;
        to.side = t.src_side == H2X_LHS ? H2X_RHS : H2X_LHS;
        from.inner = t.is_reverse ? 0 : 1;
        to.inner = t.is_reverse ? 1 : 0;
        if (t.num_dims < 1 || t.num_dims > H2X_MAX_DIMS)
            return H2X_ERR_INVALID_ARGUMENT;
        for (int d = 0; d < t.num_dims; ++d)
        {
            from.real_shape[d] = t.src_real_shape[d];
            to.real_shape[d] = t.dst_real_shape[d];
            if (d != t.dim && t.src_real_shape[d] != t.dst_real_shape[d])
                return H2X_ERR_INVALID_ARGUMENT;
        }
        HostBox a, b;
        int err = halo_box(from, &a, true);
        if (err == 0)
            err = halo_box(to, &b, true);
        if (err != 0)
            return err;
        // same extents, two sets of strides
        int64_t extent[kMaxBoxDims], stride_dst[kMaxBoxDims], stride_src[kMaxBoxDims];
        int64_t sd = 1, ss = 1;
        for (int d = 0; d < t.num_dims; ++d)
        {
            extent[d] = d == t.dim ? t.width : t.dst_real_shape[d];
            stride_dst[d] = sd;
            stride_src[d] = ss;
            sd *= t.dst_real_shape[d];
            ss *= t.src_real_shape[d];
        }
        boxes[i] = reduce_box(t.num_dims, extent, stride_dst, b.tensor_offset, a.tensor_offset,
                              stride_src);
        if (boxes[i].count > 0 && (!t.src || !t.dst))
            return H2X_ERR_INVALID_ARGUMENT;
        if (boxes[i].count >= (1ll << 31))
            return H2X_ERR_TOO_LARGE;
    }
    for (int op = H2X_HALO_ID; op <= H2X_HALO_MIN; ++op)
    {
        Launcher l(as_stream(stream), es, dtype, op);
        for (int i = 0; i < num_transfers; ++i)
        {
            if (transfers[i].op != op)
                continue;
            const int err = l.add(boxes[i], transfers[i].dst, const_cast<void*>(transfers[i].src),
                                  kTransfer);
            if (err != 0)
                return err;
        }
        const int err = l.flush();
        if (err != 0)
            return err;
    }
    return H2X_SUCCESS;
}

// ---- shuffle -------------------------------------------------------------------

struct h2x_shuffle_plan
{
    int elem_size;
    std::vector<HostBox> boxes; // one per peer with a non-empty intersection
};

extern "C" int h2x_shuffle_plan_create(const h2x_shuffle_geometry* g, h2x_shuffle_plan** plan)
{
    if (!g || !plan)
        return H2X_ERR_INVALID_ARGUMENT;
    *plan = nullptr;
    const int nd = g->num_dims;
    if (nd < 1 || nd > H2X_MAX_DIMS || !g->rank_limits || !g->displs)
        return H2X_ERR_INVALID_ARGUMENT;
    if (g->elem_size != 2 && g->elem_size != 4 && g->elem_size != 8)
        return H2X_ERR_UNSUPPORTED;
    int64_t num_peers = 1;
    for (int i = 0; i < nd; ++i)
    {
        if (g->local_shape[i] < 0 || g->peer_locale_shape[i] < 1 || g->strides[i] < 0)
            return H2X_ERR_INVALID_ARGUMENT;
        num_peers *= g->peer_locale_shape[i];
    }
    // limits must be non-decreasing and end at the local extent
    {
        int rl = 0;
        for (int i = 0; i < nd; ++i)
        {
            int prev = 0;
            for (int j = 0; j < g->peer_locale_shape[i]; ++j)
            {
                const int lim = g->rank_limits[rl + j];
                if (lim < prev || lim > g->local_shape[i])
                    return H2X_ERR_INVALID_ARGUMENT;
                prev = lim;
            }
            if (prev != g->local_shape[i] && g->local_shape[i] != 0)
                return H2X_ERR_INVALID_ARGUMENT;
            rl += static_cast<int>(g->peer_locale_shape[i]);
        }
    }
    h2x_shuffle_plan* p = new (std::nothrow) h2x_shuffle_plan;
    if (!p)
        return static_cast<int>(hipErrorOutOfMemory);
    p->elem_size = g->elem_size;
    for (int64_t peer = 0; peer < num_peers; ++peer)
    {
        int64_t extent[kMaxBoxDims], rem = peer, origin = 0;
        int rl = 0;
        bool empty = false;
        for (int i = 0; i < nd; ++i)
        {
            const int j = static_cast<int>(rem % g->peer_locale_shape[i]);
            rem /= g->peer_locale_shape[i];
            const int lo = j == 0 ? 0 : g->rank_limits[rl + j - 1];
            const int hi = g->rank_limits[rl + j];
            extent[i] = hi - lo;
            origin += static_cast<int64_t>(lo) * g->strides[i];
            empty = empty || extent[i] <= 0;
            rl += static_cast<int>(g->peer_locale_shape[i]);
        }
        if (empty)
            continue;
        HostBox h = reduce_box(nd, extent, g->strides, origin, g->displs[peer]);
        if (h.count >= (1ll << 31))
        {
            delete p;
            return H2X_ERR_TOO_LARGE;
        }
        p->boxes.push_back(h);
    }
    *plan = p;
    return H2X_SUCCESS;
}

extern "C" int h2x_shuffle_plan_destroy(h2x_shuffle_plan* plan)
{
    delete plan;
    return H2X_SUCCESS;
}

static int shuffle_batched(const h2x_shuffle_plan* const* plans, void* const* tensors,
                           void* const* buffers, int num_plans, int mode, h2x_stream_t stream)
{
    if (num_plans < 0 || (num_plans > 0 && (!plans || !tensors || !buffers)))
        return H2X_ERR_INVALID_ARGUMENT;
    for (int i = 0; i < num_plans; ++i)
    {
        if (!plans[i])
            return H2X_ERR_INVALID_ARGUMENT;
        if (!plans[i]->boxes.empty() && (!tensors[i] || !buffers[i]))
            return H2X_ERR_INVALID_ARGUMENT;
    }
    for (int es : {2, 4, 8})
    {
        Launcher l(as_stream(stream), es, H2X_F32, H2X_HALO_ID);
        for (int i = 0; i < num_plans; ++i)
        {
            if (plans[i]->elem_size != es)
                continue;
            for (const HostBox& h : plans[i]->boxes)
            {
                const int err = l.add(h, tensors[i], buffers[i], mode);
                if (err != 0)
                    return err;
            }
        }
        const int err = l.flush();
        if (err != 0)
            return err;
    }
    return H2X_SUCCESS;
}

extern "C" int h2x_shuffle_pack(const h2x_shuffle_plan* plan, const void* tensor, void* buffer,
                                h2x_stream_t stream)
{
    void* t = const_cast<void*>(tensor);
    return shuffle_batched(&plan, &t, &buffer, 1, kPack, stream);
}

extern "C" int h2x_shuffle_unpack(const h2x_shuffle_plan* plan, void* tensor, const void* buffer,
                                  h2x_stream_t stream)
{
    void* b = const_cast<void*>(buffer);
    return shuffle_batched(&plan, &tensor, &b, 1, kUnpack, stream);
}

extern "C" int h2x_shuffle_pack_batched(const h2x_shuffle_plan* const* plans,
                                        const void* const* tensors, void* const* buffers,
                                        int num_plans, h2x_stream_t stream)
{
    return shuffle_batched(plans, const_cast<void* const*>(tensors), buffers, num_plans, kPack, stream);
}

extern "C" int h2x_shuffle_unpack_batched(const h2x_shuffle_plan* const* plans,
                                          void* const* tensors, const void* const* buffers,
                                          int num_plans, h2x_stream_t stream)
{
    return shuffle_batched(plans, tensors, const_cast<void* const*>(buffers), num_plans, kUnpack, stream);
}

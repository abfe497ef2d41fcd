// The box copy kernel of the halo and shuffle entry points, and the launch
// descriptors it reads.
//
// Every operation moves a rectangular sub-box of a strided tensor to or from a
// contiguous image that holds the box in natural (innermost-first) order of the
// box's own extents.  The host has reduced each box to as few dimensions as
// possible, so the device index arithmetic is a short chain of multiply-high
// divisions per 16 bytes moved.
//
// Descriptors reach the kernel in one of two ways.  Up to kMaxBoxes boxes
// travel in the kernel arguments (halo strips: their tensors, buffers and
// widths change from call to call, and nothing may be allocated or copied to
// set a launch up).  A shuffle plan keeps its boxes in a device table built
// once at plan creation; a launch then names up to kMaxPlans tables plus the
// tensor and buffer each one applies to, so any number of peers and virtual
// ranks share one launch.
#pragma once

#include "h2x_device.hpp"

#include <type_traits>
#include <vector>

namespace h2x
{
namespace copy
{

constexpr int kMaxBoxes = 16;
constexpr int kMaxPlans = 64;
constexpr int kMaxBoxDims = H2X_MAX_DIMS;
// Threads per workgroup and 16-byte vectors per thread.  One vector per thread
// and many small workgroups beat fewer, longer-lived ones on every shape
// measured (8 x 130^3 x 32 halo exchange: 365 us with four vectors per thread,
// 362 with two, 343 with one; 134 MB shuffle round trip: 177 / 168 / 161 us).
constexpr int kCopyBlock = 256;
constexpr int kCopyUnroll = 1;

enum Mode : int
{
    kPack = 0,    // buffer <- tensor
    kUnpack = 1,  // tensor <- op(tensor, buffer)
    kClear = 2,   // tensor <- 0
    kTransfer = 3 // tensor <- op(tensor, source tensor)
};

// One reduced box.  Packed element g (natural order of the extents) lives at
// tensor[sum idx[i] * stride[i]].  Dimensions beyond the box's own have extent
// 1 and stride 0, so the index chain needs no dimension count; `deep` says
// whether any dimension beyond the third is in use.
struct Box
{
    char* tensor;  // origin of the box (table entries: byte offset from the plan's tensor)
    char* buffer;  // start of the contiguous image (kTransfer: origin of the source box)
    char* tensor2; // second box of identical geometry (sparse pairs), or null
    char* buffer2;
    int64_t stride[kMaxBoxDims];     // elements
    int64_t stride_src[kMaxBoxDims]; // kTransfer: strides of the source tensor
    FastDiv div[kMaxBoxDims];        // by extent[i]
    uint32_t count;                  // elements in the box (< 2^31)
    uint32_t first_block;            // first workgroup of this box when boxes follow one another
    // ragged: the runs of the box (extent of its first dimension) are not a
    // multiple of the vector width, so a vector may straddle the end of a run
    // or of the box; its two parts then move element by element.
    // seam (sparse pairs that unpack): the second box's element of row r sits
    // directly in front of the first box's element of row r + 1 (the RHS and
    // the LHS halo cell at a row seam): both are written with one store.
    // disjoint (sparse pairs): the two boxes have no element in common.
    uint8_t ragged;
    uint8_t seam;
    uint8_t deep;
    uint8_t disjoint;
};

struct BoxBatch
{
    Box box[kMaxBoxes];
    int32_t num_boxes;
    uint32_t blocks_per_box; // > 0: the boxes take turns, each for this many workgroups
};

struct PlanRef
{
    const Box* table;   // device memory
    char* tensor;       // what the table's tensor offsets are relative to
    char* buffer;
    uint32_t first_box; // index of this plan's first box among all boxes of the launch
    uint32_t reserved;
};

struct TableBatch
{
    PlanRef plan[kMaxPlans];
    int32_t num_plans;
    uint32_t num_boxes;      // over all plans
    uint32_t blocks_per_box; // the boxes always take turns
    uint32_t reserved;
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
    __host__ __device__ __forceinline__ T operator()(T, T b) const { return b; }
};
struct OpSum
{
    template <typename T>
    __host__ __device__ __forceinline__ T operator()(T a, T b) const { return a + b; }
};
struct OpMax
{
    template <typename T>
    __host__ __device__ __forceinline__ T operator()(T a, T b) const { return a > b ? a : b; }
};
struct OpMin
{
    template <typename T>
    __host__ __device__ __forceinline__ T operator()(T a, T b) const { return a < b ? a : b; }
};

#ifdef __HIPCC__

// Offset of packed element g of a box in its tensor (and, for transfers, in
// the source tensor); `first` receives the index along the first dimension.
template <bool TRANSFER>
__host__ __device__ __forceinline__ void box_offsets(const Box& box, uint32_t g, int64_t* toff, int64_t* soff,
                                            uint32_t* first)
{
    uint32_t rem = g;
    int64_t off = 0, src = 0;
    auto level = [&](int i) {
        const uint32_t q = fastdiv(rem, box.div[i]);
        const uint32_t idx = rem - q * box.div[i].divisor;
        if (i == 0)
            *first = idx;
        off += static_cast<int64_t>(idx) * box.stride[i];
        if constexpr (TRANSFER)
            src += static_cast<int64_t>(idx) * box.stride_src[i];
        rem = q;
    };
    level(0);
    level(1);
    if (box.deep) // uniform over the workgroup
    {
        level(2);
        level(3);
        level(4);
        off += static_cast<int64_t>(rem) * box.stride[5];
        if constexpr (TRANSFER)
            src += static_cast<int64_t>(rem) * box.stride_src[5];
    }
    else
    {
        off += static_cast<int64_t>(rem) * box.stride[2];
        if constexpr (TRANSFER)
            src += static_cast<int64_t>(rem) * box.stride_src[2];
    }
    *toff = off;
    *soff = src;
}

// How the kernel body below reaches memory: VEC elements at an element
// pointer, aligned to the whole vector or to one element.  The kernel uses
// DeviceMem; the launch audit plays the same body on the CPU with an accessor
// that records addresses instead of following them (h2x_copy_audit.hip).
// (The accessor takes element pointers and names the vector types itself: an
// under-aligned vector type passed as a deduced template argument would lose
// its alignment.)
struct DeviceMem
{
    template <int VEC, bool ALIGNED, typename T>
    __device__ __forceinline__ typename Words<T, VEC>::unaligned_t load(const T* p) const
    {
        if constexpr (ALIGNED)
            return *reinterpret_cast<const typename Words<T, VEC>::aligned_t*>(p);
        else
            return *reinterpret_cast<const typename Words<T, VEC>::unaligned_t*>(p);
    }
    // a load whose data is not needed again (nontemporal)
    template <int VEC, bool ALIGNED, typename T>
    __device__ __forceinline__ typename Words<T, VEC>::unaligned_t load_last_use(const T* p) const
    {
        if constexpr (ALIGNED)
            return __builtin_nontemporal_load(reinterpret_cast<const typename Words<T, VEC>::aligned_t*>(p));
        else
            return __builtin_nontemporal_load(reinterpret_cast<const typename Words<T, VEC>::unaligned_t*>(p));
    }
    template <int VEC, bool ALIGNED, typename T>
    __device__ __forceinline__ void store(T* p, typename Words<T, VEC>::unaligned_t v) const
    {
        if constexpr (ALIGNED)
            *reinterpret_cast<typename Words<T, VEC>::aligned_t*>(p) = v;
        else
            *reinterpret_cast<typename Words<T, VEC>::unaligned_t*>(p) = v;
    }
    template <typename T>
    __device__ __forceinline__ T load1(const T* p) const { return *p; }
    template <typename T>
    __device__ __forceinline__ T load1_last_use(const T* p) const { return __builtin_nontemporal_load(p); }
    template <typename T>
    __device__ __forceinline__ void store1(T* p, T v) const { *p = v; }
};

// Stores (identity) or folds (any other op) the vectors `va` / `vb` into the
// tensor at `pa` / `pb` (`pb` null: a single box).  When the two boxes of a
// pair share no element (`disjoint`), both tensor vectors are loaded before
// either is stored: one trip to memory instead of two in a row (reverse SUM
// exchange of the innermost dimension, 2 ranks a launch: 73 us -> 45 us).
template <typename T, int VEC, typename WU, typename Op, bool IDENTITY, typename Mem>
__host__ __device__ __forceinline__ void accumulate_pair(T* pa, T* pb, WU va, WU vb, bool disjoint, Op op,
                                                         const Mem& mem)
{
    if constexpr (IDENTITY)
    {
        mem.template store<VEC, false>(pa, va);
        if (pb != nullptr)
            mem.template store<VEC, false>(pb, vb);
    }
    else if (pb == nullptr)
    {
        WU ta = mem.template load<VEC, false>(pa);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            ta[j] = op(ta[j], va[j]);
        mem.template store<VEC, false>(pa, ta);
    }
    else if (disjoint)
    {
        WU ta = mem.template load<VEC, false>(pa);
        WU tb = mem.template load<VEC, false>(pb);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
        {
            ta[j] = op(ta[j], va[j]);
            tb[j] = op(tb[j], vb[j]);
        }
        mem.template store<VEC, false>(pa, ta);
        mem.template store<VEC, false>(pb, tb);
    }
    else
    {
        // the boxes may share elements: the second fold sees the first one's result
        WU ta = mem.template load<VEC, false>(pa);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            ta[j] = op(ta[j], va[j]);
        mem.template store<VEC, false>(pa, ta);
        WU tb = mem.template load<VEC, false>(pb);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            tb[j] = op(tb[j], vb[j]);
        mem.template store<VEC, false>(pb, tb);
    }
}

// T: element type the op sees (an unsigned integer of the element's size for
// plain copies).  VEC elements of one run move per thread and step; the image
// side is VEC-aligned, the tensor side may start on any element.  SPARSE boxes
// (runs shorter than a cache line, a row apart: faces of the innermost
// dimension) come in pairs of identical geometry, the LHS and RHS face of one
// tensor: one thread serves the same index of both, so that neighbouring rows'
// ends, which share a cache line, are touched by neighbouring lanes of a wave.
// All boxes of a launch share MODE.  TABLE: descriptors come from plan tables.
//
// Cache policy.  The packed image is stored normally and read back with a
// last-use load, so the memory-side cache serves it between pack and unpack.
// What is written into a tensor is stored normally: strips rarely fill whole
// cache lines, and a write-back cache merges them into the lines it still
// holds from the pack that read their neighbours, where a streaming or
// write-through store costs a partial write to memory each (innermost-
// dimension phase of 8 ranks of 130^3 x 32: 347 us -> 275 us; unpack of 520-
// byte rows: 22 us -> 14 us).  Tensor reads of plan tables (whole-tensor
// redistributions, hundreds of MB) stream past the caches with nontemporal
// loads (shuffle round trip 205 us -> 172 us); halo strips are tens of MB,
// often still cached from the kernel that produced them, and use plain loads
// (a 69 MB launch: 16 us -> 12 us when the strips are cached, no difference
// when they are not).
template <typename T, int VEC, typename Op, bool SPARSE, int MODE, bool TABLE, typename Mem>
__host__ __device__ __forceinline__ void box_copy_body(
    const typename std::conditional<TABLE, TableBatch, BoxBatch>::type& batch, Op op, const uint32_t block,
    const uint32_t thread, const Mem& mem)
{
    using WA = typename Words<T, VEC>::aligned_t;
    using WU = typename Words<T, VEC>::unaligned_t;
    constexpr bool kIdentity = std::is_same<Op, OpId>::value;
    constexpr bool kTransferMode = MODE == kTransfer;

    // Which box does this workgroup belong to?  The boxes take turns workgroup
    // by workgroup.  Workgroups go to the eight XCDs round-robin, so with 8 or
    // 16 boxes in a launch every box is served by one XCD, whose L2 then
    // streams one contiguous region (C2 exchange 425 -> 403 us, C5 round trip
    // 191 -> 180 us against box after box).  A turn beyond the end of a smaller
    // box finds every index out of range and does nothing.  Very unequal boxes
    // follow one another instead (kernel arguments only).
    const Box* entry;
    uint32_t local_block;
    char* tensor_base = nullptr;
    char* buffer_base = nullptr;
    if constexpr (TABLE)
    {
        const uint32_t gb = block % batch.num_boxes;
        local_block = block / batch.num_boxes;
        int p = 0;
#pragma unroll 1
        for (int i = 1; i < batch.num_plans; ++i)
            if (gb >= batch.plan[i].first_box)
                p = i;
        entry = batch.plan[p].table + (gb - batch.plan[p].first_box);
        tensor_base = batch.plan[p].tensor;
        buffer_base = batch.plan[p].buffer;
    }
    else
    {
        int b = 0;
        if (batch.blocks_per_box != 0)
        {
            b = block % batch.num_boxes;
            local_block = block / batch.num_boxes;
        }
        else
        {
#pragma unroll 1
            for (int i = 1; i < batch.num_boxes; ++i)
                if (block >= batch.box[i].first_block)
                    b = i;
            local_block = block - batch.box[b].first_block;
        }
        entry = &batch.box[b];
    }
    // The descriptor is read once, up front and before any store of this
    // kernel, so that it comes in through scalar loads and stays in registers.
    const Box box = *entry;
    const uint32_t count = box.count;

    constexpr uint32_t kStride = kCopyBlock * VEC;
    const uint32_t block_base = local_block * (kStride * kCopyUnroll);
    if (block_base >= count)
        return;

    int64_t toff[kCopyUnroll];
    int64_t soff[kCopyUnroll]; // kTransfer only: offset in the source tensor
    uint32_t g[kCopyUnroll];
    uint32_t head[kCopyUnroll]; // elements of the vector that lie in its first run and in the box
#pragma unroll
    for (int u = 0; u < kCopyUnroll; ++u)
    {
        g[u] = block_base + u * kStride + thread * VEC;
        uint32_t first = 0;
        box_offsets<kTransferMode>(box, g[u], &toff[u], &soff[u], &first);
        head[u] = VEC;
        if constexpr (VEC > 1 && !SPARSE)
            if (box.ragged)
            {
                const uint32_t in_run = box.div[0].divisor - first;
                const uint32_t in_box = g[u] < count ? count - g[u] : 0;
                head[u] = in_run < in_box ? in_run : in_box;
                if (head[u] > VEC)
                    head[u] = VEC;
            }
    }
    (void) head;

    if constexpr (SPARSE)
    {
        // ---- pairs of sparse boxes ---------------------------------------------
        T* const tensor_a = reinterpret_cast<T*>(box.tensor);
        T* const tensor_b = reinterpret_cast<T*>(box.tensor2); // null: a single box
        T* const buffer_a = reinterpret_cast<T*>(box.buffer);
        T* const buffer_b = reinterpret_cast<T*>(box.buffer2);
        if constexpr (MODE == kPack || MODE == kTransfer)
        {
            // both faces' loads are issued before any store, so that the two
            // touches of a shared line meet in the cache; for a transfer
            // `buffer` is the origin of the source box in the other tensor
            WU va[kCopyUnroll], vb[kCopyUnroll];
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u)
                if (g[u] < count)
                {
                    const int64_t at = MODE == kPack ? toff[u] : soff[u];
                    const T* const from_a = MODE == kPack ? tensor_a : buffer_a;
                    const T* const from_b = MODE == kPack ? tensor_b : buffer_b;
                    va[u] = mem.template load<VEC, false>(from_a + at);
                    if (tensor_b != nullptr)
                        vb[u] = mem.template load<VEC, false>(from_b + at);
                }
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u)
                if (g[u] < count)
                {
                    if constexpr (MODE == kPack)
                    {
                        mem.template store<VEC, true>(buffer_a + g[u], va[u]);
                        if (tensor_b != nullptr)
                            mem.template store<VEC, true>(buffer_b + g[u], vb[u]);
                    }
                    else
                    {
                        accumulate_pair<T, VEC, WU, Op, kIdentity, Mem>(tensor_a + toff[u], tensor_b != nullptr ? tensor_b + toff[u] : nullptr,
                                                                   va[u], vb[u], box.disjoint, op, mem);
                    }
                }
        }
        else if constexpr (MODE == kUnpack)
        {
            if (VEC == 1 && box.seam)
            {
                // thread g: element g of the second box and element g + 1 of the
                // first one are neighbours in memory and leave in one store
                typedef T Seam __attribute__((ext_vector_type(2), aligned(sizeof(T))));
                T hi[kCopyUnroll], lo[kCopyUnroll];
#pragma unroll
                for (int u = 0; u < kCopyUnroll; ++u)
                    if (g[u] < count)
                    {
                        hi[u] = mem.load1_last_use(buffer_b + g[u]);
                        if (g[u] + 1 < count)
                            lo[u] = mem.load1_last_use(buffer_a + g[u] + 1);
                    }
#pragma unroll
                for (int u = 0; u < kCopyUnroll; ++u)
                    if (g[u] < count)
                    {
                        T* const p = tensor_b + toff[u];
                        if (g[u] + 1 < count)
                        {
                            Seam t;
                            if constexpr (kIdentity)
                            {
                                t[0] = hi[u];
                                t[1] = lo[u];
                            }
                            else
                            {
                                t = mem.template load<2, false>(p);
                                t[0] = op(t[0], hi[u]);
                                t[1] = op(t[1], lo[u]);
                            }
                            mem.template store<2, false>(p, t);
                        }
                        else
                        {
                            mem.store1(p, kIdentity ? hi[u] : op(mem.load1(p), hi[u]));
                        }
                    }
                if (block_base == 0 && thread == 0) // element 0 of the first box has no partner
                {
                    const T v = mem.load1(buffer_a);
                    mem.store1(tensor_a, kIdentity ? v : op(mem.load1(tensor_a), v));
                }
            }
            else
            {
                WA va[kCopyUnroll], vb[kCopyUnroll];
#pragma unroll
                for (int u = 0; u < kCopyUnroll; ++u)
                    if (g[u] < count)
                    {
                        va[u] = mem.template load_last_use<VEC, true>(buffer_a + g[u]); // last use of the image
                        if (tensor_b != nullptr)
                            vb[u] = mem.template load_last_use<VEC, true>(buffer_b + g[u]);
                    }
#pragma unroll
                for (int u = 0; u < kCopyUnroll; ++u)
                    if (g[u] < count)
                    {
                        accumulate_pair<T, VEC, WU, Op, kIdentity, Mem>(tensor_a + toff[u], tensor_b != nullptr ? tensor_b + toff[u] : nullptr,
                                                                   static_cast<WU>(va[u]), static_cast<WU>(vb[u]), box.disjoint, op, mem);
                    }
            }
        }
        else // kClear
        {
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u)
                if (g[u] < count)
                {
                    WU z;
#pragma unroll
                    for (int j = 0; j < VEC; ++j)
                        z[j] = T(0);
                    mem.template store<VEC, false>(tensor_a + toff[u], z);
                    if (tensor_b != nullptr)
                        mem.template store<VEC, false>(tensor_b + toff[u], z);
                }
        }
    }
    else
    {
        // ---- dense boxes ---------------------------------------------------------
        T* const tensor = reinterpret_cast<T*>(TABLE ? tensor_base + reinterpret_cast<intptr_t>(box.tensor)
                                                     : box.tensor);
        T* const buffer = reinterpret_cast<T*>(TABLE ? buffer_base + reinterpret_cast<intptr_t>(box.buffer)
                                                     : box.buffer);

        // Offsets of the part of a straddling vector that lies in the next run.
        auto tail_offsets = [&](int u, int64_t* t_at, int64_t* s_at) {
            uint32_t first;
            box_offsets<kTransferMode>(box, g[u] + head[u], t_at, s_at, &first);
        };

        WU v[kCopyUnroll];
        // 1. load what moves
        if constexpr (MODE == kPack || MODE == kTransfer)
        {
            const T* const from = MODE == kPack ? tensor : buffer;
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u)
                if (g[u] < count)
                {
                    const int64_t at = MODE == kPack ? toff[u] : soff[u];
                    if (head[u] == VEC)
                    {
                        if constexpr (TABLE)
                            v[u] = mem.template load_last_use<VEC, false>(from + at);
                        else
                            v[u] = mem.template load<VEC, false>(from + at);
                    }
                    else
                    {
                        int64_t t_at, s_at;
                        tail_offsets(u, &t_at, &s_at);
                        const int64_t next = (MODE == kPack ? t_at : s_at) - head[u];
#pragma unroll
                        for (int j = 0; j < VEC; ++j)
                            if (g[u] + j < count)
                                v[u][j] = mem.load1(from + (j < static_cast<int>(head[u]) ? at + j : next + j));
                    }
                }
        }
        else if constexpr (MODE == kUnpack)
        {
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u)
                if (g[u] < count)
                {
                    if (g[u] + VEC <= count)
                    {
                        v[u] = mem.template load_last_use<VEC, true>(buffer + g[u]); // last use of the image
                    }
                    else
                    {
#pragma unroll
                        for (int j = 0; j < VEC; ++j)
                            if (g[u] + j < count)
                                v[u][j] = mem.load1(buffer + g[u] + j);
                    }
                }
        }
        else
        {
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u)
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    v[u][j] = T(0);
        }
        // 2. store it
        if constexpr (MODE == kPack)
        {
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u)
                if (g[u] < count)
                {
                    if (g[u] + VEC <= count)
                    {
                        mem.template store<VEC, true>(buffer + g[u], v[u]);
                    }
                    else
                    {
#pragma unroll
                        for (int j = 0; j < VEC; ++j)
                            if (g[u] + j < count)
                                mem.store1(buffer + g[u] + j, static_cast<T>(v[u][j]));
                    }
                }
        }
        else
        {
            constexpr bool kCombine = !kIdentity && MODE != kClear;
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u)
                if (g[u] < count)
                {
                    if (head[u] == VEC)
                    {
                        WU t = v[u];
                        if constexpr (kCombine)
                        {
                            t = mem.template load<VEC, false>(tensor + toff[u]);
#pragma unroll
                            for (int j = 0; j < VEC; ++j)
                                t[j] = op(t[j], v[u][j]);
                        }
                        mem.template store<VEC, false>(tensor + toff[u], t);
                    }
                    else
                    {
                        int64_t t_at, s_at;
                        tail_offsets(u, &t_at, &s_at);
                        const int64_t next = t_at - head[u];
#pragma unroll
                        for (int j = 0; j < VEC; ++j)
                            if (g[u] + j < count)
                            {
                                T* const p = tensor + (j < static_cast<int>(head[u]) ? toff[u] + j : next + j);
                                T e = v[u][j];
                                if constexpr (kCombine)
                                    e = op(mem.load1(p), e);
                                mem.store1(p, e);
                            }
                    }
                }
        }
    }
}


template <typename T, int VEC, typename Op, bool SPARSE, int MODE, bool TABLE>
__global__ __launch_bounds__(kCopyBlock, 8) void box_copy_kernel(
    const typename std::conditional<TABLE, TableBatch, BoxBatch>::type batch, Op op)
{
    box_copy_body<T, VEC, Op, SPARSE, MODE, TABLE, DeviceMem>(batch, op, blockIdx.x, threadIdx.x, DeviceMem());
}

// ---- launch audit: the kernel body played on the CPU -----------------------------
// While an audit is open on the calling thread (h2x_copy_audit_begin), the copy
// entry points plan their launches as usual, and every launch is played on the
// host instead of being issued: each workgroup and lane runs the body above with
// an accessor that follows no pointer but counts, byte by byte, what would be
// loaded and stored in the address ranges the caller registered, and what falls
// outside them.  No GPU call is made.
struct AuditRegion
{
    uint64_t base, bytes;
    uint8_t* loads;  // per byte, saturating; may be null
    uint8_t* stores;
};

struct Audit
{
    std::vector<AuditRegion> regions;
    uint64_t launches = 0, workgroups = 0;
    uint64_t outside_loads = 0, outside_stores = 0; // bytes outside every region
    uint64_t misaligned = 0;                        // accesses not aligned as their instruction needs

    void touch(const void* p, size_t bytes, size_t align, bool store)
    {
        const uint64_t at = reinterpret_cast<uintptr_t>(p);
        if (at % align != 0)
            ++misaligned;
        for (const AuditRegion& r : regions)
        {
            if (at >= r.base && at + bytes <= r.base + r.bytes)
            {
                uint8_t* const count = store ? r.stores : r.loads;
                if (count)
                    for (size_t i = 0; i < bytes; ++i)
                    {
                        uint8_t& c = count[at - r.base + i];
                        if (c < 255)
                            ++c;
                    }
                return;
            }
        }
        (store ? outside_stores : outside_loads) += bytes;
    }
};

// The audit open on the calling thread, or null (h2x_copy.hip).
Audit* current_audit();

struct TraceMem
{
    Audit* audit;
    template <int VEC, bool ALIGNED, typename T>
    typename Words<T, VEC>::unaligned_t load(const T* p) const
    {
        audit->touch(p, sizeof(T) * VEC, ALIGNED ? sizeof(T) * VEC : sizeof(T), false);
        typename Words<T, VEC>::unaligned_t v;
        for (int j = 0; j < VEC; ++j)
            v[j] = T(0);
        return v;
    }
    template <int VEC, bool ALIGNED, typename T>
    typename Words<T, VEC>::unaligned_t load_last_use(const T* p) const
    {
        return load<VEC, ALIGNED>(p);
    }
    template <int VEC, bool ALIGNED, typename T>
    void store(T* p, typename Words<T, VEC>::unaligned_t) const
    {
        audit->touch(p, sizeof(T) * VEC, ALIGNED ? sizeof(T) * VEC : sizeof(T), true);
    }
    template <typename T>
    T load1(const T* p) const
    {
        audit->touch(p, sizeof(T), sizeof(T), false);
        return T(0);
    }
    template <typename T>
    T load1_last_use(const T* p) const
    {
        return load1(p);
    }
    template <typename T>
    void store1(T* p, T) const
    {
        audit->touch(p, sizeof(T), sizeof(T), true);
    }
};

// Issues one launch of the kernel - or plays it for the audit.
template <typename T, int VEC, typename Op, bool SPARSE, int MODE, bool TABLE>
int run_box_copy(uint32_t grid, hipStream_t stream,
                 const typename std::conditional<TABLE, TableBatch, BoxBatch>::type& batch, Op op)
{
    if (Audit* const audit = current_audit())
    {
        const TraceMem mem{audit};
        for (uint32_t block = 0; block < grid; ++block)
            for (uint32_t thread = 0; thread < kCopyBlock; ++thread)
                box_copy_body<T, VEC, Op, SPARSE, MODE, TABLE, TraceMem>(batch, op, block, thread, mem);
        ++audit->launches;
        audit->workgroups += grid;
        return H2X_SUCCESS;
    }
    box_copy_kernel<T, VEC, Op, SPARSE, MODE, TABLE><<<dim3(grid), kCopyBlock, 0, stream>>>(batch, op);
    return launch_status();
}

#endif // __HIPCC__

// ---- launches (host) ---------------------------------------------------------
// What a launch needs besides its descriptors.
struct LaunchShape
{
    int elem_size; // 2, 4 or 8
    int op;        // h2x_halo_op
    int vec;       // elements per vector
    bool sparse;
    int mode;      // Mode
    uint32_t grid; // workgroups
    hipStream_t stream;
};

// Identity copies of 2-, 4- and 8-byte elements, every mode (h2x_copy.hip).
int launch_identity(const LaunchShape& shape, const BoxBatch& batch);
// Pack or unpack through plan tables, identity only (h2x_copy.hip).
int launch_tables(const LaunchShape& shape, const TableBatch& batch);
// SUM / MAX / MIN of float or double elements, unpack and transfer (h2x_copy_acc.hip).
int launch_accumulate(const LaunchShape& shape, h2x_dtype dtype, const BoxBatch& batch);

} // namespace copy
} // namespace h2x

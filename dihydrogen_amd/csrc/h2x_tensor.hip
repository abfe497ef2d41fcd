// Elementwise transforms over the interiors of up to four tensors and sums over
// chosen dimensions, for gfx950: what the reference builds its per-channel
// statistics, scaling and copies from
// (legacy/include/distconv/tensor/algorithms/transform_cuda.hpp:359-693,
//  reduce_sum_cuda.hpp:56-113,388-439).
//
// The reference instantiates a kernel per functor; a C interface cannot take a
// functor, so the operations this path uses are named (h2x_transform_op).  All
// tensors of a call share one local shape and bring their own strides (halos);
// the host merges dimensions that are contiguous in every tensor, and a thread
// finds its element with one multiply-high division per remaining dimension.
//
// Sums are deterministic: every output element's addends are cut into groups,
// a group is added up in fp64 by one workgroup (reduced dimension innermost) or
// one thread (kept dimension innermost), in index order, and a second kernel
// adds the groups in order and accumulates into the destination -- where the
// reference adds floats with atomics in whatever order they arrive
// (reduce_sum_cuda.hpp:108).
#include "h2x_device.hpp"

#include <algorithm>

namespace h2x
{
namespace
{

constexpr int kMaxDims = H2X_MAX_DIMS;
constexpr int kMaxTensors = 4;

struct TransformArgs
{
    char* base[kMaxTensors];
    int64_t stride[kMaxTensors][kMaxDims]; // elements; merged dimensions
    FastDiv div[kMaxDims];
    uint32_t count;
    int32_t num_dims;
    double p[4];
};

__device__ __forceinline__ float fma_t(float a, float b, float c)
{
    return __builtin_fmaf(a, b, c);
}
__device__ __forceinline__ double fma_t(double a, double b, double c)
{
    return __builtin_fma(a, b, c);
}

// legacy/src/dnn_backend/batchnorm.cu:297-312: the same operations, in the same
// order, as the dedicated statistics kernel of the batch-norm entry points
template <typename T>
__device__ __forceinline__ void sums_to_statistics(T& mean, T& var, T& rmean, T& rvar, T n, T decay)
{
    const T m = mean / n;
    const T sqmean = var / n;
    T v = fma_t(-m, m, sqmean);
    v = v > T(0) ? v : T(0);
    v *= n / (n - T(1));
    mean = m;
    var = v;
    rmean = fma_t(decay, rmean, (T(1) - decay) * m);
    rvar = fma_t(decay, rvar, (T(1) - decay) * v);
}

// One element of one operation; pointers to the element in each tensor.
template <typename T, int OP>
__device__ __forceinline__ void transform_element(T* const (&v)[4], const double (&p)[4])
{
    if constexpr (OP == H2X_TRANSFORM_SCALE)
    {
        *v[0] = *v[0] * static_cast<T>(p[0]); // internal::ScaleFunctor, tensor_mpi_cuda.cu:86-92
    }
    else if constexpr (OP == H2X_TRANSFORM_COPY)
    {
        *v[1] = *v[0];
    }
    else if constexpr (OP == H2X_TRANSFORM_SCALE_BIAS)
    {
        // CastScaleBiasFuctor with equal types: dst = alpha * src + beta (tensor_mpi_cuda.cu:113-128)
        *v[1] = static_cast<T>(p[0]) * *v[0] + static_cast<T>(p[1]);
    }
    else
    {
        T m = *v[0], var = *v[1], rm = *v[2], rv = *v[3];
        if (p[0] == 0.0) // nothing was counted: batchnorm.cu:337-345
        {
            *v[1] = T(1);
        }
        else
        {
            sums_to_statistics(m, var, rm, rv, static_cast<T>(p[0]), static_cast<T>(p[1]));
            *v[0] = m;
            *v[1] = var;
            *v[2] = rm;
            *v[3] = rv;
        }
    }
}

// A thread owns VEC neighbouring elements of the innermost merged dimension
// (VEC > 1: that dimension is contiguous in every tensor and a multiple of VEC
// long, so a vector never leaves its row; rows of haloed tensors start on any
// element, hence vector types aligned to one element).  Tensors that are only
// read come in as one vector load, tensors that are written leave as one vector
// store; a tensor that is only written (the destination of a copy or of
// scale + bias) is stored past the caches.
template <typename T, int OP, int VEC>
__global__ __launch_bounds__(kBlockSize) void transform_kernel(const TransformArgs a)
{
    constexpr int N = OP == H2X_TRANSFORM_SCALE ? 1 : OP == H2X_TRANSFORM_SUMS_TO_STATISTICS ? 4 : 2;
    constexpr bool kStreamOut = OP == H2X_TRANSFORM_COPY || OP == H2X_TRANSFORM_SCALE_BIAS;
    typedef T Vec __attribute__((ext_vector_type(VEC), aligned(sizeof(T))));
    // One vector a thread and a grid that covers them all: a loop over further
    // vectors (the grid once was capped) cost the dense copy a tenth of its time
    // (268 MB: 83 -> 75 us), and two or four vectors in flight per thread make
    // haloed destinations slower (90 -> 99 / 113 us).
    const uint32_t i = blockIdx.x * kBlockSize + threadIdx.x;
    if (i < a.count / VEC)
    {
        uint32_t rem = i * VEC;
        int64_t off[N];
#pragma unroll
        for (int t = 0; t < N; ++t)
            off[t] = 0;
#pragma unroll
        for (int d = 0; d < kMaxDims; ++d)
        {
            if (d < a.num_dims)
            {
                uint32_t idx = rem;
                if (d + 1 < a.num_dims)
                {
                    const uint32_t q = fastdiv(rem, a.div[d]);
                    idx = rem - q * a.div[d].divisor;
                    rem = q;
                }
#pragma unroll
                for (int t = 0; t < N; ++t)
                    off[t] += static_cast<int64_t>(idx) * a.stride[t][d];
            }
        }
        if constexpr (VEC == 1)
        {
            T* v[4] = {nullptr, nullptr, nullptr, nullptr};
#pragma unroll
            for (int t = 0; t < N; ++t)
                v[t] = reinterpret_cast<T*>(a.base[t]) + off[t];
            transform_element<T, OP>(v, a.p);
        }
        else
        {
            Vec reg[N];
#pragma unroll
            for (int t = 0; t < N; ++t)
                if (!(kStreamOut && t == 1))
                    reg[t] = *reinterpret_cast<const Vec*>(reinterpret_cast<const T*>(a.base[t]) + off[t]);
            T lane[4][VEC];
#pragma unroll
            for (int j = 0; j < VEC; ++j)
            {
                T* v[4] = {nullptr, nullptr, nullptr, nullptr};
#pragma unroll
                for (int t = 0; t < N; ++t)
                {
                    lane[t][j] = (kStreamOut && t == 1) ? T(0) : reg[t][j];
                    v[t] = &lane[t][j];
                }
                transform_element<T, OP>(v, a.p);
            }
#pragma unroll
            for (int t = 0; t < N; ++t)
            {
                if (OP != H2X_TRANSFORM_SCALE && OP != H2X_TRANSFORM_SUMS_TO_STATISTICS && t == 0)
                    continue; // the source of a copy is not written
                Vec out;
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    out[j] = lane[t][j];
                Vec* const dst = reinterpret_cast<Vec*>(reinterpret_cast<T*>(a.base[t]) + off[t]);
                if constexpr (kStreamOut)
                    __builtin_nontemporal_store(out, dst);
                else
                    *dst = out;
            }
        }
    }
}

// ---- reduce ------------------------------------------------------------------

struct ReduceArgs
{
    const char* src;
    char* dst;
    double* partials;
    int32_t num_kept, num_reduced;
    FastDiv kept_div[kMaxDims];
    int64_t kept_src[kMaxDims], kept_dst[kMaxDims];
    FastDiv red_div[kMaxDims];
    int64_t red_src[kMaxDims];
    uint32_t kept_count, red_count; // K outputs, R addends each
    uint32_t groups, chunk;         // addends per group
    int32_t square;                 // add x * x instead of x
};

__device__ __forceinline__ int64_t chain(uint32_t i, int nd, const FastDiv* div, const int64_t* stride,
                                         const int64_t* stride2, int64_t* off2)
{
    uint32_t rem = i;
    int64_t off = 0, o2 = 0;
#pragma unroll
    for (int d = 0; d < kMaxDims; ++d)
    {
        if (d < nd)
        {
            uint32_t idx = rem;
            if (d + 1 < nd)
            {
                const uint32_t q = fastdiv(rem, div[d]);
                idx = rem - q * div[d].divisor;
                rem = q;
            }
            off += static_cast<int64_t>(idx) * stride[d];
            if (stride2)
                o2 += static_cast<int64_t>(idx) * stride2[d];
        }
    }
    if (off2)
        *off2 = o2;
    return off;
}

// The innermost dimension is reduced: a workgroup adds one group of one output
// element's addends; neighbouring threads read neighbouring addends, VEC at a
// time (VEC > 1: the innermost reduced dimension is contiguous and a multiple of
// VEC long, and so is the group size), four loads in flight per thread.
// RUN: every group lies within one run of the innermost reduced dimension, which
// is contiguous: the group's first addend is located once and the others follow
// it in memory (no index splitting per load).
template <typename T, int VEC, bool SQUARE, bool RUN>
__global__ __launch_bounds__(kBlockSize) void reduce_inner_kernel(const ReduceArgs a)
{
    typedef T Vec __attribute__((ext_vector_type(VEC), aligned(sizeof(T))));
    constexpr int kInFlight = 4;
    __shared__ double lds[kWavesPerBlock];
    // Groups count fastest (blockIdx.x): workgroups that start together then read
    // neighbouring chunks of one output's addends.  With the outputs fastest they
    // would start a whole kept-dimension stride apart, a power of two at the usual
    // shapes, and crowd a few memory channels.
    const uint32_t g = blockIdx.x;
    const uint32_t begin = g * a.chunk;
    const uint32_t end = begin + a.chunk < a.red_count ? begin + a.chunk : a.red_count;
    constexpr uint32_t kStep = kBlockSize * VEC;
    const int64_t run_start =
        RUN ? chain(begin, a.num_reduced, a.red_div, a.red_src, nullptr, nullptr) - begin : 0;
    auto locate = [&](uint32_t r) -> int64_t {
        if constexpr (RUN)
            return run_start + r;
        else
            return chain(r, a.num_reduced, a.red_div, a.red_src, nullptr, nullptr);
    };
    for (uint32_t k = blockIdx.y; k < a.kept_count; k += gridDim.y)
    {
        const T* src = reinterpret_cast<const T*>(a.src)
                       + chain(k, a.num_kept, a.kept_div, a.kept_src, nullptr, nullptr);
        double acc[1] = {0.0};
        auto add = [&](T v) {
            const double x = static_cast<double>(v);
            if constexpr (SQUARE && sizeof(T) == 4)
                acc[0] = __builtin_fma(x, x, acc[0]); // the product of two floats is exact in fp64
            else if constexpr (SQUARE)
                acc[0] += x * x;
            else
                acc[0] += x;
        };
        uint32_t r = begin + threadIdx.x * VEC;
        for (; r + (kInFlight - 1) * kStep < end; r += kInFlight * kStep)
        {
            Vec v[kInFlight];
#pragma unroll
            for (int u = 0; u < kInFlight; ++u)
                v[u] = *reinterpret_cast<const Vec*>(src + locate(r + u * kStep));
#pragma unroll
            for (int u = 0; u < kInFlight; ++u)
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    add(v[u][j]);
        }
        for (; r < end; r += kStep)
        {
            const Vec v = *reinterpret_cast<const Vec*>(src + locate(r));
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                add(v[j]);
        }
        block_sum<1>(acc, lds);
        if (threadIdx.x == 0)
        {
            if (a.groups == 1) // the only group of its output: no finishing launch
            {
                int64_t dst_off;
                chain(k, a.num_kept, a.kept_div, a.kept_src, a.kept_dst, &dst_off);
                T* p = reinterpret_cast<T*>(a.dst) + dst_off;
                *p = *p + static_cast<T>(acc[0]);
            }
            else
            {
                a.partials[static_cast<size_t>(k) * a.groups + g] = acc[0];
            }
        }
    }
}

// The innermost dimension is kept: a thread adds one group of the addends of its
// own VEC neighbouring output elements (VEC > 1: the innermost kept dimension is
// contiguous in source and destination and a multiple of VEC long); neighbouring
// threads own neighbouring outputs.
template <typename T, int VEC>
__global__ __launch_bounds__(kBlockSize) void reduce_outer_kernel(const ReduceArgs a)
{
    typedef T Vec __attribute__((ext_vector_type(VEC), aligned(sizeof(T))));
    const uint32_t k = (blockIdx.x * kBlockSize + threadIdx.x) * VEC, g = blockIdx.y;
    if (k >= a.kept_count)
        return;
    int64_t dst_off;
    const T* src = reinterpret_cast<const T*>(a.src)
                   + chain(k, a.num_kept, a.kept_div, a.kept_src, a.kept_dst, &dst_off);
    const uint32_t begin = g * a.chunk;
    const uint32_t end = begin + a.chunk < a.red_count ? begin + a.chunk : a.red_count;
    double acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j)
        acc[j] = 0.0;
    for (uint32_t r = begin; r < end; ++r)
    {
        const Vec v = *reinterpret_cast<const Vec*>(
            src + chain(r, a.num_reduced, a.red_div, a.red_src, nullptr, nullptr));
#pragma unroll
        for (int j = 0; j < VEC; ++j)
        {
            const double x = static_cast<double>(v[j]);
            acc[j] += a.square ? x * x : x;
        }
    }
    if (a.groups == 1) // the only group of its outputs: no finishing launch
    {
        Vec* p = reinterpret_cast<Vec*>(reinterpret_cast<T*>(a.dst) + dst_off);
        Vec d = *p;
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            d[j] = d[j] + static_cast<T>(acc[j]);
        *p = d;
    }
    else
    {
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            a.partials[static_cast<size_t>(g) * a.kept_count + k + j] = acc[j];
    }
}

// The innermost dimension is reduced and an output element has few addends (at
// most 64 loads of VEC): `lanes` neighbouring lanes of a wave (a power of two)
// share an output, each loads its vectors, and the lanes are combined by
// exchanges at distance lanes/2, ..., 1 - a fixed order.  One group per output.
template <typename T, int VEC>
__global__ __launch_bounds__(kBlockSize) void reduce_inner_small_kernel(const ReduceArgs a, uint32_t lanes)
{
    typedef T Vec __attribute__((ext_vector_type(VEC), aligned(sizeof(T))));
    const uint64_t t = static_cast<uint64_t>(blockIdx.x) * kBlockSize + threadIdx.x;
    const uint64_t k64 = t / lanes;
    const uint32_t lane = static_cast<uint32_t>(t - k64 * lanes);
    const bool valid = k64 < a.kept_count;
    const uint32_t k = valid ? static_cast<uint32_t>(k64) : 0;
    double acc = 0.0;
    int64_t dst_off = 0;
    if (valid)
    {
        const T* src = reinterpret_cast<const T*>(a.src)
                       + chain(k, a.num_kept, a.kept_div, a.kept_src, a.kept_dst, &dst_off);
        for (uint32_t r = lane * VEC; r < a.red_count; r += lanes * VEC)
        {
            const Vec v = *reinterpret_cast<const Vec*>(
                src + chain(r, a.num_reduced, a.red_div, a.red_src, nullptr, nullptr));
#pragma unroll
            for (int j = 0; j < VEC; ++j)
            {
                const double x = static_cast<double>(v[j]);
                acc += a.square ? x * x : x;
            }
        }
    }
    for (uint32_t d = lanes / 2; d >= 1; d /= 2)
        acc += __shfl_xor(acc, static_cast<int>(d), kWaveSize);
    if (valid && lane == 0)
    {
        T* p = reinterpret_cast<T*>(a.dst) + dst_off;
        *p = *p + static_cast<T>(acc);
    }
}

// dst[k] += sum over the groups, in group order: a thread per output element.
template <typename T>
__global__ __launch_bounds__(kBlockSize) void reduce_finish_kernel(const ReduceArgs a, int inner)
{
    const uint32_t k = blockIdx.x * kBlockSize + threadIdx.x;
    if (k >= a.kept_count)
        return;
    double t = 0.0;
    for (uint32_t g = 0; g < a.groups; ++g)
        t += inner ? a.partials[static_cast<size_t>(k) * a.groups + g]
                   : a.partials[static_cast<size_t>(g) * a.kept_count + k];
    int64_t dst_off;
    chain(k, a.num_kept, a.kept_div, a.kept_src, a.kept_dst, &dst_off);
    T* p = reinterpret_cast<T*>(a.dst) + dst_off;
    *p = *p + static_cast<T>(t);
}

// The same for few outputs with many groups each: a workgroup per output element;
// thread t adds groups t, t + 256, ..., the workgroup combines its threads in the
// fixed order of block_sum.
template <typename T>
__global__ __launch_bounds__(kBlockSize) void reduce_finish_wide_kernel(const ReduceArgs a, int inner)
{
    __shared__ double lds[kWavesPerBlock];
    const uint32_t k = blockIdx.x;
    // the value to add to is asked for first, so that its latency passes with the partials'
    T* p = nullptr;
    T before = T(0);
    if (threadIdx.x == 0)
    {
        int64_t dst_off;
        chain(k, a.num_kept, a.kept_div, a.kept_src, a.kept_dst, &dst_off);
        p = reinterpret_cast<T*>(a.dst) + dst_off;
        before = *p;
    }
    double t[1] = {0.0};
    for (uint32_t g = threadIdx.x; g < a.groups; g += kBlockSize)
        t[0] += inner ? a.partials[static_cast<size_t>(k) * a.groups + g]
                      : a.partials[static_cast<size_t>(g) * a.kept_count + k];
    block_sum<1>(t, lds);
    if (threadIdx.x == 0)
        *p = before + static_cast<T>(t[0]);
}

// ---- host ---------------------------------------------------------------------

int check_geometry(const h2x_tensor_geometry* g)
{
    if (!g || g->num_dims < 1 || g->num_dims > kMaxDims)
        return H2X_ERR_INVALID_ARGUMENT;
    for (int i = 0; i < g->num_dims; ++i)
        if (g->local_shape[i] < 0 || g->strides[i] < 0)
            return H2X_ERR_INVALID_ARGUMENT;
    return H2X_SUCCESS;
}

template <typename T, int VEC>
int transform_vec(int op, const TransformArgs& a, hipStream_t stream)
{
    const uint32_t vectors = a.count / VEC;
    const unsigned int blocks = (vectors + kBlockSize - 1) / kBlockSize; // count < 2^32: at most 2^24 workgroups
    switch (op)
    {
    case H2X_TRANSFORM_SCALE:
        transform_kernel<T, H2X_TRANSFORM_SCALE, VEC><<<blocks, kBlockSize, 0, stream>>>(a);
        break;
    case H2X_TRANSFORM_COPY:
        transform_kernel<T, H2X_TRANSFORM_COPY, VEC><<<blocks, kBlockSize, 0, stream>>>(a);
        break;
    case H2X_TRANSFORM_SCALE_BIAS:
        transform_kernel<T, H2X_TRANSFORM_SCALE_BIAS, VEC><<<blocks, kBlockSize, 0, stream>>>(a);
        break;
    case H2X_TRANSFORM_SUMS_TO_STATISTICS:
        transform_kernel<T, H2X_TRANSFORM_SUMS_TO_STATISTICS, VEC><<<blocks, kBlockSize, 0, stream>>>(a);
        break;
    default: return H2X_ERR_UNSUPPORTED;
    }
    return launch_status();
}

// 16-byte vectors when the innermost merged dimension is contiguous in every
// tensor and a multiple of the vector long; element by element otherwise.
template <typename T>
int transform_typed(int op, int num_tensors, const TransformArgs& a, hipStream_t stream)
{
    constexpr int kVec = 16 / sizeof(T);
    bool vec = a.div[0].divisor % kVec == 0;
    for (int t = 0; t < num_tensors; ++t)
        vec = vec && a.stride[t][0] == 1;
    return vec ? transform_vec<T, kVec>(op, a, stream) : transform_vec<T, 1>(op, a, stream);
}

// How a sum is cut up.  Shared by the entry point and the workspace query.
struct ReducePlan
{
    ReduceArgs args;
    bool inner = false; // the innermost dimension with more than one element is reduced
    int vec = 1;        // elements per load of the inner reduction (a multiple divides every group)
    int outer_vec = 1;  // neighbouring outputs per thread of the outer reduction
    uint32_t small_lanes = 0; // > 0: inner reduction with few addends, this many lanes per output
    bool empty = false; // nothing to add
};

int plan_reduce(const h2x_tensor_geometry* src, const h2x_tensor_geometry* dst, int max_vec,
                ReducePlan* plan)
{
    int err = check_geometry(src);
    if (!err)
        err = check_geometry(dst);
    if (err)
        return err;
    if (src->num_dims != dst->num_dims)
        return H2X_ERR_INVALID_ARGUMENT;
    ReduceArgs& a = plan->args;
    a.num_kept = a.num_reduced = 0;
    uint64_t kept = 1, red = 1;
    bool first = true;
    int64_t kept_extent[kMaxDims], red_extent[kMaxDims];
    for (int i = 0; i < src->num_dims; ++i)
    {
        const int64_t e = src->local_shape[i];
        // reduce to a single entry or not at all: reduce_sum_cuda.hpp:160-171
        if (dst->local_shape[i] != 1 && dst->local_shape[i] != e)
            return H2X_ERR_INVALID_ARGUMENT;
        if (e == 0)
            plan->empty = true;
        if (e == 1)
            continue;
        const bool reduced = dst->local_shape[i] == 1;
        if (first)
        {
            plan->inner = reduced;
            first = false;
        }
        if (reduced)
        {
            // merge with the previous reduced dimension when contiguous in the source
            if (a.num_reduced > 0
                && src->strides[i] == a.red_src[a.num_reduced - 1] * red_extent[a.num_reduced - 1])
            {
                red_extent[a.num_reduced - 1] *= e;
            }
            else
            {
                red_extent[a.num_reduced] = e;
                a.red_src[a.num_reduced] = src->strides[i];
                ++a.num_reduced;
            }
            red *= static_cast<uint64_t>(e);
        }
        else
        {
            kept_extent[a.num_kept] = e;
            a.kept_src[a.num_kept] = src->strides[i];
            a.kept_dst[a.num_kept] = dst->strides[i];
            ++a.num_kept;
            kept *= static_cast<uint64_t>(e);
        }
    }
    if (kept >= (1ull << 31) || red >= (1ull << 31))
        return H2X_ERR_TOO_LARGE;
    for (int i = 0; i < kMaxDims; ++i)
    {
        a.kept_div[i] = make_fastdiv(i < a.num_kept ? static_cast<uint32_t>(kept_extent[i]) : 1u);
        a.red_div[i] = make_fastdiv(i < a.num_reduced ? static_cast<uint32_t>(red_extent[i]) : 1u);
        if (i >= a.num_kept)
            a.kept_src[i] = a.kept_dst[i] = 0;
        if (i >= a.num_reduced)
            a.red_src[i] = 0;
    }
    a.kept_count = static_cast<uint32_t>(kept);
    a.red_count = static_cast<uint32_t>(red);
    // about 4096 workgroups in all, and no group smaller than four passes of its team
    constexpr uint64_t kTargetBlocks = 4096;
    uint64_t groups;
    if (plan->inner)
        groups = std::min<uint64_t>((red + 4 * kBlockSize - 1) / (4 * kBlockSize),
                                    std::max<uint64_t>(kTargetBlocks / std::max<uint64_t>(kept, 1), 1));
    else
        groups = std::min<uint64_t>(
            (red + 15) / 16,
            std::max<uint64_t>(kTargetBlocks / ((kept + kBlockSize - 1) / kBlockSize), 1));
    groups = std::min<uint64_t>(std::max<uint64_t>(groups, 1), 65535);
    a.chunk = static_cast<uint32_t>((red + groups - 1) / groups);
    // 16-byte loads: the innermost reduced dimension is contiguous and a multiple of
    // the vector long; groups then start and end on whole vectors
    plan->vec = 1;
    if (plan->inner && a.num_reduced > 0 && a.red_src[0] == 1 && red_extent[0] % max_vec == 0)
    {
        plan->vec = max_vec;
        a.chunk = (a.chunk + max_vec - 1) / max_vec * max_vec;
    }
    a.groups = static_cast<uint32_t>((red + a.chunk - 1) / std::max<uint32_t>(a.chunk, 1));
    if (a.groups == 0)
        a.groups = 1;
    // few addends per output: lanes of a wave share an output instead of a workgroup
    plan->small_lanes = 0;
    if (plan->inner && red <= 64ull * plan->vec)
    {
        uint32_t lanes = 1;
        while (static_cast<uint64_t>(lanes) * plan->vec < red)
            lanes *= 2;
        plan->small_lanes = lanes;
        a.chunk = static_cast<uint32_t>(red);
        a.groups = 1;
    }
    // outer reduction: 16-byte vectors of neighbouring outputs
    plan->outer_vec = 1;
    if (!plan->inner && a.num_kept > 0 && a.kept_src[0] == 1 && a.kept_dst[0] == 1
        && kept_extent[0] % max_vec == 0)
        plan->outer_vec = max_vec;
    return H2X_SUCCESS;
}

template <typename T>
int reduce_typed(const ReducePlan& plan, hipStream_t stream)
{
    const ReduceArgs& a = plan.args;
    constexpr int kVec = 16 / sizeof(T);
    const unsigned int kept_blocks = (a.kept_count + kBlockSize - 1) / kBlockSize;
    if (plan.small_lanes > 0)
    {
        const uint64_t threads = static_cast<uint64_t>(a.kept_count) * plan.small_lanes;
        const uint64_t blocks = (threads + kBlockSize - 1) / kBlockSize;
        if (blocks > 0x7fffffffull)
            return H2X_ERR_TOO_LARGE;
        if (plan.vec == kVec)
            reduce_inner_small_kernel<T, kVec><<<static_cast<unsigned int>(blocks), kBlockSize, 0, stream>>>(
                a, plan.small_lanes);
        else
            reduce_inner_small_kernel<T, 1><<<static_cast<unsigned int>(blocks), kBlockSize, 0, stream>>>(
                a, plan.small_lanes);
        return launch_status();
    }
    if (plan.inner)
    {
        const dim3 grid(a.groups, std::min<uint32_t>(a.kept_count, 65535u));
        // every group within one contiguous run of the innermost reduced dimension?
        const bool run = a.num_reduced > 0 && a.red_src[0] == 1
                         && (a.num_reduced == 1 || a.red_div[0].divisor % a.chunk == 0);
#define H2X_REDUCE_INNER(VEC)                                                                      \
    do                                                                                             \
    {                                                                                              \
        if (a.square && run)                                                                       \
            reduce_inner_kernel<T, VEC, true, true><<<grid, kBlockSize, 0, stream>>>(a);           \
        else if (a.square)                                                                         \
            reduce_inner_kernel<T, VEC, true, false><<<grid, kBlockSize, 0, stream>>>(a);          \
        else if (run)                                                                              \
            reduce_inner_kernel<T, VEC, false, true><<<grid, kBlockSize, 0, stream>>>(a);          \
        else                                                                                       \
            reduce_inner_kernel<T, VEC, false, false><<<grid, kBlockSize, 0, stream>>>(a);         \
    } while (0)
        if (plan.vec == kVec)
            H2X_REDUCE_INNER(kVec);
        else
            H2X_REDUCE_INNER(1);
#undef H2X_REDUCE_INNER
    }
    else if (plan.outer_vec == kVec)
    {
        const unsigned int blocks = (a.kept_count / kVec + kBlockSize - 1) / kBlockSize;
        reduce_outer_kernel<T, kVec><<<dim3(blocks, a.groups), kBlockSize, 0, stream>>>(a);
    }
    else
    {
        reduce_outer_kernel<T, 1><<<dim3(kept_blocks, a.groups), kBlockSize, 0, stream>>>(a);
    }
    if (a.groups == 1)
        return launch_status(); // the reduction kernel has accumulated into the destination itself
    if (a.groups >= 16 && a.kept_count <= 4096)
        reduce_finish_wide_kernel<T><<<a.kept_count, kBlockSize, 0, stream>>>(a, plan.inner ? 1 : 0);
    else
        reduce_finish_kernel<T><<<kept_blocks, kBlockSize, 0, stream>>>(a, plan.inner ? 1 : 0);
    return launch_status();
}

} // namespace
} // namespace h2x

using namespace h2x;

extern "C" int h2x_tensor_transform(h2x_transform_op op, h2x_dtype dtype, int num_tensors,
                                    const h2x_tensor_geometry* const* geometries,
                                    void* const* tensors, const double* params,
                                    h2x_stream_t stream)
{
    const int expected = op == H2X_TRANSFORM_SCALE                ? 1
                         : op == H2X_TRANSFORM_COPY               ? 2
                         : op == H2X_TRANSFORM_SCALE_BIAS         ? 2
                         : op == H2X_TRANSFORM_SUMS_TO_STATISTICS ? 4
                                                                  : 0;
    if (expected == 0)
        return H2X_ERR_UNSUPPORTED;
    if (dtype != H2X_F32 && dtype != H2X_F64)
        return H2X_ERR_UNSUPPORTED;
    if (num_tensors != expected || !geometries || !tensors)
        return H2X_ERR_INVALID_ARGUMENT;
    if (op != H2X_TRANSFORM_COPY && !params)
        return H2X_ERR_INVALID_ARGUMENT;
    for (int t = 0; t < num_tensors; ++t)
    {
        const int err = check_geometry(geometries[t]);
        if (err)
            return err;
        if (geometries[t]->num_dims != geometries[0]->num_dims)
            return H2X_ERR_INVALID_ARGUMENT;
        for (int i = 0; i < geometries[0]->num_dims; ++i)
            if (geometries[t]->local_shape[i] != geometries[0]->local_shape[i])
                return H2X_ERR_INVALID_ARGUMENT;
    }
    // merge what is contiguous in every tensor; extent-1 dimensions vanish
    TransformArgs a;
    int nd = 0;
    int64_t extent[kMaxDims];
    uint64_t count = 1;
    for (int i = 0; i < geometries[0]->num_dims; ++i)
    {
        const int64_t e = geometries[0]->local_shape[i];
        count *= static_cast<uint64_t>(e);
        if (e == 1)
            continue;
        bool merge = nd > 0;
        for (int t = 0; merge && t < num_tensors; ++t)
            merge = geometries[t]->strides[i] == a.stride[t][nd - 1] * extent[nd - 1];
        if (merge)
        {
            extent[nd - 1] *= e;
        }
        else
        {
            extent[nd] = e;
            for (int t = 0; t < num_tensors; ++t)
                a.stride[t][nd] = geometries[t]->strides[i];
            ++nd;
        }
    }
    if (count == 0)
        return H2X_SUCCESS;
    if (count >= (1ull << 31))
        return H2X_ERR_TOO_LARGE;
    for (int t = 0; t < num_tensors; ++t)
        if (!tensors[t])
            return H2X_ERR_INVALID_ARGUMENT;
    if (nd == 0)
    {
        nd = 1;
        extent[0] = 1;
        for (int t = 0; t < num_tensors; ++t)
            a.stride[t][0] = 1;
    }
    for (int t = 0; t < kMaxTensors; ++t)
    {
        a.base[t] = t < num_tensors ? static_cast<char*>(tensors[t]) : nullptr;
        for (int i = 0; i < kMaxDims; ++i)
            if (t >= num_tensors || i >= nd)
                a.stride[t][i] = 0;
    }
    for (int i = 0; i < kMaxDims; ++i)
        a.div[i] = make_fastdiv(i < nd ? static_cast<uint32_t>(extent[i]) : 1u);
    a.count = static_cast<uint32_t>(count);
    a.num_dims = nd;
    for (int i = 0; i < 4; ++i)
        a.p[i] = params ? params[i] : 0.0;
    return dtype == H2X_F32 ? transform_typed<float>(op, num_tensors, a, as_stream(stream))
                            : transform_typed<double>(op, num_tensors, a, as_stream(stream));
}

extern "C" size_t h2x_tensor_reduce_sum_workspace_bytes(const h2x_tensor_geometry* src_geometry,
                                                        const h2x_tensor_geometry* dst_geometry)
{
    // rounding the group size up to whole vectors can only lower the number of
    // groups, so the plan without vectors bounds both element types
    ReducePlan plan;
    if (plan_reduce(src_geometry, dst_geometry, 1, &plan) != 0)
        return 0;
    const size_t n = static_cast<size_t>(plan.args.kept_count) * plan.args.groups * sizeof(double);
    return (std::max<size_t>(n, 1) + 255) / 256 * 256;
}

extern "C" int h2x_tensor_reduce_sum(h2x_dtype dtype, const h2x_tensor_geometry* src_geometry,
                                     const void* src, const h2x_tensor_geometry* dst_geometry,
                                     void* dst, int square, void* workspace, h2x_stream_t stream)
{
    if (dtype != H2X_F32 && dtype != H2X_F64)
        return H2X_ERR_UNSUPPORTED;
    ReducePlan plan;
    const int err = plan_reduce(src_geometry, dst_geometry, dtype == H2X_F32 ? 4 : 2, &plan);
    if (err)
        return err;
    if (plan.empty || plan.args.kept_count == 0 || plan.args.red_count == 0)
        return H2X_SUCCESS; // nothing to add: the destination keeps its values
    if (!src || !dst || !workspace)
        return H2X_ERR_INVALID_ARGUMENT;
    plan.args.src = static_cast<const char*>(src);
    plan.args.dst = static_cast<char*>(dst);
    plan.args.partials = static_cast<double*>(workspace);
    plan.args.square = square ? 1 : 0;
    return dtype == H2X_F32 ? reduce_typed<float>(plan, as_stream(stream))
                            : reduce_typed<double>(plan, as_stream(stream));
}

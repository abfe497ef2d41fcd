// Channel-wise batch-normalisation kernels for gfx950 and their C entry points.
//
// Two layouts (and, for tensors whose (sample, channel) segments have at most
// 256 elements, a third family of kernels that gives a workgroup a window of
// neighbouring whole channels: see "short segments" below).  Dense: element
// (n, c, i) of a tensor lives at
// base[(n*C + c)*real + i], i < spatial -- the geometry of the reference's
// optimised kernels (legacy/src/dnn_backend/batchnorm.cu:134-190).  Strided:
// the interior of a tensor with halos on any spatial dimension, addressed
// through the tensor's strides like the reference's generic kernels
// (batchnorm.cu:39-90,369-418,899-980,1303-1369); rows are padded to whole
// vectors, an index is split into (row, vector of the row) with multiply-high
// divisions, and every vector is one unaligned 16-byte access (see TensorMap).
// Every kernel is a pure HBM stream: 16-byte
// accesses when the geometry allows, several loads in flight per lane,
// per-channel parameters fetched once per workgroup.
//
// Cache policy.  The layer reads x four times (sums, apply, backprop1,
// backprop2) and dy twice, while y and dx are written once.  x of the headline
// shapes is about the size of the 256 MB memory-side cache, so what must not
// happen is that the outputs or dy push it out: y and dx are written with
// nontemporal stores and dy is read with nontemporal loads; x uses plain
// loads.  Measured on NCDHW 4x64x64^3: forward+backward 381 us -> 285 us.
//
// Reductions (forward sums, backward sums) cut every channel into contiguous
// chunks, one workgroup per chunk.  A thread accumulates in fp64, the
// workgroup combines lanes with DPP permutes and waves through LDS, and writes
// one fp64 partial per sum into the workspace.  A second, tiny kernel adds the
// partials of each channel in index order and writes the channel's result
// (a kernel boundary is the cheapest device-wide ordering on this GPU: an
// in-kernel "last workgroup finishes" scheme needs a device-scope fence per
// workgroup, which costs an L2 write-back/invalidate each and was measured
// 10x slower than the whole stream).  All orders are fixed, so results are
// deterministic; the reference's float atomics are not
// (batchnorm.cu:127-131,1047-1053).
#include "h2x_bn_maps.hpp"
#include "h2x_bn_plan.hpp"
#include "h2x_device.hpp"

#include <algorithm>
#include <mutex>

// Partial sums of h2x_bn_channel_sums_and_sqsums_static, the entry point for
// callers that can neither allocate nor bring a workspace.  Every device the
// library runs on holds its own copy of this array, at its own address, until
// the process ends.  In host code the name is only a handle for
// hipGetSymbolAddress; kernels receive the address that call returned.
static constexpr size_t kStaticScratchBytes = size_t(1) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace h2x
{
namespace
{

using namespace bn;

// The log the calling thread has installed (h2x_bn_plan.hpp): launches are then
// described instead of issued.
thread_local LaunchLog* t_launch_log = nullptr;

// Appends a planned launch to the installed log; false: no log, issue it.
bool logged(const LaunchRecord& r)
{
    if (!t_launch_log)
        return false;
    t_launch_log->records.push_back(r);
    return true;
}

// Status of the launches just issued (none while a log is installed).
int issued()
{
    return t_launch_log ? static_cast<int>(H2X_SUCCESS) : launch_status();
}

// Installs a log for the lifetime of the object and puts the previous one back.
struct ScopedLaunchLog
{
    explicit ScopedLaunchLog(LaunchLog* log) : before(t_launch_log) { t_launch_log = log; }
    ~ScopedLaunchLog() { t_launch_log = before; }
    void restore() { t_launch_log = before; }
    ScopedLaunchLog(const ScopedLaunchLog&) = delete;
    ScopedLaunchLog& operator=(const ScopedLaunchLog&) = delete;
    LaunchLog* before;
};

// Device address of `scratch` on the current device, looked up once per device.
constexpr int kMaxDevices = 64;
std::mutex static_scratch_mutex;
void* static_scratch_address[kMaxDevices] = {};

int static_scratch(void** out)
{
    int device = -1;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess)
        return static_cast<int>(err);
    if (device < 0 || device >= kMaxDevices)
        return H2X_ERR_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(static_scratch_mutex);
    if (static_scratch_address[device] == nullptr)
    {
        void* p = nullptr;
        err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (err != hipSuccess)
            return static_cast<int>(err);
        if (p == nullptr)
            return static_cast<int>(hipErrorInvalidSymbol);
        static_scratch_address[device] = p;
    }
    *out = static_scratch_address[device];
    return H2X_SUCCESS;
}

constexpr int kUnroll = 4;
// Workgroups a reduction aims at over all channels, from sweeps on MI355X: 4096
// on dense tensors, 16384 on haloed ones (the haloed C3 shard: two-launch
// forward 141 -> 134 us, backward 217 -> 211 us; dense shapes are the same or
// up to 4 % slower with more).  The workspace holds partial sums for the larger
// number.
constexpr int kTargetGroups = 16384;
constexpr int kDenseTargetGroups = 4096;
// Elementwise passes aim at 16384 workgroups (from a sweep on MI355X at the
// headline shapes) - except on haloed tensors and on tensors beyond the
// memory-side cache, where a workgroup gets two passes of its 256 lanes (8 KB
// of fp32 per tensor) however large the tensor is.  Measured against the
// budget of 16384: normalise on the haloed C3 shard 158 -> 145 us, input
// gradient 240 -> 222 us; dense tensors of 1 GB 571 -> 529 us and 896 -> 836
// us, of 537 MB 279 -> 267 us and 443 -> 423 us.  Dense tensors that the cache
// holds lose with the small chunks (268 MB: input gradient 191 -> 194 us, the
// benchmark step 676 -> 680 us; N 64 x 256 x 56 x 56: 150 -> 161 us) and keep
// the budget.
constexpr int kElementwiseBlocks = 16384;
constexpr int kUnboundedBlocks = 1 << 30;
constexpr size_t kBeyondCacheBytes = size_t(384) << 20;
constexpr int kMinGroupsPerChannel = 8;
constexpr int kMaxGroupsPerChannel = 2048;
constexpr int kMaxSums = 4;

int groups_per_channel(int num_channels, int target)
{
    const int g = (target + num_channels - 1) / std::max(num_channels, 1);
    return std::min(std::max(g, kMinGroupsPerChannel), kMaxGroupsPerChannel);
}

// Partial sums the workspace holds per channel and sum: the stride of the
// partials of a channel, and the most groups any launch uses.
int max_groups_per_channel(int num_channels)
{
    return groups_per_channel(num_channels, kTargetGroups);
}

// Groups a long-segment reduction cuts a channel into.
int reduction_groups_per_channel(int num_channels, bool strided)
{
    return strided ? max_groups_per_channel(num_channels)
                   : groups_per_channel(num_channels, kDenseTargetGroups);
}

size_t partials_bytes(int num_channels)
{
    return static_cast<size_t>(num_channels) * max_groups_per_channel(num_channels) * kMaxSums
           * sizeof(double);
}

// How one (sample, channel) segment of `spatial` elements is cut into chunks.
// With vectors, `spatial` is a whole number of them (dense: a condition of the
// aligned path; strided: rows are padded), and so is every chunk.
struct Chunking
{
    size_t chunk;        // elements per workgroup, multiple of the tile
    int chunks_per_seg;  // workgroups per (sample, channel) segment
};

// `segments`: segments that contribute workgroups to one scheduling unit
// (num_samples for a per-channel reduction, N*C for an elementwise pass);
// `budget`: workgroups wanted (reduction: cap per channel; elementwise: total).
Chunking make_chunking(size_t spatial, size_t segments, size_t budget, size_t tile, size_t min_chunk)
{
    Chunking c;
    size_t per_seg = std::max<size_t>(budget / std::max<size_t>(segments, 1), 1);
    size_t chunk = (spatial + per_seg - 1) / per_seg;
    chunk = std::max(chunk, min_chunk);
    chunk = (chunk + tile - 1) / tile * tile;
    c.chunk = chunk;
    c.chunks_per_seg = static_cast<int>((spatial + chunk - 1) / chunk);
    if (c.chunks_per_seg < 1)
        c.chunks_per_seg = 1;
    return c;
}

// ALIGNED: the address is a multiple of the vector size (dense layout); rows
// of a strided tensor may start on any element.
// STREAM: the data is not read again soon; a nontemporal load keeps it from
// displacing what should stay in the memory-side cache.
template <typename T, int VEC, bool ALIGNED = true, bool STREAM = false>
__device__ __forceinline__ void load_vec(const T* p, T (&r)[VEC])
{
    if constexpr (VEC == 1)
    {
        r[0] = STREAM ? __builtin_nontemporal_load(p) : *p;
    }
    else
    {
        typedef T V __attribute__((ext_vector_type(VEC), aligned(ALIGNED ? sizeof(T) * VEC : sizeof(T))));
        const V t = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const V*>(p))
                           : *reinterpret_cast<const V*>(p);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            r[j] = t[j];
    }
}

template <typename T, int VEC, bool ALIGNED = true>
__device__ __forceinline__ void store_vec(T* p, const T (&r)[VEC])
{
    // Outputs are written once and not read by the next kernel of the layer;
    // nontemporal stores keep them from evicting x (and dy), which the next
    // kernel reads again, from the 256 MB memory-side cache.
    if constexpr (VEC == 1)
    {
        __builtin_nontemporal_store(r[0], p);
    }
    else
    {
        typedef T V __attribute__((ext_vector_type(VEC), aligned(ALIGNED ? sizeof(T) * VEC : sizeof(T))));
        V t;
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            t[j] = r[j];
        __builtin_nontemporal_store(t, reinterpret_cast<V*>(p));
    }
}

// How a kernel walks a tensor: as it lies (dense) or row by row in vectors
// that start on any element (rows; see Place in h2x_bn_maps.hpp).
enum Layout : int
{
    kLayoutDense = 0,
    kLayoutRows = 1
};

// Where the vector at index i lies.  Worked out once per vector, from the map
// of one tensor of the launch, and shared by all of them (index splitting costs
// two multiply-high divisions; done per tensor it was a third of the
// instructions of the strided kernels).  Without vectors or index splitting
// the place is not used.
template <typename T, int VEC, int LAYOUT>
__device__ __forceinline__ Place place_at(const TensorMap& m, size_t i)
{
    Place pl{0, 0, 0, 0};
    if constexpr (VEC > 1 && LAYOUT == kLayoutRows)
        place_vector<VEC>(m, row_split<VEC>(m, i, &pl), &pl);
    return pl;
}

// The VEC elements of tensor p at index i / place pl.
template <typename T, int VEC, int LAYOUT, bool STREAM = false>
__device__ __forceinline__ void load_in(const T* p, const TensorMap& m, size_t i, const Place& pl,
                                        T (&r)[VEC])
{
    if constexpr (VEC == 1 || LAYOUT == kLayoutDense)
    {
        load_vec<T, VEC, LAYOUT == kLayoutDense, STREAM>(
            p + seg_offset<LAYOUT != kLayoutDense>(m, i), r);
    }
    else
    {
        load_vec<T, VEC, false, STREAM>(p + (row_offset(m, pl) + pl.first), r);
    }
}

// rewrite (rows layout): the elements a vector shares with the one before it
// may be stored by both (the output shares no memory with the inputs they were
// made from).
template <typename T, int VEC, int LAYOUT>
__device__ __forceinline__ void store_out(T* p, const TensorMap& m, size_t i, const Place& pl,
                                          const T (&r)[VEC], bool rewrite)
{
    if constexpr (VEC == 1 || LAYOUT == kLayoutDense)
    {
        store_vec<T, VEC, LAYOUT == kLayoutDense>(p + seg_offset<LAYOUT != kLayoutDense>(m, i), r);
    }
    else
    {
        T* q = p + (row_offset(m, pl) + pl.first);
        if (pl.skip == 0 || rewrite)
        {
            store_vec<T, VEC, false>(q, r);
        }
        else
        {
#pragma unroll
            for (int j = 1; j < VEC; ++j)
                if (j >= static_cast<int>(pl.skip))
                    __builtin_nontemporal_store(r[j], q + j);
        }
    }
}

__device__ __forceinline__ float fma_t(float a, float b, float c)
{
    return __builtin_fmaf(a, b, c);
}
__device__ __forceinline__ double fma_t(double a, double b, double c)
{
    return __builtin_fma(a, b, c);
}
__device__ __forceinline__ float inv_sqrt_t(float v)
{
    return 1.0f / __builtin_sqrtf(v);
}
__device__ __forceinline__ double inv_sqrt_t(double v)
{
    return 1.0 / __builtin_sqrt(v);
}

// Combines the K per-thread sums of a workgroup.  With a single workgroup per
// channel returns true (totals in acc[], to be written by the caller);
// otherwise stores this workgroup's partials for the finishing kernel.
template <int K>
__device__ __forceinline__ bool finish_workgroup(double (&acc)[K], double* partials, int channel,
                                                 int groups_per_channel_max, bool always_partials)
{
    __shared__ double lds[K * kWavesPerBlock];
    block_sum<K>(acc, lds);
    if (gridDim.x == 1 && !always_partials)
        return true;
    if (threadIdx.x == 0)
    {
        double* mine = partials
                       + (static_cast<size_t>(channel) * groups_per_channel_max + blockIdx.x) * K;
#pragma unroll
        for (int k = 0; k < K; ++k)
            mine[k] = acc[k];
    }
    return false;
}

// Adds the `groups` partials of every channel in index order: thread t takes
// partials t, t + 256, ...; the workgroup then combines its threads in the
// fixed order of block_sum.  out_k[c] receives sum k of channel c.
template <typename T, int K>
__global__ __launch_bounds__(kBlockSize) void bn_finish_kernel(
    const double* __restrict__ partials, int groups, int groups_per_channel_max, T* out0, T* out1,
    T* out2, T* out3)
{
    __shared__ double lds[K * kWavesPerBlock];
    const int c = blockIdx.x;
    const double* mine = partials + static_cast<size_t>(c) * groups_per_channel_max * K;
    double t[K];
#pragma unroll
    for (int k = 0; k < K; ++k)
        t[k] = 0.0;
    for (int g = threadIdx.x; g < groups; g += kBlockSize)
    {
#pragma unroll
        for (int k = 0; k < K; ++k)
            t[k] += mine[static_cast<size_t>(g) * K + k];
    }
    block_sum<K>(t, lds);
    if (threadIdx.x == 0)
    {
        T* outs[4] = {out0, out1, out2, out3};
#pragma unroll
        for (int k = 0; k < K; ++k)
            outs[k][c] = static_cast<T>(t[k]);
    }
}

// The K sums of channel c from its `groups` partials, in the order of
// bn_finish_kernel (so a consumer that adds them itself gets the same bits).
template <int K>
__device__ __forceinline__ void channel_totals(const double* __restrict__ partials, int groups,
                                               int groups_per_channel_max, int c, double (&t)[K],
                                               double* lds)
{
    const double* mine = partials + static_cast<size_t>(c) * groups_per_channel_max * K;
#pragma unroll
    for (int k = 0; k < K; ++k)
        t[k] = 0.0;
    for (int g = threadIdx.x; g < groups; g += kBlockSize)
    {
#pragma unroll
        for (int k = 0; k < K; ++k)
            t[k] += mine[static_cast<size_t>(g) * K + k];
    }
    block_sum<K>(t, lds);
}

// What the statistics kernel below makes of a channel's sum and sum of squares.
template <typename T>
__device__ __forceinline__ void sums_to_mean_var(T sum, T sqsum, T n, T* mean, T* var)
{
    const T m = sum / n;
    const T sqmean = sqsum / n;
    T v = fma_t(-m, m, sqmean);
    v = v > T(0) ? v : T(0);
    v *= n / (n - T(1));
    *mean = m;
    *var = v;
}

// ---- forward: sums and sums of squares --------------------------------------
// Replaces channel_sums_and_sqsums_opt_kernel, batchnorm.cu:92-132.
template <typename T, int VEC, bool STRIDED>
__global__ __launch_bounds__(kBlockSize) void bn_sums_kernel(
    const T* __restrict__ x, T* __restrict__ sums, T* __restrict__ sqsums, double* partials,
    const TensorMap mx, size_t spatial, size_t chunk, int chunks_per_seg, unsigned int num_units,
    int groups_per_channel_max, bool always_partials)
{
    const int c = blockIdx.y;
    constexpr int LAYOUT = STRIDED ? kLayoutRows : kLayoutDense;
    constexpr size_t kStride = static_cast<size_t>(kBlockSize) * VEC;
    constexpr size_t kTile = kStride * kUnroll;
    double acc[2] = {0.0, 0.0};

    auto accumulate = [&](T v) {
        const double d = static_cast<double>(v);
        acc[0] += d;
        if constexpr (sizeof(T) == 4)
            acc[1] = __builtin_fma(d, d, acc[1]); // the product of two floats is exact in fp64
        else
            acc[1] += d * d;
    };

    // unit = (sample, chunk); a workgroup takes units blockIdx.x, blockIdx.x + gridDim.x, ...
    for (unsigned int unit = blockIdx.x; unit < num_units; unit += gridDim.x)
    {
        const int n = unit / chunks_per_seg;
        const int k = unit - n * chunks_per_seg;
        const size_t begin = static_cast<size_t>(k) * chunk;
        const size_t end = begin + chunk < spatial ? begin + chunk : spatial;
        const T* p = x + n * mx.stride_n + c * mx.stride_c;
        size_t tile = begin;
        for (; tile + kTile <= end; tile += kTile)
        {
            T v[kUnroll][VEC];
            uint32_t skip[kUnroll];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
            {
                const size_t i = tile + u * kStride + threadIdx.x * VEC;
                const Place pl = place_at<T, VEC, LAYOUT>(mx, i);
                load_in<T, VEC, LAYOUT>(p, mx, i, pl, v[u]);
                skip[u] = pl.skip;
            }
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    if (j >= static_cast<int>(skip[u]))
                        accumulate(v[u][j]);
        }
        for (size_t i = tile + threadIdx.x * VEC; i + VEC <= end; i += kStride)
        {
            T v[VEC];
            const Place pl = place_at<T, VEC, LAYOUT>(mx, i);
            load_in<T, VEC, LAYOUT>(p, mx, i, pl, v);
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                if (j >= static_cast<int>(pl.skip))
                    accumulate(v[j]);
        }
    }
    if (finish_workgroup<2>(acc, partials, c, groups_per_channel_max, always_partials)
        && threadIdx.x == 0)
    {
        sums[c] = static_cast<T>(acc[0]);
        sqsums[c] = static_cast<T>(acc[1]);
    }
}

template <typename T>
__global__ void fill_kernel(T* p, size_t n, T value)
{
    for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < n;
         i += static_cast<size_t>(gridDim.x) * blockDim.x)
        p[i] = value;
}

// ---- forward: sums -> mean / unbiased variance / running statistics ---------
// Replaces sums_to_statistics_functor, batchnorm.cu:288-346.
template <typename T>
__global__ void bn_statistics_kernel(int num_channels, size_t num_per_sum, T decay, T* mean,
                                     T* var, T* running_mean, T* running_var)
{
    const T n = static_cast<T>(num_per_sum);
    for (int c = blockIdx.x * blockDim.x + threadIdx.x; c < num_channels;
         c += gridDim.x * blockDim.x)
    {
        if (num_per_sum == 0)
        {
            var[c] = T(1);
            continue;
        }
        T m, v;
        sums_to_mean_var(mean[c], var[c], n, &m, &v);
        mean[c] = m;
        var[c] = v;
        running_mean[c] = fma_t(decay, running_mean[c], (T(1) - decay) * m);
        running_var[c] = fma_t(decay, running_var[c], (T(1) - decay) * v);
    }
}

// What a consumer kernel needs to finish a reduction itself: the partial sums
// the reduction kernel left in the workspace, and where the channel results go.
// Every workgroup of a channel adds that channel's partials in the order of
// bn_finish_kernel and so arrives at the same bits; the channel's first
// workgroup stores them.  Saves the finishing launch (and, forward, the
// statistics launch) when no all-reduce sits between the two stages.
template <typename T>
struct FusedStats
{
    const double* partials;
    int groups;
    int groups_per_channel_max;
    size_t num_per_sum;
    T decay;
    T* out[4];          // forward: mean, var, running_mean, running_var; backward: dscale, dbias, dmean, dvar
    bool sequential;    // the partials come from a short-segment kernel and are added one after the other
};

// ---- forward: normalise ------------------------------------------------------
// Replaces batch_normalization_opt_kernel, batchnorm.cu:420-455.  FUSED: mean
// and variance are not read but made from the partial sums of bn_sums_kernel
// (bn_finish_kernel + bn_statistics_kernel folded in).
template <typename T, int VEC, int LAYOUT, bool FUSED = false>
__global__ __launch_bounds__(kBlockSize) void bn_apply_kernel(
    const T* __restrict__ x, const T* __restrict__ mean, const T* __restrict__ var,
    const T* __restrict__ scale, const T* __restrict__ bias, T* __restrict__ y, T epsilon,
    int num_channels, size_t spatial, const TensorMap mx, const TensorMap my, size_t chunk,
    int chunks_per_seg, const FusedStats<T> fused = FusedStats<T>())
{
    const size_t seg = blockIdx.x / chunks_per_seg;
    const int k = blockIdx.x - seg * chunks_per_seg;
    const int c = seg % num_channels;
    T m, variance;
    if constexpr (FUSED)
    {
        __shared__ double lds[2 * kWavesPerBlock];
        double t[2];
        channel_totals<2>(fused.partials, fused.groups, fused.groups_per_channel_max, c, t, lds);
        sums_to_mean_var(static_cast<T>(t[0]), static_cast<T>(t[1]),
                         static_cast<T>(fused.num_per_sum), &m, &variance);
        if (seg < static_cast<size_t>(num_channels) && k == 0 && threadIdx.x == 0) // sample 0, chunk 0
        {
            fused.out[0][c] = m;
            fused.out[1][c] = variance;
            fused.out[2][c] = fma_t(fused.decay, fused.out[2][c], (T(1) - fused.decay) * m);
            fused.out[3][c] = fma_t(fused.decay, fused.out[3][c], (T(1) - fused.decay) * variance);
        }
    }
    else
    {
        m = mean[c];
        variance = var[c];
    }
    const T inv_stdev = inv_sqrt_t(variance + epsilon);
    const T sc = scale[c];
    const T bi = bias[c];
    const size_t begin = static_cast<size_t>(k) * chunk;
    const size_t end = begin + chunk < spatial ? begin + chunk : spatial;
    const size_t n = seg / num_channels;
    const T* xp = x + n * mx.stride_n + c * mx.stride_c;
    T* yp = y + n * my.stride_n + c * my.stride_c;

    constexpr size_t kStride = static_cast<size_t>(kBlockSize) * VEC;
    constexpr size_t kTile = kStride * kUnroll;
    size_t tile = begin;
    for (; tile + kTile <= end; tile += kTile)
    {
        T v[kUnroll][VEC];
        Place pl[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
        {
            const size_t i = tile + u * kStride + threadIdx.x * VEC;
            pl[u] = place_at<T, VEC, LAYOUT>(my, i);
            load_in<T, VEC, LAYOUT>(xp, mx, i, pl[u], v[u]);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
        {
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                v[u][j] = fma_t((v[u][j] - m) * inv_stdev, sc, bi);
            store_out<T, VEC, LAYOUT>(yp, my, tile + u * kStride + threadIdx.x * VEC, pl[u], v[u], true);
        }
    }
    for (size_t i = tile + threadIdx.x * VEC; i + VEC <= end; i += kStride)
    {
        T v[VEC];
        const Place pl = place_at<T, VEC, LAYOUT>(my, i);
        load_in<T, VEC, LAYOUT>(xp, mx, i, pl, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            v[j] = fma_t((v[j] - m) * inv_stdev, sc, bi);
        store_out<T, VEC, LAYOUT>(yp, my, i, pl, v, true);
    }
}

// ---- backward: per-channel sums ----------------------------------------------
// Replaces backprop1_opt_kernel, batchnorm.cu:982-1054.
template <typename T, int VEC, bool STRIDED>
__global__ __launch_bounds__(kBlockSize) void bn_backprop1_kernel(
    const T* __restrict__ x, const T* __restrict__ dy, const T* __restrict__ mean,
    const T* __restrict__ var, const T* __restrict__ scale, T* __restrict__ dscale,
    T* __restrict__ dbias, T* __restrict__ dmean, T* __restrict__ dvar, T epsilon,
    double* partials, size_t spatial, const TensorMap mx, const TensorMap md, size_t chunk,
    int chunks_per_seg, unsigned int num_units, int groups_per_channel_max, bool always_partials)
{
    const int c = blockIdx.y;
    const T m = mean[c];
    const T sc = scale[c];
    const T inv_stdev = inv_sqrt_t(var[c] + epsilon);
    const T dvar_factor = inv_stdev * inv_stdev * inv_stdev / T(2);
    const double neg_inv = -static_cast<double>(inv_stdev);
    const double neg_fac = -static_cast<double>(dvar_factor);

    constexpr int LAYOUT = STRIDED ? kLayoutRows : kLayoutDense;
    constexpr size_t kStride = static_cast<size_t>(kBlockSize) * VEC;
    constexpr int kUnroll2 = kUnroll / 2; // two streams: same bytes in flight
    constexpr size_t kTile = kStride * kUnroll2;
    double acc[4] = {0.0, 0.0, 0.0, 0.0};

    auto accumulate = [&](T xv, T dv) {
        const T xm = xv - m;
        const T xhat = xm * inv_stdev;
        const T dxhat = dv * sc;
        const T t = dxhat * xm;
        const double dd = static_cast<double>(dv);
        acc[0] = __builtin_fma(dd, static_cast<double>(xhat), acc[0]);
        acc[1] += dd;
        acc[2] = __builtin_fma(static_cast<double>(dxhat), neg_inv, acc[2]);
        acc[3] = __builtin_fma(static_cast<double>(t), neg_fac, acc[3]);
    };

    for (unsigned int unit = blockIdx.x; unit < num_units; unit += gridDim.x)
    {
        const int n = unit / chunks_per_seg;
        const int k = unit - n * chunks_per_seg;
        const size_t begin = static_cast<size_t>(k) * chunk;
        const size_t end = begin + chunk < spatial ? begin + chunk : spatial;
        const T* xp = x + n * mx.stride_n + c * mx.stride_c;
        const T* dp = dy + n * md.stride_n + c * md.stride_c;
        size_t tile = begin;
        for (; tile + kTile <= end; tile += kTile)
        {
            T xv[kUnroll2][VEC], dv[kUnroll2][VEC];
            uint32_t skip[kUnroll2];
#pragma unroll
            for (int u = 0; u < kUnroll2; ++u)
            {
                const size_t i = tile + u * kStride + threadIdx.x * VEC;
                const Place pl = place_at<T, VEC, LAYOUT>(mx, i);
                load_in<T, VEC, LAYOUT>(xp, mx, i, pl, xv[u]);
                load_in<T, VEC, LAYOUT, true>(dp, md, i, pl, dv[u]);
                skip[u] = pl.skip;
            }
#pragma unroll
            for (int u = 0; u < kUnroll2; ++u)
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    if (j >= static_cast<int>(skip[u]))
                        accumulate(xv[u][j], dv[u][j]);
        }
        for (size_t i = tile + threadIdx.x * VEC; i + VEC <= end; i += kStride)
        {
            T xv[VEC], dv[VEC];
            const Place pl = place_at<T, VEC, LAYOUT>(mx, i);
            load_in<T, VEC, LAYOUT>(xp, mx, i, pl, xv);
            load_in<T, VEC, LAYOUT, true>(dp, md, i, pl, dv);
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                if (j >= static_cast<int>(pl.skip))
                    accumulate(xv[j], dv[j]);
        }
    }
    if (finish_workgroup<4>(acc, partials, c, groups_per_channel_max, always_partials)
        && threadIdx.x == 0)
    {
        dscale[c] = static_cast<T>(acc[0]);
        dbias[c] = static_cast<T>(acc[1]);
        dmean[c] = static_cast<T>(acc[2]);
        dvar[c] = static_cast<T>(acc[3]);
    }
}

// ---- backward: input gradient ------------------------------------------------
// Replaces backprop2_opt_kernel, batchnorm.cu:1371-1418.  x and dx may alias:
// each thread reads its elements before it writes them, so neither is
// restrict-qualified (`disjoint`: they share no memory).
template <typename T, int VEC, int LAYOUT, bool FUSED = false>
__global__ __launch_bounds__(kBlockSize) void bn_backprop2_kernel(
    const T* x, const T* __restrict__ dy, const T* __restrict__ mean,
    const T* __restrict__ var, const T* __restrict__ scale, const T* __restrict__ dmean,
    const T* __restrict__ dvar, T* dx, T epsilon, size_t num_per_sum, int num_channels,
    size_t spatial, const TensorMap mx, const TensorMap md, const TensorMap mo, size_t chunk,
    int chunks_per_seg, bool disjoint, const FusedStats<T> fused = FusedStats<T>())
{
    const size_t seg = blockIdx.x / chunks_per_seg;
    const int k = blockIdx.x - seg * chunks_per_seg;
    const int c = seg % num_channels;
    const T m = mean[c];
    const T sc = scale[c];
    const T inv_stdev = inv_sqrt_t(var[c] + epsilon);
    T dmean_c, dvar_c;
    if constexpr (FUSED)
    {
        // the four sums of bn_backprop1_kernel, finished here (bn_finish_kernel folded in)
        __shared__ double lds[4 * kWavesPerBlock];
        double t[4];
        channel_totals<4>(fused.partials, fused.groups, fused.groups_per_channel_max, c, t, lds);
        dmean_c = static_cast<T>(t[2]);
        dvar_c = static_cast<T>(t[3]);
        if (seg < static_cast<size_t>(num_channels) && k == 0 && threadIdx.x == 0)
        {
            fused.out[0][c] = static_cast<T>(t[0]);
            fused.out[1][c] = static_cast<T>(t[1]);
            fused.out[2][c] = dmean_c;
            fused.out[3][c] = dvar_c;
        }
    }
    else
    {
        dmean_c = dmean[c];
        dvar_c = dvar[c];
    }
    const T dmean_term = dmean_c / static_cast<T>(num_per_sum);
    const T dvar_term = dvar_c * T(2) / static_cast<T>(num_per_sum - 1);
    const size_t begin = static_cast<size_t>(k) * chunk;
    const size_t end = begin + chunk < spatial ? begin + chunk : spatial;
    const size_t n = seg / num_channels;
    const T* xp = x + n * mx.stride_n + c * mx.stride_c;
    const T* dp = dy + n * md.stride_n + c * md.stride_c;
    T* op = dx + n * mo.stride_n + c * mo.stride_c;

    constexpr size_t kStride = static_cast<size_t>(kBlockSize) * VEC;
    constexpr int kUnroll2 = kUnroll / 2;
    constexpr size_t kTile = kStride * kUnroll2;
    size_t tile = begin;
    for (; tile + kTile <= end; tile += kTile)
    {
        T xv[kUnroll2][VEC], dv[kUnroll2][VEC];
        Place pl[kUnroll2];
#pragma unroll
        for (int u = 0; u < kUnroll2; ++u)
        {
            const size_t i = tile + u * kStride + threadIdx.x * VEC;
            pl[u] = place_at<T, VEC, LAYOUT>(mo, i);
            load_in<T, VEC, LAYOUT>(xp, mx, i, pl[u], xv[u]);
            load_in<T, VEC, LAYOUT, true>(dp, md, i, pl[u], dv[u]);
        }
#pragma unroll
        for (int u = 0; u < kUnroll2; ++u)
        {
#pragma unroll
            for (int j = 0; j < VEC; ++j)
            {
                T r = fma_t(dv[u][j] * sc, inv_stdev, dmean_term);
                xv[u][j] = fma_t(xv[u][j] - m, dvar_term, r);
            }
            store_out<T, VEC, LAYOUT>(op, mo, tile + u * kStride + threadIdx.x * VEC, pl[u], xv[u], disjoint);
        }
    }
    for (size_t i = tile + threadIdx.x * VEC; i + VEC <= end; i += kStride)
    {
        T xv[VEC], dv[VEC];
        const Place pl = place_at<T, VEC, LAYOUT>(mo, i);
        load_in<T, VEC, LAYOUT>(xp, mx, i, pl, xv);
        load_in<T, VEC, LAYOUT, true>(dp, md, i, pl, dv);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
        {
            T r = fma_t(dv[j] * sc, inv_stdev, dmean_term);
            xv[j] = fma_t(xv[j] - m, dvar_term, r);
        }
        store_out<T, VEC, LAYOUT>(op, mo, i, pl, xv, disjoint);
    }
}

// ---- normalise / input gradient that leave the halo of their output cleared ----
// For tensors that share one haloed geometry.  The kernel walks the REAL local
// tensor of every (sample, channel) segment - interior and halo cells alike - in
// aligned 16-byte vectors, computes the interior elements and stores zeros into
// the halo cells: what the reference's kernel followed by Tensor::clear_halo on
// every spatial dimension leaves (legacy/src/tensor/tensor_mpi_cuda.cu:14-84;
// Convolution::forward clears the halos of its input before every exchange,
// legacy/include/distconv/dnn_backend/convolution.hpp:400-411), in one pass and
// without the partly written sectors that the gaps between interior rows cost
// the kernels above.  Halo cells of the inputs are loaded and ignored.
// BACKWARD: the input gradient (x, dy -> dx); else normalise (x -> y).  Segments
// are `real` elements long and follow one another (channel stride = real).
template <typename T, int VEC, bool BACKWARD>
__global__ __launch_bounds__(kBlockSize) void bn_clearing_kernel(
    const T* x, const T* __restrict__ dy, const T* __restrict__ mean, const T* __restrict__ var,
    const T* __restrict__ scale, const T* __restrict__ bias, const T* __restrict__ dmean,
    const T* __restrict__ dvar, T* out, T epsilon, size_t num_per_sum, int num_channels, size_t real,
    const RealBox box, size_t chunk, int chunks_per_seg)
{
    const size_t seg = blockIdx.x / chunks_per_seg;
    const int k = blockIdx.x - seg * chunks_per_seg;
    const int c = seg % num_channels;
    const T m = mean[c];
    const T sc = scale[c];
    const T inv_stdev = inv_sqrt_t(var[c] + epsilon);
    T bi = T(0), dmean_term = T(0), dvar_term = T(0);
    if constexpr (BACKWARD)
    {
        dmean_term = dmean[c] / static_cast<T>(num_per_sum);
        dvar_term = dvar[c] * T(2) / static_cast<T>(num_per_sum - 1);
    }
    else
    {
        bi = bias[c];
    }
    const size_t begin = static_cast<size_t>(k) * chunk;
    const size_t end = begin + chunk < real ? begin + chunk : real;
    const T* xp = x + seg * real;
    const T* dp = BACKWARD ? dy + seg * real : nullptr;
    T* op = out + seg * real;

    auto result = [&](T xv, T dv) {
        if constexpr (BACKWARD)
            return fma_t(xv - m, dvar_term, fma_t(dv * sc, inv_stdev, dmean_term));
        else
            return fma_t((xv - m) * inv_stdev, sc, bi);
    };
    constexpr size_t kStride = static_cast<size_t>(kBlockSize) * VEC;
    constexpr int kInFlight = BACKWARD ? kUnroll / 2 : kUnroll;
    constexpr size_t kTile = kStride * kInFlight;
    size_t tile = begin;
    for (; tile + kTile <= end; tile += kTile)
    {
        T xv[kInFlight][VEC], dv[kInFlight][VEC];
#pragma unroll
        for (int u = 0; u < kInFlight; ++u)
        {
            const size_t i = tile + u * kStride + threadIdx.x * VEC;
            load_vec<T, VEC, true>(xp + i, xv[u]);
            if constexpr (BACKWARD)
                load_vec<T, VEC, true, true>(dp + i, dv[u]);
        }
#pragma unroll
        for (int u = 0; u < kInFlight; ++u)
        {
            const size_t i = tile + u * kStride + threadIdx.x * VEC;
            bool inside[VEC];
            interior_mask<VEC>(box, static_cast<uint32_t>(i), inside);
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                xv[u][j] = inside[j] ? result(xv[u][j], BACKWARD ? dv[u][j] : T(0)) : T(0);
            store_vec<T, VEC, true>(op + i, xv[u]);
        }
    }
    for (size_t i = tile + threadIdx.x * VEC; i + VEC <= end; i += kStride)
    {
        T xv[VEC], dv[VEC];
        load_vec<T, VEC, true>(xp + i, xv);
        if constexpr (BACKWARD)
            load_vec<T, VEC, true, true>(dp + i, dv);
        bool inside[VEC];
        interior_mask<VEC>(box, static_cast<uint32_t>(i), inside);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            xv[j] = inside[j] ? result(xv[j], BACKWARD ? dv[j] : T(0)) : T(0);
        store_vec<T, VEC, true>(op + i, xv);
    }
}

// ---- short segments: whole channels side by side in one workgroup ------------
// A (sample, channel) segment of a few hundred bytes (7 x 7 or 14 x 14
// activations, 1 x 1 after a fully connected layer) shares its first and last
// cache line with the neighbouring channels.  A workgroup per channel that walks
// from sample to sample then fetches 2-3 lines for 196 bytes and leaves its
// output as partial lines (N 256, C 2048, 7 x 7: 169 MB read and 637 k partial
// writes for a 103 MB tensor; 106 MB read here, forward 102 us -> 52 us,
// backward 170 us -> 91 us; N 512, C 4096, 1 x 1: 100 -> 12 us, 138 -> 25 us).
// These kernels give a workgroup a window of
// neighbouring whole channels instead -- one contiguous piece of memory per
// sample -- and walk through a range of samples.  A segment is padded to
// `slots` vectors; lane t serves slot t mod slots of channel t div slots for
// every sample, so its channel and that channel's parameters are fixed for the
// whole kernel.  The last slot of a segment whose length is no multiple of the
// vector owns fewer elements: its vector starts that much earlier, so that it
// is still loaded whole, overlaps the slot before it, and only the elements it
// owns are added up or stored (kTailOverlap; in place of x, dx may be written
// by the neighbouring lane before this lane reads the overlap, which it does
// not use).  Segments shorter than a vector move element by element
// (kTailScalar).  When a tensor of the launch has halos inside its segments
// the slots follow the rows of the segment instead (each row padded to whole
// vectors, the last vector of a row overlapping the one before it), so that a
// slot is contiguous in every tensor; where it starts in each tensor is worked
// out once, as the lane's place in the segment never changes (N 32, C 512,
// 14 x 14 with a halo of 1: forward 34 -> 14 us, backward 46 -> 20 us against
// the strided kernels, which give such a segment a workgroup of its own).
// Where few
// channels and many samples would leave a reduction with too few workgroups,
// the lanes of a workgroup form `rows` rows that take every rows-th sample of
// a narrower window.
template <typename T, int VEC, int TAIL, bool STREAM = false>
__device__ __forceinline__ void load_slot(const T* p, const ShortLane& l, T (&r)[VEC])
{
    if constexpr (TAIL != kTailScalar)
    {
        load_vec<T, VEC, false, STREAM>(p, r);
    }
    else
    {
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            r[j] = T(0);
#pragma unroll
        for (int j = 0; j < VEC - 1; ++j)
            if (j < l.valid)
                r[j] = STREAM ? __builtin_nontemporal_load(p + j) : p[j];
    }
}

// rewrite: the output does not alias an input, so the elements in which the
// last vector of a row overlaps its neighbour may be stored by both lanes (each
// made the same values from the same inputs) and every lane stores a whole vector.
template <typename T, int VEC, int TAIL>
__device__ __forceinline__ void store_slot(T* p, const ShortLane& l, const T (&r)[VEC],
                                           bool rewrite)
{
    if (TAIL == kTailNone || (TAIL == kTailOverlap && (rewrite || l.skip == 0)))
    {
        store_vec<T, VEC, false>(p, r);
    }
    else
    {
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            if (slot_owns<VEC, TAIL>(l, j))
                __builtin_nontemporal_store(r[j], p + j);
    }
}

// The K sums of channel c from its `groups` partials, one after the other.  The
// finishing kernel and the consumers that finish a reduction themselves both
// add in this order and so arrive at the same bits.  The short-segment kernels
// keep their partials group by group, partials[(group * C + c) * K + k]:
// neighbouring lanes, which serve neighbouring channels, then read neighbouring
// memory (at most groups_per_channel_max * C * K values, like the other layout).
template <int K>
__device__ __forceinline__ void sequential_totals(const double* __restrict__ partials, int groups,
                                                  int num_channels, int c, double (&t)[K])
{
    const double* mine = partials + static_cast<size_t>(c) * K;
    const size_t pitch = static_cast<size_t>(num_channels) * K;
#pragma unroll
    for (int k = 0; k < K; ++k)
        t[k] = mine[k];
    // four groups' loads are issued together: the additions wait for one memory
    // latency per batch instead of one per group
    for (int g0 = 1; g0 < groups; g0 += 4)
    {
        double p[4][K];
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int k = 0; k < K; ++k)
                p[u][k] = g0 + u < groups ? mine[(g0 + u) * pitch + k] : 0.0;
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int k = 0; k < K; ++k)
                if (g0 + u < groups)
                    t[k] += p[u][k];
    }
}

// Adds what the lanes of each channel hold and stores the
// channel's partial sums of this range of samples, or, when the launch has a
// single range and nobody else finishes the reduction, the results themselves.
template <typename T, int K>
__device__ __forceinline__ void finish_short(const ShortGeometry& g, const ShortLane& l,
                                             const double (&acc)[K], double* partials,
                                             bool always_partials, T* const (&out)[K])
{
    __shared__ double lds[K][kBlockSize];
#pragma unroll
    for (int k = 0; k < K; ++k)
        lds[k][threadIdx.x] = acc[k];
    __syncthreads();
    // The slots of a channel in one row are added as a tree (lane v takes what
    // lane v + step holds, step = 2^k downwards), then the channel's first lane
    // adds the rows one after the other: a fixed order, a handful of steps.
    double t[K];
#pragma unroll
    for (int k = 0; k < K; ++k)
        t[k] = acc[k];
    int width = 1;
    while (width < g.slots)
        width <<= 1;
    for (int step = width >> 1; step >= 1; step >>= 1)
    {
        // lanes below `step` read lanes from `step` on and write their own: one barrier a step
        if (l.valid > 0 && l.slot < step && l.slot + step < g.slots)
        {
#pragma unroll
            for (int k = 0; k < K; ++k)
            {
                t[k] += lds[k][threadIdx.x + step];
                lds[k][threadIdx.x] = t[k];
            }
        }
        __syncthreads();
    }
    if (l.leads)
    {
        const int lanes_per_row = kBlockSize / g.rows;
        for (int r = 1; r < g.rows; ++r)
        {
#pragma unroll
            for (int k = 0; k < K; ++k)
                t[k] += lds[k][threadIdx.x + r * lanes_per_row];
        }
    }
    if (!l.leads)
        return;
    if (gridDim.y == 1 && !always_partials)
    {
#pragma unroll
        for (int k = 0; k < K; ++k)
            out[k][l.c] = static_cast<T>(t[k]);
    }
    else
    {
        double* mine =
            partials + (static_cast<size_t>(blockIdx.y) * g.num_channels + l.c) * K;
#pragma unroll
        for (int k = 0; k < K; ++k)
            mine[k] = t[k];
    }
}

template <typename T, int K>
__global__ void bn_finish_short_kernel(const double* __restrict__ partials, int groups,
                                       int num_channels, T* out0, T* out1, T* out2, T* out3)
{
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= num_channels)
        return;
    double t[K];
    sequential_totals<K>(partials, groups, num_channels, c, t);
    T* outs[4] = {out0, out1, out2, out3};
#pragma unroll
    for (int k = 0; k < K; ++k)
        outs[k][c] = static_cast<T>(t[k]);
}

template <typename T, int VEC, int TAIL>
__global__ __launch_bounds__(kBlockSize) void bn_sums_short_kernel(
    const T* __restrict__ x, T* __restrict__ sums, T* __restrict__ sqsums, double* partials,
    const ShortTensor tx, const ShortGeometry g, bool always_partials)
{
    const ShortLane l = short_lane<VEC, TAIL>(g, static_cast<int>(threadIdx.x), static_cast<int>(blockIdx.x));
    double acc[2] = {0.0, 0.0};
    if (l.valid > 0)
    {
        auto accumulate = [&](const T (&v)[VEC]) {
#pragma unroll
            for (int j = 0; j < VEC; ++j)
            {
                if (!slot_owns<VEC, TAIL>(l, j))
                    continue;
                const double d = static_cast<double>(v[j]);
                acc[0] += d;
                if constexpr (sizeof(T) == 4)
                    acc[1] = __builtin_fma(d, d, acc[1]); // the product of two floats is exact in fp64
                else
                    acc[1] += d * d;
            }
        };
        const T* p = x + l.c * tx.stride_c + slot_offset(l, tx);
        const int64_t stride_n = tx.stride_n;
        int n = blockIdx.y * g.samples_per_group;
        const int end = n + g.samples_per_group < g.num_samples ? n + g.samples_per_group
                                                                : g.num_samples;
        const int step = g.rows;
        n += l.row;
        for (; n + (kUnroll - 1) * step < end; n += kUnroll * step)
        {
            T v[kUnroll][VEC];
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
                load_slot<T, VEC, TAIL>(p + (n + u * step) * stride_n, l, v[u]);
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
                accumulate(v[u]);
        }
        for (; n < end; n += step)
        {
            T v[VEC];
            load_slot<T, VEC, TAIL>(p + n * stride_n, l, v);
            accumulate(v);
        }
    }
    T* const out[2] = {sums, sqsums};
    finish_short<T, 2>(g, l, acc, partials, always_partials, out);
}

template <typename T, int VEC, int TAIL, bool FUSED>
__global__ __launch_bounds__(kBlockSize) void bn_apply_short_kernel(
    const T* __restrict__ x, const T* __restrict__ mean, const T* __restrict__ var,
    const T* __restrict__ scale, const T* __restrict__ bias, T* __restrict__ y, T epsilon,
    const ShortTensor tx, const ShortTensor ty, const ShortGeometry g, const FusedStats<T> fused)
{
    const ShortLane l = short_lane<VEC, TAIL>(g, static_cast<int>(threadIdx.x), static_cast<int>(blockIdx.x));
    T m = T(0), variance = T(0);
    if constexpr (FUSED)
    {
        __shared__ T stats[2][kBlockSize];
        if (l.leads)
        {
            double t[2];
            sequential_totals<2>(fused.partials, fused.groups, g.num_channels, l.c, t);
            sums_to_mean_var(static_cast<T>(t[0]), static_cast<T>(t[1]),
                             static_cast<T>(fused.num_per_sum), &m, &variance);
            stats[0][l.q] = m;
            stats[1][l.q] = variance;
            if (blockIdx.y == 0)
            {
                fused.out[0][l.c] = m;
                fused.out[1][l.c] = variance;
                fused.out[2][l.c] = fma_t(fused.decay, fused.out[2][l.c], (T(1) - fused.decay) * m);
                fused.out[3][l.c] =
                    fma_t(fused.decay, fused.out[3][l.c], (T(1) - fused.decay) * variance);
            }
        }
        __syncthreads();
        if (l.valid > 0)
        {
            m = stats[0][l.q];
            variance = stats[1][l.q];
        }
    }
    else if (l.valid > 0)
    {
        m = mean[l.c];
        variance = var[l.c];
    }
    if (l.valid == 0)
        return;
    const T inv_stdev = inv_sqrt_t(variance + epsilon);
    const T sc = scale[l.c];
    const T bi = bias[l.c];
    const T* xp = x + l.c * tx.stride_c + slot_offset(l, tx);
    T* yp = y + l.c * ty.stride_c + slot_offset(l, ty);
    const int64_t x_stride_n = tx.stride_n, y_stride_n = ty.stride_n;
    int n = blockIdx.y * g.samples_per_group;
    const int end =
        n + g.samples_per_group < g.num_samples ? n + g.samples_per_group : g.num_samples;
    for (; n + kUnroll <= end; n += kUnroll)
    {
        T v[kUnroll][VEC];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
            load_slot<T, VEC, TAIL>(xp + (n + u) * x_stride_n, l, v[u]);
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
        {
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                v[u][j] = fma_t((v[u][j] - m) * inv_stdev, sc, bi);
            store_slot<T, VEC, TAIL>(yp + (n + u) * y_stride_n, l, v[u], true);
        }
    }
    for (; n < end; ++n)
    {
        T v[VEC];
        load_slot<T, VEC, TAIL>(xp + n * x_stride_n, l, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            v[j] = fma_t((v[j] - m) * inv_stdev, sc, bi);
        store_slot<T, VEC, TAIL>(yp + n * y_stride_n, l, v, true);
    }
}

template <typename T, int VEC, int TAIL>
__global__ __launch_bounds__(kBlockSize) void bn_backprop1_short_kernel(
    const T* __restrict__ x, const T* __restrict__ dy, const T* __restrict__ mean,
    const T* __restrict__ var, const T* __restrict__ scale, T* __restrict__ dscale,
    T* __restrict__ dbias, T* __restrict__ dmean, T* __restrict__ dvar, T epsilon,
    double* partials, const ShortTensor tx, const ShortTensor td, const ShortGeometry g,
    bool always_partials)
{
    const ShortLane l = short_lane<VEC, TAIL>(g, static_cast<int>(threadIdx.x), static_cast<int>(blockIdx.x));
    double acc[4] = {0.0, 0.0, 0.0, 0.0};
    if (l.valid > 0)
    {
        const T m = mean[l.c];
        const T sc = scale[l.c];
        const T inv_stdev = inv_sqrt_t(var[l.c] + epsilon);
        const T dvar_factor = inv_stdev * inv_stdev * inv_stdev / T(2);
        const double neg_inv = -static_cast<double>(inv_stdev);
        const double neg_fac = -static_cast<double>(dvar_factor);
        auto accumulate = [&](const T (&xv)[VEC], const T (&dv)[VEC]) {
#pragma unroll
            for (int j = 0; j < VEC; ++j)
            {
                if (!slot_owns<VEC, TAIL>(l, j))
                    continue;
                const T xm = xv[j] - m;
                const T xhat = xm * inv_stdev;
                const T dxhat = dv[j] * sc;
                const T t = dxhat * xm;
                const double dd = static_cast<double>(dv[j]);
                acc[0] = __builtin_fma(dd, static_cast<double>(xhat), acc[0]);
                acc[1] += dd;
                acc[2] = __builtin_fma(static_cast<double>(dxhat), neg_inv, acc[2]);
                acc[3] = __builtin_fma(static_cast<double>(t), neg_fac, acc[3]);
            }
        };
        constexpr int kUnroll2 = kUnroll / 2; // two streams: same bytes in flight
        const T* xp = x + l.c * tx.stride_c + slot_offset(l, tx);
        const T* dp = dy + l.c * td.stride_c + slot_offset(l, td);
        const int64_t x_stride_n = tx.stride_n, d_stride_n = td.stride_n;
        int n = blockIdx.y * g.samples_per_group;
        const int end = n + g.samples_per_group < g.num_samples ? n + g.samples_per_group
                                                                : g.num_samples;
        const int step = g.rows;
        n += l.row;
        for (; n + (kUnroll2 - 1) * step < end; n += kUnroll2 * step)
        {
            T xv[kUnroll2][VEC], dv[kUnroll2][VEC];
#pragma unroll
            for (int u = 0; u < kUnroll2; ++u)
            {
                load_slot<T, VEC, TAIL>(xp + (n + u * step) * x_stride_n, l, xv[u]);
                load_slot<T, VEC, TAIL, true>(dp + (n + u * step) * d_stride_n, l, dv[u]);
            }
#pragma unroll
            for (int u = 0; u < kUnroll2; ++u)
                accumulate(xv[u], dv[u]);
        }
        for (; n < end; n += step)
        {
            T xv[VEC], dv[VEC];
            load_slot<T, VEC, TAIL>(xp + n * x_stride_n, l, xv);
            load_slot<T, VEC, TAIL, true>(dp + n * d_stride_n, l, dv);
            accumulate(xv, dv);
        }
    }
    T* const out[4] = {dscale, dbias, dmean, dvar};
    finish_short<T, 4>(g, l, acc, partials, always_partials, out);
}

// x and dx may alias: each lane reads its elements before it writes them
// (`disjoint`: they share no memory).
template <typename T, int VEC, int TAIL, bool FUSED>
__global__ __launch_bounds__(kBlockSize) void bn_backprop2_short_kernel(
    const T* x, const T* __restrict__ dy, const T* __restrict__ mean, const T* __restrict__ var,
    const T* __restrict__ scale, const T* __restrict__ dmean, const T* __restrict__ dvar, T* dx,
    T epsilon, size_t num_per_sum, const ShortTensor tx, const ShortTensor td,
    const ShortTensor to, const ShortGeometry g, bool disjoint, const FusedStats<T> fused)
{
    const ShortLane l = short_lane<VEC, TAIL>(g, static_cast<int>(threadIdx.x), static_cast<int>(blockIdx.x));
    T dmean_c = T(0), dvar_c = T(0);
    if constexpr (FUSED)
    {
        __shared__ T totals[2][kBlockSize];
        if (l.leads)
        {
            double t[4];
            sequential_totals<4>(fused.partials, fused.groups, g.num_channels, l.c, t);
            totals[0][l.q] = static_cast<T>(t[2]);
            totals[1][l.q] = static_cast<T>(t[3]);
            if (blockIdx.y == 0)
            {
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    fused.out[k][l.c] = static_cast<T>(t[k]);
            }
        }
        __syncthreads();
        if (l.valid > 0)
        {
            dmean_c = totals[0][l.q];
            dvar_c = totals[1][l.q];
        }
    }
    else if (l.valid > 0)
    {
        dmean_c = dmean[l.c];
        dvar_c = dvar[l.c];
    }
    if (l.valid == 0)
        return;
    const T m = mean[l.c];
    const T sc = scale[l.c];
    const T inv_stdev = inv_sqrt_t(var[l.c] + epsilon);
    const T dmean_term = dmean_c / static_cast<T>(num_per_sum);
    const T dvar_term = dvar_c * T(2) / static_cast<T>(num_per_sum - 1);
    constexpr int kUnroll2 = kUnroll / 2;
    const T* xp = x + l.c * tx.stride_c + slot_offset(l, tx);
    const T* dp = dy + l.c * td.stride_c + slot_offset(l, td);
    T* op = dx + l.c * to.stride_c + slot_offset(l, to);
    const int64_t x_stride_n = tx.stride_n, d_stride_n = td.stride_n, o_stride_n = to.stride_n;
    int n = blockIdx.y * g.samples_per_group;
    const int end =
        n + g.samples_per_group < g.num_samples ? n + g.samples_per_group : g.num_samples;
    for (; n + kUnroll2 <= end; n += kUnroll2)
    {
        T xv[kUnroll2][VEC], dv[kUnroll2][VEC];
#pragma unroll
        for (int u = 0; u < kUnroll2; ++u)
        {
            load_slot<T, VEC, TAIL>(xp + (n + u) * x_stride_n, l, xv[u]);
            load_slot<T, VEC, TAIL, true>(dp + (n + u) * d_stride_n, l, dv[u]);
        }
#pragma unroll
        for (int u = 0; u < kUnroll2; ++u)
        {
#pragma unroll
            for (int j = 0; j < VEC; ++j)
            {
                const T r = fma_t(dv[u][j] * sc, inv_stdev, dmean_term);
                xv[u][j] = fma_t(xv[u][j] - m, dvar_term, r);
            }
            store_slot<T, VEC, TAIL>(op + (n + u) * o_stride_n, l, xv[u], disjoint);
        }
    }
    for (; n < end; ++n)
    {
        T xv[VEC], dv[VEC];
        load_slot<T, VEC, TAIL>(xp + n * x_stride_n, l, xv);
        load_slot<T, VEC, TAIL, true>(dp + n * d_stride_n, l, dv);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
        {
            const T r = fma_t(dv[j] * sc, inv_stdev, dmean_term);
            xv[j] = fma_t(xv[j] - m, dvar_term, r);
        }
        store_slot<T, VEC, TAIL>(op + n * o_stride_n, l, xv, disjoint);
    }
}

// ---- host side ---------------------------------------------------------------

template <typename T>
constexpr int full_vec()
{
    return 16 / sizeof(T);
}

bool grid_ok(size_t blocks)
{
    return blocks <= 0x7fffffffull;
}

// One tensor as the kernels see it, plus what decides the vector width.
struct HostTensor
{
    TensorMap map;
    bool strided = false; // needs index splitting
    size_t row = 0;       // contiguous interior elements per row (strided) or `spatial` (dense)
    bool aligned = false; // dense: every segment starts on a 16-byte boundary
};

// Index splitting that is the identity (x = i, y = z = 0), for a dense tensor
// that takes part in a launch of the strided kernels: every index is below the
// divisor 2^31 - 1.
void set_dense_map(TensorMap* m)
{
    m->w = make_fastdiv(0x7fffffffu);
    m->h = make_fastdiv(1);
    m->sy = m->sz = 0;
    m->spr = make_fastdiv(1);
    m->width = 0;
}

template <typename T>
HostTensor dense_tensor(const void* p, int num_channels, size_t spatial, size_t real)
{
    HostTensor t;
    t.map.stride_c = static_cast<int64_t>(real);
    t.map.stride_n = static_cast<int64_t>(real) * num_channels;
    set_dense_map(&t.map);
    t.row = spatial;
    t.aligned = aligned16(p) && real % full_vec<T>() == 0;
    return t;
}

// A tensor given by local shape and strides (innermost first; channel and
// sample are the last two dimensions).  Falls back to the dense description
// when the inner spatial dimensions carry no halo.
template <typename T>
int strided_tensor(const h2x_tensor_geometry* g, const void* p, int num_samples, HostTensor* out,
                   int* num_channels, size_t* spatial)
{
    if (!g || g->num_dims < 3 || g->num_dims > 5)
        return H2X_ERR_INVALID_ARGUMENT;
    const int nd = g->num_dims, ns = nd - 2;
    size_t sp = 1;
    for (int i = 0; i < nd; ++i)
        if (g->local_shape[i] < 0 || g->strides[i] < 0)
            return H2X_ERR_INVALID_ARGUMENT;
    if (g->strides[0] != 1 && g->local_shape[0] > 1)
        return H2X_ERR_UNSUPPORTED;
    for (int i = 0; i < ns; ++i)
        sp *= static_cast<size_t>(g->local_shape[i]);
    if (g->local_shape[nd - 1] != num_samples && num_samples != 0)
        return H2X_ERR_INVALID_ARGUMENT;
    *num_channels = static_cast<int>(g->local_shape[nd - 2]);
    *spatial = sp;
    HostTensor t;
    t.map.stride_c = g->strides[nd - 2];
    t.map.stride_n = g->strides[nd - 1];
    // dense inside a segment?  (stride of each spatial dimension = product of the extents below it)
    bool dense = true;
    int64_t expect = 1;
    for (int i = 0; i < ns; ++i)
    {
        if (g->local_shape[i] > 1 && g->strides[i] != expect)
            dense = false;
        expect *= g->local_shape[i];
    }
    if (dense)
    {
        set_dense_map(&t.map);
        t.row = sp;
        t.aligned = aligned16(p) && t.map.stride_c % full_vec<T>() == 0
                    && t.map.stride_n % full_vec<T>() == 0;
    }
    else
    {
        if (sp >= (1ull << 31))
            return H2X_ERR_TOO_LARGE;
        t.strided = true;
        t.row = static_cast<size_t>(g->local_shape[0]);
        t.map.w = make_fastdiv(static_cast<uint32_t>(g->local_shape[0]));
        t.map.h = make_fastdiv(ns > 1 ? static_cast<uint32_t>(g->local_shape[1]) : 1u);
        if ((ns > 1 && g->strides[1] > 0xffffffffll) || (ns > 2 && g->strides[2] > 0xffffffffll))
            return H2X_ERR_TOO_LARGE; // strides inside a segment are kept as 32-bit integers
        t.map.sy = ns > 1 ? static_cast<uint32_t>(g->strides[1]) : 0;
        t.map.sz = ns > 2 ? static_cast<uint32_t>(g->strides[2]) : 0;
        t.map.spr = make_fastdiv(1);
        t.map.width = 0;
        t.aligned = false;
    }
    *out = t;
    return H2X_SUCCESS;
}

// Vector width all tensors of a launch allow, and whether the strided kernels are needed.
// Dense tensors whose segments are no multiple of the vector long, or start off a
// 16-byte boundary, are handed to the strided kernels too, as tensors with one row
// per segment: vectors aligned to one element, the last one of a segment overlapping
// the one before it (N 16, C 64, 57 x 57: forward 23 -> 15 us against element by element).
constexpr size_t kMinUnalignedSegment = 256;

template <typename T>
int common_vector(std::initializer_list<const HostTensor*> ts, bool* strided)
{
    const int full = full_vec<T>();
    *strided = false;
    for (const HostTensor* t : ts)
        *strided = *strided || t->strided;
    if (!*strided)
    {
        bool aligned_vectors = true, unaligned_vectors = true;
        for (const HostTensor* t : ts)
        {
            if (t->row % full != 0 || !t->aligned)
                aligned_vectors = false;
            if (t->row < kMinUnalignedSegment || t->row >= (1ull << 31))
                unaligned_vectors = false;
        }
        if (aligned_vectors)
            return full;
        if (!unaligned_vectors)
            return 1;
        *strided = true;
        return full;
    }
    // a row of a strided tensor must hold a vector
    for (const HostTensor* t : ts)
        if (t->strided && t->row < static_cast<size_t>(full))
            return 1;
    return full;
}

// Sets the tensors of a strided launch with vectors up for padded rows (see
// TensorMap) and returns the padded length of a segment.  The rows are those of
// the tensors with halos or folded samples; a launch of dense tensors only has
// one row per segment.  Dense tensors in a launch with rows are addressed row by
// row like the others.
template <typename T>
size_t pad_rows(std::initializer_list<HostTensor*> ts, size_t spatial)
{
    const uint32_t vec = full_vec<T>();
    size_t width = spatial;
    uint32_t rows_per_plane = 1;
    for (const HostTensor* t : ts)
        if (t->strided)
        {
            width = t->row;
            rows_per_plane = t->map.h.divisor;
        }
    const size_t spr = (width + vec - 1) / vec;
    for (HostTensor* t : ts)
    {
        if (!t->strided)
        {
            t->map.h = make_fastdiv(rows_per_plane);
            t->map.sy = static_cast<uint32_t>(width);
            t->map.sz = static_cast<uint32_t>(width * rows_per_plane); // below 2^31: a segment's elements
        }
        t->map.spr = make_fastdiv(static_cast<uint32_t>(spr));
        t->map.width = static_cast<uint32_t>(width);
    }
    return spatial / width * spr * vec;
}

// Segments of 257 to 1023 elements (19 x 19, 27 x 27, 28 x 28 activations; shorter
// ones go to the short-segment kernels).  A (sample, channel) segment shorter than
// what a workgroup moves leaves lanes idle in the dense kernels.  The samples of a
// channel are then folded
// into the spatial index: the tensor is addressed as ONE sample whose segments
// are N rows of `spatial` elements, `stride_n` apart, through the index
// splitting of the strided kernels (x = i mod spatial, y = i / spatial), so
// that a workgroup streams through many samples of its channel.  (Measured on
// segments of 49 elements before those had kernels of their own: normalise
// 387 us -> 75 us, backprop2 520 us -> 110 us at N 256, C 2048.)
constexpr size_t kFoldBelow = 1024;

bool fold_samples(int* num_samples, size_t* spatial, std::initializer_list<HostTensor*> ts)
{
    if (*num_samples <= 1 || *spatial >= kFoldBelow)
        return false;
    for (const HostTensor* t : ts)
        if (t->strided || t->map.stride_n > 0xffffffffll)
            return false; // rows are already split, or lie further apart than a 32-bit stride
    for (HostTensor* t : ts)
    {
        t->strided = true;
        t->row = *spatial;
        t->map.w = make_fastdiv(static_cast<uint32_t>(*spatial));
        t->map.h = make_fastdiv(static_cast<uint32_t>(*num_samples));
        t->map.sy = static_cast<uint32_t>(t->map.stride_n);
        t->map.sz = 0;
        t->aligned = false;
    }
    *spatial *= static_cast<size_t>(*num_samples); // < 1024 * 2^31: the callers' grid checks apply
    *num_samples = 1;
    return true;
}

// Segments of at most this many elements go to the short-segment kernels: up
// to here a segment's share of the cache lines at its two ends is 11 % or more.
constexpr size_t kShortSegment = 256;
// Workgroups an elementwise short-segment pass aims at.  The input gradient
// (three tensors a sample) does better with half of what normalise takes: N 64,
// C 1024, 14 x 14 backward 55 -> 48 us, N 256, C 2048, 7 x 7 91 -> 86 us with
// 4096 (2048: 48 / 88 us); forward is the same from 2048 to 32768.
constexpr int kShortElementwiseBlocks = 8192;
constexpr int kShortGradientBlocks = 4096;

// Elements from the first to the last interior element of a segment.
size_t short_span(const HostTensor& t, size_t spatial)
{
    if (!t.strided)
        return spatial;
    const size_t w = t.map.w.divisor, h = t.map.h.divisor;
    const size_t d = spatial / (w * h);
    return (w - 1) + (h - 1) * static_cast<size_t>(t.map.sy) + (d - 1) * static_cast<size_t>(t.map.sz)
           + 1;
}

// A tensor as a short-segment launch addresses it.  When the launch goes row by
// row (some tensor has halos inside its segments), a dense tensor's rows follow
// one another: strides row and row * h.
ShortTensor short_tensor(const HostTensor& t, const ShortGeometry& g)
{
    ShortTensor r;
    r.stride_n = t.map.stride_n;
    r.stride_c = t.map.stride_c;
    r.h = g.rows_per_plane;
    r.sy = t.strided ? t.map.sy : g.row;
    r.sz = t.strided ? t.map.sz : static_cast<int64_t>(g.row) * g.rows_per_plane;
    return r;
}

// Whether a launch over these tensors takes the short-segment kernels, and the
// window of channels a workgroup serves then.
template <typename T>
bool short_segments(int num_samples, int num_channels, size_t spatial,
                    std::initializer_list<const HostTensor*> ts, ShortGeometry* g)
{
    if (spatial == 0 || spatial > kShortSegment || num_samples < 1 || num_channels < 1)
        return false;
    for (const HostTensor* t : ts)
        if (t->strided && short_span(*t, spatial) > 0x7fffffffull)
            return false; // offsets within a segment are kept as 32-bit integers
    const int vec = full_vec<T>();
    g->num_samples = num_samples;
    g->num_channels = num_channels;
    g->spatial = static_cast<int>(spatial);
    // dense tensors only: the segment is one row; else every tensor goes row by row
    g->row = g->spatial;
    g->rows_per_plane = 1;
    for (const HostTensor* t : ts)
        if (t->strided)
        {
            g->row = static_cast<int>(t->map.w.divisor);
            g->rows_per_plane = static_cast<int>(t->map.h.divisor);
        }
    g->slots_per_row = (g->row + vec - 1) / vec;
    g->slots = g->spatial / g->row * g->slots_per_row;
    if (g->slots > kBlockSize)
        return false;
    g->rows = 1;
    g->channels_per_group = kBlockSize / g->slots;
    g->samples_per_group = num_samples;
    return true;
}

int short_windows(const ShortGeometry& g)
{
    return (g.num_channels + g.channels_per_group - 1) / g.channels_per_group;
}

// How a short-segment reduction is spread over the GPU.  The lanes of a
// workgroup may split into `rows` that take every rows-th sample of a narrower
// window (never narrower than kShortMinRowBytes per sample, so that a row still
// reads whole cache lines), and the samples may be cut into ranges whose partial
// sums a later kernel adds (at most kShortMaxGroups: that kernel adds them one
// after the other).  A tensor small enough for every lane to get by with two
// batches of loads takes rows only and a single range: no partial sums, no
// finishing work.  Otherwise ranges first, up to kShortWantGroups workgroups,
// and rows only if that leaves fewer than kShortMinGroups.
constexpr int kShortWantGroups = 2048;
constexpr int kShortMinGroups = 512;
constexpr int kShortMaxGroups = 8;
constexpr size_t kShortMinRowBytes = 256;

bool short_split_rows(ShortGeometry* g, size_t elem_bytes)
{
    const int narrower = kBlockSize / (g->rows * 2) / g->slots;
    if (static_cast<size_t>(narrower) * g->spatial * elem_bytes < kShortMinRowBytes)
        return false;
    g->rows *= 2;
    g->channels_per_group = narrower;
    return true;
}

int short_reduction_groups(ShortGeometry* g, int gmax, int unroll, size_t elem_bytes)
{
    const ShortGeometry whole = *g;
    while (g->num_samples / g->rows > unroll && short_split_rows(g, elem_bytes))
    {
    }
    if ((g->num_samples + g->rows * unroll - 1) / (g->rows * unroll) <= 2)
    {
        g->samples_per_group = g->num_samples;
        return 1;
    }
    *g = whole;
    const int want = (kShortWantGroups + short_windows(*g) - 1) / short_windows(*g);
    const int groups = std::max(1, std::min({g->num_samples / unroll, gmax, kShortMaxGroups, want}));
    const int per = (g->num_samples + groups - 1) / groups;
    while (static_cast<long long>(short_windows(*g)) * groups < kShortMinGroups
           && per >= 2 * unroll * g->rows && short_split_rows(g, elem_bytes))
    {
    }
    g->samples_per_group = per;
    return (g->num_samples + per - 1) / per;
}

// Ranges of samples of a short-segment elementwise pass: whole batches of
// `unroll` samples (what a lane keeps in flight) where there are that many.  A
// pass that finishes a reduction first (`prologue_bytes` of partial sums per
// channel) takes ranges long enough to move at least as many bytes of tensors
// (`sample_bytes` per channel and sample).
int short_elementwise_groups(ShortGeometry* g, int unroll, int budget, size_t prologue_bytes = 0,
                             size_t sample_bytes = 1)
{
    const long long units = static_cast<long long>(g->num_samples) * short_windows(*g);
    long long per = std::max<long long>(unroll, units / budget);
    per = std::max<long long>(per, (prologue_bytes + sample_bytes - 1) / sample_bytes);
    per = (per + unroll - 1) / unroll * unroll;
    per = std::max<long long>(per, (g->num_samples + 65534) / 65535); // grid.y
    g->samples_per_group = static_cast<int>(std::min<long long>(per, g->num_samples));
    return (g->num_samples + g->samples_per_group - 1) / g->samples_per_group;
}

// Launches kernel<T, V, TAIL> of the short-segment family (`sg`: the geometry).
#define H2X_DISPATCH_SHORT(KERNEL, GRID, ...)                                                      \
    do                                                                                             \
    {                                                                                              \
        if (sg.row % full_vec<T>() == 0)                                                           \
            KERNEL<T, full_vec<T>(), kTailNone><<<GRID, kBlockSize, 0, stream>>>(__VA_ARGS__);     \
        else if (sg.row > full_vec<T>())                                                           \
            KERNEL<T, full_vec<T>(), kTailOverlap><<<GRID, kBlockSize, 0, stream>>>(__VA_ARGS__);  \
        else                                                                                       \
            KERNEL<T, full_vec<T>(), kTailScalar><<<GRID, kBlockSize, 0, stream>>>(__VA_ARGS__);   \
    } while (0)

#define H2X_DISPATCH_SHORT_FUSED(KERNEL, FUSED, GRID, ...)                                         \
    do                                                                                             \
    {                                                                                              \
        if (sg.row % full_vec<T>() == 0)                                                           \
            KERNEL<T, full_vec<T>(), kTailNone, FUSED>                                             \
                <<<GRID, kBlockSize, 0, stream>>>(__VA_ARGS__);                                    \
        else if (sg.row > full_vec<T>())                                                           \
            KERNEL<T, full_vec<T>(), kTailOverlap, FUSED>                                          \
                <<<GRID, kBlockSize, 0, stream>>>(__VA_ARGS__);                                    \
        else                                                                                       \
            KERNEL<T, full_vec<T>(), kTailScalar, FUSED>                                           \
                <<<GRID, kBlockSize, 0, stream>>>(__VA_ARGS__);                                    \
    } while (0)

// Launches kernel<T, V, STRIDED> for the width and layout chosen at run time.
#define H2X_DISPATCH(KERNEL, GRID, ...)                                                            \
    do                                                                                             \
    {                                                                                              \
        if (strided)                                                                               \
        {                                                                                          \
            if (vw > 1)                                                                            \
                KERNEL<T, full_vec<T>(), true><<<GRID, kBlockSize, 0, stream>>>(__VA_ARGS__);      \
            else                                                                                   \
                KERNEL<T, 1, true><<<GRID, kBlockSize, 0, stream>>>(__VA_ARGS__);                  \
        }                                                                                          \
        else                                                                                       \
        {                                                                                          \
            if (vw > 1)                                                                            \
                KERNEL<T, full_vec<T>(), false><<<GRID, kBlockSize, 0, stream>>>(__VA_ARGS__);     \
            else                                                                                   \
                KERNEL<T, 1, false><<<GRID, kBlockSize, 0, stream>>>(__VA_ARGS__);                 \
        }                                                                                          \
    } while (0)

// Launches an elementwise kernel<T, V, LAYOUT, FUSED>.
#define H2X_DISPATCH_ELEMENTWISE(KERNEL, FUSED, GRID, ...)                                         \
    do                                                                                             \
    {                                                                                              \
        if (vw > 1 && strided)                                                                     \
            KERNEL<T, full_vec<T>(), kLayoutRows, FUSED>                                           \
                <<<GRID, kBlockSize, 0, stream>>>(__VA_ARGS__);                                    \
        else if (vw > 1)                                                                           \
            KERNEL<T, full_vec<T>(), kLayoutDense, FUSED>                                          \
                <<<GRID, kBlockSize, 0, stream>>>(__VA_ARGS__);                                    \
        else if (strided)                                                                          \
            KERNEL<T, 1, kLayoutRows, FUSED><<<GRID, kBlockSize, 0, stream>>>(__VA_ARGS__);        \
        else                                                                                       \
            KERNEL<T, 1, kLayoutDense, FUSED><<<GRID, kBlockSize, 0, stream>>>(__VA_ARGS__);       \
    } while (0)

// ---- what a launch looks like to the log ----------------------------------------

LaunchRecord short_record(int kernel, const ShortGeometry& sg, dim3 grid, int vec,
                          std::initializer_list<const HostTensor*> ts, bool last_is_output)
{
    LaunchRecord r;
    r.kernel = kernel;
    r.family = kFamilyShort;
    r.vec = vec;
    r.tail = sg.row % vec == 0 ? kTailNone : sg.row > vec ? kTailOverlap : kTailScalar;
    r.grid_x = grid.x;
    r.grid_y = grid.y;
    r.num_samples = sg.num_samples;
    r.num_channels = sg.num_channels;
    r.spatial = static_cast<size_t>(sg.spatial);
    r.geometry = sg;
    r.last_is_output = last_is_output;
    for (const HostTensor* t : ts)
        r.tensor[r.num_tensors++] = short_tensor(*t, sg);
    return r;
}

LaunchRecord long_record(int kernel, bool strided, int vw, dim3 grid, int num_samples,
                         int num_channels, size_t spatial, const Chunking& ch,
                         std::initializer_list<const HostTensor*> ts, bool last_is_output)
{
    LaunchRecord r;
    r.kernel = kernel;
    r.family = strided ? kFamilyStrided : kFamilyDense;
    r.vec = vw;
    r.grid_x = grid.x;
    r.grid_y = grid.y;
    r.num_samples = num_samples;
    r.num_channels = num_channels;
    r.spatial = spatial;
    r.chunk = ch.chunk;
    r.chunks_per_seg = ch.chunks_per_seg;
    r.last_is_output = last_is_output;
    for (const HostTensor* t : ts)
        r.map[r.num_tensors++] = t->map;
    return r;
}

LaunchRecord small_record(int kernel, unsigned int grid_x, int num_channels, int num_sums = 0)
{
    LaunchRecord r;
    r.kernel = kernel;
    r.grid_x = grid_x;
    r.num_channels = num_channels;
    r.num_sums = num_sums;
    return r;
}

template <typename T>
int zero_outputs(std::initializer_list<void*> outs, int num_channels, hipStream_t stream)
{
    const int blocks = (num_channels + kBlockSize - 1) / kBlockSize;
    for (void* p : outs)
        if (!logged(small_record(kKernelFill, blocks, num_channels)))
            fill_kernel<T><<<blocks, kBlockSize, 0, stream>>>(static_cast<T*>(p), num_channels, T(0));
    return issued();
}

// `fused_out` non-null: the caller finishes the reduction itself (a fused
// consumer kernel): every workgroup stores partials, no finishing launch.
template <typename T>
int sums_impl(int num_samples, int num_channels, size_t spatial, const HostTensor& tx_in,
              const void* x, void* sums, void* sqsums, void* workspace, hipStream_t stream,
              FusedStats<T>* fused_out = nullptr)
{
    if (num_channels == 0)
        return H2X_SUCCESS;
    if (num_samples == 0 || spatial == 0)
        return zero_outputs<T>({sums, sqsums}, num_channels, stream);
    if (fused_out)
        fused_out->sequential = false;
    ShortGeometry sg;
    if (short_segments<T>(num_samples, num_channels, spatial, {&tx_in}, &sg))
    {
        const int gmax = max_groups_per_channel(num_channels);
        const int groups = short_reduction_groups(&sg, gmax, kUnroll, sizeof(T));
        double* partials = static_cast<double*>(workspace);
        const dim3 grid(short_windows(sg), groups);
        LaunchRecord rec = short_record(kKernelSums, sg, grid, full_vec<T>(), {&tx_in}, false);
        rec.num_sums = 2;
        rec.groups_max = gmax;
        rec.partials = groups > 1 || fused_out != nullptr;
        if (!logged(rec))
            H2X_DISPATCH_SHORT(bn_sums_short_kernel, grid, static_cast<const T*>(x),
                               static_cast<T*>(sums), static_cast<T*>(sqsums), partials,
                               short_tensor(tx_in, sg), sg, fused_out != nullptr);
        if (fused_out)
        {
            fused_out->groups = groups;
            fused_out->sequential = true;
            return issued();
        }
        const unsigned int blocks = (num_channels + kBlockSize - 1) / kBlockSize;
        if (groups > 1 && !logged(small_record(kKernelFinish, blocks, num_channels, 2)))
            bn_finish_short_kernel<T, 2><<<blocks, kBlockSize, 0, stream>>>(
                partials, groups, num_channels, static_cast<T*>(sums), static_cast<T*>(sqsums),
                nullptr, nullptr);
        return issued();
    }
    HostTensor tx = tx_in;
    const bool folded = fold_samples(&num_samples, &spatial, {&tx});
    if (spatial >= (1ull << 31) && tx.strided)
        return H2X_ERR_TOO_LARGE;
    bool strided;
    const int vw = common_vector<T>({&tx}, &strided);
    if (strided && vw > 1)
        spatial = pad_rows<T>({&tx}, spatial);
    if (spatial >= (1ull << 31) && strided)
        return H2X_ERR_TOO_LARGE;
    const int gmax = max_groups_per_channel(num_channels);
    const int budget = reduction_groups_per_channel(num_channels, strided);
    const size_t tile = static_cast<size_t>(kBlockSize) * vw * kUnroll;
    const Chunking ch = make_chunking(spatial, num_samples, budget, tile, tile);
    const size_t units = static_cast<size_t>(ch.chunks_per_seg) * num_samples;
    if (units > 0xffffffffull || num_channels > 65535)
        return H2X_ERR_TOO_LARGE;
    const size_t groups = std::min<size_t>(units, budget);
    double* partials = static_cast<double*>(workspace);
    const dim3 grid(static_cast<unsigned int>(groups), num_channels);
    LaunchRecord rec = long_record(kKernelSums, strided, vw, grid, num_samples, num_channels,
                                   spatial, ch, {&tx}, false);
    rec.folded = folded;
    rec.num_units = static_cast<unsigned int>(units);
    rec.num_sums = 2;
    rec.groups_max = gmax;
    rec.partials = groups > 1 || fused_out != nullptr;
    if (!logged(rec))
        H2X_DISPATCH(bn_sums_kernel, grid, static_cast<const T*>(x), static_cast<T*>(sums),
                     static_cast<T*>(sqsums), partials, tx.map, spatial, ch.chunk,
                     ch.chunks_per_seg, static_cast<unsigned int>(units), gmax,
                     fused_out != nullptr);
    if (fused_out != nullptr)
    {
        fused_out->groups = static_cast<int>(groups);
        return issued();
    }
    if (groups > 1 && !logged(small_record(kKernelFinish, num_channels, num_channels, 2)))
        bn_finish_kernel<T, 2><<<num_channels, kBlockSize, 0, stream>>>(
            partials, static_cast<int>(groups), gmax, static_cast<T*>(sums),
            static_cast<T*>(sqsums), nullptr, nullptr);
    return issued();
}

template <typename T>
int statistics_impl(int num_channels, size_t num_per_sum, double decay, void* mean, void* var,
                    void* running_mean, void* running_var, hipStream_t stream)
{
    if (num_channels == 0)
        return H2X_SUCCESS;
    const int blocks = std::min((num_channels + kBlockSize - 1) / kBlockSize, 1024);
    if (!logged(small_record(kKernelStatistics, blocks, num_channels)))
        bn_statistics_kernel<T><<<blocks, kBlockSize, 0, stream>>>(
            num_channels, num_per_sum, static_cast<T>(decay), static_cast<T*>(mean),
            static_cast<T*>(var), static_cast<T*>(running_mean), static_cast<T*>(running_var));
    return issued();
}

// Chunking of an elementwise pass over N*C segments: at least one full vector
// per thread, about kElementwiseBlocks workgroups.
Chunking elementwise_chunking(size_t spatial, size_t segments, int vw, int unroll,
                              int budget = kElementwiseBlocks)
{
    const size_t tile = static_cast<size_t>(kBlockSize) * vw * unroll;
    const size_t one_pass = static_cast<size_t>(kBlockSize) * vw;
    Chunking c = make_chunking(spatial, segments, budget, one_pass,
                               one_pass * 2 > tile ? one_pass : one_pass * 2);
    // A chunk of more than a tile is cut down to whole tiles: the passes beyond the
    // last whole tile run with one load in flight per lane instead of `unroll`
    // (5 passes as 4 + 1 took a quarter longer than 4 on the haloed C3 shard).
    if (c.chunk > tile && c.chunk % tile != 0)
    {
        c.chunk = c.chunk / tile * tile;
        c.chunks_per_seg = static_cast<int>((spatial + c.chunk - 1) / c.chunk);
    }
    return c;
}

template <typename T>
int apply_impl(int num_samples, int num_channels, size_t spatial, const HostTensor& tx_in,
               const HostTensor& ty_in, const void* x, const void* mean, const void* var,
               const void* scale, const void* bias, void* y, double epsilon, hipStream_t stream,
               const FusedStats<T>* fused = nullptr)
{
    if (static_cast<size_t>(num_samples) * num_channels == 0 || spatial == 0)
        return H2X_SUCCESS;
    ShortGeometry sg;
    const bool is_short = short_segments<T>(num_samples, num_channels, spatial, {&tx_in, &ty_in}, &sg);
    if (fused && fused->sequential != is_short)
        return H2X_ERR_UNSUPPORTED; // the partials are laid out for the other family of kernels
    if (is_short)
    {
        const dim3 grid(short_windows(sg),
                        short_elementwise_groups(&sg, kUnroll, kShortElementwiseBlocks,
                                                 fused ? fused->groups * 2 * sizeof(double) : 0,
                                                 spatial * sizeof(T) * 2));
        LaunchRecord rec =
            short_record(kKernelApply, sg, grid, full_vec<T>(), {&tx_in, &ty_in}, true);
        rec.fused = fused != nullptr;
        if (logged(rec))
            return H2X_SUCCESS;
        if (fused)
            H2X_DISPATCH_SHORT_FUSED(bn_apply_short_kernel, true, grid, static_cast<const T*>(x),
                                     nullptr, nullptr, static_cast<const T*>(scale),
                                     static_cast<const T*>(bias), static_cast<T*>(y),
                                     static_cast<T>(epsilon), short_tensor(tx_in, sg),
                                     short_tensor(ty_in, sg), sg, *fused);
        else
            H2X_DISPATCH_SHORT_FUSED(bn_apply_short_kernel, false, grid, static_cast<const T*>(x),
                                     static_cast<const T*>(mean), static_cast<const T*>(var),
                                     static_cast<const T*>(scale), static_cast<const T*>(bias),
                                     static_cast<T*>(y), static_cast<T>(epsilon),
                                     short_tensor(tx_in, sg), short_tensor(ty_in, sg), sg, FusedStats<T>());
        return issued();
    }
    HostTensor tx = tx_in, ty = ty_in;
    const bool folded = fold_samples(&num_samples, &spatial, {&tx, &ty});
    if (spatial >= (1ull << 31) && (tx.strided || ty.strided))
        return H2X_ERR_TOO_LARGE;
    const size_t segments = static_cast<size_t>(num_samples) * num_channels;
    bool strided;
    const int vw = common_vector<T>({&tx, &ty}, &strided);
    if (strided && vw > 1)
        spatial = pad_rows<T>({&tx, &ty}, spatial);
    if (spatial >= (1ull << 31) && strided)
        return H2X_ERR_TOO_LARGE;
    const bool beyond_cache = segments * spatial * sizeof(T) > kBeyondCacheBytes;
    const Chunking ch = elementwise_chunking(spatial, segments, vw, kUnroll,
                                             strided || beyond_cache ? kUnboundedBlocks : kElementwiseBlocks);
    const size_t workgroups = segments * ch.chunks_per_seg;
    if (!grid_ok(workgroups))
        return H2X_ERR_TOO_LARGE;
    const unsigned int grid = static_cast<unsigned int>(workgroups);
    LaunchRecord rec = long_record(kKernelApply, strided, vw, dim3(grid), num_samples, num_channels,
                                   spatial, ch, {&tx, &ty}, true);
    rec.folded = folded;
    rec.fused = fused != nullptr;
    if (logged(rec))
        return H2X_SUCCESS;
    if (fused)
        H2X_DISPATCH_ELEMENTWISE(bn_apply_kernel, true, grid, static_cast<const T*>(x), nullptr,
                                 nullptr, static_cast<const T*>(scale), static_cast<const T*>(bias),
                                 static_cast<T*>(y), static_cast<T>(epsilon), num_channels, spatial,
                                 tx.map, ty.map, ch.chunk, ch.chunks_per_seg, *fused);
    else
        H2X_DISPATCH_ELEMENTWISE(bn_apply_kernel, false, grid, static_cast<const T*>(x),
                                 static_cast<const T*>(mean), static_cast<const T*>(var),
                                 static_cast<const T*>(scale), static_cast<const T*>(bias),
                                 static_cast<T*>(y), static_cast<T>(epsilon), num_channels, spatial,
                                 tx.map, ty.map, ch.chunk, ch.chunks_per_seg);
    return issued();
}

template <typename T>
int backprop1_impl(int num_samples, int num_channels, size_t spatial, const HostTensor& tx_in,
                   const HostTensor& td_in, const void* x, const void* dy, const void* mean,
                   const void* var, const void* scale, void* dscale, void* dbias, void* dmean,
                   void* dvar, double epsilon, void* workspace, hipStream_t stream,
                   FusedStats<T>* fused_out = nullptr)
{
    if (num_channels == 0)
        return H2X_SUCCESS;
    if (num_samples == 0 || spatial == 0)
        return zero_outputs<T>({dscale, dbias, dmean, dvar}, num_channels, stream);
    if (fused_out)
        fused_out->sequential = false;
    ShortGeometry sg;
    if (short_segments<T>(num_samples, num_channels, spatial, {&tx_in, &td_in}, &sg))
    {
        const int gmax = max_groups_per_channel(num_channels);
        const int groups = short_reduction_groups(&sg, gmax, kUnroll / 2, sizeof(T));
        double* partials = static_cast<double*>(workspace);
        const dim3 grid(short_windows(sg), groups);
        LaunchRecord rec =
            short_record(kKernelBackprop1, sg, grid, full_vec<T>(), {&tx_in, &td_in}, false);
        rec.num_sums = 4;
        rec.groups_max = gmax;
        rec.partials = groups > 1 || fused_out != nullptr;
        if (!logged(rec))
            H2X_DISPATCH_SHORT(bn_backprop1_short_kernel, grid, static_cast<const T*>(x),
                               static_cast<const T*>(dy), static_cast<const T*>(mean),
                               static_cast<const T*>(var), static_cast<const T*>(scale),
                               static_cast<T*>(dscale), static_cast<T*>(dbias),
                               static_cast<T*>(dmean), static_cast<T*>(dvar),
                               static_cast<T>(epsilon), partials, short_tensor(tx_in, sg),
                               short_tensor(td_in, sg), sg, fused_out != nullptr);
        if (fused_out)
        {
            fused_out->groups = groups;
            fused_out->sequential = true;
            return issued();
        }
        const unsigned int blocks = (num_channels + kBlockSize - 1) / kBlockSize;
        if (groups > 1 && !logged(small_record(kKernelFinish, blocks, num_channels, 4)))
            bn_finish_short_kernel<T, 4><<<blocks, kBlockSize, 0, stream>>>(
                partials, groups, num_channels, static_cast<T*>(dscale), static_cast<T*>(dbias),
                static_cast<T*>(dmean), static_cast<T*>(dvar));
        return issued();
    }
    HostTensor tx = tx_in, td = td_in;
    const bool folded = fold_samples(&num_samples, &spatial, {&tx, &td});
    if (spatial >= (1ull << 31) && (tx.strided || td.strided))
        return H2X_ERR_TOO_LARGE;
    bool strided;
    const int vw = common_vector<T>({&tx, &td}, &strided);
    if (strided && vw > 1)
        spatial = pad_rows<T>({&tx, &td}, spatial);
    if (spatial >= (1ull << 31) && strided)
        return H2X_ERR_TOO_LARGE;
    const int gmax = max_groups_per_channel(num_channels);
    const int budget = reduction_groups_per_channel(num_channels, strided);
    const size_t tile = static_cast<size_t>(kBlockSize) * vw * (kUnroll / 2);
    const Chunking ch = make_chunking(spatial, num_samples, budget, tile, tile);
    const size_t units = static_cast<size_t>(ch.chunks_per_seg) * num_samples;
    if (units > 0xffffffffull || num_channels > 65535)
        return H2X_ERR_TOO_LARGE;
    const size_t groups = std::min<size_t>(units, budget);
    double* partials = static_cast<double*>(workspace);
    const dim3 grid(static_cast<unsigned int>(groups), num_channels);
    LaunchRecord rec = long_record(kKernelBackprop1, strided, vw, grid, num_samples, num_channels,
                                   spatial, ch, {&tx, &td}, false);
    rec.folded = folded;
    rec.num_units = static_cast<unsigned int>(units);
    rec.num_sums = 4;
    rec.groups_max = gmax;
    rec.partials = groups > 1 || fused_out != nullptr;
    if (!logged(rec))
        H2X_DISPATCH(bn_backprop1_kernel, grid, static_cast<const T*>(x),
                     static_cast<const T*>(dy), static_cast<const T*>(mean),
                     static_cast<const T*>(var), static_cast<const T*>(scale),
                     static_cast<T*>(dscale), static_cast<T*>(dbias), static_cast<T*>(dmean),
                     static_cast<T*>(dvar), static_cast<T>(epsilon), partials, spatial, tx.map,
                     td.map, ch.chunk, ch.chunks_per_seg, static_cast<unsigned int>(units), gmax,
                     fused_out != nullptr);
    if (fused_out != nullptr)
    {
        fused_out->groups = static_cast<int>(groups);
        return issued();
    }
    if (groups > 1 && !logged(small_record(kKernelFinish, num_channels, num_channels, 4)))
        bn_finish_kernel<T, 4><<<num_channels, kBlockSize, 0, stream>>>(
            partials, static_cast<int>(groups), gmax, static_cast<T*>(dscale),
            static_cast<T*>(dbias), static_cast<T*>(dmean), static_cast<T*>(dvar));
    return issued();
}

template <typename T>
int backprop2_impl(int num_samples, int num_channels, size_t spatial, size_t num_per_sum,
                   const HostTensor& tx_in, const HostTensor& td_in, const HostTensor& to_in,
                   const void* x, const void* dy, const void* mean, const void* var,
                   const void* scale, const void* dmean, const void* dvar, void* dx,
                   double epsilon, hipStream_t stream, const FusedStats<T>* fused = nullptr)
{
    if (static_cast<size_t>(num_samples) * num_channels == 0 || spatial == 0)
        return H2X_SUCCESS;
    ShortGeometry sg;
    const bool is_short =
        short_segments<T>(num_samples, num_channels, spatial, {&tx_in, &td_in, &to_in}, &sg);
    if (fused && fused->sequential != is_short)
        return H2X_ERR_UNSUPPORTED; // the partials are laid out for the other family of kernels
    // whether x and dx share memory (the reference allows dx to be x itself)
    const auto span = [&](const HostTensor& t) {
        return (static_cast<size_t>(num_samples - 1) * t.map.stride_n
                + static_cast<size_t>(num_channels - 1) * t.map.stride_c + short_span(t, spatial))
               * sizeof(T);
    };
    const char* xb = static_cast<const char*>(x);
    const char* ob = static_cast<const char*>(dx);
    const bool disjoint = xb + span(tx_in) <= ob || ob + span(to_in) <= xb;
    if (is_short)
    {
        const dim3 grid(short_windows(sg),
                        short_elementwise_groups(&sg, kUnroll / 2, kShortGradientBlocks,
                                                 fused ? fused->groups * 4 * sizeof(double) : 0,
                                                 spatial * sizeof(T) * 3));
        LaunchRecord rec = short_record(kKernelBackprop2, sg, grid, full_vec<T>(),
                                        {&tx_in, &td_in, &to_in}, true);
        rec.fused = fused != nullptr;
        rec.rewrite = disjoint;
        if (logged(rec))
            return H2X_SUCCESS;
        if (fused)
            H2X_DISPATCH_SHORT_FUSED(bn_backprop2_short_kernel, true, grid,
                                     static_cast<const T*>(x), static_cast<const T*>(dy),
                                     static_cast<const T*>(mean), static_cast<const T*>(var),
                                     static_cast<const T*>(scale), nullptr, nullptr,
                                     static_cast<T*>(dx), static_cast<T>(epsilon), num_per_sum,
                                     short_tensor(tx_in, sg), short_tensor(td_in, sg), short_tensor(to_in, sg),
                                     sg, disjoint, *fused);
        else
            H2X_DISPATCH_SHORT_FUSED(bn_backprop2_short_kernel, false, grid,
                                     static_cast<const T*>(x), static_cast<const T*>(dy),
                                     static_cast<const T*>(mean), static_cast<const T*>(var),
                                     static_cast<const T*>(scale), static_cast<const T*>(dmean),
                                     static_cast<const T*>(dvar), static_cast<T*>(dx),
                                     static_cast<T>(epsilon), num_per_sum, short_tensor(tx_in, sg),
                                     short_tensor(td_in, sg), short_tensor(to_in, sg), sg, disjoint,
                                     FusedStats<T>());
        return issued();
    }
    HostTensor tx = tx_in, td = td_in, to = to_in;
    const bool folded = fold_samples(&num_samples, &spatial, {&tx, &td, &to});
    if (spatial >= (1ull << 31) && (tx.strided || td.strided || to.strided))
        return H2X_ERR_TOO_LARGE;
    const size_t segments = static_cast<size_t>(num_samples) * num_channels;
    bool strided;
    const int vw = common_vector<T>({&tx, &td, &to}, &strided);
    if (strided && vw > 1)
        spatial = pad_rows<T>({&tx, &td, &to}, spatial);
    if (spatial >= (1ull << 31) && strided)
        return H2X_ERR_TOO_LARGE;
    const bool beyond_cache = segments * spatial * sizeof(T) > kBeyondCacheBytes;
    const Chunking ch = elementwise_chunking(spatial, segments, vw, kUnroll / 2,
                                             strided || beyond_cache ? kUnboundedBlocks : kElementwiseBlocks);
    const size_t workgroups = segments * ch.chunks_per_seg;
    if (!grid_ok(workgroups))
        return H2X_ERR_TOO_LARGE;
    const unsigned int grid = static_cast<unsigned int>(workgroups);
    LaunchRecord rec = long_record(kKernelBackprop2, strided, vw, dim3(grid), num_samples,
                                   num_channels, spatial, ch, {&tx, &td, &to}, true);
    rec.folded = folded;
    rec.fused = fused != nullptr;
    rec.rewrite = disjoint;
    if (logged(rec))
        return H2X_SUCCESS;
    if (fused)
        H2X_DISPATCH_ELEMENTWISE(bn_backprop2_kernel, true, grid, static_cast<const T*>(x),
                                 static_cast<const T*>(dy), static_cast<const T*>(mean),
                                 static_cast<const T*>(var), static_cast<const T*>(scale), nullptr,
                                 nullptr, static_cast<T*>(dx), static_cast<T>(epsilon), num_per_sum,
                                 num_channels, spatial, tx.map, td.map, to.map, ch.chunk,
                                 ch.chunks_per_seg, disjoint, *fused);
    else
        H2X_DISPATCH_ELEMENTWISE(bn_backprop2_kernel, false, grid, static_cast<const T*>(x),
                                 static_cast<const T*>(dy), static_cast<const T*>(mean),
                                 static_cast<const T*>(var), static_cast<const T*>(scale),
                                 static_cast<const T*>(dmean), static_cast<const T*>(dvar),
                                 static_cast<T*>(dx), static_cast<T>(epsilon), num_per_sum,
                                 num_channels, spatial, tx.map, td.map, to.map, ch.chunk,
                                 ch.chunks_per_seg, disjoint);
    return issued();
}

// Normalise / input gradient over tensors of one haloed geometry, the halo of
// the output cleared (bn_clearing_kernel).
template <typename T>
int clearing_impl(bool backward, size_t num_per_sum, const h2x_haloed_geometry* g, const void* x,
                  const void* dy, const void* mean, const void* var, const void* scale,
                  const void* bias, const void* dmean, const void* dvar, void* out, double epsilon,
                  hipStream_t stream)
{
    if (!g || g->num_dims < 3 || g->num_dims > 5)
        return H2X_ERR_INVALID_ARGUMENT;
    const int nd = g->num_dims, ns = nd - 2;
    RealBox box;
    size_t real = 1, extent[3] = {1, 1, 1};
    for (int d = 0; d < 3; ++d)
    {
        box.lo[d] = 0;
        box.hi[d] = 1;
    }
    for (int d = 0; d < nd; ++d)
    {
        if (g->local_shape[d] < 0 || g->lower_halo[d] < 0
            || g->lower_halo[d] + g->local_shape[d] > g->real_shape[d])
            return H2X_ERR_INVALID_ARGUMENT;
        if (d >= ns && (g->lower_halo[d] != 0 || g->real_shape[d] != g->local_shape[d]))
            return H2X_ERR_UNSUPPORTED; // no halo on the channel and sample dimensions
    }
    for (int d = 0; d < ns; ++d)
    {
        extent[d] = static_cast<size_t>(g->real_shape[d]);
        real *= extent[d];
        if (real >= (1ull << 31))
            return H2X_ERR_TOO_LARGE;
        box.lo[d] = static_cast<uint32_t>(g->lower_halo[d]);
        box.hi[d] = static_cast<uint32_t>(g->lower_halo[d] + g->local_shape[d]);
    }
    const int num_channels = static_cast<int>(g->local_shape[nd - 2]);
    const size_t segments = static_cast<size_t>(g->local_shape[nd - 1]) * num_channels;
    if (segments == 0 || real == 0)
        return H2X_SUCCESS;
    if (!x || !out || (backward && !dy))
        return H2X_ERR_INVALID_ARGUMENT;
    box.wr = make_fastdiv(static_cast<uint32_t>(extent[0]));
    box.hr = make_fastdiv(static_cast<uint32_t>(extent[1]));
    const bool vectors = real % full_vec<T>() == 0 && aligned16(x) && aligned16(out)
                         && (!backward || aligned16(dy));
    const int vw = vectors ? full_vec<T>() : 1;
    const Chunking ch = elementwise_chunking(real, segments, vw, backward ? kUnroll / 2 : kUnroll);
    const size_t workgroups = segments * ch.chunks_per_seg;
    if (!grid_ok(workgroups))
        return H2X_ERR_TOO_LARGE;
    const unsigned int grid = static_cast<unsigned int>(workgroups);
    {
        LaunchRecord rec;
        rec.kernel = kKernelClearing;
        rec.family = kFamilyDense;
        rec.vec = vw;
        rec.grid_x = grid;
        rec.num_samples = static_cast<int>(g->local_shape[nd - 1]);
        rec.num_channels = num_channels;
        rec.spatial = real;
        rec.real = real;
        rec.chunk = ch.chunk;
        rec.chunks_per_seg = ch.chunks_per_seg;
        rec.num_tensors = backward ? 3 : 2;
        rec.last_is_output = true;
        rec.box = box;
        if (logged(rec))
            return H2X_SUCCESS;
    }
#define H2X_LAUNCH_CLEARING(VEC, BACKWARD)                                                         \
    bn_clearing_kernel<T, VEC, BACKWARD><<<grid, kBlockSize, 0, stream>>>(                         \
        static_cast<const T*>(x), static_cast<const T*>(dy), static_cast<const T*>(mean),          \
        static_cast<const T*>(var), static_cast<const T*>(scale), static_cast<const T*>(bias),     \
        static_cast<const T*>(dmean), static_cast<const T*>(dvar), static_cast<T*>(out),           \
        static_cast<T>(epsilon), num_per_sum, num_channels, real, box, ch.chunk, ch.chunks_per_seg)
    if (backward)
    {
        if (vectors)
            H2X_LAUNCH_CLEARING(full_vec<T>(), true);
        else
            H2X_LAUNCH_CLEARING(1, true);
    }
    else
    {
        if (vectors)
            H2X_LAUNCH_CLEARING(full_vec<T>(), false);
        else
            H2X_LAUNCH_CLEARING(1, false);
    }
#undef H2X_LAUNCH_CLEARING
    return launch_status();
}

bool bad_geometry(int num_samples, int num_channels, size_t spatial, size_t real)
{
    return num_samples < 0 || num_channels < 0 || real < spatial;
}

// ---- typed bodies of the C entry points ----------------------------------------

template <typename T>
int sums_dense(int n, int c, size_t s, size_t sr, const void* x, void* sums, void* sqsums, void* ws,
               hipStream_t st)
{
    return sums_impl<T>(n, c, s, dense_tensor<T>(x, c, s, sr), x, sums, sqsums, ws, st);
}

template <typename T>
int sums_strided(int n, const h2x_tensor_geometry* g, const void* x, void* sums, void* sqsums,
                 void* ws, hipStream_t st)
{
    HostTensor tx;
    int c;
    size_t s;
    const int err = strided_tensor<T>(g, x, n, &tx, &c, &s);
    return err ? err : sums_impl<T>(n, c, s, tx, x, sums, sqsums, ws, st);
}

// Two geometries describe the same elements only if every local extent agrees:
// equal products are not enough (8 x 4 against 4 x 8 would pair other elements).
bool same_local_shape(const h2x_tensor_geometry* a, const h2x_tensor_geometry* b)
{
    if (a->num_dims != b->num_dims)
        return false;
    for (int i = 0; i < a->num_dims; ++i)
        if (a->local_shape[i] != b->local_shape[i])
            return false;
    return true;
}

template <typename T>
int apply_strided(int n, const h2x_tensor_geometry* gx, const h2x_tensor_geometry* gy, const void* x,
                  const void* mean, const void* var, const void* scale, const void* bias, void* y,
                  double eps, hipStream_t st)
{
    HostTensor tx, ty;
    int c, c2;
    size_t s, s2;
    int err = strided_tensor<T>(gx, x, n, &tx, &c, &s);
    if (!err)
        err = strided_tensor<T>(gy, y, n, &ty, &c2, &s2);
    if (!err && (c != c2 || s != s2 || !same_local_shape(gx, gy)))
        err = H2X_ERR_INVALID_ARGUMENT;
    return err ? err : apply_impl<T>(n, c, s, tx, ty, x, mean, var, scale, bias, y, eps, st);
}

template <typename T>
int backprop1_strided(int n, const h2x_tensor_geometry* gx, const h2x_tensor_geometry* gd,
                      const void* x, const void* dy, const void* mean, const void* var,
                      const void* scale, void* dscale, void* dbias, void* dmean, void* dvar,
                      double eps, void* ws, hipStream_t st)
{
    HostTensor tx, td;
    int c, c2;
    size_t s, s2;
    int err = strided_tensor<T>(gx, x, n, &tx, &c, &s);
    if (!err)
        err = strided_tensor<T>(gd, dy, n, &td, &c2, &s2);
    if (!err && (c != c2 || s != s2 || !same_local_shape(gx, gd)))
        err = H2X_ERR_INVALID_ARGUMENT;
    return err ? err
               : backprop1_impl<T>(n, c, s, tx, td, x, dy, mean, var, scale, dscale, dbias, dmean,
                                   dvar, eps, ws, st);
}

template <typename T>
int backprop2_strided(int n, size_t num_per_sum, const h2x_tensor_geometry* gx,
                      const h2x_tensor_geometry* gd, const h2x_tensor_geometry* go, const void* x,
                      const void* dy, const void* mean, const void* var, const void* scale,
                      const void* dmean, const void* dvar, void* dx, double eps, hipStream_t st)
{
    HostTensor tx, td, to;
    int c, c2, c3;
    size_t s, s2, s3;
    int err = strided_tensor<T>(gx, x, n, &tx, &c, &s);
    if (!err)
        err = strided_tensor<T>(gd, dy, n, &td, &c2, &s2);
    if (!err)
        err = strided_tensor<T>(go, dx, n, &to, &c3, &s3);
    if (!err
        && (c != c2 || s != s2 || c != c3 || s != s3 || !same_local_shape(gx, gd)
            || !same_local_shape(gx, go)))
        err = H2X_ERR_INVALID_ARGUMENT;
    return err ? err
               : backprop2_impl<T>(n, c, s, num_per_sum, tx, td, to, x, dy, mean, var, scale, dmean,
                                   dvar, dx, eps, st);
}

// Forward pass of a rank that shares its statistics with no one: sums, then a
// normalising kernel that finishes them itself (2 launches instead of 4).
template <typename T>
int forward_local(int n, int c, size_t s, const HostTensor& tx, const HostTensor& ty, const void* x,
                  const void* scale, const void* bias, size_t num_per_sum, double decay, double eps,
                  void* mean, void* var, void* running_mean, void* running_var, void* y, void* ws,
                  hipStream_t st)
{
    if (c == 0)
        return H2X_SUCCESS;
    if (n == 0 || s == 0 || num_per_sum == 0)
    {
        // nothing to normalise or nothing counted: the staged calls define the result
        int err = sums_impl<T>(n, c, s, tx, x, mean, var, ws, st);
        if (!err)
            err = statistics_impl<T>(c, num_per_sum, decay, mean, var, running_mean, running_var, st);
        return err ? err : apply_impl<T>(n, c, s, tx, ty, x, mean, var, scale, bias, y, eps, st);
    }
    FusedStats<T> f;
    f.sequential = false;
    f.partials = static_cast<const double*>(ws);
    f.groups_per_channel_max = max_groups_per_channel(c);
    f.num_per_sum = num_per_sum;
    f.decay = static_cast<T>(decay);
    f.out[0] = static_cast<T*>(mean);
    f.out[1] = static_cast<T*>(var);
    f.out[2] = static_cast<T*>(running_mean);
    f.out[3] = static_cast<T*>(running_var);
    {
        // both launches are planned before the first is issued: a call that is rejected writes nothing
        LaunchLog plan;
        ScopedLaunchLog scope(&plan);
        FusedStats<T> g = f;
        int err = sums_impl<T>(n, c, s, tx, x, nullptr, nullptr, ws, st, &g);
        if (!err)
            err = apply_impl<T>(n, c, s, tx, ty, x, nullptr, nullptr, scale, bias, y, eps, st, &g);
        if (err == H2X_ERR_UNSUPPORTED)
        {
            // the two tensors take different families of kernels (one of them with halos inside
            // short segments, say): the staged calls
            scope.restore();
            err = sums_impl<T>(n, c, s, tx, x, mean, var, ws, st);
            if (!err)
                err = statistics_impl<T>(c, num_per_sum, decay, mean, var, running_mean, running_var, st);
            return err ? err : apply_impl<T>(n, c, s, tx, ty, x, mean, var, scale, bias, y, eps, st);
        }
        if (err)
            return err;
    }
    const int err = sums_impl<T>(n, c, s, tx, x, nullptr, nullptr, ws, st, &f);
    return err ? err : apply_impl<T>(n, c, s, tx, ty, x, nullptr, nullptr, scale, bias, y, eps, st, &f);
}

// Backward pass likewise: the four sums, then an input-gradient kernel that
// finishes them itself (2 launches instead of 3).
template <typename T>
int backward_local(int n, int c, size_t s, const HostTensor& tx, const HostTensor& td,
                   const HostTensor& to, size_t num_per_sum, const void* x, const void* dy,
                   const void* mean, const void* var, const void* scale, void* dscale, void* dbias,
                   void* dmean, void* dvar, void* dx, double eps, void* ws, hipStream_t st)
{
    if (c == 0)
        return H2X_SUCCESS;
    if (n == 0 || s == 0)
        return backprop1_impl<T>(n, c, s, tx, td, x, dy, mean, var, scale, dscale, dbias, dmean,
                                 dvar, eps, ws, st); // zeroes the four outputs; no dx to write
    FusedStats<T> f;
    f.sequential = false;
    f.partials = static_cast<const double*>(ws);
    f.groups_per_channel_max = max_groups_per_channel(c);
    f.num_per_sum = num_per_sum;
    f.decay = T(0);
    f.out[0] = static_cast<T*>(dscale);
    f.out[1] = static_cast<T*>(dbias);
    f.out[2] = static_cast<T*>(dmean);
    f.out[3] = static_cast<T*>(dvar);
    {
        // both launches are planned before the first is issued: a call that is rejected writes nothing
        LaunchLog plan;
        ScopedLaunchLog scope(&plan);
        FusedStats<T> g = f;
        int err = backprop1_impl<T>(n, c, s, tx, td, x, dy, mean, var, scale, nullptr, nullptr,
                                    nullptr, nullptr, eps, ws, st, &g);
        if (!err)
            err = backprop2_impl<T>(n, c, s, num_per_sum, tx, td, to, x, dy, mean, var, scale,
                                    nullptr, nullptr, dx, eps, st, &g);
        if (err == H2X_ERR_UNSUPPORTED)
        {
            // the tensors take different families of kernels: the staged calls
            scope.restore();
            err = backprop1_impl<T>(n, c, s, tx, td, x, dy, mean, var, scale, dscale, dbias, dmean,
                                    dvar, eps, ws, st);
            return err ? err
                       : backprop2_impl<T>(n, c, s, num_per_sum, tx, td, to, x, dy, mean, var, scale,
                                           dmean, dvar, dx, eps, st);
        }
        if (err)
            return err;
    }
    const int err = backprop1_impl<T>(n, c, s, tx, td, x, dy, mean, var, scale, nullptr, nullptr,
                                      nullptr, nullptr, eps, ws, st, &f);
    return err ? err
               : backprop2_impl<T>(n, c, s, num_per_sum, tx, td, to, x, dy, mean, var, scale,
                                   nullptr, nullptr, dx, eps, st, &f);
}

template <typename T>
int forward_local_strided(int n, const h2x_tensor_geometry* gx, const h2x_tensor_geometry* gy,
                          const void* x, const void* scale, const void* bias, size_t num_per_sum,
                          double decay, double eps, void* mean, void* var, void* running_mean,
                          void* running_var, void* y, void* ws, hipStream_t st)
{
    HostTensor tx, ty;
    int c, c2;
    size_t s, s2;
    int err = strided_tensor<T>(gx, x, n, &tx, &c, &s);
    if (!err)
        err = strided_tensor<T>(gy, y, n, &ty, &c2, &s2);
    if (!err && (c != c2 || s != s2 || !same_local_shape(gx, gy)))
        err = H2X_ERR_INVALID_ARGUMENT;
    return err ? err
               : forward_local<T>(n, c, s, tx, ty, x, scale, bias, num_per_sum, decay, eps, mean, var,
                                  running_mean, running_var, y, ws, st);
}

template <typename T>
int backward_local_strided(int n, size_t num_per_sum, const h2x_tensor_geometry* gx,
                           const h2x_tensor_geometry* gd, const h2x_tensor_geometry* go,
                           const void* x, const void* dy, const void* mean, const void* var,
                           const void* scale, void* dscale, void* dbias, void* dmean, void* dvar,
                           void* dx, double eps, void* ws, hipStream_t st)
{
    HostTensor tx, td, to;
    int c, c2, c3;
    size_t s, s2, s3;
    int err = strided_tensor<T>(gx, x, n, &tx, &c, &s);
    if (!err)
        err = strided_tensor<T>(gd, dy, n, &td, &c2, &s2);
    if (!err)
        err = strided_tensor<T>(go, dx, n, &to, &c3, &s3);
    if (!err
        && (c != c2 || s != s2 || c != c3 || s != s3 || !same_local_shape(gx, gd)
            || !same_local_shape(gx, go)))
        err = H2X_ERR_INVALID_ARGUMENT;
    return err ? err
               : backward_local<T>(n, c, s, tx, td, to, num_per_sum, x, dy, mean, var, scale, dscale,
                                   dbias, dmean, dvar, dx, eps, ws, st);
}

} // namespace

namespace bn
{
LaunchLog* install_launch_log(LaunchLog* log)
{
    LaunchLog* before = t_launch_log;
    t_launch_log = log;
    return before;
}
} // namespace bn
} // namespace h2x

using namespace h2x;

#define H2X_BY_DTYPE(dtype, CALL_F32, CALL_F64)                                                    \
    switch (dtype)                                                                                 \
    {                                                                                              \
    case H2X_F32: return CALL_F32;                                                                 \
    case H2X_F64: return CALL_F64;                                                                 \
    }                                                                                              \
    return H2X_ERR_UNSUPPORTED

extern "C" size_t h2x_bn_workspace_bytes(int num_channels)
{
    if (num_channels <= 0)
        return 256;
    return (partials_bytes(num_channels) + 255) / 256 * 256;
}

extern "C" int h2x_bn_channel_sums_and_sqsums(h2x_dtype dtype, int num_samples, int num_channels,
                                              size_t spatial_size, size_t spatial_real_size,
                                              const void* x, void* sums, void* sqsums,
                                              void* workspace, h2x_stream_t stream)
{
    if (bad_geometry(num_samples, num_channels, spatial_size, spatial_real_size) || !sums || !sqsums
        || !workspace || (!x && num_samples > 0 && spatial_size > 0 && num_channels > 0))
        return H2X_ERR_INVALID_ARGUMENT;
    H2X_BY_DTYPE(dtype,
                 sums_dense<float>(num_samples, num_channels, spatial_size, spatial_real_size, x, sums,
                                   sqsums, workspace, as_stream(stream)),
                 sums_dense<double>(num_samples, num_channels, spatial_size, spatial_real_size, x,
                                    sums, sqsums, workspace, as_stream(stream)));
}

extern "C" size_t h2x_bn_static_max_channels(void)
{
    // largest channel count whose partial sums fit in the scratch array
    int lo = 0, hi = 65535;
    while (lo < hi)
    {
        const int mid = (lo + hi + 1) / 2;
        if (h2x_bn_workspace_bytes(mid) <= kStaticScratchBytes)
            lo = mid;
        else
            hi = mid - 1;
    }
    return static_cast<size_t>(lo);
}

extern "C" int h2x_bn_channel_sums_and_sqsums_static(h2x_dtype dtype, int num_samples,
                                                     int num_channels, size_t spatial_size,
                                                     size_t spatial_real_size, const void* x,
                                                     void* sums, void* sqsums, h2x_stream_t stream)
{
    if (num_channels > 0 && h2x_bn_workspace_bytes(num_channels) > kStaticScratchBytes)
        return H2X_ERR_SCRATCH_LIMIT;
    void* workspace = nullptr;
    const int err = static_scratch(&workspace);
    if (err != 0)
        return err;
    // The partial sums need no clearing: every slot the finishing kernel reads
    // is written by this call's reduction kernel first.
    return h2x_bn_channel_sums_and_sqsums(dtype, num_samples, num_channels, spatial_size,
                                          spatial_real_size, x, sums, sqsums, workspace, stream);
}

extern "C" int h2x_bn_channel_sums_and_sqsums_strided(h2x_dtype dtype, int num_samples,
                                                      const h2x_tensor_geometry* x_geometry,
                                                      const void* x, void* sums, void* sqsums,
                                                      void* workspace, h2x_stream_t stream)
{
    if (num_samples < 0 || !x_geometry || !sums || !sqsums || !workspace)
        return H2X_ERR_INVALID_ARGUMENT;
    H2X_BY_DTYPE(dtype,
                 sums_strided<float>(num_samples, x_geometry, x, sums, sqsums, workspace,
                                     as_stream(stream)),
                 sums_strided<double>(num_samples, x_geometry, x, sums, sqsums, workspace,
                                      as_stream(stream)));
}

extern "C" int h2x_bn_sums_to_statistics(h2x_dtype dtype, int num_channels, size_t num_per_sum,
                                         double decay, void* mean_inout, void* var_inout,
                                         void* running_mean, void* running_var,
                                         h2x_stream_t stream)
{
    if (num_channels < 0 || !mean_inout || !var_inout || !running_mean || !running_var)
        return H2X_ERR_INVALID_ARGUMENT;
    H2X_BY_DTYPE(dtype,
                 statistics_impl<float>(num_channels, num_per_sum, decay, mean_inout, var_inout,
                                        running_mean, running_var, as_stream(stream)),
                 statistics_impl<double>(num_channels, num_per_sum, decay, mean_inout, var_inout,
                                         running_mean, running_var, as_stream(stream)));
}

extern "C" int h2x_bn_batch_normalization(h2x_dtype dtype, int num_samples, int num_channels,
                                          size_t spatial_size, size_t x_spatial_real_size,
                                          size_t y_spatial_real_size, const void* x,
                                          const void* mean, const void* var, const void* scale,
                                          const void* bias, void* y, double epsilon,
                                          h2x_stream_t stream)
{
    if (bad_geometry(num_samples, num_channels, spatial_size, x_spatial_real_size)
        || y_spatial_real_size < spatial_size || !mean || !var || !scale || !bias)
        return H2X_ERR_INVALID_ARGUMENT;
    if ((!x || !y) && static_cast<size_t>(num_samples) * num_channels * spatial_size > 0)
        return H2X_ERR_INVALID_ARGUMENT;
    const int n = num_samples, c = num_channels;
    const size_t s = spatial_size;
    H2X_BY_DTYPE(dtype,
                 apply_impl<float>(n, c, s, dense_tensor<float>(x, c, s, x_spatial_real_size),
                                   dense_tensor<float>(y, c, s, y_spatial_real_size), x, mean, var,
                                   scale, bias, y, epsilon, as_stream(stream)),
                 apply_impl<double>(n, c, s, dense_tensor<double>(x, c, s, x_spatial_real_size),
                                    dense_tensor<double>(y, c, s, y_spatial_real_size), x, mean, var,
                                    scale, bias, y, epsilon, as_stream(stream)));
}

extern "C" int h2x_bn_batch_normalization_strided(h2x_dtype dtype, int num_samples,
                                                  const h2x_tensor_geometry* x_geometry,
                                                  const h2x_tensor_geometry* y_geometry,
                                                  const void* x, const void* mean, const void* var,
                                                  const void* scale, const void* bias, void* y,
                                                  double epsilon, h2x_stream_t stream)
{
    if (num_samples < 0 || !x_geometry || !y_geometry || !mean || !var || !scale || !bias)
        return H2X_ERR_INVALID_ARGUMENT;
    H2X_BY_DTYPE(dtype,
                 apply_strided<float>(num_samples, x_geometry, y_geometry, x, mean, var, scale, bias,
                                      y, epsilon, as_stream(stream)),
                 apply_strided<double>(num_samples, x_geometry, y_geometry, x, mean, var, scale,
                                       bias, y, epsilon, as_stream(stream)));
}

extern "C" int h2x_bn_backprop1(h2x_dtype dtype, int num_samples, int num_channels,
                                size_t spatial_size, size_t x_spatial_real_size,
                                size_t dy_spatial_real_size, const void* x, const void* dy,
                                const void* mean, const void* var, const void* scale, void* dscale,
                                void* dbias, void* dmean, void* dvar, double epsilon,
                                void* workspace, h2x_stream_t stream)
{
    if (bad_geometry(num_samples, num_channels, spatial_size, x_spatial_real_size)
        || dy_spatial_real_size < spatial_size || !mean || !var || !scale || !dscale || !dbias
        || !dmean || !dvar || !workspace)
        return H2X_ERR_INVALID_ARGUMENT;
    if ((!x || !dy) && static_cast<size_t>(num_samples) * num_channels * spatial_size > 0)
        return H2X_ERR_INVALID_ARGUMENT;
    const int n = num_samples, c = num_channels;
    const size_t s = spatial_size;
    H2X_BY_DTYPE(dtype,
                 backprop1_impl<float>(n, c, s, dense_tensor<float>(x, c, s, x_spatial_real_size),
                                       dense_tensor<float>(dy, c, s, dy_spatial_real_size), x, dy,
                                       mean, var, scale, dscale, dbias, dmean, dvar, epsilon,
                                       workspace, as_stream(stream)),
                 backprop1_impl<double>(n, c, s, dense_tensor<double>(x, c, s, x_spatial_real_size),
                                        dense_tensor<double>(dy, c, s, dy_spatial_real_size), x, dy,
                                        mean, var, scale, dscale, dbias, dmean, dvar, epsilon,
                                        workspace, as_stream(stream)));
}

extern "C" int h2x_bn_backprop1_strided(h2x_dtype dtype, int num_samples,
                                        const h2x_tensor_geometry* x_geometry,
                                        const h2x_tensor_geometry* dy_geometry, const void* x,
                                        const void* dy, const void* mean, const void* var,
                                        const void* scale, void* dscale, void* dbias, void* dmean,
                                        void* dvar, double epsilon, void* workspace,
                                        h2x_stream_t stream)
{
    if (num_samples < 0 || !x_geometry || !dy_geometry || !mean || !var || !scale || !dscale
        || !dbias || !dmean || !dvar || !workspace)
        return H2X_ERR_INVALID_ARGUMENT;
    H2X_BY_DTYPE(dtype,
                 backprop1_strided<float>(num_samples, x_geometry, dy_geometry, x, dy, mean, var,
                                          scale, dscale, dbias, dmean, dvar, epsilon, workspace,
                                          as_stream(stream)),
                 backprop1_strided<double>(num_samples, x_geometry, dy_geometry, x, dy, mean, var,
                                           scale, dscale, dbias, dmean, dvar, epsilon, workspace,
                                           as_stream(stream)));
}

extern "C" int h2x_bn_backprop2(h2x_dtype dtype, int num_samples, int num_channels,
                                size_t spatial_size, size_t x_spatial_real_size,
                                size_t dy_spatial_real_size, size_t dx_spatial_real_size,
                                size_t num_per_sum, const void* x, const void* dy,
                                const void* mean, const void* var, const void* scale,
                                const void* dmean, const void* dvar, void* dx, double epsilon,
                                h2x_stream_t stream)
{
    if (bad_geometry(num_samples, num_channels, spatial_size, x_spatial_real_size)
        || dy_spatial_real_size < spatial_size || dx_spatial_real_size < spatial_size || !mean
        || !var || !scale || !dmean || !dvar)
        return H2X_ERR_INVALID_ARGUMENT;
    if ((!x || !dy || !dx) && static_cast<size_t>(num_samples) * num_channels * spatial_size > 0)
        return H2X_ERR_INVALID_ARGUMENT;
    const int n = num_samples, c = num_channels;
    const size_t s = spatial_size;
    H2X_BY_DTYPE(dtype,
                 backprop2_impl<float>(n, c, s, num_per_sum,
                                       dense_tensor<float>(x, c, s, x_spatial_real_size),
                                       dense_tensor<float>(dy, c, s, dy_spatial_real_size),
                                       dense_tensor<float>(dx, c, s, dx_spatial_real_size), x, dy,
                                       mean, var, scale, dmean, dvar, dx, epsilon, as_stream(stream)),
                 backprop2_impl<double>(n, c, s, num_per_sum,
                                        dense_tensor<double>(x, c, s, x_spatial_real_size),
                                        dense_tensor<double>(dy, c, s, dy_spatial_real_size),
                                        dense_tensor<double>(dx, c, s, dx_spatial_real_size), x, dy,
                                        mean, var, scale, dmean, dvar, dx, epsilon,
                                        as_stream(stream)));
}

extern "C" int h2x_bn_backprop2_strided(h2x_dtype dtype, int num_samples, size_t num_per_sum,
                                        const h2x_tensor_geometry* x_geometry,
                                        const h2x_tensor_geometry* dy_geometry,
                                        const h2x_tensor_geometry* dx_geometry, const void* x,
                                        const void* dy, const void* mean, const void* var,
                                        const void* scale, const void* dmean, const void* dvar,
                                        void* dx, double epsilon, h2x_stream_t stream)
{
    if (num_samples < 0 || !x_geometry || !dy_geometry || !dx_geometry || !mean || !var || !scale
        || !dmean || !dvar)
        return H2X_ERR_INVALID_ARGUMENT;
    H2X_BY_DTYPE(dtype,
                 backprop2_strided<float>(num_samples, num_per_sum, x_geometry, dy_geometry,
                                          dx_geometry, x, dy, mean, var, scale, dmean, dvar, dx,
                                          epsilon, as_stream(stream)),
                 backprop2_strided<double>(num_samples, num_per_sum, x_geometry, dy_geometry,
                                           dx_geometry, x, dy, mean, var, scale, dmean, dvar, dx,
                                           epsilon, as_stream(stream)));
}

extern "C" int h2x_bn_batch_normalization_clearing(h2x_dtype dtype,
                                                   const h2x_haloed_geometry* geometry,
                                                   const void* x_buffer, const void* mean,
                                                   const void* var, const void* scale,
                                                   const void* bias, void* y_buffer, double epsilon,
                                                   h2x_stream_t stream)
{
    if (!geometry || !mean || !var || !scale || !bias)
        return H2X_ERR_INVALID_ARGUMENT;
    H2X_BY_DTYPE(dtype,
                 clearing_impl<float>(false, 0, geometry, x_buffer, nullptr, mean, var, scale, bias,
                                      nullptr, nullptr, y_buffer, epsilon, as_stream(stream)),
                 clearing_impl<double>(false, 0, geometry, x_buffer, nullptr, mean, var, scale, bias,
                                       nullptr, nullptr, y_buffer, epsilon, as_stream(stream)));
}

extern "C" int h2x_bn_backprop2_clearing(h2x_dtype dtype, size_t num_per_sum,
                                         const h2x_haloed_geometry* geometry, const void* x_buffer,
                                         const void* dy_buffer, const void* mean, const void* var,
                                         const void* scale, const void* dmean, const void* dvar,
                                         void* dx_buffer, double epsilon, h2x_stream_t stream)
{
    if (!geometry || !mean || !var || !scale || !dmean || !dvar)
        return H2X_ERR_INVALID_ARGUMENT;
    H2X_BY_DTYPE(dtype,
                 clearing_impl<float>(true, num_per_sum, geometry, x_buffer, dy_buffer, mean, var,
                                      scale, nullptr, dmean, dvar, dx_buffer, epsilon,
                                      as_stream(stream)),
                 clearing_impl<double>(true, num_per_sum, geometry, x_buffer, dy_buffer, mean, var,
                                       scale, nullptr, dmean, dvar, dx_buffer, epsilon,
                                       as_stream(stream)));
}

extern "C" int h2x_bn_forward_local(h2x_dtype dtype, int num_samples, int num_channels,
                                    size_t spatial_size, size_t x_spatial_real_size,
                                    size_t y_spatial_real_size, const void* x, const void* scale,
                                    const void* bias, size_t num_per_sum, double decay,
                                    double epsilon, void* mean, void* var, void* running_mean,
                                    void* running_var, void* y, void* workspace,
                                    h2x_stream_t stream)
{
    if (bad_geometry(num_samples, num_channels, spatial_size, x_spatial_real_size)
        || y_spatial_real_size < spatial_size || !scale || !bias || !mean || !var || !running_mean
        || !running_var || !workspace)
        return H2X_ERR_INVALID_ARGUMENT;
    if ((!x || !y) && static_cast<size_t>(num_samples) * num_channels * spatial_size > 0)
        return H2X_ERR_INVALID_ARGUMENT;
    H2X_BY_DTYPE(dtype,
                 forward_local<float>(
                     num_samples, num_channels, spatial_size,
                     dense_tensor<float>(x, num_channels, spatial_size, x_spatial_real_size),
                     dense_tensor<float>(y, num_channels, spatial_size, y_spatial_real_size), x, scale,
                     bias, num_per_sum, decay, epsilon, mean, var, running_mean, running_var, y,
                     workspace, as_stream(stream)),
                 forward_local<double>(
                     num_samples, num_channels, spatial_size,
                     dense_tensor<double>(x, num_channels, spatial_size, x_spatial_real_size),
                     dense_tensor<double>(y, num_channels, spatial_size, y_spatial_real_size), x, scale,
                     bias, num_per_sum, decay, epsilon, mean, var, running_mean, running_var, y,
                     workspace, as_stream(stream)));
}

extern "C" int h2x_bn_forward_local_strided(h2x_dtype dtype, int num_samples,
                                            const h2x_tensor_geometry* x_geometry,
                                            const h2x_tensor_geometry* y_geometry, const void* x,
                                            const void* scale, const void* bias, size_t num_per_sum,
                                            double decay, double epsilon, void* mean, void* var,
                                            void* running_mean, void* running_var, void* y,
                                            void* workspace, h2x_stream_t stream)
{
    if (num_samples < 0 || !x_geometry || !y_geometry || !scale || !bias || !mean || !var
        || !running_mean || !running_var || !workspace)
        return H2X_ERR_INVALID_ARGUMENT;
    H2X_BY_DTYPE(dtype,
                 forward_local_strided<float>(num_samples, x_geometry, y_geometry, x, scale, bias,
                                              num_per_sum, decay, epsilon, mean, var, running_mean,
                                              running_var, y, workspace, as_stream(stream)),
                 forward_local_strided<double>(num_samples, x_geometry, y_geometry, x, scale, bias,
                                               num_per_sum, decay, epsilon, mean, var, running_mean,
                                               running_var, y, workspace, as_stream(stream)));
}

extern "C" int h2x_bn_backward_local(h2x_dtype dtype, int num_samples, int num_channels,
                                     size_t spatial_size, size_t x_spatial_real_size,
                                     size_t dy_spatial_real_size, size_t dx_spatial_real_size,
                                     size_t num_per_sum, const void* x, const void* dy,
                                     const void* mean, const void* var, const void* scale,
                                     void* dscale, void* dbias, void* dmean, void* dvar, void* dx,
                                     double epsilon, void* workspace, h2x_stream_t stream)
{
    if (bad_geometry(num_samples, num_channels, spatial_size, x_spatial_real_size)
        || dy_spatial_real_size < spatial_size || dx_spatial_real_size < spatial_size || !mean
        || !var || !scale || !dscale || !dbias || !dmean || !dvar || !workspace)
        return H2X_ERR_INVALID_ARGUMENT;
    if ((!x || !dy || !dx) && static_cast<size_t>(num_samples) * num_channels * spatial_size > 0)
        return H2X_ERR_INVALID_ARGUMENT;
    H2X_BY_DTYPE(dtype,
                 backward_local<float>(
                     num_samples, num_channels, spatial_size,
                     dense_tensor<float>(x, num_channels, spatial_size, x_spatial_real_size),
                     dense_tensor<float>(dy, num_channels, spatial_size, dy_spatial_real_size),
                     dense_tensor<float>(dx, num_channels, spatial_size, dx_spatial_real_size),
                     num_per_sum, x, dy, mean, var, scale, dscale, dbias, dmean, dvar, dx, epsilon,
                     workspace, as_stream(stream)),
                 backward_local<double>(
                     num_samples, num_channels, spatial_size,
                     dense_tensor<double>(x, num_channels, spatial_size, x_spatial_real_size),
                     dense_tensor<double>(dy, num_channels, spatial_size, dy_spatial_real_size),
                     dense_tensor<double>(dx, num_channels, spatial_size, dx_spatial_real_size),
                     num_per_sum, x, dy, mean, var, scale, dscale, dbias, dmean, dvar, dx, epsilon,
                     workspace, as_stream(stream)));
}

extern "C" int h2x_bn_backward_local_strided(h2x_dtype dtype, int num_samples, size_t num_per_sum,
                                             const h2x_tensor_geometry* x_geometry,
                                             const h2x_tensor_geometry* dy_geometry,
                                             const h2x_tensor_geometry* dx_geometry, const void* x,
                                             const void* dy, const void* mean, const void* var,
                                             const void* scale, void* dscale, void* dbias,
                                             void* dmean, void* dvar, void* dx, double epsilon,
                                             void* workspace, h2x_stream_t stream)
{
    if (num_samples < 0 || !x_geometry || !dy_geometry || !dx_geometry || !mean || !var || !scale
        || !dscale || !dbias || !dmean || !dvar || !workspace)
        return H2X_ERR_INVALID_ARGUMENT;
    H2X_BY_DTYPE(dtype,
                 backward_local_strided<float>(num_samples, num_per_sum, x_geometry, dy_geometry,
                                               dx_geometry, x, dy, mean, var, scale, dscale, dbias,
                                               dmean, dvar, dx, epsilon, workspace, as_stream(stream)),
                 backward_local_strided<double>(num_samples, num_per_sum, x_geometry, dy_geometry,
                                                dx_geometry, x, dy, mean, var, scale, dscale, dbias,
                                                dmean, dvar, dx, epsilon, workspace,
                                                as_stream(stream)));
}

// Channel softmax (forward, backward) for gfx950 and the C entry points.
//
// Tensors are dense [N][C][S]; the softmax runs over C, so the C values of one
// pixel are S elements apart while neighbouring pixels are contiguous.  A
// thread owns VEC neighbouring pixels and keeps all C values of them in
// registers (the channel loop is unrolled to a compile-time bound CMAX >= C),
// so x (or y and dy) is read from HBM exactly once with fully coalesced
// 4*VEC-byte accesses and no LDS staging; the reference stages a
// C x 256 tile in LDS and walks it three times
// (legacy/src/dnn_backend/softmax.cu:538-593,621-669).  Above 32 channels the
// four waves of a workgroup share the channels of 64 * VEC pixels, still in
// registers; channel counts beyond the largest such tile fall back to a kernel
// that re-reads its inputs; tensors with one pixel per sample have kernels
// that put the channels, which are contiguous then, on the lanes of a wave or,
// beyond 2048 channels, on the threads of a workgroup.
#include "h2x_device.hpp"

#include <cfloat>
#include <cmath>

namespace h2x
{
namespace
{

template <typename T>
struct Limits;
template <>
struct Limits<float>
{
    static constexpr float min_normal = FLT_MIN;
};
template <>
struct Limits<double>
{
    static constexpr double min_normal = DBL_MIN;
};

__device__ __forceinline__ float exp_t(float v)
{
    return expf(v);
}
__device__ __forceinline__ double exp_t(double v)
{
    return exp(v);
}
__device__ __forceinline__ float fma_t(float a, float b, float c)
{
    return __builtin_fmaf(a, b, c);
}
__device__ __forceinline__ double fma_t(double a, double b, double c)
{
    return __builtin_fma(a, b, c);
}

// VEC neighbouring pixels of one channel.
template <typename T, int VEC>
struct Pack
{
    T e[VEC];
    __device__ __forceinline__ T& operator[](int j) { return e[j]; }
    __device__ __forceinline__ const T& operator[](int j) const { return e[j]; }

    static __device__ __forceinline__ Pack load(const T* p)
    {
        Pack r;
        if constexpr (VEC == 1)
        {
            r.e[0] = *p;
        }
        else
        {
            typedef T V __attribute__((ext_vector_type(VEC)));
            const V t = *reinterpret_cast<const V*>(p);
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                r.e[j] = t[j];
        }
        return r;
    }
    static __device__ __forceinline__ void store(T* p, const Pack& r)
    {
        if constexpr (VEC == 1)
        {
            *p = r.e[0];
        }
        else
        {
            typedef T V __attribute__((ext_vector_type(VEC)));
            V t;
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                t[j] = r.e[j];
            *reinterpret_cast<V*>(p) = t;
        }
    }
};

// Where the VEC pixels of a lane start (offset of their first channel) and
// whether they exist; `index` counts the lanes of the grid's x dimension in tile
// order.  Tensors with few pixels per sample (flat_samples > 0; one pixel a lane)
// count their pixels through all samples, so that a tile of 64 or 256 pixels is
// full whatever the size of a sample; otherwise blockIdx.y is the sample.
template <int VEC>
__device__ __forceinline__ bool lane_pixels(size_t index, int num_channels, size_t spatial,
                                            int flat_samples, size_t* base)
{
    const size_t p = index * VEC;
    if (flat_samples > 0)
    {
        const unsigned int n = static_cast<unsigned int>(p) / static_cast<unsigned int>(spatial);
        const bool exists = n < static_cast<unsigned int>(flat_samples);
        *base = exists ? static_cast<size_t>(n) * num_channels * spatial + (p - n * spatial) : 0;
        return exists;
    }
    const bool exists = p < spatial;
    *base = static_cast<size_t>(blockIdx.y) * num_channels * spatial + (exists ? p : 0);
    return exists;
}

// forward, register-resident.  Replaces fp_channel_kernel, softmax.cu:538-593:
// running maximum starts at min_normal (positive), the sum is taken in channel
// order, y = max(e * (1 / sum), min_normal).
template <typename T, int VEC, int CMAX>
__global__ __launch_bounds__(kBlockSize) void softmax_fwd_reg_kernel(
    const T* __restrict__ x, T* __restrict__ y, int num_channels, size_t spatial, int flat_samples)
{
    using P = Pack<T, VEC>;
    size_t base;
    if (!lane_pixels<VEC>(static_cast<size_t>(xcd_contiguous(blockIdx.x, gridDim.x)) * kBlockSize
                              + threadIdx.x,
                          num_channels, spatial, flat_samples, &base))
        return;
    const T* xp = x + base;
    T* yp = y + base;
    constexpr T kMin = Limits<T>::min_normal;

    P v[CMAX];
#pragma unroll
    for (int c = 0; c < CMAX; ++c)
        if (c < num_channels)
            v[c] = P::load(xp + static_cast<size_t>(c) * spatial);

    T mx[VEC], sum[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j)
    {
        mx[j] = kMin;
        sum[j] = T(0);
    }
#pragma unroll
    for (int c = 0; c < CMAX; ++c)
        if (c < num_channels)
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                mx[j] = v[c][j] > mx[j] ? v[c][j] : mx[j];
#pragma unroll
    for (int c = 0; c < CMAX; ++c)
        if (c < num_channels)
#pragma unroll
            for (int j = 0; j < VEC; ++j)
            {
                const T e = exp_t(v[c][j] - mx[j]);
                v[c][j] = e;
                sum[j] += e;
            }
#pragma unroll
    for (int j = 0; j < VEC; ++j)
        sum[j] = T(1) / sum[j];
#pragma unroll
    for (int c = 0; c < CMAX; ++c)
        if (c < num_channels)
        {
#pragma unroll
            for (int j = 0; j < VEC; ++j)
            {
                const T r = v[c][j] * sum[j];
                v[c][j] = r > kMin ? r : kMin;
            }
            P::store(yp + static_cast<size_t>(c) * spatial, v[c]);
        }
}

constexpr int kWideBatch = 8;

// forward, any channel count.  A workgroup serves 64 neighbouring pixels; its
// four waves share the channels (wave g takes c = g, g + 4, ...), combine their
// maxima and sums through LDS in wave order, and walk their channels again for
// the second and third pass; the tile is 64 * C elements, so those re-reads are
// served by the L2.  The sum is formed from four partial sums instead of one
// running sum over all channels (softmax.cu:565-580).
template <typename T>
__global__ __launch_bounds__(kBlockSize) void softmax_fwd_wide_kernel(
    const T* __restrict__ x, T* __restrict__ y, int num_channels, size_t spatial, int flat_samples)
{
    __shared__ T lds[kWavesPerBlock][kWaveSize];
    const int lane = threadIdx.x % kWaveSize;
    const int g = threadIdx.x / kWaveSize;
    size_t base;
    const bool active =
        lane_pixels<1>(static_cast<size_t>(xcd_contiguous(blockIdx.x, gridDim.x)) * kWaveSize + lane,
                       num_channels, spatial, flat_samples, &base);
    const T* xp = x + base;
    T* yp = y + base;
    constexpr T kMin = Limits<T>::min_normal;

    // kWideBatch loads are issued together in every pass: the channel loop of a
    // wave is a chain of dependent operations on values that are a memory
    // latency away each (N 8, C 1000, 64 x 64 backward: 334 us one by one)
    constexpr int kStep = kWavesPerBlock * kWideBatch;
    T mx = kMin;
    if (active)
        for (int c0 = g; c0 < num_channels; c0 += kStep)
        {
            T v[kWideBatch];
#pragma unroll
            for (int u = 0; u < kWideBatch; ++u)
                if (c0 + u * kWavesPerBlock < num_channels)
                    v[u] = xp[static_cast<size_t>(c0 + u * kWavesPerBlock) * spatial];
#pragma unroll
            for (int u = 0; u < kWideBatch; ++u)
                if (c0 + u * kWavesPerBlock < num_channels)
                    mx = v[u] > mx ? v[u] : mx;
        }
    lds[g][lane] = mx;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; ++w)
        mx = lds[w][lane] > mx ? lds[w][lane] : mx;
    __syncthreads();

    T sum = T(0);
    if (active)
        for (int c0 = g; c0 < num_channels; c0 += kStep)
        {
            T v[kWideBatch];
#pragma unroll
            for (int u = 0; u < kWideBatch; ++u)
                if (c0 + u * kWavesPerBlock < num_channels)
                    v[u] = xp[static_cast<size_t>(c0 + u * kWavesPerBlock) * spatial];
#pragma unroll
            for (int u = 0; u < kWideBatch; ++u)
                if (c0 + u * kWavesPerBlock < num_channels)
                    sum += exp_t(v[u] - mx);
        }
    lds[g][lane] = sum;
    __syncthreads();
    sum = lds[0][lane];
#pragma unroll
    for (int w = 1; w < kWavesPerBlock; ++w)
        sum += lds[w][lane];
    const T inv = T(1) / sum;

    if (active)
        for (int c0 = g; c0 < num_channels; c0 += kStep)
        {
            T v[kWideBatch];
#pragma unroll
            for (int u = 0; u < kWideBatch; ++u)
                if (c0 + u * kWavesPerBlock < num_channels)
                    v[u] = xp[static_cast<size_t>(c0 + u * kWavesPerBlock) * spatial];
#pragma unroll
            for (int u = 0; u < kWideBatch; ++u)
                if (c0 + u * kWavesPerBlock < num_channels)
                {
                    const T r = exp_t(v[u] - mx) * inv;
                    yp[static_cast<size_t>(c0 + u * kWavesPerBlock) * spatial] = r > kMin ? r : kMin;
                }
        }
}

// backward, register-resident.  Replaces bp_channel_kernel, softmax.cu:621-669:
// dp accumulates y*dy in channel order with fused multiply-adds.
template <typename T, int VEC, int CMAX>
__global__ __launch_bounds__(kBlockSize) void softmax_bwd_reg_kernel(
    const T* __restrict__ y, const T* __restrict__ dy, T* __restrict__ dx, int num_channels,
    size_t spatial, int flat_samples)
{
    using P = Pack<T, VEC>;
    size_t base;
    if (!lane_pixels<VEC>(static_cast<size_t>(xcd_contiguous(blockIdx.x, gridDim.x)) * kBlockSize
                              + threadIdx.x,
                          num_channels, spatial, flat_samples, &base))
        return;
    const T* yp = y + base;
    const T* gp = dy + base;
    T* op = dx + base;
    constexpr T kMin = Limits<T>::min_normal;

    P yv[CMAX], gv[CMAX];
#pragma unroll
    for (int c = 0; c < CMAX; ++c)
        if (c < num_channels)
        {
            yv[c] = P::load(yp + static_cast<size_t>(c) * spatial);
            gv[c] = P::load(gp + static_cast<size_t>(c) * spatial);
        }
    T dp[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j)
        dp[j] = T(0);
#pragma unroll
    for (int c = 0; c < CMAX; ++c)
        if (c < num_channels)
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                dp[j] = fma_t(yv[c][j], gv[c][j], dp[j]);
#pragma unroll
    for (int c = 0; c < CMAX; ++c)
        if (c < num_channels)
        {
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                yv[c][j] = yv[c][j] > kMin ? yv[c][j] * (gv[c][j] - dp[j]) : T(0);
            P::store(op + static_cast<size_t>(c) * spatial, yv[c]);
        }
}

// backward, any channel count: the same tiling; dp is formed from the four
// waves' partial dot products.
template <typename T>
__global__ __launch_bounds__(kBlockSize) void softmax_bwd_wide_kernel(
    const T* __restrict__ y, const T* __restrict__ dy, T* __restrict__ dx, int num_channels,
    size_t spatial, int flat_samples)
{
    __shared__ T lds[kWavesPerBlock][kWaveSize];
    const int lane = threadIdx.x % kWaveSize;
    const int g = threadIdx.x / kWaveSize;
    size_t base;
    const bool active =
        lane_pixels<1>(static_cast<size_t>(xcd_contiguous(blockIdx.x, gridDim.x)) * kWaveSize + lane,
                       num_channels, spatial, flat_samples, &base);
    const T* yp = y + base;
    const T* gp = dy + base;
    T* op = dx + base;
    constexpr T kMin = Limits<T>::min_normal;

    constexpr int kStep = kWavesPerBlock * kWideBatch;
    T dp = T(0);
    if (active)
        for (int c0 = g; c0 < num_channels; c0 += kStep)
        {
            T yv[kWideBatch], gv[kWideBatch];
#pragma unroll
            for (int u = 0; u < kWideBatch; ++u)
                if (c0 + u * kWavesPerBlock < num_channels)
                {
                    yv[u] = yp[static_cast<size_t>(c0 + u * kWavesPerBlock) * spatial];
                    gv[u] = gp[static_cast<size_t>(c0 + u * kWavesPerBlock) * spatial];
                }
#pragma unroll
            for (int u = 0; u < kWideBatch; ++u)
                if (c0 + u * kWavesPerBlock < num_channels)
                    dp = fma_t(yv[u], gv[u], dp);
        }
    lds[g][lane] = dp;
    __syncthreads();
    dp = lds[0][lane];
#pragma unroll
    for (int w = 1; w < kWavesPerBlock; ++w)
        dp += lds[w][lane];

    if (active)
        for (int c0 = g; c0 < num_channels; c0 += kStep)
        {
            T yv[kWideBatch], gv[kWideBatch];
#pragma unroll
            for (int u = 0; u < kWideBatch; ++u)
                if (c0 + u * kWavesPerBlock < num_channels)
                {
                    yv[u] = yp[static_cast<size_t>(c0 + u * kWavesPerBlock) * spatial];
                    gv[u] = gp[static_cast<size_t>(c0 + u * kWavesPerBlock) * spatial];
                }
#pragma unroll
            for (int u = 0; u < kWideBatch; ++u)
                if (c0 + u * kWavesPerBlock < num_channels)
                    op[static_cast<size_t>(c0 + u * kWavesPerBlock) * spatial] =
                        yv[u] > kMin ? yv[u] * (gv[u] - dp) : T(0);
        }
}

// forward, up to WAVES * CPW channels, register-resident.  A workgroup serves
// 64 * VEC neighbouring pixels; its WAVES (four, or eight above 512 channels)
// waves share the channels (wave g takes c = g, g + WAVES, ...: CPW of them at
// most) and keep their values in registers, so
// x is read once; maxima and sums are combined through LDS in wave order.  The
// arithmetic, partial sums included, is that of softmax_fwd_wide_kernel, which
// re-reads its tile twice and whose tiles of 64 * C elements the L2 does not
// hold once every CU runs eight of them (N 16, C 150, 128 x 128: 100 us there,
// 60 us with the tile in registers).
template <typename T, int VEC, int CPW, int WAVES>
__global__ __launch_bounds__(WAVES * kWaveSize) void softmax_fwd_split_kernel(
    const T* __restrict__ x, T* __restrict__ y, int num_channels, size_t spatial, int flat_samples)
{
    using P = Pack<T, VEC>;
    __shared__ T lds[WAVES][kWaveSize * VEC];
    const int lane = threadIdx.x % kWaveSize;
    const int g = threadIdx.x / kWaveSize;
    size_t base;
    const bool active = lane_pixels<VEC>(
        static_cast<size_t>(xcd_contiguous(blockIdx.x, gridDim.x)) * kWaveSize + lane, num_channels,
        spatial, flat_samples, &base);
    const T* xp = x + base;
    T* yp = y + base;
    constexpr T kMin = Limits<T>::min_normal;

    P v[CPW];
    T mx[VEC], sum[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j)
    {
        mx[j] = kMin;
        sum[j] = T(0);
    }
    if (active)
    {
#pragma unroll
        for (int k = 0; k < CPW; ++k)
            if (g + k * WAVES < num_channels)
                v[k] = P::load(xp + static_cast<size_t>(g + k * WAVES) * spatial);
#pragma unroll
        for (int k = 0; k < CPW; ++k)
            if (g + k * WAVES < num_channels)
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    mx[j] = v[k][j] > mx[j] ? v[k][j] : mx[j];
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j)
        lds[g][lane * VEC + j] = mx[j];
    __syncthreads();
#pragma unroll
    for (int j = 0; j < VEC; ++j)
#pragma unroll
        for (int w = 0; w < WAVES; ++w)
            mx[j] = lds[w][lane * VEC + j] > mx[j] ? lds[w][lane * VEC + j] : mx[j];
    __syncthreads();

    if (active)
    {
#pragma unroll
        for (int k = 0; k < CPW; ++k)
            if (g + k * WAVES < num_channels)
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                {
                    const T e = exp_t(v[k][j] - mx[j]);
                    v[k][j] = e;
                    sum[j] += e;
                }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j)
        lds[g][lane * VEC + j] = sum[j];
    __syncthreads();
    T inv[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j)
    {
        T t = lds[0][lane * VEC + j];
#pragma unroll
        for (int w = 1; w < WAVES; ++w)
            t += lds[w][lane * VEC + j];
        inv[j] = T(1) / t;
    }
    if (active)
    {
#pragma unroll
        for (int k = 0; k < CPW; ++k)
            if (g + k * WAVES < num_channels)
            {
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                {
                    const T r = v[k][j] * inv[j];
                    v[k][j] = r > kMin ? r : kMin;
                }
                P::store(yp + static_cast<size_t>(g + k * WAVES) * spatial, v[k]);
            }
    }
}

// backward likewise: y and dy of up to WAVES * CPW channels in registers.
template <typename T, int VEC, int CPW, int WAVES>
__global__ __launch_bounds__(WAVES * kWaveSize) void softmax_bwd_split_kernel(
    const T* __restrict__ y, const T* __restrict__ dy, T* __restrict__ dx, int num_channels,
    size_t spatial, int flat_samples)
{
    using P = Pack<T, VEC>;
    __shared__ T lds[WAVES][kWaveSize * VEC];
    const int lane = threadIdx.x % kWaveSize;
    const int g = threadIdx.x / kWaveSize;
    size_t base;
    const bool active = lane_pixels<VEC>(
        static_cast<size_t>(xcd_contiguous(blockIdx.x, gridDim.x)) * kWaveSize + lane, num_channels,
        spatial, flat_samples, &base);
    const T* yp = y + base;
    const T* gp = dy + base;
    T* op = dx + base;
    constexpr T kMin = Limits<T>::min_normal;

    P yv[CPW], gv[CPW];
    T dp[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j)
        dp[j] = T(0);
    if (active)
    {
#pragma unroll
        for (int k = 0; k < CPW; ++k)
            if (g + k * WAVES < num_channels)
            {
                yv[k] = P::load(yp + static_cast<size_t>(g + k * WAVES) * spatial);
                gv[k] = P::load(gp + static_cast<size_t>(g + k * WAVES) * spatial);
            }
#pragma unroll
        for (int k = 0; k < CPW; ++k)
            if (g + k * WAVES < num_channels)
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    dp[j] = fma_t(yv[k][j], gv[k][j], dp[j]);
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j)
        lds[g][lane * VEC + j] = dp[j];
    __syncthreads();
#pragma unroll
    for (int j = 0; j < VEC; ++j)
    {
        T t = lds[0][lane * VEC + j];
#pragma unroll
        for (int w = 1; w < WAVES; ++w)
            t += lds[w][lane * VEC + j];
        dp[j] = t;
    }
    if (active)
    {
#pragma unroll
        for (int k = 0; k < CPW; ++k)
            if (g + k * WAVES < num_channels)
            {
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    yv[k][j] = yv[k][j] > kMin ? yv[k][j] * (gv[k][j] - dp[j]) : T(0);
                P::store(op + static_cast<size_t>(g + k * WAVES) * spatial, yv[k]);
            }
    }
}

// One pixel per sample (the output of a fully connected layer): the channels of
// a sample are contiguous, so a wave takes a sample, lane l the channels l,
// l + 64, ... (CPL of them at most), and maxima, sums and dot products are
// combined across the lanes with a butterfly of shuffles.  The kernels above
// would put one sample on each lane and read with a stride of C elements
// (N 256, C 1000: 176 us).
template <typename T>
__device__ __forceinline__ T wave_butterfly_sum(T v)
{
#pragma unroll
    for (int m = kWaveSize / 2; m >= 1; m >>= 1)
        v += __shfl_xor(v, m, kWaveSize);
    return v;
}

template <typename T, int CPL>
__global__ __launch_bounds__(kBlockSize) void softmax_fwd_row_kernel(
    const T* __restrict__ x, T* __restrict__ y, int num_channels, int num_samples)
{
    const int lane = threadIdx.x % kWaveSize;
    const int n = blockIdx.x * kWavesPerBlock + threadIdx.x / kWaveSize;
    if (n >= num_samples)
        return;
    const T* xp = x + static_cast<size_t>(n) * num_channels;
    T* yp = y + static_cast<size_t>(n) * num_channels;
    constexpr T kMin = Limits<T>::min_normal;
    T v[CPL];
    T mx = kMin;
#pragma unroll
    for (int k = 0; k < CPL; ++k)
        if (lane + k * kWaveSize < num_channels)
            v[k] = xp[lane + k * kWaveSize];
#pragma unroll
    for (int k = 0; k < CPL; ++k)
        if (lane + k * kWaveSize < num_channels)
            mx = v[k] > mx ? v[k] : mx;
#pragma unroll
    for (int m = kWaveSize / 2; m >= 1; m >>= 1)
    {
        const T o = __shfl_xor(mx, m, kWaveSize);
        mx = o > mx ? o : mx;
    }
    T sum = T(0);
#pragma unroll
    for (int k = 0; k < CPL; ++k)
        if (lane + k * kWaveSize < num_channels)
        {
            v[k] = exp_t(v[k] - mx);
            sum += v[k];
        }
    const T inv = T(1) / wave_butterfly_sum(sum);
#pragma unroll
    for (int k = 0; k < CPL; ++k)
        if (lane + k * kWaveSize < num_channels)
        {
            const T r = v[k] * inv;
            yp[lane + k * kWaveSize] = r > kMin ? r : kMin;
        }
}

template <typename T, int CPL>
__global__ __launch_bounds__(kBlockSize) void softmax_bwd_row_kernel(
    const T* __restrict__ y, const T* __restrict__ dy, T* __restrict__ dx, int num_channels,
    int num_samples)
{
    const int lane = threadIdx.x % kWaveSize;
    const int n = blockIdx.x * kWavesPerBlock + threadIdx.x / kWaveSize;
    if (n >= num_samples)
        return;
    const size_t base = static_cast<size_t>(n) * num_channels;
    constexpr T kMin = Limits<T>::min_normal;
    T yv[CPL], gv[CPL];
    T dp = T(0);
#pragma unroll
    for (int k = 0; k < CPL; ++k)
        if (lane + k * kWaveSize < num_channels)
        {
            yv[k] = y[base + lane + k * kWaveSize];
            gv[k] = dy[base + lane + k * kWaveSize];
        }
#pragma unroll
    for (int k = 0; k < CPL; ++k)
        if (lane + k * kWaveSize < num_channels)
            dp = fma_t(yv[k], gv[k], dp);
    dp = wave_butterfly_sum(dp);
#pragma unroll
    for (int k = 0; k < CPL; ++k)
        if (lane + k * kWaveSize < num_channels)
            dx[base + lane + k * kWaveSize] = yv[k] > kMin ? yv[k] * (gv[k] - dp) : T(0);
}

// One pixel per sample and more channels than a wave holds in registers: a
// workgroup takes a sample and walks its channels (contiguous) three times
// forward, twice backward; the re-reads come from the L2.  Thread t adds up the
// channels t, t + 256, ...; the lanes of a wave are combined as a butterfly and
// the waves through LDS in wave order.
template <typename T>
__device__ __forceinline__ T block_combine(T v, bool is_max, T* lds)
{
#pragma unroll
    for (int m = kWaveSize / 2; m >= 1; m >>= 1)
    {
        const T o = __shfl_xor(v, m, kWaveSize);
        v = is_max ? (o > v ? o : v) : v + o;
    }
    __syncthreads(); // lds may still be read from the previous call
    if ((threadIdx.x & (kWaveSize - 1)) == 0)
        lds[threadIdx.x / kWaveSize] = v;
    __syncthreads();
    T r = lds[0];
#pragma unroll
    for (int w = 1; w < kWavesPerBlock; ++w)
        r = is_max ? (lds[w] > r ? lds[w] : r) : r + lds[w];
    return r;
}

template <typename T>
__global__ __launch_bounds__(kBlockSize) void softmax_fwd_long_row_kernel(
    const T* __restrict__ x, T* __restrict__ y, int num_channels)
{
    __shared__ T lds[kWavesPerBlock];
    const T* xp = x + static_cast<size_t>(blockIdx.x) * num_channels;
    T* yp = y + static_cast<size_t>(blockIdx.x) * num_channels;
    constexpr T kMin = Limits<T>::min_normal;
    T mx = kMin;
    for (int c = threadIdx.x; c < num_channels; c += kBlockSize)
        mx = xp[c] > mx ? xp[c] : mx;
    mx = block_combine(mx, true, lds);
    T sum = T(0);
    for (int c = threadIdx.x; c < num_channels; c += kBlockSize)
        sum += exp_t(xp[c] - mx);
    const T inv = T(1) / block_combine(sum, false, lds);
    for (int c = threadIdx.x; c < num_channels; c += kBlockSize)
    {
        const T r = exp_t(xp[c] - mx) * inv;
        yp[c] = r > kMin ? r : kMin;
    }
}

template <typename T>
__global__ __launch_bounds__(kBlockSize) void softmax_bwd_long_row_kernel(
    const T* __restrict__ y, const T* __restrict__ dy, T* __restrict__ dx, int num_channels)
{
    __shared__ T lds[kWavesPerBlock];
    const size_t base = static_cast<size_t>(blockIdx.x) * num_channels;
    constexpr T kMin = Limits<T>::min_normal;
    T dp = T(0);
    for (int c = threadIdx.x; c < num_channels; c += kBlockSize)
        dp = fma_t(y[base + c], dy[base + c], dp);
    dp = block_combine(dp, false, lds);
    for (int c = threadIdx.x; c < num_channels; c += kBlockSize)
    {
        const T yi = y[base + c];
        dx[base + c] = yi > kMin ? yi * (dy[base + c] - dp) : T(0);
    }
}

// Largest vector (elements) usable for all of the given pointers.
template <typename T>
int vector_width(size_t spatial, int want, std::initializer_list<const void*> ptrs)
{
    int v = want;
    while (v > 1)
    {
        bool ok = spatial % v == 0;
        for (const void* p : ptrs)
            ok = ok && (reinterpret_cast<uintptr_t>(p) % (v * sizeof(T)) == 0);
        if (ok)
            break;
        v /= 2;
    }
    return v;
}

dim3 pixel_grid(size_t spatial, int vec, int num_samples)
{
    const size_t per_block = static_cast<size_t>(kBlockSize) * vec;
    return dim3(static_cast<unsigned int>((spatial + per_block - 1) / per_block), num_samples);
}

// Samples of fewer pixels than this have their pixels counted through all
// samples (one pixel a lane): a tile is full whatever the size of a sample
// (N 256, C 100, 7 x 7: one workgroup a sample with 49 of its 64 pixels, 17 us).
constexpr size_t kFlatBelow = 128;

int flat_samples(int num_samples, size_t spatial)
{
    return spatial < kFlatBelow && spatial * static_cast<size_t>(num_samples) < (1ull << 31)
               ? num_samples
               : 0;
}

// Tiles of lanes * vec pixels, padded to a multiple of the XCD count for kernels
// that reorder their tiles with xcd_contiguous (tiles past the end do nothing).
dim3 tile_grid(size_t spatial, int lanes, int vec, int num_samples, int flat)
{
    const size_t per_block = static_cast<size_t>(lanes) * vec;
    const size_t pixels = flat > 0 ? spatial * static_cast<size_t>(flat) : spatial;
    const size_t blocks = (pixels + per_block - 1) / per_block;
    return dim3(static_cast<unsigned int>((blocks + kNumXcd - 1) / kNumXcd * kNumXcd),
                flat > 0 ? 1 : num_samples);
}

dim3 pixel_grid_xcd(size_t spatial, int vec, int num_samples, int flat)
{
    return tile_grid(spatial, kBlockSize, vec, num_samples, flat);
}

// 64 * vec pixels per workgroup.
dim3 wide_grid(size_t spatial, int vec, int num_samples, int flat)
{
    return tile_grid(spatial, kWaveSize, vec, num_samples, flat);
}

template <typename T, int VEC, int CMAX>
void launch_fwd(const T* x, T* y, int n, int c, size_t s, hipStream_t st)
{
    const int flat = VEC == 1 ? flat_samples(n, s) : 0;
    softmax_fwd_reg_kernel<T, VEC, CMAX>
        <<<pixel_grid_xcd(s, VEC, n, flat), kBlockSize, 0, st>>>(x, y, c, s, flat);
}

template <typename T, int VEC, int CMAX>
void launch_bwd(const T* y, const T* dy, T* dx, int n, int c, size_t s, hipStream_t st)
{
    const int flat = VEC == 1 ? flat_samples(n, s) : 0;
    softmax_bwd_reg_kernel<T, VEC, CMAX>
        <<<pixel_grid_xcd(s, VEC, n, flat), kBlockSize, 0, st>>>(y, dy, dx, c, s, flat);
}

// Which kernel serves which channel count (float; measured on MI355X).  Up to
// 32 channels a thread keeps all channels of its pixels (softmax_*_reg_kernel:
// config 4, 21 channels, 28 / 40 us).  Beyond, the four waves of a workgroup
// share the channels (softmax_*_split_kernel) with the smallest register tile
// that holds them and two pixels a lane where the geometry allows: against one
// thread per pixel with 64 or 128 channels in registers, N 4, C 100, 256 x 256
// takes 34 instead of 68 us forward and 53 instead of 63 us backward; against
// the re-reading kernel N 16, C 150, 128 x 128 takes 60 instead of 100 us and 89
// instead of 150 us, N 8, C 256, 64 x 64 18 instead of 59 us and 19 instead of
// 55 us.  Tiles wider than needed cost time (every lane walks the whole tile
// under a predicate), hence the steps of 16.  More channels than the largest
// tile holds (eight waves: 1024 forward, 768 backward; double: 256) take the
// re-reading kernel.
template <typename T, int VEC, int CPW, int WAVES = kWavesPerBlock>
int launch_fwd_split(const T* x, T* y, int n, int c, size_t s, hipStream_t st)
{
    const int flat = VEC == 1 ? flat_samples(n, s) : 0;
    softmax_fwd_split_kernel<T, VEC, CPW, WAVES>
        <<<wide_grid(s, VEC, n, flat), WAVES * kWaveSize, 0, st>>>(x, y, c, s, flat);
    return launch_status();
}

template <typename T, int VEC, int CPW, int WAVES = kWavesPerBlock>
int launch_bwd_split(const T* y, const T* dy, T* dx, int n, int c, size_t s, hipStream_t st)
{
    const int flat = VEC == 1 ? flat_samples(n, s) : 0;
    softmax_bwd_split_kernel<T, VEC, CPW, WAVES>
        <<<wide_grid(s, VEC, n, flat), WAVES * kWaveSize, 0, st>>>(y, dy, dx, c, s, flat);
    return launch_status();
}

template <typename T>
int forward_impl(int n, int c, size_t s, const void* xv, void* yv, hipStream_t st)
{
    const T* x = static_cast<const T*>(xv);
    T* y = static_cast<T*>(yv);
    constexpr int kWords = sizeof(T) / 4;
    if (s == 1)
    {
        const unsigned int blocks = (static_cast<unsigned int>(n) + kWavesPerBlock - 1) / kWavesPerBlock;
#define H2X_FWD_ROW(CP)                                                                            \
    do                                                                                             \
    {                                                                                              \
        softmax_fwd_row_kernel<T, CP><<<blocks, kBlockSize, 0, st>>>(x, y, c, n);                   \
        return launch_status();                                                                    \
    } while (0)
        if (c <= 1 * kWaveSize) H2X_FWD_ROW(1);
        if (c <= 2 * kWaveSize) H2X_FWD_ROW(2);
        if (c <= 4 * kWaveSize) H2X_FWD_ROW(4);
        if (c <= 8 * kWaveSize) H2X_FWD_ROW(8);
        if (c <= 16 * kWaveSize) H2X_FWD_ROW(16);
        if (c <= 32 * kWaveSize) H2X_FWD_ROW(32);
#undef H2X_FWD_ROW
        softmax_fwd_long_row_kernel<T><<<n, kBlockSize, 0, st>>>(x, y, c);
        return launch_status();
    }
    const int v4 = s < kFlatBelow ? 1 : vector_width<T>(s, 4 / kWords, {xv, yv});
#define H2X_FWD(V, CM)                                                                             \
    do                                                                                             \
    {                                                                                              \
        launch_fwd<T, V, CM>(x, y, n, c, s, st);                                                   \
        return launch_status();                                                                    \
    } while (0)
    if constexpr (sizeof(T) == 4)
    {
        // 4 pixels per thread only while the channel values fit in 64 registers;
        // above that 2 pixels per thread run faster (config 4, 21 channels:
        // 29.5 us against 32.5 us), with twice the workgroups in flight
        if (v4 == 4)
        {
            if (c <= 8) H2X_FWD(4, 8);
            if (c <= 16) H2X_FWD(4, 16);
        }
        if (v4 >= 2)
        {
            if (c <= 8) H2X_FWD(2, 8);
            if (c <= 16) H2X_FWD(2, 16);
            if (c <= 32) H2X_FWD(2, 32);
            if (c <= 64) return launch_fwd_split<T, 2, 16>(x, y, n, c, s, st);
            if (c <= 128) return launch_fwd_split<T, 2, 32>(x, y, n, c, s, st);
            if (c <= 192) return launch_fwd_split<T, 2, 48>(x, y, n, c, s, st);
            if (c <= 256) return launch_fwd_split<T, 2, 64>(x, y, n, c, s, st);
        }
        if (c <= 8) H2X_FWD(1, 8);
        if (c <= 16) H2X_FWD(1, 16);
        if (c <= 32) H2X_FWD(1, 32);
        if (c <= 64) return launch_fwd_split<T, 1, 16>(x, y, n, c, s, st);
        if (c <= 128) return launch_fwd_split<T, 1, 32>(x, y, n, c, s, st);
        if (c <= 192) return launch_fwd_split<T, 1, 48>(x, y, n, c, s, st);
        if (c <= 256) return launch_fwd_split<T, 1, 64>(x, y, n, c, s, st);
        if (c <= 384) return launch_fwd_split<T, 1, 96>(x, y, n, c, s, st);
        if (c <= 512) return launch_fwd_split<T, 1, 128>(x, y, n, c, s, st);
        if (c <= 768) return launch_fwd_split<T, 1, 96, 8>(x, y, n, c, s, st);
        if (c <= 1024) return launch_fwd_split<T, 1, 128, 8>(x, y, n, c, s, st);
    }
    else
    {
        if (v4 == 2)
        {
            if (c <= 8) H2X_FWD(2, 8);
            if (c <= 16) H2X_FWD(2, 16);
            if (c <= 32) H2X_FWD(2, 32);
        }
        if (c <= 8) H2X_FWD(1, 8);
        if (c <= 16) H2X_FWD(1, 16);
        if (c <= 32) H2X_FWD(1, 32);
        if (c <= 64) return launch_fwd_split<T, 1, 16>(x, y, n, c, s, st);
        if (c <= 128) return launch_fwd_split<T, 1, 32>(x, y, n, c, s, st);
        if (c <= 192) return launch_fwd_split<T, 1, 48>(x, y, n, c, s, st);
        if (c <= 256) return launch_fwd_split<T, 1, 64>(x, y, n, c, s, st);
    }
#undef H2X_FWD
    const int flat = flat_samples(n, s);
    softmax_fwd_wide_kernel<T><<<wide_grid(s, 1, n, flat), kBlockSize, 0, st>>>(x, y, c, s, flat);
    return launch_status();
}

template <typename T>
int backward_impl(int n, int c, size_t s, const void* yv, const void* dyv, void* dxv,
                  hipStream_t st)
{
    const T* y = static_cast<const T*>(yv);
    const T* dy = static_cast<const T*>(dyv);
    T* dx = static_cast<T*>(dxv);
    constexpr int kWords = sizeof(T) / 4;
    if (s == 1)
    {
        const unsigned int blocks = (static_cast<unsigned int>(n) + kWavesPerBlock - 1) / kWavesPerBlock;
#define H2X_BWD_ROW(CP)                                                                            \
    do                                                                                             \
    {                                                                                              \
        softmax_bwd_row_kernel<T, CP><<<blocks, kBlockSize, 0, st>>>(y, dy, dx, c, n);              \
        return launch_status();                                                                    \
    } while (0)
        if (c <= 1 * kWaveSize) H2X_BWD_ROW(1);
        if (c <= 2 * kWaveSize) H2X_BWD_ROW(2);
        if (c <= 4 * kWaveSize) H2X_BWD_ROW(4);
        if (c <= 8 * kWaveSize) H2X_BWD_ROW(8);
        if (c <= 16 * kWaveSize) H2X_BWD_ROW(16);
        if (c <= 32 * kWaveSize) H2X_BWD_ROW(32);
#undef H2X_BWD_ROW
        softmax_bwd_long_row_kernel<T><<<n, kBlockSize, 0, st>>>(y, dy, dx, c);
        return launch_status();
    }
    const int v4 = s < kFlatBelow ? 1 : vector_width<T>(s, 4 / kWords, {yv, dyv, dxv});
#define H2X_BWD(V, CM)                                                                             \
    do                                                                                             \
    {                                                                                              \
        launch_bwd<T, V, CM>(y, dy, dx, n, c, s, st);                                              \
        return launch_status();                                                                    \
    } while (0)
    if constexpr (sizeof(T) == 4)
    {
        if (v4 == 4)
        {
            if (c <= 8) H2X_BWD(4, 8);
            if (c <= 16) H2X_BWD(4, 16);
        }
        if (v4 >= 2)
        {
            if (c <= 8) H2X_BWD(2, 8);
            if (c <= 16) H2X_BWD(2, 16);
            if (c <= 32) H2X_BWD(2, 32);
            if (c <= 64) return launch_bwd_split<T, 2, 16>(y, dy, dx, n, c, s, st);
            if (c <= 128) return launch_bwd_split<T, 2, 32>(y, dy, dx, n, c, s, st);
            if (c <= 192) return launch_bwd_split<T, 2, 48>(y, dy, dx, n, c, s, st);
            if (c <= 256) return launch_bwd_split<T, 2, 64>(y, dy, dx, n, c, s, st);
        }
        if (c <= 8) H2X_BWD(1, 8);
        if (c <= 16) H2X_BWD(1, 16);
        if (c <= 32) H2X_BWD(1, 32);
        if (c <= 64) return launch_bwd_split<T, 1, 16>(y, dy, dx, n, c, s, st);
        if (c <= 128) return launch_bwd_split<T, 1, 32>(y, dy, dx, n, c, s, st);
        if (c <= 192) return launch_bwd_split<T, 1, 48>(y, dy, dx, n, c, s, st);
        if (c <= 256) return launch_bwd_split<T, 1, 64>(y, dy, dx, n, c, s, st);
        if (c <= 384) return launch_bwd_split<T, 1, 96>(y, dy, dx, n, c, s, st);
        if (c <= 512) return launch_bwd_split<T, 1, 128>(y, dy, dx, n, c, s, st);
        if (c <= 768) return launch_bwd_split<T, 1, 96, 8>(y, dy, dx, n, c, s, st);
    }
    else
    {
        if (v4 == 2)
        {
            if (c <= 8) H2X_BWD(2, 8);
            if (c <= 16) H2X_BWD(2, 16);
        }
        if (c <= 8) H2X_BWD(1, 8);
        if (c <= 16) H2X_BWD(1, 16);
        if (c <= 32) H2X_BWD(1, 32);
        if (c <= 64) return launch_bwd_split<T, 1, 16>(y, dy, dx, n, c, s, st);
        if (c <= 128) return launch_bwd_split<T, 1, 32>(y, dy, dx, n, c, s, st);
        if (c <= 192) return launch_bwd_split<T, 1, 48>(y, dy, dx, n, c, s, st);
        if (c <= 256) return launch_bwd_split<T, 1, 64>(y, dy, dx, n, c, s, st);
    }
#undef H2X_BWD
    const int flat = flat_samples(n, s);
    softmax_bwd_wide_kernel<T><<<wide_grid(s, 1, n, flat), kBlockSize, 0, st>>>(y, dy, dx, c, s, flat);
    return launch_status();
}

// ---- instance mode -----------------------------------------------------------
// Softmax over all elements of a sample (legacy/src/dnn_backend/softmax.cu:179-536,
// 705-784): per-sample maximum, exp(x - max) with per-sample sum, y / sum clamped
// to sqrt(min_normal); backward: per-sample dot product, then the gradient.  The
// reference finishes its per-sample reductions with atomics; here every
// workgroup stores a partial (fp64 for sums) and a second small kernel combines
// them in index order.  A sample is a contiguous block of `sample_size`
// elements (dense tensor), so every pass is a plain 16-byte stream.

constexpr int kInstUnroll = 4;
constexpr int kInstTargetGroups = 4096;
constexpr int kInstMaxGroupsPerSample = 2048;

int inst_groups_per_sample_max(int num_samples)
{
    const int g = (kInstTargetGroups + num_samples - 1) / (num_samples > 0 ? num_samples : 1);
    return g < 8 ? 8 : (g > kInstMaxGroupsPerSample ? kInstMaxGroupsPerSample : g);
}

template <typename T>
__device__ __forceinline__ T wave_max(T v)
{
#pragma unroll
    for (int d = 1; d < kWaveSize; d *= 2)
    {
        const T o = __shfl_xor(v, d, kWaveSize);
        v = o > v ? o : v;
    }
    return v;
}

enum InstReduce : int
{
    kInstMax = 0,   // max x                       -> T partial
    kInstExpSum = 1, // y = exp(x - max); sum y     -> double partial
    kInstDot = 2,    // sum y * dy                  -> double partial
    kInstSumExp = 3  // sum exp(x - max), y untouched -> double partial
};

// One pass over the chunk [begin, end) of sample n.  a: x (max, exp) or y (dot);
// b: dy (dot); out: y (exp).  Partials are stored as doubles in all modes.
template <typename T, int VEC, int MODE>
__global__ __launch_bounds__(kBlockSize) void softmax_inst_reduce_kernel(
    const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ out,
    const T* __restrict__ sample_param, double* partials, size_t sample_size, size_t chunk,
    int groups_max)
{
    using P = Pack<T, VEC>;
    __shared__ double lds[kWavesPerBlock];
    const int n = blockIdx.y;
    const size_t begin = static_cast<size_t>(blockIdx.x) * chunk;
    const size_t end = begin + chunk < sample_size ? begin + chunk : sample_size;
    const T* ap = a + static_cast<size_t>(n) * sample_size;
    const T* bp = MODE == kInstDot ? b + static_cast<size_t>(n) * sample_size : nullptr;
    T* op = MODE == kInstExpSum ? out + static_cast<size_t>(n) * sample_size : nullptr;
    const T shift = (MODE == kInstExpSum || MODE == kInstSumExp) ? sample_param[n] : T(0);
    constexpr size_t kStride = static_cast<size_t>(kBlockSize) * VEC;

    T mx = Limits<T>::min_normal; // softmax.cu:88-99: the maximum starts at min_normal
    double acc = 0.0;
    for (size_t i = begin + threadIdx.x * VEC; i < end; i += kStride * kInstUnroll)
    {
        P va[kInstUnroll], vb[kInstUnroll];
#pragma unroll
        for (int u = 0; u < kInstUnroll; ++u)
            if (i + u * kStride < end)
            {
                va[u] = P::load(ap + i + u * kStride);
                if constexpr (MODE == kInstDot)
                    vb[u] = P::load(bp + i + u * kStride);
            }
#pragma unroll
        for (int u = 0; u < kInstUnroll; ++u)
            if (i + u * kStride < end)
            {
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                {
                    if constexpr (MODE == kInstMax)
                    {
                        mx = va[u][j] >= mx ? va[u][j] : mx;
                    }
                    else if constexpr (MODE == kInstExpSum || MODE == kInstSumExp)
                    {
                        const T e = exp_t(va[u][j] - shift);
                        va[u][j] = e;
                        acc += static_cast<double>(e);
                    }
                    else
                    {
                        acc = __builtin_fma(static_cast<double>(va[u][j]),
                                            static_cast<double>(vb[u][j]), acc);
                    }
                }
                if constexpr (MODE == kInstExpSum)
                    P::store(op + i + u * kStride, va[u]);
            }
    }
    double part;
    if constexpr (MODE == kInstMax)
    {
        mx = wave_max(mx);
        if ((threadIdx.x & (kWaveSize - 1)) == 0)
            lds[threadIdx.x / kWaveSize] = static_cast<double>(mx);
        __syncthreads();
        part = lds[0];
#pragma unroll
        for (int w = 1; w < kWavesPerBlock; ++w)
            part = lds[w] > part ? lds[w] : part;
    }
    else
    {
        double v[1] = {acc};
        block_sum<1>(v, lds);
        part = v[0];
    }
    if (threadIdx.x == 0)
        partials[static_cast<size_t>(n) * groups_max + blockIdx.x] = part;
}

// Combines the partials of every sample in index order.
template <typename T, bool IS_MAX>
__global__ __launch_bounds__(kBlockSize) void softmax_inst_finish_kernel(
    const double* __restrict__ partials, int groups, int groups_max, T* __restrict__ out)
{
    __shared__ double lds[kWavesPerBlock];
    const int n = blockIdx.x;
    const double* mine = partials + static_cast<size_t>(n) * groups_max;
    if constexpr (IS_MAX)
    {
        double m = static_cast<double>(Limits<T>::min_normal);
        for (int g = threadIdx.x; g < groups; g += kBlockSize)
            m = mine[g] > m ? mine[g] : m;
        m = wave_max(m);
        if ((threadIdx.x & (kWaveSize - 1)) == 0)
            lds[threadIdx.x / kWaveSize] = m;
        __syncthreads();
        if (threadIdx.x == 0)
        {
            double r = lds[0];
            for (int w = 1; w < kWavesPerBlock; ++w)
                r = lds[w] > r ? lds[w] : r;
            out[n] = static_cast<T>(r);
        }
    }
    else
    {
        double t[1] = {0.0};
        for (int g = threadIdx.x; g < groups; g += kBlockSize)
            t[0] += mine[g];
        block_sum<1>(t, lds);
        if (threadIdx.x == 0)
            out[n] = static_cast<T>(t[0]);
    }
}

// kMapNormalize: y = max(y / sum, sqrt(min_normal))  (SoftmaxOp, softmax.cu:424-435);
// kMapGradient:  dx = y > sqrt(min_normal) ? y * (dy - dp) : 0  (bp_compute_func, :483-500);
// kMapFromInput: y = max(exp(x - max) / sum, sqrt(min_normal)): the exponentials are
// made again from x instead of being read back (the same bits: the same function of
// the same arguments), for samples that are whole on this rank.
enum InstMap : int
{
    kMapNormalize = 0,
    kMapGradient = 1,
    kMapFromInput = 2
};

template <typename T, int VEC, int KIND>
__global__ __launch_bounds__(kBlockSize) void softmax_inst_map_kernel(
    const T* y_in, const T* __restrict__ dy, const T* __restrict__ sample_param,
    const T* __restrict__ sample_shift, T* out, size_t sample_size, T min_output)
{
    using P = Pack<T, VEC>;
    const int n = blockIdx.y;
    const size_t i = (static_cast<size_t>(blockIdx.x) * kBlockSize + threadIdx.x) * VEC;
    if (i >= sample_size)
        return;
    const size_t off = static_cast<size_t>(n) * sample_size + i;
    const T p = sample_param[n];
    P v = P::load(y_in + off);
    if constexpr (KIND == kMapGradient)
    {
        const P g = P::load(dy + off);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
            v[j] = v[j] > min_output ? v[j] * (g[j] - p) : T(0);
    }
    else
    {
        T shift = T(0);
        if constexpr (KIND == kMapFromInput)
            shift = sample_shift[n];
#pragma unroll
        for (int j = 0; j < VEC; ++j)
        {
            const T e = KIND == kMapFromInput ? exp_t(v[j] - shift) : v[j];
            const T r = e / p;
            v[j] = r > min_output ? r : min_output;
        }
    }
    P::store(out + off, v);
}

// Samples of at most 8192 elements (the softmax behind a classifier: 10 to
// a few thousand classes): a wave -- beyond 2048 elements a workgroup -- takes a
// sample, holds it in registers (CPL elements a lane) and combines its lanes with
// shuffles (and its waves through LDS), so a reduction is one launch without
// partials, and the whole forward pass of samples that are whole on this rank is
// one launch too (N 4096, 10 elements a sample: 18 us in five launches before).
// Sums are accumulated in fp64, lane by lane and then across the lanes as a
// butterfly; the staged and the fused path add in the same order.
enum InstSmall : int
{
    kSmallMax = 0,     // result[n] = max x
    kSmallExpSum = 1,  // out = exp(x - param[n]); result[n] = sum
    kSmallSumExp = 2,  // result[n] = sum exp(x - param[n])
    kSmallDot = 3,     // result[n] = sum a * b
    kSmallForward = 4  // result[n] = max, result2[n] = sum, out = max(exp(x - max) / sum, min_output)
};

template <typename T, int CPL, int MODE, int LANES>
__global__ __launch_bounds__(kBlockSize) void softmax_inst_small_kernel(
    const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ out,
    const T* __restrict__ sample_param, T* __restrict__ result, T* __restrict__ result2,
    int sample_size, int num_samples, T min_output)
{
    // LANES lanes serve a sample: a wave, or the whole workgroup (whose waves are then
    // combined through LDS in wave order; every thread of the workgroup has the same n)
    __shared__ double lds[kWavesPerBlock];
    const int lane = threadIdx.x % LANES;
    const int n = (blockIdx.x * kBlockSize + threadIdx.x) / LANES;
    if (n >= num_samples)
        return;
    const size_t base = static_cast<size_t>(n) * sample_size;
    T va[CPL], vb[CPL];
#pragma unroll
    for (int k = 0; k < CPL; ++k)
        if (lane + k * LANES < sample_size)
        {
            va[k] = a[base + lane + k * LANES];
            if constexpr (MODE == kSmallDot)
                vb[k] = b[base + lane + k * LANES];
        }
    T shift = T(0);
    if constexpr (MODE == kSmallMax || MODE == kSmallForward)
    {
        T mx = Limits<T>::min_normal; // softmax.cu:88-99: the maximum starts at min_normal
#pragma unroll
        for (int k = 0; k < CPL; ++k)
            if (lane + k * LANES < sample_size)
                mx = va[k] >= mx ? va[k] : mx;
        if constexpr (LANES == kWaveSize)
            mx = wave_max(mx);
        else
            mx = static_cast<T>(block_combine(static_cast<double>(mx), true, lds));
        if (lane == 0)
            result[n] = mx;
        if constexpr (MODE == kSmallMax)
            return;
        shift = mx;
    }
    else if constexpr (MODE != kSmallDot)
    {
        shift = sample_param[n];
    }
    double acc = 0.0;
#pragma unroll
    for (int k = 0; k < CPL; ++k)
        if (lane + k * LANES < sample_size)
        {
            if constexpr (MODE == kSmallDot)
            {
                acc = __builtin_fma(static_cast<double>(va[k]), static_cast<double>(vb[k]), acc);
            }
            else
            {
                va[k] = exp_t(va[k] - shift);
                acc += static_cast<double>(va[k]);
            }
        }
    if constexpr (LANES == kWaveSize)
        acc = wave_butterfly_sum(acc);
    else
        acc = block_combine(acc, false, lds);
    const T total = static_cast<T>(acc);
    if (lane == 0)
        (MODE == kSmallForward ? result2 : result)[n] = total;
    if constexpr (MODE == kSmallExpSum || MODE == kSmallForward)
    {
#pragma unroll
        for (int k = 0; k < CPL; ++k)
            if (lane + k * LANES < sample_size)
            {
                if constexpr (MODE == kSmallForward)
                {
                    const T r = va[k] / total;
                    va[k] = r > min_output ? r : min_output;
                }
                out[base + lane + k * LANES] = va[k];
            }
    }
}

constexpr size_t kInstSmallSample = 32 * kBlockSize;

template <typename T, int MODE>
int inst_small(int n, size_t sample_size, const void* a, const void* b, void* out,
               const void* param, void* result, void* result2, T min_output, hipStream_t st)
{
#define H2X_INST_SMALL(CP, LN)                                                                     \
    do                                                                                             \
    {                                                                                              \
        const unsigned int teams = kBlockSize / LN;                                                \
        softmax_inst_small_kernel<T, CP, MODE, LN>                                                 \
            <<<(static_cast<unsigned int>(n) + teams - 1) / teams, kBlockSize, 0, st>>>(           \
                static_cast<const T*>(a), static_cast<const T*>(b), static_cast<T*>(out),          \
                static_cast<const T*>(param), static_cast<T*>(result), static_cast<T*>(result2),   \
                static_cast<int>(sample_size), n, min_output);                                     \
        return launch_status();                                                                    \
    } while (0)
    if (sample_size <= 1 * kWaveSize) H2X_INST_SMALL(1, kWaveSize);
    if (sample_size <= 2 * kWaveSize) H2X_INST_SMALL(2, kWaveSize);
    if (sample_size <= 4 * kWaveSize) H2X_INST_SMALL(4, kWaveSize);
    if (sample_size <= 8 * kWaveSize) H2X_INST_SMALL(8, kWaveSize);
    if (sample_size <= 16 * kWaveSize) H2X_INST_SMALL(16, kWaveSize);
    if (sample_size <= 32 * kWaveSize) H2X_INST_SMALL(32, kWaveSize);
    if (sample_size <= 16 * kBlockSize) H2X_INST_SMALL(16, kBlockSize);
    H2X_INST_SMALL(32, kBlockSize);
#undef H2X_INST_SMALL
}

template <typename T>
T inst_min_output()
{
    return static_cast<T>(std::sqrt(static_cast<double>(Limits<T>::min_normal))); // softmax.cu:156-160
}

struct InstChunking
{
    size_t chunk;
    int groups;
};

InstChunking inst_chunking(size_t sample_size, int num_samples, int vec)
{
    const int gmax = inst_groups_per_sample_max(num_samples);
    const size_t tile = static_cast<size_t>(kBlockSize) * vec * kInstUnroll;
    size_t chunk = (sample_size + gmax - 1) / gmax;
    chunk = (chunk + tile - 1) / tile * tile;
    InstChunking c;
    c.chunk = chunk;
    c.groups = static_cast<int>((sample_size + chunk - 1) / chunk);
    return c;
}

template <typename T, int MODE>
int inst_reduce(int n, size_t sample_size, const void* a, const void* b, void* out,
                const void* param, void* result, void* workspace, hipStream_t st)
{
    if (sample_size <= kInstSmallSample && n > 0)
    {
        constexpr int kSmallMode = MODE == kInstMax      ? kSmallMax
                                   : MODE == kInstExpSum ? kSmallExpSum
                                   : MODE == kInstSumExp ? kSmallSumExp
                                                         : kSmallDot;
        return inst_small<T, kSmallMode>(n, sample_size, a, b, out, param, result, nullptr, T(0), st);
    }
    constexpr int kFull = 16 / sizeof(T);
    const int v = vector_width<T>(sample_size, kFull, {a, b ? b : a, out ? out : a});
    const InstChunking ch = inst_chunking(sample_size, n, v);
    const int gmax = inst_groups_per_sample_max(n);
    const dim3 grid(ch.groups, n);
    double* partials = static_cast<double*>(workspace);
    if (v == kFull)
        softmax_inst_reduce_kernel<T, kFull, MODE><<<grid, kBlockSize, 0, st>>>(
            static_cast<const T*>(a), static_cast<const T*>(b), static_cast<T*>(out),
            static_cast<const T*>(param), partials, sample_size, ch.chunk, gmax);
    else
        softmax_inst_reduce_kernel<T, 1, MODE><<<grid, kBlockSize, 0, st>>>(
            static_cast<const T*>(a), static_cast<const T*>(b), static_cast<T*>(out),
            static_cast<const T*>(param), partials, sample_size, ch.chunk, gmax);
    softmax_inst_finish_kernel<T, MODE == kInstMax><<<n, kBlockSize, 0, st>>>(
        partials, ch.groups, gmax, static_cast<T*>(result));
    return launch_status();
}

template <typename T, int KIND>
int inst_map(int n, size_t sample_size, const void* y, const void* dy, const void* param,
             const void* shift, void* out, hipStream_t st)
{
    constexpr int kFull = 16 / sizeof(T);
    const int v = vector_width<T>(sample_size, kFull, {y, dy ? dy : y, out});
    const T min_output = inst_min_output<T>();
    if (v == kFull)
        softmax_inst_map_kernel<T, kFull, KIND><<<pixel_grid(sample_size, kFull, n), kBlockSize, 0, st>>>(
            static_cast<const T*>(y), static_cast<const T*>(dy), static_cast<const T*>(param),
            static_cast<const T*>(shift), static_cast<T*>(out), sample_size, min_output);
    else
        softmax_inst_map_kernel<T, 1, KIND><<<pixel_grid(sample_size, 1, n), kBlockSize, 0, st>>>(
            static_cast<const T*>(y), static_cast<const T*>(dy), static_cast<const T*>(param),
            static_cast<const T*>(shift), static_cast<T*>(out), sample_size, min_output);
    return launch_status();
}

// Forward pass of samples that are whole on this rank: maximum, sum of the
// exponentials (y is not written), y from x: 4 tensor passes instead of 5.
template <typename T>
int inst_forward_local(int n, size_t sample_size, const void* x, void* y, void* sample_max,
                       void* sample_exp, void* workspace, hipStream_t st)
{
    if (sample_size <= kInstSmallSample && n > 0)
        return inst_small<T, kSmallForward>(n, sample_size, x, nullptr, y, nullptr, sample_max,
                                            sample_exp, inst_min_output<T>(), st);
    int err = inst_reduce<T, kInstMax>(n, sample_size, x, nullptr, nullptr, nullptr, sample_max,
                                       workspace, st);
    // `y` takes part in the choice of the vector width only, as in the staged call,
    // so that the sum is cut up and added in the same order
    if (!err)
        err = inst_reduce<T, kInstSumExp>(n, sample_size, x, nullptr, y, sample_max, sample_exp,
                                          workspace, st);
    return err ? err : inst_map<T, kMapFromInput>(n, sample_size, x, nullptr, sample_exp, sample_max, y, st);
}

bool inst_bad(int num_samples, size_t sample_size)
{
    return num_samples < 0 || num_samples > 65535
           || (sample_size + kBlockSize - 1) / kBlockSize > 0x7fffffffull;
}

} // namespace
} // namespace h2x

using namespace h2x;

extern "C" int h2x_softmax_channel_forward(h2x_dtype dtype, int num_samples, int num_channels,
                                           size_t spatial_size, const void* x, void* y,
                                           h2x_stream_t stream)
{
    if (num_samples < 0 || num_channels < 0)
        return H2X_ERR_INVALID_ARGUMENT;
    if (num_samples == 0 || num_channels == 0 || spatial_size == 0)
        return H2X_SUCCESS; // empty local tensor: softmax.cu:600-603
    if (!x || !y)
        return H2X_ERR_INVALID_ARGUMENT;
    if (num_samples > 65535 || (spatial_size + kWaveSize - 1) / kWaveSize > 0x7ffffff0ull)
        return H2X_ERR_TOO_LARGE;
    switch (dtype)
    {
    case H2X_F32:
        return forward_impl<float>(num_samples, num_channels, spatial_size, x, y, as_stream(stream));
    case H2X_F64:
        return forward_impl<double>(num_samples, num_channels, spatial_size, x, y, as_stream(stream));
    }
    return H2X_ERR_UNSUPPORTED;
}

extern "C" int h2x_softmax_channel_backward(h2x_dtype dtype, int num_samples, int num_channels,
                                            size_t spatial_size, const void* y, const void* dy,
                                            void* dx, h2x_stream_t stream)
{
    if (num_samples < 0 || num_channels < 0)
        return H2X_ERR_INVALID_ARGUMENT;
    if (num_samples == 0 || num_channels == 0 || spatial_size == 0)
        return H2X_SUCCESS;
    if (!y || !dy || !dx)
        return H2X_ERR_INVALID_ARGUMENT;
    if (num_samples > 65535 || (spatial_size + kWaveSize - 1) / kWaveSize > 0x7ffffff0ull)
        return H2X_ERR_TOO_LARGE;
    switch (dtype)
    {
    case H2X_F32:
        return backward_impl<float>(num_samples, num_channels, spatial_size, y, dy, dx, as_stream(stream));
    case H2X_F64:
        return backward_impl<double>(num_samples, num_channels, spatial_size, y, dy, dx, as_stream(stream));
    }
    return H2X_ERR_UNSUPPORTED;
}

// ---- instance mode -------------------------------------------------------------

extern "C" size_t h2x_softmax_instance_workspace_bytes(int num_samples)
{
    const size_t n = num_samples > 0 ? num_samples : 1;
    return (n * inst_groups_per_sample_max(num_samples) * sizeof(double) + 255) / 256 * 256;
}

#define H2X_INST_ENTRY(CALL_F32, CALL_F64)                                                         \
    if (inst_bad(num_samples, sample_size))                                                        \
        return num_samples < 0 ? H2X_ERR_INVALID_ARGUMENT : H2X_ERR_TOO_LARGE;                     \
    if (num_samples == 0 || sample_size == 0)                                                      \
        return H2X_SUCCESS;                                                                        \
    switch (dtype)                                                                                 \
    {                                                                                              \
    case H2X_F32: return CALL_F32;                                                                 \
    case H2X_F64: return CALL_F64;                                                                 \
    }                                                                                              \
    return H2X_ERR_UNSUPPORTED

extern "C" int h2x_softmax_instance_max(h2x_dtype dtype, int num_samples, size_t sample_size,
                                        const void* x, void* sample_max, void* workspace,
                                        h2x_stream_t stream)
{
    if (!x || !sample_max || !workspace)
        return num_samples == 0 || sample_size == 0 ? H2X_SUCCESS : H2X_ERR_INVALID_ARGUMENT;
    H2X_INST_ENTRY((inst_reduce<float, kInstMax>(num_samples, sample_size, x, nullptr, nullptr, nullptr,
                                                 sample_max, workspace, as_stream(stream))),
                   (inst_reduce<double, kInstMax>(num_samples, sample_size, x, nullptr, nullptr,
                                                  nullptr, sample_max, workspace, as_stream(stream))));
}

extern "C" int h2x_softmax_instance_exp(h2x_dtype dtype, int num_samples, size_t sample_size,
                                        const void* x, const void* sample_max, void* y,
                                        void* sample_exp, void* workspace, h2x_stream_t stream)
{
    if (!x || !sample_max || !y || !sample_exp || !workspace)
        return num_samples == 0 || sample_size == 0 ? H2X_SUCCESS : H2X_ERR_INVALID_ARGUMENT;
    H2X_INST_ENTRY((inst_reduce<float, kInstExpSum>(num_samples, sample_size, x, nullptr, y, sample_max,
                                                    sample_exp, workspace, as_stream(stream))),
                   (inst_reduce<double, kInstExpSum>(num_samples, sample_size, x, nullptr, y,
                                                     sample_max, sample_exp, workspace,
                                                     as_stream(stream))));
}

extern "C" int h2x_softmax_instance_normalize(h2x_dtype dtype, int num_samples, size_t sample_size,
                                              const void* sample_exp, void* y, h2x_stream_t stream)
{
    if (!sample_exp || !y)
        return num_samples == 0 || sample_size == 0 ? H2X_SUCCESS : H2X_ERR_INVALID_ARGUMENT;
    H2X_INST_ENTRY((inst_map<float, kMapNormalize>(num_samples, sample_size, y, nullptr, sample_exp,
                                                   nullptr, y, as_stream(stream))),
                   (inst_map<double, kMapNormalize>(num_samples, sample_size, y, nullptr, sample_exp,
                                                    nullptr, y, as_stream(stream))));
}

extern "C" int h2x_softmax_instance_dot(h2x_dtype dtype, int num_samples, size_t sample_size,
                                        const void* y, const void* dy, void* sample_dp,
                                        void* workspace, h2x_stream_t stream)
{
    if (!y || !dy || !sample_dp || !workspace)
        return num_samples == 0 || sample_size == 0 ? H2X_SUCCESS : H2X_ERR_INVALID_ARGUMENT;
    H2X_INST_ENTRY((inst_reduce<float, kInstDot>(num_samples, sample_size, y, dy, nullptr, nullptr,
                                                 sample_dp, workspace, as_stream(stream))),
                   (inst_reduce<double, kInstDot>(num_samples, sample_size, y, dy, nullptr, nullptr,
                                                  sample_dp, workspace, as_stream(stream))));
}

extern "C" int h2x_softmax_instance_gradient(h2x_dtype dtype, int num_samples, size_t sample_size,
                                             const void* y, const void* dy, const void* sample_dp,
                                             void* dx, h2x_stream_t stream)
{
    if (!y || !dy || !sample_dp || !dx)
        return num_samples == 0 || sample_size == 0 ? H2X_SUCCESS : H2X_ERR_INVALID_ARGUMENT;
    H2X_INST_ENTRY((inst_map<float, kMapGradient>(num_samples, sample_size, y, dy, sample_dp, nullptr,
                                                  dx, as_stream(stream))),
                   (inst_map<double, kMapGradient>(num_samples, sample_size, y, dy, sample_dp, nullptr,
                                                   dx, as_stream(stream))));
}

extern "C" int h2x_softmax_instance_forward_local(h2x_dtype dtype, int num_samples,
                                                  size_t sample_size, const void* x, void* y,
                                                  void* sample_max, void* sample_exp,
                                                  void* workspace, h2x_stream_t stream)
{
    if (!x || !y || !sample_max || !sample_exp || !workspace)
        return num_samples == 0 || sample_size == 0 ? H2X_SUCCESS : H2X_ERR_INVALID_ARGUMENT;
    H2X_INST_ENTRY((inst_forward_local<float>(num_samples, sample_size, x, y, sample_max, sample_exp,
                                              workspace, as_stream(stream))),
                   (inst_forward_local<double>(num_samples, sample_size, x, y, sample_max, sample_exp,
                                               workspace, as_stream(stream))));
}

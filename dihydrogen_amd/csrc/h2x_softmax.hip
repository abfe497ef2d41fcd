// Channel softmax (forward, backward) for gfx950 and the C entry points.
//
// Tensors are dense [N][C][S]; the softmax runs over C, so the C values of one
// pixel are S elements apart while neighbouring pixels are contiguous.  A
// thread owns VEC neighbouring pixels and keeps all C values of them in
// registers (the channel loop is unrolled to a compile-time bound CMAX >= C),
// so x (or y and dy) is read from HBM exactly once with fully coalesced
// 4*VEC-byte accesses and no LDS staging; the reference stages a
// C x 256 tile in LDS and walks it three times
// (legacy/src/dnn_backend/softmax.cu:538-593,621-669).  Channel counts beyond
// the largest register tile fall back to a kernel that re-reads its inputs.
#include "h2x_device.hpp"

#include <cfloat>

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

// forward, register-resident.  Replaces fp_channel_kernel, softmax.cu:538-593:
// running maximum starts at min_normal (positive), the sum is taken in channel
// order, y = max(e * (1 / sum), min_normal).
template <typename T, int VEC, int CMAX>
__global__ __launch_bounds__(kBlockSize) void softmax_fwd_reg_kernel(
    const T* __restrict__ x, T* __restrict__ y, int num_channels, size_t spatial)
{
    using P = Pack<T, VEC>;
    const size_t s = (static_cast<size_t>(blockIdx.x) * kBlockSize + threadIdx.x) * VEC;
    if (s >= spatial)
        return;
    const size_t base = static_cast<size_t>(blockIdx.y) * num_channels * spatial + s;
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

// forward, any channel count: three passes over global memory per pixel.
template <typename T>
__global__ __launch_bounds__(kBlockSize) void softmax_fwd_stream_kernel(
    const T* __restrict__ x, T* __restrict__ y, int num_channels, size_t spatial)
{
    const size_t s = static_cast<size_t>(blockIdx.x) * kBlockSize + threadIdx.x;
    if (s >= spatial)
        return;
    const size_t base = static_cast<size_t>(blockIdx.y) * num_channels * spatial + s;
    const T* xp = x + base;
    T* yp = y + base;
    constexpr T kMin = Limits<T>::min_normal;
    T mx = kMin;
    for (int c = 0; c < num_channels; ++c)
    {
        const T v = xp[static_cast<size_t>(c) * spatial];
        mx = v > mx ? v : mx;
    }
    T sum = T(0);
    for (int c = 0; c < num_channels; ++c)
    {
        const T e = exp_t(xp[static_cast<size_t>(c) * spatial] - mx);
        yp[static_cast<size_t>(c) * spatial] = e;
        sum += e;
    }
    sum = T(1) / sum;
    for (int c = 0; c < num_channels; ++c)
    {
        const T r = yp[static_cast<size_t>(c) * spatial] * sum;
        yp[static_cast<size_t>(c) * spatial] = r > kMin ? r : kMin;
    }
}

// backward, register-resident.  Replaces bp_channel_kernel, softmax.cu:621-669:
// dp accumulates y*dy in channel order with fused multiply-adds.
template <typename T, int VEC, int CMAX>
__global__ __launch_bounds__(kBlockSize) void softmax_bwd_reg_kernel(
    const T* __restrict__ y, const T* __restrict__ dy, T* __restrict__ dx, int num_channels,
    size_t spatial)
{
    using P = Pack<T, VEC>;
    const size_t s = (static_cast<size_t>(blockIdx.x) * kBlockSize + threadIdx.x) * VEC;
    if (s >= spatial)
        return;
    const size_t base = static_cast<size_t>(blockIdx.y) * num_channels * spatial + s;
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

template <typename T>
__global__ __launch_bounds__(kBlockSize) void softmax_bwd_stream_kernel(
    const T* __restrict__ y, const T* __restrict__ dy, T* __restrict__ dx, int num_channels,
    size_t spatial)
{
    const size_t s = static_cast<size_t>(blockIdx.x) * kBlockSize + threadIdx.x;
    if (s >= spatial)
        return;
    const size_t base = static_cast<size_t>(blockIdx.y) * num_channels * spatial + s;
    const T* yp = y + base;
    const T* gp = dy + base;
    T* op = dx + base;
    constexpr T kMin = Limits<T>::min_normal;
    T dp = T(0);
    for (int c = 0; c < num_channels; ++c)
        dp = fma_t(yp[static_cast<size_t>(c) * spatial], gp[static_cast<size_t>(c) * spatial], dp);
    for (int c = 0; c < num_channels; ++c)
    {
        const T yi = yp[static_cast<size_t>(c) * spatial];
        op[static_cast<size_t>(c) * spatial] =
            yi > kMin ? yi * (gp[static_cast<size_t>(c) * spatial] - dp) : T(0);
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

template <typename T, int VEC, int CMAX>
void launch_fwd(const T* x, T* y, int n, int c, size_t s, hipStream_t st)
{
    softmax_fwd_reg_kernel<T, VEC, CMAX><<<pixel_grid(s, VEC, n), kBlockSize, 0, st>>>(x, y, c, s);
}

template <typename T, int VEC, int CMAX>
void launch_bwd(const T* y, const T* dy, T* dx, int n, int c, size_t s, hipStream_t st)
{
    softmax_bwd_reg_kernel<T, VEC, CMAX><<<pixel_grid(s, VEC, n), kBlockSize, 0, st>>>(y, dy, dx, c, s);
}

// Register budget: CMAX * VEC * sizeof(T)/4 VGPRs for the forward tile, twice
// that backward; tiles are kept at or below 128 VGPRs.
template <typename T>
int forward_impl(int n, int c, size_t s, const void* xv, void* yv, hipStream_t st)
{
    const T* x = static_cast<const T*>(xv);
    T* y = static_cast<T*>(yv);
    constexpr int kWords = sizeof(T) / 4;
    const int v4 = vector_width<T>(s, 4 / kWords, {xv, yv});
#define H2X_FWD(V, CM)                                                                             \
    do                                                                                             \
    {                                                                                              \
        launch_fwd<T, V, CM>(x, y, n, c, s, st);                                                   \
        return launch_status();                                                                    \
    } while (0)
    if constexpr (sizeof(T) == 4)
    {
        if (v4 == 4)
        {
            if (c <= 8) H2X_FWD(4, 8);
            if (c <= 16) H2X_FWD(4, 16);
            if (c <= 32) H2X_FWD(4, 32);
        }
        if (v4 >= 2)
        {
            if (c <= 8) H2X_FWD(2, 8);
            if (c <= 16) H2X_FWD(2, 16);
            if (c <= 32) H2X_FWD(2, 32);
            if (c <= 64) H2X_FWD(2, 64);
        }
        if (c <= 8) H2X_FWD(1, 8);
        if (c <= 16) H2X_FWD(1, 16);
        if (c <= 32) H2X_FWD(1, 32);
        if (c <= 64) H2X_FWD(1, 64);
        if (c <= 128) H2X_FWD(1, 128);
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
        if (c <= 64) H2X_FWD(1, 64);
    }
#undef H2X_FWD
    softmax_fwd_stream_kernel<T><<<pixel_grid(s, 1, n), kBlockSize, 0, st>>>(x, y, c, s);
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
    const int v4 = vector_width<T>(s, 4 / kWords, {yv, dyv, dxv});
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
        }
        if (c <= 8) H2X_BWD(1, 8);
        if (c <= 16) H2X_BWD(1, 16);
        if (c <= 32) H2X_BWD(1, 32);
        if (c <= 64) H2X_BWD(1, 64);
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
    }
#undef H2X_BWD
    softmax_bwd_stream_kernel<T><<<pixel_grid(s, 1, n), kBlockSize, 0, st>>>(y, dy, dx, c, s);
    return launch_status();
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
    if (num_samples > 65535 || (spatial_size + kBlockSize - 1) / kBlockSize > 0x7fffffffull)
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
    if (num_samples > 65535 || (spatial_size + kBlockSize - 1) / kBlockSize > 0x7fffffffull)
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

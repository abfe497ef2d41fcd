// Device-side helpers shared by the gfx950 kernels: wave64 reductions built on
// DPP lane permutes, a fixed-order block reduction through LDS, unaligned
// 16-byte vector types, and the host-side status plumbing.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "h2x.h"

namespace h2x
{

constexpr int kWaveSize = 64;
constexpr int kBlockSize = 256;
constexpr int kWavesPerBlock = kBlockSize / kWaveSize;

inline hipStream_t as_stream(h2x_stream_t s)
{
    return reinterpret_cast<hipStream_t>(s);
}

// Status of the launch that was just issued.
inline int launch_status()
{
    return static_cast<int>(hipGetLastError());
}

inline bool aligned16(const void* p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

// ---- division by a launch-time constant ------------------------------------
// n / d for n < 2^31 by multiply-high and shift.
struct FastDiv
{
    uint32_t divisor;
    uint32_t multiplier;
    uint32_t shift;
};

inline FastDiv make_fastdiv(uint32_t d)
{
    FastDiv f{d, 0u, 0u};
    if (d > 1)
    {
        const uint32_t log2 = 32u - static_cast<uint32_t>(__builtin_clz(d - 1)); // ceil(log2 d), d >= 2
        const uint32_t p = 31 + log2;
        f.multiplier = static_cast<uint32_t>(((1ull << p) + d - 1) / d);
        f.shift = p - 32;
    }
    return f;
}

__host__ __device__ inline uint32_t fastdiv(uint32_t n, const FastDiv& f)
{
#ifdef __HIP_DEVICE_COMPILE__
    return f.divisor == 1 ? n : __umulhi(n, f.multiplier) >> f.shift;
#else
    return f.divisor == 1
               ? n
               : static_cast<uint32_t>((static_cast<uint64_t>(n) * f.multiplier) >> 32) >> f.shift;
#endif
}

#ifdef __HIPCC__

// ---- lane permutes --------------------------------------------------------
// DPP controls: quad_perm [1,0,3,2] and [2,3,0,1] swap lanes at distance 1 and
// 2 inside a quad; row_ror:n rotates a 16-lane row.
constexpr int kDppQuadSwap1 = 0xB1;
constexpr int kDppQuadSwap2 = 0x4E;
constexpr int kDppRowRor4 = 0x124;
constexpr int kDppRowRor8 = 0x128;

template <int Ctrl>
__device__ __forceinline__ double dpp_move(double v)
{
    const long long bits = __double_as_longlong(v);
    int lo = static_cast<int>(bits & 0xffffffffll);
    int hi = static_cast<int>(bits >> 32);
    lo = __builtin_amdgcn_update_dpp(0, lo, Ctrl, 0xf, 0xf, false);
    hi = __builtin_amdgcn_update_dpp(0, hi, Ctrl, 0xf, 0xf, false);
    return __longlong_as_double((static_cast<long long>(hi) << 32)
                                | static_cast<unsigned int>(lo));
}

// Sum over the 64 lanes of a wave; every lane returns the total.  The
// combination order is fixed (distance 1, 2, 4, 8 inside a row, then rows 16
// and 32 apart), so the result does not depend on scheduling.
__device__ __forceinline__ double wave_sum(double v)
{
    v += dpp_move<kDppQuadSwap1>(v);
    v += dpp_move<kDppQuadSwap2>(v);
    v += dpp_move<kDppRowRor4>(v);
    v += dpp_move<kDppRowRor8>(v);
    v += __shfl_xor(v, 16, kWaveSize);
    v += __shfl_xor(v, 32, kWaveSize);
    return v;
}

// Sum of K values per thread over a 256-thread workgroup.  `lds` must hold
// K * kWavesPerBlock doubles.  Every thread returns the totals in v[].
template <int K>
__device__ __forceinline__ void block_sum(double (&v)[K], double* lds)
{
    const int lane = threadIdx.x & (kWaveSize - 1);
    const int wave = threadIdx.x / kWaveSize;
#pragma unroll
    for (int k = 0; k < K; ++k)
        v[k] = wave_sum(v[k]);
    __syncthreads(); // lds may still be read by a previous use
    if (lane == 0)
    {
#pragma unroll
        for (int k = 0; k < K; ++k)
            lds[k * kWavesPerBlock + wave] = v[k];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < K; ++k)
    {
        double t = lds[k * kWavesPerBlock];
#pragma unroll
        for (int w = 1; w < kWavesPerBlock; ++w)
            t += lds[k * kWavesPerBlock + w];
        v[k] = t;
    }
}

// ---- workgroup order ---------------------------------------------------------
// Workgroups go to the eight XCDs round-robin (workgroup i runs on XCD i mod
// 8) and every XCD has its own L2 with its own address-interleaved channels.
// When consecutive workgroups walk through memory in equal steps, the
// workgroups of one XCD visit addresses 8 steps apart and can end up on a
// fraction of its L2 channels; with power-of-two strides between the streams
// of one workgroup this costs a quarter of the bandwidth (channel softmax,
// N 32, C 19, 1024 x 2048: 3.9 TB/s -> 5.4 TB/s).  xcd_contiguous gives each
// XCD one contiguous eighth of the tiles instead.  `padded_grid` is the grid
// size, a multiple of 8; the result may exceed the number of tiles needed.
constexpr unsigned int kNumXcd = 8;

__device__ __forceinline__ unsigned int xcd_contiguous(unsigned int block, unsigned int padded_grid)
{
    return (block % kNumXcd) * (padded_grid / kNumXcd) + block / kNumXcd;
}

// ---- vectors --------------------------------------------------------------
// 16-byte vectors that may sit on any element boundary.
template <typename T, int N>
struct alignas(sizeof(T)) UVec
{
    T v[N];
};

template <typename T, int N>
struct alignas(sizeof(T) * N) AVec
{
    T v[N];
};

#endif // __HIPCC__

} // namespace h2x

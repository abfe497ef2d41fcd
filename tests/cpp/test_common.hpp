// Helpers shared by the C++ tests of the host-side layer.
#pragma once

#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "distconv/distconv_mi355x.hpp"

using namespace distconv;
using namespace distconv::tensor;

template <typename T>
using DevTensor = Tensor<T, LocaleVirtual, CUDAAllocator>;

#define CHECK(cond)                                                                                \
    do                                                                                             \
    {                                                                                              \
        if (!(cond))                                                                               \
        {                                                                                          \
            std::printf("FAILED %s at %s:%d\n", #cond, __FILE__, __LINE__);                        \
            std::exit(1);                                                                          \
        }                                                                                          \
    } while (0)

template <typename T>
std::vector<T> to_host(DevTensor<T>& t)
{
    std::vector<T> h(t.get_local_real_size());
    DISTCONV_CHECK_HIP(hipDeviceSynchronize());
    DISTCONV_CHECK_HIP(hipMemcpy(h.data(), t.get_buffer(), h.size() * sizeof(T), hipMemcpyDeviceToHost));
    return h;
}

template <typename T>
void to_device(DevTensor<T>& t, const std::vector<T>& h)
{
    CHECK(h.size() == t.get_local_real_size());
    DISTCONV_CHECK_HIP(hipMemcpy(t.get_buffer(), h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
}

// Interior of a rank initialised to the global linear offset of each element,
// everything else to `fill` (legacy/tests/tensor/test_halo_exchange_cuda.cu:43-102).
template <typename T>
std::vector<T> global_offset_field(const DevTensor<T>& t, T fill)
{
    const int nd = t.get_num_dims();
    std::vector<T> h(t.get_local_real_size(), fill);
    const Shape& ls = t.get_local_shape();
    for (index_t o = 0; o < t.get_local_size(); ++o)
    {
        IndexVector idx = ls.get_index(o);
        IndexVector g(nd, 0);
        for (int i = 0; i < nd; ++i)
            g[i] = idx[i] + t.get_global_index()[i];
        h[t.get_local_offset(idx)] = static_cast<T>(get_offset(g, t.get_shape()));
    }
    return h;
}

// Ends a test program the way an application does: the per-stream workspaces of the layer are
// handed back, the device is idle, and main returns, so that the exit handlers and static
// destructors of the program, of libh2x.so and of the HIP runtime run.  Tensors, layers and plans
// of main's own scope are destroyed by that return, before any exit handler.
inline int finish(int errors)
{
    release_workspaces();
    CHECK(h2x_host::StreamScratch::held_buffers() == 0);
    DISTCONV_CHECK_HIP(hipDeviceSynchronize());
    return errors ? 1 : 0;
}

// tensor::Transform, tensor::ReduceSum and tensor::TransformReduceSum of the
// reference (legacy/include/distconv/tensor/algorithms/transform_cuda.hpp:359-693,
// reduce_sum_cuda.hpp:388-439, transform_reduce_sum_cuda.hpp:17-87) over
// libh2x.so.
//
// The reference instantiates a kernel for whatever functor it is given.  The
// functors this path needs live in the library and are named here by functor
// types (ScaleFunctor, CopyFunctor, ScaleBiasFunctor, SumsToStatisticsFunctor);
// Transform with one of them goes through the C interface and works from any
// host compiler.  Any other functor -- a __device__ lambda, as in the
// reference's tests -- is compiled into a kernel by this header, which needs
// hipcc, exactly as the reference's header needs the device compiler.
#pragma once

#include <algorithm>
#include <map>
#include <tuple>
#include <type_traits>
#include <utility>

#ifdef __HIPCC__
#include <hip/hip_runtime.h>
#endif

#include "distconv/tensor_mi355x.hpp"

namespace distconv
{
namespace tensor
{

namespace internal
{

// x = x * v (legacy/src/tensor/tensor_mpi_cuda.cu:86-98)
template <typename T>
struct ScaleFunctor
{
    static constexpr h2x_transform_op h2x_op = H2X_TRANSFORM_SCALE;
    static constexpr int num_tensors = 1;
    T v;
    explicit ScaleFunctor(T value) : v(value) {}
    void params(double* p) const { p[0] = static_cast<double>(v); }
};

// y = x
template <typename T>
struct CopyFunctor
{
    static constexpr h2x_transform_op h2x_op = H2X_TRANSFORM_COPY;
    static constexpr int num_tensors = 2;
    void params(double*) const {}
};

// y = alpha * x + beta: CastScaleBiasFuctor with equal types (tensor_mpi_cuda.cu:113-135)
template <typename T>
struct ScaleBiasFunctor
{
    static constexpr h2x_transform_op h2x_op = H2X_TRANSFORM_SCALE_BIAS;
    static constexpr int num_tensors = 2;
    T alpha, beta;
    ScaleBiasFunctor(T a, T b) : alpha(a), beta(b) {}
    void params(double* p) const
    {
        p[0] = static_cast<double>(alpha);
        p[1] = static_cast<double>(beta);
    }
};

// sums -> mean, sqsums -> unbiased variance, running statistics updated:
// sums_to_statistics_functor, legacy/src/dnn_backend/batchnorm.cu:288-315
template <typename T>
struct SumsToStatisticsFunctor
{
    static constexpr h2x_transform_op h2x_op = H2X_TRANSFORM_SUMS_TO_STATISTICS;
    static constexpr int num_tensors = 4;
    index_t num_per_sum;
    T decay;
    SumsToStatisticsFunctor(index_t n, T d) : num_per_sum(n), decay(d) {}
    void params(double* p) const
    {
        p[0] = static_cast<double>(num_per_sum);
        p[1] = static_cast<double>(decay);
    }
};

template <typename F, typename = void>
struct is_library_functor : std::false_type
{
};
template <typename F>
struct is_library_functor<F, decltype((void) F::h2x_op)> : std::true_type
{
};

// local shape and strides of a tensor as the C interface takes them
template <typename Tensor>
h2x_tensor_geometry local_geometry(const Tensor& t, const Shape* region = nullptr)
{
    h2x_tensor_geometry g = {};
    g.num_dims = t.get_num_dims();
    assert_always(g.num_dims <= H2X_MAX_DIMS);
    const Shape strides = t.get_strides();
    for (int i = 0; i < g.num_dims; ++i)
    {
        g.local_shape[i] = static_cast<int64_t>(region ? (*region)[i] : t.get_local_shape()[i]);
        g.strides[i] = static_cast<int64_t>(strides[i]);
    }
    return g;
}

// Device scratch shared by the calls of one stream, grown on demand (calls on
// one stream are ordered, so they can share it).  Kept until
// distconv::release_workspaces(); nothing is freed at static destruction.
inline void* stream_scratch(hipStream_t stream, size_t bytes)
{
    hipError_t err = hipSuccess;
    void* p = h2x_host::StreamScratch::get(stream, h2x_host::StreamScratch::REDUCE_PARTIALS, bytes,
                                           &err);
    DISTCONV_CHECK_HIP(err);
    return p;
}

template <typename Tensor, typename Functor>
int transform_library(Tensor* const* tensors, int n, const Functor& op, hipStream_t stream)
{
    static_assert(std::is_same<typename Tensor::data_type, float>::value
                      || std::is_same<typename Tensor::data_type, double>::value,
                  "the library's functors compute in float or double");
    assert_always(n == Functor::num_tensors);
    h2x_tensor_geometry g[4];
    const h2x_tensor_geometry* gp[4];
    void* ptr[4];
    for (int i = 0; i < n; ++i)
    {
        // the tensors must have the same local shape (transform_cuda.hpp:383-390)
        assert_always(tensors[i]->get_local_shape() == tensors[0]->get_local_shape());
        g[i] = local_geometry(*tensors[i]);
        gp[i] = &g[i];
        ptr[i] = tensors[i]->get_base_ptr();
    }
    if (tensors[0]->get_local_size() == 0)
        return 0;
    double params[4] = {0, 0, 0, 0};
    op.params(params);
    DISTCONV_CHECK_H2X(h2x_tensor_transform(Functor::h2x_op, Tensor::h2x_type(), n, gp, ptr, params, stream));
    return 0;
}

#ifdef __HIPCC__
// Any other functor: one thread per interior element, innermost dimension
// fastest.  (A kernel per functor, as transform_cuda.hpp:34-357 has.)
template <int N>
struct FunctorArgs
{
    char* base[N];
    int64_t stride[N][H2X_MAX_DIMS];
    int64_t extent[H2X_MAX_DIMS];
    int64_t count;
    int num_dims;
};

template <typename Op, int N, typename... Ts, std::size_t... Is>
__device__ __forceinline__ void apply_functor(Op& op, const FunctorArgs<N>& a, const int64_t (&off)[N],
                                              std::index_sequence<Is...>)
{
    op(*(reinterpret_cast<Ts*>(a.base[Is]) + off[Is])...);
}

template <typename Op, typename... Ts>
__global__ void transform_functor_kernel(const FunctorArgs<static_cast<int>(sizeof...(Ts))> a, Op op)
{
    constexpr int N = static_cast<int>(sizeof...(Ts));
    for (int64_t i = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; i < a.count;
         i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    {
        int64_t rem = i, off[N] = {};
        for (int d = 0; d < a.num_dims; ++d)
        {
            const int64_t idx = rem % a.extent[d];
            rem /= a.extent[d];
            for (int t = 0; t < N; ++t)
                off[t] += idx * a.stride[t][d];
        }
        // op(*p0, *p1, ...) with each pointer cast to its tensor's element type
        apply_functor<Op, N, Ts...>(op, a, off, std::index_sequence_for<Ts...>{});
    }
}
#endif

template <typename Functor, typename... Tensors>
int transform_any(Functor op, hipStream_t stream, Tensors&... tensors)
{
    constexpr int N = static_cast<int>(sizeof...(Tensors));
    static_assert(N >= 1 && N <= 4, "Transform takes one to four tensors");
    if constexpr (is_library_functor<Functor>::value)
    {
        using First = typename std::tuple_element<0, std::tuple<Tensors...>>::type;
        First* list[] = {&tensors...};
        return transform_library(list, N, op, stream);
    }
    else
    {
#ifdef __HIPCC__
        FunctorArgs<N> a = {};
        const h2x_tensor_geometry g[] = {local_geometry(tensors)...};
        char* base[] = {reinterpret_cast<char*>(tensors.get_base_ptr())...};
        a.num_dims = g[0].num_dims;
        a.count = 1;
        for (int d = 0; d < a.num_dims; ++d)
        {
            a.extent[d] = g[0].local_shape[d];
            a.count *= a.extent[d];
            for (int t = 0; t < N; ++t)
            {
                assert_always(g[t].local_shape[d] == g[0].local_shape[d]);
                a.stride[t][d] = g[t].strides[d];
            }
        }
        for (int t = 0; t < N; ++t)
            a.base[t] = base[t];
        if (a.count == 0)
            return 0;
        const int64_t blocks = std::min<int64_t>((a.count + 255) / 256, 65536);
        transform_functor_kernel<Functor, typename Tensors::data_type...>
            <<<static_cast<unsigned int>(blocks), 256, 0, stream>>>(a, op);
        DISTCONV_CHECK_HIP(hipGetLastError());
        return 0;
#else
        static_assert(is_library_functor<Functor>::value,
                      "Transform with a functor of your own needs the device compiler (hipcc); the "
                      "library's functors (ScaleFunctor, CopyFunctor, ...) work from any compiler");
        return -1;
#endif
    }
}

} // namespace internal

// transform_cuda.hpp:359-693: op is applied to corresponding interior elements
// of the tensors, which it may modify in place.
template <typename Tensor, typename Functor>
int Transform(Tensor& t1, Functor op, hipStream_t stream = nullptr)
{
    return internal::transform_any(op, stream, t1);
}
template <typename Tensor1, typename Tensor2, typename Functor>
int Transform(Tensor1& t1, Tensor2& t2, Functor op, hipStream_t stream = nullptr)
{
    return internal::transform_any(op, stream, t1, t2);
}
template <typename Tensor1, typename Tensor2, typename Tensor3, typename Functor>
int Transform(Tensor1& t1, Tensor2& t2, Tensor3& t3, Functor op, hipStream_t stream = nullptr)
{
    return internal::transform_any(op, stream, t1, t2, t3);
}
template <typename Tensor1, typename Tensor2, typename Tensor3, typename Tensor4, typename Functor>
int Transform(Tensor1& t1, Tensor2& t2, Tensor3& t3, Tensor4& t4, Functor op,
              hipStream_t stream = nullptr)
{
    return internal::transform_any(op, stream, t1, t2, t3, t4);
}

// What TransformReduceSum may apply to an element before it is added.
struct IdentityOp
{
    static constexpr int square = 0;
};
struct SquareOp
{
    static constexpr int square = 1;
};

namespace internal
{

// reduction_sanity_check, reduce_sum_cuda.hpp:353-371
template <typename Tensor>
void reduction_sanity_check(const Tensor& src, const Tensor& dst)
{
    const auto& sd = src.get_distribution();
    const auto& dd = dst.get_distribution();
    for (int i = 0; i < src.get_num_dims(); ++i)
    {
        assert_always(sd.get_locale_shape()[i] == dd.get_locale_shape()[i]);
        if (src.get_shape()[i] == dst.get_shape()[i])
        {
            assert_always(sd.get_split_shape()[i] == dd.get_split_shape()[i]);
        }
        else
        {
            assert_always(dst.get_shape()[i] == 1);
            assert_always(dd.get_split_shape()[i] == 1);
        }
    }
}

template <typename Tensor>
int reduce_sum(Tensor& src, const Shape& region, Tensor& dst, int square, hipStream_t stream)
{
    reduction_sanity_check(src, dst);
    if (region.get_size() == 0)
        return 0;
    const h2x_tensor_geometry gs = local_geometry(src, &region), gd = local_geometry(dst);
    void* ws = stream_scratch(stream, h2x_tensor_reduce_sum_workspace_bytes(&gs, &gd));
    DISTCONV_CHECK_H2X(h2x_tensor_reduce_sum(Tensor::h2x_type(), &gs, src.get_const_base_ptr(), &gd,
                                             dst.get_base_ptr(), square, ws, stream));
    // The reference ends with dst.allreduce over the reduced dimensions
    // (reduce_sum_cuda.hpp:186-192); virtual ranks combine their destinations
    // themselves.
    return 0;
}

} // namespace internal

// reduce_sum_cuda.hpp:388-439.  dst's extent is 1 along every reduced dimension;
// dst is accumulated into, so the caller clears it first.  ND is 3 or 4 in the
// reference; any rank up to H2X_MAX_DIMS here.
template <int ND, typename Tensor>
int ReduceSum(Tensor& src, Tensor& dst, hipStream_t stream = nullptr)
{
    return internal::reduce_sum(src, src.get_local_shape(), dst, 0, stream);
}
template <int ND, typename Tensor>
int ReduceSum(Tensor& src, const Shape& local_reduction_region, Tensor& dst, hipStream_t stream = nullptr)
{
    return internal::reduce_sum(src, local_reduction_region, dst, 0, stream);
}
template <int ND, typename Tensor>
int ReduceSum(Tensor& src, Tensor& dst1, Tensor& dst2, hipStream_t stream = nullptr)
{
    internal::reduce_sum(src, src.get_local_shape(), dst1, 0, stream);
    return internal::reduce_sum(src, src.get_local_shape(), dst2, 0, stream);
}

// transform_reduce_sum_cuda.hpp:17-87 with the two unary operations this path
// has a use for: the element itself and its square (sum and sum of squares).
template <int ND, typename Tensor, typename Op1>
int TransformReduceSum(Tensor& src, const Shape& local_reduction_region, Tensor& dst, const Op1&,
                       hipStream_t stream = nullptr)
{
    return internal::reduce_sum(src, local_reduction_region, dst, Op1::square, stream);
}
template <int ND, typename Tensor, typename Op1, typename Op2>
int TransformReduceSum(Tensor& src, const Shape& local_reduction_region, Tensor& dst1, const Op1&,
                       Tensor& dst2, const Op2&, hipStream_t stream = nullptr)
{
    internal::reduce_sum(src, local_reduction_region, dst1, Op1::square, stream);
    return internal::reduce_sum(src, local_reduction_region, dst2, Op2::square, stream);
}

} // namespace tensor
} // namespace distconv

// The remaining operators of the path as h2 operators: elementwise transforms
// and sums over dimensions, clear_halo, the tensor-to-tensor halo transfer,
// the shuffler's pack / unpack and instance-mode softmax.  Included by
// h2/ops_mi355x.hpp, whose layering it follows:
//   impl::<op>_impl(CPUDev_t | GPUDev_t, Tensor<T>...)   device implementations,
//   <op>(Tensor<T>...)                                    typed front: H2_DEVICE_DISPATCH on the
//                                                         tensor's device (include/h2/core/device.hpp:92-157),
//   <op>(BaseTensor...)                                   type-erased front through the registry.
// The GPU implementations call libh2x.  The CPU implementations are plain
// loops in this header, for tensors that live in host memory -- the data
// movement operators and the transforms and sums, which is also where h2's own
// CPU operators stop (copy, cast, zero, fill: src/tensor/copy.cpp:117-141,
// src/tensor/init/fill.cpp:38-59); batch-norm, softmax and the shuffler have no
// host implementation and raise for a CPU tensor.
#pragma once

#include <vector>

namespace h2
{

// include/h2/core/device.hpp:92-157
#define H2_DEVICE_DISPATCH(device, cpu_code, gpu_code)                                            \
    do                                                                                            \
    {                                                                                             \
        if ((device) == ::h2::Device::CPU)                                                        \
        {                                                                                         \
            [[maybe_unused]] constexpr ::h2::Device Dev = ::h2::Device::CPU;                      \
            cpu_code;                                                                             \
        }                                                                                         \
        else if ((device) == ::h2::Device::GPU)                                                   \
        {                                                                                         \
            [[maybe_unused]] constexpr ::h2::Device Dev = ::h2::Device::GPU;                      \
            gpu_code;                                                                             \
        }                                                                                         \
        else                                                                                      \
        {                                                                                         \
            throw H2FatalException("Unknown device");                                             \
        }                                                                                         \
    } while (0)

namespace mi355x
{

// shape and strides of any tensor as the C interface takes them
inline h2x_tensor_geometry plain_geometry(const BaseTensor& t, const char* what)
{
    if (t.ndim() < 1 || t.ndim() > H2X_MAX_DIMS)
        throw H2FatalException(what, ": 1 to ", H2X_MAX_DIMS, " dimensions");
    h2x_tensor_geometry g = {};
    g.num_dims = t.ndim();
    for (NDimType i = 0; i < t.ndim(); ++i)
    {
        g.local_shape[i] = t.shape(i);
        g.strides[i] = t.stride(i);
    }
    return g;
}

// Calls f(offsets...) for every element of equally shaped strided tensors,
// innermost dimension fastest (host loops of the CPU implementations).
template <std::size_t N, typename F>
void for_each_element(const ShapeTuple& shape, const StrideTuple (&strides)[N], F f)
{
    const NDimType nd = shape.size();
    std::vector<DimType> idx(nd, 0);
    DataIndexType off[N] = {};
    const DataIndexType total = product<DataIndexType>(shape);
    for (DataIndexType i = 0; i < total; ++i)
    {
        f(off);
        for (NDimType d = 0; d < nd; ++d)
        {
            ++idx[d];
            for (std::size_t t = 0; t < N; ++t)
                off[t] += strides[t][d];
            if (idx[d] < shape[d])
                break;
            for (std::size_t t = 0; t < N; ++t)
                off[t] -= static_cast<DataIndexType>(shape[d]) * strides[t][d];
            idx[d] = 0;
        }
    }
}

template <typename T>
T combine(int op, T a, T b)
{
    switch (op)
    {
    case H2X_HALO_SUM: return a + b;
    case H2X_HALO_MAX: return a > b ? a : b;
    case H2X_HALO_MIN: return a < b ? a : b;
    default: return b;
    }
}

// start of a strip along `dim`: legacy/include/distconv/tensor/halo_cuda.hpp:59-81
inline DimType strip_start(DimType len, int side, int width, bool inner)
{
    if (side == H2X_RHS)
        return inner ? len - 2 * width : len - width;
    return inner ? width : 0;
}

} // namespace mi355x

namespace impl
{

// ---- transforms (legacy/include/distconv/tensor/algorithms/transform_cuda.hpp:359-693) --------
template <typename T>
void scale_impl(GPUDev_t, Tensor<T>& t, T alpha)
{
    const h2x_tensor_geometry g = mi355x::plain_geometry(t, "scale");
    const h2x_tensor_geometry* gp[1] = {&g};
    void* ptr[1] = {t.data()};
    const double params[4] = {static_cast<double>(alpha), 0, 0, 0};
    mi355x::check(h2x_tensor_transform(H2X_TRANSFORM_SCALE, mi355x::dtype_of<T>(), 1, gp, ptr, params,
                                       mi355x::gpu_stream(t)),
                  "scale");
}
template <typename T>
void scale_impl(CPUDev_t, Tensor<T>& t, T alpha)
{
    const StrideTuple s[1] = {t.strides()};
    T* p = t.data();
    mi355x::for_each_element(t.shape(), s, [&](const DataIndexType* o) { p[o[0]] = p[o[0]] * alpha; });
}

template <typename T>
void scale_bias_impl(GPUDev_t, const Tensor<T>& src, Tensor<T>& dst, T alpha, T beta)
{
    const h2x_tensor_geometry gs = mi355x::plain_geometry(src, "scale_bias"),
                              gd = mi355x::plain_geometry(dst, "scale_bias");
    const h2x_tensor_geometry* gp[2] = {&gs, &gd};
    void* ptr[2] = {const_cast<T*>(src.const_data()), dst.data()};
    const double params[4] = {static_cast<double>(alpha), static_cast<double>(beta), 0, 0};
    mi355x::check(h2x_tensor_transform(H2X_TRANSFORM_SCALE_BIAS, mi355x::dtype_of<T>(), 2, gp, ptr,
                                       params, mi355x::gpu_stream(dst)),
                  "scale_bias");
}
template <typename T>
void scale_bias_impl(CPUDev_t, const Tensor<T>& src, Tensor<T>& dst, T alpha, T beta)
{
    const StrideTuple s[2] = {src.strides(), dst.strides()};
    const T* a = src.const_data();
    T* b = dst.data();
    mi355x::for_each_element(src.shape(), s,
                             [&](const DataIndexType* o) { b[o[1]] = alpha * a[o[0]] + beta; });
}

// element-for-element copy between equally shaped tensors with any strides
template <typename T>
void copy_values_impl(GPUDev_t, const Tensor<T>& src, Tensor<T>& dst)
{
    const h2x_tensor_geometry gs = mi355x::plain_geometry(src, "copy_values"),
                              gd = mi355x::plain_geometry(dst, "copy_values");
    const h2x_tensor_geometry* gp[2] = {&gs, &gd};
    void* ptr[2] = {const_cast<T*>(src.const_data()), dst.data()};
    mi355x::check(h2x_tensor_transform(H2X_TRANSFORM_COPY, mi355x::dtype_of<T>(), 2, gp, ptr, nullptr,
                                       mi355x::gpu_stream(dst)),
                  "copy_values");
}
template <typename T>
void copy_values_impl(CPUDev_t, const Tensor<T>& src, Tensor<T>& dst)
{
    const StrideTuple s[2] = {src.strides(), dst.strides()};
    const T* a = src.const_data();
    T* b = dst.data();
    mi355x::for_each_element(src.shape(), s, [&](const DataIndexType* o) { b[o[1]] = a[o[0]]; });
}

// dst += sum of src (or src^2) over the dimensions where dst has extent 1
// (tensor::ReduceSum, legacy/include/distconv/tensor/algorithms/reduce_sum_cuda.hpp:388-439)
template <typename T>
void reduce_sum_impl(GPUDev_t, const Tensor<T>& src, Tensor<T>& dst, bool square)
{
    const h2x_tensor_geometry gs = mi355x::plain_geometry(src, "reduce_sum"),
                              gd = mi355x::plain_geometry(dst, "reduce_sum");
    hipStream_t s = mi355x::gpu_stream(dst);
    const size_t bytes = h2x_tensor_reduce_sum_workspace_bytes(&gs, &gd);
    if (bytes == 0)
        throw H2FatalException("reduce_sum: each extent of dst must be 1 or equal to src's");
    void* ws = mi355x::stream_scratch(s, bytes, h2x_host::StreamScratch::REDUCE_PARTIALS);
    mi355x::check(h2x_tensor_reduce_sum(mi355x::dtype_of<T>(), &gs, src.const_data(), &gd, dst.data(),
                                        square ? 1 : 0, ws, s),
                  "reduce_sum");
}
template <typename T>
void reduce_sum_impl(CPUDev_t, const Tensor<T>& src, Tensor<T>& dst, bool square)
{
    // float64 accumulators per destination cell, one rounding at the end
    StrideTuple ds = dst.strides();
    for (NDimType i = 0; i < dst.ndim(); ++i)
        if (dst.shape(i) == 1)
            ds[i] = 0;
    const StrideTuple s[2] = {src.strides(), ds};
    const T* a = src.const_data();
    T* b = dst.data();
    DataIndexType span = 1;
    for (NDimType i = 0; i < dst.ndim(); ++i)
        span += static_cast<DataIndexType>(dst.shape(i) - 1) * dst.stride(i);
    std::vector<double> acc(span, 0.0);
    mi355x::for_each_element(src.shape(), s, [&](const DataIndexType* o) {
        const double x = static_cast<double>(a[o[0]]);
        acc[o[1]] += square ? x * x : x;
    });
    const StrideTuple d1[1] = {dst.strides()};
    mi355x::for_each_element(dst.shape(), d1,
                             [&](const DataIndexType* o) { b[o[0]] = b[o[0]] + static_cast<T>(acc[o[0]]); });
}

// ---- halo ----------------------------------------------------------------------------------------
// host twin of halo_pack_or_unpack_impl(GPUDev_t, ...): the strip in natural order
// (legacy/include/distconv/tensor/halo_cuda.hpp:34-88, halo_packing_cuda.hpp:60-103)
template <typename T>
void halo_pack_or_unpack_impl(CPUDev_t, Tensor<T>& tensor, int dim, int side, int width,
                              Tensor<T>& buffer, bool is_pack, bool is_reverse, int op)
{
    if (!tensor.is_contiguous() || !buffer.is_contiguous())
        throw H2FatalException("halo_pack_or_unpack: tensors must be contiguous");
    if (width == 0)
        return;
    const bool inner = (is_pack && !is_reverse) || (!is_pack && is_reverse);
    ShapeTuple strip = tensor.shape();
    const DimType start = mi355x::strip_start(strip[dim], side, width, inner);
    if (start < 0 || start + width > strip[dim])
        throw H2FatalException("halo_pack_or_unpack: strip outside the tensor");
    strip[dim] = width;
    if (buffer.numel() < product<DataIndexType>(strip))
        throw H2FatalException("halo_pack_or_unpack: buffer smaller than the strip");
    const StrideTuple s[2] = {tensor.strides(), get_contiguous_strides(strip)};
    T* t = tensor.data() + start * tensor.stride(dim);
    T* b = buffer.data();
    mi355x::for_each_element(strip, s, [&](const DataIndexType* o) {
        if (is_pack)
            b[o[1]] = t[o[0]];
        else
            t[o[0]] = mi355x::combine(op, t[o[0]], b[o[1]]);
    });
}

// tensor[halo strips of dim] = 0 (TensorImplHelper::clear_halo, legacy/src/tensor/tensor_mpi_cuda.cu:14-84)
template <typename T>
void clear_halo_impl(GPUDev_t, Tensor<T>& tensor, int dim, int width)
{
    if (!tensor.is_contiguous())
        throw H2FatalException("clear_halo: the tensor must be contiguous");
    int64_t shape[H2X_MAX_DIMS] = {};
    for (NDimType i = 0; i < tensor.ndim(); ++i)
        shape[i] = tensor.shape(i);
    mi355x::check(h2x_halo_clear(mi355x::dtype_of<T>(), tensor.data(), tensor.ndim(), shape, dim, width,
                                 mi355x::gpu_stream(tensor)),
                  "clear_halo");
}
template <typename T>
void clear_halo_impl(CPUDev_t, Tensor<T>& tensor, int dim, int width)
{
    if (width == 0)
        return;
    ShapeTuple strip = tensor.shape();
    const DimType len = strip[dim];
    if (2 * width > len)
        throw H2FatalException("clear_halo: strips outside the tensor");
    strip[dim] = width;
    const StrideTuple s[1] = {tensor.strides()};
    for (int side = 0; side < 2; ++side)
    {
        T* t = tensor.data() + mi355x::strip_start(len, side, width, false) * tensor.stride(dim);
        mi355x::for_each_element(strip, s, [&](const DataIndexType* o) { t[o[0]] = T(0); });
    }
}

// One strip straight from `src` into its neighbour `dst` (h2x_halo_exchange_fused):
// forward, the boundary strip of src at src_side lands in the halo of dst on the
// opposite side; reverse, the halo of src is combined into dst's boundary strip.
template <typename T>
void halo_transfer_impl(GPUDev_t, const Tensor<T>& src, Tensor<T>& dst, int dim, int src_side,
                        int width, bool is_reverse, int op)
{
    if (!src.is_contiguous() || !dst.is_contiguous())
        throw H2FatalException("halo_transfer: tensors must be contiguous");
    h2x_halo_transfer m = {};
    m.src = src.const_data();
    m.dst = dst.data();
    for (NDimType i = 0; i < src.ndim(); ++i)
    {
        m.src_real_shape[i] = src.shape(i);
        m.dst_real_shape[i] = dst.shape(i);
    }
    m.num_dims = src.ndim();
    m.dim = dim;
    m.src_side = src_side;
    m.width = width;
    m.is_reverse = is_reverse ? 1 : 0;
    m.op = op;
    mi355x::check(h2x_halo_exchange_fused(mi355x::dtype_of<T>(), &m, 1, mi355x::gpu_stream(dst)),
                  "halo_transfer");
}
template <typename T>
void halo_transfer_impl(CPUDev_t, const Tensor<T>& src, Tensor<T>& dst, int dim, int src_side,
                        int width, bool is_reverse, int op)
{
    if (width == 0)
        return;
    ShapeTuple strip = dst.shape();
    strip[dim] = width;
    const DimType from = mi355x::strip_start(src.shape(dim), src_side, width, !is_reverse);
    const DimType to = mi355x::strip_start(dst.shape(dim), src_side == H2X_LHS ? H2X_RHS : H2X_LHS,
                                           width, is_reverse);
    const StrideTuple s[2] = {src.strides(), dst.strides()};
    const T* a = src.const_data() + from * src.stride(dim);
    T* b = dst.data() + to * dst.stride(dim);
    mi355x::for_each_element(strip, s, [&](const DataIndexType* o) {
        b[o[1]] = mi355x::combine(op, b[o[1]], a[o[0]]);
    });
}

} // namespace impl

// ---- shuffler plans ------------------------------------------------------------------------------
// One rank's side of a shuffle (the tables of the reference's shuffler
// constructor, legacy/include/distconv/tensor/shuffle_mpi_cuda.hpp:129-287) and
// the library's plan for it.
class ShufflePlan
{
public:
    ShufflePlan(const ShapeTuple& local_shape, const StrideTuple& strides,
                const ShapeTuple& peer_locale_shape, const std::vector<int32_t>& rank_limits,
                const std::vector<int32_t>& displs, int elem_size)
        : m_limits(rank_limits), m_displs(displs)
    {
        m_geometry = {};
        m_geometry.num_dims = local_shape.size();
        m_geometry.elem_size = elem_size;
        for (NDimType i = 0; i < local_shape.size(); ++i)
        {
            m_geometry.local_shape[i] = local_shape[i];
            m_geometry.strides[i] = strides[i];
            m_geometry.peer_locale_shape[i] = peer_locale_shape[i];
        }
        m_geometry.rank_limits = m_limits.data();
        m_geometry.displs = m_displs.data();
        mi355x::check(h2x_shuffle_plan_create(&m_geometry, &m_plan), "shuffle plan");
    }
    ~ShufflePlan() { h2x_shuffle_plan_destroy(m_plan); }
    ShufflePlan(const ShufflePlan&) = delete;
    ShufflePlan& operator=(const ShufflePlan&) = delete;
    const h2x_shuffle_plan* get() const { return m_plan; }
    int elem_size() const { return m_geometry.elem_size; }

private:
    std::vector<int32_t> m_limits, m_displs;
    h2x_shuffle_geometry m_geometry;
    h2x_shuffle_plan* m_plan = nullptr;
};

namespace impl
{

// buffer[displs[p] + o] = tensor[box_p(o)] (legacy/src/tensor/shuffle_mpi_cuda.cu:114-248);
// `tensor` starts at the first interior element
template <typename T>
void shuffle_pack_impl(GPUDev_t, const ShufflePlan& plan, const Tensor<T>& tensor, Tensor<T>& buffer)
{
    if (plan.elem_size() != static_cast<int>(sizeof(T)) || !buffer.is_contiguous())
        throw H2FatalException("shuffle_pack: element size or buffer layout does not fit the plan");
    mi355x::check(h2x_shuffle_pack(plan.get(), tensor.const_data(), buffer.data(),
                                   mi355x::gpu_stream(tensor)),
                  "shuffle_pack");
}
// tensor[box_p(o)] = buffer[displs[p] + o] (shuffle_mpi_cuda.cu:251-372)
template <typename T>
void shuffle_unpack_impl(GPUDev_t, const ShufflePlan& plan, Tensor<T>& tensor, const Tensor<T>& buffer)
{
    if (plan.elem_size() != static_cast<int>(sizeof(T)) || !buffer.is_contiguous())
        throw H2FatalException("shuffle_unpack: element size or buffer layout does not fit the plan");
    mi355x::check(h2x_shuffle_unpack(plan.get(), tensor.data(), buffer.const_data(),
                                     mi355x::gpu_stream(tensor)),
                  "shuffle_unpack");
}

// ---- instance-mode softmax (legacy/src/dnn_backend/softmax.cu:357-536,705-784) --------------------
// Softmax over all elements of a sample; tensors are contiguous
// {Spatial..., Channel, Sample}; each sample is whole on this rank.
template <typename T>
void softmax_instance_forward_impl(GPUDev_t, const Tensor<T>& x, Tensor<T>& y)
{
    mi355x::require_same(x, y, "softmax_instance_forward");
    const h2x_tensor_geometry g = mi355x::channel_geometry(x, "softmax_instance_forward");
    if (!x.is_contiguous() || !y.is_contiguous())
        throw H2FatalException("softmax_instance_forward: tensors must be contiguous");
    const int n = static_cast<int>(g.local_shape[g.num_dims - 1]);
    const size_t size = static_cast<size_t>(x.numel()) / n;
    hipStream_t s = mi355x::gpu_stream(x);
    void* ws = mi355x::stream_scratch(s, h2x_softmax_instance_workspace_bytes(n),
                                      h2x_host::StreamScratch::SOFTMAX_PARTIALS);
    T* scalars = static_cast<T*>(mi355x::stream_scratch(s, 2 * n * sizeof(T),
                                                      h2x_host::StreamScratch::SOFTMAX_SCALARS));
    const h2x_dtype dt = mi355x::dtype_of<T>();
    // an h2 tensor is one rank's whole tensor: no all-reduce between the stages
    mi355x::check(h2x_softmax_instance_forward_local(dt, n, size, x.const_data(), y.data(), scalars,
                                                     scalars + n, ws, s),
                  "softmax instance forward");
}
template <typename T>
void softmax_instance_backward_impl(GPUDev_t, const Tensor<T>& y, const Tensor<T>& dy, Tensor<T>& dx)
{
    mi355x::require_same(y, dy, "softmax_instance_backward");
    mi355x::require_same(y, dx, "softmax_instance_backward");
    const h2x_tensor_geometry g = mi355x::channel_geometry(y, "softmax_instance_backward");
    if (!y.is_contiguous() || !dy.is_contiguous() || !dx.is_contiguous())
        throw H2FatalException("softmax_instance_backward: tensors must be contiguous");
    const int n = static_cast<int>(g.local_shape[g.num_dims - 1]);
    const size_t size = static_cast<size_t>(y.numel()) / n;
    hipStream_t s = mi355x::gpu_stream(y);
    void* ws = mi355x::stream_scratch(s, h2x_softmax_instance_workspace_bytes(n),
                                      h2x_host::StreamScratch::SOFTMAX_PARTIALS);
    T* dp = static_cast<T*>(mi355x::stream_scratch(s, 2 * n * sizeof(T),
                                                      h2x_host::StreamScratch::SOFTMAX_SCALARS));
    const h2x_dtype dt = mi355x::dtype_of<T>();
    mi355x::check(h2x_softmax_instance_dot(dt, n, size, y.const_data(), dy.const_data(), dp, ws, s),
                  "softmax dot");
    mi355x::check(h2x_softmax_instance_gradient(dt, n, size, y.const_data(), dy.const_data(), dp,
                                                dx.data(), s),
                  "softmax gradient");
}

} // namespace impl

// ---- typed fronts ----------------------------------------------------------------------------------
#define H2X_BOTH(tensor, op, ...)                                                                 \
    H2_DEVICE_DISPATCH((tensor).get_device(), impl::op(DeviceT_v<Device::CPU>, __VA_ARGS__),      \
                       impl::op(DeviceT_v<Device::GPU>, __VA_ARGS__))
#define H2X_GPU_ARM(tensor, op, ...)                                                              \
    H2_DEVICE_DISPATCH((tensor).get_device(),                                                     \
                       throw H2FatalException(#op ": no CPU implementation"),                     \
                       impl::op(DeviceT_v<Device::GPU>, __VA_ARGS__))

template <typename T>
void scale(Tensor<T>& t, T alpha)
{
    H2X_BOTH(t, scale_impl, t, alpha);
}
template <typename T>
void scale_bias(const Tensor<T>& src, Tensor<T>& dst, T alpha, T beta)
{
    mi355x::require_same(src, dst, "scale_bias");
    H2X_BOTH(dst, scale_bias_impl, src, dst, alpha, beta);
}
template <typename T>
void copy_values(const Tensor<T>& src, Tensor<T>& dst)
{
    mi355x::require_same(src, dst, "copy_values");
    H2X_BOTH(dst, copy_values_impl, src, dst);
}
template <typename T>
void reduce_sum(const Tensor<T>& src, Tensor<T>& dst, bool square = false)
{
    if (src.ndim() != dst.ndim() || src.get_device() != dst.get_device())
        throw H2FatalException("reduce_sum: tensors differ in rank or device");
    for (NDimType i = 0; i < src.ndim(); ++i)
        if (dst.shape(i) != 1 && dst.shape(i) != src.shape(i))
            throw H2FatalException("reduce_sum: each extent of dst must be 1 or equal to src's");
    H2X_BOTH(dst, reduce_sum_impl, src, dst, square);
}
template <typename T>
void clear_halo(Tensor<T>& tensor, int dim, int width)
{
    H2X_BOTH(tensor, clear_halo_impl, tensor, dim, width);
}
template <typename T>
void halo_transfer(const Tensor<T>& src, Tensor<T>& dst, int dim, int src_side, int width,
                   bool is_reverse = false, int op = H2X_HALO_ID)
{
    if (src.ndim() != dst.ndim() || src.get_device() != dst.get_device())
        throw H2FatalException("halo_transfer: tensors differ in rank or device");
    for (NDimType i = 0; i < src.ndim(); ++i)
        if (static_cast<int>(i) != dim && src.shape(i) != dst.shape(i))
            throw H2FatalException("halo_transfer: shapes may differ only along the exchanged dimension");
    if (2 * width > src.shape(dim) || 2 * width > dst.shape(dim))
        throw H2FatalException("halo_transfer: strips outside the tensors");
    H2X_BOTH(dst, halo_transfer_impl, src, dst, dim, src_side, width, is_reverse, op);
}
template <typename T>
void shuffle_pack(const ShufflePlan& plan, const Tensor<T>& tensor, Tensor<T>& buffer)
{
    H2X_GPU_ARM(tensor, shuffle_pack_impl, plan, tensor, buffer);
}
template <typename T>
void shuffle_unpack(const ShufflePlan& plan, Tensor<T>& tensor, const Tensor<T>& buffer)
{
    H2X_GPU_ARM(tensor, shuffle_unpack_impl, plan, tensor, buffer);
}
template <typename T>
void softmax_instance_forward(const Tensor<T>& x, Tensor<T>& y)
{
    H2X_GPU_ARM(x, softmax_instance_forward_impl, x, y);
}
template <typename T>
void softmax_instance_backward(const Tensor<T>& y, const Tensor<T>& dy, Tensor<T>& dx)
{
    H2X_GPU_ARM(y, softmax_instance_backward_impl, y, dy, dx);
}

#undef H2X_BOTH
#undef H2X_GPU_ARM

} // namespace h2

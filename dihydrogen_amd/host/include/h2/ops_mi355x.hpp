// The batch-norm, channel-softmax and halo kernels of libh2x as h2 operators.
//
// Every operator comes in the three layers h2 uses for its own (fill, copy:
// include/h2/tensor/init/fill.hpp:96-130, src/tensor/init/fill.cpp:38-59):
//   impl::<op>_impl(GPUDev_t, Tensor<T>...)   the device implementation,
//   <op>(Tensor<T>...)                        typed front, switches on the device,
//   <op>(BaseTensor...)                       type-erased front, finds the typed
//                                             implementation in the dispatch
//                                             registry under "<op>_gpu"
//                                             (include/h2/core/dispatch.hpp:485-494).
// Which dimension is the sample, the channel and the spatial ones is read from
// the tensors' DimensionType tags (tensor_types.hpp:33-43), not from their
// position: {Spatial..., Channel, Sample}, innermost first, is what the
// kernels take; anything else is rejected.  Strided views are accepted where
// the kernels have strided forms (batch-norm), contiguity is required
// elsewhere.  Batch-norm and softmax have no CPU implementation: a CPU tensor
// raises; the halo, transform and sum operators of h2/tensor_ops_mi355x.hpp
// have both arms.
#pragma once

#include "h2/h2_mi355x.hpp"
#include "h2x.h"
#include "h2x_stream_scratch.hpp"

#include <map>
#include <mutex>

namespace h2
{
namespace mi355x
{

inline void check(int status, const char* what)
{
    if (status != 0)
        throw H2FatalException(what, " failed: ", h2x_status_string(status), " (", status, ")");
}

template <typename T>
constexpr h2x_dtype dtype_of()
{
    static_assert(std::is_same<T, float>::value || std::is_same<T, double>::value,
                  "libh2x computes in float or double");
    return std::is_same<T, float>::value ? H2X_F32 : H2X_F64;
}

// {Spatial..., Channel, Sample} -> the geometry record of the C ABI
inline h2x_tensor_geometry channel_geometry(const BaseTensor& t, const char* what)
{
    const NDimType nd = t.ndim();
    if (nd < 3 || nd > 5)
        throw H2FatalException(what, ": expected 1 to 3 spatial dimensions, channel, sample");
    if (t.dim_type(nd - 1) != DT::Sample || t.dim_type(nd - 2) != DT::Channel)
        throw H2FatalException(what, ": the outermost dimensions must be Channel and Sample");
    for (NDimType i = 0; i < nd - 2; ++i)
        if (t.dim_type(i) != DT::Spatial)
            throw H2FatalException(what, ": inner dimensions must be Spatial");
    h2x_tensor_geometry g = {};
    g.num_dims = nd;
    for (NDimType i = 0; i < nd; ++i)
    {
        g.local_shape[i] = t.shape(i);
        g.strides[i] = t.stride(i);
    }
    return g;
}

inline void require_channel_vector(const BaseTensor& t, DimType channels, const char* what)
{
    if (t.numel() != channels || !t.is_contiguous())
        throw H2FatalException(what, ": per-channel tensors must be contiguous with one value per channel");
}

inline void require_same(const BaseTensor& a, const BaseTensor& b, const char* what)
{
    if (a.shape() != b.shape() || a.dim_types() != b.dim_types())
        throw H2FatalException(what, ": tensors differ in shape or dimension types");
    if (a.get_device() != b.get_device())
        throw H2FatalException(what, ": tensors live on different devices");
}

// Device scratch shared by the calls of one stream, grown on demand (calls on a
// stream are ordered).  Kept until h2::release_workspaces(); nothing is freed at
// static destruction.
inline void* stream_scratch(hipStream_t stream, size_t bytes, int slot)
{
    hipError_t err = hipSuccess;
    void* p = h2x_host::StreamScratch::get(stream, slot, bytes, &err);
    check_hip(err, "stream scratch");
    return p;
}

// fp64 partials of the two batch-norm reductions
inline void* bn_workspace(hipStream_t stream, int channels)
{
    return stream_scratch(stream, h2x_bn_workspace_bytes(channels),
                          h2x_host::StreamScratch::BN_PARTIALS);
}

inline hipStream_t gpu_stream(const BaseTensor& t)
{
    return t.get_stream().get_stream<Device::GPU>();
}

} // namespace mi355x

// Frees the device buffers the operators keep per stream (partial sums of the
// reductions): of one stream (call it before destroying the stream) or of every
// stream of the current device.  Waits for the work in flight first.
inline void release_workspaces(hipStream_t stream)
{
    check_hip(h2x_host::StreamScratch::release(stream), "release_workspaces");
}
inline void release_workspaces()
{
    check_hip(h2x_host::StreamScratch::release_all(), "release_workspaces");
}

// ---- device implementations ---------------------------------------------------------------
namespace impl
{

// sums[c] = sum over samples and space of x, sqsums[c] = of x^2
// (batchnorm::channel_sums_and_sqsums, legacy/src/dnn_backend/batchnorm.cu:192-271)
template <typename T>
void batchnorm_channel_sums_impl(GPUDev_t, const Tensor<T>& x, Tensor<T>& sums, Tensor<T>& sqsums)
{
    const h2x_tensor_geometry g = mi355x::channel_geometry(x, "batchnorm_channel_sums");
    const int c = static_cast<int>(g.local_shape[g.num_dims - 2]);
    mi355x::require_channel_vector(sums, c, "batchnorm_channel_sums");
    mi355x::require_channel_vector(sqsums, c, "batchnorm_channel_sums");
    hipStream_t s = mi355x::gpu_stream(x);
    mi355x::check(h2x_bn_channel_sums_and_sqsums_strided(
                      mi355x::dtype_of<T>(), static_cast<int>(g.local_shape[g.num_dims - 1]), &g,
                      x.const_data(), sums.data(), sqsums.data(), mi355x::bn_workspace(s, c), s),
                  "batchnorm_channel_sums");
}

// in place: sums -> mean, sqsums -> unbiased variance; running statistics
// updated with `decay` (batchnorm::sums_to_statistics, batchnorm.cu:288-346)
template <typename T>
void batchnorm_statistics_impl(GPUDev_t, Tensor<T>& mean, Tensor<T>& var, Tensor<T>& running_mean,
                               Tensor<T>& running_var, std::size_t num_per_sum, double decay)
{
    const DimType c = static_cast<DimType>(mean.numel());
    for (const BaseTensor* t : {static_cast<BaseTensor*>(&var), static_cast<BaseTensor*>(&running_mean),
                                static_cast<BaseTensor*>(&running_var)})
        mi355x::require_channel_vector(*t, c, "batchnorm_statistics");
    mi355x::check(h2x_bn_sums_to_statistics(mi355x::dtype_of<T>(), c, num_per_sum, decay, mean.data(),
                                            var.data(), running_mean.data(), running_var.data(),
                                            mi355x::gpu_stream(mean)),
                  "batchnorm_statistics");
}

// y = (x - mean) / sqrt(var + epsilon) * scale + bias (batchnorm.cu:420-573)
template <typename T>
void batchnorm_normalize_impl(GPUDev_t, const Tensor<T>& x, const Tensor<T>& mean,
                              const Tensor<T>& var, const Tensor<T>& scale, const Tensor<T>& bias,
                              Tensor<T>& y, double epsilon)
{
    mi355x::require_same(x, y, "batchnorm_normalize");
    const h2x_tensor_geometry gx = mi355x::channel_geometry(x, "batchnorm_normalize");
    const h2x_tensor_geometry gy = mi355x::channel_geometry(y, "batchnorm_normalize");
    const DimType c = static_cast<DimType>(gx.local_shape[gx.num_dims - 2]);
    for (const BaseTensor* t : {static_cast<const BaseTensor*>(&mean), static_cast<const BaseTensor*>(&var),
                                static_cast<const BaseTensor*>(&scale),
                                static_cast<const BaseTensor*>(&bias)})
        mi355x::require_channel_vector(*t, c, "batchnorm_normalize");
    mi355x::check(h2x_bn_batch_normalization_strided(
                      mi355x::dtype_of<T>(), static_cast<int>(gx.local_shape[gx.num_dims - 1]), &gx,
                      &gy, x.const_data(), mean.const_data(), var.const_data(), scale.const_data(),
                      bias.const_data(), y.data(), epsilon, mi355x::gpu_stream(x)),
                  "batchnorm_normalize");
}

// the four per-channel sums of the backward pass (batchnorm.cu:982-1230)
template <typename T>
void batchnorm_backprop1_impl(GPUDev_t, const Tensor<T>& x, const Tensor<T>& dy,
                              const Tensor<T>& mean, const Tensor<T>& var, const Tensor<T>& scale,
                              Tensor<T>& dscale, Tensor<T>& dbias, Tensor<T>& dmean,
                              Tensor<T>& dvar, double epsilon)
{
    mi355x::require_same(x, dy, "batchnorm_backprop1");
    const h2x_tensor_geometry gx = mi355x::channel_geometry(x, "batchnorm_backprop1");
    const h2x_tensor_geometry gd = mi355x::channel_geometry(dy, "batchnorm_backprop1");
    const DimType c = static_cast<DimType>(gx.local_shape[gx.num_dims - 2]);
    for (const BaseTensor* t :
         {static_cast<const BaseTensor*>(&mean), static_cast<const BaseTensor*>(&var),
          static_cast<const BaseTensor*>(&scale), static_cast<const BaseTensor*>(&dscale),
          static_cast<const BaseTensor*>(&dbias), static_cast<const BaseTensor*>(&dmean),
          static_cast<const BaseTensor*>(&dvar)})
        mi355x::require_channel_vector(*t, c, "batchnorm_backprop1");
    hipStream_t s = mi355x::gpu_stream(x);
    mi355x::check(h2x_bn_backprop1_strided(
                      mi355x::dtype_of<T>(), static_cast<int>(gx.local_shape[gx.num_dims - 1]), &gx,
                      &gd, x.const_data(), dy.const_data(), mean.const_data(), var.const_data(),
                      scale.const_data(), dscale.data(), dbias.data(), dmean.data(), dvar.data(),
                      epsilon, mi355x::bn_workspace(s, c), s),
                  "batchnorm_backprop1");
}

// dx from dy, x and the reduced gradients (batchnorm.cu:1371-1559); dx may be x
template <typename T>
void batchnorm_backprop2_impl(GPUDev_t, const Tensor<T>& x, const Tensor<T>& dy,
                              const Tensor<T>& mean, const Tensor<T>& var, const Tensor<T>& scale,
                              const Tensor<T>& dmean, const Tensor<T>& dvar, Tensor<T>& dx,
                              std::size_t num_per_sum, double epsilon)
{
    mi355x::require_same(x, dy, "batchnorm_backprop2");
    mi355x::require_same(x, dx, "batchnorm_backprop2");
    const h2x_tensor_geometry gx = mi355x::channel_geometry(x, "batchnorm_backprop2");
    const h2x_tensor_geometry gd = mi355x::channel_geometry(dy, "batchnorm_backprop2");
    const h2x_tensor_geometry go = mi355x::channel_geometry(dx, "batchnorm_backprop2");
    const DimType c = static_cast<DimType>(gx.local_shape[gx.num_dims - 2]);
    for (const BaseTensor* t :
         {static_cast<const BaseTensor*>(&mean), static_cast<const BaseTensor*>(&var),
          static_cast<const BaseTensor*>(&scale), static_cast<const BaseTensor*>(&dmean),
          static_cast<const BaseTensor*>(&dvar)})
        mi355x::require_channel_vector(*t, c, "batchnorm_backprop2");
    mi355x::check(h2x_bn_backprop2_strided(
                      mi355x::dtype_of<T>(), static_cast<int>(gx.local_shape[gx.num_dims - 1]),
                      num_per_sum, &gx, &gd, &go, x.const_data(), dy.const_data(), mean.const_data(),
                      var.const_data(), scale.const_data(), dmean.const_data(), dvar.const_data(),
                      dx.data(), epsilon, mi355x::gpu_stream(x)),
                  "batchnorm_backprop2");
}

// The local forward pass in two launches: sums of x and of x^2, then a kernel
// that turns them into mean / unbiased variance / running statistics and
// normalises.  Same bits as channel_sums + statistics + normalize, one
// statistics launch and two reads of the partial sums fewer
// (what BatchNormalization::forward does between its allreduces when there is
// one process, legacy/include/distconv/dnn_backend/batchnorm.hpp:294-334).
template <typename T>
void batchnorm_forward_impl(GPUDev_t, const Tensor<T>& x, const Tensor<T>& scale,
                            const Tensor<T>& bias, Tensor<T>& mean, Tensor<T>& var,
                            Tensor<T>& running_mean, Tensor<T>& running_var, Tensor<T>& y,
                            std::size_t num_per_sum, double decay, double epsilon)
{
    mi355x::require_same(x, y, "batchnorm_forward");
    const h2x_tensor_geometry gx = mi355x::channel_geometry(x, "batchnorm_forward");
    const h2x_tensor_geometry gy = mi355x::channel_geometry(y, "batchnorm_forward");
    const DimType c = static_cast<DimType>(gx.local_shape[gx.num_dims - 2]);
    for (const BaseTensor* t :
         {static_cast<const BaseTensor*>(&scale), static_cast<const BaseTensor*>(&bias),
          static_cast<const BaseTensor*>(&mean), static_cast<const BaseTensor*>(&var),
          static_cast<const BaseTensor*>(&running_mean), static_cast<const BaseTensor*>(&running_var)})
        mi355x::require_channel_vector(*t, c, "batchnorm_forward");
    hipStream_t s = mi355x::gpu_stream(x);
    mi355x::check(h2x_bn_forward_local_strided(
                      mi355x::dtype_of<T>(), static_cast<int>(gx.local_shape[gx.num_dims - 1]), &gx,
                      &gy, x.const_data(), scale.const_data(), bias.const_data(), num_per_sum, decay,
                      epsilon, mean.data(), var.data(), running_mean.data(), running_var.data(),
                      y.data(), mi355x::bn_workspace(s, c), s),
                  "batchnorm_forward");
}

// The local backward pass in two launches: the four sums, then a kernel that
// adds them and writes dx.  Same bits as backprop1 + backprop2; dx may be x
// (legacy/include/distconv/dnn_backend/batchnorm.hpp:433-470 with one process).
template <typename T>
void batchnorm_backward_impl(GPUDev_t, const Tensor<T>& x, const Tensor<T>& dy,
                             const Tensor<T>& mean, const Tensor<T>& var, const Tensor<T>& scale,
                             Tensor<T>& dscale, Tensor<T>& dbias, Tensor<T>& dmean, Tensor<T>& dvar,
                             Tensor<T>& dx, std::size_t num_per_sum, double epsilon)
{
    mi355x::require_same(x, dy, "batchnorm_backward");
    mi355x::require_same(x, dx, "batchnorm_backward");
    const h2x_tensor_geometry gx = mi355x::channel_geometry(x, "batchnorm_backward");
    const h2x_tensor_geometry gd = mi355x::channel_geometry(dy, "batchnorm_backward");
    const h2x_tensor_geometry go = mi355x::channel_geometry(dx, "batchnorm_backward");
    const DimType c = static_cast<DimType>(gx.local_shape[gx.num_dims - 2]);
    for (const BaseTensor* t :
         {static_cast<const BaseTensor*>(&mean), static_cast<const BaseTensor*>(&var),
          static_cast<const BaseTensor*>(&scale), static_cast<const BaseTensor*>(&dscale),
          static_cast<const BaseTensor*>(&dbias), static_cast<const BaseTensor*>(&dmean),
          static_cast<const BaseTensor*>(&dvar)})
        mi355x::require_channel_vector(*t, c, "batchnorm_backward");
    hipStream_t s = mi355x::gpu_stream(x);
    mi355x::check(h2x_bn_backward_local_strided(
                      mi355x::dtype_of<T>(), static_cast<int>(gx.local_shape[gx.num_dims - 1]),
                      num_per_sum, &gx, &gd, &go, x.const_data(), dy.const_data(), mean.const_data(),
                      var.const_data(), scale.const_data(), dscale.data(), dbias.data(), dmean.data(),
                      dvar.data(), dx.data(), epsilon, mi355x::bn_workspace(s, c), s),
                  "batchnorm_backward");
}

// softmax over the Channel dimension (legacy/src/dnn_backend/softmax.cu:538-619)
template <typename T>
void softmax_channel_forward_impl(GPUDev_t, const Tensor<T>& x, Tensor<T>& y)
{
    mi355x::require_same(x, y, "softmax_channel_forward");
    const h2x_tensor_geometry g = mi355x::channel_geometry(x, "softmax_channel_forward");
    if (!x.is_contiguous() || !y.is_contiguous())
        throw H2FatalException("softmax_channel_forward: tensors must be contiguous");
    std::size_t spatial = 1;
    for (int i = 0; i < g.num_dims - 2; ++i)
        spatial *= static_cast<std::size_t>(g.local_shape[i]);
    mi355x::check(h2x_softmax_channel_forward(
                      mi355x::dtype_of<T>(), static_cast<int>(g.local_shape[g.num_dims - 1]),
                      static_cast<int>(g.local_shape[g.num_dims - 2]), spatial, x.const_data(),
                      y.data(), mi355x::gpu_stream(x)),
                  "softmax_channel_forward");
}

// softmax.cu:621-701
template <typename T>
void softmax_channel_backward_impl(GPUDev_t, const Tensor<T>& y, const Tensor<T>& dy, Tensor<T>& dx)
{
    mi355x::require_same(y, dy, "softmax_channel_backward");
    mi355x::require_same(y, dx, "softmax_channel_backward");
    const h2x_tensor_geometry g = mi355x::channel_geometry(y, "softmax_channel_backward");
    if (!y.is_contiguous() || !dy.is_contiguous() || !dx.is_contiguous())
        throw H2FatalException("softmax_channel_backward: tensors must be contiguous");
    std::size_t spatial = 1;
    for (int i = 0; i < g.num_dims - 2; ++i)
        spatial *= static_cast<std::size_t>(g.local_shape[i]);
    mi355x::check(h2x_softmax_channel_backward(
                      mi355x::dtype_of<T>(), static_cast<int>(g.local_shape[g.num_dims - 1]),
                      static_cast<int>(g.local_shape[g.num_dims - 2]), spatial, y.const_data(),
                      dy.const_data(), dx.data(), mi355x::gpu_stream(y)),
                  "softmax_channel_backward");
}

// One strip of width `width` at `side` of dimension `dim` of a contiguous
// tensor whose shape includes its halo, to or from a contiguous buffer
// (halo_exchange_cuda::pack_or_unpack,
// legacy/include/distconv/tensor/halo_packing_cuda.hpp:143-167).
template <typename T>
void halo_pack_or_unpack_impl(GPUDev_t, Tensor<T>& tensor, int dim, int side, int width,
                              Tensor<T>& buffer, bool is_pack, bool is_reverse, int op)
{
    if (!tensor.is_contiguous() || !buffer.is_contiguous())
        throw H2FatalException("halo_pack_or_unpack: tensors must be contiguous");
    const NDimType nd = tensor.ndim();
    if (nd > H2X_MAX_DIMS)
        throw H2FatalException("halo_pack_or_unpack: at most ", H2X_MAX_DIMS, " dimensions");
    int64_t shape[H2X_MAX_DIMS] = {};
    for (NDimType i = 0; i < nd; ++i)
        shape[i] = tensor.shape(i);
    if (static_cast<std::size_t>(buffer.numel()) < h2x_halo_size(nd, shape, dim, width))
        throw H2FatalException("halo_pack_or_unpack: buffer smaller than the strip");
    mi355x::check(h2x_halo_pack_or_unpack(mi355x::dtype_of<T>(), tensor.data(), nd, shape, dim, side,
                                          width, buffer.data(), is_pack ? 1 : 0, is_reverse ? 1 : 0,
                                          op, mi355x::gpu_stream(tensor)),
                  "halo_pack_or_unpack");
}

} // namespace impl

} // namespace h2

// scale / copy / sums, clear_halo, halo_transfer, shuffle, instance softmax, and the CPU arms
#include "h2/tensor_ops_mi355x.hpp"

namespace h2
{

// ---- typed fronts --------------------------------------------------------------------------
#define H2X_GPU_ONLY(tensor, call)                                                               \
    do                                                                                            \
    {                                                                                             \
        if ((tensor).get_device() != Device::GPU)                                                 \
            throw H2FatalException(#call ": no CPU implementation");                              \
        call;                                                                                     \
    } while (0)

template <typename T>
void batchnorm_channel_sums(const Tensor<T>& x, Tensor<T>& sums, Tensor<T>& sqsums)
{
    H2X_GPU_ONLY(x, impl::batchnorm_channel_sums_impl(DeviceT_v<Device::GPU>, x, sums, sqsums));
}
template <typename T>
void batchnorm_statistics(Tensor<T>& mean, Tensor<T>& var, Tensor<T>& running_mean,
                          Tensor<T>& running_var, std::size_t num_per_sum, double decay)
{
    H2X_GPU_ONLY(mean, impl::batchnorm_statistics_impl(DeviceT_v<Device::GPU>, mean, var,
                                                       running_mean, running_var, num_per_sum, decay));
}
template <typename T>
void batchnorm_normalize(const Tensor<T>& x, const Tensor<T>& mean, const Tensor<T>& var,
                         const Tensor<T>& scale, const Tensor<T>& bias, Tensor<T>& y, double epsilon)
{
    H2X_GPU_ONLY(x, impl::batchnorm_normalize_impl(DeviceT_v<Device::GPU>, x, mean, var, scale, bias,
                                                   y, epsilon));
}
template <typename T>
void batchnorm_backprop1(const Tensor<T>& x, const Tensor<T>& dy, const Tensor<T>& mean,
                         const Tensor<T>& var, const Tensor<T>& scale, Tensor<T>& dscale,
                         Tensor<T>& dbias, Tensor<T>& dmean, Tensor<T>& dvar, double epsilon)
{
    H2X_GPU_ONLY(x, impl::batchnorm_backprop1_impl(DeviceT_v<Device::GPU>, x, dy, mean, var, scale,
                                                   dscale, dbias, dmean, dvar, epsilon));
}
template <typename T>
void batchnorm_backprop2(const Tensor<T>& x, const Tensor<T>& dy, const Tensor<T>& mean,
                         const Tensor<T>& var, const Tensor<T>& scale, const Tensor<T>& dmean,
                         const Tensor<T>& dvar, Tensor<T>& dx, std::size_t num_per_sum,
                         double epsilon)
{
    H2X_GPU_ONLY(x, impl::batchnorm_backprop2_impl(DeviceT_v<Device::GPU>, x, dy, mean, var, scale,
                                                   dmean, dvar, dx, num_per_sum, epsilon));
}
template <typename T>
void batchnorm_forward(const Tensor<T>& x, const Tensor<T>& scale, const Tensor<T>& bias,
                       Tensor<T>& mean, Tensor<T>& var, Tensor<T>& running_mean,
                       Tensor<T>& running_var, Tensor<T>& y, std::size_t num_per_sum, double decay,
                       double epsilon)
{
    H2X_GPU_ONLY(x, impl::batchnorm_forward_impl(DeviceT_v<Device::GPU>, x, scale, bias, mean, var,
                                                 running_mean, running_var, y, num_per_sum, decay,
                                                 epsilon));
}
template <typename T>
void batchnorm_backward(const Tensor<T>& x, const Tensor<T>& dy, const Tensor<T>& mean,
                        const Tensor<T>& var, const Tensor<T>& scale, Tensor<T>& dscale,
                        Tensor<T>& dbias, Tensor<T>& dmean, Tensor<T>& dvar, Tensor<T>& dx,
                        std::size_t num_per_sum, double epsilon)
{
    H2X_GPU_ONLY(x, impl::batchnorm_backward_impl(DeviceT_v<Device::GPU>, x, dy, mean, var, scale,
                                                  dscale, dbias, dmean, dvar, dx, num_per_sum,
                                                  epsilon));
}
template <typename T>
void softmax_channel_forward(const Tensor<T>& x, Tensor<T>& y)
{
    H2X_GPU_ONLY(x, impl::softmax_channel_forward_impl(DeviceT_v<Device::GPU>, x, y));
}
template <typename T>
void softmax_channel_backward(const Tensor<T>& y, const Tensor<T>& dy, Tensor<T>& dx)
{
    H2X_GPU_ONLY(y, impl::softmax_channel_backward_impl(DeviceT_v<Device::GPU>, y, dy, dx));
}
template <typename T>
void halo_pack(Tensor<T>& tensor, int dim, int side, int width, Tensor<T>& buffer,
               bool is_reverse = false)
{
    H2_DEVICE_DISPATCH(tensor.get_device(),
                       impl::halo_pack_or_unpack_impl(DeviceT_v<Device::CPU>, tensor, dim, side, width,
                                                      buffer, true, is_reverse, H2X_HALO_ID),
                       impl::halo_pack_or_unpack_impl(DeviceT_v<Device::GPU>, tensor, dim, side, width,
                                                      buffer, true, is_reverse, H2X_HALO_ID));
}
template <typename T>
void halo_unpack(Tensor<T>& tensor, int dim, int side, int width, Tensor<T>& buffer,
                 bool is_reverse = false, int op = H2X_HALO_ID)
{
    H2_DEVICE_DISPATCH(tensor.get_device(),
                       impl::halo_pack_or_unpack_impl(DeviceT_v<Device::CPU>, tensor, dim, side, width,
                                                      buffer, false, is_reverse, op),
                       impl::halo_pack_or_unpack_impl(DeviceT_v<Device::GPU>, tensor, dim, side, width,
                                                      buffer, false, is_reverse, op));
}

#undef H2X_GPU_ONLY

// ---- type-erased fronts and their registration ---------------------------------------------
namespace mi355x
{

template <typename T>
const Tensor<T>& as(const BaseTensor& t)
{
    if (t.get_type_info() != get_h2_type<T>())
        throw H2FatalException("operator arguments must all have the same element type");
    return static_cast<const Tensor<T>&>(t);
}
template <typename T>
Tensor<T>& as(BaseTensor& t)
{
    if (t.get_type_info() != get_h2_type<T>())
        throw H2FatalException("operator arguments must all have the same element type");
    return static_cast<Tensor<T>&>(t);
}

// the functions the registry holds: BaseTensor in, typed implementation out
template <typename T>
struct Erased
{
    static void channel_sums(const BaseTensor& x, BaseTensor& sums, BaseTensor& sqsums)
    {
        batchnorm_channel_sums(as<T>(x), as<T>(sums), as<T>(sqsums));
    }
    static void statistics(BaseTensor& mean, BaseTensor& var, BaseTensor& rm, BaseTensor& rv,
                           std::size_t num_per_sum, double decay)
    {
        batchnorm_statistics(as<T>(mean), as<T>(var), as<T>(rm), as<T>(rv), num_per_sum, decay);
    }
    static void normalize(const BaseTensor& x, const BaseTensor& mean, const BaseTensor& var,
                          const BaseTensor& scale, const BaseTensor& bias, BaseTensor& y,
                          double epsilon)
    {
        batchnorm_normalize(as<T>(x), as<T>(mean), as<T>(var), as<T>(scale), as<T>(bias), as<T>(y),
                            epsilon);
    }
    static void backprop1(const BaseTensor& x, const BaseTensor& dy, const BaseTensor& mean,
                          const BaseTensor& var, const BaseTensor& scale, BaseTensor& dscale,
                          BaseTensor& dbias, BaseTensor& dmean, BaseTensor& dvar, double epsilon)
    {
        batchnorm_backprop1(as<T>(x), as<T>(dy), as<T>(mean), as<T>(var), as<T>(scale), as<T>(dscale),
                            as<T>(dbias), as<T>(dmean), as<T>(dvar), epsilon);
    }
    static void backprop2(const BaseTensor& x, const BaseTensor& dy, const BaseTensor& mean,
                          const BaseTensor& var, const BaseTensor& scale, const BaseTensor& dmean,
                          const BaseTensor& dvar, BaseTensor& dx, std::size_t num_per_sum,
                          double epsilon)
    {
        batchnorm_backprop2(as<T>(x), as<T>(dy), as<T>(mean), as<T>(var), as<T>(scale), as<T>(dmean),
                            as<T>(dvar), as<T>(dx), num_per_sum, epsilon);
    }
    static void forward(const BaseTensor& x, const BaseTensor& scale, const BaseTensor& bias,
                        BaseTensor& mean, BaseTensor& var, BaseTensor& rm, BaseTensor& rv,
                        BaseTensor& y, std::size_t num_per_sum, double decay, double epsilon)
    {
        batchnorm_forward(as<T>(x), as<T>(scale), as<T>(bias), as<T>(mean), as<T>(var), as<T>(rm),
                          as<T>(rv), as<T>(y), num_per_sum, decay, epsilon);
    }
    static void backward(const BaseTensor& x, const BaseTensor& dy, const BaseTensor& mean,
                         const BaseTensor& var, const BaseTensor& scale, BaseTensor& dscale,
                         BaseTensor& dbias, BaseTensor& dmean, BaseTensor& dvar, BaseTensor& dx,
                         std::size_t num_per_sum, double epsilon)
    {
        batchnorm_backward(as<T>(x), as<T>(dy), as<T>(mean), as<T>(var), as<T>(scale), as<T>(dscale),
                           as<T>(dbias), as<T>(dmean), as<T>(dvar), as<T>(dx), num_per_sum, epsilon);
    }
    static void softmax_forward(const BaseTensor& x, BaseTensor& y)
    {
        softmax_channel_forward(as<T>(x), as<T>(y));
    }
    static void softmax_backward(const BaseTensor& y, const BaseTensor& dy, BaseTensor& dx)
    {
        softmax_channel_backward(as<T>(y), as<T>(dy), as<T>(dx));
    }
    static void halo(BaseTensor& tensor, int dim, int side, int width, BaseTensor& buffer,
                     bool is_pack, bool is_reverse, int op)
    {
        if (is_pack)
            halo_pack(as<T>(tensor), dim, side, width, as<T>(buffer), is_reverse);
        else
            halo_unpack(as<T>(tensor), dim, side, width, as<T>(buffer), is_reverse, op);
    }
    static void scale_(BaseTensor& t, double alpha) { scale(as<T>(t), static_cast<T>(alpha)); }
    static void scale_bias_(const BaseTensor& src, BaseTensor& dst, double alpha, double beta)
    {
        scale_bias(as<T>(src), as<T>(dst), static_cast<T>(alpha), static_cast<T>(beta));
    }
    static void copy_values_(const BaseTensor& src, BaseTensor& dst) { copy_values(as<T>(src), as<T>(dst)); }
    static void reduce_sum_(const BaseTensor& src, BaseTensor& dst, bool square)
    {
        reduce_sum(as<T>(src), as<T>(dst), square);
    }
    static void clear_halo_(BaseTensor& t, int dim, int width) { clear_halo(as<T>(t), dim, width); }
    static void halo_transfer_(const BaseTensor& src, BaseTensor& dst, int dim, int src_side, int width,
                               bool is_reverse, int op)
    {
        halo_transfer(as<T>(src), as<T>(dst), dim, src_side, width, is_reverse, op);
    }
    static void shuffle_(const ShufflePlan& plan, BaseTensor& tensor, BaseTensor& buffer, bool is_pack)
    {
        if (is_pack)
            shuffle_pack(plan, as<T>(static_cast<const BaseTensor&>(tensor)), as<T>(buffer));
        else
            shuffle_unpack(plan, as<T>(tensor), as<T>(static_cast<const BaseTensor&>(buffer)));
    }
    static void softmax_instance_forward_(const BaseTensor& x, BaseTensor& y)
    {
        softmax_instance_forward(as<T>(x), as<T>(y));
    }
    static void softmax_instance_backward_(const BaseTensor& y, const BaseTensor& dy, BaseTensor& dx)
    {
        softmax_instance_backward(as<T>(y), as<T>(dy), as<T>(dx));
    }
};

template <typename T>
void register_type()
{
    const auto key = get_dispatch_key(get_h2_type<T>());
    dispatch_register("batchnorm_channel_sums_gpu", key, &Erased<T>::channel_sums);
    dispatch_register("batchnorm_statistics_gpu", key, &Erased<T>::statistics);
    dispatch_register("batchnorm_normalize_gpu", key, &Erased<T>::normalize);
    dispatch_register("batchnorm_backprop1_gpu", key, &Erased<T>::backprop1);
    dispatch_register("batchnorm_backprop2_gpu", key, &Erased<T>::backprop2);
    dispatch_register("batchnorm_forward_gpu", key, &Erased<T>::forward);
    dispatch_register("batchnorm_backward_gpu", key, &Erased<T>::backward);
    dispatch_register("softmax_channel_forward_gpu", key, &Erased<T>::softmax_forward);
    dispatch_register("softmax_channel_backward_gpu", key, &Erased<T>::softmax_backward);
    dispatch_register("halo_pack_or_unpack_gpu", key, &Erased<T>::halo);
    dispatch_register("scale_gpu", key, &Erased<T>::scale_);
    dispatch_register("scale_bias_gpu", key, &Erased<T>::scale_bias_);
    dispatch_register("copy_values_gpu", key, &Erased<T>::copy_values_);
    dispatch_register("reduce_sum_gpu", key, &Erased<T>::reduce_sum_);
    dispatch_register("clear_halo_gpu", key, &Erased<T>::clear_halo_);
    dispatch_register("halo_transfer_gpu", key, &Erased<T>::halo_transfer_);
    dispatch_register("shuffle_gpu", key, &Erased<T>::shuffle_);
    dispatch_register("softmax_instance_forward_gpu", key, &Erased<T>::softmax_instance_forward_);
    dispatch_register("softmax_instance_backward_gpu", key, &Erased<T>::softmax_instance_backward_);
}

// Registers the float and double implementations once per process.
inline void register_ops()
{
    static std::once_flag once;
    std::call_once(once, [] {
        register_type<float>();
        register_type<double>();
    });
}

template <typename... Args>
void dispatch(const char* name, const BaseTensor& key_tensor, Args&&... args)
{
    register_ops();
    internal::call_dispatch_entry(name, get_dispatch_key(key_tensor), std::forward<Args>(args)...);
}

} // namespace mi355x

// The element type of the first tensor selects the implementation; a type with
// no registered implementation raises H2FatalException.
inline void batchnorm_channel_sums(const BaseTensor& x, BaseTensor& sums, BaseTensor& sqsums)
{
    mi355x::dispatch("batchnorm_channel_sums_gpu", x, x, sums, sqsums);
}
inline void batchnorm_statistics(BaseTensor& mean, BaseTensor& var, BaseTensor& running_mean,
                                 BaseTensor& running_var, std::size_t num_per_sum, double decay)
{
    mi355x::dispatch("batchnorm_statistics_gpu", mean, mean, var, running_mean, running_var,
                     num_per_sum, decay);
}
inline void batchnorm_normalize(const BaseTensor& x, const BaseTensor& mean, const BaseTensor& var,
                                const BaseTensor& scale, const BaseTensor& bias, BaseTensor& y,
                                double epsilon)
{
    mi355x::dispatch("batchnorm_normalize_gpu", x, x, mean, var, scale, bias, y, epsilon);
}
inline void batchnorm_backprop1(const BaseTensor& x, const BaseTensor& dy, const BaseTensor& mean,
                                const BaseTensor& var, const BaseTensor& scale, BaseTensor& dscale,
                                BaseTensor& dbias, BaseTensor& dmean, BaseTensor& dvar,
                                double epsilon)
{
    mi355x::dispatch("batchnorm_backprop1_gpu", x, x, dy, mean, var, scale, dscale, dbias, dmean, dvar,
                     epsilon);
}
inline void batchnorm_backprop2(const BaseTensor& x, const BaseTensor& dy, const BaseTensor& mean,
                                const BaseTensor& var, const BaseTensor& scale,
                                const BaseTensor& dmean, const BaseTensor& dvar, BaseTensor& dx,
                                std::size_t num_per_sum, double epsilon)
{
    mi355x::dispatch("batchnorm_backprop2_gpu", x, x, dy, mean, var, scale, dmean, dvar, dx,
                     num_per_sum, epsilon);
}
inline void batchnorm_forward(const BaseTensor& x, const BaseTensor& scale, const BaseTensor& bias,
                              BaseTensor& mean, BaseTensor& var, BaseTensor& running_mean,
                              BaseTensor& running_var, BaseTensor& y, std::size_t num_per_sum,
                              double decay, double epsilon)
{
    mi355x::dispatch("batchnorm_forward_gpu", x, x, scale, bias, mean, var, running_mean, running_var,
                     y, num_per_sum, decay, epsilon);
}
inline void batchnorm_backward(const BaseTensor& x, const BaseTensor& dy, const BaseTensor& mean,
                               const BaseTensor& var, const BaseTensor& scale, BaseTensor& dscale,
                               BaseTensor& dbias, BaseTensor& dmean, BaseTensor& dvar, BaseTensor& dx,
                               std::size_t num_per_sum, double epsilon)
{
    mi355x::dispatch("batchnorm_backward_gpu", x, x, dy, mean, var, scale, dscale, dbias, dmean, dvar,
                     dx, num_per_sum, epsilon);
}
inline void softmax_channel_forward(const BaseTensor& x, BaseTensor& y)
{
    mi355x::dispatch("softmax_channel_forward_gpu", x, x, y);
}
inline void softmax_channel_backward(const BaseTensor& y, const BaseTensor& dy, BaseTensor& dx)
{
    mi355x::dispatch("softmax_channel_backward_gpu", y, y, dy, dx);
}
inline void halo_pack(BaseTensor& tensor, int dim, int side, int width, BaseTensor& buffer,
                      bool is_reverse = false)
{
    const bool is_pack = true;
    const int op = H2X_HALO_ID;
    mi355x::dispatch("halo_pack_or_unpack_gpu", tensor, tensor, dim, side, width, buffer, is_pack,
                     is_reverse, op);
}
inline void halo_unpack(BaseTensor& tensor, int dim, int side, int width, BaseTensor& buffer,
                        bool is_reverse = false, int op = H2X_HALO_ID)
{
    const bool is_pack = false;
    mi355x::dispatch("halo_pack_or_unpack_gpu", tensor, tensor, dim, side, width, buffer, is_pack,
                     is_reverse, op);
}
inline void scale(BaseTensor& t, double alpha)
{
    mi355x::dispatch("scale_gpu", t, t, alpha);
}
inline void scale_bias(const BaseTensor& src, BaseTensor& dst, double alpha, double beta)
{
    mi355x::dispatch("scale_bias_gpu", src, src, dst, alpha, beta);
}
inline void copy_values(const BaseTensor& src, BaseTensor& dst)
{
    mi355x::dispatch("copy_values_gpu", src, src, dst);
}
inline void reduce_sum(const BaseTensor& src, BaseTensor& dst, bool square = false)
{
    mi355x::dispatch("reduce_sum_gpu", src, src, dst, square);
}
inline void clear_halo(BaseTensor& t, int dim, int width)
{
    mi355x::dispatch("clear_halo_gpu", t, t, dim, width);
}
inline void halo_transfer(const BaseTensor& src, BaseTensor& dst, int dim, int src_side, int width,
                          bool is_reverse = false, int op = H2X_HALO_ID)
{
    mi355x::dispatch("halo_transfer_gpu", src, src, dst, dim, src_side, width, is_reverse, op);
}
inline void shuffle_pack(const ShufflePlan& plan, BaseTensor& tensor, BaseTensor& buffer)
{
    const bool is_pack = true;
    mi355x::dispatch("shuffle_gpu", tensor, plan, tensor, buffer, is_pack);
}
inline void shuffle_unpack(const ShufflePlan& plan, BaseTensor& tensor, BaseTensor& buffer)
{
    const bool is_pack = false;
    mi355x::dispatch("shuffle_gpu", tensor, plan, tensor, buffer, is_pack);
}
inline void softmax_instance_forward(const BaseTensor& x, BaseTensor& y)
{
    mi355x::dispatch("softmax_instance_forward_gpu", x, x, y);
}
inline void softmax_instance_backward(const BaseTensor& y, const BaseTensor& dy, BaseTensor& dx)
{
    mi355x::dispatch("softmax_instance_backward_gpu", y, y, dy, dx);
}

} // namespace h2

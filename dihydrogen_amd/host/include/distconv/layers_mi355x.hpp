// BatchNormalization and Softmax layer classes of the DistConv API on top of
// the h2x C ABI, plus the free functions that are the reference's kernel seam.
// Signatures follow legacy/include/distconv/dnn_backend/batchnorm.hpp:22-96,
// 100-581 and softmax.hpp:14-63; the backend tag is BackendMI355X.
#pragma once

#include <functional>

#include "distconv/algorithms_mi355x.hpp"
#include "distconv/tensor_mi355x.hpp"

namespace distconv
{

// The part of DNNBackend<> the two layers use: a stream
// (legacy/src/dnn_backend/dnn_backend.cpp:164-180).
class BackendMI355X
{
public:
    explicit BackendMI355X(hipStream_t stream = nullptr) : m_stream(stream) {}
    hipStream_t get_stream() const { return m_stream; }

private:
    hipStream_t m_stream;
};

namespace batchnorm
{

// True when the inner spatial dimensions carry no halo: the layout of the
// reference's optimised kernels (legacy/src/dnn_backend/batchnorm.cu:210-219).
template <typename Tensor>
bool is_dense(const Tensor& t)
{
    for (int i = 0; i < t.get_num_dims() - 3; ++i)
        if (t.get_halo_width(i) != 0)
            return false;
    return true;
}

// (num_channels, spatial, spatial_real) of a dense tensor.
template <typename Tensor>
struct ChannelGeometry
{
    int num_channels;
    size_t spatial, spatial_real;
    explicit ChannelGeometry(const Tensor& t)
    {
        const int nd = t.get_num_dims();
        assert_always(t.get_halo_width(nd - 2) == 0 && t.get_halo_width(nd - 1) == 0);
        num_channels = static_cast<int>(t.get_local_shape()[-2]);
        spatial = spatial_real = 1;
        for (int i = 0; i < nd - 2; ++i)
        {
            spatial *= t.get_local_shape()[i];
            spatial_real *= t.get_local_real_shape()[i];
        }
    }
};

// Local shape + strides for the strided entry points (tensors with a halo on
// an inner spatial dimension: the reference's generic kernels).
template <typename Tensor>
h2x_tensor_geometry tensor_geometry(const Tensor& t, int num_samples)
{
    const int nd = t.get_num_dims();
    assert_always(t.get_halo_width(nd - 2) == 0 && t.get_halo_width(nd - 1) == 0);
    h2x_tensor_geometry g = {};
    g.num_dims = nd;
    const auto strides = t.get_strides();
    for (int i = 0; i < nd; ++i)
    {
        g.local_shape[i] = static_cast<int64_t>(t.get_local_shape()[i]);
        g.strides[i] = static_cast<int64_t>(strides[i]);
    }
    g.local_shape[nd - 1] = num_samples;
    return g;
}

// Local and real extents and halo widths, for the entry points that also
// clear the halo of their output.
template <typename Tensor>
h2x_haloed_geometry haloed_geometry(const Tensor& t)
{
    h2x_haloed_geometry g = {};
    g.num_dims = t.get_num_dims();
    for (int i = 0; i < g.num_dims; ++i)
    {
        g.local_shape[i] = static_cast<int64_t>(t.get_local_shape()[i]);
        g.real_shape[i] = static_cast<int64_t>(t.get_local_real_shape()[i]);
        g.lower_halo[i] = t.get_halo_width(i);
    }
    return g;
}

// Whether `a` has a halo on a spatial dimension (and none on channel or sample).
template <typename Tensor>
bool has_spatial_halo(const Tensor& a)
{
    const int nd = a.get_num_dims();
    bool any = false;
    for (int i = 0; i < nd - 2; ++i)
        any = any || a.get_halo_width(i) > 0;
    return any && a.get_halo_width(nd - 2) == 0 && a.get_halo_width(nd - 1) == 0;
}

// Whether the local parts of two tensors lie in memory alike.
template <typename Tensor>
bool same_haloed_geometry(const Tensor& a, const Tensor& b)
{
    return a.get_local_shape() == b.get_local_shape()
           && a.get_local_real_shape() == b.get_local_real_shape()
           && a.get_halo_width() == b.get_halo_width();
}

// Workspace of fp64 partial sums.  A default-constructed one owns its memory
// (one per layer object, freed with the object); one made by
// default_workspace() refers to the buffer that the calls of one stream share.
class Workspace
{
public:
    Workspace() = default;
    void* get(int num_channels)
    {
        const size_t need = h2x_bn_workspace_bytes(num_channels);
        if (m_shared)
        {
            hipError_t err = hipSuccess;
            void* p = h2x_host::StreamScratch::get(m_stream, h2x_host::StreamScratch::BN_PARTIALS,
                                                   need, &err);
            DISTCONV_CHECK_HIP(err);
            return p;
        }
        if (m_mem.is_null() || m_mem.get_size() < need)
            m_mem.allocate(need);
        return m_mem.get();
    }

private:
    friend Workspace default_workspace(hipStream_t stream);
    explicit Workspace(hipStream_t stream) : m_shared(true), m_stream(stream) {}
    tensor::Memory<tensor::CUDAAllocator> m_mem;
    bool m_shared = false;
    hipStream_t m_stream = nullptr;
};

// Workspace used by the overloads that keep the reference's exact signatures
// (which have no workspace argument): one buffer per stream, created on first
// use (calls on one stream are ordered, so they can share it).  It is kept
// until release_workspaces(); nothing is freed at static destruction.
inline Workspace default_workspace(hipStream_t stream)
{
    return Workspace(stream);
}

// batchnorm.hpp:22-28
template <typename Tensor>
void channel_sums_and_sqsums(int num_dims, int num_samples, const Tensor& input, Tensor& sums,
                             Tensor& sqsums, hipStream_t stream, Workspace& ws)
{
    assert_always(num_dims == 4 || num_dims == 5);
    const ChannelGeometry<Tensor> g(input);
    // a rank that is not a split root, or holds nothing, only zeroes the sums
    // (batchnorm.cu:201-208)
    const bool active = input.get_local_size() > 0 && input.is_split_root();
    const int ns = active ? num_samples : 0;
    if (is_dense(input))
    {
        DISTCONV_CHECK_H2X(h2x_bn_channel_sums_and_sqsums(
            Tensor::h2x_type(), ns, g.num_channels, g.spatial, g.spatial_real,
            input.get_const_base_ptr(), sums.get_base_ptr(), sqsums.get_base_ptr(),
            ws.get(g.num_channels), stream));
    }
    else // batchnorm.cu:232-248
    {
        const h2x_tensor_geometry gx = tensor_geometry(input, ns);
        DISTCONV_CHECK_H2X(h2x_bn_channel_sums_and_sqsums_strided(
            Tensor::h2x_type(), ns, &gx, input.get_const_base_ptr(), sums.get_base_ptr(),
            sqsums.get_base_ptr(), ws.get(g.num_channels), stream));
    }
}

template <typename Tensor>
void channel_sums_and_sqsums(int num_dims, int num_samples, const Tensor& input, Tensor& sums,
                             Tensor& sqsums, hipStream_t stream)
{
    Workspace ws = default_workspace(stream);
    channel_sums_and_sqsums(num_dims, num_samples, input, sums, sqsums, stream, ws);
}

// batchnorm.hpp:30-37
template <typename Tensor>
void sums_to_statistics(index_t num_per_sum, typename Tensor::data_type decay, Tensor& global_mean,
                        Tensor& global_var, Tensor& running_mean, Tensor& running_var,
                        hipStream_t stream)
{
    // As in the reference (batchnorm.cu:317-346) this is a transform over the four
    // per-channel tensors; the functor lives in the library.
    tensor::Transform(global_mean, global_var, running_mean, running_var,
                      tensor::internal::SumsToStatisticsFunctor<typename Tensor::data_type>(
                          num_per_sum, decay),
                      stream);
}

// batchnorm.hpp:39-49
template <typename Tensor>
void batch_normalization(int num_dims, int num_samples, const Tensor& input, const Tensor& mean,
                         const Tensor& var, const Tensor& scale, const Tensor& bias, Tensor& output,
                         typename Tensor::data_type epsilon, hipStream_t stream)
{
    assert_always(num_dims == 4 || num_dims == 5);
    if (input.get_local_size() == 0)
        return;
    const ChannelGeometry<Tensor> gi(input), go(output);
    if (is_dense(input) && is_dense(output))
    {
        DISTCONV_CHECK_H2X(h2x_bn_batch_normalization(
            Tensor::h2x_type(), num_samples, gi.num_channels, gi.spatial, gi.spatial_real,
            go.spatial_real, input.get_const_base_ptr(), mean.get_const_base_ptr(),
            var.get_const_base_ptr(), scale.get_const_base_ptr(), bias.get_const_base_ptr(),
            output.get_base_ptr(), epsilon, stream));
    }
    else
    {
        const h2x_tensor_geometry gx = tensor_geometry(input, num_samples),
                                  gy = tensor_geometry(output, num_samples);
        DISTCONV_CHECK_H2X(h2x_bn_batch_normalization_strided(
            Tensor::h2x_type(), num_samples, &gx, &gy, input.get_const_base_ptr(),
            mean.get_const_base_ptr(), var.get_const_base_ptr(), scale.get_const_base_ptr(),
            bias.get_const_base_ptr(), output.get_base_ptr(), epsilon, stream));
    }
}

// No counterpart in the reference: batch_normalization for haloed tensors of one
// geometry that also clears the halo of `output`, as Tensor::clear_halo on every
// spatial dimension would (tensor_mpi_cuda.cu:14-84), in one pass.
template <typename Tensor>
void batch_normalization_clearing(const Tensor& input, const Tensor& mean, const Tensor& var,
                                  const Tensor& scale, const Tensor& bias, Tensor& output,
                                  typename Tensor::data_type epsilon, hipStream_t stream)
{
    if (input.get_local_size() == 0)
        return;
    assert_always(same_haloed_geometry(input, output));
    const h2x_haloed_geometry g = haloed_geometry(output);
    DISTCONV_CHECK_H2X(h2x_bn_batch_normalization_clearing(
        Tensor::h2x_type(), &g, input.get_const_buffer(), mean.get_const_base_ptr(),
        var.get_const_base_ptr(), scale.get_const_base_ptr(), bias.get_const_base_ptr(),
        output.get_buffer(), epsilon, stream));
}

// Likewise the input gradient; d_input may be the same tensor as input.
template <typename Tensor>
void backprop2_clearing(index_t num_per_sum, const Tensor& input, const Tensor& d_output,
                        const Tensor& mean, const Tensor& var, const Tensor& scale,
                        const Tensor& mean_gradient, const Tensor& var_gradient, Tensor& d_input,
                        typename Tensor::data_type epsilon, hipStream_t stream)
{
    if (input.get_local_size() == 0)
        return;
    assert_always(same_haloed_geometry(input, d_output) && same_haloed_geometry(input, d_input));
    const h2x_haloed_geometry g = haloed_geometry(d_input);
    DISTCONV_CHECK_H2X(h2x_bn_backprop2_clearing(
        Tensor::h2x_type(), num_per_sum, &g, input.get_const_buffer(), d_output.get_const_buffer(),
        mean.get_const_base_ptr(), var.get_const_base_ptr(), scale.get_const_base_ptr(),
        mean_gradient.get_const_base_ptr(), var_gradient.get_const_base_ptr(), d_input.get_buffer(),
        epsilon, stream));
}

// batchnorm.hpp:68-81
template <typename Tensor>
void backprop1(int num_dims, int num_samples, const Tensor& input, const Tensor& d_output,
               const Tensor& mean, const Tensor& var, const Tensor& scale, Tensor& scale_gradient,
               Tensor& bias_gradient, Tensor& mean_gradient, Tensor& var_gradient,
               typename Tensor::data_type epsilon, hipStream_t stream, Workspace& ws)
{
    assert_always(num_dims == 4 || num_dims == 5);
    const ChannelGeometry<Tensor> gi(input), go(d_output);
    const bool active = input.get_local_size() > 0 && input.is_split_root();
    const int ns = active ? num_samples : 0;
    if (is_dense(input) && is_dense(d_output))
    {
        DISTCONV_CHECK_H2X(h2x_bn_backprop1(
            Tensor::h2x_type(), ns, gi.num_channels, gi.spatial, gi.spatial_real, go.spatial_real,
            input.get_const_base_ptr(), d_output.get_const_base_ptr(), mean.get_const_base_ptr(),
            var.get_const_base_ptr(), scale.get_const_base_ptr(), scale_gradient.get_base_ptr(),
            bias_gradient.get_base_ptr(), mean_gradient.get_base_ptr(),
            var_gradient.get_base_ptr(), epsilon, ws.get(gi.num_channels), stream));
    }
    else
    {
        const h2x_tensor_geometry gx = tensor_geometry(input, ns), gd = tensor_geometry(d_output, ns);
        DISTCONV_CHECK_H2X(h2x_bn_backprop1_strided(
            Tensor::h2x_type(), ns, &gx, &gd, input.get_const_base_ptr(),
            d_output.get_const_base_ptr(), mean.get_const_base_ptr(), var.get_const_base_ptr(),
            scale.get_const_base_ptr(), scale_gradient.get_base_ptr(), bias_gradient.get_base_ptr(),
            mean_gradient.get_base_ptr(), var_gradient.get_base_ptr(), epsilon,
            ws.get(gi.num_channels), stream));
    }
}

template <typename Tensor>
void backprop1(int num_dims, int num_samples, const Tensor& input, const Tensor& d_output,
               const Tensor& mean, const Tensor& var, const Tensor& scale, Tensor& scale_gradient,
               Tensor& bias_gradient, Tensor& mean_gradient, Tensor& var_gradient,
               typename Tensor::data_type epsilon, hipStream_t stream)
{
    Workspace ws = default_workspace(stream);
    backprop1(num_dims, num_samples, input, d_output, mean, var, scale, scale_gradient,
              bias_gradient, mean_gradient, var_gradient, epsilon, stream, ws);
}

// batchnorm.hpp:83-96; d_input may be the same tensor as input
template <typename Tensor>
void backprop2(int num_dims, index_t num_samples, index_t num_per_sum, const Tensor& input,
               const Tensor& d_output, const Tensor& mean, const Tensor& var, const Tensor& scale,
               const Tensor& mean_gradient, const Tensor& var_gradient, Tensor& d_input,
               typename Tensor::data_type epsilon, hipStream_t stream)
{
    assert_always(num_dims == 4 || num_dims == 5);
    if (input.get_local_size() == 0)
        return;
    const ChannelGeometry<Tensor> gi(input), go(d_output), gd(d_input);
    const int ns = static_cast<int>(num_samples);
    // the fast path needs halo-free tensors, as in the reference (batchnorm.cu:1503-1506)
    if (is_dense(input) && is_dense(d_output) && is_dense(d_input))
    {
        DISTCONV_CHECK_H2X(h2x_bn_backprop2(
            Tensor::h2x_type(), ns, gi.num_channels, gi.spatial, gi.spatial_real, go.spatial_real,
            gd.spatial_real, num_per_sum, input.get_const_base_ptr(),
            d_output.get_const_base_ptr(), mean.get_const_base_ptr(), var.get_const_base_ptr(),
            scale.get_const_base_ptr(), mean_gradient.get_const_base_ptr(),
            var_gradient.get_const_base_ptr(), d_input.get_base_ptr(), epsilon, stream));
    }
    else
    {
        const h2x_tensor_geometry gx = tensor_geometry(input, ns), gy = tensor_geometry(d_output, ns),
                                  gz = tensor_geometry(d_input, ns);
        DISTCONV_CHECK_H2X(h2x_bn_backprop2_strided(
            Tensor::h2x_type(), ns, num_per_sum, &gx, &gy, &gz, input.get_const_base_ptr(),
            d_output.get_const_base_ptr(), mean.get_const_base_ptr(), var.get_const_base_ptr(),
            scale.get_const_base_ptr(), mean_gradient.get_const_base_ptr(),
            var_gradient.get_const_base_ptr(), d_input.get_base_ptr(), epsilon, stream));
    }
}

} // namespace batchnorm

template <typename Backend, typename DataType>
class BatchNormalization;

// batchnorm.hpp:100-581.  The allreduce between the stages is a callable
// `void(DataType* buf, size_t count)` (the reference's tensor::Allreduce<T>);
// by default it is the identity: one rank, or local statistics.
template <typename DataType>
class BatchNormalization<BackendMI355X, DataType>
{
public:
    using Allreduce = std::function<void(DataType*, size_t)>;

    BatchNormalization(BackendMI355X& backend, int num_dims, DataType decay, DataType epsilon,
                       bool global_stats, BatchnormImpl impl = BatchnormImpl::VIRTUAL)
        : m_stream(backend.get_stream()), m_num_dims(num_dims), m_num_current_samples(0),
          m_decay(decay), m_epsilon(epsilon), m_impl(impl), m_global_stats(global_stats)
    {}

    void set_allreducer(Allreduce fn) { m_allreducer = std::move(fn); }

    template <typename Tensor>
    int forward_stage1(const Tensor& input, Tensor& mean, Tensor& var, bool is_training)
    {
        set_num_samples(static_cast<int>(input.get_local_shape()[-1]));
        if (is_training)
            batchnorm::channel_sums_and_sqsums(m_num_dims, m_num_current_samples, input, mean, var,
                                               m_stream, m_ws);
        return 0;
    }

    template <typename Tensor>
    int forward_allreduce(Tensor& mean, Tensor& var, bool is_training)
    {
        if (!is_training || !m_global_stats || !m_allreducer)
            return 0;
        fused_allreduce(mean, var);
        return 0;
    }

    template <typename Tensor>
    int forward_stage2(const Tensor& input, Tensor& mean, Tensor& var, Tensor& running_mean,
                       Tensor& running_var, Tensor& scale, Tensor& bias, Tensor& output,
                       bool is_training)
    {
        if (is_training)
            batchnorm::sums_to_statistics(num_per_sum(input), m_decay, mean, var, running_mean,
                                          running_var, m_stream);
        const Tensor& m = is_training ? mean : running_mean;
        const Tensor& v = is_training ? var : running_var;
        if (clears(input) && batchnorm::same_haloed_geometry(input, output))
            batchnorm::batch_normalization_clearing(input, m, v, scale, bias, output, m_epsilon,
                                                    m_stream);
        else
            batchnorm::batch_normalization(m_num_dims, m_num_current_samples, input, m, v, scale,
                                           bias, output, m_epsilon, m_stream);
        return 0;
    }

    // forward() and backward() of a rank that all-reduces nothing between its
    // stages (one rank, or local statistics) run as two launches each: the
    // second kernel finishes the first one's sums itself.  Same results as the
    // staged calls, bit for bit.  set_fuse_local(false) keeps the staged calls.
    void set_fuse_local(bool on) { m_fuse_local = on; }

    // Haloed tensors of one geometry: normalise and the input gradient also
    // clear the halo of their output, in one pass over the real tensors (what
    // Convolution::forward does to its input with a clear_halo per dimension
    // before every exchange, convolution.hpp:400-411).  Off by default: the
    // reference's kernels leave halo cells alone.
    void set_clear_output_halo(bool on) { m_clear_output_halo = on; }

    template <typename Tensor>
    int forward(const Tensor& input, Tensor& mean, Tensor& var, Tensor& running_mean,
                Tensor& running_var, Tensor& scale, Tensor& bias, Tensor& output, bool is_training)
    {
        if (is_training && runs_local(input) && !wants_clearing(input) && !wants_clearing(output))
        {
            set_num_samples(static_cast<int>(input.get_local_shape()[-1]));
            const batchnorm::ChannelGeometry<Tensor> gi(input), go(output);
            if (batchnorm::is_dense(input) && batchnorm::is_dense(output))
            {
                DISTCONV_CHECK_H2X(h2x_bn_forward_local(
                    Tensor::h2x_type(), m_num_current_samples, gi.num_channels, gi.spatial,
                    gi.spatial_real, go.spatial_real, input.get_const_base_ptr(),
                    scale.get_const_base_ptr(), bias.get_const_base_ptr(), num_per_sum(input),
                    m_decay, m_epsilon, mean.get_base_ptr(), var.get_base_ptr(),
                    running_mean.get_base_ptr(), running_var.get_base_ptr(), output.get_base_ptr(),
                    m_ws.get(gi.num_channels), m_stream));
            }
            else
            {
                // tensors with halos on inner dimensions: the same two launches through the strides
                const h2x_tensor_geometry gx = batchnorm::tensor_geometry(input, m_num_current_samples),
                                          gy = batchnorm::tensor_geometry(output, m_num_current_samples);
                DISTCONV_CHECK_H2X(h2x_bn_forward_local_strided(
                    Tensor::h2x_type(), m_num_current_samples, &gx, &gy, input.get_const_base_ptr(),
                    scale.get_const_base_ptr(), bias.get_const_base_ptr(), num_per_sum(input),
                    m_decay, m_epsilon, mean.get_base_ptr(), var.get_base_ptr(),
                    running_mean.get_base_ptr(), running_var.get_base_ptr(), output.get_base_ptr(),
                    m_ws.get(gi.num_channels), m_stream));
            }
            return 0;
        }
        forward_stage1(input, mean, var, is_training);
        forward_allreduce(mean, var, is_training);
        forward_stage2(input, mean, var, running_mean, running_var, scale, bias, output,
                       is_training);
        return 0;
    }

    template <typename Tensor>
    int backward_stage1(const Tensor& input, const Tensor& d_output, const Tensor& mean,
                        const Tensor& var, const Tensor& scale, Tensor& scale_gradient,
                        Tensor& bias_gradient, Tensor& mean_gradient, Tensor& var_gradient)
    {
        set_num_samples(static_cast<int>(input.get_local_shape()[-1]));
        batchnorm::backprop1(m_num_dims, m_num_current_samples, input, d_output, mean, var, scale,
                             scale_gradient, bias_gradient, mean_gradient, var_gradient, m_epsilon,
                             m_stream, m_ws);
        return 0;
    }

    template <typename Tensor>
    int backward_allreduce(Tensor& scale_gradient, Tensor& bias_gradient, Tensor& mean_gradient,
                           Tensor& var_gradient, bool skip_weights = false)
    {
        if (!m_global_stats || !m_allreducer)
            return 0;
        fused_allreduce(mean_gradient, var_gradient);
        if (!skip_weights)
        {
            m_allreducer(scale_gradient.get_buffer(), scale_gradient.get_local_pitched_size());
            m_allreducer(bias_gradient.get_buffer(), bias_gradient.get_local_pitched_size());
        }
        return 0;
    }

    template <typename Tensor>
    int backward_stage2(const Tensor& input, const Tensor& d_output, const Tensor& mean,
                        const Tensor& var, const Tensor& scale, const Tensor& mean_gradient,
                        const Tensor& var_gradient, Tensor& d_input)
    {
        if (clears(input) && batchnorm::same_haloed_geometry(input, d_output)
            && batchnorm::same_haloed_geometry(input, d_input))
            batchnorm::backprop2_clearing(num_per_sum(input), input, d_output, mean, var, scale,
                                          mean_gradient, var_gradient, d_input, m_epsilon, m_stream);
        else
            batchnorm::backprop2(m_num_dims, m_num_current_samples, num_per_sum(input), input,
                                 d_output, mean, var, scale, mean_gradient, var_gradient, d_input,
                                 m_epsilon, m_stream);
        return 0;
    }

    template <typename Tensor>
    int backward(const Tensor& input, const Tensor& d_output, const Tensor& mean, const Tensor& var,
                 const Tensor& scale, Tensor& scale_gradient, Tensor& bias_gradient,
                 Tensor& mean_gradient, Tensor& var_gradient, Tensor& d_input)
    {
        if (runs_local(input) && !wants_clearing(input) && !wants_clearing(d_input))
        {
            set_num_samples(static_cast<int>(input.get_local_shape()[-1]));
            const batchnorm::ChannelGeometry<Tensor> gi(input), go(d_output), gd(d_input);
            if (batchnorm::is_dense(input) && batchnorm::is_dense(d_output)
                && batchnorm::is_dense(d_input))
            {
                DISTCONV_CHECK_H2X(h2x_bn_backward_local(
                    Tensor::h2x_type(), m_num_current_samples, gi.num_channels, gi.spatial,
                    gi.spatial_real, go.spatial_real, gd.spatial_real, num_per_sum(input),
                    input.get_const_base_ptr(), d_output.get_const_base_ptr(),
                    mean.get_const_base_ptr(), var.get_const_base_ptr(), scale.get_const_base_ptr(),
                    scale_gradient.get_base_ptr(), bias_gradient.get_base_ptr(),
                    mean_gradient.get_base_ptr(), var_gradient.get_base_ptr(),
                    d_input.get_base_ptr(), m_epsilon, m_ws.get(gi.num_channels), m_stream));
            }
            else
            {
                const int ns = m_num_current_samples;
                const h2x_tensor_geometry gx = batchnorm::tensor_geometry(input, ns),
                                          gy = batchnorm::tensor_geometry(d_output, ns),
                                          gz = batchnorm::tensor_geometry(d_input, ns);
                DISTCONV_CHECK_H2X(h2x_bn_backward_local_strided(
                    Tensor::h2x_type(), ns, num_per_sum(input), &gx, &gy, &gz,
                    input.get_const_base_ptr(), d_output.get_const_base_ptr(),
                    mean.get_const_base_ptr(), var.get_const_base_ptr(), scale.get_const_base_ptr(),
                    scale_gradient.get_base_ptr(), bias_gradient.get_base_ptr(),
                    mean_gradient.get_base_ptr(), var_gradient.get_base_ptr(),
                    d_input.get_base_ptr(), m_epsilon, m_ws.get(gi.num_channels), m_stream));
            }
            return 0;
        }
        backward_stage1(input, d_output, mean, var, scale, scale_gradient, bias_gradient,
                        mean_gradient, var_gradient);
        backward_allreduce(scale_gradient, bias_gradient, mean_gradient, var_gradient);
        backward_stage2(input, d_output, mean, var, scale, mean_gradient, var_gradient, d_input);
        return 0;
    }

    // n: number of samples of the current local mini-batch (batchnorm.hpp:467-475)
    void set_num_samples(int n) { m_num_current_samples = n; }

private:
    // no all-reduce would run between the stages, and the rank owns elements
    template <typename Tensor>
    bool runs_local(const Tensor& input) const
    {
        return m_fuse_local && !(m_global_stats && m_allreducer) && input.get_local_size() > 0
               && input.is_split_root();
    }

    // the clearing entry points serve this tensor: it has a halo on a spatial
    // dimension and the whole local mini-batch is current
    template <typename Tensor>
    bool clears(const Tensor& t) const
    {
        return wants_clearing(t) && m_num_current_samples == static_cast<int>(t.get_local_shape()[-1]);
    }
    template <typename Tensor>
    bool wants_clearing(const Tensor& t) const
    {
        return m_clear_output_halo && batchnorm::has_spatial_halo(t);
    }

    // elements per channel of the global (global statistics) or local shape:
    // batchnorm.hpp:232-236,414-418
    template <typename Tensor>
    index_t num_per_sum(const Tensor& input) const
    {
        const auto& s = m_global_stats ? input.get_shape() : input.get_local_shape();
        return s[-2] ? s.get_size() / s[-2] : 0;
    }

    // mean|var (and their gradients) go out as one message when they are
    // adjacent in memory: batchnorm.hpp:196-211,375-390
    template <typename Tensor>
    void fused_allreduce(Tensor& a, Tensor& b)
    {
        auto pa = a.get_buffer();
        auto pb = b.get_buffer();
        const size_t count = a.get_local_pitched_size();
        assert_always(count == b.get_local_pitched_size());
        if (pa + count == pb)
            m_allreducer(pa, count * 2);
        else if (pa == pb + count)
            m_allreducer(pb, count * 2);
        else
        {
            m_allreducer(pa, count);
            m_allreducer(pb, count);
        }
    }

    hipStream_t m_stream;
    int m_num_dims;
    int m_num_current_samples;
    DataType m_decay;
    DataType m_epsilon;
    BatchnormImpl m_impl;
    bool m_global_stats;
    bool m_fuse_local = true;
    bool m_clear_output_halo = false;
    Allreduce m_allreducer;
    batchnorm::Workspace m_ws;
};

template <typename Backend>
class Softmax;

// softmax.hpp:14-63.  Channel mode is one launch; instance mode runs the
// reference's stages (legacy/src/dnn_backend/softmax.cu:705-784) with an
// optional all-reduce of the per-sample scalars between them.
template <>
class Softmax<BackendMI355X>
{
public:
    // allreduce(values, count, is_max): sums (or maximises) `count` per-sample
    // scalars of type T over the ranks that share a sample (softmax.hpp:52-62)
    using Allreduce = std::function<void(void*, size_t, bool)>;

    explicit Softmax(BackendMI355X const& backend) : m_stream(backend.get_stream()) {}
    explicit Softmax(hipStream_t stream) : m_stream(stream) {}

    void set_allreducer(Allreduce fn) { m_allreducer = std::move(fn); }

    template <typename Tensor>
    void setup(const Tensor& input, SoftmaxMode mode)
    {
        (void) input;
        m_mode = mode;
    }

    template <typename Tensor>
    int forward(const Tensor& x, Tensor& y)
    {
        if (x.get_local_size() == 0)
            return 0; // softmax.cu:600-603,717-720
        size_t spatial;
        int n, c;
        geometry(x, n, c, spatial);
        const h2x_dtype dt = Tensor::h2x_type();
        if (m_mode == SoftmaxMode::CHANNEL)
        {
            DISTCONV_CHECK_H2X(h2x_softmax_channel_forward(dt, n, c, spatial, x.get_const_base_ptr(),
                                                           y.get_base_ptr(), m_stream));
            return 0;
        }
        using T = typename Tensor::data_type;
        const size_t size = spatial * c;
        T* scalars = per_sample<T>(n);
        T *smax = scalars, *sexp = scalars + n;
        if (!m_allreducer)
        {
            // every sample is whole on this rank: the stages need not be separate calls
            DISTCONV_CHECK_H2X(h2x_softmax_instance_forward_local(dt, n, size, x.get_const_base_ptr(),
                                                                  y.get_base_ptr(), smax, sexp,
                                                                  workspace(n), m_stream));
            return 0;
        }
        DISTCONV_CHECK_H2X(h2x_softmax_instance_max(dt, n, size, x.get_const_base_ptr(), smax,
                                                    workspace(n), m_stream));
        if (m_allreducer)
            m_allreducer(smax, n, true);
        DISTCONV_CHECK_H2X(h2x_softmax_instance_exp(dt, n, size, x.get_const_base_ptr(), smax,
                                                    y.get_base_ptr(), sexp, workspace(n), m_stream));
        if (m_allreducer)
            m_allreducer(sexp, n, false);
        DISTCONV_CHECK_H2X(h2x_softmax_instance_normalize(dt, n, size, sexp, y.get_base_ptr(),
                                                          m_stream));
        return 0;
    }

    template <typename Tensor>
    int backward(const Tensor& y, const Tensor& dy, Tensor& dx)
    {
        if (dx.get_local_size() == 0)
            return 0;
        size_t spatial;
        int n, c;
        geometry(dx, n, c, spatial);
        const h2x_dtype dt = Tensor::h2x_type();
        if (m_mode == SoftmaxMode::CHANNEL)
        {
            DISTCONV_CHECK_H2X(h2x_softmax_channel_backward(dt, n, c, spatial,
                                                            y.get_const_base_ptr(),
                                                            dy.get_const_base_ptr(),
                                                            dx.get_base_ptr(), m_stream));
            return 0;
        }
        using T = typename Tensor::data_type;
        const size_t size = spatial * c;
        T* sdp = per_sample<T>(n);
        DISTCONV_CHECK_H2X(h2x_softmax_instance_dot(dt, n, size, y.get_const_base_ptr(),
                                                    dy.get_const_base_ptr(), sdp, workspace(n),
                                                    m_stream));
        if (m_allreducer)
            m_allreducer(sdp, n, false);
        DISTCONV_CHECK_H2X(h2x_softmax_instance_gradient(dt, n, size, y.get_const_base_ptr(),
                                                         dy.get_const_base_ptr(), sdp,
                                                         dx.get_base_ptr(), m_stream));
        return 0;
    }

private:
    // dense [N][C][spatial] interior, as the reference assumes (softmax.cu:562-563)
    template <typename Tensor>
    static void geometry(const Tensor& t, int& n, int& c, size_t& spatial)
    {
        for (int i = 0; i < t.get_num_dims(); ++i)
            assert_always(t.get_halo_width(i) == 0);
        n = static_cast<int>(t.get_local_shape()[-1]);
        c = static_cast<int>(t.get_local_shape()[-2]);
        spatial = t.get_local_size() / n / c;
    }

    // The reference takes these from its device memory pool per call
    // (softmax.cu:723-731); here they live with the layer object.
    void* workspace(int n)
    {
        const size_t need = h2x_softmax_instance_workspace_bytes(n);
        if (m_ws.is_null() || m_ws.get_size() < need)
            m_ws.allocate(need);
        return m_ws.get();
    }
    template <typename T>
    T* per_sample(int n)
    {
        const size_t need = 2 * static_cast<size_t>(n) * sizeof(T);
        if (m_scalars.is_null() || m_scalars.get_size() < need)
            m_scalars.allocate(need);
        return static_cast<T*>(m_scalars.get());
    }

    hipStream_t m_stream;
    SoftmaxMode m_mode = SoftmaxMode::CHANNEL;
    Allreduce m_allreducer;
    tensor::Memory<tensor::CUDAAllocator> m_ws, m_scalars;
};

} // namespace distconv

// Distributed-tensor model: Distribution, locales, allocators and
// Tensor<DataType, Locale, Allocator>, with the accessors the hot path and its
// callers use.  Mirrors legacy/include/distconv/tensor/{distribution.hpp,
// tensor.hpp, tensor_mpi.hpp, memory.hpp} of the reference.  The one new type is
// LocaleVirtual: a (rank, size) pair without a communicator, so that several
// ranks' local tensors can live in one process on one GPU; the only collective
// the reference's LocaleMPI tensor needs at construction (the all-gather of
// local extents, tensor_mpi.hpp:509-564) is closed-form for block partitions.
#pragma once

#include <memory>

#include "distconv/base_mi355x.hpp"
#include "h2x_stream_scratch.hpp"

namespace distconv
{

// Frees the device buffers that the free functions with the reference's exact
// signatures (batchnorm::channel_sums_and_sqsums, backprop1, tensor::ReduceSum,
// ...) keep per stream: of one stream (call it before destroying the stream) or
// of every stream of the current device.  Waits for the work in flight first.
// Layer objects own their workspaces and free them with the object; nothing in
// this layer frees device memory from a destructor of static storage duration.
inline void release_workspaces(hipStream_t stream)
{
    DISTCONV_CHECK_HIP(h2x_host::StreamScratch::release(stream));
}
inline void release_workspaces()
{
    DISTCONV_CHECK_HIP(h2x_host::StreamScratch::release_all());
}

namespace tensor
{

// legacy/include/distconv/tensor/distribution.hpp:14-275
class Distribution
{
public:
    Distribution() = default;
    Distribution(const Shape& locale_shape, const Shape& split_shape, const IntVector& overlap)
        : m_locale_shape(locale_shape), m_split_shape(split_shape), m_overlap(overlap)
    {
        assert_always(m_split_shape.length() == num_dims() && m_overlap.length() == num_dims());
        for (int i = 0; i < num_dims(); ++i)
        {
            assert_always(m_split_shape[i] >= 1 && m_locale_shape[i] % m_split_shape[i] == 0);
            if (!is_distributed(i))
                m_overlap[i] = 0; // distribution.hpp:245-251
        }
    }

    static Distribution make_localized_distribution(int num_dims)
    {
        return Distribution(Shape(num_dims, 1), Shape(num_dims, 1), IntVector(num_dims, 0));
    }
    static Distribution make_distribution(const Shape& locale_shape)
    {
        return Distribution(locale_shape, locale_shape, IntVector(locale_shape.length(), 0));
    }
    static Distribution make_overlapped_distribution(const Shape& locale_shape,
                                                     const IntVector& overlap)
    {
        return Distribution(locale_shape, locale_shape, overlap);
    }
    static Distribution make_shared_distribution(const Shape& locale_shape)
    {
        return Distribution(locale_shape, Shape(locale_shape.length(), 1),
                            IntVector(locale_shape.length(), 0));
    }
    static Distribution make_shared_distribution(const Shape& locale_shape,
                                                 const Shape& split_shape)
    {
        return Distribution(locale_shape, split_shape, IntVector(locale_shape.length(), 0));
    }

    int num_dims() const { return m_locale_shape.length(); }
    const Shape& get_locale_shape() const { return m_locale_shape; }
    const Shape& get_split_shape() const { return m_split_shape; }
    const IntVector& get_overlap() const { return m_overlap; }
    int get_overlap(int dim) const { return m_overlap[dim]; }
    void set_overlap(const IntVector& o) { m_overlap = o; }
    void clear_overlap() { m_overlap = 0; }
    index_t get_num_ranks_per_split(int dim) const { return m_locale_shape[dim] / m_split_shape[dim]; }
    bool is_distributed(int dim) const { return m_split_shape[dim] > 1; }
    bool is_shared(int dim) const { return get_num_ranks_per_split(dim) > 1; }
    bool is_shared() const
    {
        for (int i = 0; i < num_dims(); ++i)
            if (is_shared(i))
                return true;
        return false;
    }
    bool is_split_root(int dim, int rank) const { return rank % get_num_ranks_per_split(dim) == 0; }
    template <typename Idx>
    bool is_split_root(const Idx& rank_idx) const
    {
        for (int i = 0; i < num_dims(); ++i)
            if (!is_split_root(i, static_cast<int>(rank_idx[i])))
                return false;
        return true;
    }
    Distribution get_non_overlapped_distribution() const
    {
        Distribution d(*this);
        d.clear_overlap();
        return d;
    }
    bool operator==(const Distribution& d) const
    {
        return m_locale_shape == d.m_locale_shape && m_split_shape == d.m_split_shape
               && m_overlap == d.m_overlap;
    }
    bool operator!=(const Distribution& d) const { return !(*this == d); }

private:
    Shape m_locale_shape;
    Shape m_split_shape;
    IntVector m_overlap;
};

// Stand-in for LocaleMPI (tensor_mpi.hpp:16-90): rank `rank` of `size` ranks
// that all live in this process.
class LocaleVirtual
{
public:
    LocaleVirtual(int rank = 0, int size = 1) : m_rank(rank), m_size(size)
    {
        assert_always(rank >= 0 && rank < size);
    }
    int get_rank() const { return m_rank; }
    int get_size() const { return m_size; }
    // rank -> grid index, dimension 0 fastest (tensor_mpi.hpp:47-56)
    IndexVector get_rank_idx(const Distribution& dist) const
    {
        IndexVector idx(dist.num_dims(), 0);
        int r = m_rank;
        for (int i = 0; i < dist.num_dims(); ++i)
        {
            idx[i] = r % dist.get_locale_shape()[i];
            r /= static_cast<int>(dist.get_locale_shape()[i]);
        }
        return idx;
    }

private:
    int m_rank, m_size;
};

// Allocators (legacy/include/distconv/tensor/memory.hpp, memory_rocm.hpp:29-77;
// the reference keeps the name CUDAAllocator on ROCm).
struct BaseAllocator
{
    static void* allocate(size_t bytes) { return std::calloc(bytes ? bytes : 1, 1); }
    static void deallocate(void* p) { std::free(p); }
};
struct CUDAAllocator
{
    static void* allocate(size_t bytes)
    {
        void* p = nullptr;
        DISTCONV_CHECK_HIP(hipMalloc(&p, bytes ? bytes : 1));
        DISTCONV_CHECK_HIP(hipMemset(p, 0, bytes ? bytes : 1));
        return p;
    }
    static void deallocate(void* p) { (void) hipFree(p); }
};

template <typename Allocator>
class Memory
{
public:
    Memory() = default;
    ~Memory() { release(); }
    Memory(const Memory&) = delete;
    Memory& operator=(const Memory&) = delete;
    void allocate(size_t bytes)
    {
        release();
        m_ptr = Allocator::allocate(bytes);
        m_bytes = bytes;
    }
    void release()
    {
        if (m_ptr)
            Allocator::deallocate(m_ptr);
        m_ptr = nullptr;
        m_bytes = 0;
    }
    bool is_null() const { return m_ptr == nullptr; }
    void* get() const { return m_ptr; }
    size_t get_size() const { return m_bytes; }

private:
    void* m_ptr = nullptr;
    size_t m_bytes = 0;
};

// First element of part `index` when `extent` is cut into `parts` blocks, the
// first extent % parts of them one longer (tensor_mpi.hpp:458-488).
inline index_t block_start(index_t extent, index_t parts, index_t index)
{
    const index_t base = extent / parts, rem = extent % parts;
    return index * base + (index < rem ? index : rem);
}

template <typename DataType, typename Locale, typename Allocator>
class Tensor
{
public:
    using data_type = DataType;
    using const_data_type = const DataType;
    using locale_type = Locale;
    using allocator_type = Allocator;

    Tensor() = default;
    Tensor(const Shape& shape, const Locale& locale, const Distribution& dist)
        : m_shape(shape), m_locale(locale), m_dist(dist)
    {
        const int nd = shape.length();
        assert_always(dist.num_dims() == nd);
        assert_always(static_cast<index_t>(locale.get_size()) == dist.get_locale_shape().get_size());
        m_proc_idx = locale.get_rank_idx(dist);
        m_split_idx = IndexVector(nd, 0);
        m_local_shape = Shape(nd, 0);
        m_local_real_shape = Shape(nd, 0);
        m_global_index = IndexVector(nd, 0);
        for (int i = 0; i < nd; ++i)
        {
            m_split_idx[i] = m_proc_idx[i] / dist.get_num_ranks_per_split(i);
            const index_t parts = dist.get_split_shape()[i];
            index_t lo = 0, hi = shape[i];
            if (parts > 1)
            {
                lo = block_start(shape[i], parts, m_split_idx[i]);
                hi = block_start(shape[i], parts, m_split_idx[i] + 1);
            }
            m_global_index[i] = lo;
            m_local_shape[i] = hi - lo;
            m_local_real_shape[i] = hi - lo + 2 * static_cast<index_t>(dist.get_overlap(i));
        }
    }

    // geometry ----------------------------------------------------------------
    int get_num_dims() const { return m_shape.length(); }
    int get_num_spatial_dims() const { return get_num_dims() - 2; }
    const Shape& get_shape() const { return m_shape; }
    index_t get_size() const { return m_shape.get_size(); }
    const Shape& get_local_shape() const { return m_local_shape; }
    const Shape& get_local_real_shape() const { return m_local_real_shape; }
    index_t get_local_size() const { return m_local_shape.get_size(); }
    index_t get_local_real_size() const { return m_local_real_shape.get_size(); }
    index_t get_local_pitched_size() const { return get_local_real_size(); }
    const Distribution& get_distribution() const { return m_dist; }
    const Locale& get_locale() const { return m_locale; }
    const Shape& get_locale_shape() const { return m_dist.get_locale_shape(); }
    const Shape& get_split_shape() const { return m_dist.get_split_shape(); }
    const IntVector& get_overlap() const { return m_dist.get_overlap(); }
    const IntVector& get_halo_width() const { return m_dist.get_overlap(); }
    int get_halo_width(int dim) const { return m_dist.get_overlap(dim); }
    const IndexVector& get_proc_index() const { return m_proc_idx; }
    const IndexVector& get_split_index() const { return m_split_idx; }
    const IndexVector& get_global_index() const { return m_global_index; }
    bool is_split_root() const { return m_dist.is_split_root(m_proc_idx); }

    // tensor.hpp:291-298
    Shape get_strides() const
    {
        Shape s(get_num_dims(), 1);
        for (int i = 1; i < get_num_dims(); ++i)
            s[i] = s[i - 1] * m_local_real_shape[i - 1];
        return s;
    }
    index_t get_dimension_rank_offset(int dim, int rank) const
    {
        const index_t parts = m_dist.get_split_shape()[dim];
        if (parts == 1)
            return 0;
        return block_start(m_shape[dim], parts, rank / m_dist.get_num_ranks_per_split(dim));
    }
    // tensor.hpp:322-335
    index_t get_remote_dimension(int dim, index_t rank_idx) const
    {
        const index_t parts = m_dist.get_split_shape()[dim];
        if (parts == 1)
            return m_shape[dim];
        const index_t si = rank_idx / m_dist.get_num_ranks_per_split(dim);
        return block_start(m_shape[dim], parts, si + 1) - block_start(m_shape[dim], parts, si);
    }
    IndexVector get_remote_index(const IndexVector& rank_idx) const
    {
        IndexVector r(get_num_dims(), 0);
        for (int i = 0; i < get_num_dims(); ++i)
            r[i] = get_dimension_rank_offset(i, static_cast<int>(rank_idx[i]));
        return r;
    }
    Shape get_remote_shape(const IndexVector& rank_idx) const
    {
        Shape r(get_num_dims(), 0);
        for (int i = 0; i < get_num_dims(); ++i)
            r[i] = get_remote_dimension(i, rank_idx[i]);
        return r;
    }
    // offset of a local (halo-free) index inside the real allocation
    index_t get_local_offset(const IndexVector& idx) const
    {
        const Shape strides = get_strides();
        index_t off = 0;
        for (int i = 0; i < get_num_dims(); ++i)
            off += (idx[i] + static_cast<index_t>(get_halo_width(i))) * strides[i];
        return off;
    }
    index_t get_local_offset() const { return get_local_offset(IndexVector(get_num_dims(), 0)); }

    // storage -----------------------------------------------------------------
    int allocate()
    {
        m_mem = std::make_shared<Memory<Allocator>>();
        m_mem->allocate(get_local_real_size() * sizeof(DataType));
        return 0;
    }
    void nullify() { m_mem.reset(); }
    bool is_null() const { return !m_mem || m_mem->is_null(); }
    // start of the real (haloed) allocation: tensor.hpp:449-460
    DataType* get_buffer() { return m_mem ? static_cast<DataType*>(m_mem->get()) : nullptr; }
    const DataType* get_const_buffer() const
    {
        return m_mem ? static_cast<const DataType*>(m_mem->get()) : nullptr;
    }
    // first interior element: tensor.hpp:462-481
    DataType* get_base_ptr() { return m_mem ? get_buffer() + get_local_offset() : nullptr; }
    const DataType* get_const_base_ptr() const
    {
        return m_mem ? get_const_buffer() + get_local_offset() : nullptr;
    }
    const DataType* get_base_ptr() const { return get_const_base_ptr(); }

    // Zeroes both halo strips of `dim` (tensor_mpi.hpp:396-398 ->
    // legacy/src/tensor/tensor_mpi_cuda.cu:14-84).  Device tensors only.
    void clear_halo(int dim, hipStream_t stream)
    {
        const int w = get_halo_width(dim);
        if (w == 0 || get_local_size() == 0)
            return;
        int64_t shape[H2X_MAX_DIMS];
        for (int i = 0; i < get_num_dims(); ++i)
            shape[i] = static_cast<int64_t>(m_local_real_shape[i]);
        DISTCONV_CHECK_H2X(h2x_halo_clear(h2x_type(), get_buffer(), get_num_dims(), shape, dim, w,
                                          stream));
    }

    static h2x_dtype h2x_type()
    {
        static_assert(sizeof(DataType) == 4 || sizeof(DataType) == 8, "float or double tensors");
        return sizeof(DataType) == 4 ? H2X_F32 : H2X_F64;
    }

private:
    Shape m_shape;
    Locale m_locale;
    Distribution m_dist;
    IndexVector m_proc_idx, m_split_idx, m_global_index;
    Shape m_local_shape, m_local_real_shape;
    std::shared_ptr<Memory<Allocator>> m_mem;
};

} // namespace tensor
} // namespace distconv

// The part of the h2 tensor front-end that operators are written against, for
// one MI355X: devices and streams, dimension-type tags, shape/stride tuples,
// the type-erased BaseTensor and the typed Tensor<T>, and the run-time dispatch
// registry.  Names and semantics follow the reference:
//   Device / CPUDev_t / GPUDev_t        include/h2/core/device.hpp:30-75
//   ComputeStream                       include/h2/core/sync.hpp
//   DimensionType, ShapeTuple, ...      include/h2/tensor/tensor_types.hpp:33-118
//   TypeInfo, get_h2_type               include/h2/core/types.hpp:109-220
//   BaseTensor                          include/h2/tensor/tensor_base.hpp
//   Tensor<T>                           include/h2/tensor/tensor.hpp:34-128
//   dispatch_register / get_dispatch_key / call through a registry
//                                       include/h2/core/dispatch.hpp:330-494
// Dimension 0 is the fastest-varying one, as in h2 (strided_memory.hpp:32-42):
// an NCHW tensor has shape {W, H, C, N} and types {Spatial, Spatial, Channel,
// Sample}.
#pragma once

#include <hip/hip_runtime.h>

#include <array>
#include <cstddef>
#include <cstdint>
#include <initializer_list>
#include <map>
#include <mutex>
#include <sstream>
#include <stdexcept>
#include <string>
#include <typeinfo>
#include <utility>

namespace h2
{

// ---- errors (include/h2/utils/Error.hpp:61-125) --------------------------------
class H2ExceptionBase : public std::runtime_error
{
public:
    using std::runtime_error::runtime_error;
};

class H2FatalException : public H2ExceptionBase
{
public:
    template <typename... Args>
    explicit H2FatalException(const Args&... args) : H2ExceptionBase(join(args...))
    {}

private:
    template <typename... Args>
    static std::string join(const Args&... args)
    {
        std::ostringstream os;
        (os << ... << args);
        return os.str();
    }
};

inline void check_hip(hipError_t err, const char* what)
{
    if (err != hipSuccess)
        throw H2FatalException(what, ": ", hipGetErrorString(err));
}

// ---- devices and streams ---------------------------------------------------------
enum class Device
{
    CPU,
    GPU
};

template <Device Dev>
struct DeviceTag
{
    static constexpr Device device = Dev;
    using device_t = std::integral_constant<Device, Dev>;
};

using CPUDev_t = DeviceTag<Device::CPU>::device_t;
using GPUDev_t = DeviceTag<Device::GPU>::device_t;

template <Device Dev>
inline constexpr typename DeviceTag<Dev>::device_t DeviceT_v = {};

// A stream of work on a device.  A GPU stream wraps a hipStream_t it does not
// own; the default-constructed GPU stream is the null stream.
class ComputeStream
{
public:
    explicit ComputeStream(Device device) : m_device(device), m_stream(nullptr) {}
    explicit ComputeStream(hipStream_t stream) : m_device(Device::GPU), m_stream(stream) {}

    Device get_device() const noexcept { return m_device; }

    template <Device Dev>
    auto get_stream() const
    {
        static_assert(Dev == Device::GPU, "only GPU streams carry a handle");
        if (m_device != Device::GPU)
            throw H2FatalException("GPU stream requested from a CPU ComputeStream");
        return m_stream;
    }

    void wait_for_this() const
    {
        if (m_device == Device::GPU)
            check_hip(hipStreamSynchronize(m_stream), "hipStreamSynchronize");
    }

    bool operator==(const ComputeStream& o) const noexcept
    {
        return m_device == o.m_device && m_stream == o.m_stream;
    }
    bool operator!=(const ComputeStream& o) const noexcept { return !(*this == o); }

private:
    Device m_device;
    hipStream_t m_stream;
};

// ---- dimension tags and tuples ---------------------------------------------------
enum class DimensionType
{
    Any,
    Scalar,
    Sample,
    Channel,
    Filter,
    Spatial,
    Sequence
};
using DT = DimensionType;

using NDimType = std::int32_t;
using DimType = std::int32_t;
using DataIndexType = std::int64_t;
static constexpr NDimType MAX_TENSOR_DIMS = 8;

// Up to MAX_TENSOR_DIMS values with a run-time length.
template <typename T>
class NDimTuple
{
public:
    using type = T;
    using size_type = NDimType;

    constexpr NDimTuple() = default;
    constexpr NDimTuple(std::initializer_list<T> v)
    {
        if (v.size() > static_cast<std::size_t>(MAX_TENSOR_DIMS))
            throw H2FatalException("tuple longer than MAX_TENSOR_DIMS");
        for (const T& x : v)
            m_v[m_size++] = x;
    }
    NDimTuple(size_type n, const T& value)
    {
        if (n < 0 || n > MAX_TENSOR_DIMS)
            throw H2FatalException("tuple longer than MAX_TENSOR_DIMS");
        for (m_size = 0; m_size < n; ++m_size)
            m_v[m_size] = value;
    }

    constexpr size_type size() const noexcept { return m_size; }
    constexpr bool is_empty() const noexcept { return m_size == 0; }
    constexpr T& operator[](size_type i) { return m_v[i]; }
    constexpr const T& operator[](size_type i) const { return m_v[i]; }
    void append(const T& x)
    {
        if (m_size == MAX_TENSOR_DIMS)
            throw H2FatalException("tuple longer than MAX_TENSOR_DIMS");
        m_v[m_size++] = x;
    }
    constexpr const T* begin() const noexcept { return m_v.data(); }
    constexpr const T* end() const noexcept { return m_v.data() + m_size; }

    bool operator==(const NDimTuple& o) const noexcept
    {
        if (m_size != o.m_size)
            return false;
        for (size_type i = 0; i < m_size; ++i)
            if (!(m_v[i] == o.m_v[i]))
                return false;
        return true;
    }
    bool operator!=(const NDimTuple& o) const noexcept { return !(*this == o); }

private:
    std::array<T, MAX_TENSOR_DIMS> m_v{};
    size_type m_size = 0;
};

using ShapeTuple = NDimTuple<DimType>;
using DimensionTypeTuple = NDimTuple<DimensionType>;
using DTTuple = DimensionTypeTuple;
using StrideTuple = NDimTuple<DataIndexType>;

template <typename Acc, typename Tuple>
inline Acc product(const Tuple& t)
{
    Acc p = 1;
    for (const auto& x : t)
        p *= static_cast<Acc>(x);
    return p;
}

// strided_memory.hpp:32-42
inline StrideTuple get_contiguous_strides(const ShapeTuple& shape)
{
    StrideTuple strides(shape.size(), 1);
    for (NDimType i = 1; i < shape.size(); ++i)
        strides[i] = static_cast<DataIndexType>(shape[i - 1]) * strides[i - 1];
    return strides;
}

inline bool are_strides_contiguous(const ShapeTuple& shape, const StrideTuple& strides)
{
    return strides == get_contiguous_strides(shape);
}

// ---- run-time type information ----------------------------------------------------
// Tokens index the compute types in the reference's order: float, double,
// int32, uint32 (types.hpp:109-119); other types get max_token.
struct TypeInfo
{
    using TokenType = std::uint8_t;
    static constexpr TokenType max_token = 255;

    TokenType token;
    std::size_t size;
    const std::type_info* info;

    TokenType get_token() const noexcept { return token; }
    std::size_t get_size() const noexcept { return size; }
    const std::type_info* get_type_info() const noexcept { return info; }
};

inline bool operator==(const TypeInfo& a, const TypeInfo& b)
{
    return a.token == b.token && *a.info == *b.info;
}
inline bool operator!=(const TypeInfo& a, const TypeInfo& b) { return !(a == b); }

static constexpr unsigned long NumComputeTypes = 4;

template <typename T>
inline TypeInfo get_h2_type()
{
    TypeInfo::TokenType token = TypeInfo::max_token;
    if (std::is_same<T, float>::value)
        token = 0;
    else if (std::is_same<T, double>::value)
        token = 1;
    else if (std::is_same<T, std::int32_t>::value)
        token = 2;
    else if (std::is_same<T, std::uint32_t>::value)
        token = 3;
    return TypeInfo{token, sizeof(T), &typeid(T)};
}

inline bool is_h2_compute_type(const TypeInfo& ti) { return ti.get_token() < NumComputeTypes; }
inline bool is_compute_type(const TypeInfo& ti) { return ti.get_token() < TypeInfo::max_token; }

// ---- tensors -------------------------------------------------------------------------
enum class ViewType
{
    None,
    Mutable,
    Const
};

class BaseTensor
{
public:
    BaseTensor(const ShapeTuple& shape, const DimensionTypeTuple& dim_types)
        : BaseTensor(ViewType::None, shape, dim_types)
    {}
    virtual ~BaseTensor() = default;

    virtual TypeInfo get_type_info() const noexcept = 0;
    ShapeTuple shape() const noexcept { return tensor_shape; }
    DimType shape(NDimType i) const noexcept { return tensor_shape[i]; }
    DimensionTypeTuple dim_types() const noexcept { return tensor_dim_types; }
    DimensionType dim_type(NDimType i) const noexcept { return tensor_dim_types[i]; }
    virtual StrideTuple strides() const noexcept = 0;
    virtual DataIndexType stride(NDimType i) const noexcept = 0;
    NDimType ndim() const noexcept { return tensor_shape.size(); }
    DataIndexType numel() const noexcept
    {
        return tensor_shape.is_empty() ? 0 : product<DataIndexType>(tensor_shape);
    }
    bool is_empty() const noexcept { return numel() == 0; }
    virtual bool is_contiguous() const noexcept = 0;
    bool is_view() const noexcept { return tensor_view_type != ViewType::None; }
    bool is_const_view() const noexcept { return tensor_view_type == ViewType::Const; }
    virtual Device get_device() const noexcept = 0;
    virtual ComputeStream get_stream() const noexcept = 0;
    virtual void set_stream(const ComputeStream& stream) = 0;
    virtual void* storage_data() = 0;
    virtual const void* storage_data() const = 0;
    virtual const void* const_storage_data() const = 0;

protected:
    BaseTensor(ViewType view_type, const ShapeTuple& shape, const DimensionTypeTuple& dim_types)
        : tensor_shape(shape), tensor_dim_types(dim_types), tensor_view_type(view_type)
    {
        if (shape.size() != dim_types.size())
            throw H2FatalException("tensor shape and dimension types must be the same size");
        for (DimType e : shape)
            if (e <= 0)
                throw H2FatalException("zero-length dimensions are not permitted");
    }

    ShapeTuple tensor_shape;
    DimensionTypeTuple tensor_dim_types;
    ViewType tensor_view_type;
};

// A tensor that owns its memory (device memory for Device::GPU) or wraps a
// caller's buffer as a mutable or constant view (tensor.hpp:42-92).
template <typename T>
class Tensor : public BaseTensor
{
public:
    using value_type = T;

    Tensor(Device device, const ShapeTuple& shape, const DimensionTypeTuple& dim_types,
           const ComputeStream& stream)
        : Tensor(device, shape, dim_types, get_contiguous_strides(shape), stream)
    {}
    Tensor(Device device, const ShapeTuple& shape, const DimensionTypeTuple& dim_types)
        : Tensor(device, shape, dim_types, ComputeStream(device))
    {}
    Tensor(Device device, const ShapeTuple& shape, const DimensionTypeTuple& dim_types,
           const StrideTuple& strides, const ComputeStream& stream)
        : BaseTensor(shape, dim_types), m_device(device), m_stream(stream), m_strides(strides)
    {
        check_strides();
        const std::size_t bytes = extent() * sizeof(T);
        if (bytes == 0)
            return;
        if (device == Device::GPU)
            check_hip(hipMalloc(&m_owned, bytes), "hipMalloc");
        else
            m_owned = ::operator new(bytes);
        m_data = static_cast<T*>(m_owned);
    }
    Tensor(Device device, T* buffer, const ShapeTuple& shape, const DimensionTypeTuple& dim_types,
           const StrideTuple& strides, const ComputeStream& stream)
        : BaseTensor(ViewType::Mutable, shape, dim_types), m_device(device), m_stream(stream),
          m_strides(strides), m_data(buffer)
    {
        check_strides();
    }
    Tensor(Device device, const T* buffer, const ShapeTuple& shape,
           const DimensionTypeTuple& dim_types, const StrideTuple& strides,
           const ComputeStream& stream)
        : BaseTensor(ViewType::Const, shape, dim_types), m_device(device), m_stream(stream),
          m_strides(strides), m_data(const_cast<T*>(buffer))
    {
        check_strides();
    }
    ~Tensor() override
    {
        if (!m_owned)
            return;
        if (m_device == Device::GPU)
            (void) hipFree(m_owned);
        else
            ::operator delete(m_owned);
    }
    Tensor(const Tensor&) = delete;
    Tensor& operator=(const Tensor&) = delete;

    TypeInfo get_type_info() const noexcept override { return get_h2_type<T>(); }
    StrideTuple strides() const noexcept override { return m_strides; }
    DataIndexType stride(NDimType i) const noexcept override { return m_strides[i]; }
    bool is_contiguous() const noexcept override
    {
        return are_strides_contiguous(tensor_shape, m_strides);
    }
    Device get_device() const noexcept override { return m_device; }
    ComputeStream get_stream() const noexcept override { return m_stream; }
    void set_stream(const ComputeStream& stream) override { m_stream = stream; }

    T* data()
    {
        if (is_const_view())
            throw H2FatalException("cannot access a mutable pointer of a const view");
        return m_data;
    }
    const T* data() const { return m_data; }
    const T* const_data() const { return m_data; }
    void* storage_data() override { return data(); }
    const void* storage_data() const override { return m_data; }
    const void* const_storage_data() const override { return m_data; }

private:
    void check_strides() const
    {
        if (m_strides.size() != tensor_shape.size())
            throw H2FatalException("shape and strides must be the same size");
    }
    // elements spanned by the strides (strided_memory.hpp: get_extent_from_strides)
    std::size_t extent() const
    {
        if (tensor_shape.is_empty())
            return 0;
        std::size_t last = 0;
        for (NDimType i = 0; i < tensor_shape.size(); ++i)
            last += static_cast<std::size_t>(tensor_shape[i] - 1) * m_strides[i];
        return last + 1;
    }

    Device m_device;
    ComputeStream m_stream;
    StrideTuple m_strides;
    T* m_data = nullptr;
    void* m_owned = nullptr;
};

// ---- run-time dispatch ------------------------------------------------------------------
// Operators on BaseTensor look their typed implementation up by name and by a
// key made of the arguments' type tokens (dispatch.hpp:446-494).
namespace internal
{

using DispatchKeyT = std::uint64_t;
constexpr std::size_t max_dispatch_types = 7;
constexpr unsigned dispatch_bits_per_compute_type = 8;
constexpr unsigned dispatch_key_top_byte_shift = 56;

struct DispatchFunctionEntry
{
    void* func_ptr;                 // the registered function
    void (*caller)(void*, void**);  // casts func_ptr and the argument pointers back
};

template <typename... Args>
struct DispatchFunctionWrapper
{
    static void call(void* f, void** args) { call_impl(f, args, std::index_sequence_for<Args...>{}); }

private:
    template <std::size_t... I>
    static void call_impl(void* f, void** args, std::index_sequence<I...>)
    {
        reinterpret_cast<void (*)(Args...)>(f)(
            static_cast<Args>(*static_cast<std::remove_reference_t<Args>*>(args[I]))...);
    }
};

inline std::map<std::pair<std::string, DispatchKeyT>, DispatchFunctionEntry>& dispatch_table()
{
    static std::map<std::pair<std::string, DispatchKeyT>, DispatchFunctionEntry> table;
    return table;
}
inline std::mutex& dispatch_mutex()
{
    static std::mutex m;
    return m;
}

inline void add_dispatch_entry(const std::string& name, const DispatchKeyT& key,
                               const DispatchFunctionEntry& entry)
{
    std::lock_guard<std::mutex> lock(dispatch_mutex());
    dispatch_table()[{name, key}] = entry;
}

inline bool has_dispatch_entry(const std::string& name, const DispatchKeyT& key)
{
    std::lock_guard<std::mutex> lock(dispatch_mutex());
    return dispatch_table().count({name, key}) > 0;
}

inline DispatchFunctionEntry get_dispatch_entry(const std::string& name, const DispatchKeyT& key)
{
    std::lock_guard<std::mutex> lock(dispatch_mutex());
    auto it = dispatch_table().find({name, key});
    if (it == dispatch_table().end())
        throw H2FatalException("No dispatch entry for ", name, " with key ", key);
    return it->second;
}

// Arguments are passed as they are declared by the registered function: the
// caller must use exactly those types.
template <typename... Args>
void call_dispatch_entry(const std::string& name, const DispatchKeyT& key, Args&&... args)
{
    const DispatchFunctionEntry entry = get_dispatch_entry(name, key);
    void* ptrs[] = {const_cast<void*>(static_cast<const void*>(&args))..., nullptr};
    entry.caller(entry.func_ptr, ptrs);
}

template <std::size_t N>
constexpr DispatchKeyT get_dispatch_key(const std::array<TypeInfo::TokenType, N>& tokens)
{
    static_assert(N <= max_dispatch_types, "too many types in a dispatch key");
    DispatchKeyT key = static_cast<DispatchKeyT>(N) << dispatch_key_top_byte_shift;
    for (std::size_t i = 0; i < N; ++i)
        key |= static_cast<DispatchKeyT>(tokens[i]) << (dispatch_bits_per_compute_type * (N - 1 - i));
    return key;
}

inline TypeInfo type_info_of(const TypeInfo& t) { return t; }
inline TypeInfo type_info_of(const BaseTensor& t) { return t.get_type_info(); }

} // namespace internal

// Key for the run-time types of `args` (tensors or TypeInfo), first leftmost.
template <typename... TypeInfoHavers>
internal::DispatchKeyT get_dispatch_key(const TypeInfoHavers&... args)
{
    const std::array<TypeInfo, sizeof...(args)> infos = {{internal::type_info_of(args)...}};
    std::array<TypeInfo::TokenType, sizeof...(args)> tokens{};
    for (std::size_t i = 0; i < infos.size(); ++i)
    {
        if (!is_compute_type(infos[i]))
            throw H2FatalException("Cannot construct dispatch keys for non-compute types");
        tokens[i] = infos[i].get_token();
    }
    return internal::get_dispatch_key(tokens);
}

template <typename... Args>
void dispatch_register(const std::string& name, const internal::DispatchKeyT& key,
                       void (*func)(Args...))
{
    internal::add_dispatch_entry(
        name, key,
        internal::DispatchFunctionEntry{reinterpret_cast<void*>(func),
                                        &internal::DispatchFunctionWrapper<Args...>::call});
}

inline void dispatch_unregister(const std::string& name, const internal::DispatchKeyT& key)
{
    std::lock_guard<std::mutex> lock(internal::dispatch_mutex());
    internal::dispatch_table().erase({name, key});
}

} // namespace h2

// Basic vocabulary of the DistConv API surface that the MI355X hot path is
// written against: index types, sides, small integer vectors and shapes.
// Names and meaning follow legacy/include/distconv/base.hpp and
// legacy/include/distconv/vector.hpp / tensor/tensor_base.hpp of the
// reference, so that code written against those headers compiles against
// these; the implementation is independent.
#pragma once

#include <cassert>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <initializer_list>
#include <ostream>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "h2x.h"

namespace distconv
{

using index_t = size_t; // legacy/include/distconv/base.hpp:19

// legacy/include/distconv/base.hpp:23-28
enum Side
{
    LHS = 0,
    RHS = 1
};
const Side SIDES[2] = {LHS, RHS};
inline Side operator~(const Side& s)
{
    return s == LHS ? RHS : LHS;
}

// legacy/include/distconv/base.hpp:316-324 (only the back-ends that exist here)
enum class BatchnormImpl
{
    MPI,
    AL_NCCL,
    VIRTUAL
};

// legacy/include/distconv/base.hpp (SoftmaxMode)
enum class SoftmaxMode
{
    INSTANCE,
    CHANNEL
};

namespace util
{

// Precondition failures abort, as assert_always does in the reference
// (legacy/include/distconv/util/util.hpp:22-34).
[[noreturn]] inline void fail(const char* what, const char* file, int line)
{
    std::fprintf(stderr, "distconv: %s failed at %s:%d\n", what, file, line);
    std::abort();
}

// A failing library call prints the h2x status and aborts: the behaviour of
// DISTCONV_CHECK_HIP (legacy/include/distconv/util/util_rocm.hpp:24-38)
// without the device reset.
inline void check_h2x(int status, const char* what, const char* file, int line)
{
    if (status != 0)
    {
        std::fprintf(stderr, "distconv: %s: %s (%d) at %s:%d\n", what, h2x_status_string(status),
                     status, file, line);
        std::abort();
    }
}

inline void check_hip(hipError_t e, const char* file, int line)
{
    if (e != hipSuccess)
    {
        std::fprintf(stderr, "distconv: HIP error %s at %s:%d\n", hipGetErrorString(e), file, line);
        std::abort();
    }
}

// `later` continues only after the work queued on `earlier` so far
// (util::wait_stream, legacy/include/distconv/util/util_rocm.hpp).  The event
// is released as soon as the wait is queued; the runtime keeps it alive until
// it has fired.
inline void wait_stream(hipStream_t earlier, hipStream_t later)
{
    if (earlier == later)
        return;
    hipEvent_t ev;
    check_hip(hipEventCreateWithFlags(&ev, hipEventDisableTiming), __FILE__, __LINE__);
    check_hip(hipEventRecord(ev, earlier), __FILE__, __LINE__);
    check_hip(hipStreamWaitEvent(later, ev, 0), __FILE__, __LINE__);
    check_hip(hipEventDestroy(ev), __FILE__, __LINE__);
}

inline void wait_stream(hipStream_t earlier, const hipStream_t* later, int num_streams)
{
    for (int i = 0; i < num_streams; ++i)
        wait_stream(earlier, later[i]);
}

// Each stream continues only after the work queued on the other so far
// (util::sync_stream, legacy/src/util/util_rocm.cpp:164-175).
inline void sync_stream(hipStream_t s1, hipStream_t s2)
{
    if (s1 == s2)
        return;
    hipEvent_t ev1, ev2;
    check_hip(hipEventCreateWithFlags(&ev1, hipEventDisableTiming), __FILE__, __LINE__);
    check_hip(hipEventCreateWithFlags(&ev2, hipEventDisableTiming), __FILE__, __LINE__);
    check_hip(hipEventRecord(ev1, s1), __FILE__, __LINE__);
    check_hip(hipEventRecord(ev2, s2), __FILE__, __LINE__);
    check_hip(hipStreamWaitEvent(s2, ev1, 0), __FILE__, __LINE__);
    check_hip(hipStreamWaitEvent(s1, ev2, 0), __FILE__, __LINE__);
    check_hip(hipEventDestroy(ev1), __FILE__, __LINE__);
    check_hip(hipEventDestroy(ev2), __FILE__, __LINE__);
}

// Event timer on one stream (util::Clock,
// legacy/include/distconv/util/util_rocm.hpp:110-138): start() and stop()
// record events, get_time() waits for the second and returns milliseconds.
struct Clock
{
    explicit Clock(hipStream_t s) : m_s(s)
    {
        check_hip(hipEventCreate(&m_ev1), __FILE__, __LINE__);
        check_hip(hipEventCreate(&m_ev2), __FILE__, __LINE__);
    }
    Clock(const Clock& c) : Clock(c.m_s) {}
    Clock& operator=(const Clock& c)
    {
        m_s = c.m_s;
        return *this;
    }
    ~Clock()
    {
        (void) hipEventDestroy(m_ev2);
        (void) hipEventDestroy(m_ev1);
    }
    void start() { check_hip(hipEventRecord(m_ev1, m_s), __FILE__, __LINE__); }
    void stop() { check_hip(hipEventRecord(m_ev2, m_s), __FILE__, __LINE__); }
    float get_time()
    {
        check_hip(hipEventSynchronize(m_ev2), __FILE__, __LINE__);
        float elapsed = 0;
        check_hip(hipEventElapsedTime(&elapsed, m_ev1, m_ev2), __FILE__, __LINE__);
        return elapsed;
    }

    hipStream_t m_s;
    hipEvent_t m_ev1 = nullptr;
    hipEvent_t m_ev2 = nullptr;
};

} // namespace util

#define assert_always(cond)                                                                        \
    do                                                                                             \
    {                                                                                              \
        if (!(cond))                                                                               \
            ::distconv::util::fail(#cond, __FILE__, __LINE__);                                     \
    } while (0)
#define DISTCONV_CHECK_H2X(call) ::distconv::util::check_h2x((call), #call, __FILE__, __LINE__)
#define DISTCONV_CHECK_HIP(call) ::distconv::util::check_hip((call), __FILE__, __LINE__)

// Small vector of per-dimension values; negative indices count from the end
// (legacy/include/distconv/tensor/tensor_base.hpp:73-80).
template <typename T>
class Vector
{
public:
    Vector() = default;
    Vector(int num_dims, T value) : m_v(num_dims, value) {}
    Vector(std::initializer_list<T> v) : m_v(v) {}
    explicit Vector(const std::vector<T>& v) : m_v(v) {}
    template <typename U>
    explicit Vector(const Vector<U>& o)
    {
        for (int i = 0; i < o.length(); ++i)
            m_v.push_back(static_cast<T>(o[i]));
    }

    int length() const { return static_cast<int>(m_v.size()); }
    int num_dims() const { return length(); }
    T& operator[](int i) { return m_v[wrap(i)]; }
    const T& operator[](int i) const { return m_v[wrap(i)]; }
    void push_back(T v) { m_v.push_back(v); }
    const T* data() const { return m_v.data(); }
    typename std::vector<T>::const_iterator begin() const { return m_v.begin(); }
    typename std::vector<T>::const_iterator end() const { return m_v.end(); }

    T reduce_sum() const
    {
        T s = T(0);
        for (auto v : m_v)
            s += v;
        return s;
    }
    T reduce_prod() const
    {
        T s = T(1);
        for (auto v : m_v)
            s *= v;
        return s;
    }
    bool operator==(const Vector& o) const { return m_v == o.m_v; }
    bool operator!=(const Vector& o) const { return !(*this == o); }
    Vector& operator=(T value)
    {
        for (auto& v : m_v)
            v = value;
        return *this;
    }

protected:
    int wrap(int i) const
    {
        const int n = length();
        const int j = i < 0 ? i + n : i;
        assert_always(j >= 0 && j < n);
        return j;
    }
    std::vector<T> m_v;
};

using IntVector = Vector<int>;
using IndexVector = Vector<index_t>;

template <typename T>
std::ostream& operator<<(std::ostream& os, const Vector<T>& v)
{
    os << "(";
    for (int i = 0; i < v.length(); ++i)
        os << (i ? ", " : "") << v[i];
    return os << ")";
}

namespace tensor
{

// Innermost-first extents (legacy/include/distconv/tensor/tensor_base.hpp).
class Shape : public Vector<index_t>
{
public:
    using Vector<index_t>::Vector;
    Shape() = default;
    Shape(const Vector<index_t>& v) : Vector<index_t>(v) {}
    Shape(std::initializer_list<int> v)
    {
        for (int e : v)
            m_v.push_back(static_cast<index_t>(e));
    }
    index_t get_size() const { return reduce_prod(); }
    index_t size() const { return get_size(); }

    // linear offset -> index, dimension 0 fastest
    IndexVector get_index(index_t offset) const
    {
        IndexVector idx(length(), 0);
        for (int i = 0; i < length(); ++i)
        {
            idx[i] = m_v[i] ? offset % m_v[i] : 0;
            offset = m_v[i] ? offset / m_v[i] : 0;
        }
        return idx;
    }
};

// index -> linear offset, dimension 0 fastest
// (legacy/include/distconv/tensor/tensor_base.hpp:344-361)
template <typename Idx>
inline index_t get_offset(const Idx& idx, const Shape& shape)
{
    index_t off = 0, stride = 1;
    for (int i = 0; i < shape.length(); ++i)
    {
        off += static_cast<index_t>(idx[i]) * stride;
        stride *= shape[i];
    }
    return off;
}

// Axis-aligned box; intersect as in tensor_base.hpp:515-567.
struct Region
{
    IndexVector offset;
    Shape shape;
    Region(const IndexVector& o, const Shape& s) : offset(o), shape(s) {}
    index_t get_size() const { return shape.get_size(); }
    Region intersect(const Region& r) const
    {
        const int nd = shape.length();
        IndexVector o(nd, 0);
        Shape s(nd, 0);
        for (int i = 0; i < nd; ++i)
        {
            const index_t lo = offset[i] > r.offset[i] ? offset[i] : r.offset[i];
            const index_t a = offset[i] + shape[i], b = r.offset[i] + r.shape[i];
            const index_t hi = a < b ? a : b;
            o[i] = lo;
            s[i] = hi > lo ? hi - lo : 0;
        }
        return Region(o, s);
    }
};

} // namespace tensor
} // namespace distconv

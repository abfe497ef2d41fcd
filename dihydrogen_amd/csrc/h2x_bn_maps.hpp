// Index maps of the batch-normalisation kernels: where the element (or vector)
// that a lane works on lies in a tensor.  Host and device code: the kernels use
// them to address memory, and the launch audit walks the same functions on the
// CPU over every workgroup and lane of a planned launch to check that each
// interior element is visited exactly once and nothing else is touched.
#pragma once

#include "h2x_device.hpp"

namespace h2x
{
namespace bn
{

// Where the elements of one tensor live.  Element i of segment (n, c) is at
// base[n*stride_n + c*stride_c + offset(i)]; offset(i) = i for the dense layout.
// Strided layout (tensors with halos inside their segments, samples folded into
// rows, dense tensors that vectors cannot address aligned): element by element,
// i is the flat index over the interior extents, innermost first.  With vectors,
// every row (the `width` contiguous interior elements) is padded to `spr`
// vectors and i counts the elements of the padded rows: vector k of a row
// starts at element min(k * VEC, width - VEC), so the last vector of a row that
// is no multiple of VEC long overlaps the one before it instead of running into
// the next row, and every vector is contiguous in every tensor of the launch.
// The `skip` leading elements of such a vector belong to its neighbour:
// reductions leave them out; elementwise kernels store them twice (the same
// values) where the output shares no memory with an input, else one by one.
struct TensorMap
{
    int64_t stride_n, stride_c;
    FastDiv w, h;     // interior extents of spatial dimensions 0 and 1 (strided layout)
    uint32_t sy, sz;  // strides of spatial dimensions 1 and 2 (strided layout); the host rejects larger ones
    FastDiv spr;      // vectors a row is padded to (strided layout with vectors)
    uint32_t width;   // elements of a row (strided layout with vectors)
};

template <bool STRIDED>
__host__ __device__ __forceinline__ size_t seg_offset(const TensorMap& m, size_t i)
{
    if constexpr (!STRIDED)
    {
        return i;
    }
    else
    {
        const uint32_t t = fastdiv(static_cast<uint32_t>(i), m.w);
        const uint32_t x = static_cast<uint32_t>(i) - t * m.w.divisor;
        const uint32_t z = fastdiv(t, m.h);
        const uint32_t y = t - z * m.h.divisor;
        return x + y * static_cast<size_t>(m.sy) + z * static_cast<size_t>(m.sz);
    }
}

// Where the vector at a padded index lies: the row of the segment and the row
// element its first lane holds.  Worked out once per vector from one map of the
// launch (all maps of a launch share extents and padding) and then applied to
// every tensor through that tensor's own strides.
// Vector k of a row starts at element min(k * VEC, width - VEC); `skip` leading
// elements belong to the vector before it.
struct Place
{
    uint32_t y, z; // the row within its segment
    int first;     // row element of the first lane
    uint32_t skip; // leading elements that the vector before owns
};

// Row (y, z) of the vector at padded index i (a multiple of VEC); returns the vector's index within the row.
template <int VEC>
__host__ __device__ __forceinline__ uint32_t row_split(const TensorMap& m, size_t i, Place* pl)
{
    const uint32_t slot = static_cast<uint32_t>(i) / VEC;
    const uint32_t r = fastdiv(slot, m.spr);
    pl->z = fastdiv(r, m.h);
    pl->y = r - pl->z * m.h.divisor;
    return slot - r * m.spr.divisor;
}

__host__ __device__ __forceinline__ size_t row_offset(const TensorMap& m, const Place& pl)
{
    return static_cast<size_t>(pl.y) * m.sy + static_cast<size_t>(pl.z) * m.sz;
}

template <int VEC>
__host__ __device__ __forceinline__ void place_vector(const TensorMap& m, uint32_t k, Place* pl)
{
    const uint32_t x = k * VEC, last = m.width - VEC;
    pl->first = static_cast<int>(x > last ? last : x);
    pl->skip = x > last ? x - last : 0;
}

struct ShortGeometry
{
    int num_samples, num_channels, spatial;
    int row;                // elements that are contiguous in every tensor of the launch: the
                            // whole segment, or a row of it when some tensor has halos inside
    int slots_per_row;      // vectors a row is padded to
    int slots;              // vectors a segment is padded to: its rows * slots_per_row
    int rows_per_plane;     // rows in a plane of the segment (launches that go row by row)
    int rows;               // rows of lanes, each on samples of its own
    int channels_per_group; // whole channels one workgroup serves: kBlockSize / rows / slots
    int samples_per_group;  // samples one workgroup walks through (the second grid dimension counts these ranges)
};

// One tensor of a short-segment launch: where sample n, channel c starts and
// where the rows of its segment lie.
struct ShortTensor
{
    int64_t stride_n, stride_c;
    int h;          // rows per plane (interior extent of spatial dimension 1)
    int64_t sy, sz; // strides of spatial dimensions 1 and 2
};

enum ShortTail : int
{
    kTailNone = 0,    // segments are whole vectors
    kTailOverlap = 1, // the last vector of a segment overlaps the one before it
    kTailScalar = 2   // segments shorter than a vector
};

struct ShortLane
{
    int row;    // row of lanes: its samples are row, row + rows, ... of the workgroup's range
    int q;      // channel within the workgroup's window
    int slot;   // slot of the channel's segment
    int c;      // channel
    int line;   // row of the segment the slot lies in
    int first;  // first element of the slot's vector within its row
    int valid;  // elements the slot owns; 0: an idle lane
    int skip;   // leading elements of its vector that the slot before it owns (kTailOverlap)
    bool heads; // first lane of its channel in its row
    bool leads; // first lane of its channel in row 0
};

template <int VEC, int TAIL>
__host__ __device__ __forceinline__ ShortLane short_lane(const ShortGeometry& g, int thread, int window)
{
    ShortLane l;
    const int lanes_per_row = kBlockSize / g.rows;
    l.row = thread / lanes_per_row;
    const int t = thread - l.row * lanes_per_row;
    l.q = t / g.slots;
    const int v = t - l.q * g.slots;
    l.slot = v;
    l.c = window * g.channels_per_group + l.q;
    l.line = v / g.slots_per_row;
    const int k = v - l.line * g.slots_per_row;
    const int left = g.row - k * VEC;
    const bool active = l.q < g.channels_per_group && l.c < g.num_channels;
    l.valid = active ? (left < VEC ? left : VEC) : 0;
    l.skip = TAIL == kTailOverlap && active ? VEC - l.valid : 0;
    l.first = k * VEC - l.skip;
    l.heads = active && v == 0;
    l.leads = l.heads && l.row == 0;
    return l;
}

// Whether element j of the lane's vector is one the lane owns.
template <int VEC, int TAIL>
__host__ __device__ __forceinline__ bool slot_owns(const ShortLane& l, int j)
{
    if constexpr (TAIL == kTailNone)
        return true;
    else if constexpr (TAIL == kTailOverlap)
        return j >= l.skip;
    else
        return j < l.valid;
}

// Where a lane's slot starts in one tensor, relative to the start of the
// (sample, channel) segment.  The lane's place in the segment never changes, so
// this is worked out once.
__host__ __device__ __forceinline__ int slot_offset(const ShortLane& l, const ShortTensor& t)
{
    const int z = l.line / t.h;
    const int y = l.line - z * t.h;
    return static_cast<int>(l.first + y * t.sy + z * t.sz);
}

// The real (allocated) local tensor of the halo-clearing kernels: they walk
// every cell of a (sample, channel) segment, interior and halo alike.
struct RealBox
{
    FastDiv wr, hr;        // real extents of spatial dimensions 0 and 1
    uint32_t lo[3], hi[3]; // interior: lo <= index < hi, per spatial dimension (real coordinates)
};

// Whether the elements i ... i + VEC - 1 of a real segment are interior ones.
template <int VEC>
__host__ __device__ __forceinline__ void interior_mask(const RealBox& b, uint32_t i, bool (&inside)[VEC])
{
    uint32_t t = fastdiv(i, b.wr);
    uint32_t x = i - t * b.wr.divisor;
    uint32_t z = fastdiv(t, b.hr);
    uint32_t y = t - z * b.hr.divisor;
#pragma unroll
    for (int j = 0; j < VEC; ++j)
    {
        inside[j] = x >= b.lo[0] && x < b.hi[0] && y >= b.lo[1] && y < b.hi[1] && z >= b.lo[2] && z < b.hi[2];
        if (++x == b.wr.divisor)
        {
            x = 0;
            if (++y == b.hr.divisor)
            {
                y = 0;
                ++z;
            }
        }
    }
}

} // namespace bn
} // namespace h2x

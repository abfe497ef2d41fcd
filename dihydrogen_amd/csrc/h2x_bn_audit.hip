// Launch audit of the batch-normalisation entry points: host code only, no GPU
// call.  h2x_bn_audit has an entry point plan its launches into a log
// (h2x_bn_plan.hpp) and then plays every workgroup and lane of every planned
// launch on the CPU through the index maps the kernels themselves use
// (h2x_bn_maps.hpp), counting per tensor what is loaded and stored.  Against
// the interior of each tensor, enumerated independently from its shape and
// strides, this shows whether a launch touches anything but interior elements,
// leaves one out, or has two lanes own the same one.
//
// The loops below follow the kernels' loops over chunks, vectors and samples:
//   dense / strided family, reductions (bn_sums_kernel, bn_backprop1_kernel):
//     grid (groups, C); a workgroup takes units blockIdx.x, + gridDim.x, ...;
//     unit = (sample, chunk); vectors i = begin, begin + VEC, ... with
//     i + VEC <= end.
//   dense / strided family, elementwise (bn_apply_kernel, bn_backprop2_kernel):
//     workgroup b = (segment, chunk), segment = (sample, channel), same vectors.
//   short family: lane = short_lane(thread, window); reductions walk samples
//     first + row, + rows, ...; elementwise kernels every sample of the range.
//   halo-clearing kernel (bn_clearing_kernel): workgroup b = (segment, chunk)
//     over the real tensor, vectors as above, interior_mask per vector.
#include "h2x_bn_plan.hpp"

#include <algorithm>
#include <cstring>
#include <type_traits>
#include <vector>

namespace h2x
{
namespace
{

using namespace bn;

// What the walk counts for one tensor of one launch.
struct TensorCount
{
    const h2x_tensor_geometry* geometry = nullptr;
    std::vector<uint8_t> interior; // 1: an interior element lives at this offset from the base pointer
    std::vector<uint8_t> owned;    // times a lane owned the element (saturating)
    uint64_t loads = 0, stores = 0, outside = 0;

    void prepare(const h2x_tensor_geometry* g)
    {
        geometry = g;
        loads = stores = outside = 0;
        int64_t span = 1;
        bool empty = false;
        for (int d = 0; d < g->num_dims; ++d)
        {
            if (g->local_shape[d] == 0)
                empty = true;
            span += (g->local_shape[d] - 1) * g->strides[d];
        }
        if (empty)
            span = 0;
        interior.assign(static_cast<size_t>(span), 0);
        owned.assign(static_cast<size_t>(span), 0);
        if (empty)
            return;
        // every index of the local shape, innermost first: independent of the kernels' maps
        int64_t idx[H2X_MAX_DIMS] = {};
        while (true)
        {
            int64_t off = 0;
            for (int d = 0; d < g->num_dims; ++d)
                off += idx[d] * g->strides[d];
            interior[static_cast<size_t>(off)] = 1;
            int d = 0;
            for (; d < g->num_dims; ++d)
            {
                if (++idx[d] < g->local_shape[d])
                    break;
                idx[d] = 0;
            }
            if (d == g->num_dims)
                break;
        }
    }

    void touch(int64_t off, bool store, bool owns)
    {
        if (store)
            ++stores;
        else
            ++loads;
        if (off < 0 || off >= static_cast<int64_t>(interior.size()) || !interior[static_cast<size_t>(off)])
        {
            ++outside;
            return;
        }
        uint8_t& n = owned[static_cast<size_t>(off)];
        if (owns && n < 255)
            ++n;
    }

    void finish(h2x_bn_audit_tensor* out) const
    {
        out->loads = loads;
        out->stores = stores;
        out->outside = outside;
        out->missed = out->owned_twice = 0;
        for (size_t i = 0; i < interior.size(); ++i)
        {
            if (!interior[i])
                continue;
            if (owned[i] == 0)
                ++out->missed;
            else if (owned[i] > 1)
                ++out->owned_twice;
        }
    }
};

bool is_reduction(int kernel)
{
    return kernel == kKernelSums || kernel == kKernelBackprop1;
}

template <int VEC, bool STRIDED>
void walk_long(const LaunchRecord& r, TensorCount* count)
{
    const auto visit_chunk = [&](size_t n, int c, int k) {
        const size_t begin = static_cast<size_t>(k) * r.chunk;
        const size_t end = std::min(begin + r.chunk, r.spatial);
        // the kernels place a vector by the map of the output (elementwise) or of x (reductions)
        const TensorMap& placing = r.map[r.last_is_output ? r.num_tensors - 1 : 0];
        for (size_t i = begin; i + VEC <= end; i += VEC)
        {
            Place pl{0, 0, 0, 0};
            if constexpr (STRIDED && VEC > 1)
                place_vector<VEC>(placing, row_split<VEC>(placing, i, &pl), &pl);
            for (int t = 0; t < r.num_tensors; ++t)
            {
                const TensorMap& m = r.map[t];
                size_t off;
                if constexpr (!STRIDED || VEC == 1)
                    off = seg_offset<STRIDED>(m, i);
                else
                    off = row_offset(m, pl) + pl.first;
                const int64_t base = static_cast<int64_t>(n) * m.stride_n
                                     + static_cast<int64_t>(c) * m.stride_c + static_cast<int64_t>(off);
                const bool output = r.last_is_output && t == r.num_tensors - 1;
                for (int j = 0; j < VEC; ++j)
                {
                    const bool owns = j >= static_cast<int>(pl.skip);
                    if (output && !(pl.skip == 0 || r.rewrite) && !owns)
                        continue; // store_out leaves the shared elements to their owner
                    count[t].touch(base + j, output, owns);
                }
            }
        }
    };
    if (is_reduction(r.kernel))
    {
        // grid (groups, C); every unit is taken by workgroup unit mod gridDim.x of its channel
        for (int c = 0; c < static_cast<int>(r.grid_y); ++c)
            for (unsigned int unit = 0; unit < r.num_units && r.grid_x > 0; ++unit)
                visit_chunk(unit / r.chunks_per_seg, c, static_cast<int>(unit % r.chunks_per_seg));
    }
    else
    {
        for (unsigned int b = 0; b < r.grid_x; ++b)
        {
            const size_t seg = b / r.chunks_per_seg;
            visit_chunk(seg / r.num_channels, static_cast<int>(seg % r.num_channels),
                        static_cast<int>(b % r.chunks_per_seg));
        }
    }
}

template <int VEC, int TAIL>
void walk_short(const LaunchRecord& r, TensorCount* count)
{
    const ShortGeometry& g = r.geometry;
    const bool reduction = is_reduction(r.kernel);
    for (unsigned int bx = 0; bx < r.grid_x; ++bx)
        for (unsigned int by = 0; by < r.grid_y; ++by)
            for (int thread = 0; thread < kBlockSize; ++thread)
            {
                const ShortLane l = short_lane<VEC, TAIL>(g, thread, static_cast<int>(bx));
                if (l.valid == 0)
                    continue;
                const int first = static_cast<int>(by) * g.samples_per_group;
                const int end = std::min(first + g.samples_per_group, g.num_samples);
                const int step = reduction ? g.rows : 1;
                for (int n = first + (reduction ? l.row : 0); n < end; n += step)
                {
                    for (int t = 0; t < r.num_tensors; ++t)
                    {
                        const ShortTensor& st = r.tensor[t];
                        const int64_t base = static_cast<int64_t>(n) * st.stride_n
                                             + static_cast<int64_t>(l.c) * st.stride_c
                                             + slot_offset(l, st);
                        const bool output = r.last_is_output && t == r.num_tensors - 1;
                        for (int j = 0; j < VEC; ++j)
                        {
                            const bool owns = slot_owns<VEC, TAIL>(l, j);
                            bool moved;
                            if (output) // store_slot
                                moved = TAIL == kTailNone
                                        || (TAIL == kTailOverlap && (r.rewrite || l.skip == 0)) || owns;
                            else // load_slot
                                moved = TAIL != kTailScalar || (j < VEC - 1 && j < l.valid);
                            if (moved)
                                count[t].touch(base + j, output, owns);
                        }
                    }
                }
            }
}

template <int VEC>
void walk(const LaunchRecord& r, TensorCount* count)
{
    if (r.family == kFamilyShort)
    {
        if (r.tail == kTailNone)
            walk_short<VEC, kTailNone>(r, count);
        else if (r.tail == kTailOverlap)
            walk_short<VEC, kTailOverlap>(r, count);
        else
            walk_short<VEC, kTailScalar>(r, count);
    }
    else if (r.family == kFamilyStrided)
    {
        if (r.vec > 1)
            walk_long<VEC, true>(r, count);
        else
            walk_long<1, true>(r, count);
    }
    else
    {
        if (r.vec > 1)
            walk_long<VEC, false>(r, count);
        else
            walk_long<1, false>(r, count);
    }
}

} // namespace
} // namespace h2x

using namespace h2x;

extern "C" int h2x_bn_audit(h2x_bn_stage stage, h2x_dtype dtype, int num_samples,
                            const h2x_tensor_geometry* const* geometry, const uint64_t* address,
                            h2x_bn_audit_report* report)
{
    if (!geometry || !address || !report || (dtype != H2X_F32 && dtype != H2X_F64))
        return H2X_ERR_INVALID_ARGUMENT;
    int tensors;
    switch (stage)
    {
    case H2X_BN_STAGE_SUMS: tensors = 1; break;
    case H2X_BN_STAGE_NORMALIZE:
    case H2X_BN_STAGE_BACKPROP1:
    case H2X_BN_STAGE_FORWARD_LOCAL: tensors = 2; break;
    case H2X_BN_STAGE_BACKPROP2:
    case H2X_BN_STAGE_BACKWARD_LOCAL: tensors = 3; break;
    default: return H2X_ERR_INVALID_ARGUMENT;
    }
    for (int t = 0; t < tensors; ++t)
        if (!geometry[t] || geometry[t]->num_dims < 3 || geometry[t]->num_dims > 5)
            return H2X_ERR_INVALID_ARGUMENT;
    std::memset(report, 0, sizeof(*report));

    // Pointers that are never followed: the entry points only look at their
    // alignment and at whether x and dx share memory.
    void* const param = reinterpret_cast<void*>(static_cast<uintptr_t>(4096));
    const auto ptr = [&](int t) { return reinterpret_cast<void*>(static_cast<uintptr_t>(address[t])); };
    const auto dense = [&](int t, int* c, size_t* s, size_t* real) {
        // the two-launch entry points take (samples, channels, spatial, real) only
        const h2x_tensor_geometry* g = geometry[t];
        if (g->num_dims != 3 || g->strides[0] != 1 || g->strides[2] != g->strides[1] * g->local_shape[1])
            return false;
        *s = static_cast<size_t>(g->local_shape[0]);
        *c = static_cast<int>(g->local_shape[1]);
        *real = static_cast<size_t>(g->strides[1]);
        return g->local_shape[2] == num_samples;
    };

    LaunchLog log;
    LaunchLog* before = install_launch_log(&log);
    int err = H2X_ERR_INVALID_ARGUMENT;
    switch (stage)
    {
    case H2X_BN_STAGE_SUMS:
        err = h2x_bn_channel_sums_and_sqsums_strided(dtype, num_samples, geometry[0], ptr(0), param,
                                                     param, param, nullptr);
        break;
    case H2X_BN_STAGE_NORMALIZE:
        err = h2x_bn_batch_normalization_strided(dtype, num_samples, geometry[0], geometry[1], ptr(0),
                                                 param, param, param, param, ptr(1), 1e-5, nullptr);
        break;
    case H2X_BN_STAGE_BACKPROP1:
        err = h2x_bn_backprop1_strided(dtype, num_samples, geometry[0], geometry[1], ptr(0), ptr(1),
                                       param, param, param, param, param, param, param, 1e-5, param,
                                       nullptr);
        break;
    case H2X_BN_STAGE_BACKPROP2:
        err = h2x_bn_backprop2_strided(dtype, num_samples, 2, geometry[0], geometry[1], geometry[2],
                                       ptr(0), ptr(1), param, param, param, param, param, ptr(2),
                                       1e-5, nullptr);
        break;
    case H2X_BN_STAGE_FORWARD_LOCAL:
    {
        int c, c2;
        size_t s, s2, xr, yr;
        if (dense(0, &c, &s, &xr) && dense(1, &c2, &s2, &yr) && c == c2 && s == s2)
            err = h2x_bn_forward_local(dtype, num_samples, c, s, xr, yr, ptr(0), param, param, 2, 0.9,
                                       1e-5, param, param, param, param, ptr(1), param, nullptr);
        else
            err = h2x_bn_forward_local_strided(dtype, num_samples, geometry[0], geometry[1], ptr(0), param,
                                               param, 2, 0.9, 1e-5, param, param, param, param, ptr(1),
                                               param, nullptr);
        break;
    }
    case H2X_BN_STAGE_BACKWARD_LOCAL:
    {
        int c, c2, c3;
        size_t s, s2, s3, xr, dr, orl;
        if (dense(0, &c, &s, &xr) && dense(1, &c2, &s2, &dr) && dense(2, &c3, &s3, &orl) && c == c2
            && c == c3 && s == s2 && s == s3)
            err = h2x_bn_backward_local(dtype, num_samples, c, s, xr, dr, orl, 2, ptr(0), ptr(1), param,
                                        param, param, param, param, param, param, ptr(2), 1e-5,
                                        param, nullptr);
        else
            err = h2x_bn_backward_local_strided(dtype, num_samples, 2, geometry[0], geometry[1], geometry[2],
                                                ptr(0), ptr(1), param, param, param, param, param, param,
                                                param, ptr(2), 1e-5, param, nullptr);
        break;
    }
    }
    install_launch_log(before);
    if (err)
        return err;

    const int channels = static_cast<int>(geometry[0]->local_shape[geometry[0]->num_dims - 2]);
    report->workspace_bytes = h2x_bn_workspace_bytes(channels);
    report->num_launches = static_cast<int32_t>(log.records.size());
    if (log.records.size() > H2X_BN_AUDIT_MAX_LAUNCHES)
        return H2X_ERR_TOO_LARGE;
    std::vector<TensorCount> count(kMaxLaunchTensors);
    for (size_t i = 0; i < log.records.size(); ++i)
    {
        const LaunchRecord& r = log.records[i];
        h2x_bn_audit_launch& out = report->launch[i];
        out.kernel = r.kernel;
        out.family = r.family;
        out.vector_width = r.vec;
        out.tail = r.tail;
        out.folded = r.folded;
        out.fused = r.fused;
        out.grid_x = r.grid_x;
        out.grid_y = r.grid_y;
        out.num_tensors = r.num_tensors;
        // bytes of partial sums the launch may write: every (channel, group, sum) slot it can address
        if (is_reduction(r.kernel) && r.partials)
            out.partials_bytes = static_cast<uint64_t>(r.num_channels)
                                 * (r.family == kFamilyShort ? r.grid_y : r.grid_x) * r.num_sums
                                 * sizeof(double);
        out.partials_capacity = static_cast<uint64_t>(r.num_channels) * r.groups_max * r.num_sums
                                * sizeof(double);
        if (r.kernel > kKernelBackprop2)
            continue;
        for (int t = 0; t < r.num_tensors; ++t)
            count[t].prepare(geometry[t]);
        if (dtype == H2X_F32)
            walk<4>(r, count.data());
        else
            walk<2>(r, count.data());
        for (int t = 0; t < r.num_tensors; ++t)
            count[t].finish(&out.tensor[t]);
    }
    return H2X_SUCCESS;
}

extern "C" int h2x_bn_audit_clearing(int backward, h2x_dtype dtype, const h2x_haloed_geometry* geometry,
                                     const uint64_t* address, h2x_bn_audit_report* report)
{
    if (!geometry || !address || !report || (dtype != H2X_F32 && dtype != H2X_F64))
        return H2X_ERR_INVALID_ARGUMENT;
    std::memset(report, 0, sizeof(*report));
    void* const param = reinterpret_cast<void*>(static_cast<uintptr_t>(4096));
    const auto ptr = [&](int t) { return reinterpret_cast<void*>(static_cast<uintptr_t>(address[t])); };
    LaunchLog log;
    LaunchLog* before = install_launch_log(&log);
    const int err = backward ? h2x_bn_backprop2_clearing(dtype, 2, geometry, ptr(0), ptr(1), param, param, param,
                                                         param, param, ptr(2), 1e-5, nullptr)
                             : h2x_bn_batch_normalization_clearing(dtype, geometry, ptr(0), param, param, param,
                                                                   param, ptr(1), 1e-5, nullptr);
    install_launch_log(before);
    if (err)
        return err;
    report->num_launches = static_cast<int32_t>(log.records.size());
    if (log.records.size() > H2X_BN_AUDIT_MAX_LAUNCHES)
        return H2X_ERR_TOO_LARGE;
    for (size_t l = 0; l < log.records.size(); ++l)
    {
        const LaunchRecord& r = log.records[l];
        h2x_bn_audit_launch& out = report->launch[l];
        out.kernel = r.kernel;
        out.family = r.family;
        out.vector_width = r.vec;
        out.grid_x = r.grid_x;
        out.grid_y = r.grid_y;
        out.num_tensors = r.num_tensors;
        if (r.kernel != kKernelClearing)
            return H2X_ERR_UNSUPPORTED;
        // the interior of one real segment, from the local shape and the halo widths alone
        const int ns = geometry->num_dims - 2;
        int64_t real_extent[3] = {1, 1, 1}, lo[3] = {0, 0, 0}, len[3] = {1, 1, 1};
        for (int d = 0; d < ns; ++d)
        {
            real_extent[d] = geometry->real_shape[d];
            lo[d] = geometry->lower_halo[d];
            len[d] = geometry->local_shape[d];
        }
        std::vector<uint8_t> interior(r.real, 0);
        for (int64_t z = 0; z < len[2]; ++z)
            for (int64_t y = 0; y < len[1]; ++y)
                for (int64_t x = 0; x < len[0]; ++x)
                    interior[static_cast<size_t>(((z + lo[2]) * real_extent[1] + (y + lo[1])) * real_extent[0]
                                                 + (x + lo[0]))] = 1;
        const size_t segments = static_cast<size_t>(r.num_samples) * r.num_channels;
        const size_t cells = segments * r.real;
        std::vector<uint8_t> stored(cells, 0);
        h2x_bn_audit_tensor* t = out.tensor;
        const int last = r.num_tensors - 1;
        const auto play = [&](auto vec_tag) {
            constexpr int VEC = decltype(vec_tag)::value;
            for (unsigned int b = 0; b < r.grid_x; ++b)
            {
                const size_t seg = b / r.chunks_per_seg;
                const size_t begin = static_cast<size_t>(b % r.chunks_per_seg) * r.chunk;
                const size_t end = std::min(begin + r.chunk, r.real);
                for (size_t i = begin; i + VEC <= end; i += VEC)
                {
                    bool inside[VEC];
                    interior_mask<VEC>(r.box, static_cast<uint32_t>(i), inside);
                    for (int j = 0; j < VEC; ++j)
                    {
                        const size_t at = seg * r.real + i + j;
                        const bool beyond = seg >= segments || i + j >= r.real;
                        for (int k = 0; k < last; ++k) // x (and dy): halo cells are loaded and ignored
                        {
                            ++t[k].loads;
                            t[k].outside += beyond;
                        }
                        ++t[last].stores;
                        if (beyond)
                        {
                            ++t[last].outside;
                            continue;
                        }
                        t[last].outside += inside[j] != (interior[i + j] != 0);
                        if (stored[at] < 255)
                            ++stored[at];
                    }
                }
            }
        };
        if (r.vec == 4)
            play(std::integral_constant<int, 4>());
        else if (r.vec == 2)
            play(std::integral_constant<int, 2>());
        else
            play(std::integral_constant<int, 1>());
        for (size_t i = 0; i < cells; ++i)
        {
            t[last].missed += stored[i] == 0;
            t[last].owned_twice += stored[i] > 1;
        }
    }
    return H2X_SUCCESS;
}

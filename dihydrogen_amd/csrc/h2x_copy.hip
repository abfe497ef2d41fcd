// Box copy engine for gfx950: halo pack/unpack/clear and tensor-shuffler
// pack/unpack, with the C entry points of both.
//
// Both operations move a rectangular sub-box of a strided tensor to or from a
// contiguous buffer that holds the box in natural (innermost-first) order of
// the box's own extents:
//   - a halo strip is the box {shape[0..dim-1], width, shape[dim+1..]} at the
//     strip's start along `dim` (legacy/include/distconv/tensor/halo_cuda.hpp:34-88);
//   - the part of a local tensor that goes to one peer rank of a shuffle is
//     the intersection box of the two ranks' regions, and the order
//     find_destination produces inside a peer's chunk is the natural order of
//     that box (legacy/src/tensor/shuffle_mpi_cuda.cu:42-98).
// The host reduces every box to as few dimensions as possible (extent-1
// dimensions vanish, dimensions that are contiguous in the tensor merge), so a
// halo strip becomes "outer runs of `run` contiguous elements" and the device
// index arithmetic is one or two multiply-high divisions per 16 bytes moved,
// instead of a division chain per element (halo_cuda.hpp:47-81) or a search
// per element (shuffle_mpi_cuda.cu:70-84).  Up to kMaxBoxes boxes -- both
// sides of a dimension, all peers of a rank, several virtual ranks -- share a
// launch; their descriptors travel in the kernel arguments, so nothing is
// allocated or copied to set a launch up.
//
// A fourth mode moves a strip straight from one tensor into another (the
// neighbour's interior strip into this rank's halo) when both live on the same
// device: pack and unpack of a halo exchange without the buffer in between.
#include "h2x_copy_kernel.hpp"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <new>
#include <vector>

namespace h2x
{
namespace copy
{

// ---- launches of the identity instantiations -------------------------------------

namespace
{

template <typename T, int VEC, bool SPARSE>
int launch_mode(const LaunchShape& s, const BoxBatch& batch)
{
    switch (s.mode)
    {
    case kPack: return run_box_copy<T, VEC, OpId, SPARSE, kPack, false>(s.grid, s.stream, batch, OpId());
    case kUnpack: return run_box_copy<T, VEC, OpId, SPARSE, kUnpack, false>(s.grid, s.stream, batch, OpId());
    case kClear: return run_box_copy<T, VEC, OpId, SPARSE, kClear, false>(s.grid, s.stream, batch, OpId());
    case kTransfer: return run_box_copy<T, VEC, OpId, SPARSE, kTransfer, false>(s.grid, s.stream, batch, OpId());
    default: return H2X_ERR_UNSUPPORTED;
    }
}

template <typename T, int VEC>
int launch_sparse(const LaunchShape& s, const BoxBatch& batch)
{
    return s.sparse ? launch_mode<T, VEC, true>(s, batch) : launch_mode<T, VEC, false>(s, batch);
}

template <typename T, int VEC>
int launch_table_mode(const LaunchShape& s, const TableBatch& batch)
{
    if (s.mode == kPack)
        return run_box_copy<T, VEC, OpId, false, kPack, true>(s.grid, s.stream, batch, OpId());
    if (s.mode == kUnpack)
        return run_box_copy<T, VEC, OpId, false, kUnpack, true>(s.grid, s.stream, batch, OpId());
    return H2X_ERR_UNSUPPORTED;
}

// The audit the calling thread has opened with h2x_copy_audit_begin.
thread_local Audit* t_audit = nullptr;

} // namespace

Audit* current_audit()
{
    return t_audit;
}

int launch_identity(const LaunchShape& s, const BoxBatch& batch)
{
    switch (s.elem_size * 16 + s.vec)
    {
    case 2 * 16 + 8: return launch_sparse<uint16_t, 8>(s, batch);
    case 2 * 16 + 4: return launch_sparse<uint16_t, 4>(s, batch);
    case 2 * 16 + 2: return launch_sparse<uint16_t, 2>(s, batch);
    case 2 * 16 + 1: return launch_sparse<uint16_t, 1>(s, batch);
    case 4 * 16 + 4: return launch_sparse<uint32_t, 4>(s, batch);
    case 4 * 16 + 2: return launch_sparse<uint32_t, 2>(s, batch);
    case 4 * 16 + 1: return launch_sparse<uint32_t, 1>(s, batch);
    case 8 * 16 + 2: return launch_sparse<uint64_t, 2>(s, batch);
    case 8 * 16 + 1: return launch_sparse<uint64_t, 1>(s, batch);
    }
    return H2X_ERR_UNSUPPORTED;
}

int launch_tables(const LaunchShape& s, const TableBatch& batch)
{
    switch (s.elem_size * 16 + s.vec)
    {
    case 2 * 16 + 8: return launch_table_mode<uint16_t, 8>(s, batch);
    case 2 * 16 + 4: return launch_table_mode<uint16_t, 4>(s, batch);
    case 2 * 16 + 2: return launch_table_mode<uint16_t, 2>(s, batch);
    case 2 * 16 + 1: return launch_table_mode<uint16_t, 1>(s, batch);
    case 4 * 16 + 4: return launch_table_mode<uint32_t, 4>(s, batch);
    case 4 * 16 + 2: return launch_table_mode<uint32_t, 2>(s, batch);
    case 4 * 16 + 1: return launch_table_mode<uint32_t, 1>(s, batch);
    case 8 * 16 + 2: return launch_table_mode<uint64_t, 2>(s, batch);
    case 8 * 16 + 1: return launch_table_mode<uint64_t, 1>(s, batch);
    }
    return H2X_ERR_UNSUPPORTED;
}

} // namespace copy

using namespace copy;

namespace
{

// ---- host: box reduction ------------------------------------------------------

struct HostBox
{
    int nd = 0;
    int64_t extent[kMaxBoxDims];
    int64_t stride[kMaxBoxDims];
    int64_t stride_src[kMaxBoxDims] = {}; // transfers: strides of the source tensor
    int64_t tensor_offset = 0; // elements from the tensor pointer to the box origin
    int64_t buffer_offset = 0; // elements from the buffer (transfers: source tensor) pointer
    int64_t count = 1;
    bool transfer = false;
};

// Drops extent-1 dimensions and merges neighbours that are contiguous in the
// tensor (for a transfer: in both tensors); the natural order of the reduced
// box is the natural order of the original one.
HostBox reduce_box(int nd, const int64_t* extent, const int64_t* stride, int64_t tensor_offset,
                   int64_t buffer_offset, const int64_t* stride_src = nullptr)
{
    HostBox h;
    h.tensor_offset = tensor_offset;
    h.buffer_offset = buffer_offset;
    h.transfer = stride_src != nullptr;
    for (int i = 0; i < nd; ++i)
    {
        h.count *= extent[i];
        if (extent[i] == 1)
            continue;
        const bool merge =
            h.nd > 0 && stride[i] == h.stride[h.nd - 1] * h.extent[h.nd - 1]
            && (!stride_src || stride_src[i] == h.stride_src[h.nd - 1] * h.extent[h.nd - 1]);
        if (merge)
        {
            h.extent[h.nd - 1] *= extent[i];
        }
        else
        {
            h.extent[h.nd] = extent[i];
            h.stride[h.nd] = stride[i];
            h.stride_src[h.nd] = stride_src ? stride_src[i] : 0;
            ++h.nd;
        }
    }
    if (h.nd == 0)
    {
        h.nd = 1;
        h.extent[0] = 1;
        h.stride[0] = 1;
        h.stride_src[0] = 1;
    }
    return h;
}

// Vector width (elements, at most 16 bytes) of a box.  The image side must be
// aligned to it.  Runs that are a multiple of it move in whole vectors; longer
// runs of any other length still move in 16-byte vectors indexed from the
// image side, and the few vectors that straddle the end of a run are split
// (`ragged`): a 130-element row is 32 vectors and one straddler instead of 65
// 8-byte pieces.
constexpr int64_t kMinRaggedRun = 16; // shorter runs: straddlers would be the rule

int box_vector(const HostBox& h, int elem_size, const void* buffer, bool allow_ragged, bool* ragged)
{
    *ragged = false;
    int v = 16 / elem_size;
    if (h.stride[0] != 1 || (h.transfer && h.stride_src[0] != 1))
        return 1;
    // a transfer has no image side: both tensors take unaligned vectors
    auto buffer_ok = [&](int w) {
        return h.transfer
               || (h.buffer_offset % w == 0
                   && reinterpret_cast<uintptr_t>(buffer) % (static_cast<size_t>(w) * elem_size) == 0);
    };
    if (allow_ragged && v > 1 && h.extent[0] % v != 0 && h.extent[0] >= kMinRaggedRun && buffer_ok(v))
    {
        *ragged = true;
        return v;
    }
    while (v > 1)
    {
        if (h.extent[0] % v == 0 && buffer_ok(v))
            break;
        v /= 2;
    }
    return v;
}

// sparse: every run is shorter than a cache line and the runs are apart
bool box_is_sparse(const HostBox& h, int elem_size)
{
    return h.nd > 1 ? h.extent[0] * h.stride[0] * elem_size < 128
                    : (h.stride[0] != 1 && h.extent[0] > 1);
}

// Two boxes of identical geometry whose origins are `delta` elements apart
// share no element if, with every stride a multiple of the row pitch, the
// shift within a row is at least one run and at most a pitch less one run.
// (A sufficient test: false means "not known to be disjoint".)
bool translated_boxes_are_disjoint(const HostBox& h, int64_t delta)
{
    int64_t run = 1, pitch = 0;
    int first = 0;
    if (h.stride[0] == 1)
    {
        run = h.extent[0];
        first = 1;
    }
    for (int i = first; i < h.nd; ++i)
        if (h.extent[i] > 1)
            pitch = pitch == 0 ? std::llabs(h.stride[i]) : std::min<int64_t>(pitch, std::llabs(h.stride[i]));
    if (delta < 0)
        delta = -delta;
    if (pitch == 0) // a single run
        return delta >= run;
    for (int i = first; i < h.nd; ++i)
        if (h.extent[i] > 1 && h.stride[i] % pitch != 0)
            return false;
    const int64_t shift = delta % pitch;
    return shift >= run && shift <= pitch - run;
}

bool same_geometry(const HostBox& a, const HostBox& b)
{
    if (a.nd != b.nd || a.count != b.count)
        return false;
    for (int i = 0; i < a.nd; ++i)
        if (a.extent[i] != b.extent[i] || a.stride[i] != b.stride[i]
            || a.stride_src[i] != b.stride_src[i])
            return false;
    return true;
}

// Geometry of a device descriptor; pointers and flags are the caller's.
void fill_box(Box* b, const HostBox& h)
{
    for (int i = 0; i < kMaxBoxDims; ++i)
    {
        b->stride[i] = i < h.nd ? h.stride[i] : 0;
        b->stride_src[i] = i < h.nd ? h.stride_src[i] : 0;
        b->div[i] = make_fastdiv(i < h.nd ? static_cast<uint32_t>(h.extent[i]) : 1u);
    }
    b->count = static_cast<uint32_t>(h.count);
    b->first_block = 0;
    b->ragged = 0;
    b->seam = 0;
    b->deep = h.nd > 3;
    b->disjoint = 0;
    b->tensor2 = nullptr;
    b->buffer2 = nullptr;
}

uint64_t box_blocks(int64_t count, int vec)
{
    const uint64_t per_block = static_cast<uint64_t>(kCopyBlock) * vec * kCopyUnroll;
    return (static_cast<uint64_t>(count) + per_block - 1) / per_block;
}

// Queues boxes whose descriptors travel in the kernel arguments and launches
// them, kMaxBoxes at a time; boxes of one launch share vector width, kind
// (sparse or dense) and mode.
struct Launcher
{
    hipStream_t stream;
    int elem_size;
    h2x_dtype dtype; // meaningful for accumulate ops only
    int op;          // h2x_halo_op
    int vec = 0;
    bool sparse = false;
    int mode = -1;
    HostBox last;    // geometry of the most recently queued box
    uint32_t num_blocks = 0;
    BoxBatch batch;

    Launcher(hipStream_t s, int es, h2x_dtype dt, int o) : stream(s), elem_size(es), dtype(dt), op(o)
    {
        batch.num_boxes = 0;
    }

    int flush()
    {
        if (batch.num_boxes == 0)
            return H2X_SUCCESS;
        // Taking turns needs one workgroup count for all boxes: the largest.  The
        // surplus workgroups of smaller boxes find nothing to do; if they would
        // more than double the grid, the boxes follow one another instead.
        batch.blocks_per_box = 0;
        uint32_t grid_blocks = num_blocks;
        if (batch.num_boxes > 1)
        {
            uint32_t most = 0;
            for (int i = 0; i < batch.num_boxes; ++i)
            {
                const uint32_t end = i + 1 < batch.num_boxes ? batch.box[i + 1].first_block : num_blocks;
                most = std::max(most, end - batch.box[i].first_block);
            }
            const uint64_t turns = static_cast<uint64_t>(most) * batch.num_boxes;
            if (turns <= 2ull * num_blocks && turns <= 0x7fffffffull)
            {
                batch.blocks_per_box = most;
                grid_blocks = static_cast<uint32_t>(turns);
            }
        }
        LaunchShape shape{elem_size, op, vec, sparse, mode, grid_blocks, stream};
        const int err = op == H2X_HALO_ID ? launch_identity(shape, batch)
                                          : launch_accumulate(shape, dtype, batch);
        batch.num_boxes = 0;
        num_blocks = 0;
        vec = 0;
        mode = -1;
        return err;
    }

    // Queues one box; launches what is queued when the batch is full or the
    // new box needs another kernel.
    int add(const HostBox& h, void* tensor, void* buffer, int box_mode)
    {
        if (h.count == 0)
            return H2X_SUCCESS;
        if (h.count >= (1ll << 31))
            return H2X_ERR_TOO_LARGE;
        const bool sp = box_is_sparse(h, elem_size);
        bool rg;
        const int v = box_vector(h, elem_size, box_mode == kClear ? nullptr : buffer, !sp, &rg);
        char* const tptr = static_cast<char*>(tensor) + h.tensor_offset * elem_size;
        char* const bptr = static_cast<char*>(buffer) + h.buffer_offset * elem_size;
        // second box of a sparse pair: same geometry and mode as the box queued last
        if (sp && batch.num_boxes > 0 && sparse && v == vec && mode == box_mode
            && batch.box[batch.num_boxes - 1].tensor2 == nullptr && same_geometry(h, last))
        {
            Box& first = batch.box[batch.num_boxes - 1];
            first.tensor2 = tptr;
            first.buffer2 = bptr;
            // one element per row on each side, and this box's element of a row
            // lies directly in front of the first box's element of the next row
            // (the RHS and the LHS halo cell at a row seam): unpacked in one store
            first.seam = box_mode == kUnpack && v == 1 && h.nd == 1
                         && tptr + elem_size == first.tensor + h.stride[0] * elem_size;
            first.disjoint = translated_boxes_are_disjoint(h, (tptr - first.tensor) / elem_size);
            return H2X_SUCCESS;
        }
        if (batch.num_boxes == kMaxBoxes
            || (batch.num_boxes > 0 && (v != vec || sp != sparse || box_mode != mode)))
        {
            const int err = flush();
            if (err != 0)
                return err;
        }
        vec = v;
        sparse = sp;
        mode = box_mode;
        last = h;
        Box& b = batch.box[batch.num_boxes];
        fill_box(&b, h);
        b.tensor = tptr;
        b.buffer = bptr;
        b.ragged = rg;
        b.first_block = num_blocks;
        const uint64_t blocks = box_blocks(h.count, v);
        if (num_blocks + blocks > 0x7fffffffull)
            return H2X_ERR_TOO_LARGE;
        num_blocks += static_cast<uint32_t>(blocks);
        ++batch.num_boxes;
        return H2X_SUCCESS;
    }
};

// The reduced boxes of one call: on the stack for the usual handful of faces,
// on the heap beyond that.
class BoxList
{
public:
    explicit BoxList(int n) : m_data(m_local)
    {
        if (n > kLocal)
        {
            m_heap.resize(static_cast<size_t>(n));
            m_data = m_heap.data();
        }
    }
    HostBox& operator[](int i) { return m_data[i]; }

private:
    static constexpr int kLocal = 32;
    HostBox m_local[kLocal];
    std::vector<HostBox> m_heap;
    HostBox* m_data;
};

int elem_size_of(h2x_dtype dtype)
{
    return dtype == H2X_F32 ? 4 : dtype == H2X_F64 ? 8 : 0;
}

// The strip of a halo face as a box over the real tensor.
int halo_box(const h2x_halo_face& f, HostBox* out, bool origin_only = false)
{
    const int nd = f.num_dims;
    if (nd < 1 || nd > H2X_MAX_DIMS || f.dim < 0 || f.dim >= nd || f.width < 0
        || (f.side != H2X_LHS && f.side != H2X_RHS))
        return H2X_ERR_INVALID_ARGUMENT;
    int64_t extent[kMaxBoxDims], stride[kMaxBoxDims];
    int64_t s = 1;
    for (int i = 0; i < nd; ++i)
    {
        if (f.real_shape[i] < 0)
            return H2X_ERR_INVALID_ARGUMENT;
        extent[i] = f.real_shape[i];
        stride[i] = s;
        s *= f.real_shape[i];
    }
    const int64_t len = f.real_shape[f.dim];
    const int64_t w = f.width;
    int64_t start;
    if (f.side == H2X_RHS)
        start = f.inner ? len - 2 * w : len - w;
    else
        start = f.inner ? w : 0;
    if (w > 0 && (start < 0 || start + w > len))
        return H2X_ERR_INVALID_ARGUMENT;
    extent[f.dim] = w;
    if (origin_only)
    {
        *out = HostBox();
        out->tensor_offset = start * stride[f.dim];
        return H2X_SUCCESS;
    }
    *out = reduce_box(nd, extent, stride, start * stride[f.dim], 0);
    return H2X_SUCCESS;
}

} // namespace
} // namespace h2x

using namespace h2x;

// ---- halo ----------------------------------------------------------------------

extern "C" size_t h2x_halo_size(int num_dims, const int64_t* real_shape, int dim, int width)
{
    size_t s = 1;
    for (int i = 0; i < num_dims; ++i)
        s *= static_cast<size_t>(i == dim ? width : real_shape[i]);
    return s;
}

extern "C" int h2x_halo_pack_or_unpack_batched(h2x_dtype dtype, const h2x_halo_face* faces,
                                               int num_faces, h2x_stream_t stream)
{
    const int es = elem_size_of(dtype);
    if (es == 0)
        return H2X_ERR_UNSUPPORTED;
    if (num_faces < 0 || (num_faces > 0 && !faces))
        return H2X_ERR_INVALID_ARGUMENT;
    // validate everything before anything is launched
    BoxList boxes(num_faces);
    unsigned int ops_present = 0;
    for (int i = 0; i < num_faces; ++i)
    {
        const int err = halo_box(faces[i], &boxes[i]);
        if (err != 0)
            return err;
        if (boxes[i].count > 0 && (!faces[i].tensor || !faces[i].buffer))
            return H2X_ERR_INVALID_ARGUMENT;
        if (boxes[i].count >= (1ll << 31))
            return H2X_ERR_TOO_LARGE;
        if (faces[i].op < H2X_HALO_ID || faces[i].op > H2X_HALO_MIN)
            return H2X_ERR_INVALID_ARGUMENT;
        ops_present |= 1u << (faces[i].is_pack ? H2X_HALO_ID : faces[i].op);
    }
    // faces with the same effective op share launches
    for (int op = H2X_HALO_ID; op <= H2X_HALO_MIN; ++op)
    {
        if (!(ops_present & (1u << op)))
            continue;
        Launcher l(as_stream(stream), es, dtype, op);
        for (int i = 0; i < num_faces; ++i)
        {
            const int eff = faces[i].is_pack ? H2X_HALO_ID : faces[i].op;
            if (eff != op)
                continue;
            const int err = l.add(boxes[i], faces[i].tensor, faces[i].buffer,
                                  faces[i].is_pack ? kPack : kUnpack);
            if (err != 0)
                return err;
        }
        const int err = l.flush();
        if (err != 0)
            return err;
    }
    return H2X_SUCCESS;
}

extern "C" int h2x_halo_pack_or_unpack(h2x_dtype dtype, void* tensor, int num_dims,
                                       const int64_t* real_shape, int dim, int side, int width,
                                       void* buffer, int is_pack, int is_reverse, int op,
                                       h2x_stream_t stream)
{
    if (width == 0)
        return H2X_SUCCESS; // halo_packing_cuda.hpp:153-154
    if (!real_shape || num_dims < 1 || num_dims > H2X_MAX_DIMS)
        return H2X_ERR_INVALID_ARGUMENT;
    h2x_halo_face f;
    std::memset(&f, 0, sizeof(f));
    f.tensor = tensor;
    f.buffer = buffer;
    for (int i = 0; i < num_dims; ++i)
        f.real_shape[i] = real_shape[i];
    f.num_dims = num_dims;
    f.dim = dim;
    f.side = side;
    f.width = width;
    f.inner = ((is_pack && !is_reverse) || (!is_pack && is_reverse)) ? 1 : 0;
    f.is_pack = is_pack ? 1 : 0;
    f.op = op;
    return h2x_halo_pack_or_unpack_batched(dtype, &f, 1, stream);
}

extern "C" int h2x_halo_clear(h2x_dtype dtype, void* tensor, int num_dims,
                              const int64_t* real_shape, int dim, int width, h2x_stream_t stream)
{
    const int es = elem_size_of(dtype);
    if (es == 0)
        return H2X_ERR_UNSUPPORTED;
    if (width == 0)
        return H2X_SUCCESS;
    if (!tensor || !real_shape || num_dims < 1 || num_dims > H2X_MAX_DIMS)
        return H2X_ERR_INVALID_ARGUMENT;
    Launcher l(as_stream(stream), es, dtype, H2X_HALO_ID);
    for (int side = 0; side < 2; ++side)
    {
        h2x_halo_face f;
        std::memset(&f, 0, sizeof(f));
        for (int i = 0; i < num_dims; ++i)
            f.real_shape[i] = real_shape[i];
        f.num_dims = num_dims;
        f.dim = dim;
        f.side = side;
        f.width = width;
        f.inner = 0;
        HostBox h;
        int err = halo_box(f, &h);
        if (err != 0)
            return err;
        err = l.add(h, tensor, nullptr, kClear);
        if (err != 0)
            return err;
    }
    return l.flush();
}

extern "C" int h2x_halo_clear_batched(h2x_dtype dtype, const h2x_halo_face* faces, int num_faces,
                                      h2x_stream_t stream)
{
    const int es = elem_size_of(dtype);
    if (es == 0)
        return H2X_ERR_UNSUPPORTED;
    if (num_faces < 0 || (num_faces > 0 && !faces))
        return H2X_ERR_INVALID_ARGUMENT;
    // validate everything before anything is launched
    BoxList boxes(num_faces);
    for (int i = 0; i < num_faces; ++i)
    {
        const int err = halo_box(faces[i], &boxes[i]);
        if (err != 0)
            return err;
        if (boxes[i].count > 0 && !faces[i].tensor)
            return H2X_ERR_INVALID_ARGUMENT;
        if (boxes[i].count >= (1ll << 31))
            return H2X_ERR_TOO_LARGE;
    }
    // sparse strips first, then the others: boxes of one kind share launches
    Launcher l(as_stream(stream), es, dtype, H2X_HALO_ID);
    for (int pass = 0; pass < 2; ++pass)
        for (int i = 0; i < num_faces; ++i)
        {
            if (boxes[i].count == 0 || box_is_sparse(boxes[i], es) != (pass == 0))
                continue;
            const int err = l.add(boxes[i], faces[i].tensor, nullptr, kClear);
            if (err != 0)
                return err;
        }
    return l.flush();
}

extern "C" int h2x_halo_exchange_fused(h2x_dtype dtype, const h2x_halo_transfer* transfers,
                                       int num_transfers, h2x_stream_t stream)
{
    const int es = elem_size_of(dtype);
    if (es == 0)
        return H2X_ERR_UNSUPPORTED;
    if (num_transfers < 0 || (num_transfers > 0 && !transfers))
        return H2X_ERR_INVALID_ARGUMENT;
    // validate everything before anything is launched
    BoxList boxes(num_transfers);
    unsigned int ops_present = 0;
    for (int i = 0; i < num_transfers; ++i)
    {
        const h2x_halo_transfer& t = transfers[i];
        if (t.op < H2X_HALO_ID || t.op > H2X_HALO_MIN
            || (t.src_side != H2X_LHS && t.src_side != H2X_RHS))
            return H2X_ERR_INVALID_ARGUMENT;
        // the strip as pack sees it in src and as unpack sees it in dst
        h2x_halo_face from, to;
        std::memset(&from, 0, sizeof(from));
        std::memset(&to, 0, sizeof(to));
        from.num_dims = to.num_dims = t.num_dims;
        from.dim = to.dim = t.dim;
        from.width = to.width = t.width;
        from.side = t.src_side;
        to.side = t.src_side == H2X_LHS ? H2X_RHS : H2X_LHS;
        from.inner = t.is_reverse ? 0 : 1;
        to.inner = t.is_reverse ? 1 : 0;
        if (t.num_dims < 1 || t.num_dims > H2X_MAX_DIMS)
            return H2X_ERR_INVALID_ARGUMENT;
        for (int d = 0; d < t.num_dims; ++d)
        {
            from.real_shape[d] = t.src_real_shape[d];
            to.real_shape[d] = t.dst_real_shape[d];
            if (d != t.dim && t.src_real_shape[d] != t.dst_real_shape[d])
                return H2X_ERR_INVALID_ARGUMENT;
        }
        HostBox a, b;
        int err = halo_box(from, &a, true);
        if (err == 0)
            err = halo_box(to, &b, true);
        if (err != 0)
            return err;
        // same extents, two sets of strides
        int64_t extent[kMaxBoxDims], stride_dst[kMaxBoxDims], stride_src[kMaxBoxDims];
        int64_t sd = 1, ss = 1;
        for (int d = 0; d < t.num_dims; ++d)
        {
            extent[d] = d == t.dim ? t.width : t.dst_real_shape[d];
            stride_dst[d] = sd;
            stride_src[d] = ss;
            sd *= t.dst_real_shape[d];
            ss *= t.src_real_shape[d];
        }
        boxes[i] = reduce_box(t.num_dims, extent, stride_dst, b.tensor_offset, a.tensor_offset,
                              stride_src);
        if (boxes[i].count > 0 && (!t.src || !t.dst))
            return H2X_ERR_INVALID_ARGUMENT;
        if (boxes[i].count >= (1ll << 31))
            return H2X_ERR_TOO_LARGE;
        ops_present |= 1u << t.op;
    }
    for (int op = H2X_HALO_ID; op <= H2X_HALO_MIN; ++op)
    {
        if (!(ops_present & (1u << op)))
            continue;
        Launcher l(as_stream(stream), es, dtype, op);
        for (int i = 0; i < num_transfers; ++i)
        {
            if (transfers[i].op != op)
                continue;
            const int err = l.add(boxes[i], transfers[i].dst, const_cast<void*>(transfers[i].src),
                                  kTransfer);
            if (err != 0)
                return err;
        }
        const int err = l.flush();
        if (err != 0)
            return err;
    }
    return H2X_SUCCESS;
}

// ---- shuffle -------------------------------------------------------------------

struct h2x_shuffle_plan
{
    int elem_size;
    std::vector<HostBox> boxes; // one per peer with a non-empty intersection
    // Device table of the same boxes for launches that take their descriptors
    // from memory (null if the plan does not qualify: sparse boxes).  Entries
    // hold byte offsets where a launch from kernel arguments holds addresses.
    Box* table = nullptr;
    int table_device = -1;
    // A plan made while a launch audit is open keeps the table on the host
    // instead (no GPU call is made); it serves audited launches only.
    std::vector<Box> host_table;
    int table_vec = 0;         // vector width the table's `ragged` flags were made for
    uint32_t most_blocks = 0;  // workgroups of the largest box at table_vec
    uint64_t total_blocks = 0; // over all boxes
};

namespace
{

// Builds the device table of a plan.  Assumes buffers aligned to 16 bytes; a
// launch with a less aligned buffer goes through the kernel arguments instead.
int make_table(h2x_shuffle_plan* p)
{
    const int n = static_cast<int>(p->boxes.size());
    if (n == 0)
        return H2X_SUCCESS;
    int vec = 16 / p->elem_size;
    for (const HostBox& h : p->boxes)
    {
        if (box_is_sparse(h, p->elem_size))
            return H2X_SUCCESS; // pairs of sparse boxes are formed per launch
        bool rg;
        vec = std::min(vec, box_vector(h, p->elem_size, nullptr, true, &rg));
    }
    std::vector<Box> host(static_cast<size_t>(n));
    for (int i = 0; i < n; ++i)
    {
        const HostBox& h = p->boxes[i];
        fill_box(&host[i], h);
        host[i].tensor = reinterpret_cast<char*>(static_cast<intptr_t>(h.tensor_offset * p->elem_size));
        host[i].buffer = reinterpret_cast<char*>(static_cast<intptr_t>(h.buffer_offset * p->elem_size));
        host[i].ragged = vec > 1 && h.extent[0] % vec != 0;
        const uint64_t blocks = box_blocks(h.count, vec);
        p->most_blocks = std::max<uint64_t>(p->most_blocks, blocks);
        p->total_blocks += blocks;
    }
    if (current_audit())
    {
        p->host_table = host;
        p->table_vec = vec;
        return H2X_SUCCESS;
    }
    hipError_t err = hipGetDevice(&p->table_device);
    if (err == hipSuccess)
        err = hipMalloc(reinterpret_cast<void**>(&p->table), sizeof(Box) * host.size());
    if (err == hipSuccess)
        err = hipMemcpy(p->table, host.data(), sizeof(Box) * host.size(), hipMemcpyHostToDevice);
    if (err != hipSuccess)
    {
        if (p->table)
            (void) hipFree(p->table);
        p->table = nullptr;
        return static_cast<int>(err);
    }
    p->table_vec = vec;
    return H2X_SUCCESS;
}

} // namespace

extern "C" int h2x_shuffle_plan_create(const h2x_shuffle_geometry* g, h2x_shuffle_plan** plan)
{
    if (!g || !plan)
        return H2X_ERR_INVALID_ARGUMENT;
    *plan = nullptr;
    const int nd = g->num_dims;
    if (nd < 1 || nd > H2X_MAX_DIMS || !g->rank_limits || !g->displs)
        return H2X_ERR_INVALID_ARGUMENT;
    if (g->elem_size != 2 && g->elem_size != 4 && g->elem_size != 8)
        return H2X_ERR_UNSUPPORTED;
    int64_t num_peers = 1;
    for (int i = 0; i < nd; ++i)
    {
        if (g->local_shape[i] < 0 || g->peer_locale_shape[i] < 1 || g->strides[i] < 0)
            return H2X_ERR_INVALID_ARGUMENT;
        num_peers *= g->peer_locale_shape[i];
    }
    // limits must be non-decreasing and end at the local extent
    {
        int rl = 0;
        for (int i = 0; i < nd; ++i)
        {
            int prev = 0;
            for (int j = 0; j < g->peer_locale_shape[i]; ++j)
            {
                const int lim = g->rank_limits[rl + j];
                if (lim < prev || lim > g->local_shape[i])
                    return H2X_ERR_INVALID_ARGUMENT;
                prev = lim;
            }
            if (prev != g->local_shape[i] && g->local_shape[i] != 0)
                return H2X_ERR_INVALID_ARGUMENT;
            rl += static_cast<int>(g->peer_locale_shape[i]);
        }
    }
    h2x_shuffle_plan* p = new (std::nothrow) h2x_shuffle_plan;
    if (!p)
        return static_cast<int>(hipErrorOutOfMemory);
    p->elem_size = g->elem_size;
    for (int64_t peer = 0; peer < num_peers; ++peer)
    {
        int64_t extent[kMaxBoxDims], rem = peer, origin = 0;
        int rl = 0;
        bool empty = false;
        for (int i = 0; i < nd; ++i)
        {
            const int j = static_cast<int>(rem % g->peer_locale_shape[i]);
            rem /= g->peer_locale_shape[i];
            const int lo = j == 0 ? 0 : g->rank_limits[rl + j - 1];
            const int hi = g->rank_limits[rl + j];
            extent[i] = hi - lo;
            origin += static_cast<int64_t>(lo) * g->strides[i];
            empty = empty || extent[i] <= 0;
            rl += static_cast<int>(g->peer_locale_shape[i]);
        }
        if (empty)
            continue;
        HostBox h = reduce_box(nd, extent, g->strides, origin, g->displs[peer]);
        if (h.count >= (1ll << 31))
        {
            delete p;
            return H2X_ERR_TOO_LARGE;
        }
        p->boxes.push_back(h);
    }
    const int err = make_table(p);
    if (err != 0)
    {
        delete p;
        return err;
    }
    *plan = p;
    return H2X_SUCCESS;
}

extern "C" int h2x_shuffle_plan_destroy(h2x_shuffle_plan* plan)
{
    if (plan && plan->table)
        (void) hipFree(plan->table);
    delete plan;
    return H2X_SUCCESS;
}

// All plans of a call through their device tables, kMaxPlans per launch.
// Returns false (nothing launched) if the call does not qualify: a plan
// without a table or made on another device, mixed element sizes or vector
// widths, a buffer that is not 16-byte aligned, or boxes so unequal that
// taking turns would more than double the grid.
static bool shuffle_through_tables(const h2x_shuffle_plan* const* plans, void* const* tensors,
                                   void* const* buffers, int num_plans, int mode,
                                   h2x_stream_t stream, int* status)
{
    const bool audited = current_audit() != nullptr;
    int device = -1;
    if (!audited && hipGetDevice(&device) != hipSuccess)
        return false;
    const h2x_shuffle_plan* first = nullptr;
    uint32_t most = 0;
    uint64_t total = 0, boxes = 0;
    for (int i = 0; i < num_plans; ++i)
    {
        const h2x_shuffle_plan* p = plans[i];
        if (p->boxes.empty())
            continue;
        const bool has_table = audited ? !p->host_table.empty() : (p->table && p->table_device == device);
        if (!has_table || reinterpret_cast<uintptr_t>(buffers[i]) % 16 != 0)
            return false;
        if (!first)
            first = p;
        if (p->elem_size != first->elem_size || p->table_vec != first->table_vec)
            return false;
        most = std::max(most, p->most_blocks);
        total += p->total_blocks;
        boxes += p->boxes.size();
    }
    *status = H2X_SUCCESS;
    if (!first)
        return true; // nothing to move
    if (static_cast<uint64_t>(most) * boxes > 2 * total)
        return false;
    int i = 0;
    while (i < num_plans)
    {
        TableBatch batch;
        batch.num_plans = 0;
        batch.num_boxes = 0;
        batch.reserved = 0;
        uint32_t launch_most = 0;
        for (; i < num_plans && batch.num_plans < kMaxPlans; ++i)
        {
            const h2x_shuffle_plan* p = plans[i];
            if (p->boxes.empty())
                continue;
            PlanRef& ref = batch.plan[batch.num_plans++];
            ref.table = audited ? p->host_table.data() : p->table;
            ref.tensor = static_cast<char*>(tensors[i]);
            ref.buffer = static_cast<char*>(buffers[i]);
            ref.first_box = batch.num_boxes;
            ref.reserved = 0;
            batch.num_boxes += static_cast<uint32_t>(p->boxes.size());
            launch_most = std::max(launch_most, p->most_blocks);
        }
        if (batch.num_plans == 0)
            break;
        const uint64_t grid = static_cast<uint64_t>(launch_most) * batch.num_boxes;
        if (grid > 0x7fffffffull)
        {
            *status = H2X_ERR_TOO_LARGE;
            return true;
        }
        batch.blocks_per_box = launch_most;
        LaunchShape shape{first->elem_size, H2X_HALO_ID, first->table_vec, false, mode,
                          static_cast<uint32_t>(grid), as_stream(stream)};
        *status = launch_tables(shape, batch);
        if (*status != 0)
            return true;
    }
    return true;
}

static int shuffle_batched(const h2x_shuffle_plan* const* plans, void* const* tensors,
                           void* const* buffers, int num_plans, int mode, h2x_stream_t stream)
{
    if (num_plans < 0 || (num_plans > 0 && (!plans || !tensors || !buffers)))
        return H2X_ERR_INVALID_ARGUMENT;
    for (int i = 0; i < num_plans; ++i)
    {
        if (!plans[i])
            return H2X_ERR_INVALID_ARGUMENT;
        if (!plans[i]->boxes.empty() && (!tensors[i] || !buffers[i]))
            return H2X_ERR_INVALID_ARGUMENT;
    }
    int status = H2X_SUCCESS;
    if (shuffle_through_tables(plans, tensors, buffers, num_plans, mode, stream, &status))
        return status;
    for (int es : {2, 4, 8})
    {
        Launcher l(as_stream(stream), es, H2X_F32, H2X_HALO_ID);
        for (int i = 0; i < num_plans; ++i)
        {
            if (plans[i]->elem_size != es)
                continue;
            for (const HostBox& h : plans[i]->boxes)
            {
                const int err = l.add(h, tensors[i], buffers[i], mode);
                if (err != 0)
                    return err;
            }
        }
        const int err = l.flush();
        if (err != 0)
            return err;
    }
    return H2X_SUCCESS;
}

extern "C" int h2x_shuffle_pack(const h2x_shuffle_plan* plan, const void* tensor, void* buffer,
                                h2x_stream_t stream)
{
    void* t = const_cast<void*>(tensor);
    return shuffle_batched(&plan, &t, &buffer, 1, kPack, stream);
}

extern "C" int h2x_shuffle_unpack(const h2x_shuffle_plan* plan, void* tensor, const void* buffer,
                                  h2x_stream_t stream)
{
    void* b = const_cast<void*>(buffer);
    return shuffle_batched(&plan, &tensor, &b, 1, kUnpack, stream);
}

extern "C" int h2x_shuffle_pack_batched(const h2x_shuffle_plan* const* plans,
                                        const void* const* tensors, void* const* buffers,
                                        int num_plans, h2x_stream_t stream)
{
    return shuffle_batched(plans, const_cast<void* const*>(tensors), buffers, num_plans, kPack, stream);
}

extern "C" int h2x_shuffle_unpack_batched(const h2x_shuffle_plan* const* plans,
                                          void* const* tensors, const void* const* buffers,
                                          int num_plans, h2x_stream_t stream)
{
    return shuffle_batched(plans, tensors, const_cast<void* const*>(buffers), num_plans, kUnpack, stream);
}

// ---- launch audit ------------------------------------------------------------------

extern "C" int h2x_copy_audit_begin(void)
{
    if (t_audit)
        return H2X_ERR_INVALID_ARGUMENT;
    t_audit = new (std::nothrow) Audit;
    return t_audit ? static_cast<int>(H2X_SUCCESS) : static_cast<int>(hipErrorOutOfMemory);
}

extern "C" int h2x_copy_audit_add_region(const h2x_copy_audit_region* region)
{
    if (!t_audit || !region)
        return H2X_ERR_INVALID_ARGUMENT;
    t_audit->regions.push_back(AuditRegion{region->base, region->bytes, region->loads, region->stores});
    return H2X_SUCCESS;
}

extern "C" int h2x_copy_audit_end(h2x_copy_audit_report* report)
{
    if (!t_audit)
        return H2X_ERR_INVALID_ARGUMENT;
    if (report)
    {
        report->launches = t_audit->launches;
        report->workgroups = t_audit->workgroups;
        report->outside_loads = t_audit->outside_loads;
        report->outside_stores = t_audit->outside_stores;
        report->misaligned = t_audit->misaligned;
    }
    delete t_audit;
    t_audit = nullptr;
    return H2X_SUCCESS;
}

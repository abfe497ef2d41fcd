// HaloExchange and the tensor shuffler of the DistConv API on top of the h2x
// C ABI.  Interfaces follow
//   legacy/include/distconv/tensor/halo_exchange_cuda.hpp:18-423 (HaloExchange),
//   legacy/include/distconv/tensor/halo_packing_cuda.hpp:143-167 (pack_or_unpack),
//   legacy/include/distconv/tensor/shuffle_mpi_cuda.hpp:14-512 (TensorMPICUDAShuffler).
// The transports of the reference (MPI, Aluminum, CUDA IPC, NVSHMEM) are
// replaced by one: virtual ranks inside the process, connected by handing out
// device pointers.  Per-rank objects keep the reference's interface; the
// *Virtual group classes own one object per rank and run a collective step for
// all of them with as few launches as possible.
#pragma once

#include <algorithm>
#include <fstream>
#include <memory>
#include <sstream>
#include <string>
#include <vector>

#include "distconv/tensor_mi355x.hpp"

namespace distconv
{
namespace tensor
{

// legacy/include/distconv/tensor/halo_exchange.hpp:8-9
enum class HaloExchangeAccumOp
{
    ID,
    SUM,
    MAX,
    MIN
};

// Tag standing where the reference has an Aluminum back-end type.
struct VirtualBackend
{
};

namespace halo_exchange_cuda
{

// halo_packing_cuda.hpp:143-167
template <typename DataType, typename Locale>
void pack_or_unpack(Tensor<DataType, Locale, CUDAAllocator>& tensor, int dim, Side side, int width,
                    hipStream_t stream, void* buf, bool is_pack, bool is_reverse,
                    HaloExchangeAccumOp op)
{
    if (width == 0)
        return;
    // TraverseHalo's preconditions, legacy/include/distconv/tensor/halo_cuda.hpp:909-916
    assert_always(width <= tensor.get_halo_width(dim));
    const bool inner = (is_pack && !is_reverse) || (!is_pack && is_reverse);
    if (inner)
        assert_always(tensor.get_local_shape()[dim] >= static_cast<size_t>(width));
    int64_t shape[H2X_MAX_DIMS];
    for (int i = 0; i < tensor.get_num_dims(); ++i)
        shape[i] = static_cast<int64_t>(tensor.get_local_real_shape()[i]);
    using T = Tensor<DataType, Locale, CUDAAllocator>;
    DISTCONV_CHECK_H2X(h2x_halo_pack_or_unpack(T::h2x_type(), tensor.get_buffer(),
                                               tensor.get_num_dims(), shape, dim,
                                               static_cast<int>(side), width, buf, is_pack,
                                               is_reverse, static_cast<int>(op), stream));
}

} // namespace halo_exchange_cuda

// One (dim, side) slot per boundary: legacy/include/distconv/base.hpp BoundaryAttributesV.
template <typename T>
class BoundaryAttributesV
{
public:
    BoundaryAttributesV() = default;
    explicit BoundaryAttributesV(int num_dims) : m_v(static_cast<size_t>(num_dims) * 2) {}
    BoundaryAttributesV(int num_dims, const T& init) : m_v(static_cast<size_t>(num_dims) * 2, init) {}
    T& operator()(int dim, Side side) { return m_v[static_cast<size_t>(dim) * 2 + side]; }
    const T& operator()(int dim, Side side) const { return m_v[static_cast<size_t>(dim) * 2 + side]; }

private:
    std::vector<T> m_v;
};

constexpr int kProcNull = -1; // MPI_PROC_NULL of the reference

template <typename DataType, typename Allocator, typename Backend>
class HaloExchange;

// halo_exchange_cuda.hpp:18-423 for one rank.  The per-dimension exchange is
// pure virtual, as in the reference; HaloExchangeVirtual below implements it.
template <typename DataType>
class HaloExchange<DataType, CUDAAllocator, VirtualBackend>
{
public:
    using TensorType = Tensor<DataType, LocaleVirtual, CUDAAllocator>;

    explicit HaloExchange(TensorType& tensor, bool periodic = false)
        : m_tensor(tensor), m_periodic(periodic), m_halo_send(tensor.get_num_dims()),
          m_halo_recv(tensor.get_num_dims()), m_peers(tensor.get_num_dims(), kProcNull)
    {
        bool required = false;
        for (int i = 0; i < tensor.get_num_dims(); ++i)
            required = required || is_exchange_required(i);
        if (required)
        {
            assert_always(!tensor.get_distribution().is_shared()); // :30-31
            set_peer_ranks();
        }
    }
    virtual ~HaloExchange() = default;

    virtual void exchange(int dim, int width_rhs_send, int width_rhs_recv, int width_lhs_send,
                          int width_lhs_recv, hipStream_t stream_rhs, hipStream_t stream_lhs,
                          bool rendezvous, bool is_reverse, bool skip_unpack,
                          HaloExchangeAccumOp op = HaloExchangeAccumOp::ID) = 0;

    // All dimensions, innermost first (halo_exchange_cuda.hpp:56-106): the two
    // boundary streams of a dimension wait for the streams the previous
    // exchanged dimension ran on (the main stream for the first), and with
    // `sync_back` the main stream waits for the last ones.  `streams(dim, side)`
    // stands for the stream of the reference's per-boundary communicator.
    virtual void exchange(const IntVector& widths_rhs_send, const IntVector& widths_rhs_recv,
                          const IntVector& widths_lhs_send, const IntVector& widths_lhs_recv,
                          BoundaryAttributesV<hipStream_t>& streams, hipStream_t stream_main,
                          bool rendezvous, bool sync_back, bool is_reverse, bool skip_unpack,
                          HaloExchangeAccumOp op = HaloExchangeAccumOp::ID)
    {
        hipStream_t prev_streams[2] = {stream_main, stream_main};
        for (int i = 0; i < m_tensor.get_num_dims(); ++i)
        {
            if (!is_exchange_required(i, widths_rhs_send[i], widths_rhs_recv[i], widths_lhs_send[i],
                                      widths_lhs_recv[i]))
                continue;
            for (Side side : SIDES)
            {
                const hipStream_t cur_streams[2] = {streams(i, RHS), streams(i, LHS)};
                util::wait_stream(prev_streams[side], cur_streams, 2);
                prev_streams[side] = streams(i, side);
            }
            exchange(i, widths_rhs_send[i], widths_rhs_recv[i], widths_lhs_send[i],
                     widths_lhs_recv[i], streams(i, RHS), streams(i, LHS), rendezvous, is_reverse,
                     skip_unpack, op);
        }
        if (sync_back)
            for (Side side : SIDES)
                util::wait_stream(prev_streams[side], stream_main);
    }

    // halo_exchange_cuda.hpp:107-125: the tensor's own halo widths
    virtual void exchange(BoundaryAttributesV<hipStream_t>& streams, hipStream_t stream_main,
                          bool rendezvous, bool sync_back, bool is_reverse, bool skip_unpack,
                          HaloExchangeAccumOp op = HaloExchangeAccumOp::ID)
    {
        const IntVector& w = m_tensor.get_halo_width();
        exchange(w, w, w, w, streams, stream_main, rendezvous, sync_back, is_reverse, skip_unpack, op);
    }

    TensorType& get_tensor() { return m_tensor; }
    int get_peer(int dim, Side side) const { return m_peers(dim, side); }

    // :267-275
    size_t get_halo_size(int dim, int width) const
    {
        Shape s = m_tensor.get_local_real_shape();
        s[dim] = width;
        return s.get_size();
    }
    size_t get_halo_size(int dim) const { return get_halo_size(dim, m_tensor.get_halo_width(dim)); }

    void* get_send_buffer(int dim, Side side) { return m_halo_send(dim, side).get(); }
    void* get_recv_buffer(int dim, Side side) { return m_halo_recv(dim, side).get(); }

    // :204-255 -- debugging aids: the packed strips of a dimension as text, one
    // value a line, in send_halo_<rank>_<dim>_<side>.txt and recv_halo_... under
    // `directory` (the reference writes into the working directory).  They copy
    // with the blocking hipMemcpy, like the reference's mem_copy; sides without
    // a peer and buffers that were never allocated are left out.
    void dump_packed_halo(int dim, const std::string& directory = ".")
    {
        for (Side side : SIDES)
        {
            if (get_peer(dim, side) == kProcNull)
                continue;
            dump_buffer(get_send_buffer(dim, side), "send_halo_", dim, side, directory);
            dump_buffer(get_recv_buffer(dim, side), "recv_halo_", dim, side, directory);
        }
    }
    void dump_recv_halo(int dim, const std::string& directory = ".")
    {
        for (Side side : SIDES)
            dump_buffer(get_recv_buffer(dim, side), "recv_halo_", dim, side, directory);
    }

    // :285-303 -- buffers are sized for the full halo width and zero-filled
    void ensure_halo_buffers(int dim)
    {
        const size_t bytes = get_halo_size(dim) * sizeof(DataType);
        assert_always(bytes > 0);
        for (Side side : SIDES)
        {
            if (get_peer(dim, side) == kProcNull)
                continue;
            if (m_halo_send(dim, side).is_null())
                m_halo_send(dim, side).allocate(bytes);
            if (m_halo_recv(dim, side).is_null())
                m_halo_recv(dim, side).allocate(bytes);
        }
    }

    // :305-320
    bool is_exchange_required(int dim, int wrs, int wrr, int wls, int wlr) const
    {
        const auto& dist = m_tensor.get_distribution();
        return dist.is_distributed(dim) && dist.get_split_shape()[dim] > 1
               && (wrs > 0 || wrr > 0 || wls > 0 || wlr > 0) && m_tensor.get_local_size() > 0;
    }
    bool is_exchange_required(int dim) const
    {
        const int w = m_tensor.get_halo_width(dim);
        return is_exchange_required(dim, w, w, w, w);
    }

    // :365-384
    void pack_dim(int dim, Side side, int width, hipStream_t stream, void* buf, bool is_reverse)
    {
        halo_exchange_cuda::pack_or_unpack(m_tensor, dim, side, width, stream, buf, true, is_reverse,
                                           HaloExchangeAccumOp::ID);
    }
    void unpack_dim(int dim, Side side, int width, hipStream_t stream, void* buf, bool is_reverse,
                    HaloExchangeAccumOp op = HaloExchangeAccumOp::ID)
    {
        halo_exchange_cuda::pack_or_unpack(m_tensor, dim, side, width, stream, buf, false,
                                           is_reverse, op);
    }

    // :395-422
    virtual bool unpack(int dim, int width_rhs_recv, int width_lhs_recv, hipStream_t stream_rhs,
                        hipStream_t stream_lhs, bool is_reverse,
                        HaloExchangeAccumOp op = HaloExchangeAccumOp::ID)
    {
        bool done = false;
        for (Side side : SIDES)
        {
            if (get_peer(dim, side) == kProcNull)
                continue;
            const int w = side == RHS ? width_rhs_recv : width_lhs_recv;
            if (w == 0)
                continue;
            unpack_dim(dim, side, w, side == RHS ? stream_rhs : stream_lhs,
                       get_recv_buffer(dim, side), is_reverse, op);
            done = true;
        }
        return done;
    }

protected:
    void dump_buffer(const void* device, const char* prefix, int dim, Side side,
                     const std::string& directory)
    {
        if (!device)
            return;
        std::vector<DataType> h(get_halo_size(dim));
        DISTCONV_CHECK_HIP(hipMemcpy(h.data(), device, h.size() * sizeof(DataType), hipMemcpyDeviceToHost));
        std::ostringstream path;
        path << directory << "/" << prefix << m_tensor.get_locale().get_rank() << "_" << dim << "_"
             << (side == LHS ? "LHS" : "RHS") << ".txt"; // base.hpp:30-36 prints a side by name
        std::ofstream out(path.str(), std::ios::out | std::ios::trunc);
        for (const DataType& v : h)
            out << v << std::endl;
    }

    // :322-357; with `periodic` the grid wraps, which the reference never does
    int find_peer_rank(int dim, Side side) const
    {
        if (!is_exchange_required(dim) || m_tensor.get_local_size() == 0)
            return kProcNull;
        const auto& locale_shape = m_tensor.get_distribution().get_locale_shape();
        const int extent = static_cast<int>(locale_shape[dim]);
        int p = static_cast<int>(m_tensor.get_proc_index()[dim]) + (side == RHS ? 1 : -1);
        if (p < 0 || p >= extent)
        {
            if (!m_periodic)
                return kProcNull;
            p = (p + extent) % extent;
        }
        // a neighbour without elements sends nothing
        if (!m_periodic && m_tensor.get_dimension_rank_offset(dim, p) == m_tensor.get_shape()[dim])
            return kProcNull;
        IndexVector idx = m_tensor.get_proc_index();
        idx[dim] = static_cast<index_t>(p);
        return static_cast<int>(get_offset(idx, locale_shape));
    }
    void set_peer_ranks()
    {
        for (int d = 0; d < m_tensor.get_num_dims(); ++d)
            for (Side side : SIDES)
                m_peers(d, side) = find_peer_rank(d, side);
    }

    TensorType& m_tensor;
    bool m_periodic;
    BoundaryAttributesV<Memory<CUDAAllocator>> m_halo_send;
    BoundaryAttributesV<Memory<CUDAAllocator>> m_halo_recv;
    BoundaryAttributesV<int> m_peers;
};

// All virtual ranks of one distributed tensor.  exchange() is the dimension
// loop of halo_exchange_cuda.hpp:56-106 (innermost dimension first, each phase
// seeing the halo cells the previous ones filled) with the message order of
// halo_exchange_cuda_mpi.hpp:25-100 (pack and send both sides, then unpack).
// A rank's send buffer for (dim, side) is its neighbour's receive buffer for
// the opposite side, so nothing is copied between ranks, and each phase is
// two launches: every rank's packs, then every rank's unpacks.
template <typename DataType>
class HaloExchangeVirtual
{
public:
    using Rank = HaloExchange<DataType, CUDAAllocator, VirtualBackend>;
    using TensorType = typename Rank::TensorType;

    explicit HaloExchangeVirtual(const std::vector<TensorType*>& tensors, bool periodic = false)
    {
        for (TensorType* t : tensors)
            m_ranks.emplace_back(new Member(*t, periodic));
        for (auto& r : m_ranks)
            for (int d = 0; d < r->get_tensor().get_num_dims(); ++d)
                if (r->is_exchange_required(d))
                    r->ensure_halo_buffers(d);
    }

    Rank& rank(int r) { return *m_ranks[r]; }
    int num_ranks() const { return static_cast<int>(m_ranks.size()); }

    void exchange(const IntVector& widths_rhs_send, const IntVector& widths_rhs_recv,
                  const IntVector& widths_lhs_send, const IntVector& widths_lhs_recv,
                  hipStream_t stream, bool is_reverse = false, bool skip_unpack = false,
                  HaloExchangeAccumOp op = HaloExchangeAccumOp::ID)
    {
        const int nd = m_ranks[0]->get_tensor().get_num_dims();
        for (int d = 0; d < nd; ++d)
            exchange(d, widths_rhs_send[d], widths_rhs_recv[d], widths_lhs_send[d],
                     widths_lhs_recv[d], stream, is_reverse, skip_unpack, op);
    }

    void exchange(hipStream_t stream, bool is_reverse = false, bool skip_unpack = false,
                  HaloExchangeAccumOp op = HaloExchangeAccumOp::ID)
    {
        const IntVector& w = m_ranks[0]->get_tensor().get_halo_width();
        exchange(w, w, w, w, stream, is_reverse, skip_unpack, op);
    }

    // The reference's driver signature (halo_exchange_cuda.hpp:56-82) for the
    // whole group: boundary streams are fenced dimension after dimension as
    // there; both sides of a dimension share launches here, which go to the
    // RHS boundary stream.
    void exchange(const IntVector& widths_rhs_send, const IntVector& widths_rhs_recv,
                  const IntVector& widths_lhs_send, const IntVector& widths_lhs_recv,
                  BoundaryAttributesV<hipStream_t>& streams, hipStream_t stream_main,
                  bool /*rendezvous*/, bool sync_back, bool is_reverse, bool skip_unpack,
                  HaloExchangeAccumOp op = HaloExchangeAccumOp::ID)
    {
        hipStream_t prev_streams[2] = {stream_main, stream_main};
        const int nd = m_ranks[0]->get_tensor().get_num_dims();
        for (int i = 0; i < nd; ++i)
        {
            bool required = false;
            for (auto& r : m_ranks)
                required = required
                           || r->is_exchange_required(i, widths_rhs_send[i], widths_rhs_recv[i],
                                                      widths_lhs_send[i], widths_lhs_recv[i]);
            if (!required)
                continue;
            for (Side side : SIDES)
            {
                const hipStream_t cur_streams[2] = {streams(i, RHS), streams(i, LHS)};
                util::wait_stream(prev_streams[side], cur_streams, 2);
                prev_streams[side] = streams(i, side);
            }
            exchange(i, widths_rhs_send[i], widths_rhs_recv[i], widths_lhs_send[i],
                     widths_lhs_recv[i], streams(i, RHS), is_reverse, skip_unpack, op);
        }
        if (sync_back)
            for (Side side : SIDES)
                util::wait_stream(prev_streams[side], stream_main);
    }

    void exchange(int dim, int wrs, int wrr, int wls, int wlr, hipStream_t stream, bool is_reverse,
                  bool skip_unpack, HaloExchangeAccumOp op)
    {
        const h2x_dtype dt = TensorType::h2x_type();
        const int width = std::max(std::max(wrs, wrr), std::max(wls, wlr));
        for (const std::vector<int>& group : rank_groups(dim, width))
        {
            std::vector<h2x_halo_face> packs, unpacks;
            for (int member : group)
            {
                auto& r = m_ranks[member];
                if (!r->is_exchange_required(dim, wrs, wrr, wls, wlr))
                    continue;
                for (Side side : SIDES)
                {
                    const int peer = r->get_peer(dim, side);
                    if (peer == kProcNull)
                        continue;
                    const int w_send = side == RHS ? wrs : wls;
                    const int w_recv = side == RHS ? wrr : wlr;
                    if (w_send > 0) // my RHS strip lands in my RHS neighbour's LHS receive buffer
                        packs.push_back(face(*r, dim, side, w_send,
                                             m_ranks[peer]->get_recv_buffer(dim, ~side), true,
                                             is_reverse, op));
                    if (w_recv > 0 && !skip_unpack)
                        unpacks.push_back(face(*r, dim, side, w_recv,
                                               r->get_recv_buffer(dim, side), false, is_reverse,
                                               op));
                }
            }
            if (!packs.empty())
                DISTCONV_CHECK_H2X(h2x_halo_pack_or_unpack_batched(
                    dt, packs.data(), static_cast<int>(packs.size()), stream));
            if (!unpacks.empty())
                DISTCONV_CHECK_H2X(h2x_halo_pack_or_unpack_batched(
                    dt, unpacks.data(), static_cast<int>(unpacks.size()), stream));
        }
    }

    // Tensor::clear_halo for every dimension that has a halo, on every rank, in
    // batched launches: the loop that precedes the forward exchange in
    // Convolution::forward (convolution.hpp:400-411).  only_unfilled: only the
    // sides without a neighbour are cleared.  A full-width exchange() that
    // follows overwrites every other halo strip completely (a strip spans the
    // whole real extent of the other dimensions), and the stale values it moves
    // into corner cells in the meantime are themselves overwritten by a later
    // dimension's phase -- neighbours along one dimension sit at the same
    // position of every other dimension, so a corner that no later phase fills
    // receives cleared cells -- so the tensors end up exactly as after clearing
    // everything first.
    void clear_halos(hipStream_t stream, bool only_unfilled = false)
    {
        std::vector<h2x_halo_face> faces;
        for (auto& r : m_ranks)
        {
            auto& t = r->get_tensor();
            if (t.get_local_size() == 0)
                continue;
            for (int d = 0; d < t.get_num_dims(); ++d)
            {
                const int width = t.get_halo_width(d);
                if (width == 0)
                    continue;
                for (Side side : SIDES)
                {
                    if (only_unfilled && r->get_peer(d, side) != kProcNull)
                        continue;
                    h2x_halo_face f = {};
                    f.tensor = t.get_buffer();
                    for (int i = 0; i < t.get_num_dims(); ++i)
                        f.real_shape[i] = static_cast<int64_t>(t.get_local_real_shape()[i]);
                    f.num_dims = t.get_num_dims();
                    f.dim = d;
                    f.side = static_cast<int>(side);
                    f.width = width;
                    faces.push_back(f);
                }
            }
        }
        if (!faces.empty())
            DISTCONV_CHECK_H2X(h2x_halo_clear_batched(TensorType::h2x_type(), faces.data(),
                                                      static_cast<int>(faces.size()), stream));
    }

    // The exchange of all dimensions with every strip moved straight from the
    // neighbour's tensor into this rank's (one launch per dimension and group
    // of ranks, no buffers).  The tensors end up as after exchange().
    void exchange_fused(hipStream_t stream, bool is_reverse = false,
                        HaloExchangeAccumOp op = HaloExchangeAccumOp::ID)
    {
        const IntVector& w = m_ranks[0]->get_tensor().get_halo_width();
        const int nd = m_ranks[0]->get_tensor().get_num_dims();
        for (int d = 0; d < nd; ++d)
            exchange_fused(d, w[d], w[d], stream, is_reverse, op);
    }

    // width_rhs: strips that cross a rank's RHS face (sent from its RHS side and
    // received on the neighbour's LHS side); width_lhs likewise.
    void exchange_fused(int dim, int width_rhs, int width_lhs, hipStream_t stream, bool is_reverse,
                        HaloExchangeAccumOp op)
    {
        const h2x_dtype dt = TensorType::h2x_type();
        // all ranks in one launch: nothing is read back between launches here,
        // so rank groups would only add launches
        {
            std::vector<h2x_halo_transfer> moves;
            for (int member = 0; member < num_ranks(); ++member)
            {
                auto& r = m_ranks[member]; // the receiver
                if (!r->is_exchange_required(dim, width_rhs, width_rhs, width_lhs, width_lhs))
                    continue;
                for (Side side : SIDES)
                {
                    const int peer = r->get_peer(dim, side);
                    // my RHS halo holds what my RHS neighbour sends from its LHS side
                    const int width = side == RHS ? width_lhs : width_rhs;
                    if (peer == kProcNull || width == 0)
                        continue;
                    auto& src = m_ranks[peer]->get_tensor();
                    auto& dst = r->get_tensor();
                    assert_always(width <= dst.get_halo_width(dim));
                    h2x_halo_transfer m = {};
                    m.src = src.get_buffer();
                    m.dst = dst.get_buffer();
                    for (int i = 0; i < dst.get_num_dims(); ++i)
                    {
                        m.src_real_shape[i] = static_cast<int64_t>(src.get_local_real_shape()[i]);
                        m.dst_real_shape[i] = static_cast<int64_t>(dst.get_local_real_shape()[i]);
                    }
                    m.num_dims = dst.get_num_dims();
                    m.dim = dim;
                    m.src_side = static_cast<int>(~side);
                    m.width = width;
                    m.is_reverse = is_reverse ? 1 : 0;
                    m.op = static_cast<int>(op);
                    moves.push_back(m);
                }
            }
            if (!moves.empty())
                DISTCONV_CHECK_H2X(h2x_halo_exchange_fused(dt, moves.data(),
                                                           static_cast<int>(moves.size()), stream));
        }
    }

    // Ranks that exchange dimension `dim` together, group after group.  Faces
    // of the innermost dimension touch one short run per row, each costing a
    // 128-byte line, and the unpack writes into the lines its rank's pack has
    // just read: a group is kept small enough (160 MB of lines) for those
    // lines to stay in the 256 MB memory-side cache between the two launches,
    // where the unpack's partial writes merge into whole lines.  Neighbours
    // along `dim` always share a group.
    std::vector<std::vector<int>> rank_groups(int dim, int width) const
    {
        constexpr size_t kLineBytes = 128;
        constexpr size_t kGroupBytes = size_t(160) << 20;
        std::vector<std::vector<int>> groups;
        if (dim != 0 || width * sizeof(DataType) >= kLineBytes)
        {
            groups.emplace_back();
            for (int r = 0; r < num_ranks(); ++r)
                groups.back().push_back(r);
            return groups;
        }
        std::vector<bool> placed(m_ranks.size(), false);
        size_t group_bytes = 0;
        for (int r = 0; r < num_ranks(); ++r)
        {
            if (placed[r])
                continue;
            // the line of ranks through r along `dim`
            std::vector<int> line;
            size_t line_bytes = 0;
            const auto& pr = m_ranks[r]->get_tensor().get_proc_index();
            for (int q = r; q < num_ranks(); ++q)
            {
                const auto& t = m_ranks[q]->get_tensor();
                bool same = !placed[q];
                for (int i = 0; same && i < t.get_num_dims(); ++i)
                    same = i == dim || t.get_proc_index()[i] == pr[i];
                if (!same)
                    continue;
                placed[q] = true;
                line.push_back(q);
                size_t rows = 1;
                for (int i = 1; i < t.get_num_dims(); ++i)
                    rows *= static_cast<size_t>(t.get_local_real_shape()[i]);
                line_bytes += rows * kLineBytes;
            }
            if (groups.empty() || group_bytes + line_bytes > kGroupBytes)
            {
                groups.emplace_back();
                group_bytes = 0;
            }
            groups.back().insert(groups.back().end(), line.begin(), line.end());
            group_bytes += line_bytes;
        }
        return groups;
    }

private:
    // exchange(dim, ...) of one rank alone cannot complete inside one process
    // (its neighbours must pack first); the group runs the phases instead.
    struct Member : public Rank
    {
        using Rank::Rank;
        using Rank::exchange;
        void exchange(int, int, int, int, int, hipStream_t, hipStream_t, bool, bool, bool,
                      HaloExchangeAccumOp) override
        {
            util::fail("per-rank exchange: use HaloExchangeVirtual::exchange", __FILE__, __LINE__);
        }
    };

    static h2x_halo_face face(Rank& r, int dim, Side side, int width, void* buf, bool is_pack,
                              bool is_reverse, HaloExchangeAccumOp op)
    {
        h2x_halo_face f = {};
        auto& t = r.get_tensor();
        assert_always(width <= t.get_halo_width(dim));
        f.tensor = t.get_buffer();
        f.buffer = buf;
        for (int i = 0; i < t.get_num_dims(); ++i)
            f.real_shape[i] = static_cast<int64_t>(t.get_local_real_shape()[i]);
        f.num_dims = t.get_num_dims();
        f.dim = dim;
        f.side = static_cast<int>(side);
        f.width = width;
        f.inner = ((is_pack && !is_reverse) || (!is_pack && is_reverse)) ? 1 : 0;
        f.is_pack = is_pack ? 1 : 0;
        f.op = static_cast<int>(op);
        return f;
    }

    std::vector<std::unique_ptr<Member>> m_ranks;
};

// shuffle_mpi_cuda.hpp:14-512 for one rank.  The constructor builds the
// reference's tables (rank limits of the peer grid in local coordinates,
// counts and displacements in rank order, :129-287); `transfer` is virtual, as
// in the reference.  The reference's default is the all-to-all over the ranks
// (:342-403); one rank of a virtual locale can deliver only to itself, so the
// default here moves the rank's own chunk and aborts if another rank has
// anything to send or receive (TensorShufflerVirtual does the all-to-all).
template <typename DataType>
class TensorMPICUDAShuffler
{
public:
    using TensorType = Tensor<DataType, LocaleVirtual, CUDAAllocator>;

    TensorMPICUDAShuffler(const TensorType& src_tensor, const TensorType& dst_tensor,
                          DataType* src_buf = nullptr, DataType* dst_buf = nullptr)
        : m_src_local_size(src_tensor.get_local_size()), m_dst_local_size(dst_tensor.get_local_size()),
          m_src_split_root(src_tensor.is_split_root()), m_dst_split_root(dst_tensor.is_split_root()),
          m_rank(src_tensor.get_locale().get_rank()), m_src_buf(src_buf), m_dst_buf(dst_buf)
    {
        const int n = src_tensor.get_locale().get_size();
        m_rank_limits_fwd = rank_limits(src_tensor, dst_tensor);
        m_rank_limits_bwd = rank_limits(dst_tensor, src_tensor);
        int send = 0, recv = 0;
        for (int pid = 0; pid < n; ++pid)
        {
            m_send_displs.push_back(send);
            m_recv_displs.push_back(recv);
            m_send_counts.push_back(count(src_tensor, dst_tensor, pid));
            m_recv_counts.push_back(count(dst_tensor, src_tensor, pid));
            send += m_send_counts.back();
            recv += m_recv_counts.back();
        }
        m_pack_fwd = make_plan(src_tensor, dst_tensor, m_rank_limits_fwd, m_send_displs);
        m_unpack_fwd = make_plan(dst_tensor, src_tensor, m_rank_limits_bwd, m_recv_displs);
    }
    virtual ~TensorMPICUDAShuffler()
    {
        h2x_shuffle_plan_destroy(m_pack_fwd);
        h2x_shuffle_plan_destroy(m_unpack_fwd);
    }
    TensorMPICUDAShuffler(const TensorMPICUDAShuffler&) = delete;
    TensorMPICUDAShuffler& operator=(const TensorMPICUDAShuffler&) = delete;

    // :83-90
    static size_t get_buf_size(const TensorType& tensor)
    {
        return tensor.get_local_shape().get_size() * sizeof(DataType);
    }

    // legacy/src/tensor/shuffle_mpi_cuda.cu:378-490: pack -> transfer -> unpack.
    // Backward uses the same tables with the roles of the tensors swapped.
    void shuffle_forward(const DataType* src, DataType* dst, hipStream_t stream = nullptr)
    {
        shuffle(src, dst, stream, true);
    }
    void shuffle_backward(const DataType* src, DataType* dst, hipStream_t stream = nullptr)
    {
        shuffle(src, dst, stream, false);
    }

    // Steps of shuffle(), usable on their own by a group of virtual ranks.
    void pack(const DataType* src, DataType* send_buf, hipStream_t stream, bool is_forward)
    {
        const size_t n = is_forward ? m_src_local_size : m_dst_local_size;
        if (n && (is_forward ? m_src_split_root : m_dst_split_root))
        {
            if (is_forward)
                DISTCONV_CHECK_H2X(h2x_shuffle_pack(m_pack_fwd, src, send_buf, stream));
            else // the forward unpack plan describes the dst tensor cut by the src grid
                DISTCONV_CHECK_H2X(h2x_shuffle_pack(m_unpack_fwd, src, send_buf, stream));
        }
    }
    void unpack(DataType* dst, const DataType* recv_buf, hipStream_t stream, bool is_forward)
    {
        const size_t n = is_forward ? m_dst_local_size : m_src_local_size;
        if (n && (is_forward ? m_dst_split_root : m_src_split_root))
        {
            if (is_forward)
                DISTCONV_CHECK_H2X(h2x_shuffle_unpack(m_unpack_fwd, dst, recv_buf, stream));
            else
                DISTCONV_CHECK_H2X(h2x_shuffle_unpack(m_pack_fwd, dst, recv_buf, stream));
        }
    }

    const std::vector<int>& get_rank_limits_fwd(bool is_forward) const
    {
        return is_forward ? m_rank_limits_fwd : m_rank_limits_bwd;
    }
    const std::vector<int>& get_send_counts(bool is_forward) const
    {
        return is_forward ? m_send_counts : m_recv_counts;
    }
    const std::vector<int>& get_recv_counts(bool is_forward) const
    {
        return is_forward ? m_recv_counts : m_send_counts;
    }
    const std::vector<int>& get_send_displs_h(bool is_forward) const
    {
        return is_forward ? m_send_displs : m_recv_displs;
    }
    const std::vector<int>& get_recv_displs_h(bool is_forward) const
    {
        return is_forward ? m_recv_displs : m_send_displs;
    }
    size_t send_buffer_size(bool is_forward) const
    {
        return (is_forward ? m_src_local_size : m_dst_local_size) * sizeof(DataType);
    }
    size_t recv_buffer_size(bool is_forward) const
    {
        return (is_forward ? m_dst_local_size : m_src_local_size) * sizeof(DataType);
    }

protected:
    // shuffle_mpi_cuda.hpp:342-403: moves the packed chunks between ranks.  One
    // rank alone can deliver only its own chunk; a shuffle that involves other
    // ranks must go through TensorShufflerVirtual (or an override), so a non-zero
    // count for another rank aborts instead of leaving `recv_buf` unwritten.
    virtual void transfer(const DataType* send_buf, size_t send_buffer_size, DataType* recv_buf,
                          size_t recv_buffer_size, bool is_forward, hipStream_t stream)
    {
        const std::vector<int>& send_counts = get_send_counts(is_forward);
        const std::vector<int>& recv_counts = get_recv_counts(is_forward);
        for (size_t p = 0; p < send_counts.size(); ++p)
            if (static_cast<int>(p) != m_rank)
                assert_always(send_counts[p] == 0 && recv_counts[p] == 0);
        const size_t bytes = static_cast<size_t>(send_counts[m_rank]) * sizeof(DataType);
        assert_always(send_counts[m_rank] == recv_counts[m_rank]);
        const size_t from = static_cast<size_t>(get_send_displs_h(is_forward)[m_rank]);
        const size_t to = static_cast<size_t>(get_recv_displs_h(is_forward)[m_rank]);
        assert_always(from * sizeof(DataType) + bytes <= send_buffer_size
                      && to * sizeof(DataType) + bytes <= recv_buffer_size);
        if (bytes > 0)
            DISTCONV_CHECK_HIP(hipMemcpyAsync(recv_buf + to, send_buf + from, bytes,
                                              hipMemcpyDeviceToDevice, stream));
    }

    void shuffle(const DataType* src, DataType* dst, hipStream_t stream, bool is_forward)
    {
        Memory<CUDAAllocator> tmp_send, tmp_recv;
        DataType* send_buf = buffer(is_forward ? m_src_buf : m_dst_buf, send_buffer_size(is_forward), tmp_send);
        DataType* recv_buf = buffer(is_forward ? m_dst_buf : m_src_buf, recv_buffer_size(is_forward), tmp_recv);
        pack(src, send_buf, stream, is_forward);
        transfer(send_buf, send_buffer_size(is_forward), recv_buf, recv_buffer_size(is_forward),
                 is_forward, stream);
        unpack(dst, recv_buf, stream, is_forward);
        if (!tmp_send.is_null() || !tmp_recv.is_null())
            DISTCONV_CHECK_HIP(hipStreamSynchronize(stream)); // temporaries die with this scope
    }

private:
    static DataType* buffer(DataType* passed, size_t bytes, Memory<CUDAAllocator>& tmp)
    {
        if (passed || bytes == 0)
            return passed;
        tmp.allocate(bytes);
        return static_cast<DataType*>(tmp.get());
    }

    // setup_rank_limits, :129-173 (plain limits; the "-1" lookup shortcut of
    // :175-213 encodes the same slabs)
    static std::vector<int> rank_limits(const TensorType& a, const TensorType& b)
    {
        std::vector<int> out;
        for (int d = 0; d < a.get_num_dims(); ++d)
        {
            const int extent = static_cast<int>(b.get_locale_shape()[d]);
            const int per = static_cast<int>(b.get_distribution().get_num_ranks_per_split(d));
            for (int j = 0; j < extent; ++j)
            {
                const int next_root = (j / per + 1) * per;
                const index_t next = next_root < extent ? b.get_dimension_rank_offset(d, next_root)
                                                        : b.get_shape()[d];
                index_t lim = 0;
                if (next >= a.get_global_index()[d])
                {
                    lim = next - a.get_global_index()[d];
                    if (lim > a.get_local_shape()[d])
                        lim = a.get_local_shape()[d];
                }
                out.push_back(static_cast<int>(lim));
            }
        }
        return out;
    }

    // elements rank `a` exchanges with rank `pid` of b's grid (setup_displs, :215-287)
    static int count(const TensorType& a, const TensorType& b, int pid)
    {
        const IndexVector idx = LocaleVirtual(pid, a.get_locale().get_size()).get_rank_idx(b.get_distribution());
        if (!a.is_split_root() || !b.get_distribution().is_split_root(idx))
            return 0;
        const Region mine(a.get_global_index(), a.get_local_shape());
        const Region theirs(b.get_remote_index(idx), b.get_remote_shape(idx));
        return static_cast<int>(mine.intersect(theirs).get_size());
    }

    static h2x_shuffle_plan* make_plan(const TensorType& mine, const TensorType& other,
                                       const std::vector<int>& limits, const std::vector<int>& displs)
    {
        h2x_shuffle_geometry g = {};
        g.num_dims = mine.get_num_dims();
        g.elem_size = sizeof(DataType);
        const Shape strides = mine.get_strides();
        for (int i = 0; i < g.num_dims; ++i)
        {
            g.local_shape[i] = static_cast<int64_t>(mine.get_local_shape()[i]);
            g.strides[i] = static_cast<int64_t>(strides[i]);
            g.peer_locale_shape[i] = static_cast<int64_t>(other.get_locale_shape()[i]);
        }
        g.rank_limits = limits.data();
        g.displs = displs.data();
        h2x_shuffle_plan* plan = nullptr;
        DISTCONV_CHECK_H2X(h2x_shuffle_plan_create(&g, &plan));
        return plan;
    }

    size_t m_src_local_size, m_dst_local_size;
    bool m_src_split_root, m_dst_split_root;
    int m_rank;
    std::vector<int> m_rank_limits_fwd, m_rank_limits_bwd;
    std::vector<int> m_send_counts, m_recv_counts, m_send_displs, m_recv_displs;
    DataType* m_src_buf;
    DataType* m_dst_buf;
    h2x_shuffle_plan* m_pack_fwd = nullptr;
    h2x_shuffle_plan* m_unpack_fwd = nullptr;
};

// All virtual ranks of a (src, dst) pair: pack on every rank, the all-to-all of
// the reference's default transfer (MPI_Alltoallv with the counts and
// displacements above, shuffle_mpi_cuda.hpp:342-403) as device-to-device
// copies between the ranks' buffers, unpack on every rank.
template <typename DataType>
class TensorShufflerVirtual
{
public:
    using Rank = TensorMPICUDAShuffler<DataType>;
    using TensorType = typename Rank::TensorType;

    TensorShufflerVirtual(const std::vector<TensorType*>& src, const std::vector<TensorType*>& dst)
        : m_src(src), m_dst(dst)
    {
        assert_always(src.size() == dst.size());
        for (size_t r = 0; r < src.size(); ++r)
        {
            m_ranks.emplace_back(new Rank(*src[r], *dst[r]));
            m_send.emplace_back(new Memory<CUDAAllocator>);
            m_recv.emplace_back(new Memory<CUDAAllocator>);
            const size_t bytes = std::max(Rank::get_buf_size(*src[r]), Rank::get_buf_size(*dst[r]));
            m_send.back()->allocate(bytes);
            m_recv.back()->allocate(bytes);
        }
    }

    Rank& rank(int r) { return *m_ranks[r]; }

    void shuffle_forward(hipStream_t stream = nullptr) { run(stream, true); }
    void shuffle_backward(hipStream_t stream = nullptr) { run(stream, false); }

private:
    void run(hipStream_t stream, bool fwd)
    {
        const int n = static_cast<int>(m_ranks.size());
        auto& from = fwd ? m_src : m_dst;
        auto& to = fwd ? m_dst : m_src;
        for (int r = 0; r < n; ++r)
            m_ranks[r]->pack(from[r]->get_const_base_ptr(),
                             static_cast<DataType*>(m_send[r]->get()), stream, fwd);
        for (int r = 0; r < n; ++r) // receiver r, sender p
            for (int p = 0; p < n; ++p)
            {
                const int cnt = m_ranks[r]->get_recv_counts(fwd)[p];
                assert_always(cnt == m_ranks[p]->get_send_counts(fwd)[r]);
                if (cnt == 0)
                    continue;
                DISTCONV_CHECK_HIP(hipMemcpyAsync(
                    static_cast<DataType*>(m_recv[r]->get()) + m_ranks[r]->get_recv_displs_h(fwd)[p],
                    static_cast<const DataType*>(m_send[p]->get()) + m_ranks[p]->get_send_displs_h(fwd)[r],
                    static_cast<size_t>(cnt) * sizeof(DataType), hipMemcpyDeviceToDevice, stream));
            }
        for (int r = 0; r < n; ++r)
            m_ranks[r]->unpack(to[r]->get_base_ptr(), static_cast<const DataType*>(m_recv[r]->get()),
                               stream, fwd);
    }

    std::vector<TensorType*> m_src, m_dst;
    std::vector<std::unique_ptr<Rank>> m_ranks;
    std::vector<std::unique_ptr<Memory<CUDAAllocator>>> m_send, m_recv;
};

} // namespace tensor
} // namespace distconv

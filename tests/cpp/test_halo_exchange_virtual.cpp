// Halo exchange through the C++ layer, checked by the closed form of
// legacy/tests/tensor/test_halo_exchange_cuda.cu:104-233: after the exchange
// every halo cell whose source exists (or wraps, on a periodic grid) holds the
// global offset of its source.
#include "test_common.hpp"

#include <cstdlib>
#include <fstream>
#include <string>

enum Mode
{
    kBuffers,        // pack, unpack through receive buffers, one stream
    kFused,          // tensor-to-tensor transfers
    kBoundaryStreams, // the reference's driver signature with two boundary streams per dimension
    kClearBatched,    // pack, unpack; the halos cleared by one batched call for all ranks and dimensions
    kClearUnfilled    // pack, unpack; only the halo strips without a neighbour cleared beforehand
};

static int run_case(const Shape& shape, const Shape& locale, const IntVector& overlap, bool periodic,
                    Mode mode = kBuffers)
{
    const int nd = shape.length();
    const int n = static_cast<int>(locale.get_size());
    const Distribution dist = Distribution::make_overlapped_distribution(locale, overlap);
    std::vector<std::unique_ptr<DevTensor<float>>> ranks;
    std::vector<DevTensor<float>*> ptrs;
    for (int r = 0; r < n; ++r)
    {
        ranks.emplace_back(new DevTensor<float>(shape, LocaleVirtual(r, n), dist));
        CHECK(ranks.back()->allocate() == 0);
        to_device(*ranks.back(), global_offset_field(*ranks.back(), -1.0f));
        ptrs.push_back(ranks.back().get());
    }
    HaloExchangeVirtual<float> xch(ptrs, periodic);
    // Convolution clears the halo before every exchange (the fields carry -1 there)
    if (mode == kClearBatched || mode == kClearUnfilled)
        xch.clear_halos(nullptr, mode == kClearUnfilled);
    else
        for (int d = 0; d < nd; ++d)
            for (auto* t : ptrs)
                t->clear_halo(d, nullptr);
    if (mode == kFused)
    {
        xch.exchange_fused(nullptr);
    }
    else if (mode == kBoundaryStreams)
    {
        hipStream_t main_stream;
        DISTCONV_CHECK_HIP(hipStreamCreate(&main_stream));
        BoundaryAttributesV<hipStream_t> streams(nd);
        for (int d = 0; d < nd; ++d)
            for (Side side : SIDES)
                DISTCONV_CHECK_HIP(hipStreamCreate(&streams(d, side)));
        DISTCONV_CHECK_HIP(hipDeviceSynchronize()); // the fields were written on the null stream
        const IntVector& w = ranks[0]->get_halo_width();
        xch.exchange(w, w, w, w, streams, main_stream, false, true, false, false);
        DISTCONV_CHECK_HIP(hipStreamSynchronize(main_stream)); // sync_back: main waits for the boundaries
        for (int d = 0; d < nd; ++d)
            for (Side side : SIDES)
                DISTCONV_CHECK_HIP(hipStreamDestroy(streams(d, side)));
        DISTCONV_CHECK_HIP(hipStreamDestroy(main_stream));
    }
    else
    {
        xch.exchange(nullptr);
    }
    int errors = 0;
    for (int r = 0; r < n; ++r)
    {
        auto& t = *ranks[r];
        std::vector<float> h = to_host(t);
        const Shape& rs = t.get_local_real_shape();
        for (index_t o = 0; o < h.size(); ++o)
        {
            IndexVector idx = rs.get_index(o);
            IndexVector g(nd, 0);
            bool exists = true;
            for (int i = 0; i < nd; ++i)
            {
                long long c = static_cast<long long>(idx[i] + t.get_global_index()[i]) - t.get_halo_width(i);
                const long long ext = static_cast<long long>(shape[i]);
                if (periodic && t.get_distribution().is_distributed(i))
                    c = (c % ext + ext) % ext;
                if (c < 0 || c >= ext)
                    exists = false;
                g[i] = static_cast<index_t>(c < 0 ? 0 : c);
            }
            const float want = exists ? static_cast<float>(get_offset(g, shape)) : 0.0f; // cleared
            if (h[o] != want)
            {
                if (errors < 5)
                    std::printf("rank %d offset %zu: got %f want %f\n", r, (size_t) o, h[o], want);
                ++errors;
            }
        }
    }
    return errors;
}

int main()
{
    std::setvbuf(stdout, nullptr, _IONBF, 0); // what was printed survives a crash
    int errors = 0;
    for (bool periodic : {false, true})
    {
        errors += run_case(Shape({12, 10, 3, 2}), Shape({2, 2, 1, 1}), IntVector({1, 1, 0, 0}), periodic);
        errors += run_case(Shape({12, 10, 3, 2}), Shape({2, 2, 1, 1}), IntVector({2, 2, 0, 0}), periodic);
        errors += run_case(Shape({13, 11, 3, 2}), Shape({3, 2, 1, 1}), IntVector({1, 2, 0, 0}), periodic);
        errors += run_case(Shape({8, 10, 12, 3, 2}), Shape({2, 2, 2, 1, 1}), IntVector({1, 1, 1, 0, 0}), periodic);
        errors += run_case(Shape({8, 9, 10, 2, 1}), Shape({1, 2, 2, 1, 1}), IntVector({0, 2, 1, 0, 0}), periodic);
        // tensor-to-tensor transfers instead of pack + unpack
        errors += run_case(Shape({13, 11, 3, 2}), Shape({3, 2, 1, 1}), IntVector({1, 2, 0, 0}), periodic, kFused);
        errors += run_case(Shape({8, 10, 12, 3, 2}), Shape({2, 2, 2, 1, 1}), IntVector({1, 1, 1, 0, 0}), periodic, kFused);
        errors += run_case(Shape({8, 10, 12, 3, 2}), Shape({2, 2, 2, 1, 1}), IntVector({1, 1, 1, 0, 0}), periodic,
                           kBoundaryStreams);
        // the clearing batched, and cut down to the strips the exchange does not overwrite
        for (Mode m : {kClearBatched, kClearUnfilled})
        {
            errors += run_case(Shape({13, 11, 3, 2}), Shape({3, 2, 1, 1}), IntVector({1, 2, 0, 0}), periodic, m);
            errors += run_case(Shape({8, 10, 12, 3, 2}), Shape({2, 2, 2, 1, 1}), IntVector({1, 1, 1, 0, 0}), periodic, m);
            errors += run_case(Shape({9, 12, 12, 3, 2}), Shape({1, 3, 2, 1, 1}), IntVector({0, 2, 1, 0, 0}), periodic, m);
        }
    }
    // reverse exchange with SUM: transfers and pack + unpack leave the same tensors
    {
        const Shape shape({12, 10, 3, 2}), locale({2, 2, 1, 1});
        const Distribution dist = Distribution::make_overlapped_distribution(locale, IntVector({1, 2, 0, 0}));
        std::vector<std::unique_ptr<DevTensor<float>>> a, b;
        std::vector<DevTensor<float>*> pa, pb;
        std::mt19937 gen(5);
        std::uniform_int_distribution<int> d(-8, 8);
        for (int r = 0; r < 4; ++r)
        {
            a.emplace_back(new DevTensor<float>(shape, LocaleVirtual(r, 4), dist));
            b.emplace_back(new DevTensor<float>(shape, LocaleVirtual(r, 4), dist));
            CHECK(a.back()->allocate() == 0 && b.back()->allocate() == 0);
            std::vector<float> h(a.back()->get_local_real_size());
            for (auto& v : h)
                v = static_cast<float>(d(gen));
            to_device(*a.back(), h);
            to_device(*b.back(), h);
            pa.push_back(a.back().get());
            pb.push_back(b.back().get());
        }
        HaloExchangeVirtual<float> xa(pa, true), xb(pb, true);
        xa.exchange(nullptr, true, false, HaloExchangeAccumOp::SUM);
        xb.exchange_fused(nullptr, true, HaloExchangeAccumOp::SUM);
        for (int r = 0; r < 4; ++r)
        {
            const std::vector<float> ha = to_host(*a[r]), hb = to_host(*b[r]);
            for (size_t i = 0; i < ha.size(); ++i)
                errors += ha[i] != hb[i];
        }
    }
    // per-rank interface: pack one strip, unpack it on the neighbour
    {
        const Shape shape({8, 6, 2, 1}), locale({2, 1, 1, 1});
        const Distribution dist = Distribution::make_overlapped_distribution(locale, IntVector({1, 0, 0, 0}));
        DevTensor<float> a(shape, LocaleVirtual(0, 2), dist), b(shape, LocaleVirtual(1, 2), dist);
        a.allocate();
        b.allocate();
        to_device(a, global_offset_field(a, -1.0f));
        to_device(b, global_offset_field(b, -1.0f));
        HaloExchangeVirtual<float> xch({&a, &b});
        CHECK(xch.rank(0).get_peer(0, RHS) == 1 && xch.rank(0).get_peer(0, LHS) == kProcNull);
        CHECK(xch.rank(0).get_halo_size(0, 1) == 6 * 2 * 1);
        xch.rank(0).pack_dim(0, RHS, 1, nullptr, xch.rank(1).get_recv_buffer(0, LHS), false);
        CHECK(xch.rank(1).unpack(0, 0, 1, nullptr, nullptr, false));
        std::vector<float> h = to_host(b);
        for (int y = 0; y < 6; ++y) // b's LHS halo column holds global x = 3
            if (h[y * 6 + 0] != static_cast<float>(3 + 8 * y))
                ++errors;
    }
    // debugging dumps (halo_exchange_cuda.hpp:204-255): after an exchange of dimension 0 the receive
    // buffer of rank 1's LHS side holds rank 0's RHS boundary column, one value a line
    {
        const Shape shape({8, 6, 2, 1}), locale({2, 1, 1, 1});
        const Distribution dist = Distribution::make_overlapped_distribution(locale, IntVector({1, 0, 0, 0}));
        DevTensor<float> a(shape, LocaleVirtual(0, 2), dist), b(shape, LocaleVirtual(1, 2), dist);
        a.allocate();
        b.allocate();
        to_device(a, global_offset_field(a, -1.0f));
        to_device(b, global_offset_field(b, -1.0f));
        HaloExchangeVirtual<float> xch({&a, &b});
        xch.exchange(nullptr);
        DISTCONV_CHECK_HIP(hipDeviceSynchronize());
        const char* tmp = std::getenv("TMPDIR");
        const std::string dir = tmp ? tmp : "/tmp";
        xch.rank(1).dump_packed_halo(0, dir);
        std::ifstream in(dir + "/recv_halo_1_0_LHS.txt");
        CHECK(in.good());
        int lines = 0;
        float v;
        while (in >> v)
        {
            const int y = lines % 6, c = lines / 6; // strip of width 1: rows of the plane, then channels
            if (v != static_cast<float>(3 + 8 * y + 48 * c))
                ++errors;
            ++lines;
        }
        errors += lines != 12;
        // the local part of rank 1, raw: its real allocation, which now holds the filled LHS halo column
        CHECK(dump_local_tensor(b, dir + "/h2x_dump_test", true) == 0);
        std::ifstream raw(dir + "/h2x_dump_test_1.out", std::ios::binary);
        std::vector<float> got(b.get_local_real_size());
        raw.read(reinterpret_cast<char*>(got.data()), got.size() * sizeof(float));
        CHECK(raw.gcount() == static_cast<std::streamsize>(got.size() * sizeof(float)));
        errors += got != to_host(b);
        std::remove((dir + "/h2x_dump_test_1.out").c_str());
        std::remove((dir + "/recv_halo_1_0_LHS.txt").c_str());
        std::remove((dir + "/send_halo_1_0_LHS.txt").c_str());
    }
    std::printf("test_halo_exchange_virtual: %d errors\n", errors);
    return finish(errors);
}

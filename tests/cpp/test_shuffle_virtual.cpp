// Tensor shuffler through the C++ layer with the closed form of
// legacy/tests/tensor/test_tensor_mpi_shuffle.cpp:26-154: every element holds its
// global offset; after shuffle_forward every destination element holds its own
// global offset; shuffle_backward restores the source.
#include "test_common.hpp"

template <typename T = float>
static int run_case(const Shape& shape, const Distribution& sd, const Distribution& dd)
{
    const int n = static_cast<int>(sd.get_locale_shape().get_size());
    std::vector<std::unique_ptr<DevTensor<T>>> own;
    std::vector<DevTensor<T>*> src, dst;
    for (int r = 0; r < n; ++r)
    {
        own.emplace_back(new DevTensor<T>(shape, LocaleVirtual(r, n), sd));
        src.push_back(own.back().get());
        own.emplace_back(new DevTensor<T>(shape, LocaleVirtual(r, n), dd));
        dst.push_back(own.back().get());
        src[r]->allocate();
        dst[r]->allocate();
        to_device(*src[r], global_offset_field(*src[r], static_cast<T>(-1)));
        to_device(*dst[r], std::vector<T>(dst[r]->get_local_real_size(), static_cast<T>(-7)));
    }
    TensorShufflerVirtual<T> sh(src, dst);
    sh.shuffle_forward();
    int errors = 0;
    for (int r = 0; r < n; ++r)
    {
        std::vector<T> want = dst[r]->is_split_root() ? global_offset_field(*dst[r], static_cast<T>(-7))
                                                          : std::vector<T>(dst[r]->get_local_real_size(), static_cast<T>(-7));
        std::vector<T> got = to_host(*dst[r]);
        for (size_t i = 0; i < got.size(); ++i)
            errors += got[i] != want[i];
    }
    std::vector<std::vector<T>> keep;
    for (int r = 0; r < n; ++r)
    {
        keep.push_back(to_host(*src[r]));
        if (src[r]->is_split_root()) // interior is rewritten by the backward shuffle
        {
            std::vector<T> h = keep.back();
            const Shape& ls = src[r]->get_local_shape();
            for (index_t o = 0; o < src[r]->get_local_size(); ++o)
                h[src[r]->get_local_offset(ls.get_index(o))] = static_cast<T>(-3);
            to_device(*src[r], h);
        }
    }
    sh.shuffle_backward();
    for (int r = 0; r < n; ++r)
    {
        std::vector<T> got = to_host(*src[r]);
        for (size_t i = 0; i < got.size(); ++i)
            errors += got[i] != keep[r][i];
    }
    return errors;
}

int main()
{
    std::setvbuf(stdout, nullptr, _IONBF, 0); // what was printed survives a crash
    int errors = 0;
    const Shape s4({8, 8, 2, 4});
    const IntVector none(4, 0);
    // same distribution
    errors += run_case(s4, Distribution::make_distribution(Shape({2, 2, 1, 1})),
                       Distribution::make_distribution(Shape({2, 2, 1, 1})));
    // sample-parallel -> spatial-parallel and back
    errors += run_case(s4, Distribution::make_distribution(Shape({1, 1, 1, 4})),
                       Distribution::make_distribution(Shape({2, 2, 1, 1})));
    // ... into a destination with halo
    errors += run_case(s4, Distribution::make_distribution(Shape({1, 1, 1, 4})),
                       Distribution::make_overlapped_distribution(Shape({2, 2, 1, 1}), IntVector({1, 1, 0, 0})));
    // overlapped source -> plain destination
    errors += run_case(s4, Distribution::make_overlapped_distribution(Shape({2, 2, 1, 1}), IntVector({1, 2, 0, 0})),
                       Distribution::make_distribution(Shape({2, 2, 1, 1})));
    // uneven partition
    errors += run_case(Shape({11, 7, 3, 5}), Distribution::make_distribution(Shape({1, 1, 1, 4})),
                       Distribution::make_distribution(Shape({2, 2, 1, 1})));
    // shrink the spatial split (shared distribution)
    errors += run_case(s4, Distribution::make_distribution(Shape({2, 2, 1, 1})),
                       Distribution::make_shared_distribution(Shape({2, 2, 1, 1}), Shape({2, 1, 1, 1})));
    // the other element types the reference instantiates (shuffle_mpi_cuda.cu:492-499): 2, 4 and 8 bytes
    errors += run_case<short>(s4, Distribution::make_distribution(Shape({1, 1, 1, 4})),
                              Distribution::make_distribution(Shape({2, 2, 1, 1})));
    errors += run_case<unsigned short>(s4, Distribution::make_distribution(Shape({1, 1, 1, 4})),
                                       Distribution::make_overlapped_distribution(Shape({2, 2, 1, 1}),
                                                                                  IntVector({1, 1, 0, 0})));
    errors += run_case<int>(Shape({11, 7, 3, 5}), Distribution::make_distribution(Shape({1, 1, 1, 4})),
                            Distribution::make_distribution(Shape({2, 2, 1, 1})));
    errors += run_case<unsigned>(s4, Distribution::make_distribution(Shape({2, 2, 1, 1})),
                                 Distribution::make_distribution(Shape({1, 1, 1, 4})));
    errors += run_case<long>(s4, Distribution::make_distribution(Shape({1, 1, 1, 4})),
                             Distribution::make_distribution(Shape({2, 2, 1, 1})));
    errors += run_case<unsigned long>(Shape({11, 7, 3, 5}), Distribution::make_distribution(Shape({1, 1, 1, 4})),
                                      Distribution::make_distribution(Shape({2, 2, 1, 1})));
    errors += run_case<double>(s4, Distribution::make_distribution(Shape({1, 1, 1, 4})),
                               Distribution::make_overlapped_distribution(Shape({2, 2, 1, 1}),
                                                                          IntVector({1, 1, 0, 0})));
    // 5-D
    errors += run_case(Shape({6, 8, 4, 2, 4}), Distribution::make_distribution(Shape({1, 1, 1, 1, 4})),
                       Distribution::make_overlapped_distribution(Shape({1, 2, 2, 1, 1}), IntVector({0, 1, 1, 0, 0})));
    // tables of one rank: N split over 4 -> H/2 x W/2, rank 1
    {
        DevTensor<float> a(s4, LocaleVirtual(1, 4), Distribution::make_distribution(Shape({1, 1, 1, 4})));
        DevTensor<float> b(s4, LocaleVirtual(1, 4), Distribution::make_distribution(Shape({2, 2, 1, 1})));
        TensorMPICUDAShuffler<float> sh(a, b);
        CHECK((sh.get_rank_limits_fwd(true) == std::vector<int>{4, 8, 4, 8, 2, 1}));
        CHECK((sh.get_send_counts(true) == std::vector<int>{32, 32, 32, 32}));
        CHECK((sh.get_send_displs_h(true) == std::vector<int>{0, 32, 64, 96}));
        CHECK(TensorMPICUDAShuffler<float>::get_buf_size(a) == 8 * 8 * 2 * 1 * sizeof(float));
    }
    // one rank alone: shuffle_forward / shuffle_backward of the per-rank class itself
    // (pack -> default transfer of the rank's own chunk -> unpack), plain source into a
    // haloed destination and back
    {
        const Shape s1({6, 5, 3, 2});
        DevTensor<float> a(s1, LocaleVirtual(0, 1), Distribution::make_distribution(Shape({1, 1, 1, 1})));
        DevTensor<float> b(s1, LocaleVirtual(0, 1),
                           Distribution::make_overlapped_distribution(Shape({1, 1, 1, 1}), IntVector({1, 2, 0, 0})));
        a.allocate();
        b.allocate();
        const std::vector<float> field = global_offset_field(a, -1.0f);
        to_device(a, field);
        to_device(b, std::vector<float>(b.get_local_real_size(), -7.0f));
        TensorMPICUDAShuffler<float> sh(a, b);
        sh.shuffle_forward(a.get_const_base_ptr(), b.get_base_ptr());
        DISTCONV_CHECK_HIP(hipDeviceSynchronize());
        const std::vector<float> want = global_offset_field(b, -7.0f), got = to_host(b);
        for (size_t i = 0; i < got.size(); ++i)
            errors += got[i] != want[i];
        to_device(a, std::vector<float>(a.get_local_real_size(), -3.0f));
        sh.shuffle_backward(b.get_const_base_ptr(), a.get_base_ptr());
        DISTCONV_CHECK_HIP(hipDeviceSynchronize());
        const std::vector<float> back = to_host(a);
        for (size_t i = 0; i < back.size(); ++i)
            errors += back[i] != field[i];
    }
    std::printf("test_shuffle_virtual: %d errors\n", errors);
    return finish(errors);
}

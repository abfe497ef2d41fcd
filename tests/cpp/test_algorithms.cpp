// tensor::Transform / ReduceSum / TransformReduceSum of the host layer with the
// closed forms of the reference's own test
// (legacy/tests/tensor/test_tensor_mpi_cuda_algorithms.cu:100-460): every
// interior element holds its global offset; Transform doubles it (a device
// lambda on an int tensor, as there), a copy functor carries it into a tensor
// with another halo, and a lambda casts it to long; ReduceSum gives the plain
// sum of each reduced cell and, reduced again to one cell, (size - 1) * size / 2;
// halo cells are never touched.  Then the functors that live in the library
// (scale, copy, scale-bias, sums-to-statistics), and sum / sum of squares in one
// call.  Every virtual rank of a 2 x 2 spatial decomposition is run.
#include "test_common.hpp"

template <typename T>
struct times2_functor
{
    __host__ __device__ T operator()(T x) const { return x * 2; }
};

template <typename T>
static std::vector<T> interior_values(DevTensor<T>& t, const std::vector<T>& real)
{
    std::vector<T> v;
    const Shape& ls = t.get_local_shape();
    for (index_t o = 0; o < t.get_local_size(); ++o)
        v.push_back(real[t.get_local_offset(ls.get_index(o))]);
    return v;
}

static int test_transform(const Shape& shape, const Distribution& dist, const Distribution& dist2)
{
    int errors = 0;
    const int n = static_cast<int>(dist.get_locale_shape().get_size());
    for (int r = 0; r < n; ++r)
    {
        DevTensor<int> t(shape, LocaleVirtual(r, n), dist), t2(shape, LocaleVirtual(r, n), dist2);
        DevTensor<long> t3(shape, LocaleVirtual(r, n), dist);
        t.allocate();
        t2.allocate();
        t3.allocate();
        const std::vector<int> field = global_offset_field(t, -1);
        to_device(t, field);
        to_device(t2, std::vector<int>(t2.get_local_real_size(), -7));
        to_device(t3, std::vector<long>(t3.get_local_real_size(), -9));
        Transform(t, [] __device__(int& x) { x = x * 2; });
        std::vector<int> got = to_host(t);
        for (size_t i = 0; i < got.size(); ++i)
            errors += got[i] != (field[i] == -1 ? -1 : 2 * field[i]); // halo cells keep -1 (no offset is -1)
        Transform(t, t2, [] __device__(int& x, int& y) { y = x; });
        std::vector<int> want2 = global_offset_field(t2, -7);
        std::vector<int> got2 = to_host(t2);
        for (size_t i = 0; i < got2.size(); ++i)
            errors += got2[i] != (want2[i] == -7 ? -7 : 2 * want2[i]);
        Transform(t2, t3, [] __device__(int& x, long& y) { y = static_cast<long>(x); });
        std::vector<long> got3 = to_host(t3);
        for (size_t i = 0; i < got3.size(); ++i)
            errors += got3[i] != (field[i] == -1 ? -9 : 2l * field[i]);
    }
    return errors;
}

// the library's functors on float tensors, against the same arithmetic on the host
static int test_library_functors(const Shape& shape, const Distribution& dist, const Distribution& dist2)
{
    int errors = 0;
    const int n = static_cast<int>(dist.get_locale_shape().get_size());
    for (int r = 0; r < n; ++r)
    {
        DevTensor<float> a(shape, LocaleVirtual(r, n), dist), b(shape, LocaleVirtual(r, n), dist2);
        a.allocate();
        b.allocate();
        const std::vector<float> field = global_offset_field(a, -1.0f);
        to_device(a, field);
        to_device(b, std::vector<float>(b.get_local_real_size(), -7.0f));
        Transform(a, internal::ScaleFunctor<float>(0.5f));
        std::vector<float> got = to_host(a);
        for (size_t i = 0; i < got.size(); ++i)
            errors += got[i] != (field[i] == -1.0f ? -1.0f : 0.5f * field[i]);
        Transform(a, b, internal::CopyFunctor<float>());
        const std::vector<float> wb = global_offset_field(b, -7.0f);
        std::vector<float> gb = to_host(b);
        for (size_t i = 0; i < gb.size(); ++i)
            errors += gb[i] != (wb[i] == -7.0f ? -7.0f : 0.5f * wb[i]);
        Transform(a, b, internal::ScaleBiasFunctor<float>(4.0f, 1.0f));
        gb = to_host(b);
        for (size_t i = 0; i < gb.size(); ++i)
            errors += gb[i] != (wb[i] == -7.0f ? -7.0f : 4.0f * (0.5f * wb[i]) + 1.0f);
    }
    return errors;
}

static int test_reduce(const Shape& shape, const Shape& reduce_shape, const Distribution& dist)
{
    int errors = 0;
    const int nd = shape.length();
    const int n = static_cast<int>(dist.get_locale_shape().get_size());
    Shape split = dist.get_split_shape();
    Shape locale = dist.get_locale_shape();
    for (int i = 0; i < nd; ++i)
        if (reduce_shape[i] == 1)
            split[i] = 1;
    const Distribution reduce_dist(locale, split, IntVector(nd, 0));
    // what the all-reduce over the ranks of the reference would add up: sum the ranks' results here
    std::vector<double> total;
    for (int r = 0; r < n; ++r)
    {
        DevTensor<double> t(shape, LocaleVirtual(r, n), dist);
        DevTensor<double> red(reduce_shape, LocaleVirtual(r, n), reduce_dist);
        t.allocate();
        red.allocate();
        const std::vector<double> field = global_offset_field(t, -1.0);
        to_device(t, field);
        to_device(red, std::vector<double>(red.get_local_real_size(), 0.0));
        ReduceSum<4>(t, t.get_local_shape(), red);
        const std::vector<double> got = to_host(red);
        // reference check (:243-275): each reduced cell against the plain sum of this rank's addends
        const Shape& ls = t.get_local_shape();
        std::vector<double> want(got.size(), 0.0);
        for (index_t o = 0; o < t.get_local_size(); ++o)
        {
            IndexVector idx = ls.get_index(o);
            IndexVector ridx(nd, 0);
            for (int i = 0; i < nd; ++i)
                ridx[i] = red.get_local_shape()[i] == 1 ? 0 : idx[i];
            want[red.get_local_offset(ridx)] += field[t.get_local_offset(idx)];
        }
        for (size_t i = 0; i < got.size(); ++i)
            errors += got[i] != want[i];
        // nested reduction of this rank's result to a single cell (:277-298)
        DevTensor<double> one(Shape(nd, 1), LocaleVirtual(r, n),
                              Distribution(locale, Shape(nd, 1), IntVector(nd, 0)));
        one.allocate();
        to_device(one, std::vector<double>(1, 0.0));
        ReduceSum<4>(red, red.get_local_shape(), one);
        total.push_back(to_host(one)[0]);
        // sum and sum of squares in one call
        DevTensor<double> s1(reduce_shape, LocaleVirtual(r, n), reduce_dist), s2(reduce_shape, LocaleVirtual(r, n), reduce_dist);
        s1.allocate();
        s2.allocate();
        to_device(s1, std::vector<double>(s1.get_local_real_size(), 0.0));
        to_device(s2, std::vector<double>(s2.get_local_real_size(), 0.0));
        TransformReduceSum<4>(t, t.get_local_shape(), s1, IdentityOp(), s2, SquareOp());
        const std::vector<double> g1 = to_host(s1), g2 = to_host(s2);
        std::vector<double> w2(g2.size(), 0.0);
        for (index_t o = 0; o < t.get_local_size(); ++o)
        {
            IndexVector idx = ls.get_index(o);
            IndexVector ridx(nd, 0);
            for (int i = 0; i < nd; ++i)
                ridx[i] = s2.get_local_shape()[i] == 1 ? 0 : idx[i];
            const double x = field[t.get_local_offset(idx)];
            w2[s2.get_local_offset(ridx)] += x * x;
        }
        for (size_t i = 0; i < g1.size(); ++i)
            errors += g1[i] != want[i] || g2[i] != w2[i];
    }
    double sum = 0;
    for (double v : total)
        sum += v;
    const double size = static_cast<double>(shape.get_size());
    errors += sum != (size - 1) * size / 2;
    return errors;
}

// sums_to_statistics through the four-tensor transform, against the dedicated entry point
static int test_statistics()
{
    const int C = 11;
    const Shape cs({1, 1, C, 1});
    const Distribution d = Distribution::make_localized_distribution(4);
    std::vector<float> s(C), q(C);
    for (int c = 0; c < C; ++c)
    {
        s[c] = 3.0f * c - 7.0f;
        q[c] = 50.0f + 9.0f * c;
    }
    int errors = 0;
    for (index_t n : {index_t(0), index_t(1), index_t(1000)})
    {
        DevTensor<float> mean(cs, LocaleVirtual(0, 1), d), var(cs, LocaleVirtual(0, 1), d),
            rm(cs, LocaleVirtual(0, 1), d), rv(cs, LocaleVirtual(0, 1), d);
        for (auto* t : {&mean, &var, &rm, &rv})
            t->allocate();
        to_device(mean, s);
        to_device(var, q);
        to_device(rm, std::vector<float>(C, 0.25f));
        to_device(rv, std::vector<float>(C, 0.75f));
        batchnorm::sums_to_statistics(n, 0.9f, mean, var, rm, rv, nullptr); // the Transform route
        float *m2, *v2, *rm2, *rv2;
        for (float** p : {&m2, &v2, &rm2, &rv2})
            DISTCONV_CHECK_HIP(hipMalloc(reinterpret_cast<void**>(p), C * sizeof(float)));
        std::vector<float> quarter(C, 0.25f), three(C, 0.75f);
        DISTCONV_CHECK_HIP(hipMemcpy(m2, s.data(), C * 4, hipMemcpyHostToDevice));
        DISTCONV_CHECK_HIP(hipMemcpy(v2, q.data(), C * 4, hipMemcpyHostToDevice));
        DISTCONV_CHECK_HIP(hipMemcpy(rm2, quarter.data(), C * 4, hipMemcpyHostToDevice));
        DISTCONV_CHECK_HIP(hipMemcpy(rv2, three.data(), C * 4, hipMemcpyHostToDevice));
        DISTCONV_CHECK_H2X(h2x_bn_sums_to_statistics(H2X_F32, C, n, 0.9, m2, v2, rm2, rv2, nullptr));
        std::vector<float> ref(C);
        int k = 0;
        for (auto* t : {&mean, &var, &rm, &rv})
        {
            const std::vector<float> got = to_host(*t);
            float* dev = k == 0 ? m2 : k == 1 ? v2 : k == 2 ? rm2 : rv2;
            DISTCONV_CHECK_HIP(hipMemcpy(ref.data(), dev, C * 4, hipMemcpyDeviceToHost));
            errors += std::memcmp(got.data(), ref.data(), C * 4) != 0; // bit for bit, NaNs included
            ++k;
        }
        for (float* p : {m2, v2, rm2, rv2})
            DISTCONV_CHECK_HIP(hipFree(p));
    }
    return errors;
}

int main()
{
    std::setvbuf(stdout, nullptr, _IONBF, 0); // what was printed survives a crash
    int errors = 0;
    const Shape s4({12, 10, 3, 4});
    const Distribution plain = Distribution::make_distribution(Shape({2, 2, 1, 1}));
    const Distribution halo = Distribution::make_overlapped_distribution(Shape({2, 2, 1, 1}), IntVector({1, 2, 0, 0}));
    errors += test_transform(s4, halo, plain);
    errors += test_transform(s4, plain, halo);
    errors += test_library_functors(s4, halo, plain);
    errors += test_library_functors(Shape({7, 5, 3, 2, 2}), Distribution::make_overlapped_distribution(Shape({1, 2, 2, 1, 1}), IntVector({0, 1, 1, 0, 0})),
                                    Distribution::make_distribution(Shape({1, 2, 2, 1, 1})));
    for (const Shape& rs : {Shape({1, 1, 3, 1}), Shape({12, 10, 1, 1}), Shape({1, 10, 3, 4}), Shape({1, 1, 1, 1}),
                            Shape({12, 1, 1, 4})})
    {
        errors += test_reduce(s4, rs, halo);
        errors += test_reduce(s4, rs, plain);
    }
    errors += test_statistics();
    std::printf("test_algorithms: %d errors\n", errors);
    // tensor::ReduceSum keep a buffer per stream until release_workspaces(), which finish() calls
    CHECK(h2x_host::StreamScratch::held_buffers() > 0);
    return finish(errors);
}

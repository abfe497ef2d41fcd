// BatchNormalization<BackendMI355X, float> and Softmax<BackendMI355X> through
// the C++ layer against the CPU oracle (linked from oracle/libh2x_oracle.so),
// with the reference's comparison metric max(|d/v1|, |d/v2|) <= 1e-5
// (legacy/tests/compare_binary_files.cpp:47-49).  Setup follows
// legacy/benchmarks/distconv_benchmark_bn.cpp:200-213: running_mean = 0,
// running_var = 1, decay 0.9, epsilon 1e-5.
#include "test_common.hpp"

extern "C" {
void orc_bn_channel_sums_and_sqsums_f32(int, int, size_t, size_t, const float*, float*, float*);
void orc_bn_sums_to_statistics_f32(int, size_t, float, float*, float*, float*, float*);
void orc_bn_batch_normalization_f32(int, int, size_t, size_t, size_t, const float*, const float*,
                                    const float*, const float*, const float*, float*, float);
void orc_bn_backprop1_f32(int, int, size_t, size_t, size_t, const float*, const float*, const float*,
                          const float*, const float*, float*, float*, float*, float*, float);
void orc_bn_backprop2_f32(int, int, size_t, size_t, size_t, size_t, size_t, const float*, const float*,
                          const float*, const float*, const float*, const float*, const float*, float*,
                          float);
void orc_softmax_channel_forward_f32(int, int, size_t, const float*, float*);
void orc_softmax_channel_backward_f32(int, int, size_t, const float*, const float*, float*);
}

static double max_rel(const std::vector<float>& a, const std::vector<float>& b)
{
    CHECK(a.size() == b.size());
    double m = 0;
    for (size_t i = 0; i < a.size(); ++i)
    {
        const double d = std::fabs((double) a[i] - (double) b[i]);
        if (d == 0)
            continue;
        m = std::max(m, std::max(d / std::fabs((double) a[i]), d / std::fabs((double) b[i])));
    }
    return m;
}

static std::vector<float> randn(size_t n, unsigned seed, float sigma = 1.0f, float mu = 0.0f)
{
    std::mt19937 gen(seed);
    std::normal_distribution<float> d(mu, sigma);
    std::vector<float> v(n);
    for (auto& x : v)
        x = d(gen);
    return v;
}

static int test_bn(const Shape& shape)
{
    const int nd = shape.length();
    const int C = static_cast<int>(shape[-2]), N = static_cast<int>(shape[-1]);
    const size_t S = shape.get_size() / C / N;
    const Distribution dist = Distribution::make_localized_distribution(nd);
    const LocaleVirtual loc(0, 1);
    Shape pshape(nd, 1);
    pshape[-2] = C;
    DevTensor<float> x(shape, loc, dist), y(shape, loc, dist), dy(shape, loc, dist), dx(shape, loc, dist);
    DevTensor<float> mean(pshape, loc, dist), var(pshape, loc, dist), rmean(pshape, loc, dist),
        rvar(pshape, loc, dist), scale(pshape, loc, dist), bias(pshape, loc, dist),
        dscale(pshape, loc, dist), dbias(pshape, loc, dist), dmean(pshape, loc, dist), dvar(pshape, loc, dist);
    for (auto* t : {&x, &y, &dy, &dx, &mean, &var, &rmean, &rvar, &scale, &bias, &dscale, &dbias, &dmean, &dvar})
        t->allocate();
    const auto hx = randn(shape.get_size(), 1), hdy = randn(shape.get_size(), 2);
    auto hscale = randn(C, 3, 0.25f, 1.0f), hbias = randn(C, 4, 0.1f);
    to_device(x, hx);
    to_device(dy, hdy);
    to_device(scale, hscale);
    to_device(bias, hbias);
    to_device(rvar, std::vector<float>(C, 1.0f));

    BackendMI355X backend;
    BatchNormalization<BackendMI355X, float> bn(backend, nd, 0.9f, 1e-5f, false);
    CHECK(bn.forward(x, mean, var, rmean, rvar, scale, bias, y, true) == 0);
    CHECK(bn.backward(x, dy, mean, var, scale, dscale, dbias, dmean, dvar, dx) == 0);

    std::vector<float> om(C), ov(C), orm(C, 0.0f), orv(C, 1.0f), oy(hx.size()), ods(C), odb(C), odm(C),
        odv(C), odx(hx.size());
    orc_bn_channel_sums_and_sqsums_f32(N, C, S, S, hx.data(), om.data(), ov.data());
    orc_bn_sums_to_statistics_f32(C, (size_t) N * S, 0.9f, om.data(), ov.data(), orm.data(), orv.data());
    orc_bn_batch_normalization_f32(N, C, S, S, S, hx.data(), om.data(), ov.data(), hscale.data(),
                                   hbias.data(), oy.data(), 1e-5f);
    orc_bn_backprop1_f32(N, C, S, S, S, hx.data(), hdy.data(), om.data(), ov.data(), hscale.data(),
                         ods.data(), odb.data(), odm.data(), odv.data(), 1e-5f);
    orc_bn_backprop2_f32(N, C, S, S, S, S, (size_t) N * S, hx.data(), hdy.data(), om.data(), ov.data(),
                         hscale.data(), odm.data(), odv.data(), odx.data(), 1e-5f);
    int errors = 0;
    const double tol = 1e-5;
    errors += max_rel(to_host(mean), om) > tol;
    errors += max_rel(to_host(var), ov) > tol;
    errors += max_rel(to_host(rmean), orm) > tol;
    errors += max_rel(to_host(rvar), orv) > tol;
    errors += max_rel(to_host(y), oy) > tol;
    errors += max_rel(to_host(dscale), ods) > tol;
    errors += max_rel(to_host(dbias), odb) > tol;
    errors += max_rel(to_host(dmean), odm) > tol;
    errors += max_rel(to_host(dvar), odv) > tol;
    errors += max_rel(to_host(dx), odx) > tol;

    // the free functions with the reference's own signatures
    batchnorm::channel_sums_and_sqsums(nd, N, x, mean, var, (hipStream_t) nullptr);
    batchnorm::sums_to_statistics((index_t) N * S, 0.9f, mean, var, rmean, rvar, (hipStream_t) nullptr);
    errors += max_rel(to_host(mean), om) > tol;
    // inference path normalises with the running statistics
    CHECK(bn.forward(x, mean, var, rmean, rvar, scale, bias, y, false) == 0);
    const auto hrm = to_host(rmean), hrv = to_host(rvar);
    orc_bn_batch_normalization_f32(N, C, S, S, S, hx.data(), hrm.data(), hrv.data(), hscale.data(),
                                   hbias.data(), oy.data(), 1e-5f);
    errors += max_rel(to_host(y), oy) > tol;
    return errors;
}

static int test_softmax(const Shape& shape)
{
    const int nd = shape.length();
    const int C = static_cast<int>(shape[-2]), N = static_cast<int>(shape[-1]);
    const size_t S = shape.get_size() / C / N;
    const Distribution dist = Distribution::make_localized_distribution(nd);
    const LocaleVirtual loc(0, 1);
    DevTensor<float> x(shape, loc, dist), y(shape, loc, dist), dy(shape, loc, dist), dx(shape, loc, dist);
    for (auto* t : {&x, &y, &dy, &dx})
        t->allocate();
    const auto hx = randn(shape.get_size(), 5, 2.0f), hdy = randn(shape.get_size(), 6);
    to_device(x, hx);
    to_device(dy, hdy);
    BackendMI355X backend;
    Softmax<BackendMI355X> sm(backend);
    sm.setup(x, SoftmaxMode::CHANNEL);
    CHECK(sm.forward(x, y) == 0);
    CHECK(sm.backward(y, dy, dx) == 0);
    const auto hy = to_host(y);
    std::vector<float> oy(hx.size()), odx(hx.size());
    orc_softmax_channel_forward_f32(N, C, S, hx.data(), oy.data());
    orc_softmax_channel_backward_f32(N, C, S, hy.data(), hdy.data(), odx.data());
    return (max_rel(hy, oy) > 1e-5) + (max_rel(to_host(dx), odx) > 1e-5);
}

int main()
{
    int errors = 0;
    errors += test_bn(Shape({56, 56, 64, 8}));   // BASELINE config 1
    errors += test_bn(Shape({5, 7, 3, 2}));
    errors += test_bn(Shape({16, 16, 16, 8, 4})); // 5-D
    errors += test_softmax(Shape({64, 64, 21, 4}));
    errors += test_softmax(Shape({5, 3, 7, 2}));
    std::printf("test_batchnorm_softmax: %d errors\n", errors);
    return errors ? 1 : 0;
}

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
void orc_softmax_instance_max_f32(int, size_t, const float*, float*);
void orc_softmax_instance_exp_f32(int, size_t, const float*, const float*, float*, float*);
void orc_softmax_instance_normalize_f32(int, size_t, const float*, float*);
void orc_softmax_instance_dot_f32(int, size_t, const float*, const float*, float*);
void orc_softmax_instance_gradient_f32(int, size_t, const float*, const float*, const float*, float*);
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

static int test_softmax_instance(const Shape& shape)
{
    const int nd = shape.length();
    const int N = static_cast<int>(shape[-1]);
    const size_t size = shape.get_size() / N;
    const Distribution dist = Distribution::make_localized_distribution(nd);
    const LocaleVirtual loc(0, 1);
    DevTensor<float> x(shape, loc, dist), y(shape, loc, dist), dy(shape, loc, dist), dx(shape, loc, dist);
    for (auto* t : {&x, &y, &dy, &dx})
        t->allocate();
    const auto hx = randn(shape.get_size(), 7, 2.0f), hdy = randn(shape.get_size(), 8);
    to_device(x, hx);
    to_device(dy, hdy);
    BackendMI355X backend;
    Softmax<BackendMI355X> sm(backend);
    sm.setup(x, SoftmaxMode::INSTANCE);
    CHECK(sm.forward(x, y) == 0);
    CHECK(sm.backward(y, dy, dx) == 0);
    const auto hy = to_host(y), hdx = to_host(dx);
    std::vector<float> mx(N), ex(N), dp(N), oy(hx.size()), odx(hx.size());
    orc_softmax_instance_max_f32(N, size, hx.data(), mx.data());
    orc_softmax_instance_exp_f32(N, size, hx.data(), mx.data(), oy.data(), ex.data());
    orc_softmax_instance_normalize_f32(N, size, ex.data(), oy.data());
    orc_softmax_instance_dot_f32(N, size, hy.data(), hdy.data(), dp.data());
    orc_softmax_instance_gradient_f32(N, size, hy.data(), hdy.data(), dp.data(), odx.data());
    int errors = max_rel(hy, oy) > 1e-5;
    // dx = y * (dy - dp) cancels where dy ~ dp: bound relative to the operands
    for (size_t i = 0; i < hdx.size(); ++i)
    {
        const double bound = 1e-5 * std::fabs(hy[i]) * (std::fabs(hdy[i]) + std::fabs(dp[i / size]) + 1e-3);
        if (std::fabs((double) hdx[i] - (double) odx[i]) > bound + 1e-30)
        {
            ++errors;
            break;
        }
    }
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

// A spatially decomposed tensor with halos on the inner spatial dimensions must
// give, rank by rank, what a halo-free tensor with the same interior gives
// (generic vs optimised kernels, the reference's own validation idea:
// legacy/tests/dnn_backend/test_cudnn_util.sh.in:339-410).
static int test_bn_haloed()
{
    const Shape shape({16, 12, 6, 2});
    const Shape locale({2, 2, 1, 1});
    const Distribution dh = Distribution::make_overlapped_distribution(locale, IntVector({1, 2, 0, 0}));
    const Distribution dp = Distribution::make_distribution(locale);
    Shape pshape({1, 1, 6, 1});
    const Distribution dl = Distribution::make_localized_distribution(4);
    int errors = 0;
    for (int r = 0; r < 4; ++r)
    {
        const LocaleVirtual loc(r, 4), one(0, 1);
        DevTensor<float> xh(shape, loc, dh), yh(shape, loc, dh), dyh(shape, loc, dp), dxh(shape, loc, dh);
        DevTensor<float> xp(shape, loc, dp), yp(shape, loc, dp), dxp(shape, loc, dp);
        std::vector<DevTensor<float>> pv;
        for (int i = 0; i < 20; ++i)
        {
            pv.emplace_back(pshape, one, dl);
            pv.back().allocate();
        }
        for (auto* t : {&xh, &yh, &dyh, &dxh, &xp, &yp, &dxp})
            t->allocate();
        // same interior in the haloed and the plain tensor
        const auto vals = randn(xp.get_local_size(), 100 + r), dvals = randn(xp.get_local_size(), 200 + r);
        std::vector<float> hx(xh.get_local_real_size(), NAN);
        const Shape& ls = xh.get_local_shape();
        for (index_t o = 0; o < xh.get_local_size(); ++o)
            hx[xh.get_local_offset(ls.get_index(o))] = vals[o];
        to_device(xh, hx);
        to_device(xp, vals);
        to_device(dyh, dvals);
        to_device(pv[4], randn(6, 3, 0.25f, 1.0f)); // scale
        to_device(pv[5], randn(6, 4, 0.1f));         // bias
        to_device(pv[14], to_host(pv[4]));
        to_device(pv[15], to_host(pv[5]));
        to_device(pv[3], std::vector<float>(6, 1.0f));
        to_device(pv[13], std::vector<float>(6, 1.0f));
        BackendMI355X backend;
        BatchNormalization<BackendMI355X, float> bh(backend, 4, 0.9f, 1e-5f, false), bp(backend, 4, 0.9f, 1e-5f, false);
        bh.forward(xh, pv[0], pv[1], pv[2], pv[3], pv[4], pv[5], yh, true);
        bh.backward(xh, dyh, pv[0], pv[1], pv[4], pv[6], pv[7], pv[8], pv[9], dxh);
        bp.forward(xp, pv[10], pv[11], pv[12], pv[13], pv[14], pv[15], yp, true);
        bp.backward(xp, dyh, pv[10], pv[11], pv[14], pv[16], pv[17], pv[18], pv[19], dxp);
        // the two paths add the same fp64 terms in different orders: equal to rounding
        for (int k : {0, 1, 2, 3, 6, 7, 8, 9})
            errors += max_rel(to_host(pv[k]), to_host(pv[k + 10])) > 1e-6;
        const auto hy = to_host(yh), py = to_host(yp), hdx = to_host(dxh), pdx = to_host(dxp);
        std::vector<float> iy(py.size()), idx(py.size());
        for (index_t o = 0; o < xh.get_local_size(); ++o)
        {
            const index_t off = xh.get_local_offset(ls.get_index(o));
            iy[o] = hy[off];
            idx[o] = hdx[off];
        }
        errors += max_rel(iy, py) > 1e-5;
        errors += max_rel(idx, pdx) > 1e-5;
        // halo cells of the outputs keep the allocator's zeros
        double halo_sum = 0;
        for (float v : hy)
            halo_sum += std::fabs(v);
        double inner_sum = 0;
        for (float v : iy)
            inner_sum += std::fabs(v);
        errors += std::fabs(halo_sum - inner_sum) > 1e-3 * inner_sum;
    }
    return errors;
}

// set_clear_output_halo: the outputs of normalise and of the input gradient equal, in every cell
// of the real tensors, what the plain calls followed by clear_halo on every dimension leave.
static int test_bn_clearing()
{
    const Shape shape({20, 12, 10, 3, 2});
    const Shape locale({2, 2, 2, 1, 1});
    const Distribution dh = Distribution::make_overlapped_distribution(locale, IntVector({1, 2, 1, 0, 0}));
    Shape pshape({1, 1, 1, 3, 1});
    const Distribution dl = Distribution::make_localized_distribution(5);
    int errors = 0;
    for (int r : {0, 5})
    {
        const LocaleVirtual loc(r, 8), one(0, 1);
        std::vector<std::vector<float>> outs[2];
        for (int clearing = 0; clearing < 2; ++clearing)
        {
            DevTensor<float> x(shape, loc, dh), y(shape, loc, dh), dy(shape, loc, dh), dx(shape, loc, dh);
            std::vector<DevTensor<float>> pv;
            for (int i = 0; i < 10; ++i)
            {
                pv.emplace_back(pshape, one, dl);
                pv.back().allocate();
            }
            for (auto* t : {&x, &y, &dy, &dx})
                t->allocate();
            to_device(x, randn(x.get_local_real_size(), 300 + r));   // halo cells hold values too
            to_device(dy, randn(x.get_local_real_size(), 400 + r));
            to_device(y, std::vector<float>(x.get_local_real_size(), NAN));
            to_device(dx, std::vector<float>(x.get_local_real_size(), NAN));
            to_device(pv[4], randn(3, 3, 0.25f, 1.0f));
            to_device(pv[5], randn(3, 4, 0.1f));
            to_device(pv[3], std::vector<float>(3, 1.0f));
            BackendMI355X backend;
            BatchNormalization<BackendMI355X, float> bn(backend, 5, 0.9f, 1e-5f, false);
            bn.set_clear_output_halo(clearing == 1);
            bn.forward(x, pv[0], pv[1], pv[2], pv[3], pv[4], pv[5], y, true);
            bn.backward(x, dy, pv[0], pv[1], pv[4], pv[6], pv[7], pv[8], pv[9], dx);
            if (!clearing)
                for (int d = 0; d < 3; ++d)
                {
                    y.clear_halo(d, nullptr);
                    dx.clear_halo(d, nullptr);
                }
            outs[clearing] = {to_host(y), to_host(dx), to_host(pv[0]), to_host(pv[1]), to_host(pv[6]),
                              to_host(pv[7]), to_host(pv[8]), to_host(pv[9])};
        }
        for (size_t k = 0; k < outs[0].size(); ++k)
            errors += std::memcmp(outs[0][k].data(), outs[1][k].data(), outs[0][k].size() * sizeof(float)) != 0;
    }
    return errors;
}

int main()
{
    std::setvbuf(stdout, nullptr, _IONBF, 0); // what was printed survives a crash
    int errors = 0;
    errors += test_bn_haloed();
    errors += test_bn_clearing();
    {
        // util::Clock brackets work on a stream, as the reference's benchmark does
        // (legacy/benchmarks/distconv_benchmark_bn.cpp:254-295); sync_stream orders two streams
        hipStream_t a, b;
        DISTCONV_CHECK_HIP(hipStreamCreate(&a));
        DISTCONV_CHECK_HIP(hipStreamCreate(&b));
        util::Clock clk(a);
        clk.start();
        util::sync_stream(a, b);
        clk.stop();
        const float ms = clk.get_time();
        CHECK(ms >= 0.0f && ms < 1000.0f);
        DISTCONV_CHECK_HIP(hipStreamSynchronize(b));
        DISTCONV_CHECK_HIP(hipStreamDestroy(a));
        DISTCONV_CHECK_HIP(hipStreamDestroy(b));
    }
    errors += test_bn(Shape({56, 56, 64, 8}));   // BASELINE config 1
    errors += test_bn(Shape({5, 7, 3, 2}));
    errors += test_bn(Shape({16, 16, 16, 8, 4})); // 5-D
    errors += test_softmax(Shape({64, 64, 21, 4}));
    errors += test_softmax(Shape({5, 3, 7, 2}));
    errors += test_softmax_instance(Shape({32, 32, 21, 4}));
    errors += test_softmax_instance(Shape({5, 3, 7, 2}));
    std::printf("test_batchnorm_softmax: %d errors\n", errors);
    // the free functions with the reference's signatures keep a buffer per stream until release_workspaces(), which finish() calls
    CHECK(h2x_host::StreamScratch::held_buffers() > 0);
    return finish(errors);
}

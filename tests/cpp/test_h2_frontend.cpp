// The h2 operator front-end (dihydrogen_amd/host/include/h2) over libh2x.so:
// typed and type-erased calls against the CPU oracle (reference metric
// max(|d/v1|, |d/v2|) <= 1e-5, legacy/tests/compare_binary_files.cpp:47-49),
// strided views against contiguous tensors, halo pack/unpack bit-exact, and the
// errors of the dispatch registry (tests of the same shape as
// test/unit_test/core/unit_test_dispatch.cpp and tensor/unit_test_fill.cpp).
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include <unistd.h>

#include "h2/ops_mi355x.hpp"

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

using namespace h2;

#define CHECK(cond)                                                                                \
    do                                                                                             \
    {                                                                                              \
        if (!(cond))                                                                               \
        {                                                                                          \
            std::printf("FAILED %s at %s:%d\n", #cond, __FILE__, __LINE__);                        \
            std::exit(1);                                                                          \
        }                                                                                          \
    } while (0)

#define CHECK_THROWS(stmt)                                                                         \
    do                                                                                             \
    {                                                                                              \
        bool thrown = false;                                                                       \
        try                                                                                        \
        {                                                                                          \
            stmt;                                                                                  \
        }                                                                                          \
        catch (const H2FatalException&)                                                            \
        {                                                                                          \
            thrown = true;                                                                         \
        }                                                                                          \
        if (!thrown)                                                                               \
        {                                                                                          \
            std::printf("FAILED: no exception from %s at %s:%d\n", #stmt, __FILE__, __LINE__);     \
            std::exit(1);                                                                          \
        }                                                                                          \
    } while (0)

template <typename T>
static void upload(Tensor<T>& t, const std::vector<T>& h)
{
    CHECK(t.is_contiguous() && static_cast<size_t>(t.numel()) == h.size());
    check_hip(hipMemcpy(t.data(), h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice), "upload");
}

template <typename T>
static std::vector<T> download(const Tensor<T>& t)
{
    CHECK(t.is_contiguous());
    std::vector<T> h(t.numel());
    check_hip(hipDeviceSynchronize(), "sync");
    check_hip(hipMemcpy(h.data(), t.const_data(), h.size() * sizeof(T), hipMemcpyDeviceToHost),
              "download");
    return h;
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

static DTTuple channel_types(int nd)
{
    DTTuple t;
    for (int i = 0; i < nd - 2; ++i)
        t.append(DT::Spatial);
    t.append(DT::Channel);
    t.append(DT::Sample);
    return t;
}

// A strided tensor holding `values` at its elements (natural order), everything else `fill`.
template <typename T>
static std::vector<T> scatter_strided(const ShapeTuple& shape, const StrideTuple& strides, size_t span,
                                      const std::vector<T>& values, T fill)
{
    std::vector<T> h(span, fill);
    size_t i = 0;
    const StrideTuple s[1] = {strides};
    mi355x::for_each_element(shape, s, [&](const DataIndexType* o) { h[o[0]] = values[i++]; });
    return h;
}

// Batch norm forward + backward through the type-erased operators.
static void test_batchnorm(const ShapeTuple& shape)
{
    const int nd = shape.size();
    const int C = shape[nd - 2], N = shape[nd - 1];
    const size_t total = product<size_t>(shape), S = total / C / N;
    const ComputeStream stream(Device::GPU);
    const DTTuple types = channel_types(nd);
    Tensor<float> x(Device::GPU, shape, types, stream), y(Device::GPU, shape, types, stream),
        dy(Device::GPU, shape, types, stream), dx(Device::GPU, shape, types, stream);
    const ShapeTuple cshape{C};
    const DTTuple ctypes{DT::Channel};
    auto cvec = [&] { return Tensor<float>(Device::GPU, cshape, ctypes, stream); };
    Tensor<float> mean = cvec(), var = cvec(), rm = cvec(), rv = cvec(), scale = cvec(), bias = cvec(),
                  dscale = cvec(), dbias = cvec(), dmean = cvec(), dvar = cvec();
    const std::vector<float> hx = randn(total, 1, 1.0f, 0.3f), hdy = randn(total, 2);
    std::vector<float> hscale(C), hbias(C);
    for (int c = 0; c < C; ++c)
    {
        hscale[c] = 0.5f + 0.01f * c;
        hbias[c] = 0.1f * std::sin((float) c);
    }
    upload(x, hx);
    upload(dy, hdy);
    upload(scale, hscale);
    upload(bias, hbias);
    upload(rm, std::vector<float>(C, 0.0f));
    upload(rv, std::vector<float>(C, 1.0f));

    BaseTensor &bx = x, &by = y, &bdy = dy, &bdx = dx, &bmean = mean, &bvar = var, &brm = rm, &brv = rv,
               &bscale = scale, &bbias = bias, &bdscale = dscale, &bdbias = dbias, &bdmean = dmean,
               &bdvar = dvar;
    const size_t n = (size_t) N * S;
    batchnorm_channel_sums(bx, bmean, bvar);
    batchnorm_statistics(bmean, bvar, brm, brv, n, 0.9);
    batchnorm_normalize(bx, bmean, bvar, bscale, bbias, by, 1e-5);
    batchnorm_backprop1(bx, bdy, bmean, bvar, bscale, bdscale, bdbias, bdmean, bdvar, 1e-5);
    batchnorm_backprop2(bx, bdy, bmean, bvar, bscale, bdmean, bdvar, bdx, n, 1e-5);

    std::vector<float> om(C), ov(C), orm(C, 0.0f), orv(C, 1.0f), oy(total), ods(C), odb(C), odm(C),
        odv(C), odx(total);
    orc_bn_channel_sums_and_sqsums_f32(N, C, S, S, hx.data(), om.data(), ov.data());
    orc_bn_sums_to_statistics_f32(C, n, 0.9f, om.data(), ov.data(), orm.data(), orv.data());
    orc_bn_batch_normalization_f32(N, C, S, S, S, hx.data(), om.data(), ov.data(), hscale.data(),
                                   hbias.data(), oy.data(), 1e-5f);
    orc_bn_backprop1_f32(N, C, S, S, S, hx.data(), hdy.data(), om.data(), ov.data(), hscale.data(),
                         ods.data(), odb.data(), odm.data(), odv.data(), 1e-5f);
    orc_bn_backprop2_f32(N, C, S, S, S, S, n, hx.data(), hdy.data(), om.data(), ov.data(),
                         hscale.data(), odm.data(), odv.data(), odx.data(), 1e-5f);
    CHECK(max_rel(download(mean), om) <= 1e-5);
    CHECK(max_rel(download(var), ov) <= 1e-5);
    CHECK(max_rel(download(rm), orm) <= 1e-5);
    CHECK(max_rel(download(rv), orv) <= 1e-5);
    CHECK(max_rel(download(y), oy) <= 1e-5);
    CHECK(max_rel(download(dscale), ods) <= 1e-5);
    CHECK(max_rel(download(dbias), odb) <= 1e-5);
    CHECK(max_rel(download(dmean), odm) <= 1e-5);
    CHECK(max_rel(download(dvar), odv) <= 1e-5);
    CHECK(max_rel(download(dx), odx) <= 1e-5);

    // the typed front gives the same bits as the type-erased one
    Tensor<float> y2(Device::GPU, shape, types, stream);
    batchnorm_normalize(x, mean, var, scale, bias, y2, 1e-5);
    CHECK(download(y2) == download(y));

    // the two-launch operators give the bits of the staged ones, dx in place included
    Tensor<float> mean2 = cvec(), var2 = cvec(), rm2 = cvec(), rv2 = cvec(), dscale2 = cvec(),
                  dbias2 = cvec(), dmean2 = cvec(), dvar2 = cvec();
    Tensor<float> y3(Device::GPU, shape, types, stream), xc(Device::GPU, shape, types, stream);
    upload(rm2, std::vector<float>(C, 0.0f));
    upload(rv2, std::vector<float>(C, 1.0f));
    upload(xc, hx);
    BaseTensor &bmean2 = mean2, &bvar2 = var2, &brm2 = rm2, &brv2 = rv2, &by3 = y3, &bxc = xc,
               &bdscale2 = dscale2, &bdbias2 = dbias2, &bdmean2 = dmean2, &bdvar2 = dvar2;
    batchnorm_forward(bx, bscale, bbias, bmean2, bvar2, brm2, brv2, by3, n, 0.9, 1e-5);
    CHECK(download(mean2) == download(mean));
    CHECK(download(var2) == download(var));
    CHECK(download(rm2) == download(rm));
    CHECK(download(rv2) == download(rv));
    CHECK(download(y3) == download(y));
    batchnorm_backward(bxc, bdy, bmean, bvar, bscale, bdscale2, bdbias2, bdmean2, bdvar2, bxc, n, 1e-5);
    CHECK(download(dscale2) == download(dscale));
    CHECK(download(dbias2) == download(dbias));
    CHECK(download(dmean2) == download(dmean));
    CHECK(download(dvar2) == download(dvar));
    CHECK(download(xc) == download(dx));
}

// A view with padded rows (stride of dimension 1 larger than the extent of
// dimension 0) gives what the contiguous tensor gives on the same elements.
static void test_strided_view()
{
    const int W = 12, H = 5, C = 6, N = 3, pitch = 16;
    const ShapeTuple shape{W, H, C, N};
    const DTTuple types = channel_types(4);
    const ComputeStream stream(Device::GPU);
    const StrideTuple padded{1, pitch, (DataIndexType) pitch * H, (DataIndexType) pitch * H * C};
    const size_t total = (size_t) W * H * C * N, padded_total = (size_t) pitch * H * C * N;
    const std::vector<float> hx = randn(total, 7, 2.0f, -1.0f);
    std::vector<float> hp(padded_total, 1e30f); // the padding must never be read
    for (size_t i = 0; i < total; ++i)
    {
        const size_t w = i % W, rest = i / W;
        hp[rest * pitch + w] = hx[i];
    }
    Tensor<float> x(Device::GPU, shape, types, stream);
    upload(x, hx);
    float* raw = nullptr;
    check_hip(hipMalloc(&raw, padded_total * sizeof(float)), "hipMalloc");
    check_hip(hipMemcpy(raw, hp.data(), padded_total * sizeof(float), hipMemcpyHostToDevice), "copy");
    Tensor<float> view(Device::GPU, raw, shape, types, padded, stream);
    CHECK(!view.is_contiguous() && view.is_view());
    const ShapeTuple cshape{C};
    const DTTuple ctypes{DT::Channel};
    Tensor<float> s1(Device::GPU, cshape, ctypes, stream), q1(Device::GPU, cshape, ctypes, stream),
        s2(Device::GPU, cshape, ctypes, stream), q2(Device::GPU, cshape, ctypes, stream);
    batchnorm_channel_sums(x, s1, q1);
    batchnorm_channel_sums(view, s2, q2);
    CHECK(max_rel(download(s1), download(s2)) <= 1e-6);
    CHECK(max_rel(download(q1), download(q2)) <= 1e-6);

    // the two-launch forward reads the view and leaves the bits of the staged operators
    Tensor<float> scale(Device::GPU, cshape, ctypes, stream), bias(Device::GPU, cshape, ctypes, stream),
        rm(Device::GPU, cshape, ctypes, stream), rv(Device::GPU, cshape, ctypes, stream),
        rm2(Device::GPU, cshape, ctypes, stream), rv2(Device::GPU, cshape, ctypes, stream),
        m2(Device::GPU, cshape, ctypes, stream), v2(Device::GPU, cshape, ctypes, stream);
    Tensor<float> y1(Device::GPU, shape, types, stream), y2(Device::GPU, shape, types, stream);
    upload(scale, std::vector<float>(C, 1.5f));
    upload(bias, std::vector<float>(C, -0.25f));
    for (Tensor<float>* t : {&rm, &rm2})
        upload(*t, std::vector<float>(C, 0.0f));
    for (Tensor<float>* t : {&rv, &rv2})
        upload(*t, std::vector<float>(C, 1.0f));
    const size_t n = (size_t) W * H * N;
    batchnorm_statistics(s2, q2, rm, rv, n, 0.9);
    batchnorm_normalize(view, s2, q2, scale, bias, y1, 1e-5);
    batchnorm_forward(view, scale, bias, m2, v2, rm2, rv2, y2, n, 0.9, 1e-5);
    CHECK(download(m2) == download(s2));
    CHECK(download(v2) == download(q2));
    CHECK(download(rm2) == download(rm));
    CHECK(download(y2) == download(y1));
    check_hip(hipDeviceSynchronize(), "sync");
    check_hip(hipFree(raw), "hipFree");
}

static void test_softmax()
{
    const ShapeTuple shape{16, 8, 21, 2};
    const DTTuple types = channel_types(4);
    const ComputeStream stream(Device::GPU);
    const size_t total = product<size_t>(shape), S = 16 * 8;
    Tensor<float> x(Device::GPU, shape, types, stream), y(Device::GPU, shape, types, stream),
        dy(Device::GPU, shape, types, stream), dx(Device::GPU, shape, types, stream);
    const std::vector<float> hx = randn(total, 3, 2.0f), hdy = randn(total, 4);
    upload(x, hx);
    upload(dy, hdy);
    BaseTensor &bx = x, &by = y, &bdy = dy, &bdx = dx;
    softmax_channel_forward(bx, by);
    softmax_channel_backward(by, bdy, bdx);
    std::vector<float> oy(total), odx(total);
    orc_softmax_channel_forward_f32(2, 21, S, hx.data(), oy.data());
    orc_softmax_channel_backward_f32(2, 21, S, oy.data(), hdy.data(), odx.data());
    CHECK(max_rel(download(y), oy) <= 1e-5);
    CHECK(max_rel(download(dx), odx) <= 1e-5);
}

// Pack the RHS interior strip of one tensor, unpack it into the LHS halo of
// another: the halo then holds the neighbour's boundary values, bit for bit.
static void test_halo()
{
    const ShapeTuple shape{10, 6, 3, 2}; // 8 interior columns + one halo column on each side
    const DTTuple types = channel_types(4);
    const ComputeStream stream(Device::GPU);
    const size_t total = product<size_t>(shape);
    std::vector<double> ha(total), hb(total, -1.0);
    for (size_t i = 0; i < total; ++i)
        ha[i] = 0.5 * (double) i;
    Tensor<double> a(Device::GPU, shape, types, stream), b(Device::GPU, shape, types, stream);
    upload(a, ha);
    upload(b, hb);
    Tensor<double> buf(Device::GPU, ShapeTuple{6 * 3 * 2}, DTTuple{DT::Any}, stream);
    BaseTensor &ba = a, &bb = b, &bbuf = buf;
    halo_pack(ba, 0, H2X_RHS, 1, bbuf);
    halo_unpack(bb, 0, H2X_LHS, 1, bbuf);
    const std::vector<double> got = download(b);
    for (size_t row = 0; row < total / 10; ++row)
        for (int w = 0; w < 10; ++w)
            CHECK(got[row * 10 + w] == (w == 0 ? ha[row * 10 + 8] : -1.0));
    // SUM unpack of the reverse direction adds the neighbour's halo onto the boundary cells
    halo_pack(ba, 0, H2X_RHS, 1, bbuf, true);           // a's RHS halo column (w = 9)
    halo_unpack(bb, 0, H2X_LHS, 1, bbuf, true, H2X_HALO_SUM); // onto b's first interior column (w = 1)
    const std::vector<double> sum = download(b);
    for (size_t row = 0; row < total / 10; ++row)
        CHECK(sum[row * 10 + 1] == -1.0 + ha[row * 10 + 9]);
}

static void test_errors()
{
    const ComputeStream stream(Device::GPU);
    const ShapeTuple shape{8, 4, 3, 2};
    Tensor<float> x(Device::GPU, shape, channel_types(4), stream);
    Tensor<float> s(Device::GPU, ShapeTuple{3}, DTTuple{DT::Channel}, stream),
        q(Device::GPU, ShapeTuple{3}, DTTuple{DT::Channel}, stream);
    // dimension tags decide the layout: a tensor tagged differently is rejected
    Tensor<float> wrong(Device::GPU, shape, DTTuple{DT::Spatial, DT::Channel, DT::Spatial, DT::Sample},
                        stream);
    CHECK_THROWS(batchnorm_channel_sums(wrong, s, q));
    // per-channel vectors of the wrong length
    Tensor<float> s4(Device::GPU, ShapeTuple{4}, DTTuple{DT::Channel}, stream);
    CHECK_THROWS(batchnorm_channel_sums(x, s4, q));
    // no CPU implementation
    Tensor<float> cx(Device::CPU, shape, channel_types(4)), cs(Device::CPU, ShapeTuple{3}, DTTuple{DT::Channel}),
        cq(Device::CPU, ShapeTuple{3}, DTTuple{DT::Channel});
    CHECK_THROWS(batchnorm_channel_sums(cx, cs, cq));
    // an element type nobody registered
    Tensor<std::int32_t> ix(Device::GPU, shape, channel_types(4), stream),
        is(Device::GPU, ShapeTuple{3}, DTTuple{DT::Channel}, stream),
        iq(Device::GPU, ShapeTuple{3}, DTTuple{DT::Channel}, stream);
    BaseTensor &bix = ix, &bis = is, &biq = iq;
    CHECK_THROWS(batchnorm_channel_sums(bix, bis, biq));
    // mixed element types
    Tensor<double> ds(Device::GPU, ShapeTuple{3}, DTTuple{DT::Channel}, stream);
    BaseTensor &bx = x, &bds = ds, &bq = q;
    CHECK_THROWS(batchnorm_channel_sums(bx, bds, bq));
}

// The dispatch registry: register, call, unregister (test/unit_test/core/unit_test_dispatch.cpp).
// Needs no device: keys are made from element types.
static void test_registry()
{
    const ShapeTuple shape{8, 4, 3, 2};
    Tensor<float> x(Device::CPU, shape, channel_types(4));
    static int calls = 0;
    struct Probe
    {
        static void fn(const BaseTensor&, int v) { calls += v; }
    };
    const auto key = get_dispatch_key(x);
    CHECK(key == get_dispatch_key(get_h2_type<float>()));
    CHECK(key != get_dispatch_key(get_h2_type<double>()));
    dispatch_register("probe_gpu", key, &Probe::fn);
    CHECK(internal::has_dispatch_entry("probe_gpu", key));
    const BaseTensor& cbx = x;
    int five = 5;
    internal::call_dispatch_entry("probe_gpu", key, cbx, five);
    CHECK(calls == 5);
    dispatch_unregister("probe_gpu", key);
    CHECK(!internal::has_dispatch_entry("probe_gpu", key));
    CHECK_THROWS(internal::call_dispatch_entry("probe_gpu", key, cbx, five));
}

// The host arms of the operators against plain arithmetic, the operators without a host arm
// raising for a host tensor, and the OpenMP oracle at work: everything this program does that
// needs no GPU.  With --host-only the program runs only this and returns from main, so that the
// exit handlers of a process that has libh2x.so (and with it the HIP runtime) and the OpenMP
// runtime loaded are exercised where there is no GPU as well.
static void test_host_arms()
{
    const ComputeStream cs(Device::CPU);
    const ShapeTuple shape{7, 5, 3, 2};
    const StrideTuple halo_strides{1, 9, 9 * 8, 9 * 8 * 3}; // a 7 x 5 interior inside 9 x 8 rows
    const size_t span = 9 * 8 * 3 * 2;
    const DTTuple types = channel_types(4);
    const size_t n = product<size_t>(shape);
    std::vector<double> vals(n);
    for (size_t i = 0; i < n; ++i)
        vals[i] = 0.25 * (double) i - 3.0;
    const std::vector<double> image = scatter_strided(shape, halo_strides, span, vals, -99.0);
    std::vector<double> host_a = image, host_b(n, 0.0);
    Tensor<double> ca(Device::CPU, host_a.data(), shape, types, halo_strides, cs);
    Tensor<double> cb(Device::CPU, host_b.data(), shape, types, get_contiguous_strides(shape), cs);
    scale(ca, 2.0);
    for (size_t i = 0; i < span; ++i)
        CHECK(host_a[i] == (image[i] == -99.0 ? -99.0 : 2.0 * image[i])); // the gaps are not touched
    copy_values(ca, cb);
    for (size_t i = 0; i < n; ++i)
        CHECK(host_b[i] == 2.0 * vals[i]);
    BaseTensor &bca = ca, &bcb = cb;
    scale_bias(bca, bcb, 0.5, 1.0); // type-erased front
    for (size_t i = 0; i < n; ++i)
        CHECK(host_b[i] == vals[i] + 1.0);
    const ShapeTuple rshape{1, 1, 3, 1};
    std::vector<double> host_r(3, 10.0);
    Tensor<double> cr(Device::CPU, host_r.data(), rshape, types, get_contiguous_strides(rshape), cs);
    reduce_sum(ca, cr, true);
    for (int c = 0; c < 3; ++c)
    {
        double want = 10.0;
        for (int s = 0; s < 2; ++s)
            for (int i = 0; i < 35; ++i)
            {
                const double x = 2.0 * vals[(s * 3 + c) * 35 + i];
                want += x * x;
            }
        CHECK(std::fabs(host_r[c] - want) <= 1e-12 * want);
    }
    // halo operators on contiguous tensors whose shape includes the halo
    const ShapeTuple hshape{10, 6, 3, 2};
    const size_t ht = product<size_t>(hshape);
    std::vector<double> c1(ht), c2(ht), cbuf(ht, 0.0);
    for (size_t i = 0; i < ht; ++i)
    {
        c1[i] = 1.0 + (double) i;
        c2[i] = -2.0 * (double) i;
    }
    const std::vector<double> h1 = c1, h2v = c2;
    Tensor<double> t1(Device::CPU, c1.data(), hshape, types, get_contiguous_strides(hshape), cs);
    Tensor<double> t2(Device::CPU, c2.data(), hshape, types, get_contiguous_strides(hshape), cs);
    Tensor<double> tbuf(Device::CPU, cbuf.data(), ShapeTuple{(DimType) ht}, DTTuple{DT::Any}, StrideTuple{1}, cs);
    clear_halo(t2, 1, 1);
    for (size_t i = 0; i < ht; ++i)
    {
        const size_t h = (i / 10) % 6;
        CHECK(c2[i] == ((h == 0 || h == 5) ? 0.0 : h2v[i]));
    }
    // the RHS boundary column of t1 (w = 8) lands in the LHS halo column of t2 (w = 0)
    halo_pack(t1, 0, H2X_RHS, 1, tbuf);
    halo_unpack(t2, 0, H2X_LHS, 1, tbuf);
    for (size_t row = 0; row < ht / 10; ++row)
        CHECK(c2[row * 10] == h1[row * 10 + 8]);
    // a transfer is that pack and unpack in one
    std::vector<double> c3 = h2v;
    Tensor<double> t3(Device::CPU, c3.data(), hshape, types, get_contiguous_strides(hshape), cs);
    halo_transfer(t1, t3, 0, H2X_RHS, 1);
    for (size_t row = 0; row < ht / 10; ++row)
        for (int w = 0; w < 10; ++w)
            CHECK(c3[row * 10 + w] == (w == 0 ? h1[row * 10 + 8] : h2v[row * 10 + w]));
    Tensor<double> bad(Device::CPU, ShapeTuple{1, 2, 3, 1}, types, cs);
    CHECK_THROWS(reduce_sum(ca, bad)); // extent 2 is neither 1 nor 5

    // operators without a host arm raise for a host tensor
    const ShapeTuple fshape{8, 4, 3, 2};
    Tensor<float> cx(Device::CPU, fshape, channel_types(4)), cy(Device::CPU, fshape, channel_types(4)),
        csum(Device::CPU, ShapeTuple{3}, DTTuple{DT::Channel}), cq(Device::CPU, ShapeTuple{3}, DTTuple{DT::Channel});
    CHECK_THROWS(batchnorm_channel_sums(cx, csum, cq));
    CHECK_THROWS(softmax_channel_forward(cx, cy));
    CHECK_THROWS(softmax_instance_forward(cx, cy));

    // the oracle on a tensor large enough for its OpenMP team to start: mean 0.3, variance 1
    const int N = 8, C = 16;
    const size_t S = 32 * 32;
    const std::vector<float> hx = randn((size_t) N * C * S, 11, 1.0f, 0.3f);
    std::vector<float> sums(C), sqsums(C), rm(C, 0.0f), rv(C, 1.0f);
    orc_bn_channel_sums_and_sqsums_f32(N, C, S, S, hx.data(), sums.data(), sqsums.data());
    orc_bn_sums_to_statistics_f32(C, (size_t) N * S, 0.9f, sums.data(), sqsums.data(), rm.data(), rv.data());
    for (int c = 0; c < C; ++c)
        CHECK(std::fabs(sums[c] - 0.3f) < 0.05f && std::fabs(sqsums[c] - 1.0f) < 0.05f);
}

// Every operator of tensor_ops_mi355x.hpp on a GPU tensor and on a CPU tensor with the
// same contents: the two arms must leave the same bits (sums: the same value to 1e-12,
// both add in float64), and both must match plain host arithmetic.
static void test_both_arms()
{
    const ComputeStream gs(Device::GPU), cs(Device::CPU);
    const ShapeTuple shape{7, 5, 3, 2};
    const StrideTuple halo_strides{1, 9, 9 * 8, 9 * 8 * 3}; // a 7 x 5 interior inside 9 x 8 rows
    const size_t span = 9 * 8 * 3 * 2;
    const DTTuple types = channel_types(4);
    const size_t n = product<size_t>(shape);
    std::vector<double> vals(n);
    for (size_t i = 0; i < n; ++i)
        vals[i] = 0.25 * (double) i - 3.0;
    const std::vector<double> image = scatter_strided(shape, halo_strides, span, vals, -99.0);
    double *dev_a = nullptr, *dev_b = nullptr;
    check_hip(hipMalloc(reinterpret_cast<void**>(&dev_a), span * 8), "hipMalloc");
    check_hip(hipMalloc(reinterpret_cast<void**>(&dev_b), n * 8), "hipMalloc");
    std::vector<double> host_a = image, host_b(n, 0.0);
    check_hip(hipMemcpy(dev_a, image.data(), span * 8, hipMemcpyHostToDevice), "upload");
    Tensor<double> ga(Device::GPU, dev_a, shape, types, halo_strides, gs);
    Tensor<double> gb(Device::GPU, dev_b, shape, types, get_contiguous_strides(shape), gs);
    Tensor<double> ca(Device::CPU, host_a.data(), shape, types, halo_strides, cs);
    Tensor<double> cb(Device::CPU, host_b.data(), shape, types, get_contiguous_strides(shape), cs);
    auto same = [&](const char* what) {
        std::vector<double> a(span), b(n);
        check_hip(hipDeviceSynchronize(), "sync");
        check_hip(hipMemcpy(a.data(), dev_a, span * 8, hipMemcpyDeviceToHost), "download");
        check_hip(hipMemcpy(b.data(), dev_b, n * 8, hipMemcpyDeviceToHost), "download");
        if (std::memcmp(a.data(), host_a.data(), span * 8) != 0 || std::memcmp(b.data(), host_b.data(), n * 8) != 0)
        {
            std::printf("FAILED: GPU and CPU arms differ after %s\n", what);
            std::exit(1);
        }
    };
    scale(ga, 2.0);
    scale(ca, 2.0);
    same("scale");
    for (size_t i = 0; i < span; ++i)
        CHECK(host_a[i] == (image[i] == -99.0 ? -99.0 : 2.0 * image[i])); // the gaps are not touched
    copy_values(ga, gb);
    copy_values(ca, cb);
    same("copy_values");
    for (size_t i = 0; i < n; ++i)
        CHECK(host_b[i] == 2.0 * vals[i]);
    scale_bias(ga, gb, 0.5, 1.0);
    scale_bias(ca, cb, 0.5, 1.0);
    same("scale_bias");
    for (size_t i = 0; i < n; ++i)
        CHECK(host_b[i] == vals[i] + 1.0);
    // sums over space and samples into a per-channel tensor, through the type-erased front too
    const ShapeTuple rshape{1, 1, 3, 1};
    Tensor<double> gr(Device::GPU, rshape, types, gs);
    std::vector<double> host_r(3, 10.0);
    upload(gr, host_r);
    Tensor<double> cr(Device::CPU, host_r.data(), rshape, types, get_contiguous_strides(rshape), cs);
    const BaseTensor& bga = ga;
    BaseTensor& bgr = gr;
    reduce_sum(bga, bgr, true);
    reduce_sum(ca, cr, true);
    const std::vector<double> got_r = download(gr);
    for (int c = 0; c < 3; ++c)
    {
        double want = 10.0;
        for (int s = 0; s < 2; ++s)
            for (int i = 0; i < 35; ++i)
            {
                const double x = 2.0 * vals[(s * 3 + c) * 35 + i];
                want += x * x;
            }
        CHECK(std::fabs(got_r[c] - want) <= 1e-12 * want && std::fabs(host_r[c] - want) <= 1e-12 * want);
    }
    // clear_halo, halo pack / unpack and halo_transfer on contiguous tensors whose shape includes the halo
    const ShapeTuple hshape{10, 6, 3, 2};
    const size_t ht = product<size_t>(hshape);
    std::vector<double> h1(ht), h2v(ht);
    for (size_t i = 0; i < ht; ++i)
    {
        h1[i] = 1.0 + (double) i;
        h2v[i] = -2.0 * (double) i;
    }
    std::vector<double> c1 = h1, c2 = h2v, cbuf(ht, 0.0); // room for the largest strip
    Tensor<double> g1(Device::GPU, hshape, types, gs), g2(Device::GPU, hshape, types, gs);
    Tensor<double> gbuf(Device::GPU, ShapeTuple{(DimType) ht}, DTTuple{DT::Any}, gs);
    upload(g1, h1);
    upload(g2, h2v);
    upload(gbuf, cbuf);
    Tensor<double> t1(Device::CPU, c1.data(), hshape, types, get_contiguous_strides(hshape), cs);
    Tensor<double> t2(Device::CPU, c2.data(), hshape, types, get_contiguous_strides(hshape), cs);
    Tensor<double> tbuf(Device::CPU, cbuf.data(), ShapeTuple{(DimType) ht}, DTTuple{DT::Any}, StrideTuple{1}, cs);
    auto same_halo = [&](const char* what) {
        const std::vector<double> a = download(g1), b = download(g2), c = download(gbuf);
        if (a != c1 || b != c2 || c != cbuf)
        {
            std::printf("FAILED: GPU and CPU arms differ after %s\n", what);
            std::exit(1);
        }
    };
    clear_halo(g2, 1, 1);
    clear_halo(t2, 1, 1);
    same_halo("clear_halo");
    for (size_t i = 0; i < ht; ++i)
    {
        const size_t h = (i / 10) % 6;
        CHECK(c2[i] == ((h == 0 || h == 5) ? 0.0 : h2v[i]));
    }
    for (int width : {1, 2})
        for (int dim : {0, 1, 2})
        {
            if (2 * width > hshape[dim])
                continue;
            halo_pack(g1, dim, H2X_RHS, width, gbuf);
            halo_pack(t1, dim, H2X_RHS, width, tbuf);
            halo_unpack(g2, dim, H2X_LHS, width, gbuf);
            halo_unpack(t2, dim, H2X_LHS, width, tbuf);
            same_halo("halo pack + unpack");
            halo_pack(g1, dim, H2X_LHS, width, gbuf, true);
            halo_pack(t1, dim, H2X_LHS, width, tbuf, true);
            halo_unpack(g2, dim, H2X_RHS, width, gbuf, true, H2X_HALO_SUM);
            halo_unpack(t2, dim, H2X_RHS, width, tbuf, true, H2X_HALO_SUM);
            same_halo("reverse halo pack + SUM unpack");
            halo_transfer(g1, g2, dim, H2X_RHS, width);
            halo_transfer(t1, t2, dim, H2X_RHS, width);
            same_halo("halo_transfer");
            halo_transfer(g2, g1, dim, H2X_LHS, width, true, H2X_HALO_MAX);
            halo_transfer(t2, t1, dim, H2X_LHS, width, true, H2X_HALO_MAX);
            same_halo("reverse halo_transfer with MAX");
        }
    // a transfer equals pack on the source + unpack on the destination
    {
        std::vector<double> ref = c2;
        Tensor<double> tr(Device::CPU, ref.data(), hshape, types, get_contiguous_strides(hshape), cs);
        halo_pack(t1, 0, H2X_LHS, 1, tbuf);
        halo_unpack(tr, 0, H2X_RHS, 1, tbuf);
        halo_transfer(t1, t2, 0, H2X_LHS, 1);
        CHECK(ref == c2);
    }
    CHECK_THROWS(halo_transfer(g1, t2, 0, H2X_LHS, 1));   // tensors on different devices
    Tensor<double> bad(Device::CPU, ShapeTuple{1, 2, 3, 1}, types, cs);
    CHECK_THROWS(reduce_sum(ca, bad));                    // extent 2 is neither 1 nor 5
    check_hip(hipFree(dev_a), "hipFree");
    check_hip(hipFree(dev_b), "hipFree");
}

// shuffle pack / unpack of one rank through a ShufflePlan: a 8 x 6 x 2 x 2 local tensor cut
// for a 2 x 2 peer grid; the buffer holds the four boxes one after the other, each in its
// own natural order (legacy/src/tensor/shuffle_mpi_cuda.cu:42-98).
static void test_shuffle()
{
    const ComputeStream gs(Device::GPU);
    const ShapeTuple shape{8, 6, 2, 2};
    const size_t n = product<size_t>(shape);
    const std::vector<int32_t> limits{4, 8, 3, 6, 2, 2};
    const std::vector<int32_t> displs{0, 48, 96, 144};
    ShufflePlan plan(shape, get_contiguous_strides(shape), ShapeTuple{2, 2, 1, 1}, limits, displs, 4);
    std::vector<float> h(n);
    for (size_t i = 0; i < n; ++i)
        h[i] = (float) i;
    Tensor<float> t(Device::GPU, shape, channel_types(4), gs), back(Device::GPU, shape, channel_types(4), gs);
    Tensor<float> buf(Device::GPU, ShapeTuple{(DimType) n}, DTTuple{DT::Any}, gs);
    upload(t, h);
    upload(back, std::vector<float>(n, -1.0f));
    shuffle_pack(plan, t, buf);
    const std::vector<float> packed = download(buf);
    size_t o = 0;
    for (int ph = 0; ph < 2; ++ph)          // peers in rank order: dimension 0 of the grid fastest
        for (int pw = 0; pw < 2; ++pw)
        {
            o = displs[ph * 2 + pw];
            for (int s = 0; s < 2; ++s)
                for (int c = 0; c < 2; ++c)
                    for (int y = 0; y < 3; ++y)
                        for (int x = 0; x < 4; ++x)
                            CHECK(packed[o++] == h[((s * 2 + c) * 6 + ph * 3 + y) * 8 + pw * 4 + x]);
        }
    BaseTensor &bt = back, &bb = buf;
    shuffle_unpack(plan, bt, bb);           // type-erased front
    CHECK(download(back) == h);
    Tensor<float> cpu(Device::CPU, shape, channel_types(4)), cbuf(Device::CPU, ShapeTuple{(DimType) n}, DTTuple{DT::Any});
    CHECK_THROWS(shuffle_pack(plan, cpu, cbuf));   // no CPU implementation
}

static void test_softmax_instance()
{
    const ShapeTuple shape{9, 7, 5, 3};
    const size_t total = product<size_t>(shape), size = total / 3;
    const ComputeStream stream(Device::GPU);
    Tensor<float> x(Device::GPU, shape, channel_types(4), stream), y(Device::GPU, shape, channel_types(4), stream),
        dy(Device::GPU, shape, channel_types(4), stream), dx(Device::GPU, shape, channel_types(4), stream);
    const std::vector<float> hx = randn(total, 5, 2.0f), hdy = randn(total, 6);
    upload(x, hx);
    upload(dy, hdy);
    softmax_instance_forward(x, y);
    const BaseTensor &by = y, &bdy = dy;
    BaseTensor& bdx = dx;
    softmax_instance_backward(by, bdy, bdx);
    std::vector<float> wy(total), wdx(total), smax(3), sexp(3), sdp(3);
    orc_softmax_instance_max_f32(3, size, hx.data(), smax.data());
    orc_softmax_instance_exp_f32(3, size, hx.data(), smax.data(), wy.data(), sexp.data());
    orc_softmax_instance_normalize_f32(3, size, sexp.data(), wy.data());
    const std::vector<float> gy = download(y);
    orc_softmax_instance_dot_f32(3, size, gy.data(), hdy.data(), sdp.data());
    orc_softmax_instance_gradient_f32(3, size, gy.data(), hdy.data(), sdp.data(), wdx.data());
    CHECK(max_rel(gy, wy) <= 1e-5);
    // dx = y * (dy - dp) cancels: compare against the scale of its terms
    const std::vector<float> gdx = download(dx);
    for (size_t i = 0; i < total; ++i)
        CHECK(std::fabs(gdx[i] - wdx[i]) <= 1e-5 * (std::fabs(gy[i] * hdy[i]) + std::fabs(gy[i])));
}

int main(int argc, char** argv)
{
    std::setvbuf(stdout, nullptr, _IONBF, 0); // what was printed survives a crash
#define RUN(call)                                                                                  \
    do                                                                                             \
    {                                                                                              \
        std::printf("%s\n", #call);                                                                \
        call;                                                                                      \
    } while (0)
    RUN(test_host_arms());
    RUN(test_registry());
    if (argc > 1 && std::strcmp(argv[1], "--host-only") == 0)
    {
        std::printf("test_h2_frontend: host-only ok\n");
        return 0;
    }
    RUN(test_both_arms());
    RUN(test_shuffle());
    RUN(test_softmax_instance());
    RUN(test_batchnorm(ShapeTuple{14, 14, 8, 4}));
    RUN(test_batchnorm(ShapeTuple{6, 5, 7, 3, 2}));
    RUN(test_batchnorm(ShapeTuple{33, 5, 2})); // one spatial dimension, odd length
    RUN(test_strided_view());
    RUN(test_softmax());
    RUN(test_halo());
    RUN(test_errors());
#undef RUN
    release_workspaces();
    check_hip(hipDeviceSynchronize(), "sync");
    std::printf("test_h2_frontend: ok\n");
    // The GPU run of this one program leaves without exit handlers.  It ended with SIGSEGV after
    // the line above, i.e. inside the exit handlers, in 2 of about 50 runs on the GPU, and the
    // cause is not established.  Ruled out: every object of this program that owns device memory,
    // a plan or a stream has function scope and is gone by now; the headers free nothing from
    // static destructors; the same exit path with the HIP runtime loaded but not initialised and
    // the OpenMP team of the oracle alive (--host-only, which returns from main) is clean under
    // ASan, UBSan and TSan and in hundreds of plain runs.  What is left needs an initialised
    // runtime: its own teardown beside its helper threads.  The other test programs return from
    // main and so exercise that path.
    std::fflush(nullptr);
    _exit(0);
}

// Exercises the C++ `small::` API of the MI355X build the way the reference's own unit tests
// exercise theirs (test/test_relu.cpp:53-135, test_leaky.cpp:53-133, test_shortcut.cpp:29-60,
// test_upsample2d.cpp:43-62, test_route_concat.cpp, test_conv2d.cpp:1284-1379, test_maxpool.cpp,
// test_buffer.cpp): closed-form checks plus the reference's regression fixtures, packed with
// pack_buffer for this platform's blocking and compared in packed space.
//
// usage: test_small_api <dir with the regression .bin fixtures>
#include <small.h>

#include <cmath>
#include <cstdio>
#include <fstream>
#include <memory>
#include <string>
#include <vector>

using small::FloatBuffer;
using small::QUInt8Buffer;

static int g_fail = 0;
#define CHECK(cond)                                                                    \
    do                                                                                 \
    {                                                                                  \
        if (!(cond))                                                                   \
        {                                                                              \
            std::printf("  CHECK FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);      \
            ++g_fail;                                                                  \
        }                                                                              \
    } while (0)

static bool almost_equal(float a, float b, float rtol = 5e-3f, float atol = 1e-5f)
{
    return std::fabs(a - b) <= atol + rtol * std::fabs(b);
}

// 4-byte big-endian count, then little-endian float32
static FloatBuffer read_bin(std::string const &path)
{
    std::ifstream f(path, std::ios::binary);
    if (!f) { std::printf("  cannot open %s\n", path.c_str()); ++g_fail; return FloatBuffer(); }
    unsigned char h[4];
    f.read(reinterpret_cast<char *>(h), 4);
    const size_t n = (size_t(h[0]) << 24) | (size_t(h[1]) << 16) | (size_t(h[2]) << 8) | size_t(h[3]);
    FloatBuffer buf(n);
    f.read(reinterpret_cast<char *>(buf.data()), n * sizeof(float));
    return buf;
}

static void test_buffer_semantics()
{
    std::printf("buffer semantics\n");
    FloatBuffer a(64);
    for (size_t i = 0; i < 64; ++i) a[i] = float(i) - 20.f;
    FloatBuffer b(a);                 // deep copy
    b[3] = 99.f;
    CHECK(a[3] == -17.f && b[3] == 99.f && b[4] == a[4]);
    FloatBuffer c(std::move(b));
    CHECK(c.size() == 64 && b.size() == 0 && c[3] == 99.f);
    a.swap(c);
    CHECK(a[3] == 99.f && c[3] == -17.f);
    FloatBuffer d;
    d = c;
    CHECK(d.size() == 64 && d[0] == -20.f);
    // a copy taken while the newest data is on the device
    small::ReLUActivation(16, 2, 2, c, c);
    FloatBuffer e(c);
    CHECK(e[0] == 0.f && e[63] == 43.f);
    CHECK(FloatBuffer::C_ob == 16 && FloatBuffer::C_ib == 16 && QUInt8Buffer::C_ob == 16);
    QUInt8Buffer q(16);
    CHECK(q.zero() == 128 && q.multiplier == 1077952576 && q.lshift == 0 && q.rshift == 6);
    CHECK(q.min_val == 0 && q.max_val == 255 && q.b == 8 && q.offset == 0);
    q.m_zero = -3;
    QUInt8Buffer q2(q);
    CHECK(q2.zero() == -3);
    std::unique_ptr<FloatBuffer, void (*)(FloatBuffer *)> p(small::alloc_buffer<FloatBuffer>(8),
                                                            small::free_buffer<FloatBuffer>);
    CHECK(p->size() == 8);
}

static void test_shapes_and_packing()
{
    std::printf("shapes and packing\n");
    uint8_t f, b;
    small::calc_padding(56, 3, 1, f, b); CHECK(f == 1 && b == 1);
    small::calc_padding(224, 3, 2, f, b); CHECK(f == 0 && b == 1);
    small::calc_padding(13, 2, 1, f, b); CHECK(f == 0 && b == 1);
    small::calc_padding(49, 10, 2, f, b); CHECK(f == 4 && b == 5);
    small::calc_padding(10, 4, 2, f, b); CHECK(f == 1 && b == 1);
    CHECK(small::output_dim(56, 2, 3) == 27 && small::output_dim(2, 1, 3) == 0);
    CHECK(small::compute_output_dim(224, 3, 2, small::PADDING_F) == 112);
    size_t od;
    small::compute_padding_output_dim(416, 3, 1, small::PADDING_F, f, b, od);
    CHECK(f == 1 && b == 1 && od == 416);
    // index maps against the layout formulas
    CHECK(small::packed_buffer_index(32, 5, 7, 16, 17, 2, 3) == 1 * 5 * 7 * 16 + (2 * 7 + 3) * 16 + 1);
    CHECK(small::packed_buffer_index(3, 4, 4, 16, 2, 1, 1) == (1 * 4 + 1) * 3 + 2);
    CHECK(small::packed_weight_index(32, 32, 3, 3, 16, 16, 17, 18, 1, 2) ==
          1 * (2 * 9 * 256) + 1 * (9 * 256) + (1 * 3 + 2) * 256 + 2 * 16 + 1);
    bool threw = false;
    try { small::packed_buffer_index(5, 2, 2, 16, 0, 0, 0); } catch (std::runtime_error const &) { threw = true; }
    CHECK(threw);
    // pack / unpack round trip
    FloatBuffer flat(32 * 3 * 5), packed(32 * 3 * 5), back(32 * 3 * 5);
    for (size_t i = 0; i < flat.size(); ++i) flat[i] = float(i);
    CHECK(small::pack_buffer(flat, small::INPUT, 1, 32, 3, 5, 16, 16, packed) == 480);
    CHECK(packed[small::packed_buffer_index(32, 3, 5, 16, 20, 1, 4)] == flat[(20 * 3 + 1) * 5 + 4]);
    small::unpack_buffer(packed, small::INPUT, 1, 32, 3, 5, 16, 16, back);
    CHECK(small::equals(480, flat, back));
    // the device pack agrees with the host index walk for every tensor type
    struct { small::BufferTypeEnum t; uint32_t d0, d1, d2, d3; } shapes[] = {
        {small::INPUT, 1, 3, 8, 6}, {small::OUTPUT, 1, 48, 4, 5}, {small::FILTER_DW, 32, 1, 3, 3},
        {small::FILTER_CONV, 32, 48, 3, 3}, {small::FILTER_CONV, 16, 3, 3, 3}, {small::FILTER_FC, 32, 64, 1, 1}};
    for (auto const &sh : shapes)
    {
        const size_t n = (size_t)sh.d0 * sh.d1 * sh.d2 * sh.d3;
        FloatBuffer fl(n), dev(n), host(n);
        for (size_t i = 0; i < n; ++i) fl[i] = float(i) * 0.5f - 7.f;
        CHECK(small::pack_buffer(fl, sh.t, sh.d0, sh.d1, sh.d2, sh.d3, 16, 16, dev) == n);
        CHECK(small::convert_tensor2dc<float>(fl.data(), sh.t, sh.d0, sh.d1, sh.d2, sh.d3, 16, 16, host.data()) == n);
        CHECK(small::equals(n, dev, host, 0.f));
    }
    QUInt8Buffer qf(3 * 16 * 16), qp(3 * 16 * 16), qh(3 * 16 * 16);
    for (size_t i = 0; i < qf.size(); ++i) qf[i] = uint8_t(i * 7);
    CHECK(small::pack_buffer(qf, small::INPUT, 1, 3, 16, 16, 16, 16, qp) == 768);
    small::convert_tensor2dc<uint8_t>(qf.data(), small::INPUT, 1, 3, 16, 16, 16, 16, qh.data());
    CHECK(small::equals(768, qp, qh));
    threw = false;
    try { small::pack_buffer(flat, small::INPUT, 1, 20, 3, 8, 16, 16, packed); } catch (std::invalid_argument const &) { threw = true; }
    CHECK(threw);
}

static void test_relu_leaky_accum_upsample_concat()
{
    std::printf("relu / leaky / accum / upsample / concat (closed forms)\n");
    const int C = 32, H = 5, W = 7, n = C * H * W;
    FloatBuffer in(n), out(n);
    small::init(in, n);
    small::ReLUActivation(C, H, W, in, out);
    for (int i = 0; i < n; ++i) CHECK(out[i] == (in[i] >= 0 ? in[i] : 0.f));
    FloatBuffer slope(1);
    slope[0] = 0.1f;
    small::LeakyReLUActivation(C, H, W, in, slope, out);
    for (int i = 0; i < n; ++i) CHECK(out[i] == (in[i] > 0 ? in[i] : in[i] * 0.1f));
    // in place
    FloatBuffer io(in);
    small::ReLUActivation(C, H, W, io, io);
    for (int i = 0; i < n; ++i) CHECK(io[i] == (in[i] >= 0 ? in[i] : 0.f));
    // accum: out == in + old out, exactly
    FloatBuffer acc(n);
    small::init(acc, n);
    FloatBuffer old(acc);
    small::Accum(C, H, W, in, acc);
    for (int i = 0; i < n; ++i) CHECK(acc[i] == in[i] + old[i]);
    // upsample: out[k,i,j] == in[k,i/2,j/2]
    FloatBuffer up(4 * n);
    small::UpSample2D(2, C, H, W, in, up);
    for (int k = 0; k < C; ++k)
        for (int i = 0; i < 2 * H; ++i)
            for (int j = 0; j < 2 * W; ++j)
                CHECK(up[small::packed_buffer_index(C, 2 * H, 2 * W, 16, k, i, j)] ==
                      in[small::packed_buffer_index(C, H, W, 16, k, i / 2, j / 2)]);
    FloatBuffer same(1);
    small::UpSample2D(1, C, H, W, in, same);
    CHECK(same.size() == (size_t)n && small::equals(n, in, same));
    // concat along channels
    FloatBuffer cat(3 * n), two(2 * n);
    small::init(two, 2 * n);
    small::Concat(C, 2 * C, H, W, in, two, cat);
    for (int i = 0; i < n; ++i) CHECK(cat[i] == in[i]);
    for (int i = 0; i < 2 * n; ++i) CHECK(cat[n + i] == two[i]);
    // bias
    FloatBuffer bias(C), bo(n);
    small::init(bias, C);
    small::Bias(C, H, W, bias, bo);
    for (int k = 0; k < C; ++k) CHECK(bo[small::packed_buffer_index(C, H, W, 16, k, 2, 3)] == bias[k]);
}

static void test_exceptions()
{
    std::printf("error behaviour\n");
    FloatBuffer a(16 * 8 * 8), f(16 * 16 * 9), o(16 * 8 * 8);
    auto expect = [&](auto &&fn, char const *msg) {
        try { fn(); std::printf("  no exception, wanted: %s\n", msg); ++g_fail; }
        catch (std::invalid_argument const &e)
        {
            if (std::string(e.what()) != msg) { std::printf("  got '%s' wanted '%s'\n", e.what(), msg); ++g_fail; }
        }
    };
    expect([&] { small::Conv2D(3, 3, 3, 0, 0, 0, 0, 16, 16, 8, 8, a, f, o); }, "Conv2D<float> ERROR: stride unsupported.");
    expect([&] { small::Conv2D(3, 3, 1, 0, 0, 0, 0, 16, 5, 8, 8, a, f, o); }, "Conv2D<float> ERROR: in_channels unsupported.");
    expect([&] { small::PartialConv2D(3, 3, 4, 0, 0, 0, 0, 16, 16, 8, 8, a, f, o); }, "PartialConv2D<float> ERROR: stride unsupported.");
    expect([&] { small::MaxPool2D(3, 3, 3, 0, 0, 0, 0, 16, 8, 8, a, o); }, "MaxPool2D<float> ERROR: stride unsupported.");
    expect([&] { small::AveragePool2D(3, 3, 4, 0, 0, 0, 0, 16, 8, 8, a, o); }, "AveragePool2D<float> ERROR: stride unsupported.");
    expect([&] { small::DepthwiseConv2D(3, 3, 1, 0, 0, 0, 0, 24, 8, 8, a, f, o); }, "DepthwiseConv2D<float> ERROR: in_channels unsupported.");
    expect([&] { small::ReLUActivation(5, 4, 4, a, o); }, "ReLUActivation<float> ERROR: in_channels unsupported.");
    expect([&] { small::UpSample2D(3, 16, 4, 4, a, o); }, "Upsample<float> ERROR: scale factor unsupported (only 1 or 2).");
    expect([&] { small::GroupConv2D(3, 3, 3, 1, 0, 0, 0, 0, 16, 6, 6, a, f, o); }, "GroupConv2D<float> ERROR: stride unsupported.");
    expect([&] { small::GroupConv2D(3, 3, 1, 2, 0, 0, 0, 0, 8, 6, 6, a, f, o); }, "GroupConv2D<float> ERROR: in_channels unsupported.");
    expect([&] { small::PartialGroupConv2D(3, 3, 3, 1, 0, 0, 0, 0, 16, 6, 6, a, f, o); }, "PartialGroupConv2D<float> ERROR: stride unsupported.");
    QUInt8Buffer qa(16 * 64), qf(16 * 16 * 9), qo(16 * 64);
    expect([&] { small::GroupConv2D(3, 3, 3, 1, 0, 0, 0, 0, 16, 6, 6, qa, qf, qo); }, "GroupConv2D<quint8> ERROR: stride unsupported.");
    expect([&] { small::Conv2D(3, 3, 3, 0, 0, 0, 0, 16, 16, 8, 8, qa, qf, qo); }, "Conv2D<quint8> ERROR: stride unsupported.");
    expect([&] { small::ReLUActivation(5, 4, 4, qa, qo); }, "ReLUActivation<quint8> ERROR: in_channels unsupported.");
}

struct Params { uint32_t Ci, H, W, k, s; char p; uint32_t Co; };

static std::string fname(std::string const &dir, char const *kind, char const *layer, Params const &q,
                         size_t numel, bool with_co)
{
    char buf[256];
    if (with_co)
        std::snprintf(buf, sizeof(buf), "%s/%s__%s_Ci%u_H%u_W%u_k%u_s%u_%c_Co%u_%zu.bin", dir.c_str(), kind, layer,
                      q.Ci, q.H, q.W, q.k, q.s, q.p, q.Co, numel);
    else
        std::snprintf(buf, sizeof(buf), "%s/%s__%s_Ci%u_H%u_W%u_k%u_s%u_%c_%zu.bin", dir.c_str(), kind, layer, q.Ci,
                      q.H, q.W, q.k, q.s, q.p, numel);
    return buf;
}

static void pads_of(Params const &q, uint8_t &t, uint8_t &b, uint8_t &l, uint8_t &r)
{
    t = b = l = r = 0;
    if (q.p == 'f')
    {
        small::calc_padding(q.H, q.k, q.s, t, b);
        small::calc_padding(q.W, q.k, q.s, l, r);
    }
}

static void test_conv2d_fixtures(std::string const &dir)
{
    std::printf("Conv2D regression fixtures\n");
    const Params cases[] = {{3, 3, 3, 1, 1, 'v', 16},   {3, 3, 3, 3, 1, 'v', 16},   {3, 1, 1, 1, 1, 'f', 16},
                            {16, 1, 6, 1, 1, 'v', 16},  {16, 3, 8, 3, 1, 'v', 16},  {16, 30, 30, 3, 1, 'v', 16},
                            {16, 1, 6, 1, 1, 'v', 96},  {96, 3, 8, 3, 1, 'v', 16},  {16, 3, 3, 3, 1, 'f', 16},
                            {16, 3, 3, 3, 2, 'f', 16},  {16, 3, 8, 3, 1, 'f', 96},  {16, 3, 13, 3, 2, 'f', 96},
                            {96, 3, 13, 3, 2, 'f', 16}, {96, 30, 30, 3, 2, 'f', 96}};
    for (Params const &q : cases)
    {
        uint8_t t, b, l, r;
        pads_of(q, t, b, l, r);
        const size_t Ho = small::compute_output_dim(q.H, q.k, q.s, q.p == 'f' ? small::PADDING_F : small::PADDING_V);
        const size_t Wo = small::compute_output_dim(q.W, q.k, q.s, q.p == 'f' ? small::PADDING_F : small::PADDING_V);
        FloatBuffer in = read_bin(fname(dir, "in", "conv2d", q, q.Ci * q.H * q.W, true));
        FloatBuffer fl = read_bin(fname(dir, "filter", "conv2d", q, q.Ci * q.k * q.k * q.Co, true));
        FloatBuffer ex = read_bin(fname(dir, "out", "conv2d", q, q.Co * Ho * Wo, true));
        if (!in.size() || !fl.size() || !ex.size()) continue;
        FloatBuffer pin(in.size()), pfl(fl.size()), pex(ex.size()), out(ex.size());
        small::pack_buffer(in, small::INPUT, 1, q.Ci, q.H, q.W, FloatBuffer::C_ib, FloatBuffer::C_ob, pin);
        small::pack_buffer(fl, small::FILTER_CONV, q.Co, q.Ci, q.k, q.k, FloatBuffer::C_ib, FloatBuffer::C_ob, pfl);
        small::pack_buffer(ex, small::OUTPUT, 1, q.Co, Ho, Wo, FloatBuffer::C_ib, FloatBuffer::C_ob, pex);
        small::Conv2D(q.k, q.k, q.s, t, b, l, r, q.Co, q.Ci, q.H, q.W, pin, pfl, out);
        size_t bad = 0;
        for (size_t i = 0; i < pex.size(); ++i) bad += !almost_equal(out[i], pex[i]);
        if (bad) std::printf("  Ci%u H%u W%u k%u s%u %c Co%u: %zu mismatches\n", q.Ci, q.H, q.W, q.k, q.s, q.p, q.Co, bad);
        CHECK(bad == 0);
        // PartialConv2D on top of itself doubles the result
        small::PartialConv2D(q.k, q.k, q.s, t, b, l, r, q.Co, q.Ci, q.H, q.W, pin, pfl, out);
        bad = 0;
        for (size_t i = 0; i < pex.size(); ++i) bad += !almost_equal(out[i], 2.f * pex[i]);
        CHECK(bad == 0);
    }
}

static void test_window_fixtures(std::string const &dir)
{
    std::printf("DepthwiseConv2D / MaxPool2D / AveragePool2D / ReLU regression fixtures\n");
    const Params cases[] = {{16, 3, 3, 3, 2, 'v', 0}, {16, 3, 3, 3, 2, 'f', 0},  {16, 3, 13, 3, 2, 'v', 0},
                            {16, 3, 13, 3, 2, 'f', 0}, {96, 3, 13, 3, 2, 'f', 0}, {96, 30, 30, 3, 2, 'f', 0},
                            {16, 30, 30, 3, 2, 'v', 0}};
    for (Params const &q : cases)
    {
        uint8_t t, b, l, r;
        pads_of(q, t, b, l, r);
        const auto pe = q.p == 'f' ? small::PADDING_F : small::PADDING_V;
        const size_t Ho = small::compute_output_dim(q.H, q.k, q.s, pe), Wo = small::compute_output_dim(q.W, q.k, q.s, pe);
        FloatBuffer in = read_bin(fname(dir, "in", "pool", q, q.Ci * q.H * q.W, false));
        FloatBuffer exm = read_bin(fname(dir, "out", "pool", q, q.Ci * Ho * Wo, false));
        FloatBuffer exa = read_bin(fname(dir, "out", "averagepool", q, q.Ci * Ho * Wo, false));
        if (!in.size() || !exm.size() || !exa.size()) continue;
        FloatBuffer pin(in.size()), pexm(exm.size()), pexa(exa.size()), out(exm.size());
        small::pack_buffer(in, small::INPUT, 1, q.Ci, q.H, q.W, 16, 16, pin);
        small::pack_buffer(exm, small::OUTPUT, 1, q.Ci, Ho, Wo, 16, 16, pexm);
        small::pack_buffer(exa, small::OUTPUT, 1, q.Ci, Ho, Wo, 16, 16, pexa);
        small::MaxPool2D(q.k, q.k, q.s, t, b, l, r, q.Ci, q.H, q.W, pin, out);
        size_t bad = 0;
        for (size_t i = 0; i < out.size(); ++i) bad += out[i] != pexm[i];   // exact, as in test_maxpool.cpp
        CHECK(bad == 0);
        small::AveragePool2D(q.k, q.k, q.s, t, b, l, r, q.Ci, q.H, q.W, pin, out);
        bad = 0;
        for (size_t i = 0; i < out.size(); ++i) bad += !almost_equal(out[i], pexa[i]);
        CHECK(bad == 0);
    }
    const Params dw[] = {{16, 3, 3, 3, 1, 'v', 0}, {16, 3, 3, 3, 2, 'f', 0}, {16, 3, 8, 3, 1, 'f', 0},
                         {96, 3, 13, 3, 2, 'f', 0}, {96, 30, 30, 3, 2, 'f', 0}, {16, 30, 30, 3, 1, 'v', 0}};
    for (Params const &q : dw)
    {
        uint8_t t, b, l, r;
        pads_of(q, t, b, l, r);
        const auto pe = q.p == 'f' ? small::PADDING_F : small::PADDING_V;
        const size_t Ho = small::compute_output_dim(q.H, q.k, q.s, pe), Wo = small::compute_output_dim(q.W, q.k, q.s, pe);
        FloatBuffer in = read_bin(fname(dir, "in", "dw_conv", q, q.Ci * q.H * q.W, false));
        FloatBuffer fl = read_bin(fname(dir, "filter", "dw_conv", q, q.Ci * q.k * q.k, false));
        FloatBuffer ex = read_bin(fname(dir, "out", "dw_conv", q, q.Ci * Ho * Wo, false));
        if (!in.size() || !fl.size() || !ex.size()) continue;
        FloatBuffer pin(in.size()), pfl(fl.size()), pex(ex.size()), out(ex.size());
        small::pack_buffer(in, small::INPUT, 1, q.Ci, q.H, q.W, 16, 16, pin);
        small::pack_buffer(fl, small::FILTER_DW, q.Ci, 1, q.k, q.k, 16, 16, pfl);
        small::pack_buffer(ex, small::OUTPUT, 1, q.Ci, Ho, Wo, 16, 16, pex);
        small::DepthwiseConv2D(q.k, q.k, q.s, t, b, l, r, q.Ci, q.H, q.W, pin, pfl, out);
        size_t bad = 0;
        for (size_t i = 0; i < out.size(); ++i) bad += !almost_equal(out[i], pex[i]);
        CHECK(bad == 0);
    }
}

static void test_quint8_and_batched()
{
    std::printf("quint8 conv + relu, batched entry points\n");
    // identity-like quantised conv: 1x1 filter with a single tap of (1 - zF) picks channel 0
    const int C = 16, H = 4, W = 4;
    QUInt8Buffer in(C * H * W), fl(C * C), out(C * H * W);
    small::init(in, C * H * W);
    for (size_t i = 0; i < fl.size(); ++i) fl[i] = 0;
    in.m_zero = 0; fl.m_zero = 0;
    for (int c = 0; c < C; ++c) fl[small::packed_weight_index(C, C, 1, 1, 16, 16, c, c, 0, 0)] = 1;
    out.multiplier = (1 << 30); out.lshift = 1; out.rshift = 0;     // acc * 2 * 2^30 / 2^31 = acc
    small::Conv2D(1, 1, 1, 0, 0, 0, 0, C, C, H, W, in, fl, out);
    for (int i = 0; i < C * H * W; ++i) CHECK(out[i] == in[i]);
    // batched float conv: image n of the batched call == the batch-1 call on image n
    const int B = 3, Ci = 16, Co = 32, n_in = Ci * 6 * 6, n_out = Co * 6 * 6;
    FloatBuffer bx(B * n_in), bf(Co * Ci * 9), by(B * n_out), y1(n_out), x1(n_in);
    small::init(bx, B * n_in);
    small::init(bf, Co * Ci * 9);
    small::batched::Conv2D(B, 3, 3, 1, 1, 1, 1, 1, Co, Ci, 6, 6, bx, bf, by);
    for (int n = 0; n < B; ++n)
    {
        for (int i = 0; i < n_in; ++i) x1[i] = bx[n * n_in + i];
        small::Conv2D(3, 3, 1, 1, 1, 1, 1, Co, Ci, 6, 6, x1, bf, y1);
        for (int i = 0; i < n_out; ++i) CHECK(y1[i] == by[n * n_out + i]);
    }
    // fused bias + conv + relu == Bias, PartialConv2D, ReLUActivation
    FloatBuffer bias(Co), fused(n_out), seq(n_out);
    small::init(bias, Co);
    small::batched::Conv2D_Bias_Act(1, 3, 3, 1, 1, 1, 1, 1, Co, Ci, 6, 6, x1, bf, bias, small::RELU, 0.f, fused);
    small::Bias(Co, 6, 6, bias, seq);
    small::PartialConv2D(3, 3, 1, 1, 1, 1, 1, Co, Ci, 6, 6, x1, bf, seq);
    small::ReLUActivation(Co, 6, 6, seq, seq);
    for (int i = 0; i < n_out; ++i) CHECK(almost_equal(fused[i], seq[i], 1e-4f));
    // Dense == Conv2D on a 1x1 image
    FloatBuffer dx(64), dw(32 * 64), dy(32), cy(32);
    small::init(dx, 64);
    small::init(dw, 32 * 64);
    small::Dense(32, 64, dx, dw, dy);
    small::Conv2D(1, 1, 1, 0, 0, 0, 0, 32, 64, 1, 1, dx, dw, cy);
    for (int i = 0; i < 32; ++i) CHECK(dy[i] == cy[i]);
}

static void test_fused_conv_pool_dropout_softmax()
{
    std::printf("fused convolution + pooling, dropout, softmax\n");
    // Conv2D_Bias_ReLU_Maxpool2D == Conv2D_Bias_Act, then MaxPool2D: 2x2 stride 2 (one launch) and 3x3 stride 2
    // (runs through the intermediate buffer)
    const int Ci = 16, Co = 32, H = 12, W = 16;      // 4 x 8 pixel tiles fill this map: the 2x2 pool is fused
    FloatBuffer x(Ci * H * W), f(Co * Ci * 9), bias(Co), mid(Co * H * W), inter(Co * H * W);
    small::init(x, x.size());
    small::init(f, f.size());
    small::init(bias, Co);
    small::batched::Conv2D_Bias_Act(1, 3, 3, 1, 1, 1, 1, 1, Co, Ci, H, W, x, f, bias, small::RELU, 0.f, mid);
    for (int pk = 2; pk <= 3; ++pk)
    {
        const int Hp = (H - pk) / 2 + 1, Wp = (W - pk) / 2 + 1;
        FloatBuffer want(Co * Hp * Wp), got(Co * Hp * Wp);
        small::MaxPool2D(pk, pk, 2, 0, 0, 0, 0, Co, H, W, mid, want);
        small::Conv2D_Bias_ReLU_Maxpool2D(3, 3, 1, 1, 1, 1, 1, pk, pk, 2, 0, 0, 0, 0, Co, Ci, H, W, x, f, bias, inter, got);
        for (size_t i = 0; i < want.size(); ++i) CHECK(almost_equal(got[i], want[i], 1e-4f));
    }
    // Timer brackets device work: a launch between start() and stop() shows up as a positive interval
    small::Timer timer;
    timer.start();
    small::batched::Conv2D_Bias_Act(1, 3, 3, 1, 1, 1, 1, 1, Co, Ci, H, W, x, f, bias, small::RELU, 0.f, mid);
    timer.stop();
    CHECK(timer.elapsed() > 0.0 && timer.elapsed() < 5.0e9);
    // Dropout = multiplication by filter[0]; SoftMax sums to one over the whole tensor
    FloatBuffer rate(1), d(Ci * H * W), sm(Ci * H * W);
    rate[0] = 0.75f;
    small::Dropout(Ci, H, W, x, rate, d);
    for (size_t i = 0; i < d.size(); ++i) CHECK(d[i] == x[i] * 0.75f);
    small::SoftMax(Ci, H, W, x, sm);
    double total = 0;
    for (size_t i = 0; i < sm.size(); ++i) total += sm[i];
    CHECK(std::fabs(total - 1.0) < 1e-5);
    CHECK(almost_equal(sm[5] / sm[6], std::exp(x[5] - x[6]), 1e-4f));
}

static void test_group_conv()
{
    std::printf("grouped convolution\n");
    // GroupConv2D over G slabs of C channels == Conv2D(C -> C) on each slab with its own filter block;
    // PartialGroupConv2D adds the same into the output
    const int G = 3, Cg = 16, H = 7, W = 9, nf = Cg * Cg * 9, nx = Cg * H * W;
    FloatBuffer x(G * nx), f(G * nf), got(G * nx), twice(G * nx);
    small::init(x, x.size());
    small::init(f, f.size());
    small::GroupConv2D(3, 3, 1, G, 1, 1, 1, 1, Cg, H, W, x, f, got);
    for (size_t i = 0; i < twice.size(); ++i) twice[i] = got[i];
    small::PartialGroupConv2D(3, 3, 1, G, 1, 1, 1, 1, Cg, H, W, x, f, twice);
    for (int g = 0; g < G; ++g)
    {
        FloatBuffer xs(nx), fs(nf), want(nx);
        for (int i = 0; i < nx; ++i) xs[i] = x[g * nx + i];
        for (int i = 0; i < nf; ++i) fs[i] = f[g * nf + i];
        small::Conv2D(3, 3, 1, 1, 1, 1, 1, Cg, Cg, H, W, xs, fs, want);
        for (int i = 0; i < nx; ++i)
        {
            CHECK(got[g * nx + i] == want[i]);
            CHECK(almost_equal(twice[g * nx + i], want[i] + want[i], 1e-4f));
        }
    }
}

int main(int argc, char **argv)
{
    const std::string dir = argc > 1 ? argv[1] : "tests/golden/ref_regression";
    if (small_hip_device_count() < 1) { std::printf("no GPU\n"); return 2; }
    test_buffer_semantics();
    test_shapes_and_packing();
    test_relu_leaky_accum_upsample_concat();
    test_exceptions();
    test_conv2d_fixtures(dir);
    test_window_fixtures(dir);
    test_quint8_and_batched();
    test_fused_conv_pool_dropout_softmax();
    test_group_conv();
    std::printf(g_fail ? "FAILED: %d checks\n" : "ALL PASSED\n", g_fail);
    return g_fail ? 1 : 0;
}

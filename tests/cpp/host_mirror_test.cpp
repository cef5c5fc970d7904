// Exercises the C++ host layer (include/autograph_hip.hpp) end to end.
//
//   host_mirror_test cpu
//       no GPU: option shape formulas, bf16 conversion, error behaviour before agh_init.
//   host_mirror_test gpu <in.bin> <out.bin>
//       in.bin  (f32, little endian): bs, then x[bs,1,28,28], w1[6,1,5,5], w2[16,6,5,5], wd1[256,128],
//               wd2[128,84], wd3[84,10], b3[10], a[37,53], b[41,53]
//       out.bin (f32): logits of LeNet5.forward [bs,10], logits of forward_single_launch [bs,10],
//               bf16 LeNet5.forward logits widened to f32 [bs,10], a.dot(b.t()) [37,41],
//               col2im(im2col(x)) with a 5x5 filter [bs,1,28,28], act = relu(conv1(x)) [bs,6,24,24],
//               max_pool2_backward of ones on act [bs,6,24,24]
// The pytest side writes in.bin, runs this program and compares out.bin with the CPU oracle.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <string>

#include "autograph_hip.hpp"

using namespace agh;

#define REQUIRE(cond)                                                        \
    do {                                                                     \
        if (!(cond)) {                                                       \
            std::fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            return 1;                                                        \
        }                                                                    \
    } while (0)

static int run_cpu() {
    Im2ColConv2Options o;
    o.filter = {3, 5}; o.padding = {1, 0}; o.stride = {2, 1}; o.dilation = {1, 2};
    REQUIRE((o.output_shape({9, 14}) == std::array<int64_t, 2>{5, 6}));
    Col2ImConv2Options c;
    c.shape = {5, 6}; c.filter = {3, 5}; c.padding = {1, 0}; c.stride = {2, 1}; c.dilation = {1, 2};
    REQUIRE((c.output_shape() == std::array<int64_t, 2>{9, 14}));
    MaxPool2Options p;
    p.size = {2, 3}; p.strides = {2, 2};
    REQUIRE((p.output_shape({9, 8}) == std::array<int64_t, 2>{4, 3}));
    // bf16: ties to even, NaN stays NaN with its quiet bit, round trip of representable values
    REQUIRE(bf16::from_f32(1.0f).bits == 0x3F80);
    REQUIRE(bf16::from_f32(1.00390625f).bits == 0x3F80);   // 1 + 2^-8: tie, even mantissa below
    REQUIRE(bf16::from_f32(1.01171875f).bits == 0x3F82);   // 1 + 3*2^-8: tie, rounds up to even
    REQUIRE(bf16::from_f32(-0.0f).bits == 0x8000);
    REQUIRE((bf16::from_f32(std::nanf("")).bits & 0x7FC0) == 0x7FC0);
    for (uint32_t b = 0; b < 65536; ++b) {
        const bf16 h = bf16::from_bits((uint16_t)b);
        if ((b & 0x7FFF) > 0x7F80) continue;
        REQUIRE(bf16::from_f32(h.to_f32()).bits == b);
    }
    REQUIRE((standard_strides({2, 3, 4}) == Shape{12, 4, 1}));
    // before agh_init every call reports AGH_ENOINIT as an exception, nothing crashes
    try {
        Tensor<float>::uninit({2, 2});
        REQUIRE(false);
    } catch (const Error &e) {
        REQUIRE(e.code() == AGH_ENOINIT);
        REQUIRE(std::string(e.what()).find("agh_init") != std::string::npos);
    }
    // serde: the documents the Python mirror writes for the same data (known answers), and back
    {
        const std::vector<float> f = {1.0f, 2.0f, -0.5f};
        const std::string jf = serde::to_json<float>({3, 1}, f);
        REQUIRE(jf == "{\"dim\":[3,1],\"buffer\":[\"F32\",3,[141008071295040,820338753536]]}");
        const std::vector<bf16> h = {bf16::from_bits(0x3F80), bf16::from_bits(0x4000), bf16::from_bits(0xBF00), bf16::from_bits(0x7FC0),
                                     bf16::from_bits(0x0001)};
        const std::string jh = serde::to_json<bf16>({5}, h);
        REQUIRE(jh == "{\"dim\":[5],\"buffer\":[\"BF16\",5,[9241105235278020735,72057594037927936]]}");
        Shape dim;
        std::vector<float> fb;
        serde::from_json<float>(" { \"buffer\" : [ \"F32\", 3, [141008071295040, 820338753536] ], \"dim\": [3, 1] } ", dim, fb);
        REQUIRE((dim == Shape{3, 1}) && fb == f);
        std::vector<bf16> hb;
        serde::from_json<bf16>(jh, dim, hb);
        REQUIRE((dim == Shape{5}) && hb.size() == 5 && hb[3].bits == 0x7FC0 && hb[4].bits == 0x0001);
        const char *bad[] = {"{\"dim\":[3],\"buffer\":[\"BF16\",3,[1,2]]}",         // wrong scalar type for Tensor<f32>
                             "{\"dim\":[4],\"buffer\":[\"F32\",3,[1,2]]}",          // dim does not hold 3 elements
                             "{\"dim\":[3],\"buffer\":[\"F32\",3,[1]]}",            // too few items
                             "{\"dim\":[3],\"buffer\":[\"F32\",3,[1,2]],\"x\":1}",  // unknown field
                             "{\"dim\":[3]}"};
        for (const char *b : bad) {
            bool threw = false;
            try {
                serde::from_json<float>(b, dim, fb);
            } catch (const Error &) {
                threw = true;
            }
            REQUIRE(threw);
        }
    }
    std::puts("cpu ok");
    return 0;
}

template <typename T> static std::vector<T> convert(const std::vector<float> &v);
template <> std::vector<float> convert<float>(const std::vector<float> &v) { return v; }
template <> std::vector<bf16> convert<bf16>(const std::vector<float> &v) {
    std::vector<bf16> r(v.size());
    for (size_t i = 0; i < v.size(); ++i) r[i] = bf16::from_f32(v[i]);
    return r;
}

template <typename T> static LeNet5<T> make_model(const std::vector<std::vector<float>> &p) {
    LeNet5<T> m;
    m.conv1.weight = Tensor<T>::from_vec({6, 1, 5, 5}, convert<T>(p[0]));
    m.conv2.weight = Tensor<T>::from_vec({16, 6, 5, 5}, convert<T>(p[1]));
    m.dense1.weight = Tensor<T>::from_vec({256, 128}, convert<T>(p[2]));
    m.dense2.weight = Tensor<T>::from_vec({128, 84}, convert<T>(p[3]));
    m.dense3.weight = Tensor<T>::from_vec({84, 10}, convert<T>(p[4]));
    m.dense3.bias = std::make_shared<Tensor<T>>(Tensor<T>::from_vec({10}, convert<T>(p[5])));
    return m;
}

static int run_gpu(const char *in_path, const char *out_path) {
    FILE *f = std::fopen(in_path, "rb");
    REQUIRE(f != nullptr);
    float bsf = 0;
    REQUIRE(std::fread(&bsf, 4, 1, f) == 1);
    const int64_t bs = (int64_t)bsf;
    auto read = [&](size_t n) {
        std::vector<float> v(n);
        if (std::fread(v.data(), 4, n, f) != n) { std::fprintf(stderr, "short read\n"); std::exit(2); }
        return v;
    };
    const std::vector<float> x = read((size_t)bs * 784);
    std::vector<std::vector<float>> p = {read(150), read(2400), read(256 * 128), read(128 * 84), read(840), read(10)};
    const std::vector<float> a = read(37 * 53), b = read(41 * 53);
    std::fclose(f);

    Device device(0);
    std::vector<float> out;
    auto append = [&](const std::vector<float> &v) { out.insert(out.end(), v.begin(), v.end()); };

    const LeNet5<float> model = make_model<float>(p);
    const Tensor<float> tx = Tensor<float>::from_vec({bs, 1, 28, 28}, x);
    append(model.forward(tx).into_vec());
    Tensor<float> logits = Tensor<float>::uninit({bs, 10});
    model.forward_single_launch(tx, logits.buffer_ptr());
    append(logits.into_vec());

    const LeNet5<bf16> model16 = make_model<bf16>(p);
    const Tensor<bf16> tx16 = Tensor<bf16>::from_vec({bs, 1, 28, 28}, convert<bf16>(x));
    for (bf16 h : model16.forward(tx16).into_vec()) out.push_back(h.to_f32());

    // dot with a transposed view: [37,53] x [41,53]^T
    const Tensor<float> ta = Tensor<float>::from_vec({37, 53}, a), tb = Tensor<float>::from_vec({41, 53}, b);
    append(ta.dot(tb.t()).into_vec());
    // shape errors are the reference's messages, raised before any launch
    try {
        ta.dot(tb);
        REQUIRE(false);
    } catch (const Error &e) {
        REQUIRE(std::string(e.what()) == "a_cols != b_rows, 53 != 41");
    }
    try {
        ta.t().into_shape({53 * 37});
        REQUIRE(false);
    } catch (const Error &e) {
        REQUIRE(e.code() == AGH_EINVAL);
    }

    Im2ColConv2Options io;
    io.filter = {5, 5};
    Col2ImConv2Options co;
    co.shape = {24, 24};
    co.filter = {5, 5};
    append(tx.im2col_conv2(io).col2im_conv2(co).into_vec());

    const Tensor<float> act = model.conv1.forward(tx).relu();  // [bs,6,24,24]
    append(act.into_vec());
    const MaxPool2Options po;
    const Tensor<float> pooled = act.max_pool2(po);
    Tensor<float> grad = act.clone();
    grad.max_pool2_backward(Tensor<float>::from_vec(pooled.shape(), std::vector<float>((size_t)pooled.len(), 1.0f)), po);
    append(grad.into_vec());
    // the fused Relu -> MaxPool2 pair and its backward equal the separate calls bit for bit
    const Tensor<float> pre = model.conv1.forward(tx);  // [bs,6,24,24], the relu's input
    REQUIRE(pre.relu_max_pool2(po).into_vec() == pooled.into_vec());
    const Tensor<float> ones = Tensor<float>::from_vec(pooled.shape(), std::vector<float>((size_t)pooled.len(), 1.0f));
    const Tensor<float> fused_grad = pre.max_pool2_relu_backward(ones, po);
    REQUIRE(fused_grad.into_vec() == pre.relu_backward(grad).into_vec());
    REQUIRE(pre.max_pool2_relu_backward(ones, po, true).into_vec() ==
            fused_grad.permuted_axes({0, 2, 3, 1}).to_standard_layout().into_vec());
    // Dense as the reference's separate calls (dot, broadcast add_assign, relu) equals the fused launch bit for bit
    {
        const Tensor<float> h = Tensor<float>::from_vec({37, 53}, a);
        Dense<float> dn;
        dn.weight = Tensor<float>::from_vec({53, 41}, b);
        dn.bias = std::make_shared<Tensor<float>>(Tensor<float>::from_vec({41}, std::vector<float>(b.begin(), b.begin() + 41)));
        REQUIRE(dn.forward(h, true).into_vec() == dn.forward_unfused(h, true).into_vec());
        REQUIRE(dn.forward(h).into_vec() == dn.forward_unfused(h).into_vec());
        // scaled_add into a transposed view: (y^T += 2 x) == (y += 2 x^T)
        Tensor<float> y1 = Tensor<float>::from_vec({37, 53}, a), y2 = Tensor<float>::from_vec({37, 53}, a);
        const Tensor<float> xs = Tensor<float>::from_vec({53, 37}, std::vector<float>(b.begin(), b.begin() + 53 * 37));
        Tensor<float> y1t = y1.t();
        y1t.scaled_add(2.0f, xs);
        y2.scaled_add(2.0f, xs.t().to_standard_layout());
        REQUIRE(y1.into_vec() == y2.into_vec());
        try {
            y1.scaled_add(1.0f, Tensor<float>::from_vec({5}, std::vector<float>(5, 1.0f)));
            REQUIRE(false);
        } catch (const Error &e) {
            REQUIRE(std::string(e.what()).rfind("Broadcast not possible!", 0) == 0);
        }
    }
    // a permuted view copies into standard layout
    REQUIRE(act.permuted_axes({0, 2, 3, 1}).to_standard_layout().permuted_axes({0, 3, 1, 2}).into_vec() == act.into_vec());
    device.wait();

    FILE *g = std::fopen(out_path, "wb");
    REQUIRE(g != nullptr);
    REQUIRE(std::fwrite(out.data(), 4, out.size(), g) == out.size());
    std::fclose(g);
    std::puts("gpu ok");
    return 0;
}

int main(int argc, char **argv) {
    try {
        if (argc == 2 && std::string(argv[1]) == "cpu") return run_cpu();
        if (argc == 4 && std::string(argv[1]) == "gpu") return run_gpu(argv[2], argv[3]);
    } catch (const Error &e) {
        std::fprintf(stderr, "agh::Error [%d]: %s\n", e.code(), e.what());
        return 3;
    }
    std::fprintf(stderr, "usage: host_mirror_test cpu | gpu <in.bin> <out.bin>\n");
    return 64;
}

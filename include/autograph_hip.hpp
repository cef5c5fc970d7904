// C++17 host layer over the C ABI of autograph_hip.h: the reference's tensor and layer
// interface for the dense-contraction path (Device, Buffer, Tensor{dim, strides, offset}, the
// option structs, Conv2 / Dense / MaxPool2 / Relu / Flatten, LeNet5), with the same names,
// argument meaning and error behaviour as the Rust originals cited at each item.  Header only;
// link against libautograph_hip.so.  Errors are exceptions (agh::Error) where the reference
// returns anyhow::Result.
#ifndef AUTOGRAPH_HIP_HPP
#define AUTOGRAPH_HIP_HPP

#include <array>
#include <cstdint>
#include <cstring>
#include <memory>
#include <numeric>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

#include "autograph_hip.h"

namespace agh {

class Error : public std::runtime_error {
public:
    Error(int code, const std::string &msg) : std::runtime_error(msg), code_(code) {}
    int code() const { return code_; }

private:
    int code_;
};

inline void check(int status) {
    if (status != AGH_OK) throw Error(status, agh_last_error_string());
}
[[noreturn]] inline void bail(const std::string &msg) { throw Error(AGH_EINVAL, msg); }

// half::bf16 (crate `half`): raw bits, round-to-nearest-even from f32, NaN keeps its top payload
// bits and gets the quiet bit.
struct bf16 {
    uint16_t bits = 0;
    bf16() = default;
    static bf16 from_bits(uint16_t b) { bf16 r; r.bits = b; return r; }
    static bf16 from_f32(float v) {
        uint32_t x;
        std::memcpy(&x, &v, 4);
        if ((x & 0x7FFFFFFFu) > 0x7F800000u) return from_bits((uint16_t)((x >> 16) | 0x0040u));
        const uint32_t round_bit = 0x8000u;
        if ((x & round_bit) != 0 && (x & (3 * round_bit - 1)) != 0) return from_bits((uint16_t)((x >> 16) + 1));
        return from_bits((uint16_t)(x >> 16));
    }
    float to_f32() const {
        uint32_t x = (uint32_t)bits << 16;
        float f;
        std::memcpy(&f, &x, 4);
        return f;
    }
};
static_assert(sizeof(bf16) == 2, "bf16 is the raw 16-bit pattern");

template <typename T> struct Scalar;
template <> struct Scalar<float> { static constexpr const char *name = "F32"; };
template <> struct Scalar<bf16> { static constexpr const char *name = "BF16"; };

// krnl `Device`: one device, one in-order queue.
class Device {
public:
    explicit Device(int index = 0) : index_(index) { check(agh_init(index)); }
    int index() const { return index_; }
    void wait() const { check(agh_sync()); }  // `device.wait()`
    int compute_units() const {
        int cus = 0;
        check(agh_device_info(nullptr, 0, &cus, nullptr));
        return cus;
    }

private:
    int index_;
};

// krnl `Buffer<T>`: owning device allocation, freed on drop.
template <typename T> class Buffer {
public:
    explicit Buffer(size_t len) : len_(len) { check(agh_malloc(&ptr_, (len ? len : 1) * sizeof(T))); }
    Buffer(const Buffer &) = delete;
    Buffer &operator=(const Buffer &) = delete;
    ~Buffer() { if (ptr_) agh_free(ptr_); }
    void *ptr() const { return ptr_; }
    size_t len() const { return len_; }

private:
    void *ptr_ = nullptr;
    size_t len_;
};

// ---- option structs, src/ops.rs:9-108 ----
struct Im2ColConv2Options {
    std::array<int64_t, 2> filter{0, 0}, padding{0, 0}, stride{1, 1}, dilation{1, 1};
    // src/ops.rs:35: o = (i + 2p - d(f-1) - 1)/s + 1
    std::array<int64_t, 2> output_shape(std::array<int64_t, 2> input) const {
        std::array<int64_t, 2> o{};
        for (int a = 0; a < 2; ++a) o[a] = (input[a] + 2 * padding[a] - dilation[a] * (filter[a] - 1) - 1) / stride[a] + 1;
        return o;
    }
};
struct Col2ImConv2Options {
    std::array<int64_t, 2> shape{0, 0}, filter{0, 0}, padding{0, 0}, stride{1, 1}, dilation{1, 1};
    // src/ops.rs:75: o = (i-1)s + d(f-1) + 1 - 2p
    std::array<int64_t, 2> output_shape() const {
        std::array<int64_t, 2> o{};
        for (int a = 0; a < 2; ++a) o[a] = (shape[a] - 1) * stride[a] + dilation[a] * (filter[a] - 1) + 1 - 2 * padding[a];
        return o;
    }
};
struct MaxPool2Options {
    std::array<int64_t, 2> size{2, 2}, strides{2, 2};
    // src/ops.rs:99: o = (i - x)/s + 1
    std::array<int64_t, 2> output_shape(std::array<int64_t, 2> input) const {
        return {(input[0] - size[0]) / strides[0] + 1, (input[1] - size[1]) / strides[1] + 1};
    }
};

using Shape = std::vector<int64_t>;

inline Shape standard_strides(const Shape &dim) {
    Shape s(dim.size());
    int64_t acc = 1;
    for (size_t i = dim.size(); i-- > 0;) { s[i] = acc; acc *= dim[i]; }
    return s;
}
inline int64_t shape_len(const Shape &dim) {
    return std::accumulate(dim.begin(), dim.end(), (int64_t)1, std::multiplies<int64_t>());
}
inline std::string shape_str(const Shape &d) {
    std::string s = "[";
    for (size_t i = 0; i < d.size(); ++i) s += (i ? ", " : "") + std::to_string(d[i]);
    return s + "]";
}

template <typename T> class Tensor;
template <typename T> void gemm(float alpha, const Tensor<T> &a, const Tensor<T> &b, float beta, Tensor<T> &c,
                                const Tensor<T> *bias = nullptr, bool relu = false);

// `TensorBase` = {dim, strides, buffer, offset} (src/tensor.rs:327-332); views share the buffer.
template <typename T> class Tensor {
    static_assert(std::is_same<T, float>::value || std::is_same<T, bf16>::value, "f32 and bf16 only");
    static constexpr bool kBf16 = std::is_same<T, bf16>::value;

public:
    Tensor() = default;
    Tensor(std::shared_ptr<Buffer<T>> buffer, Shape dim, Shape strides, int64_t offset)
        : buffer_(std::move(buffer)), dim_(std::move(dim)), strides_(std::move(strides)), offset_(offset) {}

    // -- construction / transfer (src/tensor.rs:1377-1416, :1775-1833, :1923-1934) --
    static Tensor uninit(const Shape &dim) {
        return Tensor(std::make_shared<Buffer<T>>((size_t)shape_len(dim)), dim, standard_strides(dim), 0);
    }
    static Tensor zeros(const Shape &dim) {
        Tensor t = uninit(dim);
        check(agh_memset(t.buffer_->ptr(), 0, (size_t)shape_len(dim) * sizeof(T)));
        return t;
    }
    static Tensor from_vec(const Shape &dim, const std::vector<T> &data) {
        if ((int64_t)data.size() != shape_len(dim)) bail("from_vec: " + std::to_string(data.size()) + " elements for shape " + shape_str(dim));
        Tensor t = uninit(dim);
        check(agh_memcpy_h2d(t.buffer_->ptr(), data.data(), data.size() * sizeof(T)));
        check(agh_sync());
        return t;
    }
    // `into_array().into_raw_vec()`: blocking, standard layout
    std::vector<T> into_vec() const {
        const Tensor s = as_standard_layout();
        std::vector<T> out((size_t)s.len());
        check(agh_memcpy_d2h(out.data(), s.data_ptr(), out.size() * sizeof(T)));
        return out;
    }

    // -- shape --
    const Shape &shape() const { return dim_; }
    const Shape &strides() const { return strides_; }
    int64_t offset() const { return offset_; }
    size_t ndim() const { return dim_.size(); }
    int64_t len() const { return shape_len(dim_); }
    void *buffer_ptr() const { return buffer_->ptr(); }
    void *data_ptr() const { return (char *)buffer_->ptr() + offset_ * (int64_t)sizeof(T); }
    bool is_standard_layout() const {
        const Shape s = standard_strides(dim_);
        for (size_t i = 0; i < dim_.size(); ++i)
            if (dim_[i] != 1 && strides_[i] != s[i]) return false;
        return true;
    }

    // -- views (src/tensor.rs:695-703, :103-122) --
    Tensor t() const { return reversed_axes(); }
    Tensor reversed_axes() const {
        return Tensor(buffer_, Shape(dim_.rbegin(), dim_.rend()), Shape(strides_.rbegin(), strides_.rend()), offset_);
    }
    Tensor permuted_axes(const std::vector<size_t> &axes) const {
        if (axes.size() != ndim()) bail("permuted_axes: wrong number of axes");
        Shape d, s;
        for (size_t a : axes) { d.push_back(dim_.at(a)); s.push_back(strides_.at(a)); }
        return Tensor(buffer_, d, s, offset_);
    }
    Tensor into_shape(const Shape &dim) const {
        if (!is_standard_layout()) bail("into_shape: incompatible layout");  // ShapeError::IncompatibleLayout
        if (shape_len(dim) != len()) bail("into_shape: incompatible shape " + shape_str(dim_) + " -> " + shape_str(dim));
        return Tensor(buffer_, dim, standard_strides(dim), offset_);
    }
    Tensor flatten() const { return into_shape({dim_.at(0), len() / std::max<int64_t>(1, dim_.at(0))}); }
    Tensor as_standard_layout() const { return is_standard_layout() ? *this : to_standard_layout(); }
    // strided copy: `assign` with BinaryOp::Identity (src/tensor/ops.rs:257-318)
    Tensor to_standard_layout() const {
        if (ndim() > 4) bail("to_standard_layout: more than 4 dimensions");
        Tensor out = uninit(dim_);
        int64_t d[4] = {1, 1, 1, 1}, sx[4] = {0, 0, 0, 0}, sy[4] = {0, 0, 0, 0};
        const size_t pad = 4 - ndim();
        for (size_t i = 0; i < ndim(); ++i) { d[pad + i] = dim_[i]; sx[pad + i] = strides_[i]; sy[pad + i] = out.strides_[i]; }
        check((kBf16 ? agh_assign_bf16 : agh_assign_f32)(buffer_ptr(), offset_, sx[0], sx[1], sx[2], sx[3], out.buffer_ptr(), 0,
                                                         sy[0], sy[1], sy[2], sy[3], d[0], d[1], d[2], d[3]));
        return out;
    }

    // -- Dot (src/tensor/linalg.rs:362-468): fresh standard-layout output, alpha = 1, beta = 0 --
    Tensor dot(const Tensor &rhs) const { return dot_impl(rhs, nullptr, false); }
    // Dense epilogue fused into the same launch: + bias (broadcast over rows), then relu
    Tensor dot_bias_relu(const Tensor &rhs, const Tensor *bias, bool relu) const { return dot_impl(rhs, bias, relu); }

    // -- Im2ColConv2 / Col2ImConv2 (src/tensor/ops.rs:831-888, :982-1037) --
    Tensor im2col_conv2(const Im2ColConv2Options &o) const {
        if (ndim() != 4) bail("im2col_conv2: expected a 4-D tensor");
        const Tensor x = as_standard_layout();
        const int64_t bs = dim_[0], c = dim_[1], ih = dim_[2], iw = dim_[3];
        const auto out = o.output_shape({ih, iw});
        Tensor y = uninit({bs * out[0] * out[1], c * o.filter[0] * o.filter[1]});
        check((kBf16 ? agh_im2col_conv2_bf16 : agh_im2col_conv2_f32)(x.data_ptr(), y.buffer_ptr(), bs, c, ih, iw, o.filter[0], o.filter[1],
                                                                     o.padding[0], o.padding[1], o.stride[0], o.stride[1],
                                                                     o.dilation[0], o.dilation[1]));
        return y;
    }
    Tensor col2im_conv2(const Col2ImConv2Options &o) const {
        if (ndim() != 2) bail("col2im_conv2: expected a 2-D tensor");
        const Tensor x = as_standard_layout();
        const int64_t ih = o.shape[0], iw = o.shape[1], ff = o.filter[0] * o.filter[1];
        if (ih * iw == 0 || ff == 0 || dim_[0] % (ih * iw) != 0 || dim_[1] % ff != 0)
            bail("col2im_conv2: input " + shape_str(dim_) + " does not match the patch grid / filter");
        const int64_t bs = dim_[0] / (ih * iw), c = dim_[1] / ff;
        const auto out = o.output_shape();
        Tensor y = uninit({bs, c, out[0], out[1]});
        check((kBf16 ? agh_col2im_conv2_bf16 : agh_col2im_conv2_f32)(x.data_ptr(), y.buffer_ptr(), bs, c, ih, iw, o.filter[0], o.filter[1],
                                                                     o.padding[0], o.padding[1], o.stride[0], o.stride[1],
                                                                     o.dilation[0], o.dilation[1]));
        return y;
    }

    // -- MaxPool2 / MaxPool2Backward (src/tensor/ops.rs:1106-1141, :1228-1275) --
    Tensor max_pool2(const MaxPool2Options &o) const {
        if (ndim() != 4) bail("max_pool2: expected a 4-D tensor");
        const Tensor x = as_standard_layout();
        const auto out = o.output_shape({dim_[2], dim_[3]});
        Tensor y = uninit({dim_[0], dim_[1], out[0], out[1]});
        check((kBf16 ? agh_max_pool2_bf16 : agh_max_pool2_f32)(x.data_ptr(), y.buffer_ptr(), dim_[0] * dim_[1], dim_[2], dim_[3], o.size[0],
                                                               o.size[1], o.strides[0], o.strides[1]));
        return y;
    }
    // in place: *this holds x on entry and the input gradient on return (layer.rs:1203-1211 clones x first)
    void max_pool2_backward(const Tensor &output_grad, const MaxPool2Options &o) {
        if (!is_standard_layout()) bail("max_pool2_backward: input gradient must be in standard layout");
        const Tensor dy = output_grad.as_standard_layout();
        check((kBf16 ? agh_max_pool2_backward_bf16 : agh_max_pool2_backward_f32)(data_ptr(), dy.data_ptr(), dim_[0] * dim_[1], dim_[2],
                                                                                 dim_[3], o.size[0], o.size[1], o.strides[0],
                                                                                 o.strides[1]));
    }

    // Relu then MaxPool2 in one launch (layer.rs:1253-1267, :1193-1216): same bits as relu().max_pool2(o)
    Tensor relu_max_pool2(const MaxPool2Options &o) const {
        if (ndim() != 4) bail("relu_max_pool2: expected a 4-D tensor");
        const Tensor x = as_standard_layout();
        const auto out = o.output_shape({dim_[2], dim_[3]});
        Tensor y = uninit({dim_[0], dim_[1], out[0], out[1]});
        check((kBf16 ? agh_relu_max_pool2_bf16 : agh_relu_max_pool2_f32)(x.data_ptr(), y.buffer_ptr(), dim_[0] * dim_[1], dim_[2], dim_[3],
                                                                         o.size[0], o.size[1], o.strides[0], o.strides[1]));
        return y;
    }
    // the backward edges of that pair in one launch, *this being the relu's input (layer.rs:205-220, :1542-1565);
    // `nhwc` returns the gradient as [bs, h, w, c] in standard layout (autograd.rs:429-445).  Windows must not overlap.
    Tensor max_pool2_relu_backward(const Tensor &output_grad, const MaxPool2Options &o, bool nhwc = false) const {
        if (ndim() != 4) bail("max_pool2_relu_backward: expected a 4-D tensor");
        const Tensor x = as_standard_layout(), dy = output_grad.as_standard_layout();
        Tensor dx = nhwc ? uninit({dim_[0], dim_[2], dim_[3], dim_[1]}) : uninit(dim_);
        check((kBf16 ? agh_max_pool2_relu_backward_bf16 : agh_max_pool2_relu_backward_f32)(
            x.data_ptr(), dy.data_ptr(), dx.buffer_ptr(), dim_[0], dim_[1], dim_[2], dim_[3], o.size[0], o.size[1], o.strides[0],
            o.strides[1], nhwc ? 1 : 0));
        return dx;
    }

    // -- relu (layer.rs:1269-1510) --
    Tensor relu() const {
        const Tensor x = as_standard_layout();
        Tensor y = uninit(dim_);
        check((kBf16 ? agh_relu_bf16 : agh_relu_f32)(x.data_ptr(), y.buffer_ptr(), len()));
        return y;
    }
    Tensor relu_backward(const Tensor &output_grad) const {
        const Tensor x = as_standard_layout(), dy = output_grad.as_standard_layout();
        Tensor dx = uninit(dim_);
        check((kBf16 ? agh_relu_backward_bf16 : agh_relu_backward_f32)(x.data_ptr(), dy.data_ptr(), dx.buffer_ptr(), len()));
        return dx;
    }

    // -- broadcast (ndarray `broadcast`: trailing axes aligned, stride 0 where a dimension of 1 is stretched) --
    bool broadcast(const Shape &shape, Tensor &out) const {
        if (shape.size() < ndim()) return false;
        const size_t pad = shape.size() - ndim();
        Shape st(shape.size(), 0);
        for (size_t i = 0; i < ndim(); ++i) {
            if (dim_[i] == shape[pad + i]) st[pad + i] = strides_[i];
            else if (dim_[i] != 1) return false;
        }
        out = Tensor(buffer_, shape, st, offset_);
        return true;
    }
    // -- scaled_add / add_assign (src/tensor/ops.rs:192-204, :245-255, :257-318), sum_axis(Axis(0)) (reduce.rs:59-113) --
    void scaled_add(float alpha, const Tensor &rhs) {
        Tensor x;
        if (!rhs.broadcast(dim_, x)) bail("Broadcast not possible! " + shape_str(rhs.dim_) + " -> " + shape_str(dim_));
        if (is_standard_layout() && rhs.dim_ == dim_ && rhs.is_standard_layout()) {
            check((kBf16 ? agh_scaled_add_bf16 : agh_scaled_add_f32)(data_ptr(), alpha, rhs.data_ptr(), len()));
            return;
        }
        if (ndim() > 4) bail("scaled_add: more than 4 dimensions");
        int64_t d[4] = {1, 1, 1, 1}, sx[4] = {0, 0, 0, 0}, sy[4] = {0, 0, 0, 0};
        const size_t pad = 4 - ndim();
        for (size_t i = 0; i < ndim(); ++i) { d[pad + i] = dim_[i]; sx[pad + i] = x.strides_[i]; sy[pad + i] = strides_[i]; }
        check((kBf16 ? agh_scaled_add_strided_bf16 : agh_scaled_add_strided_f32)(
            buffer_ptr(), offset_, sy[0], sy[1], sy[2], sy[3], alpha, x.buffer_ptr(), x.offset_, sx[0], sx[1], sx[2], sx[3],
            d[0], d[1], d[2], d[3]));
    }
    void add_assign(const Tensor &rhs) { scaled_add(1.0f, rhs); }
    Tensor sum_axis0() const {
        if (ndim() != 2) bail("sum_axis0: expected a 2-D tensor");
        const Tensor x = as_standard_layout();
        Tensor y = uninit({dim_[1]});
        check((kBf16 ? agh_sum_axis0_bf16 : agh_sum_axis0_f32)(x.data_ptr(), y.buffer_ptr(), dim_[0], dim_[1]));
        return y;
    }
    Tensor clone() const {
        const Tensor x = as_standard_layout();
        Tensor out = uninit(dim_);
        check(agh_memcpy_d2d(out.buffer_ptr(), x.data_ptr(), (size_t)len() * sizeof(T)));
        return out;
    }

private:
    Tensor dot_impl(const Tensor &rhs, const Tensor *bias, bool relu) const {
        if (ndim() != 2 || rhs.ndim() != 2) bail("dot: both operands must be 2-D");
        Tensor out = uninit({dim_[0], rhs.dim_[1]});
        gemm<T>(1.0f, *this, rhs, 0.0f, out, bias, relu);
        return out;
    }
    std::shared_ptr<Buffer<T>> buffer_;
    Shape dim_, strides_;
    int64_t offset_ = 0;
};

// `fn gemm(alpha, a, b, beta, c)` with the reference's checks (src/tensor/linalg.rs:249-299)
template <typename T>
void gemm(float alpha, const Tensor<T> &a, const Tensor<T> &b, float beta, Tensor<T> &c, const Tensor<T> *bias, bool relu) {
    constexpr bool kBf16 = std::is_same<T, bf16>::value;
    if (a.ndim() != 2 || b.ndim() != 2 || c.ndim() != 2) bail("gemm: operands must be 2-D");
    const int64_t m = a.shape()[0], k = a.shape()[1], k2 = b.shape()[0], n = b.shape()[1], m2 = c.shape()[0], n2 = c.shape()[1];
    if (m != m2) bail("a_rows != c_rows, " + std::to_string(m) + " != " + std::to_string(m2));
    if (k != k2) bail("a_cols != b_rows, " + std::to_string(k) + " != " + std::to_string(k2));
    if (n != n2) bail("b_cols != c_rows, " + std::to_string(n) + " != " + std::to_string(n2));
    if (!bias && !relu) {
        check((kBf16 ? agh_gemm_bf16 : agh_gemm_f32)(m, k, n, alpha, a.buffer_ptr(), a.offset(), a.strides()[0], a.strides()[1], b.buffer_ptr(),
                                                     b.offset(), b.strides()[0], b.strides()[1], beta, c.buffer_ptr(), c.offset(),
                                                     c.strides()[0], c.strides()[1]));
    } else {
        if (bias && (bias->ndim() != 1 || bias->shape()[0] != n)) bail("bias must be a vector of length " + std::to_string(n));
        check((kBf16 ? agh_gemm_bf16_bias_act : agh_gemm_f32_bias_act)(
            m, k, n, alpha, a.buffer_ptr(), a.offset(), a.strides()[0], a.strides()[1], b.buffer_ptr(), b.offset(), b.strides()[0],
            b.strides()[1], beta, c.buffer_ptr(), c.offset(), c.strides()[0], c.strides()[1], bias ? bias->buffer_ptr() : nullptr,
            bias ? bias->offset() : 0, bias ? bias->strides()[0] : 0, relu ? AGH_ACT_RELU : AGH_ACT_NONE));
    }
}

// ---- layers (src/learn/neural_network/layer.rs) ----
// `Conv2` (layer.rs:844-1047): weight [outputs, inputs, fh, fw]; forward = `conv2` (layer.rs:930-948):
// a direct kernel when the geometry has one, else `conv2_im2col` (layer.rs:950-1005) with the
// NHWC -> NCHW copy folded into the batched GEMM.
template <typename T> struct Conv2 {
    Tensor<T> weight;
    std::array<int64_t, 2> padding{0, 0}, stride{1, 1}, dilation{1, 1};
    Tensor<T> forward(const Tensor<T> &input) const {
        constexpr bool kBf16 = std::is_same<T, bf16>::value;
        if (input.ndim() != 4 || weight.ndim() != 4) bail("conv2: expected 4-D input and weight");
        const int64_t bs = input.shape()[0], ic = input.shape()[1], ih = input.shape()[2], iw = input.shape()[3];
        const int64_t oc = weight.shape()[0], fh = weight.shape()[2], fw = weight.shape()[3];
        if (ic != weight.shape()[1]) bail("conv2: input has " + std::to_string(ic) + " channels, weight expects " + std::to_string(weight.shape()[1]));
        Im2ColConv2Options o;
        o.filter = {fh, fw}; o.padding = padding; o.stride = stride; o.dilation = dilation;
        const auto out = o.output_shape({ih, iw});
        Tensor<T> y = Tensor<T>::uninit({bs, oc, out[0], out[1]});
        // like the reference's host, which takes a direct kernel when it can: the library's direct /
        // implicit-GEMM kernels first; AGH_ERANGE says the geometry is not theirs, then im2col + GEMM
        if (input.is_standard_layout() && weight.is_standard_layout()) {
            const int rc = (kBf16 ? agh_conv2_direct_bf16 : agh_conv2_direct_f32)(
                input.data_ptr(), weight.data_ptr(), nullptr, y.buffer_ptr(), bs, ic, ih, iw, oc, fh, fw, padding[0], padding[1], stride[0],
                stride[1], dilation[0], dilation[1], AGH_ACT_NONE, 0);
            if (rc == AGH_OK) return y;
            if (rc != AGH_ERANGE) check(rc);
        }
        const Tensor<T> cols = input.im2col_conv2(o);
        const Tensor<T> wm = weight.into_shape({oc, ic * fh * fw});
        const int64_t L = out[0] * out[1], K = ic * fh * fw;
        check((kBf16 ? agh_gemm_bf16_batched : agh_gemm_f32_batched)(bs, L, K, oc, 1.0f, cols.buffer_ptr(), cols.offset(), K, 1, L * K,
                                                                     wm.buffer_ptr(), wm.offset(), 1, K, 0, 0.0f, y.buffer_ptr(), 0, 1, L,
                                                                     oc * L, nullptr, 0, 0, AGH_ACT_NONE));
        return y;
    }
};
// `Dense` (layer.rs:1050-1143): weight [inputs, outputs], optional bias [outputs]
template <typename T> struct Dense {
    Tensor<T> weight;
    std::shared_ptr<Tensor<T>> bias;
    Tensor<T> forward(const Tensor<T> &input, bool relu = false) const { return input.dot_bias_relu(weight, bias.get(), relu); }
    // the reference's separate calls (layer.rs:1137-1140): dot, broadcast add_assign, then the Relu layer; same bits
    Tensor<T> forward_unfused(const Tensor<T> &input, bool relu = false) const {
        Tensor<T> out = input.dot(weight);
        if (bias) out.add_assign(*bias);
        return relu ? out.relu() : out;
    }
};
// `MaxPool2` (layer.rs:1149-1216); the stride defaults to the filter (layer.rs:535-539)
template <typename T> struct MaxPool2 {
    std::array<int64_t, 2> filter{2, 2}, stride{2, 2};
    Tensor<T> forward(const Tensor<T> &input) const { return input.max_pool2(MaxPool2Options{filter, stride}); }
};
template <typename T> struct Relu { Tensor<T> forward(const Tensor<T> &input) const { return input.relu(); } };
template <typename T> struct Flatten { Tensor<T> forward(const Tensor<T> &input) const { return input.flatten(); } };

// The benchmark's LeNet5 (benches/neural-network-benches/src/autograph_backend.rs:88-162)
template <typename T> struct LeNet5 {
    Conv2<T> conv1, conv2;
    Dense<T> dense1, dense2, dense3;
    // what #[derive(Forward)] expands to: the layers in order
    Tensor<T> forward(const Tensor<T> &x) const {
        const MaxPool2<T> pool;
        const Relu<T> relu;
        Tensor<T> h = pool.forward(relu.forward(conv1.forward(x)));
        h = pool.forward(relu.forward(conv2.forward(h)));
        h = Flatten<T>().forward(h);
        h = relu.forward(dense1.forward(h));
        h = relu.forward(dense2.forward(h));
        return dense3.forward(h);
    }
    // the whole forward pass as one launch; `logits` may point to device memory or memory from agh_host_alloc
    void forward_single_launch(const Tensor<T> &x, void *logits) const {
        constexpr bool kBf16 = std::is_same<T, bf16>::value;
        if (x.ndim() != 4 || x.shape()[1] != 1 || x.shape()[2] != 28 || x.shape()[3] != 28) bail("LeNet5 expects [bs, 1, 28, 28] inputs, got " + shape_str(x.shape()));
        const Tensor<T> xs = x.as_standard_layout();
        check((kBf16 ? agh_lenet5_forward_bf16 : agh_lenet5_forward_f32)(
            xs.data_ptr(), conv1.weight.as_standard_layout().data_ptr(), conv2.weight.as_standard_layout().data_ptr(),
            dense1.weight.as_standard_layout().data_ptr(), dense2.weight.as_standard_layout().data_ptr(),
            dense3.weight.as_standard_layout().data_ptr(), dense3.bias->as_standard_layout().data_ptr(), logits, x.shape()[0]));
    }
};


// ---- serde (src/tensor.rs:1199-1249) ----
// The reference's data model `Tensor { dim: (u64, ..), buffer: Buffer(scalar type, len, [u64, ..]) }` as
// serde_json writes it: {"dim":[..],"buffer":["F32",n,[..]]}.  The u64 items are the buffer's bytes taken
// eight at a time, each group read as a big-endian integer (pinned by the reference's token test,
// src/tensor.rs:2236-2277); a last group that is not full is padded with zero bytes.
namespace serde {
template <typename T> inline const char *scalar_name() { return std::is_same<T, bf16>::value ? "BF16" : "F32"; }

template <typename T> inline std::string to_json(const Shape &dim, const std::vector<T> &data) {
    static_assert(std::is_same<T, float>::value || std::is_same<T, bf16>::value, "f32 and bf16 tensors");
    std::string out = "{\"dim\":[";
    for (size_t i = 0; i < dim.size(); ++i) out += (i ? "," : "") + std::to_string(dim[i]);
    out += std::string("],\"buffer\":[\"") + scalar_name<T>() + "\"," + std::to_string(data.size()) + ",[";
    const unsigned char *raw = reinterpret_cast<const unsigned char *>(data.data());
    const size_t nbytes = data.size() * sizeof(T);
    for (size_t b = 0; b < nbytes; b += 8) {
        uint64_t v = 0;
        for (size_t j = 0; j < 8; ++j) v = (v << 8) | (b + j < nbytes ? raw[b + j] : 0);
        out += (b ? "," : "") + std::to_string(v);
    }
    return out + "]]}";
}

// A reader for exactly this shape of document (any JSON whitespace, the two fields in either order).
class Reader {
public:
    explicit Reader(const std::string &s) : s_(s) {}
    void ws() { while (i_ < s_.size() && (s_[i_] == ' ' || s_[i_] == '\t' || s_[i_] == '\n' || s_[i_] == '\r')) ++i_; }
    bool peek(char c) { ws(); return i_ < s_.size() && s_[i_] == c; }
    void expect(char c) { if (!peek(c)) bail(std::string("serde: expected '") + c + "' at offset " + std::to_string(i_)); ++i_; }
    std::string str() {
        expect('"');
        std::string out;
        while (i_ < s_.size() && s_[i_] != '"') {
            if (s_[i_] == '\\') bail("serde: escapes do not occur in field or type names");
            out += s_[i_++];
        }
        expect('"');
        return out;
    }
    uint64_t u64() {
        ws();
        if (i_ >= s_.size() || s_[i_] < '0' || s_[i_] > '9') bail("serde: expected an unsigned integer at offset " + std::to_string(i_));
        uint64_t v = 0;
        while (i_ < s_.size() && s_[i_] >= '0' && s_[i_] <= '9') {
            const uint64_t d = (uint64_t)(s_[i_++] - '0');
            if (v > (UINT64_MAX - d) / 10) bail("serde: integer does not fit u64");
            v = v * 10 + d;
        }
        return v;
    }
    std::vector<uint64_t> u64_array() {
        std::vector<uint64_t> out;
        expect('[');
        if (peek(']')) { ++i_; return out; }
        for (;;) {
            out.push_back(u64());
            if (peek(',')) { ++i_; continue; }
            expect(']');
            return out;
        }
    }
    void end() { ws(); if (i_ != s_.size()) bail("serde: trailing characters"); }

private:
    const std::string &s_;
    size_t i_ = 0;
};

template <typename T> inline void from_json(const std::string &text, Shape &dim, std::vector<T> &data) {
    Reader r(text);
    bool have_dim = false, have_buf = false;
    std::vector<uint64_t> d, items;
    uint64_t count = 0;
    r.expect('{');
    for (;;) {
        const std::string key = r.str();
        r.expect(':');
        if (key == "dim" && !have_dim) {
            d = r.u64_array();
            have_dim = true;
        } else if (key == "buffer" && !have_buf) {
            r.expect('[');
            const std::string name = r.str();
            if (name != scalar_name<T>()) bail(std::string("Expected ") + scalar_name<T>() + " found " + name);
            r.expect(',');
            count = r.u64();
            r.expect(',');
            items = r.u64_array();
            r.expect(']');
            have_buf = true;
        } else {
            bail("serde: unknown or repeated field `" + key + "`");
        }
        if (r.peek(',')) { r.expect(','); continue; }
        r.expect('}');
        break;
    }
    r.end();
    if (!have_dim || !have_buf) bail("serde: missing field");
    const uint64_t nbytes = count * sizeof(T);
    if (items.size() != (nbytes + 7) / 8) bail("serde: buffer length does not match its items");
    uint64_t prod = 1;
    for (uint64_t x : d) prod *= x;
    if (prod != count) bail("serde: IncompatibleShape");  // into_shape, src/tensor.rs:1245-1247
    dim.assign(d.begin(), d.end());
    data.resize((size_t)count);
    unsigned char *raw = reinterpret_cast<unsigned char *>(data.data());
    for (uint64_t b = 0; b < nbytes; ++b) raw[b] = (unsigned char)(items[b / 8] >> (8 * (7 - b % 8)));
}
}  // namespace serde

template <typename T> inline std::string to_json(const Tensor<T> &t) { return serde::to_json<T>(t.shape(), t.into_vec()); }
template <typename T> inline Tensor<T> from_json(const std::string &text) {
    Shape dim;
    std::vector<T> data;
    serde::from_json<T>(text, dim, data);
    return Tensor<T>::from_vec(dim, data);
}

}  // namespace agh

#endif  // AUTOGRAPH_HIP_HPP

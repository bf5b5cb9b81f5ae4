// wrq.hpp -- host-side mirror, in C++, of the reference's interface for the quantized
// matrix path, on top of the C ABI in wrq.h.  Header only.
//
// The reference is a Rust crate; a Rust binding of wrq.h would put these same types in
// front of the `extern "C"` calls.  Names, argument order, checks and error text follow
//   src/tensor/shape.rs   Shape                      src/tensor/mod.rs   View, TensorGpu, TensorGpuView, TensorError
//   src/tensor/ops.rs     TensorOp, Activation       src/tensor/matrix.rs Matrix, Float4Quant
//   src/runtime/infer/rnn.rs  RnnInput / RnnIter (token schedule)   src/runtime/v6.rs:568-570  turbo
// so that code written against the reference reads the same here.  What differs by design:
// an op is recorded as a closure over the C ABI call instead of a wgpu pipeline + bind
// groups, and `Context::encode` + `queue.submit` become `Queue::submit`, which replays the
// ops in order on one HIP stream and lets neighbouring decode products that do not depend
// on each other share launches.
#pragma once

#include <cmath>
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <array>
#include <cstdint>
#include <cstring>
#include <functional>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <variant>
#include <vector>

#include "wrq.h"

namespace wrq {

// ---------------------------------------------------------------- errors

// TensorError / TensorErrorKind (src/tensor/mod.rs:87-155); `status` is the wrq_status.
struct TensorError : std::runtime_error {
    int status;
    TensorError(int status, const std::string &what) : std::runtime_error(what), status(status) {}
};

inline void check(int status) {
    if (status != WRQ_OK) throw TensorError(status, wrq_last_error());
}

// ----------------------------------------------------------------- shape

// Shape([usize; 4]), x fastest (src/tensor/shape.rs:96-153).
struct Shape {
    std::array<uint32_t, 4> d{1, 1, 1, 1};
    Shape() = default;
    Shape(uint32_t x, uint32_t y, uint32_t z, uint32_t w) : d{x, y, z, w} {}
    uint32_t operator[](size_t i) const { return d[i]; }
    uint64_t len() const { return (uint64_t)d[0] * d[1] * d[2] * d[3]; }
    bool operator==(const Shape &o) const { return d == o.d; }
    bool operator!=(const Shape &o) const { return !(*this == o); }
    std::string to_string() const {
        return "(" + std::to_string(d[0]) + ", " + std::to_string(d[1]) + ", " + std::to_string(d[2]) + ", " +
               std::to_string(d[3]) + ")";
    }
};

// View { shape, stride, offset } (src/tensor/mod.rs:26-43): stride is the parent's shape.
struct View {
    Shape shape, stride, offset{0, 0, 0, 0};
};

enum class Activation : int { // src/tensor/ops.rs:146-160
    None = WRQ_ACT_NONE,
    SquaredRelu = WRQ_ACT_SQUARED_RELU,
    Tanh = WRQ_ACT_TANH,
    StableExp = WRQ_ACT_STABLE_EXP,
    OppositeExp = WRQ_ACT_OPPOSITE_EXP,
    Softplus = WRQ_ACT_SOFTPLUS,
    Sigmoid = WRQ_ACT_SIGMOID,
    Silu = WRQ_ACT_SILU,
};

struct f16 { // storage only
    uint16_t bits;
};

template <typename T>
struct dtype_of;
template <>
struct dtype_of<f16> {
    static constexpr int value = WRQ_F16;
};
template <>
struct dtype_of<float> {
    static constexpr int value = WRQ_F32;
};

// --------------------------------------------------------------- tensors

// TensorGpu<T, K>: a device buffer and its shape.  Owns its memory when created with
// `init` / `from_data`; `wrap` adopts a pointer the caller keeps alive.
template <typename T>
class TensorGpu {
  public:
    TensorGpu() = default;
    static TensorGpu init(Shape shape) { // Context::tensor_init
        TensorGpu t;
        t.shape_ = shape;
        void *p = nullptr;
        if (hipMalloc(&p, std::max<uint64_t>(shape.len() * sizeof(T), 16)) != hipSuccess)
            throw TensorError(WRQ_ERR_DEVICE, "hipMalloc failed");
        t.data_ = std::shared_ptr<void>(p, [](void *q) { (void)hipFree(q); });
        return t;
    }
    static TensorGpu from_data(Shape shape, const std::vector<T> &host) { // Context::tensor_from_data
        if (host.size() != shape.len())
            throw TensorError(WRQ_ERR_SIZE, "data size not match: " + std::to_string(host.size()) + " vs. " +
                                                std::to_string(shape.len()));
        TensorGpu t = init(shape);
        if (hipMemcpy(t.data(), host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess)
            throw TensorError(WRQ_ERR_DEVICE, "hipMemcpy failed");
        return t;
    }
    static TensorGpu wrap(void *device_ptr, Shape shape) {
        TensorGpu t;
        t.shape_ = shape;
        t.data_ = std::shared_ptr<void>(device_ptr, [](void *) {});
        return t;
    }
    std::vector<T> back() const { // TensorGpu::back: synchronous read-back
        std::vector<T> host(shape_.len());
        if (hipMemcpy(host.data(), data(), host.size() * sizeof(T), hipMemcpyDeviceToHost) != hipSuccess)
            throw TensorError(WRQ_ERR_DEVICE, "hipMemcpy failed");
        return host;
    }
    Shape shape() const { return shape_; }
    void *data() const { return data_.get(); }
    void check_shape(Shape want) const { // TensorShape::check_shape, src/tensor/mod.rs:213-219
        if (shape_ != want)
            throw TensorError(WRQ_ERR_SHAPE, "tensor shape not match: " + shape_.to_string() + " vs. " + want.to_string());
    }
    wrq_tensor c() const { return wrq_tensor{data(), {shape_[0], shape_[1], shape_[2], shape_[3]}}; }

  private:
    Shape shape_;
    std::shared_ptr<void> data_;
};

// TensorGpuView<'a, T> (src/tensor/mod.rs:1119-1142).
template <typename T>
struct TensorGpuView {
    TensorGpu<T> tensor;
    View view;
    TensorGpuView(const TensorGpu<T> &t) : tensor(t), view{t.shape(), t.shape(), Shape{0, 0, 0, 0}} {} // whole tensor
    TensorGpuView(const TensorGpu<T> &t, View v) : tensor(t), view(v) {}
    Shape shape() const { return view.shape; }
    wrq_tensor_view c() const {
        wrq_tensor_view v;
        v.data = tensor.data();
        for (int i = 0; i < 4; i++) {
            v.view.shape[i] = view.shape[i];
            v.view.stride[i] = view.stride[i];
            v.view.offset[i] = view.offset[i];
        }
        if constexpr (std::is_same_v<T, uint8_t>)
            v.dtype = WRQ_F16; // ignored for matrices
        else
            v.dtype = (wrq_dtype)dtype_of<T>::value;
        return v;
    }
};

// `tensor.view(x, y, z, w)` with start..end ranges per axis (src/tensor/mod.rs:1121-1141).
template <typename T>
TensorGpuView<T> view_of(const TensorGpu<T> &t, std::array<std::pair<uint32_t, uint32_t>, 4> ranges) {
    View v;
    v.stride = t.shape();
    for (int i = 0; i < 4; i++) {
        const auto [start, end] = ranges[i];
        if (start > end || end > t.shape()[i])
            throw TensorError(WRQ_ERR_SHAPE, "slice " + std::to_string(start) + ".." + std::to_string(end) +
                                                 " out of range for dimension size " + std::to_string(t.shape()[i]));
        v.offset.d[i] = start;
        v.shape.d[i] = end - start;
    }
    return TensorGpuView<T>(t, v);
}

// ------------------------------------------------------------------- ops

// TensorOp { Atom, List, Sep } (src/tensor/ops.rs:280-288).  An Atom is checked when it is
// built -- the constructors below throw TensorError exactly where the reference returns
// Err -- and runs when a Queue replays it.
class TensorOp {
  public:
    enum class Kind { Atom, List, Sep };
    struct VecInt8 {
        TensorGpu<uint8_t> matrix;
        TensorGpu<f16> minmax;
        wrq_tensor_view input, output;
        std::shared_ptr<void> keep_in, keep_out;
        int act, sparse;
    };
    struct VecNf4 {
        TensorGpu<uint8_t> matrix;
        TensorGpu<float> quant;
        TensorGpu<f16> absmax;
        wrq_tensor_view input, output;
        std::shared_ptr<void> keep_in, keep_out;
        int act, sparse;
    };
    using Payload = std::variant<std::monostate, std::function<int(wrq_stream)>, VecInt8, VecNf4>;

    static constexpr uint32_t NF4_BLOCK_SIZE = WRQ_NF4_BLOCK_SIZE;   // src/tensor/ops.rs:291
    static constexpr uint32_t INT8_BLOCK_SIZE = WRQ_INT8_BLOCK_SIZE; // src/tensor/ops.rs:292

    static TensorOp empty() { return List({}); }
    static TensorOp List(std::vector<TensorOp> ops) {
        TensorOp op;
        op.kind_ = Kind::List;
        op.list_ = std::move(ops);
        return op;
    }
    static TensorOp Sep() {
        TensorOp op;
        op.kind_ = Kind::Sep;
        return op;
    }

    // src/tensor/ops.rs:2393-2486
    static TensorOp quantize_mat_int8(const TensorGpu<f16> &input, const TensorGpu<f16> &minmax,
                                      const TensorGpu<uint8_t> &output) {
        const Shape shape = output.shape();
        const uint32_t minmax_len = (uint32_t)((shape.len() + INT8_BLOCK_SIZE - 1) / INT8_BLOCK_SIZE);
        input.check_shape(shape);
        minmax.check_shape(Shape(minmax_len << 1, 1, 1, 1));
        return atom([=](wrq_stream s) {
            const wrq_tensor i = input.c(), m = minmax.c(), o = output.c();
            return wrq_quantize_mat_int8(s, &i, &m, &o);
        });
    }

    // src/tensor/ops.rs:2488-2589
    static TensorOp quantize_mat_nf4(const TensorGpu<f16> &input, const TensorGpu<float> &quant,
                                     const TensorGpu<f16> &absmax, const TensorGpu<uint8_t> &output) {
        const Shape shape = output.shape();
        const Shape input_shape(shape[0] << 1, shape[1], shape[2], shape[3]);
        const uint32_t absmax_len = (uint32_t)((input_shape.len() + NF4_BLOCK_SIZE - 1) / NF4_BLOCK_SIZE);
        input.check_shape(input_shape);
        absmax.check_shape(Shape(absmax_len, 1, 1, 1));
        return atom([=](wrq_stream s) {
            const wrq_tensor i = input.c(), q = quant.c(), m = absmax.c(), o = output.c();
            return wrq_quantize_mat_nf4(s, &i, &q, &m, &o);
        });
    }

    // src/tensor/ops.rs:791-886
    template <typename F0, typename F1>
    static TensorOp matmul_vec_int8(const TensorGpu<uint8_t> &matrix, const TensorGpu<f16> &minmax,
                                    const TensorGpuView<F0> &input, const TensorGpuView<F1> &output, Activation act,
                                    bool sparse) {
        const Shape os = output.shape(), is = input.shape();
        const uint32_t m = os[0], n = os[1], b = os[2], k = is[0];
        const uint64_t len = matrix.shape().len();
        minmax.check_shape(Shape((uint32_t)(((len << 1) + INT8_BLOCK_SIZE - 1) / INT8_BLOCK_SIZE), 1, 1, 1));
        matrix.check_shape(Shape(k, m, b, 1));
        check_view_shape(input, Shape(k, n, b, 1));
        check_view_shape(output, Shape(m, n, b, 1));
        TensorOp op;
        op.kind_ = Kind::Atom;
        VecInt8 v{matrix, minmax, input.c(), output.c(), hold(input.tensor), hold(output.tensor), (int)act, sparse};
        precheck_vec(v);
        op.payload_ = std::move(v);
        return op;
    }

    // src/tensor/ops.rs:892-991
    template <typename F0, typename F1>
    static TensorOp matmul_vec_nf4(const TensorGpu<uint8_t> &matrix, const TensorGpu<float> &quant,
                                   const TensorGpu<f16> &absmax, const TensorGpuView<F0> &input,
                                   const TensorGpuView<F1> &output, Activation act, bool sparse) {
        const Shape os = output.shape(), is = input.shape();
        const uint32_t m = os[0], n = os[1], b = os[2], k = is[0];
        const uint64_t len = matrix.shape().len() << 1;
        absmax.check_shape(Shape((uint32_t)((len + NF4_BLOCK_SIZE - 1) / NF4_BLOCK_SIZE), 1, 1, 1));
        matrix.check_shape(Shape(k >> 1, m, b, 1));
        check_view_shape(input, Shape(k, n, b, 1));
        check_view_shape(output, Shape(m, n, b, 1));
        TensorOp op;
        op.kind_ = Kind::Atom;
        op.payload_ = VecNf4{matrix,          quant, absmax, input.c(), output.c(), hold(input.tensor), hold(output.tensor),
                             (int)act, sparse};
        return op;
    }

    // src/tensor/ops.rs:1072-1140
    template <typename F0, typename F1>
    static TensorOp matmul_mat_int8(const TensorGpuView<uint8_t> &matrix, const TensorGpu<f16> &minmax,
                                    const TensorGpuView<F0> &input, const TensorGpuView<F1> &output, Activation act) {
        const Shape os = output.shape(), is = input.shape();
        const uint32_t m = os[0], n = os[1], b = os[2], k = is[0];
        const uint64_t len = matrix.shape().len();
        minmax.check_shape(Shape((uint32_t)(((len << 1) + INT8_BLOCK_SIZE - 1) / INT8_BLOCK_SIZE), 1, 1, 1));
        check_view_shape(matrix, Shape(k, m, b, 1));
        check_view_shape(input, Shape(k, n, b, 1));
        check_view_shape(output, Shape(m, n, b, 1));
        return atom([=](wrq_stream s) {
            const wrq_tensor_view a = matrix.c(), i = input.c(), o = output.c();
            const wrq_tensor mm = minmax.c();
            return wrq_matmul_mat_int8(s, &a, &mm, &i, &o, (int)act);
        });
    }

    // src/tensor/ops.rs:1150-1221
    template <typename F0, typename F1>
    static TensorOp matmul_mat_nf4(const TensorGpuView<uint8_t> &matrix, const TensorGpu<float> &quant,
                                   const TensorGpu<f16> &absmax, const TensorGpuView<F0> &input,
                                   const TensorGpuView<F1> &output, Activation act) {
        const Shape os = output.shape(), is = input.shape();
        const uint32_t m = os[0], n = os[1], b = os[2], k = is[0];
        const uint64_t len = matrix.shape().len() << 1;
        absmax.check_shape(Shape((uint32_t)((len + NF4_BLOCK_SIZE - 1) / NF4_BLOCK_SIZE), 1, 1, 1));
        check_view_shape(matrix, Shape(k >> 1, m, b, 1));
        check_view_shape(input, Shape(k, n, b, 1));
        check_view_shape(output, Shape(m, n, b, 1));
        return atom([=](wrq_stream s) {
            const wrq_tensor_view a = matrix.c(), i = input.c(), o = output.c();
            const wrq_tensor q = quant.c(), am = absmax.c();
            return wrq_matmul_mat_nf4(s, &a, &q, &am, &i, &o, (int)act);
        });
    }

    // src/tensor/ops.rs:697-784: matrix f16 [K, R, B]
    template <typename F0, typename F1>
    static TensorOp matmul_vec_fp16(const TensorGpu<f16> &matrix, const TensorGpuView<F0> &input,
                                    const TensorGpuView<F1> &output, Activation act, bool sparse) {
        const Shape os = output.shape(), is = input.shape();
        const uint32_t m = os[0], n = os[1], b = os[2], k = is[0];
        matrix.check_shape(Shape(k, m, b, 1));
        check_view_shape(input, Shape(k, n, b, 1));
        check_view_shape(output, Shape(m, n, b, 1));
        return atom([=](wrq_stream s) {
            const wrq_tensor a = matrix.c();
            const wrq_tensor_view i = input.c(), o = output.c();
            return wrq_matmul_vec_fp16(s, &a, &i, &o, (int)act, sparse);
        });
    }

    // src/tensor/ops.rs:999-1061
    template <typename F0, typename F1>
    static TensorOp matmul_mat_fp16(const TensorGpuView<f16> &matrix, const TensorGpuView<F0> &input,
                                    const TensorGpuView<F1> &output, Activation act) {
        const Shape os = output.shape(), is = input.shape();
        const uint32_t m = os[0], n = os[1], b = os[2], k = is[0];
        check_view_shape(matrix, Shape(k, m, b, 1));
        check_view_shape(input, Shape(k, n, b, 1));
        check_view_shape(output, Shape(m, n, b, 1));
        return atom([=](wrq_stream s) {
            const wrq_tensor_view a = matrix.c(), i = input.c(), o = output.c();
            return wrq_matmul_mat_fp16(s, &a, &i, &o, (int)act);
        });
    }

    // ---- the ops between the matrix products; shapes are checked by the library as the reference's
    // constructors check them, a failed check throws TensorError

    // src/tensor/ops.rs:300-347
    template <typename F>
    static TensorOp softmax(const TensorGpu<F> &x) {
        return checked([=](wrq_stream s) { const wrq_tensor t = x.c(); return wrq_softmax(s, &t, (wrq_dtype)dtype_of<F>::value); });
    }
    // src/tensor/ops.rs:407-458, :460-509
    template <typename F>
    static TensorOp layer_norm(const TensorGpu<f16> &w, const TensorGpu<f16> &b, const TensorGpu<F> &x, float eps) {
        x.check_shape(Shape(x.shape()[0], x.shape()[1], x.shape()[2], 1));
        w.check_shape(Shape(x.shape()[0], 1, 1, 1));
        b.check_shape(Shape(x.shape()[0], 1, 1, 1));
        return checked([=](wrq_stream s) { const wrq_tensor tw = w.c(), tb = b.c(), tx = x.c(); return wrq_layer_norm(s, &tw, &tb, &tx, (wrq_dtype)dtype_of<F>::value, eps); });
    }
    template <typename F>
    static TensorOp group_norm(const TensorGpu<f16> &w, const TensorGpu<f16> &b, const TensorGpu<F> &x, float eps) {
        w.check_shape(Shape(x.shape()[0], x.shape()[1], 1, 1));
        b.check_shape(Shape(x.shape()[0], x.shape()[1], 1, 1));
        return checked([=](wrq_stream s) { const wrq_tensor tw = w.c(), tb = b.c(), tx = x.c(); return wrq_group_norm(s, &tw, &tb, &tx, (wrq_dtype)dtype_of<F>::value, eps); });
    }
    // src/tensor/ops.rs:1227-1391
    template <typename F0, typename F1>
    static TensorOp add_activate(const TensorGpuView<F0> &input, const TensorGpuView<F1> &output, Activation x, Activation y, Activation out) {
        return checked([=](wrq_stream s) { const wrq_tensor_view i = input.c(), o = output.c(); return wrq_add_activate(s, &i, &o, (int)x, (int)y, (int)out); });
    }
    template <typename F0, typename F1>
    static TensorOp mul_activate(const TensorGpuView<F0> &input, const TensorGpuView<F1> &output, Activation x, Activation y, Activation out) {
        return checked([=](wrq_stream s) { const wrq_tensor_view i = input.c(), o = output.c(); return wrq_mul_activate(s, &i, &o, (int)x, (int)y, (int)out); });
    }
    template <typename F0, typename F1>
    static TensorOp add(const TensorGpuView<F0> &input, const TensorGpuView<F1> &output) {
        return add_activate(input, output, Activation::None, Activation::None, Activation::None);
    }
    template <typename F0, typename F1>
    static TensorOp mul(const TensorGpuView<F0> &input, const TensorGpuView<F1> &output) {
        return mul_activate(input, output, Activation::None, Activation::None, Activation::None);
    }
    // src/tensor/ops.rs:350-405
    template <typename F>
    static TensorOp embed(const TensorGpu<uint32_t> &tokens, const TensorGpu<f16> &input, const TensorGpu<F> &output) {
        return checked([=](wrq_stream s) { const wrq_tensor t = tokens.c(), i = input.c(), o = output.c(); return wrq_embed(s, &t, &i, &o, (wrq_dtype)dtype_of<F>::value); });
    }
    // src/tensor/ops.rs:2015-2068, :2121-2169, :1973-2013, :2352-2391, :2284-2350
    template <typename F0, typename F1>
    static TensorOp blit(const TensorGpuView<F0> &input, const TensorGpuView<F1> &output) {
        return checked([=](wrq_stream s) { const wrq_tensor_view i = input.c(), o = output.c(); return wrq_blit(s, &i, &o); });
    }
    template <typename F0, typename F1>
    static TensorOp transpose(const TensorGpuView<F0> &input, const TensorGpuView<F1> &output) {
        return checked([=](wrq_stream s) { const wrq_tensor_view i = input.c(), o = output.c(); return wrq_transpose(s, &i, &o); });
    }
    template <typename F>
    static TensorOp activate(const TensorGpuView<F> &x, Activation act) {
        return checked([=](wrq_stream s) { const wrq_tensor_view v = x.c(); return wrq_activate(s, &v, (int)act); });
    }
    template <typename F>
    static TensorOp affine(const TensorGpu<F> &x, float scale, float bias) {
        return checked([=](wrq_stream s) { const wrq_tensor t = x.c(); return wrq_affine(s, &t, (wrq_dtype)dtype_of<F>::value, scale, bias); });
    }
    template <typename F0, typename F1, typename F2>
    static TensorOp lerp(const TensorGpuView<F0> &input, const TensorGpuView<F1> &output, const TensorGpuView<F2> &factor, bool reversed) {
        return checked([=](wrq_stream s) { const wrq_tensor_view i = input.c(), o = output.c(), f = factor.c(); return wrq_lerp(s, &i, &o, &f, reversed ? 1 : 0); });
    }
    // src/tensor/ops.rs:1393-1462, :1860-1915, :1601-1677
    template <typename FT, typename F0, typename F1>
    static TensorOp token_shift(const TensorGpu<uint32_t> &cursors, const TensorGpuView<FT> &time_mix, const TensorGpuView<float> &state,
                                const TensorGpu<F0> &input, const TensorGpu<F1> &output, bool reversed) {
        return checked([=](wrq_stream s) {
            const wrq_tensor c = cursors.c(), i = input.c(), o = output.c();
            const wrq_tensor_view t = time_mix.c(), st = state.c();
            return wrq_token_shift(s, &c, &t, &st, &i, (wrq_dtype)dtype_of<F0>::value, &o, (wrq_dtype)dtype_of<F1>::value, reversed ? 1 : 0);
        });
    }
    template <typename F>
    static TensorOp channel_mix(const TensorGpu<uint32_t> &cursors, const TensorGpuView<float> &state, const TensorGpu<F> &r, const TensorGpu<F> &v,
                                const TensorGpu<F> &x) {
        return checked([=](wrq_stream s) {
            const wrq_tensor c = cursors.c(), tr = r.c(), tv = v.c(), tx = x.c();
            const wrq_tensor_view st = state.c();
            return wrq_channel_mix(s, &c, &st, &tr, &tv, &tx, (wrq_dtype)dtype_of<F>::value);
        });
    }
    template <typename F>
    static TensorOp time_mix_v4(const TensorGpu<uint32_t> &cursors, const TensorGpu<float> &time_decay, const TensorGpu<float> &time_first,
                                const TensorGpuView<float> &state, const TensorGpu<F> &k, const TensorGpu<F> &v, const TensorGpu<F> &r, const TensorGpu<F> &x) {
        return checked([=](wrq_stream s) {
            const wrq_tensor c = cursors.c(), td = time_decay.c(), tf = time_first.c(), tk = k.c(), tv = v.c(), tr = r.c(), tx = x.c();
            const wrq_tensor_view st = state.c();
            return wrq_time_mix_v4(s, &c, &td, &tf, &st, &tk, &tv, &tr, &tx, (wrq_dtype)dtype_of<F>::value);
        });
    }

    template <typename F>
    static TensorOp time_mix_v5(const TensorGpu<uint32_t> &cursors, const TensorGpu<float> &time_decay, const TensorGpu<float> &time_first,
                                const TensorGpuView<float> &state, const TensorGpu<F> &k, const TensorGpu<F> &v, const TensorGpu<F> &r, const TensorGpu<F> &x) {
        return checked([=](wrq_stream s) {
            const wrq_tensor c = cursors.c(), td = time_decay.c(), tf = time_first.c(), tk = k.c(), tv = v.c(), tr = r.c(), tx = x.c();
            const wrq_tensor_view st = state.c();
            return wrq_time_mix_v5(s, &c, &td, &tf, &st, &tk, &tv, &tr, &tx, (wrq_dtype)dtype_of<F>::value);
        });
    }

    template <typename F>
    static TensorOp time_mix_v6(const TensorGpu<uint32_t> &cursors, const TensorGpu<float> &time_decay, const TensorGpu<float> &time_first,
                                const TensorGpuView<float> &state, const TensorGpu<F> &k, const TensorGpu<F> &v, const TensorGpu<F> &r, const TensorGpu<F> &x) {
        return checked([=](wrq_stream s) {
            const wrq_tensor c = cursors.c(), td = time_decay.c(), tf = time_first.c(), tk = k.c(), tv = v.c(), tr = r.c(), tx = x.c();
            const wrq_tensor_view st = state.c();
            return wrq_time_mix_v6(s, &c, &td, &tf, &st, &tk, &tv, &tr, &tx, (wrq_dtype)dtype_of<F>::value);
        });
    }

    // the rest of the op set: src/tensor/ops.rs:511-564, :566-640, :2070-2119, :2171-2224, :2226-2282
    template <typename F>
    static TensorOp recenter(const TensorGpu<F> &x) {
        return checked([=](wrq_stream s) { const wrq_tensor tx = x.c(); return wrq_recenter(s, &tx, (wrq_dtype)dtype_of<F>::value); });
    }
    template <typename F>
    static TensorOp rms_norm(const TensorGpu<f16> &w, const TensorGpu<f16> &b, const TensorGpu<F> &x, float eps) {
        return checked([=](wrq_stream s) { const wrq_tensor tw = w.c(), tb = b.c(), tx = x.c(); return wrq_rms_norm(s, &tw, &tb, &tx, (wrq_dtype)dtype_of<F>::value, eps); });
    }
    template <typename F0, typename F1>
    static TensorOp broadcast(const TensorGpuView<F0> &input, const TensorGpuView<F1> &output) {
        return checked([=](wrq_stream s) { const wrq_tensor_view i = input.c(), o = output.c(); return wrq_broadcast(s, &i, &o); });
    }
    template <typename F0, typename F1>
    static TensorOp blend(const TensorGpu<float> &factor, const TensorGpu<F0> &input, const TensorGpu<F1> &output) {
        return checked([=](wrq_stream s) {
            const wrq_tensor f = factor.c(), i = input.c(), o = output.c();
            return wrq_blend(s, &f, &i, (wrq_dtype)dtype_of<F0>::value, &o, (wrq_dtype)dtype_of<F1>::value);
        });
    }
    static TensorOp blend_lora(const TensorGpu<float> &factor, const TensorGpuView<f16> &xa, const TensorGpuView<f16> &xb, const TensorGpuView<f16> &output) {
        return checked([=](wrq_stream s) {
            const wrq_tensor f = factor.c();
            const wrq_tensor_view a = xa.c(), b = xb.c(), o = output.c();
            return wrq_blend_lora(s, &f, &a, &b, &o);
        });
    }
    // the ops an RWKV-v7 layer adds: src/tensor/ops.rs:642-700, :1800-1858, :1679-1741, :1743-1798, :1917-1970
    template <typename F>
    static TensorOp l2_norm(const TensorGpu<F> &x, float eps) {
        return checked([=](wrq_stream s) { const wrq_tensor tx = x.c(); return wrq_l2_norm(s, &tx, (wrq_dtype)dtype_of<F>::value, eps); });
    }
    template <typename F0, typename F1>
    static TensorOp control_k_v7(const TensorGpu<f16> &p, const TensorGpuView<F0> &a, const TensorGpuView<F1> &k) {
        return checked([=](wrq_stream s) {
            const wrq_tensor tp = p.c();
            const wrq_tensor_view ta = a.c(), tk = k.c();
            return wrq_control_k_v7(s, &tp, &ta, &tk);
        });
    }
    template <typename F>
    static TensorOp time_mix_v7(const TensorGpu<uint32_t> &cursors, const TensorGpuView<float> &state, const TensorGpu<F> &r, const TensorGpu<F> &w,
                                const TensorGpu<F> &n, const TensorGpu<F> &x) {
        return checked([=](wrq_stream s) {
            const wrq_tensor c = cursors.c(), tr = r.c(), tw = w.c(), tn = n.c(), tx = x.c();
            const wrq_tensor_view st = state.c();
            return wrq_time_mix_v7(s, &c, &st, &tr, &tw, &tn, &tx, (wrq_dtype)dtype_of<F>::value);
        });
    }
    template <typename F>
    static TensorOp time_first_v7(const TensorGpu<f16> &u, const TensorGpu<F> &r, const TensorGpu<F> &n, const TensorGpu<F> &x) {
        return checked([=](wrq_stream s) {
            const wrq_tensor tu = u.c(), tr = r.c(), tn = n.c(), tx = x.c();
            return wrq_time_first_v7(s, &tu, &tr, &tn, &tx, (wrq_dtype)dtype_of<F>::value);
        });
    }
    template <typename F>
    static TensorOp channel_mix_v7(const TensorGpu<uint32_t> &cursors, const TensorGpuView<float> &state, const TensorGpu<F> &v, const TensorGpu<F> &x) {
        return checked([=](wrq_stream s) {
            const wrq_tensor c = cursors.c(), tv = v.c(), tx = x.c();
            const wrq_tensor_view st = state.c();
            return wrq_channel_mix_v7(s, &c, &st, &tv, &tx, (wrq_dtype)dtype_of<F>::value);
        });
    }

    Kind kind() const { return kind_; }
    const std::vector<TensorOp> &list() const { return list_; }
    const Payload &payload() const { return payload_; }

  private:
    template <typename T>
    static std::shared_ptr<void> hold(const TensorGpu<T> &t) {
        return std::make_shared<TensorGpu<T>>(t);
    }
    template <typename T>
    static void check_view_shape(const TensorGpuView<T> &v, Shape want) {
        if (v.shape() != want)
            throw TensorError(WRQ_ERR_SHAPE, "tensor shape not match: " + v.shape().to_string() + " vs. " + want.to_string());
    }
    static void precheck_vec(const VecInt8 &) {}
    // an op whose shapes the library checks when it runs (the Queue turns a failed status into TensorError)
    static TensorOp checked(std::function<int(wrq_stream)> f) { return atom(std::move(f)); }
    static TensorOp atom(std::function<int(wrq_stream)> f) {
        TensorOp op;
        op.kind_ = Kind::Atom;
        op.payload_ = std::move(f);
        return op;
    }
    Kind kind_ = Kind::List;
    std::vector<TensorOp> list_;
    Payload payload_;
};

// `context.queue.submit(context.encode(&op))` (src/tensor/ops.rs:78-144): the ops of a list
// run in order on one stream.  Neighbouring decode products of one kind are handed to the
// grouped entry point when none of them reads or writes another's output (checked on the
// device address ranges of their views' parents); a `Sep` always ends a group.
class Queue {
  public:
    explicit Queue(hipStream_t stream = nullptr) : stream_(stream) {}
    void submit(const TensorOp &op) {
        std::vector<const TensorOp *> flat;
        flatten(op, flat);
        size_t i = 0;
        while (i < flat.size()) {
            const TensorOp &o = *flat[i];
            if (o.kind() == TensorOp::Kind::Sep) {
                i++;
                continue;
            }
            if (auto f = std::get_if<std::function<int(wrq_stream)>>(&o.payload())) {
                check((*f)(stream_));
                i++;
            } else if (std::holds_alternative<TensorOp::VecInt8>(o.payload())) {
                i = run_group<TensorOp::VecInt8>(flat, i);
            } else if (std::holds_alternative<TensorOp::VecNf4>(o.payload())) {
                i = run_group<TensorOp::VecNf4>(flat, i);
            } else {
                i++;
            }
        }
    }
    void sync() {
        if (hipStreamSynchronize(stream_) != hipSuccess) throw TensorError(WRQ_ERR_DEVICE, "hipStreamSynchronize failed");
    }

  private:
    static void flatten(const TensorOp &op, std::vector<const TensorOp *> &out) {
        if (op.kind() == TensorOp::Kind::List)
            for (const auto &o : op.list()) flatten(o, out);
        else
            out.push_back(&op);
    }
    static bool overlaps(const wrq_tensor_view &a, size_t sa, const wrq_tensor_view &b, size_t sb) {
        auto bytes = [](const wrq_tensor_view &v, size_t s) {
            return (uint64_t)v.view.stride[0] * v.view.stride[1] * v.view.stride[2] * v.view.stride[3] * s;
        };
        const uintptr_t a0 = (uintptr_t)a.data, a1 = a0 + bytes(a, sa), b0 = (uintptr_t)b.data, b1 = b0 + bytes(b, sb);
        return a0 < b1 && b0 < a1;
    }
    static size_t esize(const wrq_tensor_view &v) { return v.dtype == WRQ_F16 ? 2 : 4; }
    template <typename V>
    size_t run_group(const std::vector<const TensorOp *> &flat, size_t i) {
        std::vector<const V *> group;
        while (i < flat.size() && group.size() < WRQ_MAX_GROUP) {
            const V *v = std::get_if<V>(&flat[i]->payload());
            if (!v) break;
            bool independent = true;
            for (const V *g : group)
                independent = independent && !overlaps(v->input, esize(v->input), g->output, esize(g->output)) &&
                              !overlaps(v->output, esize(v->output), g->output, esize(g->output)) &&
                              !overlaps(v->output, esize(v->output), g->input, esize(g->input));
            if (!independent) break;
            group.push_back(v);
            i++;
        }
        if constexpr (std::is_same_v<V, TensorOp::VecInt8>) {
            std::vector<wrq_tensor> m(group.size()), s(group.size());
            std::vector<wrq_vec_int8_op> ops(group.size());
            for (size_t k = 0; k < group.size(); k++) {
                m[k] = group[k]->matrix.c();
                s[k] = group[k]->minmax.c();
                ops[k] = wrq_vec_int8_op{&m[k], &s[k], &group[k]->input, &group[k]->output, group[k]->act, group[k]->sparse};
            }
            check(wrq_matmul_vec_int8_group(stream_, ops.data(), (int)ops.size()));
        } else {
            std::vector<wrq_tensor> m(group.size()), q(group.size()), s(group.size());
            std::vector<wrq_vec_nf4_op> ops(group.size());
            for (size_t k = 0; k < group.size(); k++) {
                m[k] = group[k]->matrix.c();
                q[k] = group[k]->quant.c();
                s[k] = group[k]->absmax.c();
                ops[k] = wrq_vec_nf4_op{&m[k], &q[k], &s[k], &group[k]->input, &group[k]->output, group[k]->act, group[k]->sparse};
            }
            check(wrq_matmul_vec_nf4_group(stream_, ops.data(), (int)ops.size()));
        }
        return i;
    }
    hipStream_t stream_;
};

// ---------------------------------------------------------------- matrix

// Float4Quant::new (src/tensor/matrix.rs:46-70): the normal-float table.
inline std::vector<float> float4_quant() {
    return {-1.0f,
            -0.6961928009986877f,
            -0.5250730514526367f,
            -0.39491748809814453f,
            -0.28444138169288635f,
            -0.18477343022823334f,
            -0.09105003625154495f,
            0.0f,
            0.07958029955625534f,
            0.16093020141124725f,
            0.24611230194568634f,
            0.33791524171829224f,
            0.44070982933044434f,
            0.5626170039176941f,
            0.7229568362236023f,
            1.0f};
}

// Float4Quant::new_student / quantile_student (src/tensor/matrix.rs:29-44): 16 quantiles of
// Student's t with `nu` degrees of freedom at the probabilities delta + i (0.5 - delta) / 7
// (i < 7) and 0.5 + i (0.5 - delta) / 8 (i < 9), delta = (1/32 + 1/30) / 2, divided by the
// largest.  The reference takes the quantile from the `statrs` crate (0.18, not vendored);
// here the t CDF is the regularised incomplete beta function (Lentz continued fraction) and
// is inverted by bisection in double precision, which agrees with statrs far inside f32.
namespace detail {
inline double betacf(double a, double b, double x) {
    const double tiny = 1e-300;
    double qab = a + b, qap = a + 1.0, qam = a - 1.0, c = 1.0, d = 1.0 - qab * x / qap;
    if (std::fabs(d) < tiny) d = tiny;
    d = 1.0 / d;
    double h = d;
    for (int m = 1; m <= 400; m++) {
        const int m2 = 2 * m;
        double aa = m * (b - m) * x / ((qam + m2) * (a + m2));
        d = 1.0 + aa * d;
        if (std::fabs(d) < tiny) d = tiny;
        c = 1.0 + aa / c;
        if (std::fabs(c) < tiny) c = tiny;
        d = 1.0 / d;
        h *= d * c;
        aa = -(a + m) * (qab + m) * x / ((a + m2) * (qap + m2));
        d = 1.0 + aa * d;
        if (std::fabs(d) < tiny) d = tiny;
        c = 1.0 + aa / c;
        if (std::fabs(c) < tiny) c = tiny;
        d = 1.0 / d;
        const double del = d * c;
        h *= del;
        if (std::fabs(del - 1.0) < 1e-16) break;
    }
    return h;
}
inline double betai(double a, double b, double x) { // regularised incomplete beta I_x(a, b)
    if (x <= 0.0) return 0.0;
    if (x >= 1.0) return 1.0;
    const double bt = std::exp(std::lgamma(a + b) - std::lgamma(a) - std::lgamma(b) + a * std::log(x) + b * std::log(1.0 - x));
    return x < (a + 1.0) / (a + b + 2.0) ? bt * betacf(a, b, x) / a : 1.0 - bt * betacf(b, a, 1.0 - x) / b;
}
inline double student_cdf(double t, double nu) {
    const double tail = 0.5 * betai(0.5 * nu, 0.5, nu / (nu + t * t));
    return t > 0 ? 1.0 - tail : tail;
}
inline double student_quantile(double p, double nu) {
    if (p == 0.5) return 0.0; // the median, exactly (table entry 7)
    double lo = -1e6, hi = 1e6;
    for (int i = 0; i < 200; i++) {
        const double mid = 0.5 * (lo + hi);
        (student_cdf(mid, nu) < p ? lo : hi) = mid;
    }
    return 0.5 * (lo + hi);
}
} // namespace detail

inline std::vector<float> float4_quant_student(double nu) {
    const double delta = (1.0 / 32.0 + 1.0 / 30.0) / 2.0;
    std::vector<double> p;
    for (int i = 0; i < 7; i++) p.push_back(delta + (0.5 - delta) / 7.0 * i);
    for (int i = 0; i < 9; i++) p.push_back(0.5 + (1.0 - delta - 0.5) / 8.0 * i);
    std::vector<double> q;
    double most = -1e300;
    for (double v : p) {
        q.push_back(detail::student_quantile(v, nu));
        most = std::max(most, q.back());
    }
    std::vector<float> out;
    for (double v : q) out.push_back((float)(v / most));
    return out;
}

// Matrix { Fp16(w), Int8 { w, m }, Fp4 { q, w, m } } (src/tensor/matrix.rs:29-44, :80-94).
struct Matrix {
    enum class Kind { Int8, Fp4, Fp16 } kind;
    TensorGpu<uint8_t> w;
    TensorGpu<f16> m;
    TensorGpu<float> q; // Fp4 only
    TensorGpu<f16> h;   // Fp16 only: the weights as they are

    static Matrix fp16(const TensorGpu<f16> &matrix) { return Matrix{Kind::Fp16, {}, {}, {}, matrix}; }

    // src/tensor/matrix.rs:162-178
    static Matrix quant_u8(const TensorGpu<f16> &matrix, Queue &queue) {
        const Shape shape = matrix.shape();
        auto w = TensorGpu<uint8_t>::init(shape);
        auto m = TensorGpu<f16>::init(
            Shape((uint32_t)(((shape.len() << 1) + TensorOp::INT8_BLOCK_SIZE - 1) / TensorOp::INT8_BLOCK_SIZE), 1, 1, 1));
        queue.submit(TensorOp::quantize_mat_int8(matrix, m, w));
        return Matrix{Kind::Int8, w, m, {}, {}};
    }
    // src/tensor/matrix.rs:180-200; `table` other than the default is quant_sf4's job (:202-222)
    static Matrix quant_nf4(const TensorGpu<f16> &matrix, Queue &queue, std::vector<float> table = float4_quant()) {
        const Shape shape = matrix.shape();
        const Shape matrix_shape(shape[0] / 2, shape[1], shape[2], shape[3]);
        const Shape absmax_shape((uint32_t)((shape.len() + TensorOp::NF4_BLOCK_SIZE - 1) / TensorOp::NF4_BLOCK_SIZE), 1, 1, 1);
        auto q = TensorGpu<float>::from_data(Shape(16, 1, 1, 1), table);
        auto w = TensorGpu<uint8_t>::init(matrix_shape);
        auto m = TensorGpu<f16>::init(absmax_shape);
        queue.submit(TensorOp::quantize_mat_nf4(matrix, q, m, w));
        return Matrix{Kind::Fp4, w, m, q, {}};
    }

    // src/tensor/matrix.rs:202-222
    static Matrix quant_sf4(const TensorGpu<f16> &matrix, Queue &queue, double nu) {
        return quant_nf4(matrix, queue, float4_quant_student(nu));
    }

    template <typename F0, typename F1>
    TensorOp matmul_vec_op(const TensorGpuView<F0> &input, const TensorGpuView<F1> &output, Activation act,
                           bool sparse = false) const {
        if (kind == Kind::Fp16) return TensorOp::matmul_vec_fp16(h, input, output, act, sparse);
        return kind == Kind::Int8 ? TensorOp::matmul_vec_int8(w, m, input, output, act, sparse)
                                  : TensorOp::matmul_vec_nf4(w, q, m, input, output, act, sparse);
    }
    template <typename F0, typename F1>
    TensorOp matmul_vec_op_sparse(const TensorGpuView<F0> &input, const TensorGpuView<F1> &output, Activation act) const {
        return matmul_vec_op(input, output, act, true);
    }
    template <typename F0, typename F1>
    TensorOp matmul_mat_op(const TensorGpuView<F0> &input, const TensorGpuView<F1> &output, Activation act) const {
        if (kind == Kind::Fp16) return TensorOp::matmul_mat_fp16(TensorGpuView<f16>(h), input, output, act);
        return kind == Kind::Int8 ? TensorOp::matmul_mat_int8(TensorGpuView<uint8_t>(w), m, input, output, act)
                                  : TensorOp::matmul_mat_nf4(TensorGpuView<uint8_t>(w), q, m, input, output, act);
    }
    // src/tensor/matrix.rs:136-160
    template <typename F0, typename F1>
    TensorOp matmul_op(const TensorGpuView<F0> &input, const TensorGpuView<F1> &output, Activation act, bool turbo) const {
        return turbo ? matmul_mat_op(input, output, act) : matmul_vec_op(input, output, act);
    }
    template <typename F0, typename F1>
    TensorOp matmul_op_sparse(const TensorGpuView<F0> &input, const TensorGpuView<F1> &output, Activation act,
                              bool turbo) const {
        return turbo ? matmul_mat_op(input, output, act) : matmul_vec_op_sparse(input, output, act);
    }
};

// -------------------------------------------------------- token schedule

// The builders pick the chunk kernels iff the run has a multiple of 32 tokens
// (src/runtime/v6.rs:568-570).
inline bool turbo(size_t num_token) { return num_token % 32 == 0; }

constexpr size_t MIN_TOKEN_CHUNK_SIZE = 32; // src/runtime/infer/rnn.rs:10

enum class RnnOption { Last, Full };

struct RnnInfoBatch { // src/runtime/infer/rnn.rs:25-29
    size_t len = 0;
    std::optional<RnnOption> option;
    bool operator==(const RnnInfoBatch &o) const { return len == o.len && option == o.option; }
};

struct RnnRedirect { // src/runtime/infer/rnn.rs:88-96
    std::vector<size_t> headers;
    std::vector<std::pair<size_t, size_t>> inputs, outputs;
};

struct RnnInfo { // src/runtime/infer/rnn.rs:22-81
    std::vector<RnnInfoBatch> batches;
    size_t num_token() const {
        size_t n = 0;
        for (const auto &b : batches) n += b.len;
        return n;
    }
    RnnRedirect redirect() const {
        RnnRedirect r;
        r.inputs.assign(batches.size(), {0, 0});
        r.outputs.assign(batches.size(), {0, 0});
        size_t p_in = 0, p_out = 0;
        for (size_t i = 0; i < batches.size(); i++) {
            const size_t len = batches[i].len;
            r.inputs[i] = {p_in, p_in + len};
            if (!batches[i].option) {
                r.outputs[i] = {p_out, p_out};
            } else if (*batches[i].option == RnnOption::Last) {
                if (len == 0) {
                    r.outputs[i] = {p_out, p_out};
                } else {
                    r.outputs[i] = {p_out, p_out + 1};
                    r.headers.push_back(p_in + len - 1);
                    p_out += 1;
                }
            } else {
                r.outputs[i] = {p_out, p_out + len};
                for (size_t t = p_in; t < p_in + len; t++) r.headers.push_back(t);
                p_out += len;
            }
            p_in += len;
        }
        return r;
    }
};

// RnnInput + RnnIter (src/runtime/infer/rnn.rs:194-335): how many tokens of each slot go
// into the next run; this fixes T, and with it the kernel, of every product of the run.
class RnnInput {
  public:
    struct Batch {
        size_t tokens; // tokens still to read
        RnnOption option;
    };
    RnnInput(std::vector<Batch> batches, size_t token_chunk_size) : batches_(std::move(batches)) {
        token_chunk_size = std::max(token_chunk_size, MIN_TOKEN_CHUNK_SIZE);
        token_chunk_size_ = (token_chunk_size + MIN_TOKEN_CHUNK_SIZE - 1) / MIN_TOKEN_CHUNK_SIZE * MIN_TOKEN_CHUNK_SIZE;
    }
    size_t token_chunk_size() const { return token_chunk_size_; }

    class Iter {
      public:
        RnnInfo next() { // Iterator::next, rnn.rs:280-335
            std::vector<size_t> remains(state_.size());
            for (size_t i = 0; i < state_.size(); i++) remains[i] = state_[i].gen ? 1 : state_[i].read;
            size_t num_token = 0;
            for (size_t r : remains) num_token += r;
            num_token = std::min(num_token, chunk_);
            if (num_token > MIN_TOKEN_CHUNK_SIZE) num_token -= num_token % MIN_TOKEN_CHUNK_SIZE;

            std::vector<RnnInfoBatch> info(state_.size());
            while (num_token > 0) {
                size_t mid = 0;
                bool any = false;
                for (size_t r : remains)
                    if (r > 0 && (!any || r < mid)) mid = r, any = true;
                if (!any) break;
                for (size_t i = 0; i < remains.size(); i++) {
                    if (remains[i] == 0) continue;
                    const size_t take = std::min(mid, num_token);
                    num_token -= take;
                    info[i].len += take;
                    remains[i] -= take;
                }
            }
            for (size_t i = 0; i < state_.size(); i++) {
                if (info[i].len > 0) {
                    state_[i].gen = remains[i] == 0;
                    state_[i].read = remains[i];
                }
                if (state_[i].option == RnnOption::Full)
                    info[i].option = RnnOption::Full;
                else if (remains[i] == 0)
                    info[i].option = RnnOption::Last;
                else
                    info[i].option = std::nullopt;
            }
            return RnnInfo{info};
        }

      private:
        friend class RnnInput;
        struct State {
            bool gen;
            size_t read;
            RnnOption option;
        };
        std::vector<State> state_;
        size_t chunk_;
    };

    Iter iter() const {
        Iter it;
        it.chunk_ = token_chunk_size_;
        for (const auto &b : batches_) it.state_.push_back({false, b.tokens, b.option});
        return it;
    }
    void step() { // JobInput::step, rnn.rs:233-240
        const RnnInfo info = iter().next();
        for (size_t i = 0; i < batches_.size(); i++) batches_[i].tokens -= info.batches[i].len;
    }

  private:
    std::vector<Batch> batches_;
    size_t token_chunk_size_;
};

} // namespace wrq

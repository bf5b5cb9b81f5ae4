// Row-wise and element-wise ops that sit between the matrix products of a layer:
//   softmax                 src/tensor/ops.rs:300-347,   src/shaders/softmax.wgsl
//   layer_norm, group_norm  src/tensor/ops.rs:407-509,   src/shaders/layer_norm.wgsl
//   add / mul (+activations) src/tensor/ops.rs:1227-1391, src/shaders/binary.wgsl
//
// All are bound by memory latency, not bandwidth, at the sizes of this path (a row is 2 - 16 KiB, a
// run has 1 - 256 rows): one workgroup per row keeps the row in registers between the statistics
// and the write-back where it fits (one read, one write per element), reductions go through DPP and
// one LDS exchange, every access is a whole 8- or 16-byte vector of 4 elements as in the shaders.
// The statistics are two-pass (mean, then the sum of squared deviations) in f32: the shaders merge
// per-lane Welford states; both agree with the exact value far inside the reference's 1e-3 test bar.
#include "layer_device.h"

namespace wrq {

namespace {

constexpr int kRowThreads = 256;
constexpr int kRowCache = 8; // vectors of 4 elements a thread keeps: rows up to 8192 elements stay in registers

// One workgroup per row of `n` elements (n % 4 == 0).  MODE 0: softmax; 1: layer norm (w, b of the
// row's length); 2: group norm (w, b indexed by head * n, the row index modulo `heads`).
template <typename XT, int MODE, int THREADS>
__global__ __launch_bounds__(THREADS) void row_kernel(XT *x, const uint16_t *w, const uint16_t *b, uint32_t n, uint32_t heads, float eps) {
    __shared__ float red[THREADS / 64];
    XT *row = x + (uint64_t)blockIdx.x * n;
    const uint32_t nv = n / 4;
    float4 cache[kRowCache];
    const bool cached = nv <= (uint32_t)(THREADS * kRowCache);
    // a cached row asks for its weights together with the row: they are needed only after both reductions, and
    // fetched then they would add a memory round trip to a kernel that is little more than round trips
    uint2 wq[MODE == 0 ? 1 : kRowCache], bq[MODE == 0 ? 1 : kRowCache];
    const uint16_t *wr = MODE == 2 ? w + (uint64_t)(blockIdx.x % heads) * n : w;
    const uint16_t *br = MODE == 2 ? b + (uint64_t)(blockIdx.x % heads) * n : b;
    if constexpr (MODE != 0) {
        if (cached) {
#pragma unroll
            for (int c = 0; c < kRowCache; c++) {
                const uint32_t i = threadIdx.x + c * THREADS;
                if (i < nv) wq[c] = *reinterpret_cast<const uint2 *>(wr + 4 * i), bq[c] = *reinterpret_cast<const uint2 *>(br + 4 * i);
            }
        }
    }
    // pass 1: the row into registers (or a first reading), maximum / sum
    float part = MODE == 0 ? -1.0e30f : 0.0f;
    if (cached) {
#pragma unroll
        for (int c = 0; c < kRowCache; c++) {
            const uint32_t i = threadIdx.x + c * THREADS;
            if (i < nv) {
                cache[c] = load_vec4(row + 4 * i);
                if (MODE == 0) part = fmaxf(part, fmaxf(fmaxf(cache[c].x, cache[c].y), fmaxf(cache[c].z, cache[c].w)));
                else part += (cache[c].x + cache[c].y) + (cache[c].z + cache[c].w);
            }
        }
    } else {
        for (uint32_t i = threadIdx.x; i < nv; i += THREADS) {
            const float4 v = load_vec4(row + 4 * i);
            if (MODE == 0) part = fmaxf(part, fmaxf(fmaxf(v.x, v.y), fmaxf(v.z, v.w)));
            else part += (v.x + v.y) + (v.z + v.w);
        }
    }
    const float first = block_reduce<MODE == 0, THREADS>(part, red); // maximum, or the sum
    const float centre = MODE == 0 ? first : first / (float)n;
    // pass 2: sum of exp(x - max), or of squared deviations
    float acc = 0.0f;
    auto term = [&](float v) { return MODE == 0 ? expf(v - centre) : (v - centre) * (v - centre); };
    if (cached) {
#pragma unroll
        for (int c = 0; c < kRowCache; c++)
            if (threadIdx.x + c * THREADS < nv) acc += (term(cache[c].x) + term(cache[c].y)) + (term(cache[c].z) + term(cache[c].w));
    } else {
        for (uint32_t i = threadIdx.x; i < nv; i += THREADS) {
            const float4 v = load_vec4(row + 4 * i);
            acc += (term(v.x) + term(v.y)) + (term(v.z) + term(v.w));
        }
    }
    const float total = block_reduce<false, THREADS>(acc, red);
    const float scale = MODE == 0 ? 1.0f / total : rsqrtf(total / (float)n + eps);
    auto unpack = [](uint2 v) {
        return make_float4(h2f((uint16_t)(v.x & 0xffffu)), h2f((uint16_t)(v.x >> 16)), h2f((uint16_t)(v.y & 0xffffu)), h2f((uint16_t)(v.y >> 16)));
    };
    auto finish = [&](uint32_t i, float4 v, int c) { // c: the vector's place in the cache, or -1
        float4 o;
        if (MODE == 0) {
            o = make_float4(expf(v.x - centre) * scale, expf(v.y - centre) * scale, expf(v.z - centre) * scale, expf(v.w - centre) * scale);
        } else {
            const float4 wv = c >= 0 ? unpack(wq[MODE == 0 ? 0 : c]) : load_vec4(wr + 4 * i), bv = c >= 0 ? unpack(bq[MODE == 0 ? 0 : c]) : load_vec4(br + 4 * i);
            o = make_float4(fmaf((v.x - centre) * scale, wv.x, bv.x), fmaf((v.y - centre) * scale, wv.y, bv.y),
                            fmaf((v.z - centre) * scale, wv.z, bv.z), fmaf((v.w - centre) * scale, wv.w, bv.w));
        }
        store_vec4(row + 4 * i, o);
    };
    if (cached) {
#pragma unroll
        for (int c = 0; c < kRowCache; c++) {
            const uint32_t i = threadIdx.x + c * THREADS;
            if (i < nv) finish(i, cache[c], c);
        }
    } else {
        for (uint32_t i = threadIdx.x; i < nv; i += THREADS) finish(i, load_vec4(row + 4 * i), -1);
    }
}

// output = ACT_OUT(ACT_X(input) op ACT_Y(output)); input broadcast over tokens / batches of extent 1
template <typename IT, typename OT, bool MUL>
__global__ __launch_bounds__(256) void binary_kernel(const IT *input, OT *output, ViewArgs src, ViewArgs dst, int act_x, int act_y, int act_out) {
    const uint32_t index = blockIdx.x * 256 + threadIdx.x, token = blockIdx.y, batch = blockIdx.z;
    if (index >= dst.shape[0] / 4) return;
    const float4 x = load_vec4(input + 4 * view_index(src, src.shape[2] == 1 ? 0u : batch, src.shape[1] == 1 ? 0u : token, index));
    OT *out = output + 4 * view_index(dst, batch, token, index);
    const float4 y = load_vec4(out);
    auto f = [&](float a, float c) {
        const float p = act_apply(act_x, a), q = act_apply(act_y, c);
        return act_apply(act_out, MUL ? p * q : p + q);
    };
    store_vec4(out, make_float4(f(x.x, y.x), f(x.y, y.y), f(x.z, y.z), f(x.w, y.w)));
}

// output view <- input view, element types converted (blit); MODE 1 swaps token and batch on the
// way out (transpose); src/shaders/blit.wgsl:35-53, reshape.wgsl:58-77
template <typename IT, typename OT, int MODE>
__global__ __launch_bounds__(256) void copy_kernel(const IT *input, OT *output, ViewArgs src, ViewArgs dst) {
    const uint32_t index = blockIdx.x * 256 + threadIdx.x, token = blockIdx.y, batch = blockIdx.z;
    if (index >= src.shape[0] / 4) return;
    const float4 x = load_vec4(input + 4 * view_index(src, batch, token, index));
    store_vec4(output + 4 * (MODE == 1 ? view_index(dst, token, batch, index) : view_index(dst, batch, token, index)), x);
}

// x <- act(x) over a view (src/shaders/activation.wgsl:30-45), or scale * x + bias (affine.wgsl:16-30)
template <typename XT, bool AFFINE>
__global__ __launch_bounds__(256) void unary_kernel(XT *x, ViewArgs v, int act, float scale, float bias) {
    const uint32_t index = blockIdx.x * 256 + threadIdx.x, token = blockIdx.y, batch = blockIdx.z;
    if (index >= v.shape[0] / 4) return;
    XT *p = x + 4 * view_index(v, batch, token, index);
    const float4 a = load_vec4(p);
    if (AFFINE) store_vec4(p, make_float4(scale * a.x + bias, scale * a.y + bias, scale * a.z + bias, scale * a.w + bias));
    else store_vec4(p, make_float4(act_apply(act, a.x), act_apply(act, a.y), act_apply(act, a.z), act_apply(act, a.w)));
}

// y <- mix(x, y, f) = x (1 - f) + y f, or mix(y, x, f) when reversed; f broadcast over extents of 1
// (src/shaders/lerp.wgsl:72-93)
template <typename FT, typename IT, typename OT>
__global__ __launch_bounds__(256) void lerp_kernel(const FT *f, const IT *x, OT *y, ViewArgs vf, ViewArgs vx, ViewArgs vy, int reversed) {
    const uint32_t index = blockIdx.x * 256 + threadIdx.x, token = blockIdx.y, batch = blockIdx.z;
    if (index >= vy.shape[0] / 4) return;
    const float4 ff = load_vec4(f + 4 * view_index(vf, vf.shape[2] == 1 ? 0u : batch, vf.shape[1] == 1 ? 0u : token, index));
    const float4 a = load_vec4(x + 4 * view_index(vx, batch, token, index));
    OT *out = y + 4 * view_index(vy, batch, token, index);
    const float4 c = load_vec4(out);
    auto mix = [&](float p, float q, float t) { return reversed ? q * (1.0f - t) + p * t : p * (1.0f - t) + q * t; };
    store_vec4(out, make_float4(mix(a.x, c.x, ff.x), mix(a.y, c.y, ff.y), mix(a.z, c.z, ff.z), mix(a.w, c.w, ff.w)));
}

// output[batch][token] <- row tokens[batch][token] of the f16 table (src/shaders/embed.wgsl:22-38); an
// id beyond the table reads its last row (the host cannot check ids that live in device memory)
template <typename OT>
__global__ __launch_bounds__(256) void embed_kernel(const uint32_t *tokens, const uint16_t *table, OT *output, uint32_t C, uint32_t T, uint32_t vocab) {
    const uint32_t index = blockIdx.x * 256 + threadIdx.x, token = blockIdx.y, batch = blockIdx.z;
    if (index >= C / 4) return;
    const uint32_t id = min(tokens[batch * T + token], vocab - 1);
    store_vec4(output + ((uint64_t)(batch * T + token) * C + 4 * index), load_vec4(table + ((uint64_t)id * C + 4 * index)));
}

int check_row_tensor(const wrq_tensor *x, int dtype, const char *what) {
    if (!x || !x->data) return fail(WRQ_ERR_NULL, "%s: null tensor", what);
    if (dtype != WRQ_F16 && dtype != WRQ_F32) return fail(WRQ_ERR_TYPE, "%s: unsupported element type %d", what, dtype);
    if (x->shape[3] != 1) return fail(WRQ_ERR_SHAPE, "%s: data shape [%u, %u, %u, %u] not match", what, x->shape[0], x->shape[1], x->shape[2], x->shape[3]);
    if (x->shape[0] % 4) return fail(WRQ_ERR_ALIGNMENT, "%s: row length %u not a multiple of 4", what, x->shape[0]);
    if ((uintptr_t)x->data % 16) return fail(WRQ_ERR_ALIGNMENT, "%s: device pointers must be 16-byte aligned", what);
    return WRQ_OK;
}

template <int MODE>
int launch_rows(hipStream_t stream, void *x, int dtype, const void *w, const void *b, uint32_t n, uint64_t rows, uint32_t heads, float eps, const char *what) {
    if (rows == 0 || n == 0) return WRQ_OK;
    if (rows > 0x7fffffffull) return fail(WRQ_ERR_SIZE, "%s: data size not match", what);
    const uint16_t *wp = static_cast<const uint16_t *>(w), *bp = static_cast<const uint16_t *>(b);
    // short rows (a head of a group norm) take one wave, no LDS exchange
    if (n > 16384) {
        // a vocabulary-sized row (softmax over the logits): 1024 threads
        if (dtype == WRQ_F16) hipLaunchKernelGGL((row_kernel<uint16_t, MODE, 1024>), dim3((uint32_t)rows), dim3(1024), 0, stream, static_cast<uint16_t *>(x), wp, bp, n, heads, eps);
        else hipLaunchKernelGGL((row_kernel<float, MODE, 1024>), dim3((uint32_t)rows), dim3(1024), 0, stream, static_cast<float *>(x), wp, bp, n, heads, eps);
    } else if (n <= 1024) {
        if (dtype == WRQ_F16) hipLaunchKernelGGL((row_kernel<uint16_t, MODE, 64>), dim3((uint32_t)rows), dim3(64), 0, stream, static_cast<uint16_t *>(x), wp, bp, n, heads, eps);
        else hipLaunchKernelGGL((row_kernel<float, MODE, 64>), dim3((uint32_t)rows), dim3(64), 0, stream, static_cast<float *>(x), wp, bp, n, heads, eps);
    } else {
        if (dtype == WRQ_F16) hipLaunchKernelGGL((row_kernel<uint16_t, MODE, kRowThreads>), dim3((uint32_t)rows), dim3(kRowThreads), 0, stream, static_cast<uint16_t *>(x), wp, bp, n, heads, eps);
        else hipLaunchKernelGGL((row_kernel<float, MODE, kRowThreads>), dim3((uint32_t)rows), dim3(kRowThreads), 0, stream, static_cast<float *>(x), wp, bp, n, heads, eps);
    }
    return check_launch(what);
}

template <bool MUL>
int binary(hipStream_t stream, const wrq_tensor_view *input, const wrq_tensor_view *output, int act_x, int act_y, int act_out) {
    const char *what = MUL ? "mul" : "add";
    int s = check_layer_view(input, what);
    if (s != WRQ_OK) return s;
    s = check_layer_view(output, what);
    if (s != WRQ_OK) return s;
    for (int a : {act_x, act_y, act_out})
        if (a < 0 || a > WRQ_ACT_SILU) return fail(WRQ_ERR_UNSUPPORTED, "%s: unknown activation %d", what, a);
    const uint32_t *o = output->view.shape, *i = input->view.shape;
    // the shapes check_shape_any accepts (src/tensor/ops.rs:1243-1249)
    const bool ok = o[3] == 1 && i[0] == o[0] &&
                    ((i[1] == o[1] && i[2] == o[2] && i[3] == 1) || (i[1] == o[1] && i[2] == 1 && i[3] == o[2]) || (i[1] == 1 && i[2] == o[2] && i[3] == 1) ||
                     (i[1] == 1 && i[2] == 1 && i[3] == 1));
    if (!ok) return fail(WRQ_ERR_SHAPE, "%s: data shape [%u, %u, %u, %u] not match [%u, %u, %u, %u]", what, i[0], i[1], i[2], i[3], o[0], o[1], o[2], o[3]);
    if (o[0] == 0 || o[1] == 0 || o[2] == 0) return WRQ_OK;
    if (o[1] > 65535u || o[2] > 65535u) return fail(WRQ_ERR_SIZE, "%s: data size not match", what);
    const dim3 grid((o[0] / 4 + 255) / 256, o[1], o[2]);
    const ViewArgs src = view_args(input->view), dst = view_args(output->view);
    const bool i16 = input->dtype == WRQ_F16, o16 = output->dtype == WRQ_F16;
    if (i16 && o16) hipLaunchKernelGGL((binary_kernel<uint16_t, uint16_t, MUL>), grid, dim3(256), 0, stream, static_cast<const uint16_t *>(input->data), static_cast<uint16_t *>(output->data), src, dst, act_x, act_y, act_out);
    else if (i16) hipLaunchKernelGGL((binary_kernel<uint16_t, float, MUL>), grid, dim3(256), 0, stream, static_cast<const uint16_t *>(input->data), static_cast<float *>(output->data), src, dst, act_x, act_y, act_out);
    else if (o16) hipLaunchKernelGGL((binary_kernel<float, uint16_t, MUL>), grid, dim3(256), 0, stream, static_cast<const float *>(input->data), static_cast<uint16_t *>(output->data), src, dst, act_x, act_y, act_out);
    else hipLaunchKernelGGL((binary_kernel<float, float, MUL>), grid, dim3(256), 0, stream, static_cast<const float *>(input->data), static_cast<float *>(output->data), src, dst, act_x, act_y, act_out);
    return check_launch(what);
}

template <int MODE>
int copy(hipStream_t stream, const wrq_tensor_view *input, const wrq_tensor_view *output) {
    const char *what = MODE == 1 ? "transpose" : "blit";
    int s = check_layer_view(input, what);
    if (s != WRQ_OK) return s;
    s = check_layer_view(output, what);
    if (s != WRQ_OK) return s;
    const uint32_t *i = input->view.shape, *o = output->view.shape;
    const bool ok = MODE == 1 ? (o[0] == i[0] && o[1] == i[2] && o[2] == i[1] && o[3] == 1 && i[3] == 1) : (o[0] == i[0] && o[1] == i[1] && o[2] == i[2] && o[3] == i[3]);
    if (!ok) return fail(WRQ_ERR_SHAPE, "%s: data shape [%u, %u, %u, %u] not match [%u, %u, %u, %u]", what, i[0], i[1], i[2], i[3], o[0], o[1], o[2], o[3]);
    if (i[0] == 0 || i[1] == 0 || i[2] == 0) return WRQ_OK;
    if (i[1] > 65535u || i[2] > 65535u) return fail(WRQ_ERR_SIZE, "%s: data size not match", what);
    const dim3 grid((i[0] / 4 + 255) / 256, i[1], i[2]);
    const ViewArgs src = view_args(input->view), dst = view_args(output->view);
    const bool i16 = input->dtype == WRQ_F16, o16 = output->dtype == WRQ_F16;
    if (i16 && o16) hipLaunchKernelGGL((copy_kernel<uint16_t, uint16_t, MODE>), grid, dim3(256), 0, stream, static_cast<const uint16_t *>(input->data), static_cast<uint16_t *>(output->data), src, dst);
    else if (i16) hipLaunchKernelGGL((copy_kernel<uint16_t, float, MODE>), grid, dim3(256), 0, stream, static_cast<const uint16_t *>(input->data), static_cast<float *>(output->data), src, dst);
    else if (o16) hipLaunchKernelGGL((copy_kernel<float, uint16_t, MODE>), grid, dim3(256), 0, stream, static_cast<const float *>(input->data), static_cast<uint16_t *>(output->data), src, dst);
    else hipLaunchKernelGGL((copy_kernel<float, float, MODE>), grid, dim3(256), 0, stream, static_cast<const float *>(input->data), static_cast<float *>(output->data), src, dst);
    return check_launch(what);
}

template <bool AFFINE>
int unary(hipStream_t stream, const wrq_tensor_view *x, int act, float scale, float bias) {
    const char *what = AFFINE ? "affine" : "activate";
    const int s = check_layer_view(x, what);
    if (s != WRQ_OK) return s;
    if (!AFFINE && (act < 0 || act > WRQ_ACT_SILU)) return fail(WRQ_ERR_UNSUPPORTED, "%s: unknown activation %d", what, act);
    const uint32_t *v = x->view.shape;
    if (v[3] != 1) return fail(WRQ_ERR_SHAPE, "%s: data shape [%u, %u, %u, %u] not match", what, v[0], v[1], v[2], v[3]);
    if (v[0] == 0 || v[1] == 0 || v[2] == 0) return WRQ_OK;
    if (v[1] > 65535u || v[2] > 65535u) return fail(WRQ_ERR_SIZE, "%s: data size not match", what);
    const dim3 grid((v[0] / 4 + 255) / 256, v[1], v[2]);
    const ViewArgs va = view_args(x->view);
    if (x->dtype == WRQ_F16) hipLaunchKernelGGL((unary_kernel<uint16_t, AFFINE>), grid, dim3(256), 0, stream, static_cast<uint16_t *>(x->data), va, act, scale, bias);
    else hipLaunchKernelGGL((unary_kernel<float, AFFINE>), grid, dim3(256), 0, stream, static_cast<float *>(x->data), va, act, scale, bias);
    return check_launch(what);
}

template <typename FT, typename IT>
int lerp_out(hipStream_t stream, const wrq_tensor_view *f, const wrq_tensor_view *x, const wrq_tensor_view *y, dim3 grid, int reversed) {
    const ViewArgs vf = view_args(f->view), vx = view_args(x->view), vy = view_args(y->view);
    if (y->dtype == WRQ_F16) hipLaunchKernelGGL((lerp_kernel<FT, IT, uint16_t>), grid, dim3(256), 0, stream, static_cast<const FT *>(f->data), static_cast<const IT *>(x->data), static_cast<uint16_t *>(y->data), vf, vx, vy, reversed);
    else hipLaunchKernelGGL((lerp_kernel<FT, IT, float>), grid, dim3(256), 0, stream, static_cast<const FT *>(f->data), static_cast<const IT *>(x->data), static_cast<float *>(y->data), vf, vx, vy, reversed);
    return check_launch("lerp");
}

} // namespace

} // namespace wrq

using namespace wrq;

extern "C" {

int wrq_softmax(wrq_stream stream, const wrq_tensor *x, wrq_dtype dtype) {
    const int s = check_row_tensor(x, dtype, "softmax");
    if (s != WRQ_OK) return s;
    return launch_rows<0>(static_cast<hipStream_t>(stream), x->data, dtype, nullptr, nullptr, x->shape[0], (uint64_t)x->shape[1] * x->shape[2], 1, 0.0f, "softmax");
}

int wrq_layer_norm(wrq_stream stream, const wrq_tensor *w, const wrq_tensor *b, const wrq_tensor *x, wrq_dtype dtype, float eps) {
    const int s = check_row_tensor(x, dtype, "layer_norm");
    if (s != WRQ_OK) return s;
    if (!w || !b || !w->data || !b->data) return fail(WRQ_ERR_NULL, "layer_norm: null tensor");
    for (const wrq_tensor *t : {w, b})
        if (t->shape[0] != x->shape[0] || t->shape[1] != 1 || t->shape[2] != 1 || t->shape[3] != 1)
            return fail(WRQ_ERR_SHAPE, "layer_norm: data shape [%u, %u, %u, %u] not match [%u, 1, 1, 1]", t->shape[0], t->shape[1], t->shape[2], t->shape[3], x->shape[0]);
    if ((uintptr_t)w->data % 8 || (uintptr_t)b->data % 8) return fail(WRQ_ERR_ALIGNMENT, "layer_norm: device pointers must be 8-byte aligned");
    return launch_rows<1>(static_cast<hipStream_t>(stream), x->data, dtype, w->data, b->data, x->shape[0], (uint64_t)x->shape[1] * x->shape[2], 1, eps, "layer_norm");
}

int wrq_group_norm(wrq_stream stream, const wrq_tensor *w, const wrq_tensor *b, const wrq_tensor *x, wrq_dtype dtype, float eps) {
    const int s = check_row_tensor(x, dtype, "group_norm");
    if (s != WRQ_OK) return s;
    if (!w || !b || !w->data || !b->data) return fail(WRQ_ERR_NULL, "group_norm: null tensor");
    for (const wrq_tensor *t : {w, b})
        if (t->shape[0] != x->shape[0] || t->shape[1] != x->shape[1] || t->shape[2] != 1 || t->shape[3] != 1)
            return fail(WRQ_ERR_SHAPE, "group_norm: data shape [%u, %u, %u, %u] not match [%u, %u, 1, 1]", t->shape[0], t->shape[1], t->shape[2], t->shape[3], x->shape[0], x->shape[1]);
    if ((uintptr_t)w->data % 8 || (uintptr_t)b->data % 8) return fail(WRQ_ERR_ALIGNMENT, "group_norm: device pointers must be 8-byte aligned");
    return launch_rows<2>(static_cast<hipStream_t>(stream), x->data, dtype, w->data, b->data, x->shape[0], (uint64_t)x->shape[1] * x->shape[2], x->shape[1], eps, "group_norm");
}

int wrq_add_activate(wrq_stream stream, const wrq_tensor_view *input, const wrq_tensor_view *output, int act_x, int act_y, int act_out) {
    return binary<false>(static_cast<hipStream_t>(stream), input, output, act_x, act_y, act_out);
}

int wrq_mul_activate(wrq_stream stream, const wrq_tensor_view *input, const wrq_tensor_view *output, int act_x, int act_y, int act_out) {
    return binary<true>(static_cast<hipStream_t>(stream), input, output, act_x, act_y, act_out);
}

int wrq_blit(wrq_stream stream, const wrq_tensor_view *input, const wrq_tensor_view *output) {
    return copy<0>(static_cast<hipStream_t>(stream), input, output);
}

int wrq_transpose(wrq_stream stream, const wrq_tensor_view *input, const wrq_tensor_view *output) {
    return copy<1>(static_cast<hipStream_t>(stream), input, output);
}

int wrq_activate(wrq_stream stream, const wrq_tensor_view *x, int act) {
    return unary<false>(static_cast<hipStream_t>(stream), x, act, 1.0f, 0.0f);
}

int wrq_affine(wrq_stream stream, const wrq_tensor *x, wrq_dtype dtype, float scale, float bias) {
    if (!x) return fail(WRQ_ERR_NULL, "affine: null tensor");
    wrq_tensor_view v;
    v.data = x->data;
    v.dtype = dtype;
    for (int i = 0; i < 4; i++) v.view.shape[i] = v.view.stride[i] = x->shape[i], v.view.offset[i] = 0;
    return unary<true>(static_cast<hipStream_t>(stream), &v, 0, scale, bias);
}

int wrq_lerp(wrq_stream stream, const wrq_tensor_view *input, const wrq_tensor_view *output, const wrq_tensor_view *factor, int reversed) {
    int s = check_layer_view(input, "lerp");
    if (s == WRQ_OK) s = check_layer_view(output, "lerp");
    if (s == WRQ_OK) s = check_layer_view(factor, "lerp");
    if (s != WRQ_OK) return s;
    const uint32_t *o = output->view.shape, *i = input->view.shape, *f = factor->view.shape;
    // src/tensor/ops.rs:2298-2307
    const bool fok = f[0] == o[0] && f[3] == 1 && (f[1] == o[1] || f[1] == 1) && (f[2] == o[2] || f[2] == 1);
    if (o[3] != 1 || !fok || i[0] != o[0] || i[1] != o[1] || i[2] != o[2] || i[3] != 1)
        return fail(WRQ_ERR_SHAPE, "lerp: data shape [%u, %u, %u, %u] / [%u, %u, %u, %u] not match [%u, %u, %u, %u]", i[0], i[1], i[2], i[3], f[0], f[1], f[2], f[3], o[0], o[1], o[2], o[3]);
    if (o[0] == 0 || o[1] == 0 || o[2] == 0) return WRQ_OK;
    if (o[1] > 65535u || o[2] > 65535u) return fail(WRQ_ERR_SIZE, "lerp: data size not match");
    const dim3 grid((o[0] / 4 + 255) / 256, o[1], o[2]);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool f16 = factor->dtype == WRQ_F16, i16 = input->dtype == WRQ_F16;
    if (f16 && i16) return lerp_out<uint16_t, uint16_t>(st, factor, input, output, grid, reversed);
    if (f16) return lerp_out<uint16_t, float>(st, factor, input, output, grid, reversed);
    if (i16) return lerp_out<float, uint16_t>(st, factor, input, output, grid, reversed);
    return lerp_out<float, float>(st, factor, input, output, grid, reversed);
}

int wrq_embed(wrq_stream stream, const wrq_tensor *tokens, const wrq_tensor *input, const wrq_tensor *output, wrq_dtype dtype) {
    const int s = check_row_tensor(output, dtype, "embed");
    if (s != WRQ_OK) return s;
    if (!tokens || !input || !tokens->data || !input->data) return fail(WRQ_ERR_NULL, "embed: null tensor");
    const uint32_t *o = output->shape, *t = tokens->shape, *i = input->shape;
    // src/tensor/ops.rs:357-364
    if (t[0] != o[1] || t[1] != o[2] || t[2] != 1 || t[3] != 1 || i[0] != o[0] || i[2] != 1 || i[3] != 1 || i[1] == 0)
        return fail(WRQ_ERR_SHAPE, "embed: data shape not match [%u, %u, %u, %u]", o[0], o[1], o[2], o[3]);
    if ((uintptr_t)input->data % 8) return fail(WRQ_ERR_ALIGNMENT, "embed: device pointers must be 8-byte aligned");
    if (o[0] == 0 || o[1] == 0 || o[2] == 0) return WRQ_OK;
    if (o[1] > 65535u || o[2] > 65535u) return fail(WRQ_ERR_SIZE, "embed: data size not match");
    const dim3 grid((o[0] / 4 + 255) / 256, o[1], o[2]);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    if (dtype == WRQ_F16)
        hipLaunchKernelGGL((embed_kernel<uint16_t>), grid, dim3(256), 0, hs, static_cast<const uint32_t *>(tokens->data), static_cast<const uint16_t *>(input->data), static_cast<uint16_t *>(output->data), o[0], o[1], i[1]);
    else
        hipLaunchKernelGGL((embed_kernel<float>), grid, dim3(256), 0, hs, static_cast<const uint32_t *>(tokens->data), static_cast<const uint16_t *>(input->data), static_cast<float *>(output->data), o[0], o[1], i[1]);
    return check_launch("embed");
}

} // extern "C"


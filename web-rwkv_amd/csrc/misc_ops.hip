// The remaining ops of the reference's op set: two row normalisations, and what its loader uses to
// lay out states and to blend low-rank adapters into matrices at load time.
//   recenter     src/tensor/ops.rs:511-564,   src/shaders/normalize.wgsl:46-80
//   rms_norm     src/tensor/ops.rs:566-640,   src/shaders/normalize.wgsl:82-116
//   broadcast    src/tensor/ops.rs:2070-2119, src/shaders/reshape.wgsl:35-56
//   blend        src/tensor/ops.rs:2171-2224, src/shaders/blend.wgsl
//   blend_lora   src/tensor/ops.rs:2226-2282, src/shaders/blend_lora.wgsl
// None of them is on a per-token path except rms_norm; they are written for simplicity: a wave per row,
// a thread per 4-element vector, a thread per output element of the rank-r product.
#include "layer_device.h"

namespace wrq {

namespace {

// RMS: x <- x / sqrt(mean(x^2) + eps) * w + b;  otherwise x <- x - mean(x)
template <typename XT, bool RMS>
__global__ __launch_bounds__(64) void center_kernel(XT *x, const uint16_t *w, const uint16_t *b, uint32_t C, float eps) {
    XT *row = x + (uint64_t)blockIdx.x * C;
    float sum = 0.0f;
    for (uint32_t i = 4 * threadIdx.x; i < C; i += 256) {
        const float4 v = load_vec4(row + i);
        sum += RMS ? v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w : (v.x + v.y) + (v.z + v.w);
    }
    sum = wave_sum(sum) / (float)C;
    const float norm = RMS ? 1.0f / sqrtf(sum + eps) : 0.0f;
    for (uint32_t i = 4 * threadIdx.x; i < C; i += 256) {
        const float4 v = load_vec4(row + i);
        if constexpr (RMS) {
            const float4 ww = load_vec4(w + i), bb = load_vec4(b + i);
            store_vec4(row + i, make_float4(fmaf(v.x * norm, ww.x, bb.x), fmaf(v.y * norm, ww.y, bb.y), fmaf(v.z * norm, ww.z, bb.z), fmaf(v.w * norm, ww.w, bb.w)));
        } else {
            store_vec4(row + i, make_float4(v.x - sum, v.y - sum, v.z - sum, v.w - sum));
        }
    }
}

// output[batch][token] <- input[batch % its batches][token % its tokens]
template <typename IT, typename OT>
__global__ __launch_bounds__(256) void broadcast_kernel(const IT *input, OT *output, ViewArgs vi, ViewArgs vo) {
    const uint32_t index = blockIdx.x * 256 + threadIdx.x, token = blockIdx.y, batch = blockIdx.z;
    if (index >= vo.shape[0] / 4) return;
    store_vec4(output + view_elem(vo, batch, token, 4 * index), load_vec4(input + view_elem(vi, batch % vi.shape[2], token % vi.shape[1], 4 * index)));
}

// output <- factor[0] input + factor[1] output
template <typename IT, typename OT>
__global__ __launch_bounds__(256) void blend_kernel(const float *factor, const IT *input, OT *output, uint64_t vectors) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= vectors) return;
    const float fx = factor[0], fy = factor[1];
    const float4 x = load_vec4(input + 4 * i), y = load_vec4(output + 4 * i);
    store_vec4(output + 4 * i, make_float4(fx * x.x + fy * y.x, fx * x.y + fy * y.y, fx * x.z + fy * y.z, fx * x.w + fy * y.w));
}

// output[b][n][m] <- factor[0] sum_k xa[b][m][k] xb[b][n][k] + factor[1] output[b][n][m]; a thread per 4 adjacent m
__global__ __launch_bounds__(256) void blend_lora_kernel(const float *factor, const uint16_t *xa, const uint16_t *xb, uint16_t *output, ViewArgs va, ViewArgs vb,
                                                         ViewArgs vo, uint32_t K) {
    const uint32_t m4 = blockIdx.x * 64 + (threadIdx.x & 63), n = blockIdx.y * 4 + (threadIdx.x >> 6), batch = blockIdx.z;
    if (4 * m4 >= vo.shape[0] || n >= vo.shape[1]) return;
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    const uint16_t *bp = xb + view_elem(vb, batch, n, 0);
    for (uint32_t k = 0; k < K; k += 4) {
        const float4 bv = load_vec4(bp + k);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float4 av = load_vec4(xa + view_elem(va, batch, 4 * m4 + e, k));
            acc[e] += av.x * bv.x + av.y * bv.y + av.z * bv.z + av.w * bv.w;
        }
    }
    const float fx = factor[0], fy = factor[1];
    uint16_t *op = output + view_elem(vo, batch, n, 4 * m4);
    const float4 u = load_vec4(op);
    store_vec4(op, make_float4(fx * acc[0] + fy * u.x, fx * acc[1] + fy * u.y, fx * acc[2] + fy * u.z, fx * acc[3] + fy * u.w));
}

int row_op(const char *name, bool rms, wrq_stream stream, const wrq_tensor *w, const wrq_tensor *b, const wrq_tensor *x, wrq_dtype dtype, float eps) {
    int s = check_layer_tensor(x, name);
    if (rms && s == WRQ_OK) s = check_layer_tensor(w, name);
    if (rms && s == WRQ_OK) s = check_layer_tensor(b, name);
    if (s != WRQ_OK) return s;
    if (dtype != WRQ_F16 && dtype != WRQ_F32) return fail(WRQ_ERR_TYPE, "%s: unsupported element type %d", name, (int)dtype);
    const uint32_t *sh = x->shape;
    const uint32_t vec[4] = {sh[0], 1, 1, 1};
    if (sh[3] != 1 || (rms && (!same_shape(w->shape, vec) || !same_shape(b->shape, vec))))
        return fail(WRQ_ERR_SHAPE, "%s: data shape not match [%u, %u, %u, %u]", name, sh[0], sh[1], sh[2], sh[3]);
    if (sh[0] % 4) return fail(WRQ_ERR_ALIGNMENT, "%s: row length %u not a multiple of 4", name, sh[0]);
    const uint64_t rows = (uint64_t)sh[1] * sh[2];
    if (sh[0] == 0 || rows == 0) return WRQ_OK;
    if (rows > 0x7fffffffull) return fail(WRQ_ERR_SIZE, "%s: data size not match", name);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    const uint16_t *wp = rms ? static_cast<const uint16_t *>(w->data) : nullptr, *bp = rms ? static_cast<const uint16_t *>(b->data) : nullptr;
    const dim3 grid((uint32_t)rows);
    if (dtype == WRQ_F16) {
        if (rms) hipLaunchKernelGGL((center_kernel<uint16_t, true>), grid, dim3(64), 0, hs, static_cast<uint16_t *>(x->data), wp, bp, sh[0], eps);
        else hipLaunchKernelGGL((center_kernel<uint16_t, false>), grid, dim3(64), 0, hs, static_cast<uint16_t *>(x->data), wp, bp, sh[0], eps);
    } else {
        if (rms) hipLaunchKernelGGL((center_kernel<float, true>), grid, dim3(64), 0, hs, static_cast<float *>(x->data), wp, bp, sh[0], eps);
        else hipLaunchKernelGGL((center_kernel<float, false>), grid, dim3(64), 0, hs, static_cast<float *>(x->data), wp, bp, sh[0], eps);
    }
    return check_launch(name);
}

} // namespace

} // namespace wrq

using namespace wrq;

extern "C" {

int wrq_recenter(wrq_stream stream, const wrq_tensor *x, wrq_dtype dtype) { return row_op("recenter", false, stream, nullptr, nullptr, x, dtype, 0.0f); }

int wrq_rms_norm(wrq_stream stream, const wrq_tensor *w, const wrq_tensor *b, const wrq_tensor *x, wrq_dtype dtype, float eps) {
    return row_op("rms_norm", true, stream, w, b, x, dtype, eps);
}

int wrq_broadcast(wrq_stream stream, const wrq_tensor_view *input, const wrq_tensor_view *output) {
    int s = check_layer_view(input, "broadcast");
    if (s == WRQ_OK) s = check_layer_view(output, "broadcast");
    if (s != WRQ_OK) return s;
    const uint32_t *o = output->view.shape, *i = input->view.shape;
    // src/tensor/ops.rs:2082
    if (i[0] != o[0] || i[3] != 1 || o[3] != 1) return fail(WRQ_ERR_SHAPE, "broadcast: data shape not match [%u, %u, %u, %u]", o[0], o[1], o[2], o[3]);
    if (o[0] == 0 || o[1] == 0 || o[2] == 0) return WRQ_OK;
    if (i[1] == 0 || i[2] == 0) return fail(WRQ_ERR_SHAPE, "broadcast: empty input");
    if (o[1] > 65535u || o[2] > 65535u) return fail(WRQ_ERR_SIZE, "broadcast: data size not match");
    const dim3 grid((o[0] / 4 + 255) / 256, o[1], o[2]);
    const ViewArgs vi = view_args(input->view), vo = view_args(output->view);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    const bool i16 = input->dtype == WRQ_F16, o16 = output->dtype == WRQ_F16;
    if (i16 && o16) hipLaunchKernelGGL((broadcast_kernel<uint16_t, uint16_t>), grid, dim3(256), 0, hs, static_cast<const uint16_t *>(input->data), static_cast<uint16_t *>(output->data), vi, vo);
    else if (i16) hipLaunchKernelGGL((broadcast_kernel<uint16_t, float>), grid, dim3(256), 0, hs, static_cast<const uint16_t *>(input->data), static_cast<float *>(output->data), vi, vo);
    else if (o16) hipLaunchKernelGGL((broadcast_kernel<float, uint16_t>), grid, dim3(256), 0, hs, static_cast<const float *>(input->data), static_cast<uint16_t *>(output->data), vi, vo);
    else hipLaunchKernelGGL((broadcast_kernel<float, float>), grid, dim3(256), 0, hs, static_cast<const float *>(input->data), static_cast<float *>(output->data), vi, vo);
    return check_launch("broadcast");
}

int wrq_blend(wrq_stream stream, const wrq_tensor *factor, const wrq_tensor *input, wrq_dtype input_dtype, const wrq_tensor *output, wrq_dtype output_dtype) {
    int s = check_layer_tensor(factor, "blend");
    if (s == WRQ_OK) s = check_layer_tensor(input, "blend");
    if (s == WRQ_OK) s = check_layer_tensor(output, "blend");
    if (s != WRQ_OK) return s;
    for (int d : {(int)input_dtype, (int)output_dtype})
        if (d != WRQ_F16 && d != WRQ_F32) return fail(WRQ_ERR_TYPE, "blend: unsupported element type %d", d);
    const uint32_t *sh = output->shape;
    // src/tensor/ops.rs:2178-2179
    const uint32_t fs[4] = {4, 1, 1, 1};
    if (!same_shape(input->shape, sh) || !same_shape(factor->shape, fs))
        return fail(WRQ_ERR_SHAPE, "blend: data shape not match [%u, %u, %u, %u]", sh[0], sh[1], sh[2], sh[3]);
    if (sh[0] % 4) return fail(WRQ_ERR_ALIGNMENT, "blend: row length %u not a multiple of 4", sh[0]);
    const uint64_t vectors = (uint64_t)sh[0] / 4 * sh[1] * sh[2] * sh[3];
    if (vectors == 0) return WRQ_OK;
    if ((vectors + 255) / 256 > 0x7fffffffull) return fail(WRQ_ERR_SIZE, "blend: data size not match");
    const dim3 grid((uint32_t)((vectors + 255) / 256));
    hipStream_t hs = static_cast<hipStream_t>(stream);
    const float *f = static_cast<const float *>(factor->data);
    const bool i16 = input_dtype == WRQ_F16, o16 = output_dtype == WRQ_F16;
    if (i16 && o16) hipLaunchKernelGGL((blend_kernel<uint16_t, uint16_t>), grid, dim3(256), 0, hs, f, static_cast<const uint16_t *>(input->data), static_cast<uint16_t *>(output->data), vectors);
    else if (i16) hipLaunchKernelGGL((blend_kernel<uint16_t, float>), grid, dim3(256), 0, hs, f, static_cast<const uint16_t *>(input->data), static_cast<float *>(output->data), vectors);
    else if (o16) hipLaunchKernelGGL((blend_kernel<float, uint16_t>), grid, dim3(256), 0, hs, f, static_cast<const float *>(input->data), static_cast<uint16_t *>(output->data), vectors);
    else hipLaunchKernelGGL((blend_kernel<float, float>), grid, dim3(256), 0, hs, f, static_cast<const float *>(input->data), static_cast<float *>(output->data), vectors);
    return check_launch("blend");
}

int wrq_blend_lora(wrq_stream stream, const wrq_tensor *factor, const wrq_tensor_view *xa, const wrq_tensor_view *xb, const wrq_tensor_view *output) {
    int s = check_layer_tensor(factor, "blend_lora");
    for (const wrq_tensor_view *t : {xa, xb, output})
        if (s == WRQ_OK) s = check_layer_view(t, "blend_lora");
    if (s != WRQ_OK) return s;
    if (xa->dtype != WRQ_F16 || xb->dtype != WRQ_F16 || output->dtype != WRQ_F16) return fail(WRQ_ERR_TYPE, "blend_lora: the three tensors are f16");
    const uint32_t *o = output->view.shape, *a = xa->view.shape, *b = xb->view.shape;
    // src/tensor/ops.rs:2241-2243
    const uint32_t fs[4] = {4, 1, 1, 1};
    if (!same_shape(factor->shape, fs) || a[1] != o[0] || a[2] != o[2] || a[3] != 1 || b[1] != o[1] || b[2] != o[2] || b[3] != 1 || o[3] != 1)
        return fail(WRQ_ERR_SHAPE, "blend_lora: data shape not match [%u, %u, %u, %u]", o[0], o[1], o[2], o[3]);
    if (o[0] == 0 || o[1] == 0 || o[2] == 0) return WRQ_OK;
    if ((o[1] + 3) / 4 > 65535u || o[2] > 65535u) return fail(WRQ_ERR_SIZE, "blend_lora: data size not match");
    const uint32_t K = a[0] < b[0] ? a[0] : b[0]; // the shader sums over the shorter of the two rows
    const dim3 grid((o[0] / 4 + 63) / 64, (o[1] + 3) / 4, o[2]);
    hipLaunchKernelGGL(blend_lora_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<const float *>(factor->data),
                       static_cast<const uint16_t *>(xa->data), static_cast<const uint16_t *>(xb->data), static_cast<uint16_t *>(output->data), view_args(xa->view),
                       view_args(xb->view), view_args(output->view), K);
    return check_launch("blend_lora");
}

} // extern "C"

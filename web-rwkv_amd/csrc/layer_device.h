// Device and host helpers shared by the layer ops (layer_ops.hip, recurrent_ops.hip, fused_ops.hip).
#pragma once

#include "wrq_device.h"
#include "wrq_host.h"

namespace wrq {

struct ViewArgs {
    uint32_t shape[4], stride[4], offset[4];
};

inline ViewArgs view_args(const wrq_view &v) {
    ViewArgs a;
    for (int i = 0; i < 4; i++) a.shape[i] = v.shape[i], a.stride[i] = v.stride[i], a.offset[i] = v.offset[i];
    return a;
}

// element index of (batch, token, element) in a view: compute_index of the shaders
// (src/shaders/binary.wgsl:30-34), in units of one element
__device__ __forceinline__ uint64_t view_elem(const ViewArgs &v, uint32_t batch, uint32_t token, uint32_t elem) {
    return ((uint64_t)(batch + v.offset[2]) * v.stride[1] + (token + v.offset[1])) * v.stride[0] + elem + v.offset[0];
}
// the same in units of 4 elements (`index` counts vectors)
__device__ __forceinline__ uint64_t view_index(const ViewArgs &v, uint32_t batch, uint32_t token, uint32_t index) {
    const uint64_t stride = v.stride[0] >> 2;
    return ((uint64_t)(batch + v.offset[2]) * v.stride[1] + (token + v.offset[1])) * stride + index + (v.offset[0] >> 2);
}

template <typename XT>
__device__ __forceinline__ float4 load_vec4(const XT *p) {
    if constexpr (sizeof(XT) == 2) {
        const uint2 v = *reinterpret_cast<const uint2 *>(p);
        return make_float4(h2f((uint16_t)(v.x & 0xffffu)), h2f((uint16_t)(v.x >> 16)), h2f((uint16_t)(v.y & 0xffffu)), h2f((uint16_t)(v.y >> 16)));
    } else {
        return *reinterpret_cast<const float4 *>(p);
    }
}

template <typename XT>
__device__ __forceinline__ void store_vec4(XT *p, float4 v) {
    if constexpr (sizeof(XT) == 2) {
        *reinterpret_cast<uint2 *>(p) = make_uint2((uint32_t)f2h(v.x) | ((uint32_t)f2h(v.y) << 16), (uint32_t)f2h(v.z) | ((uint32_t)f2h(v.w) << 16));
    } else {
        *reinterpret_cast<float4 *>(p) = v;
    }
}

template <typename XT>
__device__ __forceinline__ float load_one(const XT *p) {
    if constexpr (sizeof(XT) == 2) return h2f(*p);
    else return *p;
}

struct Cursor {
    uint32_t batch, token, len;
};
__device__ __forceinline__ Cursor unpack_cursor(uint32_t x) { return Cursor{x & 0xffu, (x >> 8) & 0xffffu, (x >> 24) & 0xffu}; }
// Cursors live in device memory, the host cannot check them: a state slot beyond the view is clamped
// to its last slot and a first token beyond the token itself counts as the token itself, so that a
// malformed cursor reads and writes inside the tensors (the shaders rely on WebGPU's bounds clamping).
__device__ __forceinline__ Cursor read_cursor(const uint32_t *cursors, uint32_t stack, const ViewArgs &vs) {
    Cursor c = unpack_cursor(cursors[stack]);
    c.batch = min(c.batch, vs.shape[2] - 1);
    c.token = min(c.token, stack);
    return c;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// sum or maximum over the workgroup, the same value in every thread; `red` holds THREADS / 64 floats
template <bool MAX, int THREADS>
__device__ __forceinline__ float block_reduce(float v, float *red) {
    v = MAX ? wave_max(v) : wave_sum(v);
    if constexpr (THREADS == 64) return v;
    const uint32_t wave = threadIdx.x >> 6;
    __syncthreads(); // `red` may still be read from the previous reduction
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for (int w = 1; w < THREADS / 64; w++) r = MAX ? fmaxf(r, red[w]) : r + red[w];
    return r;
}

// host-side checks shared by the entry points
inline int check_layer_view(const wrq_tensor_view *t, const char *what) {
    if (!t || !t->data) return fail(WRQ_ERR_NULL, "%s: null tensor", what);
    if (t->dtype != WRQ_F16 && t->dtype != WRQ_F32) return fail(WRQ_ERR_TYPE, "%s: unsupported element type %d", what, (int)t->dtype);
    for (int i = 0; i < 4; i++)
        if ((uint64_t)t->view.offset[i] + t->view.shape[i] > t->view.stride[i]) return fail(WRQ_ERR_SHAPE, "%s: slice out of range", what);
    if (t->view.shape[0] % 4 || t->view.stride[0] % 4 || t->view.offset[0] % 4) return fail(WRQ_ERR_ALIGNMENT, "%s: rows not in units of 4 elements", what);
    if ((uintptr_t)t->data % 16) return fail(WRQ_ERR_ALIGNMENT, "%s: device pointers must be 16-byte aligned", what);
    return WRQ_OK;
}

// A state view: cursors address its slots (axis 2) and token_shift its row 0, and the kernels clamp both into
// the view, so a view without slots or rows has nothing to clamp to and is refused.
inline int check_state_view(const wrq_tensor_view *t, const char *what) {
    const int s = check_layer_view(t, what);
    if (s != WRQ_OK) return s;
    if (t->view.shape[1] == 0 || t->view.shape[2] == 0)
        return fail(WRQ_ERR_SHAPE, "%s: state view [%u, %u, %u, %u] has no rows or no slots", what, t->view.shape[0], t->view.shape[1], t->view.shape[2],
                    t->view.shape[3]);
    return WRQ_OK;
}

inline int check_layer_tensor(const wrq_tensor *t, const char *what) {
    if (!t || !t->data) return fail(WRQ_ERR_NULL, "%s: null tensor", what);
    if ((uintptr_t)t->data % 16) return fail(WRQ_ERR_ALIGNMENT, "%s: device pointers must be 16-byte aligned", what);
    return WRQ_OK;
}

inline bool same_shape(const uint32_t *a, const uint32_t *b) { return a[0] == b[0] && a[1] == b[1] && a[2] == b[2] && a[3] == b[3]; }

} // namespace wrq

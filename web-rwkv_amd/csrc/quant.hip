// Weight packing for gfx950: quant_mat_int8 and quant_mat_nf4.
//
// Both are single-pass, bandwidth-bound kernels (2 B read, 1 or 0.5 B written per
// element): a block of the quantisation grid is held by 16 (int8) or 8 (nf4)
// adjacent lanes with one 16-byte load each, the block statistic is reduced with
// DPP inside the lane group, and every lane packs its own eight elements.  The
// reference's two/three dispatches per matrix (statistics, quantise, f32->f16 blit;
// src/tensor/ops.rs:2393-2486, :2488-2589) collapse into one launch with no
// temporary.
//
// The arithmetic is the reference shaders' arithmetic bit for bit
// (src/shaders/quant_mat_int8.wgsl:24-59, quant_mat_nf4.wgsl:24-81): IEEE f32
// division, no fused operations (this file is built with -ffp-contract=off),
// round-half-even for the unorm code, `<=` scan so that the last minimum wins.
#include "wrq_device.h"
#include "wrq_host.h"

namespace wrq {

__device__ __forceinline__ float dpp_f(float v, int ctrl) {
    switch (ctrl) {
    case 0: return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xf, 0xf, true));
    case 1: return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xf, 0xf, true));
    case 2: return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xf, 0xf, true));
    default: return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xf, 0xf, true));
    }
}

// One lane per 8 elements; 16 lanes (one DPP row) per 128-element block.
__global__ __launch_bounds__(256) void quant_int8_kernel(const uint16_t *__restrict__ in,
                                                         uint32_t *__restrict__ minmax,
                                                         uint8_t *__restrict__ out, uint64_t ngroup) {
    uint64_t gid = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    const bool live = gid < ngroup;
    if (!live) gid = ngroup - 1; // keep every lane of the row in the reduction
    float v[8];
    unpack8h(load128(in + gid * 8), v);

    float mn = 65504.0f, mx = -65504.0f; // quant_mat_int8.wgsl:32-33
#pragma unroll
    for (int i = 0; i < 8; i++) {
        mn = fminf(v[i], mn);
        mx = fmaxf(v[i], mx);
    }
#pragma unroll
    for (int s = 0; s < 4; s++) {
        mn = fminf(mn, dpp_f(mn, s));
        mx = fmaxf(mx, dpp_f(mx, s));
    }
    // the quantise pass of the reference reads the pair back through f16: exact, since
    // the extrema of f16 values are f16 values
    const float range = mx - mn;
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        float q = __fdiv_rn(v[i] - mn, range);
        q = fminf(fmaxf(q, 0.0f), 1.0f); // NaN (constant block) -> 0
        uint32_t b = (uint32_t)__builtin_rintf(q * 255.0f);
        if (i < 4)
            lo |= b << (8 * i);
        else
            hi |= b << (8 * (i - 4));
    }
    if (live) {
        *reinterpret_cast<uint2 *>(out + gid * 8) = make_uint2(lo, hi);
        if ((gid & 15) == 0) minmax[gid >> 4] = (uint32_t)f2h(mn) | ((uint32_t)f2h(mx) << 16);
    }
}

// One lane per 8 elements (one output u32); 8 lanes per 64-element block.
__global__ __launch_bounds__(256) void quant_nf4_kernel(const uint16_t *__restrict__ in,
                                                        const float *__restrict__ quant,
                                                        uint16_t *__restrict__ absmax,
                                                        uint32_t *__restrict__ out, uint64_t ngroup) {
    float q[16];
#pragma unroll
    for (int j = 0; j < 16; j++) q[j] = quant[j];

    uint64_t gid = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    const bool live = gid < ngroup;
    if (!live) gid = ngroup - 1;
    float v[8];
    unpack8h(load128(in + gid * 8), v);

    float am = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) am = fmaxf(fabsf(v[i]), am);
#pragma unroll
    for (int s = 0; s < 3; s++) am = fmaxf(am, dpp_f(am, s)); // 8 lanes: two quad steps + half mirror

    const float inv = __fdiv_rn(1.0f, am); // quant_mat_nf4.wgsl:59
    uint32_t y = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float xx = v[i] * inv;
        float min_err = 1.0f;
        uint32_t min_index = 0;
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const float err = fabsf(q[j] - xx);
            if (err <= min_err) { // false for NaN: an all-zero block packs to nibble 0
                min_err = err;
                min_index = j;
            }
        }
        y |= min_index << (4 * i);
    }
    if (live) {
        out[gid] = y;
        if ((gid & 7) == 0) absmax[gid >> 3] = f2h(am);
    }
}

int launch_quant_int8(hipStream_t stream, const void *in, void *minmax, void *out, uint64_t len) {
    const uint64_t ngroup = len / 8;
    if (ngroup == 0) return WRQ_OK;
    const uint64_t grid = (ngroup + 255) / 256;
    if (grid > 0x7fffffffull) return fail(WRQ_ERR_SIZE, "data size not match: %llu vs. %llu", (unsigned long long)len, 0x7fffffffull * 2048ull);
    hipLaunchKernelGGL(quant_int8_kernel, dim3((uint32_t)grid), dim3(256), 0, stream,
                       (const uint16_t *)in, (uint32_t *)minmax, (uint8_t *)out, ngroup);
    return check_launch("quant_mat_int8");
}

int launch_quant_nf4(hipStream_t stream, const void *in, const void *quant, void *absmax, void *out,
                     uint64_t len) {
    const uint64_t ngroup = len / 8;
    if (ngroup == 0) return WRQ_OK;
    const uint64_t grid = (ngroup + 255) / 256;
    if (grid > 0x7fffffffull) return fail(WRQ_ERR_SIZE, "data size not match: %llu vs. %llu", (unsigned long long)len, 0x7fffffffull * 2048ull);
    hipLaunchKernelGGL(quant_nf4_kernel, dim3((uint32_t)grid), dim3(256), 0, stream,
                       (const uint16_t *)in, (const float *)quant, (uint16_t *)absmax, (uint32_t *)out,
                       ngroup);
    return check_launch("quant_mat_nf4");
}

} // namespace wrq

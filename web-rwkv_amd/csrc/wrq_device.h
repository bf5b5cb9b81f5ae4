// Device-side helpers shared by the gfx950 kernels: vector loads, wave64 reductions,
// f16 conversion and the activation epilogue.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "../../include/wrq.h"

namespace wrq {

constexpr int kWave = 64;

// Operands of one product launch, resolved on the host from tensors and views.
struct MatmulArgs {
    const uint8_t *w;     // packed weights, row-major [B][R][K or K/2]
    const uint16_t *scale; // int8: (min, max) f16 pairs per 128 flat elements; nf4: absmax f16 per 64
    const float *quant;   // nf4: 16-entry table (device); int8: unused
    const void *x;        // first element of the input view (offset applied)
    void *out;            // first element of the output view (offset applied)
    uint32_t K, R, T, B;
    uint64_t x_token_stride, x_batch_stride;     // elements
    uint64_t out_token_stride, out_batch_stride; // elements
    int out_f16; // 1: f16 stores, 0: f32
    int act;
};

// One activation, chosen at compile time (src/tensor/ops.rs:205-235).
template <int ACT>
__device__ __forceinline__ float act_one(float x) {
    if constexpr (ACT == WRQ_ACT_SQUARED_RELU) {
        const float p = fmaxf(x, 0.0f);
        return p * p;
    } else if constexpr (ACT == WRQ_ACT_TANH) {
        return x > 42.0f ? 1.0f : tanhf(x);
    } else if constexpr (ACT == WRQ_ACT_STABLE_EXP) {
        return expf(-expf(x));
    } else if constexpr (ACT == WRQ_ACT_OPPOSITE_EXP) {
        return -expf(x);
    } else if constexpr (ACT == WRQ_ACT_SOFTPLUS) {
        return logf(1.0f + expf(x));
    } else if constexpr (ACT == WRQ_ACT_SIGMOID) {
        return 1.0f / (1.0f + expf(-x));
    } else if constexpr (ACT == WRQ_ACT_SILU) {
        return x / (1.0f + expf(-x));
    } else {
        return x;
    }
}

__device__ __forceinline__ float act_apply(int act, float x) {
    switch (act) {
    case WRQ_ACT_SQUARED_RELU: return act_one<WRQ_ACT_SQUARED_RELU>(x);
    case WRQ_ACT_TANH: return act_one<WRQ_ACT_TANH>(x);
    case WRQ_ACT_STABLE_EXP: return act_one<WRQ_ACT_STABLE_EXP>(x);
    case WRQ_ACT_OPPOSITE_EXP: return act_one<WRQ_ACT_OPPOSITE_EXP>(x);
    case WRQ_ACT_SOFTPLUS: return act_one<WRQ_ACT_SOFTPLUS>(x);
    case WRQ_ACT_SIGMOID: return act_one<WRQ_ACT_SIGMOID>(x);
    case WRQ_ACT_SILU: return act_one<WRQ_ACT_SILU>(x);
    default: return x;
    }
}

// Calls f(std::integral_constant<int, ACT>) for the run-time activation: hoists the
// choice out of element loops.
template <typename F>
__device__ __forceinline__ void act_dispatch(int act, F &&f) {
    switch (act) {
    case WRQ_ACT_SQUARED_RELU: f(std::integral_constant<int, WRQ_ACT_SQUARED_RELU>{}); break;
    case WRQ_ACT_TANH: f(std::integral_constant<int, WRQ_ACT_TANH>{}); break;
    case WRQ_ACT_STABLE_EXP: f(std::integral_constant<int, WRQ_ACT_STABLE_EXP>{}); break;
    case WRQ_ACT_OPPOSITE_EXP: f(std::integral_constant<int, WRQ_ACT_OPPOSITE_EXP>{}); break;
    case WRQ_ACT_SOFTPLUS: f(std::integral_constant<int, WRQ_ACT_SOFTPLUS>{}); break;
    case WRQ_ACT_SIGMOID: f(std::integral_constant<int, WRQ_ACT_SIGMOID>{}); break;
    case WRQ_ACT_SILU: f(std::integral_constant<int, WRQ_ACT_SILU>{}); break;
    default: f(std::integral_constant<int, WRQ_ACT_NONE>{}); break;
    }
}

__device__ __forceinline__ float h2f(uint16_t h) {
    return __half2float(__ushort_as_half(h));
}

__device__ __forceinline__ uint16_t f2h(float f) {
    return __half_as_ushort(__float2half_rn(f));
}

__device__ __forceinline__ void store_out(void *out, int out_f16, uint64_t idx, float v) {
    if (out_f16)
        reinterpret_cast<uint16_t *>(out)[idx] = f2h(v);
    else
        reinterpret_cast<float *>(out)[idx] = v;
}

__device__ __forceinline__ uint4 load128(const void *p) {
    return *reinterpret_cast<const uint4 *>(p);
}

// Streaming 16-byte load for data touched once (packed weights): keeps it from
// displacing the activation vector in the caches.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint4 load128_stream(const void *p) {
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

__device__ __forceinline__ uint2 load64_stream(const void *p) {
    const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(p));
    return make_uint2(v.x, v.y);
}

// Workgroup barrier that orders LDS traffic only: global loads issued before it stay in
// flight across it (a full __syncthreads() would wait for them).
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Sum over the 64 lanes of a wave; the result is valid in every lane.
__device__ __forceinline__ float wave_sum(float v) {
    // within rows of 16 lanes: quad permutes, then half-mirror and mirror
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xf, 0xf, true));  // quad_perm [1,0,3,2]
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xf, 0xf, true));  // quad_perm [2,3,0,1]
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xf, 0xf, true)); // row_half_mirror
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xf, 0xf, true)); // row_mirror
    // across the four rows
    float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return (r0 + r1) + (r2 + r3);
}

// Unpack 8 f16 values held in a uint4 to f32.
__device__ __forceinline__ void unpack8h(const uint4 &v, float *f) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        f[2 * i] = h2f((uint16_t)(w[i] & 0xffffu));
        f[2 * i + 1] = h2f((uint16_t)(w[i] >> 16));
    }
}

// Load N (multiple of 8) consecutive activations as f32 from an f16 or f32 row.
template <typename XT, int N>
__device__ __forceinline__ void load_x(const XT *p, float *f) {
    if constexpr (sizeof(XT) == 2) {
#pragma unroll
        for (int i = 0; i < N / 8; i++) unpack8h(load128(p + 8 * i), f + 8 * i);
    } else {
#pragma unroll
        for (int i = 0; i < N / 4; i++) {
            uint4 v = load128(p + 4 * i);
            f[4 * i] = __uint_as_float(v.x);
            f[4 * i + 1] = __uint_as_float(v.y);
            f[4 * i + 2] = __uint_as_float(v.z);
            f[4 * i + 3] = __uint_as_float(v.w);
        }
    }
}

} // namespace wrq

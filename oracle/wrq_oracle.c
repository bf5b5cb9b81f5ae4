/*
 * wrq_oracle.c -- CPU restatement of web-rwkv's quantized-weight matrix path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker for the HIP library: it
 * is linked or loaded only by tests, by the smoke check and by the CPU-baseline
 * leg of the benchmark.  Nothing in the shipped library calls it, and the
 * library has no CPU fallback.
 *
 * Every function follows one reference shader op for op (same block sizes,
 * same per-element arithmetic in f32, same lane striding and tree reduction
 * where the shader defines them).  Citations are relative to the reference
 * checkout (src/...).
 *
 * Arithmetic policy where the shading language leaves a choice open:
 *   - `/` and `1.0 / x` are IEEE-754 correctly rounded f32 operations.
 *   - pack4x8unorm(x) rounds fl32(clamp(x,0,1) * 255.0f) half-to-even
 *     (the lowering Mesa's NIR uses for lavapipe); clamp(NaN) is 0.
 *   - f32 -> f16 stores round to nearest even.
 *   - fma() is a real fused multiply-add where the shader writes fma(), and a
 *     4-term dot product is evaluated left to right with fused steps.
 *   Compile with -ffp-contract=off so the compiler adds no fusions of its own.
 *
 * Parity status of this oracle (what pins it, see tests/test_oracle_*.py):
 *   - packing: pinned by the closed forms of the reference's own unit tests
 *     (src/tensor/ops.rs:2939-2962 int8, :3114-3144 nf4), by exhaustive and
 *     brute-force cases, and by invariants (block min -> 0, max -> 255, ...).
 *     The rounding of an int8 code whose scaled value lies within one ulp of
 *     n + 0.5 is "parity unpinned": the reference's test accepts +-1 there
 *     (src/tensor/ops.rs:2995-3000).  wrq_oracle_quant_int8 counts those
 *     elements so that tests can report them.
 *   - products: pinned against f64 dequantise-then-matmul (numpy) and the
 *     reference tests' formulas (src/tensor/ops.rs:3004-3018, :3199-3211).
 *   - fp16 matrices (matmul_vec_fp16 / matmul_mat_fp16): pinned against f64 matmul of
 *     the same f16 values (numpy), the transposed-operand trap, views and activations.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define WRQ_INT8_BLOCK 128u /* src/tensor/ops.rs:292 */
#define WRQ_NF4_BLOCK 64u   /* src/tensor/ops.rs:291 */
#define WG 128u             /* BLOCK_SIZE of the vec kernels, src/tensor/ops.rs:799,901 */

/* ------------------------------------------------------------------ f16 */

static float h2f(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            /* subnormal: normalise */
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while (!(man & 0x400u));
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* round-to-nearest-even f32 -> f16 */
static uint16_t f2h(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t abs = x & 0x7fffffffu;
    if (abs >= 0x7f800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | ((abs > 0x7f800000u) ? 0x200u : 0u));
    }
    if (abs >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (abs < 0x33000001u) { /* <= 2^-25 -> 0 (2^-25 ties to even = 0) */
        return (uint16_t)sign;
    }
    int32_t e = (int32_t)(abs >> 23) - 127;
    uint32_t m = (abs & 0x7fffffu) | 0x800000u;
    uint32_t shift, half;
    if (e < -14) { /* subnormal result */
        shift = (uint32_t)(13 + (-14 - e));
        uint32_t r = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        half = 1u << (shift - 1);
        if (rem > half || (rem == half && (r & 1u))) r++;
        return (uint16_t)(sign | r);
    }
    shift = 13;
    uint32_t r = ((uint32_t)(e + 15) << 10) | ((m >> shift) & 0x3ffu);
    uint32_t rem = m & 0x1fffu;
    half = 0x1000u;
    if (rem > half || (rem == half && (r & 1u))) r++; /* carry may bump the exponent: fine */
    return (uint16_t)(sign | r);
}

void wrq_oracle_f16_to_f32(const uint16_t *src, float *dst, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = h2f(src[i]);
}

void wrq_oracle_f32_to_f16(const float *src, uint16_t *dst, size_t n) {
    for (size_t i = 0; i < n; i++) dst[i] = f2h(src[i]);
}

/* ------------------------------------------------------------ views */

/* Byte layout of the reference's View uniform: shape, stride (= shape of the
 * parent tensor), offset; src/tensor/mod.rs:26-43, built at :1121-1141. */
typedef struct {
    uint32_t shape[4];
    uint32_t stride[4];
    uint32_t offset[4];
} wrq_view;

/* compute_index of the shaders, in units of (1 << step) elements;
 * src/shaders/matmul_vec_int8.wgsl:31-35, matmul_vec_nf4.wgsl:32-36. */
static size_t view_index(const wrq_view *v, uint32_t batch, uint32_t token, uint32_t index,
                         uint32_t step) {
    size_t stride = v->stride[0] >> step;
    size_t ox = v->offset[0] >> step;
    return ((size_t)(batch + v->offset[2]) * v->stride[1] + (token + v->offset[1])) * stride +
           (index + ox);
}

enum { WRQ_F16 = 0, WRQ_F32 = 1 };

static void load4(const void *base, int dtype, size_t idx4, float out[4]) {
    if (dtype == WRQ_F16) {
        const uint16_t *p = (const uint16_t *)base + idx4 * 4;
        for (int i = 0; i < 4; i++) out[i] = h2f(p[i]);
    } else {
        const float *p = (const float *)base + idx4 * 4;
        for (int i = 0; i < 4; i++) out[i] = p[i];
    }
}

static void store4(void *base, int dtype, size_t idx4, const float v[4]) {
    if (dtype == WRQ_F16) {
        uint16_t *p = (uint16_t *)base + idx4 * 4;
        for (int i = 0; i < 4; i++) p[i] = f2h(v[i]);
    } else {
        float *p = (float *)base + idx4 * 4;
        for (int i = 0; i < 4; i++) p[i] = v[i];
    }
}

/* ------------------------------------------------------ activations */

/* src/tensor/ops.rs:146-160 (order of the enum) and :205-235 (definitions). */
enum {
    ACT_NONE = 0,
    ACT_SQUARED_RELU,
    ACT_TANH,
    ACT_STABLE_EXP,
    ACT_OPPOSITE_EXP,
    ACT_SOFTPLUS,
    ACT_SIGMOID,
    ACT_SILU
};

static float activate(int act, float x) {
    switch (act) {
    case ACT_SQUARED_RELU: {
        float p = x > 0.0f ? x : 0.0f;
        return p * p;
    }
    case ACT_TANH:
        return x > 42.0f ? 1.0f : tanhf(x);
    case ACT_STABLE_EXP:
        return expf(-expf(x));
    case ACT_OPPOSITE_EXP:
        return -expf(x);
    case ACT_SOFTPLUS:
        return logf(1.0f + expf(x));
    case ACT_SIGMOID:
        return 1.0f / (1.0f + expf(-x));
    case ACT_SILU:
        return x / (1.0f + expf(-x));
    default:
        return x;
    }
}

static float dot4(const float a[4], const float b[4]) {
    float t = a[0] * b[0];
    t = fmaf(a[1], b[1], t);
    t = fmaf(a[2], b[2], t);
    t = fmaf(a[3], b[3], t);
    return t;
}

/* -------------------------------------------------------- int8 pack */

/* pack4x8unorm component under the stated policy. */
static uint8_t unorm8(float q, int *sensitive) {
    float c = q > 0.0f ? q : 0.0f; /* NaN -> 0 */
    c = c < 1.0f ? c : 1.0f;
    float s = c * 255.0f;
    float r = rintf(s); /* default rounding mode: nearest even */
    if (sensitive) {
        /* within one ulp of a tie n + 0.5 ? */
        float fl = floorf(s);
        float d = fabsf((s - fl) - 0.5f);
        float ulp = nextafterf(s, INFINITY) - s;
        *sensitive = (d <= ulp) || (q != q);
    }
    return (uint8_t)r;
}

/*
 * src/shaders/quant_mat_int8.wgsl:24-46 (compute_minmax) and :48-59 (quantize).
 * `len` elements, a multiple of 128.  minmax gets 2 * len / 128 f16 values
 * (min, max interleaved).  Returns the number of policy-sensitive codes.
 */
uint64_t wrq_oracle_quant_int8(const uint16_t *input, size_t len, uint16_t *minmax, uint8_t *output) {
    uint64_t flagged = 0;
    size_t nblk = len / WRQ_INT8_BLOCK;
#pragma omp parallel for reduction(+ : flagged) schedule(static)
    for (size_t j = 0; j < nblk; j++) {
        float mn = 65504.0f, mx = -65504.0f;
        const uint16_t *blk = input + j * WRQ_INT8_BLOCK;
        for (uint32_t i = 0; i < WRQ_INT8_BLOCK; i++) {
            float v = h2f(blk[i]);
            mn = v < mn ? v : mn;
            mx = v > mx ? v : mx;
        }
        minmax[2 * j] = f2h(mn);
        minmax[2 * j + 1] = f2h(mx);
        /* the quantize pass reads the pair back through f16 (exact here) */
        float m0 = h2f(minmax[2 * j]), m1 = h2f(minmax[2 * j + 1]);
        float range = m1 - m0;
        for (uint32_t i = 0; i < WRQ_INT8_BLOCK; i++) {
            float v = h2f(blk[i]);
            float q = (v - m0) / range;
            int s;
            output[j * WRQ_INT8_BLOCK + i] = unorm8(q, &s);
            flagged += (uint64_t)s;
        }
    }
    return flagged;
}

/* --------------------------------------------------------- nf4 pack */

/*
 * src/shaders/quant_mat_nf4.wgsl:24-45 (compute_absmax), :47-81 (quantize) and
 * the f32 -> f16 blit of absmax (src/tensor/ops.rs:2586).  `len` elements, a
 * multiple of 64; output len / 2 bytes; absmax len / 64 f16 values.
 */
void wrq_oracle_quant_nf4(const uint16_t *input, size_t len, const float quant[16], uint16_t *absmax,
                          uint8_t *output) {
    size_t nblk = len / WRQ_NF4_BLOCK;
#pragma omp parallel for schedule(static)
    for (size_t j = 0; j < nblk; j++) {
        const uint16_t *blk = input + j * WRQ_NF4_BLOCK;
        float am = 0.0f;
        for (uint32_t i = 0; i < WRQ_NF4_BLOCK; i++) {
            float a = fabsf(h2f(blk[i]));
            am = a > am ? a : am;
        }
        absmax[j] = f2h(am);
        float inv = 1.0f / am;
        for (uint32_t g = 0; g < WRQ_NF4_BLOCK / 8; g++) {
            uint32_t y = 0;
            for (uint32_t i = 0; i < 8; i++) {
                float xx = h2f(blk[g * 8 + i]) * inv;
                float min_err = 1.0f;
                uint32_t min_index = 0;
                for (uint32_t n = 0; n < 16; n++) {
                    float err = fabsf(quant[n] - xx);
                    if (err <= min_err) {
                        min_err = err;
                        min_index = n;
                    }
                }
                y |= min_index << (i * 4);
            }
            uint8_t *o = output + (j * WRQ_NF4_BLOCK) / 2 + g * 4;
            o[0] = (uint8_t)y;
            o[1] = (uint8_t)(y >> 8);
            o[2] = (uint8_t)(y >> 16);
            o[3] = (uint8_t)(y >> 24);
        }
    }
}

/* ---------------------------------------------------------- helpers */

static uint32_t load_u32(const uint8_t *m, size_t idx) {
    const uint8_t *p = m + idx * 4;
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

/* fma(unpack4x8unorm(w), max - min, min); src/shaders/matmul_vec_int8.wgsl:89 */
static void deq_int8(uint32_t w, const uint16_t *minmax, size_t ci, float out[4]) {
    size_t blk = ci / (WRQ_INT8_BLOCK / 4);
    float mn = h2f(minmax[2 * blk]), mx = h2f(minmax[2 * blk + 1]);
    float range = mx - mn;
    for (int d = 0; d < 4; d++) {
        float u = (float)((w >> (8 * d)) & 0xffu) / 255.0f;
        out[d] = fmaf(u, range, mn);
    }
}

static void tree_reduce(float (*sketch)[4]) {
    /* src/shaders/matmul_vec_int8.wgsl:50-55,98-104 */
    for (uint32_t s = WG / 2; s > 0; s >>= 1)
        for (uint32_t i = 0; i < s; i++)
            for (int r = 0; r < 4; r++) sketch[i][r] += sketch[i + s][r];
}

/* --------------------------------------------------------- int8 GEMV */

/*
 * src/shaders/matmul_vec_int8.wgsl:57-115 with the host side of
 * src/tensor/ops.rs:791-886: matrix [K, R, B] u8, input view [K, T, B],
 * output view [R, T, B]; one 128-lane group per (4 rows, token, batch).
 */
void wrq_oracle_matmul_vec_int8(const uint8_t *matrix, const uint16_t *minmax, uint32_t K, uint32_t R,
                                uint32_t B, const void *input, const wrq_view *src, int in_dtype,
                                void *output, const wrq_view *dst, int out_dtype, int act,
                                int sparse) {
    uint32_t T = dst->shape[1];
    size_t stride = K / 4;
    for (uint32_t batch = 0; batch < B; batch++)
        for (uint32_t token = 0; token < T; token++) {
#pragma omp parallel for schedule(static)
            for (uint32_t channel = 0; channel < R / 4; channel++) {
                float sketch[WG][4];
                size_t bb = view_index(src, batch, token, 0, 2);
                size_t cb = (size_t)batch * R * stride + (size_t)channel * 4 * stride;
                for (uint32_t lane = 0; lane < WG; lane++) {
                    float local[4] = {0, 0, 0, 0};
                    for (size_t i = lane; i < stride; i += WG) {
                        float x[4];
                        load4(input, in_dtype, bb + i, x);
                        if (sparse && x[0] == 0.0f && x[1] == 0.0f && x[2] == 0.0f && x[3] == 0.0f)
                            continue;
                        for (int r = 0; r < 4; r++) {
                            size_t ci = cb + i + (size_t)r * stride;
                            float m[4];
                            deq_int8(load_u32(matrix, ci), minmax, ci, m);
                            local[r] += dot4(m, x);
                        }
                    }
                    memcpy(sketch[lane], local, sizeof(local));
                }
                tree_reduce(sketch);
                float out[4];
                for (int r = 0; r < 4; r++) out[r] = activate(act, sketch[0][r]);
                store4(output, out_dtype, view_index(dst, batch, token, channel, 2), out);
            }
        }
}

/* ---------------------------------------------------------- nf4 GEMV */

/* unpack_absmax; src/shaders/matmul_vec_nf4.wgsl:46-49 (index in u32 units) */
static float absmax_at(const uint16_t *absmax, size_t ci) {
    return h2f(absmax[ci / (WRQ_NF4_BLOCK / 8)]);
}

/*
 * src/shaders/matmul_vec_nf4.wgsl:90-173 with src/tensor/ops.rs:892-991:
 * matrix [K/2, R, B] bytes, two nibbles per byte, element i of a u32 in bits
 * [4i, 4i+4).
 */
void wrq_oracle_matmul_vec_nf4(const uint8_t *matrix, const float quant[16], const uint16_t *absmax,
                               uint32_t K, uint32_t R, uint32_t B, const void *input,
                               const wrq_view *src, int in_dtype, void *output, const wrq_view *dst,
                               int out_dtype, int act, int sparse) {
    uint32_t T = dst->shape[1];
    size_t stride = K / 8; /* u32 per row */
    for (uint32_t batch = 0; batch < B; batch++)
        for (uint32_t token = 0; token < T; token++) {
#pragma omp parallel for schedule(static)
            for (uint32_t channel = 0; channel < R / 4; channel++) {
                float sketch[WG][4];
                size_t bb = view_index(src, batch, token, 0, 3); /* units of 8 elements */
                size_t cb = (size_t)batch * R * stride + (size_t)channel * 4 * stride;
                for (uint32_t lane = 0; lane < WG; lane++) {
                    float local[4] = {0, 0, 0, 0};
                    for (size_t i = lane; i < stride; i += WG) {
                        float xlo[4], xhi[4];
                        load4(input, in_dtype, (bb + i) * 2, xlo);
                        load4(input, in_dtype, (bb + i) * 2 + 1, xhi);
                        if (sparse) {
                            int zero = 1;
                            for (int d = 0; d < 4; d++) zero &= (xlo[d] == 0.0f) & (xhi[d] == 0.0f);
                            if (zero) continue;
                        }
                        uint32_t v[4];
                        float a[4];
                        for (int r = 0; r < 4; r++) {
                            size_t ci = cb + i + (size_t)r * stride;
                            v[r] = load_u32(matrix, ci);
                            a[r] = absmax_at(absmax, ci);
                        }
                        for (int r = 0; r < 4; r++) {
                            float m[4];
                            for (int d = 0; d < 4; d++) m[d] = quant[(v[r] >> (4 * d)) & 0xfu];
                            local[r] = fmaf(dot4(m, xlo), a[r], local[r]);
                        }
                        for (int r = 0; r < 4; r++) {
                            float m[4];
                            for (int d = 0; d < 4; d++) m[d] = quant[(v[r] >> (16 + 4 * d)) & 0xfu];
                            local[r] = fmaf(dot4(m, xhi), a[r], local[r]);
                        }
                    }
                    memcpy(sketch[lane], local, sizeof(local));
                }
                tree_reduce(sketch);
                float out[4];
                for (int r = 0; r < 4; r++) out[r] = activate(act, sketch[0][r]);
                store4(output, out_dtype, view_index(dst, batch, token, channel, 2), out);
            }
        }
}

/* --------------------------------------------------------- int8 GEMM */

/*
 * src/shaders/matmul_mat_int8.wgsl:62-153 with src/tensor/ops.rs:1072-1140.
 * Each output (row r, token t) accumulates k-steps of 8 u32 (32 elements);
 * the (min, max) pair of a row is fetched once per k-step at the step's first
 * column (:99-104), so the result is the dequantised product only when no
 * 128-block boundary falls inside a k-step (K % 32 == 0).  The matrix view is
 * [K, R, B]; its offset applies to both weights and scale lookup as in the
 * shader.
 */
void wrq_oracle_matmul_mat_int8(const uint8_t *matrix, const wrq_view *va, const uint16_t *minmax,
                                const void *input, const wrq_view *vb, int in_dtype, void *output,
                                const wrq_view *dst, int out_dtype, int act) {
    uint32_t K4a = va->shape[0] / 4, R = va->shape[1];
    uint32_t K4b = vb->shape[0] / 4, T = vb->shape[1];
    uint32_t B = dst->shape[2];
    uint32_t stride = K4a < K4b ? K4a : K4b;
    for (uint32_t batch = 0; batch < B; batch++) {
#pragma omp parallel for schedule(static)
        for (uint32_t r4 = 0; r4 < R / 4; r4++) {
            for (uint32_t t = 0; t < T; t++) {
                float acc[4] = {0, 0, 0, 0};
                for (uint32_t k = 0; k < stride; k += 8) {
                    for (int j = 0; j < 4; j++) {
                        uint32_t r = r4 * 4 + j;
                        /* the shader steps the scale index by `stride` per row (:100-103) */
                        size_t blk = (view_index(va, batch, r4 * 4, k, 2) + (size_t)j * stride) /
                                     (WRQ_INT8_BLOCK / 4);
                        float mn = h2f(minmax[2 * blk]), mx = h2f(minmax[2 * blk + 1]);
                        float range = mx - mn;
                        for (uint32_t x = 0; x < 8 && k + x < stride; x++) {
                            uint32_t w = load_u32(matrix, view_index(va, batch, r, k + x, 2));
                            float m[4], xb[4];
                            for (int d = 0; d < 4; d++)
                                m[d] = fmaf((float)((w >> (8 * d)) & 0xffu) / 255.0f, range, mn);
                            load4(input, in_dtype, view_index(vb, batch, t, k + x, 2), xb);
                            acc[j] += dot4(m, xb);
                        }
                    }
                }
                float out[4];
                for (int j = 0; j < 4; j++) out[j] = activate(act, acc[j]);
                store4(output, out_dtype, view_index(dst, batch, t, r4, 2), out);
            }
        }
    }
}

/* ---------------------------------------------------------- nf4 GEMM */

/*
 * src/shaders/matmul_mat_nf4.wgsl:94-220 with src/tensor/ops.rs:1150-1221.
 * The matrix view is [K/2, R, B] in bytes; k-steps of 8 u32 = 64 elements =
 * one absmax block; weights are scaled by absmax before the dot (:154-159).
 */
void wrq_oracle_matmul_mat_nf4(const uint8_t *matrix, const wrq_view *va, const float quant[16],
                               const uint16_t *absmax, const void *input, const wrq_view *vb,
                               int in_dtype, void *output, const wrq_view *dst, int out_dtype,
                               int act) {
    uint32_t K8a = va->shape[0] / 4, R = va->shape[1]; /* u32 per row */
    uint32_t K8b = vb->shape[0] / 8, T = vb->shape[1];
    uint32_t B = dst->shape[2];
    uint32_t stride = K8a < K8b ? K8a : K8b;
    for (uint32_t batch = 0; batch < B; batch++) {
#pragma omp parallel for schedule(static)
        for (uint32_t r4 = 0; r4 < R / 4; r4++) {
            for (uint32_t t = 0; t < T; t++) {
                float acc[4] = {0, 0, 0, 0};
                for (uint32_t k = 0; k < stride; k += 8) {
                    for (int j = 0; j < 4; j++) {
                        uint32_t r = r4 * 4 + j;
                        size_t ai = view_index(va, batch, r4 * 4, k, 2) + (size_t)j * stride;
                        float a = absmax_at(absmax, ai);
                        for (uint32_t x = 0; x < 8 && k + x < stride; x++) {
                            uint32_t w = load_u32(matrix, view_index(va, batch, r, k + x, 2));
                            float m[4], xb[4];
                            for (int d = 0; d < 4; d++) m[d] = a * quant[(w >> (4 * d)) & 0xfu];
                            load4(input, in_dtype, view_index(vb, batch, t, k + x, 3) * 2, xb);
                            acc[j] += dot4(m, xb);
                            for (int d = 0; d < 4; d++)
                                m[d] = a * quant[(w >> (16 + 4 * d)) & 0xfu];
                            load4(input, in_dtype, view_index(vb, batch, t, k + x, 3) * 2 + 1, xb);
                            acc[j] += dot4(m, xb);
                        }
                    }
                }
                float out[4];
                for (int j = 0; j < 4; j++) out[j] = activate(act, acc[j]);
                store4(output, out_dtype, view_index(dst, batch, t, r4, 2), out);
            }
        }
    }
}

/* ---------------------------------------------------------- fp16 matrices */

/*
 * src/shaders/matmul_vec_fp16.wgsl:57-120 with src/tensor/ops.rs:697-784: matrix f16
 * [K, R, B]; 128 lanes stride over groups of 4 elements, 4 rows per workgroup, tree reduce.
 */
void wrq_oracle_matmul_vec_fp16(const uint16_t *matrix, uint32_t K, uint32_t R, uint32_t B,
                                const void *input, const wrq_view *src, int in_dtype, void *output,
                                const wrq_view *dst, int out_dtype, int act, int sparse) {
    uint32_t T = dst->shape[1];
    size_t stride = K / 4;
    for (uint32_t batch = 0; batch < B; batch++)
        for (uint32_t token = 0; token < T; token++) {
#pragma omp parallel for schedule(static)
            for (uint32_t channel = 0; channel < R / 4; channel++) {
                float sketch[WG][4];
                size_t bb = view_index(src, batch, token, 0, 2);
                size_t cb = (size_t)batch * R * stride + (size_t)channel * 4 * stride;
                for (uint32_t lane = 0; lane < WG; lane++) {
                    float local[4] = {0, 0, 0, 0};
                    for (size_t i = lane; i < stride; i += WG) {
                        float x[4];
                        load4(input, in_dtype, bb + i, x);
                        if (sparse && x[0] == 0.0f && x[1] == 0.0f && x[2] == 0.0f && x[3] == 0.0f)
                            continue;
                        for (int r = 0; r < 4; r++) {
                            float m[4];
                            load4(matrix, 0, cb + i + (size_t)r * stride, m);
                            local[r] += dot4(m, x);
                        }
                    }
                    memcpy(sketch[lane], local, sizeof(local));
                }
                tree_reduce(sketch);
                float out[4];
                for (int r = 0; r < 4; r++) out[r] = activate(act, sketch[0][r]);
                store4(output, out_dtype, view_index(dst, batch, token, channel, 2), out);
            }
        }
}

/*
 * src/shaders/matmul_mat_fp16.wgsl:57-140 with src/tensor/ops.rs:999-1061: matrix view
 * [K, R, B] f16; k runs in groups of 4 elements, 8 groups per tile step, in order.
 */
void wrq_oracle_matmul_mat_fp16(const uint16_t *matrix, const wrq_view *va, const void *input,
                                const wrq_view *vb, int in_dtype, void *output, const wrq_view *dst,
                                int out_dtype, int act) {
    uint32_t K4a = va->shape[0] / 4, R = va->shape[1];
    uint32_t K4b = vb->shape[0] / 4, T = vb->shape[1];
    uint32_t B = dst->shape[2];
    uint32_t stride = K4a < K4b ? K4a : K4b;
    for (uint32_t batch = 0; batch < B; batch++) {
#pragma omp parallel for schedule(static)
        for (uint32_t r4 = 0; r4 < R / 4; r4++) {
            for (uint32_t t = 0; t < T; t++) {
                float acc[4] = {0, 0, 0, 0};
                for (uint32_t k = 0; k < stride; k++) {
                    float xb[4];
                    load4(input, in_dtype, view_index(vb, batch, t, k, 2), xb);
                    for (int j = 0; j < 4; j++) {
                        float m[4];
                        load4(matrix, 0, view_index(va, batch, r4 * 4 + j, k, 2), m);
                        acc[j] += dot4(m, xb);
                    }
                }
                float out[4];
                for (int j = 0; j < 4; j++) out[j] = activate(act, acc[j]);
                store4(output, out_dtype, view_index(dst, batch, t, r4, 2), out);
            }
        }
    }
}

int wrq_oracle_abi_version(void) { return 1; }

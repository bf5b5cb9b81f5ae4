// Chunk-shaped products on packed weights for gfx950: matmul_mat_int8 / matmul_mat_nf4
// on the f16 matrix cores (v_mfma_f32_16x16x32_f16, f32 accumulate).
//
// out[t, r] = ACT( sum_k deq(W[r, k]) * x[t, k] )      (src/shaders/matmul_mat_int8.wgsl:62-153,
//                                                        src/shaders/matmul_mat_nf4.wgsl:94-220)
//
// Layout of one workgroup (4 waves): 64 weight rows x (16 * NTILE) tokens, K walked in
// steps of 128.  Wave w owns rows 16w..16w+15 as the MFMA "A" side.  Weight bytes go
// from HBM straight into the A registers of the one wave that uses them (each byte is
// read once and never shared, so an LDS tile for them would only add traffic); the
// activation tile, shared by all four waves, is staged as f16 in double-buffered LDS
// and read back as "B" operands with ds_read_b128.
//
// The scales never enter the matrix cores, which keeps the f16 operands exact:
//   int8: A holds the codes as f16 (1024 + u, built with one v_perm_b32 per two
//         weights); after each 128-block   out += s * D + (min - 1024 s) * sum_k x
//         with s = (max - min) / 255, and sum_k x taken from the B registers.
//   nf4:  A holds table values split into two f16 halves (hi + lo * 2^-11, exact to
//         2^-22), fetched per byte (two weights) from a 256-entry LDS table; after
//         each 64-block   out += absmax * (D_hi + 2^-11 D_lo).
#include "wrq_device.h"
#include "wrq_host.h"

namespace wrq {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));

union HalfPack {
    uint32_t u[4];
    half8 h;
};

constexpr int kStep = 128;        // K elements per step
constexpr int kPitch = kStep + 8; // f16 elements per LDS row: 272 B keeps 16-byte alignment and rotates banks

__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
    return (uint32_t)f2h(a) | ((uint32_t)f2h(b) << 16);
}

typedef _Float16 half2v __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float dot2_ones(uint32_t v, float acc) {
    // acc + lo(v) + hi(v) with f32 accumulation: v_dot2_f32_f16 against (1.0, 1.0)
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, v), half2v{(_Float16)1.0f, (_Float16)1.0f}, acc, false);
}

template <int NTILE>
constexpr size_t gemm_lds_bytes(int quant) {
    return (size_t)2 * 16 * NTILE * kPitch * sizeof(uint16_t) + (quant == kNf4 ? 256 * sizeof(uint2) : 0);
}

template <int QUANT, typename XT, int NTILE>
__global__ __launch_bounds__(256) void gemm_kernel(const MatmulArgs a) {
    constexpr int BN = 16 * NTILE;
    extern __shared__ __align__(16) uint8_t smem[];
    uint16_t(*xs)[BN * kPitch] = reinterpret_cast<uint16_t(*)[BN * kPitch]>(smem);
    uint2 *pair = reinterpret_cast<uint2 *>(smem + (size_t)2 * BN * kPitch * sizeof(uint16_t));

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t r16 = lane & 15, g = lane >> 4;
    const uint32_t b = blockIdx.z, t0 = blockIdx.y * BN;
    const uint32_t K = a.K;
    const uint32_t row_base = blockIdx.x * 64 + wave * 16;
    const uint32_t row = min(row_base + r16, a.R - 1);       // A-side row of this lane
    const uint32_t frow = min(row_base + 4 * g, a.R - 4);    // first of the 4 D-side rows of this lane
    const uint64_t e_row = ((uint64_t)b * a.R + row) * K;    // flat element index of (row, 0)
    const uint64_t e_frow = ((uint64_t)b * a.R + frow) * K;

    if (QUANT == kNf4) {
        // entry for byte v: (hi(q[v & 15]), hi(q[v >> 4])), (lo(..), lo(..)); lo scaled by 2^11
        const float q0 = a.quant[tid & 15], q1 = a.quant[tid >> 4];
        const float h0 = h2f(f2h(q0)), h1 = h2f(f2h(q1));
        pair[tid] = make_uint2(pack_h2(q0, q1), pack_h2((q0 - h0) * 2048.0f, (q1 - h1) * 2048.0f));
    }

    // activation tile staging: piece p of a tile is 8 consecutive k of one token
    constexpr int NPIECE = NTILE; // pieces per thread: BN * 16 / 256
    const XT *xbase = reinterpret_cast<const XT *>(a.x) + (uint64_t)b * a.x_batch_stride;
    uint4 xreg[NPIECE];
    auto load_tile = [&](uint32_t kb) {
#pragma unroll
        for (int p = 0; p < NPIECE; p++) {
            const uint32_t piece = tid + 256 * p;
            const uint32_t tok = min(t0 + (piece >> 4), a.T - 1);
            const XT *src = xbase + (uint64_t)tok * a.x_token_stride + kb + ((piece & 15) << 3);
            if constexpr (sizeof(XT) == 2) {
                xreg[p] = load128(src);
            } else {
                const uint4 v0 = load128(src), v1 = load128(src + 4);
                xreg[p] = make_uint4(pack_h2(__uint_as_float(v0.x), __uint_as_float(v0.y)),
                                     pack_h2(__uint_as_float(v0.z), __uint_as_float(v0.w)),
                                     pack_h2(__uint_as_float(v1.x), __uint_as_float(v1.y)),
                                     pack_h2(__uint_as_float(v1.z), __uint_as_float(v1.w)));
            }
        }
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int p = 0; p < NPIECE; p++) {
            const uint32_t piece = tid + 256 * p;
            *reinterpret_cast<uint4 *>(&xs[buf][(piece >> 4) * kPitch + ((piece & 15) << 3)]) = xreg[p];
        }
    };

    // packed weights of one step for this lane: int8 2 x 16 B, nf4 2 x 8 B
    uint4 wreg[2];
    auto load_w = [&](uint32_t kb) {
        if (QUANT == kInt8) {
            wreg[0] = load128_stream(a.w + e_row + kb + 16 * g);
            wreg[1] = load128_stream(a.w + e_row + kb + 64 + 16 * g);
        } else {
            const uint8_t *p = a.w + ((e_row + kb) >> 1);
            const uint2 v0 = load64_stream(p + 8 * g);
            const uint2 v1 = load64_stream(p + 32 + 8 * g);
            wreg[0] = make_uint4(v0.x, v0.y, v1.x, v1.y);
        }
    };

    float4v out[NTILE];
#pragma unroll
    for (int n = 0; n < NTILE; n++) out[n] = float4v{0.f, 0.f, 0.f, 0.f};

    load_tile(0);
    load_w(0);
    int buf = 0;
    for (uint32_t kb = 0; kb < K; kb += kStep, buf ^= 1) {
        store_tile(buf);
        __syncthreads();
        uint4 wcur[2] = {wreg[0], wreg[1]};
        // scales of the 4 D-side rows for this step
        float s_row[4], c_row[4], am_row[2][4];
        if (QUANT == kInt8) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t mm = reinterpret_cast<const uint32_t *>(a.scale)[(e_frow + (uint64_t)i * K + kb) >> 7];
                const float mn = h2f((uint16_t)(mm & 0xffffu)), mx = h2f((uint16_t)(mm >> 16));
                s_row[i] = (mx - mn) * (1.0f / 255.0f);
                c_row[i] = fmaf(-1024.0f, s_row[i], mn);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t am2 = *reinterpret_cast<const uint32_t *>(&a.scale[(e_frow + (uint64_t)i * K + kb) >> 6]);
                am_row[0][i] = h2f((uint16_t)(am2 & 0xffffu));
                am_row[1][i] = h2f((uint16_t)(am2 >> 16));
            }
        }
        if (kb + kStep < K) {
            load_tile(kb + kStep);
            load_w(kb + kStep);
        }

        const uint16_t *xt = xs[buf];
        if (QUANT == kInt8) {
            HalfPack A[4];
            const uint32_t w[8] = {wcur[0].x, wcur[0].y, wcur[0].z, wcur[0].w, wcur[1].x, wcur[1].y, wcur[1].z, wcur[1].w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                // 8 weights = dwords 2i, 2i+1 -> f16 codes 1024 + u
                A[i].u[0] = __builtin_amdgcn_perm(0x64646464u, w[2 * i], 0x04010400u);
                A[i].u[1] = __builtin_amdgcn_perm(0x64646464u, w[2 * i], 0x04030402u);
                A[i].u[2] = __builtin_amdgcn_perm(0x64646464u, w[2 * i + 1], 0x04010400u);
                A[i].u[3] = __builtin_amdgcn_perm(0x64646464u, w[2 * i + 1], 0x04030402u);
            }
#pragma unroll
            for (int n = 0; n < NTILE; n++) {
                float4v D = {0.f, 0.f, 0.f, 0.f};
                float sx = 0.0f;
                const uint16_t *xrow = xt + (n * 16 + r16) * kPitch + 16 * g;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    // A[i] covers k = 64 (i / 2) + 16 g + 8 (i % 2) .. + 8
                    HalfPack B;
                    const uint4 v = *reinterpret_cast<const uint4 *>(xrow + 64 * (i >> 1) + 8 * (i & 1));
                    B.u[0] = v.x; B.u[1] = v.y; B.u[2] = v.z; B.u[3] = v.w;
                    sx = dot2_ones(v.x, sx); sx = dot2_ones(v.y, sx);
                    sx = dot2_ones(v.z, sx); sx = dot2_ones(v.w, sx);
                    D = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[i].h, B.h, D, 0, 0, 0);
                }
                // sum over the four k-groups held by lanes l, l^16, l^32, l^48
                sx += __shfl_xor(sx, 16);
                sx += __shfl_xor(sx, 32);
#pragma unroll
                for (int i = 0; i < 4; i++) out[n][i] = fmaf(s_row[i], D[i], fmaf(c_row[i], sx, out[n][i]));
            }
        } else {
            const uint32_t w[4] = {wcur[0].x, wcur[0].y, wcur[0].z, wcur[0].w};
            HalfPack Ah[4], Al[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint2 e = pair[(w[i] >> (8 * j)) & 0xffu];
                    Ah[i].u[j] = e.x;
                    Al[i].u[j] = e.y;
                }
            }
#pragma unroll
            for (int n = 0; n < NTILE; n++) {
                const uint16_t *xrow = xt + (n * 16 + r16) * kPitch + 16 * g;
#pragma unroll
                for (int blk = 0; blk < 2; blk++) {
                    float4v Dh = {0.f, 0.f, 0.f, 0.f}, Dl = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        // dword 2 blk + j covers k = 64 blk + 16 g + 8 j .. + 8
                        HalfPack B;
                        const uint4 v = *reinterpret_cast<const uint4 *>(xrow + 64 * blk + 8 * j);
                        B.u[0] = v.x; B.u[1] = v.y; B.u[2] = v.z; B.u[3] = v.w;
                        Dh = __builtin_amdgcn_mfma_f32_16x16x32_f16(Ah[2 * blk + j].h, B.h, Dh, 0, 0, 0);
                        Dl = __builtin_amdgcn_mfma_f32_16x16x32_f16(Al[2 * blk + j].h, B.h, Dl, 0, 0, 0);
                    }
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        out[n][i] = fmaf(am_row[blk][i], fmaf(Dl[i], 1.0f / 2048.0f, Dh[i]), out[n][i]);
                }
            }
        }
    }

    // D layout of the 16x16 tile: lane holds token column (lane & 15), rows 4 g .. 4 g + 3
    const uint32_t orow = row_base + 4 * g;
#pragma unroll
    for (int n = 0; n < NTILE; n++) {
        const uint32_t t = t0 + n * 16 + r16;
        if (t < a.T && orow < a.R) {
            const uint64_t idx = (uint64_t)b * a.out_batch_stride + (uint64_t)t * a.out_token_stride + orow;
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = act_apply(a.act, out[n][i]);
            if (a.out_f16) {
                *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(a.out) + idx) =
                    make_uint2(pack_h2(v[0], v[1]), pack_h2(v[2], v[3]));
            } else {
                *reinterpret_cast<float4 *>(reinterpret_cast<float *>(a.out) + idx) = make_float4(v[0], v[1], v[2], v[3]);
            }
        }
    }
}

namespace {

template <int QUANT, typename XT, int NTILE>
void launch_one(hipStream_t stream, const MatmulArgs &a) {
    dim3 grid((a.R + 63) / 64, (a.T + 16 * NTILE - 1) / (16 * NTILE), a.B);
    constexpr size_t lds = gemm_lds_bytes<NTILE>(QUANT);
    if (lds > 48 * 1024) {
        // one-time opt-in to more than the default dynamic LDS limit
        static const hipError_t once = hipFuncSetAttribute(
            reinterpret_cast<const void *>(&gemm_kernel<QUANT, XT, NTILE>),
            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        (void)once;
    }
    hipLaunchKernelGGL((gemm_kernel<QUANT, XT, NTILE>), grid, dim3(256), lds, stream, a);
}

template <int QUANT, typename XT>
void launch_ntile(hipStream_t stream, const MatmulArgs &a) {
    if (a.T <= 16)
        launch_one<QUANT, XT, 1>(stream, a);
    else if (a.T <= 32)
        launch_one<QUANT, XT, 2>(stream, a);
    else if (a.T <= 64)
        launch_one<QUANT, XT, 4>(stream, a);
    else
        launch_one<QUANT, XT, 8>(stream, a);
}

} // namespace

// Preconditions (checked by the caller): K % 128 == 0, R % 4 == 0, 16-byte aligned
// activation rows and output rows of 4.
int launch_gemm(hipStream_t stream, Quant quant, int in_f16, const MatmulArgs &a) {
    if (a.R == 0 || a.T == 0 || a.B == 0) return WRQ_OK;
    if (a.B > 65535u) return fail(WRQ_ERR_SIZE, "data size not match: %u vs. %u", a.B, 65535u);
    if (quant == kInt8) {
        if (in_f16)
            launch_ntile<kInt8, __half>(stream, a);
        else
            launch_ntile<kInt8, float>(stream, a);
    } else {
        if (in_f16)
            launch_ntile<kNf4, __half>(stream, a);
        else
            launch_ntile<kNf4, float>(stream, a);
    }
    return check_launch("matmul_mat");
}

} // namespace wrq

// Decode-shaped products on packed weights for gfx950: matmul_vec_int8 / matmul_vec_nf4.
//
// out[t, r] = ACT( sum_k deq(W[r, k]) * x[t, k] )      (src/shaders/matmul_vec_int8.wgsl:57-115,
//                                                        src/shaders/matmul_vec_nf4.wgsl:90-173)
//
// The kernels are HBM-bound: every packed byte is read exactly once with 16-byte
// lane loads (1 KiB per wave instruction, contiguous along a weight row), all loads
// of a lane are issued before the first use, and a workgroup owns ROWS consecutive
// rows so the activation chunk a lane converts to f32 is reused ROWS times.
//
//   int8: 16 weights per lane load lie inside one 128-block, so the affine dequant
//         factors out of the dot product:
//             sum_j (u_j * s + m) * x_j = s * sum_j u_j x_j + m * sum_j x_j
//         with s = (max - min) / 255; one v_cvt_f32_ubyteN + one FMA per weight.
//   nf4:  32 weights per lane load lie inside one 64-block; the 16-entry table sits
//         in LDS (16 consecutive dwords = 16 distinct banks, lanes reading the same
//         entry are a broadcast, so lookups never conflict); absmax scales the
//         32-term partial sum once.
//
// Lanes reduce with DPP inside rows of 16 and readlane across rows, waves through
// one LDS exchange.  Accumulation is f32 throughout.
#include "wrq_device.h"
#include "wrq_host.h"

#include <stdlib.h>

namespace wrq {

template <int ROWS, int TT, int NT>
__device__ __forceinline__ void reduce_and_store(const MatmulArgs &a, float (&acc)[ROWS][TT],
                                                 uint32_t row0, uint32_t t0, uint32_t b) {
    constexpr int NW = NT / kWave;
    __shared__ float red[NW][ROWS * TT];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
#pragma unroll
    for (int r = 0; r < ROWS; r++)
#pragma unroll
        for (int t = 0; t < TT; t++) {
            const float s = wave_sum(acc[r][t]);
            if (NW == 1) {
                acc[r][t] = s;
            } else if (lane == 0) {
                red[wave][t * ROWS + r] = s;
            }
        }
    if (NW > 1) __syncthreads();
    if (tid < ROWS * TT) {
        float s = 0.0f;
        if (NW == 1) {
            // every lane holds all sums; pick this lane's one without dynamic indexing
#pragma unroll
            for (int r = 0; r < ROWS; r++)
#pragma unroll
                for (int t = 0; t < TT; t++)
                    if (tid == (uint32_t)(t * ROWS + r)) s = acc[r][t];
        } else {
#pragma unroll
            for (int w = 0; w < NW; w++) s += red[w][tid];
        }
        const uint32_t r = row0 + tid % ROWS, t = t0 + tid / ROWS;
        if (r < a.R && t < a.T) {
            const uint64_t idx = (uint64_t)b * a.out_batch_stride + (uint64_t)t * a.out_token_stride + r;
            store_out(a.out, a.out_f16, idx, act_apply(a.act, s));
        }
    }
}

template <typename XT, int ROWS, int TT, int NT>
__global__ __launch_bounds__(NT) void gemv_int8_kernel(const MatmulArgs a) {
    const uint32_t tid = threadIdx.x;
    const uint32_t row0 = blockIdx.x * ROWS, t0 = blockIdx.y * TT, b = blockIdx.z;
    const uint32_t K = a.K, nchunk = K >> 4;
    const uint64_t e0 = ((uint64_t)b * a.R + row0) * K; // flat index of element (row0, 0)
    const uint8_t *wbase = a.w + e0;
    const uint32_t *mm = reinterpret_cast<const uint32_t *>(a.scale);
    const XT *xb = reinterpret_cast<const XT *>(a.x) + (uint64_t)b * a.x_batch_stride;
    const uint32_t rows_valid = min((uint32_t)ROWS, a.R - row0);

    float acc[ROWS][TT];
#pragma unroll
    for (int r = 0; r < ROWS; r++)
#pragma unroll
        for (int t = 0; t < TT; t++) acc[r][t] = 0.0f;

    for (uint32_t c = tid; c < nchunk; c += NT) {
        uint4 wv[ROWS];
        uint32_t sc[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            const uint32_t rr = min((uint32_t)r, rows_valid - 1);
            const uint64_t off = (uint64_t)rr * K + ((uint64_t)c << 4);
            wv[r] = load128_stream(wbase + off);
            sc[r] = mm[(e0 + off) >> 7];
        }
#pragma unroll
        for (int t = 0; t < TT; t++) {
            const uint32_t tt = min(t0 + t, a.T - 1);
            float xf[16];
            load_x<XT, 16>(xb + (uint64_t)tt * a.x_token_stride + ((uint64_t)c << 4), xf);
            float sx = 0.0f;
#pragma unroll
            for (int j = 0; j < 16; j++) sx += xf[j];
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                const uint32_t w[4] = {wv[r].x, wv[r].y, wv[r].z, wv[r].w};
                float p = 0.0f;
#pragma unroll
                for (int j = 0; j < 16; j++)
                    p = fmaf((float)((w[j >> 2] >> (8 * (j & 3))) & 0xffu), xf[j], p);
                const float mn = h2f((uint16_t)(sc[r] & 0xffffu));
                const float mx = h2f((uint16_t)(sc[r] >> 16));
                const float s = (mx - mn) * (1.0f / 255.0f);
                acc[r][t] = fmaf(s, p, fmaf(mn, sx, acc[r][t]));
            }
        }
    }
    reduce_and_store<ROWS, TT, NT>(a, acc, row0, t0, b);
}

template <typename XT, int ROWS, int TT, int NT>
__global__ __launch_bounds__(NT) void gemv_nf4_kernel(const MatmulArgs a) {
    __shared__ float q[16];
    const uint32_t tid = threadIdx.x;
    if (tid < 16) q[tid] = a.quant[tid];
    __syncthreads();

    const uint32_t row0 = blockIdx.x * ROWS, t0 = blockIdx.y * TT, b = blockIdx.z;
    const uint32_t K = a.K, nchunk = K >> 5;
    const uint64_t e0 = ((uint64_t)b * a.R + row0) * K; // flat element index of (row0, 0)
    const uint8_t *wbase = a.w + (e0 >> 1);
    const XT *xb = reinterpret_cast<const XT *>(a.x) + (uint64_t)b * a.x_batch_stride;
    const uint32_t rows_valid = min((uint32_t)ROWS, a.R - row0);

    float acc[ROWS][TT];
#pragma unroll
    for (int r = 0; r < ROWS; r++)
#pragma unroll
        for (int t = 0; t < TT; t++) acc[r][t] = 0.0f;

    for (uint32_t c = tid; c < nchunk; c += NT) {
        uint4 wv[ROWS];
        float am[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            const uint32_t rr = min((uint32_t)r, rows_valid - 1);
            const uint64_t off = (uint64_t)rr * K + ((uint64_t)c << 5); // elements
            wv[r] = load128_stream(wbase + (off >> 1));
            am[r] = h2f(a.scale[(e0 + off) >> 6]);
        }
#pragma unroll
        for (int t = 0; t < TT; t++) {
            const uint32_t tt = min(t0 + t, a.T - 1);
            float xf[32];
            load_x<XT, 32>(xb + (uint64_t)tt * a.x_token_stride + ((uint64_t)c << 5), xf);
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                const uint32_t w[4] = {wv[r].x, wv[r].y, wv[r].z, wv[r].w};
                float p = 0.0f;
#pragma unroll
                for (int j = 0; j < 32; j++)
                    p = fmaf(q[(w[j >> 3] >> (4 * (j & 7))) & 0xfu], xf[j], p);
                acc[r][t] = fmaf(p, am[r], acc[r][t]);
            }
        }
    }
    reduce_and_store<ROWS, TT, NT>(a, acc, row0, t0, b);
}

// Any K the reference accepts (K % 4 for int8, K % 8 for nf4, with blocks that may
// straddle rows): one wave per (row, token), scale looked up per group by flat index
// exactly as the shaders do.  Slow path for odd shapes and unaligned views only.
template <typename XT, int QUANT>
__global__ __launch_bounds__(64) void gemv_generic_kernel(const MatmulArgs a) {
    const uint32_t lane = threadIdx.x, row = blockIdx.x, t = blockIdx.y, b = blockIdx.z;
    const uint32_t K = a.K;
    const uint64_t e0 = ((uint64_t)b * a.R + row) * K;
    const XT *x = reinterpret_cast<const XT *>(a.x) + (uint64_t)b * a.x_batch_stride +
                  (uint64_t)t * a.x_token_stride;
    float acc = 0.0f;
    if (QUANT == kInt8) {
        for (uint32_t k = lane * 4; k < K; k += 64 * 4) {
            const uint64_t e = e0 + k;
            const uint32_t w = *reinterpret_cast<const uint32_t *>(a.w + e);
            const float mn = h2f(a.scale[2 * (e >> 7)]), mx = h2f(a.scale[2 * (e >> 7) + 1]);
            const float range = mx - mn;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float u = __fdiv_rn((float)((w >> (8 * j)) & 0xffu), 255.0f);
                acc = fmaf(fmaf(u, range, mn), (float)x[k + j], acc);
            }
        }
    } else {
        float q[16];
#pragma unroll
        for (int j = 0; j < 16; j++) q[j] = a.quant[j];
        for (uint32_t k = lane * 8; k < K; k += 64 * 8) {
            const uint64_t e = e0 + k;
            const uint32_t w = *reinterpret_cast<const uint32_t *>(a.w + (e >> 1));
            const float am = h2f(a.scale[e >> 6]);
            float p = 0.0f;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const uint32_t n = (w >> (4 * j)) & 0xfu;
                float qv = q[0];
#pragma unroll
                for (int i = 1; i < 16; i++) qv = (n == (uint32_t)i) ? q[i] : qv;
                p = fmaf(qv, (float)x[k + j], p);
            }
            acc = fmaf(p, am, acc);
        }
    }
    acc = wave_sum(acc);
    if (lane == 0) {
        const uint64_t idx = (uint64_t)b * a.out_batch_stride + (uint64_t)t * a.out_token_stride + row;
        store_out(a.out, a.out_f16, idx, act_apply(a.act, acc));
    }
}

namespace {

template <typename XT, int ROWS, int TT, int NT>
void launch_fast(hipStream_t stream, Quant quant, const MatmulArgs &a) {
    dim3 grid((a.R + ROWS - 1) / ROWS, (a.T + TT - 1) / TT, a.B);
    if (quant == kInt8)
        hipLaunchKernelGGL((gemv_int8_kernel<XT, ROWS, TT, NT>), grid, dim3(NT), 0, stream, a);
    else
        hipLaunchKernelGGL((gemv_nf4_kernel<XT, ROWS, TT, NT>), grid, dim3(NT), 0, stream, a);
}

template <typename XT, int ROWS, int TT>
void launch_fast_nt(hipStream_t stream, Quant quant, const MatmulArgs &a, int nt) {
    if (nt >= 256)
        launch_fast<XT, ROWS, TT, 256>(stream, quant, a);
    else if (nt >= 128)
        launch_fast<XT, ROWS, TT, 128>(stream, quant, a);
    else
        launch_fast<XT, ROWS, TT, 64>(stream, quant, a);
}

template <typename XT>
void launch_fast_xt(hipStream_t stream, Quant quant, const MatmulArgs &a, int rows, int tt, int nt) {
    if (tt >= 4)
        launch_fast_nt<XT, 4, 4>(stream, quant, a, nt);
    else if (tt == 2)
        launch_fast_nt<XT, 4, 2>(stream, quant, a, nt);
    else if (rows >= 8)
        launch_fast_nt<XT, 8, 1>(stream, quant, a, nt);
    else
        launch_fast_nt<XT, 4, 1>(stream, quant, a, nt);
}

int env_int(const char *name, int fallback) {
    const char *s = getenv(name);
    return (s && *s) ? atoi(s) : fallback;
}

} // namespace

int launch_gemv(hipStream_t stream, Quant quant, int in_f16, const MatmulArgs &a) {
    if (a.R == 0 || a.T == 0 || a.B == 0) return WRQ_OK;
    const uint32_t chunk = quant == kInt8 ? 16 : 32;
    const size_t xs = in_f16 ? 2 : 4;
    const bool aligned = (a.K % chunk == 0) && ((uintptr_t)a.w % 16 == 0) && ((uintptr_t)a.x % 16 == 0) &&
                         ((a.x_token_stride * xs) % 16 == 0) && ((a.x_batch_stride * xs) % 16 == 0);
    if (a.R > 0x7fffffffu || a.T > 65535u || a.B > 65535u)
        return fail(WRQ_ERR_SIZE, "data size not match: %u vs. %u", a.T > a.B ? a.T : a.B, 65535u);
    if (!aligned) {
        dim3 grid(a.R, a.T, a.B);
        if (quant == kInt8) {
            if (in_f16)
                hipLaunchKernelGGL((gemv_generic_kernel<__half, kInt8>), grid, dim3(64), 0, stream, a);
            else
                hipLaunchKernelGGL((gemv_generic_kernel<float, kInt8>), grid, dim3(64), 0, stream, a);
        } else {
            if (in_f16)
                hipLaunchKernelGGL((gemv_generic_kernel<__half, kNf4>), grid, dim3(64), 0, stream, a);
            else
                hipLaunchKernelGGL((gemv_generic_kernel<float, kNf4>), grid, dim3(64), 0, stream, a);
        }
        return check_launch("matmul_vec (generic)");
    }
    const uint32_t nchunk = a.K / chunk;
    // workgroup width: enough lanes to cover a row in one pass, at most 256
    int nt = nchunk >= 256 ? 256 : nchunk >= 128 ? 128 : 64;
    int tt = a.T >= 3 ? 4 : (int)a.T;
    // rows per workgroup: 8 unless that leaves too few workgroups to fill 256 CUs
    int rows = (a.R / 8) * a.B >= 512 ? 8 : 4;
    rows = env_int("WRQ_GEMV_ROWS", rows);
    nt = env_int("WRQ_GEMV_NT", nt);
    if (in_f16)
        launch_fast_xt<__half>(stream, quant, a, rows, tt, nt);
    else
        launch_fast_xt<float>(stream, quant, a, rows, tt, nt);
    return check_launch("matmul_vec");
}

} // namespace wrq

// Decode-shaped products on packed weights for gfx950: matmul_vec_int8 / matmul_vec_nf4.
//
// out[t, r] = ACT( sum_k deq(W[r, k]) * x[t, k] )      (src/shaders/matmul_vec_int8.wgsl:57-115,
//                                                        src/shaders/matmul_vec_nf4.wgsl:90-173)
//
// One launch serves a *group* of up to kMaxGroup independent products (the four
// attention projections of a layer, or ffn.key + ffn.receptance): at batch 1 a single
// 4096 x 4096 product is 17 MB, a few microseconds of HBM time, and a dispatch of its
// own costs about as much again.
//
// Every packed byte is read once, 16 bytes per lane, 1 KiB per wave instruction, contiguous
// along a weight row; accumulation is f32 throughout.  Four kernel families:
//
//   * the wave-owns-rows and K-split kernels (gemv_int8_rows_*_kernel, gemv_int8_ksplit_*_kernel) -- int8 decode with f16
//     activations and K a multiple of 1024, one token or a run of up to 4: a wave streams whole rows (or, for long rows, a
//     1024-element slice of 8 rows) with full-line loads and closes its sums without a workgroup-wide exchange.  Their
//     arguments are scalars that arrive preloaded in SGPRs, for groups the first product's descriptor among them.
//   * one-shot kernels (gemv_int8_oneshot_kernel, gemv_nf4_oneshot_kernel,
//     gemv_fp16_oneshot_kernel) -- the decode path: one token, or a run of up to 4 (int8) /
//     2 (nf4) tokens of f16 activations.  One short-lived workgroup per task (4 or 8 rows over
//     the whole K, one lane per 16-byte chunk of a row) requests everything it needs at once and
//     consumes it in arrival order; thousands of workgroups keep the memory system full.
//     Details stand above each kernel.
//   * the resident kernel (gemv_kernel) -- longer runs that the matrix-core kernel cannot take
//     (K no multiple of 128, f32 activations below 16 tokens): workgroups of 8 waves (two per
//     CU) stage the activation rows of the group in LDS once, then every wave pulls tasks --
//     ROWS consecutive weight rows over the full K -- from a strided sequence, so consecutive
//     tasks land on different CUs; a wave walks its rows in slices of 64 lanes x 16 bytes,
//     loads of slice s+1 in flight while slice s is consumed, and finishes a task with a
//     DPP/readlane reduction: no barrier and no LDS exchange after the prologue.
//       int8: the 16 weights of a lane load lie inside one 128-block, so the affine
//         dequantisation factors out of the dot product,
//             sum_j (u_j s + m) x_j = s sum_j u_j x_j + m sum_j x_j ,  s = (max - min) / 255:
//         one v_cvt_f32_ubyteN and one FMA per weight;
//       nf4: a 256-entry LDS table maps a packed byte to its two f32 table values with one
//         ds_read_b64 (2 address ops + 2 FMA per two weights instead of 4 + 2); each of 32
//         lane groups reads its own copy of the table; absmax scales the 32-term partial sum
//         of a lane load, which lies inside one 64-block.
//   * generic kernels (gemv_generic_kernel, gemv_fp16_generic_kernel) -- any shape the
//     reference accepts (K % 4, blocks straddling rows, unaligned views); correctness path.
#include "wrq_device.h"
#include "wrq_host.h"

namespace wrq {

constexpr int kGemvWaves = 8;                 // waves per workgroup
constexpr int kGemvThreads = kGemvWaves * 64; //
constexpr int kTabCopies = 32;                // nf4 byte-pair table: copies (one per lane & 31), 256 B per entry
constexpr size_t kTabBytes = 256 * kTabCopies * sizeof(float2);
constexpr size_t kGemvLdsBudget = 128 * 1024;

struct GemvProblem {
    const uint8_t *w;      // packed rows of this product
    const uint16_t *scale; // its scale blocks, indexed by flat element index as below
    const float *quant;    // nf4: the 16-entry table of this product
    const void *x;         // first activation row (view offset applied)
    void *out;             // first output row (view offset applied)
    uint64_t e_base;       // flat element index of w's first element inside the matrix (batch offset)
    uint64_t x_token_stride, out_token_stride;
    uint32_t K, R;
    uint32_t x_lds;      // byte offset of this product's activations in LDS
    uint32_t task_begin; // first task of this product
    int out_f16, act;
};

struct GemvGroup {
    // first task of every product, unused entries 0xffffffff: one scalar load finds the product
    // of a task, without a chain of dependent loads at the start of every workgroup
    uint32_t task_begin[kMaxGroup];
    GemvProblem p[kMaxGroup];
    const float *quant;
    uint32_t n, T, total_tasks;
    uint32_t x_pieces; // 16-byte pieces of activations staged in LDS (all products, TT tokens)
};

// What a wave needs to know about the task it is working on (all wave-uniform).
struct TaskCtx;
template <int ROWS, int TT>
__device__ __forceinline__ void finish_task(const TaskCtx &p, float (&acc)[ROWS][TT], uint32_t t0, uint32_t T,
                                            uint32_t lane);


struct TaskCtx {
    uint32_t task, K, R, row0, rows_valid, nslice, x_lds;
    uint64_t e0;           // flat element index of (row0, 0) in the matrix
    const uint8_t *wbase;  // packed bytes of (row0, 0)
    const uint16_t *scale; // scale blocks of the product
    void *out;
    uint64_t out_token_stride;
    int out_f16, act;
};


template <int ROWS, int TT>
__device__ __forceinline__ void finish_task(const TaskCtx &p, float (&acc)[ROWS][TT], uint32_t t0, uint32_t T,
                                            uint32_t lane) {
    float mine = 0.0f;
#pragma unroll
    for (int t = 0; t < TT; t++)
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            const float s = wave_sum(acc[r][t]);
            if (lane == (uint32_t)(t * ROWS + r)) mine = s;
        }
    if (lane < ROWS * TT) {
        const uint32_t r = p.row0 + lane % ROWS, t = t0 + lane / ROWS;
        if (r < p.R && t < T)
            store_out(p.out, p.out_f16, (uint64_t)t * p.out_token_stride + r, act_apply(p.act, mine));
    }
}

template <int QUANT, typename XT, int ROWS, int SL, int TT>
__global__ __launch_bounds__(kGemvThreads) void gemv_kernel(const GemvGroup g) {
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int CH = QUANT == kInt8 ? 16 : 32; // weights per 16-byte lane load
    float2 *tab = reinterpret_cast<float2 *>(smem);
    uint8_t *xs = smem + (QUANT == kNf4 ? kTabBytes : 0);

    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6); // wave-uniform, and known to be
    const uint32_t t0 = blockIdx.y * TT;
    const uint32_t stride = gridDim.x * kGemvWaves;

    auto setup = [&](uint32_t task) {
        TaskCtx c;
        c.task = task;
        uint32_t pi = 0;
#pragma unroll
        for (uint32_t i = 1; i < (uint32_t)kMaxGroup; i++)
            if (task >= g.task_begin[i]) pi = i;
        pi = __builtin_amdgcn_readfirstlane(pi); // uniform: the descriptor is read with scalar loads
        const GemvProblem p = g.p[pi]; // by value: one batch of scalar loads
        c.K = p.K;
        c.R = p.R;
        c.x_lds = p.x_lds;
        c.scale = p.scale;
        c.out = p.out;
        c.out_token_stride = p.out_token_stride;
        c.out_f16 = p.out_f16;
        c.act = p.act;
        c.row0 = (task - p.task_begin) * ROWS;
        c.rows_valid = min((uint32_t)ROWS, c.R - c.row0);
        c.e0 = p.e_base + (uint64_t)c.row0 * c.K;
        c.wbase = p.w + (QUANT == kInt8 ? (uint64_t)c.row0 * c.K : ((uint64_t)c.row0 * c.K) >> 1);
        c.nslice = (c.K + 64 * SL * CH - 1) / (64 * SL * CH);
        return c;
    };
    // 16-byte loads of slice s of a task: ROWS rows x SL chunks per lane, lanes along K (a wave
    // instruction covers 1 KiB of one row); scale blocks beside them
    auto issue = [&](const TaskCtx &c, uint32_t s, uint4(&wdst)[ROWS * SL], uint32_t(&sdst)[ROWS * SL]) {
        const uint16_t *scale = c.scale;
#pragma unroll
        for (int i = 0; i < SL; i++) {
            // lanes past the row end re-read its last chunk
            const uint32_t k0 = min(((s * SL + i) * 64 + lane) * CH, c.K - CH);
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                const uint32_t rr = min((uint32_t)r, c.rows_valid - 1);
                const uint64_t off = (uint64_t)rr * c.K + k0; // elements from (row0, 0)
                if (QUANT == kInt8) {
                    wdst[i * ROWS + r] = load128_stream(c.wbase + off);
                    sdst[i * ROWS + r] = reinterpret_cast<const uint32_t *>(scale)[(c.e0 + off) >> 7];
                } else {
                    wdst[i * ROWS + r] = load128_stream(c.wbase + (off >> 1));
                    sdst[i * ROWS + r] = scale[(c.e0 + off) >> 6];
                }
            }
        }
    };

    // ---- prologue: the first weight slice is requested before anything else so that HBM is
    // busy while the activations of the group (TT tokens) are staged in LDS
    uint4 wa[ROWS * SL], wb[ROWS * SL];
    uint32_t sa[ROWS * SL], sb[ROWS * SL]; // int8: (min, max) pair; nf4: absmax f16 in the low half
    const uint32_t first = blockIdx.x + gridDim.x * wave;
    bool have = first < g.total_tasks;
    TaskCtx cur = setup(have ? first : 0);
    if (have) issue(cur, 0, wa, sa);
    for (uint32_t i = 0; i < g.n; i++) {
        const GemvProblem &p = g.p[i];
        const uint32_t per_row = p.K * sizeof(XT) / 16; // 16-byte pieces per token row
        for (uint32_t j = tid; j < per_row * TT; j += kGemvThreads) {
            const uint32_t t = j / per_row, c = j - t * per_row;
            const uint32_t tt = min(t0 + t, g.T - 1);
            const XT *src = reinterpret_cast<const XT *>(p.x) + (uint64_t)tt * p.x_token_stride;
            *reinterpret_cast<uint4 *>(xs + p.x_lds + (size_t)j * 16) =
                load128(reinterpret_cast<const uint8_t *>(src) + (size_t)c * 16);
        }
    }
    if (QUANT == kNf4) {
        // entry for byte v: (q[v & 15], q[v >> 4]); copy c of the table at tab[v * 32 + c]
        for (uint32_t j = tid; j < 256 * kTabCopies; j += kGemvThreads) {
            const uint32_t v = j / kTabCopies;
            tab[j] = make_float2(g.quant[v & 15], g.quant[v >> 4]);
        }
    }
    lds_barrier();

    // byte address of table entry v for this lane: v * 256 + (lane & 31) * 8, built by one
    // v_perm_b32 from the packed word (entry byte -> address byte 1, lane offset -> byte 0)
    const uint32_t lane_off = (lane & (kTabCopies - 1)) * 8;
    const uint8_t *tabb = reinterpret_cast<const uint8_t *>(tab);

    float acc[ROWS][TT];
#pragma unroll
    for (int r = 0; r < ROWS; r++)
#pragma unroll
        for (int t = 0; t < TT; t++) acc[r][t] = 0.0f;

    // consume slice s of task c from (wv, sc); the last slice of a task reduces and stores
    auto compute = [&](const TaskCtx &c, uint32_t s, const uint4(&wv)[ROWS * SL], const uint32_t(&sc)[ROWS * SL]) {
        const uint32_t K = c.K;
        const XT *xl = reinterpret_cast<const XT *>(xs + c.x_lds);
#pragma unroll
        for (int i = 0; i < SL; i++) {
            const uint32_t k0 = ((s * SL + i) * 64 + lane) * CH;
            if (k0 < K) {
#pragma unroll
                for (int t = 0; t < TT; t++) {
                    float xf[CH];
                    const XT *xp = xl + (size_t)t * K + k0;
                    if constexpr (sizeof(XT) == 2) {
#pragma unroll
                        for (int u = 0; u < CH / 8; u++) unpack8h(*reinterpret_cast<const uint4 *>(xp + 8 * u), xf + 8 * u);
                    } else {
#pragma unroll
                        for (int u = 0; u < CH / 4; u++) {
                            const float4 v = *reinterpret_cast<const float4 *>(xp + 4 * u);
                            xf[4 * u] = v.x; xf[4 * u + 1] = v.y; xf[4 * u + 2] = v.z; xf[4 * u + 3] = v.w;
                        }
                    }
                    if (QUANT == kInt8) {
                        float sx = 0.0f;
#pragma unroll
                        for (int j = 0; j < 16; j++) sx += xf[j];
#pragma unroll
                        for (int r = 0; r < ROWS; r++) {
                            const uint4 &v = wv[i * ROWS + r];
                            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
                            float pr = 0.0f;
#pragma unroll
                            for (int j = 0; j < 16; j++)
                                pr = fmaf((float)((w[j >> 2] >> (8 * (j & 3))) & 0xffu), xf[j], pr);
                            const uint32_t mm = sc[i * ROWS + r];
                            const float mn = h2f((uint16_t)(mm & 0xffffu));
                            const float mx = h2f((uint16_t)(mm >> 16));
                            const float sc1 = (mx - mn) * (1.0f / 255.0f);
                            acc[r][t] = fmaf(sc1, pr, fmaf(mn, sx, acc[r][t]));
                        }
                    } else {
#pragma unroll
                        for (int r = 0; r < ROWS; r++) {
                            const uint4 &v = wv[i * ROWS + r];
                            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
                            float pr = 0.0f;
#pragma unroll
                            for (int j = 0; j < 16; j++) {
                                const uint32_t addr = __builtin_amdgcn_perm(lane_off, w[j >> 2], 0x0c0c0004u | ((j & 3) << 8));
                                const float2 e = *reinterpret_cast<const float2 *>(tabb + addr);
                                pr = fmaf(e.x, xf[2 * j], pr);
                                pr = fmaf(e.y, xf[2 * j + 1], pr);
                            }
                            acc[r][t] = fmaf(pr, h2f((uint16_t)sc[i * ROWS + r]), acc[r][t]);
                        }
                    }
                }
            }
        }
        if (s + 1 == c.nslice) {
            finish_task<ROWS, TT>(c, acc, t0, g.T, lane);
#pragma unroll
            for (int r = 0; r < ROWS; r++)
#pragma unroll
                for (int t = 0; t < TT; t++) acc[r][t] = 0.0f;
        }
    };
    // the step after (c, s): next slice of the task, or slice 0 of this wave's next task;
    // consecutive tasks go to different workgroups first, then to the next wave
    auto advance = [&](TaskCtx &c, uint32_t &s) {
        if (s + 1 < c.nslice) {
            s++;
            return true;
        }
        const uint32_t next = c.task + stride;
        if (next >= g.total_tasks) return false;
        c = setup(next);
        s = 0;
        return true;
    };

    // two register buffers in ping-pong: the loads of step i+1 are in flight while step i is consumed
    uint32_t s = 0;
    while (have) {
        TaskCtx nx = cur;
        uint32_t ns = s;
        const bool nhave = advance(nx, ns);
        if (nhave) issue(nx, ns, wb, sb);
        compute(cur, s, wa, sa);
        if (!nhave) break;
        cur = nx;
        s = ns;
        have = advance(nx, ns);
        if (have) issue(nx, ns, wa, sa);
        compute(cur, s, wb, sb);
        cur = nx;
        s = ns;
    }
}

typedef _Float16 half2v __attribute__((ext_vector_type(2)));

// acc + a.lo * b.lo + a.hi * b.hi on two packed f16 pairs, f32 accumulate (v_dot2_f32_f16)
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, a), __builtin_bit_cast(half2v, b), acc, false);
}

// Sum inside rows of 16 lanes (DPP only); every lane of a row ends with the row's sum.
__device__ __forceinline__ float row_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xf, 0xf, true));  // quad_perm [1,0,3,2]
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xf, 0xf, true));  // quad_perm [2,3,0,1]
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xf, 0xf, true)); // row_half_mirror
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xf, 0xf, true)); // row_mirror
    return v;
}

// End of a one-shot task: lanes reduce inside DPP rows, the NT / 16 row partials of every
// (output row, token) meet in LDS and 16 lanes sum them, again with DPP.
template <int ROWS, int NT, int TT>
__device__ __forceinline__ void oneshot_reduce_store(float (&acc)[ROWS][TT], float (&red)[ROWS * TT][NT / 16], const GemvProblem &p,
                                                     uint32_t row0, uint32_t T) {
    constexpr int NROW16 = NT / 16;
    const uint32_t tid = threadIdx.x;
#pragma unroll
    for (int r = 0; r < ROWS; r++)
#pragma unroll
        for (int t = 0; t < TT; t++) {
            const float s = row_sum(acc[r][t]);
            if ((tid & 15) == 0) red[r * TT + t][tid >> 4] = s;
        }
    __syncthreads();
    const uint32_t l = tid & 15;
    for (uint32_t o = tid >> 4; o < (uint32_t)(ROWS * TT); o += NROW16) {
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < NROW16 / 16; i++) s += red[o][l + 16 * i];
        if (NROW16 < 16) s = l < NROW16 ? red[o][l] : 0.0f;
        s = row_sum(s);
        const uint32_t row = row0 + o / TT, t = o % TT;
        if (l == 0 && row < p.R && t < T) store_out(p.out, p.out_f16, (uint64_t)t * p.out_token_stride + row, act_apply(p.act, s));
    }
}

// int8, one token: one workgroup per task, everything it needs requested at once.  At the
// 7B shapes the whole matrix is a fraction of what the CUs can keep in flight, so a task
// (ROWS rows, NT lanes along K) issues all its loads -- activations first, they are needed
// first and come from L2 -- and consumes the rows in arrival order.
//
// With f16 activations the products run on v_dot2_f32_f16: one v_perm_b32 turns two codes
// into the f16 pair (1024 + u0, 1024 + u1) (exact), the pair meets two activations in one
// dot2, and the bias joins the affine term:
//     sum_j (u_j s + m) x_j = s * sum_j (1024 + u_j) x_j + (m - 1024 s) * sum_j x_j
// -- one VALU op per weight.  f32 activations keep v_cvt_f32_ubyteN + FMA.
// Lanes reduce inside DPP rows; rows and waves meet once in LDS.
// SINGLE: the launch holds one product; its descriptor sits at a fixed place in the kernel
// arguments and is read in the first round of scalar loads.
// TT > 1 (f16 activations only): the same pass serves up to TT tokens of a short run -- the
// converted codes of a row meet the activations of every token, (TT + 1) / 2 VALU ops per weight.
template <typename XT, int ROWS, int NT, bool SINGLE, int TT>
__global__ __launch_bounds__(NT) void gemv_int8_oneshot_kernel(const uint32_t tb1, const uint32_t tb2, const uint32_t tb3, const uint32_t kflags,
                                                               const uint8_t *w0, const uint16_t *scale0, const void *x0, const uint32_t R0,
                                                               const GemvGroup g) {
    // The scalar arguments in front describe the launch's first product (kflags: K in bits 0 .. 23, f16 output in bit 24, the
    // activation in bits 25 .. 27, bit 31: more than four products) and arrive preloaded in SGPRs: the workgroups that open a
    // launch belong to the first product and request their loads without waiting for a scalar load of cold argument memory.
    static_assert(TT == 1 || sizeof(XT) == 2, "several tokens per pass: f16 activations only");
    constexpr int NROW16 = NT / 16; // DPP rows per workgroup
    constexpr int XW = sizeof(XT) == 2 ? 2 : 4; // 16-byte loads per token and chunk
    __shared__ float red[ROWS * TT][NROW16];
    const uint32_t tid = threadIdx.x;
    const uint32_t task = blockIdx.x;
    uint32_t pi = 0;
    if constexpr (!SINGLE) {
        pi = task >= tb1 ? 1u : pi;
        pi = task >= tb2 ? 2u : pi;
        pi = task >= tb3 ? 3u : pi;
        if (kflags >> 31) {
#pragma unroll
            for (uint32_t i = 4; i < (uint32_t)kMaxGroup; i++)
                if (task >= g.task_begin[i]) pi = i;
        }
        pi = __builtin_amdgcn_readfirstlane(pi);
    }
    GemvProblem p;
    if (pi == 0) {
        p = g.p[0]; // the fields not among the scalar arguments (output, token strides) are needed late or not at all
        p.w = w0, p.scale = scale0, p.x = x0;
        p.e_base = 0, p.task_begin = 0;
        p.K = kflags & 0xffffffu, p.R = R0;
        p.out_f16 = (int)((kflags >> 24) & 1u), p.act = (int)((kflags >> 25) & 7u);
    } else {
        p = g.p[pi]; // by value: one batch of scalar loads
    }
    const uint32_t K = p.K, nchunk = K >> 4;
    const uint32_t row0 = (task - p.task_begin) * ROWS;
    const uint32_t rows_valid = min((uint32_t)ROWS, p.R - row0);
    const uint64_t e0 = p.e_base + (uint64_t)row0 * K; // flat index of element (row0, 0)
    const uint8_t *wbase = p.w + (uint64_t)row0 * K;
    const uint32_t *mm = reinterpret_cast<const uint32_t *>(p.scale);
    const XT *x = reinterpret_cast<const XT *>(p.x);

    float acc[ROWS][TT];
#pragma unroll
    for (int r = 0; r < ROWS; r++)
#pragma unroll
        for (int t = 0; t < TT; t++) acc[r][t] = 0.0f;

    for (uint32_t c = tid; c < nchunk; c += NT) {
        uint4 xv[TT][XW];
#pragma unroll
        for (int t = 0; t < TT; t++) {
            const uint32_t tok = TT == 1 ? 0u : min((uint32_t)t, g.T - 1); // tokens past the run repeat the last one
#pragma unroll
            for (int i = 0; i < XW; i++)
                xv[t][i] = load128(reinterpret_cast<const uint8_t *>(x + (uint64_t)tok * p.x_token_stride + ((uint64_t)c << 4)) + 16 * i);
        }
        uint4 wv[ROWS];
        uint32_t sc[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            const uint32_t rr = min((uint32_t)r, rows_valid - 1);
            const uint64_t off = (uint64_t)rr * K + ((uint64_t)c << 4);
            wv[r] = load128_stream(wbase + off);
            sc[r] = mm[(e0 + off) >> 7];
        }
        if constexpr (sizeof(XT) == 2) {
            float sx[TT];
#pragma unroll
            for (int t = 0; t < TT; t++) {
                const uint32_t xd[8] = {xv[t][0].x, xv[t][0].y, xv[t][0].z, xv[t][0].w, xv[t][1].x, xv[t][1].y, xv[t][1].z, xv[t][1].w};
                sx[t] = 0.0f;
#pragma unroll
                for (int j = 0; j < 8; j++) sx[t] = dot2(xd[j], 0x3c003c00u, sx[t]); // (1.0, 1.0)
            }
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                const uint32_t w[4] = {wv[r].x, wv[r].y, wv[r].z, wv[r].w};
                uint32_t code[8]; // f16 pairs (1024 + u0, 1024 + u1)
#pragma unroll
                for (int d = 0; d < 4; d++) {
                    code[2 * d] = __builtin_amdgcn_perm(0x64646464u, w[d], 0x04010400u);
                    code[2 * d + 1] = __builtin_amdgcn_perm(0x64646464u, w[d], 0x04030402u);
                }
                const float mn = h2f((uint16_t)(sc[r] & 0xffffu));
                const float mx = h2f((uint16_t)(sc[r] >> 16));
                const float s = (mx - mn) * (1.0f / 255.0f);
                const float c0 = fmaf(-1024.0f, s, mn);
#pragma unroll
                for (int t = 0; t < TT; t++) {
                    const uint32_t xd[8] = {xv[t][0].x, xv[t][0].y, xv[t][0].z, xv[t][0].w, xv[t][1].x, xv[t][1].y, xv[t][1].z, xv[t][1].w};
                    float pr = 0.0f;
#pragma unroll
                    for (int j = 0; j < 8; j++) pr = dot2(code[j], xd[j], pr);
                    acc[r][t] = fmaf(s, pr, fmaf(c0, sx[t], acc[r][t]));
                }
            }
        } else {
            float xf[16];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                xf[4 * i] = __uint_as_float(xv[0][i].x);
                xf[4 * i + 1] = __uint_as_float(xv[0][i].y);
                xf[4 * i + 2] = __uint_as_float(xv[0][i].z);
                xf[4 * i + 3] = __uint_as_float(xv[0][i].w);
            }
            float sx = 0.0f;
#pragma unroll
            for (int j = 0; j < 16; j++) sx += xf[j];
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                const uint32_t w[4] = {wv[r].x, wv[r].y, wv[r].z, wv[r].w};
                float pr = 0.0f;
#pragma unroll
                for (int j = 0; j < 16; j++) pr = fmaf((float)((w[j >> 2] >> (8 * (j & 3))) & 0xffu), xf[j], pr);
                const float mn = h2f((uint16_t)(sc[r] & 0xffffu));
                const float mx = h2f((uint16_t)(sc[r] >> 16));
                const float s = (mx - mn) * (1.0f / 255.0f);
                acc[r][0] = fmaf(s, pr, fmaf(mn, sx, acc[r][0]));
            }
        }
    }
    oneshot_reduce_store<ROWS, NT, TT>(acc, red, p, row0, g.T);
}

// int8, one token, f16 activations, K = BPL * 1024: a wave owns RW whole rows.
//
// Lane L = (g = L >> 3, sub = L & 7) holds, for j < BPL, the 16 bytes at 128-block g * BPL + j, offset sub * 16 of each of its
// rows: a wave instruction covers 8 full 128-byte lines, and the BPL (min, max) words of a lane's blocks are contiguous -- one
// wide load per row instead of one word load per 16 weight bytes.  The activations reach LDS once per workgroup (4 waves; an
// LDS-only barrier, the weight loads stay in flight across it) and every wave reads the 32 bytes that meet each of its chunks.
// Request order: activations, scale words, weights chunk by chunk; rows are consumed in arrival order.  A row's sum closes
// inside its wave (DPP + readlane): no LDS exchange and no barrier behind the last bytes.
// Workgroups are handed to the 8 XCDs round-robin: tasks are renumbered so that an XCD takes runs of 64 consecutive output
// rows, i.e. whole 128-byte lines of an f16 output, and no output line is dirty in two L2s.
// The scalar arguments come first so that they arrive preloaded in SGPRs (no dependent scalar load in front of the first
// vector load); a single product needs no descriptor load at all.
// STAMP builds (separate kernels behind wrq_debug_stamps, never the ones a product call launches) record four wall-clock
// readings per wave: entry, every load requested, every row accumulated, result stored.
template <int BPL, int RW, bool STAMP = false>
__device__ __forceinline__ void rows_task_int8(const uint8_t *w, const uint32_t *mm, const uint16_t *x, void *out, const uint32_t R,
                                               const int out_f16, const int act, const uint32_t task, uint4 *xs,
                                               unsigned long long *stamps = nullptr) {
    unsigned long long t0 = 0, t1 = 0, t2 = 0;
    if constexpr (STAMP) { t0 = wall_clock64(); __builtin_amdgcn_sched_barrier(0); }
    constexpr int K = BPL * 1024;
    constexpr int XP = (K / 8 + 255) / 256; // 16-byte pieces of the activations per thread
    const uint32_t tid = threadIdx.x, lane = tid & 63, g = lane >> 3, sub = lane & 7;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t row0 = task * (4 * RW) + wave * RW;
    uint4 xp[XP];
#pragma unroll
    for (int i = 0; i < XP; i++) {
        const uint32_t idx = tid + i * 256;
        if (XP * 256 == K / 8 || idx < K / 8) xp[i] = load128(reinterpret_cast<const uint4 *>(x) + idx);
    }
    __builtin_amdgcn_sched_barrier(0);
    uint32_t sc[RW][BPL];
    const uint8_t *wrow[RW];
#pragma unroll
    for (int r = 0; r < RW; r++) {
        const uint32_t row = min(row0 + r, R - 1); // rows past the end repeat the last one and are not stored
        wrow[r] = w + (uint64_t)row * K + (g * BPL) * 128 + sub * 16;
        const uint32_t *sp = mm + (uint64_t)row * (K / 128) + g * BPL;
        if constexpr (BPL % 4 == 0) {
#pragma unroll
            for (int q = 0; q < BPL / 4; q++) {
                const uint4 v = load128(sp + 4 * q);
                sc[r][4 * q] = v.x, sc[r][4 * q + 1] = v.y, sc[r][4 * q + 2] = v.z, sc[r][4 * q + 3] = v.w;
            }
        } else if constexpr (BPL % 2 == 0) {
#pragma unroll
            for (int q = 0; q < BPL / 2; q++) {
                const uint2 v = *reinterpret_cast<const uint2 *>(sp + 2 * q);
                sc[r][2 * q] = v.x, sc[r][2 * q + 1] = v.y;
            }
        } else {
#pragma unroll
            for (int j = 0; j < BPL; j++) sc[r][j] = sp[j];
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    uint4 wv[RW][BPL];
#pragma unroll
    for (int j = 0; j < BPL; j++)
#pragma unroll
        for (int r = 0; r < RW; r++) wv[r][j] = load128_stream(wrow[r] + j * 128);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (STAMP) { t1 = wall_clock64(); __builtin_amdgcn_sched_barrier(0); }
#pragma unroll
    for (int i = 0; i < XP; i++) {
        const uint32_t idx = tid + i * 256;
        if (XP * 256 == K / 8 || idx < K / 8) xs[idx] = xp[i];
    }
    lds_barrier();
    float acc[RW];
#pragma unroll
    for (int r = 0; r < RW; r++) acc[r] = 0.0f;
#pragma unroll
    for (int j = 0; j < BPL; j++) {
        const uint4 x0 = xs[((g * BPL + j) * 8 + sub) * 2], x1 = xs[((g * BPL + j) * 8 + sub) * 2 + 1];
        const uint32_t xd[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
        float sx = 0.0f;
#pragma unroll
        for (int q = 0; q < 8; q++) sx = dot2(xd[q], 0x3c003c00u, sx); // (1.0, 1.0)
#pragma unroll
        for (int r = 0; r < RW; r++) {
            const uint32_t wd[4] = {wv[r][j].x, wv[r][j].y, wv[r][j].z, wv[r][j].w};
            uint32_t code[8]; // f16 pairs (1024 + u0, 1024 + u1)
#pragma unroll
            for (int d = 0; d < 4; d++) {
                code[2 * d] = __builtin_amdgcn_perm(0x64646464u, wd[d], 0x04010400u);
                code[2 * d + 1] = __builtin_amdgcn_perm(0x64646464u, wd[d], 0x04030402u);
            }
            const float mn = h2f((uint16_t)(sc[r][j] & 0xffffu));
            const float mx = h2f((uint16_t)(sc[r][j] >> 16));
            const float s = (mx - mn) * (1.0f / 255.0f);
            const float c0 = fmaf(-1024.0f, s, mn);
            float pr = 0.0f;
#pragma unroll
            for (int q = 0; q < 8; q++) pr = dot2(code[q], xd[q], pr);
            acc[r] = fmaf(s, pr, fmaf(c0, sx, acc[r]));
        }
    }
    if constexpr (STAMP) { __builtin_amdgcn_sched_barrier(0); t2 = wall_clock64(); __builtin_amdgcn_sched_barrier(0); }
    float mine = 0.0f;
#pragma unroll
    for (int r = 0; r < RW; r++) {
        const float s = wave_sum(acc[r]);
        if (lane == (uint32_t)r) mine = s;
    }
    if (lane < (uint32_t)RW && row0 + lane < R) store_out(out, out_f16, row0 + lane, act_apply(act, mine));
    if constexpr (STAMP) {
        __builtin_amdgcn_sched_barrier(0);
        const unsigned long long t3 = wall_clock64();
        if (lane == 0) {
            ulonglong4 *st = reinterpret_cast<ulonglong4 *>(stamps) + (blockIdx.x * 4 + wave);
            *st = ulonglong4{t0, t1, t2, t3};
        }
    }
}

// Runs of `run` consecutive tasks per XCD (workgroup b starts on XCD b % 8); the tail that does not fill 8 runs keeps its numbers.
__device__ __forceinline__ uint32_t xcd_task(uint32_t b, uint32_t total, uint32_t run) {
    const uint32_t full = total / (8 * run) * (8 * run);
    if (b >= full) return b;
    const uint32_t xcd = b & 7, idx = b >> 3;
    return ((idx / run) * 8 + xcd) * run + idx % run;
}

template <int BPL, int RW>
__global__ __launch_bounds__(256) void gemv_int8_rows_single_kernel(const uint8_t *w, const uint32_t *mm, const uint16_t *x, void *out,
                                                                    const uint32_t R, const uint32_t total_tasks, const uint32_t flags) {
    __shared__ uint4 xs[BPL * 128];
    const uint32_t task = xcd_task(blockIdx.x, total_tasks, 16 / RW);
    rows_task_int8<BPL, RW>(w, mm, x, out, R, (int)(flags & 1u), (int)(flags >> 1), task, xs);
}

template <int BPL, int RW>
__global__ __launch_bounds__(256) void gemv_int8_rows_group_kernel(const uint32_t tb1, const uint32_t tb2, const uint32_t tb3, const uint32_t tb4,
                                                                   const uint32_t tb5, const uint32_t tb6, const uint32_t tb7,
                                                                   const uint32_t total_tasks, const GemvGroup g) {
    __shared__ uint4 xs[BPL * 128];
    const uint32_t task = xcd_task(blockIdx.x, total_tasks, 16 / RW);
    uint32_t pi = 0;
    pi = task >= tb1 ? 1u : pi;
    pi = task >= tb2 ? 2u : pi;
    pi = task >= tb3 ? 3u : pi;
    pi = task >= tb4 ? 4u : pi;
    pi = task >= tb5 ? 5u : pi;
    pi = task >= tb6 ? 6u : pi;
    pi = task >= tb7 ? 7u : pi;
    pi = __builtin_amdgcn_readfirstlane(pi);
    const GemvProblem p = g.p[pi]; // by value: one batch of scalar loads
    rows_task_int8<BPL, RW>(p.w, reinterpret_cast<const uint32_t *>(p.scale) + (p.e_base >> 7), reinterpret_cast<const uint16_t *>(p.x), p.out, p.R,
                            p.out_f16, p.act, task - p.task_begin, xs);
}

// Runs of TT tokens on the same layout (tokens past the run repeat the last one and are not stored; built for TT = 2, 3 and 4):
// the activations of all tokens reach LDS once per workgroup, a wave converts the codes of a chunk once and meets every
// token's 32 bytes with them, two rows per wave share each activation read.  Per 16 weight bytes that is 8 permutes
// and 10 TT dot products and fmas; the sums of a chunk's activations are taken once per workgroup while they are staged.
template <int BPL, int RW, int TT>
__device__ __forceinline__ void rows_tokens_task_int8(const uint8_t *w, const uint32_t *mm, const uint16_t *x, const uint64_t x_token_stride,
                                                      void *out, const uint64_t out_token_stride, const uint32_t R, const uint32_t T,
                                                      const int out_f16, const int act, const uint32_t task, uint4 *xs, float *sxs) {
    constexpr int K = BPL * 1024;
    constexpr int PIECES = TT * (K / 8);       // 16-byte pieces of the activations, all tokens
    constexpr int XP = (PIECES + 255) / 256;   // ... per thread
    const uint32_t tid = threadIdx.x, lane = tid & 63, g = lane >> 3, sub = lane & 7;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t row0 = task * (4 * RW) + wave * RW;
    uint4 xp[XP];
#pragma unroll
    for (int i = 0; i < XP; i++) {
        const uint32_t idx = tid + i * 256;
        if (XP * 256 == PIECES || idx < (uint32_t)PIECES) {
            const uint32_t tok = min(idx / (K / 8), T - 1); // tokens past the run repeat the last one
            xp[i] = load128(reinterpret_cast<const uint4 *>(x + (uint64_t)tok * x_token_stride) + idx % (K / 8));
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    uint32_t sc[RW][BPL];
    const uint8_t *wrow[RW];
#pragma unroll
    for (int r = 0; r < RW; r++) {
        const uint32_t row = min(row0 + r, R - 1); // rows past the end repeat the last one and are not stored
        wrow[r] = w + (uint64_t)row * K + (g * BPL) * 128 + sub * 16;
        const uint32_t *sp = mm + (uint64_t)row * (K / 128) + g * BPL;
        if constexpr (BPL % 4 == 0) {
#pragma unroll
            for (int q = 0; q < BPL / 4; q++) {
                const uint4 v = load128(sp + 4 * q);
                sc[r][4 * q] = v.x, sc[r][4 * q + 1] = v.y, sc[r][4 * q + 2] = v.z, sc[r][4 * q + 3] = v.w;
            }
        } else if constexpr (BPL % 2 == 0) {
#pragma unroll
            for (int q = 0; q < BPL / 2; q++) {
                const uint2 v = *reinterpret_cast<const uint2 *>(sp + 2 * q);
                sc[r][2 * q] = v.x, sc[r][2 * q + 1] = v.y;
            }
        } else {
#pragma unroll
            for (int j = 0; j < BPL; j++) sc[r][j] = sp[j];
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    uint4 wv[RW][BPL];
#pragma unroll
    for (int j = 0; j < BPL; j++)
#pragma unroll
        for (int r = 0; r < RW; r++) wv[r][j] = load128_stream(wrow[r] + j * 128);
    __builtin_amdgcn_sched_barrier(0);
    // the sum of a chunk's 16 activations (the offset term of the dequantisation) is taken once per workgroup: a piece is
    // half a chunk, its other half sits in the neighbouring lane
#pragma unroll
    for (int i = 0; i < XP; i++) {
        const uint32_t idx = tid + i * 256;
        if (XP * 256 == PIECES || idx < (uint32_t)PIECES) {
            xs[idx] = xp[i];
            float h = dot2(xp[i].x, 0x3c003c00u, 0.0f); // (1.0, 1.0)
            h = dot2(xp[i].y, 0x3c003c00u, h);
            h = dot2(xp[i].z, 0x3c003c00u, h);
            h = dot2(xp[i].w, 0x3c003c00u, h);
            h += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(h), 0xB1, 0xf, 0xf, true)); // quad_perm [1,0,3,2]
            if ((tid & 1u) == 0) sxs[idx >> 1] = h;
        }
    }
    lds_barrier();
    float acc[RW][TT];
#pragma unroll
    for (int r = 0; r < RW; r++)
#pragma unroll
        for (int t = 0; t < TT; t++) acc[r][t] = 0.0f;
#pragma unroll
    for (int j = 0; j < BPL; j++) {
        uint32_t code[RW][8]; // f16 pairs (1024 + u0, 1024 + u1)
        float s[RW], c0[RW];
#pragma unroll
        for (int r = 0; r < RW; r++) {
            const uint32_t wd[4] = {wv[r][j].x, wv[r][j].y, wv[r][j].z, wv[r][j].w};
#pragma unroll
            for (int d = 0; d < 4; d++) {
                code[r][2 * d] = __builtin_amdgcn_perm(0x64646464u, wd[d], 0x04010400u);
                code[r][2 * d + 1] = __builtin_amdgcn_perm(0x64646464u, wd[d], 0x04030402u);
            }
            const float mn = h2f((uint16_t)(sc[r][j] & 0xffffu));
            const float mx = h2f((uint16_t)(sc[r][j] >> 16));
            s[r] = (mx - mn) * (1.0f / 255.0f);
            c0[r] = fmaf(-1024.0f, s[r], mn);
        }
#pragma unroll
        for (int t = 0; t < TT; t++) {
            const uint4 *xt = xs + t * (K / 8);
            const uint4 x0 = xt[((g * BPL + j) * 8 + sub) * 2], x1 = xt[((g * BPL + j) * 8 + sub) * 2 + 1];
            const uint32_t xd[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
            const float sx = sxs[t * (K / 16) + (g * BPL + j) * 8 + sub];
#pragma unroll
            for (int r = 0; r < RW; r++) {
                float pr = 0.0f;
#pragma unroll
                for (int q = 0; q < 8; q++) pr = dot2(code[r][q], xd[q], pr);
                acc[r][t] = fmaf(s[r], pr, fmaf(c0[r], sx, acc[r][t]));
            }
        }
    }
    float mine = 0.0f;
#pragma unroll
    for (int r = 0; r < RW; r++)
#pragma unroll
        for (int t = 0; t < TT; t++) {
            const float v = wave_sum(acc[r][t]);
            if (lane == (uint32_t)(r * TT + t)) mine = v;
        }
    const uint32_t r = lane / TT, t = lane % TT;
    if (lane < (uint32_t)(RW * TT) && row0 + r < R && t < T) store_out(out, out_f16, (uint64_t)t * out_token_stride + row0 + r, act_apply(act, mine));
}

// tflags: the run's token count in bits 0 .. 7, f16 output of the first product in bit 8, its activation in bits 9 .. 11, bit 31:
// more than four products.  As in the one-token kernel the first product's descriptor comes with the (preloaded) arguments.
template <int BPL, int RW, int TT>
__global__ __launch_bounds__(256) void gemv_int8_rows_tokens_kernel(const uint32_t tb1, const uint32_t tb2, const uint32_t tb3, const uint32_t total_tasks,
                                                                    const uint8_t *w0, const uint32_t *mm0, const uint16_t *x0, const uint32_t R0,
                                                                    const uint32_t tflags, const uint32_t x_token_stride0, const GemvGroup g) {
    __shared__ uint4 xs[TT * BPL * 128];
    __shared__ float sxs[TT * BPL * 64];
    const uint32_t task = xcd_task(blockIdx.x, total_tasks, 16 / RW);
    const uint32_t T = tflags & 0xffu;
    uint32_t pi = 0;
    pi = task >= tb1 ? 1u : pi;
    pi = task >= tb2 ? 2u : pi;
    pi = task >= tb3 ? 3u : pi;
    if (tflags >> 31) {
#pragma unroll
        for (uint32_t i = 4; i < (uint32_t)kMaxGroup; i++)
            if (task >= g.task_begin[i]) pi = i;
    }
    pi = __builtin_amdgcn_readfirstlane(pi);
    if (pi == 0) {
        // the output pointer and its token stride are needed last: their scalar load is in flight all the while
        rows_tokens_task_int8<BPL, RW, TT>(w0, mm0, x0, x_token_stride0, g.p[0].out, g.p[0].out_token_stride, R0, T, (int)((tflags >> 8) & 1u),
                                           (int)((tflags >> 9) & 7u), task, xs, sxs);
    } else {
        const GemvProblem p = g.p[pi]; // by value: one batch of scalar loads
        rows_tokens_task_int8<BPL, RW, TT>(p.w, reinterpret_cast<const uint32_t *>(p.scale) + (p.e_base >> 7), reinterpret_cast<const uint16_t *>(p.x),
                                           p.x_token_stride, p.out, p.out_token_stride, p.R, T, p.out_f16, p.act, task - p.task_begin, xs, sxs);
    }
}

// The same two kernels with wall-clock stamps (one 32-byte record per wave at stamps[(workgroup * 4 + wave) * 4]).
template <int BPL, int RW>
__global__ __launch_bounds__(256) void gemv_int8_rows_single_stamped_kernel(const uint8_t *w, const uint32_t *mm, const uint16_t *x, void *out,
                                                                            const uint32_t R, const uint32_t total_tasks, const uint32_t flags,
                                                                            unsigned long long *stamps) {
    __shared__ uint4 xs[BPL * 128];
    const uint32_t task = xcd_task(blockIdx.x, total_tasks, 16 / RW);
    rows_task_int8<BPL, RW, true>(w, mm, x, out, R, (int)(flags & 1u), (int)(flags >> 1), task, xs, stamps);
}

template <int BPL, int RW>
__global__ __launch_bounds__(256) void gemv_int8_rows_group_stamped_kernel(const uint32_t tb1, const uint32_t tb2, const uint32_t tb3,
                                                                           const uint32_t tb4, const uint32_t tb5, const uint32_t tb6,
                                                                           const uint32_t tb7, const uint32_t total_tasks,
                                                                           unsigned long long *stamps, const GemvGroup g) {
    __shared__ uint4 xs[BPL * 128];
    const uint32_t task = xcd_task(blockIdx.x, total_tasks, 16 / RW);
    uint32_t pi = 0;
    pi = task >= tb1 ? 1u : pi;
    pi = task >= tb2 ? 2u : pi;
    pi = task >= tb3 ? 3u : pi;
    pi = task >= tb4 ? 4u : pi;
    pi = task >= tb5 ? 5u : pi;
    pi = task >= tb6 ? 6u : pi;
    pi = task >= tb7 ? 7u : pi;
    pi = __builtin_amdgcn_readfirstlane(pi);
    const GemvProblem p = g.p[pi];
    rows_task_int8<BPL, RW, true>(p.w, reinterpret_cast<const uint32_t *>(p.scale) + (p.e_base >> 7), reinterpret_cast<const uint16_t *>(p.x), p.out,
                                  p.R, p.out_f16, p.act, task - p.task_begin, xs, stamps);
}

// Groups of up to four products: the descriptor of the FIRST product arrives with the kernel arguments (14 dwords, all preloaded
// in SGPRs), so the workgroups that start a launch -- the first tasks belong to the first product -- issue their loads without
// waiting for a scalar load of cold argument memory (0.35 - 0.45 us, measured as the difference in first-wave start between this
// kernel and the single-product one); workgroups of the other products fetch their descriptor as before, when the machine is busy.
template <int BPL, int RW, bool STAMP>
__device__ __forceinline__ void rows_group4_body(const uint32_t tb1, const uint32_t tb2, const uint32_t tb3, const uint32_t total_tasks,
                                                 const uint8_t *w0, const uint32_t *mm0, const uint16_t *x0, void *out0, const uint32_t R0,
                                                 const uint32_t flags0, const GemvGroup &g, uint4 *xs, unsigned long long *stamps) {
    const uint32_t task = xcd_task(blockIdx.x, total_tasks, 16 / RW);
    uint32_t pi = 0;
    pi = task >= tb1 ? 1u : pi;
    pi = task >= tb2 ? 2u : pi;
    pi = task >= tb3 ? 3u : pi;
    pi = __builtin_amdgcn_readfirstlane(pi);
    if (pi == 0) {
        rows_task_int8<BPL, RW, STAMP>(w0, mm0, x0, out0, R0, (int)(flags0 & 1u), (int)(flags0 >> 1), task, xs, stamps);
    } else {
        const GemvProblem p = g.p[pi]; // by value: one batch of scalar loads
        rows_task_int8<BPL, RW, STAMP>(p.w, reinterpret_cast<const uint32_t *>(p.scale) + (p.e_base >> 7), reinterpret_cast<const uint16_t *>(p.x),
                                       p.out, p.R, p.out_f16, p.act, task - p.task_begin, xs, stamps);
    }
}

template <int BPL, int RW>
__global__ __launch_bounds__(256) void gemv_int8_rows_group4_kernel(const uint32_t tb1, const uint32_t tb2, const uint32_t tb3, const uint32_t total_tasks,
                                                                    const uint8_t *w0, const uint32_t *mm0, const uint16_t *x0, void *out0,
                                                                    const uint32_t R0, const uint32_t flags0, const GemvGroup g) {
    __shared__ uint4 xs[BPL * 128];
    rows_group4_body<BPL, RW, false>(tb1, tb2, tb3, total_tasks, w0, mm0, x0, out0, R0, flags0, g, xs, nullptr);
}

template <int BPL, int RW>
__global__ __launch_bounds__(256) void gemv_int8_rows_group4_stamped_kernel(const uint32_t tb1, const uint32_t tb2, const uint32_t tb3,
                                                                            const uint32_t total_tasks, const uint8_t *w0, const uint32_t *mm0,
                                                                            const uint16_t *x0, void *out0, const uint32_t R0, const uint32_t flags0,
                                                                            unsigned long long *stamps, const GemvGroup g) {
    __shared__ uint4 xs[BPL * 128];
    rows_group4_body<BPL, RW, true>(tb1, tb2, tb3, total_tasks, w0, mm0, x0, out0, R0, flags0, g, xs, stamps);
}

// int8, one token, f16 activations, long rows (K = WK * 1024: 10240, 12288, 14336): the WK waves of a workgroup split K, every wave
// takes all RWG rows of the task over its 1024 elements -- one 16-byte chunk per lane and row, the lane's 16 activations in
// registers for all rows (each activation crosses into the workgroup once, no LDS staging), one (min, max) word per chunk.
// Request order: activations, scale words, weights; rows are consumed in arrival order; the partial sums of the waves meet in
// LDS behind one barrier.  Same task numbering and argument passing as the wave-owns-rows kernel.
template <int RWG, int WK, bool STAMP = false>
__device__ __forceinline__ void ksplit_task_int8(const uint8_t *w, const uint32_t *mm, const uint16_t *x, void *out, const uint32_t R,
                                                 const uint32_t total_tasks, const uint32_t flags, float (*red)[RWG],
                                                 unsigned long long *stamps = nullptr) {
    unsigned long long t0 = 0, t1 = 0, t2 = 0;
    if constexpr (STAMP) { t0 = wall_clock64(); __builtin_amdgcn_sched_barrier(0); }
    constexpr int K = WK * 1024;
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t task = xcd_task(blockIdx.x, total_tasks, 64 / RWG);
    const uint32_t row0 = task * RWG;
    const uint32_t k0 = wave * 1024 + lane * 16; // first element of this lane's chunk
    const uint4 *xp = reinterpret_cast<const uint4 *>(x + k0);
    const uint4 x0 = load128(xp), x1 = load128(xp + 1);
    __builtin_amdgcn_sched_barrier(0);
    uint32_t sc[RWG];
    const uint8_t *wrow[RWG];
#pragma unroll
    for (int r = 0; r < RWG; r++) {
        const uint32_t row = min(row0 + r, R - 1); // rows past the end repeat the last one and are not stored
        wrow[r] = w + (uint64_t)row * K + k0;
        sc[r] = mm[(uint64_t)row * (K / 128) + (k0 >> 7)];
    }
    __builtin_amdgcn_sched_barrier(0);
    uint4 wv[RWG];
#pragma unroll
    for (int r = 0; r < RWG; r++) wv[r] = load128_stream(wrow[r]);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (STAMP) { t1 = wall_clock64(); __builtin_amdgcn_sched_barrier(0); }
    const uint32_t xd[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
    float sx = 0.0f;
#pragma unroll
    for (int q = 0; q < 8; q++) sx = dot2(xd[q], 0x3c003c00u, sx); // (1.0, 1.0)
    float mine = 0.0f;
#pragma unroll
    for (int r = 0; r < RWG; r++) {
        const uint32_t wd[4] = {wv[r].x, wv[r].y, wv[r].z, wv[r].w};
        uint32_t code[8]; // f16 pairs (1024 + u0, 1024 + u1)
#pragma unroll
        for (int d = 0; d < 4; d++) {
            code[2 * d] = __builtin_amdgcn_perm(0x64646464u, wd[d], 0x04010400u);
            code[2 * d + 1] = __builtin_amdgcn_perm(0x64646464u, wd[d], 0x04030402u);
        }
        const float mn = h2f((uint16_t)(sc[r] & 0xffffu));
        const float mx = h2f((uint16_t)(sc[r] >> 16));
        const float s = (mx - mn) * (1.0f / 255.0f);
        const float c0 = fmaf(-1024.0f, s, mn);
        float pr = 0.0f;
#pragma unroll
        for (int q = 0; q < 8; q++) pr = dot2(code[q], xd[q], pr);
        const float sum = wave_sum(fmaf(s, pr, c0 * sx));
        if (lane == (uint32_t)r) mine = sum;
    }
    if constexpr (STAMP) { __builtin_amdgcn_sched_barrier(0); t2 = wall_clock64(); __builtin_amdgcn_sched_barrier(0); }
    if (lane < (uint32_t)RWG) red[wave][lane] = mine;
    __syncthreads();
    if (tid < (uint32_t)RWG) {
        float s = 0.0f;
#pragma unroll
        for (int q = 0; q < WK; q++) s += red[q][tid];
        if (row0 + tid < R) store_out(out, (int)(flags & 1u), row0 + tid, act_apply((int)(flags >> 1), s));
    }
    if constexpr (STAMP) {
        __builtin_amdgcn_sched_barrier(0);
        const unsigned long long t3 = wall_clock64();
        if (lane == 0) {
            ulonglong4 *st = reinterpret_cast<ulonglong4 *>(stamps) + (blockIdx.x * WK + wave);
            *st = ulonglong4{t0, t1, t2, t3};
        }
    }
}

template <int RWG, int WK>
__global__ __launch_bounds__(WK * 64) void gemv_int8_ksplit_kernel(const uint8_t *w, const uint32_t *mm, const uint16_t *x, void *out, const uint32_t R,
                                                                  const uint32_t total_tasks, const uint32_t flags) {
    __shared__ float red[WK][RWG];
    ksplit_task_int8<RWG, WK>(w, mm, x, out, R, total_tasks, flags, red);
}

// Runs of TT tokens on the K-split layout (built for TT = 2, 3 and 4): a lane keeps its 16 activations of every token in registers, converts a
// row's codes once and meets every token with them; the RWG x TT partial sums of a wave close inside DPP rows and meet in LDS.
template <int RWG, int WK, int TT>
__global__ __launch_bounds__(WK * 64) void gemv_int8_ksplit_tokens_kernel(const uint8_t *w, const uint32_t *mm, const uint16_t *x, void *out,
                                                                         const uint32_t R, const uint32_t total_tasks, const uint32_t flags,
                                                                         const uint32_t T, const uint32_t x_token_stride,
                                                                         const uint32_t out_token_stride) {
    constexpr int K = WK * 1024;
    __shared__ float red[RWG * TT][WK * 4]; // per output: one partial sum per DPP row of 16 lanes
    static_assert(RWG * TT * 16 <= WK * 64, "16 lanes per output close the sums");
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t task = xcd_task(blockIdx.x, total_tasks, 64 / RWG);
    const uint32_t row0 = task * RWG;
    const uint32_t k0 = wave * 1024 + lane * 16; // first element of this lane's chunk
    uint4 xv[TT][2];
#pragma unroll
    for (int t = 0; t < TT; t++) {
        const uint32_t tok = min((uint32_t)t, T - 1); // tokens past the run repeat the last one
        const uint4 *xp = reinterpret_cast<const uint4 *>(x + (uint64_t)tok * x_token_stride + k0);
        xv[t][0] = load128(xp), xv[t][1] = load128(xp + 1);
    }
    __builtin_amdgcn_sched_barrier(0);
    uint32_t sc[RWG];
    const uint8_t *wrow[RWG];
#pragma unroll
    for (int r = 0; r < RWG; r++) {
        const uint32_t row = min(row0 + r, R - 1); // rows past the end repeat the last one and are not stored
        wrow[r] = w + (uint64_t)row * K + k0;
        sc[r] = mm[(uint64_t)row * (K / 128) + (k0 >> 7)];
    }
    __builtin_amdgcn_sched_barrier(0);
    uint4 wv[RWG];
#pragma unroll
    for (int r = 0; r < RWG; r++) wv[r] = load128_stream(wrow[r]);
    __builtin_amdgcn_sched_barrier(0);
    float sx[TT];
#pragma unroll
    for (int t = 0; t < TT; t++) {
        const uint32_t xd[8] = {xv[t][0].x, xv[t][0].y, xv[t][0].z, xv[t][0].w, xv[t][1].x, xv[t][1].y, xv[t][1].z, xv[t][1].w};
        sx[t] = 0.0f;
#pragma unroll
        for (int q = 0; q < 8; q++) sx[t] = dot2(xd[q], 0x3c003c00u, sx[t]); // (1.0, 1.0)
    }
#pragma unroll
    for (int r = 0; r < RWG; r++) {
        const uint32_t wd[4] = {wv[r].x, wv[r].y, wv[r].z, wv[r].w};
        uint32_t code[8]; // f16 pairs (1024 + u0, 1024 + u1)
#pragma unroll
        for (int d = 0; d < 4; d++) {
            code[2 * d] = __builtin_amdgcn_perm(0x64646464u, wd[d], 0x04010400u);
            code[2 * d + 1] = __builtin_amdgcn_perm(0x64646464u, wd[d], 0x04030402u);
        }
        const float mn = h2f((uint16_t)(sc[r] & 0xffffu));
        const float mx = h2f((uint16_t)(sc[r] >> 16));
        const float s = (mx - mn) * (1.0f / 255.0f);
        const float c0 = fmaf(-1024.0f, s, mn);
#pragma unroll
        for (int t = 0; t < TT; t++) {
            const uint32_t xd[8] = {xv[t][0].x, xv[t][0].y, xv[t][0].z, xv[t][0].w, xv[t][1].x, xv[t][1].y, xv[t][1].z, xv[t][1].w};
            float pr = 0.0f;
#pragma unroll
            for (int q = 0; q < 8; q++) pr = dot2(code[q], xd[q], pr);
            const float v = row_sum(fmaf(s, pr, c0 * sx[t])); // over the 16 lanes of a DPP row
            if ((lane & 15) == 0) red[r * TT + t][wave * 4 + (lane >> 4)] = v;
        }
    }
    __syncthreads();
    if (tid < (uint32_t)(RWG * TT * 16)) { // whole waves: RWG * TT is a multiple of 4
        const uint32_t o = tid >> 4, l = tid & 15;
        float v = 0.0f;
#pragma unroll
        for (int q = 0; q < (WK * 4 + 15) / 16; q++)
            if (l + 16 * q < (uint32_t)(WK * 4)) v += red[o][l + 16 * q];
        v = row_sum(v);
        const uint32_t r = o / TT, t = o % TT;
        if (l == 0 && row0 + r < R && t < T)
            store_out(out, (int)(flags & 1u), (uint64_t)t * out_token_stride + row0 + r, act_apply((int)(flags >> 1), v));
    }
}

// ... and with wall-clock stamps (one record per wave at stamps[(workgroup * WK + wave) * 4]).
template <int RWG, int WK>
__global__ __launch_bounds__(WK * 64) void gemv_int8_ksplit_stamped_kernel(const uint8_t *w, const uint32_t *mm, const uint16_t *x, void *out,
                                                                          const uint32_t R, const uint32_t total_tasks, const uint32_t flags,
                                                                          unsigned long long *stamps) {
    __shared__ float red[WK][RWG];
    ksplit_task_int8<RWG, WK, true>(w, mm, x, out, R, total_tasks, flags, red, stamps);
}

// nf4, one token: the same one-shot shape (one workgroup per task of ROWS rows, NT lanes along
// K, every load of the task requested up front).  A lane holds 32 weights (16 packed bytes) of
// each row and the 32 activations they meet.  A packed byte is two weights: a 256-entry LDS
// table maps it to both table values at once,
//   f16 activations: as two f16 pairs (hi, lo * 2^11) with hi + lo exact to 2^-22, so that a
//                    byte costs one ds_read_b64 and two v_dot2_f32_f16 against the activation pair;
//   f32 activations: as an f32 pair and two fmas.
// The lookups, not HBM, bound this kernel: a CU sustains about 8 of them per clock.
// TT > 1 (f16 activations only): up to TT tokens of a short run share the pass and its lookups.
template <typename XT, int ROWS, int NT, bool SINGLE, int TT>
__global__ __launch_bounds__(NT) void gemv_nf4_oneshot_kernel(const uint32_t tb1, const uint32_t tb2, const uint32_t tb3, const uint32_t kflags,
                                                              const uint8_t *w0, const uint16_t *scale0, const float *quant0, const void *x0,
                                                              const uint32_t R0, const GemvGroup g) {
    // The scalar arguments in front describe the launch's first product (kflags: K in bits 0 .. 23, f16 output in bit 24, the
    // activation in bits 25 .. 27, bit 31: more than four products) and arrive preloaded in SGPRs: the workgroups that open a
    // launch belong to the first product and request their table values, activations and weights without waiting for a
    // scalar load of cold argument memory first; workgroups of the other products fetch their descriptor, by then from cache.
    static_assert(TT == 1 || sizeof(XT) == 2, "several tokens per pass: f16 activations only");
    constexpr int NROW16 = NT / 16; // DPP rows per workgroup
    constexpr bool F16 = sizeof(XT) == 2;
    __shared__ float red[ROWS * TT][NROW16];
    __shared__ uint2 tab[256];
    const uint32_t tid = threadIdx.x;
    const uint32_t task = blockIdx.x;
    uint32_t pi = 0;
    if constexpr (!SINGLE) {
        pi = task >= tb1 ? 1u : pi;
        pi = task >= tb2 ? 2u : pi;
        pi = task >= tb3 ? 3u : pi;
        if (kflags >> 31) {
#pragma unroll
            for (uint32_t i = 4; i < (uint32_t)kMaxGroup; i++)
                if (task >= g.task_begin[i]) pi = i;
        }
        pi = __builtin_amdgcn_readfirstlane(pi);
    }
    GemvProblem p;
    if (pi == 0) {
        p = g.p[0]; // the fields not among the scalar arguments (output, token strides) are needed late or not at all
        p.w = w0, p.scale = scale0, p.quant = quant0, p.x = x0;
        p.e_base = 0, p.task_begin = 0;
        p.K = kflags & 0xffffffu, p.R = R0;
        p.out_f16 = (int)((kflags >> 24) & 1u), p.act = (int)((kflags >> 25) & 7u);
    } else {
        p = g.p[pi]; // by value: one batch of scalar loads
    }
    const uint32_t K = p.K, nchunk = K >> 5;
    const uint32_t row0 = (task - p.task_begin) * ROWS;
    const uint32_t rows_valid = min((uint32_t)ROWS, p.R - row0);
    const uint64_t e0 = p.e_base + (uint64_t)row0 * K; // flat index of element (row0, 0)
    const uint8_t *wbase = p.w + (((uint64_t)row0 * K) >> 1);
    const XT *x = reinterpret_cast<const XT *>(p.x);

    float acc[ROWS][TT];
#pragma unroll
    for (int r = 0; r < ROWS; r++)
#pragma unroll
        for (int t = 0; t < TT; t++) acc[r][t] = 0.0f;

    // the table values this thread turns into entries: requested before anything else, so that
    // they are back first (loads return in order) and the table is built while the weights arrive
    constexpr int NE = NT >= 256 ? 1 : 256 / NT; // entries per thread
    float tq0[NE], tq1[NE];
#pragma unroll
    for (int e = 0; e < NE; e++) {
        const uint32_t v = (tid + e * NT) & 255u;
        tq0[e] = p.quant[v & 15];
        tq1[e] = p.quant[v >> 4];
    }

    bool table_ready = false;
    for (uint32_t c = tid; c < nchunk || !table_ready; c += NT) {
        const bool live = c < nchunk;
        const uint32_t cc = live ? c : 0; // idle lanes of the first pass repeat chunk 0 and drop it
        constexpr int NX = F16 ? 4 : 8;
        uint4 xv[TT][NX];
#pragma unroll
        for (int t = 0; t < TT; t++) {
            const uint32_t tok = TT == 1 ? 0u : min((uint32_t)t, g.T - 1); // tokens past the run repeat the last one
#pragma unroll
            for (int i = 0; i < NX; i++)
                xv[t][i] = load128(reinterpret_cast<const uint8_t *>(x + (uint64_t)tok * p.x_token_stride + ((uint64_t)cc << 5)) + 16 * i);
        }
        uint4 wv[ROWS];
        uint16_t sc[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            const uint32_t rr = min((uint32_t)r, rows_valid - 1);
            const uint64_t off = (uint64_t)rr * K + ((uint64_t)cc << 5);
            wv[r] = load128_stream(wbase + (off >> 1));
            sc[r] = p.scale[(e0 + off) >> 6];
        }
        if (!table_ready) {
            // built once, behind the loads of the first pass, which stay in flight across the barrier
#pragma unroll
            for (int e = 0; e < NE; e++) {
                const uint32_t v = tid + e * NT;
                const float q0 = tq0[e], q1 = tq1[e];
                if (v < 256) {
                    if constexpr (F16) {
                        const float h0 = h2f(f2h(q0)), h1 = h2f(f2h(q1));
                        tab[v] = make_uint2((uint32_t)f2h(q0) | ((uint32_t)f2h(q1) << 16),
                                            (uint32_t)f2h((q0 - h0) * 2048.0f) | ((uint32_t)f2h((q1 - h1) * 2048.0f) << 16));
                    } else {
                        tab[v] = make_uint2(__float_as_uint(q0), __float_as_uint(q1));
                    }
                }
            }
            lds_barrier();
            table_ready = true;
        }
        if (!live) continue;
        if constexpr (F16) {
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                const uint32_t w[4] = {wv[r].x, wv[r].y, wv[r].z, wv[r].w};
                float ph[TT], pl[TT];
#pragma unroll
                for (int t = 0; t < TT; t++) ph[t] = pl[t] = 0.0f;
#pragma unroll
                for (int j = 0; j < 16; j++) {
                    const uint2 e = tab[(w[j >> 2] >> (8 * (j & 3))) & 0xffu];
#pragma unroll
                    for (int t = 0; t < TT; t++) {
                        const uint4 &xq = xv[t][j >> 2];
                        const uint32_t xd = (j & 3) == 0 ? xq.x : (j & 3) == 1 ? xq.y : (j & 3) == 2 ? xq.z : xq.w;
                        ph[t] = dot2(e.x, xd, ph[t]);
                        pl[t] = dot2(e.y, xd, pl[t]);
                    }
                }
                const float am = h2f(sc[r]);
#pragma unroll
                for (int t = 0; t < TT; t++) acc[r][t] = fmaf(am, fmaf(pl[t], 1.0f / 2048.0f, ph[t]), acc[r][t]);
            }
        } else {
            float xf[32];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                xf[4 * i] = __uint_as_float(xv[0][i].x);
                xf[4 * i + 1] = __uint_as_float(xv[0][i].y);
                xf[4 * i + 2] = __uint_as_float(xv[0][i].z);
                xf[4 * i + 3] = __uint_as_float(xv[0][i].w);
            }
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                const uint32_t w[4] = {wv[r].x, wv[r].y, wv[r].z, wv[r].w};
                float pr = 0.0f;
#pragma unroll
                for (int j = 0; j < 16; j++) {
                    const uint2 e = tab[(w[j >> 2] >> (8 * (j & 3))) & 0xffu];
                    pr = fmaf(__uint_as_float(e.x), xf[2 * j], pr);
                    pr = fmaf(__uint_as_float(e.y), xf[2 * j + 1], pr);
                }
                acc[r][0] = fmaf(h2f(sc[r]), pr, acc[r][0]);
            }
        }
    }
    oneshot_reduce_store<ROWS, NT, TT>(acc, red, p, row0, g.T);
}

// f16 weights, one token (matmul_vec_fp16, src/shaders/matmul_vec_fp16.wgsl:57-120): the same
// one-shot shape without any dequantisation.  A lane holds 8 weights (16 bytes) of each of its
// ROWS rows and the 8 activations they meet; f16 activations go through v_dot2_f32_f16, f32
// activations through converts and fmas.  HBM-bound: 2 bytes per weight.
// TT > 1 (f16 activations only): tokens token .. token + TT - 1 of a short run share the pass.
template <typename XT, int ROWS, int NT, int TT>
__global__ __launch_bounds__(NT) void gemv_fp16_oneshot_kernel(const MatmulArgs a, uint32_t first_token) {
    const uint32_t token = first_token + blockIdx.z * TT; // grid.z: consecutive groups of TT tokens
    static_assert(TT == 1 || sizeof(XT) == 2, "several tokens per pass: f16 activations only");
    constexpr int NROW16 = NT / 16; // DPP rows per workgroup
    constexpr bool F16 = sizeof(XT) == 2;
    __shared__ float red[ROWS * TT][NROW16];
    const uint32_t tid = threadIdx.x;
    const uint32_t b = blockIdx.y;
    const uint32_t K = a.K, nchunk = K >> 3;
    const uint32_t row0 = blockIdx.x * ROWS;
    const uint32_t rows_valid = min((uint32_t)ROWS, a.R - row0);
    const uint16_t *wbase = reinterpret_cast<const uint16_t *>(a.w) + ((uint64_t)b * a.R + row0) * K;
    const XT *x = reinterpret_cast<const XT *>(a.x) + (uint64_t)b * a.x_batch_stride;

    float acc[ROWS][TT];
#pragma unroll
    for (int r = 0; r < ROWS; r++)
#pragma unroll
        for (int t = 0; t < TT; t++) acc[r][t] = 0.0f;

    for (uint32_t c = tid; c < nchunk; c += NT) {
        constexpr int NX = F16 ? 1 : 2;
        uint4 xv[TT][NX];
#pragma unroll
        for (int t = 0; t < TT; t++) {
            const uint32_t tok = min(token + t, a.T - 1); // tokens past the run repeat the last one
#pragma unroll
            for (int i = 0; i < NX; i++)
                xv[t][i] = load128(reinterpret_cast<const uint8_t *>(x + (uint64_t)tok * a.x_token_stride + ((uint64_t)c << 3)) + 16 * i);
        }
        uint4 wv[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            const uint32_t rr = min((uint32_t)r, rows_valid - 1);
            wv[r] = load128_stream(wbase + (uint64_t)rr * K + ((uint64_t)c << 3));
        }
        if constexpr (F16) {
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                const uint32_t w[4] = {wv[r].x, wv[r].y, wv[r].z, wv[r].w};
#pragma unroll
                for (int t = 0; t < TT; t++) {
                    const uint32_t xd[4] = {xv[t][0].x, xv[t][0].y, xv[t][0].z, xv[t][0].w};
#pragma unroll
                    for (int d = 0; d < 4; d++) acc[r][t] = dot2(w[d], xd[d], acc[r][t]);
                }
            }
        } else {
            const float xf[8] = {__uint_as_float(xv[0][0].x), __uint_as_float(xv[0][0].y), __uint_as_float(xv[0][0].z), __uint_as_float(xv[0][0].w),
                                 __uint_as_float(xv[0][1].x), __uint_as_float(xv[0][1].y), __uint_as_float(xv[0][1].z), __uint_as_float(xv[0][1].w)};
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                float wf[8];
                unpack8h(wv[r], wf);
#pragma unroll
                for (int j = 0; j < 8; j++) acc[r][0] = fmaf(wf[j], xf[j], acc[r][0]);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < ROWS; r++)
#pragma unroll
        for (int t = 0; t < TT; t++) {
            const float s = row_sum(acc[r][t]);
            if ((tid & 15) == 0) red[r * TT + t][tid >> 4] = s;
        }
    __syncthreads();
    const uint32_t l = tid & 15;
    for (uint32_t o = tid >> 4; o < (uint32_t)(ROWS * TT); o += NROW16) {
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < NROW16 / 16; i++) s += red[o][l + 16 * i];
        if (NROW16 < 16) s = l < NROW16 ? red[o][l] : 0.0f;
        s = row_sum(s);
        const uint32_t row = row0 + o / TT, t = token + o % TT;
        if (l == 0 && row < a.R && t < a.T)
            store_out(a.out, a.out_f16, (uint64_t)b * a.out_batch_stride + (uint64_t)t * a.out_token_stride + row, act_apply(a.act, s));
    }
}

// f16 weights, any shape the reference accepts (K % 4): one wave per (row, token).
template <typename XT>
__global__ __launch_bounds__(64) void gemv_fp16_generic_kernel(const MatmulArgs a) {
    const uint32_t lane = threadIdx.x, row = blockIdx.x, t = blockIdx.y, b = blockIdx.z;
    const uint32_t K = a.K;
    const uint16_t *w = reinterpret_cast<const uint16_t *>(a.w) + ((uint64_t)b * a.R + row) * K;
    const XT *x = reinterpret_cast<const XT *>(a.x) + (uint64_t)b * a.x_batch_stride + (uint64_t)t * a.x_token_stride;
    float acc = 0.0f;
    for (uint32_t k = lane * 4; k < K; k += 64 * 4) {
#pragma unroll
        for (int j = 0; j < 4; j++) acc = fmaf(h2f(w[k + j]), (float)x[k + j], acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) {
        const uint64_t idx = (uint64_t)b * a.out_batch_stride + (uint64_t)t * a.out_token_stride + row;
        store_out(a.out, a.out_f16, idx, act_apply(a.act, acc));
    }
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

template <int QUANT, typename XT, int ROWS, int SL, int TT>
int launch_group_rt(hipStream_t stream, const GemvGroup &g, uint32_t grid_x, uint32_t grid_y, size_t lds) {
    auto *kern = &gemv_kernel<QUANT, XT, ROWS, SL, TT>;
    if (lds > 48 * 1024) {
        static const hipError_t once = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                           hipFuncAttributeMaxDynamicSharedMemorySize,
                                                           (int)kGemvLdsBudget);
        (void)once;
    }
    hipLaunchKernelGGL(kern, dim3(grid_x, grid_y), dim3(kGemvThreads), lds, stream, g);
    return check_launch("matmul_vec");
}

// (rows per task, chunks per lane and row in one slice): rows * sl 16-byte loads per lane are in
// flight per register buffer, two buffers
template <int QUANT, typename XT>
int launch_group_xt(hipStream_t stream, const GemvGroup &g, int rows, int sl, int tt, uint32_t grid_x,
                    uint32_t grid_y, size_t lds) {
    if (tt == 4) return launch_group_rt<QUANT, XT, 4, 1, 4>(stream, g, grid_x, grid_y, lds);
    if (tt == 2) return launch_group_rt<QUANT, XT, 4, 1, 2>(stream, g, grid_x, grid_y, lds);
    if (rows == 2 && sl == 4) return launch_group_rt<QUANT, XT, 2, 4, 1>(stream, g, grid_x, grid_y, lds);
    if (rows == 2 && sl == 2) return launch_group_rt<QUANT, XT, 2, 2, 1>(stream, g, grid_x, grid_y, lds);
    if (rows == 4 && sl == 2) return launch_group_rt<QUANT, XT, 4, 2, 1>(stream, g, grid_x, grid_y, lds);
    if (rows == 4 && sl == 4) return launch_group_rt<QUANT, XT, 4, 4, 1>(stream, g, grid_x, grid_y, lds);
    if (rows == 2) return launch_group_rt<QUANT, XT, 2, 1, 1>(stream, g, grid_x, grid_y, lds);
    return launch_group_rt<QUANT, XT, 4, 1, 1>(stream, g, grid_x, grid_y, lds);
}

template <typename XT, int ROWS, bool SINGLE, int TT>
int launch_oneshot_nt_n(hipStream_t stream, const GemvGroup &g, int nt) {
    const dim3 grid(g.total_tasks);
    const GemvProblem &p = g.p[0];
    if (p.K > 0xffffffu) return fail(WRQ_ERR_SIZE, "data size not match: %u vs. %u", p.K, 0xffffffu);
    const uint32_t kflags = p.K | ((uint32_t)(p.out_f16 ? 1u : 0u) << 24) | (((uint32_t)p.act & 7u) << 25) | (g.n > 4 ? 0x80000000u : 0u);
#define WRQ_I8_LAUNCH(N, T_) hipLaunchKernelGGL((gemv_int8_oneshot_kernel<XT, ROWS, N, SINGLE, T_>), grid, dim3(N), 0, stream, g.task_begin[1], g.task_begin[2], \
                                                g.task_begin[3], kflags, p.w, p.scale, p.x, p.R, g)
    if (nt >= 1024 && TT == 1)
        WRQ_I8_LAUNCH(1024, 1);
    else if (nt >= 512)
        WRQ_I8_LAUNCH(512, TT);
    else if (nt >= 256)
        WRQ_I8_LAUNCH(256, TT);
    else if (nt >= 128)
        WRQ_I8_LAUNCH(128, TT);
    else
        WRQ_I8_LAUNCH(64, TT);
#undef WRQ_I8_LAUNCH
    return check_launch("matmul_vec_int8");
}

// tt tokens per pass: 1, or 2 / 4 for short runs of f16 activations.  (8 tokens per pass were
// measured slower than the matrix-core kernel: every task re-reads the activations of all tokens
// from L2, four times the weight bytes at 4 rows per task.)
template <typename XT, int ROWS>
int launch_oneshot_nt(hipStream_t stream, const GemvGroup &g, int nt, int tt) {
    if constexpr (sizeof(XT) == 2) {
        if (tt == 4) return launch_oneshot_nt_n<XT, ROWS, false, 4>(stream, g, nt);
        if (tt == 2) return launch_oneshot_nt_n<XT, ROWS, false, 2>(stream, g, nt);
    }
    return g.n == 1 ? launch_oneshot_nt_n<XT, ROWS, true, 1>(stream, g, nt) : launch_oneshot_nt_n<XT, ROWS, false, 1>(stream, g, nt);
}

template <typename XT, int ROWS, bool SINGLE, int TT>
int launch_oneshot_nf4_nt_n(hipStream_t stream, const GemvGroup &g, int nt) {
    const dim3 grid(g.total_tasks);
    const GemvProblem &p = g.p[0];
    if (p.K > 0xffffffu) return fail(WRQ_ERR_SIZE, "data size not match: %u vs. %u", p.K, 0xffffffu);
    const uint32_t kflags = p.K | ((uint32_t)(p.out_f16 ? 1u : 0u) << 24) | (((uint32_t)p.act & 7u) << 25) | (g.n > 4 ? 0x80000000u : 0u);
#define WRQ_NF4_LAUNCH(N) hipLaunchKernelGGL((gemv_nf4_oneshot_kernel<XT, ROWS, N, SINGLE, TT>), grid, dim3(N), 0, stream, g.task_begin[1], g.task_begin[2], \
                                             g.task_begin[3], kflags, p.w, p.scale, p.quant, p.x, p.R, g)
    if (nt >= 512)
        WRQ_NF4_LAUNCH(512);
    else if (nt >= 256)
        WRQ_NF4_LAUNCH(256);
    else if (nt >= 128)
        WRQ_NF4_LAUNCH(128);
    else
        WRQ_NF4_LAUNCH(64);
#undef WRQ_NF4_LAUNCH
    return check_launch("matmul_vec_nf4");
}

template <typename XT, int ROWS>
int launch_oneshot_nf4_nt(hipStream_t stream, const GemvGroup &g, int nt, int tt) {
    if constexpr (sizeof(XT) == 2) {
        if (tt == 2) return launch_oneshot_nf4_nt_n<XT, ROWS, false, 2>(stream, g, nt);
        if constexpr (ROWS == 4) {
            if (tt == 3) return launch_oneshot_nf4_nt_n<XT, ROWS, false, 3>(stream, g, nt);
        }
    }
    return g.n == 1 ? launch_oneshot_nf4_nt_n<XT, ROWS, true, 1>(stream, g, nt) : launch_oneshot_nf4_nt_n<XT, ROWS, false, 1>(stream, g, nt);
}

// Timeline measurements (wrq_debug_stamps): while a stamp buffer is set, the launches of the 7B decode shapes (wave-owns-rows
// at K = 4096, K-split at K = 14336) run their stamped builds, each into the next slot of the buffer.
constexpr uint64_t kStampSlotBytes = 1u << 20; // 32768 records of 32 bytes: enough for 8192 workgroups of 4 waves
unsigned long long *g_stamp_buf = nullptr;
uint64_t g_stamp_slots = 0, g_stamp_next = 0;

unsigned long long *next_stamp_slot(uint32_t records) {
    if (!g_stamp_buf || records * 32ull > kStampSlotBytes) return nullptr;
    const uint64_t slot = g_stamp_next++ % g_stamp_slots;
    return g_stamp_buf + slot * (kStampSlotBytes / 8);
}

} // namespace

int stamps_set(void *buf, uint64_t bytes) {
    if (buf && (bytes < kStampSlotBytes || bytes % kStampSlotBytes != 0))
        return fail(WRQ_ERR_SIZE, "stamp buffer of %llu bytes is not a multiple of %llu", (unsigned long long)bytes,
                    (unsigned long long)kStampSlotBytes);
    g_stamp_buf = static_cast<unsigned long long *>(buf);
    g_stamp_slots = buf ? bytes / kStampSlotBytes : 0;
    g_stamp_next = 0;
    return WRQ_OK;
}

namespace {

template <int BPL, int RW>
int launch_rows_int8(hipStream_t stream, const GemvGroup &g) {
    const dim3 grid(g.total_tasks);
    if constexpr (BPL == 4) {
        if (unsigned long long *st = next_stamp_slot(g.total_tasks * 4)) {
            if (g.n == 1) {
                const GemvProblem &p = g.p[0];
                hipLaunchKernelGGL((gemv_int8_rows_single_stamped_kernel<BPL, RW>), grid, dim3(256), 0, stream, p.w,
                                   reinterpret_cast<const uint32_t *>(p.scale) + (p.e_base >> 7), reinterpret_cast<const uint16_t *>(p.x), p.out,
                                   p.R, g.total_tasks, (uint32_t)(p.out_f16 ? 1u : 0u) | ((uint32_t)p.act << 1), st);
            } else if (g.n <= 4 && tune(kTuneGemvWaveRows, 1) != 3) {
                const GemvProblem &p = g.p[0];
                hipLaunchKernelGGL((gemv_int8_rows_group4_stamped_kernel<BPL, RW>), grid, dim3(256), 0, stream, g.task_begin[1], g.task_begin[2],
                                   g.task_begin[3], g.total_tasks, p.w, reinterpret_cast<const uint32_t *>(p.scale) + (p.e_base >> 7),
                                   reinterpret_cast<const uint16_t *>(p.x), p.out, p.R, (uint32_t)(p.out_f16 ? 1u : 0u) | ((uint32_t)p.act << 1), st, g);
            } else {
                hipLaunchKernelGGL((gemv_int8_rows_group_stamped_kernel<BPL, RW>), grid, dim3(256), 0, stream, g.task_begin[1], g.task_begin[2],
                                   g.task_begin[3], g.task_begin[4], g.task_begin[5], g.task_begin[6], g.task_begin[7], g.total_tasks, st, g);
            }
            return check_launch("matmul_vec_int8");
        }
    }
    if (g.n == 1) {
        const GemvProblem &p = g.p[0];
        hipLaunchKernelGGL((gemv_int8_rows_single_kernel<BPL, RW>), grid, dim3(256), 0, stream, p.w,
                           reinterpret_cast<const uint32_t *>(p.scale) + (p.e_base >> 7), reinterpret_cast<const uint16_t *>(p.x), p.out, p.R,
                           g.total_tasks, (uint32_t)(p.out_f16 ? 1u : 0u) | ((uint32_t)p.act << 1));
    } else if (g.n <= 4 && tune(kTuneGemvWaveRows, 1) != 3) { // (gemv_waverows = 3 keeps every group on the general kernel)
        const GemvProblem &p = g.p[0];
        hipLaunchKernelGGL((gemv_int8_rows_group4_kernel<BPL, RW>), grid, dim3(256), 0, stream, g.task_begin[1], g.task_begin[2], g.task_begin[3],
                           g.total_tasks, p.w, reinterpret_cast<const uint32_t *>(p.scale) + (p.e_base >> 7), reinterpret_cast<const uint16_t *>(p.x),
                           p.out, p.R, (uint32_t)(p.out_f16 ? 1u : 0u) | ((uint32_t)p.act << 1), g);
    } else {
        hipLaunchKernelGGL((gemv_int8_rows_group_kernel<BPL, RW>), grid, dim3(256), 0, stream, g.task_begin[1], g.task_begin[2], g.task_begin[3],
                           g.task_begin[4], g.task_begin[5], g.task_begin[6], g.task_begin[7], g.total_tasks, g);
    }
    return check_launch("matmul_vec_int8");
}

// Rows per wave of the wave-owns-rows kernel: two for short rows (at least four 16-byte loads per lane in flight), else one.
constexpr int rows_per_wave(int bpl) { return bpl <= 2 ? 2 : 1; }

// K / 1024 values the wave-owns-rows kernel is built for.
bool rows_kernel_built(uint32_t K) {
    if (K % 1024 != 0) return false;
    switch (K / 1024) {
    case 1: case 2: case 3: case 4: case 5: case 6: case 7: case 8: case 10: case 12: case 14: case 16: return true;
    default: return false;
    }
}

// ... and those it is used for unless an override says otherwise (gemv_waverows = 2 takes every built one).  Measured against
// the one-shot kernel, cold, one product: 2048 x 2048 2.72 against 3.22 us, 2048 -> 7168 4.40 / 5.07, 7168 -> 2048 4.68 / 5.19,
// 4096 x 4096 4.74 / 5.34, 4096 -> 14336 10.87 / 11.53, 2048 -> 65536 21.4 / 22.4; 14336 -> 4096 12.9 against 12.15: with rows
// that long every wave pulls 28 KiB of activations through LDS for one row, and the one-shot kernel, whose lanes keep
// their slice of the activations in registers for 8 rows, stays ahead.
bool rows_kernel_has(uint32_t K) { return rows_kernel_built(K) && (K <= 8192 || tune(kTuneGemvWaveRows, 1) == 2); }

// Long rows of a single product: the K-split kernel (8 rows per task).
// (K = 16384 would be 16 waves per workgroup: 15.6 us against 13.2 us for the one-shot kernel on 4096 x 16384)
bool ksplit_kernel_has(uint32_t K) { return K == 10240 || K == 12288 || K == 14336; }

template <int WK>
int launch_ksplit_int8(hipStream_t stream, const GemvGroup &g) {
    const GemvProblem &p = g.p[0];
    if constexpr (WK == 14) {
        if (unsigned long long *st = next_stamp_slot(g.total_tasks * WK)) {
            hipLaunchKernelGGL((gemv_int8_ksplit_stamped_kernel<8, WK>), dim3(g.total_tasks), dim3(WK * 64), 0, stream, p.w,
                               reinterpret_cast<const uint32_t *>(p.scale) + (p.e_base >> 7), reinterpret_cast<const uint16_t *>(p.x), p.out, p.R,
                               g.total_tasks, (uint32_t)(p.out_f16 ? 1u : 0u) | ((uint32_t)p.act << 1), st);
            return check_launch("matmul_vec_int8");
        }
    }
    hipLaunchKernelGGL((gemv_int8_ksplit_kernel<8, WK>), dim3(g.total_tasks), dim3(WK * 64), 0, stream, p.w,
                       reinterpret_cast<const uint32_t *>(p.scale) + (p.e_base >> 7), reinterpret_cast<const uint16_t *>(p.x), p.out, p.R, g.total_tasks,
                       (uint32_t)(p.out_f16 ? 1u : 0u) | ((uint32_t)p.act << 1));
    return check_launch("matmul_vec_int8");
}

int launch_ksplit_int8_k(hipStream_t stream, const GemvGroup &g, uint32_t K) {
    switch (K / 1024) {
    case 10: return launch_ksplit_int8<10>(stream, g);
    case 12: return launch_ksplit_int8<12>(stream, g);
    case 14: return launch_ksplit_int8<14>(stream, g);
    default: return fail(WRQ_ERR_UNSUPPORTED, "no K-split kernel for K = %u", K);
    }
}

template <int BPL, int TT>
int launch_rows_tokens_int8(hipStream_t stream, const GemvGroup &g) {
    const GemvProblem &p = g.p[0];
    const uint32_t tflags = (g.T & 0xffu) | ((uint32_t)(p.out_f16 ? 1u : 0u) << 8) | (((uint32_t)p.act & 7u) << 9) | (g.n > 4 ? 0x80000000u : 0u);
    hipLaunchKernelGGL((gemv_int8_rows_tokens_kernel<BPL, 2, TT>), dim3(g.total_tasks), dim3(256), 0, stream, g.task_begin[1], g.task_begin[2],
                       g.task_begin[3], g.total_tasks, p.w, reinterpret_cast<const uint32_t *>(p.scale) + (p.e_base >> 7),
                       reinterpret_cast<const uint16_t *>(p.x), p.R, tflags, (uint32_t)p.x_token_stride, g);
    return check_launch("matmul_vec_int8");
}

// A run of T = 2, 3 or 4 tokens takes T tokens per pass.  7B step against the one-shot kernel: 1.47 / 1.67 / 1.87 ms at 2 / 3 / 4
// tokens against 1.55 / 1.95 / 1.95.  At 4 tokens the activations a workgroup stages equal its weight bytes and a launch is one
// or two rounds of workgroups that load, then compute, in step: memory, LDS and vector time add up instead of overlapping
// (taking the activation sums once per workgroup instead of once per wave removed a quarter of the vector instructions and
// 2.6 % of the time; capping the occupancy to stagger the rounds lost 0 - 5 %; one row per wave at 2 tokens 1.51 against 1.47 ms).
int launch_rows_tokens_int8_k(hipStream_t stream, const GemvGroup &g, uint32_t K) {
    switch (K / 1024) {
#define WRQ_ROWS_CASE(B) case B: return g.T <= 2 ? launch_rows_tokens_int8<B, 2>(stream, g) : g.T == 3 ? launch_rows_tokens_int8<B, 3>(stream, g) : launch_rows_tokens_int8<B, 4>(stream, g);
    WRQ_ROWS_CASE(1) WRQ_ROWS_CASE(2) WRQ_ROWS_CASE(3) WRQ_ROWS_CASE(4) WRQ_ROWS_CASE(5) WRQ_ROWS_CASE(6) WRQ_ROWS_CASE(7) WRQ_ROWS_CASE(8)
#undef WRQ_ROWS_CASE
    default: return fail(WRQ_ERR_UNSUPPORTED, "no wave-owns-rows kernel for K = %u at %u tokens", K, g.T);
    }
}

template <int WK, int TT>
int launch_ksplit_tokens_int8(hipStream_t stream, const GemvGroup &g) {
    const GemvProblem &p = g.p[0];
    hipLaunchKernelGGL((gemv_int8_ksplit_tokens_kernel<8, WK, TT>), dim3(g.total_tasks), dim3(WK * 64), 0, stream, p.w,
                       reinterpret_cast<const uint32_t *>(p.scale) + (p.e_base >> 7), reinterpret_cast<const uint16_t *>(p.x), p.out, p.R,
                       g.total_tasks, (uint32_t)(p.out_f16 ? 1u : 0u) | ((uint32_t)p.act << 1), g.T, (uint32_t)p.x_token_stride,
                       (uint32_t)p.out_token_stride);
    return check_launch("matmul_vec_int8");
}

int launch_ksplit_tokens_int8_k(hipStream_t stream, const GemvGroup &g, uint32_t K) {
    switch (K / 1024) {
    // three tokens only: at two and four the one-shot kernel is faster (see launch_gemv_group)
    case 10: return launch_ksplit_tokens_int8<10, 3>(stream, g);
    case 12: return launch_ksplit_tokens_int8<12, 3>(stream, g);
    case 14: return launch_ksplit_tokens_int8<14, 3>(stream, g);
    default: return fail(WRQ_ERR_UNSUPPORTED, "no K-split kernel for K = %u at %u tokens", K, g.T);
    }
}

int launch_rows_int8_k(hipStream_t stream, const GemvGroup &g, uint32_t K) {
    switch (K / 1024) {
#define WRQ_ROWS_CASE(B) case B: return launch_rows_int8<B, rows_per_wave(B)>(stream, g);
    WRQ_ROWS_CASE(1) WRQ_ROWS_CASE(2) WRQ_ROWS_CASE(3) WRQ_ROWS_CASE(4) WRQ_ROWS_CASE(5) WRQ_ROWS_CASE(6) WRQ_ROWS_CASE(7) WRQ_ROWS_CASE(8)
    WRQ_ROWS_CASE(10) WRQ_ROWS_CASE(12) WRQ_ROWS_CASE(14) WRQ_ROWS_CASE(16)
#undef WRQ_ROWS_CASE
    default: return fail(WRQ_ERR_UNSUPPORTED, "no wave-owns-rows kernel for K = %u", K);
    }
}

bool fast_ok(Quant quant, int in_f16, const MatmulArgs &a) {
    const uint32_t chunk = quant == kInt8 ? 16 : 32;
    const size_t xs = in_f16 ? 2 : 4;
    return (a.K % chunk == 0) && (a.K >= chunk) && ((uintptr_t)a.w % 16 == 0) && ((uintptr_t)a.x % 16 == 0) &&
           ((a.x_token_stride * xs) % 16 == 0) && ((a.x_batch_stride * xs) % 16 == 0);
}

int launch_generic(hipStream_t stream, Quant quant, int in_f16, const MatmulArgs &a) {
    if (a.T > 65535u || a.B > 65535u)
        return fail(WRQ_ERR_SIZE, "data size not match: %u vs. %u", a.T > a.B ? a.T : a.B, 65535u);
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

} // namespace

// Measured task shapes of the one-shot kernels.  web-rwkv_amd/tune_gemm.py (sweep --decode) times lanes per task x rows per
// task for the launches of the RWKV model sizes at 1 .. 4 tokens and writes the fastest, where it beats the rules below by more
// than 4 %, into gemv_tuned.inc; a launch of f16 activations on one batch whose rows and K lie within 7 % of a measured product
// takes that entry.
namespace {
struct TunedDecodeRow {
    uint32_t quant, rows, K;
    uint16_t cfg[4]; // runs of 1, 2, 3, 4 tokens: lanes per task | rows per task << 12; 0: the rules decide
};
const TunedDecodeRow kTunedDecode[] = {
#include "gemv_tuned.inc"
    {~0u, 0u, 0u, {0, 0, 0, 0}}, // end marker
};

uint32_t tuned_decode_lookup(int quant, uint64_t rows, uint64_t K, uint32_t T) {
    if (T < 1 || T > 4 || rows == 0 || K == 0) return 0;
    uint32_t best = 0;
    uint64_t best_d = ~0ull;
    for (const TunedDecodeRow &r : kTunedDecode) {
        if (r.quant != (uint32_t)quant || !r.cfg[T - 1]) continue;
        const uint64_t dr = rows > r.rows ? rows - r.rows : r.rows - rows, dk = K > r.K ? K - r.K : r.K - K;
        if (dr * 100 > (uint64_t)r.rows * 7 || dk * 100 > (uint64_t)r.K * 7) continue;
        const uint64_t d = dr * 1000 / r.rows + dk * 1000 / r.K;
        if (d < best_d) best_d = d, best = r.cfg[T - 1];
    }
    return best;
}
} // namespace

// `n` independent products with the same quantisation, input type and token count.
// Products that do not fit the streaming kernel (odd K, unaligned views, activations too
// large for LDS together) are launched one by one on the generic kernel.
int launch_gemv_group(hipStream_t stream, Quant quant, int in_f16, const MatmulArgs *args, int n) {
    if (n <= 0) return WRQ_OK;
    const uint32_t T = args[0].T;
    const int tt = T >= 3 ? 4 : (int)T;
    const size_t xsz = in_f16 ? 2 : 4;
    const size_t lds_base = quant == kNf4 ? kTabBytes : 0;

    int i = 0;
    while (i < n) {
        GemvGroup g{};
        for (int j = 0; j < kMaxGroup; j++) g.task_begin[j] = 0xffffffffu;
        g.quant = args[i].quant;
        g.T = T;
        size_t lds = lds_base;
        uint32_t tasks = 0;
        // rows per task: 4, or 2 when the group is too small to give every wave of 256 CUs a task
        uint64_t rows_total = 0;
        for (int j = i; j < n; j++) rows_total += (uint64_t)args[j].R * args[j].B;
        // one token or a short run: the one-shot kernels (4 rows per workgroup; 8 once that still gives
        // every CU eight workgroups)
        // up to 8 tokens of f16 activations: the same kernel, several tokens per pass
        // (nf4: 3, with 4 rows per task at 3 tokens -- 7B step 1.87 ms against 2.02 with 8 rows and 2.26 on the matrix-core kernel;
        // at 4 tokens the activations crowd the registers: 2.76 - 3.11 ms against 2.28)
        const bool oneshot = (T == 1 || (in_f16 && T <= (quant == kNf4 ? 3u : 4u))) && tune(kTuneGemvOneshot, 1);
        const int ott = T == 1 ? 1 : T == 2 ? 2 : (quant == kNf4 ? 3 : 4); // tokens per pass of the one-shot kernel
        int rows = tt > 1 ? 4 : (rows_total / 4 >= 256u * 2 * kGemvWaves ? 4 : 2);
        if (oneshot) rows = rows_total / 8 >= 2048u ? 8 : 4;
        // one token of f16 activations on int8 rows of a multiple of 1024: the wave-owns-rows kernel (all products of a launch share K)
        // (runs of 2 .. 4 tokens take the same layouts with all their tokens in one pass; K up to 8192: their activations have to fit LDS)
        const bool tokens_ok = T == 1 || (T <= 4 && tune(kTuneGemvRowsTokens, 1) && args[i].x_token_stride <= 0xffffffffull &&
                                          args[i].out_token_stride <= 0xffffffffull);
        const bool waverows = oneshot && quant == kInt8 && in_f16 && tokens_ok && rows_kernel_has(args[i].K) && (T == 1 || args[i].K <= 8192) &&
                              ((uintptr_t)args[i].scale % 16 == 0) && tune(kTuneGemvWaveRows, 1);
        // ... and long rows (K = 10240, 12288, 14336): the K-split kernel, one product per launch
        // (one and three tokens only: measured against the one-shot kernel on 4096 x 14336, the K-split layout takes 10.9 against
        // 11.9 us at one token but 14.0 / 18.3 against 13.0 / 15.9 us at two / four tokens -- the one-shot kernel has no
        // three-token pass and spends a four-token one there; 7B step 1.47 -> 1.45 ms at two tokens, 1.87 -> 1.81 ms at four)
        const bool ksplit = oneshot && !waverows && quant == kInt8 && in_f16 && tokens_ok && ksplit_kernel_has(args[i].K) && args[i].B == 1 &&
                            (T == 1 || T == 3) && tune(kTuneGemvWaveRows, 1);
        // long rows (ffn.value, K = 14336): 8 rows x 512 lanes, two chunks per lane, measured best
        if (oneshot && quant == kInt8 && args[i].K / 16 > 512) rows = 8;
        // chunks per lane: cover a whole row at once when it is short enough
        const uint32_t groups = (args[i].K / (quant == kInt8 ? 16 : 32) + 63) / 64;
        int sl = groups >= 4 ? 4 : groups >= 2 ? 2 : 1;
        if (rows == 4 && sl == 4) sl = 2;
        rows = tune(kTuneGemvRows, rows);
        sl = tune(kTuneGemvSl, sl);
        if (!oneshot && tt > 1) rows = 4, sl = 1;
        if (oneshot && rows != 8) rows = 4;
        // int8, two tokens per pass: 4 rows per task measured faster than 8 (7B step 1.62 against 1.86 ms;
        // nf4 the other way round, 1.82 against 1.65)
        if (oneshot && quant == kInt8 && ott == 2 && !tune_is_set(kTuneGemvRows)) rows = 4;
        // nf4, two tokens per pass on long rows (more than 128 chunks of 32): 8 rows per task also where the product is small
        // (7B ffn.value 12.4 against 13.8 us, 1.6B ffn.value 5.8 against 6.5 us)
        if (oneshot && quant == kNf4 && ott == 2 && args[i].K / 32 > 128 && !tune_is_set(kTuneGemvRows)) rows = 8;
        uint32_t measured = 0; // lanes | rows << 12 of a measured product of this shape (one-shot kernels only)
        if (oneshot && in_f16 && args[i].B == 1 && !tune_is_set(kTuneGemvRows) && !tune_is_set(kTuneGemvNt) && tune(kTuneGemvTable, 1))
            measured = tuned_decode_lookup(quant, rows_total, args[i].K, T);
        if (measured) rows = (int)(measured >> 12);
        if (oneshot && quant == kNf4 && ott == 3) rows = 4; // three tokens per pass are built for 4 rows per task only
        // 8 rows per task need 128 lanes for the final reduction: short rows keep 4
        if (oneshot && args[i].K / (quant == kInt8 ? 16 : 32) < 128) rows = 4;
        if (waverows) rows = T == 1 ? 4 * rows_per_wave((int)(args[i].K / 1024)) : 8; // several tokens: two rows per wave
        if (ksplit) rows = 8;
        while (i < n && g.n < (uint32_t)kMaxGroup) {
            const MatmulArgs &a = args[i];
            if (a.R == 0 || a.T == 0 || a.B == 0) {
                i++;
                continue;
            }
            const size_t need = oneshot ? 0 : (size_t)a.K * tt * xsz; // LDS for the staged activations
            if (!fast_ok(quant, in_f16, a) || lds_base + need > kGemvLdsBudget) {
                if (g.n) break; // flush what is collected, then come back to this one
                const int s = launch_generic(stream, quant, in_f16, a);
                if (s != WRQ_OK) return s;
                i++;
                continue;
            }
            // the resident kernel builds one table per workgroup: its groups share the table tensor
            if (!oneshot && a.quant != g.quant && g.n) break;
            if (ksplit && g.n) break; // one product per launch
            if (waverows && g.n && (a.K != g.p[0].K || (uintptr_t)a.scale % 16 != 0)) break;
            if (waverows && !g.n && (a.K != args[i].K || !rows_kernel_has(a.K) || (uintptr_t)a.scale % 16 != 0)) break;
            if (a.B > 1 && g.n + a.B > (uint32_t)kMaxGroup && g.n) break;
            if (lds + need * a.B > kGemvLdsBudget && g.n) break;
            // the batch axis unrolls into products of its own
            uint32_t b = 0;
            for (; b < a.B && g.n < (uint32_t)kMaxGroup && lds + need <= kGemvLdsBudget; b++) {
                GemvProblem &p = g.p[g.n++];
                const uint64_t e_base = (uint64_t)b * a.R * a.K;
                p.w = a.w + (quant == kInt8 ? e_base : e_base >> 1);
                p.scale = a.scale;
                p.quant = a.quant;
                p.e_base = e_base;
                p.x = static_cast<const uint8_t *>(a.x) + (uint64_t)b * a.x_batch_stride * xsz;
                p.out = static_cast<uint8_t *>(a.out) + (uint64_t)b * a.out_batch_stride * (a.out_f16 ? 2 : 4);
                p.x_token_stride = a.x_token_stride;
                p.out_token_stride = a.out_token_stride;
                p.K = a.K;
                p.R = a.R;
                p.x_lds = (uint32_t)(lds - lds_base);
                p.task_begin = tasks;
                g.task_begin[g.n - 1] = tasks;
                p.out_f16 = a.out_f16;
                p.act = a.act;
                lds += need;
                tasks += (a.R + rows - 1) / rows;
            }
            if (b < a.B) {
                // a batch too deep for one group: finish it with single-product launches
                for (; b < a.B; b++) {
                    MatmulArgs one = a;
                    const uint64_t e_base = (uint64_t)b * a.R * a.K;
                    // keep flat scale indexing: shift pointers instead of the batch index
                    if ((quant == kInt8 ? e_base % 128 : e_base % 64) != 0) return fail(WRQ_ERR_UNSUPPORTED, "batched matrix rows not block aligned");
                    one.B = 1;
                    one.w = a.w + (quant == kInt8 ? e_base : e_base >> 1);
                    one.scale = a.scale + (quant == kInt8 ? 2 * (e_base >> 7) : (e_base >> 6));
                    one.x = static_cast<const uint8_t *>(a.x) + (uint64_t)b * a.x_batch_stride * xsz;
                    one.out = static_cast<uint8_t *>(a.out) + (uint64_t)b * a.out_batch_stride * (a.out_f16 ? 2 : 4);
                    const int s = launch_gemv_group(stream, quant, in_f16, &one, 1);
                    if (s != WRQ_OK) return s;
                }
            }
            i++;
        }
        if (!g.n) continue;
        g.total_tasks = tasks;
        if (oneshot && quant == kNf4) {
            const uint32_t nchunk = g.p[0].K / 32;
            // a row in one pass where a workgroup can hold its chunks (idle lanes cost less than a second pass)
            int nt = nchunk > 256 ? 512 : nchunk > 128 ? 256 : nchunk > 64 ? 128 : 64;
            if (ott == 3 && nt == 512) nt = 256; // three tokens per pass: two passes of 256 lanes beat one of 512 (7B ffn.value 15.4 against 16.8 us)
            if (measured) nt = (int)(measured & 0xfffu);
            nt = tune(kTuneGemvNt, nt);
            if (nt > 512) nt = 512;
            if (rows == 8 && nt < 128) nt = 128; // the tasks were cut for 8 rows
            int s1;
            if (rows == 8 && nt >= 128)
                s1 = in_f16 ? launch_oneshot_nf4_nt<__half, 8>(stream, g, nt, ott) : launch_oneshot_nf4_nt<float, 8>(stream, g, nt, ott);
            else
                s1 = in_f16 ? launch_oneshot_nf4_nt<__half, 4>(stream, g, nt, ott) : launch_oneshot_nf4_nt<float, 4>(stream, g, nt, ott);
            if (s1 != WRQ_OK) return s1;
            continue;
        }
        if (ksplit && g.n == 1 && ksplit_kernel_has(g.p[0].K) && rows == 8) {
            const int s1 = T == 1 ? launch_ksplit_int8_k(stream, g, g.p[0].K) : launch_ksplit_tokens_int8_k(stream, g, g.p[0].K);
            if (s1 != WRQ_OK) return s1;
            continue;
        }
        if (waverows && rows_kernel_has(g.p[0].K) && T > 1 && rows == 8) {
            const int s1 = launch_rows_tokens_int8_k(stream, g, g.p[0].K);
            if (s1 != WRQ_OK) return s1;
            continue;
        }
        if (waverows && rows_kernel_has(g.p[0].K) && T == 1 && rows == 4 * rows_per_wave((int)(g.p[0].K / 1024))) {
            const int s1 = launch_rows_int8_k(stream, g, g.p[0].K);
            if (s1 != WRQ_OK) return s1;
            continue;
        }
        if (oneshot) {
            const uint32_t nchunk = g.p[0].K / 16;
            // one lane per 16-byte chunk of a row where a workgroup can hold that many
            // (the smallest workgroup that takes a row in one pass: 160 chunks on 256 lanes beat two passes of 128 lanes)
            int nt = nchunk > 256 ? 512 : nchunk > 128 ? 256 : nchunk > 64 ? 128 : 64;
            if (measured) nt = (int)(measured & 0xfffu);
            nt = tune(kTuneGemvNt, nt);
            if (rows == 8 && nt < 128) nt = 128; // the tasks were cut for 8 rows
            int s1;
            if (rows == 8 && nt >= 128) // the final reduction uses 16 lanes per output row
                s1 = in_f16 ? launch_oneshot_nt<__half, 8>(stream, g, nt, ott) : launch_oneshot_nt<float, 8>(stream, g, nt, ott);
            else
                s1 = in_f16 ? launch_oneshot_nt<__half, 4>(stream, g, nt, ott) : launch_oneshot_nt<float, 4>(stream, g, nt, ott);
            if (s1 != WRQ_OK) return s1;
            continue;
        }
        g.x_pieces = (uint32_t)((lds - lds_base) / 16);
        const uint32_t want = (tasks + kGemvWaves - 1) / kGemvWaves;
        const uint32_t cap = quant == kNf4 ? 256u : 512u; // resident workgroups: the nf4 table leaves LDS for one per CU
        uint32_t grid_x = want < cap ? want : cap;
        grid_x = (uint32_t)tune(kTuneGemvGrid, (int)grid_x);
        const uint32_t grid_y = (T + tt - 1) / tt;
        if (grid_y > 65535u) return fail(WRQ_ERR_SIZE, "data size not match: %u vs. %u", T, 65535u * 4);
        int s;
        if (quant == kInt8)
            s = in_f16 ? launch_group_xt<kInt8, __half>(stream, g, rows, sl, tt, grid_x, grid_y, lds)
                       : launch_group_xt<kInt8, float>(stream, g, rows, sl, tt, grid_x, grid_y, lds);
        else
            s = in_f16 ? launch_group_xt<kNf4, __half>(stream, g, rows, sl, tt, grid_x, grid_y, lds)
                       : launch_group_xt<kNf4, float>(stream, g, rows, sl, tt, grid_x, grid_y, lds);
        if (s != WRQ_OK) return s;
    }
    return WRQ_OK;
}

// f16 weights with short rows (K <= 128: the low-rank adapters of a layer) over a run of tokens: a
// thread keeps one weight row in registers and meets TCH tokens, whose activations the workgroup
// stages in LDS once (broadcast reads); outputs of a token are consecutive over the threads.  The
// one-shot kernel above spends a workgroup of 128 lanes on 4 - 16 sixteen-byte chunks of such a row.
template <typename XT, int KV, int TCH>
__global__ __launch_bounds__(256) void gemv_fp16_thin_kernel(const MatmulArgs a) {
    __shared__ __align__(16) uint16_t xs[TCH][8 * KV]; // KV = K / 8 sixteen-byte chunks per row
    const uint32_t tid = threadIdx.x, b = blockIdx.z;
    const uint32_t row = blockIdx.x * 256 + tid, t0 = blockIdx.y * TCH;
    const uint32_t nt = min((uint32_t)TCH, a.T - t0);
    const XT *x = reinterpret_cast<const XT *>(a.x) + (uint64_t)b * a.x_batch_stride;
    for (uint32_t e = tid; e < nt * KV; e += 256) {
        const uint32_t t = e / KV, c = e % KV;
        const XT *src = x + (uint64_t)(t0 + t) * a.x_token_stride + 8 * c;
        uint4 v;
        if constexpr (sizeof(XT) == 2) {
            v = load128(src);
        } else {
            const uint4 v0 = load128(src), v1 = load128(src + 4);
            v = make_uint4((uint32_t)f2h(__uint_as_float(v0.x)) | ((uint32_t)f2h(__uint_as_float(v0.y)) << 16),
                           (uint32_t)f2h(__uint_as_float(v0.z)) | ((uint32_t)f2h(__uint_as_float(v0.w)) << 16),
                           (uint32_t)f2h(__uint_as_float(v1.x)) | ((uint32_t)f2h(__uint_as_float(v1.y)) << 16),
                           (uint32_t)f2h(__uint_as_float(v1.z)) | ((uint32_t)f2h(__uint_as_float(v1.w)) << 16));
        }
        *reinterpret_cast<uint4 *>(&xs[t][8 * c]) = v;
    }
    uint4 w[KV];
    const uint32_t r = min(row, a.R - 1);
    const uint16_t *wrow = reinterpret_cast<const uint16_t *>(a.w) + ((uint64_t)b * a.R + r) * (8 * KV);
#pragma unroll
    for (int c = 0; c < KV; c++) w[c] = load128(wrow + 8 * c);
    __syncthreads();
    if (row >= a.R) return;
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    for (uint32_t t = 0; t < nt; t++) {
        float acc = 0.0f;
#pragma unroll
        for (int c = 0; c < KV; c++) {
            const uint4 xv = *reinterpret_cast<const uint4 *>(&xs[t][8 * c]);
            acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, w[c].x), __builtin_bit_cast(h2, xv.x), acc, false);
            acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, w[c].y), __builtin_bit_cast(h2, xv.y), acc, false);
            acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, w[c].z), __builtin_bit_cast(h2, xv.z), acc, false);
            acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, w[c].w), __builtin_bit_cast(h2, xv.w), acc, false);
        }
        store_out(a.out, a.out_f16, (uint64_t)b * a.out_batch_stride + (uint64_t)(t0 + t) * a.out_token_stride + row, act_apply(a.act, acc));
    }
}

template <typename XT, int KV>
void launch_fp16_thin(hipStream_t stream, const MatmulArgs &a) {
    constexpr int TCH = 16;
    const dim3 grid((a.R + 255) / 256, (a.T + TCH - 1) / TCH, a.B);
    hipLaunchKernelGGL((gemv_fp16_thin_kernel<XT, KV, TCH>), grid, dim3(256), 0, stream, a);
}

template <typename XT, int ROWS, int TT>
void launch_fp16_nt(hipStream_t stream, const MatmulArgs &a, uint32_t token, int nt, uint32_t groups = 1) {
    const dim3 grid((a.R + ROWS - 1) / ROWS, a.B, groups);
    if (nt >= 512)
        hipLaunchKernelGGL((gemv_fp16_oneshot_kernel<XT, ROWS, 512, TT>), grid, dim3(512), 0, stream, a, token);
    else if (nt >= 256)
        hipLaunchKernelGGL((gemv_fp16_oneshot_kernel<XT, ROWS, 256, TT>), grid, dim3(256), 0, stream, a, token);
    else
        hipLaunchKernelGGL((gemv_fp16_oneshot_kernel<XT, ROWS, 128, TT>), grid, dim3(128), 0, stream, a, token);
}

// f16 weights, decode-shaped: one pass over the weights per 1 - 4 tokens (the chunk kernel takes
// the longer runs); odd shapes and unaligned views go to the generic kernel.
int launch_gemv_fp16(hipStream_t stream, int in_f16, const MatmulArgs &a) {
    if (a.R == 0 || a.T == 0 || a.B == 0) return WRQ_OK;
    if (a.T > 65535u || a.B > 65535u) return fail(WRQ_ERR_SIZE, "data size not match: %u vs. %u", a.T > a.B ? a.T : a.B, 65535u);
    const size_t xs = in_f16 ? 2 : 4;
    const bool fast = (a.K % 8 == 0) && (a.K >= 8) && ((uintptr_t)a.w % 16 == 0) && ((uintptr_t)a.x % 16 == 0) &&
                      ((a.x_token_stride * xs) % 16 == 0) && ((a.x_batch_stride * xs) % 16 == 0);
    if (!fast) {
        const dim3 grid(a.R, a.T, a.B);
        if (in_f16)
            hipLaunchKernelGGL((gemv_fp16_generic_kernel<__half>), grid, dim3(64), 0, stream, a);
        else
            hipLaunchKernelGGL((gemv_fp16_generic_kernel<float>), grid, dim3(64), 0, stream, a);
        return check_launch("matmul_vec_fp16 (generic)");
    }
    const uint32_t nchunk = a.K / 8;
    if (a.T >= 4 && (a.K == 32 || a.K == 64 || a.K == 128) && a.T <= 65535u * 16u) {
        // short rows over a run (the adapters' second halves): the thin kernel
        switch (a.K) {
        case 32: in_f16 ? launch_fp16_thin<__half, 4>(stream, a) : launch_fp16_thin<float, 4>(stream, a); break;
        case 64: in_f16 ? launch_fp16_thin<__half, 8>(stream, a) : launch_fp16_thin<float, 8>(stream, a); break;
        default: in_f16 ? launch_fp16_thin<__half, 16>(stream, a) : launch_fp16_thin<float, 16>(stream, a); break;
        }
        return check_launch("matmul_vec_fp16 (short rows)");
    }
    const int nt = nchunk > 256 ? 512 : nchunk > 128 ? 256 : 128;
    const bool rows8 = (uint64_t)a.R * a.B / 8 >= 2048u;
    // f16 activations: up to 4 tokens per pass over the weights; f32: one
    for (uint32_t t = 0; t < a.T;) {
        const uint32_t left = a.T - t;
        if (in_f16 && left >= 4) {
            // whole groups of 4 tokens in one launch (long runs come here when K rules out the matrix cores)
            const uint32_t groups = left / 4;
            if (rows8) launch_fp16_nt<__half, 8, 4>(stream, a, t, nt, groups); else launch_fp16_nt<__half, 4, 4>(stream, a, t, nt, groups);
            t += 4 * groups;
        } else if (in_f16 && left == 3) {
            if (rows8) launch_fp16_nt<__half, 8, 4>(stream, a, t, nt); else launch_fp16_nt<__half, 4, 4>(stream, a, t, nt);
            t += 4;
        } else if (in_f16 && left == 2) {
            if (rows8) launch_fp16_nt<__half, 8, 2>(stream, a, t, nt); else launch_fp16_nt<__half, 4, 2>(stream, a, t, nt);
            t += 2;
        } else {
            if (rows8) {
                if (in_f16) launch_fp16_nt<__half, 8, 1>(stream, a, t, nt); else launch_fp16_nt<float, 8, 1>(stream, a, t, nt);
            } else {
                if (in_f16) launch_fp16_nt<__half, 4, 1>(stream, a, t, nt); else launch_fp16_nt<float, 4, 1>(stream, a, t, nt);
            }
            t += 1;
        }
    }
    return check_launch("matmul_vec_fp16");
}

int launch_gemv(hipStream_t stream, Quant quant, int in_f16, const MatmulArgs &a) {
    return launch_gemv_group(stream, quant, in_f16, &a, 1);
}

} // namespace wrq

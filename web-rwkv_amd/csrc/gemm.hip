// Chunk-shaped products on packed weights for gfx950: matmul_mat_int8 / matmul_mat_nf4
// on the f16 matrix cores (v_mfma_f32_16x16x32_f16, f32 accumulate).
//
// out[t, r] = ACT( sum_k deq(W[r, k]) * x[t, k] )      (src/shaders/matmul_mat_int8.wgsl:62-153,
//                                                        src/shaders/matmul_mat_nf4.wgsl:94-220)
//
// The shapes of this path are skinny: 16..256 tokens against thousands of weight rows, so
// even the chunk products are bound by streaming the packed weights once (below ~100
// tokens) or sit close to that point.  The decomposition follows from it:
//   * a workgroup (4 waves) owns 64*MRT/KG weight rows x 16*NTILE tokens x one K range; a wave
//     owns MRT row tiles of 16 as the MFMA "A" side, and with KG > 1 the waves form KG groups
//     that share rows and activations and take alternate K steps (summed through LDS at the
//     end): small grids get about two workgroups per CU from that instead of from a split
//     of K over the grid.  Weight bytes go from HBM straight
//     into registers of the one wave that uses them (each byte is read once and never
//     shared, an LDS tile for them would only add traffic); the activation tile, shared by
//     the four waves, is staged as f16 in double-buffered LDS, several K steps per barrier
//     for narrow token tiles, and read back as "B" operands with ds_read_b128, each B
//     operand serving MRT MFMAs;
//   * weights are prefetched NBUF K steps ahead through a ring of register buffers, the
//     next activation stage sits in registers while the current one is consumed from LDS;
//   * token tiles up to 64 wide are bound by the vector memory path: their weight loads are
//     line-wise (a row's bytes of a step in adjacent lanes, whole 128-byte lines per wave
//     instruction) and pass through a wave-private LDS slot into the operand layout; only the
//     128-token tile gathers the operand layout straight from memory (see Geometry);
//   * the grid numbers workgroups so that the token blocks of one row tile run on one XCD
//     (one L2) at about the same time: their weights cross HBM once;
//   * K is split over workgroups (grid.y) only until there is about one workgroup per CU
//     (small products) or a few (large ones); every split stores its partial tile, in the
//     register layout of the tile (1 KiB per store instruction), to its own slice of an f32
//     scratch array and a second, tiny kernel sums the slices, applies the activation and
//     stores the output type.  Without a split the first kernel stores directly.
//
// The scales never enter the matrix cores, which keeps the f16 operands exact (rounding a
// dequantised weight to f16 would cost ~2^-11 of its block's range per weight, too much for
// sums that cancel):
//   int8: A holds the codes as f16 integers (1024 + u, one v_perm_b32 per two weights);
//         after each 128-block   out += s * D + (min - 1024 s) * sum_k x,
//         s = (max - min) / 255; (s, min - 1024 s) per row and sum_k x per token are staged
//         in LDS next to the activation tile by the threads that load them.
//   nf4:  A holds table values split into two f16 halves (hi + lo * 2^-11, exact to
//         2^-22), fetched per byte (two weights) from a 256-entry LDS table; after each
//         64-block   out += absmax * (D_hi + 2^-11 D_lo).
// f32 activations are split the same way while they are staged (hi + lo * 2^-11 as two f16 tiles, exact to 2^-22):
// every product term is then taken against both tiles.
// D is produced by MFMAs that start from a zero C operand, in ordinary vector registers,
// so the only per-block work outside the matrix cores is one or two fmas per output.
// Plain f16 weights (matmul_mat_fp16, src/shaders/matmul_mat_fp16.wgsl:57-140) take the same
// kernel: they are A operands as loaded and accumulate in the matrix cores over the whole K.
#include "wrq_device.h"
#include "wrq_host.h"

#include <algorithm>
#include <atomic>

namespace wrq {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));

union HalfPack {
    uint32_t u[4];
    half8 h;
};

constexpr int kStep = 128; // K elements per step
#ifndef WRQ_UNROLL_STAGES
#define WRQ_UNROLL_STAGES 2
#endif
constexpr int kUnrollStages = WRQ_UNROLL_STAGES; // even

// Partial tiles of split-K launches, in the tile order of the kernel.  Calls on one stream run one after the
// other and share a slice; calls on different streams may overlap in time, so every stream that launches a split
// product gets a slice of its own, kScratchSlices per device, handed out in order of first use and kept for the
// life of the process.  A stream beyond those gets none: its products run unsplit (correct, slower).  Nothing in
// a slice outlives a call.
constexpr size_t kScratchFloats = 8u << 20; // 32 MiB: splits * R * T up to 8 Mi partial outputs
constexpr int kScratchSlices = 4;
__device__ __align__(256) float g_splitk_scratch[kScratchSlices * kScratchFloats];

// The same for wrq_matmul_mat_int8_noalloc: a file-scope array of its own (16 MiB), so that the entry
// point for callers that cannot allocate never shares partial sums with the other entry points.  In
// host code the name is only a handle: the device address comes from hipGetSymbolAddress, once per
// device (static_scratch_ptr), and only that pointer is ever handed to a kernel.
constexpr size_t kStaticScratchFloats = 4u << 20;
static __device__ __align__(256) float scratch[kStaticScratchFloats];

__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
    return (uint32_t)f2h(a) | ((uint32_t)f2h(b) << 16);
}

__device__ __forceinline__ half2v as_h2(uint32_t v) { return __builtin_bit_cast(half2v, v); }
__device__ __forceinline__ uint32_t as_u32(half2v v) { return __builtin_bit_cast(uint32_t, v); }

__device__ __forceinline__ float dot2_ones(uint32_t v, float acc) {
    // acc + lo(v) + hi(v) with f32 accumulation: v_dot2_f32_f16 against (1.0, 1.0)
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, v), half2v{(_Float16)1.0f, (_Float16)1.0f}, acc, false);
}

__device__ __forceinline__ float row16_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xf, 0xf, true));
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xf, 0xf, true));
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xf, 0xf, true));
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xf, 0xf, true));
    return v;
}

// Tile geometry of one instantiation.  The 4 waves of a workgroup are RW row groups times KG
// "k groups": the k groups share the rows and the staged activations and take alternate K
// steps; their partial tiles are added through LDS at the end.  Products with few rows get
// their workgroups (about one per CU) from KG instead of from a split of K over the grid,
// which would cost a round trip through the scratch array and a second launch.  A stage is
// what one barrier covers: KSUB steps of 128 k of the activation tile, so that narrow token
// tiles do not pay a barrier per 128 k.
template <int MRT, int NTILE, int KG>
struct Geometry {
    static constexpr int THREADS = 256;
    static constexpr int RW = 4 / KG;          // row groups: waves side by side along the rows
    static constexpr int BN = 16 * NTILE;      // tokens per workgroup
    static constexpr int BM = 16 * MRT * RW;   // weight rows per workgroup
    static constexpr int KSUB0 = (NTILE >= 8 ? 1 : NTILE == 4 ? 2 : 4) / MRT;
    static constexpr int KSUB = KSUB0 > KG ? KSUB0 : KG;                   // steps per stage
    static constexpr int LSUB = KSUB / KG;                                 // steps per stage and k group
    static constexpr int PITCH = kStep * KSUB + 8;                         // f16 per LDS row: +16 B rotates the banks
    static constexpr int NPIECE = NTILE * KSUB;                            // 16-byte activation pieces per thread and stage
    // weight steps in flight per wave: two stages (an even number of them), one for plain f16
    // weights, whose steps take twice the registers
    static constexpr int NBUFQ = (LSUB >= 2 || MRT >= 2) ? 2 * LSUB : 4;
    static constexpr int NBUFH = LSUB >= 2 ? LSUB : 2;
    static constexpr int nbuf(int quant) { return quant == kFp16 ? NBUFH : NBUFQ; }
    static constexpr int TILE_FLOATS = 256 * RW * MRT * NTILE;             // outputs of one workgroup
    // Token tiles up to 64 wide are bound by the vector memory path, not by arithmetic: a wave
    // instruction that gathers the A-operand layout straight from memory (16 rows x 64 B, or x 32 B
    // for nf4) costs the texture path about 54 clocks, three times a line-wise one.  There the weights
    // are fetched line-wise (a row's bytes of a step in adjacent lanes: 8 rows x 128 B per instruction
    // for int8, 16 x 64 B for nf4, 4 x 256 B for f16) and turned into the A-operand layout through a
    // wave-private LDS slot.  The widest tile keeps the direct gather: its LDS is the busiest unit.
    static constexpr bool transposed_loads(int) { return NTILE <= 4; }
    static constexpr int wstep(int quant) { return quant == kFp16 ? 2 * kStep : quant == kInt8 ? kStep : kStep / 2; } // weight bytes per row and step
    static constexpr int tpitch(int quant) { return wstep(quant) + 16; }    // bytes per row of a slot: +16 B rotates the banks
    static constexpr size_t tslot_bytes(int quant) { return transposed_loads(quant) ? (size_t)4 * MRT * 16 * tpitch(quant) : 0; }
    // LDS: 2 x activation tile [BN][PITCH] f16 | 2 x row scales [KSUB][BM] float2 | 2 x token sums [KSUB][BN] f32 | nf4 pair table
    static constexpr size_t lds_bytes(int quant) {
        return (size_t)2 * BN * PITCH * sizeof(uint16_t) + (size_t)2 * KSUB * BM * sizeof(float2) + (size_t)2 * KSUB * BN * sizeof(float) +
               (quant == kNf4 ? 256 * sizeof(uint2) : 0) + tslot_bytes(quant);
    }
    static_assert((size_t)(KG - 1) * RW * MRT * NTILE * 1024 <= (size_t)2 * BN * PITCH * sizeof(uint16_t), "partial tiles of the k groups fit the activation buffers");
};

// One launch serves up to kMaxGroup independent products with the same K, token count and
// types (the attention projections of a layer, or ffn.key + ffn.receptance): together they
// fill the CUs without a split of K, where each alone would need one plus its finish kernel.
struct GemmArgs {
    uint32_t tile_begin[kMaxGroup]; // first blockIdx.x of every product, unused entries 0xffffffff
    uint32_t row_tiles[kMaxGroup];  // ceil(R / BM) of every product
    MatmulArgs m[kMaxGroup];
    float *scratch[kMaxGroup]; // partial tiles of every product; null: store directly
    uint32_t k_per_split;      // K range of one workgroup, a multiple of kStep
    uint32_t tblocks;          // ceil(T / BN)
    uint32_t tile_offset;      // blockIdx.x + tile_offset numbers the tiles of the group: a launch may cover a range of them
    uint32_t split_from;       // finish kernel: tiles from this number on have `splits` partial tiles, ...
    uint32_t splits_low;       // ... those below have this many (0 or 1: stored directly, nothing to finish)
    uint32_t prio;             // nonzero: a wave raises its issue priority (s_setprio) around the matrix work of a step, so that the other
                               // wave of the SIMD fills the gaps with its loads, conversions and staging instead of taking turns with it
                               // (7B step at 256 tokens: int8 6.92 -> 6.80 ms, nf4 9.49 -> 9.12 ms; 128 tokens: 4.58 -> 4.55, 5.88 -> 5.72)
};

// blockIdx.x -> (row tile, token block).  Workgroups are dealt round-robin to the 8 XCDs, each
// with its own L2: the token blocks of one row tile get ids that differ by multiples of 8 and
// follow each other, so they run on one XCD at about the same time and the weights they share
// cross HBM once.
__device__ __forceinline__ void tile_of_block(uint32_t id, uint32_t tblocks, uint32_t &row_tile, uint32_t &tblock) {
    const uint32_t xcd = id & 7u, slot = id >> 3;
    tblock = slot % tblocks;
    row_tile = (slot / tblocks) * 8u + xcd;
}

template <int QUANT, typename XT, int MRT, int NTILE, int KG>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void gemm_kernel(const GemmArgs ga) {
    using G = Geometry<MRT, NTILE, KG>;
    // the product of this workgroup: one scalar load of the tile starts, then its descriptor
    const uint32_t gid = blockIdx.x + ga.tile_offset; // tile number inside the group
    uint32_t pi = 0;
#pragma unroll
    for (uint32_t i = 1; i < (uint32_t)kMaxGroup; i++)
        if (gid >= ga.tile_begin[i]) pi = i;
    pi = __builtin_amdgcn_readfirstlane(pi);
    const MatmulArgs a = ga.m[pi];
    const uint32_t tile_id = gid - ga.tile_begin[pi];
    const uint32_t my_row_tiles = ga.row_tiles[pi];
    float *const my_scratch = ga.scratch[pi];
    constexpr int BN = G::BN, BM = G::BM, RW = G::RW, KSUB = G::KSUB, LSUB = G::LSUB, PITCH = G::PITCH, NPIECE = G::NPIECE, NBUF = G::nbuf(QUANT), THREADS = G::THREADS;
    constexpr int NW = QUANT == kFp16 ? 4 : QUANT == kInt8 ? 2 : 1;                        // 16-byte weight registers per row tile and step
    constexpr int WSTEP = QUANT == kFp16 ? 2 * kStep : QUANT == kInt8 ? kStep : kStep / 2; // weight bytes per row and step
    extern __shared__ __align__(16) uint8_t smem[];
    uint16_t(*xs)[BN * PITCH] = reinterpret_cast<uint16_t(*)[BN * PITCH]>(smem);
    float2(*scl)[KSUB][BM] = reinterpret_cast<float2(*)[KSUB][BM]>(smem + (size_t)2 * BN * PITCH * sizeof(uint16_t));
    float(*sxs)[KSUB][BN] =
        reinterpret_cast<float(*)[KSUB][BN]>(smem + (size_t)2 * BN * PITCH * sizeof(uint16_t) + (size_t)2 * KSUB * BM * sizeof(float2));
    uint2 *pair = reinterpret_cast<uint2 *>(smem + (size_t)2 * BN * PITCH * sizeof(uint16_t) + (size_t)2 * KSUB * BM * sizeof(float2) +
                                            (size_t)2 * KSUB * BN * sizeof(float));
    constexpr bool TRW = G::transposed_loads(QUANT);
    constexpr int TPITCH = G::tpitch(QUANT);
    uint8_t *tslots = smem + (size_t)2 * BN * PITCH * sizeof(uint16_t) + (size_t)2 * KSUB * BM * sizeof(float2) +
                      (size_t)2 * KSUB * BN * sizeof(float) + (QUANT == kNf4 ? 256 * sizeof(uint2) : 0);
    // f32 activations are split into two f16 tiles, x = hi + lo * 2^-11 (exact to 2^-22 of x, like the nf4 table
    // values): every product term is then taken twice, against hi and against lo.  The lo tile sits behind the rest.
    constexpr bool XLO = sizeof(XT) == 4;
    uint16_t(*xsl)[BN * PITCH] = reinterpret_cast<uint16_t(*)[BN * PITCH]>(smem + G::lds_bytes(QUANT));

    uint32_t row_tile, tblock;
    tile_of_block(tile_id, ga.tblocks, row_tile, tblock);
    if (row_tile >= my_row_tiles) return; // padding of the XCD-aware grid
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    // without k groups the k group is a compile-time zero: step offsets into LDS stay immediates
    const uint32_t wv = KG == 1 ? ((tid >> 6) & 3) : __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wave = KG == 1 ? wv : wv % RW; // row group of this wave
    const uint32_t kg = KG == 1 ? 0u : wv / RW;   // its k group
    const uint32_t r16 = lane & 15, g = lane >> 4;
    const uint32_t b = blockIdx.z;
    const uint32_t t0 = tblock * BN;
    const uint32_t K = a.K;
    const uint32_t k_begin = blockIdx.y * ga.k_per_split;
    const uint32_t k_end = min(K, k_begin + ga.k_per_split);
    const uint32_t nsteps = (k_end - k_begin) / kStep;
    const uint32_t last = nsteps - 1;
    const uint32_t nstages = (nsteps + KSUB - 1) / KSUB;
    const uint32_t row_local = wave * (16 * MRT); // first row of this wave inside the workgroup
    const uint32_t row_base = row_tile * BM + row_local;

    // this lane's A-side row of every row tile
    const uint8_t *wp[MRT];
#pragma unroll
    for (int i = 0; i < MRT; i++) {
        const uint32_t row = min(row_base + 16 * i + r16, a.R - 1);
        const uint64_t e = ((uint64_t)b * a.R + row) * K + k_begin; // flat element index of (row, k_begin)
        wp[i] = QUANT == kFp16 ? a.w + 2 * e + 16 * g : QUANT == kInt8 ? a.w + e + 16 * g : a.w + (e >> 1) + 8 * g;
    }
    // line-wise fetch: the WSTEP bytes of a row and step sit in LPR adjacent lanes, load j of a row tile
    // takes rows RPL j .. RPL j + RPL - 1
    constexpr int LPR = WSTEP / 16, RPL = 64 / LPR; // lanes per row, rows per load (NW * RPL = 16)
    static_assert(NW * RPL == 16, "a row tile is NW line-wise loads");
    const uint8_t *wq[MRT][NW];
    if constexpr (TRW) {
#pragma unroll
        for (int i = 0; i < MRT; i++)
#pragma unroll
            for (int j = 0; j < NW; j++) {
                const uint32_t row = min(row_base + 16 * i + RPL * j + lane / LPR, a.R - 1);
                const uint64_t e = ((uint64_t)b * a.R + row) * K + k_begin; // flat element index of (row, k_begin)
                wq[i][j] = (QUANT == kFp16 ? a.w + 2 * e : QUANT == kInt8 ? a.w + e : a.w + (e >> 1)) + 16 * (lane % LPR);
            }
    }
    uint8_t *tslot = tslots + (size_t)wv * (MRT * 16 * TPITCH); // this wave's transposition slot
    // scale words (one 32-bit word per row and step for both formats: a (min, max) pair, or the
    // absmax of two 64-blocks): thread t < BM fetches those of workgroup row t
    const uint32_t *sp;
    {
        const uint32_t row = min(row_tile * BM + min(tid, (uint32_t)BM - 1), a.R - 1);
        sp = QUANT == kFp16 ? nullptr : reinterpret_cast<const uint32_t *>(a.scale) + ((((uint64_t)b * a.R + row) * K + k_begin) >> 7);
    }

    // nf4: the two table values behind this thread's entry of the byte table, requested before the
    // first weights so that they are back first; the entry is written once those are on their way
    float tq0 = 0.0f, tq1 = 0.0f;
    if (QUANT == kNf4) {
        tq0 = a.quant[tid & 15];
        tq1 = a.quant[(tid >> 4) & 15];
    }

    // activation staging: piece p of a stage is 8 consecutive k of one token; the 16 pieces of a
    // token and step sit in 16 adjacent lanes, one DPP row
    struct Stage {
        uint4 x[NPIECE];
        uint4 xl[XLO ? NPIECE : 1]; // lo halves of f32 activations
        uint32_t sc[KSUB];
    };
    const XT *xp[NPIECE]; // (token, k_begin + 8 * (piece & 15)) of each piece
#pragma unroll
    for (int p = 0; p < NPIECE; p++) {
        const uint32_t piece = tid + THREADS * p;
        const uint32_t tok = min(t0 + piece / (16 * KSUB), a.T - 1);
        xp[p] = reinterpret_cast<const XT *>(a.x) + (uint64_t)b * a.x_batch_stride + (uint64_t)tok * a.x_token_stride + k_begin +
                ((piece & 15) << 3);
    }
    // loads of a stage; steps past the K range re-read the last step (their data is not used)
    auto load_stage = [&](uint32_t stage, Stage &st) {
#pragma unroll
        for (int p = 0; p < NPIECE; p++) {
            const uint32_t sub = ((tid + THREADS * p) / 16) % KSUB;
            const XT *src = xp[p] + min(stage * KSUB + sub, last) * kStep;
            if constexpr (sizeof(XT) == 2) {
                st.x[p] = load128(src);
            } else {
                const uint4 v0 = load128(src), v1 = load128(src + 4);
                const float raw[8] = {__uint_as_float(v0.x), __uint_as_float(v0.y), __uint_as_float(v0.z), __uint_as_float(v0.w),
                                      __uint_as_float(v1.x), __uint_as_float(v1.y), __uint_as_float(v1.z), __uint_as_float(v1.w)};
                // both halves stay finite f16 values: hi is clamped to the largest f16 magnitude before lo is formed, and lo
                // saturates too.  Exact to 2^-22 for |x| <= 65535 (65504 + 31.98); beyond that the activation acts as +-65536
                // instead of turning the sum into inf - inf.
                float f[8], l[8];
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    f[e] = fminf(fmaxf(raw[e], -65504.0f), 65504.0f);
                    l[e] = fminf(fmaxf((raw[e] - h2f(f2h(f[e]))) * 2048.0f, -65504.0f), 65504.0f);
                }
                st.x[p] = make_uint4(pack_h2(f[0], f[1]), pack_h2(f[2], f[3]), pack_h2(f[4], f[5]), pack_h2(f[6], f[7]));
                st.xl[XLO ? p : 0] = make_uint4(pack_h2(l[0], l[1]), pack_h2(l[2], l[3]), pack_h2(l[4], l[5]), pack_h2(l[6], l[7]));
            }
        }
        if constexpr (QUANT == kFp16) {
#pragma unroll
            for (int u = 0; u < KSUB; u++) st.sc[u] = 0u;
        } else {
            // the scale words of a row's steps are adjacent: one 8- or 16-byte load per row and stage
            // where the stage is whole and aligned (a load per word touches one line per row each time)
            const uint32_t *q = sp + stage * KSUB;
            if (KSUB == 4 && stage * KSUB + 3 <= last && (reinterpret_cast<uintptr_t>(q) & 15) == 0) {
                const uint4 v = load128(q);
                st.sc[0] = v.x; st.sc[KSUB > 1 ? 1 : 0] = v.y; st.sc[KSUB > 2 ? 2 : 0] = v.z; st.sc[KSUB > 3 ? 3 : 0] = v.w;
            } else if (KSUB == 2 && stage * KSUB + 1 <= last && (reinterpret_cast<uintptr_t>(q) & 7) == 0) {
                const uint2 v = *reinterpret_cast<const uint2 *>(q);
                st.sc[0] = v.x; st.sc[KSUB > 1 ? 1 : 0] = v.y;
            } else {
#pragma unroll
                for (int u = 0; u < KSUB; u++) st.sc[u] = sp[min(stage * KSUB + u, last)];
            }
        }
    };
    auto store_stage = [&](const Stage &st, int buf) {
#pragma unroll
        for (int p = 0; p < NPIECE; p++) {
            const uint32_t piece = tid + THREADS * p;
            const uint32_t tok = piece / (16 * KSUB), c = piece % (16 * KSUB);
            *reinterpret_cast<uint4 *>(&xs[buf][tok * PITCH + (c << 3)]) = st.x[p];
            if constexpr (XLO) *reinterpret_cast<uint4 *>(&xsl[buf][tok * PITCH + (c << 3)]) = st.xl[p];
            if (QUANT == kInt8) {
                float s = dot2_ones(st.x[p].x, 0.0f);
                s = dot2_ones(st.x[p].y, s);
                s = dot2_ones(st.x[p].z, s);
                s = dot2_ones(st.x[p].w, s);
                if constexpr (XLO) {
                    float sl = dot2_ones(st.xl[p].x, 0.0f);
                    sl = dot2_ones(st.xl[p].y, sl);
                    sl = dot2_ones(st.xl[p].z, sl);
                    sl = dot2_ones(st.xl[p].w, sl);
                    s = fmaf(sl, 1.0f / 2048.0f, s);
                }
                s = row16_sum(s);
                if ((tid & 15) == 0) sxs[buf][c >> 4][tok] = s;
            }
        }
        if (QUANT != kFp16 && tid < BM) {
#pragma unroll
            for (int u = 0; u < KSUB; u++) {
                const float lo = h2f((uint16_t)(st.sc[u] & 0xffffu)), hi = h2f((uint16_t)(st.sc[u] >> 16));
                if (QUANT == kInt8) {
                    const float s = (hi - lo) * (1.0f / 255.0f); // (min, max) -> (s, min - 1024 s)
                    scl[buf][u][tid] = make_float2(s, fmaf(-1024.0f, s, lo));
                } else {
                    scl[buf][u][tid] = make_float2(lo, hi); // absmax of the step's two 64-blocks
                }
            }
        }
    };

    // packed weights of one step for this lane, per row tile: int8 2 x 16 B of codes, nf4 2 x 8 B
    struct StepRegs {
        uint4 w[MRT][NW];
    };
    // k group `kg` owns the steps kg, kg + KG, ...: local step m is step m * KG + kg
    const uint32_t nlocal = (nsteps + KG - 1 - kg) / KG;
    // Weight loads.  From 32-token tiles on they are plain cacheable loads: marked nontemporal, the compiler's
    // load-counter bookkeeping falls back to a full wait at the head of the main loop and the ring of prefetched
    // K steps drains once per iteration.  The 16-token tile keeps streaming loads: its launches are short, the
    // drain costs little there and weights that bypass the caches leave them to the activations.
    constexpr bool STREAM_W = NTILE == 1;
    auto lw128 = [&](const uint8_t *p) { return STREAM_W ? load128_stream(p) : load128(p); };
    auto lw64 = [&](const uint8_t *p) { return STREAM_W ? load64_stream(p) : *reinterpret_cast<const uint2 *>(p); };
    auto load_w = [&](uint32_t m, StepRegs &dst) {
        const uint32_t step = min(min(m, max(nlocal, 1u) - 1) * KG + kg, last); // clamped to the K range
#pragma unroll
        for (int i = 0; i < MRT; i++) {
            const uint8_t *p = wp[i] + step * WSTEP;
            if constexpr (TRW) {
#pragma unroll
                for (int j = 0; j < NW; j++) dst.w[i][j] = lw128(wq[i][j] + step * WSTEP);
            } else if (QUANT == kFp16) {
#pragma unroll
                for (int j = 0; j < NW; j++) dst.w[i][j] = lw128(p + 64 * j); // operand j: k = 32 j + 8 g .. + 8
            } else if (QUANT == kInt8) {
                dst.w[i][0] = lw128(p);
                dst.w[i][NW - 1] = lw128(p + 64);
            } else {
                const uint2 v0 = lw64(p), v1 = lw64(p + 32);
                dst.w[i][0] = make_uint4(v0.x, v0.y, v1.x, v1.y);
            }
        }
    };

    float4v out[MRT][NTILE];
#pragma unroll
    for (int i = 0; i < MRT; i++)
#pragma unroll
        for (int n = 0; n < NTILE; n++) out[i][n] = float4v{0.f, 0.f, 0.f, 0.f};
    const float4v zero4 = float4v{0.f, 0.f, 0.f, 0.f};
    // plain f16 weights against the lo halves of f32 activations: a second set of accumulators, added at the end
    float4v outl[(XLO && QUANT == kFp16) ? MRT : 1][(XLO && QUANT == kFp16) ? NTILE : 1];
    if constexpr (XLO && QUANT == kFp16) {
#pragma unroll
        for (int i = 0; i < MRT; i++)
#pragma unroll
            for (int n = 0; n < NTILE; n++) outl[i][n] = zero4;
    }

    // lane offsets into the staged tile, the row scales and the token sums; the k group of the wave is
    // part of them, so that the step of a stage stays an immediate offset
    const uint32_t xlane8 = r16 * PITCH + kg * kStep + 8 * g, xlane16 = r16 * PITCH + kg * kStep + 16 * g;
    const uint32_t scl_lane = kg * BM + row_local + 4 * g, sxs_lane = kg * BN + r16;
    // one K step on the matrix cores: weights `cur` against step `sub` (+ the k group) of the stage in
    // LDS buffer `buf`.  Operand j of a step covers k = 64 (j / 2) + 16 g + 8 (j % 2) .. + 8
    auto compute = [&](const StepRegs &cur, int buf, int sub) {
        // the step's packed weights of this lane in A-operand layout: as loaded, or line-wise loads
        // passed through the wave's LDS slot (one wave writes and reads a slot, in program order: no barrier)
        uint4 wa[MRT][NW];
        if constexpr (TRW) {
#pragma unroll
            for (int i = 0; i < MRT; i++)
#pragma unroll
                for (int j = 0; j < NW; j++)
                    *reinterpret_cast<uint4 *>(tslot + (i * 16 + RPL * j + lane / LPR) * TPITCH + 16 * (lane % LPR)) = cur.w[i][j];
#pragma unroll
            for (int i = 0; i < MRT; i++) {
                const uint8_t *row = tslot + (i * 16 + r16) * TPITCH;
                if constexpr (QUANT == kNf4) {
                    const uint2 v0 = *reinterpret_cast<const uint2 *>(row + 8 * g), v1 = *reinterpret_cast<const uint2 *>(row + 32 + 8 * g);
                    wa[i][0] = make_uint4(v0.x, v0.y, v1.x, v1.y);
                } else {
#pragma unroll
                    for (int j = 0; j < NW; j++) wa[i][j] = *reinterpret_cast<const uint4 *>(row + 64 * j + 16 * g);
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < MRT; i++)
#pragma unroll
                for (int j = 0; j < NW; j++) wa[i][j] = cur.w[i][j];
        }
        if constexpr (QUANT == kFp16) {
            // plain f16 weights are the A operands as loaded; the accumulators stay in the matrix cores
            const uint16_t *xh = xs[buf] + sub * kStep + xlane8;
            const uint16_t *xlo = xsl[buf] + sub * kStep + xlane8;
#pragma unroll
            for (int j = 0; j < 4; j++) {
#pragma unroll
                for (int n = 0; n < NTILE; n++) {
                    HalfPack B, Bl;
                    const uint4 v = *reinterpret_cast<const uint4 *>(xh + n * 16 * PITCH + 32 * j);
                    B.u[0] = v.x; B.u[1] = v.y; B.u[2] = v.z; B.u[3] = v.w;
                    if constexpr (XLO) {
                        const uint4 vl = *reinterpret_cast<const uint4 *>(xlo + n * 16 * PITCH + 32 * j);
                        Bl.u[0] = vl.x; Bl.u[1] = vl.y; Bl.u[2] = vl.z; Bl.u[3] = vl.w;
                    }
#pragma unroll
                    for (int i = 0; i < MRT; i++) {
                        HalfPack A;
                        const uint4 &wv = wa[i][j < NW ? j : 0];
                        A.u[0] = wv.x; A.u[1] = wv.y; A.u[2] = wv.z; A.u[3] = wv.w;
                        out[i][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A.h, B.h, out[i][n], 0, 0, 0);
                        if constexpr (XLO) outl[i][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A.h, Bl.h, outl[i][n], 0, 0, 0);
                    }
                }
            }
            return;
        }
        const uint16_t *xt = xs[buf] + sub * kStep + xlane16;
        const uint16_t *xtl = xsl[buf] + sub * kStep + xlane16;
        // scales of the 4 D-side rows of this lane, per row tile: (s, c) x 4 or (absmax0, absmax1) x 4
        float4 sc0[MRT], sc1[MRT];
#pragma unroll
        for (int i = 0; i < MRT; i++) {
            const float4 *q = reinterpret_cast<const float4 *>(&scl[buf][sub][0] + scl_lane + 16 * i);
            sc0[i] = q[0];
            sc1[i] = q[1];
        }
        if (QUANT == kInt8) {
            HalfPack A[MRT][4];
#pragma unroll
            for (int i = 0; i < MRT; i++) {
                const uint32_t w[8] = {wa[i][0].x,      wa[i][0].y,      wa[i][0].z,      wa[i][0].w,
                                       wa[i][NW - 1].x, wa[i][NW - 1].y, wa[i][NW - 1].z, wa[i][NW - 1].w};
#pragma unroll
                for (int d = 0; d < 8; d++) {
                    // 4 codes of one dword -> f16 pairs 1024 + u
                    A[i][d >> 1].u[2 * (d & 1)] = __builtin_amdgcn_perm(0x64646464u, w[d], 0x04010400u);
                    A[i][d >> 1].u[2 * (d & 1) + 1] = __builtin_amdgcn_perm(0x64646464u, w[d], 0x04030402u);
                }
            }
            if (ga.prio) __builtin_amdgcn_s_setprio(3);
#pragma unroll
            for (int n = 0; n < NTILE; n++) {
                float4v D[MRT], Dx[MRT];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    HalfPack B;
                    const uint4 v = *reinterpret_cast<const uint4 *>(xt + n * 16 * PITCH + 64 * (j >> 1) + 8 * (j & 1));
                    B.u[0] = v.x; B.u[1] = v.y; B.u[2] = v.z; B.u[3] = v.w;
#pragma unroll
                    for (int i = 0; i < MRT; i++) D[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[i][j].h, B.h, j == 0 ? zero4 : D[i], 0, 0, 0);
                    if constexpr (XLO) {
                        HalfPack Bl;
                        const uint4 vl = *reinterpret_cast<const uint4 *>(xtl + n * 16 * PITCH + 64 * (j >> 1) + 8 * (j & 1));
                        Bl.u[0] = vl.x; Bl.u[1] = vl.y; Bl.u[2] = vl.z; Bl.u[3] = vl.w;
#pragma unroll
                        for (int i = 0; i < MRT; i++) Dx[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[i][j].h, Bl.h, j == 0 ? zero4 : Dx[i], 0, 0, 0);
                    }
                }
                if constexpr (XLO) {
#pragma unroll
                    for (int i = 0; i < MRT; i++)
#pragma unroll
                        for (int d = 0; d < 4; d++) D[i][d] = fmaf(Dx[i][d], 1.0f / 2048.0f, D[i][d]);
                }
                const float sx = (&sxs[buf][sub][0])[sxs_lane + n * 16];
#pragma unroll
                for (int i = 0; i < MRT; i++) {
                    out[i][n][0] = fmaf(sc0[i].x, D[i][0], fmaf(sc0[i].y, sx, out[i][n][0]));
                    out[i][n][1] = fmaf(sc0[i].z, D[i][1], fmaf(sc0[i].w, sx, out[i][n][1]));
                    out[i][n][2] = fmaf(sc1[i].x, D[i][2], fmaf(sc1[i].y, sx, out[i][n][2]));
                    out[i][n][3] = fmaf(sc1[i].z, D[i][3], fmaf(sc1[i].w, sx, out[i][n][3]));
                }
            }
            if (ga.prio) __builtin_amdgcn_s_setprio(0);
        } else {
            HalfPack Ah[MRT][4], Al[MRT][4];
#pragma unroll
            for (int i = 0; i < MRT; i++) {
                const uint32_t w[4] = {wa[i][0].x, wa[i][0].y, wa[i][0].z, wa[i][0].w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        const uint2 e = pair[(w[j] >> (8 * c)) & 0xffu];
                        Ah[i][j].u[c] = e.x;
                        Al[i][j].u[c] = e.y;
                    }
                }
            }
            if (ga.prio) __builtin_amdgcn_s_setprio(3);
#pragma unroll
            for (int n = 0; n < NTILE; n++) {
#pragma unroll
                for (int blk = 0; blk < 2; blk++) {
                    float4v Dh[MRT], Dl[MRT];
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        HalfPack B;
                        const uint4 v = *reinterpret_cast<const uint4 *>(xt + n * 16 * PITCH + 64 * blk + 8 * j);
                        B.u[0] = v.x; B.u[1] = v.y; B.u[2] = v.z; B.u[3] = v.w;
#pragma unroll
                        for (int i = 0; i < MRT; i++) {
                            Dh[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Ah[i][2 * blk + j].h, B.h, j == 0 ? zero4 : Dh[i], 0, 0, 0);
                            Dl[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Al[i][2 * blk + j].h, B.h, j == 0 ? zero4 : Dl[i], 0, 0, 0);
                        }
                        if constexpr (XLO) { // hi table values against the lo halves of the activations join the 2^-11 sum
                            HalfPack Bl;
                            const uint4 vl = *reinterpret_cast<const uint4 *>(xtl + n * 16 * PITCH + 64 * blk + 8 * j);
                            Bl.u[0] = vl.x; Bl.u[1] = vl.y; Bl.u[2] = vl.z; Bl.u[3] = vl.w;
#pragma unroll
                            for (int i = 0; i < MRT; i++) Dl[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Ah[i][2 * blk + j].h, Bl.h, Dl[i], 0, 0, 0);
                        }
                    }
#pragma unroll
                    for (int i = 0; i < MRT; i++) {
                        const float am[4] = {blk ? sc0[i].y : sc0[i].x, blk ? sc0[i].w : sc0[i].z, blk ? sc1[i].y : sc1[i].x,
                                             blk ? sc1[i].w : sc1[i].z};
#pragma unroll
                        for (int d = 0; d < 4; d++) out[i][n][d] = fmaf(am[d], fmaf(Dl[i][d], 1.0f / 2048.0f, Dh[i][d]), out[i][n][d]);
                    }
                }
            }
            if (ga.prio) __builtin_amdgcn_s_setprio(0);
        }
    };

    // Ring of NBUF weight steps in flight, the next activation stage in registers while the
    // current one is consumed from LDS.  The loop is unrolled over NBUF steps (an even number of
    // stages) so that every ring slot and LDS buffer is fixed at compile time.  Refills are
    // unconditional and clamped to the K range, so the ring registers never pass through a
    // control-flow join; only stores and matrix work of stages and steps past the range are
    // skipped.
    StepRegs ring[NBUF];
    Stage stage;
    load_stage(0, stage);
#pragma unroll
    for (int j = 0; j < NBUF; j++) load_w(j, ring[j]);
    if (QUANT == kNf4) {
        // entry for byte v: (hi(q[v & 15]), hi(q[v >> 4])), (lo(..), lo(..)); lo scaled by 2^11
        const float h0 = h2f(f2h(tq0)), h1 = h2f(f2h(tq1));
        if (tid < 256) pair[tid] = make_uint2(pack_h2(tq0, tq1), pack_h2((tq0 - h0) * 2048.0f, (tq1 - h1) * 2048.0f));
    }
    constexpr int STAGES = kUnrollStages > NBUF / LSUB ? kUnrollStages : NBUF / LSUB; // stages per loop iteration
    for (uint32_t S0 = 0; S0 < nstages; S0 += STAGES) {
#pragma unroll
        for (int q = 0; q < STAGES; q++) {
            const uint32_t S = S0 + q;
            const int buf = q & 1;
            __builtin_amdgcn_sched_barrier(0);
            if (S < nstages) store_stage(stage, buf);
            __builtin_amdgcn_sched_barrier(0);
            load_stage(min(S + 1, nstages - 1), stage);
            if (S < nstages) lds_barrier();
#pragma unroll
            for (int u = 0; u < LSUB; u++) {
                const int sub = u * KG; // + kg: step of the stage taken by this k group
                const int slot = (q * LSUB + u) % NBUF;
                __builtin_amdgcn_sched_barrier(0); // steps do not interleave: one set of operand registers
                if (S * KSUB + sub + kg < nsteps) compute(ring[slot], buf, sub);
                // refill the slot just consumed; the scheduling barrier keeps the loads below the
                // last use of the old values, so they can target the same registers
                __builtin_amdgcn_sched_barrier(0);
                load_w(S * LSUB + u + NBUF, ring[slot]);
            }
        }
    }

    if constexpr (XLO && QUANT == kFp16) {
#pragma unroll
        for (int i = 0; i < MRT; i++)
#pragma unroll
            for (int n = 0; n < NTILE; n++)
#pragma unroll
                for (int d = 0; d < 4; d++) out[i][n][d] = fmaf(outl[i][n][d], 1.0f / 2048.0f, out[i][n][d]);
    }
    // add the partial tiles of the k groups through LDS (the activation buffers are free now)
    if constexpr (KG > 1) {
        float4 *red = reinterpret_cast<float4 *>(smem);
        lds_barrier();
        if (kg != 0) {
#pragma unroll
            for (int i = 0; i < MRT; i++)
#pragma unroll
                for (int n = 0; n < NTILE; n++)
                    red[((((kg - 1) * RW + wave) * MRT + i) * NTILE + n) * 64 + lane] =
                        make_float4(out[i][n][0], out[i][n][1], out[i][n][2], out[i][n][3]);
        }
        lds_barrier();
        if (kg != 0) return;
#pragma unroll
        for (int q = 1; q < KG; q++)
#pragma unroll
            for (int i = 0; i < MRT; i++)
#pragma unroll
                for (int n = 0; n < NTILE; n++) {
                    const float4 v = red[((((q - 1) * RW + wave) * MRT + i) * NTILE + n) * 64 + lane];
                    out[i][n][0] += v.x; out[i][n][1] += v.y; out[i][n][2] += v.z; out[i][n][3] += v.w;
                }
    }

    // D layout of a 16x16 tile: lane holds token column (lane & 15), rows 4 g .. 4 g + 3
    if (my_scratch) {
        // partial tile of this split, stored tile-major so that every store instruction writes
        // 1 KiB in one piece: [split][batch][workgroup][wave][i][n][lane][4]
        const uint32_t wg = tile_id, nwg = (my_row_tiles + 7) / 8 * 8 * ga.tblocks;
        float *dst = my_scratch + ((((uint64_t)blockIdx.y * a.B + b) * nwg + wg) * (RW * MRT * NTILE) + wave * (MRT * NTILE)) * 256 + lane * 4;
#pragma unroll
        for (int i = 0; i < MRT; i++)
#pragma unroll
            for (int n = 0; n < NTILE; n++)
                *reinterpret_cast<float4 *>(dst + (i * NTILE + n) * 256) = make_float4(out[i][n][0], out[i][n][1], out[i][n][2], out[i][n][3]);
        return;
    }
    act_dispatch(a.act, [&](auto act_tag) {
        constexpr int ACT = decltype(act_tag)::value;
#pragma unroll
        for (int i = 0; i < MRT; i++) {
            const uint32_t orow = row_base + 16 * i + 4 * g;
#pragma unroll
            for (int n = 0; n < NTILE; n++) {
                const uint32_t t = t0 + n * 16 + r16;
                if (t < a.T && orow < a.R) {
                    const uint64_t idx = (uint64_t)b * a.out_batch_stride + (uint64_t)t * a.out_token_stride + orow;
                    float v[4];
#pragma unroll
                    for (int d = 0; d < 4; d++) v[d] = act_one<ACT>(out[i][n][d]);
                    if (a.out_f16) {
                        *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(a.out) + idx) =
                            make_uint2(pack_h2(v[0], v[1]), pack_h2(v[2], v[3]));
                    } else {
                        *reinterpret_cast<float4 *>(reinterpret_cast<float *>(a.out) + idx) = make_float4(v[0], v[1], v[2], v[3]);
                    }
                }
            }
        }
    });
}

// Second half of a split-K launch: sum of the partial tiles over the splits, activation, output type, for every
// product of the launch (blockIdx.y).  One thread per lane slot of the first kernel's tiles (same decoding).
// The launch is a few microseconds long, so the scalar load of cold argument memory in front of its first load counts: what the
// first product needs (its partial tiles, output, extents) comes as leading scalar arguments, preloaded in SGPRs; the other
// products of a group read their descriptor.  geom: rw | mrt << 4 | ntile << 8 | f16 output of the first product << 16 | its
// activation << 17.
__global__ __launch_bounds__(256) void gemm_finish_kernel(uint32_t splits, const uint32_t geom, const float *scratch0, void *out0, const uint32_t row_tiles0,
                                                          const uint32_t tblocks, const uint32_t B0, const uint32_t T0, const uint32_t R0,
                                                          const uint32_t out_token_stride0, const uint32_t split_from, const uint32_t splits_low,
                                                          const GemmArgs ga) {
    const uint32_t rw = geom & 15u, mrt = (geom >> 4) & 15u, ntile = (geom >> 8) & 255u;
    const uint32_t pi = blockIdx.y;
    MatmulArgs a;
    const float *scratch;
    uint32_t row_tiles, tile_begin;
    if (pi == 0) {
        a.out = out0, a.B = B0, a.T = T0, a.R = R0, a.out_token_stride = out_token_stride0;
        a.out_batch_stride = B0 > 1 ? ga.m[0].out_batch_stride : 0;
        a.out_f16 = (int)((geom >> 16) & 1u), a.act = (int)((geom >> 17) & 7u);
        scratch = scratch0, row_tiles = row_tiles0, tile_begin = 0;
    } else {
        a = ga.m[pi];
        scratch = ga.scratch[pi], row_tiles = ga.row_tiles[pi], tile_begin = ga.tile_begin[pi];
    }
    if (!scratch) return; // no tile of this product was split
    const uint32_t nwg = (row_tiles + 7) / 8 * 8 * tblocks;
    const uint32_t per_wg = rw * mrt * ntile * 64; // lane slots per workgroup tile
    const uint64_t slots = (uint64_t)a.B * nwg * per_wg;
    const uint64_t q = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (q >= slots) return;
    const uint32_t lane = (uint32_t)(q & 63), r16 = lane & 15, g = lane >> 4;
    const uint32_t tp = (uint32_t)((q >> 6) % (rw * mrt * ntile));
    const uint64_t bw = q / per_wg;
    const uint32_t wg = (uint32_t)(bw % nwg), b = (uint32_t)(bw / nwg);
    const uint32_t n = tp % ntile, wi = tp / ntile; // wi = wave * mrt + i
    if (tile_begin + wg < split_from) splits = splits_low;
    if (splits <= 1) return; // stored directly by a launch without a split
    uint32_t row_tile, tblock;
    tile_of_block(wg, tblocks, row_tile, tblock);
    if (row_tile >= row_tiles) return;
    const uint32_t row = row_tile * 16 * rw * mrt + wi * 16 + 4 * g;
    const uint32_t t = tblock * 16 * ntile + n * 16 + r16;
    if (t >= a.T || row >= a.R) return;
    const float *src = scratch + q * 4;
    const uint64_t slice = slots * 4;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    uint32_t k = 0;
    for (; k + 4 <= splits; k += 4) { // four slices in flight
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) v[u] = *reinterpret_cast<const float4 *>(src + (k + u) * slice);
#pragma unroll
        for (int u = 0; u < 4; u++) { s.x += v[u].x; s.y += v[u].y; s.z += v[u].z; s.w += v[u].w; }
    }
    for (; k < splits; k++) {
        const float4 v = *reinterpret_cast<const float4 *>(src + k * slice);
        s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    const float v[4] = {act_apply(a.act, s.x), act_apply(a.act, s.y), act_apply(a.act, s.z), act_apply(a.act, s.w)};
    const uint64_t idx = (uint64_t)b * a.out_batch_stride + (uint64_t)t * a.out_token_stride + row;
    if (a.out_f16) {
        *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(a.out) + idx) = make_uint2(pack_h2(v[0], v[1]), pack_h2(v[2], v[3]));
    } else {
        *reinterpret_cast<float4 *>(reinterpret_cast<float *>(a.out) + idx) = make_float4(v[0], v[1], v[2], v[3]);
    }
}

namespace {

constexpr int kMaxDevices = 64;

// Device address of a __device__ array on the current device, looked up once per device (every GPU
// holds its own copy at its own address).  Threads may race to the first lookup: both get the same
// answer and the slot is an atomic.
template <typename Lookup>
float *device_array(std::atomic<float *> (&slots)[kMaxDevices], Lookup lookup) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    float *p = slots[dev].load(std::memory_order_acquire);
    if (!p) {
        void *q = nullptr;
        if (lookup(&q) != hipSuccess || !q) return nullptr;
        p = static_cast<float *>(q);
        slots[dev].store(p, std::memory_order_release);
    }
    return p;
}

// Compute units of the current device (256 on MI355X); 0 if the query fails.
uint32_t cu_count() {
    static std::atomic<int> cached[kMaxDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n <= 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return (uint32_t)n;
}

float *scratch_base() {
    static std::atomic<float *> slots[kMaxDevices];
    return device_array(slots, [](void **q) { return hipGetSymbolAddress(q, HIP_SYMBOL(g_splitk_scratch)); });
}

// The slice of `stream` on the current device: the one it already owns, else the first free one (claimed with a
// compare-and-swap, so two threads that meet here with different streams never share one); null when all are taken.
float *scratch_ptr(hipStream_t stream) {
    static std::atomic<uintptr_t> owner[kMaxDevices][kScratchSlices]; // stream handle + 1; 0 = free
    float *base = scratch_base();
    int dev = 0;
    if (!base || hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    const uintptr_t key = reinterpret_cast<uintptr_t>(stream) + 1;
    for (int i = 0; i < kScratchSlices; i++) {
        uintptr_t cur = owner[dev][i].load(std::memory_order_acquire);
        if (cur == 0 && owner[dev][i].compare_exchange_strong(cur, key, std::memory_order_acq_rel)) cur = key;
        if (cur == key) return base + (size_t)i * kScratchFloats;
    }
    return nullptr;
}

float *static_scratch_ptr() {
    static std::atomic<float *> slots[kMaxDevices];
    return device_array(slots, [](void **q) { return hipGetSymbolAddress(q, HIP_SYMBOL(scratch)); });
}

template <int QUANT, typename XT, int MRT, int NTILE, int KG>
int launch_one(hipStream_t stream, const MatmulArgs *args, int n, uint32_t ksplit, const ScratchPolicy *sp) {
    using G = Geometry<MRT, NTILE, KG>;
    constexpr size_t lds = G::lds_bytes(QUANT) + (sizeof(XT) == 4 ? (size_t)2 * G::BN * G::PITCH * sizeof(uint16_t) : 0);
    auto *kern = &gemm_kernel<QUANT, XT, MRT, NTILE, KG>;
    if (lds > 48 * 1024) {
        // one-time opt-in to more than the default dynamic LDS limit
        static const hipError_t once = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        (void)once;
    }
    GemmArgs ga;
    const MatmulArgs &a0 = args[0];
    ga.tblocks = (a0.T + G::BN - 1) / G::BN;
    uint32_t nwg[kMaxGroup], total = 0;
    uint64_t slice[kMaxGroup], slices = 0; // partial-tile floats of one split, per product
    for (int i = 0; i < kMaxGroup; i++) {
        ga.tile_begin[i] = 0xffffffffu;
        ga.row_tiles[i] = 0;
        ga.scratch[i] = nullptr;
        if (i >= n) continue;
        ga.m[i] = args[i];
        ga.row_tiles[i] = (args[i].R + G::BM - 1) / G::BM;
        nwg[i] = (ga.row_tiles[i] + 7) / 8 * 8 * ga.tblocks; // padded for the XCD-aware numbering
        ga.tile_begin[i] = total;
        total += nwg[i];
        slice[i] = (uint64_t)args[i].B * nwg[i] * G::TILE_FLOATS;
        slices += slice[i];
    }
    const uint32_t steps = a0.K / kStep;
    if (ksplit > steps) ksplit = steps;
    if (ksplit < 1) ksplit = 1;
    // the partial tiles of all splits must fit the scratch array, whoever chose `ksplit`: the shared
    // array takes fewer splits then, the fixed one of the no-allocation entry point refuses
    const uint64_t cap = sp ? sp->floats : kScratchFloats;
    // the slice of this stream, claimed when a launch first needs one; a stream that came after all slices were
    // handed out runs its products unsplit
    float *slice_cached = nullptr;
    bool slice_asked = false;
    auto slice_base = [&]() -> float * {
        if (sp) return sp->base;
        if (!slice_asked) slice_cached = scratch_ptr(stream), slice_asked = true;
        return slice_cached;
    };
    if (ksplit > 1 && !slice_base()) ksplit = 1;
    // the fixed array of the no-allocation entry point: a split the caller pinned is not second-guessed and is refused when
    // its partial sums do not fit; the library's own choice gives way to the largest split that fits, as on the plain path
    if (sp && sp->strict && ksplit > 1 && slices * ksplit > cap && tune_is_set(kTuneGemmKsplit))
        return fail(WRQ_ERR_SIZE, "split-K partial sums of this product need %llu bytes of scratch, the fixed array holds %llu",
                    (unsigned long long)(slices * ksplit * sizeof(float)), (unsigned long long)(cap * sizeof(float)));
    while (ksplit > 1 && slices * ksplit > cap) ksplit /= 2;
    const uint32_t steps_per = (steps + ksplit - 1) / ksplit;
    ga.k_per_split = steps_per * kStep;
    const uint32_t splits = (steps + steps_per - 1) / steps_per;
    if (splits > 1) {
        float *base = slice_base();
        if (!base) return fail(WRQ_ERR_DEVICE, "split-K scratch not resolvable");
        if (slices * splits > cap)
            return fail(WRQ_ERR_SIZE, "data size not match: %llu vs. %llu", (unsigned long long)(slices * splits), (unsigned long long)cap);
        uint64_t off = 0;
        for (int i = 0; i < n; i++) {
            ga.scratch[i] = base + off;
            off += slice[i] * splits;
        }
    }
    if (a0.B > 65535u || splits > 65535u) return fail(WRQ_ERR_SIZE, "data size not match: %u vs. %u", a0.B > splits ? a0.B : splits, 65535u);
    ga.tile_offset = 0;
    auto launch_finish = [&](const GemmArgs &gx, uint32_t nsplits, uint64_t slots) {
        const MatmulArgs &m0 = gx.m[0];
        const uint32_t geom = (uint32_t)G::RW | ((uint32_t)MRT << 4) | ((uint32_t)NTILE << 8) | ((uint32_t)(m0.out_f16 ? 1u : 0u) << 16) |
                              (((uint32_t)m0.act & 7u) << 17);
        hipLaunchKernelGGL(gemm_finish_kernel, dim3((uint32_t)((slots + 255) / 256), (uint32_t)n), dim3(256), 0, stream, nsplits, geom,
                           (const float *)gx.scratch[0], m0.out, gx.row_tiles[0], gx.tblocks, m0.B, m0.T, m0.R, (uint32_t)m0.out_token_stride,
                           gx.split_from, gx.splits_low, gx);
    };
    ga.split_from = 0;
    ga.splits_low = 0;
    ga.prio = (uint32_t)tune(kTuneGemmPrio, 1);
    // Grid quantisation: two workgroups of the kernels with 64-token tiles or wider fit a CU, 512 run at a time (the
    // narrower tiles leave room for more, and their grids need no cut).  A grid a little above that
    // (the 576 workgroups of {ffn.key, ffn.receptance} at 128 and 256 tokens) leaves most CUs waiting for the few
    // that got a third one.  Such a launch is cut in two: the tiles that fill the CUs evenly run as they are, the
    // rest follows with K split over up to 8 times as many workgroups per tile, so that the second round is short
    // and wide.  One finish launch sums both kinds of tiles.
    const uint32_t wgs_all = total * splits;
    const uint32_t resident = 2 * cu_count(); // workgroups that run at a time at two per CU
    // (f32 activations carry a second LDS tile: one workgroup per CU, the premise of the cut does not hold for them)
    if (NTILE >= 4 && sizeof(XT) == 2 && a0.B == 1 && resident >= 64 && wgs_all > resident && wgs_all <= resident + resident / 4 && steps % splits == 0 &&
        tune(kTuneGemmTail, 1)) {
        const uint32_t even = resident / splits, rest = total - even; // tiles of the two launches
        uint32_t ks = 8 * splits;
        while (ks > splits && (rest * ks > resident || steps / ks < 2 || steps % ks != 0)) ks /= 2;
        // partial tiles of the rest lie like those of a product split `ks` times: room for every product with tiles in it
        auto planes = [&](int i, uint32_t k) { return ga.tile_begin[i] + nwg[i] > even ? k : splits > 1 ? splits : 0u; };
        auto need = [&](uint32_t k) {
            uint64_t f = 0;
            for (int i = 0; i < n; i++) f += slice[i] * planes(i, k);
            return f;
        };
        while (ks > splits && need(ks) > cap) ks /= 2;
        float *base = ks > splits ? slice_base() : nullptr;
        if (ks > splits && base) {
            GemmArgs gb = ga;
            uint64_t off = 0;
            for (int i = 0; i < n; i++) {
                gb.scratch[i] = planes(i, ks) ? base + off : nullptr;
                off += slice[i] * planes(i, ks);
            }
            gb.tile_offset = even;
            gb.split_from = even;
            gb.splits_low = splits;
            gb.k_per_split = steps / ks * kStep;
            if (splits > 1)
                for (int i = 0; i < n; i++) ga.scratch[i] = gb.scratch[i];
            hipLaunchKernelGGL(kern, dim3(even, splits, 1), dim3(G::THREADS), lds, stream, ga);
            int s = check_launch("matmul_mat");
            if (s != WRQ_OK) return s;
            hipLaunchKernelGGL(kern, dim3(rest, ks, 1), dim3(G::THREADS), lds, stream, gb);
            s = check_launch("matmul_mat (rest)");
            if (s != WRQ_OK) return s;
            uint64_t slots = 0;
            for (int i = 0; i < n; i++)
                if (gb.scratch[i]) slots = std::max(slots, slice[i] / 4);
            launch_finish(gb, ks, slots);
            return check_launch("matmul_mat (finish)");
        }
    }
    dim3 grid(total, splits, a0.B);
    hipLaunchKernelGGL(kern, grid, dim3(G::THREADS), lds, stream, ga);
    int s = check_launch("matmul_mat");
    if (s != WRQ_OK) return s;
    if (splits > 1) {
        uint64_t slots = 0; // of the largest product: smaller ones leave the rest of their grid row idle
        for (int i = 0; i < n; i++) slots = std::max(slots, slice[i] / 4);
        launch_finish(ga, splits, slots);
        s = check_launch("matmul_mat (finish)");
    }
    return s;
}

// `n` products with one K, token count and batch count (the caller groups them so).
// Measured tile choices.  web-rwkv_amd/tune_gemm.py times every tile shape and split for the launches of the RWKV model sizes
// (the four attention projections, att.output, {ffn.key, ffn.receptance}, ffn.key, ffn.value, the head; 8 .. 512 tokens) and
// writes the fastest per (format, rows, K, run-length bucket) into gemm_tuned.inc.  A launch of f16 activations on one batch
// whose rows and K lie within 7 % of a measured product takes that entry; everything else goes by the rules below.
struct TunedRow {
    uint32_t quant, rows, K;
    uint16_t cfg[18]; // MRT | NTILE << 4 | KG << 8 | split << 12 per bucket; 0: the rules decide
};
constexpr int kTunedBucketCount = 18;
constexpr uint32_t kTunedBuckets[kTunedBucketCount] = {8, 16, 24, 32, 48, 64, 80, 96, 112, 128, 160, 192, 224, 256, 320, 384, 448, 512};
const TunedRow kTuned[] = {
#include "gemm_tuned.inc"
    {~0u, 0u, 0u, {0}}, // end marker
};

uint32_t tuned_lookup(int quant, uint64_t rows, uint64_t K, uint32_t T) {
    if (T > kTunedBuckets[kTunedBucketCount - 1] || rows == 0 || K == 0) return 0;
    int b = 0;
    while (kTunedBuckets[b] < T) b++;
    uint32_t best = 0;
    uint64_t best_d = ~0ull;
    for (const TunedRow &r : kTuned) {
        if (r.quant != (uint32_t)quant || !r.cfg[b]) continue;
        const uint64_t dr = rows > r.rows ? rows - r.rows : r.rows - rows, dk = K > r.K ? K - r.K : r.K - K;
        if (dr * 100 > (uint64_t)r.rows * 7 || dk * 100 > (uint64_t)r.K * 7) continue;
        const uint64_t d = dr * 1000 / r.rows + dk * 1000 / r.K; // per mille off the measured shape
        if (d < best_d) best_d = d, best = r.cfg[b];
    }
    return best;
}

template <int QUANT, typename XT>
int launch_shape(hipStream_t stream, const MatmulArgs *args, int n, const ScratchPolicy *sp) {
    // Tile choice, from sweeps over the launch shapes of this path (rows 4096 .. 65536, K 2048 ..
    // 14336, 5 .. 256 tokens, single products and groups).  A group counts as one product with the
    // rows of all its members.  Token tile: as narrow as the run up to 32 tokens; beyond that 64
    // tokens (32 for small products with short rows), which still fetch their weights line-wise;
    // only very large products (the 65536-row head from 128 tokens on) take the 128-token tile.
    const MatmulArgs &a = args[0];
    const uint32_t T = a.T;
    const uint32_t steps = a.K / kStep;
    uint64_t rows = 0;
    for (int i = 0; i < n; i++) rows += args[i].R;
    const uint64_t rt = rows * a.B * T;
    const bool small = rt <= (1u << 20);
    // long rows against 256 tokens and more also take the 128-token tile (measured on 4096 x 14336: 7 % faster)
    // (long rows from 193 tokens on: two 128-token blocks, 4096 x 14336 at 224 tokens 54.0 against 56.6 - 59.6 us; beyond 256
    // tokens the 128-token tile from 6 M outputs on: 16384 x 4096 at 384 tokens 92 against 106 us, 18432 rows 94 against 115 us)
    int ntile = T <= 16 ? 1 : T <= 32 ? 2 : (small && a.K <= 8192 && T <= 128 && n == 1) ? 2 : (T > 64 && (rt >= (1u << 23) || (T > 256 && rt >= (6u << 20)) || (T > 192 && a.K >= 8192))) ? 8 : 4;
    int mrt = 2, kg = 1;
    uint32_t ksplit = 1, pinned_split = 0; // pinned_split: a measured choice that the rule of split_for() does not produce
    uint64_t wgs = 0; // workgroups of one split
    auto tblocks_of = [&](int nt) { return (uint64_t)(T + 16 * nt - 1) / (16 * nt); };
    // K is split over the grid until there are one (narrow tiles) to four workgroups per CU, at most
    // 8 ways.  A split launch costs one finish launch for all its products: with 64-token tiles a group is
    // split like a single product (two workgroups per CU beat one: the attention group at 128 tokens 42.4
    // against 46.2 us, nf4 at 64 tokens 35.8 against 43.7 us), with narrower tiles a group that fills most
    // CUs stays unsplit
    auto split_for = [&]() {
        wgs = (uint64_t)((rows * kg + 64 * mrt - 1) / (64 * mrt)) * tblocks_of(ntile) * a.B;
        // (64-token tiles of long rows: three workgroups per CU still pay -- 4096 x 14336 at 160 and 192 tokens, 96 tiles: an
        // 8-way split 50.4 / 51.2 us against 53.7 / 54.0 us with 4)
        const uint64_t target = ntile <= 2 ? 256 : ntile == 4 ? (steps >= 64 ? 768 : 640) : 1024;
        ksplit = 1;
        while (kg == 1 && ksplit < 8 && wgs * ksplit * 2 <= target && steps / (ksplit * 2) >= 4) ksplit *= 2;
        if (n >= 2 && wgs >= 200 && ntile != 4) ksplit = 1;
        if (pinned_split) ksplit = pinned_split;
    };
    // 64-row tiles where they give about one workgroup per CU without a split of K (a 16-token tile:
    // also below that); otherwise 128-row tiles, fewer activation copies per weight byte, and more splits
    const uint64_t wgs64 = (uint64_t)((rows + 63) / 64) * tblocks_of(ntile) * a.B;
    if ((ntile == 1 && wgs64 <= 256) || (ntile == 2 && wgs64 >= 200 && wgs64 <= 256)) mrt = 1;
    if (QUANT != kFp16 && wgs64 >= 200 && wgs64 <= 320 && (ntile == 1 || (QUANT == kNf4 && ntile == 2))) {
        // about one 64-row workgroup per CU at a narrow token tile: two workgroups of 32 rows with two
        // k groups each keep twice the weight bytes in flight per CU
        mrt = 1;
        kg = 2;
    }
    // The choices below were checked against a sweep of all sixteen tile shapes x four splits per launch kind of the 7B layer
    // ({att.k, v, r, g}, att.output, {ffn.key, ffn.receptance}, ffn.value) at 4 .. 256 tokens, both formats.
    if (QUANT == kInt8 && ntile == 2 && wgs64 >= 200 && wgs64 <= 256) {
        // int8, 17 .. 32 tokens, about 16384 rows: 64 rows x 32 tokens with two k groups (the attention group 20.2 - 20.7 us
        // against 22.6 - 22.9 us with 64-row tiles of one k group)
        mrt = 2;
        kg = 2;
    }
    if (QUANT == kNf4 && ntile == 2 && wgs64 > 256 && wgs64 <= 320) {
        // nf4, 17 .. 32 tokens, a little more than one 64-row tile per CU ({ffn.key, ffn.receptance}): the same tile with K
        // split four ways over the grid, 29.4 - 30.4 us against 33.0 - 34.2 us unsplit with 32-row tiles
        mrt = 2;
        kg = 2;
        pinned_split = 4;
    }
    if (QUANT == kNf4 && n == 1 && a.B == 1 && a.K > 8192 && rows > 2048 && rows <= 4096 && T <= 32) {
        // nf4, a small product with long rows (ffn.value) at up to 32 tokens: 64 rows x two k groups, K split 8 ways
        // (19.4 - 19.7 us against 21.1 - 21.5 us up to 16 tokens, 22.2 - 22.8 against 24.0 from 17 on)
        mrt = 2;
        kg = 2;
        pinned_split = 8;
    }
    if (QUANT != kFp16 && T > 64 && T <= 96 && ntile == 4 && a.B == 1) {
        // 65 .. 96 tokens are three 32-token blocks or two 64-token blocks, the second one at most half full.  Where the wide
        // blocks give a little more than one 128-row tile per CU (and the grid then needs a split and a cut), the narrow ones
        // fill the CUs unsplit: {ffn.key, ffn.receptance} 40.5 - 41.2 us against 48 - 50 us (int8), 56 against 60 - 61 us (nf4)
        const uint64_t row_tiles = (rows + 127) / 128;
        if (row_tiles * 2 > 256 && row_tiles * 3 <= 512) {
            ntile = 2;
            pinned_split = 1;
        }
    }
    if (QUANT == kInt8 && n == 1 && a.B == 1 && a.K <= 8192 && rows > 2048 && rows <= 4096 && T > 16 && T <= 64) {
        // int8, a small single product (att.output) at 17 .. 64 tokens: 32 rows x 16 tokens with two k groups and no split over
        // the grid -- no partial sums, no finish launch (11.7 - 11.9 us against 12.8 - 13.4 us up to 32 tokens, 14.2 - 14.7
        // against 14.3 - 15.3 us up to 64)
        ntile = 1;
        mrt = 1;
        kg = 2;
    }
    if (QUANT != kFp16 && n == 1 && a.B == 1 && a.K <= 4096 && rows > 1024 && rows <= 2048 && T > 256) {
        // a small single product with short rows beyond 256 tokens: 64 rows x 32 tokens with two k groups, unsplit
        // (2048 x 2048 at 384 / 512 tokens: int8 14.9 / 15.1 against 19.6 / 20.4 us, nf4 18.5 / 18.9 against 21.8 / 24.2 us)
        ntile = 2;
        mrt = 2;
        kg = 2;
    }
    if (QUANT == kNf4 && n == 1 && a.B == 1 && a.K <= 8192 && rows > 2048 && rows <= 4096 && T <= 128) {
        // a small single product gets its workgroups from k groups instead of a split over the grid
        // (measured on 4096 x 4096: no scratch round trip, no finish launch)
        ntile = T <= 16 ? 1 : 2;
        mrt = T > 128 ? 2 : 1;
        kg = T <= 32 ? 4 : 2;
    }
    if (QUANT == kInt8 && n == 1 && a.B == 1 && a.K <= 8192 && rows > 2048 && rows <= 4096 && T > 64 && T <= 128) {
        // the same for int8 at 65 .. 128 tokens (4096 x 4096 x 128: 19.9 us against 23.7 us with a split over the grid)
        ntile = 2;
        mrt = 2;
        kg = 2;
    }
    bool measured = false;
    if (QUANT != kFp16 && sizeof(XT) == 2 && a.B == 1 && tune(kTuneGemmTable, 1)) {
        if (const uint32_t c = tuned_lookup(QUANT, rows, a.K, T)) {
            mrt = (int)(c & 15u), ntile = (int)((c >> 4) & 15u), kg = (int)((c >> 8) & 15u), pinned_split = c >> 12;
            measured = true;
        }
    }
    split_for();
    if (QUANT == kInt8 && kg == 1 && T > 64 && !measured) {
        // two workgroups fit a CU (512 slots).  A grid of 64-token tiles that fills half of them runs at
        // one wave per SIMD: 32-token tiles double it.
        if (ntile == 4 && wgs * ksplit <= 256) {
            ntile = 2;
            split_for();
        }
    }
    ntile = tune(kTuneGemmNtile, ntile);
    mrt = tune(kTuneGemmMrt, mrt);
    kg = tune(kTuneGemmKg, kg);
    if (kg != 1 && kg != 2 && kg != 4) kg = 1;
    if (kg == 4 && (mrt != 1 || ntile > 2)) kg = 2;
    if (kg == 2 && ntile > 4) kg = 1;
    if (tune_is_set(kTuneGemmNtile) || tune_is_set(kTuneGemmMrt) || tune_is_set(kTuneGemmKg)) {
        pinned_split = 0; // a pinned tile shape takes the split of the general rule
        split_for();
    }
    ksplit = (uint32_t)tune(kTuneGemmKsplit, (int)ksplit);
    if (ksplit < 1) ksplit = 1;

    if (sizeof(XT) == 4 && (ntile == 8 || (mrt == 2 && ntile == 4 && kg == 2))) {
        // f32 activations keep a second (lo) activation tile and a second set of products: the widest tiles
        // would not fit the registers, and 128 rows x 64 tokens x 2 k groups not the LDS
        if (ntile == 8) ntile = 4;
        if (mrt == 2 && ntile == 4) kg = 1;
        split_for();
        ksplit = (uint32_t)tune(kTuneGemmKsplit, (int)ksplit); // a pinned split survives the adjustment
        if (ksplit < 1) ksplit = 1;
    }
#define WRQ_CASE(M, N, G) \
    if (mrt == M && ntile == N && kg == G) return launch_one<QUANT, XT, M, N, G>(stream, args, n, ksplit, sp);
    WRQ_CASE(1, 1, 1) WRQ_CASE(1, 2, 1) WRQ_CASE(1, 4, 1) WRQ_CASE(1, 8, 1)
    WRQ_CASE(2, 1, 1) WRQ_CASE(2, 2, 1) WRQ_CASE(2, 4, 1) WRQ_CASE(2, 8, 1)
    WRQ_CASE(1, 1, 2) WRQ_CASE(1, 2, 2) WRQ_CASE(1, 4, 2)
    WRQ_CASE(2, 1, 2) WRQ_CASE(2, 2, 2) WRQ_CASE(2, 4, 2)
    WRQ_CASE(1, 1, 4) WRQ_CASE(1, 2, 4)
#undef WRQ_CASE
    return launch_one<QUANT, XT, 1, 2, 1>(stream, args, n, ksplit, sp);
}

} // namespace

int prepare_gemm_scratch() {
    return scratch_base() && static_scratch_ptr() ? WRQ_OK : fail(WRQ_ERR_DEVICE, "split-K scratch not resolvable");
}

int launch_gemm_noalloc(hipStream_t stream, Quant quant, int in_f16, const MatmulArgs &a) {
    float *base = static_scratch_ptr(); // looked up by wrq_init, or here on the first call on this device
    if (!base) return fail(WRQ_ERR_DEVICE, "fixed scratch array not resolvable");
    const ScratchPolicy sp{base, kStaticScratchFloats, true};
    return launch_gemm_group(stream, quant, in_f16, &a, 1, &sp);
}

// Preconditions (checked by the caller): K % 128 == 0, R % 4 == 0, 16-byte aligned
// activation rows and output rows of 4.
int launch_gemm(hipStream_t stream, Quant quant, int in_f16, const MatmulArgs &a) {
    return launch_gemm_group(stream, quant, in_f16, &a, 1, nullptr);
}

// `n` <= kMaxGroup independent products of one quantisation and input type; those that share K,
// T and B = 1 go into one launch, the others are launched one by one.
int launch_gemm_group(hipStream_t stream, Quant quant, int in_f16, const MatmulArgs *args, int n, const ScratchPolicy *sp) {
    int i = 0;
    while (i < n) {
        if (args[i].R == 0 || args[i].T == 0 || args[i].B == 0) {
            i++;
            continue;
        }
        int m = 1;
        if (args[i].B == 1)
            while (i + m < n && m < kMaxGroup && args[i + m].B == 1 && args[i + m].R > 0 && args[i + m].K == args[i].K &&
                   args[i + m].T == args[i].T)
                m++;
        int s;
        if (quant == kInt8)
            s = in_f16 ? launch_shape<kInt8, __half>(stream, args + i, m, sp) : launch_shape<kInt8, float>(stream, args + i, m, sp);
        else if (quant == kFp16)
            s = in_f16 ? launch_shape<kFp16, __half>(stream, args + i, m, sp) : launch_shape<kFp16, float>(stream, args + i, m, sp);
        else
            s = in_f16 ? launch_shape<kNf4, __half>(stream, args + i, m, sp) : launch_shape<kNf4, float>(stream, args + i, m, sp);
        if (s != WRQ_OK) return s;
        i += m;
    }
    return WRQ_OK;
}

} // namespace wrq

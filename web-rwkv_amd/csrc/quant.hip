// Weight packing for gfx950: quant_mat_int8 and quant_mat_nf4.
//
// Both are single-pass, bandwidth-bound kernels (2 B read, 1 or 0.5 B written per
// element): a block of the quantisation grid is held by 16 (int8) or 8 (nf4)
// adjacent lanes with one 16-byte load each, the block statistic is reduced with
// DPP inside the lane group, and every lane packs its own eight elements.  The
// reference's two/three dispatches per matrix (statistics, quantise, f32->f16 blit;
// src/tensor/ops.rs:2393-2486, :2488-2589) collapse into one launch with no
// temporary.  Workgroups are resident and walk the matrix with a grid stride, the next
// 16 bytes of a lane already in flight while it packs the current ones.
//
// The results are the reference shaders' results bit for bit
// (src/shaders/quant_mat_int8.wgsl:24-59, quant_mat_nf4.wgsl:24-81): IEEE f32
// division, no fused operations on the shaders' own expressions (this file is built with
// -ffp-contract=off), round-half-even for the unorm code, `<=` scan so that the last
// minimum wins.  Two places reach those results with fewer instructions per element than
// the literal expression; both are exact, not approximations:
//  * int8: the 8 quotients of a lane share their divisor, so the reciprocal refinement of
//    the correctly rounded division sequence is done once per lane (div_shared);
//  * nf4: for a table in ascending order the 16-way scan equals counting the decision
//    thresholds <= x; the 15 thresholds are found per launch by bisection on the scan's own
//    comparison (nf4_threshold) and the count is one LDS lookup on a 256-cell grid plus one
//    comparison; any other table takes the literal scan.
#include "wrq_device.h"
#include "wrq_host.h"

namespace wrq {

// Packed output is written once and not read by the kernel: streaming stores let it leave the
// cache while the kernel runs instead of in the write-back at its end.
__device__ __forceinline__ void store64_stream(void *p, uint32_t lo, uint32_t hi) {
    u32x2 v;
    v.x = lo;
    v.y = hi;
    __builtin_nontemporal_store(v, reinterpret_cast<u32x2 *>(p));
}

__device__ __forceinline__ float dpp_f(float v, int ctrl) {
    switch (ctrl) {
    case 0: return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xf, 0xf, true));
    case 1: return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xf, 0xf, true));
    case 2: return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xf, 0xf, true));
    default: return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xf, 0xf, true));
    }
}

// Large workgroups, few of them: workgroups are handed out at a limited rate, and a packer's
// whole run is a handful of microseconds.
constexpr uint32_t kPackThreads = 1024;

// Resident grid: two workgroups of 16 waves per CU, never more than the work.
static uint32_t resident_grid(uint64_t ngroup) {
    const uint64_t need = (ngroup + kPackThreads - 1) / kPackThreads;
    const uint64_t cap = 256 * 2;
    return (uint32_t)(need < cap ? need : cap);
}

// ---------------------------------------------------------------------------------- int8

// Correctly rounded a / b for one divisor and many dividends.  This is the sequence the
// compiler emits for an IEEE f32 division (reciprocal estimate, one refinement of the
// reciprocal, two of the quotient) without its range scaling and special-case fix-up, with
// the divisor's part hoisted.  Here a = v - min and b = max - min come from f16 values, so
// both lie in [2^-24, 2^17] or are 0 and no step leaves the normal range.  b == 0 (constant
// block), an infinite b and NaN give NaN or 0 where IEEE gives NaN or 0; the caller's clamp
// maps both to code 0.
__device__ __forceinline__ float recip_refined(float b) {
    const float r0 = __builtin_amdgcn_rcpf(b);
    const float e = fmaf(-b, r0, 1.0f);
    return fmaf(e, r0, r0);
}

__device__ __forceinline__ float div_shared(float a, float b, float r) {
    float q = a * r;
    float e = fmaf(-b, q, a);
    q = fmaf(e, r, q);
    e = fmaf(-b, q, a);
    return fmaf(e, r, q);
}

// Groups of 8 elements a lane packs per pass over its loop; the loads of the next pass are
// issued before the current one is packed, so a wave keeps 2 * kPassGroups KiB in flight.
// Measured: 4 groups per pass (68 - 82 registers, 5 - 7 waves per SIMD) are 5 - 15 % slower than 1
// (26 - 41 registers, 8 waves) on every shape.
constexpr int kPassGroups = 1;

// One lane per 8 elements; 16 lanes (one DPP row) per 128-element block.  ngroup is a
// multiple of 16, so a row of lanes is live or idle as a whole.
__global__ __launch_bounds__(kPackThreads) void quant_int8_kernel(const uint16_t *__restrict__ in,
                                                         uint32_t *__restrict__ minmax,
                                                         uint8_t *__restrict__ out, uint64_t ngroup) {
    const uint64_t stride = (uint64_t)gridDim.x * kPackThreads;
    uint64_t gid = (uint64_t)blockIdx.x * kPackThreads + threadIdx.x;
    uint4 raw[kPassGroups];
#pragma unroll
    for (int u = 0; u < kPassGroups; u++) {
        raw[u] = make_uint4(0, 0, 0, 0);
        if (gid + u * stride < ngroup) raw[u] = load128_stream(in + (gid + u * stride) * 8);
    }
    while (gid < ngroup) {
        const uint64_t next = gid + kPassGroups * stride;
        uint4 raw_next[kPassGroups];
#pragma unroll
        for (int u = 0; u < kPassGroups; u++) {
            raw_next[u] = make_uint4(0, 0, 0, 0);
            if (next + u * stride < ngroup) raw_next[u] = load128_stream(in + (next + u * stride) * 8);
        }
#pragma unroll
        for (int u = 0; u < kPassGroups; u++) {
            const uint64_t g = gid + u * stride;
            if (g >= ngroup) break;
            float v[8];
            unpack8h(raw[u], v);
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
            const float rr = recip_refined(range);
            uint32_t code[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                // 0 <= v - mn <= range after rounding, so q <= 1 needs no clamp; NaN (constant
                // block, infinities) -> 0
                const float q = fmaxf(div_shared(v[i] - mn, range, rr), 0.0f);
                // adding 2^23 rounds q * 255 (in [0, 255]) to an integer, half to even, and leaves
                // it in the low byte
                code[i] = __float_as_uint(q * 255.0f + 0x1p23f);
            }
            const uint32_t lo = __builtin_amdgcn_perm(__builtin_amdgcn_perm(code[3], code[2], 0x0c0c0400u),
                                                      __builtin_amdgcn_perm(code[1], code[0], 0x0c0c0400u), 0x05040100u);
            const uint32_t hi = __builtin_amdgcn_perm(__builtin_amdgcn_perm(code[7], code[6], 0x0c0c0400u),
                                                      __builtin_amdgcn_perm(code[5], code[4], 0x0c0c0400u), 0x05040100u);
            store64_stream(out + g * 8, lo, hi);
            if ((g & 15) == 0) minmax[g >> 4] = (uint32_t)f2h(mn) | ((uint32_t)f2h(mx) << 16);
        }
        gid = next;
#pragma unroll
        for (int u = 0; u < kPassGroups; u++) raw[u] = raw_next[u];
    }
}

// ----------------------------------------------------------------------------------- nf4

// f32 <-> unsigned key with the same order as the values (finite values and infinities).
__device__ __forceinline__ uint32_t f32_key(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_f32(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// The scan of quant_mat_nf4.wgsl:62-72 prefers entry j+1 to entry j exactly when this holds.
__device__ __forceinline__ bool nf4_prefers_upper(float qa, float qb, float xx) {
    return fabsf(qb - xx) <= fabsf(qa - xx);
}

// Smallest f32 x for which the scan prefers qb (the upper entry) to qa.  Rounding is monotone,
// so the comparison is false at qa, true at qb and changes once in between: bisection over
// the ordered keys finds the exact switch point, rounding of the two differences included.
__device__ __forceinline__ float nf4_threshold(float qa, float qb) {
    // the switch point is within rounding of the midpoint: try a narrow bracket first
    const float mid = 0.5f * (qa + qb);
    const float wl = fmaxf(qa, mid - 0x1p-21f), wh = fminf(qb, mid + 0x1p-21f);
    uint32_t lo = f32_key(qa), hi = f32_key(qb);
    if (!nf4_prefers_upper(qa, qb, wl)) lo = f32_key(wl);
    if (nf4_prefers_upper(qa, qb, wh)) hi = f32_key(wh);
    while (hi - lo > 1) {
        const uint32_t m = lo + ((hi - lo) >> 1);
        if (nf4_prefers_upper(qa, qb, key_f32(m)))
            hi = m;
        else
            lo = m;
    }
    return key_f32(hi);
}

// Cell of x on a uniform grid of 256 cells over [-1, 1]; monotone in x, NaN -> 0.
__device__ __forceinline__ uint32_t nf4_cell(float x) {
    const float f = fminf(fmaxf(fmaf(x, 128.0f, 128.0f), 0.0f), 255.0f);
    return (uint32_t)f;
}

// One lane per 8 elements (one output u32); 8 lanes per 64-element block.  ngroup is a
// multiple of 8, so a lane group is live or idle as a whole.
__global__ __launch_bounds__(kPackThreads) void quant_nf4_kernel(const uint16_t *__restrict__ in,
                                                        const float *__restrict__ quant,
                                                        uint16_t *__restrict__ absmax,
                                                        uint32_t *__restrict__ out, uint64_t ngroup) {
    __shared__ uint2 lut[256]; // per cell: (threshold inside the cell or +inf, thresholds below the cell)
    __shared__ float thr_value[15];
    __shared__ uint32_t thr_cell[16]; // [15]: whether the table qualifies for the search path
    const uint64_t stride = (uint64_t)gridDim.x * kPackThreads;
    uint64_t gid = (uint64_t)blockIdx.x * kPackThreads + threadIdx.x;
    uint4 raw[kPassGroups]; // in flight during the threshold search
#pragma unroll
    for (int u = 0; u < kPassGroups; u++) {
        raw[u] = make_uint4(0, 0, 0, 0);
        if (gid + u * stride < ngroup) raw[u] = load128_stream(in + (gid + u * stride) * 8);
    }

    // Lane j < 15 of the first wave looks at the table interval [q[j], q[j+1]].  The search path
    // needs: ascending entries at least 2^-20 apart (then the rounded errors of two entries on
    // the same side of x differ, and the minimum is one of the two neighbours of x), no
    // interval wider than 1 and ends in [-1, -0.5] and [0.5, 1] (then the nearest entry of any
    // x = v / absmax is within the scan's initial bound of 1.0), and no two thresholds in one
    // cell of the grid.  The scan's answer is then the number of thresholds <= x: those in
    // cells below x's cell (cells are monotone in x) plus one comparison inside the cell.
    if (threadIdx.x < 64) {
        const uint32_t lane = threadIdx.x;
        const uint32_t j = lane < 15 ? lane : 14;
        const float qa = quant[j], qb = quant[j + 1];
        bool ok = (qb - qa >= 0x1p-20f) && (qb - qa <= 1.0f);
        if (lane == 0) ok = ok && qa >= -1.0f && qa <= -0.5f;
        if (lane >= 14) ok = ok && qb >= 0.5f && qb <= 1.0f;
        bool usable = __ballot(ok) == ~0ull;
        float mine = 0.0f;
        uint32_t cell = 0;
        if (usable) {
            mine = nf4_threshold(qa, qb);
            cell = nf4_cell(mine);
            const uint32_t upper = (uint32_t)__shfl_down((int)cell, 1);
            usable = __ballot(lane >= 14 || cell != upper) == ~0ull;
        }
        if (lane < 15) {
            thr_value[lane] = mine;
            thr_cell[lane] = cell;
        }
        if (lane == 15) thr_cell[15] = usable ? 1u : 0u;
    }
    lds_barrier(); // the first loads stay in flight
    const bool search = __builtin_amdgcn_readfirstlane((int)thr_cell[15]) != 0;

    if (search) {
        if (threadIdx.x < 256) {
            uint32_t below = 0, inside = 0x7f800000u; // +inf: never reached by x
#pragma unroll
            for (int k = 0; k < 15; k++) {
                const uint32_t c = thr_cell[k];
                below += c < threadIdx.x ? 1u : 0u;
                if (c == threadIdx.x) inside = __float_as_uint(thr_value[k]);
            }
            lut[threadIdx.x] = make_uint2(inside, below);
        }
        lds_barrier();
        while (gid < ngroup) {
            const uint64_t next = gid + kPassGroups * stride;
            uint4 raw_next[kPassGroups];
#pragma unroll
            for (int u = 0; u < kPassGroups; u++) {
                raw_next[u] = make_uint4(0, 0, 0, 0);
                if (next + u * stride < ngroup) raw_next[u] = load128_stream(in + (next + u * stride) * 8);
            }
#pragma unroll
            for (int u = 0; u < kPassGroups; u++) {
                const uint64_t g = gid + u * stride;
                if (g >= ngroup) break;
                float v[8];
                unpack8h(raw[u], v);
                float am = 0.0f;
#pragma unroll
                for (int i = 0; i < 8; i++) am = fmaxf(fabsf(v[i]), am);
#pragma unroll
                for (int s = 0; s < 3; s++) am = fmaxf(am, dpp_f(am, s)); // 8 lanes: two quad steps + half mirror
                const float inv = __fdiv_rn(1.0f, am); // quant_mat_nf4.wgsl:59
                uint32_t y = 0;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const float xx = v[i] * inv; // NaN in an all-zero block: cell 0, comparison false, nibble 0
                    const uint2 e = lut[nf4_cell(xx)];
                    const uint32_t idx = e.y + (xx >= __uint_as_float(e.x) ? 1u : 0u);
                    y |= idx << (4 * i);
                }
                __builtin_nontemporal_store(y, out + g);
                if ((g & 7) == 0) absmax[g >> 3] = f2h(am);
            }
            gid = next;
#pragma unroll
            for (int u = 0; u < kPassGroups; u++) raw[u] = raw_next[u];
        }
        return;
    }

    // any other table: the scan as written in the shader
    if (gid >= ngroup) return;
    float q[16];
#pragma unroll
    for (int k = 0; k < 16; k++) q[k] = quant[k];
    uint4 cur = raw[0];
    while (true) {
        float v[8];
        unpack8h(cur, v);
        float am = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) am = fmaxf(fabsf(v[i]), am);
#pragma unroll
        for (int s = 0; s < 3; s++) am = fmaxf(am, dpp_f(am, s));
        const float inv = __fdiv_rn(1.0f, am);
        uint32_t y = 0;
#pragma unroll 2 // the rare path: kept small so that it does not set the kernel's register count
        for (int i = 0; i < 8; i++) {
            const float xx = v[i] * inv;
            float min_err = 1.0f;
            uint32_t min_index = 0;
#pragma unroll
            for (int k = 0; k < 16; k++) {
                const float err = fabsf(q[k] - xx);
                if (err <= min_err) { // false for NaN: an all-zero block packs to nibble 0
                    min_err = err;
                    min_index = k;
                }
            }
            y |= min_index << (4 * i);
        }
        out[gid] = y;
        if ((gid & 7) == 0) absmax[gid >> 3] = f2h(am);
        gid += stride;
        if (gid >= ngroup) break;
        cur = load128_stream(in + gid * 8);
    }
}

int launch_quant_int8(hipStream_t stream, const void *in, void *minmax, void *out, uint64_t len) {
    const uint64_t ngroup = len / 8;
    if (ngroup == 0) return WRQ_OK;
    hipLaunchKernelGGL(quant_int8_kernel, dim3(resident_grid(ngroup)), dim3(kPackThreads), 0, stream,
                       (const uint16_t *)in, (uint32_t *)minmax, (uint8_t *)out, ngroup);
    return check_launch("quant_mat_int8");
}

int launch_quant_nf4(hipStream_t stream, const void *in, const void *quant, void *absmax, void *out,
                     uint64_t len) {
    const uint64_t ngroup = len / 8;
    if (ngroup == 0) return WRQ_OK;
    hipLaunchKernelGGL(quant_nf4_kernel, dim3(resident_grid(ngroup)), dim3(kPackThreads), 0, stream,
                       (const uint16_t *)in, (const float *)quant, (uint16_t *)absmax, (uint32_t *)out,
                       ngroup);
    return check_launch("quant_mat_nf4");
}

} // namespace wrq

// Fused forms of the small ops of an RWKV-v6 layer (src/runtime/v6.rs:758-955).  At batch 1 every
// op of a layer is bound by its launch (about 2.3 us under HIP-graph replay, 27 of them per layer
// beside the 8 quantized products); these entry points do the work of 3 - 5 consecutive ops of the
// reference's list in one launch each and bring a layer from 35 launches to 12.  Each computes what the
// op list computes, with the same roundings where the list stores an f16 buffer in between:
//   wrq_v6_pre          (add) + blit + layer_norm + token_shift x 1..2     v6.rs:759-777, :906-933
//   wrq_v6_time_mix     transpose + time_mix_w2 + add + token_shift(5)     v6.rs:785-805
//   wrq_v6_decay        time_decay_w2 + add + activate(StableExp)          v6.rs:839-848
//   wrq_v6_wkv_gate     blit + time_mix_v6 + group_norm + blit + mul(Silu) v6.rs:851-887
//   wrq_v6_post_ffn     channel_mix + add (+ affine 0.5)                   v6.rs:942-955
// They have no counterpart among the reference's constructors; buffers are the f16 / f32 tensors of
// `Runtime<f16>` (v6.rs:270-303), contiguous, [C, A, 1, 1].
#include "layer_device.h"

namespace wrq {

namespace {

constexpr int kPreThreads = 256;
constexpr int kPreCache = 8; // 4-element vectors a thread keeps of a row: rows up to 8192 elements

__device__ __forceinline__ float round_h(float v) { return h2f(f2h(v)); }

// One workgroup per token.  row = x[t] (+ add[t]), written to x_out when given; ln = f16(LN(row)) -> ln_out;
// shift_out[s][t] = f16(mix(ln, prev, factor[s])) with prev = the request's state row for its first
// token of the stack, else f16(LN(row t-1)) recomputed here.
template <int NS>
__global__ __launch_bounds__(kPreThreads) void v6_pre_kernel(const uint32_t *cursors, const uint16_t *x, const uint16_t *add, uint16_t *x_out,
                                                             const uint16_t *ln_w, const uint16_t *ln_b, float eps, const float *state, ViewArgs vs,
                                                             const uint16_t *factor0, const uint16_t *factor1, uint16_t *ln_out, uint16_t *shift0,
                                                             uint16_t *shift1, uint32_t C) {
    __shared__ float red[kPreThreads / 64];
    const uint32_t t = blockIdx.x, nv = C / 4;
    // Everything that does not depend on the row statistics is requested first: a workgroup is a chain of
    // dependent memory round trips otherwise (cursor, row, weights after the reductions, state, factors),
    // and at one token per launch that chain is the kernel's whole time.
    uint2 wq[kPreCache], bq[kPreCache], fq[NS][kPreCache];
#pragma unroll
    for (int c = 0; c < kPreCache; c++) {
        const uint32_t i = threadIdx.x + c * kPreThreads;
        if (i < nv) {
            wq[c] = *reinterpret_cast<const uint2 *>(ln_w + 4 * i);
            bq[c] = *reinterpret_cast<const uint2 *>(ln_b + 4 * i);
#pragma unroll
            for (int s = 0; s < NS; s++) fq[s][c] = *reinterpret_cast<const uint2 *>((s == 0 ? factor0 : factor1) + 4 * i);
        }
    }
    auto unpack = [](uint2 v) {
        return make_float4(h2f((uint16_t)(v.x & 0xffffu)), h2f((uint16_t)(v.x >> 16)), h2f((uint16_t)(v.y & 0xffffu)), h2f((uint16_t)(v.y >> 16)));
    };
    const Cursor cur = read_cursor(cursors, t, vs);
    const bool first = t == cur.token;
    float4 pst[kPreCache]; // the request's state row, for its first token of the stack
    if (first) {
#pragma unroll
        for (int c = 0; c < kPreCache; c++) {
            const uint32_t i = threadIdx.x + c * kPreThreads;
            if (i < nv) pst[c] = load_vec4(state + view_elem(vs, cur.batch, 0, 4 * i));
        }
    }
    // rows t (which = 0) and t - 1 (which = 1): normalised, rounded to f16 as the op list stores them
    float4 ln[2][kPreCache];
#pragma unroll
    for (int which = 0; which < 2; which++) {
        if (which == 1 && first) break;
        const uint64_t base = (uint64_t)(t - which) * C;
        float4 row[kPreCache];
        float part = 0.0f;
#pragma unroll
        for (int c = 0; c < kPreCache; c++) {
            const uint32_t i = threadIdx.x + c * kPreThreads;
            if (i < nv) {
                float4 v = load_vec4(x + base + 4 * i);
                if (add) {
                    const float4 a = load_vec4(add + base + 4 * i);
                    v = make_float4(round_h(a.x + v.x), round_h(a.y + v.y), round_h(a.z + v.z), round_h(a.w + v.w));
                    if (which == 0) store_vec4(x_out + base + 4 * i, v);
                }
                row[c] = v;
                part += (v.x + v.y) + (v.z + v.w);
            }
        }
        const float mean = block_reduce<false, kPreThreads>(part, red) / (float)C;
        float acc = 0.0f;
#pragma unroll
        for (int c = 0; c < kPreCache; c++)
            if (threadIdx.x + c * kPreThreads < nv) {
                const float4 v = row[c];
                acc += ((v.x - mean) * (v.x - mean) + (v.y - mean) * (v.y - mean)) + ((v.z - mean) * (v.z - mean) + (v.w - mean) * (v.w - mean));
            }
        const float dev = rsqrtf(block_reduce<false, kPreThreads>(acc, red) / (float)C + eps);
#pragma unroll
        for (int c = 0; c < kPreCache; c++) {
            const uint32_t i = threadIdx.x + c * kPreThreads;
            if (i < nv) {
                const float4 v = row[c], w = unpack(wq[c]), b = unpack(bq[c]);
                ln[which][c] = make_float4(round_h(fmaf((v.x - mean) * dev, w.x, b.x)), round_h(fmaf((v.y - mean) * dev, w.y, b.y)),
                                           round_h(fmaf((v.z - mean) * dev, w.z, b.z)), round_h(fmaf((v.w - mean) * dev, w.w, b.w)));
                if (which == 0) store_vec4(ln_out + base + 4 * i, ln[0][c]);
            }
        }
    }
#pragma unroll
    for (int c = 0; c < kPreCache; c++) {
        const uint32_t i = threadIdx.x + c * kPreThreads;
        if (i >= nv) continue;
        const float4 p = first ? pst[c] : ln[1][c];
        const float4 a = ln[0][c];
        auto mix = [](float xx, float pp, float f) { return xx * (1.0f - f) + pp * f; }; // reversed token shift: mix(x, prev, f)
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const float4 f = unpack(fq[s][c]);
            store_vec4((s == 0 ? shift0 : shift1) + (uint64_t)t * C + 4 * i, make_float4(mix(a.x, p.x, f.x), mix(a.y, p.y, f.y), mix(a.z, p.z, f.z), mix(a.w, p.w, f.w)));
        }
    }
}

// thread = (token, channel c): f[s] = f16(f16(sum_k w2[s][c][k] lora[t][s][k]) + time_mix[s][c]),
// out[s][t][c] = f16(mix(att_x[t][c], prev[c], f[s])), s = 0..4
template <int KL>
__global__ __launch_bounds__(256) void v6_time_mix_kernel(const uint32_t *cursors, const uint16_t *lora, const uint16_t *w2, const uint16_t *time_mix,
                                                          const float *state, ViewArgs vs, const uint16_t *att_x, uint16_t *out, uint32_t C, uint32_t A) {
    __shared__ __align__(16) uint16_t ls[5 * KL];
    const uint32_t t = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
    const uint32_t cc = min(c, C - 1); // threads past the row repeat its last channel and store nothing
    // every operand is requested before the first wait: the rows of w2, the mix vectors, the token and the
    // one before it (the state row needs the cursor: one more round trip, for a request's first token only)
    uint4 wv[5][KL / 8];
    float tm[5];
#pragma unroll
    for (int s = 0; s < 5; s++) {
        const uint16_t *wrow = w2 + ((uint64_t)s * C + cc) * KL;
#pragma unroll
        for (int k8 = 0; k8 < KL / 8; k8++) wv[s][k8] = load128(wrow + 8 * k8);
        tm[s] = h2f(time_mix[(uint64_t)s * C + cc]);
    }
    const Cursor cur = read_cursor(cursors, t, vs);
    const float a = h2f(att_x[(uint64_t)t * C + cc]);
    const float before = h2f(att_x[(uint64_t)(t ? t - 1 : 0) * C + cc]);
    for (uint32_t e = threadIdx.x; e < 5 * KL / 8; e += 256) *reinterpret_cast<uint4 *>(&ls[8 * e]) = load128(lora + (uint64_t)t * 5 * KL + 8 * e);
    const float p = t == cur.token ? state[view_elem(vs, cur.batch, 0, cc)] : before;
    lds_barrier();
    if (c >= C) return;
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int s = 0; s < 5; s++) {
        float acc = 0.0f;
#pragma unroll
        for (int k8 = 0; k8 < KL / 8; k8++) {
            const uint4 xv = *reinterpret_cast<const uint4 *>(&ls[s * KL + 8 * k8]);
            acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, wv[s][k8].x), __builtin_bit_cast(h2, xv.x), acc, false);
            acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, wv[s][k8].y), __builtin_bit_cast(h2, xv.y), acc, false);
            acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, wv[s][k8].z), __builtin_bit_cast(h2, xv.z), acc, false);
            acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, wv[s][k8].w), __builtin_bit_cast(h2, xv.w), acc, false);
        }
        const float f = round_h(round_h(acc) + tm[s]);
        out[((uint64_t)s * A + t) * C + c] = f2h(a * (1.0f - f) + p * f);
    }
}

// thread = (token, channel c): out[t][c] = exp(-exp(sum_k w2[c][k] lora[t][k] + time_decay[c])) in f32
template <int KL>
__global__ __launch_bounds__(256) void v6_decay_kernel(const uint16_t *lora, const uint16_t *w2, const uint16_t *time_decay, float *out, uint32_t C) {
    __shared__ __align__(16) uint16_t ls[KL];
    const uint32_t t = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
    const uint32_t cc = min(c, C - 1); // threads past the row repeat its last channel and store nothing
    // the row of w2 and the bias are requested together with the token's vector, before the first wait
    const uint16_t *wrow = w2 + (uint64_t)cc * KL;
    uint4 wv[KL / 8];
#pragma unroll
    for (int k8 = 0; k8 < KL / 8; k8++) wv[k8] = load128(wrow + 8 * k8);
    const float bias = h2f(time_decay[cc]);
    for (uint32_t e = threadIdx.x; e < KL / 8; e += 256) *reinterpret_cast<uint4 *>(&ls[8 * e]) = load128(lora + (uint64_t)t * KL + 8 * e);
    lds_barrier();
    if (c >= C) return;
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    float acc = 0.0f;
#pragma unroll
    for (int k8 = 0; k8 < KL / 8; k8++) {
        const uint4 xv = *reinterpret_cast<const uint4 *>(&ls[8 * k8]);
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, wv[k8].x), __builtin_bit_cast(h2, xv.x), acc, false);
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, wv[k8].y), __builtin_bit_cast(h2, xv.y), acc, false);
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, wv[k8].z), __builtin_bit_cast(h2, xv.z), acc, false);
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, wv[k8].w), __builtin_bit_cast(h2, xv.w), acc, false);
    }
    out[(uint64_t)t * C + c] = act_one<WRQ_ACT_STABLE_EXP>(bias + acc);
}

// One wave per head of 64: lane i keeps the whole column S[.][i] of the request's state in registers;
// k, r, w of a token go round the wave through LDS.  After the recurrence of a token: group norm over
// the head (wave reduction), rounded to f16, times silu(g).
__global__ __launch_bounds__(64) void v6_wkv_gate_kernel(const uint32_t *cursors, const float *decay, const float *time_first, float *state, ViewArgs vs,
                                                         const float *k, const float *v, const float *r, const uint16_t *g, const uint16_t *gn_w,
                                                         const uint16_t *gn_b, float eps, uint16_t *att_x, uint32_t H, uint32_t A) {
    constexpr int S = 64;
    __shared__ __align__(16) float ks[S], rs[S], ws[S], us[S];
    const uint32_t head = blockIdx.x, i = threadIdx.x;
    const uint32_t C = S * H, chan = head * S + i;
    us[i] = time_first[chan];
    const float gw = h2f(gn_w[chan]), gb = h2f(gn_b[chan]);
    float s[S];
    uint32_t held = 0xffffffffu;
    // the operands of the next token are fetched while this one is worked on (clamped at the end)
    float nk = k[chan], nr = r[chan], nw = decay[chan], nv = v[chan];
    uint16_t ng = g[chan], nx = att_x[chan];
    uint32_t ncur = cursors[0];
    for (uint32_t t = 0; t < A; t++) {
        const float ck = nk, cr = nr, cw = nw, vv = nv;
        const uint16_t cg = ng, cx = nx;
        Cursor cur = unpack_cursor(ncur);
        cur.batch = min(cur.batch, vs.shape[2] - 1); // as read_cursor
        cur.token = min(cur.token, t);
        const uint64_t ti = (uint64_t)t * C + chan;
        {
            const uint64_t tn = (uint64_t)min(t + 1, A - 1) * C + chan;
            nk = k[tn], nr = r[tn], nw = decay[tn], nv = v[tn], ng = g[tn], nx = att_x[tn];
            ncur = cursors[min(t + 1, A - 1)];
        }
        __syncthreads(); // the previous token's reads of ks / rs / ws are done
        ks[i] = ck, rs[i] = cr, ws[i] = cw;
        if (cur.batch != held) {
            if (held != 0xffffffffu) {
#pragma unroll
                for (int j = 0; j < S; j++) state[view_elem(vs, held, j + 1, chan)] = s[j];
            }
            held = cur.batch;
#pragma unroll
            for (int j = 0; j < S; j++) s[j] = state[view_elem(vs, held, j + 1, chan)];
        }
        // row 0 of the request's state keeps the layer's normalised input at its last token
        if (t - cur.token + 1 == cur.len) state[view_elem(vs, cur.batch, 0, chan)] = h2f(cx);
        __syncthreads();
        float y4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j4 = 0; j4 < S / 4; j4++) {
            const float4 k4 = *reinterpret_cast<const float4 *>(&ks[4 * j4]), r4 = *reinterpret_cast<const float4 *>(&rs[4 * j4]),
                         w4 = *reinterpret_cast<const float4 *>(&ws[4 * j4]), u4 = *reinterpret_cast<const float4 *>(&us[4 * j4]);
            const float kk[4] = {k4.x, k4.y, k4.z, k4.w}, rr[4] = {r4.x, r4.y, r4.z, r4.w}, ww[4] = {w4.x, w4.y, w4.z, w4.w}, uu[4] = {u4.x, u4.y, u4.z, u4.w};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float kv = kk[e] * vv;
                y4[e] += rr[e] * fmaf(uu[e], kv, s[4 * j4 + e]);
                s[4 * j4 + e] = fmaf(ww[e], s[4 * j4 + e], kv);
            }
        }
        const float y = (y4[0] + y4[1]) + (y4[2] + y4[3]);
        const float mean = wave_sum(y) * (1.0f / S);
        const float dev = rsqrtf(wave_sum((y - mean) * (y - mean)) * (1.0f / S) + eps);
        const float gn = round_h(fmaf((y - mean) * dev, gw, gb));
        att_x[ti] = f2h(act_one<WRQ_ACT_SILU>(h2f(cg)) * gn);
    }
    if (held != 0xffffffffu) {
#pragma unroll
        for (int j = 0; j < S; j++) state[view_elem(vs, held, j + 1, chan)] = s[j];
    }
}

// state[request] <- ffn_x at its last token; x_out = f16(f16(sigmoid(r) v) + x_in) (halved when `rescale`)
__global__ __launch_bounds__(256) void v6_post_ffn_kernel(const uint32_t *cursors, float *state, ViewArgs vs, const uint16_t *r, const uint16_t *v,
                                                          const uint16_t *ffn_x, const uint16_t *x_in, uint16_t *x_out, uint32_t C, int rescale) {
    const uint32_t index = blockIdx.x * 256 + threadIdx.x, t = blockIdx.y;
    if (index >= C / 4) return;
    const uint64_t bti = (uint64_t)t * C + 4 * index;
    // all loads before the store into the state: the compiler cannot move them across it (the pointers may
    // alias), and behind it they would wait for the cursor's round trip first
    const float4 rr = load_vec4(r + bti), vv = load_vec4(v + bti), xx = load_vec4(x_in + bti), fx = load_vec4(ffn_x + bti);
    const Cursor cur = read_cursor(cursors, t, vs);
    if (t - cur.token + 1 == cur.len) *reinterpret_cast<float4 *>(state + view_elem(vs, cur.batch, 0, 4 * index)) = fx;
    const float sc = rescale ? 0.5f : 1.0f;
    auto f = [&](float a, float b, float c) { return round_h(round_h(1.0f / (1.0f + expf(-a)) * b) + c) * sc; };
    store_vec4(x_out + bti, make_float4(f(rr.x, vv.x, xx.x), f(rr.y, vv.y, xx.y), f(rr.z, vv.z, xx.z), f(rr.w, vv.w, xx.w)));
}

int check_ptr(const void *p, const char *what) {
    if (!p) return fail(WRQ_ERR_NULL, "%s: null pointer", what);
    if ((uintptr_t)p % 16) return fail(WRQ_ERR_ALIGNMENT, "%s: device pointers must be 16-byte aligned", what);
    return WRQ_OK;
}

int check_state(const wrq_tensor_view *state, uint32_t C, uint32_t rows, const char *what) {
    const int s = check_state_view(state, what);
    if (s != WRQ_OK) return s;
    if (state->dtype != WRQ_F32) return fail(WRQ_ERR_TYPE, "%s: the state is f32", what);
    if (state->view.shape[0] != C || state->view.shape[1] != rows || state->view.shape[2] == 0 || state->view.shape[3] != 1)
        return fail(WRQ_ERR_SHAPE, "%s: state shape [%u, %u, %u, %u] not match [%u, %u, _, 1]", what, state->view.shape[0], state->view.shape[1],
                    state->view.shape[2], state->view.shape[3], C, rows);
    return WRQ_OK;
}

} // namespace

} // namespace wrq

using namespace wrq;

extern "C" {

int wrq_v6_pre(wrq_stream stream, uint32_t C, uint32_t A, const void *cursors, const void *x, const void *add, void *x_out, const void *ln_w,
               const void *ln_b, float eps, const wrq_tensor_view *state, int shifts, const void *factor0, const void *factor1, void *ln_out,
               void *shift0, void *shift1) {
    const char *what = "v6_pre";
    if (C == 0 || A == 0) return WRQ_OK;
    if (C % 4 || C > 4u * kPreThreads * kPreCache) return fail(WRQ_ERR_UNSUPPORTED, "%s: %u channels (a multiple of 4 up to %d is built)", what, C, 4 * kPreThreads * kPreCache);
    if (shifts != 1 && shifts != 2) return fail(WRQ_ERR_UNSUPPORTED, "%s: %d token shifts (1 or 2)", what, shifts);
    int s = check_state(state, C, state ? state->view.shape[1] : 0, what);
    for (const void *p : {cursors, x, ln_w, ln_b, factor0, (const void *)ln_out, (const void *)shift0})
        if (s == WRQ_OK) s = check_ptr(p, what);
    if (s == WRQ_OK && shifts == 2) s = check_ptr(factor1, what);
    if (s == WRQ_OK && shifts == 2) s = check_ptr(shift1, what);
    if (s == WRQ_OK && add) s = check_ptr(x_out, what);
    if (s != WRQ_OK) return s;
    if (add) {
        // workgroup t rebuilds row t - 1 from x and add while workgroup t - 1 stores x_out: the sum may overlap neither
        const uintptr_t lo = (uintptr_t)x_out, hi = lo + (size_t)A * C * 2;
        for (const void *src : {x, add}) {
            const uintptr_t a0 = (uintptr_t)src, a1 = a0 + (size_t)A * C * 2;
            if (lo < a1 && a0 < hi)
                return fail(WRQ_ERR_UNSUPPORTED, "%s: the sum must go to a buffer that overlaps neither input (a token's workgroup reads its neighbour's row)", what);
        }
    }
    const ViewArgs vs = view_args(state->view);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    auto u16 = [](const void *p) { return static_cast<const uint16_t *>(p); };
    auto o16 = [](void *p) { return static_cast<uint16_t *>(p); };
    if (shifts == 1)
        hipLaunchKernelGGL((v6_pre_kernel<1>), dim3(A), dim3(kPreThreads), 0, hs, static_cast<const uint32_t *>(cursors), u16(x), u16(add), o16(x_out), u16(ln_w),
                           u16(ln_b), eps, static_cast<const float *>(state->data), vs, u16(factor0), u16(factor1), o16(ln_out), o16(shift0), o16(shift1), C);
    else
        hipLaunchKernelGGL((v6_pre_kernel<2>), dim3(A), dim3(kPreThreads), 0, hs, static_cast<const uint32_t *>(cursors), u16(x), u16(add), o16(x_out), u16(ln_w),
                           u16(ln_b), eps, static_cast<const float *>(state->data), vs, u16(factor0), u16(factor1), o16(ln_out), o16(shift0), o16(shift1), C);
    return check_launch(what);
}

int wrq_v6_time_mix(wrq_stream stream, uint32_t C, uint32_t A, uint32_t lora_size, const void *cursors, const void *lora, const void *w2, const void *time_mix,
                    const wrq_tensor_view *state, const void *att_x, void *att_sx) {
    const char *what = "v6_time_mix";
    if (C == 0 || A == 0) return WRQ_OK;
    if (lora_size != 32 && lora_size != 64) return fail(WRQ_ERR_UNSUPPORTED, "%s: adapter size %u (32 or 64 is built)", what, lora_size);
    if (A > 65535u) return fail(WRQ_ERR_SIZE, "%s: data size not match", what);
    int s = check_state(state, C, state ? state->view.shape[1] : 0, what);
    for (const void *p : {cursors, lora, w2, time_mix, att_x, (const void *)att_sx})
        if (s == WRQ_OK) s = check_ptr(p, what);
    if (s != WRQ_OK) return s;
    const ViewArgs vs = view_args(state->view);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    const dim3 grid((C + 255) / 256, A);
    auto u16 = [](const void *p) { return static_cast<const uint16_t *>(p); };
    if (lora_size == 32)
        hipLaunchKernelGGL((v6_time_mix_kernel<32>), grid, dim3(256), 0, hs, static_cast<const uint32_t *>(cursors), u16(lora), u16(w2), u16(time_mix),
                           static_cast<const float *>(state->data), vs, u16(att_x), static_cast<uint16_t *>(att_sx), C, A);
    else
        hipLaunchKernelGGL((v6_time_mix_kernel<64>), grid, dim3(256), 0, hs, static_cast<const uint32_t *>(cursors), u16(lora), u16(w2), u16(time_mix),
                           static_cast<const float *>(state->data), vs, u16(att_x), static_cast<uint16_t *>(att_sx), C, A);
    return check_launch(what);
}

int wrq_v6_decay(wrq_stream stream, uint32_t C, uint32_t A, uint32_t lora_size, const void *lora, const void *w2, const void *time_decay, void *out) {
    const char *what = "v6_decay";
    if (C == 0 || A == 0) return WRQ_OK;
    if (lora_size != 64 && lora_size != 128) return fail(WRQ_ERR_UNSUPPORTED, "%s: adapter size %u (64 or 128 is built)", what, lora_size);
    if (A > 65535u) return fail(WRQ_ERR_SIZE, "%s: data size not match", what);
    int s = WRQ_OK;
    for (const void *p : {lora, w2, time_decay, (const void *)out})
        if (s == WRQ_OK) s = check_ptr(p, what);
    if (s != WRQ_OK) return s;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    const dim3 grid((C + 255) / 256, A);
    auto u16 = [](const void *p) { return static_cast<const uint16_t *>(p); };
    if (lora_size == 64) hipLaunchKernelGGL((v6_decay_kernel<64>), grid, dim3(256), 0, hs, u16(lora), u16(w2), u16(time_decay), static_cast<float *>(out), C);
    else hipLaunchKernelGGL((v6_decay_kernel<128>), grid, dim3(256), 0, hs, u16(lora), u16(w2), u16(time_decay), static_cast<float *>(out), C);
    return check_launch(what);
}

int wrq_v6_wkv_gate(wrq_stream stream, uint32_t S, uint32_t H, uint32_t A, const void *cursors, const void *time_decay, const void *time_first,
                    const wrq_tensor_view *state, const void *k, const void *v, const void *r, const void *g, const void *gn_w, const void *gn_b, float eps,
                    void *att_x) {
    const char *what = "v6_wkv_gate";
    if (H == 0 || A == 0) return WRQ_OK;
    if (S != 64) return fail(WRQ_ERR_UNSUPPORTED, "%s: head size %u (64 is built)", what, S);
    int s = check_state(state, S * H, S + 1, what);
    for (const void *p : {cursors, time_decay, time_first, k, v, r, g, gn_w, gn_b, (const void *)att_x})
        if (s == WRQ_OK) s = check_ptr(p, what);
    if (s != WRQ_OK) return s;
    const ViewArgs vs = view_args(state->view);
    auto f32 = [](const void *p) { return static_cast<const float *>(p); };
    auto u16 = [](const void *p) { return static_cast<const uint16_t *>(p); };
    hipLaunchKernelGGL(v6_wkv_gate_kernel, dim3(H), dim3(64), 0, static_cast<hipStream_t>(stream), static_cast<const uint32_t *>(cursors), f32(time_decay),
                       f32(time_first), static_cast<float *>(state->data), vs, f32(k), f32(v), f32(r), u16(g), u16(gn_w), u16(gn_b), eps,
                       static_cast<uint16_t *>(att_x), H, A);
    return check_launch(what);
}

int wrq_v6_post_ffn(wrq_stream stream, uint32_t C, uint32_t A, const void *cursors, const wrq_tensor_view *state, const void *r, const void *v, const void *ffn_x,
                    const void *x_in, void *x_out, int rescale) {
    const char *what = "v6_post_ffn";
    if (C == 0 || A == 0) return WRQ_OK;
    if (C % 4) return fail(WRQ_ERR_ALIGNMENT, "%s: row length %u not a multiple of 4", what, C);
    if (A > 65535u) return fail(WRQ_ERR_SIZE, "%s: data size not match", what);
    int s = check_state(state, C, 1, what);
    for (const void *p : {cursors, r, v, ffn_x, x_in, (const void *)x_out})
        if (s == WRQ_OK) s = check_ptr(p, what);
    if (s != WRQ_OK) return s;
    const ViewArgs vs = view_args(state->view);
    auto u16 = [](const void *p) { return static_cast<const uint16_t *>(p); };
    hipLaunchKernelGGL(v6_post_ffn_kernel, dim3((C / 4 + 255) / 256, A), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<const uint32_t *>(cursors),
                       static_cast<float *>(state->data), vs, u16(r), u16(v), u16(ffn_x), u16(x_in), static_cast<uint16_t *>(x_out), C, rescale);
    return check_launch(what);
}

} // extern "C"

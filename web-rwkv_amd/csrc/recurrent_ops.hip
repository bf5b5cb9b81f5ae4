// The ops of a v5 / v6 layer that carry state from token to token:
//   token_shift   src/tensor/ops.rs:1393-1462, src/shaders/token_shift.wgsl
//   channel_mix   src/tensor/ops.rs:1860-1915, src/shaders/channel_mix.wgsl
//   time_mix_v4   src/tensor/ops.rs:1464-1528, src/shaders/time_mix_v4.wgsl
//   time_mix_v5   src/tensor/ops.rs:1530-1599, src/shaders/time_mix_v5.wgsl
//   time_mix_v6   src/tensor/ops.rs:1601-1677, src/shaders/time_mix_v6.wgsl
//
// A run is a stack of A tokens from several requests; `cursors[a]` packs, for the request of token
// a, its state slot (8 bits), the position of its first token in the stack (16 bits) and the number
// of its tokens in the stack (8 bits) (`compute_cursor` of the shaders).
//
// time_mix_v6 is the recurrence  y[i] = sum_j r[j] (u[j] k[j] v[i] + S[j][i]),  S[j][i] <- w[j] S[j][i] + k[j] v[i]
// per head, token after token; time_mix_v5 is the same recurrence with a decay w that is a constant of
// the channel instead of a value per token (one kernel, TOKEN_DECAY tells them apart).  The shader re-reads and re-writes the head's S (64 x 64 f32) in memory
// for every token; here a request's S stays in registers for all its tokens of the run: four lanes
// share an output element i and hold a quarter of j each (16 values of S), one DPP quad reduction
// per token; S is read when a request's tokens begin and written when they end.  The sum over j is
// therefore taken in interleaved partial sums instead of one chain (a difference of rounding order only).
#include "layer_device.h"

namespace wrq {

namespace {

// output[count][stack] = mix(previous token, this token, time_mix) (reversed: the two swapped); the
// previous token of a request's first token in the stack is its state row
template <typename FT, typename IT, typename OT>
__global__ __launch_bounds__(256) void token_shift_kernel(const uint32_t *cursors, const FT *time_mix, const float *state, const IT *input, OT *output,
                                                          ViewArgs vt, ViewArgs vs, uint32_t C, uint32_t A, int reversed) {
    const uint32_t index = blockIdx.x * 256 + threadIdx.x, stack = blockIdx.y, count = blockIdx.z;
    if (index >= C / 4) return;
    const Cursor cur = read_cursor(cursors, stack, vs);
    const float4 f = load_vec4(time_mix + view_elem(vt, count, vt.shape[1] == 1 ? 0u : stack, 4 * index));
    const float4 x = load_vec4(input + ((uint64_t)stack * C + 4 * index));
    const float4 p = stack == cur.token ? load_vec4(state + view_elem(vs, cur.batch, 0, 4 * index)) : load_vec4(input + ((uint64_t)(stack - 1) * C + 4 * index));
    // mix(a, b, t) = a (1 - t) + b t
    auto mix = [&](float a, float b, float t) { return reversed ? a * (1.0f - t) + b * t : b * (1.0f - t) + a * t; };
    store_vec4(output + (((uint64_t)count * A + stack) * C + 4 * index), make_float4(mix(x.x, p.x, f.x), mix(x.y, p.y, f.y), mix(x.z, p.z, f.z), mix(x.w, p.w, f.w)));
}

// state[request] <- x at the request's last token of the stack; x <- sigmoid(r) * v
template <typename XT>
__global__ __launch_bounds__(256) void channel_mix_kernel(const uint32_t *cursors, float *state, const XT *r, const XT *v, XT *x, ViewArgs vs, uint32_t C) {
    const uint32_t index = blockIdx.x * 256 + threadIdx.x, stack = blockIdx.y;
    if (index >= C / 4) return;
    const uint64_t bti = (uint64_t)stack * C + 4 * index;
    // all loads before the store into the state (the compiler cannot move them across it: the pointers may alias)
    const float4 rr = load_vec4(r + bti), vv = load_vec4(v + bti), xx = load_vec4(x + bti);
    const Cursor cur = read_cursor(cursors, stack, vs);
    if (stack - cur.token + 1 == cur.len) *reinterpret_cast<float4 *>(state + view_elem(vs, cur.batch, 0, 4 * index)) = xx;
    auto g = [](float a, float b) { return 1.0f / (1.0f + expf(-a)) * b; };
    store_vec4(x + bti, make_float4(g(rr.x, vv.x), g(rr.y, vv.y), g(rr.z, vv.z), g(rr.w, vv.w)));
}

__device__ __forceinline__ float quad_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xf, 0xf, true)); // quad_perm [1,0,3,2]
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xf, 0xf, true)); // quad_perm [2,3,0,1]
    return v;
}

// One workgroup per head: thread = (output element i of the head, quarter q of the j range), four
// waves of 16 i x 4 q; JQ = S / 4 values of S[.][i] per lane.  The operands of the head (k, r, w, v:
// S values each per token) come in chunks of 1024 / S tokens: every thread fetches one 4-element
// vector of each while the previous chunk is worked on, and the chunk is passed round through LDS
// (two buffers), from where the lanes of a quarter read their j range as broadcasts.
template <typename XT, int JQ, bool TOKEN_DECAY>
__global__ __launch_bounds__(256) void time_mix_kernel(const uint32_t *cursors, const float *time_decay, const float *time_first, float *state, const XT *k,
                                                          const XT *v, const XT *r, XT *x, ViewArgs vs, uint32_t S, uint32_t H, uint32_t A) {
    constexpr int SZ = 4 * JQ;      // head size
    constexpr int TB = 1024 / SZ;   // tokens per chunk
    __shared__ __align__(16) float ks[2][1024], rs[2][1024], ws[2][1024], vsh[2][1024];
    __shared__ uint32_t csh[2][TB]; // the chunk's cursors
    const uint32_t head = blockIdx.x, tid = threadIdx.x;
    const uint32_t q = tid & 3;
    const uint32_t C = S * H;
    const uint32_t nchunk = (A + TB - 1) / TB;
    // this thread's vector of a chunk: token tid / (SZ / 4) of the chunk, elements 4 (tid % (SZ / 4)) ..
    const uint32_t lt = tid / (SZ / 4), le = 4 * (tid % (SZ / 4));
    float4 fk, fr, fw, fv;
    uint32_t fc = 0;
    auto fetch = [&](uint32_t chunk) {
        const uint32_t t = min(chunk * TB + lt, A - 1); // clamped: tokens past the run are never used
        const uint64_t g = (uint64_t)t * C + head * SZ + le;
        fk = load_vec4(k + g), fr = load_vec4(r + g), fv = load_vec4(v + g);
        if constexpr (TOKEN_DECAY) fw = load_vec4(time_decay + g);
        if (tid < (uint32_t)TB) fc = cursors[min(chunk * TB + tid, A - 1)];
    };
    auto stage = [&](int buf) {
        *reinterpret_cast<float4 *>(&ks[buf][4 * tid]) = fk;
        *reinterpret_cast<float4 *>(&rs[buf][4 * tid]) = fr;
        if constexpr (TOKEN_DECAY) *reinterpret_cast<float4 *>(&ws[buf][4 * tid]) = fw;
        *reinterpret_cast<float4 *>(&vsh[buf][4 * tid]) = fv;
        if (tid < (uint32_t)TB) csh[buf][tid] = fc;
    };
    for (uint32_t i0 = 0; i0 < SZ; i0 += 64) {
        const uint32_t i = i0 + (tid >> 2);
        const bool live = i < SZ; // head sizes below 64 leave waves without an output element
        const uint32_t chan = head * SZ + min(i, (uint32_t)SZ - 1);
        float u[JQ], s[JQ], wc[TOKEN_DECAY ? 1 : JQ]; // wc: the constant decay of this lane's j range
#pragma unroll
        for (int c = 0; c < JQ / 4; c++) {
            const float4 t4 = *reinterpret_cast<const float4 *>(time_first + head * SZ + q * JQ + 4 * c);
            u[4 * c] = t4.x, u[4 * c + 1] = t4.y, u[4 * c + 2] = t4.z, u[4 * c + 3] = t4.w;
            if constexpr (!TOKEN_DECAY) {
                const float4 d4 = *reinterpret_cast<const float4 *>(time_decay + head * SZ + q * JQ + 4 * c);
                wc[4 * c] = d4.x, wc[4 * c + 1] = d4.y, wc[4 * c + 2] = d4.z, wc[4 * c + 3] = d4.w;
            }
        }
        uint32_t held = 0xffffffffu; // request whose S is in registers
        fetch(0);
        __syncthreads(); // the buffers may still be read by the previous pass over i
        stage(0);
        for (uint32_t chunk = 0; chunk < nchunk; chunk++) {
            const int buf = chunk & 1;
            if (chunk + 1 < nchunk) fetch(chunk + 1);
            __syncthreads(); // chunk `chunk` is in LDS; buffer buf ^ 1 is free
            const uint32_t tend = min((uint32_t)TB, A - chunk * TB);
            if (live) {
                for (uint32_t tt = 0; tt < tend; tt++) {
                    const uint32_t t = chunk * TB + tt;
                    Cursor cur = unpack_cursor(csh[buf][tt]);
                    cur.batch = min(cur.batch, vs.shape[2] - 1); // as read_cursor
                    cur.token = min(cur.token, t);
                    if (cur.batch != held) {
                        if (held != 0xffffffffu) {
#pragma unroll
                            for (int jj = 0; jj < JQ; jj++) state[view_elem(vs, held, q * JQ + jj + 1, chan)] = s[jj];
                        }
                        held = cur.batch;
#pragma unroll
                        for (int jj = 0; jj < JQ; jj++) s[jj] = state[view_elem(vs, held, q * JQ + jj + 1, chan)];
                    }
                    const uint64_t ti = (uint64_t)t * C + chan;
                    // row 0 of the request's state keeps the layer's input at its last token (read before x is overwritten)
                    if (q == 0 && t - cur.token + 1 == cur.len) state[view_elem(vs, cur.batch, 0, chan)] = load_one(x + ti);
                    const float vv = vsh[buf][tt * SZ + i];
                    const float *kp = &ks[buf][tt * SZ + q * JQ], *rp = &rs[buf][tt * SZ + q * JQ], *wp = &ws[buf][tt * SZ + q * JQ];
                    float y4[4] = {0.0f, 0.0f, 0.0f, 0.0f}; // four chains instead of one of JQ dependent adds
#pragma unroll
                    for (int c = 0; c < JQ / 4; c++) {
                        const float4 k4 = *reinterpret_cast<const float4 *>(kp + 4 * c), r4 = *reinterpret_cast<const float4 *>(rp + 4 * c);
                        const float kk[4] = {k4.x, k4.y, k4.z, k4.w}, rr[4] = {r4.x, r4.y, r4.z, r4.w};
                        float ww[4];
                        if constexpr (TOKEN_DECAY) {
                            const float4 w4 = *reinterpret_cast<const float4 *>(wp + 4 * c);
                            ww[0] = w4.x, ww[1] = w4.y, ww[2] = w4.z, ww[3] = w4.w;
                        } else {
                            ww[0] = wc[4 * c], ww[1] = wc[4 * c + 1], ww[2] = wc[4 * c + 2], ww[3] = wc[4 * c + 3];
                        }
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const float kv = kk[e] * vv;
                            y4[e] += rr[e] * fmaf(u[4 * c + e], kv, s[4 * c + e]);
                            s[4 * c + e] = fmaf(ww[e], s[4 * c + e], kv);
                        }
                    }
                    const float y = quad_sum((y4[0] + y4[1]) + (y4[2] + y4[3]));
                    if (q == 0) {
                        if constexpr (sizeof(XT) == 2) x[ti] = f2h(y);
                        else x[ti] = y;
                    }
                }
            }
            if (chunk + 1 < nchunk) stage(buf ^ 1); // read two chunks ago, before the barrier above
        }
        if (live && held != 0xffffffffu) {
#pragma unroll
            for (int jj = 0; jj < JQ; jj++) state[view_elem(vs, held, q * JQ + jj + 1, chan)] = s[jj];
        }
    }
}

// The v4 recurrence, per channel: a numerator aa, a denominator bb and their common exponent pp,
//   x <- sigmoid(r) (e^(pp-q) aa + e^(u+k-q) v) / (e^(pp-q) bb + e^(u+k-q)),  q = max(pp, u + k)
//   aa, bb <- e^(w+pp-q') (aa, bb) + e^(k-q') (v, 1),  pp <- q' = max(w + pp, k)
// One thread per channel walks the tokens of the run; a request's three values stay in registers over
// its tokens (the shader reads and writes them per token), the next token's operands are fetched ahead.
template <typename XT>
__global__ __launch_bounds__(256) void time_mix_v4_kernel(const uint32_t *cursors, const float *time_decay, const float *time_first, float *state, const XT *k,
                                                          const XT *v, const XT *r, XT *x, ViewArgs vs, uint32_t C, uint32_t A) {
    const uint32_t c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const float u = time_first[c], w = time_decay[c];
    float aa = 0.0f, bb = 0.0f, pp = 0.0f;
    uint32_t held = 0xffffffffu;
    float fk = load_one(k + c), fv = load_one(v + c), fr = load_one(r + c);
    for (uint32_t t = 0; t < A; t++) {
        const Cursor cur = read_cursor(cursors, t, vs);
        const float kk = fk, vv = fv, rr = 1.0f / (1.0f + expf(-fr));
        if (t + 1 < A) {
            const uint64_t nx = (uint64_t)(t + 1) * C + c;
            fk = load_one(k + nx), fv = load_one(v + nx), fr = load_one(r + nx);
        }
        if (cur.batch != held) {
            if (held != 0xffffffffu)
                state[view_elem(vs, held, 1, c)] = aa, state[view_elem(vs, held, 2, c)] = bb, state[view_elem(vs, held, 3, c)] = pp;
            held = cur.batch;
            aa = state[view_elem(vs, held, 1, c)], bb = state[view_elem(vs, held, 2, c)], pp = state[view_elem(vs, held, 3, c)];
        }
        const uint64_t ti = (uint64_t)t * C + c;
        // row 0 of the request's state keeps the layer's input at its last token (read before x is overwritten)
        if (t - cur.token + 1 == cur.len) state[view_elem(vs, cur.batch, 0, c)] = load_one(x + ti);
        float ww = u + kk;
        float q = fmaxf(pp, ww);
        float e1 = expf(pp - q), e2 = expf(ww - q);
        const float y = rr * (e1 * aa + e2 * vv) / (e1 * bb + e2);
        if constexpr (sizeof(XT) == 2) x[ti] = f2h(y);
        else x[ti] = y;
        ww = w + pp;
        q = fmaxf(ww, kk);
        e1 = expf(ww - q), e2 = expf(kk - q);
        aa = e1 * aa + e2 * vv;
        bb = e1 * bb + e2;
        pp = q;
    }
    if (held != 0xffffffffu) state[view_elem(vs, held, 1, c)] = aa, state[view_elem(vs, held, 2, c)] = bb, state[view_elem(vs, held, 3, c)] = pp;
}

template <typename FT, typename IT>
int token_shift_out(hipStream_t stream, const wrq_tensor *cursors, const wrq_tensor_view *time_mix, const wrq_tensor_view *state, const wrq_tensor *input,
                    const wrq_tensor *output, int out_dtype, dim3 grid, int reversed) {
    const ViewArgs vt = view_args(time_mix->view), vs = view_args(state->view);
    const uint32_t C = output->shape[0], A = output->shape[1];
    const uint32_t *cur = static_cast<const uint32_t *>(cursors->data);
    if (out_dtype == WRQ_F16)
        hipLaunchKernelGGL((token_shift_kernel<FT, IT, uint16_t>), grid, dim3(256), 0, stream, cur, static_cast<const FT *>(time_mix->data), static_cast<const float *>(state->data),
                           static_cast<const IT *>(input->data), static_cast<uint16_t *>(output->data), vt, vs, C, A, reversed);
    else
        hipLaunchKernelGGL((token_shift_kernel<FT, IT, float>), grid, dim3(256), 0, stream, cur, static_cast<const FT *>(time_mix->data), static_cast<const float *>(state->data),
                           static_cast<const IT *>(input->data), static_cast<float *>(output->data), vt, vs, C, A, reversed);
    return check_launch("token_shift");
}

} // namespace

} // namespace wrq

using namespace wrq;

extern "C" {

int wrq_token_shift(wrq_stream stream, const wrq_tensor *cursors, const wrq_tensor_view *time_mix, const wrq_tensor_view *state, const wrq_tensor *input,
                    wrq_dtype input_dtype, const wrq_tensor *output, wrq_dtype output_dtype, int reversed) {
    int s = check_layer_tensor(cursors, "token_shift");
    if (s == WRQ_OK) s = check_layer_tensor(input, "token_shift");
    if (s == WRQ_OK) s = check_layer_tensor(output, "token_shift");
    if (s == WRQ_OK) s = check_layer_view(time_mix, "token_shift");
    if (s == WRQ_OK) s = check_state_view(state, "token_shift");
    if (s != WRQ_OK) return s;
    if (state->dtype != WRQ_F32) return fail(WRQ_ERR_TYPE, "token_shift: the state is f32");
    for (int d : {(int)input_dtype, (int)output_dtype})
        if (d != WRQ_F16 && d != WRQ_F32) return fail(WRQ_ERR_TYPE, "token_shift: unsupported element type %d", d);
    const uint32_t *o = output->shape, *i = input->shape, *t = time_mix->view.shape, *st = state->view.shape;
    // src/tensor/ops.rs:1409-1414
    const bool ok = o[3] == 1 && i[0] == o[0] && i[1] == o[1] && (i[2] == o[2] || i[2] == 1) && i[3] == 1 &&
                    ((t[0] == o[0] && t[1] == o[1] && t[2] == o[2] && t[3] == 1) || (t[0] == o[0] && t[1] == 1 && t[2] == 1 && t[3] == 1)) && st[0] == o[0] && st[3] == 1;
    if (!ok) return fail(WRQ_ERR_SHAPE, "token_shift: data shape not match [%u, %u, %u, %u]", o[0], o[1], o[2], o[3]);
    if (cursors->shape[0] < o[1]) return fail(WRQ_ERR_SHAPE, "token_shift: %u cursors for %u tokens", cursors->shape[0], o[1]);
    if (o[0] % 4) return fail(WRQ_ERR_ALIGNMENT, "token_shift: row length %u not a multiple of 4", o[0]);
    if (o[0] == 0 || o[1] == 0 || o[2] == 0) return WRQ_OK;
    if (o[1] > 65535u || o[2] > 65535u) return fail(WRQ_ERR_SIZE, "token_shift: data size not match");
    const dim3 grid((o[0] / 4 + 255) / 256, o[1], o[2]);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    const bool f16 = time_mix->dtype == WRQ_F16, i16 = input_dtype == WRQ_F16;
    if (f16 && i16) return token_shift_out<uint16_t, uint16_t>(hs, cursors, time_mix, state, input, output, output_dtype, grid, reversed);
    if (f16) return token_shift_out<uint16_t, float>(hs, cursors, time_mix, state, input, output, output_dtype, grid, reversed);
    if (i16) return token_shift_out<float, uint16_t>(hs, cursors, time_mix, state, input, output, output_dtype, grid, reversed);
    return token_shift_out<float, float>(hs, cursors, time_mix, state, input, output, output_dtype, grid, reversed);
}

int wrq_channel_mix(wrq_stream stream, const wrq_tensor *cursors, const wrq_tensor_view *state, const wrq_tensor *r, const wrq_tensor *v, const wrq_tensor *x,
                    wrq_dtype dtype) {
    int s = check_layer_tensor(cursors, "channel_mix");
    for (const wrq_tensor *t : {r, v, x})
        if (s == WRQ_OK) s = check_layer_tensor(t, "channel_mix");
    if (s == WRQ_OK) s = check_state_view(state, "channel_mix");
    if (s != WRQ_OK) return s;
    if (state->dtype != WRQ_F32) return fail(WRQ_ERR_TYPE, "channel_mix: the state is f32");
    if (dtype != WRQ_F16 && dtype != WRQ_F32) return fail(WRQ_ERR_TYPE, "channel_mix: unsupported element type %d", (int)dtype);
    const uint32_t *sh = x->shape, *st = state->view.shape;
    // src/tensor/ops.rs:1873-1877
    if (!same_shape(r->shape, sh) || !same_shape(v->shape, sh) || st[0] != sh[0] || st[1] != 1 || st[3] != 1 || sh[2] != 1 || sh[3] != 1)
        return fail(WRQ_ERR_SHAPE, "channel_mix: data shape not match [%u, %u, %u, %u]", sh[0], sh[1], sh[2], sh[3]);
    if (cursors->shape[0] < sh[1]) return fail(WRQ_ERR_SHAPE, "channel_mix: %u cursors for %u tokens", cursors->shape[0], sh[1]);
    if (sh[0] % 4) return fail(WRQ_ERR_ALIGNMENT, "channel_mix: row length %u not a multiple of 4", sh[0]);
    if (sh[0] == 0 || sh[1] == 0) return WRQ_OK;
    if (sh[1] > 65535u) return fail(WRQ_ERR_SIZE, "channel_mix: data size not match");
    const dim3 grid((sh[0] / 4 + 255) / 256, sh[1]);
    const ViewArgs vs = view_args(state->view);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    const uint32_t *cur = static_cast<const uint32_t *>(cursors->data);
    if (dtype == WRQ_F16)
        hipLaunchKernelGGL((channel_mix_kernel<uint16_t>), grid, dim3(256), 0, hs, cur, static_cast<float *>(state->data), static_cast<const uint16_t *>(r->data),
                           static_cast<const uint16_t *>(v->data), static_cast<uint16_t *>(x->data), vs, sh[0]);
    else
        hipLaunchKernelGGL((channel_mix_kernel<float>), grid, dim3(256), 0, hs, cur, static_cast<float *>(state->data), static_cast<const float *>(r->data),
                           static_cast<const float *>(v->data), static_cast<float *>(x->data), vs, sh[0]);
    return check_launch("channel_mix");
}

} // extern "C"

namespace {

// time_mix_v5 (token_decay == false: time_decay [S, H, 1, 1]) and time_mix_v6 (time_decay [S, H, A, 1])
int time_mix(const char *name, bool token_decay, wrq_stream stream, const wrq_tensor *cursors, const wrq_tensor *time_decay, const wrq_tensor *time_first,
             const wrq_tensor_view *state, const wrq_tensor *k, const wrq_tensor *v, const wrq_tensor *r, const wrq_tensor *x, wrq_dtype dtype) {
    int s = check_layer_tensor(cursors, name);
    for (const wrq_tensor *t : {time_decay, time_first, k, v, r, x})
        if (s == WRQ_OK) s = check_layer_tensor(t, name);
    if (s == WRQ_OK) s = check_state_view(state, name);
    if (s != WRQ_OK) return s;
    if (state->dtype != WRQ_F32) return fail(WRQ_ERR_TYPE, "%s: the state is f32", name);
    if (dtype != WRQ_F16 && dtype != WRQ_F32) return fail(WRQ_ERR_TYPE, "%s: unsupported element type %d", name, (int)dtype);
    const uint32_t *sh = x->shape, *st = state->view.shape; // [S, H, A, 1]
    const uint32_t S = sh[0], H = sh[1], A = sh[2];
    // src/tensor/ops.rs:1546-1553 (v5), 1620-1625 (v6)
    const uint32_t tf[4] = {S, H, 1, 1};
    if (sh[3] != 1 || !same_shape(k->shape, sh) || !same_shape(v->shape, sh) || !same_shape(r->shape, sh) || !same_shape(time_decay->shape, token_decay ? sh : tf) ||
        !same_shape(time_first->shape, tf) || st[0] != S * H || st[1] != S + 1 || st[3] != 1)
        return fail(WRQ_ERR_SHAPE, "%s: data shape not match [%u, %u, %u, %u]", name, sh[0], sh[1], sh[2], sh[3]);
    if (cursors->shape[0] < A) return fail(WRQ_ERR_SHAPE, "%s: %u cursors for %u tokens", name, cursors->shape[0], A);
    if (S == 0 || H == 0 || A == 0) return WRQ_OK;
    const ViewArgs vs = view_args(state->view);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    const uint32_t *cur = static_cast<const uint32_t *>(cursors->data);
    const float *td = static_cast<const float *>(time_decay->data), *tfp = static_cast<const float *>(time_first->data);
    float *sp = static_cast<float *>(state->data);
#define WRQ_TM_LAUNCH(XT, JQ, TD)                                                                                                                \
    hipLaunchKernelGGL((time_mix_kernel<XT, JQ, TD>), dim3(H), dim3(256), 0, hs, cur, td, tfp, sp, static_cast<const XT *>(k->data),               \
                       static_cast<const XT *>(v->data), static_cast<const XT *>(r->data), static_cast<XT *>(x->data), vs, S, H, A)
#define WRQ_TM(JQ)                                                                                                                               \
    if (S == 4 * JQ) {                                                                                                                           \
        if (dtype == WRQ_F16) {                                                                                                                  \
            if (token_decay) WRQ_TM_LAUNCH(uint16_t, JQ, true);                                                                                  \
            else WRQ_TM_LAUNCH(uint16_t, JQ, false);                                                                                             \
        } else {                                                                                                                                 \
            if (token_decay) WRQ_TM_LAUNCH(float, JQ, true);                                                                                     \
            else WRQ_TM_LAUNCH(float, JQ, false);                                                                                                \
        }                                                                                                                                        \
        return check_launch(name);                                                                                                               \
    }
    WRQ_TM(4) WRQ_TM(8) WRQ_TM(16) WRQ_TM(32) WRQ_TM(64)
#undef WRQ_TM
#undef WRQ_TM_LAUNCH
    return fail(WRQ_ERR_UNSUPPORTED, "%s: head size %u (16, 32, 64, 128 or 256 is built)", name, S);
}

} // namespace

extern "C" {

int wrq_time_mix_v4(wrq_stream stream, const wrq_tensor *cursors, const wrq_tensor *time_decay, const wrq_tensor *time_first, const wrq_tensor_view *state,
                    const wrq_tensor *k, const wrq_tensor *v, const wrq_tensor *r, const wrq_tensor *x, wrq_dtype dtype) {
    int s = check_layer_tensor(cursors, "time_mix_v4");
    for (const wrq_tensor *t : {time_decay, time_first, k, v, r, x})
        if (s == WRQ_OK) s = check_layer_tensor(t, "time_mix_v4");
    if (s == WRQ_OK) s = check_state_view(state, "time_mix_v4");
    if (s != WRQ_OK) return s;
    if (state->dtype != WRQ_F32) return fail(WRQ_ERR_TYPE, "time_mix_v4: the state is f32");
    if (dtype != WRQ_F16 && dtype != WRQ_F32) return fail(WRQ_ERR_TYPE, "time_mix_v4: unsupported element type %d", (int)dtype);
    const uint32_t *sh = x->shape, *st = state->view.shape; // [C, A, 1, 1]
    // src/tensor/ops.rs:1480-1485
    const uint32_t vec[4] = {sh[0], 1, 1, 1};
    if (sh[2] != 1 || sh[3] != 1 || !same_shape(k->shape, sh) || !same_shape(v->shape, sh) || !same_shape(r->shape, sh) || !same_shape(time_decay->shape, vec) ||
        !same_shape(time_first->shape, vec) || st[0] != sh[0] || st[1] != 4 || st[3] != 1)
        return fail(WRQ_ERR_SHAPE, "time_mix_v4: data shape not match [%u, %u, %u, %u]", sh[0], sh[1], sh[2], sh[3]);
    if (cursors->shape[0] < sh[1]) return fail(WRQ_ERR_SHAPE, "time_mix_v4: %u cursors for %u tokens", cursors->shape[0], sh[1]);
    if (sh[0] == 0 || sh[1] == 0) return WRQ_OK;
    const ViewArgs vs = view_args(state->view);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    const uint32_t *cur = static_cast<const uint32_t *>(cursors->data);
    const float *td = static_cast<const float *>(time_decay->data), *tfp = static_cast<const float *>(time_first->data);
    const dim3 grid((sh[0] + 255) / 256);
    if (dtype == WRQ_F16)
        hipLaunchKernelGGL((time_mix_v4_kernel<uint16_t>), grid, dim3(256), 0, hs, cur, td, tfp, static_cast<float *>(state->data), static_cast<const uint16_t *>(k->data),
                           static_cast<const uint16_t *>(v->data), static_cast<const uint16_t *>(r->data), static_cast<uint16_t *>(x->data), vs, sh[0], sh[1]);
    else
        hipLaunchKernelGGL((time_mix_v4_kernel<float>), grid, dim3(256), 0, hs, cur, td, tfp, static_cast<float *>(state->data), static_cast<const float *>(k->data),
                           static_cast<const float *>(v->data), static_cast<const float *>(r->data), static_cast<float *>(x->data), vs, sh[0], sh[1]);
    return check_launch("time_mix_v4");
}

int wrq_time_mix_v5(wrq_stream stream, const wrq_tensor *cursors, const wrq_tensor *time_decay, const wrq_tensor *time_first, const wrq_tensor_view *state,
                    const wrq_tensor *k, const wrq_tensor *v, const wrq_tensor *r, const wrq_tensor *x, wrq_dtype dtype) {
    return time_mix("time_mix_v5", false, stream, cursors, time_decay, time_first, state, k, v, r, x, dtype);
}

int wrq_time_mix_v6(wrq_stream stream, const wrq_tensor *cursors, const wrq_tensor *time_decay, const wrq_tensor *time_first, const wrq_tensor_view *state,
                    const wrq_tensor *k, const wrq_tensor *v, const wrq_tensor *r, const wrq_tensor *x, wrq_dtype dtype) {
    return time_mix("time_mix_v6", true, stream, cursors, time_decay, time_first, state, k, v, r, x, dtype);
}

} // extern "C"

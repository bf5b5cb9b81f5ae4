// The ops an RWKV-v7 layer adds to the ones of v5 / v6:
//   l2_norm          src/tensor/ops.rs:642-700,   src/shaders/normalize.wgsl:118-152
//   control_k_v7     src/tensor/ops.rs:1800-1858, src/shaders/control_k_v7.wgsl
//   time_mix_v7      src/tensor/ops.rs:1679-1741, src/shaders/time_mix_v7.wgsl:137-212
//   time_first_v7    src/tensor/ops.rs:1743-1798, src/shaders/time_mix_v7.wgsl:214-255
//   channel_mix_v7   src/tensor/ops.rs:1917-1970, src/shaders/channel_mix.wgsl (V7)
//
// time_mix_v7 is, per head and token, with S[j][i] the head's state, a = -kk, b = kk * a_in and
// w = exp(-exp(-0.5) sigmoid(w_in)):
//   sa[i] = sum_j S[j][i] a[j];   S[j][i] <- S[j][i] w[j] + k[j] v[i] + sa[i] b[j];   y[i] = sum_j r[j] S[j][i]
// The shader walks the state in memory twice per token; here four lanes share column i of S and hold a
// quarter of its j range each in registers for all tokens of a request in the run (two quad reductions
// per token, for sa and for y); the vectors over j of 1024 / S tokens at a time are fetched a chunk ahead
// and passed round through LDS (two buffers, one barrier per chunk).  One workgroup of 256 lanes per head.
#include "layer_device.h"

namespace wrq {

namespace {

template <typename XT>
__global__ __launch_bounds__(64) void l2_norm_kernel(XT *x, uint32_t C, float eps) {
    XT *row = x + (uint64_t)blockIdx.x * C;
    float sum = 0.0f;
    for (uint32_t i = 4 * threadIdx.x; i < C; i += 256) {
        const float4 v = load_vec4(row + i);
        sum += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    }
    const float norm = 1.0f / sqrtf(wave_sum(sum) + eps);
    for (uint32_t i = 4 * threadIdx.x; i < C; i += 256) {
        const float4 v = load_vec4(row + i);
        store_vec4(row + i, make_float4(v.x * norm, v.y * norm, v.z * norm, v.w * norm));
    }
}

// k <- k (1 + (a - 1) p)
template <typename AT, typename KT>
__global__ __launch_bounds__(256) void control_k_kernel(const uint16_t *p, const AT *a, KT *k, ViewArgs va, ViewArgs vk, uint32_t C) {
    const uint32_t index = blockIdx.x * 256 + threadIdx.x, token = blockIdx.y, batch = blockIdx.z;
    if (index >= C / 4) return;
    const float4 pp = load_vec4(p + 4 * index), aa = load_vec4(a + view_elem(va, batch, token, 4 * index));
    KT *kp = k + view_elem(vk, batch, token, 4 * index);
    const float4 kk = load_vec4(kp);
    auto f = [](float kv, float av, float pv) { return kv * (1.0f + (av - 1.0f) * pv); };
    store_vec4(kp, make_float4(f(kk.x, aa.x, pp.x), f(kk.y, aa.y, pp.y), f(kk.z, aa.z, pp.z), f(kk.w, aa.w, pp.w)));
}

__device__ __forceinline__ float quad_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xf, 0xf, true)); // quad_perm [1,0,3,2]
    v += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xf, 0xf, true)); // quad_perm [2,3,0,1]
    return v;
}

// One workgroup of 256 threads per head: thread = (column i of S, quarter q of the j range), JQ = SZ / 4
// values of S per lane; heads of more than 64 columns take several passes over the run.  The operands of the
// head come in chunks of 1024 / SZ tokens: every thread fetches one 4-element vector of each of the six
// while the previous chunk is worked on, the chunk is passed round through LDS (two buffers, one barrier per
// chunk), and the lanes of a quarter read their j range as broadcasts.  Within a chunk a token needs no
// barrier: both sums over j close inside a quad.
template <typename XT, int SZ>
__global__ __launch_bounds__(256) void time_mix_v7_kernel(const uint32_t *cursors, float *state, const XT *r, const XT *w, const XT *n, XT *x, ViewArgs vs,
                                                          uint32_t H, uint32_t A) {
    constexpr int JQ = SZ / 4;
    constexpr int TB = 1024 / SZ; // tokens per chunk
    __shared__ __align__(16) float rs[2][1024], ws[2][1024], ks[2][1024], as[2][1024], bs[2][1024], vsh[2][1024];
    __shared__ uint32_t csh[2][TB]; // the chunk's cursors
    const uint32_t head = blockIdx.x, tid = threadIdx.x, q = tid & 3;
    const uint32_t C = SZ * H;
    const uint64_t plane = (uint64_t)A * C; // n holds k, v, a, kk one after the other
    const uint32_t nchunk = (A + TB - 1) / TB;
    // this thread's vector of a chunk: token tid / (SZ / 4) of the chunk, elements 4 (tid % (SZ / 4)) ..
    const uint32_t lt = tid / (SZ / 4), le = 4 * (tid % (SZ / 4));
    float4 fr, fw, fk, fv, fa, fkk;
    uint32_t fc = 0;
    auto fetch = [&](uint32_t chunk) {
        const uint32_t t = min(chunk * TB + lt, A - 1); // clamped: tokens past the run are never used
        const uint64_t g = (uint64_t)t * C + head * SZ + le;
        fr = load_vec4(r + g), fw = load_vec4(w + g), fk = load_vec4(n + g), fv = load_vec4(n + plane + g);
        fa = load_vec4(n + 2 * plane + g), fkk = load_vec4(n + 3 * plane + g);
        if (tid < (uint32_t)TB) fc = cursors[min(chunk * TB + tid, A - 1)];
    };
    auto decay = [](float v) { return expf(-0.606531f / (1.0f + expf(-v))); }; // exp(-exp(-0.5) sigmoid(w))
    auto stage = [&](int buf) {
        *reinterpret_cast<float4 *>(&rs[buf][4 * tid]) = fr;
        *reinterpret_cast<float4 *>(&ws[buf][4 * tid]) = make_float4(decay(fw.x), decay(fw.y), decay(fw.z), decay(fw.w));
        *reinterpret_cast<float4 *>(&ks[buf][4 * tid]) = fk;
        *reinterpret_cast<float4 *>(&as[buf][4 * tid]) = make_float4(-fkk.x, -fkk.y, -fkk.z, -fkk.w);
        *reinterpret_cast<float4 *>(&bs[buf][4 * tid]) = make_float4(fkk.x * fa.x, fkk.y * fa.y, fkk.z * fa.z, fkk.w * fa.w);
        *reinterpret_cast<float4 *>(&vsh[buf][4 * tid]) = fv;
        if (tid < (uint32_t)TB) csh[buf][tid] = fc;
    };
    for (uint32_t i0 = 0; i0 < SZ; i0 += 64) {
        const uint32_t i = i0 + (tid >> 2);
        const bool live = i < SZ; // head sizes below 64 leave waves without a column
        const uint32_t chan = head * SZ + min(i, (uint32_t)SZ - 1);
        float s[JQ];
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
                    const float *ap = &as[buf][tt * SZ + q * JQ], *wp = &ws[buf][tt * SZ + q * JQ], *kp = &ks[buf][tt * SZ + q * JQ],
                                *bp = &bs[buf][tt * SZ + q * JQ], *rp = &rs[buf][tt * SZ + q * JQ];
                    float sa4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int jj = 0; jj < JQ; jj++) sa4[jj & 3] += s[jj] * ap[jj];
                    const float sa = quad_sum((sa4[0] + sa4[1]) + (sa4[2] + sa4[3]));
                    float y4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int jj = 0; jj < JQ; jj++) {
                        s[jj] = s[jj] * wp[jj] + kp[jj] * vv + sa * bp[jj];
                        y4[jj & 3] += rp[jj] * s[jj];
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

// x[i] += (sum_j u[j] k[j] r[j]) v[i] per head and token; one wave per (token, head)
template <typename XT>
__global__ __launch_bounds__(64) void time_first_v7_kernel(const uint16_t *u, const XT *r, const XT *n, XT *x, uint32_t S, uint32_t H, uint32_t A) {
    const uint32_t head = blockIdx.x, t = blockIdx.y;
    const uint32_t C = S * H;
    const uint64_t base = (uint64_t)t * C + head * S, plane = (uint64_t)A * C;
    float sum = 0.0f;
    for (uint32_t j = threadIdx.x; j < S; j += 64) sum += h2f(u[head * S + j]) * load_one(n + base + j) * load_one(r + base + j);
    sum = wave_sum(sum);
    for (uint32_t i = threadIdx.x; i < S; i += 64) {
        const float y = load_one(x + base + i) + sum * load_one(n + plane + base + i);
        if constexpr (sizeof(XT) == 2) x[base + i] = f2h(y);
        else x[base + i] = y;
    }
}

// state[request] <- x at the request's last token of the stack; x <- v
template <typename XT>
__global__ __launch_bounds__(256) void channel_mix_v7_kernel(const uint32_t *cursors, float *state, const XT *v, XT *x, ViewArgs vs, uint32_t C) {
    const uint32_t index = blockIdx.x * 256 + threadIdx.x, stack = blockIdx.y;
    if (index >= C / 4) return;
    const uint64_t bti = (uint64_t)stack * C + 4 * index;
    const float4 vv = load_vec4(v + bti), xx = load_vec4(x + bti); // both before the cursor's round trip and the store into the state
    const Cursor cur = read_cursor(cursors, stack, vs);
    if (stack - cur.token + 1 == cur.len) *reinterpret_cast<float4 *>(state + view_elem(vs, cur.batch, 0, 4 * index)) = xx;
    store_vec4(x + bti, vv);
}

int check_float(wrq_dtype dtype, const char *name) {
    if (dtype != WRQ_F16 && dtype != WRQ_F32) return fail(WRQ_ERR_TYPE, "%s: unsupported element type %d", name, (int)dtype);
    return WRQ_OK;
}

} // namespace

} // namespace wrq

using namespace wrq;

extern "C" {

int wrq_l2_norm(wrq_stream stream, const wrq_tensor *x, wrq_dtype dtype, float eps) {
    int s = check_layer_tensor(x, "l2_norm");
    if (s == WRQ_OK) s = check_float(dtype, "l2_norm");
    if (s != WRQ_OK) return s;
    const uint32_t *sh = x->shape;
    if (sh[3] != 1) return fail(WRQ_ERR_SHAPE, "l2_norm: data shape not match [%u, %u, %u, %u]", sh[0], sh[1], sh[2], sh[3]);
    if (sh[0] % 4) return fail(WRQ_ERR_ALIGNMENT, "l2_norm: row length %u not a multiple of 4", sh[0]);
    const uint64_t rows = (uint64_t)sh[1] * sh[2];
    if (sh[0] == 0 || rows == 0) return WRQ_OK;
    if (rows > 0x7fffffffull) return fail(WRQ_ERR_SIZE, "l2_norm: data size not match");
    hipStream_t hs = static_cast<hipStream_t>(stream);
    if (dtype == WRQ_F16) hipLaunchKernelGGL((l2_norm_kernel<uint16_t>), dim3((uint32_t)rows), dim3(64), 0, hs, static_cast<uint16_t *>(x->data), sh[0], eps);
    else hipLaunchKernelGGL((l2_norm_kernel<float>), dim3((uint32_t)rows), dim3(64), 0, hs, static_cast<float *>(x->data), sh[0], eps);
    return check_launch("l2_norm");
}

int wrq_control_k_v7(wrq_stream stream, const wrq_tensor *p, const wrq_tensor_view *a, const wrq_tensor_view *k) {
    int s = check_layer_tensor(p, "control_k_v7");
    if (s == WRQ_OK) s = check_layer_view(a, "control_k_v7");
    if (s == WRQ_OK) s = check_layer_view(k, "control_k_v7");
    if (s != WRQ_OK) return s;
    const uint32_t *sh = k->view.shape;
    // src/tensor/ops.rs:1812-1815
    const uint32_t ps[4] = {sh[0], 1, 1, 1};
    if (sh[3] != 1 || !same_shape(a->view.shape, sh) || !same_shape(p->shape, ps))
        return fail(WRQ_ERR_SHAPE, "control_k_v7: data shape not match [%u, %u, %u, %u]", sh[0], sh[1], sh[2], sh[3]);
    if (sh[0] == 0 || sh[1] == 0 || sh[2] == 0) return WRQ_OK;
    if (sh[1] > 65535u || sh[2] > 65535u) return fail(WRQ_ERR_SIZE, "control_k_v7: data size not match");
    const dim3 grid((sh[0] / 4 + 255) / 256, sh[1], sh[2]);
    const ViewArgs va = view_args(a->view), vk = view_args(k->view);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    const uint16_t *pp = static_cast<const uint16_t *>(p->data);
    const bool a16 = a->dtype == WRQ_F16, k16 = k->dtype == WRQ_F16;
    if (a16 && k16) hipLaunchKernelGGL((control_k_kernel<uint16_t, uint16_t>), grid, dim3(256), 0, hs, pp, static_cast<const uint16_t *>(a->data), static_cast<uint16_t *>(k->data), va, vk, sh[0]);
    else if (a16) hipLaunchKernelGGL((control_k_kernel<uint16_t, float>), grid, dim3(256), 0, hs, pp, static_cast<const uint16_t *>(a->data), static_cast<float *>(k->data), va, vk, sh[0]);
    else if (k16) hipLaunchKernelGGL((control_k_kernel<float, uint16_t>), grid, dim3(256), 0, hs, pp, static_cast<const float *>(a->data), static_cast<uint16_t *>(k->data), va, vk, sh[0]);
    else hipLaunchKernelGGL((control_k_kernel<float, float>), grid, dim3(256), 0, hs, pp, static_cast<const float *>(a->data), static_cast<float *>(k->data), va, vk, sh[0]);
    return check_launch("control_k_v7");
}

int wrq_time_mix_v7(wrq_stream stream, const wrq_tensor *cursors, const wrq_tensor_view *state, const wrq_tensor *r, const wrq_tensor *w, const wrq_tensor *n,
                    const wrq_tensor *x, wrq_dtype dtype) {
    int s = check_layer_tensor(cursors, "time_mix_v7");
    for (const wrq_tensor *t : {r, w, n, x})
        if (s == WRQ_OK) s = check_layer_tensor(t, "time_mix_v7");
    if (s == WRQ_OK) s = check_state_view(state, "time_mix_v7");
    if (s == WRQ_OK) s = check_float(dtype, "time_mix_v7");
    if (s != WRQ_OK) return s;
    if (state->dtype != WRQ_F32) return fail(WRQ_ERR_TYPE, "time_mix_v7: the state is f32");
    const uint32_t *sh = x->shape, *st = state->view.shape; // [S, H, A, 1]
    const uint32_t S = sh[0], H = sh[1], A = sh[2];
    // src/tensor/ops.rs:1695-1698
    const uint32_t ns[4] = {S, H, A, 4};
    if (sh[3] != 1 || !same_shape(r->shape, sh) || !same_shape(w->shape, sh) || !same_shape(n->shape, ns) || st[0] != S * H || st[1] != S + 1 || st[3] != 1)
        return fail(WRQ_ERR_SHAPE, "time_mix_v7: data shape not match [%u, %u, %u, %u]", sh[0], sh[1], sh[2], sh[3]);
    if (cursors->shape[0] < A) return fail(WRQ_ERR_SHAPE, "time_mix_v7: %u cursors for %u tokens", cursors->shape[0], A);
    if (S == 0 || H == 0 || A == 0) return WRQ_OK;
    const ViewArgs vs = view_args(state->view);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    const uint32_t *cur = static_cast<const uint32_t *>(cursors->data);
    float *sp = static_cast<float *>(state->data);
#define WRQ_TM7(SZ)                                                                                                                                  \
    if (S == SZ) {                                                                                                                                   \
        if (dtype == WRQ_F16)                                                                                                                        \
            hipLaunchKernelGGL((time_mix_v7_kernel<uint16_t, SZ>), dim3(H), dim3(256), 0, hs, cur, sp, static_cast<const uint16_t *>(r->data),        \
                               static_cast<const uint16_t *>(w->data), static_cast<const uint16_t *>(n->data), static_cast<uint16_t *>(x->data), vs, H, A); \
        else                                                                                                                                         \
            hipLaunchKernelGGL((time_mix_v7_kernel<float, SZ>), dim3(H), dim3(256), 0, hs, cur, sp, static_cast<const float *>(r->data),              \
                               static_cast<const float *>(w->data), static_cast<const float *>(n->data), static_cast<float *>(x->data), vs, H, A);   \
        return check_launch("time_mix_v7");                                                                                                          \
    }
    WRQ_TM7(32) WRQ_TM7(64) WRQ_TM7(128)
#undef WRQ_TM7
    return fail(WRQ_ERR_UNSUPPORTED, "time_mix_v7: head size %u (32, 64 or 128 is built)", S);
}

int wrq_time_first_v7(wrq_stream stream, const wrq_tensor *u, const wrq_tensor *r, const wrq_tensor *n, const wrq_tensor *x, wrq_dtype dtype) {
    int s = WRQ_OK;
    for (const wrq_tensor *t : {u, r, n, x})
        if (s == WRQ_OK) s = check_layer_tensor(t, "time_first_v7");
    if (s == WRQ_OK) s = check_float(dtype, "time_first_v7");
    if (s != WRQ_OK) return s;
    const uint32_t *sh = x->shape;
    const uint32_t S = sh[0], H = sh[1], A = sh[2];
    // src/tensor/ops.rs:1755-1757
    const uint32_t us[4] = {S, H, 1, 1}, ns[4] = {S, H, A, 4};
    if (sh[3] != 1 || !same_shape(r->shape, sh) || !same_shape(u->shape, us) || !same_shape(n->shape, ns))
        return fail(WRQ_ERR_SHAPE, "time_first_v7: data shape not match [%u, %u, %u, %u]", sh[0], sh[1], sh[2], sh[3]);
    if (S == 0 || H == 0 || A == 0) return WRQ_OK;
    if (A > 65535u) return fail(WRQ_ERR_SIZE, "time_first_v7: data size not match");
    hipStream_t hs = static_cast<hipStream_t>(stream);
    const uint16_t *up = static_cast<const uint16_t *>(u->data);
    if (dtype == WRQ_F16)
        hipLaunchKernelGGL((time_first_v7_kernel<uint16_t>), dim3(H, A), dim3(64), 0, hs, up, static_cast<const uint16_t *>(r->data), static_cast<const uint16_t *>(n->data),
                           static_cast<uint16_t *>(x->data), S, H, A);
    else
        hipLaunchKernelGGL((time_first_v7_kernel<float>), dim3(H, A), dim3(64), 0, hs, up, static_cast<const float *>(r->data), static_cast<const float *>(n->data),
                           static_cast<float *>(x->data), S, H, A);
    return check_launch("time_first_v7");
}

int wrq_channel_mix_v7(wrq_stream stream, const wrq_tensor *cursors, const wrq_tensor_view *state, const wrq_tensor *v, const wrq_tensor *x, wrq_dtype dtype) {
    int s = check_layer_tensor(cursors, "channel_mix_v7");
    for (const wrq_tensor *t : {v, x})
        if (s == WRQ_OK) s = check_layer_tensor(t, "channel_mix_v7");
    if (s == WRQ_OK) s = check_state_view(state, "channel_mix_v7");
    if (s == WRQ_OK) s = check_float(dtype, "channel_mix_v7");
    if (s != WRQ_OK) return s;
    if (state->dtype != WRQ_F32) return fail(WRQ_ERR_TYPE, "channel_mix_v7: the state is f32");
    const uint32_t *sh = x->shape, *st = state->view.shape;
    // src/tensor/ops.rs:1929-1930
    if (!same_shape(v->shape, sh) || st[0] != sh[0] || st[1] != 1 || st[3] != 1 || sh[2] != 1 || sh[3] != 1)
        return fail(WRQ_ERR_SHAPE, "channel_mix_v7: data shape not match [%u, %u, %u, %u]", sh[0], sh[1], sh[2], sh[3]);
    if (cursors->shape[0] < sh[1]) return fail(WRQ_ERR_SHAPE, "channel_mix_v7: %u cursors for %u tokens", cursors->shape[0], sh[1]);
    if (sh[0] % 4) return fail(WRQ_ERR_ALIGNMENT, "channel_mix_v7: row length %u not a multiple of 4", sh[0]);
    if (sh[0] == 0 || sh[1] == 0) return WRQ_OK;
    if (sh[1] > 65535u) return fail(WRQ_ERR_SIZE, "channel_mix_v7: data size not match");
    const dim3 grid((sh[0] / 4 + 255) / 256, sh[1]);
    const ViewArgs vs = view_args(state->view);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    const uint32_t *cur = static_cast<const uint32_t *>(cursors->data);
    if (dtype == WRQ_F16)
        hipLaunchKernelGGL((channel_mix_v7_kernel<uint16_t>), grid, dim3(256), 0, hs, cur, static_cast<float *>(state->data), static_cast<const uint16_t *>(v->data),
                           static_cast<uint16_t *>(x->data), vs, sh[0]);
    else
        hipLaunchKernelGGL((channel_mix_v7_kernel<float>), grid, dim3(256), 0, hs, cur, static_cast<float *>(state->data), static_cast<const float *>(v->data),
                           static_cast<float *>(x->data), vs, sh[0]);
    return check_launch("channel_mix_v7");
}

} // extern "C"

// C ABI of libwrq_hip.so: argument checks of the reference's op constructors, view
// resolution and kernel selection.  No kernel lives here.
#include "wrq_device.h"
#include "wrq_host.h"

#include <stdlib.h>

#include <ctype.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <mutex>

namespace wrq {

namespace {
thread_local char g_error[512] = "";
}

int fail(int status, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return status;
}

// ---- tuning overrides: read from the environment once, then only from this table
namespace {
const char *const kTuneNames[kTuneCount] = {"gemv_oneshot", "gemv_rows", "gemv_sl", "gemv_nt", "gemv_grid", "gemm_ntile", "gemm_mrt",
                                            "gemm_kg", "gemm_ksplit", "vec_chunk_min_t", "gemm_tail", "gemv_waverows", "gemm_prio", "gemv_rows_tokens", "gemm_table", "gemv_table"};
std::atomic<int> g_tune[kTuneCount];
std::once_flag g_tune_once;
std::atomic<bool> g_test_hooks{false}; // WRQ_TEST_HOOKS was set when the library first looked: overrides stay allowed
std::atomic<bool> g_launched{false};   // some kernel of the library has been launched by this process

void tune_load_env() {
    for (int k = 0; k < kTuneCount; k++) {
        char name[64] = "WRQ_";
        size_t n = 4;
        for (const char *c = kTuneNames[k]; *c && n + 1 < sizeof(name); c++) name[n++] = (char)toupper((unsigned char)*c);
        name[n] = 0;
        const char *e = getenv(name);
        g_tune[k].store((e && *e) ? atoi(e) : -1, std::memory_order_relaxed);
    }
    const char *hooks = getenv("WRQ_TEST_HOOKS");
    g_test_hooks.store(hooks && *hooks && atoi(hooks) != 0, std::memory_order_relaxed);
}
} // namespace

int tune(TuneKey key, int fallback) {
    std::call_once(g_tune_once, tune_load_env);
    const int v = g_tune[key].load(std::memory_order_relaxed);
    return v >= 0 ? v : fallback;
}

bool tune_is_set(TuneKey key) {
    std::call_once(g_tune_once, tune_load_env);
    return g_tune[key].load(std::memory_order_relaxed) >= 0;
}

int tune_set(const char *name, int value) {
    std::call_once(g_tune_once, tune_load_env);
    // the table is process-wide and the launch path reads it without a lock: once launches have begun, only a
    // process that declared itself a test (WRQ_TEST_HOOKS=1 in its environment at load time) may still change it
    if (g_launched.load(std::memory_order_relaxed) && !g_test_hooks.load(std::memory_order_relaxed))
        return fail(WRQ_ERR_UNSUPPORTED, "overrides are refused once a kernel has been launched (WRQ_TEST_HOOKS=1 in the environment keeps them)");
    for (int k = 0; k < kTuneCount; k++)
        if (strcmp(name, kTuneNames[k]) == 0) {
            g_tune[k].store(value < 0 ? -1 : value, std::memory_order_relaxed);
            return WRQ_OK;
        }
    return fail(WRQ_ERR_UNSUPPORTED, "unknown tuning key %s", name);
}

int check_launch(const char *what) {
    g_launched.store(true, std::memory_order_relaxed);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(WRQ_ERR_DEVICE, "%s: %s", what, hipGetErrorString(e));
    return WRQ_OK;
}

namespace {

struct Shape4 {
    uint64_t d[4];
    uint64_t len() const { return d[0] * d[1] * d[2] * d[3]; }
    bool operator==(const Shape4 &o) const { return memcmp(d, o.d, sizeof(d)) == 0; }
};

Shape4 shape_of(const uint32_t s[4]) { return Shape4{{s[0], s[1], s[2], s[3]}}; }

// TensorShape::check_shape, src/tensor/mod.rs:213-219
int check_shape(const Shape4 &got, const Shape4 &want) {
    if (got == want) return WRQ_OK;
    return fail(WRQ_ERR_SHAPE, "tensor shape not match: (%llu, %llu, %llu, %llu) vs. (%llu, %llu, %llu, %llu)",
                (unsigned long long)got.d[0], (unsigned long long)got.d[1], (unsigned long long)got.d[2],
                (unsigned long long)got.d[3], (unsigned long long)want.d[0], (unsigned long long)want.d[1],
                (unsigned long long)want.d[2], (unsigned long long)want.d[3]);
}

uint64_t div_ceil(uint64_t a, uint64_t b) { return (a + b - 1) / b; }

#define WRQ_TRY(expr)                  \
    do {                               \
        const int _s = (expr);         \
        if (_s != WRQ_OK) return _s;   \
    } while (0)

int need(const void *p, const char *name) {
    return p ? WRQ_OK : fail(WRQ_ERR_NULL, "null pointer: %s", name);
}

int need_tensor(const wrq_tensor *t, const char *name) {
    WRQ_TRY(need(t, name));
    if (!t->data) return fail(WRQ_ERR_NULL, "null pointer: %s.data", name);
    return WRQ_OK;
}

int need_view(const wrq_tensor_view *v, const char *name, bool typed) {
    WRQ_TRY(need(v, name));
    if (!v->data) return fail(WRQ_ERR_NULL, "null pointer: %s.data", name);
    if (typed && v->dtype != WRQ_F16 && v->dtype != WRQ_F32) return fail(WRQ_ERR_TYPE, "data type mismatch");
    for (int i = 0; i < 4; i++) {
        // a view is a slice of its parent (src/tensor/mod.rs:1121-1141)
        if ((uint64_t)v->view.offset[i] + v->view.shape[i] > v->view.stride[i])
            return fail(WRQ_ERR_SHAPE, "slice %u..%llu out of range for dimension size %u", v->view.offset[i],
                        (unsigned long long)v->view.offset[i] + v->view.shape[i], v->view.stride[i]);
    }
    if (v->view.shape[3] != 1 || v->view.offset[3] != 0)
        return fail(WRQ_ERR_UNSUPPORTED, "views along the fourth axis are not supported");
    return WRQ_OK;
}

// Matrix views of the chunk products.  The reference sizes the scale tensor by the *view's* length
// (src/tensor/ops.rs:1088-1090, :1166-1169) while its shader indexes the scales by the flat index in the
// *parent* and steps from row to row by the view's width (src/shaders/matmul_mat_int8.wgsl:66-68, :99-103):
// the two agree only for a view that starts at the origin and keeps whole rows and row counts, that is the
// whole tensor or its leading batches.  Those are taken; any other slice has no consistent meaning there and
// is refused.  The model builders pass `w.view(.., .., .., ..)` (src/tensor/matrix.rs:136-160).
int check_matrix_view(const wrq_view &v) {
    for (int i = 0; i < 4; i++)
        if (v.offset[i] != 0) return fail(WRQ_ERR_UNSUPPORTED, "sliced matrix views are not supported: offset %u along axis %d", v.offset[i], i);
    if (v.shape[0] != v.stride[0] || v.shape[1] != v.stride[1] || v.shape[3] != v.stride[3])
        return fail(WRQ_ERR_UNSUPPORTED, "sliced matrix views are not supported: (%u, %u, %u, %u) of (%u, %u, %u, %u)", v.shape[0],
                    v.shape[1], v.shape[2], v.shape[3], v.stride[0], v.stride[1], v.stride[2], v.stride[3]);
    return WRQ_OK;
}

// Resolves views into element strides and offset pointers (compute_index of the
// shaders, src/shaders/matmul_vec_int8.wgsl:31-35).
void resolve(const wrq_tensor_view &in, const wrq_tensor_view &out, MatmulArgs &a) {
    const wrq_view &vi = in.view, &vo = out.view;
    const size_t si = in.dtype == WRQ_F16 ? 2 : 4, so = out.dtype == WRQ_F16 ? 2 : 4;
    a.x_token_stride = vi.stride[0];
    a.x_batch_stride = (uint64_t)vi.stride[0] * vi.stride[1];
    a.out_token_stride = vo.stride[0];
    a.out_batch_stride = (uint64_t)vo.stride[0] * vo.stride[1];
    const uint64_t xo = ((uint64_t)vi.offset[2] * vi.stride[1] + vi.offset[1]) * vi.stride[0] + vi.offset[0];
    const uint64_t oo = ((uint64_t)vo.offset[2] * vo.stride[1] + vo.offset[1]) * vo.stride[0] + vo.offset[0];
    a.x = static_cast<const uint8_t *>(in.data) + xo * si;
    a.out = static_cast<uint8_t *>(out.data) + oo * so;
    a.out_f16 = out.dtype == WRQ_F16;
}

enum Entry { kVec, kMat };

// Shared body of the four product entry points.  `mshape` is the matrix shape in
// bytes-per-row terms as the reference sees it: [K, R, B, 1] (int8) or [K/2, R, B, 1] (nf4).
struct Prepared {
    MatmulArgs a;
    int in_f16;
    bool mfma; // route to the matrix-core kernel
};

int prepare(Entry entry, Quant quant, const void *w, const Shape4 &mshape, const wrq_tensor *scale,
            const wrq_tensor *table, const wrq_tensor_view *input, const wrq_tensor_view *output, int act,
            Prepared &out) {
    if (act < WRQ_ACT_NONE || act > WRQ_ACT_SILU) return fail(WRQ_ERR_UNSUPPORTED, "unknown activation %d", act);
    const Shape4 os = shape_of(output->view.shape), is = shape_of(input->view.shape);
    const uint64_t m = os.d[0], n = os.d[1], b = os.d[2], k = is.d[0];
    // src/tensor/ops.rs:805-813 (int8), :907-916 (nf4), :1094-1103, :1172-1181
    if (quant == kFp16) {
        WRQ_TRY(check_shape(mshape, Shape4{{k, m, b, 1}})); // src/tensor/ops.rs:713-720, :1015-1022
    } else if (quant == kInt8) {
        const uint64_t len = mshape.len();
        WRQ_TRY(check_shape(shape_of(scale->shape), Shape4{{div_ceil(len << 1, WRQ_INT8_BLOCK_SIZE), 1, 1, 1}}));
        WRQ_TRY(check_shape(mshape, Shape4{{k, m, b, 1}}));
    } else {
        const uint64_t len = mshape.len() << 1;
        WRQ_TRY(check_shape(shape_of(scale->shape), Shape4{{div_ceil(len, WRQ_NF4_BLOCK_SIZE), 1, 1, 1}}));
        WRQ_TRY(check_shape(mshape, Shape4{{k >> 1, m, b, 1}}));
        WRQ_TRY(check_shape(shape_of(table->shape), Shape4{{16, 1, 1, 1}}));
    }
    WRQ_TRY(check_shape(is, Shape4{{k, n, b, 1}}));
    WRQ_TRY(check_shape(os, Shape4{{m, n, b, 1}}));

    // preconditions the reference leaves to the caller
    const uint64_t block = quant == kFp16 ? 1 : quant == kInt8 ? WRQ_INT8_BLOCK_SIZE : WRQ_NF4_BLOCK_SIZE;
    const uint64_t group = quant == kNf4 ? 8 : 4; // elements per load unit of the shaders (vec4 / 8 nibbles)
    if ((k * m * b) % block)
        return fail(WRQ_ERR_ALIGNMENT, "matrix size %llu is not a multiple of the %llu-element block",
                    (unsigned long long)(k * m * b), (unsigned long long)block);
    if (m % 4) return fail(WRQ_ERR_ALIGNMENT, "output rows %llu not a multiple of 4", (unsigned long long)m);
    if (k % group) return fail(WRQ_ERR_ALIGNMENT, "input columns %llu not a multiple of %llu", (unsigned long long)k, (unsigned long long)group);
    if (input->view.offset[0] % group || input->view.stride[0] % group)
        return fail(WRQ_ERR_ALIGNMENT, "input view offset/stride along x not a multiple of %llu", (unsigned long long)group);
    if (output->view.offset[0] % 4 || output->view.stride[0] % 4)
        return fail(WRQ_ERR_ALIGNMENT, "output view offset/stride along x not a multiple of 4");
    if ((uintptr_t)w % (quant == kFp16 ? 8 : 4) || (scale && (uintptr_t)scale->data % 4) || (uintptr_t)input->data % 16 || (uintptr_t)output->data % 16)
        return fail(WRQ_ERR_ALIGNMENT, "device pointers must be 16-byte aligned");
    if (entry == kMat) {
        // src/tensor/ops.rs:1068-1070, :1146-1149; the k-step of the shaders fetches one
        // scale per 32 (int8) / 64 (nf4) columns
        if (n % 4) return fail(WRQ_ERR_ALIGNMENT, "tokens %llu not a multiple of 4", (unsigned long long)n);
        const uint64_t kstep = quant == kFp16 ? 4 : quant == kInt8 ? 32 : 64;
        if (k % kstep) return fail(WRQ_ERR_ALIGNMENT, "input columns %llu not a multiple of %llu", (unsigned long long)k, (unsigned long long)kstep);
    }
    if (m > 0xffffffffull || n > 0xffffffffull || k > 0xffffffffull) return fail(WRQ_ERR_SIZE, "data size not match");

    MatmulArgs &a = out.a;
    a = MatmulArgs{};
    a.w = static_cast<const uint8_t *>(w);
    a.scale = scale ? static_cast<const uint16_t *>(scale->data) : nullptr;
    a.quant = table ? static_cast<const float *>(table->data) : nullptr;
    a.K = (uint32_t)k;
    a.R = (uint32_t)m;
    a.T = (uint32_t)n;
    a.B = (uint32_t)b;
    a.act = act;
    resolve(*input, *output, a);
    const int in_f16 = input->dtype == WRQ_F16;

    // Matrix cores need K in whole 128-steps, 16-byte activation rows and output quads on
    // their natural alignment; everything else runs on the VALU kernels, which accept
    // every shape the reference accepts.
    const size_t xs = in_f16 ? 2 : 4, osz = a.out_f16 ? 2 : 4;
    const bool mfma_ok = (k % 128 == 0) && ((uintptr_t)a.w % 16 == 0) && ((uintptr_t)a.x % 16 == 0) &&
                         ((a.x_token_stride * xs) % 16 == 0) && ((a.x_batch_stride * xs) % 16 == 0) &&
                         ((uintptr_t)a.out % (4 * osz) == 0) && ((a.out_token_stride * osz) % (4 * osz) == 0) &&
                         ((a.out_batch_stride * osz) % (4 * osz) == 0);
    // decode entry point with several tokens: up to 4 (int8, fp16) or 3 (nf4) tokens of f16
    // activations share one pass of the one-shot VALU kernels (7B int8 step: 1.8 - 2.1 ms at 2 - 4
    // tokens against 2.8 ms; f16 head: 97 us at 4 tokens against 120); longer runs go to the
    // matrix-core kernel.
    const uint64_t chunk_min_t = (uint64_t)tune(kTuneVecChunkMinT, quant == kNf4 ? 4 : 5);
    // f32 activations cost the matrix-core kernel a second LDS tile and a second product chain (they are split
    // into two f16 halves there, exact to 2^-22 for |x| <= 65535): below 16 tokens the VALU kernels, which take
    // f32 as it is, are the faster choice and have no range limit
    const bool chunk = entry == kMat ? true : n >= (in_f16 ? chunk_min_t : (uint64_t)16);
    out.in_f16 = in_f16;
    out.mfma = chunk && mfma_ok;
    return WRQ_OK;
}

int launch_vec(hipStream_t stream, Quant quant, const Prepared &p) {
    return quant == kFp16 ? launch_gemv_fp16(stream, p.in_f16, p.a) : launch_gemv(stream, quant, p.in_f16, p.a);
}

int launch_chunk(hipStream_t stream, Quant quant, const Prepared &p, bool noalloc) {
    if (p.a.K == 0) return launch_vec(stream, quant, p); // nothing to stream: plain zeros through the generic kernel
    return noalloc ? launch_gemm_noalloc(stream, quant, p.in_f16, p.a) : launch_gemm(stream, quant, p.in_f16, p.a);
}

int matmul(hipStream_t stream, Entry entry, Quant quant, const void *w, const Shape4 &mshape,
           const wrq_tensor *scale, const wrq_tensor *table, const wrq_tensor_view *input,
           const wrq_tensor_view *output, int act, bool noalloc = false) {
    Prepared p;
    WRQ_TRY(prepare(entry, quant, w, mshape, scale, table, input, output, act, p));
    if (p.mfma) return launch_chunk(stream, quant, p, noalloc);
    return launch_vec(stream, quant, p);
}

// Runs of consecutive decode-shaped ops with one input type and token count share launches.
int dispatch_group(hipStream_t stream, Quant quant, const Prepared *ops, int n) {
    int i = 0;
    while (i < n) {
        // a run of ops of one kernel family, input type and token count (every op brings its own
        // nf4 table: each Matrix of the reference owns a table tensor)
        MatmulArgs run[kMaxGroup];
        int m = 0;
        while (i + m < n && m < kMaxGroup && ops[i + m].mfma == ops[i].mfma && ops[i + m].in_f16 == ops[i].in_f16 &&
               ops[i + m].a.T == ops[i].a.T) {
            run[m] = ops[i + m].a;
            m++;
        }
        if (ops[i].mfma && ops[i].a.K != 0)
            WRQ_TRY(launch_gemm_group(stream, quant, ops[i].in_f16, run, m));
        else
            WRQ_TRY(launch_gemv_group(stream, quant, ops[i].in_f16, run, m));
        i += m;
    }
    return WRQ_OK;
}

} // namespace
} // namespace wrq

using namespace wrq;

extern "C" {

int wrq_abi_version(void) { return WRQ_ABI_VERSION; }
int wrq_abi_minor(void) { return WRQ_ABI_MINOR; }

const char *wrq_last_error(void) { return g_error; }

const char *wrq_status_string(int status) {
    switch (status) {
    case WRQ_OK: return "ok";
    case WRQ_ERR_SHAPE: return "tensor shape not match";
    case WRQ_ERR_SIZE: return "data size not match";
    case WRQ_ERR_TYPE: return "data type mismatch";
    case WRQ_ERR_ALIGNMENT: return "operand alignment or multiple not met";
    case WRQ_ERR_UNSUPPORTED: return "not supported";
    case WRQ_ERR_NULL: return "null pointer";
    case WRQ_ERR_DEVICE: return "device error";
    default: return "unknown status";
    }
}

int wrq_debug_override(const char *key, int value) {
    if (!key) return fail(WRQ_ERR_NULL, "null pointer: key");
    return tune_set(key, value);
}

int wrq_debug_stamps(void *buffer, uint64_t bytes) {
    (void)tune(kTuneGemvOneshot, 0); // makes sure the environment has been read
    if (!g_test_hooks.load(std::memory_order_relaxed))
        return fail(WRQ_ERR_UNSUPPORTED, "wrq_debug_stamps needs WRQ_TEST_HOOKS=1 in the environment");
    return stamps_set(buffer, bytes);
}

int wrq_init(void) {
    (void)tune(kTuneGemvOneshot, 0); // reads the environment overrides now rather than at the first product
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(WRQ_ERR_DEVICE, "hipGetDevice: %s", hipGetErrorString(e));
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return fail(WRQ_ERR_DEVICE, "hipGetDeviceProperties: %s", hipGetErrorString(e));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(WRQ_ERR_UNSUPPORTED, "device %d is %s; this library holds gfx950 code only", dev, prop.gcnArchName);
    return prepare_gemm_scratch();
}

int wrq_quantize_mat_int8(wrq_stream stream, const wrq_tensor *input, const wrq_tensor *minmax,
                          const wrq_tensor *output) {
    WRQ_TRY(need_tensor(input, "input"));
    WRQ_TRY(need_tensor(minmax, "minmax"));
    WRQ_TRY(need_tensor(output, "output"));
    // src/tensor/ops.rs:2400-2406
    const Shape4 shape = shape_of(output->shape);
    const uint64_t len = shape.len();
    WRQ_TRY(check_shape(shape_of(input->shape), shape));
    WRQ_TRY(check_shape(shape_of(minmax->shape), Shape4{{div_ceil(len, WRQ_INT8_BLOCK_SIZE) << 1, 1, 1, 1}}));
    if (len % WRQ_INT8_BLOCK_SIZE)
        return fail(WRQ_ERR_ALIGNMENT, "matrix size %llu is not a multiple of the 128-element block", (unsigned long long)len);
    if ((uintptr_t)input->data % 16 || (uintptr_t)output->data % 8 || (uintptr_t)minmax->data % 4)
        return fail(WRQ_ERR_ALIGNMENT, "device pointers must be 16-byte aligned");
    return launch_quant_int8(static_cast<hipStream_t>(stream), input->data, minmax->data, output->data, len);
}

int wrq_quantize_mat_nf4(wrq_stream stream, const wrq_tensor *input, const wrq_tensor *quant,
                         const wrq_tensor *absmax, const wrq_tensor *output) {
    WRQ_TRY(need_tensor(input, "input"));
    WRQ_TRY(need_tensor(quant, "quant"));
    WRQ_TRY(need_tensor(absmax, "absmax"));
    WRQ_TRY(need_tensor(output, "output"));
    // src/tensor/ops.rs:2496-2503
    const Shape4 shape = shape_of(output->shape);
    const Shape4 input_shape{{shape.d[0] << 1, shape.d[1], shape.d[2], shape.d[3]}};
    const uint64_t len = input_shape.len();
    WRQ_TRY(check_shape(shape_of(input->shape), input_shape));
    WRQ_TRY(check_shape(shape_of(absmax->shape), Shape4{{div_ceil(len, WRQ_NF4_BLOCK_SIZE), 1, 1, 1}}));
    WRQ_TRY(check_shape(shape_of(quant->shape), Shape4{{16, 1, 1, 1}}));
    if (len % WRQ_NF4_BLOCK_SIZE)
        return fail(WRQ_ERR_ALIGNMENT, "matrix size %llu is not a multiple of the 64-element block", (unsigned long long)len);
    if ((uintptr_t)input->data % 16 || (uintptr_t)output->data % 4 || (uintptr_t)absmax->data % 2 || (uintptr_t)quant->data % 4)
        return fail(WRQ_ERR_ALIGNMENT, "device pointers must be 16-byte aligned");
    return launch_quant_nf4(static_cast<hipStream_t>(stream), input->data, quant->data, absmax->data, output->data, len);
}

int wrq_matmul_vec_int8(wrq_stream stream, const wrq_tensor *matrix, const wrq_tensor *minmax,
                        const wrq_tensor_view *input, const wrq_tensor_view *output, int act, int sparse) {
    (void)sparse; // skipping all-zero input groups never changes a finite result
    WRQ_TRY(need_tensor(matrix, "matrix"));
    WRQ_TRY(need_tensor(minmax, "minmax"));
    WRQ_TRY(need_view(input, "input", true));
    WRQ_TRY(need_view(output, "output", true));
    return matmul(static_cast<hipStream_t>(stream), kVec, kInt8, matrix->data, shape_of(matrix->shape), minmax,
                  nullptr, input, output, act);
}

int wrq_matmul_vec_nf4(wrq_stream stream, const wrq_tensor *matrix, const wrq_tensor *quant,
                       const wrq_tensor *absmax, const wrq_tensor_view *input,
                       const wrq_tensor_view *output, int act, int sparse) {
    (void)sparse;
    WRQ_TRY(need_tensor(matrix, "matrix"));
    WRQ_TRY(need_tensor(quant, "quant"));
    WRQ_TRY(need_tensor(absmax, "absmax"));
    WRQ_TRY(need_view(input, "input", true));
    WRQ_TRY(need_view(output, "output", true));
    return matmul(static_cast<hipStream_t>(stream), kVec, kNf4, matrix->data, shape_of(matrix->shape), absmax, quant,
                  input, output, act);
}

int wrq_matmul_vec_int8_group(wrq_stream stream, const wrq_vec_int8_op *ops, int count) {
    if (count < 0 || count > WRQ_MAX_GROUP) return fail(WRQ_ERR_SIZE, "data size not match: %d vs. %d", count, WRQ_MAX_GROUP);
    if (count == 0) return WRQ_OK;
    WRQ_TRY(need(ops, "ops"));
    Prepared prepared[WRQ_MAX_GROUP];
    for (int i = 0; i < count; i++) { // every op is checked before anything is launched
        const wrq_vec_int8_op &o = ops[i];
        WRQ_TRY(need_tensor(o.matrix, "matrix"));
        WRQ_TRY(need_tensor(o.minmax, "minmax"));
        WRQ_TRY(need_view(o.input, "input", true));
        WRQ_TRY(need_view(o.output, "output", true));
        WRQ_TRY(prepare(kVec, kInt8, o.matrix->data, shape_of(o.matrix->shape), o.minmax, nullptr, o.input, o.output,
                        o.act, prepared[i]));
    }
    return dispatch_group(static_cast<hipStream_t>(stream), kInt8, prepared, count);
}

int wrq_matmul_vec_nf4_group(wrq_stream stream, const wrq_vec_nf4_op *ops, int count) {
    if (count < 0 || count > WRQ_MAX_GROUP) return fail(WRQ_ERR_SIZE, "data size not match: %d vs. %d", count, WRQ_MAX_GROUP);
    if (count == 0) return WRQ_OK;
    WRQ_TRY(need(ops, "ops"));
    Prepared prepared[WRQ_MAX_GROUP];
    for (int i = 0; i < count; i++) {
        const wrq_vec_nf4_op &o = ops[i];
        WRQ_TRY(need_tensor(o.matrix, "matrix"));
        WRQ_TRY(need_tensor(o.quant, "quant"));
        WRQ_TRY(need_tensor(o.absmax, "absmax"));
        WRQ_TRY(need_view(o.input, "input", true));
        WRQ_TRY(need_view(o.output, "output", true));
        WRQ_TRY(prepare(kVec, kNf4, o.matrix->data, shape_of(o.matrix->shape), o.absmax, o.quant, o.input, o.output,
                        o.act, prepared[i]));
    }
    return dispatch_group(static_cast<hipStream_t>(stream), kNf4, prepared, count);
}

int wrq_matmul_mat_int8(wrq_stream stream, const wrq_tensor_view *matrix, const wrq_tensor *minmax,
                        const wrq_tensor_view *input, const wrq_tensor_view *output, int act) {
    WRQ_TRY(need_view(matrix, "matrix", false));
    WRQ_TRY(need_tensor(minmax, "minmax"));
    WRQ_TRY(need_view(input, "input", true));
    WRQ_TRY(need_view(output, "output", true));
    WRQ_TRY(check_matrix_view(matrix->view));
    return matmul(static_cast<hipStream_t>(stream), kMat, kInt8, matrix->data, shape_of(matrix->view.shape), minmax,
                  nullptr, input, output, act);
}

int wrq_matmul_mat_int8_noalloc(wrq_stream stream, const wrq_tensor_view *matrix, const wrq_tensor *minmax,
                                const wrq_tensor_view *input, const wrq_tensor_view *output, int act) {
    WRQ_TRY(need_view(matrix, "matrix", false));
    WRQ_TRY(need_tensor(minmax, "minmax"));
    WRQ_TRY(need_view(input, "input", true));
    WRQ_TRY(need_view(output, "output", true));
    WRQ_TRY(check_matrix_view(matrix->view));
    return matmul(static_cast<hipStream_t>(stream), kMat, kInt8, matrix->data, shape_of(matrix->view.shape), minmax,
                  nullptr, input, output, act, true);
}

int wrq_matmul_mat_nf4(wrq_stream stream, const wrq_tensor_view *matrix, const wrq_tensor *quant,
                       const wrq_tensor *absmax, const wrq_tensor_view *input,
                       const wrq_tensor_view *output, int act) {
    WRQ_TRY(need_view(matrix, "matrix", false));
    WRQ_TRY(need_tensor(quant, "quant"));
    WRQ_TRY(need_tensor(absmax, "absmax"));
    WRQ_TRY(need_view(input, "input", true));
    WRQ_TRY(need_view(output, "output", true));
    WRQ_TRY(check_matrix_view(matrix->view));
    return matmul(static_cast<hipStream_t>(stream), kMat, kNf4, matrix->data, shape_of(matrix->view.shape), absmax,
                  quant, input, output, act);
}

/* plain f16 weights */

int wrq_matmul_vec_fp16(wrq_stream stream, const wrq_tensor *matrix, const wrq_tensor_view *input,
                        const wrq_tensor_view *output, int act, int sparse) {
    (void)sparse;
    WRQ_TRY(need_tensor(matrix, "matrix"));
    WRQ_TRY(need_view(input, "input", true));
    WRQ_TRY(need_view(output, "output", true));
    return matmul(static_cast<hipStream_t>(stream), kVec, kFp16, matrix->data, shape_of(matrix->shape), nullptr, nullptr,
                  input, output, act);
}

int wrq_matmul_mat_fp16(wrq_stream stream, const wrq_tensor_view *matrix, const wrq_tensor_view *input,
                        const wrq_tensor_view *output, int act) {
    WRQ_TRY(need_view(matrix, "matrix", false));
    WRQ_TRY(need_view(input, "input", true));
    WRQ_TRY(need_view(output, "output", true));
    WRQ_TRY(check_matrix_view(matrix->view));
    return matmul(static_cast<hipStream_t>(stream), kMat, kFp16, matrix->data, shape_of(matrix->view.shape), nullptr,
                  nullptr, input, output, act);
}

} // extern "C"

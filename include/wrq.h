/*
 * wrq.h -- C ABI of libwrq_hip.so: web-rwkv's quantized-weight matrix path
 * (Int8 / NF4 packing and the products on packed weights) for MI355X (gfx950).
 *
 * Every entry point replaces one constructor of the reference's `TensorOp`
 * (src/tensor/ops.rs) and takes the same operands in the same order.  Where the
 * reference builds a deferred op that `Context::encode` later records into the
 * single wgpu queue (src/tensor/ops.rs:78-144), these calls enqueue the work on
 * the HIP stream given as first argument and return at once; work on one stream
 * runs in call order with no host synchronisation, like ops of one command
 * buffer.  All pointers inside tensors are device pointers owned by the caller
 * and must stay valid until the stream has passed the call.  No entry point
 * allocates, frees or copies to the host.  All may be called from several threads at
 * once, and calls on different streams may overlap in time: products on the matrix-core kernel
 * (wrq_matmul_mat_*, and wrq_matmul_vec_* from 5 tokens on, nf4: 4) may split K over workgroups
 * and keep partial sums in library-owned scratch memory, of which every stream gets a slice of its
 * own (4 per device, 32 MiB each, handed out in order of first use and kept until the process ends;
 * products on further streams run unsplit: correct, slower).  A call recorded into a HIP graph keeps
 * the slice of the stream it was captured on, so two graphs captured on ONE stream must not be
 * replayed at the same time on different streams; wrq_matmul_mat_int8_noalloc has one fixed array
 * per device and its calls must not overlap at all.  Streams are told apart by their handle:
 * hipStreamPerThread is one handle for every thread, so split products issued on it from several
 * threads share a slice and must not overlap either (give such threads streams of their own).
 *
 * Shapes use the reference's order, x fastest (src/tensor/shape.rs:97): a matrix
 * `[K, R, B, 1]` holds B * R rows of K contiguous elements.
 *
 * Return value: WRQ_OK or a wrq_status error; the checks of the reference's
 * op constructors (`check_shape`, src/tensor/mod.rs:213-219) are made before
 * anything is launched, and its unchecked preconditions (R % 4, K % 4 ...) are
 * checked here too.  wrq_last_error() gives the message of the calling thread's
 * last failure, worded like the reference's TensorErrorKind (src/tensor/mod.rs:127-155).
 */
#ifndef WRQ_H
#define WRQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define WRQ_ABI_VERSION 1
/* Counts additions that leave every existing signature as it is (new entry points, new override keys);
 * a binding built against minor m runs on any library of the same WRQ_ABI_VERSION with minor >= m. */
#define WRQ_ABI_MINOR 3
#define WRQ_INT8_BLOCK_SIZE 128u /* TensorOp::INT8_BLOCK_SIZE, src/tensor/ops.rs:292 */
#define WRQ_NF4_BLOCK_SIZE 64u   /* TensorOp::NF4_BLOCK_SIZE, src/tensor/ops.rs:291 */

typedef enum wrq_status {
    WRQ_OK = 0,
    WRQ_ERR_SHAPE = 1,       /* TensorErrorKind::Shape(got, want) */
    WRQ_ERR_SIZE = 2,        /* TensorErrorKind::Size */
    WRQ_ERR_TYPE = 3,        /* TensorErrorKind::Type: dtype is neither F16 nor F32 */
    WRQ_ERR_ALIGNMENT = 4,   /* a precondition the reference leaves unchecked: row/column multiples, pointer alignment */
    WRQ_ERR_UNSUPPORTED = 5, /* legal in the reference, not provided here (sliced matrix views) */
    WRQ_ERR_NULL = 6,        /* null pointer argument */
    WRQ_ERR_DEVICE = 7       /* HIP runtime error at launch */
} wrq_status;

/* `Float::DEF` of the reference: "FP16" / "FP32" (src/num.rs:98-108). */
typedef enum wrq_dtype { WRQ_F16 = 0, WRQ_F32 = 1 } wrq_dtype;

/* `Activation`, in declaration order (src/tensor/ops.rs:146-160). */
typedef enum wrq_activation {
    WRQ_ACT_NONE = 0,
    WRQ_ACT_SQUARED_RELU = 1,
    WRQ_ACT_TANH = 2, /* "custom_tanh": 1.0 above 42 */
    WRQ_ACT_STABLE_EXP = 3,
    WRQ_ACT_OPPOSITE_EXP = 4,
    WRQ_ACT_SOFTPLUS = 5,
    WRQ_ACT_SIGMOID = 6,
    WRQ_ACT_SILU = 7
} wrq_activation;

/* `TensorGpu<T, K>`: a device buffer and its shape (src/tensor/mod.rs). */
typedef struct wrq_tensor {
    void *data;
    uint32_t shape[4];
} wrq_tensor;

/* `View`, byte for byte the reference's uniform (src/tensor/mod.rs:26-43):
 * `stride` is the shape of the parent tensor, `offset` the start of the slice. */
typedef struct wrq_view {
    uint32_t shape[4];
    uint32_t stride[4];
    uint32_t offset[4];
} wrq_view;

/* `TensorGpuView<F>`: parent buffer + view + element type. */
typedef struct wrq_tensor_view {
    void *data; /* start of the parent tensor */
    wrq_view view;
    wrq_dtype dtype;
} wrq_tensor_view;

/* `hipStream_t`, spelled as a plain pointer so that bindings need no HIP headers;
 * NULL is the default stream. */
typedef void *wrq_stream;

/* Loads the code object on the current device, checks that it is a gfx950 and resolves the
 * library's per-device scratch array.  Optional, but call it once per device before
 * capturing entry points into a HIP graph: first use otherwise does the same lookups. */
int wrq_init(void);

/*
 * Test and sweep hook; no counterpart in the reference.  The library chooses kernels and tiles by
 * shape.  An override pins one choice so that a test can reach every instantiation: keys are
 * "gemm_ntile", "gemm_mrt", "gemm_kg", "gemm_ksplit", "gemv_rows", "gemv_nt", "gemv_oneshot",
 * "vec_chunk_min_t", "gemm_tail" (0: a chunk grid a little above two workgroups per CU stays one
 * launch), "gemv_waverows" (0: one-token int8 products stay off the wave-owns-rows kernel), "gemv_rows_tokens" (0: nor do runs of 2 .. 4 tokens), "gemm_prio", "gemm_table" / "gemv_table" (0: chunk tiles / one-shot decode tasks by the rules alone, without the measured tables), ...; value < 0 clears the key.  An environment variable WRQ_<KEY> seen when the
 * library first looks (wrq_init, or the first product) presets the same table; nothing on the launch
 * path reads the environment.  Overrides are process-wide and the launch path reads them without a lock,
 * so a product library must not have them changed under it: once the process has launched any kernel of
 * the library the call is refused with WRQ_ERR_UNSUPPORTED, unless WRQ_TEST_HOOKS=1 was in the environment
 * when the library first looked (test and sweep processes set it; they change overrides only between
 * launches of their own).
 */
int wrq_debug_override(const char *key, int value);

/*
 * Measurement hook; no counterpart in the reference, and refused unless WRQ_TEST_HOOKS=1 was in the
 * environment when the library first looked.  While a buffer is set, the one-token int8 products of the
 * 7B shapes (the wave-owns-rows kernel at K = 4096, the K-split kernel at K = 14336) launch builds of
 * the same kernels that also write four wall-clock readings (100 MHz counter) per wave: entry, every
 * load requested, every row accumulated, result stored.  `buffer` is device memory of `bytes` bytes, a
 * multiple of 1 MiB; launch i after the call writes slot i mod (bytes >> 20), record
 * (workgroup * waves_per_workgroup + wave) of 4 x uint64 each.  NULL switches the hook off.  The
 * product kernels carry no stamp code; `python3 bench.py --stamps` prints the timeline of a decode step.
 */
int wrq_debug_stamps(void *buffer, uint64_t bytes);

int wrq_abi_version(void);
int wrq_abi_minor(void); /* WRQ_ABI_MINOR of the loaded library */
const char *wrq_status_string(int status);
const char *wrq_last_error(void);

/*
 * TensorOp::quantize_mat_int8(input, minmax, output)       src/tensor/ops.rs:2393-2486
 *   input  f16 [K, R, B, 1]; output u8 [K, R, B, 1];
 *   minmax f16 [2 * ceil(len / 128), 1, 1, 1], (min, max) per flat 128-block.
 *   len % 128 == 0 is required (the two minmax-shape formulas of the reference,
 *   ops.rs:809 and :2402-2403, agree only then).
 */
int wrq_quantize_mat_int8(wrq_stream stream, const wrq_tensor *input, const wrq_tensor *minmax,
                          const wrq_tensor *output);

/*
 * TensorOp::quantize_mat_nf4(input, quant, absmax, output)  src/tensor/ops.rs:2488-2589
 *   input f16 [K, R, B, 1]; quant f32 [16, 1, 1, 1] (device); output u8 [K/2, R, B, 1];
 *   absmax f16 [ceil(len / 64), 1, 1, 1].  len % 64 == 0 is required.  The f32
 *   temporary and the f32 -> f16 blit of the reference (ops.rs:2505, :2586) are fused.
 */
int wrq_quantize_mat_nf4(wrq_stream stream, const wrq_tensor *input, const wrq_tensor *quant,
                         const wrq_tensor *absmax, const wrq_tensor *output);

/*
 * TensorOp::matmul_vec_int8(matrix, minmax, input, output, act, sparse)
 *                                                          src/tensor/ops.rs:791-886
 *   matrix u8 [K, R, B, 1]; input view [K, T, B, 1]; output view [R, T, B, 1].
 *   Any T: tokens share one pass over the weights (up to 4, nf4: 2, on the decode kernels,
 *   more on the matrix-core kernel).  `sparse` (SPARSE_INPUT) never changes results for finite
 *   weights and is accepted as a hint.
 */
int wrq_matmul_vec_int8(wrq_stream stream, const wrq_tensor *matrix, const wrq_tensor *minmax,
                        const wrq_tensor_view *input, const wrq_tensor_view *output, int act,
                        int sparse);

/* TensorOp::matmul_vec_nf4(matrix, quant, absmax, input, output, act, sparse)
 *                                                          src/tensor/ops.rs:892-991
 *   matrix u8 [K/2, R, B, 1]. */
int wrq_matmul_vec_nf4(wrq_stream stream, const wrq_tensor *matrix, const wrq_tensor *quant,
                       const wrq_tensor *absmax, const wrq_tensor_view *input,
                       const wrq_tensor_view *output, int act, int sparse);

/*
 * Grouped decode products.  No counterpart in the reference's op constructors: it is the
 * HIP side of `TensorOp::List` (src/tensor/ops.rs:280-288), for the step where
 * `Context::encode` (ops.rs:78-144) walks a list of ops.  `count` decode-shaped products
 * that do not depend on each other -- the attention key / value / receptance / gate
 * projections of a layer (src/runtime/v6.rs:806-829), or ffn.key and ffn.receptance
 * (v6.rs:920-938) -- run as if wrq_matmul_vec_* were called on each in order, but share
 * kernel launches: at batch 1 a 4096 x 4096 product is a few microseconds of HBM time and a
 * dispatch of its own costs about as much.  The caller guarantees that no op of a group
 * reads or writes the output of another.  Every op is checked like the single call, before
 * anything is launched.  count <= WRQ_MAX_GROUP.
 */
#define WRQ_MAX_GROUP 8

typedef struct wrq_vec_int8_op {
    const wrq_tensor *matrix;
    const wrq_tensor *minmax;
    const wrq_tensor_view *input;
    const wrq_tensor_view *output;
    int act;
    int sparse;
} wrq_vec_int8_op;

typedef struct wrq_vec_nf4_op {
    const wrq_tensor *matrix;
    const wrq_tensor *quant;
    const wrq_tensor *absmax;
    const wrq_tensor_view *input;
    const wrq_tensor_view *output;
    int act;
    int sparse;
} wrq_vec_nf4_op;

int wrq_matmul_vec_int8_group(wrq_stream stream, const wrq_vec_int8_op *ops, int count);
int wrq_matmul_vec_nf4_group(wrq_stream stream, const wrq_vec_nf4_op *ops, int count);

/*
 * TensorOp::matmul_mat_int8(matrix, minmax, input, output, act)
 *                                                          src/tensor/ops.rs:1072-1140
 *   matrix: view of a u8 tensor, `[K, R, B, 1]`: the whole parent, or its leading batches.  The
 *   reference sizes `minmax` by the view (ops.rs:1088-1090) but indexes it by the position in the
 *   parent and steps rows by the view's width (src/shaders/matmul_mat_int8.wgsl:66-68, :99-103), so
 *   any other slice has no consistent meaning there; it is refused with WRQ_ERR_UNSUPPORTED.  No
 *   call site of the reference slices a matrix (src/tensor/matrix.rs:136-160 pass full views).
 *   R and T multiples of 4 (ops.rs:1068-1069), K a multiple of 32.
 */
int wrq_matmul_mat_int8(wrq_stream stream, const wrq_tensor_view *matrix, const wrq_tensor *minmax,
                        const wrq_tensor_view *input, const wrq_tensor_view *output, int act);

/*
 * wrq_matmul_mat_int8 for callers that cannot allocate or must know that nothing they call does:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart
 * in the reference.  Same operands, checks and results as wrq_matmul_mat_int8 (the same kernels).
 * When the product splits K over workgroups, the partial sums go to a fixed 16 MiB array that the
 * library's code object holds on every GPU it runs on, used by this entry point only; its address on
 * a device is looked up once (wrq_init, else the first call on that device).  A product whose
 * partial sums would not fit at the split the library prefers takes fewer splits (down to none: an
 * unsplit product needs no array), so its result can differ from the plain entry point's in summation
 * order; a split pinned through wrq_debug_override that does not fit is refused with WRQ_ERR_SIZE
 * before anything is launched.  The array keeps nothing between calls and every call
 * writes the part it reads, but calls that overlap in time on one GPU share it: they race.
 */
int wrq_matmul_mat_int8_noalloc(wrq_stream stream, const wrq_tensor_view *matrix, const wrq_tensor *minmax,
                                const wrq_tensor_view *input, const wrq_tensor_view *output, int act);

/* TensorOp::matmul_mat_nf4(matrix, quant, absmax, input, output, act)
 *                                                          src/tensor/ops.rs:1150-1221
 *   matrix: view `[K/2, R, B, 1]` of u8 (whole parent or leading batches, as above); K a multiple of 64. */
int wrq_matmul_mat_nf4(wrq_stream stream, const wrq_tensor_view *matrix, const wrq_tensor *quant,
                       const wrq_tensor *absmax, const wrq_tensor_view *input,
                       const wrq_tensor_view *output, int act);

/*
 * Plain f16 weights: the head and the low-rank matrices of a model, which the reference keeps
 * unquantised behind the same Matrix interface (Matrix::Fp16, src/tensor/matrix.rs:29-44).
 *
 * TensorOp::matmul_vec_fp16(matrix, input, output, act, sparse)   src/tensor/ops.rs:697-784
 *   matrix f16 [K, R, B, 1]; input view [K, T, B, 1]; output view [R, T, B, 1]; K % 4 == 0.
 *   Up to 4 tokens share a pass over the weights on the decode kernel, more on the matrix-core kernel.
 * TensorOp::matmul_mat_fp16(matrix, input, output, act)           src/tensor/ops.rs:999-1061
 *   matrix: view of an f16 tensor (whole parent or leading batches); K, R and T multiples of 4.
 */
int wrq_matmul_vec_fp16(wrq_stream stream, const wrq_tensor *matrix, const wrq_tensor_view *input,
                        const wrq_tensor_view *output, int act, int sparse);
int wrq_matmul_mat_fp16(wrq_stream stream, const wrq_tensor_view *matrix, const wrq_tensor_view *input,
                        const wrq_tensor_view *output, int act);

/*
 * The ops between the matrix products of a layer.  Tensors are in place, rows of 4-element units
 * as in the shaders (row length % 4 == 0); `dtype` is the element type of `x`.
 *
 * TensorOp::softmax(x)                      src/tensor/ops.rs:300-347, src/shaders/softmax.wgsl
 *   x [C, T, B, 1]: every row of C elements becomes exp(x - max) / sum.
 * TensorOp::layer_norm(w, b, x, eps)        src/tensor/ops.rs:407-458, src/shaders/layer_norm.wgsl
 *   x [C, T, B, 1]; w, b f16 [C, 1, 1, 1]: (x - mean) / sqrt(var + eps) * w + b, biased variance.
 * TensorOp::group_norm(w, b, x, eps)        src/tensor/ops.rs:460-509 (the same shader, GROUP_NORM)
 *   x [S, H, A, 1]; w, b f16 [S, H, 1, 1]: the same per row of S elements, head h uses w[.., h].
 */
int wrq_softmax(wrq_stream stream, const wrq_tensor *x, wrq_dtype dtype);
int wrq_layer_norm(wrq_stream stream, const wrq_tensor *w, const wrq_tensor *b, const wrq_tensor *x,
                   wrq_dtype dtype, float eps);
int wrq_group_norm(wrq_stream stream, const wrq_tensor *w, const wrq_tensor *b, const wrq_tensor *x,
                   wrq_dtype dtype, float eps);

/*
 * TensorOp::add_activate / mul_activate(input, output, act_x, act_y, act_out)
 *                                           src/tensor/ops.rs:1227-1391, src/shaders/binary.wgsl
 *   output [C, T, B, 1] = act_out(act_x(input) + act_y(output))   (mul: the product);
 *   input [C, T, B, 1], [C, T, 1, B], [C, 1, B, 1] or [C, 1, 1, 1]: an extent of 1 is broadcast.
 *   TensorOp::add / mul are these with WRQ_ACT_NONE three times.
 */
int wrq_add_activate(wrq_stream stream, const wrq_tensor_view *input, const wrq_tensor_view *output,
                     int act_x, int act_y, int act_out);
int wrq_mul_activate(wrq_stream stream, const wrq_tensor_view *input, const wrq_tensor_view *output,
                     int act_x, int act_y, int act_out);

/*
 * TensorOp::embed(tokens, input, output)    src/tensor/ops.rs:350-405, src/shaders/embed.wgsl
 *   tokens u32 [T, B, 1, 1]; input f16 [C, V, 1, 1]; output [C, T, B, 1] <- the tokens' rows.
 * TensorOp::blit(input, output)             src/tensor/ops.rs:2015-2068, src/shaders/blit.wgsl
 *   copies a view into a view of the same shape, converting the element type.
 * TensorOp::transpose(input, output)        src/tensor/ops.rs:2121-2169, src/shaders/reshape.wgsl:58-77
 *   input [C, T, B, 1] -> output [C, B, T, 1].
 * TensorOp::activate(x, act)                src/tensor/ops.rs:1973-2013, src/shaders/activation.wgsl
 * TensorOp::affine(x, scale, bias)          src/tensor/ops.rs:2352-2391, src/shaders/affine.wgsl
 *   x <- scale * x + bias on a whole tensor [C, T, B, 1].
 * TensorOp::lerp(input, output, factor, reversed)   src/tensor/ops.rs:2284-2350, src/shaders/lerp.wgsl
 *   output <- input (1 - f) + output f (reversed: the two swapped); factor [C, T|1, B|1, 1].
 */
int wrq_embed(wrq_stream stream, const wrq_tensor *tokens, const wrq_tensor *input, const wrq_tensor *output,
              wrq_dtype dtype);
int wrq_blit(wrq_stream stream, const wrq_tensor_view *input, const wrq_tensor_view *output);
int wrq_transpose(wrq_stream stream, const wrq_tensor_view *input, const wrq_tensor_view *output);
int wrq_activate(wrq_stream stream, const wrq_tensor_view *x, int act);
int wrq_affine(wrq_stream stream, const wrq_tensor *x, wrq_dtype dtype, float scale, float bias);
int wrq_lerp(wrq_stream stream, const wrq_tensor_view *input, const wrq_tensor_view *output,
             const wrq_tensor_view *factor, int reversed);

/*
 * The ops that carry state from token to token.  A run is a stack of A tokens of several requests;
 * cursors u32 [A, 1, 1, 1]: for the request of token a, its state slot | first token in the stack << 8
 * | number of its tokens in the stack << 24 (compute_cursor of the shaders).  States are f32 views.
 *
 * TensorOp::token_shift(cursors, time_mix, state, input, output, reversed)
 *                                           src/tensor/ops.rs:1393-1462, src/shaders/token_shift.wgsl
 *   output [C, A, I, 1] <- mix(previous token, this token, time_mix) (reversed: the two swapped);
 *   input [C, A, 1|I, 1] (slice 0 is read), time_mix [C, A, I, 1] or [C, 1, 1, 1], state [C, _, B, 1]
 *   (row 0 of the view is the token before a request's first token of the stack).
 * TensorOp::channel_mix(cursors, state, r, v, x)
 *                                           src/tensor/ops.rs:1860-1915, src/shaders/channel_mix.wgsl
 *   state [C, 1, B, 1] <- x at every request's last token; x [C, A, 1, 1] <- sigmoid(r) * v.
 * TensorOp::time_mix_v4(cursors, time_decay, time_first, state, k, v, r, x)
 *                                           src/tensor/ops.rs:1464-1528, src/shaders/time_mix_v4.wgsl
 *   x, k, v, r [C, A, 1, 1]; time_decay, time_first f32 [C, 1, 1, 1]; state [C, 4, B, 1]: row 0 <- x at
 *   every request's last token, rows 1..3 the numerator, the denominator and their common exponent;
 *   x <- sigmoid(r) * wkv, the exponent-shifted weighted average of v over the request's past.
 * TensorOp::time_mix_v5(cursors, time_decay, time_first, state, k, v, r, x)
 *                                           src/tensor/ops.rs:1530-1599, src/shaders/time_mix_v5.wgsl
 *   as time_mix_v6 below with time_decay f32 [S, H, 1, 1]: one decay per channel for every token.
 * TensorOp::time_mix_v6(cursors, time_decay, time_first, state, k, v, r, x)
 *                                           src/tensor/ops.rs:1601-1677, src/shaders/time_mix_v6.wgsl
 *   x, k, v, r, time_decay(f32) [S, H, A, 1]; time_first f32 [S, H, 1, 1]; state [S H, S + 1, B, 1]:
 *   row 0 <- x at every request's last token, rows 1 + j hold S[j][.];
 *   x[i] <- sum_j r[j] (time_first[j] k[j] v[i] + S[j][i]),  S[j][i] <- time_decay[j] S[j][i] + k[j] v[i].
 *   Head sizes 16, 32, 64, 128 and 256 are built.
 */
int wrq_token_shift(wrq_stream stream, const wrq_tensor *cursors, const wrq_tensor_view *time_mix,
                    const wrq_tensor_view *state, const wrq_tensor *input, wrq_dtype input_dtype,
                    const wrq_tensor *output, wrq_dtype output_dtype, int reversed);
int wrq_channel_mix(wrq_stream stream, const wrq_tensor *cursors, const wrq_tensor_view *state,
                    const wrq_tensor *r, const wrq_tensor *v, const wrq_tensor *x, wrq_dtype dtype);
int wrq_time_mix_v4(wrq_stream stream, const wrq_tensor *cursors, const wrq_tensor *time_decay,
                    const wrq_tensor *time_first, const wrq_tensor_view *state, const wrq_tensor *k,
                    const wrq_tensor *v, const wrq_tensor *r, const wrq_tensor *x, wrq_dtype dtype);
int wrq_time_mix_v5(wrq_stream stream, const wrq_tensor *cursors, const wrq_tensor *time_decay,
                    const wrq_tensor *time_first, const wrq_tensor_view *state, const wrq_tensor *k,
                    const wrq_tensor *v, const wrq_tensor *r, const wrq_tensor *x, wrq_dtype dtype);
int wrq_time_mix_v6(wrq_stream stream, const wrq_tensor *cursors, const wrq_tensor *time_decay,
                    const wrq_tensor *time_first, const wrq_tensor_view *state, const wrq_tensor *k,
                    const wrq_tensor *v, const wrq_tensor *r, const wrq_tensor *x, wrq_dtype dtype);

/*
 * The ops an RWKV-v7 layer adds (src/runtime/v7.rs:757-1006).
 * TensorOp::l2_norm(x, eps)                 src/tensor/ops.rs:642-700, src/shaders/normalize.wgsl:118-152
 *   x [C, T, B, 1] <- x / sqrt(sum of squares over the row + eps).
 * TensorOp::control_k_v7(p, a, k)           src/tensor/ops.rs:1800-1858, src/shaders/control_k_v7.wgsl
 *   k [C, T, B, 1] <- k (1 + (a - 1) p); p f16 [C, 1, 1, 1]; a, k views of f16 or f32 tensors.
 * TensorOp::time_mix_v7(cursors, state, r, w, n, x)
 *                                           src/tensor/ops.rs:1679-1741, src/shaders/time_mix_v7.wgsl:137-212
 *   x, r, w [S, H, A, 1]; n [S, H, A, 4] holds k, v, a, kk; state [S H, S + 1, B, 1] as for time_mix_v6.
 *   With a' = -kk, b = kk a, w' = exp(-exp(-0.5) sigmoid(w)):  sa[i] = sum_j S[j][i] a'[j],
 *   S[j][i] <- S[j][i] w'[j] + k[j] v[i] + sa[i] b[j],  x[i] <- sum_j r[j] S[j][i].  Head sizes 32, 64, 128.
 * TensorOp::time_first_v7(u, r, n, x)       src/tensor/ops.rs:1743-1798, src/shaders/time_mix_v7.wgsl:214-255
 *   x[i] <- x[i] + (sum_j u[j] k[j] r[j]) v[i] per head and token; u f16 [S, H, 1, 1].
 * TensorOp::channel_mix_v7(cursors, state, v, x)
 *                                           src/tensor/ops.rs:1917-1970, src/shaders/channel_mix.wgsl (V7)
 *   state [C, 1, B, 1] <- x at every request's last token; x [C, A, 1, 1] <- v.
 */
int wrq_l2_norm(wrq_stream stream, const wrq_tensor *x, wrq_dtype dtype, float eps);
int wrq_control_k_v7(wrq_stream stream, const wrq_tensor *p, const wrq_tensor_view *a,
                     const wrq_tensor_view *k);
int wrq_time_mix_v7(wrq_stream stream, const wrq_tensor *cursors, const wrq_tensor_view *state,
                    const wrq_tensor *r, const wrq_tensor *w, const wrq_tensor *n, const wrq_tensor *x,
                    wrq_dtype dtype);
int wrq_time_first_v7(wrq_stream stream, const wrq_tensor *u, const wrq_tensor *r, const wrq_tensor *n,
                      const wrq_tensor *x, wrq_dtype dtype);
int wrq_channel_mix_v7(wrq_stream stream, const wrq_tensor *cursors, const wrq_tensor_view *state,
                       const wrq_tensor *v, const wrq_tensor *x, wrq_dtype dtype);

/*
 * The rest of the reference's op set: two row normalisations, and what its loader uses for states and
 * for blending low-rank adapters into matrices at load time (src/runtime/loader.rs:568-686).
 * TensorOp::recenter(x)                     src/tensor/ops.rs:511-564, src/shaders/normalize.wgsl:46-80
 *   x [C, T, B, 1] <- x - mean over the row.
 * TensorOp::rms_norm(w, b, x, eps)          src/tensor/ops.rs:566-640, src/shaders/normalize.wgsl:82-116
 *   x <- x / sqrt(mean of squares over the row + eps) * w + b; w, b f16 [C, 1, 1, 1].
 * TensorOp::broadcast(input, output)        src/tensor/ops.rs:2070-2119, src/shaders/reshape.wgsl:35-56
 *   output [C, T, B, 1] <- input [C, t, b, 1] repeated along tokens and batches (index modulo t, b).
 * TensorOp::blend(factor, input, output)    src/tensor/ops.rs:2171-2224, src/shaders/blend.wgsl
 *   output <- factor[0] input + factor[1] output; factor f32 [4, 1, 1, 1] on the device, equal shapes.
 * TensorOp::blend_lora(factor, xa, xb, output)
 *                                           src/tensor/ops.rs:2226-2282, src/shaders/blend_lora.wgsl
 *   output [M, N, B, 1] <- factor[0] xa^T xb + factor[1] output with xa [K, M, B, 1], xb [K', N, B, 1], f16,
 *   summed in f32 over min(K, K').
 */
int wrq_recenter(wrq_stream stream, const wrq_tensor *x, wrq_dtype dtype);
int wrq_rms_norm(wrq_stream stream, const wrq_tensor *w, const wrq_tensor *b, const wrq_tensor *x,
                 wrq_dtype dtype, float eps);
int wrq_broadcast(wrq_stream stream, const wrq_tensor_view *input, const wrq_tensor_view *output);
int wrq_blend(wrq_stream stream, const wrq_tensor *factor, const wrq_tensor *input, wrq_dtype input_dtype,
              const wrq_tensor *output, wrq_dtype output_dtype);
int wrq_blend_lora(wrq_stream stream, const wrq_tensor *factor, const wrq_tensor_view *xa,
                   const wrq_tensor_view *xb, const wrq_tensor_view *output);

/*
 * Fused forms of consecutive small ops of an RWKV-v6 layer (src/runtime/v6.rs:758-955).  They have no
 * counterpart among the reference's constructors; they are for callers that run a layer without hooks
 * between its ops: at batch 1 every op costs its launch, and these bring a layer from 35 launches to 12.
 * Each computes what the listed ops compute, rounding to f16 where the list stores an f16 buffer.
 * Buffers are contiguous device arrays of `Runtime<f16>` (v6.rs:270-303): C channels x A tokens.
 *
 * wrq_v6_pre: [add(add, x) ->] blit + layer_norm + token_shift x `shifts` (reversed)   v6.rs:759-777, :906-933
 *   x_out (f16, only with `add`; its A * C elements may overlap neither x nor add) <- add + x;  ln_out <- LN(row);  shift_s <- mix(ln, previous, factor_s).
 * wrq_v6_time_mix: transpose + time_mix_w2 + add(time_mix) + token_shift(5)           v6.rs:785-805
 *   lora f16 [lora_size, 5, A]; w2 f16 [lora_size, C, 5]; time_mix f16 [C, 1, 5]; att_sx f16 [C, A, 5].
 * wrq_v6_decay: time_decay_w2 + add(time_decay) + activate(StableExp)                 v6.rs:839-848
 *   lora f16 [lora_size, A]; w2 f16 [lora_size, C]; out f32 [C, A].
 * wrq_v6_wkv_gate: blit + time_mix_v6 + group_norm + blit + mul_activate(Silu)        v6.rs:851-887
 *   k, v, r, time_decay f32 [C, A]; g f16; att_x f16 in (the normalised layer input) and out. Head size 64.
 * wrq_v6_post_ffn: channel_mix + add (+ affine(0.5) when `rescale`)                   v6.rs:942-955
 */
int wrq_v6_pre(wrq_stream stream, uint32_t C, uint32_t A, const void *cursors, const void *x, const void *add,
               void *x_out, const void *ln_w, const void *ln_b, float eps, const wrq_tensor_view *state, int shifts,
               const void *factor0, const void *factor1, void *ln_out, void *shift0, void *shift1);
int wrq_v6_time_mix(wrq_stream stream, uint32_t C, uint32_t A, uint32_t lora_size, const void *cursors,
                    const void *lora, const void *w2, const void *time_mix, const wrq_tensor_view *state,
                    const void *att_x, void *att_sx);
int wrq_v6_decay(wrq_stream stream, uint32_t C, uint32_t A, uint32_t lora_size, const void *lora, const void *w2,
                 const void *time_decay, void *out);
int wrq_v6_wkv_gate(wrq_stream stream, uint32_t S, uint32_t H, uint32_t A, const void *cursors,
                    const void *time_decay, const void *time_first, const wrq_tensor_view *state, const void *k,
                    const void *v, const void *r, const void *g, const void *gn_w, const void *gn_b, float eps,
                    void *att_x);
int wrq_v6_post_ffn(wrq_stream stream, uint32_t C, uint32_t A, const void *cursors, const wrq_tensor_view *state,
                    const void *r, const void *v, const void *ffn_x, const void *x_in, void *x_out, int rescale);

#ifdef __cplusplus
}
#endif
#endif /* WRQ_H */

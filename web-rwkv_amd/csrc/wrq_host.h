// Host-side declarations shared by the translation units of libwrq_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/wrq.h"

namespace wrq {

struct MatmulArgs;

// Records a message for wrq_last_error() of the calling thread and returns `status`.
int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

// Turns a launch failure (hipGetLastError) into WRQ_ERR_DEVICE.
int check_launch(const char *what);

int launch_quant_int8(hipStream_t stream, const void *in, void *minmax, void *out, uint64_t len);
int launch_quant_nf4(hipStream_t stream, const void *in, const void *quant, void *absmax, void *out,
                     uint64_t len);

enum Quant { kInt8 = 0, kNf4 = 1, kFp16 = 2 }; // kFp16: plain f16 weights (matmul_*_fp16), no scales

constexpr int kMaxGroup = 8; // products per grouped decode launch

// Decode-shaped products (few tokens): VALU dequantisation, wave reductions.
int launch_gemv(hipStream_t stream, Quant quant, int in_f16, const MatmulArgs &args);
// The same for `n` independent products of one quantisation, input type and token count,
// in as few launches as their activations fit in LDS together.
int launch_gemv_group(hipStream_t stream, Quant quant, int in_f16, const MatmulArgs *args, int n);
// Decode-shaped products on plain f16 weights (matmul_vec_fp16).
int launch_gemv_fp16(hipStream_t stream, int in_f16, const MatmulArgs &args);
// Where split-K partial sums go: null means the library's shared array, which takes fewer splits when
// a product would not fit; `strict` refuses instead.
struct ScratchPolicy {
    float *base;
    uint64_t floats;
    bool strict;
};
// Chunk-shaped products: f16 MFMA.
int launch_gemm(hipStream_t stream, Quant quant, int in_f16, const MatmulArgs &args);
// The same with the partial sums in the fixed array of the no-allocation entry point.
int launch_gemm_noalloc(hipStream_t stream, Quant quant, int in_f16, const MatmulArgs &args);
// The same for `n` independent products of one quantisation and input type: those with one K
// and token count share a launch (and then rarely need a split of K).
int launch_gemm_group(hipStream_t stream, Quant quant, int in_f16, const MatmulArgs *args, int n, const ScratchPolicy *sp = nullptr);
// Overrides of the kernel and tile choice, for tests and sweeps that must reach one particular
// instantiation.  Every key is unset (-1) unless the environment variable of the same name (WRQ_ +
// upper-case key) was set when the library first looked, or wrq_debug_override() set it since; the
// launch path reads an atomic, never the environment.
enum TuneKey {
    kTuneGemvOneshot, // gemv_oneshot: 0 sends one-token products to the resident kernel
    kTuneGemvRows,    // gemv_rows: rows per task of the decode kernels
    kTuneGemvSl,      // gemv_sl: chunks per lane and row of the resident kernel
    kTuneGemvNt,      // gemv_nt: lanes per task of the decode kernels
    kTuneGemvGrid,    // gemv_grid: workgroups of the resident kernel
    kTuneGemmNtile,   // gemm_ntile, gemm_mrt, gemm_kg, gemm_ksplit: tile of the chunk kernel
    kTuneGemmMrt,
    kTuneGemmKg,
    kTuneGemmKsplit,
    kTuneVecChunkMinT, // vec_chunk_min_t: first token count the decode entry sends to the chunk kernel
    kTuneGemmTail,     // gemm_tail: 0 keeps a grid a little above two workgroups per CU in one launch
    kTuneGemvWaveRows, // gemv_waverows: 0 keeps one-token int8 products off the wave-owns-rows kernel, 2 sends every K it is built for there
    kTuneGemmPrio,     // gemm_prio: 0 leaves the wave priority alone around the matrix work of a chunk step (default: raised)
    kTuneGemvRowsTokens, // gemv_rows_tokens: 0 keeps int8 runs of 2 .. 4 tokens off the wave-owns-rows and K-split kernels
    kTuneGemmTable,    // gemm_table: 0 leaves the measured tile table (gemm_tuned.inc) out and picks chunk tiles by the rules alone
    kTuneGemvTable,    // gemv_table: 0 leaves the measured table of the one-shot decode kernels (gemv_tuned.inc) out
    kTuneCount
};
// The override of `key`, or `fallback` when it is unset.
int tune(TuneKey key, int fallback);
bool tune_is_set(TuneKey key);
// Sets (value >= 0) or clears (value < 0) the override called `name`; unknown names fail.
int tune_set(const char *name, int value);

// Timeline measurement hook of the one-token int8 kernels (gemv.hip): `buf` (device memory, `bytes` long, a multiple of 1 MiB)
// takes the wall-clock records of the following launches, one 1 MiB slot per launch, round-robin; nullptr switches it off.
int stamps_set(void *buf, uint64_t bytes);

// Resolves the split-K scratch array of the current device (also done lazily by the first
// chunk product; calling it from wrq_init keeps the lookup out of stream capture).
int prepare_gemm_scratch();

} // namespace wrq

// Measurement probes of bench.py, built into their own small library (bench_probe.so beside this
// file, by bench.py::build_probe): a streaming read and a plain copy of a known number of bytes.  They
// give the read ceiling of the box that the product kernels are compared with, and the
// reference dispatch against which rocprofv3's FETCH_SIZE / WRITE_SIZE counters are scaled.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Each thread reads U 16-byte words, one block-stride apart, and keeps them live.
template <int U, bool NT>
__global__ __launch_bounds__(256) void read_kernel(const u32x4 *__restrict__ src, uint32_t *sink, uint64_t n16) {
    const uint64_t base = (uint64_t)blockIdx.x * (256 * U) + threadIdx.x;
    u32x4 v[U];
#pragma unroll
    for (int i = 0; i < U; i++) {
        const uint64_t idx = base + (uint64_t)i * 256;
        const u32x4 *p = src + (idx < n16 ? idx : n16 - 1);
        v[i] = NT ? __builtin_nontemporal_load(p) : *p;
    }
    uint32_t acc = 0;
#pragma unroll
    for (int i = 0; i < U; i++) acc |= (v[i].x & v[i].y & v[i].z & v[i].w);
    if (acc == 0xdeadbeefu) *sink = acc; // never true for the benchmark's data; keeps the loads
}

__global__ __launch_bounds__(256) void copy_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, uint64_t n16) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n16) dst[i] = src[i];
}

template <int U, bool NT>
static int launch_read(hipStream_t s, const void *p, uint32_t *sink, uint64_t n16) {
    const uint64_t per_block = 256ull * U;
    hipLaunchKernelGGL((read_kernel<U, NT>), dim3((uint32_t)((n16 + per_block - 1) / per_block)), dim3(256), 0, s,
                       (const u32x4 *)p, sink, n16);
    return (int)hipGetLastError();
}

extern "C" {

// Reads `bytes` (multiple of 16) once.  unroll in {1,2,4,8}; nt != 0 uses streaming loads.
int wrq_probe_read(void *stream, const void *src, void *sink, uint64_t bytes, int unroll, int nt) {
    hipStream_t s = (hipStream_t)stream;
    const uint64_t n16 = bytes / 16;
    if (n16 == 0) return 0;
    switch (unroll * 2 + (nt ? 1 : 0)) {
    case 2: return launch_read<1, false>(s, src, (uint32_t *)sink, n16);
    case 3: return launch_read<1, true>(s, src, (uint32_t *)sink, n16);
    case 4: return launch_read<2, false>(s, src, (uint32_t *)sink, n16);
    case 5: return launch_read<2, true>(s, src, (uint32_t *)sink, n16);
    case 8: return launch_read<4, false>(s, src, (uint32_t *)sink, n16);
    case 9: return launch_read<4, true>(s, src, (uint32_t *)sink, n16);
    case 16: return launch_read<8, false>(s, src, (uint32_t *)sink, n16);
    case 17: return launch_read<8, true>(s, src, (uint32_t *)sink, n16);
    default: return -1;
    }
}

// Copies `bytes` (multiple of 16): reads `bytes`, writes `bytes`.
int wrq_probe_copy(void *stream, void *dst, const void *src, uint64_t bytes) {
    const uint64_t n16 = bytes / 16;
    if (n16 == 0) return 0;
    hipLaunchKernelGGL(copy_kernel, dim3((uint32_t)((n16 + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const u32x4 *)src, (u32x4 *)dst, n16);
    return (int)hipGetLastError();
}
}

// Measurement probes: what this GPU's memory and matrix units deliver to the simplest possible
// kernels, as the ceilings that the engine's kernels are priced against beside the published peaks.
// Nothing on the product path calls them (bench.py does).
//
//  fx_probe_read : every byte of a buffer once, 16 bytes per lane and load, summed so that the loads stay;
//                  `stream` != 0: the loads carry the non-temporal hint, as the engine's loads of weights, keys
//                  and values do
//  fx_probe_copy : buffer to buffer, 16 bytes per lane
//  fx_probe_mfma : a loop of independent bf16 MFMA products on registers, no memory traffic
//  fx_probe_mark : an empty kernel whose grid size is a label: in a profiler's kernel trace it says which part
//                  of the model the kernels after it (on the same stream) belong to
#include "common.h"

FX_DEFINE_LAST_ERROR()

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 probe_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float probe_f32x4;

template <bool STREAM>
__device__ __forceinline__ uint4 probe_load(const uint4* p) {
    if constexpr (STREAM) return load_lines16(p);
    else return *p;
}
template <bool STREAM>
__global__ __launch_bounds__(256) void probe_read_kernel(const uint4* __restrict__ src, size_t n16, unsigned* __restrict__ out) {
    const size_t groups = n16 / 1024;                 // whole groups of 1024 x 16 bytes: four loads in flight per lane
    unsigned acc = 0;
    for (size_t g = blockIdx.x; g < groups; g += gridDim.x) {
        const uint4* p = src + g * 1024 + threadIdx.x;
        const uint4 a = probe_load<STREAM>(p), b = probe_load<STREAM>(p + 256), c = probe_load<STREAM>(p + 512), d = probe_load<STREAM>(p + 768);
        acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
    }
    if (blockIdx.x == 0)                              // what is left of the buffer
        for (size_t i = groups * 1024 + threadIdx.x; i < n16; i += 256) {
            const uint4 a = src[i];
            acc ^= a.x ^ a.y ^ a.z ^ a.w;
        }
    if (acc == 0x9e3779b9u) out[0] = acc;             // practically never: the sum only keeps the loads alive
}

__global__ __launch_bounds__(256) void probe_copy_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t n16) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

__global__ __launch_bounds__(256) void probe_mfma_kernel(int iters, float* __restrict__ out) {
    probe_bf16x8 a, b;
    for (int i = 0; i < 8; ++i) {
        a[i] = (__bf16)(float)((threadIdx.x + i) & 3);
        b[i] = (__bf16)(float)((threadIdx.x * 3 + i) & 1);
    }
    probe_f32x4 acc[8];
    for (int j = 0; j < 8; ++j) acc[j] = (probe_f32x4){0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[j], 0, 0, 0);
    }
    float s = 0.f;
    for (int j = 0; j < 8; ++j) s += acc[j][0] + acc[j][1] + acc[j][2] + acc[j][3];
    if (s == -1.f) out[0] = s;                        // never: the products are non-negative
}

__global__ void probe_mark_kernel() {}

FX_API int fx_probe_mark(void* stream, int label) {
    FX_REQUIRE(label >= 0 && label < 65535, "probe_mark: label %d", label);
    probe_mark_kernel<<<label + 1, 64, 0, (hipStream_t)stream>>>();
    FX_CHECK_LAUNCH("probe_mark");
    return 0;
}

FX_API int fx_probe_read(void* stream, const void* src, long n_bytes, void* out, int non_temporal) {
    FX_REQUIRE(n_bytes > 0 && n_bytes % 16 == 0 && ((uintptr_t)src % 16) == 0, "probe_read: a 16-byte aligned buffer of whole 16 bytes");
    const size_t n16 = (size_t)n_bytes / 16;
    const unsigned blocks = (unsigned)((n16 + 1023) / 1024 < 256 * 16 ? (n16 + 1023) / 1024 : 256 * 16);
    if (non_temporal) probe_read_kernel<true><<<blocks, 256, 0, (hipStream_t)stream>>>((const uint4*)src, n16, (unsigned*)out);
    else probe_read_kernel<false><<<blocks, 256, 0, (hipStream_t)stream>>>((const uint4*)src, n16, (unsigned*)out);
    FX_CHECK_LAUNCH("probe_read");
    return 0;
}

FX_API int fx_probe_copy(void* stream, void* dst, const void* src, long n_bytes) {
    FX_REQUIRE(n_bytes > 0 && n_bytes % 16 == 0 && (((uintptr_t)src | (uintptr_t)dst) % 16) == 0, "probe_copy: 16-byte aligned buffers of whole 16 bytes");
    const size_t n16 = (size_t)n_bytes / 16;
    const unsigned blocks = (unsigned)((n16 + 255) / 256 < 256 * 32 ? (n16 + 255) / 256 : 256 * 32);
    probe_copy_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>((uint4*)dst, (const uint4*)src, n16);
    FX_CHECK_LAUNCH("probe_copy");
    return 0;
}

// flops of one call: blocks * 4 waves * iters * 8 products * 2 * 16 * 16 * 32
FX_API int fx_probe_mfma(void* stream, int blocks, int iters, void* out) {
    FX_REQUIRE(blocks > 0 && iters > 0, "probe_mfma: blocks and iterations must be positive");
    probe_mfma_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>(iters, (float*)out);
    FX_CHECK_LAUNCH("probe_mfma");
    return 0;
}

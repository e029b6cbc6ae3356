// Shared by every kernel library of the engine (gfx950 only).
//
// Each library is a plain shared object with `extern "C"` entry points that take
// raw device pointers and a HIP stream; Python calls them through ctypes.  An
// entry point checks its sizes on the host before it launches anything and
// returns 0, or a non-zero code after storing a message for fx_last_error().
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <math.h>
#include <string.h>

#define FX_API extern "C" __attribute__((visibility("default")))

// element types as the Python side numbers them
enum FxDtype { FX_F32 = 0, FX_BF16 = 1 };

static thread_local char fx_err_buf[512];

static int fx_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(fx_err_buf, sizeof(fx_err_buf), fmt, ap);
    va_end(ap);
    return 1;
}

#define FX_DEFINE_LAST_ERROR() \
    FX_API const char* fx_last_error() { return fx_err_buf; }

#define FX_REQUIRE(cond, ...)                      \
    do {                                           \
        if (!(cond)) return fx_fail(__VA_ARGS__);  \
    } while (0)

#define FX_CHECK_LAUNCH(name)                                                     \
    do {                                                                          \
        hipError_t e_ = hipGetLastError();                                        \
        if (e_ != hipSuccess) return fx_fail("%s: %s", name, hipGetErrorString(e_)); \
    } while (0)

// ---- bfloat16 as raw bits --------------------------------------------------
struct bf16 {
    uint16_t bits;
};

__device__ __forceinline__ float bf16_to_float(bf16 v) { return __uint_as_float(((uint32_t)v.bits) << 16); }

// round to nearest even; NaN stays NaN (the hardware conversion of gfx950)
__device__ __forceinline__ bf16 float_to_bf16(float f) {
    const __bf16 b = (__bf16)f;
    bf16 r;
    r.bits = __builtin_bit_cast(uint16_t, b);
    return r;
}

// two floats to two packed bfloat16 (first in the low half)
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
    bf16x2_t v;
    v[0] = (__bf16)a;
    v[1] = (__bf16)b;
    return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16 v) { return bf16_to_float(v); }
__device__ __forceinline__ void from_float(float* p, float v) { *p = v; }
__device__ __forceinline__ void from_float(bf16* p, float v) { *p = float_to_bf16(v); }

// load one element of a tensor whose element type is only known at run time
// Without a branch: two 16-bit loads (the halves of a float, or the same bfloat16 twice).  A branch on the
// type around a load makes the compiler wait for that load before the paths join, so a thread that
// loads several such values would wait for each in turn.  In two steps, so that a caller can ask for
// its other loads between the fetch and the first use.
struct RawElement {
    unsigned lo, hi, shift, keep_hi;
};
__device__ __forceinline__ RawElement fetch_element(const void* p, int dtype, size_t i) {
    const unsigned short* q = (const unsigned short*)p;
    const bool f32 = dtype == FX_F32;
    const size_t e = f32 ? 2 * i : i;
    // float: lo | hi << 16; bfloat16: lo << 16.  The three constants pass through an empty statement so that
    // the compiler cannot tell the cases apart and bring the branch back.
    int second = f32 ? 1 : 0;
    RawElement r;
    r.shift = f32 ? 0u : 16u;
    r.keep_hi = f32 ? 0xffff0000u : 0u;
    asm volatile("" : "+v"(second), "+v"(r.shift), "+v"(r.keep_hi));
    r.lo = q[e];
    r.hi = q[e + second];
    return r;
}
__device__ __forceinline__ float element_as_float(const RawElement& r) {
    return __uint_as_float((r.lo << r.shift) | ((r.hi << 16) & r.keep_hi));
}
__device__ __forceinline__ float load_as_float(const void* p, int dtype, size_t i) {
    return element_as_float(fetch_element(p, dtype, i));
}

// N elements first, first + STRIDE, ... (zero from `limit` on) of such a tensor.  The branch on the type
// is taken once around all N loads, so that they are on their way together: taken per element it makes
// every load wait for the one before.
template <typename WT, int N, int STRIDE>
__device__ __forceinline__ void load_strided_typed(const WT* p, int first, int limit, float (&out)[N]) {
    WT raw[N];
#pragma unroll
    for (int i = 0; i < N; ++i) raw[i] = p[min(first + i * STRIDE, limit - 1)];
#pragma unroll
    for (int i = 0; i < N; ++i) out[i] = first + i * STRIDE < limit ? to_float(raw[i]) : 0.f;
}
template <int N, int STRIDE>
__device__ __forceinline__ void load_strided_as_float(const void* p, int dtype, int first, int limit, float (&out)[N]) {
    if (dtype == FX_F32) load_strided_typed<float, N, STRIDE>((const float*)p, first, limit, out);
    else load_strided_typed<bf16, N, STRIDE>((const bf16*)p, first, limit, out);
}

// The rotation of one pair by an angle, (a, b) -> (a cos - b sin, a sin + b cos), with its roundings spelled
// out (one product rounded, then a fused multiply-add), so that every kernel that rotates gets the same bits
// whatever the compiler would have made of the plain expression.
__device__ __forceinline__ void rotate_pair(float a, float b, float cs, float sn, float& y0, float& y1) {
    y0 = fmaf(a, cs, -(b * sn));
    y1 = fmaf(a, sn, b * cs);
}

// ---- wave (64 lanes) and block reductions in a fixed order ------------------
// Sum and maximum over the 64 lanes of a wave, in every lane: a butterfly over the lanes 32, 16, 8, 4, 2 and 1
// away, in that order (the order fixes the sum's bits).  The exchanges stay in the vector unit: the halves of the
// wave and the rows of 16 lanes pairwise by the lane-swapping moves of gfx950, then rotations inside a row by DPP
// (after the step over 8 lanes the lanes i and i ^ 8 hold the same value, so the lane four further round the row
// holds what lane i ^ 4 holds, and so on down): the same values in the same order as exchanges through the LDS
// crossbar (__shfl_xor) give, without waiting for it six times.
__device__ __forceinline__ float wave_partner_32(float v, float& other) {
    const unsigned u = __float_as_uint(v);
    const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    other = __uint_as_float(a[1]);
    return __uint_as_float(a[0]);
}
__device__ __forceinline__ float wave_partner_16(float v, float& other) {
    const unsigned u = __float_as_uint(v);
    const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    other = __uint_as_float(a[1]);
    return __uint_as_float(a[0]);
}
template <int CTRL>
__device__ __forceinline__ float row_rotated(float v) {
    return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float wave_sum(float v) {
    float o;
    v = wave_partner_32(v, o) + o;
    v = wave_partner_16(v, o) + o;
    v += row_rotated<0x128>(v);      // row_ror:8
    v += row_rotated<0x124>(v);      // row_ror:4
    v += row_rotated<0x122>(v);      // row_ror:2
    v += row_rotated<0x121>(v);      // row_ror:1
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
    float o;
    v = fmaxf(wave_partner_32(v, o), o);
    v = fmaxf(wave_partner_16(v, o), o);
    v = fmaxf(v, row_rotated<0x128>(v));
    v = fmaxf(v, row_rotated<0x124>(v));
    v = fmaxf(v, row_rotated<0x122>(v));
    v = fmaxf(v, row_rotated<0x121>(v));
    return v;
}

// sum over a block of NW waves; every thread gets the result.  `red` has NW floats.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NW; ++i) s += red[i];
    return s;
}

// A block barrier that waits for this wave's LDS traffic only.  __syncthreads() also waits for
// every global load in flight, which would stall a pipeline that fetches tiles ahead of their
// use; the compiler still waits for a load where its registers are consumed.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ---- results that blocks of one launch hand to each other ----------------------
// The eight XCDs have an L2 each, so a plain store of one block need not be seen by a block on
// another XCD before the kernel ends.  Values that the launch's last block gathers are therefore
// written and read at device scope (they go past the caches that are not shared), which costs
// nothing like a fence: a fence would write a whole L2 back.
__device__ __forceinline__ void store_shared(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_shared(int* p, int v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_shared(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ int load_shared(const int* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// True, in every thread, in the block that is the last of `total` blocks to get here.  What the
// other blocks wrote with store_shared() before they came can be read there with load_shared().
// The last block leaves the counter (one zeroed word in device memory) at zero again.  Every
// thread of a block must call it.
__device__ __forceinline__ bool last_block_arrives(unsigned* counter, unsigned total) {
    __shared__ int fx_last_flag;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this thread's stores have arrived
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned old = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        fx_last_flag = (old == total - 1u);
        if (old == total - 1u) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    return fx_last_flag != 0;
}

// Streams that are read once (weights, the keys and values of a decode step) in whole 128-byte lines.  An MFMA
// operand wants lane (li, g) of a wave to hold 16 bytes of row li, so a plain 16-byte load per lane takes 64 bytes
// of each of 16 rows: half of every line, the other half with the next load.  Instead one load takes whole lines
// of eight rows (lanes li < 8 the low half of row li, lanes li >= 8 the high half of row li - 8), the next load
// rows 8 .. 15 the same way, and before the products the halves of each row of 16 lanes change places
// (`swap_halves`, one DPP move a register).  Loads of whole lines can carry the non-temporal hint (the data needs
// no place in the caches), which memory answers a tenth to a fifth faster; on half lines the hint costs time.
typedef unsigned int fx_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_lines16(const void* p) {
    const fx_u32x4 v = __builtin_nontemporal_load((const fx_u32x4*)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}
// keep: this lane's value where its bank (four lanes) is not in BANKS, else other's value from the lane eight
// further round its row of 16 lanes.  With (first, second) the two loads described above:
// low half of row li = swap_halves<0xC>(first, second), high half = swap_halves<0x3>(second, first).
template <int BANKS>
__device__ __forceinline__ uint4 swap_halves(uint4 keep, uint4 other) {
    uint4 r;
    r.x = __builtin_amdgcn_update_dpp(keep.x, other.x, 0x128, 0xF, BANKS, false);      // 0x128: row_ror:8
    r.y = __builtin_amdgcn_update_dpp(keep.y, other.y, 0x128, 0xF, BANKS, false);
    r.z = __builtin_amdgcn_update_dpp(keep.z, other.z, 0x128, 0xF, BANKS, false);
    r.w = __builtin_amdgcn_update_dpp(keep.w, other.w, 0x128, 0xF, BANKS, false);
    return r;
}

// v of this lane and of all lanes below it, added up: inside each row of 16 lanes by four shifted adds, then
// row 0's total onto row 1 and row 2's onto row 3, then the lower half's total onto the upper half (DPP moves of
// gfx9, no LDS; a lane with no source lane adds 0)
__device__ __forceinline__ int wave_inclusive_sum(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xF, 0xF, false);      // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xF, 0xF, false);      // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xF, 0xF, false);      // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xF, 0xF, false);      // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false);      // row_bcast:15 into rows 1 and 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false);      // row_bcast:31 into rows 2 and 3
    return v;
}

static inline int ceil_div(long a, long b) { return (int)((a + b - 1) / b); }

// Compute units of the current device, asked for once per device.  Dispatch decisions that weigh a launch's
// blocks against the CUs (tile shapes, one or two groups of waves) take the number from here; the measurements
// behind their ratios were made on 256.
static inline int fx_compute_units() {
    static int cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED);
    if (n <= 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        __atomic_store_n(&cached[dev], n, __ATOMIC_RELAXED);
    }
    return n;
}

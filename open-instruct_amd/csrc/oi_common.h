// Shared device helpers for the gfx950 policy-loss kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "oi_kernels.h"

#define OI_WAVE 64

#define OI_LOG2E 1.4426950408889634f
#define OI_LN2 0.6931471805599453f
// Finite stand-in for -inf as the starting value of a running maximum: keeps (m_old - m_new)
// finite so that exp2 of it is 1 and not NaN when nothing has been seen yet.
#define OI_NEG_BIG (-3.0e38f)

#define OI_RETURN_IF(cond, code) \
    do {                         \
        if (cond) return (code); \
    } while (0)

static inline int oi_launch_status() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? OI_OK : (int)e;
}

static inline bool oi_aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// Number of CUs of the current device.  Looked up once per device and source file; the value never
// changes afterwards, so a relaxed atomic is all the concurrency control the cache needs.
static inline int oi_cu_count() {
    static std::atomic<int> cus_of_device[64];  // 0 = not looked up yet
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    int cus = cus_of_device[dev].load(std::memory_order_relaxed);
    if (cus == 0) {
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        cus_of_device[dev].store(cus, std::memory_order_relaxed);
    }
    return cus;
}

typedef uint32_t oi_u32x4 __attribute__((ext_vector_type(4)));
typedef float oi_f32x4 __attribute__((ext_vector_type(4)));

// ---- bf16 / f16 <-> f32 ------------------------------------------------------------------
__device__ __forceinline__ float oi_bf16lo_to_f32(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float oi_bf16hi_to_f32(uint32_t packed) { return __uint_as_float(packed & 0xffff0000u); }

// f32 -> bf16, round to nearest even: one v_cvt_pk_bf16_f32 per pair on gfx950
typedef __bf16 oi_bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t oi_pack_bf16x2(float lo, float hi) {
    const oi_bf16x2 v = {(__bf16)lo, (__bf16)hi};
    uint32_t u;
    __builtin_memcpy(&u, &v, 4);
    return u;
}
__device__ __forceinline__ uint32_t oi_f32_to_bf16_bits(float f) { return oi_pack_bf16x2(f, 0.f) & 0xffffu; }

__device__ __forceinline__ float oi_f16bits_to_f32(uint16_t h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
}
__device__ __forceinline__ uint16_t oi_f32_to_f16bits(float f) {
    _Float16 v = (_Float16)f;
    uint16_t h;
    __builtin_memcpy(&h, &v, 2);
    return h;
}

// ---- wavefront (64 lanes) reductions -------------------------------------------------------
__device__ __forceinline__ float oi_wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, OI_WAVE);
    return v;
}
__device__ __forceinline__ double oi_wave_sum(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, OI_WAVE);
    return v;
}
__device__ __forceinline__ float oi_wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, OI_WAVE));
    return v;
}

// Block-wide sum for blockDim.x a multiple of 64, up to 1024 threads; `scratch` holds >= 16
// floats.  Every thread gets the total; summation order is fixed (deterministic).
__device__ __forceinline__ float oi_block_sum(float v, float* scratch) {
    v = oi_wave_sum(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int w = 0; w < nw; ++w) t += scratch[w];
    return t;
}

// ---- per-sequence ranges of a batch of token positions ---------------------------------------------
// cu != null: one packed row of `total` positions with sequence boundaries cu[0 .. n_seqs]
// (open_instruct/padding_free_collator.py:202-229); cu == null: n_seqs padded rows of `total`
// positions each (open_instruct/dpo_utils.py:689-712).
// Segment [start, end) of scored positions for sequence s; position t is scored against labels[t+1].
__device__ __forceinline__ void oi_seq_range(const int32_t* cu, int64_t s, int64_t n_seqs, int64_t total, int64_t* start,
                                          int64_t* end) {
    if (cu) {
        // boundaries shifted left by one, leading 0 kept, everything past the last start stays in the
        // last segment; the packed row has total-1 scored positions
        int64_t a = s == 0 ? 0 : (int64_t)cu[s] - 1;
        int64_t b = s == n_seqs - 1 ? total - 1 : (int64_t)cu[s + 1] - 1;
        a = a < 0 ? 0 : (a > total - 1 ? total - 1 : a);
        b = b < a ? a : (b > total - 1 ? total - 1 : b);
        *start = a;
        *end = b;
    } else {
        *start = s * total;
        *end = s * total + total - 1;
    }
}

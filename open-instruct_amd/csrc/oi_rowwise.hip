// Row-wise log-softmax gather / entropy over materialised logits, forward and backward.
//
// One workgroup streams one row of `vocab` logits exactly once with 16-byte non-temporal loads.
// Every lane keeps an online (max, sum-exp, sum exp*z) triple in the log2 domain, rescaled once
// per 16-byte vector rather than per element; lanes are merged by wave shuffles and the four
// waves through LDS.  The kernel is HBM-bound: 2 (bf16) or 4 (fp32) bytes per logit, nothing
// else of size [rows, vocab] is read or written by the forward.
#include "oi_common.h"
#include "oi_grpo_math.h"

#include <type_traits>

namespace {

struct F32Row {
    typedef float elem_t;
    static constexpr int VEC = 4;
    typedef oi_f32x4 raw_t;
    static __device__ __forceinline__ raw_t load_raw(const elem_t* p) {
        return __builtin_nontemporal_load(reinterpret_cast<const oi_f32x4*>(p));
    }
    static __device__ __forceinline__ raw_t load_raw_cached(const elem_t* p) { return *reinterpret_cast<const oi_f32x4*>(p); }
    static __device__ __forceinline__ void unpack(raw_t v, float (&z)[VEC]) { z[0] = v.x; z[1] = v.y; z[2] = v.z; z[3] = v.w; }
    static __device__ __forceinline__ void load_vec(const elem_t* p, float (&z)[VEC]) { unpack(load_raw(p), z); }
    static __device__ __forceinline__ float load_one(const elem_t* p) { return *p; }
    static __device__ __forceinline__ void store_vec(elem_t* p, const float (&z)[VEC]) {
        oi_f32x4 v = {z[0], z[1], z[2], z[3]};
        __builtin_nontemporal_store(v, reinterpret_cast<oi_f32x4*>(p));
    }
    static __device__ __forceinline__ void store_one(elem_t* p, float z) { *p = z; }
};

struct BF16Row {
    typedef uint16_t elem_t;
    static constexpr int VEC = 8;
    typedef oi_u32x4 raw_t;
    static __device__ __forceinline__ raw_t load_raw(const elem_t* p) {
        return __builtin_nontemporal_load(reinterpret_cast<const oi_u32x4*>(p));
    }
    static __device__ __forceinline__ raw_t load_raw_cached(const elem_t* p) { return *reinterpret_cast<const oi_u32x4*>(p); }
    static __device__ __forceinline__ void unpack(raw_t v, float (&z)[VEC]) {
        z[0] = oi_bf16lo_to_f32(v.x); z[1] = oi_bf16hi_to_f32(v.x);
        z[2] = oi_bf16lo_to_f32(v.y); z[3] = oi_bf16hi_to_f32(v.y);
        z[4] = oi_bf16lo_to_f32(v.z); z[5] = oi_bf16hi_to_f32(v.z);
        z[6] = oi_bf16lo_to_f32(v.w); z[7] = oi_bf16hi_to_f32(v.w);
    }
    static __device__ __forceinline__ void load_vec(const elem_t* p, float (&z)[VEC]) { unpack(load_raw(p), z); }
    static __device__ __forceinline__ float load_one(const elem_t* p) { return __uint_as_float((uint32_t)(*p) << 16); }
    static __device__ __forceinline__ void store_vec(elem_t* p, const float (&z)[VEC]) {
        oi_u32x4 v = {oi_pack_bf16x2(z[0], z[1]), oi_pack_bf16x2(z[2], z[3]), oi_pack_bf16x2(z[4], z[5]),
                      oi_pack_bf16x2(z[6], z[7])};
        __builtin_nontemporal_store(v, reinterpret_cast<oi_u32x4*>(p));
    }
    static __device__ __forceinline__ void store_one(elem_t* p, float z) { *p = (uint16_t)oi_f32_to_bf16_bits(z); }
};

struct F16Row {
    typedef uint16_t elem_t;
    static constexpr int VEC = 8;
    typedef oi_u32x4 raw_t;
    static __device__ __forceinline__ raw_t load_raw(const elem_t* p) {
        return __builtin_nontemporal_load(reinterpret_cast<const oi_u32x4*>(p));
    }
    static __device__ __forceinline__ raw_t load_raw_cached(const elem_t* p) { return *reinterpret_cast<const oi_u32x4*>(p); }
    static __device__ __forceinline__ void unpack(raw_t v, float (&z)[VEC]) {
        uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            z[2 * i] = oi_f16bits_to_f32((uint16_t)(w[i] & 0xffffu));
            z[2 * i + 1] = oi_f16bits_to_f32((uint16_t)(w[i] >> 16));
        }
    }
    static __device__ __forceinline__ void load_vec(const elem_t* p, float (&z)[VEC]) { unpack(load_raw(p), z); }
    static __device__ __forceinline__ float load_one(const elem_t* p) { return oi_f16bits_to_f32(*p); }
    static __device__ __forceinline__ void store_vec(elem_t* p, const float (&z)[VEC]) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            w[i] = (uint32_t)oi_f32_to_f16bits(z[2 * i]) | ((uint32_t)oi_f32_to_f16bits(z[2 * i + 1]) << 16);
        oi_u32x4 v = {w[0], w[1], w[2], w[3]};
        __builtin_nontemporal_store(v, reinterpret_cast<oi_u32x4*>(p));
    }
    static __device__ __forceinline__ void store_one(elem_t* p, float z) { *p = oi_f32_to_f16bits(z); }
};

// Online softmax statistics of the scaled logits x = z * c (c = log2(e) / T), log2 domain:
//   m = running max of x,  s = sum 2^(x - m),  t = sum 2^(x - m) * (x - m)   (t only when ENT).
// Keeping t relative to the running maximum makes the entropy ln2 * (log2 s - t / s) a difference
// of two small numbers instead of lse - sum p*z, two numbers of the size of the logits.
struct RowStat {
    float m, s, t;
};

template <int VEC, bool ENT>
__device__ __forceinline__ void stat_update(RowStat& st, const float (&z)[VEC], float c) {
    float x[VEC];
    float vmax = OI_NEG_BIG;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        x[j] = z[j] * c;
        vmax = fmaxf(vmax, x[j]);
    }
    const float mn = fmaxf(st.m, vmax);
    const float shift = st.m - mn;  // <= 0
    const float alpha = __builtin_amdgcn_exp2f(shift);
    float s = st.s * alpha;
    float t = ENT ? alpha * fmaf(shift, st.s, st.t) : 0.f;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        const float d = x[j] - mn;
        const float e = __builtin_amdgcn_exp2f(d);
        s += e;
        if (ENT) t = fmaf(e, d, t);
    }
    st.m = mn;
    st.s = s;
    st.t = t;
}

// The same update with one multiply less per logit: the maximum is taken over the unscaled logits
// (c > 0) and every exponent is a single fma.  The running maximum is then the rounded product
// max(z) * c while the exponents are rounded once, so the largest term is 2^(a few ulp) instead of
// exactly 1: far below the accuracy of the sum.
template <int VEC, bool ENT>
__device__ __forceinline__ void stat_update_fma(RowStat& st, const float (&z)[VEC], float c) {
    float zmax = z[0];
#pragma unroll
    for (int j = 1; j < VEC; ++j) zmax = fmaxf(zmax, z[j]);
    const float mn = fmaxf(st.m, zmax * c);
    const float shift = st.m - mn;  // <= 0
    const float alpha = __builtin_amdgcn_exp2f(shift);
    float s = st.s * alpha;
    float t = ENT ? alpha * fmaf(shift, st.s, st.t) : 0.f;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
        const float d = fmaf(z[j], c, -mn);
        const float e = __builtin_amdgcn_exp2f(d);
        s += e;
        if (ENT) t = fmaf(e, d, t);
    }
    st.m = mn;
    st.s = s;
    st.t = t;
}

template <bool ENT>
__device__ __forceinline__ void stat_update1(RowStat& st, float z, float c) {
    const float zz[1] = {z};
    stat_update<1, ENT>(st, zz, c);
}

__device__ __forceinline__ RowStat stat_merge(const RowStat& a, const RowStat& b) {
    RowStat r;
    r.m = fmaxf(a.m, b.m);
    const float da = a.m - r.m, db = b.m - r.m;
    const float fa = __builtin_amdgcn_exp2f(da), fb = __builtin_amdgcn_exp2f(db);
    r.s = a.s * fa + b.s * fb;
    r.t = fa * fmaf(da, a.s, a.t) + fb * fmaf(db, b.s, b.t);
    return r;
}

__device__ __forceinline__ int64_t row_offset(int64_t row, int64_t n_inner, int64_t stride_outer, int64_t stride_inner) {
    const int64_t o = row / n_inner, i = row - o * n_inner;
    return o * stride_outer + i * stride_inner;
}

constexpr int FWD_UNROLL = 4;

template <typename R, bool VECTORISED, bool ENT>
__global__ void __launch_bounds__(256) lsg_entropy_fwd_kernel(const typename R::elem_t* __restrict__ logits,
                                                              int64_t n_inner, int64_t stride_outer,
                                                              int64_t stride_inner, int64_t vocab,
                                                              const int64_t* __restrict__ index, float inv_t,
                                                              float* __restrict__ logprob, float* __restrict__ entropy,
                                                              float* __restrict__ lse_out) {
    constexpr int VEC = R::VEC;
    const int64_t row = blockIdx.x;
    const typename R::elem_t* p = logits + row_offset(row, n_inner, stride_outer, stride_inner);
    const float c = inv_t * OI_LOG2E;
    const int tid = threadIdx.x, nthr = blockDim.x;

    RowStat st = {OI_NEG_BIG, 0.f, 0.f};
    int64_t done = 0;
    if (VECTORISED) {
        const int64_t nvec = vocab / VEC;
        int64_t i = tid;
        // full groups of FWD_UNROLL vectors per lane: all loads are issued before the first use
        for (; i + (int64_t)(FWD_UNROLL - 1) * nthr < nvec; i += (int64_t)FWD_UNROLL * nthr) {
            float z[FWD_UNROLL][VEC];
#pragma unroll
            for (int u = 0; u < FWD_UNROLL; ++u) R::load_vec(p + (i + (int64_t)u * nthr) * VEC, z[u]);
#pragma unroll
            for (int u = 0; u < FWD_UNROLL; ++u) stat_update<VEC, ENT>(st, z[u], c);
        }
        for (; i < nvec; i += nthr) {
            float z[VEC];
            R::load_vec(p + i * VEC, z);
            stat_update<VEC, ENT>(st, z, c);
        }
        done = nvec * VEC;
    }
    for (int64_t j = done + tid; j < vocab; j += nthr) stat_update1<ENT>(st, R::load_one(p + j), c);

    // lanes -> wave
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        RowStat o;
        o.m = __shfl_xor(st.m, off, OI_WAVE);
        o.s = __shfl_xor(st.s, off, OI_WAVE);
        o.t = ENT ? __shfl_xor(st.t, off, OI_WAVE) : 0.f;
        st = stat_merge(st, o);
    }
    // waves -> block
    __shared__ float sm[3][4];
    const int wave = tid >> 6, lane = tid & 63, nw = nthr >> 6;
    if (lane == 0) {
        sm[0][wave] = st.m;
        sm[1][wave] = st.s;
        sm[2][wave] = st.t;
    }
    __syncthreads();
    if (tid == 0) {
        RowStat tot = {sm[0][0], sm[1][0], sm[2][0]};
        for (int w = 1; w < nw; ++w) {
            RowStat o = {sm[0][w], sm[1][w], sm[2][w]};
            tot = stat_merge(tot, o);
        }
        // once per row: assemble in fp64 so that the result carries only the rounding of m, s and t
        const double ln2 = 0.69314718055994530942;
        const double log2s = log2((double)tot.s);
        const double lse = ((double)tot.m + log2s) * ln2;
        int64_t y = index[row];
        y = y < 0 ? 0 : (y >= vocab ? vocab - 1 : y);
        const float zy = R::load_one(p + y);
        logprob[row] = (float)((double)zy * (double)inv_t - lse);
        if (ENT) entropy[row] = (float)((log2s - (double)tot.t / (double)tot.s) * ln2);
        if (lse_out) lse_out[row] = (float)lse;
    }
}

template <typename R, bool VECTORISED>
__global__ void __launch_bounds__(256) lsg_bwd_kernel(const typename R::elem_t* logits, int64_t n_inner,
                                                      int64_t stride_outer, int64_t stride_inner, int64_t vocab,
                                                      const int64_t* __restrict__ index,
                                                      const float* __restrict__ lse,
                                                      const float* __restrict__ grad_logprob, float inv_t,
                                                      typename R::elem_t* dlogits, int64_t out_stride_outer,
                                                      int64_t out_stride_inner) {
    constexpr int VEC = R::VEC;
    const int64_t row = blockIdx.x;
    const typename R::elem_t* p = logits + row_offset(row, n_inner, stride_outer, stride_inner);
    typename R::elem_t* q = dlogits + row_offset(row, n_inner, out_stride_outer, out_stride_inner);
    const int tid = threadIdx.x, nthr = blockDim.x;
    const float g = grad_logprob[row] * inv_t;
    const int64_t nvec = VECTORISED ? vocab / VEC : 0;

    if (g == 0.f) {  // masked-out token: the gradient row is zero, the logits are not needed
        float zero[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) zero[j] = 0.f;
        for (int64_t i = tid; i < nvec; i += nthr) R::store_vec(q + i * VEC, zero);
        for (int64_t j = nvec * VEC + tid; j < vocab; j += nthr) R::store_one(q + j, 0.f);
        return;
    }

    const float c = inv_t * OI_LOG2E;
    const float l2 = lse[row] * OI_LOG2E;
    int64_t y = index[row];
    y = y < 0 ? 0 : (y >= vocab ? vocab - 1 : y);
    const float ng = -g;

    int64_t i = tid;
    constexpr int U = 4;
    for (; i + (int64_t)(U - 1) * nthr < nvec; i += (int64_t)U * nthr) {
        float z[U][VEC];
#pragma unroll
        for (int u = 0; u < U; ++u) R::load_vec(p + (i + (int64_t)u * nthr) * VEC, z[u]);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t base = (i + (int64_t)u * nthr) * VEC;
#pragma unroll
            for (int j = 0; j < VEC; ++j) z[u][j] = ng * __builtin_amdgcn_exp2f(fmaf(z[u][j], c, -l2));
            if (y >= base && y < base + VEC) {
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    if (base + j == y) z[u][j] += g;
            }
            R::store_vec(q + base, z[u]);
        }
    }
    for (; i < nvec; i += nthr) {
        float z[VEC];
        const int64_t base = i * VEC;
        R::load_vec(p + base, z);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            z[j] = ng * __builtin_amdgcn_exp2f(fmaf(z[j], c, -l2));
            if (base + j == y) z[j] += g;
        }
        R::store_vec(q + base, z);
    }
    for (int64_t j = nvec * VEC + tid; j < vocab; j += nthr) {
        float d = ng * __builtin_amdgcn_exp2f(fmaf(R::load_one(p + j), c, -l2));
        if (j == y) d += g;
        R::store_one(q + j, d);
    }
}

// Long rows (>= BURST_MIN_VECS 16-byte vectors): one 1024-thread workgroup per row, so that a CU
// holds one row at a time, and a two-deep software pipeline over batches of 64 KB: the loads of
// batch n+1 are issued and unpacked before batch n is exponentiated and stored.  Measured on
// [65536, 128256] bf16 (read 16.8 GB + write 16.8 GB): 5.7 ms against 6.6 ms for the four-wave
// kernel above, i.e. 5.9 instead of 5.1 TB/s; fewer, longer streams suit the memory system better
// than many short ones once writes are involved.
constexpr int BURST_THREADS = 1024;
constexpr int BURST_U = 4;
constexpr int64_t BURST_MIN_VECS = 3 * BURST_U * BURST_THREADS;

template <typename R>
__global__ void __launch_bounds__(BURST_THREADS)
    lsg_bwd_burst_kernel(const typename R::elem_t* logits, int64_t n_inner, int64_t stride_outer, int64_t stride_inner,
                         int64_t vocab, const int64_t* __restrict__ index, const float* __restrict__ lse,
                         const float* __restrict__ grad_logprob, float inv_t, typename R::elem_t* dlogits,
                         int64_t out_stride_outer, int64_t out_stride_inner) {
    constexpr int VEC = R::VEC;
    constexpr int U = BURST_U;
    const int64_t row = blockIdx.x;
    const typename R::elem_t* p = logits + row_offset(row, n_inner, stride_outer, stride_inner);
    typename R::elem_t* q = dlogits + row_offset(row, n_inner, out_stride_outer, out_stride_inner);
    const int tid = threadIdx.x;
    constexpr int64_t nthr = BURST_THREADS;
    const float g = grad_logprob[row] * inv_t;
    const int64_t nvec = vocab / VEC;

    if (g == 0.f) {  // masked-out token: the gradient row is zero, the logits are not needed
        float zero[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) zero[j] = 0.f;
        for (int64_t i = tid; i < nvec; i += nthr) R::store_vec(q + i * VEC, zero);
        for (int64_t j = nvec * VEC + tid; j < vocab; j += nthr) R::store_one(q + j, 0.f);
        return;
    }

    const float c = inv_t * OI_LOG2E;
    const float l2 = lse[row] * OI_LOG2E;
    int64_t y = index[row];
    y = y < 0 ? 0 : (y >= vocab ? vocab - 1 : y);
    const float ng = -g;

    int64_t i = tid;
    float z[U][VEC], zn[U][VEC];
    if (i + (U - 1) * nthr < nvec) {
#pragma unroll
        for (int u = 0; u < U; ++u) R::load_vec(p + (i + u * nthr) * VEC, z[u]);
    }
    for (; i + (U - 1) * nthr < nvec; i += U * nthr) {
        const int64_t nx = i + U * nthr;
        const bool more = nx + (U - 1) * nthr < nvec;
        if (more) {
#pragma unroll
            for (int u = 0; u < U; ++u) R::load_vec(p + (nx + u * nthr) * VEC, zn[u]);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t base = (i + u * nthr) * VEC;
#pragma unroll
            for (int j = 0; j < VEC; ++j) z[u][j] = ng * __builtin_amdgcn_exp2f(fmaf(z[u][j], c, -l2));
            if (y >= base && y < base + VEC) {
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    if (base + j == y) z[u][j] += g;
            }
            R::store_vec(q + base, z[u]);
        }
        if (more) {
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int j = 0; j < VEC; ++j) z[u][j] = zn[u][j];
        }
    }
    for (; i < nvec; i += nthr) {
        float w[VEC];
        const int64_t base = i * VEC;
        R::load_vec(p + base, w);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            w[j] = ng * __builtin_amdgcn_exp2f(fmaf(w[j], c, -l2));
            if (base + j == y) w[j] += g;
        }
        R::store_vec(q + base, w);
    }
    for (int64_t j = nvec * VEC + tid; j < vocab; j += nthr) {
        float d = ng * __builtin_amdgcn_exp2f(fmaf(R::load_one(p + j), c, -l2));
        if (j == y) d += g;
        R::store_one(q + j, d);
    }
}

inline int block_for_vocab(int64_t vocab, int vec) {
    // one 16-byte vector per lane per trip; short rows do not need four waves
    const int64_t vecs = vocab / vec;
    if (vecs >= 1024) return 256;
    if (vecs >= 256) return 128;
    return 64;
}

template <typename R>
int launch_fwd(const void* logits, int64_t rows, int64_t n_inner, int64_t so, int64_t si, int64_t vocab,
               const int64_t* index, float inv_t, float* logprob, float* entropy, float* lse, hipStream_t stream) {
    typedef typename R::elem_t E;
    const bool vec = oi_aligned(logits, 16) && (so % R::VEC == 0) && (si % R::VEC == 0);
    const dim3 grid((unsigned)rows), block(block_for_vocab(vocab, R::VEC));
    const E* p = static_cast<const E*>(logits);
#define OI_FWD(V_, E_)                                                                                              \
    hipLaunchKernelGGL((lsg_entropy_fwd_kernel<R, V_, E_>), grid, block, 0, stream, p, n_inner, so, si, vocab, index, \
                       inv_t, logprob, entropy, lse)
    if (vec) {
        if (entropy) OI_FWD(true, true); else OI_FWD(true, false);
    } else {
        if (entropy) OI_FWD(false, true); else OI_FWD(false, false);
    }
#undef OI_FWD
    return oi_launch_status();
}

template <typename R>
int launch_bwd(const void* logits, int64_t rows, int64_t n_inner, int64_t so, int64_t si, int64_t vocab,
               const int64_t* index, const float* lse, const float* grad, float inv_t, void* dlogits, int64_t oso,
               int64_t osi, hipStream_t stream) {
    typedef typename R::elem_t E;
    const bool vec = oi_aligned(logits, 16) && oi_aligned(dlogits, 16) && (so % R::VEC == 0) && (si % R::VEC == 0) &&
                     (oso % R::VEC == 0) && (osi % R::VEC == 0);
    const dim3 grid((unsigned)rows), block(block_for_vocab(vocab, R::VEC));
    const E* p = static_cast<const E*>(logits);
    E* q = static_cast<E*>(dlogits);
    if (vec && vocab / R::VEC >= BURST_MIN_VECS)
        hipLaunchKernelGGL((lsg_bwd_burst_kernel<R>), grid, dim3(BURST_THREADS), 0, stream, p, n_inner, so, si, vocab,
                           index, lse, grad, inv_t, q, oso, osi);
    else if (vec)
        hipLaunchKernelGGL((lsg_bwd_kernel<R, true>), grid, block, 0, stream, p, n_inner, so, si, vocab, index, lse,
                           grad, inv_t, q, oso, osi);
    else
        hipLaunchKernelGGL((lsg_bwd_kernel<R, false>), grid, block, 0, stream, p, n_inner, so, si, vocab, index, lse,
                           grad, inv_t, q, oso, osi);
    return oi_launch_status();
}

// ---------------------------------------------------------------------------------------------
// GRPO on materialised logits in one launch: forward statistics and the gradient with respect to
// the logits, with HBM seeing every row read once and its gradient written once.
//
// A token's upstream gradient depends on nothing but that token's own logprob and side inputs
// (old / reference logprobs, advantage, weight) once the loss denominators are known, and those
// depend on the mask alone.  So a 1024-thread workgroup reduces the softmax statistics of a row
// while parking the row on the CU (144 KB of it in the LDS, the rest in registers: 16 sweeps of
// 1024 16-byte pieces hold a row of 131072 bf16 logits), evaluates the GRPO derivative of the
// token and writes d logits from the parked copy.  What a longer row has beyond that is read a
// second time, from the caches.
//
// One workgroup per CU stays for the whole launch and takes every gridDim.x-th row: the loads of
// the next row are issued while the stores of the previous one are still draining (a fresh
// workgroup per row cannot start before the last store of its predecessor has left the CU, 4 us of
// a 25 us row), and the row's side inputs are requested at the top of the row, long before the
// lane that needs them gets there.  `token_coef` carries scale / denominator per token (0 on
// masked-out tokens).
// ---------------------------------------------------------------------------------------------
constexpr int FUSED_ROW_THREADS = 1024;
// sweeps of the workgroup over the row that are parked in the LDS (9 x 16 KB = 144 KB of the CU's
// 160 KB) and in registers (7 x 4 VGPRs per thread)
constexpr int FUSED_STASH_SWEEPS = 9;
constexpr int FUSED_KEEP_SWEEPS = 7;
constexpr int FUSED_SWEEPS = FUSED_STASH_SWEEPS + FUSED_KEEP_SWEEPS;
constexpr int FUSED_STASH_VECS = FUSED_STASH_SWEEPS * FUSED_ROW_THREADS;
constexpr int FUSED_RESIDENT_VECS = FUSED_SWEEPS * FUSED_ROW_THREADS;
// 16-byte loads per thread in flight during the first pass
constexpr int FUSED_LOOKAHEAD = 7;

template <typename R>
__global__ void __launch_bounds__(FUSED_ROW_THREADS)
    lsg_grpo_fused_kernel(const typename R::elem_t* __restrict__ logits, int64_t n_rows, int64_t n_inner,
                          int64_t stride_outer, int64_t stride_inner, int64_t vocab,
                          const int64_t* __restrict__ index, float inv_t, const float* __restrict__ old_lp,
                          const float* __restrict__ ref_lp, const float* __restrict__ adv,
                          const float* __restrict__ rho, const float* __restrict__ token_coef, GrpoCfg cfg,
                          float beta, float* __restrict__ logprob, float* __restrict__ entropy,
                          float* __restrict__ lse_out, typename R::elem_t* __restrict__ dlogits,
                          int64_t out_stride_outer, int64_t out_stride_inner) {
    constexpr int VEC = R::VEC;
    constexpr int NW = FUSED_ROW_THREADS / OI_WAVE;
    constexpr int64_t nthr = FUSED_ROW_THREADS;
    __shared__ float sm[3][NW];
    __shared__ float bcast[2];
    __shared__ __align__(16) typename R::raw_t stash[FUSED_STASH_VECS];
    static_assert(sizeof(typename R::raw_t) == 16, "row pieces are 16 bytes");
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int64_t nvec = vocab / VEC;
    const float c = inv_t * OI_LOG2E;
    // the offset of this thread's first piece of a row, as a value the optimiser cannot trace: the
    // addresses of the 16 sweeps are then formed where they are used instead of once for both passes,
    // where they would occupy 64 registers from the first load to the last store
    auto untraced = [](int off) {
        asm volatile("" : "+v"(off));
        return off;
    };
    const int first_piece = tid * VEC;
    // loads past the end of a short row are redirected to its last piece instead of being skipped:
    // unconditional loads are waited for one by one, guarded ones all at once
    const int last_piece = (int)((nvec - 1) * VEC);  // the launcher refuses rows without a whole piece

    typename R::raw_t raw[FUSED_SWEEPS];  // sweeps past the LDS part stay here for the second pass
    auto issue = [&](const typename R::elem_t* src, int k) {
        const int piece = untraced(first_piece) + k * (int)nthr * VEC;
        raw[k] = R::load_raw(src + (piece < last_piece ? piece : last_piece));
    };
    static_assert(FUSED_LOOKAHEAD <= FUSED_STASH_SWEEPS, "the registers of the first sweeps must be free in the second pass");
    if ((int64_t)blockIdx.x < n_rows) {
        const typename R::elem_t* first = logits + row_offset(blockIdx.x, n_inner, stride_outer, stride_inner);
#pragma unroll
        for (int k = 0; k < FUSED_LOOKAHEAD; ++k) issue(first, k);
    }
    for (int64_t row = blockIdx.x; row < n_rows; row += gridDim.x) {
        const typename R::elem_t* p = logits + row_offset(row, n_inner, stride_outer, stride_inner);
        typename R::elem_t* q = dlogits + row_offset(row, n_inner, out_stride_outer, out_stride_inner);
        // side inputs of the row, requested now and consumed after the first pass
        int64_t y = index[row];
        y = y < 0 ? 0 : (y >= vocab ? vocab - 1 : y);
        const float coef = token_coef[row];
        const float old_row = old_lp ? old_lp[row] : 0.f;
        const float ref_row = ref_lp ? ref_lp[row] : 0.f;
        const float adv_row = adv[row];
        const float rho_row = rho ? rho[row] : 1.f;

        // first pass: statistics, and the row is parked.  A rolling window: the load of sweep
        // k + FUSED_LOOKAHEAD is issued before sweep k is consumed, so that many 16-byte loads per
        // thread are in flight throughout; the first FUSED_LOOKAHEAD sweeps were requested before
        // the previous row's second pass and arrived while it ran.  Parked pieces are fetched with
        // non-temporal loads, what lies beyond with ordinary ones so that it stays cached for the
        // second pass.
        RowStat st = {OI_NEG_BIG, 0.f, 0.f};
        const float zy = R::load_one(p + y);
#pragma unroll
        for (int k = 0; k < FUSED_SWEEPS; ++k) {
            if (k + FUSED_LOOKAHEAD < FUSED_SWEEPS) issue(p, k + FUSED_LOOKAHEAD);
            const int64_t v = tid + (int64_t)k * nthr;
            if (k < FUSED_STASH_SWEEPS) stash[v] = raw[k];
            if (v < nvec) {
                float z[VEC];
                R::unpack(raw[k], z);
                stat_update_fma<VEC, true>(st, z, c);
            }
            // one piece's temporaries at a time: the parked pieces need the registers
            __builtin_amdgcn_sched_barrier(0);
        }
        for (int64_t i = FUSED_RESIDENT_VECS + tid; i < nvec; i += nthr) {
            float z[VEC];
            R::unpack(R::load_raw_cached(p + i * VEC), z);
            stat_update<VEC, true>(st, z, c);
        }
        for (int64_t j = nvec * VEC + tid; j < vocab; j += nthr) stat_update1<true>(st, R::load_one(p + j), c);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            RowStat o;
            o.m = __shfl_xor(st.m, off, OI_WAVE);
            o.s = __shfl_xor(st.s, off, OI_WAVE);
            o.t = __shfl_xor(st.t, off, OI_WAVE);
            st = stat_merge(st, o);
        }
        if (lane == 0) {
            sm[0][wave] = st.m;
            sm[1][wave] = st.s;
            sm[2][wave] = st.t;
        }
        __syncthreads();
        {
            // The registers of the first sweeps are free now (those sweeps wait in the LDS): the next
            // row's first loads travel while this row's gradient is computed and stored, so the CU
            // keeps reading during its write phase.  After the last row the same row is read again,
            // which keeps the loads unconditional.
            const int64_t next = row + gridDim.x < n_rows ? row + gridDim.x : row;
            const typename R::elem_t* pn = logits + row_offset(next, n_inner, stride_outer, stride_inner);
#pragma unroll
            for (int k = 0; k < FUSED_LOOKAHEAD; ++k) issue(pn, k);
        }
        if (tid == 0) {
            RowStat tot = {sm[0][0], sm[1][0], sm[2][0]};
            for (int w = 1; w < NW; ++w) {
                RowStat o = {sm[0][w], sm[1][w], sm[2][w]};
                tot = stat_merge(tot, o);
            }
            const double ln2 = 0.69314718055994530942;
            const double log2s = log2((double)tot.s);
            const double lse = ((double)tot.m + log2s) * ln2;
            const float lp = (float)((double)zy * (double)inv_t - lse);
            logprob[row] = lp;
            if (entropy) entropy[row] = (float)((log2s - (double)tot.t / (double)tot.s) * ln2);
            if (lse_out) lse_out[row] = (float)lse;
            float g = 0.f;
            if (coef != 0.f) {
                const float ratio = old_lp ? expf(lp - old_row) : 1.f;
                g = coef * grpo_token_dnew(lp, ratio, adv_row, ref_lp != nullptr, ref_row, rho_row, cfg, beta);
            }
            bcast[0] = g * inv_t;
            bcast[1] = (float)lse * OI_LOG2E;
        }
        __syncthreads();
        // (the next row's writes of sm / bcast come after that row's first barrier, which no thread
        // passes before it has read these two values)
        const float g = bcast[0], l2 = bcast[1];
        const float ng = -g;
        // - g 2^(x - l2) = -+ 2^(x - l2 + log2 |g|): one multiply less per logit in the parked part
        const float l2g = l2 - __builtin_amdgcn_logf(fabsf(g));
        const bool g_positive = g > 0.f;
        if (g == 0.f) {
            float zero[VEC];
#pragma unroll
            for (int j = 0; j < VEC; ++j) zero[j] = 0.f;
            for (int64_t i = tid; i < nvec; i += nthr) R::store_vec(q + i * VEC, zero);
            for (int64_t j = nvec * VEC + tid; j < vocab; j += nthr) R::store_one(q + j, 0.f);
            continue;
        }
        // second pass: the parked part (every thread reads back exactly the LDS entries it wrote, so
        // no barrier guards them), then what lies beyond it
        auto emit = [&](typename R::raw_t piece, typename R::elem_t* dst) {
            float w[VEC];
            R::unpack(piece, w);
#pragma unroll
            for (int j = 0; j < VEC; ++j) w[j] = ng * __builtin_amdgcn_exp2f(fmaf(w[j], c, -l2));
            R::store_vec(dst, w);
        };
        auto emit_signed = [&](typename R::raw_t piece, typename R::elem_t* dst, auto negative_tag) {
            float w[VEC];
            R::unpack(piece, w);
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const float e = __builtin_amdgcn_exp2f(fmaf(w[j], c, -l2g));
                w[j] = decltype(negative_tag)::value ? -e : e;
            }
            R::store_vec(dst, w);
        };
        auto parked_sweeps = [&](auto negative_tag) {
#pragma unroll
            for (int k = 0; k < FUSED_SWEEPS; ++k) {
                const int64_t v = tid + (int64_t)k * nthr;
                if (v < nvec) {
                    typename R::elem_t* dst = q + untraced(first_piece) + (int64_t)k * nthr * VEC;
                    if (k < FUSED_STASH_SWEEPS) emit_signed(stash[v], dst, negative_tag);
                    else emit_signed(raw[k], dst, negative_tag);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        if (g_positive) parked_sweeps(std::true_type{});  // d logits = - g softmax
        else parked_sweeps(std::false_type{});
        for (int64_t i = FUSED_RESIDENT_VECS + tid; i < nvec; i += nthr) emit(R::load_raw(p + i * VEC), q + i * VEC);
        // the label's entry gets + g.  The thread that stored the piece holding it stores the entry
        // again (stores of one thread to one address keep their order): no sweep has to look for it.
        if (y < nvec * VEC && (int)((y / VEC) % nthr) == tid)
            R::store_one(q + y, ng * __builtin_amdgcn_exp2f(fmaf(zy, c, -l2)) + g);
        for (int64_t j = nvec * VEC + tid; j < vocab; j += nthr) {
            float d = ng * __builtin_amdgcn_exp2f(fmaf(R::load_one(p + j), c, -l2));
            if (j == y) d += g;
            R::store_one(q + j, d);
        }
    }
}

template <typename R>
int launch_grpo_fused(const void* logits, int64_t rows, int64_t n_inner, int64_t so, int64_t si, int64_t vocab,
                      const int64_t* index, float inv_t, const float* old_lp, const float* ref_lp, const float* adv,
                      const float* rho, const float* coef, GrpoCfg cfg, float beta, float* logprob, float* entropy,
                      float* lse, void* dlogits, int64_t oso, int64_t osi, hipStream_t stream) {
    typedef typename R::elem_t E;
    const bool vec = oi_aligned(logits, 16) && oi_aligned(dlogits, 16) && (so % R::VEC == 0) && (si % R::VEC == 0) &&
                     (oso % R::VEC == 0) && (osi % R::VEC == 0);
    OI_RETURN_IF(!vec || vocab < R::VEC, OI_EALIGN);
    // one resident workgroup per CU (its LDS share leaves room for no second one)
    const int64_t cus = oi_cu_count();
    hipLaunchKernelGGL((lsg_grpo_fused_kernel<R>), dim3((unsigned)(rows < cus ? rows : cus)), dim3(FUSED_ROW_THREADS), 0,
                       stream, static_cast<const E*>(logits), rows, n_inner, so, si, vocab, index, inv_t, old_lp, ref_lp,
                       adv, rho, coef, cfg, beta, logprob, entropy, lse, static_cast<E*>(dlogits), oso, osi);
    return oi_launch_status();
}

// data[i] *= *scale for a contiguous tensor, skipped altogether when the device scalar is exactly 1
// (the upstream gradient of a loss that is differentiated directly): every workgroup reads the
// scalar and leaves, so the host never has to look at it.
template <typename R>
__global__ void __launch_bounds__(256) scale_by_scalar_kernel(typename R::elem_t* __restrict__ data, int64_t n,
                                                              bool vectorised, const float* __restrict__ scale) {
    const float s = *scale;
    if (s == 1.f) return;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x, first = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (vectorised) {
        for (int64_t v = first; v < n / R::VEC; v += stride) {
            float z[R::VEC];
            R::load_vec(data + v * R::VEC, z);
#pragma unroll
            for (int e = 0; e < R::VEC; ++e) z[e] *= s;
            R::store_vec(data + v * R::VEC, z);
        }
        for (int64_t i = n / R::VEC * R::VEC + first; i < n; i += stride) R::store_one(data + i, R::load_one(data + i) * s);
    } else {
        for (int64_t i = first; i < n; i += stride) R::store_one(data + i, R::load_one(data + i) * s);
    }
}

template <typename R>
int launch_scale(void* data, int64_t n, const float* scale, hipStream_t stream) {
    typedef typename R::elem_t E;
    const int64_t vecs = (n + R::VEC - 1) / R::VEC;
    const int64_t want = (vecs + 255) / 256;
    const unsigned blocks = (unsigned)(want < 1 ? 1 : (want > 16384 ? 16384 : want));
    hipLaunchKernelGGL((scale_by_scalar_kernel<R>), dim3(blocks), dim3(256), 0, stream, static_cast<E*>(data), n,
                       oi_aligned(data, 16), scale);
    return oi_launch_status();
}

int check_rows(const void* logits, int64_t n_outer, int64_t n_inner, int64_t so, int64_t si, int64_t vocab,
               const int64_t* index, float inv_t, int64_t* rows) {
    OI_RETURN_IF(n_outer < 0 || n_inner < 0 || vocab <= 0, OI_EINVAL);
    OI_RETURN_IF(!(inv_t > 0.f) || !(inv_t < 3.0e38f), OI_EINVAL);
    *rows = n_outer * n_inner;
    OI_RETURN_IF(*rows > 0x7fffffffLL, OI_EINVAL);
    if (*rows == 0) return OI_OK;
    OI_RETURN_IF(!logits || !index, OI_ENULL);
    OI_RETURN_IF(si < vocab && n_inner > 1, OI_EINVAL);
    OI_RETURN_IF(so < 0 || si < 0, OI_EINVAL);
    return OI_OK;
}

}  // namespace

extern "C" int oi_lsg_entropy_fwd(const void* logits, int dtype, int64_t n_outer, int64_t n_inner,
                                  int64_t stride_outer, int64_t stride_inner, int64_t vocab, const int64_t* index,
                                  float inv_temperature, float* logprob, float* entropy, float* lse, void* stream) {
    int64_t rows = 0;
    const int rc = check_rows(logits, n_outer, n_inner, stride_outer, stride_inner, vocab, index, inv_temperature, &rows);
    if (rc != OI_OK) return rc;
    OI_RETURN_IF(dtype != OI_DTYPE_F32 && dtype != OI_DTYPE_BF16 && dtype != OI_DTYPE_F16, OI_EDTYPE);
    if (rows == 0) return OI_OK;
    OI_RETURN_IF(!logprob, OI_ENULL);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case OI_DTYPE_F32:
            OI_RETURN_IF(!oi_aligned(logits, 4), OI_EALIGN);
            return launch_fwd<F32Row>(logits, rows, n_inner, stride_outer, stride_inner, vocab, index, inv_temperature,
                                      logprob, entropy, lse, s);
        case OI_DTYPE_BF16:
            OI_RETURN_IF(!oi_aligned(logits, 2), OI_EALIGN);
            return launch_fwd<BF16Row>(logits, rows, n_inner, stride_outer, stride_inner, vocab, index,
                                       inv_temperature, logprob, entropy, lse, s);
        default:
            OI_RETURN_IF(!oi_aligned(logits, 2), OI_EALIGN);
            return launch_fwd<F16Row>(logits, rows, n_inner, stride_outer, stride_inner, vocab, index, inv_temperature,
                                      logprob, entropy, lse, s);
    }
}

extern "C" int oi_lsg_bwd(const void* logits, int dtype, int64_t n_outer, int64_t n_inner, int64_t stride_outer,
                          int64_t stride_inner, int64_t vocab, const int64_t* index, const float* lse,
                          const float* grad_logprob, float inv_temperature, void* dlogits, int64_t out_stride_outer,
                          int64_t out_stride_inner, void* stream) {
    int64_t rows = 0;
    const int rc = check_rows(logits, n_outer, n_inner, stride_outer, stride_inner, vocab, index, inv_temperature, &rows);
    if (rc != OI_OK) return rc;
    OI_RETURN_IF(dtype != OI_DTYPE_F32 && dtype != OI_DTYPE_BF16 && dtype != OI_DTYPE_F16, OI_EDTYPE);
    if (rows == 0) return OI_OK;
    OI_RETURN_IF(!lse || !grad_logprob || !dlogits, OI_ENULL);
    OI_RETURN_IF(out_stride_outer < 0 || out_stride_inner < 0, OI_EINVAL);
    OI_RETURN_IF(out_stride_inner < vocab && n_inner > 1, OI_EINVAL);
    // in-place use is only defined when every row maps onto itself
    OI_RETURN_IF(dlogits == logits && (out_stride_outer != stride_outer || out_stride_inner != stride_inner),
                 OI_EINVAL);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t esz = dtype == OI_DTYPE_F32 ? 4 : 2;
    OI_RETURN_IF(!oi_aligned(logits, esz) || !oi_aligned(dlogits, esz), OI_EALIGN);
    switch (dtype) {
        case OI_DTYPE_F32:
            return launch_bwd<F32Row>(logits, rows, n_inner, stride_outer, stride_inner, vocab, index, lse,
                                      grad_logprob, inv_temperature, dlogits, out_stride_outer, out_stride_inner, s);
        case OI_DTYPE_BF16:
            return launch_bwd<BF16Row>(logits, rows, n_inner, stride_outer, stride_inner, vocab, index, lse,
                                       grad_logprob, inv_temperature, dlogits, out_stride_outer, out_stride_inner, s);
        default:
            return launch_bwd<F16Row>(logits, rows, n_inner, stride_outer, stride_inner, vocab, index, lse,
                                      grad_logprob, inv_temperature, dlogits, out_stride_outer, out_stride_inner, s);
    }
}

extern "C" int oi_lsg_grpo_fwd_bwd(const void* logits, int dtype, int64_t n_outer, int64_t n_inner, int64_t stride_outer,
                                   int64_t stride_inner, int64_t vocab, const int64_t* index, float inv_temperature,
                                   const float* old_logprobs, const float* ref_logprobs, const float* advantages,
                                   const float* rho_weights, const float* token_coef, int loss_fn, float ratio_lo,
                                   float ratio_hi, int kl_estimator, float beta, float* logprob, float* entropy,
                                   float* lse, void* dlogits, int64_t out_stride_outer, int64_t out_stride_inner,
                                   void* stream) {
    int64_t rows = 0;
    const int rc = check_rows(logits, n_outer, n_inner, stride_outer, stride_inner, vocab, index, inv_temperature, &rows);
    if (rc != OI_OK) return rc;
    OI_RETURN_IF(dtype != OI_DTYPE_F32 && dtype != OI_DTYPE_BF16 && dtype != OI_DTYPE_F16, OI_EDTYPE);
    OI_RETURN_IF(loss_fn != OI_LOSS_DAPO && loss_fn != OI_LOSS_CISPO, OI_EINVAL);
    OI_RETURN_IF(kl_estimator < 0 || kl_estimator > 3, OI_EINVAL);
    if (rows == 0) return OI_OK;
    OI_RETURN_IF(!advantages || !token_coef || !logprob || !dlogits, OI_ENULL);
    OI_RETURN_IF(dlogits == logits, OI_EINVAL);  // a row is read again after its gradient has started to land
    OI_RETURN_IF(out_stride_outer < 0 || out_stride_inner < 0 || (out_stride_inner < vocab && n_inner > 1), OI_EINVAL);
    const GrpoCfg cfg = {loss_fn, ratio_lo, ratio_hi, kl_estimator};
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case OI_DTYPE_F32:
            return launch_grpo_fused<F32Row>(logits, rows, n_inner, stride_outer, stride_inner, vocab, index,
                                             inv_temperature, old_logprobs, ref_logprobs, advantages, rho_weights,
                                             token_coef, cfg, beta, logprob, entropy, lse, dlogits, out_stride_outer,
                                             out_stride_inner, s);
        case OI_DTYPE_BF16:
            return launch_grpo_fused<BF16Row>(logits, rows, n_inner, stride_outer, stride_inner, vocab, index,
                                              inv_temperature, old_logprobs, ref_logprobs, advantages, rho_weights,
                                              token_coef, cfg, beta, logprob, entropy, lse, dlogits, out_stride_outer,
                                              out_stride_inner, s);
        default:
            return launch_grpo_fused<F16Row>(logits, rows, n_inner, stride_outer, stride_inner, vocab, index,
                                             inv_temperature, old_logprobs, ref_logprobs, advantages, rho_weights,
                                             token_coef, cfg, beta, logprob, entropy, lse, dlogits, out_stride_outer,
                                             out_stride_inner, s);
    }
}

extern "C" int oi_scale_by_device_scalar(void* data, int dtype, int64_t n, const float* scale, void* stream) {
    OI_RETURN_IF(n < 0, OI_EINVAL);
    OI_RETURN_IF(dtype != OI_DTYPE_F32 && dtype != OI_DTYPE_BF16 && dtype != OI_DTYPE_F16, OI_EDTYPE);
    if (n == 0) return OI_OK;
    OI_RETURN_IF(!data || !scale, OI_ENULL);
    OI_RETURN_IF(!oi_aligned(data, dtype == OI_DTYPE_F32 ? 4 : 2), OI_EALIGN);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case OI_DTYPE_F32: return launch_scale<F32Row>(data, n, scale, s);
        case OI_DTYPE_BF16: return launch_scale<BF16Row>(data, n, scale, s);
        default: return launch_scale<F16Row>(data, n, scale, s);
    }
}

// GRPO / DPO loss arithmetic and the masked reductions around it.
//
// All of it is O(tokens) fp32 work on [rows, cols] side tensors (a few MB at most); what matters
// here is doing each micro-batch in two launches instead of dozens, fixed (deterministic)
// summation order, and exact agreement with the branch semantics of torch.clamp / torch.max.
#include "oi_common.h"
#include "oi_grpo_math.h"

#include <mutex>

// Partial sums of oi_grpo_fused_fwd_static, the entry point for callers that cannot allocate.
// Every GPU the library runs on holds its own copy of this array at its own address until the
// process ends.  In host code the name is only a handle for hipGetSymbolAddress: kernels are given
// the per-device address that static_scratch_ptr() looked up, never the name.
static __device__ __align__(256) float oi_static_scratch[OI_GRPO_STATIC_MAX_BLOCKS * 15];

namespace {

__global__ void grpo_terms_fwd_kernel(const float* __restrict__ nlp, const float* __restrict__ ratio,
                                      const float* __restrict__ adv, const float* __restrict__ ref,
                                      const float* __restrict__ w, int64_t n, GrpoCfg c, float* __restrict__ pg,
                                      float* __restrict__ clipfrac, float* __restrict__ kl) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const GrpoOut o = grpo_token_fwd(nlp[i], ratio[i], adv[i], ref != nullptr, ref ? ref[i] : 0.f, w[i], c);
    pg[i] = o.pg;
    clipfrac[i] = o.clipfrac;
    kl[i] = o.kl[c.kl_est];
}

__global__ void grpo_terms_bwd_kernel(const float* __restrict__ nlp, const float* __restrict__ ratio,
                                      const float* __restrict__ adv, const float* __restrict__ ref,
                                      const float* __restrict__ w, const float* __restrict__ gpg,
                                      const float* __restrict__ gkl, int64_t n, GrpoCfg c,
                                      float* __restrict__ d_new, float* __restrict__ d_ratio) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const GrpoGrad g = grpo_token_bwd(nlp[i], ratio[i], adv[i], ref != nullptr, ref ? ref[i] : 0.f, w[i], c);
    const float a = gpg ? gpg[i] : 0.f, b = gkl ? gkl[i] : 0.f;
    if (d_new) d_new[i] = a * g.dpg_dnew + b * g.dkl_dnew;
    if (d_ratio) d_ratio[i] = a * g.dpg_dratio + b * g.dkl_dratio;
}

// ---- fused scalar loss -----------------------------------------------------------------------
constexpr int FUSED_THREADS = 256;
constexpr int FUSED_PER_THREAD = 4;
constexpr int FUSED_CHUNK = FUSED_THREADS * FUSED_PER_THREAD;
constexpr int NSUM = 15;  // partial sums kept per (row, chunk): entries 0..14 of the statistics vector
static_assert(NSUM + 1 == OI_GRPO_NUM_STATS, "the last statistic is derived from the sums");

// Per-token inputs of the statistics pass.  Two ways to obtain the loss terms of a token:
//   from the logprobs (pg == nullptr): ratio = exp(new - old), terms by grpo_token_fwd;
//   from tensors the caller already holds (pg != nullptr): pg, clipfrac and ratio are read, the
//   four KL estimators are evaluated from new - ref and ratio.
// The remaining pointers are optional tensors that are only averaged over the mask.
struct StatIn {
    const float *nlp, *old, *ref, *adv, *rho;
    const float *pg, *clipfrac, *ratio;
    const float *ent, *drop_any, *drop_low, *drop_high, *rho_clipped;
    const uint8_t* mask;
};

__global__ void __launch_bounds__(FUSED_THREADS)
    grpo_stats_partial_kernel(StatIn in, int64_t cols, int64_t nchunks, GrpoCfg c, float beta,
                              float* __restrict__ partial) {
    const int64_t row = blockIdx.x / nchunks, chunk = blockIdx.x - row * nchunks;
    float acc[NSUM];
#pragma unroll
    for (int q = 0; q < NSUM; ++q) acc[q] = 0.f;
    const int64_t base = row * cols;
#pragma unroll
    for (int k = 0; k < FUSED_PER_THREAD; ++k) {
        const int64_t col = chunk * FUSED_CHUNK + (int64_t)k * FUSED_THREADS + threadIdx.x;
        if (col < cols) {
            const int64_t i = base + col;
            const float x = in.nlp ? in.nlp[i] : 0.f;
            const float w = in.rho ? in.rho[i] : 1.f;
            GrpoOut o;
            float ratio;
            if (in.pg) {
                ratio = in.ratio[i];
                o = grpo_token_fwd(x, ratio, 0.f, in.ref != nullptr, in.ref ? in.ref[i] : 0.f, 1.f, c);
                o.pg = in.pg[i];
                o.clipfrac = in.clipfrac[i];
            } else {
                ratio = in.old ? expf(x - in.old[i]) : 1.f;
                o = grpo_token_fwd(x, ratio, in.adv[i], in.ref != nullptr, in.ref ? in.ref[i] : 0.f, w, c);
            }
            const float mf = in.mask[i] ? 1.f : 0.f;
            acc[0] += (o.pg + beta * o.kl[c.kl_est]) * mf;
            acc[1] += o.pg * mf;
            acc[2] += o.kl[0] * mf;
            acc[3] += o.kl[1] * mf;
            acc[4] += o.kl[2] * mf;
            acc[5] += o.kl[3] * mf;
            acc[6] += o.clipfrac * mf;
            acc[7] += ratio * mf;
            acc[8] += in.ent ? in.ent[i] * mf : 0.f;
            acc[9] += mf;
            acc[10] += in.drop_any ? in.drop_any[i] * mf : 0.f;
            acc[11] += in.drop_low ? in.drop_low[i] * mf : 0.f;
            acc[12] += in.drop_high ? in.drop_high[i] * mf : 0.f;
            acc[13] += w * mf;
            acc[14] += in.rho_clipped ? in.rho_clipped[i] * mf : 0.f;
        }
    }
    // wave sums first, then one pass over the four waves: fixed order, one barrier
    __shared__ float wave_sums[FUSED_THREADS / OI_WAVE][NSUM];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int q = 0; q < NSUM; ++q) {
        const float t = oi_wave_sum(acc[q]);
        if (lane == 0) wave_sums[wave][q] = t;
    }
    __syncthreads();
    if (threadIdx.x < NSUM) {
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < FUSED_THREADS / OI_WAVE; ++w) t += wave_sums[w][threadIdx.x];
        partial[(size_t)blockIdx.x * NSUM + threadIdx.x] = t;
    }
}

__device__ __forceinline__ double block_sum_f64(double v, double* scratch) {
    v = oi_wave_sum(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    double t = 0.0;
    for (int w = 0; w < nw; ++w) t += scratch[w];
    return t;
}

// One workgroup: per-row totals in fp64 in chunk order, then the loss and the statistics.
// Statistic q goes to out_stats[q * out_stride] when bit q of write_mask is set.
__global__ void __launch_bounds__(256)
    grpo_stats_final_kernel(const float* __restrict__ partial, int64_t rows, int64_t nchunks, int axis_mode,
                            float denominator, float scale, float beta, int kl_est, float* __restrict__ out_stats,
                            int64_t out_stride, uint32_t write_mask, float* __restrict__ row_denoms) {
    __shared__ double scratch[4];
    double tot[NSUM];
    for (int q = 0; q < NSUM; ++q) tot[q] = 0.0;
    double row_mean_sum = 0.0;
    // pass 1: totals, and for axis_mode 1 the per-row means and reciprocal denominators
    for (int64_t r = threadIdx.x; r < rows; r += blockDim.x) {
        double rt[NSUM];
        for (int q = 0; q < NSUM; ++q) rt[q] = 0.0;
        for (int64_t ch = 0; ch < nchunks; ++ch) {
            const float* p = partial + (r * nchunks + ch) * NSUM;
            for (int q = 0; q < NSUM; ++q) rt[q] += (double)p[q];
        }
        for (int q = 0; q < NSUM; ++q) tot[q] += rt[q];
        if (axis_mode == 1) {
            const double den = denominator > 0.f ? (double)denominator : rt[9];
            const double inv = den > 0.0 ? 1.0 / den : 0.0;
            row_mean_sum += rt[0] * inv;
            if (row_denoms) row_denoms[r] = (float)(inv / (double)rows);
        }
    }
    double all[NSUM];
    for (int q = 0; q < NSUM; ++q) all[q] = block_sum_f64(tot[q], scratch);
    const double rms = block_sum_f64(row_mean_sum, scratch);
    double inv_global = 0.0;
    if (axis_mode == 0) {
        const double den = denominator > 0.f ? (double)denominator : all[9];
        inv_global = den > 0.0 ? 1.0 / den : 0.0;
        if (row_denoms)
            for (int64_t r = threadIdx.x; r < rows; r += blockDim.x) row_denoms[r] = (float)inv_global;
    }
    if (threadIdx.x == 0) {
        float st[OI_GRPO_NUM_STATS];
        const double loss = axis_mode == 0 ? all[0] * inv_global : rms / (double)rows;
        st[0] = (float)(loss * (double)scale);
        const double invc = all[9] > 0.0 ? 1.0 / all[9] : 0.0;
        for (int q = 1; q < NSUM; ++q) st[q] = (float)(all[q] * invc);
        st[9] = (float)all[9];
        // the KL share of the loss, rounded as the caller's fp32 product of the mean and beta
        st[15] = st[2 + kl_est] * beta;
        for (int q = 0; q < OI_GRPO_NUM_STATS; ++q)
            if ((write_mask >> q) & 1u) out_stats[q * out_stride] = st[q];
    }
}

__global__ void grpo_fused_bwd_kernel(const float* __restrict__ nlp, const float* __restrict__ old,
                                      const float* __restrict__ ref, const float* __restrict__ adv,
                                      const uint8_t* __restrict__ mask, const float* __restrict__ rho, int64_t rows,
                                      int64_t cols, GrpoCfg c, float beta, float scale,
                                      const float* __restrict__ row_denoms, const float* __restrict__ grad_loss,
                                      float* __restrict__ d_new) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * cols) return;
    if (!mask[i]) {
        d_new[i] = 0.f;
        return;
    }
    const int64_t r = i / cols;
    const float x = nlp[i];
    const float ratio = old ? expf(x - old[i]) : 1.f;
    const float w = rho ? rho[i] : 1.f;
    const float per_token = grpo_token_dnew(x, ratio, adv[i], ref != nullptr, ref ? ref[i] : 0.f, w, c, beta);
    d_new[i] = (grad_loss ? grad_loss[0] : 1.f) * scale * row_denoms[r] * per_token;
}

// ---- group-normalised advantages ----------------------------------------------------------------
__global__ void group_adv_kernel(const double* __restrict__ scores, int64_t n_groups, int64_t gsz, int mode,
                                 float* __restrict__ out) {
    const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= n_groups) return;
    const double* s = scores + g * gsz;
    double sum = 0.0;
    for (int64_t k = 0; k < gsz; ++k) sum += s[k];
    const double mean = sum / (double)gsz;
    double var = 0.0;
    for (int64_t k = 0; k < gsz; ++k) {
        const double d = s[k] - mean;
        var += d * d;
    }
    const double sd = sqrt(var / (double)gsz);
    for (int64_t k = 0; k < gsz; ++k) {
        const double a = mode == 0 ? (s[k] - mean) / (sd + 1e-8) : (s[k] - mean);
        out[g * gsz + k] = (float)a;
    }
}

// ---- masked mean ----------------------------------------------------------------------------------
__device__ __forceinline__ float mask_at(const void* mask, int is_float, int64_t i) {
    return is_float ? static_cast<const float*>(mask)[i] : (static_cast<const uint8_t*>(mask)[i] ? 1.f : 0.f);
}

// partial[(e * rows + r) * nchunks + ch] = sum values*mask ; cnt[r * nchunks + ch] = sum mask
__global__ void __launch_bounds__(FUSED_THREADS)
    masked_partial_kernel(const float* __restrict__ values, const void* __restrict__ mask, int mask_is_float,
                          int64_t rows, int64_t cols, int64_t nchunks, float* __restrict__ partial,
                          float* __restrict__ cnt) {
    // one block per (extra, row, chunk)
    const int64_t chunk = blockIdx.x % nchunks, er = blockIdx.x / nchunks, row = er % rows, e = er / rows;
    float num = 0.f, c = 0.f;
#pragma unroll
    for (int k = 0; k < FUSED_PER_THREAD; ++k) {
        const int64_t col = chunk * FUSED_CHUNK + (int64_t)k * FUSED_THREADS + threadIdx.x;
        if (col < cols) {
            const float m = mask_at(mask, mask_is_float, row * cols + col);
            num += values[(e * rows + row) * cols + col] * m;
            c += m;
        }
    }
    __shared__ float scratch[16];
    num = oi_block_sum(num, scratch);
    c = oi_block_sum(c, scratch);
    if (threadIdx.x == 0) {
        partial[(e * rows + row) * nchunks + chunk] = num;
        if (e == 0) cnt[row * nchunks + chunk] = c;
    }
}

__global__ void __launch_bounds__(256)
    masked_final_kernel(const float* __restrict__ partial, const float* __restrict__ cnt, int64_t rows,
                        int64_t nchunks, int axis_mode, float denominator, float* __restrict__ out,
                        float* __restrict__ row_denoms) {
    __shared__ double scratch[4];
    const int64_t e = blockIdx.x;
    double num_tot = 0.0, cnt_tot = 0.0, mean_sum = 0.0;
    for (int64_t r = threadIdx.x; r < rows; r += blockDim.x) {
        double rn = 0.0, rc = 0.0;
        for (int64_t ch = 0; ch < nchunks; ++ch) {
            rn += (double)partial[(e * rows + r) * nchunks + ch];
            rc += (double)cnt[r * nchunks + ch];
        }
        num_tot += rn;
        cnt_tot += rc;
        if (axis_mode == 1) {
            const double den = denominator > 0.f ? (double)denominator : rc;
            const double inv = den > 0.0 ? 1.0 / den : 0.0;
            mean_sum += rn * inv;
            if (row_denoms && e == 0) row_denoms[r] = (float)(inv / (double)rows);
        }
    }
    num_tot = block_sum_f64(num_tot, scratch);
    cnt_tot = block_sum_f64(cnt_tot, scratch);
    mean_sum = block_sum_f64(mean_sum, scratch);
    double inv_global = 0.0;
    if (axis_mode == 0) {
        const double den = denominator > 0.f ? (double)denominator : cnt_tot;
        inv_global = den > 0.0 ? 1.0 / den : 0.0;
        if (row_denoms && e == 0)
            for (int64_t r = threadIdx.x; r < rows; r += blockDim.x) row_denoms[r] = (float)inv_global;
    }
    if (threadIdx.x == 0) out[e] = (float)(axis_mode == 0 ? num_tot * inv_global : mean_sum / (double)rows);
}

__global__ void masked_bwd_kernel(const float* __restrict__ grad_out, const void* __restrict__ mask,
                                  int mask_is_float, const float* __restrict__ row_denoms, int64_t extra,
                                  int64_t rows, int64_t cols, float* __restrict__ d_values) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t per = rows * cols;
    if (i >= extra * per) return;
    const int64_t e = i / per, rc = i - e * per, r = rc / cols;
    d_values[i] = grad_out[e] * mask_at(mask, mask_is_float, rc) * row_denoms[r];
}

// ---- per-sequence logprob sums ------------------------------------------------------------------
__global__ void __launch_bounds__(256)
    seq_logp_fwd_kernel(const float* __restrict__ lp, const int64_t* __restrict__ labels,
                        const int32_t* __restrict__ cu, int64_t n_seqs, int64_t total, int average,
                        float* __restrict__ out, float* __restrict__ counts) {
    const int64_t s = blockIdx.x;
    int64_t a, b;
    oi_seq_range(cu, s, n_seqs, total, &a, &b);
    float sum = 0.f, cnt = 0.f;
    for (int64_t t = a + threadIdx.x; t < b; t += blockDim.x) {
        const float keep = labels[t + 1] != -100 ? 1.f : 0.f;
        sum += lp[t] * keep;
        cnt += keep;
    }
    __shared__ float scratch[16];
    sum = oi_block_sum(sum, scratch);
    cnt = oi_block_sum(cnt, scratch);
    if (threadIdx.x == 0) {
        out[s] = average ? sum / fmaxf(cnt, 1.f) : sum;
        if (counts) counts[s] = cnt;
    }
}

__global__ void __launch_bounds__(256)
    seq_logp_bwd_kernel(const float* __restrict__ grad_out, const int64_t* __restrict__ labels,
                        const int32_t* __restrict__ cu, const float* __restrict__ counts, int64_t n_seqs,
                        int64_t total, int average, float* __restrict__ d_lp) {
    const int64_t s = blockIdx.x;
    int64_t a, b;
    oi_seq_range(cu, s, n_seqs, total, &a, &b);
    const float g = average ? grad_out[s] / fmaxf(counts[s], 1.f) : grad_out[s];
    for (int64_t t = a + threadIdx.x; t < b; t += blockDim.x) d_lp[t] = labels[t + 1] != -100 ? g : 0.f;
    // the unscored last position of a padded row, or of the packed row
    if (threadIdx.x == 0) {
        if (!cu) d_lp[s * total + total - 1] = 0.f;
        else if (s == n_seqs - 1) d_lp[total - 1] = 0.f;
    }
}

// ---- sigmoid preference loss -------------------------------------------------------------------
__device__ __forceinline__ float log_sigmoid(float u) { return fminf(u, 0.f) - log1pf(expf(-fabsf(u))); }
__device__ __forceinline__ float sigmoid(float u) { return 1.f / (1.f + expf(-u)); }

__global__ void dpo_fwd_kernel(const float* __restrict__ pc, const float* __restrict__ pr,
                               const float* __restrict__ rc, const float* __restrict__ rr,
                               const float* __restrict__ wts, int64_t n, float beta, float ls, float margin,
                               float* __restrict__ losses, float* __restrict__ cr, float* __restrict__ rj) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float refc = rc ? rc[i] : 0.f, refr = rr ? rr[i] : 0.f;
    float x = pc[i] - pr[i];
    if (rc && rr) x -= (refc - refr);
    x -= margin;
    float l = -log_sigmoid(beta * x) * (1.f - ls) - log_sigmoid(-beta * x) * ls;
    if (wts) l *= wts[i];
    losses[i] = l;
    if (cr) cr[i] = beta * (pc[i] - refc);
    if (rj) rj[i] = beta * (pr[i] - refr);
}

__global__ void dpo_bwd_kernel(const float* __restrict__ pc, const float* __restrict__ pr,
                               const float* __restrict__ rc, const float* __restrict__ rr,
                               const float* __restrict__ wts, const float* __restrict__ gl, int64_t n, float beta,
                               float ls, float margin, float* __restrict__ dpc, float* __restrict__ dpr) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float x = pc[i] - pr[i];
    if (rc && rr) x -= (rc[i] - rr[i]);
    x -= margin;
    float dx = beta * (-(1.f - ls) * sigmoid(-beta * x) + ls * sigmoid(beta * x));
    if (wts) dx *= wts[i];
    dx *= gl[i];
    if (dpc) dpc[i] = dx;
    if (dpr) dpr[i] = -dx;
}


// ---- small per-token helpers of the GRPO step ------------------------------------------------
__global__ void estimate_kl_fwd_kernel(const float* __restrict__ d, const float* __restrict__ ratio, int64_t n,
                                       float* __restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float x = d[i];
    out[i] = x;
    out[n + i] = x * x / 2.f;
    out[2 * n + i] = expm1f(-x) + x;
    out[3 * n + i] = ratio[i] * x;
}

__global__ void estimate_kl_bwd_kernel(const float* __restrict__ d, const float* __restrict__ ratio,
                                       const float* __restrict__ g, int64_t n, float* __restrict__ dd,
                                       float* __restrict__ dratio) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float x = d[i];
    if (dd) dd[i] = g[i] + g[n + i] * x + g[2 * n + i] * (-expm1f(-x)) + g[3 * n + i] * ratio[i];
    if (dratio) dratio[i] = g[3 * n + i] * x;
}

__global__ void mask_logprobs_kernel(const float* __restrict__ lp, const uint8_t* __restrict__ mask, int64_t n,
                                     float fill, float* __restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float x = lp[i];
    out[i] = (mask[i] && x == x) ? x : fill;
}

__global__ void mask_logprobs_bwd_kernel(const float* __restrict__ lp, const uint8_t* __restrict__ mask,
                                         const float* __restrict__ g, int64_t n, float* __restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float x = lp[i];
    out[i] = (mask[i] && x == x) ? g[i] : 0.f;
}

struct RhoCfg {
    int seq_level, tv;
    float mask_lo, mask_hi, clamp_lo, clamp_hi;
};

// One workgroup per row: row means first (sequence-level rho, TV divergence), then the tokens.
__global__ void __launch_bounds__(256)
    rho_correction_kernel(const float* __restrict__ old, const float* __restrict__ vllm,
                          const uint8_t* __restrict__ mask, const float* __restrict__ adv, int64_t cols, RhoCfg c,
                          float* __restrict__ rho_out, float* __restrict__ weights, float* __restrict__ drop_any,
                          float* __restrict__ drop_low, float* __restrict__ drop_high,
                          float* __restrict__ clipped_flag) {
    const int64_t base = (int64_t)blockIdx.x * cols;
    __shared__ float scratch[16];
    float sum_diff = 0.f, sum_tv = 0.f, cnt = 0.f;
    if (c.seq_level || c.tv) {
        for (int64_t j = threadIdx.x; j < cols; j += blockDim.x) {
            const bool m = mask[base + j] != 0;
            const float diff = m ? clamp_keep_nan(old[base + j] - vllm[base + j], -10.f, 10.f) : 0.f;
            const float mf = m ? 1.f : 0.f;
            sum_diff += diff * mf;
            sum_tv += fabsf(expf(diff) - 1.f) * mf;
            cnt += mf;
        }
        sum_diff = oi_block_sum(sum_diff, scratch);
        sum_tv = oi_block_sum(sum_tv, scratch);
        cnt = oi_block_sum(cnt, scratch);
    }
    const float n = fmaxf(cnt, 1.f);
    const float seq_rho = expf(sum_diff / n);
    const float tv_row = sum_tv / n;
    for (int64_t j = threadIdx.x; j < cols; j += blockDim.x) {
        const int64_t i = base + j;
        const bool m = mask[i] != 0;
        const float diff = m ? clamp_keep_nan(old[i] - vllm[i], -10.f, 10.f) : 0.f;
        const float rho = expf(diff);
        const float eff = c.seq_level ? seq_rho : rho;
        const float probe = c.tv ? tv_row : eff;
        bool low = c.mask_lo > 0.f && probe < c.mask_lo && m;
        bool high = c.mask_hi > 0.f && probe > c.mask_hi && m;
        if (c.tv) {
            const float sgn = diff > 0.f ? 1.f : (diff < 0.f ? -1.f : diff);
            const bool grows = sgn * adv[i] > 0.f;
            low = low && grows;
            high = high && grows;
        }
        float cl = eff;
        if (c.clamp_lo > 0.f) cl = cl < c.clamp_lo ? c.clamp_lo : cl;
        if (c.clamp_hi > 0.f) cl = cl > c.clamp_hi ? c.clamp_hi : cl;
        const bool keep = m && !low && !high;
        rho_out[i] = rho;
        weights[i] = keep ? cl : 0.f;
        drop_any[i] = (low || high) ? 1.f : 0.f;
        drop_low[i] = low ? 1.f : 0.f;
        drop_high[i] = high ? 1.f : 0.f;
        clipped_flag[i] = cl != eff ? 1.f : 0.f;
    }
}

inline unsigned blocks_for(int64_t n, int threads) { return (unsigned)((n + threads - 1) / threads); }

int check_cfg(int loss_fn, int kl_estimator) {
    OI_RETURN_IF(loss_fn != OI_LOSS_DAPO && loss_fn != OI_LOSS_CISPO, OI_EINVAL);
    OI_RETURN_IF(kl_estimator < 0 || kl_estimator > 3, OI_EINVAL);
    return OI_OK;
}

// ---- debug statistics of two logprob tensors over a mask (one workgroup, fp64 accumulation) ----
__global__ void __launch_bounds__(1024)
    logprob_diff_stats_kernel(const float* __restrict__ local, const float* __restrict__ other,
                              const uint8_t* __restrict__ mask, int64_t n, float* __restrict__ out) {
    __shared__ double red[5][16];
    double cnt = 0.0, sd = 0.0, sd2 = 0.0, skl = 0.0;
    float mx = 0.f;
    bool bad = false;
    for (int64_t i = threadIdx.x; i < n; i += 1024) {
        const float o = other[i];
        if (!mask[i] || o != o) continue;
        const float l = local[i];
        const float d = fabsf(l - o);
        cnt += 1.0;
        sd += (double)d;
        sd2 += (double)d * (double)d;
        skl += (double)(__expf(o) * (o - l));
        bad |= d != d;
        mx = fmaxf(mx, d);
    }
    if (bad) mx = __builtin_nanf("");
    cnt = oi_wave_sum(cnt);
    sd = oi_wave_sum(sd);
    sd2 = oi_wave_sum(sd2);
    skl = oi_wave_sum(skl);
    float wmx = oi_wave_max(mx);
    const unsigned long long any_bad = __ballot(bad);
    if (any_bad) wmx = __builtin_nanf("");
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) {
        red[0][wave] = cnt;
        red[1][wave] = sd;
        red[2][wave] = sd2;
        red[3][wave] = skl;
        red[4][wave] = (double)wmx;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        double c = 0, a = 0, b = 0, k = 0, m = 0;
        bool nan_max = false;
        for (int w = 0; w < 16; ++w) {
            c += red[0][w];
            a += red[1][w];
            b += red[2][w];
            k += red[3][w];
            nan_max |= red[4][w] != red[4][w];
            m = red[4][w] > m ? red[4][w] : m;
        }
        double var = c > 1.0 ? (b - a * a / c) / (c - 1.0) : 0.0;
        var = var > 0.0 ? var : (var != var ? var : 0.0);
        out[0] = c > 0.0 ? (float)(a / c) : 0.f;
        out[1] = c > 0.0 ? (nan_max ? __builtin_nanf("") : (float)m) : 0.f;
        out[2] = c > 1.0 ? (float)sqrt(var) : 0.f;
        out[3] = c > 0.0 ? (float)(k / c) : 0.f;
    }
}

}  // namespace

extern "C" int oi_grpo_terms_fwd(const float* new_logprobs, const float* ratio, const float* advantages,
                                 const float* ref_logprobs, const float* rho_weights, int64_t n, int loss_fn,
                                 float ratio_lo, float ratio_hi, int kl_estimator, float* pg_loss, float* clipfrac,
                                 float* kl, void* stream) {
    OI_RETURN_IF(n < 0, OI_EINVAL);
    const int rc = check_cfg(loss_fn, kl_estimator);
    if (rc != OI_OK) return rc;
    if (n == 0) return OI_OK;
    OI_RETURN_IF(!new_logprobs || !ratio || !advantages || !rho_weights || !pg_loss || !clipfrac || !kl, OI_ENULL);
    const GrpoCfg c = {loss_fn, ratio_lo, ratio_hi, kl_estimator};
    hipLaunchKernelGGL(grpo_terms_fwd_kernel, dim3(blocks_for(n, 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       new_logprobs, ratio, advantages, ref_logprobs, rho_weights, n, c, pg_loss, clipfrac, kl);
    return oi_launch_status();
}

extern "C" int oi_grpo_terms_bwd(const float* new_logprobs, const float* ratio, const float* advantages,
                                 const float* ref_logprobs, const float* rho_weights, const float* grad_pg,
                                 const float* grad_kl, int64_t n, int loss_fn, float ratio_lo, float ratio_hi,
                                 int kl_estimator, float* d_new_logprobs, float* d_ratio, void* stream) {
    OI_RETURN_IF(n < 0, OI_EINVAL);
    const int rc = check_cfg(loss_fn, kl_estimator);
    if (rc != OI_OK) return rc;
    if (n == 0) return OI_OK;
    OI_RETURN_IF(!new_logprobs || !ratio || !advantages || !rho_weights, OI_ENULL);
    const GrpoCfg c = {loss_fn, ratio_lo, ratio_hi, kl_estimator};
    hipLaunchKernelGGL(grpo_terms_bwd_kernel, dim3(blocks_for(n, 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       new_logprobs, ratio, advantages, ref_logprobs, rho_weights, grad_pg, grad_kl, n, c,
                       d_new_logprobs, d_ratio);
    return oi_launch_status();
}

extern "C" size_t oi_grpo_fused_workspace_bytes(int64_t rows, int64_t cols) {
    if (rows <= 0 || cols <= 0) return 0;
    const int64_t nchunks = (cols + FUSED_CHUNK - 1) / FUSED_CHUNK;
    return (size_t)(rows * nchunks * NSUM) * sizeof(float);
}

namespace {
// Shared launch sequence of the statistics entry points: one block per (row, chunk), then one
// workgroup that adds the partial sums up in a fixed order.
int launch_grpo_stats(const StatIn& in, int64_t rows, int64_t cols, const GrpoCfg& c, float beta, int axis_mode,
                      float denominator, float scale, float* out_stats, int64_t out_stride, uint32_t write_mask,
                      float* row_denoms, float* partial, hipStream_t s) {
    const int64_t nchunks = (cols + FUSED_CHUNK - 1) / FUSED_CHUNK;
    hipLaunchKernelGGL(grpo_stats_partial_kernel, dim3((unsigned)(rows * nchunks)), dim3(FUSED_THREADS), 0, s, in,
                       cols, nchunks, c, beta, partial);
    hipLaunchKernelGGL(grpo_stats_final_kernel, dim3(1), dim3(256), 0, s, partial, rows, nchunks, axis_mode,
                       denominator, scale, beta, c.kl_est, out_stats, out_stride, write_mask, row_denoms);
    return oi_launch_status();
}

int check_stats_shape(int64_t rows, int64_t cols) {
    OI_RETURN_IF(rows <= 0 || cols <= 0, OI_EINVAL);
    const int64_t nchunks = (cols + FUSED_CHUNK - 1) / FUSED_CHUNK;
    OI_RETURN_IF(rows > 0x7fffffffLL / nchunks, OI_EINVAL);  // one block per (row, chunk)
    return OI_OK;
}
}  // namespace

extern "C" int oi_grpo_fused_fwd(const float* new_logprobs, const float* old_logprobs, const float* ref_logprobs,
                                 const float* advantages, const uint8_t* mask, const float* rho_weights,
                                 const float* entropy, const float* rho_drop_any, const float* rho_drop_low,
                                 const float* rho_drop_high, const float* rho_clipped, int64_t rows, int64_t cols,
                                 int loss_fn, float ratio_lo, float ratio_hi, int kl_estimator, float beta,
                                 int axis_mode, float denominator, float scale, float* out_stats, float* row_denoms,
                                 void* workspace, size_t workspace_bytes, void* stream) {
    int rc = check_stats_shape(rows, cols);
    if (rc != OI_OK) return rc;
    OI_RETURN_IF(axis_mode != 0 && axis_mode != 1, OI_EINVAL);
    rc = check_cfg(loss_fn, kl_estimator);
    if (rc != OI_OK) return rc;
    OI_RETURN_IF(!new_logprobs || !advantages || !mask || !out_stats || !row_denoms || !workspace, OI_ENULL);
    OI_RETURN_IF(workspace_bytes < oi_grpo_fused_workspace_bytes(rows, cols), OI_EWORKSPACE);
    const GrpoCfg c = {loss_fn, ratio_lo, ratio_hi, kl_estimator};
    const StatIn in = {new_logprobs, old_logprobs, ref_logprobs, advantages, rho_weights, nullptr, nullptr,
                       nullptr,      entropy,      rho_drop_any, rho_drop_low, rho_drop_high, rho_clipped, mask};
    return launch_grpo_stats(in, rows, cols, c, beta, axis_mode, denominator, scale, out_stats, 1, 0xffffu, row_denoms,
                             static_cast<float*>(workspace), static_cast<hipStream_t>(stream));
}

namespace {
std::mutex static_scratch_mutex;
float* static_scratch_of_device[64] = {};

// Address of oi_static_scratch on the current device, looked up once per device.
int static_scratch_ptr(float** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    OI_RETURN_IF(dev < 0 || dev >= 64, OI_EINVAL);
    std::lock_guard<std::mutex> lock(static_scratch_mutex);
    if (!static_scratch_of_device[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(oi_static_scratch));
        if (e != hipSuccess) return (int)e;
        OI_RETURN_IF(!p, OI_ENULL);
        static_scratch_of_device[dev] = static_cast<float*>(p);
    }
    *out = static_scratch_of_device[dev];
    return OI_OK;
}
}  // namespace

extern "C" int oi_grpo_fused_fwd_static(const float* new_logprobs, const float* old_logprobs,
                                        const float* ref_logprobs, const float* advantages, const uint8_t* mask,
                                        const float* rho_weights, const float* entropy, const float* rho_drop_any,
                                        const float* rho_drop_low, const float* rho_drop_high,
                                        const float* rho_clipped, int64_t rows, int64_t cols, int loss_fn,
                                        float ratio_lo, float ratio_hi, int kl_estimator, float beta, int axis_mode,
                                        float denominator, float scale, float* out_stats, float* row_denoms,
                                        void* stream) {
    static_assert(sizeof(oi_static_scratch) == sizeof(float) * OI_GRPO_STATIC_MAX_BLOCKS * NSUM, "scratch size");
    int rc = check_stats_shape(rows, cols);
    if (rc != OI_OK) return rc;
    OI_RETURN_IF(axis_mode != 0 && axis_mode != 1, OI_EINVAL);
    rc = check_cfg(loss_fn, kl_estimator);
    if (rc != OI_OK) return rc;
    OI_RETURN_IF(!new_logprobs || !advantages || !mask || !out_stats || !row_denoms, OI_ENULL);
    const int64_t nchunks = (cols + FUSED_CHUNK - 1) / FUSED_CHUNK;
    OI_RETURN_IF(rows * nchunks > OI_GRPO_STATIC_MAX_BLOCKS, OI_ETOOLARGE);
    float* partial = nullptr;
    rc = static_scratch_ptr(&partial);
    if (rc != OI_OK) return rc;
    // nothing in the array has to start at zero: the first kernel writes every partial sum that the
    // second one reads (rows * nchunks * NSUM floats), whatever an earlier call left there
    const GrpoCfg c = {loss_fn, ratio_lo, ratio_hi, kl_estimator};
    const StatIn in = {new_logprobs, old_logprobs, ref_logprobs, advantages, rho_weights, nullptr, nullptr,
                       nullptr,      entropy,      rho_drop_any, rho_drop_low, rho_drop_high, rho_clipped, mask};
    return launch_grpo_stats(in, rows, cols, c, beta, axis_mode, denominator, scale, out_stats, 1, 0xffffu, row_denoms,
                             partial, static_cast<hipStream_t>(stream));
}

extern "C" int oi_grpo_stats_from_terms(const float* pg_loss, const float* clipfrac, const float* ratio,
                                        const float* new_logprobs, const float* ref_logprobs, const uint8_t* mask,
                                        const float* entropy, const float* rho_weight, const float* rho_drop_any,
                                        const float* rho_drop_low, const float* rho_drop_high,
                                        const float* rho_clipped, int64_t rows, int64_t cols, int kl_estimator,
                                        float beta, float* out_stats, int64_t out_stride, uint32_t write_mask,
                                        void* workspace, size_t workspace_bytes, void* stream) {
    int rc = check_stats_shape(rows, cols);
    if (rc != OI_OK) return rc;
    OI_RETURN_IF(kl_estimator < 0 || kl_estimator > 3 || out_stride < 1, OI_EINVAL);
    OI_RETURN_IF(!pg_loss || !clipfrac || !ratio || !mask || !out_stats || !workspace, OI_ENULL);
    OI_RETURN_IF(ref_logprobs && !new_logprobs, OI_ENULL);
    OI_RETURN_IF(workspace_bytes < oi_grpo_fused_workspace_bytes(rows, cols), OI_EWORKSPACE);
    const GrpoCfg c = {OI_LOSS_DAPO, 0.f, 0.f, kl_estimator};
    const StatIn in = {new_logprobs, nullptr, ref_logprobs, nullptr,      rho_weight,   pg_loss,       clipfrac,
                       ratio,        entropy, rho_drop_any, rho_drop_low, rho_drop_high, rho_clipped, mask};
    // the loss itself belongs to the caller here: entry 0 is never written
    return launch_grpo_stats(in, rows, cols, c, beta, 0, 0.f, 1.f, out_stats, out_stride, write_mask & 0xfffeu,
                             nullptr, static_cast<float*>(workspace), static_cast<hipStream_t>(stream));
}

extern "C" int oi_grpo_fused_bwd(const float* new_logprobs, const float* old_logprobs, const float* ref_logprobs,
                                 const float* advantages, const uint8_t* mask, const float* rho_weights, int64_t rows,
                                 int64_t cols, int loss_fn, float ratio_lo, float ratio_hi, int kl_estimator,
                                 float beta, float scale, const float* row_denoms, const float* grad_loss,
                                 float* d_new_logprobs, void* stream) {
    OI_RETURN_IF(rows <= 0 || cols <= 0, OI_EINVAL);
    const int rc = check_cfg(loss_fn, kl_estimator);
    if (rc != OI_OK) return rc;
    OI_RETURN_IF(!new_logprobs || !advantages || !mask || !row_denoms || !d_new_logprobs, OI_ENULL);
    const GrpoCfg c = {loss_fn, ratio_lo, ratio_hi, kl_estimator};
    hipLaunchKernelGGL(grpo_fused_bwd_kernel, dim3(blocks_for(rows * cols, 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), new_logprobs, old_logprobs, ref_logprobs, advantages, mask,
                       rho_weights, rows, cols, c, beta, scale, row_denoms, grad_loss, d_new_logprobs);
    return oi_launch_status();
}

extern "C" int oi_group_advantages(const double* scores, int64_t n_groups, int64_t group_size, int mode,
                                   float* advantages, void* stream) {
    OI_RETURN_IF(n_groups < 0 || group_size <= 0 || (mode != 0 && mode != 1), OI_EINVAL);
    if (n_groups == 0) return OI_OK;
    OI_RETURN_IF(!scores || !advantages, OI_ENULL);
    hipLaunchKernelGGL(group_adv_kernel, dim3(blocks_for(n_groups, 64)), dim3(64), 0, static_cast<hipStream_t>(stream),
                       scores, n_groups, group_size, mode, advantages);
    return oi_launch_status();
}

extern "C" size_t oi_masked_mean_workspace_bytes(int64_t extra, int64_t rows, int64_t cols) {
    if (extra <= 0 || rows <= 0 || cols <= 0) return 0;
    const int64_t nchunks = (cols + FUSED_CHUNK - 1) / FUSED_CHUNK;
    return (size_t)((extra + 1) * rows * nchunks) * sizeof(float);
}

extern "C" int oi_masked_mean_fwd(const float* values, const void* mask, int mask_is_float, int64_t extra,
                                  int64_t rows, int64_t cols, int axis_mode, float denominator, float* out,
                                  float* row_denoms, void* workspace, size_t workspace_bytes, void* stream) {
    OI_RETURN_IF(extra <= 0 || rows <= 0 || cols <= 0 || extra > 65535, OI_EINVAL);
    OI_RETURN_IF(axis_mode != 0 && axis_mode != 1, OI_EINVAL);
    OI_RETURN_IF(!values || !mask || !out || !workspace, OI_ENULL);
    OI_RETURN_IF(workspace_bytes < oi_masked_mean_workspace_bytes(extra, rows, cols), OI_EWORKSPACE);
    const int64_t nchunks = (cols + FUSED_CHUNK - 1) / FUSED_CHUNK;
    OI_RETURN_IF(rows > 0x7fffffffLL / nchunks / extra, OI_EINVAL);  // one block per (extra, row, chunk)
    float* partial = static_cast<float*>(workspace);
    float* cnt = partial + extra * rows * nchunks;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(masked_partial_kernel, dim3((unsigned)(extra * rows * nchunks)), dim3(FUSED_THREADS), 0, s,
                       values, mask, mask_is_float, rows, cols, nchunks, partial, cnt);
    hipLaunchKernelGGL(masked_final_kernel, dim3((unsigned)extra), dim3(256), 0, s, partial, cnt, rows, nchunks,
                       axis_mode, denominator, out, row_denoms);
    return oi_launch_status();
}

extern "C" int oi_masked_mean_bwd(const float* grad_out, const void* mask, int mask_is_float, const float* row_denoms,
                                  int64_t extra, int64_t rows, int64_t cols, float* d_values, void* stream) {
    OI_RETURN_IF(extra <= 0 || rows <= 0 || cols <= 0, OI_EINVAL);
    OI_RETURN_IF(!grad_out || !mask || !row_denoms || !d_values, OI_ENULL);
    hipLaunchKernelGGL(masked_bwd_kernel, dim3(blocks_for(extra * rows * cols, 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), grad_out, mask, mask_is_float, row_denoms, extra, rows, cols,
                       d_values);
    return oi_launch_status();
}

extern "C" int oi_seq_logp_fwd(const float* per_token_logps, const int64_t* labels, const int32_t* cu_seq_lens,
                               int64_t n_seqs, int64_t total, int average, float* out, float* counts, void* stream) {
    OI_RETURN_IF(n_seqs < 0 || total < 1, OI_EINVAL);
    if (n_seqs == 0) return OI_OK;
    OI_RETURN_IF(!per_token_logps || !labels || !out, OI_ENULL);
    hipLaunchKernelGGL(seq_logp_fwd_kernel, dim3((unsigned)n_seqs), dim3(256), 0, static_cast<hipStream_t>(stream),
                       per_token_logps, labels, cu_seq_lens, n_seqs, total, average, out, counts);
    return oi_launch_status();
}

extern "C" int oi_seq_logp_bwd(const float* grad_out, const int64_t* labels, const int32_t* cu_seq_lens,
                               const float* counts, int64_t n_seqs, int64_t total, int average,
                               float* d_per_token_logps, void* stream) {
    OI_RETURN_IF(n_seqs < 0 || total < 1, OI_EINVAL);
    if (n_seqs == 0) return OI_OK;
    OI_RETURN_IF(!grad_out || !labels || !d_per_token_logps, OI_ENULL);
    OI_RETURN_IF(average && !counts, OI_ENULL);
    hipLaunchKernelGGL(seq_logp_bwd_kernel, dim3((unsigned)n_seqs), dim3(256), 0, static_cast<hipStream_t>(stream),
                       grad_out, labels, cu_seq_lens, counts, n_seqs, total, average, d_per_token_logps);
    return oi_launch_status();
}

extern "C" int oi_dpo_sigmoid_fwd(const float* policy_chosen, const float* policy_rejected, const float* ref_chosen,
                                  const float* ref_rejected, const float* weights, int64_t n_pairs, float beta,
                                  float label_smoothing, float margin, float* losses, float* chosen_rewards,
                                  float* rejected_rewards, void* stream) {
    OI_RETURN_IF(n_pairs < 0, OI_EINVAL);
    if (n_pairs == 0) return OI_OK;
    OI_RETURN_IF(!policy_chosen || !policy_rejected || !losses, OI_ENULL);
    hipLaunchKernelGGL(dpo_fwd_kernel, dim3(blocks_for(n_pairs, 64)), dim3(64), 0, static_cast<hipStream_t>(stream),
                       policy_chosen, policy_rejected, ref_chosen, ref_rejected, weights, n_pairs, beta,
                       label_smoothing, margin, losses, chosen_rewards, rejected_rewards);
    return oi_launch_status();
}

extern "C" int oi_dpo_sigmoid_bwd(const float* policy_chosen, const float* policy_rejected, const float* ref_chosen,
                                  const float* ref_rejected, const float* weights, const float* grad_losses,
                                  int64_t n_pairs, float beta, float label_smoothing, float margin,
                                  float* d_policy_chosen, float* d_policy_rejected, void* stream) {
    OI_RETURN_IF(n_pairs < 0, OI_EINVAL);
    if (n_pairs == 0) return OI_OK;
    OI_RETURN_IF(!policy_chosen || !policy_rejected || !grad_losses, OI_ENULL);
    hipLaunchKernelGGL(dpo_bwd_kernel, dim3(blocks_for(n_pairs, 64)), dim3(64), 0, static_cast<hipStream_t>(stream),
                       policy_chosen, policy_rejected, ref_chosen, ref_rejected, weights, grad_losses, n_pairs, beta,
                       label_smoothing, margin, d_policy_chosen, d_policy_rejected);
    return oi_launch_status();
}


extern "C" int oi_estimate_kl_fwd(const float* ref_logprobs_diff, const float* ratio, int64_t n, float* out,
                                  void* stream) {
    OI_RETURN_IF(n < 0, OI_EINVAL);
    if (n == 0) return OI_OK;
    OI_RETURN_IF(!ref_logprobs_diff || !ratio || !out, OI_ENULL);
    hipLaunchKernelGGL(estimate_kl_fwd_kernel, dim3(blocks_for(n, 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), ref_logprobs_diff, ratio, n, out);
    return oi_launch_status();
}

extern "C" int oi_estimate_kl_bwd(const float* ref_logprobs_diff, const float* ratio, const float* grad_out, int64_t n,
                                  float* d_diff, float* d_ratio, void* stream) {
    OI_RETURN_IF(n < 0, OI_EINVAL);
    if (n == 0) return OI_OK;
    OI_RETURN_IF(!ref_logprobs_diff || !ratio || !grad_out, OI_ENULL);
    hipLaunchKernelGGL(estimate_kl_bwd_kernel, dim3(blocks_for(n, 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), ref_logprobs_diff, ratio, grad_out, n, d_diff, d_ratio);
    return oi_launch_status();
}

extern "C" int oi_mask_logprobs_fwd(const float* logprobs, const uint8_t* mask, int64_t n, float fill, float* out,
                                    void* stream) {
    OI_RETURN_IF(n < 0, OI_EINVAL);
    if (n == 0) return OI_OK;
    OI_RETURN_IF(!logprobs || !mask || !out, OI_ENULL);
    hipLaunchKernelGGL(mask_logprobs_kernel, dim3(blocks_for(n, 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       logprobs, mask, n, fill, out);
    return oi_launch_status();
}

extern "C" int oi_mask_logprobs_bwd(const float* logprobs, const uint8_t* mask, const float* grad_out, int64_t n,
                                    float* d_logprobs, void* stream) {
    OI_RETURN_IF(n < 0, OI_EINVAL);
    if (n == 0) return OI_OK;
    OI_RETURN_IF(!logprobs || !mask || !grad_out || !d_logprobs, OI_ENULL);
    hipLaunchKernelGGL(mask_logprobs_bwd_kernel, dim3(blocks_for(n, 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), logprobs, mask, grad_out, n, d_logprobs);
    return oi_launch_status();
}

extern "C" int oi_rho_correction(const float* old_logprobs, const float* vllm_logprobs, const uint8_t* mask,
                                 const float* advantages, int64_t rows, int64_t cols, int sequence_level,
                                 int tv_divergence, float mask_lower, float mask_upper, float clamp_lower,
                                 float clamp_upper, float* rho, float* weights, float* drop_any, float* drop_low,
                                 float* drop_high, float* clipped, void* stream) {
    OI_RETURN_IF(rows < 0 || cols < 0 || rows > 0x7fffffffLL, OI_EINVAL);
    if (rows == 0 || cols == 0) return OI_OK;
    OI_RETURN_IF(!old_logprobs || !vllm_logprobs || !mask || !advantages, OI_ENULL);
    OI_RETURN_IF(!rho || !weights || !drop_any || !drop_low || !drop_high || !clipped, OI_ENULL);
    const RhoCfg c = {sequence_level, tv_divergence, mask_lower, mask_upper, clamp_lower, clamp_upper};
    hipLaunchKernelGGL(rho_correction_kernel, dim3((unsigned)rows), dim3(256), 0, static_cast<hipStream_t>(stream),
                       old_logprobs, vllm_logprobs, mask, advantages, cols, c, rho, weights, drop_any, drop_low,
                       drop_high, clipped);
    return oi_launch_status();
}

extern "C" int oi_logprob_diff_stats(const float* local_logprobs, const float* other_logprobs, const uint8_t* mask,
                                     int64_t n, float* out_stats, void* stream) {
    OI_RETURN_IF(n < 0, OI_EINVAL);
    OI_RETURN_IF(!out_stats, OI_ENULL);
    OI_RETURN_IF(n > 0 && (!local_logprobs || !other_logprobs || !mask), OI_ENULL);
    hipLaunchKernelGGL(logprob_diff_stats_kernel, dim3(1), dim3(1024), 0, static_cast<hipStream_t>(stream),
                       local_logprobs, other_logprobs, mask, n, out_stats);
    return oi_launch_status();
}

extern "C" int oi_version(void) { return 1200; }

extern "C" const char* oi_error_string(int code) {
    switch (code) {
        case OI_OK: return "ok";
        case OI_EINVAL: return "a size or scalar argument is out of range";
        case OI_ENULL: return "a required pointer is NULL";
        case OI_EALIGN: return "pointer or stride alignment is not met";
        case OI_EDTYPE: return "unknown or unsupported dtype tag";
        case OI_EWORKSPACE: return "workspace is too small";
        case OI_ETOOLARGE: return "problem is larger than the static scratch of this entry point";
        default: return code > 0 ? "HIP launch error (value is a hipError_t)" : "unknown error code";
    }
}

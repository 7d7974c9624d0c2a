// Per-token GRPO arithmetic shared by the loss kernels and the fused logits kernel: forward terms
// and partial derivatives with the exact branch semantics of torch.clamp / torch.maximum.
#pragma once

#include "oi_common.h"

namespace {

struct GrpoCfg {
    int loss_fn;
    float lo, hi;
    int kl_est;
};

// torch.clamp keeps NaN; written with comparisons so that NaN falls through unchanged
__device__ __forceinline__ float clamp_keep_nan(float x, float lo, float hi) { return x < lo ? lo : (x > hi ? hi : x); }
// torch.maximum returns NaN if either side is NaN
__device__ __forceinline__ float max_keep_nan(float a, float b) { return (a >= b || a != a) ? a : b; }

struct GrpoOut {
    float pg, clipfrac, kl[4];
};

// Forward terms for one token (compute_grpo_loss + estimate_kl of the reference).
__device__ __forceinline__ GrpoOut grpo_token_fwd(float nlp, float ratio, float adv, bool has_ref, float ref, float w,
                                                  const GrpoCfg& c) {
    GrpoOut o;
    if (c.loss_fn == OI_LOSS_DAPO) {
        const float plain = -adv * ratio;
        const float clipped = -adv * clamp_keep_nan(ratio, c.lo, c.hi);
        o.clipfrac = clipped > plain ? 1.f : 0.f;
        o.pg = max_keep_nan(plain, clipped);
    } else {
        o.clipfrac = ratio > c.hi ? 1.f : 0.f;
        o.pg = -adv * (ratio > c.hi ? c.hi : ratio) * nlp;
    }
    o.pg *= w;
    o.clipfrac *= (w != 0.f) ? 1.f : 0.f;
    if (has_ref) {
        const float d = clamp_keep_nan(nlp - ref, -40.f, 40.f);
        o.kl[0] = d;
        o.kl[1] = d * d / 2.f;
        o.kl[2] = expm1f(-d) + d;
        o.kl[3] = ratio * d;
    } else {
        o.kl[0] = o.kl[1] = o.kl[2] = o.kl[3] = 0.f;
    }
    return o;
}

// Partial derivatives for one token:
//   dpg_dratio, dpg_dnew: of pg (after the rho weight); dkl_dnew, dkl_dratio: of the selected KL.
// torch.maximum sends half of the gradient to each side on a tie and torch.clamp passes the
// gradient on the closed interval [lo, hi]; inside the clip range both DAPO branches are equal, so
// the two halves add up to the full -A.
struct GrpoGrad {
    float dpg_dratio, dpg_dnew, dkl_dnew, dkl_dratio;
};

__device__ __forceinline__ GrpoGrad grpo_token_bwd(float nlp, float ratio, float adv, bool has_ref, float ref, float w,
                                                   const GrpoCfg& c) {
    GrpoGrad g = {0.f, 0.f, 0.f, 0.f};
    if (c.loss_fn == OI_LOSS_DAPO) {
        const float plain = -adv * ratio;
        const float clipped = -adv * clamp_keep_nan(ratio, c.lo, c.hi);
        const float inr = (ratio >= c.lo && ratio <= c.hi) ? 1.f : 0.f;
        float coef;
        if (plain > clipped) coef = 1.f;
        else if (plain == clipped) coef = 0.5f + 0.5f * inr;
        else coef = inr;
        g.dpg_dratio = -adv * coef * w;
    } else {
        g.dpg_dnew = -adv * (ratio > c.hi ? c.hi : ratio) * w;
    }
    if (has_ref) {
        const float raw = nlp - ref;
        const float inside = (raw >= -40.f && raw <= 40.f) ? 1.f : 0.f;
        const float d = clamp_keep_nan(raw, -40.f, 40.f);
        switch (c.kl_est) {
            case 0: g.dkl_dnew = inside; break;
            case 1: g.dkl_dnew = d * inside; break;
            case 2: g.dkl_dnew = -expm1f(-d) * inside; break;
            default:
                g.dkl_dnew = ratio * inside;
                g.dkl_dratio = d;
                break;
        }
    }
    return g;
}

// d loss_token / d new_logprob for one token, with ratio = exp(new - old) folded in
__device__ __forceinline__ float grpo_token_dnew(float nlp, float ratio, float adv, bool has_ref, float ref, float w,
                                                 const GrpoCfg& c, float beta) {
    const GrpoGrad g = grpo_token_bwd(nlp, ratio, adv, has_ref, ref, w, c);
    return (g.dpg_dratio + beta * g.dkl_dratio) * ratio + g.dpg_dnew + beta * g.dkl_dnew;
}

}  // namespace

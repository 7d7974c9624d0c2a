// Packing of query/response token sequences into training rows for gfx950: pure integer / byte
// movement, one workgroup per sequence, coalesced 8-byte stores into seven per-token arrays.
#include "oi_common.h"

namespace {

constexpr int PACK_THREADS = 256;

// Sequence i = query i (copied as is) followed by the response with its padding tokens dropped
// (stable compaction).  All per-token outputs of the sequence start at dst_offsets[i].
__global__ void __launch_bounds__(PACK_THREADS)
    pack_scatter_kernel(const int64_t* __restrict__ q_tokens, const int64_t* __restrict__ q_offsets,
                        const int64_t* __restrict__ r_tokens, const int64_t* __restrict__ r_offsets,
                        const uint8_t* __restrict__ r_tool_mask, const float* __restrict__ r_logprobs,
                        const float* __restrict__ advantages, const int64_t* __restrict__ dst_offsets,
                        const int32_t* __restrict__ mask_base, int64_t pad_token_id, int mask_tool_use,
                        int64_t* __restrict__ query_responses, int64_t* __restrict__ attention_masks,
                        int64_t* __restrict__ position_ids, int64_t* __restrict__ response_masks,
                        int64_t* __restrict__ dones, float* __restrict__ vllm_logprobs,
                        float* __restrict__ out_advantages) {
    __shared__ int wave_count[PACK_THREADS / OI_WAVE];
    const int64_t i = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t q0 = q_offsets[i], qn = q_offsets[i + 1] - q0;
    const int64_t r0 = r_offsets[i], rn = r_offsets[i + 1] - r0;
    const int64_t dst = dst_offsets[i];
    const int64_t doc = i + 1;
    const int64_t att = doc - (int64_t)mask_base[i];
    const float adv = advantages ? advantages[i] : 0.f;
    const float nan = __builtin_nanf("");

    for (int64_t j = tid; j < qn; j += PACK_THREADS) {
        const int64_t o = dst + j;
        query_responses[o] = q_tokens[q0 + j];
        attention_masks[o] = att;
        position_ids[o] = j;
        response_masks[o] = 0;
        dones[o] = 0;
        vllm_logprobs[o] = nan;
        if (out_advantages) out_advantages[o] = 0.f;
    }

    // response: keep tokens != pad, in order; `kept` = tokens kept by earlier chunks
    int64_t kept = 0;
    for (int64_t base = 0; base < rn; base += PACK_THREADS) {
        const int64_t j = base + tid;
        const bool in = j < rn;
        const int64_t tok = in ? r_tokens[r0 + j] : pad_token_id;
        const bool keep = in && tok != pad_token_id;
        const unsigned long long ballot = __ballot(keep);
        const int before_in_wave = __popcll(ballot & ((1ull << lane) - 1ull));
        __syncthreads();  // wave_count of the previous chunk has been read by everyone
        if (lane == 0) wave_count[wave] = __popcll(ballot);
        __syncthreads();
        int before = before_in_wave, total = 0;
#pragma unroll
        for (int w = 0; w < PACK_THREADS / OI_WAVE; ++w) {
            const int c = wave_count[w];
            before += w < wave ? c : 0;
            total += c;
        }
        if (keep) {
            const int64_t pos = qn + kept + before;  // position inside the sequence
            const int64_t o = dst + pos;
            const bool scored = !mask_tool_use || r_tool_mask[r0 + j] != 0;
            query_responses[o] = tok;
            attention_masks[o] = att;
            position_ids[o] = pos;
            response_masks[o] = scored ? doc : 0;
            dones[o] = 0;
            vllm_logprobs[o] = r_logprobs[r0 + j];
            if (out_advantages) out_advantages[o] = scored ? adv : 0.f;
        }
        kept += total;
    }
    // the last token of the sequence carries the sequence id in `dones`
    __syncthreads();
    if (tid == 0 && qn + kept > 0) dones[dst + qn + kept - 1] = doc;
}

}  // namespace

extern "C" int oi_pack_sequences(const int64_t* q_tokens, const int64_t* q_offsets, const int64_t* r_tokens,
                                 const int64_t* r_offsets, const uint8_t* r_tool_mask, const float* r_logprobs,
                                 const float* advantages, const int64_t* dst_offsets, const int32_t* mask_base,
                                 int64_t n_seqs, int64_t pad_token_id, int mask_tool_use, int64_t* query_responses,
                                 int64_t* attention_masks, int64_t* position_ids, int64_t* response_masks,
                                 int64_t* dones, float* vllm_logprobs, float* out_advantages, void* stream) {
    OI_RETURN_IF(n_seqs < 0 || n_seqs > 0x7fffffffLL, OI_EINVAL);
    if (n_seqs == 0) return OI_OK;
    OI_RETURN_IF(!q_tokens || !q_offsets || !r_tokens || !r_offsets || !r_logprobs || !dst_offsets || !mask_base,
                 OI_ENULL);
    OI_RETURN_IF(mask_tool_use && !r_tool_mask, OI_ENULL);
    OI_RETURN_IF(!query_responses || !attention_masks || !position_ids || !response_masks || !dones || !vllm_logprobs,
                 OI_ENULL);
    OI_RETURN_IF((advantages == nullptr) != (out_advantages == nullptr), OI_ENULL);
    hipLaunchKernelGGL(pack_scatter_kernel, dim3((unsigned)n_seqs), dim3(PACK_THREADS), 0,
                       static_cast<hipStream_t>(stream), q_tokens, q_offsets, r_tokens, r_offsets, r_tool_mask,
                       r_logprobs, advantages, dst_offsets, mask_base, pad_token_id, mask_tool_use, query_responses,
                       attention_masks, position_ids, response_masks, dones, vllm_logprobs, out_advantages);
    return oi_launch_status();
}

"""CPU oracle for the policy-loss hot path of allenai/open-instruct.

TEST INFRASTRUCTURE ONLY.  This package restates, with stock ``torch`` CPU routines, the
arithmetic of the reference functions listed below.  It exists so that the HIP kernels can be
checked against the reference's results.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it; the product package never does and fails loudly
when its HIP library is missing.

Reference functions restated (paths relative to the reference checkout):

=============================  =====================================================  ==========
oracle function                reference                                              pinned by
=============================  =====================================================  ==========
logprob.log_softmax_and_gather open_instruct/model_utils.py:587-600                   brute force Python loops; shift invariance; sum_j exp(logp_j)=1; reference test invariants (test_model_utils.py:49-64)
logprob.entropy_from_logits    open_instruct/model_utils.py:326-333                   closed forms (uniform -> ln V, one-hot -> 0), -sum p ln p brute force
logprob.estimate_kl            open_instruct/model_utils.py:793-818                   closed forms (d=0 -> 0, k3>=0, Taylor d^2/2), math.expm1 brute force
logprob.calculate_per_token_logps  open_instruct/padding_free_collator.py:10-16        brute force with explicit shift; reference DPOLMHead identity (test_padding_free_collator.py:366-386)
reductions.masked_mean         open_instruct/rl_utils.py:426-448                      six reference known-answer tests (test_rl_utils.py:341-412)
reductions.get_batch_logps_padded  open_instruct/dpo_utils.py:689-712                  two reference known-answer vectors (test_dpo_utils.py:95-110)
reductions.get_batch_logps_packed  open_instruct/padding_free_collator.py:202-229      packed == padded equivalence, brute-force segment loop, reference all-masked-segment test (test_padding_free_collator.py:334-346)
grpo.mask_logprobs             open_instruct/grpo_utils.py:340-344                    all-masked => INVALID_LOGPROB (test_olmo_core_train_modules.py:49-82)
grpo.compute_rho_correction    open_instruct/grpo_utils.py:372-463                    three reference known-answer tests (test_olmo_core_train_modules.py:305-371)
grpo.compute_grpo_loss         open_instruct/grpo_utils.py:504-538                    reference known-answer tests (test_olmo_core_train_modules.py:135-152,200-303,373-402) + branch grid in fp64
grpo.group_advantages          open_instruct/data_loader.py:1472-1484                 numpy.std(ddof=0) library routine; zero-variance group -> exact 0
grpo.grpo_token_loss           open_instruct/grpo_fast.py:702-724                     composition of the pinned functions above
dpo.dpo_loss                   open_instruct/dpo_utils.py:523-563                     closed forms (x=0 -> ln 2, L(x,ls)=L(-x,1-ls)), math.log1p brute force; reference tests (test_dpo_utils.py:30-88)
dpo.simpo_loss / dpo.wpo_loss  open_instruct/dpo_utils.py:566-642                     closed forms only (no reference known-answer vector)
lm_head.lm_head_logprobs       HF nn.Linear lm_head + padding_free_collator.py:10-16  textbook F.linear in fp32/fp64 (the GEMM itself lives in third-party code; no reference vector)
lm_head.linear_cross_entropy   open_instruct/finetune.py:818-824 (HF ForCausalLMLoss)    transformers.loss.loss_utils.ForCausalLMLoss itself (the third-party routine the reference calls), brute force
grpo.populate_sample_loss_stats  open_instruct/grpo_utils.py:674-742                   hand-computed table (tests/test_oracle_pins.py): means of three tokens by hand, untouched keys stay 0, weighted mean / variance by hand
grpo.compute_vllm_local_debug_metrics  open_instruct/grpo_utils.py:345-369             pure-Python math / statistics.stdev brute force; empty and single-token masks
packing.pack_sequences         open_instruct/rl_utils.py:215-375                      reference known-answer vectors (test_rl_utils.py:125-158), reference test properties (test_rl_utils.py:98-123,299-334)
packing.broadcast_advantages   open_instruct/data_loader.py:1509-1514                 hand-written example
=============================  =====================================================  ==========

Every gradient is taken by ``torch.autograd`` on these restatements (fp64 ``gradcheck`` in
``tests/``); the reference defines no backward code of its own.
"""

from oracle import dpo, grpo, lm_head, logprob, packing, reductions  # noqa: F401

INVALID_LOGPROB = 1.0  # open_instruct/utils.py:83
IGNORE_LABEL = -100  # open_instruct/dpo_utils.py:62

"""CPU oracle for the per-token RL loss path.  TEST INFRASTRUCTURE ONLY.

This package is a plain torch/numpy restatement, on the CPU, of the arithmetic that the
reference (sii-research/siiRL) performs on its per-token loss path.  It exists so that the
HIP kernels in ``siirl_amd`` can be checked against an independent statement of the same
maths on the same seeded inputs.  It is never part of the product:

* only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``
  may import it, and there only as the checker (or as the thing timed on the host cores);
* nothing under ``siirl_amd/`` imports it, and ``siirl_amd`` has no CPU fallback: without the
  HIP library its ops raise.

Every function cites the reference ``file:line`` it follows.  The reference package itself is
not importable in the build container (its dependencies ``loguru``, ``omegaconf``, ``hydra``,
``tensordict`` and ``ray`` are absent), so nothing here imports it.

How each function is pinned (see ``tests/test_oracle_*.py``):

=====================================  ==========================================================
function                               pinned by
=====================================  ==========================================================
logprobs_from_logits                   ``-F.cross_entropy``; ``log_softmax().gather()``; fp64
                                       brute force; shift invariance; uniform row -> -log V
entropy_from_logits                    ``torch.distributions.Categorical.entropy``; uniform ->
                                       log V; two equal logits -> log 2; bounds 0 <= H <= log V
logprob_entropy_backward               ``torch.autograd.grad`` on the fp64 forward;
                                       ``gradcheck``; rows of the gradient sum to zero
masked_sum / masked_mean               direct arithmetic on hand-written cases
compute_grpo_outcome_advantage         brute-force dict loop; unbiased-std known answers
                                       1.78885 / -0.73030 logged in the reference's quickstart
                                       (docs/start/quickstart.rst:137); group sums are zero
agg_loss                               four closed forms on hand-written cases
compute_policy_loss_vanilla / _gspo    hand-computed cases at ratio = 1, 1 +- eps, c, |d| = 20;
                                       closed-form gradient vs autograd; GSPO with L = 1 == PPO
compute_gae_advantage_return           gamma = lam = 1 -> reward-to-go minus value; lam = 0 -> TD
                                       error; brute-force double sum; padding == truncation;
                                       interior masked tokens == deleted columns; whitened
                                       selection has mean 0 / unbiased variance 1 (numpy)
masked_var / masked_whiten             numpy mean / var(ddof) of the selected elements; the two
                                       ValueErrors
pf_ppo_weights /                       the three weightings by hand (|s|^p, 1 at max and min,
compute_pf_ppo_reweight_data           0.4 / 0.1); one draw indexes tensors, arrays, lists and
                                       meta lists alike; the input is left alone
marft_gae_unwhitened /                 a two-agent, two-step request worked by hand (float and
compute_marft_gae_advantage_return     truncated outputs); single agent == the GAE scan above;
                                       gamma = lam = 1 -> rewards met so far minus value; keys
                                       written, id list growth, dtypes and the four errors
compute_value_loss                     hand-computed cases either side of the clip range; zero
                                       gradient where clipped
compute_policy_loss_cpgd / drift       hand-computed tokens with log(1 +- eps) bounds; gradient
                                       vanishes exactly on the clipped fraction; detached weight
compute_policy_loss_gpg                identity with agg_loss(-lp * A [* w])
compute_policy_loss_geo_mean           explicit product of token ratios ** (1 / L); L = 1 cases
                                       for each clipping side; weights as their geometric mean
compute_policy_loss_kl_cov             worked case with math (covariances, the picked token, loss);
                                       brute-force sort of the products; closed-form gradient
compute_policy_loss_clip_cov           candidate set by hand; loss after a given draw with math;
                                       generator state shows one randperm(len(candidates)); no
                                       candidates -> the plain clip loss
compute_cpgd_outcome_advantage         the GRPO oracle (STD_weight, naive); hand case for
                                       clip_filter_like_weight
kl_penalty                             closed forms per mode; k3 >= 0; straight-through identities
apply_kl_penalty / KL controllers      hand-computed controller step
dynamic_sampling_keep_indices          worked example of the reference's docs
                                       (docs/user_interface/filter_interface.rst:72-77); brute force
make_uid / filter_by_indices           uid layout and ordered index select pinned by the
                                       reference's tests (tests/dag_worker/test_dapo_pipeline.py:14-49,
                                       tests/dag_worker/test_dapo_merge.py:90-120)
unpad_input / pad_input / ...          transformers' pure-torch restatement of bert_padding
                                       (modeling_flash_attention_utils._unpad_input / _pad_input);
                                       pad(unpad(x)) == x * mask; hand-written left/right padding
compute_data_metric                    numpy mean / max / min / var(ddof=1) of the selected elements
                                       on seeded inputs; hand-written lengths and clip ratios
merge_leftover / place_outcome_reward  the reference's leftover-cache test vectors
                                       (tests/dag_worker/test_dapo_pipeline.py:145-195); hand-computed
                                       penalties either side of the expected length
micro_batch_step                       closed-form uniform-logits case written out with ``math``; a
                                       torch-free scalar restatement of dp_actor.py:425-513: equal
                                       loss, ``dlogits`` == its central differences (vanilla with
                                       every aggregation, gspo, cpgd + drift, entropy / KL terms,
                                       importance weights, on-policy); metric scalings
compute_entropy_loss                   uniform rows -> log V under each aggregation;
                                       ``Categorical.entropy`` aggregated by hand
fused_linear_for_ppo_fwd / _bwd        equals logprob/entropy of ``(h @ W.T)/T`` in fp64 and
                                       autograd through that expression
=====================================  ==========================================================

Parity unpinned (third-party arithmetic absent from the reference tree, no fixture in the
reference's tests): the exact rounding of flash-attn's Triton ``cross_entropy_loss`` (the
reference's CUDA dispatch target for ``logprobs_from_logits``) and of the Triton kernels in
``siirl/utils/kernel/kernels.py``.  The oracle states their published algorithm (fp32
log-softmax / online softmax) instead.
"""

from . import torch_functional, core_algos, dapo_filter, fused_linear, actor_step, padding, metric_utils  # noqa: F401

"""siirl_amd -- the per-token RL loss path of siiRL as hand-written HIP kernels for MI355X (gfx950).

The kernels live in ``csrc/`` and are reached through the C ABI of ``include/siirl_hip.h``
(``lib/libsiirl_hip.so``).  The Python modules mirror the reference's callables:

* ``siirl_amd.torch_functional`` -- ``logprobs_from_logits``, ``entropy_from_logits``, ``masked_mean`` ...
  (reference ``siirl/utils/model_utils/torch_functional.py``)
* ``siirl_amd.core_algos`` -- ``compute_grpo_outcome_advantage``, ``compute_policy_loss_vanilla`` / ``_gspo``,
  ``agg_loss``, ``kl_penalty``, the two registries (reference ``siirl/dag_worker/core_algos.py``)

There is no CPU path: the ops need CUDA(HIP) tensors and the built library, and raise otherwise.
"""

__version__ = "0.1.0"

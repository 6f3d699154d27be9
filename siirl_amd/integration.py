"""Installs the package's functions over the reference's module globals, for a deployment that does not want to
touch the reference's import lines.

``patch_reference(ref_torch_functional, ref_core_algos)`` takes the two already imported reference modules
(``siirl.utils.model_utils.torch_functional`` and ``siirl.dag_worker.core_algos``) -- or any objects with those
attributes -- and replaces, by name, only the functions whose every caller in the reference hands them device
tensors of the actor's micro-batch:

* ``logprobs_from_logits``, ``entropy_from_logits``, ``entropy_from_logits_with_chunking``
  (``siirl/engine/actor/dp_actor.py:75-84,179-195,254-260``);
* ``agg_loss``, ``kl_penalty``, ``compute_policy_loss`` and the seven registered policy losses
  (``compute_policy_loss_vanilla`` / ``_gspo`` / ``_cpgd`` / ``_gpg`` / ``_clip_cov`` / ``_kl_cov`` / ``_geo_mean``) with
  their registry entries (``dp_actor.py:453-486``).  Three of the reference's own (``clip_cov``, ``kl_cov``,
  ``geo_mean``) refuse the stock actors' config class (``core_algos.py:940,1031,1104``); the replacements read the
  same attributes from any config object and have no such check;
* ``compute_grpo_outcome_advantage``, ``compute_marft_gae_advantage_return`` and ``apply_kl_penalty``, which the
  reference runs on host tensors (``siirl/dag_worker/dagworker.py:542-560,585-630``): the replacements stage host inputs
  to the GPU and return host results.  (The multi-agent GAE is a Python loop over every token in the reference,
  ``core_algos.py:400-448``.)

**Consumers that bound the names by value.**  The reference's actors and worker import most of these functions with
``from ... import name`` (``siirl/engine/actor/dp_actor.py:32,39``, ``siirl/engine/actor/megatron_actor.py:48``,
``siirl/dag_worker/dagworker.py:45-48``): a module imported before the patch keeps its own reference to the original
function, and setting the attribute on the defining module does not reach it.  Either call ``patch_reference``
before ``siirl.engine.actor.*`` and ``siirl.dag_worker.dagworker`` are imported, or let it repair the late case: it
walks the already imported modules named in ``CONSUMER_MODULES`` (plus any passed as ``consumers=``) and rebinds
every global that ``is`` one of the replaced originals; the names it rebinds are listed under ``"rebound"`` in the
returned dict, and ``undo_patch`` restores them too.  Attribute-style calls (``F.entropy_from_logits``,
``core_algos.compute_grpo_outcome_advantage``) and registry look-ups need none of this.

Deliberately NOT replaced: ``masked_sum`` / ``masked_mean`` / ``masked_var`` / ``masked_whiten``.  The reference's own
``compute_gae_advantage_return`` resolves those globals and calls them on host tensors, where this package's versions
raise (no CPU path); import them from ``siirl_amd.torch_functional`` explicitly where the tensors are on the GPU.
"""

from __future__ import annotations

TORCH_FUNCTIONAL_NAMES = ("logprobs_from_logits", "entropy_from_logits", "entropy_from_logits_with_chunking")
POLICY_LOSSES = {"vanilla": "compute_policy_loss_vanilla", "gspo": "compute_policy_loss_gspo",
                 "cpgd": "compute_policy_loss_cpgd", "gpg": "compute_policy_loss_gpg",
                 "clip_cov": "compute_policy_loss_clip_cov", "kl_cov": "compute_policy_loss_kl_cov",
                 "geo_mean": "compute_policy_loss_geo_mean"}
CORE_ALGOS_NAMES = ("agg_loss", "kl_penalty", "compute_policy_loss", *POLICY_LOSSES.values(),
                    "compute_grpo_outcome_advantage", "compute_marft_gae_advantage_return", "apply_kl_penalty")


# modules of the reference that bind the replaced functions by value at import (file:line in the module docstring)
CONSUMER_MODULES = ("siirl.engine.actor.dp_actor", "siirl.engine.actor.megatron_actor", "siirl.engine.actor.embodied_actor",
                    "siirl.dag_worker.dagworker")


def patch_reference(ref_torch_functional, ref_core_algos, consumers=()) -> dict:
    """Returns ``{"module.name": original}`` so that the caller can undo the patch (``undo_patch``).  ``consumers``:
    further already imported modules (objects or ``sys.modules`` names) whose by-value bindings of the replaced
    functions are to be redirected as well; the reference's own (``CONSUMER_MODULES``) are looked up in
    ``sys.modules`` and treated the same when present."""
    import sys

    from . import core_algos as A
    from . import torch_functional as F

    undo = {}
    replaced = {}  # id(original) -> (original, replacement)
    for prefix, module, names, source in (("torch_functional", ref_torch_functional, TORCH_FUNCTIONAL_NAMES, F),
                                          ("core_algos", ref_core_algos, CORE_ALGOS_NAMES, A)):
        for name in names:
            original = getattr(module, name, None)
            undo[f"{prefix}.{name}"] = original
            setattr(module, name, getattr(source, name))
            if original is not None:
                replaced[id(original)] = (original, getattr(source, name))
    losses = getattr(ref_core_algos, "POLICY_LOSS_REGISTRY", None)
    if losses is not None:
        losses.update({mode: getattr(A, fn) for mode, fn in POLICY_LOSSES.items()})
    estimators = getattr(ref_core_algos, "ADV_ESTIMATOR_REGISTRY", None)
    if estimators is not None:
        estimators["grpo"] = A.compute_grpo_outcome_advantage
    # modules imported before the patch hold the originals under their own global names: redirect those bindings
    rebound = []
    modules = [sys.modules[n] for n in CONSUMER_MODULES if n in sys.modules]
    for c in consumers:
        c = sys.modules.get(c) if isinstance(c, str) else c
        if c is not None and c not in modules:
            modules.append(c)
    for mod in modules:
        if mod is ref_torch_functional or mod is ref_core_algos:
            continue
        for attr, value in list(vars(mod).items()):
            hit = replaced.get(id(value))
            if hit is not None and hit[0] is value:
                setattr(mod, attr, hit[1])
                rebound.append((mod, attr, value))
    undo["rebound"] = rebound
    return undo


def undo_patch(ref_torch_functional, ref_core_algos, undo: dict) -> None:
    """Restores what ``patch_reference`` replaced: the two modules' attributes, the registry entries of the replaced
    policy losses and of ``grpo``, and the consumers' rebound globals."""
    for key, original in undo.items():
        if key == "rebound":
            continue
        prefix, name = key.split(".", 1)
        module = ref_torch_functional if prefix == "torch_functional" else ref_core_algos
        if original is None:
            if hasattr(module, name):
                delattr(module, name)
        else:
            setattr(module, name, original)
    losses = getattr(ref_core_algos, "POLICY_LOSS_REGISTRY", None)
    if losses is not None:
        for mode, fn in POLICY_LOSSES.items():
            if undo.get(f"core_algos.{fn}") is not None:
                losses[mode] = undo[f"core_algos.{fn}"]
    estimators = getattr(ref_core_algos, "ADV_ESTIMATOR_REGISTRY", None)
    if estimators is not None and undo.get("core_algos.compute_grpo_outcome_advantage") is not None:
        estimators["grpo"] = undo["core_algos.compute_grpo_outcome_advantage"]
    for mod, attr, original in undo.get("rebound", ()):
        setattr(mod, attr, original)

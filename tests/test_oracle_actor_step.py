"""Pins ``oracle/actor_step.py::micro_batch_step`` and ``oracle/core_algos.py::compute_entropy_loss`` on the CPU.

``micro_batch_step`` restates the micro-batch loop body of the reference actor
(``siirl/engine/actor/dp_actor.py:425-513`` after ``:170-231``).  It is checked here against

* a closed-form case (uniform logits) whose every term is written out with ``math``;
* ``_hand_loss``, a scalar evaluator in plain Python floats that follows the cited lines token by token and
  knows nothing of torch: the loss value must agree, and ``dlogits`` must agree with central differences of
  that scalar -- which fixes the sign and the scale of every term of the composition independently of autograd;
* the scalings of the logged metrics, the on-policy shortcut and the CPGD drift term.
"""

import math

import pytest
import torch

from oracle import core_algos as OC
from oracle.actor_step import ActorConfig, micro_batch_step


# ------------------------------------------------------------------ a torch-free statement of the same step


def _row_stats(row, temperature, label):
    z = [v / temperature for v in row]  # dp_actor.py:176
    mx = max(z)
    lse = mx + math.log(sum(math.exp(v - mx) for v in z))
    p = [math.exp(v - lse) for v in z]
    return z[label] - lse, lse - sum(pi * zi for pi, zi in zip(p, z))  # log-prob, entropy


def _agg(mat, mask, mode):
    """agg_loss, siirl/dag_worker/core_algos.py:536-569, on nested lists."""
    B, L = len(mat), len(mat[0])
    if mode == "token-mean":
        return sum(mat[b][t] * mask[b][t] for b in range(B) for t in range(L)) / (sum(map(sum, mask)) + 1e-8)
    rows = [sum(mat[b][t] * mask[b][t] for t in range(L)) for b in range(B)]
    if mode == "seq-mean-token-sum":
        return sum(rows) / B
    if mode == "seq-mean-token-mean":
        return sum(r / sum(mask[b]) for b, r in enumerate(rows)) / B
    if mode == "seq-mean-token-sum-norm":
        return sum(rows) / L
    raise ValueError(mode)


def _kl_token(lp, ref, kind):
    """kl_penalty_forward, siirl/dag_worker/core_algos.py:1241-1276."""
    if kind in ("kl", "k1"):
        return lp - ref
    if kind == "abs":
        return abs(lp - ref)
    if kind in ("mse", "k2"):
        return 0.5 * (lp - ref) ** 2
    k = min(max(ref - lp, -20.0), 20.0)
    return min(max(math.exp(k) - k - 1.0, -10.0), 10.0)


def _hand_loss(x, labels, old, adv, mask, cfg, ref=None, temperature=1.0, scale=1.0, frozen=None, isw=None):
    """The scalar that ``loss.backward()`` differentiates at dp_actor.py:501, from nested lists of floats.
    ``frozen`` holds the quantities the reference detaches (log-probs at the base point): the on-policy
    ``old = log_prob.detach()`` (:436-437), GSPO's sequence ratio (core_algos.py:836-840) and the drift weight
    (dp_actor.py:490).  Returns ``(loss, parts)``."""
    B, L = len(labels), len(labels[0])
    lp = [[0.0] * L for _ in range(B)]
    ent = [[0.0] * L for _ in range(B)]
    for b in range(B):
        for t in range(L):
            lp[b][t], ent[b][t] = _row_stats(x[b][t], temperature, labels[b][t])
    lp0 = lp if frozen is None else frozen
    if old is None:  # on policy
        old = lp0
    lo = cfg.clip_ratio_low if cfg.clip_ratio_low is not None else cfg.clip_ratio
    hi = cfg.clip_ratio_high if cfg.clip_ratio_high is not None else cfg.clip_ratio
    tok = [[0.0] * L for _ in range(B)]
    agg_mode = cfg.loss_agg_mode
    for b in range(B):
        if cfg.loss_mode == "gspo":
            n = max(sum(mask[b]), 1)
            s0 = sum((lp0[b][t] - old[b][t]) * mask[b][t] for t in range(L)) / n
        for t in range(L):
            A = adv[b][t]
            if cfg.loss_mode == "vanilla":  # core_algos.py:756-789
                r = math.exp(min(max(lp[b][t] - old[b][t], -20.0), 20.0))
                l1, l2 = -A * r, -A * min(max(r, 1 - lo), 1 + hi)
                c1 = max(l1, l2)
                v = min(-A * cfg.clip_ratio_c, c1) if A < 0 else c1
            elif cfg.loss_mode == "gspo":  # :827-851
                rho = math.exp(min(lp[b][t] - lp0[b][t] + s0, 10.0))
                v = max(-A * rho, -A * min(max(rho, 1 - lo), 1 + hi))
            elif cfg.loss_mode == "cpgd":  # :606-616
                if A > 0:
                    v = -min(lp[b][t], math.log(1 + hi) + old[b][t]) * A
                else:
                    v = -max(lp[b][t], math.log(1 - lo) + old[b][t]) * A
            else:
                raise ValueError(cfg.loss_mode)
            if isw is not None and cfg.loss_mode != "cpgd":
                v *= isw[b][t]
            tok[b][t] = v
    pg = _agg(tok, mask, "seq-mean-token-mean" if cfg.loss_mode == "gspo" else agg_mode)
    policy = pg
    parts = {"pg": pg}
    if cfg.entropy_coeff != 0:  # dp_actor.py:468-472
        parts["entropy"] = _agg(ent, mask, agg_mode)
        policy = pg - parts["entropy"] * cfg.entropy_coeff
    if cfg.use_kl_loss:  # :476-486
        kl = [[_kl_token(lp[b][t], ref[b][t], cfg.kl_loss_type) for t in range(L)] for b in range(B)]
        parts["kl"] = _agg(kl, mask, agg_mode)
        policy = policy + parts["kl"] * cfg.kl_loss_coef
    if cfg.use_cpgd_loss and cfg.policy_drift_coeff != 0:  # :488-494
        dr = [[min(math.exp(lp0[b][t] - old[b][t]) - 1.0, 2.0) * lp[b][t] for t in range(L)] for b in range(B)]
        parts["drift"] = _agg(dr, mask, agg_mode)
        policy = policy + parts["drift"] * cfg.policy_drift_coeff
    return policy * scale, parts


def _logprobs(x, labels, temperature):
    return [[_row_stats(x[b][t], temperature, labels[b][t])[0] for t in range(len(labels[0]))]
            for b in range(len(labels))]


def _central_differences(x, h, f):
    g = [[[0.0] * len(x[0][0]) for _ in x[0]] for _ in x]
    for b in range(len(x)):
        for t in range(len(x[0])):
            for v in range(len(x[0][0])):
                keep = x[b][t][v]
                x[b][t][v] = keep + h
                up = f(x)
                x[b][t][v] = keep - h
                dn = f(x)
                x[b][t][v] = keep
                g[b][t][v] = (up - dn) / (2 * h)
    return g


def _t(v, dtype=torch.float64):
    return torch.tensor(v, dtype=dtype)


# ------------------------------------------------------------------ closed form


def test_uniform_logits_closed_form():
    """B = 1, L = 2, V = 3, all logits equal: lp = -log 3, H = log 3 whatever the temperature.  old = lp - log 1.1
    gives ratio 1.1 inside the clip band, so tok = -A * 1.1; A = (1, -2) -> pg = (-1.1 + 2.2) / 2 = 0.55.
    ref = lp + log 2 -> k3 = e^{log 2} - log 2 - 1 = 1 - log 2 per token.
    loss = (0.55 - 0.01 * log 3 + 0.5 * (1 - log 2)) * 0.25."""
    lp = -math.log(3.0)
    cfg = ActorConfig(entropy_coeff=0.01, use_kl_loss=True, kl_loss_coef=0.5, kl_loss_type="low_var_kl")
    x = torch.full((1, 2, 3), 0.7, dtype=torch.float64)
    old = _t([[lp - math.log(1.1)] * 2])
    ref = _t([[lp + math.log(2.0)] * 2])
    loss, dlogits, metrics, log_prob, entropy = micro_batch_step(
        x, torch.tensor([[1, 0]]), old, _t([[1.0, -2.0]]), _t([[1.0, 1.0]]), cfg, ref_log_prob=ref, temperature=2.0,
        loss_scale_factor=0.25, dtype=torch.float64)
    f = 2.0 / (2.0 + 1e-8)  # token-mean divides by (sum of the mask + 1e-8)
    want = (0.55 - 0.01 * math.log(3.0) + 0.5 * (1.0 - math.log(2.0))) * f * 0.25
    assert abs(loss.item() - want) < 1e-12
    assert torch.allclose(log_prob, _t([[lp, lp]]), atol=1e-12)
    assert torch.allclose(entropy, _t([[math.log(3.0)] * 2]), atol=1e-12)
    # metric scalings of dp_actor.py:485,503-513: pg_loss and kl_loss carry loss_scale_factor, the rest do not
    assert abs(metrics["actor/pg_loss"] - 0.55 * f * 0.25) < 1e-12
    assert abs(metrics["actor/kl_loss"] - (1.0 - math.log(2.0)) * f * 0.25) < 1e-12
    assert metrics["actor/kl_coef"] == 0.5
    assert abs(metrics["actor/entropy_loss"] - math.log(3.0) * f) < 1e-12
    assert metrics["actor/pg_clipfrac"] == 0.0 and metrics["actor/pg_clipfrac_lower"] == 0.0
    assert abs(metrics["actor/ppo_kl"] + math.log(1.1) * f) < 1e-12
    for k in ("actor/pg_clip_mean", "actor/pg_clip_min", "actor/pg_clip_max"):
        assert abs(metrics[k] - 1.1) < 1e-9
    # gradient by hand.  d lp / d z_v = 1[v = y] - 1/3; entropy is stationary at the uniform point;
    # d loss / d lp_t = (w * (-A_t * 1.1) + 0.5 * w * (-(e^k - 1))) * 0.25 with w = 1 / (2 + 1e-8), k = log 2;
    # and z = x / 2.
    w = 1.0 / (2.0 + 1e-8)
    for t, (A, y) in enumerate(((1.0, 1), (-2.0, 0))):
        g_lp = (w * (-A * 1.1) + 0.5 * w * (-1.0)) * 0.25
        for v in range(3):
            want_g = g_lp * ((1.0 if v == y else 0.0) - 1.0 / 3.0) / 2.0
            assert abs(dlogits[0, t, v].item() - want_g) < 1e-12


# ------------------------------------------------------------------ value and finite differences, every branch


def _case(seed, B=2, L=3, V=4):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(B, L, V, generator=g, dtype=torch.float64) * 1.5).tolist()
    labels = torch.randint(0, V, (B, L), generator=g).tolist()
    adv = (torch.randn(B, L, generator=g, dtype=torch.float64)).tolist()
    mask = [[1.0, 1.0, 0.0], [1.0, 1.0, 1.0]][:B]
    mask = [row[:L] for row in mask]
    return g, x, labels, adv, mask


CASES = [
    dict(loss_mode="vanilla", loss_agg_mode="token-mean", entropy_coeff=0.02, use_kl_loss=True, kl_loss_type="low_var_kl",
         kl_loss_coef=0.3),
    dict(loss_mode="vanilla", loss_agg_mode="seq-mean-token-mean", entropy_coeff=0.0, use_kl_loss=True,
         kl_loss_type="mse", kl_loss_coef=0.7, clip_ratio_low=0.05, clip_ratio_high=0.08, clip_ratio_c=1.5),
    dict(loss_mode="vanilla", loss_agg_mode="seq-mean-token-sum", entropy_coeff=-0.1, use_kl_loss=True,
         kl_loss_type="kl", kl_loss_coef=0.2),
    dict(loss_mode="vanilla", loss_agg_mode="seq-mean-token-sum-norm", entropy_coeff=0.05, use_kl_loss=False),
    dict(loss_mode="gspo", loss_agg_mode="token-mean", entropy_coeff=0.03, use_kl_loss=True, kl_loss_type="abs",
         kl_loss_coef=0.4, clip_ratio_low=0.01, clip_ratio_high=0.02),
    dict(loss_mode="cpgd", loss_agg_mode="token-mean", entropy_coeff=0.01, use_kl_loss=True, kl_loss_type="k3",
         kl_loss_coef=0.1, use_cpgd_loss=True, policy_drift_coeff=0.6, clip_ratio_low=0.1, clip_ratio_high=0.1),
]


@pytest.mark.parametrize("ci", range(len(CASES)))
@pytest.mark.parametrize("with_weights", [False, True])
def test_value_and_gradient_against_plain_python(ci, with_weights):
    cfg = ActorConfig(**CASES[ci])
    g, x, labels, adv, mask = _case(100 + ci)
    temperature, scale = 0.7, 0.125
    lp0 = _logprobs(x, labels, temperature)
    noise = (torch.randn(2, 3, generator=g, dtype=torch.float64) * 0.15).tolist()
    old = [[lp0[b][t] + noise[b][t] for t in range(3)] for b in range(2)]
    noise = (torch.randn(2, 3, generator=g, dtype=torch.float64) * 0.3).tolist()
    ref = [[lp0[b][t] + noise[b][t] for t in range(3)] for b in range(2)]
    isw = (torch.rand(2, 3, generator=g, dtype=torch.float64) + 0.5).tolist() if with_weights else None
    want, parts = _hand_loss(x, labels, old, adv, mask, cfg, ref, temperature, scale, frozen=lp0, isw=isw)
    loss, dlogits, metrics, log_prob, entropy = micro_batch_step(
        _t(x), torch.tensor(labels), _t(old), _t(adv), _t(mask), cfg, ref_log_prob=_t(ref), temperature=temperature,
        loss_scale_factor=scale, rollout_is_weights=None if isw is None else _t(isw), dtype=torch.float64)
    assert abs(loss.item() - want) < 1e-12 * max(1.0, abs(want))
    assert torch.allclose(log_prob, _t(lp0), atol=1e-12)
    assert abs(metrics["actor/pg_loss"] - parts["pg"] * scale) < 1e-12
    if cfg.use_kl_loss:
        assert abs(metrics["actor/kl_loss"] - parts["kl"] * scale) < 1e-12
    if cfg.entropy_coeff != 0:
        assert abs(metrics["actor/entropy_loss"] - parts["entropy"]) < 1e-12
    fd = _central_differences(x, 1e-5, lambda xx: _hand_loss(xx, labels, old, adv, mask, cfg, ref, temperature, scale,
                                                             frozen=lp0, isw=isw)[0])
    assert torch.allclose(dlogits, _t(fd), atol=2e-9, rtol=1e-6), (dlogits - _t(fd)).abs().max()
    assert dlogits.abs().max() > 1e-4  # the comparison is not between two zeros


def test_on_policy_branch():
    """dp_actor.py:436-437: old = log_prob.detach() -> ratio 1 everywhere, ppo_kl 0, nothing clipped, and the
    gradient is that of -A * r at r = 1 (the detached old receives none)."""
    cfg = ActorConfig(loss_mode="vanilla", entropy_coeff=0.0)
    g, x, labels, adv, mask = _case(7)
    lp0 = _logprobs(x, labels, 1.0)
    loss, dlogits, metrics, _, entropy = micro_batch_step(_t(x), torch.tensor(labels), None, _t(adv), _t(mask), cfg,
                                                          on_policy=True, dtype=torch.float64)
    assert entropy is None
    assert metrics["actor/ppo_kl"] == 0.0 and metrics["actor/pg_clipfrac"] == 0.0
    assert metrics["actor/pg_clip_mean"] == 1.0 and metrics["actor/pg_clip_min"] == 1.0 == metrics["actor/pg_clip_max"]
    want = -sum(adv[b][t] * mask[b][t] for b in range(2) for t in range(3)) / (sum(map(sum, mask)) + 1e-8)
    assert abs(loss.item() - want) < 1e-12
    fd = _central_differences(x, 1e-5, lambda xx: _hand_loss(xx, labels, None, adv, mask, cfg, frozen=lp0)[0])
    assert torch.allclose(dlogits, _t(fd), atol=2e-9, rtol=1e-6)
    # masked tokens receive no gradient
    assert dlogits[0, 2].abs().max().item() == 0.0


def test_cpgd_drift_term_alone():
    """With zero advantages only the drift term is left: loss = c_d * agg(clamp(e^{lp - old} - 1, max=2) * lp)
    with the weight detached, so d loss / d lp = c_d * w * clamp(...).  One token sits past the clamp."""
    cfg = ActorConfig(loss_mode="cpgd", use_cpgd_loss=True, policy_drift_coeff=0.5, clip_ratio_low=0.2,
                      clip_ratio_high=0.2)
    x = [[[0.0, 0.0]], [[0.0, math.log(3.0)]]]  # lp of label 0: -log 2, -log 4
    labels = [[0], [0]]
    old = [[-math.log(2.0) - math.log(1.5)], [-math.log(4.0) - math.log(10.0)]]  # ratios 1.5 and 10
    adv = [[0.0], [0.0]]
    mask = [[1.0], [1.0]]
    loss, dlogits, _, _, _ = micro_batch_step(_t(x), torch.tensor(labels), _t(old), _t(adv), _t(mask), cfg,
                                              dtype=torch.float64)
    w = 1.0 / (2.0 + 1e-8)
    want = 0.5 * w * (0.5 * -math.log(2.0) + 2.0 * -math.log(4.0))
    assert abs(loss.item() - want) < 1e-12
    # d lp / d x_0 = 1 - p_0 : 1/2 and 3/4
    assert abs(dlogits[0, 0, 0].item() - 0.5 * w * 0.5 * 0.5) < 1e-12
    assert abs(dlogits[1, 0, 0].item() - 0.5 * w * 2.0 * 0.75) < 1e-12
    # the flag gates the term (dp_actor.py:488)
    off = ActorConfig(loss_mode="cpgd", use_cpgd_loss=False, policy_drift_coeff=0.5)
    loss_off, *_ = micro_batch_step(_t(x), torch.tensor(labels), _t(old), _t(adv), _t(mask), off, dtype=torch.float64)
    assert loss_off.item() == 0.0


def test_entropy_and_kl_signs():
    """The entropy bonus enters with a minus sign and the KL loss with a plus sign (dp_actor.py:472,484): at zero
    advantage the loss falls when the entropy rises, and rises with the distance to the reference."""
    cfg = ActorConfig(entropy_coeff=1.0, use_kl_loss=True, kl_loss_coef=1.0, kl_loss_type="mse")
    labels, adv, mask = torch.tensor([[0]]), _t([[0.0]]), _t([[1.0]])
    flat, peaked = _t([[[0.0, 0.0, 0.0]]]), _t([[[4.0, 0.0, 0.0]]])
    lp_flat, lp_peak = -math.log(3.0), 4.0 - math.log(math.exp(4.0) + 2.0)
    l_flat, *_ = micro_batch_step(flat, labels, _t([[lp_flat]]), adv, mask, cfg, ref_log_prob=_t([[lp_flat]]),
                                  dtype=torch.float64)
    l_peak, *_ = micro_batch_step(peaked, labels, _t([[lp_peak]]), adv, mask, cfg, ref_log_prob=_t([[lp_peak]]),
                                  dtype=torch.float64)
    assert abs(l_flat.item() + math.log(3.0) / (1 + 1e-8)) < 1e-12  # -H, KL = 0
    assert l_flat.item() < l_peak.item() < 0.0
    l_far, *_ = micro_batch_step(flat, labels, _t([[lp_flat]]), adv, mask, cfg, ref_log_prob=_t([[lp_flat - 2.0]]),
                                 dtype=torch.float64)
    assert abs(l_far.item() - (l_flat.item() + 0.5 * 4.0 / (1 + 1e-8))) < 1e-12


def test_fp32_matches_fp64_on_a_wider_case():
    """The fp32 mode (what the GPU tests compare with) agrees with the fp64 evaluation of the same step."""
    g = torch.Generator().manual_seed(11)
    B, L, V = 3, 5, 37
    x = torch.randn(B, L, V, generator=g) * 2
    y = torch.randint(0, V, (B, L), generator=g)
    mask = (torch.arange(L)[None, :] < torch.tensor([5, 2, 4])[:, None]).float()
    adv = torch.randn(B, L, generator=g)
    from oracle.torch_functional import logprobs_from_logits

    base = logprobs_from_logits(x, y)
    old, ref = base + torch.randn(B, L, generator=g) * 0.05, base + torch.randn(B, L, generator=g) * 0.1
    cfg = ActorConfig(entropy_coeff=0.01, use_kl_loss=True)
    l32, d32, m32, *_ = micro_batch_step(x, y, old, adv, mask, cfg, ref_log_prob=ref, loss_scale_factor=0.5)
    l64, d64, m64, *_ = micro_batch_step(x.double(), y, old.double(), adv.double(), mask.double(), cfg,
                                         ref_log_prob=ref.double(), loss_scale_factor=0.5, dtype=torch.float64)
    assert abs(l32.item() - l64.item()) < 1e-6
    assert torch.allclose(d32.double(), d64, atol=1e-7)
    for k in m64:
        assert abs(m32[k] - m64[k]) < 1e-5, k


# ------------------------------------------------------------------ compute_entropy_loss


def test_compute_entropy_loss():
    """core_algos.py:1156-1170: agg_loss(entropy_from_logits(logits), mask, mode).  Uniform rows have entropy
    log V; a general case is checked against torch.distributions and an explicit aggregation."""
    V = 11
    mask = torch.tensor([[1.0, 1.0, 0.0], [1.0, 0.0, 0.0]])
    for mode in ("token-mean", "seq-mean-token-sum", "seq-mean-token-mean", "seq-mean-token-sum-norm"):
        got = OC.compute_entropy_loss(torch.zeros(2, 3, V, dtype=torch.float64), mask.double(), mode).item()
        want = {"token-mean": math.log(V) * 3 / (3 + 1e-8), "seq-mean-token-sum": math.log(V) * 1.5,
                "seq-mean-token-mean": math.log(V), "seq-mean-token-sum-norm": math.log(V)}[mode]
        assert abs(got - want) < 1e-12, mode
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 3, V, generator=g, dtype=torch.float64)
    H = torch.distributions.Categorical(logits=x).entropy()
    got = OC.compute_entropy_loss(x, mask.double(), "token-mean").item()
    assert abs(got - (H[0, 0] + H[0, 1] + H[1, 0]).item() / (3 + 1e-8)) < 1e-12
    got = OC.compute_entropy_loss(x, mask.double(), "seq-mean-token-mean").item()
    assert abs(got - ((H[0, 0] + H[0, 1]) / 2 + H[1, 0]).item() / 2) < 1e-12

"""The torch.library layer: every entry point of the path is a ``torch.ops.siirl_hip.*`` custom op with a fake
kernel (shape inference without a GPU), and on the GPU the ops pass ``torch.library.opcheck``."""
import pytest
import torch

import siirl_amd.ops  # noqa: F401  (registers the ops)

OPS = ("logprob_entropy_fwd", "logprob_entropy_bwd", "logprob_entropy_bwd_", "grpo_advantage", "group_keep_mask",
       "agg_loss_fwd", "agg_loss_bwd", "masked_reduce_fwd", "masked_reduce_bwd", "policy_loss_fwd", "policy_loss_bwd",
       "cov_scores", "topk_mark", "range_indices", "kl_penalty_fwd", "kl_penalty_bwd",
       "fused_linear_logprob_entropy_fwd", "fused_linear_logprob_entropy_bwd")


DIFFERENTIABLE = ("logprob_entropy", "actor_loss", "agg_loss", "masked_reduce", "value_loss", "kl_penalty",
                  "fused_linear_logprob_entropy")


def test_ops_are_registered():
    for name in OPS + DIFFERENTIABLE:
        op = getattr(torch.ops.siirl_hip, name)
        assert op.default._schema.name == f"siirl_hip::{name}"
    # the in-place backward declares what it overwrites
    assert "Tensor(a!) logits" in str(torch.ops.siirl_hip.logprob_entropy_bwd_.default._schema)


def test_the_layer_is_the_cpp_library():
    """The operators come from lib/libsiirl_torch.so (TORCH_LIBRARY(siirl_hip) in csrc/torch_ops.cpp), not from
    Python-side registrations: they dispatch to a C++ kernel for the GPU key and have none for the CPU."""
    import siirl_amd.ops as ops

    assert ops.TORCH_LIB_PATH.exists() and ops.TORCH_LIB_PATH.name == "libsiirl_torch.so"
    assert torch._C._dispatch_has_kernel_for_dispatch_key("siirl_hip::logprob_entropy_fwd", "CUDA")
    assert not torch._C._dispatch_has_kernel_for_dispatch_key("siirl_hip::logprob_entropy_fwd", "CPU")
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.siirl_hip.kl_penalty_fwd(torch.zeros(2, 3), torch.zeros(2, 3), 0)


def _loss_args(mk, B, L, with_optional):
    f = lambda: mk((B, L), torch.float32)  # noqa: E731
    opt = (f(), f(), f()) if with_optional else (None, None, None)
    return (f(), f(), f(), mk((B, L), torch.int64), *opt, 0, 0.2, 0.28, 3.0, 20.0, 0, 0.001, 3, False, 0.001, 0.0, 1.0)


@pytest.mark.parametrize("with_optional", [False, True])
def test_fake_kernels_give_shapes_without_a_gpu(with_optional):
    from torch._subclasses.fake_tensor import FakeTensorMode

    ns = torch.ops.siirl_hip
    with FakeTensorMode():
        mk = lambda shape, dtype: torch.empty(shape, dtype=dtype, device="meta")  # noqa: E731
        B, L, T, V, H = 6, 40, 24, 1000, 64
        out16, row_msum, row_s = ns.policy_loss_fwd(*_loss_args(mk, B, L, with_optional))
        assert out16.shape == (16,) and row_msum.shape == (B,) and row_s.shape == (B,)
        a = _loss_args(mk, B, L, with_optional)
        d_lp, d_ent = ns.policy_loss_bwd(mk((1,), torch.float32), *a, out16, row_msum, row_s)
        assert d_lp.shape == (B, L) and d_ent.shape == ((B, L) if with_optional else (0,))
        o, r = ns.agg_loss_fwd(mk((B, L), torch.float32), mk((B, L), torch.bool), 0)
        assert o.shape == (16,) and r.shape == (B,)
        assert ns.agg_loss_bwd(mk((1,), torch.float32), mk((B, L), torch.bool), o, r, 0).shape == (B, L)
        r, ms = ns.masked_reduce_fwd(mk((B, L), torch.float32), mk((B, L), torch.int64), True, True)
        assert r.shape == (B,) and ms.shape == (B,)
        r, ms = ns.masked_reduce_fwd(mk((B, L), torch.float32), mk((B, L), torch.int64), False, False)
        assert r.shape == (2,) and ms.shape == (1,)
        assert ns.masked_reduce_bwd(mk((B,), torch.float32), mk((B, L), torch.bool), True, None).shape == (B, L)
        cov, stats = ns.cov_scores(mk((B, L), torch.float32), mk((B, L), torch.float32), mk((B, L), torch.float32),
                                   mk((B, L), torch.int64), 6, 0.2, 0.28)
        assert cov.shape == (B, L) and stats.shape == (6,) and cov.dtype == torch.float32
        a5 = list(_loss_args(mk, B, L, with_optional))
        a5[7] = 5
        o5, _, _ = ns.policy_loss_fwd(*a5, mk((B, L), torch.float32))
        assert o5.shape == (16,)
        assert ns.kl_penalty_fwd(mk((B, L), torch.float32), mk((B, L), torch.float32), 3).shape == (B, L)
        d1, d2 = ns.kl_penalty_bwd(mk((B, L), torch.float32), mk((B, L), torch.float32), mk((B, L), torch.float32), 3,
                                   False, True, False)
        assert d1.shape == (B, L) and d2.shape == (0,)
        adv = ns.grpo_advantage(mk((B, L), torch.float32), mk((B, L), torch.int64), mk((B,), torch.int64), 1e-6, True)
        assert adv.shape == (B, L) and adv.dtype == torch.float32
        keep, gsz = ns.group_keep_mask(mk((B,), torch.float64), mk((B,), torch.int64))
        assert keep.dtype == torch.uint8 and gsz.dtype == torch.int32 and keep.shape == gsz.shape == (B,)
        lp, ent, lse, ex, sv = ns.fused_linear_logprob_entropy_fwd(mk((T, H), torch.bfloat16),
                                                                   mk((V, H), torch.bfloat16), mk((T,), torch.int64), 1.0)
        assert lp.shape == ent.shape == lse.shape == ex.shape == (T,) and lp.dtype == torch.float32 and sv.numel() == 0
        sv = ns.fused_linear_logprob_entropy_fwd(mk((T, H), torch.bfloat16), mk((V, H), torch.bfloat16),
                                                 mk((T,), torch.int64), 1.0, True)[4]
        assert sv.numel() == ((V + 255) // 256) * ((T + 255) // 256) * 65536 and sv.dtype == torch.float32
        dh, dw = ns.fused_linear_logprob_entropy_bwd(mk((T, H), torch.bfloat16), mk((V, H), torch.bfloat16),
                                                     mk((T,), torch.int64), 1.0, lse, ex, mk((T,), torch.float32), None,
                                                     True, False)
        assert dh.shape == (T, H) and dh.dtype == torch.bfloat16 and dw.shape == (0,)
        lp, ent, lse, ex = ns.logprob_entropy_fwd(mk((3, 5, V), torch.bfloat16), mk((3, 5), torch.int64), 1.0, True)
        assert lp.shape == ent.shape == lse.shape == (3, 5)


@pytest.mark.gpu
def test_opcheck_on_the_gpu():
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(0)
    ns = torch.ops.siirl_hip
    checks = ("test_schema", "test_faketensor")
    B, L, T, V, H = 6, 40, 24, 1000, 64
    mk = lambda shape, dtype: (torch.randn(shape, device=dev, generator=g) * 0.1).to(dtype) if dtype.is_floating_point \
        else torch.ones(shape, dtype=dtype, device=dev)  # noqa: E731
    args = _loss_args(mk, B, L, True)
    torch.library.opcheck(ns.policy_loss_fwd, args, test_utils=checks)
    out16, row_msum, row_s = ns.policy_loss_fwd(*args)
    torch.library.opcheck(ns.policy_loss_bwd, (torch.ones(1, device=dev), *args, out16, row_msum, row_s), test_utils=checks)
    lm, m = mk((B, L), torch.float32), torch.ones(B, L, dtype=torch.bool, device=dev)
    torch.library.opcheck(ns.agg_loss_fwd, (lm, m, 2), test_utils=checks)
    torch.library.opcheck(ns.cov_scores, (lm, mk((B, L), torch.float32), mk((B, L), torch.float32), m, 6, 0.2, 0.28),
                          test_utils=checks)
    torch.library.opcheck(ns.cov_scores, (None, mk((B, L), torch.float32), mk((B, L), torch.float32), m, 5, 0.0, 0.0),
                          test_utils=checks)
    cov_args = list(args)
    cov_args[7] = 5
    torch.library.opcheck(ns.policy_loss_fwd, (*cov_args, mk((B, L), torch.float32)), test_utils=checks)
    torch.library.opcheck(ns.kl_penalty_fwd, (lm, mk((B, L), torch.float32), 3), test_utils=checks)
    torch.library.opcheck(ns.masked_reduce_fwd, (lm, m, True, True), test_utils=checks)
    torch.library.opcheck(ns.masked_reduce_fwd, (lm, m, False, True), test_utils=checks)
    _, msum = ns.masked_reduce_fwd(lm, m, True, True)
    torch.library.opcheck(ns.masked_reduce_bwd, (torch.ones(B, device=dev), m, True, msum), test_utils=checks)
    torch.library.opcheck(ns.logprob_entropy_bwd_, (mk((T, V), torch.bfloat16), torch.randint(0, V, (T,), device=dev),
                                                     1.0, torch.zeros(T, device=dev), torch.zeros(T, device=dev),
                                                     torch.ones(T, device=dev), torch.ones(T, device=dev), False),
                          test_utils=checks)
    uid = torch.arange(B, device=dev) // 2
    torch.library.opcheck(ns.grpo_advantage, (lm, torch.ones(B, L, dtype=torch.int64, device=dev), uid, 1e-6, True),
                          test_utils=checks)
    torch.library.opcheck(ns.group_keep_mask, (torch.rand(B, device=dev, dtype=torch.float64), uid), test_utils=checks)
    h, w = mk((T, H), torch.bfloat16), mk((V, H), torch.bfloat16)
    y = torch.randint(0, V, (T,), device=dev)
    torch.library.opcheck(ns.fused_linear_logprob_entropy_fwd, (h, w, y, 1.0), test_utils=checks)
    torch.library.opcheck(ns.fused_linear_logprob_entropy_fwd, (h, w, y, 1.0, True), test_utils=checks)
    lp, ent, lse, ex, sv = ns.fused_linear_logprob_entropy_fwd(h, w, y, 1.0, True)
    torch.library.opcheck(ns.fused_linear_logprob_entropy_bwd, (h, w, y, 1.0, lse, ex, torch.ones(T, device=dev), None,
                                                                True, True), test_utils=checks)
    torch.library.opcheck(ns.fused_linear_logprob_entropy_bwd, (h, w, y, 1.0, lse, ex, torch.ones(T, device=dev), None,
                                                                True, True, sv), test_utils=checks)
    x = mk((T, V), torch.bfloat16)
    torch.library.opcheck(ns.logprob_entropy_fwd, (x, y, 1.0, True), test_utils=checks)


@pytest.mark.gpu
def test_plain_operators_refuse_misplaced_or_short_operands():
    """The plain operators pass raw pointers to kernels sized from one operand: a secondary operand on the host, or
    with fewer elements than the kernel would touch, must raise on the host, before anything is launched."""
    dev = torch.device("cuda:0")
    ns = torch.ops.siirl_hip
    B, L, T, V, H = 4, 24, 16, 300, 64
    f = lambda *s: torch.randn(*s, device=dev) * 0.1  # noqa: E731
    ones = torch.ones(B, L, dtype=torch.int64, device=dev)
    uid = torch.arange(B, device=dev) // 2
    bad = (RuntimeError, ValueError, TypeError)

    with pytest.raises(bad):
        ns.grpo_advantage(f(B, L), ones.cpu(), uid, 1e-6, True)
    with pytest.raises(bad):
        ns.grpo_advantage(f(B, L), ones, uid.cpu(), 1e-6, True)
    with pytest.raises(bad):
        ns.group_keep_mask(torch.rand(B, device=dev, dtype=torch.float64), uid.cpu())
    with pytest.raises(bad):
        ns.agg_loss_fwd(f(B, L), ones[:, : L // 2].contiguous(), 0)
    with pytest.raises(bad):
        ns.agg_loss_fwd(f(B, L), ones.cpu(), 0)
    out16, row_msum = ns.agg_loss_fwd(f(B, L), ones, 0)
    g1 = torch.ones(1, device=dev)
    with pytest.raises(bad):
        ns.agg_loss_bwd(g1, ones, out16[:8].contiguous(), row_msum, 0)
    with pytest.raises(bad):
        ns.agg_loss_bwd(g1, ones, out16, row_msum[:-1].contiguous(), 0)
    with pytest.raises(bad):
        ns.agg_loss_bwd(g1, ones, out16.cpu(), row_msum, 0)
    with pytest.raises(bad):
        ns.masked_reduce_fwd(f(B, L), ones.cpu(), True, True)
    with pytest.raises(bad):
        ns.masked_reduce_bwd(torch.ones(B, device=dev), ones.cpu(), True, None)

    args = list(_loss_args(lambda s, d: f(*s) if d.is_floating_point else torch.ones(s, dtype=d, device=dev), B, L, True))
    for i in (0, 2, 3, 4, 5, 6):  # every operand but log_prob itself, in turn: wrong extent, then wrong device
        short = list(args)
        short[i] = args[i][:, : L // 2].contiguous()
        with pytest.raises(bad):
            ns.policy_loss_fwd(*short)
        host = list(args)
        host[i] = args[i].cpu()
        with pytest.raises(bad):
            ns.policy_loss_fwd(*host)
    o16, rm, rs = ns.policy_loss_fwd(*args)
    with pytest.raises(bad):
        ns.policy_loss_bwd(g1, *args, o16, rm[:-1].contiguous(), rs)
    with pytest.raises(bad):
        ns.policy_loss_bwd(g1.cpu(), *args, o16, rm, rs)
    short = list(args)
    short[1] = args[1][:, : L // 2].contiguous()  # log_prob shorter than the others
    with pytest.raises(bad):
        ns.policy_loss_bwd(g1, *short, o16, rm, rs)

    with pytest.raises(bad):
        ns.kl_penalty_fwd(f(B, L), f(B, L).cpu(), 3)
    with pytest.raises(bad):
        ns.kl_penalty_bwd(f(B, L // 2), f(B, L), f(B, L), 3, False, True, False)

    x = f(T, V).to(torch.bfloat16)
    y = torch.randint(0, V, (T,), device=dev)
    lp, ent, lse, ex = ns.logprob_entropy_fwd(x, y, 1.0, True)
    gl = torch.ones(T, device=dev)
    with pytest.raises(bad):
        ns.logprob_entropy_bwd(x, y, 1.0, lse[:-1].contiguous(), ex, gl, gl, False)
    with pytest.raises(bad):
        ns.logprob_entropy_bwd(x, y, 1.0, lse, ex, gl[:-1].contiguous(), gl, False)
    with pytest.raises(bad):
        ns.logprob_entropy_bwd(x, y[:-1].contiguous(), 1.0, lse, ex, gl, gl, False)
    with pytest.raises(bad):
        ns.logprob_entropy_bwd(x, y, 1.0, lse, ex[:-1].contiguous(), gl, gl, False)

    h, w = f(T, H).to(torch.bfloat16), f(V, H).to(torch.bfloat16)
    with pytest.raises(bad):
        ns.fused_linear_logprob_entropy_fwd(h, w, y.cpu(), 1.0)
    with pytest.raises(bad):
        ns.fused_linear_logprob_entropy_fwd(h, w.cpu(), y, 1.0)
    lp, ent, lse, ex, _ = ns.fused_linear_logprob_entropy_fwd(h, w, y, 1.0)
    with pytest.raises(bad):
        ns.fused_linear_logprob_entropy_bwd(h, w, y, 1.0, lse[:-1].contiguous(), ex, gl, None, True, True)
    with pytest.raises(bad):
        ns.fused_linear_logprob_entropy_bwd(h, w, y, 1.0, lse, ex, gl[:-1].contiguous(), None, True, True)
    with pytest.raises(bad):
        ns.fused_linear_logprob_entropy_bwd(h, w, y.cpu(), 1.0, lse, ex, gl, None, True, True)
    with pytest.raises(bad):
        ns.fused_linear_logprob_entropy_bwd(h, w, y, 1.0, lse.cpu(), ex, gl, None, True, True)
    # and the well-formed calls still run
    torch.cuda.synchronize()
    dh, dw = ns.fused_linear_logprob_entropy_bwd(h, w, y, 1.0, lse, ex, gl, None, True, True)
    assert torch.isfinite(dh.float()).all() and torch.isfinite(dw.float()).all()

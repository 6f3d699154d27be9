"""``torch.compile(dynamic=True)`` over the drop-in functions, as the reference's actor wraps its entropy function
(``siirl/engine/actor/dp_actor.py:80-84``): the compiled call must give the uncompiled call's bits, forward and
backward, also when the shape changes between calls and when an eager in-place log-prob call precedes it (the padded
path, ``dp_actor.py:254-260``).  The reference-named functions leave the graph for the call; the explicitly traceable
form (plain custom ops with fake kernels inside one ``autograd.Function``) is compiled with ``fullgraph=True``.  The
``eager`` and ``aot_eager`` backends exercise tracing and the fake kernels without a code generator."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("backend", ["eager", "aot_eager"])
def test_compiled_entropy_and_logprob_match_eager(dev, backend):
    import siirl_amd.torch_functional as SF

    g = torch.Generator(device=dev).manual_seed(0)
    fn = torch.compile(SF.entropy_from_logits, backend=backend, dynamic=True)
    for shape in ((4, 64, 1000), (2, 33, 1000)):
        x = (torch.randn(*shape, device=dev, generator=g) * 2).to(torch.bfloat16).requires_grad_(True)
        e = fn(x)
        e.sum().backward()
        got = x.grad.clone()
        x.grad = None
        e2 = SF.entropy_from_logits(x)
        e2.sum().backward()
        assert torch.equal(e, e2) and torch.equal(got, x.grad)

    def both(x, y):
        return SF.logprobs_from_logits(x, y, inplace_backward=False), SF.entropy_from_logits(x)

    cb = torch.compile(both, backend=backend, dynamic=True)
    x = (torch.randn(3, 20, 500, device=dev, generator=g) * 2).requires_grad_(True)
    y = torch.randint(0, 500, (3, 20), device=dev, generator=g)
    lp, en = cb(x, y)
    assert en.grad_fn is lp.grad_fn  # the pairing survives the compiled wrapper
    (lp.sum() + en.sum()).backward()
    got = x.grad.clone()
    x.grad = None
    lp2, en2 = both(x, y)
    (lp2.sum() + en2.sum()).backward()
    assert torch.equal(lp, lp2) and torch.equal(en, en2) and torch.equal(got, x.grad)


@pytest.mark.parametrize("backend", ["eager", "aot_eager"])
def test_eager_inplace_logprob_then_compiled_entropy(dev, backend):
    """The padded actor path with ``use_torch_compile=True``: eager ``logprobs_from_logits(logits, responses)``
    (in-place backward by default), then the compiled entropy function on the same tensor."""
    import siirl_amd.torch_functional as SF
    from oracle import torch_functional as OF

    g = torch.Generator().manual_seed(1)
    full = (torch.randn(2, 9, 300, generator=g) * 2).to(torch.bfloat16)
    y = torch.randint(0, 300, (2, 5), generator=g)
    w1, w2 = torch.randn(2, 5, generator=g), torch.randn(2, 5, generator=g)
    fn = torch.compile(SF.entropy_from_logits, backend=backend, dynamic=True)
    leaf = full.to(dev).requires_grad_(True)
    logits = (leaf * 1.0)[:, -6:-1, :]
    lp = SF.logprobs_from_logits(logits, y.to(dev))
    ent = fn(logits)
    ((lp * w1.to(dev)).sum() + (ent * w2.to(dev)).sum()).backward()
    xs = full[:, -6:-1, :]
    want = OF.logprob_entropy_backward(xs, y, w1, w2, dtype=torch.float64)
    err = (leaf.grad.cpu()[:, -6:-1, :].double() - want).abs()
    assert bool((err <= 2.0 ** -7 * want.abs() + 1e-6).all()), err.max()


@pytest.mark.parametrize("backend", ["eager", "aot_eager"])
def test_traceable_form_compiles_as_one_graph(dev, backend):
    import siirl_amd.torch_functional as SF

    def f(x, y):
        lp, ent = SF.logprob_entropy_traceable(x, y, temperature=0.7)
        return (lp * 2.0).sum() + ent.sum()

    cf = torch.compile(f, backend=backend, dynamic=True, fullgraph=True)
    g = torch.Generator(device=dev).manual_seed(2)
    for shape in ((6, 40, 700), (3, 11, 700)):
        x = (torch.randn(*shape, device=dev, generator=g) * 2).requires_grad_(True)
        y = torch.randint(0, 700, shape[:-1], device=dev, generator=g)
        cf(x, y).backward()
        got = x.grad.clone()
        x.grad = None
        lp, ent = SF.logprobs_and_entropy_from_logits(x, y, temperature=0.7)
        ((lp * 2.0).sum() + ent.sum()).backward()
        assert torch.equal(got, x.grad)

"""``torch.compile(dynamic=True)`` over the drop-in functions, as the reference's actor wraps its entropy function
(``siirl/engine/actor/dp_actor.py:80-84``): Dynamo must get through the custom ops (opaque, with fake kernels) and
the results must equal the uncompiled call, forward and backward, also when the shape changes between calls.  The
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
    (lp.sum() + en.sum()).backward()
    got = x.grad.clone()
    x.grad = None
    lp2, en2 = both(x, y)
    (lp2.sum() + en2.sum()).backward()
    assert torch.equal(lp, lp2) and torch.equal(en, en2) and torch.equal(got, x.grad)

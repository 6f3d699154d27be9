"""The allocation-free entry point ``siirl_actor_loss_fwd_static`` against ``siirl_actor_loss_fwd`` through the C ABI:
same kernels over a buffer inside the library's device image instead of the caller's workspace, so every output must
agree bit for bit -- on two calls in a row, the second on a smaller problem (the shared buffer then still holds the
first call's partial sums), for the loss kinds that use each region of the scratch (segment partials, the row
pre-pass of gspo / geo_mean, the two-level finish above 2048 rows); that it takes no device memory (the free bytes
the runtime reports do not move over many calls); and that calls on two streams with a slot of the buffer each do
not disturb one another."""

import pytest
import torch

pytestmark = pytest.mark.gpu

VANILLA, GSPO, CPGD, GPG, GEO = range(5)


def _inputs(B, L, seed, dev):
    g = torch.Generator().manual_seed(seed)
    lp = torch.randn(B, L, generator=g) - 1.5
    old = lp + torch.randn(B, L, generator=g) * 0.1
    ref = lp + torch.randn(B, L, generator=g) * 0.2
    adv = torch.randn(B, L, generator=g)
    ent = torch.rand(B, L, generator=g) * 3
    lens = torch.randint(1, L + 1, (B,), generator=g)
    mask = (torch.arange(L)[None, :] < lens[:, None]).to(torch.int64)
    return [t.to(dev).contiguous() for t in (old, lp, adv, mask, ent, ref)]


def _call(static, ops, B, L, mode, dev, slot=0, outs=None, stream=None):
    from siirl_amd import _lib

    h = _lib.lib()
    old, lp, adv, mask, ent, ref = ops
    if outs is None:
        outs = (torch.full((16,), float("nan"), device=dev), torch.full((B,), float("nan"), device=dev),
                torch.full((B,), float("nan"), device=dev))
    out16, row_msum, row_s = outs
    head = (_lib.ptr(old), _lib.ptr(lp), _lib.ptr(adv), _lib.ptr(mask), _lib.I64, None, _lib.ptr(ent), _lib.ptr(ref), B,
            L, mode, 0.2, 0.28, 3.0, 20.0, 0, 0.01, 3, 0, 0.05, 0.0, 0.5, _lib.ptr(out16), _lib.ptr(row_msum),
            _lib.ptr(row_s))
    stream = _lib.current_stream(dev) if stream is None else stream
    if static:
        rc = h.siirl_actor_loss_fwd_static(*head, slot, stream)
    else:
        n = h.siirl_loss_workspace_bytes(B, L)
        ws = torch.empty(n, dtype=torch.uint8, device=dev)
        rc = h.siirl_actor_loss_fwd(*head, _lib.ptr(ws), n, stream)
    return rc, out16, row_msum, row_s


def _same_bits(a, b):
    return torch.equal(a.view(torch.int32), b.view(torch.int32))


@pytest.mark.parametrize("mode", [VANILLA, GSPO, GEO])
def test_static_scratch_matches_workspace_variant(dev, mode):
    # first a problem large enough for the two-level finish (B > 2048), then a smaller one, then a tiny one
    shapes = [(2304, 4100), (37, 2500), (3, 16)]
    for k, (B, L) in enumerate(shapes):
        print(f"[no-alloc] mode {mode} call {k}: B={B} L={L}", flush=True)
        ops = _inputs(B, L, 1000 * mode + k, dev)
        rc_w, out_w, msum_w, s_w = _call(False, ops, B, L, mode, dev)
        rc_s, out_s, msum_s, s_s = _call(True, ops, B, L, mode, dev, slot=k % 4)
        torch.cuda.synchronize(dev)
        assert rc_w == 0 and rc_s == 0
        assert torch.isfinite(out_w[:13]).all()
        assert _same_bits(out_s, out_w), (out_s, out_w)
        assert _same_bits(msum_s, msum_w)
        if mode in (GSPO, GEO):
            assert _same_bits(s_s, s_w)


def test_static_entry_takes_no_device_memory(dev):
    """Free device memory as the runtime reports it (hipMemGetInfo: it sees hipMalloc / hipFree of any caller, not
    only torch's allocator) is the same before and after 50 calls into pre-allocated outputs, on every slot."""
    B, L = 300, 3000
    ops = _inputs(B, L, 77, dev)
    outs = (torch.empty(16, device=dev), torch.empty(B, device=dev), torch.empty(B, device=dev))
    assert _call(True, ops, B, L, GSPO, dev, outs=outs)[0] == 0  # warm-up: resolves the buffer's address
    torch.cuda.synchronize(dev)
    free_before, _ = torch.cuda.mem_get_info(dev)
    for i in range(50):
        assert _call(True, ops, B, L, (VANILLA, GSPO, GEO)[i % 3], dev, slot=i % 4, outs=outs)[0] == 0
    torch.cuda.synchronize(dev)
    free_after, _ = torch.cuda.mem_get_info(dev)
    assert free_after == free_before, (free_before, free_after)


def test_two_streams_with_a_slot_each(dev):
    """Calls issued on two streams at once, each with its own slot of the static buffer, give the workspace variant's
    bits; repeated, so that the two really overlap."""
    import ctypes

    shapes = {0: (2304, 4100), 1: (1500, 6000)}
    ops = {k: _inputs(B, L, 500 + k, dev) for k, (B, L) in shapes.items()}
    want = {k: _call(False, ops[k], *shapes[k], GSPO, dev) for k in shapes}
    torch.cuda.synchronize(dev)
    streams = {k: torch.cuda.Stream(device=dev) for k in shapes}
    outs = {k: [(torch.empty(16, device=dev), torch.empty(shapes[k][0], device=dev), torch.empty(shapes[k][0], device=dev))
                for _ in range(8)] for k in shapes}
    for s in streams.values():
        s.wait_stream(torch.cuda.current_stream(dev))
    for rep in range(8):
        for k in shapes:
            rc = _call(True, ops[k], *shapes[k], GSPO, dev, slot=k + 1, outs=outs[k][rep],
                       stream=ctypes.c_void_p(streams[k].cuda_stream))[0]
            assert rc == 0
    for s in streams.values():
        torch.cuda.current_stream(dev).wait_stream(s)
    torch.cuda.synchronize(dev)
    for k in shapes:
        _, out_w, msum_w, s_w = want[k]
        for rep in range(8):
            out_s, msum_s, s_s = outs[k][rep]
            assert _same_bits(out_s, out_w) and _same_bits(msum_s, msum_w) and _same_bits(s_s, s_w), (k, rep)


def test_static_scratch_limit_is_reported(dev):
    from siirl_amd import _lib

    B, L = 70000, 2048  # 70000 segments of 64 bytes: beyond the 4 MiB buffer
    z = torch.zeros(1, device=dev)
    h = _lib.lib()
    rc = h.siirl_actor_loss_fwd_static(_lib.ptr(z), _lib.ptr(z), _lib.ptr(z), _lib.ptr(z), _lib.F32, None, None, None, B, L,
                                       0, 0.2, 0.2, 3.0, 20.0, 0, 0.0, 0, 0, 0.0, 0.0, 1.0, _lib.ptr(z), _lib.ptr(z),
                                       _lib.ptr(z), 0, _lib.current_stream(dev))
    assert rc == -4 and b"static buffer" in h.siirl_hip_last_error()
    assert h.siirl_loss_workspace_bytes(B, L) > (4 << 20)

"""GPU parity: remove-padding bookkeeping (through the C ABI) vs the numpy oracle.  Index and integer work:
bit-exact; the float payloads are moved, not computed, so they are bit-exact too."""
import numpy as np
import pytest
import torch

from oracle import padding as OP

pytestmark = pytest.mark.gpu


def _case(B, S, seed, full_first=True):
    rng = np.random.default_rng(seed)
    mask = np.zeros((B, S), dtype=np.int64)
    for b in range(B):
        lo = rng.integers(0, max(S // 2, 1))
        hi = S - rng.integers(0, max(S // 2, 1))
        mask[b, lo:max(hi, lo + 1)] = 1
    if full_first:
        mask[0, :] = 1
    ids = rng.integers(0, 150000, (B, S)).astype(np.int64)
    return ids, mask


@pytest.mark.parametrize("B,S", [(1, 2), (3, 9), (8, 1300), (300, 257), (2, 70000)])
@pytest.mark.parametrize("mdt", [torch.int64, torch.bool, torch.int32, torch.float32, torch.bfloat16])
def test_unpad_input(dev, B, S, mdt):
    import siirl_amd.padding as P

    ids, mask = _case(B, S, B + S)
    h = np.random.default_rng(3).standard_normal((B, S, 2)).astype(np.float32)
    rm_o, idx_o, cu_o, mx_o, sl_o = OP.unpad_input(h, mask)
    rm, idx, cu, mx, sl = P.unpad_input(torch.from_numpy(h).to(dev), torch.from_numpy(mask).to(dev).to(mdt))
    assert idx.dtype == torch.int64 and cu.dtype == torch.int32 and sl.dtype == torch.int32
    assert np.array_equal(idx.cpu().numpy(), idx_o) and np.array_equal(cu.cpu().numpy(), cu_o)
    assert mx == mx_o and np.array_equal(sl.cpu().numpy(), sl_o)
    assert np.array_equal(rm.cpu().numpy(), rm_o)
    back = P.pad_input(rm, idx, B, S)
    assert np.array_equal(back.cpu().numpy(), OP.pad_input(rm_o, idx_o, B, S))


def test_empty_rows_and_empty_batch(dev):
    import siirl_amd.padding as P

    mask = np.array([[0, 0, 0], [0, 1, 0], [0, 0, 0]])
    rm, idx, cu, mx, sl = P.unpad_input(torch.arange(9.0, device=dev).reshape(3, 3, 1), torch.from_numpy(mask).to(dev))
    assert idx.tolist() == [4] and cu.tolist() == [0, 0, 1, 1] and mx == 1 and rm.flatten().tolist() == [4.0]
    rm, idx, cu, mx, sl = P.unpad_input(torch.arange(9.0, device=dev).reshape(3, 3, 1), torch.zeros(3, 3, dtype=torch.int64, device=dev))
    assert idx.numel() == 0 and rm.shape == (0, 1) and cu.tolist() == [0, 0, 0, 0] and mx == 0
    assert float(P.pad_input(rm, idx, 3, 3).abs().sum()) == 0.0


@pytest.mark.parametrize("B,S", [(4, 64), (16, 2048)])
def test_ids_and_rolled_labels(dev, B, S):
    import siirl_amd.padding as P

    ids, mask = _case(B, S, 7 * B + S)
    rm_o, idx_o, cu_o, mx_o, _ = OP.unpad_input(ids[..., None], mask)
    rm, rolled, idx, cu, mx = P.unpad_ids_and_labels(torch.from_numpy(ids).to(dev), torch.from_numpy(mask).to(dev))
    assert rm.shape == (1, idx_o.size)
    assert np.array_equal(rm[0].cpu().numpy(), rm_o[:, 0])
    assert np.array_equal(rolled.cpu().numpy(), OP.rolled_labels(rm_o[:, 0]))
    assert np.array_equal(idx.cpu().numpy(), idx_o) and np.array_equal(cu.cpu().numpy(), cu_o) and mx == mx_o


@pytest.mark.parametrize("B,S,L", [(3, 9, 4), (8, 1300, 512), (2, 5, 4), (4, 600, 599)])
def test_pad_and_slice_response(dev, B, S, L):
    import siirl_amd.padding as P

    ids, mask = _case(B, S, S + L, full_first=False)
    _, idx_o, *_ = OP.unpad_input(ids[..., None], mask)
    v = np.random.default_rng(5).standard_normal(idx_o.size).astype(np.float32)
    want = OP.pad_and_slice_response(v, idx_o, B, S, L)
    x = torch.from_numpy(v).to(dev).requires_grad_(True)
    idx = torch.from_numpy(idx_o).to(dev)
    got = P.pad_and_slice_response(x, idx, B, S, L)
    assert got.shape == (B, L) and np.array_equal(got.detach().cpu().numpy(), want)
    # backward == the reference's composition under autograd
    g = torch.from_numpy(np.random.default_rng(6).standard_normal((B, L)).astype(np.float32))
    got.backward(g.to(dev))
    x_o = torch.from_numpy(v).requires_grad_(True)
    full = torch.zeros(B * S).index_put((torch.from_numpy(idx_o),), x_o).reshape(B, S)
    full[:, -L - 1:-1].backward(g)
    assert torch.equal(x.grad.cpu(), x_o.grad)
    with pytest.raises(ValueError):
        P.pad_and_slice_response(x, idx, B, S, S)


def test_index_first_axis_autograd_and_dtypes(dev):
    import siirl_amd.padding as P

    x = torch.randn(50, 6, device=dev, dtype=torch.bfloat16, requires_grad=True)
    idx = torch.tensor([3, 3, 49, 0, 17], device=dev)
    y = P.index_first_axis(x, idx)
    assert torch.equal(y, x.detach()[idx])
    y.float().sum().backward()
    want = torch.zeros(50, 6)
    want[[3, 49, 0, 17]] = 1.0  # a repeated index: the scatter keeps one copy (the reference's pad_input does too)
    assert torch.equal((x.grad.float().cpu() != 0), want != 0)
    with pytest.raises(ValueError):
        P.index_first_axis(torch.zeros(4, 1, dtype=torch.bfloat16, device=dev), idx[:1] * 0)
    with pytest.raises(RuntimeError):
        P.unpad_input(torch.zeros(2, 2, 1), torch.ones(2, 2))


def test_indices_outside_the_tensor_touch_no_memory(dev):
    """An index outside the indexed tensor reads as zero (gathers; -1 for token ids) or is dropped (scatters)."""
    import siirl_amd.padding as PD

    x = torch.arange(12, dtype=torch.float32, device=dev).reshape(6, 2)
    idx = torch.tensor([0, 5, 6, -1, 2 ** 40, 3], device=dev)
    got = PD.index_first_axis(x, idx).cpu()
    want = torch.tensor([[0., 1.], [10., 11.], [0., 0.], [0., 0.], [0., 0.], [6., 7.]])
    assert torch.equal(got, want)
    out = PD.pad_input(torch.ones(6, 2, device=dev), idx, 2, 3).cpu().reshape(6, 2)
    assert torch.equal(out[:, 0], torch.tensor([1., 0., 0., 1., 0., 1.]))
    B, S, L = 2, 6, 3
    vals = torch.arange(1, 7, dtype=torch.float32, device=dev).requires_grad_(True)
    bad = torch.tensor([2, 3, 12, -5, 9, 2 ** 41], device=dev)  # window of row 0: positions 2..4; row 1: 8..10
    w = PD.pad_and_slice_response(vals, bad, B, S, L)
    assert torch.equal(w.detach().cpu(), torch.tensor([[1., 2., 0.], [0., 5., 0.]]))
    w.sum().backward()
    assert torch.equal(vals.grad.cpu(), torch.tensor([1., 1., 0., 0., 1., 0.]))


@pytest.mark.parametrize("B,L", [(4, 7), (1, 1), (33, 64), (17, 65), (300, 1000), (2, 70001)])
@pytest.mark.parametrize("idt", [torch.int64, torch.int32])
def test_response_mask_from_eos(dev, B, L, idt):
    import siirl_amd.torch_functional as TF

    rng = np.random.default_rng(B * 31 + L)
    ids = rng.integers(0, max(L // 3, 4), (B, L)).astype(np.int64)
    ids[0, :] = 3  # a row with no end-of-sequence token
    x = torch.from_numpy(ids).to(dev).to(idt)
    for eos in (1, [1, 2], [0, 2, 1, 7, 9]):
        want = OP.get_response_mask(ids, eos)
        got = TF.get_response_mask(x, eos)
        assert got.dtype == torch.int64 and np.array_equal(got.cpu().numpy(), want), (B, L, eos)
    assert np.array_equal(TF.get_eos_mask(x, 2).cpu().numpy(), OP.get_response_mask(ids, 2))
    want = OP.get_response_mask(ids, 1)
    for dt in (torch.bool, torch.int32, torch.float32, torch.bfloat16, torch.float16, torch.uint8):
        got = TF.get_response_mask(x, 1, dtype=dt)
        assert got.dtype == dt and np.array_equal(got.float().cpu().numpy(), want.astype(np.float32))


def test_response_mask_docstring_examples_and_errors(dev):
    import siirl_amd.torch_functional as TF

    ids = torch.tensor([[20, 10, 34, 1, 0, 0, 0], [78, 0, 76, 2, 1, 0, 0], [23, 98, 1, 0, 0, 0, 0],
                        [33, 3, 98, 45, 1, 0, 0]], device=dev)
    assert TF.get_response_mask(ids, 1).tolist() == [[1, 1, 1, 1, 0, 0, 0], [1, 1, 1, 1, 1, 0, 0], [1, 1, 1, 0, 0, 0, 0],
                                                     [1, 1, 1, 1, 1, 0, 0]]
    assert TF.get_response_mask(ids, [1, 2]).tolist() == [[1, 1, 1, 1, 0, 0, 0], [1, 1, 1, 1, 0, 0, 0],
                                                          [1, 1, 1, 0, 0, 0, 0], [1, 1, 1, 1, 1, 0, 0]]
    assert TF.get_response_mask(ids[:0], 1).shape == (0, 7)
    with pytest.raises(ValueError):
        TF.get_response_mask(ids, list(range(17)))
    with pytest.raises(RuntimeError):
        TF.get_response_mask(ids.cpu(), 1)
    with pytest.raises(TypeError):
        TF.get_response_mask(ids.float(), 1)


def test_unpad_data_and_remove_pad_token(dev):
    import siirl_amd.torch_functional as TF

    ids, mask = _case(9, 130, 4)
    # left-padded rows, as remove_pad_token expects
    for b in range(9):
        n = int(mask[b].sum())
        mask[b] = 0
        mask[b, 130 - n:] = 1
    idx_o, cu_o, mx_o = OP.get_unpad_data(mask)
    idx, cu, mx = TF.get_unpad_data(torch.from_numpy(mask).to(dev))
    assert np.array_equal(idx.cpu().numpy(), idx_o) and np.array_equal(cu.cpu().numpy(), cu_o) and mx == mx_o
    assert TF.remove_pad_token(torch.from_numpy(ids).to(dev), torch.from_numpy(mask).to(dev)) == \
        OP.remove_pad_token(ids, mask)


@pytest.mark.parametrize("B,S,L,V,dt", [(3, 12, 4, 29, torch.float32), (4, 300, 128, 1531, torch.bfloat16),
                                        (2, 40, 39, 4096, torch.float16)])
def test_response_logprobs_padded_and_packed(dev, B, S, L, V, dt):
    """log_probs_from_logits_response / _response_rmpad / _all_rmpad against the oracle (1e-3 absolute, the
    log-prob tolerance), values and the gradient with respect to the logits."""
    import siirl_amd.torch_functional as TF
    from oracle import torch_functional as OT

    g = torch.Generator().manual_seed(B * S + L)
    logits = (torch.randn(B, S, V, generator=g) * 2).to(dt)
    ids = torch.randint(0, V, (B, S), generator=g)
    mask = torch.ones(B, S, dtype=torch.int64)
    mask[0, :S // 3] = 0
    mask[B - 1, :1] = 0
    w = torch.randn(B, L, generator=g)

    lo = logits.float().clone().requires_grad_(True)
    want = OT.log_probs_from_logits_response(ids, lo, L)
    (want * w).sum().backward()
    x = logits.detach().to(dev).requires_grad_(True)
    got = TF.log_probs_from_logits_response(ids.to(dev), x, L)
    assert got.shape == (B, L) and (got.detach().cpu() - want.detach()).abs().max() < 1e-3
    (got * w.to(dev)).sum().backward()
    assert (x.grad.float().cpu() - lo.grad).abs().max() < (1e-5 if dt == torch.float32 else 1e-2)

    idx = torch.nonzero(mask.flatten()).flatten()
    packed = logits.reshape(B * S, V)[idx]
    po = packed.float().clone().requires_grad_(True)
    want = OT.log_probs_from_logits_response_rmpad(ids, mask, po, L)
    (want * w).sum().backward()
    for route in ("response_rmpad", "all_rmpad"):
        p = packed.detach().to(dev).requires_grad_(True)
        if route == "response_rmpad":
            got = TF.log_probs_from_logits_response_rmpad(ids.to(dev), mask.to(dev), p, L)
        else:
            got = TF.log_probs_from_logits_all_rmpad(ids.flatten()[idx][None].to(dev), p, idx.to(dev), B, S, L)
        assert got.shape == (B, L) and (got.detach().cpu() - want.detach()).abs().max() < 1e-3, route
        (got * w.to(dev)).sum().backward()
        # logprobs_from_logits defaults to the in-place backward: the gradient comes back in the logits' storage
        assert (p.grad.float().cpu() - po.grad).abs().max() < (1e-5 if dt == torch.float32 else 1e-2), route


@pytest.mark.parametrize("cols,dtype", [(1, torch.float32), (3, torch.float32), (4, torch.float32), (2, torch.bfloat16),
                                        (8, torch.bfloat16), (100, torch.float32), (511, torch.float32),
                                        (512, torch.float32), (1000, torch.int64), (4100, torch.float32),
                                        (8192, torch.bfloat16)])
def test_row_moves_every_size_and_alignment(dev, cols, dtype):
    """index_first_axis / pad_input over rows of 4 bytes to 32 KB: 4-byte and 16-byte units, short rows that share
    workgroups and long rows cut into pieces, a source view that starts off a 16-byte boundary, repeated and unsorted
    indices: equal to torch's own indexing, bit for bit."""
    import siirl_amd.padding as PD

    g = torch.Generator().manual_seed(cols)
    n_src, n = 77, 50
    x = (torch.randn(n_src + 1, cols, generator=g) * 100).to(dtype).to(dev)
    idx = torch.randint(0, n_src, (n,), generator=g).to(dev)
    assert torch.equal(PD.index_first_axis(x[:n_src], idx), x[:n_src][idx])
    off = x.flatten()[1:1 + n_src * cols].view(n_src, cols)  # rows start 2 or 4 or 8 bytes off the allocation
    if (off.data_ptr() % 4) == 0:
        assert torch.equal(PD.index_first_axis(off, idx), off[idx])
    # pad_input: distinct target rows, the others zero
    rows = torch.randperm(n_src, generator=g)[:n].to(dev)
    src = x[:n]
    out = PD.pad_input(src, rows, 7, 11)  # 77 rows
    want = torch.zeros(n_src, cols, dtype=dtype, device=dev)
    want[rows] = src
    assert torch.equal(out.reshape(n_src, cols), want)


def test_row_moves_ignore_indices_outside_the_tensor(dev):
    from siirl_amd import _lib

    lib = _lib.lib()
    for cols in (2, 64, 3000):
        x = torch.randn(10, cols, device=dev)
        idx = torch.tensor([3, -1, 9, 10, 0, 2 ** 40], device=dev)
        out = torch.full((6, cols), 7.0, device=dev)
        rc = lib.siirl_gather_rows(_lib.ptr(x), _lib.ptr(idx), 6, cols * 4, 10, _lib.ptr(out), _lib.current_stream(dev))
        assert rc == 0
        want = torch.stack([x[3], torch.zeros(cols, device=dev), x[9], torch.zeros(cols, device=dev), x[0],
                            torch.zeros(cols, device=dev)])
        assert torch.equal(out, want)
        dst = torch.full((10, cols), 7.0, device=dev)
        rc = lib.siirl_scatter_rows(_lib.ptr(x[:6].contiguous()), _lib.ptr(idx), 6, cols * 4, 10, _lib.ptr(dst),
                                    _lib.current_stream(dev))
        assert rc == 0
        want = torch.zeros(10, cols, device=dev)
        want[3], want[9], want[0] = x[0], x[2], x[4]
        assert torch.equal(dst, want)

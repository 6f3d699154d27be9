"""``torch.library`` registration of the HIP entry points as ``torch.ops.siirl_hip.*``.

Each op is a thin shim: it checks shapes, allocates outputs with torch, and hands raw device
pointers plus the current stream to the C ABI.  Fake (meta) kernels give shapes to FakeTensor
tracing; there is deliberately no CPU kernel."""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib

_NS = "siirl_hip"


def _require_gpu(t: torch.Tensor, name: str):
    if not t.is_cuda:
        raise RuntimeError(f"siirl_amd: `{name}` is on {t.device}; these ops run on the GPU only (no CPU fallback)")


def row_blocks(x: torch.Tensor):
    """Splits a ``(..., V)`` tensor with unit inner stride into blocks of uniformly strided rows:
    yields ``(element_offset, n_rows, row_stride)``.  A contiguous tensor, or a row-sliced 2-D view,
    is a single block; a ``[B, S, V]`` slice along ``S`` gives ``B`` blocks."""
    V = x.shape[-1]
    if x.stride(-1) != 1 and V > 1:
        raise ValueError("siirl_amd: the vocab axis of logits must have stride 1")
    lead_shape, lead_stride = list(x.shape[:-1]), list(x.stride()[:-1])
    # drop size-1 axes, then peel trailing leading-axes that collapse into one uniformly strided axis
    dims = [(n, s) for n, s in zip(lead_shape, lead_stride) if n != 1]
    if not dims:
        yield 0, 1 if x.numel() else 0, max(V, 1)
        return
    n_in, s_in = dims[-1]
    k = len(dims) - 1
    while k > 0 and dims[k - 1][1] == n_in * s_in:
        n_in *= dims[k - 1][0]
        k -= 1
    outer = dims[:k]
    if s_in < V:
        raise ValueError("siirl_amd: overlapping logits rows are not supported")

    def rec(level, off):
        if level == len(outer):
            yield off, n_in, s_in
            return
        n, s = outer[level]
        for i in range(n):
            yield from rec(level + 1, off + i * s)

    yield from rec(0, 0)


@torch.library.custom_op(f"{_NS}::logprob_entropy_fwd", mutates_args=())
def logprob_entropy_fwd(logits: torch.Tensor, labels: Optional[torch.Tensor], inv_temperature: float,
                        want_entropy: bool) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """-> (logprob, entropy, lse, ex), fp32, shape ``logits.shape[:-1]``; tensors not requested are empty."""
    _require_gpu(logits, "logits")
    lead = logits.shape[:-1]
    V = logits.shape[-1]
    dev = logits.device
    want_lp = labels is not None
    if want_lp:
        if labels.shape != lead:
            raise ValueError(f"labels shape {tuple(labels.shape)} does not match logits {tuple(logits.shape)}")
        labels = labels.to(device=dev, dtype=torch.int64).contiguous()
    f32 = dict(dtype=torch.float32, device=dev)
    lp = torch.empty(lead if want_lp else (0,), **f32)
    ent = torch.empty(lead if want_entropy else (0,), **f32)
    ex = torch.empty(lead if want_entropy else (0,), **f32)
    lse = torch.empty(lead, **f32)
    L = _lib.lib()
    es = logits.element_size()
    code = _lib.dtype_code(logits.dtype)
    stream = _lib.current_stream(dev)
    base = logits.data_ptr()
    done = 0
    with torch.cuda.device(dev):
        for off, rows, stride in row_blocks(logits):
            if rows == 0:
                continue
            o4 = done * 4
            rc = L.siirl_logprob_entropy_fwd(
                base + off * es, code, rows, V, stride,
                labels.data_ptr() + done * 8 if want_lp else None, inv_temperature,
                lp.data_ptr() + o4 if want_lp else None,
                ent.data_ptr() + o4 if want_entropy else None,
                lse.data_ptr() + o4,
                ex.data_ptr() + o4 if want_entropy else None, stream)
            _lib.check(rc, "siirl_logprob_entropy_fwd")
            done += rows
    return lp, ent, lse, ex


@logprob_entropy_fwd.register_fake
def _(logits, labels, inv_temperature, want_entropy):
    lead = logits.shape[:-1]
    mk = lambda shape: logits.new_empty(shape, dtype=torch.float32)  # noqa: E731
    return (mk(lead if labels is not None else (0,)), mk(lead if want_entropy else (0,)), mk(lead),
            mk(lead if want_entropy else (0,)))


def _bwd_launch(logits, labels, inv_temperature, lse, ex, g_logprob, g_entropy, out, skip_zero_rows):
    _require_gpu(logits, "logits")
    dev = logits.device
    V = logits.shape[-1]
    es = logits.element_size()
    code = _lib.dtype_code(logits.dtype)
    L = _lib.lib()
    stream = _lib.current_stream(dev)
    f = lambda t: None if t is None else t.to(device=dev, dtype=torch.float32).contiguous()  # noqa: E731
    g_logprob, g_entropy, lse, ex = f(g_logprob), f(g_entropy), f(lse), f(ex)
    if labels is not None:
        labels = labels.to(device=dev, dtype=torch.int64).contiguous()
    in_blocks = list(row_blocks(logits))
    if out is logits:
        out_blocks = in_blocks
    else:  # a fresh contiguous tensor: rows follow one another whatever the blocking of the input
        if not out.is_contiguous() or out.shape != logits.shape:
            raise ValueError("siirl_amd: dlogits must be contiguous and shaped like logits")
        out_blocks, r = [], 0
        for _, rows, _ in in_blocks:
            out_blocks.append((r * V, rows, V))
            r += rows
    flags = _lib.BWD_SKIP_ZERO_ROWS if skip_zero_rows else 0
    done = 0
    with torch.cuda.device(dev):
        for (off, rows, stride), (ooff, _, ostride) in zip(in_blocks, out_blocks):
            if rows == 0:
                continue
            o4 = done * 4
            rc = L.siirl_logprob_entropy_bwd(
                logits.data_ptr() + off * es, code, rows, V, stride,
                labels.data_ptr() + done * 8 if g_logprob is not None else None, inv_temperature,
                lse.data_ptr() + o4, ex.data_ptr() + o4 if g_entropy is not None else None,
                g_logprob.data_ptr() + o4 if g_logprob is not None else None,
                g_entropy.data_ptr() + o4 if g_entropy is not None else None,
                out.data_ptr() + ooff * es, ostride, flags, stream)
            _lib.check(rc, "siirl_logprob_entropy_bwd")
            done += rows


@torch.library.custom_op(f"{_NS}::logprob_entropy_bwd", mutates_args=())
def logprob_entropy_bwd(logits: torch.Tensor, labels: Optional[torch.Tensor], inv_temperature: float,
                        lse: torch.Tensor, ex: Optional[torch.Tensor], g_logprob: Optional[torch.Tensor],
                        g_entropy: Optional[torch.Tensor], skip_zero_rows: bool) -> torch.Tensor:
    """Gradient w.r.t. ``logits`` as a fresh contiguous tensor of the logits' dtype and shape."""
    out = torch.empty(logits.shape, dtype=logits.dtype, device=logits.device)
    _bwd_launch(logits, labels, inv_temperature, lse, ex, g_logprob, g_entropy, out, skip_zero_rows)
    return out


@logprob_entropy_bwd.register_fake
def _(logits, labels, inv_temperature, lse, ex, g_logprob, g_entropy, skip_zero_rows):
    return logits.new_empty(logits.shape)


@torch.library.custom_op(f"{_NS}::logprob_entropy_bwd_", mutates_args=("logits",))
def logprob_entropy_bwd_(logits: torch.Tensor, labels: Optional[torch.Tensor], inv_temperature: float,
                         lse: torch.Tensor, ex: Optional[torch.Tensor], g_logprob: Optional[torch.Tensor],
                         g_entropy: Optional[torch.Tensor], skip_zero_rows: bool) -> None:
    """In-place variant: overwrites ``logits`` with its own gradient."""
    _bwd_launch(logits, labels, inv_temperature, lse, ex, g_logprob, g_entropy, logits, skip_zero_rows)

"""The C ABI (CPU only, no kernel is launched): libsiirl_hip.so loads, exports every function that
include/siirl_hip.h declares, the ctypes table covers exactly those, and argument validation reports errors."""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "siirl_hip.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(siirl_[a-z0-9_]+)\s*\(", text)))


def _lib():
    from siirl_amd import _lib

    if not _lib.LIB_PATH.exists():
        from siirl_amd import build

        build.build()
    return _lib


def test_header_symbols_are_exported_and_bound():
    L = _lib()
    names = _declared()
    assert len(names) >= 14
    h = L.lib()
    for n in names:
        assert hasattr(h, n), f"{n} is declared in siirl_hip.h but not exported"
    assert sorted(L.SIGNATURES) == names, "ctypes table and header disagree"
    assert h.siirl_hip_abi_version() == L.ABI_VERSION
    assert f"#define SIIRL_HIP_ABI_VERSION {L.ABI_VERSION}\n" in open(HEADER).read()


def test_every_entry_point_cites_the_reference():
    text = open(HEADER).read()
    for n in _declared():
        if n == "siirl_actor_loss_fwd_static":  # the allocation-free variant: says that the reference has no such thing
            pos = text.index(n + "(")
            assert "no counterpart in the reference" in text[text.rfind("/*", 0, pos):pos]
            continue
        if n in ("siirl_hip_abi_version", "siirl_hip_last_error", "siirl_agg_loss_bwd", "siirl_actor_loss_bwd",
                 "siirl_kl_penalty_bwd", "siirl_masked_reduce_bwd", "siirl_actor_loss_cov_bwd",
                 "siirl_range_select_write") or n.endswith("_workspace_bytes") or n.endswith("_workspace_bytes_dtype") or n.endswith("_logits_bytes"):
            continue  # utilities and backward halves documented with their forward
        pos = text.index(n + "(")
        comment = text[text.rfind("/*", 0, pos):pos]
        assert "Replaces:" in comment and re.search(r"siirl/[\w/]+\.py:\d+", comment), f"{n} lacks a reference citation"


def test_argument_validation_without_gpu():
    L = _lib()
    h = L.lib()
    buf = (ctypes.c_float * 64)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    # V = 0
    assert h.siirl_logprob_entropy_fwd(p, L.BF16, 4, 0, 0, p, 1.0, p, p, p, p, None) == -1
    assert b"V=0" in h.siirl_hip_last_error()
    # unsupported logits dtype
    assert h.siirl_logprob_entropy_fwd(p, L.I64, 4, 8, 8, p, 1.0, p, p, p, p, None) == -1
    # labels without logprob
    assert h.siirl_logprob_entropy_fwd(p, L.F32, 1, 8, 8, p, 1.0, None, p, p, p, None) == -1
    # backward: overlapping but distinct buffers
    q = ctypes.c_void_p(p.value + 8)
    assert h.siirl_logprob_entropy_bwd(p, L.F32, 1, 8, 8, p, 1.0, p, p, p, p, q, 8, 0, None) == -1
    assert b"overlaps" in h.siirl_hip_last_error()
    # loss: bad aggregation mode / clip_ratio_c / workspace
    assert h.siirl_agg_loss_fwd(p, p, L.F32, 2, 4, 9, p, p, p, 1 << 20, None) == -1
    assert b"Invalid loss_agg_mode" in h.siirl_hip_last_error()
    assert h.siirl_actor_loss_fwd(p, p, p, p, L.F32, None, None, None, 2, 4, 0, 0.2, 0.2, 1.0, 20.0, 0, 0.0, 0, 0, 0.0,
                                  0.0, 1.0, p, p, p, p, 1 << 20, None) == -1
    assert b"clip_ratio_c" in h.siirl_hip_last_error()
    assert h.siirl_actor_loss_fwd(p, p, p, p, L.F32, None, None, None, 2, 4, 9, 0.2, 0.2, 3.0, 20.0, 0, 0.0, 0, 0, 0.0,
                                  0.0, 1.0, p, p, p, p, 1 << 20, None) == -1
    assert b"Unsupported loss mode" in h.siirl_hip_last_error()
    assert h.siirl_actor_loss_fwd(p, p, p, p, L.F32, None, None, None, 2, 4, 4, 0.2, 0.2, 3.0, 20.0, 0, 0.0, 0, 0, 0.0,
                                  0.0, 1.0, p, p, None, p, 1 << 20, None) == -1  # geo_mean needs row_s
    # the allocation-free variant refuses what its fixed buffer cannot hold, before any device call
    assert h.siirl_actor_loss_fwd_static(p, p, p, p, L.F32, None, None, None, 1 << 20, 4096, 0, 0.2, 0.2, 3.0, 20.0, 0,
                                         0.0, 0, 0, 0.0, 0.0, 1.0, p, p, p, 0, None) == -4
    assert b"static buffer" in h.siirl_hip_last_error()
    for bad_slot in (-1, 4):  # and a slot outside its slices
        assert h.siirl_actor_loss_fwd_static(p, p, p, p, L.F32, None, None, None, 2, 4, 0, 0.2, 0.2, 3.0, 20.0, 0, 0.0, 0,
                                             0, 0.0, 0.0, 1.0, p, p, p, bad_slot, None) == -1
        assert b"slot" in h.siirl_hip_last_error()
    # the covariance losses: their two modes go through their own entry points and nowhere else
    assert h.siirl_actor_loss_fwd(p, p, p, p, L.F32, None, None, None, 2, 4, 5, 0.2, 0.2, 3.0, 20.0, 0, 0.0, 0, 0, 0.0,
                                  0.0, 1.0, p, p, p, p, 1 << 20, None) == -1
    assert b"Unsupported loss mode" in h.siirl_hip_last_error()
    assert h.siirl_actor_loss_cov_fwd(p, p, p, p, L.F32, None, None, None, p, 2, 4, 0, 0.2, 0.2, 0, 0.0, 0, 0, 0.0, 0.0,
                                      1.0, p, p, p, 1 << 20, None) == -1
    assert b"per-token selection" in h.siirl_hip_last_error()
    assert h.siirl_actor_loss_cov_fwd(p, p, p, p, L.F32, None, None, None, None, 2, 4, 5, 0.2, 0.2, 0, 0.0, 0, 0, 0.0,
                                      0.0, 1.0, p, p, p, 1 << 20, None) == -1
    assert b"token_aux" in h.siirl_hip_last_error()
    assert h.siirl_actor_loss_cov_bwd(p, p, p, p, p, L.F32, None, None, None, p, 2, 4, 6, 0.2, 0.2, 9, 0.0, 0, 0, 0.0,
                                      0.0, 1.0, p, p, p, None, None) == -1
    assert h.siirl_cov_scores(p, p, p, p, L.F32, 2, 4, 0, 0.2, 0.2, p, p, p, 1 << 20, None) == -1
    assert b"kl_cov and clip_cov" in h.siirl_hip_last_error()
    assert h.siirl_cov_scores(None, p, p, p, L.F32, 2, 4, 6, 0.2, 0.2, p, p, p, 1 << 20, None) == -1  # clip_cov: old
    assert h.siirl_cov_scores(p, p, p, p, L.F32, 2, 4, 6, 0.2, 0.2, p, p, p, 8, None) == -4
    assert h.siirl_cov_workspace_bytes() > 0
    q2 = ctypes.c_void_p(p.value + 64)
    assert h.siirl_topk_mark(p, 8, 9, 1.0, q2, p, 1 << 20, None) == -1  # k > n
    assert h.siirl_topk_mark(p, 8, 2, 1.0, p, p, 1 << 20, None) == -1  # marks alias scores
    assert h.siirl_topk_mark(p, 8, 2, 1.0, q2, p, 8, None) == -4
    assert h.siirl_topk_mark(p, 0, 0, 1.0, q2, None, 0, None) == 0  # nothing to mark: no workspace, no launch
    assert h.siirl_topk_mark_workspace_bytes() > 0
    assert h.siirl_range_select_count(p, 8, 0.0, 1.0, None, p, 1 << 20, None) == -1  # no place for the count
    assert h.siirl_range_select_count(p, 8, 0.0, 1.0, p, p, 8, None) == -4
    assert h.siirl_range_select_write(p, 8, 0.0, 1.0, p, None, 4, None) == -1
    assert h.siirl_range_select_write(p, 8, 0.0, 1.0, p, None, 0, None) == 0  # an empty list: nothing to write
    assert h.siirl_range_select_workspace_bytes() > 0
    assert h.siirl_value_loss_fwd(p, p, p, p, L.F32, 2, 4, 0.5, 7, p, p, p, 1 << 20, None) == -1
    assert h.siirl_gae_advantage_return(p, p, p, L.F32, 2, 4, 1.0, 1.0, p, p, p, p, 8, 0, None) == -1  # adv == returns
    q2 = ctypes.c_void_p(p.value + 64)
    assert h.siirl_gae_advantage_return(p, p, p, L.F32, 2, 4, 1.0, 1.0, p, q2, p, p, 1 << 20, 7, None) == -1
    assert b"scan order" in h.siirl_hip_last_error()
    assert h.siirl_gae_workspace_bytes(4, 8192) >= h.siirl_whiten_workspace_bytes()
    assert h.siirl_masked_whiten(p, p, L.F64, 4, 1, p, p, p, 1 << 20, None) == -1
    assert h.siirl_whiten_workspace_bytes() > 0
    assert h.siirl_agg_loss_fwd(p, p, L.F32, 2, 4, 0, p, p, p, 8, None) == -4
    assert h.siirl_loss_workspace_bytes(2, 4) > 0 and h.siirl_loss_workspace_bytes(0, 4) == 0
    assert h.siirl_kl_penalty_fwd(p, p, 4, 7, p, None) == -1
    assert h.siirl_group_keep_mask(p, L.BF16, p, 4, p, None, None) == -1
    eos = (ctypes.c_int64 * 17)()
    assert h.siirl_eos_response_mask(p, L.F32, 2, 4, eos, 1, p, L.I64, None) == -1  # ids must be integers
    assert h.siirl_eos_response_mask(p, L.I64, 2, 4, eos, 17, p, L.I64, None) == -1
    assert b"n_eos" in h.siirl_hip_last_error()
    assert h.siirl_eos_response_mask(p, L.I64, 2, 4, eos, 1, p, L.F64, None) == -1
    assert h.siirl_eos_response_mask(p, L.I64, 0, 4, eos, 1, p, L.I64, None) == 0  # nothing to do, no launch
    with pytest.raises(ValueError):
        L.check(-1, "x")
    with pytest.raises(NotImplementedError):
        L.check(-2, "x")
    with pytest.raises(L.SiirlHipError):
        L.check(-3, "x")


def test_size_queries_agree_with_the_host_side():
    """Pure size arithmetic (no GPU): the buffer the Python layer plans for the parked logits is the one the library
    asks for, and the backward scratch grows with the requested gradients."""
    L = _lib()
    h = L.lib()
    import siirl_amd.fused_linear as FL

    for T, V in ((1, 1), (256, 256), (257, 255), (16384, 152064), (70, 500)):
        assert h.siirl_fused_linear_saved_logits_bytes(T, V) == FL._saved_logits_bytes(T, V)
    assert h.siirl_fused_linear_saved_logits_bytes(0, 5) == 0
    both = h.siirl_fused_linear_bwd_workspace_bytes(512, 128, 4096, 1, 1)
    assert both > h.siirl_fused_linear_bwd_workspace_bytes(512, 128, 4096, 1, 0) > 0
    assert both > h.siirl_fused_linear_bwd_workspace_bytes(512, 128, 4096, 0, 1) > 0
    # the row-subset backward: the dense workspace for its rows plus the gathered operands
    rows = h.siirl_fused_linear_bwd_rows_workspace_bytes(100, 128, 4096, 1, 1)
    assert rows > h.siirl_fused_linear_bwd_workspace_bytes(100, 128, 4096, 1, 1)
    assert h.siirl_fused_linear_bwd_rows_workspace_bytes(0, 128, 4096, 1, 1) < 4096
    assert h.siirl_fused_linear_bwd_rows_workspace_bytes(-1, 128, 4096, 1, 1) == 0
    assert h.siirl_fused_linear_fwd_workspace_bytes(512, 128, 4096) > 512 * 128 * 2


def test_python_constants_transcribe_the_header():
    """The enum values and defines that the Python layer repeats by value are those of the header."""
    L = _lib()
    text = open(HEADER).read()

    def enum_value(name):
        m = re.search(rf"\b{name}\s*=\s*(-?\d+)", text)
        assert m, name
        return int(m.group(1))

    assert re.search(r"#define SIIRL_LABEL_SKIP_ROW \((-?\d+)\)", text).group(1) == str(L.LABEL_SKIP_ROW)
    assert re.search(r"#define SIIRL_MARFT_MAX_AGENTS (\d+)", text).group(1) == str(L.MARFT_MAX_AGENTS)
    for name, value in (("SIIRL_MARFT_STORE_FLOAT", L.MARFT_STORE_FLOAT), ("SIIRL_MARFT_STORE_TRUNCATED", L.MARFT_STORE_TRUNCATED),
                        ("SIIRL_MARFT_STORE_NONZERO", L.MARFT_STORE_NONZERO), ("SIIRL_F32", L.F32), ("SIIRL_BF16", L.BF16)):
        assert enum_value(name) == value, name
    import siirl_amd.core_algos as CA

    for name, value in (("SIIRL_LOSS_VANILLA", CA.LOSS_VANILLA), ("SIIRL_LOSS_GSPO", CA.LOSS_GSPO),
                        ("SIIRL_LOSS_KL_COV", CA.LOSS_KL_COV), ("SIIRL_LOSS_CLIP_COV", CA.LOSS_CLIP_COV)):
        assert enum_value(name) == value, name

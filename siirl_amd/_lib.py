"""ctypes binding of ``libsiirl_hip.so`` (the C ABI declared in ``include/siirl_hip.h``).

There is no fallback: if the library is missing or a call fails, an exception is raised."""

from __future__ import annotations

import ctypes as C
import threading
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libsiirl_hip.so"

# dtype codes of siirl_dtype
F32, BF16, F16, F64, I64, I32, U8 = range(7)
MARFT_MAX_AGENTS = 16  # SIIRL_MARFT_MAX_AGENTS
LABEL_SKIP_ROW = -101  # SIIRL_LABEL_SKIP_ROW
MARFT_STORE_FLOAT, MARFT_STORE_TRUNCATED, MARFT_STORE_NONZERO = range(3)  # siirl_marft_store
MAX_EOS_TOKENS = 16  # SIIRL_MAX_EOS_TOKENS
ABI_VERSION = 1010  # SIIRL_HIP_ABI_VERSION of include/siirl_hip.h that SIGNATURES below transcribes
BWD_SKIP_ZERO_ROWS = 1

_p, _i64, _i32, _f32, _u32, _sz, _f64 = (C.c_void_p, C.c_int64, C.c_int, C.c_float, C.c_uint32, C.c_size_t,
                                        C.c_double)

# name -> (restype, argtypes); one entry per function declared in include/siirl_hip.h
SIGNATURES = {
    "siirl_hip_abi_version": (_i32, []),
    "siirl_hip_last_error": (C.c_char_p, []),
    "siirl_logprob_entropy_fwd": (_i32, [_p, _i32, _i64, _i64, _i64, _p, _f32, _p, _p, _p, _p, _p]),
    "siirl_logprob_entropy_bwd": (_i32, [_p, _i32, _i64, _i64, _i64, _p, _f32, _p, _p, _p, _p, _p, _i64, _u32, _p]),
    "siirl_logprob_entropy_fwd_bwd": (_i32, [_p, _i32, _i64, _i64, _i64, _p, _f32, _p, _p, _p, _p, _p, _i64, _p]),
    "siirl_actor_step_fused": (_i32, [_p, _i32, _i64, _i64, _i64, _p, _f32, _p, _p, _p, _p, _p, _p, _i32, _f32, _f32,
                                      _f32, _f32, _f32, _i32, _i32, _f32, _f32, _f32, _p, _p, _p, _i64, _p]),
    "siirl_agg_weights": (_i32, [_p, _i32, _i64, _i64, _i32, _p, _p, _p, _p, _sz, _p]),
    "siirl_loss_workspace_bytes": (_sz, [_i64, _i64]),
    "siirl_agg_loss_fwd": (_i32, [_p, _p, _i32, _i64, _i64, _i32, _p, _p, _p, _sz, _p]),
    "siirl_agg_loss_bwd": (_i32, [_p, _p, _i32, _p, _p, _i64, _i64, _i32, _p, _p]),
    "siirl_actor_loss_fwd": (_i32, [_p, _p, _p, _p, _i32, _p, _p, _p, _i64, _i64, _i32, _f32, _f32, _f32, _f32, _i32,
                                    _f32, _i32, _i32, _f32, _f32, _f32, _p, _p, _p, _p, _sz, _p]),
    "siirl_actor_loss_fwd_static": (_i32, [_p, _p, _p, _p, _i32, _p, _p, _p, _i64, _i64, _i32, _f32, _f32, _f32, _f32,
                                           _i32, _f32, _i32, _i32, _f32, _f32, _f32, _p, _p, _p, _i32, _p]),
    "siirl_actor_loss_bwd": (_i32, [_p, _p, _p, _p, _p, _i32, _p, _p, _p, _i64, _i64, _i32, _f32, _f32, _f32, _f32,
                                    _i32, _f32, _i32, _i32, _f32, _f32, _f32, _p, _p, _p, _p, _p, _p]),
    "siirl_cov_workspace_bytes": (_sz, []),
    "siirl_cov_scores": (_i32, [_p, _p, _p, _p, _i32, _i64, _i64, _i32, _f32, _f32, _p, _p, _p, _sz, _p]),
    "siirl_range_select_workspace_bytes": (_sz, []),
    "siirl_range_select_count": (_i32, [_p, _i64, _f32, _f32, _p, _p, _sz, _p]),
    "siirl_range_select_write": (_i32, [_p, _i64, _f32, _f32, _p, _p, _i64, _p]),
    "siirl_topk_mark_workspace_bytes": (_sz, []),
    "siirl_topk_mark": (_i32, [_p, _i64, _i64, _f32, _p, _p, _sz, _p]),
    "siirl_actor_loss_cov_fwd": (_i32, [_p, _p, _p, _p, _i32, _p, _p, _p, _p, _i64, _i64, _i32, _f32, _f32, _i32, _f32,
                                        _i32, _i32, _f32, _f32, _f32, _p, _p, _p, _sz, _p]),
    "siirl_actor_loss_cov_bwd": (_i32, [_p, _p, _p, _p, _p, _i32, _p, _p, _p, _p, _i64, _i64, _i32, _f32, _f32, _i32,
                                        _f32, _i32, _i32, _f32, _f32, _f32, _p, _p, _p, _p, _p]),
    "siirl_value_loss_fwd": (_i32, [_p, _p, _p, _p, _i32, _i64, _i64, _f32, _i32, _p, _p, _p, _sz, _p]),
    "siirl_value_loss_bwd": (_i32, [_p, _p, _p, _p, _p, _i32, _i64, _i64, _f32, _i32, _p, _p, _p, _p]),
    "siirl_unpad_indices": (_i32, [_p, _i32, _i64, _i64, _p, _p, _p, _p, _p]),
    "siirl_gather_rows": (_i32, [_p, _p, _i64, _i64, _i64, _p, _p]),
    "siirl_scatter_rows": (_i32, [_p, _p, _i64, _i64, _i64, _p, _p]),
    "siirl_unpad_ids_labels": (_i32, [_p, _i64, _p, _i64, _p, _p, _p]),
    "siirl_mark_rows_outside_response": (_i32, [_p, _i64, _i64, _i64, _p, _p]),
    "siirl_response_scatter": (_i32, [_p, _p, _i64, _i64, _i64, _i64, _p, _p]),
    "siirl_response_gather": (_i32, [_p, _p, _i64, _i64, _i64, _i64, _p, _p]),
    "siirl_eos_response_mask": (_i32, [_p, _i32, _i64, _i64, _p, _i32, _p, _i32, _p]),
    "siirl_place_outcome_reward": (_i32, [_p, _p, _i32, _i64, _i64, _i64, _i32, _f64, _f64, _f64, _p, _p, _p, _p]),
    "siirl_data_metrics_workspace_bytes": (_sz, [_i64, _i64]),
    "siirl_data_metrics": (_i32, [_p, _p, _p, _p, _p, _p, _i32, _p, _i32, _i64, _i64, _i64, _p, _p, _sz, _p]),
    "siirl_whiten_workspace_bytes": (_sz, []),
    "siirl_masked_whiten": (_i32, [_p, _p, _i32, _i64, _i32, _p, _p, _p, _sz, _p]),
    "siirl_gae_workspace_bytes": (_sz, [_i64, _i64]),
    "siirl_gae_advantage_return": (_i32, [_p, _p, _p, _i32, _i64, _i64, _f64, _f64, _p, _p, _p, _p, _sz, _i32, _p]),
    "siirl_kl_penalty_fwd": (_i32, [_p, _p, _i64, _i32, _p, _p]),
    "siirl_kl_penalty_bwd": (_i32, [_p, _p, _p, _i64, _i32, _i32, _p, _p, _p]),
    "siirl_masked_reduce": (_i32, [_p, _p, _i32, _i64, _i64, _p, _p, _p, _p, _p, _p, _sz, _p]),
    "siirl_masked_reduce_bwd": (_i32, [_p, _p, _i32, _i64, _i64, _i32, _p, _p, _p]),
    "siirl_kl_in_reward": (_i32, [_p, _p, _p, _p, _i32, _i64, _i64, _i32, _f32, _p, _p, _p, _p]),
    "siirl_grpo_outcome_advantage": (_i32, [_p, _p, _i32, _p, _i64, _i64, _f32, _i32, _p, _p, _p]),
    "siirl_group_keep_mask": (_i32, [_p, _i32, _p, _i64, _p, _p, _p]),
    "siirl_fused_linear_fwd_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "siirl_fused_linear_bwd_workspace_bytes": (_sz, [_i64, _i64, _i64, _i32, _i32]),
    "siirl_fused_linear_fwd_workspace_bytes_dtype": (_sz, [_i32, _i64, _i64, _i64]),
    "siirl_fused_linear_bwd_workspace_bytes_dtype": (_sz, [_i32, _i64, _i64, _i64, _i32, _i32]),
    "siirl_fused_linear_saved_logits_bytes": (_sz, [_i64, _i64]),
    "siirl_fused_linear_logprob_entropy_fwd": (_i32, [_p, _p, _i32, _p, _i64, _i64, _i64, _f32, _p, _p, _p, _p, _p, _p,
                                                      _sz, _p]),
    "siirl_fused_linear_logprob_entropy_bwd": (_i32, [_p, _p, _i32, _p, _i64, _i64, _i64, _f32, _p, _p, _p, _p, _p, _p,
                                                      _p, _p, _sz, _p]),
    "siirl_marft_gae": (_i32, [_p, _p, _p, _i32, _p, _i32, _i64, _p, _p, _i64, _f32, _f32, _i32, _p, _p, _p, _p]),
    "siirl_fused_linear_bwd_rows_workspace_bytes": (_sz, [_i64, _i64, _i64, _i32, _i32]),
    "siirl_fused_linear_bwd_rows_workspace_bytes_dtype": (_sz, [_i32, _i64, _i64, _i64, _i32, _i32]),
    "siirl_fused_linear_logprob_entropy_bwd_rows": (_i32, [_p, _p, _i32, _p, _i64, _i64, _i64, _f32, _p, _p, _p, _p,
                                                           _p, _i64, _p, _p, _p, _sz, _p]),
}

_lock = threading.Lock()
_lib = None


class SiirlHipError(RuntimeError):
    pass


def lib():
    """The loaded library.  torch must be imported first so that the HIP runtime torch uses is the
    one this library binds to (both carry the soname libamdhip64.so.7)."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                import torch  # noqa: F401  (loads torch's libamdhip64 before ours is resolved)

                if not LIB_PATH.exists():
                    raise SiirlHipError(
                        f"{LIB_PATH} is missing: build it with `python -m siirl_amd.build` "
                        "(hipcc, gfx950).  siirl_amd has no CPU or eager fallback.")
                h = C.CDLL(str(LIB_PATH))
                for name, (res, args) in SIGNATURES.items():
                    fn = getattr(h, name)  # AttributeError if the symbol is not exported
                    fn.restype, fn.argtypes = res, args
                if h.siirl_hip_abi_version() != ABI_VERSION:
                    raise SiirlHipError(
                        f"{LIB_PATH} was built from ABI version {h.siirl_hip_abi_version()}, this package binds "
                        f"version {ABI_VERSION}: rebuild it with `python -m siirl_amd.build`")
                _lib = h
    return _lib


def check(rc: int, what: str):
    if rc != 0:
        msg = lib().siirl_hip_last_error().decode("utf-8", "replace")
        if rc == -1:
            raise ValueError(f"{what}: {msg}")
        if rc == -2:
            raise NotImplementedError(f"{what}: {msg}")
        raise SiirlHipError(f"{what} failed (status {rc}): {msg}")


def dtype_code(torch_dtype) -> int:
    import torch

    table = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16, torch.float64: F64,
             torch.int64: I64, torch.int32: I32, torch.uint8: U8, torch.bool: U8}
    if torch_dtype not in table:
        raise TypeError(f"dtype {torch_dtype} is not supported by libsiirl_hip")
    return table[torch_dtype]


def ptr(t):
    """Device pointer of a tensor (or NULL for None)."""
    return None if t is None else C.c_void_p(t.data_ptr())


def current_stream(device):
    import torch

    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)

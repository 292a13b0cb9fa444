"""ctypes binding of libaxon_amd.so — the C ABI declared in include/axon_amd.h.

There is no CPU fallback: every product entry point goes through this library
and raises if it is missing or if a call returns an error code.
"""

from __future__ import annotations

import ctypes
import os
import threading

from . import _build

_i32, _i64, _f32 = ctypes.c_int, ctypes.c_int64, ctypes.c_float
_ptr = ctypes.c_void_p

# name -> (restype, argtypes); mirrors include/axon_amd.h one to one
SIGNATURES: dict[str, tuple] = {
    "axon_amd_abi_version": (_i32, []),
    "axon_amd_error_string": (ctypes.c_char_p, [_i32]),
    "axon_lmhead_fwd_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "axon_seq_start_flags": (_i32, [_ptr, _i64, _i64, _ptr, _ptr]),
    "axon_lmhead_stash_bytes": (_i64, [_i64, _i64, _i64]),
    "axon_lmhead_fwd": (_i32, [_ptr, _ptr, _ptr, _i32, _i64, _i64, _i64, _f32, _f32, _ptr,
                               _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _ptr, _i64, _ptr]),
    "axon_lmhead_bwd_workspace_bytes": (_i64, [_i64, _i64, _i64, _i64]),
    "axon_lmhead_bwd": (_i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _i32, _ptr, _ptr, _i64, _i64, _i64,
                               _f32, _f32, _ptr, _ptr, _ptr, _i64, _ptr, _i64, _ptr, _i64, _ptr]),
    "axon_timer_create": (_ptr, [_ptr]),
    "axon_timer_collect": (_i32, [_ptr, _ptr, _ptr]),
    "axon_timer_destroy": (None, [_ptr]),
    "axon_lmhead_fwd_timed": (_i32, [_ptr, _ptr, _ptr, _i32, _i64, _i64, _i64, _f32, _f32, _ptr,
                                     _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _ptr, _i64, _ptr, _ptr]),
    "axon_lmhead_bwd_timed": (_i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _i32, _ptr, _ptr, _i64, _i64, _i64,
                                     _f32, _f32, _ptr, _ptr, _ptr, _i64, _ptr, _i64, _ptr, _i64, _ptr, _ptr]),
    "axon_lmhead_block_dw_acc_bytes": (_i64, [_i64, _i64]),
    "axon_lmhead_block_begin": (_i32, [_ptr, _i64, _i64, _i64, _ptr, _i64, _ptr, _ptr]),
    "axon_lmhead_block_fwd": (_i32, [_ptr, _ptr, _ptr, _i32, _i64, _i64, _i64, _f32, _f32, _ptr, _i64,
                                     _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _ptr, _i64, _ptr, _ptr]),
    "axon_lmhead_block_bwd": (_i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _i32, _ptr, _ptr, _i64, _i64, _i64,
                                     _f32, _f32, _ptr, _i64, _ptr, _ptr, _ptr, _i32, _i32, _i64, _i32, _i64,
                                     _i64, _ptr, _i64, _ptr, _i64, _ptr, _ptr]),
    "axon_lmhead_block_can_group": (_i32, [_i64, _i64, _i64]),
    "axon_lmhead_bwd_dlogit_copies": (_i32, [_i64, _i64, _i64]),
    "axon_scale_bf16_unless_one": (_i32, [_ptr, _i64, _ptr, _ptr]),
    "axon_lmhead_active_rows": (_i32, [_ptr, _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _ptr]),
    "axon_lmhead_gather_rows": (_i32, [_ptr, _ptr, _i32, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _ptr, _i64,
                                       _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr]),
    "axon_lmhead_scatter_rows": (_i32, [_ptr, _ptr, _i64, _i64, _ptr, _ptr]),
    "axon_gemm_nt_bf16": (_i32, [_ptr, _i64, _ptr, _i64, _ptr, _i64, _i64, _i64, _i64, _ptr]),
    "axon_gemm_bf16": (_i32, [_ptr, _i64, _i32, _ptr, _i64, _i32, _ptr, _i64, _i64, _i64, _i64, _ptr]),
    "axon_row_stats_workspace_bytes": (_i64, [_i64]),
    "axon_row_stats": (_i32, [_ptr, _ptr, _ptr, _i32, _ptr, _i64, _i64, _i64, _i32, _f32,
                              _ptr, _ptr, _ptr, _ptr, _ptr]),
    "axon_group_stats": (_i32, [_ptr, _ptr, _i64, _i64, _f32, _i32, _ptr, _ptr, _ptr, _ptr, _ptr]),
    "axon_row_broadcast_mask": (_i32, [_ptr, _ptr, _i32, _ptr, _i64, _i64, _i64, _f32, _ptr, _ptr]),
    "axon_fill_zero": (_i32, [_ptr, _i64, _ptr]),
    "axon_scale_f32": (_i32, [_ptr, _ptr, _ptr, _ptr, _i64, _ptr]),
    "axon_logits_fwd": (_i32, [_ptr, _i32, _i64, _i64, _i64, _ptr, _i32, _ptr, _ptr, _ptr, _ptr]),
    "axon_logits_bwd": (_i32, [_ptr, _i32, _i64, _i64, _i64, _ptr, _i32, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _ptr]),
    "axon_reverse_scan": (_i32, [_i32, _ptr, _ptr, _ptr, _i32, _ptr, _i64, _i64, _i64, _f32, _f32, _ptr, _ptr, _ptr,
                                 _ptr]),
    "axon_masked_whiten_workspace_bytes": (_i64, [_i64]),
    "axon_masked_whiten": (_i32, [_ptr, _ptr, _i32, _i64, _i32, _ptr, _ptr, _ptr, _ptr]),
    "axon_group_scalar": (_i32, [_i32, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _f32, _i32, _f32, _f32, _ptr, _ptr]),
    "axon_sampler_correction": (_i32, [_ptr, _ptr, _ptr, _i32, _ptr, _i64, _i64, _i64, _i32, _f32,
                                       _i32, _f32, _f32, _i32, _f32, _ptr, _ptr, _ptr, _ptr, _ptr,
                                       _ptr, _ptr, _ptr]),
    "axon_reduce_partials_bytes": (_i64, [_i64]),
    "axon_gmpo_loss": (_i32, [_ptr, _ptr, _ptr, _ptr, _i32, _ptr, _ptr, _i64, _i64, _i64, _f32, _f32, _ptr, _ptr, _ptr,
                              _ptr, _ptr]),
    "axon_cov_select_state_bytes": (_i64, []),
    "axon_cov_select_workspace_bytes": (_i64, [_i64]),
    "axon_cov_select": (_i32, [_i32, _ptr, _ptr, _ptr, _ptr, _i32, _i64, ctypes.c_double, _f32, _f32, _f32, _f32,
                               ctypes.c_uint32, _ptr, _ptr, _ptr, _ptr]),
    "axon_cov_policy_loss": (_i32, [_i32, _ptr, _ptr, _ptr, _ptr, _i32, _ptr, _ptr, _i64, _i64, _i64, _ptr, _f32,
                                    _i32, _ptr, _f32, _f32, _f32, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr]),
    "axon_kl_penalty": (_i32, [_ptr, _ptr, _i64, _i32, _i32, _ptr, _ptr, _ptr]),
    "axon_kl_reward": (_i32, [_ptr, _ptr, _ptr, _ptr, _i32, _ptr, _i64, _i64, _i64, _i32, _f32, _ptr, _ptr, _ptr]),
    "axon_side_terms": (_i32, [_ptr, _ptr, _ptr, _ptr, _i32, _ptr, _i64, _i64, _i64, _ptr, _f32, _i32, _ptr, _i32,
                               _i32, _ptr, _ptr, _ptr, _ptr, _ptr]),
    "axon_sampler_diag_workspace_bytes": (_i64, [_i64, _i64]),
    "axon_sampler_diag": (_i32, [_ptr, _ptr, _ptr, _i32, _ptr, _i64, _i64, _i64, _i32, _f32, _f32, _i32, _f32,
                                 _f32, _f32, _f32, _f32, _f32, _f32, _f32, _ptr, _ptr, _ptr]),
    "axon_loss_row_scale": (_i32, [_ptr, _ptr, _i64, _i64, _i32, _i32, _ptr, _ptr, _ptr, _ptr,
                                   _ptr, _ptr, _ptr]),
    "axon_policy_loss": (_i32, [_i32, _ptr, _ptr, _ptr, _ptr, _i32, _ptr, _ptr, _i64, _i64, _i64,
                                _ptr, _ptr, _f32, _i32, _ptr, _f32, _f32, _f32, _ptr, _ptr, _ptr,
                                _ptr]),
    "axon_policy_loss_rows": (_i32, [_i32, _ptr, _ptr, _ptr, _ptr, _i32, _ptr, _ptr, _i64, _i64, _i64, _i32, _i32,
                                     _ptr, _ptr, _ptr, _ptr, _f32, _f32, _f32, _ptr, _ptr, _ptr, _ptr]),
    "axon_sampler_correction_rows": (_i32, [_ptr, _ptr, _ptr, _i32, _ptr, _i64, _i64, _i64, _i32, _f32, _i32,
                                            _f32, _f32, _i32, _f32, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr,
                                            _ptr]),
    "axon_policy_loss_noalloc": (_i32, [_i32, _ptr, _ptr, _ptr, _ptr, _i32, _ptr, _ptr, _i64, _i64, _i64,
                                        _ptr, _ptr, _f32, _i32, _ptr, _f32, _f32, _f32, _ptr, _ptr, _ptr]),
}

ABI_VERSION = 20
MASK_F32, MASK_I64 = 0, 1

_lock = threading.Lock()
_lib = None


class AxonAmdError(RuntimeError):
    """A C-ABI call returned a negative status."""


def load() -> ctypes.CDLL:
    """Load the library (building it if no built copy exists) and bind every symbol."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        # The process must hold ONE HIP runtime: torch ships its own libamdhip64, so torch is loaded
        # first and the library's dependency then resolves to that copy (loaded the other way round,
        # the library's runtime sees no device).
        import torch  # noqa: F401

        path = _build.ensure_built()
        if not os.path.exists(path):
            raise AxonAmdError(f"{path} is missing and could not be built")
        lib = ctypes.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the symbol is not exported
            fn.restype = res
            fn.argtypes = args
        got = lib.axon_amd_abi_version()
        if got != ABI_VERSION:
            raise AxonAmdError(f"libaxon_amd.so ABI {got}, bindings expect {ABI_VERSION}")
        _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().axon_amd_error_string(rc).decode()
        raise AxonAmdError(f"{what}: {msg} (code {rc})")


def require_device(t, what: str) -> None:
    """The HIP path only: tensors must live on a GPU."""
    if not t.is_cuda:
        raise AxonAmdError(
            f"{what}: tensor is on {t.device}; the axon_amd path runs on MI355X only and has no CPU fallback"
        )


def stream_ptr() -> int:
    """The current device's current stream as the handle the C ABI takes.  Asked of the runtime directly where
    this torch offers it: building a ``torch.cuda.Stream`` object per call costs several microseconds, as much
    as everything else an eager call of a small operator does on the host."""
    import torch

    raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    if raw is not None:
        return raw(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def ptr(t) -> int | None:
    return None if t is None else t.data_ptr()

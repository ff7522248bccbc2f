"""ctypes binding of ``libareal_amd.so`` (the C ABI declared in ``include/areal_amd.h``).

The library is loaded from the package directory.  There is no fallback: if it
is missing or a call returns a non-zero status, an exception is raised.
"""
from __future__ import annotations

import ctypes as C
import threading
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libareal_amd.so"

AA_OK = 0
AA_ERR_INVALID_ARGUMENT = 1
AA_LMHEAD_COUNT_ON_DEVICE = -1  # a kept_per_chunk entry: the device counts the rows itself
AA_ERR_UNSUPPORTED = 2
AA_ERR_LAUNCH = 3
AA_BF16, AA_F16, AA_F32 = 0, 1, 2

RS_LEVEL = {"token": 0, "sequence": 1}
RS_ACTION = {"mask": 0, "clamp": 1}
RS_METRIC = {"ratio": 0, "kl_k1": 1, "kl_k2": 2, "kl_k3": 3}
RS_AGG = {"sum": 0, "mean": 1, "max": 2}


class NativeLibraryError(RuntimeError):
    """The HIP library is missing, incomplete, or a call into it failed."""


class PpoParams(C.Structure):
    """``aa_ppo_params``"""

    _fields_ = [
        ("clip_lo", C.c_float),
        ("clip_hi", C.c_float),
        ("c_clip", C.c_float),
        ("has_c_clip", C.c_int32),
        ("has_behave_weight", C.c_int32),
        ("loss_kind", C.c_int32),
        ("sapo_tau_pos", C.c_float),
        ("sapo_tau_neg", C.c_float),
    ]


class NormParams(C.Structure):
    """``aa_norm_params``"""

    _fields_ = [
        ("mean_level", C.c_int32),
        ("mean_leave1out", C.c_int32),
        ("std_level", C.c_int32),
        ("std_unbiased", C.c_int32),
        ("eps", C.c_float),
        ("group_size", C.c_int64),
    ]


_p = C.c_void_p
_i64 = C.c_int64
_f = C.c_float
_i = C.c_int
_d = C.c_double

# name -> (restype, argtypes); must list every function of include/areal_amd.h
SIGNATURES = {
    "aa_version": (_i, []),
    "aa_status_string": (C.c_char_p, [_i]),
    "aa_logits_fwd": (_i, [_p, _i, _i64, _i64, _i64, _p, _f, _p, _p, _p, _p, _p, _p, _p]),
    "aa_logits_bwd": (_i, [_p, _i, _i64, _i64, _i64, _p, _f, _p, _p, _p, _p, _i64, _p, _p]),
    "aa_logits_ppo_fused": (
        _i,
        [_p, _i, _i64, _i64, _i64, _p, _f, _i64, _p, _p, _p, _p, C.POINTER(PpoParams), _p, _p,
         _p, _p, _p, _p, _p, _p, _p, _p, _p, _p],
    ),
    "aa_vocab_partials_combine": (_i, [_p, _p, _p, _i, _i64, _p, _p, _p, _p, _p]),
    "aa_logits_pairs_fwd": (_i, [_p, _i, _i64, _i64, _i64, _p, _p, _i64, _f, _p, _p, _p, _p, _p]),
    "aa_logits_pairs_scatter": (_i, [_p, _i, _i64, _i64, _i64, _p, _p, _i64, _p, _f, _p]),
    "aa_rejection_sampling": (_i, [_p, _p, _p, _i64, _p, _i64, _i, _i, _i, _i, _f, _f, _i, _p, _p, _p, _p]),
    "aa_count_nonzero_u8": (_i, [_p, _i64, _p, _p]),
    "aa_ppo_loss": (_i, [_p, _p, _p, _p, _p, _i64, _p, _i64, _i, C.POINTER(PpoParams), _p, _p, _p, _p, _p, _p]),
    "aa_masked_sum": (_i, [_p, _p, _i64, _p, _p, _p, _p]),
    "aa_ppo_stat_outputs": (_i, [_p, _p, _p, _p, _p, _p, _i64, _p, _p, _p, _p, _p, _p]),
    "aa_scale_inplace": (_i, [_p, _i, _i64, _p, _p]),
    "aa_scale_rows_inplace": (_i, [_p, _i, _i64, _i64, _i64, _p, _p]),
    "aa_lmhead_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "aa_lmhead_fwd_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "aa_lmhead_fwd_stats_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "aa_lmhead_prepare": (_i, []),
    "aa_lmhead_fwd": (_i, [_p, _p, _i64, _i64, _i64, _p, _f, _p, _p, _p, _p, _p, _p, _p, _i64, _p]),
    "aa_lmhead_chunk_tokens": (_i64, []),
    "aa_lmhead_fwd_static": (_i, [_p, _p, _i64, _i64, _i64, _p, _f, _p, _p, _p, _p, _p]),
    "aa_lmhead_fwd_static_scratch_bytes": (_i64, []),
    "aa_lmhead_fwd_static_max_vocab": (_i64, []),
    "aa_lmhead_bwd": (_i, [_p, _p, _i64, _i64, _i64, _p, _f, _p, _p, _p, _p, _p, _p, _p, _p, _i, _p, _i64, _p]),
    "aa_lmhead_carry_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "aa_lmhead_panel_pitch": (_i64, [_i64]),
    "aa_lmhead_fwd_carry": (_i, [_p, _p, _i64, _i64, _i64, _p, _f, _p, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _p, _i64, _p]),
    "aa_lmhead_bwd_carry": (_i, [_p, _p, _i64, _i64, _i64, _p, _f, _p, _p, _p, _p, _p, _p, _i64, _p, _p, _i, _p, _i64, _p]),
    "aa_lmhead_ppo_fused": (
        _i,
        [_p, _p, _i64, _i64, _i64, _p, _f, _i64, _p, _p, _p, _p, C.POINTER(PpoParams), _p, _p, _p, _i,
         _p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _p, _i64, _p],
    ),
    "aa_sapo_loss": (_i, [_p, _p, _p, _p, _i64, _p, _i64, _i, _f, _f, _p, _p, _p, _p, _p, _p]),
    "aa_critic_loss": (_i, [_p, _p, _p, _p, _i64, _f, _i, _p, _p, _p, _p, _p]),
    "aa_prox_logp_approx": (_i, [_p, _p, _p, _i64, _i, _i, _p, _p]),
    "aa_masked_normalization_scratch_bytes": (_i64, [_i64, _i64]),
    "aa_masked_normalization": (_i, [_p, _p, _i64, _i64, _i, _d, _p, _p, _i64, _p]),
    "aa_kl_estimate": (_i, [_p, _p, _i64, _i, _i, _p, _p]),
    "aa_overlong_penalty": (_i, [_p, _p, _i64, _i64, _i, _f, _i64, _p]),
    "aa_kd_terms": (_i, [_p, _p, _p, _p, _i64, _i, _p, _p, _p]),
    "aa_sft_loss": (_i, [_p, _p, _i64, _p, _i64, _p, _p, _p, _p, _p, _p, _p, _p, _p]),
    "aa_dpo_seq_sums": (_i, [_p, _p, _p, _p, _i64, _i64, _p, _p, _p, _p]),
    "aa_dpo_seq_sums_bwd": (_i, [_p, _p, _p, _p, _i64, _i64, _p, _p]),
    "aa_dpo_preference_loss": (_i, [_p, _i64, _d, _i, _p, _p, _p]),
    "aa_dpo_pair_loss": (_i, [_p, _p, _p, _p, _i64, _d, _i, _p, _p, _p, _p, _p, _p, _p, _p]),
    "aa_logging_stats_scratch_bytes": (_i64, [_i64]),
    "aa_logging_stats": (_i, [_p, _p, _p, _p, _p, _i64, _i, _i, _i, _p, _p, _i64, _p]),
    "aa_rw_pair_loss": (_i, [_p, _i64, _p, _i64, _p, _p, _p, _p, _p, _p, _p, _p]),
    "aa_m2po_workspace_bytes": (_i64, [_i64]),
    "aa_m2po_mask": (_i, [_p, _p, _p, _i64, _f, _p, _p, _p, _i64, _p]),
    "aa_kl_rewards": (_i, [_p, _p, _p, _p, _p, _i64, _i64, _f, _i, _i, _p, _p, _p]),
    "aa_gae": (_i, [_p, _p, _p, _p, _i64, _i64, _f, _f, _p, _p, _p]),
    "aa_normalize_scratch_bytes": (_i64, [_i64, _i64, _i64]),
    "aa_normalize": (_i, [_p, _p, _i64, _i64, C.POINTER(NormParams), _p, _p, _i64, _p]),
    "aa_masked_moments": (_i, [C.POINTER(C.c_void_p), _i, _p, _i64, _p, _p]),
    "aa_segment_copy": (_i, [_p, _p, _i64, _p, _p, _p, _i64, _i64, _p]),
    "aa_copy_bytes": (_i, [_p, _p, _i64, _p]),
    "aa_mfma_only_loop": (_i, [_i, _i, _i, _i, _p, _p]),
    "aa_hbm_stream_probe": (_i, [_i, _i, _p, _p, _i64, _i, _p]),
}

_lib = None
_lock = threading.Lock()


def load() -> C.CDLL:
    """Load the shared library once and bind the signatures."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not LIB_PATH.exists():
            raise NativeLibraryError(
                f"{LIB_PATH} not found: build it with `python -m areal_amd.build` "
                "(there is no CPU or PyTorch fallback for these ops)"
            )
        try:
            lib = C.CDLL(str(LIB_PATH))
        except OSError as e:  # missing ROCm runtime etc.
            raise NativeLibraryError(f"cannot load {LIB_PATH}: {e}") from e
        for name, (res, args) in SIGNATURES.items():
            try:
                fn = getattr(lib, name)
            except AttributeError as e:
                raise NativeLibraryError(f"{LIB_PATH} does not export {name}") from e
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(status: int, what: str) -> None:
    if status != AA_OK:
        msg = load().aa_status_string(status).decode()
        raise NativeLibraryError(f"{what} failed: {msg} (status {status})")

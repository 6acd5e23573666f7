"""ctypes binding of libtrlk.so (the C ABI declared in include/trlk.h).

The library is built in-tree by `python trl_amd/build.py` / `make -C trl_amd/csrc`; there is no
fallback implementation: if it is missing, importing this module raises.
`import torch` happens first on purpose, so that the HIP runtime torch ships is the one
the kernels are enqueued on (stream handles and device pointers are shared with torch).
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_double, c_float, c_int32, c_int64, c_size_t, c_void_p

import torch  # noqa: F401  (loads the HIP runtime the library binds to)

# TRLK_LIBRARY_PATH points at another build of the same library (kernel experiments)
LIB_PATH = os.environ.get("TRLK_LIBRARY_PATH") or os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libtrlk.so")

F32, BF16, F16 = 0, 1, 2
GRPO, BNPO, DR_GRPO, DAPO, LUSPO = 0, 1, 2, 3, 4
TERM_CLIP, TERM_CISPO, TERM_SAPO, TERM_WEIGHTED_LOGP = 0, 1, 2, 3
SCALE_GROUP, SCALE_BATCH, SCALE_NONE = 0, 1, 2
FLAG_INDEX_OUT_OF_RANGE = 1
GRPO_NUM_METRICS = 16
DPO_NUM_METRICS = 8
RLOO_NUM_METRICS = 8

# name -> (restype, argtypes); must list every symbol include/trlk.h declares
SIGNATURES = {
    "trlk_version": (c_int32, []),
    "trlk_last_error": (c_char_p, []),
    "trlk_logp_entropy_fwd": (
        c_int32,
        [c_void_p, c_int32, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int32, c_float, c_void_p,
         c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_void_p],
    ),
    "trlk_logp_entropy_bwd": (
        c_int32,
        [c_void_p, c_int32, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int32, c_float, c_void_p,
         c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p],
    ),
    "trlk_logp_entropy_fwd_f64": (
        c_int32,
        [c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int32, c_double, c_void_p, c_void_p,
         c_void_p, c_void_p, c_void_p, c_void_p],
    ),
    "trlk_logp_entropy_bwd_f64": (
        c_int32,
        [c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int32, c_double, c_void_p, c_void_p,
         c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p],
    ),
    "trlk_group_advantages": (c_int32, [c_void_p, c_int64, c_int32, c_int32, c_void_p, c_void_p]),
    "trlk_grpo_workspace_bytes": (c_size_t, [c_int64]),
    "trlk_grpo_loss": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int64, c_int64, c_int32, c_int32, c_int32, c_float, c_float, c_float, c_float, c_int32, c_float, c_float,
         c_void_p, c_float, c_float, c_float, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
         c_void_p],
    ),
    "trlk_init": (c_int32, []),
    "trlk_grpo_loss_static_max_seq": (c_int64, []),
    "trlk_grpo_loss_static": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int64, c_int64, c_int32, c_int32, c_int32, c_float, c_float, c_float, c_float, c_int32, c_float, c_float,
         c_void_p, c_float, c_float, c_float, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    ),
    "trlk_grpo_fused_max_vocab": (c_int64, [c_int32]),
    "trlk_grpo_fused_fwd_bwd": (
        c_int32,
        [c_void_p, c_int32, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_float, c_void_p, c_void_p, c_void_p,
         c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_float, c_float, c_float, c_float,
         c_int32, c_float, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int32,
         c_void_p, c_void_p],
    ),
    "trlk_scale_unless_one": (c_int32, [c_void_p, c_int32, c_int64, c_void_p, c_void_p]),
    "trlk_split_bf16x3": (c_int32, [c_void_p, c_int64, c_int64, c_int64, c_int32, c_void_p, c_int64, c_void_p]),
    "trlk_gemm_nt": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_int64, c_int32, c_int64, c_int64, c_int64, c_void_p, c_int64, c_int32, c_void_p],
    ),
    "trlk_dpo_loss": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_float, c_void_p, c_void_p, c_void_p, c_void_p,
         c_void_p],
    ),
    "trlk_fused_head_fwd_workspace_bytes": (c_size_t, [c_int64]),
    "trlk_fused_head_bwd_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64, c_int64]),
    "trlk_fused_head_fwd": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int64, c_int64, c_int64, c_int64, c_float, c_float,
         c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_size_t,
         c_void_p],
    ),
    "trlk_fused_head_bwd": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int64, c_int64, c_int64, c_int64, c_float, c_float,
         c_float, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
         c_void_p, c_size_t, c_void_p],
    ),
    "trlk_fused_head_stash_bytes": (c_size_t, [c_int64, c_int64, c_void_p]),
    "trlk_rloo_loss": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_float, c_float, c_void_p, c_void_p, c_void_p,
         c_void_p, c_void_p],
    ),
}


ABI_VERSION = 2  # TRLK_VERSION of include/trlk.h that SIGNATURES was written against


class TrlkError(RuntimeError):
    """A launch failed (positive status = hipError_t)."""


class TrlkArgumentError(ValueError):
    """The library rejected the arguments before launching anything (negative status)."""


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build the HIP kernels first (python trl_amd/build.py, or "
            "make -C trl_amd/csrc). There is no fallback implementation."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here = the built library is stale
        fn.restype = restype
        fn.argtypes = argtypes
    built = lib.trlk_version()
    if built != ABI_VERSION:  # the signatures above would not match the library's
        raise ImportError(f"{LIB_PATH} was built for interface version {built}, this package binds version "
                          f"{ABI_VERSION}: rebuild it (python trl_amd/build.py)")
    return lib


lib = _load()


def last_error() -> str:
    return lib.trlk_last_error().decode()


def check(status: int) -> None:
    if status == 0:
        return
    if status < 0:
        raise TrlkArgumentError(f"trlk status {status}: {last_error()}")
    raise TrlkError(f"trlk launch failed with hipError_t {status}: {last_error()}")


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}[dtype]
    except KeyError:
        raise TypeError(f"trl_amd kernels take float32, bfloat16 or float16 logits, got {dtype}") from None


def ptr(t: torch.Tensor | None):
    return None if t is None else t.data_ptr()


def current_stream(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream

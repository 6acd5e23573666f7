"""PyTorch custom ops over the C ABI (include/trlk.h).

Each op hands raw device pointers, sizes, strides and the current HIP stream to
libtrlk.so; torch only owns the memory.  The ops exist for device tensors only
(`device_types="cuda"`, which is the ROCm device in a ROCm build): there is no CPU or
eager fallback, a CPU tensor raises.

Autograd is registered on the forward ops; the backward of the log-prob op recomputes the
softmax from the saved per-row logsumexp (4 bytes per row are kept, never a `[rows, vocab]`
tensor).
"""
from __future__ import annotations

import ctypes
import math
import os
from typing import Optional

import torch
from torch import Tensor

from . import _lib
from ._lib import check, current_stream, dtype_code, lib, ptr

_SYNC_CHECKS = os.environ.get("TRL_AMD_SYNC_CHECKS", "0") == "1"
_error_flags: dict[int, Tensor] = {}


def _error_flag(device: torch.device) -> Tensor:
    """Per-device int32 word the kernels OR error bits into (see `check_device_errors`)."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    flag = _error_flags.get(idx)
    if flag is None:
        flag = torch.zeros(1, dtype=torch.int32, device=device)
        _error_flags[idx] = flag
    return flag


def check_device_errors() -> None:
    """Raises IndexError if any kernel since the last call saw an index outside [0, vocab).

    The reference raises synchronously on CPU and device-asserts on GPU
    (`torch.gather`, trl/trainer/utils.py:507,516); here the entry gets NaN, a flag is set on
    the device, and this function (one device->host read, i.e. a synchronisation) reports it.
    Set TRL_AMD_SYNC_CHECKS=1 to run it after every forward call.
    """
    for flag in _error_flags.values():
        bits = int(flag.item())
        if bits:
            flag.zero_()
            if bits & _lib.FLAG_INDEX_OUT_OF_RANGE:
                raise IndexError("trl_amd: an index passed to a log-prob kernel was outside [0, vocab)")
            raise RuntimeError(f"trl_amd: device error flag {bits:#x}")


def device_error_bits(device: torch.device) -> Tensor:
    """The error word of `device` as a one-element fp32 tensor, for callers that are about to copy metrics to the
    host anyway and append it to that copy (then pass the value to `raise_for_error_bits`): no extra sync."""
    return _error_flag(device).to(torch.float32)


def raise_for_error_bits(bits: float, device: torch.device) -> None:
    """Raises what `check_device_errors` would for an error word already on the host (and clears the word)."""
    bits = int(bits)
    if bits:
        _error_flag(device).zero_()
        if bits & _lib.FLAG_INDEX_OUT_OF_RANGE:
            raise IndexError("trl_amd: an index passed to a log-prob kernel was outside [0, vocab)")
        raise RuntimeError(f"trl_amd: device error flag {bits:#x}")


# --------------------------------------------------------------------------------------------
# log-prob + entropy (K1 / K3)
# --------------------------------------------------------------------------------------------
def _check_logits3d(logits: Tensor) -> None:
    if logits.dim() != 3:
        raise ValueError(f"expected [n_seq, rows, vocab] logits, got shape {tuple(logits.shape)}")
    if logits.shape[-1] > 1 and logits.stride(-1) != 1:
        raise ValueError("the vocabulary axis of the logits must be contiguous")


def _run_logp_entropy_fwd(logits, index, temperature, keep_start, keep_len, row_mask, with_stats, sum_p2=True):
    _check_logits3d(logits)
    n_seq, _, vocab = logits.shape
    rows = n_seq * keep_len
    k = index.shape[-1]
    dev = logits.device
    logp = torch.empty((rows, k), dtype=torch.float32, device=dev)
    ent = torch.empty((rows,), dtype=torch.float32, device=dev)
    lse = torch.empty((rows,), dtype=torch.float32, device=dev)
    stats = torch.empty((rows, 4), dtype=torch.float32, device=dev) if with_stats else None
    if rows == 0:
        return logp, ent, lse, stats
    index = index.contiguous()
    view = logits[:, keep_start : keep_start + keep_len]
    with torch.cuda.device(dev):
        check(
            lib.trlk_logp_entropy_fwd(
                view.data_ptr(), dtype_code(logits.dtype), n_seq, keep_len, vocab, view.stride(0), view.stride(1),
                ptr(index), k, temperature, ptr(row_mask), ptr(logp), ptr(ent), ptr(lse), ptr(stats),
                int(bool(sum_p2)), ptr(_error_flag(dev)), current_stream(dev),
            )
        )
    if _SYNC_CHECKS:
        check_device_errors()
    return logp, ent, lse, stats


@torch.library.custom_op("trl_amd::logp_entropy_fwd", mutates_args=(), device_types="cuda")
def logp_entropy_fwd(
    logits: Tensor, index: Tensor, temperature: float, keep_start: int, keep_len: int, row_mask: Optional[Tensor]
) -> tuple[Tensor, Tensor, Tensor]:
    """logits [n_seq, L, V] (strided view, last axis contiguous); rows keep_start..keep_start+keep_len
    of every sequence are processed.  index int64 [n_seq*keep_len, K].  Returns fp32
    (logp [rows, K], entropy [rows], lse [rows])."""
    return _run_logp_entropy_fwd(logits, index, temperature, keep_start, keep_len, row_mask, False)[:3]


@logp_entropy_fwd.register_fake
def _(logits, index, temperature, keep_start, keep_len, row_mask):
    rows = logits.shape[0] * keep_len
    f = lambda *s: torch.empty(s, dtype=torch.float32, device=logits.device)  # noqa: E731
    return f(rows, index.shape[-1]), f(rows), f(rows)


@torch.library.custom_op("trl_amd::logp_entropy_stats_fwd", mutates_args=(), device_types="cuda")
def logp_entropy_stats_fwd(
    logits: Tensor, index: Tensor, temperature: float, keep_start: int, keep_len: int, row_mask: Optional[Tensor],
    sum_p2: bool = True,
) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    """As `logp_entropy_fwd`, plus the fp32 row statistics `[rows, 4]` of the same pass: mean logit,
    log sum_v p_v^2 (0 without `sum_p2`: the kernel is bound by its arithmetic and runs 4 % faster without that
    sum), whether index[:, 0] is the row's arg-max (first maximal position), 0."""
    return _run_logp_entropy_fwd(logits, index, temperature, keep_start, keep_len, row_mask, True, sum_p2)


@logp_entropy_stats_fwd.register_fake
def _(logits, index, temperature, keep_start, keep_len, row_mask, sum_p2=True):
    rows = logits.shape[0] * keep_len
    f = lambda *s: torch.empty(s, dtype=torch.float32, device=logits.device)  # noqa: E731
    return f(rows, index.shape[-1]), f(rows), f(rows), f(rows, 4)


@torch.library.custom_op("trl_amd::logp_entropy_bwd", mutates_args=(), device_types="cuda")
def logp_entropy_bwd(
    logits: Tensor, index: Tensor, temperature: float, keep_start: int, keep_len: int, lse: Tensor,
    entropy: Optional[Tensor], g_logp: Optional[Tensor], g_entropy: Optional[Tensor],
) -> Tensor:
    """d(loss)/d(logits) for the whole [n_seq, L, V] input (contiguous, same dtype): rows outside
    the kept window and rows whose upstream gradients are all zero are zero-filled."""
    _check_logits3d(logits)
    n_seq, length, vocab = logits.shape
    dlogits = torch.empty((n_seq, length, vocab), dtype=logits.dtype, device=logits.device)
    if dlogits.numel() == 0:
        return dlogits
    dev = logits.device
    view = logits[:, keep_start : keep_start + keep_len]
    k = index.shape[-1] if g_logp is not None else 0
    index = index.contiguous()
    g_logp = None if g_logp is None else g_logp.contiguous().float()
    g_entropy = None if g_entropy is None else g_entropy.contiguous().float()
    with torch.cuda.device(dev):
        check(
            lib.trlk_logp_entropy_bwd(
                view.data_ptr(), dtype_code(logits.dtype), n_seq, keep_len, vocab, view.stride(0), view.stride(1),
                ptr(index), k, temperature, ptr(lse), ptr(entropy if g_entropy is not None else None), ptr(g_logp),
                ptr(g_entropy), ptr(dlogits), length, keep_start, dlogits.stride(0), dlogits.stride(1),
                current_stream(dev),
            )
        )
    return dlogits


@logp_entropy_bwd.register_fake
def _(logits, index, temperature, keep_start, keep_len, lse, entropy, g_logp, g_entropy):
    return torch.empty(logits.shape, dtype=logits.dtype, device=logits.device)


def _lpe_setup(ctx, inputs, output):
    logits, index, temperature, keep_start, keep_len, row_mask = inputs[:6]
    ctx.n_inputs = len(inputs)
    _, ent, lse = output[:3]
    ctx.save_for_backward(logits, index, lse, ent)
    ctx.cfg = (temperature, keep_start, keep_len)
    ctx.set_materialize_grads(False)


def _lpe_backward(ctx, g_logp, g_ent, g_lse, g_stats=None):
    logits, index, lse, ent = ctx.saved_tensors
    temperature, keep_start, keep_len = ctx.cfg
    # the lse output only exists to be saved for this backward; a gradient arriving there is ignored
    rest = (None,) * (ctx.n_inputs - 1)
    if g_logp is None and g_ent is None:
        return (None, *rest)
    if g_logp is None and index.shape[-1] > 0:
        g_logp = torch.zeros(index.shape, dtype=torch.float32, device=logits.device)
    d = logp_entropy_bwd(logits, index, temperature, keep_start, keep_len, lse, ent, g_logp, g_ent)
    return (d, *rest)


logp_entropy_fwd.register_autograd(_lpe_backward, setup_context=_lpe_setup)
logp_entropy_stats_fwd.register_autograd(_lpe_backward, setup_context=_lpe_setup)


# ---- the same pair for fp64 logits: double operands, arithmetic and outputs --------------------------------
@torch.library.custom_op("trl_amd::logp_entropy_fwd_f64", mutates_args=(), device_types="cuda")
def logp_entropy_fwd_f64(
    logits: Tensor, index: Tensor, temperature: float, keep_start: int, keep_len: int, row_mask: Optional[Tensor]
) -> tuple[Tensor, Tensor, Tensor]:
    """`logp_entropy_fwd` for float64 logits (trl/trainer/utils.py:506-510): returns float64
    (logp [rows, K], entropy [rows], lse [rows])."""
    _check_logits3d(logits)
    if logits.dtype != torch.float64:
        raise TypeError("logp_entropy_fwd_f64 takes float64 logits")
    n_seq, _, vocab = logits.shape
    rows, k, dev = n_seq * keep_len, index.shape[-1], logits.device
    logp = torch.empty((rows, k), dtype=torch.float64, device=dev)
    ent = torch.empty((rows,), dtype=torch.float64, device=dev)
    lse = torch.empty((rows,), dtype=torch.float64, device=dev)
    if rows == 0:
        return logp, ent, lse
    index = index.contiguous()
    view = logits[:, keep_start : keep_start + keep_len]
    with torch.cuda.device(dev):
        check(lib.trlk_logp_entropy_fwd_f64(view.data_ptr(), n_seq, keep_len, vocab, view.stride(0), view.stride(1),
                                            ptr(index), k, temperature, ptr(row_mask), ptr(logp), ptr(ent), ptr(lse),
                                            ptr(_error_flag(dev)), current_stream(dev)))
    if _SYNC_CHECKS:
        check_device_errors()
    return logp, ent, lse


@logp_entropy_fwd_f64.register_fake
def _(logits, index, temperature, keep_start, keep_len, row_mask):
    rows = logits.shape[0] * keep_len
    f = lambda *s: torch.empty(s, dtype=torch.float64, device=logits.device)  # noqa: E731
    return f(rows, index.shape[-1]), f(rows), f(rows)


@torch.library.custom_op("trl_amd::logp_entropy_bwd_f64", mutates_args=(), device_types="cuda")
def logp_entropy_bwd_f64(
    logits: Tensor, index: Tensor, temperature: float, keep_start: int, keep_len: int, lse: Tensor,
    entropy: Optional[Tensor], g_logp: Optional[Tensor], g_entropy: Optional[Tensor],
) -> Tensor:
    """`logp_entropy_bwd` for float64 logits: the float64 gradient of the whole [n_seq, L, V] input."""
    _check_logits3d(logits)
    n_seq, length, vocab = logits.shape
    dlogits = torch.empty((n_seq, length, vocab), dtype=torch.float64, device=logits.device)
    if dlogits.numel() == 0:
        return dlogits
    dev = logits.device
    view = logits[:, keep_start : keep_start + keep_len]
    k = index.shape[-1] if g_logp is not None else 0
    index = index.contiguous()
    g_logp = None if g_logp is None else g_logp.contiguous().double()
    g_entropy = None if g_entropy is None else g_entropy.contiguous().double()
    with torch.cuda.device(dev):
        check(lib.trlk_logp_entropy_bwd_f64(view.data_ptr(), n_seq, keep_len, vocab, view.stride(0), view.stride(1),
                                            ptr(index), k, temperature, ptr(lse),
                                            ptr(entropy if g_entropy is not None else None), ptr(g_logp), ptr(g_entropy),
                                            ptr(dlogits), length, keep_start, dlogits.stride(0), dlogits.stride(1),
                                            current_stream(dev)))
    return dlogits


@logp_entropy_bwd_f64.register_fake
def _(logits, index, temperature, keep_start, keep_len, lse, entropy, g_logp, g_entropy):
    return torch.empty(logits.shape, dtype=torch.float64, device=logits.device)


def _lpe64_backward(ctx, g_logp, g_ent, g_lse):
    logits, index, lse, ent = ctx.saved_tensors
    temperature, keep_start, keep_len = ctx.cfg
    if g_logp is None and g_ent is None:
        return None, None, None, None, None, None
    if g_logp is None and index.shape[-1] > 0:
        g_logp = torch.zeros(index.shape, dtype=torch.float64, device=logits.device)
    d = logp_entropy_bwd_f64(logits, index, temperature, keep_start, keep_len, lse, ent, g_logp, g_ent)
    return d, None, None, None, None, None


logp_entropy_fwd_f64.register_autograd(_lpe64_backward, setup_context=_lpe_setup)


def logp_entropy_forward(logits: Tensor, index: Tensor, temperature: float, keep_start: int, keep_len: int,
                         row_mask: Optional[Tensor]) -> tuple[Tensor, Tensor, Tensor]:
    """The forward op for these logits: the double-precision pair for float64, the streaming kernels otherwise."""
    op = logp_entropy_fwd_f64 if logits.dtype == torch.float64 else logp_entropy_fwd
    return op(logits, index, temperature, keep_start, keep_len, row_mask)


# --------------------------------------------------------------------------------------------
# group advantages (K2a)
# --------------------------------------------------------------------------------------------
_SCALE_MODES = {"group": _lib.SCALE_GROUP, "batch": _lib.SCALE_BATCH, "none": _lib.SCALE_NONE}


@torch.library.custom_op("trl_amd::group_advantages", mutates_args=(), device_types="cuda")
def _group_advantages(rewards: Tensor, group_size: int, scale_mode: int) -> Tensor:
    rewards = rewards.contiguous().float()
    out = torch.empty_like(rewards)
    dev = rewards.device
    with torch.cuda.device(dev):
        check(lib.trlk_group_advantages(ptr(rewards), rewards.numel(), group_size, scale_mode, ptr(out), current_stream(dev)))
    return out


@_group_advantages.register_fake
def _(rewards, group_size, scale_mode):
    return torch.empty(rewards.shape, dtype=torch.float32, device=rewards.device)


def group_advantages(rewards: Tensor, num_generations: int, scale_rewards: str = "group") -> Tensor:
    """Group-relative advantages of fp32 `rewards` [B] (NaN = unscorable); groups are
    `num_generations` consecutive entries (trl/trainer/grpo_trainer.py:2685-2707, 2730)."""
    if scale_rewards not in _SCALE_MODES:
        raise ValueError(f"Invalid value for scale_rewards: {scale_rewards}. Must be one of 'batch', 'group', or 'none'.")
    if rewards.dim() != 1:
        raise ValueError("rewards must be 1-D")
    return _group_advantages(rewards, num_generations, _SCALE_MODES[scale_rewards])


# --------------------------------------------------------------------------------------------
# GRPO loss (K2)
# --------------------------------------------------------------------------------------------
# reference loss_type -> (normalisation, per-token policy term)   (trl/trainer/grpo_trainer.py:3080-3148)
LOSS_TYPES = {
    "grpo": (_lib.GRPO, _lib.TERM_CLIP),
    "bnpo": (_lib.BNPO, _lib.TERM_CLIP),
    "dr_grpo": (_lib.DR_GRPO, _lib.TERM_CLIP),
    "dapo": (_lib.DAPO, _lib.TERM_CLIP),
    "luspo": (_lib.LUSPO, _lib.TERM_CLIP),
    "cispo": (_lib.DAPO, _lib.TERM_CISPO),
    "sapo": (_lib.GRPO, _lib.TERM_SAPO),
    "vespo": (_lib.DAPO, _lib.TERM_WEIGHTED_LOGP),
}


def _f32c(t: Optional[Tensor]) -> Optional[Tensor]:
    return None if t is None else t.contiguous().float()


@torch.library.custom_op("trl_amd::grpo_loss", mutates_args=(), device_types="cuda")
def grpo_loss_op(
    logp: Tensor, old_logp: Optional[Tensor], ref_logp: Optional[Tensor], entropy: Optional[Tensor],
    advantages: Tensor, mask: Tensor, token_weight: Optional[Tensor], entropy_mask: Optional[Tensor],
    dapo_normalizer: Optional[Tensor], loss_type: int, epsilon_low: float, epsilon_high: float, delta: float,
    beta: float, use_bias_correction_kl: bool, grad_accum_steps: float, dr_grpo_denominator: float,
    num_processes: float, entropy_coef: float, policy_term: int = 0, sequence_level: bool = False,
    seq_coef: Optional[Tensor] = None, sapo_temperature_pos: float = 1.0, sapo_temperature_neg: float = 1.05,
) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    """Returns (loss [], metrics [16], d loss/d logp [B,T], d loss/d entropy [B,T])."""
    if logp.dim() != 2:
        raise ValueError("grpo_loss: per-token log-probs must be [B, T]")
    B, T = logp.shape
    dev = logp.device
    logp, old_logp, ref_logp, entropy = _f32c(logp), _f32c(old_logp), _f32c(ref_logp), _f32c(entropy)
    mask, token_weight, entropy_mask = _f32c(mask), _f32c(token_weight), _f32c(entropy_mask)
    advantages = _f32c(advantages)
    if advantages.dim() == 1 or (advantages.dim() == 2 and advantages.shape[1] == 1):
        if advantages.numel() != B:
            raise ValueError("grpo_loss: advantages must have one entry per sequence")
        sb, st = 1, 0
    elif tuple(advantages.shape) == (B, T):
        sb, st = T, 1
    else:
        raise ValueError(f"grpo_loss: advantages of shape {tuple(advantages.shape)} do not match [B]={B} or [B,T]")
    for name, t in (("old_logp", old_logp), ("ref_logp", ref_logp), ("entropy", entropy), ("mask", mask),
                    ("token_weight", token_weight), ("entropy_mask", entropy_mask)):
        if t is not None and tuple(t.shape) != (B, T):
            raise ValueError(f"grpo_loss: {name} has shape {tuple(t.shape)}, expected {(B, T)}")
    dapo_normalizer = None if dapo_normalizer is None else dapo_normalizer.reshape(1).contiguous().float()
    if seq_coef is not None:
        if seq_coef.numel() != B:
            raise ValueError("grpo_loss: seq_coef must have one entry per sequence")
        seq_coef = seq_coef.reshape(B).contiguous().float()
    loss = torch.empty((), dtype=torch.float32, device=dev)
    metrics = torch.empty((_lib.GRPO_NUM_METRICS,), dtype=torch.float32, device=dev)
    dlogp = torch.empty((B, T), dtype=torch.float32, device=dev)
    dent = torch.empty((B, T), dtype=torch.float32, device=dev) if entropy_coef != 0.0 else None
    ws_bytes = lib.trlk_grpo_workspace_bytes(B)
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        check(
            lib.trlk_grpo_loss(
                ptr(logp), ptr(old_logp), ptr(ref_logp), ptr(entropy), ptr(advantages), sb, st, ptr(mask),
                ptr(token_weight), ptr(entropy_mask), ptr(seq_coef), B, T, loss_type, policy_term,
                int(sequence_level), epsilon_low, epsilon_high, delta, beta, int(use_bias_correction_kl),
                grad_accum_steps, dr_grpo_denominator, ptr(dapo_normalizer), num_processes, entropy_coef,
                sapo_temperature_pos, sapo_temperature_neg, ptr(loss), ptr(metrics), ptr(dlogp), ptr(dent), ptr(ws),
                ws_bytes, current_stream(dev),
            )
        )
    if dent is None:
        dent = torch.zeros((0,), dtype=torch.float32, device=dev)
    return loss, metrics, dlogp, dent


@grpo_loss_op.register_fake
def _(logp, old_logp, ref_logp, entropy, advantages, mask, token_weight, entropy_mask, dapo_normalizer, loss_type,
      epsilon_low, epsilon_high, delta, beta, use_bias_correction_kl, grad_accum_steps, dr_grpo_denominator,
      num_processes, entropy_coef, policy_term=0, sequence_level=False, seq_coef=None, sapo_temperature_pos=1.0,
      sapo_temperature_neg=1.05):
    f = lambda *s: torch.empty(s, dtype=torch.float32, device=logp.device)  # noqa: E731
    return f(), f(_lib.GRPO_NUM_METRICS), f(*logp.shape), (f(*logp.shape) if entropy_coef != 0.0 else f(0))


def _grpo_setup(ctx, inputs, output):
    _, _, dlogp, dent = output
    ctx.save_for_backward(dlogp, dent)
    ctx.logp_dtype = inputs[0].dtype
    ctx.has_ent_grad = inputs[18] != 0.0 and inputs[3] is not None
    ctx.set_materialize_grads(False)


def _grpo_backward(ctx, g_loss, g_metrics, g_dlogp, g_dent):
    dlogp, dent = ctx.saved_tensors
    grads = [None] * 24
    if g_loss is not None:
        grads[0] = (g_loss * dlogp).to(ctx.logp_dtype)
        if ctx.has_ent_grad:
            grads[3] = g_loss * dent
    return tuple(grads)


grpo_loss_op.register_autograd(_grpo_backward, setup_context=_grpo_setup)


def grpo_loss_static_max_seq() -> int:
    """Most sequences `grpo_loss_static_` takes (the size of the scratch array built into the library)."""
    return int(lib.trlk_grpo_loss_static_max_seq())


def grpo_loss_static_(
    out_loss: Tensor, out_metrics: Tensor, out_dlogp: Tensor, out_dentropy: Optional[Tensor], logp: Tensor,
    old_logp: Optional[Tensor], ref_logp: Optional[Tensor], entropy: Optional[Tensor], advantages: Tensor, mask: Tensor,
    token_weight: Optional[Tensor], entropy_mask: Optional[Tensor], dapo_normalizer: Optional[Tensor], loss_type: int,
    epsilon_low: float, epsilon_high: float, delta: float, beta: float, use_bias_correction_kl: bool,
    grad_accum_steps: float, dr_grpo_denominator: float, num_processes: float, entropy_coef: float,
    policy_term: int = 0, sequence_level: bool = False, seq_coef: Optional[Tensor] = None,
    sapo_temperature_pos: float = 1.0, sapo_temperature_neg: float = 1.05,
) -> None:
    """The GRPO loss (`grpo_loss_op`'s arithmetic, bit for bit) for callers that must not allocate: every operand
    is a contiguous fp32 device tensor the caller owns (`logp`, `mask`, ... `[B, T]`; `advantages` `[B]` or
    `[B, T]`; outputs `out_loss []`, `out_metrics [16]`, `out_dlogp [B, T]`, `out_dentropy [B, T]` when
    `entropy_coef != 0`), nothing is converted or copied, and the kernels' partial sums go to a scratch array built
    into the library instead of a workspace tensor.  At most `grpo_loss_static_max_seq()` sequences; calls that
    overlap on one GPU race (they share the array).  No autograd."""
    B, T = logp.shape
    for name, t in (("logp", logp), ("old_logp", old_logp), ("ref_logp", ref_logp), ("entropy", entropy),
                    ("mask", mask), ("token_weight", token_weight), ("entropy_mask", entropy_mask),
                    ("out_dlogp", out_dlogp), ("out_dentropy", out_dentropy)):
        if t is not None and (t.dtype != torch.float32 or not t.is_contiguous() or tuple(t.shape) != (B, T)):
            raise ValueError(f"grpo_loss_static_: {name} must be a contiguous fp32 [{B}, {T}] tensor")
    if advantages.dtype != torch.float32 or not advantages.is_contiguous():
        raise ValueError("grpo_loss_static_: advantages must be contiguous fp32")
    if tuple(advantages.shape) in ((B,), (B, 1)):
        sb, st = 1, 0
    elif tuple(advantages.shape) == (B, T):
        sb, st = T, 1
    else:
        raise ValueError(f"grpo_loss_static_: advantages of shape {tuple(advantages.shape)} do not match [B] or [B, T]")
    if (out_loss.dtype != torch.float32 or out_loss.numel() != 1 or out_metrics.dtype != torch.float32
            or out_metrics.dim() != 1 or out_metrics.numel() < _lib.GRPO_NUM_METRICS or not out_metrics.is_contiguous()):
        raise ValueError("grpo_loss_static_: out_loss / out_metrics must be contiguous fp32 ([] and [16])")
    if seq_coef is not None and (seq_coef.dtype != torch.float32 or not seq_coef.is_contiguous()
                                 or tuple(seq_coef.shape) != (B,)):
        raise ValueError(f"grpo_loss_static_: seq_coef must be a contiguous fp32 [{B}] tensor")
    if dapo_normalizer is not None and (dapo_normalizer.dtype != torch.float32 or dapo_normalizer.numel() != 1):
        raise ValueError("grpo_loss_static_: dapo_normalizer must be a one-element fp32 tensor")
    dev = logp.device
    if dev.type != "cuda":
        raise ValueError("grpo_loss_static_: the operands must live on the GPU")
    for name, t in (("old_logp", old_logp), ("ref_logp", ref_logp), ("entropy", entropy), ("advantages", advantages),
                    ("mask", mask), ("token_weight", token_weight), ("entropy_mask", entropy_mask),
                    ("dapo_normalizer", dapo_normalizer), ("seq_coef", seq_coef), ("out_loss", out_loss),
                    ("out_metrics", out_metrics), ("out_dlogp", out_dlogp), ("out_dentropy", out_dentropy)):
        if t is not None and t.device != dev:
            raise ValueError(f"grpo_loss_static_: {name} is on {t.device}, logp on {dev}")
    with torch.cuda.device(dev):
        check(
            lib.trlk_grpo_loss_static(
                ptr(logp), ptr(old_logp), ptr(ref_logp), ptr(entropy), ptr(advantages), sb, st, ptr(mask),
                ptr(token_weight), ptr(entropy_mask), ptr(seq_coef), B, T, loss_type, policy_term,
                int(sequence_level), epsilon_low, epsilon_high, delta, beta, int(use_bias_correction_kl),
                grad_accum_steps, dr_grpo_denominator, ptr(dapo_normalizer), num_processes, entropy_coef,
                sapo_temperature_pos, sapo_temperature_neg, ptr(out_loss), ptr(out_metrics), ptr(out_dlogp),
                ptr(out_dentropy), current_stream(dev),
            )
        )


# --------------------------------------------------------------------------------------------
# GRPO gradient straight from the logits (K7)
# --------------------------------------------------------------------------------------------
def grpo_fused_max_vocab(dtype: torch.dtype) -> int:
    """Largest vocabulary the single-pass kernel takes for this dtype (0: not supported)."""
    return int(lib.trlk_grpo_fused_max_vocab(dtype_code(dtype))) if dtype in (torch.bfloat16, torch.float16, torch.float32) else 0


def grpo_fused_fwd_bwd(
    logits: Tensor, index: Tensor, temperature: float, keep_start: int, keep_len: int, mask: Tensor, advantages: Tensor,
    row_scale: Tensor, old_logp: Optional[Tensor], ref_logp: Optional[Tensor], token_weight: Optional[Tensor],
    seq_coef: Optional[Tensor], policy_term: int, epsilon_low: float, epsilon_high: float, delta: float, beta: float,
    use_bias_correction_kl: bool, sapo_temperature_pos: float, sapo_temperature_neg: float,
    compute_masked_rows: bool = False, entropy_weight: Optional[Tensor] = None,
) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    """One pass over `logits[:, keep_start : keep_start + keep_len]` (`[B, L, V]`, bf16 / fp16 / fp32): returns
    `(logp [B, K], entropy [B, K], lse [B, K], dlogits [B, L, V])`, the gradient for an upstream gradient of 1 on
    the loss whose per-sequence normalisation is `row_scale [B]`.  Rows with `mask == 0` are not read (outputs 0)
    unless `compute_masked_rows`.  `entropy_weight [B, K]` is d loss / d entropy per token (entropy bonus)."""
    _check_logits3d(logits)
    n_seq, length, vocab = logits.shape
    dev = logits.device
    if tuple(index.shape) != (n_seq, keep_len) or tuple(mask.shape) != (n_seq, keep_len):
        raise ValueError(f"grpo_fused: index and mask must be [{n_seq}, {keep_len}]")
    index = index.contiguous()
    if index.dtype != torch.int64:
        index = index.long()
    mask, old_logp, ref_logp, token_weight = _f32c(mask), _f32c(old_logp), _f32c(ref_logp), _f32c(token_weight)
    entropy_weight = _f32c(entropy_weight)
    for name, t in (("old_logp", old_logp), ("ref_logp", ref_logp), ("token_weight", token_weight),
                    ("entropy_weight", entropy_weight)):
        if t is not None and tuple(t.shape) != (n_seq, keep_len):
            raise ValueError(f"grpo_fused: {name} has shape {tuple(t.shape)}, expected {(n_seq, keep_len)}")
    advantages = _f32c(advantages)
    if advantages.dim() == 1 or (advantages.dim() == 2 and advantages.shape[1] == 1):
        if advantages.numel() != n_seq:
            raise ValueError("grpo_fused: advantages must have one entry per sequence")
        sb, st = 1, 0
    elif tuple(advantages.shape) == (n_seq, keep_len):
        sb, st = keep_len, 1
    else:
        raise ValueError(f"grpo_fused: advantages of shape {tuple(advantages.shape)} do not match [B] or [B, K]")
    row_scale = row_scale.reshape(n_seq).contiguous().float()
    seq_coef = None if seq_coef is None else seq_coef.reshape(n_seq).contiguous().float()
    logp = torch.empty((n_seq, keep_len), dtype=torch.float32, device=dev)
    ent = torch.empty_like(logp)
    lse = torch.empty_like(logp)
    dlogits = torch.empty((n_seq, length, vocab), dtype=logits.dtype, device=dev)
    if dlogits.numel() == 0:
        return logp, ent, lse, dlogits
    view = logits[:, keep_start : keep_start + keep_len]
    with torch.cuda.device(dev):
        check(
            lib.trlk_grpo_fused_fwd_bwd(
                view.data_ptr(), dtype_code(logits.dtype), n_seq, keep_len, vocab, view.stride(0), view.stride(1),
                ptr(index), temperature, ptr(old_logp), ptr(ref_logp), ptr(advantages), sb, st, ptr(mask),
                ptr(token_weight), ptr(seq_coef), ptr(row_scale), ptr(entropy_weight), policy_term, epsilon_low, epsilon_high, delta, beta,
                int(use_bias_correction_kl), sapo_temperature_pos, sapo_temperature_neg, ptr(logp), ptr(ent), ptr(lse),
                ptr(dlogits), length, keep_start, dlogits.stride(0), dlogits.stride(1), int(compute_masked_rows),
                ptr(_error_flag(dev)), current_stream(dev),
            )
        )
    if _SYNC_CHECKS:
        check_device_errors()
    return logp, ent, lse, dlogits


def scale_unless_one_(data: Tensor, scale: Tensor) -> Tensor:
    """In place `data *= scale` for a contiguous bf16 / fp16 / fp32 tensor and a one-element device scalar; when the
    scalar is exactly 1 the launched kernel touches nothing (no host synchronisation either way)."""
    if not data.is_contiguous() or data.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise ValueError("scale_unless_one_: contiguous bf16 / fp16 / fp32 data expected")
    scale = scale.reshape(1).to(device=data.device, dtype=torch.float32)
    with torch.cuda.device(data.device):
        check(lib.trlk_scale_unless_one(data.data_ptr(), dtype_code(data.dtype), data.numel(), ptr(scale),
                                        current_stream(data.device)))
    return data


# --------------------------------------------------------------------------------------------
# DPO / RLOO sequence losses (K4)
# --------------------------------------------------------------------------------------------
@torch.library.custom_op("trl_amd::dpo_loss", mutates_args=(), device_types="cuda")
def dpo_loss_op(token_logp: Tensor, mask: Tensor, ref_chosen: Tensor, ref_rejected: Tensor, beta: float
                ) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    """Returns (loss [], seq_logps [B], metrics [8], d loss/d token_logp [B,T])."""
    if token_logp.dim() != 2:
        raise ValueError("dpo_loss: per-token log-probs must be [B, T]")
    B, T = token_logp.shape
    if B % 2 or B < 2:
        raise ValueError("dpo_loss: the batch must be [chosen; rejected], i.e. an even number of sequences")
    dev = token_logp.device
    token_logp, mask = _f32c(token_logp), _f32c(mask)
    ref_chosen, ref_rejected = _f32c(ref_chosen), _f32c(ref_rejected)
    if tuple(mask.shape) != (B, T) or ref_chosen.numel() != B // 2 or ref_rejected.numel() != B // 2:
        raise ValueError("dpo_loss: mask must be [B, T] and the reference log-probs [B/2] each")
    loss = torch.empty((), dtype=torch.float32, device=dev)
    seq = torch.empty((B,), dtype=torch.float32, device=dev)
    metrics = torch.empty((_lib.DPO_NUM_METRICS,), dtype=torch.float32, device=dev)
    dlogp = torch.empty((B, T), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        check(lib.trlk_dpo_loss(ptr(token_logp), ptr(mask), ptr(ref_chosen), ptr(ref_rejected), B, T, beta, ptr(seq),
                                ptr(loss), ptr(metrics), ptr(dlogp), current_stream(dev)))
    return loss, seq, metrics, dlogp


@dpo_loss_op.register_fake
def _(token_logp, mask, ref_chosen, ref_rejected, beta):
    f = lambda *s: torch.empty(s, dtype=torch.float32, device=token_logp.device)  # noqa: E731
    return f(), f(token_logp.shape[0]), f(_lib.DPO_NUM_METRICS), f(*token_logp.shape)


def _seq_setup(ctx, inputs, output):
    ctx.save_for_backward(output[3], inputs[1])
    ctx.n_inputs = len(inputs)
    ctx.logp_dtype = inputs[0].dtype
    ctx.indicator = True
    ctx.set_materialize_grads(False)


def _seq_backward(ctx, g_loss, g_seq, g_metrics, g_dlogp):
    dlogp, mask = ctx.saved_tensors
    g = None
    if g_loss is not None:
        g = g_loss * dlogp
    if g_seq is not None:
        w = (mask != 0).float() if ctx.indicator else mask.float()
        extra = g_seq.unsqueeze(1) * w
        g = extra if g is None else g + extra
    return (None if g is None else g.to(ctx.logp_dtype),) + (None,) * (ctx.n_inputs - 1)


dpo_loss_op.register_autograd(_seq_backward, setup_context=_seq_setup)


@torch.library.custom_op("trl_amd::rloo_loss", mutates_args=(), device_types="cuda")
def rloo_loss_op(token_logp: Tensor, mask: Tensor, old_seq_logps: Tensor, advantages: Tensor, epsilon_low: float,
                 epsilon_high: float) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    """Returns (loss [], seq_logps [B], metrics [8], d loss/d token_logp [B,T])."""
    if token_logp.dim() != 2:
        raise ValueError("rloo_loss: per-token log-probs must be [B, T]")
    B, T = token_logp.shape
    dev = token_logp.device
    token_logp, mask = _f32c(token_logp), _f32c(mask)
    old_seq_logps, advantages = _f32c(old_seq_logps), _f32c(advantages)
    if tuple(mask.shape) != (B, T) or old_seq_logps.numel() != B or advantages.numel() != B:
        raise ValueError("rloo_loss: mask must be [B, T]; old_logps and advantages [B]")
    loss = torch.empty((), dtype=torch.float32, device=dev)
    seq = torch.empty((B,), dtype=torch.float32, device=dev)
    metrics = torch.empty((_lib.RLOO_NUM_METRICS,), dtype=torch.float32, device=dev)
    dlogp = torch.empty((B, T), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        check(lib.trlk_rloo_loss(ptr(token_logp), ptr(mask), ptr(old_seq_logps), ptr(advantages), B, T, epsilon_low,
                                 epsilon_high, ptr(seq), ptr(loss), ptr(metrics), ptr(dlogp), current_stream(dev)))
    return loss, seq, metrics, dlogp


@rloo_loss_op.register_fake
def _(token_logp, mask, old_seq_logps, advantages, epsilon_low, epsilon_high):
    f = lambda *s: torch.empty(s, dtype=torch.float32, device=token_logp.device)  # noqa: E731
    return f(), f(token_logp.shape[0]), f(_lib.RLOO_NUM_METRICS), f(*token_logp.shape)


def _rloo_setup(ctx, inputs, output):
    _seq_setup(ctx, inputs, output)
    ctx.indicator = False


rloo_loss_op.register_autograd(_seq_backward, setup_context=_rloo_setup)



# --------------------------------------------------------------------------------------------
# fused lm_head + log-prob (K5 / K6)
# --------------------------------------------------------------------------------------------
def _head_operands(hidden: Tensor, weight: Tensor, targets: Tensor):
    if hidden.dim() != 2 or weight.dim() != 2 or targets.dim() != 1:
        raise ValueError("fused head: expected hidden [N, H], weight [V, H], targets [N]")
    if hidden.shape[1] != weight.shape[1] or hidden.shape[0] != targets.shape[0]:
        raise ValueError(f"fused head: shapes do not match: hidden {tuple(hidden.shape)}, weight {tuple(weight.shape)}, "
                         f"targets {tuple(targets.shape)}")
    if hidden.dtype not in (torch.bfloat16, torch.float16):
        raise TypeError(f"fused head: hidden must be bfloat16 or float16 (got {hidden.dtype}); the matrix-core kernels "
                        "have no fp32/fp64 operand path")
    if weight.dtype != hidden.dtype:
        weight = weight.to(hidden.dtype)  # the reference casts the weight slab to the hidden dtype (utils.py:1328)
    if hidden.shape[1] % 8 != 0:
        # rows of 16-byte vectors: zero columns up to the next multiple of 8 add nothing to any product (copies of
        # both operands per call -- hidden sizes of real models are multiples of 8 and never come here)
        pad = (-hidden.shape[1]) % 8
        hidden = torch.nn.functional.pad(hidden, (0, pad))
        weight = torch.nn.functional.pad(weight, (0, pad))

    def rows_ok(t):
        return t.stride(1) == 1 and t.stride(0) % 8 == 0 and t.stride(0) >= t.shape[1] and t.data_ptr() % 16 == 0

    if not rows_ok(hidden):
        hidden = hidden.contiguous()
    if not rows_ok(weight):
        weight = weight.contiguous()
    if targets.dtype != torch.int64:
        targets = targets.long()
    return hidden, weight, targets.contiguous()


def _head_stash_shape(n_tokens: int, vocab: int) -> tuple[int, int, int]:
    """Shape of the stash as an fp16 tensor `[rows, tokens padded, 4]`: the library's own layout (softmax numerators
    of 4 vocabulary rows per token, then their reference exponents and the targets' logits)."""
    ld = ctypes.c_int64(0)
    nbytes = lib.trlk_fused_head_stash_bytes(n_tokens, vocab, ctypes.addressof(ld))
    return nbytes // (8 * ld.value), ld.value, 4


def head_stash_fits(n_tokens: int, vocab: int) -> bool:
    """Whether the forward should keep its softmax numerators for the backward: the buffer (2.07 bytes per logit,
    both dimensions padded to 256) must fit the budget `TRL_AMD_HEAD_STASH_GIB` (GiB, default 24; 0 = always
    recompute)."""
    budget = float(os.environ.get("TRL_AMD_HEAD_STASH_GIB", "24"))
    if n_tokens <= 0 or budget <= 0:
        return False
    return lib.trlk_fused_head_stash_bytes(n_tokens, vocab, None) <= budget * 2**30


def _head_bias(bias, vocab):
    if bias is None:
        return None
    if bias.shape != (vocab,):
        raise ValueError(f"fused head: bias must have shape [{vocab}], got {tuple(bias.shape)}")
    return bias.detach().float().contiguous()


@torch.library.custom_op("trl_amd::fused_head_fwd", mutates_args=(), device_types="cuda")
def fused_head_fwd(hidden: Tensor, weight: Tensor, targets: Tensor, temperature: float, softcap: float,
                   logit_scale: float, bias: Optional[Tensor] = None,
                   stash: bool = False) -> tuple[Tensor, Tensor, Tensor, Tensor, Tensor]:
    """hidden [N, H], weight [V, H] (bf16/fp16), targets int64 [N] -> fp32 (logp, entropy, log_z, target_is_max),
    each [N]; target_is_max is 1 where argmax(logits) == target.  `softcap <= 0` means no soft-capping.
    `bias` [V] (any float dtype) is added to `hidden @ weight.T` before scaling.  With `stash` the fifth
    output holds the softmax numerators (fp16, in the library's own layout) for `fused_head_bwd`; it is empty
    otherwise."""
    hidden, weight, targets = _head_operands(hidden, weight, targets)
    n, h = hidden.shape
    v = weight.shape[0]
    dev = hidden.device
    bias32 = _head_bias(bias, v)
    logp = torch.empty((n,), dtype=torch.float32, device=dev)
    ent = torch.empty((n,), dtype=torch.float32, device=dev)
    log_z = torch.empty((n,), dtype=torch.float32, device=dev)
    hit = torch.empty((n,), dtype=torch.float32, device=dev)
    if n == 0:
        return logp, ent, log_z, hit, torch.empty((0, 0, 4), dtype=torch.float16, device=dev)
    if stash:
        saved = torch.empty(_head_stash_shape(n, v), dtype=torch.float16, device=dev)
    else:
        saved = torch.empty((0, 0, 4), dtype=torch.float16, device=dev)
    ws_bytes = lib.trlk_fused_head_fwd_workspace_bytes(n)
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        check(lib.trlk_fused_head_fwd(ptr(hidden), ptr(weight), ptr(targets), dtype_code(hidden.dtype), n, v, h,
                                      hidden.stride(0), weight.stride(0), temperature, softcap, logit_scale,
                                      ptr(bias32), ptr(logp), ptr(ent), ptr(log_z), ptr(hit),
                                      ptr(saved) if stash else None, saved.shape[1] if stash else 0,
                                      ptr(_error_flag(dev)), ptr(ws), ws_bytes, current_stream(dev)))
    if _SYNC_CHECKS:
        check_device_errors()
    return logp, ent, log_z, hit, saved


@fused_head_fwd.register_fake
def _(hidden, weight, targets, temperature, softcap, logit_scale, bias=None, stash=False):
    f = lambda: torch.empty((hidden.shape[0],), dtype=torch.float32, device=hidden.device)  # noqa: E731
    vpad, cols = ((weight.shape[0] + 255) // 256 * 256, (hidden.shape[0] + 255) // 256 * 256) if stash else (0, 0)
    rows = vpad // 4 + vpad // 128 + 1 if stash else 0
    return f(), f(), f(), f(), torch.empty((rows, cols, 4), dtype=torch.float16, device=hidden.device)


@torch.library.custom_op("trl_amd::fused_head_bwd", mutates_args=(), device_types="cuda")
def fused_head_bwd(hidden: Tensor, weight: Tensor, targets: Tensor, temperature: float, softcap: float,
                   logit_scale: float, log_z: Tensor, g_logp: Tensor, chunk_size: int,
                   bias: Optional[Tensor] = None, stash: Optional[Tensor] = None,
                   stash_cols: Optional[Tensor] = None) -> tuple[Tensor, Tensor, Tensor]:
    """Returns (d hidden [N, H], d weight [V, H]) in the operand dtype and d bias (fp32 [V]; empty without a bias).
    `stash`: the fifth output of a `fused_head_fwd(..., stash=True)` on the same operands (skips the recompute);
    `stash_cols` (int32 [N]): the forward's row of each token when rows were dropped since (see `head_backward`)."""
    w_dtype = weight.dtype
    h_true = hidden.shape[1] if hidden.dim() == 2 else 0
    hidden, weight, targets = _head_operands(hidden, weight, targets)
    n, h = hidden.shape
    v = weight.shape[0]
    dev = hidden.device
    d_hidden = torch.empty((n, h), dtype=hidden.dtype, device=dev)
    d_weight = torch.empty((v, h), dtype=hidden.dtype, device=dev)
    g = g_logp.contiguous().float()
    bias32 = _head_bias(bias, v)
    d_bias = torch.empty((v if bias is not None else 0,), dtype=torch.float32, device=dev)
    if stash is not None and stash.numel() == 0:
        stash = None
    if stash is None:
        stash_cols = None
    if stash_cols is not None:
        if stash_cols.dtype != torch.int32 or stash_cols.shape != (n,):
            raise ValueError("fused head: stash_cols must be int32 [N]")
        stash_cols = stash_cols.contiguous()
    if stash is not None and (stash.dtype != torch.float16 or stash.dim() != 3 or stash.shape[2] != 4 or
                              not stash.is_contiguous() or stash.shape[0] != _head_stash_shape(1, v)[0] or
                              (stash_cols is None and stash.shape[1] < (n + 255) // 256 * 256)):
        raise ValueError("fused head: the stash does not belong to these operands")
    ws_bytes = lib.trlk_fused_head_bwd_workspace_bytes(max(n, 1), v, h, chunk_size)
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        check(lib.trlk_fused_head_bwd(ptr(hidden), ptr(weight), ptr(targets), dtype_code(hidden.dtype), n, v, h,
                                      hidden.stride(0), weight.stride(0), temperature, softcap, logit_scale,
                                      ptr(bias32), ptr(log_z), ptr(g), chunk_size, ptr(stash),
                                      stash.shape[1] if stash is not None else 0, ptr(stash_cols), ptr(d_hidden),
                                      ptr(d_weight),
                                      ptr(d_bias) if bias is not None else None, ptr(ws), ws_bytes, current_stream(dev)))
    if h != h_true:  # the operands were padded to a multiple of 8 columns
        d_hidden, d_weight = d_hidden[:, :h_true].contiguous(), d_weight[:, :h_true].contiguous()
    return d_hidden, (d_weight if w_dtype == d_weight.dtype else d_weight.to(w_dtype)), d_bias


@fused_head_bwd.register_fake
def _(hidden, weight, targets, temperature, softcap, logit_scale, log_z, g_logp, chunk_size, bias=None, stash=None,
      stash_cols=None):
    return (torch.empty_like(hidden), torch.empty_like(weight),
            torch.empty((weight.shape[0] if bias is not None else 0,), dtype=torch.float32, device=hidden.device))


def split_bf16x3(x: Tensor, side: int) -> Tensor:
    """fp32 `[R, C]` -> bf16 `[R, 6 * cpad]` (`cpad` = C rounded up to 8): the three bf16 pieces of every entry, laid
    out along the contraction axis for the left (`side` 0) or right (`side` 1) operand of an NT product, so that the
    matrix cores return the fp32 product to fp32 rounding (`trlk_split_bf16x3`)."""
    if x.dim() != 2 or x.dtype != torch.float32 or not x.is_cuda:
        raise TypeError("split_bf16x3: expected a 2-D float32 tensor on the GPU")
    if x.stride(1) != 1:
        x = x.contiguous()
    rows, cols = x.shape
    cpad = (cols + 7) // 8 * 8
    out = torch.empty((rows, 6 * cpad), dtype=torch.bfloat16, device=x.device)
    with torch.cuda.device(x.device):
        check(lib.trlk_split_bf16x3(ptr(x), rows, cols, x.stride(0) if rows > 1 else cols, side, ptr(out), 6 * cpad,
                                    current_stream(x.device)))
    return out


def gemm_nt(a: Tensor, b: Tensor, out: Optional[Tensor] = None, accumulate: bool = False) -> Tensor:
    """`a [M, K] @ b [N, K].T` on the matrix cores (bf16 / fp16 operands with K contiguous, fp32 accumulation) into a
    float32 `[M, N]` tensor; with `accumulate` the product is added to `out` (`trlk_gemm_nt`)."""
    if a.dim() != 2 or b.dim() != 2 or a.shape[1] != b.shape[1] or a.dtype != b.dtype or not a.is_cuda:
        raise ValueError(f"gemm_nt: operands do not match: {tuple(a.shape)} {a.dtype}, {tuple(b.shape)} {b.dtype}")
    a = a if a.stride(1) == 1 else a.contiguous()
    b = b if b.stride(1) == 1 else b.contiguous()
    m, k = a.shape
    n = b.shape[0]
    if out is None:
        if accumulate:
            raise ValueError("gemm_nt: accumulate needs an output to add to")
        out = torch.empty((m, n), dtype=torch.float32, device=a.device)
    elif out.shape != (m, n) or out.dtype != torch.float32 or out.stride(1) != 1:
        raise ValueError("gemm_nt: out must be a float32 [M, N] tensor with contiguous rows")
    with torch.cuda.device(a.device):
        check(lib.trlk_gemm_nt(ptr(a), a.stride(0), ptr(b), b.stride(0), dtype_code(a.dtype), m, n, k, ptr(out),
                               out.stride(0), int(accumulate), current_stream(a.device)))
    return out


def head_backward(hidden: Tensor, weight: Tensor, targets: Tensor, temperature: float, softcap: float,
                  logit_scale: float, log_z: Tensor, g_logp: Tensor, chunk_size: int, bias: Optional[Tensor] = None,
                  stash: Optional[Tensor] = None) -> tuple[Tensor, Tensor, Tensor]:
    """`fused_head_bwd` that first drops the tokens whose upstream gradient is exactly zero (masked positions of
    a policy loss): their dz row is zero, so they add nothing to d weight and their d hidden row is zero.  Both
    products shrink with the share of such tokens; one host synchronisation (the count) per call.  Tokens are only
    dropped when at least a tenth of them can go."""
    n = hidden.shape[0]
    g = g_logp.reshape(-1)
    if n == 0 or os.environ.get("TRL_AMD_HEAD_DROP_ZERO_GRAD", "1") == "0":
        return fused_head_bwd(hidden, weight, targets, temperature, softcap, logit_scale, log_z, g, chunk_size, bias, stash)
    active = g != 0
    n_active = int(active.sum())
    if n_active > 0.9 * n:
        return fused_head_bwd(hidden, weight, targets, temperature, softcap, logit_scale, log_z, g, chunk_size, bias, stash)
    idx = active.nonzero().squeeze(1)
    d_hidden = torch.zeros_like(hidden)
    if n_active == 0:
        d_bias = torch.zeros((weight.shape[0] if bias is not None else 0,), dtype=torch.float32, device=hidden.device)
        return d_hidden, torch.zeros_like(weight), d_bias
    cols = idx.to(torch.int32) if stash is not None and stash.numel() else None
    d_h, d_weight, d_bias = fused_head_bwd(
        hidden.index_select(0, idx), weight, targets.index_select(0, idx), temperature, softcap, logit_scale,
        log_z.index_select(0, idx), g.index_select(0, idx), chunk_size, bias, stash, cols)
    d_hidden.index_copy_(0, idx, d_h)
    return d_hidden, d_weight, d_bias


NAN = math.nan

"""The log-prob / loss part of the reference's `GRPOTrainer`, as mix-in methods with the
reference's signatures plus the functional forms they are built from.

`GRPOLossMixin._get_per_token_logps_and_entropies` and `GRPOLossMixin._compute_loss` read the
same trainer attributes and `inputs` keys as the reference methods
(trl/trainer/grpo_trainer.py:1435-1541, 2991-3260) and can be bound onto a `GRPOTrainer`
(see `trl_amd.integration.patch_trl`).  Differences, all deliberate:
  * the logits are never divided in place; the temperature is applied inside the kernel;
  * log-probs and entropies come back in fp32 whatever the logits dtype;
  * one kernel call returns every metric; they reach the host in a single copy.
"""
from __future__ import annotations

import math

import torch
from torch import Tensor

from .. import _lib, ops
from .utils import logps_and_entropies, nanmax, nanmin  # noqa: F401  (re-exported for callers that patch)

__all__ = [
    "per_token_logps_and_entropies",
    "grpo_loss",
    "grpo_loss_from_logits",
    "grpo_single_pass_supported",
    "group_advantages",
    "get_off_policy_mask",
    "get_high_entropy_mask",
    "get_gamma_weights",
    "vllm_importance_sampling_ratio",
    "GRPOLossMixin",
]

group_advantages = ops.group_advantages


def per_token_logps_and_entropies(
    logits: Tensor, input_ids: Tensor, logits_to_keep: int, temperature: float = 1.0, compute_entropy: bool = True,
    entropy_requires_grad: bool = False, row_mask: Tensor | None = None,
) -> tuple[Tensor, Tensor | None]:
    """`[B, L, V]` model logits -> fp32 `(logps [B, K], entropies [B, K] | None)` for the last
    `K = logits_to_keep` tokens of `input_ids`: drops the last position, keeps the last K, divides by
    the temperature (trl/trainer/grpo_trainer.py:1514-1521) -- as index arithmetic on the full tensor,
    so the backward writes the `[B, L, V]` gradient directly (rows outside the window zero).
    `row_mask` (`[B, K]`, zero = skip) makes the kernel skip those rows: they are not read and yield 0."""
    if logits.dim() != 3:
        raise ValueError("expected [B, L, V] logits")
    length = logits.shape[1]
    keep_len = min(logits_to_keep, length - 1)
    keep_start = length - 1 - keep_len
    ids = input_ids[:, -keep_len:] if keep_len > 0 else input_ids[:, :0]
    if logits.shape[-1] > 1 and logits.stride(-1) != 1:
        logits = logits.contiguous()
    logp, ent = logps_and_entropies(logits, ids, temperature, keep_start, keep_len, row_mask)
    if not compute_entropy:
        return logp, None
    return logp, (ent if entropy_requires_grad else ent.detach())


def get_off_policy_mask(advantages, per_token_logps, sampling_per_token_logps, mask, off_policy_threshold):
    """(B, 1) keep-mask of trl/trainer/grpo_trainer.py:2920-2939 ([B, T]-sized torch ops)."""
    gap = sampling_per_token_logps - per_token_logps.detach()
    mean_gap = (gap * mask).sum(dim=1, keepdim=True) / mask.sum(dim=1, keepdim=True).clamp(min=1.0)
    return ((advantages >= 0) | (mean_gap <= off_policy_threshold)).to(dtype=mask.dtype)


_IS_MODES = ("token_truncate", "token_mask", "sequence_truncate", "sequence_mask")


def vllm_importance_sampling_ratio(old_per_token_logps, sampling_per_token_logps, completion_mask, tool_mask=None,
                                   mode="sequence_mask", clip_min=None, clip_max=None):
    """Correction factor for the sampler/trainer distribution mismatch (trl/trainer/grpo_trainer.py:2578-2623):
    `exp((old - sampling) * mask)` per token (`token_*` modes, `(B, T)`) or of the per-sequence sum
    (`sequence_*`, `(B, 1)`), clamped to `[clip_min, clip_max]` (`*_truncate`) or zeroed outside it (`*_mask`).
    Also returns the five logged statistics (:2779-2813) as 0-d tensors of this process's batch:
    `sampling_logp_difference/{mean,max}`, `importance_sampling_ratio/{min,mean,max}` (0 when no token is active)."""
    if mode not in _IS_MODES:
        raise ValueError(f"Unknown vLLM importance sampling level: {mode}. Possible values are 'token_truncate', "
                         "'token_mask', 'sequence_truncate', and 'sequence_mask'.")
    mask = completion_mask if tool_mask is None else completion_mask * tool_mask
    diff = (old_per_token_logps - sampling_per_token_logps) * mask
    sequence_level = mode.startswith("sequence")
    ratio = torch.exp(diff.sum(dim=-1, keepdim=True) if sequence_level else diff)
    if mode.endswith("truncate"):
        ratio = torch.clamp(ratio, min=clip_min, max=clip_max)
    else:
        lo = -math.inf if clip_min is None else clip_min
        hi = math.inf if clip_max is None else clip_max
        ratio = ratio.masked_fill((ratio < lo) | (ratio > hi), 0.0)
    keep = mask.bool()
    delta = torch.abs(old_per_token_logps - sampling_per_token_logps)[keep]
    flat = ratio.flatten() if sequence_level else ratio[keep]
    zero = torch.zeros((), dtype=ratio.dtype, device=ratio.device)
    stats = {
        "sampling/sampling_logp_difference/mean": delta.mean() if delta.numel() else zero,
        "sampling/sampling_logp_difference/max": delta.max() if delta.numel() else zero,
        "sampling/importance_sampling_ratio/min": flat.min() if flat.numel() else zero,
        "sampling/importance_sampling_ratio/mean": flat.mean() if flat.numel() else zero,
        "sampling/importance_sampling_ratio/max": flat.max() if flat.numel() else zero,
    }
    return ratio, stats


def get_high_entropy_mask(entropies, mask, threshold, accelerator=None):
    """Boolean mask of the tokens at or above the `threshold` entropy quantile
    (trl/trainer/grpo_trainer.py:1396-1432); with an `accelerator` the active entropies are padded
    and gathered across processes first, as the reference does."""
    local = entropies[mask.bool()].float()
    if accelerator is not None:
        pad_value = -1e9
        gathered = accelerator.gather(accelerator.pad_across_processes(local, dim=0, pad_index=pad_value))
        gathered = gathered[gathered != pad_value]
    else:
        gathered = local
    if gathered.numel() == 0:
        return torch.zeros_like(entropies, dtype=torch.bool)
    cut = torch.quantile(gathered, threshold)
    return ((entropies * mask.float()) >= cut) & mask.bool()


@torch.no_grad()
def get_gamma_weights(advantages, log_ratio_per_token, mask, importance_sampling_ratio=None, k_pos=2.0,
                      lambda_pos=3.0, k_neg=3.0, lambda_neg=2.0):
    """VESPO's detached `(B, 1)` sequence coefficients phi(w) = e^lambda w^k e^(-lambda w), evaluated in
    log space with w = exp(sum over active tokens of the clamped log-ratios), optionally times the
    sampler correction (trl/trainer/grpo_trainer.py:2941-2989).  `[B, T]`-sized torch ops."""
    floor = math.log(1e-8)
    log_w = (log_ratio_per_token.clamp(-20.0, 20.0) * mask).sum(dim=-1, keepdim=True)
    if importance_sampling_ratio is not None:
        log_w = log_w + torch.log(importance_sampling_ratio).clamp(floor, 20.0).sum(dim=-1, keepdim=True)
    log_w = log_w.clamp(floor, 20.0)
    nonneg = advantages >= 0
    k = torch.where(nonneg, k_pos, k_neg)
    lam = torch.where(nonneg, lambda_pos, lambda_neg).clamp(min=1e-4)
    phi = torch.exp(lam + k * log_w - lam * torch.exp(log_w))
    return phi.nan_to_num(nan=0.0, posinf=0.0, neginf=0.0)


def grpo_loss(
    per_token_logps: Tensor,
    advantages: Tensor,
    mask: Tensor,
    *,
    entropies: Tensor | None = None,
    old_per_token_logps: Tensor | None = None,
    ref_per_token_logps: Tensor | None = None,
    loss_type: str = "dapo",
    epsilon_low: float = 0.2,
    epsilon_high: float = 0.2,
    beta: float = 0.0,
    delta: float | None = None,
    max_completion_length: int | None = None,
    num_items_in_batch: Tensor | float | None = None,
    num_processes: int = 1,
    grad_accum_steps: float = 1.0,
    use_bias_correction_kl: bool = False,
    token_weight: Tensor | None = None,
    entropy_mask: Tensor | None = None,
    entropy_coef: float = 0.0,
    importance_sampling_level: str = "token",
    sapo_temperature_pos: float = 1.0,
    sapo_temperature_neg: float = 1.05,
    vespo_params: tuple[float, float, float, float] = (2.0, 3.0, 3.0, 2.0),
    importance_sampling_ratio: Tensor | None = None,
) -> tuple[Tensor, Tensor]:
    """Fused GRPO-family loss on `[B, T]` log-probs: loss types grpo, bnpo, dr_grpo, dapo, luspo, cispo,
    sapo and vespo, token- or sequence-level importance weights.

    `token_weight` is the product of every `[B, T]` factor the reference multiplies onto the policy term
    (off-policy mask, entropy mask, sampler importance ratio).  `importance_sampling_ratio` is only read
    by vespo, whose sequence coefficients `(k_pos, lambda_pos, k_neg, lambda_neg) = vespo_params` absorb it.

    Returns `(loss, metrics)`; `metrics` is the fp32 device vector indexed by
    `trl_amd._lib`'s `trlk_grpo_metric` order (see include/trlk.h).  Differentiable w.r.t.
    `per_token_logps` (and `entropies` when `entropy_coef != 0`)."""
    if loss_type not in ops.LOSS_TYPES:
        raise ValueError(f"Unknown loss type: {loss_type}")
    if importance_sampling_level not in ("token", "sequence"):
        raise ValueError(
            f"Unknown importance sampling level: {importance_sampling_level}. Possible values are 'token' "
            "and 'sequence'."
        )
    if beta != 0.0 and ref_per_token_logps is None:
        raise KeyError("ref_per_token_logps")
    seq_level = importance_sampling_level == "sequence"
    reduce_code, term_code = ops.LOSS_TYPES[loss_type]
    dev = per_token_logps.device
    seq_coef = None
    phi_tokens = None
    if loss_type == "vespo":
        old = per_token_logps.detach() if old_per_token_logps is None else old_per_token_logps
        adv2 = advantages.unsqueeze(1) if advantages.dim() == 1 else advantages
        phi = get_gamma_weights(adv2.float(), per_token_logps.detach().float() - old.float(), mask.float(),
                                importance_sampling_ratio, *vespo_params)
        if phi.shape[1] == 1:
            seq_coef = phi
        else:
            # per-token advantages make the coefficients per token (the sign of each advantage picks k and lambda):
            # they act exactly like a per-token weight on -A * logp, so that is how the kernel gets them
            phi_tokens = phi
            seq_coef = torch.ones((phi.shape[0], 1), dtype=torch.float32, device=dev)
            token_weight = phi if token_weight is None else token_weight.float() * phi
    dapo_norm = None
    dr_denominator = 1.0
    if reduce_code == _lib.DAPO:
        if num_items_in_batch is None:
            raise KeyError("num_items_in_batch")
        dapo_norm = (
            num_items_in_batch.to(device=dev, dtype=torch.float32)
            if torch.is_tensor(num_items_in_batch)
            else torch.tensor(float(num_items_in_batch), dtype=torch.float32, device=dev)
        )
    if loss_type == "dr_grpo":
        if max_completion_length is None:
            raise ValueError("dr_grpo needs max_completion_length")
        dr_denominator = float(per_token_logps.shape[0] * max_completion_length)
    loss, metrics, _, _ = ops.grpo_loss_op(
        per_token_logps, old_per_token_logps, ref_per_token_logps if beta != 0.0 else None, entropies, advantages,
        mask, token_weight, entropy_mask, dapo_norm, reduce_code, float(epsilon_low),
        float(epsilon_high), math.nan if delta is None else float(delta), float(beta), bool(use_bias_correction_kl),
        float(grad_accum_steps), dr_denominator, float(num_processes), float(entropy_coef), term_code, seq_level,
        seq_coef, float(sapo_temperature_pos), float(sapo_temperature_neg),
    )
    if phi_tokens is not None:  # the logged coefficient is then the masked token mean of phi (grpo_trainer.py:3257-3258)
        m = mask.float()
        metrics = metrics.clone()
        metrics[_METRIC_INDEX["AUX_SUM"]] = (phi_tokens * m).sum()
        metrics[_METRIC_INDEX["AUX_COUNT"]] = m.sum()
        metrics[_METRIC_INDEX["AUX_MEAN"]] = metrics[_METRIC_INDEX["AUX_SUM"]] / m.sum().clamp(min=1.0)
    return loss, metrics


_SINGLE_PASS_LOSS_TYPES = ("grpo", "bnpo", "dr_grpo", "dapo", "cispo", "sapo")


# Rows shorter than this go through the two-pass kernels by default: on bf16 [64, 1024, V] logits with half of the
# rows masked the one pass takes 0.70 / 0.78 / 0.82 / 1.15 ms at V = 8192 / 16384 / 20480 / 32000, the two passes
# 0.51 / 0.79 / 0.94 / 1.41 ms.
_SINGLE_PASS_MIN_ROW_BYTES = 40960


def grpo_single_pass_supported(logits: Tensor, loss_type: str = "dapo", importance_sampling_level: str = "token",
                               entropy_coef: float = 0.0, entropy_mask: Tensor | None = None) -> bool:
    """Whether `grpo_loss_from_logits` can go from these logits to their gradient in one pass: a token-level
    loss type, with or without entropy bonus but without an entropy-quantile mask (the gradient coefficients of
    a token then depend on nothing but that token), bf16 / fp16 / fp32 logits whose rows the kernel takes
    (`ops.grpo_fused_max_vocab`)."""
    if loss_type not in _SINGLE_PASS_LOSS_TYPES or importance_sampling_level != "token":
        return False
    if entropy_mask is not None:  # (a mask derived from every token's entropy needs the forward pass first)
        return False
    if logits.dim() != 3 or not logits.is_cuda or logits.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        return False
    vocab = logits.shape[-1]
    per_vector = 16 // logits.element_size()
    if vocab > ops.grpo_fused_max_vocab(logits.dtype) or (vocab > 1 and logits.stride(-1) != 1):
        return False
    whole = (vocab % per_vector == 0 and logits.data_ptr() % 16 == 0 and logits.stride(0) % per_vector == 0
             and logits.stride(1) % per_vector == 0)
    # (rows that are not whole aligned 16-byte vectors are peeled to their alignment by the kernel, and must still
    # hold a whole vector then)
    return vocab >= (per_vector if whole else 2 * per_vector)


class _GRPOFromLogits(torch.autograd.Function):
    """loss (and the detached log-probs / entropies) from the logits; the gradient w.r.t. the logits was
    written by the same pass and is only scaled by the upstream gradient in `backward`."""

    @staticmethod
    def forward(ctx, logits, completion_ids, advantages, mask, temperature, kw):
        length = logits.shape[1]
        if kw["keep_start"] is None:
            keep_len = min(completion_ids.shape[1], length - 1)
            keep_start = length - 1 - keep_len
        else:
            keep_len, keep_start = completion_ids.shape[1], int(kw["keep_start"])
            if keep_start < 0 or keep_start + keep_len > length:
                raise ValueError("grpo_loss_from_logits: keep_start + K exceeds the logits' rows")
        ids = completion_ids[:, -keep_len:] if keep_len > 0 else completion_ids[:, :0]
        mask_f = mask[:, -keep_len:].float() if keep_len > 0 else mask[:, :0].float()
        n_seq = logits.shape[0]
        reduce_code, term_code = ops.LOSS_TYPES[kw["loss_type"]]
        ga = 1.0 if reduce_code == _lib.DAPO else float(kw["grad_accum_steps"])
        # d loss / d (masked token loss of sequence b): what the loss kernel's second pass applies to its rows
        if reduce_code == _lib.GRPO:
            row_scale = (1.0 / n_seq) / ga / mask_f.sum(dim=1).clamp(min=1.0)
        elif reduce_code == _lib.BNPO:
            row_scale = ((1.0 / mask_f.sum().clamp(min=1.0)) / ga).expand(n_seq)
        elif reduce_code == _lib.DR_GRPO:
            row_scale = torch.full((n_seq,), (1.0 / float(n_seq * kw["max_completion_length"])) / ga, device=logits.device)
        else:  # DAPO
            n_items = kw["num_items_in_batch"]
            n_items = (n_items.to(device=logits.device, dtype=torch.float32) if torch.is_tensor(n_items)
                       else torch.tensor(float(n_items), dtype=torch.float32, device=logits.device))
            row_scale = (float(kw["num_processes"]) / n_items.clamp(min=1.0)).reshape(1).expand(n_seq)
        ent_weight = None
        if kw["entropy_coef"] != 0.0:  # d loss / d entropy = -coef * mask / normaliser (grpo_trainer.py:3155-3181)
            if reduce_code == _lib.DAPO:
                ent_weight = mask_f * (-float(kw["entropy_coef"]) * row_scale[0])
            else:
                ent_weight = mask_f * (-float(kw["entropy_coef"]) / mask_f.sum().clamp(min=1.0) / ga)
        up = kw.get("upstream_scale")
        if up is not None:
            # the caller will multiply the loss by this factor before backward (a gradient scaler's scale, a loss
            # divisor): the gradient is written already scaled -- before its single rounding to the logits dtype --
            # and `backward` has nothing left to do
            up = (up.to(device=logits.device, dtype=torch.float32).reshape(()) if torch.is_tensor(up)
                  else torch.tensor(float(up), dtype=torch.float32, device=logits.device))
            row_scale = row_scale * up
            if ent_weight is not None:
                ent_weight = ent_weight * up
        delta = kw["delta"]
        logp, ent, _, dlogits = ops.grpo_fused_fwd_bwd(
            logits, ids, float(temperature), keep_start, keep_len, mask_f, advantages, row_scale,
            kw["old_per_token_logps"], kw["ref_per_token_logps"] if kw["beta"] != 0.0 else None, kw["token_weight"],
            None, term_code, float(kw["epsilon_low"]), float(kw["epsilon_high"]),
            math.nan if delta is None else float(delta), float(kw["beta"]), bool(kw["use_bias_correction_kl"]),
            float(kw["sapo_temperature_pos"]), float(kw["sapo_temperature_neg"]), False, ent_weight)
        if not kw["skip_masked_rows"] and keep_len > 0:
            # the outputs of the rows without gradient come from the streaming forward kernel, which reads them
            # faster than the one-workgroup-per-CU kernel would (its `compute_masked_rows` mode)
            rest = mask_f == 0
            lp0, ent0, _ = ops.logp_entropy_fwd(logits.detach(), ids.reshape(-1, 1), float(temperature), keep_start,
                                                keep_len, rest.view(torch.uint8).reshape(-1))
            logp = torch.where(rest, lp0.view_as(logp), logp)
            ent = torch.where(rest, ent0.view_as(ent), ent)
        # loss value and every metric from the [B, K]-sized kernel, on the log-probs of the same pass
        loss, metrics = grpo_loss(
            logp, advantages, mask_f, entropies=ent, old_per_token_logps=kw["old_per_token_logps"],
            ref_per_token_logps=kw["ref_per_token_logps"], loss_type=kw["loss_type"], epsilon_low=kw["epsilon_low"],
            epsilon_high=kw["epsilon_high"], beta=kw["beta"], delta=delta,
            max_completion_length=kw["max_completion_length"], num_items_in_batch=kw["num_items_in_batch"],
            num_processes=kw["num_processes"], grad_accum_steps=kw["grad_accum_steps"],
            use_bias_correction_kl=kw["use_bias_correction_kl"], token_weight=kw["token_weight"],
            entropy_coef=kw["entropy_coef"],
            sapo_temperature_pos=kw["sapo_temperature_pos"], sapo_temperature_neg=kw["sapo_temperature_neg"])
        ctx.save_for_backward(dlogits, *(() if up is None else (up,)))
        ctx.mark_non_differentiable(metrics, logp, ent)
        ctx.set_materialize_grads(False)  # (no zero tensors for the outputs that carry no gradient)
        ctx.consumed = False
        return loss, metrics, logp, ent

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, g_loss, g_metrics, g_logp, g_ent):
        dlogits, *rest = ctx.saved_tensors
        if g_loss is None:
            return None, None, None, None, None, None
        if ctx.consumed:
            # the gradient buffer is scaled in place and handed on: a second pass would scale it again
            raise RuntimeError("grpo_loss_from_logits: its backward can run only once (the gradient written by the "
                               "forward pass is handed to the graph in place); call the function again instead of "
                               "retain_graph=True")
        ctx.consumed = True
        if rest:  # the forward already applied this factor: what remains is g_loss / factor, exactly 1 as a rule
            g_loss = g_loss.to(torch.float32) / rest[0]
        # in place: the buffer belongs to this node and is handed on once (the kernel returns at once for a scale of 1)
        return ops.scale_unless_one_(dlogits, g_loss), None, None, None, None, None


def grpo_loss_from_logits(
    logits: Tensor,
    completion_ids: Tensor,
    advantages: Tensor,
    mask: Tensor,
    *,
    temperature: float = 1.0,
    old_per_token_logps: Tensor | None = None,
    ref_per_token_logps: Tensor | None = None,
    loss_type: str = "dapo",
    epsilon_low: float = 0.2,
    epsilon_high: float = 0.2,
    beta: float = 0.0,
    delta: float | None = None,
    max_completion_length: int | None = None,
    num_items_in_batch: Tensor | float | None = None,
    num_processes: int = 1,
    grad_accum_steps: float = 1.0,
    use_bias_correction_kl: bool = False,
    token_weight: Tensor | None = None,
    entropy_coef: float = 0.0,
    sapo_temperature_pos: float = 1.0,
    sapo_temperature_neg: float = 1.05,
    skip_masked_rows: bool = True,
    keep_start: int | None = None,
    upstream_scale: Tensor | float | None = None,
) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    """`[B, L, V]` model logits -> `(loss, metrics, per_token_logps [B, K], entropies [B, K])` with ONE pass over
    the logits: what `per_token_logps_and_entropies` + `grpo_loss` + `loss.backward()` do with two reads and a
    write of the logits-sized data (trl/trainer/grpo_trainer.py:1514-1532, 3026-3150) costs one read and one
    write here, because the pass that computes a row's log-prob also writes that row's gradient.

    Same window as the reference (`logits[:, :-1][:, -K:]`, `K = completion_ids.shape[1]`), same arguments
    as `grpo_loss`; `keep_start` names another first row of the window.  Only for
    `grpo_single_pass_supported(...)` configurations.  The rows outside `mask` are never read and their log-prob /
    entropy come back as 0, unless `skip_masked_rows=False` asks for them (their gradient is zero either way).  `loss.backward()` hands the `[B, L, V]` gradient
    to the graph behind `logits`; the returned log-probs and entropies are detached.

    The gradient is written by the forward pass for an upstream gradient of 1; any other upstream gradient costs
    `backward` one more read and write of the buffer.  A caller that knows the factor it will put on the loss
    before `backward()` -- the scale of a `GradScaler`, a loss divisor -- passes it as `upstream_scale` (a float or a
    0-d device tensor): the forward pass then writes the scaled gradient (scaled in fp32 before its one rounding,
    which is what keeps small fp16 gradients from flushing to zero) and `backward` leaves the buffer alone.  The
    returned loss is NOT multiplied by it.  `backward` can run once per call."""
    if loss_type not in ops.LOSS_TYPES:
        raise ValueError(f"Unknown loss type: {loss_type}")
    if not grpo_single_pass_supported(logits, loss_type):
        raise NotImplementedError(
            "grpo_loss_from_logits: this configuration needs the two-pass path (per_token_logps_and_entropies + "
            "grpo_loss): token-level loss types, bf16 / fp16 / fp32 logits with a contiguous vocabulary axis of at most "
            f"{ops.grpo_fused_max_vocab(logits.dtype) if logits.dtype in (torch.bfloat16, torch.float16, torch.float32) else 0} "
            "entries long")
    if beta != 0.0 and ref_per_token_logps is None:
        raise KeyError("ref_per_token_logps")
    if ops.LOSS_TYPES[loss_type][0] == _lib.DAPO and num_items_in_batch is None:
        raise KeyError("num_items_in_batch")
    if loss_type == "dr_grpo" and max_completion_length is None:
        raise ValueError("dr_grpo needs max_completion_length")
    if not (torch.is_grad_enabled() and logits.requires_grad):
        # nobody will ask for the gradient: the forward kernel alone (one read, nothing logits-sized written)
        length = logits.shape[1]
        keep_len = completion_ids.shape[1] if keep_start is not None else min(completion_ids.shape[1], length - 1)
        start = int(keep_start) if keep_start is not None else length - 1 - keep_len
        if start < 0 or start + keep_len > length:
            raise ValueError("grpo_loss_from_logits: keep_start + K exceeds the logits' rows")
        ids = completion_ids[:, -keep_len:] if keep_len > 0 else completion_ids[:, :0]
        m = mask[:, -keep_len:] if keep_len > 0 else mask[:, :0]
        logp, ent = logps_and_entropies(logits, ids, temperature, start, keep_len, m if skip_masked_rows else None)
        loss, metrics = grpo_loss(
            logp, advantages, m, entropies=ent, old_per_token_logps=old_per_token_logps,
            ref_per_token_logps=ref_per_token_logps, loss_type=loss_type, epsilon_low=epsilon_low,
            epsilon_high=epsilon_high, beta=beta, delta=delta, max_completion_length=max_completion_length,
            num_items_in_batch=num_items_in_batch, num_processes=num_processes, grad_accum_steps=grad_accum_steps,
            use_bias_correction_kl=use_bias_correction_kl, token_weight=token_weight, entropy_coef=entropy_coef,
            sapo_temperature_pos=sapo_temperature_pos, sapo_temperature_neg=sapo_temperature_neg)
        return loss, metrics, logp.detach(), ent.detach()
    kw = dict(old_per_token_logps=old_per_token_logps, ref_per_token_logps=ref_per_token_logps, loss_type=loss_type,
              epsilon_low=epsilon_low, epsilon_high=epsilon_high, beta=beta, delta=delta,
              max_completion_length=max_completion_length, num_items_in_batch=num_items_in_batch,
              num_processes=num_processes, grad_accum_steps=grad_accum_steps,
              use_bias_correction_kl=use_bias_correction_kl, token_weight=token_weight, entropy_coef=entropy_coef,
              sapo_temperature_pos=sapo_temperature_pos, sapo_temperature_neg=sapo_temperature_neg,
              skip_masked_rows=skip_masked_rows, keep_start=keep_start, upstream_scale=upstream_scale)
    return _GRPOFromLogits.apply(logits, completion_ids, advantages, mask, temperature, kw)


class GRPOLossMixin:
    """Methods with the reference's names and signatures; bind them onto a `GRPOTrainer`."""

    def _model_inputs(self, input_ids, attention_mask, start, stop, logits_to_keep, compute_aux_loss, *, pixel_values=None,
                      image_grid_thw=None, num_images=None, pixel_attention_mask=None, spatial_shapes=None,
                      num_tiles=None, image_sizes=None, token_type_ids=None, mm_token_type_ids=None,
                      image_position_ids=None):
        """Keyword arguments of the model call for the samples `start:stop` (trl/trainer/grpo_trainer.py:1463-1510).
        The vision tensors are indexed by patch row, image or tile rather than by sample, so the sample range is
        translated through `image_grid_thw` / `num_images` / `num_tiles`; those two lists only steer the slicing
        and are never model arguments."""
        out = {"input_ids": input_ids[start:stop], "attention_mask": attention_mask[start:stop]}
        if pixel_values is not None:
            if image_grid_thw is not None:  # patch rows of all images concatenated; one grid row per image
                first_image = [0]
                for n in num_images:
                    first_image.append(first_image[-1] + int(n))
                rows_per_image = image_grid_thw.prod(dim=-1)
                img0, img1 = first_image[start], first_image[stop]
                row0 = int(rows_per_image[:img0].sum())
                row1 = row0 + int(rows_per_image[img0:img1].sum())
                out["pixel_values"] = pixel_values[row0:row1]
                out["image_grid_thw"] = image_grid_thw[img0:img1]
            elif image_position_ids is not None:  # image-indexed tensors
                img0, img1 = sum(int(n) for n in num_images[:start]), sum(int(n) for n in num_images[:stop])
                out["pixel_values"] = pixel_values[img0:img1]
                out["image_position_ids"] = image_position_ids[img0:img1]
            elif spatial_shapes is not None:  # tile-indexed tensors
                t0, t1 = sum(int(n) for n in num_tiles[:start]), sum(int(n) for n in num_tiles[:stop])
                out["pixel_values"] = pixel_values[t0:t1]
                out["pixel_attention_mask"] = pixel_attention_mask[t0:t1]
                out["spatial_shapes"] = spatial_shapes[t0:t1]
            else:
                out["pixel_values"] = pixel_values[start:stop]
        if pixel_attention_mask is not None and spatial_shapes is None:
            out["pixel_attention_mask"] = pixel_attention_mask[start:stop]
        for name, value in (("image_sizes", image_sizes), ("token_type_ids", token_type_ids),
                            ("mm_token_type_ids", mm_token_type_ids)):
            if value is not None:
                out[name] = value[start:stop]
        if "logits_to_keep" in getattr(self, "model_kwarg_keys", ()):
            out["logits_to_keep"] = logits_to_keep + 1  # (the last position is dropped afterwards)
        out["use_cache"] = False
        if compute_aux_loss:
            out["output_router_logits"] = True
        return out

    def _get_per_token_logps_and_entropies(
        self, model, input_ids, attention_mask, logits_to_keep, batch_size=None, compute_entropy=False,
        compute_aux_loss=False, pixel_values=None, image_grid_thw=None, num_images=None, pixel_attention_mask=None,
        spatial_shapes=None, num_tiles=None, image_sizes=None, token_type_ids=None, mm_token_type_ids=None,
        image_position_ids=None, skip_rows_mask=None,
    ):
        """Reference: trl/trainer/grpo_trainer.py:1435-1541, sub-batches and multimodal inputs included.
        `skip_rows_mask` (`[B, logits_to_keep]`, not in the reference) names rows whose log-prob and
        entropy the caller will discard: they are not read and come back as 0."""
        total = input_ids.size(0)
        batch_size = batch_size or total
        vision = dict(pixel_values=pixel_values, image_grid_thw=image_grid_thw, num_images=num_images,
                      pixel_attention_mask=pixel_attention_mask, spatial_shapes=spatial_shapes, num_tiles=num_tiles,
                      image_sizes=image_sizes, token_type_ids=token_type_ids, mm_token_type_ids=mm_token_type_ids,
                      image_position_ids=image_position_ids)
        all_logps, all_entropies, all_aux = [], [], []
        entropy_grad = bool(getattr(self, "_entropy_bonus_enabled", False))
        for start in range(0, total, batch_size):
            stop = min(start + batch_size, total)
            model_inputs = self._model_inputs(input_ids, attention_mask, start, stop, logits_to_keep, compute_aux_loss,
                                              **vision)
            outputs = model(**model_inputs)
            rows = None if skip_rows_mask is None else skip_rows_mask[start:stop]
            logps, ent = per_token_logps_and_entropies(
                outputs.logits, model_inputs["input_ids"], logits_to_keep, self.temperature, compute_entropy,
                entropy_grad, rows
            )
            all_logps.append(logps)
            if compute_entropy:
                all_entropies.append(ent)
            if compute_aux_loss:
                all_aux.append(outputs.aux_loss)
        logps = torch.cat(all_logps, dim=0) if len(all_logps) > 1 else all_logps[0]
        entropies = (torch.cat(all_entropies, dim=0) if len(all_entropies) > 1 else all_entropies[0]) if compute_entropy else None
        aux_loss = torch.stack(all_aux).mean() if compute_aux_loss else None
        return logps, entropies, aux_loss

    def _compute_loss(self, model, inputs):
        """Reference: trl/trainer/grpo_trainer.py:2991-3260: every loss type, token- and sequence-level
        importance weights, static and adaptive entropy bonus."""
        if self.loss_type not in ops.LOSS_TYPES:
            raise ValueError(f"Unknown loss type: {self.loss_type}")
        prompt_ids, prompt_mask = inputs["prompt_ids"], inputs["prompt_mask"]
        completion_ids, completion_mask = inputs["completion_ids"], inputs["completion_mask"]
        input_ids = torch.cat([prompt_ids, completion_ids], dim=1)
        attention_mask = torch.cat([prompt_mask, completion_mask], dim=1)
        logits_to_keep = completion_ids.size(1)
        mask = completion_mask if "tool_mask" not in inputs else completion_mask * inputs["tool_mask"]
        aux_enabled = bool(getattr(self, "aux_loss_enabled", False))
        extra_keys = ("pixel_values", "image_grid_thw", "num_images", "pixel_attention_mask", "spatial_shapes",
                      "num_tiles", "image_sizes", "token_type_ids", "mm_token_type_ids", "image_position_ids")
        # Every use of the log-probs and entropies below is multiplied by `mask`, so rows with mask == 0
        # need not be computed at all (set `trl_amd_skip_masked_rows = False` on the trainer to compute them).
        skip = mask if getattr(self, "trl_amd_skip_masked_rows", True) else None
        if self.loss_type == "luspo":
            skip = None  # (its [B, T] forms average over the padding as well: every row's log-prob is needed)
        advantages = inputs["advantages"]
        mode = "train" if self.model.training else "eval"
        grad_accum = self.current_gradient_accumulation_steps if mode == "train" else 1.0
        bonus = bool(getattr(self, "_entropy_bonus_enabled", False))
        # One pass over the logits (log-probs and gradient from the same read) when nothing between the two
        # needs the log-probs of other tokens: token-level weights, no mask derived from the log-probs or
        # entropies.  `trl_amd_single_pass` on the trainer: False keeps the two-pass path, True takes the one pass
        # whenever the kernel accepts the logits, unset (the default) takes it when it also pays: rows of at least
        # `_SINGLE_PASS_MIN_ROW_BYTES` (a workgroup per row spends more time between rows than on them below that).
        adaptive = bonus and bool(getattr(self, "use_adaptive_entropy", False))
        # the coefficient of the end of the previous optimizer step applies to the whole accumulation window;
        # under adaptive control only while the last window's entropy was at or below the target (:3173-3179)
        apply_coef = self.entropy_coef if bonus else 0.0
        if adaptive and not (self._last_world_entropy <= self.args.entropy_target):
            apply_coef = 0.0
        want_single = getattr(self, "trl_amd_single_pass", None)
        single_pass = (
            want_single is not False and skip is not None
            and self.loss_type in _SINGLE_PASS_LOSS_TYPES and self.importance_sampling_level == "token"
            and self.top_entropy_quantile >= 1.0 and self.off_policy_mask_threshold is None
        )
        if single_pass:
            model_inputs = self._model_inputs(input_ids, attention_mask, 0, input_ids.size(0), logits_to_keep, aux_enabled,
                                              **{k: inputs.get(k) for k in extra_keys})
            outputs = model(**model_inputs)
            aux_loss = outputs.aux_loss if aux_enabled else None
            logits = outputs.logits
            if logits.shape[-1] > 1 and logits.stride(-1) != 1:
                logits = logits.contiguous()
            # the factor the training step will put on the loss before `backward`: a 0-d device tensor, no sync
            upstream = self._announced_upstream_scale(logits.device, mode)
            # fp16 gradients of a 1e5-entry softmax row sit near the bottom of the fp16 range: the one pass rounds
            # them once, so it is only taken when the scale is known at that point (or on request)
            scaler = getattr(self.accelerator, "scaler", None)
            scaled = scaler is not None and getattr(scaler, "is_enabled", lambda: True)()
            fp16_ok = scaled or getattr(self, "trl_amd_single_pass_fp16", False)
            pays = want_single is True or logits.shape[-1] * logits.element_size() >= _SINGLE_PASS_MIN_ROW_BYTES
            if (pays and grpo_single_pass_supported(logits, self.loss_type)
                    and (logits.dtype != torch.float16 or fp16_ok)):
                token_weight = None
                if self.use_vllm and self.vllm_importance_sampling_correction:
                    token_weight = inputs["importance_sampling_ratio"].float().expand(mask.shape)
                loss, metrics, per_token_logps, entropies = grpo_loss_from_logits(
                    logits, completion_ids, advantages, mask, temperature=self.temperature,
                    old_per_token_logps=inputs.get("old_per_token_logps"),
                    ref_per_token_logps=inputs["ref_per_token_logps"] if self.beta != 0.0 else None,
                    loss_type=self.loss_type, epsilon_low=self.epsilon_low, epsilon_high=self.epsilon_high,
                    beta=self.beta, delta=self.args.delta, max_completion_length=self.max_completion_length,
                    num_items_in_batch=inputs.get("num_items_in_batch"), num_processes=self.accelerator.num_processes,
                    grad_accum_steps=grad_accum, use_bias_correction_kl=self.args.use_bias_correction_kl,
                    token_weight=token_weight, entropy_coef=apply_coef,
                    sapo_temperature_pos=getattr(self.args, "sapo_temperature_pos", 1.0),
                    sapo_temperature_neg=getattr(self.args, "sapo_temperature_neg", 1.05), upstream_scale=upstream)
                return self._finish_loss(loss, metrics, entropies, mask, None, aux_loss, aux_enabled, grad_accum, mode, bonus)
            # these logits need the two-pass kernels (fp32, a vocabulary too large for one workgroup, ...)
            per_token_logps, entropies = per_token_logps_and_entropies(
                logits, input_ids, logits_to_keep, self.temperature, True, bonus, skip)
        else:
            per_token_logps, entropies, aux_loss = self._get_per_token_logps_and_entropies(
                model, input_ids, attention_mask, logits_to_keep, compute_entropy=True, compute_aux_loss=aux_enabled,
                skip_rows_mask=skip, **{k: inputs.get(k) for k in extra_keys},
            )
        entropy_mask = None
        if self.top_entropy_quantile < 1.0:
            entropy_mask = get_high_entropy_mask(entropies.detach(), mask, 1 - self.top_entropy_quantile, self.accelerator)
        token_weight = None
        old = inputs.get("old_per_token_logps")
        if self.off_policy_mask_threshold is not None:
            adv2 = advantages.unsqueeze(1) if advantages.dim() == 1 else advantages
            sampling = inputs.get("sampling_per_token_logps", per_token_logps.detach() if old is None else old)
            token_weight = get_off_policy_mask(adv2, per_token_logps, sampling, mask, self.off_policy_mask_threshold)
            token_weight = token_weight.float().expand_as(per_token_logps)
        if entropy_mask is not None:
            em = entropy_mask.float()
            token_weight = em if token_weight is None else token_weight * em
        if self.use_vllm and self.vllm_importance_sampling_correction and self.loss_type != "vespo":
            isr = inputs["importance_sampling_ratio"].float().expand_as(per_token_logps)
            token_weight = isr if token_weight is None else token_weight * isr

        loss, metrics = grpo_loss(
            per_token_logps, advantages, mask, entropies=entropies, old_per_token_logps=old,
            ref_per_token_logps=inputs["ref_per_token_logps"] if self.beta != 0.0 else None,
            loss_type=self.loss_type, epsilon_low=self.epsilon_low, epsilon_high=self.epsilon_high, beta=self.beta,
            delta=self.args.delta, max_completion_length=self.max_completion_length,
            num_items_in_batch=inputs.get("num_items_in_batch"), num_processes=self.accelerator.num_processes,
            grad_accum_steps=grad_accum, use_bias_correction_kl=self.args.use_bias_correction_kl,
            token_weight=token_weight, entropy_mask=None if entropy_mask is None else entropy_mask.float(),
            entropy_coef=apply_coef,
            importance_sampling_level=self.importance_sampling_level,
            sapo_temperature_pos=getattr(self.args, "sapo_temperature_pos", 1.0),
            sapo_temperature_neg=getattr(self.args, "sapo_temperature_neg", 1.05),
            vespo_params=(getattr(self.args, "vespo_k_pos", 2.0), getattr(self.args, "vespo_lambda_pos", 3.0),
                          getattr(self.args, "vespo_k_neg", 3.0), getattr(self.args, "vespo_lambda_neg", 2.0)),
            importance_sampling_ratio=inputs.get("importance_sampling_ratio"),
        )
        return self._finish_loss(loss, metrics, entropies, mask, entropy_mask, aux_loss, aux_enabled, grad_accum, mode, bonus)

    def _announced_upstream_scale(self, device, mode):
        """The upstream gradient `loss.backward()` will deliver to `_compute_loss`'s result, as far as the trainer's
        own attributes tell it, or None when that is 1.  Three factors sit between the returned loss and `backward`
        (transformers `Trainer.training_step`, accelerate `Accelerator.backward`):
        - `Trainer.training_step` divides by `current_gradient_accumulation_steps` unless `compute_loss_func` is set
          or the model takes loss kwargs.  The reference's `GRPOTrainer` sets `model_accepts_loss_kwargs = False`
          (trl/trainer/grpo_trainer.py:1128-1131) and hands the parent a non-None `compute_loss_func`
          (:944-950) to switch that division off; a trainer that only does the former gets the division;
        - `Accelerator.backward` divides by the accelerator's own `gradient_accumulation_steps` (1 under `Trainer`)
          except with DeepSpeed;
        - a gradient scaler (fp16 mixed precision) multiplies by its scale.
        The factors are applied to a 0-d tensor in the order autograd's backward meets them, with the operations it
        uses, so that `g_loss / factor` comes out as exactly 1 and `backward` has nothing to rescale.  A trainer whose
        step does something else still gets the right gradient: `backward` applies whatever part of the upstream
        gradient was not announced."""
        factor = None
        scaler = getattr(self.accelerator, "scaler", None)
        if scaler is not None and getattr(scaler, "is_enabled", lambda: True)():
            factor = scaler.scale(torch.ones((), dtype=torch.float32, device=device))
        if mode != "train":
            return factor
        divisors = []
        acc_steps = getattr(self.accelerator, "gradient_accumulation_steps", 1)
        if isinstance(acc_steps, (int, float)) and acc_steps != 1 and "DEEPSPEED" not in str(
                getattr(self.accelerator, "distributed_type", "")):
            divisors.append(acc_steps)
        # (attributes of transformers.Trainer; an object without them is no Trainer and divides nothing)
        if (hasattr(self, "model_accepts_loss_kwargs") and not self.model_accepts_loss_kwargs
                and getattr(self, "compute_loss_func", None) is None
                and getattr(self, "trl_amd_trainer_divides_loss", True)):
            ga = self.current_gradient_accumulation_steps
            if isinstance(ga, (int, float)) and ga != 1:
                divisors.append(ga)
        for d in divisors:
            if factor is None:
                factor = torch.ones((), dtype=torch.float32, device=device)
            factor = factor / d
        return factor

    def _finish_loss(self, loss, metrics, entropies, mask, entropy_mask, aux_loss, aux_enabled, grad_accum, mode, bonus):
        """Auxiliary loss, the adaptive entropy controller and the logged metrics (grpo_trainer.py:3152-3258)."""
        adaptive = bonus and bool(getattr(self, "use_adaptive_entropy", False))
        if aux_enabled:
            loss = loss + self.router_aux_loss_coef * aux_loss / grad_accum
            self._metrics[mode]["aux_loss"].append(self.accelerator.gather_for_metrics(aux_loss).mean().item())

        # metrics: cross-process sums of (sum, count) pairs, then one host copy
        m = metrics.detach()
        i = _METRIC_INDEX
        sums = m[[i["KL_SUM"], i["ENTROPY_SUM"], i["MASK_SUM"], i["CLIP_COUNT"], i["AUX_SUM"], i["AUX_COUNT"]]]
        clip = m[2:5] * m[i["CLIP_COUNT"]].clamp(min=1.0)
        totals = self.accelerator.reduce(torch.cat([sums, clip]), reduction="sum")
        low_min = nanmin(self.accelerator.gather(m[5:6]))
        high_max = nanmax(self.accelerator.gather(m[6:7]))
        # (the kernels' error word rides along: a token id outside the vocabulary raises here, as the reference's
        # gather would, instead of surfacing as a NaN loss)
        host = torch.cat([totals, low_min.reshape(1), high_max.reshape(1), m[7:8], ops.device_error_bits(m.device)]).tolist()
        kl_sum, ent_sum, cnt, clip_cnt, aux_sum, aux_cnt, low, high, region, lmin, hmax, policy_loss, bits = host
        ops.raise_for_error_bits(bits, m.device)
        cnt, clip_cnt, aux_cnt = max(cnt, 1.0), max(clip_cnt, 1.0), max(aux_cnt, 1.0)
        log = self._metrics[mode]
        if bonus:
            log["policy_loss"].append(policy_loss)
            if adaptive and mode == "train":  # window-global entropy drives the coefficient of the next step (:3186-3210)
                eff = mask.float() if entropy_mask is None else mask.float() * entropy_mask.float()
                stats = torch.stack([(entropies.detach() * eff).sum(), eff.sum()])
                window = getattr(self, "_entropy_window_stats", None)
                self._entropy_window_stats = stats if window is None else window.to(stats.device) + stats
                if self.accelerator.sync_gradients:
                    total = self.accelerator.reduce(self._entropy_window_stats, reduction="sum")
                    world_entropy = (total[0] / total[1].clamp(min=1.0)).item()
                    if world_entropy <= self.args.entropy_target:
                        self.entropy_coef = min(self.entropy_coef + self.args.entropy_coef_delta, self.args.entropy_coef_max)
                    else:
                        self.entropy_coef = max(self.entropy_coef - self.args.entropy_coef_delta, self.args.entropy_coef_min)
                    self._last_world_entropy = world_entropy
                    self._entropy_window_stats = None
            if mode == "train" and self.accelerator.sync_gradients:
                log["entropy_coef"].append(self.entropy_coef)
        if self.beta != 0.0:
            log["kl"].append(kl_sum / cnt)
        log["entropy"].append(ent_sum / cnt)
        if self.loss_type in ("grpo", "bnpo", "dr_grpo", "dapo", "luspo"):
            log["clip_ratio/low_mean"].append(low / clip_cnt)
            log["clip_ratio/high_mean"].append(high / clip_cnt)
            log["clip_ratio/region_mean"].append(region / clip_cnt)
            log["clip_ratio/low_min"].append(lmin)
            log["clip_ratio/high_max"].append(hmax)
        elif self.loss_type == "cispo":
            log["cispo_clip_ratio"].append(aux_sum / aux_cnt)
        elif self.loss_type == "vespo":
            log["vespo/phi_seq_mean"].append(aux_sum / aux_cnt)
        return loss


_METRIC_INDEX = {"KL_MEAN": 0, "ENTROPY_MEAN": 1, "CLIP_LOW_MEAN": 2, "CLIP_HIGH_MEAN": 3, "CLIP_REGION_MEAN": 4,
                 "CLIP_LOW_MIN": 5, "CLIP_HIGH_MAX": 6, "POLICY_LOSS": 7, "MASK_SUM": 8, "KL_SUM": 9, "ENTROPY_SUM": 10,
                 "AUX_MEAN": 11, "CLIP_COUNT": 12, "AUX_SUM": 13, "AUX_COUNT": 14}


def metrics_to_dict(metrics: Tensor, beta: float, has_entropy: bool = True, loss_type: str = "dapo") -> dict[str, float]:
    """Host dictionary with the reference's metric names (single device->host copy)."""
    m = metrics.detach().tolist()
    i = _METRIC_INDEX
    out = {}
    if beta != 0.0:
        out["kl"] = m[i["KL_MEAN"]]
    if has_entropy:
        out["entropy"] = m[i["ENTROPY_MEAN"]]
    if loss_type == "cispo":
        out["cispo_clip_ratio"] = m[i["AUX_MEAN"]]
    elif loss_type == "vespo":
        out["vespo/phi_seq_mean"] = m[i["AUX_MEAN"]]
    elif loss_type != "sapo":
        out["clip_ratio/low_mean"] = m[i["CLIP_LOW_MEAN"]]
        out["clip_ratio/high_mean"] = m[i["CLIP_HIGH_MEAN"]]
        out["clip_ratio/region_mean"] = m[i["CLIP_REGION_MEAN"]]
        out["clip_ratio/low_min"] = m[i["CLIP_LOW_MIN"]]
        out["clip_ratio/high_max"] = m[i["CLIP_HIGH_MAX"]]
    out["policy_loss"] = m[i["POLICY_LOSS"]]
    return out

"""Fused-linear losses: lm_head + log-prob + policy loss from the last hidden states, with the call
signatures of the operators the reference plugs in behind `use_liger_kernel`
(`LigerFusedLinearGRPOLoss`, trl/trainer/grpo_trainer.py:1027-1044, 2885-2907;
`LigerFusedLinearDPOLoss`, trl/trainer/dpo_trainer.py:834, 1287-1327;
`LigerFusedLinearKTOLoss`, trl/trainer/kto_trainer.py:978, 1415-1435).

Those operators live in the third-party `liger-kernel` package (pinned `>=0.8.0,<0.8.1` by the
reference, not importable here), so what is mirrored is the call contract the reference relies on:
argument names and meaning, the `(loss, metrics)` return and the position of each metric.  The
arithmetic is the reference's own `_compute_loss` (same kernels as `GRPOLossMixin._compute_loss` /
`dpo_sigmoid_loss`), fed by the fused head instead of materialised logits.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import Tensor

from .. import ops
from .grpo_trainer import _METRIC_INDEX, grpo_loss
from .utils import _ChunkedLogProbFunction

__all__ = ["FusedLinearGRPOLoss", "FusedLinearDPOLoss", "FusedLinearKTOLoss"]


def _head_logps(hidden: Tensor, weight: Tensor, targets: Tensor, keep: Tensor, temperature: float,
                chunk_size: int, bias: Tensor | None = None) -> Tensor:
    """fp32 log-probs of `targets` `[B, T]` under `softmax((hidden @ weight.T + bias) / temperature)`; only the
    rows with `keep != 0` go through the head, the others are 0 (and receive no gradient)."""
    b, t, h = hidden.shape
    sel = keep.reshape(b * t) != 0
    flat_h = hidden.reshape(b * t, h)[sel]
    flat_t = targets.reshape(b * t)[sel]
    lp_v, _ = _ChunkedLogProbFunction.apply(flat_h, weight, flat_t, float(temperature), int(chunk_size), None, 1.0,
                                            bias)
    lp = torch.zeros(b * t, dtype=torch.float32, device=hidden.device)
    lp[sel] = lp_v
    return lp.view(b, t)


class FusedLinearGRPOLoss(torch.nn.Module):
    """`loss, metrics = op(_input=hidden [B, T, H], lin_weight=W [V, H], selected_token_ids [B, T],
    attention_mask=loss_mask [B, T], advantages [B], bias=None, old_per_token_logps=None,
    ref_per_token_logps=None, vllm_is_ratio=None)`.

    `metrics = [mean_kl] (only if beta != 0) + [clip_ratio]`, the positions `compute_liger_loss` reads
    (grpo_trainer.py:2900-2901).  `loss` is not divided by the gradient-accumulation steps (the caller
    does that, :2907); the `dapo`-family normaliser is the number of active tokens of the batch, summed
    over processes and divided by their number when `torch.distributed` is initialised."""

    def __init__(self, beta: float = 0.04, epsilon_low: float = 0.2, epsilon_high: float = 0.2, temperature: float = 1.0,
                 use_ref_model: bool = True, loss_type: str = "dapo", max_completion_length: int | None = None,
                 importance_sampling_level: str = "token", delta: float | None = None,
                 use_bias_correction_kl: bool = False, sapo_temperature_pos: float = 1.0,
                 sapo_temperature_neg: float = 1.05, vespo_k_pos: float = 2.0, vespo_lambda_pos: float = 3.0,
                 vespo_k_neg: float = 3.0, vespo_lambda_neg: float = 2.0, chunk_size: int = 32768):
        super().__init__()
        if loss_type not in ops.LOSS_TYPES:
            raise ValueError(f"Unknown loss type: {loss_type}")
        self.beta = float(beta) if use_ref_model else 0.0
        self.epsilon_low, self.epsilon_high = float(epsilon_low), float(epsilon_high)
        self.temperature = float(temperature)
        self.loss_type = loss_type
        self.max_completion_length = max_completion_length
        self.importance_sampling_level = importance_sampling_level
        self.delta = delta
        self.use_bias_correction_kl = bool(use_bias_correction_kl)
        self.sapo_temperatures = (float(sapo_temperature_pos), float(sapo_temperature_neg))
        self.vespo_params = (float(vespo_k_pos), float(vespo_lambda_pos), float(vespo_k_neg), float(vespo_lambda_neg))
        self.chunk_size = int(chunk_size)

    def forward(self, _input: Tensor, lin_weight: Tensor, selected_token_ids: Tensor, attention_mask: Tensor,
                advantages: Tensor, bias: Tensor | None = None, old_per_token_logps: Tensor | None = None,
                ref_per_token_logps: Tensor | None = None, vllm_is_ratio: Tensor | None = None):
        if _input.dim() != 3:
            raise ValueError("_input must be [B, T, H] hidden states")
        if self.beta != 0.0 and ref_per_token_logps is None:
            raise ValueError("ref_per_token_logps is required when beta != 0")
        mask = attention_mask
        logps = _head_logps(_input, lin_weight, selected_token_ids, mask, self.temperature, self.chunk_size, bias)
        n_items = mask.sum().float()
        n_proc = 1
        if torch.distributed.is_available() and torch.distributed.is_initialized():
            n_proc = torch.distributed.get_world_size()
            torch.distributed.all_reduce(n_items)
        vespo = self.loss_type == "vespo"
        token_weight = None
        if vllm_is_ratio is not None and not vespo:
            token_weight = vllm_is_ratio.float().expand_as(logps)
        loss, m = grpo_loss(
            logps, advantages, mask, old_per_token_logps=old_per_token_logps,
            ref_per_token_logps=ref_per_token_logps if self.beta != 0.0 else None, loss_type=self.loss_type,
            epsilon_low=self.epsilon_low, epsilon_high=self.epsilon_high, beta=self.beta, delta=self.delta,
            max_completion_length=self.max_completion_length, num_items_in_batch=n_items, num_processes=n_proc,
            grad_accum_steps=1.0, use_bias_correction_kl=self.use_bias_correction_kl, token_weight=token_weight,
            importance_sampling_level=self.importance_sampling_level, sapo_temperature_pos=self.sapo_temperatures[0],
            sapo_temperature_neg=self.sapo_temperatures[1], vespo_params=self.vespo_params,
            importance_sampling_ratio=vllm_is_ratio if vespo else None,
        )
        m = m.detach()
        metrics = []
        if self.beta != 0.0:
            metrics.append(m[_METRIC_INDEX["KL_MEAN"]])
        metrics.append(m[_METRIC_INDEX["CLIP_REGION_MEAN"]])
        return loss, metrics


class FusedLinearDPOLoss(torch.nn.Module):
    """`loss, metrics = op(lin_weight [V, H], _input [2P, T, H], target [2P, T] (-100 = ignored),
    bias=None, ref_input=None, ref_weight=None, ref_bias=None)`; rows `[0, P)` are the chosen, `[P, 2P)`
    the rejected sequences; without `ref_weight` the reference model shares `lin_weight` and `bias`.  `metrics = (chosen_logps [P], rejected_logps [P], chosen_logits_mean,
    rejected_logits_mean, nll_loss, chosen_rewards [P], rejected_rewards [P])`, the order
    `_compute_loss_liger` unpacks (dpo_trainer.py:1293-1301).  Loss types: `sigmoid` (one fused loss kernel) and
    the other pair losses of the third-party operator, `apo_zero`, `apo_down`, `sppo_hard`, `nca_pair`, with the
    reference's own formulas (dpo_trainer.py:1396-1519).  The logits means are taken over every position and the
    whole vocabulary, computed as `hidden . sum_v W[v]` (no logits)."""

    LOSS_TYPES = ("sigmoid", "apo_zero", "apo_down", "sppo_hard", "nca_pair")

    def __init__(self, ignore_index: int = -100, beta: float = 0.1, loss_type: str = "sigmoid", use_ref_model: bool = True,
                 chunk_size: int = 32768):
        super().__init__()
        if loss_type not in self.LOSS_TYPES:
            raise NotImplementedError(f"loss_type={loss_type!r}: the fused-linear DPO loss has {self.LOSS_TYPES}")
        self.loss_type = loss_type
        self.ignore_index = int(ignore_index)
        self.beta = float(beta)
        self.use_ref_model = bool(use_ref_model)
        self.chunk_size = int(chunk_size)

    def forward(self, lin_weight: Tensor, _input: Tensor, target: Tensor, bias: Tensor | None = None,
                ref_input: Tensor | None = None, ref_weight: Tensor | None = None, ref_bias: Tensor | None = None):
        if _input.dim() != 3 or _input.shape[0] % 2:
            raise ValueError("_input must be [2P, T, H]: chosen sequences first, rejected second")
        pairs = _input.shape[0] // 2
        keep = target != self.ignore_index
        labels = torch.where(keep, target, torch.zeros_like(target))
        logps = _head_logps(_input, lin_weight, labels, keep, 1.0, self.chunk_size, bias)
        if self.use_ref_model:
            if ref_input is None:
                raise ValueError("ref_input is required when use_ref_model=True")
            with torch.no_grad():
                ref_logps = _head_logps(ref_input, lin_weight if ref_weight is None else ref_weight, labels, keep, 1.0,
                                        self.chunk_size, bias if ref_weight is None else ref_bias)
                ref_seq = (ref_logps * keep).sum(-1)
        else:
            ref_seq = torch.zeros(2 * pairs, dtype=torch.float32, device=_input.device)
        if self.loss_type == "sigmoid":
            loss, seq, _, _ = ops.dpo_loss_op(logps, keep, ref_seq[:pairs], ref_seq[pairs:], self.beta)
        else:  # [P]-sized fp32 arithmetic on the sequence log-ratios
            seq = (logps * keep).sum(-1)
            c_lr, r_lr = seq[:pairs] - ref_seq[:pairs], seq[pairs:] - ref_seq[pairs:]
            b = self.beta
            if self.loss_type == "apo_zero":
                per_pair = 1 - torch.sigmoid(b * c_lr) + torch.sigmoid(b * r_lr)
            elif self.loss_type == "apo_down":
                per_pair = torch.sigmoid(b * c_lr) + 1 - torch.sigmoid(b * (c_lr - r_lr))
            elif self.loss_type == "sppo_hard":
                per_pair = (c_lr - 0.5 / b) ** 2 + (r_lr + 0.5 / b) ** 2
            else:  # nca_pair
                per_pair = (-F.logsigmoid(b * c_lr) - 0.5 * F.logsigmoid(-b * c_lr) - 0.5 * F.logsigmoid(-b * r_lr))
            loss = per_pair.mean()
        with torch.no_grad():
            seq = seq.detach()
            wsum = lin_weight.float().sum(0)
            logits_mean = (_input.float() @ wsum).mean(dim=1) / lin_weight.shape[0]  # [2P], over T and V
            if bias is not None:
                logits_mean = logits_mean + bias.float().mean()
            rewards = self.beta * (seq - ref_seq)
            nll = torch.zeros((), dtype=torch.float32, device=_input.device)
        metrics = (seq[:pairs], seq[pairs:], logits_mean[:pairs].mean(), logits_mean[pairs:].mean(), nll,
                   rewards[:pairs], rewards[pairs:])
        return loss, metrics


class FusedLinearKTOLoss(torch.nn.Module):
    """`loss, sums = op(_input [B, T, H], lin_weight [V, H], target [B, T] (-100 = ignored), bias=None,
    preference_labels [B] (true = desirable), ref_input=None, ref_weight=None, ref_bias=None, kl=None)` with
    `sums = (chosen_logps_sum, rejected_logps_sum, chosen_logits_sum, rejected_logits_sum, chosen_rewards_sum,
    rejected_rewards_sum)`, the order `_compute_loss_liger` unpacks (kto_trainer.py:1415-1424); the caller divides
    each by the number of desirable / undesirable examples.  The loss is the reference's `kto` loss with unit
    class weights (kto_trainer.py:1558-1560, 1576-1577, 1586-1589, 1655); a sequence's "logits" entry is its mean
    logit over positions and vocabulary."""

    def __init__(self, ignore_index: int = -100, beta: float = 0.1, use_ref_model: bool = True, chunk_size: int = 32768):
        super().__init__()
        self.ignore_index = int(ignore_index)
        self.beta = float(beta)
        self.use_ref_model = bool(use_ref_model)
        self.chunk_size = int(chunk_size)

    def forward(self, _input: Tensor, lin_weight: Tensor, target: Tensor, bias: Tensor | None = None,
                preference_labels: Tensor | None = None, ref_input: Tensor | None = None,
                ref_weight: Tensor | None = None, ref_bias: Tensor | None = None, kl: Tensor | None = None):
        if _input.dim() != 3:
            raise ValueError("_input must be [B, T, H] hidden states")
        if preference_labels is None or len(preference_labels) != _input.shape[0]:
            raise ValueError("preference_labels must hold one entry per sequence")
        dev = _input.device
        keep = target != self.ignore_index
        labels = torch.where(keep, target, torch.zeros_like(target))
        seq = (_head_logps(_input, lin_weight, labels, keep, 1.0, self.chunk_size, bias) * keep).sum(-1)
        if self.use_ref_model:
            if ref_input is None:
                raise ValueError("ref_input is required when use_ref_model=True")
            with torch.no_grad():
                ref_seq = (_head_logps(ref_input, lin_weight if ref_weight is None else ref_weight, labels, keep, 1.0,
                                       self.chunk_size, bias if ref_weight is None else ref_bias) * keep).sum(-1)
        else:
            ref_seq = torch.zeros_like(seq)
        chosen = torch.as_tensor(preference_labels, dtype=torch.bool, device=dev)
        kl_term = torch.zeros((), device=dev) if kl is None else kl.to(dev).float().reshape(-1)[0].detach()
        lr = seq - ref_seq
        per_example = torch.where(chosen, 1 - torch.sigmoid(self.beta * (lr - kl_term)),
                                  1 - torch.sigmoid(self.beta * (kl_term - lr)))
        loss = per_example.mean()
        with torch.no_grad():
            c = chosen.to(torch.float32)
            wsum = lin_weight.float().sum(0)
            logits_mean = (_input.float() @ wsum).mean(dim=1) / lin_weight.shape[0]
            if bias is not None:
                logits_mean = logits_mean + bias.float().mean()
            rewards = self.beta * lr.detach()
            s = seq.detach()
            sums = ((s * c).sum(), (s * (1 - c)).sum(), (logits_mean * c).sum(), (logits_mean * (1 - c)).sum(),
                    (rewards * c).sum(), (rewards * (1 - c)).sum())
        return loss, sums

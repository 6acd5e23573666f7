"""Sequence-level clipped loss of the reference's `RLOOTrainer._compute_loss`
(trl/trainer/rloo_trainer.py:1683-1694, 1711-1721) and its leave-one-out advantages (:1537-1561)."""
from __future__ import annotations

import torch
from torch import Tensor

from .. import ops
from .utils import nanstd

__all__ = ["rloo_loss", "rloo_advantages", "RLOO_METRIC_NAMES"]

RLOO_METRIC_NAMES = ("clip_ratio/low_mean", "clip_ratio/low_min", "clip_ratio/high_mean", "clip_ratio/high_max",
                     "clip_ratio/region_mean")


def rloo_loss(per_token_logps: Tensor, completion_mask: Tensor, old_logps: Tensor, advantages: Tensor,
              epsilon_low: float, epsilon_high: float):
    """Returns `(loss, sequence_logps [B], metrics [8])`; metric order = `RLOO_METRIC_NAMES`."""
    loss, seq, metrics, _ = ops.rloo_loss_op(per_token_logps, completion_mask, old_logps, advantages,
                                             float(epsilon_low), float(epsilon_high))
    return loss, seq, metrics


def rloo_advantages(rewards: Tensor, num_generations: int, normalize_advantages: bool = False) -> Tensor:
    """Leave-one-out baseline over scorable siblings; O(B) torch ops as in the reference."""
    grouped = rewards.view(-1, num_generations)
    if num_generations > 1:
        n = (~torch.isnan(grouped)).sum(dim=1, keepdim=True)
        total = torch.nansum(grouped, dim=1, keepdim=True)
        adv = rewards - ((total - grouped) / (n - 1)).view(-1)
    else:
        adv = torch.zeros_like(rewards)
    if normalize_advantages:
        adv = (adv - torch.nanmean(adv)) / (nanstd(adv) + 1e-4)
    return torch.nan_to_num(adv, nan=0.0)

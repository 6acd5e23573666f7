"""Sequence log-prob reduction and sigmoid loss of the reference's `DPOTrainer._compute_loss`
(trl/trainer/dpo_trainer.py:1329-1435, 1578, 1634-1653) on the HIP kernels."""
from __future__ import annotations

import torch
from torch import Tensor

from .. import ops
from .utils import logps_and_entropies

__all__ = ["dpo_per_token_logps", "dpo_sigmoid_loss", "dpo_loss_from_logits", "DPO_METRIC_NAMES"]

DPO_METRIC_NAMES = ("rewards/chosen", "rewards/rejected", "rewards/accuracies", "rewards/margins", "logps/chosen",
                    "logps/rejected")


def dpo_per_token_logps(logits: Tensor, input_ids: Tensor, compute_entropy: bool = False):
    """Shifted per-token log-probs: `logits[:, :-1]` scored against `input_ids[:, 1:]`
    (dpo_trainer.py:1344-1347) in fp32, `[B, L-1]`; the gradient is written for all `L` rows.
    With `compute_entropy` also returns the (detached) entropies the reference logs (:1587)."""
    length = logits.shape[1]
    logp, ent = logps_and_entropies(logits, input_ids[:, 1:], 1.0, 0, length - 1)
    return (logp, ent.detach()) if compute_entropy else logp


def dpo_sigmoid_loss(token_logps: Tensor, shift_completion_mask: Tensor, ref_chosen_logps: Tensor,
                     ref_rejected_logps: Tensor, beta: float):
    """Masked sum over the sequence (dpo_trainer.py:1348-1350), `[chosen; rejected]` split (:1362),
    `mean(-logsigmoid(beta * ((pi_c - ref_c) - (pi_r - ref_r))))` (:1397-1402, 1435, 1578).
    Returns `(loss, sequence_logps [B], metrics [8])`; metric order = `DPO_METRIC_NAMES`."""
    loss, seq, metrics, _ = ops.dpo_loss_op(token_logps, shift_completion_mask, ref_chosen_logps, ref_rejected_logps,
                                            float(beta))
    return loss, seq, metrics


def dpo_loss_from_logits(logits: Tensor, input_ids: Tensor, completion_mask: Tensor, ref_chosen_logps: Tensor,
                         ref_rejected_logps: Tensor, beta: float = 0.1, compute_entropy: bool = False):
    """The arithmetic of `DPOTrainer._compute_loss` after the model call, for `loss_type="sigmoid"`
    with precomputed reference log-probs.  Returns `(loss, metrics_dict_of_device_scalars)`."""
    out = dpo_per_token_logps(logits, input_ids, compute_entropy)
    token_logps, ent = out if compute_entropy else (out, None)
    shift_mask = completion_mask[:, 1:]
    loss, seq, metrics = dpo_sigmoid_loss(token_logps, shift_mask, ref_chosen_logps, ref_rejected_logps, beta)
    named = {name: metrics[i] for i, name in enumerate(DPO_METRIC_NAMES)}
    if ent is not None:
        m = shift_mask.float()
        named["entropy"] = (ent * m).sum() / m.sum().clamp(min=1.0)
    named["sequence_logps"] = seq
    return loss, named

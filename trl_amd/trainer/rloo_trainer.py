"""Sequence-level clipped loss of the reference's `RLOOTrainer._compute_loss`
(trl/trainer/rloo_trainer.py:1683-1694, 1711-1721) and its leave-one-out advantages (:1537-1561)."""
from __future__ import annotations

import torch
from torch import Tensor

from .. import ops
from .utils import nanstd

__all__ = ["rloo_loss", "rloo_advantages", "RLOO_METRIC_NAMES", "RLOOLossMixin"]

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


class RLOOLossMixin:
    """`_get_per_token_logps_and_entropies` / `_compute_loss` with the reference's names and signatures
    (trl/trainer/rloo_trainer.py:882-982, 1655-1722); bind them onto an `RLOOTrainer`."""

    # the log-prob pass is the GRPO one (rloo_trainer.py:882-982 is a copy of grpo_trainer.py:1435-1541)
    from .grpo_trainer import GRPOLossMixin as _G

    _get_per_token_logps_and_entropies = _G._get_per_token_logps_and_entropies
    _model_inputs = _G._model_inputs
    del _G

    def _compute_loss(self, model, inputs):
        prompt_ids, prompt_mask = inputs["prompt_ids"], inputs["prompt_mask"]
        completion_ids, completion_mask = inputs["completion_ids"], inputs["completion_mask"]
        input_ids = torch.cat([prompt_ids, completion_ids], dim=1)
        attention_mask = torch.cat([prompt_mask, completion_mask], dim=1)
        logits_to_keep = completion_ids.size(1)
        aux_enabled = bool(getattr(self, "aux_loss_enabled", False))
        extra_keys = ("pixel_values", "image_grid_thw", "num_images", "pixel_attention_mask", "spatial_shapes",
                      "num_tiles", "image_sizes", "token_type_ids", "mm_token_type_ids", "image_position_ids")
        # log-probs and entropies only enter through `* completion_mask`: masked rows need not be computed
        skip = completion_mask if getattr(self, "trl_amd_skip_masked_rows", True) else None
        per_token_logps, entropies, aux_loss = self._get_per_token_logps_and_entropies(
            model, input_ids, attention_mask, logits_to_keep, compute_entropy=True, compute_aux_loss=aux_enabled,
            skip_rows_mask=skip, **{k: inputs.get(k) for k in extra_keys})
        loss, _, metrics = rloo_loss(per_token_logps, completion_mask, inputs["old_logps"], inputs["advantages"],
                                     self.epsilon_low, self.epsilon_high)
        mode = "train" if self.model.training else "eval"
        log = self._metrics[mode]
        if aux_enabled:
            loss = loss + self.router_aux_loss_coef * aux_loss
            log["aux_loss"].append(self.accelerator.gather_for_metrics(aux_loss).mean().item())
        m = completion_mask.to(torch.float32)
        ent = self.accelerator.reduce(torch.stack([(entropies.detach() * m).sum(), m.sum()]), reduction="sum")
        single = self.accelerator.num_processes == 1
        # (one copy to the host: the entropy, the error word and, on one process, the loss kernel's metrics)
        ent_ratio, bits, *values = torch.cat(
            [(ent[0] / ent[1].clamp(min=1.0)).reshape(1), ops.device_error_bits(ent.device).to(torch.float32)]
            + ([metrics.detach()[: len(RLOO_METRIC_NAMES)].to(torch.float32)] if single else [])).tolist()
        ops.raise_for_error_bits(bits, ent.device)  # (a token id outside the vocabulary raises here)
        log["entropy"].append(ent_ratio)
        if single:
            for name, value in zip(RLOO_METRIC_NAMES, values):
                log[name].append(value)
        else:  # per-sequence flags are gathered as in the reference (:1711-1721)
            from .utils import nanmax, nanmin

            with torch.no_grad():
                seq = (per_token_logps.detach() * m).sum(1)
                c = torch.exp(seq - inputs["old_logps"])
                adv = inputs["advantages"]
                low = ((c < 1 - self.epsilon_low) & (adv < 0)).float()
                high = ((c > 1 + self.epsilon_high) & (adv > 0)).float()
                g_low, g_high = self.accelerator.gather(low), self.accelerator.gather(high)
                g_reg = self.accelerator.gather(torch.maximum(low, high))
            log["clip_ratio/low_mean"].append(g_low.nanmean().item())
            log["clip_ratio/low_min"].append(nanmin(g_low).item())
            log["clip_ratio/high_mean"].append(g_high.nanmean().item())
            log["clip_ratio/high_max"].append(nanmax(g_high).item())
            log["clip_ratio/region_mean"].append(g_reg.nanmean().item())
        return loss

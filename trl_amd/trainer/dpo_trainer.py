"""The reference's `DPOTrainer._compute_loss` (trl/trainer/dpo_trainer.py:1329-1655) on the HIP kernels:
the fused sigmoid path (`dpo_sigmoid_loss`, one loss kernel) and the general one (`dpo_compute_loss`: all
loss types, `ld_alpha`, WPO weighting, f-divergences, every logged metric from one pass over the logits)."""
from __future__ import annotations

from contextlib import contextmanager

import torch
import torch.nn.functional as F
from torch import Tensor

from .. import ops
from .utils import logps_and_entropies

__all__ = ["dpo_per_token_logps", "dpo_sigmoid_loss", "dpo_loss_from_logits", "DPO_METRIC_NAMES", "dpo_compute_loss",
           "dpo_metrics_to_dict", "dpo_sequence_logps", "DPOLossMixin"]

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


# ----------------------------------------------------------------------------------------------
# the whole of `DPOTrainer._compute_loss` after the model call
# ----------------------------------------------------------------------------------------------
def _f_divergence_scores(chosen_lr: Tensor, rejected_lr: Tensor, kind: str, alpha: float):
    """Scores of the log-ratios under the configured f-divergence (dpo_trainer.py:1402-1429)."""
    if kind == "reverse_kl" or (kind == "alpha_divergence" and abs(alpha - 1.0) < 1e-6):
        return chosen_lr, rejected_lr
    if kind == "forward_kl":
        return -torch.exp(-chosen_lr), -torch.exp(-rejected_lr)
    if kind == "js_divergence":
        return F.logsigmoid(chosen_lr), F.logsigmoid(rejected_lr)
    if kind == "alpha_divergence":
        k = alpha - 1.0
        return tuple(torch.exp(torch.clamp(k * lr, max=80.0)) / k for lr in (chosen_lr, rejected_lr))
    raise ValueError(f"Unknown f_divergence_type: {kind}")


def dpo_compute_loss(
    logits: Tensor, input_ids: Tensor, completion_mask: Tensor, ref_chosen_logps: Tensor, ref_rejected_logps: Tensor,
    beta: float = 0.1, loss_types=("sigmoid",), loss_weights=None, label_smoothing: float = 0.0,
    ld_alpha: float | None = None, use_weighting: bool = False, f_divergence_type: str = "reverse_kl",
    f_alpha_divergence_coef: float = 1.0, discopop_tau: float = 0.05, skip_masked_rows: bool = True,
):
    """Loss and metrics of `DPOTrainer._compute_loss` (dpo_trainer.py:1342-1653) from `[2P, L, V]` logits with
    given reference log-probs: every loss type, `ld_alpha`, WPO weighting, f-divergences.

    ONE pass over the logits yields the per-token log-probs, the entropies, and the row statistics behind the
    WPO weights (`log sum_v p_v^2`), the logits means and the token accuracy (the reference makes five more
    passes for those); everything after that is `[2P, L]`- or `[P]`-sized torch arithmetic in fp32.  Rows outside
    the completion mask contribute to nothing and are not read unless `skip_masked_rows=False`.
    Returns `(loss, metrics)`, `metrics` a dict of device scalars keyed like the reference's log."""
    if logits.dim() != 3 or logits.shape[0] % 2:
        raise ValueError("logits must be [2P, L, V]: chosen sequences first, rejected second")
    n_seq, length, _ = logits.shape
    labels = input_ids[:, 1:]
    smask = completion_mask[:, 1:]
    idx = labels.reshape(n_seq * (length - 1), 1)
    if idx.dtype != torch.int64:
        idx = idx.long()
    rm = (smask.reshape(-1) != 0).to(torch.uint8).contiguous() if skip_masked_rows else None
    # (the sum of squared probabilities is wanted by the WPO weights only)
    logp, ent, _, stats = ops.logp_entropy_stats_fwd(logits, idx, 1.0, 0, length - 1, rm, bool(use_weighting))
    m = smask.to(torch.float32)
    ent = ent.view(n_seq, length - 1).detach()
    stats = stats.view(n_seq, length - 1, 4).detach()
    ref_c, ref_r = ref_chosen_logps.to(torch.float32), ref_rejected_logps.to(torch.float32)
    ls = float(label_smoothing)
    if (tuple(loss_types) == ("sigmoid",) and ls == 0.0 and ld_alpha is None and not use_weighting
            and f_divergence_type == "reverse_kl" and (loss_weights is None or [float(x) for x in loss_weights] == [1.0])):
        # the default configuration: masked sequence sums, loss and d loss / d log-prob from one loss kernel
        loss, seq, _, _ = ops.dpo_loss_op(logp.view(n_seq, length - 1), m, ref_c, ref_r, float(beta))
        chosen, rejected = seq.detach().chunk(2)
        return loss, _dpo_metric_parts(ent, stats, m, chosen, rejected, ref_c, ref_r, beta)
    tok = logp.view(n_seq, length - 1) * m

    if ld_alpha is None:
        seq = _masked_row_sums(logp.view(n_seq, length - 1), m)
    else:  # tokens beyond the shorter completion of a pair count with weight ld_alpha (:1351-1361)
        pos = smask.cumsum(dim=1)
        lens = smask.sum(dim=1)
        shared = torch.minimum(*lens.chunk(2)).repeat(2).unsqueeze(1)
        head = ((pos > 0) & (pos <= shared)).to(torch.float32)
        tail = (pos > shared).to(torch.float32)
        seq = (tok * head).sum(dim=1) + ld_alpha * (tok * tail).sum(dim=1)
    chosen, rejected = seq.chunk(2)
    c_lr, r_lr = chosen - ref_c, rejected - ref_r
    c_sc, r_sc = _f_divergence_scores(c_lr, r_lr, f_divergence_type, f_alpha_divergence_coef)
    d = c_sc - r_sc
    c_n, r_n = (x.to(torch.float32).sum(dim=1).clamp(min=1.0) for x in completion_mask.chunk(2))

    def smoothed(delta):
        return -F.logsigmoid(beta * delta) * (1 - ls) - F.logsigmoid(-beta * delta) * ls

    def exo_pair():
        eps = torch.tensor(ls, device=d.device)
        qw, ql = torch.sigmoid(beta * d), torch.sigmoid(-beta * d)
        return qw * (F.logsigmoid(beta * d) - torch.log1p(-eps)) + ql * (F.logsigmoid(-beta * d) - torch.log(eps))

    def discopop():
        x = beta * d
        mix = torch.sigmoid(x / discopop_tau)
        return -F.logsigmoid(x) * (1 - mix) + torch.exp(-x) * mix

    def sft():  # cross-entropy of the chosen completion tokens = -mean of their log-probs
        cm = m.chunk(2)[0]
        return (-(tok.chunk(2)[0]).sum() / cm.sum()).expand(chosen.shape[0])

    per_pair = {
        "sigmoid": lambda: -F.logsigmoid(beta * d),
        "hinge": lambda: torch.relu(1 - beta * d),
        "ipo": lambda: ((c_sc / c_n - r_sc / r_n) - 1 / (2 * beta)) ** 2,
        "exo_pair": exo_pair,
        "nca_pair": lambda: -F.logsigmoid(beta * c_sc) - 0.5 * F.logsigmoid(-beta * c_sc) - 0.5 * F.logsigmoid(-beta * r_sc),
        "robust": lambda: (-(1 - ls) * F.logsigmoid(beta * d) + ls * F.logsigmoid(-beta * d)) / (1 - 2 * ls),
        "bco_pair": lambda: -F.logsigmoid(beta * c_sc) - F.logsigmoid(-beta * r_sc),
        "sppo_hard": lambda: (c_sc - 0.5 / beta) ** 2 + (r_sc + 0.5 / beta) ** 2,
        "aot": lambda: smoothed(torch.sort(chosen - rejected, dim=0)[0] - torch.sort(ref_c - ref_r, dim=0)[0]),
        "aot_unpaired": lambda: smoothed(torch.sort(c_lr, dim=0)[0] - torch.sort(r_lr, dim=0)[0]),
        "apo_zero": lambda: 1 - torch.sigmoid(beta * c_lr) + torch.sigmoid(beta * r_lr),
        "apo_down": lambda: torch.sigmoid(beta * c_lr) + 1 - torch.sigmoid(beta * d),
        "discopop": discopop,
        "sft": sft,
        "sigmoid_norm": lambda: -F.logsigmoid(beta * (c_sc / c_n - r_sc / r_n)),
    }
    pair_weight = None
    if use_weighting:  # WPO (:1563-1574): exp(mean over the completion of logp - log sum_v p_v^2), product over the pair
        aligned = (tok.detach() - stats[..., 1] * m).sum(dim=1) / m.sum(dim=1).clamp_min(1.0)
        w = torch.exp(aligned)
        pair_weight = w.chunk(2)[0] * w.chunk(2)[1]
    loss_weights = [1.0] * len(loss_types) if loss_weights is None else loss_weights
    loss = 0.0
    for name, lw in zip(loss_types, loss_weights, strict=True):
        if name not in per_pair:
            raise ValueError(
                f"Unknown loss type: {name}. Should be one of ['sigmoid', 'hinge', 'ipo', 'exo_pair', 'nca_pair', "
                "'robust', 'bco_pair', 'sppo_hard', 'aot', 'aot_unpaired', 'apo_zero', 'apo_down', 'discopop', 'sft', "
                "'sigmoid_norm']")
        term = per_pair[name]()
        if pair_weight is not None:
            term = term * pair_weight
        loss = loss + term.mean() * lw

    return loss, _dpo_metric_parts(ent, stats, m, chosen.detach(), rejected.detach(), ref_c, ref_r, beta)


def _masked_row_sums(token_logps: Tensor, mask: Tensor) -> Tensor:
    """`[2P]` sums of the log-probs inside the mask, from the loss kernel's own row reduction (differentiable).  Every
    place that sums a sequence uses this one order of summation: reference log-probs taken from the same logits then
    cancel the policy's exactly, and the first step of a run starts at ln 2 as it does in the reference."""
    if token_logps.shape[0] % 2:  # not a batch of pairs (a caller summing sequences on their own): plain torch
        return (token_logps.float() * (mask != 0)).sum(dim=1)
    zero = token_logps.new_zeros((token_logps.shape[0] // 2,), dtype=torch.float32)
    return ops.dpo_loss_op(token_logps, mask, zero, zero, 1.0)[1]


@torch.no_grad()
def _dpo_metric_parts(ent, stats, m, chosen, rejected, ref_c, ref_r, beta):
    """The parts of the logged metrics (dpo_trainer.py:1587-1653) as device scalars / `[P]` vectors: masked sums of
    the entropies, the mean logits and the arg-max hits per half of the batch, from one stacked reduction."""
    n_seq = m.shape[0]
    vals = torch.stack((ent, stats[..., 0], stats[..., 2], torch.ones_like(ent)), dim=0)  # [4, 2P, L-1]
    halves = (vals * m).view(4, 2, (n_seq // 2) * m.shape[1]).sum(dim=2)  # [quantity, chosen | rejected]
    both = halves.sum(dim=1)
    return {
        "entropy_sum": both[0], "n_tokens": both[3],
        "logits_chosen_sum": halves[1, 0], "n_chosen_tokens": halves[3, 0],
        "logits_rejected_sum": halves[1, 1], "n_rejected_tokens": halves[3, 1],
        "correct_tokens": halves[2, 0],
        "chosen_rewards": beta * (chosen - ref_c), "rejected_rewards": beta * (rejected - ref_r),
        "chosen_logps": chosen, "rejected_logps": rejected,
    }


def dpo_metrics_to_dict(metrics: dict) -> dict[str, float]:
    """Single-process reduction of `dpo_compute_loss`'s metric parts to the reference's logged values."""
    def ratio(a, b):
        b = float(metrics[b])
        return float(metrics[a]) / b if b > 0 else 0.0

    c, r = metrics["chosen_rewards"], metrics["rejected_rewards"]
    return {
        "entropy": ratio("entropy_sum", "n_tokens"),
        "logits/chosen": ratio("logits_chosen_sum", "n_chosen_tokens"),
        "logits/rejected": ratio("logits_rejected_sum", "n_rejected_tokens"),
        "mean_token_accuracy": ratio("correct_tokens", "n_chosen_tokens"),
        "rewards/chosen": float(c.mean()), "rewards/rejected": float(r.mean()),
        "rewards/accuracies": float((c > r).float().mean()), "rewards/margins": float((c - r).mean()),
        "logps/chosen": float(metrics["chosen_logps"].mean()), "logps/rejected": float(metrics["rejected_logps"].mean()),
    }


@contextmanager
def _reference_adapter(peft_model):
    """Puts a PEFT model into its reference state for the block (trl/trainer/utils.py:1199-1236 as used at
    dpo_trainer.py:1187-1195, 1373-1380): the adapter named "ref" if there is one, otherwise no adapter at all;
    the previous state comes back afterwards."""
    if "ref" in peft_model.peft_config:
        previous = peft_model.active_adapter
        peft_model.set_adapter("ref")
        try:
            yield
        finally:
            peft_model.set_adapter(previous)
    else:
        with peft_model.disable_adapter():
            yield


class DPOLossMixin:
    """`_compute_loss` with the reference's name and signature; bind it onto a `DPOTrainer`."""

    def _compute_loss(self, model, inputs, return_outputs):
        """Reference: trl/trainer/dpo_trainer.py:1329-1655.  The policy forward is the model's own; the log-prob,
        loss and metric arithmetic runs on the kernels.  Without precomputed reference log-probs the reference
        model is run under `no_grad`, or the policy itself with its PEFT adapters switched to the reference."""
        mode = "train" if self.model.training else "eval"
        skip = {"completion_mask", "ref_chosen_logps", "ref_rejected_logps"}
        model_kwargs = {k: v for k, v in inputs.items() if k not in skip}
        model_kwargs["use_cache"] = False
        aux_enabled = bool(getattr(self, "aux_loss_enabled", False))
        if aux_enabled:
            model_kwargs["output_router_logits"] = True
        outputs = model(**model_kwargs)
        input_ids, completion_mask = inputs["input_ids"], inputs["completion_mask"]
        cfg = dict(
            ld_alpha=self.ld_alpha, f_divergence_type=self.f_divergence_type,
            f_alpha_divergence_coef=getattr(self, "f_alpha_divergence_coef", 1.0))
        if self.precompute_ref_logps:
            ref_c, ref_r = inputs["ref_chosen_logps"], inputs["ref_rejected_logps"]
        else:
            with torch.no_grad():
                ref_kwargs = {k: v for k, v in model_kwargs.items() if k != "output_router_logits"}
                if getattr(self, "ref_model", None) is not None:
                    ref_logits = self.ref_model(**ref_kwargs).logits
                else:
                    # adapter training without a separate reference model: the reference is the same network with
                    # its adapters switched off, or with the frozen copy named "ref" active (dpo_trainer.py:1373-1380)
                    peft_model = self.accelerator.unwrap_model(model)
                    if not hasattr(peft_model, "peft_config"):
                        raise ValueError("DPO needs reference log-probs: precomputed, from `ref_model`, or from a PEFT "
                                         "model whose adapters can be switched off")
                    with _reference_adapter(peft_model):
                        ref_logits = self.model(**ref_kwargs).logits
                ref_seq = dpo_sequence_logps(ref_logits, input_ids, completion_mask, self.ld_alpha)
            ref_c, ref_r = ref_seq.chunk(2)
        loss, parts = dpo_compute_loss(
            outputs.logits, input_ids, completion_mask, ref_c, ref_r, beta=self.beta, loss_types=self.loss_types,
            loss_weights=self.loss_weights, label_smoothing=self.label_smoothing, use_weighting=self.use_weighting,
            discopop_tau=getattr(getattr(self, "args", None), "discopop_tau", 0.05), **cfg)
        log = self._metrics[mode]
        if aux_enabled:
            loss = loss + self.router_aux_loss_coef * outputs.aux_loss
            log["aux_loss"].append(self.accelerator.gather_for_metrics(outputs.aux_loss).mean().item())
        acc = self.accelerator
        counts = torch.stack([parts[k] for k in ("entropy_sum", "n_tokens", "logits_chosen_sum", "n_chosen_tokens",
                                                  "logits_rejected_sum", "n_rejected_tokens", "correct_tokens")])
        bits = ops.device_error_bits(counts.device)  # (a token id outside the vocabulary raises here)
        c_rew, r_rew = acc.gather(parts["chosen_rewards"]), acc.gather(parts["rejected_rewards"])
        means = torch.stack([c_rew.mean(), r_rew.mean(), (c_rew > r_rew).float().mean(), (c_rew - r_rew).mean(),
                             acc.gather(parts["chosen_logps"]).mean(), acc.gather(parts["rejected_logps"]).mean()])
        n_train = (acc.gather_for_metrics(inputs["attention_mask"].sum()).sum().reshape(1) if mode == "train"
                   else counts.new_zeros(1))
        # every logged number in ONE copy to the host (each `.item()` would make the host wait for the device again)
        (ent_sum, n_tok, lc, nc, lr, nr, correct, bits, rew_c, rew_r, rew_acc, rew_margin, logp_c, logp_r,
         n_train) = torch.cat([acc.gather_for_metrics(counts.unsqueeze(0)).sum(dim=0).double(), bits.double(),
                               means.double(), n_train.double()]).tolist()
        ops.raise_for_error_bits(bits, counts.device)
        log["entropy"].append(ent_sum / n_tok if n_tok > 0 else 0.0)
        if mode == "train":
            self._total_train_tokens += int(n_train)
        log["num_tokens"] = [self._total_train_tokens]
        log["logits/chosen"].append(lc / nc if nc > 0 else 0.0)
        log["logits/rejected"].append(lr / nr if nr > 0 else 0.0)
        log["mean_token_accuracy"].append(correct / nc if nc > 0 else 0.0)
        log["rewards/chosen"].append(rew_c)
        log["rewards/rejected"].append(rew_r)
        log["rewards/accuracies"].append(rew_acc)
        log["rewards/margins"].append(rew_margin)
        log["logps/chosen"].append(logp_c)
        log["logps/rejected"].append(logp_r)
        return (loss, outputs) if return_outputs else loss


def dpo_sequence_logps(logits: Tensor, input_ids: Tensor, completion_mask: Tensor, ld_alpha: float | None = None):
    """Detached `[2P]` sequence log-probs as `compute_ref_log_probs` / the in-loss reference pass take them
    (dpo_trainer.py:1196-1219, 1381-1394): masked sum of the shifted per-token log-probs, with the `ld_alpha`
    split when set.  Rows outside the completion mask are not read."""
    n_seq, length, _ = logits.shape
    smask = completion_mask[:, 1:]
    rm = (smask.reshape(-1) != 0).to(torch.uint8).contiguous()
    with torch.no_grad():
        logp, _ = logps_and_entropies(logits, input_ids[:, 1:], 1.0, 0, length - 1, rm.view(n_seq, length - 1))
        if ld_alpha is None:
            return _masked_row_sums(logp, smask.to(torch.float32))
        tok = logp * smask
        pos = smask.cumsum(dim=1)
        shared = torch.minimum(*smask.sum(dim=1).chunk(2)).repeat(2).unsqueeze(1)
        return (tok * ((pos > 0) & (pos <= shared))).sum(dim=1) + ld_alpha * (tok * (pos > shared)).sum(dim=1)

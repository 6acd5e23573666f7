"""KTO loss of the reference's `KTOTrainer._compute_loss` (trl/trainer/kto_trainer.py:1478-1663): sequence
log-probs of unpaired completions, the KL baseline from mismatched prompt/completion pairs, the `kto` and
`apo_zero_unpaired` losses and every logged metric."""
from __future__ import annotations

import torch
from torch import Tensor

from .. import ops
from .dpo_trainer import _reference_adapter

__all__ = ["kto_sequence_logps", "kto_compute_loss", "KTOLossMixin"]

LOSS_TYPES = ("kto", "apo_zero_unpaired")


def _shifted_logps(logits: Tensor, input_ids: Tensor, completion_mask: Tensor, skip_masked_rows: bool, stats: bool):
    n_seq, length, _ = logits.shape
    smask = completion_mask[:, 1:]
    idx = input_ids[:, 1:].reshape(n_seq * (length - 1), 1)
    if idx.dtype != torch.int64:
        idx = idx.long()
    rm = (smask.reshape(-1) != 0).to(torch.uint8).contiguous() if skip_masked_rows else None
    if stats:
        logp, ent, _, st = ops.logp_entropy_stats_fwd(logits, idx, 1.0, 0, length - 1, rm, False)
        st = st.view(n_seq, length - 1, 4).detach()
        ent = ent.view(n_seq, length - 1).detach()
    else:
        logp, ent, _ = ops.logp_entropy_fwd(logits, idx, 1.0, 0, length - 1, rm)
        st = None
    m = smask.to(torch.float32)
    return logp.view(n_seq, length - 1) * m, ent, st, m


def kto_sequence_logps(logits: Tensor, input_ids: Tensor, completion_mask: Tensor, skip_masked_rows: bool = True) -> Tensor:
    """Detached `[B]` masked sums of the shifted per-token log-probs: the KL-estimate and reference passes
    (kto_trainer.py:1265-1276, 1323-1327, 1542-1545)."""
    with torch.no_grad():
        tok, _, _, _ = _shifted_logps(logits, input_ids, completion_mask, skip_masked_rows, False)
        return tok.sum(dim=1)


def kto_compute_loss(
    logits: Tensor, input_ids: Tensor, completion_mask: Tensor, label: Tensor, ref_logps: Tensor,
    kl_logps: Tensor | None = None, ref_kl_logps: Tensor | None = None, beta: float = 0.1, loss_type: str = "kto",
    desirable_weight: float = 1.0, undesirable_weight: float = 1.0, skip_masked_rows: bool = True, kl_reduce=None,
):
    """Loss and metric parts of kto_trainer.py:1506-1663 from `[B, L, V]` logits; `label[b]` true = desirable.

    ONE pass over the logits gives the per-token log-probs, the entropies and the mean logit of every completion
    row (the reference makes three); the rest is `[B]`-sized fp32 torch arithmetic.  `kl_logps`/`ref_kl_logps`
    (`[B]`, detached) give the batch KL estimate `mean(kl_logps - ref_kl_logps)`, reduced across processes by
    `kl_reduce` (a callable on the 0-d tensor; identity when None) and clamped at 0; without them KL = 0.
    Returns `(loss, metrics)`, `metrics` a dict of device tensors."""
    if loss_type not in LOSS_TYPES:
        raise ValueError(f"Unknown loss type: {loss_type}. Should be one of {list(LOSS_TYPES)}")
    if logits.dim() != 3:
        raise ValueError("logits must be [B, L, V]")
    if logits.shape[0] != len(label):
        raise ValueError("There is a mismatch between the number of examples in this batch and the number of "
                         "examples for which an output sequence was predicted.")
    tok, ent, stats, m = _shifted_logps(logits, input_ids, completion_mask, skip_masked_rows, True)
    seq = tok.sum(dim=1)
    dev = logits.device
    is_chosen = torch.as_tensor(label, dtype=torch.bool, device=dev)
    # (desirable and undesirable examples are told apart by masks, not gathered by index: `nonzero` would make the
    # host wait for the pass over the logits that was just launched)
    lr = seq - ref_logps.to(torch.float32)
    if kl_logps is not None:
        kl = (kl_logps.float() - ref_kl_logps.float()).mean().detach()
        kl = (kl if kl_reduce is None else kl_reduce(kl)).clamp(min=0)
    else:
        kl = torch.zeros(1, device=dev)
    if loss_type == "kto":
        c_loss = 1 - torch.sigmoid(beta * (lr - kl))
        r_loss = 1 - torch.sigmoid(beta * (kl - lr))
    else:
        c_loss = 1 - torch.sigmoid(beta * lr)
        r_loss = torch.sigmoid(beta * lr)
    loss = torch.where(is_chosen, desirable_weight * c_loss, undesirable_weight * r_loss).nanmean()
    with torch.no_grad():
        chosen_f = is_chosen.to(torch.float32)
        cm, rm_ = m * chosen_f[:, None], m * (1 - chosen_f)[:, None]
        mean_logit = stats[..., 0]
        zero = torch.zeros((), device=dev)
        lr_d, seq_d = lr.detach(), seq.detach()
        metrics = {
            "kl": kl, "entropy_sum": (ent * m).sum(), "n_tokens": m.sum(),
            "logits_chosen_sum": torch.where(cm > 0, mean_logit, zero).sum(), "n_chosen_tokens": cm.sum(),
            "logits_rejected_sum": torch.where(rm_ > 0, mean_logit, zero).sum(), "n_rejected_tokens": rm_.sum(),
            "num_chosen": is_chosen.sum(), "num_rejected": (~is_chosen).sum(),
            "chosen_rewards_sum": torch.where(is_chosen, beta * lr_d, zero).nansum(),
            "rejected_rewards_sum": torch.where(is_chosen, zero, beta * lr_d).nansum(),
            "chosen_logps_sum": torch.where(is_chosen, seq_d, zero).nansum(),
            "rejected_logps_sum": torch.where(is_chosen, zero, seq_d).nansum(),
        }
    return loss, metrics


class KTOLossMixin:
    """`_compute_kl_logps` / `_compute_loss` with the reference's names and signatures
    (kto_trainer.py:1280-1330, 1478-1663; the path without `use_liger_kernel`); bind them onto a `KTOTrainer`."""

    _NON_MODEL_KEYS = ("completion_mask", "KL_input_ids", "KL_attention_mask", "KL_completion_mask", "KL_token_type_ids",
                       "KL_mm_token_type_ids", "label", "ref_logps", "ref_KL_logps")

    def _compute_kl_logps(self, model, batch):
        if not self.calculate_KL:
            return None
        kw = {k: v for k, v in batch.items() if k not in ("input_ids", "attention_mask") + self._NON_MODEL_KEYS}
        kw["input_ids"], kw["attention_mask"] = batch["KL_input_ids"], batch["KL_attention_mask"]
        for name in ("token_type_ids", "mm_token_type_ids"):
            if "KL_" + name in batch:
                kw[name] = batch["KL_" + name]
        with torch.no_grad():
            logits = model(**kw).logits
        return kto_sequence_logps(logits, batch["KL_input_ids"], batch["KL_completion_mask"])

    def _compute_loss(self, model, inputs, return_outputs):
        mode = "train" if self.model.training else "eval"
        acc = self.accelerator
        batch = {k: (v.to(acc.device) if isinstance(v, torch.Tensor) else v) for k, v in inputs.items()}
        kl_logps = self._compute_kl_logps(model, batch)
        model_kwargs = {k: v for k, v in batch.items() if k not in self._NON_MODEL_KEYS}
        aux_enabled = bool(getattr(self, "aux_loss_enabled", False))
        if aux_enabled:
            model_kwargs["output_router_logits"] = True
        outputs = model(**model_kwargs)
        if self.precompute_ref_logps:
            ref_logps = batch["ref_logps"]
            ref_kl = batch["ref_KL_logps"] if self.calculate_KL else None
        else:
            ref_kwargs = {k: v for k, v in model_kwargs.items() if k != "output_router_logits"}
            if getattr(self, "ref_model", None) is not None:
                ref_kl = self._compute_kl_logps(self.ref_model, batch)
                with torch.no_grad():
                    ref_logits = self.ref_model(**ref_kwargs).logits
            else:
                # adapter training without a separate reference model: the same network with its adapters switched
                # off, or with the frozen copy named "ref" active (kto_trainer.py:1534-1541)
                peft_model = acc.unwrap_model(self.model)
                if not hasattr(peft_model, "peft_config"):
                    raise ValueError("KTO needs reference log-probs: precomputed, from `ref_model`, or from a PEFT "
                                     "model whose adapters can be switched off")
                with _reference_adapter(peft_model):
                    ref_kl = self._compute_kl_logps(self.model, batch)
                    with torch.no_grad():
                        ref_logits = self.model(**ref_kwargs).logits
            ref_logps = kto_sequence_logps(ref_logits, batch["input_ids"], batch["completion_mask"])
        loss, parts = kto_compute_loss(
            outputs.logits, batch["input_ids"], batch["completion_mask"], batch["label"], ref_logps, kl_logps, ref_kl,
            beta=self.beta, loss_type=self.loss_type, desirable_weight=self.desirable_weight,
            undesirable_weight=self.undesirable_weight, kl_reduce=lambda kl: acc.gather_for_metrics(kl).mean())
        log = self._metrics[mode]
        names = ("entropy_sum", "n_tokens", "logits_chosen_sum", "n_chosen_tokens", "logits_rejected_sum",
                 "n_rejected_tokens", "num_chosen", "num_rejected", "chosen_rewards_sum", "rejected_rewards_sum",
                 "chosen_logps_sum", "rejected_logps_sum")
        sums = torch.stack([parts[k].to(torch.float32) for k in names])
        n_train = (acc.gather_for_metrics(batch["attention_mask"].sum()).sum().reshape(1) if mode == "train"
                   else sums.new_zeros(1))
        # every logged number in ONE copy to the host
        (ent_sum, n_tok, lc, nc, lr, nr, n_c, n_r, rew_c, rew_r, lp_c, lp_r, bits, kl, n_train) = torch.cat(
            [acc.gather_for_metrics(sums.unsqueeze(0)).nansum(dim=0).double(), ops.device_error_bits(sums.device).double(),
             parts["kl"].reshape(1).double(), n_train.double()]).tolist()
        ops.raise_for_error_bits(bits, sums.device)  # (a token id outside the vocabulary raises here)
        log["kl"].append(kl)
        log["entropy"].append(ent_sum / n_tok if n_tok > 0 else 0.0)
        if mode == "train":
            self._total_train_tokens += int(n_train)
        log["num_tokens"] = [self._total_train_tokens]
        if nc > 0:
            log["logits/chosen"].append(lc / nc)
        if nr > 0:
            log["logits/rejected"].append(lr / nr)
        if n_c > 0:
            log["rewards/chosen"].append(rew_c / n_c)
            log["logps/chosen"].append(lp_c / n_c)
        if n_r > 0:
            log["rewards/rejected"].append(rew_r / n_r)
            log["logps/rejected"].append(lp_r / n_r)
        if n_c > 0 and n_r > 0:
            log["rewards/margins"].append(log["rewards/chosen"][-1] - log["rewards/rejected"][-1])
        if aux_enabled:
            loss = loss + self.router_aux_loss_coef * outputs.aux_loss
            log["aux_loss"].append(acc.gather_for_metrics(outputs.aux_loss).mean().item())
        return (loss, outputs) if return_outputs else loss

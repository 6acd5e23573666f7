"""Fused-head counterpart of the reference's SFT `chunked_nll` loss
(`_chunked_cross_entropy_loss`, trl/trainer/sft_trainer.py:117-234)."""
from __future__ import annotations

import torch
from torch import Tensor

from .. import ops
from .utils import _fp32_head_backward, _fp32_head_forward

__all__ = ["_chunked_cross_entropy_loss"]


class _FusedNLLFunction(torch.autograd.Function):
    """(hidden [N, H], weight [V, H], labels [N]) -> fp32 per-token (log-prob, entropy, argmax-hit); only the
    log-prob is differentiable.  One matrix-core sweep forward; the backward works from the forward's stashed
    products when they fit `ops.head_stash_fits`, from a chunked recompute otherwise."""

    @staticmethod
    def forward(ctx, hidden, weight, labels, chunk_size, softcap, logit_scale, bias=None):
        ctx.cfg = (int(chunk_size), softcap, logit_scale)
        if hidden.dtype == torch.float32:  # fp32 operands: three bf16 pieces each through the same kernels
            if not hidden.is_cuda:
                raise NotImplementedError("the fused head runs on the GPU only")
            logp, ent, log_z, hit = _fp32_head_forward(hidden, weight.float(), labels.long(), 1.0, softcap, logit_scale,
                                                       None if bias is None else bias.float(), True)
            ctx.save_for_backward(hidden, weight, labels, log_z, None, bias)
            ctx.mark_non_differentiable(ent, hit)
            return logp, ent, hit
        stash = any(ctx.needs_input_grad[:2]) and ops.head_stash_fits(hidden.shape[0], weight.shape[0])
        logp, ent, log_z, hit, saved = ops.fused_head_fwd(hidden, weight, labels, 1.0, softcap, logit_scale, bias, stash)
        ctx.save_for_backward(hidden, weight, labels, log_z, saved, bias)
        ctx.mark_non_differentiable(ent, hit)
        return logp, ent, hit

    @staticmethod
    def backward(ctx, g_logp, g_ent, g_hit):
        hidden, weight, labels, log_z, saved, bias = ctx.saved_tensors
        chunk_size, softcap, logit_scale = ctx.cfg
        if hidden.dtype == torch.float32:
            d_hidden, d_weight, d_bias = _fp32_head_backward(hidden, weight.float(), labels.long(), 1.0, softcap,
                                                             logit_scale, None if bias is None else bias.float(), log_z,
                                                             g_logp)
            d_weight = d_weight.to(weight.dtype)
        else:
            d_hidden, d_weight, d_bias = ops.head_backward(hidden, weight, labels, 1.0, softcap, logit_scale, log_z,
                                                            g_logp, chunk_size, bias, saved)
        return d_hidden, d_weight, None, None, None, None, None if bias is None else d_bias.to(bias.dtype)


def _chunked_cross_entropy_loss(
    hidden_states: Tensor,
    lm_head_weight: Tensor,
    chunk_size: int,
    labels: Tensor | None = None,
    shift_labels: Tensor | None = None,
    num_items_in_batch: Tensor | int | None = None,
    logit_scale: float = 1.0,
    final_logit_softcapping: float | None = None,
    lm_head_bias: Tensor | None = None,
) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    """Next-token cross-entropy over hidden states and an `lm_head` weight without materialising logits.

    Same arguments and return value as the reference: `(loss, correct_count, entropy_sum, n_valid)` over the
    local batch; `labels` are shifted here, `shift_labels` are taken as already aligned; `-100` positions are
    dropped before the matmul; the loss is `sum / num_items_in_batch` if that is given, else the mean over
    valid tokens.  `chunk_size` sizes the backward's vocabulary-chunk workspace (the reference chunks tokens;
    the kernels need no token chunking).  `correct_count` counts tokens whose label holds the row maximum."""
    if labels is None and shift_labels is None:
        raise ValueError("At least one of `labels` or `shift_labels` must be provided.")
    if shift_labels is not None:
        hidden = hidden_states.reshape(-1, hidden_states.size(-1))
        flat_labels = shift_labels.reshape(-1)
    else:
        hidden = hidden_states[..., :-1, :].reshape(-1, hidden_states.size(-1))
        flat_labels = labels[..., 1:].reshape(-1)
    valid = flat_labels != -100
    n_valid = valid.sum()
    if int(n_valid) == 0:
        # whole micro-batch masked: keep the loss attached to every trainable input (sft_trainer.py:186-195)
        loss = (hidden_states.float().sum() + lm_head_weight.float().sum()) * 0.0
        if lm_head_bias is not None:
            loss = loss + lm_head_bias.float().sum() * 0.0
        zero = hidden.new_zeros((), dtype=torch.float32)
        return loss, zero, zero.clone(), n_valid
    cap = 0.0 if final_logit_softcapping is None else float(final_logit_softcapping)
    logp, ent, hit = _FusedNLLFunction.apply(hidden[valid], lm_head_weight, flat_labels[valid], chunk_size, cap,
                                             float(logit_scale), lm_head_bias)
    loss = -logp.sum()
    if num_items_in_batch is None:
        loss = loss / n_valid
    else:
        if isinstance(num_items_in_batch, Tensor):
            num_items_in_batch = num_items_in_batch.to(loss.device)
        loss = loss / num_items_in_batch
    return loss, hit.sum(), ent.sum(), n_valid

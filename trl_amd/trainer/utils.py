"""Drop-in counterparts of the hot-path helpers in the reference's `trl/trainer/utils.py`.

Same names, argument meaning and error behaviour as the reference functions; the arithmetic
runs in the HIP kernels behind `trl_amd.ops` (device tensors only).
"""
from __future__ import annotations

import torch
from torch import Tensor

from .. import ops

__all__ = ["selective_log_softmax", "entropy_from_logits", "logps_and_entropies", "nanstd", "nanmin", "nanmax",
           "_ChunkedLogProbFunction", "chunked_logprobs_from_hidden", "patch_chunked_lm_head"]


def _as_3d(logits: Tensor) -> Tensor:
    """View `[..., V]` logits as `[n_seq, rows, V]` without copying when the strides allow it."""
    if logits.dim() == 0:
        raise ValueError("logits must have at least one dimension")
    v = logits.shape[-1]
    if v > 1 and logits.stride(-1) != 1:
        logits = logits.contiguous()
    if logits.dim() == 1:
        return logits.view(1, 1, v)
    if logits.dim() == 2:
        out = logits.unsqueeze(0)
    elif logits.dim() == 3:
        out = logits
    else:
        try:
            out = logits.view(-1, logits.shape[-2], v)
        except RuntimeError:
            out = logits.reshape(-1, logits.shape[-2], v)
    if out.shape[1] > 1 and out.stride(1) < v:  # expanded / overlapping rows
        out = out.contiguous()
    return out


def logps_and_entropies(
    logits: Tensor, index: Tensor, temperature: float = 1.0, keep_start: int = 0, keep_len: int | None = None,
    row_mask: Tensor | None = None,
) -> tuple[Tensor, Tensor]:
    """One streaming pass over `[n_seq, L, V]` logits: fp32 log-probs of `index` and fp32 entropies
    of rows `keep_start .. keep_start + keep_len` of every sequence, of `softmax(logits / temperature)`.
    `index` is `[n_seq, keep_len]` or `[n_seq, keep_len, K]`.  Differentiable w.r.t. `logits` (both
    outputs); the gradient covers all `L` rows (zero outside the window).  With `row_mask`
    (`[n_seq, keep_len]`, zero = skip) masked rows are not read and yield 0."""
    if logits.dim() != 3:
        raise ValueError("logps_and_entropies expects [n_seq, L, V] logits")
    n_seq, length, _ = logits.shape
    keep_len = length - keep_start if keep_len is None else keep_len
    if keep_start < 0 or keep_len < 0 or keep_start + keep_len > length:
        raise ValueError(f"rows [{keep_start}, {keep_start + keep_len}) are outside the {length} rows of the logits")
    squeeze = index.dim() == 2
    idx = index.reshape(n_seq * keep_len, 1 if squeeze else index.shape[-1])
    if idx.dtype != torch.int64:
        idx = idx.long()
    rm = None
    if row_mask is not None:
        rm = (row_mask.reshape(-1) != 0).to(torch.uint8).contiguous()
    logp, ent, _ = ops.logp_entropy_forward(logits, idx, float(temperature), keep_start, keep_len, rm)
    logp = logp.view(n_seq, keep_len) if squeeze else logp.view(n_seq, keep_len, index.shape[-1])
    return logp, ent.view(n_seq, keep_len)


def selective_log_softmax(logits: Tensor, index: Tensor, out_dtype: torch.dtype | None = None) -> Tensor:
    """`torch.gather(logits.log_softmax(-1), -1, index)` without materialising the log-softmax
    (reference: trl/trainer/utils.py:479-523).  `index` has shape `(...)` or `(..., K)`.

    The kernel computes in fp32 (in fp64 for float64 logits).  `out_dtype=None` returns the logits dtype as the
    reference does (for bf16/fp16 logits the fp32 result is rounded once to that dtype);
    `out_dtype=torch.float32` keeps the unrounded values."""
    squeeze = index.dim() == logits.dim() - 1
    if not squeeze and index.dim() != logits.dim():
        raise ValueError(f"index of shape {tuple(index.shape)} does not match logits of shape {tuple(logits.shape)}")
    if tuple(index.shape[: logits.dim() - 1]) != tuple(logits.shape[:-1]):
        raise RuntimeError(
            f"Size does not match at the leading dimensions: index {tuple(index.shape)}, logits {tuple(logits.shape)}"
        )
    x = _as_3d(logits)
    k = 1 if squeeze else index.shape[-1]
    idx = index.reshape(x.shape[0] * x.shape[1], k)
    if idx.dtype != torch.int64:
        raise RuntimeError(f"gather(): Expected dtype int64 for index, got {idx.dtype}")
    logp, _, _ = ops.logp_entropy_forward(x, idx, 1.0, 0, x.shape[1], None)
    logp = logp.view(index.shape)
    out_dtype = logits.dtype if out_dtype is None else out_dtype
    return logp if out_dtype == logp.dtype else logp.to(out_dtype)


def entropy_from_logits(logits: Tensor, chunk_size: int = 128, out_dtype: torch.dtype | None = None) -> Tensor:
    """Shannon entropy (nats) of `softmax(logits)` over the last axis, shape `logits.shape[:-1]`
    (reference: trl/trainer/utils.py:526-560).  `chunk_size` is accepted for signature
    compatibility; the kernel streams each row once and needs no chunking."""
    x = _as_3d(logits)
    idx = torch.empty((x.shape[0] * x.shape[1], 0), dtype=torch.int64, device=logits.device)
    _, ent, _ = ops.logp_entropy_forward(x, idx, 1.0, 0, x.shape[1], None)
    ent = ent.view(logits.shape[:-1])
    out_dtype = logits.dtype if out_dtype is None else out_dtype
    return ent if out_dtype == ent.dtype else ent.to(out_dtype)


# ----------------------------------------------------------------------------------------------
# O(B) helpers on tiny tensors: plain torch, as in the reference (trl/trainer/utils.py:857-890, 960-987)
# ----------------------------------------------------------------------------------------------
def nanstd(tensor: Tensor, dim=None, keepdim: bool = False) -> Tensor:
    """Bessel-corrected standard deviation ignoring NaNs; NaN where fewer than two values remain."""
    mean = torch.nanmean(tensor, dim=dim, keepdim=True)
    var = torch.nanmean((tensor - mean) ** 2, dim=dim, keepdim=True)
    count = torch.sum(~torch.isnan(tensor), dim=dim, keepdim=True)
    var = var * torch.where(count > 1, count / (count - 1), torch.full_like(var, float("nan")))
    std = var.sqrt()
    if keepdim:
        return std
    if dim is None:
        return std.squeeze()
    dims = (dim,) if isinstance(dim, int) else dim
    for d in sorted((d % std.dim() for d in dims), reverse=True):
        std = std.squeeze(d)
    return std


def nanmin(tensor: Tensor) -> Tensor:
    """Minimum of a 1-D tensor ignoring NaNs; NaN if every entry is NaN."""
    keep = ~torch.isnan(tensor)
    if not keep.any():
        return torch.tensor(float("nan"), dtype=tensor.dtype, device=tensor.device)
    return tensor[keep].min()


def nanmax(tensor: Tensor) -> Tensor:
    """Maximum of a 1-D tensor ignoring NaNs; NaN if every entry is NaN."""
    keep = ~torch.isnan(tensor)
    if not keep.any():
        return torch.tensor(float("nan"), dtype=tensor.dtype, device=tensor.device)
    return tensor[keep].max()


# ----------------------------------------------------------------------------------------------
# fused lm_head + log-prob (reference: trl/trainer/utils.py:1291-1517)
# ----------------------------------------------------------------------------------------------
def _fp32_head_block_rows(vocab: int) -> int:
    """Token rows per block of the fp32-operand backward: about 1 GiB of fp32 logits at a time."""
    return max(64, min(8192, (1 << 28) // max(vocab, 1)))


def _fp32_head_forward(hidden, weight, targets, temperature, cap, logit_scale, bias, want_hit=False):
    """fp32 operands through the same fused kernel: both are split into three bf16 pieces laid out along the
    contraction axis (`ops.split_bf16x3`), on which the matrix cores return the fp32 products to fp32 rounding; the
    logits are never written to memory.  Costs six times the matrix work of bf16 operands and a `[V, 6 H]` bf16 copy
    of the weight: this is the dtype of the reference's unit test (tests/test_utils.py:1161-1232), not of training."""
    hp, wp = ops.split_bf16x3(hidden, 0), ops.split_bf16x3(weight, 1)
    logp, ent, lse, hit, _ = ops.fused_head_fwd(hp, wp, targets, temperature, cap, logit_scale, bias, False)
    return (logp, ent, lse, hit) if want_hit else (logp, ent, lse)


def _fp32_head_backward(hidden, weight, targets, temperature, cap, logit_scale, bias, lse, grad_logprobs):
    """fp32 operands: per block of tokens the logits are recomputed (`ops.gemm_nt` on bf16 pieces), d logits come
    from the streaming backward kernel in fp32, and both gradient products run on the bf16 pieces of d logits,
    W^T and hidden^T -- everything on this library's matrix-core kernel at fp32 accuracy, as the reference's fp32
    `grad_logits @ w_chunk.float()` / `grad_logits.t() @ hidden.float()` (trl/trainer/utils.py:1421-1422)."""
    n, v = hidden.shape[0], weight.shape[0]
    # (dense rows whatever the operands' strides: the products write through `out=` with a unit inner stride)
    d_hidden = torch.empty(hidden.shape, dtype=hidden.dtype, device=hidden.device)
    d_weight = torch.zeros(weight.shape, dtype=weight.dtype, device=weight.device)
    d_bias = torch.zeros(v, dtype=torch.float32, device=hidden.device) if bias is not None else None
    g = grad_logprobs.contiguous().float()
    wp = ops.split_bf16x3(weight, 1)                   # [V, 6 H]: right operand of the logits
    wtp = ops.split_bf16x3(weight.t().contiguous(), 1)  # [H, 6 V]: right operand of d hidden = dz @ W
    step = _fp32_head_block_rows(v)
    for r0 in range(0, n, step):
        r1 = min(r0 + step, n)
        y = ops.gemm_nt(ops.split_bf16x3(hidden[r0:r1], 0), wp)
        if bias is not None:
            y += bias
        if logit_scale != 1.0:
            y *= logit_scale
        th = None
        if cap > 0.0:
            th = torch.tanh(y / cap)
            y = th * cap
        dz = ops.logp_entropy_bwd(y.unsqueeze(0), targets[r0:r1].reshape(-1, 1), temperature, 0, r1 - r0, lse[r0:r1], None,
                                  g[r0:r1].reshape(-1, 1), None).squeeze(0)
        if th is not None:
            dz *= 1.0 - th * th
        if logit_scale != 1.0:
            dz *= logit_scale
        ops.gemm_nt(ops.split_bf16x3(dz, 0), wtp, out=d_hidden[r0:r1])
        ops.gemm_nt(ops.split_bf16x3(dz.t().contiguous(), 0), ops.split_bf16x3(hidden[r0:r1].t().contiguous(), 1),
                    out=d_weight, accumulate=r0 > 0)
        if d_bias is not None:
            d_bias += dz.sum(0)
    return d_hidden, d_weight, d_bias


class _ChunkedLogProbFunction(torch.autograd.Function):
    """Per-token log-probs and entropy of `softmax((hidden @ weight.T) / temperature)` without ever
    materialising the `[N, V]` logits.  Same call signature as the reference operator
    (utils.py:1298-1307): `apply(last_hidden [N, H], weight [V, H], targets [N], temperature,
    chunk_size, final_logit_softcapping=None, logit_scale=1.0) -> (logprobs fp32 [N], entropy fp32 [N])`.

    The forward is one matrix-core kernel sweep (no vocabulary chunking is needed, `chunk_size` only
    sizes the backward's dz workspace).  When a gradient is required and the fp32 `[V, N]` products fit
    `ops.head_stash_fits` (24 GiB by default), the forward keeps them and the backward skips the
    reference's recompute of the logits; otherwise it recomputes them chunk by chunk as the reference does.
    fp32 operands run through the same kernels as three bf16 pieces each (`ops.split_bf16x3`: the matrix cores take
    16-bit operands, six piece products give the fp32 product to fp32 rounding); their backward recomputes the logits
    per block of tokens and takes d logits in fp32 from the streaming backward kernel.  fp64 is rejected.
    The entropy output is not differentiable, as in the reference.
    One argument beyond the reference's: `bias` [V], the `lm_head` bias the fused-linear losses take."""

    @staticmethod
    def forward(ctx, last_hidden, weight, targets, temperature, chunk_size, final_logit_softcapping=None,
                logit_scale=1.0, bias=None):
        cap = 0.0 if final_logit_softcapping is None else float(final_logit_softcapping)
        if last_hidden.dtype == torch.float32:
            if not last_hidden.is_cuda:
                raise NotImplementedError("the fused head runs on the GPU only")
            w32 = weight.float()
            logp, ent, log_z = _fp32_head_forward(last_hidden, w32, targets.long(), float(temperature), cap,
                                                  float(logit_scale), None if bias is None else bias.float())
            ctx.save_for_backward(last_hidden, weight, targets, log_z, bias, None)
            ctx.cfg = (float(temperature), int(chunk_size), cap, float(logit_scale))
            ctx.mark_non_differentiable(ent)
            return logp, ent
        stash = any(ctx.needs_input_grad[:2]) and ops.head_stash_fits(last_hidden.shape[0], weight.shape[0])
        logp, ent, log_z, _, saved = ops.fused_head_fwd(last_hidden, weight, targets, float(temperature), cap,
                                                        float(logit_scale), bias, stash)
        ctx.save_for_backward(last_hidden, weight, targets, log_z, bias, saved)
        ctx.cfg = (float(temperature), int(chunk_size), cap, float(logit_scale))
        ctx.mark_non_differentiable(ent)
        return logp, ent

    @staticmethod
    def backward(ctx, grad_logprobs, grad_entropy):
        hidden, weight, targets, log_z, bias, saved = ctx.saved_tensors
        temperature, chunk_size, cap, logit_scale = ctx.cfg
        if hidden.dtype == torch.float32:
            d_hidden, d_weight, d_bias = _fp32_head_backward(hidden, weight.float(), targets.long(), temperature, cap,
                                                             logit_scale, None if bias is None else bias.float(), log_z,
                                                             grad_logprobs)
            return (d_hidden, d_weight.to(weight.dtype), None, None, None, None, None,
                    None if bias is None else d_bias.to(bias.dtype))
        d_hidden, d_weight, d_bias = ops.head_backward(hidden, weight, targets, temperature, cap, logit_scale,
                                                        log_z, grad_logprobs, chunk_size, bias, saved)
        return (d_hidden, d_weight, None, None, None, None, None,
                None if bias is None else d_bias.to(bias.dtype))


def chunked_logprobs_from_hidden(hidden_states: Tensor, lm_head_weight: Tensor, labels: Tensor,
                                 completion_mask: Tensor | None, temperature: float, chunk_size: int = 8192,
                                 final_logit_softcapping: float | None = None, logit_scale: float = 1.0):
    """The tensor part of the reference's patched forward (utils.py:1449-1484): shift by one, keep only
    completion rows, run the fused head on them, scatter into zero-filled `[B, S-1]` outputs.
    Returns `(log_probs, entropy)`."""
    hs = hidden_states[:, :-1, :]
    lab = labels[:, 1:]
    b, s, h = hs.shape
    flat_h = hs.reshape(b * s, h)
    flat_t = lab.reshape(b * s)
    keep = None
    if completion_mask is not None:
        keep = completion_mask[:, 1:].bool().reshape(b * s)
        flat_h = flat_h[keep]
        flat_t = flat_t[keep]
    lp_v, ent_v = _ChunkedLogProbFunction.apply(flat_h, lm_head_weight, flat_t, temperature, chunk_size,
                                                final_logit_softcapping, logit_scale)
    if keep is None:
        return lp_v.reshape(b, s), ent_v.reshape(b, s)
    lp = torch.zeros(b * s, device=lp_v.device, dtype=lp_v.dtype)
    ent = torch.zeros(b * s, device=ent_v.device, dtype=ent_v.dtype)
    lp[keep] = lp_v
    ent[keep] = ent_v
    return lp.reshape(b, s), ent.reshape(b, s)


def patch_chunked_lm_head(model: torch.nn.Module, chunk_size: int, temperature: float,
                          output_router_logits: bool = False) -> None:
    """Replaces `model.forward` by one that runs the backbone, then the fused head, and returns
    `{"log_probs" [B, S-1], "entropy" [B, S-1], "aux_loss"}` (reference: utils.py:1427-1517).
    With `output_router_logits` the backbone is asked for its router logits and `aux_loss` is the transformers
    load-balancing loss of them (the function every MoE family shares), as in the reference (:1484-1508)."""
    import types

    final_logit_softcapping = getattr(model.config, "final_logit_softcapping", None)

    def _chunked_forward(self, input_ids=None, attention_mask=None, labels=None, completion_mask=None,
                         use_cache=False, **kwargs):
        assert labels is not None, "requires labels to not be None for logprob computation"
        decoder_kwargs = {"output_router_logits": True} if output_router_logits else {}
        outputs = self.model(input_ids=input_ids, attention_mask=attention_mask, use_cache=use_cache, **decoder_kwargs,
                             **kwargs)
        logit_scale = getattr(self.config, "logit_scale", 1.0)
        log_probs, entropy = chunked_logprobs_from_hidden(
            outputs.last_hidden_state, self.lm_head.weight, labels, completion_mask, temperature, chunk_size,
            final_logit_softcapping, logit_scale)
        aux_loss = None
        if output_router_logits:
            from transformers.models.mixtral.modeling_mixtral import load_balancing_loss_func

            # the expert counts live on the config (on the module itself for some families / older transformers)
            num_experts = getattr(self.config, "num_experts", None) or getattr(self, "num_experts")
            top_k = getattr(self.config, "num_experts_per_tok", None) or getattr(self, "num_experts_per_tok")
            aux_loss = load_balancing_loss_func(outputs.router_logits, num_experts, top_k, attention_mask)
        return {"log_probs": log_probs, "entropy": entropy, "aux_loss": aux_loss}

    model.forward = types.MethodType(_chunked_forward, model)

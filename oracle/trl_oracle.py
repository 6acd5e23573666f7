"""CPU restatement (PyTorch, host only) of the reference's log-probability / entropy /
policy-loss path.  TEST INFRASTRUCTURE: this module is the *checker* for the HIP
kernels and the CPU baseline of the benchmark.  The shipped package never imports it.

Every function cites the reference lines (paths relative to the reference tree) whose
arithmetic it follows.  The functions keep the reference's *order of operations and
dtypes* (row loops, 128-row chunks, in-dtype temperature division) because those are
what a user of the reference observes; `*_f32` variants are the same mathematics with
fp32 op-math on the same (possibly bf16-valued) inputs and are what low-precision
kernel outputs are compared against.

Pinning status (what checks each function against something other than itself):
  selective_log_softmax / entropy_from_logits : torch library routines
      (`log_softmax().gather()`, `-(p*log p).sum()`), closed forms (uniform row,
      shift invariance), reference unit-test shapes  -> tests/test_oracle.py
  nanstd / nanmin / nanmax  : reference unit-test vectors (tests/test_utils.py:316-331)
  group_advantages          : torch.std(unbiased) on NaN-free groups, zero-variance
                              closed form, golden vectors from the reference's formula
  grpo_loss                 : golden vectors written by the reference's
                              `GRPOTrainer._compute_loss` on a mocked trainer
                              (tests/golden/), closed forms (on-policy, ref == logps)
  dpo_*                     : golden vectors from the reference's
                              `DPOTrainer._compute_loss` (mocked; all fifteen loss types, ld_alpha, WPO
                              weighting, f-divergences, arg-max ties), closed form ln 2
  rloo_loss                 : golden vectors from `RLOOTrainer._compute_loss` (mocked)
  kto_*                     : golden vectors from `KTOTrainer._compute_loss` (mocked, KL pass included),
                              closed form 1/2 at policy == reference
  vllm_importance_sampling_ratio : hand-computed values per mode (no reference test holds numbers for it)
  chunked_logprob           : naive `(h @ W.T).float()/T -> log_softmax` routine and
                              autograd of it (reference test tests/test_utils.py:1161-1232)
  chunked_cross_entropy_loss: golden vectors from the reference's `_chunked_cross_entropy_loss`,
                              `F.cross_entropy` library routine
  fused_linear_grpo_loss / fused_linear_dpo_loss / fused_linear_kto_loss : PARITY UNPINNED against the third-party operators
                              they stand in for (liger-kernel >=0.8.0,<0.8.1 is not importable here and no
                              reference test holds their numbers); they compose pinned pieces only -- the naive
                              head routine + `grpo_loss` / `dpo_sigmoid_loss` -- in the metric order the
                              reference's call sites read (grpo_trainer.py:2900-2901, dpo_trainer.py:1293-1301)
  get_off_policy_mask       : reference unit-test vectors (tests/test_grpo_trainer.py:1456-1520)
  get_high_entropy_mask     : reference unit-test vectors (tests/test_grpo_trainer.py:110-160)
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

__all__ = [
    "selective_log_softmax",
    "selective_log_softmax_f32",
    "entropy_from_logits",
    "entropy_from_logits_f32",
    "nanstd",
    "nanmin",
    "nanmax",
    "group_advantages",
    "rloo_advantages",
    "get_off_policy_mask",
    "get_high_entropy_mask",
    "get_gamma_weights",
    "vllm_importance_sampling_ratio",
    "logps_and_entropies_from_logits",
    "grpo_loss",
    "dpo_sequence_logps",
    "dpo_sigmoid_loss",
    "dpo_compute_loss",
    "rloo_loss",
    "kto_sequence_logps",
    "kto_compute_loss",
    "chunked_logprob_naive",
    "chunked_logprob_online",
    "chunked_logprob_backward",
    "ChunkedLogProbOracle",
    "patch_chunked_rows",
    "chunked_cross_entropy_loss",
    "fused_linear_grpo_loss",
    "fused_linear_dpo_loss",
    "fused_linear_kto_loss",
]


# --------------------------------------------------------------------------------------
# A1  selective_log_softmax               trl/trainer/utils.py:479-523
# --------------------------------------------------------------------------------------
def selective_log_softmax(logits: torch.Tensor, index: torch.Tensor) -> torch.Tensor:
    """`log_softmax(logits)[..., index]` with the reference's two dtype branches.

    fp32/fp64 (utils.py:506-510): gather the selected logits, subtract a per-leading-row
    `logsumexp`.  Other dtypes (utils.py:511-518): per-leading-row `log_softmax` in the
    input dtype followed by `gather` (output stays in the low-precision dtype).
    `index` has either the leading shape of `logits` or one extra trailing axis K
    (utils.py:502-504, 520-521).
    """
    drop_last = index.ndim == logits.ndim - 1
    idx = index.unsqueeze(-1) if drop_last else index
    if logits.dtype in (torch.float32, torch.float64):
        picked = logits.gather(-1, idx)
        lse = torch.stack([torch.logsumexp(block, dim=-1) for block in logits])
        out = picked - lse.unsqueeze(-1)
    else:
        rows = []
        for block, block_idx in zip(logits, idx, strict=True):
            rows.append(F.log_softmax(block, dim=-1).gather(-1, block_idx))
        out = torch.stack(rows)
    return out.squeeze(-1) if drop_last else out


def selective_log_softmax_f32(logits: torch.Tensor, index: torch.Tensor, temperature: float = 1.0) -> torch.Tensor:
    """Same quantity with fp32 op-math on the stored values: the reference function
    applied to `logits.float() / temperature` (grpo_trainer.py:1519 + utils.py:506-510).
    Processed block-wise so that a bf16 input is never widened all at once."""
    drop_last = index.ndim == logits.ndim - 1
    idx = index.unsqueeze(-1) if drop_last else index
    flat = logits.reshape(-1, logits.shape[-1]) if logits.ndim > 1 else logits.unsqueeze(0)
    flat_idx = idx.reshape(-1, idx.shape[-1])
    out = torch.empty(flat_idx.shape, dtype=torch.float32)
    for r0 in range(0, flat.shape[0], 256):
        z = flat[r0 : r0 + 256].float() / temperature
        out[r0 : r0 + 256] = z.gather(-1, flat_idx[r0 : r0 + 256]) - torch.logsumexp(z, -1, keepdim=True)
    out = out.reshape(idx.shape)
    return out.squeeze(-1) if drop_last else out


# --------------------------------------------------------------------------------------
# A2  entropy_from_logits                 trl/trainer/utils.py:526-560
# --------------------------------------------------------------------------------------
def entropy_from_logits(logits: torch.Tensor, chunk_size: int = 128) -> torch.Tensor:
    """Shannon entropy (nats) of softmax(logits) per row.  Rows are flattened
    (utils.py:551) and handled `chunk_size` at a time (utils.py:554-557) with all
    intermediates in the input dtype: H = -sum(exp(lp) * lp), lp = log_softmax(row)."""
    lead = logits.shape[:-1]
    rows = logits.reshape(-1, logits.shape[-1])
    pieces = []
    for piece in rows.split(chunk_size, dim=0):
        lp = F.log_softmax(piece, dim=-1)
        pieces.append(-(lp.exp() * lp).sum(-1))
    return torch.cat(pieces, 0).reshape(lead)


def entropy_from_logits_f32(logits: torch.Tensor, temperature: float = 1.0) -> torch.Tensor:
    """fp32 op-math entropy of `softmax(logits.float() / temperature)`."""
    lead = logits.shape[:-1]
    rows = logits.reshape(-1, logits.shape[-1])
    out = torch.empty(rows.shape[0], dtype=torch.float32)
    for r0 in range(0, rows.shape[0], 256):
        lp = F.log_softmax(rows[r0 : r0 + 256].float() / temperature, dim=-1)
        out[r0 : r0 + 256] = -(lp.exp() * lp).sum(-1)
    return out.reshape(lead)


# --------------------------------------------------------------------------------------
# nanstd / nanmin / nanmax                trl/trainer/utils.py:857-890, 960-987
# --------------------------------------------------------------------------------------
def nanstd(x: torch.Tensor, dim=None, keepdim: bool = False) -> torch.Tensor:
    """Bessel-corrected standard deviation over the non-NaN entries (utils.py:874-880):
    sqrt(nanmean((x - nanmean(x))^2) * n/(n-1)), NaN when n <= 1."""
    mu = torch.nanmean(x, dim=dim, keepdim=True)
    var = torch.nanmean((x - mu) ** 2, dim=dim, keepdim=True)
    n = (~x.isnan()).sum(dim=dim, keepdim=True)
    bessel = torch.where(n > 1, n / (n - 1), torch.full_like(var, float("nan")))
    sd = (var * bessel).sqrt()
    if keepdim:
        return sd
    if dim is None:
        return sd.squeeze()
    if isinstance(dim, int):
        return sd.squeeze(dim)
    for d in sorted((d % sd.ndim for d in dim), reverse=True):
        sd = sd.squeeze(d)
    return sd


def nanmin(x: torch.Tensor) -> torch.Tensor:
    """Minimum over non-NaN entries of a 1-D tensor; NaN if there are none (utils.py:960-972)."""
    keep = ~x.isnan()
    return x[keep].min() if keep.any() else x.new_tensor(float("nan"))


def nanmax(x: torch.Tensor) -> torch.Tensor:
    """Maximum over non-NaN entries of a 1-D tensor; NaN if there are none (utils.py:975-987)."""
    keep = ~x.isnan()
    return x[keep].max() if keep.any() else x.new_tensor(float("nan"))


# --------------------------------------------------------------------------------------
# A5  group-relative advantages           trl/trainer/grpo_trainer.py:2685-2707, 2730
# --------------------------------------------------------------------------------------
def group_advantages(rewards: torch.Tensor, num_generations: int, scale_rewards: str = "group") -> torch.Tensor:
    """`rewards` [B] (NaN = unscorable), groups are `num_generations` consecutive rows
    (`view(-1, G)`, grpo_trainer.py:2685).  A = r - nanmean_g; divided by
    (nanstd_g + 1e-4) for "group", by (nanstd_all + 1e-4) for "batch", not at all for
    "none" (grpo_trainer.py:2687-2707); NaN -> 0 (grpo_trainer.py:2730)."""
    G = num_generations
    grouped = rewards.view(-1, G)
    mean_g = torch.nanmean(grouped, dim=1).repeat_interleave(G)
    if scale_rewards in ("group", "none"):
        std = nanstd(grouped, dim=1).repeat_interleave(G) if G > 1 else torch.zeros_like(rewards)
    elif scale_rewards == "batch":
        std = nanstd(rewards).expand_as(rewards) if rewards.numel() > 1 else torch.zeros_like(rewards)
    else:
        raise ValueError(f"Invalid value for scale_rewards: {scale_rewards}")
    adv = rewards - mean_g
    if scale_rewards != "none":
        adv = adv / (std + 1e-4)
    return torch.nan_to_num(adv, nan=0.0)


def rloo_advantages(rewards: torch.Tensor, num_generations: int, normalize_advantages: bool = False) -> torch.Tensor:
    """Leave-one-out baseline over scorable siblings (rloo_trainer.py:1537-1561):
    b_i = (nansum_g - r_i) / (n_scorable - 1), A = r - b, optional global
    (A - nanmean)/(nanstd + 1e-4), NaN -> 0."""
    G = num_generations
    grouped = rewards.view(-1, G)
    if G > 1:
        n = (~grouped.isnan()).sum(1, keepdim=True)
        total = torch.nansum(grouped, dim=1, keepdim=True)
        adv = rewards - ((total - grouped) / (n - 1)).view(-1)
    else:
        adv = torch.zeros_like(rewards)
    if normalize_advantages:
        adv = (adv - torch.nanmean(adv)) / (nanstd(adv) + 1e-4)
    return torch.nan_to_num(adv, nan=0.0)


# --------------------------------------------------------------------------------------
# sequence masks                          trl/trainer/grpo_trainer.py:2920-2939, 1396-1432
# --------------------------------------------------------------------------------------
def get_off_policy_mask(advantages, per_token_logps, sampling_per_token_logps, mask, off_policy_threshold):
    """(B,1) keep-mask: keep if A >= 0 or masked-mean(sampling_logp - logp) <= threshold
    (grpo_trainer.py:2934-2939)."""
    gap = sampling_per_token_logps - per_token_logps.detach()
    mean_gap = (gap * mask).sum(1, keepdim=True) / mask.sum(1, keepdim=True).clamp(min=1.0)
    return ((advantages >= 0) | (mean_gap <= off_policy_threshold)).to(mask.dtype)


def vllm_importance_sampling_ratio(old_logps, sampling_logps, completion_mask, tool_mask, mode, clip_min, clip_max):
    """Sampler/trainer mismatch correction, trl/trainer/grpo_trainer.py:2578-2623, one branch per mode."""
    mask = completion_mask if tool_mask is None else completion_mask * tool_mask
    d = (old_logps - sampling_logps) * mask
    if mode in ("sequence_mask", "sequence_truncate"):
        d = d.sum(dim=-1, keepdim=True)
    r = torch.exp(d)
    if mode in ("sequence_truncate", "token_truncate"):
        return torch.clamp(r, min=clip_min, max=clip_max)
    if mode in ("sequence_mask", "token_mask"):
        lo = -math.inf if clip_min is None else clip_min
        hi = math.inf if clip_max is None else clip_max
        return torch.where((r < lo) | (r > hi), torch.zeros_like(r), r)
    raise ValueError(mode)


def get_high_entropy_mask(entropies, mask, threshold):
    """Boolean mask of active tokens whose entropy is >= the `threshold` quantile of all
    active-token entropies (single process: the cross-rank gather is the identity)
    (grpo_trainer.py:1413-1432)."""
    active = entropies[mask.bool()].float()
    if active.numel() == 0:
        return torch.zeros_like(entropies, dtype=torch.bool)
    cut = torch.quantile(active, threshold)
    return ((entropies * mask.float()) >= cut) & mask.bool()


@torch.no_grad()
def get_gamma_weights(advantages, log_ratio_per_token, mask, importance_sampling_ratio=None, k_pos=2.0, lambda_pos=3.0,
                      k_neg=3.0, lambda_neg=2.0):
    """VESPO sequence weights phi(w) = e^lambda * w^k * e^(-lambda w) in log space, w = exp(sum of the clamped
    per-token log-ratios) (grpo_trainer.py:2941-2989); (B, 1), no gradient."""
    floor = math.log(1e-8)
    seq = (log_ratio_per_token.clamp(-20.0, 20.0) * mask).sum(-1, keepdim=True)
    if importance_sampling_ratio is not None:
        seq = seq + importance_sampling_ratio.log().clamp(floor, 20.0).sum(-1, keepdim=True)
    log_w = seq.clamp(floor, 20.0)
    w = log_w.exp()
    pos = advantages >= 0
    k = torch.where(pos, k_pos, k_neg)
    lam = torch.where(pos, lambda_pos, lambda_neg).clamp(min=1e-4)
    return (lam + k * log_w - lam * w).exp().nan_to_num(nan=0.0, posinf=0.0, neginf=0.0)


# --------------------------------------------------------------------------------------
# A3 + A4  logits -> per-token logps / entropies   trl/trainer/grpo_trainer.py:1511-1533
# --------------------------------------------------------------------------------------
def logps_and_entropies_from_logits(
    logits: torch.Tensor,
    input_ids: torch.Tensor,
    logits_to_keep: int,
    temperature: float = 1.0,
    compute_entropy: bool = True,
    entropy_requires_grad: bool = False,
):
    """The part of `_get_per_token_logps_and_entropies` after the model call: drop the
    last position (grpo_trainer.py:1514), keep the last `logits_to_keep` (:1516),
    divide by the temperature *in the logits dtype* (:1519, here out of place so the
    caller's tensor survives), select log-probs of `input_ids[:, -K:]` (:1520-1521),
    entropy with or without grad (:1528-1532)."""
    z = logits[:, :-1, :][:, -logits_to_keep:, :]
    z = z / temperature
    ids = input_ids[:, -logits_to_keep:]
    logps = selective_log_softmax(z, ids)
    ent = None
    if compute_entropy:
        if entropy_requires_grad:
            ent = entropy_from_logits(z)
        else:
            with torch.no_grad():
                ent = entropy_from_logits(z)
    return logps, ent


# --------------------------------------------------------------------------------------
# A6-A9  GRPO loss                        trl/trainer/grpo_trainer.py:3026-3258
# --------------------------------------------------------------------------------------
def grpo_loss(
    per_token_logps: torch.Tensor,
    advantages: torch.Tensor,
    mask: torch.Tensor,
    *,
    entropies: torch.Tensor | None = None,
    old_per_token_logps: torch.Tensor | None = None,
    ref_per_token_logps: torch.Tensor | None = None,
    loss_type: str = "dapo",
    epsilon_low: float = 0.2,
    epsilon_high: float = 0.2,
    beta: float = 0.0,
    delta: float | None = None,
    max_completion_length: int | None = None,
    num_items_in_batch: torch.Tensor | float | None = None,
    num_processes: int = 1,
    grad_accum_steps: float = 1.0,
    importance_sampling_level: str = "token",
    use_bias_correction_kl: bool = False,
    off_policy_mask_threshold: float | None = None,
    sampling_per_token_logps: torch.Tensor | None = None,
    top_entropy_quantile: float = 1.0,
    importance_sampling_ratio: torch.Tensor | None = None,
    entropy_coef: float = 0.0,
    adaptive_entropy: dict | None = None,
    sapo_temperature_pos: float = 1.0,
    sapo_temperature_neg: float = 1.05,
    vespo_params: tuple[float, float, float, float] = (2.0, 3.0, 3.0, 2.0),
):
    """Clipped-surrogate GRPO family loss on `[B, T]` log-probs.  Returns
    `(loss, metrics)` where `metrics` holds python floats named as the reference logs
    them (grpo_trainer.py:3237-3258).  Covers loss types grpo / bnpo / dr_grpo / dapo / luspo / cispo /
    sapo / vespo (grpo_trainer.py:3080-3107, 3124-3148), token- and sequence-level importance
    weights (:3054-3059), k3 KL (:3069-3076), delta clamp (:3086-3087), off-policy and
    entropy-quantile masks (:3039-3052, 3020-3021, 3111-3115), a given importance
    sampling ratio (:3117-3118) and the static entropy bonus (:3155-3181)."""
    adv = advantages.unsqueeze(1) if advantages.dim() == 1 else advantages
    old = per_token_logps.detach() if old_per_token_logps is None else old_per_token_logps

    entropy_mask = None
    if top_entropy_quantile < 1.0:
        entropy_mask = get_high_entropy_mask(entropies, mask, 1 - top_entropy_quantile)

    off_mask = None
    if off_policy_mask_threshold is not None:
        sampling = old if sampling_per_token_logps is None else sampling_per_token_logps
        off_mask = get_off_policy_mask(adv, per_token_logps, sampling, mask, off_policy_mask_threshold)

    log_ratio = per_token_logps - old
    if importance_sampling_level == "token":
        log_w = log_ratio
    elif importance_sampling_level == "sequence":
        log_w = ((log_ratio * mask).sum(-1) / mask.sum(-1).clamp(min=1.0)).unsqueeze(-1)
    else:
        raise ValueError(f"Unknown importance sampling level: {importance_sampling_level}")
    coef_1 = log_w.exp()

    per_token_kl = None
    if beta != 0.0:
        # the difference is formed twice, as in the reference: with low-precision log-probs each
        # use is a separate cast in autograd and the gradient contributions are rounded separately
        per_token_kl = (
            torch.exp(ref_per_token_logps - per_token_logps) - (ref_per_token_logps - per_token_logps) - 1
        )
        if use_bias_correction_kl:
            per_token_kl = per_token_kl * coef_1

    phi_seq = None
    if loss_type == "cispo":  # (:3080-3082)
        per_token_loss = -coef_1.clamp(max=epsilon_high).detach() * adv * per_token_logps
    elif loss_type in ("grpo", "bnpo", "dr_grpo", "dapo", "luspo"):  # (:3083-3091)
        coef_2 = coef_1.clamp(1 - epsilon_low, 1 + epsilon_high)
        if delta is not None:
            coef_1 = coef_1.clamp(max=delta)
        per_token_loss = -torch.min(coef_1 * adv, coef_2 * adv)
    elif loss_type == "sapo":  # (:3092-3095)
        temps = torch.where(adv > 0, sapo_temperature_pos, sapo_temperature_neg)
        per_token_loss = -(torch.sigmoid(temps * (coef_1 - 1)) * 4 / temps) * adv
    elif loss_type == "vespo":  # (:3096-3107)
        phi_seq = get_gamma_weights(adv, log_ratio, mask, importance_sampling_ratio, *vespo_params)
        per_token_loss = -phi_seq * adv * per_token_logps
    else:
        raise ValueError(f"Unknown loss type: {loss_type}")

    if off_mask is not None:
        per_token_loss = per_token_loss * off_mask
    if entropy_mask is not None:
        per_token_loss = per_token_loss * entropy_mask
    if importance_sampling_ratio is not None and loss_type != "vespo":  # vespo folds it into phi (:3117)
        per_token_loss = per_token_loss * importance_sampling_ratio
    if beta != 0.0:
        per_token_loss = per_token_loss + beta * per_token_kl

    # policy_loss is taken before the division by the gradient-accumulation steps (:3127, 3132, 3137, 3142)
    if loss_type in ("grpo", "sapo"):
        loss = ((per_token_loss * mask).sum(-1) / mask.sum(-1).clamp(min=1.0)).mean()
        normalizer = grad_accum_steps
        policy_loss = loss.detach()
        loss = loss / normalizer
    elif loss_type == "luspo":  # (:3143-3148): no mask on the per-token term
        loss = (per_token_loss * mask.sum(1, keepdim=True)).mean()
        normalizer = grad_accum_steps
        policy_loss = loss.detach()
        loss = loss / normalizer
    elif loss_type == "bnpo":
        loss = (per_token_loss * mask).sum() / mask.sum().clamp(min=1.0)
        normalizer = grad_accum_steps
        policy_loss = loss.detach()
        loss = loss / normalizer
    elif loss_type == "dr_grpo":
        loss = (per_token_loss * mask).sum() / (per_token_loss.size(0) * max_completion_length)
        normalizer = grad_accum_steps
        policy_loss = loss.detach()
        loss = loss / normalizer
    else:  # dapo, cispo, vespo
        n_items = num_items_in_batch
        if not torch.is_tensor(n_items):
            n_items = torch.tensor(float(n_items))
        normalizer = n_items.clamp(min=1.0) / num_processes
        loss = (per_token_loss * mask).sum() / normalizer
        policy_loss = loss.detach()

    metrics: dict[str, float] = {}
    ad = adaptive_entropy
    if entropy_coef != 0.0 or ad is not None:
        eff = mask if entropy_mask is None else mask * entropy_mask
        if loss_type in ("dapo", "cispo", "vespo"):
            ent_term = (entropies * eff).sum() / normalizer
        else:
            ent_term = (entropies * eff).sum() / eff.sum().clamp(min=1.0) / normalizer
        # adaptive control applies the coefficient only while the last window's entropy is at or below the target (:3176-3179)
        apply_coef = entropy_coef if ad is None or ad["last_world_entropy"] <= ad["target"] else 0.0
        loss = loss - apply_coef * ent_term
        metrics["policy_loss"] = float(policy_loss)
        coef_after = entropy_coef
        sync = True if ad is None else ad.get("sync_gradients", True)
        if ad is not None and ad.get("train", True):  # window accumulation and update at the step boundary (:3186-3210)
            stats = torch.stack([(entropies * eff).sum(), eff.sum().float()]).detach()
            window = stats if ad.get("window") is None else torch.as_tensor(ad["window"], dtype=stats.dtype) + stats
            last = ad["last_world_entropy"]
            if sync:
                last = float(window[0] / window[1].clamp(min=1.0))
                if last <= ad["target"]:
                    coef_after = min(entropy_coef + ad["delta"], ad["max"])
                else:
                    coef_after = max(entropy_coef - ad["delta"], ad["min"])
                window = None
            metrics["state/entropy_coef"] = float(coef_after)
            metrics["state/last_world_entropy"] = float(last)
            metrics["state/window"] = None if window is None else [float(x) for x in window]
        if sync:
            metrics["entropy_coef"] = float(coef_after)  # logged at optimizer-step boundaries (:3214-3215)

    def seq_mean(x):
        if x.shape[1] == 1:
            return x.squeeze(1)
        return (x * mask).sum(-1) / mask.sum(-1)  # unclamped: NaN for empty rows (:3227)

    def global_mean(x):
        if x.shape[1] == 1:
            s, c = x.sum(), torch.tensor(float(x.shape[0]))
        else:
            s, c = (x * mask).sum(), mask.sum().float()
        return float(s / c.clamp(min=1.0))

    if beta != 0.0:
        metrics["kl"] = global_mean(per_token_kl.detach())
    if entropies is not None:
        metrics["entropy"] = global_mean(entropies.detach())
    if loss_type in ("grpo", "bnpo", "dr_grpo", "dapo", "luspo"):
        low = ((coef_1 < 1 - epsilon_low) & (adv < 0)).float()
        high = ((coef_1 > 1 + epsilon_high) & (adv > 0)).float()
        region = ((low + high) > 0).float()
        metrics["clip_ratio/low_mean"] = global_mean(low)
        metrics["clip_ratio/high_mean"] = global_mean(high)
        metrics["clip_ratio/region_mean"] = global_mean(region)
        metrics["clip_ratio/low_min"] = float(nanmin(seq_mean(low)))
        metrics["clip_ratio/high_max"] = float(nanmax(seq_mean(high)))
    elif loss_type == "cispo":
        metrics["cispo_clip_ratio"] = global_mean(((coef_1 > epsilon_high) & (adv > 0)).float())
    elif loss_type == "vespo":
        metrics["vespo/phi_seq_mean"] = global_mean(phi_seq)
    return loss, metrics


# --------------------------------------------------------------------------------------
# A10-A11  DPO                             trl/trainer/dpo_trainer.py:1342-1362, 1396-1435, 1578
# --------------------------------------------------------------------------------------
def dpo_sequence_logps(logits: torch.Tensor, input_ids: torch.Tensor, completion_mask: torch.Tensor):
    """Shift by one (dpo_trainer.py:1344-1346), per-token log-probs (:1347), zero the
    non-completion positions (:1348), sum over the sequence (:1350).  Returns
    `(sequence_logps [B], per_token_logps [B, L-1])`."""
    shift_logits = logits[..., :-1, :]
    shift_labels = input_ids[..., 1:]
    shift_mask = completion_mask[..., 1:]
    tok = selective_log_softmax(shift_logits, shift_labels)
    tok = torch.where(shift_mask == 0, torch.zeros_like(tok), tok)
    return tok.sum(dim=1), tok


def dpo_sigmoid_loss(seq_logps: torch.Tensor, ref_chosen_logps: torch.Tensor, ref_rejected_logps: torch.Tensor, beta: float):
    """Batch layout [chosen; rejected] (dpo_trainer.py:1362).  delta = (pi_c - ref_c) -
    (pi_r - ref_r) (:1397-1402, 1430); loss = mean(-logsigmoid(beta * delta))
    (:1435, 1578).  Metrics as logged at dpo_trainer.py:1634-1653."""
    chosen, rejected = seq_logps.chunk(2, dim=0)
    chosen_lr = chosen - ref_chosen_logps
    rejected_lr = rejected - ref_rejected_logps
    loss = (-F.logsigmoid(beta * (chosen_lr - rejected_lr))).mean()
    c_rew = beta * chosen_lr.detach()
    r_rew = beta * rejected_lr.detach()
    metrics = {
        "rewards/chosen": float(c_rew.mean()),
        "rewards/rejected": float(r_rew.mean()),
        "rewards/accuracies": float((c_rew > r_rew).float().mean()),
        "rewards/margins": float((c_rew - r_rew).mean()),
        "logps/chosen": float(chosen.detach().mean()),
        "logps/rejected": float(rejected.detach().mean()),
    }
    return loss, metrics


def _dpo_scores(chosen_lr, rejected_lr, f_divergence_type, f_alpha):
    """f-divergence scores of the log-ratios (dpo_trainer.py:1402-1429)."""
    if f_divergence_type == "reverse_kl" or (f_divergence_type == "alpha_divergence" and abs(f_alpha - 1.0) < 1e-6):
        return chosen_lr, rejected_lr
    if f_divergence_type == "forward_kl":
        return -torch.exp(-chosen_lr), -torch.exp(-rejected_lr)
    if f_divergence_type == "js_divergence":
        return F.logsigmoid(chosen_lr), F.logsigmoid(rejected_lr)
    if f_divergence_type == "alpha_divergence":
        cap = {torch.float16: 11.0, torch.bfloat16: 80.0, torch.float32: 80.0}[chosen_lr.dtype]
        k = f_alpha - 1.0
        out = []
        for lr in (chosen_lr, rejected_lr):
            out.append(torch.exp(torch.clamp((k * lr).float(), max=cap)).to(lr.dtype) / k)
        return tuple(out)
    raise ValueError(f"Unknown f_divergence_type: {f_divergence_type}")


def dpo_compute_loss(logits, input_ids, completion_mask, ref_chosen_logps, ref_rejected_logps, beta, loss_types=("sigmoid",),
                     loss_weights=None, label_smoothing=0.0, ld_alpha=None, use_weighting=False,
                     f_divergence_type="reverse_kl", f_alpha=1.0, discopop_tau=0.05):
    """`DPOTrainer._compute_loss` after the model call with precomputed reference log-probs
    (dpo_trainer.py:1342-1362 sequence log-probs incl. the `ld_alpha` split, :1397-1431 scores, :1433-1561 the
    fifteen per-pair losses, :1563-1574 WPO weights, :1584-1653 metrics).  Returns `(loss, metrics)`."""
    shift_logits = logits[..., :-1, :]
    labels = input_ids[..., 1:]
    smask = completion_mask[..., 1:]
    tok = selective_log_softmax(shift_logits, labels)
    tok = torch.where(smask == 0, torch.zeros_like(tok), tok)
    if ld_alpha is None:
        seq = tok.sum(dim=1)
    else:  # tokens beyond the shorter completion of the pair count with weight ld_alpha
        pos = smask.cumsum(dim=1)
        lens = smask.sum(dim=1).long()
        c_len, r_len = lens.chunk(2)
        shared = torch.minimum(c_len, r_len).repeat(2).unsqueeze(1)
        head = (pos > 0) & (pos <= shared)
        tail = pos > shared
        seq = (tok * head).sum(dim=1) + ld_alpha * (tok * tail).sum(dim=1)
    chosen, rejected = seq.chunk(2)
    c_lr, r_lr = chosen - ref_chosen_logps, rejected - ref_rejected_logps
    c_sc, r_sc = _dpo_scores(c_lr, r_lr, f_divergence_type, f_alpha)
    d = c_sc - r_sc
    c_n, r_n = (m.sum(dim=1).clamp(min=1.0) for m in completion_mask.chunk(2))
    ls = label_smoothing

    def smoothed(delta):
        return -F.logsigmoid(beta * delta) * (1 - ls) - F.logsigmoid(-beta * delta) * ls

    def sft_loss():
        cm = smask.chunk(2)[0].bool()
        ce = F.cross_entropy(shift_logits.chunk(2)[0][cm], labels.chunk(2)[0][cm])
        return ce.expand(chosen.shape[0])

    def exo():
        eps = torch.tensor(ls)
        qw, ql = torch.sigmoid(beta * d), torch.sigmoid(-beta * d)
        return qw * (F.logsigmoid(beta * d) - torch.log1p(-eps)) + ql * (F.logsigmoid(-beta * d) - torch.log(eps))

    def discopop():
        x = beta * d
        mix = torch.sigmoid(x / discopop_tau)
        return -F.logsigmoid(x) * (1 - mix) + torch.exp(-x) * mix

    per_pair = {
        "sigmoid": lambda: -F.logsigmoid(beta * d),
        "hinge": lambda: torch.relu(1 - beta * d),
        "ipo": lambda: ((c_sc / c_n - r_sc / r_n) - 1 / (2 * beta)) ** 2,
        "exo_pair": exo,
        "nca_pair": lambda: -F.logsigmoid(beta * c_sc) - 0.5 * F.logsigmoid(-beta * c_sc) - 0.5 * F.logsigmoid(-beta * r_sc),
        "robust": lambda: (-(1 - ls) * F.logsigmoid(beta * d) + ls * F.logsigmoid(-beta * d)) / (1 - 2 * ls),
        "bco_pair": lambda: -F.logsigmoid(beta * c_sc) - F.logsigmoid(-beta * r_sc),
        "sppo_hard": lambda: (c_sc - 0.5 / beta) ** 2 + (r_sc + 0.5 / beta) ** 2,
        "aot": lambda: smoothed(torch.sort(chosen - rejected, dim=0)[0]
                                - torch.sort(ref_chosen_logps - ref_rejected_logps, dim=0)[0]),
        "aot_unpaired": lambda: smoothed(torch.sort(c_lr, dim=0)[0] - torch.sort(r_lr, dim=0)[0]),
        "apo_zero": lambda: 1 - torch.sigmoid(beta * c_lr) + torch.sigmoid(beta * r_lr),
        "apo_down": lambda: torch.sigmoid(beta * c_lr) + 1 - torch.sigmoid(beta * d),
        "discopop": discopop,
        "sft": sft_loss,
        "sigmoid_norm": lambda: -F.logsigmoid(beta * (c_sc / c_n - r_sc / r_n)),
    }
    weights = None
    if use_weighting:  # WPO: exp(mean over the completion of logp - log sum_v p_v^2), product over the pair (:1563-1574)
        with torch.no_grad():
            log_denom = torch.logsumexp(2.0 * shift_logits, dim=-1) - 2.0 * torch.logsumexp(shift_logits, dim=-1)
            aligned = (tok - log_denom) * smask
        w = torch.exp(aligned.sum(dim=1) / smask.sum(dim=1).clamp_min(1))
        weights = w.chunk(2)[0] * w.chunk(2)[1]
    loss_weights = [1.0] * len(loss_types) if loss_weights is None else loss_weights
    loss = 0.0
    for name, lw in zip(loss_types, loss_weights):
        if name not in per_pair:
            raise ValueError(f"Unknown loss type: {name}")
        term = per_pair[name]()
        if weights is not None:
            term = term * weights
        loss = loss + term.mean() * lw

    det = shift_logits.detach()
    ent = entropy_from_logits(det)
    n_tok = smask.sum()
    c_logits, r_logits = det.chunk(2)
    c_m, r_m = (m.bool() for m in smask.chunk(2))
    c_rew, r_rew = beta * c_lr.detach(), beta * r_lr.detach()
    hits = (c_logits.argmax(dim=-1) == labels.chunk(2)[0]) & c_m
    metrics = {
        "entropy": float((ent * smask).sum() / n_tok) if n_tok > 0 else 0.0,
        # sums leave the device in the logits dtype, the division happens on the host (:1609-1616)
        "logits/chosen": float(c_logits[c_m].mean(-1).sum()) / float(c_m.sum()) if c_m.any() else 0.0,
        "logits/rejected": float(r_logits[r_m].mean(-1).sum()) / float(r_m.sum()) if r_m.any() else 0.0,
        "mean_token_accuracy": float(hits.sum() / c_m.sum()) if c_m.any() else 0.0,
        "rewards/chosen": float(c_rew.mean()),
        "rewards/rejected": float(r_rew.mean()),
        "rewards/accuracies": float((c_rew > r_rew).float().mean()),
        "rewards/margins": float((c_rew - r_rew).mean()),
        "logps/chosen": float(chosen.detach().mean()),
        "logps/rejected": float(rejected.detach().mean()),
    }
    return loss, metrics


# --------------------------------------------------------------------------------------
# A12  RLOO sequence-level loss            trl/trainer/rloo_trainer.py:1683-1694, 1711-1721
# --------------------------------------------------------------------------------------
def rloo_loss(per_token_logps, completion_mask, old_logps, advantages, epsilon_low: float, epsilon_high: float):
    """Sequence log-prob = sum(logp * mask) (rloo_trainer.py:1683); ratio, clamp, min and
    mean over sequences (:1685-1694); clip metrics (:1711-1721)."""
    seq = (per_token_logps * completion_mask).sum(1)
    coef_1 = (seq - old_logps).exp()
    coef_2 = coef_1.clamp(1 - epsilon_low, 1 + epsilon_high)
    loss = (-torch.min(coef_1 * advantages, coef_2 * advantages)).mean()
    low = ((coef_1 < 1 - epsilon_low) & (advantages < 0)).float()
    high = ((coef_1 > 1 + epsilon_high) & (advantages > 0)).float()
    region = ((low + high) > 0).float()
    metrics = {
        "clip_ratio/low_mean": float(low.mean()),
        "clip_ratio/low_min": float(nanmin(low)),
        "clip_ratio/high_mean": float(high.mean()),
        "clip_ratio/high_max": float(nanmax(high)),
        "clip_ratio/region_mean": float(region.mean()),
    }
    return loss, metrics


# --------------------------------------------------------------------------------------
# KTO  sequence log-probs, KL baseline, loss and logged metrics   trl/trainer/kto_trainer.py:1478-1663
# --------------------------------------------------------------------------------------
def kto_sequence_logps(logits, input_ids, completion_mask):
    """Masked sum of the shifted per-token log-probs in the logits dtype (kto_trainer.py:1506-1509; the same four
    lines serve the KL-estimate and reference passes, :1265-1276, :1323-1327)."""
    tok = selective_log_softmax(logits[:, :-1, :], input_ids[:, 1:])
    tok = torch.where(completion_mask[:, 1:] == 0, torch.zeros_like(tok), tok)
    return tok.sum(-1)


def kto_compute_loss(logits, input_ids, completion_mask, label, ref_logps, kl_logps=None, ref_kl_logps=None, beta=0.1,
                     loss_type="kto", desirable_weight=1.0, undesirable_weight=1.0):
    """`KTOTrainer._compute_loss` (kto_trainer.py:1506-1663) for one process with precomputed reference log-probs.
    Returns `(loss, metrics)` with the logged names."""
    seq = kto_sequence_logps(logits, input_ids, completion_mask)
    lab = torch.as_tensor(label, dtype=torch.bool)
    ci, ri = torch.nonzero(lab).view(-1), torch.nonzero(~lab).view(-1)
    c_lp, r_lp = seq[ci], seq[ri]
    if kl_logps is not None:  # :1549-1553
        kl = (kl_logps - ref_kl_logps).mean().detach().clamp(min=0)
    else:
        kl = torch.zeros(1)
    c_lr, r_lr = c_lp - ref_logps[ci], r_lp - ref_logps[ri]
    if loss_type == "kto":  # :1558-1560, :1576-1577
        c_loss = 1 - torch.sigmoid(beta * (c_lr - kl))
        r_loss = 1 - torch.sigmoid(beta * (kl - r_lr))
    elif loss_type == "apo_zero_unpaired":  # :1561-1564, :1578-1579
        c_loss = 1 - torch.sigmoid(beta * c_lr)
        r_loss = torch.sigmoid(beta * r_lr)
    else:
        raise ValueError(loss_type)
    loss = torch.cat((desirable_weight * c_loss, undesirable_weight * r_loss), 0).nanmean()  # :1586-1589, :1655
    metrics = {"kl": float(kl)}
    with torch.no_grad():
        shift = logits[:, :-1, :].detach()
        mask = completion_mask[:, 1:]
        ent = entropy_from_logits(shift)  # :1594-1603
        total = mask.sum()
        metrics["entropy"] = float((ent * mask).sum() / total) if total > 0 else 0.0
        for name, idx in (("chosen", ci), ("rejected", ri)):  # :1612-1628
            mk = mask[idx]
            if mk.sum() > 0:
                metrics["logits/" + name] = float(shift[idx][mk.bool()].mean(-1).sum()) / float(mk.sum())
        if len(ci) > 0:  # :1633-1647
            metrics["rewards/chosen"] = float((beta * c_lr).nansum()) / len(ci)
            metrics["logps/chosen"] = float(c_lp.nansum()) / len(ci)
        if len(ri) > 0:
            metrics["rewards/rejected"] = float((beta * r_lr).nansum()) / len(ri)
            metrics["logps/rejected"] = float(r_lp.nansum()) / len(ri)
        if len(ci) > 0 and len(ri) > 0:
            metrics["rewards/margins"] = metrics["rewards/chosen"] - metrics["rewards/rejected"]
    return loss, metrics


# --------------------------------------------------------------------------------------
# A13-A14  fused lm_head + log-prob        trl/trainer/utils.py:1291-1424
# --------------------------------------------------------------------------------------
def _head_logits(hidden, w_rows, temperature, softcap, logit_scale):
    """fp32 logits of one vocab slab: matmul in the hidden dtype, widen, scale, optional
    soft-cap, inverse temperature (utils.py:1328-1337)."""
    z = (hidden @ w_rows.to(hidden.dtype).t()).float() * logit_scale
    if softcap is not None:
        z = torch.tanh(z / softcap) * softcap
    return z * (1 / temperature)


def chunked_logprob_naive(hidden, weight, targets, temperature=1.0, softcap=None, logit_scale=1.0):
    """Library-routine form: full `[N, V]` fp32 logits then log_softmax / gather /
    entropy (the expression the reference's own test uses, tests/test_utils.py:1165-1171)."""
    z = _head_logits(hidden, weight, temperature, softcap, logit_scale)
    lp = F.log_softmax(z, dim=-1)
    return lp.gather(-1, targets.unsqueeze(-1)).squeeze(-1), -(lp.exp() * lp).sum(-1)


def chunked_logprob_online(hidden, weight, targets, temperature=1.0, chunk_size=8192, softcap=None, logit_scale=1.0):
    """Vocabulary-slab sweep with running (max, sum e, sum e*z) per row and target pick
    (utils.py:1323-1357).  Returns (logprobs, entropy, log_z), all fp32 [N]."""
    n = hidden.shape[0]
    v = weight.shape[0]
    run_max = torch.full((n,), -math.inf)
    run_s = torch.zeros(n)
    run_u = torch.zeros(n)
    tgt = torch.zeros(n)
    rows = torch.arange(n)
    for lo in range(0, v, chunk_size):
        hi = min(lo + chunk_size, v)
        z = _head_logits(hidden, weight[lo:hi], temperature, softcap, logit_scale)
        new_max = torch.maximum(run_max, z.amax(-1))
        keep = (run_max - new_max).exp()
        e = (z - new_max[:, None]).exp()
        run_s = run_s * keep + e.sum(-1)
        run_u = run_u * keep + (e * z).sum(-1)
        run_max = new_max
        inside = (targets >= lo) & (targets < hi)
        tgt = tgt + z[rows, (targets - lo).clamp(0, hi - lo - 1)] * inside
    log_z = run_max + run_s.log()
    return tgt - log_z, log_z - run_u / run_s, log_z


def chunked_logprob_backward(hidden, weight, targets, log_z, grad_logprobs, temperature=1.0, chunk_size=8192,
                             softcap=None, logit_scale=1.0):
    """Recompute each slab, dz = g * (onehot - p) with p = exp(z - log_z), chain through
    1/T, soft-cap and logit_scale, accumulate dHidden / dW in fp32 and round once to the
    input dtypes (utils.py:1380-1424).  The entropy output carries no gradient (:1368)."""
    n = hidden.shape[0]
    v = weight.shape[0]
    g = grad_logprobs.float()
    d_hidden = torch.zeros(hidden.shape, dtype=torch.float32)
    d_weight = torch.zeros(weight.shape, dtype=torch.float32)
    rows = torch.arange(n)
    for lo in range(0, v, chunk_size):
        hi = min(lo + chunk_size, v)
        w_rows = weight[lo:hi]
        y = (hidden @ w_rows.to(hidden.dtype).t()).float() * logit_scale
        if softcap is not None:
            th = torch.tanh(y / softcap)
            y = th * softcap
        z = y * (1 / temperature)
        dz = -g[:, None] * (z - log_z[:, None]).exp()
        inside = (targets >= lo) & (targets < hi)
        dz[rows, (targets - lo).clamp(0, hi - lo - 1)] += g * inside
        dz = dz * (1 / temperature)
        if softcap is not None:
            dz = dz * (1 - th.pow(2))
        dz = dz * logit_scale
        d_hidden += dz @ w_rows.float()
        d_weight[lo:hi] += dz.t() @ hidden.float()
    return d_hidden.to(hidden.dtype), d_weight.to(weight.dtype)


class ChunkedLogProbOracle(torch.autograd.Function):
    """autograd wrapper with the reference operator's argument order (utils.py:1298-1307)."""

    @staticmethod
    def forward(ctx, last_hidden, weight, targets, temperature, chunk_size, final_logit_softcapping=None, logit_scale=1.0):
        logp, ent, log_z = chunked_logprob_online(
            last_hidden, weight, targets, temperature, chunk_size, final_logit_softcapping, logit_scale
        )
        ctx.save_for_backward(last_hidden, weight, targets, log_z)
        ctx.cfg = (temperature, chunk_size, final_logit_softcapping, logit_scale)
        return logp, ent

    @staticmethod
    def backward(ctx, grad_logprobs, grad_entropy):
        hidden, weight, targets, log_z = ctx.saved_tensors
        t, c, cap, scale = ctx.cfg
        dh, dw = chunked_logprob_backward(hidden, weight, targets, log_z, grad_logprobs, t, c, cap, scale)
        return dh, dw, None, None, None, None, None


# --------------------------------------------------------------------------------------
# A15  row compaction / scatter around the fused head   trl/trainer/utils.py:1452-1481
# --------------------------------------------------------------------------------------
def patch_chunked_rows(hidden_states, labels, completion_mask, weight, temperature, chunk_size,
                       softcap=None, logit_scale=1.0):
    """Shift (utils.py:1452-1453), keep completion rows only (:1461-1465), run the fused
    head on them, scatter into zero-filled `[B, S-1]` outputs (:1477-1481)."""
    hs = hidden_states[:, :-1, :]
    lab = labels[:, 1:]
    b, s, h = hs.shape
    flat_h = hs.reshape(b * s, h)
    flat_t = lab.reshape(b * s)
    keep = None
    if completion_mask is not None:
        keep = completion_mask[:, 1:].bool().reshape(b * s)
        flat_h, flat_t = flat_h[keep], flat_t[keep]
    lp_v, ent_v = ChunkedLogProbOracle.apply(flat_h, weight, flat_t, temperature, chunk_size, softcap, logit_scale)
    if keep is None:
        return lp_v.reshape(b, s), ent_v.reshape(b, s)
    lp = torch.zeros(b * s, dtype=lp_v.dtype)
    ent = torch.zeros(b * s, dtype=ent_v.dtype)
    lp[keep] = lp_v
    ent[keep] = ent_v
    return lp.reshape(b, s), ent.reshape(b, s)


# --------------------------------------------------------------------------------------
# SFT chunked cross-entropy              trl/trainer/sft_trainer.py:99-234
# --------------------------------------------------------------------------------------
def chunked_cross_entropy_loss(hidden_states, lm_head_weight, chunk_size, labels=None, shift_labels=None,
                               num_items_in_batch=None, logit_scale=1.0, final_logit_softcapping=None, lm_head_bias=None):
    """Shift (or take pre-shifted labels) (sft_trainer.py:175-180), drop `-100` rows, and over token
    chunks of `chunk_size` accumulate fp32 NLL sum, argmax hits and entropy sum (`_chunk`, :99-114);
    loss = sum / num_items_in_batch, or / n_valid (:228-233).  Returns (loss, correct, entropy_sum, n_valid)."""
    if shift_labels is not None:
        hidden = hidden_states.reshape(-1, hidden_states.size(-1))
        lab = shift_labels.reshape(-1)
    else:
        hidden = hidden_states[..., :-1, :].reshape(-1, hidden_states.size(-1))
        lab = labels[..., 1:].reshape(-1)
    keep = lab != -100
    n_valid = keep.sum()
    if int(n_valid) == 0:
        zero = torch.zeros((), dtype=torch.float32)
        loss = (hidden_states.float().sum() + lm_head_weight.float().sum()) * 0.0
        if lm_head_bias is not None:
            loss = loss + lm_head_bias.float().sum() * 0.0
        return loss, zero, zero.clone(), n_valid
    hidden, lab = hidden[keep], lab[keep]
    loss = torch.zeros((), dtype=torch.float32)
    correct = torch.zeros((), dtype=torch.float32)
    entropy_sum = torch.zeros((), dtype=torch.float32)
    for lo in range(0, hidden.shape[0], chunk_size):
        z = hidden[lo : lo + chunk_size].float() @ lm_head_weight.float().t()
        if lm_head_bias is not None:  # sft_trainer.py:102-103
            z = z + lm_head_bias.float()
        if logit_scale != 1.0:
            z = z * logit_scale
        if final_logit_softcapping is not None:
            z = final_logit_softcapping * torch.tanh(z / final_logit_softcapping)
        lp = F.log_softmax(z, dim=-1)
        tgt = lab[lo : lo + chunk_size]
        loss = loss + F.nll_loss(lp, tgt, reduction="sum")
        correct = correct + (z.argmax(-1) == tgt).sum().float()
        entropy_sum = entropy_sum + (-(lp.exp() * lp).sum(-1)).sum()
    denom = n_valid if num_items_in_batch is None else num_items_in_batch
    return loss / denom, correct, entropy_sum, n_valid


# --------------------------------------------------------------------------------------
# Fused-linear operator contracts          trl/trainer/grpo_trainer.py:2885-2907, dpo_trainer.py:1287-1327
# --------------------------------------------------------------------------------------
def fused_linear_grpo_loss(hidden, weight, selected_token_ids, loss_mask, advantages, temperature=1.0,
                           old_per_token_logps=None, ref_per_token_logps=None, vllm_is_ratio=None, bias=None,
                           **loss_kwargs):
    """What `compute_liger_loss` expects of `self.liger_loss` (grpo_trainer.py:2885-2901), stated with the
    reference's own arithmetic: logits `(hidden @ W.T).float() / T` of every position (utils.py:1328-1337 without
    chunking), `selective_log_softmax`, then `_compute_loss`'s loss (`grpo_loss` above, not divided by the
    accumulation steps, dapo normaliser = active tokens of the batch).  Returns `(loss, [mean_kl]? + [clip_ratio])`
    with clip_ratio = the region clip ratio.  `bias` is the `lm_head` bias (`nn.Linear`: `x @ W.T + b`)."""
    b, t, h = hidden.shape
    logits = hidden.reshape(b * t, h) @ weight.t()
    if bias is not None:
        logits = logits + bias
    logits = logits.float() / temperature
    logps = selective_log_softmax(logits, selected_token_ids.reshape(b * t)).view(b, t)
    beta = loss_kwargs.get("beta", 0.0)
    loss, metrics = grpo_loss(
        logps, advantages, loss_mask, old_per_token_logps=old_per_token_logps,
        ref_per_token_logps=ref_per_token_logps, num_items_in_batch=loss_mask.sum().float(),
        importance_sampling_ratio=vllm_is_ratio, grad_accum_steps=1.0, **loss_kwargs)
    out = [metrics["kl"]] if beta != 0.0 else []
    out.append(metrics.get("clip_ratio/region_mean", float("nan")))
    return loss, out


def fused_linear_dpo_loss(weight, hidden, target, ref_hidden, ref_weight, beta, ignore_index=-100, bias=None,
                          ref_bias=None, loss_type="sigmoid"):
    """What `_compute_loss_liger` expects of `self.liger_loss` (dpo_trainer.py:1287-1301):
    summed log-probs of the non-ignored targets (as dpo_trainer.py:1347-1350), reference ones without grad,
    `dpo_sigmoid_loss` above (other loss types: `dpo_compute_loss` above on the same logits).  Returns `(loss, (chosen_logps, rejected_logps, chosen_logits_mean,
    rejected_logits_mean, nll_loss, chosen_rewards, rejected_rewards))`; the logits means run over all
    positions and the whole vocabulary."""
    b, t, h = hidden.shape
    keep = target != ignore_index
    labels = torch.where(keep, target, torch.zeros_like(target))

    def seq_logps(hs, w, bi):
        logits = hs.reshape(b * t, h) @ w.t()
        if bi is not None:
            logits = logits + bi
        logits = logits.float()
        tok = selective_log_softmax(logits, labels.reshape(b * t)).view(b, t)
        return (tok * keep).sum(-1), logits.view(b, t, -1)

    seq, logits = seq_logps(hidden, weight, bias)
    with torch.no_grad():
        ref_seq, _ = seq_logps(ref_hidden, ref_weight, ref_bias)
    pairs = b // 2
    if loss_type == "sigmoid":
        loss, _ = dpo_sigmoid_loss(seq, ref_seq[:pairs], ref_seq[pairs:], beta)
    else:  # undo the shift `dpo_compute_loss` applies: a dummy last position, a dummy first label
        pad_l = torch.zeros(b, 1, logits.shape[-1], dtype=logits.dtype)
        pad_i = torch.zeros(b, 1, dtype=labels.dtype)
        loss, _ = dpo_compute_loss(torch.cat([logits, pad_l], 1), torch.cat([pad_i, labels], 1),
                                   torch.cat([pad_i, keep.to(labels.dtype)], 1), ref_seq[:pairs], ref_seq[pairs:], beta,
                                   loss_types=(loss_type,))
    rewards = beta * (seq.detach() - ref_seq)
    metrics = (seq.detach()[:pairs], seq.detach()[pairs:], logits.detach()[:pairs].mean(), logits.detach()[pairs:].mean(),
               torch.zeros(()), rewards[:pairs], rewards[pairs:])
    return loss, metrics


def fused_linear_kto_loss(weight, hidden, target, preference_labels, ref_hidden, ref_weight, beta, kl=None,
                          ignore_index=-100, bias=None, ref_bias=None):
    """What `KTOTrainer._compute_loss_liger` expects of `self.liger_loss` (kto_trainer.py:1415-1435), stated with the
    reference's own `kto` arithmetic (`kto_compute_loss` above, unit class weights) on naive logits.  Returns
    `(loss, (chosen_logps_sum, rejected_logps_sum, chosen_logits_sum, rejected_logits_sum, chosen_rewards_sum,
    rejected_rewards_sum))`; a sequence's logits entry is its mean logit over positions and vocabulary."""
    b, t, h = hidden.shape
    keep = target != ignore_index
    labels = torch.where(keep, target, torch.zeros_like(target))

    def logits_of(hs, w, bi):
        z = hs.reshape(b * t, h) @ w.t()
        return (z if bi is None else z + bi).float().view(b, t, -1)

    logits = logits_of(hidden, weight, bias)
    pad_l = torch.zeros(b, 1, logits.shape[-1])
    pad_i = torch.zeros(b, 1, dtype=labels.dtype)
    ids, cm = torch.cat([pad_i, labels], 1), torch.cat([pad_i, keep.to(labels.dtype)], 1)
    with torch.no_grad():
        ref_seq = kto_sequence_logps(torch.cat([logits_of(ref_hidden, ref_weight, ref_bias), pad_l], 1), ids, cm)
    zero = torch.zeros(b)
    kl_pair = (None, None) if kl is None else (zero + kl, zero)  # mean(kl_logps - ref_kl_logps) = kl
    loss, _ = kto_compute_loss(torch.cat([logits, pad_l], 1), ids, cm, preference_labels, ref_seq, *kl_pair, beta=beta)
    with torch.no_grad():
        seq = kto_sequence_logps(torch.cat([logits, pad_l], 1), ids, cm)
        c = torch.as_tensor(preference_labels, dtype=torch.bool).float()
        lm = logits.mean(dim=(1, 2))
        rew = beta * (seq - ref_seq)
        sums = ((seq * c).sum(), (seq * (1 - c)).sum(), (lm * c).sum(), (lm * (1 - c)).sum(), (rew * c).sum(),
                (rew * (1 - c)).sum())
    return loss, sums

"""Writes the golden fixtures in this directory by running the *reference* implementation.

Run only in the development container (needs the reference tree, default
/root/reference; nothing here runs on the GPU box):

    python tests/golden/make_goldens.py [--reference /root/reference]

The reference's trainer methods are called unbound on a `Mock` trainer -- the pattern
its own tests use (tests/test_grpo_trainer.py:95-108) -- whose `accelerator.gather /
reduce / gather_for_metrics` are the identity and whose "model" is a callable that
returns fixed synthetic logits.  Outputs: loss, logged metrics, per-token log-probs,
entropies and the gradient w.r.t. the logits.  Fixtures are small `.npz` files (plain
arrays, loadable with `allow_pickle=False`) plus a JSON index of the case settings.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from collections import defaultdict
from types import SimpleNamespace
from unittest.mock import Mock

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def _np(t):
    t = t.detach()
    if t.dtype == torch.bfloat16:
        t = t.float()
    return t.cpu().numpy()


def _identity(x, *a, **k):
    return x


def _fake_accelerator():
    acc = Mock()
    acc.gather = _identity
    acc.gather_for_metrics = _identity
    acc.reduce = _identity
    acc.pad_across_processes = _identity
    acc.num_processes = 1
    acc.device = torch.device("cpu")
    acc.sync_gradients = True
    return acc


class _FixedLogitsModel:
    """Stands in for the policy: returns clones of fixed logits, sliced like the batch."""

    def __init__(self, logits):
        self.logits = logits
        self.training = True

    def __call__(self, input_ids=None, **kw):
        return SimpleNamespace(logits=self.logits[: input_ids.shape[0]].clone(), aux_loss=None)


def _lengths_mask(lengths, t):
    return (torch.arange(t)[None, :] < torch.tensor(lengths)[:, None]).long()


# ------------------------------------------------------------------------------------ GRPO
GRPO_CASES = [
    dict(name="dapo_beta0", loss_type="dapo", beta=0.0, eps_low=0.2, eps_high=0.2),
    dict(name="dapo_beta", loss_type="dapo", beta=0.04, eps_low=0.2, eps_high=0.28),
    dict(name="grpo_beta", loss_type="grpo", beta=0.04, eps_low=0.2, eps_high=0.2, grad_accum=2),
    dict(name="dr_grpo_beta", loss_type="dr_grpo", beta=0.04, eps_low=0.1, eps_high=0.3, grad_accum=4),
    dict(name="bnpo_beta", loss_type="bnpo", beta=0.1, eps_low=0.2, eps_high=0.2),
    dict(name="grpo_onpolicy", loss_type="grpo", beta=0.0, eps_low=0.2, eps_high=0.2, on_policy=True),
    dict(name="dapo_delta", loss_type="dapo", beta=0.04, eps_low=0.2, eps_high=0.2, delta=1.05),
    dict(name="grpo_seq_is", loss_type="grpo", beta=0.04, eps_low=0.05, eps_high=0.05, is_level="sequence"),
    dict(name="dapo_bf16", loss_type="dapo", beta=0.04, eps_low=0.2, eps_high=0.2, dtype="bfloat16", temperature=0.9),
    dict(name="grpo_temp", loss_type="grpo", beta=0.04, eps_low=0.2, eps_high=0.2, temperature=0.7),
    dict(name="dapo_biaskl", loss_type="dapo", beta=0.04, eps_low=0.2, eps_high=0.2, bias_kl=True),
    dict(name="grpo_offpolicy", loss_type="grpo", beta=0.0, eps_low=0.2, eps_high=0.2, off_policy=0.02),
    dict(name="dapo_entq", loss_type="dapo", beta=0.0, eps_low=0.2, eps_high=0.2, top_entropy_quantile=0.5),
    dict(name="grpo_entbonus", loss_type="grpo", beta=0.04, eps_low=0.2, eps_high=0.2, entropy_coef=0.01),
    dict(name="dapo_entbonus", loss_type="dapo", beta=0.0, eps_low=0.2, eps_high=0.2, entropy_coef=0.02),
    dict(name="dapo_emptyrow", loss_type="dapo", beta=0.04, eps_low=0.2, eps_high=0.2, empty_row=True),
    dict(name="grpo_entbonus_ga", loss_type="grpo", beta=0.04, eps_low=0.2, eps_high=0.2, entropy_coef=0.01, grad_accum=4),
    dict(name="bnpo_entbonus_ga", loss_type="bnpo", beta=0.0, eps_low=0.2, eps_high=0.2, entropy_coef=0.02, grad_accum=2),
    dict(name="dr_grpo_entq_bonus", loss_type="dr_grpo", beta=0.04, eps_low=0.2, eps_high=0.2, entropy_coef=0.02,
         top_entropy_quantile=0.6, grad_accum=2),
    dict(name="cispo", loss_type="cispo", beta=0.04, eps_low=0.2, eps_high=1.1),
    dict(name="sapo", loss_type="sapo", beta=0.0, eps_low=0.2, eps_high=0.2, grad_accum=2),
    dict(name="sapo_beta_seq", loss_type="sapo", beta=0.04, eps_low=0.2, eps_high=0.2, is_level="sequence"),
    dict(name="vespo", loss_type="vespo", beta=0.04, eps_low=0.2, eps_high=0.2),
    dict(name="luspo_seq", loss_type="luspo", beta=0.0, eps_low=0.05, eps_high=0.05, is_level="sequence", grad_accum=2),
    dict(name="dapo_seq_is", loss_type="dapo", beta=0.04, eps_low=0.03, eps_high=0.04, is_level="sequence", bias_kl=True),
    dict(name="bnpo_seq_delta", loss_type="bnpo", beta=0.0, eps_low=0.03, eps_high=0.04, is_level="sequence", delta=1.02),
    dict(name="grpo_seq_offpolicy_entq", loss_type="grpo", beta=0.04, eps_low=0.05, eps_high=0.05, is_level="sequence",
         off_policy=0.02, top_entropy_quantile=0.5),
    dict(name="adaptive_below_target", loss_type="grpo", beta=0.04, eps_low=0.2, eps_high=0.2, entropy_coef=0.01,
         adaptive=dict(target=5.0, delta=0.005, max=0.012, min=0.0, last=1.0, sync=True)),
    dict(name="adaptive_above_target", loss_type="dapo", beta=0.0, eps_low=0.2, eps_high=0.2, entropy_coef=0.02,
         adaptive=dict(target=0.5, delta=0.005, max=0.1, min=0.0, last=float("inf"), sync=True)),
    dict(name="adaptive_accumulating", loss_type="bnpo", beta=0.0, eps_low=0.2, eps_high=0.2, entropy_coef=0.02,
         grad_accum=2, adaptive=dict(target=5.0, delta=0.005, max=0.1, min=0.0, last=2.0, sync=False, window=[3.0, 2.0])),
    dict(name="adaptive_window_close", loss_type="dr_grpo", beta=0.0, eps_low=0.2, eps_high=0.2, entropy_coef=0.0,
         grad_accum=2, adaptive=dict(target=5.0, delta=0.005, max=0.1, min=0.0, last=9.0, sync=True, window=[30.0, 12.0])),
    dict(name="vllm_is_ratio", loss_type="dapo", beta=0.04, eps_low=0.2, eps_high=0.2, is_ratio=True),
    dict(name="vespo_is_ratio", loss_type="vespo", beta=0.0, eps_low=0.2, eps_high=0.2, is_ratio=True),
    # forms whose per-token term is [B, T] where the common configuration has [B, 1]
    dict(name="luspo_token", loss_type="luspo", beta=0.04, eps_low=0.2, eps_high=0.2, grad_accum=2),
    dict(name="luspo_seq_beta", loss_type="luspo", beta=0.04, eps_low=0.05, eps_high=0.05, is_level="sequence", old_noise=0.05),
    dict(name="luspo_seq_is_ratio", loss_type="luspo", beta=0.0, eps_low=0.05, eps_high=0.05, is_level="sequence",
         is_ratio=True, old_noise=0.05),
    dict(name="grpo_seq_is_adv2d", loss_type="grpo", beta=0.04, eps_low=0.05, eps_high=0.05, is_level="sequence",
         adv_2d=True, old_noise=0.05),
    dict(name="vespo_adv2d", loss_type="vespo", beta=0.04, eps_low=0.2, eps_high=0.2, adv_2d=True),
    dict(name="cispo_seq_adv2d", loss_type="cispo", beta=0.0, eps_low=0.2, eps_high=1.02, is_level="sequence", adv_2d=True,
         old_noise=0.05),
]


def _grpo_case(GRPOTrainer, case, seed, dims, lengths, adv_2d=False):
    """Runs the reference's `_compute_loss` (+ backward) on one mocked trainer; returns (arrays, index entry).
    `case["values"]` (optional) names a 16-bit dtype whose values the fp32 logits are rounded to: the reference
    then does fp32 arithmetic on numbers a bf16 / fp16 tensor holds exactly, so a kernel that reads that 16-bit
    tensor and accumulates in fp32 can be compared with these outputs at fp32 tolerance."""
    g = torch.Generator().manual_seed(seed)
    B, P, T, V = dims
    dtype = getattr(torch, case.get("dtype", "float32"))
    temperature = case.get("temperature", 1.0)
    logits = (2.0 * torch.randn(B, P + T, V, generator=g)).to(dtype)
    if case.get("values"):
        logits = logits.to(getattr(torch, case["values"])).to(dtype)
    prompt_ids = torch.randint(0, V, (B, P), generator=g)
    completion_ids = torch.randint(0, V, (B, T), generator=g)
    lengths = list(lengths)
    if case.get("empty_row"):
        lengths[3] = 0
    completion_mask = _lengths_mask(lengths, T)
    prompt_mask = torch.ones(B, P, dtype=torch.long)
    advantages = torch.randn(B, generator=g)
    advantages[1] = 0.0

    trainer = Mock(spec=GRPOTrainer)
    trainer.accelerator = _fake_accelerator()
    trainer.temperature = temperature
    trainer.model_kwarg_keys = set()
    ad = case.get("adaptive")
    trainer._entropy_bonus_enabled = case.get("entropy_coef", 0.0) != 0.0 or ad is not None
    trainer.entropy_coef = case.get("entropy_coef", 0.0)
    trainer.use_adaptive_entropy = ad is not None
    if ad is not None:
        trainer._last_world_entropy = ad["last"]
        trainer._entropy_window_stats = torch.tensor(ad["window"]) if "window" in ad else None
        trainer.accelerator.sync_gradients = ad["sync"]
    trainer.aux_loss_enabled = False
    trainer.top_entropy_quantile = case.get("top_entropy_quantile", 1.0)
    trainer.off_policy_mask_threshold = case.get("off_policy")
    trainer.importance_sampling_level = case.get("is_level", "token")
    trainer.beta = case["beta"]
    trainer.loss_type = case["loss_type"]
    trainer.epsilon_low = case["eps_low"]
    trainer.epsilon_high = case["eps_high"]
    trainer.use_vllm = bool(case.get("is_ratio"))
    trainer.vllm_importance_sampling_correction = bool(case.get("is_ratio"))
    trainer.max_completion_length = T
    trainer.current_gradient_accumulation_steps = case.get("grad_accum", 1)
    trainer.args = SimpleNamespace(delta=case.get("delta"), use_bias_correction_kl=case.get("bias_kl", False),
                                   sapo_temperature_pos=1.0, sapo_temperature_neg=1.05, vespo_k_pos=2.0,
                                   vespo_lambda_pos=3.0, vespo_k_neg=3.0, vespo_lambda_neg=2.0)
    if ad is not None:
        trainer.args.entropy_target, trainer.args.entropy_coef_delta = ad["target"], ad["delta"]
        trainer.args.entropy_coef_max, trainer.args.entropy_coef_min = ad["max"], ad["min"]
    trainer.get_gamma_weights = GRPOTrainer.get_gamma_weights
    trainer._metrics = {"train": defaultdict(list), "eval": defaultdict(list)}
    trainer.model = SimpleNamespace(training=True)
    trainer._get_per_token_logps_and_entropies = (
        lambda *a, **k: GRPOTrainer._get_per_token_logps_and_entropies(trainer, *a, **k)
    )
    trainer.get_high_entropy_mask = lambda *a, **k: GRPOTrainer.get_high_entropy_mask(trainer, *a, **k)
    trainer.get_off_policy_mask = GRPOTrainer.get_off_policy_mask

    # old / ref log-probs: perturbations of the no-grad policy log-probs
    input_ids = torch.cat([prompt_ids, completion_ids], 1)
    attn = torch.cat([prompt_mask, completion_mask], 1)
    with torch.no_grad():
        base_logps, _, _ = GRPOTrainer._get_per_token_logps_and_entropies(
            trainer, _FixedLogitsModel(logits), input_ids, attn, T, compute_entropy=False
        )
    base_logps = base_logps.float()
    inputs = dict(
        prompt_ids=prompt_ids,
        prompt_mask=prompt_mask,
        completion_ids=completion_ids,
        completion_mask=completion_mask,
        advantages=advantages,
        num_items_in_batch=completion_mask.sum().float() * 2.0,  # as if a second, equal micro-batch existed
    )
    if not case.get("on_policy"):
        inputs["old_per_token_logps"] = base_logps + case.get("old_noise", 0.15) * torch.randn(B, T, generator=g)
    if case["beta"] != 0.0:
        inputs["ref_per_token_logps"] = base_logps + 0.3 * torch.randn(B, T, generator=g)
    if case.get("is_ratio"):
        inputs["importance_sampling_ratio"] = 0.5 + torch.rand(B, T, generator=g)
    if case.get("adv_2d"):  # per-token advantages, as subclasses of the trainer provide them (grpo_trainer.py:3026-3030)
        inputs["advantages"] = advantages[:, None] * (0.5 + torch.rand(B, T, generator=g)) - 0.3 * torch.rand(B, T, generator=g)

    leaf = logits.clone().requires_grad_(True)

    class _Model(_FixedLogitsModel):
        def __call__(self, input_ids=None, **kw):
            return SimpleNamespace(logits=leaf[: input_ids.shape[0]] * 1.0, aux_loss=None)

    captured = {}
    real = GRPOTrainer._get_per_token_logps_and_entropies

    def spy(*a, **k):
        out = real(trainer, *a, **k)
        captured["logps"], captured["entropies"] = out[0], out[1]
        return out

    trainer._get_per_token_logps_and_entropies = spy
    loss = GRPOTrainer._compute_loss(trainer, _Model(logits), inputs)
    loss.backward()

    arrays = {}
    arrays["logits"] = _np(logits)
    arrays["prompt_ids"] = _np(prompt_ids)
    arrays["completion_ids"] = _np(completion_ids)
    arrays["completion_mask"] = _np(completion_mask)
    arrays["advantages"] = _np(inputs["advantages"])
    arrays["num_items_in_batch"] = _np(inputs["num_items_in_batch"])
    if "old_per_token_logps" in inputs:
        arrays["old_per_token_logps"] = _np(inputs["old_per_token_logps"])
    if "ref_per_token_logps" in inputs:
        arrays["ref_per_token_logps"] = _np(inputs["ref_per_token_logps"])
    if "importance_sampling_ratio" in inputs:
        arrays["importance_sampling_ratio"] = _np(inputs["importance_sampling_ratio"])
    arrays["out_logps"] = _np(captured["logps"])
    arrays["out_entropies"] = _np(captured["entropies"])
    arrays["out_loss"] = _np(loss)
    arrays["out_dlogits"] = _np(leaf.grad)
    metrics = {k: float(v[-1]) for k, v in trainer._metrics["train"].items()}
    entry = dict(case, id=None, shape=[B, P, T, V], metrics=metrics)
    if ad is not None:  # the controller's state after the call
        win = trainer._entropy_window_stats
        entry["state_after"] = dict(entropy_coef=float(trainer.entropy_coef),
                                    last_world_entropy=float(trainer._last_world_entropy),
                                    window=None if win is None else [float(x) for x in win])
    return arrays, entry


def make_grpo(GRPOTrainer, out_dir):
    index = []
    arrays = {}
    for ci, case in enumerate(GRPO_CASES):
        got, entry = _grpo_case(GRPOTrainer, case, 1000 + ci, (6, 3, 7, 41), [7, 3, 5, 1, 6, 4])
        for k, v in got.items():
            arrays[f"c{ci}_{k}"] = v
        entry["id"] = ci
        index.append(entry)
    np.savez_compressed(os.path.join(out_dir, "grpo_compute_loss.npz"), **arrays)
    with open(os.path.join(out_dir, "grpo_compute_loss.json"), "w") as f:
        json.dump(index, f, indent=1)


# Configurations that one pass over 16-bit logits can serve (a token-level loss type, no mask derived from other
# tokens' log-probs or entropies), on vocabularies that are multiples of 8.  Each runs twice: on logits holding
# bf16-exact values and on logits holding fp16-exact values (fp32 arithmetic in the reference both times).
SINGLE_PASS_CASES = [
    dict(name="dapo_beta0", loss_type="dapo", beta=0.0, eps_low=0.2, eps_high=0.2),
    dict(name="dapo_beta_temp", loss_type="dapo", beta=0.04, eps_low=0.2, eps_high=0.28, temperature=0.9),
    dict(name="grpo_beta_ga", loss_type="grpo", beta=0.04, eps_low=0.2, eps_high=0.2, grad_accum=2, temperature=0.9),
    dict(name="dr_grpo_beta_ga", loss_type="dr_grpo", beta=0.04, eps_low=0.1, eps_high=0.3, grad_accum=4, temperature=0.9),
    dict(name="bnpo_beta", loss_type="bnpo", beta=0.1, eps_low=0.2, eps_high=0.2),
    dict(name="grpo_beta0", loss_type="grpo", beta=0.0, eps_low=0.2, eps_high=0.2),
    dict(name="dr_grpo_beta0", loss_type="dr_grpo", beta=0.0, eps_low=0.2, eps_high=0.2),
    dict(name="bnpo_beta0_ga", loss_type="bnpo", beta=0.0, eps_low=0.05, eps_high=0.05, grad_accum=2),
    dict(name="grpo_onpolicy", loss_type="grpo", beta=0.0, eps_low=0.2, eps_high=0.2, on_policy=True),
    dict(name="dapo_onpolicy_beta", loss_type="dapo", beta=0.04, eps_low=0.2, eps_high=0.2, on_policy=True, temperature=0.7),
    dict(name="dapo_delta", loss_type="dapo", beta=0.04, eps_low=0.2, eps_high=0.2, delta=1.05),
    dict(name="bnpo_delta_beta0", loss_type="bnpo", beta=0.0, eps_low=0.03, eps_high=0.04, delta=1.02),
    dict(name="dapo_biaskl", loss_type="dapo", beta=0.04, eps_low=0.2, eps_high=0.2, bias_kl=True),
    dict(name="grpo_biaskl_delta_temp", loss_type="grpo", beta=0.1, eps_low=0.1, eps_high=0.1, bias_kl=True, delta=1.1,
         temperature=0.8, grad_accum=2),
    dict(name="grpo_entbonus", loss_type="grpo", beta=0.04, eps_low=0.2, eps_high=0.2, entropy_coef=0.01),
    dict(name="dapo_entbonus", loss_type="dapo", beta=0.0, eps_low=0.2, eps_high=0.2, entropy_coef=0.02, temperature=0.9),
    dict(name="bnpo_entbonus_ga", loss_type="bnpo", beta=0.0, eps_low=0.2, eps_high=0.2, entropy_coef=0.02, grad_accum=2),
    dict(name="dr_grpo_entbonus_ga", loss_type="dr_grpo", beta=0.04, eps_low=0.2, eps_high=0.2, entropy_coef=0.02, grad_accum=2),
    dict(name="dapo_emptyrow", loss_type="dapo", beta=0.04, eps_low=0.2, eps_high=0.2, empty_row=True),
    dict(name="grpo_emptyrow_entbonus", loss_type="grpo", beta=0.0, eps_low=0.2, eps_high=0.2, empty_row=True, entropy_coef=0.01),
    dict(name="cispo_beta", loss_type="cispo", beta=0.04, eps_low=0.2, eps_high=1.1),
    dict(name="cispo_beta0_temp", loss_type="cispo", beta=0.0, eps_low=0.2, eps_high=1.05, temperature=0.9),
    dict(name="cispo_entbonus", loss_type="cispo", beta=0.0, eps_low=0.2, eps_high=1.1, entropy_coef=0.02),
    dict(name="sapo_beta0_ga", loss_type="sapo", beta=0.0, eps_low=0.2, eps_high=0.2, grad_accum=2),
    dict(name="sapo_beta_temp", loss_type="sapo", beta=0.04, eps_low=0.2, eps_high=0.2, temperature=0.9),
    dict(name="adaptive_below_target", loss_type="grpo", beta=0.04, eps_low=0.2, eps_high=0.2, entropy_coef=0.01,
         adaptive=dict(target=5.0, delta=0.005, max=0.012, min=0.0, last=1.0, sync=True)),
    dict(name="adaptive_above_target", loss_type="dapo", beta=0.0, eps_low=0.2, eps_high=0.2, entropy_coef=0.02,
         adaptive=dict(target=0.5, delta=0.005, max=0.1, min=0.0, last=float("inf"), sync=True)),
    dict(name="adaptive_accumulating", loss_type="bnpo", beta=0.0, eps_low=0.2, eps_high=0.2, entropy_coef=0.02,
         grad_accum=2, adaptive=dict(target=5.0, delta=0.005, max=0.1, min=0.0, last=2.0, sync=False, window=[3.0, 2.0])),
    dict(name="vllm_is_ratio_dapo", loss_type="dapo", beta=0.04, eps_low=0.2, eps_high=0.2, is_ratio=True),
    dict(name="vllm_is_ratio_cispo", loss_type="cispo", beta=0.0, eps_low=0.2, eps_high=1.1, is_ratio=True, temperature=0.9),
    dict(name="vllm_is_ratio_sapo_entbonus", loss_type="sapo", beta=0.04, eps_low=0.2, eps_high=0.2, is_ratio=True,
         entropy_coef=0.01),
    dict(name="dapo_per_token_advantages", loss_type="dapo", beta=0.04, eps_low=0.2, eps_high=0.28, adv_2d=True),
    # the reference's own 16-bit arithmetic (log-probs rounded to the logits dtype): comparable at 2e-2 only
    dict(name="dapo_true_bf16", loss_type="dapo", beta=0.04, eps_low=0.2, eps_high=0.2, dtype="bfloat16", temperature=0.9),
    dict(name="grpo_true_fp16_entbonus", loss_type="grpo", beta=0.04, eps_low=0.2, eps_high=0.2, dtype="float16",
         entropy_coef=0.01),
]


def make_grpo_single_pass(GRPOTrainer, out_dir):
    index, arrays = [], {}
    vocabs = (48, 264, 56, 72)
    ci = 0
    for k, case in enumerate(SINGLE_PASS_CASES):
        variants = ([None] if "dtype" in case else ["bfloat16", "float16"])
        for j, values in enumerate(variants):
            c = dict(case) if values is None else dict(case, values=values)
            V = vocabs[(k + j) % len(vocabs)]
            got, entry = _grpo_case(GRPOTrainer, c, 6000 + ci, (6, 2, 6, V), [6, 3, 5, 1, 6, 4])
            got["logits"] = got["logits"].astype(np.float32)
            for key, v in got.items():
                arrays[f"c{ci}_{key}"] = v
            entry["id"] = ci
            index.append(entry)
            ci += 1
    np.savez_compressed(os.path.join(out_dir, "grpo_single_pass.npz"), **arrays)
    with open(os.path.join(out_dir, "grpo_single_pass.json"), "w") as f:
        json.dump(index, f, indent=1)


# ------------------------------------------------------------------------------------ DPO
DPO_CASES = [
    dict(name="sigmoid_f32", beta=0.1, dtype="float32"),
    dict(name="sigmoid_beta05", beta=0.5, dtype="float32"),
    dict(name="sigmoid_bf16", beta=0.1, dtype="bfloat16"),
    dict(name="sigmoid_ref_equal", beta=0.1, dtype="float32", ref_equal=True),
    dict(name="hinge", beta=0.1, dtype="float32", loss_types=["hinge"]),
    dict(name="ipo", beta=0.1, dtype="float32", loss_types=["ipo"]),
    dict(name="exo_pair", beta=0.1, dtype="float32", loss_types=["exo_pair"], label_smoothing=0.1),
    dict(name="nca_pair", beta=0.1, dtype="float32", loss_types=["nca_pair"]),
    dict(name="robust", beta=0.1, dtype="float32", loss_types=["robust"], label_smoothing=0.1),
    dict(name="bco_pair", beta=0.1, dtype="float32", loss_types=["bco_pair"]),
    dict(name="sppo_hard", beta=0.1, dtype="float32", loss_types=["sppo_hard"]),
    dict(name="aot", beta=0.1, dtype="float32", loss_types=["aot"], label_smoothing=0.05),
    dict(name="aot_unpaired", beta=0.1, dtype="float32", loss_types=["aot_unpaired"]),
    dict(name="apo_zero", beta=0.1, dtype="float32", loss_types=["apo_zero"]),
    dict(name="apo_down", beta=0.1, dtype="float32", loss_types=["apo_down"]),
    dict(name="discopop", beta=0.1, dtype="float32", loss_types=["discopop"]),
    dict(name="sft", beta=0.1, dtype="float32", loss_types=["sft"]),
    dict(name="sigmoid_norm", beta=0.1, dtype="float32", loss_types=["sigmoid_norm"]),
    dict(name="sigmoid_plus_sft", beta=0.1, dtype="float32", loss_types=["sigmoid", "sft"], loss_weights=[1.0, 0.5]),
    dict(name="ld_alpha", beta=0.1, dtype="float32", ld_alpha=0.5),
    dict(name="wpo", beta=0.1, dtype="float32", use_weighting=True),
    dict(name="wpo_bf16", beta=0.1, dtype="bfloat16", use_weighting=True),
    dict(name="forward_kl", beta=0.1, dtype="float32", f_divergence_type="forward_kl"),
    dict(name="js_divergence", beta=0.1, dtype="float32", f_divergence_type="js_divergence"),
    dict(name="alpha_divergence", beta=0.1, dtype="float32", f_divergence_type="alpha_divergence", f_alpha=0.5),
    dict(name="ipo_ld_alpha_wpo", beta=0.2, dtype="float32", loss_types=["ipo"], ld_alpha=0.3, use_weighting=True),
    dict(name="argmax_ties", beta=0.1, dtype="float32", ties=True),
]


def make_dpo(DPOTrainer, out_dir):
    index, arrays = [], {}
    for ci, case in enumerate(DPO_CASES):
        g = torch.Generator().manual_seed(2000 + ci)
        Pn, L, V = 3, 10, 37
        B = 2 * Pn
        dtype = getattr(torch, case["dtype"])
        logits = (2.0 * torch.randn(B, L, V, generator=g)).to(dtype)
        input_ids = torch.randint(0, V, (B, L), generator=g)
        if ci >= 4:  # later cases: a third of the labels are the arg-max token, so the accuracy metric is exercised
            g2 = torch.Generator().manual_seed(2500 + ci)
            pick = torch.rand(B, L - 1, generator=g2) < 0.33
            input_ids[:, 1:] = torch.where(pick, logits[:, :-1].float().argmax(-1), input_ids[:, 1:])
        if case.get("ties"):  # two equal maxima per row: arg-max is the first one
            top = logits.float().amax(-1) + 1.0
            logits[..., 5] = top.to(dtype)
            logits[..., 20] = top.to(dtype)
            input_ids[:, 1:] = torch.where(torch.arange(L - 1)[None] % 2 == 0, 5, 20)
        prompt_len = [2, 3, 4]
        comp_len = [5, 4, 6, 8, 3, 2]
        completion_mask = torch.zeros(B, L, dtype=torch.long)
        attention_mask = torch.zeros(B, L, dtype=torch.long)
        for i in range(B):
            lp = prompt_len[i % Pn]
            completion_mask[i, lp : lp + comp_len[i]] = 1
            attention_mask[i, : lp + comp_len[i]] = 1

        trainer = Mock(spec=DPOTrainer)
        trainer.accelerator = _fake_accelerator()
        trainer.aux_loss_enabled = False
        trainer.ld_alpha = case.get("ld_alpha")
        trainer.precompute_ref_logps = True
        trainer.f_divergence_type = case.get("f_divergence_type", "reverse_kl")
        trainer.f_alpha_divergence_coef = case.get("f_alpha", 1.0)
        trainer.loss_types = case.get("loss_types", ["sigmoid"])
        trainer.loss_weights = case.get("loss_weights", [1.0] * len(trainer.loss_types))
        trainer.beta = case["beta"]
        trainer.label_smoothing = case.get("label_smoothing", 0.0)
        trainer.use_weighting = case.get("use_weighting", False)
        trainer.args = SimpleNamespace(discopop_tau=0.05)
        trainer._metrics = {"train": defaultdict(list), "eval": defaultdict(list)}
        trainer._total_train_tokens = 0
        trainer.model = SimpleNamespace(training=True)

        leaf = logits.clone().requires_grad_(True)

        def model(**kw):
            return SimpleNamespace(logits=leaf * 1.0, aux_loss=None)

        # reference log-probs: the policy's own sequence log-probs, perturbed
        from trl.trainer.utils import selective_log_softmax as ref_sls

        with torch.no_grad():
            tok = ref_sls(logits[..., :-1, :], input_ids[..., 1:]).float()
            tok = tok * completion_mask[..., 1:]
            seq = tok.sum(1)
        noise = torch.zeros(B) if case.get("ref_equal") else 0.5 * torch.randn(B, generator=g)
        ref = seq + noise
        if case.get("ref_equal"):
            ref = ref.to(dtype)
        inputs = dict(
            input_ids=input_ids,
            attention_mask=attention_mask,
            completion_mask=completion_mask,
            ref_chosen_logps=ref[:Pn],
            ref_rejected_logps=ref[Pn:],
        )
        loss = DPOTrainer._compute_loss(trainer, model, inputs, False)
        loss.backward()
        pre = f"c{ci}_"
        arrays[pre + "logits"] = _np(logits)
        arrays[pre + "input_ids"] = _np(input_ids)
        arrays[pre + "completion_mask"] = _np(completion_mask)
        arrays[pre + "attention_mask"] = _np(attention_mask)
        arrays[pre + "ref_chosen_logps"] = _np(ref[:Pn])
        arrays[pre + "ref_rejected_logps"] = _np(ref[Pn:])
        arrays[pre + "out_loss"] = _np(loss)
        arrays[pre + "out_dlogits"] = _np(leaf.grad)
        metrics = {k: float(v[-1]) for k, v in trainer._metrics["train"].items()}
        index.append(dict(case, id=ci, shape=[B, L, V], metrics=metrics))
    np.savez_compressed(os.path.join(out_dir, "dpo_compute_loss.npz"), **arrays)
    with open(os.path.join(out_dir, "dpo_compute_loss.json"), "w") as f:
        json.dump(index, f, indent=1)


# ------------------------------------------------------------------------------------ KTO
KTO_CASES = [
    dict(name="kto_fp32", dtype="float32", loss_type="kto", beta=0.1, labels=[1, 0, 1, 1, 0, 0], kl=True),
    dict(name="kto_weights", dtype="float32", loss_type="kto", beta=0.25, labels=[1, 0, 0, 1, 0, 0], kl=True,
         desirable_weight=1.33, undesirable_weight=0.8),
    dict(name="kto_negative_kl", dtype="float32", loss_type="kto", beta=0.1, labels=[0, 1, 1, 0, 1, 0], kl=True, kl_shift=-3.0),
    dict(name="apo_zero_unpaired", dtype="float32", loss_type="apo_zero_unpaired", beta=0.1, labels=[1, 0, 1, 0, 1, 0], kl=False),
    dict(name="kto_all_chosen", dtype="float32", loss_type="kto", beta=0.1, labels=[1, 1, 1, 1, 1, 1], kl=True),
    dict(name="kto_all_rejected", dtype="float32", loss_type="apo_zero_unpaired", beta=0.1, labels=[0, 0, 0, 0, 0, 0], kl=False),
    dict(name="kto_bf16", dtype="bfloat16", loss_type="kto", beta=0.1, labels=[1, 0, 1, 1, 0, 0], kl=True),
]


def make_kto(KTOTrainer, out_dir):
    from trl.trainer.utils import selective_log_softmax as ref_sls

    index, arrays = [], {}
    for ci, case in enumerate(KTO_CASES):
        g = torch.Generator().manual_seed(4000 + ci)
        B, L, LK, V = 6, 10, 12, 37
        dtype = getattr(torch, case["dtype"])
        logits = (2.0 * torch.randn(B, L, V, generator=g)).to(dtype)
        kl_logits = (2.0 * torch.randn(B, LK, V, generator=g)).to(dtype)
        input_ids = torch.randint(0, V, (B, L), generator=g)
        kl_input_ids = torch.randint(0, V, (B, LK), generator=g)
        prompt_len, comp_len, kl_comp_len = [2, 3, 4, 1, 2, 5], [5, 4, 6, 8, 3, 2], [4, 7, 3, 9, 5, 6]
        completion_mask = torch.zeros(B, L, dtype=torch.long)
        attention_mask = torch.zeros(B, L, dtype=torch.long)
        kl_completion_mask = torch.zeros(B, LK, dtype=torch.long)
        kl_attention_mask = torch.zeros(B, LK, dtype=torch.long)
        for i in range(B):
            lp = prompt_len[i]
            completion_mask[i, lp : lp + comp_len[i]] = 1
            attention_mask[i, : lp + comp_len[i]] = 1
            kl_completion_mask[i, lp : lp + kl_comp_len[i]] = 1
            kl_attention_mask[i, : lp + kl_comp_len[i]] = 1

        def seq_logps(lg, ids, cm):
            with torch.no_grad():
                tok = ref_sls(lg[:, :-1, :], ids[:, 1:]).float()
                return (tok * cm[:, 1:]).sum(1)

        ref_logps = seq_logps(logits, input_ids, completion_mask) + 0.7 * torch.randn(B, generator=g)
        ref_kl_logps = (seq_logps(kl_logits, kl_input_ids, kl_completion_mask) + 0.3 * torch.randn(B, generator=g)
                        - case.get("kl_shift", 1.5))

        trainer = Mock(spec=KTOTrainer)
        trainer.accelerator = _fake_accelerator()
        trainer.aux_loss_enabled = False
        trainer.use_liger_kernel = False
        trainer.calculate_KL = case["kl"]
        trainer.precompute_ref_logps = True
        trainer.loss_type = case["loss_type"]
        trainer.beta = case["beta"]
        trainer.desirable_weight = case.get("desirable_weight", 1.0)
        trainer.undesirable_weight = case.get("undesirable_weight", 1.0)
        trainer._metrics = {"train": defaultdict(list), "eval": defaultdict(list)}
        trainer._total_train_tokens = 0
        trainer.model = SimpleNamespace(training=True)
        trainer._compute_kl_logps = lambda model, batch, t=trainer: KTOTrainer._compute_kl_logps(t, model, batch)

        leaf = logits.clone().requires_grad_(True)

        def model(input_ids=None, **kw):  # the KL pass is told apart by its sequence length
            if input_ids.shape[1] == LK:
                return SimpleNamespace(logits=kl_logits.clone(), aux_loss=None)
            return SimpleNamespace(logits=leaf * 1.0, aux_loss=None)

        inputs = dict(
            input_ids=input_ids, attention_mask=attention_mask, completion_mask=completion_mask,
            label=torch.tensor(case["labels"], dtype=torch.bool), ref_logps=ref_logps,
        )
        if case["kl"]:
            inputs.update(KL_input_ids=kl_input_ids, KL_attention_mask=kl_attention_mask,
                          KL_completion_mask=kl_completion_mask, ref_KL_logps=ref_kl_logps)
        loss = KTOTrainer._compute_loss(trainer, model, inputs, False)
        loss.backward()
        pre = f"c{ci}_"
        for key, val in dict(logits=logits, kl_logits=kl_logits, input_ids=input_ids, kl_input_ids=kl_input_ids,
                             completion_mask=completion_mask, attention_mask=attention_mask,
                             kl_completion_mask=kl_completion_mask, kl_attention_mask=kl_attention_mask,
                             ref_logps=ref_logps, ref_kl_logps=ref_kl_logps, out_loss=loss, out_dlogits=leaf.grad).items():
            arrays[pre + key] = _np(val)
        metrics = {k: float(v[-1]) for k, v in trainer._metrics["train"].items()}
        index.append(dict(case, id=ci, shape=[B, L, V], kl_len=LK, metrics=metrics))
    np.savez_compressed(os.path.join(out_dir, "kto_compute_loss.npz"), **arrays)
    with open(os.path.join(out_dir, "kto_compute_loss.json"), "w") as f:
        json.dump(index, f, indent=1)


# ------------------------------------------------------------------------------------ RLOO
RLOO_CASES = [
    dict(name="rloo_sym", eps_low=0.2, eps_high=0.2, temperature=1.0),
    dict(name="rloo_asym_temp", eps_low=0.1, eps_high=0.3, temperature=0.8),
]


def make_rloo(RLOOTrainer, out_dir):
    index, arrays = [], {}
    for ci, case in enumerate(RLOO_CASES):
        g = torch.Generator().manual_seed(3000 + ci)
        B, P, T, V = 6, 2, 5, 29
        logits = 2.0 * torch.randn(B, P + T, V, generator=g)
        prompt_ids = torch.randint(0, V, (B, P), generator=g)
        completion_ids = torch.randint(0, V, (B, T), generator=g)
        completion_mask = _lengths_mask([5, 2, 4, 1, 3, 5], T)
        prompt_mask = torch.ones(B, P, dtype=torch.long)
        advantages = torch.randn(B, generator=g)

        trainer = Mock(spec=RLOOTrainer)
        trainer.accelerator = _fake_accelerator()
        trainer.temperature = case["temperature"]
        trainer.model_kwarg_keys = set()
        trainer.aux_loss_enabled = False
        trainer.epsilon_low = case["eps_low"]
        trainer.epsilon_high = case["eps_high"]
        trainer._metrics = {"train": defaultdict(list), "eval": defaultdict(list)}
        trainer.model = SimpleNamespace(training=True)
        trainer._get_per_token_logps_and_entropies = (
            lambda *a, **k: RLOOTrainer._get_per_token_logps_and_entropies(trainer, *a, **k)
        )
        input_ids = torch.cat([prompt_ids, completion_ids], 1)
        attn = torch.cat([prompt_mask, completion_mask], 1)
        with torch.no_grad():
            base, _, _ = RLOOTrainer._get_per_token_logps_and_entropies(
                trainer, _FixedLogitsModel(logits), input_ids, attn, T
            )
        old_logps = (base * completion_mask).sum(1) + 0.2 * torch.randn(B, generator=g)
        leaf = logits.clone().requires_grad_(True)

        def model(input_ids=None, **kw):
            return SimpleNamespace(logits=leaf[: input_ids.shape[0]] * 1.0, aux_loss=None)

        inputs = dict(
            prompt_ids=prompt_ids,
            prompt_mask=prompt_mask,
            completion_ids=completion_ids,
            completion_mask=completion_mask,
            advantages=advantages,
            old_logps=old_logps,
        )
        loss = RLOOTrainer._compute_loss(trainer, model, inputs)
        loss.backward()
        pre = f"c{ci}_"
        for k, v in dict(
            logits=logits, prompt_ids=prompt_ids, completion_ids=completion_ids, completion_mask=completion_mask,
            advantages=advantages, old_logps=old_logps, out_loss=loss, out_dlogits=leaf.grad,
        ).items():
            arrays[pre + k] = _np(v)
        metrics = {k: float(v[-1]) for k, v in trainer._metrics["train"].items()}
        index.append(dict(case, id=ci, shape=[B, P, T, V], metrics=metrics))
    np.savez_compressed(os.path.join(out_dir, "rloo_compute_loss.npz"), **arrays)
    with open(os.path.join(out_dir, "rloo_compute_loss.json"), "w") as f:
        json.dump(index, f, indent=1)


# ------------------------------------------------------------------------------------ fused head
HEAD_CASES = [
    dict(name="plain", temperature=1.0, softcap=None, logit_scale=1.0, dtype="float32", chunk=32),
    dict(name="temp", temperature=0.7, softcap=None, logit_scale=1.0, dtype="float32", chunk=48),
    dict(name="softcap_scale", temperature=0.9, softcap=5.0, logit_scale=0.5, dtype="float32", chunk=32),
    dict(name="bf16", temperature=0.7, softcap=None, logit_scale=1.0, dtype="bfloat16", chunk=32),
]


def make_head(ChunkedFn, out_dir):
    index, arrays = [], {}
    for ci, case in enumerate(HEAD_CASES):
        torch.manual_seed(42)  # the seed the reference's own test uses (tests/test_utils.py:1175)
        N, H, V = 64, 32, 128
        dtype = getattr(torch, case["dtype"])
        hidden = torch.randn(N, H, dtype=dtype, requires_grad=True)
        weight = torch.randn(V, H, dtype=dtype, requires_grad=True)
        labels = torch.randint(0, V, (N,))
        gout = torch.randn(N)
        lp, ent = ChunkedFn.apply(hidden, weight, labels, case["temperature"], case["chunk"], case["softcap"], case["logit_scale"])
        (lp * gout).sum().backward()
        pre = f"c{ci}_"
        for k, v in dict(hidden=hidden, weight=weight, labels=labels, grad_out=gout, out_logprobs=lp, out_entropy=ent,
                         out_dhidden=hidden.grad, out_dweight=weight.grad).items():
            arrays[pre + k] = _np(v)
        index.append(dict(case, id=ci, shape=[N, H, V]))
    np.savez_compressed(os.path.join(out_dir, "chunked_logprob.npz"), **arrays)
    with open(os.path.join(out_dir, "chunked_logprob.json"), "w") as f:
        json.dump(index, f, indent=1)


# ------------------------------------------------------------------------------------ SFT chunked NLL
SFT_CASES = [
    dict(name="labels_mean", dtype="float32", chunk=16, shift=False, nitems=None, softcap=None, scale=1.0),
    dict(name="shift_labels_nitems", dtype="float32", chunk=7, shift=True, nitems=50.0, softcap=None, scale=1.0),
    dict(name="softcap_scale", dtype="float32", chunk=32, shift=False, nitems=None, softcap=4.0, scale=0.5),
    dict(name="bf16", dtype="bfloat16", chunk=16, shift=False, nitems=None, softcap=None, scale=1.0),
    dict(name="bias", dtype="float32", chunk=16, shift=False, nitems=None, softcap=None, scale=1.0, bias=True),
    dict(name="bias_softcap_bf16", dtype="bfloat16", chunk=8, shift=True, nitems=None, softcap=6.0, scale=0.7, bias=True),
]


def make_sft(chunked_ce, out_dir):
    index, arrays = [], {}
    for ci, case in enumerate(SFT_CASES):
        g = torch.Generator().manual_seed(5000 + ci)
        B, S, H, V = 3, 12, 32, 96
        dtype = getattr(torch, case["dtype"])
        hs = torch.randn(B, S, H, generator=g).to(dtype).requires_grad_(True)
        w = (torch.randn(V, H, generator=g) * 0.4).to(dtype).requires_grad_(True)
        labels = torch.randint(0, V, (B, S), generator=g)
        labels[0, :4] = -100
        labels[1, 7:] = -100
        labels[2, 5] = -100
        kw = dict(shift_labels=labels) if case["shift"] else dict(labels=labels)
        bias = None
        if case.get("bias"):  # drawn after everything else, so the earlier cases keep their arrays
            bias = torch.randn(V, generator=g).to(dtype).requires_grad_(True)
            kw["lm_head_bias"] = bias
        loss, correct, ent, nv = chunked_ce(hs, w, case["chunk"], num_items_in_batch=case["nitems"],
                                            logit_scale=case["scale"], final_logit_softcapping=case["softcap"], **kw)
        loss.backward()
        pre = f"c{ci}_"
        for k, v in dict(hidden=hs, weight=w, labels=labels, out_loss=loss, out_correct=correct, out_entropy_sum=ent,
                         out_n_valid=nv, out_dhidden=hs.grad, out_dweight=w.grad).items():
            arrays[pre + k] = _np(v)
        if bias is not None:
            arrays[pre + "bias"], arrays[pre + "out_dbias"] = _np(bias), _np(bias.grad)
        index.append(dict(case, id=ci, shape=[B, S, H, V]))
    np.savez_compressed(os.path.join(out_dir, "sft_chunked_nll.npz"), **arrays)
    with open(os.path.join(out_dir, "sft_chunked_nll.json"), "w") as f:
        json.dump(index, f, indent=1)


# ------------------------------------------------------------------------------------ utils
def make_utils(utils, out_dir):
    """selective_log_softmax / entropy_from_logits on bf16 and fp32 rows, incl. strided views and K > 1."""
    g = torch.Generator().manual_seed(4000)
    arrays = {}
    for tag, dtype in (("f32", torch.float32), ("bf16", torch.bfloat16)):
        logits = (3.0 * torch.randn(3, 9, 257, generator=g)).to(dtype)
        idx = torch.randint(0, 257, (3, 9), generator=g)
        idxk = torch.randint(0, 257, (3, 9, 4), generator=g)
        arrays[f"{tag}_logits"] = _np(logits)
        arrays[f"{tag}_index"] = _np(idx)
        arrays[f"{tag}_index_k"] = _np(idxk)
        arrays[f"{tag}_out_logps"] = _np(utils.selective_log_softmax(logits, idx))
        arrays[f"{tag}_out_logps_k"] = _np(utils.selective_log_softmax(logits, idxk))
        arrays[f"{tag}_out_entropy"] = _np(utils.entropy_from_logits(logits))
        view = logits[:, :-1, :][:, -5:, :]
        arrays[f"{tag}_out_logps_view"] = _np(utils.selective_log_softmax(view, idx[:, -5:]))
        arrays[f"{tag}_out_entropy_view"] = _np(utils.entropy_from_logits(view))
    np.savez_compressed(os.path.join(out_dir, "utils_logps_entropy.npz"), **arrays)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--reference", default="/root/reference")
    ap.add_argument("--out", default=HERE)
    args = ap.parse_args()
    sys.path.insert(0, args.reference)
    import trl.trainer.utils as ref_utils
    from trl.trainer.dpo_trainer import DPOTrainer
    from trl.trainer.grpo_trainer import GRPOTrainer
    from trl.trainer.kto_trainer import KTOTrainer
    from trl.trainer.rloo_trainer import RLOOTrainer

    from trl.trainer.sft_trainer import _chunked_cross_entropy_loss

    make_sft(_chunked_cross_entropy_loss, args.out)
    make_utils(ref_utils, args.out)
    make_head(ref_utils._ChunkedLogProbFunction, args.out)
    make_grpo(GRPOTrainer, args.out)
    make_grpo_single_pass(GRPOTrainer, args.out)
    make_dpo(DPOTrainer, args.out)
    make_rloo(RLOOTrainer, args.out)
    make_kto(KTOTrainer, args.out)
    print("golden fixtures written to", args.out)


if __name__ == "__main__":
    main()

"""Shared pytest configuration: the `gpu` marker, repo root on sys.path, golden loader."""
import json
import os
import sys
from collections import defaultdict
from types import SimpleNamespace

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def load_golden(stem):
    """Returns (cases, arrays): the JSON index (or None) and the npz arrays of one fixture."""
    arrays = np.load(os.path.join(GOLDEN_DIR, stem + ".npz"), allow_pickle=False)
    index_path = os.path.join(GOLDEN_DIR, stem + ".json")
    cases = None
    if os.path.exists(index_path):
        with open(index_path) as f:
            cases = json.load(f)
    return cases, arrays


@pytest.fixture(scope="session")
def golden():
    return load_golden


class IdentityAccelerator:
    """Single-process stand-in for `accelerate.Accelerator`: every collective is the identity."""

    num_processes = 1
    sync_gradients = True

    def gather(self, x):
        return x

    gather_for_metrics = reduce = gather

    def reduce(self, x, reduction="sum"):
        return x

    def pad_across_processes(self, x, dim=0, pad_index=0):
        return x

    def unwrap_model(self, model):
        return model


def fake_grpo_trainer(amd, case, T, skip_masked=False, single_pass=False):
    """A bare object with `GRPOLossMixin`'s methods and the trainer attributes they read, set from one golden case
    (the same attributes the fixture generator sets on its mocked reference trainer)."""
    import torch

    class Trainer(amd.GRPOLossMixin):
        pass

    tr = Trainer()
    tr.accelerator = IdentityAccelerator()
    tr.temperature = case.get("temperature", 1.0)
    tr.model_kwarg_keys = set()
    ad = case.get("adaptive")
    tr._entropy_bonus_enabled = case.get("entropy_coef", 0.0) != 0.0 or ad is not None
    tr.entropy_coef = case.get("entropy_coef", 0.0)
    tr.use_adaptive_entropy = ad is not None
    if ad is not None:
        tr._last_world_entropy = ad["last"]
        tr._entropy_window_stats = torch.tensor(ad["window"]) if "window" in ad else None
        tr.accelerator.sync_gradients = ad["sync"]
    tr.aux_loss_enabled = False
    tr.top_entropy_quantile = case.get("top_entropy_quantile", 1.0)
    tr.off_policy_mask_threshold = case.get("off_policy")
    tr.importance_sampling_level = case.get("is_level", "token")
    tr.beta = case["beta"]
    tr.loss_type = case["loss_type"]
    tr.epsilon_low, tr.epsilon_high = case["eps_low"], case["eps_high"]
    tr.use_vllm = bool(case.get("is_ratio"))
    tr.vllm_importance_sampling_correction = bool(case.get("is_ratio"))
    tr.max_completion_length = T
    tr.current_gradient_accumulation_steps = case.get("grad_accum", 1)
    tr.args = SimpleNamespace(delta=case.get("delta"), use_bias_correction_kl=case.get("bias_kl", False))
    if ad is not None:
        tr.args.entropy_target, tr.args.entropy_coef_delta = ad["target"], ad["delta"]
        tr.args.entropy_coef_max, tr.args.entropy_coef_min = ad["max"], ad["min"]
    tr._metrics = {"train": defaultdict(list), "eval": defaultdict(list)}
    tr.model = SimpleNamespace(training=True)
    tr.trl_amd_skip_masked_rows = skip_masked
    tr.trl_amd_single_pass = single_pass
    return tr

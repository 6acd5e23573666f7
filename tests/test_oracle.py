"""Pins the CPU oracle: golden vectors written by the reference itself (tests/golden),
the reference's own unit-test vectors, torch library routines and closed forms."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from conftest import load_golden


def _t(a, dtype=None):
    t = torch.from_numpy(np.asarray(a))
    return t.to(dtype) if dtype is not None else t


# ----------------------------------------------------------------------------- A1 / A2
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("k", [None, 1, 8])
def test_selective_log_softmax_library_routine(dtype, k):
    # shapes / tolerances of reference tests/test_utils.py:866-905
    torch.manual_seed(0)
    logits = torch.randn(4, 32, 1024, dtype=dtype)
    idx = torch.randint(0, 1024, (4, 32) if k is None else (4, 32, k))
    want = torch.gather(logits.log_softmax(-1), -1, idx.unsqueeze(-1) if k is None else idx)
    want = want.squeeze(-1) if k is None else want
    got = oracle.selective_log_softmax(logits, idx)
    assert got.shape == idx.shape and got.dtype == dtype
    if dtype in (torch.float16, torch.bfloat16):
        assert torch.equal(got, want)
    else:
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("shape", [(768,), (32, 768), (8, 16, 768), (2, 4, 8, 768)])
@pytest.mark.parametrize("chunk_size", [1, 16])
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32, torch.float16, torch.bfloat16])
def test_entropy_library_routine(dtype, chunk_size, shape):
    # reference tests/test_utils.py:615-628
    torch.manual_seed(1)
    logits = torch.randn(*shape, dtype=dtype)
    if dtype in (torch.float64, torch.float32):
        p = logits.softmax(-1)
        want = -(p * p.log()).sum(-1)
    else:
        lp = logits.log_softmax(-1)
        want = -(lp.exp() * lp).sum(-1)
    torch.testing.assert_close(oracle.entropy_from_logits(logits, chunk_size), want, rtol=1e-5, atol=1e-5)


def test_closed_forms_uniform_and_shift():
    v = 513
    flat = torch.full((3, v), 1.25)
    idx = torch.tensor([0, 7, v - 1])
    torch.testing.assert_close(oracle.selective_log_softmax(flat, idx), torch.full((3,), -math.log(v)))
    torch.testing.assert_close(oracle.entropy_from_logits(flat), torch.full((3,), math.log(v)))
    torch.manual_seed(2)
    x = torch.randn(2, 5, 100, dtype=torch.float64)
    i = torch.randint(0, 100, (2, 5))
    torch.testing.assert_close(oracle.selective_log_softmax(x + 3.5, i), oracle.selective_log_softmax(x, i))
    # all-index gather sums to one in probability space
    allidx = torch.arange(100).expand(2, 5, 100)
    torch.testing.assert_close(oracle.selective_log_softmax(x, allidx).exp().sum(-1), torch.ones(2, 5, dtype=torch.float64))
    # H = lse - E_p[z]  (identity used at reference utils.py:1357)
    lse = torch.logsumexp(x, -1)
    torch.testing.assert_close(oracle.entropy_from_logits(x), lse - (x.softmax(-1) * x).sum(-1))
    # two-level distribution: one logit a above the rest
    a, n = 2.0, 50
    row = torch.zeros(1, n, dtype=torch.float64)
    row[0, 3] = a
    z = math.exp(a) + n - 1
    h = math.log(z) - a * math.exp(a) / z
    torch.testing.assert_close(oracle.entropy_from_logits(row), torch.tensor([h], dtype=torch.float64))


def test_f32_variants_match_reference_on_widened_input():
    torch.manual_seed(3)
    x = (2 * torch.randn(3, 6, 300)).bfloat16()
    i = torch.randint(0, 300, (3, 6))
    z = x.float() / 0.9
    torch.testing.assert_close(oracle.selective_log_softmax_f32(x, i, 0.9), oracle.selective_log_softmax(z, i))
    torch.testing.assert_close(oracle.entropy_from_logits_f32(x, 0.9), oracle.entropy_from_logits(z), rtol=1e-5, atol=1e-5)


def test_golden_utils():
    _, g = load_golden("utils_logps_entropy")
    for tag, dtype in (("f32", torch.float32), ("bf16", torch.bfloat16)):
        logits = _t(g[f"{tag}_logits"], dtype)
        idx, idxk = _t(g[f"{tag}_index"]), _t(g[f"{tag}_index_k"])
        exact = dtype == torch.bfloat16
        pairs = [
            (oracle.selective_log_softmax(logits, idx), g[f"{tag}_out_logps"]),
            (oracle.selective_log_softmax(logits, idxk), g[f"{tag}_out_logps_k"]),
            (oracle.entropy_from_logits(logits), g[f"{tag}_out_entropy"]),
            (oracle.selective_log_softmax(logits[:, :-1][:, -5:], idx[:, -5:]), g[f"{tag}_out_logps_view"]),
            (oracle.entropy_from_logits(logits[:, :-1][:, -5:]), g[f"{tag}_out_entropy_view"]),
        ]
        for got, want in pairs:
            want = _t(want)
            if exact:
                assert torch.equal(got.float(), want)
            else:
                torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-6)


# ----------------------------------------------------------------------------- nanstd & co
def test_nanstd_reference_vectors():
    # reference tests/test_utils.py:316-331
    torch.testing.assert_close(oracle.nanstd(torch.tensor([1.0, 2.0, 3.0, float("nan")])), torch.tensor(1.0))
    r = oracle.nanstd(torch.tensor([[1.0, float("nan")], [3.0, 5.0]]), dim=1, keepdim=True)
    assert torch.isnan(r[0, 0])
    torch.testing.assert_close(r[1, 0], torch.tensor(1.4142135), rtol=1e-5, atol=1e-6)
    assert torch.isnan(oracle.nanstd(torch.tensor([float("nan"), float("nan")])))
    x = torch.randn(5, 8)
    torch.testing.assert_close(oracle.nanstd(x, dim=1), x.std(dim=1, unbiased=True))
    assert torch.isnan(oracle.nanmin(torch.tensor([float("nan")])))
    assert oracle.nanmin(torch.tensor([3.0, float("nan"), 1.0])) == 1.0
    assert oracle.nanmax(torch.tensor([3.0, float("nan"), 1.0])) == 3.0


def test_group_advantages_properties():
    torch.manual_seed(4)
    r = torch.randn(24)
    a = oracle.group_advantages(r, 8)
    grp = r.view(-1, 8)
    want = ((grp - grp.mean(1, keepdim=True)) / (grp.std(1, unbiased=True, keepdim=True) + 1e-4)).view(-1)
    torch.testing.assert_close(a, want)
    # zero-variance group -> exactly zero; NaN reward -> zero advantage and excluded from the baseline
    r2 = torch.tensor([1.0, 1.0, 1.0, 1.0, 0.0, float("nan"), 2.0, 4.0])
    a2 = oracle.group_advantages(r2, 4)
    assert torch.equal(a2[:4], torch.zeros(4)) and a2[5] == 0
    m, s = 2.0, math.sqrt(((0 - 2) ** 2 + 0 + (4 - 2) ** 2) / 2)
    torch.testing.assert_close(a2[[4, 6, 7]], torch.tensor([(0 - m) / (s + 1e-4), 0.0, (4 - m) / (s + 1e-4)]))
    torch.testing.assert_close(oracle.group_advantages(r, 8, "none"), (grp - grp.mean(1, keepdim=True)).view(-1))
    torch.testing.assert_close(
        oracle.group_advantages(r, 8, "batch"), (grp - grp.mean(1, keepdim=True)).view(-1) / (r.std() + 1e-4)
    )


def test_rloo_advantages_bruteforce():
    r = torch.tensor([1.0, 2.0, 4.0, 0.5, float("nan"), 2.5])
    a = oracle.rloo_advantages(r, 3)
    want = torch.tensor([1 - 3.0, 2 - 2.5, 4 - 1.5, 0.5 - 2.5, 0.0, 2.5 - 0.5])
    torch.testing.assert_close(a, want)


# ----------------------------------------------------------------------------- masks
def test_vllm_importance_sampling_ratio_closed_forms():
    """trl/trainer/grpo_trainer.py:2578-2623 by hand: log-prob gaps ln2, -ln4, (masked) 5 and 0, ln3."""
    import math

    import trl_amd

    ln = math.log
    old = torch.tensor([[ln(2.0), -ln(4.0), 5.0], [0.0, ln(3.0), 0.0]])
    samp = torch.zeros(2, 3)
    mask = torch.tensor([[1.0, 1.0, 0.0], [1.0, 1.0, 1.0]])
    want = {
        ("token_truncate", 0.5, 2.5): [[2.0, 0.5, 1.0], [1.0, 2.5, 1.0]],
        ("token_mask", 0.5, 2.5): [[2.0, 0.0, 1.0], [1.0, 0.0, 1.0]],
        ("token_mask", None, 2.5): [[2.0, 0.25, 1.0], [1.0, 0.0, 1.0]],
        ("token_truncate", None, 4.0): [[2.0, 0.25, 1.0], [1.0, 3.0, 1.0]],
        ("sequence_truncate", 0.75, 2.0): [[0.75], [2.0]],
        ("sequence_mask", 0.4, 2.0): [[0.5], [0.0]],
        ("sequence_mask", None, None): [[0.5], [3.0]],
    }
    for (mode, lo, hi), expect in want.items():
        got = oracle.vllm_importance_sampling_ratio(old, samp, mask, None, mode, lo, hi)
        torch.testing.assert_close(got, torch.tensor(expect), rtol=1e-6, atol=0)
        ratio, stats = trl_amd.vllm_importance_sampling_ratio(old, samp, mask, None, mode, lo, hi)
        assert torch.equal(ratio, got)
    # a tool mask removes tokens from the ratio and from the statistics
    tool = torch.tensor([[1.0, 0.0, 1.0], [1.0, 1.0, 0.0]])
    got = oracle.vllm_importance_sampling_ratio(old, samp, mask, tool, "sequence_truncate", None, 4.0)
    torch.testing.assert_close(got, torch.tensor([[2.0], [3.0]]), rtol=1e-6, atol=0)
    ratio, stats = trl_amd.vllm_importance_sampling_ratio(old, samp, mask, tool, "token_truncate", None, 2.5)
    torch.testing.assert_close(ratio, torch.tensor([[2.0, 1.0, 1.0], [1.0, 2.5, 1.0]]), rtol=1e-6, atol=0)
    assert abs(float(stats["sampling/sampling_logp_difference/mean"]) - (ln(2.0) + 0.0 + ln(3.0)) / 3) < 1e-6
    assert abs(float(stats["sampling/sampling_logp_difference/max"]) - ln(3.0)) < 1e-6
    assert abs(float(stats["sampling/importance_sampling_ratio/min"]) - 1.0) < 1e-6
    assert abs(float(stats["sampling/importance_sampling_ratio/mean"]) - (2.0 + 1.0 + 2.5) / 3) < 1e-6
    assert abs(float(stats["sampling/importance_sampling_ratio/max"]) - 2.5) < 1e-6
    _, stats = trl_amd.vllm_importance_sampling_ratio(old, samp, torch.zeros(2, 3), None, "token_mask", 0.5, 2.0)
    assert all(float(v) == 0.0 for v in stats.values())
    with pytest.raises(ValueError):
        trl_amd.vllm_importance_sampling_ratio(old, samp, mask, None, "token", None, None)


def test_off_policy_mask_reference_vectors():
    # reference tests/test_grpo_trainer.py:1456-1520
    mask = torch.ones(3, 4)
    adv = torch.tensor([1.0, -1.0, -1.0]).unsqueeze(-1)
    samp = torch.zeros(3, 4)
    lp = torch.zeros(3, 4)
    lp[0], lp[1], lp[2] = -2.0, -0.5, -2.0
    torch.testing.assert_close(oracle.get_off_policy_mask(adv, lp, samp, mask, 1.0), torch.tensor([[1.0], [1.0], [0.0]]))
    mask = torch.tensor([[1.0, 1.0, 0.0, 0.0]])
    adv = torch.tensor([[-1.0]])
    lp = torch.tensor([[-2.0, -2.0, -10000.0, 10000.0]])
    torch.testing.assert_close(oracle.get_off_policy_mask(adv, lp, torch.zeros(1, 4), mask, 1.0), torch.tensor([[0.0]]))
    lp[0, :2] = -0.5
    torch.testing.assert_close(oracle.get_off_policy_mask(adv, lp, torch.zeros(1, 4), mask, 1.0), torch.tensor([[1.0]]))


def test_high_entropy_mask_reference_vectors():
    # reference tests/test_grpo_trainer.py:110-160
    ent = torch.tensor([[0.1, 0.2, 0.3, 0.4, 0.5, 0.6, 0.7, 0.8, 0.9, 1.0, 1.1, 1.2]])
    assert torch.equal(oracle.get_high_entropy_mask(ent, torch.ones_like(ent), 0.8),
                       torch.tensor([[False] * 9 + [True] * 3]))
    ent = torch.tensor([[0.1, 0.2, 0.3, 1.4, 0.5, 0.14], [0.5, 0.6, 0.7, 0.8, 0.9, 1.0]])
    mask = torch.tensor([[1, 1, 1, 1, 1, 0], [1, 1, 1, 1, 1, 0]])
    assert torch.equal(oracle.get_high_entropy_mask(ent, mask, 0.8),
                       torch.tensor([[False, False, False, True, False, False], [False, False, False, False, True, False]]))
    ent = torch.tensor([[0.1, 0.2, 0.3, 0.4, 0.5, 0.6], [0.7, 0.8, 0.9, 1.0, 1.1, 1.2]])
    assert torch.equal(oracle.get_high_entropy_mask(ent, torch.ones_like(ent), 0.0), torch.ones_like(ent, dtype=torch.bool))
    m = oracle.get_high_entropy_mask(ent, torch.ones_like(ent), 1.0)
    assert m.sum() == 1 and m[1, 5]
    assert not oracle.get_high_entropy_mask(ent, torch.zeros_like(ent), 0.5).any()


# ----------------------------------------------------------------------------- GRPO goldens
def _grpo_case(case, g):
    c = f"c{case['id']}_"
    dtype = getattr(torch, case.get("dtype", "float32"))
    B, P, T, V = case["shape"]
    logits = _t(g[c + "logits"], dtype).requires_grad_(True)
    input_ids = torch.cat([_t(g[c + "prompt_ids"]), _t(g[c + "completion_ids"])], 1)
    mask = _t(g[c + "completion_mask"])
    ad = case.get("adaptive")
    ent_bonus = case.get("entropy_coef", 0.0) != 0.0 or ad is not None
    logps, ent = oracle.logps_and_entropies_from_logits(
        logits, input_ids, T, case.get("temperature", 1.0), True, entropy_requires_grad=ent_bonus
    )
    kw = dict(
        entropies=ent,
        old_per_token_logps=_t(g[c + "old_per_token_logps"]) if c + "old_per_token_logps" in g else None,
        ref_per_token_logps=_t(g[c + "ref_per_token_logps"]) if c + "ref_per_token_logps" in g else None,
        loss_type=case["loss_type"], epsilon_low=case["eps_low"], epsilon_high=case["eps_high"], beta=case["beta"],
        delta=case.get("delta"), max_completion_length=T, num_items_in_batch=_t(g[c + "num_items_in_batch"]),
        grad_accum_steps=case.get("grad_accum", 1), importance_sampling_level=case.get("is_level", "token"),
        use_bias_correction_kl=case.get("bias_kl", False), off_policy_mask_threshold=case.get("off_policy"),
        top_entropy_quantile=case.get("top_entropy_quantile", 1.0), entropy_coef=case.get("entropy_coef", 0.0),
        importance_sampling_ratio=_t(g[c + "importance_sampling_ratio"]) if c + "importance_sampling_ratio" in g else None,
    )
    if ad is not None:
        kw["adaptive_entropy"] = dict(last_world_entropy=ad["last"], window=ad.get("window"), target=ad["target"],
                                      delta=ad["delta"], max=ad["max"], min=ad["min"], sync_gradients=ad["sync"])
    loss, metrics = oracle.grpo_loss(logps, _t(g[c + "advantages"]), mask, **kw)
    loss.backward()
    return logits, logps, ent, loss, metrics


def test_golden_grpo_compute_loss():
    cases, g = load_golden("grpo_compute_loss")
    assert len(cases) >= 33
    for case in cases:
        c = f"c{case['id']}_"
        logits, logps, ent, loss, metrics = _grpo_case(case, g)
        if "state_after" in case:  # adaptive entropy controller (grpo_trainer.py:3176-3215)
            want = case["state_after"]
            assert abs(metrics["state/entropy_coef"] - want["entropy_coef"]) < 1e-9, case["name"]
            assert abs(metrics["state/last_world_entropy"] - want["last_world_entropy"]) < 1e-5, case["name"]
            if want["window"] is None:
                assert metrics["state/window"] is None
            else:
                assert max(abs(a - b) for a, b in zip(metrics["state/window"], want["window"])) < 1e-4
            assert ("entropy_coef" in metrics) == ("entropy_coef" in case["metrics"]), case["name"]
        tol = dict(rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(logps.detach().float(), _t(g[c + "out_logps"]), **tol)
        torch.testing.assert_close(ent.detach().float(), _t(g[c + "out_entropies"]), **tol)
        torch.testing.assert_close(loss.detach().float(), _t(g[c + "out_loss"]).float(), **tol)
        torch.testing.assert_close(logits.grad.float(), _t(g[c + "out_dlogits"]), rtol=1e-5, atol=1e-7)
        for name, want in case["metrics"].items():
            got = metrics[name]
            assert (math.isnan(got) and math.isnan(want)) or abs(got - want) <= 1e-6 + 1e-5 * abs(want), (case["name"], name)


def test_grpo_closed_forms():
    torch.manual_seed(5)
    B, T = 4, 6
    lp = (-2 + torch.randn(B, T)).requires_grad_(True)
    adv = torch.tensor([0.7, -0.3, 0.0, 1.1])
    mask = (torch.arange(T)[None] < torch.tensor([6, 2, 4, 1])[:, None]).long()
    # on-policy, beta = 0: loss = -sum(A m)/norm; dL/dlogp = -A m / norm exactly; no clipping
    for lt, norm in (("dapo", float(mask.sum())), ("dr_grpo", B * 9.0), ("bnpo", float(mask.sum()))):
        lp.grad = None
        loss, m = oracle.grpo_loss(lp, adv, mask, loss_type=lt, max_completion_length=9, num_items_in_batch=mask.sum().float())
        loss.backward()
        torch.testing.assert_close(loss.detach(), -(adv[:, None] * mask).sum() / norm)
        torch.testing.assert_close(lp.grad, -(adv[:, None] * mask) / norm)
        assert m["clip_ratio/region_mean"] == 0.0
    lp.grad = None
    loss, _ = oracle.grpo_loss(lp, adv, mask, loss_type="grpo")
    loss.backward()
    torch.testing.assert_close(lp.grad, -(adv[:, None] * mask) / mask.sum(1, keepdim=True) / B)
    # ref == logps: kl = 0 with zero gradient contribution
    lp.grad = None
    loss_b, m = oracle.grpo_loss(lp, adv, mask, loss_type="grpo", beta=0.5, ref_per_token_logps=lp.detach().clone())
    loss_b.backward()
    assert m["kl"] == 0.0
    torch.testing.assert_close(lp.grad, -(adv[:, None] * mask) / mask.sum(1, keepdim=True) / B)
    # entropy bonus invariant (reference tests/test_grpo_trainer.py:1800-1805): (policy_loss - loss)/entropy = coef
    ent = torch.rand(B, T) + 0.5
    loss_e, m = oracle.grpo_loss(lp, adv, mask, loss_type="grpo", entropies=ent, entropy_coef=0.03)
    assert abs((m["policy_loss"] - float(loss_e.detach())) / m["entropy"] - 0.03) < 1e-6


# ----------------------------------------------------------------------------- DPO / RLOO goldens
def _dpo_case_kwargs(case):
    return dict(loss_types=case.get("loss_types", ["sigmoid"]), loss_weights=case.get("loss_weights"),
                label_smoothing=case.get("label_smoothing", 0.0), ld_alpha=case.get("ld_alpha"),
                use_weighting=case.get("use_weighting", False), f_divergence_type=case.get("f_divergence_type", "reverse_kl"),
                f_alpha=case.get("f_alpha", 1.0), discopop_tau=0.05)


def test_golden_dpo_compute_loss():
    """Every case the reference's `DPOTrainer._compute_loss` ran (mocked trainer): loss, dlogits and all ten
    logged metrics, for the fifteen loss types, ld_alpha, WPO weighting, f-divergences and arg-max ties."""
    cases, g = load_golden("dpo_compute_loss")
    assert len(cases) >= 27 and {"aot", "sft", "wpo", "ld_alpha", "argmax_ties"} <= {c["name"] for c in cases}
    for case in cases:
        c = f"c{case['id']}_"
        dtype = getattr(torch, case["dtype"])
        low = dtype != torch.float32
        logits = _t(g[c + "logits"], dtype).requires_grad_(True)
        refc, refr = _t(g[c + "ref_chosen_logps"]), _t(g[c + "ref_rejected_logps"])
        if case.get("ref_equal"):
            refc, refr = refc.to(dtype), refr.to(dtype)
        loss, metrics = oracle.dpo_compute_loss(logits, _t(g[c + "input_ids"]), _t(g[c + "completion_mask"]), refc, refr,
                                                case["beta"], **_dpo_case_kwargs(case))
        loss.backward()
        torch.testing.assert_close(loss.detach().float(), _t(g[c + "out_loss"]).float(), rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(logits.grad.float(), _t(g[c + "out_dlogits"]), rtol=1e-5, atol=1e-8)
        for name, want in case["metrics"].items():
            if name == "num_tokens":
                continue
            tol = 1e-6 + (1e-2 if low and name == "entropy" else 1e-5) * abs(want)
            assert abs(metrics[name] - want) <= tol, (case["name"], name, metrics[name], want)
        if case.get("ref_equal") and dtype == torch.float32:
            # closed form: policy == reference -> ln 2 (tests/invariant/references/dpo.json step 1)
            assert abs(float(loss.detach()) - 0.6931471824645996) < 1e-6
        if case["name"] == "sigmoid_f32":  # the sequence-level pieces agree with the full restatement
            seq, _ = oracle.dpo_sequence_logps(logits.detach(), _t(g[c + "input_ids"]), _t(g[c + "completion_mask"]))
            l2, _ = oracle.dpo_sigmoid_loss(seq, refc, refr, case["beta"])
            assert abs(float(l2.detach()) - float(loss.detach())) < 1e-7


def test_golden_kto_compute_loss():
    """Every case the reference's `KTOTrainer._compute_loss` ran (mocked trainer): kto with the KL baseline (also
    one clamped at 0), weights, apo_zero_unpaired, all-desirable and all-undesirable batches, bf16."""
    cases, g = load_golden("kto_compute_loss")
    assert len(cases) >= 7
    for case in cases:
        c = f"c{case['id']}_"
        dtype = getattr(torch, case["dtype"])
        low = dtype != torch.float32
        logits = _t(g[c + "logits"], dtype).requires_grad_(True)
        kl = ref_kl = None
        if case["kl"]:
            kl = oracle.kto_sequence_logps(_t(g[c + "kl_logits"], dtype), _t(g[c + "kl_input_ids"]),
                                           _t(g[c + "kl_completion_mask"]))
            ref_kl = _t(g[c + "ref_kl_logps"])
        loss, metrics = oracle.kto_compute_loss(
            logits, _t(g[c + "input_ids"]), _t(g[c + "completion_mask"]), case["labels"], _t(g[c + "ref_logps"]), kl,
            ref_kl, case["beta"], case["loss_type"], case.get("desirable_weight", 1.0), case.get("undesirable_weight", 1.0))
        loss.backward()
        torch.testing.assert_close(loss.detach().float(), _t(g[c + "out_loss"]).float(), rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(logits.grad.float(), _t(g[c + "out_dlogits"]), rtol=1e-5, atol=1e-8)
        assert set(metrics) == set(case["metrics"]) - {"num_tokens"}, case["name"]
        for name, got in metrics.items():
            want = case["metrics"][name]
            assert abs(got - want) <= 1e-6 + (1e-2 if low else 1e-5) * abs(want), (case["name"], name, got, want)
        if case["name"] == "kto_negative_kl":
            assert metrics["kl"] == 0.0
    # closed form: policy == reference and KL = 0 -> every loss is 1 - sigmoid(0) = 1/2
    logits = _t(g["c0_logits"])
    seq = oracle.kto_sequence_logps(logits, _t(g["c0_input_ids"]), _t(g["c0_completion_mask"]))
    loss, _ = oracle.kto_compute_loss(logits, _t(g["c0_input_ids"]), _t(g["c0_completion_mask"]), [1, 0, 1, 1, 0, 0], seq)
    assert abs(float(loss.detach()) - 0.5) < 1e-7


def test_golden_rloo_compute_loss():
    cases, g = load_golden("rloo_compute_loss")
    for case in cases:
        c = f"c{case['id']}_"
        B, P, T, V = case["shape"]
        logits = _t(g[c + "logits"]).requires_grad_(True)
        ids = torch.cat([_t(g[c + "prompt_ids"]), _t(g[c + "completion_ids"])], 1)
        logps, _ = oracle.logps_and_entropies_from_logits(logits, ids, T, case["temperature"], True)
        loss, metrics = oracle.rloo_loss(logps, _t(g[c + "completion_mask"]), _t(g[c + "old_logps"]),
                                         _t(g[c + "advantages"]), case["eps_low"], case["eps_high"])
        loss.backward()
        torch.testing.assert_close(loss.detach(), _t(g[c + "out_loss"]), rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(logits.grad, _t(g[c + "out_dlogits"]), rtol=1e-5, atol=1e-8)
        for name, got in metrics.items():
            assert abs(got - case["metrics"][name]) <= 1e-6


# ----------------------------------------------------------------------------- fused head
def test_golden_chunked_logprob():
    cases, g = load_golden("chunked_logprob")
    for case in cases:
        c = f"c{case['id']}_"
        dtype = getattr(torch, case["dtype"])
        hidden = _t(g[c + "hidden"], dtype).requires_grad_(True)
        weight = _t(g[c + "weight"], dtype).requires_grad_(True)
        labels, gout = _t(g[c + "labels"]), _t(g[c + "grad_out"])
        lp, ent = oracle.ChunkedLogProbOracle.apply(hidden, weight, labels, case["temperature"], case["chunk"],
                                                    case["softcap"], case["logit_scale"])
        (lp * gout).sum().backward()
        tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
        torch.testing.assert_close(lp.detach(), _t(g[c + "out_logprobs"]), **tol)
        torch.testing.assert_close(ent.detach(), _t(g[c + "out_entropy"]), **tol)
        torch.testing.assert_close(hidden.grad.float(), _t(g[c + "out_dhidden"]), **tol)
        torch.testing.assert_close(weight.grad.float(), _t(g[c + "out_dweight"]), **tol)


@pytest.mark.parametrize("temperature", [1.0, 0.7])
def test_chunked_logprob_vs_naive_autograd(temperature):
    # reference tests/test_utils.py:1161-1210: N,H,V = 64,32,128, chunk 32, seed 42
    torch.manual_seed(42)
    hidden = torch.randn(64, 32, requires_grad=True)
    weight = torch.randn(128, 32, requires_grad=True)
    labels = torch.randint(0, 128, (64,))
    lp, ent = oracle.ChunkedLogProbOracle.apply(hidden, weight, labels, temperature, 32)
    lp.sum().backward()
    gh, gw = hidden.grad.clone(), weight.grad.clone()
    hidden.grad = weight.grad = None
    lp2, ent2 = oracle.chunked_logprob_naive(hidden, weight, labels, temperature)
    lp2.sum().backward()
    torch.testing.assert_close(lp, lp2, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(ent, ent2, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(gh, hidden.grad, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(gw, weight.grad, atol=1e-5, rtol=1e-5)


def test_patch_chunked_rows_masking():
    # reference tests/test_utils.py:1338-1398: masked == unmasked on completion rows, exact zeros elsewhere
    torch.manual_seed(6)
    B, S, H, V = 2, 9, 16, 50
    hs = torch.randn(B, S, H)
    w = torch.randn(V, H)
    labels = torch.randint(0, V, (B, S))
    cm = torch.zeros(B, S, dtype=torch.long)
    cm[0, 3:7] = 1
    cm[1, 5:] = 1
    lp_m, ent_m = oracle.patch_chunked_rows(hs, labels, cm, w, 0.8, 16)
    lp_u, ent_u = oracle.patch_chunked_rows(hs, labels, None, w, 0.8, 16)
    keep = cm[:, 1:].bool()
    torch.testing.assert_close(lp_m[keep], lp_u[keep])
    torch.testing.assert_close(ent_m[keep], ent_u[keep])
    assert torch.equal(lp_m[~keep], torch.zeros_like(lp_m[~keep])) and torch.equal(ent_m[~keep], torch.zeros_like(ent_m[~keep]))


# ----------------------------------------------------------------------------- SFT chunked NLL
def test_golden_sft_chunked_nll():
    cases, g = load_golden("sft_chunked_nll")
    for case in cases:
        c = f"c{case['id']}_"
        dtype = getattr(torch, case["dtype"])
        hs = _t(g[c + "hidden"], dtype).requires_grad_(True)
        w = _t(g[c + "weight"], dtype).requires_grad_(True)
        labels = _t(g[c + "labels"])
        kw = dict(shift_labels=labels) if case["shift"] else dict(labels=labels)
        bias = _t(g[c + "bias"], dtype).requires_grad_(True) if case.get("bias") else None
        loss, correct, ent, nv = oracle.chunked_cross_entropy_loss(
            hs, w, case["chunk"], num_items_in_batch=case["nitems"], logit_scale=case["scale"],
            final_logit_softcapping=case["softcap"], lm_head_bias=bias, **kw)
        loss.backward()
        tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
        torch.testing.assert_close(loss.detach().float(), _t(g[c + "out_loss"]).float(), **tol)
        assert float(correct) == float(g[c + "out_correct"]) and int(nv) == int(g[c + "out_n_valid"])
        torch.testing.assert_close(ent.detach(), _t(g[c + "out_entropy_sum"]), rtol=1e-5, atol=1e-4)
        torch.testing.assert_close(hs.grad.float(), _t(g[c + "out_dhidden"]), **tol)
        torch.testing.assert_close(w.grad.float(), _t(g[c + "out_dweight"]), **tol)
        if bias is not None:
            torch.testing.assert_close(bias.grad.float(), _t(g[c + "out_dbias"]), **tol)
    assert sum(bool(c.get("bias")) for c in cases) >= 2
    # library routine: mean cross-entropy over the valid positions
    torch.manual_seed(9)
    hs, w = torch.randn(2, 7, 16), torch.randn(40, 16)
    labels = torch.randint(0, 40, (2, 7))
    labels[0, 2] = -100
    loss, _, _, nv = oracle.chunked_cross_entropy_loss(hs, w, 4, labels=labels)
    want = F.cross_entropy((hs[:, :-1] @ w.t()).reshape(-1, 40), labels[:, 1:].reshape(-1), ignore_index=-100)
    torch.testing.assert_close(loss, want)
    # an all-masked batch still yields a differentiable zero
    hs.requires_grad_(True)
    loss, correct, ent, nv = oracle.chunked_cross_entropy_loss(hs, w, 4, labels=torch.full((2, 7), -100))
    loss.backward()
    assert float(loss.detach()) == 0.0 and int(nv) == 0 and torch.count_nonzero(hs.grad) == 0


def test_fused_linear_contracts_reduce_to_closed_forms():
    """The fused-linear oracle functions only compose pinned pieces; what is checked here is the contract of
    the call sites: metric positions (grpo_trainer.py:2900-2901, dpo_trainer.py:1293-1301) and two closed forms
    (policy == reference gives ln 2 and zero rewards; on-policy GRPO has clip ratio 0 and kl 0 when ref == logps)."""
    g = torch.Generator().manual_seed(5)
    P, T, H, V = 3, 7, 16, 29
    hidden = torch.randn(2 * P, T, H, generator=g)
    weight = torch.randn(V, H, generator=g) * 0.3
    target = torch.randint(0, V, (2 * P, T), generator=g)
    target[:, :2] = -100
    loss, m = oracle.fused_linear_dpo_loss(weight, hidden, target, hidden, weight, beta=0.1)
    assert abs(float(loss.detach()) - math.log(2.0)) < 1e-6 and len(m) == 7
    assert torch.equal(m[5], torch.zeros(P)) and torch.equal(m[6], torch.zeros(P)) and float(m[4]) == 0.0
    logits = hidden.reshape(-1, H) @ weight.t()
    assert abs(float(m[2]) - float(logits.view(2 * P, T, V)[:P].mean())) < 1e-6

    ids = torch.randint(0, V, (2 * P, T), generator=g)
    mask = torch.ones(2 * P, T, dtype=torch.long)
    adv = torch.randn(2 * P, generator=g)
    logps = oracle.selective_log_softmax(logits.float(), ids.reshape(-1)).view(2 * P, T)
    loss, m = oracle.fused_linear_grpo_loss(hidden, weight, ids, mask, adv, 1.0, None, logps, None, beta=0.04,
                                            loss_type="bnpo")
    assert len(m) == 2 and abs(m[0]) < 1e-7 and m[1] == 0.0
    assert abs(float(loss.detach()) + float(adv.mean())) < 1e-6  # -(sum A * 1) / tokens
    loss, m = oracle.fused_linear_grpo_loss(hidden, weight, ids, mask, adv, 1.0, beta=0.0, loss_type="bnpo")
    assert len(m) == 1

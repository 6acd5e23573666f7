"""GPU parity of the loss epilogues (K2 GRPO, K2a advantages, K4 DPO / RLOO) against the golden
vectors written by the reference's own `_compute_loss` methods and against the CPU oracle.
Tolerance: losses, metrics and gradients within 1e-3 relative (fp32 cases are far tighter)."""
import math
from collections import defaultdict
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import oracle
from conftest import IdentityAccelerator as _Identity, fake_grpo_trainer as _fake_trainer, load_golden

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _t(a, dtype=None):
    t = torch.from_numpy(np.asarray(a))
    return t.to(dtype) if dtype is not None else t


def _rel_l2(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    return float((got - want).norm() / want.norm().clamp(min=1e-30))


@pytest.fixture(scope="module")
def amd():
    import trl_amd

    return trl_amd


@pytest.mark.parametrize("skip_masked,single_pass", [(False, False), (True, False), (True, True)])
def test_golden_grpo_compute_loss_through_trainer_methods(amd, skip_masked, single_pass):
    """The reference's `GRPOTrainer._compute_loss` ran these inputs on a mocked trainer; the same
    mock drives our mix-in methods on the device.  With `skip_masked` the forward kernel skips the
    rows the completion mask zeroes; loss, metrics and gradients must not change.  With `single_pass` the
    trainer asks for the one-pass kernel: the cases whose configuration it takes go through it (fp32 logits of 41
    entries: rows that are not whole vectors, peeled to their alignment), the others (sequence-level weights,
    masks derived from the log-probs, vespo, luspo) fall back to the two kernels on the logits of the same model
    call.  More reference-written vectors for the one-pass kernel: `grpo_single_pass.*`
    (tests/test_gpu_grpo_single_pass.py)."""
    cases, g = load_golden("grpo_compute_loss")
    ran = 0
    for case in cases:
        c = f"c{case['id']}_"
        B, P, T, V = case["shape"]
        dtype = getattr(torch, case.get("dtype", "float32"))
        tr = _fake_trainer(amd, case, T, skip_masked, single_pass)
        leaf = _t(g[c + "logits"], dtype).to(DEV).requires_grad_(True)
        inputs = dict(
            prompt_ids=_t(g[c + "prompt_ids"]).to(DEV), prompt_mask=torch.ones(B, P, dtype=torch.long, device=DEV),
            completion_ids=_t(g[c + "completion_ids"]).to(DEV), completion_mask=_t(g[c + "completion_mask"]).to(DEV),
            advantages=_t(g[c + "advantages"]).to(DEV), num_items_in_batch=_t(g[c + "num_items_in_batch"]).to(DEV),
        )
        for key in ("old_per_token_logps", "ref_per_token_logps", "importance_sampling_ratio"):
            if c + key in g:
                inputs[key] = _t(g[c + key]).to(DEV)
        model = lambda **kw: SimpleNamespace(logits=leaf, aux_loss=None)  # noqa: E731
        captured = {}
        inner = tr._get_per_token_logps_and_entropies

        def spy(*a, _inner=inner, **k):
            out = _inner(*a, **k)
            captured["lp"], captured["ent"] = out[0], out[1]
            return out

        tr._get_per_token_logps_and_entropies = spy
        loss = tr._compute_loss(model, inputs)
        loss.backward()
        low = dtype != torch.float32
        tol = 2e-3 if low else 1e-5
        # bf16 case: the reference's own log-probs are rounded to bf16, ours are fp32 -> compare to the
        # fp32-op-math oracle on the same stored logits instead, then the reference loss at 1e-3 rel
        if low:
            cpu_logits = _t(g[c + "logits"], dtype)
            ids = torch.cat([_t(g[c + "prompt_ids"]), _t(g[c + "completion_ids"])], 1)
            want_lp = oracle.selective_log_softmax_f32(cpu_logits[:, :-1][:, -T:], ids[:, -T:], tr.temperature)
            want_ent = oracle.entropy_from_logits_f32(cpu_logits[:, :-1][:, -T:], tr.temperature)
        else:
            want_lp, want_ent = _t(g[c + "out_logps"]), _t(g[c + "out_entropies"])
        # (luspo's [B, T] forms average over the padding too, so its rows are never skipped)
        keep = (_t(g[c + "completion_mask"]).float() if skip_masked and case["loss_type"] != "luspo"
                else torch.ones_like(want_lp))
        if captured:  # (the one-pass branch does not go through the log-prob method)
            torch.testing.assert_close(captured["lp"].detach().cpu(), want_lp * keep, atol=tol, rtol=0)
            torch.testing.assert_close(captured["ent"].detach().cpu(), want_ent * keep, atol=tol, rtol=0)
        want_loss = float(g[c + "out_loss"])
        assert abs(float(loss.detach()) - want_loss) <= (2e-2 if low else 1e-5) * max(1.0, abs(want_loss)), case["name"]
        rel = _rel_l2(leaf.grad.float(), _t(g[c + "out_dlogits"]))
        assert rel < (2e-2 if low else 1e-4), (case["name"], rel)
        got_metrics = {k: v[-1] for k, v in tr._metrics["train"].items()}
        for name, want in case["metrics"].items():
            got = got_metrics[name]
            ok = (math.isnan(got) and math.isnan(want)) or abs(got - want) <= (2e-2 if low else 1e-5) * max(1.0, abs(want))
            assert ok, (case["name"], name, got, want)
        if "state_after" in case:  # the adaptive entropy controller's state after the call
            want = case["state_after"]
            assert abs(tr.entropy_coef - want["entropy_coef"]) < 1e-9, case["name"]
            assert abs(tr._last_world_entropy - want["last_world_entropy"]) < 1e-4, case["name"]
            if want["window"] is None:
                assert tr._entropy_window_stats is None
            else:
                torch.testing.assert_close(tr._entropy_window_stats.cpu(), torch.tensor(want["window"]), rtol=1e-5, atol=1e-4)
            assert ("entropy_coef" in got_metrics) == ("entropy_coef" in case["metrics"]), case["name"]
        ran += 1
    assert ran >= 39


def test_grpo_loss_against_oracle_random(amd):
    """Larger random [B, T] problems, all four normalisations, against the oracle's autograd."""
    g = torch.Generator().manual_seed(21)
    B, T = 16, 700
    lp = -3.0 * torch.rand(B, T, generator=g)
    old = lp + 0.3 * torch.randn(B, T, generator=g)
    ref = lp + 0.2 * torch.randn(B, T, generator=g)
    ent = torch.rand(B, T, generator=g) * 3
    adv = torch.randn(B, generator=g)
    lengths = torch.randint(0, T + 1, (B,), generator=g)
    lengths[3] = 0
    mask = (torch.arange(T)[None] < lengths[:, None]).long()
    n_items = mask.sum().float() * 3
    for lt in ("grpo", "bnpo", "dr_grpo", "dapo"):
        for delta in (None, 1.3):
            kw = dict(entropies=ent, old_per_token_logps=old, ref_per_token_logps=ref, loss_type=lt, epsilon_low=0.2,
                      epsilon_high=0.28, beta=0.04, delta=delta, max_completion_length=T, num_items_in_batch=n_items,
                      grad_accum_steps=2.0, entropy_coef=0.01)
            olp = lp.clone().requires_grad_(True)
            oent = ent.clone().requires_grad_(True)
            oloss, ometrics = oracle.grpo_loss(olp, adv, mask, **{**kw, "entropies": oent})
            oloss.backward()
            dlp = lp.to(DEV).requires_grad_(True)
            dent = ent.to(DEV).requires_grad_(True)
            dkw = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in kw.items()}
            dkw["entropies"] = dent
            loss, metrics = amd.grpo_loss(dlp, adv.to(DEV), mask.to(DEV), **dkw)
            loss.backward()
            assert abs(float(loss.detach()) - float(oloss.detach())) <= 1e-5 * max(1.0, abs(float(oloss.detach()))), (lt, delta)
            assert _rel_l2(dlp.grad, olp.grad) < 1e-5, (lt, delta)
            assert _rel_l2(dent.grad, oent.grad) < 1e-5, (lt, delta)
            md = amd.trainer.metrics_to_dict(metrics, 0.04)
            for name, want in ometrics.items():
                if name == "entropy_coef":
                    continue
                assert abs(md[name] - want) <= 1e-5 * max(1.0, abs(want)), (lt, name, md[name], want)
    # the remaining policy terms and sequence-level importance weights
    variants = [("cispo", "token", 0.04), ("cispo", "sequence", 0.0), ("sapo", "token", 0.04), ("sapo", "sequence", 0.04),
                ("vespo", "token", 0.04), ("vespo", "sequence", 0.04), ("luspo", "sequence", 0.0),
                ("grpo", "sequence", 0.04), ("bnpo", "sequence", 0.04), ("dr_grpo", "sequence", 0.0),
                ("dapo", "sequence", 0.04)]
    old_seq = lp + 0.02 * torch.randn(B, T, generator=g)  # sequence means of the token ratios stay near the clip range
    for lt, level, beta in variants:
        for bias_kl in (False, True):
            o = old_seq if level == "sequence" or lt == "vespo" else old
            kw = dict(entropies=ent, old_per_token_logps=o, ref_per_token_logps=ref, loss_type=lt, epsilon_low=0.002,
                      epsilon_high=1.05 if lt == "cispo" else 0.003, beta=beta, max_completion_length=T,
                      num_items_in_batch=n_items, grad_accum_steps=2.0, entropy_coef=0.01,
                      importance_sampling_level=level, use_bias_correction_kl=bias_kl)
            olp = lp.clone().requires_grad_(True)
            oloss, ometrics = oracle.grpo_loss(olp, adv, mask, **kw)
            oloss.backward()
            dlp = lp.to(DEV).requires_grad_(True)
            dkw = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in kw.items()}
            loss, metrics = amd.grpo_loss(dlp, adv.to(DEV), mask.to(DEV), **dkw)
            loss.backward()
            tag = (lt, level, bias_kl)
            assert abs(float(loss.detach()) - float(oloss.detach())) <= 1e-5 * max(1.0, abs(float(oloss.detach()))), tag
            assert _rel_l2(dlp.grad, olp.grad) < 1e-5, tag
            md = amd.trainer.metrics_to_dict(metrics, beta, loss_type=lt)
            for name, want in ometrics.items():
                if name == "entropy_coef":
                    continue
                assert abs(md[name] - want) <= 1e-5 * max(1.0, abs(want)), (tag, name, md[name], want)
    # the [B, T] forms: LUSPO with token-level weights / a KL term (its mean then runs over the padding too), and
    # per-token advantages under sequence-level weights and under vespo
    adv_bt = adv[:, None] * (0.5 + torch.rand(B, T, generator=g)) - 0.2
    for lt, level, beta, a_in, o in (("luspo", "token", 0.0, adv, old), ("luspo", "token", 0.04, adv, old),
                                     ("luspo", "sequence", 0.04, adv, old_seq), ("luspo", "sequence", 0.0, adv_bt, old_seq),
                                     ("grpo", "sequence", 0.04, adv_bt, old_seq), ("cispo", "sequence", 0.0, adv_bt, old_seq),
                                     ("dapo", "token", 0.04, adv_bt, old), ("vespo", "token", 0.04, adv_bt, old_seq)):
        kw = dict(entropies=ent, old_per_token_logps=o, ref_per_token_logps=ref, loss_type=lt, epsilon_low=0.002,
                  epsilon_high=1.05 if lt == "cispo" else 0.003, beta=beta, max_completion_length=T,
                  num_items_in_batch=n_items, grad_accum_steps=2.0, importance_sampling_level=level)
        olp = lp.clone().requires_grad_(True)
        oloss, ometrics = oracle.grpo_loss(olp, a_in, mask, **kw)
        oloss.backward()
        dlp = lp.to(DEV).requires_grad_(True)
        dkw = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in kw.items()}
        loss, metrics = amd.grpo_loss(dlp, a_in.to(DEV), mask.to(DEV), **dkw)
        loss.backward()
        tag = (lt, level, beta, tuple(a_in.shape))
        assert abs(float(loss.detach()) - float(oloss.detach())) <= 1e-5 * max(1.0, abs(float(oloss.detach()))), (tag, float(loss.detach()), float(oloss.detach()))
        assert _rel_l2(dlp.grad, olp.grad) < 1e-5, tag
        md = amd.trainer.metrics_to_dict(metrics, beta, loss_type=lt)
        for name, want in ometrics.items():
            assert abs(md[name] - want) <= 1e-5 * max(1.0, abs(want)), (tag, name, md[name], want)
    # determinism: identical bits on a second call
    a = amd.grpo_loss(lp.to(DEV), adv.to(DEV), mask.to(DEV), loss_type="grpo", old_per_token_logps=old.to(DEV))
    b = amd.grpo_loss(lp.to(DEV), adv.to(DEV), mask.to(DEV), loss_type="grpo", old_per_token_logps=old.to(DEV))
    assert torch.equal(a[0], b[0]) and torch.equal(a[1].nan_to_num(), b[1].nan_to_num())


def test_grpo_on_policy_closed_form(amd):
    # old = logps.detach(): ratio == 1 everywhere -> d loss / d logp = -A * m / norm exactly
    B, T = 8, 33
    g = torch.Generator().manual_seed(22)
    lp = (-2 * torch.rand(B, T, generator=g)).to(DEV).requires_grad_(True)
    adv = torch.randn(B, generator=g).to(DEV)
    mask = (torch.rand(B, T, generator=g) < 0.7).long().to(DEV)
    loss, metrics = amd.grpo_loss(lp, adv, mask, loss_type="dapo", num_items_in_batch=mask.sum().float())
    loss.backward()
    want = -(adv[:, None] * mask) / mask.sum()
    torch.testing.assert_close(lp.grad, want, rtol=1e-6, atol=1e-9)
    torch.testing.assert_close(loss.detach(), -(adv[:, None] * mask).sum() / mask.sum(), rtol=1e-5, atol=1e-7)
    assert float(metrics.detach()[4]) == 0.0


def test_group_advantages(amd):
    g = torch.Generator().manual_seed(23)
    r = torch.randn(64, generator=g)
    r[5] = float("nan")
    r[8:16] = 1.0  # zero-variance group
    r[16:24] = float("nan")  # a group with no scorable completion
    for G in (8, 16, 1):
        for mode in ("group", "batch", "none"):
            got = amd.group_advantages(r.to(DEV), G, mode).cpu()
            want = oracle.group_advantages(r, G, mode)
            torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)
    assert torch.equal(amd.group_advantages(r.to(DEV), 8, "group").cpu()[8:24], torch.zeros(16))
    # Bernoulli rewards of benchmark configuration 4 (G = 16): all-equal groups give exactly zero
    rb = (torch.rand(32, generator=g) < 0.3).float()
    torch.testing.assert_close(amd.group_advantages(rb.to(DEV), 16).cpu(), oracle.group_advantages(rb, 16), rtol=1e-5, atol=1e-6)


def _dpo_kwargs(case):
    return dict(loss_types=case.get("loss_types", ["sigmoid"]), loss_weights=case.get("loss_weights"),
                label_smoothing=case.get("label_smoothing", 0.0), ld_alpha=case.get("ld_alpha"),
                use_weighting=case.get("use_weighting", False), f_divergence_type=case.get("f_divergence_type", "reverse_kl"),
                f_alpha_divergence_coef=case.get("f_alpha", 1.0), discopop_tau=0.05)


@pytest.mark.parametrize("skip_masked", [False, True])
def test_golden_dpo_compute_loss_all_loss_types(amd, skip_masked):
    """Every case the reference's `DPOTrainer._compute_loss` ran on a mocked trainer (fifteen loss types, ld_alpha,
    WPO weighting, f-divergences, arg-max ties): loss, dlogits and the ten logged metrics, from one pass over the
    logits.  bf16 cases: the reference rounds log-probs, entropies and the WPO log-sum-exps to bf16, hence 2e-2."""
    cases, g = load_golden("dpo_compute_loss")
    for case in cases:
        c = f"c{case['id']}_"
        dtype = getattr(torch, case["dtype"])
        low = dtype != torch.float32
        leaf = _t(g[c + "logits"], dtype).to(DEV).requires_grad_(True)
        loss, parts = amd.dpo_compute_loss(
            leaf, _t(g[c + "input_ids"]).to(DEV), _t(g[c + "completion_mask"]).to(DEV),
            _t(g[c + "ref_chosen_logps"]).to(DEV), _t(g[c + "ref_rejected_logps"]).to(DEV), beta=case["beta"],
            skip_masked_rows=skip_masked, **_dpo_kwargs(case))
        loss.backward()
        want = float(g[c + "out_loss"])
        rel = 5e-2 if low else 1e-5
        assert abs(float(loss.detach()) - want) <= rel * max(1.0, abs(want)), (case["name"], float(loss.detach()), want)
        assert _rel_l2(leaf.grad.float(), _t(g[c + "out_dlogits"])) < (5e-2 if low else 1e-4), case["name"]
        got = amd.dpo_metrics_to_dict(parts)
        for name, want_m in case["metrics"].items():
            if name == "num_tokens" or (name == "rewards/accuracies" and (low or case.get("ref_equal"))):
                continue  # accuracies: ties / near-ties between the rewards are decided by rounding noise
            tol = (0.15 if low else 1e-5) * max(1.0, abs(want_m))
            if name in ("logits/chosen", "logits/rejected"):
                tol = max(tol, 2e-6)  # means of ~N(0, 4) logits over V: absolute fp32 summation noise
            assert abs(got[name] - want_m) <= tol, (case["name"], name, got[name], want_m)


def test_dpo_mixin_compute_loss(amd):
    """The mix-in method with the reference's signature on a mocked trainer (wpo + ld_alpha + ipo case)."""
    cases, g = load_golden("dpo_compute_loss")
    case = next(c for c in cases if c["name"] == "ipo_ld_alpha_wpo")
    c = f"c{case['id']}_"

    class Trainer(amd.DPOLossMixin):
        pass

    tr = Trainer()
    tr.accelerator = _Identity()
    tr.accelerator.gather_for_metrics = lambda x: x
    tr.model = SimpleNamespace(training=True)
    tr.aux_loss_enabled = False
    tr.precompute_ref_logps = True
    tr.beta, tr.loss_types, tr.loss_weights = case["beta"], case["loss_types"], [1.0]
    tr.label_smoothing, tr.ld_alpha, tr.use_weighting = 0.0, case["ld_alpha"], True
    tr.f_divergence_type, tr.f_alpha_divergence_coef = "reverse_kl", 1.0
    tr.args = SimpleNamespace(discopop_tau=0.05)
    tr._metrics = {"train": defaultdict(list), "eval": defaultdict(list)}
    tr._total_train_tokens = 0
    leaf = _t(g[c + "logits"]).to(DEV).requires_grad_(True)
    inputs = dict(input_ids=_t(g[c + "input_ids"]).to(DEV), attention_mask=_t(g[c + "attention_mask"]).to(DEV),
                  completion_mask=_t(g[c + "completion_mask"]).to(DEV),
                  ref_chosen_logps=_t(g[c + "ref_chosen_logps"]).to(DEV),
                  ref_rejected_logps=_t(g[c + "ref_rejected_logps"]).to(DEV))
    loss = tr._compute_loss(lambda **kw: SimpleNamespace(logits=leaf, aux_loss=None), inputs, False)
    loss.backward()
    assert abs(float(loss.detach()) - float(g[c + "out_loss"])) <= 1e-5 * max(1.0, abs(float(g[c + "out_loss"])))
    assert _rel_l2(leaf.grad, _t(g[c + "out_dlogits"])) < 1e-4
    got = {k: v[-1] for k, v in tr._metrics["train"].items()}
    for name, want in case["metrics"].items():
        assert abs(got[name] - want) <= 1e-5 * max(1.0, abs(want)), (name, got[name], want)
    # the reference-model pass: sequence log-probs of the same logits, with and without the ld_alpha split
    seq = amd.dpo_sequence_logps(leaf.detach(), inputs["input_ids"], inputs["completion_mask"])
    oseq, _ = oracle.dpo_sequence_logps(_t(g[c + "logits"]), _t(g[c + "input_ids"]), _t(g[c + "completion_mask"]))
    torch.testing.assert_close(seq.cpu(), oseq, rtol=1e-5, atol=1e-5)
    # reference log-probs computed inside the loss: from `ref_model`, and from the policy itself with its PEFT
    # adapters switched off or switched to the adapter named "ref" (dpo_trainer.py:1187-1195, 1373-1394).  The
    # stand-in model answers with other logits while it is in its reference state; the loss must equal the one
    # computed from those logits' sequence log-probs handed in precomputed.
    g2 = torch.Generator().manual_seed(5)
    ref_logits = (_t(g[c + "logits"]) + 0.3 * torch.randn(_t(g[c + "logits"]).shape, generator=g2)).to(DEV)
    ref_seq = amd.dpo_sequence_logps(ref_logits, inputs["input_ids"], inputs["completion_mask"], case["ld_alpha"])
    tr.precompute_ref_logps = True
    want = tr._compute_loss(lambda **kw: SimpleNamespace(logits=leaf, aux_loss=None),
                            dict(inputs, ref_chosen_logps=ref_seq[:3], ref_rejected_logps=ref_seq[3:]), False)

    class FakePeft:
        def __init__(self, adapters):
            self.peft_config = {name: object() for name in adapters}
            self.active_adapter = "default"
            self.disabled = False
            self.log = []

        def set_adapter(self, name):
            self.log.append(name)
            self.active_adapter = name

        def disable_adapter(self):
            from contextlib import contextmanager

            @contextmanager
            def ctx():
                self.disabled = True
                self.log.append("off")
                try:
                    yield
                finally:
                    self.disabled = False
                    self.log.append("on")

            return ctx()

        def __call__(self, **kw):
            assert "output_router_logits" not in kw
            in_ref_state = self.disabled or self.active_adapter == "ref"
            return SimpleNamespace(logits=ref_logits if in_ref_state else leaf, aux_loss=None)

    live = {k: v for k, v in inputs.items() if not k.startswith("ref_")}
    tr.precompute_ref_logps = False
    for adapters, trace in ((["default"], ["off", "on"]), (["default", "ref"], ["ref", "default"])):
        peft = FakePeft(adapters)
        tr.ref_model, tr.model = None, peft
        peft.training = True
        got = tr._compute_loss(peft, live, False)
        assert torch.equal(got, want) and peft.log == trace and peft.active_adapter == "default" and not peft.disabled
    tr.ref_model = lambda **kw: SimpleNamespace(logits=ref_logits)
    tr.model = SimpleNamespace(training=True)
    assert torch.equal(tr._compute_loss(lambda **kw: SimpleNamespace(logits=leaf, aux_loss=None), live, False), want)
    tr.ref_model = None
    with pytest.raises(ValueError, match="reference log-probs"):
        tr._compute_loss(lambda **kw: SimpleNamespace(logits=leaf, aux_loss=None), live, False)


@pytest.mark.parametrize("skip_masked", [True, False])
def test_golden_kto_compute_loss(amd, skip_masked):
    """The reference's `KTOTrainer._compute_loss` cases: loss, dlogits and the logged metrics through the mix-in
    method on a mocked trainer (KL pass included).  bf16: the reference sums bf16-rounded log-probs, hence 5e-2."""
    cases, g = load_golden("kto_compute_loss")
    for case in cases:
        c = f"c{case['id']}_"
        dtype = getattr(torch, case["dtype"])
        low = dtype != torch.float32

        class Trainer(amd.KTOLossMixin):
            pass

        tr = Trainer()
        tr.accelerator = _Identity()
        tr.accelerator.gather_for_metrics = lambda x: x
        tr.accelerator.device = torch.device(DEV)
        tr.model = SimpleNamespace(training=True)
        tr.aux_loss_enabled = False
        tr.precompute_ref_logps, tr.calculate_KL = True, case["kl"]
        tr.beta, tr.loss_type = case["beta"], case["loss_type"]
        tr.desirable_weight = case.get("desirable_weight", 1.0)
        tr.undesirable_weight = case.get("undesirable_weight", 1.0)
        tr._metrics = {"train": defaultdict(list), "eval": defaultdict(list)}
        tr._total_train_tokens = 0
        leaf = _t(g[c + "logits"], dtype).to(DEV).requires_grad_(True)
        kl_logits = _t(g[c + "kl_logits"], dtype).to(DEV)
        kl_len = case["kl_len"]

        def model(input_ids=None, **kw):
            return SimpleNamespace(logits=kl_logits if input_ids.shape[1] == kl_len else leaf, aux_loss=None)

        inputs = dict(input_ids=_t(g[c + "input_ids"]), attention_mask=_t(g[c + "attention_mask"]),
                      completion_mask=_t(g[c + "completion_mask"]), label=torch.tensor(case["labels"], dtype=torch.bool),
                      ref_logps=_t(g[c + "ref_logps"]))
        if case["kl"]:
            inputs.update(KL_input_ids=_t(g[c + "kl_input_ids"]), KL_attention_mask=_t(g[c + "kl_attention_mask"]),
                          KL_completion_mask=_t(g[c + "kl_completion_mask"]), ref_KL_logps=_t(g[c + "ref_kl_logps"]))
        if skip_masked:
            loss = tr._compute_loss(model, inputs, False)
            got = {k: v[-1] for k, v in tr._metrics["train"].items()}
        else:
            dev = {k: v.to(DEV) for k, v in inputs.items()}
            kl = amd.kto_sequence_logps(kl_logits, dev["KL_input_ids"], dev["KL_completion_mask"], False) if case["kl"] else None
            loss, parts = amd.kto_compute_loss(
                leaf, dev["input_ids"], dev["completion_mask"], dev["label"], dev["ref_logps"], kl,
                dev.get("ref_KL_logps"), case["beta"], case["loss_type"], tr.desirable_weight, tr.undesirable_weight,
                skip_masked_rows=False)
            got = {"kl": float(parts["kl"])}
        loss.backward()
        want = float(g[c + "out_loss"])
        assert abs(float(loss.detach()) - want) <= (5e-2 if low else 1e-5) * max(1.0, abs(want)), (case["name"], float(loss.detach()), want)
        assert _rel_l2(leaf.grad.float(), _t(g[c + "out_dlogits"])) < (5e-2 if low else 1e-4), case["name"]
        if skip_masked:
            assert set(got) == set(case["metrics"]), (case["name"], sorted(got))
        for name, value in got.items():
            want_m = case["metrics"][name]
            tol = max((0.15 if low else 1e-5) * max(1.0, abs(want_m)), 2e-6)
            assert abs(value - want_m) <= tol, (case["name"], name, value, want_m)


def test_kto_reference_pass_inside_the_loss(amd):
    """Reference log-probs computed inside `_compute_loss` (kto_trainer.py:1532-1549): from `ref_model`, and from
    the policy itself with its PEFT adapters switched off or switched to the adapter named "ref".  The stand-in
    model answers with other logits while it is in its reference state; the loss must equal the one computed from
    those logits' sequence log-probs handed in precomputed, and the model must be back in its training state."""
    from contextlib import contextmanager

    cases, g = load_golden("kto_compute_loss")
    case = next(c for c in cases if c["kl"] and c["dtype"] == "float32")
    c = f"c{case['id']}_"
    leaf = _t(g[c + "logits"]).to(DEV)
    kl_logits = _t(g[c + "kl_logits"]).to(DEV)
    gen = torch.Generator().manual_seed(11)
    ref_logits = (leaf.cpu() + 0.3 * torch.randn(leaf.shape, generator=gen)).to(DEV)
    ref_kl_logits = (kl_logits.cpu() + 0.3 * torch.randn(kl_logits.shape, generator=gen)).to(DEV)
    kl_len = case["kl_len"]
    assert kl_len != leaf.shape[1]

    class Trainer(amd.KTOLossMixin):
        pass

    tr = Trainer()
    tr.accelerator = _Identity()
    tr.accelerator.gather_for_metrics = lambda x: x
    tr.accelerator.device = torch.device(DEV)
    tr.aux_loss_enabled = False
    tr.calculate_KL = True
    tr.beta, tr.loss_type = case["beta"], case["loss_type"]
    tr.desirable_weight, tr.undesirable_weight = case.get("desirable_weight", 1.0), case.get("undesirable_weight", 1.0)
    tr._metrics = {"train": defaultdict(list), "eval": defaultdict(list)}
    tr._total_train_tokens = 0
    live = dict(input_ids=_t(g[c + "input_ids"]), attention_mask=_t(g[c + "attention_mask"]),
                completion_mask=_t(g[c + "completion_mask"]), label=torch.tensor(case["labels"], dtype=torch.bool),
                KL_input_ids=_t(g[c + "kl_input_ids"]), KL_attention_mask=_t(g[c + "kl_attention_mask"]),
                KL_completion_mask=_t(g[c + "kl_completion_mask"]))

    def answer(in_ref_state, input_ids):
        is_kl = input_ids.shape[1] == kl_len
        return SimpleNamespace(logits=(ref_kl_logits if is_kl else ref_logits) if in_ref_state else (kl_logits if is_kl else leaf),
                               aux_loss=None)

    ref_seq = amd.kto_sequence_logps(ref_logits, live["input_ids"].to(DEV), live["completion_mask"].to(DEV))
    ref_kl_seq = amd.kto_sequence_logps(ref_kl_logits, live["KL_input_ids"].to(DEV), live["KL_completion_mask"].to(DEV))
    tr.precompute_ref_logps = True
    tr.model = SimpleNamespace(training=True)
    want = tr._compute_loss(lambda input_ids=None, **kw: answer(False, input_ids),
                            dict(live, ref_logps=ref_seq, ref_KL_logps=ref_kl_seq), False)
    assert math.isfinite(float(want))

    class FakePeft:
        training = True

        def __init__(self, adapters):
            self.peft_config = {name: object() for name in adapters}
            self.active_adapter = "default"
            self.disabled = False
            self.log = []

        def set_adapter(self, name):
            self.log.append(name)
            self.active_adapter = name

        @contextmanager
        def disable_adapter(self):
            self.disabled = True
            self.log.append("off")
            try:
                yield
            finally:
                self.disabled = False
                self.log.append("on")

        def __call__(self, input_ids=None, **kw):
            assert "output_router_logits" not in kw
            return answer(self.disabled or self.active_adapter == "ref", input_ids)

    tr.precompute_ref_logps = False
    for adapters, trace in ((["default"], ["off", "on"]), (["default", "ref"], ["ref", "default"])):
        peft = FakePeft(adapters)
        tr.ref_model, tr.model = None, peft
        got = tr._compute_loss(peft, live, False)
        assert torch.equal(got, want) and peft.log == trace and peft.active_adapter == "default" and not peft.disabled
    tr.ref_model = lambda input_ids=None, **kw: answer(True, input_ids)
    tr.model = SimpleNamespace(training=True)
    assert torch.equal(tr._compute_loss(lambda input_ids=None, **kw: answer(False, input_ids), live, False), want)
    tr.ref_model = None
    with pytest.raises(ValueError, match="reference log-probs"):
        tr._compute_loss(lambda input_ids=None, **kw: answer(False, input_ids), live, False)


def test_golden_dpo_compute_loss(amd):
    """The fused sigmoid path (one loss kernel) on the plain sigmoid cases."""
    cases, g = load_golden("dpo_compute_loss")
    plain = [c for c in cases if not ({"loss_types", "ld_alpha", "use_weighting", "f_divergence_type"} & set(c))]
    assert len(plain) >= 5
    for case in plain:
        c = f"c{case['id']}_"
        dtype = getattr(torch, case["dtype"])
        low = dtype != torch.float32
        leaf = _t(g[c + "logits"], dtype).to(DEV).requires_grad_(True)
        loss, named = amd.dpo_loss_from_logits(
            leaf, _t(g[c + "input_ids"]).to(DEV), _t(g[c + "completion_mask"]).to(DEV),
            _t(g[c + "ref_chosen_logps"]).to(DEV), _t(g[c + "ref_rejected_logps"]).to(DEV), case["beta"], True)
        loss.backward()
        want = float(g[c + "out_loss"])
        assert abs(float(loss.detach()) - want) <= (2e-2 if low else 1e-5) * max(1.0, abs(want)), case["name"]
        assert _rel_l2(leaf.grad.float(), _t(g[c + "out_dlogits"])) < (2e-2 if low else 1e-4), case["name"]
        for name in ("rewards/chosen", "rewards/rejected", "rewards/accuracies", "rewards/margins", "logps/chosen",
                     "logps/rejected", "entropy"):
            want_m = case["metrics"][name]
            tol = (0.15 if low else 1e-5) * max(1.0, abs(want_m))  # bf16 reference sums bf16-rounded log-probs
            if name == "rewards/accuracies" and (low or case.get("ref_equal")):
                continue  # ties / near-ties between chosen and rejected rewards: decided by rounding noise
            got_m = float(named[name].detach())
            assert abs(got_m - want_m) <= tol, (case["name"], name, got_m, want_m)
        if case.get("ref_equal") and not low:
            assert abs(float(loss.detach()) - math.log(2.0)) < 1e-6


def test_dpo_against_oracle_config2_shape_subsample(amd):
    """benchmark configuration 2 layout (prompt mask + right padding, [chosen; rejected]) on a reduced
    sequence count/length at the real vocabulary; bf16 logits vs fp32-op-math oracle."""
    g = torch.Generator().manual_seed(24)
    P, L, V = 2, 48, 128256
    B = 2 * P
    logits = (2.0 * torch.randn(B, L, V, generator=g)).bfloat16()
    ids = torch.randint(0, V, (B, L), generator=g)
    cm = torch.zeros(B, L, dtype=torch.long)
    lp_len = torch.randint(4, 12, (P,), generator=g)
    for i in range(B):
        lc = int(torch.randint(8, 30, (1,), generator=g))
        cm[i, lp_len[i % P] : lp_len[i % P] + lc] = 1
    of = logits.float().requires_grad_(True)
    seq, _ = oracle.dpo_sequence_logps(of, ids, cm)
    ref = seq.detach() + 0.5 * torch.randn(B, generator=g)
    oloss, ometrics = oracle.dpo_sigmoid_loss(seq, ref[:P], ref[P:], 0.1)
    oloss.backward()
    leaf = logits.to(DEV).requires_grad_(True)
    loss, named = amd.dpo_loss_from_logits(leaf, ids.to(DEV), cm.to(DEV), ref[:P].to(DEV), ref[P:].to(DEV), 0.1)
    loss.backward()
    assert abs(float(loss.detach()) - float(oloss.detach())) <= 1e-3 * abs(float(oloss.detach()))
    torch.testing.assert_close(named["sequence_logps"].cpu(), seq.detach(), rtol=1e-3, atol=2e-3 * 30)
    assert _rel_l2(leaf.grad.float(), of.grad) < 3e-3
    assert torch.count_nonzero(leaf.grad[:, -1]) == 0
    assert torch.equal((leaf.grad[:, :-1] != 0).any(-1).cpu(), cm[:, 1:] != 0)
    for name, want in ometrics.items():
        assert abs(float(named[name].detach()) - want) <= 1e-3 * max(1.0, abs(want)), name


def test_dpo_full_size_config2_closed_form_and_properties(amd):
    """benchmark configuration 2 at full size (64 x 2048 x 128256 bf16, 32 pairs, prompt + right padding): with the
    reference log-probs equal to the policy's the loss is ln 2 and every pair carries the gradient -beta/(2P) on
    the chosen and +beta/(2P) on the rejected sequence; rows outside the shifted completion mask and the last
    position get exactly zero gradient; sum_v dlogits = 0 on the others."""
    B, L, V, beta = 64, 2048, 128256, 0.1
    P = B // 2
    g = torch.Generator(device=DEV).manual_seed(2)
    logits = torch.empty(B, L, V, dtype=torch.bfloat16, device=DEV)
    for b in range(B):
        for t0 in range(0, L, 1024):
            logits[b, t0 : t0 + 1024] = (2.0 * torch.randn(1024, V, generator=g, device=DEV)).bfloat16()
    ids = torch.randint(0, V, (B, L), generator=g, device=DEV)
    lp_len = torch.randint(64, 513, (P,), generator=g, device=DEV).repeat(2)
    lc_len = torch.randint(128, 1537, (B,), generator=g, device=DEV)
    pos = torch.arange(L, device=DEV)[None]
    cm = ((pos >= lp_len[:, None]) & (pos < (lp_len + lc_len)[:, None])).long()
    seq = amd.dpo_sequence_logps(logits, ids, cm)
    logits.requires_grad_(True)
    loss, parts = amd.dpo_compute_loss(logits, ids, cm, seq[:P], seq[P:], beta=beta)
    assert abs(float(loss.detach()) - math.log(2.0)) < 1e-6
    loss.backward()
    grad = logits.grad
    shift = cm[:, 1:].bool()
    row_nonzero = torch.stack([(grad[b] != 0).any(-1) for b in range(B)])
    assert not row_nonzero[:, -1].any() and torch.equal(row_nonzero[:, :-1], shift)
    row_sum = torch.stack([grad[b, :-1].float().sum(-1) for b in range(B)])
    coef = beta / (2 * P)
    assert (row_sum.abs() <= 2e-2 * coef).all()
    # the target's entry: -/+ coef * (1 - p_target) on chosen / rejected rows
    tgt = torch.stack([grad[b, :-1].gather(-1, ids[b, 1:, None]).squeeze(-1).float() for b in range(B)])
    assert (tgt[:P][shift[:P]] < 0).all() and (tgt[P:][shift[P:]] > 0).all()
    assert (tgt.abs() <= coef * (1 + 2e-2)).all()
    m = amd.dpo_metrics_to_dict(parts)
    assert abs(m["rewards/margins"]) < 1e-6 and 0.0 < m["entropy"] <= math.log(V)


def test_golden_rloo_compute_loss(amd):
    cases, g = load_golden("rloo_compute_loss")
    for case in cases:
        c = f"c{case['id']}_"
        B, P, T, V = case["shape"]
        leaf = _t(g[c + "logits"]).to(DEV).requires_grad_(True)
        ids = torch.cat([_t(g[c + "prompt_ids"]), _t(g[c + "completion_ids"])], 1).to(DEV)
        lp, ent = amd.per_token_logps_and_entropies(leaf, ids, T, case["temperature"], True)
        loss, seq, metrics = amd.rloo_loss(lp, _t(g[c + "completion_mask"]).to(DEV), _t(g[c + "old_logps"]).to(DEV),
                                           _t(g[c + "advantages"]).to(DEV), case["eps_low"], case["eps_high"])
        loss.backward()
        want = float(g[c + "out_loss"])
        assert abs(float(loss.detach()) - want) <= 1e-5 * max(1.0, abs(want))
        assert _rel_l2(leaf.grad, _t(g[c + "out_dlogits"])) < 1e-4
        from trl_amd.trainer.rloo_trainer import RLOO_METRIC_NAMES

        for i, name in enumerate(RLOO_METRIC_NAMES):
            assert abs(float(metrics.detach()[i]) - case["metrics"][name]) <= 1e-6, name
    r = torch.tensor([1.0, 2.0, 4.0, 0.5, float("nan"), 2.5])
    torch.testing.assert_close(amd.rloo_advantages(r.to(DEV), 3).cpu(), oracle.rloo_advantages(r, 3))


@pytest.mark.parametrize("skip_masked", [False, True])
def test_rloo_mixin_compute_loss(amd, skip_masked):
    """`RLOOLossMixin._compute_loss` on the mocked trainer the reference's own method ran on."""
    cases, g = load_golden("rloo_compute_loss")
    for case in cases:
        c = f"c{case['id']}_"
        B, P, T, V = case["shape"]

        class Trainer(amd.RLOOLossMixin):
            pass

        tr = Trainer()
        tr.accelerator = _Identity()
        tr.temperature = case["temperature"]
        tr.model_kwarg_keys = set()
        tr.aux_loss_enabled = False
        tr.epsilon_low, tr.epsilon_high = case["eps_low"], case["eps_high"]
        tr._metrics = {"train": defaultdict(list), "eval": defaultdict(list)}
        tr.model = SimpleNamespace(training=True)
        tr.trl_amd_skip_masked_rows = skip_masked
        leaf = _t(g[c + "logits"]).to(DEV).requires_grad_(True)
        inputs = dict(
            prompt_ids=_t(g[c + "prompt_ids"]).to(DEV), prompt_mask=torch.ones(B, P, dtype=torch.long, device=DEV),
            completion_ids=_t(g[c + "completion_ids"]).to(DEV), completion_mask=_t(g[c + "completion_mask"]).to(DEV),
            old_logps=_t(g[c + "old_logps"]).to(DEV), advantages=_t(g[c + "advantages"]).to(DEV))
        loss = tr._compute_loss(lambda **kw: SimpleNamespace(logits=leaf, aux_loss=None), inputs)
        loss.backward()
        want = float(g[c + "out_loss"])
        assert abs(float(loss.detach()) - want) <= 1e-5 * max(1.0, abs(want))
        assert _rel_l2(leaf.grad, _t(g[c + "out_dlogits"])) < 1e-4
        got = {k: v[-1] for k, v in tr._metrics["train"].items()}
        for name, want_m in case["metrics"].items():
            assert abs(got[name] - want_m) <= 1e-5 * max(1.0, abs(want_m)), (name, got[name], want_m)


def test_multimodal_sub_batches_through_the_logprob_method(amd):
    """`_get_per_token_logps_and_entropies` with `batch_size < B` on a multimodal batch
    (trl/trainer/grpo_trainer.py:1460-1510): a model whose forward accepts exactly the reference's keyword set sees,
    per sub-batch, the patch rows and grid rows of that sub-batch's images; the log-probs equal those of one call on
    the whole batch.  Same keyword set on the one-pass branch of `_compute_loss`."""
    B, P, T, V, D = 4, 2, 6, 64, 3
    g = torch.Generator().manual_seed(91)
    logits = (2.0 * torch.randn(B, P + T, V, generator=g)).bfloat16().to(DEV)
    ids = torch.randint(0, V, (B, P + T), generator=g).to(DEV)
    attn = torch.ones(B, P + T, dtype=torch.long, device=DEV)
    grid = torch.tensor([[1, 2, 2], [1, 2, 3], [1, 1, 4], [1, 3, 2]], device=DEV)
    num_images = [1, 2, 0, 1]
    pixels = torch.randn(20, D, generator=g).to(DEV)
    seen = []

    def model(*, input_ids, attention_mask, pixel_values, image_grid_thw, use_cache, mm_token_type_ids=None):
        seen.append((input_ids.shape[0], pixel_values.shape[0], image_grid_thw.shape[0]))
        assert int(image_grid_thw.prod(-1).sum()) == pixel_values.shape[0]
        rows = [int((ids == r).all(1).nonzero()[0]) for r in input_ids]  # which samples these are
        return SimpleNamespace(logits=logits[rows], aux_loss=None)

    case = dict(loss_type="dapo", beta=0.0, eps_low=0.2, eps_high=0.2)
    tr = _fake_trainer(amd, case, T)
    kw = dict(pixel_values=pixels, image_grid_thw=grid, num_images=num_images)
    whole, ent_whole, _ = tr._get_per_token_logps_and_entropies(model, ids, attn, T, compute_entropy=True, **kw)
    parts, ent_parts, _ = tr._get_per_token_logps_and_entropies(model, ids, attn, T, batch_size=2, compute_entropy=True, **kw)
    assert seen == [(4, 20, 4), (2, 14, 3), (2, 6, 1)]
    assert torch.equal(whole, parts) and torch.equal(ent_whole, ent_parts)
    one, _, _ = tr._get_per_token_logps_and_entropies(model, ids, attn, T, batch_size=1, **kw)
    assert torch.equal(whole, one) and seen[-4:] == [(1, 4, 1), (1, 10, 2), (1, 0, 0), (1, 6, 1)]
    # `_compute_loss`, both branches: the same keyword set reaches the model (num_images is never passed on)
    for single_pass in (False, True):
        tr = _fake_trainer(amd, case, T, skip_masked=True, single_pass=single_pass)
        inputs = dict(prompt_ids=ids[:, :P], prompt_mask=attn[:, :P], completion_ids=ids[:, P:], completion_mask=attn[:, P:],
                      advantages=torch.randn(B, generator=g).to(DEV), num_items_in_batch=torch.tensor(24.0, device=DEV),
                      pixel_values=pixels, image_grid_thw=grid, num_images=num_images)
        seen.clear()
        loss = tr._compute_loss(model, inputs)
        assert seen == [(4, 20, 4)] and math.isfinite(float(loss.detach()))


@pytest.mark.parametrize("single_pass", [False, True])
def test_trainer_method_raises_on_a_token_id_outside_the_vocabulary(amd, single_pass):
    """The reference's gather raises (CPU) or device-asserts (GPU) on an id outside [0, V)
    (trl/trainer/utils.py:507,516); the kernels set a device flag instead, and the mix-in reads it with the copy of
    the metrics it makes anyway: `_compute_loss` raises IndexError, and the next clean call passes."""
    B, P, T, V = 2, 1, 4, 64
    g = torch.Generator().manual_seed(7)
    leaf = (torch.randn(B, P + T, V, generator=g)).bfloat16().to(DEV).requires_grad_(True)
    case = dict(loss_type="grpo", beta=0.0, eps_low=0.2, eps_high=0.2)
    inputs = dict(prompt_ids=torch.zeros(B, P, dtype=torch.long, device=DEV), prompt_mask=torch.ones(B, P, dtype=torch.long, device=DEV),
                  completion_ids=torch.randint(0, V, (B, T), generator=g).to(DEV),
                  completion_mask=torch.ones(B, T, dtype=torch.long, device=DEV), advantages=torch.randn(B, generator=g).to(DEV))
    model = lambda **kw: SimpleNamespace(logits=leaf, aux_loss=None)  # noqa: E731
    bad = dict(inputs, completion_ids=inputs["completion_ids"].clone())
    bad["completion_ids"][1, 2] = V + 3
    tr = _fake_trainer(amd, case, T, skip_masked=True, single_pass=single_pass)
    with pytest.raises(IndexError):
        tr._compute_loss(model, bad)
    assert math.isfinite(float(tr._compute_loss(model, inputs).detach()))
    amd.check_device_errors()

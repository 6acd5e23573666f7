"""Seeded random sweeps over configurations, shapes and dtypes: the HIP path against the CPU oracle (GRPO and DPO
losses with their gradients), the single-pass GRPO kernel against the two-pass path, and the fused head against
fp32 autograd.  The golden vectors pin chosen configurations; these sweeps walk the combinations between them (loss
type x importance-sampling level x delta x KL x masks x advantage shape x entropy bonus ..., odd sizes, empty
sequences).  Bars as in the other GPU tests: fp32 2e-5, 16-bit gradients by relative L2."""
import math
import os
import random

import pytest
import torch
import torch.nn.functional as F

import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def amd():
    import trl_amd

    return trl_amd


def _amax(x):
    """Largest magnitude, 0 for an empty tensor."""
    return float(x.abs().max()) if x.numel() else 0.0


def _rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp(min=1e-30))


def _grad_close(got, want, bar, dt, zmax, g_norm):
    """|got - want| <= bar * |want| + what the arithmetic itself leaves: a probability comes out of exp(z - lse) with
    a relative error of a few ulps of lse's magnitude, so g * (onehot - p) carries that much of g as an ABSOLUTE error,
    which is all that is left of it where p is within 1e-5 of 1 and the gradient cancels.  16-bit: the upstream
    gradients reach the kernel rounded to that type, each its own way, so where the log-prob and the entropy term of
    a row cancel, half an ulp of each remains.  Returns (ok, excess)."""
    eps = 2.0**-53 if dt == torch.float64 else 2.0**-24
    half_ulp = {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}.get(dt, 0.0)
    diff = float((got.double().cpu() - want.double().cpu()).norm())
    allowed = bar * float(want.double().norm()) + (4 * eps * max(1.0, zmax) + half_ulp) * g_norm
    return diff <= allowed, diff / max(allowed, 1e-300)


def test_grpo_loss_kernel_against_the_oracle(amd):
    """300 configurations of the `[B, T]` loss kernel: loss and d loss / d logp (and d loss / d entropy) against the
    oracle's autograd."""
    rnd = random.Random(1)
    torch.manual_seed(1)
    ran = 0
    for case in range(300):
        B, T = rnd.choice([1, 2, 3, 8]), rnd.choice([1, 5, 17, 64])
        lt = rnd.choice(["grpo", "bnpo", "dr_grpo", "dapo", "cispo", "sapo", "luspo", "vespo"])
        beta = rnd.choice([0.0, 0.04, 0.5])
        lp = -3 * torch.rand(B, T)
        old = rnd.choice([None, lp + rnd.choice([0.0, 0.05, 0.5, 2.0]) * torch.randn(B, T)])
        ref = lp + 0.2 * torch.randn(B, T) if beta else None
        mask = (torch.arange(T)[None] < torch.randint(0, T + 1, (B,))[:, None]).long()
        if rnd.random() < 0.2:
            mask = (torch.rand(B, T) < 0.6).long()
        adv = rnd.choice([torch.randn(B), torch.randn(B, T) if lt != "luspo" else torch.randn(B)])
        if rnd.random() < 0.1:
            adv = torch.zeros_like(adv)
        ent = 3 * torch.rand(B, T)
        kw = dict(old_per_token_logps=old, ref_per_token_logps=ref, loss_type=lt, epsilon_low=rnd.choice([0.2, 0.1]),
                  epsilon_high=rnd.choice([0.2, 0.28, 3.0 if lt == "cispo" else 0.2]), beta=beta,
                  delta=rnd.choice([None, None, 1.5, 4.0]) if lt not in ("cispo", "sapo", "vespo") else None,
                  max_completion_length=T, num_items_in_batch=float(int(mask.sum())) * rnd.choice([1.0, 2.0]),
                  num_processes=rnd.choice([1, 2]), grad_accum_steps=rnd.choice([1.0, 4.0]),
                  importance_sampling_level=rnd.choice(["token", "token", "sequence"]),
                  use_bias_correction_kl=old is not None and rnd.random() < 0.3, entropy_coef=rnd.choice([0.0, 0.0, 0.01]))
        olp, oent = lp.clone().requires_grad_(True), ent.clone().requires_grad_(True)
        try:
            oloss, _ = oracle.grpo_loss(olp, adv, mask, entropies=oent, **kw)
        except (ValueError, NotImplementedError):
            continue  # a combination the reference rejects too
        oloss.backward()
        glp, gent = lp.to(DEV).requires_grad_(True), ent.to(DEV).requires_grad_(True)
        gkw = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in kw.items()}
        gloss, _ = amd.grpo_loss(glp, adv.to(DEV), mask.to(DEV), entropies=gent, **gkw)
        gloss.backward()
        what = (case, lt, kw["importance_sampling_level"], beta, kw["delta"], tuple(adv.shape))
        assert abs(float(gloss.detach()) - float(oloss.detach())) <= 2e-5 * max(1.0, abs(float(oloss.detach()))), what
        scale = float(olp.grad.abs().max())
        assert float((glp.grad.cpu() - olp.grad).abs().max()) <= 2e-5 * scale + 1e-7, what
        if kw["entropy_coef"]:
            ge = gent.grad.cpu() if gent.grad is not None else torch.zeros_like(ent)
            assert float((ge - oent.grad).abs().max()) <= 2e-5 * float(oent.grad.abs().max()) + 1e-8, what
        ran += 1
    assert ran >= 200


def test_logprob_kernels_against_fp64(amd):
    """400 problems through `logps_and_entropies` and its gradient: fp32 / bf16 / fp16 / fp64 logits, vocabularies
    that are and are not multiples of the vector width, one to three indices per row, a window of the rows, views
    with strides in both leading dimensions, row masks, temperatures; the reference is torch's log_softmax in fp64
    on the stored values, forward and autograd."""
    rnd = random.Random(7)
    torch.manual_seed(7)
    for case in range(400):
        n_seq, length = rnd.choice([1, 2, 3]), rnd.choice([1, 2, 5, 9])
        V = rnd.choice([1, 2, 7, 8, 33, 256, 257, 1000, 4096, 4099, 20488])
        dt = rnd.choice([torch.float32, torch.float32, torch.bfloat16, torch.float16, torch.float64])
        K = rnd.choice([0, 1, 1, 2, 3])  # 0: index without the trailing axis
        T = rnd.choice([1.0, 0.7, 1.3])
        keep_start = rnd.randrange(0, length)
        keep_len = rnd.randrange(0, length - keep_start + 1)
        scale = rnd.choice([0.5, 3.0, 8.0])
        pad0, pad1 = rnd.choice([0, 1]), rnd.choice([0, 2])
        big = (scale * torch.randn(n_seq + pad0, length + pad1, V, device=DEV)).to(dt)
        view = big[pad0:, pad1 // 2 : pad1 // 2 + length]  # strides of the larger tensor
        leaf = view.detach().clone().requires_grad_(True) if rnd.random() < 0.3 else None
        src = leaf if leaf is not None else view.detach().requires_grad_(True)
        shape = (n_seq, keep_len) if K == 0 else (n_seq, keep_len, K)
        index = torch.randint(0, V, shape, device=DEV)
        row_mask = (torch.rand(n_seq, keep_len, device=DEV) < 0.6) if rnd.random() < 0.3 else None
        logp, ent = amd.logps_and_entropies(src, index, T, keep_start, keep_len, row_mask)
        assert logp.shape == shape and ent.shape == (n_seq, keep_len)
        out_dt = torch.float64 if dt == torch.float64 else torch.float32
        assert logp.dtype == out_dt and ent.dtype == out_dt
        ref_src = view.detach().double().requires_grad_(True)
        z = ref_src[:, keep_start : keep_start + keep_len] / T
        lsm = F.log_softmax(z, dim=-1)
        want_lp = lsm.gather(-1, index if K else index.unsqueeze(-1))
        want_lp = want_lp if K else want_lp.squeeze(-1)
        want_h = -(lsm.exp() * lsm).sum(-1)
        live = torch.ones(n_seq, keep_len, dtype=torch.bool, device=DEV) if row_mask is None else row_mask
        what = (case, str(dt), V, K, T, keep_start, keep_len, pad0, pad1, row_mask is not None)
        tol = 1e-12 if dt == torch.float64 else 2e-5
        zmax = float(z.detach().abs().max()) if z.numel() else 0.0
        if keep_len:
            lm = live if K == 0 else live.unsqueeze(-1).expand(shape)
            assert _amax((logp.detach().double() - want_lp.detach())[lm]) <= tol * max(1.0, zmax), what
            assert _amax((ent.detach().double() - want_h.detach())[live]) <= tol * max(1.0, zmax) + (0 if dt == torch.float64 else 2.5e-7 * zmax), what
            if row_mask is not None:  # skipped rows come back as exact zeros
                assert _amax(logp.detach()[~lm]) == 0.0 and _amax(ent.detach()[~live]) == 0.0, what
        g_lp = torch.randn(shape, device=DEV, dtype=torch.float64)
        g_h = torch.randn(n_seq, keep_len, device=DEV, dtype=torch.float64) * (0.0 if rnd.random() < 0.5 else 1.0)
        lmask = live.double() if K == 0 else live.double().unsqueeze(-1)
        ((logp.double() * g_lp * lmask).sum() + (ent.double() * g_h * live.double()).sum()).backward()
        ((want_lp * g_lp * lmask).sum() + (want_h * g_h * live.double()).sum()).backward()
        got = src.grad
        assert got.shape == view.shape and got.dtype == dt, what
        want = ref_src.grad
        bar = {torch.float64: 1e-12, torch.float32: 2e-5, torch.bfloat16: 4e-3, torch.float16: 2e-3}[dt]
        if float(want.abs().max()) == 0.0:  # (a one-entry vocabulary has no gradient; rounding may leave g * (1 - p))
            assert _amax(got.double()) <= bar * (_amax(g_lp) + _amax(g_h)), what
        else:
            ok, excess = _grad_close(got, want, bar, dt, zmax, float((g_lp * lmask).norm() + (g_h * live.double()).norm()))
            assert ok, (what, excess)
        outside = torch.ones(length, dtype=torch.bool, device=DEV)
        outside[keep_start : keep_start + keep_len] = False
        assert _amax(got[:, outside].double()) == 0.0, what  # rows outside the window: exact zeros
    amd.check_device_errors()


def test_drop_in_functions_at_any_shape(amd):
    """300 calls of `selective_log_softmax` / `entropy_from_logits` as the reference's callers make them: logits
    of one to four dimensions, views whose leading dimensions are strided or permuted, index with and without a
    trailing axis, every float dtype; results in the logits' dtype (one rounding of the fp32 value for 16-bit
    logits) against torch in fp64, gradients against fp64 autograd."""
    rnd = random.Random(8)
    torch.manual_seed(8)
    ulp = {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}
    for case in range(300):
        lead = rnd.choice([(), (5,), (3, 4), (2, 3, 2), (1, 1), (4, 1)])
        V = rnd.choice([2, 8, 41, 768, 1000, 4099])
        dt = rnd.choice([torch.float32, torch.float32, torch.bfloat16, torch.float16, torch.float64])
        base = (rnd.choice([1.0, 4.0]) * torch.randn(*lead, V, device=DEV)).to(dt)
        how = rnd.choice(["plain", "permute", "slice"]) if len(lead) >= 2 else "plain"
        if how == "permute":
            perm = list(range(len(lead)))
            rnd.shuffle(perm)
            inv = [perm.index(i) for i in range(len(lead))]
            view = base.permute(*perm, len(lead)).contiguous().permute(*inv, len(lead))  # same values, permuted strides
        elif how == "slice":
            big = torch.cat([base, base], dim=0)
            view = big[::2] if lead[0] > 1 else big[:1]
            base = view.clone()
        else:
            view = base
        K = rnd.choice([None, 1, 3])
        index = torch.randint(0, V, lead + (() if K is None else (K,)), device=DEV)
        leaf = view.detach().requires_grad_(True)
        got_lp = amd.selective_log_softmax(leaf, index)
        got_h = amd.entropy_from_logits(leaf, chunk_size=rnd.choice([1, 16, 128]))
        assert got_lp.shape == index.shape and got_h.shape == lead and got_lp.dtype == dt and got_h.dtype == dt
        ref = base.detach().double().requires_grad_(True)
        lsm = F.log_softmax(ref, dim=-1)
        want_lp = lsm.gather(-1, index.unsqueeze(-1)).squeeze(-1) if K is None else lsm.gather(-1, index)
        want_h = -(lsm.exp() * lsm).sum(-1)
        what = (case, lead, V, str(dt), how, K)
        for got, want in ((got_lp, want_lp), (got_h, want_h)):
            err = (got.detach().double() - want.detach()).abs()
            if dt == torch.float64:
                assert _amax(err) <= 1e-12, what
            elif dt == torch.float32:
                assert _amax(err) <= 2e-5, what
            else:  # one rounding of a value that is itself good to 2e-5
                assert bool((err <= 0.5 * ulp[dt] * want.detach().abs().clamp(min=2.0**-14) * 2 + 2e-5).all()), what
        g_lp, g_h = torch.randn(index.shape, device=DEV, dtype=torch.float64), torch.randn(lead, device=DEV, dtype=torch.float64)
        ((got_lp.double() * g_lp).sum() + (got_h.double() * g_h).sum()).backward()
        ((want_lp * g_lp).sum() + (want_h * g_h).sum()).backward()
        assert leaf.grad.shape == view.shape and leaf.grad.dtype == dt
        # 16-bit: the upstream gradients reach the kernel rounded to the outputs' dtype, then one rounding of dlogits
        # (bf16: three roundings -- both upstream gradients and the result -- with nothing to average them out in a
        # two-entry row)
        bar = {torch.float64: 1e-12, torch.float32: 2e-5, torch.bfloat16: 1.2e-2, torch.float16: 2e-3}[dt]
        ok, excess = _grad_close(leaf.grad, ref.grad, bar, dt, float(base.abs().max()), float(g_lp.norm() + g_h.norm()))
        assert ok, (what, excess)
    amd.check_device_errors()


def test_advantages_against_the_oracle(amd):
    """300 reward vectors through the group-advantage kernel and the leave-one-out baseline: group sizes 1 ... 16,
    the three scaling modes, NaN rewards (single ones, whole groups), constant groups; against the oracle."""
    rnd = random.Random(9)
    torch.manual_seed(9)
    for case in range(300):
        G = rnd.choice([1, 2, 3, 8, 16])
        n_groups = rnd.choice([1, 2, 5, 32])
        rewards = rnd.choice([1.0, 100.0]) * torch.randn(G * n_groups)
        if rnd.random() < 0.3:
            rewards = torch.bernoulli(torch.full((G * n_groups,), 0.3))
        if rnd.random() < 0.4:
            rewards[torch.rand(G * n_groups) < 0.2] = float("nan")
        if rnd.random() < 0.2:
            rewards.view(n_groups, G)[rnd.randrange(n_groups)] = float("nan")
        if rnd.random() < 0.2:
            rewards.view(n_groups, G)[rnd.randrange(n_groups)] = 0.5
        mode = rnd.choice(["group", "batch", "none"])
        # (absolute bar: a reward minus a mean of rewards is held to a few ulps of the rewards' size, 3e-5 at 300)
        finite = rewards[~rewards.isnan()]
        atol = max(2e-5, 5e-7 * float(finite.abs().max())) if finite.numel() else 2e-5
        got = amd.group_advantages(rewards.to(DEV), G, mode).cpu()
        want = oracle.group_advantages(rewards, G, mode)
        torch.testing.assert_close(got, want, rtol=2e-5, atol=atol if mode == "none" else 2e-5,
                                   msg=lambda m: f"{(case, G, n_groups, mode)}: {m}")
        assert bool((got[want == 0] == 0).all())  # constant and unscorable groups: exactly zero
        norm = rnd.random() < 0.5
        got = amd.rloo_advantages(rewards.to(DEV), G, norm).cpu()
        want = oracle.rloo_advantages(rewards, G, norm)
        torch.testing.assert_close(got, want, rtol=2e-5, atol=2e-5 if norm else atol,
                                   msg=lambda m: f"{(case, G, n_groups, norm)}: {m}")


def test_single_pass_kernel_against_the_two_pass_path(amd):
    """250 configurations the single-pass kernel takes (loss types, KL, delta, bias-corrected KL, token weights,
    per-token advantages, entropy bonus, temperatures, bf16 / fp16 / fp32, vocabularies 8 ... 20488 (two that are no multiple of the vector) and one whose rows overflow
    into LDS, empty sequences, ragged
    masks): loss, metrics, log-probs and dlogits against K1 + loss kernel + K3."""
    rnd = random.Random(2)
    torch.manual_seed(2)
    for case in range(250):
        B, K, V = rnd.choice([1, 2, 5]), rnd.choice([1, 7, 33]), rnd.choice([8, 64, 264, 1000, 1003, 4096, 4099, 20488, 172040])
        L = K + rnd.choice([1, 1, 3])
        dt = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
        if dt == torch.float32 and V > 167936:  # (fp32 rows hold half as many logits)
            V = 83976
        lt = rnd.choice(["grpo", "bnpo", "dr_grpo", "dapo", "cispo", "sapo"])
        beta, T = rnd.choice([0.0, 0.04]), rnd.choice([1.0, 0.7, 1.3])
        logits = (rnd.choice([0.5, 2.0, 6.0]) * torch.randn(B, L, V, device=DEV)).to(dt)
        ids = torch.randint(0, V, (B, K), device=DEV)
        mask = (torch.arange(K, device=DEV)[None] < torch.randint(0, K + 1, (B,), device=DEV)[:, None]).long()
        if rnd.random() < 0.2:
            mask = (torch.rand(B, K, device=DEV) < 0.5).long()
        adv = rnd.choice([torch.randn(B, device=DEV), torch.randn(B, K, device=DEV)])
        with torch.no_grad():
            base, _ = amd.per_token_logps_and_entropies(logits, ids, K, T)
        old = rnd.choice([None, base + rnd.choice([0.05, 0.5]) * torch.randn(B, K, device=DEV)])
        kw = dict(old_per_token_logps=old, ref_per_token_logps=base + 0.2 * torch.randn(B, K, device=DEV) if beta else None,
                  loss_type=lt, epsilon_low=0.2, epsilon_high=0.28, beta=beta,
                  delta=rnd.choice([None, 2.0]) if lt not in ("cispo", "sapo") else None, max_completion_length=K,
                  num_items_in_batch=mask.sum().float() * 2, grad_accum_steps=rnd.choice([1.0, 2.0]),
                  use_bias_correction_kl=old is not None and rnd.random() < 0.3,
                  token_weight=rnd.choice([None, None, 0.5 + torch.rand(B, K, device=DEV)]),
                  entropy_coef=rnd.choice([0.0, 0.0, 0.02]))
        leaf2 = logits.detach().clone().requires_grad_(True)
        lp2, ent2 = amd.per_token_logps_and_entropies(leaf2, ids, K, T, True, True)
        loss2, met2 = amd.grpo_loss(lp2, adv, mask, entropies=ent2, **kw)
        loss2.backward()
        leaf1 = logits.detach().clone().requires_grad_(True)
        loss1, met1, lp1, _ = amd.grpo_loss_from_logits(leaf1, ids, adv, mask, temperature=T, **kw)
        loss1.backward()
        what = (case, lt, str(dt), V, beta, T, kw["delta"], kw["entropy_coef"])
        assert abs(float(loss1.detach()) - float(loss2.detach())) <= 2e-5 * max(1.0, abs(float(loss2.detach()))), what
        # (atol: the entropy of a row is the difference of two numbers the size of its largest logit, held to an ulp
        # of that, 4e-6 at 32, whichever kernel computes it)
        torch.testing.assert_close(met1, met2, rtol=1e-4, atol=3e-5, equal_nan=True)
        m = mask.bool()
        if bool(m.any()):
            assert float((lp1[m] - lp2.detach()[m]).abs().max()) <= 2e-5 * max(1.0, float(lp2.detach()[m].abs().max())), what
        if float(leaf2.grad.float().abs().max()) > 0:
            # Both paths hold a log-prob to a few ulps of its magnitude (4e-6 at -40), and a token's gradient coefficient
            # -- the ratio exp(logp - old) times the advantage, plus beta * (1 - exp(ref - logp)) -- carries that over,
            # amplified without bound where its terms nearly cancel.  So the bar is what the loss kernel's own
            # coefficients move by when the log-probs move by four ulps, on top of the rounding of the result.
            def coefficients(lp):
                lp = lp.detach().clone().requires_grad_(True)
                amd.grpo_loss(lp, adv, mask, entropies=ent2.detach(), **kw)[0].backward()
                return lp.grad

            c0, c1 = coefficients(lp2), coefficients(lp2 * (1.0 + 2.0**-21))
            moved = _rel(c1, c0) if float(c0.abs().max()) > 0 else 0.0
            # (bf16: each path rounds its own fp32 value, so an entry may differ by a whole ulp, 2^-7, and a problem of
            # eight logits has nothing to average that out)
            bar = {torch.float32: 2e-5, torch.bfloat16: 8e-3, torch.float16: 4e-3}[dt] + 2.0 * moved
            # (and what either path's arithmetic leaves of c * (onehot - p) where a target's probability is within 1e-4
            # of 1: a few ulps of the log-sum-exp's magnitude times the coefficient, as an absolute error; with an entropy
            # bonus the same ulps of the entropy itself, which multiplies every probability of the row)
            zmax = float(logits.float().abs().max()) / T
            floor = 8 * 2.0**-24 * max(1.0, zmax) * (float(c0.norm()) + abs(kw["entropy_coef"]) * float(mask.sum()) ** 0.5)
            diff = float((leaf1.grad.double() - leaf2.grad.double()).norm())
            assert diff < bar * float(leaf2.grad.double().norm()) + floor, (what, _rel(leaf1.grad, leaf2.grad), moved)
        else:
            assert float(leaf1.grad.float().abs().max()) == 0.0, what
    amd.check_device_errors()


def test_dpo_loss_against_the_oracle(amd):
    """300 configurations of `dpo_compute_loss` (fifteen loss types alone and in weighted pairs, label smoothing,
    ld_alpha, WPO weighting, f-divergences, fp32 and bf16 logits, ragged completion masks): loss and dlogits."""
    rnd = random.Random(3)
    torch.manual_seed(3)
    types = ["sigmoid", "hinge", "ipo", "exo_pair", "nca_pair", "robust", "bco_pair", "sppo_hard", "aot", "aot_unpaired",
             "apo_zero", "apo_down", "discopop", "sft", "sigmoid_norm"]
    ran = 0
    for case in range(300):
        P, L, V = rnd.choice([1, 2, 5]), rnd.choice([2, 6, 19]), rnd.choice([5, 64, 257, 1000])
        dt = rnd.choice([torch.float32, torch.float32, torch.bfloat16])
        logits = (2.0 * torch.randn(2 * P, L, V)).to(dt)
        ids = torch.randint(0, V, (2 * P, L))
        start, end = torch.randint(0, L, (2 * P,)), torch.randint(0, L + 1, (2 * P,))
        ar = torch.arange(L)[None]
        cm = ((ar >= start[:, None]) & (ar < torch.maximum(end, start + 1)[:, None])).long()
        refc, refr = -5 * torch.rand(P), -5 * torch.rand(P)
        n_types = rnd.choice([1, 1, 2])
        kw = dict(beta=rnd.choice([0.1, 0.5]), loss_types=tuple(rnd.sample(types, n_types)),
                  loss_weights=None if n_types == 1 else [0.7, 1.3], label_smoothing=rnd.choice([0.0, 0.1]),
                  ld_alpha=rnd.choice([None, None, 0.3]), use_weighting=rnd.random() < 0.25,
                  f_divergence_type=rnd.choice(["reverse_kl", "reverse_kl", "js_divergence", "alpha_divergence"]))
        ol = logits.float().clone().requires_grad_(True)
        oloss, _ = oracle.dpo_compute_loss(ol, ids, cm, refc, refr, f_alpha=0.5, **kw)
        if not math.isfinite(float(oloss.detach())) or abs(float(oloss.detach())) > 1e6:
            continue  # (exo_pair without label smoothing is log 0, an f-divergence may overflow: in the reference too)
        oloss.backward()
        gl = logits.clone().to(DEV).requires_grad_(True)
        gloss, _ = amd.dpo_compute_loss(gl, ids.to(DEV), cm.to(DEV), refc.to(DEV), refr.to(DEV), f_alpha_divergence_coef=0.5, **kw)
        gloss.backward()
        what = (case, kw["loss_types"], str(dt), kw["ld_alpha"], kw["use_weighting"], kw["f_divergence_type"])
        # (fp32: a sequence's summed log-probs are a few hundred, held to 3e-5 each way, and ipo squares their difference)
        tol = 5e-5 if dt == torch.float32 else 2e-2
        assert abs(float(gloss.detach()) - float(oloss.detach())) <= tol * max(1.0, abs(float(oloss.detach()))), what
        if float(ol.grad.abs().max()) > 1e-10:
            # (discopop puts the difference of two summed log-probs, each a few hundred and held to 3e-5, through a
            # sigmoid of temperature 0.05: twenty times that difference in the gradient coefficient, before its two
            # terms cancel)
            g32 = 2e-3 if "discopop" in kw["loss_types"] else 2e-4
            assert _rel(gl.grad.float(), ol.grad) <= (g32 if dt == torch.float32 else 2e-2), what
        else:
            assert float(gl.grad.float().abs().max()) <= 1e-7, what
        ran += 1
    assert ran >= 200


def test_fused_head_against_fp32_autograd(amd, monkeypatch):
    """120 fused-head problems: token / hidden / vocabulary sizes around the tile edges (1, 255, 256, 257, ...; hidden sizes that are no multiple
    of the 8-element vector too), chunk
    sizes, temperature, soft-capping, logit scale, bias, bf16 / fp16 / fp32 operands, with and without the stash,
    with and without tokens whose upstream gradient is zero."""
    rnd = random.Random(4)
    torch.manual_seed(4)
    for case in range(120):
        n, h = rnd.choice([1, 3, 64, 255, 256, 257, 300, 513, 700]), rnd.choice([8, 24, 64, 136, 256, 520, 5, 100])
        v = rnd.choice([2, 7, 255, 256, 257, 1000, 2305, 5000])
        chunk, T = rnd.choice([1, 100, 256, 1024, 8192]), rnd.choice([1.0, 0.7])
        cap, scale = rnd.choice([None, None, 5.0]), rnd.choice([1.0, 0.5])
        dt = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
        use_bias = rnd.random() < 0.3
        monkeypatch.setenv("TRL_AMD_HEAD_STASH_GIB", rnd.choice(["24", "0"]))
        hidden, weight = torch.randn(n, h).to(dt), (torch.randn(v, h) * (2.0 / h**0.5)).to(dt)
        bias = torch.randn(v).to(dt) if use_bias else None
        labels, gout = torch.randint(0, v, (n,)), torch.randn(n)
        if rnd.random() < 0.4:
            gout[torch.rand(n) < 0.6] = 0.0
        rh, rw = hidden.clone().float().requires_grad_(True), weight.clone().float().requires_grad_(True)
        rb = bias.clone().float().requires_grad_(True) if use_bias else None
        y0 = rh @ rw.t()
        y0.retain_grad()
        y = (y0 + rb if use_bias else y0) * scale
        if cap:
            y = torch.tanh(y / cap) * cap
        lsm = F.log_softmax(y / T, -1)
        rlp, rent = lsm.gather(-1, labels[:, None]).squeeze(-1), -(lsm.exp() * lsm).sum(-1)
        (rlp * gout).sum().backward()
        dh, dw = hidden.clone().to(DEV).requires_grad_(True), weight.clone().to(DEV).requires_grad_(True)
        db = bias.clone().to(DEV).requires_grad_(True) if use_bias else None
        lp, ent = amd._ChunkedLogProbFunction.apply(dh, dw, labels.to(DEV), T, chunk, cap, scale, db)
        (lp * gout.to(DEV)).sum().backward()
        what = (case, n, h, v, chunk, str(dt), cap, use_bias, os.environ["TRL_AMD_HEAD_STASH_GIB"])
        ftol = 1e-5 if dt == torch.float32 else 3e-3
        assert float((lp.detach().cpu() - rlp.detach()).abs().max()) <= ftol * max(1.0, float(rlp.detach().abs().max())), what
        assert float((ent.cpu() - rent.detach()).abs().max()) <= 4 * ftol, what
        # (a vocabulary of a few entries is ill-conditioned: d logits = g (1 - p) cancels for a target of probability
        # near 1, and the sums over tokens of a gradient of two or seven signed terms cancel again, so the rounding of
        # the 16-bit d logits -- and fp32's own -- shows in the relative error of the result)
        gtol = {torch.float32: 2e-5, torch.bfloat16: 1.2e-2, torch.float16: 2e-3}[dt]
        if v < 16:
            gtol = 2e-3 if dt == torch.float32 else 3e-2
        # The bar is relative to the gradient as it would be if its terms did not cancel (|d logits| against |hidden|
        # or |weight|): every term carries its own rounding, so that is what the error of a sum scales with, and the
        # sum itself can be far smaller (two tokens pulling a two-entry vocabulary in opposite directions).
        dy = y0.grad.abs()
        # A probability comes out of exp(y - lse) good to a few ulps of lse's magnitude, so a token's d logits carry
        # that fraction of its upstream gradient as an absolute error, however small g * (1 - p) itself is.
        ulps = 8 * 2.0**-24 * max(1.0, float(y.detach().abs().max()) / T) * float(gout.norm())
        pairs = [(dh.grad, rh.grad, dy @ rw.detach().abs(), ulps * float(rw.detach().norm(dim=1).max())),
                 (dw.grad, rw.grad, dy.t() @ rh.detach().abs(), ulps * float(rh.detach().norm(dim=1).max()))]
        if use_bias:
            pairs.append((db.grad, rb.grad, dy.sum(0), ulps))
        for got, want, uncancelled, arithmetic in pairs:
            if float(gout.abs().max()) == 0.0:
                assert float(got.float().abs().max()) == 0.0, what
            else:
                # (fp16 gradients are stored in fp16: entries under 6e-5 are subnormal, spaced 6e-8 apart whatever their
                # size, which is all the accuracy a gradient has when the one upstream gradient of the batch is 1e-4)
                floor = 2.0**-25 * got.numel() ** 0.5 if dt == torch.float16 else 0.0
                diff = float((got.double().cpu() - want.double()).norm())
                assert diff < gtol * float(uncancelled.double().norm()) + floor + arithmetic, (what, _rel(got, want))
    amd.check_device_errors()


def test_sft_chunked_loss_against_the_oracle(amd):
    """120 problems through the SFT `chunked_nll` loss: labels or pre-shifted labels with -100 holes (all of them
    in some), bias, logit scale, soft-capping, `num_items_in_batch`, bf16 / fp16 / fp32 operands; loss, argmax
    count, entropy sum and the gradients of hidden states, weight and bias against the oracle's autograd."""
    from trl_amd.trainer.sft_trainer import _chunked_cross_entropy_loss

    rnd = random.Random(10)
    torch.manual_seed(10)
    for case in range(120):
        B, S, H, V = rnd.choice([1, 2, 3]), rnd.choice([2, 7, 33]), rnd.choice([8, 64, 72]), rnd.choice([8, 250, 256, 1000])
        dt = rnd.choice([torch.float32, torch.bfloat16, torch.float16])
        hidden = torch.randn(B, S, H)
        weight = rnd.choice([0.05, 0.3]) * torch.randn(V, H)
        bias = 0.5 * torch.randn(V) if rnd.random() < 0.3 else None
        labels = torch.randint(0, V, (B, S))
        labels[torch.rand(B, S) < rnd.choice([0.0, 0.3, 1.0])] = -100
        shifted = rnd.random() < 0.4
        kw = dict(logit_scale=rnd.choice([1.0, 1.0, 0.5]), final_logit_softcapping=rnd.choice([None, None, 5.0]),
                  num_items_in_batch=rnd.choice([None, 17, torch.tensor(23.0)]))
        lab_kw = dict(shift_labels=labels) if shifted else dict(labels=labels)
        q = lambda t: None if t is None else t.to(dt)  # noqa: E731
        dev_in = [q(hidden).to(DEV).requires_grad_(True), q(weight).to(DEV).requires_grad_(True),
                  None if bias is None else q(bias).to(DEV).requires_grad_(True)]
        host_in = [q(hidden).float().requires_grad_(True), q(weight).float().requires_grad_(True),
                   None if bias is None else q(bias).float().requires_grad_(True)]
        got = _chunked_cross_entropy_loss(dev_in[0], dev_in[1], rnd.choice([16, 4096]), lm_head_bias=dev_in[2],
                                          **{k: v.to(DEV) for k, v in lab_kw.items()}, **kw)
        want = oracle.chunked_cross_entropy_loss(host_in[0], host_in[1], 64, lm_head_bias=host_in[2], **lab_kw, **kw)
        what = (case, B, S, H, V, str(dt), shifted, bias is not None, kw["logit_scale"], kw["final_logit_softcapping"])
        assert int(got[3]) == int(want[3]), what
        low = dt != torch.float32
        assert abs(float(got[0].detach()) - float(want[0].detach())) <= (2e-4 if low else 2e-5) * max(1.0, abs(float(want[0].detach()))), what
        assert abs(float(got[2].detach()) - float(want[2].detach())) <= (2e-4 if low else 2e-5) * max(1.0, abs(float(want[2].detach()))), what
        assert abs(float(got[1].detach()) - float(want[1].detach())) <= (1 if low else 0), what  # (a near-tie may flip under 16-bit products)
        got[0].backward()
        want[0].backward()
        for g_t, w_t, name in zip(dev_in, host_in, ("hidden", "weight", "bias")):
            if g_t is None:
                continue
            if float(w_t.grad.abs().max()) == 0.0:
                assert g_t.grad is None or float(g_t.grad.float().abs().max()) == 0.0, (what, name)
            else:
                assert _rel(g_t.grad, w_t.grad) <= (6e-3 if dt == torch.bfloat16 else 1e-3 if low else 2e-5), (what, name, _rel(g_t.grad, w_t.grad))
    amd.check_device_errors()


def test_rloo_and_kto_losses_against_the_oracle(amd):
    """150 RLOO problems (sequence-level clipped loss, its gradient and clip metrics) and 150 KTO problems (both loss
    types, class weights, with and without the KL baseline, all-desirable and all-undesirable batches, fp32 / bf16)."""
    rnd = random.Random(5)
    torch.manual_seed(5)
    for case in range(150):
        B, T = rnd.choice([1, 2, 7, 16]), rnd.choice([1, 9, 40])
        lp = -2 * torch.rand(B, T)
        mask = (torch.arange(T)[None] < torch.randint(0, T + 1, (B,))[:, None]).float()
        seq = (lp * mask).sum(1)
        old = seq + rnd.choice([0.0, 0.1, 0.5]) * torch.randn(B)
        adv = torch.randn(B)
        eps = (rnd.choice([0.2, 0.1]), rnd.choice([0.2, 0.3]))
        olp = lp.clone().requires_grad_(True)
        oloss, om = oracle.rloo_loss(olp, mask, old, adv, *eps)
        oloss.backward()
        glp = lp.to(DEV).requires_grad_(True)
        gloss, gseq, gm = amd.rloo_loss(glp, mask.to(DEV), old.to(DEV), adv.to(DEV), *eps)
        gloss.backward()
        assert abs(float(gloss.detach()) - float(oloss.detach())) <= 2e-5 * max(1.0, abs(float(oloss.detach()))), case
        torch.testing.assert_close(gseq.detach().cpu(), seq, rtol=1e-5, atol=1e-5)
        assert float((glp.grad.cpu() - olp.grad).abs().max()) <= 2e-5 * float(olp.grad.abs().max()) + 1e-7, case
        want = [om["clip_ratio/low_mean"], om["clip_ratio/low_min"], om["clip_ratio/high_mean"], om["clip_ratio/high_max"],
                om["clip_ratio/region_mean"]]
        torch.testing.assert_close(gm[:5].cpu(), torch.tensor(want), rtol=1e-5, atol=1e-6, equal_nan=True)
    for case in range(150):
        B, L, V = rnd.choice([1, 2, 6]), rnd.choice([2, 7, 20]), rnd.choice([5, 64, 257])
        dt = rnd.choice([torch.float32, torch.float32, torch.bfloat16])
        logits = (2.0 * torch.randn(B, L, V)).to(dt)
        ids = torch.randint(0, V, (B, L))
        start = torch.randint(0, L, (B,))
        cm = (torch.arange(L)[None] >= start[:, None]).long()
        label = torch.rand(B) < rnd.choice([0.0, 0.5, 0.5, 1.0])
        ref = -5 * torch.rand(B)
        with_kl = rnd.random() < 0.6
        kw = dict(kl_logps=-5 * torch.rand(B) if with_kl else None, ref_kl_logps=-5 * torch.rand(B) if with_kl else None,
                  beta=rnd.choice([0.1, 0.5]), loss_type=rnd.choice(["kto", "apo_zero_unpaired"]),
                  desirable_weight=rnd.choice([1.0, 1.33]), undesirable_weight=rnd.choice([1.0, 0.7]))
        ol = logits.float().clone().requires_grad_(True)
        oloss, _ = oracle.kto_compute_loss(ol, ids, cm, label, ref, **kw)
        oloss.backward()
        gl = logits.clone().to(DEV).requires_grad_(True)
        gkw = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in kw.items()}
        gloss, _ = amd.kto_compute_loss(gl, ids.to(DEV), cm.to(DEV), label.to(DEV), ref.to(DEV), **gkw)
        gloss.backward()
        what = (case, str(dt), kw["loss_type"], with_kl, label.tolist())
        tol = 2e-5 if dt == torch.float32 else 2e-2
        assert abs(float(gloss.detach()) - float(oloss.detach())) <= tol * max(1.0, abs(float(oloss.detach()))), what
        if float(ol.grad.abs().max()) > 1e-10:
            assert _rel(gl.grad.float(), ol.grad) <= (2e-4 if dt == torch.float32 else 2e-2), what
        else:
            assert gl.grad is None or float(gl.grad.float().abs().max()) <= 1e-7, what

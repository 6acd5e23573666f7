"""GPU parity of the single-pass GRPO operator (logits -> loss + dlogits in one kernel pass) against the
two-pass path (K1 log-probs, [B, T] loss kernel, K3 gradient), which the other GPU tests pin to the golden
vectors and the oracle.  Bars: loss and metrics 1e-5 relative, log-probs / entropies 1e-5 abs on the rows of the
mask (the other rows are 0 by contract), dlogits 2e-3 relative L2 (both sides round to bf16) with the rows
outside the mask exactly zero."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def amd():
    import trl_amd

    return trl_amd


def _inputs(B, K, V, dtype=torch.bfloat16, seed=0, extra_rows=3):
    g = torch.Generator(device=DEV).manual_seed(seed)
    L = K + extra_rows
    logits = (2.0 * torch.randn((B, L, V), generator=g, device=DEV)).to(dtype)
    ids = torch.randint(0, V, (B, K), generator=g, device=DEV)
    lengths = torch.randint(1, K + 1, (B,), generator=g, device=DEV)
    lengths[0] = 0  # a sequence without any active token
    mask = (torch.arange(K, device=DEV)[None] < lengths[:, None]).long()
    adv = torch.randn((B,), generator=g, device=DEV)
    return logits, ids, mask, adv, g


def _two_pass(amd, logits, ids, mask, adv, temperature, **kw):
    leaf = logits.detach().clone().requires_grad_(True)
    logp, ent = amd.per_token_logps_and_entropies(leaf, ids, ids.shape[1], temperature)
    loss, metrics = amd.grpo_loss(logp, adv, mask, entropies=ent, **kw)
    return leaf, loss, metrics, logp.detach(), ent.detach()


def _rel_l2(a, b):
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm().clamp(min=1e-30))


@pytest.mark.parametrize("loss_type", ["dapo", "grpo", "bnpo", "dr_grpo", "cispo", "sapo"])
@pytest.mark.parametrize("beta", [0.0, 0.04])
def test_matches_two_pass(amd, loss_type, beta):
    B, K, V, T = 8, 32, 4096, 0.9
    logits, ids, mask, adv, g = _inputs(B, K, V, seed=3)
    with torch.no_grad():
        base, _ = amd.per_token_logps_and_entropies(logits, ids, K, T)
    old = base + 0.3 * torch.randn(base.shape, generator=g, device=DEV)
    ref = base + 0.1 * torch.randn(base.shape, generator=g, device=DEV)
    kw = dict(old_per_token_logps=old, ref_per_token_logps=ref if beta else None, loss_type=loss_type, epsilon_low=0.2,
              epsilon_high=0.28, beta=beta, max_completion_length=K, num_items_in_batch=mask.sum().float(),
              grad_accum_steps=2.0)
    leaf, loss2, met2, lp2, ent2 = _two_pass(amd, logits, ids, mask, adv, T, **kw)
    loss2.backward()
    leaf1 = logits.detach().clone().requires_grad_(True)
    loss1, met1, lp1, ent1 = amd.grpo_loss_from_logits(leaf1, ids, adv, mask, temperature=T, **kw)
    loss1.backward()
    torch.testing.assert_close(loss1, loss2, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(met1, met2, rtol=1e-5, atol=1e-6, equal_nan=True)
    m = mask.bool()
    torch.testing.assert_close(lp1[m], lp2[m], rtol=0, atol=1e-5)
    torch.testing.assert_close(ent1[m], ent2[m], rtol=0, atol=1e-5)
    assert float(lp1[~m].abs().max()) == 0.0 and float(ent1[~m].abs().max()) == 0.0
    g1, g2 = leaf1.grad, leaf.grad
    assert g1.shape == logits.shape and g1.dtype == logits.dtype
    assert _rel_l2(g1, g2) < 2e-3
    # rows outside the window or the mask: exactly zero on both sides
    full_mask = torch.zeros(logits.shape[:2], dtype=torch.bool, device=DEV)
    start = logits.shape[1] - 1 - K
    full_mask[:, start:start + K] = m
    assert float(g1[~full_mask].abs().max()) == 0.0 and float(g2[~full_mask].abs().max()) == 0.0
    # every gradient row sums to zero up to the rounding of its 4096 bf16 entries
    assert float(g1.float().sum(-1).abs().max()) < 1e-3
    # with the rows outside the mask computed too: their outputs match the two-pass values, nothing else moves
    leaf3 = logits.detach().clone().requires_grad_(True)
    loss3, met3, lp3, ent3 = amd.grpo_loss_from_logits(leaf3, ids, adv, mask, temperature=T, skip_masked_rows=False, **kw)
    loss3.backward()
    torch.testing.assert_close(lp3, lp2, rtol=0, atol=1e-5)
    torch.testing.assert_close(ent3, ent2, rtol=0, atol=1e-5)
    assert torch.equal(loss3, loss1) and torch.equal(leaf3.grad, g1)
    amd.check_device_errors()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rows_that_leave_the_fast_reduction(amd, dtype):
    """The kernel sums the exponentials against the maximum of a lane's FIRST vector while the row still arrives; a
    row whose later logits exceed that by more than 128 / (log2(e) / T), or that holds an infinity or a NaN, takes
    the exact two-sweep reduction instead.  Such rows -- a spike late in the row, a wide ramp, -inf entries (a masked
    vocabulary), one +inf, one NaN -- against the two-pass path and, where the row is finite, against float64."""
    B, K, V, T = 4, 12, 8192, 0.7
    logits, ids, _, adv, g = _inputs(B, K, V, dtype=dtype, seed=21, extra_rows=1)
    mask = torch.ones((B, K), dtype=torch.long, device=DEV)
    big = 30000.0 if dtype == torch.float16 else 1e4
    x = logits.float()
    x[0, 0, V - 5] = 300.0                                   # one spike at the end of the row
    x[0, 1] = torch.linspace(-400.0, 400.0, V, device=DEV)   # a ramp: every later vector is larger than the first
    x[0, 2, 1024:] = float("-inf")                           # most of the vocabulary masked out
    x[0, 3] = float("-inf")
    x[0, 3, 77] = 1.5                                        # a single admissible token
    x[0, 4, 4000] = big                                      # near the largest finite value of the dtype
    x[0, 5, 123] = float("inf")
    x[0, 6, 4567] = float("nan")
    x[1, 0, :8] = -300.0                                     # the FIRST vector far below the rest
    ids[0, 2], ids[0, 3] = 5, 77
    logits = x.to(dtype)
    kw = dict(loss_type="grpo", epsilon_low=0.2, epsilon_high=0.28, beta=0.0, max_completion_length=K,
              num_items_in_batch=mask.sum().float())
    leaf2, loss2, _, lp2, ent2 = _two_pass(amd, logits, ids, mask, adv, T, **kw)
    loss2.backward()
    leaf1 = logits.detach().clone().requires_grad_(True)
    loss1, _, lp1, ent1 = amd.grpo_loss_from_logits(leaf1, ids, adv, mask, temperature=T, **kw)
    loss1.backward()
    torch.testing.assert_close(lp1, lp2, rtol=1e-5, atol=1e-5, equal_nan=True)
    # (the entropy is lse - E_p[z] on both paths, as in the reference's fused operator, utils.py:1357: its absolute
    # error grows with the size of the logits, two fp32 steps of the largest |z| of the row)
    zmax = (logits[:, :K].float().nan_to_num(nan=0.0, posinf=0.0, neginf=0.0).abs().amax(-1) / T)
    ent_tol = 2e-5 + 2.5e-7 * zmax
    ok = ((ent1 - ent2).abs() <= ent_tol) | (torch.isnan(ent1) & torch.isnan(ent2))
    assert bool(ok.all()), (ent1 - ent2).abs().max()
    g1, g2 = leaf1.grad[:, :K].float(), leaf2.grad[:, :K].float()
    bad = torch.zeros((B, K), dtype=torch.bool, device=DEV)
    bad[0, 5] = bad[0, 6] = True  # +inf / NaN rows: NaN outputs on both paths, as the reference's log_softmax gives
    assert bool(torch.isnan(lp1[bad]).all()) and bool(torch.isnan(lp2[bad]).all())
    finite = ~bad
    assert bool(torch.isfinite(lp1[finite]).all()) and bool(torch.isfinite(g1[finite]).all())
    for b, t in ((0, 0), (0, 1), (0, 2), (0, 3), (0, 4), (1, 0), (2, 3)):
        assert float((g1[b, t] - g2[b, t]).norm()) <= 2e-3 * float(g2[b, t].norm()) + 1e-7, (b, t)
        z = logits[b, t].double() / T
        want = torch.log_softmax(z, -1)
        assert abs(float(lp1[b, t]) - float(want[ids[b, t]])) < 1e-5 * max(1.0, abs(float(want[ids[b, t]]))), (b, t)
        if bool(torch.isinf(z).any()):  # the reference's -sum p log p is NaN for a row with a -inf logit (0 * -inf)
            assert math.isnan(float(ent1[b, t])) and math.isnan(float(ent2[b, t]))
            continue
        h = -(want.exp() * want).sum()
        assert abs(float(ent1[b, t]) - float(h)) < float(ent_tol[b, t]) + 2e-5 * float(h), (b, t, float(ent1[b, t]), float(h))
    # the single admissible token: log-prob 0, gradient zero (the entropy of a row with -inf entries is NaN, as the
    # reference's -sum p log p is)
    assert abs(float(lp1[0, 3])) < 1e-6 and float(g1[0, 3].abs().max()) < 1e-6


def test_window_given_by_keep_start(amd):
    """`keep_start` places the K-row window anywhere in the logits (here: all rows, no position dropped)."""
    B, K, V = 3, 8, 512
    logits, ids, mask, adv, _ = _inputs(B, K, V, seed=17, extra_rows=0)
    leaf = logits.detach().clone().requires_grad_(True)
    lp2, ent2 = amd.logps_and_entropies(leaf, ids, 1.0)
    loss2, _ = amd.grpo_loss(lp2, adv, mask, entropies=ent2.detach(), loss_type="bnpo")
    loss2.backward()
    leaf1 = logits.detach().clone().requires_grad_(True)
    loss1, _, lp1, _ = amd.grpo_loss_from_logits(leaf1, ids, adv, mask, loss_type="bnpo", keep_start=0, skip_masked_rows=False)
    loss1.backward()
    torch.testing.assert_close(loss1, loss2, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(lp1, lp2.detach(), rtol=0, atol=1e-5)
    assert _rel_l2(leaf1.grad, leaf.grad) < 2e-3
    with pytest.raises(ValueError):
        amd.grpo_loss_from_logits(leaf1, ids, adv, mask, loss_type="bnpo", keep_start=1)


@pytest.mark.parametrize("loss_type", ["dapo", "grpo", "bnpo"])
def test_entropy_bonus_matches_two_pass(amd, loss_type):
    """With an entropy bonus the gradient also has the entropy's own term (through every logit of the row)."""
    B, K, V, T = 6, 24, 2048, 0.8
    logits, ids, mask, adv, g = _inputs(B, K, V, seed=31)
    with torch.no_grad():
        base, _ = amd.per_token_logps_and_entropies(logits, ids, K, T)
    kw = dict(old_per_token_logps=base + 0.2 * torch.randn(base.shape, generator=g, device=DEV), loss_type=loss_type,
              num_items_in_batch=mask.sum().float() * 2, grad_accum_steps=2.0, entropy_coef=0.05)
    leaf = logits.detach().clone().requires_grad_(True)
    logp, ent = amd.per_token_logps_and_entropies(leaf, ids, K, T, True, True)
    loss2, met2 = amd.grpo_loss(logp, adv, mask, entropies=ent, **kw)
    loss2.backward()
    leaf1 = logits.detach().clone().requires_grad_(True)
    loss1, met1, _, _ = amd.grpo_loss_from_logits(leaf1, ids, adv, mask, temperature=T, **kw)
    loss1.backward()
    torch.testing.assert_close(loss1, loss2, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(met1, met2, rtol=1e-5, atol=1e-6, equal_nan=True)
    assert _rel_l2(leaf1.grad, leaf.grad) < 2e-3
    # the entropy term is really there: without it the gradient is a different one
    leaf0 = logits.detach().clone().requires_grad_(True)
    amd.grpo_loss_from_logits(leaf0, ids, adv, mask, temperature=T, **dict(kw, entropy_coef=0.0))[0].backward()
    assert _rel_l2(leaf0.grad, leaf.grad) > 1e-2


def test_upstream_gradient_scales(amd):
    B, K, V = 4, 16, 2048
    logits, ids, mask, adv, _ = _inputs(B, K, V, seed=5)
    kw = dict(loss_type="dapo", num_items_in_batch=mask.sum().float(), temperature=1.0)
    a = logits.detach().clone().requires_grad_(True)
    amd.grpo_loss_from_logits(a, ids, adv, mask, **kw)[0].backward()
    b = logits.detach().clone().requires_grad_(True)
    (amd.grpo_loss_from_logits(b, ids, adv, mask, **kw)[0] * 0.25).backward()
    torch.testing.assert_close(b.grad.float(), a.grad.float() * 0.25, rtol=1e-2, atol=0)  # 0.25 is exact in bf16
    assert _rel_l2(b.grad.float(), a.grad.float() * 0.25) == 0.0


def test_scale_kernel_reaches_every_element(amd):
    """`ops.scale_unless_one_` on buffers from one element to many pieces per workgroup and region (its workgroups
    step through eight regions of the buffer piece by piece): every element scaled exactly once, bit for bit what
    torch gives; a scale of 1 leaves the buffer as it is."""
    from trl_amd import ops

    g = torch.Generator(device=DEV).manual_seed(91)
    piece = 8 * 1024  # 16-bit elements of one 16 KiB piece
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        per = piece if dtype != torch.float32 else piece // 2
        for n in (1, 5, 8, per - 1, per, 3 * per + 1, 8 * per, 9 * per + 7, 520 * per + 13, (64 * 8 * 2 + 77) * per + 5):
            x = torch.randn((n,), generator=g, device=DEV).to(dtype)
            want = (x.float() * 0.37).to(dtype)
            got = ops.scale_unless_one_(x.clone(), torch.tensor(0.37, device=DEV))
            assert torch.equal(got, want), (dtype, n)
            same = ops.scale_unless_one_(x.clone(), torch.tensor(1.0, device=DEV))
            assert torch.equal(same, x), (dtype, n)


def test_fp16_and_token_weight_and_per_token_advantages(amd):
    B, K, V = 4, 24, 1024
    logits, ids, mask, _, g = _inputs(B, K, V, dtype=torch.float16, seed=7)
    adv = torch.randn((B, K), generator=g, device=DEV)
    tw = torch.rand((B, K), generator=g, device=DEV)
    kw = dict(loss_type="grpo", token_weight=tw, delta=1.5, epsilon_low=0.1, epsilon_high=0.3)
    with torch.no_grad():
        base, _ = amd.per_token_logps_and_entropies(logits, ids, K, 0.7)
    kw["old_per_token_logps"] = base + 0.5 * torch.randn(base.shape, generator=g, device=DEV)
    leaf, loss2, met2, _, _ = _two_pass(amd, logits, ids, mask, adv, 0.7, **kw)
    loss2.backward()
    leaf1 = logits.detach().clone().requires_grad_(True)
    loss1, met1, _, _ = amd.grpo_loss_from_logits(leaf1, ids, adv, mask, temperature=0.7, **kw)
    loss1.backward()
    torch.testing.assert_close(loss1, loss2, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(met1, met2, rtol=1e-5, atol=1e-6, equal_nan=True)
    assert _rel_l2(leaf1.grad, leaf.grad) < 2e-3


def test_real_vocabulary_and_limits(amd):
    """A row of 151936 logits (19 vectors per lane, the last one ragged) and the largest supported row."""
    for V in (151936, 163840):
        B, K = 2, 6
        logits, ids, mask, adv, _ = _inputs(B, K, V, seed=V % 97, extra_rows=1)
        mask[:] = 1
        mask[1, 4:] = 0
        ids[0, 0], ids[0, 1] = 0, V - 1
        kw = dict(loss_type="bnpo", beta=0.0)
        leaf, loss2, met2, lp2, ent2 = _two_pass(amd, logits, ids, mask, adv, 0.9, **kw)
        loss2.backward()
        leaf1 = logits.detach().clone().requires_grad_(True)
        loss1, met1, lp1, ent1 = amd.grpo_loss_from_logits(leaf1, ids, adv, mask, temperature=0.9, **kw)
        loss1.backward()
        m = mask.bool()
        torch.testing.assert_close(loss1, loss2, rtol=1e-5, atol=1e-7)
        torch.testing.assert_close(lp1[m], lp2[m], rtol=0, atol=1e-5)
        torch.testing.assert_close(ent1[m], ent2[m], rtol=0, atol=1e-5)
        assert _rel_l2(leaf1.grad, leaf.grad) < 2e-3
    amd.check_device_errors()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_rows_that_overflow_into_lds(amd, dtype):
    """Rows longer than the registers hold (more than 163840 logits): the rest of the row waits in the CU's LDS, and
    what does not fit there either (more than 237568 logits) is read twice.  Vocabularies of current 200k- and
    256k-entry tokenizers, one that ends inside every LDS build (3, 6, 9 vectors per lane), the first sizes past the
    registers and past the LDS, and the largest one; targets in the register part, in the LDS part and on the
    row's last entry; entropy bonus on (its gradient term runs over the LDS part too).  Against the two-pass path,
    and log-probs / entropies / gradient of one case against the oracle."""
    import oracle

    assert amd.ops.grpo_fused_max_vocab(dtype) == 41 * 1024 * 8
    # (beyond 29 * 8192 = 237568 logits the last vectors of a row are read twice instead of kept: 256000, 262144, ...)
    for V in (163848, 180000, 200064, 202048, 221184, 237568, 237576, 256000, 262144, 335872):
        B, K = 2, 3
        logits, ids, mask, adv, g = _inputs(B, K, V, dtype=dtype, seed=V % 89, extra_rows=1)
        mask[:] = 1
        mask[1, 2] = 0
        ids[0, 0], ids[0, 1], ids[0, 2], ids[1, 0] = 5, 163840 + 7, V - 1, 20 * 8192 - 1
        assert amd.grpo_single_pass_supported(logits)
        kw = dict(loss_type="bnpo", beta=0.0, entropy_coef=0.02 if V % 3 == 0 else 0.0)
        leaf, loss2, met2, lp2, ent2 = _two_pass(amd, logits, ids, mask, adv, 0.9, **kw) if not kw["entropy_coef"] else (None,) * 5
        if leaf is None:
            leaf = logits.detach().clone().requires_grad_(True)
            lp_g, ent_g = amd.per_token_logps_and_entropies(leaf, ids, K, 0.9, True, True)
            loss2, met2 = amd.grpo_loss(lp_g, adv, mask, entropies=ent_g, **kw)
            lp2, ent2 = lp_g.detach(), ent_g.detach()
        loss2.backward()
        leaf1 = logits.detach().clone().requires_grad_(True)
        loss1, met1, lp1, ent1 = amd.grpo_loss_from_logits(leaf1, ids, adv, mask, temperature=0.9, **kw)
        loss1.backward()
        m = mask.bool()
        torch.testing.assert_close(loss1, loss2, rtol=1e-5, atol=1e-7)
        torch.testing.assert_close(lp1[m], lp2[m], rtol=0, atol=1e-5)
        torch.testing.assert_close(ent1[m], ent2[m], rtol=0, atol=1e-5)
        assert _rel_l2(leaf1.grad, leaf.grad) < 2e-3, V
        assert float(leaf1.grad[1, 2].float().abs().max()) == 0.0 and float(leaf1.grad[:, K:].float().abs().max()) == 0.0
        assert float(leaf1.grad[0, 0, 163840:].float().abs().max()) > 0.0  # the part of the row that came through LDS
        if V == 200064:
            cpu_leaf = logits.detach().float().cpu().requires_grad_(True)
            lp, ent = oracle.logps_and_entropies_from_logits(cpu_leaf, ids.cpu(), K, 0.9, True)
            want, _ = oracle.grpo_loss(lp, adv.cpu(), mask.cpu(), entropies=ent, loss_type="bnpo", beta=0.0,
                                       entropy_coef=kw["entropy_coef"])
            want.backward()
            torch.testing.assert_close(lp1.cpu()[m.cpu()], lp.detach()[m.cpu()], atol=2e-3, rtol=0)
            torch.testing.assert_close(ent1.cpu()[m.cpu()], ent.detach()[m.cpu()], atol=2e-3, rtol=0)
            torch.testing.assert_close(loss1.detach().cpu(), want.detach(), atol=1e-6, rtol=1e-3)
            assert _rel_l2(leaf1.grad.float().cpu(), cpu_leaf.grad) < 5e-3
    amd.check_device_errors()


def test_fp32_logits(amd):
    """fp32 logits (four per 16-byte vector): rows that fit the registers (32000), that overflow into LDS (100000)
    and whose end is read twice (151936, 167936); the gradient is fp32 and not rounded, so it agrees with the
    two-pass path to fp32 rounding, and with the oracle's autograd on one case."""
    import oracle

    assert amd.ops.grpo_fused_max_vocab(torch.float32) == 41 * 1024 * 4
    for V in (32000, 81920, 100000, 151936, 167936):
        B, K = 2, 3
        logits, ids, mask, adv, g = _inputs(B, K, V, dtype=torch.float32, seed=V % 83, extra_rows=1)
        mask[:] = 1
        mask[1, 2] = 0
        ids[0, 0], ids[0, 1], ids[0, 2] = 3, V // 2 + 1, V - 1
        assert amd.grpo_single_pass_supported(logits)
        with torch.no_grad():
            base, _ = amd.per_token_logps_and_entropies(logits, ids, K, 0.9)
        kw = dict(loss_type="dapo", beta=0.04, old_per_token_logps=base + 0.3 * torch.randn(base.shape, generator=g, device=DEV),
                  ref_per_token_logps=base - 0.1, num_items_in_batch=mask.sum().float(), epsilon_low=0.2, epsilon_high=0.28)
        leaf, loss2, met2, lp2, ent2 = _two_pass(amd, logits, ids, mask, adv, 0.9, **kw)
        loss2.backward()
        leaf1 = logits.detach().clone().requires_grad_(True)
        loss1, met1, lp1, ent1 = amd.grpo_loss_from_logits(leaf1, ids, adv, mask, temperature=0.9, **kw)
        loss1.backward()
        assert leaf1.grad.dtype == torch.float32
        m = mask.bool()
        torch.testing.assert_close(loss1, loss2, rtol=1e-5, atol=1e-7)
        torch.testing.assert_close(met1, met2, rtol=1e-5, atol=1e-6, equal_nan=True)
        torch.testing.assert_close(lp1[m], lp2[m], rtol=0, atol=1e-5)
        torch.testing.assert_close(ent1[m], ent2[m], rtol=0, atol=1e-5)
        assert _rel_l2(leaf1.grad, leaf.grad) < 2e-5, V
        assert float(leaf1.grad[1, 2].abs().max()) == 0.0 and float(leaf1.grad[:, K:].abs().max()) == 0.0
        if V == 100000:
            cpu_leaf = logits.detach().cpu().requires_grad_(True)
            lp, ent = oracle.logps_and_entropies_from_logits(cpu_leaf, ids.cpu(), K, 0.9, True)
            okw = {k: (v.cpu() if torch.is_tensor(v) else v) for k, v in kw.items()}
            want, _ = oracle.grpo_loss(lp, adv.cpu(), mask.cpu(), entropies=ent, **okw)
            want.backward()
            torch.testing.assert_close(lp1.cpu()[m.cpu()], lp.detach()[m.cpu()], atol=2e-5, rtol=0)
            torch.testing.assert_close(loss1.detach().cpu(), want.detach(), atol=1e-6, rtol=1e-5)
            assert _rel_l2(leaf1.grad.cpu(), cpu_leaf.grad) < 2e-5
    # an upstream gradient other than 1 scales the fp32 buffer in place
    leaf1 = logits.detach().clone().requires_grad_(True)
    loss1, _, _, _ = amd.grpo_loss_from_logits(leaf1, ids, adv, mask, temperature=0.9, **kw)
    (loss1 * 3.0).backward()
    assert _rel_l2(leaf1.grad, 3.0 * leaf.grad) < 2e-5
    amd.check_device_errors()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bf16", "fp16", "fp32"])
def test_rows_that_are_not_whole_vectors(amd, dtype):
    """Vocabularies that are no multiple of the 16-byte vector (50257, 32001 and 151665 after a tokenizer gained
    tokens; sizes that also overflow into LDS or are read twice at the end): every row sits at another alignment,
    the kernel peels it to its first 16-byte boundary.  Targets in the peeled head, in the last elements and in
    the body; entropy bonus on; a view whose rows are aligned while the gradient's are not.  Against the two-pass
    path (itself checked against fp64 on such rows)."""
    per_vec = 16 // torch.empty((), dtype=dtype).element_size()
    sizes = [2 * per_vec + 1, 41, 1019, 32001, 50257, 151665]
    sizes += [83971] if dtype == torch.float32 else [200067, 262147]
    for V in sizes:
        B, K = 3, 3
        logits, ids, mask, adv, g = _inputs(B, K, V, dtype=dtype, seed=V % 79, extra_rows=1)
        mask[:] = 1
        mask[2, 1:] = 0
        ids[0, 0], ids[0, 1], ids[0, 2] = 0, V - 1, V // 2
        ids[1, 0], ids[1, 1], ids[1, 2] = min(3, V - 1), V - 2, 1
        assert amd.grpo_single_pass_supported(logits)
        kw = dict(loss_type="bnpo", beta=0.0, entropy_coef=0.02 if V % 2 else 0.0)
        leaf = logits.detach().clone().requires_grad_(True)
        lp_g, ent_g = amd.per_token_logps_and_entropies(leaf, ids, K, 0.9, True, True)
        loss2, met2 = amd.grpo_loss(lp_g, adv, mask, entropies=ent_g, **kw)
        loss2.backward()
        leaf1 = logits.detach().clone().requires_grad_(True)
        loss1, met1, lp1, ent1 = amd.grpo_loss_from_logits(leaf1, ids, adv, mask, temperature=0.9, **kw)
        loss1.backward()
        m = mask.bool()
        torch.testing.assert_close(loss1, loss2, rtol=1e-5, atol=1e-7)
        torch.testing.assert_close(met1, met2, rtol=1e-5, atol=1e-6, equal_nan=True)
        torch.testing.assert_close(lp1[m], lp_g.detach()[m], rtol=0, atol=1e-5)
        torch.testing.assert_close(ent1[m], ent_g.detach()[m], rtol=0, atol=1e-5)
        assert _rel_l2(leaf1.grad, leaf.grad) < (2e-5 if dtype == torch.float32 else 2e-3), V
        assert float(leaf1.grad[2, 1:].float().abs().max()) == 0.0  # masked rows and the row past the window: exact zeros
        # an upstream gradient other than 1: the buffer (not a whole number of vectors) is scaled in place; and the
        # rows outside the mask read for their log-probs and entropies as well
        leaf3 = logits.detach().clone().requires_grad_(True)
        loss3, _, lp3, ent3 = amd.grpo_loss_from_logits(leaf3, ids, adv, mask, temperature=0.9, skip_masked_rows=False, **kw)
        (loss3 * 0.5).backward()
        assert _rel_l2(leaf3.grad.float(), 0.5 * leaf1.grad.float()) < (1e-6 if dtype == torch.float32 else 3e-3), V
        torch.testing.assert_close(lp3, lp_g.detach(), rtol=0, atol=1e-5)
        torch.testing.assert_close(ent3, ent_g.detach(), rtol=0, atol=1e-5)
    # rows of the logits aligned (a slice of a wider tensor), rows of the gradient not
    wide, ids, mask, adv, g = _inputs(2, 3, 1024, dtype=dtype, seed=5, extra_rows=1)
    mask[:] = 1
    view = wide[..., :1019]
    ids = ids.clamp(max=1018)
    assert amd.grpo_single_pass_supported(view)
    leaf = view.detach().clone().requires_grad_(True)
    lp_g, ent_g = amd.per_token_logps_and_entropies(leaf, ids, 3, 1.0, True, False)
    loss2, _ = amd.grpo_loss(lp_g, adv, mask, entropies=ent_g, loss_type="bnpo")
    loss2.backward()
    src = wide.detach().clone().requires_grad_(True)
    loss1, _, _, _ = amd.grpo_loss_from_logits(src[..., :1019], ids, adv, mask, loss_type="bnpo")
    loss1.backward()
    torch.testing.assert_close(loss1, loss2, rtol=1e-5, atol=1e-7)
    assert _rel_l2(src.grad[..., :1019], leaf.grad) < (2e-5 if dtype == torch.float32 else 2e-3)
    assert float(src.grad[..., 1019:].float().abs().max()) == 0.0
    amd.check_device_errors()


def test_unsupported_configurations_raise(amd):
    logits, ids, mask, adv, _ = _inputs(2, 4, 1024)
    assert amd.grpo_single_pass_supported(logits)
    assert amd.grpo_single_pass_supported(logits.float()) and not amd.grpo_single_pass_supported(logits.double())
    assert amd.grpo_single_pass_supported(logits.float()[..., :1022]) and amd.grpo_single_pass_supported(logits[..., :1019])
    assert not amd.grpo_single_pass_supported(logits[..., :15]) and not amd.grpo_single_pass_supported(logits[..., ::2])
    assert not amd.grpo_single_pass_supported(logits, "vespo")
    assert not amd.grpo_single_pass_supported(logits, "dapo", "sequence")
    assert amd.grpo_single_pass_supported(logits, entropy_coef=0.01)
    assert not amd.grpo_single_pass_supported(logits, entropy_mask=mask)
    big = torch.empty((1, 2, amd.ops.grpo_fused_max_vocab(torch.bfloat16) + 8), dtype=torch.bfloat16, device=DEV)
    assert not amd.grpo_single_pass_supported(big)
    with pytest.raises(NotImplementedError):
        amd.grpo_loss_from_logits(logits.double(), ids, adv, mask, loss_type="bnpo")
    with pytest.raises(KeyError):
        amd.grpo_loss_from_logits(logits, ids, adv, mask, loss_type="dapo")
    with pytest.raises(KeyError):
        amd.grpo_loss_from_logits(logits, ids, adv, mask, loss_type="bnpo", beta=0.1)


def test_index_out_of_range_is_flagged(amd):
    logits, ids, mask, adv, _ = _inputs(2, 4, 1024, seed=9)
    mask[:] = 1
    ids[1, 2] = 1024
    leaf = logits.detach().clone().requires_grad_(True)
    loss, _, lp, _ = amd.grpo_loss_from_logits(leaf, ids, adv, mask, loss_type="bnpo")
    assert math.isnan(float(lp[1, 2]))
    with pytest.raises(IndexError):
        amd.check_device_errors()


@pytest.mark.parametrize("loss_type,beta,is_ratio,ent_coef", [("dapo", 0.04, False, 0.0), ("grpo", 0.0, True, 0.0),
                                                              ("cispo", 0.0, False, 0.0), ("dapo", 0.0, False, 0.02)])
def test_trainer_method_takes_the_single_pass(amd, loss_type, beta, is_ratio, ent_coef):
    """`GRPOLossMixin._compute_loss` on a mocked trainer: with 16-bit logits and a token-level loss it goes
    through the one-pass operator (the log-prob method is never called) and logs the same metrics, returns
    the same loss and leaves the same gradient as with `trl_amd_single_pass = False`."""
    from types import SimpleNamespace

    from test_gpu_losses import _fake_trainer

    B, P, K, V = 6, 3, 20, 1024
    g = torch.Generator(device=DEV).manual_seed(13)
    logits = (2.0 * torch.randn((B, P + K, V), generator=g, device=DEV)).bfloat16()
    completion_ids = torch.randint(0, V, (B, K), generator=g, device=DEV)
    lengths = torch.randint(1, K + 1, (B,), generator=g, device=DEV)
    cmask = (torch.arange(K, device=DEV)[None] < lengths[:, None]).long()
    with torch.no_grad():
        ids_all = torch.cat([torch.zeros((B, P), dtype=torch.long, device=DEV), completion_ids], 1)
        base, _ = amd.per_token_logps_and_entropies(logits, ids_all, K, 0.8)
    inputs = dict(
        prompt_ids=torch.zeros((B, P), dtype=torch.long, device=DEV), prompt_mask=torch.ones((B, P), dtype=torch.long, device=DEV),
        completion_ids=completion_ids, completion_mask=cmask, advantages=torch.randn((B,), generator=g, device=DEV),
        num_items_in_batch=cmask.sum().float(), old_per_token_logps=base + 0.3 * torch.randn(base.shape, generator=g, device=DEV),
        ref_per_token_logps=base + 0.1 * torch.randn(base.shape, generator=g, device=DEV),
        importance_sampling_ratio=0.5 + torch.rand((B, K), generator=g, device=DEV))
    case = dict(temperature=0.8, beta=beta, loss_type=loss_type, eps_low=0.2, eps_high=0.28, is_ratio=is_ratio, grad_accum=2,
                entropy_coef=ent_coef)
    results = []
    for single in (False, True):
        tr = _fake_trainer(amd, case, K, skip_masked=True, single_pass=single)
        leaf = logits.detach().clone().requires_grad_(True)
        calls = []
        inner = tr._get_per_token_logps_and_entropies
        tr._get_per_token_logps_and_entropies = lambda *a, _i=inner, **k: (calls.append(1), _i(*a, **k))[1]
        loss = tr._compute_loss(lambda **kw: SimpleNamespace(logits=leaf, aux_loss=None), inputs)
        loss.backward()
        assert bool(calls) == (not single)
        results.append((loss.detach(), leaf.grad, {k: v[-1] for k, v in tr._metrics["train"].items()}))
    (l2, g2, m2), (l1, g1, m1) = results
    torch.testing.assert_close(l1, l2, rtol=1e-5, atol=1e-7)
    assert _rel_l2(g1, g2) < 2e-3
    assert m1.keys() == m2.keys()
    for k in m2:
        assert (math.isnan(m1[k]) and math.isnan(m2[k])) or abs(m1[k] - m2[k]) <= 1e-5 * max(1.0, abs(m2[k])), k


def test_trainer_method_picks_the_path_by_row_length(amd, monkeypatch):
    """Without `trl_amd_single_pass` on the trainer the one pass is taken for rows of at least 40 KiB only (shorter
    rows are faster through the two kernels); `True` takes it for every row the kernel accepts, `False` never."""
    from types import SimpleNamespace

    from test_gpu_losses import _fake_trainer
    from trl_amd import ops

    B, P, K = 2, 1, 5
    g = torch.Generator(device=DEV).manual_seed(17)
    case = dict(temperature=1.0, beta=0.0, loss_type="dapo", eps_low=0.2, eps_high=0.2)
    calls = []
    inner = ops.grpo_fused_fwd_bwd
    monkeypatch.setattr(ops, "grpo_fused_fwd_bwd", lambda *a, **k: (calls.append(1), inner(*a, **k))[1])
    for V, dtype, want, expect in ((1024, torch.bfloat16, None, 0), (20480, torch.bfloat16, None, 1), (20472, torch.bfloat16, None, 0),
                                   (10240, torch.float32, None, 1), (1024, torch.bfloat16, True, 1),
                                   (20480, torch.bfloat16, False, 0)):
        logits = torch.randn((B, P + K, V), generator=g, device=DEV).to(dtype)
        completion_ids = torch.randint(0, V, (B, K), generator=g, device=DEV)
        cmask = torch.ones((B, K), dtype=torch.long, device=DEV)
        inputs = dict(prompt_ids=torch.zeros((B, P), dtype=torch.long, device=DEV),
                      prompt_mask=torch.ones((B, P), dtype=torch.long, device=DEV), completion_ids=completion_ids,
                      completion_mask=cmask, advantages=torch.randn((B,), generator=g, device=DEV),
                      num_items_in_batch=cmask.sum().float())
        tr = _fake_trainer(amd, case, K, skip_masked=True, single_pass=want)
        if want is None:
            del tr.trl_amd_single_pass
        leaf = logits.detach().clone().requires_grad_(True)
        del calls[:]
        tr._compute_loss(lambda **kw: SimpleNamespace(logits=leaf, aux_loss=None), inputs).backward()
        assert len(calls) == expect, (V, dtype, want)
        assert leaf.grad is not None and torch.isfinite(leaf.grad.float()).all()


@pytest.mark.parametrize("loss_type", ["dapo", "grpo", "dr_grpo", "bnpo"])
def test_against_the_oracle_autograd(amd, loss_type):
    """Independent of the two-pass kernels: the CPU oracle's log-probs, loss and autograd gradient on the same
    stored bf16 logits (fp32 op-math).  Log-probs 2e-3 abs, loss 1e-3 relative, dlogits 5e-3 relative L2 (the
    output is rounded to bf16)."""
    import oracle

    B, L, K, V, temp = 4, 9, 6, 4096, 0.9
    g = torch.Generator().manual_seed(2)
    logits = (2.0 * torch.randn(B, L, V, generator=g)).bfloat16()
    ids = torch.randint(0, V, (B, L), generator=g)
    mask = (torch.arange(K)[None] < torch.tensor([6, 3, 0, 5])[:, None]).long()
    adv = torch.randn(B, generator=g)
    with torch.no_grad():
        base, _ = oracle.logps_and_entropies_from_logits(logits.float(), ids, K, temp, False)
    old, ref = base + 0.2 * torch.randn(base.shape, generator=g), base - 0.1
    kw = dict(loss_type=loss_type, epsilon_low=0.2, epsilon_high=0.28, beta=0.04, max_completion_length=K,
              num_items_in_batch=mask.sum().float(), grad_accum_steps=2.0)
    cpu_leaf = logits.float().requires_grad_(True)
    lp, ent = oracle.logps_and_entropies_from_logits(cpu_leaf, ids, K, temp, True)
    want_loss, _ = oracle.grpo_loss(lp, adv, mask, entropies=ent, old_per_token_logps=old, ref_per_token_logps=ref, **kw)
    want_loss.backward()
    leaf = logits.to(DEV).requires_grad_(True)
    kw["num_items_in_batch"] = kw["num_items_in_batch"].to(DEV)
    loss, _, got_lp, got_ent = amd.grpo_loss_from_logits(
        leaf, ids[:, -K:].to(DEV), adv.to(DEV), mask.to(DEV), temperature=temp, old_per_token_logps=old.to(DEV),
        ref_per_token_logps=ref.to(DEV), **kw)
    loss.backward()
    m = mask.bool()
    torch.testing.assert_close(got_lp.cpu()[m], lp.detach()[m], atol=2e-3, rtol=0)
    torch.testing.assert_close(got_ent.cpu()[m], ent.detach()[m], atol=2e-3, rtol=0)
    torch.testing.assert_close(loss.detach().cpu(), want_loss.detach(), atol=1e-6, rtol=1e-3)
    assert _rel_l2(leaf.grad.float().cpu(), cpu_leaf.grad) < 5e-3


def test_without_gradient_only_the_forward_runs(amd):
    """Under `no_grad` (evaluation) the operator returns the same loss, metrics, log-probs and entropies without
    writing a logits-sized gradient."""
    B, K, V = 4, 16, 2048
    logits, ids, mask, adv, _ = _inputs(B, K, V, seed=23)
    kw = dict(loss_type="dapo", num_items_in_batch=mask.sum().float(), temperature=0.9)
    leaf = logits.detach().clone().requires_grad_(True)
    want = amd.grpo_loss_from_logits(leaf, ids, adv, mask, **kw)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    with torch.no_grad():
        got = amd.grpo_loss_from_logits(leaf, ids, adv, mask, **kw)
    assert torch.cuda.memory_allocated() - before < logits.numel()  # no [B, L, V] buffer was kept
    assert not got[0].requires_grad
    torch.testing.assert_close(got[0], want[0].detach(), rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(got[1], want[1], rtol=1e-5, atol=1e-6, equal_nan=True)
    torch.testing.assert_close(got[2], want[2], rtol=0, atol=1e-5)
    torch.testing.assert_close(got[3], want[3], rtol=0, atol=1e-5)


def test_kernel_reads_masked_rows_when_asked(amd):
    """`compute_masked_rows` of the C entry point (the Python operator fills those outputs with the streaming
    forward kernel instead): log-prob and entropy of every row, the same gradient."""
    from trl_amd import ops

    B, K, V = 4, 12, 1024
    logits, ids, mask, adv, _ = _inputs(B, K, V, seed=41, extra_rows=0)
    scale = torch.full((B,), 0.01, device=DEV)
    args = (logits, ids, 0.9, 0, K, mask.float(), adv, scale, None, None, None, None, 0, 0.2, 0.2, float("nan"), 0.0, False,
            1.0, 1.05)
    lp_a, ent_a, lse_a, g_a = ops.grpo_fused_fwd_bwd(*args, True)
    lp_s, ent_s, lse_s, g_s = ops.grpo_fused_fwd_bwd(*args, False)
    want_lp, want_ent = amd.logps_and_entropies(logits, ids, 0.9)
    torch.testing.assert_close(lp_a, want_lp, rtol=0, atol=1e-5)
    torch.testing.assert_close(ent_a, want_ent, rtol=0, atol=1e-5)
    m = mask.bool()
    assert torch.equal(lp_a[m], lp_s[m]) and float(lp_s[~m].abs().max()) == 0.0
    assert torch.equal(g_a, g_s)


# ------------------------------------------------------------------ vectors written by the reference
def _round_to(t, dtype):
    return t.to(dtype).float()


@pytest.mark.parametrize("keep_fp32", [False, True], ids=["as16bit", "as_fp32"])
def test_golden_vectors_go_through_the_single_pass_kernel(amd, monkeypatch, keep_fp32):
    """`tests/golden/grpo_single_pass.*`: the reference's `GRPOTrainer._compute_loss` + backward on a mocked trainer
    (trl/trainer/grpo_trainer.py:2991-3260), for every configuration the one-pass kernel takes, on vocabularies
    that are multiples of 8.  The fixture's fp32 logits hold bf16-exact (or fp16-exact) values, so the reference did
    fp32 arithmetic on exactly the numbers the kernel reads from the 16-bit tensor: loss, metrics, log-probs and
    entropies are held to fp32 bars, and the gradient to the reference's gradient ROUNDED to the 16-bit dtype (what
    an exact kernel would store).  Two cases ran the reference in true bf16 / fp16 arithmetic (its log-probs are
    rounded to 16 bits) and are comparable at 2e-2 only.  The call into the one-pass kernel is counted: a case
    that falls back to the two-pass path fails.  `as_fp32`: the fixture's fp32 logits go in as they are, which is
    the very computation the reference ran: loss, metrics and the fp32 gradient are held to fp32 bars."""
    from conftest import fake_grpo_trainer, load_golden
    from types import SimpleNamespace

    import numpy as np

    from trl_amd import ops

    calls = []
    real = ops.grpo_fused_fwd_bwd

    def spy(*a, **k):
        out = real(*a, **k)
        calls.append(out[3])
        return out

    monkeypatch.setattr(ops, "grpo_fused_fwd_bwd", spy)
    cases, g = load_golden("grpo_single_pass")
    assert len(cases) >= 60
    seen = set()
    for case in cases:
        c = f"c{case['id']}_"
        B, P, T, V = case["shape"]
        true_low = "dtype" in case
        if true_low and keep_fp32:
            continue  # (the reference ran these two in 16-bit arithmetic)
        dtype = getattr(torch, case["dtype"] if true_low else case["values"])
        logits32 = torch.from_numpy(g[c + "logits"])
        assert torch.equal(logits32.to(dtype).float(), logits32)  # the 16-bit tensor holds the reference's inputs exactly
        if keep_fp32:
            dtype = torch.float32
        tr = fake_grpo_trainer(amd, case, T, skip_masked=True, single_pass=True)
        tr.trl_amd_single_pass_fp16 = True  # (fp16 logits take the one pass only with a gradient scaler or on request)
        leaf = logits32.to(dtype).to(DEV).requires_grad_(True)
        dev = lambda key: torch.from_numpy(np.asarray(g[c + key])).to(DEV)  # noqa: E731
        inputs = dict(prompt_ids=dev("prompt_ids"), prompt_mask=torch.ones(B, P, dtype=torch.long, device=DEV),
                      completion_ids=dev("completion_ids"), completion_mask=dev("completion_mask"),
                      advantages=dev("advantages"), num_items_in_batch=dev("num_items_in_batch"))
        for key in ("old_per_token_logps", "ref_per_token_logps", "importance_sampling_ratio"):
            if c + key in g:
                inputs[key] = dev(key)
        n_before = len(calls)
        loss = tr._compute_loss(lambda **kw: SimpleNamespace(logits=leaf, aux_loss=None), inputs)
        loss.backward()
        assert len(calls) == n_before + 1, f"{case['name']}: the one-pass kernel was not taken"
        assert leaf.grad.data_ptr() == calls[-1].data_ptr() or torch.equal(leaf.grad, calls[-1])
        name = (case["name"], str(dtype))
        rtol = 2e-2 if true_low else 2e-5
        want_loss = float(g[c + "out_loss"])
        assert abs(float(loss.detach()) - want_loss) <= rtol * max(1.0, abs(want_loss)), (name, float(loss.detach()), want_loss)
        got_metrics = {k: v[-1] for k, v in tr._metrics["train"].items()}
        assert set(case["metrics"]) <= set(got_metrics), (name, set(case["metrics"]) - set(got_metrics))
        for key, want in case["metrics"].items():
            got = got_metrics[key]
            ok = (math.isnan(got) and math.isnan(want)) or abs(got - want) <= rtol * max(1.0, abs(want))
            assert ok, (name, key, got, want)
        want_g = torch.from_numpy(g[c + "out_dlogits"]).float()
        got_g = leaf.grad.float().cpu()
        mask = torch.from_numpy(g[c + "completion_mask"]).bool()
        full = torch.zeros(B, P + T, dtype=torch.bool)
        full[:, P - 1 : P - 1 + T] = mask
        assert float(got_g[~full].abs().max()) == 0.0 and float(want_g[~full].abs().max()) == 0.0, name
        if true_low:
            assert _rel_l2(got_g, want_g) < 2e-2, (name, _rel_l2(got_g, want_g))
        elif keep_fp32:
            assert _rel_l2(got_g, want_g) < 2e-5, (name, _rel_l2(got_g, want_g))
        else:
            # against what an exact kernel would store: the fp32 gradient rounded once to the logits dtype
            exact = _round_to(want_g, dtype)
            rel = _rel_l2(got_g, exact)
            assert rel < 5e-4, (name, rel)
            assert float((got_g == exact).float().mean()) > 0.98, name
            assert _rel_l2(got_g, want_g) < (3e-3 if dtype == torch.bfloat16 else 6e-4), name
        if "state_after" in case:
            want = case["state_after"]
            assert abs(tr.entropy_coef - want["entropy_coef"]) < 1e-9, name
            assert abs(tr._last_world_entropy - want["last_world_entropy"]) < 1e-4, name
            if want["window"] is None:
                assert tr._entropy_window_stats is None
            else:
                torch.testing.assert_close(tr._entropy_window_stats.cpu(), torch.tensor(want["window"]), rtol=1e-5, atol=1e-4)
        seen.add((case["loss_type"], str(dtype)))
    for lt in ("dapo", "grpo", "dr_grpo", "bnpo", "cispo", "sapo"):
        if keep_fp32:
            assert (lt, "torch.float32") in seen
        else:
            assert (lt, "torch.bfloat16") in seen and (lt, "torch.float16") in seen
    amd.check_device_errors()


def test_golden_vectors_functional_form_logps_and_entropies(amd):
    """The same fixture through `grpo_loss_from_logits` directly: per-token log-probs and entropies of the active
    rows against the reference's (fp32 arithmetic on the same 16-bit values), 1e-5 absolute."""
    from conftest import load_golden

    cases, g = load_golden("grpo_single_pass")
    for case in cases:
        if "dtype" in case or case.get("is_ratio") or case.get("adaptive"):
            continue
        c = f"c{case['id']}_"
        B, P, T, V = case["shape"]
        dtype = getattr(torch, case["values"])
        leaf = torch.from_numpy(g[c + "logits"]).to(dtype).to(DEV).requires_grad_(True)
        t = lambda key: torch.from_numpy(g[c + key]).to(DEV) if c + key in g else None  # noqa: E731
        loss, _, lp, ent = amd.grpo_loss_from_logits(
            leaf, t("completion_ids"), t("advantages"), t("completion_mask"), temperature=case.get("temperature", 1.0),
            old_per_token_logps=t("old_per_token_logps"), ref_per_token_logps=t("ref_per_token_logps"),
            loss_type=case["loss_type"], epsilon_low=case["eps_low"], epsilon_high=case["eps_high"], beta=case["beta"],
            delta=case.get("delta"), max_completion_length=T, num_items_in_batch=t("num_items_in_batch"),
            grad_accum_steps=float(case.get("grad_accum", 1)), use_bias_correction_kl=case.get("bias_kl", False),
            entropy_coef=case.get("entropy_coef", 0.0), skip_masked_rows=False)
        torch.testing.assert_close(lp.cpu(), torch.from_numpy(g[c + "out_logps"]), atol=1e-5, rtol=0)
        torch.testing.assert_close(ent.cpu(), torch.from_numpy(g[c + "out_entropies"]), atol=1e-5, rtol=0)
        want_loss = float(g[c + "out_loss"])
        assert abs(float(loss.detach()) - want_loss) <= 2e-5 * max(1.0, abs(want_loss)), case["name"]


# ------------------------------------------------------------------ the benchmark shapes through the single pass
def _big_logits(B, L, V, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    logits = torch.empty(B, L, V, dtype=torch.bfloat16, device=DEV)
    for b in range(B):
        for t0 in range(0, L, 1024):  # blocks keep the fp32 temporary small
            t1 = min(t0 + 1024, L)
            logits[b, t0:t1] = (2.0 * torch.randn(t1 - t0, V, generator=g, device=DEV)).bfloat16()
    return logits, g


def _full_size_check(amd, monkeypatch, logits, g, K, temperature, lengths_lo, adv, pick_b, pick_t, **kw):
    """`grpo_loss_from_logits` on benchmark-sized logits: the call reaches the one-pass kernel; rows without gradient
    are exactly zero; every gradient row sums to zero; a row subsample of log-prob, entropy and dlogits equals the
    CPU oracle's autograd on the same stored values; the loss equals the oracle's loss on the forward kernel's
    log-probs of all rows."""
    import oracle
    from trl_amd import ops

    B, L, V = logits.shape
    calls = []
    real = ops.grpo_fused_fwd_bwd
    monkeypatch.setattr(ops, "grpo_fused_fwd_bwd", lambda *a, **k: calls.append(1) or real(*a, **k))
    ids = torch.randint(0, V, (B, K), generator=g, device=DEV)
    lengths = torch.randint(lengths_lo, K + 1, (B,), generator=g, device=DEV)
    mask = (torch.arange(K, device=DEV)[None] < lengths[:, None]).long()
    with torch.no_grad():
        base, base_ent = amd.per_token_logps_and_entropies(logits, torch.cat([ids[:, :1], ids], 1), K, temperature)
    old = base + 0.05 * torch.randn(base.shape, generator=g, device=DEV)
    ref = base + 0.1 * torch.randn(base.shape, generator=g, device=DEV)
    beta = kw["beta"]
    kw = dict(kw, old_per_token_logps=old, ref_per_token_logps=ref if beta else None, max_completion_length=K,
              num_items_in_batch=mask.sum().float())
    logits.requires_grad_(True)
    logits.grad = None
    loss, metrics, lp, ent = amd.grpo_loss_from_logits(logits, ids, adv, mask, temperature=temperature,
                                                       skip_masked_rows=False, **kw)
    loss.backward()
    assert len(calls) == 1
    grad = logits.grad
    assert grad.shape == logits.shape and grad.dtype == logits.dtype
    start = L - 1 - K
    # (1) rows outside the window or the mask: exactly zero; active rows: not all zero
    nz = torch.stack([(grad[b] != 0).any(-1) for b in range(B)])
    want_nz = torch.zeros(B, L, dtype=torch.bool, device=DEV)
    if beta:  # the KL term moves every active token, whatever its advantage
        want_nz[:, start:start + K] = mask.bool()
        assert torch.equal(nz, want_nz)
    else:  # a token whose ratio left the clip range on the clipped side has no gradient either (a handful of rows)
        want_nz[:, start:start + K] = mask.bool() & (adv.reshape(B, -1) != 0)
        assert not bool((nz & ~want_nz).any())
        assert int((want_nz & ~nz).sum()) <= 2e-3 * int(want_nz.sum())
        assert int(want_nz.sum()) > 0.2 * B * K
    # (2) sum_v dlogits = 0 up to the bf16 rounding of the row's entries
    for b in range(B):
        gb = grad[b, start:start + K].float()
        assert bool((gb.sum(-1).abs() <= 3e-3 * gb.abs().sum(-1) + 1e-12).all()), b
    # (3) every row's log-prob and entropy: the forward kernel's (all rows were asked for)
    torch.testing.assert_close(lp, base, atol=1e-5, rtol=0)
    torch.testing.assert_close(ent, base_ent, atol=1e-4, rtol=0)  # (entropies of ~7 nats from differently ordered sums)
    # (4) the loss: the oracle's arithmetic on the forward kernel's log-probs of all rows
    okw = {k: (v.cpu() if torch.is_tensor(v) else v) for k, v in kw.items()}
    o_lp = base.cpu().clone().requires_grad_(True)
    o_loss, o_metrics = oracle.grpo_loss(o_lp, adv.cpu(), mask.cpu(), entropies=base_ent.cpu(), **okw)
    assert abs(float(loss.detach()) - float(o_loss.detach())) <= 2e-6 + 1e-4 * abs(float(o_loss.detach())), (float(loss.detach()), float(o_loss.detach()))
    md = amd.trainer.metrics_to_dict(metrics, beta, loss_type=kw["loss_type"])
    for name, want in o_metrics.items():
        if name in md:
            assert abs(md[name] - want) <= 1e-4 * max(1.0, abs(want)), (name, md[name], want)
    # (5) a row subsample through the oracle's autograd, from the stored logits to dlogits
    pb, pt = torch.tensor(pick_b), torch.tensor(pick_t)
    sub = logits.detach()[pb.to(DEV)][:, (start + pt).to(DEV)].cpu().float().requires_grad_(True)
    sub_ids = ids[pb.to(DEV)][:, pt.to(DEV)].cpu()
    sub_lp = oracle.selective_log_softmax_f32(sub, sub_ids, temperature)
    sub_ent = oracle.entropy_from_logits_f32(sub, temperature)
    torch.testing.assert_close(lp[pb.to(DEV)][:, pt.to(DEV)].cpu(), sub_lp.detach(), atol=2e-3, rtol=0)
    torch.testing.assert_close(ent[pb.to(DEV)][:, pt.to(DEV)].cpu(), sub_ent.detach(), atol=2e-3, rtol=0)
    spliced = base.cpu().index_put((pb[:, None], pt[None, :]), sub_lp)
    o_loss2, _ = oracle.grpo_loss(spliced, adv.cpu(), mask.cpu(), entropies=base_ent.cpu(), **okw)
    o_loss2.backward()
    got = grad[pb.to(DEV)][:, (start + pt).to(DEV)].float().cpu()
    active = mask.cpu()[pb][:, pt].bool()
    assert int(active.sum()) >= 4
    assert _rel_l2(got[active], sub.grad[active]) < 3e-3, _rel_l2(got[active], sub.grad[active])
    assert _rel_l2(got[active], sub.grad[active].bfloat16().float()) < 1e-3
    assert float(got[~active].abs().max() if (~active).any() else 0.0) == 0.0
    logits.requires_grad_(False)
    amd.check_device_errors()


def test_full_size_config3_single_pass(amd, monkeypatch):
    """Benchmark configuration 3 (64 sequences x 1024 completion tokens, V = 151936, bf16, T = 0.9, G = 8,
    eps = 0.2, beta = 0.04) through `grpo_loss_from_logits` for loss_type grpo, dapo and dr_grpo."""
    B, K, V = 64, 1024, 151936
    logits, g = _big_logits(B, K + 1, V, seed=33)
    rewards = torch.randn(B, generator=g, device=DEV)
    adv = amd.group_advantages(rewards, 8)
    for lt in ("grpo", "dapo", "dr_grpo"):
        _full_size_check(amd, monkeypatch, logits, g, K, 0.9, 64, adv, [0, 17, 63], [0, 1, 40, 500, 1023],
                         loss_type=lt, epsilon_low=0.2, epsilon_high=0.2, beta=0.04)
        monkeypatch.undo()


def test_full_size_config4_single_pass(amd, monkeypatch):
    """Benchmark configuration 4 (32 sequences x 4096 completion tokens, V = 151936, 39.8 GB of bf16 logits, G = 16,
    Bernoulli(0.3) rewards, eps_low = 0.2, eps_high = 0.28, beta = 0) through `grpo_loss_from_logits`."""
    B, K, V = 32, 4096, 151936
    logits, g = _big_logits(B, K + 1, V, seed=44)
    rewards = (torch.rand(B, generator=g, device=DEV) < 0.3).float()
    adv = amd.group_advantages(rewards, 16)
    _full_size_check(amd, monkeypatch, logits, g, K, 1.0, 512, adv, [0, 13, 31], [0, 300, 511, 2047, 4095],
                     loss_type="dapo", epsilon_low=0.2, epsilon_high=0.28, beta=0.0)


# ------------------------------------------------------------------ upstream gradients other than 1
def test_known_upstream_scale_is_folded_into_the_forward(amd, monkeypatch):
    """fp16 logits, a 32768-entry vocabulary and a loss scale of 65536 (what a `GradScaler` starts with): with
    `upstream_scale` the forward writes the scaled gradient -- scaled in fp32 before the one rounding to fp16 -- and
    `backward` leaves the buffer untouched; the result matches the two-pass path, which scales in fp32 as the
    reference's autograd does (trl/trainer/grpo_trainer.py:3124-3142 for who divides what).  Without it the
    gradient is rounded to fp16 first and most of a softmax row (p_v * 1e-4 * 1e-5) is flushed to zero."""
    from trl_amd import ops

    B, K, V, T = 2, 8, 32768, 1.0
    logits, ids, mask, adv, g = _inputs(B, K, V, dtype=torch.float16, seed=41)
    mask[:] = 1
    scale = torch.tensor(65536.0, device=DEV)
    kw = dict(loss_type="dapo", beta=0.0, num_items_in_batch=torch.tensor(4096.0, device=DEV))
    leaf2, loss2, _, _, _ = _two_pass(amd, logits, ids, mask, adv, T, **kw)
    (loss2 * scale).backward()
    written = []
    real = ops.grpo_fused_fwd_bwd
    monkeypatch.setattr(ops, "grpo_fused_fwd_bwd", lambda *a, **k: written.append(real(*a, **k)) or written[-1])
    leaf1 = logits.detach().clone().requires_grad_(True)
    loss1 = amd.grpo_loss_from_logits(leaf1, ids, adv, mask, temperature=T, upstream_scale=scale, **kw)[0]
    torch.testing.assert_close(loss1, loss2, rtol=1e-5, atol=1e-7)  # the returned loss is not scaled
    before = written[-1][3].clone()
    (loss1 * scale).backward()
    assert torch.equal(leaf1.grad, before)  # bit for bit what the forward wrote: nothing was rescaled
    assert _rel_l2(leaf1.grad, leaf2.grad) < 2e-3
    nz2 = float((leaf2.grad != 0).float().mean())
    assert abs(float((leaf1.grad != 0).float().mean()) - nz2) < 1e-3
    # a float works as well as a device scalar; an unexpected upstream gradient is still honoured
    leaf3 = logits.detach().clone().requires_grad_(True)
    (amd.grpo_loss_from_logits(leaf3, ids, adv, mask, temperature=T, upstream_scale=65536.0, **kw)[0] * (2 * scale)).backward()
    assert _rel_l2(leaf3.grad.float(), 2 * leaf2.grad.float()) < 2e-3
    # scaling after the rounding loses the small entries: this is what the scale argument is for
    leaf0 = logits.detach().clone().requires_grad_(True)
    (amd.grpo_loss_from_logits(leaf0, ids, adv, mask, temperature=T, **kw)[0] * scale).backward()
    assert float((leaf0.grad != 0).float().mean()) < 0.9 * nz2 or _rel_l2(leaf0.grad, leaf2.grad) > 2e-3


def test_backward_runs_once(amd):
    logits, ids, mask, adv, _ = _inputs(2, 4, 512, seed=43)
    leaf = logits.detach().clone().requires_grad_(True)
    loss = amd.grpo_loss_from_logits(leaf, ids, adv, mask, loss_type="bnpo")[0]
    loss.backward(retain_graph=True)
    first = leaf.grad.clone()
    with pytest.raises(RuntimeError, match="only once"):
        loss.backward()
    assert torch.equal(leaf.grad, first)


@pytest.mark.parametrize("with_scaler", [True, False])
def test_trainer_method_takes_fp16_only_with_a_known_scale(amd, monkeypatch, with_scaler):
    """`GRPOLossMixin._compute_loss` on fp16 logits: with a gradient scaler on the accelerator the one-pass kernel runs
    with the scaler's factor folded in; without one the two-pass path runs (its gradient is scaled in fp32)."""
    from conftest import fake_grpo_trainer
    from types import SimpleNamespace

    from trl_amd import ops

    B, P, K, V = 4, 2, 8, 4096
    g = torch.Generator(device=DEV).manual_seed(47)
    logits = (2.0 * torch.randn((B, P + K, V), generator=g, device=DEV)).half()
    case = dict(loss_type="grpo", beta=0.0, eps_low=0.2, eps_high=0.2)
    inputs = dict(prompt_ids=torch.randint(0, V, (B, P), generator=g, device=DEV),
                  prompt_mask=torch.ones(B, P, dtype=torch.long, device=DEV),
                  completion_ids=torch.randint(0, V, (B, K), generator=g, device=DEV),
                  completion_mask=torch.ones(B, K, dtype=torch.long, device=DEV),
                  advantages=torch.randn(B, generator=g, device=DEV))
    calls = []
    real = ops.grpo_fused_fwd_bwd
    monkeypatch.setattr(ops, "grpo_fused_fwd_bwd", lambda *a, **k: calls.append(1) or real(*a, **k))

    class Scaler:
        def is_enabled(self):
            return True

        def scale(self, x):
            return x * 1024.0

    grads = {}
    for single in (True, False):
        tr = fake_grpo_trainer(amd, case, K, skip_masked=True, single_pass=single)
        tr.accelerator.scaler = Scaler() if with_scaler else None
        leaf = logits.detach().clone().requires_grad_(True)
        n = len(calls)
        loss = tr._compute_loss(lambda **kw: SimpleNamespace(logits=leaf, aux_loss=None), inputs)
        assert len(calls) == n + (1 if single and with_scaler else 0)
        (tr.accelerator.scaler.scale(loss) if with_scaler else loss).backward()
        grads[single] = leaf.grad
    assert _rel_l2(grads[True], grads[False]) < 2e-3


@pytest.mark.parametrize("with_scaler", [False, True])
@pytest.mark.parametrize("loss_type", ["grpo", "dapo", "dr_grpo"])
@pytest.mark.parametrize("grad_accum", [2, 3, 8])
def test_trainer_divisor_is_folded_into_the_forward(amd, monkeypatch, grad_accum, loss_type, with_scaler):
    """`transformers.Trainer.training_step` divides the loss by `current_gradient_accumulation_steps` before
    `accelerator.backward` when the trainer has `model_accepts_loss_kwargs = False` and no `compute_loss_func`
    (the reference sets the former, trl/trainer/grpo_trainer.py:1128-1131, and passes a placeholder for the latter,
    :944-950; a trainer that only does the former gets the division).  `_compute_loss` must announce that divisor
    (times the gradient scaler's factor) to the single pass, so that `backward` finds an upstream gradient of exactly
    1 and leaves the gradient buffer as the forward wrote it; a trainer that switches the division off must find
    the same."""
    from conftest import fake_grpo_trainer
    from types import SimpleNamespace

    from trl_amd import ops

    B, P, K, V = 4, 2, 8, 4096
    g = torch.Generator(device=DEV).manual_seed(53 + grad_accum)
    logits = (2.0 * torch.randn((B, P + K, V), generator=g, device=DEV)).bfloat16()
    case = dict(loss_type=loss_type, beta=0.04, eps_low=0.2, eps_high=0.2, grad_accum=grad_accum)
    lengths = torch.tensor([8, 3, 0, 5], device=DEV)
    inputs = dict(prompt_ids=torch.randint(0, V, (B, P), generator=g, device=DEV),
                  prompt_mask=torch.ones(B, P, dtype=torch.long, device=DEV),
                  completion_ids=torch.randint(0, V, (B, K), generator=g, device=DEV),
                  completion_mask=(torch.arange(K, device=DEV)[None] < lengths[:, None]).long(),
                  advantages=torch.randn(B, generator=g, device=DEV),
                  num_items_in_batch=torch.tensor(37.0, device=DEV))
    with torch.no_grad():
        base, _ = amd.per_token_logps_and_entropies(logits, torch.cat([inputs["prompt_ids"], inputs["completion_ids"]], 1), K, 1.0)
    inputs["old_per_token_logps"] = base + 0.2 * torch.randn(base.shape, generator=g, device=DEV)
    inputs["ref_per_token_logps"] = base + 0.1 * torch.randn(base.shape, generator=g, device=DEV)
    written = []
    real = ops.grpo_fused_fwd_bwd
    monkeypatch.setattr(ops, "grpo_fused_fwd_bwd", lambda *a, **k: written.append(real(*a, **k)) or written[-1])

    class Scaler:
        def is_enabled(self):
            return True

        def scale(self, x):
            return x * 4096.0

    def training_step(tr, leaf):
        """What the parent class does around `compute_loss` (transformers Trainer.training_step, accelerate
        Accelerator.backward), for a single process."""
        loss = tr._compute_loss(lambda **kw: SimpleNamespace(logits=leaf, aux_loss=None), inputs)
        if not tr.model_accepts_loss_kwargs and tr.compute_loss_func is None:
            loss = loss / tr.current_gradient_accumulation_steps
        loss = loss / tr.accelerator.gradient_accumulation_steps
        if tr.accelerator.scaler is not None:
            loss = tr.accelerator.scaler.scale(loss)
        return loss

    for divides in (True, False):
        grads = {}
        for single in (True, False):
            tr = fake_grpo_trainer(amd, case, K, skip_masked=True, single_pass=single)
            tr.accelerator.scaler = Scaler() if with_scaler else None
            tr.accelerator.gradient_accumulation_steps = 1
            tr.model_accepts_loss_kwargs = False
            tr.compute_loss_func = None if divides else "non-None value to disable scaling"
            leaf = logits.detach().clone().requires_grad_(True)
            n = len(written)
            loss = training_step(tr, leaf)
            assert len(written) == n + (1 if single else 0)
            before = written[-1][3].clone() if single else None
            loss.backward()
            if single:  # bit for bit what the forward wrote: the scale kernel had nothing left to do
                assert torch.equal(leaf.grad, before), (divides, grad_accum, loss_type)
            grads[single] = leaf.grad
        assert _rel_l2(grads[True], grads[False]) < 1e-3

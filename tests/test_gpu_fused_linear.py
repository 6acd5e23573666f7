"""GPU tests of the fused-linear operators (hidden states -> loss without logits) that stand in for the
third-party operators behind the reference's `use_liger_kernel` switch.  Their numbers are checked against the
oracle's composition of pinned pieces (naive head + the reference's loss arithmetic); parity with the third-party
package itself is unpinned (it is not importable here).  Tolerances: loss and metrics 1e-3 relative, gradients
1e-2 relative L2 (the backward's dz is rounded to bf16)."""
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _rel_l2(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    return float((got - want).norm() / want.norm().clamp(min=1e-30))


@pytest.fixture(scope="module")
def amd():
    import trl_amd

    return trl_amd


def _problem(seed, B, T, H, V):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(B, T, H, generator=g).bfloat16()
    weight = (0.3 * torch.randn(V, H, generator=g)).bfloat16()
    ids = torch.randint(0, V, (B, T), generator=g)
    lengths = torch.randint(1, T + 1, (B,), generator=g)
    mask = (torch.arange(T)[None] < lengths[:, None]).long()
    return g, hidden, weight, ids, mask


@pytest.mark.parametrize("loss_type,level,beta", [("dapo", "token", 0.04), ("grpo", "token", 0.0), ("bnpo", "sequence", 0.04),
                                                   ("cispo", "token", 0.04), ("sapo", "token", 0.0), ("dr_grpo", "token", 0.04)])
def test_fused_linear_grpo_loss(amd, loss_type, level, beta):
    B, T, H, V = 6, 24, 64, 517
    g, hidden, weight, ids, mask = _problem(31, B, T, H, V)
    temperature = 0.9
    with torch.no_grad():
        base = oracle.selective_log_softmax((hidden.float().reshape(B * T, H) @ weight.float().t()) / temperature,
                                            ids.reshape(-1)).view(B, T)
    old = base + 0.05 * torch.randn(B, T, generator=g)
    ref = base + 0.1 * torch.randn(B, T, generator=g)
    adv = torch.randn(B, generator=g)
    ratio = 0.5 + torch.rand(B, T, generator=g)
    kw = dict(beta=beta, epsilon_low=0.03, epsilon_high=1.05 if loss_type == "cispo" else 0.04, loss_type=loss_type,
              max_completion_length=T, importance_sampling_level=level)
    oh = hidden.float().requires_grad_(True)
    ow = weight.float().requires_grad_(True)
    oloss, ometrics = oracle.fused_linear_grpo_loss(oh, ow, ids, mask, adv, temperature, old, ref if beta else None,
                                                    ratio, **kw)
    oloss.backward()

    op = amd.FusedLinearGRPOLoss(temperature=temperature, use_ref_model=beta != 0.0, **kw)
    dh = hidden.to(DEV).requires_grad_(True)
    dw = weight.to(DEV).requires_grad_(True)
    loss, metrics = op(_input=dh, lin_weight=dw, selected_token_ids=ids.to(DEV), attention_mask=mask.to(DEV),
                       advantages=adv.to(DEV), bias=None, old_per_token_logps=old.to(DEV),
                       ref_per_token_logps=ref.to(DEV) if beta else None, vllm_is_ratio=ratio.to(DEV))
    loss.backward()
    assert abs(float(loss.detach()) - float(oloss.detach())) <= 1e-3 * max(1.0, abs(float(oloss.detach())))
    assert len(metrics) == len(ometrics) == (2 if beta else 1)
    for got, want in zip(metrics, ometrics):
        if want == want:  # sapo / cispo log no clip ratio in the reference
            assert abs(float(got) - want) <= 1e-3 * max(1.0, abs(want))
    # masked positions take no gradient; the rest matches the oracle's autograd
    assert torch.count_nonzero(dh.grad.float().cpu()[mask == 0]) == 0
    assert _rel_l2(dh.grad.float(), oh.grad) < 1e-2
    assert _rel_l2(dw.grad.float(), ow.grad) < 1e-2
    with pytest.raises(ValueError):  # a bias of the wrong length
        op(_input=dh, lin_weight=dw, selected_token_ids=ids.to(DEV), attention_mask=mask.to(DEV),
           advantages=adv.to(DEV), bias=torch.zeros(V + 1, device=DEV))


@pytest.mark.parametrize("loss_type", ["sigmoid", "apo_zero", "apo_down", "sppo_hard", "nca_pair"])
def test_fused_linear_dpo_loss(amd, loss_type):
    P, T, H, V = 4, 20, 64, 389
    g, hidden, weight, ids, mask = _problem(32, 2 * P, T, H, V)
    ref_hidden = (hidden.float() + 0.1 * torch.randn(2 * P, T, H, generator=g)).bfloat16()
    ref_weight = (weight.float() + 0.02 * torch.randn(V, H, generator=g)).bfloat16()
    target = torch.where(mask == 1, ids, torch.full_like(ids, -100))
    target[:, 0] = -100  # prompt position
    beta = 0.1
    oh = hidden.float().requires_grad_(True)
    ow = weight.float().requires_grad_(True)
    oloss, om = oracle.fused_linear_dpo_loss(ow, oh, target, ref_hidden.float(), ref_weight.float(), beta,
                                             loss_type=loss_type)
    oloss.backward()

    op = amd.FusedLinearDPOLoss(beta=beta, loss_type=loss_type)
    dh = hidden.to(DEV).requires_grad_(True)
    dw = weight.to(DEV).requires_grad_(True)
    loss, m = op(dw, dh, target.to(DEV), None, ref_hidden.to(DEV), ref_weight.to(DEV), None)
    loss.backward()
    assert abs(float(loss.detach()) - float(oloss.detach())) <= 1e-3 * max(1.0, abs(float(oloss.detach())))
    assert len(m) == 7
    for i in (0, 1, 5, 6):
        torch.testing.assert_close(m[i].cpu(), om[i], rtol=1e-3, atol=2e-3)
    for i in (2, 3):
        assert abs(float(m[i]) - float(om[i])) <= 1e-3
    assert float(m[4]) == 0.0
    assert _rel_l2(dh.grad.float(), oh.grad) < 1e-2
    assert _rel_l2(dw.grad.float(), ow.grad) < 1e-2
    with pytest.raises(NotImplementedError):
        amd.FusedLinearDPOLoss(beta=beta, loss_type="ipo")


def test_fused_linear_losses_with_lm_head_bias(amd):
    """`bias` of both operators (`nn.Linear` form `x @ W.T + b`): loss, metrics and the three gradients."""
    B, T, H, V = 6, 20, 64, 389
    g, hidden, weight, ids, mask = _problem(33, B, T, H, V)
    bias = torch.randn(V, generator=g).bfloat16()
    ref_bias = (bias.float() + 0.1 * torch.randn(V, generator=g)).bfloat16()
    temperature = 0.9
    adv = torch.randn(B, generator=g)
    kw = dict(beta=0.0, epsilon_low=0.2, epsilon_high=0.2, loss_type="dapo", max_completion_length=T)
    oh, ow, ob = (x.float().requires_grad_(True) for x in (hidden, weight, bias))
    oloss, om = oracle.fused_linear_grpo_loss(oh, ow, ids, mask, adv, temperature, bias=ob, **kw)
    oloss.backward()
    op = amd.FusedLinearGRPOLoss(temperature=temperature, use_ref_model=False, **kw)
    dh, dw, db = (x.to(DEV).requires_grad_(True) for x in (hidden, weight, bias))
    loss, m = op(dh, dw, ids.to(DEV), mask.to(DEV), adv.to(DEV), db)
    loss.backward()
    assert abs(float(loss.detach()) - float(oloss.detach())) <= 1e-3 * max(1.0, abs(float(oloss.detach())))
    assert db.grad.dtype == torch.bfloat16 and db.grad.shape == (V,)
    for got, want in ((dh, oh), (dw, ow), (db, ob)):
        assert _rel_l2(got.grad.float(), want.grad) < 1e-2

    target = torch.where(mask == 1, ids, torch.full_like(ids, -100))
    ref_hidden = (hidden.float() + 0.1 * torch.randn(B, T, H, generator=g)).bfloat16()
    ref_weight = (weight.float() + 0.02 * torch.randn(V, H, generator=g)).bfloat16()
    oh, ow, ob = (x.float().requires_grad_(True) for x in (hidden, weight, bias))
    oloss, om = oracle.fused_linear_dpo_loss(ow, oh, target, ref_hidden.float(), ref_weight.float(), 0.1, bias=ob,
                                             ref_bias=ref_bias.float())
    oloss.backward()
    dh, dw, db = (x.to(DEV).requires_grad_(True) for x in (hidden, weight, bias))
    loss, m = amd.FusedLinearDPOLoss(beta=0.1)(dw, dh, target.to(DEV), db, ref_hidden.to(DEV), ref_weight.to(DEV),
                                                ref_bias.to(DEV))
    loss.backward()
    assert abs(float(loss.detach()) - float(oloss.detach())) <= 1e-3 * max(1.0, abs(float(oloss.detach())))
    for i in (0, 1, 5, 6):
        torch.testing.assert_close(m[i].cpu(), om[i], rtol=1e-3, atol=2e-3)
    for i in (2, 3):
        assert abs(float(m[i]) - float(om[i])) <= 1e-3
    for got, want in ((dh, oh), (dw, ow), (db, ob)):
        assert _rel_l2(got.grad.float(), want.grad) < 1e-2


@pytest.mark.parametrize("kl", [None, 0.7])
def test_fused_linear_kto_loss(amd, kl):
    B, T, H, V = 6, 18, 64, 389
    g, hidden, weight, ids, mask = _problem(34, B, T, H, V)
    ref_hidden = (hidden.float() + 0.1 * torch.randn(B, T, H, generator=g)).bfloat16()
    ref_weight = (weight.float() + 0.02 * torch.randn(V, H, generator=g)).bfloat16()
    bias = torch.randn(V, generator=g).bfloat16()
    target = torch.where(mask == 1, ids, torch.full_like(ids, -100))
    pref = torch.tensor([1, 0, 1, 1, 0, 0], dtype=torch.bool)
    oh, ow, ob = (x.float().requires_grad_(True) for x in (hidden, weight, bias))
    oloss, osums = oracle.fused_linear_kto_loss(ow, oh, target, pref, ref_hidden.float(), ref_weight.float(), 0.2, kl,
                                                bias=ob, ref_bias=bias.float())
    oloss.backward()
    dh, dw, db = (x.to(DEV).requires_grad_(True) for x in (hidden, weight, bias))
    op = amd.FusedLinearKTOLoss(beta=0.2, use_ref_model=True)
    loss, sums = op(_input=dh, lin_weight=dw, target=target.to(DEV), bias=db, preference_labels=pref.to(DEV),
                    ref_input=ref_hidden.to(DEV), ref_weight=ref_weight.to(DEV), ref_bias=bias.to(DEV),
                    kl=None if kl is None else torch.tensor([kl], device=DEV))
    loss.backward()
    assert abs(float(loss.detach()) - float(oloss.detach())) <= 1e-3 * max(1.0, abs(float(oloss.detach())))
    assert len(sums) == 6
    for got, want in zip(sums, osums):
        assert abs(float(got) - float(want)) <= 2e-3 * max(1.0, abs(float(want))), (float(got), float(want))
    for got, want in ((dh, oh), (dw, ow), (db, ob)):
        assert _rel_l2(got.grad.float(), want.grad) < 1e-2

"""GPU parity of the fused lm_head + log-prob kernels (K5 forward, K6 backward) against the golden
vectors written by the reference's `_ChunkedLogProbFunction`, and against the CPU oracle / plain
fp32 autograd on the same bf16-valued operands.

Tolerances: the reference's own bf16 test uses 1e-2 (tests/test_utils.py:1212-1232).  Against
fp32 op-math on the same stored values: log-probs / entropies 2e-3 abs; gradients 1e-2 relative L2 against the
unrounded fp32 result, and 1.5e-3 (bf16) / 5e-4 (fp16) against that result rounded to the output dtype."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from conftest import load_golden

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


def _fp32_reference(hidden, weight, labels, temperature, softcap, scale, gout):
    """fp32 op-math on the stored (bf16-valued) operands, autograd for the gradients."""
    h = hidden.float().requires_grad_(True)
    w = weight.float().requires_grad_(True)
    y = (h @ w.t()) * scale
    if softcap:
        y = torch.tanh(y / softcap) * softcap
    z = y / temperature
    lp_all = F.log_softmax(z, -1)
    lp = lp_all.gather(-1, labels[:, None]).squeeze(-1)
    ent = -(lp_all.exp() * lp_all).sum(-1)
    (lp * gout).sum().backward()
    return lp.detach(), ent.detach(), h.grad, w.grad


def _run_device(amd, hidden, weight, labels, temperature, chunk, softcap, scale, gout):
    h = hidden.to(DEV).requires_grad_(True)
    w = weight.to(DEV).requires_grad_(True)
    lp, ent = amd._ChunkedLogProbFunction.apply(h, w, labels.to(DEV), temperature, chunk, softcap, scale)
    (lp * gout.to(DEV)).sum().backward()
    assert lp.dtype == torch.float32 and ent.dtype == torch.float32 and not ent.requires_grad
    return lp.detach().cpu(), ent.detach().cpu(), h.grad.cpu(), w.grad.cpu()


def _check_beyond_output_rounding(dh, dw, rdh, rdw, dtype):
    """The gradients leave the kernels in the operand dtype, which alone costs 2^-9 (bf16) or 2^-12 (fp16) per entry
    against an fp32 result.  Against the fp32 reference ROUNDED to that dtype this rounding cancels and what is
    left is the arithmetic's own error: the d logits that feed the two matrix-core products are scaled fp16 (11
    significant bits) where the reference keeps fp32 `grad_logits` and fp32 products (trl/trainer/utils.py:1405-1424).
    That costs 2.5e-4 .. 3.5e-4 relative L2 -- which is what fp16 outputs show; with bf16 outputs an error of that size
    flips the final rounding of about one entry in twenty, and a flipped entry is off by a whole bf16 step, so the
    same arithmetic shows as about 1e-3.  Bars: fp16 5e-4, bf16 1.5e-3."""
    bar = 5e-4 if dtype == torch.float16 else 1.5e-3
    if dw.numel() < 4096:  # a gradient made of a handful of 16-bit d logits does not average
        bar *= 3
    for got, want in ((dh, rdh), (dw, rdw)):
        err = _rel_l2(got.float(), want.to(dtype).float())
        total, rounding = _rel_l2(got.float(), want), _rel_l2(want.to(dtype).float(), want)
        arith = max(total**2 - rounding**2, 0.0) ** 0.5
        print(f"gradient error vs the rounded fp32 reference: {err:.2e}; vs fp32 {total:.2e} of which output rounding "
              f"{rounding:.2e} -> arithmetic {arith:.2e} ({dtype}, {tuple(got.shape)})")
        assert err < bar, err


def test_golden_chunked_logprob_bf16(amd):
    cases, g = load_golden("chunked_logprob")
    ran = 0
    for case in cases:
        if case["dtype"] != "bfloat16":
            continue
        c = f"c{case['id']}_"
        hidden, weight = _t(g[c + "hidden"], torch.bfloat16), _t(g[c + "weight"], torch.bfloat16)
        labels, gout = _t(g[c + "labels"]), _t(g[c + "grad_out"])
        lp, ent, dh, dw = _run_device(amd, hidden, weight, labels, case["temperature"], case["chunk"], case["softcap"],
                                      case["logit_scale"], gout)
        tol = dict(atol=1e-2, rtol=1e-2)  # the reference's bf16 tolerance; its logits are rounded to bf16, ours are not
        torch.testing.assert_close(lp, _t(g[c + "out_logprobs"]), atol=6e-2, rtol=1e-2)
        torch.testing.assert_close(ent, _t(g[c + "out_entropy"]), atol=6e-2, rtol=1e-2)
        assert _rel_l2(dh.float(), _t(g[c + "out_dhidden"])) < 2e-2
        assert _rel_l2(dw.float(), _t(g[c + "out_dweight"])) < 2e-2
        # and tightly against fp32 op-math on the same stored operands
        rlp, rent, rdh, rdw = _fp32_reference(hidden, weight, labels, case["temperature"], case["softcap"],
                                              case["logit_scale"], gout)
        torch.testing.assert_close(lp, rlp, atol=2e-3, rtol=0)
        torch.testing.assert_close(ent, rent, atol=2e-3, rtol=0)
        assert _rel_l2(dh.float(), rdh) < 1e-2 and _rel_l2(dw.float(), rdw) < 1e-2
        del tol
        ran += 1
    assert ran >= 1


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,h,v,chunk,temperature,softcap,scale", [
    (64, 32, 128, 32, 0.7, None, 1.0),       # the reference test's shape (tests/test_utils.py:1161-1163)
    (300, 256, 1000, 256, 0.9, None, 1.0),   # ragged in every dimension, four vocabulary chunks
    (257, 136, 777, 512, 1.0, 5.0, 0.5),     # soft-capping + logit_scale, K tail, odd vocabulary
    (1, 8, 3, 8192, 1.3, None, 1.0),         # minimal sizes
    (600, 512, 2304, 1024, 0.8, None, 1.0),  # several token blocks x several vocabulary tiles
])
def test_fused_head_against_fp32_reference(amd, dtype, n, h, v, chunk, temperature, softcap, scale):
    g = torch.Generator().manual_seed(n * 7 + v)
    hidden = torch.randn(n, h, generator=g).to(dtype)
    weight = (torch.randn(v, h, generator=g) * (2.0 / h**0.5)).to(dtype)
    labels = torch.randint(0, v, (n,), generator=g)
    gout = torch.randn(n, generator=g)
    lp, ent, dh, dw = _run_device(amd, hidden, weight, labels, temperature, chunk, softcap, scale, gout)
    rlp, rent, rdh, rdw = _fp32_reference(hidden, weight, labels, temperature, softcap, scale, gout)
    torch.testing.assert_close(lp, rlp, atol=2e-3, rtol=0)
    torch.testing.assert_close(ent, rent, atol=2e-3, rtol=0)
    assert dh.dtype == dtype and dw.dtype == dtype and dh.shape == hidden.shape and dw.shape == weight.shape
    assert _rel_l2(dh.float(), rdh) < 1e-2, _rel_l2(dh.float(), rdh)
    assert _rel_l2(dw.float(), rdw) < 1e-2, _rel_l2(dw.float(), rdw)
    _check_beyond_output_rounding(dh, dw, rdh, rdw, dtype)
    # the oracle's online sweep (chunked like the reference) agrees as well
    olp, oent, _ = oracle.chunked_logprob_online(hidden.float(), weight.float(), labels, temperature, max(chunk, 8),
                                                 softcap, scale)
    torch.testing.assert_close(lp, olp, atol=2e-3, rtol=0)
    torch.testing.assert_close(ent, oent, atol=2e-3, rtol=0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("stash", [True, False])
def test_backward_scales_its_fp16_operands(amd, monkeypatch, dtype, stash):
    """The backward's products run on fp16 copies of d logits, W^T and hidden^T, each multiplied by a power of two
    taken from its largest magnitude.  Small upstream gradients (a loss divided by many tokens; bf16: 1e-9 .. 1e-5,
    d logits down to 1e-15, far below the smallest fp16 number) and, for bf16, hidden states of magnitude 1e5 against
    weights of 1e-6 (beyond / below the fp16 range) must come out as accurately as ordinary ones; tokens whose
    upstream gradient is a million times smaller than the largest keep their own relative accuracy in dHidden."""
    monkeypatch.setenv("TRL_AMD_HEAD_STASH_GIB", "24" if stash else "0")
    n, h, v = 300, 256, 1000
    g = torch.Generator().manual_seed(11)
    wide = dtype == torch.bfloat16
    hidden = (torch.randn(n, h, generator=g) * (1e5 if wide else 1.0)).to(dtype)
    weight = (torch.randn(v, h, generator=g) * (2.0 / h**0.5) * (1e-5 if wide else 1.0)).to(dtype)
    labels = torch.randint(0, v, (n,), generator=g)
    # (fp16 OUTPUTS cannot hold gradients of 1e-6: there the upstream gradients stay at 1e-2, d logits down to 1e-9)
    gout = torch.randn(n, generator=g) * (1e-5 if wide else 1e-2)
    if wide:
        gout[: n // 2] *= 1e-4 * torch.rand(n // 2, generator=g)  # half of the tokens: 1e-9 and below
    lp, ent, dh, dw = _run_device(amd, hidden, weight, labels, 0.9, 256, None, 1.0, gout)
    rlp, rent, rdh, rdw = _fp32_reference(hidden, weight, labels, 0.9, None, 1.0, gout)
    torch.testing.assert_close(lp, rlp, atol=2e-3, rtol=0)
    _check_beyond_output_rounding(dh, dw, rdh, rdw, dtype)
    if wide:
        small = slice(0, n // 2)  # the rows of dHidden that belong to the tokens with the tiny gradients
        err = _rel_l2(dh[small].float(), rdh[small].to(dtype).float())
        assert err < 1.5e-3, err


@pytest.mark.parametrize("n,h,v,chunk,softcap,scale", [(300, 256, 1000, 256, None, 1.0), (257, 136, 777, 512, 5.0, 0.5)])
def test_fused_head_with_bias(amd, n, h, v, chunk, softcap, scale):
    """z = softcap((hidden @ W.T + bias) * scale) / T: outputs, and the gradients of all three operands."""
    g = torch.Generator().manual_seed(n + v)
    hidden = torch.randn(n, h, generator=g).bfloat16()
    weight = (torch.randn(v, h, generator=g) * (2.0 / h**0.5)).bfloat16()
    bias = (2.0 * torch.randn(v, generator=g)).bfloat16()
    labels = torch.randint(0, v, (n,), generator=g)
    gout = torch.randn(n, generator=g)
    temperature = 0.8
    rh, rw, rb = (x.float().requires_grad_(True) for x in (hidden, weight, bias))
    y = (rh @ rw.t() + rb) * scale
    if softcap:
        y = torch.tanh(y / softcap) * softcap
    lp_all = F.log_softmax(y / temperature, -1)
    rlp = lp_all.gather(-1, labels[:, None]).squeeze(-1)
    rent = -(lp_all.exp() * lp_all).sum(-1)
    (rlp * gout).sum().backward()
    dh, dw, db = (x.to(DEV).requires_grad_(True) for x in (hidden, weight, bias))
    lp, ent = amd._ChunkedLogProbFunction.apply(dh, dw, labels.to(DEV), temperature, chunk, softcap, scale, db)
    (lp * gout.to(DEV)).sum().backward()
    torch.testing.assert_close(lp.detach().cpu(), rlp.detach(), atol=2e-3, rtol=0)
    torch.testing.assert_close(ent.cpu(), rent.detach(), atol=2e-3, rtol=0)
    assert db.grad.dtype == torch.bfloat16
    for got, want in ((dh, rh), (dw, rw), (db, rb)):
        assert _rel_l2(got.grad.float(), want.grad) < 1e-2, _rel_l2(got.grad.float(), want.grad)


@pytest.mark.parametrize("n,h,v,chunk,softcap,scale,bias", [
    (300, 256, 1000, 256, None, 1.0, False),   # ragged tokens and vocabulary, four chunks
    (257, 136, 777, 512, 5.0, 0.5, True),      # soft-capping + logit_scale + bias (general epilogue)
    (600, 512, 2304, 1024, None, 1.0, False),  # several token blocks x several vocabulary tiles
    (1, 8, 3, 8192, None, 1.0, False),
])
def test_backward_from_stashed_products_equals_recompute(amd, monkeypatch, n, h, v, chunk, softcap, scale, bias):
    """The backward fed by the forward's stashed softmax numerators gives the recompute path's gradients (same
    accumulators; the numerators carry fp16's 11 bits, like dz itself), and the forward's outputs do not depend on
    stashing."""
    g = torch.Generator().manual_seed(n * 3 + v)
    hidden = torch.randn(n, h, generator=g).bfloat16().to(DEV)
    weight = (torch.randn(v, h, generator=g) * (2.0 / h**0.5)).bfloat16().to(DEV)
    b = (2.0 * torch.randn(v, generator=g)).bfloat16().to(DEV) if bias else None
    labels = torch.randint(0, v, (n,), generator=g).to(DEV)
    gout = torch.randn(n, generator=g).to(DEV)
    gout[torch.rand(n, generator=g).to(DEV) < 0.45] = 0.0  # rows without an upstream gradient (masked positions)
    out = {}
    for mode, gib in (("stash", "1"), ("recompute", "0")):
        for drop in ("1", "0"):  # with and without dropping the zero-gradient tokens before the backward
            monkeypatch.setenv("TRL_AMD_HEAD_STASH_GIB", gib)
            monkeypatch.setenv("TRL_AMD_HEAD_DROP_ZERO_GRAD", drop)
            assert amd.ops.head_stash_fits(n, v) == (mode == "stash")
            hh, ww = hidden.clone().requires_grad_(True), weight.clone().requires_grad_(True)
            bb = b.clone().requires_grad_(True) if bias else None
            lp, ent = amd._ChunkedLogProbFunction.apply(hh, ww, labels, 0.9, chunk, softcap, scale, bb)
            (lp * gout).sum().backward()
            out[mode, drop] = (lp.detach(), ent, hh.grad, ww.grad, bb.grad if bias else None)
    want_all = out["recompute", "0"]
    for key, got_all in out.items():
        assert torch.equal(got_all[0], want_all[0]) and torch.equal(got_all[1], want_all[1]), key
        assert torch.count_nonzero(got_all[2][gout == 0]) == 0, key  # no gradient for tokens without an upstream one
        for got, want in zip(got_all[2:], want_all[2:]):
            if want is not None:
                # (a handful of bf16 outputs: one flipped last bit is already 3e-3 of the norm)
                one_ulp = bool(((got.float() - want.float()).abs() <= want.float().abs() * 2.0**-7).all())
                assert _rel_l2(got.float(), want.float()) < 2e-3 or (got.numel() <= 64 and one_ulp), (
                    key, _rel_l2(got.float(), want.float()))
    monkeypatch.setenv("TRL_AMD_HEAD_DROP_ZERO_GRAD", "1")
    hh, ww = hidden.clone().requires_grad_(True), weight.clone().requires_grad_(True)
    lp, _ = amd._ChunkedLogProbFunction.apply(hh, ww, labels, 0.9, chunk, softcap, scale)
    (lp * 0.0).sum().backward()  # no token has a gradient
    assert torch.count_nonzero(hh.grad) == 0 and torch.count_nonzero(ww.grad) == 0
    # the op rejects a stash of the wrong shape
    lp, ent, log_z, _, saved = amd.ops.fused_head_fwd(hidden, weight, labels, 0.9, 0.0, 1.0, None, True)
    vpad = (v + 255) // 256 * 256
    assert saved.shape == (vpad // 4 + vpad // 128 + 1, (n + 255) // 256 * 256, 4) and saved.dtype == torch.float16
    with pytest.raises(ValueError):
        amd.ops.fused_head_bwd(hidden, weight, labels, 0.9, 0.0, 1.0, log_z, gout, chunk, None, saved[:, :128])
    with pytest.raises(ValueError):
        amd.ops.fused_head_bwd(hidden, weight, labels, 0.9, 0.0, 1.0, log_z, gout, chunk, None, saved[:-1])


@pytest.mark.parametrize("kind", ["flat", "peaked", "capped_deep_target"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_stashed_numerators_on_flat_peaked_and_capped_rows(amd, monkeypatch, kind, dtype):
    """The stash holds fp16 softmax numerators relative to a running maximum.  Rows on which that could show: nearly
    uniform ones (every numerator close to 1), sharply peaked ones (most numerators below fp16's range: flushed,
    their probabilities are below 2e-12), and soft-capped rows whose target sits 50 nats under the maximum (its
    numerator is flushed, the chain factor of its one-hot term comes from the target logit the forward keeps)."""
    n, h, v, chunk = 300, 128, 1500, 512
    g = torch.Generator().manual_seed({"flat": 1, "peaked": 2, "capped_deep_target": 3}[kind])
    hidden = torch.randn(n, h, generator=g).to(dtype)
    gain = {"flat": 0.01, "peaked": 12.0, "capped_deep_target": 12.0}[kind]
    weight = (torch.randn(v, h, generator=g) * (gain / h**0.5)).to(dtype)
    softcap = 30.0 if kind == "capped_deep_target" else None
    logits = hidden.float() @ weight.float().t()
    if kind == "capped_deep_target":
        labels = logits.argmin(-1)  # capped to about -30 where the row's maximum is about +30
        z = torch.tanh(logits / softcap) * softcap
        assert float((z.max(-1).values - z.gather(-1, labels[:, None]).squeeze(-1)).median()) > 40.0
    else:
        labels = torch.randint(0, v, (n,), generator=g)
    gout = torch.randn(n, generator=g)
    rlp, rent, rdh, rdw = _fp32_reference(hidden, weight, labels, 1.0, softcap, 1.0, gout)
    for gib in ("1", "0"):  # from the stash, and recomputed
        monkeypatch.setenv("TRL_AMD_HEAD_STASH_GIB", gib)
        assert amd.ops.head_stash_fits(n, v) == (gib == "1")
        lp, ent, dh, dw = _run_device(amd, hidden, weight, labels, 1.0, chunk, softcap, 1.0, gout)
        torch.testing.assert_close(lp, rlp, atol=2e-3, rtol=2e-5)
        torch.testing.assert_close(ent, rent, atol=2e-3, rtol=0)
        assert torch.isfinite(dh.float()).all() and torch.isfinite(dw.float()).all()
        _check_beyond_output_rounding(dh, dw, rdh, rdw, dtype)


def test_masked_rows_and_scatter(amd):
    # reference tests/test_utils.py:1338-1398: masked == unmasked on completion rows, exact zeros elsewhere,
    # and the lm_head gradient only sees completion rows
    g = torch.Generator().manual_seed(5)
    B, S, H, V = 3, 17, 64, 500
    hs = torch.randn(B, S, H, generator=g).bfloat16().to(DEV)
    w = (torch.randn(V, H, generator=g) * 0.3).bfloat16().to(DEV).requires_grad_(True)
    labels = torch.randint(0, V, (B, S), generator=g).to(DEV)
    cm = torch.zeros(B, S, dtype=torch.long)
    cm[0, 3:9] = 1
    cm[1, 10:] = 1
    cm = cm.to(DEV)
    lp_m, ent_m = amd.chunked_logprobs_from_hidden(hs, w, labels, cm, 0.8, 256)
    lp_u, ent_u = amd.chunked_logprobs_from_hidden(hs, w, labels, None, 0.8, 256)
    keep = cm[:, 1:].bool()
    torch.testing.assert_close(lp_m[keep], lp_u[keep], atol=1e-5, rtol=0)
    torch.testing.assert_close(ent_m[keep], ent_u[keep], atol=1e-5, rtol=0)
    assert torch.count_nonzero(lp_m[~keep]) == 0 and torch.count_nonzero(ent_m[~keep]) == 0
    lp_m.sum().backward()
    gm = w.grad.clone()
    w.grad = None
    (lp_u * keep).sum().backward()
    assert _rel_l2(gm.float(), w.grad.float()) < 1e-2
    # an empty selection is a valid call
    lp_e, _ = amd.chunked_logprobs_from_hidden(hs, w, labels, torch.zeros_like(cm), 0.8, 256)
    assert torch.count_nonzero(lp_e) == 0


def test_patch_chunked_lm_head_with_router_logits(amd):
    """The patched forward on a stand-in MoE model: log-probs as the unpatched pieces give them, and the
    auxiliary loss equal to transformers' load-balancing loss of the backbone's router logits."""
    from types import SimpleNamespace

    from transformers.models.mixtral.modeling_mixtral import load_balancing_loss_func

    g = torch.Generator().manual_seed(6)
    B, S, H, V, E = 2, 9, 32, 120, 4
    hs = torch.randn(B, S, H, generator=g).bfloat16().to(DEV)
    router = tuple(torch.randn(B * S, E, generator=g).to(DEV) for _ in range(2))
    seen = {}

    class Backbone(torch.nn.Module):
        def forward(self, input_ids=None, attention_mask=None, use_cache=False, **kw):
            seen.update(kw)
            return SimpleNamespace(last_hidden_state=hs, router_logits=router)

    class Model(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.model = Backbone()
            self.lm_head = torch.nn.Linear(H, V, bias=False, device=DEV, dtype=torch.bfloat16)
            self.config = SimpleNamespace(num_experts=E, num_experts_per_tok=2, logit_scale=0.5)

    model = Model()
    amd.patch_chunked_lm_head(model, chunk_size=64, temperature=0.9, output_router_logits=True)
    ids = torch.randint(0, V, (B, S), generator=g).to(DEV)
    am = torch.ones(B, S, dtype=torch.long, device=DEV)
    am[1, 6:] = 0
    cm = am.clone()
    cm[:, :3] = 0
    out = model(input_ids=ids, attention_mask=am, labels=ids, completion_mask=cm)
    assert seen.get("output_router_logits") is True
    want_aux = load_balancing_loss_func(router, E, 2, am)
    torch.testing.assert_close(out["aux_loss"], want_aux)
    lp, ent = amd.chunked_logprobs_from_hidden(hs, model.lm_head.weight, ids, cm, 0.9, 64, None, 0.5)
    assert torch.equal(out["log_probs"], lp) and torch.equal(out["entropy"], ent)
    assert out["log_probs"].shape == (B, S - 1)


def test_golden_chunked_logprob_fp32(amd):
    """fp32 operands (the dtype of the reference's own unit test, tests/test_utils.py:1161-1232) at its tolerance:
    forward and backward within 1e-5 of what the reference operator wrote."""
    cases, g = load_golden("chunked_logprob")
    ran = 0
    for case in cases:
        if case["dtype"] != "float32":
            continue
        c = f"c{case['id']}_"
        hidden, weight = _t(g[c + "hidden"]), _t(g[c + "weight"])
        labels, gout = _t(g[c + "labels"]), _t(g[c + "grad_out"])
        lp, ent, dh, dw = _run_device(amd, hidden, weight, labels, case["temperature"], case["chunk"], case["softcap"],
                                      case["logit_scale"], gout)
        assert dh.dtype == torch.float32 and dw.dtype == torch.float32
        torch.testing.assert_close(lp, _t(g[c + "out_logprobs"]), atol=1e-5, rtol=1e-5)
        torch.testing.assert_close(ent, _t(g[c + "out_entropy"]), atol=1e-5, rtol=1e-5)
        torch.testing.assert_close(dh, _t(g[c + "out_dhidden"]), atol=1e-5, rtol=1e-5)
        torch.testing.assert_close(dw, _t(g[c + "out_dweight"]), atol=1e-5, rtol=1e-5)
        ran += 1
    assert ran >= 1


def test_fp32_operands_blocks_bias_and_ragged_shapes(amd, monkeypatch):
    """The fp32-operand path over several token blocks, with bias, soft-capping and odd sizes, against autograd."""
    from trl_amd.trainer import utils as tu

    monkeypatch.setattr(tu, "_fp32_head_block_rows", lambda vocab: 64)
    g = torch.Generator().manual_seed(91)
    n, h, v = 150, 37, 301
    hidden, weight, bias = torch.randn(n, h, generator=g), 0.3 * torch.randn(v, h, generator=g), torch.randn(v, generator=g)
    labels, gout = torch.randint(0, v, (n,), generator=g), torch.randn(n, generator=g)
    rh, rw, rb = (x.clone().requires_grad_(True) for x in (hidden, weight, bias))
    y = (rh @ rw.t() + rb) * 0.5
    y = torch.tanh(y / 5.0) * 5.0
    lp_all = F.log_softmax(y / 0.8, -1)
    rlp = lp_all.gather(-1, labels[:, None]).squeeze(-1)
    rent = -(lp_all.exp() * lp_all).sum(-1)
    (rlp * gout).sum().backward()
    dh, dw, db = (x.to(DEV).requires_grad_(True) for x in (hidden, weight, bias))

    def no_library_product(*args, **kwargs):
        raise AssertionError("the fp32 head must not call the GEMM library")

    with monkeypatch.context() as mp:  # every product of the operator comes from this library's matrix-core kernels
        for name in ("matmul", "mm", "addmm", "bmm", "einsum"):
            mp.setattr(torch, name, no_library_product)
        for name in ("__matmul__", "matmul", "mm", "addmm_", "addmm"):
            mp.setattr(torch.Tensor, name, no_library_product)
        lp, ent = amd._ChunkedLogProbFunction.apply(dh, dw, labels.to(DEV), 0.8, 64, 5.0, 0.5, db)
        (lp * gout.to(DEV)).sum().backward()
    torch.testing.assert_close(lp.detach().cpu(), rlp.detach(), atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(ent.cpu(), rent.detach(), atol=1e-5, rtol=1e-5)
    for got, want in ((dh, rh), (dw, rw), (db, rb)):
        torch.testing.assert_close(got.grad.cpu(), want.grad, atol=2e-5, rtol=1e-4)


def test_bf16_pieces_give_the_fp32_product(amd):
    """`split_bf16x3`: the three pieces add up to the fp32 value (to 2^-24), padding columns are zero, and
    `gemm_nt` of a left-side and a right-side split equals the float64 product of the fp32 matrices to fp32 rounding
    -- on values spread over 12 orders of magnitude, ragged sizes, with and without accumulation."""
    from trl_amd import ops

    g = torch.Generator().manual_seed(5)
    m, n, k = 300, 517, 203
    a = (torch.randn(m, k, generator=g) * torch.exp(4 * torch.randn(m, k, generator=g))).to(DEV)
    b = (torch.randn(n, k, generator=g) * torch.exp(4 * torch.randn(n, k, generator=g))).to(DEV)
    kp = (k + 7) // 8 * 8
    for side, x in ((0, a), (1, b)):
        p = ops.split_bf16x3(x, side).float().view(x.shape[0], 6, kp)
        assert float(p[:, :, k:].abs().max()) == 0.0
        slots = {0: (2, 1, 0, 1, 0, 0), 1: (0, 1, 2, 0, 1, 0)}[side]
        first = {piece: slots.index(piece) for piece in (0, 1, 2)}
        total = p[:, first[0], :k].double() + p[:, first[1], :k].double() + p[:, first[2], :k].double()
        assert float(((total - x.double()).abs() / x.double().abs().clamp(min=1e-300)).max()) <= 2.0**-23
        for sl, piece in enumerate(slots):
            assert torch.equal(p[:, sl], p[:, first[piece]])
        assert torch.equal(p[:, first[0], :k], x.bfloat16().float())
    want = a.double() @ b.double().t()
    scale = a.double().abs() @ b.double().abs().t()  # the size of the terms that were added
    got = ops.gemm_nt(ops.split_bf16x3(a, 0), ops.split_bf16x3(b, 1))
    err = (got.double() - want).abs() / scale
    lib_err = ((a @ b.t()).double() - want).abs() / scale  # the GEMM library's fp32 product of the same matrices
    print(f"error / sum of |terms|: pieces max {float(err.max()):.2e} rms {float(err.pow(2).mean().sqrt()):.2e}; "
          f"library fp32 max {float(lib_err.max()):.2e} rms {float(lib_err.pow(2).mean().sqrt()):.2e}")
    assert float(err.max()) < 2e-6 and float(err.pow(2).mean().sqrt()) < 2e-7
    assert float(err.pow(2).mean().sqrt()) <= float(lib_err.pow(2).mean().sqrt())  # measured: about half
    twice = ops.gemm_nt(ops.split_bf16x3(a, 0), ops.split_bf16x3(b, 1), out=got.clone(), accumulate=True)
    torch.testing.assert_close(twice, 2 * got, rtol=1e-6, atol=0)
    # plain 16-bit operands: exact products, fp32 accumulation
    for dt in (torch.bfloat16, torch.float16):
        a16, b16 = torch.randn(70, 72, generator=g).to(dt).to(DEV), torch.randn(33, 72, generator=g).to(dt).to(DEV)
        torch.testing.assert_close(ops.gemm_nt(a16, b16), a16.float() @ b16.float().t(), rtol=1e-5, atol=1e-5)
    with pytest.raises(ValueError):
        ops.gemm_nt(a16, b16[:, :64])
    with pytest.raises(ValueError):
        ops.gemm_nt(a16[:, :68], b16[:, :68])  # K must be a multiple of 8


def test_fp32_operands_with_strides(amd):
    """fp32 hidden states and weight that are views with other strides (a transposed buffer, every other row): the
    gradients come back dense, equal to those of contiguous copies."""
    g = torch.Generator(device=DEV).manual_seed(91)
    n, h, v = 70, 48, 200
    hidden_t = torch.randn((h, n), generator=g, device=DEV)
    weight_2 = 0.2 * torch.randn((2 * v, h), generator=g, device=DEV)
    labels = torch.randint(0, v, (n,), generator=g, device=DEV)
    gout = torch.randn((n,), generator=g, device=DEV)
    res = []
    for hid, wt in ((hidden_t.t(), weight_2[::2]), (hidden_t.t().contiguous(), weight_2[::2].contiguous())):
        hh, ww = hid.detach().requires_grad_(True), wt.detach().requires_grad_(True)
        assert hh.is_contiguous() == ww.is_contiguous()
        lp, _ = amd._ChunkedLogProbFunction.apply(hh, ww, labels, 0.9, 64)
        (lp * gout).sum().backward()
        res.append((lp.detach(), hh.grad, ww.grad))
    assert not hidden_t.t().is_contiguous() and not weight_2[::2].is_contiguous()
    for a, b in zip(res[0], res[1]):
        torch.testing.assert_close(a, b, rtol=1e-6, atol=1e-7)
    rlp, _, rdh, rdw = _fp32_reference(hidden_t.t().cpu(), weight_2[::2].cpu(), labels.cpu(), 0.9, None, 1.0, gout.cpu())
    torch.testing.assert_close(res[0][0].cpu(), rlp, rtol=1e-5, atol=1e-5)
    assert _rel_l2(res[0][1], rdh) < 1e-5 and _rel_l2(res[0][2], rdw) < 1e-5


def test_fp64_operands_are_rejected_loudly(amd):
    with pytest.raises(TypeError):
        amd._ChunkedLogProbFunction.apply(torch.randn(4, 8, device=DEV, dtype=torch.float64),
                                          torch.randn(16, 8, device=DEV, dtype=torch.float64),
                                          torch.zeros(4, dtype=torch.long, device=DEV), 1.0, 8)


def test_real_head_shape_row_subsample(amd):
    """Qwen2.5-7B head shape of benchmark configuration 5 (H = 3584, V = 151936) on 256 tokens."""
    g = torch.Generator().manual_seed(55)
    n, h, v = 256, 3584, 151936
    hidden = torch.randn(n, h, generator=g).bfloat16()
    weight = (0.02 * torch.randn(v, h, generator=g)).bfloat16()
    labels = torch.randint(0, v, (n,), generator=g)
    gout = torch.randn(n, generator=g)
    lp, ent, dh, dw = _run_device(amd, hidden, weight, labels, 1.0, 8192, None, 1.0, gout)
    rlp, rent, rdh, rdw = _fp32_reference(hidden, weight, labels, 1.0, None, 1.0, gout)
    torch.testing.assert_close(lp, rlp, atol=2e-3, rtol=0)
    torch.testing.assert_close(ent, rent, atol=2e-3, rtol=0)
    assert _rel_l2(dh.float(), rdh) < 1e-2
    assert _rel_l2(dw.float(), rdw) < 1e-2
    _check_beyond_output_rounding(dh, dw, rdh, rdw, torch.bfloat16)


def test_real_head_shape_paths_agree(amd, monkeypatch):
    """benchmark configuration 5's head shape on 4096 tokens (16 token blocks, 594 vocabulary tiles, 5 backward chunks, a
    prefix mask on the upstream gradient): the stash + token-dropping path gives the recompute path's results, and
    size-independent properties hold -- rows without an upstream gradient get none, dW sums to zero over the
    vocabulary (softmax gradients are orthogonal to the constant shift) and the probabilities behind the entropy are
    normalised (0 <= H <= ln V)."""
    gdev = torch.Generator(device=DEV).manual_seed(77)
    n, h, v = 4096, 3584, 151936
    hidden = torch.randn(n, h, generator=gdev, device=DEV).bfloat16()
    weight = (0.02 * torch.randn(v, h, generator=gdev, device=DEV)).bfloat16()
    labels = torch.randint(0, v, (n,), generator=gdev, device=DEV)
    lengths = torch.randint(16, 257, (16,), generator=gdev, device=DEV)
    active = (torch.arange(256, device=DEV)[None] < lengths[:, None]).reshape(-1)
    gout = torch.randn(n, generator=gdev, device=DEV) * active
    out = {}
    for mode, gib, drop in (("stash", "24", "1"), ("recompute", "0", "0")):
        monkeypatch.setenv("TRL_AMD_HEAD_STASH_GIB", gib)
        monkeypatch.setenv("TRL_AMD_HEAD_DROP_ZERO_GRAD", drop)
        hh, ww = hidden.clone().requires_grad_(True), weight.clone().requires_grad_(True)
        lp, ent = amd._ChunkedLogProbFunction.apply(hh, ww, labels, 1.0, 32768)
        (lp * gout).sum().backward()
        out[mode] = (lp.detach(), ent, hh.grad, ww.grad)
    a, b = out["stash"], out["recompute"]
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    assert _rel_l2(a[2].float(), b[2].float()) < 2e-3 and _rel_l2(a[3].float(), b[3].float()) < 2e-3
    assert torch.count_nonzero(a[2][~active]) == 0 and torch.count_nonzero(a[2][active]) > 0
    col_sum = a[3].float().sum(0)  # sum_v dW[v, :] = sum_n (sum_v dz[n, v]) hidden[n, :] = 0
    assert float(col_sum.abs().max()) < 2e-2 * float(a[3].float().abs().sum(0).max())
    assert float(a[1].min()) >= 0.0 and float(a[1].max()) <= float(torch.log(torch.tensor(float(v)))) + 1e-3
    assert float(a[0].max()) <= 0.0


def test_full_size_config5(amd, monkeypatch):
    """Benchmark configuration 5 at its size: hidden bf16 [16 x 2048, 3584], W bf16 [151936, 3584], a prefix mask per
    sequence, `_ChunkedLogProbFunction` -> GRPO loss (G = 8, beta = 0.04) -> backward.  Run three ways -- forward
    products kept and zero-gradient tokens dropped (what the operator does by default), logits recomputed with every
    token in the products (the reference's scheme, trl/trainer/utils.py:1291-1424), and `FusedLinearGRPOLoss` on the
    same inputs.  Size-independent properties on the whole result, and a 64-token subsample of log-prob / entropy /
    dHidden plus a 64-row slab of dW against the naive fp32 head evaluated on the host (the comparison the reference's
    own test makes at N, H, V = 64, 32, 128, tests/test_utils.py:1161-1232)."""
    B, T, H, V, G, temperature = 16, 2048, 3584, 151936, 8, 1.0
    N = B * T
    g = torch.Generator(device=DEV).manual_seed(5)
    hidden = torch.randn((N, H), generator=g, device=DEV).bfloat16()
    weight = (0.02 * torch.randn((V, H), generator=g, device=DEV)).bfloat16()
    targets = torch.randint(0, V, (N,), generator=g, device=DEV)
    lengths = torch.randint(64, T + 1, (B,), generator=g, device=DEV)
    mask = (torch.arange(T, device=DEV)[None] < lengths[:, None]).long()
    active = mask.bool().reshape(-1)
    adv = amd.group_advantages(torch.randn((B,), generator=g, device=DEV), G)
    with torch.no_grad():
        base = amd._ChunkedLogProbFunction.apply(hidden, weight, targets, temperature, 32768)[0].view(B, T)
    old = base + 0.05 * torch.randn(base.shape, generator=g, device=DEV)
    ref = base + 0.1 * torch.randn(base.shape, generator=g, device=DEV)
    loss_kw = dict(old_per_token_logps=old, ref_per_token_logps=ref, loss_type="dapo", epsilon_low=0.2,
                   epsilon_high=0.2, beta=0.04, max_completion_length=T, num_items_in_batch=mask.sum().float())
    out = {}
    for mode, gib, drop in (("stash", "24", "1"), ("recompute", "0", "0")):
        monkeypatch.setenv("TRL_AMD_HEAD_STASH_GIB", gib)
        monkeypatch.setenv("TRL_AMD_HEAD_DROP_ZERO_GRAD", drop)
        hh, ww = hidden.clone().requires_grad_(True), weight.clone().requires_grad_(True)
        lp, ent = amd._ChunkedLogProbFunction.apply(hh, ww, targets, temperature, 32768)
        loss, _ = amd.grpo_loss(lp.view(B, T), adv, mask, entropies=ent.view(B, T), **loss_kw)
        loss.backward()
        out[mode] = (lp.detach(), ent.detach(), hh.grad, ww.grad, loss.detach())
        del hh, ww, lp, ent, loss
    monkeypatch.setenv("TRL_AMD_HEAD_STASH_GIB", "24")
    monkeypatch.setenv("TRL_AMD_HEAD_DROP_ZERO_GRAD", "1")
    fl = amd.FusedLinearGRPOLoss(beta=0.04, epsilon_low=0.2, epsilon_high=0.2, temperature=temperature,
                                 use_ref_model=True, loss_type="dapo", max_completion_length=T, chunk_size=32768)
    hh, ww = hidden.clone().requires_grad_(True), weight.clone().requires_grad_(True)
    fl_loss, _ = fl(hh.view(B, T, H), ww, targets.view(B, T), mask, adv, None, old, ref)
    fl_loss.backward()
    a, b = out["stash"], out["recompute"]
    # the forward does not depend on what it keeps for the backward
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    assert bool(torch.equal(a[0].view(B, T), base))
    # the three losses
    assert float(a[4]) == float(b[4])
    assert abs(float(fl_loss.detach()) - float(a[4])) <= 1e-6 * max(1.0, abs(float(a[4])))
    # gradients: the two schemes agree; tokens outside the mask get exactly nothing
    assert _rel_l2(a[2].float(), b[2].float()) < 2e-3 and _rel_l2(a[3].float(), b[3].float()) < 2e-3
    assert _rel_l2(hh.grad.float(), a[2].float()) < 2e-3 and _rel_l2(ww.grad.float(), a[3].float()) < 2e-3
    for dh in (a[2], b[2], hh.grad):
        assert torch.count_nonzero(dh[~active]) == 0 and torch.count_nonzero(dh[active]) > 0
    # softmax gradients are orthogonal to a constant shift of the logits: sum_v dW[v, :] = 0
    for dw in (a[3], b[3]):
        assert float(dw.float().sum(0).abs().max()) < 2e-2 * float(dw.float().abs().sum(0).max())
    assert float(a[1].min()) >= 0.0 and float(a[1].max()) <= float(np.log(V)) + 1e-3 and float(a[0].max()) <= 0.0

    # ---- against the host: the upstream gradient of every token from the oracle's loss on the device's log-probs
    lp_host = a[0].view(B, T).cpu().clone().requires_grad_(True)
    host_kw = {k: (v.cpu() if torch.is_tensor(v) else v) for k, v in loss_kw.items()}
    oloss, _ = oracle.grpo_loss(lp_host, adv.cpu(), mask.cpu(), entropies=a[1].view(B, T).cpu(), **host_kw)
    oloss.backward()
    assert abs(float(oloss.detach()) - float(a[4])) <= 1e-5 * max(1.0, abs(float(oloss.detach())))
    g_tok = lp_host.grad.reshape(-1)
    # 64 tokens: first and last of a sequence, around the end of a mask, and a random draw over the active ones
    first_len = int(lengths[0])
    picks = [0, 1, first_len - 1, first_len, N - T, N - 1]
    act_idx = torch.nonzero(active.cpu()).reshape(-1)
    sel = torch.randperm(act_idx.numel(), generator=torch.Generator().manual_seed(6))[: 64 - len(picks)]
    sub = torch.tensor(picks + act_idx[sel].tolist())
    host_w = weight.cpu()
    sub_h = hidden[sub.to(DEV)].cpu().float().requires_grad_(True)
    ow = host_w.float()
    olp, oent = oracle.chunked_logprob_naive(sub_h, ow, targets.cpu()[sub], temperature)
    (olp * g_tok[sub]).sum().backward()
    torch.testing.assert_close(a[0].cpu()[sub], olp.detach(), atol=2e-3, rtol=0)
    torch.testing.assert_close(a[1].cpu()[sub], oent.detach(), atol=2e-3, rtol=0)
    for dh in (a[2], b[2], hh.grad):
        got = dh[sub.to(DEV)].cpu().float()
        assert _rel_l2(got, sub_h.grad) < 1e-2
        assert _rel_l2(got, sub_h.grad.bfloat16().float()) < 3e-3
    # a 64-row slab of dW needs every active token: dW[v, :] = sum_n dz[n, v] hidden[n, :] with
    # dz[n, v] = g[n] (1[v == target_n] - exp(z[n, v] - lse_n)) / T.  The log-sum-exp of every token comes from plain
    # torch on the device (fp32 matrix product + logsumexp in blocks of tokens, none of this library's kernels) and is
    # itself checked against the host's naive head on the 64 tokens above; the slab arithmetic runs on the host.
    lse = torch.empty(N, device=DEV)
    w32 = weight.float()
    for lo in range(0, N, 1024):
        lse[lo:lo + 1024] = torch.logsumexp((hidden[lo:lo + 1024].float() @ w32.t()) / temperature, dim=-1)
    del w32
    with torch.no_grad():
        olse = torch.logsumexp((sub_h.detach() @ ow.t()) / temperature, dim=-1)
    torch.testing.assert_close(lse.cpu()[sub], olse, atol=1e-4, rtol=0)
    for v0 in (0, 75008, V - 64):
        rows = act_idx
        hid_a = hidden.cpu()[rows].double()
        z = (hid_a @ host_w[v0:v0 + 64].double().t()) / temperature
        p = torch.exp(z - lse.cpu()[rows].double()[:, None])
        onehot = (targets.cpu()[rows][:, None] == torch.arange(v0, v0 + 64)[None]).double()
        dz = g_tok[rows].double()[:, None] * (onehot - p) / temperature
        want = dz.t() @ hid_a
        for dw in (a[3], b[3], ww.grad):
            got = dw[v0:v0 + 64].cpu().float()
            assert _rel_l2(got, want) < 1e-2
            assert _rel_l2(got, want.float().bfloat16().float()) < 3e-3


def test_golden_sft_chunked_nll(amd):
    """The reference's `_chunked_cross_entropy_loss` wrote these; fp32 cases are run in bf16 on the device
    (the matrix-core kernels take bf16/fp16) and compared with the oracle on the bf16-rounded operands."""
    from trl_amd.trainer.sft_trainer import _chunked_cross_entropy_loss

    cases, g = load_golden("sft_chunked_nll")
    for case in cases:
        c = f"c{case['id']}_"
        hs = _t(g[c + "hidden"]).bfloat16()
        w = _t(g[c + "weight"]).bfloat16()
        labels = _t(g[c + "labels"])
        kw = dict(shift_labels=labels) if case["shift"] else dict(labels=labels)
        common = dict(num_items_in_batch=case["nitems"], logit_scale=case["scale"], final_logit_softcapping=case["softcap"])
        has_bias = bool(case.get("bias"))
        b = _t(g[c + "bias"]).bfloat16() if has_bias else None
        ohs, ow = hs.float().requires_grad_(True), w.float().requires_grad_(True)
        ob = b.float().requires_grad_(True) if has_bias else None
        oloss, ocorrect, oent, onv = oracle.chunked_cross_entropy_loss(ohs, ow, case["chunk"], lm_head_bias=ob, **common, **kw)
        oloss.backward()
        dhs, dw = hs.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
        db = b.to(DEV).requires_grad_(True) if has_bias else None
        dkw = {k: v.to(DEV) for k, v in kw.items()}
        loss, correct, ent, nv = _chunked_cross_entropy_loss(dhs, dw, 256, lm_head_bias=db, **common, **dkw)
        loss.backward()
        if has_bias:
            assert _rel_l2(db.grad.float(), ob.grad) < 1e-2
        assert int(nv) == int(onv) == int(g[c + "out_n_valid"])
        assert abs(float(loss.detach()) - float(oloss.detach())) <= 1e-3 * abs(float(oloss.detach()))
        assert abs(float(correct.detach()) - float(ocorrect.detach())) <= 1.0  # a near-tie between the two largest logits may flip
        assert abs(float(ent.detach()) - float(oent.detach())) <= 2e-3 * int(nv)
        assert _rel_l2(dhs.grad.float(), ohs.grad) < 1e-2 and _rel_l2(dw.grad.float(), ow.grad) < 1e-2
        if case["dtype"] == "float32":  # and loosely against the reference's own fp32 numbers (bf16 operand rounding)
            assert abs(float(loss.detach()) - float(g[c + "out_loss"])) <= 2e-2 * abs(float(g[c + "out_loss"]))
            # fp32 operands: the reference's numbers at fp32 accuracy
            fhs, fw = _t(g[c + "hidden"]).to(DEV).requires_grad_(True), _t(g[c + "weight"]).to(DEV).requires_grad_(True)
            fb = _t(g[c + "bias"]).to(DEV).requires_grad_(True) if has_bias else None
            loss, correct, ent, nv = _chunked_cross_entropy_loss(fhs, fw, 256, lm_head_bias=fb, **common, **dkw)
            loss.backward()
            if has_bias:
                torch.testing.assert_close(fb.grad.cpu(), _t(g[c + "out_dbias"]), atol=1e-6, rtol=1e-4)
            assert abs(float(loss.detach()) - float(g[c + "out_loss"])) <= 1e-5 * max(1.0, abs(float(g[c + "out_loss"])))
            assert float(correct.detach()) == float(g[c + "out_correct"])
            assert abs(float(ent.detach()) - float(g[c + "out_entropy_sum"])) <= 1e-4 * abs(float(g[c + "out_entropy_sum"]))
            torch.testing.assert_close(fhs.grad.cpu(), _t(g[c + "out_dhidden"]), atol=1e-6, rtol=1e-4)
            torch.testing.assert_close(fw.grad.cpu(), _t(g[c + "out_dweight"]), atol=1e-6, rtol=1e-4)
    # all positions masked: zero loss that still backpropagates
    dhs = torch.randn(2, 5, 32, device=DEV).bfloat16().requires_grad_(True)
    dw = torch.randn(64, 32, device=DEV).bfloat16().requires_grad_(True)
    loss, correct, ent, nv = _chunked_cross_entropy_loss(dhs, dw, 256, labels=torch.full((2, 5), -100, device=DEV))
    loss.backward()
    assert float(loss.detach()) == 0.0 and int(nv) == 0 and torch.count_nonzero(dw.grad) == 0


def test_target_logit_every_tile_position(amd):
    """The forward picks the target's logit out of the accumulators of the tile that holds it.  Every pair of
    (token position inside its 256-token block, vocabulary row inside its 256-row tile) occurs once here, in both
    vocabulary tiles and in a ragged last tile; a wrong accumulator would be off by the spread of the logits
    (about 1), the bar is the 2e-3 of bf16 operands against fp32 op-math."""
    from trl_amd import ops

    n_blocks, H, V = 256, 64, 512 + 40
    N = 256 * n_blocks
    g = torch.Generator().manual_seed(11)
    hidden = torch.randn(N, H, generator=g).bfloat16()
    weight = (0.2 * torch.randn(V, H, generator=g)).bfloat16()
    n = torch.arange(N)
    col, blk = n % 256, n // 256
    labels = (col + blk) % 256 + 256 * (blk % 2)          # every (column, row) pair, alternating tiles
    labels[::517] = 512 + (n[::517] % 40)                 # and some targets in the ragged third tile
    want = F.log_softmax(hidden.double() @ weight.double().t(), -1).gather(-1, labels[:, None]).squeeze(-1).float()
    for stash in (False, True):
        out = ops.fused_head_fwd(hidden.to(DEV), weight.to(DEV), labels.to(DEV), 1.0, 0.0, 1.0, None, stash)
        torch.testing.assert_close(out[0].cpu(), want, atol=2e-3, rtol=0)
    amd.check_device_errors()  # no index was out of range

"""The drop-in methods around a real `transformers` model (a two-layer Qwen2 built from its config with random
weights: nothing is downloaded).  What the other tests do on stand-in models is done here with the real
`model(**inputs).logits`, `model.model` / `model.lm_head` and the model's own backward.

Every case compares two routes through the SAME model on the GPU.  Route one is the method under test.  Route two
takes the model's logits to the host, evaluates the oracle's restatement of the reference loss there in fp32,
and hands the oracle's gradient w.r.t. the logits back to the model's backward.  Loss and parameter gradients of
the two routes must agree: fp32 models to 1e-4, bf16 models to the rounding of the bf16 gradient both routes
hand the model (the oracle's fp32 gradient is cast once, the kernels round once)."""
import copy
from collections import defaultdict
from types import SimpleNamespace

import pytest
import torch

from conftest import IdentityAccelerator, fake_grpo_trainer

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
VOCAB = 1024


@pytest.fixture(scope="module")
def amd():
    import trl_amd

    return trl_amd


@pytest.fixture(scope="module")
def base_model():
    from transformers import Qwen2Config, Qwen2ForCausalLM

    cfg = Qwen2Config(vocab_size=VOCAB, hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4,
                      num_key_value_heads=2, max_position_embeddings=64, tie_word_embeddings=False,
                      attn_implementation="eager")
    torch.manual_seed(0)
    model = Qwen2ForCausalLM(cfg)
    with torch.no_grad():  # random heads give near-uniform rows; sharpen them so that ratios and clipping matter
        model.lm_head.weight.mul_(8.0)
    return model


def _on_gpu(base_model, dtype):
    model = copy.deepcopy(base_model).to(device=DEV, dtype=dtype)
    model.train()
    return model


def _grads(model):
    out = {n: p.grad.detach().float().clone() for n, p in model.named_parameters() if p.grad is not None}
    model.zero_grad(set_to_none=True)
    return out


def _compare_grads(got, want, tol):
    """Largest relative L2 distance over the parameters.  Parameters whose gradient is zero in exact arithmetic and
    rounding noise in practice (the key bias: a shift of every key leaves the attention weights as they are) are
    measured against the largest gradient norm instead of their own."""
    assert set(got) == set(want) and len(got) > 10
    top = max(float(w.norm()) for w in want.values())
    worst, where = 0.0, None
    for name, w in want.items():
        scale = max(float(w.norm()), 1e-3 * top)
        err = float((got[name] - w).norm()) / scale
        if err > worst:
            worst, where = err, name
    assert top > 0.0 and worst <= tol, (worst, where)
    return worst


def _oracle_route(model, input_ids, attention_mask, host_loss):
    """loss and parameter gradients with the loss evaluated by `host_loss(fp32 logits on the host)`."""
    logits = model(input_ids=input_ids, attention_mask=attention_mask, use_cache=False).logits
    leaf = logits.detach().float().cpu().requires_grad_(True)
    loss = host_loss(leaf)
    loss.backward()
    logits.backward(leaf.grad.to(device=DEV, dtype=logits.dtype))
    return float(loss.detach()), _grads(model)


def _grpo_inputs(model, n_seq, n_prompt, n_comp, temperature, seed):
    g = torch.Generator().manual_seed(seed)
    prompt_ids = torch.randint(0, VOCAB, (n_seq, n_prompt), generator=g)
    completion_ids = torch.randint(0, VOCAB, (n_seq, n_comp), generator=g)
    pad = torch.randint(0, n_prompt // 2, (n_seq,), generator=g)
    prompt_mask = (torch.arange(n_prompt)[None] >= pad[:, None]).long()  # left padding
    lengths = torch.randint(1, n_comp + 1, (n_seq,), generator=g)
    lengths[0] = n_comp
    completion_mask = (torch.arange(n_comp)[None] < lengths[:, None]).long()
    advantages = torch.randn((n_seq,), generator=g)
    input_ids = torch.cat([prompt_ids, completion_ids], 1).to(DEV)
    attention_mask = torch.cat([prompt_mask, completion_mask], 1).to(DEV)
    import oracle

    with torch.no_grad():
        logits = model(input_ids=input_ids, attention_mask=attention_mask, use_cache=False).logits.float().cpu()
        base, _ = oracle.logps_and_entropies_from_logits(logits, input_ids.cpu(), n_comp, temperature, False)
    old = base + 0.3 * torch.randn(base.shape, generator=g)  # wide enough for both clip bounds to be crossed
    ref = base + 0.1 * torch.randn(base.shape, generator=g)
    inputs = dict(prompt_ids=prompt_ids, prompt_mask=prompt_mask, completion_ids=completion_ids,
                  completion_mask=completion_mask, advantages=advantages, old_per_token_logps=old,
                  ref_per_token_logps=ref, num_items_in_batch=completion_mask.sum().float())
    return {k: v.to(DEV) for k, v in inputs.items()}, input_ids, attention_mask


@pytest.mark.parametrize("loss_type", ["dapo", "grpo"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_grpo_compute_loss_through_a_real_model(amd, base_model, dtype, loss_type, monkeypatch):
    import oracle
    from trl_amd import ops

    model = _on_gpu(base_model, dtype)
    n_comp, temperature = 12, 0.9
    inputs, input_ids, attention_mask = _grpo_inputs(model, 6, 8, n_comp, temperature, 3)
    case = dict(beta=0.04, loss_type=loss_type, eps_low=0.2, eps_high=0.2, temperature=temperature)
    tr = fake_grpo_trainer(amd, case, n_comp, skip_masked=True, single_pass=True)
    tr.model = model
    calls = []
    real = ops.grpo_fused_fwd_bwd
    monkeypatch.setattr(ops, "grpo_fused_fwd_bwd", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    loss = tr._compute_loss(model, inputs)
    loss.backward()
    got_loss, got = float(loss.detach()), _grads(model)
    assert len(calls) == 1  # the single pass, for fp32 logits as for bf16 ones

    host = {k: v.cpu() for k, v in inputs.items()}

    def host_loss(leaf):
        lp, ent = oracle.logps_and_entropies_from_logits(leaf, input_ids.cpu(), n_comp, temperature, True, False)
        return oracle.grpo_loss(
            lp, host["advantages"], host["completion_mask"], entropies=ent, old_per_token_logps=host["old_per_token_logps"],
            ref_per_token_logps=host["ref_per_token_logps"], loss_type=loss_type, epsilon_low=0.2, epsilon_high=0.2,
            beta=0.04, max_completion_length=n_comp, num_items_in_batch=host["num_items_in_batch"])[0]

    want_loss, want = _oracle_route(model, input_ids, attention_mask, host_loss)
    low = dtype == torch.bfloat16
    assert abs(got_loss - want_loss) <= (1e-4 if low else 1e-5) * max(1.0, abs(want_loss)), (got_loss, want_loss)
    worst = _compare_grads(got, want, 6e-3 if low else 1e-4)
    log = tr._metrics["train"]
    assert log["clip_ratio/region_mean"][-1] > 0.0  # the case exercises the clipped branch
    print(f"grpo {loss_type} {dtype}: loss {got_loss:.6f} vs {want_loss:.6f}, worst parameter-gradient rel-L2 {worst:.2e}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_dpo_compute_loss_through_a_real_model(amd, base_model, dtype):
    import oracle

    model = _on_gpu(base_model, dtype)
    g = torch.Generator().manual_seed(9)
    n_pairs, length = 3, 20
    input_ids = torch.randint(0, VOCAB, (2 * n_pairs, length), generator=g)
    prompt = torch.randint(2, 8, (n_pairs,), generator=g).repeat(2)
    comp = torch.randint(3, 12, (2 * n_pairs,), generator=g)
    pos = torch.arange(length)[None]
    completion_mask = ((pos >= prompt[:, None]) & (pos < (prompt + comp)[:, None])).long()
    attention_mask = (pos < (prompt + comp)[:, None]).long()
    with torch.no_grad():
        logits = model(input_ids=input_ids.to(DEV), attention_mask=attention_mask.to(DEV), use_cache=False).logits.float().cpu()
        seq, _ = oracle.dpo_sequence_logps(logits, input_ids, completion_mask)
    ref = seq + 0.5 * torch.randn(seq.shape, generator=g)

    class Trainer(amd.DPOLossMixin):
        pass

    tr = Trainer()
    tr.accelerator = IdentityAccelerator()
    tr.accelerator.gather_for_metrics = lambda x: x
    tr.model = model
    tr.aux_loss_enabled = False
    tr.precompute_ref_logps = True
    tr.beta, tr.loss_types, tr.loss_weights = 0.1, ["sigmoid"], [1.0]
    tr.label_smoothing, tr.ld_alpha, tr.use_weighting = 0.0, None, False
    tr.f_divergence_type, tr.f_alpha_divergence_coef = "reverse_kl", 1.0
    tr.args = SimpleNamespace(discopop_tau=0.05)
    tr._metrics = {"train": defaultdict(list), "eval": defaultdict(list)}
    tr._total_train_tokens = 0
    inputs = dict(input_ids=input_ids.to(DEV), attention_mask=attention_mask.to(DEV), completion_mask=completion_mask.to(DEV),
                  ref_chosen_logps=ref[:n_pairs].to(DEV), ref_rejected_logps=ref[n_pairs:].to(DEV))
    loss = tr._compute_loss(model, inputs, False)
    loss.backward()
    got_loss, got = float(loss.detach()), _grads(model)

    def host_loss(leaf):
        s, _ = oracle.dpo_sequence_logps(leaf, input_ids, completion_mask)
        return oracle.dpo_sigmoid_loss(s, ref[:n_pairs], ref[n_pairs:], 0.1)[0]

    want_loss, want = _oracle_route(model, inputs["input_ids"], inputs["attention_mask"], host_loss)
    low = dtype == torch.bfloat16
    assert abs(got_loss - want_loss) <= (1e-4 if low else 1e-5) * max(1.0, abs(want_loss)), (got_loss, want_loss)
    worst = _compare_grads(got, want, 6e-3 if low else 1e-4)
    print(f"dpo {dtype}: loss {got_loss:.6f} vs {want_loss:.6f}, worst parameter-gradient rel-L2 {worst:.2e}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_patched_head_of_a_real_model(amd, base_model, dtype):
    """`patch_chunked_lm_head` on the model: log-probs and entropies without logits, and the gradients of a weighted
    sum of the log-probs into every parameter."""
    import oracle
    from trl_amd.trainer.utils import patch_chunked_lm_head

    model = _on_gpu(base_model, dtype)
    patched = _on_gpu(base_model, dtype)
    temperature = 0.8
    patch_chunked_lm_head(patched, chunk_size=256, temperature=temperature)
    g = torch.Generator().manual_seed(4)
    n_seq, length = 4, 18
    input_ids = torch.randint(0, VOCAB, (n_seq, length), generator=g)
    start = torch.randint(2, 8, (n_seq,), generator=g)
    stop = start + torch.randint(2, 10, (n_seq,), generator=g)
    pos = torch.arange(length)[None]
    completion_mask = ((pos >= start[:, None]) & (pos < stop[:, None])).long()
    attention_mask = (pos < stop[:, None]).long()
    weight = torch.randn((n_seq, length - 1), generator=g)
    out = patched(input_ids=input_ids.to(DEV), attention_mask=attention_mask.to(DEV), labels=input_ids.to(DEV),
                  completion_mask=completion_mask.to(DEV))
    assert set(out) == {"log_probs", "entropy", "aux_loss"} and out["aux_loss"] is None
    assert out["log_probs"].dtype == torch.float32 and out["log_probs"].shape == (n_seq, length - 1)
    (out["log_probs"] * weight.to(DEV)).sum().backward()
    got = _grads(patched)
    keep = completion_mask[:, 1:].bool()
    # route two, the reference's arithmetic for this function (utils.py:1328, 1421-1424): fp32 logits from the
    # model's hidden states and head weight on the host, gradients cast to the operands' dtype
    hidden = model.model(input_ids=input_ids.to(DEV), attention_mask=attention_mask.to(DEV), use_cache=False).last_hidden_state
    h_leaf = hidden.detach().float().cpu().requires_grad_(True)
    w_leaf = model.lm_head.weight.detach().float().cpu().requires_grad_(True)
    z = (h_leaf @ w_leaf.t())[:, :-1, :] / temperature
    want_lp = oracle.selective_log_softmax(z, input_ids[:, 1:])
    want_ent = oracle.entropy_from_logits(z.detach())
    (want_lp * weight * keep).sum().backward()
    hidden.backward(h_leaf.grad.to(device=DEV, dtype=dtype))
    model.lm_head.weight.grad = w_leaf.grad.to(device=DEV, dtype=dtype)
    want = _grads(model)
    low = dtype == torch.bfloat16
    lp, ent = out["log_probs"].detach().cpu(), out["entropy"].detach().cpu()
    assert float(lp[~keep].abs().max()) == 0.0 and float(ent[~keep].abs().max()) == 0.0
    assert float((lp - want_lp.detach())[keep].abs().max()) <= 2e-5
    assert float((ent - want_ent)[keep].abs().max()) <= 2e-5
    # bf16: the two routes hand the backbone d hidden values that differ in the last bf16 bit here and there (2e-4 of
    # arithmetic difference against a rounding step of 4e-3), and the backbone's own bf16 backward spreads that over
    # its small parameters; the head's arithmetic error is measured on its own in the fused-head tests
    worst = _compare_grads(got, want, 2e-2 if low else 1e-4)
    print(f"patched head {dtype}: worst parameter-gradient rel-L2 {worst:.2e}")

"""GPU parity of K1/K3 (log-prob + entropy forward, recompute backward) against the CPU oracle,
the reference-written golden vectors, and size-independent properties at the benchmark shape.

Tolerances (from the north star): fp32 logits 1e-5 abs on log-probs/entropies; bf16/fp16 logits
2e-3 abs against the fp32-op-math oracle on the same stored values; gradients 1e-3 relative
(relative L2 per tensor, plus an element-wise bound of one output-dtype ulp-scale for bf16)."""
import math

import numpy as np
import pytest
import torch

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


# ------------------------------------------------------------------ golden vectors + dtypes
def test_golden_utils_vectors(amd):
    _, g = load_golden("utils_logps_entropy")
    for tag, dtype, tol in (("f32", torch.float32, 1e-5), ("bf16", torch.bfloat16, 2e-3)):
        logits = _t(g[f"{tag}_logits"], dtype).to(DEV)
        idx, idxk = _t(g[f"{tag}_index"]).to(DEV), _t(g[f"{tag}_index_k"]).to(DEV)
        f32 = torch.float32
        # fp32 outputs against the fp32-op-math oracle
        cpu = logits.cpu()
        torch.testing.assert_close(amd.selective_log_softmax(logits, idx, out_dtype=f32).cpu(),
                                   oracle.selective_log_softmax_f32(cpu, idx.cpu()), atol=tol, rtol=0)
        torch.testing.assert_close(amd.selective_log_softmax(logits, idxk, out_dtype=f32).cpu(),
                                   oracle.selective_log_softmax_f32(cpu, idxk.cpu()), atol=tol, rtol=0)
        torch.testing.assert_close(amd.entropy_from_logits(logits, out_dtype=f32).cpu(),
                                   oracle.entropy_from_logits_f32(cpu), atol=tol, rtol=0)
        # reference outputs (dtype of the logits): fp32 within 1e-5; bf16 within one bf16 ulp of the reference
        got = amd.selective_log_softmax(logits, idx)
        assert got.dtype == dtype and got.shape == idx.shape
        want = _t(g[f"{tag}_out_logps"])
        ulp = 1e-5 if dtype == torch.float32 else 0.0625  # bf16 spacing for 8 <= |x| < 16
        assert (got.float().cpu() - want).abs().max() <= ulp
        # strided view [:, :-1][:, -5:], as the trainers slice
        view = logits[:, :-1, :][:, -5:, :]
        got = amd.selective_log_softmax(view, idx[:, -5:], out_dtype=f32).cpu()
        torch.testing.assert_close(got, oracle.selective_log_softmax_f32(view.cpu(), idx[:, -5:].cpu()), atol=tol, rtol=0)
        got = amd.entropy_from_logits(view, out_dtype=f32).cpu()
        torch.testing.assert_close(got, oracle.entropy_from_logits_f32(view.cpu()), atol=tol, rtol=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("k", [None, 1, 8])
def test_reference_unit_test_shapes(amd, dtype, k):
    # shapes of reference tests/test_utils.py:866-905
    torch.manual_seed(0)
    logits = torch.randn(4, 32, 1024, dtype=dtype)
    idx = torch.randint(0, 1024, (4, 32) if k is None else (4, 32, k))
    got = amd.selective_log_softmax(logits.to(DEV), idx.to(DEV))
    want = oracle.selective_log_softmax(logits, idx)
    assert got.dtype == dtype and got.shape == want.shape
    if dtype == torch.float32:
        torch.testing.assert_close(got.cpu(), want, rtol=1e-5, atol=1e-5)
    else:
        # the reference output is the rounded value; ours is the fp32 result rounded once: <= 1 ulp apart
        ulp = {torch.float16: 2.0**-7, torch.bfloat16: 2.0**-4}[dtype]  # spacing for |x| < 16
        assert (got.float().cpu() - want.float()).abs().max() <= ulp
        f32 = amd.selective_log_softmax(logits.to(DEV), idx.to(DEV), out_dtype=torch.float32).cpu()
        torch.testing.assert_close(f32, oracle.selective_log_softmax_f32(logits, idx), atol=2e-3, rtol=0)


@pytest.mark.parametrize("shape", [(768,), (32, 768), (8, 16, 768), (2, 4, 8, 768)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_entropy_reference_unit_test_shapes(amd, dtype, shape):
    # shapes of reference tests/test_utils.py:615-628
    torch.manual_seed(1)
    logits = torch.randn(*shape, dtype=dtype)
    got = amd.entropy_from_logits(logits.to(DEV), chunk_size=16, out_dtype=torch.float32).cpu()
    assert got.shape == logits.shape[:-1]
    tol = 1e-5 if dtype == torch.float32 else 2e-3
    torch.testing.assert_close(got, oracle.entropy_from_logits_f32(logits), atol=tol, rtol=0)
    if dtype == torch.float32:
        torch.testing.assert_close(amd.entropy_from_logits(logits.to(DEV)).cpu(), oracle.entropy_from_logits(logits),
                                   rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("k", [None, 1, 8])
def test_float64_logits(amd, k):
    """The float64 case of the reference's unit tests (tests/test_utils.py:866-905, 615-628): double in, double
    out, against torch's own double `log_softmax` / entropy on the host, forward and gradient (duplicate indices,
    a strided view, a skipped row and a temperature included)."""
    g = torch.Generator().manual_seed(64)
    logits = torch.randn(4, 32, 1024, generator=g, dtype=torch.float64)
    idx = torch.randint(0, 1024, (4, 32) if k is None else (4, 32, k), generator=g)
    if k == 8:
        idx[0, 0, 1] = idx[0, 0, 0]
    got = amd.selective_log_softmax(logits.to(DEV), idx.to(DEV))
    want = torch.gather(logits.log_softmax(-1), -1, idx.unsqueeze(-1) if k is None else idx)
    want = want.squeeze(-1) if k is None else want
    assert got.dtype == torch.float64 and got.shape == want.shape
    torch.testing.assert_close(got.cpu(), want, rtol=1e-12, atol=1e-12)
    ent = amd.entropy_from_logits(logits.to(DEV))
    lsm = logits.log_softmax(-1)
    assert ent.dtype == torch.float64
    torch.testing.assert_close(ent.cpu(), -(lsm.exp() * lsm).sum(-1), rtol=1e-12, atol=1e-12)
    # gradients through a window of the rows, with a temperature and an entropy term
    dl = logits.to(DEV).requires_grad_(True)
    ids3 = idx if k is not None else idx.unsqueeze(-1)
    win = ids3[:, 3:29]
    rm = torch.ones(4, 26, dtype=torch.long)
    rm[2, 5] = 0
    lp, h = amd.logps_and_entropies(dl, win.to(DEV), 0.8, 3, 26, rm.to(DEV))
    # (a skipped row's outputs are the constant 0: by contract no gradient arrives there)
    glp = torch.randn(lp.shape, generator=g, dtype=torch.float64) * rm.double().unsqueeze(-1)
    gh = torch.randn(h.shape, generator=g, dtype=torch.float64) * rm.double()
    ((lp * glp.to(DEV)).sum() + (h * gh.to(DEV)).sum()).backward()
    ol = logits.clone().requires_grad_(True)
    z = (ol / 0.8)[:, 3:29].log_softmax(-1)
    keep = rm.double()
    olp = torch.gather(z, -1, win) * keep.unsqueeze(-1)
    oh = -(z.exp() * z).sum(-1) * keep
    ((olp * glp).sum() + (oh * gh).sum()).backward()
    assert lp.dtype == torch.float64 and float(lp.detach()[2, 5].abs().sum()) == 0.0 and float(h.detach()[2, 5]) == 0.0
    torch.testing.assert_close(lp.detach().cpu(), olp.detach(), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(h.detach().cpu(), oh.detach(), rtol=1e-12, atol=1e-12)
    assert dl.grad.dtype == torch.float64
    torch.testing.assert_close(dl.grad.cpu(), ol.grad, rtol=1e-10, atol=1e-13)
    assert float(dl.grad[:, :3].abs().max()) == 0.0 and float(dl.grad[:, 29:].abs().max()) == 0.0
    amd.check_device_errors()


# ------------------------------------------------------------------ benchmark configuration 1 at full size
def test_config1_full_size_fp32(amd):
    g = torch.Generator().manual_seed(0)
    logits = 3.0 * torch.randn(8, 256, 32000, generator=g)
    idx = torch.randint(0, 32000, (8, 256), generator=g)
    dl = logits.to(DEV)
    got_lp = amd.selective_log_softmax(dl, idx.to(DEV)).cpu()
    got_h = amd.entropy_from_logits(dl).cpu()
    want_lp, want_h = oracle.selective_log_softmax(logits, idx), oracle.entropy_from_logits(logits)
    torch.testing.assert_close(got_lp, want_lp, atol=1e-5, rtol=0)
    # The fp32 entropy of the reference formulation (sum of exp(lp) * lp over 32000 terms) is itself up to
    # ~1.3e-5 away from the exact value on this input, so the 1e-5 bar is applied against the fp64
    # evaluation of the same formula, and the fp32 oracle is allowed its own rounding error on top.
    exact_h = oracle.entropy_from_logits(logits.double())
    exact_lp = oracle.selective_log_softmax(logits.double(), idx)
    assert (got_h.double() - exact_h).abs().max() <= 1e-5
    assert (got_lp.double() - exact_lp).abs().max() <= 1e-5
    slack = (want_h.double() - exact_h).abs()
    assert ((got_h - want_h).abs().double() <= 1e-5 + slack).all()


# ------------------------------------------------------------------ real vocabulary sizes, bf16
@pytest.mark.parametrize("vocab,temperature", [(151936, 0.9), (128256, 1.0)])
def test_bf16_real_vocab_forward_backward(amd, vocab, temperature):
    g = torch.Generator().manual_seed(7)
    B, L, K = 2, 9, 6
    logits = (2.0 * torch.randn(B, L, vocab, generator=g)).bfloat16()
    ids = torch.randint(0, vocab, (B, L), generator=g)
    glp = torch.randn(B, K, generator=g)
    glp[0, 2] = 0.0  # a row with zero upstream gradient -> zero-filled
    # device
    dl = logits.to(DEV).requires_grad_(True)
    lp, ent = amd.per_token_logps_and_entropies(dl, ids.to(DEV), K, temperature, True)
    (lp * glp.to(DEV)).sum().backward()
    # oracle in fp32 op-math on the same stored values
    ol = logits.float().requires_grad_(True)
    z = ol[:, :-1][:, -K:] / temperature
    olp = oracle.selective_log_softmax(z, ids[:, -K:])
    oent = oracle.entropy_from_logits(z.detach())
    (olp * glp).sum().backward()
    torch.testing.assert_close(lp.detach().cpu(), olp.detach(), atol=2e-3, rtol=0)
    torch.testing.assert_close(ent.cpu(), oent, atol=2e-3, rtol=0)
    grad = dl.grad.float().cpu()
    assert dl.grad.dtype == torch.bfloat16 and dl.grad.shape == logits.shape
    assert _rel_l2(grad, ol.grad) < 3e-3  # bf16 rounding of the output alone is ~2^-9 per element
    assert (grad - ol.grad).abs().max() <= 2.0**-8 * ol.grad.abs().max() + 1e-12
    assert torch.count_nonzero(grad[:, : L - 1 - K]) == 0 and torch.count_nonzero(grad[:, -1]) == 0
    assert torch.count_nonzero(grad[0, L - 1 - K + 2]) == 0


def test_fp32_gradients_with_entropy_term(amd):
    g = torch.Generator().manual_seed(8)
    B, T, V = 3, 5, 1000
    logits = 2.0 * torch.randn(B, T, V, generator=g)
    idx = torch.randint(0, V, (B, T, 3), generator=g)
    idx[0, 0, 1] = idx[0, 0, 0]  # duplicate index in one row
    glp, gh = torch.randn(B, T, 3, generator=g), torch.randn(B, T, generator=g)
    dl = logits.to(DEV).requires_grad_(True)
    lp, ent = amd.logps_and_entropies(dl, idx.to(DEV), 0.7)
    ((lp * glp.to(DEV)).sum() + (ent * gh.to(DEV)).sum()).backward()
    ol = logits.clone().requires_grad_(True)
    z = ol / 0.7
    ((oracle.selective_log_softmax(z, idx) * glp).sum() + (oracle.entropy_from_logits(z) * gh).sum()).backward()
    torch.testing.assert_close(dl.grad.cpu(), ol.grad, rtol=1e-3, atol=1e-6)
    assert _rel_l2(dl.grad, ol.grad) < 1e-5
    # entropy-only gradient
    dl.grad = None
    amd.entropy_from_logits(dl).sum().backward()
    ol.grad = None
    oracle.entropy_from_logits(ol).sum().backward()
    torch.testing.assert_close(dl.grad.cpu(), ol.grad, rtol=1e-3, atol=1e-6)


# ------------------------------------------------------------------ edge cases
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("vocab", [1, 7, 257, 1031])
def test_unaligned_vocab_and_views(amd, dtype, vocab):
    g = torch.Generator().manual_seed(9)
    logits = (2.0 * torch.randn(3, 6, vocab, generator=g)).to(dtype)
    idx = torch.randint(0, vocab, (3, 6), generator=g)
    gl = torch.randn(3, 4, generator=g)
    view_dev = logits.to(DEV).requires_grad_(True)
    lp = amd.selective_log_softmax(view_dev[:, 1:-1], idx[:, 1:-1].to(DEV), out_dtype=torch.float32)
    (lp * gl.to(DEV)).sum().backward()
    ol = logits.float().requires_grad_(True)
    olp = oracle.selective_log_softmax(ol[:, 1:-1], idx[:, 1:-1])
    (olp * gl).sum().backward()
    tol = 1e-5 if dtype == torch.float32 else 2e-3
    torch.testing.assert_close(lp.detach().cpu(), olp.detach(), atol=tol, rtol=0)
    if vocab > 1:
        assert _rel_l2(view_dev.grad.float(), ol.grad) < (1e-5 if dtype == torch.float32 else 4e-3)


def test_empty_inputs(amd):
    logits = torch.randn(0, 4, 64, device=DEV)
    assert amd.selective_log_softmax(logits, torch.zeros(0, 4, dtype=torch.long, device=DEV)).shape == (0, 4)
    assert amd.entropy_from_logits(torch.randn(2, 0, 64, device=DEV)).shape == (2, 0)


def test_minus_inf_logits_and_row_mask(amd):
    g = torch.Generator().manual_seed(10)
    logits = torch.randn(2, 4, 512, generator=g)
    logits[:, :, 100:300] = -math.inf  # a masked-out vocabulary range
    idx = torch.randint(0, 100, (2, 4), generator=g)
    got = amd.selective_log_softmax(logits.to(DEV), idx.to(DEV)).cpu()
    torch.testing.assert_close(got, oracle.selective_log_softmax(logits, idx), atol=1e-5, rtol=0)
    # entropy: the reference yields NaN (0 * -inf); so do we
    assert torch.isnan(amd.entropy_from_logits(logits.to(DEV))).all()
    assert torch.isnan(oracle.entropy_from_logits(logits)).all()
    # row mask: masked rows are skipped and come back as zeros
    logits = torch.randn(2, 4, 512, generator=g)
    mask = torch.tensor([[1, 1, 0, 0], [1, 0, 0, 0]])
    lp, ent = amd.logps_and_entropies(logits.to(DEV), idx.to(DEV), row_mask=mask.to(DEV))
    want = oracle.selective_log_softmax(logits, idx) * mask
    torch.testing.assert_close(lp.cpu(), want, atol=1e-5, rtol=0)
    assert torch.count_nonzero(ent.cpu()[mask == 0]) == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float64])
def test_minus_inf_logits_backward(amd, dtype):
    """The gradient of the log-probs at a -inf logit (a masked-out vocabulary entry) is 0, as autograd's
    log_softmax backward gives (trl/trainer/utils.py:510 / :519-521), and the other entries are unaffected."""
    g = torch.Generator().manual_seed(12)
    logits = (2.0 * torch.randn(2, 5, 512, generator=g)).to(dtype)
    logits[:, :, 100:300] = -math.inf
    logits[0, 1, 300:] = -math.inf  # one row with a single block of admissible tokens
    idx = torch.randint(0, 100, (2, 5), generator=g)
    gout = torch.randn(2, 5, generator=g)
    ref = logits.clone().double().requires_grad_(True)
    (torch.log_softmax(ref / 0.8, -1).gather(-1, idx[..., None]).squeeze(-1) * gout.double()).sum().backward()
    leaf = logits.clone().to(DEV).requires_grad_(True)
    lp, _ = amd.logps_and_entropies(leaf, idx.to(DEV), temperature=0.8)
    (lp.double() * gout.to(DEV).double()).sum().backward()
    got = leaf.grad.double().cpu()
    assert bool(torch.isfinite(got).all())
    assert float(got[:, :, 100:300].abs().max()) == 0.0
    tol = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float64: 1e-12}[dtype]
    assert float((got - ref.grad).norm() / ref.grad.norm()) < tol


def test_index_out_of_range_sets_flag(amd):
    logits = torch.randn(1, 2, 64, device=DEV)
    idx = torch.tensor([[3, 64]], device=DEV)
    out = amd.selective_log_softmax(logits, idx)
    assert torch.isnan(out[0, 1]) and not torch.isnan(out[0, 0])
    with pytest.raises(IndexError):
        amd.check_device_errors()
    amd.check_device_errors()  # flag was cleared


def test_bitwise_reproducible(amd):
    g = torch.Generator().manual_seed(11)
    logits = (2.0 * torch.randn(4, 8, 4096, generator=g)).bfloat16().to(DEV)
    idx = torch.randint(0, 4096, (4, 8), generator=g).to(DEV)
    a = amd.logps_and_entropies(logits, idx, 0.9)
    b = amd.logps_and_entropies(logits, idx, 0.9)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


# ------------------------------------------------------------------ properties at the benchmark shape
def test_full_size_properties_config3_shape(amd):
    """benchmark configuration 3 shape (64 x 1024 rows, V = 151936, bf16) is too large for the CPU oracle:
    check a row subsample against the oracle and size-independent properties on all rows."""
    B, T, V, temp = 64, 1024, 151936, 0.9
    g = torch.Generator(device=DEV).manual_seed(3)
    logits = torch.empty(B, T + 1, V, dtype=torch.bfloat16, device=DEV)
    for b in range(B):  # row-block generation keeps the fp32 temporary small
        logits[b] = (2.0 * torch.randn(T + 1, V, generator=g, device=DEV)).bfloat16()
    ids = torch.randint(0, V, (B, T + 1), generator=g, device=DEV)
    lengths = torch.randint(64, T + 1, (B,), generator=g, device=DEV)
    mask = (torch.arange(T, device=DEV)[None] < lengths[:, None]).float()
    logits.requires_grad_(True)
    lp, ent = amd.per_token_logps_and_entropies(logits, ids, T, temp, True)
    assert lp.shape == (B, T) and (lp <= 0).all() and (ent >= 0).all() and (ent <= math.log(V) + 1e-3).all()
    gl = torch.randn(B, T, generator=g, device=DEV) * mask
    (lp * gl).sum().backward()
    grad = logits.grad
    # masked rows and the dropped last position are exactly zero
    row_nonzero = (grad != 0).any(-1)
    assert not row_nonzero[:, -1].any()
    assert torch.equal(row_nonzero[:, :T], (gl != 0))
    # sum_v dlogits = g * (1 - sum p) / T = 0 up to the bf16 rounding of ~V elements
    row_sum = grad[:, :T].float().sum(-1)
    assert (row_sum.abs() <= 2e-2 * gl.abs() + 1e-6).all()
    # row subsample against the oracle (fp32 op-math on the same stored values)
    pick_b = torch.tensor([0, 17, 63])
    pick_t = torch.tensor([0, 1, 500, 1023])
    sub = logits.detach()[pick_b][:, pick_t].cpu()
    sub_ids = ids[pick_b][:, pick_t + 1].cpu()
    want_lp = oracle.selective_log_softmax_f32(sub, sub_ids, temp)
    want_h = oracle.entropy_from_logits_f32(sub, temp)
    torch.testing.assert_close(lp.detach()[pick_b][:, pick_t].cpu(), want_lp, atol=2e-3, rtol=0)
    torch.testing.assert_close(ent[pick_b][:, pick_t].cpu(), want_h, atol=2e-3, rtol=0)
    # gradient of those rows: g * (onehot - p) / T
    z = sub.float() / temp
    p = torch.softmax(z, -1)
    onehot = torch.zeros_like(p).scatter_(-1, sub_ids.unsqueeze(-1), 1.0)
    want_g = gl[pick_b][:, pick_t].cpu().unsqueeze(-1) * (onehot - p) / temp
    got_g = grad[pick_b][:, pick_t].float().cpu()
    assert _rel_l2(got_g, want_g) < 3e-3


def test_long_context_config4_saved_state_and_properties(amd):
    """benchmark configuration 4 (32 x 4096 rows, V = 151936, bf16: 39.8 GB of logits): what the forward keeps for the
    backward is a few bytes per row (the reference keeps a [T, V] log-softmax per sequence), masked rows and the
    dropped last position get exactly zero gradient, and sum_v dlogits = 0 on the active rows."""
    B, T, V = 32, 4096, 151936
    g = torch.Generator(device=DEV).manual_seed(4)
    logits = torch.empty(B, T + 1, V, dtype=torch.bfloat16, device=DEV)
    for b in range(B):
        for t0 in range(0, T + 1, 1024):  # blocks keep the fp32 temporary small
            t1 = min(t0 + 1024, T + 1)
            logits[b, t0:t1] = (2.0 * torch.randn(t1 - t0, V, generator=g, device=DEV)).bfloat16()
    ids = torch.randint(0, V, (B, T + 1), generator=g, device=DEV)
    lengths = torch.randint(512, T + 1, (B,), generator=g, device=DEV)
    mask = (torch.arange(T, device=DEV)[None] < lengths[:, None]).float()
    logits.requires_grad_(True)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    lp, ent = amd.per_token_logps_and_entropies(logits, ids, T, 1.0, True)
    torch.cuda.synchronize()
    held = torch.cuda.memory_allocated() - before
    rows = B * T
    # outputs (lp, ent: fp32 per row) + saved for backward (lse, entropy: fp32 per row) + int64 index per row
    assert held <= rows * (4 * 4 + 8) + (1 << 20), held
    assert (lp <= 0).all() and (ent >= 0).all() and (ent <= math.log(V) + 1e-3).all()
    gl = torch.randn(B, T, generator=g, device=DEV) * mask
    (lp * gl).sum().backward()
    grad = logits.grad
    row_nonzero = torch.stack([(grad[b] != 0).any(-1) for b in range(B)])
    assert not row_nonzero[:, -1].any() and torch.equal(row_nonzero[:, :T], gl != 0)
    row_sum = torch.stack([grad[b, :T].float().sum(-1) for b in range(B)])
    assert (row_sum.abs() <= 2e-2 * gl.abs() + 1e-6).all()
    # a few rows against fp32 op-math on the same stored values
    pick_b, pick_t = torch.tensor([0, 31]), torch.tensor([0, 2047, 4095])
    sub = logits.detach()[pick_b][:, pick_t].cpu()
    sub_ids = ids[pick_b][:, pick_t + 1].cpu()
    torch.testing.assert_close(lp.detach()[pick_b][:, pick_t].cpu(), oracle.selective_log_softmax_f32(sub, sub_ids, 1.0),
                               atol=2e-3, rtol=0)
    torch.testing.assert_close(ent[pick_b][:, pick_t].cpu(), oracle.entropy_from_logits_f32(sub, 1.0), atol=2e-3, rtol=0)


def test_row_statistics_of_the_same_pass():
    """`logp_entropy_stats_fwd`: mean logit, log sum_v p_v^2 and the arg-max flag (first maximal position, as
    `torch.argmax`) against torch on the same values, at a real vocabulary size, with ties and masked rows."""
    import trl_amd
    from trl_amd import ops

    g = torch.Generator().manual_seed(77)
    for dtype, V, tol in ((torch.bfloat16, 128256, 2e-3), (torch.float32, 32000, 1e-5), (torch.float16, 1003, 2e-3)):
        B, L = 2, 9
        logits = (2.0 * torch.randn(B, L, V, generator=g)).to(dtype)
        ids = torch.randint(0, V, (B, L), generator=g)
        top = logits.float().argmax(-1)
        ids[:, 1::3] = top[:, 1::3]                      # every third target is the arg-max
        logits[0, 2, 7] = logits[0, 2, 11] = logits[0, 2].max() + 1   # tie: position 7 wins
        ids[0, 2] = 11
        logits[1, 4, 3] = logits[1, 4, 900] = logits[1, 4].max() + 1  # tie, target is the first one
        ids[1, 4] = 3
        mask = torch.ones(B, L, dtype=torch.uint8)
        mask[1, 6] = 0
        x = logits.float()
        want_mean = x.mean(-1)
        want_lsp2 = torch.logsumexp(2 * x, -1) - 2 * torch.logsumexp(x, -1)
        want_hit = (x.argmax(-1) == ids).float()
        logp, ent, lse, stats = ops.logp_entropy_stats_fwd(logits.to(DEV), ids.reshape(-1, 1).to(DEV), 1.0, 0, L,
                                                           mask.reshape(-1).to(DEV))
        stats = stats.cpu().view(B, L, 4)
        keep = mask.bool()
        torch.testing.assert_close(stats[..., 0][keep], want_mean[keep], atol=tol, rtol=0)
        torch.testing.assert_close(stats[..., 1][keep], want_lsp2[keep], atol=10 * tol, rtol=0)
        assert torch.equal(stats[..., 2][keep], want_hit[keep])
        assert want_hit[0, 2] == 0 and want_hit[1, 4] == 1 and want_hit[:, 1].sum() == B
        assert torch.equal(stats[1, 6], torch.zeros(4)) and float(logp.view(B, L)[1, 6]) == 0.0
        # without the sum of squared probabilities: the same pass minus that sum, 0 in its slot, all else bit for bit
        logp1, ent1, lse1, stats1 = ops.logp_entropy_stats_fwd(logits.to(DEV), ids.reshape(-1, 1).to(DEV), 1.0, 0, L,
                                                               mask.reshape(-1).to(DEV), False)
        stats1 = stats1.cpu().view(B, L, 4)
        assert torch.equal(logp1, logp) and torch.equal(ent1, ent) and torch.equal(lse1, lse)
        assert torch.equal(stats1[..., 1], torch.zeros(B, L))
        assert torch.equal(stats1[..., [0, 2, 3]], stats[..., [0, 2, 3]])
        # the other outputs are those of the plain forward
        lp2, ent2, lse2 = ops.logp_entropy_fwd(logits.to(DEV), ids.reshape(-1, 1).to(DEV), 1.0, 0, L,
                                               mask.reshape(-1).to(DEV))
        assert torch.equal(logp, lp2) and torch.equal(ent, ent2) and torch.equal(lse, lse2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["fp32", "bf16", "fp16"])
def test_rows_that_are_not_whole_vectors(amd, dtype):
    """Vocabularies that are no multiple of the 16-byte vector (a tokenizer with a few added tokens: 32001, 50257,
    128257 ...): every row then starts at another alignment; the kernels peel it to its first 16-byte boundary, take
    aligned vectors from there and finish element by element.  Targets, duplicate targets and the row maximum are put
    into the peeled head, into the body and into the last elements of rows at every alignment; vocabularies around one
    and several gradient chunks; forward, row statistics and gradient against torch in fp64."""
    import torch.nn.functional as F

    from trl_amd import ops

    per_vec = 16 // torch.empty((), dtype=dtype).element_size()
    chunk = 8192 // torch.empty((), dtype=dtype).element_size()  # elements per gradient workgroup
    for V in (1, 3, per_vec - 1, per_vec + 1, 41, 2 * per_vec + 3, chunk + 3, chunk + per_vec + 1, 2 * chunk - 1, 32001, 50257):
        n_seq, L = 2, 9  # 18 rows: every row alignment of an odd vocabulary occurs
        g = torch.Generator(device=DEV).manual_seed(V)
        logits = (3.0 * torch.randn((n_seq, L, V), generator=g, device=DEV)).to(dtype)
        K = 3
        index = torch.randint(0, V, (n_seq, L, K), generator=g, device=DEV)
        index[:, :, 0] = torch.arange(L, device=DEV)[None].clamp(max=V - 1)  # positions 0 .. 8: inside every possible head
        index[:, 1::2, 1] = V - 1 - torch.arange(L, device=DEV)[None, 1::2].clamp(max=V - 1) % min(V, per_vec)  # the last elements
        index[:, ::3, 2] = index[:, ::3, 0]  # a duplicate target
        peak = index[:, :, 0].clone()
        peak[:, 2::3] = index[:, 2::3, 1]
        logits.scatter_(-1, peak.unsqueeze(-1), 40.0)  # the row maximum sits on the first target of most rows
        leaf = logits.detach().clone().requires_grad_(True)
        lp, ent = amd.logps_and_entropies(leaf, index, 0.8)
        ref = logits.detach().double().requires_grad_(True)
        lsm = F.log_softmax(ref / 0.8, -1)
        want_lp, want_h = lsm.gather(-1, index), -(lsm.exp() * lsm).sum(-1)
        assert float((lp.detach().double() - want_lp.detach()).abs().max()) <= 2e-5 * 50, V
        assert float((ent.detach().double() - want_h.detach()).abs().max()) <= 2e-5 * 50, V
        gl, gh = torch.randn(lp.shape, generator=g, device=DEV, dtype=torch.float64), torch.randn(ent.shape, generator=g, device=DEV, dtype=torch.float64)
        ((lp.double() * gl).sum() + (ent.double() * gh).sum()).backward()
        ((want_lp * gl).sum() + (want_h * gh).sum()).backward()
        bar = {torch.float32: 2e-5, torch.bfloat16: 4e-3, torch.float16: 1e-3}[dtype]
        if V == 1:  # (no gradient in exact arithmetic: g * (1 - p) with p one rounding away from 1)
            assert float(leaf.grad.double().abs().max()) <= bar * float(gl.abs().max() + gh.abs().max()), V
        else:
            err = float((leaf.grad.double() - ref.grad).norm() / ref.grad.norm())
            assert err <= bar, (V, err)
        # row statistics: mean logit, and whether the first target is the row's arg-max (first maximal position)
        idx = index.reshape(n_seq * L, K)
        _, _, _, stats = ops.logp_entropy_stats_fwd(logits, idx, 1.0, 0, L, None)
        x = logits.double()
        assert float((stats[:, 0].double() - x.mean(-1).reshape(-1)).abs().max()) <= 1e-4 * 50, V
        want_hit = (x.argmax(-1) == index[:, :, 0]).reshape(-1)
        assert torch.equal(stats[:, 2] != 0, want_hit), V
    amd.check_device_errors()

"""The GRPO loss entry point that allocates nothing (`trlk_grpo_loss_static`: its per-sequence partial sums live in
a device array built into the library) against `trlk_grpo_loss` with a caller workspace, through the C ABI: same
kernels, same reduction order, so every output must be bit-identical.  Two calls in a row share the array; the
second is smaller, so stale partial sums of the first call sit behind its own."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _problem(B, T, seed):
    g = torch.Generator().manual_seed(seed)
    lp = -3.0 * torch.rand(B, T, generator=g)
    lengths = torch.randint(0, T + 1, (B,), generator=g)
    lengths[B // 2] = 0
    t = dict(
        logp=lp, old=lp + 0.3 * torch.randn(B, T, generator=g), ref=lp + 0.2 * torch.randn(B, T, generator=g),
        ent=3.0 * torch.rand(B, T, generator=g), adv=torch.randn(B, generator=g),
        mask=(torch.arange(T)[None] < lengths[:, None]).float(),
        weight=0.5 + torch.rand(B, T, generator=g),
    )
    t = {k: v.to(DEV).contiguous() for k, v in t.items()}
    t["n_items"] = (t["mask"].sum() * 2.0).reshape(1)
    return t


@pytest.mark.parametrize("loss_type,term,seq_level,beta,coef", [
    ("dapo", "clip", False, 0.04, 0.01), ("grpo", "clip", True, 0.04, 0.0), ("bnpo", "sapo", False, 0.0, 0.02),
    ("dr_grpo", "cispo", False, 0.04, 0.0)])
def test_static_scratch_entry_matches_workspace_entry(loss_type, term, seq_level, beta, coef):
    from trl_amd import _lib, ops

    lt = {"grpo": _lib.GRPO, "bnpo": _lib.BNPO, "dr_grpo": _lib.DR_GRPO, "dapo": _lib.DAPO}[loss_type]
    tm = {"clip": _lib.TERM_CLIP, "sapo": _lib.TERM_SAPO, "cispo": _lib.TERM_CISPO}[term]
    assert ops.grpo_loss_static_max_seq() == 8192
    assert _lib.lib.trlk_init() == 0
    for B, T, seed in ((96, 333, 5), (7, 41, 6)):  # the second call is smaller than the first
        p = _problem(B, T, seed)
        weight = None if seq_level else p["weight"]
        cfg = (lt, 0.2, 0.28, math.nan, beta, True, 2.0, float(B * T), 1.0, coef, tm, seq_level, None, 1.0, 1.05)
        want = ops.grpo_loss_op(p["logp"], p["old"], p["ref"] if beta else None, p["ent"], p["adv"], p["mask"], weight,
                                None, p["n_items"], *cfg)
        loss = torch.full((), math.nan, device=DEV)
        metrics = torch.full((_lib.GRPO_NUM_METRICS,), math.nan, device=DEV)
        dlogp = torch.full((B, T), math.nan, device=DEV)
        dent = torch.full((B, T), math.nan, device=DEV) if coef else None
        torch.cuda.synchronize()
        held = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.memory_stats()["allocation.all.allocated"])
        ops.grpo_loss_static_(loss, metrics, dlogp, dent, p["logp"], p["old"], p["ref"] if beta else None, p["ent"],
                              p["adv"], p["mask"], weight, None, p["n_items"], *cfg)
        torch.cuda.synchronize()
        # nothing was allocated through torch, not even a block that was freed again before the call returned
        assert held == (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(),
                        torch.cuda.memory_stats()["allocation.all.allocated"])
        assert torch.equal(loss, want[0]), (B, float(loss), float(want[0]))
        assert torch.equal(metrics.nan_to_num(nan=-7.0), want[1].nan_to_num(nan=-7.0))
        assert torch.equal(dlogp, want[2])
        if coef:
            assert torch.equal(dent, want[3])
        assert math.isfinite(float(loss))


def test_static_scratch_entry_checks_its_operands():
    """The Python wrapper hands raw pointers to the library: layout, dtype and device of every operand are checked
    before that."""
    from trl_amd import _lib, ops

    B, T = 4, 8
    p = _problem(B, T, 9)
    out = dict(loss=torch.zeros((), device=DEV), metrics=torch.zeros(_lib.GRPO_NUM_METRICS, device=DEV),
               dlogp=torch.zeros(B, T, device=DEV))
    cfg = [_lib.DAPO, 0.2, 0.2, math.nan, 0.0, False, 1.0, float(B * T), 1.0, 0.0, _lib.TERM_CLIP, False, None, 1.0, 1.05]

    def call(loss=None, metrics=None, n_items=None, seq_coef=None, adv=None, term=_lib.TERM_CLIP):
        c = list(cfg)
        c[10], c[12] = term, seq_coef
        ops.grpo_loss_static_(out["loss"] if loss is None else loss, out["metrics"] if metrics is None else metrics,
                              out["dlogp"], None, p["logp"], p["old"], None, None, p["adv"] if adv is None else adv,
                              p["mask"], None, None, p["n_items"] if n_items is None else n_items, *c)

    call()  # the well-formed call goes through
    with pytest.raises(ValueError, match="out_metrics"):
        call(metrics=torch.zeros(2 * _lib.GRPO_NUM_METRICS, device=DEV)[::2])
    with pytest.raises(ValueError, match="dapo_normalizer"):
        call(n_items=p["n_items"].bfloat16())
    with pytest.raises(ValueError, match="seq_coef"):
        call(seq_coef=torch.ones(B, 2, device=DEV)[:, 0], term=_lib.TERM_WEIGHTED_LOGP)
    with pytest.raises(ValueError, match="is on cpu"):
        call(adv=p["adv"].cpu())
    with pytest.raises(ValueError, match="advantages"):
        call(adv=torch.zeros(2, B // 2, device=DEV).t())


def test_static_scratch_entry_rejects_what_does_not_fit():
    from trl_amd import _lib

    fake = 0x1000  # never dereferenced: the size check comes before any launch
    rc = _lib.lib.trlk_grpo_loss_static(fake, None, None, None, fake, 1, 0, fake, None, None, None, 8193, 16, _lib.GRPO,
                                        _lib.TERM_CLIP, 0, 0.2, 0.2, math.nan, 0.0, 0, 1.0, 1.0, None, 1.0, 0.0, 1.0, 1.05,
                                        fake, fake, fake, None, None)
    assert rc == -6 and "8192" in _lib.last_error()

"""CPU-only checks of the C-ABI boundary: the library loads, exports every symbol the header
declares, and rejects bad arguments on the host without touching a device."""
import ctypes
import os
import re

import pytest

from conftest import ROOT

HEADER = os.path.join(ROOT, "include", "trlk.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(trlk_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from trl_amd import _lib

    names = _declared_symbols()
    assert "trlk_logp_entropy_fwd" in names and "trlk_grpo_loss" in names and len(names) >= 9
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in names:
        assert hasattr(raw, name), f"{name} is declared in include/trlk.h but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature in trl_amd/_lib.py"
    assert _lib.lib.trlk_version() == _lib.ABI_VERSION == 2


def test_host_side_argument_validation():
    from trl_amd import _lib

    lib = _lib.lib
    fake = 0x1000  # never dereferenced: every call below must fail validation first
    # vocab = 0
    rc = lib.trlk_logp_entropy_fwd(fake, _lib.BF16, 1, 1, 0, 0, 0, fake, 1, 1.0, None, fake, None, None, None, 0, None, None)
    assert rc == -2 and "vocab" in _lib.last_error()
    # unsupported dtype code
    rc = lib.trlk_logp_entropy_fwd(fake, 7, 1, 1, 8, 8, 8, fake, 1, 1.0, None, fake, None, None, None, 0, None, None)
    assert rc == -3 and "dtype" in _lib.last_error()
    # null logits
    rc = lib.trlk_logp_entropy_fwd(None, _lib.F32, 1, 1, 8, 8, 8, fake, 1, 1.0, None, fake, None, None, None, 0, None, None)
    assert rc == -1
    # overlapping rows
    rc = lib.trlk_logp_entropy_fwd(fake, _lib.F32, 1, 4, 8, 32, 4, fake, 1, 1.0, None, fake, None, None, None, 0, None, None)
    assert rc == -4 and "row_stride" in _lib.last_error()
    # temperature <= 0
    rc = lib.trlk_logp_entropy_fwd(fake, _lib.F32, 1, 4, 8, 32, 8, fake, 1, 0.0, None, fake, None, None, None, 0, None, None)
    assert rc == -5 and "temperature" in _lib.last_error()
    # row statistics: vocabulary too large for the exact count
    rc = lib.trlk_logp_entropy_fwd(fake, _lib.BF16, 1, 1, 1 << 24, 1 << 24, 1 << 24, fake, 1, 1.0, None, fake, None, None,
                                   fake, 1, None, None)
    assert rc == -7 and "row statistics" in _lib.last_error()
    # backward: window does not fit the output rows
    rc = lib.trlk_logp_entropy_bwd(fake, _lib.F32, 1, 4, 8, 32, 8, fake, 1, 1.0, fake, None, fake, None, fake, 4, 1, 32,
                                   8, None)
    assert rc == -2 and "do not fit" in _lib.last_error()
    # backward: too many indices per row
    rc = lib.trlk_logp_entropy_bwd(fake, _lib.F32, 1, 4, 8, 32, 8, fake, 65, 1.0, fake, None, fake, None, fake, 4, 0,
                                   32, 8, None)
    assert rc == -7
    # advantages: n not a multiple of the group size
    assert lib.trlk_group_advantages(fake, 7, 2, 0, fake, None) == -2
    assert lib.trlk_group_advantages(fake, 8, 2, 5, fake, None) == -5
    # grpo: beta != 0 without reference log-probs; missing workspace; bad loss type
    args = dict(ref=None, beta=0.04, ws=fake, ws_bytes=1 << 20, loss_type=_lib.GRPO, term=_lib.TERM_CLIP, seq=0,
                adv_stride_t=0, tau=1.0)

    def grpo(**kw):
        a = dict(args, **kw)
        return lib.trlk_grpo_loss(fake, None, a["ref"], None, fake, 1, a["adv_stride_t"], fake, None, None, None, 4,
                                  16, a["loss_type"], a["term"], a["seq"], 0.2, 0.2, float("nan"), a["beta"], 0, 1.0,
                                  1.0, None, 1.0, 0.0, a["tau"], 1.05, fake, fake, fake, None, a["ws"], a["ws_bytes"],
                                  None)

    assert grpo() == -1 and "reference log-probs" in _lib.last_error()
    assert grpo(beta=0.0, ws_bytes=8) == -6
    assert grpo(beta=0.0, loss_type=9) == -5
    assert grpo(beta=0.0, loss_type=_lib.DAPO) == -1  # DAPO needs the normaliser scalar
    assert grpo(beta=0.0, term=7) == -5
    assert grpo(beta=0.0, term=_lib.TERM_WEIGHTED_LOGP) == -1  # needs the per-sequence coefficients
    assert grpo(beta=0.0, term=_lib.TERM_SAPO, tau=0.0) == -5
    assert lib.trlk_grpo_workspace_bytes(64) >= 64 * 10 * 4
    # dpo: odd batch
    assert lib.trlk_dpo_loss(fake, fake, fake, fake, 3, 8, 0.1, fake, fake, fake, fake, None) == -2
    assert lib.trlk_rloo_loss(fake, fake, fake, fake, 0, 8, 0.2, 0.2, fake, fake, fake, fake, None) == -2
    # single-pass GRPO: fp32 logits, a vocabulary that does not fit one workgroup, ragged or misaligned rows,
    # beta != 0 without reference log-probs, a window that does not fit the output rows
    fake16 = 0x1000

    def fused(dtype=_lib.BF16, vocab=4096, logits=fake16, row_stride=None, beta=0.0, ref=None, out_rows=4, offset=0,
              term=_lib.TERM_CLIP):
        rs = vocab if row_stride is None else row_stride
        return lib.trlk_grpo_fused_fwd_bwd(logits, dtype, 2, 4, vocab, 4 * rs, rs, fake, 1.0, None, ref, fake, 1, 0, fake,
                                           None, None, fake, None, term, 0.2, 0.2, float("nan"), beta, 0, 1.0, 1.05, fake, fake,
                                           fake, fake16, out_rows, offset, out_rows * vocab, vocab, 0, None, None)

    assert lib.trlk_grpo_fused_max_vocab(_lib.BF16) == 41 * 1024 * 8 and lib.trlk_grpo_fused_max_vocab(_lib.F32) == 41 * 1024 * 4
    assert lib.trlk_grpo_fused_max_vocab(99) == 0
    assert fused(dtype=99) == -3 and "two-pass" in _lib.last_error()
    assert fused(vocab=12) == -7 and fused(vocab=41 * 1024 * 8 + 8) == -7  # (4100 would go ahead: rows need not be whole vectors)
    assert fused(logits=fake16 + 1) == -4  # (not even aligned to an element; 2-byte aligned rows are taken)
    assert fused(beta=0.1) == -1 and fused(term=9) == -5
    assert fused(out_rows=3) == -2 and fused(out_rows=8, offset=5) == -2
    assert lib.trlk_scale_unless_one(fake16, 99, 64, fake, None) == -3
    assert lib.trlk_scale_unless_one(fake16, _lib.BF16, -8, fake, None) == -2
    # fused head: fp32 operands, ragged hidden size, a stash whose rows are too short, missing workspace

    def head_fwd(dtype=_lib.BF16, h=64, stash=None, stash_ld=0, ws=fake16, ws_bytes=1 << 30):
        return lib.trlk_fused_head_fwd(fake16, fake16, fake, dtype, 300, 1000, h, h, h, 1.0, 0.0, 1.0, None, fake, fake,
                                       fake, None, stash, stash_ld, None, ws, ws_bytes, None)

    assert head_fwd(dtype=_lib.F32) == -3 and "bf16 or fp16" in _lib.last_error()
    assert head_fwd(h=60) == -4
    assert head_fwd(stash=fake16, stash_ld=300) == -4 and "stash" in _lib.last_error()
    assert head_fwd(ws_bytes=16) == -6
    ld = ctypes.c_int64(0)
    assert lib.trlk_fused_head_stash_bytes(300, 1000, ctypes.addressof(ld)) == (1024 // 4 + 1024 // 128 + 1) * 512 * 8 and ld.value == 512
    assert lib.trlk_fused_head_bwd(fake16, fake16, fake, _lib.BF16, 300, 1000, 64, 64, 64, 1.0, 0.0, 1.0, None, fake, fake,
                                   256, fake16, 256, None, fake16, fake16, None, fake16, 1 << 40, None) == -4
    assert lib.trlk_fused_head_bwd(fake16, fake16, fake, _lib.BF16, 300, 1000, 64, 64, 64, 1.0, 0.0, 1.0, None, fake, fake,
                                   0, None, 0, None, fake16, fake16, None, fake16, 1 << 40, None) == -5  # chunk_size
    assert lib.trlk_fused_head_bwd(fake16, fake16, fake, _lib.BF16, 300, 1000, 64, 64, 64, 1.0, 0.0, 1.0, None, fake, fake,
                                   256, None, 0, fake16, fake16, fake16, None, fake16, 1 << 40, None) == -1  # columns, no stash
    # fp32 operands as bf16 pieces, and the plain product on them: side, strides, contraction length, dtype, alignment
    assert lib.trlk_split_bf16x3(fake16, 4, 10, 10, 2, fake16, 96, None) == -5 and "side" in _lib.last_error()
    assert lib.trlk_split_bf16x3(fake16, 4, 10, 10, 0, fake16, 60, None) == -4  # 6 * 16 columns are needed
    assert lib.trlk_split_bf16x3(fake16, 4, 10, 8, 0, fake16, 96, None) == -4
    assert lib.trlk_split_bf16x3(None, 4, 10, 10, 0, fake16, 96, None) == -1
    assert lib.trlk_split_bf16x3(None, 0, 10, 10, 0, None, 96, None) == 0

    def gemm(a=fake16, lda=64, ldb=64, dtype=_lib.BF16, k=64, ldo=16):
        return lib.trlk_gemm_nt(a, lda, fake16, ldb, dtype, 8, 16, k, fake16, ldo, 0, None)

    assert gemm(dtype=_lib.F32) == -3 and gemm(k=60) == -4 and gemm(lda=56) == -4 and gemm(ldo=8) == -4
    assert gemm(a=fake16 + 2) == -4 and gemm(a=None) == -1 and gemm(k=0) == -2
    # an empty problem is a successful no-op
    assert lib.trlk_logp_entropy_fwd(None, _lib.F32, 0, 4, 8, 32, 8, None, 1, 1.0, None, None, None, None, None, 0, None, None) == 0
    assert _lib.last_error() == ""


def test_check_raises_python_exceptions():
    from trl_amd import _lib

    with pytest.raises(_lib.TrlkArgumentError, match="vocab"):
        _lib.check(_lib.lib.trlk_logp_entropy_fwd(0x1000, _lib.BF16, 1, 1, 0, 0, 0, 0x1000, 1, 1.0, None, 0x1000, None,
                                                  None, None, 0, None, None))
    with pytest.raises(TypeError):
        import torch

        _lib.dtype_code(torch.complex64)


def test_cpu_tensors_fail_loudly():
    """The ops are registered for the device only: no silent CPU path."""
    import torch

    import trl_amd

    with pytest.raises((NotImplementedError, RuntimeError)):
        trl_amd.selective_log_softmax(torch.randn(2, 3, 16), torch.zeros(2, 3, dtype=torch.long))

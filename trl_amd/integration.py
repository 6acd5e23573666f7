"""Binds the kernels into an installed `trl` (the reference) at run time.

TRL has no plugin registry: its hot-path helpers are module-level functions imported *by name* into
every trainer module, and the loss is a trainer method.  `patch_trl()` therefore rebinds
  * `selective_log_softmax`, `entropy_from_logits`, `_ChunkedLogProbFunction`, `patch_chunked_lm_head`
    in `trl.trainer.utils` **and** in every already-imported `trl.*` module that holds its own reference;
  * `trl.trainer.sft_trainer._chunked_cross_entropy_loss` (the default SFT loss);
  * `GRPOTrainer._get_per_token_logps_and_entropies` / `_compute_loss` (optional, `grpo=True`);
  * `DPOTrainer._compute_loss` (optional, `dpo=True`): one pass over the logits instead of six;
  * `RLOOTrainer._get_per_token_logps_and_entropies` / `_compute_loss` (optional, `rloo=True`);
  * the fused-linear loss operators behind `use_liger_kernel` (optional, `liger=True`): the names
    `LigerFusedLinearGRPOLoss` / `LigerFusedLinearDPOLoss` and `is_liger_kernel_available` in
    `trl.trainer.grpo_trainer` / `trl.trainer.dpo_trainer` (trl/trainer/grpo_trainer.py:1020-1044,
    trl/trainer/dpo_trainer.py:834), so that `compute_liger_loss` / `_compute_loss_liger` call the fused head.
`unpatch_trl()` restores the originals.
"""
from __future__ import annotations

import sys

from .trainer import grpo_trainer as _grpo
from .trainer import utils as _utils

_FUNCTIONS = ("selective_log_softmax", "entropy_from_logits", "_ChunkedLogProbFunction", "patch_chunked_lm_head")
_saved: list[tuple[object, str, object]] = []


_MISSING = object()


def _set(mod, name, value) -> None:
    _saved.append((mod, name, getattr(mod, name, _MISSING)))
    setattr(mod, name, value)


def patch_trl(grpo: bool = True, liger: bool = False, dpo: bool = False, rloo: bool = False, kto: bool = False) -> int:
    """Returns the number of names rebound.  Needs `trl` to be importable."""
    import trl.trainer.utils as ref_utils

    if _saved:
        return 0
    originals = {name: getattr(ref_utils, name) for name in _FUNCTIONS if hasattr(ref_utils, name)}
    count = 0
    for mod_name, mod in list(sys.modules.items()):
        if mod is None or not (mod_name == "trl" or mod_name.startswith("trl.")):
            continue
        for name, orig in originals.items():
            if getattr(mod, name, None) is orig:
                _saved.append((mod, name, orig))
                setattr(mod, name, getattr(_utils, name))
                count += 1
    try:  # SFT's default `chunked_nll` loss (trl/trainer/sft_trainer.py:117-234)
        import trl.trainer.sft_trainer as ref_sft

        from .trainer.sft_trainer import _chunked_cross_entropy_loss

        if hasattr(ref_sft, "_chunked_cross_entropy_loss"):
            _saved.append((ref_sft, "_chunked_cross_entropy_loss", ref_sft._chunked_cross_entropy_loss))
            ref_sft._chunked_cross_entropy_loss = _chunked_cross_entropy_loss
            count += 1
    except ImportError:
        pass
    if grpo:
        from trl.trainer.grpo_trainer import GRPOTrainer

        for name in ("_get_per_token_logps_and_entropies", "_compute_loss"):
            _saved.append((GRPOTrainer, name, GRPOTrainer.__dict__[name]))
            setattr(GRPOTrainer, name, getattr(_grpo.GRPOLossMixin, name))
            count += 1
        # helpers of the mix-in's methods (no methods of these names in the reference class)
        for name in ("_finish_loss", "_model_inputs"):
            _saved.append((GRPOTrainer, name, GRPOTrainer.__dict__.get(name, _MISSING)))
            setattr(GRPOTrainer, name, getattr(_grpo.GRPOLossMixin, name))
    if rloo:
        from trl.trainer.rloo_trainer import RLOOTrainer

        from .trainer.rloo_trainer import RLOOLossMixin

        for name in ("_get_per_token_logps_and_entropies", "_compute_loss"):
            _saved.append((RLOOTrainer, name, RLOOTrainer.__dict__[name]))
            setattr(RLOOTrainer, name, getattr(RLOOLossMixin, name))
            count += 1
        _saved.append((RLOOTrainer, "_model_inputs", RLOOTrainer.__dict__.get("_model_inputs", _MISSING)))
        RLOOTrainer._model_inputs = RLOOLossMixin._model_inputs
    if kto:
        from trl.trainer.kto_trainer import KTOTrainer

        from .trainer.kto_trainer import KTOLossMixin

        for name in ("_compute_kl_logps", "_compute_loss"):
            _saved.append((KTOTrainer, name, KTOTrainer.__dict__[name]))
            setattr(KTOTrainer, name, getattr(KTOLossMixin, name))
            count += 1
        _set(KTOTrainer, "_NON_MODEL_KEYS", KTOLossMixin._NON_MODEL_KEYS)
    if dpo:
        from trl.trainer.dpo_trainer import DPOTrainer

        from .trainer.dpo_trainer import DPOLossMixin

        _saved.append((DPOTrainer, "_compute_loss", DPOTrainer.__dict__["_compute_loss"]))
        DPOTrainer._compute_loss = DPOLossMixin._compute_loss
        count += 1
    if liger:
        import trl.trainer.dpo_trainer as ref_dpo
        import trl.trainer.grpo_trainer as ref_grpo

        from .trainer.fused_linear import FusedLinearDPOLoss, FusedLinearGRPOLoss

        _set(ref_grpo, "LigerFusedLinearGRPOLoss", FusedLinearGRPOLoss)
        _set(ref_grpo, "is_liger_kernel_available", lambda *a, **k: True)
        _set(ref_dpo, "LigerFusedLinearDPOLoss", FusedLinearDPOLoss)
        try:
            import trl.trainer.kto_trainer as ref_kto

            from .trainer.fused_linear import FusedLinearKTOLoss

            _set(ref_kto, "LigerFusedLinearKTOLoss", FusedLinearKTOLoss)
            _set(ref_kto, "is_liger_kernel_available", lambda *a, **k: True)
        except ImportError:
            pass
        _set(ref_dpo, "is_liger_kernel_available", lambda *a, **k: True)
        count += 4
    return count


def unpatch_trl() -> None:
    while _saved:
        obj, name, orig = _saved.pop()
        if orig is _MISSING:
            delattr(obj, name)
        else:
            setattr(obj, name, orig)

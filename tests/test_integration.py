"""`patch_trl()` rebinding, exercised against the reference tree when it is present (development
container only; skipped on the GPU box, which has no reference)."""
import os
import sys

import pytest

REFERENCE = "/root/reference"


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "trl")), reason="reference tree not present")
def test_patch_trl_rebinds_every_importer():
    sys.path.insert(0, REFERENCE)
    try:
        import trl.trainer.dpo_trainer as ref_dpo
        import trl.trainer.grpo_trainer as ref_grpo
        import trl.trainer.utils as ref_utils

        import trl_amd
        from trl_amd import integration

        orig = ref_utils.selective_log_softmax
        orig_loss = ref_grpo.GRPOTrainer._compute_loss
        n = integration.patch_trl()
        try:
            assert n >= 8
            for mod in (ref_utils, ref_grpo, ref_dpo):
                assert mod.selective_log_softmax is trl_amd.selective_log_softmax
            assert ref_grpo.entropy_from_logits is trl_amd.entropy_from_logits
            assert ref_utils._ChunkedLogProbFunction is trl_amd._ChunkedLogProbFunction
            assert ref_grpo.GRPOTrainer._compute_loss is trl_amd.GRPOLossMixin._compute_loss
            assert ref_grpo.GRPOTrainer._finish_loss is trl_amd.GRPOLossMixin._finish_loss
            assert integration.patch_trl() == 0  # idempotent
        finally:
            integration.unpatch_trl()
        assert ref_grpo.selective_log_softmax is orig and ref_grpo.GRPOTrainer._compute_loss is orig_loss
        assert not hasattr(ref_grpo.GRPOTrainer, "_finish_loss")
    finally:
        sys.path.remove(REFERENCE)


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "trl")), reason="reference tree not present")
def test_patch_trl_binds_the_fused_linear_operators():
    """`liger=True` puts the fused-linear operators under the names the reference's trainers construct
    (trl/trainer/grpo_trainer.py:1027, trl/trainer/dpo_trainer.py:834) and removes them again."""
    sys.path.insert(0, REFERENCE)
    try:
        import trl.trainer.dpo_trainer as ref_dpo
        import trl.trainer.grpo_trainer as ref_grpo

        import trl_amd
        from trl_amd import integration

        had = hasattr(ref_grpo, "LigerFusedLinearGRPOLoss")
        integration.patch_trl(grpo=False, liger=True)
        try:
            assert ref_grpo.LigerFusedLinearGRPOLoss is trl_amd.FusedLinearGRPOLoss
            assert ref_dpo.LigerFusedLinearDPOLoss is trl_amd.FusedLinearDPOLoss
            assert ref_grpo.is_liger_kernel_available() and ref_dpo.is_liger_kernel_available()
            # the constructor calls of the reference (keyword sets at grpo_trainer.py:1027-1044, dpo_trainer.py:834)
            op = ref_grpo.LigerFusedLinearGRPOLoss(
                beta=0.04, epsilon_low=0.2, epsilon_high=0.2, temperature=1.0, use_ref_model=True, loss_type="dapo",
                max_completion_length=16, importance_sampling_level="token", delta=None, use_bias_correction_kl=False,
                sapo_temperature_pos=1.0, sapo_temperature_neg=1.05, vespo_k_pos=2.0, vespo_lambda_pos=3.0,
                vespo_k_neg=3.0, vespo_lambda_neg=2.0)
            assert op.beta == 0.04
            ref_dpo.LigerFusedLinearDPOLoss(beta=0.1, loss_type="sigmoid")
            import trl.trainer.kto_trainer as ref_kto

            assert ref_kto.LigerFusedLinearKTOLoss is trl_amd.FusedLinearKTOLoss
            ref_kto.LigerFusedLinearKTOLoss(beta=0.1, use_ref_model=True)  # kto_trainer.py:978
        finally:
            integration.unpatch_trl()
        assert hasattr(ref_grpo, "LigerFusedLinearGRPOLoss") == had
    finally:
        sys.path.remove(REFERENCE)


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "trl")), reason="reference tree not present")
def test_patch_trl_rebinds_the_other_trainers():
    """`dpo`, `rloo`, `kto`: the loss methods of those trainers are rebound and restored."""
    sys.path.insert(0, REFERENCE)
    try:
        from trl.trainer.dpo_trainer import DPOTrainer
        from trl.trainer.kto_trainer import KTOTrainer
        from trl.trainer.rloo_trainer import RLOOTrainer

        import trl_amd
        from trl_amd import integration

        before = (DPOTrainer._compute_loss, KTOTrainer._compute_loss, KTOTrainer._compute_kl_logps, RLOOTrainer._compute_loss)
        integration.patch_trl(grpo=False, dpo=True, rloo=True, kto=True)
        try:
            assert DPOTrainer._compute_loss is trl_amd.DPOLossMixin._compute_loss
            assert KTOTrainer._compute_loss is trl_amd.KTOLossMixin._compute_loss
            assert KTOTrainer._compute_kl_logps is trl_amd.KTOLossMixin._compute_kl_logps
            assert RLOOTrainer._compute_loss is trl_amd.RLOOLossMixin._compute_loss
        finally:
            integration.unpatch_trl()
        assert before == (DPOTrainer._compute_loss, KTOTrainer._compute_loss, KTOTrainer._compute_kl_logps,
                          RLOOTrainer._compute_loss)
        assert not hasattr(KTOTrainer, "_NON_MODEL_KEYS")
    finally:
        sys.path.remove(REFERENCE)

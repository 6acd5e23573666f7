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
            assert integration.patch_trl() == 0  # idempotent
        finally:
            integration.unpatch_trl()
        assert ref_grpo.selective_log_softmax is orig and ref_grpo.GRPOTrainer._compute_loss is orig_loss
    finally:
        sys.path.remove(REFERENCE)

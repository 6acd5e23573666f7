"""MI355X-native kernels for TRL's per-token log-probability, entropy and policy-loss path.

Importing the package loads `trl_amd/lib/libtrlk.so`; there is no fallback if it is missing.
"""
from . import _lib, ops
from .ops import check_device_errors
from .trainer import (RLOOLossMixin, KTOLossMixin, kto_compute_loss, kto_sequence_logps, vllm_importance_sampling_ratio, DPOLossMixin, dpo_compute_loss, dpo_metrics_to_dict, dpo_sequence_logps, FusedLinearDPOLoss, FusedLinearGRPOLoss, FusedLinearKTOLoss, GRPOLossMixin, _ChunkedLogProbFunction, chunked_logprobs_from_hidden, patch_chunked_lm_head, dpo_loss_from_logits, dpo_per_token_logps, dpo_sigmoid_loss, entropy_from_logits,
                      group_advantages, grpo_loss, grpo_loss_from_logits, grpo_single_pass_supported, logps_and_entropies, per_token_logps_and_entropies, rloo_advantages,
                      rloo_loss, selective_log_softmax)

__version__ = "0.1.0"

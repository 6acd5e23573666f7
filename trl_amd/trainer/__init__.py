from .dpo_trainer import (DPOLossMixin, dpo_compute_loss, dpo_loss_from_logits, dpo_metrics_to_dict, dpo_per_token_logps,
                          dpo_sequence_logps, dpo_sigmoid_loss)
from .grpo_trainer import (GRPOLossMixin, get_high_entropy_mask, get_off_policy_mask, group_advantages, grpo_loss,
                           grpo_loss_from_logits, grpo_single_pass_supported,
                           metrics_to_dict, per_token_logps_and_entropies, vllm_importance_sampling_ratio)
from .kto_trainer import KTOLossMixin, kto_compute_loss, kto_sequence_logps
from .rloo_trainer import RLOOLossMixin, rloo_advantages, rloo_loss
from .utils import (_ChunkedLogProbFunction, chunked_logprobs_from_hidden, entropy_from_logits, logps_and_entropies,
                    nanmax, nanmin, nanstd, patch_chunked_lm_head, selective_log_softmax)
from .sft_trainer import _chunked_cross_entropy_loss
from .fused_linear import FusedLinearDPOLoss, FusedLinearGRPOLoss, FusedLinearKTOLoss

"""mindspeed_rl_amd - MI355X (gfx950) kernels for MindSpeed-RL's actor log-probability and
GRPO / DAPO policy-loss path, behind the reference's own Python call surface.

Everything here dispatches to libmrl_hip.so (C ABI in ``include/mrl_hip.h``); there is no CPU
or eager fallback.  Build the library with ``python -m mindspeed_rl_amd._build``.
"""
from . import _lib
from .advantage import (FixedKLController, compute_group_norm_advantage_return, dynamic_sampling_keep, get_last_reward,
                        dynamic_sampling_keep_mask)
from .functional import clip_by_value, is_multimodal, masked_mean, masked_sum
from .lmhead import fused_lmhead_policy_loss, lmhead_logprob
from .loss import (BaseLossFunc, DAPOActorLossFunc, DeferredStats, GradScaleState, GRPOActorLossFunc, LossFuncFactory, LossRegister,
                   MultimodalLogProbComputer, PPOActorLossFunc, ReferenceLossFunc, RewardLossFunc,
                   StandardLogProbComputer, fused_logprob_policy_loss, fused_supported, policy_loss)
from .packing import (generate_mask, pack_index, postprocess_packed_seqs, preprocess_packed_seqs, response_window,
                      truncate_middle_and_pad, truncate_prompt_and_pad)
from .seqlen_balancing import (balanced_bin_packing, get_reverse_idx, get_seqlen_balanced_partitions, heapq_partition,
                               heapq_partition_with_max, karmarkar_karp, rearrange_micro_batches,
                               split_batches_with_dynamic_bsz)
from .value_path import (AdaptiveKLController, CriticLossFunc, compute_gae_advantage_return, kl_token_level_rewards,
                         masked_var, masked_whiten, value_loss)
from .wire import (pack_experience_columns, pack_padded_columns, pad_multiple, padding_dict_to_tensor_dict,
                   remove_padding_and_split_to_list, remove_padding_tensor_dict_to_dict, truncate_rows,
                   unpack_pad_experience)
from .vocab_ops import (compute_kl_penalty, compute_log_probs, get_parallel_state, get_vocab_parallel,
                        merge_vocab_shard_stats, set_parallel_state, set_vocab_parallel, vocab_logprob_entropy,
                        vocab_parallel_cross_entropy, vocab_parallel_entropy, vocab_shard_backward, vocab_shard_stats)

__version__ = "0.1.0"


def library_version():
    """MRL_VERSION of the loaded libmrl_hip.so (loads it; raises if it is not built)."""
    return _lib.load().mrl_version()

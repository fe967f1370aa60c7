"""Oracle (test infrastructure): group-relative advantages and the DAPO group filter.

* ``mindspeed_rl/trainer/utils/compute_utils.py:152-191``  ``compute_group_norm_advantage_return``
  (fp64, unbiased std, eps 1e-6, group id = row // n_sample_per_prompt because the rows of
  one prompt are consecutive, ``trainer/utils/transfer_dock.py:1221-1225``)
* ``mindspeed_rl/trainer/utils/compute_utils.py:51-58``    ``FixedKLController``
* ``mindspeed_rl/workers/dynamic_sampling.py:81-86``       keep a group iff ``np.std(group) > 0``
  (population std, exact comparison) or it has a single member

* ``mindspeed_rl/trainer/utils/compute_utils.py:33-48``    ``AdaptiveKLController``
* ``mindspeed_rl/trainer/utils/compute_utils.py:61-104``   the arithmetic inside ``apply_kl_penalty``
  (token-level rewards = score at the last response token - beta * KL penalty; the Ray / TransferDock
  loop around it is not restated)
* ``mindspeed_rl/trainer/utils/compute_utils.py:107-149``  ``compute_gae_advantage_return``

Pinned by ``tests/ut/utils/test_compute_utils.py:7-76`` (+-0.7071 for rewards [1, 2]; the adaptive
controller's 1.1 / 0.9; the GAE vector with gamma 0).
"""
from copy import deepcopy

import numpy as np
import torch


def compute_group_norm_advantage_return(token_level_rewards, eos_mask, response_length, n_sample_per_prompt):
    scores = torch.as_tensor(token_level_rewards).detach().clone().to(torch.float64)
    scores = scores.reshape(-1, n_sample_per_prompt)
    scores = (scores - scores.mean(dim=1, keepdim=True)) / (scores.std(dim=1, keepdim=True) + 1e-6)
    scores = scores.reshape(response_length.shape).to(torch.float32)
    spread = scores.repeat(1, eos_mask.shape[1]) * eos_mask
    advantages = deepcopy(spread)
    returns = deepcopy(advantages)
    return advantages, returns


class AdaptiveKLController:
    """``compute_utils.py:33-48``."""

    def __init__(self, init_kl_coef, target_kl, horizon):
        self.value = init_kl_coef
        self.target = target_kl
        self.horizon = horizon

    def update(self, current_kl, n_steps):
        proportional_error = np.clip(current_kl / self.target - 1, -0.2, 0.2)
        mult = 1 + proportional_error * n_steps / self.horizon
        self.value *= mult


class FixedKLController:
    def __init__(self, init_kl_coef):
        self.value = init_kl_coef

    def update(self, current_kl, n_steps):
        pass


def dynamic_sampling_keep(metric_values, n_samples_per_prompt):
    """Row indices kept by the DAPO filter, in order.  ``np.std`` runs in the dtype it is given
    (float32 metrics stay float32, python lists become float64), as in the reference."""
    values = np.asarray(metric_values).reshape(-1)
    kept = []
    for lo in range(0, len(values), n_samples_per_prompt):
        group = values[lo:lo + n_samples_per_prompt]
        if np.std(group) > 0 or len(group) == 1:
            kept.extend(range(lo, lo + n_samples_per_prompt))
    return kept


def kl_token_level_rewards(old_log_prob, ref_log_prob, response_length, rm_scores, beta, penalty="kl"):
    """``compute_utils.py:80-97``: returns ``(token_level_rewards [B, L], current_kl)``; the score
    of a sample is added at its last response token, ``beta`` is ``kl_ctrl.value``."""
    from . import loss, packing
    response_mask = packing.generate_mask(old_log_prob, response_length)
    kld = loss.compute_kl_penalty(old_log_prob, ref_log_prob, kl_penalty=penalty)
    kld = kld * response_mask
    reward_tensor = torch.zeros_like(old_log_prob, dtype=torch.float32)
    for i in range(old_log_prob.shape[0]):
        valid_response_length = response_length[i] - 1
        reward_tensor[i, int(valid_response_length.item())] = rm_scores[i]
    token_level_rewards = reward_tensor - beta * kld
    current_kl = loss.masked_mean(kld, mask=response_mask, axis=-1)
    current_kl = torch.mean(current_kl, dim=0).item()
    return token_level_rewards, current_kl


def compute_gae_advantage_return(token_level_rewards, values, eos_mask, gamma, lam):
    """``compute_utils.py:107-149``: reverse scan over the full width (the mask only enters the
    whitening), fp32, one torch op per step as in the reference."""
    from . import loss
    with torch.no_grad():
        lastgaelam = 0
        advantages_reversed = []
        gen_len = token_level_rewards.shape[-1]
        for t in reversed(range(gen_len)):
            nextvalues = values[:, t + 1] if t < gen_len - 1 else 0.0
            delta = token_level_rewards[:, t] + gamma * nextvalues - values[:, t]
            lastgaelam = delta + gamma * lam * lastgaelam
            advantages_reversed.append(lastgaelam)
        advantages = torch.stack(advantages_reversed[::-1], dim=1)
        returns = advantages + values
        advantages = loss.masked_whiten(advantages, eos_mask)
    return advantages, returns


def get_last_reward(rm_scores, n_sample_batch):
    """``compute_utils.py:277-291``."""
    reward = rm_scores.reshape(-1, n_sample_batch)
    last_reward = (reward - reward.mean(dim=1, keepdim=True)) / (reward.std(dim=1, keepdim=True) + 1e-8)
    return last_reward.reshape(rm_scores.shape)

"""Oracle (test infrastructure): group-relative advantages and the DAPO group filter.

* ``mindspeed_rl/trainer/utils/compute_utils.py:152-191``  ``compute_group_norm_advantage_return``
  (fp64, unbiased std, eps 1e-6, group id = row // n_sample_per_prompt because the rows of
  one prompt are consecutive, ``trainer/utils/transfer_dock.py:1221-1225``)
* ``mindspeed_rl/trainer/utils/compute_utils.py:51-58``    ``FixedKLController``
* ``mindspeed_rl/workers/dynamic_sampling.py:81-86``       keep a group iff ``np.std(group) > 0``
  (population std, exact comparison) or it has a single member

Pinned by ``tests/ut/utils/test_compute_utils.py:61-76`` (+-0.7071 for rewards [1, 2]).
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

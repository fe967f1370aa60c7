"""Group-relative advantages, the fixed KL controller and the DAPO group filter.

Host-side mirror of ``compute_group_norm_advantage_return`` and ``FixedKLController``
(``mindspeed_rl/trainer/utils/compute_utils.py:51-58,152-191``) and of the keep-rule inside
``DynamicSampling.dynamic_sampling`` (``mindspeed_rl/workers/dynamic_sampling.py:81-86``).
"""
import torch

from . import _lib


class FixedKLController:
    """Reference: ``trainer/utils/compute_utils.py:51-58``."""

    def __init__(self, init_kl_coef):
        self.value = init_kl_coef

    def update(self, current_kl, n_steps):
        pass


def compute_group_norm_advantage_return(token_level_rewards, eos_mask, response_length, n_sample_per_prompt):
    """Reference: ``trainer/utils/compute_utils.py:152-191``.

    ``token_level_rewards`` holds one scalar reward per response (any shape with ``B`` elements),
    rows of one prompt are consecutive; ``eos_mask`` is ``[B, L]``.  Returns ``(advantages,
    returns)``, two separate fp32 ``[B, L]`` tensors with identical values.  The normalisation is
    done in fp64 with the unbiased standard deviation and eps 1e-6, on the device of ``eos_mask``.
    """
    mask = eos_mask
    if mask.dtype not in (torch.float32, torch.int64, torch.int32, torch.uint8, torch.bool):
        mask = mask.to(torch.float32)
    dev = _lib.require_device(mask)
    rewards = torch.as_tensor(token_level_rewards).detach()
    if rewards.dtype not in (torch.float32, torch.float64):
        rewards = rewards.to(torch.float64)
    rewards = rewards.to(dev).reshape(-1).contiguous()
    batch = rewards.numel()
    if batch != response_length.numel():
        raise RuntimeError("shape '%s' is invalid for input of size %d" % (list(response_length.shape), batch))
    if batch % n_sample_per_prompt != 0:
        raise RuntimeError("shape '[-1, %d]' is invalid for input of size %d" % (n_sample_per_prompt, batch))
    if mask.dim() != 2 or mask.shape[0] not in (1, batch):
        raise RuntimeError("eos_mask must have shape (%d, L) or (1, L)" % batch)
    mask = mask.expand(batch, mask.shape[1]).contiguous()      # the reference broadcasts the mask
    width = mask.shape[1]
    adv = torch.empty((batch, width), dtype=torch.float32, device=dev)
    ret = torch.empty((batch, width), dtype=torch.float32, device=dev)
    _lib.call("mrl_group_advantage", _lib.ptr(rewards), _lib.dtype_code(rewards), batch, int(n_sample_per_prompt),
              _lib.ptr(mask), _lib.dtype_code(mask), width, _lib.ptr(adv), _lib.ptr(ret), _lib.stream(dev))
    return adv, ret


def get_last_reward(rm_scores, n_sample_batch: int):
    """Reference: ``trainer/utils/compute_utils.py:277-291``: every reward standardised inside its
    group of ``n_sample_batch`` consecutive samples, ``(r - mean) / (std + 1e-8)`` with the unbiased
    standard deviation; same shape as ``rm_scores``, fp32."""
    dev = _lib.require_device(rm_scores)
    rewards = rm_scores.detach()
    if rewards.dtype not in (torch.float32, torch.float64):
        rewards = rewards.to(torch.float32)
    flat = rewards.reshape(-1).contiguous()
    n = flat.numel()
    if n % n_sample_batch != 0:
        raise RuntimeError("shape '[-1, %d]' is invalid for input of size %d" % (n_sample_batch, n))
    out = torch.empty(n, dtype=torch.float32, device=dev)
    _lib.call("mrl_group_standardize", _lib.ptr(flat), _lib.dtype_code(flat), n, int(n_sample_batch), 1e-8, _lib.ptr(out),
              _lib.stream(dev))
    return out.view(rm_scores.shape)


def dynamic_sampling_keep_mask(metric_values, n_samples_per_prompt):
    """uint8 ``[N]`` device mask: 1 for the rows of every group the DAPO filter keeps
    (``numpy.std(group) > 0`` or a single-member group), following numpy's arithmetic in the
    metric's own dtype (fp32 or fp64)."""
    metric = torch.as_tensor(metric_values)
    if metric.dtype not in (torch.float32, torch.float64):
        metric = metric.to(torch.float64)
    metric = metric.reshape(-1).contiguous()
    dev = _lib.require_device(metric)
    keep = torch.empty(metric.numel(), dtype=torch.uint8, device=dev)
    _lib.call("mrl_group_keep_mask", _lib.ptr(metric), _lib.dtype_code(metric), metric.numel(),
              int(n_samples_per_prompt), _lib.ptr(keep), _lib.stream(dev))
    return keep


def dynamic_sampling_keep(metric_values, n_samples_per_prompt):
    """Kept row indices as a python list, in order (what the reference's loop builds)."""
    keep = dynamic_sampling_keep_mask(metric_values, n_samples_per_prompt)
    return torch.nonzero(keep, as_tuple=False).flatten().tolist()

"""Oracle (test infrastructure): masked reductions, KL penalties, GRPO / DAPO policy loss.

Restates with stock torch ops (so that autograd supplies the backward the reference gets):

* ``mindspeed_rl/utils/torch_functional.py:38-59``                 ``masked_sum`` / ``masked_mean``
* ``mindspeed_rl/utils/compute.py:100-133``                        ``compute_kl_penalty``
* ``mindspeed_rl/models/loss/grpo_actor_loss_func.py:100-144``     ``_compute_grpo_policy_loss``
* ``mindspeed_rl/models/loss/dapo_actor_loss_func.py:105-152``     ``_compute_dapo_policy_loss``
* ``mindspeed_rl/models/loss/grpo_actor_loss_func.py:43-98`` and
  ``dapo_actor_loss_func.py:47-102``                                ``compute_loss`` tail (scale + stats)
* ``mindspeed_rl/models/loss/ppo_actor_loss_func.py:39-133``       PPO actor (the GRPO surrogate without KL)
* ``mindspeed_rl/models/loss/logprob_computer.py:94-145``          ``StandardLogProbComputer.compute``
* ``mindspeed_rl/utils/torch_functional.py:62-106``                ``masked_var`` / ``masked_whiten``
* ``mindspeed_rl/models/loss/critic_loss_func.py:37-111``          critic value loss (``compute_loss`` + clipped MSE)

Pinned by ``tests/ut/utils/test_compute_utils.py:92-108`` (KL vectors),
``tests/ut/utils/test_torch_functional.py:24-29`` (masked mean) and hand-derived cases.
"""
import torch

from . import packing, vocab


def masked_sum(values, mask, axis=None):
    """``torch_functional.py:38-43``: values outside the mask are replaced by 0 first, so
    NaN/Inf there cannot leak; the mask still multiplies (non-binary weights count)."""
    kept = torch.where(mask.bool(), values, 0.0)
    return (kept * mask).sum(axis=axis)


def masked_mean(values, mask, axis=None, epsilon=1e-8):
    """``torch_functional.py:46-59``."""
    return masked_sum(values, mask, axis) / (mask.sum(axis=axis) + epsilon)


def masked_var(values, mask, unbiased=True):
    """``torch_functional.py:62-87``."""
    mean = masked_mean(values, mask)
    centered_values = values - mean
    variance = masked_mean(centered_values ** 2, mask)
    if unbiased:
        mask_sum = mask.sum()
        if mask_sum == 0:
            raise ValueError("At least one element in the mask has to be 1.")
        elif mask_sum == 1:
            bessel_correction = mask_sum
        else:
            bessel_correction = mask_sum / (mask_sum - 1)
        variance = variance * bessel_correction
    return variance


def masked_whiten(values, mask, shift_mean=True):
    """``torch_functional.py:90-106``."""
    mean, var = masked_mean(values, mask), masked_var(values, mask)
    whitened = (values - mean) * torch.rsqrt(var + 1e-8)
    if not shift_mean:
        whitened += mean
    return whitened


def compute_kl_penalty(logprob, ref_logprob, kl_penalty="low_var_kl"):
    """``utils/compute.py:100-133``."""
    if kl_penalty == "kl":
        return logprob - ref_logprob
    if kl_penalty == "abs":
        return (logprob - ref_logprob).abs()
    if kl_penalty == "mse":
        return 0.5 * (logprob - ref_logprob).square()
    if kl_penalty == "low_var_kl":
        delta = torch.clamp(ref_logprob - logprob, min=-20, max=20)
        k3 = (torch.exp(delta) - delta - 1).contiguous()
        return torch.clamp(k3, min=-10, max=10)
    raise NotImplementedError


def grpo_policy_loss(old_log_prob, log_prob, ref_log_prob, advantages, entropy, eos_mask,
                     cliprange, kl_coef, kl_penalty, entropy_coeff):
    """``grpo_actor_loss_func.py:127-144``; ``kl_coef`` is ``kl_ctrl.value``."""
    if old_log_prob is None:
        old_log_prob = log_prob.detach().clone()
    log_ratio = log_prob - old_log_prob
    ratio = torch.exp(log_ratio)
    ppo_kl = masked_mean(-log_ratio, eos_mask)
    entropy_loss = masked_mean(entropy, eos_mask)
    surr1 = -advantages * ratio
    surr2 = -advantages * torch.clamp(ratio, 1.0 - cliprange, 1.0 + cliprange)
    pg_mean = masked_mean(torch.max(surr1, surr2), eos_mask)
    clipfrac = masked_mean(torch.gt(surr2, surr1).float(), eos_mask)
    kl_mean = masked_mean(compute_kl_penalty(log_prob, ref_log_prob, kl_penalty), eos_mask)
    pg_loss = pg_mean + kl_mean * kl_coef - entropy_coeff * entropy_loss
    return pg_loss, clipfrac, ppo_kl, kl_mean, entropy_loss


def ppo_policy_loss(old_log_prob, log_prob, advantages, eos_mask, cliprange, entropy, entropy_coeff):
    """``ppo_actor_loss_func.py:91-133``: the GRPO surrogate without the KL term."""
    if old_log_prob is None:
        old_log_prob = log_prob.detach().clone()
    log_ratio = log_prob - old_log_prob
    ratio = torch.exp(log_ratio)
    ppo_kl = masked_mean(-log_ratio, eos_mask)
    entropy_loss = masked_mean(entropy, eos_mask)
    surr1 = -advantages * ratio
    surr2 = -advantages * torch.clamp(ratio, 1.0 - cliprange, 1.0 + cliprange)
    pg_mean = masked_mean(torch.max(surr1, surr2), eos_mask)
    clipfrac = masked_mean(torch.gt(surr2, surr1).float(), eos_mask)
    return pg_mean - entropy_coeff * entropy_loss, clipfrac, ppo_kl, entropy_loss


def dapo_policy_loss(old_log_prob, log_prob, entropy, entropy_coeff, advantages, eos_mask,
                     clip_ratio_low, clip_ratio_high, token_level_loss):
    """``dapo_actor_loss_func.py:129-152``.  In the sequence-mean branch the reference
    overwrites ``pg_losses`` with the element-wise maximum before the clip fraction is
    taken, and divides by the row's mask sum without an epsilon; both are kept."""
    if old_log_prob is None:
        old_log_prob = log_prob.detach().clone()
    log_ratio = log_prob - old_log_prob
    ratio = torch.exp(log_ratio)
    ppo_kl = masked_mean(-log_ratio, eos_mask)
    entropy_loss = masked_mean(entropy, eos_mask)
    surr1 = -advantages * ratio
    surr2 = -advantages * torch.clamp(ratio, 1.0 - clip_ratio_low, 1.0 + clip_ratio_high)
    if token_level_loss:
        pg_mean = masked_mean(torch.max(surr1, surr2), eos_mask)
    else:
        surr1 = torch.max(surr1, surr2)
        per_seq = torch.sum(surr1 * eos_mask, dim=-1) / torch.sum(eos_mask, dim=-1)
        pg_mean = torch.mean(per_seq)
    clipfrac = masked_mean(torch.gt(surr2, surr1).float(), eos_mask)
    kl_loss = torch.zeros_like(pg_mean)
    pg_loss = pg_mean - entropy_coeff * entropy_loss
    return pg_loss, clipfrac, ppo_kl, kl_loss, entropy_loss


def logprob_computer(output, batch, skip_entropy=True, **kwargs):
    """``logprob_computer.py:94-145`` at context-parallel size 1 (the CP all-gather is the
    identity): packed ``[1,T,V]`` logits or padded ``[B,S,V]`` logits -> ``[B,L]``."""
    labels = batch["labels"]
    log_probs = vocab.compute_log_probs(output, labels)
    if kwargs.get("use_remove_padding", False):
        seqlens = kwargs.get("seqlens_in_batch")
        cu = kwargs.get("cu_seqlens_padded")
        width = batch["responses"].shape[-1]

        def unpack(x):
            return packing.postprocess_packed_seqs(x, seqlens, cu, width,
                                                   prompt_length=batch["prompt_length"])
    else:
        window = packing.response_window(batch["prompt_length"], batch["response_length"])

        def unpack(x):
            return packing.truncate_prompt_and_pad(batch["responses"], x, window)

    log_probs = unpack(log_probs)
    if skip_entropy:
        entropy = torch.zeros_like(log_probs)
    else:
        entropy = unpack(vocab.vocab_parallel_entropy(output))
    return log_probs, entropy


def _finish(pg_loss, clipfrac, ppo_kl, kl_loss, entropy_loss, batch, forward_only, kwargs):
    """``grpo_actor_loss_func.py:72-98``: dynamic-batch rescale, then the five stats with
    ``abs`` on the policy loss, one ``.item()`` each."""
    if kwargs.get("use_dynamic_bsz", False) and not forward_only:
        policy_loss = pg_loss * (batch["responses"].size(0) / kwargs.get("actual_micro_batch_size"))
    else:
        policy_loss = pg_loss
    stats = {
        "actor/pg_loss": abs(pg_loss.detach().item()),
        "actor/pg_clipfrac": clipfrac.detach().item(),
        "actor/ppo_kl": ppo_kl.detach().item(),
        "actor/kl_loss": kl_loss.detach().item(),
        "actor/entropy": entropy_loss.detach().item(),
    }
    return policy_loss, stats


def grpo_compute_loss(output, batch, meta, forward_only=False, **kwargs):
    """``grpo_actor_loss_func.py:43-98``; ``meta`` holds clip_ratio, kl_coef, kl_penalty,
    entropy_coeff.  ``batch['response_mask']`` is ignored, as in the reference."""
    if forward_only:
        return logprob_computer(output, batch, True, **kwargs)[0]
    entropy_coeff = meta.get("entropy_coeff", 0.0)
    log_probs, entropy = logprob_computer(output, batch, entropy_coeff == 0, **kwargs)
    if "responses" not in batch:
        raise ValueError("The responses is None")
    mask = packing.generate_mask(batch["responses"], batch["response_length"])
    out = grpo_policy_loss(batch.get("old_log_prob"), log_probs, batch.get("ref_log_prob"),
                           batch.get("advantages"), entropy, mask, meta.get("clip_ratio", 0.2),
                           meta["kl_coef"], meta["kl_penalty"], entropy_coeff)
    return _finish(*out, batch, forward_only, kwargs)


def dapo_compute_loss(output, batch, meta, forward_only=False, **kwargs):
    """``dapo_actor_loss_func.py:47-102``."""
    if forward_only:
        return logprob_computer(output, batch, True, **kwargs)[0]
    entropy_coeff = meta.get("entropy_coeff", 0.0)
    log_probs, entropy = logprob_computer(output, batch, entropy_coeff == 0, **kwargs)
    if "responses" not in batch:
        raise ValueError("The responses is None")
    mask = batch["response_mask"] if "response_mask" in batch else \
        packing.generate_mask(batch["responses"], batch["response_length"])
    clip = meta.get("clip_ratio", 0.2)
    if meta.get("clip_higher_enable", False):
        lo, hi = meta["clip_ratio_low"], meta["clip_ratio_high"]
    else:
        lo = hi = clip
    out = dapo_policy_loss(batch.get("old_log_prob"), log_probs, entropy, entropy_coeff,
                           batch.get("advantages"), mask, lo, hi, meta["token_level_loss"])
    return _finish(*out, batch, forward_only, kwargs)


def ppo_compute_loss(output, batch, meta, forward_only=False, **kwargs):
    """``ppo_actor_loss_func.py:39-89``: four statistics, no ``actor/kl_loss``."""
    if forward_only:
        return logprob_computer(output, batch, True, **kwargs)[0]
    entropy_coeff = meta.get("entropy_coeff", 0.0)
    log_probs, entropy = logprob_computer(output, batch, entropy_coeff == 0, **kwargs)
    if "responses" not in batch:
        raise ValueError("The responses is None")
    mask = packing.generate_mask(batch["responses"], batch["response_length"])
    pg_loss, clipfrac, ppo_kl, ent = ppo_policy_loss(batch.get("old_log_prob"), log_probs, batch.get("advantages"),
                                                     mask, meta.get("clip_ratio", 0.2), entropy, entropy_coeff)
    policy_loss, stats = _finish(pg_loss, clipfrac, ppo_kl, torch.zeros(()), ent, batch, forward_only, kwargs)
    del stats["actor/kl_loss"]
    return policy_loss, stats


def value_loss(vpreds, returns, values, response_mask, cliprange_value):
    """``critic_loss_func.py:82-111``."""
    vpreds = vpreds.squeeze()
    vpredclipped = torch.clamp(vpreds, values - cliprange_value, values + cliprange_value)
    vf_losses1 = (vpreds - returns) ** 2
    vf_losses2 = (vpredclipped - returns) ** 2
    vf_loss = 0.5 * masked_mean(torch.max(vf_losses1, vf_losses2), response_mask)
    vf_clipfrac = masked_mean(torch.gt(vf_losses2, vf_losses1).float(), response_mask)
    return vf_loss, vf_clipfrac


def critic_compute_loss(output, batch, cliprange_value=0.5, forward_only=False, **kwargs):
    """``critic_loss_func.py:37-80``: ``output`` is the value head's ``[B, S, 1]`` (or packed
    ``[1, T, 1]``); the response window is cut with ``truncate_middle_and_pad``."""
    if kwargs.get("use_remove_padding", False):
        output = packing.postprocess_packed_seqs(output, kwargs.get("seqlens_in_batch"),
                                                 kwargs.get("cu_seqlens_padded"), kwargs.get("seq_len"))
    if "responses" not in batch:
        raise ValueError("The responses is None")
    truncate_lengths = torch.cat([batch["prompt_length"], batch["prompt_length"] + batch["response_length"]],
                                 dim=1) - 1
    vpreds = packing.truncate_middle_and_pad(batch["responses"], output, truncate_lengths)
    if forward_only:
        return vpreds
    response_mask = packing.generate_mask(batch["responses"], batch["response_length"])
    vf_loss, vf_clipfrac = value_loss(vpreds, batch.get("returns"), batch.get("values"), response_mask,
                                      cliprange_value)
    if kwargs.get("use_dynamic_bsz", False) and not forward_only:
        loss = vf_loss * (batch["responses"].size(0) / kwargs.get("actual_micro_batch_size"))
    else:
        loss = vf_loss
    stats = {"critic/vf_loss": abs(vf_loss.detach().item()), "critic/vf_clipfrac": vf_clipfrac.detach().item()}
    return loss, stats

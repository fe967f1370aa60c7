"""PPO's value side: KL-penalised token rewards, GAE, masked whitening and the critic loss.

Host-side mirror of ``AdaptiveKLController``, the arithmetic inside ``apply_kl_penalty`` and
``compute_gae_advantage_return`` (``mindspeed_rl/trainer/utils/compute_utils.py:33-48,80-97,107-149``),
``masked_var`` / ``masked_whiten`` (``mindspeed_rl/utils/torch_functional.py:62-106``) and
``CriticLossFunc`` (``mindspeed_rl/models/loss/critic_loss_func.py``), with the reference's names,
signatures and error behaviour; the arithmetic runs in the kernels of ``csrc/value_path.hip``.
"""
from typing import Dict, Tuple

import numpy as np
import torch

from . import _lib
from .loss import BaseLossFunc, LossFuncFactory, _dynamic_scale, _mask_args
from .packing import postprocess_packed_seqs, truncate_middle_and_pad


class AdaptiveKLController:
    """Reference: ``trainer/utils/compute_utils.py:33-48``."""

    def __init__(self, init_kl_coef, target_kl, horizon):
        self.value = init_kl_coef
        self.target = target_kl
        self.horizon = horizon

    def update(self, current_kl, n_steps):
        proportional_error = np.clip(current_kl / self.target - 1, -0.2, 0.2)
        mult = 1 + proportional_error * n_steps / self.horizon
        self.value *= mult


def _f32(t, dev):
    return t.detach().to(device=dev, dtype=torch.float32).contiguous()


def _lengths(response_length, dev):
    lens = response_length
    if lens.dtype not in (torch.int32, torch.int64):
        lens = lens.to(torch.int64)
    return lens.to(dev).reshape(-1).contiguous()


def kl_token_level_rewards(old_log_prob, ref_log_prob, response_length, rm_scores, beta, penalty="kl"):
    """The arithmetic of ``apply_kl_penalty`` (``compute_utils.py:80-97``) for one padded batch:
    ``(token_level_rewards [B, L], current_kl)`` where the reward of sample ``i`` is its score at the
    last response token minus ``beta`` times the masked KL penalty, and ``current_kl`` (a python
    float, the value handed to ``kl_ctrl.update``) is the batch mean of the per-sample masked means."""
    if penalty not in _lib.KL_BY_NAME:
        raise NotImplementedError
    dev = _lib.require_device(old_log_prob, ref_log_prob)
    old, ref = _f32(old_log_prob, dev), _f32(ref_log_prob, dev)
    batch, width = old.shape
    lens = _lengths(response_length, dev)
    scores = _f32(torch.as_tensor(rm_scores), dev).reshape(-1)
    if lens.numel() != batch or scores.numel() != batch:
        raise ValueError("response_length and rm_scores need one entry per sample")
    rewards = torch.empty_like(old)
    row_kl = torch.empty(batch, dtype=torch.float32, device=dev)
    _lib.call("mrl_kl_token_rewards", _lib.ptr(old), _lib.ptr(ref), _lib.ptr(lens), _lib.dtype_code(lens),
              _lib.ptr(scores), batch, width, _lib.KL_BY_NAME[penalty], float(beta), _lib.ptr(rewards),
              _lib.ptr(row_kl), _lib.stream(dev))
    return rewards, torch.mean(row_kl, dim=0).item()


def _whiten(values, mask, shift_mean):
    dev = _lib.require_device(values, mask)
    x = _f32(values, dev)
    m, _ = _mask_args(mask.expand_as(values) if mask.shape != values.shape else mask, None, dev)
    out = torch.empty_like(x)
    info = torch.empty(3, dtype=torch.float64, device=dev)
    _lib.call("mrl_masked_whiten", _lib.ptr(x), _lib.ptr(m), _lib.dtype_code(m), x.numel(), 1 if shift_mean else 0,
              _lib.ptr(out), _lib.ptr(info), _lib.stream(dev))
    return out, info


def masked_var(values, mask, unbiased=True):
    """Reference: ``torch_functional.py:62-87``; a 0-d fp32 tensor.  ``unbiased=False`` undoes the
    Bessel correction the kernel applies."""
    _, info = _whiten(values, mask, True)
    count, _, var = info.cpu().tolist()
    if unbiased and count == 0:
        raise ValueError("At least one element in the mask has to be 1.")
    if not unbiased and count > 1:
        var = var * (count - 1) / count
    return torch.tensor(var, dtype=torch.float32, device=values.device)


def masked_whiten(values, mask, shift_mean=True):
    """Reference: ``torch_functional.py:90-106``."""
    out, info = _whiten(values, mask, shift_mean)
    if info[0].item() == 0:
        raise ValueError("At least one element in the mask has to be 1.")
    return out.view(values.shape)


def compute_gae_advantage_return(token_level_rewards, values, eos_mask, gamma, lam):
    """Reference: ``compute_utils.py:107-149``.  The reverse scan runs over the full width (the mask
    only enters the whitening) with the reference's fp32 operation order, so ``returns`` and the
    advantages before whitening are bit-identical to the torch loop."""
    dev = _lib.require_device(token_level_rewards, values, eos_mask)
    rewards, vals = _f32(token_level_rewards, dev), _f32(values, dev)
    if rewards.dim() != 2 or rewards.shape != vals.shape:
        raise ValueError("token_level_rewards and values must both be [batch, response_length]")
    batch, width = rewards.shape
    adv = torch.empty_like(rewards)
    ret = torch.empty_like(rewards)
    # `gamma * lam` as python evaluates it inside the reference's `gamma * lam * lastgaelam`: in double
    # for python floats (the config's values), in the tensors' own precision for 0-dim tensors
    _lib.call("mrl_gae_scan", _lib.ptr(rewards), _lib.ptr(vals), batch, width, float(gamma), float(gamma * lam),
              _lib.ptr(adv), _lib.ptr(ret), _lib.stream(dev))
    return masked_whiten(adv, eos_mask), ret


class _ValueLoss(torch.autograd.Function):
    """vpreds [B, L] -> (scaled loss, out[4]) through mrl_value_loss_fwd / _bwd."""

    @staticmethod
    def forward(ctx, vpreds, returns, values, mask, lens, clip, loss_scale):
        dev = _lib.require_device(vpreds, returns, values, mask, lens)
        vp = vpreds.to(torch.float32).contiguous()
        ret, val = _f32(returns, dev), _f32(values, dev)
        batch, width = vp.shape
        out = torch.empty(4, dtype=torch.float32, device=dev)
        args = (_lib.ptr(vp), _lib.ptr(ret), _lib.ptr(val), _lib.ptr(mask),
                _lib.dtype_code(mask) if mask is not None else _lib.F32, _lib.ptr(lens),
                _lib.dtype_code(lens) if lens is not None else _lib.I32, batch, width, float(clip), float(loss_scale))
        _lib.call("mrl_value_loss_fwd", *args, _lib.ptr(out), _lib.stream(dev))
        ctx.save_for_backward(vp, ret, val, mask, lens, out)
        ctx.scalars = (float(clip), float(loss_scale))
        ctx.in_dtype = vpreds.dtype
        ctx.mark_non_differentiable(out)
        return out[0].clone(), out

    @staticmethod
    def backward(ctx, g_loss, _g_out):
        vp, ret, val, mask, lens, out = ctx.saved_tensors
        dev = vp.device
        batch, width = vp.shape
        upstream = g_loss.to(torch.float32).reshape(1).contiguous()
        g = torch.empty_like(vp)
        _lib.call("mrl_value_loss_bwd", _lib.ptr(vp), _lib.ptr(ret), _lib.ptr(val), _lib.ptr(mask),
                  _lib.dtype_code(mask) if mask is not None else _lib.F32, _lib.ptr(lens),
                  _lib.dtype_code(lens) if lens is not None else _lib.I32, batch, width, *ctx.scalars, _lib.ptr(out),
                  _lib.ptr(upstream), _lib.ptr(g), _lib.stream(dev))
        return g.to(ctx.in_dtype), None, None, None, None, None, None


def value_loss(vpreds, returns, values, response_mask=None, response_length=None, *, cliprange_value,
               loss_scale=1.0):
    """Clipped value loss: ``(loss_scale * vf_loss, out)`` with ``out = [scaled loss, vf_loss,
    vf_clipfrac, sum(mask)]`` on the device; differentiable with respect to ``vpreds`` ``[B, L]``."""
    dev = _lib.require_device(vpreds)
    if vpreds.dim() != 2:
        raise ValueError("vpreds must be [batch, response_length]")
    mask, lens = _mask_args(response_mask, response_length, dev)
    return _ValueLoss.apply(vpreds, returns, values, mask, lens, cliprange_value, loss_scale)


@LossFuncFactory.register_loss("ray_ppo", "critic")
class CriticLossFunc(BaseLossFunc):
    """Reference: ``critic_loss_func.py:14-111``."""

    def __init__(self):
        super(CriticLossFunc, self).__init__()
        self.cliprange_value = 0.5

    def add_loss_meta_info(self, meta_info: Dict):
        if meta_info is None:
            return
        if "cliprange_value" in meta_info.keys():
            self.cliprange_value = float(meta_info["cliprange_value"])

    @staticmethod
    def _get_policy_loss_input(batch: Dict[str, torch.Tensor]):
        if "responses" not in batch:
            raise ValueError("The responses is None")
        values = batch["values"] if "values" in batch else None
        returns = batch["returns"] if "returns" in batch else None
        response_length = batch["response_length"]
        from .packing import generate_mask
        response_mask = generate_mask(batch["responses"], response_length)
        return response_mask, values, returns, response_length

    @staticmethod
    def _get_compute_vpreds(output: torch.Tensor, batch: Dict[str, torch.Tensor]):
        if "responses" not in batch:
            raise ValueError("The responses is None")
        responses = batch["responses"]
        truncate_lengths = torch.cat([batch["prompt_length"], batch["prompt_length"] + batch["response_length"]],
                                     dim=1) - 1
        return truncate_middle_and_pad(responses, output, truncate_lengths)

    def compute_loss(self, output: torch.Tensor, batch: Dict[str, torch.Tensor], forward_only=False,
                     non_loss_data=True, **kwargs) -> Tuple[torch.Tensor, Dict]:
        if kwargs.get("use_remove_padding", False):
            output = postprocess_packed_seqs(output=output, seqlens_in_batch=kwargs.get("seqlens_in_batch", None),
                                             cu_seqlens_padded=kwargs.get("cu_seqlens_padded", None),
                                             seq_len=kwargs.get("seq_len", None))
        vpreds = self._get_compute_vpreds(output, batch)
        if forward_only:
            return vpreds
        if "responses" not in batch:
            raise ValueError("The responses is None")
        scale = _dynamic_scale(batch, forward_only, kwargs)
        # the mask is (j < response_length), evaluated inside the kernel
        loss, out = value_loss(vpreds.reshape(vpreds.shape[0], vpreds.shape[1]), batch.get("returns"),
                               batch.get("values"), None, batch["response_length"],
                               cliprange_value=self.cliprange_value, loss_scale=scale)
        host = out.detach().cpu().tolist()      # one device-to-host copy for both statistics
        stats = {"critic/vf_loss": abs(host[1]), "critic/vf_clipfrac": host[2]}
        return loss, stats

    @staticmethod
    def _compute_value_loss(vpreds, returns, values, response_mask, cliprange_value):
        """``(vf_loss, vf_clipfrac)`` as 0-d tensors (``critic_loss_func.py:82-111``)."""
        vp = vpreds.squeeze()
        if vp.dim() == 1:
            vp = vp.unsqueeze(0)
        loss, out = value_loss(vp, returns.reshape(vp.shape), values.reshape(vp.shape),
                               response_mask.reshape(vp.shape), None, cliprange_value=cliprange_value)
        return loss, out[2]

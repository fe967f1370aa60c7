"""Masked reductions with the reference's semantics.

Host-side mirror of ``masked_sum`` / ``masked_mean`` of
``mindspeed_rl/utils/torch_functional.py:38-59`` for callers that use them stand-alone; the
fused policy-loss kernel has the same reductions built in and does not go through these.
"""
import torch


def masked_sum(values, mask, axis=None):
    """Values outside the mask are replaced by 0 before the mask multiplies them, so NaN / Inf
    there cannot leak into the sum; non-binary mask weights still count."""
    kept = torch.where(mask.bool(), values, 0.0)
    return (kept * mask).sum(axis=axis)


def masked_mean(values, mask, axis=None, epsilon=1e-8):
    return masked_sum(values, mask, axis) / (mask.sum(axis=axis) + epsilon)


def clip_by_value(x, tensor_min, tensor_max):
    """Reference: ``torch_functional.py:22-35``: ``max(min(x, tensor_max), tensor_min)``."""
    return torch.max(torch.min(x, tensor_max), tensor_min)

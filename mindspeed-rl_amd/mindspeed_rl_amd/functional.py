"""Masked reductions with the reference's semantics, and the multimodal switch.

Host-side mirror of ``masked_sum`` / ``masked_mean`` of
``mindspeed_rl/utils/torch_functional.py:38-59`` for callers that use them stand-alone; the
fused policy-loss kernel has the same reductions built in and does not go through these.
"""
import ast
import os

import torch


def is_multimodal():
    """Reference: ``utils/utils.py:719-720``: the process-wide switch is the environment variable
    IS_MULTIMODAL, read as a python literal at every call (``"True"`` / ``"False"``, default False).
    The loss objects choose their log-prob strategy by it when they are constructed and
    ``rearrange_micro_batches`` its partitioner when it is called, as in the reference."""
    return ast.literal_eval(os.getenv("IS_MULTIMODAL", "False"))


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

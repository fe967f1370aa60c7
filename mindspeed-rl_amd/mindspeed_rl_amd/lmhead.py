"""Fused lm_head + log-prob: hidden states and the vocabulary projection weight go in, per-token
log-prob / entropy / logsumexp come out, and the ``[T, V]`` logits are never written to memory.

The reference has no such function: ``GPTModel.output_layer`` materialises the logits and
``compute_log_probs`` (``mindspeed_rl/utils/compute.py:29-51``) reads them back.  This is the
forward-only form, which serves ``compute_log_prob`` / ``compute_ref_log_prob`` (two of the three
vocabulary sweeps of a GRPO iteration).
"""
import torch

from . import _lib

# (name, start, end, rows) appended per call when set to a list, like vocab_ops.kernel_events
kernel_events = None


def lmhead_logprob(hidden, weight, labels, inv_temperature=1.0, want_entropy=True):
    """``hidden`` ``[..., H]`` bf16, ``weight`` ``[V, H]`` bf16 (``nn.Linear`` layout), ``labels``
    ``[...]`` int32/int64 -> ``(logp, entropy, lse)`` fp32 shaped like ``labels`` (entropy is zeros
    if not wanted).  No autograd: use it under ``torch.no_grad()`` for old / reference log-probs."""
    dev = _lib.require_device(hidden, weight, labels)
    if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise TypeError("hidden and weight must be bfloat16")
    hdim = hidden.shape[-1]
    if weight.dim() != 2 or weight.shape[1] != hdim:
        raise ValueError("weight must have shape (vocab, hidden_dim)")
    lead = hidden.shape[:-1]
    if tuple(labels.shape) != tuple(lead):
        raise ValueError("labels shape %s does not match hidden leading shape %s" % (tuple(labels.shape), tuple(lead)))
    h = hidden.detach().reshape(-1, hdim).contiguous()
    w = weight.detach().contiguous()
    lab = labels.reshape(-1)
    if lab.dtype not in (torch.int32, torch.int64):
        lab = lab.to(torch.int64)
    lab = lab.contiguous()
    n_tokens, vocab = h.shape[0], w.shape[0]
    logp = torch.empty(n_tokens, dtype=torch.float32, device=dev)
    lse = torch.empty(n_tokens, dtype=torch.float32, device=dev)
    ent = torch.empty(n_tokens, dtype=torch.float32, device=dev) if want_entropy else None
    ws_bytes = _lib.load().mrl_lmhead_workspace_bytes(n_tokens, vocab)
    workspace = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    args = (_lib.ptr(h), _lib.ptr(w), n_tokens, vocab, hdim, _lib.ptr(lab), _lib.dtype_code(lab),
            float(inv_temperature), _lib.ptr(logp), _lib.ptr(ent), _lib.ptr(lse), _lib.ptr(workspace), ws_bytes,
            _lib.stream(dev))
    if kernel_events is None:
        _lib.call("mrl_lmhead_logprob_fwd", *args)
    else:
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        stream = torch.cuda.current_stream(dev)
        start.record(stream)
        _lib.call("mrl_lmhead_logprob_fwd", *args)
        end.record(stream)
        kernel_events.append(("mrl_lmhead_logprob_fwd", start, end, n_tokens))
    ent_out = ent.view(lead) if want_entropy else torch.zeros(lead, dtype=torch.float32, device=dev)
    return logp.view(lead), ent_out, lse.view(lead)

"""Per-token log-probability, entropy and KL penalties over the vocabulary.

Host-side mirror of ``mindspeed_rl/utils/compute.py`` of the reference (same function names,
argument order and error behaviour), backed by the one-pass HIP kernels
``mrl_vocab_logprob_fwd`` / ``mrl_vocab_logprob_bwd``.
"""
import torch

from . import _lib

_ParallelState = None
_VocabParallel = None

# Optional kernel timing: set to a list and every vocabulary sweep appends
# (name, start_event, end_event, rows) with HIP events recorded on the launch stream.
kernel_events = None


def _timed_call(name, rows, dev, *args):
    if kernel_events is None:
        _lib.call(name, *args)
        return
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    stream = torch.cuda.current_stream(dev)
    start.record(stream)
    _lib.call(name, *args)
    end.record(stream)
    kernel_events.append((name, start, end, rows))


def set_parallel_state(obj):
    """Reference: ``utils/compute.py:9-11``.  Kept for call-compatibility; unused at tp = cp = 1."""
    global _ParallelState
    _ParallelState = obj


def get_parallel_state():
    return _ParallelState


def set_vocab_parallel(obj):
    """Reference: ``utils/compute.py:19-21``.  A caller may still inject its own cross-entropy;
    when none is set (or it is this module's :func:`vocab_parallel_cross_entropy`) the fused
    kernel is used directly."""
    global _VocabParallel
    _VocabParallel = obj


def get_vocab_parallel():
    return _VocabParallel


class _VocabLogprobEntropy(torch.autograd.Function):
    """(logits[..., V], labels[...]) -> (logp[...], entropy[...]) in one sweep; the backward
    recomputes the softmax from the saved logsumexp (one read of logits, one write of dlogits)."""

    @staticmethod
    def forward(ctx, logits, labels, inv_temperature, want_entropy, row_active, grad_inplace):
        dev = _lib.require_device(logits, labels, row_active)
        vocab = logits.shape[-1]
        if logits.stride(-1) != 1:
            logits = logits.contiguous()
        lead = logits.shape[:-1]
        if tuple(labels.shape) != tuple(lead):
            raise ValueError("labels shape %s does not match logits leading shape %s"
                             % (tuple(labels.shape), tuple(lead)))
        flat = logits.reshape(-1, vocab) if logits.dim() != 2 else logits
        if flat.stride(-1) != 1 or (flat.shape[0] > 1 and flat.stride(0) < vocab):
            flat = flat.contiguous()
        n_rows = flat.shape[0]
        row_stride = flat.stride(0) if n_rows > 1 else vocab
        lab = labels.reshape(-1)
        if lab.dtype not in (torch.int32, torch.int64):
            lab = lab.to(torch.int64)
        lab = lab.contiguous()
        act = None
        if row_active is not None:
            act = row_active.reshape(-1).to(torch.uint8).contiguous()
            if act.numel() != n_rows:
                raise ValueError("row_active must have one entry per row")
        logp = torch.empty(n_rows, dtype=torch.float32, device=dev)
        lse = torch.empty(n_rows, dtype=torch.float32, device=dev)
        ent = torch.empty(n_rows, dtype=torch.float32, device=dev) if want_entropy else None
        _timed_call("mrl_vocab_logprob_fwd", n_rows, dev, _lib.ptr(flat), _lib.dtype_code(flat), n_rows, vocab, row_stride,
                  _lib.ptr(lab), _lib.dtype_code(lab), _lib.ptr(act), float(inv_temperature), _lib.ptr(logp),
                  _lib.ptr(ent), _lib.ptr(lse), _lib.stream(dev))
        ctx.save_for_backward(flat, lab, lse, ent if want_entropy else None)
        ctx.meta = (tuple(logits.shape), float(inv_temperature), row_stride, bool(grad_inplace))
        lse_out = lse.view(lead)
        ent_out = ent.view(lead) if want_entropy else torch.zeros(lead, dtype=torch.float32, device=dev)
        if want_entropy:
            ctx.mark_non_differentiable(lse_out)
        else:
            ctx.mark_non_differentiable(lse_out, ent_out)
        return logp.view(lead), ent_out, lse_out

    @staticmethod
    def backward(ctx, g_logp, g_entropy, _g_lse):
        flat, lab, lse, ent = ctx.saved_tensors
        shape, inv_t, row_stride, inplace = ctx.meta
        dev = flat.device
        n_rows, vocab = flat.shape
        g_lp = None if g_logp is None else g_logp.reshape(-1).to(torch.float32).contiguous()
        g_h = None
        if ent is not None and g_entropy is not None:
            g_h = g_entropy.reshape(-1).to(torch.float32).contiguous()
        if inplace:
            dlogits, d_stride = flat, row_stride
        else:
            dlogits = torch.empty((n_rows, vocab), dtype=flat.dtype, device=dev)
            d_stride = vocab
        _timed_call("mrl_vocab_logprob_bwd", n_rows, dev, _lib.ptr(flat), _lib.dtype_code(flat), n_rows, vocab, row_stride,
                  _lib.ptr(lab), _lib.dtype_code(lab), inv_t, _lib.ptr(lse), _lib.ptr(ent), _lib.ptr(g_lp),
                  _lib.ptr(g_h), _lib.ptr(dlogits), _lib.dtype_code(dlogits), d_stride, _lib.stream(dev))
        return dlogits.view(shape), None, None, None, None, None


def vocab_logprob_entropy(logits, labels, inv_temperature=1.0, want_entropy=True, row_active=None,
                          grad_inplace=False):
    """Fused sweep: returns ``(logp, entropy, lse)`` as fp32 tensors shaped like ``labels``.

    ``logits`` (fp32 / bf16 / fp16, ``[..., V]``) is only read.  ``inv_temperature`` folds the
    caller's ``logits / temperature`` into the sweep.  ``row_active`` (bool/uint8, optional)
    skips rows whose result is not needed.  ``grad_inplace=True`` lets the backward overwrite the
    logits storage with dlogits (saves one ``[T, V]`` buffer; the caller must not read the logits
    afterwards).  With ``want_entropy=False`` the entropy output is zeros.
    """
    return _VocabLogprobEntropy.apply(logits, labels, inv_temperature, want_entropy, row_active, grad_inplace)


# ------------------------------------------------------------------- one rank's share of a sharded vocabulary
def vocab_shard_stats(logits_shard, labels, vocab_start, inv_temperature=1.0, row_active=None):
    """One tensor-parallel rank's share of the forward sweep: ``logits_shard`` ``[..., V/tp]`` holds
    the vocabulary entries ``[vocab_start, vocab_start + V/tp)`` of every row, ``labels`` the global
    token ids.  Returns fp32 ``[..., 3]`` = (logsumexp over the shard, label logit if the label lies
    in the shard else 0, softmax-weighted mean logit of the shard): 12 bytes per token, which is all
    the ranks have to exchange (Megatron's ``vocab_parallel_cross_entropy`` and the reference's
    ``_VocabParallelEntropy.forward``, ``utils/compute.py:56-73``, all-reduce the row maximum, the
    predicted logit, the exponential sum and the weighted sum one after the other).  No autograd."""
    width = logits_shard.shape[-1]
    local = labels.to(torch.int64) - int(vocab_start)
    own = (local >= 0) & (local < width)
    with torch.no_grad():
        logp, ent, lse = vocab_logprob_entropy(logits_shard.detach(), local, inv_temperature=inv_temperature,
                                               want_entropy=True, row_active=row_active)
    label_logit = torch.where(own, logp + lse, torch.zeros_like(logp))
    if row_active is not None:
        lse = torch.where(row_active.reshape(lse.shape) != 0, lse, torch.full_like(lse, float("-inf")))
    return torch.stack([lse, label_logit, lse - ent], dim=-1)


def merge_vocab_shard_stats(stats):
    """``stats`` ``[tp, ..., 3]``: every rank's :func:`vocab_shard_stats` (what an all-gather
    delivers).  Returns ``(logp, entropy, lse)`` of the full vocabulary, fp32.  Rows that no rank
    scored (``row_active`` 0 everywhere) return 0."""
    lse_s, label_s, mean_s = stats.unbind(-1)
    lse = torch.logsumexp(lse_s, dim=0)
    dead = torch.isinf(lse) & (lse < 0)
    lse = torch.where(dead, torch.zeros_like(lse), lse)
    share = torch.exp(lse_s - lse.unsqueeze(0))                    # each shard's probability mass
    share = torch.where(dead.unsqueeze(0), torch.zeros_like(share), share)
    mean_logit = (share * torch.where(share > 0, mean_s, torch.zeros_like(mean_s))).sum(0)
    logp = torch.where(dead, torch.zeros_like(lse), label_s.sum(0) - lse)
    return logp, lse - mean_logit, lse


def vocab_shard_backward(logits_shard, labels, vocab_start, lse, entropy, g_logp, g_entropy=None, inv_temperature=1.0,
                         grad_inplace=False):
    """One rank's share of the backward sweep: dlogits of the shard from the MERGED ``lse`` and
    ``entropy`` (Megatron's cross-entropy backward and ``_VocabParallelEntropy.backward``,
    ``utils/compute.py:76-85``, on the rank's vocabulary range).  One read of the shard, one write."""
    dev = _lib.require_device(logits_shard, labels, lse, entropy, g_logp, g_entropy)
    width = logits_shard.shape[-1]
    flat = logits_shard.detach().reshape(-1, width)
    if flat.stride(-1) != 1 or (flat.shape[0] > 1 and flat.stride(0) < width):
        flat = flat.contiguous()
    n_rows = flat.shape[0]
    row_stride = flat.stride(0) if n_rows > 1 else width
    local = (labels.to(torch.int64) - int(vocab_start)).reshape(-1).contiguous()

    def f32(t):
        return None if t is None else t.reshape(-1).to(torch.float32).contiguous()

    lse_f, ent_f, g_lp, g_h = f32(lse), f32(entropy), f32(g_logp), f32(g_entropy)
    if grad_inplace:
        dlogits, d_stride = flat, row_stride
    else:
        dlogits, d_stride = torch.empty((n_rows, width), dtype=flat.dtype, device=dev), width
    _timed_call("mrl_vocab_logprob_bwd", n_rows, dev, _lib.ptr(flat), _lib.dtype_code(flat), n_rows, width, row_stride,
                _lib.ptr(local), _lib.dtype_code(local), float(inv_temperature), _lib.ptr(lse_f), _lib.ptr(ent_f),
                _lib.ptr(g_lp), _lib.ptr(g_h), _lib.ptr(dlogits), _lib.dtype_code(dlogits), d_stride, _lib.stream(dev))
    return dlogits.view(logits_shard.shape)


def vocab_parallel_cross_entropy(vocab_parallel_logits, target, label_smoothing=0.0):
    """Drop-in for Megatron's ``vocab_parallel_cross_entropy`` at tp = 1 (the function the
    reference injects through ``set_vocab_parallel``, ``workers/base_worker.py:279-284``):
    per-token cross entropy in fp32, differentiable w.r.t. the logits.  Unlike Megatron's it does
    not clobber its logits argument."""
    if label_smoothing != 0.0:
        raise NotImplementedError("label_smoothing is not used on this path")
    logp, _, _ = vocab_logprob_entropy(vocab_parallel_logits, target, want_entropy=False)
    return -logp


def compute_log_probs(logits, labels, **kwargs):
    """Reference: ``utils/compute.py:29-51``.  The reference clones both inputs because Megatron's
    cross entropy mutates them; the kernel only reads them, so no copy is made."""
    injected = get_vocab_parallel()
    if injected is not None and injected is not vocab_parallel_cross_entropy:
        return -injected(vocab_parallel_logits=logits.clone(), target=labels.clone())
    logp, _, _ = vocab_logprob_entropy(logits, labels, want_entropy=False)
    return logp


def vocab_parallel_entropy(vocab_parallel_logits):
    """Reference: ``utils/compute.py:88-97``: ``(total_nnz, V) -> (total_nnz,)`` entropy of the
    softmax, differentiable.  Computed in fp32 whatever the logits dtype."""
    lead = vocab_parallel_logits.shape[:-1]
    dummy = torch.zeros(lead, dtype=torch.int32, device=vocab_parallel_logits.device)
    _, ent, _ = vocab_logprob_entropy(vocab_parallel_logits, dummy, want_entropy=True)
    return ent


def compute_kl_penalty(logprob, ref_logprob, kl_penalty="low_var_kl"):
    """Reference: ``utils/compute.py:100-133``.  Stand-alone form for callers outside the fused
    loss (the loss kernel has these four penalties built in)."""
    if kl_penalty == "kl":
        return logprob - ref_logprob
    if kl_penalty == "abs":
        return (logprob - ref_logprob).abs()
    if kl_penalty == "mse":
        return 0.5 * (logprob - ref_logprob).square()
    if kl_penalty == "low_var_kl":
        delta = torch.clamp(ref_logprob - logprob, min=-20, max=20)
        return torch.clamp(torch.exp(delta) - delta - 1, min=-10, max=10)
    raise NotImplementedError

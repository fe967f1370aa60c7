"""Fused lm_head + log-prob: hidden states and the vocabulary projection weight go in, per-token
log-prob / entropy / logsumexp come out, and the ``[T, V]`` logits are never written to memory.

The reference has no such function: ``GPTModel.output_layer`` materialises the logits and
``compute_log_probs`` (``mindspeed_rl/utils/compute.py:29-51``) reads them back.  This is the
forward-only form, which serves ``compute_log_prob`` / ``compute_ref_log_prob`` (two of the three
vocabulary sweeps of a GRPO iteration).
"""
import torch

from . import _lib, vocab_ops

# (name, start, end, rows) appended per call when set to a list, like vocab_ops.kernel_events
kernel_events = None


def _timed(name, rows, dev, *args):
    """_lib.call with HIP events around it when kernel_events is a list."""
    if kernel_events is None:
        _lib.call(name, *args)
        return
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    stream = torch.cuda.current_stream(dev)
    start.record(stream)
    _lib.call(name, *args)
    end.record(stream)
    kernel_events.append((name, start, end, rows))


def lmhead_logprob(hidden, weight, labels, inv_temperature=1.0, want_entropy=True, row_active=None):
    """``hidden`` ``[..., H]`` bf16, ``weight`` ``[V, H]`` bf16 (``nn.Linear`` layout), ``labels``
    ``[...]`` int32/int64 -> ``(logp, entropy, lse)`` fp32 shaped like ``labels`` (entropy is zeros
    if not wanted).  No autograd: use it under ``torch.no_grad()`` for old / reference log-probs.
    ``row_active`` (bool / integer, shaped like ``labels``): only rows with a non-zero flag are
    projected and scored, the others return 0 in all three outputs (one host synchronisation reads
    the number of active rows)."""
    if row_active is not None:
        if tuple(row_active.shape) != tuple(labels.shape):
            raise ValueError("row_active must have the shape of labels")
        dev = _lib.require_device(hidden, weight, labels, row_active)
        live = torch.nonzero(row_active.reshape(-1) != 0).flatten()
        n_all = labels.numel()
        if live.numel() == 0:
            return tuple(torch.zeros(labels.shape, dtype=torch.float32, device=dev) for _ in range(3))
        res = lmhead_logprob(hidden.reshape(-1, hidden.shape[-1]).index_select(0, live), weight,
                             labels.reshape(-1).index_select(0, live), inv_temperature, want_entropy)
        outs = []
        for part in res:
            full = torch.zeros(n_all, dtype=torch.float32, device=dev)
            full.index_copy_(0, live, part)
            outs.append(full.view(labels.shape))
        return tuple(outs)
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


def _round_up(x, to):
    return (x + to - 1) // to * to


class _FusedLmHeadLoss(torch.autograd.Function):
    """(hidden, weight) -> (loss, out[8]) with dHidden and dWeight produced during the forward.

    The rows are processed in chunks: ``logits_c = hidden_c @ weight^T`` (``mrl_lmhead_logits``),
    the fused sweep turns the chunk into dlogits in place (one read, one write), then
    ``dHidden_c = dlogits_c @ weight`` and ``dWeight += dlogits_c^T @ hidden_c``
    (``mrl_lmhead_logprob_bwd``, fp32 accumulation across chunks in stream order).  All three
    products run on the hand-written bf16 MFMA kernels; only ``chunk_rows x V`` logits exist at any
    time."""

    @staticmethod
    def forward(ctx, hidden, weight, labels, batch, cfg):
        from .loss import _FusedOperands
        dev = _lib.require_device(hidden, weight, labels)
        hdim = hidden.shape[-1]
        h2d = hidden.detach().reshape(-1, hdim).contiguous()
        w = weight.detach().contiguous()
        n_rows, vocab = h2d.shape[0], w.shape[0]
        lab = labels.reshape(-1)
        if lab.dtype not in (torch.int32, torch.int64):
            lab = lab.to(torch.int64)
        lab = lab.contiguous()
        n_seq, width = batch["responses"].shape[0], batch["responses"].shape[-1]
        layout, padded_s = (0, 0) if cfg["packed"] else (1, hidden.shape[1])
        chunk_cap = max(1, min(int(cfg["chunk_rows"]), max(n_rows, 1)))
        ops = _FusedOperands(dev, batch, cfg, n_rows, n_seq, width, layout, padded_s, _lib.BF16, vocab, chunk_cap)
        want_ent = cfg["entropy_coeff"] != 0
        ent = torch.empty(max(n_rows, 1), dtype=torch.float32, device=dev) if want_ent else None
        stream = _lib.stream(dev)
        ops.prepare(stream)
        row_ops = ops.rows[:max(n_rows, 1) * 8]
        # Rows whose mask is zero (prompts, padding, masked tokens) add nothing to the loss, to dWeight or
        # to their own dHidden: when they are more than a twentieth of the rows, the live rows are gathered
        # and only they go through the products.  The row count sizes the products, so it is read back (one
        # host synchronisation per call; compact_rows=False avoids it).
        live = None
        if cfg["compact_rows"] and n_rows > 0:
            live = torch.nonzero(row_ops.view(n_rows, 8)[:, 3] != 0).flatten()
            if live.numel() * 20 > n_rows * 19:
                live = None
        all_rows, h_all = n_rows, h2d
        p_ops, p_terms = ops.p_ops, ops.p_terms
        if live is not None:
            n_rows = live.numel()
            h2d = h_all.index_select(0, live)
            lab = lab.index_select(0, live)
            row_ops = row_ops.view(all_rows, 8).index_select(0, live).reshape(-1)
            row_terms = torch.empty(max(n_rows, 1) * 8, dtype=torch.float32, device=dev)
            p_ops, p_terms = row_ops.data_ptr(), row_terms.data_ptr()
        chunk = max(1, min(chunk_cap, n_rows))
        # the chunk of logits: rows padded to whole k-steps of the dHidden product; the padding columns
        # are zeroed once and never written (they meet rows of the weight that read as zero)
        v_pad = _round_up(vocab, 64)
        if v_pad != vocab:
            logits = torch.zeros((chunk, v_pad), dtype=h2d.dtype, device=dev)
        else:
            logits = torch.empty((chunk, v_pad), dtype=h2d.dtype, device=dev)
        d_hidden = torch.empty_like(h2d)
        d_weight32 = torch.zeros((vocab, hdim), dtype=torch.float32, device=dev)
        esz = h2d.element_size()
        for c0 in range(0, n_rows, chunk):
            rows = min(n_rows, c0 + chunk) - c0
            h_c = h2d.data_ptr() + c0 * hdim * esz
            _timed("mrl_lmhead_logits", rows, dev, h_c, _lib.ptr(w), rows, vocab, hdim, _lib.ptr(logits), v_pad, stream)
            # the first sweep finds the workspace cleared by the prepare step, the others clear it themselves
            vocab_ops._timed_call(
                "mrl_fused_logprob_loss", rows, dev, _lib.ptr(logits), _lib.dtype_code(logits), rows, vocab, v_pad,
                lab.data_ptr() + c0 * lab.element_size(), _lib.dtype_code(lab), cfg["inv_temperature"],
                p_ops + c0 * 32, 0 if ops.old is None else 1, cfg["clip_lo"], cfg["clip_hi"], cfg["kl_penalty"],
                cfg["kl_coef"], cfg["entropy_coeff"], cfg["loss_scale"], _lib.ptr(ops.applied), _lib.ptr(logits), v_pad,
                None, (ent.data_ptr() + c0 * 4) if want_ent else None, p_terms + c0 * 32, ops.workspace,
                ops.ws_bytes, 1 if c0 == 0 else 0, stream)
            _timed("mrl_lmhead_logprob_bwd", rows, dev, h_c, _lib.ptr(w), _lib.ptr(logits), v_pad, rows, vocab, hdim,
                   d_hidden.data_ptr() + c0 * hdim * esz, _lib.ptr(d_weight32), stream)
        if live is not None:
            compact_dh = d_hidden
            d_hidden = torch.zeros_like(h_all)
            d_hidden.index_copy_(0, live, compact_dh)
            terms_all = ops.rows[all_rows * 8:all_rows * 16].zero_()
            terms_all.view(all_rows, 8).index_copy_(0, live, row_terms[:n_rows * 8].view(n_rows, 8))
        ops.reduce(stream)
        applied = ops.applied
        d_weight = d_weight32.to(w.dtype)
        ctx.save_for_backward(d_hidden, d_weight, applied)
        ctx.meta = (tuple(hidden.shape), cfg.get("scale_state"))
        ctx.handed_out = False
        ctx.mark_non_differentiable(ops.out)
        ctx.set_materialize_grads(False)
        return ops.loss, ops.out

    @staticmethod
    def backward(ctx, g_loss, _g_out):
        from .loss import _deliver_eager_grads
        if g_loss is None:
            return None, None, None, None, None
        d_hidden, d_weight, applied = ctx.saved_tensors
        shape, state = ctx.meta
        d_hidden, d_weight = _deliver_eager_grads(ctx, (d_hidden, d_weight), applied, state, g_loss)
        return d_hidden.view(shape), d_weight, None, None, None


def fused_lmhead_policy_loss(hidden, weight, batch, *, packed, seqlens=None, cu_seqlens=None, mask=None,
                             ref_log_prob=None, clip_low, clip_high, kl_penalty=None, kl_coef=0.0, entropy_coeff=0.0,
                             token_level_loss=True, loss_scale=1.0, inv_temperature=1.0, expected_upstream=None,
                             scale_state=None, chunk_rows=32768, compact_rows=True):
    """Policy loss straight from the hidden states: ``hidden`` is packed ``[1, T, H]`` (or padded
    ``[B, S, H]``) bf16, ``weight`` the ``[V, H]`` bf16 lm_head weight; ``batch`` as for
    :func:`mindspeed_rl_amd.fused_logprob_policy_loss` (``labels, responses, response_length,
    prompt_length, advantages``, optional ``old_log_prob``).  Returns ``(loss, out)``; ``backward()``
    yields dHidden and dWeight.  Full ``[T, V]`` logits are never materialised: at most
    ``chunk_rows x V`` exist at a time.  ``hidden_dim`` must be a multiple of 64, ``V`` of 8 and at
    most ``mrl_fused_max_vocab`` (311 296); fp16 operands are not taken.  With ``compact_rows`` (default) rows without a live response token
    skip the GEMMs when they are more than 5 % of all rows; finding them costs one host
    synchronisation per call."""
    if kl_penalty is None:
        kl_code = _lib.KL_NONE
    elif kl_penalty in _lib.KL_BY_NAME:
        kl_code = _lib.KL_BY_NAME[kl_penalty]
    else:
        raise NotImplementedError
    if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise TypeError("hidden and weight must both be bfloat16")
    if hidden.shape[-1] % 64 != 0 or weight.shape[0] % 8 != 0:
        raise ValueError("hidden_dim must be a multiple of 64 and the vocabulary of 8")
    cfg = dict(packed=bool(packed), seqlens=seqlens, cu=cu_seqlens, mask=mask, ref_log_prob=ref_log_prob,
               clip_lo=float(1.0 - clip_low), clip_hi=float(1.0 + clip_high), kl_penalty=kl_code,
               kl_coef=float(kl_coef), entropy_coeff=float(entropy_coeff), seq_mean=0 if token_level_loss else 1,
               loss_scale=float(loss_scale), inv_temperature=float(inv_temperature),
               expected_upstream=None if expected_upstream is None else float(expected_upstream),
               scale_state=scale_state, chunk_rows=int(chunk_rows), compact_rows=bool(compact_rows))
    return _FusedLmHeadLoss.apply(hidden, weight, batch["labels"], batch, cfg)

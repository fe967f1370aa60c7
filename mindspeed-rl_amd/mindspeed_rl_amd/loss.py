"""Loss registry and the GRPO / DAPO / reference loss objects.

Host-side mirror of ``mindspeed_rl/models/loss/`` of the reference: the registry
(``loss_register.py``, ``loss_func_factory.py``), ``BaseLossFunc`` (``base_loss_func.py``), the
text-only log-prob strategy (``logprob_computer.py:73-145``), ``GRPOActorLossFunc``
(``grpo_actor_loss_func.py``), ``DAPOActorLossFunc`` (``dapo_actor_loss_func.py``) and
``ReferenceLossFunc`` (``reference_loss_func.py``).  Class names, registry keys, method
signatures, keyword arguments, return values and error behaviour are the reference's; the work
is done by the HIP kernels of libmrl_hip.so.
"""
import os
from abc import ABC, abstractmethod
from typing import Dict, Tuple

import torch

from . import _lib, vocab_ops
from .functional import is_multimodal
from .packing import (generate_mask, postprocess_packed_seqs, response_window, truncate_middle_and_pad,
                      truncate_prompt_and_pad)
from .vocab_ops import compute_log_probs, vocab_logprob_entropy, vocab_parallel_entropy

STAT_KEYS = ("actor/pg_loss", "actor/pg_clipfrac", "actor/ppo_kl", "actor/kl_loss", "actor/entropy")


# ------------------------------------------------------------------------------------ registry
class LossRegister:
    """Class registry keyed ``stage + "_" + role`` (reference: ``loss_register.py:4-23``).
    Registering a key again replaces the previous class - that is the plug-in point."""

    class_map = dict()

    @classmethod
    def _key(cls, stage: str, role: str) -> str:
        return stage + "_" + role

    @classmethod
    def register_loss(cls, stage: str, role: str):
        def decorate(klass):
            cls.class_map[cls._key(stage, role)] = klass
            return klass

        return decorate

    @classmethod
    def get_class(cls, stage: str, role: str):
        return cls.class_map.get(cls._key(stage, role))

    @classmethod
    def get_instance(cls, stage: str, role: str, *args, **kwargs):
        klass = cls.get_class(stage, role)
        return None if klass is None else klass(*args, **kwargs)


class LossFuncFactory(LossRegister):
    """Reference: ``loss_func_factory.py:5-6`` - its own map, separate from the base class."""

    class_map = dict()


# ------------------------------------------------------------------------------------ policy loss op
def _mask_args(mask, response_length, dev):
    """(mask tensor or None, length tensor or None) in a dtype the kernel reads directly."""
    if mask is not None:
        if mask.dtype not in (torch.float32, torch.int64, torch.int32, torch.uint8, torch.bool):
            mask = mask.to(torch.float32)
        return mask.to(dev).contiguous(), None
    lens = response_length
    if lens.dtype not in (torch.int32, torch.int64):
        lens = lens.to(torch.int64)
    return None, lens.to(dev).reshape(-1).contiguous()


class _PolicyLoss(torch.autograd.Function):
    """log_prob [B,L] (+ entropy [B,L]) -> (scaled loss, out[8]) through mrl_policy_loss_fwd/_bwd."""

    @staticmethod
    def forward(ctx, log_prob, entropy, old_log_prob, ref_log_prob, advantages, mask, lens, cfg):
        dev = _lib.require_device(log_prob, entropy, old_log_prob, ref_log_prob, advantages, mask, lens)
        batch, width = log_prob.shape

        def dense(t):
            return None if t is None else t.to(torch.float32).contiguous()

        lp, ent, old, ref, adv = dense(log_prob), dense(entropy), dense(old_log_prob), dense(ref_log_prob), dense(
            advantages)
        row_sums = torch.empty(max(batch, 1) * 8, dtype=torch.float32, device=dev)
        out = torch.empty(8, dtype=torch.float32, device=dev)
        scalars = (cfg["clip_lo"], cfg["clip_hi"], cfg["kl_penalty"], cfg["kl_coef"], cfg["entropy_coeff"],
                   cfg["seq_mean"], cfg["loss_scale"])
        _lib.call("mrl_policy_loss_fwd", _lib.ptr(lp), _lib.ptr(old), _lib.ptr(ref), _lib.ptr(adv), _lib.ptr(ent),
                  _lib.ptr(mask), _lib.dtype_code(mask) if mask is not None else _lib.F32, _lib.ptr(lens),
                  _lib.dtype_code(lens) if lens is not None else _lib.I32, batch, width, *scalars,
                  _lib.ptr(row_sums), _lib.ptr(out), _lib.stream(dev))
        ctx.save_for_backward(lp, old, ref, adv, mask, lens, row_sums, out)
        ctx.scalars = scalars
        ctx.want_entropy_grad = entropy is not None and entropy.requires_grad
        ctx.mark_non_differentiable(out)
        ctx.set_materialize_grads(False)
        return out[0].clone(), out      # the loss gets its own storage: autograd outputs must not alias

    @staticmethod
    def backward(ctx, g_loss, _g_out):
        if g_loss is None:
            return (None,) * 8
        lp, old, ref, adv, mask, lens, row_sums, out = ctx.saved_tensors
        dev = lp.device
        batch, width = lp.shape
        upstream = g_loss.to(torch.float32).reshape(1).contiguous()
        g_lp = torch.empty_like(lp)
        g_ent = torch.empty_like(lp) if ctx.want_entropy_grad else None
        _lib.call("mrl_policy_loss_bwd", _lib.ptr(lp), _lib.ptr(old), _lib.ptr(ref), _lib.ptr(adv), _lib.ptr(mask),
                  _lib.dtype_code(mask) if mask is not None else _lib.F32, _lib.ptr(lens),
                  _lib.dtype_code(lens) if lens is not None else _lib.I32, batch, width, *ctx.scalars,
                  _lib.ptr(row_sums), _lib.ptr(out), _lib.ptr(upstream), _lib.ptr(g_lp), _lib.ptr(g_ent),
                  _lib.stream(dev))
        return g_lp, g_ent, None, None, None, None, None, None


def policy_loss(log_prob, entropy, old_log_prob, ref_log_prob, advantages, mask=None, response_length=None, *,
                clip_low, clip_high, kl_penalty=None, kl_coef=0.0, entropy_coeff=0.0, token_level_loss=True,
                loss_scale=1.0):
    """Fused clipped-ratio surrogate + KL penalty + entropy bonus.

    Returns ``(loss, out)``: ``loss`` is the 0-dim tensor to back-propagate (``loss_scale *
    pg_loss``), ``out`` the 8 device scalars ``[scaled loss, pg_loss, pg_clipfrac, ppo_kl,
    kl_loss, entropy, sum(mask), rows]``.  ``clip_low`` / ``clip_high`` are the epsilons;
    ``kl_penalty`` is one of ``None, 'kl', 'abs', 'mse', 'low_var_kl'``.
    """
    if kl_penalty is None:
        kl_code = _lib.KL_NONE
    elif kl_penalty in _lib.KL_BY_NAME:
        kl_code = _lib.KL_BY_NAME[kl_penalty]
    else:
        raise NotImplementedError          # 'full' and unknown kinds, as compute_kl_penalty does
    dev = log_prob.device
    mask_t, lens_t = _mask_args(mask, response_length, dev)
    cfg = dict(clip_lo=float(1.0 - clip_low), clip_hi=float(1.0 + clip_high), kl_penalty=kl_code,
               kl_coef=float(kl_coef), entropy_coeff=float(entropy_coeff), seq_mean=0 if token_level_loss else 1,
               loss_scale=float(loss_scale))
    return _PolicyLoss.apply(log_prob, entropy, old_log_prob, ref_log_prob, advantages, mask_t, lens_t, cfg)


# ------------------------------------------------------------------------------------ fused sweep
def fused_supported(output, grad_inplace=False):
    """True if the row-in-registers kernel can take these logits: a floating dtype it knows,
    16-byte aligned dense rows and a vocabulary that fits the register files of one workgroup
    or of two.  (``grad_inplace`` is accepted for call compatibility: every supported shape can
    also be swept in place.)"""
    if output.dtype not in (torch.float32, torch.bfloat16, torch.float16) or not output.is_cuda:
        return False
    vocab = output.shape[-1]
    per_vec = 16 // output.element_size()
    limit = _lib.load().mrl_fused_max_vocab(_lib.dtype_code(output))
    if vocab % per_vec != 0 or vocab > limit:
        return False
    return output.is_contiguous() and output.data_ptr() % 16 == 0


class GradScaleState:
    """What a loss object remembers, in device memory, about the scalar that autograd multiplies its
    loss by: Megatron divides the loss by ``num_microbatches`` (and applies the loss scale) AFTER
    the loss function has returned, and the reference's caller does not tell the loss function
    (``models/base/base_training_engine.py:238-270``).  ``learned`` is the upstream gradient of the
    most recent backward; the next fused sweep reads it on the device and writes its dlogits with
    that scale already applied, so the backward finds nothing to rescale.  Everything is ordered
    by the stream: no host synchronisation, and a wrong guess only costs one rescale pass.
    ``rescales`` counts the backwards that had to move memory."""

    def __init__(self, device):
        self.learned = torch.ones(1, dtype=torch.float32, device=device)
        self.rescales = torch.zeros(1, dtype=torch.int32, device=device)


def _expected_scale(cfg):
    """(device scalar or None, host factor): the scale the sweep writes into its gradients is their
    product.  An explicit ``expected_upstream`` wins; else the loss object's learned scale is read
    on the device; else 1."""
    state, explicit = cfg.get("scale_state"), cfg.get("expected_upstream")
    if explicit is None and state is not None:
        return state.learned, 1.0
    return None, 1.0 if explicit is None else float(explicit)


def _deliver_eager_grads(ctx, buffers, applied, state, g_loss):
    """Backward of an eager-gradient op: ``buffers`` hold the gradients at scale ``applied[0]`` (a
    device scalar, followed by the counter of mrl_scale_rows_note); returns them at the scale of
    ``g_loss``.  The first backward rescales the stored buffers in place and hands them out; a later
    backward over a retained graph must not touch what the first one handed out, so it scales
    copies.  An upstream gradient of 0, Inf or NaN cannot be undone: a later backward over the
    same graph then yields NaN."""
    dev = buffers[0].device
    stream = _lib.stream(dev)
    upstream = g_loss.to(torch.float32).reshape(1).contiguous()
    first = not ctx.handed_out
    ctx.handed_out = True
    if not first:
        buffers = tuple(t.clone() for t in buffers)
        applied = applied.clone()
    learned = _lib.ptr(state.learned) if state is not None else None
    rescales = _lib.ptr(state.rescales) if state is not None else None
    flats = [t.view(-1, t.shape[-1]) for t in buffers]
    if len(flats) == 1 and flats[0].shape[0] > 0:
        flat = flats[0]
        _lib.call("mrl_scale_rows_note", _lib.ptr(flat), _lib.dtype_code(flat), flat.shape[0], flat.shape[1],
                  flat.shape[1], _lib.ptr(upstream), _lib.ptr(applied), learned, rescales, stream)
        return buffers
    for flat in flats:
        _lib.call("mrl_scale_rows", _lib.ptr(flat), _lib.dtype_code(flat), flat.shape[0], flat.shape[1],
                  flat.shape[1], _lib.ptr(upstream), _lib.ptr(applied), stream)
    # the stored buffers now carry `upstream` (first backward) or still what they carried (copies)
    _lib.call("mrl_grad_scale_note", _lib.ptr(upstream), _lib.ptr(applied), learned, rescales, stream)
    return buffers


def _align(n, to):
    return (n + to - 1) // to * to


class _FusedOperands:
    """Device memory and normalised operands of one fused step, and its prepare / reduce launches.

    Everything small lives in ONE allocation (window tables, per-sequence sums, the eight output
    scalars, the gradient scale with its counter, the sweep's workspace) and the per-row operands and
    terms in a second one; the kernels get addresses inside them."""

    def __init__(self, dev, batch, cfg, n_rows, n_seq, width, layout, padded_s, sweep_dtype_code, vocab, sweep_rows):
        lib = _lib.load()

        def f32(t):
            return None if t is None else t.to(dev).to(torch.float32).contiguous()

        def idx(t):
            if t is None:
                return None
            if t.dtype not in (torch.int32, torch.int64):
                t = t.to(torch.int64)
            return t.to(dev).reshape(-1).contiguous()

        self.dev, self.cfg = dev, cfg
        self.n_rows, self.n_seq, self.width, self.layout, self.padded_s = n_rows, n_seq, width, layout, padded_s
        self.old, self.ref, self.adv = f32(batch.get("old_log_prob")), f32(cfg["ref_log_prob"]), f32(batch.get("advantages"))
        self.mask_t, _ = _mask_args(cfg["mask"], batch["response_length"], dev)
        self.prompt, self.resp = idx(batch["prompt_length"]), idx(batch["response_length"])
        if layout == 0:
            self.seqlens = cfg["seqlens"].to(dev).to(torch.int32).contiguous()
            self.cu = cfg["cu"].to(dev).to(torch.int32).contiguous()
        else:
            self.seqlens = self.cu = None
        self.mdt = _lib.dtype_code(self.mask_t) if self.mask_t is not None else _lib.F32
        self.pdt, self.rdt = _lib.dtype_code(self.prompt), _lib.dtype_code(self.resp)
        # the sweep's workspace is sized for the largest launch (a chunk, for the lm_head step)
        # (at least its 16-byte header, whose second word the reduce step borrows as its counter)
        self.ws_bytes = max(16, lib.mrl_fused_workspace_bytes(sweep_dtype_code, sweep_rows, vocab))
        seqs = max(n_seq, 1)
        o_out = 0                                   # float[8]
        o_applied = 32                              # float[2]
        o_ws = 48                                   # the sweep workspace, 16-byte aligned
        o_start = _align(o_ws + self.ws_bytes, 16)  # int64[n_seq]
        o_sums = o_start + 8 * seqs                 # float[n_seq * 8]
        o_count = o_sums + 32 * seqs                # int32[n_seq]
        o_msum = o_count + 4 * seqs                 # float[n_seq]
        self.small = torch.empty(o_msum + 4 * seqs, dtype=torch.uint8, device=dev)
        base = self.small.data_ptr()
        self.out = self.small[o_out:o_out + 32].view(torch.float32)
        self.applied = self.small[o_applied:o_applied + 8].view(torch.float32)
        self.workspace = base + o_ws
        self.p_start, self.p_sums, self.p_count, self.p_msum = base + o_start, base + o_sums, base + o_count, base + o_msum
        self.rows = torch.empty(max(n_rows, 1) * 16, dtype=torch.float32, device=dev)
        self.p_ops = self.rows.data_ptr()
        self.p_terms = self.p_ops + max(n_rows, 1) * 32
        self.loss = torch.empty((), dtype=torch.float32, device=dev)

    def prepare(self, stream):
        cfg = self.cfg
        scale_dev, scale_host = _expected_scale(cfg)
        _lib.call("mrl_fused_loss_prepare", self.layout, self.n_seq, self.width, self.n_rows, _lib.ptr(self.seqlens),
                  _lib.ptr(self.cu), self.padded_s, _lib.ptr(self.prompt), self.pdt, _lib.ptr(self.resp), self.rdt,
                  _lib.ptr(self.old), _lib.ptr(self.ref), _lib.ptr(self.adv), _lib.ptr(self.mask_t), self.mdt,
                  cfg["seq_mean"], self.p_start, self.p_count, self.p_msum, self.p_ops,
                  self.workspace if self.n_rows > 0 else None, self.ws_bytes if self.n_rows > 0 else 0,
                  _lib.ptr(scale_dev), scale_host, _lib.ptr(self.applied) if self.n_rows > 0 else None, stream)
        if self.n_rows == 0:
            self.applied[0] = scale_host if scale_dev is None else scale_dev[0] * scale_host
            self.applied[1] = 0.0

    def reduce(self, stream, p_terms=None):
        cfg = self.cfg
        # word 1 of the cleared sweep workspace counts the workgroups of the reduce step
        done = self.workspace + 4 if self.n_rows > 0 else None
        _lib.call("mrl_fused_loss_reduce", self.p_terms if p_terms is None else p_terms, self.p_start, self.p_count,
                  self.n_seq, self.width, _lib.ptr(self.old), _lib.ptr(self.ref), _lib.ptr(self.adv),
                  _lib.ptr(self.mask_t), self.mdt, _lib.ptr(self.resp), self.rdt, cfg["clip_lo"], cfg["clip_hi"],
                  cfg["kl_penalty"], cfg["kl_coef"], cfg["entropy_coeff"], cfg["seq_mean"], cfg["loss_scale"],
                  self.p_sums, _lib.ptr(self.out), done, _lib.ptr(self.loss), stream)


class _FusedLogprobLoss(torch.autograd.Function):
    """logits -> (loss, out[8]) with dlogits produced in the same sweep (one read, one write of
    the [T, V] tensor for forward + backward).  The backward only rescales the stored dlogits if
    the upstream gradient differs from the scale they already carry (kept in a device scalar, so
    a second backward over a retained graph rescales by the ratio of the two upstream values).
    Three launches in the forward (prepare, sweep, reduce) and one in the backward."""

    @staticmethod
    def forward(ctx, output, labels, batch, cfg):
        dev = _lib.require_device(output, labels)
        vocab = output.shape[-1]
        flat = output.reshape(-1, vocab)
        n_rows = flat.shape[0]
        lab = labels.reshape(-1)
        if lab.dtype not in (torch.int32, torch.int64):
            lab = lab.to(torch.int64)
        lab = lab.contiguous()
        n_seq, width = batch["responses"].shape[0], batch["responses"].shape[-1]
        layout, padded_s = (0, 0) if cfg["packed"] else (1, output.shape[1])
        ops = _FusedOperands(dev, batch, cfg, n_rows, n_seq, width, layout, padded_s, _lib.dtype_code(flat), vocab,
                             n_rows)
        ent = torch.empty(n_rows, dtype=torch.float32, device=dev) if cfg["entropy_coeff"] != 0 else None
        dlogits = flat if cfg["grad_inplace"] else torch.empty_like(flat)
        stream = _lib.stream(dev)
        ops.prepare(stream)
        vocab_ops._timed_call("mrl_fused_logprob_loss", n_rows, dev, _lib.ptr(flat), _lib.dtype_code(flat), n_rows,
                              vocab, vocab, _lib.ptr(lab), _lib.dtype_code(lab), cfg["inv_temperature"],
                              ops.p_ops, 0 if ops.old is None else 1, cfg["clip_lo"], cfg["clip_hi"],
                              cfg["kl_penalty"], cfg["kl_coef"], cfg["entropy_coeff"], cfg["loss_scale"],
                              _lib.ptr(ops.applied), _lib.ptr(dlogits), vocab, None, _lib.ptr(ent), ops.p_terms,
                              ops.workspace, ops.ws_bytes, 1, stream)
        ops.reduce(stream)
        ctx.save_for_backward(dlogits, ops.applied)
        ctx.meta = (tuple(output.shape), cfg.get("scale_state"))
        ctx.handed_out = False
        ctx.mark_non_differentiable(ops.out)
        ctx.set_materialize_grads(False)        # no zero tensor for the statistics output in every backward
        return ops.loss, ops.out

    @staticmethod
    def backward(ctx, g_loss, _g_out):
        if g_loss is None:
            return None, None, None, None
        dlogits, applied = ctx.saved_tensors
        shape, state = ctx.meta
        (grad,) = _deliver_eager_grads(ctx, (dlogits,), applied, state, g_loss)
        return grad.view(shape), None, None, None


def fused_logprob_policy_loss(output, batch, *, packed, seqlens=None, cu_seqlens=None, mask=None, ref_log_prob=None,
                              clip_low, clip_high, kl_penalty=None, kl_coef=0.0, entropy_coeff=0.0,
                              token_level_loss=True, loss_scale=1.0, inv_temperature=1.0, grad_inplace=False,
                              expected_upstream=None, scale_state=None):
    """Log-prob, entropy, policy loss AND dlogits in one sweep over the logits.

    ``output`` is the packed ``[1, T, V]`` (``packed=True``, with ``seqlens`` / ``cu_seqlens``) or
    padded ``[B, S, V]`` logits; ``batch`` holds ``labels, responses, response_length,
    prompt_length, advantages`` and optionally ``old_log_prob``.  Returns ``(loss, out)`` like
    :func:`policy_loss`.  The gradients are written with the scale the caller is expected to
    multiply the loss by before ``backward()``: ``expected_upstream`` if given, else what
    ``scale_state`` (a :class:`GradScaleState`) learned from the previous backward, else 1; any
    other upstream value is honoured by one rescale pass in the backward."""
    if kl_penalty is None:
        kl_code = _lib.KL_NONE
    elif kl_penalty in _lib.KL_BY_NAME:
        kl_code = _lib.KL_BY_NAME[kl_penalty]
    else:
        raise NotImplementedError
    cfg = dict(packed=bool(packed), seqlens=seqlens, cu=cu_seqlens, mask=mask, ref_log_prob=ref_log_prob,
               clip_lo=float(1.0 - clip_low), clip_hi=float(1.0 + clip_high), kl_penalty=kl_code,
               kl_coef=float(kl_coef), entropy_coeff=float(entropy_coeff), seq_mean=0 if token_level_loss else 1,
               loss_scale=float(loss_scale), inv_temperature=float(inv_temperature), grad_inplace=bool(grad_inplace),
               expected_upstream=None if expected_upstream is None else float(expected_upstream),
               scale_state=scale_state)
    return _FusedLogprobLoss.apply(output, batch["labels"], batch, cfg)


def _use_fused(output, kwargs):
    """The fused sweep is the default for a training step; ``fused=False`` (or the environment
    variable MRL_FUSED=0) selects the split forward / backward kernels."""
    if not kwargs.get("fused", os.environ.get("MRL_FUSED", "1") != "0"):
        return False
    injected = vocab_ops.get_vocab_parallel()
    if injected is not None and injected is not vocab_ops.vocab_parallel_cross_entropy:
        return False            # a caller's own cross entropy must be the one that scores the rows
    return (torch.is_grad_enabled() and output.requires_grad
            and fused_supported(output, bool(kwargs.get("grad_inplace", False))))


def _fused_kwargs(kwargs, scale_state=None):
    return dict(packed=kwargs.get("use_remove_padding", False), seqlens=kwargs.get("seqlens_in_batch"),
                cu_seqlens=kwargs.get("cu_seqlens_padded"), inv_temperature=float(kwargs.get("inv_temperature", 1.0)),
                grad_inplace=bool(kwargs.get("grad_inplace", False)),
                expected_upstream=kwargs.get("expected_grad_scale"), scale_state=scale_state)


# ------------------------------------------------------------------------------------ log-prob strategy
class LogProbComputer:
    def compute(self, output, batch, skip_entropy, **kwargs):
        raise NotImplementedError


class StandardLogProbComputer(LogProbComputer):
    """Reference: ``logprob_computer.py:73-145`` at context-parallel size 1.

    One fused sweep gives log-prob and (unless skipped) entropy of every packed / padded row; the
    index-map kernels then cut out the ``[B, L]`` response window.  Extra keyword
    ``inv_temperature`` folds the caller's temperature division into the sweep (default 1)."""

    @staticmethod
    def _get_log_probs_remove_prompt_pad(logprob, batch):
        window = response_window(batch["prompt_length"], batch["response_length"])
        return truncate_prompt_and_pad(batch["responses"], logprob, window)

    @staticmethod
    def _rows_in_windows(output, batch, kwargs):
        """uint8 flag per logits row: 1 where the row lies in a response window, i.e. where the cut
        below reads it.  Rows outside every window (prompts, padding) are not swept at all: their
        log-prob, entropy and gradient are never looked at by the reference either."""
        dev = output.device
        width = batch["responses"].shape[-1]
        prompt = batch["prompt_length"].reshape(-1).to(device=dev, dtype=torch.int64)
        if kwargs.get("use_remove_padding", False):
            n_rows = output.shape[-2]
            n = kwargs["seqlens_in_batch"].reshape(-1).to(device=dev, dtype=torch.int64)
            start = kwargs["cu_seqlens_padded"].reshape(-1).to(device=dev, dtype=torch.int64)[:-1]
            cut = (prompt - 1) < n                     # postprocess_packed_seqs: start += P-1, len -= P
            start = torch.where(cut, start + prompt - 1, start)
            n = torch.where(cut, n - prompt, n)
        else:
            n_seq, padded = output.shape[0], output.shape[1]
            n_rows = n_seq * padded
            resp = batch["response_length"].reshape(-1).to(device=dev, dtype=torch.int64)
            lo = (prompt - 1).clamp(0, padded)
            hi = (prompt + resp - 1).clamp(0, padded)
            start = lo + torch.arange(n_seq, device=dev, dtype=torch.int64) * padded
            n = hi - lo
        n = n.clamp(0, width)
        start = start.clamp(0, n_rows)
        end = (start + n).clamp(max=n_rows)
        edge = torch.zeros(n_rows + 1, dtype=torch.int32, device=dev)
        one = torch.ones_like(start, dtype=torch.int32)
        edge.index_add_(0, start, one)
        edge.index_add_(0, end, -one)
        return (torch.cumsum(edge[:-1], 0) > 0).to(torch.uint8)

    def compute(self, output, batch, skip_entropy, **kwargs):
        labels = batch["labels"]
        inv_t = float(kwargs.get("inv_temperature", 1.0))
        injected = vocab_ops.get_vocab_parallel()
        weight = kwargs.get("lm_head_weight")
        if weight is not None:
            # `output` holds the hidden states: the rows of the response windows are projected and scored
            # tile by tile on the matrix cores, no logits are written (forward only, no autograd)
            from .lmhead import lmhead_logprob
            active = self._rows_in_windows(output, batch, kwargs).view(labels.shape)
            log_probs, entropy, _ = lmhead_logprob(output, weight, labels, inv_temperature=inv_t,
                                                   want_entropy=not skip_entropy, row_active=active)
        elif injected is not None and injected is not vocab_ops.vocab_parallel_cross_entropy:
            # a caller's own cross entropy (the reference's hook) scores the rows, as in the reference
            scaled = output if inv_t == 1.0 else output * inv_t
            log_probs = compute_log_probs(scaled, labels)
            entropy = None if skip_entropy else vocab_parallel_entropy(scaled)
        else:
            active = self._rows_in_windows(output, batch, kwargs).view(labels.shape)
            log_probs, entropy, _ = vocab_logprob_entropy(output, labels, inv_temperature=inv_t,
                                                          want_entropy=not skip_entropy, row_active=active,
                                                          grad_inplace=bool(kwargs.get("grad_inplace", False)))
        if kwargs.get("use_remove_padding", False):
            seqlens = kwargs.get("seqlens_in_batch", None)
            cu = kwargs.get("cu_seqlens_padded", None)
            seq_len = batch["responses"].shape[-1]

            def cut(x):
                return postprocess_packed_seqs(x, seqlens, cu, seq_len, prompt_length=batch["prompt_length"])
        else:
            def cut(x):
                return self._get_log_probs_remove_prompt_pad(x, batch)

        log_probs = cut(log_probs)
        entropy = torch.zeros_like(log_probs) if skip_entropy else cut(entropy)
        return log_probs, entropy


class MultimodalLogProbComputer(LogProbComputer):
    """Reference: ``logprob_computer.py:40-70``: the logits of the response window are scored against
    ``responses`` (not ``labels``); entropy is taken over the full output.

    The reference first copies the window out of the ``[B, S, V]`` logits
    (``truncate_middle_and_pad``) and scores the zero-padded copy, so positions past a sequence's
    window come out as ``log_softmax(0)[token] = -log V``.  Here the sweep runs over the window's
    rows where they lie (the responses are scattered to those rows as labels, every other row is
    skipped), the per-row results are cut to ``[B, L]`` with ``-log V`` as the pad value, and the
    gradient flows back through the sweep: no ``[B, L, V]`` copy in either direction."""

    def compute(self, output, batch, skip_entropy, **kwargs):
        responses = batch["responses"]
        if output.dim() != 3:
            raise ValueError("output must have shape (mbs, seq_len, vocab_size)")
        window = response_window(batch["prompt_length"], batch["response_length"])
        n_seq, seq_len, vocab = output.shape
        out_len = responses.shape[-1]
        start = window[:, 0].to(torch.int64).clamp(0, seq_len)
        end = window[:, 1].to(torch.int64).clamp(0, seq_len)
        count = (end - start).clamp(0, out_len)
        j = torch.arange(out_len, device=output.device)
        valid = j[None, :] < count[:, None]
        rows = (start[:, None] + j[None, :]).clamp(max=seq_len - 1)
        labels = torch.zeros((n_seq, seq_len), dtype=torch.int64, device=output.device)
        active = torch.zeros((n_seq, seq_len), dtype=torch.uint8, device=output.device)
        seq_idx = torch.arange(n_seq, device=output.device)[:, None].expand_as(rows)
        labels[seq_idx[valid], rows[valid]] = responses.to(torch.int64)[valid]
        active[seq_idx[valid], rows[valid]] = 1
        inv_t = float(kwargs.get("inv_temperature", 1.0))
        row_logp, _, _ = vocab_logprob_entropy(output, labels, inv_temperature=inv_t, want_entropy=False,
                                               row_active=active)
        pad = -float(torch.log(torch.tensor(float(vocab), dtype=torch.float32)))
        log_probs = truncate_prompt_and_pad(responses, row_logp, window, pad_value=pad)
        entropy = torch.zeros_like(log_probs) if skip_entropy else vocab_parallel_entropy(output)
        return log_probs, entropy


# ------------------------------------------------------------------------------------ loss objects
class BaseLossFunc(ABC):
    """Reference: ``base_loss_func.py:13-57``."""

    def __init__(self):
        # base_loss_func.py:15
        self.logprob_computer = MultimodalLogProbComputer() if is_multimodal() else StandardLogProbComputer()
        self._grad_scale_states = {}

    def add_loss_meta_info(self, meta_info: Dict):
        pass

    def grad_scale_state(self, device) -> GradScaleState:
        """This object's learned upstream gradient scale on ``device`` (created on first use)."""
        key = torch.device(device)
        if key not in self._grad_scale_states:
            self._grad_scale_states[key] = GradScaleState(key)
        return self._grad_scale_states[key]

    @abstractmethod
    def compute_loss(self, output: torch.Tensor, batch: Dict[str, torch.Tensor], forward_only=False,
                     non_loss_data=True, **kwargs) -> Tuple[torch.Tensor, Dict]:
        pass

    def _fused(self, output, kwargs):
        """The one-pass sweep scores rows against ``labels``: it stands in for the standard log-prob
        strategy only (a caller that installs another ``logprob_computer`` gets the split path)."""
        return type(self.logprob_computer) is StandardLogProbComputer and _use_fused(output, kwargs)

    def _from_hidden(self, output, batch, kwargs, **loss_args):
        """The training step when the caller hands over the hidden states and ``lm_head_weight=``
        instead of logits (keyword arguments ``lm_head_chunk_rows``, ``lm_head_compact_rows``):
        logits exist for one chunk of rows at a time, and ``backward()`` reaches the hidden states
        and the weight.  Forward-only calls take the same keyword through ``compute_log_probs``."""
        from .lmhead import fused_lmhead_policy_loss
        if type(self.logprob_computer) is not StandardLogProbComputer:
            raise NotImplementedError("lm_head_weight= needs the standard log-prob strategy")
        return fused_lmhead_policy_loss(
            output, kwargs["lm_head_weight"], batch, packed=kwargs.get("use_remove_padding", False),
            seqlens=kwargs.get("seqlens_in_batch"), cu_seqlens=kwargs.get("cu_seqlens_padded"),
            inv_temperature=float(kwargs.get("inv_temperature", 1.0)),
            expected_upstream=kwargs.get("expected_grad_scale"), scale_state=self.grad_scale_state(output.device),
            chunk_rows=int(kwargs.get("lm_head_chunk_rows", 32768)),
            compact_rows=bool(kwargs.get("lm_head_compact_rows", True)), **loss_args)

    @staticmethod
    def _get_compute_log_probs_input(output: torch.Tensor, batch: Dict[str, torch.Tensor]):
        if "responses" not in batch:
            raise ValueError("The responses is None")
        responses = batch["responses"]
        window = response_window(batch["prompt_length"], batch["response_length"])
        return responses, truncate_middle_and_pad(responses, output, window)

    @staticmethod
    def _get_log_probs_remove_prompt_pad(logprob: torch.Tensor, batch: Dict[str, torch.Tensor]):
        window = response_window(batch["prompt_length"], batch["response_length"])
        return truncate_prompt_and_pad(batch["responses"], logprob, window)

    def compute_log_probs(self, output, batch: Dict[str, torch.Tensor], skip_entropy=True, **kwargs):
        return self.logprob_computer.compute(output, batch, skip_entropy, **kwargs)


class DeferredStats(dict):
    """The statistics dict of ``compute_loss`` with the device-to-host copy taken off the critical path:
    the eight output scalars are copied into pinned host memory asynchronously, and the python floats
    are made when a value is first looked at (``stats[key]``, ``items()``, ``values()``, ``get``,
    printing, copying, pickling) - typically after the backward, when the reference's engine gathers
    the metrics of all micro-batches.  Keys, ``len`` and ``in`` need no synchronisation.  Selected with
    ``deferred_stats=True`` (keyword of ``compute_loss``) or the environment variable
    MRL_DEFERRED_STATS=1; the default returns plain floats at once, like the reference.

    A ``compute_loss`` that runs while its stream is being captured into a graph (``torch.cuda.graph``)
    always returns this type, bound to the device scalars instead of a host copy: it must not be read
    during the capture, and after every replay it yields that replay's values (one synchronous
    32-byte copy per access)."""

    __slots__ = ("_pending", "__weakref__")

    def __init__(self, spec, host, event):
        super().__init__((key, None) for key, _, _ in spec)
        self._pending = (spec, host, event)

    def _fetch(self):
        if self._pending is not None:
            spec, source, event = self._pending
            if event is None:
                # made while a graph was being captured: `source` is the device tensor, which every
                # replay rewrites, so it is read afresh on every access and nothing is cached
                values = source.detach().cpu().tolist()
            else:
                self._pending = None
                event.synchronize()
                values = source.tolist()
            for key, index, use_abs in spec:
                dict.__setitem__(self, key, abs(values[index]) if use_abs else values[index])
        return self

    # every way to a value goes through _fetch(); __iter__ / keys are overridden so that dict(), {**x} and
    # update() cannot take the interpreter's short cut past these methods
    def __getitem__(self, key):
        return dict.__getitem__(self._fetch(), key)

    def get(self, key, default=None):
        return dict.get(self._fetch(), key, default)

    def items(self):
        return dict.items(self._fetch())

    def values(self):
        return dict.values(self._fetch())

    def keys(self):
        return dict.keys(self)

    def __iter__(self):
        return dict.__iter__(self)

    def pop(self, key, *default):
        return dict.pop(self._fetch(), key, *default)

    def popitem(self):
        return dict.popitem(self._fetch())

    def setdefault(self, key, default=None):
        return dict.setdefault(self._fetch(), key, default)

    def copy(self):
        return dict(dict.items(self._fetch()))

    def __eq__(self, other):
        return dict.__eq__(self._fetch(), other)

    def __ne__(self, other):
        return not self.__eq__(other)

    __hash__ = None

    def __repr__(self):
        return dict.__repr__(self._fetch())

    def __reduce__(self):
        return (dict, (self.copy(),))


class _PinnedRing:
    """Pinned host slots for the deferred statistics of one device: allocated once, used in turn.  A
    slot is handed out again only after 256 later calls; whoever still holds it then is fetched first."""

    def __init__(self, slots=256):
        import weakref
        self._weakref = weakref
        self.buffer = torch.empty((slots, 8), dtype=torch.float32, pin_memory=True)
        self.holders = [None] * slots
        self.next = 0

    def take(self, make):
        slot = self.next
        self.next = (slot + 1) % len(self.holders)
        old = self.holders[slot]
        old = old() if old is not None else None
        if old is not None:
            old._fetch()
        holder = make(self.buffer[slot])
        self.holders[slot] = self._weakref.ref(holder)
        return holder


_pinned_rings = {}


def _finish(loss, out, kwargs=None, skip=()):
    """The five statistics as python floats from ONE device-to-host copy (the reference issues five
    ``.item()`` calls); ``abs`` on the policy loss as in ``grpo_actor_loss_func.py:91-97``.  With
    deferred statistics the copy is asynchronous and the floats are made on first access."""
    spec = [(STAT_KEYS[i], i + 1, i == 0) for i in range(5) if STAT_KEYS[i] not in skip]
    deferred = (kwargs or {}).get("deferred_stats", os.environ.get("MRL_DEFERRED_STATS", "0") == "1")
    if out.is_cuda and torch.cuda.is_current_stream_capturing():
        # under graph capture nothing may wait for the device: the dict reads the device scalars when it
        # is looked at (after a replay), whatever was asked for
        return loss, DeferredStats(spec, out, None)
    if not deferred:
        host = out.detach().cpu().tolist()
        return loss, {key: (abs(host[index]) if use_abs else host[index]) for key, index, use_abs in spec}
    dev = out.device
    ring = _pinned_rings.get(dev)
    if ring is None:
        ring = _pinned_rings[dev] = _PinnedRing()

    def make(host):
        host.copy_(out.detach(), non_blocking=True)
        event = torch.cuda.Event()
        event.record(torch.cuda.current_stream(dev))
        return DeferredStats(spec, host, event)

    return loss, ring.take(make)


def _dynamic_scale(batch, forward_only, kwargs):
    """``responses.size(0) / actual_micro_batch_size`` under dynamic batch size, else 1."""
    if kwargs.get("use_dynamic_bsz", False) and not forward_only:
        return batch["responses"].size(0) / kwargs.get("actual_micro_batch_size", None)
    return 1.0


@LossFuncFactory.register_loss("ray_grpo", "actor")
class GRPOActorLossFunc(BaseLossFunc):
    """Reference: ``grpo_actor_loss_func.py:14-144``."""

    def __init__(self):
        super().__init__()
        self.clip_ratio = 0.2
        self.entropy_coeff = 0.0

    def add_loss_meta_info(self, meta_info: Dict):
        if meta_info is None:
            return
        if "clip_ratio" in meta_info.keys():
            self.clip_ratio = float(meta_info["clip_ratio"])
        for key in ("kl_ctrl", "entropy_coeff", "kl_penalty"):
            if key in meta_info.keys():
                setattr(self, key, meta_info[key])

    @staticmethod
    def _get_policy_loss_input(batch: Dict[str, torch.Tensor]):
        if "responses" not in batch:
            raise ValueError("The responses is None")
        response_mask = generate_mask(batch["responses"], batch["response_length"])
        return (response_mask, batch.get("old_log_prob"), batch.get("advantages"), batch.get("ref_log_prob"))

    def compute_loss(self, output: torch.Tensor, batch: Dict[str, torch.Tensor], forward_only=False,
                     non_loss_data=True, **kwargs) -> Tuple[torch.Tensor, Dict]:
        if "responses" not in batch:
            raise ValueError("The responses is None")
        if forward_only:
            log_probs, _ = super().compute_log_probs(output=output, batch=batch, **kwargs)
            return log_probs
        if kwargs.get("lm_head_weight") is not None:
            loss, out = self._from_hidden(
                output, batch, kwargs, ref_log_prob=batch.get("ref_log_prob"), clip_low=self.clip_ratio,
                clip_high=self.clip_ratio, kl_penalty=self.kl_penalty, kl_coef=self.kl_ctrl.value,
                entropy_coeff=self.entropy_coeff, token_level_loss=True,
                loss_scale=_dynamic_scale(batch, forward_only, kwargs))
            return _finish(loss, out, kwargs)
        if self._fused(output, kwargs):
            loss, out = fused_logprob_policy_loss(
                output, batch, ref_log_prob=batch.get("ref_log_prob"), clip_low=self.clip_ratio,
                clip_high=self.clip_ratio, kl_penalty=self.kl_penalty, kl_coef=self.kl_ctrl.value,
                entropy_coeff=self.entropy_coeff, token_level_loss=True,
                loss_scale=_dynamic_scale(batch, forward_only, kwargs),
                **_fused_kwargs(kwargs, self.grad_scale_state(output.device)))
            return _finish(loss, out, kwargs)
        log_probs, entropy = super().compute_log_probs(output=output, batch=batch,
                                                       skip_entropy=(self.entropy_coeff == 0), **kwargs)
        # batch['response_mask'] is ignored here, as in the reference: the mask is j < response_length
        loss, out = policy_loss(log_probs, entropy if self.entropy_coeff != 0 else None, batch.get("old_log_prob"),
                                batch.get("ref_log_prob"), batch.get("advantages"),
                                response_length=batch["response_length"], clip_low=self.clip_ratio,
                                clip_high=self.clip_ratio, kl_penalty=self.kl_penalty, kl_coef=self.kl_ctrl.value,
                                entropy_coeff=self.entropy_coeff, token_level_loss=True,
                                loss_scale=_dynamic_scale(batch, forward_only, kwargs))
        return _finish(loss, out, kwargs)

    @staticmethod
    def _compute_grpo_policy_loss(old_log_prob, log_prob, ref_log_prob, advantages, entropy, eos_mask, cliprange,
                                  kl_ctrl, kl_penalty, entropy_coeff):
        """Reference: ``grpo_actor_loss_func.py:100-144``.  Returns ``(pg_loss, pg_clipfrac, ppo_kl,
        kl_loss, entropy_loss)`` as 0-dim tensors; ``pg_loss`` is differentiable."""
        loss, out = policy_loss(log_prob, entropy, old_log_prob, ref_log_prob, advantages, mask=eos_mask,
                                clip_low=cliprange, clip_high=cliprange, kl_penalty=kl_penalty,
                                kl_coef=kl_ctrl.value, entropy_coeff=entropy_coeff, token_level_loss=True)
        return loss, out[2], out[3], out[4], out[5]


@LossFuncFactory.register_loss("ray_dapo", "actor")
class DAPOActorLossFunc(BaseLossFunc):
    """Reference: ``dapo_actor_loss_func.py:13-152``."""

    def __init__(self):
        super().__init__()
        self.clip_ratio = 0.2
        self.entropy_coeff = 0.0

    def add_loss_meta_info(self, meta_info: Dict):
        if meta_info is None:
            return
        casts = (("clip_ratio", float), ("kl_ctrl", None), ("entropy_coeff", None), ("token_level_loss", bool),
                 ("clip_higher_enable", bool), ("clip_ratio_low", float), ("clip_ratio_high", float))
        for key, cast in casts:
            if key in meta_info.keys():
                setattr(self, key, meta_info[key] if cast is None else cast(meta_info[key]))

    @staticmethod
    def _get_policy_loss_input(batch: Dict[str, torch.Tensor]):
        if "responses" not in batch:
            raise ValueError("The responses is None")
        response_mask = batch["response_mask"] if "response_mask" in batch else \
            generate_mask(batch["responses"], batch["response_length"])
        return response_mask, batch.get("old_log_prob"), batch.get("advantages")

    def compute_loss(self, output: torch.Tensor, batch: Dict[str, torch.Tensor], forward_only=False,
                     non_loss_data=True, **kwargs) -> Tuple[torch.Tensor, Dict]:
        if "responses" not in batch:
            raise ValueError("The responses is None")
        if forward_only:
            log_probs, _ = super().compute_log_probs(output=output, batch=batch, **kwargs)
            return log_probs
        if not self.clip_higher_enable:
            self.clip_ratio_low = self.clip_ratio
            self.clip_ratio_high = self.clip_ratio
        mask = batch["response_mask"] if "response_mask" in batch else None
        if kwargs.get("lm_head_weight") is not None:
            loss, out = self._from_hidden(
                output, batch, kwargs, mask=mask, clip_low=self.clip_ratio_low, clip_high=self.clip_ratio_high,
                kl_penalty=None, entropy_coeff=self.entropy_coeff, token_level_loss=self.token_level_loss,
                loss_scale=_dynamic_scale(batch, forward_only, kwargs))
            return _finish(loss, out, kwargs)
        if self._fused(output, kwargs):
            loss, out = fused_logprob_policy_loss(
                output, batch, mask=mask, clip_low=self.clip_ratio_low, clip_high=self.clip_ratio_high,
                kl_penalty=None, entropy_coeff=self.entropy_coeff, token_level_loss=self.token_level_loss,
                loss_scale=_dynamic_scale(batch, forward_only, kwargs),
                **_fused_kwargs(kwargs, self.grad_scale_state(output.device)))
            return _finish(loss, out, kwargs)
        log_probs, entropy = super().compute_log_probs(output=output, batch=batch,
                                                       skip_entropy=(self.entropy_coeff == 0), **kwargs)
        loss, out = policy_loss(log_probs, entropy if self.entropy_coeff != 0 else None, batch.get("old_log_prob"),
                                None, batch.get("advantages"), mask=mask,
                                response_length=None if mask is not None else batch["response_length"],
                                clip_low=self.clip_ratio_low, clip_high=self.clip_ratio_high, kl_penalty=None,
                                entropy_coeff=self.entropy_coeff, token_level_loss=self.token_level_loss,
                                loss_scale=_dynamic_scale(batch, forward_only, kwargs))
        return _finish(loss, out, kwargs)

    @staticmethod
    def _compute_dapo_policy_loss(old_log_prob, log_prob, entropy, entropy_coeff, advantages, eos_mask,
                                  clip_ratio_low, clip_ratio_high, token_level_loss):
        """Reference: ``dapo_actor_loss_func.py:105-152``.  In sequence-mean mode the clip fraction
        is 0 and a row with an empty mask makes the loss NaN, as in the reference."""
        loss, out = policy_loss(log_prob, entropy, old_log_prob, None, advantages, mask=eos_mask,
                                clip_low=clip_ratio_low, clip_high=clip_ratio_high, kl_penalty=None,
                                entropy_coeff=entropy_coeff, token_level_loss=token_level_loss)
        return loss, out[2], out[3], out[4], out[5]


@LossFuncFactory.register_loss("ray_ppo", "actor")
class PPOActorLossFunc(BaseLossFunc):
    """Reference: ``ppo_actor_loss_func.py:13-133``: the GRPO surrogate without the KL term; four
    statistics (no ``actor/kl_loss``)."""

    def __init__(self):
        super().__init__()
        self.clip_ratio = 0.2
        self.entropy_coeff = 0.0

    def add_loss_meta_info(self, meta_info: Dict):
        if meta_info is None:
            return
        if "clip_ratio" in meta_info.keys():
            self.clip_ratio = float(meta_info["clip_ratio"])
        for key in ("kl_ctrl", "entropy_coeff"):
            if key in meta_info.keys():
                setattr(self, key, meta_info[key])

    @staticmethod
    def _get_policy_loss_input(batch: Dict[str, torch.Tensor]):
        if "responses" not in batch:
            raise ValueError("The responses is None")
        response_mask = generate_mask(batch["responses"], batch["response_length"])
        return (response_mask, batch.get("old_log_prob"), batch.get("advantages"), batch.get("ref_log_prob"))

    def compute_loss(self, output: torch.Tensor, batch: Dict[str, torch.Tensor], forward_only=False,
                     non_loss_data=True, **kwargs) -> Tuple[torch.Tensor, Dict]:
        if "responses" not in batch:
            raise ValueError("The responses is None")
        if forward_only:
            log_probs, _ = super().compute_log_probs(output=output, batch=batch, **kwargs)
            return log_probs
        common = dict(clip_low=self.clip_ratio, clip_high=self.clip_ratio, kl_penalty=None,
                      entropy_coeff=self.entropy_coeff, token_level_loss=True,
                      loss_scale=_dynamic_scale(batch, forward_only, kwargs))
        if kwargs.get("lm_head_weight") is not None:
            loss, out = self._from_hidden(output, batch, kwargs, **common)
        elif self._fused(output, kwargs):
            loss, out = fused_logprob_policy_loss(output, batch, **common,
                                                  **_fused_kwargs(kwargs, self.grad_scale_state(output.device)))
        else:
            log_probs, entropy = super().compute_log_probs(output=output, batch=batch,
                                                           skip_entropy=(self.entropy_coeff == 0), **kwargs)
            loss, out = policy_loss(log_probs, entropy if self.entropy_coeff != 0 else None,
                                    batch.get("old_log_prob"), None, batch.get("advantages"),
                                    response_length=batch["response_length"], **common)
        return _finish(loss, out, kwargs, skip=(STAT_KEYS[3],))          # PPO reports no actor/kl_loss

    @staticmethod
    def _compute_ppo_policy_loss(old_log_prob, log_prob, advantages, eos_mask, cliprange, entropy, entropy_coeff):
        """Reference: ``ppo_actor_loss_func.py:91-133``: ``(pg_loss, pg_clipfrac, ppo_kl, entropy_loss)``."""
        loss, out = policy_loss(log_prob, entropy, old_log_prob, None, advantages, mask=eos_mask, clip_low=cliprange,
                                clip_high=cliprange, kl_penalty=None, entropy_coeff=entropy_coeff,
                                token_level_loss=True)
        return loss, out[2], out[3], out[5]


@LossFuncFactory.register_loss("ray_grpo", "reference")
@LossFuncFactory.register_loss("ray_ppo", "reference")
class ReferenceLossFunc(BaseLossFunc):
    """Reference: ``reference_loss_func.py:9-25``: forward-only log-prob of the reference policy."""

    def __init__(self):
        super(ReferenceLossFunc, self).__init__()

    def compute_loss(self, output: torch.Tensor, batch: Dict[str, torch.Tensor], forward_only=False,
                     non_loss_data=True, **kwargs) -> Tuple[torch.Tensor, Dict]:
        log_probs, _ = super().compute_log_probs(output=output, batch=batch, **kwargs)
        if forward_only:
            return log_probs
        return None


@LossFuncFactory.register_loss("ray_grpo", "reward")
@LossFuncFactory.register_loss("ray_ppo", "reward")
class RewardLossFunc(BaseLossFunc):
    """Reference: ``reward_loss_func.py:11-31``: the reward model's scores, unpacked to
    ``[B, seq_len, ...]`` when the batch was packed."""

    def __init__(self):
        super(RewardLossFunc, self).__init__()

    def compute_loss(self, output: torch.Tensor, batch: Dict[str, torch.Tensor], forward_only=False,
                     non_loss_data=True, **kwargs) -> Tuple[torch.Tensor, Dict]:
        if kwargs.get("use_remove_padding", False):
            output = postprocess_packed_seqs(output=output, seqlens_in_batch=kwargs.get("seqlens_in_batch", None),
                                             cu_seqlens_padded=kwargs.get("cu_seqlens_padded", None),
                                             seq_len=kwargs.get("seq_len", None))
        return output

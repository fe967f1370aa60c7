"""Remove-padding pack / unpack, the padded response window and the length mask.

Host-side mirror of ``mindspeed_rl/utils/remove_padding.py``, the two ``truncate_*_and_pad``
functions of ``mindspeed_rl/utils/pad_process.py`` and ``generate_mask`` of
``mindspeed_rl/utils/utils.py`` - same names, arguments and return values - backed by the index
map kernels.  Where the reference runs a Python loop with two or three ``.item()`` calls per
sequence, these launch one kernel; ``preprocess_packed_seqs`` keeps a single host read (the
packed length, needed to size its outputs).
"""
import torch

from . import _lib


def _as_index(t):
    """int32 / int64 tensor, flattened and dense, for a [B] or [B,1] length column."""
    if t.dtype not in (torch.int32, torch.int64):
        t = t.to(torch.int64)
    return t.reshape(-1).contiguous()


def generate_mask(data_pad, seq_lengths):
    """Reference: ``utils/utils.py:57-67``.  ``[B, data_pad.size(1)]`` int64 mask with
    ``seq_lengths[i]`` leading ones per row, built on the device of ``seq_lengths``."""
    lengths = _as_index(seq_lengths)
    if not lengths.is_cuda and data_pad.is_cuda:
        lengths = lengths.to(data_pad.device)      # the reference builds the mask on the host
    dev = _lib.require_device(lengths)
    batch, width = lengths.numel(), data_pad.size(1)
    out = torch.empty((batch, width), dtype=torch.int64, device=dev)
    _lib.call("mrl_generate_mask", _lib.ptr(lengths), _lib.dtype_code(lengths), batch, width, _lib.ptr(out),
              _lib.stream(dev))
    return out


def pack_index(attention_mask_1d, tp_size):
    """``(seqlens_in_batch int32 [B], cu_seqlens_padded int32 [B+1], total int64 [1])`` on the
    device, without any host synchronisation."""
    mask = attention_mask_1d
    if mask.dtype not in (torch.int64, torch.int32, torch.uint8, torch.bool, torch.float32):
        mask = mask.to(torch.int64)
    mask = mask.contiguous()
    dev = _lib.require_device(mask)
    batch, width = mask.shape
    seqlens = torch.empty(batch, dtype=torch.int32, device=dev)
    cu = torch.empty(batch + 1, dtype=torch.int32, device=dev)
    total = torch.empty(1, dtype=torch.int64, device=dev)
    _lib.call("mrl_pack_index_build", _lib.ptr(mask), _lib.dtype_code(mask), batch, width, int(tp_size),
              _lib.ptr(seqlens), _lib.ptr(cu), _lib.ptr(total), _lib.stream(dev))
    return seqlens, cu, total


def preprocess_packed_seqs(input_ids, labels, attention_mask_1d, tp_size):
    """Reference: ``utils/remove_padding.py:10-87``.  Returns ``(input_ids_packed [1,T],
    position_ids_packed [1,T] int32, labels_packed [1,T], seqlens_in_batch [B] int32,
    cu_seqlens_padded [B+1] int32)``."""
    batch, width = input_ids.shape
    if attention_mask_1d.shape != (batch, width):
        raise ValueError("attention_mask_1d must have shape (batch_size, seq_len) matching input_ids")
    dev = _lib.require_device(input_ids, labels, attention_mask_1d)
    seqlens, cu, total = pack_index(attention_mask_1d, tp_size)
    pack_length = int(total.item())          # the one host read: sizes the packed outputs
    ids = input_ids.contiguous()
    lab = labels.to(ids.dtype).contiguous()
    if ids.dtype not in (torch.int32, torch.int64):
        raise TypeError("input_ids must be int32 or int64")
    ids_packed = torch.empty(pack_length, dtype=ids.dtype, device=dev)
    labels_packed = torch.empty(pack_length, dtype=ids.dtype, device=dev)
    pos_packed = torch.empty(pack_length, dtype=torch.int32, device=dev)
    _lib.call("mrl_pack_rows", _lib.ptr(ids), _lib.ptr(ids_packed), _lib.ptr(lab), _lib.ptr(labels_packed),
              ids.element_size(), batch, width, _lib.ptr(seqlens), _lib.ptr(cu), pack_length, _lib.ptr(pos_packed),
              _lib.stream(dev))
    return (ids_packed.unsqueeze(0), pos_packed.unsqueeze(0), labels_packed.unsqueeze(0), seqlens, cu)


class _UnpadGather(torch.autograd.Function):
    """packed [1,T] fp32 -> [B,L]; backward is the deterministic gather-form scatter."""

    @staticmethod
    def forward(ctx, packed, seqlens, cu, seq_len, prompt):
        out = _unpad_raw(packed, seqlens, cu, seq_len, prompt)
        ctx.save_for_backward(seqlens, cu, prompt)
        ctx.meta = (tuple(packed.shape), int(seq_len))
        return out

    @staticmethod
    def backward(ctx, g_out):
        seqlens, cu, prompt = ctx.saved_tensors
        shape, seq_len = ctx.meta
        dev = g_out.device
        total = shape[1]
        g = g_out.to(torch.float32).contiguous()
        g_packed = torch.empty(total, dtype=torch.float32, device=dev)
        _lib.call("mrl_pad_scatter", _lib.ptr(g), seqlens.numel(), seq_len, _lib.ptr(seqlens), _lib.ptr(cu),
                  _lib.ptr(prompt), _lib.dtype_code(prompt) if prompt is not None else _lib.I32, total,
                  _lib.ptr(g_packed), _lib.stream(dev))
        return g_packed.view(shape), None, None, None, None


def _unpad_raw(packed, seqlens, cu, seq_len, prompt):
    dev = _lib.require_device(packed, seqlens, cu, prompt)
    src = packed.contiguous()
    total = src.shape[1]
    trailing = list(src.shape[2:])
    inner = 1
    for d in trailing:
        inner *= d
    batch = seqlens.shape[0]
    if src.element_size() not in (2, 4, 8):
        raise TypeError("unsupported element size %d" % src.element_size())
    out = torch.empty([batch, seq_len] + trailing, dtype=src.dtype, device=dev)
    _lib.call("mrl_unpad_gather", _lib.ptr(src), src.element_size(), total, inner, _lib.ptr(seqlens), _lib.ptr(cu),
              _lib.ptr(prompt), _lib.dtype_code(prompt) if prompt is not None else _lib.I32, batch, int(seq_len),
              _lib.ptr(out), _lib.stream(dev))
    return out


def postprocess_packed_seqs(output, seqlens_in_batch, cu_seqlens_padded, seq_len, prompt_length=None):
    """Reference: ``utils/remove_padding.py:90-136``: packed ``[1,T,...]`` -> ``[B,seq_len,...]``
    with optional prompt truncation (``start += P-1``, ``len -= P``).  Differentiable for fp32
    ``[1,T]`` and ``[1,T,1]`` inputs.  A window longer than ``seq_len`` is cut to ``seq_len`` (the reference
    raises there)."""
    if output.shape[0] != 1:
        raise ValueError("Expected output tensor to have shape[0] == 1 (packed batch dimension)")
    seqlens = seqlens_in_batch.to(torch.int32).contiguous()
    cu = cu_seqlens_padded.to(torch.int32).contiguous()
    prompt = None if prompt_length is None else _as_index(prompt_length)
    if output.requires_grad and torch.is_grad_enabled():
        scalar_rows = output.dim() == 2 or (output.dim() == 3 and output.shape[2] == 1)
        if not scalar_rows or output.dtype != torch.float32:
            raise TypeError("gradients are supported for fp32 [1, T] or [1, T, 1] inputs only")
        out = _UnpadGather.apply(output.reshape(1, output.shape[1]), seqlens, cu, seq_len, prompt)
        return out.unsqueeze(-1) if output.dim() == 3 else out
    return _unpad_raw(output, seqlens, cu, seq_len, prompt)


class _WindowGather(torch.autograd.Function):
    @staticmethod
    def forward(ctx, src, window, out_len, pad_value):
        out = _window_raw(src, window, out_len, pad_value)
        ctx.save_for_backward(window)
        ctx.meta = (tuple(src.shape), int(out_len))
        return out

    @staticmethod
    def backward(ctx, g_out):
        (window,) = ctx.saved_tensors
        shape, out_len = ctx.meta
        dev = g_out.device
        g = g_out.to(torch.float32).contiguous()
        g_src = torch.empty(shape, dtype=torch.float32, device=dev)
        _lib.call("mrl_window_scatter", _lib.ptr(g), shape[0], shape[1], _lib.ptr(window), _lib.dtype_code(window),
                  out_len, _lib.ptr(g_src), _lib.stream(dev))
        return g_src, None, None, None


def _pad_bits(dtype, pad_value):
    t = torch.tensor([pad_value], dtype=dtype)
    if t.element_size() == 2:
        return int(t.view(torch.int16).item()) & 0xFFFF
    if t.element_size() == 4:
        return int(t.view(torch.int32).item()) & 0xFFFFFFFF
    return int(t.view(torch.int64).item()) & 0xFFFFFFFFFFFFFFFF


def _window_raw(src, window, out_len, pad_value):
    dev = _lib.require_device(src, window)
    s = src.contiguous()
    if s.element_size() not in (2, 4, 8):
        raise TypeError("unsupported element size %d" % s.element_size())
    batch, width = s.shape[0], s.shape[1]
    trailing = list(s.shape[2:])
    inner = 1
    for d in trailing:
        inner *= d
    out = torch.empty([batch, out_len] + trailing, dtype=s.dtype, device=dev)
    _lib.call("mrl_window_gather", _lib.ptr(s), s.element_size(), batch, width, inner, _lib.ptr(window),
              _lib.dtype_code(window), int(out_len), _pad_bits(s.dtype, pad_value), _lib.ptr(out), _lib.stream(dev))
    return out


def _window_tensor(truncate_lengths):
    w = truncate_lengths
    if w.dtype not in (torch.int32, torch.int64):
        w = w.to(torch.int64)
    if w.dim() != 2 or w.shape[1] != 2:
        raise ValueError("truncate_lengths must have shape (mbs, 2)")
    return w.contiguous()


def truncate_prompt_and_pad(responses, input_tensor, truncate_lengths, pad_value=0.0):
    """Reference: ``utils/pad_process.py:109-141``: ``[mbs, seq_len]`` -> ``[mbs, responses.shape[-1]]``,
    row i holding ``input_tensor[i, start_i:end_i]`` (window clamped to ``[0, seq_len]``).
    Differentiable for fp32 inputs."""
    if input_tensor.dim() != 2:
        raise ValueError("input_tensor must have shape (mbs, seq_len)")
    window = _window_tensor(truncate_lengths)
    out_len = responses.shape[-1]
    if input_tensor.requires_grad and torch.is_grad_enabled():
        if input_tensor.dtype != torch.float32:
            raise TypeError("gradients are supported for fp32 inputs only")
        return _WindowGather.apply(input_tensor, window, out_len, pad_value)
    return _window_raw(input_tensor, window, out_len, pad_value)


def truncate_middle_and_pad(responses, input_tensor, truncate_lengths, pad_value=0.0):
    """Reference: ``utils/pad_process.py:74-106``: ``[mbs, seq_len, vocab]`` ->
    ``[mbs, responses.shape[-1], vocab]``.  Differentiable for fp32 inputs with a last dimension of 1
    (the value head's output); wider inputs are forward only."""
    if input_tensor.dim() != 3:
        raise ValueError("input_tensor must have shape (mbs, seq_len, vocab_size)")
    window = _window_tensor(truncate_lengths)
    out_len = responses.shape[-1]
    if input_tensor.requires_grad and torch.is_grad_enabled():
        if input_tensor.shape[2] != 1 or input_tensor.dtype != torch.float32:
            raise TypeError("gradients are supported for fp32 inputs with a last dimension of 1 only")
        flat = input_tensor.reshape(input_tensor.shape[0], input_tensor.shape[1])
        return _WindowGather.apply(flat, window, out_len, pad_value).unsqueeze(-1)
    return _window_raw(input_tensor, window, out_len, pad_value)


def response_window(prompt_length, response_length):
    """``cat([P, P+R], dim=1) - 1`` (reference: ``models/loss/base_loss_func.py:47-53``)."""
    return torch.cat([prompt_length, prompt_length + response_length], dim=1) - 1

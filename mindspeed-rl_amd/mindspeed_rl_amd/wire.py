"""Ragged <-> padded experience columns: the on-wire layout either side of the loss path.

Host-side mirror of ``pack_experience_columns`` / ``unpack_pad_experience``
(``mindspeed_rl/trainer/utils/transfer_dock.py:1014-1198``) and ``truncate_rows`` (``mindspeed_rl/utils/pad_process.py:144-166``) with the
reference's signatures.  The reference walks the rows in Python with one or two ``.item()`` calls
per row; here each column costs one scan launch, one host read of two integers (to size the
output) and one gather launch.
"""
import torch

from . import _lib
from .packing import _pad_bits

_SCALAR_COLUMNS = ("prompt_length", "response_length", "age")


def _index(t):
    if t.dtype not in (torch.int32, torch.int64):
        t = t.to(torch.int64)
    return t.reshape(-1).contiguous()


def pack_padded_columns(padded, lengths, left_pad=False):
    """Device form of the packing step: ``padded`` maps column -> ``[B, W]`` tensor (4- or 8-byte
    elements), ``lengths`` column -> ``[B]`` or ``[B, 1]`` integer lengths.  Returns
    ``(batch_data, batch_data_length)`` in the layout of :func:`pack_experience_columns`: one flat
    tensor per column holding ``padded[i, :len_i]`` back to back (``padded[i, W - len_i:]`` with
    ``left_pad``) and the int32 lengths.  One scan launch, one host read (the total, to size the
    output) and one gather launch per column."""
    if not padded:
        raise ValueError("ERROR: when pack, get an empty experience_dict")
    if set(padded.keys()) != set(lengths.keys()):
        raise ValueError("ERROR: when pack, keys of the columns and of their lengths do not match")
    batch_data, batch_data_length = {}, {}
    for key, src in padded.items():
        dev = _lib.require_device(src)
        src = src.contiguous()
        if src.dim() != 2 or src.element_size() not in (4, 8):
            raise TypeError("pack_padded_columns takes [B, W] columns with 4- or 8-byte elements")
        batch, width = src.shape
        idx = _index(lengths[key].to(dev))
        if idx.numel() != batch:
            raise ValueError("ERROR: when pack, experience '%s' number=%d does not match experience_count=%d"
                             % (key, idx.numel(), batch))
        eff = torch.empty(batch, dtype=torch.int32, device=dev)
        cu = torch.empty(batch + 1, dtype=torch.int32, device=dev)
        info = torch.empty(2, dtype=torch.int64, device=dev)
        stream = _lib.stream(dev)
        _lib.call("mrl_ragged_layout", _lib.ptr(idx), _lib.dtype_code(idx), batch, 1, None, src.element_size(), width,
                  0, _lib.ptr(eff), _lib.ptr(cu), _lib.ptr(info), stream)
        total = int(info[0].item())
        flat = torch.empty(total, dtype=src.dtype, device=dev)
        _lib.call("mrl_padded_to_ragged", _lib.ptr(src), src.element_size(), batch, width, _lib.ptr(cu),
                  1 if left_pad else 0, total, _lib.ptr(flat), stream)
        batch_data[key] = flat
        batch_data_length[key] = eff
    return batch_data, batch_data_length


def pack_experience_columns(experience_consumer_stage, experience_dict, experience_count, enable_partial_rollout=False):
    """Mirror of ``pack_experience_columns`` (``trainer/utils/transfer_dock.py:1014-1089``) for lists of
    per-sample DEVICE tensors: one flat tensor per column (``[D, sum]`` for 2-D samples) plus int32
    lengths.  The samples are separate allocations, so the concatenation is the library's batched
    copy (``torch.cat``); the lengths come from the shapes, without a device read.  The reference
    goes through ``.tolist()`` for every sample."""
    if not experience_dict:
        raise ValueError("ERROR: when pack, get an empty experience_dict")
    if enable_partial_rollout and experience_consumer_stage == "actor_rollout":
        experience_count = len(experience_dict["prompts"])
    else:
        for key, value in experience_dict.items():
            if len(value) != experience_count:
                raise ValueError("ERROR: when pack, experience '%s' number=%d does not match experience_count=%d"
                                 % (key, len(value), experience_count))
    batch_data, batch_data_length = {}, {}
    for key, value in experience_dict.items():
        value = list(value[:experience_count])
        dev = _lib.require_device(value[0])
        if value[0].dim() > 1:
            first_dim = value[0].shape[0]
            if any(v.shape[0] != first_dim for v in value):
                raise ValueError("ERROR: when pack 2D tensor, first dimension must be the same for all experiences")
            batch_data[key] = torch.cat(value, dim=1)
            sizes = [v.shape[1] for v in value]
        else:
            batch_data[key] = torch.cat(value, dim=0)
            sizes = [v.shape[0] for v in value]
        batch_data_length[key] = torch.tensor(sizes, dtype=torch.int32).to(dev)
    return batch_data, batch_data_length


def unpack_pad_experience(batch_data, batch_data_length, pad_id, multiple):
    """Restores padded ``[B, max_len]`` columns (``[B, D, max_len]`` for 2-D columns such as mrope
    position ids) from flat packed columns and their per-sample lengths; ``max_len`` is rounded up
    to ``multiple``; floating columns are padded with 0.0, integer columns with ``pad_id``;
    ``prompt_length`` / ``response_length`` / ``age`` become ``[B, 1]`` views."""
    if not batch_data:
        raise ValueError("ERROR: empty batch_data")
    if set(batch_data.keys()) != set(batch_data_length.keys()):
        raise ValueError("ERROR: when unpack, keys from batch_data and batch_data_length dictionaries do not match")
    out = {}
    for key, length_list in batch_data_length.items():
        data = batch_data[key]
        if key in _SCALAR_COLUMNS:
            out[key] = data.view(-1, 1)
            continue
        dev = _lib.require_device(data)
        lengths = _index(length_list.to(dev))
        batch = lengths.numel()
        cu = torch.empty(batch + 1, dtype=torch.int32, device=dev)
        info = torch.empty(2, dtype=torch.int64, device=dev)
        stream = _lib.stream(dev)
        _lib.call("mrl_ragged_layout", _lib.ptr(lengths), _lib.dtype_code(lengths), batch, int(multiple), None, 0, 0, 0,
                  None, _lib.ptr(cu), _lib.ptr(info), stream)
        width = int(info[1].item())              # the one host read per column: sizes the output
        src = data.contiguous()
        if src.element_size() not in (2, 4, 8):
            raise TypeError("unsupported element size %d" % src.element_size())
        pad = 0.0 if src.is_floating_point() else pad_id
        if src.dim() > 1:
            first_dim, stride = src.shape[0], src.shape[1]
            result = torch.empty((batch, first_dim, width), dtype=src.dtype, device=dev)
        else:
            first_dim, stride = 1, src.shape[0]
            result = torch.empty((batch, width), dtype=src.dtype, device=dev)
        _lib.call("mrl_ragged_to_padded", _lib.ptr(src), src.element_size(), first_dim, stride, _lib.ptr(cu), batch,
                  width, _pad_bits(src.dtype, pad), _lib.ptr(result), stream)
        out[key] = result
    return out


def truncate_rows(tensor, index_tensor, left_pad=False):
    """``tensor`` ``[mbs, seq_len]`` (4- or 8-byte elements), ``index_tensor`` ``[mbs, 1]``: list of
    CPU rows ``tensor[i, :index_i]`` (``tensor[i, -index_i:]`` when ``left_pad``), an empty int32
    row where ``index_i == 0`` and ``tensor[i, 0] == -1``.  One packed device-to-host copy instead
    of one per row.  Negative indices are treated as 0."""
    dev = _lib.require_device(tensor)
    src = tensor.contiguous()
    if src.element_size() not in (4, 8):
        raise TypeError("truncate_rows supports 4- and 8-byte elements")
    batch, width = src.shape
    idx = _index(index_tensor.to(dev))
    eff = torch.empty(batch, dtype=torch.int32, device=dev)
    cu = torch.empty(batch + 1, dtype=torch.int32, device=dev)
    info = torch.empty(2, dtype=torch.int64, device=dev)
    stream = _lib.stream(dev)
    # the -1 marker is an integer convention; float rows are cut by the index alone
    rows_ptr = _lib.ptr(src) if not src.is_floating_point() else None
    _lib.call("mrl_ragged_layout", _lib.ptr(idx), _lib.dtype_code(idx), batch, 1, rows_ptr, src.element_size(), width,
              1 if left_pad else 0, _lib.ptr(eff), _lib.ptr(cu), _lib.ptr(info), stream)
    total = int(info[0].item())
    flat = torch.empty(total, dtype=src.dtype, device=dev)
    _lib.call("mrl_padded_to_ragged", _lib.ptr(src), src.element_size(), batch, width, _lib.ptr(cu),
              1 if left_pad else 0, total, _lib.ptr(flat), stream)
    host = flat.cpu()
    lens = eff.cpu().tolist()
    first = src[:, 0].cpu().tolist() if not src.is_floating_point() else [0] * batch
    idx_host = idx.cpu().tolist()
    rows, lo = [], 0
    for i, n in enumerate(lens):
        if idx_host[i] == 0 and first[i] == -1:
            rows.append(torch.tensor([], dtype=torch.int32))
        else:
            rows.append(host[lo:lo + n])
        lo += n
    return rows


def _ragged_to_padded(flat, sizes, width, pad, dev):
    """flat 1-D device tensor holding the samples back to back -> [n, width]."""
    n = len(sizes)
    cu = torch.zeros(n + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(torch.tensor(sizes, dtype=torch.int64), 0).to(torch.int32)
    cu = cu.to(dev)
    out = torch.empty((n, width), dtype=flat.dtype, device=dev)
    if flat.element_size() not in (2, 4, 8):
        raise TypeError("unsupported element size %d" % flat.element_size())
    _lib.call("mrl_ragged_to_padded", _lib.ptr(flat), flat.element_size(), 1, max(flat.shape[0], 1), _lib.ptr(cu), n,
              width, _pad_bits(flat.dtype, pad), _lib.ptr(out), _lib.stream(dev))
    return out


def pad_multiple(data_list, pad_id, multiple=1):
    """Reference: ``utils/pad_process.py:65-71``.  A list of 1-D device tensors -> ``[n, L]`` padded
    with ``pad_id``, ``L`` the longest sample rounded up to ``multiple``.  The lengths come from
    the shapes (no device read); one concatenation and one gather launch."""
    dev = _lib.require_device(data_list[0])
    sizes = [int(t.shape[0]) for t in data_list]
    width = (max(sizes) + multiple - 1) // multiple * multiple
    return _ragged_to_padded(torch.cat(list(data_list)).contiguous(), sizes, width, pad_id, dev)


def padding_dict_to_tensor_dict(experience_data):
    """Reference: ``utils/pad_process.py:13-25``, returning a plain dict (the reference wraps it in a
    TensorDict): each column, a list of 1-D device tensors, becomes a zero-padded ``[n, max_len]``
    tensor; ``original_length`` (int64, on the device) lists the sample lengths column after column."""
    batch, lengths, dev = {}, [], None
    for column, value in experience_data.items():
        dev = _lib.require_device(value[0])
        sizes = [int(t.shape[0]) for t in value]
        batch[column] = _ragged_to_padded(torch.cat(list(value)).contiguous(), sizes, max(sizes), 0, dev)
        lengths.extend(sizes)
    batch["original_length"] = torch.tensor(lengths, dtype=torch.int64).to(dev)
    return batch


def remove_padding_tensor_dict_to_dict(data_dict):
    """Reference: ``utils/pad_process.py:28-40``: the inverse of :func:`padding_dict_to_tensor_dict`,
    lists of CPU rows (see :func:`truncate_rows`)."""
    out = {}
    if data_dict is None:
        return out
    if "original_length" not in data_dict.keys():
        return data_dict
    data_lengths = data_dict["original_length"]
    for idx, (key, value) in enumerate(data_dict.items()):
        if key == "original_length":
            continue
        out[key] = truncate_rows(value, data_lengths[idx * len(value):(idx + 1) * len(value)])
    return out


def remove_padding_and_split_to_list(responses, eos_token_id, pad_token_id, to_list=False):
    """Reference: ``utils/pad_process.py:44-62``: every row of the integer ``[B, L]`` tensor cut at
    its first ``pad_token_id`` (the pad token itself is kept when it is also the end-of-sequence
    token).  Returns device tensors, or python lists without the last token when ``to_list``.  One
    search launch, one packing launch and one host read of the ``B`` lengths replace the
    reference's ``nonzero`` per row."""
    dev = _lib.require_device(responses)
    src = responses.contiguous()
    if src.dim() != 2 or src.is_floating_point() or src.element_size() not in (4, 8):
        raise TypeError("responses must be a [B, L] tensor of 4- or 8-byte integers")
    batch, width = src.shape
    first = torch.empty(batch, dtype=torch.int32, device=dev)
    stream = _lib.stream(dev)
    _lib.call("mrl_first_match", _lib.ptr(src), src.element_size(), batch, width, int(pad_token_id),
              1 if pad_token_id == eos_token_id else 0, _lib.ptr(first), stream)
    cu = torch.empty(batch + 1, dtype=torch.int32, device=dev)
    info = torch.empty(2, dtype=torch.int64, device=dev)
    _lib.call("mrl_ragged_layout", _lib.ptr(first), _lib.I32, batch, 1, None, src.element_size(), width, 0, None,
              _lib.ptr(cu), _lib.ptr(info), stream)
    lens = first.cpu().tolist()
    total = sum(lens)
    flat = torch.empty(total, dtype=src.dtype, device=dev)
    _lib.call("mrl_padded_to_ragged", _lib.ptr(src), src.element_size(), batch, width, _lib.ptr(cu), 0, total,
              _lib.ptr(flat), stream)
    if to_list:
        host = flat.cpu().tolist()
        out, lo = [], 0
        for n in lens:
            out.append(host[lo:lo + n][:-1])
            lo += n
        return out
    return list(torch.split(flat, lens))

"""Oracle (test infrastructure): remove-padding pack / unpack index maps and masks.

Pure integer logic, restated as the per-sequence Python loops the reference uses:

* ``mindspeed_rl/utils/remove_padding.py:10-87``   ``preprocess_packed_seqs``
* ``mindspeed_rl/utils/remove_padding.py:90-136``  ``postprocess_packed_seqs``
* ``mindspeed_rl/utils/pad_process.py:74-141``     ``truncate_middle_and_pad`` / ``truncate_prompt_and_pad``
* ``mindspeed_rl/utils/utils.py:57-67``            ``generate_mask``
* ``mindspeed_rl/models/loss/base_loss_func.py:47-53`` window ``[P-1, P+R-1)``

* ``mindspeed_rl/trainer/utils/transfer_dock.py:1092-1198``  ``unpack_pad_experience``
* ``mindspeed_rl/utils/pad_process.py:144-166``               ``truncate_rows``

Pinned by the reference-held vectors of ``tests/ut/utils/test_utils.py:22-28`` and
``tests/ut/utils/test_pad_process.py:48-62`` and by round-trip / brute-force properties.
"""
import torch


def generate_mask(data_pad, seq_lengths):
    """``utils/utils.py:57-67``: ``[B, data_pad.size(1)]`` int64, ones then trailing zeros."""
    width = data_pad.size(1)
    rows = []
    for n in seq_lengths.flatten().tolist():
        n_pad = width - n
        row = [1.0] * width
        if n_pad > 0:
            # python slice semantics of ``row[-n_pad:] = 0``: a length above ``width`` cannot
            # occur here (n_pad <= 0), a negative length zeroes at most the whole row
            for k in range(max(width - n_pad, 0), width):
                row[k] = 0.0
        rows.append(row)
    return torch.tensor(rows, dtype=torch.int64)


def preprocess_packed_seqs(input_ids, labels, attention_mask_1d, tp_size):
    """``utils/remove_padding.py:10-87``.

    Returns ``(ids[1,T], position_ids[1,T], labels[1,T], seqlens[B] int32, cu_seqlens_padded[B+1] int32)``.
    """
    batch, width = input_ids.shape
    if attention_mask_1d.shape != (batch, width):
        raise ValueError("attention_mask_1d must have shape (batch_size, seq_len) matching input_ids")
    seqlens = attention_mask_1d.sum(dim=1, dtype=torch.int32)
    pad = (tp_size - (seqlens % tp_size)) % tp_size
    padded = seqlens + pad
    cu_padded = torch.zeros(batch + 1, dtype=torch.int32)
    cu_padded[1:] = torch.cumsum(padded, dim=0)
    total = int(padded.sum().item())

    ids_packed = torch.zeros(total, dtype=input_ids.dtype)
    pos_packed = torch.zeros(total, dtype=torch.int32)
    labels_packed = torch.zeros(total, dtype=input_ids.dtype)
    for i in range(batch):
        lo = cu_padded[i].item()
        hi = cu_padded[i + 1].item()
        n = seqlens[i].item()
        ids_packed[lo:lo + n] = input_ids[i, :n]
        labels_packed[lo:lo + n] = labels[i, :n]
        pos_packed[lo:hi] = torch.arange(hi - lo, dtype=torch.int32)
    return (ids_packed.unsqueeze(0), pos_packed.unsqueeze(0), labels_packed.unsqueeze(0),
            seqlens, cu_padded)


def postprocess_packed_seqs(output, seqlens_in_batch, cu_seqlens_padded, seq_len, prompt_length=None):
    """``utils/remove_padding.py:90-136``: packed ``[1,T,...]`` -> ``[B,seq_len,...]``."""
    if output.shape[0] != 1:
        raise ValueError("Expected output tensor to have shape[0] == 1 (packed batch dimension)")
    batch = seqlens_in_batch.shape[0]
    unpacked = torch.zeros([batch, seq_len] + list(output.shape[2:]), dtype=output.dtype)
    for i in range(batch):
        lo = cu_seqlens_padded[i].item()
        n = seqlens_in_batch[i].item()
        if prompt_length is not None:
            skip = prompt_length[i].item() - 1
            if skip < n:
                n -= skip + 1
                lo += skip
        unpacked[i, :n] = output[0, lo:lo + n]
    return unpacked


def _window_copy(responses, input_tensor, truncate_lengths, pad_value, trailing):
    rows, width = input_tensor.shape[0], input_tensor.shape[1]
    window = torch.clamp(truncate_lengths, 0, width)
    out = torch.full((rows, responses.shape[-1]) + trailing, pad_value, dtype=input_tensor.dtype)
    for i in range(rows):
        lo = window[i, 0].item()
        hi = window[i, 1].item()
        out[i, :hi - lo] = input_tensor[i, lo:hi]
    return out


def truncate_prompt_and_pad(responses, input_tensor, truncate_lengths, pad_value=0.0):
    """``utils/pad_process.py:109-141``: ``[B,S]`` -> ``[B, responses.shape[-1]]``."""
    return _window_copy(responses, input_tensor, truncate_lengths, pad_value, ())


def truncate_middle_and_pad(responses, input_tensor, truncate_lengths, pad_value=0.0):
    """``utils/pad_process.py:74-106``: ``[B,S,V]`` -> ``[B, responses.shape[-1], V]``."""
    return _window_copy(responses, input_tensor, truncate_lengths, pad_value, (input_tensor.shape[2],))


def response_window(prompt_length, response_length):
    """``models/loss/base_loss_func.py:47-53``: ``cat([P, P+R], dim=1) - 1``."""
    return torch.cat([prompt_length, prompt_length + response_length], dim=1) - 1


def pack_experience_columns(experience_consumer_stage, experience_dict, experience_count, enable_partial_rollout=False):
    """``trainer/utils/transfer_dock.py:1014-1089``: lists of per-sample tensors -> one flat tensor per
    column (``[D, sum]`` for 2-D samples ``[D, n_i]``) plus int32 lengths."""
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
        if value[0].dim() > 1:
            first_dim = value[0].shape[0]
            for i in range(experience_count):
                if value[i].shape[0] != first_dim:
                    raise ValueError("ERROR: when pack 2D tensor, first dimension must be the same for all experiences")
            rows = [[x for i in range(experience_count) for x in value[i][d].tolist()] for d in range(first_dim)]
            batch_data[key] = torch.tensor(rows, dtype=value[0].dtype)
            batch_data_length[key] = torch.tensor([value[i].shape[1] for i in range(experience_count)],
                                                  dtype=torch.int32)
        else:
            flat, lengths = [], []
            for i in range(experience_count):
                flat.extend(value[i].tolist())
                lengths.append(len(value[i]))
            batch_data[key] = torch.tensor(flat, dtype=value[0].dtype)
            batch_data_length[key] = torch.tensor(lengths, dtype=torch.int32)
    return batch_data, batch_data_length


def unpack_pad_experience(batch_data, batch_data_length, pad_id, multiple):
    """``trainer/utils/transfer_dock.py:1092-1198``: flat packed columns + lengths -> padded columns."""
    if not batch_data:
        raise ValueError("ERROR: empty batch_data")
    if set(batch_data.keys()) != set(batch_data_length.keys()):
        raise ValueError("ERROR: when unpack, keys from batch_data and batch_data_length dictionaries do not match")
    out = {}
    for key, lengths in batch_data_length.items():
        if key in ("prompt_length", "response_length", "age"):
            out[key] = batch_data[key].view(-1, 1)
            continue
        data = batch_data[key]
        width = torch.max(lengths).item()
        if multiple > 1:
            width = ((width + multiple - 1) // multiple) * multiple
        fill = 0.0 if data.is_floating_point() else pad_id
        cum = torch.cat([torch.tensor([0]), torch.cumsum(lengths, 0)])
        if data.dim() > 1:
            padded = torch.full((len(lengths), data.shape[0], width), fill, dtype=data.dtype)
            for i in range(len(lengths)):
                n = lengths[i]
                for d in range(data.shape[0]):
                    padded[i, d, :n] = data[d, cum[i]:cum[i] + n]
        else:
            padded = torch.full((len(lengths), width), fill, dtype=data.dtype)
            for i in range(len(lengths)):
                padded[i, :lengths[i]] = data[cum[i]:cum[i + 1]]
        out[key] = padded
    return out


def truncate_rows(tensor, index_tensor, left_pad=False):
    """``utils/pad_process.py:144-166``: list of CPU rows cut at ``index_tensor``."""
    rows = []
    for i in range(tensor.shape[0]):
        if index_tensor[i].item() == 0 and tensor[i, 0].item() == -1:
            row = torch.tensor([], dtype=torch.int32).cpu()
        else:
            n = index_tensor[i].item()
            row = tensor[i, -n:].cpu() if left_pad else tensor[i, :n].cpu()
        rows.append(row)
    return rows


def pad_multiple(data_list, pad_id, multiple=1):
    """``utils/pad_process.py:65-71``: right-pad to the longest sample, rounded up to ``multiple``."""
    padded = torch.nn.utils.rnn.pad_sequence(data_list, batch_first=True, padding_value=pad_id)
    max_len = padded.size(1)
    target_len = ((max_len + multiple - 1) // multiple) * multiple
    return torch.nn.functional.pad(padded, (0, target_len - max_len), value=pad_id)


def remove_padding_and_split_to_list(responses, eos_token_id, pad_token_id, to_list=False):
    """``utils/pad_process.py:44-62``: cut every row at its first pad token (keeping it when the pad
    token is also the end-of-sequence token)."""
    output = []
    for i in range(responses.shape[0]):
        response = responses[i]
        nonzeros = torch.nonzero(response == pad_token_id, as_tuple=False)
        first_pad_index = nonzeros[0][0] if len(nonzeros) != 0 else len(response)
        response = response[:first_pad_index + 1] if pad_token_id == eos_token_id else response[:first_pad_index]
        if to_list:
            response = response[:-1].cpu().numpy().tolist()
        output.append(response)
    return output


def padding_dict_to_tensor_dict(experience_data):
    """``utils/pad_process.py:13-25`` with a plain dict in place of the TensorDict: every column
    (a list of 1-D samples) becomes a zero-padded ``[n, max_len]`` tensor; ``original_length`` holds
    the sample lengths column after column."""
    batch, lengths = {}, []
    for column, value in experience_data.items():
        max_length = max(len(exp) for exp in value)
        batch[column] = torch.stack([torch.nn.functional.pad(exp, (0, max_length - len(exp)), mode="constant", value=0)
                                     for exp in value], dim=0)
        lengths.extend([torch.tensor(len(exp)) for exp in value])
    batch["original_length"] = torch.stack(lengths)
    return batch


def remove_padding_tensor_dict_to_dict(data_dict):
    """``utils/pad_process.py:28-40``."""
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

"""Oracle for the padded-layout helpers around the per-step Experience fields. Test
infrastructure, CPU torch."""
import torch
import torch.nn.functional as F


def zero_pad_sequences(sequences, side="left", value=0, stack=False):
    """openrlhf/utils/utils.py:93-106: pad every tensor's last dimension to the longest, then
    stack or concatenate along dimension 0."""
    assert side in ("left", "right")
    max_len = max(seq.size(-1) for seq in sequences)
    padded = []
    for seq in sequences:
        pad_len = max_len - seq.size(-1)
        padding = (pad_len, 0) if side == "left" else (0, pad_len)
        padded.append(F.pad(seq, padding, value=value))
    return torch.stack(padded, dim=0) if stack else torch.cat(padded, dim=0)


def unpadded_length(attention_mask_row):
    """Length remove_padding_in_sequences keeps of one sample's per-step fields
    (openrlhf/trainer/ppo_utils/experience.py:236-247): everything but the trailing zeros of
    the attention mask (``flip(0).argmax()`` of them)."""
    right_pad = int(attention_mask_row.flip(0).argmax())
    return attention_mask_row.numel() - right_pad


def unpad_boundaries(attention_mask):
    """cu_seqlens as flash-attn's unpad_input reports them for a [B, T] attention mask
    (openrlhf/models/ring_attn_utils.py:129-140): cumulative count of attended tokens per row."""
    lens = attention_mask.long().sum(dim=-1)
    return torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)])


def unpad_and_rebatch(field, attention_mask):
    """One per-step field of a batch after the reference's hops split_experience_batch ->
    remove_padding_in_sequences -> make_experience_batch
    (openrlhf/trainer/ppo_utils/experience.py:164-247): every row loses as many trailing columns
    as its attention-mask row has trailing zeros (none if the mask row is all zeros or ends in a
    one: ``right_pad == 0 -> None``), then the rows are right-padded with 0 to the longest and
    stacked. Returns (batch, kept lengths)."""
    rows, kept = [], []
    for value, mask_row in zip(field, attention_mask):
        right_pad = int(mask_row.flip(0).argmax())
        rows.append(value[: -right_pad] if right_pad else value)
        kept.append(rows[-1].numel())
    return zero_pad_sequences(rows, "right", 0, stack=True), kept


def unpad_and_slice_tensor(sequences, attention_mask):
    """unpad_and_slice_tensor with ring_attn_group=None (openrlhf/models/ring_attn_utils.py:103-148).

    It calls unpad_input / index_first_axis of flash-attn 2.8.3 (flash_attn/bert_padding.py, a
    dependency that is not in the reference tree); restated from its published definition:
    ``indices = nonzero(attention_mask.flatten())``, ``seqlens = attention_mask.sum(-1)``,
    ``cu_seqlens = pad(cumsum(seqlens), (1, 0))``, ``index_first_axis(x, indices) = x[indices]``
    on the flattened ``(b s)`` axis. Returns what the reference returns, plus cu_seqlens:
    (sequences [1, Ttot], position_ids [1, Ttot], rolled_sequences [1, Ttot], 0, indices, cu_seqlens).
    Pins: the reference's own docstring example (:112-118) and a cell-by-cell loop, in
    tests/test_oracle_pins.py."""
    rolled = torch.roll(sequences, shifts=-1, dims=1)  # :129
    indices = torch.nonzero(attention_mask.flatten(), as_tuple=False).flatten()
    seqlens = attention_mask.sum(dim=-1, dtype=torch.int32)
    cu_seqlens = F.pad(torch.cumsum(seqlens, dim=0, dtype=torch.int32), (1, 0))
    packed = sequences.reshape(-1)[indices].unsqueeze(0)  # :130-131
    rolled = rolled.reshape(-1)[indices].unsqueeze(0)  # :132-136
    position_ids = torch.clip(torch.cumsum(attention_mask, dim=-1) - 1, min=0, max=None)  # :137
    position_ids = position_ids.reshape(-1)[indices].unsqueeze(0)  # :138-140
    return packed, position_ids, rolled, 0, indices, cu_seqlens


def gather_and_pad_tensor(tensor, indices, batch, seqlen):
    """gather_and_pad_tensor with ring_attn_group=None (openrlhf/models/ring_attn_utils.py:151-182):
    flash-attn's pad_input on the transposed [Ttot, 1] tensor, i.e. zeros of batch * seqlen rows
    with ``output[indices] = input``, reshaped to [batch, seqlen]."""
    values = tensor.transpose(0, 1)  # [Ttot, 1] or [Ttot, ...]
    out = torch.zeros(batch * seqlen, *values.shape[1:], dtype=values.dtype)
    out[indices] = values
    return out.view(batch, seqlen, *values.shape[1:]).squeeze(-1)

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

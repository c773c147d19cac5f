"""Sequence padding with the signature of ``openrlhf.utils.utils.zero_pad_sequences``."""
from typing import List

import torch

from ..trainer.ppo_utils.experience import pad_packed
from ..trainer.ppo_utils.experience_maker import _gpu_device


def zero_pad_sequences(sequences: List[torch.Tensor], side: str = "left", value: int = 0,
                       stack: bool = False) -> torch.Tensor:
    """Pads tensors that differ in their last dimension to the longest one on ``side`` and stacks
    (new leading dimension) or concatenates them along dimension 0
    (openrlhf/utils/utils.py:93-106). One gather of the inputs plus one kernel instead of one
    ``F.pad`` per sequence; row lengths come from the shapes, nothing is read back. CPU tensors
    (the reference pads on the controller) are gathered, copied to the current GPU in one piece,
    padded there and copied back."""
    assert side in ("left", "right")
    if not sequences:
        raise ValueError("max() arg is an empty sequence")
    lead = sequences[0].shape[:-1]
    if stack and any(s.shape[:-1] != lead for s in sequences):
        raise RuntimeError("stack expects each tensor to be equal size apart from the last dimension")
    if any(s.dim() != sequences[0].dim() or s.shape[1:-1] != sequences[0].shape[1:-1] for s in sequences):
        raise RuntimeError("Sizes of tensors must match except in the first and last dimension")
    dtype = sequences[0].dtype
    for s in sequences[1:]:
        dtype = torch.promote_types(dtype, s.dtype)
    max_len = max(s.size(-1) for s in sequences)
    lengths, rows_per = [], []
    for s in sequences:
        rows = s.numel() // s.size(-1) if s.size(-1) else (int(torch.tensor(s.shape[:-1]).prod()) if s.dim() > 1 else 1)
        rows_per.append(rows)
        lengths.extend([s.size(-1)] * rows)
    home = sequences[0].device
    dev = home if home.type == "cuda" else _gpu_device()
    flat = torch.cat([s.reshape(-1).to(dtype) for s in sequences]).to(dev)
    cu = torch.tensor([0] + lengths, dtype=torch.int64).cumsum(0).to(dev)
    out = pad_packed(flat, cu, max_len, side, value).to(home)
    if stack:
        return out.view(len(sequences), *lead, max_len)
    inner = sequences[0].shape[1:-1]
    if sequences[0].dim() == 1:
        # torch.cat of 1-D padded tensors is one long vector
        return out.reshape(-1)
    return out.view(-1, *inner, max_len)

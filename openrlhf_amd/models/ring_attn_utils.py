"""The unpadding around the packed model forward, on one GPU.

Mirrors ``unpad_and_slice_tensor`` and ``gather_and_pad_tensor`` of
openrlhf/models/ring_attn_utils.py:103-182 for ``ring_attn_group=None`` (one GPU: no slicing of
the packed row among ranks, no all-gather). The reference goes through flash-attn's
``unpad_input`` / ``index_first_axis`` / ``pad_input`` and eight eager launches; here the
non-zero positions of the attention mask are ranked inside one kernel and every output is written
from there. The one host read is the total number of attended tokens, which sizes the outputs
(the reference's ``nonzero`` does the same read); ``total_tokens=`` skips it.
"""
from typing import Optional

import torch

from .. import _lib
from .._lib import call, ptr, require_gpu, stream_of


def _no_ring(ring_attn_group):
    if ring_attn_group is not None:
        raise NotImplementedError("one GPU: ring_attn_group must be None")


def _count(mptr, mcode, batch, seqlen, dev):
    """One pass over the mask: cu_seqlens [B + 1] and the attended columns of every (row, tile)."""
    cu = torch.empty(batch + 1, dtype=torch.int64, device=dev)
    counts = torch.empty(max(batch, 1), dtype=torch.int64, device=dev)
    n_tiles = (seqlen + _lib.UNPAD_TILE - 1) // _lib.UNPAD_TILE
    tiles = torch.empty(max(batch * n_tiles, 1), dtype=torch.int32, device=dev)
    with _lib.on_device(dev):
        st = stream_of(dev)
        call("orlhf_mask_row_counts", mptr, mcode, batch, seqlen, ptr(counts), ptr(tiles), st)
        call("orlhf_cu_seqlens", ptr(counts), batch, ptr(cu), st)
    return cu, tiles


def unpad_and_slice_tensor(sequences: torch.Tensor, attention_mask: torch.Tensor, ring_attn_group=None,
                           total_tokens: Optional[int] = None, return_cu_seqlens: bool = False):
    """``(sequences [1, Ttot], position_ids [1, Ttot], rolled_sequences [1, Ttot], 0, indices [Ttot])``
    of the attended positions of ``sequences [B, T]`` in row-major order, as the reference returns
    them; with ``return_cu_seqlens`` the int64 ``cu_seqlens [B + 1]`` is appended. The attention
    mask holds zeros and ones (any placement of the ones)."""
    _no_ring(ring_attn_group)
    dev = require_gpu(sequences, attention_mask)
    if sequences.dim() != 2 or attention_mask.shape != sequences.shape:
        raise ValueError(f"sequences {tuple(sequences.shape)} and attention_mask {tuple(attention_mask.shape)} must be the same [B, T]")
    batch, seqlen = sequences.shape
    seqs = sequences.to(torch.int64).contiguous()
    mkeep, mptr, mcode = _lib.mask_arg(attention_mask)
    cu, tiles = _count(mptr, mcode, batch, seqlen, dev)
    total = int(cu[-1]) if total_tokens is None else int(total_tokens)
    out = torch.empty(4, max(total, 1), dtype=torch.int64, device=dev)
    if total > 0:
        with _lib.on_device(dev):
            call("orlhf_unpad_sequences", ptr(seqs), mptr, mcode, batch, seqlen, ptr(cu), ptr(tiles), total, ptr(out[0]),
                 ptr(out[1]), ptr(out[2]), ptr(out[3]), stream_of(dev))
    indices, packed, rolled, position_ids = (out[i, :total] for i in range(4))
    packed = packed.to(sequences.dtype).unsqueeze(0)
    rolled = rolled.to(sequences.dtype).unsqueeze(0)
    result = (packed, position_ids.unsqueeze(0), rolled, 0, indices)
    return result + (cu,) if return_cu_seqlens else result


def unpad_indices(attention_mask: torch.Tensor, total_tokens: Optional[int] = None) -> torch.Tensor:
    """Flat positions of the attended tokens in row-major order: the ``indices`` flash-attn's
    unpad_input returns (openrlhf/models/ring_attn_utils.py:130)."""
    dev = require_gpu(attention_mask)
    if attention_mask.dim() != 2:
        raise ValueError(f"attention_mask must be [B, T], got {tuple(attention_mask.shape)}")
    batch, seqlen = attention_mask.shape
    mkeep, mptr, mcode = _lib.mask_arg(attention_mask)
    cu, tiles = _count(mptr, mcode, batch, seqlen, dev)
    total = int(cu[-1]) if total_tokens is None else int(total_tokens)
    indices = torch.empty(max(total, 1), dtype=torch.int64, device=dev)
    if total > 0:
        with _lib.on_device(dev):
            call("orlhf_unpad_sequences", None, mptr, mcode, batch, seqlen, ptr(cu), ptr(tiles), total, ptr(indices), None,
                 None, None, stream_of(dev))
    return indices[:total]


class _PadByIndices(torch.autograd.Function):
    """zeros(n_dst, ...) with rows ``indices`` set to ``values``; the gradient is the gather of
    those rows (flash-attn's IndexPutFirstAxis)."""

    @staticmethod
    def forward(ctx, values, indices, n_dst):
        dev = values.device
        n = values.shape[0]
        inner = 1
        for d in values.shape[1:]:
            inner *= d
        out = torch.empty((n_dst,) + tuple(values.shape[1:]), dtype=values.dtype, device=dev)
        with _lib.on_device(dev):
            call("orlhf_pad_by_indices", ptr(values), values.element_size(), n, max(inner, 1), ptr(indices), n_dst,
                 ptr(out), stream_of(dev))
        ctx.save_for_backward(indices)
        return out

    @staticmethod
    def backward(ctx, g):
        (indices,) = ctx.saved_tensors
        g = g.contiguous()
        inner = 1
        for d in g.shape[1:]:
            inner *= d
        out = torch.empty((indices.numel(),) + tuple(g.shape[1:]), dtype=g.dtype, device=g.device)
        with _lib.on_device(g.device):
            call("orlhf_gather_by_indices", ptr(g), g.element_size(), g.shape[0], max(inner, 1), ptr(indices),
                 indices.numel(), ptr(out), stream_of(g.device))
        return out, None, None


def gather_and_pad_tensor(tensor: torch.Tensor, ring_attn_group, ring_attn_pad_len, indices: torch.Tensor,
                          batch: int, seqlen: int) -> torch.Tensor:
    """``[1, Ttot, ...]`` per-token values back on the ``[batch, seqlen]`` grid: zeros, then
    position ``indices[i]`` receives token i (flash-attn's pad_input, as
    openrlhf/models/ring_attn_utils.py:181 applies it to the transposed ``[Ttot, 1, ...]`` tensor,
    followed by ``.squeeze(-1)``: ``[1, Ttot]`` gives ``[batch, seqlen]``, ``[1, Ttot, V]`` gives
    ``[batch, seqlen, 1, V]`` as in the reference). Differentiable in ``tensor``."""
    _no_ring(ring_attn_group)
    if ring_attn_pad_len:
        raise NotImplementedError("one GPU: ring_attn_pad_len must be 0")
    require_gpu(tensor, indices)
    if tensor.dim() < 2 or tensor.shape[0] != 1:
        raise ValueError(f"expected a packed [1, Ttot, ...] tensor, got {tuple(tensor.shape)}")
    values = tensor[0].contiguous()
    if indices.numel() != values.shape[0]:
        raise ValueError(f"{values.shape[0]} packed tokens but {indices.numel()} indices")
    if values.element_size() not in (1, 2, 4, 8):
        raise TypeError(f"unsupported dtype {values.dtype}")
    out = _PadByIndices.apply(values, indices.to(torch.int64).contiguous(), batch * seqlen)
    return out.view(batch, seqlen, 1, *values.shape[1:]).squeeze(-1)

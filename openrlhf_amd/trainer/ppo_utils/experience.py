"""Packed layout of the per-step Experience fields on hand-written HIP kernels.

The reference keeps every per-step field as a right-padded ``[B, A]`` tensor plus masks
(openrlhf/trainer/ppo_utils/experience.py:29-69) and re-pads at every hop:
``make_experience_batch`` (:199-233) pads single samples with ``zero_pad_sequences(..., "right",
stack=True)``, ``remove_padding_in_sequences`` (:236-247) strips the padding again per sample from
``attention_mask.flip(0).argmax()``. The per-token kernels of this library take the packed form
(flat tokens + ``cu_seqlens``) directly, so a batch can be packed once and stay packed through
reward shaping, GAE, whitening and the losses. This module holds the conversions, all index work
on the GPU and bit-exact: row extents of a mask, ``cu_seqlens``, pack and pad.
"""
from dataclasses import dataclass, field
from typing import Dict, Optional, Tuple

import torch

from ... import _lib
from ..._lib import call, ptr, require_gpu, stream_of

_BITS = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}


def _fill_bits(value, dtype: torch.dtype) -> int:
    """The bit pattern of ``value`` in ``dtype`` as an unsigned integer."""
    t = torch.tensor(value, dtype=dtype)
    width = t.element_size()
    return int(t.view(_BITS[width]).item()) & ((1 << (8 * width)) - 1)


def row_extents(mask: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(first, end, length) per row of a ``[B, A]`` mask: first non-zero column (A if none), one
    past the last non-zero column (0 if none) and their difference. For a right-padded row,
    ``length`` is what ``remove_padding_in_sequences`` keeps."""
    dev = require_gpu(mask)
    if mask.dim() != 2:
        raise ValueError(f"mask must be [B, A], got {tuple(mask.shape)}")
    n_rows, n_cols = mask.shape
    mkeep, mptr, mcode = _lib.mask_arg(mask)
    first = torch.empty(n_rows, dtype=torch.int64, device=dev)
    end, length = torch.empty_like(first), torch.empty_like(first)
    with torch.cuda.device(dev):
        call("orlhf_row_extents", mptr, mcode, n_rows, n_cols, ptr(first), ptr(end), ptr(length), stream_of(dev))
    return first, end, length


def cu_seqlens_of(lengths: torch.Tensor) -> torch.Tensor:
    """int64 ``[B+1]`` boundaries ``[0, l0, l0+l1, ...]`` of rows of the given lengths."""
    dev = require_gpu(lengths)
    lens = lengths.reshape(-1).to(torch.int64).contiguous()
    cu = torch.empty(lens.numel() + 1, dtype=torch.int64, device=dev)
    with torch.cuda.device(dev):
        call("orlhf_cu_seqlens", ptr(lens), lens.numel(), ptr(cu), stream_of(dev))
    return cu


def pack_padded(x: torch.Tensor, cu_seqlens: torch.Tensor, first: Optional[torch.Tensor] = None,
                total: Optional[int] = None) -> torch.Tensor:
    """Flat ``[total]`` tensor holding, row after row, columns ``first[b] .. first[b]+len_b-1`` of
    the padded ``x [B, A]`` (``first`` defaults to 0: right-padded rows). ``total`` is the packed
    length ``cu_seqlens[-1]``; pass it when it is known on the host, otherwise it is read back
    (one synchronisation)."""
    dev = require_gpu(x, cu_seqlens, first)
    if x.dim() != 2 or cu_seqlens.numel() != x.shape[0] + 1:
        raise ValueError(f"x {tuple(x.shape)} needs cu_seqlens of {x.shape[0] + 1} entries, got {cu_seqlens.numel()}")
    if x.element_size() not in _BITS:
        raise ValueError(f"unsupported element size {x.element_size()}")
    src = x.contiguous()
    total = int(cu_seqlens[-1]) if total is None else int(total)
    out = torch.empty(total, dtype=x.dtype, device=dev)
    cu = cu_seqlens.to(torch.int64).contiguous()
    f = None if first is None else first.to(torch.int64).contiguous()
    with torch.cuda.device(dev):
        call("orlhf_pack_rows", ptr(src), src.element_size(), x.shape[0], x.shape[1], ptr(f), ptr(cu), ptr(out),
             stream_of(dev))
    return out


def pad_packed(flat: torch.Tensor, cu_seqlens: torch.Tensor, n_cols: int, side: str = "right", value=0) -> torch.Tensor:
    """``[B, n_cols]`` tensor whose row b holds tokens ``cu[b] .. cu[b+1]-1`` of ``flat`` with
    ``value`` as padding on ``side`` — ``zero_pad_sequences(rows, side, value, stack=True)``
    (openrlhf/utils/utils.py:93-106) without materialising the rows."""
    if side not in ("left", "right"):
        raise AssertionError("side must be 'left' or 'right'")
    dev = require_gpu(flat, cu_seqlens)
    if flat.element_size() not in _BITS:
        raise ValueError(f"unsupported element size {flat.element_size()}")
    src = flat.reshape(-1).contiguous()
    n_rows = cu_seqlens.numel() - 1
    cu = cu_seqlens.to(torch.int64).contiguous()
    out = torch.empty(n_rows, int(n_cols), dtype=flat.dtype, device=dev)
    with torch.cuda.device(dev):
        call("orlhf_pad_rows", ptr(src), src.element_size(), ptr(cu), n_rows, int(n_cols), 1 if side == "left" else 0,
             _fill_bits(value, flat.dtype), ptr(out), stream_of(dev))
    return out


@dataclass
class PackedSteps:
    """Per-step fields of a batch in the packed layout: every tensor in ``fields`` is flat
    ``[total]`` and row b is ``cu_seqlens[b] .. cu_seqlens[b+1]-1``. ``first`` and ``n_cols``
    remember where the rows sat in the padded ``[B, n_cols]`` grid."""

    cu_seqlens: torch.Tensor
    first: torch.Tensor
    n_cols: int
    total: int
    fields: Dict[str, torch.Tensor] = field(default_factory=dict)

    @classmethod
    def from_padded(cls, fields: Dict[str, Optional[torch.Tensor]], mask: torch.Tensor,
                    total: Optional[int] = None) -> "PackedSteps":
        """Packs every ``[B, A]`` tensor of ``fields`` over the extent of ``mask``'s rows (first to
        last non-zero column; interior zeros are kept, so pack the mask itself as a field when it
        has holes). ``None`` entries are carried through."""
        first, _, length = row_extents(mask)
        cu = cu_seqlens_of(length)
        total = int(cu[-1]) if total is None else int(total)
        packed = {k: (None if v is None else pack_padded(v, cu, first, total)) for k, v in fields.items()}
        return cls(cu, first, mask.shape[1], total, packed)

    @property
    def max_seqlen(self) -> int:
        """A bound on the longest row, known without reading anything back: the padded width."""
        return self.n_cols

    def to_padded(self, name: str, side: str = "right", value=0) -> torch.Tensor:
        """The named field back as a right- (or left-) padded ``[B, n_cols]`` tensor."""
        return pad_packed(self.fields[name], self.cu_seqlens, self.n_cols, side, value)

    def __getitem__(self, name: str) -> torch.Tensor:
        return self.fields[name]

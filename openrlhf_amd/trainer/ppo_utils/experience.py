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
    with _lib.on_device(dev):
        call("orlhf_row_extents", mptr, mcode, n_rows, n_cols, ptr(first), ptr(end), ptr(length), stream_of(dev))
    return first, end, length


def cu_seqlens_of(lengths: torch.Tensor) -> torch.Tensor:
    """int64 ``[B+1]`` boundaries ``[0, l0, l0+l1, ...]`` of rows of the given lengths."""
    dev = require_gpu(lengths)
    lens = lengths.reshape(-1).to(torch.int64).contiguous()
    cu = torch.empty(lens.numel() + 1, dtype=torch.int64, device=dev)
    with _lib.on_device(dev):
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
    if total == 0:  # every row is empty: nothing to copy (and no destination to hand over)
        return out
    cu = cu_seqlens.to(torch.int64).contiguous()
    f = None if first is None else first.to(torch.int64).contiguous()
    with _lib.on_device(dev):
        call("orlhf_pack_rows", ptr(src), src.element_size(), x.shape[0], x.shape[1], ptr(f), ptr(cu), ptr(out),
             stream_of(dev))
    return out


def pack_padded_fields(fields: Dict[str, Optional[torch.Tensor]], cu_seqlens: torch.Tensor,
                       first: Optional[torch.Tensor], total: int) -> Dict[str, Optional[torch.Tensor]]:
    """``pack_padded`` of every ``[B, A]`` tensor in ``fields`` (``None`` entries are carried through)
    with one launch per eight fields instead of one per field."""
    live = {k: v for k, v in fields.items() if v is not None}
    out: Dict[str, Optional[torch.Tensor]] = {k: None for k in fields}
    if not live:
        return out
    dev = require_gpu(cu_seqlens, first, *live.values())
    shape = next(iter(live.values())).shape
    for k, v in live.items():
        if v.dim() != 2 or v.shape != shape or cu_seqlens.numel() != shape[0] + 1:
            raise ValueError(f"field {k}: {tuple(v.shape)} against {tuple(shape)} and {cu_seqlens.numel()} boundaries")
        if v.element_size() not in _BITS:
            raise ValueError(f"unsupported element size {v.element_size()}")
    srcs = {k: v.contiguous() for k, v in live.items()}
    for k, v in srcs.items():
        out[k] = torch.empty(total, dtype=v.dtype, device=dev)
    if total == 0:
        return out
    cu = cu_seqlens.to(torch.int64).contiguous()
    f = None if first is None else first.to(torch.int64).contiguous()
    arr = (_lib.PackField * len(srcs))()
    for i, (k, v) in enumerate(srcs.items()):
        arr[i].src, arr[i].dst, arr[i].elem_bytes = v.data_ptr(), out[k].data_ptr(), v.element_size()
    with _lib.on_device(dev):
        call("orlhf_pack_rows_multi", arr, len(srcs), shape[0], shape[1], ptr(f), ptr(cu), stream_of(dev))
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
    with _lib.on_device(dev):
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
        packed = pack_padded_fields(fields, cu, first, total)
        return cls(cu, first, mask.shape[1], total, packed)

    @property
    def max_seqlen(self) -> int:
        """A bound on the longest row, known without reading anything back: the padded width."""
        return self.n_cols

    @property
    def longest_first(self) -> torch.Tensor:
        """The rows ordered by decreasing length (int64 [B], computed once per batch): what the
        one-workgroup-per-row scans take as ``row_order`` so that a ragged batch does not end on a
        single long row's walk."""
        order = getattr(self, "_longest_first", None)
        if order is None:
            lengths = self.cu_seqlens[1:] - self.cu_seqlens[:-1]
            order = torch.argsort(lengths, descending=True, stable=True)
            object.__setattr__(self, "_longest_first", order)
        return order

    def to_padded(self, name: str, side: str = "right", value=0) -> torch.Tensor:
        """The named field back as a right- (or left-) padded ``[B, n_cols]`` tensor."""
        return pad_packed(self.fields[name], self.cu_seqlens, self.n_cols, side, value)

    def __getitem__(self, name: str) -> torch.Tensor:
        return self.fields[name]


# ---------------------------------------------------------------------------------------------
# The Experience container (openrlhf/trainer/ppo_utils/experience.py:29-283) with the reference's
# field names and batch helpers. Per-step fields are [B, T] / [B, A] tensors padded on the right,
# per-episode fields are [B]; everything else is per-sample metadata. Padding and un-padding go
# through the row kernels above; `packed()` hands the per-step fields to the per-token kernels in
# the packed layout.
# ---------------------------------------------------------------------------------------------
import itertools
from dataclasses import fields as _dc_fields
from typing import Any, List

STEP_FIELDS = ("sequences", "attention_mask", "action_mask", "action_log_probs", "base_action_log_probs",
               "rollout_log_probs", "values", "returns", "advantages", "kl")
EPISODE_FIELDS = ("rewards", "scores", "response_length", "truncated", "total_length")


def _map_tensors(value, fn):
    """fn applied to every tensor inside a tensor / list / dict value; anything else is returned as is."""
    if isinstance(value, torch.Tensor):
        return fn(value)
    if isinstance(value, list):
        return [_map_tensors(v, fn) for v in value]
    if isinstance(value, dict):
        return {k: _map_tensors(v, fn) for k, v in value.items()}
    return value


def _pad_rows(tensors: List[torch.Tensor], value, stack: bool) -> torch.Tensor:
    from ...utils.utils import zero_pad_sequences

    return zero_pad_sequences(tensors, side="right", value=value, stack=stack)


@dataclass
class Experience:
    """One batch of rollout data (openrlhf/trainer/ppo_utils/experience.py:29-69)."""

    sequences: Optional[torch.Tensor] = None            # (B, T) prompt + response token ids
    attention_mask: Optional[torch.Tensor] = None       # (B, T)
    action_mask: Optional[torch.Tensor] = None          # (B, A)
    action_log_probs: Optional[torch.Tensor] = None     # (B, A) current policy
    base_action_log_probs: Optional[torch.Tensor] = None  # (B, A) reference policy
    rollout_log_probs: Optional[torch.Tensor] = None    # (B, A) rollout engine
    values: Optional[torch.Tensor] = None               # (B, A)
    returns: Optional[torch.Tensor] = None              # (B, A)
    advantages: Optional[torch.Tensor] = None           # (B, A)
    kl: Optional[torch.Tensor] = None                   # (B, A)
    rewards: Optional[torch.Tensor] = None              # (B,)
    scores: Optional[torch.Tensor] = None               # (B,)
    response_length: Optional[torch.Tensor] = None      # (B,)
    truncated: Optional[torch.Tensor] = None            # (B,)
    total_length: Optional[torch.Tensor] = None         # (B,)
    index: Optional[List[int]] = None
    prompts: list = field(default_factory=list)
    labels: list = field(default_factory=list)
    images: list = field(default_factory=list)
    mm_train_inputs: list = field(default_factory=list)
    info: dict = field(default_factory=dict)

    @classmethod
    def is_step_tensor_field(cls, name: str) -> bool:
        return name in STEP_FIELDS

    @classmethod
    def is_episode_tensor_field(cls, name: str) -> bool:
        return name in EPISODE_FIELDS

    @torch.no_grad()
    def to_device(self, device) -> "Experience":
        for f in _dc_fields(self):
            setattr(self, f.name, _map_tensors(getattr(self, f.name), lambda t: t.to(device)))
        return self

    def pin_memory(self) -> "Experience":
        for f in _dc_fields(self):
            setattr(self, f.name, _map_tensors(getattr(self, f.name), lambda t: t.pin_memory()))
        return self

    @staticmethod
    def _merge_item(items: List, pad_value: int = 0) -> Any:
        """Tensors of differing width are right-padded and concatenated along the batch; lists are
        chained; dicts are merged key by key (experience.py:103-129)."""
        head = items[0]
        if isinstance(head, torch.Tensor):
            return _pad_rows(items, pad_value, stack=False)
        if isinstance(head, list):
            return list(itertools.chain.from_iterable(items))
        if isinstance(head, dict):
            keys = []
            for d in items:
                keys.extend(k for k in d if k not in keys)
            return {k: Experience._merge_item([d[k] for d in items if k in d], pad_value) for k in keys}
        if head is None:
            return None
        raise ValueError(f"Unsupported type: {type(head)}")

    @staticmethod
    def concat_experiences(experiences_list: List["Experience"], pad_token_id) -> "Experience":
        """All batches as one; token ids are padded with ``pad_token_id``, everything else with 0
        (experience.py:131-158)."""
        if not experiences_list:
            return Experience()
        merged = {}
        for f in _dc_fields(Experience):
            pad = pad_token_id if f.name == "sequences" else 0
            merged[f.name] = Experience._merge_item([getattr(e, f.name) for e in experiences_list], pad)
        return Experience(**merged)

    def packed(self, names=None, total: Optional[int] = None) -> PackedSteps:
        """The ``[B, A]`` per-step fields (``names``: default every one that is set) packed over the
        extent of the action mask, for the per-token kernels' ``cu_seqlens`` form."""
        width = self.action_mask.shape[1]
        if names is None:
            names = [n for n in STEP_FIELDS if getattr(self, n) is not None and getattr(self, n).shape[1:] == (width,)]
        return PackedSteps.from_padded({n: getattr(self, n) for n in names}, self.action_mask, total=total)


def split_experience_batch(experience: Experience) -> List[Experience]:
    """One single-sample Experience per row of the batch (experience.py:164-196)."""
    batch_size = len(experience.sequences)
    experience.index = None

    def row_of(name, value, i):
        if value is None:
            return None
        if isinstance(value, torch.Tensor):
            if len(value) != batch_size:
                raise ValueError(f"Size of {name} ({len(value)}) does not match batch_size ({batch_size})")
            return value[i]
        if isinstance(value, dict):
            out = {}
            for k, v in value.items():
                if not isinstance(v, (torch.Tensor, list)):
                    raise TypeError(f"Unsupported type for {name}[{k}]: {type(v)}")
                if len(v) != batch_size:
                    raise ValueError(f"Size of {name}[{k}] ({len(v)}) does not match batch_size ({batch_size})")
                out[k] = v[i]
            return out
        if isinstance(value, list):
            return [value[i]] if len(value) == batch_size else value
        return value

    return [Experience(**{f.name: row_of(f.name, getattr(experience, f.name), i) for f in _dc_fields(Experience)})
            for i in range(batch_size)]


def make_experience_batch(items: List[Experience], packing_samples=False) -> Experience:
    """Single-sample Experiences back into one batch: per-step tensors are right-padded with 0 and
    stacked, per-episode tensors stacked, numeric info entries become tensors, lists are chained
    (experience.py:199-233)."""
    if not items:
        raise ValueError("Empty items list")
    batch = {}
    for f in _dc_fields(Experience):
        values = [getattr(it, f.name) for it in items]
        head = values[0]
        if head is None:
            batch[f.name] = None
        elif isinstance(head, torch.Tensor):
            if Experience.is_step_tensor_field(f.name):
                batch[f.name] = _pad_rows(values, 0, stack=True)
            elif Experience.is_episode_tensor_field(f.name) or head.dim() == 0:
                batch[f.name] = torch.stack(values)
            else:
                raise ValueError(f"Unsupported tensor field batching rule for {f.name}")
        elif isinstance(head, dict):
            out = {}
            for key in head:
                vals = [v[key] for v in values]
                kind = type(vals[0])
                if not all(isinstance(v, kind) for v in vals):
                    raise TypeError(f"Inconsistent types in {f.name}[{key}]")
                out[key] = torch.tensor(vals) if all(isinstance(v, (int, float)) for v in vals) else vals
            batch[f.name] = out
        elif isinstance(head, list):
            batch[f.name] = list(itertools.chain.from_iterable(values))
    return Experience(**batch)


def remove_padding_in_sequences(items: List[Experience]) -> List[Experience]:
    """Per-step fields of single-sample Experiences cut after the last attended position: what
    ``attention_mask.flip(0).argmax()`` trailing zeros remove (experience.py:236-247). The cut
    lengths of all samples come from one extent kernel over the stacked masks when they share a
    width, else sample by sample."""
    if not items:
        return items
    masks = [it.attention_mask for it in items]
    if all(m.is_cuda for m in masks) and len({m.numel() for m in masks}) == 1:
        _, end, _ = row_extents(torch.stack(masks))
        keep = end.tolist()
    else:
        keep = [m.numel() - int(m.flip(0).argmax()) for m in masks]
    for it, mask, n in zip(items, masks, keep):
        pad = mask.numel() - (n if n > 0 else mask.numel())  # an all-zero mask keeps everything (argmax 0)
        if pad == 0:
            continue
        for name in STEP_FIELDS:
            value = getattr(it, name)
            if isinstance(value, torch.Tensor):
                setattr(it, name, value[:-pad])
    return items


def gather_packed_rows(flat: torch.Tensor, src_start: torch.Tensor, cu_seqlens: torch.Tensor, max_len: int,
                       total: int) -> torch.Tensor:
    """Rows picked out of a packed array: output row b (``cu_seqlens[b] .. cu_seqlens[b+1]-1`` of
    the result) holds the elements of ``flat`` from ``src_start[b]`` on. ``max_len`` bounds the row
    lengths, ``total`` is ``cu_seqlens[-1]``."""
    dev = require_gpu(flat, src_start, cu_seqlens)
    if flat.element_size() not in _BITS:
        raise ValueError(f"unsupported element size {flat.element_size()}")
    src = flat.reshape(-1).contiguous()
    out = torch.empty(int(total), dtype=flat.dtype, device=dev)
    n_rows = cu_seqlens.numel() - 1
    if total == 0 or n_rows == 0:
        return out
    with _lib.on_device(dev):
        call("orlhf_gather_rows", ptr(src), src.element_size(), n_rows, int(max_len),
             ptr(src_start.to(torch.int64).contiguous()), ptr(cu_seqlens.to(torch.int64).contiguous()), ptr(out),
             stream_of(dev))
    return out


@dataclass
class PackedExperience:
    """A batch whose per-step fields stay packed between the rollout and the training step.

    The reference moves a rollout batch to the trainer as ``split_experience_batch`` ->
    ``remove_padding_in_sequences`` -> (replay buffer) -> ``make_experience_batch``
    (openrlhf/trainer/ppo_utils/experience.py:164-247): every hop slices or pads each field of each
    sample. Here the batch is packed once (``from_experience``): every per-step field is one flat
    tensor holding, row after row, what ``remove_padding_in_sequences`` keeps of it (everything but
    the columns behind the last attended token), with one ``cu_seqlens`` per field width (``T`` for
    ``sequences`` / ``attention_mask``, ``A`` for the action fields). The per-token kernels take
    these tensors as they are (``actions()`` is a ``PackedSteps``); ``select`` hands out any rows as
    a new packed batch (a replay buffer's micro-batch) with one gather launch per field;
    ``to_experience`` is the padded batch ``make_experience_batch`` would have built from the same
    samples."""

    steps: Dict[str, torch.Tensor]          # name -> flat tensor
    widths: Dict[str, int]                  # name -> width of the padded field it came from
    cu: Dict[int, torch.Tensor]             # width -> int64 [B+1] boundaries
    totals: Dict[int, int]                  # width -> cu[width][-1]
    episode: Dict[str, torch.Tensor] = field(default_factory=dict)   # [B] tensors
    meta: Dict[str, Any] = field(default_factory=dict)               # index / prompts / labels / images / mm_train_inputs / info

    def __len__(self) -> int:
        return next(iter(self.cu.values())).numel() - 1 if self.cu else 0

    @classmethod
    def from_experience(cls, exp: "Experience") -> "PackedExperience":
        att = exp.attention_mask
        if att is None or att.dim() != 2:
            raise ValueError("a batched Experience with an attention_mask [B, T] is needed")
        t = att.shape[1]
        _, end, _ = row_extents(att)
        keep_t = torch.where(end > 0, end, torch.full_like(end, t))  # an all-zero mask keeps everything (argmax 0)
        steps, widths, cu, totals = {}, {}, {}, {}
        for name in STEP_FIELDS:
            value = getattr(exp, name)
            if value is None:
                continue
            if value.dim() != 2 or value.shape[0] != att.shape[0]:
                raise ValueError(f"{name} must be [B, width], got {tuple(value.shape)}")
            w = value.shape[1]
            if w not in cu:
                lengths = (keep_t - (t - w)).clamp_(min=0)  # the same number of trailing columns goes
                cu[w] = cu_seqlens_of(lengths)
                totals[w] = int(cu[w][-1])
            steps[name] = pack_padded(value, cu[w], None, totals[w])
            widths[name] = w
        episode = {n: getattr(exp, n) for n in EPISODE_FIELDS if getattr(exp, n) is not None}
        meta = {n: getattr(exp, n) for n in ("index", "prompts", "labels", "images", "mm_train_inputs", "info")}
        return cls(steps, widths, cu, totals, episode, meta)

    def actions(self, names=None) -> PackedSteps:
        """The action-wide fields (the width of ``action_mask``) as a ``PackedSteps``: what the
        per-token kernels take with ``cu_seqlens=``."""
        w = self.widths["action_mask"]
        names = [n for n, wn in self.widths.items() if wn == w] if names is None else names
        first = torch.zeros(len(self), dtype=torch.int64, device=self.cu[w].device)
        return PackedSteps(self.cu[w], first, w, self.totals[w], {n: self.steps[n] for n in names})

    def set_step(self, name: str, flat: torch.Tensor, like: str = "action_mask") -> None:
        """Adds or replaces a per-step field computed in the packed layout (advantages, returns, kl)."""
        w = self.widths[like]
        if flat.numel() != self.totals[w]:
            raise ValueError(f"{name}: {flat.numel()} elements, the packed fields of width {w} hold {self.totals[w]}")
        self.steps[name], self.widths[name] = flat.reshape(-1), w

    def select(self, rows) -> "PackedExperience":
        """The given rows (a list of ints; any order, repeats allowed) as a new packed batch."""
        rows = [int(r) for r in rows]
        n = len(self)
        if any(r < -n or r >= n for r in rows):
            raise IndexError(f"row index out of range for a batch of {n}")
        rows = [r % n for r in rows]
        dev = next(iter(self.cu.values())).device
        idx = torch.tensor(rows, dtype=torch.int64, device=dev)
        cu, totals, starts = {}, {}, {}
        for w, old in self.cu.items():
            starts[w] = old[idx]
            cu[w] = cu_seqlens_of(old[idx + 1] - starts[w])
            totals[w] = int(cu[w][-1])
        steps = {name: gather_packed_rows(flat, starts[self.widths[name]], cu[self.widths[name]], self.widths[name],
                                          totals[self.widths[name]])
                 for name, flat in self.steps.items()}
        episode = {n_: v[idx.to(v.device)] for n_, v in self.episode.items()}

        def pick(value):
            if isinstance(value, list):
                return [value[r] for r in rows] if len(value) == n else value
            if isinstance(value, torch.Tensor):
                return value[idx.to(value.device)] if value.dim() > 0 and len(value) == n else value
            if isinstance(value, dict):
                return {k: pick(v) for k, v in value.items()}
            return value

        return PackedExperience(steps, dict(self.widths), cu, totals, episode, {k: pick(v) for k, v in self.meta.items()})

    @staticmethod
    def concat(batches: List["PackedExperience"]) -> "PackedExperience":
        """Several packed batches as one (rows in the order given)."""
        if not batches:
            raise ValueError("Empty batch list")
        head = batches[0]
        if any(b.widths.keys() != head.widths.keys() for b in batches):
            raise ValueError("batches hold different per-step fields")
        # a field's width only bounds its rows: the joint batch takes the largest
        cu, totals, width_of = {}, {}, {}
        for name in head.widths:
            width_of[name] = max(b.widths[name] for b in batches)
        for name, w in width_of.items():
            if w in cu:
                continue
            parts, offset = [head.cu[head.widths[name]][:1]], 0
            for b in batches:
                c = b.cu[b.widths[name]]
                parts.append(c[1:] + offset)
                offset += b.totals[b.widths[name]]
            cu[w], totals[w] = torch.cat(parts), offset
        steps = {name: torch.cat([b.steps[name] for b in batches]) for name in head.widths}
        episode = {n_: torch.cat([b.episode[n_] for b in batches]) for n_ in head.episode}
        meta = {k: Experience._merge_item([b.meta[k] for b in batches]) if head.meta.get(k) is not None else None
                for k in head.meta}
        return PackedExperience(steps, width_of, cu, totals, episode, meta)

    def to_experience(self, widths: Optional[Dict[int, int]] = None) -> "Experience":
        """The padded batch ``make_experience_batch`` builds from the un-padded samples: every
        per-step field right-padded with 0 to its longest row. ``widths`` (packed width -> padded
        width) saves reading the longest row back. Fields added with ``set_step`` under a name the
        Experience does not have stay behind."""
        out = {}
        for name, flat in self.steps.items():
            if name not in STEP_FIELDS:  # a working field of the packed batch, no Experience attribute
                continue
            w = self.widths[name]
            c = self.cu[w]
            n_cols = widths[w] if widths is not None and w in widths else (int((c[1:] - c[:-1]).max()) if len(self) else 0)
            out[name] = pad_packed(flat, c, n_cols, "right", 0)
        out.update(self.episode)
        out.update({k: v for k, v in self.meta.items() if v is not None})
        return Experience(**out)


def balance_experiences(experiences, args):
    """Spreads long and short sequences evenly over the data-parallel ranks by pairing chunks of
    the length-sorted samples from both ends (experience.py:250-283)."""
    samples = [s for exp in experiences for s in split_experience_batch(exp)]
    samples.sort(key=lambda s: s.total_length, reverse=True)
    width = args.actor.num_nodes * args.actor.num_gpus_per_node // args.ds.ring_attn_size // args.ds.tensor_parallel_size
    chunks = [samples[i: i + width] for i in range(0, len(samples), width)]
    half = len(chunks) // 2
    front, back = chunks[:half], [c[::-1] for c in chunks[half:]]
    order = []
    for i in range(half):
        order += [front[i], back[-(i + 1)]]
    if len(back) > len(front):
        order.append(back[0])
    columns = itertools.zip_longest(*order)
    return [make_experience_batch([s for s in col if s is not None]) for col in columns]

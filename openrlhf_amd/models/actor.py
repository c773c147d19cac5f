"""The numerics tail of ``Actor.forward`` as one fused call.

Mirrors what openrlhf/models/actor.py:265-296 does after the model has produced logits:
(fp32 up-cast,) entropy on the unscaled logits, log-prob of the next token on logits/T, re-pad
of packed outputs with the unpadding indices (openrlhf/models/ring_attn_utils.py:129-140,181),
drop of the last column, slice of the last A columns, multiplication by the action mask.

Differences by construction: bf16 logits are consumed directly (no [N, V] fp32 copy), log-prob
and entropy come from ONE pass over the logits, and with ``skip_masked=True`` (default) positions
whose log-prob the reference multiplies by zero are not read at all, forward or backward; their
entropy is returned as 0 (the trainer only ever aggregates entropy under the same mask,
openrlhf/trainer/ray/ppo_actor.py:345-350). ``actor_forward_tail_from_hidden`` starts one step
earlier, at the decoder's last hidden states, and never stores the logits.
"""
from typing import Optional, Tuple, Union

import torch

from .utils import logprobs_and_entropy_from_logits


from .ring_attn_utils import gather_and_pad_tensor, unpad_indices  # noqa: F401  (unpad_indices is part of this module's API)


def actor_forward_tail(
    logits: torch.Tensor,
    sequences: torch.Tensor,
    action_mask: Optional[torch.Tensor] = None,
    attention_mask: Optional[torch.Tensor] = None,
    temperature: float = 1.0,
    packed_indices: Optional[torch.Tensor] = None,
    return_entropy: bool = False,
    inplace_backward: bool = False,
    skip_masked: bool = True,
) -> Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
    """Action log-probs ``[B, A]`` (or all ``[B, T-1]`` log-probs when ``action_mask`` is None)
    from the model's logits, plus ``entropy[:, :-1]`` when ``return_entropy``.

    logits: ``[B, T, V]`` (padded batch) or ``[1, Ttot, V]`` / ``[Ttot, V]`` with
    ``packed_indices`` = the flat positions of the packed tokens in the ``[B, T]`` grid
    (``unpad_indices(attention_mask)``). sequences: ``[B, T]`` token ids; labels are the sequences
    rolled left by one per padded row, as in the reference.
    """
    batch, seqlen = sequences.shape
    rolled = torch.roll(sequences, shifts=-1, dims=1)

    # which (b, t) positions are needed: the last A of the first T-1 columns, under the action mask
    need = torch.zeros(batch, seqlen, dtype=torch.bool, device=sequences.device)
    if action_mask is not None:
        width = action_mask.shape[1]
        need[:, seqlen - 1 - width : seqlen - 1] = action_mask != 0
    else:
        need[:, : seqlen - 1] = True if attention_mask is None else attention_mask[:, : seqlen - 1] != 0
    if not skip_masked:
        need = None

    if packed_indices is None:
        labels = rolled
        row_mask = need
        lp, ent = logprobs_and_entropy_from_logits(
            logits, labels, temperature, inplace_backward=inplace_backward, row_mask=row_mask
        ) if return_entropy else (_lp_only(logits, labels, temperature, inplace_backward, row_mask), None)
    else:
        from .utils import _index_rows

        flat_logits = logits.reshape(-1, logits.shape[-1])
        idx = packed_indices.to(torch.int64).contiguous()
        labels = _index_rows(rolled.reshape(-1).to(torch.int64), idx)
        row_mask = None if need is None else _index_rows(need.reshape(-1).to(torch.uint8), idx)
        if return_entropy:
            lp_p, ent_p = logprobs_and_entropy_from_logits(
                flat_logits, labels, temperature, inplace_backward=inplace_backward, row_mask=row_mask
            )
        else:
            lp_p, ent_p = _lp_only(flat_logits, labels, temperature, inplace_backward, row_mask), None
        lp = gather_and_pad_tensor(lp_p.unsqueeze(0), None, 0, idx, batch, seqlen)
        ent = None if ent_p is None else gather_and_pad_tensor(ent_p.unsqueeze(0), None, 0, idx, batch, seqlen)

    lp = lp[:, :-1]
    if action_mask is not None:
        lp = lp[:, -action_mask.shape[1] :] * action_mask.float()
    if return_entropy:
        return lp, ent[:, :-1]
    return lp


def actor_forward_tail_from_hidden(
    hidden_states: torch.Tensor,
    lm_head_weight: torch.Tensor,
    sequences: torch.Tensor,
    action_mask: Optional[torch.Tensor] = None,
    attention_mask: Optional[torch.Tensor] = None,
    temperature: float = 1.0,
    packed_indices: Optional[torch.Tensor] = None,
    return_entropy: bool = False,
    skip_masked: bool = True,
    keep_logits_mib: Optional[float] = None,
) -> Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
    """The same tail with the lm-head projection in front and the logits never stored: what
    openrlhf/models/actor.py:263-296 computes from ``self.model(...)["logits"]``, from the decoder's
    last hidden states ``[B, T, H]`` (or ``[1, Ttot, H]`` / ``[Ttot, H]`` with ``packed_indices``)
    and ``lm_head.weight [V, H]`` (bf16 or fp16). With ``skip_masked=True`` (default) positions
    whose log-prob the reference multiplies by zero (outside the action mask; with
    ``action_mask=None`` the last column and the positions outside the attention mask) are left out
    of the projection altogether: their log-prob and entropy are returned as 0 and they get no
    gradient. ``skip_masked=False`` projects every row, which is what reproduces the reference's
    values at padded positions when ``action_mask`` is None. Gradients reach the hidden states and
    the weight. Same outputs and shapes as ``actor_forward_tail``."""
    from .utils import _index_rows, lm_head_logprobs_and_entropy

    batch, seqlen = sequences.shape
    rolled = torch.roll(sequences, shifts=-1, dims=1)
    need = None
    if skip_masked:
        need = torch.zeros(batch, seqlen, dtype=torch.bool, device=sequences.device)
        if action_mask is not None:
            width = action_mask.shape[1]
            need[:, seqlen - 1 - width : seqlen - 1] = action_mask != 0
        else:
            need[:, : seqlen - 1] = True if attention_mask is None else attention_mask[:, : seqlen - 1] != 0
    if packed_indices is None:
        lp, ent = lm_head_logprobs_and_entropy(hidden_states, lm_head_weight, rolled, temperature, row_mask=need,
                                               keep_logits_mib=keep_logits_mib)
    else:
        flat = hidden_states.reshape(-1, hidden_states.shape[-1])
        idx = packed_indices.to(torch.int64).contiguous()
        labels = _index_rows(rolled.reshape(-1).to(torch.int64), idx)
        row_mask = None if need is None else _index_rows(need.reshape(-1).to(torch.uint8), idx)
        lp_p, ent_p = lm_head_logprobs_and_entropy(flat, lm_head_weight, labels, temperature, row_mask=row_mask,
                                                   keep_logits_mib=keep_logits_mib)
        lp = gather_and_pad_tensor(lp_p.unsqueeze(0), None, 0, idx, batch, seqlen)
        ent = gather_and_pad_tensor(ent_p.unsqueeze(0), None, 0, idx, batch, seqlen)
    lp = lp[:, :-1]
    if action_mask is not None:
        lp = lp[:, -action_mask.shape[1] :] * action_mask.float()
    if return_entropy:
        return lp, ent[:, :-1]
    return lp


def _lp_only(logits, labels, temperature, inplace_backward, row_mask):
    from .utils import _LogprobEntropy

    return _LogprobEntropy.apply(logits, labels, temperature, True, False, inplace_backward, row_mask)[0]

"""The sequence-level numerics of the DPO training step on hand-written HIP kernels.

Mirrors openrlhf/trainer/dpo_trainer.py:306-382 (``concatenated_forward`` after the model call,
``concatenated_inputs``, ``_get_batch_logps``) and the loss assembly at :168-180. The loss mask of
``_get_batch_logps`` (attention mask with the prompt cleared, shifted by one) is built inside the
kernel from the attention mask and the prompt lengths: no clone, no per-row Python loop.
"""
from typing import Sequence, Union

import torch

from .. import _lib
from .._lib import call, ptr, require_gpu, stream_of
from ..models.actor import actor_forward_tail, actor_forward_tail_from_hidden
from ..models.loss import DPOLoss
from ..models.utils import _f32


def _prompt_lens(prompt_id_lens, n_rows, dev):
    if prompt_id_lens is None:
        return None
    t = torch.as_tensor(prompt_id_lens, dtype=torch.int64).reshape(-1).to(dev)
    if t.numel() != n_rows:
        raise ValueError(f"{t.numel()} prompt lengths for {n_rows} sequences")
    return t.contiguous()


class _SequenceLogps(torch.autograd.Function):
    @staticmethod
    def forward(ctx, per_token_logps, attention_mask, prompt_lens):
        dev = require_gpu(per_token_logps, attention_mask, prompt_lens)
        lp = _f32(per_token_logps)
        if lp.dim() != 2 or attention_mask.shape != (lp.shape[0], lp.shape[1] + 1):
            raise ValueError(f"per_token_logps {tuple(per_token_logps.shape)} needs an attention mask of one more "
                             f"column, got {tuple(attention_mask.shape)}")
        n_rows, n_cols = lp.shape
        mkeep, mptr, mcode = _lib.mask_arg(attention_mask)
        sums = torch.empty(n_rows, dtype=torch.float32, device=dev)
        means, counts = torch.empty_like(sums), torch.empty_like(sums)
        with _lib.on_device(dev):
            call("orlhf_sequence_logps_fwd", ptr(lp), mptr, mcode, ptr(prompt_lens), n_rows, n_cols, ptr(sums),
                 ptr(means), ptr(counts), stream_of(dev))
        ctx.save_for_backward(mkeep, prompt_lens, counts)
        ctx.cfg = (mcode, n_rows, n_cols, per_token_logps.dtype)
        return sums, means

    @staticmethod
    def backward(ctx, g_sums, g_means):
        mkeep, prompt_lens, counts = ctx.saved_tensors
        mcode, n_rows, n_cols, dtype = ctx.cfg
        dev = counts.device
        gs, gm = _f32(g_sums), _f32(g_means)
        g = torch.empty(n_rows, n_cols, dtype=torch.float32, device=dev)
        with _lib.on_device(dev):
            call("orlhf_sequence_logps_bwd", ptr(gs), ptr(gm), ptr(mkeep), mcode, ptr(prompt_lens), ptr(counts),
                 n_rows, n_cols, ptr(g), stream_of(dev))
        return g.to(dtype), None, None


def get_batch_logps(per_token_logps: torch.Tensor, attention_mask: torch.Tensor,
                    prompt_id_lens: Union[Sequence[int], torch.Tensor, None]):
    """(sum, mean) of the per-token log-probs ``[B, T-1]`` over each sequence's response tokens
    (openrlhf/trainer/dpo_trainer.py:362-382): token t counts when ``attention_mask[b, t+1]`` is
    set and ``t+1 >= prompt_id_lens[b]``. A sequence without response tokens has mean NaN."""
    dev = require_gpu(per_token_logps, attention_mask)
    return _SequenceLogps.apply(per_token_logps, attention_mask,
                                _prompt_lens(prompt_id_lens, per_token_logps.shape[0], dev))


def response_mask(attention_mask: torch.Tensor, prompt_id_lens) -> torch.Tensor:
    """The ``[B, T-1]`` loss mask ``get_batch_logps`` applies, as a bool tensor."""
    cols = torch.arange(1, attention_mask.shape[1], device=attention_mask.device)[None, :]
    lens = torch.as_tensor(prompt_id_lens, dtype=torch.int64).reshape(-1, 1).to(attention_mask.device)
    return (attention_mask[:, 1:] != 0) & (cols >= lens)


def concatenated_inputs(chosen_ids, c_mask, reject_ids, r_mask, prompt_id_lens, pad_token_id: int):
    """Chosen and rejected batches right-padded to a common length and stacked along the batch
    (openrlhf/trainer/dpo_trainer.py:328-360); prompt lengths are repeated for both halves."""

    def pad_to(t, length, value):
        if t.size(-1) >= length:
            return t
        return torch.nn.functional.pad(t, (0, length - t.size(-1)), value=value)

    length = max(chosen_ids.shape[1], reject_ids.shape[1])
    input_ids = torch.cat((pad_to(chosen_ids, length, pad_token_id), pad_to(reject_ids, length, pad_token_id)), dim=0)
    length = max(c_mask.shape[1], r_mask.shape[1])
    att_masks = torch.cat((pad_to(c_mask, length, 0), pad_to(r_mask, length, 0)), dim=0)
    if isinstance(prompt_id_lens, torch.Tensor):
        lens = torch.cat((prompt_id_lens.reshape(-1), prompt_id_lens.reshape(-1)))
    else:
        lens = list(prompt_id_lens) * 2
    return input_ids, att_masks, lens


def concatenated_logps(logits, input_ids, att_masks, prompt_id_lens, n_chosen: int, temperature: float = 1.0,
                       inplace_backward: bool = False, lm_head_weight=None):
    """What ``concatenated_forward`` returns after the model call (dpo_trainer.py:314-326):
    ``(chosen_logps, rejected_logps, nll_loss)`` from the logits of the stacked batch, where
    ``nll_loss = -mean(per-sequence mean log-prob of the chosen half)``. Only response positions
    are read from the logits. With ``lm_head_weight [V, H]`` the first argument holds the decoder's
    last hidden states and the projection is fused in (logits never stored)."""
    need = response_mask(att_masks, prompt_id_lens)
    if lm_head_weight is not None:
        lp = actor_forward_tail_from_hidden(logits, lm_head_weight, input_ids, action_mask=need, temperature=temperature)
    else:
        lp = actor_forward_tail(logits, input_ids, action_mask=need, temperature=temperature,
                                inplace_backward=inplace_backward)
    sums, means = get_batch_logps(lp, att_masks, prompt_id_lens)
    return sums[:n_chosen], sums[n_chosen:], -means[:n_chosen].mean()


def dpo_loss_step(logits, input_ids, att_masks, prompt_id_lens, n_chosen: int, reference_chosen_logps,
                  reference_rejected_logps, loss_fn: DPOLoss, nll_loss_coef: float = 0.0,
                  temperature: float = 1.0, inplace_backward: bool = False, lm_head_weight=None):
    """Policy half of the DPO step (dpo_trainer.py:157-180) from the stacked batch's logits:
    returns a dict with ``loss = preference_loss + nll_loss * nll_loss_coef`` (the Mixtral
    auxiliary loss is the caller's), the preference loss, both reward estimates and the NLL."""
    chosen, rejected, nll = concatenated_logps(logits, input_ids, att_masks, prompt_id_lens, n_chosen,
                                               temperature=temperature, inplace_backward=inplace_backward,
                                               lm_head_weight=lm_head_weight)
    preference_loss, chosen_reward, reject_reward = loss_fn(chosen, rejected, reference_chosen_logps,
                                                            reference_rejected_logps)
    loss = preference_loss + nll * nll_loss_coef if nll_loss_coef else preference_loss
    return dict(loss=loss, preference_loss=preference_loss, chosen_reward=chosen_reward,
                reject_reward=reject_reward, nll_loss=nll, chosen_logps=chosen, rejected_logps=rejected)

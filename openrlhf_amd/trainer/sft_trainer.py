"""The loss part of the SFT training step on hand-written HIP kernels.

Mirrors openrlhf/trainer/sft_trainer.py:161-179 between the model call and ``strategy.backward``:
per-token log-probs of the next token (``Actor.forward(return_logprobs=True)``,
openrlhf/models/actor.py:265-296) and ``SFTLoss`` over ``loss_mask[:, :-1]`` with the
``loss_batch_info`` normalisers (openrlhf/utils/loss_utils.py:15-105).

``sft_loss_step(..., fused=False)`` is an ordinary autograd graph on the separate kernels.
``fused=True`` uses that the SFT loss is linear in the log-probs with weights known before the
pass (``-mask * aggregation weight``): ONE pass over the logits returns the log-probs and writes
d(loss)/d(logits) over the logits. Positions outside the loss mask are neither read nor computed
in either mode.
"""
import torch

from ..models.actor import actor_forward_tail, actor_forward_tail_from_hidden
from ..models.loss import SFTLoss
from ..models.utils import fused_logprob_entropy_fwd_bwd
from .ray.ppo_actor import _HandOverGradient, _row_coef


def sft_loss_step(logits, inputs, attention_mask, loss_mask, loss_fn: SFTLoss = None, fused: bool = False,
                  dp_size=1, batch_num_tokens=None, global_batch_size=None, loss_scale: float = 1.0,
                  inplace_backward: bool = False, lm_head_weight=None):
    """logits ``[B, T, V]``, inputs / attention_mask / loss_mask ``[B, T]``. Returns
    ``(gpt_loss, per_token_log_probs [B, T-1])``. With ``fused=True`` the logits are consumed (their
    storage holds ``loss_scale * d(gpt_loss)/d(logits)``) and ``(gpt_loss * loss_scale).backward()``
    hands that gradient to the layer that produced them. With ``lm_head_weight [V, H]`` the first
    argument holds the decoder's last hidden states ``[B, T, H]`` and the projection is fused into
    the log-probs (logits never stored; ``fused`` does not apply)."""
    loss_fn = loss_fn if loss_fn is not None else SFTLoss()
    info = dict(dp_size=dp_size, batch_num_tokens=batch_num_tokens, global_batch_size=global_batch_size)
    shifted = loss_mask[:, :-1]
    batch, seqlen = inputs.shape
    if lm_head_weight is not None:
        lp = actor_forward_tail_from_hidden(logits, lm_head_weight, inputs, action_mask=(shifted != 0), temperature=1.0)
        return loss_fn(lp, shifted, **info), lp
    if not fused:
        # log-probs are needed where the loss mask is set; the attention mask only marks padding
        lp = actor_forward_tail(logits, inputs, action_mask=(shifted != 0), temperature=1.0,
                                inplace_backward=inplace_backward)
        return loss_fn(lp, shifted, **info), lp

    with torch.no_grad():
        norm = batch_num_tokens if loss_fn.token_level_loss else global_batch_size
        coef = _row_coef(shifted, loss_fn.token_level_loss, dp_size, norm)[:batch, None] * shifted.to(torch.float32)  # [B, T-1], 0 off the mask
        w = torch.zeros(batch, seqlen, dtype=torch.float32, device=logits.device)
        w[:, : seqlen - 1] = -coef * loss_scale
        need = torch.zeros(batch, seqlen, dtype=torch.uint8, device=logits.device)
        need[:, : seqlen - 1] = shifted != 0
        labels = torch.roll(inputs, shifts=-1, dims=1)
        lp_all, _, grad = fused_logprob_entropy_fwd_bwd(logits, labels, w_logprob=w, inplace=True, row_mask=need)
        lp = lp_all[:, : seqlen - 1] * (shifted != 0).float()
        loss = loss_fn(lp, shifted, **info)
    if logits.requires_grad:
        loss = _HandOverGradient.apply(logits, loss, grad, loss_scale)
    return loss, lp

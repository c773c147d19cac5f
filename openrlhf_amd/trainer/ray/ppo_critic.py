"""The loss assembly of the PPO critic training step on hand-written HIP kernels.

Mirrors openrlhf/trainer/ray/ppo_critic.py:151-176 (CriticPPOTrainer.training_step between the
critic forward and strategy.backward): the clipped value loss over the action columns, the
auxiliary loss term, their sum, and the two statuses that depend on per-token data
(``critic_loss`` and the masked mean of the values). The value loss and the mean of the values
come out of ONE pass over ``values`` / ``old_values`` / ``returns`` / ``action_mask`` (13 bytes
per token) instead of the reference's two chains of eager kernels.

Not mirrored: the critic model forward, the optimizer step, the learning-rate and gradient-norm
statuses.
"""
from ...models.loss import ValueLoss


def critic_loss_step(values, old_values, returns, action_mask, critic_loss_fn: ValueLoss, aux_loss=0,
                     aux_loss_coef=0.0, dynamic_loss_scale=None, dp_size=1, batch_num_tokens=None,
                     global_batch_size=None, cu_seqlens=None, max_seqlen=None):
    """Returns ``{"loss", "critic_loss", "values_mean"}``: ``loss = critic_loss + aux_loss *
    aux_loss_coef [* dynamic_loss_scale]`` is what the caller hands to ``strategy.backward``
    (ppo_critic.py:160-169; the dynamic-batch scale multiplies the auxiliary term only, as
    there); ``critic_loss.detach()`` and ``values_mean`` are the statuses of ppo_critic.py:173-174,
    left on the device (no ``.item()`` synchronisation here). ``dp_size`` / ``batch_num_tokens`` /
    ``global_batch_size`` are the ``loss_batch_info`` of openrlhf/utils/loss_utils.py:15-52."""
    critic_loss, values_mean = critic_loss_fn.loss_and_values_mean(
        values, old_values, returns, action_mask=action_mask, dp_size=dp_size, batch_num_tokens=batch_num_tokens,
        global_batch_size=global_batch_size, cu_seqlens=cu_seqlens, max_seqlen=max_seqlen)
    aux = aux_loss * aux_loss_coef
    if dynamic_loss_scale is not None:
        aux = aux * dynamic_loss_scale
    return {"loss": critic_loss + aux, "critic_loss": critic_loss, "values_mean": values_mean}

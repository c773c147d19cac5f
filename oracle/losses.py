"""Oracle for openrlhf/models/loss.py (aggregate_loss, PolicyLoss, ValueLoss, DPOLoss, PairWiseLoss,
LogExpLoss) and the DPO trainer's per-sequence log-prob sums. Test
infrastructure, CPU torch; differentiable, so torch autograd is the gradient oracle."""
import torch

from .token_numerics import masked_mean


def aggregate_seq_token_sum(loss, loss_mask, dp_size=1, global_batch_size=None):
    """Sequence mean of token SUMS. Not in the reference (openrlhf/models/loss.py:29-39 divides
    every sequence by its token count): the same lines with that division removed."""
    cnt = loss_mask.sum(dim=-1)
    seq = (loss * loss_mask).sum(dim=-1)
    seq_mask = (cnt > 0).to(loss.dtype)
    if global_batch_size is None:
        return masked_mean(seq, seq_mask)
    return (seq * seq_mask).sum() / global_batch_size * dp_size


def aggregate_loss(loss, loss_mask, token_level_loss=True, dp_size=1, batch_num_tokens=None, global_batch_size=None):
    """Token-mean or mean of per-sequence token-means (openrlhf/models/loss.py:11-39)."""
    if token_level_loss:
        if batch_num_tokens is None:
            return masked_mean(loss, loss_mask)
        return (loss * loss_mask).sum() / batch_num_tokens * dp_size
    counts = loss_mask.sum(dim=-1)
    per_seq = (loss * loss_mask).sum(dim=-1) / (counts + 1e-8)
    non_empty = (counts > 0).to(per_seq.dtype)
    if global_batch_size is None:
        return masked_mean(per_seq, non_empty)
    return (per_seq * non_empty).sum() / global_batch_size * dp_size


def policy_loss(
    log_probs,
    old_log_probs,
    advantages,
    action_mask=None,
    rollout_log_probs=None,
    *,
    clip_eps_low=0.2,
    clip_eps_high=0.2,
    dual_clip=None,
    token_level_loss=True,
    policy_loss_type="ppo",
    enable_vllm_is_correction=False,
    vllm_is_truncated_threshold=None,
    vllm_is_correction_type="tis",
    dp_size=1,
    batch_num_tokens=None,
    global_batch_size=None,
):
    """PolicyLoss.__init__ + forward as one function (openrlhf/models/loss.py:116-230).
    Returns (loss, clip_ratio, ppo_kl, vllm_kl or None)."""
    if policy_loss_type == "gspo":
        token_level_loss = False
    if dual_clip is not None:
        assert dual_clip > 1.0, f"dual_clip must be > 1.0, got {dual_clip}"
    if vllm_is_correction_type not in {"tis", "icepop", "seq-mask-tis"}:
        raise ValueError(f"Invalid vllm_is_correction_type: {vllm_is_correction_type}")

    raw = log_probs - old_log_probs
    if policy_loss_type == "ppo":
        ratio = raw.clamp(min=-20.0, max=20.0).exp()
    elif policy_loss_type == "gspo":
        lr = (log_probs - rollout_log_probs) if enable_vllm_is_correction else raw
        seq = (lr * action_mask).sum(dim=-1) / action_mask.sum(dim=-1).clamp(min=1)
        ratio = seq.exp().unsqueeze(-1) * action_mask
    else:
        raise ValueError(f"Invalid policy loss type: {policy_loss_type}")

    s1 = ratio * advantages
    s2 = ratio.clamp(1 - clip_eps_low, 1 + clip_eps_high) * advantages
    if dual_clip is None:
        loss = -torch.min(s1, s2)
    else:
        lower = torch.min(s1, s2)
        floor = torch.max(lower, dual_clip * advantages)
        loss = -torch.where(advantages < 0, floor, lower)

    vllm_kl = None
    if enable_vllm_is_correction and policy_loss_type == "ppo":
        lo, hi = vllm_is_truncated_threshold
        mismatch = old_log_probs - rollout_log_probs
        if vllm_is_correction_type == "icepop":
            w = torch.exp(mismatch).detach()
            w = w * ((w >= lo) & (w <= hi))
            loss = w * loss
        elif vllm_is_correction_type == "seq-mask-tis":
            seq_w = torch.exp(masked_mean(mismatch, action_mask, dim=-1))
            keep = (seq_w >= lo) & (seq_w <= hi)
            loss = keep.unsqueeze(-1) * torch.exp(mismatch).detach() * loss
        else:
            loss = torch.exp(mismatch).clamp(min=lo, max=hi).detach() * loss
        vllm_kl = masked_mean(rollout_log_probs - old_log_probs, action_mask)

    total = aggregate_loss(
        loss, action_mask, token_level_loss=token_level_loss, dp_size=dp_size,
        batch_num_tokens=batch_num_tokens, global_batch_size=global_batch_size,
    )
    clip_ratio = masked_mean((s2 < s1).to(s1.dtype), action_mask)
    ppo_kl = masked_mean(-raw.detach(), action_mask)
    return total, clip_ratio, ppo_kl, vllm_kl


def value_loss(values, old_values, returns, action_mask=None, *, clip_eps=None, token_level_loss=True,
               dp_size=1, batch_num_tokens=None, global_batch_size=None):
    """ValueLoss.forward (openrlhf/models/loss.py:244-269)."""
    if clip_eps is not None:
        clipped = old_values + (values - old_values).clamp(-clip_eps, clip_eps)
        loss = torch.max((clipped - returns) ** 2, (values - returns) ** 2)
    else:
        loss = (values - returns) ** 2
    total = aggregate_loss(
        loss, action_mask, token_level_loss=token_level_loss, dp_size=dp_size,
        batch_num_tokens=batch_num_tokens, global_batch_size=global_batch_size,
    )
    return 0.5 * total


def loss_batch_info(loss_mask):
    """Single-process form of get_loss_batch_info (openrlhf/utils/loss_utils.py:15-52)."""
    tokens = loss_mask.sum().to(torch.float32)
    samples = (loss_mask.reshape(loss_mask.shape[0], -1).sum(dim=-1) > 0).sum().to(torch.float32)
    return {"dp_size": 1, "batch_num_tokens": tokens, "global_batch_size": samples}


def get_batch_logps(per_token_logps, attention_mask, prompt_id_lens):
    """DPOTrainer._get_batch_logps (openrlhf/trainer/dpo_trainer.py:362-382): clone the attention
    mask as bool, clear each row's prompt, drop the first column, then masked sum and mean."""
    loss_masks = attention_mask.clone().bool()
    for mask, source_len in zip(loss_masks, prompt_id_lens):
        mask[:source_len] = False
    loss_masks = loss_masks[:, 1:]
    sums = (per_token_logps * loss_masks).sum(-1)
    means = (per_token_logps * loss_masks).sum(-1) / loss_masks.sum(-1)
    return sums, means


def dpo_loss(policy_chosen, policy_rejected, reference_chosen, reference_rejected, beta, label_smoothing=0.0,
             ipo=False):
    """DPOLoss.forward (openrlhf/models/loss.py:300-335)."""
    F = torch.nn.functional
    logits = (policy_chosen - policy_rejected) - (reference_chosen - reference_rejected)
    if ipo:
        losses = (logits - 1 / (2 * beta)) ** 2
    else:
        losses = -F.logsigmoid(beta * logits) * (1 - label_smoothing) - F.logsigmoid(-beta * logits) * label_smoothing
    chosen_rewards = beta * (policy_chosen - reference_chosen).detach()
    rejected_rewards = beta * (policy_rejected - reference_rejected).detach()
    return losses.mean(), chosen_rewards, rejected_rewards


def pairwise_loss(chosen_reward, reject_reward, margin=None):
    """PairWiseLoss.forward (openrlhf/models/loss.py:272-284)."""
    F = torch.nn.functional
    if margin is not None:
        return (-F.logsigmoid(chosen_reward - reject_reward - margin)).mean()
    return (-F.logsigmoid(chosen_reward - reject_reward)).mean()


def logexp_loss(chosen_reward, reject_reward, margin=None):
    """LogExpLoss.forward (openrlhf/models/loss.py:287-297); the margin is unused there too."""
    return torch.log(1 + torch.exp(reject_reward - chosen_reward)).mean()

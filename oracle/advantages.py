"""Oracle for the advantage functions of openrlhf/trainer/ppo_utils/experience_maker.py.
Test infrastructure, CPU torch; keeps the reference's reverse-time Python loops."""
import torch


def get_advantages_and_returns(values, rewards, action_mask, gamma, lambd):
    """GAE over every column of the padded [B, A] block, outputs not re-masked
    (experience_maker.py:332-377)."""
    width = rewards.size(1)
    if action_mask is not None:
        values = action_mask * values
        rewards = action_mask * rewards
    carry = 0
    cols = []
    for t in range(width - 1, -1, -1):
        nxt = values[:, t + 1] if t + 1 < width else 0.0
        delta = rewards[:, t] + gamma * nxt - values[:, t]
        carry = delta + gamma * lambd * carry
        cols.append(carry)
    adv = torch.stack(cols[::-1], dim=1)
    return adv, adv + values


def get_cumulative_returns(rewards, action_mask, gamma):
    """Discounted reward-to-go with an fp32 accumulator (experience_maker.py:379-411)."""
    out = torch.zeros_like(rewards)
    acc = torch.zeros(rewards.size(0), dtype=rewards.dtype if rewards.dtype == torch.float64 else torch.float32)
    if action_mask is not None:
        rewards = action_mask * rewards
    for t in range(rewards.size(1) - 1, -1, -1):
        acc = rewards[:, t] + gamma * acc
        out[:, t] = acc
    return out


def group_normalize(rewards, indices, n_samples, estimator):
    """Group baseline / normalisation of scalar rewards (experience_maker.py:246-272).
    rewards: [P*n] in experience order; indices[i] = prompt-order slot of sample i.
    Returns (shaped rewards in experience order, per-sample group std or None)."""
    ordered = torch.empty_like(rewards)
    ordered[indices] = rewards
    grid = ordered.reshape(-1, n_samples)
    group_std = None
    if n_samples > 1:
        group_std = grid.std(-1, keepdim=True).repeat(1, n_samples).reshape(-1)[indices]
    if estimator == "rloo":
        grid = grid - (grid.sum(-1, keepdim=True) - grid) / (n_samples - 1)
    elif estimator in ("reinforce_baseline", "dr_grpo"):
        grid = grid - grid.mean(-1, keepdim=True)
    elif estimator == "group_norm":
        grid = (grid - grid.mean(-1, keepdim=True)) / (grid.std(-1, keepdim=True) + 1e-9)
    return grid.reshape(-1)[indices], group_std


def whiten_advantages(advantages_list, masks_list, no_std_norm=False):
    """Global masked whitening over a list of [B, A] blocks, applied to every column
    (experience_maker.py:314-328). float64 blocks stay float64 (the fp64 oracle)."""
    up = torch.float64 if advantages_list[0].dtype == torch.float64 else torch.float32
    flat = torch.cat([a.flatten() for a in advantages_list]).to(up)
    mask = torch.cat([m.flatten() for m in masks_list])
    count = mask.sum()
    mean = (flat * mask).sum() / count
    if not no_std_norm:
        var = ((flat - mean).pow(2) * mask).sum() / count
        rstd = var.clamp(min=1e-8).rsqrt()
    else:
        rstd = 1
    return [(a - mean) * rstd for a in advantages_list], mean, rstd

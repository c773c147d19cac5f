"""Oracle for openrlhf/models/utils.py (token numerics). Test infrastructure, CPU torch."""
import torch


def logsumexp_rows(rows: torch.Tensor, chunk: int = 1024) -> torch.Tensor:
    """Row-wise logsumexp in blocks of `chunk` rows (openrlhf/models/utils.py:129-136)."""
    out = torch.empty(rows.shape[0], dtype=rows.dtype)
    for lo in range(0, rows.shape[0], chunk):
        out[lo : lo + chunk] = torch.logsumexp(rows[lo : lo + chunk], dim=-1)
    return out


def log_probs_from_logits(logits: torch.Tensor, labels: torch.Tensor, temperature: float = 1.0) -> torch.Tensor:
    """x[label]/T - logsumexp(x/T) (openrlhf/models/utils.py:139-155, the gather + chunked
    logsumexp branch). Unlike the reference the caller's tensor is left untouched: the division
    makes a copy. Floating inputs narrower than fp32 are up-cast first, which is what the
    caller does before it gets here (openrlhf/models/actor.py:267)."""
    if logits.dtype not in (torch.float32, torch.float64):
        logits = logits.float()
    z = logits / temperature if temperature != 1.0 else logits
    vocab = z.shape[-1]
    picked = torch.gather(z, -1, labels.unsqueeze(-1)).squeeze(-1)
    lse = logsumexp_rows(z.reshape(-1, vocab)).view(z.shape[:-1])
    return picked - lse


def compute_entropy(logits: torch.Tensor) -> torch.Tensor:
    """logsumexp(x) - sum(softmax(x) * x) (openrlhf/models/utils.py:182-186), eager."""
    if logits.dtype not in (torch.float32, torch.float64):
        logits = logits.float()
    p = torch.softmax(logits, dim=-1)
    return torch.logsumexp(logits, dim=-1) - (p * logits).sum(dim=-1)


def compute_approx_kl(log_probs: torch.Tensor, log_probs_base: torch.Tensor, kl_estimator: str = "k1") -> torch.Tensor:
    """k1 / k2 / k3 estimators, clamped to [-10, 10] (openrlhf/models/utils.py:64-95). The
    reference up-casts to fp32; float64 inputs are kept so the same code is the fp64 oracle."""
    up = torch.float64 if log_probs.dtype == torch.float64 else torch.float32
    d = log_probs.to(up) - log_probs_base.to(up)
    if kl_estimator == "k1":
        est = d
    elif kl_estimator == "k2":
        est = d * d / 2.0
    elif kl_estimator == "k3":
        est = torch.exp(-d) - 1 + d
    else:
        raise ValueError(f"Unknown kl_estimator: {kl_estimator}")
    return est.clamp(min=-10, max=10)


def masked_mean(tensor: torch.Tensor, mask, dim=None) -> torch.Tensor:
    """sum(t*m)/sum(m), no epsilon (openrlhf/models/utils.py:166-169)."""
    if mask is None:
        return tensor.mean(dim=dim)
    return (tensor * mask).sum(dim=dim) / mask.sum(dim=dim)


def compute_reward(r, kl_coef, kl, action_mask, reward_clip_range=None):
    """Terminal reward at each row's last unmasked column minus kl_coef * kl
    (openrlhf/models/utils.py:98-126)."""
    coef = max(float(kl_coef), 0.0)
    if reward_clip_range:
        r = r.clamp(min=reward_clip_range[0], max=reward_clip_range[1])
    width = action_mask.shape[1]
    last = width - 1 - torch.argmax(action_mask.long().flip(1), dim=1, keepdim=True)
    terminal = torch.zeros_like(kl).scatter_(1, last, r.unsqueeze(1).to(kl.dtype))
    return terminal + (-coef) * kl


def last_unmasked_column(action_mask: torch.Tensor) -> torch.Tensor:
    """The `eos_indices` of openrlhf/models/utils.py:121 as an int64 [B] tensor."""
    width = action_mask.shape[1]
    return width - 1 - torch.argmax(action_mask.long().flip(1), dim=1)


def actor_forward_tail(logits, sequences, attention_mask, action_mask, temperature=1.0, packed=False):
    """What Actor.forward does after the model call (openrlhf/models/actor.py:265-296), for
    padded [B, T, V] logits or, with packed=True, [1, Ttot, V] logits of the unpadded tokens
    (openrlhf/models/ring_attn_utils.py:129-140,181): fp32 up-cast, entropy on the unscaled
    logits, log-prob of the next token on logits/T, re-pad, drop the last column, keep the last
    A columns, multiply the log-probs by the action mask. Returns (action_log_probs, entropy[:, :-1])."""
    batch, seqlen = sequences.shape
    rolled = torch.roll(sequences, shifts=-1, dims=1)
    logits = logits.float()
    if packed:
        keep = attention_mask.reshape(-1).bool().nonzero().squeeze(-1)
        labels = rolled.reshape(-1)[keep].unsqueeze(0)
    else:
        labels = rolled
    ent = compute_entropy(logits)
    lp = log_probs_from_logits(logits, labels, temperature)
    if packed:
        def repad(flat):
            full = torch.zeros(batch * seqlen, dtype=flat.dtype)
            full[keep] = flat.reshape(-1)
            return full.view(batch, seqlen)
        ent, lp = repad(ent), repad(lp)
    ent, lp = ent[:, :-1], lp[:, :-1]
    width = action_mask.shape[1]
    return lp[:, -width:] * action_mask.float(), ent


def masked_normalize(tensor: torch.Tensor, mask: torch.Tensor, dim: int = 1, eps: float = 1e-8) -> torch.Tensor:
    """openrlhf/models/utils.py:172-179: masked per-row whitening with the count clamped to >= 1
    and the biased variance clamped to >= eps."""
    mask_sum = mask.sum(dim=dim, keepdim=True).clamp(min=1)
    mean = (tensor * mask).sum(dim=dim, keepdim=True) / mask_sum
    mean_centered = (tensor - mean) * mask
    var = (mean_centered**2).sum(dim=dim, keepdim=True) / mask_sum
    return mean_centered * var.clamp(min=eps).rsqrt()


def experience_kl(action_log_probs, base_action_log_probs, action_mask, kl_estimator="k1"):
    """The KL block of make_experience (openrlhf/trainer/ppo_utils/experience_maker.py:202-216):
    per-token KL estimate and the per-sequence masked means the trainer logs."""
    if base_action_log_probs is not None:
        kl = compute_approx_kl(action_log_probs, base_action_log_probs, kl_estimator=kl_estimator)
        diff = action_log_probs.float() - base_action_log_probs.float()
    else:
        kl = torch.zeros_like(action_log_probs)
        diff = torch.zeros_like(action_log_probs)
    return kl, masked_mean(kl, action_mask, dim=-1), masked_mean(diff, action_mask, dim=-1)

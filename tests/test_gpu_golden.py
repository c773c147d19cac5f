"""The HIP path against the committed brute-force vectors of tests/golden/ (fp32 inputs:
1e-5 abs for log-probs, KL and losses, 1e-5 relative for GAE / returns)."""
import json
import math
import os

import pytest
import torch

pytestmark = pytest.mark.gpu
GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "token_numerics_golden.json")))


def F(x, dev):
    return torch.tensor(x, dtype=torch.float32, device=dev)


def close(got, ref, tol=1e-5, rel=False):
    got = torch.as_tensor(got).detach().cpu().double().reshape(-1)
    ref = torch.tensor(ref, dtype=torch.float64).reshape(-1)
    scale = max(1.0, ref.abs().max().item()) if rel else 1.0
    assert (got - ref).abs().max().item() <= tol * scale, (got - ref).abs().max().item()


def test_vocab_rows(cuda):
    from openrlhf_amd.models.utils import logprobs_and_entropy_from_logits

    v = GOLD["vocab_rows"]
    labels = torch.tensor(v["labels"], device=cuda)
    for case in v["cases"]:
        x = F(v["logits"], cuda).requires_grad_(True)
        lp, ent = logprobs_and_entropy_from_logits(x, labels, case["temperature"])
        close(lp, case["logprob"])
        close(ent, case["entropy"])
        ((lp * F(v["g_logprob"], cuda)).sum() + (ent * F(v["g_entropy"], cuda)).sum()).backward()
        close(x.grad, case["grad"])


def test_per_token(cuda):
    from openrlhf_amd.models.loss import PolicyLoss, ValueLoss, aggregate_loss
    from openrlhf_amd.models.utils import compute_approx_kl, masked_mean

    tok = GOLD["tokens"]
    lp, old, roll = F(tok["log_probs"], cuda), F(tok["old_log_probs"], cuda), F(tok["rollout_log_probs"], cuda)
    base, adv, mask = F(tok["base_log_probs"], cuda), F(tok["advantages"], cuda), F(tok["mask"], cuda)
    for est in ("k1", "k2", "k3"):
        close(compute_approx_kl(lp, base, est), GOLD["approx_kl"][est])
    a = GOLD["aggregate"]
    close(aggregate_loss(adv, mask), a["token_mean"])
    close(aggregate_loss(adv, mask, dp_size=2, batch_num_tokens=50.0), a["token_mean_global"])
    close(aggregate_loss(adv, mask.bool(), token_level_loss=False), a["seq_mean"])
    close(aggregate_loss(adv, mask, token_level_loss=False, dp_size=2, global_batch_size=5.0), a["seq_mean_global"])
    rows = masked_mean(adv, mask, dim=-1).cpu().tolist()
    for got, ref in zip(rows, a["row_mean"]):
        assert (math.isnan(got) and ref is None) or abs(got - ref) <= 1e-5
    for case in GOLD["policy_loss"]:
        cfg, ref = case["cfg"], case["out"]
        out = PolicyLoss(**cfg)(lp, old, adv, action_mask=mask,
                                rollout_log_probs=roll if cfg.get("enable_vllm_is_correction") else None, **case["norm"])
        close(out[0], ref["loss"], rel=True)
        close(out[1], ref["clip_ratio"])
        close(out[2], ref["ppo_kl"])
        assert (out[3] is None) == (ref["vllm_kl"] is None)
        if out[3] is not None:
            close(out[3], ref["vllm_kl"])
    v = GOLD["value_loss"]
    for case in v["cases"]:
        fn = ValueLoss(case["clip_eps"], token_level_loss=case["token_level_loss"])
        close(fn(F(v["values"], cuda), F(v["old_values"], cuda), F(v["returns"], cuda), action_mask=mask), case["out"])


def test_advantages(cuda):
    from openrlhf_amd.models.utils import compute_reward
    from openrlhf_amd.trainer.ppo_utils.experience_maker import (
        get_advantages_and_returns, get_cumulative_returns, group_normalize_rewards, whiten_advantages)

    mask = F(GOLD["tokens"]["mask"], cuda)
    c = GOLD["compute_reward"]
    close(compute_reward(F(c["r"], cuda), c["kl_coef"], F(c["kl"], cuda), action_mask=mask, reward_clip_range=tuple(c["clip"])),
          c["out"], 1e-6)
    values, rewards = F(GOLD["gae_inputs"]["values"], cuda), F(GOLD["gae_inputs"]["rewards"], cuda)
    for case in GOLD["gae"]:
        adv, ret = get_advantages_and_returns(values, rewards, mask, case["gamma"], case["lambd"])
        close(adv, case["advantages"], rel=True)
        close(ret, case["returns"], rel=True)
    for case in GOLD["cumulative_returns"]:
        close(get_cumulative_returns(rewards, mask, case["gamma"]), case["out"], rel=True)
    gn = GOLD["group_normalize"]
    for case in gn["cases"]:
        out, std = group_normalize_rewards(F(gn["rewards"], cuda), torch.tensor(gn["indices"], device=cuda), gn["n"], case["estimator"])
        close(out, case["out"], rel=True)
        close(std, case["group_std"], 1e-6)
    adv = F(GOLD["tokens"]["advantages"], cuda)
    for case in GOLD["whiten"]:
        out = whiten_advantages([adv[:2], adv[2:]], [mask[:2], mask[2:]], case["no_std_norm"])
        close(torch.cat(out), case["out"], rel=True)

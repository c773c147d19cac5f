"""Pins the CPU oracle (oracle/) before anything is compared with it: the brute-force golden
vectors in tests/golden/, closed forms, invariants, library routines (numpy/scipy) and the
identities the reference's own tests assert (tests/test_loss_aggregation.py of the reference,
restated here, not imported). Runs without a GPU."""
import json
import math
import os

import numpy as np
import pytest
import torch
from scipy.special import logsumexp as scipy_lse

from oracle import advantages as oa
from oracle import losses as ol
from oracle import token_numerics as otn

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "token_numerics_golden.json")))


def T(x, dtype=torch.float64):
    return torch.tensor(x, dtype=dtype)


def close(got, ref, tol=1e-10):
    got, ref = torch.as_tensor(got, dtype=torch.float64), torch.as_tensor(ref, dtype=torch.float64)
    assert got.shape == ref.shape
    scale = max(1.0, ref.abs().max().item()) if ref.numel() else 1.0
    assert (got - ref).abs().max().item() <= tol * scale, (got - ref).abs().max().item()


# ------------------------------------------------------------------ vocabulary rows
def test_logprob_entropy_against_golden_and_scipy():
    v = GOLD["vocab_rows"]
    x, labels = T(v["logits"]), torch.tensor(v["labels"])
    for case in v["cases"]:
        t = case["temperature"]
        close(otn.log_probs_from_logits(x, labels, t), case["logprob"])
        close(otn.compute_entropy(x), case["entropy"])
        # library routine: scipy logsumexp, and H = -sum p log p
        z = x.numpy() / t
        close(otn.log_probs_from_logits(x, labels, t), z[np.arange(len(labels)), labels.numpy()] - scipy_lse(z, axis=-1))
    p = torch.softmax(x, -1)
    close(otn.compute_entropy(x), -(p * torch.log(p)).sum(-1), 1e-9)
    # gradient of the oracle (autograd) against the golden analytic gradient
    for case in v["cases"]:
        xg = x.clone().requires_grad_(True)
        lp = otn.log_probs_from_logits(xg, labels, case["temperature"])
        ent = otn.compute_entropy(xg)
        ((lp * T(v["g_logprob"])).sum() + (ent * T(v["g_entropy"])).sum()).backward()
        close(xg.grad, case["grad"], 1e-9)


def test_logprob_entropy_invariants():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(6, 50, generator=g, dtype=torch.float64) * 3
    labels = torch.randint(0, 50, (6,), generator=g)
    lp = otn.log_probs_from_logits(x, labels, 0.8)
    assert (lp <= 0).all()
    # probabilities over all labels sum to one
    all_lp = torch.stack([otn.log_probs_from_logits(x, torch.full((6,), j), 0.8) for j in range(50)], -1)
    close(all_lp.exp().sum(-1), torch.ones(6), 1e-12)
    # shift invariance, bounds, uniform row, input left untouched, chunked logsumexp == plain
    close(otn.log_probs_from_logits(x + 7.0, labels, 0.8), lp, 1e-12)
    ent = otn.compute_entropy(x)
    assert (ent >= 0).all() and (ent <= math.log(50) + 1e-12).all()
    close(otn.compute_entropy(torch.full((2, 50), 3.0, dtype=torch.float64)), [math.log(50)] * 2, 1e-12)
    before = x.clone()
    otn.log_probs_from_logits(x, labels, 0.5)
    assert torch.equal(x, before)
    big = torch.randn(2500, 9, generator=g, dtype=torch.float64)
    close(otn.logsumexp_rows(big), torch.logsumexp(big, -1), 1e-13)
    # narrow dtypes are up-cast first (what Actor.forward does before calling)
    xb = x.to(torch.bfloat16)
    close(otn.log_probs_from_logits(xb, labels), otn.log_probs_from_logits(xb.float(), labels), 0.0)
    assert torch.autograd.gradcheck(lambda t: otn.log_probs_from_logits(t, labels[:2] % 9, 0.7), (x[:2, :9].clone().requires_grad_(True),))
    assert torch.autograd.gradcheck(otn.compute_entropy, (x[:2, :9].clone().requires_grad_(True),))


def test_actor_forward_tail_packed_equals_padded():
    """Index arithmetic of Actor.forward's tail: packed [1, Ttot, V] logits re-padded with the
    attention-mask indices give the same [B, A] action log-probs as the padded layout."""
    g = torch.Generator().manual_seed(1)
    b, t, vocab, a = 3, 9, 11, 5
    attn = torch.tensor([[1] * 9, [1] * 6 + [0] * 3, [1] * 8 + [0]])
    seqs = torch.randint(1, vocab, (b, t), generator=g) * attn
    logits = torch.randn(b, t, vocab, generator=g)
    action_mask = attn[:, 1:][:, -a:].bool()
    lp_pad, ent_pad = otn.actor_forward_tail(logits, seqs, attn, action_mask, temperature=0.9)
    packed = logits.reshape(-1, vocab)[attn.reshape(-1).bool()].unsqueeze(0)
    lp_pk, ent_pk = otn.actor_forward_tail(packed, seqs, attn, action_mask, temperature=0.9, packed=True)
    keep = action_mask
    close(lp_pk[keep], lp_pad[keep], 1e-6)
    valid = attn[:, :-1].bool()
    close(ent_pk[valid], ent_pad[valid], 1e-6)
    # brute force for one entry: log-softmax of position t at the NEXT token
    i, pos = 1, 3
    col = pos - (t - 1 - a)
    expect = torch.log_softmax(logits[i, pos].double() / 0.9, -1)[seqs[i, pos + 1]]
    close(lp_pad[i, col], expect, 1e-6)


# ------------------------------------------------------------------ KL, masked mean, aggregate
def test_approx_kl_golden_closed_forms_and_errors():
    tok = GOLD["tokens"]
    lp, base = T(tok["log_probs"]), T(tok["base_log_probs"])
    for est in ("k1", "k2", "k3"):
        out = otn.compute_approx_kl(lp, base, est)
        close(out, GOLD["approx_kl"][est], 1e-12)
        assert out.max() <= 10 and out.min() >= -10
    assert (otn.compute_approx_kl(lp, base, "k2") >= 0).all() and (otn.compute_approx_kl(lp, base, "k3") >= 0).all()
    assert otn.compute_approx_kl(T([30.0]), T([0.0]), "k1").item() == 10.0  # k1 is clamped too
    assert otn.compute_approx_kl(lp.float(), base.float(), "k1").dtype == torch.float32
    assert otn.compute_approx_kl(lp.to(torch.bfloat16), base.to(torch.bfloat16), "k1").dtype == torch.float32
    with pytest.raises(ValueError):
        otn.compute_approx_kl(lp, base, "k9")


def test_masked_mean_and_aggregate_golden():
    tok = GOLD["tokens"]
    adv, mask = T(tok["advantages"]), T(tok["mask"])
    a = GOLD["aggregate"]
    close(ol.aggregate_loss(adv, mask), a["token_mean"], 1e-12)
    close(ol.aggregate_loss(adv, mask, dp_size=2, batch_num_tokens=50.0), a["token_mean_global"], 1e-12)
    close(ol.aggregate_loss(adv, mask, token_level_loss=False), a["seq_mean"], 1e-9)
    close(ol.aggregate_loss(adv, mask, token_level_loss=False, dp_size=2, global_batch_size=5.0), a["seq_mean_global"], 1e-9)
    rows = otn.masked_mean(adv, mask, dim=-1)
    for got, ref in zip(rows.tolist(), a["row_mean"]):
        assert (math.isnan(got) and ref is None) or abs(got - ref) <= 1e-12
    assert math.isnan(otn.masked_mean(adv, torch.zeros_like(mask)).item())  # no epsilon
    close(otn.masked_mean(adv, None), adv.mean(), 0.0)


def test_reference_aggregation_identities():
    """The identities and the two literals of the reference's tests/test_loss_aggregation.py
    (:47-94, :151-193), restated on the oracle."""
    loss = T([[1.0, 2.0, 0.0], [3.0, 4.0, 5.0], [7.0, 0.0, 0.0]], torch.float32)
    mask = T([[1.0, 1.0, 0.0], [1.0, 1.0, 1.0], [1.0, 0.0, 0.0]], torch.float32)
    full = ol.aggregate_loss(loss, mask)
    n = mask.sum()
    r0 = ol.aggregate_loss(loss[:2], mask[:2], dp_size=2, batch_num_tokens=n)
    r1 = ol.aggregate_loss(loss[2:], mask[2:], dp_size=2, batch_num_tokens=n)
    assert torch.allclose((r0 + r1) / 2, full)
    loss = T([[1.0, 3.0, 9.0], [2.0, 4.0, 0.0], [8.0, 0.0, 0.0]], torch.float32)
    mask = T([[1.0, 1.0, 0.0], [1.0, 1.0, 0.0], [1.0, 0.0, 0.0]], torch.float32)
    full = ol.aggregate_loss(loss, mask, token_level_loss=False)
    r0 = ol.aggregate_loss(loss[:2], mask[:2], token_level_loss=False, dp_size=2, global_batch_size=3.0)
    r1 = ol.aggregate_loss(loss[2:], mask[2:], token_level_loss=False, dp_size=2, global_batch_size=3.0)
    assert torch.allclose((r0 + r1) / 2, full)
    loss = T([[1.0, 3.0], [5.0, 7.0]], torch.float32)
    mask = T([[1.0, 1.0], [0.0, 0.0]], torch.float32)
    info = ol.loss_batch_info(mask)
    assert info["global_batch_size"].item() == 1.0
    assert torch.allclose(ol.aggregate_loss(loss, mask, token_level_loss=False, **info), torch.tensor(2.0))
    # gradient-accumulation window: same global normaliser for every micro-batch (gas = 2)
    mb0, m0 = T([[1.0, 2.0, 0.0]], torch.float32), T([[1.0, 1.0, 0.0]], torch.float32)
    mb1, m1 = T([[3.0, 4.0, 5.0], [6.0, 7.0, 0.0]], torch.float32), T([[1.0, 1.0, 1.0], [1.0, 1.0, 0.0]], torch.float32)
    n_global = m0.sum() + m1.sum()
    expected = ((mb0 * m0).sum() + (mb1 * m1).sum()) / n_global
    acc = sum(ol.aggregate_loss(x, m, batch_num_tokens=n_global / 2) / 2 for x, m in ((mb0, m0), (mb1, m1)))
    assert torch.allclose(acc, expected)
    assert not torch.allclose((ol.aggregate_loss(mb0, m0) + ol.aggregate_loss(mb1, m1)) / 2, expected)


# ------------------------------------------------------------------ PolicyLoss / ValueLoss
def test_policy_loss_golden():
    tok = GOLD["tokens"]
    lp, old, roll = T(tok["log_probs"]), T(tok["old_log_probs"]), T(tok["rollout_log_probs"])
    adv, mask = T(tok["advantages"]), T(tok["mask"])
    for case in GOLD["policy_loss"]:
        out = ol.policy_loss(lp, old, adv, mask, roll, **case["cfg"], **case["norm"])
        ref = case["out"]
        close(out[0], ref["loss"], 1e-9)
        close(out[1], ref["clip_ratio"], 1e-12)
        close(out[2], ref["ppo_kl"], 1e-12)
        if ref["vllm_kl"] is None:
            assert out[3] is None
        else:
            close(out[3], ref["vllm_kl"], 1e-12)


def test_policy_loss_reference_identities_and_closed_forms():
    lp = T([[-0.20, -0.40, -0.10], [-0.70, -0.30, -0.20], [-0.60, -0.10, -0.50]], torch.float32)
    old = lp - T([[0.03, -0.04, 0.01], [0.02, 0.05, -0.03], [0.04, 0.0, -0.02]], torch.float32)
    adv = T([[1.0, -0.5, 0.0], [0.3, -1.2, 0.5], [1.5, 0.0, -0.7]], torch.float32)
    mask = T([[1.0, 1.0, 0.0], [1.0, 1.0, 1.0], [1.0, 0.0, 1.0]], torch.float32)
    full = ol.policy_loss(lp, old, adv, mask)[0]
    n = mask.sum()
    r0 = ol.policy_loss(lp[:2], old[:2], adv[:2], mask[:2], dp_size=2, batch_num_tokens=n)[0]
    r1 = ol.policy_loss(lp[2:], old[2:], adv[2:], mask[2:], dp_size=2, batch_num_tokens=n)[0]
    assert torch.allclose((r0 + r1) / 2, full)
    lp2, old2, roll2 = T([[-0.2, -0.4]], torch.float32), T([[-0.3, -0.1]], torch.float32), T([[-1.3, -1.1]], torch.float32)
    _, _, kl, vk = ol.policy_loss(lp2, old2, torch.ones_like(lp2), torch.ones_like(lp2), roll2,
                                  enable_vllm_is_correction=True, vllm_is_truncated_threshold=[0.1, 10.0])
    assert torch.allclose(kl, (old2 - lp2).mean()) and torch.allclose(vk, (roll2 - old2).mean())
    big = T([[100.0]], torch.float32)
    assert ol.policy_loss(big, torch.zeros_like(big), torch.ones_like(big), torch.ones_like(big))[2].item() == -100.0
    # closed forms: identical policies; dual clip floor; 4-tuple; constructor errors
    out = ol.policy_loss(lp, lp, adv, mask)
    close(out[0], -(adv * mask).sum() / mask.sum(), 1e-7)
    assert out[1].item() == 0.0 and out[3] is None and len(out) == 4
    hi = torch.full((1, 4), math.log(10.0))
    close(ol.policy_loss(hi, torch.zeros(1, 4), -torch.ones(1, 4), torch.ones(1, 4), dual_clip=3.0)[0], 3.0, 1e-6)
    with pytest.raises(AssertionError):
        ol.policy_loss(lp, old, adv, mask, dual_clip=1.0)
    with pytest.raises(ValueError):
        ol.policy_loss(lp, old, adv, mask, vllm_is_correction_type="x")
    with pytest.raises(ValueError):
        ol.policy_loss(lp, old, adv, mask, policy_loss_type="x")
    x = lp.double().requires_grad_(True)
    assert torch.autograd.gradcheck(lambda t: ol.policy_loss(t, old.double(), adv.double() + 0.01, mask.double(), dual_clip=3.0)[0], (x,))


def test_value_loss_golden_and_closed_forms():
    v = GOLD["value_loss"]
    values, old, ret, mask = T(v["values"]), T(v["old_values"]), T(v["returns"]), T(GOLD["tokens"]["mask"])
    for case in v["cases"]:
        out = ol.value_loss(values, old, ret, mask, clip_eps=case["clip_eps"], token_level_loss=case["token_level_loss"])
        close(out, case["out"], 1e-9)
    close(ol.value_loss(values, old, ret, mask, clip_eps=1e9), ol.value_loss(values, old, ret, mask), 1e-12)
    close(ol.value_loss(values, old, ret, mask), 0.5 * (((values - ret) ** 2) * mask).sum() / mask.sum(), 1e-12)


# ------------------------------------------------------------------ advantages
def test_compute_reward_golden_and_edge_cases():
    c = GOLD["compute_reward"]
    mask = T(GOLD["tokens"]["mask"])
    out = otn.compute_reward(T(c["r"]), c["kl_coef"], T(c["kl"]), mask, tuple(c["clip"]))
    close(out, c["out"], 1e-12)
    assert otn.last_unmasked_column(mask).tolist() == [15, 11, 15, 15]  # empty row -> last column
    assert torch.equal(otn.compute_reward(T(c["r"]), -3.0, T(c["kl"]), mask), otn.compute_reward(T(c["r"]), 0.0, T(c["kl"]), mask))
    assert otn.compute_reward(T(c["r"]), 0.0, T(c["kl"]), mask)[0, 15].item() == 12.5  # no clip range given


def test_gae_and_returns_golden_and_closed_forms():
    values, rewards = T(GOLD["gae_inputs"]["values"]), T(GOLD["gae_inputs"]["rewards"])
    mask = T(GOLD["tokens"]["mask"])
    for case in GOLD["gae"]:
        adv, ret = oa.get_advantages_and_returns(values, rewards, mask, case["gamma"], case["lambd"])
        close(adv, case["advantages"], 1e-12)
        close(ret, case["returns"], 1e-12)
    for case in GOLD["cumulative_returns"]:
        close(oa.get_cumulative_returns(rewards, mask, case["gamma"]), case["out"], 1e-12)
    ones = torch.ones_like(values)
    adv, ret = oa.get_advantages_and_returns(values, rewards, ones, 1.0, 1.0)
    togo = rewards.flip(1).cumsum(1).flip(1)
    close(adv, togo - values, 1e-12)
    close(ret, togo, 1e-12)
    adv, _ = oa.get_advantages_and_returns(values, rewards, ones, 0.9, 0.0)
    nxt = torch.cat([values[:, 1:], torch.zeros(4, 1, dtype=torch.float64)], 1)
    close(adv, rewards + 0.9 * nxt - values, 1e-12)
    # docstring closed form of the reference (experience_maker.py:345-351)
    g_, l_ = 0.98, 0.9
    adv, _ = oa.get_advantages_and_returns(values[:1], rewards[:1], ones[:1], g_, l_)
    width = values.shape[1]
    expect0 = sum((g_ * l_) ** k * rewards[0, k] for k in range(width)) - values[0, 0] + sum(
        g_ ** k * l_ ** (k - 1) * (1 - l_) * values[0, k] for k in range(1, width))
    close(adv[0, 0], expect0, 1e-12)
    # masked prompt columns keep non-zero values, right padding is exactly zero
    adv, ret = oa.get_advantages_and_returns(values, rewards, mask, 1.0, 0.95)
    assert adv[1, 12:].abs().max() == 0 and adv[0, 0].abs() > 0
    assert oa.get_cumulative_returns(rewards.float(), mask.float(), 1.0).dtype == torch.float32


def test_group_normalize_and_whiten_golden():
    gn = GOLD["group_normalize"]
    rewards, idx = T(gn["rewards"]), torch.tensor(gn["indices"])
    for case in gn["cases"]:
        out, std = oa.group_normalize(rewards, idx, gn["n"], case["estimator"])
        close(out, case["out"], 1e-9)
        close(std, case["group_std"], 1e-12)
    ordered = torch.empty_like(rewards)
    ordered[idx] = rewards
    close(oa.group_normalize(rewards, idx, gn["n"], "gae")[1], np.std(ordered.view(-1, gn["n"]).numpy(), axis=1, ddof=1).repeat(gn["n"])[idx.numpy()], 1e-12)
    out, _ = oa.group_normalize(rewards, idx, gn["n"], "group_norm")
    assert out[(idx // gn["n"]) == 0].abs().max() == 0  # all-equal group: exactly 0/(0+1e-9)
    assert oa.group_normalize(rewards, idx, 1, "reinforce")[1] is None
    adv, mask = T(GOLD["tokens"]["advantages"]), T(GOLD["tokens"]["mask"])
    for case in GOLD["whiten"]:
        out, mean, rstd = oa.whiten_advantages([adv[:2], adv[2:]], [mask[:2], mask[2:]], case["no_std_norm"])
        close(torch.cat(out), case["out"], 1e-10)
    out, _, _ = oa.whiten_advantages([adv], [mask])
    close((out[0] * mask).sum() / mask.sum(), 0.0, 1e-12)
    close(((out[0] ** 2) * mask).sum() / mask.sum(), 1.0, 1e-9)
    assert out[0][2].abs().min() > 0  # the fully masked row is whitened too


# ------------------------------------------------------------------ sequence level (DPO / RM)
def test_sequence_logps_golden_and_closed_forms():
    s = GOLD["sequence_logps"]
    lp = T(GOLD["tokens"]["log_probs"]).requires_grad_(True)
    att, lens = torch.tensor(s["attention_mask"]), s["prompt_id_lens"]
    sums, means = ol.get_batch_logps(lp, att, lens)
    close(sums.detach(), s["sums"], 1e-12)
    for b, ref in enumerate(s["means"]):
        if ref is None:
            assert torch.isnan(means[b])
        else:
            close(means[b].detach(), ref, 1e-12)
    keep = [b for b, ref in enumerate(s["means"]) if ref is not None]
    (g,) = torch.autograd.grad((sums * T(s["g_sums"])).sum() + (means[keep] * T(s["g_means"])[keep]).sum(), lp)
    for b in keep:
        close(g[b], s["grad"][b], 1e-12)
    # no prompt, full attention: plain row sums and means of every column
    full = torch.ones(4, 17, dtype=torch.long)
    sums, means = ol.get_batch_logps(lp.detach(), full, [0, 0, 0, 0])
    close(sums, lp.detach().sum(-1), 1e-12)
    close(means, lp.detach().mean(-1), 1e-12)
    # the prompt length counts in tokens of the unshifted sequence: prompt p leaves columns p-1..
    sums, _ = ol.get_batch_logps(lp.detach(), full, [4, 4, 4, 4])
    close(sums, lp.detach()[:, 3:].sum(-1), 1e-12)


def test_pair_losses_golden_and_closed_forms():
    p = GOLD["pair_loss"]
    c, r, rc, rr = (T(p[k]) for k in ("chosen", "rejected", "ref_chosen", "ref_rejected"))
    for case in p["dpo"]:
        cg = c.clone().requires_grad_(True)
        rg = r.clone().requires_grad_(True)
        loss, cr_, rr_ = ol.dpo_loss(cg, rg, rc, rr, case["beta"], case["label_smoothing"], case["ipo"])
        close(loss.detach(), case["out"]["loss"], 1e-11)
        close(cr_, case["out"]["chosen_rewards"], 1e-12)
        close(rr_, case["out"]["rejected_rewards"], 1e-12)
        gc, gr = torch.autograd.grad(loss, (cg, rg))
        close(gc, case["out"]["g_chosen"], 1e-11)
        close(gr, -T(case["out"]["g_chosen"]), 1e-11)
    a, b, m = T(p["chosen_reward"]), T(p["reject_reward"]), T(p["margin"])
    close(ol.pairwise_loss(a, b), p["pairwise"]["loss"], 1e-12)
    close(ol.pairwise_loss(a, b, m), p["pairwise_margin"]["loss"], 1e-12)
    close(ol.logexp_loss(a, b), p["logexp"]["loss"], 1e-12)
    # closed forms: equal rewards give ln 2; the two reward-model losses are the same function
    z = torch.zeros(5, dtype=torch.float64)
    close(ol.pairwise_loss(z, z), math.log(2.0), 1e-15)
    close(ol.logexp_loss(a, b), ol.pairwise_loss(a, b), 1e-12)
    # DPO at the reference policy is ln 2 whatever beta; IPO's minimum sits at z = 1/(2 beta)
    close(ol.dpo_loss(c, r, c, r, 0.3)[0], math.log(2.0), 1e-15)
    close(ol.dpo_loss(c + 1 / (2 * 0.25), c, rc, rc, 0.25, ipo=True)[0], 0.0, 1e-12)
    # label smoothing 0.5 makes the loss even in z
    close(ol.dpo_loss(c, r, rc, rr, 0.2, 0.5)[0], ol.dpo_loss(r, c, rr, rc, 0.2, 0.5)[0], 1e-12)


# ------------------------------------------------------------------ layout helpers
def test_layout_oracle_known_answers():
    from oracle import layout as olay

    a, b = torch.tensor([1, 2, 3]), torch.tensor([4])
    assert olay.zero_pad_sequences([a, b], "left", 0, stack=True).tolist() == [[1, 2, 3], [0, 0, 4]]
    assert olay.zero_pad_sequences([a, b], "right", 9, stack=True).tolist() == [[1, 2, 3], [4, 9, 9]]
    assert olay.zero_pad_sequences([a, b], "right", 9).tolist() == [1, 2, 3, 4, 9, 9]
    m = olay.zero_pad_sequences([torch.ones(2, 2), torch.full((1, 3), 2.0)], "right")
    assert m.tolist() == [[1, 1, 0], [1, 1, 0], [2, 2, 2]]
    assert olay.unpadded_length(torch.tensor([0, 1, 1, 0, 1, 0, 0])) == 5
    assert olay.unpadded_length(torch.tensor([1, 1, 1])) == 3
    assert olay.unpad_boundaries(torch.tensor([[1, 1, 0], [1, 1, 1], [0, 0, 0]])).tolist() == [0, 2, 5, 5]


def test_masked_normalize_kl_rows_and_token_sum_golden():
    tok = GOLD["tokens"]
    adv, mask = T(tok["advantages"]), T(tok["mask"])
    out = otn.masked_normalize(adv, mask, dim=1, eps=GOLD["masked_normalize"]["eps"])
    close(out, GOLD["masked_normalize"]["out"], 1e-10)
    full = torch.ones_like(mask)
    z = otn.masked_normalize(adv, full)
    close(z.mean(dim=1), torch.zeros(4), 1e-12)
    close((z ** 2).mean(dim=1), torch.ones(4), 1e-9)  # biased variance 1 over the row
    assert (otn.masked_normalize(adv, mask)[mask == 0] == 0).all()
    lp, base = T(tok["log_probs"]), T(tok["base_log_probs"])
    for est, ref in GOLD["kl_rows"].items():
        kl, kl_mean, diff_mean = otn.experience_kl(lp, base, mask, est)
        close(kl, GOLD["approx_kl"][est], 1e-10)
        for b in range(4):
            if ref["kl_mean"][b] is None:
                assert torch.isnan(kl_mean[b]) and torch.isnan(diff_mean[b])
            else:
                close(kl_mean[b], ref["kl_mean"][b], 1e-10)
                close(diff_mean[b], ref["diff_mean"][b], 1e-7)  # the reference forms lp.float() - base.float()
    kl, kl_mean, _ = otn.experience_kl(lp, None, full, "k1")
    assert (kl == 0).all() and (kl_mean == 0).all()
    agg = GOLD["aggregate"]
    close(ol.aggregate_seq_token_sum(adv, mask), agg["seq_token_sum"], 1e-12)
    close(ol.aggregate_seq_token_sum(adv, mask, dp_size=2, global_batch_size=5.0), agg["seq_token_sum_global"], 1e-12)
    # every sequence of the same length L: token-sum mode = L * the reference's seq-mean mode
    close(ol.aggregate_seq_token_sum(adv, full), 16 * ol.aggregate_loss(adv, full, token_level_loss=False), 1e-9)


def test_layout_unpad_and_rebatch_known_answer():
    """The three hops on a literal batch (openrlhf/trainer/ppo_utils/experience.py:164-247): trailing
    zeros of the attention mask go, an all-zero mask row and a row ending in a one keep everything,
    the A = T - 1 wide field loses the same number of columns, rows are right-padded with zeros."""
    import torch

    from oracle import layout as olay

    att = torch.tensor([[1, 1, 1, 0, 0], [0, 0, 0, 0, 0], [1, 1, 0, 1, 1], [1, 0, 0, 0, 0]])
    seq = torch.arange(20).view(4, 5) + 1
    out, kept = olay.unpad_and_rebatch(seq, att)
    assert kept == [3, 5, 5, 1]
    assert out.tolist() == [[1, 2, 3, 0, 0], [6, 7, 8, 9, 10], [11, 12, 13, 14, 15], [16, 0, 0, 0, 0]]
    act = torch.arange(16).view(4, 4) + 1.0
    out, kept = olay.unpad_and_rebatch(act, att)
    assert kept == [2, 4, 4, 0]
    assert out.tolist() == [[1, 2, 0, 0], [5, 6, 7, 8], [9, 10, 11, 12], [0, 0, 0, 0]]


def test_layout_unpad_and_slice_known_answers():
    """unpad_and_slice_tensor / gather_and_pad_tensor restatements: the example in the reference's
    docstrings (openrlhf/models/ring_attn_utils.py:112-118, :155-164) and a cell-by-cell walk of a
    mask with left padding, right padding and holes."""
    from oracle import layout as olay

    seq = torch.tensor([[1, 2, 3, 0], [4, 5, 0, 0]])
    att = torch.tensor([[1, 1, 1, 0], [1, 1, 0, 0]])
    packed, pos, rolled, pad_len, indices, cu = olay.unpad_and_slice_tensor(seq, att)
    assert packed.tolist() == [[1, 2, 3, 4, 5]] and pad_len == 0
    assert indices.tolist() == [0, 1, 2, 4, 5] and cu.tolist() == [0, 3, 5]
    assert pos.tolist() == [[0, 1, 2, 0, 1]] and rolled.tolist() == [[2, 3, 0, 5, 0]]
    assert olay.gather_and_pad_tensor(packed, indices, 2, 4).tolist() == [[1, 2, 3, 0], [4, 5, 0, 0]]

    g = torch.Generator().manual_seed(0)
    att = (torch.rand(5, 13, generator=g) < 0.5).long()
    att[0] = 0
    att[1, :4] = 0
    att[2, 9:] = 0
    seq = torch.randint(0, 100, (5, 13), generator=g)
    packed, pos, rolled, _, indices, cu = olay.unpad_and_slice_tensor(seq, att)
    want_i, want_p, want_r, want_pos, want_cu = [], [], [], [], [0]
    for b in range(5):
        rank = 0
        for t in range(13):
            if att[b, t]:
                want_i.append(b * 13 + t)
                want_p.append(int(seq[b, t]))
                want_r.append(int(seq[b, (t + 1) % 13]))
                want_pos.append(rank)
                rank += 1
        want_cu.append(want_cu[-1] + rank)
    assert indices.tolist() == want_i and packed[0].tolist() == want_p and rolled[0].tolist() == want_r
    assert pos[0].tolist() == want_pos and cu.tolist() == want_cu
    vals = torch.arange(1.0, len(want_i) + 1).unsqueeze(0)
    padded = olay.gather_and_pad_tensor(vals, indices, 5, 13)
    for b in range(5):
        for t in range(13):
            assert padded[b, t] == (vals[0, want_i.index(b * 13 + t)] if att[b, t] else 0)

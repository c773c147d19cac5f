"""The five benchmark configurations of the headline metric at their full sizes on one MI355X.

Configs 1, 3 and 4 are compared with the CPU oracle in full. Configs 2 and 5 (9.4 GB / 34 GB of
logits) are compared with the fp64 oracle on a row sample and, over all rows, through properties
that do not depend on size: rows are independent (re-running a sample of rows alone gives the
same bits), log-prob <= 0, 0 <= entropy <= ln V, every gradient row sums to zero, fully masked
tokens get exactly zero gradient. "N(0, s)" is read as standard deviation s.
"""
import math

import pytest
import torch

from oracle import advantages as oa
from oracle import losses as ol
from oracle import token_numerics as otn

pytestmark = pytest.mark.gpu


def _fill_normal(n, v, std, dev, seed, dtype=torch.bfloat16, slab=2048):
    g = torch.Generator(device=dev).manual_seed(seed)
    x = torch.empty(n, v, dtype=dtype, device=dev)
    for lo in range(0, n, slab):
        hi = min(lo + slab, n)
        x[lo:hi] = (torch.randn(hi - lo, v, generator=g, device=dev) * std).to(dtype)
    return x


def _analytic_grad64(x, labels, temperature, g_lp, g_ent):
    x64 = x.double()
    p_t = torch.softmax(x64 / temperature, -1)
    p = torch.softmax(x64, -1)
    onehot = torch.zeros_like(x64).scatter_(1, labels.unsqueeze(1), 1.0)
    ex = (p * x64).sum(-1, keepdim=True)
    return g_lp.double()[:, None] * (onehot - p_t) / temperature + g_ent.double()[:, None] * p * (ex - x64)


def _vocab_config(cuda, n, vocab, std, temperature, seed, spike_frac, sample):
    from openrlhf_amd.models.utils import logprobs_and_entropy_from_logits

    g = torch.Generator().manual_seed(seed)
    x = _fill_normal(n, vocab, std, cuda, seed)
    if spike_frac:
        k = max(1, int(n * spike_frac))
        rows = torch.randperm(n, generator=g)[:k].to(cuda)
        cols = torch.randint(0, vocab, (k,), generator=g).to(cuda)
        x[rows, cols] += 15.0
    labels = torch.randint(0, vocab, (n,), generator=g).to(cuda)
    g_lp = torch.randn(n, generator=g).to(cuda)
    g_ent = torch.randn(n, generator=g).to(cuda)
    dead = torch.randperm(n, generator=g)[: n // 50].to(cuda)  # masked tokens: zero upstream grads
    g_lp[dead] = 0
    g_ent[dead] = 0
    pick = torch.randperm(n, generator=g)[:sample].to(cuda)
    x_pick = x[pick].clone()

    xr = x.requires_grad_(True)
    lp, ent = logprobs_and_entropy_from_logits(xr, labels, temperature, inplace_backward=True)
    # forward properties over all rows
    assert lp.max().item() <= 0.0 and torch.isfinite(lp).all()
    assert ent.min().item() >= -1e-4 and ent.max().item() <= math.log(vocab) + 1e-4
    # sample vs fp64 oracle (2e-3 abs for bf16 inputs)
    lp64 = otn.log_probs_from_logits(x_pick.cpu().double(), labels[pick].cpu(), temperature)
    ent64 = otn.compute_entropy(x_pick.cpu().double())
    assert (lp[pick].cpu().double() - lp64).abs().max().item() <= 2e-3
    assert (ent[pick].cpu().double() - ent64).abs().max().item() <= 2e-3
    # rows are independent: the sample alone gives the same bits (repeated up to 256 rows, the size
    # from which rows are not cut into segments), and the same values to the rounding of the fp32
    # partial sums when its few rows are cut
    reps = -(-256 // sample)
    lp_s, ent_s = logprobs_and_entropy_from_logits(x_pick.repeat(reps, 1), labels[pick].repeat(reps), temperature)
    assert torch.equal(lp_s[:sample], lp[pick]) and torch.equal(ent_s[:sample], ent[pick])
    lp_c, ent_c = logprobs_and_entropy_from_logits(x_pick, labels[pick], temperature)
    assert (lp_c - lp[pick]).abs().max().item() <= 2e-5 and (ent_c - ent[pick]).abs().max().item() <= 2e-5  # values up to 45

    (grad,) = torch.autograd.grad([lp, ent], [xr], [g_lp, g_ent])
    assert grad.data_ptr() == x.data_ptr()  # in place
    ref = _analytic_grad64(x_pick.cpu(), labels[pick].cpu(), temperature, g_lp[pick].cpu(), g_ent[pick].cpu())
    err = (grad[pick].cpu().double() - ref).abs()
    assert (err <= 2.0 ** -8 * ref.abs() + 1e-6).all(), err.max().item()
    # every gradient row sums to zero (bf16 rounding noise only); masked tokens are exactly zero
    sums = torch.cat([grad[lo:lo + 4096].float().sum(-1) for lo in range(0, n, 4096)])
    assert sums.abs().max().item() <= 5e-2
    assert grad[dead].abs().max().item() == 0.0
    return lp.detach(), labels


def test_config2_packed_bf16_policy_step(cuda):
    """16 sequences, lengths uniform in [512, 3072], packed; bf16 logits [Ttot, 151936] ~ N(0, 3),
    1% of rows with one +15 spike, T = 1; fused forward and in-place backward."""
    g = torch.Generator().manual_seed(2)
    lens = torch.randint(512, 3073, (16,), generator=g)
    n = int(lens.sum())
    _vocab_config(cuda, n, 151936, 3.0, 1.0, seed=22, spike_frac=0.01, sample=48)
    torch.cuda.empty_cache()


def test_config5_large_vocab_long_context(cuda):
    """bf16 logits [65536 (4 x 16384 packed), 262144] ~ N(0, 4), T = 0.6, in-place gradient over
    34 GB of resident logits, then per-token k3 KL and token-mean PolicyLoss on the packed rows."""
    from openrlhf_amd.models.loss import PolicyLoss
    from openrlhf_amd.models.utils import compute_approx_kl

    n = 65536
    lp, _ = _vocab_config(cuda, n, 262144, 4.0, 0.6, seed=55, spike_frac=0.0, sample=16)
    torch.cuda.empty_cache()
    g = torch.Generator().manual_seed(5)
    cu = torch.arange(0, n + 1, 16384, dtype=torch.int64)
    ref_lp = lp.cpu() + torch.randn(n, generator=g) * 0.1
    old = lp.cpu() + torch.randn(n, generator=g) * 0.02
    adv = torch.randn(n, generator=g)
    mask = torch.rand(n, generator=g) > 0.3
    kl = compute_approx_kl(lp, ref_lp.to(cuda), "k3")
    assert (kl.cpu().double() - otn.compute_approx_kl(lp.cpu().double(), ref_lp.double(), "k3")).abs().max().item() <= 1e-5
    x = lp.clone().requires_grad_(True)
    out = PolicyLoss()(x, old.to(cuda), adv.to(cuda), action_mask=mask.to(cuda), cu_seqlens=cu.to(cuda))
    x64 = lp.cpu().double().requires_grad_(True)
    ref = ol.policy_loss(x64.view(4, 16384), old.double().view(4, 16384), adv.double().view(4, 16384), mask.double().view(4, 16384))
    for got, want in zip(out[:3], ref[:3]):
        assert abs(got.item() - want.item()) <= 1e-5
    out[0].backward()
    ref[0].backward()
    assert (x.grad.cpu().double() - x64.grad).abs().max().item() <= 1e-9


def test_config3_critic_gae_path(cuda):
    """256 sequences, lengths lognormal(7, 0.8) clipped to [16, 8192], fp32 values ~ N(0, 1);
    reward Bernoulli(0.5) at the last token minus 0.01 * k1; gamma 1, lambda 0.95; GAE, masked
    whitening, ValueLoss(0.2). Full size against the oracle's sequential loops."""
    from openrlhf_amd.models.loss import ValueLoss
    from openrlhf_amd.models.utils import compute_approx_kl, compute_reward
    from openrlhf_amd.trainer.ppo_utils.experience_maker import get_advantages_and_returns, whiten_advantages

    g = torch.Generator().manual_seed(3)
    b = 256
    lens = torch.clamp(torch.exp(torch.randn(b, generator=g) * 0.8 + 7.0), 16, 8192).long()
    a = int(lens.max())
    mask = torch.arange(a)[None, :] < lens[:, None]
    values = torch.randn(b, a, generator=g)
    lp = -torch.rand(b, a, generator=g) * 2
    ref_lp = lp + torch.randn(b, a, generator=g) * 0.05
    r = (torch.rand(b, generator=g) < 0.5).float()

    kl64 = otn.compute_approx_kl(lp.double(), ref_lp.double(), "k1")
    rew64 = otn.compute_reward(r.double(), 0.01, kl64, mask)
    adv64, ret64 = oa.get_advantages_and_returns(values.double(), rew64, mask.double(), 1.0, 0.95)
    (white64,), _, _ = oa.whiten_advantages([adv64], [mask.double()])
    new_values = values + torch.randn(b, a, generator=g) * 0.3
    v64 = new_values.double().requires_grad_(True)
    loss64 = ol.value_loss(v64, values.double(), ret64, mask.double(), clip_eps=0.2)
    loss64.backward()

    d = cuda
    kl = compute_approx_kl(lp.to(d), ref_lp.to(d), "k1")
    rew = compute_reward(r.to(d), 0.01, kl, action_mask=mask.to(d))
    adv, ret = get_advantages_and_returns(values.to(d), rew, mask.to(d), 1.0, 0.95)
    (white,) = whiten_advantages([adv], [mask.to(d)])
    for got, want in ((rew, rew64), (adv, adv64), (ret, ret64), (white, white64)):
        scale = want.abs().max().item()
        assert (got.cpu().double() - want).abs().max().item() <= 1e-5 * scale
    # reward shaping and GAE in one pass: the same bits, and the row sums of the reward
    from openrlhf_amd.trainer.ppo_utils.experience_maker import reward_advantages_and_returns
    adv1, ret1, total = reward_advantages_and_returns(r.to(d), 0.01, kl, values.to(d), mask.to(d), 1.0, 0.95)
    assert torch.equal(adv1, adv) and torch.equal(ret1, ret)
    assert (total.cpu().double() - rew64.sum(1)).abs().max().item() <= 1e-5 * rew64.sum(1).abs().max().item()
    v = new_values.to(d).requires_grad_(True)
    loss = ValueLoss(0.2)(v, values.to(d), ret, action_mask=mask.to(d))
    assert abs(loss.item() - loss64.item()) <= 1e-5
    loss.backward()
    assert (v.grad.cpu().double() - v64.grad).abs().max().item() <= 1e-5 * v64.grad.abs().max().item() + 1e-12


def test_config4_grpo_group_step(cuda):
    """512 prompts x 8 samples, rewards Bernoulli(0.3), response lengths uniform in [64, 16384];
    group mean/std normalisation broadcast to tokens (discounted returns with gamma 1), k3 KL vs
    ref = lp + N(0, 0.1), dual-clip PPO (eps 0.2, c 3) with sequence-level aggregation, fp32."""
    from openrlhf_amd.models.loss import PolicyLoss
    from openrlhf_amd.models.utils import compute_approx_kl, compute_reward, masked_mean
    from openrlhf_amd.trainer.ppo_utils.experience_maker import get_cumulative_returns, group_normalize_rewards

    g = torch.Generator().manual_seed(4)
    p, n = 512, 8
    b = p * n
    lens = torch.randint(64, 16385, (b,), generator=g)
    a = int(lens.max())
    mask = torch.arange(a)[None, :] < lens[:, None]
    rewards = (torch.rand(b, generator=g) < 0.3).float()
    perm = torch.randperm(b, generator=g)
    lp = -torch.rand(b, a, generator=g) * 2
    ref_lp = lp + torch.randn(b, a, generator=g) * 0.1
    old = lp + torch.randn(b, a, generator=g) * 0.05
    d = cuda

    shaped, std = group_normalize_rewards(rewards.to(d), perm.to(d), n, "group_norm")
    shaped64, std64 = oa.group_normalize(rewards.double(), perm, n, "group_norm")
    assert (shaped.cpu().double() - shaped64).abs().max().item() <= 1e-5 * shaped64.abs().max().item()
    zero_kl = torch.zeros(b, a, device=d)
    tok_reward = compute_reward(shaped, 0.0, zero_kl, action_mask=mask.to(d))
    adv = get_cumulative_returns(tok_reward, mask.to(d), 1.0)
    # gamma = 1, no KL penalty: the shaped reward at every column up to the last token, 0 after
    expect = shaped.cpu()[:, None] * mask
    assert torch.equal(adv.cpu(), expect)
    del zero_kl, tok_reward

    kl = compute_approx_kl(lp.to(d), ref_lp.to(d), "k3")
    kl_mean = masked_mean(kl, mask.to(d), dim=-1)
    kl64 = otn.compute_approx_kl(lp.double(), ref_lp.double(), "k3")
    assert (kl_mean.cpu().double() - otn.masked_mean(kl64, mask.double(), dim=-1)).abs().max().item() <= 1e-5
    del kl, kl64

    x = lp.to(d).requires_grad_(True)
    out = PolicyLoss(0.2, 0.2, dual_clip=3.0, token_level_loss=False)(x, old.to(d), adv, action_mask=mask.to(d))
    x64 = lp.double().requires_grad_(True)
    ref = ol.policy_loss(x64, old.double(), expect.double(), mask.double(), dual_clip=3.0, token_level_loss=False)
    for got, want in zip(out[:3], ref[:3]):
        assert abs(got.item() - want.item()) <= 1e-5
    out[0].backward()
    ref[0].backward()
    assert (x.grad.cpu().double() - x64.grad).abs().max().item() <= 1e-5 * x64.grad.abs().max().item() + 1e-12


def _rounding_excess(got, want, eps, slab=2048):
    """max over all elements of |got - want| - eps * |want|, slab by slab on the device."""
    worst = -1.0
    for lo in range(0, got.shape[0], slab):
        a, b = got[lo:lo + slab].float(), want[lo:lo + slab].float()
        worst = max(worst, ((a - b).abs() - eps * b.abs()).max().item())
    return worst


def _one_pass_config(cuda, n, vocab, std, temperature, seed, spike_frac, sample):
    """The one-pass forward+backward kernel on a full-size batch: every row against the separate
    forward and in-place backward kernels (run on a copy), a row sample against the fp64 oracle."""
    from openrlhf_amd.models.utils import fused_logprob_entropy_fwd_bwd, logprobs_and_entropy_from_logits

    g = torch.Generator().manual_seed(seed)
    x = _fill_normal(n, vocab, std, cuda, seed)
    if spike_frac:
        k = max(1, int(n * spike_frac))
        x[torch.randperm(n, generator=g)[:k].to(cuda), torch.randint(0, vocab, (k,), generator=g).to(cuda)] += 15.0
    labels = torch.randint(0, vocab, (n,), generator=g).to(cuda)
    g_lp, g_ent = torch.randn(n, generator=g).to(cuda), torch.randn(n, generator=g).to(cuda)
    dead = torch.randperm(n, generator=g)[: n // 50].to(cuda)
    g_lp[dead] = 0
    g_ent[dead] = 0
    pick = torch.randperm(n, generator=g)[:sample].to(cuda)
    x_pick = x[pick].cpu()

    xa = x.clone().requires_grad_(True)
    lp2, ent2 = logprobs_and_entropy_from_logits(xa, labels, temperature, inplace_backward=True)
    (g2,) = torch.autograd.grad([lp2, ent2], [xa], [g_lp, g_ent])
    lp, ent, grad = fused_logprob_entropy_fwd_bwd(x, labels, g_lp, g_ent, temperature, inplace=True)
    assert grad.data_ptr() == x.data_ptr() and g2.data_ptr() == xa.data_ptr()
    assert (lp - lp2).abs().max().item() <= 2e-5 and (ent - ent2).abs().max().item() <= 2e-5
    assert _rounding_excess(grad, g2, 2.0 ** -7) <= 4e-6
    assert grad[dead].abs().max().item() == 0.0
    lp64 = otn.log_probs_from_logits(x_pick.double(), labels[pick].cpu(), temperature)
    ent64 = otn.compute_entropy(x_pick.double())
    assert (lp[pick].cpu().double() - lp64).abs().max().item() <= 2e-3
    assert (ent[pick].cpu().double() - ent64).abs().max().item() <= 2e-3
    ref = _analytic_grad64(x_pick, labels[pick].cpu(), temperature, g_lp[pick].cpu(), g_ent[pick].cpu())
    err = (grad[pick].cpu().double() - ref).abs()
    assert (err <= 2.0 ** -8 * ref.abs() + 1e-6).all(), err.max().item()


def test_config2_one_pass_kernel_full_size(cuda):
    """Config 2 through the one-pass kernel the benchmark times: ~30 K rows on one workgroup per
    CU, i.e. ~120 rows per workgroup through the row-to-row register pipeline."""
    g = torch.Generator().manual_seed(2)
    n = int(torch.randint(512, 3073, (16,), generator=g).sum())
    _one_pass_config(cuda, n, 151936, 3.0, 1.0, seed=23, spike_frac=0.01, sample=48)
    torch.cuda.empty_cache()


def test_config5_one_pass_kernel_full_size(cuda):
    """Config 5 through the one-pass kernel: 65536 rows of 262144 bf16 logits at T = 0.6, half of
    every row resident in registers and half streamed twice, two statistic sets."""
    _one_pass_config(cuda, 65536, 262144, 4.0, 0.6, seed=56, spike_frac=0.0, sample=16)
    torch.cuda.empty_cache()


def test_config2_fused_actor_step_full_size(cuda):
    """The whole PPO actor loss step at config 2's size from one pass over the packed logits,
    against the composed step on the separate kernels (values and all gradient rows), and a row
    sample against the oracle: d(loss)/d(logprob) and d(loss)/d(entropy) from torch autograd
    through the oracle's losses in fp64, pushed through the analytic row gradient."""
    from openrlhf_amd.models.actor import unpad_indices
    from openrlhf_amd.models.loss import PolicyLoss
    from openrlhf_amd.trainer.ray.ppo_actor import actor_loss_step, fused_actor_loss_step

    vocab = 151936
    g = torch.Generator().manual_seed(2)
    lens = torch.randint(512, 3073, (16,), generator=g)
    b, t = 16, int(lens.max())
    n = int(lens.sum())
    attn = (torch.arange(t)[None, :] < lens[:, None]).long()
    seqs = torch.randint(1, vocab, (b, t), generator=g) * attn
    a = t - 1
    amask = attn[:, 1:].bool().clone()
    amask[:, :200] = False                      # prompt
    amask[3, 700:760] = False                   # a hole (environment tokens)
    old = -torch.rand(b, a, generator=g) * 14
    base = -torch.rand(b, a, generator=g) * 14
    adv = torch.randn(b, a, generator=g)
    x = _fill_normal(n, vocab, 3.0, cuda, 24)
    d = cuda
    idx = unpad_indices(attn.to(d))
    labels_rows = torch.roll(seqs, -1, 1).reshape(-1)[idx.cpu()]
    pick = torch.randperm(n, generator=g)[:32]
    x_pick = x[pick.to(d)].cpu()
    fn = PolicyLoss(0.2, 0.28, dual_clip=3.0)
    kw = dict(base_action_log_probs=base.to(d), kl_estimator="k3", kl_coef=0.01, entropy_coef=0.001,
              packed_indices=idx)
    tensors = (seqs.to(d), attn.to(d), amask.to(d), old.to(d), adv.to(d), fn)

    xa = x.clone().requires_grad_(True)
    ref = actor_loss_step(xa, *tensors, inplace_backward=True, **kw)
    ref["loss"].backward()
    out = fused_actor_loss_step(x, *tensors, **kw)
    grad = out["grad_logits"]
    assert grad.data_ptr() == x.data_ptr()
    for key in ("loss", "actor_loss", "kl_loss", "entropy_loss", "clip_ratio", "ppo_kl"):
        assert abs(out[key].item() - ref[key].item()) <= 2e-5 * max(1.0, abs(ref[key].item())), key
    assert (out["action_log_probs"] - ref["action_log_probs"]).abs().max().item() <= 2e-5
    gscale = xa.grad.float().abs().max().item()
    assert _rounding_excess(grad, xa.grad, 2.0 ** -7) <= 1e-6 * gscale + 1e-12

    # oracle: the losses in fp64 on the action log-probs / entropy the device produced
    alp = out["action_log_probs"].cpu().double().requires_grad_(True)
    ent = out["entropy"].cpu().double().requires_grad_(True)
    m = amask.double()
    pl = ol.policy_loss(alp, old.double(), adv.double(), m, dual_clip=3.0, clip_eps_low=0.2, clip_eps_high=0.28)
    kl_loss = ol.aggregate_loss(otn.compute_approx_kl(alp, base.double(), "k3"), m)
    ent_loss = ol.aggregate_loss(ent, m)
    loss = pl[0] + kl_loss * 0.01 - ent_loss * 0.001
    assert abs(out["loss"].item() - loss.item()) <= 1e-5
    loss.backward()

    def rows_of(t_ba):  # [B, A] -> one value per packed logits row
        full = torch.zeros(b, t, dtype=torch.float64)
        full[:, : t - 1] = t_ba
        return full.reshape(-1)[idx.cpu()]

    w_lp, w_ent = rows_of(alp.grad * m), rows_of(ent.grad)
    want = _analytic_grad64(x_pick, labels_rows[pick], 1.0, w_lp[pick], w_ent[pick])
    got = grad[pick.to(d)].cpu().double()
    err = (got - want).abs()
    assert (err <= 2.0 ** -7 * want.abs() + 1e-4 * want.abs().max().item() + 1e-12).all(), err.max().item()
    torch.cuda.empty_cache()

"""Parity of the advantage kernels (compute_reward, GAE, discounted returns, group baselines,
whitening) with the CPU oracle. GAE tolerance: 1e-5 relative (to the largest magnitude in the
block, so that exact cancellations do not dominate)."""
import math
from types import SimpleNamespace

import pytest
import torch

from oracle import advantages as oa
from oracle import token_numerics as otn

pytestmark = pytest.mark.gpu
RTOL = 1e-5


def _rel_close(got, ref, rtol=RTOL):
    got = got.detach().cpu().double()
    ref = ref.detach().double()
    assert got.shape == ref.shape
    scale = max(ref.abs().max().item(), 1e-30) if ref.numel() else 1.0
    err = (got - ref).abs().max().item() if ref.numel() else 0.0
    assert err <= rtol * scale, (err, scale)


def _mask(b, a, seed, kind="mixed"):
    g = torch.Generator().manual_seed(seed)
    m = torch.ones(b, a)
    for i in range(b):
        left = int(torch.randint(0, max(a // 3, 1), (1,), generator=g))
        right = int(torch.randint(0, max(a // 3, 1), (1,), generator=g))
        m[i, :left] = 0
        if right:
            m[i, a - right:] = 0
        if kind == "mixed" and a > 16:
            h = int(torch.randint(0, a - 3, (1,), generator=g))
            m[i, h:h + 3] = 0
    return m


# ------------------------------------------------------------------ compute_reward
@pytest.mark.parametrize("mask_dtype", [torch.bool, torch.float32, torch.int64])
def test_compute_reward_matches_oracle_and_brute_force(cuda, mask_dtype):
    from openrlhf_amd.models.utils import compute_reward

    b, a = 40, 777
    g = torch.Generator().manual_seed(1)
    mask = _mask(b, a, 1)
    mask[3] = 0  # all-zero row: the reward lands on the last column
    mask[4] = 1
    r = torch.randn(b, generator=g) * 8
    kl = torch.randn(b, a, generator=g)
    ref = otn.compute_reward(r, 0.05, kl, mask, reward_clip_range=(-10, 10))
    out = compute_reward(r.to(cuda), 0.05, kl.to(cuda), action_mask=mask.to(mask_dtype).to(cuda), reward_clip_range=(-10, 10))
    assert torch.equal(out.cpu(), ref)  # same fp32 operations: bit-exact
    # the double loop given as a comment in the reference (models/utils.py:112-120)
    brute = torch.zeros(b, a)
    for i in range(b):
        for t in reversed(range(a)):
            if mask[i, t] > 0.5:
                brute[i, t] = r[i].clamp(-10, 10)
                break
    rows = [i for i in range(b) if mask[i].sum() > 0]
    assert torch.equal((out.cpu() - (-0.05) * kl)[rows].round(decimals=4), brute[rows].round(decimals=4))
    assert abs(out[3, a - 1].item() - (r[3].clamp(-10, 10) - 0.05 * kl[3, a - 1]).item()) < 1e-6
    # negative coefficient is treated as 0; no clip range
    out2 = compute_reward(r.to(cuda), -1.0, kl.to(cuda), action_mask=mask.to(cuda))
    assert torch.equal(out2.cpu(), otn.compute_reward(r, -1.0, kl, mask))


# ------------------------------------------------------------------ GAE / returns
@pytest.mark.parametrize("a", [1, 7, 8, 9, 255, 2047, 2048, 2049, 5000])
@pytest.mark.parametrize("gamma,lambd", [(1.0, 0.95), (0.99, 0.9), (1.0, 1.0)])
def test_gae_matches_sequential_oracle(cuda, a, gamma, lambd):
    from openrlhf_amd.trainer.ppo_utils.experience_maker import get_advantages_and_returns

    b = 13
    g = torch.Generator().manual_seed(a)
    values = torch.randn(b, a, generator=g)
    rewards = torch.randn(b, a, generator=g) * 0.1
    mask = _mask(b, a, a)
    adv64, ret64 = oa.get_advantages_and_returns(values.double(), rewards.double(), mask.double(), gamma, lambd)
    adv, ret = get_advantages_and_returns(values.to(cuda), rewards.to(cuda), mask.to(cuda), gamma, lambd)
    _rel_close(adv, adv64)
    _rel_close(ret, ret64)
    # CPU tensors in, CPU tensors out (the reference's experiences live on the CPU)
    adv_c, ret_c = get_advantages_and_returns(values, rewards, mask.bool(), gamma, lambd)
    assert adv_c.device.type == "cpu" and torch.equal(adv_c, adv.cpu()) and torch.equal(ret_c, ret.cpu())


def test_gae_closed_forms(cuda):
    from openrlhf_amd.trainer.ppo_utils.experience_maker import get_advantages_and_returns

    b, a = 5, 300
    g = torch.Generator().manual_seed(3)
    values = torch.randn(b, a, generator=g)
    rewards = torch.randn(b, a, generator=g)
    ones = torch.ones(b, a)
    # lambda = gamma = 1: A_t = sum_{s >= t} r_s - v_t
    adv, ret = get_advantages_and_returns(values.to(cuda), rewards.to(cuda), ones.to(cuda), 1.0, 1.0)
    togo = rewards.double().flip(1).cumsum(1).flip(1)
    _rel_close(adv, togo - values.double())
    _rel_close(ret, togo)
    # lambda = 0: one-step TD error
    adv, _ = get_advantages_and_returns(values.to(cuda), rewards.to(cuda), ones.to(cuda), 0.9, 0.0)
    nxt = torch.cat([values[:, 1:], torch.zeros(b, 1)], 1).double()
    _rel_close(adv, rewards.double() + 0.9 * nxt - values.double())
    # right padding gives exact zeros; masked prompt columns are NOT zero (nothing is re-masked)
    mask = ones.clone()
    mask[:, 250:] = 0
    mask[:, :20] = 0
    adv, ret = get_advantages_and_returns(values.to(cuda), rewards.to(cuda), mask.to(cuda), 1.0, 0.95)
    assert adv[:, 250:].abs().max().item() == 0.0 and ret[:, 250:].abs().max().item() == 0.0
    assert adv[:, :20].abs().min().item() > 0.0


@pytest.mark.parametrize("a", [1, 100, 2048, 4097])
def test_cumulative_returns(cuda, a):
    from openrlhf_amd.trainer.ppo_utils.experience_maker import get_cumulative_returns

    b = 9
    g = torch.Generator().manual_seed(a + 1)
    rewards = torch.randn(b, a, generator=g)
    mask = _mask(b, a, a + 1)
    for gamma in (1.0, 0.97):
        ref = oa.get_cumulative_returns(rewards.double(), mask.double(), gamma)
        _rel_close(get_cumulative_returns(rewards.to(cuda), mask.to(cuda), gamma), ref)
    # gamma = 1 and a single terminal reward: every column up to it holds that reward
    one = torch.zeros(b, a)
    one[:, -1] = 2.5
    out = get_cumulative_returns(one.to(cuda), torch.ones(b, a).to(cuda), 1.0)
    assert torch.equal(out.cpu(), torch.full((b, a), 2.5))


def test_packed_scan_equals_padded(cuda):
    from openrlhf_amd.trainer.ppo_utils.experience_maker import get_advantages_and_returns, get_cumulative_returns

    g = torch.Generator().manual_seed(5)
    lens = torch.randint(1, 6000, (21,), generator=g)
    a = int(lens.max())
    values = torch.randn(21, a, generator=g)
    rewards = torch.randn(21, a, generator=g) * 0.1
    valid = torch.arange(a)[None, :] < lens[:, None]
    inner = (torch.rand(21, a, generator=g) > 0.1) & valid
    cu = torch.cat([torch.zeros(1, dtype=torch.int64), lens.cumsum(0)]).to(cuda)
    adv, ret = get_advantages_and_returns(values.to(cuda), rewards.to(cuda), inner.to(cuda), 1.0, 0.95)
    adv_p, ret_p = get_advantages_and_returns(values[valid].to(cuda), rewards[valid].to(cuda), inner[valid].to(cuda),
                                              1.0, 0.95, cu_seqlens=cu)
    assert torch.equal(adv_p, adv[valid.to(cuda)]) and torch.equal(ret_p, ret[valid.to(cuda)])
    assert adv[~valid.to(cuda)].abs().max().item() == 0.0  # what unpacking restores
    g1 = get_cumulative_returns(rewards.to(cuda), inner.to(cuda), 0.99)
    g2 = get_cumulative_returns(rewards[valid].to(cuda), inner[valid].to(cuda), 0.99, cu_seqlens=cu)
    assert torch.equal(g2, g1[valid.to(cuda)])
    # rows handed out longest first (any permutation): the schedule changes, no bit of the results does
    from openrlhf_amd.trainer.ppo_utils.experience_maker import reward_advantages_and_returns
    for order in (torch.argsort(lens, descending=True), torch.randperm(21, generator=g)):
        adv_o, ret_o = get_advantages_and_returns(values[valid].to(cuda), rewards[valid].to(cuda), inner[valid].to(cuda),
                                                  1.0, 0.95, cu_seqlens=cu, row_order=order.to(cuda))
        assert torch.equal(adv_o, adv_p) and torch.equal(ret_o, ret_p)
        g3 = get_cumulative_returns(rewards[valid].to(cuda), inner[valid].to(cuda), 0.99, cu_seqlens=cu,
                                    row_order=order.to(cuda))
        assert torch.equal(g3, g2)
        adv_o2, ret_o2 = get_advantages_and_returns(values.to(cuda), rewards.to(cuda), inner.to(cuda), 1.0, 0.95,
                                                    row_order=order.to(cuda))
        assert torch.equal(adv_o2, adv) and torch.equal(ret_o2, ret)
        r_seq = torch.randn(21, generator=torch.Generator().manual_seed(1)).to(cuda)
        one = reward_advantages_and_returns(r_seq, 0.01, rewards[valid].to(cuda), values[valid].to(cuda),
                                            inner[valid].to(cuda), 1.0, 0.95, cu_seqlens=cu)
        two = reward_advantages_and_returns(r_seq, 0.01, rewards[valid].to(cuda), values[valid].to(cuda),
                                            inner[valid].to(cuda), 1.0, 0.95, cu_seqlens=cu, row_order=order.to(cuda))
        assert all(torch.equal(x, y) for x, y in zip(one, two))
    with pytest.raises(ValueError):
        get_cumulative_returns(rewards.to(cuda), inner.to(cuda), 0.99, row_order=torch.arange(5, device=cuda))


# ------------------------------------------------------------------ group baselines
@pytest.mark.parametrize("estimator", ["gae", "reinforce", "rloo", "reinforce_baseline", "dr_grpo", "group_norm"])
@pytest.mark.parametrize("n", [2, 8, 5])
def test_group_normalize(cuda, estimator, n):
    from openrlhf_amd.trainer.ppo_utils.experience_maker import group_normalize_rewards

    p = 64
    g = torch.Generator().manual_seed(n)
    rewards = (torch.rand(p * n, generator=g) < 0.3).float()  # Bernoulli(0.3): many all-equal groups
    rewards[: 2 * n] = torch.randn(2 * n, generator=g)
    perm = torch.randperm(p * n, generator=g)
    ref, ref_std = oa.group_normalize(rewards.double(), perm, n, estimator)
    out, std = group_normalize_rewards(rewards.to(cuda), perm.to(cuda), n, estimator)
    assert (out.cpu().double() - ref).abs().max().item() <= 1e-5 * max(1.0, ref.abs().max().item())
    assert (std.cpu().double() - ref_std).abs().max().item() <= 1e-6
    # numpy-style cross-check of the unbiased std and of exact zeros for all-equal groups
    ordered = torch.empty_like(rewards)
    ordered[perm] = rewards
    grid = ordered.view(p, n)
    flat_group = (perm // n)
    if estimator in ("reinforce_baseline", "dr_grpo", "group_norm", "rloo"):
        equal = (grid.max(1).values == grid.min(1).values)[flat_group]
        assert out.cpu()[equal].abs().max().item() == 0.0
    if estimator == "rloo":
        sums = torch.zeros(p).index_add_(0, flat_group, out.cpu())
        assert sums.abs().max().item() <= 1e-5
    if estimator in ("gae", "reinforce"):
        assert torch.equal(out.cpu(), rewards)


def test_group_normalize_single_sample_and_errors(cuda):
    from openrlhf_amd.trainer.ppo_utils.experience_maker import group_normalize_rewards

    r = torch.randn(10)
    out, std = group_normalize_rewards(r.to(cuda), None, 1, "reinforce")
    assert std is None and torch.equal(out.cpu(), r)
    with pytest.raises(Exception):
        group_normalize_rewards(r.to(cuda), None, 2, "unknown")
    with pytest.raises(ValueError):
        group_normalize_rewards(r.to(cuda), None, 3, "rloo")


# ------------------------------------------------------------------ whitening
@pytest.mark.parametrize("no_std_norm", [False, True])
def test_whitening(cuda, no_std_norm):
    from openrlhf_amd.trainer.ppo_utils.experience_maker import whiten_advantages

    g = torch.Generator().manual_seed(11)
    shapes = [(4, 300), (7, 1111), (1, 5)]
    advs = [torch.randn(s, generator=g) * 3 + 1.5 for s in shapes]
    masks = [_mask(s[0], s[1], i + 20) for i, s in enumerate(shapes)]
    ref, mean, rstd = oa.whiten_advantages([a.double() for a in advs], [m.double() for m in masks], no_std_norm)
    out = whiten_advantages([a.to(cuda) for a in advs], [m.to(cuda).bool() for m in masks], no_std_norm)
    for o, r in zip(out, ref):
        _rel_close(o, r)
    flat = torch.cat([o.cpu().double().flatten() for o in out])
    m = torch.cat([x.flatten() for x in masks]).double()
    assert abs(((flat * m).sum() / m.sum()).item()) <= 1e-5
    if not no_std_norm:
        assert abs((((flat ** 2) * m).sum() / m.sum()).item() - 1.0) <= 1e-4
    # masked columns are whitened too (not zeroed)
    assert out[0].cpu()[masks[0] == 0].abs().min().item() > 0.0


def test_whitening_over_many_blocks(cuda):
    """More blocks than one launch carries, empty blocks among them, blocks longer than one
    workgroup's span, odd storage offsets and mask dtypes that differ between blocks: the
    statistics are taken over all of them together (experience_maker.py:314-328)."""
    from openrlhf_amd.trainer.ppo_utils.experience_maker import whiten_advantages

    g = torch.Generator().manual_seed(12)
    shapes = [(3, 41), (0, 7), (2, 9001), (1, 1)] * 9 + [(5, 8192)]
    advs = [torch.randn(s, generator=g) * 2 - 0.7 for s in shapes]
    masks = [(torch.rand(s, generator=g) > 0.3) for s in shapes]
    ref, mean, rstd = oa.whiten_advantages([a.double() for a in advs], [m.double() for m in masks])

    def on_gpu(t, i):  # every third block off the 16-byte boundary
        t = t.to(cuda)
        if i % 3 == 0 or t.numel() == 0:
            return t
        buf = torch.empty(t.numel() + 1, dtype=t.dtype, device=cuda)
        view = buf[1:].view(t.shape)
        view.copy_(t)
        return view

    out = whiten_advantages([on_gpu(a, i) for i, a in enumerate(advs)], [on_gpu(m, i) for i, m in enumerate(masks)])
    for o, r, s_ in zip(out, ref, shapes):
        assert tuple(o.shape) == s_
        if o.numel():
            _rel_close(o, r)
    # 30 blocks go block by block in two launches, the 37 above are gathered first
    k = 30
    ref30, _, _ = oa.whiten_advantages([a.double() for a in advs[:k]], [m.double() for m in masks[:k]])
    out30 = whiten_advantages([on_gpu(a, i) for i, a in enumerate(advs[:k])],
                              [on_gpu(m, i) for i, m in enumerate(masks[:k])])
    for o, r in zip(out30, ref30):
        if o.numel():
            _rel_close(o, r)
    advs, masks, ref = advs[:k], masks[:k], ref30
    mixed = whiten_advantages([a.to(cuda) for a in advs],
                              [m.to(cuda).long() if i % 2 else m.to(cuda) for i, m in enumerate(masks)])
    for o, r in zip(mixed, ref):
        if o.numel():
            _rel_close(o, r)


# ------------------------------------------------------------------ config 3 shape, end to end
@pytest.mark.parametrize("estimator", ["gae", "reinforce_baseline", "group_norm", "rloo"])
def test_compute_advantages_and_returns_pipeline(cuda, estimator):
    """A down-scaled PPO / GRPO batch: experiences with CPU tensors as the reference's
    controller holds them; k1 KL penalty 0.01, gamma 1, lambda 0.95; compared with the oracle's
    composition of the same steps (experience_maker.py:237-330)."""
    from openrlhf_amd.trainer.ppo_utils.experience_maker import AdvantageFunctions

    g = torch.Generator().manual_seed(33)
    n_prompts, n = 12, 4
    total = n_prompts * n
    lens = torch.clamp(torch.exp(torch.randn(total, generator=g) * 0.8 + 5.5), 16, 2048).long()
    perm = torch.randperm(total, generator=g)
    exps, ref_exps = [], []
    per_exp = 8
    for lo in range(0, total, per_exp):
        ids = list(range(lo, lo + per_exp))
        a = int(lens[ids].max())
        mask = (torch.arange(a)[None, :] < lens[ids][:, None])
        mask[:, :3] = False
        kl = torch.randn(per_exp, a, generator=g) * 0.05
        values = torch.randn(per_exp, a, generator=g)
        rewards = (torch.rand(per_exp, generator=g) < 0.5).float()
        index = perm[ids].tolist()
        for store in (exps, ref_exps):
            store.append(SimpleNamespace(index=index, rewards=rewards.clone(), kl=kl.clone(), action_mask=mask.clone(),
                                         values=values.clone(), info={}, advantages=None, returns=None))
    args = SimpleNamespace(
        algo=SimpleNamespace(advantage=SimpleNamespace(estimator=estimator, gamma=1.0, lambd=0.95, no_std_norm=False)),
        rollout=SimpleNamespace(n_samples_per_prompt=n),
        reward=SimpleNamespace(clip_range=(-10, 10)),
    )
    fn = AdvantageFunctions(strategy=SimpleNamespace(args=args), kl_ctl=SimpleNamespace(value=0.01))
    out = fn.compute_advantages_and_returns(exps)

    # oracle composition in fp64
    raw = torch.cat([e.rewards for e in ref_exps]).double()
    idx = torch.tensor([i for e in ref_exps for i in e.index])
    shaped, gstd = oa.group_normalize(raw, idx, n, estimator)
    advs, rets, infos = [], [], []
    for e, r in zip(ref_exps, shaped.split([per_exp] * len(ref_exps))):
        rew = otn.compute_reward(r, 0.01, e.kl.double(), e.action_mask, (-10, 10))
        if estimator == "gae":
            a_, r_ = oa.get_advantages_and_returns(e.values.double(), rew, e.action_mask, 1.0, 0.95)
        else:
            r_ = oa.get_cumulative_returns(rew, e.action_mask, 1.0)
            a_ = r_.clone()
        advs.append(a_)
        rets.append(r_)
        infos.append(rew.sum(-1))
    if estimator in ("gae", "reinforce", "reinforce_baseline"):
        advs, _, _ = oa.whiten_advantages(advs, [e.action_mask for e in ref_exps])
    for e, a_, r_, i_ in zip(out, advs, rets, infos):
        assert e.advantages.device.type == "cpu" and e.kl is None
        _rel_close(e.advantages, a_, 2e-5)
        _rel_close(e.returns, r_)
        _rel_close(e.info["return"], i_, 1e-5)
    std_all = torch.cat([e.info["group_reward_std"] for e in out])
    assert (std_all.double() - gstd).abs().max().item() <= 1e-6


# ------------------------------------------------------------------ reward + scan in one pass
@pytest.mark.parametrize("mask_dtype", [torch.bool, torch.int64, torch.float32])
@pytest.mark.parametrize("gae", [True, False])
def test_reward_scan_equals_the_two_calls_and_the_oracle(cuda, mask_dtype, gae):
    """compute_reward + GAE / discounted returns without the per-token reward in memory: the
    same bits as the two separate kernels, padded and packed, and the oracle's composition
    (openrlhf/models/utils.py:98-126, experience_maker.py:332-411) within the GAE tolerance."""
    from openrlhf_amd.models.utils import compute_reward
    from openrlhf_amd.trainer.ppo_utils.experience import PackedSteps
    from openrlhf_amd.trainer.ppo_utils.experience_maker import (
        get_advantages_and_returns, get_cumulative_returns, reward_advantages_and_returns)

    g = torch.Generator().manual_seed(91)
    b, a = 9, 3001
    mask = _mask(b, a, 5)
    mask[3] = 0            # a row without any action token: the reward lands on its last column
    mask[4, -1] = 1
    kl = torch.randn(b, a, generator=g) * 0.1
    values = torch.randn(b, a, generator=g) if gae else None
    r = torch.randn(b, generator=g) * 3
    clip = (-2.0, 2.0)
    gamma, lambd = 0.99, 0.95
    dm = mask.to(mask_dtype).to(cuda)
    dkl, dr = kl.to(cuda), r.to(cuda)
    dv = None if values is None else values.to(cuda)

    adv, ret, total = reward_advantages_and_returns(dr, 0.05, dkl, dv, dm, gamma, lambd, reward_clip_range=clip)
    rew = compute_reward(dr, 0.05, dkl, dm, reward_clip_range=clip)
    if gae:
        adv2, ret2 = get_advantages_and_returns(dv, rew, dm, gamma, lambd)
        assert torch.equal(adv, adv2)
    else:
        ret2 = get_cumulative_returns(rew, dm, gamma)
        assert adv is None
    assert torch.equal(ret, ret2)
    _rel_close(total, rew.double().sum(-1).cpu(), 1e-6)

    o_rew = otn.compute_reward(r.double(), 0.05, kl.double(), mask, clip)
    if gae:
        o_adv, o_ret = oa.get_advantages_and_returns(values.double(), o_rew, mask, gamma, lambd)
        _rel_close(adv, o_adv)
    else:
        o_ret = oa.get_cumulative_returns(o_rew, mask, gamma)
    _rel_close(ret, o_ret)
    _rel_close(total, o_rew.sum(-1), 1e-5)

    # packed rows (a row of length zero among them), starts on every residue
    keep = torch.ones(b, a, dtype=torch.bool)
    lens = torch.tensor([3001, 17, 1024, 0, 2050, 1, 1027, 4, 999])
    keep = torch.arange(a)[None, :] < lens[:, None]
    fields = dict(kl=dkl, mask=dm)
    if gae:
        fields["v"] = dv
    ps = PackedSteps.from_padded(fields, keep.to(cuda))
    p_adv, p_ret, p_total = reward_advantages_and_returns(dr, 0.05, ps["kl"], ps["v"] if gae else None, ps["mask"],
                                                          gamma, lambd, reward_clip_range=clip, cu_seqlens=ps.cu_seqlens)
    p_rew = compute_reward(dr, 0.05, ps["kl"], ps["mask"], reward_clip_range=clip, cu_seqlens=ps.cu_seqlens, max_seqlen=a)
    if gae:
        q_adv, q_ret = get_advantages_and_returns(ps["v"], p_rew, ps["mask"], gamma, lambd, cu_seqlens=ps.cu_seqlens)
        assert torch.equal(p_adv, q_adv)
    else:
        q_ret = get_cumulative_returns(p_rew, ps["mask"], gamma, cu_seqlens=ps.cu_seqlens)
    assert torch.equal(p_ret, q_ret)
    cu = ps.cu_seqlens.cpu()
    for i in range(b):
        seg = p_rew[cu[i]:cu[i + 1]].double().sum().item()
        assert abs(p_total[i].item() - seg) <= 1e-6 * max(1.0, abs(seg))


def test_reward_scan_argument_errors(cuda):
    from openrlhf_amd.trainer.ppo_utils.experience_maker import reward_advantages_and_returns

    kl = torch.zeros(2, 8, device=cuda)
    with pytest.raises(ValueError):
        reward_advantages_and_returns(torch.zeros(3, device=cuda), 0.0, kl, None, None, 1.0)
    with pytest.raises(ValueError):
        reward_advantages_and_returns(torch.zeros(2, device=cuda), 0.0, kl, torch.zeros(2, 7, device=cuda), None, 1.0, 1.0)
    adv, ret, total = reward_advantages_and_returns(torch.ones(2, device=cuda), 0.0, kl, None, None, 1.0)
    assert adv is None and torch.equal(ret, torch.ones(2, 8, device=cuda)) and torch.equal(total, torch.ones(2, device=cuda))

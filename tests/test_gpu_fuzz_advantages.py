"""Seeded random sweep over the row kernels of experience making: per-token reward, GAE and
discounted returns (separately and in one pass), the KL block and masked_normalize; shapes, mask
patterns and dtypes, storage offsets and the padded / packed layouts drawn at random, against the
fp64 oracle's restatement of the reference loops."""
import random

import pytest
import torch

from oracle import advantages as oa
from oracle import token_numerics as otn

pytestmark = pytest.mark.gpu


def _rel(got, ref, rtol, tag, at_least=1e-30):
    """Within rtol of the largest reference entry, or of `at_least` (the size of the inputs, where
    the outputs are differences of them and may all be small)."""
    got, ref = got.detach().cpu().double(), ref.detach().double()
    assert got.shape == ref.shape, tag
    if ref.numel() == 0:
        return
    scale = max(ref.abs().max().item(), at_least)
    assert (got - ref).abs().max().item() <= rtol * scale, (tag, (got - ref).abs().max().item(), scale)


def _mask(rng, g, b, a):
    lens = torch.randint(0 if rng.random() < 0.2 else 1, a + 1, (b,), generator=g)
    left = torch.randint(0, max(1, a // 3), (b,), generator=g)
    cols = torch.arange(a)[None, :]
    m = (cols < lens[:, None]) & (cols >= left[:, None])
    if a > 8 and rng.random() < 0.5:
        m[torch.arange(b), torch.randint(0, a, (b,), generator=g)] = False
    return m


def _offset(t, off, dev):
    """t on the device, in storage that starts `off` elements past an allocation boundary."""
    t = t.to(dev)
    if off == 0 or t.numel() == 0:
        return t
    buf = torch.empty(t.numel() + off, dtype=t.dtype, device=dev)
    view = buf[off:].view(t.shape)
    view.copy_(t)
    return view


@pytest.mark.parametrize("seed", list(range(36)) + [2325, 2648, 3639])
def test_random_rows(cuda, seed):
    from openrlhf_amd.models.utils import compute_reward, masked_normalize
    from openrlhf_amd.trainer.ppo_utils.experience_maker import (
        experience_kl, get_advantages_and_returns, get_cumulative_returns, reward_advantages_and_returns)

    rng = random.Random(900 + seed)
    g = torch.Generator().manual_seed(seed)
    b = rng.choice([1, 3, 8, 41])
    a = rng.choice([1, 4, 63, 1023, 1024, 1025, 2049, 5000, 8191]) if b < 20 else rng.choice([1, 77, 1500])
    mask = _mask(rng, g, b, a)
    mask_dtype = rng.choice([torch.bool, torch.float32, torch.int64, None])
    off = rng.choice([0, 0, 1, 2, 3])
    gamma, lambd = rng.choice([1.0, 0.99, 0.9]), rng.choice([1.0, 0.95, 0.5])
    clip = rng.choice([None, (-1.0, 1.0)])
    kl_coef = rng.choice([0.0, 0.02, -1.0])
    est = rng.choice(["k1", "k2", "k3"])
    tag = (seed, b, a, mask_dtype, off, gamma, lambd, clip, kl_coef, est)

    lp = -torch.rand(b, a, generator=g) * 2
    base = lp + torch.randn(b, a, generator=g) * 0.3
    values = torch.randn(b, a, generator=g)
    r = torch.randn(b, generator=g) * 2
    m64 = mask.double() if mask_dtype is not None else torch.ones(b, a, dtype=torch.float64)
    dm = None if mask_dtype is None else _offset(mask.to(mask_dtype), off, cuda)
    put = lambda t: _offset(t, off, cuda)  # noqa: E731

    # KL block
    kl, kl_mean, diff_mean = experience_kl(put(lp), put(base), dm, est)
    o_kl, o_klm, o_dm = otn.experience_kl(lp.double(), base.double(), m64, est)
    assert (kl.cpu().double() - o_kl).abs().max().item() <= 1e-5, tag
    live = m64.sum(1) > 0
    assert (kl_mean.cpu().double() - o_klm)[live].abs().max().item() <= 1e-5 if live.any() else True, tag
    assert (diff_mean.cpu().double() - o_dm)[live].abs().max().item() <= 1e-5 if live.any() else True, tag
    assert torch.isnan(kl_mean.cpu()[~live]).all(), tag

    # reward, scans, and both in one pass
    o_rew = otn.compute_reward(r.double(), kl_coef, o_kl, m64, clip)
    rew = compute_reward(r.to(cuda), kl_coef, put(o_kl.float()), dm, reward_clip_range=clip)
    _rel(rew, o_rew, 1e-6, tag)
    o_adv, o_ret = oa.get_advantages_and_returns(values.double(), o_rew, m64, gamma, lambd)
    adv, ret = get_advantages_and_returns(put(values), put(o_rew.float()), dm, gamma, lambd)
    _rel(adv, o_adv, 1e-5, tag)
    _rel(ret, o_ret, 1e-5, tag)
    o_g = oa.get_cumulative_returns(o_rew, m64, gamma)
    _rel(get_cumulative_returns(put(o_rew.float()), dm, gamma), o_g, 1e-5, tag)
    f_adv, f_ret, f_sum = reward_advantages_and_returns(r.to(cuda), kl_coef, put(o_kl.float()), put(values), dm,
                                                        gamma, lambd, reward_clip_range=clip)
    _rel(f_adv, o_adv, 1e-5, tag)
    _rel(f_ret, o_ret, 1e-5, tag)
    _rel(f_sum, o_rew.sum(1), 1e-5, tag)
    n_adv, n_ret, n_sum = reward_advantages_and_returns(r.to(cuda), kl_coef, put(o_kl.float()), None, dm, gamma,
                                                        reward_clip_range=clip)
    assert n_adv is None, tag
    _rel(n_ret, o_g, 1e-5, tag)

    # masked_normalize
    # masked_normalize: the reference forms x - mean in fp32, and a row whose kept values nearly
    # coincide divides that rounding (2^-24 |x|) by its tiny standard deviation
    if mask_dtype is not None:
        want = otn.masked_normalize(values.double(), m64)
        cnt = m64.sum(1, keepdim=True).clamp(min=1)
        mean = (values.double() * m64).sum(1, keepdim=True) / cnt
        var = ((((values.double() - mean) * m64) ** 2).sum(1, keepdim=True) / cnt).clamp(min=1e-8)
        slack = 2.0 ** -22 * values.abs().amax(1, keepdim=True).double() * var.rsqrt()
        err = (masked_normalize(put(values), dm).cpu().double() - want).abs()
        assert bool((err <= 2e-5 * max(want.abs().max().item(), 1e-30) + slack).all()), (tag, err.max().item())

    # packed layout: each row from its first to its last kept column, holes included
    if mask.any(1).all():
        first = mask.float().argmax(1)
        end = a - mask.flip(1).float().argmax(1)
        cu = torch.cat([torch.zeros(1, dtype=torch.long), (end - first).cumsum(0)]).to(cuda)
        pick = torch.cat([torch.arange(int(f), int(e)) + i * a for i, (f, e) in enumerate(zip(first, end))])
        pk = lambda t: _offset(t.reshape(-1)[pick], off, cuda)  # noqa: E731
        pm = None if mask_dtype is None else pk(mask.to(mask_dtype))
        p_adv, p_ret, p_sum = reward_advantages_and_returns(r.to(cuda), kl_coef, pk(o_kl.float()), pk(values), pm,
                                                            gamma, lambd, reward_clip_range=clip, cu_seqlens=cu)
        # the oracle on each row's own extent
        for i in range(b):
            f, e = int(first[i]), int(end[i])
            row_m = m64[i:i + 1, f:e]
            row_rew = otn.compute_reward(r[i:i + 1].double(), kl_coef, o_kl[i:i + 1, f:e], row_m, clip)
            ra, rr = oa.get_advantages_and_returns(values[i:i + 1, f:e].double(), row_rew, row_m, gamma, lambd)
            lo, hi = int(cu[i]), int(cu[i + 1])
            size = max(values[i, f:e].abs().max().item(), row_rew.abs().max().item())
            _rel(p_adv[lo:hi], ra[0], 1e-5, tag, at_least=size)
            _rel(p_ret[lo:hi], rr[0], 1e-5, tag, at_least=size)
            assert abs(p_sum[i].item() - row_rew.sum().item()) <= 1e-5 * max(1.0, row_rew.abs().sum().item()), tag

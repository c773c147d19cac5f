"""Seeded random sweep over the per-token losses: shapes, mask patterns and dtypes, clip /
dual-clip / importance-correction / GSPO settings, normalisers and layouts drawn at random;
values and gradients against the fp64 oracle and torch autograd through it, and the packed
layout against the padded one."""
import random

import pytest
import torch

from oracle import losses as ol

pytestmark = pytest.mark.gpu


def _mask(rng, g, b, a):
    lens = torch.randint(0 if rng.random() < 0.3 else 1, a + 1, (b,), generator=g)
    left = torch.randint(0, max(1, a // 3), (b,), generator=g)
    cols = torch.arange(a)[None, :]
    m = (cols < lens[:, None]) & (cols >= left[:, None])
    if a > 8 and rng.random() < 0.5:
        m[torch.arange(b), torch.randint(0, a, (b,), generator=g)] = False
    if not m.any():
        m[0, 0] = True
    return m


def _on_an_edge(lp, old, roll, mask, cfg, kind, margin=2e-6):
    """Entries that sit on a step: the clipped surrogate, the dual clip and the importance filters
    are step functions of a ratio, so an entry whose ratio lies within `margin` (relative) of a
    threshold may take one branch in fp32 and the other in the fp64 oracle (among 300 000 entries
    one does now and then), which moves its gradient and the loss by that entry's whole term.
    Token-level ratios mark their entry, sequence-level ones (GSPO, seq-mask-tis) their whole row."""
    m = mask.double()
    cnt = m.sum(-1, keepdim=True).clamp(min=1)

    def near(x, *edges):
        hit = torch.zeros_like(x, dtype=torch.bool)
        for e in edges:
            if e is not None:
                hit |= (x - e).abs() <= margin * abs(e)
        return hit

    if kind.startswith("gspo"):
        log_ratio = (lp.double() - roll.double()) if kind == "gspo-is" else (lp.double() - old.double())
        ratio = ((log_ratio * m).sum(-1, keepdim=True) / cnt).exp().expand_as(m)
    else:
        ratio = (lp.double() - old.double()).clamp(-20.0, 20.0).exp()
    edge = near(ratio, 1 - cfg["clip_eps_low"], 1 + cfg["clip_eps_high"], cfg["dual_clip"])
    if kind in ("tis", "icepop", "seq-mask-tis"):
        lo, hi = cfg["vllm_is_truncated_threshold"]
        log_is = old.double() - roll.double()
        edge |= near(log_is.exp(), lo, hi)
        if kind == "seq-mask-tis":
            edge |= near(((log_is * m).sum(-1, keepdim=True) / cnt).exp().expand_as(m), lo, hi)
    return edge


@pytest.mark.parametrize("seed", list(range(40)) + [1760, 1934, 2972])
def test_random_policy_and_value_loss(cuda, seed):
    from openrlhf_amd.models.loss import PolicyLoss, ValueLoss

    rng = random.Random(500 + seed)
    g = torch.Generator().manual_seed(seed)
    b = rng.choice([1, 2, 7, 33, 200])
    a = rng.choice([1, 5, 255, 1024, 4095, 4097, 9000]) if b < 100 else rng.choice([1, 17, 300])
    mask = _mask(rng, g, b, a)
    lp = -torch.rand(b, a, generator=g) * 3
    old = lp + torch.randn(b, a, generator=g) * rng.choice([0.01, 0.2, 1.0])
    roll = old + torch.randn(b, a, generator=g) * 0.05
    adv = torch.randn(b, a, generator=g)
    cfg = dict(clip_eps_low=rng.choice([0.1, 0.2]), clip_eps_high=rng.choice([0.2, 0.28]),
               dual_clip=rng.choice([None, None, 3.0]), token_level_loss=rng.random() < 0.5)
    kind = rng.choice(["ppo", "ppo", "tis", "icepop", "seq-mask-tis", "gspo", "gspo-is"])
    if kind in ("tis", "icepop", "seq-mask-tis"):
        cfg.update(enable_vllm_is_correction=True, vllm_is_truncated_threshold=[0.9, 1.1], vllm_is_correction_type=kind)
    elif kind.startswith("gspo"):
        cfg.update(policy_loss_type="gspo")
        if kind == "gspo-is":
            cfg.update(enable_vllm_is_correction=True, vllm_is_truncated_threshold=[0.5, 2.0])
    for _ in range(4):  # entries drawn onto a step are moved off it: the comparison is about arithmetic, not about ties
        edge = _on_an_edge(lp, old, roll, mask, {"dual_clip": None, **cfg}, kind)
        if not edge.any():
            break
        lp, roll = torch.where(edge, lp + 1e-3, lp), torch.where(edge, roll - 2e-3, roll)
    assert not _on_an_edge(lp, old, roll, mask, {"dual_clip": None, **cfg}, kind).any()
    info = rng.choice([{}, dict(dp_size=2, batch_num_tokens=float(mask.sum()) * 1.7, global_batch_size=float(b) * 1.3)])
    mask_dtype = rng.choice([torch.bool, torch.float32, torch.int64])
    use_roll = cfg.get("enable_vllm_is_correction", False)
    tag = (seed, b, a, kind, cfg, bool(info), mask_dtype)

    x64 = lp.double().requires_grad_(True)
    ref = ol.policy_loss(x64, old.double(), adv.double(), mask.double(), roll.double() if use_roll else None, **cfg, **info)
    (g_ref,) = torch.autograd.grad(ref[0], x64)
    xd = lp.to(cuda).requires_grad_(True)
    pol = PolicyLoss(**cfg)
    out = pol(xd, old.to(cuda), adv.to(cuda), action_mask=mask.to(mask_dtype).to(cuda),
              rollout_log_probs=roll.to(cuda) if use_roll else None, **info)
    for got, want in zip(out, ref):
        if want is None:
            assert got is None, tag
            continue
        w = want.detach().item()
        assert abs(got.item() - w) <= 1e-5 * max(1.0, abs(w)) or (w != w and got.item() != got.item()), (tag, got.item(), w)
    (gd,) = torch.autograd.grad(out[0], xd)
    gs = max(1e-12, g_ref.abs().max().item())
    assert (gd.cpu().double() - g_ref).abs().max().item() <= 2e-5 * gs, tag

    # packed layout of the same rows (extent of the mask, holes kept) gives the same numbers
    nz = mask.any(1)
    if nz.all() and kind != "seq-mask-tis":
        first = mask.float().argmax(1)
        end = a - mask.flip(1).float().argmax(1)
        cu = torch.cat([torch.zeros(1, dtype=torch.long), (end - first).cumsum(0)])
        pick = torch.cat([torch.arange(int(f), int(e)) + r * a for r, (f, e) in enumerate(zip(first, end))])
        pk = lambda t: t.reshape(-1)[pick].to(cuda)  # noqa: E731
        xp = pk(lp).requires_grad_(True)
        outp = pol(xp, pk(old), pk(adv), action_mask=pk(mask.to(mask_dtype)), rollout_log_probs=pk(roll) if use_roll else None,
                   cu_seqlens=cu.to(cuda), max_seqlen=a, **info)
        assert abs(outp[0].item() - out[0].item()) <= 2e-6 * max(1.0, abs(out[0].item())), tag
        (gp,) = torch.autograd.grad(outp[0], xp)
        assert (gp - gd.reshape(-1)[pick.to(cuda)]).abs().max().item() <= 1e-6 * gs + 1e-12, tag

    # value loss on the same shapes
    clip = rng.choice([None, 0.2, 0.5])
    tl = rng.random() < 0.5
    v64 = adv.double().requires_grad_(True)
    vref = ol.value_loss(v64, old.double(), lp.double(), mask.double(), clip_eps=clip, token_level_loss=tl, **info)
    (gv_ref,) = torch.autograd.grad(vref, v64)
    vd = adv.to(cuda).requires_grad_(True)
    vgot = ValueLoss(clip, tl)(vd, old.to(cuda), lp.to(cuda), action_mask=mask.to(mask_dtype).to(cuda), **info)
    assert abs(vgot.item() - vref.item()) <= 1e-5 * max(1.0, abs(vref.item())), tag
    (gv,) = torch.autograd.grad(vgot, vd)
    assert (gv.cpu().double() - gv_ref).abs().max().item() <= 2e-5 * max(1e-12, gv_ref.abs().max().item()), tag

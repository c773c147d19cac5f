"""Seeded random sweep over the lm-head + log-prob / entropy path: token counts, hidden sizes (any
even number), vocabularies, dtypes, temperatures, padded row strides and row masks drawn at random,
and the memory budget for kept logits (none, a sliver, everything), every case against the fp64
oracle applied to ``hidden @ W.T`` rounded to the 16-bit dtype as the lm_head output is
(tests/lmhead_util.py; values 2e-3 abs; gradients within the rounding of a 16-bit logits gradient
and a 16-bit result)."""
import random

import pytest
import torch

from oracle import token_numerics as otn
from tests.lmhead_util import straight_through_logits

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", list(range(40)) + [42, 229, 255, 5024, 5025, 5028, 5044, 5051, 5054, 2064])  # the last seven: a vocabulary of one entry
def test_random_case(cuda, seed):
    from openrlhf_amd.models.utils import lm_head_logprobs_and_entropy

    rng = random.Random(7000 + seed)
    dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16])
    n = rng.choice([1, 2, 63, 64, 255, 256, 257]) if rng.random() < 0.4 else rng.randint(1, 700)
    hdim = 2 * (rng.choice([1, 4, 31, 32, 33, 64, 100]) if rng.random() < 0.5 else rng.randint(1, 300))
    vocab = rng.choice([1, 2, 255, 256, 257, 1000]) if rng.random() < 0.4 else rng.randint(1, 3000)
    temperature = rng.choice([1.0, 1.0, 0.6, 1.5])
    pad_h, pad_w = 2 * rng.choice([0, 0, 1, 4]), 2 * rng.choice([0, 0, 3])
    use_mask = rng.random() < 0.5
    keep_mib = rng.choice([None, None, 0.3, 1e6])       # drawn last: the earlier draws of a seed stay what they were
    info = (seed, dtype, n, hdim, vocab, temperature, pad_h, pad_w, use_mask, keep_mib)

    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(n, hdim, generator=g).to(dtype)
    weight = (torch.randn(vocab, hdim, generator=g) * (2.0 / hdim ** 0.5)).to(dtype)
    labels = torch.randint(0, vocab, (n,), generator=g)
    mask = (torch.rand(n, generator=g) > 0.3) if use_mask else None
    g_lp, g_ent = torch.randn(n, generator=g), torch.randn(n, generator=g)

    h64 = hidden.double().requires_grad_(True)
    w64 = weight.double().requires_grad_(True)
    logits = straight_through_logits(hidden, weight, h64, w64, cuda)
    km = torch.ones(n, dtype=torch.float64) if mask is None else mask.double()
    ref_lp = otn.log_probs_from_logits(logits, labels, temperature) * km
    ref_ent = otn.compute_entropy(logits) * km
    torch.autograd.backward([ref_lp, ref_ent], [g_lp.double(), g_ent.double()])

    # operands as views with padded row strides (NaN in the padding: it must never be read)
    hbuf = torch.full((n, hdim + pad_h), float("nan"), dtype=dtype, device=cuda)
    wbuf = torch.full((vocab, hdim + pad_w), float("nan"), dtype=dtype, device=cuda)
    hbuf[:, :hdim] = hidden.to(cuda)
    wbuf[:, :hdim] = weight.to(cuda)
    hd = hbuf[:, :hdim].requires_grad_(True)
    wd = wbuf[:, :hdim].requires_grad_(True)
    lp, ent = lm_head_logprobs_and_entropy(hd, wd, labels.to(cuda), temperature,
                                           row_mask=None if mask is None else mask.to(cuda), keep_logits_mib=keep_mib)
    assert (lp.detach().cpu().double() - ref_lp.detach()).abs().max().item() <= 2e-3, info
    assert (ent.detach().cpu().double() - ref_ent.detach()).abs().max().item() <= 2e-3, info
    if mask is not None and not bool(mask.any()):
        return  # nothing to differentiate
    gh, gw = torch.autograd.grad([lp, ent], [hd, wd], [g_lp.to(cuda), g_ent.to(cuda)])
    eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    # the floors: softmax weights come from an fp32 exponent, so a weight that is exactly 1 (a
    # vocabulary of one entry, where every gradient is exactly 0) comes out as 1 - 2e-7, times the
    # upstream gradients (the entropy's enters twice) and the other operand; a weight gradient sums
    # that over the tokens
    gsz = g_lp.abs().max().item() + 2 * g_ent.abs().max().item()
    floor_h = 5e-7 * gsz * weight.float().abs().max().item()
    floor_w = (5e-7 + 5e-8 * n) * gsz * hidden.float().abs().max().item()
    for got, ref, floor in ((gh, h64.grad, floor_h), (gw, w64.grad, floor_w)):
        err = (got.cpu().double() - ref).abs()
        scale = ref.abs().max().item()
        assert torch.isfinite(got).all(), info
        assert err.max().item() <= 4 * eps * scale + floor, (info, err.max().item(), scale)
    if mask is not None:
        assert gh[~mask.to(cuda)].abs().max().item() == 0.0 if bool((~mask).any()) else True

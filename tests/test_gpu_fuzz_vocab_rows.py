"""Seeded random sweep over the vocabulary-row kernels: shapes, row strides, base misalignment,
dtypes, temperatures, row masks and output selections drawn at random, every case checked
against the fp64 oracle (forward, two-kernel backward and the one-pass kernel)."""
import random

import pytest
import torch

from oracle import token_numerics as otn

pytestmark = pytest.mark.gpu

_DT = {torch.float32: (1e-5, 2e-5), torch.bfloat16: (2e-3, 2.0 ** -8), torch.float16: (2e-3, 2.0 ** -10)}


def _case(rng):
    dtype = rng.choice([torch.float32, torch.bfloat16, torch.bfloat16, torch.float16])
    vocab = rng.choice([1, 2, 7, 8, 9, 63, 64, 65, 255, 1000, 4097, 32000, 50257]) if rng.random() < 0.7 \
        else rng.randint(1, 70000)
    rows = rng.randint(1, 40 if vocab > 20000 else 300)
    pad = rng.choice([0, 0, 1, 3, 8, 17])
    shift = rng.choice([0, 0, 1, 2, 3, 5])  # elements the base is moved off its natural alignment
    temperature = rng.choice([1.0, 1.0, 0.6, 1.7])
    std = rng.choice([0.5, 2.0, 4.0]) if dtype != torch.float16 else rng.choice([0.5, 2.0])
    return dtype, vocab, rows, pad, shift, temperature, std


def _maxabs(t):
    """max |t|, 0 for an empty selection (every row masked out)."""
    return t.abs().max().item() if t.numel() else 0.0


@pytest.mark.parametrize("seed", range(48))
def test_random_case(cuda, seed):
    from openrlhf_amd.models.utils import fused_logprob_entropy_fwd_bwd, logprobs_and_entropy_from_logits

    rng = random.Random(1000 + seed)
    dtype, vocab, rows, pad, shift, temperature, std = _case(rng)
    g = torch.Generator().manual_seed(seed)
    stride = vocab + pad
    x = (torch.randn(rows, vocab, generator=g) * std).to(dtype)
    labels = torch.randint(0, vocab, (rows,), generator=g)
    keep = torch.rand(rows, generator=g) > 0.25 if rng.random() < 0.5 else None
    g_lp, g_ent = torch.randn(rows, generator=g), torch.randn(rows, generator=g)

    def device_rows():  # [rows, vocab] view with the drawn stride and base offset
        flat = torch.zeros(rows * stride + shift + 8, dtype=dtype, device=cuda)
        view = flat[shift: shift + rows * stride].view(rows, stride)[:, :vocab]
        view.copy_(x.to(cuda))
        return view

    x64 = x.double().requires_grad_(True)
    lp_ref = otn.log_probs_from_logits(x64, labels, temperature)
    ent_ref = otn.compute_entropy(x64)
    km = torch.ones(rows) if keep is None else keep.double()
    (g_ref,) = torch.autograd.grad((lp_ref * g_lp.double() * km).sum() + (ent_ref * g_ent.double() * km).sum(), x64)
    atol, gtol = _DT[dtype]
    # rounding error of (onehot - p) * g_lp is relative to g_lp / T even where the exact value is 0 (V = 1)
    gscale = max(g_ref.abs().max().item(), g_lp.abs().max().item() / temperature)
    info = (seed, dtype, vocab, rows, pad, shift, temperature)

    xd = device_rows().requires_grad_(True)
    rm = None if keep is None else keep.to(cuda)
    lp, ent = logprobs_and_entropy_from_logits(xd, labels.to(cuda), temperature, row_mask=rm)
    sel = torch.ones(rows, dtype=torch.bool) if keep is None else keep
    assert _maxabs((lp.cpu().double() - lp_ref.detach())[sel]) <= atol * max(1.0, std), info
    assert _maxabs((ent.cpu().double() - ent_ref.detach())[sel]) <= atol * max(1.0, std), info
    if keep is not None:
        assert (lp.cpu()[~keep] == 0).all() and (ent.cpu()[~keep] == 0).all(), info
    (gd,) = torch.autograd.grad((lp * g_lp.to(cuda)).sum() + (ent * g_ent.to(cuda)).sum(), xd)
    assert (gd.cpu().double() - g_ref).abs().max().item() <= gtol * gscale + 1e-12, info

    xf = device_rows()
    lp1, ent1, grad1 = fused_logprob_entropy_fwd_bwd(xf, labels.to(cuda), g_lp.to(cuda), g_ent.to(cuda),
                                                     temperature=temperature, inplace=bool(seed % 2), row_mask=rm)
    assert _maxabs((lp1.cpu().double() - lp_ref.detach())[sel]) <= atol * max(1.0, std), info
    assert _maxabs((ent1.cpu().double() - ent_ref.detach())[sel]) <= atol * max(1.0, std), info
    assert (grad1.cpu().double() - g_ref).abs().max().item() <= gtol * gscale + 1e-12, info

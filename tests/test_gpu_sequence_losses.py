"""Sequence-level kernels next to the hot path: DPO per-sequence log-prob sums
(openrlhf/trainer/dpo_trainer.py:362-382), DPOLoss / PairWiseLoss / LogExpLoss
(openrlhf/models/loss.py:272-335) and the SFT / DPO loss steps built on them, against the oracle
and the committed golden vectors. Tolerances: 1e-5 relative for sums of fp32 log-probs (like the
scans), 1e-5 absolute for the losses."""
import json
import math
import os

import pytest
import torch

from oracle import losses as ol
from oracle import token_numerics as otn

pytestmark = pytest.mark.gpu

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "token_numerics_golden.json")))
REL = 1e-5
ABS = 1e-5


def _close(got, ref, tol, relative=False):
    got, ref = got.detach().cpu().double(), torch.as_tensor(ref, dtype=torch.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    nan_g, nan_r = torch.isnan(got), torch.isnan(ref)
    assert torch.equal(nan_g, nan_r)
    scale = max(1.0, ref[~nan_r].abs().max().item()) if relative and (~nan_r).any() else 1.0
    if (~nan_r).any():
        err = (got[~nan_r] - ref[~nan_r]).abs().max().item()
        assert err <= tol * scale, (err, tol * scale)


def test_sequence_logps_golden(cuda):
    from openrlhf_amd.trainer.dpo_trainer import get_batch_logps

    s = GOLD["sequence_logps"]
    lp = torch.tensor(GOLD["tokens"]["log_probs"], dtype=torch.float32, device=cuda, requires_grad=True)
    att = torch.tensor(s["attention_mask"], device=cuda)
    sums, means = get_batch_logps(lp, att, s["prompt_id_lens"])
    _close(sums, s["sums"], REL, relative=True)
    _close(means, [math.nan if m is None else m for m in s["means"]], REL, relative=True)
    keep = [b for b, m in enumerate(s["means"]) if m is not None]
    gs = torch.tensor(s["g_sums"], device=cuda)
    gm = torch.tensor(s["g_means"], device=cuda)
    gm_used = torch.zeros_like(gm)
    gm_used[keep] = gm[keep]
    (g,) = torch.autograd.grad((sums * gs).sum() + (means * gm_used).sum(), lp)
    for b in keep:
        _close(g[b], s["grad"][b], ABS)
    # a sequence without response tokens: the reference's 0 * (g / 0) = NaN gradient
    empty = [b for b, m in enumerate(s["means"]) if m is None]
    assert torch.isnan(g[empty]).all()


@pytest.mark.parametrize("mask_dtype", [torch.bool, torch.int64, torch.float32, torch.int32])
@pytest.mark.parametrize("shape", [(1, 1), (5, 300), (37, 1031)])
def test_sequence_logps_vs_oracle(cuda, mask_dtype, shape):
    from openrlhf_amd.trainer.dpo_trainer import get_batch_logps, response_mask

    b, a = shape
    g = torch.Generator().manual_seed(11 * b + a)
    lp = -torch.rand(b, a, generator=g, dtype=torch.float64) * 9
    lens = torch.randint(1, a + 2, (b,), generator=g)
    left = torch.randint(0, 3, (b,), generator=g)
    cols = torch.arange(a + 1)[None, :]
    att = ((cols < lens[:, None]) & (cols >= left[:, None])).long()
    prompt = torch.minimum(torch.randint(0, a + 2, (b,), generator=g), lens)
    prompt[0] = 0
    ref_in = lp.clone().requires_grad_(True)
    r_sums, r_means = ol.get_batch_logps(ref_in, att, prompt.tolist())
    x = lp.float().to(cuda).requires_grad_(True)
    sums, means = get_batch_logps(x, att.to(mask_dtype).to(cuda), prompt.tolist())
    _close(sums, r_sums.detach(), REL, relative=True)
    _close(means, r_means.detach(), REL, relative=True)
    ok = ~torch.isnan(r_means.detach())
    w1 = torch.randn(b, generator=g, dtype=torch.float64)
    w2 = torch.randn(b, generator=g, dtype=torch.float64) * ok
    (rg,) = torch.autograd.grad((r_sums * w1).sum() + (r_means[ok] * w2[ok]).sum(), ref_in)
    (gg,) = torch.autograd.grad((sums * w1.float().to(cuda)).sum() + (means * w2.float().to(cuda)).sum(), x)
    _close(gg[ok.to(cuda)], rg[ok], ABS)
    # bit-exact mask: the on-the-fly mask equals the reference's clone / clear / shift construction
    ref_mask = att.clone().bool()
    for row, p in zip(ref_mask, prompt.tolist()):
        row[:p] = False
    assert torch.equal(response_mask(att.to(cuda), prompt.tolist()).cpu(), ref_mask[:, 1:])
    # tensor prompt lengths behave like the list
    sums_t, _ = get_batch_logps(x, att.to(mask_dtype).to(cuda), prompt.to(cuda))
    assert torch.equal(sums_t, sums)


def test_pair_losses_golden(cuda):
    from openrlhf_amd.models.loss import DPOLoss, LogExpLoss, PairWiseLoss

    p = GOLD["pair_loss"]
    dev = lambda k: torch.tensor(p[k], dtype=torch.float32, device=cuda)  # noqa: E731
    for case in p["dpo"]:
        c, r = dev("chosen").requires_grad_(True), dev("rejected").requires_grad_(True)
        loss, cr, rr = DPOLoss(case["beta"], case["label_smoothing"], case["ipo"])(c, r, dev("ref_chosen"), dev("ref_rejected"))
        tol = ABS * max(1.0, abs(case["out"]["loss"]))
        _close(loss, case["out"]["loss"], tol)
        _close(cr, case["out"]["chosen_rewards"], ABS)
        _close(rr, case["out"]["rejected_rewards"], ABS)
        assert not cr.requires_grad and not rr.requires_grad
        gc, gr = torch.autograd.grad(loss, (c, r))
        gtol = ABS * max(1.0, max(abs(v) for v in case["out"]["g_chosen"]))
        _close(gc, case["out"]["g_chosen"], gtol)
        _close(gr, [-v for v in case["out"]["g_chosen"]], gtol)
    a, b, m = dev("chosen_reward"), dev("reject_reward"), dev("margin")
    _close(PairWiseLoss()(a, b), p["pairwise"]["loss"], ABS)
    _close(PairWiseLoss()(a, b, m), p["pairwise_margin"]["loss"], ABS)
    _close(LogExpLoss()(a, b), p["logexp"]["loss"], ABS)
    _close(LogExpLoss()(a, b, m), p["logexp"]["loss"], ABS)  # margin ignored, as in the reference
    a.requires_grad_(True)
    (ga,) = torch.autograd.grad(PairWiseLoss()(a, b, m), a)
    _close(ga, p["pairwise_margin"]["g_chosen"], ABS)
    (ga,) = torch.autograd.grad(LogExpLoss()(a, b), a)
    _close(ga, p["logexp"]["g_chosen"], ABS)


@pytest.mark.parametrize("n", [1, 64, 1000])
def test_pair_losses_vs_oracle(cuda, n):
    from openrlhf_amd.models.loss import DPOLoss, LogExpLoss, PairWiseLoss

    g = torch.Generator().manual_seed(n)
    c = torch.randn(n, generator=g, dtype=torch.float64) * 20 - 50
    r = c + torch.randn(n, generator=g, dtype=torch.float64) * 8
    rc = c + torch.randn(n, generator=g, dtype=torch.float64) * 2
    rr = r + torch.randn(n, generator=g, dtype=torch.float64) * 2
    for beta, smooth, ipo in ((0.1, 0.0, False), (0.3, 0.2, False), (0.05, 0.0, True)):
        c32 = c.float()
        r32 = r.float()
        cref, rref = c32.double().requires_grad_(True), r32.double().requires_grad_(True)
        ref_loss, ref_cr, ref_rr = ol.dpo_loss(cref, rref, rc.float().double(), rr.float().double(), beta, smooth, ipo)
        cg, rg = c32.to(cuda).requires_grad_(True), r32.to(cuda).requires_grad_(True)
        loss, cr, rr_ = DPOLoss(beta, smooth, ipo)(cg, rg, rc.float().to(cuda), rr.float().to(cuda))
        # the logit is formed in fp32 from values of magnitude ~50: its rounding (3e-6) times the slope
        scale = max(1.0, ref_loss.abs().item())
        _close(loss, ref_loss.detach(), 3e-5 * scale)
        _close(cr, ref_cr, ABS)
        _close(rr_, ref_rr, ABS)
        ref_g = torch.autograd.grad(ref_loss, (cref, rref))
        got_g = torch.autograd.grad(loss, (cg, rg))
        gscale = max(1.0, ref_g[0].abs().max().item())
        _close(got_g[0], ref_g[0], 3e-5 * gscale)
        _close(got_g[1], ref_g[1], 3e-5 * gscale)
    a = (torch.randn(n, generator=g) * 3)
    b = (torch.randn(n, generator=g) * 3)
    m = torch.rand(n, generator=g)
    for fn, ref_fn, margin in ((PairWiseLoss(), ol.pairwise_loss, None), (PairWiseLoss(), ol.pairwise_loss, m),
                               (LogExpLoss(), ol.logexp_loss, None)):
        aref = a.double().requires_grad_(True)
        ref = ref_fn(aref, b.double(), None if margin is None else margin.double())
        ag = a.to(cuda).requires_grad_(True)
        out = fn(ag, b.to(cuda), None if margin is None else margin.to(cuda))
        _close(out, ref.detach(), ABS)
        _close(torch.autograd.grad(out, ag)[0], torch.autograd.grad(ref, aref)[0], ABS)


def test_pair_losses_extremes_match_torch_fp32(cuda):
    """Saturated logits, the unguarded exp of LogExpLoss and the empty batch behave as the
    reference's fp32 torch expressions do."""
    from openrlhf_amd.models.loss import DPOLoss, LogExpLoss, PairWiseLoss

    c = torch.tensor([0.0, 500.0, -500.0, 3.0, 100.0])
    r = torch.tensor([0.0, -500.0, 500.0, 3.0, 0.0])
    z = torch.zeros_like(c)
    ref = ol.dpo_loss(c, r, z, z, 1.0)[0]
    assert torch.isfinite(ref)
    _close(DPOLoss(1.0)(c.to(cuda), r.to(cuda), z.to(cuda), z.to(cuda))[0], ref.double(), 1e-4 * ref.item())
    _close(PairWiseLoss()(c.to(cuda), r.to(cuda)), ol.pairwise_loss(c, r).double(), 1e-4 * ref.item())
    ref = ol.logexp_loss(c, r)  # exp(1000) overflows: inf, like the reference
    got = LogExpLoss()(c.to(cuda), r.to(cuda))
    assert torch.isinf(ref) and torch.isinf(got.cpu())
    e = torch.empty(0, device=cuda)
    assert torch.isnan(PairWiseLoss()(e, e)) and torch.isnan(ol.pairwise_loss(e.cpu(), e.cpu()))
    with pytest.raises(ValueError):
        PairWiseLoss()(c.to(cuda), r[:3].to(cuda))
    with pytest.raises(RuntimeError):
        PairWiseLoss()(c, r)


def _dpo_batch(seed, b=3, t=40, vocab=2003):
    g = torch.Generator().manual_seed(seed)
    c_len = torch.randint(12, t + 1, (b,), generator=g)
    r_len = torch.randint(12, t - 5, (b,), generator=g)
    prompt = torch.randint(2, 10, (b,), generator=g)
    c_mask = (torch.arange(t)[None, :] < c_len[:, None]).long()
    r_mask = (torch.arange(t - 6)[None, :] < r_len[:, None]).long()
    c_ids = torch.randint(1, vocab, (b, t), generator=g) * c_mask
    r_ids = torch.randint(1, vocab, (b, t - 6), generator=g) * r_mask
    return c_ids, c_mask, r_ids, r_mask, prompt.tolist(), g


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nll_coef", [0.0, 0.3])
def test_dpo_loss_step_vs_oracle(cuda, dtype, nll_coef):
    from openrlhf_amd.models.loss import DPOLoss
    from openrlhf_amd.trainer.dpo_trainer import concatenated_inputs, dpo_loss_step

    c_ids, c_mask, r_ids, r_mask, prompt, g = _dpo_batch(5)
    ids, att, lens = concatenated_inputs(c_ids, c_mask, r_ids, r_mask, prompt, pad_token_id=0)
    assert ids.shape == (6, 40) and att.shape == (6, 40) and lens == prompt * 2
    assert torch.equal(ids[3:, :34], r_ids) and (ids[3:, 34:] == 0).all() and (att[3:, 34:] == 0).all()
    vocab = 2003
    logits = (torch.randn(6, 40, vocab, generator=g) * 2).to(dtype)
    ref_c = -torch.rand(3, generator=g) * 60
    ref_r = -torch.rand(3, generator=g) * 60
    beta = 0.1

    x64 = logits.double().requires_grad_(True)
    lp = otn.log_probs_from_logits(x64, torch.roll(ids, -1, 1), 1.0)[:, :-1]
    sums, means = ol.get_batch_logps(lp, att, lens)
    ref_pref, ref_cr, ref_rr = ol.dpo_loss(sums[:3], sums[3:], ref_c.double(), ref_r.double(), beta)
    ref_nll = -means[:3].mean()
    ref_loss = ref_pref + ref_nll * nll_coef
    (ref_g,) = torch.autograd.grad(ref_loss, x64)

    xd = logits.to(cuda).requires_grad_(True)
    out = dpo_loss_step(xd, ids.to(cuda), att.to(cuda), lens, 3, ref_c.to(cuda), ref_r.to(cuda), DPOLoss(beta),
                        nll_loss_coef=nll_coef)
    lp_tol = 1e-5 if dtype == torch.float32 else 2e-3
    _close(out["chosen_logps"], sums[:3].detach(), lp_tol * 40)
    _close(out["rejected_logps"], sums[3:].detach(), lp_tol * 40)
    _close(out["nll_loss"], ref_nll.detach(), lp_tol)
    _close(out["preference_loss"], ref_pref.detach(), 1e-4 if dtype == torch.float32 else 2e-2)
    _close(out["chosen_reward"], ref_cr, beta * lp_tol * 40)
    (gd,) = torch.autograd.grad(out["loss"], xd)
    gtol = (2e-5 if dtype == torch.float32 else 2.0 ** -8) * ref_g.abs().max().item()
    _close(gd.float(), ref_g, gtol)
    # prompt and padding positions receive exactly zero gradient
    need = torch.zeros(6, 40, dtype=torch.bool)
    m = att.clone().bool()
    for row, p in zip(m, lens):
        row[:p] = False
    need[:, :-1] = m[:, 1:]
    assert (gd.cpu()[~need] == 0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("token_level", [True, False])
@pytest.mark.parametrize("global_norm", [False, True])
def test_sft_loss_step_fused_and_unfused_vs_oracle(cuda, dtype, token_level, global_norm):
    from openrlhf_amd.models.loss import SFTLoss
    from openrlhf_amd.trainer.sft_trainer import sft_loss_step

    g = torch.Generator().manual_seed(3)
    b, t, vocab = 4, 33, 3001
    lens = torch.tensor([33, 20, 9, 27])
    att = (torch.arange(t)[None, :] < lens[:, None]).long()
    ids = torch.randint(1, vocab, (b, t), generator=g) * att
    loss_mask = att.clone()
    loss_mask[:, :5] = 0          # prompt
    loss_mask[1, 11:14] = 0       # a masked turn
    loss_mask[2] = 0              # a sample without supervised tokens
    logits = (torch.randn(b, t, vocab, generator=g) * 2).to(dtype)
    info = dict(dp_size=2, batch_num_tokens=131.0, global_batch_size=7.0) if global_norm else {}
    shifted = loss_mask[:, :-1]

    x64 = logits.double().requires_grad_(True)
    lp_ref = otn.log_probs_from_logits(x64, torch.roll(ids, -1, 1), 1.0)[:, :-1]
    ref_loss = ol.aggregate_loss(-lp_ref, shifted.double(), token_level_loss=token_level, **info)
    (ref_g,) = torch.autograd.grad(ref_loss, x64)
    tol = 1e-5 if dtype == torch.float32 else 2e-3
    gtol = (2e-5 if dtype == torch.float32 else 2.0 ** -8) * ref_g.abs().max().item()

    xd = logits.to(cuda).requires_grad_(True)
    loss, lp = sft_loss_step(xd, ids.to(cuda), att.to(cuda), loss_mask.to(cuda), SFTLoss(token_level), **info)
    _close(loss, ref_loss.detach(), tol * max(1.0, abs(ref_loss.item())))
    _close(lp * shifted.to(cuda), (lp_ref * shifted).detach(), tol)
    (gd,) = torch.autograd.grad(loss, xd)
    _close(gd.float(), ref_g, gtol)

    for scale in (1.0, 0.25):
        xf = logits.to(cuda).requires_grad_(True)
        work = xf * 1  # the step consumes the tensor it is given; keep the leaf intact
        loss_f, lp_f = sft_loss_step(work, ids.to(cuda), att.to(cuda), loss_mask.to(cuda), SFTLoss(token_level),
                                     fused=True, loss_scale=scale, **info)
        _close(loss_f, ref_loss.detach(), tol * max(1.0, abs(ref_loss.item())))
        _close(lp_f, (lp_ref * (shifted != 0)).detach(), tol)
        (loss_f * scale).backward()
        _close(xf.grad.float(), ref_g * scale, gtol * scale)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gpt_lm_loss_vs_torch_cross_entropy(cuda, dtype):
    """GPTLMLoss against the library routine the reference calls (nn.CrossEntropyLoss with
    ignore_index=-100 on the shifted logits / labels), value and gradient."""
    from openrlhf_amd.models.loss import GPTLMLoss

    g = torch.Generator().manual_seed(21)
    b, t, vocab = 3, 29, 4099
    logits = (torch.randn(b, t, vocab, generator=g) * 2).to(dtype)
    labels = torch.randint(0, vocab, (b, t), generator=g)
    labels[:, :6] = -100
    labels[1, 15:19] = -100
    labels[2, 1:] = -100  # a sample whose every shifted label is ignored
    x64 = logits.double().requires_grad_(True)
    ref = torch.nn.CrossEntropyLoss(ignore_index=-100)(x64[..., :-1, :].reshape(-1, vocab), labels[..., 1:].reshape(-1))
    (ref_g,) = torch.autograd.grad(ref, x64)
    xd = logits.to(cuda).requires_grad_(True)
    loss = GPTLMLoss()(xd, labels.to(cuda))
    _close(loss, ref.detach(), 1e-5 if dtype == torch.float32 else 2e-3)
    (gd,) = torch.autograd.grad(loss, xd)
    _close(gd.float(), ref_g, (2e-5 if dtype == torch.float32 else 2.0 ** -8) * ref_g.abs().max().item())
    assert (gd.cpu()[:, -1] == 0).all() and (gd.cpu()[2] == 0).all()
    everything_ignored = torch.full((b, t), -100)
    assert torch.isnan(GPTLMLoss()(logits.to(cuda), everything_ignored.to(cuda)))
    with pytest.raises(NotImplementedError):
        GPTLMLoss(ring_attn_group=object())


def test_sft_and_dpo_steps_from_hidden_states(cuda):
    """Both steps with the lm-head projection fused in (hidden states and lm_head.weight in place of
    logits): the oracle on ``hidden @ W.T`` rounded to bf16 as the lm_head output is
    (tests/lmhead_util.py), in fp64, values within 2e-3 (sums of up to 40 log-probs: 40 x that),
    gradients within the rounding of a bf16 logits gradient and result."""
    from tests.lmhead_util import straight_through_logits
    from openrlhf_amd.models.loss import DPOLoss, SFTLoss
    from openrlhf_amd.trainer.dpo_trainer import concatenated_inputs, dpo_loss_step
    from openrlhf_amd.trainer.sft_trainer import sft_loss_step

    hdim, vocab = 96, 1201
    c_ids, c_mask, r_ids, r_mask, prompt, g = _dpo_batch(6)
    ids, att, lens = concatenated_inputs(c_ids, c_mask, r_ids, r_mask, prompt, pad_token_id=0)
    ids = ids % vocab
    hidden = torch.randn(6, 40, hdim, generator=g).to(torch.bfloat16)
    weight = (torch.randn(vocab, hdim, generator=g) * 0.25).to(torch.bfloat16)
    ref_c, ref_r, beta = -torch.rand(3, generator=g) * 60, -torch.rand(3, generator=g) * 60, 0.1

    def grads_close(got, want):
        err = (got.cpu().double() - want).abs()
        assert err.max().item() <= 6 * 2.0 ** -8 * want.abs().max().item() + 1e-9, (err.max().item(), want.abs().max().item())

    # DPO
    h64, w64 = hidden.double().requires_grad_(True), weight.double().requires_grad_(True)
    lp = otn.log_probs_from_logits(straight_through_logits(hidden, weight, h64, w64, cuda), torch.roll(ids, -1, 1), 1.0)[:, :-1]
    sums, means = ol.get_batch_logps(lp, att, lens)
    ref_pref, _, _ = ol.dpo_loss(sums[:3], sums[3:], ref_c.double(), ref_r.double(), beta)
    ref_loss = ref_pref + (-means[:3].mean()) * 0.3
    ref_loss.backward()
    hd, wd = hidden.to(cuda).requires_grad_(True), weight.to(cuda).requires_grad_(True)
    out = dpo_loss_step(hd, ids.to(cuda), att.to(cuda), lens, 3, ref_c.to(cuda), ref_r.to(cuda), DPOLoss(beta),
                        nll_loss_coef=0.3, lm_head_weight=wd)
    _close(out["chosen_logps"], sums[:3].detach(), 2e-3 * 40)
    _close(out["rejected_logps"], sums[3:].detach(), 2e-3 * 40)
    _close(out["loss"], ref_loss.detach(), 2e-2)
    out["loss"].backward()
    grads_close(hd.grad, h64.grad)
    grads_close(wd.grad, w64.grad)

    # SFT
    loss_mask = att.clone()
    loss_mask[:, :5] = 0
    loss_mask[4] = 0
    shifted = loss_mask[:, :-1]
    h64, w64 = hidden.double().requires_grad_(True), weight.double().requires_grad_(True)
    lp_ref = otn.log_probs_from_logits(straight_through_logits(hidden, weight, h64, w64, cuda), torch.roll(ids, -1, 1), 1.0)[:, :-1]
    ref_loss = ol.aggregate_loss(-lp_ref, shifted.double(), token_level_loss=True)
    ref_loss.backward()
    hd, wd = hidden.to(cuda).requires_grad_(True), weight.to(cuda).requires_grad_(True)
    loss, lp_d = sft_loss_step(hd, ids.to(cuda), att.to(cuda), loss_mask.to(cuda), SFTLoss(True), lm_head_weight=wd)
    _close(loss, ref_loss.detach(), 2e-3 * max(1.0, abs(ref_loss.item())))
    _close(lp_d, (lp_ref * shifted).detach(), 2e-3)
    loss.backward()
    grads_close(hd.grad, h64.grad)
    grads_close(wd.grad, w64.grad)

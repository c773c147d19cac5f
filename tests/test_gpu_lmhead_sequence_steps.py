"""The SFT and DPO steps on the lm-head path (hidden states and lm_head.weight in place of logits:
openrlhf/trainer/sft_trainer.py:151-167, openrlhf/trainer/dpo_trainer.py:157-180,341-382) at the
depth the kernels run at in training: 6 sequences of up to 1536 tokens, hidden size 4096,
vocabulary 151 936, bf16 (9216 rows through the projection, every CU busy).

Reference, in the two steps of tests/lmhead_util.py: the path's own rounded logits of every
position (the C entry stores them; a row sample is checked against the fp64 product), the
log-probs of those logits by closed form in fp32 on the GPU (a row sample against the CPU oracle in
fp64), the sequence-level losses on top by the oracle's own functions in fp64, whose gradient
with respect to the log-probs goes back through the closed forms of the vocabulary part. Values
within 2e-3 per log-prob (sums of n log-probs: n times that), every gradient entry within its
rounding bound (tests/lmhead_util.gradient_bounds)."""
import pytest
import torch

from oracle import losses as ol

pytestmark = pytest.mark.gpu

B, T, H, V = 6, 1536, 4096, 151936


@pytest.fixture(scope="module")
def batch(cuda):
    from tests.lmhead_util import check_rounded_logits, closed_form_from_logits, forward_keeping_logits, oracle_from_logits

    g = torch.Generator().manual_seed(77)
    lens = torch.tensor([T, 900, 1300, 1100, T - 1, 700])
    att = (torch.arange(T)[None, :] < lens[:, None]).long()
    ids = torch.randint(1, V, (B, T), generator=g) * att
    prompt_lens = [300, 120, 512, 300, 120, 512]            # chosen and rejected share their prompts
    gd = torch.Generator(device=cuda).manual_seed(78)
    hidden = torch.randn(B, T, H, device=cuda, generator=gd).to(torch.bfloat16)
    weight = (torch.randn(V, H, device=cuda, generator=gd) * (3.0 / H ** 0.5)).to(torch.bfloat16)
    rows = hidden.reshape(-1, H)
    labels = torch.roll(ids, -1, 1).reshape(-1).to(cuda)
    _, _, _, kept, _ = forward_keeping_logits(rows, weight, labels, 1.0)
    sample = torch.randperm(B * T, generator=g)[:10]
    sd = sample.to(cuda)
    check_rounded_logits(kept[sd].cpu(), rows[sd].cpu(), weight.cpu())
    zeros = torch.zeros(B * T, device=cuda)
    lp, _, _, _, _, _ = closed_form_from_logits(kept[:, :V], rows, weight, labels, 1.0, zeros, zeros)
    lp64, _, _, _, _, _ = oracle_from_logits(kept[sd][:, :V], rows[sd], weight, labels[sd], 1.0, zeros[sd].cpu(), zeros[sd].cpu())
    assert (lp[sd].cpu().double() - lp64).abs().max().item() <= 2e-5       # the closed form is the oracle's
    return dict(att=att, ids=ids, prompt_lens=prompt_lens, hidden=hidden, weight=weight, rows=rows, labels=labels, kept=kept,
                lp=lp.cpu().double().view(B, T)[:, :-1], gen=g)


def _check_grads(c, cuda, g_lp, grad_hidden, grad_weight, what):
    """g_lp [B, T-1]: the reference loss's gradient with respect to the log-probs."""
    from tests.lmhead_util import assert_gradient, closed_form_from_logits

    full = torch.zeros(B, T)
    full[:, :-1] = g_lp.float()
    rows_g = full.reshape(-1).to(cuda)
    _, _, gh, gw, bound_h, bound_w = closed_form_from_logits(c["kept"][:, :V], c["rows"], c["weight"], c["labels"], 1.0, rows_g,
                                                             torch.zeros_like(rows_g))
    assert_gradient(grad_hidden.reshape(-1, H), gh, bound_h, what + ": dHidden")
    assert_gradient(grad_weight, gw, bound_w, what + ": dWeight")
    assert grad_hidden.reshape(-1, H)[rows_g == 0].abs().max().item() == 0.0      # positions outside the loss: left out


def test_dpo_step_from_hidden_at_training_depth(cuda, batch):
    from openrlhf_amd.models.loss import DPOLoss
    from openrlhf_amd.trainer.dpo_trainer import dpo_loss_step

    c = batch
    beta, coef = 0.1, 0.3
    lp = c["lp"].clone().requires_grad_(True)
    sums, means = ol.get_batch_logps(lp, c["att"], c["prompt_lens"])
    ref_c = (sums[:3].detach() + torch.randn(3, generator=c["gen"]) * 5).float()
    ref_r = (sums[3:].detach() + torch.randn(3, generator=c["gen"]) * 5).float()
    pref, chosen_reward, _ = ol.dpo_loss(sums[:3], sums[3:], ref_c.double(), ref_r.double(), beta)
    ref_loss = pref + (-means[:3].mean()) * coef
    ref_loss.backward()

    hd = c["hidden"].clone().requires_grad_(True)
    wd = c["weight"].clone().requires_grad_(True)
    out = dpo_loss_step(hd, c["ids"].to(cuda), c["att"].to(cuda), c["prompt_lens"], 3, ref_c.to(cuda), ref_r.to(cuda), DPOLoss(beta),
                        nll_loss_coef=coef, lm_head_weight=wd)
    n_max = float(c["att"].sum(-1).max())
    assert (out["chosen_logps"].cpu().double() - sums[:3].detach()).abs().max().item() <= 2e-3 * n_max
    assert (out["rejected_logps"].cpu().double() - sums[3:].detach()).abs().max().item() <= 2e-3 * n_max
    assert abs(out["loss"].item() - ref_loss.item()) <= 2e-3 * n_max * beta + 2e-3 * coef + 1e-4
    assert (out["chosen_reward"].cpu().double() - chosen_reward).abs().max().item() <= 2e-3 * n_max * beta
    out["loss"].backward()
    _check_grads(c, cuda, lp.grad, hd.grad, wd.grad, "dpo")


def test_sft_step_from_hidden_at_training_depth(cuda, batch):
    from openrlhf_amd.models.loss import SFTLoss
    from openrlhf_amd.trainer.sft_trainer import sft_loss_step

    c = batch
    loss_mask = c["att"].clone()
    for b_, p in enumerate(c["prompt_lens"]):
        loss_mask[b_, :p] = 0
    loss_mask[4] = 0                                           # a sample without a response
    shifted = loss_mask[:, :-1]
    lp = c["lp"].clone().requires_grad_(True)
    ref_loss = ol.aggregate_loss(-lp, shifted.double(), token_level_loss=True)
    ref_loss.backward()

    hd = c["hidden"].clone().requires_grad_(True)
    wd = c["weight"].clone().requires_grad_(True)
    loss, lp_d = sft_loss_step(hd, c["ids"].to(cuda), c["att"].to(cuda), loss_mask.to(cuda), SFTLoss(True), lm_head_weight=wd)
    assert abs(loss.item() - ref_loss.item()) <= 2e-3 * max(1.0, abs(ref_loss.item()))
    assert (lp_d.detach().cpu().double() - (c["lp"] * shifted)).abs().max().item() <= 2e-3
    loss.backward()
    _check_grads(c, cuda, lp.grad, hd.grad, wd.grad, "sft")

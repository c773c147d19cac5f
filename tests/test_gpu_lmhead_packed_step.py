"""The lm-head path at the depth and shape it runs at in training, through the wrappers a trainer
calls: 16 sequences of 512..3072 tokens packed into one row (about 30 000 tokens), hidden size
4096, vocabulary 151 936, bf16, an action mask over each sequence's response, through
``actor_forward_tail_from_hidden`` (openrlhf/models/actor.py:263-296) and
``actor_loss_step(lm_head_weight=...)`` (openrlhf/trainer/ray/ppo_actor.py:294-352).

The reference is built in the two steps of tests/lmhead_util.py: the path's own rounded logits of
the rows inside the action mask (the C entry stores them; a row sample is checked against the fp64
product) and, from those logits, the closed forms in fp32 on the GPU for every row plus the CPU
oracle in fp64 on a row sample; the token-level losses on top are the oracle's own functions in
fp64. Tolerances: values 2e-3 abs (bf16 logits), gradients element by element within the
rounding bounds of tests/lmhead_util.gradient_bounds. The route through materialised logits
(torch.matmul, then the logits kernels) is compared as well: its matmul accumulates in another
order, so a logit that sits on a bf16 rounding boundary can come out one ulp away; the comparison
says how many rows that may touch."""
import pytest
import torch

from oracle import losses as ol
from oracle import token_numerics as otn

pytestmark = pytest.mark.gpu

B, T, A, H, V = 16, 3072, 2048, 4096, 151936


@pytest.fixture(scope="module")
def packed_case(cuda):
    from tests.lmhead_util import check_rounded_logits, forward_keeping_logits

    g = torch.Generator().manual_seed(2024)
    lens = torch.randint(512, T + 1, (B,), generator=g)
    lens[0], lens[1] = T, 512
    attn = (torch.arange(T)[None, :] < lens[:, None]).long()
    seqs = torch.randint(1, V, (B, T), generator=g) * attn
    prompt = lens // 3
    pos = torch.arange(T - 1)[None, :]
    # position t scores token t + 1: the response runs from the prompt's end to the sequence's last token
    inside = (pos >= prompt[:, None]) & (pos < (lens - 1)[:, None])
    amask = inside[:, -A:].clone()
    amask[2, 100:140] = False                       # a hole, as a truncated tool output leaves one
    gd = torch.Generator(device=cuda).manual_seed(7)
    hidden = torch.randn(B, T, H, device=cuda, generator=gd).to(torch.bfloat16)
    weight = (torch.randn(V, H, device=cuda, generator=gd) * (3.0 / H ** 0.5)).to(torch.bfloat16)
    keep = attn.reshape(-1).bool()
    packed_hidden = hidden.reshape(-1, H)[keep.to(cuda)].contiguous()      # [Ttot, H]

    need = torch.zeros(B, T, dtype=torch.bool)
    need[:, T - 1 - A: T - 1] = amask
    idx = need.reshape(-1).nonzero().squeeze(-1)     # row-major: the order of the packed row
    rows = hidden.reshape(-1, H)[idx.to(cuda)].contiguous()
    labels = torch.roll(seqs, -1, 1).reshape(-1)[idx].to(cuda)
    lp, ent, _, kept, _ = forward_keeping_logits(rows, weight, labels, 1.0)
    sample = torch.randperm(idx.numel(), generator=g)[:12]
    check_rounded_logits(kept[sample.to(cuda)].cpu(), rows[sample.to(cuda)].cpu(), weight.cpu())
    return dict(lens=lens, attn=attn, seqs=seqs, amask=amask, hidden=hidden, weight=weight, keep=keep,
                packed_hidden=packed_hidden, need=need, idx=idx, rows=rows, labels=labels, kept=kept, sample=sample,
                n_tokens=int(keep.sum()), gen=g)


def _scatter_a(flat, case):
    """Values of the needed rows (packed order) into [B, A] (the action window), zeros elsewhere."""
    full = torch.zeros(B * T, dtype=flat.dtype)
    full[case["idx"]] = flat.cpu()
    return full.view(B, T)[:, T - 1 - A: T - 1]


def _gather_a(window, case):
    """[B, A] -> the needed rows in packed order."""
    full = torch.zeros(B, T, dtype=window.dtype)
    full[:, T - 1 - A: T - 1] = window
    return full.reshape(-1)[case["idx"]]


def _check_gradients(case, cuda, g_lp_rows, g_ent_rows, grad_hidden_packed, grad_weight, what):
    """Both gradients against the closed forms on the path's own logits (every element within its
    rounding bound), a row sample of dHidden against the CPU oracle in fp64, and exact zeros in the
    rows outside the action mask."""
    from tests.lmhead_util import assert_gradient, closed_form_from_logits, oracle_from_logits

    kept, rows, weight, labels = case["kept"], case["rows"], case["weight"], case["labels"]
    _, _, gh, gw, bound_h, bound_w = closed_form_from_logits(kept[:, :V], rows, weight, labels, 1.0,
                                                             g_lp_rows.to(cuda), g_ent_rows.to(cuda))
    # packed row p of the hidden states <- needed row k
    packed_of = torch.cumsum(case["keep"].long(), 0) - 1
    at = packed_of[case["idx"]].to(cuda)
    assert_gradient(grad_hidden_packed[at], gh, bound_h, what + ": dHidden")
    assert_gradient(grad_weight, gw, bound_w, what + ": dWeight")
    untouched = torch.ones(grad_hidden_packed.shape[0], dtype=torch.bool, device=cuda)
    untouched[at] = False
    assert grad_hidden_packed[untouched].abs().max().item() == 0.0
    s = case["sample"]
    sd = s.to(cuda)
    _, _, gh64, _, bh64, _ = oracle_from_logits(kept[sd][:, :V], rows[sd], weight, labels[sd], 1.0, g_lp_rows[s], g_ent_rows[s])
    err = (grad_hidden_packed[at[sd]].cpu().double() - gh64).abs()
    assert (err / bh64).max().item() <= 1.0, (what, (err / bh64).max().item())
    return gh, gw, bound_h, bound_w, at


def test_tail_from_hidden_at_training_depth(cuda, packed_case):
    from openrlhf_amd.models.actor import actor_forward_tail, actor_forward_tail_from_hidden, unpad_indices
    from tests.lmhead_util import closed_form_from_logits, oracle_from_logits

    c = packed_case
    assert 20000 <= c["n_tokens"] <= 40000 and 4000 <= c["idx"].numel()
    zeros = torch.zeros(c["idx"].numel(), device=cuda)
    ref_lp, ref_ent, _, _, _, _ = closed_form_from_logits(c["kept"][:, :V], c["rows"], c["weight"], c["labels"], 1.0, zeros, zeros)
    s = c["sample"]
    sd = s.to(cuda)
    lp64, ent64, _, _, _, _ = oracle_from_logits(c["kept"][sd][:, :V], c["rows"][sd], c["weight"], c["labels"][sd], 1.0,
                                                 zeros[sd].cpu(), zeros[sd].cpu())
    assert (ref_lp[sd].cpu().double() - lp64).abs().max().item() <= 2e-5     # the closed forms are the oracle's
    assert (ref_ent[sd].cpu().double() - ent64).abs().max().item() <= 2e-5

    d = cuda
    attn_d, seqs_d, amask_d = c["attn"].to(d), c["seqs"].to(d), c["amask"].to(d)
    hd = c["packed_hidden"].clone().unsqueeze(0).requires_grad_(True)
    wd = c["weight"].clone().requires_grad_(True)
    indices = unpad_indices(attn_d)
    lp, ent = actor_forward_tail_from_hidden(hd, wd, seqs_d, amask_d, attn_d, temperature=1.0, packed_indices=indices,
                                             return_entropy=True)
    assert lp.shape == (B, A) and ent.shape == (B, T - 1)
    want_lp, want_ent = _scatter_a(ref_lp, c), _scatter_a(ref_ent, c)
    assert (lp.detach().cpu() - want_lp).abs().max().item() <= 2e-3
    ent_window = ent[:, -A:].detach().cpu()
    assert (ent_window - want_ent).abs().max().item() <= 2e-3
    assert lp.detach().cpu()[~c["amask"]].abs().max().item() == 0.0 and ent_window[~c["amask"]].abs().max().item() == 0.0
    assert ent[:, : T - 1 - A].abs().max().item() == 0.0
    assert (_gather_a(lp.detach().cpu(), c)[s].double() - lp64).abs().max().item() <= 2e-3
    assert (_gather_a(ent_window.detach(), c)[s].double() - ent64).abs().max().item() <= 2e-3

    w_lp = torch.randn(B, A, generator=c["gen"])
    w_ent = torch.randn(B, A, generator=c["gen"]) * c["amask"]
    ((lp * w_lp.to(d)).sum() + (ent[:, -A:] * w_ent.to(d)).sum()).backward()
    g_lp_rows, g_ent_rows = _gather_a(w_lp, c), _gather_a(w_ent, c)
    gh, gw, bound_h, bound_w, at = _check_gradients(c, cuda, g_lp_rows, g_ent_rows, hd.grad[0], wd.grad, "tail")

    # the route a trainer without this path takes: materialise the logits, then the logits kernels
    h2 = c["packed_hidden"].clone().requires_grad_(True)
    w2 = c["weight"].clone().requires_grad_(True)
    logits = torch.matmul(h2, w2.T)
    lp2, ent2 = actor_forward_tail(logits.unsqueeze(0), seqs_d, amask_d, attn_d, temperature=1.0, packed_indices=indices,
                                   return_entropy=True)
    diff = (lp2 - lp).detach().abs().cpu()
    x_label = c["kept"].gather(1, c["labels"][:, None]).squeeze(1).float().abs()
    one_ulp = _scatter_a(x_label * 2.0 ** -7, c)
    assert (diff <= one_ulp + 2e-3).all()                     # at most the label's logit one bf16 step away
    assert (diff > 2e-3).float().mean().item() <= 0.01         # and that in few places
    ent_diff = (ent2 - ent).detach().abs()
    assert ent_diff.max().item() <= 2e-2 and ent_diff.mean().item() <= 2e-4
    ((lp2 * w_lp.to(d)).sum() + (ent2[:, -A:] * w_ent.to(d)).sum()).backward()
    del logits
    for got, ref, bound, name in ((h2.grad[at], gh, bound_h, "dHidden"), (w2.grad, gw, bound_w, "dWeight")):
        err = (got.float() - ref).abs()
        rel = (err.double().pow(2).sum() / ref.double().pow(2).sum()).sqrt().item()
        assert rel <= 4 * 2.0 ** -8, (name, rel)
        rows_off = ((err > 2 * bound).any(1)).float().mean().item()
        assert rows_off <= 0.02, (name, rows_off)


def test_actor_step_from_hidden_at_training_depth(cuda, packed_case):
    """The PPO step (dual-clip surrogate, k3 KL, entropy bonus, token mean over the batch's tokens)
    from hidden states at the same depth: the loss terms against the oracle's loss functions applied
    in fp64 to the reference log-probs and entropies, the gradients through the oracle's own
    d loss / d(log-prob, entropy) and the closed forms of the vocabulary part."""
    from openrlhf_amd.models.actor import unpad_indices
    from openrlhf_amd.models.loss import PolicyLoss
    from openrlhf_amd.trainer.ray.ppo_actor import actor_loss_step
    from tests.lmhead_util import closed_form_from_logits

    c = packed_case
    g = c["gen"]
    zeros = torch.zeros(c["idx"].numel(), device=cuda)
    ref_lp, ref_ent, _, _, _, _ = closed_form_from_logits(c["kept"][:, :V], c["rows"], c["weight"], c["labels"], 1.0, zeros, zeros)
    m = c["amask"].double()
    alp = (_scatter_a(ref_lp, c).double() * m).requires_grad_(True)
    ent_a = _scatter_a(ref_ent, c).double().requires_grad_(True)
    old = (alp.detach() + torch.randn(B, A, generator=g) * 0.15) * m
    base = (alp.detach() + torch.randn(B, A, generator=g) * 0.1) * m
    adv = torch.randn(B, A, generator=g).double()
    pol = dict(dual_clip=3.0, clip_eps_low=0.2, clip_eps_high=0.28)
    kl_coef, ent_coef = 0.05, 0.01

    pl = ol.policy_loss(alp, old, adv, m, None, **pol)
    kl_loss = ol.aggregate_loss(otn.compute_approx_kl(alp, base, "k3"), m)
    ent_loss = ol.aggregate_loss(ent_a, m)
    ref_loss = pl[0] + kl_loss * kl_coef - ent_loss * ent_coef
    ref_loss.backward()

    d = cuda
    hd = c["packed_hidden"].clone().requires_grad_(True)
    wd = c["weight"].clone().requires_grad_(True)
    attn_d = c["attn"].to(d)
    out = actor_loss_step(hd, c["seqs"].to(d), attn_d, c["amask"].to(d), old.float().to(d), adv.float().to(d),
                          PolicyLoss(**pol), base_action_log_probs=base.float().to(d), kl_estimator="k3", kl_coef=kl_coef,
                          entropy_coef=ent_coef, temperature=1.0, packed_indices=unpad_indices(attn_d), lm_head_weight=wd)
    out["loss"].backward()
    for key, want in (("loss", ref_loss), ("actor_loss", pl[0]), ("clip_ratio", pl[1]), ("ppo_kl", pl[2]),
                      ("kl_loss", kl_loss), ("entropy_loss", ent_loss)):
        assert abs(out[key].item() - want.item()) <= 2e-3 * max(1.0, abs(want.item())), (key, out[key].item(), want.item())
    assert (out["action_log_probs"].cpu().double() - alp.detach()).abs().max().item() <= 2e-3
    g_lp_rows, g_ent_rows = _gather_a(alp.grad, c).float(), _gather_a(ent_a.grad, c).float()
    _check_gradients(c, cuda, g_lp_rows, g_ent_rows, hd.grad, wd.grad, "step")

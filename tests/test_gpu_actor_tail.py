"""The fused Actor.forward tail against the oracle's restatement of openrlhf/models/actor.py:265-296,
padded and packed, forward and backward, with and without skipping masked positions."""
import pytest
import torch

from oracle import token_numerics as otn

pytestmark = pytest.mark.gpu


def _batch(seed, b=5, t=40, vocab=3001, a=17):
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(a + 3, t + 1, (b,), generator=g)
    lens[0] = t
    attn = (torch.arange(t)[None, :] < lens[:, None]).long()
    seqs = torch.randint(1, vocab, (b, t), generator=g) * attn
    # action mask over the last A of the first T-1 positions: prompt zeros left, a hole, padding right
    amask = attn[:, 1:][:, -a:].bool().clone()
    amask[:, :4] = False
    amask[1, 8:10] = False
    logits = torch.randn(b, t, vocab, generator=g) * 2
    return logits, seqs, attn, amask


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("skip", [True, False])
def test_tail_matches_oracle(cuda, dtype, packed, skip):
    from openrlhf_amd.models.actor import actor_forward_tail, unpad_indices

    logits, seqs, attn, amask = _batch(1)
    logits = logits.to(dtype)
    temperature = 0.8
    ref_x = logits.double().requires_grad_(True)
    flat_keep = attn.reshape(-1).bool()
    if packed:
        ref_in = ref_x.reshape(-1, ref_x.shape[-1])[flat_keep].unsqueeze(0)
    else:
        ref_in = ref_x
    # the oracle up-casts with .float(); run it on the fp64 copy for a clean target
    ref_lp, ref_ent = _oracle_tail64(ref_in, seqs, attn, amask, temperature, packed)
    w_lp = torch.randn(ref_lp.shape, generator=torch.Generator().manual_seed(2))
    w_ent = torch.randn(ref_ent.shape, generator=torch.Generator().manual_seed(3))
    width = amask.shape[1]
    ent_mask = torch.zeros_like(ref_ent)
    ent_mask[:, -width:] = amask.double()
    ((ref_lp * w_lp.double()).sum() + (ref_ent * w_ent.double() * ent_mask).sum()).backward()

    xd = logits.to(cuda)
    if packed:
        xd = xd.reshape(-1, xd.shape[-1])[flat_keep.to(cuda)].unsqueeze(0).contiguous()
    xd.requires_grad_(True)
    lp, ent = actor_forward_tail(
        xd, seqs.to(cuda), amask.to(cuda), attn.to(cuda), temperature=temperature,
        packed_indices=unpad_indices(attn.to(cuda)) if packed else None, return_entropy=True, skip_masked=skip)
    atol = 1e-5 if dtype == torch.float32 else 2e-3
    assert lp.shape == ref_lp.shape and ent.shape == ref_ent.shape
    assert (lp.cpu().double() - ref_lp.detach()).abs().max().item() <= atol
    sel = ent_mask.bool() if skip else (attn[:, :-1].bool() if packed else torch.ones_like(ent_mask).bool())
    assert (ent.cpu().double() - ref_ent.detach())[sel].abs().max().item() <= atol
    if skip:
        assert ent.cpu()[~ent_mask.bool()].abs().max().item() == 0.0
    ((lp * w_lp.to(cuda)).sum() + (ent * w_ent.to(cuda) * ent_mask.float().to(cuda)).sum()).backward()
    ref_grad = ref_x.grad
    if packed:
        ref_grad = ref_grad.reshape(-1, ref_grad.shape[-1])[flat_keep].unsqueeze(0)
    err = (xd.grad.cpu().double() - ref_grad).abs()
    if dtype == torch.float32:
        assert err.max().item() <= 1e-5
    else:
        assert (err <= 2.0 ** -8 * ref_grad.abs() + 1e-6).all()


def _oracle_tail64(logits64, seqs, attn, amask, temperature, packed):
    """otn.actor_forward_tail without its .float() up-cast (fp64 target)."""
    batch, seqlen = seqs.shape
    rolled = torch.roll(seqs, shifts=-1, dims=1)
    if packed:
        keep = attn.reshape(-1).bool().nonzero().squeeze(-1)
        labels = rolled.reshape(-1)[keep].unsqueeze(0)
    else:
        labels = rolled
    ent = otn.compute_entropy(logits64)
    lp = otn.log_probs_from_logits(logits64, labels, temperature)
    if packed:
        def repad(flat):
            full = torch.zeros(batch * seqlen, dtype=flat.dtype)
            return full.index_copy(0, keep, flat.reshape(-1)).view(batch, seqlen)
        ent, lp = repad(ent), repad(lp)
    ent, lp = ent[:, :-1], lp[:, :-1]
    return lp[:, -amask.shape[1]:] * amask.double(), ent


def test_oracle_tail_helper_is_the_oracle():
    logits, seqs, attn, amask = _batch(4, b=3, t=12, vocab=50, a=5)
    a1, e1 = otn.actor_forward_tail(logits, seqs, attn, amask, 0.9)
    a2, e2 = _oracle_tail64(logits.double(), seqs, attn, amask, 0.9, False)
    assert (a1.double() - a2).abs().max() <= 1e-5 and (e1.double() - e2).abs().max() <= 1e-5


def test_return_all_logprobs_for_sft(cuda):
    """action_mask=None: every [B, T-1] log-prob (the SFT / DPO callers, sft_trainer.py:161)."""
    from openrlhf_amd.models.actor import actor_forward_tail

    logits, seqs, attn, _ = _batch(5)
    out = actor_forward_tail(logits.to(cuda), seqs.to(cuda), None, attn.to(cuda), temperature=1.0)
    ref = otn.log_probs_from_logits(logits.double(), torch.roll(seqs, -1, 1))[:, :-1]
    keep = attn[:, :-1].bool()
    assert out.shape == ref.shape
    assert (out.cpu().double() - ref)[keep].abs().max().item() <= 1e-5
    assert out.cpu()[~keep].abs().max().item() == 0.0


@pytest.mark.parametrize("packed", [False, True])
def test_tail_from_hidden_states(cuda, packed):
    """The same tail from the decoder's last hidden states and lm_head.weight, logits never stored:
    against the oracle on ``hidden @ W.T`` rounded to bf16 as the lm_head output is
    (tests/lmhead_util.py), in fp64 (2e-3 abs; gradients of the hidden states and of the weight
    within the rounding of a bf16 logits gradient and result)."""
    from openrlhf_amd.models.actor import actor_forward_tail_from_hidden, unpad_indices
    from tests.lmhead_util import straight_through_logits

    b, t, a, hdim, vocab, temperature = 4, 36, 15, 96, 1234, 0.8
    _, seqs, attn, amask = _batch(7, b=b, t=t, vocab=vocab, a=a)
    g = torch.Generator().manual_seed(8)
    hidden = torch.randn(b, t, hdim, generator=g).to(torch.bfloat16)
    weight = (torch.randn(vocab, hdim, generator=g) * 0.3).to(torch.bfloat16)
    flat_keep = attn.reshape(-1).bool()

    h64 = hidden.double().requires_grad_(True)
    w64 = weight.double().requires_grad_(True)
    logits64 = straight_through_logits(hidden, weight, h64, w64, cuda)
    ref_in = logits64.reshape(-1, vocab)[flat_keep].unsqueeze(0) if packed else logits64
    ref_lp, ref_ent = _oracle_tail64(ref_in, seqs, attn, amask, temperature, packed)
    w_lp = torch.randn(ref_lp.shape, generator=g)
    w_ent = torch.randn(ref_ent.shape, generator=g)
    ent_mask = torch.zeros_like(ref_ent)
    ent_mask[:, -a:] = amask.double()
    ((ref_lp * w_lp.double()).sum() + (ref_ent * w_ent.double() * ent_mask).sum()).backward()

    hd = hidden.to(cuda)
    if packed:
        hd = hd.reshape(-1, hdim)[flat_keep.to(cuda)].unsqueeze(0).contiguous()
    hd.requires_grad_(True)
    wd = weight.to(cuda).requires_grad_(True)
    lp, ent = actor_forward_tail_from_hidden(
        hd, wd, seqs.to(cuda), amask.to(cuda), attn.to(cuda), temperature=temperature,
        packed_indices=unpad_indices(attn.to(cuda)) if packed else None, return_entropy=True)
    assert lp.shape == ref_lp.shape and ent.shape == ref_ent.shape
    assert (lp.cpu().double() - ref_lp.detach()).abs().max().item() <= 2e-3
    assert (ent.cpu().double() - ref_ent.detach())[ent_mask.bool()].abs().max().item() <= 2e-3
    assert ent.cpu()[~ent_mask.bool()].abs().max().item() == 0.0
    ((lp * w_lp.to(cuda)).sum() + (ent * w_ent.to(cuda) * ent_mask.float().to(cuda)).sum()).backward()
    ref_gh = h64.grad.reshape(-1, hdim)[flat_keep].unsqueeze(0) if packed else h64.grad
    for got, ref in ((hd.grad, ref_gh), (wd.grad, w64.grad)):
        err = (got.cpu().double() - ref).abs()
        scale = ref.abs().max().item()
        assert err.max().item() <= 4 * 2.0 ** -8 * scale + 1e-9, (err.max().item(), scale)
        assert (err.pow(2).sum() / ref.pow(2).sum()).sqrt().item() <= 2 * 2.0 ** -8
    # positions outside the action mask are left out of the projection: no gradient reaches them
    need = torch.zeros(b, t, dtype=torch.bool)
    need[:, t - 1 - a : t - 1] = amask
    dead = ~need.reshape(-1)[flat_keep] if packed else ~need.reshape(-1)
    assert hd.grad.reshape(-1, hdim)[dead.to(cuda)].abs().max().item() == 0.0


def test_tail_from_hidden_states_every_position(cuda):
    """``action_mask=None`` on a padded batch: the reference returns real log-probs and entropies at
    padded positions too (actor.py:283-290 multiply by no mask); ``skip_masked=False`` projects
    every row and reproduces them, the default leaves the positions outside the attention mask at 0."""
    from openrlhf_amd.models.actor import actor_forward_tail_from_hidden
    from tests.lmhead_util import straight_through_logits

    b, t, hdim, vocab, temperature = 3, 20, 64, 777, 0.9
    _, seqs, attn, _ = _batch(21, b=b, t=t, vocab=vocab, a=7)
    g = torch.Generator().manual_seed(22)
    hidden = torch.randn(b, t, hdim, generator=g).to(torch.bfloat16)
    weight = (torch.randn(vocab, hdim, generator=g) * 0.3).to(torch.bfloat16)
    logits64 = straight_through_logits(hidden, weight, hidden.double(), weight.double(), cuda)
    ref_lp = otn.log_probs_from_logits(logits64, torch.roll(seqs, -1, 1), temperature)[:, :-1]
    ref_ent = otn.compute_entropy(logits64)[:, :-1]
    args = (hidden.to(cuda), weight.to(cuda), seqs.to(cuda), None, attn.to(cuda))
    lp, ent = actor_forward_tail_from_hidden(*args, temperature=temperature, return_entropy=True, skip_masked=False)
    assert lp.shape == ref_lp.shape and ent.shape == ref_ent.shape
    assert (lp.cpu().double() - ref_lp).abs().max().item() <= 2e-3
    assert (ent.cpu().double() - ref_ent).abs().max().item() <= 2e-3
    keep = attn[:, :-1].bool()
    assert bool((~keep).any())
    lp_s, ent_s = actor_forward_tail_from_hidden(*args, temperature=temperature, return_entropy=True)
    assert (lp_s.cpu().double() - ref_lp)[keep].abs().max().item() <= 2e-3
    assert lp_s.cpu()[~keep].abs().max().item() == 0.0 and ent_s.cpu()[~keep].abs().max().item() == 0.0

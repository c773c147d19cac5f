"""The same numbers whatever form the caller's tensors take: non-contiguous views, broadcast
masks, other integer / float dtypes, higher-rank logits, sliced vocabularies, normalisers given
as Python numbers, CPU scalars or device scalars."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_per_token_inputs_in_other_forms(cuda):
    from openrlhf_amd.models.loss import PolicyLoss, ValueLoss, aggregate_loss
    from openrlhf_amd.models.utils import compute_approx_kl, masked_mean

    g = torch.Generator().manual_seed(2)
    b, a = 12, 333
    lp = (-torch.rand(b, a, generator=g) * 2).to(cuda)
    old = lp + (torch.randn(b, a, generator=g) * 0.1).to(cuda)
    adv = torch.randn(b, a, generator=g).to(cuda)
    mask = (torch.rand(b, a, generator=g) > 0.3).to(cuda)
    pol = PolicyLoss(0.2, 0.2, dual_clip=3.0)
    base = pol(lp, old, adv, action_mask=mask)

    def same(out):
        for p, q in zip(out, base):
            assert (p is None and q is None) or torch.equal(p, q)

    # transposed storage, strided slices, a batch dimension in front
    same(pol(lp.t().contiguous().t(), old.t().contiguous().t(), adv, action_mask=mask.t().contiguous().t()))
    wide = torch.zeros(b, 2 * a, device=cuda)
    wide[:, ::2] = lp
    same(pol(wide[:, ::2], old, adv, action_mask=mask))
    same(pol(lp.view(3, 4, a), old.view(3, 4, a), adv.view(3, 4, a), action_mask=mask.view(3, 4, a)))
    # mask dtypes: int32, int64, uint8, fp16, fp64 all mean the same 0 / 1 weights
    for dt in (torch.int32, torch.int64, torch.uint8, torch.float16, torch.float64):
        same(pol(lp, old, adv, action_mask=mask.to(dt)))
    # half-precision per-token inputs are up-cast: equal to the call on the up-cast tensors
    h = lp.to(torch.bfloat16)
    assert torch.equal(pol(h, old, adv, action_mask=mask)[0], pol(h.float(), old, adv, action_mask=mask)[0])
    # an advantage per sequence broadcast over the tokens, a mask row broadcast over the batch
    per_seq = adv[:, :1]
    assert torch.equal(pol(lp, old, per_seq, action_mask=mask)[0], pol(lp, old, per_seq.expand(b, a).contiguous(), action_mask=mask)[0])
    row_mask = mask[:1]
    assert torch.equal(masked_mean(adv, row_mask), masked_mean(adv, row_mask.expand(b, a).contiguous()))
    # normalisers: Python numbers, 0-dim CPU tensors and 0-dim device tensors are interchangeable
    ref = aggregate_loss(adv, mask, dp_size=2, batch_num_tokens=1234.0)
    for n in (1234, torch.tensor(1234.0), torch.tensor(1234.0, device=cuda), torch.tensor(1234, device=cuda)):
        assert torch.equal(aggregate_loss(adv, mask, dp_size=2, batch_num_tokens=n), ref)
    vref = ValueLoss(0.2, token_level_loss=False)(adv, old, lp, action_mask=mask, dp_size=2, global_batch_size=7.0)
    assert torch.equal(ValueLoss(0.2, token_level_loss=False)(adv, old, lp, action_mask=mask, dp_size=2,
                                                              global_batch_size=torch.tensor(7.0, device=cuda)), vref)
    # KL on mixed dtypes is the KL of the up-cast pair
    assert torch.equal(compute_approx_kl(h, old, "k3"), compute_approx_kl(h.float(), old, "k3"))


def test_logits_in_other_forms(cuda):
    from openrlhf_amd.models.utils import compute_entropy, log_probs_from_logits, logprobs_and_entropy_from_logits

    g = torch.Generator().manual_seed(3)
    b, t, v = 3, 17, 5003
    x = (torch.randn(b, t, v, generator=g) * 2).to(torch.bfloat16).to(cuda)
    labels = torch.randint(0, v, (b, t), generator=g).to(cuda)
    lp, ent = logprobs_and_entropy_from_logits(x, labels, 0.8)
    assert lp.shape == (b, t) and ent.shape == (b, t)
    flat_lp, flat_ent = logprobs_and_entropy_from_logits(x.view(-1, v), labels.view(-1), 0.8)
    assert torch.equal(lp.view(-1), flat_lp) and torch.equal(ent.view(-1), flat_ent)
    assert torch.equal(log_probs_from_logits(x, labels.int(), 0.8), lp)          # int32 labels
    assert torch.equal(compute_entropy(x), ent)
    assert torch.equal(log_probs_from_logits(x.unsqueeze(0), labels.unsqueeze(0), 0.8)[0], lp)  # rank 4
    # a vocabulary padded for the GEMM and sliced off: 2-D rows are read in place through their stride,
    # higher ranks through one contiguous copy; both equal the call on a compact tensor
    padded = torch.zeros(b, t, v + 61, dtype=torch.bfloat16, device=cuda)
    padded[..., :v] = x
    padded[..., v:] = 50.0  # would dominate the softmax if it were read
    assert torch.equal(log_probs_from_logits(padded[..., :v], labels, 0.8), lp)
    # (rows at another 16-byte phase are summed in another order: equal to rounding, not bit for bit)
    strided = log_probs_from_logits(padded.view(-1, v + 61)[:, :v], labels.view(-1), 0.8)
    assert (strided - lp.view(-1)).abs().max().item() <= 1e-5
    # the gradient of a strided 2-D view lands in the view, the padding columns stay untouched
    rows = padded.view(-1, v + 61).clone().requires_grad_(True)
    out = log_probs_from_logits(rows[:, :v], labels.view(-1), 0.8).sum()
    (gr,) = torch.autograd.grad(out, rows)
    assert (gr[:, v:] == 0).all() and gr[:, :v].abs().sum() > 0
    xr = x.view(-1, v).clone().requires_grad_(True)
    (gx,) = torch.autograd.grad(log_probs_from_logits(xr, labels.view(-1), 0.8).sum(), xr)
    assert (gr[:, :v].float() - gx.float()).abs().max().item() <= 2.0 ** -8 * gx.float().abs().max().item()
    # a transposed tensor goes through one contiguous copy and gives the same values
    xt = x.view(-1, v).t().contiguous().t()
    assert not xt.is_contiguous()
    assert torch.equal(log_probs_from_logits(xt, labels.view(-1), 0.8), lp.view(-1))


def _at_offset(t, off):
    """The same values in storage that starts `off` elements past an allocation boundary."""
    buf = torch.empty(t.numel() + off, dtype=t.dtype, device=t.device)
    view = buf[off:off + t.numel()].view(t.shape)
    view.copy_(t)
    return view


@pytest.mark.parametrize("off", [1, 2, 3])
def test_per_token_arrays_off_the_16_byte_boundary(cuda, off):
    """The four-token vector loads promise the element's alignment only: arrays that start off a
    16-byte boundary give the same losses and gradients."""
    from openrlhf_amd.models.loss import PolicyLoss, ValueLoss, aggregate_loss
    from openrlhf_amd.trainer.ppo_utils.experience import PackedSteps

    g = torch.Generator().manual_seed(20 + off)
    b, a = 6, 5003
    lp = (-torch.rand(b, a, generator=g) * 2).to(cuda)
    old = lp + (torch.randn(b, a, generator=g) * 0.1).to(cuda)
    adv = torch.randn(b, a, generator=g).to(cuda)
    lens = torch.tensor([5003, 4097, 1023, 1, 2050, 3333])
    mask = (torch.arange(a)[None, :] < lens[:, None]).to(cuda)
    pol, val = PolicyLoss(0.2, 0.28, dual_clip=3.0), ValueLoss(0.2)

    def run(lp_, old_, adv_, mask_, **kw):
        x = lp_.detach().requires_grad_()
        loss = pol(x, old_, adv_, action_mask=mask_, **kw)
        v = val(x, old_, adv_, action_mask=mask_, **kw)
        agg = aggregate_loss(x * adv_, mask_, **{k: w for k, w in kw.items()})
        (loss[0] + v + agg).backward()
        return torch.stack([loss[0], loss[1], loss[2], v, agg]).detach(), x.grad

    for m in (mask, mask.float(), mask.long()):
        ref, gref = run(lp, old, adv, m)
        out, gout = run(_at_offset(lp, off), _at_offset(old, off), _at_offset(adv, off), _at_offset(m, off))
        assert torch.allclose(out, ref, rtol=1e-6, atol=1e-7)
        assert torch.allclose(gout, gref, rtol=1e-5, atol=1e-9)
    # packed rows: starts fall on every residue; shifting the storage shifts them all
    ps = PackedSteps.from_padded(dict(lp=lp, old=old, adv=adv, mask=mask), mask)
    kw = dict(cu_seqlens=ps.cu_seqlens, max_seqlen=a)
    ref, gref = run(lp, old, adv, mask)
    for o in (0, off):
        out, gout = run(_at_offset(ps["lp"], o), _at_offset(ps["old"], o), _at_offset(ps["adv"], o),
                        _at_offset(ps["mask"], o), **kw)
        assert torch.allclose(out, ref, rtol=1e-6, atol=1e-7)
        packed_ref = PackedSteps.from_padded(dict(g=gref), mask)["g"]
        assert torch.allclose(gout, packed_ref, rtol=1e-5, atol=1e-9)


@pytest.mark.parametrize("off", [1, 3])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_flat_kernels_off_the_16_byte_boundary(cuda, off, dtype):
    """The flat kernels (approximate KL forward / backward, global whitening) on storage that
    does not start on a 16-byte boundary and with a length that is not a multiple of four: the
    same bits as on aligned storage."""
    from openrlhf_amd.models.utils import compute_approx_kl
    from openrlhf_amd.trainer.ppo_utils.experience_maker import whiten_advantages

    g = torch.Generator().manual_seed(40 + off)
    n = 7 * 1031 + 2
    lp = (-torch.rand(n, generator=g) * 2).to(dtype).to(cuda)
    base = (lp.float() + torch.randn(n, generator=g).to(cuda) * 0.3).to(dtype)
    up = torch.randn(n, generator=g).to(cuda)
    for est in ("k1", "k2", "k3"):
        x = lp.clone().requires_grad_()
        ref = compute_approx_kl(x, base, est)
        ref.backward(up)
        y = _at_offset(lp, off).requires_grad_()
        out = compute_approx_kl(y, _at_offset(base, off), est)
        out.backward(_at_offset(up, off))
        assert torch.equal(out, ref) and torch.equal(y.grad, x.grad)
    adv = lp.float()[:7 * 1031].view(7, 1031).contiguous()
    mask = (torch.rand(7, 1031, generator=g) > 0.4).to(cuda)
    ref = whiten_advantages([adv], [mask])[0]
    out = whiten_advantages([_at_offset(adv, off)], [_at_offset(mask, off)])[0]
    assert torch.allclose(out, ref, rtol=1e-6, atol=1e-7)

"""Shapes at the ends of the launch-geometry ranges: millions of tiny rows, one enormous row,
empty inputs. Results against torch on the GPU in fp64 (the shapes are too big for the CPU
oracle to be worth its time; the arithmetic is pinned by the other tests)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_millions_of_tiny_vocabulary_rows(cuda):
    from openrlhf_amd.models.utils import fused_logprob_entropy_fwd_bwd, logprobs_and_entropy_from_logits

    n, v = 3_000_001, 8
    g = torch.Generator(device=cuda).manual_seed(1)
    x = torch.randn(n, v, device=cuda, generator=g)
    labels = torch.randint(0, v, (n,), device=cuda, generator=g)
    ref = torch.log_softmax(x.double(), -1)
    ref_lp = ref.gather(1, labels[:, None]).squeeze(1)
    ref_ent = -(ref.exp() * ref).sum(-1)
    xr = x.clone().requires_grad_(True)
    lp, ent = logprobs_and_entropy_from_logits(xr, labels)
    assert (lp.double() - ref_lp).abs().max().item() <= 1e-5 and (ent.double() - ref_ent).abs().max().item() <= 1e-5
    (gx,) = torch.autograd.grad(lp.sum(), xr)
    want = torch.zeros_like(ref).scatter_(1, labels[:, None], 1.0) - ref.exp()
    assert (gx.double() - want).abs().max().item() <= 1e-5
    lp1, _, g1 = fused_logprob_entropy_fwd_bwd(x.clone(), labels, torch.ones(n, device=cuda), None)
    assert (lp1 - lp).abs().max().item() <= 2e-6 and (g1 - gx).abs().max().item() <= 2e-6


def test_many_short_rows_and_one_enormous_row_per_token(cuda):
    from openrlhf_amd.models.loss import PolicyLoss, aggregate_loss
    from openrlhf_amd.trainer.ppo_utils.experience_maker import get_cumulative_returns

    for b, a in ((1_000_003, 5), (1, 40_000_001)):
        g = torch.Generator(device=cuda).manual_seed(b)
        x = torch.randn(b, a, device=cuda, generator=g)
        mask = torch.rand(b, a, device=cuda, generator=g) > 0.3
        got = aggregate_loss(x, mask, token_level_loss=False)
        cnt = mask.sum(-1).double()
        seq = (x.double() * mask).sum(-1) / (cnt + 1e-8)
        want = (seq * (cnt > 0)).sum() / (cnt > 0).sum()
        assert abs(got.item() - want.item()) <= 1e-5 * max(1.0, abs(want.item()))
        ret = get_cumulative_returns(x, mask, 1.0)
        ref = ((x.double() * mask).flip(1).cumsum(1).flip(1))
        assert (ret.double() - ref).abs().max().item() <= 1e-5 * max(1.0, ref.abs().max().item())
        lp = x.clone().requires_grad_(True)
        loss = PolicyLoss()(lp, x + 0.01, x, action_mask=mask)[0]
        (gl,) = torch.autograd.grad(loss, lp)
        assert torch.isfinite(loss) and torch.isfinite(gl).all() and (gl[~mask] == 0).all()


def test_empty_inputs(cuda):
    from openrlhf_amd.models.loss import PolicyLoss, ValueLoss, aggregate_loss
    from openrlhf_amd.models.utils import compute_approx_kl, logprobs_and_entropy_from_logits, masked_mean
    from openrlhf_amd.trainer.ppo_utils.experience import cu_seqlens_of, pad_packed, row_extents
    from openrlhf_amd.trainer.ppo_utils.experience_maker import get_advantages_and_returns

    e2 = torch.empty(0, 16, device=cuda)
    lp, ent = logprobs_and_entropy_from_logits(torch.empty(0, 100, device=cuda), torch.empty(0, dtype=torch.long, device=cuda))
    assert lp.shape == (0,) and ent.shape == (0,)
    assert compute_approx_kl(e2, e2, "k3").shape == (0, 16)
    assert torch.isnan(masked_mean(e2, e2.bool()))          # 0 / 0, as the reference
    assert torch.isnan(aggregate_loss(e2, e2.bool()))
    assert torch.isnan(PolicyLoss()(e2, e2, e2, action_mask=e2.bool())[0])
    assert torch.isnan(ValueLoss(0.2)(e2, e2, e2, action_mask=e2.bool()))
    adv, ret = get_advantages_and_returns(e2, e2, e2.bool(), 1.0, 0.95)
    assert adv.shape == (0, 16) and ret.shape == (0, 16)
    zero_cols = torch.empty(4, 0, device=cuda)
    adv, ret = get_advantages_and_returns(zero_cols, zero_cols, zero_cols.bool(), 1.0, 0.95)
    assert adv.shape == (4, 0)
    first, end, length = row_extents(torch.zeros(3, 0, dtype=torch.bool, device=cuda))
    assert first.tolist() == [0, 0, 0] and end.tolist() == [0, 0, 0] and length.tolist() == [0, 0, 0]
    assert cu_seqlens_of(torch.empty(0, dtype=torch.long, device=cuda)).tolist() == [0]
    assert pad_packed(torch.empty(0, device=cuda), torch.zeros(3, dtype=torch.long, device=cuda), 4, value=7.0).tolist() == [[7.0] * 4] * 2


def test_empty_inputs_of_the_sequence_and_layout_mirrors(cuda):
    from openrlhf_amd.models.utils import masked_normalize
    from openrlhf_amd.trainer.dpo_trainer import get_batch_logps
    from openrlhf_amd.trainer.ppo_utils.experience import PackedSteps
    from openrlhf_amd.trainer.ppo_utils.experience_maker import experience_kl
    from openrlhf_amd.utils.loss_utils import mask_counts

    e = torch.empty(0, 9, device=cuda)
    sums, means = get_batch_logps(e, torch.empty(0, 10, dtype=torch.long, device=cuda), [])
    assert sums.shape == (0,) and means.shape == (0,)
    kl, kl_mean, diff = experience_kl(e, e, e.bool(), "k2")
    assert kl.shape == (0, 9) and kl_mean.shape == (0,) and diff.shape == (0,)
    assert masked_normalize(e, e.bool()).shape == (0, 9)
    tokens, samples = mask_counts(torch.zeros(5, 7, dtype=torch.bool, device=cuda))
    assert tokens.item() == 0.0 and samples.item() == 0.0
    x = torch.randn(4, 6, device=cuda)
    ps = PackedSteps.from_padded(dict(x=x), torch.zeros(4, 6, dtype=torch.bool, device=cuda))  # nothing to keep
    assert ps.total == 0 and ps["x"].shape == (0,) and ps.cu_seqlens.tolist() == [0, 0, 0, 0, 0]
    assert torch.equal(ps.to_padded("x", value=0.0), torch.zeros(4, 6, device=cuda))

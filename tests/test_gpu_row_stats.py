"""The KL block of experience making (openrlhf/trainer/ppo_utils/experience_maker.py:202-216),
masked_normalize (openrlhf/models/utils.py:172-179) and the sequence-mean-of-token-sums
aggregation against the oracle and the golden vectors; 1e-5 absolute for fp32 inputs."""
import json
import math
import os

import pytest
import torch

from oracle import losses as ol
from oracle import token_numerics as otn

pytestmark = pytest.mark.gpu

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "token_numerics_golden.json")))
ATOL = 1e-5


def _close(got, ref, tol=ATOL):
    got, ref = got.detach().cpu().double(), torch.as_tensor(ref, dtype=torch.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    nan_g, nan_r = torch.isnan(got), torch.isnan(ref)
    assert torch.equal(nan_g, nan_r)
    if (~nan_r).any():
        err = (got[~nan_r] - ref[~nan_r]).abs().max().item()
        assert err <= tol, err


def _nan(v):
    return [math.nan if x is None else x for x in v]


def test_golden(cuda):
    from openrlhf_amd.models.loss import aggregate_loss
    from openrlhf_amd.models.utils import masked_normalize
    from openrlhf_amd.trainer.ppo_utils.experience_maker import experience_kl

    tok = GOLD["tokens"]
    f = lambda k: torch.tensor(tok[k], dtype=torch.float32, device=cuda)  # noqa: E731
    adv, mask, lp, base = f("advantages"), f("mask"), f("log_probs"), f("base_log_probs")
    _close(masked_normalize(adv, mask, dim=1, eps=1e-8), GOLD["masked_normalize"]["out"])
    for est, ref in GOLD["kl_rows"].items():
        kl, kl_mean, diff_mean = experience_kl(lp, base, mask.bool(), est)
        _close(kl, GOLD["approx_kl"][est])
        _close(kl_mean, _nan(ref["kl_mean"]))
        _close(diff_mean, _nan(ref["diff_mean"]))
    agg = GOLD["aggregate"]
    _close(aggregate_loss(adv, mask, token_level_loss=False, seq_token_sum=True), agg["seq_token_sum"])
    _close(aggregate_loss(adv, mask, token_level_loss=False, seq_token_sum=True, dp_size=2, global_batch_size=5.0),
           agg["seq_token_sum_global"])
    with pytest.raises(ValueError):
        aggregate_loss(adv, mask, seq_token_sum=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("est", ["k1", "k2", "k3"])
def test_experience_kl_vs_oracle(cuda, dtype, est):
    from openrlhf_amd.trainer.ppo_utils.experience_maker import experience_kl

    g = torch.Generator().manual_seed(4)
    b, a = 19, 1300
    lp = (-torch.rand(b, a, generator=g) * 6).to(dtype)
    base = (lp.float() + torch.randn(b, a, generator=g) * 1.5).to(dtype)
    base[0, :4] = lp[0, :4] + 14.0  # clamp at +-10 on both sides
    base[0, 4:8] = lp[0, 4:8] - 14.0
    lens = torch.randint(0, a + 1, (b,), generator=g)
    mask = torch.arange(a)[None, :] < lens[:, None]
    mask[3] = False
    r_kl, r_mean, r_diff = otn.experience_kl(lp.double(), base.double(), mask.double(), est)
    kl, kl_mean, diff_mean = experience_kl(lp.to(cuda), base.to(cuda), mask.to(cuda), est)
    assert kl.dtype == torch.float32
    _close(kl, r_kl)
    _close(kl_mean, r_mean)
    _close(diff_mean, r_diff)
    # CPU tensors (the controller's) come back on the CPU; the packed layout gives the same rows
    kl_c, mean_c, _ = experience_kl(lp, base, mask, est)
    assert kl_c.device.type == "cpu" and torch.equal(kl_c, kl.cpu()) and torch.equal(mean_c.isnan(), r_mean.isnan())
    keep = mask.reshape(-1)
    cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.masked_fill(~mask.any(1), 0).cumsum(0)]).to(cuda)
    kl_p, mean_p, diff_p = experience_kl(lp.reshape(-1)[keep].to(cuda), base.reshape(-1)[keep].to(cuda), None, est,
                                         cu_seqlens=cu)
    assert torch.equal(kl_p, kl.reshape(-1)[keep.to(cuda)])
    ok = ~r_mean.isnan()
    _close(mean_p[ok.to(cuda)], r_mean[ok])
    _close(diff_p[ok.to(cuda)], r_diff[ok])
    # no reference model: zeros and means of zeros (NaN for the empty row, as 0/0)
    kl0, mean0, diff0 = experience_kl(lp.to(cuda), None, mask.to(cuda), est)
    assert kl0.dtype == dtype and (kl0 == 0).all()
    _close(mean0, otn.experience_kl(lp.double(), None, mask.double(), est)[1])
    with pytest.raises(ValueError):
        experience_kl(lp.to(cuda), base.to(cuda), mask.to(cuda), "k4")


@pytest.mark.parametrize("shape,dim", [((1, 1), 1), ((6, 700), 1), ((6, 700), 0), ((3, 5, 257), -1), ((3, 5, 257), 1)])
def test_masked_normalize_vs_oracle(cuda, shape, dim):
    from openrlhf_amd.models.utils import masked_normalize

    g = torch.Generator().manual_seed(sum(shape))
    x = torch.randn(shape, generator=g) * 3 + 1
    mask = (torch.rand(shape, generator=g) > 0.3)
    if x.numel() > 10:
        mask.select(dim, 0)[...] = True
        mask.movedim(dim, -1).reshape(-1, shape[dim])[1] = False  # a row with no unmasked entry
    ref = otn.masked_normalize(x.double(), mask.double(), dim=dim)
    got = masked_normalize(x.to(cuda), mask.to(cuda), dim=dim)
    assert got.shape == x.shape
    _close(got, ref, 2e-5)
    assert (got.cpu()[~mask] == 0).all()
    # a constant row: variance 0 is clamped at eps, the output is 0 / sqrt(eps) = 0
    c = torch.full((2, 40), 2.5)
    assert (masked_normalize(c.to(cuda), torch.ones(2, 40, device=cuda)) == 0).all()


@pytest.mark.parametrize("global_norm", [False, True])
def test_seq_token_sum_vs_oracle_with_gradient(cuda, global_norm):
    from openrlhf_amd.models.loss import aggregate_loss

    g = torch.Generator().manual_seed(12)
    b, a = 37, 5000
    x = torch.randn(b, a, generator=g)
    lens = torch.randint(0, a + 1, (b,), generator=g)
    lens[5] = 0
    mask = torch.arange(a)[None, :] < lens[:, None]
    info = dict(dp_size=4, global_batch_size=29.0) if global_norm else {}
    xr = x.double().requires_grad_(True)
    ref = ol.aggregate_seq_token_sum(xr, mask.double(), **info)
    xd = x.to(cuda).requires_grad_(True)
    got = aggregate_loss(xd, mask.to(cuda), token_level_loss=False, seq_token_sum=True, **info)
    _close(got, ref.detach(), 1e-5 * max(1.0, abs(ref.item())))
    (gr,) = torch.autograd.grad(ref, xr)
    (gg,) = torch.autograd.grad(got, xd)
    _close(gg, gr, 1e-6)

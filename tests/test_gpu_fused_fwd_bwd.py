"""The one-pass forward+backward kernel against the fp64 oracle and against the separate
forward and backward kernels (same tolerances: 1e-5 abs for fp32 logits, 2e-3 abs for bf16/fp16;
gradients within the rounding of the logits dtype)."""
import pytest
import torch

from oracle import token_numerics as otn

pytestmark = pytest.mark.gpu


def _case(rows, vocab, dtype, std, seed):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(rows, vocab, generator=g) * std)
    r = torch.randperm(rows, generator=g)[: max(1, rows // 10)]
    x[r, torch.randint(0, vocab, (len(r),), generator=g)] += 15.0
    x = x.to(dtype)
    labels = torch.randint(0, vocab, (rows,), generator=g)
    w_lp, w_ent = torch.randn(rows, generator=g), torch.randn(rows, generator=g)
    w_lp[0] = 0.0
    w_ent[0] = 0.0
    return x, labels, w_lp, w_ent


def _analytic_grad64(x, labels, temperature, g_lp, g_ent):
    x64 = x.double()
    p_t = torch.softmax(x64 / temperature, -1)
    p = torch.softmax(x64, -1)
    onehot = torch.zeros_like(x64).scatter_(1, labels.unsqueeze(1), 1.0)
    ex = (p * x64).sum(-1, keepdim=True)
    return g_lp.double()[:, None] * (onehot - p_t) / temperature + g_ent.double()[:, None] * p * (ex - x64)


@pytest.mark.parametrize(
    "rows,vocab,dtype,std,temperature",
    [
        (40, 151936, torch.bfloat16, 3.0, 1.0),   # config-2 row: registers only
        (12, 262144, torch.bfloat16, 4.0, 0.6),   # config-5 row: half in registers, half streamed twice; two statistic sets
        (12, 200000, torch.float16, 2.0, 1.0),    # streamed tail, fp16
        (9, 155649, torch.bfloat16, 3.0, 1.0),    # one element more than the registers hold
        (33, 32000, torch.float32, 2.0, 1.0),
        (33, 50257, torch.bfloat16, 3.0, 0.7),    # scalar tail
        (17, 100003, torch.float32, 2.0, 1.3),    # fp32 streamed tail, odd vocabulary
        (300, 7, torch.float32, 1.0, 1.0),
        (64, 4096, torch.bfloat16, 2.0, 1.0),
        (5, 400000, torch.bfloat16, 2.0, 1.0),    # two thirds of the row streamed
        (3, 600000, torch.bfloat16, 2.0, 1.0),    # beyond the one-pass limit: separate kernels
    ],
)
@pytest.mark.parametrize("inplace", [True, False])
def test_fused_matches_oracle_and_two_kernel_path(cuda, rows, vocab, dtype, std, temperature, inplace):
    from openrlhf_amd.models.utils import fused_logprob_entropy_fwd_bwd, logprobs_and_entropy_from_logits

    x, labels, w_lp, w_ent = _case(rows, vocab, dtype, std, seed=rows + vocab)
    ref_lp = otn.log_probs_from_logits(x.double(), labels, temperature)
    ref_ent = otn.compute_entropy(x.double())
    ref_grad = _analytic_grad64(x, labels, temperature, w_lp, w_ent)

    xd = x.to(cuda)
    lp2, ent2 = logprobs_and_entropy_from_logits(xd, labels.to(cuda), temperature)
    lp, ent, grad = fused_logprob_entropy_fwd_bwd(xd, labels.to(cuda), w_lp.to(cuda), w_ent.to(cuda), temperature,
                                                  inplace=inplace)
    assert (grad.data_ptr() == xd.data_ptr()) == inplace and grad.dtype == dtype and grad.shape == x.shape
    atol = 1e-5 if dtype == torch.float32 else 2e-3
    assert (lp.cpu().double() - ref_lp).abs().max().item() <= atol
    assert (ent.cpu().double() - ref_ent).abs().max().item() <= atol
    assert (lp - lp2).abs().max().item() <= 2e-5 and (ent - ent2).abs().max().item() <= 2e-5
    err = (grad.cpu().double() - ref_grad).abs()
    if dtype == torch.float32:  # 1e-5 relative to the gradient scale (entries reach |w| * |x| ~ 20 here)
        assert err.max().item() <= 1e-5 * max(1.0, ref_grad.abs().max().item())
    else:
        eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
        assert (err <= eps * ref_grad.abs() + 1e-6).all(), err.max().item()
    assert grad[0].abs().max().item() == 0.0


def test_fused_misaligned_rows_row_mask_and_optional_weights(cuda):
    from openrlhf_amd.models.utils import fused_logprob_entropy_fwd_bwd

    rows, vocab, stride = 10, 4099, 4099 + 5
    g = torch.Generator().manual_seed(3)
    base = (torch.randn(rows * stride + 3, generator=g) * 2).to(torch.bfloat16)
    labels = torch.randint(0, vocab, (rows,), generator=g)
    w_lp = torch.randn(rows, generator=g)
    mask = torch.ones(rows, dtype=torch.bool)
    mask[3] = False
    for off in (0, 1, 3):
        x = base[off : off + rows * stride].view(rows, stride)[:, :vocab]
        xd = base.to(cuda)[off : off + rows * stride].view(rows, stride)[:, :vocab]
        lp, ent, grad = fused_logprob_entropy_fwd_bwd(xd, labels.to(cuda), w_lp.to(cuda), None, 1.0, inplace=True,
                                                      row_mask=mask.to(cuda))
        assert grad.data_ptr() == xd.data_ptr()
        ref_lp = otn.log_probs_from_logits(x.contiguous().double(), labels)
        ref = _analytic_grad64(x.contiguous(), labels, 1.0, w_lp, torch.zeros(rows))
        keep = mask
        assert (lp.cpu().double() - ref_lp)[keep].abs().max().item() <= 2e-3
        assert lp[3].item() == 0.0 and ent[3].item() == 0.0 and grad[3].abs().max().item() == 0.0
        err = (grad.cpu().double() - ref)[keep].abs()
        assert (err <= 2.0 ** -8 * ref[keep].abs() + 1e-6).all()


def test_fused_extreme_values_in_the_streamed_tail(cuda):
    """Long rows whose awkward entries sit in the streamed part: a late spike and a very low start
    force the exact-maximum pass over registers AND tail; -inf / +inf / NaN entries in the tail give
    the separate kernels' results."""
    from openrlhf_amd.models.utils import fused_logprob_entropy_fwd_bwd, logprobs_and_entropy_from_logits

    vocab = 200003
    g = torch.Generator().manual_seed(19)
    x = (torch.randn(6, vocab, generator=g) * 2).to(torch.bfloat16)
    x[0, vocab - 5] = 400.0
    x[1, :150000] = -3.0e4
    x[2, 160000::3] = float("-inf")
    x[3, vocab - 9] = float("inf")
    x[4, vocab - 2] = float("nan")
    labels = torch.tensor([vocab - 5, 190000, 160001, 3, 4, 7])
    w1, w2 = torch.randn(6, generator=g), torch.randn(6, generator=g)
    a = x.to(cuda).requires_grad_(True)
    lp2, ent2 = logprobs_and_entropy_from_logits(a, labels.to(cuda), 0.8)
    (g2,) = torch.autograd.grad((lp2 * w1.to(cuda)).sum() + (ent2 * w2.to(cuda)).sum(), a)
    lp, ent, grad = fused_logprob_entropy_fwd_bwd(x.to(cuda), labels.to(cuda), w1.to(cuda), w2.to(cuda), 0.8, inplace=True)

    def same(p, q, tol):
        p, q = p.float().cpu(), q.float().cpu()
        assert torch.equal(torch.isnan(p), torch.isnan(q))
        fin = torch.isfinite(p) & torch.isfinite(q)
        assert torch.equal(p[~fin & ~torch.isnan(p)], q[~fin & ~torch.isnan(q)])  # same infinities
        if fin.any():
            assert (p[fin] - q[fin]).abs().max().item() <= tol * max(1.0, q[fin].abs().max().item())

    same(lp, lp2, 2e-5)
    same(ent, ent2, 2e-5)
    same(grad, g2, 2.0 ** -7)
    ref_lp = otn.log_probs_from_logits(x[:3].double(), labels[:3], 0.8)
    assert (lp[:3].cpu().double() - ref_lp).abs().max().item() <= 2e-3 * max(1.0, ref_lp.abs().max().item() * 1e-2)


def test_fused_extreme_rows(cuda):
    """Rows the reference-maximum shortcut cannot handle (late huge spike, very low start, -inf
    entries) go through the on-chip exact-maximum path of the one-pass kernel and agree with the
    separate kernels and the oracle; +inf / NaN rows give the same inf / NaN pattern."""
    import math

    from openrlhf_amd.models.utils import fused_logprob_entropy_fwd_bwd, logprobs_and_entropy_from_logits

    vocab = 20000
    g = torch.Generator().manual_seed(9)
    x = torch.randn(6, vocab, generator=g)
    x[0, vocab - 5] = 500.0
    x[1, :1000] = -1.0e4
    x[2, ::3] = float("-inf")
    x[3, 17] = float("inf")
    x[4, 9] = float("nan")
    x[5] = x[5] * 30.0
    labels = torch.tensor([vocab - 5, 5000, 1, 3, 4, 7])
    w = torch.randn(6, generator=g)
    ref_lp = otn.log_probs_from_logits(x.double(), labels)
    ref_ent = otn.compute_entropy(x.double())
    xd = x.to(cuda)
    lp2, ent2 = logprobs_and_entropy_from_logits(xd, labels.to(cuda))
    lp, ent, grad = fused_logprob_entropy_fwd_bwd(xd, labels.to(cuda), w.to(cuda), None, 1.0, inplace=False)
    lp, ent = lp.cpu().double(), ent.cpu().double()
    for i in (0, 1, 5):
        assert abs(lp[i] - ref_lp[i]) <= 1e-5 * max(1.0, abs(ref_lp[i].item()) * 1e-1)
        assert abs(ent[i] - ref_ent[i]) <= 1e-4
        gref = _analytic_grad64(x[i:i + 1], labels[i:i + 1], 1.0, w[i:i + 1], torch.zeros(1))
        # softmax of fp32 logits of magnitude |x| carries ~1e-7 * |x| of rounding in the exponent
        tol = 1e-5 * max(1.0, gref.abs().max().item()) + 2e-7 * x[i].abs()[x[i].abs() < 1e30].max().item()
        assert (grad[i:i + 1].cpu().double() - gref).abs().max().item() <= tol
    assert abs(lp[2] - ref_lp[2]) <= 1e-5 and math.isnan(ent[2])
    assert lp[3] == float("-inf") and math.isnan(ent[3])
    assert math.isnan(lp[4]) and math.isnan(ent[4])
    assert torch.equal(lp2.cpu().isnan(), lp.isnan()) and torch.equal(ent2.cpu().isnan(), ent.isnan())


def _device_case(cuda, rows, vocab, dtype, std, seed):
    g = torch.Generator(device=cuda).manual_seed(seed)
    x = torch.empty(rows, vocab, dtype=dtype, device=cuda)
    for lo in range(0, rows, 512):
        hi = min(lo + 512, rows)
        x[lo:hi] = (torch.randn(hi - lo, vocab, generator=g, device=cuda) * std).to(dtype)
    spiked = torch.randperm(rows, generator=g, device=cuda)[: max(1, rows // 50)]
    x[spiked, torch.randint(0, vocab, (len(spiked),), generator=g, device=cuda)] += 15.0
    labels = torch.randint(0, vocab, (rows,), generator=g, device=cuda)
    w_lp = torch.randn(rows, generator=g, device=cuda)
    w_ent = torch.randn(rows, generator=g, device=cuda)
    return x, labels, w_lp, w_ent


def _close_to_rounding(got, want, dtype, slab=1024):
    """got / want: [N, V] gradients of two kernels that round the same fp32 value independently."""
    eps = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 2e-5}[dtype]
    worst = 0.0
    for lo in range(0, got.shape[0], slab):
        a, b = got[lo:lo + slab].float(), want[lo:lo + slab].float()
        excess = ((a - b).abs() - eps * b.abs()).max().item()
        worst = max(worst, excess)
    return worst


@pytest.mark.parametrize(
    "rows,vocab,dtype,std,temperature",
    [
        (1200, 151936, torch.bfloat16, 3.0, 1.0),   # 4-5 rows per workgroup, all 38 register chunks refilled
        (700, 151936, torch.bfloat16, 3.0, 0.8),    # the same with two statistic sets
        (600, 200003, torch.bfloat16, 3.0, 1.0),    # register part + streamed tail, odd vocabulary (scalar tail)
        (530, 262144, torch.bfloat16, 4.0, 0.6),    # config-5 row shape, streamed half, two statistic sets
        (2000, 32000, torch.float32, 2.0, 1.0),     # fp32, 16 of 38 chunks live
        (1500, 50257, torch.bfloat16, 3.0, 1.0),    # scalar tail, 13 of 38 chunks live
        (300, 77825, torch.float32, 2.0, 1.3),      # fp32 row one element longer than the registers hold
        (257, 155648, torch.float16, 2.0, 1.0),     # exactly the register capacity; one workgroup gets a second row
    ],
)
@pytest.mark.parametrize("masked", [False, True])
def test_fused_many_rows_per_workgroup(cuda, rows, vocab, dtype, std, temperature, masked):
    """More rows than workgroups (one per CU): the row-to-row pipeline, where every register chunk
    is refilled from the workgroup's next row while the current row's gradient is stored. All rows
    against the separate forward and backward kernels, a row sample against the fp64 oracle. With
    `masked`, half of the rows are switched off at random, so unwanted rows fall before, between
    and after the wanted rows of one workgroup."""
    from openrlhf_amd.models.utils import fused_logprob_entropy_fwd_bwd, logprobs_and_entropy_from_logits

    x, labels, w_lp, w_ent = _device_case(cuda, rows, vocab, dtype, std, seed=rows * 7 + vocab)
    g = torch.Generator().manual_seed(rows + 1)
    row_mask = None
    if masked:
        row_mask = (torch.rand(rows, generator=g) < 0.5)
        row_mask[:3] = torch.tensor([False, True, False])
        row_mask[256:259] = False  # second rows of workgroups 0-2 off
        row_mask[-2:] = False
        row_mask = row_mask.to(cuda)
    keep = torch.ones(rows, dtype=torch.bool, device=cuda) if row_mask is None else row_mask
    pick = torch.nonzero(keep).squeeze(-1)
    pick = pick[torch.randperm(len(pick), generator=g)[:12].to(cuda)]
    x_pick = x[pick].cpu()

    xa = x.clone().requires_grad_(True)
    lp2, ent2 = logprobs_and_entropy_from_logits(xa, labels, temperature, inplace_backward=True, row_mask=row_mask)
    (g2,) = torch.autograd.grad([lp2, ent2], [xa], [w_lp, w_ent])
    lp, ent, grad = fused_logprob_entropy_fwd_bwd(x, labels, w_lp, w_ent, temperature, inplace=True, row_mask=row_mask)
    assert grad.data_ptr() == x.data_ptr()

    atol = 1e-5 if dtype == torch.float32 else 2e-3
    assert (lp - lp2).abs().max().item() <= 2e-5 and (ent - ent2).abs().max().item() <= 2e-5
    assert _close_to_rounding(grad, g2, dtype) <= 4e-6
    if masked:
        off = ~keep
        assert lp[off].abs().max().item() == 0.0 and ent[off].abs().max().item() == 0.0
        assert grad[off].abs().max().item() == 0.0
    ref_lp = otn.log_probs_from_logits(x_pick.double(), labels[pick].cpu(), temperature)
    ref_ent = otn.compute_entropy(x_pick.double())
    assert (lp[pick].cpu().double() - ref_lp).abs().max().item() <= atol
    assert (ent[pick].cpu().double() - ref_ent).abs().max().item() <= atol
    ref = _analytic_grad64(x_pick, labels[pick].cpu(), temperature, w_lp[pick].cpu(), w_ent[pick].cpu())
    err = (grad[pick].cpu().double() - ref).abs()
    if dtype == torch.float32:
        assert err.max().item() <= 1e-5 * max(1.0, ref.abs().max().item())
    else:
        eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
        assert (err <= eps * ref.abs() + 1e-6).all(), err.max().item()

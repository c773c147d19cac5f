"""Launches with fewer vocabulary rows than the GPU has compute units: every row is cut into
segments, one workgroup each (openrlhf/models/utils.py:139-163,182-186 on a short rollout or a
small micro-batch). Forward and backward against the CPU oracle (1e-5 abs for fp32 logits, 2e-3
for 16-bit logits), against the whole-row kernels on the same rows, and on rows with extreme
values in one segment only."""
import math

import pytest
import torch

from oracle import token_numerics as otn

pytestmark = pytest.mark.gpu


def _case(rows, vocab, dtype, std, seed):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(rows, vocab, generator=g) * std).to(dtype)
    labels = torch.randint(0, vocab, (rows,), generator=g)
    g_lp, g_ent = torch.randn(rows, generator=g), torch.randn(rows, generator=g)
    return x, labels, g_lp, g_ent


def _analytic_grad64(x, labels, temperature, g_lp, g_ent):
    x64 = x.double()
    p_t = torch.softmax(x64 / temperature, -1)
    p = torch.softmax(x64, -1)
    onehot = torch.zeros_like(x64).scatter_(1, labels.unsqueeze(1), 1.0)
    ex = (p * x64).sum(-1, keepdim=True)
    return g_lp.double().unsqueeze(1) * (onehot - p_t) / temperature + g_ent.double().unsqueeze(1) * p * (ex - x64)


def _is_cut(x):
    from openrlhf_amd import _lib

    return _lib.load().orlhf_logprob_entropy_split_workspace_bytes(_lib.dtype_code(x), x.shape[0], x.shape[1]) > 0


def _whole_rows(xd, labels, temperature):
    """The same rows through the whole-row kernel: the batch padded to 256 rows is not cut."""
    from openrlhf_amd.models.utils import logprobs_and_entropy_from_logits

    n = xd.shape[0]
    pad = torch.cat([xd, xd[:1].expand(256 - n, -1)], 0).contiguous()
    lab = torch.cat([labels, labels[:1].expand(256 - n)], 0)
    assert not _is_cut(pad)
    lp, ent = logprobs_and_entropy_from_logits(pad, lab, temperature)
    return lp[:n], ent[:n]


@pytest.mark.parametrize("rows", [1, 7, 64, 255])
@pytest.mark.parametrize(
    "vocab,dtype,std,temperature",
    [
        (151936, torch.bfloat16, 3.0, 1.0),   # the headline vocabulary
        (151936, torch.bfloat16, 3.0, 0.6),   # two statistic sets
        (50257, torch.float32, 2.0, 0.7),     # odd vocabulary: the last segment is ragged
        (65536, torch.float16, 2.0, 1.0),
    ],
)
def test_few_rows_forward_backward(cuda, rows, vocab, dtype, std, temperature):
    from openrlhf_amd.models.utils import logprobs_and_entropy_from_logits

    x, labels, g_lp, g_ent = _case(rows, vocab, dtype, std, seed=rows * 31 + vocab)
    assert _is_cut(x)
    # labels at the ends of the row and around a segment boundary as well as random ones
    labels[0] = vocab - 1
    if rows > 2:
        labels[1], labels[2] = 0, vocab // 2
    ref_lp = otn.log_probs_from_logits(x.double(), labels, temperature)
    ref_ent = otn.compute_entropy(x.double())
    atol = 1e-5 if dtype == torch.float32 else 2e-3
    xd = x.to(cuda).requires_grad_(True)
    lp, ent = logprobs_and_entropy_from_logits(xd, labels.to(cuda), temperature)
    assert (lp.detach().cpu().double() - ref_lp).abs().max().item() <= atol
    assert (ent.detach().cpu().double() - ref_ent).abs().max().item() <= atol
    # against the whole-row kernel: only the grouping of the fp32 partial sums differs
    lp_w, ent_w = _whole_rows(xd.detach(), labels.to(cuda), temperature)
    assert (lp.detach() - lp_w).abs().max().item() <= 4e-6
    assert (ent.detach() - ent_w).abs().max().item() <= 4e-6

    torch.autograd.backward([lp, ent], [g_lp.to(cuda), g_ent.to(cuda)])
    ref_g = _analytic_grad64(x, labels, temperature, g_lp, g_ent)
    err = (xd.grad.cpu().double() - ref_g).abs()
    eps = {torch.float32: 2.0 ** -22, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[dtype]
    assert (err <= eps * ref_g.abs() + 2e-6).all(), err.max().item()


def test_few_rows_one_pass_entry_and_row_mask(cuda):
    """`fused_logprob_entropy_fwd_bwd` on a small batch takes the cut forward and backward; rows
    the mask leaves out give zeros and are not differentiated."""
    from openrlhf_amd.models.utils import fused_logprob_entropy_fwd_bwd

    rows, vocab = 40, 151936
    x, labels, w_lp, w_ent = _case(rows, vocab, torch.bfloat16, 3.0, seed=77)
    mask = torch.ones(rows, dtype=torch.bool)
    mask[[0, 5, 6, 39]] = False
    ref_lp = otn.log_probs_from_logits(x.double(), labels, 1.0) * mask
    ref_ent = otn.compute_entropy(x.double()) * mask
    ref_g = _analytic_grad64(x, labels, 1.0, w_lp * mask, w_ent * mask)
    xd = x.to(cuda)
    lp, ent, grad = fused_logprob_entropy_fwd_bwd(xd, labels.to(cuda), w_logprob=w_lp.to(cuda), w_entropy=w_ent.to(cuda),
                                                  inplace=True, row_mask=mask.to(cuda))
    assert grad.data_ptr() == xd.data_ptr()
    assert (lp.cpu().double() - ref_lp).abs().max().item() <= 2e-3
    assert (ent.cpu().double() - ref_ent).abs().max().item() <= 2e-3
    err = (grad.cpu().double() - ref_g).abs()
    assert (err <= 2.0 ** -8 * ref_g.abs() + 2e-6).all(), err.max().item()
    assert grad[~mask.to(cuda)].abs().max().item() == 0.0


def test_few_rows_extreme_segments(cuda):
    """Extreme values confined to one segment: a late spike far above the rest, a segment that is
    all -inf, +inf and NaN logits. Values follow torch's logsumexp / softmax semantics, i.e. what
    the whole-row kernel returns on the same rows."""
    from openrlhf_amd.models.utils import logprobs_and_entropy_from_logits

    vocab = 100000
    g = torch.Generator().manual_seed(19)
    x = torch.randn(8, vocab, generator=g)
    x[0, vocab - 5] = 500.0
    x[1, :30000] = -1.0e4
    x[2, 40000:70000] = float("-inf")
    x[3, 60017] = float("inf")
    x[4, 99999] = float("nan")
    x[5] = x[5] * 30.0
    x[6, :] = float("-inf")
    x[6, 12345] = 2.0
    labels = torch.tensor([vocab - 5, 50000, 1, 3, 4, 7, 12345, 99999])
    assert _is_cut(x)
    ref_lp = otn.log_probs_from_logits(x.double(), labels)
    ref_ent = otn.compute_entropy(x.double())
    xd = x.to(cuda)
    lp, ent = logprobs_and_entropy_from_logits(xd, labels.to(cuda))
    lp_w, ent_w = _whole_rows(xd, labels.to(cuda), 1.0)
    assert torch.allclose(lp, lp_w, rtol=1e-6, atol=1e-5, equal_nan=True), (lp, lp_w)
    assert torch.allclose(ent, ent_w, rtol=1e-6, atol=1e-4, equal_nan=True), (ent, ent_w)
    lp, ent = lp.cpu().double(), ent.cpu().double()
    for i in (0, 1, 5, 7):
        assert abs(lp[i] - ref_lp[i]) <= 1e-5 * max(1.0, abs(ref_lp[i].item()) * 1e-1), (i, lp[i], ref_lp[i])
        assert abs(ent[i] - ref_ent[i]) <= 1e-4, (i, ent[i], ref_ent[i])
    assert abs(lp[2] - ref_lp[2]) <= 1e-5 and math.isnan(ent[2]) and math.isnan(ref_ent[2])
    assert lp[3] == ref_lp[3] == float("-inf") and math.isnan(ent[3])
    assert math.isnan(lp[4]) and math.isnan(ent[4])
    assert abs(lp[6] - ref_lp[6]) <= 1e-6 and math.isnan(ent[6])
    bad = torch.tensor([-100, -1, vocab, 0, 0, 0, 0, 0])
    lp2, _ = logprobs_and_entropy_from_logits(xd, bad.to(cuda))
    assert lp2[0].item() == 0.0 and math.isnan(lp2[1].item()) and math.isnan(lp2[2].item())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_few_rows_unaligned_and_strided(cuda, dtype):
    """Row starts off the 16-byte grid and an odd row stride: every segment inherits its row's phase."""
    from openrlhf_amd.models.utils import logprobs_and_entropy_from_logits

    rows, vocab, stride = 5, 70001, 70001 + 5
    g = torch.Generator().manual_seed(23)
    base = (torch.randn(rows * stride + 3, generator=g) * 2).to(dtype)
    labels = torch.randint(0, vocab, (rows,), generator=g)
    g_lp, g_ent = torch.randn(rows, generator=g), torch.randn(rows, generator=g)
    for off in (0, 1, 3):
        x = base[off : off + rows * stride].view(rows, stride)[:, :vocab]
        ref_lp = otn.log_probs_from_logits(x.double(), labels, 1.0)
        ref_ent = otn.compute_entropy(x.double())
        xd = base.to(cuda)[off : off + rows * stride].view(rows, stride)[:, :vocab].requires_grad_(True)
        lp, ent = logprobs_and_entropy_from_logits(xd, labels.to(cuda), 1.0)
        atol = 1e-5 if dtype == torch.float32 else 2e-3
        assert (lp.detach().cpu().double() - ref_lp).abs().max().item() <= atol
        assert (ent.detach().cpu().double() - ref_ent).abs().max().item() <= atol
        (grad,) = torch.autograd.grad([lp, ent], [xd], [g_lp.to(cuda), g_ent.to(cuda)])
        ref_g = _analytic_grad64(x.contiguous(), labels, 1.0, g_lp, g_ent)
        eps = 2.0 ** -22 if dtype == torch.float32 else 2.0 ** -8
        err = (grad.cpu().double() - ref_g).abs()
        assert (err <= eps * ref_g.abs() + 2e-6).all(), err.max().item()


def test_split_entry_contract(cuda):
    """The C entry: no workspace needed when rows are not cut, an error when one is needed and
    missing or too small, and the plain entry still runs whole rows on a small batch."""
    from openrlhf_amd import _lib
    from openrlhf_amd._lib import call, ptr, stream_of

    lib = _lib.load()
    assert lib.orlhf_logprob_entropy_split_workspace_bytes(1, 256, 151936) == 0
    assert lib.orlhf_logprob_entropy_split_workspace_bytes(1, 64, 8192) == 0       # rows too short to cut
    need = lib.orlhf_logprob_entropy_split_workspace_bytes(1, 64, 151936)
    assert need == 64 * 8 * 32
    x, labels, _, _ = _case(64, 151936, torch.bfloat16, 3.0, seed=3)
    xd, ld = x.to(cuda), labels.to(cuda)
    lp, ent = torch.empty(64, device=cuda), torch.empty(64, device=cuda)
    ws = torch.empty(need, dtype=torch.uint8, device=cuda)
    args = (ptr(xd), 1, 64, 151936, 151936, ptr(ld), 1.0, ptr(lp), ptr(ent), None, None)
    with pytest.raises(_lib.KernelError, match="workspace"):
        call("orlhf_logprob_entropy_fwd_split", *args, None, 0, None, stream_of(cuda))
    with pytest.raises(_lib.KernelError, match="workspace"):
        call("orlhf_logprob_entropy_fwd_split", *args, ptr(ws), need - 1, None, stream_of(cuda))
    call("orlhf_logprob_entropy_fwd_split", *args, ptr(ws), need, None, stream_of(cuda))
    lp2, ent2 = torch.empty(64, device=cuda), torch.empty(64, device=cuda)
    call("orlhf_logprob_entropy_fwd", ptr(xd), 1, 64, 151936, 151936, ptr(ld), 1.0, ptr(lp2), ptr(ent2), None, None, 0,
         stream_of(cuda))
    assert (lp - lp2).abs().max().item() <= 4e-6 and (ent - ent2).abs().max().item() <= 4e-6


@pytest.mark.parametrize("rows", [1, 7, 64, 255])
@pytest.mark.parametrize(
    "vocab,dtype,temperature,want",
    [
        (151936, torch.bfloat16, 1.0, "both"),
        (151936, torch.bfloat16, 0.6, "both"),
        (151936, torch.bfloat16, 0.6, "logprob"),
        (50257, torch.float32, 0.7, "entropy"),
        (65536, torch.float16, 1.0, "both"),
    ],
)
def test_merge_by_last_segment_is_bit_identical(cuda, rows, vocab, dtype, temperature, want):
    """With tickets the forward kernel merges a row in the workgroup that finishes its last segment;
    without, a second kernel does. Same records, same order: the same bits, whichever workgroup
    came last, launch after launch on the same ticket array (the kernel leaves it zero), with rows
    masked out, extreme rows (the safe pass) and labels outside the vocabulary among them."""
    from openrlhf_amd import _lib
    from openrlhf_amd._lib import call, ptr, stream_of

    lib = _lib.load()
    x, labels, _, _ = _case(rows, vocab, dtype, 3.0, seed=rows + vocab)
    x[0, 5] = 30000.0 if dtype == torch.float16 else 3e38   # the fast pass overflows on this row
    if rows > 2:
        labels[1] = -100
        x[2, vocab // 2:] = -float("inf")
    mask = torch.ones(rows, dtype=torch.uint8)
    if rows > 4:
        mask[3] = 0
    xd, ld, md = x.to(cuda), labels.to(cuda), mask.to(cuda)
    need = lib.orlhf_logprob_entropy_split_workspace_bytes(_lib.dtype_code(xd), rows, vocab)
    assert need > 0
    tickets = torch.zeros(rows, dtype=torch.int32, device=cuda)

    def run(t):
        ws = torch.full((need,), 0xFF, dtype=torch.uint8, device=cuda)
        lp = torch.full((rows,), 7.0, device=cuda) if want != "entropy" else None
        ent = torch.full((rows,), 7.0, device=cuda) if want != "logprob" else None
        stats = torch.full((rows, 4), 7.0, device=cuda)
        call("orlhf_logprob_entropy_fwd_split", ptr(xd), _lib.dtype_code(xd), rows, vocab, vocab, ptr(ld), temperature,
             ptr(lp), ptr(ent), ptr(stats), ptr(md), ptr(ws), need, ptr(t), stream_of(cuda))
        return [o for o in (lp, ent, stats) if o is not None]

    two_launches = run(None)
    for _ in range(3):
        one_launch = run(tickets)
        assert int(tickets.abs().sum().item()) == 0
        for a, b in zip(two_launches, one_launch):
            assert torch.equal(a.view(torch.int32), b.view(torch.int32))
    if rows > 4:
        assert all(float(o[3].abs().sum().item()) == 0.0 for o in two_launches)


def test_mirror_keeps_one_ticket_array_per_stream(cuda):
    """The Python mirror's ticket array: one per (device, stream), zero between calls, reused."""
    from openrlhf_amd.models import utils

    x, labels, _, _ = _case(64, 151936, torch.bfloat16, 3.0, seed=11)
    xd, ld = x.to(cuda), labels.to(cuda)
    lp0, ent0 = utils.logprobs_and_entropy_from_logits(xd, ld, 1.0)
    side = torch.cuda.Stream(device=cuda)
    side.wait_stream(torch.cuda.current_stream(cuda))
    with torch.cuda.stream(side):
        lp1, ent1 = utils.logprobs_and_entropy_from_logits(xd, ld, 1.0)
    side.synchronize()
    torch.cuda.synchronize()
    assert torch.equal(lp0, lp1) and torch.equal(ent0, ent1)
    mine = [t for (d, _), t in utils._TICKETS.items() if d == cuda.index]
    assert len(mine) >= 2 and all(int(t.abs().sum().item()) == 0 for t in mine)


def test_merge_by_last_segment_over_many_launches(cuda):
    """The same ticket array through 600 launches back to back (three shapes in rotation, no
    synchronisation between launches): every launch's outputs are the two-launch form's bits and the
    tickets are back at zero at the end. Which workgroup draws a row's last ticket changes from launch
    to launch; the records it reads must be complete whoever it is."""
    from openrlhf_amd import _lib
    from openrlhf_amd._lib import call, ptr, stream_of

    lib = _lib.load()
    shapes = [(64, 151936, torch.bfloat16), (255, 65536, torch.float16), (7, 50257, torch.float32)]
    tickets = torch.zeros(256, dtype=torch.int32, device=cuda)
    cases = []
    for k, (rows, vocab, dtype) in enumerate(shapes):
        x, labels, _, _ = _case(rows, vocab, dtype, 3.0, seed=100 + k)
        xd, ld = x.to(cuda), labels.to(cuda)
        need = lib.orlhf_logprob_entropy_split_workspace_bytes(_lib.dtype_code(xd), rows, vocab)
        ws = torch.empty(need, dtype=torch.uint8, device=cuda)
        want = [torch.empty(rows, device=cuda), torch.empty(rows, device=cuda), torch.empty(rows, 4, device=cuda)]
        args = (ptr(xd), _lib.dtype_code(xd), rows, vocab, vocab, ptr(ld), 0.8)
        call("orlhf_logprob_entropy_fwd_split", *args, *(ptr(o) for o in want), None, ptr(ws), need, None, stream_of(cuda))
        cases.append((args, ws, need, want, xd, ld))
    torch.cuda.synchronize()
    rounds = 200
    outs = [[torch.full_like(w, 7.0) for w in want] for (_, _, _, want, _, _) in cases]
    bad = torch.zeros((), dtype=torch.int64, device=cuda)
    for r in range(rounds):
        for (args, ws, need, want, _, _), got in zip(cases, outs):
            call("orlhf_logprob_entropy_fwd_split", *args, *(ptr(o) for o in got), None, ptr(ws), need, ptr(tickets),
                 stream_of(cuda))
            for a, b in zip(want, got):
                bad += (a.view(torch.int32) != b.view(torch.int32)).sum()
                b.fill_(7.0)
    assert int(bad.item()) == 0
    assert int(tickets.abs().sum().item()) == 0

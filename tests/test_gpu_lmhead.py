"""lm-head + log-prob / entropy without the logits in memory (openrlhf/models/actor.py:263-285 with
the projection in front): the matrix-core path against the CPU oracle.

The path rounds its logits to the 16-bit dtype as the reference's lm_head output is rounded, so the
comparison is made in the two steps tests/lmhead_util.py describes: the rounded logits against the
fp64 product (half a 16-bit ulp), then log-probs / entropies (1e-4 abs: 16-bit logits in, fp32
statistics) and both gradients (entry by entry within the rounding of a 16-bit logits gradient and
a 16-bit result) against the oracle applied to exactly those logits. Against the oracle on the
UNROUNDED fp64 logits the values agree to the 16-bit rounding of the logits themselves."""
import pytest
import torch

from oracle import token_numerics as otn
from tests.lmhead_util import (assert_gradient, check_rounded_logits, closed_form_from_logits, forward_keeping_logits,
                               oracle_from_logits, unit_roundoff)

pytestmark = pytest.mark.gpu


def _case(n, hdim, vocab, dtype, seed, std=3.0):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(n, hdim, generator=g).to(dtype)
    weight = (torch.randn(vocab, hdim, generator=g) * (std / hdim ** 0.5)).to(dtype)
    labels = torch.randint(0, vocab, (n,), generator=g)
    g_lp, g_ent = torch.randn(n, generator=g), torch.randn(n, generator=g)
    return hidden, weight, labels, g_lp, g_ent


def _check_against_oracle(cuda, hidden, weight, labels, temperature, g_lp, g_ent, **kw):
    """Forward + backward through the public mirror against the two-step reference; returns the
    device results."""
    from openrlhf_amd.models.utils import lm_head_logprobs_and_entropy

    dtype = hidden.dtype
    hd = hidden.to(cuda).requires_grad_(True)
    wd = weight.to(cuda).requires_grad_(True)
    lab = labels.to(cuda)
    lp_k, ent_k, _, kept, _ = forward_keeping_logits(hd.detach(), wd.detach(), lab, temperature)
    x64 = check_rounded_logits(kept.cpu(), hidden, weight)
    logits = kept[:, : weight.shape[0]]
    ref_lp, ref_ent, ref_gh, ref_gw, bound_h, bound_w = oracle_from_logits(logits, hidden, weight, labels, temperature, g_lp, g_ent)

    lp, ent = lm_head_logprobs_and_entropy(hd, wd, lab, temperature, **kw)
    assert lp.dtype == torch.float32 and lp.shape == labels.shape
    assert torch.equal(lp, lp_k) and torch.equal(ent, ent_k)  # keeping the logits changes nothing
    assert (lp.detach().cpu().double() - ref_lp).abs().max().item() <= 1e-4
    assert (ent.detach().cpu().double() - ref_ent).abs().max().item() <= 1e-4
    # and the reference's own rounding apart, the unrounded product gives the same numbers
    u = unit_roundoff(dtype)
    loose = 4 * u * x64.abs().max().item() / min(temperature, 1.0) + 1e-4
    assert (lp.detach().cpu().double() - otn.log_probs_from_logits(x64, labels, temperature)).abs().max().item() <= loose
    assert (ent.detach().cpu().double() - otn.compute_entropy(x64)).abs().max().item() <= loose
    torch.autograd.backward([lp, ent], [g_lp.to(cuda), g_ent.to(cuda)])
    assert hd.grad.dtype == dtype and wd.grad.dtype == dtype
    assert_gradient(hd.grad.cpu(), ref_gh, bound_h, "grad_hidden")
    assert_gradient(wd.grad.cpu(), ref_gw, bound_w, "grad_weight")
    return lp.detach(), ent.detach(), hd.grad, wd.grad


@pytest.mark.parametrize(
    "n,hdim,vocab,dtype,temperature",
    [
        (256, 64, 256, torch.bfloat16, 1.0),      # exactly one tile, one slab
        (300, 128, 1000, torch.bfloat16, 1.0),    # ragged tokens and vocabulary
        (513, 200, 5003, torch.bfloat16, 0.7),    # hidden size not a multiple of the slab, odd vocabulary, T != 1
        (70, 4100, 777, torch.float16, 1.3),      # long ragged contraction, fp16
        (1, 64, 50, torch.bfloat16, 1.0),         # a single token, tiny vocabulary
        (1500, 512, 20000, torch.bfloat16, 0.6),  # several token blocks; a last vocabulary tile with whole lanes past the end
        (260, 96, 2336, torch.float16, 0.6),      # fp16, T != 1, last tile with 32 entries
    ],
)
def test_lmhead_matches_oracle(cuda, n, hdim, vocab, dtype, temperature):
    hidden, weight, labels, g_lp, g_ent = _case(n, hdim, vocab, dtype, seed=n + hdim + vocab)
    _check_against_oracle(cuda, hidden, weight, labels, temperature, g_lp, g_ent)


@pytest.mark.parametrize("temperature", [1.0, 0.8])
def test_lmhead_memory_budgets_give_the_same_bits(cuda, temperature):
    """keep_logits_mib decides how many vocabulary columns of logits the forward stores and
    backward_chunk_mib how the rest is cut: neither changes a bit of any result (the kept logits are
    what the recompute rounds to, and the hidden-state gradient's sum over the vocabulary is
    continued inside the accumulators in one order)."""
    from openrlhf_amd.models.utils import lm_head_logprobs_and_entropy

    n, hdim, vocab = 1500, 256, 20011
    hidden, weight, labels, g_lp, g_ent = _case(n, hdim, vocab, torch.bfloat16, seed=77)
    base = _check_against_oracle(cuda, hidden, weight, labels, temperature, g_lp, g_ent)
    # n * (cols + 64) * 2 bytes: 1 MiB holds 256 columns, 16 MiB 5376, 64 MiB everything
    for keep, chunk in ((None, 1), (None, 3), (None, 4096), (1, None), (16, 2), (16, None), (64, None)):
        hd = hidden.to(cuda).requires_grad_(True)
        wd = weight.to(cuda).requires_grad_(True)
        lp, ent = lm_head_logprobs_and_entropy(hd, wd, labels.to(cuda), temperature, keep_logits_mib=keep,
                                               backward_chunk_mib=chunk)
        torch.autograd.backward([lp, ent], [g_lp.to(cuda), g_ent.to(cuda)])
        for got, want in zip((lp.detach(), ent.detach(), hd.grad, wd.grad), base):
            assert torch.equal(got, want), (keep, chunk)


def test_lmhead_kept_logits_are_consumed_once(cuda):
    """The backward turns the stored logits into their gradient in place: a second backward through
    the same graph raises instead of differentiating gradients."""
    from openrlhf_amd.models.utils import lm_head_logprobs_and_entropy

    hidden, weight, labels, g_lp, g_ent = _case(300, 128, 1000, torch.bfloat16, seed=3)
    hd = hidden.to(cuda).requires_grad_(True)
    wd = weight.to(cuda).requires_grad_(True)
    lp, ent = lm_head_logprobs_and_entropy(hd, wd, labels.to(cuda), 1.0, keep_logits_mib=64)
    loss = (lp * g_lp.to(cuda)).sum() + (ent * g_ent.to(cuda)).sum()
    loss.backward(retain_graph=True)
    with pytest.raises(RuntimeError, match="stored logits"):
        loss.backward()
    # without stored logits the graph can be walked twice
    lp, ent = lm_head_logprobs_and_entropy(hd, wd, labels.to(cuda), 1.0)
    loss = (lp * g_lp.to(cuda)).sum()
    g1 = torch.autograd.grad(loss, [hd], retain_graph=True)[0]
    g2 = torch.autograd.grad(loss, [hd])[0]
    assert torch.equal(g1, g2)


def test_lmhead_batch_shape_row_mask_and_strides(cuda):
    """[B, T, H] hidden states with masked positions (left out of the projection altogether), a
    weight that is a strided view, and labels outside the vocabulary."""
    from openrlhf_amd.models.utils import lm_head_logprobs_and_entropy

    b, t, hdim, vocab = 3, 50, 96, 700
    g = torch.Generator().manual_seed(5)
    hidden = torch.randn(b, t, hdim, generator=g).to(torch.bfloat16)
    wbig = (torch.randn(vocab, hdim + 8, generator=g) * 0.3).to(torch.bfloat16)
    weight = wbig[:, :hdim]
    labels = torch.randint(0, vocab, (b, t), generator=g)
    mask = torch.rand(b, t, generator=g) > 0.4
    g_lp, g_ent = torch.randn(b, t, generator=g), torch.randn(b, t, generator=g)

    hd = hidden.to(cuda).requires_grad_(True)
    wd_big = wbig.to(cuda)
    wd = wd_big[:, :hdim].requires_grad_(True)
    flat_h, flat_lab = hd.detach().reshape(-1, hdim), labels.reshape(-1).to(cuda)
    _, _, _, kept, _ = forward_keeping_logits(flat_h, wd.detach(), flat_lab, 0.9)
    check_rounded_logits(kept.cpu(), hidden.reshape(-1, hdim), weight)
    km = mask.reshape(-1).double()
    ref_lp, ref_ent, ref_gh, ref_gw, bound_h, bound_w = oracle_from_logits(
        kept[:, :vocab], hidden.reshape(-1, hdim), weight, labels.reshape(-1), 0.9, g_lp.reshape(-1) * km, g_ent.reshape(-1) * km)

    for keep_mib in (None, 1):
        hd.grad = wd.grad = None
        lp, ent = lm_head_logprobs_and_entropy(hd, wd, labels.to(cuda), 0.9, row_mask=mask.to(cuda), keep_logits_mib=keep_mib)
        assert lp.shape == (b, t)
        assert (lp.detach().cpu().double().reshape(-1) - ref_lp * km).abs().max().item() <= 1e-4
        assert (ent.detach().cpu().double().reshape(-1) - ref_ent * km).abs().max().item() <= 1e-4
        assert lp[~mask.to(cuda)].abs().max().item() == 0.0
        torch.autograd.backward([lp, ent], [g_lp.to(cuda), g_ent.to(cuda)])
        assert_gradient(hd.grad.cpu().reshape(-1, hdim), ref_gh, bound_h, "grad_hidden")
        assert_gradient(wd.grad.cpu(), ref_gw, bound_w, "grad_weight")
        assert hd.grad[~mask.to(cuda)].abs().max().item() == 0.0

    # labels: -100 gives log-prob 0, anything else outside the vocabulary NaN, neither reads out of bounds
    odd = labels.clone().reshape(-1)
    odd[0], odd[1] = -100, vocab + 5
    lp2, _ = lm_head_logprobs_and_entropy(hidden.to(cuda), wd.detach(), odd.view(b, t).to(cuda), 0.9)
    assert lp2.reshape(-1)[0].item() == 0.0 and torch.isnan(lp2.reshape(-1)[1])
    assert torch.equal(lp2.reshape(-1)[2:], lm_head_logprobs_and_entropy(hidden.to(cuda), wd.detach(), labels.to(cuda), 0.9)[0].reshape(-1)[2:])


def test_lmhead_rejects_what_it_cannot_run(cuda):
    from openrlhf_amd.models.utils import lm_head_logprobs_and_entropy

    h = torch.randn(4, 64, device=cuda)
    w = torch.randn(10, 64, device=cuda)
    with pytest.raises(TypeError):
        lm_head_logprobs_and_entropy(h, w, torch.zeros(4, dtype=torch.long, device=cuda))
    with pytest.raises(ValueError):
        lm_head_logprobs_and_entropy(h.bfloat16(), w.bfloat16()[:, :32], torch.zeros(4, dtype=torch.long, device=cuda))
    with pytest.raises(RuntimeError):
        lm_head_logprobs_and_entropy(h.bfloat16().cpu(), w.bfloat16().cpu(), torch.zeros(4, dtype=torch.long))


def _full_size(cuda, n, hdim, vocab, dtype, temperature, seed, keep_logits_mib=None, std=3.0):
    """One full-depth case (every CU busy, thousands of slabs): every row against closed forms on the
    path's own rounded logits, the gradients entry by entry, a row sample against the CPU oracle."""
    from openrlhf_amd.models.utils import lm_head_logprobs_and_entropy

    g = torch.Generator(device=cuda).manual_seed(seed)
    hidden = torch.randn(n, hdim, generator=g, device=cuda).to(dtype)
    weight = (torch.randn(vocab, hdim, generator=g, device=cuda) * (std / hdim ** 0.5)).to(dtype)
    labels = torch.randint(0, vocab, (n,), generator=g, device=cuda)
    g_lp, g_ent = torch.randn(n, generator=g, device=cuda), torch.randn(n, generator=g, device=cuda)
    g_lp[::17] = 0
    g_ent[::17] = 0
    # tokens whose upstream weights are tiny: their rows of the gradient must be right on their own scale
    g_lp[5::29] *= 1e-4
    g_ent[5::29] *= 1e-4

    lp_k, ent_k, _, kept, _ = forward_keeping_logits(hidden, weight, labels, temperature)
    pick = torch.randperm(n, generator=torch.Generator().manual_seed(1))[:16].to(cuda)
    check_rounded_logits(kept[pick].cpu(), hidden[pick].cpu(), weight.cpu())
    logits = kept[:, :vocab]
    ref_lp, ref_ent, ref_gh, ref_gw, bound_h, bound_w = closed_form_from_logits(logits, hidden, weight, labels, temperature, g_lp, g_ent)
    o_lp = otn.log_probs_from_logits(logits[pick].cpu().double(), labels[pick].cpu(), temperature)
    o_ent = otn.compute_entropy(logits[pick].cpu().double())
    del kept, logits

    hd, wd = hidden.clone().requires_grad_(True), weight.clone().requires_grad_(True)
    lp, ent = lm_head_logprobs_and_entropy(hd, wd, labels, temperature, keep_logits_mib=keep_logits_mib)
    assert torch.equal(lp, lp_k) and torch.equal(ent, ent_k)
    assert (lp - ref_lp).abs().max().item() <= 1e-4 and (ent - ref_ent).abs().max().item() <= 1e-4
    assert (lp[pick].detach().cpu().double() - o_lp).abs().max().item() <= 1e-4
    assert (ent[pick].detach().cpu().double() - o_ent).abs().max().item() <= 1e-4
    torch.autograd.backward([lp, ent], [g_lp, g_ent])
    assert_gradient(hd.grad, ref_gh, bound_h, "grad_hidden")
    assert_gradient(wd.grad, ref_gw, bound_w, "grad_weight")
    assert hd.grad[::17].abs().max().item() == 0.0
    return lp.detach(), ent.detach(), hd.grad, wd.grad


def test_lmhead_full_size(cuda):
    """N = 4096 tokens, H = 4096, V = 151936 bf16 (the vocabulary of the headline metric), T = 1;
    with nothing kept and with every logit kept, which must agree bit for bit."""
    a = _full_size(cuda, 4096, 4096, 151936, torch.bfloat16, 1.0, seed=11)
    b = _full_size(cuda, 4096, 4096, 151936, torch.bfloat16, 1.0, seed=11, keep_logits_mib=2048)
    for x, y in zip(a, b):
        assert torch.equal(x, y)


def test_lmhead_full_size_large_vocabulary_and_temperature(cuda):
    """V = 262144 at T = 0.6 (the vocabulary and temperature of the large-vocabulary configuration):
    1024 vocabulary tiles, the two-temperature kernels forward and backward; half of the logits kept."""
    _full_size(cuda, 4096, 4096, 262144, torch.bfloat16, 0.6, seed=12, keep_logits_mib=1024)


def test_lmhead_full_size_fp16(cuda):
    _full_size(cuda, 4096, 4096, 151936, torch.float16, 1.0, seed=13, std=2.0)


def test_lmhead_repeats_bit_for_bit(cuda):
    """Forward and backward at full size, with every CU busy and the slab loads at their longest
    latencies, give the same bits every time (a slab published before its loads had landed would
    show up as a run that differs): recomputed chunks (five, and one for everything: the deepest
    hidden-state product, 2374 slabs) and kept logits."""
    from openrlhf_amd.models.utils import lm_head_logprobs_and_entropy

    n, hdim, vocab = 4096, 4096, 151936
    g = torch.Generator(device=cuda).manual_seed(23)
    hidden = torch.randn(n, hdim, generator=g, device=cuda).to(torch.bfloat16)
    weight = (torch.randn(vocab, hdim, generator=g, device=cuda) * (3.0 / hdim ** 0.5)).to(torch.bfloat16)
    labels = torch.randint(0, vocab, (n,), generator=g, device=cuda)
    g_lp, g_ent = torch.randn(n, generator=g, device=cuda), torch.randn(n, generator=g, device=cuda)
    first = None
    for temperature, chunk_mib, keep_mib in ((1.0, None, None), (1.0, 2048, None), (1.0, None, 2048), (0.7, None, 600)):
        runs = []
        for _ in range(3):
            hd, wd = hidden.clone().requires_grad_(True), weight.clone().requires_grad_(True)
            lp, ent = lm_head_logprobs_and_entropy(hd, wd, labels, temperature, backward_chunk_mib=chunk_mib, keep_logits_mib=keep_mib)
            torch.autograd.backward([lp, ent], [g_lp, g_ent])
            runs.append((lp.detach(), ent.detach(), hd.grad, wd.grad))
        for other in runs[1:]:
            for a, b in zip(runs[0], other):
                assert torch.equal(a, b)
        if temperature == 1.0:  # and across the memory budgets
            first = first or runs[0]
            for a, b in zip(first, runs[0]):
                assert torch.equal(a, b)


def test_lmhead_every_row_masked(cuda):
    """A row mask that leaves nothing: zeros out, zero gradients, nothing launched on an empty batch."""
    from openrlhf_amd.models.utils import lm_head_logprobs_and_entropy

    h = torch.randn(5, 64, device=cuda).bfloat16().requires_grad_(True)
    w = torch.randn(100, 64, device=cuda).bfloat16().requires_grad_(True)
    labels = torch.randint(0, 100, (5,), device=cuda)
    lp, ent = lm_head_logprobs_and_entropy(h, w, labels, 1.0, row_mask=torch.zeros(5, dtype=torch.bool, device=cuda))
    assert lp.shape == (5,) and lp.abs().max().item() == 0.0 and ent.abs().max().item() == 0.0
    (lp.sum() + ent.sum()).backward()
    assert h.grad.abs().max().item() == 0.0 and w.grad.abs().max().item() == 0.0
    # and an empty batch
    lp0, ent0 = lm_head_logprobs_and_entropy(h[:0], w, labels[:0], 1.0)
    assert lp0.shape == (0,) and ent0.shape == (0,)


def test_lmhead_outputs_at_any_stride_and_alignment_hold_the_same_bits(cuda):
    """The weight gradient leaves its tiles in whole rows with 16-byte stores where the array allows
    it and element by element where it does not (the kept logits must be 16-byte aligned anyway):
    gradient arrays that start 2 bytes past a 16-byte boundary with odd row strides must hold the
    same bits as well-aligned ones, and nothing outside them may be written. Through the C entry
    points, at a shape with ragged tiles in every dimension."""
    from openrlhf_amd import _lib
    from openrlhf_amd._lib import call, ptr, stream_of

    n, hdim, vocab, temperature = 300, 328, 1000, 0.7
    hidden, weight, labels, g_lp, g_ent = _case(n, hdim, vocab, torch.bfloat16, seed=31)
    hd, wd, lab = hidden.to(cuda), weight.to(cuda), labels.to(cuda)
    glp, gent = g_lp.to(cuda), g_ent.to(cuda)
    lib = _lib.load()
    kept_cols = (vocab + 255) // 256 * 256

    def run(kept_ld, offset, pad):
        kept = torch.full((n * kept_ld + 8,), float("nan"), dtype=torch.bfloat16, device=cuda)[:n * kept_ld].view(n, kept_ld)
        lp, ent, stats = torch.empty(n, device=cuda), torch.empty(n, device=cuda), torch.empty(n, 4, device=cuda)
        ws = torch.empty(lib.orlhf_lmhead_workspace_bytes(n, hdim, vocab, kept_cols, 0), dtype=torch.uint8, device=cuda)
        call("orlhf_lmhead_logprob_entropy_fwd", ptr(hd), ptr(wd), _lib.BF16, n, hdim, vocab, hdim, hdim, ptr(lab), temperature,
             ptr(lp), ptr(ent), ptr(stats), ptr(kept), kept_cols, kept_ld, ptr(ws), ws.numel(), stream_of(cuda))
        logits = kept[:, :vocab].clone()
        gh_buf = torch.full((n * (hdim + pad) + offset + 8,), float("nan"), dtype=torch.bfloat16, device=cuda)
        gw_buf = torch.full((vocab * (hdim + pad) + offset + 8,), float("nan"), dtype=torch.bfloat16, device=cuda)
        gh = gh_buf[offset:offset + n * (hdim + pad)].view(n, hdim + pad)[:, :hdim]
        gw = gw_buf[offset:offset + vocab * (hdim + pad)].view(vocab, hdim + pad)[:, :hdim]
        ws2 = torch.empty(lib.orlhf_lmhead_workspace_bytes(n, hdim, vocab, kept_cols, 1), dtype=torch.uint8, device=cuda)
        call("orlhf_lmhead_logprob_entropy_bwd", ptr(hd), ptr(wd), _lib.BF16, n, hdim, vocab, hdim, hdim, ptr(lab), temperature,
             ptr(glp), ptr(gent), ptr(stats), ptr(kept), kept_cols, kept_ld, gh.data_ptr(), hdim + pad, gw.data_ptr(), hdim + pad,
             ptr(ws2), ws2.numel(), stream_of(cuda))
        torch.cuda.synchronize()
        # nothing outside the arrays was touched
        assert torch.isnan(gw_buf[:offset]).all() and torch.isnan(gw_buf[offset + vocab * (hdim + pad):]).all()
        if pad:
            assert torch.isnan(gw_buf[offset:offset + vocab * (hdim + pad)].view(vocab, hdim + pad)[:, hdim:]).all()
        return logits, lp, ent, gh.clone(), gw.clone()

    aligned = run(kept_cols + 64, 0, 0)
    assert torch.isfinite(aligned[3].float()).all() and torch.isfinite(aligned[4].float()).all()
    for kept_ld, offset, pad in ((kept_cols + 8, 1, 3), (kept_cols + 72, 3, 1), (kept_cols + 64, 8, 8), (kept_cols, 4, 0)):
        other = run(kept_ld, offset, pad)
        for a, b in zip(aligned, other):
            assert torch.equal(a.view(torch.int16) if a.dtype == torch.bfloat16 else a, b.view(torch.int16) if b.dtype == torch.bfloat16 else b), (kept_ld, offset, pad)

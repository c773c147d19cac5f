"""lm-head + log-prob / entropy with the logits never stored (openrlhf/models/actor.py:263-285 with
the projection in front): the matrix-core path against the CPU oracle applied to
``hidden.float() @ W.float().T``. Tolerance 2e-3 abs (16-bit inputs, fp32 logits on both sides);
gradients of the hidden states and the weight against torch autograd through the oracle in fp64,
within the rounding of the 16-bit logits gradient and of the 16-bit results."""
import pytest
import torch

from oracle import token_numerics as otn

pytestmark = pytest.mark.gpu


def _case(n, hdim, vocab, dtype, seed, std=3.0):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(n, hdim, generator=g).to(dtype)
    weight = (torch.randn(vocab, hdim, generator=g) * (std / hdim ** 0.5)).to(dtype)
    labels = torch.randint(0, vocab, (n,), generator=g)
    g_lp, g_ent = torch.randn(n, generator=g), torch.randn(n, generator=g)
    return hidden, weight, labels, g_lp, g_ent


def _oracle(hidden, weight, labels, temperature, g_lp, g_ent):
    h64 = hidden.double().requires_grad_(True)
    w64 = weight.double().requires_grad_(True)
    logits = h64 @ w64.T
    lp = otn.log_probs_from_logits(logits, labels, temperature)
    ent = otn.compute_entropy(logits)
    torch.autograd.backward([lp, ent], [g_lp.double(), g_ent.double()])
    return lp.detach(), ent.detach(), h64.grad, w64.grad


def _grad_close(got, ref, dtype):
    """16-bit P (2^-9 relative per element, summed over the contraction) and a 16-bit result."""
    eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    err = (got.double().cpu() - ref).abs()
    scale = ref.abs().max().item()
    assert err.max().item() <= 4 * eps * scale + 1e-9, (err.max().item(), scale)
    rel_fro = (err.pow(2).sum() / ref.pow(2).sum().clamp_min(1e-300)).sqrt().item()
    assert rel_fro <= 2 * eps, rel_fro


@pytest.mark.parametrize(
    "n,hdim,vocab,dtype,temperature",
    [
        (256, 64, 256, torch.bfloat16, 1.0),      # exactly one tile, one slab
        (300, 128, 1000, torch.bfloat16, 1.0),    # ragged tokens and vocabulary
        (513, 200, 5003, torch.bfloat16, 0.7),    # hidden size not a multiple of the slab, odd vocabulary, T != 1
        (70, 4100, 777, torch.float16, 1.3),      # long ragged contraction, fp16
        (1, 64, 50, torch.bfloat16, 1.0),         # a single token, tiny vocabulary
        (1500, 512, 20000, torch.bfloat16, 0.6),  # several token blocks and vocabulary ranges
    ],
)
def test_lmhead_matches_oracle(cuda, n, hdim, vocab, dtype, temperature):
    from openrlhf_amd.models.utils import lm_head_logprobs_and_entropy

    hidden, weight, labels, g_lp, g_ent = _case(n, hdim, vocab, dtype, seed=n + hdim + vocab)
    ref_lp, ref_ent, ref_gh, ref_gw = _oracle(hidden, weight, labels, temperature, g_lp, g_ent)
    hd = hidden.to(cuda).requires_grad_(True)
    wd = weight.to(cuda).requires_grad_(True)
    lp, ent = lm_head_logprobs_and_entropy(hd, wd, labels.to(cuda), temperature)
    assert lp.dtype == torch.float32 and lp.shape == (n,)
    assert (lp.cpu().double() - ref_lp).abs().max().item() <= 2e-3
    assert (ent.cpu().double() - ref_ent).abs().max().item() <= 2e-3
    torch.autograd.backward([lp, ent], [g_lp.to(cuda), g_ent.to(cuda)])
    assert hd.grad.dtype == dtype and wd.grad.dtype == dtype
    _grad_close(hd.grad, ref_gh, dtype)
    _grad_close(wd.grad, ref_gw, dtype)


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

    h64 = hidden.double().requires_grad_(True)
    w64 = weight.double().requires_grad_(True)
    logits = h64 @ w64.T
    ref_lp = otn.log_probs_from_logits(logits, labels, 0.9) * mask
    ref_ent = otn.compute_entropy(logits) * mask
    torch.autograd.backward([ref_lp, ref_ent], [g_lp.double(), g_ent.double()])

    hd = hidden.to(cuda).requires_grad_(True)
    wd_big = wbig.to(cuda)
    wd = wd_big[:, :hdim].requires_grad_(True)
    lp, ent = lm_head_logprobs_and_entropy(hd, wd, labels.to(cuda), 0.9, row_mask=mask.to(cuda))
    assert lp.shape == (b, t)
    assert (lp.cpu().double() - ref_lp.detach()).abs().max().item() <= 2e-3
    assert (ent.cpu().double() - ref_ent.detach()).abs().max().item() <= 2e-3
    assert lp[~mask.to(cuda)].abs().max().item() == 0.0
    torch.autograd.backward([lp, ent], [g_lp.to(cuda), g_ent.to(cuda)])
    _grad_close(hd.grad, h64.grad, torch.bfloat16)
    _grad_close(wd.grad, w64.grad, torch.bfloat16)
    assert hd.grad[~mask.to(cuda)].abs().max().item() == 0.0

    # labels: -100 gives log-prob 0, anything else outside the vocabulary NaN, neither reads out of bounds
    odd = labels.clone().reshape(-1)
    odd[0], odd[1] = -100, vocab + 5
    lp2, _ = lm_head_logprobs_and_entropy(hidden.to(cuda), wd.detach(), odd.view(b, t).to(cuda), 0.9)
    assert lp2.reshape(-1)[0].item() == 0.0 and torch.isnan(lp2.reshape(-1)[1])
    assert torch.equal(lp2.reshape(-1)[2:], lm_head_logprobs_and_entropy(hidden.to(cuda), wd.detach(), labels.to(cuda), 0.9)[0].reshape(-1)[2:])


@pytest.mark.parametrize("chunk_mib", [1, 3, 4096])
def test_lmhead_backward_chunk_sizes(cuda, chunk_mib):
    """The backward holds as much of the logits gradient at a time as its workspace offers: many
    small chunks, a last chunk that is not a whole tile column, one chunk for everything. The
    weight gradient does not depend on the cut (each entry is summed over tokens only); the hidden
    states' gradient is summed over the vocabulary chunk by chunk in fp32."""
    from openrlhf_amd.models.utils import lm_head_logprobs_and_entropy

    n, hdim, vocab, temperature = 1500, 256, 20011, 0.8
    hidden, weight, labels, g_lp, g_ent = _case(n, hdim, vocab, torch.bfloat16, seed=77)
    _, _, ref_gh, ref_gw = _oracle(hidden, weight, labels, temperature, g_lp, g_ent)
    grads = []
    for mib in (None, chunk_mib):
        hd = hidden.to(cuda).requires_grad_(True)
        wd = weight.to(cuda).requires_grad_(True)
        lp, ent = lm_head_logprobs_and_entropy(hd, wd, labels.to(cuda), temperature, backward_chunk_mib=mib)
        torch.autograd.backward([lp, ent], [g_lp.to(cuda), g_ent.to(cuda)])
        grads.append((hd.grad, wd.grad))
    _grad_close(grads[1][0], ref_gh, torch.bfloat16)
    _grad_close(grads[1][1], ref_gw, torch.bfloat16)
    assert torch.equal(grads[0][1], grads[1][1])
    assert (grads[0][0].float() - grads[1][0].float()).abs().max().item() <= 2.0 ** -7 * ref_gh.abs().max().item()


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


def test_lmhead_full_size(cuda):
    """N = 4096 tokens, H = 4096, V = 151936 bf16 (the vocabulary of the headline metric): every row
    against the vocabulary-row kernels applied to the fp32 projection (2.5 GB of logits the fused
    path never stores), gradients against fp32 products of that path's logits gradient, and a row
    sample against the CPU oracle."""
    from openrlhf_amd.models.utils import lm_head_logprobs_and_entropy, logprobs_and_entropy_from_logits

    n, hdim, vocab, temperature = 4096, 4096, 151936, 1.0
    g = torch.Generator(device=cuda).manual_seed(11)
    hidden = torch.randn(n, hdim, generator=g, device=cuda).to(torch.bfloat16)
    weight = (torch.randn(vocab, hdim, generator=g, device=cuda) * (3.0 / hdim ** 0.5)).to(torch.bfloat16)
    labels = torch.randint(0, vocab, (n,), generator=g, device=cuda)
    g_lp, g_ent = torch.randn(n, generator=g, device=cuda), torch.randn(n, generator=g, device=cuda)
    g_lp[::17] = 0
    g_ent[::17] = 0

    hd, wd = hidden.clone().requires_grad_(True), weight.clone().requires_grad_(True)
    lp, ent = lm_head_logprobs_and_entropy(hd, wd, labels, temperature)
    torch.autograd.backward([lp, ent], [g_lp, g_ent])

    logits = (hidden.float() @ weight.float().T).requires_grad_(True)
    lp2, ent2 = logprobs_and_entropy_from_logits(logits, labels, temperature)
    assert (lp - lp2).abs().max().item() <= 1e-3 and (ent - ent2).abs().max().item() <= 1e-3
    (p_ref,) = torch.autograd.grad([lp2, ent2], [logits], [g_lp, g_ent])
    gh_ref = p_ref @ weight.float()
    gw_ref = p_ref.T @ hidden.float()
    for got, ref in ((hd.grad, gh_ref), (wd.grad, gw_ref)):
        err = (got.float() - ref).abs()
        scale = ref.abs().max().item()
        assert err.max().item() <= 4 * 2.0 ** -8 * scale, (err.max().item(), scale)
        assert (err.pow(2).sum() / ref.pow(2).sum()).sqrt().item() <= 2.0 ** -7
    assert hd.grad[::17].abs().max().item() == 0.0

    pick = torch.randperm(n, generator=torch.Generator().manual_seed(1))[:24]
    x64 = hidden[pick.to(cuda)].cpu().float() @ weight.cpu().float().T
    ref_lp = otn.log_probs_from_logits(x64.double(), labels[pick.to(cuda)].cpu(), temperature)
    ref_ent = otn.compute_entropy(x64.double())
    assert (lp[pick.to(cuda)].detach().cpu().double() - ref_lp).abs().max().item() <= 2e-3
    assert (ent[pick.to(cuda)].detach().cpu().double() - ref_ent).abs().max().item() <= 2e-3


def test_lmhead_backward_repeats_bit_for_bit(cuda):
    """The three products of the backward at full size, with every CU busy and the slab loads at
    their longest latencies, give the same bits every time (a slab published before its loads had
    landed would show up as a run that differs), and so does a product deep enough for 2374 slabs."""
    from openrlhf_amd.models.utils import lm_head_logprobs_and_entropy

    n, hdim, vocab = 4096, 4096, 151936
    g = torch.Generator(device=cuda).manual_seed(23)
    hidden = torch.randn(n, hdim, generator=g, device=cuda).to(torch.bfloat16)
    weight = (torch.randn(vocab, hdim, generator=g, device=cuda) * (3.0 / hdim ** 0.5)).to(torch.bfloat16)
    labels = torch.randint(0, vocab, (n,), generator=g, device=cuda)
    g_lp, g_ent = torch.randn(n, generator=g, device=cuda), torch.randn(n, generator=g, device=cuda)
    for chunk_mib in (None, 2048):  # five chunks of the logits gradient; one chunk (the deepest dHidden product)
        runs = []
        for _ in range(3):
            hd, wd = hidden.clone().requires_grad_(True), weight.clone().requires_grad_(True)
            lp, ent = lm_head_logprobs_and_entropy(hd, wd, labels, 1.0, backward_chunk_mib=chunk_mib)
            torch.autograd.backward([lp, ent], [g_lp, g_ent])
            runs.append((lp.detach(), ent.detach(), hd.grad, wd.grad))
        for other in runs[1:]:
            for a, b in zip(runs[0], other):
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


@pytest.mark.parametrize("m,n,k", [(256, 256, 64), (300, 515, 204), (1000, 259, 4102), (64, 700, 130)])
def test_matrix_tile_probe_sums(cuda, m, n, k):
    """The measurement entry computes the product it times: the 256 thread sums of every tile add up
    to the sum of that 256 x 256 block of a @ b.T (fp32 reference on the same bf16 operands)."""
    from openrlhf_amd import _lib
    from openrlhf_amd._lib import call, ptr, stream_of

    g = torch.Generator().manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16).to(cuda)
    b = torch.randn(n, k, generator=g).to(torch.bfloat16).to(cuda)
    tm, tn = (m + 255) // 256, (n + 255) // 256
    sums = torch.full((tm * tn * 256,), float("nan"), device=cuda)
    call("orlhf_matrix_tile_probe", ptr(a), ptr(b), _lib.BF16, m, n, k, k, k, 0, ptr(sums), stream_of(cuda))
    c = a.float() @ b.float().T
    scale = c.abs().sum().item() / (tm * tn)
    for i in range(tm):
        for j in range(tn):
            want = c[i * 256:(i + 1) * 256, j * 256:(j + 1) * 256].double().sum().item()
            got = sums[(i * tn + j) * 256:(i * tn + j + 1) * 256].double().sum().item()
            assert abs(got - want) <= 1e-5 * scale + 1e-3, (i, j, got, want)
    with pytest.raises(_lib.KernelError):
        call("orlhf_matrix_tile_probe", ptr(a), ptr(b), _lib.F32, m, n, k, k, k, 0, ptr(sums), stream_of(cuda))

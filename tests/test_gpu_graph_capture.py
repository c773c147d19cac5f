"""The entry points under HIP graph capture: the launches record into a captured graph (nothing in
the C ABI allocates, synchronises or touches another stream) and every replay reproduces the
eager result on the inputs then present in the static buffers. Replays are interleaved with
eager work and synchronisations, and each one is checked."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _capture(fn, warmup=2):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(warmup):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = fn()
    return graph, out


def test_experience_chain_replays(cuda):
    from openrlhf_amd.models.loss import PolicyLoss, ValueLoss
    from openrlhf_amd.models.utils import compute_approx_kl, compute_reward
    from openrlhf_amd.trainer.ppo_utils.experience_maker import get_advantages_and_returns, whiten_advantages

    g = torch.Generator().manual_seed(0)
    b, a = 16, 900
    mask = (torch.arange(a)[None, :] < torch.randint(1, a + 1, (b,), generator=g)[:, None]).to(cuda)
    lp = (-torch.rand(b, a, generator=g) * 2).to(cuda)
    old, base, values = (torch.empty(b, a, device=cuda) for _ in range(3))
    r = torch.empty(b, device=cuda)
    pol, val = PolicyLoss(0.2, 0.2), ValueLoss(0.2)

    def fill(seed):
        gg = torch.Generator().manual_seed(seed)
        old.copy_(lp + (torch.randn(b, a, generator=gg) * 0.05).to(cuda))
        base.copy_(lp + (torch.randn(b, a, generator=gg) * 0.1).to(cuda))
        values.copy_(torch.randn(b, a, generator=gg).to(cuda))
        r.copy_(torch.randn(b, generator=gg).to(cuda))

    def chain():
        kl = compute_approx_kl(old, base, kl_estimator="k3")
        rew = compute_reward(r, 0.05, kl, action_mask=mask, reward_clip_range=(-5.0, 5.0))
        adv, ret = get_advantages_and_returns(values, rew, mask, 1.0, 0.95)
        (adv_w,) = whiten_advantages([adv], [mask])
        return pol(lp, old, adv_w, action_mask=mask)[0], val(values + 0.1, values, ret, action_mask=mask), adv_w

    fill(1)
    graph, outs = _capture(chain)
    for seed in (2, 3, 4):
        fill(seed)
        eager = [t.clone() for t in chain()]
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(outs, eager):
            assert torch.equal(got, want), seed


def test_policy_loss_forward_backward_replays(cuda):
    from openrlhf_amd.models.loss import PolicyLoss

    g = torch.Generator().manual_seed(1)
    b, a = 8, 3000
    mask = (torch.arange(a)[None, :] < torch.randint(1, a + 1, (b,), generator=g)[:, None]).to(cuda)
    x = torch.zeros(b, a, device=cuda, requires_grad=True)
    old, adv = torch.empty(b, a, device=cuda), torch.empty(b, a, device=cuda)
    pol = PolicyLoss(0.2, 0.28, dual_clip=3.0, token_level_loss=False)

    def fill(seed):
        gg = torch.Generator().manual_seed(seed)
        with torch.no_grad():
            x.copy_((-torch.rand(b, a, generator=gg) * 2).to(cuda))
        old.copy_(x.detach() + (torch.randn(b, a, generator=gg) * 0.2).to(cuda))
        adv.copy_(torch.randn(b, a, generator=gg).to(cuda))

    def step():
        loss = pol(x, old, adv, action_mask=mask)[0]
        (gx,) = torch.autograd.grad(loss, x)
        return loss, gx

    fill(1)
    graph, outs = _capture(step)
    for seed in (5, 6, 7):
        fill(seed)
        eager = [t.clone() for t in step()]
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(outs, eager):
            assert torch.equal(got, want), seed


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_logprob_entropy_kernels_replay(cuda, dtype):
    """The two-kernel forward / backward and the one-pass kernel, each in its own graph."""
    from openrlhf_amd.models.utils import fused_logprob_entropy_fwd_bwd, logprobs_and_entropy_from_logits

    n, vocab = 96, 32003
    static = torch.empty(n, vocab, device=cuda, dtype=dtype)
    labels = torch.randint(0, vocab, (n,), device=cuda)
    w_lp, w_ent = torch.randn(n, device=cuda), torch.randn(n, device=cuda)

    def fill(seed):
        gg = torch.Generator().manual_seed(seed)
        static.copy_((torch.randn(n, vocab, generator=gg) * 2).to(dtype).to(cuda))

    def forward():
        with torch.no_grad():
            return logprobs_and_entropy_from_logits(static, labels, 0.7)

    def one_pass():
        return fused_logprob_entropy_fwd_bwd(static, labels, w_lp, w_ent, temperature=0.7, inplace=False)

    fill(1)
    g_fwd, out_fwd = _capture(forward)
    g_one, out_one = _capture(one_pass)
    for seed in (8, 9):
        fill(seed)
        eager_fwd = [t.clone() for t in forward()]
        eager_one = [t.clone() for t in one_pass()]
        torch.cuda.synchronize()
        g_fwd.replay()
        g_one.replay()
        torch.cuda.synchronize()
        for got, want in zip(out_fwd, eager_fwd):
            assert torch.equal(got, want)
        for got, want in zip(out_one, eager_one):
            assert torch.equal(got, want)


def test_launches_follow_the_current_stream(cuda):
    """Work queued on a side stream is ordered with the producer of its inputs on that stream
    (the entry points take the caller's stream, not the default one)."""
    from openrlhf_amd.models.loss import PolicyLoss
    from openrlhf_amd.models.utils import logprobs_and_entropy_from_logits

    side = torch.cuda.Stream()
    n, v = 512, 32000
    labels = torch.randint(0, v, (n,), device=cuda)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        big = torch.randn(n, v, device=cuda)          # produced on the side stream ...
        for _ in range(20):
            big = big * 1.0001 + 0.0001               # ... by a chain of kernels that takes a while
        lp, ent = logprobs_and_entropy_from_logits(big, labels)   # consumed on the same stream, no sync between
        loss = PolicyLoss()(lp, lp.detach() + 0.01, ent, action_mask=None)[0]
    side.synchronize()
    ref = torch.log_softmax(big.double(), -1).gather(1, labels[:, None]).squeeze(1)
    assert (lp.double() - ref).abs().max().item() <= 1e-5
    assert torch.isfinite(loss)


def test_lmhead_forward_backward_replays(cuda):
    """The lm-head path (matrix-core tiles, chunked backward with its workspace) in one graph:
    every replay equals the eager run on the operands then in the static buffers."""
    from openrlhf_amd.models.utils import lm_head_logprobs_and_entropy

    n, hdim, vocab = 300, 192, 5003
    hidden = torch.empty(n, hdim, device=cuda, dtype=torch.bfloat16, requires_grad=True)
    weight = torch.empty(vocab, hdim, device=cuda, dtype=torch.bfloat16, requires_grad=True)
    labels = torch.randint(0, vocab, (n,), device=cuda)
    g_lp, g_ent = torch.randn(n, device=cuda), torch.randn(n, device=cuda)

    def fill(seed):
        gg = torch.Generator().manual_seed(seed)
        with torch.no_grad():
            hidden.copy_(torch.randn(n, hdim, generator=gg).to(torch.bfloat16).to(cuda))
            weight.copy_((torch.randn(vocab, hdim, generator=gg) * 0.2).to(torch.bfloat16).to(cuda))

    def step():
        lp, ent = lm_head_logprobs_and_entropy(hidden, weight, labels, 0.9)
        gh, gw = torch.autograd.grad([lp, ent], [hidden, weight], [g_lp, g_ent])
        return lp.detach(), ent.detach(), gh, gw

    fill(1)
    graph, out = _capture(step)
    for seed in (5, 6, 7):
        fill(seed)
        eager = [t.clone() for t in step()]
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(out, eager):
            assert torch.equal(got, want)

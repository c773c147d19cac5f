"""The PPO actor loss step (openrlhf/trainer/ray/ppo_actor.py:294-352): the composed mirror and the
one-pass fused step against the oracle's composition of the same lines, values and d/d(logits)."""
import pytest
import torch

from oracle import losses as ol
from oracle import token_numerics as otn

pytestmark = pytest.mark.gpu


def _batch(seed, b=6, t=48, vocab=5003, a=20):
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(a + 4, t + 1, (b,), generator=g)
    lens[0] = t
    attn = (torch.arange(t)[None, :] < lens[:, None]).long()
    seqs = torch.randint(1, vocab, (b, t), generator=g) * attn
    amask = attn[:, 1:][:, -a:].bool().clone()
    amask[:, :3] = False
    amask[2, 9:11] = False
    logits = torch.randn(b, t, vocab, generator=g) * 2
    old = -torch.rand(b, a, generator=g) * 12
    adv = torch.randn(b, a, generator=g)
    base = -torch.rand(b, a, generator=g) * 12
    roll = old + torch.randn(b, a, generator=g) * 0.1
    return logits, seqs, attn, amask, old, adv, base, roll


def _oracle_step(logits64, seqs, attn, amask, old, adv, base, roll, temperature, packed, pol_cfg, kl_est, kl_coef,
                 ent_coef, info):
    batch, seqlen = seqs.shape
    rolled = torch.roll(seqs, -1, 1)
    if packed:
        keep = attn.reshape(-1).bool().nonzero().squeeze(-1)
        labels = rolled.reshape(-1)[keep].unsqueeze(0)
    else:
        labels = rolled
    ent = otn.compute_entropy(logits64)
    lp = otn.log_probs_from_logits(logits64, labels, temperature)
    if packed:
        def repad(flat):
            return torch.zeros(batch * seqlen, dtype=flat.dtype).index_copy(0, keep, flat.reshape(-1)).view(batch, seqlen)
        ent, lp = repad(ent), repad(lp)
    a = amask.shape[1]
    alp = lp[:, :-1][:, -a:] * amask.double()
    ent = ent[:, :-1][:, -a:]
    m = amask.double()
    pl = ol.policy_loss(alp, old.double(), adv.double(), m, roll.double() if pol_cfg.get("enable_vllm_is_correction") else None,
                        **pol_cfg, **info)
    loss = pl[0]
    out = dict(actor_loss=pl[0], clip_ratio=pl[1], ppo_kl=pl[2], vllm_kl=pl[3], kl_loss=None, entropy_loss=None,
               logprobs_diff=None)
    if base is not None:
        out["kl_loss"] = ol.aggregate_loss(otn.compute_approx_kl(alp, base.double(), kl_est), m, **info)
        # the step's "logprobs_diff" status (openrlhf/trainer/ray/ppo_actor.py:327-333)
        out["logprobs_diff"] = otn.masked_mean(alp.detach() - base.double(), m)
        loss = loss + out["kl_loss"] * kl_coef
    if ent_coef is not None:
        out["entropy_loss"] = ol.aggregate_loss(ent, m, **info)
        loss = loss - out["entropy_loss"] * ent_coef
    out["loss"] = loss
    out["action_log_probs"] = alp
    return out


CASES = [
    dict(pol=dict(), kl=None, ent=None, info={}),
    dict(pol=dict(dual_clip=3.0, clip_eps_low=0.1, clip_eps_high=0.3), kl=("k3", 0.05), ent=0.01, info={}),
    dict(pol=dict(token_level_loss=False), kl=("k2", 0.1), ent=0.0,
         info=dict(dp_size=2, batch_num_tokens=300.0, global_batch_size=9.0)),
    dict(pol=dict(enable_vllm_is_correction=True, vllm_is_truncated_threshold=[0.9, 1.1], vllm_is_correction_type="tis"),
         kl=("k1", 0.02), ent=0.005, info={}),
    dict(pol=dict(enable_vllm_is_correction=True, vllm_is_truncated_threshold=[0.95, 1.05], vllm_is_correction_type="icepop"),
         kl=None, ent=None, info={}),
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("dtype,packed", [(torch.float32, False), (torch.bfloat16, True), (torch.bfloat16, False)])
@pytest.mark.parametrize("fused", [True, False])
def test_actor_step_matches_oracle(cuda, case, dtype, packed, fused):
    from openrlhf_amd.models.actor import unpad_indices
    from openrlhf_amd.models.loss import PolicyLoss
    from openrlhf_amd.trainer.ray.ppo_actor import actor_loss_step, fused_actor_loss_step

    logits, seqs, attn, amask, old, adv, base, roll = _batch(11)
    logits = logits.to(dtype)
    temperature = 1.0 if dtype == torch.bfloat16 else 0.9
    kl_est, kl_coef = case["kl"] if case["kl"] else ("k1", 0.0)
    use_base = base if case["kl"] else None
    scale = 0.25  # what a 4-step gradient accumulation multiplies the loss with

    ref_x = logits.double().requires_grad_(True)
    keep = attn.reshape(-1).bool()
    ref_in = ref_x.reshape(-1, ref_x.shape[-1])[keep].unsqueeze(0) if packed else ref_x
    ref = _oracle_step(ref_in, seqs, attn, amask, old, adv, use_base, roll, temperature, packed, case["pol"], kl_est,
                       kl_coef, case["ent"], case["info"])
    (ref["loss"] * scale).backward()
    ref_grad = ref_x.grad
    if packed:
        ref_grad = ref_grad.reshape(-1, ref_grad.shape[-1])[keep]

    d = cuda
    xd = logits.to(d)
    if packed:
        xd = xd.reshape(-1, xd.shape[-1])[keep.to(d)].contiguous()
    xd.requires_grad_(True)
    kw = dict(base_action_log_probs=None if use_base is None else use_base.to(d), kl_estimator=kl_est, kl_coef=kl_coef,
              entropy_coef=case["ent"], rollout_log_probs=roll.to(d), temperature=temperature,
              packed_indices=unpad_indices(attn.to(d)) if packed else None, **case["info"])
    fn = PolicyLoss(**case["pol"])
    args = (xd, seqs.to(d), attn.to(d), amask.to(d), old.to(d), adv.to(d), fn)
    if fused:
        out = fused_actor_loss_step(*args, loss_scale=scale, **kw)
        assert out["grad_logits"].data_ptr() == xd.data_ptr()
        (out["loss"] * scale).backward()
    else:
        out = actor_loss_step(*args, **kw)
        (out["loss"] * scale).backward()
    atol = 1e-5 if dtype == torch.float32 else 2e-3
    for key in ("loss", "actor_loss", "clip_ratio", "ppo_kl", "vllm_kl", "kl_loss", "entropy_loss", "logprobs_diff"):
        if ref[key] is None:
            assert out[key] is None, key
        else:
            want = ref[key].item()
            assert abs(out[key].item() - want) <= atol * max(1.0, abs(want)), (key, out[key].item(), want)
    assert (out["action_log_probs"].cpu().double() - ref["action_log_probs"].detach()).abs().max().item() <= atol
    grad = xd.grad.cpu().double()
    err = (grad - ref_grad).abs()
    gscale = ref_grad.abs().max().item()
    if dtype == torch.float32:
        assert err.max().item() <= 1e-5 * max(gscale, 1e-30) + 1e-12, (err.max().item(), gscale)
    else:
        assert (err <= 2.0 ** -7 * ref_grad.abs() + 2e-3 * gscale).all(), (err.max().item(), gscale)


def test_fused_step_rescales_when_upstream_differs(cuda):
    """The gradient is produced with loss_scale; a different upstream gradient is honoured."""
    from openrlhf_amd.models.loss import PolicyLoss
    from openrlhf_amd.trainer.ray.ppo_actor import fused_actor_loss_step

    logits, seqs, attn, amask, old, adv, base, roll = _batch(12, b=3, t=20, vocab=300, a=8)
    d = cuda
    grads = []
    for upstream in (1.0, 0.5):
        xd = logits.to(d).requires_grad_(True)
        out = fused_actor_loss_step(xd, seqs.to(d), attn.to(d), amask.to(d), old.to(d), adv.to(d), PolicyLoss(),
                                    loss_scale=1.0)
        (out["loss"] * upstream).backward()
        grads.append(xd.grad.clone())
    assert torch.allclose(grads[1], grads[0] * 0.5, rtol=1e-6, atol=0)
    # the stored gradient is handed over once: a second backward through the node must not rescale it again
    xd = logits.to(d).requires_grad_(True)
    out = fused_actor_loss_step(xd, seqs.to(d), attn.to(d), amask.to(d), old.to(d), adv.to(d), PolicyLoss())
    (out["loss"] * 0.5).backward(retain_graph=True)
    with pytest.raises(RuntimeError, match="once"):
        (out["loss"] * 0.5).backward()
    with pytest.raises(ValueError):
        fused_actor_loss_step(logits.to(d), seqs.to(d), attn.to(d), amask.to(d), old.to(d), adv.to(d),
                              PolicyLoss(policy_loss_type="gspo"))


def test_fused_step_on_a_vocabulary_longer_than_the_registers(cuda):
    """V = 262144 (half of every row streamed): the one-pass step against the composed one."""
    from openrlhf_amd.models.loss import PolicyLoss
    from openrlhf_amd.trainer.ray.ppo_actor import actor_loss_step, fused_actor_loss_step

    logits, seqs, attn, amask, old, adv, base, roll = _batch(13, b=3, t=16, vocab=262144, a=11)
    logits = logits.to(torch.bfloat16)
    d = cuda
    kw = dict(base_action_log_probs=base.to(d), kl_estimator="k3", kl_coef=0.05, entropy_coef=0.01, temperature=0.6)
    fn = PolicyLoss(0.2, 0.28, dual_clip=3.0)
    tensors = (seqs.to(d), attn.to(d), amask.to(d), old.to(d), adv.to(d), fn)
    xa = logits.to(d).requires_grad_(True)
    ref = actor_loss_step(xa, *tensors, **kw)
    ref["loss"].backward()
    xb = logits.to(d).requires_grad_(True)
    out = fused_actor_loss_step(xb, *tensors, **kw)
    out["loss"].backward()
    for key in ("loss", "actor_loss", "kl_loss", "entropy_loss", "clip_ratio", "ppo_kl"):
        assert abs(out[key].item() - ref[key].item()) <= 2e-5 * max(1.0, abs(ref[key].item())), key
    ga, gb = xa.grad.float(), xb.grad.float()
    assert (ga - gb).abs().max().item() <= 2.0 ** -7 * ga.abs().max().item()


@pytest.mark.parametrize("case", [CASES[1], CASES[2]])
@pytest.mark.parametrize("packed", [False, True])
def test_actor_step_from_hidden_states(cuda, case, packed):
    """The composed step with the lm-head projection fused in (hidden states and lm_head.weight in
    place of logits): the oracle's step on ``hidden @ W.T`` rounded to bf16 as the lm_head output is
    (tests/lmhead_util.py), in fp64; values within 2e-3, gradients of the hidden states and the
    weight within the rounding of a bf16 logits gradient."""
    from tests.lmhead_util import straight_through_logits

    from openrlhf_amd.models.actor import unpad_indices
    from openrlhf_amd.models.loss import PolicyLoss
    from openrlhf_amd.trainer.ray.ppo_actor import actor_loss_step

    b, t, a, hdim, vocab = 6, 48, 20, 128, 1500
    _, seqs, attn, amask, old, adv, base, roll = _batch(13, b=b, t=t, vocab=vocab, a=a)
    g = torch.Generator().manual_seed(14)
    hidden = torch.randn(b, t, hdim, generator=g).to(torch.bfloat16)
    weight = (torch.randn(vocab, hdim, generator=g) * 0.25).to(torch.bfloat16)
    kl_est, kl_coef = case["kl"]
    keep = attn.reshape(-1).bool()

    h64 = hidden.double().requires_grad_(True)
    w64 = weight.double().requires_grad_(True)
    logits64 = straight_through_logits(hidden, weight, h64, w64, cuda)
    ref_in = logits64.reshape(-1, vocab)[keep].unsqueeze(0) if packed else logits64
    ref = _oracle_step(ref_in, seqs, attn, amask, old, adv, base, roll, 1.0, packed, case["pol"], kl_est, kl_coef,
                       case["ent"], case["info"])
    ref["loss"].backward()

    d = cuda
    hd = hidden.to(d)
    if packed:
        hd = hd.reshape(-1, hdim)[keep.to(d)].contiguous()
    hd.requires_grad_(True)
    wd = weight.to(d).requires_grad_(True)
    out = actor_loss_step(hd, seqs.to(d), attn.to(d), amask.to(d), old.to(d), adv.to(d), PolicyLoss(**case["pol"]),
                          base_action_log_probs=base.to(d), kl_estimator=kl_est, kl_coef=kl_coef, entropy_coef=case["ent"],
                          rollout_log_probs=roll.to(d), temperature=1.0,
                          packed_indices=unpad_indices(attn.to(d)) if packed else None, lm_head_weight=wd, **case["info"])
    out["loss"].backward()
    for key in ("loss", "actor_loss", "clip_ratio", "ppo_kl", "kl_loss", "entropy_loss", "logprobs_diff"):
        want = ref[key].item()
        assert abs(out[key].item() - want) <= 2e-3 * max(1.0, abs(want)), (key, out[key].item(), want)
    ref_gh = h64.grad.reshape(-1, hdim)[keep] if packed else h64.grad
    for got, want in ((hd.grad, ref_gh), (wd.grad, w64.grad)):
        err = (got.cpu().double() - want).abs()
        scale = want.abs().max().item()
        assert err.max().item() <= 6 * 2.0 ** -8 * scale + 1e-9, (err.max().item(), scale)

"""Shared pieces of the lm-head tests (not a test module).

The lm-head path rounds its logits to the 16-bit dtype before anything else, as the reference's
lm_head output is rounded before ``.to(torch.float32)`` (openrlhf/models/actor.py:263-267). Which
way a logit that sits within an fp32 rounding error of a 16-bit rounding boundary goes depends on
the order of the fp32 accumulation, which no two matrix-multiply kernels share. The tests
therefore pin the path in two steps:

  1. the rounded logits themselves (the C entry point stores them when asked to keep every
     column) against the fp64 product: off by at most half a 16-bit ulp plus the fp32
     accumulation error;
  2. everything downstream (log-probs, entropies, both gradients) against the oracle applied to
     exactly those rounded logits, where the tolerances are the tight ones.
"""
import torch

from openrlhf_amd import _lib
from openrlhf_amd._lib import call, ptr, stream_of


def unit_roundoff(dtype):
    """Largest relative error of rounding to `dtype` (8 significant bits for bf16, 11 for fp16)."""
    return 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11


def forward_keeping_logits(hidden, weight, labels, temperature, kept_cols=None):
    """The C forward with the logits kept: (logprob, entropy, row_stats, kept [n, ld], kept_cols)."""
    dev = hidden.device
    n, hdim = hidden.shape
    vocab = weight.shape[0]
    vpad = (vocab + 255) // 256 * 256
    kept_cols = vpad if kept_cols is None else kept_cols
    ld = kept_cols + 64
    kept = torch.full((n, ld), float("nan"), dtype=hidden.dtype, device=dev) if kept_cols > 0 else None
    lp, ent = torch.empty(n, device=dev), torch.empty(n, device=dev)
    stats = torch.empty(n, 4, device=dev)
    lib = _lib.load()
    ws = torch.empty(lib.orlhf_lmhead_workspace_bytes(n, hdim, vocab, kept_cols, 0), dtype=torch.uint8, device=dev)
    call("orlhf_lmhead_logprob_entropy_fwd", ptr(hidden), ptr(weight), _lib.dtype_code(hidden), n, hdim, vocab,
         hidden.stride(0), weight.stride(0), ptr(labels), float(temperature), ptr(lp), ptr(ent), ptr(stats), ptr(kept),
         kept_cols, ld if kept_cols > 0 else 0, ptr(ws), ws.numel(), stream_of(dev))
    return lp, ent, stats, kept, kept_cols


def check_rounded_logits(kept, hidden, weight, rows=None):
    """Step 1: kept[:, :V] is the product rounded to the 16-bit dtype (fp64 reference on `rows`)."""
    vocab = weight.shape[0]
    sel = slice(None) if rows is None else rows
    x = hidden[sel].double() @ weight.double().T
    got = kept[sel][:, :vocab].double()
    u = unit_roundoff(kept.dtype)
    # half an ulp is at most u/2 * 2|x| relative to the binade's lower end (for fp16 never less than half
    # the spacing of its subnormals, 2^-25); the fp32 accumulation adds ~1e-6 * |h||w|
    floor = 2.0 ** -25 if kept.dtype == torch.float16 else 0.0
    slack = 2e-6 * (hidden[sel].double().abs() @ weight.double().abs().T) + floor
    excess = ((got - x).abs() - (u * x.abs() + slack)).max().item()
    assert excess <= 0, excess
    return x


def straight_through_logits(hidden, weight, h64, w64, device):
    """``h64 @ w64.T`` with the VALUES of the path's own rounded logits (computed on `device` from the
    16-bit `hidden` [..., H] and `weight` [V, H], after step 1's check) and the gradient of the plain
    product: what autograd sees through the reference's 16-bit lm_head (the rounding has no
    gradient of its own). For oracles that go on from the logits in fp64."""
    flat = hidden.reshape(-1, hidden.shape[-1]).to(device).contiguous()
    wd = weight.to(device).contiguous()
    labels = torch.zeros(flat.shape[0], dtype=torch.int64, device=device)
    _, _, _, kept, _ = forward_keeping_logits(flat, wd, labels, 1.0)
    check_rounded_logits(kept.cpu(), flat.cpu(), wd.cpu())
    rounded = kept[:, : weight.shape[0]].cpu().double().view(*hidden.shape[:-1], weight.shape[0])
    exact = h64 @ w64.T
    return exact + (rounded - exact).detach()


def gradient_bounds(P, gh, gw, hidden, weight):
    """Per-element error bounds of the two gradients, from the exact logits gradient P.

    The kernels round P to the 16-bit dtype (relative error <= u per entry, or half the smallest
    subnormal where P underflows the dtype: fp16 has no exponent range to spare for the 1e-6-sized
    entries of a softmax over 150 000 tokens, as in the reference, whose fp16 logits gradient
    underflows the same way), independent from entry to entry, and each result once more: an entry of
    a gradient is sum_k P[k] * W[k] with every term off by up to u times itself, so its error is
    bounded by u * |result| + 6 * sqrt(sum_k (max(u |P[k]| / sqrt(3), tiny) W[k])^2) (six standard
    deviations of independent rounding errors: uniform ones where P is in the normal range, errors
    of up to `tiny` each where entries are flushed towards zero) plus the share of the fp32
    exponentials and accumulation."""
    u = unit_roundoff(hidden.dtype)
    tiny = 2.0 ** -25 if hidden.dtype == torch.float16 else 0.0
    h, w = hidden.to(P.dtype), weight.to(P.dtype)
    Pa = P.abs()
    E2 = torch.clamp(u / 3 ** 0.5 * Pa, min=tiny) ** 2  # variance of the rounding error of an entry of P, at most
    bound_h = u * gh.abs() + 6 * (E2 @ (w * w)).sqrt() + 4e-7 * (Pa @ w.abs()) + 1e-12
    bound_w = u * gw.abs() + 6 * (E2.T @ (h * h)).sqrt() + 4e-7 * (Pa.T @ h.abs()) + 1e-12
    return bound_h, bound_w


def oracle_from_logits(logits, hidden, weight, labels, temperature, g_lp, g_ent):
    """Step 2's reference on the CPU: the oracle's log_probs_from_logits / compute_entropy applied to
    the given (already rounded) logits in fp64, torch autograd through them for the logits gradient
    P, and the two products. Returns (lp, ent, gh, gw, bound_h, bound_w)."""
    from oracle import token_numerics as otn

    x = logits.detach().cpu().double().requires_grad_(True)
    lab = labels.cpu()
    lp = otn.log_probs_from_logits(x, lab, temperature)
    ent = otn.compute_entropy(x)
    torch.autograd.backward([lp, ent], [g_lp.cpu().double(), g_ent.cpu().double()])
    P = x.grad
    h, w = hidden.detach().cpu().double(), weight.detach().cpu().double()
    gh, gw = P @ w, P.T @ h
    bound_h, bound_w = gradient_bounds(P, gh, gw, hidden.detach().cpu(), weight.detach().cpu())
    return lp.detach(), ent.detach(), gh, gw, bound_h, bound_w


def closed_form_from_logits(logits, hidden, weight, labels, temperature, g_lp, g_ent, dtype=torch.float32):
    """The same reference as closed forms on the GPU, for sizes the CPU oracle takes too long on (the
    full-size cases check a row sample against the oracle as well)."""
    x = logits.to(dtype)
    z = x / temperature
    lp = z.gather(1, labels[:, None])[:, 0] - torch.logsumexp(z, -1)
    p1 = torch.softmax(x, -1)
    ex = (p1 * x).sum(-1)
    ent = torch.logsumexp(x, -1) - ex
    g_lp, g_ent = g_lp.to(dtype), g_ent.to(dtype)
    P = p1 * (ex[:, None] - x)
    P *= g_ent[:, None]
    del p1
    P -= torch.softmax(z, -1) * (g_lp / temperature)[:, None]
    del z, x
    P.scatter_add_(1, labels[:, None], (g_lp / temperature)[:, None])
    gh = P @ weight.to(dtype)
    gw = P.T @ hidden.to(dtype)
    bound_h, bound_w = gradient_bounds(P, gh, gw, hidden, weight)
    return lp, ent, gh, gw, bound_h, bound_w


def assert_gradient(got, ref, bound, what):
    """Every entry within its own bound, and the whole matrix within u in the Frobenius norm."""
    err = (got.to(ref.dtype) - ref).abs()
    worst = (err / bound).max().item()
    assert worst <= 1.0, (what, worst)
    u = unit_roundoff(got.dtype)
    rel_fro = (err.pow(2).sum() / ref.pow(2).sum().clamp_min(1e-300)).sqrt().item()
    assert rel_fro <= 2 * u + (bound.pow(2).sum() / ref.pow(2).sum().clamp_min(1e-300)).sqrt().item() / 6, (what, rel_fro)

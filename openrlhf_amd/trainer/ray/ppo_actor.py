"""The loss assembly of the PPO actor training step on hand-written HIP kernels.

Mirrors openrlhf/trainer/ray/ppo_actor.py:294-352 (ActorPPOTrainer.training_step between the
model forward and strategy.backward): action log-probs and entropy from the logits
(openrlhf/models/actor.py:265-296), PolicyLoss, the optional KL loss
``aggregate_loss(compute_approx_kl(...))`` times the KL coefficient, the optional entropy bonus,
and their sum.

``actor_loss_step`` composes the separate kernels in the reference's order and is an ordinary
autograd graph. ``fused_actor_loss_step`` produces the same numbers from ONE pass over the logits:
the per-token derivative of the whole loss is evaluated inside the vocabulary-row kernel as soon
as a row's log-prob is known, and d(loss)/d(logits) is written over the logits (2 x V bytes per
token instead of 3 x; prompt and padding rows are neither read nor computed). It needs the
aggregation weights before the pass, which only depend on the action mask and on the
``loss_batch_info`` normalisers (openrlhf/utils/loss_utils.py:15-105).

Not mirrored: the Mixtral auxiliary loss (a scalar the model returns, added by the caller), the
optimizer step, DeepSpeed. GSPO and seq-mask-TIS need a sequence-level ratio before any token can
be differentiated; ``fused_actor_loss_step`` refuses them (use ``actor_loss_step``).
"""
import torch

from ... import _lib
from ..._lib import call, ptr, require_gpu, stream_of
from ...models.actor import actor_forward_tail, actor_forward_tail_from_hidden
from ...models.loss import PolicyLoss, aggregate_loss
from ...models.utils import _KL_CODES, _as_rows, _workspace, compute_approx_kl, masked_mean


def actor_loss_step(
    logits, sequences, attention_mask, action_mask, old_action_log_probs, advantages, policy_loss_fn: PolicyLoss,
    base_action_log_probs=None, kl_estimator="k1", kl_coef=0.0, entropy_coef=None, rollout_log_probs=None,
    temperature=1.0, packed_indices=None, dp_size=1, batch_num_tokens=None, global_batch_size=None,
    inplace_backward=False, lm_head_weight=None, keep_logits_mib=None,
):
    """Reference-order composition (ppo_actor.py:294-352) on the separate kernels; differentiable.
    With ``lm_head_weight [V, H]`` the first argument holds the decoder's last hidden states instead
    of logits and the projection is fused into the log-prob / entropy (the logits are not stored,
    or only as many 16-bit columns of them as ``keep_logits_mib`` holds; gradients reach the hidden
    states and the weight)."""
    info = dict(dp_size=dp_size, batch_num_tokens=batch_num_tokens, global_batch_size=global_batch_size)
    want_entropy = entropy_coef is not None
    if lm_head_weight is not None:
        out = actor_forward_tail_from_hidden(logits, lm_head_weight, sequences, action_mask, attention_mask,
                                             temperature=temperature, packed_indices=packed_indices,
                                             return_entropy=want_entropy, keep_logits_mib=keep_logits_mib)
    else:
        out = actor_forward_tail(logits, sequences, action_mask, attention_mask, temperature=temperature,
                                 packed_indices=packed_indices, return_entropy=want_entropy,
                                 inplace_backward=inplace_backward)
    action_log_probs, entropy = out if want_entropy else (out, None)
    actor_loss, clip_ratio, ppo_kl, vllm_kl = policy_loss_fn(
        action_log_probs, old_action_log_probs, advantages, action_mask=action_mask,
        rollout_log_probs=rollout_log_probs, **info)
    result = dict(actor_loss=actor_loss, clip_ratio=clip_ratio, ppo_kl=ppo_kl, vllm_kl=vllm_kl,
                  action_log_probs=action_log_probs, entropy=entropy, kl_loss=None, entropy_loss=None,
                  logprobs_diff=None)
    loss = actor_loss
    if base_action_log_probs is not None:
        kl = compute_approx_kl(action_log_probs, base_action_log_probs, kl_estimator=kl_estimator)
        result["kl_loss"] = aggregate_loss(kl, action_mask, **info)
        # the "logprobs_diff" status of the step (ppo_actor.py:327-333): masked mean of lp - base
        with torch.no_grad():
            result["logprobs_diff"] = masked_mean(action_log_probs.float() - base_action_log_probs.float(), action_mask)
        loss = loss + result["kl_loss"] * kl_coef
    if want_entropy:
        result["entropy_loss"] = aggregate_loss(entropy[:, -action_mask.shape[1]:], action_mask, **info)
        if entropy_coef != 0:
            loss = loss - result["entropy_loss"] * entropy_coef
    result["loss"] = loss
    return result


def _row_coef(action_mask, token_level, dp_size, norm_value):
    """d(aggregate_loss)/d(masked token sum of row b) for every row: the weight of a token of row b
    in the aggregated loss is row_coef[b] * mask[b, t]."""
    dev = action_mask.device
    b, a = action_mask.shape
    mkeep, mptr, mcode = _lib.mask_arg(action_mask)
    keep = []
    norm = _lib.make_norm(dp_size, norm_value, keep)
    ws = _workspace(b, a, dev)
    row_coef = torch.empty(max(b, 1), dtype=torch.float32, device=dev)
    with _lib.on_device(dev):
        call("orlhf_mask_row_coef", mptr, mcode, b, a, _lib.AGG_TOKEN_MEAN if token_level else _lib.AGG_SEQ_MEAN, norm,
             ptr(ws), ptr(row_coef), stream_of(dev))
    return row_coef


def _f32c(t):
    return t.to(torch.float32).contiguous()


class _HandOverGradient(torch.autograd.Function):
    """Connects a loss value to logits whose gradient has already been written: backward hands
    that gradient over, rescaled on the device only if the upstream gradient is not the scale
    it was produced with."""

    @staticmethod
    def forward(ctx, logits, loss_value, grad_logits, produced_scale):
        ctx.save_for_backward(grad_logits)
        ctx.produced_scale = float(produced_scale)
        return loss_value.clone()

    @staticmethod
    def backward(ctx, g):
        (grad,) = ctx.saved_tensors
        if getattr(ctx, "handed_over", False):
            # the stored gradient may have been rescaled in place by the first backward
            raise RuntimeError("the gradient of a fused actor step can be handed over once; run the step again")
        ctx.handed_over = True
        dev = grad.device
        gf = g.reshape(-1)[:1].to(torch.float32).contiguous()
        with _lib.on_device(dev):
            call("orlhf_rescale_inplace_if", ptr(grad), _lib.dtype_code(grad), grad.numel(), ptr(gf),
                 ctx.produced_scale, stream_of(dev))
        return grad, None, None, None


def fused_actor_loss_step(
    logits, sequences, attention_mask, action_mask, old_action_log_probs, advantages, policy_loss_fn: PolicyLoss,
    base_action_log_probs=None, kl_estimator="k1", kl_coef=0.0, entropy_coef=None, rollout_log_probs=None,
    temperature=1.0, packed_indices=None, dp_size=1, batch_num_tokens=None, global_batch_size=None,
    loss_scale=1.0,
):
    """Same results as ``actor_loss_step`` followed by ``(loss * loss_scale).backward()`` down to
    the logits, from one pass over them. Returns the same dict plus ``grad_logits`` (aliasing the
    logits storage, already holding ``loss_scale * d(loss)/d(logits)``). ``result["loss"]`` is
    attached to ``logits`` in the autograd graph: ``(result["loss"] * loss_scale).backward()``
    (what a gradient-accumulating engine does with ``loss_scale = 1 / accumulation_steps``) hands
    the stored gradient to the layer that produced the logits without another pass.

    logits: contiguous ``[B, T, V]``, or packed ``[Ttot, V]`` / ``[1, Ttot, V]`` with
    ``packed_indices``. The logits are consumed: their storage holds the gradient afterwards.
    """
    if policy_loss_fn.policy_loss_type != "ppo":
        raise ValueError("fused_actor_loss_step fuses the token-level PPO surrogate only; use actor_loss_step for "
                         f"policy_loss_type={policy_loss_fn.policy_loss_type!r}")
    use_is = bool(policy_loss_fn.enable_vllm_is_correction)
    if use_is and policy_loss_fn.vllm_is_correction_type == "seq-mask-tis":
        raise ValueError("seq-mask-tis needs a sequence-level ratio first; use actor_loss_step")
    if use_is and rollout_log_probs is None:
        raise ValueError("enable_vllm_is_correction needs rollout_log_probs")
    if base_action_log_probs is not None and kl_estimator not in _KL_CODES:
        raise ValueError(f"Unknown kl_estimator: {kl_estimator}")
    dev = require_gpu(logits, sequences, action_mask, old_action_log_probs, advantages)
    batch, seqlen = sequences.shape
    width = action_mask.shape[1]
    lo_col, hi_col = seqlen - 1 - width, seqlen - 1
    info = dict(dp_size=dp_size, batch_num_tokens=batch_num_tokens, global_batch_size=global_batch_size)

    with torch.no_grad():
        rows, row_stride, aliases = _as_rows(logits.detach().reshape(-1, logits.shape[-1]) if logits.dim() == 3
                                            else logits.detach())
        if not aliases or rows.data_ptr() != logits.data_ptr():
            raise ValueError("fused_actor_loss_step needs logits it can overwrite: contiguous [B, T, V] or [Ttot, V]")
        n_rows, vocab = rows.shape
        expect_rows = batch * seqlen if packed_indices is None else packed_indices.numel()
        if n_rows != expect_rows:
            raise ValueError(f"{n_rows} logits rows for {expect_rows} token positions")
        code = _lib.dtype_code(rows)
        if vocab > _lib.load().orlhf_logprob_entropy_fwd_bwd_max_vocab(code):
            raise ValueError(f"a row of {vocab} {rows.dtype} logits is too long for the one-pass kernel; use actor_loss_step")

        # aggregation weights per batch row (they only depend on the mask and the normalisers)
        token_rc = _row_coef(action_mask, True, dp_size, batch_num_tokens)
        policy_rc = token_rc if policy_loss_fn.token_level_loss else _row_coef(action_mask, False, dp_size, global_batch_size)

        # one gather launch: everything the vocabulary-row kernel needs per logits row
        want_entropy = entropy_coef is not None
        has_base = base_action_log_probs is not None
        f32 = dict(dtype=torch.float32, device=dev)
        per_row = torch.empty(7, n_rows, **f32)
        weight_r, old_r, adv_r, pc_r, tc_r = per_row[0], per_row[1], per_row[2], per_row[3], per_row[4]
        roll_r = per_row[5] if use_is else None
        base_r = per_row[6] if has_base else None
        labels = torch.empty(n_rows, dtype=torch.int64, device=dev)
        need_r = torch.empty(n_rows, dtype=torch.uint8, device=dev)
        mkeep, mptr, mcode = _lib.mask_arg(action_mask)
        seqs = sequences.to(torch.int64).contiguous()
        idx = None if packed_indices is None else packed_indices.to(torch.int64).contiguous()
        old_in, adv_in = _f32c(old_action_log_probs), _f32c(advantages)
        roll_in = _f32c(rollout_log_probs) if use_is else None
        base_in = _f32c(base_action_log_probs) if has_base else None

        terms = _lib.StepTerms()
        terms.old_log_probs, terms.advantages = ptr(old_r), ptr(adv_r)
        terms.rollout_log_probs, terms.base_log_probs = ptr(roll_r), ptr(base_r)
        terms.policy_coef, terms.token_coef = ptr(pc_r), ptr(tc_r)
        terms.clip_eps_low, terms.clip_eps_high = float(policy_loss_fn.clip_eps_low), float(policy_loss_fn.clip_eps_high)
        terms.dual_clip = float(policy_loss_fn.dual_clip) if policy_loss_fn.dual_clip is not None else 0.0
        terms.is_correction = ({"tis": _lib.IS_TIS, "icepop": _lib.IS_ICEPOP}[policy_loss_fn.vllm_is_correction_type]
                               if use_is else _lib.IS_NONE)
        if use_is:
            terms.is_low, terms.is_high = (float(v) for v in policy_loss_fn.vllm_is_truncated_threshold)
        terms.kl_estimator = _KL_CODES.get(kl_estimator, 0)
        terms.kl_coef = float(kl_coef) if has_base else 0.0
        terms.entropy_coef = float(entropy_coef) if want_entropy else 0.0

        lp_r = torch.empty(n_rows, **f32)
        ent_r = torch.empty(n_rows, **f32) if want_entropy else None
        action_log_probs = torch.zeros(batch, width, **f32)
        entropy = torch.zeros(batch, width, **f32) if want_entropy else None
        out8 = torch.empty(8, **f32)
        lib = _lib.load()
        ws = torch.empty(lib.orlhf_actor_step_values_workspace_bytes(n_rows), dtype=torch.uint8, device=dev)
        with _lib.on_device(dev):
            stream = stream_of(dev)
            call("orlhf_actor_step_gather", ptr(seqs), mptr, mcode, ptr(idx), batch, seqlen, width, n_rows, ptr(old_in),
                 ptr(adv_in), ptr(roll_in), ptr(base_in), ptr(policy_rc), ptr(token_rc), float(loss_scale), ptr(labels),
                 ptr(need_r), ptr(weight_r), ptr(old_r), ptr(adv_r), ptr(roll_r), ptr(base_r), ptr(pc_r), ptr(tc_r), stream)
            call("orlhf_policy_step_fwd_bwd", ptr(rows), ptr(rows), code, n_rows, vocab, row_stride, row_stride,
                 ptr(labels), float(temperature), terms, ptr(lp_r), ptr(ent_r), ptr(need_r), stream)
            # every value of the step from the per-row results, and their scatter back to [B, A]
            call("orlhf_actor_step_values", ptr(lp_r), ptr(ent_r), ptr(weight_r), ptr(old_r), ptr(adv_r), ptr(roll_r),
                 ptr(base_r), ptr(pc_r), ptr(tc_r), ptr(idx), seqlen, width, n_rows, terms, float(loss_scale),
                 1 if (want_entropy and entropy_coef != 0) else 0, ptr(ws), ptr(action_log_probs), ptr(entropy),
                 ptr(out8), stream)
        torch.autograd.graph.increment_version(rows)
        loss, actor_loss, clip_ratio, ppo_kl = out8[0], out8[1], out8[2], out8[3]
        vllm_kl = out8[4] if use_is else None
        kl_loss = out8[5] if has_base else None
        entropy_loss = out8[6] if want_entropy else None
        logprobs_diff = out8[7] if has_base else None

    grad_logits = rows if rows.shape == logits.shape else rows.view(logits.shape)
    if logits.requires_grad:
        loss = _HandOverGradient.apply(logits, loss, grad_logits, loss_scale)
    return dict(loss=loss, actor_loss=actor_loss, clip_ratio=clip_ratio, ppo_kl=ppo_kl, vllm_kl=vllm_kl,
                kl_loss=kl_loss, entropy_loss=entropy_loss, logprobs_diff=logprobs_diff,
                action_log_probs=action_log_probs, entropy=entropy, grad_logits=grad_logits)

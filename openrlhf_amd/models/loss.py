"""Losses with the signatures of ``openrlhf.models.loss`` on hand-written HIP kernels.

Mirrors (paths relative to the OpenRLHF tree):
  aggregate_loss   openrlhf/models/loss.py:11-39
  GPTLMLoss        openrlhf/models/loss.py:42-84
  SFTLoss          openrlhf/models/loss.py:87-113
  PolicyLoss       openrlhf/models/loss.py:116-230
  ValueLoss        openrlhf/models/loss.py:233-269
  PairWiseLoss     openrlhf/models/loss.py:272-284
  LogExpLoss       openrlhf/models/loss.py:287-297
  DPOLoss          openrlhf/models/loss.py:300-335

Each loss is one elementwise + reduction launch pair forward and one elementwise launch
backward instead of the reference's chain of ~20 eager kernels. Per-token inputs are consumed
as fp32. ``batch_num_tokens`` / ``global_batch_size`` may be Python numbers or 0-dim tensors
(device tensors are read on the device, no host synchronisation). Every loss also accepts the
packed layout: flat per-token tensors plus ``cu_seqlens`` (int64 [B+1]) and ``max_seqlen``, a
bound on the longest row that sizes the launch (rows longer than it would be cut; when it is
omitted the longest row is read back from ``cu_seqlens``, one synchronisation).
"""
from typing import Optional

import torch
import torch.nn as nn

from .. import _lib
from .._lib import call, ptr, require_gpu, stream_of
from .utils import _Aggregate, _cu_arg, _f32, _packed, _rows_of, _workspace, masked_mean  # noqa: F401


def aggregate_loss(
    loss: torch.Tensor,
    loss_mask: torch.Tensor,
    token_level_loss: bool = True,
    dp_size: int = 1,
    batch_num_tokens: Optional[float] = None,
    global_batch_size: Optional[float] = None,
    cu_seqlens: Optional[torch.Tensor] = None,
    max_seqlen: Optional[int] = None,
    seq_token_sum: bool = False,
) -> torch.Tensor:
    """token_level_loss=True: sum(loss*mask) / (sum(mask) or batch_num_tokens) [* dp_size when
    the global count is given]; False: mean over non-empty rows of sum(loss*mask)/(count+1e-8),
    or that sum / global_batch_size * dp_size (openrlhf/models/loss.py:11-39).

    ``seq_token_sum=True`` (not in the reference; with ``token_level_loss=False``) averages the
    per-sequence token SUMS instead of the per-sequence token means."""
    cu_seqlens = _packed(cu_seqlens, max_seqlen)
    if seq_token_sum:
        if token_level_loss:
            raise ValueError("seq_token_sum is a sequence-level mode: pass token_level_loss=False")
        return _Aggregate.apply(loss, loss_mask, _lib.AGG_SEQ_MEAN_TOKEN_SUM, dp_size, global_batch_size, cu_seqlens)
    if token_level_loss:
        return _Aggregate.apply(loss, loss_mask, _lib.AGG_TOKEN_MEAN, dp_size, batch_num_tokens, cu_seqlens)
    return _Aggregate.apply(loss, loss_mask, _lib.AGG_SEQ_MEAN, dp_size, global_batch_size, cu_seqlens)


class GPTLMLoss(nn.Module):
    """Next-token cross entropy with ``ignore_index = -100`` averaged over the kept positions
    (openrlhf/models/loss.py:42-84, the path without ring attention): position t is scored against
    ``labels[..., t+1]``. The logits are read in place (no shifted contiguous copy), ignored
    positions are neither read nor differentiated; all labels ignored gives NaN, as
    ``nn.CrossEntropyLoss`` does."""

    def __init__(self, ring_attn_group=None):
        super().__init__()
        if ring_attn_group is not None:
            raise NotImplementedError("GPTLMLoss over a ring-attention group needs collectives; one GPU is built")
        self.IGNORE_INDEX = -100

    def forward(self, logits: torch.Tensor, labels: torch.Tensor, inplace_backward: bool = False) -> torch.Tensor:
        from .utils import _LogprobEntropy

        if labels.shape != logits.shape[:-1]:
            raise ValueError(f"labels {tuple(labels.shape)} do not match logits {tuple(logits.shape)}")
        nxt = torch.roll(labels, shifts=-1, dims=-1).clone()
        nxt[..., -1] = self.IGNORE_INDEX
        keep = nxt != self.IGNORE_INDEX
        lp = _LogprobEntropy.apply(logits, nxt, 1.0, True, False, inplace_backward, keep)[0]
        return _Aggregate.apply(-lp, keep, _lib.AGG_TOKEN_MEAN, 1, None, None)


class SFTLoss(nn.Module):
    """-log-prob aggregated over the loss mask (openrlhf/models/loss.py:87-113)."""

    def __init__(self, token_level_loss: bool = True):
        super().__init__()
        self.token_level_loss = token_level_loss

    def forward(self, per_token_logps, loss_mask, dp_size=1, batch_num_tokens=None, global_batch_size=None):
        return aggregate_loss(
            -per_token_logps, loss_mask, token_level_loss=self.token_level_loss, dp_size=dp_size,
            batch_num_tokens=batch_num_tokens, global_batch_size=global_batch_size,
        )


_IS_CODES = {"tis": _lib.IS_TIS, "icepop": _lib.IS_ICEPOP, "seq-mask-tis": _lib.IS_SEQ_MASK_TIS}


def _weights_known(token_level, norm_value):
    """A token's weight in the loss is known before any token is read: token mean over a given count."""
    return bool(token_level) and norm_value is not None


def _hand_over(ctx, g, dev):
    """The gradient the forward already wrote for a unit upstream gradient, multiplied in place by
    the upstream gradient on the device (the kernel returns at once when that is 1). The stored
    tensor is given away: a second backward through the same node (retain_graph) recomputes."""
    grad, ctx.ready_grad = ctx.ready_grad, None
    with _lib.on_device(dev):
        call("orlhf_rescale_inplace_if", ptr(grad), _lib.F32, grad.numel(), ptr(g), 1.0, stream_of(dev))
    return grad


class _PolicyLossFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, log_probs, old_log_probs, advantages, action_mask, rollout_log_probs, cfg, dp_size,
                norm_value, cu_seqlens):
        ctx.set_materialize_grads(False)  # no zero-filled gradients for the three statistics
        dev = require_gpu(log_probs, old_log_probs, advantages, action_mask, rollout_log_probs)
        lp, old, adv = _f32(log_probs), _f32(old_log_probs.detach()), _f32(advantages.detach())
        if old.shape != lp.shape or adv.shape != lp.shape:
            old, adv = old.expand_as(lp).contiguous(), adv.expand_as(lp).contiguous()
        rollout = None if rollout_log_probs is None else _f32(rollout_log_probs.detach())
        n_rows, n_cols = _rows_of(lp, cu_seqlens)
        if action_mask is not None and action_mask.shape != lp.shape:
            action_mask = action_mask.expand_as(lp)
        mkeep, mptr, mcode = _lib.mask_arg(action_mask)
        cu = _cu_arg(cu_seqlens, dev)
        keep = []
        params = _lib.PolicyParams()
        params.clip_eps_low, params.clip_eps_high = cfg["clip_eps_low"], cfg["clip_eps_high"]
        params.dual_clip = cfg["dual_clip"] if cfg["dual_clip"] is not None else 0.0
        params.policy_type = cfg["policy_type"]
        params.is_correction = cfg["is_correction"]
        params.is_low, params.is_high = cfg["is_low"], cfg["is_high"]
        params.token_level = 1 if cfg["token_level"] else 0
        params.norm = _lib.make_norm(dp_size, norm_value, keep)
        ws = _workspace(n_rows, n_cols, dev)
        out4 = torch.empty(4, dtype=torch.float32, device=dev)
        row_coef = torch.empty(max(n_rows, 1), dtype=torch.float32, device=dev)
        row_aux = torch.empty(max(n_rows, 1) * 2, dtype=torch.float32, device=dev)
        # token mean over a given count (the trainers' loss_batch_info): every token's weight is known
        # before the pass, so the gradient for a unit upstream gradient is written by the forward
        ctx.ready_grad = None
        if ctx.needs_input_grad[0] and _weights_known(cfg["token_level"], norm_value) \
                and cfg["policy_type"] == _lib.POLICY_PPO:
            ctx.ready_grad = torch.empty(lp.shape, dtype=torch.float32, device=dev)
        with _lib.on_device(dev):
            if ctx.ready_grad is not None:
                call("orlhf_policy_loss_fwd_grad", ptr(lp), ptr(old), ptr(adv), mptr, mcode, ptr(rollout), n_rows,
                     n_cols, ptr(cu), params, ptr(ws), ptr(out4), ptr(row_coef), ptr(row_aux), ptr(ctx.ready_grad),
                     stream_of(dev))
            else:
                call("orlhf_policy_loss_fwd", ptr(lp), ptr(old), ptr(adv), mptr, mcode, ptr(rollout), n_rows, n_cols,
                     ptr(cu), params, ptr(ws), ptr(out4), ptr(row_coef), ptr(row_aux), stream_of(dev))
        ctx.params, ctx.keep, ctx.dims, ctx.mcode = params, keep, (n_rows, n_cols), mcode
        ctx.lp_shape, ctx.lp_dtype = log_probs.shape, log_probs.dtype
        ctx.save_for_backward(lp, old, adv, mkeep, rollout, cu, row_coef, row_aux)
        loss, clip_ratio, ppo_kl, vllm_kl = out4[0], out4[1], out4[2], out4[3]
        ctx.mark_non_differentiable(clip_ratio, ppo_kl, vllm_kl)
        return loss, clip_ratio, ppo_kl, vllm_kl

    @staticmethod
    def backward(ctx, g_loss, _g1, _g2, _g3):
        if g_loss is None:
            return (None,) * 9
        lp, old, adv, mkeep, rollout, cu, row_coef, row_aux = ctx.saved_tensors
        dev = lp.device
        n_rows, n_cols = ctx.dims
        g = _f32(g_loss).reshape(-1)
        if ctx.ready_grad is not None:
            return (_hand_over(ctx, g, dev).view(ctx.lp_shape).to(ctx.lp_dtype),) + (None,) * 8
        g_lp = torch.empty(lp.shape, dtype=torch.float32, device=dev)
        ws = _workspace(n_rows, n_cols, dev) if ctx.params.policy_type == _lib.POLICY_GSPO else None
        with _lib.on_device(dev):
            call("orlhf_policy_loss_bwd", ptr(g), ptr(lp), ptr(old), ptr(adv), ptr(mkeep), ctx.mcode, ptr(rollout),
                 n_rows, n_cols, ptr(cu), ctx.params, ptr(row_coef), ptr(row_aux), ptr(ws), ptr(g_lp),
                 stream_of(dev))
        return g_lp.view(ctx.lp_shape).to(ctx.lp_dtype), None, None, None, None, None, None, None, None


class PolicyLoss(nn.Module):
    """PPO / GSPO policy loss (openrlhf/models/loss.py:116-230): low/high ratio clip, optional
    dual clip, optional TIS / ICEPOP / seq-mask-TIS importance correction against the rollout
    engine's log-probs, token- or sequence-level aggregation. forward returns
    (loss, clip_ratio, ppo_kl, vllm_kl-or-None)."""

    def __init__(
        self,
        clip_eps_low: float = 0.2,
        clip_eps_high: float = 0.2,
        dual_clip: float = None,
        token_level_loss: bool = True,
        policy_loss_type: str = "ppo",
        enable_vllm_is_correction: bool = False,
        vllm_is_truncated_threshold: list = None,
        vllm_is_correction_type: str = "tis",
    ) -> None:
        super().__init__()
        self.clip_eps_low = clip_eps_low
        self.clip_eps_high = clip_eps_high
        self.token_level_loss = token_level_loss
        self.dual_clip = dual_clip
        self.policy_loss_type = policy_loss_type
        self.enable_vllm_is_correction = enable_vllm_is_correction
        self.vllm_is_truncated_threshold = vllm_is_truncated_threshold
        self.vllm_is_correction_type = vllm_is_correction_type

        if policy_loss_type == "gspo":  # GSPO is defined on per-sequence means
            self.token_level_loss = False
        if dual_clip is not None:
            assert dual_clip > 1.0, f"dual_clip must be > 1.0, got {dual_clip}"
        if self.vllm_is_correction_type not in _IS_CODES:
            raise ValueError(
                f"Invalid vllm_is_correction_type: {self.vllm_is_correction_type}, must be one of tis/icepop/seq-mask-tis"
            )

    def forward(
        self,
        log_probs: torch.Tensor,
        old_log_probs: torch.Tensor,
        advantages: torch.Tensor,
        action_mask: Optional[torch.Tensor] = None,
        rollout_log_probs: Optional[torch.Tensor] = None,
        dp_size: int = 1,
        batch_num_tokens: Optional[float] = None,
        global_batch_size: Optional[float] = None,
        cu_seqlens: Optional[torch.Tensor] = None,
        max_seqlen: Optional[int] = None,
    ):
        if self.policy_loss_type == "ppo":
            policy_type = _lib.POLICY_PPO
        elif self.policy_loss_type == "gspo":
            policy_type = _lib.POLICY_GSPO
        else:
            raise ValueError(f"Invalid policy loss type: {self.policy_loss_type}")
        use_is = bool(self.enable_vllm_is_correction)
        if use_is and rollout_log_probs is None:
            raise ValueError("enable_vllm_is_correction needs rollout_log_probs")
        lo, hi = (self.vllm_is_truncated_threshold if use_is and policy_type == _lib.POLICY_PPO else (0.0, 0.0))
        cfg = dict(
            clip_eps_low=float(self.clip_eps_low),
            clip_eps_high=float(self.clip_eps_high),
            dual_clip=None if self.dual_clip is None else float(self.dual_clip),
            policy_type=policy_type,
            is_correction=_IS_CODES[self.vllm_is_correction_type] if use_is else _lib.IS_NONE,
            is_low=float(lo),
            is_high=float(hi),
            token_level=bool(self.token_level_loss),
        )
        norm_value = batch_num_tokens if (self.token_level_loss and policy_type == _lib.POLICY_PPO) else global_batch_size
        loss, clip_ratio, ppo_kl, vllm_kl = _PolicyLossFn.apply(
            log_probs, old_log_probs, advantages, action_mask, rollout_log_probs if use_is else None, cfg,
            dp_size, norm_value, _packed(cu_seqlens, max_seqlen),
        )
        if not (use_is and policy_type == _lib.POLICY_PPO):
            vllm_kl = None
        return loss, clip_ratio, ppo_kl, vllm_kl


class _ValueLossFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, values, old_values, returns, action_mask, clip_eps, token_level, dp_size, norm_value,
                cu_seqlens):
        ctx.set_materialize_grads(False)  # no zero-filled gradient for the mean of the values
        dev = require_gpu(values, old_values, returns, action_mask)
        v, ret = _f32(values), _f32(returns.detach())
        old = None if old_values is None else _f32(old_values.detach())
        n_rows, n_cols = _rows_of(v, cu_seqlens)
        if action_mask is not None and action_mask.shape != v.shape:
            action_mask = action_mask.expand_as(v)
        mkeep, mptr, mcode = _lib.mask_arg(action_mask)
        cu = _cu_arg(cu_seqlens, dev)
        keep = []
        norm = _lib.make_norm(dp_size, norm_value, keep)
        ws = _workspace(n_rows, n_cols, dev)
        out = torch.empty(2, dtype=torch.float32, device=dev)  # loss, masked mean of the values
        row_coef = torch.empty(max(n_rows, 1), dtype=torch.float32, device=dev)
        has_clip = clip_eps is not None
        ctx.ready_grad = None
        if ctx.needs_input_grad[0] and _weights_known(token_level, norm_value):
            ctx.ready_grad = torch.empty(v.shape, dtype=torch.float32, device=dev)
        with _lib.on_device(dev):
            if ctx.ready_grad is not None:
                call("orlhf_value_loss_fwd_grad", ptr(v), ptr(old), ptr(ret), mptr, mcode, n_rows, n_cols, ptr(cu),
                     1 if has_clip else 0, float(clip_eps) if has_clip else 0.0, norm, ptr(ws), ptr(out),
                     ptr(row_coef), ptr(ctx.ready_grad), stream_of(dev))
            else:
                call("orlhf_value_loss_fwd", ptr(v), ptr(old), ptr(ret), mptr, mcode, n_rows, n_cols, ptr(cu),
                     1 if has_clip else 0, float(clip_eps) if has_clip else 0.0, 1 if token_level else 0, norm,
                     ptr(ws), ptr(out), ptr(row_coef), stream_of(dev))
        ctx.clip, ctx.dims, ctx.mcode = (has_clip, float(clip_eps) if has_clip else 0.0), (n_rows, n_cols), mcode
        ctx.v_shape, ctx.v_dtype = values.shape, values.dtype
        ctx.save_for_backward(v, old, ret, mkeep, cu, row_coef)
        loss, values_mean = out[0], out[1]
        ctx.mark_non_differentiable(values_mean)
        return loss, values_mean

    @staticmethod
    def backward(ctx, g_out, _g_mean):
        if g_out is None:
            return (None,) * 9
        v, old, ret, mkeep, cu, row_coef = ctx.saved_tensors
        dev = v.device
        n_rows, n_cols = ctx.dims
        g = _f32(g_out).reshape(-1)
        if ctx.ready_grad is not None:
            return (_hand_over(ctx, g, dev).view(ctx.v_shape).to(ctx.v_dtype),) + (None,) * 8
        g_v = torch.empty(v.shape, dtype=torch.float32, device=dev)
        with _lib.on_device(dev):
            call("orlhf_value_loss_bwd", ptr(g), ptr(v), ptr(old), ptr(ret), ptr(mkeep), ctx.mcode, n_rows, n_cols,
                 ptr(cu), 1 if ctx.clip[0] else 0, ctx.clip[1], ptr(row_coef), ptr(g_v), stream_of(dev))
        return g_v.view(ctx.v_shape).to(ctx.v_dtype), None, None, None, None, None, None, None, None


class ValueLoss(nn.Module):
    """Clipped value loss (openrlhf/models/loss.py:233-269): 0.5 * aggregate(max((clip(v) - R)^2,
    (v - R)^2)); no clip_eps gives 0.5 * aggregate((v - R)^2)."""

    def __init__(self, clip_eps: float = None, token_level_loss: bool = True) -> None:
        super().__init__()
        self.clip_eps = clip_eps
        self.token_level_loss = token_level_loss

    def forward(
        self,
        values: torch.Tensor,
        old_values: torch.Tensor,
        returns: torch.Tensor,
        action_mask: Optional[torch.Tensor] = None,
        dp_size: int = 1,
        batch_num_tokens: Optional[float] = None,
        global_batch_size: Optional[float] = None,
        cu_seqlens: Optional[torch.Tensor] = None,
        max_seqlen: Optional[int] = None,
    ) -> torch.Tensor:
        return self.loss_and_values_mean(values, old_values, returns, action_mask, dp_size, batch_num_tokens,
                                         global_batch_size, cu_seqlens, max_seqlen)[0]

    def loss_and_values_mean(self, values, old_values, returns, action_mask=None, dp_size=1, batch_num_tokens=None,
                             global_batch_size=None, cu_seqlens=None, max_seqlen=None):
        """(loss, masked_mean(values, action_mask)) from one pass: the second is the "values"
        status the critic trainer logs next to the loss (openrlhf/trainer/ray/ppo_critic.py:174),
        detached."""
        norm_value = batch_num_tokens if self.token_level_loss else global_batch_size
        return _ValueLossFn.apply(
            values, old_values if self.clip_eps is not None else None, returns, action_mask, self.clip_eps,
            self.token_level_loss, dp_size, norm_value, _packed(cu_seqlens, max_seqlen),
        )


class _PairLossFn(torch.autograd.Function):
    """mean over pairs of a pairwise loss of z = (chosen - rejected) - (ref_chosen - ref_rejected)."""

    @staticmethod
    def forward(ctx, chosen, rejected, ref_chosen, ref_rejected, kind, beta, label_smoothing, want_rewards):
        ctx.set_materialize_grads(False)  # no zero-filled gradients for the two reward estimates
        dev = require_gpu(chosen, rejected, ref_chosen, ref_rejected)
        if chosen.shape != rejected.shape:
            raise ValueError(f"chosen {tuple(chosen.shape)} and rejected {tuple(rejected.shape)} differ in shape")
        a, b = _f32(chosen).reshape(-1), _f32(rejected).reshape(-1)
        c = None if ref_chosen is None else _f32(ref_chosen.detach()).expand_as(chosen).reshape(-1).contiguous()
        d = None if ref_rejected is None else _f32(ref_rejected.detach()).expand_as(chosen).reshape(-1).contiguous()
        n = a.numel()
        loss = torch.empty(1, dtype=torch.float32, device=dev)
        cr = torch.empty(n, dtype=torch.float32, device=dev) if want_rewards else None
        rr = torch.empty(n, dtype=torch.float32, device=dev) if want_rewards else None
        with _lib.on_device(dev):
            call("orlhf_pair_loss_fwd", ptr(a), ptr(b), ptr(c), ptr(d), n, kind, float(beta), float(label_smoothing),
                 ptr(loss), ptr(cr), ptr(rr), stream_of(dev))
        ctx.save_for_backward(a, b, c, d)
        ctx.cfg = (kind, float(beta), float(label_smoothing), chosen.shape, chosen.dtype, rejected.dtype)
        if want_rewards:
            cr, rr = cr.view(chosen.shape), rr.view(chosen.shape)
            ctx.mark_non_differentiable(cr, rr)
        return loss.reshape(()), cr, rr

    @staticmethod
    def backward(ctx, g_loss, _g_cr, _g_rr):
        if g_loss is None:
            return (None,) * 8
        a, b, c, d = ctx.saved_tensors
        kind, beta, smooth, shape, dt_a, dt_b = ctx.cfg
        dev = a.device
        g = g_loss.reshape(1).to(torch.float32).contiguous()
        ga = torch.empty_like(a) if ctx.needs_input_grad[0] else None
        gb = torch.empty_like(b) if ctx.needs_input_grad[1] else None
        with _lib.on_device(dev):
            call("orlhf_pair_loss_bwd", ptr(g), ptr(a), ptr(b), ptr(c), ptr(d), a.numel(), kind, beta, smooth,
                 ptr(ga), ptr(gb), stream_of(dev))
        ga = None if ga is None else ga.view(shape).to(dt_a)
        gb = None if gb is None else gb.view(shape).to(dt_b)
        return ga, gb, None, None, None, None, None, None


class DPOLoss(nn.Module):
    """DPO / conservative DPO / IPO preference loss (openrlhf/models/loss.py:300-335): returns
    ``(loss, chosen_rewards, rejected_rewards)``; the reference log-probs carry no gradient."""

    def __init__(self, beta: float, label_smoothing: float = 0.0, ipo: bool = False) -> None:
        super().__init__()
        self.beta = beta
        self.label_smoothing = label_smoothing
        self.ipo = ipo

    def forward(self, policy_chosen_logps, policy_rejected_logps, reference_chosen_logps, reference_rejected_logps):
        kind = _lib.PAIR_DPO_IPO if self.ipo else _lib.PAIR_DPO_SIGMOID
        return _PairLossFn.apply(policy_chosen_logps, policy_rejected_logps, reference_chosen_logps,
                                 reference_rejected_logps, kind, self.beta, self.label_smoothing, True)


class PairWiseLoss(nn.Module):
    """Reward-model pairwise loss -logsigmoid(chosen - rejected [- margin]).mean()
    (openrlhf/models/loss.py:272-284)."""

    def forward(self, chosen_reward, reject_reward, margin=None):
        return _PairLossFn.apply(chosen_reward, reject_reward, margin, None, _lib.PAIR_LOGSIGMOID, 1.0, 0.0, False)[0]


class LogExpLoss(nn.Module):
    """Reward-model loss log(1 + exp(rejected - chosen)).mean(); the margin is ignored, as in the
    reference (openrlhf/models/loss.py:287-297)."""

    def forward(self, chosen_reward, reject_reward, margin=None):
        return _PairLossFn.apply(chosen_reward, reject_reward, None, None, _lib.PAIR_LOGEXP, 1.0, 0.0, False)[0]

"""Token-level numerics with the call signatures of ``openrlhf.models.utils``.

Mirrors (paths relative to the OpenRLHF tree):
  compute_approx_kl        openrlhf/models/utils.py:64-95
  compute_reward           openrlhf/models/utils.py:98-126
  log_probs_from_logits    openrlhf/models/utils.py:139-163
  masked_mean              openrlhf/models/utils.py:166-169
  masked_normalize         openrlhf/models/utils.py:172-179
  compute_entropy          openrlhf/models/utils.py:182-186
plus ``logprobs_and_entropy_from_logits``, the one-pass form of what Actor.forward does with
two calls (openrlhf/models/actor.py:269-285), and ``lm_head_logprobs_and_entropy``, the same from
the last hidden states and the lm_head weight with the logits never stored
(openrlhf/models/actor.py:263-285).

Every function launches hand-written HIP kernels through the C ABI; tensors must be on the GPU.

Deliberate differences from the reference, all on the value-preserving side:
  * bf16 / fp16 logits are accumulated in fp32 and the result is returned in fp32 (the reference
    computes and returns the input dtype for those);
  * ``log_probs_from_logits`` does not divide the caller's logits in place when
    ``temperature != 1``; the division is folded into the loads;
  * ``compute_reward`` takes tensors only (the reference's list-of-tensors form of ``kl`` is not
    used by any caller).
"""
from typing import Optional, Tuple

import torch

from .. import _lib
from .._lib import call, ptr, require_gpu, stream_of

_KL_CODES = {"k1": _lib.KL_K1, "k2": _lib.KL_K2, "k3": _lib.KL_K3}


# ------------------------------------------------------------------ vocabulary rows
def _as_rows(logits: torch.Tensor):
    """[..., V] -> (2-D tensor, row stride in elements, whether it aliases the input's storage:
    it does unless the layout forces a contiguous copy)."""
    vocab = logits.shape[-1]
    if logits.is_contiguous():
        return logits.view(-1, vocab), vocab, True
    if logits.dim() == 2 and logits.stride(1) == 1 and logits.stride(0) >= vocab:
        return logits, logits.stride(0), True
    return logits.contiguous().view(-1, vocab), vocab, False



_TICKETS = {}  # (device index, stream handle) -> int32 tickets, all zero whenever no forward is in flight


def _row_tickets(dev, n_rows):
    """The tickets of the few-row forward: zero on entry, put back to zero by the kernel itself, so one
    array per (device, stream) serves every call (calls on one stream do not overlap). Allocated and
    zeroed outside any graph capture: the few-row launch is at most 255 rows, so 256 always do."""
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), stream_of(dev))
    t = _TICKETS.get(key)
    if t is None or t.numel() < n_rows:
        if torch.cuda.is_current_stream_capturing():
            return None  # first use of this stream is under capture: the two-launch form needs no state
        t = _TICKETS[key] = torch.zeros(max(256, n_rows), dtype=torch.int32, device=dev)
    return t


def _forward_rows(rows, code, n_rows, vocab, row_stride, lab, temperature, logprob, entropy, stats, rmask, dev):
    """One forward launch over vocabulary rows. With fewer rows than the GPU has compute units the
    rows are cut into segments (one workgroup each); the workgroup that finishes a row's last segment
    merges the row's partial sums."""
    ws_bytes = _lib.load().orlhf_logprob_entropy_split_workspace_bytes(code, n_rows, vocab)
    if ws_bytes > 0:
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        call("orlhf_logprob_entropy_fwd_split", ptr(rows), code, n_rows, vocab, row_stride, ptr(lab),
             float(temperature), ptr(logprob), ptr(entropy), ptr(stats), ptr(rmask), ptr(ws), ws_bytes,
             ptr(_row_tickets(dev, n_rows)), stream_of(dev))
    else:
        call("orlhf_logprob_entropy_fwd", ptr(rows), code, n_rows, vocab, row_stride, ptr(lab),
             float(temperature), ptr(logprob), ptr(entropy), ptr(stats), ptr(rmask), 0, stream_of(dev))


class _LogprobEntropy(torch.autograd.Function):
    """logits -> (log-prob of label, entropy), one vocabulary pass forward, one backward."""

    @staticmethod
    def forward(ctx, logits, labels, temperature, want_logprob, want_entropy, inplace_backward, row_mask=None):
        dev = require_gpu(logits, labels if want_logprob else None, row_mask)
        code = _lib.dtype_code(logits)
        batch_shape = logits.shape[:-1]
        # a detached alias: shares storage and the version counter with `logits`, but is not a
        # view autograd tracks, so handing it back as the (in-place) gradient is legal
        rows, row_stride, aliases = _as_rows(logits.detach())
        n_rows, vocab = rows.shape
        if want_logprob:
            if labels.shape != batch_shape:
                raise ValueError(f"labels shape {tuple(labels.shape)} != logits batch shape {tuple(batch_shape)}")
            lab = labels.reshape(-1)
            if lab.dtype != torch.int64:
                lab = lab.long()
            lab = lab.contiguous()
        else:
            lab = None
        if row_mask is not None:
            if row_mask.shape != batch_shape:
                raise ValueError(f"row_mask shape {tuple(row_mask.shape)} != logits batch shape {tuple(batch_shape)}")
            rmask = (row_mask != 0).reshape(-1).to(torch.uint8).contiguous()
        else:
            rmask = None
        needs_grad = ctx.needs_input_grad[0]
        opts = dict(device=dev, dtype=torch.float32)
        logprob = torch.empty(n_rows, **opts) if want_logprob else None
        entropy = torch.empty(n_rows, **opts) if want_entropy else None
        stats = torch.empty(n_rows, 4, **opts) if needs_grad else None
        with _lib.on_device(dev):
            _forward_rows(rows, code, n_rows, vocab, row_stride, lab, temperature, logprob, entropy, stats, rmask, dev)
        ctx.temperature = float(temperature)
        ctx.inplace = bool(inplace_backward)
        ctx.row_stride = row_stride
        ctx.shares_storage = aliases
        ctx.logits_shape = logits.shape
        ctx.set_materialize_grads(False)
        if needs_grad:
            ctx.save_for_backward(rows, lab, stats, rmask)
        out_lp = logprob.view(batch_shape) if want_logprob else None
        out_ent = entropy.view(batch_shape) if want_entropy else None
        return out_lp, out_ent

    @staticmethod
    def backward(ctx, g_logprob, g_entropy):
        rows, lab, stats, rmask = ctx.saved_tensors
        if g_logprob is None and g_entropy is None:
            return None, None, None, None, None, None, None
        dev = rows.device
        n_rows, vocab = rows.shape
        code = _lib.dtype_code(rows)
        glp = None if g_logprob is None else g_logprob.reshape(-1).to(torch.float32).contiguous()
        gent = None if g_entropy is None else g_entropy.reshape(-1).to(torch.float32).contiguous()
        if ctx.inplace and ctx.shares_storage:
            grad_rows, grad_stride = rows, ctx.row_stride
        else:
            grad_rows = torch.empty((n_rows, vocab), device=dev, dtype=rows.dtype)
            grad_stride = vocab
        with _lib.on_device(dev):
            call(
                "orlhf_logprob_entropy_bwd", ptr(rows), ptr(grad_rows), code, n_rows, vocab,
                ctx.row_stride, grad_stride, ptr(lab), ctx.temperature, ptr(glp), ptr(gent),
                ptr(stats), ptr(rmask), stream_of(dev),
            )
        if grad_rows is rows:
            # the logits storage now holds the gradient: bump the shared version counter so that
            # any later use of the saved logits by autograd raises instead of reading gradients
            # as logits
            torch.autograd.graph.increment_version(rows)
        grad = grad_rows if grad_rows.shape == ctx.logits_shape else grad_rows.view(ctx.logits_shape)
        return grad, None, None, None, None, None, None


def logprobs_and_entropy_from_logits(
    logits: torch.Tensor,
    labels: torch.Tensor,
    temperature: float = 1.0,
    inplace_backward: bool = False,
    row_mask: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """(log_probs_from_logits(logits, labels, temperature), compute_entropy(logits)) from one
    pass over the logits: the log-prob uses logits / temperature, the entropy the unscaled
    logits, the order Actor.forward applies them in (openrlhf/models/actor.py:269-285).

    ``inplace_backward=True`` writes d(loss)/d(logits) over the logits storage in backward
    instead of allocating a second [N, V] tensor; the logits are unusable afterwards.
    ``row_mask`` (same shape as ``labels``): positions with 0 are skipped, their outputs are 0
    and their logits get zero gradient without being read (prompt and padding positions).
    """
    return _LogprobEntropy.apply(logits, labels, temperature, True, True, inplace_backward, row_mask)


def log_probs_from_logits(
    logits: torch.Tensor,
    labels: torch.Tensor,
    temperature: float = 1.0,
    inplace_backward: bool = False,
    mutate_logits: bool = False,
    out_dtype: Optional[torch.dtype] = None,
) -> torch.Tensor:
    """log_softmax(logits / temperature) gathered at ``labels``
    (openrlhf/models/utils.py:139-163), fp32 result.

    ``mutate_logits=True`` reproduces the reference's side effect for ``temperature != 1``: the
    caller's logits are divided by the temperature in place (rounded to their dtype) and the
    log-prob is taken from the stored quotient, exactly the reference's order of operations.
    It costs an extra read+write of the logits and is for inference-mode callers that read the
    scaled logits afterwards; it refuses tensors that require grad.

    ``out_dtype`` casts the fp32 result (``out_dtype=logits.dtype`` gives the dtype the
    reference's bf16 / fp16 branch returns, computed in fp32 and rounded once)."""
    if mutate_logits and temperature != 1.0:
        if logits.requires_grad and torch.is_grad_enabled():
            raise RuntimeError("mutate_logits=True changes the logits in place and is not tracked by autograd; "
                               "call it under torch.no_grad() or leave mutate_logits=False")
        dev = require_gpu(logits)
        rows, row_stride, aliases = _as_rows(logits.detach())
        if not aliases:
            raise ValueError("mutate_logits=True needs logits whose rows can be addressed in place")
        with _lib.on_device(dev):
            call("orlhf_divide_rows_inplace", ptr(rows), _lib.dtype_code(rows), rows.shape[0], rows.shape[1],
                 row_stride, float(temperature), stream_of(dev))
        torch.autograd.graph.increment_version(rows)
        temperature = 1.0
    out = _LogprobEntropy.apply(logits, labels, temperature, True, False, inplace_backward)[0]
    return out if out_dtype is None or out_dtype == out.dtype else out.to(out_dtype)


def compute_entropy(logits: torch.Tensor, inplace_backward: bool = False) -> torch.Tensor:
    """logsumexp(x) - sum(softmax(x) * x) over the last dim (openrlhf/models/utils.py:182-186),
    fp32 result."""
    return _LogprobEntropy.apply(logits, None, 1.0, False, True, inplace_backward)[1]


# ------------------------------------------------------------------ lm-head + log-prob, logits not stored
def _index_rows(src: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    """src[indices] along the first axis (rows of any width) with the library's gather kernel."""
    src = src.contiguous()
    inner = 1
    for d in src.shape[1:]:
        inner *= d
    out = torch.empty((indices.numel(),) + tuple(src.shape[1:]), dtype=src.dtype, device=src.device)
    with _lib.on_device(src.device):
        call("orlhf_gather_by_indices", ptr(src), src.element_size(), src.shape[0], max(inner, 1), ptr(indices),
             indices.numel(), ptr(out), stream_of(src.device))
    return out


def _scatter_rows(values: torch.Tensor, indices: torch.Tensor, n_dst: int) -> torch.Tensor:
    """zeros(n_dst, ...) with rows ``indices`` set to ``values`` (the library's pad_by_indices)."""
    values = values.contiguous()
    inner = 1
    for d in values.shape[1:]:
        inner *= d
    out = torch.empty((n_dst,) + tuple(values.shape[1:]), dtype=values.dtype, device=values.device)
    with _lib.on_device(values.device):
        call("orlhf_pad_by_indices", ptr(values), values.element_size(), values.shape[0], max(inner, 1), ptr(indices),
             n_dst, ptr(out), stream_of(values.device))
    return out


def _kept_columns(n_rows: int, vocab: int, keep_logits_mib) -> int:
    """How many vocabulary columns of 16-bit logits (whole tiles of 256, row pitch columns + 64) a
    budget in MiB holds for n_rows tokens; None keeps nothing."""
    if not keep_logits_mib or n_rows == 0:
        return 0
    vpad = (vocab + 255) // 256 * 256
    cols = int(keep_logits_mib * (1 << 20)) // (2 * n_rows) - 64
    return max(0, min(vpad, cols // 256 * 256))


class _LmHeadLogprobEntropy(torch.autograd.Function):
    """(hidden states, lm_head weight) -> (log-prob of label, entropy) on matrix-core tiles.
    ``keep`` (int64 row indices or None): only those rows of hidden / labels take part; the outputs
    of the others are 0 and they get zero gradient."""

    @staticmethod
    def forward(ctx, hidden, weight, labels, temperature, backward_chunk_mib=None, keep_logits_mib=None, keep=None):
        dev = require_gpu(hidden, weight, labels, keep)
        ctx.backward_chunk_mib = backward_chunk_mib
        if hidden.dtype != weight.dtype or hidden.dtype not in (torch.bfloat16, torch.float16):
            raise TypeError(f"hidden ({hidden.dtype}) and weight ({weight.dtype}) must both be bfloat16 or float16")
        if hidden.dim() != 2 or weight.dim() != 2 or hidden.shape[1] != weight.shape[1]:
            raise ValueError(f"hidden {tuple(hidden.shape)} and weight {tuple(weight.shape)} must be [N, H] and [V, H]")
        if labels.shape != hidden.shape[:1]:
            raise ValueError(f"labels shape {tuple(labels.shape)} != ({hidden.shape[0]},)")
        h = hidden.detach()
        w = weight.detach()
        lab = labels.to(torch.int64).contiguous()
        n_all = h.shape[0]
        if keep is not None:
            h, lab = _index_rows(h, keep), _index_rows(lab, keep)
        h = h if h.stride(1) == 1 and h.stride(0) % 2 == 0 and h.data_ptr() % 4 == 0 else h.contiguous()
        w = w if w.stride(1) == 1 and w.stride(0) % 2 == 0 and w.data_ptr() % 4 == 0 else w.contiguous()
        n, hdim = h.shape
        vocab = w.shape[0]
        code = _lib.dtype_code(h)
        opts = dict(device=dev, dtype=torch.float32)
        logprob, entropy, stats = torch.empty(n, **opts), torch.empty(n, **opts), torch.empty(n, 4, **opts)
        lib = _lib.load()
        want_grad = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        kept_cols = _kept_columns(n, vocab, keep_logits_mib) if want_grad else 0
        kept = torch.empty((n, kept_cols + 64), dtype=h.dtype, device=dev) if kept_cols > 0 else None
        kept_ld = kept_cols + 64 if kept_cols > 0 else 0
        ws = torch.empty(lib.orlhf_lmhead_workspace_bytes(n, hdim, vocab, kept_cols, 0), dtype=torch.uint8, device=dev)
        with _lib.on_device(dev):
            call("orlhf_lmhead_logprob_entropy_fwd", ptr(h), ptr(w), code, n, hdim, vocab, h.stride(0), w.stride(0),
                 ptr(lab), float(temperature), ptr(logprob), ptr(entropy), ptr(stats), ptr(kept), kept_cols, kept_ld,
                 ptr(ws), ws.numel(), stream_of(dev))
        ctx.temperature = float(temperature)
        ctx.kept, ctx.kept_cols, ctx.kept_ld = kept, kept_cols, kept_ld
        ctx.n_all = n_all
        ctx.set_materialize_grads(False)
        ctx.save_for_backward(h, w, lab, stats, keep)
        if keep is not None:
            logprob, entropy = _scatter_rows(logprob, keep, n_all), _scatter_rows(entropy, keep, n_all)
        return logprob, entropy

    @staticmethod
    def backward(ctx, g_logprob, g_entropy):
        h, w, lab, stats, keep = ctx.saved_tensors
        need_h, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        if (g_logprob is None and g_entropy is None) or not (need_h or need_w):
            return None, None, None, None, None, None, None
        if ctx.kept_cols > 0 and ctx.kept is None:
            raise RuntimeError("the stored logits of this lm-head call were turned into their gradient by an earlier "
                               "backward; call it again (or use keep_logits_mib=None) to differentiate twice")
        dev = h.device
        n, hdim = h.shape
        vocab = w.shape[0]

        def rows(g):
            if g is None:
                return None
            g = g.reshape(-1).to(torch.float32).contiguous()
            return g if keep is None else _index_rows(g, keep)

        glp, gent = rows(g_logprob), rows(g_entropy)
        grad_h = torch.empty((n, hdim), device=dev, dtype=h.dtype) if need_h else None
        grad_w = torch.empty((vocab, hdim), device=dev, dtype=w.dtype) if need_w else None
        lib = _lib.load()
        ws_bytes = lib.orlhf_lmhead_workspace_bytes(n, hdim, vocab, ctx.kept_cols, 1)
        if ctx.backward_chunk_mib is not None and ctx.kept_cols < (vocab + 255) // 256 * 256:
            # the library's default holds 256 MiB of the logits gradient at a time; the entry point
            # takes whatever the workspace offers (whole vocabulary tiles, at most what is not kept)
            floor = lib.orlhf_lmhead_workspace_bytes(n, hdim, 256, 0, 1)
            ws_bytes = max(floor, n * hdim * 4 + 256 + int(ctx.backward_chunk_mib) * (1 << 20))
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        kept, ctx.kept = ctx.kept, None
        with _lib.on_device(dev):
            call("orlhf_lmhead_logprob_entropy_bwd", ptr(h), ptr(w), _lib.dtype_code(h), n, hdim, vocab, h.stride(0),
                 w.stride(0), ptr(lab), ctx.temperature, ptr(glp), ptr(gent), ptr(stats), ptr(kept), ctx.kept_cols,
                 ctx.kept_ld, ptr(grad_h), hdim, ptr(grad_w), hdim, ptr(ws), ws.numel(), stream_of(dev))
        if keep is not None and grad_h is not None:
            grad_h = _scatter_rows(grad_h, keep, ctx.n_all)
        return grad_h, grad_w, None, None, None, None, None


def lm_head_logprobs_and_entropy(
    hidden_states: torch.Tensor,
    lm_head_weight: torch.Tensor,
    labels: torch.Tensor,
    temperature: float = 1.0,
    row_mask: Optional[torch.Tensor] = None,
    backward_chunk_mib: Optional[int] = None,
    keep_logits_mib: Optional[float] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``logits = hidden_states @ lm_head_weight.T`` followed by ``log_probs_from_logits(logits,
    labels, temperature)`` and ``compute_entropy(logits)`` (openrlhf/models/actor.py:263-285 with
    the projection that produces ``output["logits"]``), without the ``[..., V]`` logits being
    stored: matrix-core tiles of the projection are rounded to the 16-bit dtype (as the reference's
    lm_head output is before its fp32 up-cast) and folded into per-token statistics on chip, and
    the backward recomputes them chunk by chunk to produce the gradients of the hidden states and
    of the weight. fp32 results.

    hidden_states ``[..., H]`` and lm_head_weight ``[V, H]`` in bfloat16 or float16; labels
    ``[...]``. ``row_mask`` (same shape as labels): positions with 0 are left out of the projection
    altogether; their outputs are 0 and they receive zero gradient. ``keep_logits_mib``: the forward
    stores the 16-bit logits of as many vocabulary columns as this budget holds (it produces them
    anyway) and the backward recomputes only the others: with everything kept the backward is two
    products instead of three. Results and gradients are the same bits for every budget.
    ``backward_chunk_mib``: how much of the logits gradient of the columns that are NOT kept the
    backward holds at a time (default 256 MiB)."""
    batch_shape = hidden_states.shape[:-1]
    if labels.shape != batch_shape:
        raise ValueError(f"labels shape {tuple(labels.shape)} != hidden batch shape {tuple(batch_shape)}")
    rows = hidden_states.reshape(-1, hidden_states.shape[-1])
    lab = labels.reshape(-1)
    keep = None
    if row_mask is not None:
        if row_mask.shape != batch_shape:
            raise ValueError(f"row_mask shape {tuple(row_mask.shape)} != hidden batch shape {tuple(batch_shape)}")
        from .ring_attn_utils import unpad_indices

        flat = row_mask.reshape(1, -1)
        keep = unpad_indices(flat if flat.dtype in (torch.bool, torch.uint8) else flat != 0)
    lp, ent = _LmHeadLogprobEntropy.apply(rows, lm_head_weight, lab, temperature, backward_chunk_mib, keep_logits_mib, keep)
    return lp.view(batch_shape), ent.view(batch_shape)


# ------------------------------------------------------------------ per-token helpers
def _f32(t: torch.Tensor) -> torch.Tensor:
    """Per-token tensors are consumed as contiguous fp32 (the callers' tensors already are)."""
    if t.dtype != torch.float32:
        t = t.float()
    return t.contiguous()


def _packed(cu_seqlens, max_seqlen):
    """What the mirrors hand down for the packed layout: the boundaries with the caller's bound on
    the longest row (None: measured from the boundaries when the launch is sized)."""
    return None if cu_seqlens is None else (cu_seqlens, max_seqlen)


def _split_packed(cu_seqlens):
    return cu_seqlens if isinstance(cu_seqlens, tuple) else (cu_seqlens, None)


def _rows_of(t: torch.Tensor, cu_seqlens):
    """(n_rows, n_cols) of a padded [..., A] tensor, or of a packed flat tensor + cu_seqlens, where
    n_cols bounds the longest row: it sizes the launch grid and the workspace, so it has to be
    tight. Without the caller's ``max_seqlen`` it is read back from the boundaries (one
    synchronisation)."""
    if cu_seqlens is not None:
        cu, bound = _split_packed(cu_seqlens)
        n_rows = cu.numel() - 1
        if bound is None:
            bound = int((cu[1:] - cu[:-1]).max()) if n_rows > 0 else 1
        return n_rows, max(int(bound), 1)
    if t.dim() == 0:
        return 1, 1
    n_cols = t.shape[-1]
    return (t.numel() // n_cols if n_cols > 0 else 0), n_cols


def _cu_arg(cu_seqlens, dev):
    if cu_seqlens is None:
        return None
    cu, _ = _split_packed(cu_seqlens)
    return cu.to(device=dev, dtype=torch.int64).contiguous()


def _workspace(n_rows, n_cols, dev):
    nbytes = _lib.load().orlhf_token_workspace_bytes(n_rows, n_cols)
    return torch.empty(nbytes, dtype=torch.uint8, device=dev)


class _ApproxKL(torch.autograd.Function):
    @staticmethod
    def forward(ctx, log_probs, log_probs_base, estimator):
        dev = require_gpu(log_probs, log_probs_base)
        if log_probs.dtype == log_probs_base.dtype and log_probs.dtype in _lib._DTYPES:
            lp, base = log_probs.contiguous(), log_probs_base.contiguous()
        else:
            lp, base = _f32(log_probs), _f32(log_probs_base)
        lp, base = torch.broadcast_tensors(lp, base)
        lp, base = lp.contiguous(), base.contiguous()
        out = torch.empty(lp.shape, dtype=torch.float32, device=dev)
        with _lib.on_device(dev):
            call("orlhf_approx_kl_fwd", ptr(lp), ptr(base), _lib.dtype_code(lp), lp.numel(), estimator,
                 ptr(out), stream_of(dev))
        ctx.estimator = estimator
        ctx.in_shapes = (log_probs.shape, log_probs_base.shape)
        ctx.in_dtypes = (log_probs.dtype, log_probs_base.dtype)
        ctx.save_for_backward(lp, base)
        return out

    @staticmethod
    def backward(ctx, g_out):
        lp, base = ctx.saved_tensors
        dev = lp.device
        g_out = _f32(g_out)
        need_lp, need_base = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        g_lp = torch.empty(lp.shape, dtype=torch.float32, device=dev) if need_lp else None
        g_base = torch.empty(lp.shape, dtype=torch.float32, device=dev) if need_base else None
        if need_lp or need_base:
            with _lib.on_device(dev):
                call("orlhf_approx_kl_bwd", ptr(lp), ptr(base), _lib.dtype_code(lp), lp.numel(),
                     ctx.estimator, ptr(g_out), ptr(g_lp), ptr(g_base), stream_of(dev))

        def fit(g, shape, dtype):
            if g is None:
                return None
            if g.shape != shape:
                g = g.sum_to_size(shape)
            return g.to(dtype)

        return fit(g_lp, ctx.in_shapes[0], ctx.in_dtypes[0]), fit(g_base, ctx.in_shapes[1], ctx.in_dtypes[1]), None


def compute_approx_kl(
    log_probs: torch.Tensor,
    log_probs_base: torch.Tensor,
    kl_estimator: str = "k1",
) -> torch.Tensor:
    """k1: d, k2: d^2/2, k3: exp(-d) - 1 + d with d = log_probs - log_probs_base, clamped to
    [-10, 10], fp32 (openrlhf/models/utils.py:64-95). Differentiable."""
    if kl_estimator not in _KL_CODES:
        raise ValueError(f"Unknown kl_estimator: {kl_estimator}")
    return _ApproxKL.apply(log_probs, log_probs_base, _KL_CODES[kl_estimator])


class _Aggregate(torch.autograd.Function):
    """Masked token-mean / sequence-mean / per-row mean of a per-token tensor."""

    @staticmethod
    def forward(ctx, x, mask, mode, dp_size, norm_value, cu_seqlens):
        dev = require_gpu(x, mask)
        xf = _f32(x)
        n_rows, n_cols = _rows_of(xf, cu_seqlens)
        if mask is not None and mask.shape != x.shape:
            mask = mask.expand_as(x)
        mkeep, mptr, mcode = _lib.mask_arg(mask)
        cu = _cu_arg(cu_seqlens, dev)
        keep = []
        norm = _lib.make_norm(dp_size, norm_value, keep)
        ws = _workspace(n_rows, n_cols, dev)
        out = torch.empty(n_rows if mode == _lib.AGG_ROW_MEAN else 1, dtype=torch.float32, device=dev)
        row_coef = torch.empty(max(n_rows, 1), dtype=torch.float32, device=dev)
        with _lib.on_device(dev):
            call("orlhf_masked_aggregate_fwd", ptr(xf), mptr, mcode, n_rows, n_cols, ptr(cu), mode, norm,
                 ptr(ws), ptr(out), ptr(row_coef), stream_of(dev))
        ctx.mode, ctx.dims, ctx.mcode = mode, (n_rows, n_cols), mcode
        ctx.x_shape, ctx.x_dtype = x.shape, x.dtype
        ctx.save_for_backward(mkeep, cu, row_coef)
        if mode == _lib.AGG_ROW_MEAN:
            return out.view(x.shape[:-1]) if cu is None else out
        return out.view(())

    @staticmethod
    def backward(ctx, g_out):
        mkeep, cu, row_coef = ctx.saved_tensors
        dev = row_coef.device
        n_rows, n_cols = ctx.dims
        g = _f32(g_out).reshape(-1)
        g_x = torch.empty(ctx.x_shape, dtype=torch.float32, device=dev)
        with _lib.on_device(dev):
            call("orlhf_masked_aggregate_bwd", ptr(g), ptr(mkeep), ctx.mcode, n_rows, n_cols, ptr(cu), ctx.mode,
                 ptr(row_coef), ptr(g_x), stream_of(dev))
        return g_x.to(ctx.x_dtype), None, None, None, None, None


def masked_mean(tensor: torch.Tensor, mask: Optional[torch.Tensor], dim: int = None) -> torch.Tensor:
    """sum(tensor * mask) / sum(mask) over everything (dim=None) or over `dim`; no epsilon, so
    an all-zero mask gives NaN (openrlhf/models/utils.py:166-169). mask=None is a plain mean."""
    if dim is None:
        return _Aggregate.apply(tensor, mask, _lib.AGG_TOKEN_MEAN, 1, None, None)
    nd = tensor.dim()
    d = dim if dim >= 0 else dim + nd
    if d != nd - 1:
        tensor = tensor.movedim(d, -1)
        if mask is not None:
            mask = mask.expand(torch.broadcast_shapes(mask.shape, tensor.movedim(-1, d).shape)).movedim(d, -1)
    return _Aggregate.apply(tensor, mask, _lib.AGG_ROW_MEAN, 1, None, None)


def compute_reward(
    r: torch.Tensor,
    kl_coef: float,
    kl: torch.Tensor,
    action_mask: Optional[torch.Tensor] = None,
    reward_clip_range: Tuple[float, float] = None,
    cu_seqlens: Optional[torch.Tensor] = None,
    max_seqlen: Optional[int] = None,
) -> torch.Tensor:
    """Per-token reward: -max(kl_coef, 0) * kl everywhere plus the (clipped) scalar reward r[b]
    at row b's last unmasked column (openrlhf/models/utils.py:98-126). Forward only."""
    dev = require_gpu(r, kl, action_mask)
    klf, rf = _f32(kl.detach()), _f32(r.detach()).reshape(-1)
    # one workgroup per row walks the row from its own boundaries: the bound is not used
    cu_seqlens = _packed(cu_seqlens, max_seqlen if max_seqlen is not None else klf.numel())
    n_rows, n_cols = _rows_of(klf, cu_seqlens)
    if rf.numel() != n_rows:
        raise ValueError(f"r has {rf.numel()} entries for {n_rows} rows")
    mkeep, mptr, mcode = _lib.mask_arg(action_mask)
    cu = _cu_arg(cu_seqlens, dev)
    out = torch.empty_like(klf)
    lo, hi = (reward_clip_range[0], reward_clip_range[1]) if reward_clip_range else (0.0, 0.0)
    with _lib.on_device(dev):
        call("orlhf_compute_reward", ptr(rf), float(kl_coef), ptr(klf), mptr, mcode, n_rows, n_cols, ptr(cu),
             1 if reward_clip_range else 0, float(lo), float(hi), ptr(out), None, stream_of(dev))
    return out


@torch.no_grad()
def masked_normalize(tensor: torch.Tensor, mask: torch.Tensor, dim: int = 1, eps: float = 1e-8) -> torch.Tensor:
    """Per-row masked whitening (openrlhf/models/utils.py:172-179): mean and biased variance over
    the unmasked entries along ``dim`` (count clamped to >= 1), result zero at masked entries.
    Forward only: nothing in the reference calls it, it is kept for API completeness."""
    dev = require_gpu(tensor, mask)
    nd = tensor.dim()
    d = dim if dim >= 0 else dim + nd
    x = _f32(tensor.movedim(d, -1)) if d != nd - 1 else _f32(tensor)
    m = mask.expand_as(tensor)
    m = m.movedim(d, -1) if d != nd - 1 else m
    mkeep, mptr, mcode = _lib.mask_arg(m)
    n_cols = x.shape[-1]
    n_rows = x.numel() // n_cols if n_cols else 0
    out = torch.empty_like(x)
    with _lib.on_device(dev):
        call("orlhf_masked_normalize_rows", ptr(x), mptr, mcode, n_rows, n_cols, None, float(eps), ptr(out),
             stream_of(dev))
    out = out.movedim(-1, d) if d != nd - 1 else out
    return out.to(tensor.dtype)


# ------------------------------------------------------------------ one-pass forward + backward
@torch.no_grad()
def fused_logprob_entropy_fwd_bwd(
    logits: torch.Tensor,
    labels: torch.Tensor,
    w_logprob: Optional[torch.Tensor] = None,
    w_entropy: Optional[torch.Tensor] = None,
    temperature: float = 1.0,
    inplace: bool = True,
    row_mask: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Forward and backward of ``logprobs_and_entropy_from_logits`` in one pass over the logits
    for a loss that is linear in the outputs: ``loss = sum(w_logprob * logprob) + sum(w_entropy *
    entropy)`` with weights known up front (SFT: ``w_logprob = -mask / n_tokens``). Returns
    ``(logprob, entropy, d loss / d logits)``; with ``inplace=True`` the gradient overwrites the
    logits storage. Every row is read once and written once (2 x V x itemsize bytes per token
    instead of 3 x); rows that do not fit on one CU take the separate forward and backward
    kernels, with the same results. Not an autograd function: the gradient is returned."""
    dev = require_gpu(logits, labels, w_logprob, w_entropy, row_mask)
    code = _lib.dtype_code(logits)
    batch_shape = logits.shape[:-1]
    rows, row_stride, shares = _as_rows(logits.detach())
    n_rows, vocab = rows.shape
    if labels.shape != batch_shape:
        raise ValueError(f"labels shape {tuple(labels.shape)} != logits batch shape {tuple(batch_shape)}")
    lab = labels.reshape(-1).to(torch.int64).contiguous()

    def flat(t, name):
        if t is None:
            return None
        if t.shape != batch_shape:
            raise ValueError(f"{name} shape {tuple(t.shape)} != logits batch shape {tuple(batch_shape)}")
        return t.reshape(-1).to(torch.float32).contiguous()

    wlp, went = flat(w_logprob, "w_logprob"), flat(w_entropy, "w_entropy")
    rmask = None if row_mask is None else (row_mask != 0).reshape(-1).to(torch.uint8).contiguous()
    opts = dict(device=dev, dtype=torch.float32)
    logprob, entropy = torch.empty(n_rows, **opts), torch.empty(n_rows, **opts)
    if inplace and shares:
        grad_rows, grad_stride = rows, row_stride
    else:
        grad_rows, grad_stride = torch.empty((n_rows, vocab), device=dev, dtype=rows.dtype), vocab
    lib = _lib.load()
    fits = vocab <= lib.orlhf_logprob_entropy_fwd_bwd_max_vocab(code)
    same_phase = ((rows.data_ptr() ^ grad_rows.data_ptr()) & 15) == 0 and (
        ((row_stride - grad_stride) * rows.element_size()) & 15
    ) == 0
    with _lib.on_device(dev):
        few_rows = lib.orlhf_logprob_entropy_split_workspace_bytes(code, n_rows, vocab) > 0
        if fits and same_phase and not few_rows:
            call("orlhf_logprob_entropy_fwd_bwd", ptr(rows), ptr(grad_rows), code, n_rows, vocab, row_stride,
                 grad_stride, ptr(lab), float(temperature), ptr(wlp), ptr(went), ptr(logprob), ptr(entropy),
                 ptr(rmask), stream_of(dev))
        else:
            stats = torch.empty(n_rows, 4, **opts)
            zeros = torch.zeros(n_rows, **opts)
            _forward_rows(rows, code, n_rows, vocab, row_stride, lab, temperature, logprob, entropy, stats, rmask, dev)
            call("orlhf_logprob_entropy_bwd", ptr(rows), ptr(grad_rows), code, n_rows, vocab, row_stride,
                 grad_stride, ptr(lab), float(temperature), ptr(wlp if wlp is not None else zeros),
                 ptr(went if went is not None else zeros), ptr(stats), ptr(rmask), stream_of(dev))
    if grad_rows is rows:
        torch.autograd.graph.increment_version(rows)
    grad = grad_rows if grad_rows.shape == logits.shape else grad_rows.view(logits.shape)
    return logprob.view(batch_shape), entropy.view(batch_shape), grad

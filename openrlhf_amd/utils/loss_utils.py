"""Loss normalisers with the signatures of ``openrlhf.utils.loss_utils`` (single process).

Mirrors openrlhf/utils/loss_utils.py:15-105: ``get_loss_batch_info`` and
``iter_grad_accum_global_norm`` produce ``dp_size``, ``batch_num_tokens`` (unmasked tokens) and
``global_batch_size`` (sequences with at least one unmasked token) that ``aggregate_loss`` and the
losses consume. The counts come from one HIP reduction over the mask and stay on the device as
0-dim fp32 tensors, which the loss kernels read without a host synchronisation.

One GPU is built: the reference's all-reduce over the data-parallel group (:35,43,75,76) would be
two scalar SUM all-reduces of these device tensors; with more than one rank initialised these
functions raise instead of returning local counts under a global name.
"""
from typing import Optional

import torch
import torch.distributed as dist

from .. import _lib
from .._lib import call, ptr, stream_of
from ..models.utils import _workspace


def _require_single_process():
    if dist.is_available() and dist.is_initialized() and dist.get_world_size() > 1:
        raise NotImplementedError("openrlhf_amd.utils.loss_utils counts one process's batch only; the data-parallel "
                                  "all-reduce of the two counts is not part of this build")


def mask_counts(loss_mask: torch.Tensor):
    """(sum(mask), number of rows with sum(mask) > 0) as two 0-dim fp32 device tensors."""
    dev = _lib.require_gpu(loss_mask)
    rows = loss_mask.reshape(loss_mask.shape[0], -1) if loss_mask.dim() != 2 else loss_mask
    b, a = rows.shape
    mkeep, mptr, mcode = _lib.mask_arg(rows)
    ws = _workspace(b, a, dev)
    out = torch.empty(2, dtype=torch.float32, device=dev)
    with _lib.on_device(dev):
        call("orlhf_mask_counts", mptr, mcode, b, a, None, ptr(ws), ptr(out), stream_of(dev))
    return out[0], out[1]


def get_loss_batch_info(
    strategy,
    loss_mask: torch.Tensor,
    *,
    replay_buffer=None,
    step: Optional[int] = None,
    dynamic_batch: bool = False,
    batch_num_tokens: Optional[float] = None,
    global_batch_size: Optional[float] = None,
):
    """openrlhf/utils/loss_utils.py:15-52 for one process: the dict ``aggregate_loss`` takes."""
    _require_single_process()
    if dynamic_batch and replay_buffer is not None and step is not None:
        batch_num_tokens = replay_buffer.dynamic_batch_num_tokens[step]
        global_batch_size = replay_buffer.dynamic_global_batch_size[step]
    tokens = samples = None
    if batch_num_tokens is None or global_batch_size is None:
        tokens, samples = mask_counts(loss_mask)
    as_t = lambda v: torch.as_tensor(v, device=loss_mask.device, dtype=torch.float32)  # noqa: E731
    return {
        "dp_size": 1,
        "batch_num_tokens": tokens if batch_num_tokens is None else as_t(batch_num_tokens),
        "global_batch_size": samples if global_batch_size is None else as_t(global_batch_size),
    }


def iter_grad_accum_global_norm(data_iter, strategy, accumulated_gradient, mask_fn):
    """openrlhf/utils/loss_utils.py:80-105: yields ``(item, info)`` where every micro-batch of one
    optimizer step (a window of ``accumulated_gradient`` items) gets the same normalisers, the
    window totals divided by the window length, so that the engine's 1/gas loss scaling turns the
    accumulated loss into one mean over the whole step."""
    _require_single_process()
    gas = max(int(accumulated_gradient), 1)

    def window_info(window):
        tokens = samples = None
        for it in window:
            t, s = mask_counts(mask_fn(it))
            tokens = t if tokens is None else tokens + t
            samples = s if samples is None else samples + s
        return {"dp_size": 1, "batch_num_tokens": tokens / gas, "global_batch_size": samples / gas}

    window = []
    for item in data_iter:
        window.append(item)
        if len(window) == gas:
            info = window_info(window)
            for it in window:
                yield it, info
            window = []
    if window:
        info = window_info(window)
        for it in window:
            yield it, info

"""Advantage functions of the experience maker on hand-written HIP kernels.

Mirrors (paths relative to the OpenRLHF tree, all in
openrlhf/trainer/ppo_utils/experience_maker.py):
  compute_advantages_and_returns   :237-330  (group baseline :246-272, per-experience reward and
                                              GAE / returns :275-312, global whitening :314-328)
  get_advantages_and_returns       :332-377  (GAE)
  get_cumulative_returns           :379-411  (discounted reward-to-go)

The reference runs these on the controller's CPU with Python loops over time. Here every
function is a GPU kernel launch; tensors that arrive on the CPU (the reference's experiences
are CPU tensors) are copied to the current GPU, processed there and the results copied back to
where the inputs lived, so callers see the same devices as before. There is no CPU compute path:
without a GPU the functions raise.

Only the numerics are mirrored. Length penalties (apply_length_penalties) and the Ray dispatch
half of RemoteExperienceMaker are outside this package; ``compute_advantages_and_returns`` takes a
``length_penalty_fn`` hook for the former.
"""
import ctypes
import itertools
from typing import List, Optional, Tuple

import torch

from ... import _lib
from ..._lib import call, ptr, stream_of
from ...models.utils import _KL_CODES, _cu_arg, _f32, _packed, _rows_of

_GROUP_CODES = {
    "gae": _lib.GROUP_IDENTITY,
    "reinforce": _lib.GROUP_IDENTITY,
    "rloo": _lib.GROUP_RLOO,
    "reinforce_baseline": _lib.GROUP_BASELINE,
    "dr_grpo": _lib.GROUP_BASELINE,
    "group_norm": _lib.GROUP_NORM,
}
# whiten_advantages: lists longer than this are gathered into one array first (measured: 512 blocks
# of 131 072 tokens 5.6 ms block by block against 0.8 ms gathered; 8 blocks 0.18 ms against 0.34 ms)
_WHITEN_GATHER_ABOVE = 32
_RETURN_ESTIMATORS = ("reinforce", "rloo", "reinforce_baseline", "group_norm", "dr_grpo")


def _gpu_device() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("openrlhf_amd needs a GPU: the advantage functions are HIP kernels, there is no CPU path")
    return torch.device("cuda", torch.cuda.current_device())


def _on_gpu(t: Optional[torch.Tensor], dev: torch.device) -> Optional[torch.Tensor]:
    if t is None or t.is_cuda:
        return t
    return t.to(dev)


def _device_for(*tensors) -> Tuple[torch.device, torch.device]:
    """(GPU to compute on, device the results go back to)."""
    home = next(t.device for t in tensors if t is not None)
    gpu = next((t.device for t in tensors if t is not None and t.is_cuda), None)
    return (gpu if gpu is not None else _gpu_device()), home


@torch.no_grad()
def experience_kl(
    action_log_probs: torch.Tensor,
    base_action_log_probs: Optional[torch.Tensor],
    action_mask: Optional[torch.Tensor],
    kl_estimator: str = "k1",
    cu_seqlens: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """The KL block of ``make_experience`` (experience_maker.py:202-216) in one pass over the
    log-probs: ``(kl, kl_mean, logprobs_diff_mean)`` with ``kl = compute_approx_kl(lp, base)``,
    ``kl_mean = masked_mean(kl, mask, dim=-1)`` and the masked row mean of ``lp - base``.
    ``base_action_log_probs=None`` is the branch without a reference model (or with the KL taken
    as a loss): zeros, and means of zeros."""
    if kl_estimator not in _KL_CODES:
        raise ValueError(f"Unknown kl_estimator: {kl_estimator}")
    dev, home = _device_for(action_log_probs, base_action_log_probs, action_mask)
    lp = _on_gpu(action_log_probs, dev)
    enabled = base_action_log_probs is not None
    if enabled:
        base = _on_gpu(base_action_log_probs, dev)
        if lp.dtype == base.dtype and lp.dtype in _lib._DTYPES:
            lp, base = lp.contiguous(), base.contiguous()
        else:
            lp, base = _f32(lp), _f32(base)
        if base.shape != lp.shape:
            raise ValueError(f"log-prob shapes differ: {tuple(lp.shape)} vs {tuple(base.shape)}")
    else:
        lp, base = lp.contiguous(), None
    mkeep, mptr, mcode = _lib.mask_arg(_on_gpu(action_mask, dev))
    n_rows, n_cols = _rows_of(lp, _packed(cu_seqlens, lp.numel()))
    cu = _cu_arg(cu_seqlens, dev)
    kl = torch.empty(lp.shape, dtype=torch.float32, device=dev)
    kl_mean = torch.empty(n_rows, dtype=torch.float32, device=dev)
    diff_mean = torch.empty(n_rows, dtype=torch.float32, device=dev)
    code = _lib.dtype_code(lp) if enabled else _lib.F32
    with _lib.on_device(dev):
        call("orlhf_kl_rows", ptr(lp) if enabled else None, ptr(base), code, mptr, mcode, n_rows, n_cols, ptr(cu),
             _KL_CODES[kl_estimator], 1 if enabled else 0, ptr(kl), ptr(kl_mean), ptr(diff_mean), stream_of(dev))
    if not enabled:  # the reference keeps the log-prob dtype for its zeros
        kl = kl.to(action_log_probs.dtype)
    return kl.to(home), kl_mean.to(home), diff_mean.to(home)


def _order_arg(row_order, n_rows, dev):
    """A row permutation as the kernels take it (int64 on the device), or None. The kernels trust it:
    a row that it does not name keeps whatever its outputs held. An order that arrives on the host
    is checked here (sorting it must give 0 .. n_rows - 1); one that is already on the device
    (``PackedSteps.longest_first`` builds it there with a sort) is not read back."""
    if row_order is None:
        return None
    if row_order.numel() != n_rows:
        raise ValueError(f"row_order has {row_order.numel()} entries for {n_rows} rows")
    if row_order.device.type == "cpu":
        if not torch.equal(torch.sort(row_order.reshape(-1).to(torch.int64)).values, torch.arange(n_rows, dtype=torch.int64)):
            raise ValueError("row_order is not a permutation of the rows")
    return row_order.to(device=dev, dtype=torch.int64).contiguous()


@torch.no_grad()
def get_advantages_and_returns(
    values: torch.Tensor,
    rewards: torch.Tensor,
    action_mask: Optional[torch.Tensor],
    gamma: float,
    lambd: float,
    cu_seqlens: Optional[torch.Tensor] = None,
    max_seqlen: Optional[int] = None,
    row_order: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """GAE (experience_maker.py:332-377): with v = mask*values, r = mask*rewards,
    delta_t = r_t + gamma*v_{t+1} - v_t, A_t = delta_t + gamma*lambd*A_{t+1}; returns = A + v.
    Every column of the [B, A] block takes part and the outputs are not re-masked.
    ``row_order`` (int64 permutation of the rows, e.g. ``PackedSteps.longest_first``): the order
    rows are handed to workgroups in; it changes the schedule of a ragged batch, never a result."""
    dev, home = _device_for(values, rewards, action_mask)
    v, r = _f32(_on_gpu(values, dev)), _f32(_on_gpu(rewards, dev))
    mkeep, mptr, mcode = _lib.mask_arg(_on_gpu(action_mask, dev))
    # the scans walk each row from its own boundaries: the bound on the row length is not used
    n_rows, n_cols = _rows_of(v, _packed(cu_seqlens, max_seqlen if max_seqlen is not None else v.numel()))
    cu = _cu_arg(cu_seqlens, dev)
    adv, ret = torch.empty_like(v), torch.empty_like(v)
    with _lib.on_device(dev):
        call("orlhf_gae_scan", ptr(v), ptr(r), mptr, mcode, n_rows, n_cols, ptr(cu), ptr(_order_arg(row_order, n_rows, dev)),
             float(gamma), float(lambd), ptr(adv), ptr(ret), stream_of(dev))
    return adv.to(home), ret.to(home)


@torch.no_grad()
def get_cumulative_returns(
    rewards: torch.Tensor,
    action_mask: Optional[torch.Tensor],
    gamma: float,
    cu_seqlens: Optional[torch.Tensor] = None,
    max_seqlen: Optional[int] = None,
    row_order: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Discounted reward-to-go G_t = mask_t*r_t + gamma*G_{t+1} (experience_maker.py:379-411)."""
    dev, home = _device_for(rewards, action_mask)
    r = _f32(_on_gpu(rewards, dev))
    mkeep, mptr, mcode = _lib.mask_arg(_on_gpu(action_mask, dev))
    n_rows, n_cols = _rows_of(r, _packed(cu_seqlens, max_seqlen if max_seqlen is not None else r.numel()))
    cu = _cu_arg(cu_seqlens, dev)
    ret = torch.empty_like(r)
    with _lib.on_device(dev):
        call("orlhf_discounted_returns", ptr(r), mptr, mcode, n_rows, n_cols, ptr(cu), ptr(_order_arg(row_order, n_rows, dev)),
             float(gamma), ptr(ret), stream_of(dev))
    return ret.to(home)


@torch.no_grad()
def reward_advantages_and_returns(
    r: torch.Tensor,
    kl_coef: float,
    kl: torch.Tensor,
    values: Optional[torch.Tensor],
    action_mask: Optional[torch.Tensor],
    gamma: float,
    lambd: float = 1.0,
    reward_clip_range: Optional[Tuple[float, float]] = None,
    cu_seqlens: Optional[torch.Tensor] = None,
    row_order: Optional[torch.Tensor] = None,
) -> Tuple[Optional[torch.Tensor], torch.Tensor, torch.Tensor]:
    """``compute_reward`` followed by GAE (``values`` given) or by the discounted returns
    (``values=None``) in one pass that never stores the per-token reward: the per-experience body
    of compute_advantages_and_returns (experience_maker.py:276-312). Returns ``(advantages,
    returns, reward_sum)``; ``advantages`` is None without values (the reference clones the
    returns there) and ``reward_sum[b]`` is the per-token reward summed over every column, the
    reference's ``info["return"]``. Same numbers as the two separate calls."""
    dev, home = _device_for(r, kl, values, action_mask)
    klf = _f32(_on_gpu(kl, dev))
    rf = _f32(_on_gpu(r, dev)).reshape(-1)
    v = None if values is None else _f32(_on_gpu(values, dev))
    if v is not None and v.shape != klf.shape:
        raise ValueError(f"values {tuple(v.shape)} do not match kl {tuple(klf.shape)}")
    mkeep, mptr, mcode = _lib.mask_arg(_on_gpu(action_mask, dev))
    n_rows, n_cols = _rows_of(klf, _packed(cu_seqlens, klf.numel()))
    if rf.numel() != n_rows:
        raise ValueError(f"r has {rf.numel()} entries for {n_rows} rows")
    cu = _cu_arg(cu_seqlens, dev)
    adv = None if v is None else torch.empty_like(klf)
    ret = torch.empty_like(klf)
    total = torch.empty(n_rows, dtype=torch.float32, device=dev)
    lo, hi = (reward_clip_range[0], reward_clip_range[1]) if reward_clip_range else (0.0, 0.0)
    with _lib.on_device(dev):
        call("orlhf_reward_scan", ptr(rf), float(kl_coef), ptr(klf), ptr(v), mptr, mcode, n_rows, n_cols, ptr(cu),
             ptr(_order_arg(row_order, n_rows, dev)), 1 if reward_clip_range else 0, float(lo), float(hi), float(gamma), float(lambd), ptr(adv), ptr(ret),
             ptr(total), stream_of(dev))
    return (None if adv is None else adv.to(home)), ret.to(home), total.to(home)


@torch.no_grad()
def group_normalize_rewards(
    rewards: torch.Tensor,
    indices: Optional[torch.Tensor],
    n_samples_per_prompt: int,
    estimator: str,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Group baseline / normalisation of scalar rewards (experience_maker.py:246-272).

    rewards: [P*n] in experience order; indices[i] = position of sample i in prompt order (None:
    already in prompt order), so samples whose positions fall in one block of n share a prompt.
    rloo: r - mean of the other n-1; reinforce_baseline / dr_grpo: r - group mean; group_norm:
    (r - mean) / (unbiased std + 1e-9); gae / reinforce: unchanged. Returns (shaped rewards in
    experience order, the unbiased group std per sample or None when n == 1)."""
    if estimator not in _GROUP_CODES:
        raise Exception(f"Unkown advantage_estimator {estimator}")
    dev, home = _device_for(rewards)
    r = _f32(_on_gpu(rewards, dev)).reshape(-1)
    n_total = r.numel()
    n = int(n_samples_per_prompt)
    if n < 1 or n_total % n != 0:
        raise ValueError(f"{n_total} rewards do not split into groups of {n}")
    idx = None if indices is None else _on_gpu(indices, dev).to(torch.int64).contiguous()
    out = torch.empty_like(r)
    std = torch.empty_like(r) if n > 1 else None
    ws = torch.empty(max(n_total, 1), dtype=torch.float32, device=dev)
    with _lib.on_device(dev):
        call("orlhf_group_normalize", ptr(r), ptr(idx), n_total // n, n, _GROUP_CODES[estimator], ptr(out), ptr(std),
             ptr(ws), stream_of(dev))
    return out.to(home), (None if std is None else std.to(home))


@torch.no_grad()
def whiten_advantages(
    advantages: List[torch.Tensor],
    action_masks: List[torch.Tensor],
    no_std_norm: bool = False,
) -> List[torch.Tensor]:
    """Global masked whitening over all experiences (experience_maker.py:314-328): mean and
    biased variance over the unmasked tokens of every block, rstd = rsqrt(max(var, 1e-8)) (1 when
    no_std_norm); (adv - mean) * rstd is applied to every column, masked or not."""
    dev, home = _device_for(*advantages)
    if len(advantages) > _WHITEN_GATHER_ABOVE:
        # many small blocks: per-block host work would outweigh the copy that gathering costs
        flat = torch.cat([_on_gpu(a, dev).reshape(-1) for a in advantages]).float()
        mask = torch.cat([_on_gpu(m if m.shape == a.shape else m.expand_as(a), dev).reshape(-1)
                          for m, a in zip(action_masks, advantages)])
        pieces = whiten_advantages([flat], [mask], no_std_norm)[0].split([a.numel() for a in advantages])
        out = [p.view(a.shape) for p, a in zip(pieces, advantages)]
        return out if home == dev else [o.to(home) for o in out]
    xs = [_f32(_on_gpu(a, dev)) for a in advantages]
    masks = [_lib.mask_arg(_on_gpu(m, dev).expand_as(a)) for m, a in zip(action_masks, advantages)]
    if len(xs) == 1:  # one array: the flat entry (a fixed grid, 10 % faster than the block list of one)
        x, (mkeep, mptr, mcode) = xs[0], masks[0]
        out = torch.empty_like(x)
        ws = torch.empty(_lib.load().orlhf_whiten_workspace_bytes(x.numel()), dtype=torch.uint8, device=dev)
        with _lib.on_device(dev):
            call("orlhf_masked_whiten", ptr(x), mptr, mcode, x.numel(), 0 if no_std_norm else 1, ptr(ws), ptr(out), None,
                 stream_of(dev))
        return [out.view(advantages[0].shape).to(home)]
    codes = {code for _, _, code in masks}
    if len(codes) != 1:  # mixed mask dtypes: whiten with float masks
        masks = [_lib.mask_arg(_on_gpu(m, dev).expand_as(a).float()) for m, a in zip(action_masks, advantages)]
    mcode = masks[0][2]
    k = len(xs)
    ns = (ctypes.c_int64 * k)(*[x.numel() for x in xs])
    outs = [torch.empty_like(x) for x in xs]
    ws = torch.empty(_lib.load().orlhf_whiten_multi_workspace_bytes(ns, k), dtype=torch.uint8, device=dev)
    x_ptrs = (ctypes.c_void_p * k)(*[x.data_ptr() for x in xs])
    m_ptrs = (ctypes.c_void_p * k)(*[mp for _, mp, _ in masks])
    o_ptrs = (ctypes.c_void_p * k)(*[o.data_ptr() for o in outs])
    with _lib.on_device(dev):
        call("orlhf_masked_whiten_multi", x_ptrs, m_ptrs, mcode, ns, k, 0 if no_std_norm else 1, ptr(ws), o_ptrs,
             None, stream_of(dev))
    return [o.view(a.shape).to(home) for o, a in zip(outs, advantages)]


@torch.no_grad()
def compute_advantages_and_returns(
    experiences: list,
    *,
    advantage_estimator: str,
    n_samples_per_prompt: int,
    kl_coef: float,
    gamma: float = 1.0,
    lambd: float = 1.0,
    reward_clip_range: Optional[Tuple[float, float]] = None,
    no_std_norm: bool = False,
    length_penalty_fn=None,
) -> list:
    """The numerics of RemoteExperienceMaker.compute_advantages_and_returns
    (experience_maker.py:237-330) on a list of experience objects with the attributes the
    reference reads and writes: index, rewards, kl, action_mask, values, info, advantages,
    returns. Group baseline over prompts, per-token reward (compute_reward), GAE or discounted
    returns, then global whitening for gae / reinforce / reinforce_baseline."""
    if length_penalty_fn is not None:
        length_penalty_fn(experiences)
    exp_len = [len(e.index) for e in experiences]
    indices = torch.tensor(list(itertools.chain.from_iterable(e.index for e in experiences)), dtype=torch.int64)
    raw = torch.cat([e.rewards for e in experiences], dim=0)
    shaped, group_std = group_normalize_rewards(raw, indices.to(raw.device), n_samples_per_prompt, advantage_estimator)
    if group_std is not None:
        for e, s in zip(experiences, group_std.split(exp_len)):
            e.info["group_reward_std"] = s

    if advantage_estimator != "gae" and advantage_estimator not in _RETURN_ESTIMATORS:
        raise Exception(f"Unkown advantage_estimator {advantage_estimator}")
    dev = _gpu_device()
    for e, reward in zip(experiences, shaped.split(exp_len)):
        home = e.kl.device
        if advantage_estimator == "gae":
            values, g, lam = _on_gpu(e.values, dev), gamma, lambd
        else:
            values, lam = None, 1.0
            g = gamma if advantage_estimator == "reinforce" else 1.0  # the reference forces gamma = 1 here
        # per-token reward, scan and the row sums of the reward in one pass over kl
        adv, ret, total = reward_advantages_and_returns(
            _on_gpu(reward, dev), kl_coef, _on_gpu(e.kl, dev), values, _on_gpu(e.action_mask, dev), g, lam,
            reward_clip_range=reward_clip_range,
        )
        e.returns = ret.to(home)
        e.advantages = e.returns.clone() if adv is None else adv.to(home)
        e.info["return"] = total.to(home)
        e.kl = None

    if advantage_estimator in ("gae", "reinforce", "reinforce_baseline"):
        whitened = whiten_advantages([e.advantages for e in experiences], [e.action_mask for e in experiences],
                                     no_std_norm=no_std_norm)
        for e, a in zip(experiences, whitened):
            e.advantages = a
    return experiences


class AdvantageFunctions:
    """The three advantage methods of RemoteExperienceMaker with their reference signatures, for
    code that calls them as bound methods. ``strategy.args`` and ``kl_ctl`` are read the way the
    reference reads them (experience_maker.py:240-330)."""

    def __init__(self, strategy=None, kl_ctl=None, length_penalty_fn=None):
        self.strategy = strategy
        self.kl_ctl = kl_ctl
        self.length_penalty_fn = length_penalty_fn
        self.advantage_estimator = None if strategy is None else strategy.args.algo.advantage.estimator

    def get_advantages_and_returns(self, values, rewards, action_mask, gamma, lambd):
        return get_advantages_and_returns(values, rewards, action_mask, gamma, lambd)

    def get_cumulative_returns(self, rewards, action_mask, gamma):
        return get_cumulative_returns(rewards, action_mask, gamma)

    def compute_advantages_and_returns(self, experiences):
        args = self.strategy.args
        return compute_advantages_and_returns(
            experiences,
            advantage_estimator=args.algo.advantage.estimator,
            n_samples_per_prompt=args.rollout.n_samples_per_prompt,
            kl_coef=self.kl_ctl.value,
            gamma=args.algo.advantage.gamma,
            lambd=args.algo.advantage.lambd,
            reward_clip_range=args.reward.clip_range,
            no_std_norm=args.algo.advantage.no_std_norm,
            length_penalty_fn=self.length_penalty_fn,
        )

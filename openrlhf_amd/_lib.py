"""ctypes binding of libopenrlhf_amd.so (the C ABI declared in include/openrlhf_amd.h).

There is no CPU or pure-torch fallback: if the shared library has not been built, or a tensor
is not on a GPU, the call raises. Build with ``python -m openrlhf_amd.csrc.build``.
"""
import ctypes
import math
import os
from ctypes import POINTER, Structure, c_char_p, c_double, c_float, c_int, c_int64, c_uint64, c_void_p

import torch

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libopenrlhf_amd.so")

# enums of include/openrlhf_amd.h
F32, BF16, F16 = 0, 1, 2
MASK_NONE, MASK_U8, MASK_F32, MASK_I64 = 0, 1, 2, 3
KL_K1, KL_K2, KL_K3 = 0, 1, 2
AGG_TOKEN_MEAN, AGG_SEQ_MEAN, AGG_ROW_MEAN, AGG_SEQ_MEAN_TOKEN_SUM = 0, 1, 2, 3
POLICY_PPO, POLICY_GSPO = 0, 1
IS_NONE, IS_TIS, IS_ICEPOP, IS_SEQ_MASK_TIS = 0, 1, 2, 3
GROUP_IDENTITY, GROUP_RLOO, GROUP_BASELINE, GROUP_NORM = 0, 1, 2, 3
PAIR_DPO_SIGMOID, PAIR_DPO_IPO, PAIR_LOGSIGMOID, PAIR_LOGEXP = 0, 1, 2, 3

ABI_VERSION = 23
UNPAD_TILE = 2048  # ORLHF_UNPAD_TILE


class Norm(Structure):
    _fields_ = [("dp_size", c_double), ("norm_value", c_double), ("norm_dev", c_void_p)]


class PolicyParams(Structure):
    _fields_ = [
        ("clip_eps_low", c_float),
        ("clip_eps_high", c_float),
        ("dual_clip", c_float),
        ("policy_type", c_int),
        ("is_correction", c_int),
        ("is_low", c_float),
        ("is_high", c_float),
        ("token_level", c_int),
        ("norm", Norm),
    ]


class PackField(Structure):
    _fields_ = [("src", c_void_p), ("dst", c_void_p), ("elem_bytes", c_int)]


class StepTerms(Structure):
    _fields_ = [
        ("old_log_probs", c_void_p),
        ("advantages", c_void_p),
        ("rollout_log_probs", c_void_p),
        ("base_log_probs", c_void_p),
        ("policy_coef", c_void_p),
        ("token_coef", c_void_p),
        ("clip_eps_low", c_float),
        ("clip_eps_high", c_float),
        ("dual_clip", c_float),
        ("is_correction", c_int),
        ("is_low", c_float),
        ("is_high", c_float),
        ("kl_estimator", c_int),
        ("kl_coef", c_float),
        ("entropy_coef", c_float),
    ]


P = c_void_p
I64 = c_int64

# name -> (restype, argtypes); every symbol the header declares
SIGNATURES = {
    "orlhf_version": (c_int, []),
    "orlhf_last_error": (c_char_p, []),
    "orlhf_logprob_entropy_fwd": (c_int, [P, c_int, I64, I64, I64, P, c_double, P, P, P, P, c_int, P]),
    "orlhf_logprob_entropy_split_workspace_bytes": (I64, [c_int, I64, I64]),
    "orlhf_logprob_entropy_fwd_split": (c_int, [P, c_int, I64, I64, I64, P, c_double, P, P, P, P, P, I64, P, P]),
    "orlhf_divide_rows_inplace": (c_int, [P, c_int, I64, I64, I64, c_double, P]),
    "orlhf_logprob_entropy_bwd": (c_int, [P, P, c_int, I64, I64, I64, I64, P, c_double, P, P, P, P, P]),
    "orlhf_logprob_entropy_fwd_bwd_max_vocab": (I64, [c_int]),
    "orlhf_logprob_entropy_fwd_bwd": (c_int, [P, P, c_int, I64, I64, I64, I64, P, c_double, P, P, P, P, P, P]),
    "orlhf_lmhead_workspace_bytes": (I64, [I64, I64, I64, I64, c_int]),
    "orlhf_lmhead_logprob_entropy_fwd": (c_int, [P, P, c_int, I64, I64, I64, I64, I64, P, c_double, P, P, P, P, I64, I64,
                                                 P, I64, P]),
    "orlhf_lmhead_logprob_entropy_bwd": (c_int, [P, P, c_int, I64, I64, I64, I64, I64, P, c_double, P, P, P, P, I64, I64,
                                                 P, I64, P, I64, P, I64, P]),
    "orlhf_matrix_tile_product": (c_int, [P, P, c_int, I64, I64, I64, I64, I64, c_int, c_int, c_int, P, I64, P]),
    "orlhf_matrix_tile_probe": (c_int, [P, P, c_int, I64, I64, I64, I64, I64, c_int, P, P]),
    "orlhf_policy_step_fwd_bwd": (c_int, [P, P, c_int, I64, I64, I64, I64, P, c_double, POINTER(StepTerms), P, P, P, P]),
    "orlhf_actor_step_gather": (c_int, [P, P, c_int, P, I64, I64, I64, I64, P, P, P, P, P, P, c_float, P, P, P, P, P, P, P, P,
                                        P, P]),
    "orlhf_actor_step_values_workspace_bytes": (I64, [I64]),
    "orlhf_actor_step_values": (c_int, [P, P, P, P, P, P, P, P, P, P, I64, I64, I64, POINTER(StepTerms), c_float, c_int, P, P,
                                        P, P, P]),
    "orlhf_rescale_inplace_if": (c_int, [P, c_int, I64, P, c_float, P]),
    "orlhf_approx_kl_fwd": (c_int, [P, P, c_int, I64, c_int, P, P]),
    "orlhf_approx_kl_bwd": (c_int, [P, P, c_int, I64, c_int, P, P, P, P]),
    "orlhf_token_workspace_bytes": (I64, [I64, I64]),
    "orlhf_masked_aggregate_fwd": (c_int, [P, P, c_int, I64, I64, P, c_int, POINTER(Norm), P, P, P, P]),
    "orlhf_mask_counts": (c_int, [P, c_int, I64, I64, P, P, P, P]),
    "orlhf_mask_row_coef": (c_int, [P, c_int, I64, I64, c_int, POINTER(Norm), P, P, P]),
    "orlhf_masked_aggregate_bwd": (c_int, [P, P, c_int, I64, I64, P, c_int, P, P, P]),
    "orlhf_policy_loss_fwd": (c_int, [P, P, P, P, c_int, P, I64, I64, P, POINTER(PolicyParams), P, P, P, P, P]),
    "orlhf_policy_loss_fwd_grad": (c_int, [P, P, P, P, c_int, P, I64, I64, P, POINTER(PolicyParams), P, P, P, P, P, P]),
    "orlhf_policy_loss_fwd_noalloc": (c_int, [P, P, P, P, c_int, P, I64, I64, P, POINTER(PolicyParams), P, P, P, P]),
    "orlhf_policy_loss_bwd": (c_int, [P, P, P, P, P, c_int, P, I64, I64, P, POINTER(PolicyParams), P, P, P, P, P]),
    "orlhf_value_loss_fwd": (c_int, [P, P, P, P, c_int, I64, I64, P, c_int, c_float, c_int, POINTER(Norm), P, P, P, P]),
    "orlhf_value_loss_fwd_grad": (c_int, [P, P, P, P, c_int, I64, I64, P, c_int, c_float, POINTER(Norm), P, P, P, P, P]),
    "orlhf_value_loss_bwd": (c_int, [P, P, P, P, P, c_int, I64, I64, P, c_int, c_float, P, P, P]),
    "orlhf_compute_reward": (c_int, [P, c_float, P, P, c_int, I64, I64, P, c_int, c_float, c_float, P, P, P]),
    "orlhf_gae_scan": (c_int, [P, P, P, c_int, I64, I64, P, P, c_float, c_float, P, P, P]),
    "orlhf_discounted_returns": (c_int, [P, P, c_int, I64, I64, P, P, c_float, P, P]),
    "orlhf_reward_scan": (c_int, [P, c_float, P, P, P, c_int, I64, I64, P, P, c_int, c_float, c_float, c_float, c_float,
                                  P, P, P, P]),
    "orlhf_group_normalize": (c_int, [P, P, I64, I64, c_int, P, P, P, P]),
    "orlhf_whiten_workspace_bytes": (I64, [I64]),
    "orlhf_masked_whiten": (c_int, [P, P, c_int, I64, c_int, P, P, P, P]),
    "orlhf_whiten_multi_workspace_bytes": (I64, [P, c_int]),
    "orlhf_masked_whiten_multi": (c_int, [P, P, c_int, P, c_int, c_int, P, P, P, P]),
    "orlhf_kl_rows": (c_int, [P, P, c_int, P, c_int, I64, I64, P, c_int, c_int, P, P, P, P]),
    "orlhf_masked_normalize_rows": (c_int, [P, P, c_int, I64, I64, P, c_float, P, P]),
    "orlhf_row_extents": (c_int, [P, c_int, I64, I64, P, P, P, P]),
    "orlhf_cu_seqlens": (c_int, [P, I64, P, P]),
    "orlhf_pack_rows": (c_int, [P, c_int, I64, I64, P, P, P, P]),
    "orlhf_pack_rows_multi": (c_int, [POINTER(PackField), c_int, I64, I64, P, P, P]),
    "orlhf_gather_rows": (c_int, [P, c_int, I64, I64, P, P, P, P]),
    "orlhf_pad_rows": (c_int, [P, c_int, P, I64, I64, c_int, c_uint64, P, P]),
    "orlhf_mask_row_counts": (c_int, [P, c_int, I64, I64, P, P, P]),
    "orlhf_unpad_sequences": (c_int, [P, P, c_int, I64, I64, P, P, I64, P, P, P, P, P]),
    "orlhf_pad_by_indices": (c_int, [P, c_int, I64, I64, P, I64, P, P]),
    "orlhf_gather_by_indices": (c_int, [P, c_int, I64, I64, P, I64, P, P]),
    "orlhf_sequence_logps_fwd": (c_int, [P, P, c_int, P, I64, I64, P, P, P, P]),
    "orlhf_sequence_logps_bwd": (c_int, [P, P, P, c_int, P, P, I64, I64, P, P]),
    "orlhf_pair_loss_fwd": (c_int, [P, P, P, P, I64, c_int, c_double, c_double, P, P, P, P]),
    "orlhf_pair_loss_bwd": (c_int, [P, P, P, P, P, I64, c_int, c_double, c_double, P, P, P]),
}

_lib = None


class KernelError(RuntimeError):
    """A C-ABI entry point returned a negative status."""


def load(path=None):
    """Loads the shared library once and declares every prototype. Raises if it is missing."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    path = path or LIB_PATH
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: the HIP extension is not built. "
            "Run `python -m openrlhf_amd.csrc.build` (needs hipcc); there is no CPU fallback."
        )
    lib = ctypes.CDLL(path)
    missing = [name for name in SIGNATURES if not hasattr(lib, name)]
    if missing:
        raise ImportError(f"{path} lacks symbols declared in include/openrlhf_amd.h: {missing}; rebuild it")
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    got = lib.orlhf_version()
    if got != ABI_VERSION:
        raise ImportError(f"{path}: ABI version {got}, binding expects {ABI_VERSION}")
    _lib = lib
    return lib


def check(status, what):
    if status != 0:
        msg = load().orlhf_last_error().decode("utf-8", "replace")
        raise KernelError(f"{what} failed with status {status}: {msg}")


def call(name, *args):
    """Calls entry point `name` and raises KernelError on a non-zero status."""
    check(getattr(load(), name)(*args), name)


# ------------------------------------------------------------------ tensor plumbing
_DTYPES = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}


def dtype_code(t):
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}; expected float32, bfloat16 or float16") from None


def require_gpu(*tensors):
    """All given tensors must live on one GPU; returns its device."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "openrlhf_amd runs on the GPU only (hand-written HIP kernels, no CPU fallback); "
                f"got a tensor on {t.device}"
            )
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
    if dev is None:
        raise RuntimeError("no tensor given")
    return dev


def ptr(t):
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_of(device):
    """The hipStream_t of torch's current stream on `device` (what every launch follows)."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)  # no Stream object: a fifth of the time on the launch path
    return torch.cuda.current_stream(device).cuda_stream


class on_device:
    """``with on_device(dev):`` makes `dev` the current GPU for the launches inside, like
    torch.cuda.device, but does nothing at all when it already is (the usual case: two calls into
    the runtime saved per kernel launch)."""

    __slots__ = ("index", "previous")

    def __init__(self, device):
        self.index = device.index
        self.previous = -1

    def __enter__(self):
        if self.index is not None:
            current = torch.cuda.current_device()
            if current != self.index:
                self.previous = current
                torch.cuda.set_device(self.index)
        return self

    def __exit__(self, *exc):
        if self.previous >= 0:
            torch.cuda.set_device(self.previous)
            self.previous = -1
        return False


def mask_arg(mask):
    """(tensor kept alive, pointer, mask dtype code) for a mask of any torch dtype."""
    if mask is None:
        return None, None, MASK_NONE
    if mask.dtype in (torch.bool, torch.uint8):
        m = mask.contiguous()
        return m, m.data_ptr(), MASK_U8
    if mask.dtype == torch.float32:
        m = mask.contiguous()
        return m, m.data_ptr(), MASK_F32
    if mask.dtype == torch.int64:
        m = mask.contiguous()
        return m, m.data_ptr(), MASK_I64
    m = mask.to(torch.float32).contiguous()  # other int / float types: exact for 0/1 masks
    return m, m.data_ptr(), MASK_F32


def make_norm(dp_size, value, keep):
    """orlhf_norm from a Python number, a 0-dim tensor or None. Device tensors are passed by
    pointer (no host synchronisation); `keep` collects tensors that must outlive the call."""
    n = Norm()
    n.dp_size = float(dp_size)
    n.norm_value = math.nan
    n.norm_dev = None
    if value is None:
        return n
    if isinstance(value, torch.Tensor):
        if value.is_cuda:
            v = value.detach().reshape(-1)[:1].to(torch.float32).contiguous()
            keep.append(v)
            n.norm_dev = v.data_ptr()
        else:
            n.norm_value = float(value)
    else:
        n.norm_value = float(value)
    return n

"""Headline benchmark: fused log-prob + entropy forward + in-place backward over packed bf16
logits at V = 151936 (the 16-sequence packed workload of the headline metric), one GPU.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]

One step = log-prob + entropy forward AND backward over the whole packed batch (16 sequences,
lengths uniform in [512, 3072], ~30 K tokens, ~9 GB of logits) with the upstream gradients of
the config given, called through the public Python API, i.e. through the C ABI into the HIP
kernels. The gradient overwrites the logits, so every step gets logits nobody has touched: a
ring of buffers is refilled from a pristine copy between timed segments (the refill is outside
the timed segments; each segment is bracketed by torch.cuda.synchronize()).

Two ways of doing the step are timed back to back on the same data, K steps each:
  * `fused_one_pass` (reported as `value`): ``fused_logprob_entropy_fwd_bwd``, one kernel that
    reads every row once, keeps it in the registers of a CU and writes the gradient once;
  * `autograd_two_kernels`: ``logprobs_and_entropy_from_logits`` forward, then
    ``torch.autograd.grad`` running the in-place backward kernel (the reference's call pattern).
Both produce logprob, entropy and d/d(logits); the tests check them against the same oracle.

Prints ONE JSON line. `value` = tokens/s with inputs resident in HBM; `roofline` prices the
dominant kernel against the published 8 TB/s with the bytes its one-pass algorithm moves (2 x V x
2 bytes per token: every row read once, its gradient written once), from HIP-event durations on
the launch stream inside the timed steps, next to the figure in the accounting of a separate
forward and backward (3 x V x 2) and to what plain read / read+write / copy / fill streams reach
on the same buffers (`ceiling_gbs`); `traffic` is what the counters saw (rocprofv3, from the
committed summary of the same ABI version); `checked` says whether a row sample of the last timed
buffer agreed with the separate kernels; `cpu_baseline` is the CPU oracle on a row sample.
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

VOCAB = 151936
N_SEQ = 16
LEN_LO, LEN_HI = 512, 3072
HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = 2500.0  # dense bf16
METRIC = "logprob+entropy fwd+bwd tokens/s at V=151936 bf16; achieved HBM GB/s vs peak"


def _ensure_built():
    from openrlhf_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        from openrlhf_amd.csrc.build import build

        build(verbose=False)
    return _lib.load()


def make_workload(dev, seed=1234):
    """Config 2: packed bf16 logits ~ N(0, 3) with 1% of the rows given one +15 spike, labels
    uniform, upstream grads ~ N(0, 1). Returns (pristine logits, labels, g_lp, g_ent, cu_seqlens)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    lens = torch.randint(LEN_LO, LEN_HI + 1, (N_SEQ,), generator=g)
    cu = torch.cat([torch.zeros(1, dtype=torch.int64), lens.cumsum(0)])
    n = int(cu[-1])
    gd = torch.Generator(device=dev).manual_seed(seed)
    logits = torch.empty(n, VOCAB, dtype=torch.bfloat16, device=dev)
    for lo in range(0, n, 2048):  # fp32 noise in slabs keeps the transient small
        hi = min(lo + 2048, n)
        logits[lo:hi] = (torch.randn(hi - lo, VOCAB, generator=gd, device=dev) * 3.0).to(torch.bfloat16)
    n_spike = max(1, n // 100)
    rows = torch.randperm(n, generator=g)[:n_spike].to(dev)
    cols = torch.randint(0, VOCAB, (n_spike,), generator=g).to(dev)
    logits[rows, cols] += 15.0
    labels = torch.randint(0, VOCAB, (n,), generator=g).to(dev)
    g_lp = torch.randn(n, generator=g).to(dev)
    g_ent = torch.randn(n, generator=g).to(dev)
    return logits, labels, g_lp, g_ent, cu


def cpu_baseline(logits_rows, labels, g_lp, g_ent, repeats=5):
    """The CPU oracle on a row sample: bf16 -> fp32 up-cast, entropy, gather - chunked logsumexp,
    autograd backward (the reference's op sequence, openrlhf/models/actor.py:267-285)."""
    from oracle import token_numerics as otn

    x_bf16 = logits_rows.cpu()
    labels, g_lp, g_ent = labels.cpu(), g_lp.cpu(), g_ent.cpu()
    times = []
    for _ in range(repeats + 1):
        t0 = time.perf_counter()
        x = x_bf16.to(torch.float32).requires_grad_(True)
        ent = otn.compute_entropy(x)
        lp = otn.log_probs_from_logits(x, labels, 1.0)
        torch.autograd.backward([lp, ent], [g_lp, g_ent])
        times.append(time.perf_counter() - t0)
        del x, ent, lp
    times = sorted(times[1:])  # first run is warm-up
    med = times[len(times) // 2]
    return x_bf16.shape[0] / med, med, repeats


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown CPU"


def measured_traffic(kernel, n_tok):
    """HBM bytes per launch from the committed rocprofv3 --pmc summary (FETCH_SIZE + WRITE_SIZE,
    each scaled by what the counter reads for a copy of known size); None if it does not cover
    this workload."""
    path = os.path.join(ROOT, "profiles", "logprob_entropy_fwd_bwd_config2_hbm_traffic.txt")
    try:
        text = open(path).read()
    except OSError:
        return None
    from openrlhf_amd import _lib
    if f"tokens = {n_tok})" not in text or f"abi_version = {_lib.ABI_VERSION}" not in text:
        return None  # measured on another workload or another version of the kernels
    for line in text.splitlines():
        parts = line.split()
        if len(parts) == 3 and parts[0] == "traffic_bytes_per_launch" and parts[1] == kernel:
            return float(parts[2])
    return None


def bench_ppo_step(args, pristine, bufs, cu, ring, dev):
    """Extra figure on the same packed logits: the whole PPO actor loss step (log-probs, entropy,
    clipped surrogate, k3 KL loss, entropy bonus, their derivative down to the logits) through
    ``fused_actor_loss_step``: the one-pass kernel plus the per-token kernels for the loss values."""
    from openrlhf_amd.models.actor import unpad_indices
    from openrlhf_amd.models.loss import PolicyLoss
    from openrlhf_amd.trainer.ray.ppo_actor import fused_actor_loss_step

    g = torch.Generator(device="cpu").manual_seed(99)
    lens = (cu[1:] - cu[:-1])
    b, t = lens.numel(), int(lens.max())
    attn = (torch.arange(t)[None, :] < lens[:, None]).long().to(dev)
    seqs = (torch.randint(1, VOCAB, (b, t), generator=g).to(dev)) * attn
    action_mask = attn[:, 1:].bool()  # every generated position is an action
    a = t - 1
    old = (-torch.rand(b, a, generator=g) * 14).to(dev)
    ref = (-torch.rand(b, a, generator=g) * 14).to(dev)
    adv = torch.randn(b, a, generator=g).to(dev)
    idx = unpad_indices(attn)
    fn = PolicyLoss(0.2, 0.2)
    n_tok = pristine.shape[0]

    def one(buf):
        return fused_actor_loss_step(buf, seqs, attn, action_mask, old, adv, fn, base_action_log_probs=ref,
                                     kl_estimator="k3", kl_coef=0.01, entropy_coef=0.001, packed_indices=idx)

    total, left, first = 0.0, args.steps, True
    while left > 0:
        c = min(left, ring)
        for buf in bufs[:c]:
            buf.detach_().copy_(pristine)
        if first:
            one(bufs[0])
            bufs[0].detach_().copy_(pristine)
            first = False
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(c):
            out = one(bufs[i])
        torch.cuda.synchronize()
        total += time.perf_counter() - t0
        left -= c
    return {
        "entry": "openrlhf_amd.trainer.ray.ppo_actor.fused_actor_loss_step (PPO clip 0.2 + 0.01*k3 KL loss + 0.001*entropy)",
        "value": n_tok * args.steps / total,
        "unit": "tokens/s",
        "ms_per_step": total / args.steps * 1e3,
        "loss": float(out["loss"]),
    }


def bench_ceilings(pristine, bufs, labels, dev):
    """What plain streams reach on the same buffers (bytes moved / HIP-event time, GB/s), for the
    roofline of the vocabulary-row kernels to be read against: a pure read (the library's forward
    in log-prob-only mode: one pass, a few VALU ops per element), an in-place read+write through
    the same row traversal (orlhf_divide_rows_inplace), a device-to-device copy (Tensor.copy_) and
    a fill (Tensor.zero_). Each launch works on the next buffer of the ring (9.4 GB apart)."""
    from openrlhf_amd import _lib
    from openrlhf_amd.models.utils import log_probs_from_logits

    n, v = pristine.shape
    nbytes = n * v * pristine.element_size()
    for b in bufs:
        b.detach_().copy_(pristine)
    stream = _lib.stream_of(dev)
    code = _lib.dtype_code(pristine)

    def read(b):
        with torch.no_grad():
            log_probs_from_logits(b, labels, 1.0)

    def read_write(b):
        _lib.call("orlhf_divide_rows_inplace", b.data_ptr(), code, n, v, v, 1.25, stream)

    def copy(b):
        b.copy_(pristine)

    def fill(b):
        b.zero_()

    out = {}
    for name, fn, moved in (("read", read, nbytes), ("read_write_inplace", read_write, 2 * nbytes),
                            ("copy", copy, 2 * nbytes), ("fill", fill, nbytes)):
        fn(bufs[0])
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        reps = 2 * len(bufs)
        e0.record()
        for i in range(reps):
            fn(bufs[i % len(bufs)])
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        out[name] = {"ms": ms, "gbs": moved / (ms * 1e-3) / 1e9, "bytes": moved}
    return out


def lmhead_traffic(n, hdim, vocab):
    """HBM bytes per forward launch from the committed rocprofv3 --pmc summary of this shape
    (FETCH_SIZE + WRITE_SIZE scaled by a copy of known size); None if it covers another shape or
    another version of the kernels."""
    path = os.path.join(ROOT, "profiles", f"lmhead_logprob_entropy_n{n}_h{hdim}_v{vocab}_hbm_traffic.txt")
    try:
        text = open(path).read()
    except OSError:
        return None
    from openrlhf_amd import _lib
    if f"abi_version = {_lib.ABI_VERSION}" not in text:
        return None
    for line in text.splitlines():
        parts = line.split()
        if len(parts) == 3 and parts[0] == "traffic_bytes_per_launch" and parts[1] == "lmhead_fwd_kernel":
            return float(parts[2])
    return None


def bench_lmhead(dev, n=4096, hdim=4096, vocab=VOCAB, reps=4, roofline=True):
    """The lm-head + log-prob + entropy path at N tokens x H hidden x V vocabulary in bf16, forward and
    forward + backward down to d(hidden) and d(weight), three ways on the same inputs:
      * fused, nothing kept: the backward recomputes the logits tiles (8 N H V flops in all);
      * fused, every logit kept (keep_logits_mib): forward + two products (6 N H V), the logits
        stored once by the forward's tiles and turned into their gradient in place;
      * materialised: torch.matmul (hipBLASLt) -> bf16 logits -> the one-pass vocabulary-row kernel
        (log-prob, entropy and the logits gradient in place) -> two torch.matmul products,
    each with the device memory it holds beyond the inputs at its peak. The roofline prices the
    forward kernel against the dense bf16 matrix-core peak (2.5 PFLOP/s) with 2 N H V flops."""
    from openrlhf_amd.models.utils import fused_logprob_entropy_fwd_bwd, lm_head_logprobs_and_entropy

    g = torch.Generator(device=dev).manual_seed(3)
    hidden = torch.randn(n, hdim, generator=g, device=dev).to(torch.bfloat16)
    weight = (torch.randn(vocab, hdim, generator=g, device=dev) * (3.0 / hdim ** 0.5)).to(torch.bfloat16)
    labels = torch.randint(0, vocab, (n,), generator=g, device=dev)
    g_lp, g_ent = torch.randn(n, generator=g, device=dev), torch.randn(n, generator=g, device=dev)
    all_mib = (n * ((vocab + 255) // 256 * 256 + 64) * 2 >> 20) + 1

    def ev(fn, warm=3):
        """(ms per call, peak bytes allocated beyond what was there before), after `warm` untimed calls
        (the first launches after an idle stretch run at the clock the GPU is still ramping up from)"""
        for _ in range(warm):
            out = fn()
            del out
        torch.cuda.synchronize()
        base = torch.cuda.memory_allocated(dev)
        torch.cuda.reset_peak_memory_stats(dev)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            out = fn()
            del out
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps, torch.cuda.max_memory_allocated(dev) - base

    def fwd():
        with torch.no_grad():
            return lm_head_logprobs_and_entropy(hidden, weight, labels, 1.0)

    hd, wd = hidden.clone().requires_grad_(True), weight.clone().requires_grad_(True)

    def fused(keep_mib):
        def run():
            lp, ent = lm_head_logprobs_and_entropy(hd, wd, labels, 1.0, keep_logits_mib=keep_mib)
            torch.autograd.backward([lp, ent], [g_lp, g_ent])
            gh, gw = hd.grad, wd.grad
            hd.grad = wd.grad = None
            return lp.detach(), ent.detach(), gh, gw
        return run

    def materialised():
        with torch.no_grad():
            logits = torch.matmul(hidden, weight.t())
            lp, ent, p = fused_logprob_entropy_fwd_bwd(logits, labels, g_lp, g_ent, 1.0, inplace=True)
            return lp, ent, torch.matmul(p, weight), torch.matmul(p.t(), hidden)

    def materialised_fwd():
        with torch.no_grad():
            from openrlhf_amd.models.utils import logprobs_and_entropy_from_logits
            return logprobs_and_entropy_from_logits(torch.matmul(hidden, weight.t()), labels, 1.0)

    ms_f, mem_f = ev(fwd)

    # the forward launch by itself (the C entry on a workspace allocated beforehand: the tile kernel and
    # the 28 us kernel that combines a token's tiles), on the stream the kernels run on
    from openrlhf_amd import _lib
    from openrlhf_amd._lib import call, ptr, stream_of
    ws = torch.empty(_lib.load().orlhf_lmhead_workspace_bytes(n, hdim, vocab, 0, 0), dtype=torch.uint8, device=dev)
    lp_k, ent_k, st_k = torch.empty(n, device=dev), torch.empty(n, device=dev), torch.empty(n, 4, device=dev)

    def fwd_launch():
        call("orlhf_lmhead_logprob_entropy_fwd", ptr(hidden), ptr(weight), _lib.BF16, n, hdim, vocab, hidden.stride(0),
             weight.stride(0), ptr(labels), 1.0, ptr(lp_k), ptr(ent_k), ptr(st_k), None, 0, 0, ptr(ws), ws.numel(), stream_of(dev))

    for _ in range(3):
        fwd_launch()
    launches = 2 * reps
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(launches):
        fwd_launch()
    e1.record()
    torch.cuda.synchronize()
    ms_k = e0.elapsed_time(e1) / launches
    del ws
    ms_fb, mem_fb = ev(fused(None))
    ms_fk, mem_fk = ev(fused(all_mib))
    ms_half, mem_half = ev(fused(all_mib // 2))
    ms_m, mem_m = ev(materialised)
    ms_mf, mem_mf = ev(materialised_fwd)
    flops = 2.0 * n * hdim * vocab
    # checks (outside the timed region): values and both gradients of the fused routes against the
    # materialised route (its logits differ from the tiles' by the rounding of the accumulation order:
    # a few entries per thousand tokens move by one 16-bit step), and the budgets against each other
    a, b, c = fused(None)(), fused(all_mib)(), materialised()
    same_bits = all(torch.equal(x, y) for x, y in zip(a, b))
    med = lambda x: x.abs().float().flatten()[:: max(1, x.numel() // 1000003)].median().item()  # noqa: E731
    check = {
        "budgets_bit_identical": same_bits,
        "logprob_median_abs_diff_vs_materialised": med(a[0] - c[0]),
        "entropy_median_abs_diff_vs_materialised": med(a[1] - c[1]),
        "grad_hidden_rel_fro_vs_materialised": ((a[2].float() - c[2].float()).norm() / c[2].float().norm()).item(),
        "grad_weight_rel_fro_vs_materialised": ((a[3].float() - c[3].float()).norm() / c[3].float().norm()).item(),
    }
    ok = (same_bits and check["logprob_median_abs_diff_vs_materialised"] <= 1e-3
          and check["grad_hidden_rel_fro_vs_materialised"] <= 2.0 ** -6 and check["grad_weight_rel_fro_vs_materialised"] <= 2.0 ** -6)
    del a, b, c
    out = {
        "entry": "openrlhf_amd.models.utils.lm_head_logprobs_and_entropy",
        "config": {"tokens": n, "hidden": hdim, "vocab": vocab, "dtype": "bf16"},
        "forward_ms": ms_f, "forward_tokens_per_s": n / (ms_f * 1e-3), "forward_extra_bytes": mem_f,
        "forward_backward_ms": ms_fb, "forward_backward_tokens_per_s": n / (ms_fb * 1e-3),
        "routes": {
            "fused_nothing_kept": {"forward_backward_ms": ms_fb, "peak_extra_bytes": mem_fb},
            "fused_half_of_the_logits_kept": {"forward_backward_ms": ms_half, "peak_extra_bytes": mem_half},
            "fused_all_logits_kept": {"forward_backward_ms": ms_fk, "peak_extra_bytes": mem_fk},
            "materialised_torch_matmul": {"forward_ms": ms_mf, "forward_extra_bytes": mem_mf, "forward_backward_ms": ms_m,
                                          "peak_extra_bytes": mem_m},
            "note": "peak_extra_bytes: device memory beyond the inputs at the route's peak, outputs and gradients "
                    "(0.034 + 1.245 GB at N = 4096) included",
        },
        "checked": ok, "check": check,
    }
    if roofline:
        out["roofline"] = {"bound": "mfma", "kernel": "lmhead_fwd_kernel<bf16> (256x256 MFMA 32x32x16 tiles + per-token statistics)",
                           "achieved": flops / (ms_k * 1e-3) / 1e12, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                           "frac": flops / (ms_k * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, "flops_per_launch": flops,
                           "avg_launch_ms": ms_k,
                           "traffic": lmhead_traffic(n, hdim, vocab),
                           "forward_backward_all_kept_achieved": 3 * flops / (ms_fk * 1e-3) / 1e12,
                           "forward_backward_all_kept_frac": 3 * flops / (ms_fk * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS,
                           "forward_backward_nothing_kept_achieved": 4 * flops / (ms_fb * 1e-3) / 1e12,
                           "forward_backward_nothing_kept_frac": 4 * flops / (ms_fb * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS}
    return out


def bench_few_rows(dev, n=64, vocab=VOCAB, copies=32):
    """A launch with fewer rows than the GPU has compute units (n x 151936 bf16, 19 MB at n = 64):
    forward with the rows cut into segments against the whole-row forward on the same rows, and
    the backward (which cuts its rows itself), through the C ABI. Each timed launch takes the next
    of `copies` distinct inputs (0.6 GB in all at the defaults: more than the caches hold)."""
    from openrlhf_amd import _lib
    from openrlhf_amd._lib import call, ptr, stream_of

    lib = _lib.load()
    xs = [(torch.randn(n, vocab, device=dev) * 3).to(torch.bfloat16) for _ in range(copies)]
    grads = torch.empty(n, vocab, device=dev, dtype=torch.bfloat16)
    labels = torch.randint(0, vocab, (n,), device=dev)
    g_lp, g_ent = torch.randn(n, device=dev), torch.randn(n, device=dev)
    lp, ent = torch.empty(n, device=dev), torch.empty(n, device=dev)
    stats = torch.empty(n, 4, device=dev)
    ws_bytes = lib.orlhf_logprob_entropy_split_workspace_bytes(_lib.BF16, n, vocab)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    st = stream_of(dev)

    tickets = torch.zeros(n, dtype=torch.int32, device=dev)

    def cut(x):  # one launch: the workgroup that finishes a row's last segment merges the row
        call("orlhf_logprob_entropy_fwd_split", ptr(x), _lib.BF16, n, vocab, vocab, ptr(labels), 1.0, ptr(lp), ptr(ent),
             ptr(stats), None, ptr(ws), ws_bytes, ptr(tickets), st)

    def cut_two_launches(x):  # no tickets: a second kernel merges
        call("orlhf_logprob_entropy_fwd_split", ptr(x), _lib.BF16, n, vocab, vocab, ptr(labels), 1.0, ptr(lp), ptr(ent),
             ptr(stats), None, ptr(ws), ws_bytes, None, st)

    def whole(x):
        call("orlhf_logprob_entropy_fwd", ptr(x), _lib.BF16, n, vocab, vocab, ptr(labels), 1.0, ptr(lp), ptr(ent),
             ptr(stats), None, 0, st)

    def backward(x):
        call("orlhf_logprob_entropy_bwd", ptr(x), ptr(grads), _lib.BF16, n, vocab, vocab, vocab, ptr(labels), 1.0,
             ptr(g_lp), ptr(g_ent), ptr(stats), None, st)

    def timed(fn):
        for x in xs[:4]:
            fn(x)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for x in xs:
            fn(x)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / len(xs)

    whole_ms, cut_ms, cut2_ms = timed(whole), timed(cut), timed(cut_two_launches)
    cut_two_launches(xs[0])
    lp_cut2 = lp.clone()
    cut(xs[0])
    lp_cut = lp.clone()
    whole(xs[0])
    bwd_ms = timed(backward)
    row_bytes = vocab * 2
    return {
        "workload": f"{n} rows x {vocab} bf16 logits per launch ({n * row_bytes / 1e6:.1f} MB), {copies} distinct inputs in rotation",
        "segments_per_row": ws_bytes // (n * 32) if ws_bytes else 1,
        "forward_whole_rows_us": whole_ms * 1e3, "forward_whole_rows_gbs": n * row_bytes / whole_ms / 1e6,
        "forward_cut_rows_us": cut_ms * 1e3, "forward_cut_rows_gbs": n * row_bytes / cut_ms / 1e6,
        "forward_cut_rows_merge_kernel_us": cut2_ms * 1e3,
        "cut_rows_one_launch_equals_two_launches": bool(torch.equal(lp_cut, lp_cut2)),
        "backward_cut_rows_us": bwd_ms * 1e3, "backward_cut_rows_gbs": 2 * n * row_bytes / bwd_ms / 1e6,
        "max_abs_diff_cut_vs_whole": (lp_cut - lp).abs().max().item(),
        "note": "a launch this small is a few microseconds: the times include the launch itself and the ramp of the "
                "first loads, which is what keeps them under the streaming rates of the full-size batch",
    }


def bench_matrix_tile(dev, m=8192, n=8192, k=8192, reps=10):
    """--workload matrix_tile: the matrix-core tile of the lm-head path as a plain bf16 product
    (orlhf_matrix_tile_probe), with its slab loads and with the operands resident in LDS (the same
    LDS reads, MFMAs and barriers, nothing loaded: what the tile is bounded by on this GPU and
    clock) and with all loads hitting the L1 (row stride 0: the cost of issuing the loads and
    writing LDS without the cost of fetching), on random operands and on operands whose rows are all equal (less switching in the
    multipliers, higher clock), beside torch.matmul (hipBLASLt) on the same shapes."""
    from openrlhf_amd import _lib
    from openrlhf_amd._lib import call, ptr, stream_of

    tiles = ((m + 255) // 256) * ((n + 255) // 256)
    sums = torch.empty(tiles * 256, device=dev, dtype=torch.float32)
    st = stream_of(dev)
    flops = 2.0 * m * n * k

    def timed(fn):
        fn(); fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    # the first few dozen milliseconds of matrix work after idling run at a lower clock: bring the
    # GPU to its sustained state before anything is timed
    wa, wb = torch.randn(m, k, device=dev).to(torch.bfloat16), torch.randn(n, k, device=dev).to(torch.bfloat16)
    for _ in range(60):
        call("orlhf_matrix_tile_probe", ptr(wa), ptr(wb), _lib.BF16, m, n, k, k, k, 0, ptr(sums), st)
    torch.cuda.synchronize()
    del wa, wb

    out = {}
    for name, make in (("random", lambda r, c: torch.randn(r, c, device=dev)),
                       ("equal_rows", lambda r, c: torch.randn(1, c, device=dev).expand(r, c).contiguous())):
        a, b = make(m, k).to(torch.bfloat16), make(n, k).to(torch.bfloat16)
        entry = {}
        # "one row": row stride 0, every row of an operand is its first row, so all loads hit the L1
        for label, resident, ld in (("tile", 0, k), ("tile_loads_hit_l1", 0, 0), ("tile_operands_resident", 1, k)):
            ms = timed(lambda: call("orlhf_matrix_tile_probe", ptr(a), ptr(b), _lib.BF16, m, n, k, ld, ld, resident, ptr(sums), st))
            entry[label] = {"ms": ms, "tflops": flops / ms / 1e9}
        call("orlhf_matrix_tile_probe", ptr(a), ptr(b), _lib.BF16, m, n, k, k, k, 0, ptr(sums), st)
        got = sums.view(-1, 256).sum(1)[:4].double()
        want = torch.stack([(a[:256].double().sum(0) * b[j * 256:(j + 1) * 256].double().sum(0)).sum() for j in range(4)])
        entry["checked"] = bool(((got - want).abs() <= 1e-3 * want.abs().clamp_min(1e3)).all())
        ms = timed(lambda: torch.matmul(a, b.t()))
        entry["torch_matmul"] = {"ms": ms, "tflops": flops / ms / 1e9}
        out[name] = entry
    return {"workload": f"plain bf16 product [{m}, {k}] x [{n}, {k}]^T through the lm-head path's matrix-core tile", "n_gpus": 1,
            "peak_tflops": MFMA_PEAK_TFLOPS, "entries": out}


def bench_kernels(args, dev):
    """--workload kernels: the three vocabulary-row kernels launched back to back on ONE resident
    buffer of --rows x 151936 bf16 logits (forward, in-place backward, one-pass forward+backward,
    5 launches each), for counter collection with rocprofv3 --pmc. Prints one JSON line of event
    times; the in-place launches overwrite the buffer, which does not matter for counters."""
    from openrlhf_amd.models.utils import fused_logprob_entropy_fwd_bwd, logprobs_and_entropy_from_logits

    n, vocab, temperature = args.rows, args.vocab, args.temperature
    x = torch.empty(n, vocab, device=dev, dtype=torch.bfloat16)
    for lo in range(0, n, 1024):
        x[lo:lo + 1024] = (torch.randn(min(1024, n - lo), vocab, device=dev) * 3).to(torch.bfloat16)
    labels = torch.randint(0, vocab, (n,), device=dev)
    g_lp, g_ent = torch.randn(n, device=dev), torch.randn(n, device=dev)

    def forward():
        with torch.no_grad():
            logprobs_and_entropy_from_logits(x, labels, temperature)

    def backward():
        xg = x.requires_grad_(True)
        lp, ent = logprobs_and_entropy_from_logits(xg, labels, temperature, inplace_backward=True)
        torch.autograd.backward([lp, ent], [g_lp, g_ent])
        xg.grad = None
        x.requires_grad_(False)

    def one_pass():
        fused_logprob_entropy_fwd_bwd(x, labels, g_lp, g_ent, temperature=temperature, inplace=True)

    out = {}
    for name, fn in (("forward", forward), ("forward_then_backward", backward), ("one_pass", one_pass)):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(4):
            fn()
        e1.record()
        torch.cuda.synchronize()
        out[name] = e0.elapsed_time(e1) / 4
    print(json.dumps({"workload": f"vocabulary-row kernels on {n} x {vocab} bf16 logits, temperature {temperature}",
                      "n_gpus": 1, "unit": "ms",
                      "entries": out}), flush=True)


def bench_per_token(args, dev, emit=True):
    """--workload per_token: the small kernels at the sizes of the PPO (256 x 8K) and GRPO (4096 x 16K) batches (per-token
    fp32 tensors; MBs, not GBs: these launches are latency-bound, the figures are for the record).
    Prints one JSON line with achieved GB/s per entry point (algorithmic bytes / event time)."""
    from openrlhf_amd.models.loss import PolicyLoss, ValueLoss
    from openrlhf_amd.models.utils import compute_approx_kl, compute_reward
    from openrlhf_amd.trainer.ppo_utils.experience_maker import (
        get_advantages_and_returns, get_cumulative_returns, whiten_advantages)

    g = torch.Generator(device="cpu").manual_seed(7)

    def timed(fn, n=12):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    res = {}

    def record(name, ms, tokens, bytes_per_token):
        res[name] = {"ms": ms, "tokens": tokens, "bytes_per_token": bytes_per_token,
                     "achieved_gbs": tokens * bytes_per_token / (ms * 1e-3) / 1e9,
                     "frac_of_hbm_peak": tokens * bytes_per_token / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}

    # config 3: 256 sequences, lognormal(7, 0.8) lengths in [16, 8192], padded [B, A]
    b = 256
    lens = torch.clamp(torch.exp(torch.randn(b, generator=g) * 0.8 + 7.0), 16, 8192).long()
    a = int(lens.max())
    mask = (torch.arange(a)[None, :] < lens[:, None]).to(dev)
    values = torch.randn(b, a, generator=g).to(dev)
    kl = (torch.randn(b, a, generator=g) * 0.05).to(dev)
    r = (torch.rand(b, generator=g) < 0.5).float().to(dev)
    padded = b * a
    rew = compute_reward(r, 0.01, kl, action_mask=mask)
    record("config3.compute_reward", timed(lambda: compute_reward(r, 0.01, kl, action_mask=mask)), padded, 4 + 1 + 1 + 4)
    record("config3.gae_scan", timed(lambda: get_advantages_and_returns(values, rew, mask, 1.0, 0.95)), padded, 17)
    adv, ret = get_advantages_and_returns(values, rew, mask, 1.0, 0.95)
    record("config3.whiten", timed(lambda: whiten_advantages([adv], [mask])), padded, 14)
    vnew = (values + 0.1).requires_grad_(True)
    vl = ValueLoss(0.2)

    def value_step():
        loss = vl(vnew, values, ret, action_mask=mask)
        torch.autograd.grad(loss, vnew)

    record("config3.value_loss_fwd_bwd", timed(value_step), padded, 30)

    # the whole launch-bound chain of the step (reward shaping, GAE, whitening, both losses'
    # forward), eagerly and as one captured HIP graph replayed
    from openrlhf_amd.models.loss import PolicyLoss as _PL
    pol3 = _PL(0.2, 0.2)
    old3 = -torch.rand(b, a, device=dev)
    lp3 = old3 + torch.randn(b, a, device=dev) * 0.02

    def chain():
        rew_ = compute_reward(r, 0.01, kl, action_mask=mask)
        adv_, ret_ = get_advantages_and_returns(values, rew_, mask, 1.0, 0.95)
        (adv_w,) = whiten_advantages([adv_], [mask])
        return pol3(lp3, old3, adv_w, action_mask=mask)[0], vl(values + 0.1, values, ret_, action_mask=mask)

    chain_bytes = 10 + 17 + 14 + 13 + 13
    record("config3.chain_eager", timed(chain), padded, chain_bytes)
    if emit and not getattr(args, "no_cpu_baseline", False):
        # the same chain as the reference runs it, on the host: the CPU restatement of its op sequence
        # (reward shaping, GAE as a loop over the columns, whitening, both losses' forward)
        from oracle import advantages as oadv, losses as olos, token_numerics as otn
        c_r, c_kl, c_mask, c_val = r.cpu(), kl.cpu(), mask.cpu().float(), values.cpu()
        c_lp, c_old = lp3.cpu(), old3.cpu()

        def cpu_chain():
            rew_ = otn.compute_reward(c_r, 0.01, c_kl, c_mask)
            adv_, ret_ = oadv.get_advantages_and_returns(c_val, rew_, c_mask, 1.0, 0.95)
            adv_w = oadv.whiten_advantages([adv_], [c_mask])[0][0]
            return (olos.policy_loss(c_lp, c_old, adv_w, action_mask=c_mask)[0],
                    olos.value_loss(c_val + 0.1, c_val, ret_, action_mask=c_mask, clip_eps=0.2))

        cpu_chain()
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            cpu_chain()
            times.append(time.perf_counter() - t0)
        med = sorted(times)[1]
        res["config3.chain_cpu_baseline"] = {
            "ms": med * 1e3, "tokens": padded, "tokens_per_s": padded / med, "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"the whole config 3 batch ({b} x {a} padded fp32): the oracle's restatement of the reference's op "
                      f"sequence on torch CPU, median of 3 runs after a warm-up; {cpu_model()}"}
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.no_grad():
        chain()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph), torch.no_grad():
        chain()
    record("config3.chain_graph_replay", timed(graph.replay), padded, chain_bytes)

    # config 4: 512 x 8 sequences, lengths uniform in [64, 16384], padded [B, A]. Every entry rotates
    # over RING distinct copies of its inputs (0.3-1.1 GB each, so 1.3-4.3 GB per entry against a
    # 256 MB Infinity Cache): what is timed comes from HBM, not from a cache a replay left warm.
    RING = 4
    b = 4096
    lens = torch.randint(64, 16385, (b,), generator=g)
    a = int(lens.max())
    mask0 = (torch.arange(a, device=dev)[None, :] < lens.to(dev)[:, None])
    lp0 = -torch.rand(b, a, device=dev) * 2

    def ring_of(t):
        return [t] + [t.clone() for _ in range(RING - 1)]

    mask, lp = ring_of(mask0), ring_of(lp0)
    old = ring_of(lp0 + torch.randn(b, a, device=dev) * 0.05)
    ref = ring_of(lp0 + torch.randn(b, a, device=dev) * 0.1)
    adv = ring_of(torch.randn(b, a, device=dev))
    padded = b * a
    turn = [0]

    def rot(fn):  # fn(k) with k cycling over the copies
        def call():
            turn[0] = (turn[0] + 1) % RING
            return fn(turn[0])
        return call

    record("config4.approx_kl_k3", timed(rot(lambda k: compute_approx_kl(lp[k], ref[k], "k3"))), padded, 12)
    record("config4.discounted_returns", timed(rot(lambda k: get_cumulative_returns(adv[k], mask[k], 1.0))), padded, 9)
    record("config4.gae_scan", timed(rot(lambda k: get_advantages_and_returns(old[k], adv[k], mask[k], 1.0, 0.95))), padded, 17)
    from openrlhf_amd.trainer.ppo_utils.experience_maker import experience_kl
    record("config4.kl_block_k3", timed(rot(lambda k: experience_kl(lp[k], ref[k], mask[k], "k3"))), padded, 13)
    r_seq = torch.randn(b, device=dev)
    record("config4.compute_reward", timed(rot(lambda k: compute_reward(r_seq, 0.01, adv[k], mask[k]))), padded, 4 + 1 + 1 + 4)
    from openrlhf_amd.trainer.ppo_utils.experience_maker import reward_advantages_and_returns
    # reward + GAE without the per-token reward in memory: kl, values, mask in; advantages, returns out
    record("config4.reward_gae_one_pass",
           timed(rot(lambda k: reward_advantages_and_returns(r_seq, 0.01, adv[k], old[k], mask[k], 1.0, 0.95))), padded, 17)
    xs = [t.clone().requires_grad_(True) for t in lp]
    pl = PolicyLoss(0.2, 0.2, dual_clip=3.0, token_level_loss=False)

    def policy_step(k):
        out = pl(xs[k], old[k], adv[k], action_mask=mask[k])
        torch.autograd.grad(out[0], xs[k])

    record("config4.policy_loss_fwd_bwd", timed(rot(policy_step)), padded, 13 + 17)
    # token mean: without a given count the gradient needs its own pass; with the trainers'
    # batch_num_tokens the forward writes it (13 bytes in, 4 out)
    pl_tok = PolicyLoss(0.2, 0.2, dual_clip=3.0)
    n_tok_given = float(mask0.sum()) * 2

    def policy_step_token_mean(k):
        torch.autograd.grad(pl_tok(xs[k], old[k], adv[k], action_mask=mask[k])[0], xs[k])

    def policy_step_given_count(k):
        torch.autograd.grad(pl_tok(xs[k], old[k], adv[k], action_mask=mask[k], dp_size=2, batch_num_tokens=n_tok_given)[0], xs[k])

    record("config4.policy_loss_token_mean_fwd_bwd", timed(rot(policy_step_token_mean)), padded, 13 + 17)
    record("config4.policy_loss_token_mean_given_count_fwd_bwd", timed(rot(policy_step_given_count)), padded, 13 + 4)

    # the same batch packed once (flat tokens + cu_seqlens): padding is neither stored nor read
    from openrlhf_amd.trainer.dpo_trainer import get_batch_logps
    from openrlhf_amd.trainer.ppo_utils.experience import PackedSteps, pad_packed

    real = int(lens.sum())
    fields = [dict(lp=lp[k], old=old[k], adv=adv[k], mask=mask[k]) for k in range(RING)]
    ps = [PackedSteps.from_padded(fields[k], mask[k], total=real) for k in range(RING)]
    # pack: mask extents (1 B/padded token) + per field read and write of the real tokens
    record("config4.pack_4_fields", timed(rot(lambda k: PackedSteps.from_padded(fields[k], mask[k], total=real))),
           real, 2 * 13 + padded / real)
    record("config4.pad_1_field", timed(rot(lambda k: pad_packed(ps[k]["adv"], ps[k].cu_seqlens, a))), padded, 4 + 4 * real / padded)
    record("config4.discounted_returns_packed",
           timed(rot(lambda k: get_cumulative_returns(ps[k]["adv"], ps[k]["mask"], 1.0, cu_seqlens=ps[k].cu_seqlens, max_seqlen=a))), real, 9)
    record("config4.gae_scan_packed",
           timed(rot(lambda k: get_advantages_and_returns(ps[k]["old"], ps[k]["adv"], ps[k]["mask"], 1.0, 0.95, cu_seqlens=ps[k].cu_seqlens))), real, 17)
    # the same with the rows handed out longest first (the order is computed once per packed batch)
    order = [p_.longest_first for p_ in ps]
    record("config4.discounted_returns_packed_longest_first",
           timed(rot(lambda k: get_cumulative_returns(ps[k]["adv"], ps[k]["mask"], 1.0, cu_seqlens=ps[k].cu_seqlens, max_seqlen=a,
                                                      row_order=order[k]))), real, 9)
    record("config4.gae_scan_packed_longest_first",
           timed(rot(lambda k: get_advantages_and_returns(ps[k]["old"], ps[k]["adv"], ps[k]["mask"], 1.0, 0.95,
                                                          cu_seqlens=ps[k].cu_seqlens, row_order=order[k]))), real, 17)
    xk = [p_["lp"].clone().requires_grad_(True) for p_ in ps]

    def policy_step_packed(k):
        out = pl(xk[k], ps[k]["old"], ps[k]["adv"], action_mask=ps[k]["mask"], cu_seqlens=ps[k].cu_seqlens, max_seqlen=a)
        torch.autograd.grad(out[0], xk[k])

    record("config4.policy_loss_fwd_bwd_packed", timed(rot(policy_step_packed)), real, 13 + 17)
    att = [torch.cat([m_[:, :1], m_], dim=1) for m_ in mask]
    prompt_lens = torch.randint(1, 64, (b,), generator=g).to(dev)
    record("config4.dpo_sequence_logps", timed(rot(lambda k: get_batch_logps(lp[k], att[k], prompt_lens))), padded, 5)
    # the unpadding in front of the packed forward and the re-padding behind it
    # (openrlhf/models/ring_attn_utils.py:103-182): mask read twice (counts, ranks), per attended token
    # its id read and four int64 written; back: zeros, then value and index read, value written
    from openrlhf_amd.models.ring_attn_utils import gather_and_pad_tensor, unpad_and_slice_tensor
    seqs = torch.randint(0, 151936, (b, a + 1), generator=g).to(dev)
    n_att = [int(m_.sum()) for m_ in att]
    mb = att[0].element_size()
    record("config4.unpad_and_slice_tensor",
           timed(rot(lambda k: unpad_and_slice_tensor(seqs, att[k], None, total_tokens=n_att[k]))), b * (a + 1),
           2 * mb + (8 + 32) * n_att[0] / (b * (a + 1)))
    up = [unpad_and_slice_tensor(seqs, att[k], None) for k in range(RING)]
    vals = [torch.randn(1, n_att[k], device=dev) for k in range(RING)]
    record("config4.gather_and_pad_tensor",
           timed(rot(lambda k: gather_and_pad_tensor(vals[k], None, 0, up[k][4], b, a + 1))), b * (a + 1),
           4 + (4 + 8 + 4) * n_att[0] / (b * (a + 1)))
    if emit:
        print(json.dumps({"workload": "per-token kernels at BASELINE config 3 / config 4 sizes (padded [B, A] fp32)",
                          "n_gpus": 1, "unit": "GB/s", "peak": HBM_PEAK_GBS, "entries": res}), flush=True)
    return res


def bench_torch_eager(args, dev):
    """`--workload torch_eager`: what stock OpenRLHF executes on this GPU for the same inputs - its op
    sequence in eager torch (fp32 up-cast of the logits, compute_entropy, gather - logsumexp in
    1024-row blocks, autograd backward: openrlhf/models/actor.py:267-285, models/utils.py:129-186;
    PolicyLoss and the k3 KL as elementwise chains: models/loss.py:157-230, models/utils.py:64-95;
    GAE as a Python loop over columns: experience_maker.py:358-376) - timed next to the HIP path.
    Plain torch written out here, nothing of the product runs in the eager legs; the logits leg
    uses --rows rows of config 2's shape (the eager chain holds several fp32 copies of them)."""
    from openrlhf_amd.models.loss import PolicyLoss
    from openrlhf_amd.models.utils import compute_approx_kl, fused_logprob_entropy_fwd_bwd, \
        logprobs_and_entropy_from_logits
    from openrlhf_amd.trainer.ppo_utils.experience_maker import get_advantages_and_returns

    def wall_ms(fn, n, warm=1):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e3

    g = torch.Generator(device=dev).manual_seed(0)
    n, vocab = args.rows, args.vocab
    logits = (torch.randn(n, vocab, device=dev, generator=g) * 3).to(torch.bfloat16)
    labels = torch.randint(0, vocab, (n,), device=dev, generator=g)
    g_lp, g_ent = torch.randn(n, device=dev, generator=g), torch.randn(n, device=dev, generator=g)

    def eager_logits_step():
        x = logits.detach().clone().requires_grad_(True)  # stands for the lm head's output
        f = x.to(torch.float32)
        pd = torch.softmax(f, dim=-1)
        ent = torch.logsumexp(f, dim=-1) - torch.sum(pd * f, dim=-1)
        picked = torch.gather(f, -1, labels.unsqueeze(-1)).squeeze(-1)
        lse = torch.empty(n, device=dev, dtype=f.dtype)
        for lo in range(0, n, 1024):
            lse[lo:lo + 1024] = torch.logsumexp(f[lo:lo + 1024], dim=-1)
        torch.autograd.backward([picked - lse, ent], [g_lp, g_ent])
        return x.grad

    eager_ms = wall_ms(eager_logits_step, 3) - wall_ms(lambda: logits.detach().clone(), 3)
    bufs = [logits.clone() for _ in range(4)]
    turn = [0]

    def hip_one_pass():
        turn[0] = (turn[0] + 1) % len(bufs)
        return fused_logprob_entropy_fwd_bwd(bufs[turn[0]], labels, g_lp, g_ent, 1.0, inplace=True)

    def hip_two_kernels():
        turn[0] = (turn[0] + 1) % len(bufs)
        x = bufs[turn[0]].detach().requires_grad_(True)
        lp, ent = logprobs_and_entropy_from_logits(x, labels, 1.0, inplace_backward=True)
        return torch.autograd.grad([lp, ent], [x], [g_lp, g_ent])

    res = {"logprob_entropy_fwd_bwd": {"rows": n, "vocab": vocab, "torch_eager_ms": eager_ms,
                                       "hip_one_pass_ms": wall_ms(hip_one_pass, 8, 2),
                                       "hip_two_kernels_ms": wall_ms(hip_two_kernels, 8, 2)}}
    del bufs, logits
    torch.cuda.empty_cache()

    b, a = 4096, 16384  # config 4
    lens = torch.randint(64, a + 1, (b,), device=dev, generator=g)
    mask = (torch.arange(a, device=dev)[None, :] < lens[:, None]).float()
    lp = -torch.rand(b, a, device=dev, generator=g) * 3
    old = lp + torch.randn(b, a, device=dev, generator=g) * 0.02
    ref_lp = lp + torch.randn(b, a, device=dev, generator=g) * 0.1
    adv = torch.randn(b, a, device=dev, generator=g)

    def eager_policy():
        x = lp.detach().requires_grad_(True)
        raw = x - old
        ratio = raw.clamp(min=-20.0, max=20.0).exp()
        s1, s2 = ratio * adv, ratio.clamp(0.8, 1.2) * adv
        c1 = torch.min(s1, s2)
        loss = -torch.where(adv < 0, torch.max(c1, 3.0 * adv), c1)
        cnt = mask.sum(dim=-1)
        seq, seq_mask = (loss * mask).sum(dim=-1) / (cnt + 1e-8), (cnt > 0).float()
        total = (seq * seq_mask).sum() / seq_mask.sum()
        _ = ((s2 < s1).float() * mask).sum() / mask.sum(), ((-raw.detach()) * mask).sum() / mask.sum()
        total.backward()
        return x.grad

    loss_fn = PolicyLoss(0.2, 0.2, dual_clip=3.0, token_level_loss=False)

    def hip_policy():
        x = lp.detach().requires_grad_(True)
        loss_fn(x, old, adv, action_mask=mask)[0].backward()
        return x.grad

    def eager_kl():
        d = lp.float() - ref_lp.float()
        return ((-d).exp() - 1 + d).clamp(min=-10, max=10)

    res["config4_policy_loss_fwd_bwd"] = {"torch_eager_ms": wall_ms(eager_policy, 5), "hip_ms": wall_ms(hip_policy, 20, 3)}
    res["config4_k3_kl"] = {"torch_eager_ms": wall_ms(eager_kl, 5),
                            "hip_ms": wall_ms(lambda: compute_approx_kl(lp, ref_lp, "k3"), 20, 3)}
    values, rewards = torch.randn(b, a, device=dev, generator=g), torch.randn(b, a, device=dev, generator=g)

    def eager_gae():
        v, r, last, cols = mask * values, mask * rewards, 0, []
        for t in reversed(range(a)):
            nxt = v[:, t + 1] if t < a - 1 else 0.0
            last = r[:, t] + 1.0 * nxt - v[:, t] + 0.95 * last
            cols.append(last)
        adv_ = torch.stack(cols[::-1], dim=1)
        return adv_, adv_ + v

    res["config4_gae"] = {"torch_eager_ms": wall_ms(eager_gae, 1),
                          "hip_ms": wall_ms(lambda: get_advantages_and_returns(values, rewards, mask, 1.0, 0.95), 20, 3)}
    for entry in res.values():
        hip = entry.get("hip_ms", entry.get("hip_one_pass_ms"))
        entry["speedup"] = entry["torch_eager_ms"] / hip
    print(json.dumps({"workload": "the reference's eager torch op sequence on the same GPU beside the HIP path "
                                  "(wall ms per call through the Python API)", "n_gpus": 1, "entries": res}), flush=True)
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=12)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--ring", type=int, default=6, help="distinct logits buffers per timed segment")
    ap.add_argument("--cpu-rows", type=int, default=4096, help="rows of the CPU-baseline sample")
    ap.add_argument("--workload", default="logprob", choices=["logprob", "per_token", "kernels", "torch_eager", "ceilings", "lmhead", "few_rows", "matrix_tile"],
                    help="logprob: the headline step (default); per_token: the small kernels of configs 3/4; "
                         "torch_eager: the reference's eager torch op sequence on this GPU beside the HIP path; "
                         "ceilings: plain read / read+write / copy / fill streams on the headline buffers; "
                         "lmhead: lm-head + log-prob with the logits never stored (matrix cores)")
    ap.add_argument("--rows", type=int, default=8192, help="rows of logits for --workload kernels")
    ap.add_argument("--vocab", type=int, default=VOCAB, help="vocabulary for --workload kernels")
    ap.add_argument("--temperature", type=float, default=1.0, help="temperature for --workload kernels")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-ppo-step", action="store_true", help="skip the extra fused PPO actor step measurement")
    ap.add_argument("--no-lmhead", action="store_true", help="skip the lm-head + log-prob (matrix-core) figure")
    ap.add_argument("--no-per-token", action="store_true",
                    help="skip the per-token kernels of config 4 that the default run reports beside the headline")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (the path shards by rows with no collective "
                 "on it); run with --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback")

    _ensure_built()
    from openrlhf_amd.models.utils import fused_logprob_entropy_fwd_bwd, logprobs_and_entropy_from_logits

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.workload == "kernels":
        bench_kernels(args, dev)
        return
    if args.workload == "per_token":
        bench_per_token(args, dev)
        return
    if args.workload == "torch_eager":
        bench_torch_eager(args, dev)
        return
    if args.workload == "lmhead":
        print(json.dumps({"workload": "lm-head + log-prob + entropy, fused against materialised logits", "n_gpus": 1,
                          **bench_lmhead(dev, n=args.rows if args.rows != 8192 else 4096)}), flush=True)
        return
    if args.workload == "matrix_tile":
        print(json.dumps(bench_matrix_tile(dev)), flush=True)
        return
    if args.workload == "few_rows":
        print(json.dumps({"n_gpus": 1, **bench_few_rows(dev, n=args.rows if args.rows != 8192 else 64)}), flush=True)
        return
    pristine, labels, g_lp, g_ent, cu = make_workload(dev)
    n_tok = pristine.shape[0]
    row_bytes = VOCAB * 2
    ring = max(1, min(args.ring, args.steps + args.warmup))
    bufs = [torch.empty_like(pristine) for _ in range(ring)]

    fwd_ms, bwd_ms, fused_ms = [], [], []
    last_fused = []

    def step_two_kernels(buf, timed):
        x = buf.requires_grad_(True)
        if timed:
            e0, e1, e2 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
            e0.record()
        lp, ent = logprobs_and_entropy_from_logits(x, labels, 1.0, inplace_backward=True)
        if timed:
            e1.record()
        # autograd.grad hands the gradient to the caller the way the next backward node (the
        # lm_head matmul) would receive it; .backward() on a leaf would add an accumulate step
        (grad,) = torch.autograd.grad([lp, ent], [x], [g_lp, g_ent])
        assert grad.data_ptr() == buf.data_ptr()  # written in place, nothing allocated
        if timed:
            e2.record()
            return e0, e1, e2
        return None

    def step_fused(buf, timed):
        if timed:
            e0, e1 = (torch.cuda.Event(enable_timing=True) for _ in range(2))
            e0.record()
        lp, ent, grad = fused_logprob_entropy_fwd_bwd(buf, labels, g_lp, g_ent, 1.0, inplace=True)
        assert grad.data_ptr() == buf.data_ptr()
        last_fused[:] = [buf, lp, ent]
        if timed:
            e1.record()
            return e0, e1
        return None

    def check_last_fused(sample=64):
        """Outside the timed region: a row sample of the last timed buffer (now holding the one-pass
        kernel's gradient) and its log-probs / entropies against the separate forward and backward
        kernels run on the same rows of the pristine logits."""
        buf, lp, ent = last_fused
        pick = torch.randperm(n_tok, generator=torch.Generator().manual_seed(5))[:sample].to(dev)
        x = pristine[pick].clone().requires_grad_(True)
        lp2, ent2 = logprobs_and_entropy_from_logits(x, labels[pick], 1.0)
        (g2,) = torch.autograd.grad([lp2, ent2], [x], [g_lp[pick], g_ent[pick]])
        got, want = buf[pick].float(), g2.float()
        e_lp = (lp[pick] - lp2).abs().max().item()
        e_ent = (ent[pick] - ent2).abs().max().item()
        e_grad = ((got - want).abs() - 2.0 ** -7 * want.abs()).max().item()
        ok = e_lp <= 2e-5 and e_ent <= 2e-5 and e_grad <= 4e-6 and bool(torch.isfinite(got).all())
        return ok, {"rows": sample, "logprob_abs_err": e_lp, "entropy_abs_err": e_ent,
                    "grad_excess_over_bf16_rounding": e_grad,
                    "against": "logprobs_and_entropy_from_logits + autograd on the same rows of the pristine logits"}

    def run_segment(step, count, timed):
        for b in bufs[:count]:
            b.detach_().copy_(pristine)  # fresh logits; outside the timed segment
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        evs = [step(bufs[i], timed) for i in range(count)]
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if timed:
            for ev in evs:
                if len(ev) == 3:
                    fwd_ms.append(ev[0].elapsed_time(ev[1]))
                    bwd_ms.append(ev[1].elapsed_time(ev[2]))
                else:
                    fused_ms.append(ev[0].elapsed_time(ev[1]))
        return dt

    def run(step):
        left = args.warmup
        while left > 0:
            c = min(left, ring)
            run_segment(step, c, False)
            left -= c
        total, left = 0.0, args.steps
        while left > 0:
            c = min(left, ring)
            total += run_segment(step, c, True)
            left -= c
        return total

    if args.workload == "ceilings":
        print(json.dumps({"workload": f"plain streams on {ring} x {n_tok} x {VOCAB} bf16 buffers", "n_gpus": 1, "unit": "GB/s",
                          "peak": HBM_PEAK_GBS, "entries": bench_ceilings(pristine, bufs, labels, dev)}), flush=True)
        return
    total_two = run(step_two_kernels)
    total = run(step_fused)
    checked, check_detail = check_last_fused()
    ceilings = bench_ceilings(pristine, bufs, labels, dev)
    ppo = None if args.no_ppo_step else bench_ppo_step(args, pristine, bufs, cu, ring, dev)

    ms_per_step = total / args.steps * 1e3
    tok_s = n_tok * args.steps / total
    fwd_avg = sum(fwd_ms) / len(fwd_ms)
    bwd_avg = sum(bwd_ms) / len(bwd_ms)
    fused_avg = sum(fused_ms) / len(fused_ms)
    small = 8 + 24                                  # label + logprob, entropy, 2 upstream grads / 4 row stats
    fwd_bytes = n_tok * (row_bytes + small)         # read logits
    bwd_bytes = n_tok * (2 * row_bytes + small)     # read logits, write grad
    step_bytes = n_tok * (3 * row_bytes + 2 * small)  # forward + backward, algorithmic
    fused_moved = n_tok * (2 * row_bytes + small)   # what the one-pass kernel has to move
    bwd_gbs = bwd_bytes / (bwd_avg * 1e-3) / 1e9
    fwd_gbs = fwd_bytes / (fwd_avg * 1e-3) / 1e9
    fused_gbs = step_bytes / (fused_avg * 1e-3) / 1e9
    fused_moved_gbs = fused_moved / (fused_avg * 1e-3) / 1e9
    traffic = measured_traffic("fused", n_tok)

    out = {
        "metric": METRIC,
        "value": tok_s,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "checked": checked,
        "check": check_detail,
        "config": {
            "workload": "BASELINE config 2: 16 sequences, lengths uniform in [512,3072], packed to one row; bf16 "
                        "logits [T_total,151936] ~N(0,3), 1% of rows with one +15 spike, temperature 1.0; "
                        "logprob+entropy forward and in-place backward, upstream grads ~N(0,1)",
            "total_tokens": n_tok,
            "vocab": VOCAB,
            "logits_gb": n_tok * row_bytes / 1e9,
            "entry": "openrlhf_amd.models.utils.fused_logprob_entropy_fwd_bwd(inplace=True)",
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "logprob_entropy_fused_pipe_kernel<bf16, lp+entropy, T=1> (forward+backward in one pass, in place)",
            "achieved": fused_moved_gbs,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": fused_moved_gbs / HBM_PEAK_GBS,
            "traffic": traffic,
            "bytes_per_launch": fused_moved,
            "avg_launch_ms": fused_avg,
            "note": "achieved = the bytes this kernel's algorithm moves (every row read once, its gradient written once: "
                    "2*V*2 B per token) / launch time. A separate forward and backward move 3*V*2 B per token (read, "
                    "read, write), the accounting of the metric's definition: see separate_passes_equivalent",
            "separate_passes_equivalent": {"bytes_per_launch": step_bytes, "achieved": fused_gbs,
                                           "frac": fused_gbs / HBM_PEAK_GBS},
            "ceiling_gbs": {k: round(v["gbs"], 1) for k, v in ceilings.items()},
            "frac_of_read_write_ceiling": fused_moved_gbs / max(ceilings["read_write_inplace"]["gbs"], ceilings["copy"]["gbs"]),
        },
        "autograd_two_kernels": {
            "entry": "logprobs_and_entropy_from_logits(inplace_backward=True) + torch.autograd.grad",
            "value": n_tok * args.steps / total_two,
            "unit": "tokens/s",
            "ms_per_step": total_two / args.steps * 1e3,
            "achieved_hbm_gbs": (fwd_bytes + bwd_bytes) * args.steps / total_two / 1e9,
            "kernels": {
                "logprob_entropy_bwd_kernel<bf16, lp+entropy, T=1> (in place)": {
                    "achieved": bwd_gbs, "frac": bwd_gbs / HBM_PEAK_GBS, "bytes_per_launch": bwd_bytes,
                    "avg_launch_ms": bwd_avg, "traffic": measured_traffic("backward", n_tok),
                },
                "logprob_entropy_fwd_kernel<bf16, lp+entropy, T=1>": {
                    "achieved": fwd_gbs, "frac": fwd_gbs / HBM_PEAK_GBS, "bytes_per_launch": fwd_bytes,
                    "avg_launch_ms": fwd_avg, "traffic": measured_traffic("forward", n_tok),
                },
            },
        },
    }
    if ppo is not None:
        out["ppo_actor_step_fused"] = ppo
    if not args.no_lmhead:
        del bufs[1:]  # the ring is no longer needed
        torch.cuda.empty_cache()
        out["lmhead_logprob_entropy"] = bench_lmhead(dev)
        # the same at the token count of the headline workload (config 2's packed batch)
        big = bench_lmhead(dev, n=n_tok, reps=2, roofline=False)
        out["lmhead_logprob_entropy"]["at_config2_tokens"] = {k: big[k] for k in ("config", "forward_ms", "routes", "checked", "check")}
    if not args.no_per_token:
        out["few_rows_n64"] = bench_few_rows(dev)
        entries = bench_per_token(args, dev, emit=False)
        out["per_token_config4"] = {
            "note": "the other kernels of the path at BASELINE config 4's size (4096 rows x 16384 columns fp32, 33.7 M real "
                    "tokens; 'packed' = flat tokens + cu_seqlens): ms per call through the Python API, algorithmic GB/s",
            "entries": {k[len("config4."):]: {"ms": round(v["ms"], 4), "gbs": round(v["achieved_gbs"], 0)}
                        for k, v in entries.items() if k.startswith("config4.")},
        }
    if not args.no_cpu_baseline:
        rows = min(args.cpu_rows, n_tok)
        cpu_tok_s, cpu_s, cpu_runs = cpu_baseline(pristine[:rows], labels[:rows], g_lp[:rows], g_ent[:rows])
        out["cpu_baseline"] = {
            "value": cpu_tok_s,
            "unit": "tokens/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"first {rows} rows of the same workload at full V (bf16->fp32 up-cast, entropy, gather - "
                      f"chunked logsumexp, autograd backward) on torch CPU, median of {cpu_runs} runs of "
                      f"{cpu_s:.2f} s after one warm-up run; {cpu_model()}, os.cpu_count()={os.cpu_count()}, "
                      f"torch.get_num_threads()={torch.get_num_threads()}",
        }
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()

"""CPU-only checks: the shared library exports every symbol the public header declares, the
ctypes binding covers them, argument validation returns error codes before anything touches a
GPU, and the Python mirrors raise the reference's exception types. No kernel is launched."""
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "openrlhf_amd.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(orlhf_[a-z0-9_]+)\s*\(", text)))


def test_header_binding_and_library_agree(lib):
    from openrlhf_amd import _lib

    names = _declared()
    assert len(names) >= 19
    assert sorted(_lib.SIGNATURES) == names
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in the header but not exported"
    assert lib.orlhf_version() == _lib.ABI_VERSION
    src = open(HEADER).read()
    assert f"#define ORLHF_ABI_VERSION {_lib.ABI_VERSION}" in src
    # enum values of the binding match the header
    for name, val in (("ORLHF_BF16", _lib.BF16), ("ORLHF_MASK_I64", _lib.MASK_I64), ("ORLHF_KL_K3", _lib.KL_K3),
                      ("ORLHF_AGG_ROW_MEAN", _lib.AGG_ROW_MEAN), ("ORLHF_IS_SEQ_MASK_TIS", _lib.IS_SEQ_MASK_TIS),
                      ("ORLHF_GROUP_NORM", _lib.GROUP_NORM), ("ORLHF_POLICY_GSPO", _lib.POLICY_GSPO)):
        assert re.search(rf"{name} = {val}\b", src), name


def test_entry_points_reject_bad_arguments_without_a_gpu(lib):
    from openrlhf_amd import _lib

    def err():
        return lib.orlhf_last_error().decode()

    assert lib.orlhf_logprob_entropy_fwd(None, 0, 4, 0, 0, None, 1.0, None, None, None, None, 0, None) == -1
    assert "vocab" in err()
    assert lib.orlhf_logprob_entropy_fwd(None, 0, 4, 8, 4, None, 1.0, None, None, None, None, 0, None) == -1
    assert "row_stride" in err()
    assert lib.orlhf_logprob_entropy_fwd(None, 0, 4, 8, 8, None, 1.0, None, None, None, None, 0, None) == -1
    assert "both NULL" in err()
    assert lib.orlhf_logprob_entropy_fwd(None, 0, 4, 8, 8, None, 0.0, 8, None, None, None, 0, None) == -1
    assert "temperature" in err()
    assert lib.orlhf_logprob_entropy_fwd(8, 9, 4, 8, 8, 8, 1.0, 8, None, None, None, 0, None) == -1
    assert "dtype" in err()
    assert lib.orlhf_logprob_entropy_fwd(None, 0, 0, 8, 8, None, 1.0, 8, None, None, None, 0, None) == 0  # empty: no launch
    assert lib.orlhf_logprob_entropy_bwd(None, None, 1, 2, 8, 8, 8, None, 1.0, None, None, None, None, None) == -1
    assert lib.orlhf_approx_kl_fwd(None, None, 0, 5, 7, None, None) == -1 and "estimator" in err()
    assert lib.orlhf_approx_kl_fwd(None, None, 0, 0, 0, None, None) == 0
    assert lib.orlhf_masked_aggregate_fwd(None, None, 9, 1, 1, None, 0, None, None, None, None, None) == -1
    assert "mask dtype" in err()
    p = _lib.PolicyParams()
    p.policy_type = 5
    assert lib.orlhf_policy_loss_fwd(None, None, None, None, 0, None, 0, 0, None, p, None, None, None, None, None) == -1
    p.policy_type, p.dual_clip = 0, 0.5
    assert lib.orlhf_policy_loss_fwd(None, None, None, None, 0, None, 0, 0, None, p, None, None, None, None, None) == -1
    assert "dual_clip" in err()
    p.dual_clip, p.is_correction = 0.0, 1
    assert lib.orlhf_policy_loss_fwd(None, None, None, None, 0, None, 0, 0, None, p, None, None, None, None, None) == -1
    assert "rollout" in err()
    # forward + gradient in one pass: only for the token mean over a given count
    q = _lib.PolicyParams()
    q.token_level = 1  # PPO, but no count given
    q.norm = _lib.make_norm(1, None, [])
    assert lib.orlhf_policy_loss_fwd_grad(None, None, None, None, 0, None, 0, 0, None, q, None, None, None, None, 8, None) == -1
    assert "given count" in err()
    q.norm = _lib.make_norm(1, 100.0, [])
    q.token_level = 0
    assert lib.orlhf_policy_loss_fwd_grad(None, None, None, None, 0, None, 0, 0, None, q, None, None, None, None, 8, None) == -1
    q.token_level = 1
    assert lib.orlhf_policy_loss_fwd_grad(None, None, None, None, 0, None, 0, 0, None, q, None, None, None, None, None, None) == -1
    assert "g_log_probs" in err()
    assert lib.orlhf_value_loss_fwd_grad(None, None, None, None, 0, 0, 0, None, 0, 0.0, _lib.make_norm(1, None, []), None, None, None, 8, None) == -1
    assert "given count" in err()
    assert lib.orlhf_group_normalize(None, None, 3, 0, 0, None, None, None, None) == -1
    assert lib.orlhf_group_normalize(None, None, 3, 2, 9, None, None, None, None) == -1
    assert lib.orlhf_gae_scan(None, None, None, 0, -1, 4, None, None, 1.0, 1.0, None, None, None) == -1
    assert lib.orlhf_token_workspace_bytes(4096, 16383) >= 4096 * 4 * 6 * 8  # 4096-token chunks, 6 quantities, fp64
    assert lib.orlhf_whiten_workspace_bytes(10) > 0


def test_matrix_core_entries_refuse_strides_their_offsets_cannot_address(lib):
    """Row strides of 2^23 elements and more would wrap the 32-bit byte offsets inside a slab (up to
    255 rows): refused before anything is launched. Odd strides and misaligned bases as well."""
    from openrlhf_amd import _lib

    def err():
        return lib.orlhf_last_error().decode()

    big = 1 << 23
    fwd = lambda hs, ws, h=256, w=256: lib.orlhf_lmhead_logprob_entropy_fwd(  # noqa: E731
        h, w, _lib.BF16, 4, 64, 100, hs, ws, None, 1.0, None, None, None, None, 0, 0, None, 0, None)
    assert fwd(big, 64) == -3 and "2^23" in err() and "hidden" in err()
    assert fwd(64, big) == -3 and "2^23" in err() and "weight" in err()
    assert fwd(65, 64) == -3 and "even" in err()
    assert fwd(64, 64, h=258) == -3 and "aligned" in err()
    assert fwd(32, 64) == -1 and "stride" in err()
    bwd = lib.orlhf_lmhead_logprob_entropy_bwd(256, 256, _lib.BF16, 4, 64, 100, 64, big, None, 1.0, None, None, None, None, 0, 0,
                                               256, 64, None, 64, None, 0, None)
    assert bwd == -3 and "2^23" in err()
    # the stored logits: whole tiles, at most the padded vocabulary, rows on 16 bytes
    kept = lambda cols, ld, ptr=256: lib.orlhf_lmhead_logprob_entropy_fwd(  # noqa: E731
        256, 256, _lib.BF16, 4, 64, 1000, 64, 64, None, 1.0, None, None, None, ptr, cols, ld, None, 0, None)
    assert kept(100, 1088) == -1 and "multiple of 256" in err()
    assert kept(1280, 1344) == -1 and "padded vocabulary" in err()
    assert kept(1024, 1028) == -3 and "multiple of 8" in err()
    assert kept(1024, 512) == -1 and "kept_logits" in err()
    assert kept(1024, 1088, ptr=None) == -1 and "NULL" in err()
    prod = lambda lda, ldb: lib.orlhf_matrix_tile_product(256, 256, _lib.BF16, 8, 8, 64, lda, ldb, 0, 0, 0, 256, 8, None)  # noqa: E731
    assert prod(big, 64) == -3 and "2^23" in err()
    assert lib.orlhf_matrix_tile_probe(256, 256, _lib.BF16, 8, 8, 64, 64, big, 0, 256, None) == -3 and "2^23" in err()


def _resource_report(source):
    """The compiler's own per-kernel resource remarks for one source file of the library, compiled
    for gfx950 with the library's flags: {mangled kernel name: {"VGPRs": n, "VGPRs Spill": n, ...}}."""
    import subprocess

    from openrlhf_amd.csrc import build as b

    cmd = [b.find_hipcc(), *b.HIPCC_FLAGS, "-I", os.path.join(ROOT, "include"), "--cuda-device-only", "-c",
           os.path.join(b.CSRC, source), "-o", os.devnull, "-Rpass-analysis=kernel-resource-usage"]
    out = subprocess.run(cmd, capture_output=True, text=True)
    assert out.returncode == 0, out.stderr[-2000:]
    kernels, name = {}, None
    for line in out.stderr.splitlines():
        m = re.search(r"remark:\s+Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            kernels[name] = {}
            continue
        m = re.search(r"remark:\s+(VGPRs Spill|ScratchSize \[bytes/lane\]|AGPRs|VGPRs): (\d+)", line)
        if m and name:
            kernels[name][m.group(1)] = int(m.group(2))
    return kernels


def test_matrix_core_kernels_do_not_spill():
    """With 256 accumulator registers per lane a few live values too many end up in scratch memory
    (and a spill inside the product loop would cost far more than it looks): no kernel of
    csrc/lmhead.hip may spill a vector register or use scratch."""
    kernels = _resource_report("lmhead.hip")
    tiles = {k: v for k, v in kernels.items() if v.get("AGPRs", 0) == 256}  # the kernels built on the 256 x 256 tile
    assert len(tiles) >= 20, sorted(kernels)
    for k, v in kernels.items():
        assert v["VGPRs Spill"] == 0 and v["ScratchSize [bytes/lane]"] == 0, (k, v)


def test_one_pass_kernel_of_the_benchmark_does_not_spill():
    """The one-pass forward + backward kernel holds a whole vocabulary row in registers (254-256 of
    them): its bf16, temperature-1 bodies with 38 chunks per lane, which the benchmark and the PPO
    step run, must stay free of spills (template arguments: dtype 1 = bf16, modes 0-2, 38 chunks)."""
    kernels = _resource_report("logprob_entropy_fused.hip")
    bodies = {k: v for k, v in kernels.items() if re.search(r"fused_pipe_kernelILi1ELi[012]ELi38E", k)}
    assert len(bodies) >= 6, sorted(kernels)
    for k, v in bodies.items():
        assert v["VGPRs Spill"] == 0 and v["ScratchSize [bytes/lane]"] == 0, (k, v)


def test_python_mirrors_raise_like_the_reference(lib):
    from openrlhf_amd.models.loss import PolicyLoss, ValueLoss
    from openrlhf_amd.models.utils import compute_approx_kl, log_probs_from_logits
    from openrlhf_amd.trainer.ppo_utils.experience_maker import group_normalize_rewards

    x = torch.zeros(2, 3)
    with pytest.raises(ValueError, match="Unknown kl_estimator"):
        compute_approx_kl(x, x, "k5")
    with pytest.raises(AssertionError):
        PolicyLoss(dual_clip=0.9)
    with pytest.raises(ValueError, match="Invalid vllm_is_correction_type"):
        PolicyLoss(vllm_is_correction_type="bad")
    with pytest.raises(ValueError, match="Invalid policy loss type"):
        PolicyLoss(policy_loss_type="bad")(x, x, x)
    assert PolicyLoss(policy_loss_type="gspo").token_level_loss is False
    assert ValueLoss().clip_eps is None and ValueLoss(0.2).token_level_loss is True
    with pytest.raises(Exception, match="Unkown advantage_estimator"):
        group_normalize_rewards(torch.zeros(4), None, 2, "bad")
    # no CPU fallback: CPU tensors are refused, loudly
    with pytest.raises(RuntimeError, match="GPU only"):
        log_probs_from_logits(torch.zeros(2, 8), torch.zeros(2, dtype=torch.long))
    with pytest.raises(RuntimeError, match="GPU only"):
        PolicyLoss()(x, x, x, action_mask=x)


def test_missing_library_fails_loudly(tmp_path):
    from openrlhf_amd import _lib

    with pytest.raises(ImportError, match="not built"):
        _lib.load(str(tmp_path / "nope.so"))


def test_row_view_and_norm_plumbing():
    from openrlhf_amd import _lib
    from openrlhf_amd.models.utils import _as_rows, _rows_of

    x = torch.zeros(2, 5, 16)
    rows, stride, aliases = _as_rows(x)
    assert rows.shape == (10, 16) and stride == 16 and rows.data_ptr() == x.data_ptr() and aliases
    y = torch.zeros(6, 20)[:, :16]
    rows, stride, aliases = _as_rows(y)
    assert rows.shape == (6, 16) and stride == 20 and rows.data_ptr() == y.data_ptr() and aliases
    z = torch.zeros(16, 6).t()
    rows, stride, aliases = _as_rows(z)
    assert rows.is_contiguous() and stride == 16 and not aliases
    assert _rows_of(torch.zeros(3, 4, 7), None) == (12, 7)
    # packed layout: the column count is a bound on the longest row, measured when it is not given
    assert _rows_of(torch.zeros(30), torch.tensor([0, 10, 30])) == (2, 20)
    assert _rows_of(torch.zeros(30), (torch.tensor([0, 10, 30]), 64)) == (2, 64)
    keep = []
    n = _lib.make_norm(2, None, keep)
    assert n.dp_size == 2.0 and n.norm_value != n.norm_value and not n.norm_dev
    n = _lib.make_norm(1, torch.tensor(7.0), keep)
    assert n.norm_value == 7.0 and not n.norm_dev
    assert _lib.mask_arg(None)[2] == _lib.MASK_NONE
    assert _lib.mask_arg(torch.ones(3, dtype=torch.bool))[2] == _lib.MASK_U8
    assert _lib.mask_arg(torch.ones(3, dtype=torch.int32))[2] == _lib.MASK_F32


def test_header_is_plain_c(tmp_path):
    """The public header compiles as C99 on its own (no C++, no HIP, no torch types), and a C
    caller can name every entry point."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    names = _declared()
    src = tmp_path / "use_header.c"
    body = "\n".join(f"    (void)&{n};" for n in names)
    src.write_text(f'#include "openrlhf_amd.h"\nint main(void) {{\n{body}\n    return 0;\n}}\n')
    res = subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only",
                          "-I", os.path.join(ROOT, "include"), str(src)], capture_output=True, text=True)
    assert res.returncode == 0, res.stderr


def test_later_entry_points_reject_bad_arguments_without_a_gpu(lib):
    """The sequence-level, layout, row-statistics and one-pass entries validate before they launch."""
    from openrlhf_amd import _lib

    def err():
        return lib.orlhf_last_error().decode()

    assert lib.orlhf_sequence_logps_fwd(None, None, 7, None, 2, 4, None, None, None, None) == -1 and "mask dtype" in err()
    assert lib.orlhf_sequence_logps_fwd(None, None, 1, None, 2, 4, None, None, None, None) == -1  # mask NULL for dtype u8
    assert lib.orlhf_sequence_logps_fwd(None, None, 0, None, 0, 4, None, None, None, None) == 0
    assert lib.orlhf_sequence_logps_bwd(None, 8, None, 0, None, None, 2, 4, 8, None) == -1 and "counts" in err()
    assert lib.orlhf_pair_loss_fwd(8, 8, None, None, 3, 9, 0.1, 0.0, 8, None, None, None) == -1 and "kind" in err()
    assert lib.orlhf_pair_loss_fwd(None, 8, None, None, 3, 0, 0.1, 0.0, 8, None, None, None) == -1
    assert lib.orlhf_pair_loss_fwd(8, 8, None, None, 3, 0, float("nan"), 0.0, 8, None, None, None) == -1 and "NaN" in err()
    assert lib.orlhf_pair_loss_fwd(8, 8, None, None, -1, 0, 0.1, 0.0, 8, None, None, None) == -1
    assert lib.orlhf_pair_loss_bwd(None, 8, 8, None, None, 0, 0, 0.1, 0.0, None, None, None) == 0  # nothing to do
    assert lib.orlhf_row_extents(8, 0, 2, 4, None, None, None, None) == -1 and "needs a mask" in err()
    assert lib.orlhf_row_extents(None, 1, 2, 4, None, None, None, None) == -1
    assert lib.orlhf_cu_seqlens(None, 3, None, None) == -1 and "NULL" in err()
    assert lib.orlhf_cu_seqlens(None, -1, 8, None) == -1
    assert lib.orlhf_pack_rows(8, 3, 2, 4, None, 8, 8, None) == -1 and "element size" in err()
    assert lib.orlhf_pack_rows(8, 4, 2, 4, None, None, 8, None) == -1
    assert lib.orlhf_pack_rows(None, 4, 0, 4, None, None, None, None) == 0
    assert lib.orlhf_pad_rows(8, 16, 8, 2, 4, 0, 0, 8, None) == -1 and "element size" in err()
    assert lib.orlhf_pad_rows(8, 4, None, 2, 4, 0, 0, 8, None) == -1
    assert lib.orlhf_kl_rows(8, 8, 0, None, 0, 2, 4, None, 5, 1, None, None, None, None) == -1 and "estimator" in err()
    assert lib.orlhf_kl_rows(None, None, 0, None, 0, 2, 4, None, 0, 1, None, None, None, None) == -1
    assert lib.orlhf_kl_rows(8, 8, 7, None, 0, 2, 4, None, 0, 1, None, None, None, None) == -1 and "dtype" in err()
    assert lib.orlhf_masked_normalize_rows(None, None, 0, 2, 4, None, 1e-8, None, None) == -1
    assert lib.orlhf_masked_normalize_rows(None, None, 0, 0, 4, None, 1e-8, None, None) == 0
    assert lib.orlhf_divide_rows_inplace(8, 1, 2, 8, 8, 0.0, None) == -1 and "divisor" in err()
    assert lib.orlhf_divide_rows_inplace(None, 1, 2, 8, 8, 0.5, None) == -1
    assert lib.orlhf_mask_counts(None, 1, 2, 4, None, None, None, None) == -1
    assert lib.orlhf_masked_aggregate_fwd(None, None, 0, 1, 1, None, 4, None, None, None, None, None) == -1 and "mode" in err()
    # the one-pass kernel keeps (most of) a row on one CU: rows beyond four times the resident part
    # are refused with a pointer to the two kernels
    assert lib.orlhf_logprob_entropy_fwd_bwd_max_vocab(_lib.BF16) == 524288
    assert lib.orlhf_logprob_entropy_fwd_bwd_max_vocab(_lib.F32) == 262144
    assert lib.orlhf_logprob_entropy_fwd_bwd_max_vocab(9) == 0
    assert lib.orlhf_logprob_entropy_fwd_bwd(8, 8, 1, 2, 600000, 600000, 600000, 8, 1.0, 8, None, 8, None, None, None) == -3
    assert "separate forward and backward" in err()
    assert lib.orlhf_logprob_entropy_fwd_bwd(16, 32 + 2, 1, 2, 1024, 1024, 1024, 8, 1.0, 8, None, 8, None, None, None) == -3
    assert "16-byte phases" in err()


def test_every_intra_package_import_resolves():
    """Names imported from one module of the package by another (or by a test) exist: a helper
    renamed in one file must not break a caller that is only imported lazily inside a function."""
    import ast
    import glob
    import importlib
    import os

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    files = glob.glob(os.path.join(root, "openrlhf_amd", "**", "*.py"), recursive=True)
    files += glob.glob(os.path.join(root, "tests", "*.py")) + [os.path.join(root, "bench.py")]
    missing = []
    for path in files:
        rel = os.path.relpath(path, root)
        tree = ast.parse(open(path).read())
        for node in ast.walk(tree):
            if not isinstance(node, ast.ImportFrom):
                continue
            if node.level > 0:
                parts = rel[:-3].split(os.sep)
                base = ".".join(parts[: len(parts) - node.level])
                mod = base + ("." + node.module if node.module else "")
            elif node.module and node.module.split(".")[0] == "openrlhf_amd":
                mod = node.module
            else:
                continue
            m = importlib.import_module(mod)
            for alias in node.names:
                if hasattr(m, alias.name):
                    continue
                try:
                    importlib.import_module(mod + "." + alias.name)
                except ImportError:
                    missing.append((rel, mod, alias.name))
    assert not missing, missing


def test_row_order_from_the_host_must_be_a_permutation():
    """A row order handed over as a CPU tensor is checked before it reaches the kernels (which trust
    it: a row that no entry names would keep whatever its outputs held)."""
    import torch

    from openrlhf_amd.trainer.ppo_utils.experience_maker import _order_arg

    cpu = torch.device("cpu")
    assert _order_arg(None, 4, cpu) is None
    assert _order_arg(torch.tensor([2, 0, 3, 1]), 4, cpu).tolist() == [2, 0, 3, 1]
    for bad in ([0, 0, 1, 2], [0, 1, 2, 4], [-1, 0, 1, 2]):
        with pytest.raises(ValueError, match="permutation"):
            _order_arg(torch.tensor(bad), 4, cpu)
    with pytest.raises(ValueError, match="entries"):
        _order_arg(torch.tensor([0, 1, 2]), 4, cpu)

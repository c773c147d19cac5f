"""Builds libopenrlhf_amd.so for gfx950 with hipcc (cross-compiles without a GPU).

    python -m openrlhf_amd.csrc.build            # build into openrlhf_amd/lib/
    python -m openrlhf_amd.csrc.build -DORLHF_ROW_UNROLL=4 --out /tmp/variant.so
"""
import argparse
import os
import shutil
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(CSRC)
LIB_DIR = os.path.join(PKG, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libopenrlhf_amd.so")

SOURCES = ["abi.hip", "logprob_entropy.hip", "logprob_entropy_fused.hip", "token_losses.hip", "advantages.hip",
           "sequence_losses.hip", "row_layout.hip", "row_stats.hip", "lmhead.hip", "actor_rows.hip"]

# -packed-fp32-ops off: v_pk_*_f32 forms generated from plain float code are not trusted on the
# target machines; the flag only concerns device code (the host pass warns that it is unknown).
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Werror=align-mismatch",
    "-Wno-unused-command-line-argument",
    "-Wno-option-ignored",
]


def find_hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm under /opt/rocm)")


def _run(cmd, verbose):
    if verbose:
        print("+", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = ("packed-fp32-ops' is not a recognized feature", "warning generated", "warnings generated")
    log = "\n".join(l for l in (res.stdout + res.stderr).splitlines() if not any(n in l for n in noise))
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{log}")
    return log


def build(extra_flags=(), out=LIB_PATH, verbose=True, sources=None, jobs=None):
    """Compiles every source to an object (in parallel, one hipcc per file) and links them."""
    srcs = [os.path.join(CSRC, s) for s in (sources or SOURCES) if os.path.exists(os.path.join(CSRC, s))]
    os.makedirs(os.path.dirname(out), exist_ok=True)
    hipcc = find_hipcc()
    include = os.path.join(PKG, "..", "include")
    jobs = jobs or min(len(srcs), max(1, min(8, os.cpu_count() or 1)))
    with tempfile.TemporaryDirectory(prefix="orlhf_build_") as tmpdir:
        objs = [os.path.join(tmpdir, os.path.basename(s) + ".o") for s in srcs]
        cmds = [[hipcc, *HIPCC_FLAGS, *extra_flags, "-I", include, "-c", s, "-o", o] for s, o in zip(srcs, objs)]
        with ThreadPoolExecutor(max_workers=jobs) as pool:
            logs = list(pool.map(lambda c: _run(c, verbose), cmds))
        tmp = out + ".tmp"
        logs.append(_run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp], verbose))
    log = "\n".join(l for l in logs if l.strip())
    if verbose and log.strip():
        print(log)
    os.replace(tmp, out)
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default=LIB_PATH)
    args, extra = ap.parse_known_args()
    print(build(extra_flags=extra, out=args.out))

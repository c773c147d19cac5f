"""Builds libopenrlhf_amd.so for gfx950 with hipcc (cross-compiles without a GPU).

    python -m openrlhf_amd.csrc.build            # build into openrlhf_amd/lib/
    python -m openrlhf_amd.csrc.build -DORLHF_ROW_UNROLL=4 --out /tmp/variant.so
"""
import argparse
import os
import shutil
import subprocess

CSRC = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(CSRC)
LIB_DIR = os.path.join(PKG, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libopenrlhf_amd.so")

SOURCES = ["abi.hip", "logprob_entropy.hip", "logprob_entropy_fused.hip", "token_losses.hip", "advantages.hip",
           "sequence_losses.hip", "row_layout.hip", "row_stats.hip"]

# -packed-fp32-ops off: v_pk_*_f32 forms generated from plain float code are not trusted on the
# target machines; the flag only concerns device code (the host pass warns that it is unknown).
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-option-ignored",
]


def find_hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm under /opt/rocm)")


def build(extra_flags=(), out=LIB_PATH, verbose=True, sources=None):
    srcs = [os.path.join(CSRC, s) for s in (sources or SOURCES) if os.path.exists(os.path.join(CSRC, s))]
    os.makedirs(os.path.dirname(out), exist_ok=True)
    tmp = out + ".tmp"
    cmd = [find_hipcc(), *HIPCC_FLAGS, *extra_flags, "-I", os.path.join(PKG, "..", "include"), *srcs, "-o", tmp]
    if verbose:
        print("+", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = ("packed-fp32-ops' is not a recognized feature", "warning generated", "warnings generated")
    log = "\n".join(l for l in (res.stdout + res.stderr).splitlines() if not any(n in l for n in noise))
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{log}")
    if verbose and log.strip():
        print(log)
    os.replace(tmp, out)
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default=LIB_PATH)
    args, extra = ap.parse_known_args()
    print(build(extra_flags=extra, out=args.out))

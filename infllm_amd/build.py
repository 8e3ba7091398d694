"""Build libinfllm_hip.so (gfx950) in-tree with hipcc.

    python -m infllm_amd.build

The library is cross-compiled (no GPU needed) and placed next to this file so
that it travels with the source tree.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libinfllm_hip.so")
SOURCES = ["abi.hip", "ingest.hip", "attn.hip", "score.hip", "retrieve.hip", "cache.hip", "stream.hip"]
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc_path():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm)")


def build(verbose=True, extra_flags=()):
    # ROCr (libhsa-runtime64) is linked for the DMA-engine copy of carved units; in a process it is the copy the HIP
    # runtime already loaded
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra_flags, *[os.path.join(CSRC, s) for s in SOURCES], "-o", LIB_PATH, "-lhsa-runtime64"]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass reports that it does not know the packed-fp32 feature; that is expected
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build())

"""Ahead-of-time build of libverinf_hip.so for gfx950 (no JIT, no torch extension).

    python -m verinf_amd.build

hipcc cross-compiles without a GPU; the shared library is written next to this
file and loaded through ctypes by `verinf_amd._lib`.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
SOURCES = ["field_ops.hip", "linalg.hip", "ntt.hip", "kquant.hip", "sumcheck.hip", "blake3.hip", "mle.hip"]
LIB = os.path.join(HERE, "libverinf_hip.so")

# -ffp-contract=off: the K-quant decode must round every fp32 operation separately.
# packed-fp32 ops are disabled for the device pass as this GPU pool requires.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wall", "-Wno-unused-function"]


def build(verbose: bool = False, out: str = LIB, extra_flags=()) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + list(extra_flags) + ["-shared", "-o", out] + [os.path.join(CSRC, s) for s in SOURCES]
    if verbose:
        print(" ".join(cmd))
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass notes that it does not know the packed-fp32 feature; that line is expected
    log = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + log)
    if log.strip():
        print(log)                      # compiler warnings
    return out


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))

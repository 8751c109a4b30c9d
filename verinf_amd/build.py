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
SOURCES = ["field_ops.hip", "linalg.hip", "ntt.hip", "kquant.hip", "sumcheck.hip", "blake3.hip", "mle.hip", "valu_probe.hip"]
LIB = os.path.join(HERE, "libverinf_hip.so")

# -ffp-contract=off: the K-quant decode must round every fp32 operation separately.
# packed-fp32 ops are disabled for the device pass as this GPU pool requires.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wall", "-Wno-unused-function"]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd))
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass notes that it does not know the packed-fp32 feature; that line is expected
    log = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + log)
    return log


def build(verbose: bool = False, out: str = LIB, extra_flags=()) -> str:
    """Compile every translation unit (in parallel, one hipcc each) and link the shared library."""
    import tempfile
    from concurrent.futures import ThreadPoolExecutor
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    jobs = max(1, min(len(SOURCES), int(os.environ.get("MAX_JOBS", os.cpu_count() or 1))))
    with tempfile.TemporaryDirectory(prefix="verinf_build_") as tmp:
        objs = [os.path.join(tmp, s.replace(".hip", ".o")) for s in SOURCES]
        cmds = [[hipcc] + FLAGS + list(extra_flags) + ["-c", "-o", o, os.path.join(CSRC, s)] for s, o in zip(SOURCES, objs)]
        with ThreadPoolExecutor(max_workers=jobs) as pool:
            logs = list(pool.map(lambda c: _run(c, verbose), cmds))
        logs.append(_run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + objs, verbose))
    log = "\n".join(l for l in logs if l.strip())
    if log.strip():
        print(log)                      # compiler warnings
    return out


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))

"""The CPU build of the NTT / LDE pass logic under AddressSanitizer and UBSan: every index map of the kernels is
walked over heap buffers of exactly the documented sizes (full and ragged widths, strided rows, the tile and chunk
boundaries, single- and multi-pass lengths), so an access outside them fails here and not as a GPU fault."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "cpu_build", "emul_sanitize_main.cpp")
EXE = os.path.join(HERE, "cpu_build", "emul_sanitize")


def test_pass_logic_is_clean_under_asan_and_ubsan():
    subprocess.check_call(["g++", "-O1", "-g", "-std=c++17", "-fsanitize=address,undefined",
                           "-fno-sanitize-recover=all", "-static-libasan", "-o", EXE, SRC])
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0")
    res = subprocess.run([EXE], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, timeout=600)
    assert res.returncode == 0, res.stdout[-4000:]
    assert res.stdout.strip().endswith("OK"), res.stdout[-2000:]

"""The CPU checker under AddressSanitizer and UndefinedBehaviorSanitizer (host code only, no GPU): oracle/Makefile's
`sanitize` target builds oracle/oracle_selftest.cpp with both and runs every function of fmha_oracle.hpp on small and
awkward shapes in exact-size buffers - one key, three queries over five keys, key counts around the block sizes, both
P modes, every layout of the GEMM.  An index that leaves its array or a signed overflow ends the run with a report."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_checker_is_clean_under_asan_and_ubsan():
    proc = subprocess.run(["make", "-B", "-C", os.path.join(ROOT, "oracle"), "sanitize"], stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert "oracle self-test under the sanitizers: ok" in proc.stdout

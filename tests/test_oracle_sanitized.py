"""The checker under a checker: the oracle's C++ source built with AddressSanitizer + UndefinedBehaviorSanitizer
(oracle/Makefile, target `sanitize`) runs the oracle's own CPU tests -- voxelization, hash, rulebooks with truncation
and empty inputs, convolutions, epilogues -- in a Python process that has the sanitizer runtime preloaded.  A report
(out-of-bounds access in a rulebook, signed overflow in an index product ...) aborts that process."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_oracle_tests_pass_under_address_and_ub_sanitizers():
    subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "-s", "sanitize"])
    lib = os.path.join(ROOT, "oracle", "libscn_oracle_san.so")
    asan = subprocess.check_output(["g++", "-print-file-name=libasan.so"], text=True).strip()
    ubsan = subprocess.check_output(["g++", "-print-file-name=libubsan.so"], text=True).strip()
    assert os.path.isabs(asan) and os.path.exists(asan), asan
    env = dict(os.environ, SCN_ORACLE_LIB=lib, LD_PRELOAD=asan + ":" + ubsan,
               ASAN_OPTIONS="detect_leaks=0:abort_on_error=1", UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1",
               OMP_NUM_THREADS="4")
    r = subprocess.run([sys.executable, "-m", "pytest", os.path.join(ROOT, "tests", "test_oracle.py"), "-x", "-q",
                        "-p", "no:cacheprovider"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env,
                       cwd=ROOT, timeout=1500)
    tail = r.stdout[-4000:]
    print(tail)
    assert r.returncode == 0, tail
    assert "runtime error" not in r.stdout and "AddressSanitizer" not in r.stdout
    assert " passed" in tail

"""The oracle's C source under the undefined-behaviour sanitizer: the golden vectors, the
primitives' known answers and the LBG / RVQ / OPQ / TSVQ checks are run once more against a build
with -fsanitize=undefined -fno-sanitize-recover (any finding aborts the run).  The C ABI library is
the only unsafe surface of the path besides the oracle; its host mirror is plain C++ over it."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_oracle_suite_under_ubsan():
    odir = os.path.join(ROOT, "oracle")
    subprocess.check_call(["make", "-B", "-C", odir, "libvq_oracle_ubsan.so"], stdout=subprocess.DEVNULL)
    env = dict(os.environ, VQ_ORACLE_LIB=os.path.join(odir, "libvq_oracle_ubsan.so"),
               UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1")
    res = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-p", "no:cacheprovider",
                          os.path.join(ROOT, "tests", "test_golden.py"),
                          os.path.join(ROOT, "tests", "test_oracle_prims.py"),
                          os.path.join(ROOT, "tests", "test_oracle_lbg.py")],
                         cwd=ROOT, env=env, capture_output=True, text=True)
    assert res.returncode == 0, res.stdout[-3000:] + res.stderr[-3000:]
    assert "runtime error" not in res.stderr

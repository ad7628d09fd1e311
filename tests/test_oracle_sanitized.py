"""The oracle's C source under the sanitizers: the golden vectors, the primitives' known answers
and the LBG / RVQ / OPQ / TSVQ checks are run once more against a build with
-fsanitize=undefined, and against one with -fsanitize=address,undefined, both with
-fno-sanitize-recover (any finding aborts the run).  The C ABI library is the only unsafe surface
of the path besides the oracle; its host mirror is plain C++ over it."""
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


def asan_env(**extra):
    """Environment of a child interpreter that may load address-sanitized libraries: the
    sanitizer's runtime goes in front of whatever is preloaded already, and the C++ runtime with
    it (the sanitizer looks up the real __cxa_throw when it starts; in an interpreter that loads
    libstdc++ only later it finds none and the first C++ exception aborts)."""
    rt = subprocess.check_output(["gcc", "-print-file-name=libasan.so"], text=True).strip()
    cxx = subprocess.check_output(["gcc", "-print-file-name=libstdc++.so.6"], text=True).strip()
    pre = os.environ.get("LD_PRELOAD", "")
    return dict(os.environ, LD_PRELOAD=rt + ":" + cxx + (":" + pre if pre else ""),
                ASAN_OPTIONS="detect_leaks=0:halt_on_error=1:abort_on_error=1:protect_shadow_gap=0",
                UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1", **extra)


def test_oracle_suite_under_asan_and_ubsan():
    odir = os.path.join(ROOT, "oracle")
    subprocess.check_call(["make", "-B", "-C", odir, "libvq_oracle_asan.so"], stdout=subprocess.DEVNULL)
    env = asan_env(VQ_ORACLE_LIB=os.path.join(odir, "libvq_oracle_asan.so"))
    res = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-p", "no:cacheprovider",
                          os.path.join(ROOT, "tests", "test_golden.py"),
                          os.path.join(ROOT, "tests", "test_oracle_prims.py"),
                          os.path.join(ROOT, "tests", "test_oracle_lbg.py")],
                         cwd=ROOT, env=env, capture_output=True, text=True)
    assert res.returncode == 0, res.stdout[-3000:] + res.stderr[-3000:]
    assert "AddressSanitizer" not in res.stderr and "runtime error" not in res.stderr

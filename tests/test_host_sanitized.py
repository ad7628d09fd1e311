"""The host mirror of the crate's API (vq_amd/host/vq.hpp and the flat C entry points of
vq_host_c.cpp) under -fsanitize=address,undefined WITHOUT a GPU: a C++ driver
(tests/stub/host_sanitized_main.cpp) linked against a stand-in for libvqhip
(tests/stub/vqhip_stub.cpp) whose "device" memory is host memory of exactly the size asked for.
Packing of per-row vectors, validation and panic texts, index streams, the call sequences and
buffer sizes of the four quantizers and the C flattening are host code; the kernels are not."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
STUB = os.path.join(ROOT, "tests", "stub")


def test_host_mirror_under_address_and_ub_sanitizers(tmp_path):
    exe = str(tmp_path / "host_sanitized")
    flags = ["-O1", "-g", "-std=c++17", "-fno-omit-frame-pointer", "-fsanitize=address,undefined",
             "-fno-sanitize-recover=all", "-ffp-contract=off", "-Wall"]
    subprocess.check_call(["g++", *flags, os.path.join(STUB, "host_sanitized_main.cpp"),
                           os.path.join(STUB, "vqhip_stub.cpp"), "-o", exe, "-lpthread"])
    # the harness preloads a library of its own; the sanitizer's runtime has to come first
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:verify_asan_link_order=0",
               UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1")
    res = subprocess.run([exe], env=env, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-4000:]
    assert "host mirror: ok" in res.stdout
    assert "AddressSanitizer" not in res.stderr and "runtime error" not in res.stderr

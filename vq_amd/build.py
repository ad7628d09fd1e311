"""Builds libvqhip.so (HIP kernels + C ABI) for gfx950, in-tree."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libvqhip.so")
SRC = [os.path.join(HERE, "csrc", f) for f in
       ("vq_api.hip", "vq_api_rvq_opq.hip", "vq_api_tsvq.hip", "vq_api_bigk.hip")]

# -ffp-contract=off: the exact kernels must round multiply and add separately, as the
#   reference's Rust code does.  Fused operations are written explicitly where wanted.
# -packed-fp32-ops disabled: no v_pk_*_f32 may be generated.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-fno-fast-math", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    # matrix-core accumulators stay in architectural VGPRs (no copies through the AGPR half)
    "-mllvm", "-amdgpu-mfma-vgpr-form",
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(l for l in (res.stdout + res.stderr).splitlines()
                    if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)


def build_lib(verbose=False, extra=()):
    """Compiles every translation unit (in parallel) and links libvqhip.so."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, os.path.basename(s)[:-4] + ".o") for s in SRC]
    with ThreadPoolExecutor(max_workers=4) as ex:
        list(ex.map(lambda so: _run([hipcc, *FLAGS, *extra, "-c", so[0], "-o", so[1]], verbose),
                    zip(SRC, objs)))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs], verbose)
    return LIB


HOST_LIB = os.path.join(HERE, "libvqhost.so")


HOST_LIB_UBSAN = os.path.join(HERE, "libvqhost_ubsan.so")
HOST_LIB_ASAN = os.path.join(HERE, "libvqhost_asan.so")


def build_host(verbose=False, ubsan=False, asan=False):
    """Compiles the C++ host mirror (plain g++: it only needs the C ABI) and links it to libvqhip.
    ubsan: a second build under the undefined-behaviour sanitizer (aborts at the first finding),
    which the tests load through VQ_HOST_LIB.  asan: a third one under the address and the
    undefined-behaviour sanitizers (the process that loads it preloads libasan.so)."""
    out = HOST_LIB_ASAN if asan else HOST_LIB_UBSAN if ubsan else HOST_LIB
    opt = ["-O1", "-g", "-fno-omit-frame-pointer", "-fsanitize=address,undefined", "-fno-sanitize-recover=all"] \
        if asan else \
        ["-O1", "-g", "-fsanitize=undefined", "-fno-sanitize-recover=undefined", "-static-libubsan"] \
        if ubsan else ["-O3"]
    cmd = ["g++", *opt, "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off", "-Wall",
           os.path.join(HERE, "host", "vq_host_c.cpp"), "-o", out,
           "-L" + HERE, "-lvqhip", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("g++ failed:\n" + res.stdout + res.stderr)
    return out


if __name__ == "__main__":
    print(build_lib(verbose=True, extra=sys.argv[1:]))
    print(build_host(verbose=True))
    print(build_host(verbose=True, ubsan=True))
    print(build_host(verbose=True, asan=True))

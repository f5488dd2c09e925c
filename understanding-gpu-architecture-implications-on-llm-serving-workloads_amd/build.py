"""Build script for the MI355X serving kernels (gfx950 only).

Produces, next to the sources:
    libmi355_serving.so        HIP kernels + C ABI (include/mi355_serving.h); no torch dependency
    gemm_unified/_C.so         torch operators gemm_unified::finegemm_N, linked against the library above
    fmha_unified/_C.so         torch operators fmha_unified::finefmha_N

hipcc cross-compiles for gfx950 without a GPU. Usage: ``python build.py [--only lib|ops]`` or
``from build import build_all``.
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
INCLUDE = os.path.join(ROOT, "include")
LIB_NAME = "libmi355_serving.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -packed-fp32-ops: keep the compiler from forming v_pk_{add,mul,fma}_f32 out of scalar float code.
DEVICE_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wno-inline-asm", "-Wno-unused-command-line-argument",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
KERNEL_SOURCES = ["csrc/hgemm.hip", "csrc/fmha_fwd.hip", "csrc/fmha_decode.hip", "csrc/glue.hip", "csrc/capi.hip"]
# Per-source additions. The GEMM keeps its MFMA accumulators in ordinary VGPRs: left to itself the compiler moves part of
# them to AGPRs in the 4-wave kernels and then shuffles them back and forth inside the K loop.
SOURCE_FLAGS = {"csrc/hgemm.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def _run(cmd, quiet_patterns=("is not a recognized feature for this target",)):
    proc = subprocess.run(cmd, cwd=HERE, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if not any(p in l for p in quiet_patterns))
    if proc.returncode != 0:
        raise RuntimeError("command failed (%d): %s\n%s" % (proc.returncode, " ".join(cmd), out))
    if out.strip():
        print(out)


def build_library(verbose=True):
    """Compile the HIP kernels and the C ABI into libmi355_serving.so (one object per source, compiled side by side)."""
    import tempfile
    from concurrent.futures import ThreadPoolExecutor

    with tempfile.TemporaryDirectory(prefix="mi355_build_") as tmp:
        jobs = []
        for src in KERNEL_SOURCES:
            obj = os.path.join(tmp, os.path.basename(src) + ".o")
            cmd = [HIPCC] + DEVICE_FLAGS + SOURCE_FLAGS.get(src, []) + ["-I", INCLUDE, "-c", src, "-o", obj]
            if verbose:
                print("[build] " + " ".join(cmd))
            jobs.append((cmd, obj))
        with ThreadPoolExecutor(max_workers=min(len(jobs), os.cpu_count() or 1, 8)) as pool:
            list(pool.map(lambda job: _run(job[0]), jobs))
        link = [HIPCC, "--offload-arch=gfx950", "-fPIC", "-shared"] + [obj for _, obj in jobs] + ["-o", LIB_PATH]
        if verbose:
            print("[build] " + " ".join(link))
        _run(link)
    return LIB_PATH


def _torch_flags():
    import torch
    from torch.utils import cpp_extension as ce

    inc = []
    for p in ce.include_paths():
        inc += ["-isystem", p]
    inc += ["-isystem", sysconfig.get_paths()["include"], "-isystem", "/opt/rocm/include"]
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    libdir = ce.library_paths()[0]
    defs = ["-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-D_GLIBCXX_USE_CXX11_ABI=%d" % abi,
            "-DTORCH_API_INCLUDE_EXTENSION_H", "-DTORCH_EXTENSION_NAME=_C"]
    libs = ["-L" + libdir, "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
            "-Wl,-rpath," + libdir]
    return inc, defs, libs


def build_operator(pkg, source, verbose=True):
    """Compile one torch operator module (<pkg>/_C.so). Host code only; the kernels live in the library."""
    inc, defs, libs = _torch_flags()
    out = os.path.join(HERE, pkg, "_C.so")
    cxx = os.environ.get("CXX", "g++")
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-Wno-attributes"] + defs + ["-I", INCLUDE] + inc + \
          [os.path.join(pkg, "csrc", source), "-o", out, "-L" + HERE, "-lmi355_serving", "-Wl,-rpath,$ORIGIN/.."] + libs
    if verbose:
        print("[build] " + " ".join(cmd))
    _run(cmd)
    return out


def build_all(verbose=True):
    build_library(verbose)
    build_operator("gemm_unified", "gemm_ops.cpp", verbose)
    build_operator("fmha_unified", "fmha_ops.cpp", verbose)


def is_built():
    return all(os.path.exists(p) for p in (LIB_PATH, os.path.join(HERE, "gemm_unified", "_C.so"),
                                           os.path.join(HERE, "fmha_unified", "_C.so")))


if __name__ == "__main__":
    only = sys.argv[2] if len(sys.argv) > 2 and sys.argv[1] == "--only" else None
    if only == "lib":
        build_library()
    elif only == "ops":
        build_operator("gemm_unified", "gemm_ops.cpp")
        build_operator("fmha_unified", "fmha_ops.cpp")
    else:
        build_all()

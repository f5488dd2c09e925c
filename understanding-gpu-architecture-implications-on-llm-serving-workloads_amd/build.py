"""Build script for the MI355X serving kernels (gfx950 only).

Produces, inside the three packages:
    mi355_serving/libmi355_serving.so   HIP kernels + C ABI (include/mi355_serving.h); no torch dependency
    mi355_serving/libmi355_serving_timeline.so   profiling twin: the attention kernels also record per-workgroup time stamps
    gemm_unified/_C.so                  torch operators gemm_unified::finegemm_N, linked against the library above
    fmha_unified/_C.so                  torch operators fmha_unified::finefmha_N
Each _C.so finds the library through RUNPATH $ORIGIN/../mi355_serving: the packages sit side by side both in the source
tree and in site-packages.

hipcc cross-compiles for gfx950 without a GPU. Usage: ``python build.py [--only lib|ops]`` or
``from build import build_all``.

Environment (the knobs of the reference's kernels/*/pkg/setup.py): GPU_ARCHS (setup.py:222; only "gfx950" or "native" are
accepted here), MAX_JOBS (setup.py:284-305; number of sources compiled side by side), HIPCC, CXX.
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
INCLUDE = os.path.join(ROOT, "include")
LIB_NAME = "libmi355_serving.so"
LIB_DIR = os.path.join(HERE, "mi355_serving")
LIB_PATH = os.path.join(LIB_DIR, LIB_NAME)

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -packed-fp32-ops: keep the compiler from forming v_pk_{add,mul,fma}_f32 out of scalar float code.
DEVICE_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wno-inline-asm", "-Wno-unused-command-line-argument",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
KERNEL_SOURCES = ["csrc/hgemm.hip", "csrc/fmha_fwd.hip", "csrc/fmha_decode.hip", "csrc/glue.hip", "csrc/capi.hip"]
# A source listed here is compiled once per entry, each time with that entry's defines, into objects of its own (side by
# side with the others): the GEMM source holds every tile shape for two element types and three layouts, and one
# compiler process per element type halves the time the build waits for it.
SOURCE_PARTS = {"csrc/hgemm.hip": (("fp16", ["-DMI355_HGEMM_PART=0"]), ("bf16", ["-DMI355_HGEMM_PART=1"]))}
# Per-source additions. The GEMM keeps its MFMA accumulators in ordinary VGPRs: left to itself the compiler moves part of
# them to AGPRs in the 4-wave kernels and then shuffles them back and forth inside the K loop.
SOURCE_FLAGS = {"csrc/hgemm.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def check_archs():
    """GPU_ARCHS as the reference's setup.py reads it (';'-separated). This build has gfx950 code only."""
    archs = [a for a in os.environ.get("GPU_ARCHS", "gfx950").split(";") if a]
    bad = [a for a in archs if a not in ("gfx950", "native")]
    if bad:
        raise SystemExit("GPU_ARCHS=%s: these kernels are written for gfx950 (MI355X) only" % ";".join(archs))


def max_jobs(n_sources):
    try:
        jobs = int(os.environ.get("MAX_JOBS", "0"))
    except ValueError:
        jobs = 0
    if jobs < 1:
        jobs = min(os.cpu_count() or 1, 8)
    return max(1, min(jobs, n_sources))


def _run(cmd, quiet_patterns=("is not a recognized feature for this target",)):
    proc = subprocess.run(cmd, cwd=HERE, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if not any(p in l for p in quiet_patterns))
    if proc.returncode != 0:
        raise RuntimeError("command failed (%d): %s\n%s" % (proc.returncode, " ".join(cmd), out))
    if out.strip():
        print(out)


TIMELINE_LIB_NAME = "libmi355_serving_timeline.so"
TIMELINE_LIB_PATH = os.path.join(LIB_DIR, TIMELINE_LIB_NAME)
# Sources that carry per-workgroup time stamps when compiled with -DMI355_TIMELINE (csrc/mi355_timeline.h).
TIMELINE_SOURCES = ("csrc/hgemm.hip", "csrc/fmha_fwd.hip", "csrc/fmha_decode.hip")
# Yardstick kernels that exist in the profiling twin only (a read-only kernel, matrix instructions on registers, matrix and
# VALU instructions side by side on one SIMD).
TIMELINE_ONLY_SOURCES = ("csrc/timeline_probes.hip",)


def build_library(verbose=True):
    """Compile the HIP kernels and the C ABI into libmi355_serving.so (one object per source, compiled side by side), and
    the profiling twin libmi355_serving_timeline.so: the same objects, except that the GEMM and attention sources are compiled a
    second time with -DMI355_TIMELINE (`bench.py --timeline` loads it; nothing else does)."""
    import tempfile
    from concurrent.futures import ThreadPoolExecutor

    check_archs()
    with tempfile.TemporaryDirectory(prefix="mi355_build_") as tmp:
        jobs = []
        objs, tl_objs = [], []

        def add(src, defines, suffix):
            made = []
            for tag, part_defines in SOURCE_PARTS.get(src, (("", []),)):
                obj = os.path.join(tmp, os.path.basename(src) + (("." + tag) if tag else "") + suffix + ".o")
                cmd = [HIPCC] + DEVICE_FLAGS + SOURCE_FLAGS.get(src, []) + part_defines + defines + ["-I", INCLUDE, "-c", src, "-o", obj]
                jobs.append((cmd, obj))
                made.append(obj)
            return made

        for src in KERNEL_SOURCES:
            plain = add(src, [], "")
            objs += plain
            tl_objs += add(src, ["-DMI355_TIMELINE"], ".timeline") if src in TIMELINE_SOURCES else plain
        for src in TIMELINE_ONLY_SOURCES:
            tl_objs += add(src, ["-DMI355_TIMELINE"], ".timeline")
        # the longest compilations first, so that they do not start behind the short ones
        jobs.sort(key=lambda job: 0 if "hgemm" in job[1] else 1 if "fmha_fwd" in job[1] else 2)
        if verbose:
            for cmd, _ in jobs:
                print("[build] " + " ".join(cmd))
        with ThreadPoolExecutor(max_workers=max_jobs(len(jobs))) as pool:
            list(pool.map(lambda job: _run(job[0]), jobs))
        for out, these in ((LIB_PATH, objs), (TIMELINE_LIB_PATH, tl_objs)):
            link = [HIPCC, "--offload-arch=gfx950", "-fPIC", "-shared"] + these + ["-o", out]
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
          [os.path.join(pkg, "csrc", source), "-o", out, "-L" + LIB_DIR, "-lmi355_serving", "-Wl,-rpath,$ORIGIN/../mi355_serving"] + libs
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


def run_setup(dist_name, op_packages, rel, py_modules=()):
    """setuptools.setup() for `op_packages` (gemm_unified and / or fmha_unified) plus the mi355_serving package that
    holds the kernel library. `rel` is the path from the calling setup.py (the current directory) to this directory.
    The shared objects are package data: they are compiled (if missing) by build_py, before the data files are
    collected, so a clean checkout installs complete packages."""
    from setuptools import Command, setup
    from setuptools.command.build_py import build_py

    class BuildExt(Command):
        description = "compile libmi355_serving.so and the torch operator modules in-tree"
        user_options = [("inplace", "i", "accepted for compatibility; the build is always in-tree")]

        def initialize_options(self):
            self.inplace = True

        def finalize_options(self):
            pass

        def run(self):
            build_all(verbose=True)

    class BuildPy(build_py):
        def run(self):
            check_archs()
            if not is_built():
                build_all(verbose=True)
            super().run()

    packages = list(op_packages) + ["mi355_serving"]
    data = {p: ["_C.so"] for p in op_packages}
    data["mi355_serving"] = [LIB_NAME]
    setup(
        name=dist_name,
        version="2.0.0",
        description="MI355X (gfx950) fp16 GEMM and fused attention forward behind the gemm_unified / fmha_unified operators",
        packages=packages,
        package_dir={p: os.path.join(rel, p) for p in packages} if rel != "." else {"": "."},
        package_data=data,
        py_modules=list(py_modules),
        cmdclass={"build_ext": BuildExt, "build_py": BuildPy},
        python_requires=">=3.8",
        zip_safe=False,
    )


if __name__ == "__main__":
    only = sys.argv[2] if len(sys.argv) > 2 and sys.argv[1] == "--only" else None
    if only == "lib":
        build_library()
    elif only == "ops":
        build_operator("gemm_unified", "gemm_ops.cpp")
        build_operator("fmha_unified", "fmha_ops.cpp")
    else:
        build_all()

"""`python setup.py install` of the packages (the reference's documented way of building them, README.md:37-58) into a
scratch root: where the files land, what the operator modules' RUNPATH says, and that the installed copy imports on its own
(without the source tree on sys.path). Runs without a GPU; nothing is compiled when the in-tree build already exists."""
import glob
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "understanding-gpu-architecture-implications-on-llm-serving-workloads_amd")


def install(script_dir, tmp_path):
    root = tmp_path / "root"
    cmd = [sys.executable, "setup.py", "-q", "egg_info", "--egg-base", str(tmp_path), "build", "--build-base",
           str(tmp_path / "b"), "install", "--root", str(root)]
    proc = subprocess.run(cmd, cwd=script_dir, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=900)
    assert proc.returncode == 0, proc.stdout[-4000:]
    hits = glob.glob(str(root / "**" / "mi355_serving" / "libmi355_serving.so"), recursive=True)
    assert len(hits) == 1, hits
    return os.path.dirname(os.path.dirname(hits[0]))   # the site-packages directory of the scratch root


def runpath(so):
    out = subprocess.run(["readelf", "-d", so], stdout=subprocess.PIPE, text=True, check=True).stdout
    lines = [l for l in out.splitlines() if "RUNPATH" in l or "RPATH" in l]
    assert lines, out
    return lines[0]


@pytest.mark.parametrize("script,packages,absent", [
    (".", ["gemm_unified", "fmha_unified"], []),
    (os.path.join("kernels", "gemm", "pkg"), ["gemm_unified"], ["fmha_unified"]),
    (os.path.join("kernels", "fmha", "pkg"), ["fmha_unified"], ["gemm_unified"]),
])
def test_setup_py_install_lands_a_working_copy(tmp_path, script, packages, absent):
    site = install(os.path.join(PKG, script), tmp_path)
    assert os.path.isfile(os.path.join(site, "mi355_serving", "__init__.py"))
    for p in packages:
        so = os.path.join(site, p, "_C.so")
        assert os.path.isfile(so) and os.path.isfile(os.path.join(site, p, "ops.py"))
        assert "$ORIGIN/../mi355_serving" in runpath(so)
    for p in absent:
        assert not os.path.exists(os.path.join(site, p))
    # import the installed copy alone: the operator modules must find the kernel library through their RUNPATH, and the
    # ctypes binding must find it next to itself
    code = ("import sys, os; sys.path.insert(0, %r); import torch, mi355_serving; mi355_serving.load(); "
            "assert os.path.dirname(mi355_serving.LIB_PATH).startswith(%r); " % (site, site))
    for p in packages:
        op = "finegemm_16" if p == "gemm_unified" else "finefmha_7"
        code += "import %s; assert %s.__file__.startswith(%r); torch.ops.%s.%s; " % (p, p, site, p, op)
    env = {k: v for k, v in os.environ.items() if k != "PYTHONPATH"}
    proc = subprocess.run([sys.executable, "-c", code], cwd=str(tmp_path), env=env, stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout[-4000:]


def test_build_rejects_other_gpu_archs():
    env = dict(os.environ, GPU_ARCHS="gfx90a;gfx942")
    proc = subprocess.run([sys.executable, "-c", "import build; build.check_archs()"], cwd=PKG, env=env,
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode != 0 and "gfx950" in proc.stdout
    for ok in ("gfx950", "native", "gfx950;native"):
        env = dict(os.environ, GPU_ARCHS=ok)
        assert subprocess.run([sys.executable, "-c", "import build; build.check_archs()"], cwd=PKG, env=env).returncode == 0

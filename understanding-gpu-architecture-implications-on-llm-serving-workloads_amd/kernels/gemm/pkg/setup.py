"""setup.py of the `gemm_unified` package alone, at the path the reference documents
(`cd kernels/gemm/pkg && python setup.py install`, README.md:37-58; reference script: kernels/gemm/pkg/setup.py).
Installs gemm_unified (with its _C.so) and the shared kernel library package mi355_serving; compiles first if needed.
Environment: GPU_ARCHS (gfx950 only), MAX_JOBS, HIPCC, CXX.
"""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
TOP = os.path.normpath(os.path.join(HERE, "..", "..", ".."))
sys.path.insert(0, TOP)
import build as mi355_build  # noqa: E402

if __name__ == "__main__":
    os.chdir(HERE)
    mi355_build.run_setup("gemm_unified", ["gemm_unified"], rel=os.path.join("..", "..", ".."))

"""setup.py for the MI355X `gemm_unified` and `fmha_unified` packages (both at once).

Counterpart of the reference's kernels/gemm/pkg/setup.py and kernels/fmha/pkg/setup.py (one package each, built with
CUDAExtension + hipify); kernels/gemm/pkg/setup.py and kernels/fmha/pkg/setup.py below this directory install one
package each, as the reference's README has it. Both packages share one kernel library, shipped as the data file of a
third package `mi355_serving` (its ctypes binding), and everything is compiled by plain hipcc / g++ commands (see
build.py): gfx950 only, no hipify step, no rocWMMA / CUTLASS / ThunderKittens include paths.

    python setup.py build_ext --inplace      # compile in-tree (what build.py does)
    python setup.py install                  # compile if needed, then install the packages with their shared objects

Environment: GPU_ARCHS (gfx950 only), MAX_JOBS, HIPCC (default /opt/rocm/bin/hipcc), CXX (default g++).
"""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import build as mi355_build  # noqa: E402

if __name__ == "__main__":
    os.chdir(HERE)
    mi355_build.run_setup("mi355-serving-kernels", ["gemm_unified", "fmha_unified"], rel=".", py_modules=["llama_layer"])

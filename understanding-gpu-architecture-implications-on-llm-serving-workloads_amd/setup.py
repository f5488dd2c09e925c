"""setup.py for the MI355X `gemm_unified` and `fmha_unified` packages.

Counterpart of the reference's kernels/gemm/pkg/setup.py and kernels/fmha/pkg/setup.py (one package each, built with
CUDAExtension + hipify). Here both packages share one kernel library and are built by plain hipcc / g++ commands
(see build.py): gfx950 only, no hipify step, no rocWMMA / CUTLASS / ThunderKittens include paths.

    python setup.py build_ext --inplace      # compile in-tree (what build.py does)
    python setup.py install                  # compile, then install both packages with their shared objects

Environment: HIPCC (default /opt/rocm/bin/hipcc), CXX (default g++).
"""
import os
import sys

from setuptools import Command, setup
from setuptools.command.build_py import build_py

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import build as mi355_build  # noqa: E402


class BuildExt(Command):
    description = "compile libmi355_serving.so and the two torch operator modules in-tree"
    user_options = [("inplace", "i", "accepted for compatibility; the build is always in-tree")]

    def initialize_options(self):
        self.inplace = True

    def finalize_options(self):
        pass

    def run(self):
        mi355_build.build_all(verbose=True)


class BuildPy(build_py):
    def run(self):
        if not mi355_build.is_built():
            mi355_build.build_all(verbose=True)
        super().run()


setup(
    name="mi355-serving-kernels",
    version="1.0.0",
    description="MI355X (gfx950) fp16 GEMM and fused attention forward behind the gemm_unified / fmha_unified operators",
    packages=["gemm_unified", "fmha_unified"],
    package_dir={"": "."},
    package_data={"gemm_unified": ["_C.so"], "fmha_unified": ["_C.so"]},
    data_files=[("", ["libmi355_serving.so"])] if os.path.exists(os.path.join(HERE, "libmi355_serving.so")) else [],
    py_modules=["mi355_serving"],
    cmdclass={"build_ext": BuildExt, "build_py": BuildPy},
    zip_safe=False,
)

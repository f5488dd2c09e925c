"""gemm_unified for MI355X: same package surface as the reference (kernels/gemm/pkg/gemm_unified/__init__.py:1-2).

Importing the package loads ``_C`` (whose static registrars define the ``torch.ops.gemm_unified.finegemm_N``
operators) and exposes ``ops.fine_gemm``. ``_C`` links against ``libmi355_serving.so`` (the HIP kernels behind a C
ABI) which is built next to it by ``build.py`` / ``setup.py``; if either is missing the import fails.
"""
import torch  # noqa: F401  (must be loaded before _C: it provides libtorch and the HIP runtime)
from . import _C, ops  # noqa: F401

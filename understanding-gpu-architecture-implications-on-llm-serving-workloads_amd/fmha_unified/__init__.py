"""fmha_unified for MI355X: same package surface as the reference (kernels/fmha/pkg/fmha_unified/__init__.py:1-2).

Importing the package loads ``_C`` (which defines ``torch.ops.fmha_unified.finefmha_N``) and exposes
``ops.fine_fmha``. ``_C`` links against ``libmi355_serving.so``; if either is missing the import fails.
"""
import torch  # noqa: F401  (must be loaded before _C)
from . import _C, ops  # noqa: F401

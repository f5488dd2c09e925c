"""Python entry point of the GEMM operators; mirrors kernels/gemm/pkg/gemm_unified/ops.py:7-13 of the reference."""
import torch
from torch import Tensor

__all__ = ["fine_gemm", "LAYOUT_OF_INDEX"]

# operand layout each operator index computes (kernels/gemm/test/correct.py:9-15, 30-43)
LAYOUT_OF_INDEX = {i: "NN" for i in range(12)}
LAYOUT_OF_INDEX.update({12: "TN", 16: "TN", 13: "NT", 14: "NT", 15: "NT"})


def fine_gemm(a: Tensor, b: Tensor, kernel_index: int) -> Tensor:
    """fp16 matrix product on the GPU, fp32 accumulation.

    kernel_index 0..11: ``a[M,K] @ b[K,N]``; 12 and 16: ``a[K,M].T @ b[K,N]``; 13..15: ``a[M,K] @ b[N,K].T``
    (the layouts the reference's kernels of those indices read). All indices run the same MI355X kernel family.
    """
    kernel = getattr(torch.ops.gemm_unified, f"finegemm_{int(kernel_index)}")
    return kernel.default(a, b)

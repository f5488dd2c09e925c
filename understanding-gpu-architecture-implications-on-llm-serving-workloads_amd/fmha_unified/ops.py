"""Python entry point of the attention operators; mirrors kernels/fmha/pkg/fmha_unified/ops.py:8-29.

The reference pads q, k and v to a multiple of 64 rows with ``F.pad`` (a full copy of each tensor, ops.py:19-25),
passes the un-padded key count as ``decode_length`` (ops.py:18,27) and slices the output back (ops.py:29). The
MI355X kernel masks ragged tails itself, so nothing is padded, copied or sliced here; the result is the same.
"""
from typing import Tuple

import torch
from torch import Tensor

__all__ = ["fine_fmha", "fine_fmha_with_lse"]


def fine_fmha(q: Tensor, k: Tensor, v: Tensor, causal: bool, is_decode, kernel_index: int) -> Tensor:
    """softmax(q k^T / sqrt(d) + mask) v for q [B,Hq,Sq,128], k, v [B,Hkv,Sk,128] (fp16, GPU).

    ``causal`` masks key j for query i when j > i + (Sk - Sq); ``is_decode`` (requires ``causal=False``) is the
    single-query generation step. GQA: query head h uses kv head h // (Hq // Hkv).

    Difference from the reference for ``Sq != Sk``: its kernels mask key j when j > i (top-left alignment,
    semi/fmha_2_amd.cpp:187-190); here the mask is aligned to the bottom-right corner (the KV-cache convention). The two
    are the same mask when ``Sq == Sk``, the only causal case the reference's tests and drivers use. A query row with no
    visible key (``Sq > Sk`` only) gives zeros. The result is a new contiguous [B, Hq, Sq, 128] tensor.
    """
    kernel = getattr(torch.ops.fmha_unified, f"finefmha_{int(kernel_index)}")
    decode_length = k.size(2)
    return kernel.default(q, k, v, bool(causal), bool(is_decode), decode_length)


def fine_fmha_with_lse(q: Tensor, k: Tensor, v: Tensor, causal: bool, is_decode=False) -> Tuple[Tensor, Tensor]:
    """As :func:`fine_fmha`, also returning the fp32 log-sum-exp [B,Hq,Sq] of the scaled, masked scores."""
    return torch.ops.fmha_unified.finefmha_fwd_lse.default(q, k, v, bool(causal), bool(is_decode), k.size(2))

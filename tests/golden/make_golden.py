"""Writes the small golden fixtures of tests/golden/ with the CPU oracle.

The reference's own tests hold no stored vectors, only seeded generators; the two cases below regenerate exactly
those inputs and record the oracle's fp32 answers:

  gemm_seed0_256.npz   kernels/gemm/test/correct.py:5-15: torch.manual_seed(0), a then b = randn(256, 256, fp16)
                       drawn on the CPU; expected a@b, a.T@b, a@b.T (rows 0..31 and 224..255 only, fp32)
  fmha_seed42_128.npz  kernels/fmha/test/correct.py:26-48: torch.manual_seed(42), q (1,4,128,128), k, v (1,1,128,128)
                       = randn(fp16) * 0.1 drawn on the CPU in that order; expected causal and non-causal O (query rows 0..15 and 112..127, fp32) and LSE

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(HERE)), "oracle"))
import serving_oracle as so  # noqa: E402

ROWS = list(range(32)) + list(range(224, 256))
QROWS = list(range(16)) + list(range(112, 128))


def main():
    torch.manual_seed(0)
    a = torch.randn(256, 256, dtype=torch.half)
    b = torch.randn(256, 256, dtype=torch.half)
    out = {"a": a.numpy(), "b": b.numpy(), "rows": np.array(ROWS)}
    for lay in ("NN", "TN", "NT"):
        out["c_" + lay] = so.gemm_ref(a, b, lay).numpy()[ROWS]
    np.savez(os.path.join(HERE, "gemm_seed0_256.npz"), **out)

    torch.manual_seed(42)
    q = torch.randn(size=(1, 4, 128, 128), dtype=torch.half) * 0.1
    k = torch.randn(size=(1, 1, 128, 128), dtype=torch.half) * 0.1
    v = torch.randn(size=(1, 1, 128, 128), dtype=torch.half) * 0.1
    out = {"q": q.numpy(), "k": k.numpy(), "v": v.numpy(), "qrows": np.array(QROWS)}
    for causal in (False, True):
        o, lse = so.attention_ref(q, k, v, causal=causal)
        tag = "causal" if causal else "full"
        out["o_" + tag] = o.numpy()[:, :, QROWS]
        out["lse_" + tag] = lse.numpy()
    np.savez(os.path.join(HERE, "fmha_seed42_128.npz"), **out)
    print("wrote", os.listdir(HERE))


if __name__ == "__main__":
    main()

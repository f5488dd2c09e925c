"""GEMM sweep in the protocol of the reference's kernels/gemm/test/perf_amd.py.

Same measurement: inputs `torch.randn(fp16)` drawn on the CPU and copied to the GPU (perf_amd.py:8-9), 2 warm-up calls
(:11-15), 50 calls each wrapped in its own torch.profiler session with a record_function range (:17-28), the LAST call's
key_averages, rows sorted by device time, TFLOPS = 2*M*K*N / device_time of the top row (:31-58) -- i.e. the time of the
whole operator range, allocation included. Table of kernel index x size 2^8 .. 2^13, written to finegemm_perf.csv (:62-81).
Kernel -1 is torch's `a @ b`. All indices 0..16 exist in this build (the reference skips 6, 9, 10).

Operands are generated per index in the layout that index reads (a.T for 12/16, b.T for 13..15) so every row computes the
same product; the reference feeds square a, b unchanged, which times the same amount of work.
"""
import argparse
import os
import sys

import pandas as pd
import torch
from tabulate import tabulate
from torch.profiler import ProfilerActivity, profile, record_function

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import gemm_unified  # noqa: E402


def profile_finegemm_kernel(M, K, N, kernel_index, dtype=torch.half, calls=50):
    a = torch.randn(M, K, dtype=dtype).cuda()
    b = torch.randn(K, N, dtype=dtype).cuda()
    layout = gemm_unified.ops.LAYOUT_OF_INDEX.get(kernel_index, "NN")
    if layout == "TN":
        a = a.t().contiguous()
    elif layout == "NT":
        b = b.t().contiguous()

    def call():
        if kernel_index == -1:
            return a @ b
        return gemm_unified.ops.fine_gemm(a, b, kernel_index)

    for _ in range(2):
        call()
    label = "gemm_cublas" if kernel_index == -1 else f"gemm_finegemm_{kernel_index}"
    table_data = []
    for _ in range(calls):
        with profile(activities=[ProfilerActivity.CPU, ProfilerActivity.CUDA]) as prof:
            with record_function(label):
                call()
        table_data = [[item.key, item.device_time] for item in prof.key_averages()]
    table = pd.DataFrame(table_data, columns=["Key", "CUDA Time"]).groupby("Key").mean().reset_index()
    table["Key"] = table["Key"].str[:20]
    table["TFLOPS"] = (2 * M * K * N / (table["CUDA Time"] * 1e-6)) * 1e-12
    table = table.sort_values(by="CUDA Time", ascending=False)
    print(tabulate(table[:5], headers=["Key", "CUDA Time", "TFLOPS"], tablefmt="pretty"))
    return table.iloc[0]["TFLOPS"]


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--indices", type=int, nargs="*", default=list(range(-1, 17)))
    ap.add_argument("--min-exp", type=int, default=8)
    ap.add_argument("--max-exp", type=int, default=13)
    ap.add_argument("--calls", type=int, default=50)
    ap.add_argument("--out", default="finegemm_perf.csv")
    args = ap.parse_args()
    exps = range(args.min_exp, args.max_exp + 1)
    df = pd.DataFrame(columns=[f"2^{i}" for i in exps], index=[f"Kernel {i}" for i in args.indices])
    for i in args.indices:
        for j in exps:
            df.loc[f"Kernel {i}", f"2^{j}"] = profile_finegemm_kernel(2 ** j, 2 ** j, 2 ** j, i, calls=args.calls)
    print(df)
    df.to_csv(args.out)
    print("DONE")

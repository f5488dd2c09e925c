"""Attention sweep in the protocol of the reference's kernels/fmha/test/perf_amd.py.

Same measurement: b=1, 32 q heads, GQA 32/8, d=128, causal, fp16, s = 2^8 .. 2^14 (perf_amd.py:100-112); q, k, v
`torch.randn` on the CPU then `.cuda()` (:45-47); 20 profiled calls, no warm-up (:49-66); last call's key_averages sorted by
device time; TFLOPS = 4*s^2*d*h / device_time of the top row, WITHOUT a causal discount (:89). Baselines: -1 = torch SDPA
after repeat_kv (:10-24), -2 = flash_attn_func (:26-32) -- optional here: flash_attn is imported only if it is installed.
Results go to finefmha_perf.csv.
"""
import argparse
import os
import sys

import pandas as pd
import torch
from tabulate import tabulate
from torch.nn import functional as F
from torch.profiler import ProfilerActivity, profile, record_function

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import fmha_unified  # noqa: E402

try:
    from flash_attn import flash_attn_func
except ImportError:  # not part of this image
    flash_attn_func = None


def torch_attn(q, k, v, is_causal):
    def repeat_kv(hidden_states, n_rep):
        batch, num_key_value_heads, slen, head_dim = hidden_states.shape
        if n_rep == 1:
            return hidden_states
        hidden_states = hidden_states[:, :, None, :, :].expand(batch, num_key_value_heads, n_rep, slen, head_dim)
        return hidden_states.reshape(batch, num_key_value_heads * n_rep, slen, head_dim)
    if q.size(1) != k.size(1):
        k = repeat_kv(k, q.size(1) // k.size(1))
        v = repeat_kv(v, q.size(1) // v.size(1))
    return F.scaled_dot_product_attention(q, k, v, is_causal=is_causal)


def call_flash_attn(q, k, v, is_causal):
    return flash_attn_func(q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3), v.permute(0, 2, 1, 3), causal=is_causal)


def profile_finefmha_kernel(B, H, N, d, GQA, is_causal, is_decode, kernel_index, dtype=torch.half, calls=20):
    kv_head = H // 4 if GQA else H
    q = torch.randn(size=(B, H, N, d), dtype=dtype).cuda()
    k = torch.randn(size=(B, kv_head, N, d), dtype=dtype).cuda()
    v = torch.randn(size=(B, kv_head, N, d), dtype=dtype).cuda()
    table_data = []
    for _ in range(calls):
        with profile(activities=[ProfilerActivity.CPU, ProfilerActivity.CUDA]) as prof:
            if kernel_index == -1:
                with record_function("fmha_torch"):
                    torch_attn(q, k, v, is_causal)
            elif kernel_index == -2:
                with record_function("fmha_flash"):
                    call_flash_attn(q, k, v, is_causal)
            else:
                with record_function(f"fmha_finefmha_{kernel_index}"):
                    fmha_unified.ops.fine_fmha(q, k, v, is_causal, is_decode, kernel_index)
        table_data = [[item.key, item.device_time] for item in prof.key_averages()]
    table = pd.DataFrame(table_data, columns=["Key", "CUDA Time"]).groupby("Key").mean().reset_index()
    table = table.sort_values(by="CUDA Time", ascending=False)
    table["Key"] = table["Key"].str[:25]
    table["TFLOPS"] = (4 * N * N * d * H / (table["CUDA Time"] * 1e-6)) * 1e-12
    print(tabulate(table[:3], headers=["Key", "CUDA Time", "TFLOPS"], tablefmt="pretty"))
    return table.iloc[0]["TFLOPS"]


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--indices", type=int, nargs="*", default=[0, 2, -2, -1])
    ap.add_argument("--min-exp", type=int, default=8)
    ap.add_argument("--max-exp", type=int, default=14)
    ap.add_argument("--out", default="finefmha_perf.csv")
    args = ap.parse_args()
    indices = [i for i in args.indices if not (i == -2 and flash_attn_func is None)]
    exps = range(args.min_exp, args.max_exp + 1)
    df = pd.DataFrame(columns=[f"2^{j}" for j in exps], index=[f"Kernel {i}" for i in indices])
    for i in indices:
        for j in exps:
            df.at[f"Kernel {i}", f"2^{j}"] = profile_finefmha_kernel(1, 32, 2 ** j, 128, True, True, False, i, dtype=torch.half)
    print(df)
    df.to_csv(args.out)
    print("Done")

#!/usr/bin/env python3
"""Benchmark of the MI355X serving kernels on the benchmark's headline configurations.

One "step" = one pass of the hot path over one batch of synthetic input, resident in HBM before timing starts:
    1. fp16 GEMM  C = A B, M = N = K = 8192, A ~ N(0,1), B ~ N(0, 0.02^2), fp32 accumulate        (configuration G2b)
    2. attention forward, causal GQA, b = 1, 32 q / 8 kv heads, s = 4096, d = 128, fp16, + LSE   (configuration F4)
both called through the C ABI of libmi355_serving.so on torch's current stream.

`value` is the whole-step throughput: (GEMM flops 2MNK + attention flops 4*B*Hq*d*#unmasked(q,k) pairs) / time,
in TFLOP/s. Per-kernel figures (TFLOP/s, % of the 2.5 PFLOP/s dense fp16 MFMA peak, average launch duration
measured with HIP events on the launch stream) are in `kernels`; `roofline` describes the dominant kernel (the
GEMM); `cpu_baseline` is the same step on the host cores with torch fp32 (reported, not a target);
`other_configs` lists the remaining benchmark configurations (parity cases, quick timings).

Output: ONE JSON line on stdout.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, "understanding-gpu-architecture-implications-on-llm-serving-workloads_amd")
sys.path.insert(0, PKG)
sys.path.insert(0, os.path.join(ROOT, "oracle"))

PEAK_FP16_TFLOPS = 2500.0   # MI355X dense fp16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch), each scaled by what the same
# counter reads for a 1 GiB device-to-device copy (FETCH_SIZE x2.0, WRITE_SIZE x1.0); see profiles/.
MEASURED_TRAFFIC_BYTES = (795037 * 2.0 + 131072 * 1.0) * 1024        # hgemm_main_kernel, 8192^3 NN
MEASURED_TRAFFIC_BYTES_G2C = (57882 * 2.0 + 448 * 1.0) * 1024          # hgemm_smallm_nn_kernel, 16 x 14336 x 4096
MEASURED_TRAFFIC_BYTES_FMHA = (26670 * 2.0 + 33280 * 1.0) * 1024     # fmha_fwd_pingpong_kernel, F4
# the figures above are constants copied from these counter summaries (they are not read at run time)
TRAFFIC_SOURCE = {"gemm": "constant from profiles/hgemm_main_kernel_256x256_8192_nn.md (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE)",
                  "g2c": "constant from profiles/hgemm_smallm_nn_kernel_g2c_16x14336x4096_nn.md",
                  "fmha": "constant from profiles/fmha_fwd_pingpong_kernel_f4_causal_gqa.md"}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def time_graph(fn, iters, warmup):
    """Mean duration (ms) of `iters` launches replayed from ONE HIP graph (captured after `warmup` eager launches on the
    capture stream): the kernels run back to back without the ~3 us the runtime takes between two dependent eager launches,
    which is a sizeable part of a 20 us kernel. HIP events around the replay, on the stream it runs on."""
    import torch
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(warmup):
            fn()
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for _ in range(iters):
            fn()
    graph.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    graph.replay()
    e1.record()
    e1.synchronize()
    ms = e0.elapsed_time(e1) / iters
    del graph
    return ms


def time_launches(fn, iters, warmup, stats=False):
    """Mean duration (ms) of `iters` back-to-back launches after `warmup` untimed ones: two HIP events on the current
    stream around the whole batch. With stats=True a second batch is timed with an event after every launch, for the
    median and minimum of the per-launch intervals; an event between two kernels keeps the second from starting under the
    tail of the first and adds several microseconds per launch, so those figures are upper bounds of a single launch and
    the mean of the first batch is the throughput figure."""
    import torch
    for _ in range(warmup):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    # After an idle period (a host-side check, a synchronize) the chip needs ~20 ms of work to reach the clocks it then
    # holds: 20 launches of a 1 ms kernel after 5 warm-ups measured 8 % slower than 200 after 20. Keep launching until
    # about 25 ms of this work have run, then time.
    e0.record()
    fn()
    e1.record()
    e1.synchronize()
    for _ in range(min(2000, int(25.0 / max(e0.elapsed_time(e1), 1e-3)))):
        fn()
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    e1.synchronize()
    mean = e0.elapsed_time(e1) / iters
    if not stats:
        return mean
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(iters + 1)]
    ev[0].record()
    for i in range(iters):
        fn()
        ev[i + 1].record()
    ev[-1].synchronize()
    per = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(iters))
    return {"ms": mean, "ms_median_event_per_launch": per[len(per) // 2], "ms_min_event_per_launch": per[0], "launches": iters,
            "warmup": warmup}


LAST_LEVEL_CACHE_BYTES = 256 << 20   # MI355X: 256 MB of memory-side cache in front of the HBM stacks


def rotating(call, n_sets):
    """fn() that calls `call(j)` with j = 0, 1, .., n_sets-1, 0, .. : a launch sequence over n_sets copies of the big
    operand, so that no launch finds its operand in a cache. Back-to-back launches on ONE copy of an operand smaller than
    the memory-side cache (or not much larger) are partly served from it and read faster than HBM delivers."""
    state = [0]

    def fn():
        call(state[0] % n_sets)
        state[0] += 1
    return fn


def copies_to_defeat_cache(operand_bytes):
    return int(max(2, min(24, 3 * LAST_LEVEL_CACHE_BYTES // max(1, int(operand_bytes)) + 1)))


def causal_pairs(Sq, Sk):
    shift = Sk - Sq
    return sum(max(0, min(Sk, i + shift + 1)) for i in range(Sq))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # 200 steps of ~0.93 ms after 20 warm-ups: the first ~20 ms after an idle period run at the clocks and with the caches
    # of an idle chip (20 steps after 5 warm-ups measured 8 % more per step than the steady state)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true")
    ap.add_argument("--no-check", action="store_true")
    ap.add_argument("--layer-only", choices=["prefill", "step"], default=None,
                    help="run only the Llama-3-8B-shaped decoder layer (prefill at s=8192, or a generation step at batch 8 over "
                         "8192 cached tokens) for --steps iterations and print its timing; for per-kernel profiles")
    ap.add_argument("--kernel-config", default=None, choices=sorted(KERNEL_CONFIGS),
                    help="launch one named kernel configuration --steps times (after --warmup) and print its timing; the "
                         "workload of the per-kernel rocprofv3 summaries in profiles/")
    ap.add_argument("--timeline", action="store_true",
                    help="with --kernel-config: load the profiling twin of the library (libmi355_serving_timeline.so), whose "
                         "tiled GEMM and attention kernels record wall-clock and cycle stamps per workgroup, and print a "
                         "summary of the last launch (configurations on the small-M GEMM kernels leave no records)")
    ap.add_argument("--zero-inputs", action="store_true",
                    help="with --kernel-config: all-zero operands instead of the seeded random ones (the arithmetic and its "
                         "cycle count stay the same, the switching power does not: shows what the board's power limit costs)")
    ap.add_argument("--rotate-operands", action="store_true",
                    help="with --kernel-config: every launch reads a different copy of the big operand (the weight matrix of a "
                         "GEMM, K and V of attention), enough copies to exceed the 256 MB memory-side cache three times: the "
                         "rate with operands that come from HBM, as in a decoder stack, not from a cache warmed by the launch before")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one 1 GiB device-to-device copy, so FETCH_SIZE / WRITE_SIZE read under rocprofv3 "
                         "--pmc can be scaled by what the same counter reports for a transfer of known size")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (--gpus 1); multi-GPU sharding is described in "
                 "the design notes and not implemented")

    import torch
    import mi355_serving as lib
    import serving_oracle as so

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the kernels have no CPU fallback")
    if args.timeline:
        if not args.kernel_config:
            sys.exit("bench.py: --timeline needs --kernel-config")
        lib.LIB_PATH = os.path.join(os.path.dirname(lib.LIB_PATH), "libmi355_serving_timeline.so")
    lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.kernel_config:
        run_kernel_config(args, torch, lib, so, dev)
        return

    if args.layer_only:
        layer, S5 = llama3_8b_layer(torch, so, dev)
        from llama_layer import FineKVCache
        if args.layer_only == "prefill":
            x = so.randn_fp16((1, S5, 4096), 18).to(dev)
            fn = lambda: layer(x)
        else:
            cache = FineKVCache(8, S5 + 64, 8, device=dev)
            cache.k.normal_(0, 1)
            cache.v.normal_(0, 1)
            x = so.randn_fp16((8, 1, 4096), 19).to(dev)
            def fn():
                cache.length = S5
                layer(x, kv_cache=cache)
        ms = time_launches(fn, args.steps, args.warmup)
        print(json.dumps({"layer_only": args.layer_only, "ms": ms, "steps": args.steps, "warmup": args.warmup}))
        return

    # ---- synthetic inputs, resident in HBM -------------------------------------------------------------------
    M = N = K = 8192
    a_h, b_h = so.gemm_inputs(M, N, K, seed=0, a_std=1.0, b_std=0.02)
    a, b = a_h.to(dev), b_h.to(dev)
    c = torch.empty((M, N), dtype=torch.float16, device=dev)
    B_, Hq, Hkv, S, D = 1, 32, 8, 4096, 128
    q_h, k_h, v_h = so.fmha_inputs(B_, Hq, Hkv, S, S, seed=42)
    q, k, v = q_h.to(dev), k_h.to(dev), v_h.to(dev)
    o = torch.empty_like(q)
    lse = torch.empty((B_, Hq, S), dtype=torch.float32, device=dev)
    scale = 1.0 / math.sqrt(D)
    stream = torch.cuda.current_stream().cuda_stream

    def gemm():
        lib.hgemm_raw(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, K, N, N, lib.GEMM_NN, stream)

    def fmha():
        lib.fmha_fwd_raw(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(), B_, Hq, Hkv, S, S, D,
                         scale, 1, S, stream)

    gemm_flops = 2.0 * M * N * K
    fmha_flops = 4.0 * B_ * Hq * D * causal_pairs(S, S)       # causal-discounted (algorithmic)
    fmha_flops_ref_convention = 4.0 * S * S * D * Hq          # kernels/fmha/test/perf.py:89 (no causal discount)

    # ---- correctness of what is being timed (sampled rows against the oracle) ----------------------------------
    checks = {}
    if not args.no_check:
        gemm(); fmha(); torch.cuda.synchronize()
        rows = torch.arange(0, M, 127)
        ok_g, st_g = so.gemm_tolerance_ok(c[rows.to(dev)], so.gemm_ref(a_h[rows], b_h), K)
        heads = [0, 13, 31]
        oks, stf = True, {}
        for h in heads:
            orf, lrf = so.attention_ref(q_h[:, h:h + 1], k_h[:, h // 4:h // 4 + 1], v_h[:, h // 4:h // 4 + 1], causal=True)
            okh, sth = so.fmha_tolerance_ok(o[:, h:h + 1], lse[:, h:h + 1], orf, lrf)
            oks = oks and okh
            stf = {kk: max(stf.get(kk, 0.0), vv) for kk, vv in sth.items()}
        checks = {"gemm_within_tolerance": bool(ok_g), "gemm": st_g, "fmha_within_tolerance": bool(oks), "fmha": stf}
        log("[bench] parity of the timed configuration:", checks)
        if not (ok_g and oks):
            sys.exit("bench.py: timed configuration is outside tolerance: %s" % checks)

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- timed region: exactly K steps between device synchronisations -------------------------------------------
    for _ in range(args.warmup):
        gemm(); fmha()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        gemm(); fmha()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    value = (gemm_flops + fmha_flops) / (ms_per_step * 1e-3) / 1e12

    # ---- per-kernel launch durations (HIP events on the launch stream) --------------------------------------------
    n_timed, n_warm = max(args.steps, 50), max(args.warmup, 10)
    gemm_t = time_launches(gemm, n_timed, n_warm, stats=True)
    fmha_t = time_launches(fmha, n_timed, n_warm, stats=True)
    gemm_ms, fmha_ms = gemm_t["ms"], fmha_t["ms"]
    gemm_tf = gemm_flops / (gemm_ms * 1e-3) / 1e12
    fmha_tf = fmha_flops / (fmha_ms * 1e-3) / 1e12
    kernels = {
        "hgemm_8192x8192x8192_nn": dict(gemm_t, tflops=gemm_tf, pct_of_fp16_mfma_peak=100 * gemm_tf / PEAK_FP16_TFLOPS,
                                        tflops_at_min=gemm_flops / gemm_t["ms_min_event_per_launch"] / 1e9),
        "fmha_fwd_causal_gqa_b1_h32_8_s4096_d128": dict(
            fmha_t, tflops=fmha_tf, pct_of_fp16_mfma_peak=100 * fmha_tf / PEAK_FP16_TFLOPS,
            tflops_at_min=fmha_flops / fmha_t["ms_min_event_per_launch"] / 1e9,
            tflops_reference_convention_4s2dh=fmha_flops_ref_convention / (fmha_ms * 1e-3) / 1e12),
    }
    roofline = {"kernel": "hgemm_main_kernel (8192^3, NN)", "bound": "mfma", "achieved": gemm_tf, "peak": PEAK_FP16_TFLOPS,
                "unit": "TFLOP/s", "frac": gemm_tf / PEAK_FP16_TFLOPS, "traffic": MEASURED_TRAFFIC_BYTES,
                "traffic_source": TRAFFIC_SOURCE["gemm"]}
    roofline_fmha = {"kernel": "fmha_fwd_pingpong_kernel (F4)", "bound": "mfma", "achieved": fmha_tf, "peak": PEAK_FP16_TFLOPS,
                     "unit": "TFLOP/s", "frac": fmha_tf / PEAK_FP16_TFLOPS, "traffic": MEASURED_TRAFFIC_BYTES_FMHA,
                     "traffic_source": TRAFFIC_SOURCE["fmha"]}

    # ---- the other benchmark configurations (quick timings) ----------------------------------------------------------
    other = {}
    roofline_g2c = None
    if not args.no_other_configs:
        def t_gemm(m, n, kk, iters=50, rotate_weights=False):
            x_h, w_h = so.randn_fp16((m, kk), 1), so.randn_fp16((kk, n), 2, 0.02)
            x, w = x_h.to(dev), w_h.to(dev)
            out = torch.empty((m, n), dtype=torch.float16, device=dev)
            fn_ = lambda: lib.hgemm_raw(x.data_ptr(), w.data_ptr(), out.data_ptr(), m, n, kk, kk, n, n, lib.GEMM_NN,
                                        torch.cuda.current_stream().cuda_stream)
            t = time_launches(fn_, iters, 10, stats=True)
            t["ms_eager"] = t["ms"]
            t["ms"] = time_graph(fn_, iters, 10)   # replayed from one HIP graph: without the runtime's gap between eager launches
            ms = t["ms"]
            fl, by = 2.0 * m * n * kk, 2.0 * (m * kk + kk * n + m * n)
            if rotate_weights:   # bandwidth-bound shape: also with a different copy of the weight on every launch
                ws_ = [w] + [w.clone() for _ in range(copies_to_defeat_cache(2.0 * kk * n) - 1)]
                rot_ = rotating(lambda j: lib.hgemm_raw(x.data_ptr(), ws_[j].data_ptr(), out.data_ptr(), m, n, kk, kk, n, n, lib.GEMM_NN,
                                                        torch.cuda.current_stream().cuda_stream), len(ws_))
                t["ms_weights_not_cached"] = time_graph(rot_, iters, 10)
                t["gbs_weights_not_cached"] = by / t["ms_weights_not_cached"] / 1e6
                t["weight_copies"] = len(ws_)
                del ws_
            rows_ = torch.arange(0, m, max(1, m // 64))
            ok_, _ = so.gemm_tolerance_ok(out[rows_.to(dev)], so.gemm_ref(x_h[rows_], w_h), kk)
            return dict(t, tflops=fl / ms / 1e9, pct_of_fp16_mfma_peak=100 * fl / ms / 1e9 / PEAK_FP16_TFLOPS,
                        gbs=by / ms / 1e6, pct_of_hbm_peak=100 * by / ms / 1e6 / PEAK_HBM_GBS, within_tolerance=bool(ok_))
        other["G1_gemm_1024"] = t_gemm(1024, 1024, 1024)
        other["G2a_gemm_4096"] = t_gemm(4096, 4096, 4096)
        other["G2c_gemm_decode_16x14336x4096"] = t_gemm(16, 14336, 4096, rotate_weights=True)
        g2c = other["G2c_gemm_decode_16x14336x4096"]
        # achieved = the rate with a weight that is in no cache (a different copy per launch); launches that reuse one
        # 117 MB weight find part of it in the 256 MB memory-side cache and read faster than the HBM figure they are held against
        roofline_g2c = {"kernel": "hgemm_smallm_nn_kernel (G2c: 16 x 14336 x 4096, NN)", "bound": "hbm",
                        "achieved": g2c["gbs_weights_not_cached"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                        "frac": g2c["gbs_weights_not_cached"] / PEAK_HBM_GBS, "achieved_same_weight_every_launch": g2c["gbs"],
                        "traffic": MEASURED_TRAFFIC_BYTES_G2C, "traffic_source": TRAFFIC_SOURCE["g2c"]}
        q3h, k3h, v3h = so.fmha_inputs(4, 32, 32, 1024, 1024, seed=42)
        q3, k3, v3 = q3h.to(dev), k3h.to(dev), v3h.to(dev)
        o3 = torch.empty_like(q3)
        l3 = torch.empty((4, 32, 1024), dtype=torch.float32, device=dev)
        t3 = time_launches(lambda: lib.fmha_fwd_raw(q3.data_ptr(), k3.data_ptr(), v3.data_ptr(), o3.data_ptr(), l3.data_ptr(), 4, 32,
                                                    32, 1024, 1024, 128, scale, 0, 1024, stream), 50, 10, stats=True)
        ms3 = t3["ms"]
        fl3 = 4.0 * 4 * 32 * 128 * 1024 * 1024
        ok3 = True
        for (bb, hh) in ((0, 0), (1, 17), (3, 31)):
            orf, lrf = so.attention_ref(q3h[bb:bb + 1, hh:hh + 1], k3h[bb:bb + 1, hh:hh + 1], v3h[bb:bb + 1, hh:hh + 1])
            ok3 = ok3 and so.fmha_tolerance_ok(o3[bb:bb + 1, hh:hh + 1], l3[bb:bb + 1, hh:hh + 1], orf, lrf)[0]
        other["F3_fmha_noncausal_b4_h32_s1024"] = dict(t3, tflops=fl3 / ms3 / 1e9, within_tolerance=bool(ok3),
                                                       pct_of_fp16_mfma_peak=100 * fl3 / ms3 / 1e9 / PEAK_FP16_TFLOPS)
        del q3, k3, v3, o3, l3
        # the vendor libraries on the same box, same operands, same timing loop (context for the figures above; not this code)
        cv = torch.empty_like(c)
        ms_v = time_launches(lambda: torch.matmul(a, b, out=cv), 20, 3)
        bt = b.t().contiguous()
        ms_vt = time_launches(lambda: torch.matmul(a, bt.t(), out=cv), 20, 3)
        ms_sd = time_launches(lambda: torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True), 20, 3)
        # this library on the same NT operands (B stored [N, K]), same timing loop: the like-for-like figure next to the vendor's
        cnt = torch.empty_like(c)
        ms_nt = time_launches(lambda: lib.hgemm_raw(a.data_ptr(), bt.data_ptr(), cnt.data_ptr(), M, N, K, K, K, N, lib.GEMM_NT, stream), 20, 3)
        ms_nn = time_launches(gemm, 20, 3)
        other["hgemm_8192_same_loop_as_vendor"] = {"nn": {"ms": ms_nn, "tflops": gemm_flops / ms_nn / 1e9},
                                                   "nt": {"ms": ms_nt, "tflops": gemm_flops / ms_nt / 1e9}}
        del cnt
        other["vendor_libraries_same_box"] = {
            "torch_matmul_hipblaslt_8192_nn": {"ms": ms_v, "tflops": gemm_flops / ms_v / 1e9},
            "torch_matmul_hipblaslt_8192_nt": {"ms": ms_vt, "tflops": gemm_flops / ms_vt / 1e9},
            "torch_sdpa_f4_causal_gqa": {"ms": ms_sd, "tflops": fmha_flops / ms_sd / 1e9}}
        for tag, (mv, nv, kv) in (("g1_1024", (1024, 1024, 1024)), ("g2a_4096", (4096, 4096, 4096)), ("g2c_16x14336x4096", (16, 14336, 4096))):
            xv = so.randn_fp16((mv, kv), 1).to(dev)
            wv = so.randn_fp16((kv, nv), 2, 0.02).to(dev)
            ov = torch.empty((mv, nv), dtype=torch.float16, device=dev)
            msv = time_launches(lambda: torch.matmul(xv, wv, out=ov), 20, 3)
            other["vendor_libraries_same_box"]["torch_matmul_hipblaslt_" + tag] = {"ms": msv, "tflops": 2.0 * mv * nv * kv / msv / 1e9}
        del cv, bt, xv, wv, ov
        # generation-step shapes (HBM bound): nn.Linear-layout weight GEMM and attention over a long KV cache
        xd = so.randn_fp16((16, 4096), 1).to(dev)
        wd_nt = so.randn_fp16((14336, 4096), 2, 0.02).to(dev)
        od = torch.empty((16, 14336), dtype=torch.float16, device=dev)
        msd = time_launches(lambda: lib.hgemm_raw(xd.data_ptr(), wd_nt.data_ptr(), od.data_ptr(), 16, 14336, 4096, 4096, 4096,
                                                  14336, lib.GEMM_NT, stream), 20, 3)
        byd = 2.0 * (16 * 4096 + 4096 * 14336 + 16 * 14336)
        wd_sets = [wd_nt] + [wd_nt.clone() for _ in range(copies_to_defeat_cache(wd_nt.numel() * 2) - 1)]
        msd_cold = time_launches(rotating(lambda j: lib.hgemm_raw(xd.data_ptr(), wd_sets[j].data_ptr(), od.data_ptr(), 16, 14336, 4096,
                                                                  4096, 4096, 14336, lib.GEMM_NT, stream), len(wd_sets)), 40, 3)
        other["gemm_decode_nt_16x14336x4096"] = {"ms": msd, "gbs": byd / msd / 1e6, "pct_of_hbm_peak": 100 * byd / msd / 1e6 / PEAK_HBM_GBS,
                                                 "ms_weights_not_cached": msd_cold, "gbs_weights_not_cached": byd / msd_cold / 1e6,
                                                 "pct_of_hbm_peak_weights_not_cached": 100 * byd / msd_cold / 1e6 / PEAK_HBM_GBS}
        # the same projection at batch 64 (128x64 tiles instead of the small-M kernel), and bf16 twins of the two headline kernels
        x64 = so.randn_fp16((64, 4096), 3).to(dev)
        o64 = torch.empty((64, 14336), dtype=torch.float16, device=dev)
        ms64 = time_launches(lambda: lib.hgemm_raw(x64.data_ptr(), wd_nt.data_ptr(), o64.data_ptr(), 64, 14336, 4096, 4096, 4096,
                                                   14336, lib.GEMM_NT, stream), 20, 3)
        by64 = 2.0 * (64 * 4096 + 4096 * 14336 + 64 * 14336)
        ms64_cold = time_launches(rotating(lambda j: lib.hgemm_raw(x64.data_ptr(), wd_sets[j].data_ptr(), o64.data_ptr(), 64, 14336, 4096,
                                                                   4096, 4096, 14336, lib.GEMM_NT, stream), len(wd_sets)), 40, 3)
        other["gemm_decode_nt_64x14336x4096"] = {"ms": ms64, "gbs": by64 / ms64 / 1e6, "pct_of_hbm_peak": 100 * by64 / ms64 / 1e6 / PEAK_HBM_GBS,
                                                 "ms_weights_not_cached": ms64_cold, "gbs_weights_not_cached": by64 / ms64_cold / 1e6,
                                                 "pct_of_hbm_peak_weights_not_cached": 100 * by64 / ms64_cold / 1e6 / PEAK_HBM_GBS}
        del x64, o64, wd_sets
        # a down projection at batch 64 (4096 rows of a [N, K] weight with K = 14336): 64 tiles of 64x64, split-K over 8 ranges
        xk = so.randn_fp16((64, 14336), 4).to(dev)
        wk = so.randn_fp16((4096, 14336), 5, 0.02).to(dev)
        ok_ = torch.empty((64, 4096), dtype=torch.float16, device=dev)
        wk_sets = [wk] + [wk.clone() for _ in range(copies_to_defeat_cache(wk.numel() * 2) - 1)]
        msk = time_launches(lambda: lib.hgemm_raw(xk.data_ptr(), wk.data_ptr(), ok_.data_ptr(), 64, 4096, 14336, 14336, 14336,
                                                  4096, lib.GEMM_NT, stream), 20, 3)
        msk_cold = time_launches(rotating(lambda j: lib.hgemm_raw(xk.data_ptr(), wk_sets[j].data_ptr(), ok_.data_ptr(), 64, 4096, 14336,
                                                                  14336, 14336, 4096, lib.GEMM_NT, stream), len(wk_sets)), 40, 3)
        byk = 2.0 * (64 * 14336 + 4096 * 14336 + 64 * 4096)
        other["gemm_decode_nt_64x4096x14336_split_k"] = {"ms": msk, "gbs": byk / msk / 1e6, "pct_of_hbm_peak": 100 * byk / msk / 1e6 / PEAK_HBM_GBS,
                                                        "ms_weights_not_cached": msk_cold, "gbs_weights_not_cached": byk / msk_cold / 1e6,
                                                        "pct_of_hbm_peak_weights_not_cached": 100 * byk / msk_cold / 1e6 / PEAK_HBM_GBS}
        # the same weight against a chunk of 512 tokens: 128 tiles of 128x128, split-K over 2 ranges
        xc = so.randn_fp16((512, 14336), 6).to(dev)
        oc_ = torch.empty((512, 4096), dtype=torch.float16, device=dev)
        msc_cold = time_launches(rotating(lambda j: lib.hgemm_raw(xc.data_ptr(), wk_sets[j].data_ptr(), oc_.data_ptr(), 512, 4096, 14336,
                                                                  14336, 14336, 4096, lib.GEMM_NT, stream), len(wk_sets)), 40, 3)
        msc_v = time_launches(rotating(lambda j: torch.matmul(xc, wk_sets[j].t(), out=oc_), len(wk_sets)), 40, 3)
        other["gemm_chunk_nt_512x4096x14336_split_k"] = {"ms_weights_not_cached": msc_cold,
                                                        "tflops_weights_not_cached": 2.0 * 512 * 4096 * 14336 / msc_cold / 1e9,
                                                        "ms_vendor_weights_not_cached": msc_v}
        del xk, wk, ok_, wk_sets, xc, oc_
        ab, bb = a.to(torch.bfloat16), b.to(torch.bfloat16)
        cb = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
        msb = time_launches(lambda: lib.hgemm(ab, bb, "NN", out=cb), 10, 2)
        qb_, kb_, vb_ = q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16)
        ob_ = torch.empty_like(qb_)
        msfb = time_launches(lambda: lib.fmha_fwd(qb_, kb_, vb_, causal=True, return_lse=False, out=ob_), 10, 2)
        other["bf16"] = {"gemm_8192_nn": {"ms": msb, "tflops": gemm_flops / msb / 1e9},
                         "fmha_f4_causal_gqa": {"ms": msfb, "tflops": fmha_flops / msfb / 1e9}}
        del ab, bb, cb, qb_, kb_, vb_, ob_
        for bd, skd in ((1, 8192), (8, 8192), (1, 32768)):
            qd, kd, vd = (t.to(dev) for t in so.fmha_inputs(bd, 32, 8, 1, skd, seed=7))
            o_d = torch.empty_like(qd)
            ms_d = time_launches(lambda: lib.fmha_fwd_raw(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o_d.data_ptr(), None, bd,
                                                          32, 8, 1, skd, 128, scale, 0, skd, stream), 20, 3)
            by_d = 2.0 * (2 * bd * 8 * skd * 128 + 2 * bd * 32 * 128)
            kv_sets = [(kd, vd)] + [(kd.clone(), vd.clone()) for _ in range(copies_to_defeat_cache(by_d) - 1)]
            ms_dc = time_launches(rotating(lambda j: lib.fmha_fwd_raw(qd.data_ptr(), kv_sets[j][0].data_ptr(), kv_sets[j][1].data_ptr(),
                                                                      o_d.data_ptr(), None, bd, 32, 8, 1, skd, 128, scale, 0, skd, stream),
                                           len(kv_sets)), 40, 3)
            other["fmha_decode_b%d_h32_8_sk%d" % (bd, skd)] = {"ms": ms_d, "gbs": by_d / ms_d / 1e6,
                                                               "pct_of_hbm_peak": 100 * by_d / ms_d / 1e6 / PEAK_HBM_GBS,
                                                               "ms_kv_not_cached": ms_dc, "gbs_kv_not_cached": by_d / ms_dc / 1e6,
                                                               "pct_of_hbm_peak_kv_not_cached": 100 * by_d / ms_dc / 1e6 / PEAK_HBM_GBS,
                                                               "kv_copies": len(kv_sets)}
            del kv_sets
        del xd, wd_nt, od, qd, kd, vd, o_d
        # a chunk of new tokens against a cache (causal, 32/8 heads): keys cut into ranges and merged, beside the same kernel
        # walking all keys at once (the library's variant hook)
        for sqc, skc in ((128, 8192), (512, 8192), (128, 32768)):
            qc, kc, vc = (t.to(dev) for t in so.fmha_inputs(1, 32, 8, sqc, skc, seed=9))
            o_c = torch.empty_like(qc)
            ms_r = time_launches(lambda: lib.fmha_fwd(qc, kc, vc, causal=True, return_lse=False, out=o_c), 20, 3)
            ms_w = time_launches(lambda: lib.fmha_fwd(qc, kc, vc, causal=True, return_lse=False, out=o_c, variant=1), 20, 3)
            fl_c = 4.0 * 32 * 128 * causal_pairs(sqc, skc)
            other["fmha_chunk_q%d_over_%d_causal_gqa" % (sqc, skc)] = {"ms": ms_r, "tflops": fl_c / ms_r / 1e9,
                                                                       "ms_one_walk_over_all_keys": ms_w}
        del qc, kc, vc, o_c
        # L5: Llama-3-8B-shaped prefill layer at s = 8192, per stage; every stage is checked on sampled token rows against
        # the oracle fed the GPU's own previous-stage output, and the chain's end against the pure fp32 chain
        S5, H5, F5 = 8192, 4096, 14336
        x5h = so.randn_fp16((S5, H5), 0)
        wqkv_h, wo_h = so.randn_fp16((H5, 6144), 1, 0.02), so.randn_fp16((H5, H5), 2, 0.02)
        wgu_h, wd_h = so.randn_fp16((H5, 2 * F5), 3, 0.02), so.randn_fp16((F5, H5), 4, 0.02)
        x5, wqkv, wo, wgu, wd = (t.to(dev) for t in (x5h, wqkv_h, wo_h, wgu_h, wd_h))
        st = {}
        def stage(name, fn, flops, iters=10):
            ms = time_launches(fn, iters, 3)
            st[name] = {"ms": ms, "tflops": flops / ms / 1e9}
        qkv5 = torch.empty((S5, 6144), dtype=torch.float16, device=dev)
        stage("qkv_gemm", lambda: lib.hgemm(x5, wqkv, out=qkv5), 2.0 * S5 * H5 * 6144)
        q5 = qkv5[:, :4096].reshape(S5, 32, 128).permute(1, 0, 2)[None].contiguous()
        k5 = qkv5[:, 4096:5120].reshape(S5, 8, 128).permute(1, 0, 2)[None].contiguous()
        v5 = qkv5[:, 5120:].reshape(S5, 8, 128).permute(1, 0, 2)[None].contiguous()
        o5 = torch.empty_like(q5)
        lse5 = torch.empty((1, 32, S5), dtype=torch.float32, device=dev)
        stage("fmha_causal_gqa_s8192", lambda: lib.fmha_fwd_raw(q5.data_ptr(), k5.data_ptr(), v5.data_ptr(), o5.data_ptr(),
                                                                 lse5.data_ptr(), 1, 32, 8, S5, S5, 128, scale, 1, S5, stream),
              4.0 * 32 * 128 * causal_pairs(S5, S5))
        a5 = o5[0].permute(1, 0, 2).reshape(S5, H5).contiguous()
        op5 = torch.empty((S5, H5), dtype=torch.float16, device=dev)
        stage("oproj_gemm", lambda: lib.hgemm(a5, wo, out=op5), 2.0 * S5 * H5 * H5)
        gu5 = torch.empty((S5, 2 * F5), dtype=torch.float16, device=dev)
        stage("gate_up_gemm", lambda: lib.hgemm(op5, wgu, out=gu5), 2.0 * S5 * H5 * 2 * F5)
        act5 = (torch.nn.functional.silu(gu5[:, :F5].float()) * gu5[:, F5:].float()).half()
        dn5 = torch.empty((S5, H5), dtype=torch.float16, device=dev)
        stage("down_gemm", lambda: lib.hgemm(act5, wd, out=dn5), 2.0 * S5 * F5 * H5)
        rows5 = torch.arange(0, S5, 61)
        c5 = {"qkv": qkv5.cpu(), "attn": o5.cpu(), "attn_lse": lse5.cpu(), "oproj": op5.cpu(), "gate_up": gu5.cpu(),
              "act": act5.cpu(), "down": dn5.cpu()}
        ref5 = so.llama_layer_ref(x5h, wqkv_h, wo_h, wgu_h, wd_h, rows=rows5, stage_inputs={
            "attn_in": c5["qkv"], "oproj_in": c5["attn"], "gu_in": c5["oproj"], "act_in": c5["gate_up"], "down_in": c5["act"]})
        for sname, cname, kk in (("qkv_gemm", "qkv", H5), ("oproj_gemm", "oproj", H5), ("gate_up_gemm", "gate_up", H5),
                                 ("down_gemm", "down", F5)):
            st[sname]["within_tolerance"] = bool(so.gemm_tolerance_ok(c5[cname][rows5], ref5[cname], kk)[0])
        st["fmha_causal_gqa_s8192"]["within_tolerance"] = bool(so.fmha_tolerance_ok(
            c5["attn"][:, :, rows5], c5["attn_lse"][:, :, rows5], ref5["attn"], ref5["attn_lse"])[0])
        full5 = so.llama_layer_ref(x5h, wqkv_h, wo_h, wgu_h, wd_h, rows=rows5)
        rel5 = float((c5["down"][rows5].float() - full5["down"]).norm() / full5["down"].norm())
        del c5, ref5, full5
        tot_ms = sum(s["ms"] for s in st.values())
        tot_fl = 2.0 * S5 * H5 * 6144 + 4.0 * 32 * 128 * causal_pairs(S5, S5) + 2.0 * S5 * H5 * H5 + 2.0 * S5 * H5 * 2 * F5 + 2.0 * S5 * F5 * H5
        other["L5_llama3_8b_layer_s8192"] = {"stages": st, "kernel_ms_total": tot_ms, "tflops_total": tot_fl / tot_ms / 1e9,
                                             "within_tolerance": all(s_["within_tolerance"] for s_ in st.values()) and rel5 < 2e-2,
                                             "end_to_end_relative_frobenius_error": rel5,
                                             "parity": "every 61st token row of every stage against the fp32 oracle fed the GPU's previous "
                                                       "stage; end to end against the pure fp32 chain",
                                             "note": "GEMM and attention stages only; reshapes and SiLU*up run in torch and are not timed; no RoPE/norm/residual"}

        # the same layer as the in-model adapter runs it: nn.Linear-layout weights, norms, RoPE, residuals, no layout copies
        del x5, wqkv, wo, wgu, wd, qkv5, q5, k5, v5, o5, lse5, a5, op5, gu5, act5, dn5, x5h, wqkv_h, wo_h, wgu_h, wd_h
        torch.cuda.empty_cache()
        from llama_layer import FineKVCache
        layer, _, wl_h = llama3_8b_layer(torch, so, dev, host_weights=True)
        xl_h = so.randn_fp16((1, S5, H5), 18)
        xl = xl_h.to(dev)
        ms_l = time_launches(lambda: layer(xl), 10, 3)
        out_l = layer(xl)[:, rows5.to(dev)].float().cpu()
        ref_l, _, _ = so.llama_decoder_layer_ref(xl_h, wl_h, torch.arange(S5)[None], 32, 8, rows=rows5)
        rel_l = float((out_l - ref_l).norm() / ref_l.norm())
        worst_l = float((out_l - ref_l).abs().max() / ref_l.abs().max())
        del wl_h, out_l, ref_l
        other["L5_decoder_layer_prefill_s8192"] = {
            "ms": ms_l, "tflops": tot_fl / ms_l / 1e9,
            "within_tolerance": rel_l <= 2e-3 and worst_l <= 2e-2, "relative_frobenius_error": rel_l, "worst_relative_to_max": worst_l,
            "parity": "every 61st token row against the fp32 oracle of the decoder layer with fp16 rounding between stages "
                      "(bounds: 2e-3 relative Frobenius, 2e-2 of the largest output)",
            "note": "whole FineLlamaDecoderLayer.forward (8 launches: norms, fused QKV GEMM, RoPE, attention on strided operands, "
                    "O projection + residual, gate/up GEMM with SiLU*up epilogue, down GEMM + residual), flops of the GEMMs and attention only"}
        Bd = 8
        cache = FineKVCache(Bd, S5 + 64, 8, device=dev)
        cache.k.normal_(0, 1)
        cache.v.normal_(0, 1)
        xd1 = so.randn_fp16((Bd, 1, H5), 19).to(dev)
        def step():
            cache.length = S5
            layer(xd1, kv_cache=cache)
        ms_s = time_launches(step, 20, 3)
        by_s = 2.0 * (sum(t.numel() for t in (layer.w_qkv, layer.w_o, layer.w_gu, layer.w_d)) + 2 * Bd * S5 * 8 * 128)
        other["L5_decoder_layer_generation_step_b8_past8192"] = {"ms": ms_s, "gbs": by_s / ms_s / 1e6,
                                                                 "pct_of_hbm_peak": 100 * by_s / ms_s / 1e6 / PEAK_HBM_GBS,
                                                                 "note": "bytes = layer weights + KV cache read once"}
        # the same step captured once into a HIP graph and replayed (warm-up on the capture stream first)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        cache.length = S5
        with torch.cuda.graph(graph, stream=side):
            layer(xd1, kv_cache=cache)
        ms_g = time_launches(graph.replay, 20, 3)
        other["L5_decoder_layer_generation_step_b8_past8192_hip_graph"] = {"ms": ms_g, "gbs": by_s / ms_g / 1e6,
                                                                           "pct_of_hbm_peak": 100 * by_s / ms_g / 1e6 / PEAK_HBM_GBS}
        del graph
        del layer, cache
        torch.cuda.empty_cache()
        # 32 such layers with their own weights and caches (a Llama-3-8B-sized decoder stack without embedding and LM head):
        # cold weights for every GEMM, as in serving
        n_layers = 32
        layers = [llama3_8b_layer(torch, so, dev)[0] for _ in range(n_layers)]
        caches = [FineKVCache(Bd, S5 + 64, 8, device=dev) for _ in range(n_layers)]
        for cch in caches:
            cch.kv.normal_(0, 1)
        def stack_prefill():
            hcur = xl
            for lyr in layers:
                hcur = lyr(hcur)
            return hcur
        def stack_step():
            hcur = xd1
            for lyr, cch in zip(layers, caches):
                cch.length = S5
                hcur = lyr(hcur, kv_cache=cch)
            return hcur
        ms_sp = time_launches(stack_prefill, 3, 1)
        ms_ss = time_launches(stack_step, 10, 2)
        other["L5_stack_of_32_layers"] = {
            "prefill_s8192_ms": ms_sp, "prefill_tokens_per_s": S5 / ms_sp * 1e3, "prefill_tflops": n_layers * tot_fl / ms_sp / 1e9,
            "generation_step_b8_past8192_ms": ms_ss, "generation_tokens_per_s": Bd / ms_ss * 1e3,
            "generation_gbs": n_layers * by_s / ms_ss / 1e6,
            "note": "32 decoder layers with distinct random weights and KV caches, no embedding / LM head / sampling"}
        del layers, caches

    # ---- CPU baseline: the same step with torch fp32 on the host cores -------------------------------------------------
    cpu_baseline = None
    if not args.no_cpu_baseline:
        cores = torch.get_num_threads()   # the box's CPU share for one GPU (OMP_NUM_THREADS), not every core of the host
        a32, b32 = a_h.float(), b_h.float()
        so.attention_sdpa_ref(q_h[:, :2], k_h[:, :1], v_h[:, :1], True)  # warm up the SDPA path on a small slice
        t0 = time.perf_counter()
        torch.matmul(a32, b32)
        t_g = time.perf_counter() - t0
        t0 = time.perf_counter()
        so.attention_sdpa_ref(q_h, k_h, v_h, True)
        t_f = time.perf_counter() - t0
        cpu_baseline = {"value": (gemm_flops + fmha_flops) / (t_g + t_f) / 1e12, "unit": "TFLOP/s", "cores": cores,
                        "kind": "port",
                        "sample": "one full step on the host: torch.matmul fp32 8192^3 (%.2f s, %.3f TFLOP/s) + torch SDPA fp32 "
                                  "causal GQA F4 with repeat_kv (%.2f s, %.3f TFLOP/s algorithmic); single run, no warm-up of the GEMM"
                                  % (t_g, gemm_flops / t_g / 1e12, t_f, fmha_flops / t_f / 1e12),
                        "cpu": _cpu_model(), "logical_cpus_visible": os.cpu_count(), "threads_used": cores}
        del a32, b32
        if not args.no_other_configs:
            # the other configurations on the same host cores (reported baselines): median of 3 runs after one warm-up, a
            # single run for the decoder layer chain
            def cpu_ms(fn, runs=3, warm=1):
                for _ in range(warm):
                    fn()
                ts = []
                for _ in range(runs):
                    t0_ = time.perf_counter()
                    fn()
                    ts.append((time.perf_counter() - t0_) * 1e3)
                return sorted(ts)[len(ts) // 2]
            for name, (m_, n_, k_) in (("G1_gemm_1024", (1024, 1024, 1024)), ("G2a_gemm_4096", (4096, 4096, 4096)),
                                       ("G2c_gemm_decode_16x14336x4096", (16, 14336, 4096))):
                x_c, w_c = so.randn_fp16((m_, k_), 1).float(), so.randn_fp16((k_, n_), 2, 0.02).float()
                ms_c = cpu_ms(lambda: torch.matmul(x_c, w_c))
                other[name]["cpu_ms"] = ms_c
                other[name]["cpu_tflops"] = 2.0 * m_ * n_ * k_ / ms_c / 1e9
            q3c, k3c, v3c = so.fmha_inputs(4, 32, 32, 1024, 1024, seed=42)
            ms_c = cpu_ms(lambda: so.attention_sdpa_ref(q3c, k3c, v3c, False))
            other["F3_fmha_noncausal_b4_h32_s1024"]["cpu_ms"] = ms_c
            other["F3_fmha_noncausal_b4_h32_s1024"]["cpu_tflops"] = 4.0 * 4 * 32 * 128 * 1024 * 1024 / ms_c / 1e9
            del q3c, k3c, v3c
            S5c, H5c, F5c = 8192, 4096, 14336
            x5c = so.randn_fp16((S5c, H5c), 0)
            w5c = [so.randn_fp16((H5c, 6144), 1, 0.02), so.randn_fp16((H5c, H5c), 2, 0.02), so.randn_fp16((H5c, 2 * F5c), 3, 0.02),
                   so.randn_fp16((F5c, H5c), 4, 0.02)]
            def l5_cpu():
                # the chain of the decoder layer's matrix stages in fp32 on the host (SDPA for the attention stage)
                qkv_c = x5c.float() @ w5c[0].float()
                qc = qkv_c[:, :4096].reshape(S5c, 32, 128).permute(1, 0, 2)[None]
                kc = qkv_c[:, 4096:5120].reshape(S5c, 8, 128).permute(1, 0, 2)[None]
                vc = qkv_c[:, 5120:].reshape(S5c, 8, 128).permute(1, 0, 2)[None]
                oc = so.attention_sdpa_ref(qc, kc, vc, True)
                oc = (oc[0] if isinstance(oc, tuple) else oc)[0].permute(1, 0, 2).reshape(S5c, H5c)
                gu_c = (oc @ w5c[1].float()) @ w5c[2].float()
                return (torch.nn.functional.silu(gu_c[:, :F5c]) * gu_c[:, F5c:]) @ w5c[3].float()
            t0 = time.perf_counter()
            l5_cpu()
            ms_c = (time.perf_counter() - t0) * 1e3
            fl5 = 2.0 * S5c * H5c * 6144 + 4.0 * 32 * 128 * causal_pairs(S5c, S5c) + 2.0 * S5c * H5c * H5c + 2.0 * S5c * H5c * 2 * F5c + 2.0 * S5c * F5c * H5c
            other["L5_llama3_8b_layer_s8192"]["cpu_ms"] = ms_c
            other["L5_llama3_8b_layer_s8192"]["cpu_tflops"] = fl5 / ms_c / 1e9
            other["cpu_baselines_note"] = ("cpu_ms / cpu_tflops: torch fp32 on %d threads of %s (torch.matmul; SDPA with repeat_kv; L5: the four "
                                           "products, causal SDPA and the activation chained, one run)" % (cores, _cpu_model()))
            del x5c, w5c

    step_protocol = ("value / ms_per_step: %d steps (GEMM then attention, back to back on one stream) after %d warm-up steps, host "
                     "clock between device synchronisations" % (args.steps, args.warmup))
    kernel_protocol = ("kernels / roofline*: per kernel >= 10 warm-up launches, then untimed launches until ~25 ms of that kernel "
                       "have run (clocks settle), then >= 50 launches between two HIP events on the launch stream; median / "
                       "minimum from a second batch with an event after every launch; ms_graph_replay / other_configs GEMMs: "
                       "the launches replayed from one HIP graph")
    out = {
        "metric": "TFLOP/s + % fp16 MFMA peak: GEMM 8192^3 and causal GQA FMHA s=4096 d=128",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp16 (fp32 accumulate)", "data": "synthetic",
        "config": {"workload": "one step = hgemm 8192x8192x8192 NN (G2b) + fmha fwd causal GQA b1 h32/8 s4096 d128 with LSE (F4)",
                   "flops_per_step": gemm_flops + fmha_flops, "pct_of_fp16_mfma_peak": 100 * value / PEAK_FP16_TFLOPS},
        "step_protocol": step_protocol, "kernel_protocol": kernel_protocol,
        "kernels": kernels, "roofline": roofline, "roofline_fmha": roofline_fmha, "roofline_decode_gemm": roofline_g2c,
        "cpu_baseline": cpu_baseline,
        "other_configs": other, "parity": checks,
    }
    print(json.dumps(out))


# name -> ("gemm", M, N, K, layout) or ("fmha", B, Hq, Hkv, Sq, Sk, causal); each runs one kernel of the library
KERNEL_CONFIGS = {
    "g1_gemm_1024_nn": ("gemm", 1024, 1024, 1024, "NN"),                    # 64x64 tiles, two workgroups to a CU
    "g2a_gemm_4096_nn": ("gemm", 4096, 4096, 4096, "NN"),                   # 256x256 tiles, one per CU
    "g2b_gemm_8192_nn": ("gemm", 8192, 8192, 8192, "NN"),                   # 256x256 tiles
    "g2b_gemm_8192_nt": ("gemm", 8192, 8192, 8192, "NT"),
    "gemm_2048x2048x4096_nn": ("gemm", 2048, 2048, 4096, "NN"),             # 128x128 tiles
    "gemm_2048x4096x4096_nn": ("gemm", 2048, 4096, 4096, "NN"),             # 128x256 tiles, one per CU
    "g2c_gemm_16x14336x4096_nn": ("gemm", 16, 14336, 4096, "NN"),           # split-K small-M kernel
    "gemm_16x14336x4096_nt": ("gemm", 16, 14336, 4096, "NT"),               # split-K small-M kernel (NT)
    "gemm_8x28672x4096_nt": ("gemm", 8, 28672, 4096, "NT"),                 # split-K small-M kernel (NT), A rows 0..7 only
    "gemm_64x14336x4096_nt": ("gemm", 64, 14336, 4096, "NT"),               # 64x64 tiles, 8-deep ring
    "gemm_64x4096x14336_nt": ("gemm", 64, 4096, 14336, "NT"),               # 64x64 tiles, split-K over 8 ranges
    "gemm_16x4096x14336_nt": ("gemm", 16, 4096, 14336, "NT"),               # split-K small-M kernel (NT)
    "gemm_512x4096x14336_nt": ("gemm", 512, 4096, 14336, "NT"),             # 128x128 tiles, split-K over 2 ranges
    "vendor_gemm_512x4096x14336_nt": ("vendor_gemm", 512, 4096, 14336, "NT"),
    "gemm_1024x4096x4096_nt": ("gemm", 1024, 4096, 4096, "NT"),             # 128x64 tiles
    "f3_fmha_noncausal_b4_h32_s1024": ("fmha", 4, 32, 32, 1024, 1024, False),   # ping-pong kernel, 256-query work items
    "f4_fmha_causal_gqa_s4096": ("fmha", 1, 32, 8, 4096, 4096, True),           # ping-pong kernel
    "l5_fmha_causal_gqa_s8192": ("fmha", 1, 32, 8, 8192, 8192, True),           # ping-pong kernel
    "fmha_causal_gqa_s1024": ("fmha", 1, 32, 8, 1024, 1024, True),              # ping-pong kernel, 128-query work items (128 items of 256 queries would not fill the CUs)
    "fmha_chunk_q128_over_8192": ("fmha", 1, 32, 8, 128, 8192, True),           # key ranges + merge kernel
    "fmha_chunk_q512_over_32768": ("fmha", 1, 32, 8, 512, 32768, True),
    "fmha_decode_b1_sk8192": ("fmha", 1, 32, 8, 1, 8192, False),                # split-KV kernel
    "fmha_decode_b8_sk8192": ("fmha", 8, 32, 8, 1, 8192, False),
    "fmha_decode_b64_sk8192": ("fmha", 64, 32, 8, 1, 8192, False),              # one key range per (batch, kv head)
    # a kernel that only reads (profiling twin of the library, --timeline): the yardstick of the bandwidth-bound kernels, at
    # the sizes of the big operands of a Llama-3-8B generation step at batch 8 (O, QKV, down, gate/up weights; K + V)
    "stream_read_34mb": ("read", 4096 * 4096 * 2),
    "stream_read_50mb": ("read", 6144 * 4096 * 2),
    "stream_read_117mb": ("read", 14336 * 4096 * 2),
    "stream_read_235mb": ("read", 28672 * 4096 * 2),
    "stream_read_268mb": ("read", 2 * 8 * 8 * 8192 * 128 * 2),
    # matrix instructions back to back on register operands, two waves per SIMD on every CU (profiling twin, --timeline): what
    # the matrix pipes sustain on N(0,1) operands under the board's power limit, and on zeros (--zero-inputs)
    "mfma_only_16x16x32": ("mfma", 16),
    "mfma_only_32x32x16": ("mfma", 32),
    # one wave per SIMD issues the matrix instructions of an attention key tile while the other runs the softmax's
    # instruction mix (profiling twin, --timeline): each alone, then side by side
    "mfma_valu_16x16x32": ("mfma_valu", 16),
    "mfma_valu_32x32x16": ("mfma_valu", 32),
    # the vendor library on the same box, same operands and timing loop (torch.matmul = hipBLASLt); not this code
    "vendor_gemm_8192_nn": ("vendor_gemm", 8192, 8192, 8192, "NN"),
    "vendor_gemm_8192_nt": ("vendor_gemm", 8192, 8192, 8192, "NT"),
    "vendor_gemm_4096_nn": ("vendor_gemm", 4096, 4096, 4096, "NN"),
    "vendor_gemm_2048x2048x4096_nn": ("vendor_gemm", 2048, 2048, 4096, "NN"),
    "vendor_gemm_2048x4096x4096_nn": ("vendor_gemm", 2048, 4096, 4096, "NN"),
    "vendor_gemm_1024x4096x4096_nt": ("vendor_gemm", 1024, 4096, 4096, "NT"),
    "vendor_gemm_1024_nn": ("vendor_gemm", 1024, 1024, 1024, "NN"),
}


def timeline_summary(lib, cfg):
    """Summary of the per-workgroup stamps the profiling twin of the library recorded in its last attention launch
    (csrc/mi355_timeline.h): microseconds from the first workgroup's entry, 100 MHz wall clock; cycles = shader clock."""
    import ctypes
    import numpy as np
    gemm = cfg[0] == "gemm"
    decode = (not gemm) and cfg[4] == 1
    buf = np.zeros(4096 * 8, dtype=np.uint64)
    read = (lib.load().mi355_timeline_read_hgemm if gemm else
            lib.load().mi355_timeline_read_fmha_decode if decode else lib.load().mi355_timeline_read_fmha_fwd)
    read.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
    rc = read(buf.ctypes.data_as(ctypes.c_void_p), buf.nbytes)
    if rc != 0:
        raise RuntimeError("timeline read failed: %d" % rc)
    rec = buf.reshape(4096, 8).astype(np.float64)
    rec = rec[rec[:, 0] > 0]
    t0 = rec[:, 0].min()
    us = lambda col: (col[col > 0] - t0) / 100.0
    stat = lambda x: {"workgroups": int(x.size), "min": round(float(x.min()), 2), "mean": round(float(x.mean()), 2), "max": round(float(x.max()), 2)} if x.size else None
    if decode:
        names = ["entry", "first_tile_landed", "key_range_done", "partials_stored", "ticket_drawn", "merge_partials_landed",
                 "merge_summed", "exit"]
        return {"unit": "us after the first workgroup's entry", **{n: stat(us(rec[:, i])) for i, n in enumerate(names)}}
    tiles = np.maximum(rec[:, 6], 1.0)
    loop_us = (rec[:, 2] - rec[:, 1]) / 100.0
    loop_cycles = rec[:, 5] - rec[:, 4]
    big = rec[:, 6] >= 0.75 * rec[:, 6].max()    # pipeline fill and drain weigh on workgroups with few tiles
    if gemm:   # a K tile of 64 is 64 MFMA 16x16x32 per wave of the 256x256 tile, 2 waves per SIMD
        return {"unit": "us after the first workgroup's entry", "workgroups_recorded": int(rec.shape[0]),
                "kernel_span_us": round(float((rec[:, 3].max() - t0) / 100.0), 2),
                "prologue_us": stat((rec[:, 1] - rec[:, 0]) / 100.0), "epilogue_us": stat((rec[:, 3] - rec[:, 2]) / 100.0),
                "k_tiles_per_workgroup": stat(rec[:, 6]), "loop_cycles_per_k_tile": stat(loop_cycles / tiles),
                "loop_clock_ghz": stat(loop_cycles / (loop_us * 1e3)),
                "note": "MFMA cycles per K tile and SIMD: 2048 for 256x256 tiles (8 waves), 1024 for 128x128 tiles (4 waves)"}
    return {"unit": "us after the first workgroup's entry", "workgroups": int(rec.shape[0]),
            "kernel_span_us": round(float((rec[:, 3].max() - t0) / 100.0), 2),
            "prologue_us": stat((rec[:, 1] - rec[:, 0]) / 100.0), "epilogue_us": stat((rec[:, 3] - rec[:, 2]) / 100.0),
            "key_tiles_per_workgroup": stat(rec[:, 6]),
            "loop_us_per_key_tile": stat(loop_us / tiles),
            "long_workgroups": {"loop_cycles_per_key_tile": stat((loop_cycles / tiles)[big]),
                                "loop_clock_ghz": stat((loop_cycles / (loop_us * 1e3))[big])},
            "mfma_cycles_per_key_tile_per_simd": 2 * 68 * 16}


def run_kernel_config(args, torch, lib, so, dev):
    cfg = KERNEL_CONFIGS[args.kernel_config]
    cur = lambda: torch.cuda.current_stream().cuda_stream   # at call time: graph capture runs on a stream of its own
    if cfg[0] == "read":
        import ctypes
        if not args.timeline:
            sys.exit("bench.py: the stream_read configurations live in the profiling twin of the library: add --timeline")
        read = lib.load().mi355_timeline_stream_read
        read.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p]
        read.restype = ctypes.c_int
        nbytes = cfg[1]
        n_copies = copies_to_defeat_cache(nbytes) if args.rotate_operands else 1
        bufs = [torch.full((nbytes // 2,), 1.0, dtype=torch.float16, device=dev) for _ in range(n_copies)]
        sink = torch.zeros(4, dtype=torch.float32, device=dev)

        def call(j):
            rc = read(bufs[j].data_ptr(), nbytes, sink.data_ptr(), cur())
            if rc != 0:
                raise RuntimeError("mi355_timeline_stream_read failed: %d" % rc)
        t = time_launches(rotating(call, n_copies), args.steps, args.warmup, stats=True)
        print(json.dumps(dict(t, kernel_config=args.kernel_config, rotate_operands=bool(args.rotate_operands), copies=n_copies,
                              gbs=nbytes / t["ms"] / 1e6, algorithmic_bytes=float(nbytes))))
        return
    if cfg[0] in ("mfma", "mfma_valu"):
        import ctypes
        import numpy as np
        if not args.timeline:
            sys.exit("bench.py: the mfma_* configurations live in the profiling twin of the library: add --timeline")
        L = lib.load()
        shape = cfg[1]
        fill = so.randn_fp16((8192,), 5).to(dev)
        if args.zero_inputs:
            fill.zero_()
        out = torch.empty(256 * 512, dtype=torch.float32, device=dev)
        vp, i32 = ctypes.c_void_p, ctypes.c_int
        if cfg[0] == "mfma":
            f = L.mi355_timeline_mfma_only
            f.argtypes, f.restype = [i32, vp, vp, i32, vp], i32
            iters = 2000
            def fn():
                rc = f(shape, fill.data_ptr(), out.data_ptr(), iters, cur())
                if rc != 0:
                    raise RuntimeError("mi355_timeline_mfma_only failed: %d" % rc)
            t = time_launches(fn, args.steps, args.warmup, stats=True)
            flops = 256.0 * 8 * iters * 32 * (2.0 * 16 * 16 * 32 if shape == 16 else 2.0 * 32 * 32 * 16)
            print(json.dumps(dict(t, kernel_config=args.kernel_config, zero_inputs=bool(args.zero_inputs), tflops=flops / t["ms"] / 1e9,
                                  pct_of_fp16_mfma_peak=100 * flops / t["ms"] / 1e9 / PEAK_FP16_TFLOPS,
                                  note="256 workgroups x 8 waves, %d x 32 MFMA %s per wave, operands in registers" % (
                                      iters, "16x16x32" if shape == 16 else "32x32x16"))))
            return
        f = L.mi355_timeline_mfma_valu
        f.argtypes, f.restype = [i32, vp, vp, i32, i32, vp], i32
        rd = L.mi355_timeline_read_mfma_valu
        rd.argtypes, rd.restype = [vp, ctypes.c_size_t], i32
        iters = 400
        res = {}
        modes = [(1, "matrix_wave_alone"), (2, "valu_wave_alone"), (3, "side_by_side")]
        if shape == 16:
            modes += [(5, "matrix_wave_with_lds_fragment_reads_alone"), (7, "side_by_side_with_lds_fragment_reads")]
        for mode, tag in modes:
            for _ in range(3):
                rc = f(shape, fill.data_ptr(), out.data_ptr(), iters, mode, cur())
                if rc != 0:
                    raise RuntimeError("mi355_timeline_mfma_valu failed: %d" % rc)
            torch.cuda.synchronize()
            buf = np.zeros(512, dtype=np.uint64)
            if rd(buf.ctypes.data_as(vp), buf.nbytes) != 0:
                raise RuntimeError("mi355_timeline_read_mfma_valu failed")
            cyc = buf.reshape(256, 2).astype(np.float64) / iters
            res[tag] = {"matrix_wave_cycles_per_tile": round(float(cyc[:, 0].mean()), 1) if mode & 1 else None,
                        "valu_wave_cycles_per_tile": round(float(cyc[:, 1].mean()), 1) if mode & 2 else None}
        print(json.dumps({"kernel_config": args.kernel_config, "zero_inputs": bool(args.zero_inputs), "cycles": res,
                          "matrix_pipe_cycles_per_tile": 68 * 16,
                          "note": "per key tile of a 32-query wave: matrix wave = 68 MFMA 16x16x32 (34 MFMA 32x32x16) on registers, "
                                  "VALU wave = 16 v_max3 + 32 v_fma + 32 v_exp + 16 v_cvt_pk; the two waves share one SIMD, no barriers, "
                                  "no memory traffic"}))
        return
    if cfg[0] == "vendor_gemm":
        _, M, N, K, lay = cfg
        a_h, b_h = so.gemm_inputs(M, N, K, seed=0, a_std=1.0, b_std=0.02)
        a, b = a_h.to(dev), b_h.to(dev)
        if lay == "NT":
            b = b.t().contiguous().t()   # stored [N, K], passed as its transposed view
        if args.zero_inputs:
            a.zero_(), b.zero_()
        c = torch.empty((M, N), dtype=torch.float16, device=dev)
        t = time_launches(lambda: torch.matmul(a, b, out=c), args.steps, args.warmup, stats=True)
        flops = 2.0 * M * N * K
        print(json.dumps(dict(t, kernel_config=args.kernel_config, zero_inputs=bool(args.zero_inputs), tflops=flops / t["ms"] / 1e9,
                              pct_of_fp16_mfma_peak=100 * flops / t["ms"] / 1e9 / PEAK_FP16_TFLOPS,
                              note="torch.matmul (hipBLASLt) on the operands of the configuration of that shape; the vendor library, not this code")))
        return
    if cfg[0] == "gemm":
        _, M, N, K, lay = cfg
        a_h, b_h = so.gemm_inputs(M, N, K, seed=0, a_std=1.0, b_std=0.02)
        if lay == "NT":
            b_h = b_h.t().contiguous()
        a, b = a_h.to(dev), b_h.to(dev)
        if args.zero_inputs:
            a.zero_(), b.zero_()
        c = torch.empty((M, N), dtype=torch.float16, device=dev)
        fn = lambda: lib.hgemm_raw(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, a.shape[1], b.shape[1], N, lib.LAYOUTS[lay], cur())
        flops, nbytes = 2.0 * M * N * K, 2.0 * (M * K + K * N + M * N)
        if args.rotate_operands:
            bs = [b] + [b.clone() for _ in range(copies_to_defeat_cache(2.0 * K * N) - 1)]
            fn = rotating(lambda j: lib.hgemm_raw(a.data_ptr(), bs[j].data_ptr(), c.data_ptr(), M, N, K, a.shape[1], b.shape[1], N,
                                                  lib.LAYOUTS[lay], cur()), len(bs))
    else:
        _, B, Hq, Hkv, Sq, Sk, causal = cfg
        q, k, v = (t.to(dev) for t in so.fmha_inputs(B, Hq, Hkv, Sq, Sk, seed=42))
        if args.zero_inputs:
            q.zero_(), k.zero_(), v.zero_()
        o = torch.empty_like(q)
        lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=dev)
        fn = lambda: lib.fmha_fwd_raw(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(), B, Hq, Hkv, Sq, Sk,
                                      128, 1.0 / math.sqrt(128), int(causal), Sk, cur())
        flops = 4.0 * B * Hq * 128 * (causal_pairs(Sq, Sk) if causal else Sq * Sk)
        nbytes = 2.0 * (2 * B * Hq * Sq * 128 + 2 * B * Hkv * Sk * 128) + 4.0 * B * Hq * Sq
        if args.rotate_operands:
            kvs = [(k, v)] + [(k.clone(), v.clone()) for _ in range(copies_to_defeat_cache(4.0 * B * Hkv * Sk * 128) - 1)]
            fn = rotating(lambda j: lib.fmha_fwd_raw(q.data_ptr(), kvs[j][0].data_ptr(), kvs[j][1].data_ptr(), o.data_ptr(),
                                                     lse.data_ptr(), B, Hq, Hkv, Sq, Sk, 128, 1.0 / math.sqrt(128), int(causal), Sk,
                                                     cur()), len(kvs))
    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    t = time_launches(fn, args.steps, args.warmup, stats=True)
    if args.timeline:
        fn()
        torch.cuda.synchronize()
        print(json.dumps(dict(t, kernel_config=args.kernel_config, zero_inputs=bool(args.zero_inputs), timeline=timeline_summary(lib, cfg))))
        return
    t["ms_graph_replay"] = time_graph(fn, args.steps, args.warmup)
    print(json.dumps(dict(t, kernel_config=args.kernel_config, rotate_operands=bool(args.rotate_operands),
                          tflops=flops / t["ms"] / 1e9, gbs=nbytes / t["ms"] / 1e6,
                          tflops_graph_replay=flops / t["ms_graph_replay"] / 1e9, gbs_graph_replay=nbytes / t["ms_graph_replay"] / 1e6,
                          algorithmic_flop=flops, algorithmic_bytes=nbytes)))


def llama3_8b_layer(torch, so, dev, S5=8192, H5=4096, F5=14336, host_weights=False):
    """FineLlamaDecoderLayer at Llama-3-8B shapes (32 q / 8 kv heads of 128) with seeded random weights; with
    host_weights also the dict of CPU weights the oracle takes."""
    from llama_layer import FineLlamaDecoderLayer
    gw = lambda shape, seed: so.randn_fp16(shape, seed, 0.02)
    wh = dict(q=gw((4096, H5), 11), k=gw((1024, H5), 12), v=gw((1024, H5), 13), o=gw((H5, 4096), 14), gate=gw((F5, H5), 15),
              up=gw((F5, H5), 16), down=gw((H5, F5), 17), ln1=torch.ones(H5, dtype=torch.float16),
              ln2=torch.ones(H5, dtype=torch.float16))
    layer = FineLlamaDecoderLayer({k: v.to(dev) for k, v in wh.items()}, 32, 8, max_positions=S5 + 64)
    return (layer, S5, wh) if host_weights else (layer, S5)


def _cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


if __name__ == "__main__":
    main()

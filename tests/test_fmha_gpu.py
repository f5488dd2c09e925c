"""GPU parity tests of the fused attention forward: the HIP kernel called through the C ABI (ctypes) and through
the torch operators, against the CPU oracle on the same seeded inputs. Tolerance (benchmark definition):
max|O - O_ref| <= 2e-3 and max|LSE - LSE_ref| <= 1e-3 against fp32 softmax attention."""
import math
import os

import numpy as np
import pytest
import torch

import serving_oracle as so

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def run(lib, gpu, q, k, v, causal=False, kv_valid_len=None, variant=0):
    o, lse = lib.fmha_fwd(q.to(gpu), k.to(gpu), v.to(gpu), causal=causal, kv_valid_len=kv_valid_len, variant=variant)
    torch.cuda.synchronize()
    return o.cpu(), lse.cpu()


def check(lib, gpu, q, k, v, causal=False, kv_valid_len=None, variant=0):
    o, lse = run(lib, gpu, q, k, v, causal, kv_valid_len, variant)
    o_ref, lse_ref = so.attention_ref(q, k, v, causal=causal, kv_valid_len=kv_valid_len)
    ok, st = so.fmha_tolerance_ok(o, lse, o_ref, lse_ref)
    assert ok, (tuple(q.shape), tuple(k.shape), causal, kv_valid_len, st)
    return o, lse


# ---- benchmark configurations ------------------------------------------------------------------------------------
def test_config_f3_noncausal_mha(lib, gpu):
    q, k, v = so.fmha_inputs(4, 32, 32, 1024, 1024, seed=42)
    check(lib, gpu, q, k, v, causal=False)


def test_config_f4_causal_gqa_with_lse(lib, gpu):
    q, k, v = so.fmha_inputs(1, 32, 8, 4096, 4096, seed=42)
    o, lse = check(lib, gpu, q, k, v, causal=True)
    assert lse.shape == (1, 32, 4096) and lse.dtype == torch.float32


# ---- closed forms ---------------------------------------------------------------------------------------------------
def test_equal_keys_running_mean(lib, gpu):
    B, H, S = 1, 2, 333
    q = so.randn_fp16((B, H, S, 128), 1)
    k = so.randn_fp16((B, H, 1, 128), 2).expand(B, H, S, 128).contiguous()
    v = so.randn_fp16((B, H, S, 128), 3)
    o, lse = run(lib, gpu, q, k, v, causal=True)
    vm = v.float().cumsum(2) / torch.arange(1, S + 1)[None, None, :, None]
    s0 = (q.float() * k.float()).sum(-1) / math.sqrt(128)
    assert (o.float() - vm).abs().max() <= 2e-3
    assert (lse - (s0 + torch.log(torch.arange(1, S + 1).float()))).abs().max() <= 1e-3


def test_first_causal_row_is_first_value_exactly(lib, gpu):
    q, k, v = so.fmha_inputs(2, 4, 2, 200, 200, seed=5)
    o, lse = run(lib, gpu, q, k, v, causal=True)
    assert torch.equal(o[:, :, 0], v.repeat_interleave(2, 1)[:, :, 0])
    s00 = (q.float()[:, :, 0] * k.float().repeat_interleave(2, 1)[:, :, 0]).sum(-1) / math.sqrt(128)
    assert (lse[:, :, 0] - s00).abs().max() <= 1e-4


def test_ones_value_rows_sum_to_one_and_zero_query_lse(lib, gpu):
    q, k, _ = so.fmha_inputs(1, 2, 2, 150, 777, seed=6)
    v = torch.ones(1, 2, 777, 128).half()
    o, _ = run(lib, gpu, q, k, v, causal=False)
    assert (o.float() - 1).abs().max() <= 1e-3
    o, lse = run(lib, gpu, torch.zeros_like(q), k, v, causal=True)  # Sq=150 < Sk=777: query i sees 628+i keys
    assert (lse[0, 0] - torch.log(torch.arange(628, 778).float())).abs().max() <= 1e-4


def test_dominant_key_selects_its_value(lib, gpu):
    _, k, v = so.fmha_inputs(1, 1, 1, 64, 500, seed=7)
    q = (k[:, :, 321:322] * 8).expand(1, 1, 64, 128).contiguous()
    o, _ = run(lib, gpu, q, k, v)
    assert (o.float() - v.float()[:, :, 321:322]).abs().max() <= 2e-3


def test_key_permutation_invariance_across_tiles(lib, gpu):
    q, k, v = so.fmha_inputs(1, 2, 1, 96, 1000, seed=8)
    perm = torch.randperm(1000, generator=torch.Generator().manual_seed(1))
    o1, l1 = run(lib, gpu, q, k, v)
    o2, l2 = run(lib, gpu, q, k[:, :, perm].contiguous(), v[:, :, perm].contiguous())
    assert (o1.float() - o2.float()).abs().max() <= 2e-3 and (l1 - l2).abs().max() <= 1e-4


def test_gqa_heads_sharing_kv_with_identical_queries_agree(lib, gpu):
    q1 = so.randn_fp16((1, 1, 130, 128), 9)
    q = q1.expand(1, 8, 130, 128).contiguous()
    _, k, v = so.fmha_inputs(1, 8, 2, 130, 130, seed=10)
    o, lse = run(lib, gpu, q, k, v, causal=True)
    for g in range(2):
        for h in range(1, 4):
            assert torch.equal(o[:, 4 * g + h], o[:, 4 * g]) and torch.equal(lse[:, 4 * g + h], lse[:, 4 * g])
    assert not torch.equal(o[:, 0], o[:, 4])


# ---- ragged shapes, masks, decode -----------------------------------------------------------------------------------
@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,causal,kvv", [
    (1, 1, 1, 128, 128, False, None), (1, 1, 1, 128, 128, True, None), (1, 4, 1, 128, 128, True, None),
    (2, 4, 2, 100, 77, False, None), (2, 4, 2, 100, 177, True, None), (1, 2, 1, 300, 300, True, 290),
    (1, 2, 2, 70, 40, True, None),      # Sq > Sk, causal: the first 30 queries see no key
    (1, 2, 2, 1, 333, False, None),     # decode step: one query
    (3, 6, 3, 1, 64, False, 50), (1, 2, 1, 65, 129, True, None), (1, 1, 1, 8, 8, True, None),
    (1, 2, 2, 257, 63, False, 1), (1, 3, 1, 511, 513, True, 512), (2, 2, 2, 64, 1024, True, None),
])
def test_ragged_shapes_and_masks(lib, gpu, B, Hq, Hkv, Sq, Sk, causal, kvv):
    q, k, v = so.fmha_inputs(B, Hq, Hkv, Sq, Sk, seed=Sq * 7 + Sk)
    o, lse = check(lib, gpu, q, k, v, causal, kvv)
    if causal and Sq > Sk:
        n = Sq - Sk
        assert bool((o[:, :, :n] == 0).all()) and bool(torch.isinf(lse[:, :, :n]).all()) and bool((lse[:, :, :n] < 0).all())


def _seeded_attention_shapes(n, seed):
    """n prefill shapes drawn with a fixed seed: a few to a few thousand work items (one workgroup per CU walks them in
    rounds), ragged query and key counts, GQA groups of 1..8, causal or not, sometimes a valid length short of Sk."""
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < n:
        b = int(rng.choice([1, 2, 3, 5]))
        hkv = int(rng.choice([1, 2, 4, 8]))
        hq = hkv * int(rng.choice([1, 2, 4, 8]))
        sq = int(rng.choice([33, 128, 200, 256, 384, 640, 1000, 1024, 1500]))
        sk = sq if rng.random() < 0.5 else int(rng.choice([64, 191, 256, 700, 1024, 2048]))
        causal = bool(rng.random() < 0.6)
        kvv = None if rng.random() < 0.7 else max(1, sk - int(rng.integers(1, 70)))
        if b * hq * sq * sk > 1.6e8:
            continue
        out.append((b, hq, hkv, sq, sk, causal, kvv))
    return out


@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,causal,kvv", _seeded_attention_shapes(16, 4242) + [
    (8, 32, 8, 512, 512, True, None), (4, 40, 8, 384, 384, False, None), (16, 24, 8, 130, 130, True, None)])   # many short items: several rounds per workgroup
def test_seeded_random_prefill_shapes(lib, gpu, variant, B, Hq, Hkv, Sq, Sk, causal, kvv):
    q, k, v = so.fmha_inputs(B, Hq, Hkv, Sq, Sk, seed=B + Hq + Sq + Sk)
    check(lib, gpu, q, k, v, causal, kvv, variant=variant)


@pytest.mark.parametrize("variant", [1, 2])
@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,causal,kvv", [
    (1, 4, 1, 128, 128, True, None), (2, 4, 2, 100, 177, True, None), (1, 2, 1, 300, 300, True, 290),
    (1, 2, 2, 70, 40, True, None), (1, 2, 2, 1, 333, False, None), (2, 3, 3, 600, 1000, False, 999),
    (1, 2, 1, 513, 515, True, None), (1, 1, 1, 700, 64, False, 1), (1, 2, 2, 256, 1024, True, None),
])
def test_every_kernel_variant_on_ragged_shapes(lib, gpu, variant, B, Hq, Hkv, Sq, Sk, causal, kvv):
    q, k, v = so.fmha_inputs(B, Hq, Hkv, Sq, Sk, seed=Sq + 3 * Sk + variant)
    check(lib, gpu, q, k, v, causal, kvv, variant=variant)   # pinned through the library's internal test hook


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,causal,kvv", [
    (1, 32, 8, 1, 8192, False, None),    # Llama-3-8B generation step
    (2, 8, 2, 1, 1000, False, 999), (1, 32, 8, 4, 2048, True, None), (1, 4, 4, 1, 600, False, None),
    (3, 16, 2, 3, 777, True, 700), (1, 1, 1, 1, 70000, False, None), (1, 32, 1, 1, 513, False, 512),
])
def test_generation_step_split_kv_path(lib, gpu, B, Hq, Hkv, Sq, Sk, causal, kvv):
    # Hq/Hkv * Sq <= 32 and >= 512 valid keys: the split-KV kernels; compared with the oracle and with the
    # prefill kernel on the same inputs
    q, k, v = so.fmha_inputs(B, Hq, Hkv, Sq, Sk, seed=Sk + Hq)
    o, lse = check(lib, gpu, q, k, v, causal, kvv)
    o1, lse1 = run(lib, gpu, q, k, v, causal, kvv, variant=1)
    assert (o.float() - o1.float()).abs().max() <= 2e-3 and (lse - lse1).abs().max() <= 1e-3


def test_generation_step_workspace_shared_by_calls_of_different_shapes(lib, gpu):
    # One workspace per stream serves every call. The ticket counters sit in a region of fixed size in front of the partial
    # results: calls with 8, then 4, then 64, then 8 (batch, kv head) pairs must all find their counters at zero (with a
    # counter region sized by the call, the partial results of the second call lay on counters of the fourth).
    for B, Hq, Hkv, Sk in ((1, 32, 8, 4096), (2, 8, 2, 1500), (8, 32, 8, 2048), (1, 32, 8, 4096), (170, 1, 1, 640), (3, 8, 4, 1024)):
        q, k, v = so.fmha_inputs(B, Hq, Hkv, 1, Sk, seed=B + Sk)
        check(lib, gpu, q, k, v, False, None)


def _seeded_mixed_cases(n, seed):
    """n cases drawn with a fixed seed over everything a caller can vary at once: prefill, generation-step and very short
    shapes; fp16 or bf16; contiguous [B,H,S,D] tensors or [B,S,H,D] tensors viewed as [B,H,S,D]; a valid length short of
    Sk (with NaNs behind it); the entry point that allocates nothing."""
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < n:
        mode = str(rng.choice(["prefill", "prefill", "step", "short"]))
        hkv = int(rng.choice([1, 2, 4, 8]))
        hq = hkv * int(rng.choice([1, 1, 2, 4, 8]))
        if mode == "prefill":
            b = int(rng.choice([1, 2, 3])); sq = int(rng.choice([100, 129, 255, 256, 257, 511, 777, 1024])); sk = sq + int(rng.choice([0, 0, 1, 63, 200]))
        elif mode == "step":
            b = int(rng.choice([1, 2, 4, 9])); sq = int(rng.choice([1, 1, 2, 4])); sk = int(rng.choice([512, 513, 1000, 2048, 5000]))
        else:
            b = int(rng.choice([1, 2, 7])); sq = int(rng.choice([1, 2, 5, 16, 33, 64])); sk = int(rng.choice([1, 3, 17, 63, 64, 65, 130, 400]))
        if b * hq * sq * sk > 4e7:
            continue
        causal = bool(rng.random() < 0.5)
        if causal and sq > sk:
            sk = sq
        kvv = sk if rng.random() < 0.6 else int(rng.integers(1, sk + 1))
        bf16 = bool(rng.random() < 0.25)
        out.append((b, hq, hkv, sq, sk, causal, kvv, bf16, bool(rng.random() < 0.4), (not bf16) and bool(rng.random() < 0.3)))
    return out


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,causal,kvv,bf16,strided,noalloc", _seeded_mixed_cases(48, 777))
def test_seeded_random_cases_across_dtypes_views_and_entry_points(lib, gpu, B, Hq, Hkv, Sq, Sk, causal, kvv, bf16, strided, noalloc):
    q, k, v = (bf16_inputs if bf16 else so.fmha_inputs)(B, Hq, Hkv, Sq, Sk, seed=B + 3 * Hq + 5 * Sq + 7 * Sk)
    o_ref, lse_ref = so.attention_ref(q, k, v, causal=causal, kv_valid_len=kvv)
    k, v = k.clone(), v.clone()
    k[:, :, kvv:] = float("nan")   # keys behind the valid length must not be read into the result
    v[:, :, kvv:] = float("nan")
    if strided:
        qg, kg, vg = (t.transpose(1, 2).contiguous().to(gpu).transpose(1, 2) for t in (q, k, v))
        o = torch.full((B, Sq, Hq, 128), 7.0, dtype=q.dtype, device=gpu).transpose(1, 2)
    else:
        qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
        o = torch.full((B, Hq, Sq, 128), 7.0, dtype=q.dtype, device=gpu)
    lse = None
    if noalloc:
        lse = torch.full((B, Hq, Sq), 7.0, dtype=torch.float32, device=gpu)
        try:
            lib.fmha_fwd_noalloc(qg, kg, vg, o, lse, causal=causal, kv_valid_len=kvv)
        except lib.Mi355Error as e:   # more partial results than the static scratch holds: refused, nothing written
            assert "static scratch" in str(e)
            lse = None
    if lse is None:
        o, lse = lib.fmha_fwd(qg, kg, vg, causal=causal, kv_valid_len=kvv, out=o)
    torch.cuda.synchronize()
    err_o = float((o.float().cpu() - o_ref).abs().max())
    err_l = float((lse.cpu() - lse_ref).abs().max())
    assert err_o <= (1.6e-2 if bf16 else 2e-3) and err_l <= 1e-3, (err_o, err_l)


def test_generation_step_on_two_streams(lib, gpu):
    # the split-KV workspace is per stream: interleaved calls on two streams must not disturb each other
    qa, ka, va = (t.to(gpu) for t in so.fmha_inputs(1, 32, 8, 1, 4096, seed=1))
    qb, kb, vb = (t.to(gpu) for t in so.fmha_inputs(2, 16, 4, 1, 3000, seed=2))
    ref_a = lib.fmha_fwd(qa, ka, va)[0].clone()
    ref_b = lib.fmha_fwd(qb, kb, vb)[0].clone()
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    outs_a, outs_b = [], []
    for _ in range(5):
        with torch.cuda.stream(s1):
            outs_a.append(lib.fmha_fwd(qa, ka, va)[0])
        with torch.cuda.stream(s2):
            outs_b.append(lib.fmha_fwd(qb, kb, vb)[0])
    torch.cuda.synchronize()
    assert all(torch.equal(o, ref_a) for o in outs_a) and all(torch.equal(o, ref_b) for o in outs_b)


def test_split_kv_workspace_outlives_growth_under_a_captured_graph(lib, gpu):
    # A generation step is captured into a HIP graph; afterwards an eager call on the same stream needs a larger
    # workspace than the one the graph's kernels hold the address of. The library must keep the old buffer alive (it
    # only ever adds buffers), so replays of the graph still write valid memory and still give the eager result.
    qs, ks, vs = (t.to(gpu) for t in so.fmha_inputs(1, 32, 8, 1, 4096, seed=31))
    qb, kb, vb = (t.to(gpu) for t in so.fmha_inputs(8, 32, 1, 1, 16384, seed=32))     # 256 workgroups x 32 columns: 4.3 MB
    assert lib.fmha_workspace_bytes(8, 32, 1, 1, 16384) > (4 << 20) > lib.fmha_workspace_bytes(1, 32, 8, 1, 4096) > 0
    ref_s = lib.fmha_fwd(qs, ks, vs)[0].clone()
    ref_b = lib.fmha_fwd(qb, kb, vb)[0].clone()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    out_g = torch.zeros_like(qs)
    with torch.cuda.stream(side):
        lib.fmha_fwd(qs, ks, vs, return_lse=False, out=out_g)        # first use on this stream: allocates its 4 MiB buffer
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        lib.fmha_fwd(qs, ks, vs, return_lse=False, out=out_g)
    for rep in range(3):
        out_g.zero_()
        with torch.cuda.stream(side):
            big = lib.fmha_fwd(qb, kb, vb)[0]                        # eager, same stream, larger workspace
        side.synchronize()
        assert torch.equal(big, ref_b), rep
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, ref_s), rep
    del graph


def test_split_kv_call_that_would_allocate_during_capture_is_refused(lib, gpu):
    # A stream the library has never seen (created through the HIP runtime directly: torch hands out pooled streams) has
    # no workspace yet: the library must not allocate under capture; it reports an error and launches nothing. The same
    # capture then succeeds with a caller-owned workspace.
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    raw = ctypes.c_void_p()
    assert hip.hipStreamCreate(ctypes.byref(raw)) == 0
    fresh = torch.cuda.ExternalStream(raw.value)
    B, Hq, Hkv, Sk = 1, 32, 8, 2048
    q, k, v = (t.to(gpu) for t in so.fmha_inputs(B, Hq, Hkv, 1, Sk, seed=33))
    assert lib.fmha_workspace_bytes(B, Hq, Hkv, 1, Sk) > 0
    ref = lib.fmha_fwd(q, k, v)[0].clone()      # default stream (also sets the kernel attributes outside capture)
    ws = torch.empty(lib.fmha_workspace_bytes(B, Hq, Hkv, 1, Sk), dtype=torch.uint8, device=gpu)
    out_g = torch.zeros_like(q)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    refused = None
    with torch.cuda.graph(graph, stream=fresh):
        try:
            lib.fmha_fwd(q, k, v, return_lse=False, out=out_g)
        except lib.Mi355Error as e:
            refused = e
        lib.fmha_fwd(q, k, v, return_lse=False, out=out_g, workspace=ws)
    assert refused is not None and "capturing" in str(refused)
    for _ in range(2):
        out_g.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, ref)
    del graph


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_caller_owned_workspace_entry_point(lib, gpu, dtype):
    # mi355_fmha_fwd_ws: same kernels, partial results in the caller's memory; bit-identical to the library-owned path,
    # also when the workspace is larger than needed, holds garbage, and is reused by a smaller call
    for (B, Hq, Hkv, Sq, Sk, causal) in ((2, 32, 8, 1, 5000, False), (1, 8, 2, 3, 1200, True)):
        q, k, v = (t.to(gpu).to(dtype) for t in so.fmha_inputs(B, Hq, Hkv, Sq, Sk, seed=Sk))
        need = lib.fmha_workspace_bytes(B, Hq, Hkv, Sq, Sk)
        assert need > 0
        ws = torch.full((need + 4096,), 0xFF, dtype=torch.uint8, device=gpu)
        o_ref, l_ref = lib.fmha_fwd(q, k, v, causal=causal)
        o, l = lib.fmha_fwd(q, k, v, causal=causal, workspace=ws)
        torch.cuda.synchronize()
        assert torch.equal(o, o_ref) and torch.equal(l, l_ref)
        with pytest.raises(lib.Mi355Error, match="workspace"):
            lib.fmha_fwd(q, k, v, causal=causal, workspace=ws[:need - 16])
    # prefill shapes need no workspace at all
    q, k, v = (t.to(gpu).to(dtype) for t in so.fmha_inputs(1, 4, 2, 200, 200, seed=5))
    assert lib.fmha_workspace_bytes(1, 4, 2, 200, 200) == 0
    o = lib.fmha_fwd(q, k, v, causal=True, workspace=torch.empty(0, dtype=torch.uint8, device=gpu))[0]
    assert torch.equal(o, lib.fmha_fwd(q, k, v, causal=True)[0])


def test_caller_owned_workspace_serves_key_ranges_also_under_capture(lib, gpu):
    # a chunk against a long cache: the size query reports the partial outputs of the key ranges; with that much memory of
    # the caller's the call takes the ranges (bit-identical to the library-owned path) and never allocates, so it can be
    # captured on a stream the library has never seen; with less it walks all keys in one kernel instead of failing
    import ctypes
    B, Hq, Hkv, Sq, Sk = 1, 32, 8, 128, 8192
    q, k, v = (t.to(gpu) for t in so.fmha_inputs(B, Hq, Hkv, Sq, Sk, seed=8))
    need = lib.fmha_workspace_bytes(B, Hq, Hkv, Sq, Sk)
    assert need == 8 * B * Hq * Sq * (128 * 2 + 4)
    assert lib.fmha_workspace_bytes(1, 32, 8, 2048, 8192) == 0 and lib.fmha_workspace_bytes(1, 32, 8, 128, 1024) == 0
    assert lib.fmha_workspace_bytes(1, 32, 8, 512, 8192) == 4 * 32 * 512 * (128 * 2 + 4)      # 256-query items, 4 ranges
    ranges, lse_r = lib.fmha_fwd(q, k, v, causal=True)
    whole, lse_w = lib.fmha_fwd(q, k, v, causal=True, variant=1)
    ws = torch.full((need,), 0xFF, dtype=torch.uint8, device=gpu)
    o, lse = lib.fmha_fwd(q, k, v, causal=True, workspace=ws)
    assert torch.equal(o, ranges) and torch.equal(lse, lse_r)
    o, lse = lib.fmha_fwd(q, k, v, causal=True, workspace=ws[:need - 16])
    assert torch.equal(o, whole) and torch.equal(lse, lse_w)
    hip = ctypes.CDLL("libamdhip64.so")
    raw = ctypes.c_void_p()
    assert hip.hipStreamCreate(ctypes.byref(raw)) == 0
    fresh = torch.cuda.ExternalStream(raw.value)
    out_g = torch.zeros_like(q)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=fresh):
        lib.fmha_fwd(q, k, v, causal=True, return_lse=False, out=out_g, workspace=ws)
    for _ in range(2):
        out_g.zero_()
        ws.fill_(0x7F)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, ranges)
    del graph


# ---- operands read in place from other layouts ------------------------------------------------------------------------
@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,causal", [
    (2, 8, 2, 300, 300, True),      # prefill, 128-query workgroups
    (1, 32, 8, 2048, 2048, True),   # prefill, ping-pong workgroups
    (2, 8, 2, 1, 1500, False),      # generation step, split-KV kernels
])
def test_fused_qkv_projection_layout_read_in_place(lib, gpu, B, Hq, Hkv, Sq, Sk, causal):
    # q, k, v are slices of one [B, S, (Hq + 2 Hkv) * 128] projection (k, v of a longer cache when Sq < Sk); the output is
    # written as [B, Sq, Hq * 128]. Same numbers as the contiguous call on copies of the same values.
    q, k, v = so.fmha_inputs(B, Hq, Hkv, Sq, Sk, seed=11)
    W = (Hq + 2 * Hkv) * 128
    fused = torch.zeros((B, Sk, W), dtype=torch.float16)
    fused[:, :Sq, :Hq * 128] = q.transpose(1, 2).reshape(B, Sq, Hq * 128)
    fused[:, :, Hq * 128:(Hq + Hkv) * 128] = k.transpose(1, 2).reshape(B, Sk, Hkv * 128)
    fused[:, :, (Hq + Hkv) * 128:] = v.transpose(1, 2).reshape(B, Sk, Hkv * 128)
    fused = fused.to(gpu)
    qv = fused[:, :Sq, :Hq * 128].view(B, Sq, Hq, 128).transpose(1, 2)
    kv = fused[:, :, Hq * 128:(Hq + Hkv) * 128].view(B, Sk, Hkv, 128).transpose(1, 2)
    vv = fused[:, :, (Hq + Hkv) * 128:].view(B, Sk, Hkv, 128).transpose(1, 2)
    assert not qv.is_contiguous() and not kv.is_contiguous()
    out = torch.full((B, Sq, Hq * 128), float("nan"), dtype=torch.float16, device=gpu)
    o, lse = lib.fmha_fwd(qv, kv, vv, causal=causal, out=out.view(B, Sq, Hq, 128).transpose(1, 2))
    o_c, lse_c = lib.fmha_fwd(q.to(gpu), k.to(gpu), v.to(gpu), causal=causal)
    torch.cuda.synchronize()
    assert torch.equal(out.view(B, Sq, Hq, 128).transpose(1, 2), o_c) and torch.equal(lse, lse_c)
    o_ref, lse_ref = so.attention_ref(q, k, v, causal=causal)
    assert so.fmha_tolerance_ok(o_c.cpu(), lse_c.cpu(), o_ref, lse_ref)[0]


def test_broadcast_kv_head_with_zero_stride(lib, gpu):
    # a kv head stride of 0 shares one K/V head between all kv heads (what expand() produces)
    q, k, v = so.fmha_inputs(1, 4, 1, 200, 200, seed=3)
    o1, lse1 = lib.fmha_fwd(q.to(gpu), k.to(gpu), v.to(gpu), causal=True)
    ke, ve = k.to(gpu).expand(1, 4, 200, 128), v.to(gpu).expand(1, 4, 200, 128)
    o2, lse2 = lib.fmha_fwd(q.to(gpu), ke, ve, causal=True)
    torch.cuda.synchronize()
    assert torch.equal(o1, o2) and torch.equal(lse1, lse2)


def test_masked_keys_may_hold_garbage(lib, gpu):
    # keys at or beyond kv_valid_len must not influence the result, whatever they contain
    q, k, v = so.fmha_inputs(1, 2, 2, 90, 200, seed=11)
    k2, v2 = k.clone(), v.clone()
    k2[:, :, 150:] = float("nan")
    v2[:, :, 150:] = float("inf")
    o1, l1 = run(lib, gpu, q, k, v, False, 150)
    o2, l2 = run(lib, gpu, q, k2, v2, False, 150)
    assert torch.equal(o1, o2) and torch.equal(l1, l2)


def test_lse_pointer_is_optional(lib, gpu):
    q, k, v = (t.to(gpu) for t in so.fmha_inputs(1, 2, 1, 100, 100, seed=12))
    o1 = lib.fmha_fwd(q, k, v, causal=True, return_lse=False)
    o2, _ = lib.fmha_fwd(q, k, v, causal=True)
    assert torch.equal(o1, o2)


def test_reference_seeded_case_from_golden_fixture(lib, gpu):
    z = np.load(os.path.join(GOLDEN, "fmha_seed42_128.npz"))
    q, k, v = (torch.from_numpy(z[n]) for n in ("q", "k", "v"))
    rows = z["qrows"]
    for tag, causal in (("full", False), ("causal", True)):
        o, lse = run(lib, gpu, q, k, v, causal)
        assert np.abs(o.float().numpy()[:, :, rows] - z["o_" + tag]).max() <= 2e-3
        assert np.abs(lse.numpy() - z["lse_" + tag]).max() <= 1e-3


# ---- size-independent properties at the benchmark size --------------------------------------------------------------
def test_full_size_split_kv_merge_with_lse(lib, gpu):
    # attention over all keys == LSE-weighted merge of attention over two halves of the keys (non-causal)
    q, k, v = (t.to(gpu) for t in so.fmha_inputs(1, 32, 8, 4096, 4096, seed=42))
    o, lse = lib.fmha_fwd(q, k, v)
    o1, l1 = lib.fmha_fwd(q, k[:, :, :2048].contiguous(), v[:, :, :2048].contiguous())
    o2, l2 = lib.fmha_fwd(q, k[:, :, 2048:].contiguous(), v[:, :, 2048:].contiguous())
    lm = torch.logaddexp(l1, l2)
    merged = torch.exp(l1 - lm)[..., None] * o1.float() + torch.exp(l2 - lm)[..., None] * o2.float()
    assert (lm - lse).abs().max() <= 1e-3
    assert (merged - o.float()).abs().max() <= 3e-3  # two fp16 roundings of the halves
    # causal: rows of the last tile against kv_valid_len truncation of the non-causal kernel
    oc, lc = lib.fmha_fwd(q, k, v, causal=True)
    ot, lt = lib.fmha_fwd(q[:, :, 2047:2048].contiguous(), k, v, causal=False, kv_valid_len=2048)
    assert (oc[:, :, 2047:2048].float() - ot.float()).abs().max() <= 2e-3 and (lc[:, :, 2047:2048] - lt).abs().max() <= 1e-3


# ---- torch operator path ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("index", list(range(8)))
def test_torch_operator_every_index(gpu, index):
    import fmha_unified
    q, k, v = so.fmha_inputs(1, 8, 2, 200, 200, seed=index)
    o = fmha_unified.ops.fine_fmha(q.to(gpu), k.to(gpu), v.to(gpu), True, False, index)
    assert o.dtype == torch.float16 and o.shape == q.shape
    ok, st = so.fmha_tolerance_ok(o, None, so.fine_fmha_ref(q, k, v, True, False), None)
    assert ok, (index, st)


def test_torch_operator_decode_and_lse(gpu):
    import fmha_unified
    q, k, v = so.fmha_inputs(2, 8, 2, 1, 301, seed=3)
    o = fmha_unified.ops.fine_fmha(q.to(gpu), k.to(gpu), v.to(gpu), False, True, 2)
    ok, st = so.fmha_tolerance_ok(o, None, so.fine_fmha_ref(q, k, v, False, True), None)
    assert ok, st
    o2, lse = fmha_unified.ops.fine_fmha_with_lse(q.to(gpu), k.to(gpu), v.to(gpu), False)
    o_ref, lse_ref = so.attention_ref(q, k, v)
    ok, st = so.fmha_tolerance_ok(o2, lse, o_ref, lse_ref)
    assert ok, st


def test_torch_operator_accepts_reference_style_padded_call(gpu):
    # the reference's ops.py pads q, k, v to a multiple of 64 and passes the un-padded key count as decode_length;
    # calling the operator that way must give the un-padded result in the first Sq rows
    import torch.nn.functional as F
    import fmha_unified  # noqa: F401
    q, k, v = so.fmha_inputs(1, 4, 1, 100, 100, seed=4)
    pad = lambda t: F.pad(t, (0, 0, 0, 28)).contiguous().to(gpu)
    o = torch.ops.fmha_unified.finefmha_2.default(pad(q), pad(k), pad(v), True, False, 100)[:, :, :100]
    ok, st = so.fmha_tolerance_ok(o, None, so.fine_fmha_ref(q, k, v, True, False), None)
    assert ok, st


def test_torch_operator_reads_transposed_views_in_place(gpu):
    # the in-model call of the reference: [B, S, H, D] projections viewed as [B, H, S, D]
    # (benchmarks/flashattn-cuda/modeling_llama.py:658-660), read where they lie; the result is a contiguous [B, H, S, D]
    # tensor like the reference's (semi/fmha_2_amd.cpp:336), so a caller may .view() it
    import fmha_unified
    B, S, Hq, Hkv = 2, 384, 8, 2
    q, k, v = so.fmha_inputs(B, Hq, Hkv, S, S, seed=21)
    qp = q.transpose(1, 2).contiguous().to(gpu)   # [B, S, H, D]
    kp = k.transpose(1, 2).contiguous().to(gpu)
    vp = v.transpose(1, 2).contiguous().to(gpu)
    out = fmha_unified.ops.fine_fmha(qp.transpose(1, 2), kp.transpose(1, 2), vp.transpose(1, 2), causal=True,
                                     is_decode=False, kernel_index=5)
    assert out.shape == (B, Hq, S, 128) and out.is_contiguous()
    assert out.view(B * Hq, S * 128).shape == (B * Hq, S * 128)
    o_ref, _ = so.attention_ref(q, k, v, causal=True)
    assert (out.cpu().float() - o_ref).abs().max() <= 2e-3
    # a view the kernel cannot read in place (last dimension strided) is copied, as the reference does
    q2 = torch.empty((B, Hq, S, 256), dtype=torch.float16, device=gpu)[..., ::2]
    q2.copy_(q.to(gpu))
    out2 = fmha_unified.ops.fine_fmha(q2, k.to(gpu), v.to(gpu), True, False, 2)
    assert (out2.cpu().float() - o_ref).abs().max() <= 2e-3


# ---- bfloat16 -----------------------------------------------------------------------------------------------------------
# Tolerance for bfloat16 outputs (8 significand bits; the fp16 bound of 2e-3 is below half a bf16 ulp of values near 1):
# max|O - O_ref| <= 1.6e-2 against fp32 attention over the same bf16-rounded inputs; LSE (fp32 from fp32 scores) keeps 1e-3.
# ---- a chunk of queries against a long cache: keys cut into ranges, merged by a second kernel --------------------
@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,causal,kvv", [
    (1, 32, 8, 128, 8192, True, None),     # 8 ranges of 1024 keys
    (1, 32, 8, 64, 8192, True, 8000),      # half-filled q tile, last range shorter
    (1, 16, 4, 300, 4500, True, 4097),     # 3 q tiles, ranges that are no multiple of the tile, one valid key in the last
    (2, 8, 2, 200, 5000, False, None),     # 4 ranges of 1280 keys
    (1, 32, 8, 512, 8192, False, 5000),    # 128 items: two ranges
    (3, 4, 1, 100, 4096, True, None),
    (1, 4, 4, 4096, 4096, True, None),     # causal square: the second range is invisible to the early q tiles
    (1, 8, 1, 5, 12000, True, 11000),      # 40 query rows per kv head: more than the generation-step kernels take
    (1, 32, 8, 512, 8192, True, None),     # 256-query items over 4 ranges
    (1, 32, 8, 1024, 4500, False, 4200),   # 256-query items over 2 ranges of 2112 keys
    (1, 64, 8, 480, 9000, True, 8200),     # 256-query items, second q tile ragged
    (2, 16, 4, 256, 6200, True, 6150),     # too few 256-query items for the machine: 128-query items over 4 ranges
])
def test_chunk_against_long_cache_key_ranges(lib, gpu, B, Hq, Hkv, Sq, Sk, causal, kvv):
    q, k, v = so.fmha_inputs(B, Hq, Hkv, Sq, Sk, seed=Sq + Sk + Hq)
    o, lse = check(lib, gpu, q, k, v, causal, kvv, variant=3)     # variant 3: key ranges, or an error where they do not apply
    if kvv is not None:     # keys past the valid length may hold anything
        k, v = k.clone(), v.clone()
        k[:, :, kvv:] = float("nan")
        v[:, :, kvv:] = float("inf")
        o_p, lse_p = run(lib, gpu, q, k, v, causal, kvv, variant=3)
        assert torch.equal(o, o_p) and torch.equal(lse, lse_p)
    o0, lse0 = run(lib, gpu, q, k, v, causal, kvv)                # the choice by shape takes the same path
    assert torch.equal(o, o0) and torch.equal(lse, lse0)
    o1, lse1 = run(lib, gpu, q, k, v, causal, kvv, variant=1)     # the same kernel over all keys at once
    assert (o.float() - o1.float()).abs().max() <= 2e-3 and (lse - lse1).abs().max() <= 1e-3


def test_key_ranges_with_query_rows_that_see_no_key(lib, gpu):
    # causal with more queries than keys: the first Sq - Sk rows see nothing (O = 0, LSE = -inf), also after the merge
    B, Hq, Hkv, Sq, Sk = 1, 2, 1, 5000, 4100
    q, k, v = (t.to(gpu) for t in so.fmha_inputs(B, Hq, Hkv, Sq, Sk, seed=12))
    o1, l1 = lib.fmha_fwd(q, k, v, causal=True, variant=1)
    o3, l3 = lib.fmha_fwd(q, k, v, causal=True, variant=3)
    torch.cuda.synchronize()
    empty = torch.isinf(l1)
    assert int(empty.sum()) == B * Hq * (Sq - Sk) and torch.equal(empty, torch.isinf(l3)) and bool((l3[empty] < 0).all())
    assert bool((o3[empty] == 0).all())
    assert (o1.float() - o3.float()).abs().max() <= 2e-3 and (l1[~empty] - l3[~empty]).abs().max() <= 1e-3


def test_key_ranges_only_where_they_pay(lib, gpu):
    # enough work items for the machine, a short cache, or a generation step: no ranges (variant 3 reports it)
    for B, Hq, Hkv, Sq, Sk in ((1, 32, 8, 2048, 8192), (1, 32, 8, 128, 1024), (1, 32, 8, 512, 2048)):
        q, k, v = (t.to(gpu) for t in so.fmha_inputs(B, Hq, Hkv, Sq, Sk, seed=3))
        with pytest.raises(lib.Mi355Error):
            lib.fmha_fwd(q, k, v, causal=True, variant=3)


def test_key_ranges_bfloat16_and_transposed_views(lib, gpu):
    B, Hq, Hkv, Sq, Sk = 2, 8, 2, 150, 6000
    q, k, v = so.fmha_inputs(B, Hq, Hkv, Sq, Sk, seed=77)
    qb, kb, vb = q.float().bfloat16(), k.float().bfloat16(), v.float().bfloat16()
    o, lse = lib.fmha_fwd(qb.to(gpu), kb.to(gpu), vb.to(gpu), causal=True, kv_valid_len=5555)
    o_ref, lse_ref = so.attention_ref(qb, kb, vb, causal=True, kv_valid_len=5555)
    assert (o.float().cpu() - o_ref).abs().max() <= 1.6e-2 and (lse.cpu() - lse_ref).abs().max() <= 1e-3
    q2, k2, v2 = (t.float().bfloat16() for t in so.fmha_inputs(1, 32, 8, 512, 8192, seed=78))      # 256-query items
    o, lse = lib.fmha_fwd(q2.to(gpu), k2.to(gpu), v2.to(gpu), causal=True)
    o_ref, lse_ref = so.attention_ref(q2, k2, v2, causal=True)
    assert (o.float().cpu() - o_ref).abs().max() <= 1.6e-2 and (lse.cpu() - lse_ref).abs().max() <= 1e-3
    # [B, S, H, D] storage viewed as [B, H, S, D]: inputs and output
    qt = q.transpose(1, 2).contiguous().to(gpu).transpose(1, 2)
    kt = k.transpose(1, 2).contiguous().to(gpu).transpose(1, 2)
    vt = v.transpose(1, 2).contiguous().to(gpu).transpose(1, 2)
    out = torch.full((B, Sq, Hq, 128), 7.0, dtype=torch.float16, device=gpu).transpose(1, 2)
    lib.fmha_fwd(qt, kt, vt, causal=True, return_lse=False, out=out)
    o_ref, _ = so.attention_ref(q, k, v, causal=True)
    assert (out.float().cpu() - o_ref).abs().max() <= 2e-3


def test_key_ranges_workspace_per_stream_growing_and_reused(lib, gpu):
    # one workspace per stream, replaced by a larger one when a call needs more; results are reproducible bit for bit
    small = [t.to(gpu) for t in so.fmha_inputs(1, 8, 2, 128, 4096, seed=5)]        # 4 MB of partial results
    large = [t.to(gpu) for t in so.fmha_inputs(1, 32, 8, 512, 8192, seed=6)]       # 17 MB
    ref_s = lib.fmha_fwd(*small, causal=True)
    ref_l = lib.fmha_fwd(*large, causal=True)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    got = []
    for _ in range(3):
        with torch.cuda.stream(s1):
            got.append((lib.fmha_fwd(*small, causal=True), ref_s))
            got.append((lib.fmha_fwd(*large, causal=True), ref_l))
        with torch.cuda.stream(s2):
            got.append((lib.fmha_fwd(*large, causal=True), ref_l))
            got.append((lib.fmha_fwd(*small, causal=True), ref_s))
    torch.cuda.synchronize()
    for (o, lse), (o_ref, lse_ref) in got:
        assert torch.equal(o, o_ref) and torch.equal(lse, lse_ref)


def test_key_ranges_fall_back_to_one_walk_when_capture_forbids_allocation(lib, gpu):
    # A stream the library has never seen has no workspace for the partial results; under capture none may be allocated,
    # so the call runs the kernel over all keys at once (same result as that variant, bit for bit) instead of failing.
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    raw = ctypes.c_void_p()
    assert hip.hipStreamCreate(ctypes.byref(raw)) == 0
    fresh = torch.cuda.ExternalStream(raw.value)
    q, k, v = (t.to(gpu) for t in so.fmha_inputs(1, 32, 8, 128, 4096, seed=41))
    ranges = lib.fmha_fwd(q, k, v, causal=True)[0].clone()
    whole = lib.fmha_fwd(q, k, v, causal=True, variant=1)[0].clone()
    out_g = torch.zeros_like(q)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=fresh):
        lib.fmha_fwd(q, k, v, causal=True, return_lse=False, out=out_g)
    for _ in range(2):
        out_g.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, whole)
    del graph
    # with a workspace in place (first eager call on the stream) a capture records the ranges and the merge
    with torch.cuda.stream(fresh):
        lib.fmha_fwd(q, k, v, causal=True, return_lse=False, out=out_g)
    fresh.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=fresh):
        lib.fmha_fwd(q, k, v, causal=True, return_lse=False, out=out_g)
    for _ in range(2):
        out_g.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, ranges)
    del graph


def bf16_inputs(B, Hq, Hkv, Sq, Sk, seed):
    q, k, v = so.fmha_inputs(B, Hq, Hkv, Sq, Sk, seed=seed)
    return q.float().bfloat16(), k.float().bfloat16(), v.float().bfloat16()


@pytest.mark.parametrize("B,Hq,Hkv,Sq,Sk,causal,kvv", [
    (1, 4, 1, 128, 128, True, None),      # the seeded shape of the reference's correct.py
    (2, 8, 2, 300, 333, True, 320),       # ragged, 128-query workgroups
    (1, 32, 8, 2048, 2048, True, None),   # ping-pong workgroups
    (4, 32, 32, 1024, 1024, False, None),  # configuration F3 in bf16
    (2, 8, 2, 1, 3000, False, 2900),      # generation step, split-KV kernels
    (1, 16, 2, 3, 700, True, None),
])
def test_bfloat16_attention(lib, gpu, B, Hq, Hkv, Sq, Sk, causal, kvv):
    q, k, v = bf16_inputs(B, Hq, Hkv, Sq, Sk, seed=Sq + Sk)
    o, lse = lib.fmha_fwd(q.to(gpu), k.to(gpu), v.to(gpu), causal=causal, kv_valid_len=kvv)
    assert o.dtype == torch.bfloat16 and lse.dtype == torch.float32
    o_ref, lse_ref = so.attention_ref(q, k, v, causal=causal, kv_valid_len=kvv)
    assert (o.float().cpu() - o_ref).abs().max() <= 1.6e-2
    assert (lse.cpu() - lse_ref).abs().max() <= 1e-3


def test_bfloat16_closed_forms(lib, gpu):
    # first causal row returns V[0] exactly; V = ones returns ones exactly (both representable in bf16)
    q, k, v = bf16_inputs(1, 4, 2, 200, 200, seed=9)
    o, _ = lib.fmha_fwd(q.to(gpu), k.to(gpu), v.to(gpu), causal=True)
    assert torch.equal(o[:, :, 0].cpu(), v.repeat_interleave(2, 1)[:, :, 0])
    o1, _ = lib.fmha_fwd(q.to(gpu), k.to(gpu), torch.ones_like(v).to(gpu), causal=False)
    assert (o1.float().cpu() - 1).abs().max() <= 2.0 ** -8


def test_torch_operator_bfloat16_and_mixed_dtype_rejection(gpu):
    import fmha_unified
    q, k, v = bf16_inputs(1, 8, 2, 256, 256, seed=4)
    out = fmha_unified.ops.fine_fmha(q.to(gpu), k.to(gpu), v.to(gpu), causal=True, is_decode=False, kernel_index=5)
    o_ref, _ = so.attention_ref(q, k, v, causal=True)
    assert out.dtype == torch.bfloat16 and (out.float().cpu() - o_ref).abs().max() <= 1.6e-2
    with pytest.raises(RuntimeError, match="dtype"):
        fmha_unified.ops.fine_fmha(q.to(gpu), k.half().to(gpu), v.to(gpu), True, False, 5)

"""GPU parity of the layer glue kernels (RMSNorm, fused residual add + RMSNorm, RoPE, SiLU*up) through the C ABI, and
of the decoder layer built from them (llama_layer.FineLlamaDecoderLayer) against the CPU oracle.

Tolerances (floating point, fp16 outputs of fp32 arithmetic): a glue kernel rounds once, so
|out - ref| <= 2^-10 |ref| + 1e-6 against the fp32 oracle; the layer is compared with the oracle that rounds every
stored intermediate to fp16 like the kernel chain does: relative Frobenius error <= 2e-3 and max |err| <= 2e-2 max|ref|."""
import pytest
import torch

import serving_oracle as so

pytestmark = pytest.mark.gpu


def close_one_rounding(out, ref):
    err = (out.float().cpu() - ref).abs()
    return bool((err <= 2.0 ** -10 * ref.abs() + 1e-6).all()), float(err.max())


@pytest.mark.parametrize("rows,hidden", [(1, 8), (7, 4096), (300, 512), (16, 8192), (5, 12288), (3, 1000)])
def test_rmsnorm(lib, gpu, rows, hidden):
    x = so.randn_fp16((rows, hidden), 1, 2.0)
    w = (1 + 0.1 * so.randn_fp16((hidden,), 2).float()).half()
    ref, _ = so.rmsnorm_ref(x, w, 1e-5)
    out = lib.rmsnorm(x.to(gpu), w.to(gpu), 1e-5)
    assert close_one_rounding(out, ref)[0]
    # closed form: a constant row normalises to sign * weight
    c = torch.full((2, hidden), -3.0, dtype=torch.float16)
    outc = lib.rmsnorm(c.to(gpu), w.to(gpu), 0.0)
    assert close_one_rounding(outc, -w.float().expand(2, hidden))[0]


def test_rmsnorm_with_residual_strides_and_in_place(lib, gpu):
    rows, hidden = 33, 1024
    x = so.randn_fp16((rows, hidden), 3)
    r = so.randn_fp16((rows, hidden), 4, 3.0)
    w = so.randn_fp16((hidden,), 5)
    ref, h_ref = so.rmsnorm_ref(x, w, 1e-6, residual=r)
    # x is a column slice of a wider buffer; the residual is updated in place
    wide = torch.zeros((rows, 3 * hidden), dtype=torch.float16, device=gpu)
    wide[:, hidden:2 * hidden] = x.to(gpu)
    rg = r.to(gpu)
    out, h = lib.rmsnorm(wide[:, hidden:2 * hidden], w.to(gpu), 1e-6, residual=rg, residual_out=rg)
    assert h.data_ptr() == rg.data_ptr() and torch.equal(h.cpu().float(), h_ref)   # the fp16 sum is exact
    assert close_one_rounding(out, ref)[0]
    # out of place: the residual input is left alone
    rg2 = r.to(gpu)
    out2, h2 = lib.rmsnorm(x.to(gpu), w.to(gpu), 1e-6, residual=rg2)
    assert torch.equal(rg2.cpu(), r) and torch.equal(h2, h) and torch.equal(out2, out)


@pytest.mark.parametrize("B,S,heads", [(1, 1, 1), (2, 37, 10), (1, 300, 40), (3, 5, 33)])
def test_rope_in_place_and_into_a_cache(lib, gpu, B, S, heads):
    cos, sin = so.rope_tables(512, 128, 10000.0)
    g = torch.Generator().manual_seed(7)
    pos = torch.randint(0, 512, (B, S), generator=g, dtype=torch.int32)
    x = so.randn_fp16((B, S, heads + 3, 128), 8)           # the last 3 heads must stay untouched
    ref = so.rope_ref(x[:, :, :heads].transpose(1, 2), cos, sin, pos).transpose(1, 2)
    xg = x.to(gpu)
    lib.rope(xg[:, :, :heads], cos.to(gpu), sin.to(gpu), pos.to(gpu))
    assert close_one_rounding(xg[:, :, :heads], ref)[0]
    assert torch.equal(xg[:, :, heads:].cpu(), x[:, :, heads:])
    # position 0 is the identity, bit for bit
    x0 = x.to(gpu)
    lib.rope(x0[:, :, :heads], cos.to(gpu), sin.to(gpu), torch.zeros((B, S), dtype=torch.int32, device=gpu))
    assert torch.equal(x0.cpu(), x)
    # out of place into rows [4, 4 + S) of a longer token-major cache
    cache = torch.zeros((B, S + 9, heads, 128), dtype=torch.float16, device=gpu)
    src = x.to(gpu)
    lib.rope(src[:, :, :heads], cos.to(gpu), sin.to(gpu), pos.to(gpu), out=cache[:, 4:4 + S])
    assert torch.equal(cache[:, 4:4 + S], xg[:, :, :heads]) and torch.equal(src.cpu(), x)
    assert float(cache[:, :4].abs().max()) == 0.0 and float(cache[:, 4 + S:].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,S,n_q,n_kv,shared_positions", [(2, 5, 4, 1, True), (8, 1, 32, 8, True), (1, 37, 32, 8, False),
                                                           (3, 2, 40, 5, False)])
def test_rope_qkv_equals_the_two_rope_calls_it_replaces(lib, gpu, dtype, B, S, n_q, n_kv, shared_positions):
    # q in place, k rotated + v copied into a cache tensor: one launch, bit-identical to mi355_rope on the q heads followed by
    # mi355_rope(copy_heads = n_kv) on the k and v heads (itself checked against the oracle above); everything around the new
    # rows of the cache, and the k / v heads of the projection, stay untouched
    cos, sin = so.rope_tables(128, 128, 10000.0)
    cos, sin = cos.to(gpu), sin.to(gpu)
    qkv = so.randn_fp16((B, S, n_q + 2 * n_kv, 128), 5).to(gpu).to(dtype)
    if shared_positions:
        pos = (torch.arange(S, dtype=torch.int32) + 60).to(gpu)
    else:
        pos = ((torch.arange(B * S, dtype=torch.int32) * 7) % 128).reshape(B, S).to(gpu)
    past, max_len = 11, 11 + S + 3
    cache_a = torch.full((B, max_len, 2 * n_kv, 128), 3.0, dtype=dtype, device=gpu)
    cache_b = cache_a.clone()
    two = qkv.clone()
    lib.rope(two[:, :, :n_q], cos, sin, pos)
    lib.rope(two[:, :, n_q:], cos, sin, pos, out=cache_a[:, past:past + S], copy_heads=n_kv)
    one = qkv.clone()
    lib.rope_qkv(one, cache_b[:, past:past + S], cos, sin, pos, n_q, n_kv)
    assert torch.equal(one, two) and torch.equal(cache_a, cache_b)
    assert torch.equal(one[:, :, n_q:], qkv[:, :, n_q:]) and not torch.equal(one[:, :, :n_q], qkv[:, :, :n_q])
    assert bool((cache_b[:, :past] == 3.0).all()) and bool((cache_b[:, past + S:] == 3.0).all())
    assert torch.equal(cache_b[:, past:past + S, n_kv:], qkv[:, :, n_q + n_kv:])
    # the same rows into a head-major cache [B, 2 n_kv, max_len, 128]
    cache_h = torch.full((B, 2 * n_kv, max_len, 128), 3.0, dtype=dtype, device=gpu)
    one_h = qkv.clone()
    lib.rope_qkv(one_h, cache_h[:, :, past:past + S].transpose(1, 2), cos, sin, pos, n_q, n_kv)
    assert torch.equal(one_h, two) and torch.equal(cache_h.transpose(1, 2), cache_a)


def test_rope_copies_value_heads_and_shares_one_position_table(lib, gpu):
    # k heads rotated and v heads copied into a fused K|V cache row by one launch; one [S] position table for all batch rows
    B, S, n_kv = 3, 17, 5
    cos, sin = so.rope_tables(64, 128, 10000.0)
    pos = torch.arange(20, 20 + S, dtype=torch.int32)
    kv = so.randn_fp16((B, S, 2 * n_kv, 128), 12)
    ref_k = so.rope_ref(kv[:, :, :n_kv].transpose(1, 2), cos, sin, pos[None].expand(B, S)).transpose(1, 2)
    cache = torch.zeros((B, 40, 2 * n_kv, 128), dtype=torch.float16, device=gpu)
    lib.rope(kv.to(gpu), cos.to(gpu), sin.to(gpu), pos.to(gpu), out=cache[:, 20:20 + S], copy_heads=n_kv)
    assert close_one_rounding(cache[:, 20:20 + S, :n_kv], ref_k)[0]
    assert torch.equal(cache[:, 20:20 + S, n_kv:].cpu(), kv[:, :, n_kv:])
    assert float(cache[:, :20].abs().max()) == 0.0 and float(cache[:, 20 + S:].abs().max()) == 0.0


@pytest.mark.parametrize("rows,inter", [(1, 8), (9, 14336), (70000, 16), (257, 1000)])
def test_silu_mul(lib, gpu, rows, inter):
    gu = so.randn_fp16((rows, 2 * inter), 9, 3.0)
    out = lib.silu_mul(gu.to(gpu))
    ok, worst = close_one_rounding(out, so.silu_mul_ref(gu))
    assert ok, worst
    edge = torch.tensor([[0.0, 30.0, -30.0, 1.0, 0, 0, 0, 0, 3.0, 2.0, 5.0, -4.0, 0, 0, 0, 0]], dtype=torch.float16)
    oe = lib.silu_mul(edge.to(gpu)).cpu().float()[0]
    assert oe[0] == 0.0 and oe[1] == 60.0 and abs(oe[2]) < 1e-6 and abs(oe[3] + 4 * 0.7310586) < 4e-3


@pytest.mark.parametrize("M,F,K,layout", [(256, 256, 128, "NT"), (2048, 4096, 512, "NT"), (1024, 14336, 256, "NT"),
                                          (384, 192, 64, "NT"), (512, 1024, 256, "NN"), (8, 512, 256, "NT"), (100, 96, 72, "NT"),
                                          (300, 160, 128, "NT"), (1000, 14336, 128, "NT"), (4100, 4096, 64, "NN"),
                                          (32, 14336, 256, "NT"), (64, 14336, 128, "NN"), (24, 7168, 512, "NT"),
                                          (1, 32, 64, "NT"), (8, 14336, 512, "NT"), (16, 2048, 1024, "NT"), (13, 96, 128, "NT"),
                                          (9, 4096, 4096, "NT"), (16, 14336, 4096, "NT"), (8, 7168, 4096, "NT"), (4, 3072, 4096, "NT"),
                                          (16, 512, 256, "NN"), (17, 1024, 512, "NT"), (48, 7168, 256, "NT"),
                                          (33, 512, 1024, "NN"), (64, 2048, 128, "NN"), (40, 96, 64, "NT"), (5, 256, 192, "NN")])
def test_gemm_with_gate_up_epilogue(lib, gpu, M, F, K, layout):
    # silu(x Wg^T) * (x Wu^T) from one launch on the interleaved weight (tiled shapes; up to 16 rows in layout NT on the
    # split-K kernel, with and without the second half of the A slab; up to 64 rows otherwise on the 64x64 deep-ring tiles)
    # or, where K is off the tiles' multiple, from the two-step fallback;
    # compared with the fp32 oracle. One rounding of an fp32 value: |err| <= 2^-10 |ref| + the GEMM's accumulation slack.
    x = so.randn_fp16((M, K), 1)
    wg, wu = so.randn_fp16((F, K), 2, 0.05), so.randn_fp16((F, K), 3, 0.05)
    ref = so.silu_mul_ref(torch.cat((so.gemm_ref(x, wg, "NT"), so.gemm_ref(x, wu, "NT")), 1))
    if layout == "NT":
        w = lib.interleave_gate_up(wg.to(gpu), wu.to(gpu), dim=0)
        assert w.shape == (2 * F, K) and torch.equal(w[:32].cpu(), wg[:32]) and torch.equal(w[32:64].cpu(), wu[:32])
    else:
        w = lib.interleave_gate_up(wg.t().contiguous().to(gpu), wu.t().contiguous().to(gpu), dim=1)
        assert w.shape == (K, 2 * F) and torch.equal(w[:, 32:64].cpu(), wu[:32].t())
    out = lib.hgemm_silu_mul(x.to(gpu), w, layout)
    err = (out.float().cpu() - ref).abs()
    assert bool((err <= 2.0 ** -10 * ref.abs() + 1e-3).all()), float(err.max())
    # the interleaved silu_mul on the plain product gives the same numbers up to the extra fp16 rounding of the product
    two_step = lib.silu_mul(lib.hgemm(x.to(gpu), w, layout), interleave=32)
    assert (two_step.float() - out.float()).abs().max() <= 2e-2 * ref.abs().max()


def test_gate_up_epilogue_is_one_launch_for_every_row_count(lib, gpu):
    # N a multiple of 32 and K a multiple of 64: the entry point itself never answers "unsupported", whatever M is
    K, F = 256, 512
    wg, wu = so.randn_fp16((F, K), 2, 0.05), so.randn_fp16((F, K), 3, 0.05)
    w = lib.interleave_gate_up(wg.to(gpu), wu.to(gpu), dim=0)
    for M in (1, 8, 16, 17, 31, 32, 33, 63, 64, 65, 100, 128, 300):
        x = so.randn_fp16((M, K), 10 + M)
        out = torch.empty((M, F), dtype=torch.float16, device=gpu)
        xg = x.to(gpu)
        rc = lib.load().mi355_hgemm_silu_mul(xg.data_ptr(), w.data_ptr(), out.data_ptr(), M, F, K, K, K, F, lib.GEMM_NT, 0)
        assert rc == 0, (M, rc)
        torch.cuda.synchronize()
        ref = so.silu_mul_ref(torch.cat((so.gemm_ref(x, wg, "NT"), so.gemm_ref(x, wu, "NT")), 1))
        err = (out.float().cpu() - ref).abs()
        assert bool((err <= 2.0 ** -10 * ref.abs() + 1e-3).all()), (M, float(err.max()))


def test_gate_up_single_row_activation_with_arbitrary_row_stride(lib, gpu):
    # torch calls a [1, K] tensor contiguous whatever its stride(0): the wrapper passes the logical leading dimension
    K, F = 256, 128
    x = so.randn_fp16((1, K), 4)
    wg, wu = so.randn_fp16((F, K), 5, 0.05), so.randn_fp16((F, K), 6, 0.05)
    w = lib.interleave_gate_up(wg.to(gpu), wu.to(gpu), dim=0)
    ref = so.silu_mul_ref(torch.cat((so.gemm_ref(x, wg, "NT"), so.gemm_ref(x, wu, "NT")), 1))
    base = torch.zeros(4 * K, dtype=torch.float16, device=gpu)
    base[:K] = x[0].to(gpu)
    for stride0 in (7, 0, 3 * K):
        x1 = base.as_strided((1, K), (stride0, 1))
        assert x1.is_contiguous() and x1.stride(0) == stride0
        out = lib.hgemm_silu_mul(x1, w, "NT")
        err = (out.float().cpu() - ref).abs()
        assert bool((err <= 2.0 ** -10 * ref.abs() + 1e-3).all()), (stride0, float(err.max()))


def layer_weights(H, n_q, n_kv, F, seed=0):
    D = 128
    g = lambda shape, s, std: so.randn_fp16(shape, seed + s, std)
    w = dict(q=g((n_q * D, H), 1, 0.03), k=g((n_kv * D, H), 2, 0.03), v=g((n_kv * D, H), 3, 0.03), o=g((H, n_q * D), 4, 0.03),
             gate=g((F, H), 5, 0.03), up=g((F, H), 6, 0.03), down=g((H, F), 7, 0.03))
    w["ln1"] = (1 + 0.1 * g((H,), 8, 1.0).float()).half()
    w["ln2"] = (1 + 0.1 * g((H,), 9, 1.0).float()).half()
    return w


def layer_close(out, ref):
    out, ref = out.float().cpu(), ref.float()
    rel = float((out - ref).norm() / ref.norm())
    worst = float((out - ref).abs().max() / ref.abs().max())
    return rel <= 2e-3 and worst <= 2e-2, (rel, worst)


@pytest.mark.parametrize("B,S,H,n_q,n_kv,F", [(2, 100, 512, 4, 2, 1024), (1, 700, 1024, 8, 2, 2816), (3, 1, 512, 4, 4, 1024)])
def test_decoder_layer_prefill(lib, gpu, B, S, H, n_q, n_kv, F):
    from llama_layer import FineLlamaDecoderLayer
    w = layer_weights(H, n_q, n_kv, F)
    x = so.randn_fp16((B, S, H), 42)
    pos = torch.arange(S, dtype=torch.int32)[None].expand(B, S)
    layer = FineLlamaDecoderLayer({k: v.to(gpu) for k, v in w.items()}, n_q, n_kv, rms_eps=1e-5, max_positions=1024)
    xg = x.to(gpu)
    out = layer(xg, pos.to(gpu))
    torch.cuda.synchronize()
    assert torch.equal(xg.cpu(), x)  # the input is not modified
    ref, _, _ = so.llama_decoder_layer_ref(x, w, pos, n_q, n_kv, eps=1e-5)
    ok, st = layer_close(out, ref)
    assert ok, st


def test_decoder_layer_generation_steps_with_cache(lib, gpu):
    from llama_layer import FineKVCache, FineLlamaDecoderLayer
    B, S0, H, n_q, n_kv, F, steps = 2, 600, 512, 8, 2, 1024, 3
    w = layer_weights(H, n_q, n_kv, F, seed=20)
    layer = FineLlamaDecoderLayer({k: v.to(gpu) for k, v in w.items()}, n_q, n_kv, max_positions=1024)
    cache = FineKVCache(B, S0 + steps, n_kv, device=gpu)
    x = so.randn_fp16((B, S0, H), 1)
    out = layer(x.to(gpu), kv_cache=cache, time_attention=True)
    ref, k_ref, v_ref = so.llama_decoder_layer_ref(x, w, torch.arange(S0)[None].expand(B, S0), n_q, n_kv)
    assert layer_close(out, ref)[0] and cache.length == S0
    for t in range(steps):
        xt = so.randn_fp16((B, 1, H), 100 + t)
        out = layer(xt.to(gpu), kv_cache=cache, time_attention=True)   # 8 query rows per kv head, 600+ keys: split-KV kernels
        ref, k_ref, v_ref = so.llama_decoder_layer_ref(xt, w, torch.full((B, 1), S0 + t), n_q, n_kv, past_k=k_ref, past_v=v_ref)
        ok, st = layer_close(out, ref)
        assert ok, (t, st)
    assert cache.length == S0 + steps and len(layer.attn_ms["prefill"]) == 1 and len(layer.attn_ms["decode"]) == steps
    # the cache holds the rotated keys and the values the oracle holds
    assert (cache.k.transpose(1, 2).float().cpu() - k_ref).abs().max() <= 2e-2
    assert (cache.v.transpose(1, 2).float().cpu() - v_ref).abs().max() <= 2e-2
    with pytest.raises(ValueError):
        layer(xt.to(gpu), kv_cache=cache)


def test_decoder_layer_from_transformers_weights(lib, gpu):
    # weights taken from a transformers LlamaDecoderLayer; compared with that layer run in fp32 on the CPU
    pytest.importorskip("transformers")
    from transformers import LlamaConfig
    from transformers.models.llama import modeling_llama as hf
    from llama_layer import FineLlamaDecoderLayer
    cfg = LlamaConfig(hidden_size=512, num_attention_heads=4, num_key_value_heads=2, head_dim=128, intermediate_size=1024,
                      rms_norm_eps=1e-5, rope_theta=10000.0, vocab_size=32, num_hidden_layers=1)
    cfg._attn_implementation = "eager"
    torch.manual_seed(1)
    ref_layer = hf.LlamaDecoderLayer(cfg, 0).float().eval()
    for p in ref_layer.parameters():
        torch.nn.init.normal_(p, std=0.03)
    ref_layer.input_layernorm.weight.data = 1 + 0.1 * torch.randn(512)
    ref_layer.post_attention_layernorm.weight.data = 1 + 0.1 * torch.randn(512)
    for p in ref_layer.parameters():   # the values an fp16 checkpoint would hold
        p.data = p.data.half().float()
    B, S = 2, 130
    x = so.randn_fp16((B, S, 512), 3)
    pos = torch.arange(S)[None].expand(B, S)
    cos, sin = hf.LlamaRotaryEmbedding(cfg)(x.float(), pos)
    mask = torch.full((S, S), float("-inf")).triu(1)[None, None].expand(B, 1, S, S)
    with torch.no_grad():
        y = ref_layer(x.float(), attention_mask=mask, position_ids=pos, position_embeddings=(cos, sin))
    y = y[0] if isinstance(y, tuple) else y
    layer = FineLlamaDecoderLayer.from_hf(ref_layer, cfg, max_positions=256, device=gpu)
    out = layer(x.to(gpu))
    rel = float((out.float().cpu() - y).norm() / y.norm())
    assert rel <= 3e-3, rel


def test_generation_step_replays_from_a_hip_graph(lib, gpu):
    # A serving loop captures the launch-bound generation step once and replays it. Every kernel on the path is a plain
    # launch on the current stream (no memsets, no synchronisation); the split-KV workspace is obtained by a warm-up call on
    # the capture stream. Replays are interleaved with eager work and each is compared with the eager result.
    from llama_layer import FineKVCache, FineLlamaDecoderLayer
    B, S0, H, n_q, n_kv, F = 4, 640, 512, 8, 2, 1024
    w = layer_weights(H, n_q, n_kv, F, seed=30)
    layer = FineLlamaDecoderLayer({k: v.to(gpu) for k, v in w.items()}, n_q, n_kv, max_positions=1024)
    cache = FineKVCache(B, S0 + 1, n_kv, device=gpu)
    layer(so.randn_fp16((B, S0, H), 1).to(gpu), kv_cache=cache)
    x_static = so.randn_fp16((B, 1, H), 2).to(gpu)
    cache.length = S0
    eager = layer(x_static, kv_cache=cache).clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        cache.length = S0
        layer(x_static, kv_cache=cache)            # warm-up on the capture stream: workspace and allocator pools
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    cache.length = S0
    with torch.cuda.graph(graph, stream=side):
        out_static = layer(x_static, kv_cache=cache)
    for it in range(3):
        scratch = torch.randn(1 << 20, device=gpu).sum()      # unrelated eager work between replays
        x_new = so.randn_fp16((B, 1, H), 50 + it).to(gpu)
        x_static.copy_(x_new)
        graph.replay()
        torch.cuda.synchronize()
        cache.length = S0
        want = layer(x_new, kv_cache=cache)
        torch.cuda.synchronize()
        assert torch.equal(out_static, want), it
        assert torch.isfinite(scratch)
    x_static.copy_(so.randn_fp16((B, 1, H), 2).to(gpu))
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out_static, eager)


# ---- bfloat16 ---------------------------------------------------------------------------------------------------------
def close_one_bf16_rounding(out, ref):
    err = (out.float().cpu() - ref).abs()
    return bool((err <= 2.0 ** -8 * ref.abs() + 1e-6).all()), float(err.max())


def test_bfloat16_glue_kernels(lib, gpu):
    bf = lambda t: t.float().bfloat16()
    x, r, w = bf(so.randn_fp16((33, 1024), 1, 2.0)), bf(so.randn_fp16((33, 1024), 2)), bf(so.randn_fp16((1024,), 3))
    ref, h_ref = so.rmsnorm_ref(x, w, 1e-5, residual=r, round_residual=False)
    h_ref = h_ref.bfloat16().float()                      # the kernel stores and normalises the bf16-rounded sum
    ref, _ = so.rmsnorm_ref(h_ref, w, 1e-5)
    out, h = lib.rmsnorm(x.to(gpu), w.to(gpu), 1e-5, residual=r.to(gpu))
    assert out.dtype == torch.bfloat16 and torch.equal(h.float().cpu(), h_ref) and close_one_bf16_rounding(out, ref)[0]
    cos, sin = so.rope_tables(64, 128, 10000.0)
    pos = torch.arange(5, 5 + 9, dtype=torch.int32)
    q = bf(so.randn_fp16((2, 9, 6, 128), 4))
    qg = q.to(gpu)
    lib.rope(qg, cos.to(gpu), sin.to(gpu), pos.to(gpu), copy_heads=2)
    ref_q = so.rope_ref(q[:, :, :4].transpose(1, 2), cos, sin, pos[None].expand(2, 9)).transpose(1, 2)
    assert close_one_bf16_rounding(qg[:, :, :4], ref_q)[0] and torch.equal(qg[:, :, 4:].cpu(), q[:, :, 4:])
    gu = bf(so.randn_fp16((17, 512), 5, 3.0))
    assert close_one_bf16_rounding(lib.silu_mul(gu.to(gpu)), so.silu_mul_ref(gu))[0]


def test_bfloat16_decoder_layer_prefill_and_step(lib, gpu):
    # same layer in bfloat16 (weights, activations, cache); compared with the fp32 oracle on the bf16-rounded weights.
    # bf16 intermediates carry 8 significand bits: relative Frobenius error <= 1.5e-2.
    from llama_layer import FineKVCache, FineLlamaDecoderLayer
    B, S0, H, n_q, n_kv, F = 2, 600, 512, 8, 2, 1024
    w = {k: v.float().bfloat16() for k, v in layer_weights(H, n_q, n_kv, F, seed=40).items()}
    layer = FineLlamaDecoderLayer({k: v.to(gpu) for k, v in w.items()}, n_q, n_kv, max_positions=1024, dtype=torch.bfloat16)
    cache = FineKVCache(B, S0 + 2, n_kv, device=gpu, dtype=torch.bfloat16)
    x = so.randn_fp16((B, S0, H), 1).float().bfloat16()
    out = layer(x.to(gpu), kv_cache=cache)
    ref, k_ref, v_ref = so.llama_decoder_layer_ref(x, w, torch.arange(S0)[None].expand(B, S0), n_q, n_kv, round_stages=False)
    assert out.dtype == torch.bfloat16
    rel = float((out.float().cpu() - ref).norm() / ref.norm())
    assert rel <= 1.5e-2, rel
    xt = so.randn_fp16((B, 1, H), 2).float().bfloat16()
    out = layer(xt.to(gpu), kv_cache=cache)
    ref, _, _ = so.llama_decoder_layer_ref(xt, w, torch.full((B, 1), S0), n_q, n_kv, past_k=k_ref, past_v=v_ref,
                                           round_stages=False)
    rel = float((out.float().cpu() - ref).norm() / ref.norm())
    assert rel <= 1.5e-2, rel

"""Llama-3-8B-shaped prefill decoder layer chained on the GPU (benchmark configuration 5): fused QKV GEMM ->
causal GQA attention -> O projection -> gate/up GEMM -> SiLU(gate)*up -> down GEMM. Each GPU stage is compared
with the oracle fed the GPU's own previous-stage output (so errors do not compound in the comparison)."""
import pytest
import torch

import serving_oracle as so

pytestmark = pytest.mark.gpu


def gpu_layer(lib, x, w_qkv, w_o, w_gu, w_d, n_q=32, n_kv=8, d=128):
    S = x.shape[0]
    st = {}
    st["qkv"] = lib.hgemm(x, w_qkv)
    qkv = st["qkv"]
    q = qkv[:, : n_q * d].reshape(S, n_q, d).permute(1, 0, 2)[None].contiguous()
    k = qkv[:, n_q * d:(n_q + n_kv) * d].reshape(S, n_kv, d).permute(1, 0, 2)[None].contiguous()
    v = qkv[:, (n_q + n_kv) * d:].reshape(S, n_kv, d).permute(1, 0, 2)[None].contiguous()
    st["attn"], st["attn_lse"] = lib.fmha_fwd(q, k, v, causal=True)
    a2 = st["attn"][0].permute(1, 0, 2).reshape(S, n_q * d).contiguous()
    st["oproj"] = lib.hgemm(a2, w_o)
    st["gate_up"] = lib.hgemm(st["oproj"], w_gu)
    ffn = w_gu.shape[1] // 2
    st["act"] = (torch.nn.functional.silu(st["gate_up"][:, :ffn].float()) * st["gate_up"][:, ffn:].float()).half()
    st["down"] = lib.hgemm(st["act"], w_d)
    return st


def sample_rows(S):
    """Token rows checked at the full size: a stride that visits every residue of the 256- and 128-row tiles over the
    sequence, plus the rows either side of tile boundaries and both ends."""
    rows = set(range(0, S, 53)) | {0, 1, 127, 128, 255, 256, S // 2 - 1, S // 2, S - 257, S - 256, S - 2, S - 1}
    return torch.tensor(sorted(r for r in rows if 0 <= r < S))


@pytest.mark.parametrize("S", [1024, 8192])
def test_llama3_8b_layer_stages(lib, gpu, S):
    # S = 8192 is the benchmark's configuration: 256x256 GEMM tiles and the 256-query ping-pong attention kernel (S = 1024
    # runs the 128x128 tiles and the 4-wave attention kernel). At 8192 the oracle evaluates sampled token rows (every
    # output column of them; all heads of the attention, plus two heads in full), since the full fp32 chain is minutes of
    # host work.
    H, FFN = 4096, 14336
    x = so.randn_fp16((S, H), 0, 1.0)
    w_qkv = so.randn_fp16((H, 6144), 1, 0.02)
    w_o = so.randn_fp16((H, H), 2, 0.02)
    w_gu = so.randn_fp16((H, 2 * FFN), 3, 0.02)
    w_d = so.randn_fp16((FFN, H), 4, 0.02)
    g = gpu_layer(lib, *(t.to(gpu) for t in (x, w_qkv, w_o, w_gu, w_d)))
    torch.cuda.synchronize()
    c = {n: t.cpu() for n, t in g.items()}
    rows = sample_rows(S) if S > 2048 else None
    pick = (lambda t: t) if rows is None else (lambda t: t[rows])
    ref = so.llama_layer_ref(x, w_qkv, w_o, w_gu, w_d, rows=rows, stage_inputs={
        "attn_in": c["qkv"], "oproj_in": c["attn"], "gu_in": c["oproj"], "act_in": c["gate_up"], "down_in": c["act"]})
    for name, K in (("qkv", H), ("oproj", H), ("gate_up", H), ("down", FFN)):
        ok, st = so.gemm_tolerance_ok(pick(c[name]), ref[name], K)
        assert ok, (name, st)
    o_s = c["attn"] if rows is None else c["attn"][:, :, rows]
    l_s = c["attn_lse"] if rows is None else c["attn_lse"][:, :, rows]
    ok, st = so.fmha_tolerance_ok(o_s, l_s, ref["attn"], ref["attn_lse"])
    assert ok, st
    if rows is not None:   # two q heads (different kv heads) in full
        qkv = c["qkv"]
        for h in (5, 30):
            q1 = qkv[:, h * 128:(h + 1) * 128][None, None]
            kh = 32 * 128 + (h // 4) * 128
            k1, v1 = qkv[:, kh:kh + 128][None, None], qkv[:, kh + 8 * 128:kh + 9 * 128][None, None]
            o_ref, l_ref = so.attention_ref(q1, k1, v1, causal=True)
            ok, st = so.fmha_tolerance_ok(c["attn"][:, h:h + 1], c["attn_lse"][:, h:h + 1], o_ref, l_ref)
            assert ok, (h, st)
    # end to end against the pure fp32 chain: relative Frobenius error
    full = so.llama_layer_ref(x, w_qkv, w_o, w_gu, w_d, rows=rows)
    rel = float((pick(c["down"]).float() - full["down"]).norm() / full["down"].norm())
    assert rel < 2e-2, rel


def test_decoder_layer_at_llama3_8b_shapes_prefill_8192_and_a_generation_step(lib, gpu):
    # FineLlamaDecoderLayer at the benchmark's shapes (hidden 4096, 32 q / 8 kv heads, FFN 14336, 8192 tokens into a KV
    # cache), then one generation step over that cache: the 256x256 NT tiles with the SiLU*up epilogue at N = 28672, both
    # residual epilogues, ping-pong attention on strided operands at s = 8192 and the split-KV kernels over 8193 keys,
    # against the fp32 oracle of the layer with fp16 rounding between stages (sampled token rows for the prefill).
    from llama_layer import FineKVCache, FineLlamaDecoderLayer
    H, n_q, n_kv, F, S = 4096, 32, 8, 14336, 8192
    gw = lambda shape, seed: so.randn_fp16(shape, seed, 0.02)
    w = dict(q=gw((n_q * 128, H), 11), k=gw((n_kv * 128, H), 12), v=gw((n_kv * 128, H), 13), o=gw((H, n_q * 128), 14),
             gate=gw((F, H), 15), up=gw((F, H), 16), down=gw((H, F), 17))
    w["ln1"] = (1 + 0.1 * so.randn_fp16((H,), 18).float()).half()
    w["ln2"] = (1 + 0.1 * so.randn_fp16((H,), 19).float()).half()
    layer = FineLlamaDecoderLayer({k: v.to(gpu) for k, v in w.items()}, n_q, n_kv, max_positions=S + 8)
    cache = FineKVCache(1, S + 8, n_kv, device=gpu)
    x = so.randn_fp16((1, S, H), 20)
    out = layer(x.to(gpu), kv_cache=cache)
    torch.cuda.synchronize()
    rows = sample_rows(S)
    pos = torch.arange(S)[None]
    ref, k_ref, v_ref = so.llama_decoder_layer_ref(x, w, pos, n_q, n_kv, rows=rows)
    got = out[:, rows.to(gpu)].float().cpu()
    rel = float((got - ref).norm() / ref.norm())
    worst = float((got - ref).abs().max() / ref.abs().max())
    assert rel <= 2e-3 and worst <= 2e-2, (rel, worst)
    assert cache.length == S
    assert (cache.k[:, :S].transpose(1, 2).float().cpu() - k_ref).abs().max() <= 2e-2
    assert (cache.v[:, :S].transpose(1, 2).float().cpu() - v_ref).abs().max() <= 2e-2
    # one generation step over the 8192 cached tokens
    xt = so.randn_fp16((1, 1, H), 21)
    out1 = layer(xt.to(gpu), kv_cache=cache)
    ref1, _, _ = so.llama_decoder_layer_ref(xt, w, torch.full((1, 1), S), n_q, n_kv, past_k=k_ref, past_v=v_ref)
    got1 = out1.float().cpu()
    rel1 = float((got1 - ref1).norm() / ref1.norm())
    worst1 = float((got1 - ref1).abs().max() / ref1.abs().max())
    assert rel1 <= 2e-3 and worst1 <= 2e-2, (rel1, worst1)
    assert cache.length == S + 1

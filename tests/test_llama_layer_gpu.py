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


@pytest.mark.parametrize("S", [1024])
def test_llama3_8b_layer_stages(lib, gpu, S):
    H, FFN = 4096, 14336
    x = so.randn_fp16((S, H), 0, 1.0)
    w_qkv = so.randn_fp16((H, 6144), 1, 0.02)
    w_o = so.randn_fp16((H, H), 2, 0.02)
    w_gu = so.randn_fp16((H, 2 * FFN), 3, 0.02)
    w_d = so.randn_fp16((FFN, H), 4, 0.02)
    g = gpu_layer(lib, *(t.to(gpu) for t in (x, w_qkv, w_o, w_gu, w_d)))
    torch.cuda.synchronize()
    c = {n: t.cpu() for n, t in g.items()}
    ref = so.llama_layer_ref(x, w_qkv, w_o, w_gu, w_d, stage_inputs={
        "attn_in": c["qkv"], "oproj_in": c["attn"], "gu_in": c["oproj"], "act_in": c["gate_up"], "down_in": c["act"]})
    for name, K in (("qkv", H), ("oproj", H), ("gate_up", H), ("down", FFN)):
        ok, st = so.gemm_tolerance_ok(c[name], ref[name], K)
        assert ok, (name, st)
    ok, st = so.fmha_tolerance_ok(c["attn"], c["attn_lse"], ref["attn"], ref["attn_lse"])
    assert ok, st
    # end to end against the pure fp32 chain: relative Frobenius error
    full = so.llama_layer_ref(x, w_qkv, w_o, w_gu, w_d)
    rel = float((c["down"].float() - full["down"]).norm() / full["down"].norm())
    assert rel < 2e-2, rel

"""Pins the CPU oracle (oracle/serving_oracle.py) without a GPU: closed forms, invariants, fp64 brute force
with explicit loops, torch's own SDPA as a second opinion, and the committed golden fixtures. Each check is
chosen so that a plausible mistake (transposed operand, wrong head mapping, off-by-one in a mask, missing scale,
wrong log base) fails at least one of them."""
import math
import os

import numpy as np
import pytest
import torch

import serving_oracle as so

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


# ------------------------------------------------------------------ GEMM
def test_gemm_identity_and_onehot():
    b = so.randn_fp16((48, 40), 1)
    assert torch.equal(so.gemm_ref(torch.eye(48).half(), b, "NN"), b.float())
    # one-hot row i of A picks row perm[i] of B: catches any transposition of the operands
    perm = torch.randperm(48, generator=torch.Generator().manual_seed(3))
    a = torch.zeros(48, 48).half()
    a[torch.arange(48), perm] = 1
    assert torch.equal(so.gemm_ref(a, b, "NN"), b.float()[perm])
    assert torch.equal(so.gemm_ref(a.t().contiguous(), b, "TN"), b.float()[perm])
    assert torch.equal(so.gemm_ref(a, b.t().contiguous(), "NT"), b.float()[perm])


def test_gemm_all_ones_counts_k():
    for K in (64, 1024, 2048):
        c = so.gemm_ref(torch.ones(8, K).half(), torch.ones(K, 8).half())
        assert torch.equal(c, torch.full((8, 8), float(K)))


def test_gemm_power_of_two_sums_are_exact():
    g = torch.Generator().manual_seed(5)
    a = torch.ldexp(torch.ones(16, 32), torch.randint(-3, 4, (16, 32), generator=g)).half()
    b = torch.ldexp(torch.ones(32, 16), torch.randint(-3, 4, (32, 16), generator=g)).half()
    ref = so.gemm_bruteforce_f64(a.numpy(), b.numpy())
    assert np.array_equal(so.gemm_ref(a, b).double().numpy(), ref)


@pytest.mark.parametrize("layout", ["NN", "TN", "NT"])
def test_gemm_bruteforce_nonsquare(layout):
    M, N, K = 20, 12, 36
    a = so.randn_fp16((K, M) if layout == "TN" else (M, K), 7)
    b = so.randn_fp16((N, K) if layout == "NT" else (K, N), 8)
    ref = so.gemm_bruteforce_f64(a.numpy(), b.numpy(), layout)
    got = so.gemm_ref(a, b, layout).double().numpy()
    assert got.shape == (M, N)
    assert np.abs(got - ref).max() < 1e-4


def test_gemm_index_layout_table_matches_reference_correct_py():
    # kernels/gemm/test/correct.py:39-43: 12 and 16 are called with a_format='N' (a.T @ b), 13..15 with b_format='N'
    assert [so.GEMM_LAYOUT_OF_INDEX[i] for i in (12, 13, 14, 15, 16)] == ["TN", "NT", "NT", "NT", "TN"]
    assert all(so.GEMM_LAYOUT_OF_INDEX[i] == "NN" for i in range(12))
    a, b = so.randn_fp16((8, 8), 1), so.randn_fp16((8, 8), 2)
    assert torch.allclose(so.fine_gemm_ref(a, b, 16), a.float().t() @ b.float())
    assert torch.allclose(so.fine_gemm_ref(a, b, 13), a.float() @ b.float().t())


def test_gemm_golden_fixture():
    z = np.load(os.path.join(GOLDEN, "gemm_seed0_256.npz"))
    a, b, rows = torch.from_numpy(z["a"]), torch.from_numpy(z["b"]), z["rows"]
    for lay in ("NN", "TN", "NT"):
        got = so.gemm_ref(a, b, lay).numpy()[rows]
        assert np.allclose(got, z["c_" + lay], rtol=1e-5, atol=1e-4), lay
    # the fixture inputs are the reference's seeded draw (correct.py:5-8)
    torch.manual_seed(0)
    assert torch.equal(torch.randn(256, 256, dtype=torch.half), a)


def test_gemm_tolerance_checker():
    ref = torch.full((4, 4), 100.0)
    ok, _ = so.gemm_tolerance_ok(ref + 0.5, ref, 1024)
    assert ok
    ok, st = so.gemm_tolerance_ok(ref + 1.5, ref, 1024)
    assert not ok and st["violations"] == 16


# ------------------------------------------------------------------ attention
def test_attention_equal_keys_gives_running_mean():
    # all keys equal => uniform softmax over the visible keys
    B, H, S, D = 1, 2, 37, 128
    q = so.randn_fp16((B, H, S, D), 1)
    k = so.randn_fp16((B, H, 1, D), 2).expand(B, H, S, D).contiguous()
    v = so.randn_fp16((B, H, S, D), 3)
    o, lse = so.attention_ref(q, k, v, causal=True)
    vm = v.float().cumsum(2) / torch.arange(1, S + 1)[None, None, :, None]
    assert torch.allclose(o, vm, atol=1e-5)
    s0 = (q.float() * k.float()).sum(-1) / math.sqrt(D)
    assert torch.allclose(lse, s0 + torch.log(torch.arange(1, S + 1).float()), atol=1e-4)
    o2, lse2 = so.attention_ref(q, k, v, causal=False)
    assert torch.allclose(o2, v.float().mean(2, keepdim=True).expand_as(o2), atol=1e-5)
    assert torch.allclose(lse2, s0 + math.log(S), atol=1e-4)


def test_attention_zero_query_and_ones_value():
    q = torch.zeros(1, 1, 9, 128).half()
    k, v = so.randn_fp16((1, 1, 21, 128), 4), torch.ones(1, 1, 21, 128).half()
    o, lse = so.attention_ref(q, k, v, causal=False)
    assert torch.allclose(lse, torch.full_like(lse, math.log(21)), atol=1e-6)
    assert torch.allclose(o, torch.ones_like(o), atol=1e-6)  # softmax rows sum to one
    # bottom-right causal with Sq=9 < Sk=21: query i sees keys 0..i+12
    o, lse = so.attention_ref(q, k, v, causal=True)
    assert torch.allclose(lse[0, 0], torch.log(torch.arange(13, 22).float()), atol=1e-6)


def test_attention_first_causal_row_and_dominant_key():
    q, k, v = so.fmha_inputs(1, 2, 2, 16, 16, seed=9)
    o, lse = so.attention_ref(q, k, v, causal=True)
    assert torch.allclose(o[:, :, 0], v.float()[:, :, 0], atol=1e-6)
    s00 = (q.float()[:, :, 0] * k.float()[:, :, 0]).sum(-1) / math.sqrt(128)
    assert torch.allclose(lse[:, :, 0], s00, atol=1e-5)
    # one dominant key: a query aligned with key 5 and scaled so its score leads by > 40
    k2 = k.clone()
    q2 = (k2[:, :, 5:6] * 8).expand(1, 2, 16, 128).contiguous()
    o2, _ = so.attention_ref(q2, k2, v, causal=False)
    assert torch.allclose(o2, v.float()[:, :, 5:6].expand_as(o2), atol=1e-3)


def test_attention_key_permutation_invariance_and_kv_valid_len():
    q, k, v = so.fmha_inputs(1, 1, 1, 8, 50, seed=10)
    perm = torch.randperm(50, generator=torch.Generator().manual_seed(1))
    o1, l1 = so.attention_ref(q, k, v)
    o2, l2 = so.attention_ref(q, k[:, :, perm], v[:, :, perm])
    assert torch.allclose(o1, o2, atol=1e-5) and torch.allclose(l1, l2, atol=1e-5)
    # masking keys >= 30 equals dropping them (pins the off-by-one: key 30 itself must be masked)
    o3, l3 = so.attention_ref(q, k, v, kv_valid_len=30)
    o4, l4 = so.attention_ref(q, k[:, :, :30], v[:, :, :30])
    assert torch.allclose(o3, o4, atol=1e-6) and torch.allclose(l3, l4, atol=1e-6)
    # LSE grows when keys are added
    assert bool((l1 > l3).all())


def test_attention_gqa_head_mapping():
    # kv head = q head // (Hq / Hkv): q heads 0..3 -> kv 0, 4..7 -> kv 1 (kernels/fmha/test/perf.py:10-23)
    q, k, v = so.fmha_inputs(1, 8, 2, 12, 12, seed=11)
    o, lse = so.attention_ref(q, k, v, causal=True)
    for h in range(8):
        oh, lh = so.attention_ref(q[:, h:h + 1], k[:, h // 4:h // 4 + 1], v[:, h // 4:h // 4 + 1], causal=True)
        assert torch.allclose(o[:, h:h + 1], oh, atol=1e-6) and torch.allclose(lse[:, h:h + 1], lh, atol=1e-6)


@pytest.mark.parametrize("causal,Sq,Sk,kvv", [(False, 8, 13, None), (True, 8, 8, None), (True, 5, 11, None),
                                                (True, 11, 5, None), (False, 3, 17, 9), (True, 9, 17, 14)])
def test_attention_vs_bruteforce_f64(causal, Sq, Sk, kvv):
    q, k, v = so.fmha_inputs(1, 2, 1, Sq, Sk, seed=12)
    o, lse = so.attention_ref(q, k, v, causal=causal, kv_valid_len=kvv)
    ob, lb = so.attention_bruteforce_f64(q.numpy(), k.numpy(), v.numpy(), causal, kvv)
    assert np.abs(o.double().numpy() - ob).max() < 1e-5
    fin = np.isfinite(lb)
    assert np.array_equal(np.isfinite(lse.numpy()), fin)
    assert np.abs(lse.double().numpy()[fin] - lb[fin]).max() < 1e-5
    # rows with no visible key (Sq > Sk, causal): O = 0
    assert np.all(o.numpy()[~fin] == 0)


def test_attention_vs_torch_sdpa():
    q, k, v = so.fmha_inputs(2, 8, 2, 33, 33, seed=13)
    kk, vv = k.float().repeat_interleave(4, 1), v.float().repeat_interleave(4, 1)
    for causal in (False, True):
        ref = torch.nn.functional.scaled_dot_product_attention(q.float(), kk, vv, is_causal=causal)
        assert torch.allclose(so.attention_ref(q, k, v, causal=causal)[0], ref, atol=2e-6)
        assert torch.allclose(so.fine_fmha_ref(q, k, v, causal, False), ref, atol=2e-6)
        assert torch.allclose(so.attention_sdpa_ref(q, k, v, causal), ref, atol=1e-6)
    with pytest.raises(ValueError):
        so.fine_fmha_ref(q, k, v, True, True)


def test_fmha_golden_fixture():
    z = np.load(os.path.join(GOLDEN, "fmha_seed42_128.npz"))
    q, k, v = (torch.from_numpy(z[n]) for n in ("q", "k", "v"))
    rows = z["qrows"]
    for tag, causal in (("full", False), ("causal", True)):
        o, lse = so.attention_ref(q, k, v, causal=causal)
        assert np.allclose(o.numpy()[:, :, rows], z["o_" + tag], atol=1e-6)
        assert np.allclose(lse.numpy(), z["lse_" + tag], atol=1e-6)
    torch.manual_seed(42)
    assert torch.equal(torch.randn(size=(1, 4, 128, 128), dtype=torch.half) * 0.1, q)


def test_llama_layer_ref_shapes_and_composition():
    S, H, nq, nkv, d, F = 16, 64, 4, 2, 16, 48
    g = lambda shape, seed, std: so.randn_fp16(shape, seed, std)
    x, wqkv, wo = g((S, H), 0, 1.0), g((H, (nq + 2 * nkv) * d), 1, 0.1), g((nq * d, H), 2, 0.1)
    wgu, wd = g((H, 2 * F), 3, 0.1), g((F, H), 4, 0.1)
    out = so.llama_layer_ref(x, wqkv, wo, wgu, wd, n_q=nq, n_kv=nkv, d=d)
    assert out["qkv"].shape == (S, (nq + 2 * nkv) * d) and out["attn"].shape == (1, nq, S, d)
    assert out["down"].shape == (S, H)
    # q head 0 of the chain equals attention on the sliced projections
    qkv = out["qkv"].half().float()
    q0, k0, v0 = qkv[:, :d], qkv[:, nq * d:nq * d + d], qkv[:, (nq + nkv) * d:(nq + nkv) * d + d]
    ref = torch.nn.functional.scaled_dot_product_attention(q0[None, None], k0[None, None], v0[None, None], is_causal=True)
    assert torch.allclose(out["attn"][0, 0], ref[0, 0], atol=1e-5)
    gu = out["gate_up"].half().float()
    assert torch.allclose(out["act"], torch.nn.functional.silu(gu[:, :F]) * gu[:, F:], atol=1e-6)


# ---- layer glue of the in-model path ---------------------------------------------------------------------------------
def test_rmsnorm_closed_forms():
    # a constant row c normalises to sign(c) * weight (eps = 0); scaling the input leaves the output unchanged
    w = torch.linspace(0.5, 1.5, 64)
    out, _ = so.rmsnorm_ref(torch.full((3, 64), -2.5), w, eps=0.0)
    assert torch.allclose(out, -w.expand(3, 64), atol=1e-6)
    x = so.randn_fp16((5, 64), 1).float()
    a, _ = so.rmsnorm_ref(x, w, eps=0.0)
    b, _ = so.rmsnorm_ref(4 * x, w, eps=0.0)
    assert torch.allclose(a, b, atol=1e-5)
    # unit weight: every output row has mean square 1; eps enters as mean(x^2) + eps
    one, _ = so.rmsnorm_ref(x, torch.ones(64), eps=0.0)
    assert torch.allclose(one.pow(2).mean(-1), torch.ones(5), atol=1e-5)
    e, _ = so.rmsnorm_ref(torch.ones(1, 64), torch.ones(64), eps=3.0)
    assert torch.allclose(e, torch.full((1, 64), 0.5), atol=1e-6)
    # residual: the sum is rounded to fp16 and returned
    r = torch.full((1, 64), 1.0)
    o2, h = so.rmsnorm_ref(torch.full((1, 64), 2.0 ** -12), torch.ones(64), eps=0.0, residual=r)
    assert torch.equal(h, r)  # 1 + 2^-12 rounds to 1 in fp16


def test_rope_closed_forms():
    cos, sin = so.rope_tables(50, 128, 10000.0)
    assert cos.shape == (50, 64) and torch.equal(cos[0], torch.ones(64)) and torch.equal(sin[0], torch.zeros(64))
    # frequency 0 turns by one radian per position, the last one by base^(-126/128)
    assert abs(cos[7, 0] - math.cos(7.0)) < 1e-6 and abs(sin[3, 63] - math.sin(3.0 * 10000.0 ** (-126 / 128))) < 1e-6
    x = so.randn_fp16((2, 3, 6, 128), 5).float()
    pos = torch.tensor([[0, 1, 2, 3, 4, 5], [10, 11, 12, 13, 14, 49]])
    y = so.rope_ref(x, cos, sin, pos)
    assert torch.equal(y[0, :, 0], x[0, :, 0])                      # position 0 is the identity
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), rtol=1e-5)  # a rotation
    # pair (i, i + 64) turns by the angle pos * inv_freq_i, by hand for one element
    ang = 12 * 10000.0 ** (-2 * 5 / 128)
    want = x[1, 2, 2, 5] * math.cos(ang) - x[1, 2, 2, 69] * math.sin(ang)
    want_hi = x[1, 2, 2, 69] * math.cos(ang) + x[1, 2, 2, 5] * math.sin(ang)
    assert abs(y[1, 2, 2, 5] - want) < 1e-5 and abs(y[1, 2, 2, 69] - want_hi) < 1e-5
    # scores depend only on the distance between positions
    q, k = x[:1, :1, :1], x[:1, 1:2, 1:2]
    def score(pq, pk):
        return (so.rope_ref(q, cos, sin, torch.tensor([[pq]])) * so.rope_ref(k, cos, sin, torch.tensor([[pk]]))).sum()
    assert abs(score(9, 4) - score(30, 25)) < 1e-3 and abs(score(9, 4) - score(9, 5)) > 1e-3


def test_silu_mul_closed_forms():
    gu = torch.tensor([[0.0, 20.0, -20.0, 1.0, 3.0, 2.0, 5.0, -4.0]])
    out = so.silu_mul_ref(gu)
    want = torch.tensor([[0.0, 40.0, -20.0 / (1 + math.exp(20.0)) * 5.0, 1.0 / (1 + math.exp(-1.0)) * -4.0]])
    assert torch.allclose(out, want, atol=1e-6)


def test_decoder_layer_against_transformers_llama():
    # independent second implementation: the Llama layer of the installed transformers package, fp32, eager attention
    pytest.importorskip("transformers")
    from transformers import LlamaConfig
    from transformers.models.llama import modeling_llama as hf
    cfg = LlamaConfig(hidden_size=512, num_attention_heads=4, num_key_value_heads=2, head_dim=128, intermediate_size=1024,
                      rms_norm_eps=1e-5, rope_theta=10000.0, vocab_size=32, num_hidden_layers=1, attention_bias=False,
                      mlp_bias=False)
    cfg._attn_implementation = "eager"
    torch.manual_seed(0)
    layer = hf.LlamaDecoderLayer(cfg, 0).float().eval()
    for p in layer.parameters():
        torch.nn.init.normal_(p, std=0.05)
    layer.input_layernorm.weight.data = 1 + 0.1 * torch.randn(512)
    layer.post_attention_layernorm.weight.data = 1 + 0.1 * torch.randn(512)
    B, S = 2, 37
    x = torch.randn(B, S, 512)
    pos = torch.arange(S)[None].expand(B, S)
    cos, sin = hf.LlamaRotaryEmbedding(cfg)(x, pos)
    mask = torch.full((S, S), float("-inf")).triu(1)[None, None].expand(B, 1, S, S)
    with torch.no_grad():
        y = layer(x, attention_mask=mask, position_ids=pos, position_embeddings=(cos, sin))
    y = y[0] if isinstance(y, tuple) else y
    a, mlp = layer.self_attn, layer.mlp
    w = dict(q=a.q_proj.weight, k=a.k_proj.weight, v=a.v_proj.weight, o=a.o_proj.weight, gate=mlp.gate_proj.weight,
             up=mlp.up_proj.weight, down=mlp.down_proj.weight, ln1=layer.input_layernorm.weight,
             ln2=layer.post_attention_layernorm.weight)
    out, k, v = so.llama_decoder_layer_ref(x, w, pos, 4, 2, eps=1e-5, round_stages=False)
    assert (y - out).abs().max() < 2e-5 * y.abs().max()
    # generation step with the cache of the prefill == last row of a prefill that is one token longer
    x1 = torch.randn(B, 1, 512)
    out1, _, _ = so.llama_decoder_layer_ref(x1, w, torch.full((B, 1), S), 4, 2, past_k=k, past_v=v, round_stages=False)
    full, _, _ = so.llama_decoder_layer_ref(torch.cat((x, x1), 1), w, torch.arange(S + 1)[None].expand(B, S + 1), 4, 2,
                                            round_stages=False)
    assert torch.allclose(out1[:, 0], full[:, -1], atol=1e-4)


def test_sampled_rows_are_the_rows_of_the_full_result():
    # q_rows / rows restrict the (pinned) full-size functions to some token rows for the 8192-token checks; they must
    # reproduce exactly those rows, masks included (up to fp32 summation order inside the BLAS call)
    q, k, v = so.fmha_inputs(2, 4, 2, 70, 101, seed=3)
    rows = torch.tensor([0, 3, 17, 69])
    for causal, kvv in ((True, None), (False, 90), (True, 95), (True, 20)):
        o, l = so.attention_ref(q, k, v, causal, kvv)
        o2, l2 = so.attention_ref(q, k, v, causal, kvv, q_rows=rows)
        assert (o[:, :, rows] - o2).abs().max() <= 1e-5
        fin = torch.isfinite(l[:, :, rows])
        assert torch.equal(fin, torch.isfinite(l2)) and (l[:, :, rows][fin] - l2[fin]).abs().max() <= 1e-5
    S, H, F = 300, 256, 512
    x = so.randn_fp16((S, H), 0)
    wq, wo = so.randn_fp16((H, 512), 1, 0.05), so.randn_fp16((256, H), 2, 0.05)
    wgu, wd = so.randn_fp16((H, 2 * F), 3, 0.05), so.randn_fp16((F, H), 4, 0.05)
    rows = torch.tensor([0, 5, 128, 299])
    full = so.llama_layer_ref(x, wq, wo, wgu, wd, n_q=2, n_kv=1)
    part = so.llama_layer_ref(x, wq, wo, wgu, wd, n_q=2, n_kv=1, rows=rows)
    si = {"attn_in": full["qkv"].half(), "oproj_in": full["attn"].half(), "gu_in": full["oproj"].half(),
          "act_in": full["gate_up"].half(), "down_in": full["act"].half()}
    a = so.llama_layer_ref(x, wq, wo, wgu, wd, n_q=2, n_kv=1, stage_inputs=si)
    b = so.llama_layer_ref(x, wq, wo, wgu, wd, n_q=2, n_kv=1, stage_inputs=si, rows=rows)
    for name in ("qkv", "oproj", "gate_up", "act", "down"):
        assert (full[name][rows] - part[name]).abs().max() <= 1e-4 * full[name].abs().max(), name
        assert (a[name][rows] - b[name]).abs().max() <= 1e-4 * a[name].abs().max(), name
    assert (full["attn"][:, :, rows] - part["attn"]).abs().max() <= 1e-5
    g = lambda shape, s_: so.randn_fp16(shape, s_, 0.05)
    w = dict(q=g((256, H), 1), k=g((128, H), 2), v=g((128, H), 3), o=g((H, 256), 4), gate=g((F, H), 5), up=g((F, H), 6),
             down=g((H, F), 7), ln1=torch.ones(H).half(), ln2=torch.ones(H).half())
    xb = so.randn_fp16((2, S, H), 9)
    pos = torch.arange(S)[None].expand(2, S)
    f, kf, vf = so.llama_decoder_layer_ref(xb, w, pos, 2, 1, round_stages=False)
    p, kp, vp = so.llama_decoder_layer_ref(xb, w, pos, 2, 1, round_stages=False, rows=rows)
    assert (f[:, rows] - p).abs().max() <= 1e-4 * f.abs().max() and torch.equal(kf, kp) and torch.equal(vf, vp)

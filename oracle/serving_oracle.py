"""CPU oracle for the two serving kernels: fp16 GEMM and fused attention forward.

TEST INFRASTRUCTURE ONLY. Nothing in the product (the HIP library, the torch operators, their python shims)
imports this module; it is used by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg, as
the checker and as the timed CPU baseline, never as the implementation.

What it restates. The reference's path is CUDA/HIP device code with no CPU implementation, and none of it can be
compiled or run without a GPU; every function on the path is a realisation of one of two textbook results, so the
oracle states those results directly in fp32 (torch) and, for small inputs, again in fp64 with explicit loops:

  gemm_ref            C = op(a) op(b) in fp32 over the fp16-rounded operands. Layout per operator index follows
                      kernels/gemm/test/correct.py:9-15 (a.T @ b for a_format 'N', a @ b.T for b_format 'N') and
                      the loads in manual/gemm_12_amd.cpp:52-57, gemm_13_amd.cpp:58-60, gemm_16_amd.cpp:55-57.
  attention_ref       O = softmax(scale q k^T + mask) v and LSE, fp32. GQA head mapping follows
                      kernels/fmha/test/perf.py:10-24 (repeat_kv == repeat_interleave on the head axis) and
                      semi/fmha_2_amd.cpp:33-42; causal rule "masked iff q_pos < k_pos" follows fmha_2_amd.cpp:187-190
                      generalised to the bottom-right alignment (identical when Sq == Sk); keys at or beyond
                      kv_valid_len are masked (fmha_2_amd.cpp:191 with its off-by-one corrected); scale 1/sqrt(d)
                      follows fmha_2_amd.cpp:320.
  attention_sdpa_ref  the reference's test-side baseline torch_attn (kernels/fmha/test/perf.py:10-24): repeat_kv +
                      torch SDPA; checked against attention_ref, used as the timed CPU baseline.
  fine_fmha_ref       the pad-to-64 / decode_length / slice shim of kernels/fmha/pkg/fmha_unified/ops.py:8-29
                      expressed on top of attention_ref (padding rows are masked, so it reduces to attention_ref).
  llama_layer_ref     the Llama-3-8B-shaped prefill chain of the benchmark configuration (QKV GEMM -> causal GQA
                      attention -> O projection -> gate/up GEMM -> SiLU(gate)*up -> down GEMM), fp32.

  rmsnorm_ref, rope_tables, rope_ref, silu_mul_ref, llama_decoder_layer_ref
                      the glue of the reference's in-model path in fp32: LlamaRMSNorm.forward
                      (benchmarks/flashattn-cuda/modeling_llama.py:95-100), LlamaRotaryEmbedding (:113,119-132),
                      rotate_half / apply_rotary_pos_emb (:164-168,193-194), act_fn(gate) * up (:227) and the
                      decoder layer that strings them together (LlamaSdpaAttention.forward :652-704 with a KV
                      cache, LlamaDecoderLayer.forward :755-781). Pinned by closed forms (constant rows, unit
                      weights, position 0, norm preservation, the relative-position property, d = 2 rotation by
                      hand, silu(0) / large-argument limits) and against the Llama layer of the installed
                      `transformers` package as an independent second implementation.

Reference-specific numerical behaviour (fp16 accumulation in finegemm_0..11, fp16 softmax statistics in
finefmha_0..3) is deliberately NOT restated: the parity target is the fp32 result.

Pinning. The reference's tests hold no stored vectors (only seeded generators: correct.py seeds 0 / 42), so the
oracle is pinned by what the mathematics fixes; tests/test_oracle.py checks every function below against closed
forms (identity, one-hot, all-ones, exact power-of-two sums; uniform-softmax running means, single visible key,
V = ones, dominant key, key-permutation invariance, GQA head sharing), against fp64 brute force written with
explicit loops (gemm_bruteforce_f64, attention_bruteforce_f64), and against torch's own
scaled_dot_product_attention as a second opinion. No function here is "parity unpinned".
"""
import math

import numpy as np
import torch

GEMM_LAYOUT_OF_INDEX = {i: "NN" for i in range(12)}
GEMM_LAYOUT_OF_INDEX.update({12: "TN", 16: "TN", 13: "NT", 14: "NT", 15: "NT"})


# ---------------------------------------------------------------------------------------------------------------
# GEMM
# ---------------------------------------------------------------------------------------------------------------
def gemm_ref(a: torch.Tensor, b: torch.Tensor, layout: str = "NN") -> torch.Tensor:
    """fp32 product of the (fp16-valued) operands. layout NN: a[M,K] b[K,N]; TN: a[K,M]; NT: b[N,K]."""
    a32 = a.detach().to("cpu", torch.float32)
    b32 = b.detach().to("cpu", torch.float32)
    if layout == "TN":
        a32 = a32.t()
    elif layout == "NT":
        b32 = b32.t()
    elif layout != "NN":
        raise ValueError(layout)
    return a32 @ b32


def fine_gemm_ref(a, b, kernel_index: int) -> torch.Tensor:
    """What gemm_unified.ops.fine_gemm(a, b, kernel_index) must return, in fp32."""
    return gemm_ref(a, b, GEMM_LAYOUT_OF_INDEX[int(kernel_index)])


def gemm_bruteforce_f64(a, b, layout: str = "NN") -> np.ndarray:
    """Triple loop in fp64 (small inputs only)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    if layout == "TN":
        a = a.T
    if layout == "NT":
        b = b.T
    M, K = a.shape
    K2, N = b.shape
    assert K == K2
    c = np.zeros((M, N), dtype=np.float64)
    for i in range(M):
        for j in range(N):
            s = 0.0
            for k in range(K):
                s += a[i, k] * b[k, j]
            c[i, j] = s
    return c


def gemm_tolerance_ok(c, ref, K: int):
    """Element-wise |err| <= 2e-2*sqrt(K/1024) + 1e-2*|ref| and max|err|/max|ref| <= 1e-2. Returns (ok, stats)."""
    c32 = c.detach().to("cpu", torch.float32)
    r32 = ref.detach().to("cpu", torch.float32)
    err = (c32 - r32).abs()
    bound = 2e-2 * math.sqrt(K / 1024.0) + 1e-2 * r32.abs()
    elem_ok = bool((err <= bound).all())
    max_ref = float(r32.abs().max())
    rel = float(err.max()) / max_ref if max_ref > 0 else float(err.max())
    return elem_ok and rel <= 1e-2, {"max_abs_err": float(err.max()), "max_rel_to_max": rel,
                                     "violations": int((err > bound).sum())}


# ---------------------------------------------------------------------------------------------------------------
# attention
# ---------------------------------------------------------------------------------------------------------------
def visible_mask(Sq: int, Sk: int, causal: bool, kv_valid_len=None) -> torch.Tensor:
    """Boolean [Sq, Sk]: True where key j is visible to query i."""
    if kv_valid_len is None:
        kv_valid_len = Sk
    j = torch.arange(Sk)[None, :]
    i = torch.arange(Sq)[:, None]
    vis = (j < kv_valid_len).expand(Sq, Sk).clone()
    if causal:
        vis &= j <= i + (Sk - Sq)
    return vis


def attention_ref(q, k, v, causal: bool = False, kv_valid_len=None, scale=None, q_rows=None):
    """fp32 softmax attention. q [B,Hq,Sq,D], k, v [B,Hkv,Sk,D]. Returns (O [B,Hq,Sq,D], LSE [B,Hq,Sq]) fp32.

    Rows with no visible key give O = 0 and LSE = -inf.
    q_rows (1-D index tensor): evaluate only these query rows of the Sq-row problem (same mask rows, same keys) and
    return O [B,Hq,len(q_rows),D], LSE [B,Hq,len(q_rows)]: the rows of the full result, for checks at sizes where the
    full score matrix is too much host work.
    """
    q32 = q.detach().to("cpu", torch.float32)
    k32 = k.detach().to("cpu", torch.float32)
    v32 = v.detach().to("cpu", torch.float32)
    B, Hq, Sq, D = q32.shape
    Hkv, Sk = k32.shape[1], k32.shape[2]
    assert Hq % Hkv == 0
    rep = Hq // Hkv
    if rep > 1:
        k32 = k32.repeat_interleave(rep, dim=1)
        v32 = v32.repeat_interleave(rep, dim=1)
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    vis = visible_mask(Sq, Sk, causal, kv_valid_len)
    if q_rows is not None:
        q_rows = torch.as_tensor(q_rows, dtype=torch.long)
        q32 = q32[:, :, q_rows]
        vis = vis[q_rows]
    out = torch.empty_like(q32)
    lse = torch.empty((B, Hq, q32.shape[2]), dtype=torch.float32)
    for b in range(B):  # head by head keeps the score matrix small
        for h in range(Hq):
            s = (q32[b, h] @ k32[b, h].t()) * scale
            s = s.masked_fill(~vis, float("-inf"))
            l = torch.logsumexp(s, dim=-1)
            p = torch.exp(s - torch.where(torch.isinf(l), torch.zeros_like(l), l)[:, None])
            p = torch.where(vis, p, torch.zeros_like(p))
            out[b, h] = p @ v32[b, h]
            lse[b, h] = l
    return out, lse


def fine_fmha_ref(q, k, v, causal: bool, is_decode: bool):
    """What fmha_unified.ops.fine_fmha must return (fp32): ops.py:8-29 pads to 64, passes decode_length =
    un-padded key count, slices the padded query rows off. Padded keys are masked, padded queries are dropped,
    so this equals attention over the un-padded tensors."""
    if is_decode and causal:
        raise ValueError("causal is not supported in decode mode")  # semi/fmha_2_amd.cpp:331-333
    return attention_ref(q, k, v, causal=causal, kv_valid_len=k.shape[2])[0]


def attention_sdpa_ref(q, k, v, causal: bool = False):
    """The reference's own test baseline (kernels/fmha/test/perf.py:10-24, correct.py:9-23): repeat the kv heads
    (repeat_kv == repeat_interleave on dim 1) and call torch's scaled_dot_product_attention, here in fp32 on the
    CPU. Top-left causal alignment, so only meaningful for Sq == Sk when causal. Used as the timed CPU baseline."""
    q32 = q.detach().to("cpu", torch.float32)
    k32 = k.detach().to("cpu", torch.float32)
    v32 = v.detach().to("cpu", torch.float32)
    rep = q32.shape[1] // k32.shape[1]
    if rep > 1:
        k32 = k32.repeat_interleave(rep, dim=1)
        v32 = v32.repeat_interleave(rep, dim=1)
    return torch.nn.functional.scaled_dot_product_attention(q32, k32, v32, is_causal=causal)


def attention_bruteforce_f64(q, k, v, causal=False, kv_valid_len=None, scale=None):
    """Explicit-loop fp64 attention (tiny inputs only). Returns (O, LSE) as numpy arrays."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    B, Hq, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    rep = Hq // Hkv
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    if kv_valid_len is None:
        kv_valid_len = Sk
    O = np.zeros((B, Hq, Sq, D))
    L = np.full((B, Hq, Sq), -np.inf)
    for b in range(B):
        for h in range(Hq):
            hk = h // rep
            for i in range(Sq):
                scores = []
                for j in range(Sk):
                    if j >= kv_valid_len or (causal and j > i + (Sk - Sq)):
                        continue
                    scores.append((j, scale * float(np.dot(q[b, h, i], k[b, hk, j]))))
                if not scores:
                    continue
                m = max(s for _, s in scores)
                den = sum(math.exp(s - m) for _, s in scores)
                acc = np.zeros(D)
                for j, s in scores:
                    acc += math.exp(s - m) / den * v[b, hk, j]
                O[b, h, i] = acc
                L[b, h, i] = m + math.log(den)
    return O, L


def fmha_tolerance_ok(o, lse, o_ref, lse_ref):
    """max|O - O_ref| <= 2e-3 and max|LSE - LSE_ref| <= 1e-3 (rows with -inf LSE must match exactly)."""
    o32 = o.detach().to("cpu", torch.float32)
    eo = float((o32 - o_ref).abs().max())
    stats = {"max_abs_err_o": eo}
    ok = eo <= 2e-3
    if lse is not None:
        l32 = lse.detach().to("cpu", torch.float32)
        inf_ref = torch.isinf(lse_ref)
        same_inf = bool((torch.isinf(l32) == inf_ref).all())
        fin = ~inf_ref
        el = float((l32[fin] - lse_ref[fin]).abs().max()) if fin.any() else 0.0
        stats["max_abs_err_lse"] = el
        ok = ok and same_inf and el <= 1e-3
    return ok, stats


# ---------------------------------------------------------------------------------------------------------------
# Llama-3-8B-shaped prefill layer (benchmark configuration 5): hidden 4096, 32 q / 8 kv heads, d 128, FFN 14336
# ---------------------------------------------------------------------------------------------------------------
def llama_layer_ref(x, w_qkv, w_o, w_gu, w_d, n_q=32, n_kv=8, d=128, stage_inputs=None, rows=None):
    """fp32 chain. x [S, H]; weights stored [K, N]. Returns dict of every stage's fp32 output.

    stage_inputs, when given, maps a stage name to the tensor to feed INTO that stage instead of the oracle's own
    previous output (used to check each GPU stage against an oracle fed the GPU's previous-stage result).
    rows (1-D index tensor): every returned stage holds only these token rows of the full result (the QKV product is
    still formed for all rows, because every key and value feeds the attention of the sampled rows; stage_inputs stay
    full-size tensors). For S = 8192, where the full chain is minutes of host work."""
    si = stage_inputs or {}
    f = lambda t: t.detach().to("cpu", torch.float32)
    S = x.shape[0]
    sel = (lambda t: t) if rows is None else (lambda t: t[torch.as_tensor(rows, dtype=torch.long)])
    out = {}
    qkv = f(si.get("qkv_in", x)) @ f(w_qkv)
    out["qkv"] = sel(qkv)
    qkv_used = f(si.get("attn_in", qkv.half()))
    q = qkv_used[:, : n_q * d].reshape(S, n_q, d).permute(1, 0, 2)[None]
    k = qkv_used[:, n_q * d: (n_q + n_kv) * d].reshape(S, n_kv, d).permute(1, 0, 2)[None]
    v = qkv_used[:, (n_q + n_kv) * d:].reshape(S, n_kv, d).permute(1, 0, 2)[None]
    o, lse = attention_ref(q, k, v, causal=True, q_rows=rows)
    out["attn"] = o
    out["attn_lse"] = lse
    attn_used = f(si["oproj_in"])[:, :, torch.as_tensor(rows, dtype=torch.long)] if ("oproj_in" in si and rows is not None) \
        else f(si.get("oproj_in", o.half()))
    a2 = attn_used[0].permute(1, 0, 2).reshape(-1, n_q * d)
    out["oproj"] = a2 @ f(w_o)
    gu = sel(f(si["gu_in"])) @ f(w_gu) if "gu_in" in si else f(out["oproj"].half()) @ f(w_gu)
    out["gate_up"] = gu
    gu_used = sel(f(si["act_in"])) if "act_in" in si else f(gu.half())
    ffn = w_gu.shape[1] // 2
    act = torch.nn.functional.silu(gu_used[:, :ffn]) * gu_used[:, ffn:]
    out["act"] = act
    out["down"] = (sel(f(si["down_in"])) if "down_in" in si else f(act.half())) @ f(w_d)
    return out


# ---------------------------------------------------------------------------------------------------------------
# Layer glue of the in-model path (benchmarks/flashattn-cuda/modeling_llama.py)
# ---------------------------------------------------------------------------------------------------------------
def _f32(t):
    return t.detach().to("cpu", torch.float32)


def rmsnorm_ref(x, weight, eps=1e-5, residual=None, round_residual=True):
    """modeling_llama.py:95-100 in fp32: weight * h * rsqrt(mean(h^2) + eps). With `residual`, h = fp16(residual + x)
    (the fp16 add of :776 / :781; round_residual=False keeps the sum in fp32) and the new residual h is returned too.
    Returns fp32 (out, h)."""
    h = _f32(x)
    if residual is not None:
        h = h + _f32(residual)
        if round_residual:
            h = h.to(torch.float16).float()
    var = h.pow(2).mean(-1, keepdim=True)
    return _f32(weight) * (h * torch.rsqrt(var + eps)), h


def rope_tables(n_positions, dim=128, base=10000.0):
    """cos / sin [n_positions, dim/2] fp32: inv_freq = base^(-2i/dim) (:113), angle = position * inv_freq (:128-131).
    The reference concatenates the table with itself to width dim (:129); both halves are equal, one is kept."""
    inv_freq = 1.0 / (base ** (torch.arange(0, dim, 2, dtype=torch.int64).float() / dim))
    ang = torch.arange(n_positions, dtype=torch.float32)[:, None] * inv_freq[None, :]
    return ang.cos(), ang.sin()


def rope_ref(x, cos, sin, positions):
    """x [B, H, S, D], positions [B, S] -> x * cos + rotate_half(x) * sin in fp32 (:164-168, :193-194)."""
    x = _f32(x)
    half = x.shape[-1] // 2
    c = cos[positions.long()][:, None]          # [B, 1, S, D/2]
    s_ = sin[positions.long()][:, None]
    c = torch.cat((c, c), -1)
    s_ = torch.cat((s_, s_), -1)
    rot = torch.cat((-x[..., half:], x[..., :half]), -1)
    return x * c + rot * s_


def silu_mul_ref(gate_up):
    """[rows, 2F] -> silu(gate) * up in fp32 (:227 with gate and up side by side)."""
    g = _f32(gate_up)
    F = g.shape[-1] // 2
    return torch.nn.functional.silu(g[..., :F]) * g[..., F:]


def llama_decoder_layer_ref(x, w, positions, n_q, n_kv, eps=1e-5, rope_base=10000.0, past_k=None, past_v=None,
                            round_stages=True, rows=None):
    """One Llama decoder layer in fp32 on the CPU. x [B, S, H]; w: dict with nn.Linear-layout ([out, in]) weights
    'q', 'k', 'v', 'o', 'gate', 'up', 'down' and norm weights 'ln1', 'ln2'; positions [B, S]; past_k / past_v
    [B, n_kv, P, D] (already rotated keys). Follows LlamaDecoderLayer.forward (:755-781) and
    LlamaSdpaAttention.forward (:652-704); attention is causal with the mask aligned bottom-right (prefill: P = 0;
    generation step: S = 1). round_stages rounds every intermediate to fp16 where an fp16 pipeline stores it, so a
    kernel chain is compared against the same sequence of roundings. Returns (out fp32 [B,S,H], k, v) with k, v the
    updated caches [B, n_kv, P+S, D] fp32. rows (1-D index tensor): `out` holds only these token rows [B,len(rows),H]
    (keys and values are still formed for every token; queries, attention and everything after it only for `rows`)."""
    r = (lambda t: t.to(torch.float16).float()) if round_stages else (lambda t: t)
    x = _f32(x)
    B, S, H = x.shape
    D = w["q"].shape[0] // n_q
    h1, _ = rmsnorm_ref(x, w["ln1"], eps)
    h1 = r(h1)
    if rows is not None:
        rows = torch.as_tensor(rows, dtype=torch.long)
    Sr = S if rows is None else len(rows)
    h1q = h1 if rows is None else h1[:, rows]
    pos_q = positions if rows is None else positions[:, rows]
    q = r(h1q @ _f32(w["q"]).T).view(B, Sr, n_q, D).transpose(1, 2)
    k = r(h1 @ _f32(w["k"]).T).view(B, S, n_kv, D).transpose(1, 2)
    v = r(h1 @ _f32(w["v"]).T).view(B, S, n_kv, D).transpose(1, 2)
    n_pos = int(positions.max()) + 1
    cos, sin = rope_tables(n_pos, D, rope_base)
    q = r(rope_ref(q, cos, sin, pos_q))
    k = r(rope_ref(k, cos, sin, positions))
    if past_k is not None:
        k = torch.cat((_f32(past_k), k), 2)
        v = torch.cat((_f32(past_v), v), 2)
    if rows is None:
        o, _ = attention_ref(q, k, v, causal=True)
    else:   # the sampled queries keep their place in the S-row causal problem
        qfull = torch.zeros((B, n_q, S, D), dtype=torch.float32)
        qfull[:, :, rows] = q
        o, _ = attention_ref(qfull, k, v, causal=True, q_rows=rows)
    o = r(o).transpose(1, 2).reshape(B, Sr, n_q * D)
    attn = r(o @ _f32(w["o"]).T)
    h2, res = rmsnorm_ref(attn, w["ln2"], eps, residual=x if rows is None else x[:, rows], round_residual=round_stages)
    h2 = r(h2)
    gu = r(torch.cat((h2 @ _f32(w["gate"]).T, h2 @ _f32(w["up"]).T), -1))
    act = r(silu_mul_ref(gu))
    down = r(act @ _f32(w["down"]).T)
    out = (res + down)
    return (r(out) if round_stages else out), k, v


# ---------------------------------------------------------------------------------------------------------------
# seeded synthetic inputs of the benchmark configurations (generated on the CPU, rounded to fp16)
# ---------------------------------------------------------------------------------------------------------------
def randn_fp16(shape, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(torch.float16)


def gemm_inputs(M, N, K, seed=0, a_std=1.0, b_std=1.0):
    g = torch.Generator().manual_seed(seed)
    a = (torch.randn((M, K), generator=g, dtype=torch.float32) * a_std).to(torch.float16)
    b = (torch.randn((K, N), generator=g, dtype=torch.float32) * b_std).to(torch.float16)
    return a, b


def fmha_inputs(B, Hq, Hkv, Sq, Sk, D=128, seed=42, std=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn((B, Hq, Sq, D), generator=g, dtype=torch.float32) * std).to(torch.float16)
    k = (torch.randn((B, Hkv, Sk, D), generator=g, dtype=torch.float32) * std).to(torch.float16)
    v = (torch.randn((B, Hkv, Sk, D), generator=g, dtype=torch.float32) * std).to(torch.float16)
    return q, k, v

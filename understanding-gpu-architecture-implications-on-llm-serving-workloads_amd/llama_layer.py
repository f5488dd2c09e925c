"""A Llama decoder layer on the MI355X kernels: the in-model caller of fine_fmha, rebuilt without its copies.

The reference measures its attention kernels inside a patched Hugging Face layer
(benchmarks/flashattn-cuda/modeling_llama.py): LlamaSdpaAttention.forward (:652-704) projects with three nn.Linear
calls, transposes to [B, H, S, D], applies RoPE, expands K/V with repeat_kv (:670-671), calls
``fmha_unified.ops.fine_fmha`` (:687-690), transposes back with a copy (:700) and projects; LlamaDecoderLayer.forward
(:755-781) wraps it in RMSNorm, residual adds and the gate/up/down MLP (:227), all as separate PyTorch kernels.

Here one layer is eight launches, with or without a KV cache, prefill and generation step alike (one more for 17..64 token
rows, where the gate/up epilogue does not apply and SiLU*up runs on its own), with no layout copies:
    rmsnorm -> QKV GEMM (one fused NT GEMM on the nn.Linear weights) -> RoPE in place on the q and k heads of the
    projection (k goes straight into the KV cache when there is one) -> attention reading q, k, v where they lie
    (strided operands, GQA inside the kernel, output written as [B, S, Hq*D]) -> O projection with the residual
    added in its epilogue -> rmsnorm -> gate/up GEMM with SiLU(gate)*up applied in its epilogue -> down GEMM with the
    residual added in its epilogue.
Weights keep the nn.Linear layout ([out_features, in_features]); nothing is transposed or repacked beyond
concatenating q/k/v and interleaving gate/up along the output dimension once at construction.
"""
import torch

import mi355_serving as lib

__all__ = ["FineKVCache", "FineLlamaDecoderLayer", "rope_tables"]


def rope_tables(n_positions, head_dim=128, base=10000.0, device="cuda"):
    """cos, sin [n_positions, head_dim / 2] fp32 (LlamaRotaryEmbedding, modeling_llama.py:113,119-132)."""
    inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))
    ang = torch.arange(n_positions, dtype=torch.float32)[:, None] * inv_freq[None, :]
    return ang.cos().contiguous().to(device), ang.sin().contiguous().to(device)


class FineKVCache:
    """Static key/value cache of one layer: one tensor [B, 2 * n_kv, max_len, 128], head-major (the keys of a (sequence, head)
    are one contiguous stream for the generation-step attention, which reads them from HBM 3 us faster at batch 8 over 8192
    keys than 256-byte pieces 4 KiB apart), key heads followed by value heads, so one kernel launch files both. `k` and
    `v` are [B, max_len, n_kv, 128] views of it that the attention kernel reads in place; `rows(past, S)` is the
    [B, S, 2 * n_kv, 128] view of S new tokens."""

    def __init__(self, batch, max_len, n_kv, head_dim=128, device="cuda", dtype=torch.float16):
        self.kv = torch.empty((batch, 2 * n_kv, max_len, head_dim), dtype=dtype, device=device)
        self.k = self.kv[:, :n_kv].transpose(1, 2)
        self.v = self.kv[:, n_kv:].transpose(1, 2)
        self.length = 0

    @property
    def max_len(self):
        return self.kv.shape[2]

    def rows(self, past, S):
        return self.kv[:, :, past:past + S].transpose(1, 2)


class FineLlamaDecoderLayer:
    """forward(hidden_states [B, S, H], position_ids [B, S]) -> [B, S, H]; causal attention over the cache (if any)
    plus the new tokens. `weights`: dict of GPU tensors in nn.Linear layout: q, k, v, o, gate, up, down, and the norm
    weights ln1, ln2. `dtype` (float16 or bfloat16) is the type of the weights, activations and KV cache."""

    def __init__(self, weights, n_q_heads, n_kv_heads, rms_eps=1e-5, rope_base=10000.0, max_positions=8192,
                 dtype=torch.float16):
        if dtype not in (torch.float16, torch.bfloat16):
            raise ValueError("dtype must be float16 or bfloat16")
        self.dtype = dtype
        w = {k: v.detach().to(dtype).contiguous() for k, v in weights.items()}
        self.n_q, self.n_kv = int(n_q_heads), int(n_kv_heads)
        self.hidden = w["q"].shape[1]
        self.head_dim = w["q"].shape[0] // self.n_q
        if self.head_dim != 128:
            raise ValueError("head_dim must be 128, got %d" % self.head_dim)
        self.inter = w["gate"].shape[0]
        self.w_qkv = torch.cat((w["q"], w["k"], w["v"]), 0).contiguous()   # [(Hq + 2 Hkv) * D, H]
        self.w_o = w["o"]                                                  # [H, Hq * D]
        # gate and up rows interleaved in groups of 32, so the GEMM epilogue can apply silu(gate) * up to its accumulators
        self.gu_block = lib.GATE_UP_BLOCK if self.inter % lib.GATE_UP_BLOCK == 0 else 0
        self.w_gu = (lib.interleave_gate_up(w["gate"], w["up"]) if self.gu_block
                     else torch.cat((w["gate"], w["up"]), 0).contiguous())   # [2 F, H]
        self.w_d = w["down"]                                               # [H, F]
        self.ln1, self.ln2 = w["ln1"], w["ln2"]
        self.eps = float(rms_eps)
        self.cos, self.sin = rope_tables(max_positions, self.head_dim, rope_base, device=self.w_o.device)
        self.all_positions = torch.arange(max_positions, dtype=torch.int32, device=self.w_o.device)
        self.attn_ms = {"prefill": [], "decode": []}  # filled when time_attention=True (modeling_llama.py:762-775)

    @classmethod
    def from_hf(cls, hf_layer, config, max_positions=8192, device="cuda", dtype=torch.float16):
        """Wrap the weights of a transformers LlamaDecoderLayer."""
        a, m = hf_layer.self_attn, hf_layer.mlp
        w = dict(q=a.q_proj.weight, k=a.k_proj.weight, v=a.v_proj.weight, o=a.o_proj.weight, gate=m.gate_proj.weight,
                 up=m.up_proj.weight, down=m.down_proj.weight, ln1=hf_layer.input_layernorm.weight,
                 ln2=hf_layer.post_attention_layernorm.weight)
        w = {k: v.detach().to(device) for k, v in w.items()}
        base = getattr(config, "rope_theta", None) or (getattr(config, "rope_parameters", None) or {}).get("rope_theta", 10000.0)
        return cls(w, config.num_attention_heads, config.num_key_value_heads, config.rms_norm_eps, base, max_positions, dtype)

    def forward(self, hidden_states, position_ids=None, kv_cache=None, time_attention=False):
        B, S, H = hidden_states.shape
        D, Hq, Hkv = self.head_dim, self.n_q, self.n_kv
        x = hidden_states.reshape(B * S, H)
        past = kv_cache.length if kv_cache is not None else 0
        if position_ids is None:
            pos = self.all_positions[past:past + S]   # one [S] table shared by every batch row, no kernel launched
        else:
            pos = position_ids.to(torch.int32).contiguous()

        h1 = lib.rmsnorm(x, self.ln1, self.eps)
        if time_attention:
            torch.cuda.synchronize()
            t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0.record()
        qkv = lib.hgemm(h1, self.w_qkv, "NT").view(B, S, Hq + 2 * Hkv, D)
        q = qkv[:, :, :Hq]
        if kv_cache is None:
            lib.rope(qkv[:, :, :Hq + Hkv], self.cos, self.sin, pos)           # q and k heads are adjacent
            k, v = qkv[:, :, Hq:Hq + Hkv], qkv[:, :, Hq + Hkv:]
        else:
            if past + S > kv_cache.max_len:
                raise ValueError("KV cache of %d tokens cannot take %d more after %d" % (kv_cache.max_len, S, past))
            # one launch: q rotated in place, rotated keys and plain values of the new tokens into the cache
            lib.rope_qkv(qkv, kv_cache.rows(past, S), self.cos, self.sin, pos, Hq, Hkv)
            kv_cache.length = past + S
            k, v = kv_cache.k[:, :past + S], kv_cache.v[:, :past + S]
        attn = torch.empty((B, S, Hq, D), dtype=self.dtype, device=x.device)
        # [B, S, heads, D] viewed as [B, heads, S, D]: the kernel reads and writes these layouts in place
        lib.fmha_fwd(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), causal=True, return_lse=False,
                     out=attn.transpose(1, 2))
        res = lib.hgemm(attn.view(B * S, Hq * D), self.w_o, "NT", residual=x)   # x + o_proj(attn)
        if time_attention:
            t1.record()
            torch.cuda.synchronize()
            self.attn_ms["decode" if (S == 1 and past > 0) else "prefill"].append(t0.elapsed_time(t1))
        h2 = lib.rmsnorm(res, self.ln2, self.eps)
        act = lib.hgemm_silu_mul(h2, self.w_gu, "NT") if self.gu_block else lib.silu_mul(lib.hgemm(h2, self.w_gu, "NT"))
        return lib.hgemm(act, self.w_d, "NT", out=res, residual=res).view(B, S, H)   # res + down_proj(act), in place

    __call__ = forward

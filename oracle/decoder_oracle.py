"""CPU restatement of the reference's Qwen2-style decoder around the W4A32 Linear oracle.

TEST INFRASTRUCTURE ONLY: tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may use
it as the checker; the product never imports it.

Follows (reference tree):
  mllm/Models/ds_qwen2/modeling_ds_qwen2.hpp:47-54   MLP: down(silu(gate(x)) * up(x))
  mllm/Models/ds_qwen2/modeling_ds_qwen2.hpp:106-155 attention: q,k,v Linear, RoPE, KV cache,
                                                     softmax(q k^T / sqrt(D)) v with a causal mask, o Linear
  mllm/Models/ds_qwen2/modeling_ds_qwen2.hpp:175-183 block: x + attn(norm(x)); + mlp(norm(.))
  mllm/Models/ds_qwen2/modeling_ds_qwen2.hpp:202-215 model: embedding, blocks, norm, lm_head
  mllm/Backends/Arm/Ops/RMSNormOp.cpp:36-76          y = x * (w * 1/sqrt(mean(x^2) + eps))
  mllm/Backends/Arm/Kernels/rope.cpp:20-80           half-split RoPE, theta = pos / base^(2d/D)
  mllm/Models/AutoLLM.hpp:70-88                      greedy: first maximum

Every operator here is a textbook routine in float32 numpy; the parity tests compare the HIP
operators one by one against torch's own float32 operators as well. Linears go through the scalar
oracle (w4a32_oracle.linear). lm_head is either quantised like the other Linears (the benchmark
configuration) or, with lm_head_dense=True, applied as the reference applies it: a dense matmul with
transpose_b on the f32 / f16 tensor (modeling_ds_qwen2.hpp:209-213), here numpy's float64 product.
"""
import numpy as np

import w4a32_oracle as orc

F = np.float32


def rmsnorm(x, w, eps):
    x = x.astype(F)
    ms = (x.astype(np.float64) ** 2).mean(axis=-1, keepdims=True)
    rstd = (1.0 / np.sqrt(ms + eps)).astype(F)
    return (x * (w.astype(F) * rstd)).astype(F)


def rope_tables(max_pos, dim, base):
    d = np.arange(dim // 2, dtype=F)
    inv = (F(1.0) / np.power(F(base), F(2.0) * d / F(dim))).astype(F)
    theta = (inv[None, :] * np.arange(max_pos, dtype=F)[:, None]).astype(F)
    return np.sin(theta).astype(F), np.cos(theta).astype(F)


def rope(x, sin, cos, pos0):
    """x [M][H][D] -> rotated copy; row m sits at position pos0 + m."""
    M, H, D = x.shape
    half = D // 2
    s = sin[pos0:pos0 + M, None, :]
    c = cos[pos0:pos0 + M, None, :]
    x0, x1 = x[..., :half], x[..., half:]
    return np.concatenate([x0 * c - x1 * s, x0 * s + x1 * c], axis=-1).astype(F)


def attention(q, kc, vc, pos0):
    """q [M][Hq][D]; kc, vc [Hkv][len][D] holding positions 0..pos0+M-1. -> [M][Hq*D]"""
    M, Hq, D = q.shape
    Hkv = kc.shape[0]
    rep = Hq // Hkv
    out = np.empty((M, Hq, D), dtype=F)
    scale = F(1.0 / np.sqrt(D))
    for m in range(M):
        n = pos0 + m + 1
        for h in range(Hq):
            k = kc[h // rep, :n].astype(np.float64)
            v = vc[h // rep, :n].astype(np.float64)
            s = (k @ q[m, h].astype(np.float64)) * scale
            p = np.exp(s - s.max())
            out[m, h] = (p @ v / p.sum()).astype(F)
    return out.reshape(M, Hq * D)


def silu_mul(g, u):
    g64 = g.astype(np.float64)
    return (g64 / (1.0 + np.exp(-g64)) * u).astype(F)


class Linear:
    """One W4A32 Linear: quantised once by the oracle's quantiser, applied by the oracle's matmul."""

    threads = 1   # of the C matmul (rows x columns dealt to threads: same results); tests at full shapes raise it

    def __init__(self, w, bias=None):
        self.n, self.k = w.shape
        self.u4, self.scales = orc.quant_rhs(np.ascontiguousarray(w, dtype=F))
        self.bias = None if bias is None else np.ascontiguousarray(bias, dtype=F)

    def __call__(self, x):
        return orc.linear(np.ascontiguousarray(x, dtype=F), self.u4, self.scales, bias=self.bias,
                          threads=Linear.threads)


class Decoder:
    """weights: dict with embedding [V][H], final_norm [H], lm_head [V][H] and layers = list of dicts
    (q,k,v,o,gate,up,down f32 [out][in]; q_bias,k_bias,v_bias optional; attn_norm, ffn_norm)."""

    def __init__(self, weights, n_heads, n_kv_heads, head_dim=128, rope_theta=1e6, rms_eps=1e-6, max_seq=1024,
                 lm_head_dense=False):
        self.w = weights
        self.Hq, self.Hkv, self.D = n_heads, n_kv_heads, head_dim
        self.eps = rms_eps
        self.sin, self.cos = rope_tables(max_seq, head_dim, rope_theta)
        self.layers = []
        for lw in weights["layers"]:
            self.layers.append({
                "q": Linear(lw["q"], lw.get("q_bias")), "k": Linear(lw["k"], lw.get("k_bias")),
                "v": Linear(lw["v"], lw.get("v_bias")), "o": Linear(lw["o"]),
                "gate": Linear(lw["gate"]), "up": Linear(lw["up"]), "down": Linear(lw["down"]),
                "attn_norm": lw["attn_norm"], "ffn_norm": lw["ffn_norm"],
            })
        if lm_head_dense:
            dense = np.asarray(weights["lm_head"]).astype(np.float64)   # f16 or f32 values, widened exactly
            self.lm_head = lambda x: (x.astype(np.float64) @ dense.T).astype(F)
        else:
            self.lm_head = Linear(weights["lm_head"])
        self.kc = [np.zeros((n_kv_heads, max_seq, head_dim), dtype=F) for _ in self.layers]
        self.vc = [np.zeros((n_kv_heads, max_seq, head_dim), dtype=F) for _ in self.layers]
        self.pos = 0

    def forward(self, tokens):
        """Appends the tokens at the current position; returns the last row's logits [V]."""
        tokens = np.asarray(tokens, dtype=np.int64)
        M, pos0 = len(tokens), self.pos
        h = self.w["embedding"][tokens].astype(F)
        for l, L in enumerate(self.layers):
            x = rmsnorm(h, L["attn_norm"], self.eps)
            q = L["q"](x).reshape(M, self.Hq, self.D)
            k = L["k"](x).reshape(M, self.Hkv, self.D)
            v = L["v"](x).reshape(M, self.Hkv, self.D)
            q = rope(q, self.sin, self.cos, pos0)
            k = rope(k, self.sin, self.cos, pos0)
            self.kc[l][:, pos0:pos0 + M] = k.transpose(1, 0, 2)
            self.vc[l][:, pos0:pos0 + M] = v.transpose(1, 0, 2)
            a = attention(q, self.kc[l], self.vc[l], pos0)
            h = (h + L["o"](a)).astype(F)
            x = rmsnorm(h, L["ffn_norm"], self.eps)
            h = (h + L["down"](silu_mul(L["gate"](x), L["up"](x)))).astype(F)
        self.pos += M
        x = rmsnorm(h[-1:], self.w["final_norm"], self.eps)
        return self.lm_head(x)[0]


def greedy(logits):
    """AutoLLM.hpp:70-88: strict '>' scan from -1e10, so the first maximum wins."""
    best, pos = F(-1e10), 0
    for i, v in enumerate(logits):
        if v > best:
            best, pos = v, i
    return pos

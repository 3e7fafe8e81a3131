"""CPU: the numpy restatement of the decoder operators against facts that do not depend on it:
torch's own float32 operators, invariants of a rotation, and tiny hand-made cases."""
import numpy as np
import pytest
import torch

import decoder_oracle as do


def test_rmsnorm_matches_torch_formula():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 96)).astype(np.float32)
    w = rng.standard_normal(96).astype(np.float32)
    ref = torch.nn.functional.rms_norm(torch.from_numpy(x), (96,), torch.from_numpy(w), eps=1e-6).numpy()
    assert np.allclose(do.rmsnorm(x, w, 1e-6), ref, rtol=2e-6, atol=1e-7)
    # closed form: a constant row c has mean square c^2 -> y = sign(c) * w (eps negligible)
    y = do.rmsnorm(np.full((1, 8), -3.0, np.float32), np.arange(8, dtype=np.float32), 0.0)
    assert np.allclose(y[0], -np.arange(8))


def test_rope_is_a_rotation_with_relative_phase():
    sin, cos = do.rope_tables(64, 128, 1e6)
    assert np.all(sin[0] == 0) and np.all(cos[0] == 1)
    # pair (d, d + 64) turns by pos * base^(-2d/128): d = 0 turns by pos radians
    assert np.allclose(sin[3, 0], np.sin(3.0), atol=1e-6) and np.allclose(cos[3, 0], np.cos(3.0), atol=1e-6)
    assert np.allclose(sin[5, 32], np.sin(5.0 / 1e6 ** 0.5), atol=1e-7)
    rng = np.random.default_rng(1)
    q = rng.standard_normal((1, 1, 128)).astype(np.float32)
    k = rng.standard_normal((1, 1, 128)).astype(np.float32)
    assert np.array_equal(do.rope(q, sin, cos, 0), q)                        # position 0: identity
    for p in (1, 7, 40):
        assert np.allclose(np.linalg.norm(do.rope(q, sin, cos, p)), np.linalg.norm(q), rtol=1e-5)
    # q at position a, k at position b: the product depends on a - b only
    d1 = (do.rope(q, sin, cos, 9) * do.rope(k, sin, cos, 4)).sum()
    d2 = (do.rope(q, sin, cos, 25) * do.rope(k, sin, cos, 20)).sum()
    assert np.allclose(d1, d2, rtol=1e-4, atol=1e-4)
    # the half-split convention (not interleaved): a unit vector at d = 0 moves into d = 64
    e = np.zeros((1, 1, 128), np.float32)
    e[0, 0, 0] = 1.0
    r = do.rope(e, sin, cos, 2)
    assert np.allclose(r[0, 0, 0], np.cos(2.0), atol=1e-6) and np.allclose(r[0, 0, 64], np.sin(2.0), atol=1e-6)


def test_attention_matches_torch_sdpa_with_gqa_and_causal_mask():
    rng = np.random.default_rng(2)
    M, Hq, Hkv, D, pos0 = 5, 4, 2, 128, 3
    q = rng.standard_normal((M, Hq, D)).astype(np.float32)
    kc = rng.standard_normal((Hkv, pos0 + M, D)).astype(np.float32)
    vc = rng.standard_normal((Hkv, pos0 + M, D)).astype(np.float32)
    got = do.attention(q, kc, vc, pos0).reshape(M, Hq, D)
    tq = torch.from_numpy(q).permute(1, 0, 2)[None]                                  # [1][Hq][M][D]
    tk = torch.from_numpy(kc).repeat_interleave(Hq // Hkv, dim=0)[None]              # head h -> kv head h // 2
    tv = torch.from_numpy(vc).repeat_interleave(Hq // Hkv, dim=0)[None]
    mask = torch.ones(M, pos0 + M, dtype=torch.bool).tril(diagonal=pos0)             # query m sees keys 0..pos0+m
    ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=mask)[0].permute(1, 0, 2)
    assert np.allclose(got, ref.numpy(), rtol=1e-5, atol=1e-6)
    # a single key: the output is that key's value row, whatever the score
    one = do.attention(q[:1], kc[:, :1], vc[:, :1], 0).reshape(Hq, D)
    assert np.allclose(one[0], vc[0, 0]) and np.allclose(one[3], vc[1, 0])


def test_silu_mul_and_greedy():
    g = np.array([-20.0, -1.0, 0.0, 1.0, 20.0], np.float32)
    u = np.array([2.0, 2.0, 2.0, 2.0, 2.0], np.float32)
    ref = (torch.nn.functional.silu(torch.from_numpy(g)) * torch.from_numpy(u)).numpy()
    assert np.allclose(do.silu_mul(g, u), ref, rtol=1e-6, atol=1e-9)
    assert do.greedy(np.array([0.5, 2.0, 2.0, -1.0], np.float32)) == 1     # first maximum
    assert do.greedy(np.array([-3.0, -2.0], np.float32)) == 1
    assert do.greedy(np.full(4, -np.inf, np.float32)) == 0                   # nothing beats -1e10


def test_decoder_forward_is_consistent_between_prefill_and_steps(orc):
    """Feeding a prompt at once or token by token gives the same logits (the KV cache and the
    causal mask agree), up to the row quantiser seeing the same rows: the Linears act per row."""
    rng = np.random.default_rng(3)
    H, Hq, Hkv, I, V, Lyr = 256, 2, 1, 384, 160, 2

    def w(n, k):
        return (rng.standard_normal((n, k)) * 0.05).astype(np.float32)

    weights = {"embedding": rng.standard_normal((V, H)).astype(np.float32), "lm_head": w(V, H),
               "final_norm": (1 + 0.1 * rng.standard_normal(H)).astype(np.float32), "layers": []}
    for _ in range(Lyr):
        weights["layers"].append({
            "q": w(Hq * 128, H), "k": w(Hkv * 128, H), "v": w(Hkv * 128, H), "o": w(H, Hq * 128),
            "gate": w(I, H), "up": w(I, H), "down": w(H, I),
            "q_bias": (0.1 * rng.standard_normal(Hq * 128)).astype(np.float32),
            "attn_norm": np.ones(H, np.float32), "ffn_norm": np.ones(H, np.float32)})
    toks = [3, 17, 100, 42, 7]
    a = do.Decoder(weights, Hq, Hkv, max_seq=16)
    la = a.forward(toks)
    b = do.Decoder(weights, Hq, Hkv, max_seq=16)
    for t in toks:
        lb = b.forward([t])
    assert a.pos == b.pos == 5
    assert np.allclose(la, lb, rtol=1e-4, atol=1e-5)

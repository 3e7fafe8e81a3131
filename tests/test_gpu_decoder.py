"""GPU: the decoder operators against torch's float32 operators, and the decoder runner against the
CPU oracle (teacher-forced with the runner's own tokens so both see the same history).

Tolerances (f32 operators, different summation order only): 1e-5 relative for the elementwise and
normalisation operators, 2e-5 for attention; whole-model logits 2e-3 max-abs-rel (every Linear
re-quantises its input rows to int8, so a last-bit difference upstream can flip a quantised value)."""
import numpy as np
import pytest
import torch

from conftest import make_weights, max_abs_rel

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_embedding_rmsnorm_add_silu(pkg):
    g = torch.Generator(device="cuda").manual_seed(0)
    table = torch.randn((300, 256), generator=g, device="cuda")
    ids = torch.tensor([5, 299, 0, 17, 1000, -4], dtype=torch.int64, device="cuda")   # the last two are clamped
    out = pkg.op_embedding(ids, table)
    assert torch.equal(out, table[ids.clamp(0, 299)])

    for M, D in [(1, 1536), (7, 1536), (3, 8960), (2, 96)]:
        h = torch.randn((M, D), generator=g, device="cuda") * 3
        d = torch.randn((M, D), generator=g, device="cuda")
        w = 1 + 0.1 * torch.randn((D,), generator=g, device="cuda")
        y = pkg.op_rmsnorm(h, w, 1e-6)
        ref = torch.nn.functional.rms_norm(h, (D,), w, eps=1e-6)
        assert max_abs_rel(y.cpu().numpy(), ref.cpu().numpy()) < 1e-5
        h2, y2 = pkg.op_rmsnorm(h, w, 1e-6, delta=d)
        assert torch.equal(h2, h + d)
        assert max_abs_rel(y2.cpu().numpy(), torch.nn.functional.rms_norm(h + d, (D,), w, eps=1e-6).cpu().numpy()) < 1e-5

    a = torch.randn((4, 8960), generator=g, device="cuda") * 4
    b = torch.randn((4, 8960), generator=g, device="cuda")
    assert torch.equal(pkg.op_add(a, b), a + b)
    ref = torch.nn.functional.silu(a) * b
    assert max_abs_rel(pkg.op_silu_mul(a, b).cpu().numpy(), ref.cpu().numpy()) < 1e-5


@pytest.mark.parametrize("M,K", [(40, 1536), (512, 1536), (33, 8960), (9, 96), (64, 16384)])
def test_fused_row_quantisers_match_separate_operators(pkg, M, K):
    # norm + quantiser and silu*mul + quantiser in one launch against operator, then quantiser
    g = torch.Generator(device="cuda").manual_seed(M + K)
    h = torch.randn((M, K), generator=g, device="cuda") * 2
    d = torch.randn((M, K), generator=g, device="cuda")
    w = 1 + 0.1 * torch.randn((K,), generator=g, device="cuda")
    for delta in (None, d):
        ws, h_out = pkg.quant_lhs_norm(h, w, 1e-6, delta=delta)
        if delta is None:
            y = pkg.op_rmsnorm(h, w, 1e-6)
        else:
            h_ref, y = pkg.op_rmsnorm(h, w, 1e-6, delta=delta)
            assert torch.equal(h_out, h_ref)
        aq, recip, nzp = pkg.export_lhs(ws, M, K)
        aq0, recip0, nzp0 = pkg.export_lhs(pkg.quant_lhs(y), M, K)
        # the sum of squares is taken in another order: the normalised row may differ in its last
        # bit, which moves a value that sits on a rounding boundary by one step
        assert torch.allclose(recip, recip0, rtol=1e-6, atol=0)
        assert int((nzp - nzp0).abs().max()) <= 1
        diff = (aq.int() - aq0.int()).abs()
        assert int(diff.max()) <= 1 and float((diff > 0).float().mean()) < 2e-3
        deq = (aq.float() + nzp.float()[:, None]) * recip[:, None]
        assert float((deq - y).abs().max()) <= 1.01 * float(recip.max())
    gate = torch.randn((M, K), generator=g, device="cuda") * 3
    up = torch.randn((M, K), generator=g, device="cuda")
    a1 = pkg.export_lhs(pkg.quant_lhs_silu_mul(gate, up), M, K)
    a0 = pkg.export_lhs(pkg.quant_lhs(pkg.op_silu_mul(gate, up)), M, K)
    for x1, x0 in zip(a1, a0):
        assert torch.equal(x1, x0)          # elementwise: the same arithmetic, bit for bit


@pytest.mark.parametrize("M,K,N,bias", [(512, 8960, 1536, False), (100, 6144, 288, True), (16, 8960, 1536, True),
                                          (1100, 6208, 1536, False)])
def test_split_k_parts_summed_by_the_norm_quantiser(pkg, M, K, N, bias):
    # down_proj split over K whose parts are added up by the next residual add + RMSNorm + quantiser,
    # against the same three steps with the reduction kernel in between
    g = torch.Generator(device="cuda").manual_seed(M + N)
    packed = pkg.quant_pack_rhs(torch.randn((N, K), generator=g, device="cuda") * 0.05,
                                torch.randn((N,), generator=g, device="cuda") if bias else None)
    ws_in = pkg.quant_lhs(torch.randn((M, K), generator=g, device="cuda"))
    h = torch.randn((M, N), generator=g, device="cuda") * 2
    w = 1 + 0.1 * torch.randn((N,), generator=g, device="cuda")
    delta = pkg.matmul_quantized_splitk(ws_in, packed, M, K, N)
    ws0, h0 = pkg.quant_lhs_norm(h, w, 1e-6, delta=delta)
    scratch, parts = pkg.matmul_quantized_splitk_parts(ws_in, packed, M, K, N)
    assert parts > 1
    ws1, h1 = pkg.quant_lhs_norm_parts(h, scratch, parts, packed, K, w, 1e-6)
    # the factors of the output transform are applied before the parts are added instead of after
    assert float((h1 - h0).abs().max()) <= 2e-6 * float(delta.abs().max())
    aq0, recip0, nzp0 = pkg.export_lhs(ws0, M, N)
    aq1, recip1, nzp1 = pkg.export_lhs(ws1, M, N)
    assert torch.allclose(recip1, recip0, rtol=1e-5, atol=0)
    assert int((nzp1 - nzp0).abs().max()) <= 1
    diff = (aq1.int() - aq0.int()).abs()
    assert int(diff.max()) <= 1 and float((diff > 0).float().mean()) < 5e-3
    # a problem the library does not split has no parts to hand over
    small = pkg.quant_pack_rhs(torch.randn((64, 256), generator=g, device="cuda"))
    with pytest.raises(RuntimeError):
        pkg.matmul_quantized_splitk_parts(pkg.quant_lhs(torch.randn((64, 256), generator=g, device="cuda")),
                                          small, 64, 256, 64)


def test_fused_row_quantisers_reject_what_they_do_not_take(pkg):
    h = torch.zeros((8, 64), device="cuda")
    w = torch.ones((64,), device="cuda")
    with pytest.raises(RuntimeError):
        pkg.quant_lhs_norm(h, w, 1e-6)                     # decode sizes use w4a32_decode_linear
    big = torch.zeros((16, 16416), device="cuda")
    with pytest.raises(RuntimeError):
        pkg.quant_lhs_silu_mul(big, big)                   # row too long for the register kernel


def test_rope_table_and_kv_append(pkg):
    import decoder_oracle as do

    sin, cos = pkg.op_rope_table(1024, 128, 1e6)
    rs, rc = do.rope_tables(1024, 128, 1e6)
    # The angle itself is a float32 product pos * base^(-2d/D): one ulp of difference in powf is a
    # relative 6e-8 of an angle of up to 1023 rad, i.e. up to ~6e-5 in the sine. Small angles agree closely.
    err_s = float(np.abs(sin.cpu().numpy() - rs).max())
    err_c = float(np.abs(cos.cpu().numpy() - rc).max())
    assert err_s < 1.5e-4 and err_c < 1.5e-4
    assert float(np.abs(sin.cpu().numpy() - rs)[:16].max()) < 2e-6

    rng = np.random.default_rng(1)
    M, Hq, Hkv, D, S, pos0 = 5, 4, 2, 128, 32, 9
    q = rng.standard_normal((M, Hq * D)).astype(np.float32)
    k = rng.standard_normal((M, Hkv * D)).astype(np.float32)
    v = rng.standard_normal((M, Hkv * D)).astype(np.float32)
    kc = torch.zeros((Hkv, S, D), device="cuda")
    vc = torch.zeros((Hkv, S, D), device="cuda")
    dq = dev(q)
    pkg.op_rope_kv(dq, dev(k), dev(v), sin, cos, kc, vc, Hq, Hkv, D, pos0)
    s_np, c_np = sin.cpu().numpy(), cos.cpu().numpy()
    assert np.allclose(dq.cpu().numpy().reshape(M, Hq, D), do.rope(q.reshape(M, Hq, D), s_np, c_np, pos0),
                       rtol=1e-6, atol=1e-6)
    want_k = do.rope(k.reshape(M, Hkv, D), s_np, c_np, pos0).transpose(1, 0, 2)
    assert np.allclose(kc[:, pos0:pos0 + M].cpu().numpy(), want_k, rtol=1e-6, atol=1e-6)
    assert np.array_equal(vc[:, pos0:pos0 + M].cpu().numpy(), v.reshape(M, Hkv, D).transpose(1, 0, 2))
    assert float(kc[:, :pos0].abs().max()) == 0 and float(kc[:, pos0 + M:].abs().max()) == 0
    # position from device memory (what a replayed graph uses)
    d_pos = torch.tensor([pos0], dtype=torch.int32, device="cuda")
    kc2, vc2, dq2 = torch.zeros_like(kc), torch.zeros_like(vc), dev(q)
    pkg.op_rope_kv(dq2, dev(k), dev(v), sin, cos, kc2, vc2, Hq, Hkv, D, 0, d_pos0=d_pos)
    assert torch.equal(kc2, kc) and torch.equal(vc2, vc) and torch.equal(dq2, dq)


@pytest.mark.parametrize("Hq,Hkv", [(12, 2), (4, 4), (2, 1), (3, 1)])
def test_attention_prefill_and_decode(pkg, Hq, Hkv):
    g = torch.Generator(device="cuda").manual_seed(2)
    D, S = 128, 1024
    kc = torch.randn((Hkv, S, D), generator=g, device="cuda")
    vc = torch.randn((Hkv, S, D), generator=g, device="cuda")

    def ref(q, pos0):
        M = q.shape[0]
        tq = q.view(M, Hq, D).permute(1, 0, 2)[None]
        n = pos0 + M
        tk = kc[:, :n].repeat_interleave(Hq // Hkv, dim=0)[None]
        tv = vc[:, :n].repeat_interleave(Hq // Hkv, dim=0)[None]
        mask = torch.ones(M, n, dtype=torch.bool, device="cuda").tril(diagonal=pos0)
        with torch.nn.attention.sdpa_kernel(torch.nn.attention.SDPBackend.MATH):
            o = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=mask)
        return o[0].permute(1, 0, 2).reshape(M, Hq * D)

    # 16 rows and more run on the matrix cores, 256 and more with 8 wavefronts per workgroup
    for M, pos0 in [(1, 0), (5, 0), (70, 0), (33, 100), (130, 0), (256, 0), (300, 200), (512, 512)]:
        q = torch.randn((M, Hq * D), generator=g, device="cuda")
        out = pkg.op_attention(q, kc, vc, Hq, Hkv, D, pos0)
        assert max_abs_rel(out.cpu().numpy(), ref(q, pos0).cpu().numpy()) < 2e-5, (M, pos0)

    # the same operator with scratch lent: up to 128 (head, query block) pairs the keys of a query block go
    # to several workgroups (12 heads: up to 320 rows; 4 heads and fewer: every case here). Positions
    # that are no multiples of 32 leave queries with no visible key in a chunk (97: the chunk that begins
    # at key 128).
    for M, pos0 in [(16, 0), (33, 97), (70, 0), (130, 5), (256, 0), (300, 200), (512, 0), (512, 512),
                    (64, 960), (100, 924)]:
        q = torch.randn((M, Hq * D), generator=g, device="cuda")
        want = ref(q, pos0).cpu().numpy()
        out = pkg.op_attention_prefill(q, kc, vc, Hq, Hkv, D, pos0)
        assert max_abs_rel(out.cpu().numpy(), want) < 2e-5, (M, pos0)
        d_pos = torch.tensor([pos0], dtype=torch.int32, device="cuda")
        assert torch.equal(pkg.op_attention_prefill(q, kc, vc, Hq, Hkv, D, 0, d_pos0=d_pos), out)
        # too little scratch: the operator runs unsplit
        tiny = torch.empty((1024,), dtype=torch.uint8, device="cuda")
        assert torch.equal(pkg.op_attention_prefill(q, kc, vc, Hq, Hkv, D, pos0, part=tiny),
                           pkg.op_attention(q, kc, vc, Hq, Hkv, D, pos0))

    scratch = pkg.op_scratch(Hq)
    for pos in [0, 1, 15, 16, 63, 64, 200, 767, 1023]:     # lengths around the split and chunk sizes
        q = torch.randn((1, Hq * D), generator=g, device="cuda")
        out = pkg.op_attention(q, kc, vc, Hq, Hkv, D, pos, scratch=scratch)
        assert max_abs_rel(out.cpu().numpy(), ref(q, pos).cpu().numpy()) < 2e-5, pos
        d_pos = torch.tensor([pos], dtype=torch.int32, device="cuda")
        out2 = pkg.op_attention(q, kc, vc, Hq, Hkv, D, 0, scratch=scratch, d_pos0=d_pos)
        assert torch.equal(out, out2)
    # the kernels leave the arrival counters cleared
    assert int(scratch[:4 * (Hq + 1)].view(torch.int32).abs().sum()) == 0


@pytest.mark.parametrize("Hq,Hkv", [(12, 2), (4, 4), (3, 1)])
def test_attention_prefill_on_bf16_terms(pkg, Hq, Hkv):
    """The prefill attention with both products on the 16-bit matrix pipe, every f32 operand as three bf16 terms:
    against torch's f32 attention to the same 2e-5 as the f32 kernels, on operands with a wide range of magnitudes
    (the terms keep f32's exponent range), NaN in the cache rows past the last key (they must not reach the sums),
    ragged row counts and positions."""
    g = torch.Generator(device="cuda").manual_seed(3)
    D, S = 128, 1024

    def ref(q, kc, vc, pos0):
        M = q.shape[0]
        tq = q.view(M, Hq, D).permute(1, 0, 2)[None].double()
        n = pos0 + M
        tk = kc[:, :n].repeat_interleave(Hq // Hkv, dim=0)[None].double()
        tv = vc[:, :n].repeat_interleave(Hq // Hkv, dim=0)[None].double()
        mask = torch.ones(M, n, dtype=torch.bool, device="cuda").tril(diagonal=pos0)
        with torch.nn.attention.sdpa_kernel(torch.nn.attention.SDPBackend.MATH):
            o = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=mask)
        return o[0].permute(1, 0, 2).reshape(M, Hq * D)

    for M, pos0, kscale, vscale in [(32, 0, 1.0, 1.0), (70, 0, 1.0, 1.0), (130, 5, 1.0, 1.0), (256, 0, 1.0, 1.0),
                                    (300, 200, 1.0, 1.0), (512, 0, 1.0, 1.0), (512, 512, 1.0, 1.0), (64, 960, 1.0, 1.0),
                                    (100, 924, 1.0, 1.0), (200, 37, 30.0, 1e-6), (160, 0, 1e-4, 3e4)]:
        kc = torch.randn((Hkv, S, D), generator=g, device="cuda") * kscale
        vc = torch.randn((Hkv, S, D), generator=g, device="cuda") * vscale
        # magnitudes spread over many binades inside one row as well
        vc *= torch.exp2(torch.randint(-6, 7, (Hkv, S, D), generator=g, device="cuda").float())
        q = torch.randn((M, Hq * D), generator=g, device="cuda") / max(kscale, 1.0)
        want = ref(q, kc, vc, pos0).cpu().numpy()
        kc[:, pos0 + M:] = float("nan")
        vc[:, pos0 + M:] = float("nan")
        out = pkg.op_attention_prefill_bf16x3(q, kc, vc, Hq, Hkv, D, pos0)
        torch.cuda.synchronize()
        assert max_abs_rel(out.cpu().numpy(), want) < 2e-5, (M, pos0, kscale, vscale)


@pytest.mark.parametrize("Hq,Hkv", [(12, 2), (4, 4), (3, 1)])
def test_rope_attention_prefill_on_bf16_terms_equals_the_two_operators(pkg, Hq, Hkv):
    """RoPE + cache append done by the launch that splits K and V == op_rope_kv, then op_attention_prefill_bf16x3:
    rotated q, both caches (rows outside [pos0, pos0 + M) untouched) and the output, bit for bit; positions that
    start inside a 32-key block, ragged row counts, a prompt that ends at the cache's last row."""
    g = torch.Generator(device="cuda").manual_seed(8)
    D, S = 128, 640
    sin, cos = pkg.op_rope_table(S, D, 1e6)
    for M, pos0 in [(1, 0), (32, 0), (70, 0), (256, 0), (512, 0), (100, 32), (130, 5), (64, 300), (37, 603),
                    (128, 512)]:
        kc = torch.randn((Hkv, S, D), generator=g, device="cuda")
        vc = torch.randn((Hkv, S, D), generator=g, device="cuda")
        q = torch.randn((M, Hq * D), generator=g, device="cuda")
        k = torch.randn((M, Hkv * D), generator=g, device="cuda")
        v = torch.randn((M, Hkv * D), generator=g, device="cuda")
        kc1, vc1, q1 = kc.clone(), vc.clone(), q.clone()
        pkg.op_rope_kv(q1, k, v, sin, cos, kc1, vc1, Hq, Hkv, D, pos0)
        want = pkg.op_attention_prefill_bf16x3(q1, kc1, vc1, Hq, Hkv, D, pos0)
        kc2, vc2, q2 = kc.clone(), vc.clone(), q.clone()
        got = pkg.op_rope_attention_prefill_bf16x3(q2, k, v, sin, cos, kc2, vc2, Hq, Hkv, D, pos0)
        torch.cuda.synchronize()
        assert torch.equal(q2, q1), (M, pos0)
        assert torch.equal(kc2, kc1) and torch.equal(vc2, vc1), (M, pos0)
        assert torch.equal(got, want), (M, pos0)


@pytest.mark.parametrize("Hq,Hkv", [(12, 2), (4, 4), (3, 1)])
def test_rope_attention_decode_equals_the_two_operators(pkg, Hq, Hkv):
    g = torch.Generator(device="cuda").manual_seed(6)
    D, S = 128, 256
    sin, cos = pkg.op_rope_table(S, D, 1e6)
    scratch = pkg.op_scratch(Hq)
    for pos in [0, 3, 15, 16, 17, 100, 255]:
        kc = torch.randn((Hkv, S, D), generator=g, device="cuda")
        vc = torch.randn((Hkv, S, D), generator=g, device="cuda")
        q = torch.randn((1, Hq * D), generator=g, device="cuda")
        k = torch.randn((1, Hkv * D), generator=g, device="cuda")
        v = torch.randn((1, Hkv * D), generator=g, device="cuda")
        kc1, vc1, q1 = kc.clone(), vc.clone(), q.clone()
        pkg.op_rope_kv(q1, k, v, sin, cos, kc1, vc1, Hq, Hkv, D, pos)
        want = pkg.op_attention(q1, kc1, vc1, Hq, Hkv, D, pos, scratch=scratch)
        kc2, vc2 = kc.clone(), vc.clone()
        got = pkg.op_rope_attention_decode(q, k, v, sin, cos, kc2, vc2, Hq, Hkv, D, pos, scratch)
        assert torch.equal(got, want), pos
        assert torch.equal(kc2, kc1) and torch.equal(vc2, vc1), pos


@pytest.mark.parametrize("Hq,Hkv,N,bias", [(12, 2, 1536, False), (4, 4, 272, True), (3, 1, 40, True),
                                            (24, 4, 3072, False)])
def test_attention_slices_merged_by_the_linear_that_reads_them(pkg, Hq, Hkv, N, bias):
    """Decode attention that leaves its key slices unmerged + the Linear whose row load merges them
    == the attention operator followed by the Linear, bit for bit, and the same cache rows."""
    g = torch.Generator(device="cuda").manual_seed(16)
    D, S = 128, 1024
    sin, cos = pkg.op_rope_table(S, D, 1e6)
    scratch = pkg.op_scratch(Hq)
    w = torch.randn((N, Hq * D), generator=g, device="cuda") * 0.05
    b = torch.randn((N,), generator=g, device="cuda") if bias else None
    packed = pkg.quant_pack_rhs(w, b)
    for pos in [0, 3, 15, 16, 17, 100, 255, 640, 1023]:
        kc = torch.randn((Hkv, S, D), generator=g, device="cuda")
        vc = torch.randn((Hkv, S, D), generator=g, device="cuda")
        kc[:, pos + 1:] = float("nan")       # rows past the position are never part of the result
        vc[:, pos + 1:] = float("nan")
        q = torch.randn((1, Hq * D), generator=g, device="cuda")
        k = torch.randn((1, Hkv * D), generator=g, device="cuda")
        v = torch.randn((1, Hkv * D), generator=g, device="cuda")
        kc1, vc1 = kc.clone(), vc.clone()
        attn = pkg.op_rope_attention_decode(q, k, v, sin, cos, kc1, vc1, Hq, Hkv, D, pos, scratch)
        want = pkg.matmul(attn, packed, N)
        kc2, vc2 = kc.clone(), vc.clone()
        d_pos = torch.tensor([pos], dtype=torch.int32, device="cuda")
        got = pkg.op_rope_attention_decode_linear(q, k, v, sin, cos, kc2, vc2, packed, N, Hq, Hkv, D, 0, scratch,
                                                  d_pos0=d_pos)
        assert torch.isfinite(got).all(), pos
        assert torch.equal(got, want), (pos, float((got - want).abs().max()))
        assert torch.equal(kc2[:, :pos + 1], kc1[:, :pos + 1]) and torch.equal(vc2[:, :pos + 1], vc1[:, :pos + 1]), pos
    # a Linear too long for the merging kernel is refused, not mis-computed
    wide = pkg.quant_pack_rhs(torch.randn((32, 28 * D), generator=g, device="cuda"), None)
    kc = torch.zeros((4, S, D), device="cuda")
    with pytest.raises(Exception):
        pkg.op_rope_attention_decode_linear(torch.zeros((1, 28 * D), device="cuda"), torch.zeros((1, 4 * D), device="cuda"),
                                            torch.zeros((1, 4 * D), device="cuda"), sin, cos, kc, kc.clone(), wide, 32,
                                            28, 4, D, 0, pkg.op_scratch(28))


def test_argmax_first_maximum(pkg):
    g = torch.Generator(device="cuda").manual_seed(3)
    scratch = pkg.op_scratch(12)
    for n in [151936, 1000, 7, 1]:
        x = torch.randn((n,), generator=g, device="cuda")
        assert int(pkg.op_argmax(x, scratch)) == int(torch.argmax(x))
    x = torch.zeros((151936,), device="cuda")
    x[[70000, 140000, 300]] = 5.0
    assert int(pkg.op_argmax(x, scratch)) == 300
    pos = torch.tensor([41], dtype=torch.int32, device="cuda")
    pkg.op_argmax(x, scratch, d_pos=pos)
    assert int(pos) == 42
    assert int(pkg.op_argmax(torch.full((100,), float("-inf"), device="cuda"), scratch)) == 0


def tiny_model(rng, H, Hq, Hkv, I, V, layers):
    def w(n, k):
        return (rng.standard_normal((n, k)) * 0.05).astype(np.float32)

    weights = {"embedding": rng.standard_normal((V, H)).astype(np.float32), "lm_head": w(V, H),
               "final_norm": (1 + 0.1 * rng.standard_normal(H)).astype(np.float32), "layers": []}
    for _ in range(layers):
        weights["layers"].append({
            "q": w(Hq * 128, H), "k": w(Hkv * 128, H), "v": w(Hkv * 128, H), "o": w(H, Hq * 128),
            "gate": w(I, H), "up": w(I, H), "down": w(H, I),
            "q_bias": (0.1 * rng.standard_normal(Hq * 128)).astype(np.float32),
            "k_bias": (0.1 * rng.standard_normal(Hkv * 128)).astype(np.float32),
            "v_bias": (0.1 * rng.standard_normal(Hkv * 128)).astype(np.float32),
            "attn_norm": (1 + 0.1 * rng.standard_normal(H)).astype(np.float32),
            "ffn_norm": (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)})
    return weights


def to_device_model(pkg, weights, Hq, Hkv, **kw):
    layers = []
    for lw in weights["layers"]:
        d = {}
        for name in ("q", "k", "v", "o", "gate", "up", "down"):
            b = lw.get(name + "_bias")
            d[name] = pkg.quant_pack_rhs(dev(lw[name]), None if b is None else dev(b))
        d["attn_norm"], d["ffn_norm"] = dev(lw["attn_norm"]), dev(lw["ffn_norm"])
        layers.append(d)
    V, H = weights["embedding"].shape
    return pkg.Decoder(H, Hq, Hkv, weights["layers"][0]["gate"].shape[0], V, layers, dev(weights["embedding"]),
                       dev(weights["final_norm"]), pkg.quant_pack_rhs(dev(weights["lm_head"])), **kw)


def test_decoder_runner_matches_oracle(pkg):
    import decoder_oracle as do

    rng = np.random.default_rng(4)
    H, Hq, Hkv, I, V, L = 256, 2, 1, 384, 640, 2
    weights = tiny_model(rng, H, Hq, Hkv, I, V, L)
    dec = to_device_model(pkg, weights, Hq, Hkv, max_seq=64, max_batch_tokens=16, rope_theta=1e6)
    ref = do.Decoder(weights, Hq, Hkv, rope_theta=1e6, max_seq=64)

    prompt = rng.integers(0, V, size=11)
    tok = dec.prefill(dev(prompt.astype(np.int64)))
    torch.cuda.synchronize()
    want = ref.forward(prompt)
    got = dec.logits.cpu().numpy()
    assert max_abs_rel(got, want) < 2e-3
    assert int(tok) == do.greedy(got) and dec.position == 11
    for step in range(12):
        fed = int(dec.token)                      # teacher forcing: the oracle consumes the runner's token
        dec.step()
        torch.cuda.synchronize()
        want = ref.forward([fed])
        got = dec.logits.cpu().numpy()
        assert max_abs_rel(got, want) < 2e-3, step
        assert int(dec.token) == do.greedy(got)
        assert dec.position == 12 + step


@pytest.mark.parametrize("slices", [(8, 3), (3, 8), (5, 6), (1, 2, 8), (4, 7)])
def test_decoder_prefill_in_slices_of_decode_sized_rows(pkg, slices):
    """A prompt fed in slices of 1..8 rows runs every Linear through the decode-sized kernels on several rows (short
    K: more tile rows per workgroup than at the model's widths), continuing the cache of the slices before."""
    import decoder_oracle as do

    rng = np.random.default_rng(21)
    H, Hq, Hkv, I, V, L = 256, 2, 1, 384, 640, 2
    weights = tiny_model(rng, H, Hq, Hkv, I, V, L)
    dec = to_device_model(pkg, weights, Hq, Hkv, max_seq=64, max_batch_tokens=8, rope_theta=1e6)
    ref = do.Decoder(weights, Hq, Hkv, rope_theta=1e6, max_seq=64)
    prompt = rng.integers(0, V, size=sum(slices))
    want = ref.forward(prompt)
    for rep in range(2):                          # the second pass overwrites the first one's cache rows
        pos = 0
        for n in slices:
            dec.prefill(dev(prompt[pos:pos + n].astype(np.int64)), pos0=pos)
            pos += n
        torch.cuda.synchronize()
        got = dec.logits.cpu().numpy()
        assert max_abs_rel(got, want) < 2e-3, rep
        assert int(dec.token) == do.greedy(got) and dec.position == len(prompt)


@pytest.mark.parametrize("slices", [(300, 290), (256, 256, 70), (40, 330)])
def test_decoder_prefill_in_long_slices_that_continue_a_cache(pkg, slices):
    """Prompt slices of 256 rows and more take the matrix-pipe attention, whose operand split also rotates q and k
    and appends to the caches: here at positions that continue earlier slices (inside a 32-key block too), against
    the oracle on the whole prompt, and the cache rows against a run that takes the prompt in one slice."""
    import decoder_oracle as do

    rng = np.random.default_rng(23)
    H, Hq, Hkv, I, V, L = 256, 2, 1, 384, 640, 2
    n = sum(slices)
    weights = tiny_model(rng, H, Hq, Hkv, I, V, L)
    dec = to_device_model(pkg, weights, Hq, Hkv, max_seq=640, max_batch_tokens=max(slices), rope_theta=1e6)
    one = to_device_model(pkg, weights, Hq, Hkv, max_seq=640, max_batch_tokens=n, rope_theta=1e6)
    ref = do.Decoder(weights, Hq, Hkv, rope_theta=1e6, max_seq=640)
    prompt = rng.integers(0, V, size=n)
    want = ref.forward(prompt)
    one.prefill(dev(prompt.astype(np.int64)))
    pos = 0
    for m in slices:
        dec.prefill(dev(prompt[pos:pos + m].astype(np.int64)), pos0=pos)
        pos += m
    torch.cuda.synchronize()
    got = dec.logits.cpu().numpy()
    # 2e-2 throughout: after 600 tokens the logits come out either identical to the oracle's (1e-7) or between
    # 1e-3 and 1e-2 off, with either attention kernel and however the prompt is sliced (582 tokens: 9e-3 through
    # the matrix-pipe kernel, 1.3e-3 through the f32 one; 590 tokens: 3e-7 and 0): one int8 of a re-quantised row
    # that flips on a last-bit difference moves a logit by a weight times a quantisation step. The operators
    # themselves are held to 2e-5 and to bit-identity with the separate launches by the tests above; what this
    # test looks for is a wrong or missing cache row, which is off by the size of the logits themselves.
    assert max_abs_rel(got, want) < 2e-2
    assert max_abs_rel(one.logits.cpu().numpy(), want) < 2e-2
    assert int(dec.token) == do.greedy(got) and dec.position == n
    # two more tokens continue from what the slices left in the caches
    for _ in range(2):
        fed = int(dec.token)
        dec.step()
        want = ref.forward([fed])
        torch.cuda.synchronize()
        assert max_abs_rel(dec.logits.cpu().numpy(), want) < 2e-2


def test_decoder_ignores_what_its_state_memory_held(pkg):
    # The state is caller-owned memory that init does not clear: rows of the KV cache behind the position,
    # scratch areas and activations hold whatever was there. Bytes 0xFF (NaN as f32) against zeros: prefill
    # and decode steps must give the same logits bit for bit. (The decode attention loads the row of the new
    # token's position before anybody has written it.)
    import ctypes

    rng = np.random.default_rng(7)
    H, Hq, Hkv, I, V, L = 256, 2, 1, 384, 640, 2
    weights = tiny_model(rng, H, Hq, Hkv, I, V, L)
    prompt = dev(rng.integers(0, V, size=21).astype(np.int64))
    runs = []
    for fill in (0, 255):
        dec = to_device_model(pkg, weights, Hq, Hkv, max_seq=64, max_batch_tokens=32, rope_theta=1e6)
        dec.state.fill_(fill)
        assert pkg.lib().w4a32_decoder_init(ctypes.byref(dec.cfg), dec.state.data_ptr(), None) == 0
        out = []
        dec.step()                                  # a first token at position 0, nothing cached yet
        out.append(dec.logits.clone())
        dec.prefill(prompt)                         # (from position 0 again)
        out.append(dec.logits.clone())
        for _ in range(20):                         # positions 21..40: every place inside a block of 16 keys
            dec.step()
            out.append(dec.logits.clone())
        torch.cuda.synchronize()
        runs.append(out)
    for a, b in zip(*runs):
        assert not bool(torch.isnan(b).any())
        assert torch.equal(a, b)


def test_decoder_step_gathers_the_token_s_embedding_row_itself(pkg):
    # The first launch of a step reads row `token` of the embedding table (no gather launch in front of it):
    # a step on token t must equal a one-token prefill of [t] bit for bit in what it leaves as the residual
    # stream's start and in its logits' token, and ids outside the table are clamped to it as the embedding
    # operator clamps them (LLMEmbeddingTokenOp.cpp:24-50 reads the row; out-of-range ids are undefined there).
    rng = np.random.default_rng(11)
    H, Hq, Hkv, I, V, L = 256, 2, 1, 384, 640, 2
    weights = tiny_model(rng, H, Hq, Hkv, I, V, L)
    emb = weights["embedding"]
    outs = {}
    for tok in (0, 5, V - 1, V + 7, -3):
        dec = to_device_model(pkg, weights, Hq, Hkv, max_seq=32, max_batch_tokens=16, rope_theta=1e6)
        dec.token.fill_(tok)
        dec.step()
        torch.cuda.synchronize()
        outs[tok] = (dec.logits.clone(), int(dec.token))
        row = min(max(tok, 0), V - 1)
        ref = to_device_model(pkg, weights, Hq, Hkv, max_seq=32, max_batch_tokens=16, rope_theta=1e6)
        ref.prefill(dev(np.array([row], dtype=np.int64)))
        torch.cuda.synchronize()
        assert int(ref.token) == outs[tok][1], tok
        assert max_abs_rel(outs[tok][0].cpu().numpy(), ref.logits.cpu().numpy()) < 2e-3, tok
        assert np.isfinite(outs[tok][0].cpu().numpy()).all()
    assert torch.equal(outs[V + 7][0], outs[V - 1][0]) and torch.equal(outs[-3][0], outs[0][0])
    assert not torch.equal(outs[0][0], outs[5][0]) and emb.shape == (V, H)


@pytest.mark.parametrize("prompt_len", [300, 520])
def test_decoder_runner_at_the_model_s_widths(pkg, prompt_len):
    # hidden 1536, 12 / 2 heads, MLP 8960 (two layers, small vocabulary): the prefill runs the kernels the
    # real model runs - grouped q,k,v, the gate,up pair launch, split-K down with K = 8960, the matrix-core
    # attention with its keys dealt to several workgroups (300 rows) and in one launch per query block (520).
    # Tolerance: at these widths the model itself amplifies last-bit differences. Every Linear re-quantises
    # its input rows to int8, and a 1e-7 difference in a row (f32 summation order of the attention) flips a
    # few roundings; one flip moves an output by weight x step (down_proj: 0.02 x 0.03), a row of 8960
    # collects about 15 of them, and the logits end up 0 (no flip), 1e-7 or about 1e-2 apart - measured on
    # operators that each agree with the oracle to 3e-7 on the oracle's own inputs. So 5e-2 here: this test
    # shows that the runner strings the operators together correctly (and picks the greedy token of its own
    # logits); that no operator at these widths is off by more than 2e-5 is the business of
    # test_prefill_layer_at_the_model_s_widths_every_operator_on_its_own_inputs, which feeds the oracle the
    # HIP path's own quantised rows so that nothing is amplified.
    import decoder_oracle as do

    rng = np.random.default_rng(prompt_len)
    H, Hq, Hkv, I, V, L = 1536, 12, 2, 8960, 1024, 2
    weights = tiny_model(rng, H, Hq, Hkv, I, V, L)
    for lw in weights["layers"]:                  # N(0, 0.02^2) as in the benchmark's synthetic weights
        for name in ("q", "k", "v", "o", "gate", "up", "down"):
            lw[name] *= np.float32(0.4)
    dec = to_device_model(pkg, weights, Hq, Hkv, max_seq=576, max_batch_tokens=prompt_len, rope_theta=1e6)
    do.Linear.threads = 16
    try:
        ref = do.Decoder(weights, Hq, Hkv, rope_theta=1e6, max_seq=576)
        prompt = rng.integers(0, V, size=prompt_len)
        tok = dec.prefill(dev(prompt.astype(np.int64)))
        torch.cuda.synchronize()
        want = ref.forward(prompt)
        got = dec.logits.cpu().numpy()
        assert max_abs_rel(got, want) < 5e-2
        assert int(tok) == do.greedy(got) and dec.position == prompt_len
        for step in range(3):
            fed = int(dec.token)
            dec.step()
            torch.cuda.synchronize()
            want = ref.forward([fed])
            got = dec.logits.cpu().numpy()
            assert max_abs_rel(got, want) < 5e-2, step
            assert int(dec.token) == do.greedy(got)
    finally:
        do.Linear.threads = 1


def _lhs_raw(aq, recip, neg_zp):
    """The oracle's packed row format (f32 reciprocal scale, i32 negated zero point, K int8 values) from
    what w4a32_export_lhs returns: the rows exactly as the product kernel consumed them."""
    m, k = aq.shape
    raw = np.empty((m, k + 8), dtype=np.int8)
    raw[:, 0:4] = recip.reshape(m, 1).view(np.int8)
    raw[:, 4:8] = neg_zp.reshape(m, 1).view(np.int8)
    raw[:, 8:] = aq
    return raw


@pytest.mark.parametrize("M", [300, 520])
def test_prefill_layer_at_the_model_s_widths_every_operator_on_its_own_inputs(pkg, orc, M):
    """One decoder layer at hidden 1536, 12 / 2 heads, MLP 8960, issued as the runner's prefill issues it
    (fused add + norm + quantiser, grouped q,k,v, rope + append, matrix-core attention, o, gate,up pair,
    split-K down whose parts the next quantiser adds up), with every operator checked against the oracle
    on the HIP path's OWN inputs: the quantised rows are exported from the workspace and fed to the
    oracle's product, so no difference can be amplified by a re-quantisation in between and every Linear
    is held to 2e-5 (block sums are exact integers on both sides; only f32 summation order differs)."""
    import decoder_oracle as do

    H, Hq, Hkv, I, D = 1536, 12, 2, 8960, 128
    eps = 1e-6
    rng = np.random.default_rng(1000 + M)
    w = {n: (rng.standard_normal(shape) * 0.02).astype(np.float32) for n, shape in
         [("q", (Hq * D, H)), ("k", (Hkv * D, H)), ("v", (Hkv * D, H)), ("o", (H, Hq * D)),
          ("gate", (I, H)), ("up", (I, H)), ("down", (H, I))]}
    bias = {n: (rng.standard_normal(w[n].shape[0]) * 0.1).astype(np.float32) for n in ("q", "k", "v")}
    norm1 = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    norm2 = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32)
    q4 = {n: orc.quant_rhs(w[n]) for n in w}
    packed = {n: pkg.repack_native(dev(q4[n][0]), dev(q4[n][1].view(np.int16)),
                                   dev(bias[n]) if n in bias else None, *w[n].shape) for n in w}
    rows = np.unique(np.concatenate([np.arange(0, M, 23), [M - 1, 31, 32, 255, 256]]))

    def product_ok(ws, K, name, got, what):
        aq, recip, nzp = (t.cpu().numpy() for t in pkg.export_lhs(ws, M, K))
        raw = _lhs_raw(aq[rows], recip[rows], nzp[rows])
        ref = orc.matmul_packed(raw, *q4[name], bias=bias.get(name), threads=16)
        err = max_abs_rel(got.cpu().numpy()[rows], ref)
        assert err <= 2e-5, (what, err)
        return raw

    h0 = (rng.standard_normal((M, H)) * 2).astype(np.float32)
    d0 = rng.standard_normal((M, H)).astype(np.float32)

    # [add + norm + quantiser]: the sum is exact, the quantised rows reconstruct the normalised rows to half a step
    ws1, h1 = pkg.quant_lhs_norm(dev(h0), dev(norm1), eps, delta=dev(d0))
    assert np.array_equal(h1.cpu().numpy(), h0 + d0)
    aq, recip, nzp = (t.cpu().numpy() for t in pkg.export_lhs(ws1, M, H))
    want_rows = do.rmsnorm(h0 + d0, norm1, eps)
    back = (aq.astype(np.float32) + nzp[:, None]) * recip[:, None]
    assert np.all(np.abs(back - want_rows) <= recip[:, None] * 0.5001 + 1e-6)

    # [q, k, v grouped]
    qkv = pkg.matmul_quantized_grouped(ws1, [packed["q"], packed["k"], packed["v"]], [Hq * D, Hkv * D, Hkv * D], M, H)
    for name, y in zip("qkv", qkv):
        product_ok(ws1, H, name, y, name + "_proj")

    # [rope + append] [attention] on the HIP path's own q, k, v
    q_h, k_h, v_h = (t.cpu().numpy() for t in qkv)
    sin, cos = pkg.op_rope_table(M, D, 1e6)
    kc = torch.zeros((Hkv, M, D), dtype=torch.float32, device="cuda")
    vc = torch.zeros_like(kc)
    q_rot = qkv[0].clone()
    pkg.op_rope_kv(q_rot, qkv[1], qkv[2], sin, cos, kc, vc, Hq, Hkv, D, 0)
    attn = pkg.op_attention_prefill(q_rot, kc, vc, Hq, Hkv, D, 0)
    s_ref, c_ref = do.rope_tables(M, D, 1e6)
    q_ref = do.rope(q_h.reshape(M, Hq, D), s_ref, c_ref, 0)
    k_ref = do.rope(k_h.reshape(M, Hkv, D), s_ref, c_ref, 0)
    assert max_abs_rel(q_rot.cpu().numpy(), q_ref.reshape(M, -1)) <= 6e-5      # one ulp of powf at 500 rad
    kc_h, vc_h = kc.cpu().numpy(), vc.cpu().numpy()
    assert max_abs_rel(kc_h, k_ref.transpose(1, 0, 2)) <= 6e-5
    assert np.array_equal(vc_h, v_h.reshape(M, Hkv, D).transpose(1, 0, 2))
    arows = rows[::3]
    a_ref = np.stack([do.attention(q_rot.cpu().numpy().reshape(M, Hq, D)[r:r + 1], kc_h, vc_h, int(r))[0]
                      for r in arows])
    assert max_abs_rel(attn.cpu().numpy()[arows], a_ref) <= 2e-5
    # the kernel a prefill of this many rows runs: products on bf16 terms, with the rotation and the cache append
    # done by its operand split; same bar against the oracle, caches and rotated q bit-identical to the above
    kc16, vc16, q16 = torch.zeros_like(kc), torch.zeros_like(vc), qkv[0].clone()
    attn16 = pkg.op_rope_attention_prefill_bf16x3(q16, qkv[1], qkv[2], sin, cos, kc16, vc16, Hq, Hkv, D, 0)
    assert torch.equal(q16, q_rot) and torch.equal(kc16, kc) and torch.equal(vc16, vc)
    assert max_abs_rel(attn16.cpu().numpy()[arows], a_ref) <= 2e-5

    # [quantiser] [o]
    ws2 = pkg.quant_lhs(attn)
    o_out = pkg.matmul_quantized(ws2, packed["o"], M, Hq * D, H)
    product_ok(ws2, Hq * D, "o", o_out, "o_proj")

    # [add + norm + quantiser] [gate, up pair -> silu * mul]
    ws3, h2 = pkg.quant_lhs_norm(h1, dev(norm2), eps, delta=o_out)
    assert torch.equal(h2, h1 + o_out)
    act = pkg.matmul_quantized_silu_pair(ws3, packed["gate"], packed["up"], M, H, I)
    aq, recip, nzp = (t.cpu().numpy() for t in pkg.export_lhs(ws3, M, H))
    raw3 = _lhs_raw(aq[rows], recip[rows], nzp[rows])
    g_ref = orc.matmul_packed(raw3, *q4["gate"], threads=16)
    u_ref = orc.matmul_packed(raw3, *q4["up"], threads=16)
    assert max_abs_rel(act.cpu().numpy()[rows], do.silu_mul(g_ref, u_ref)) <= 2e-5

    # [quantiser] [down, split over K; its parts are added by the next layer's add + norm + quantiser]
    ws4 = pkg.quant_lhs(act)
    scratch, parts = pkg.matmul_quantized_splitk_parts(ws4, packed["down"], M, I, H)
    assert parts > 1, "down_proj at these sizes is expected to run split over K"
    part_sum = scratch[:parts * M * H * 4].view(torch.float32).reshape(parts, M, H).cpu().numpy()
    total = part_sum[0].copy()
    for i in range(1, parts):
        total += part_sum[i]
    product_ok(ws4, I, "down", torch.from_numpy(total), "down_proj parts")
    down_whole = pkg.matmul_quantized_splitk(ws4, packed["down"], M, I, H)
    product_ok(ws4, I, "down", down_whole, "down_proj")
    _, h3 = pkg.quant_lhs_norm_parts(h2, scratch, parts, packed["down"], I, dev(norm1), eps)
    assert np.array_equal(h3.cpu().numpy(), h2.cpu().numpy() + total)


def test_decoder_step_replays_from_a_graph(pkg):
    """The decode step's launch sequence does not depend on the position: captured once, replayed
    per token (with eager work and synchronisations in between), it produces the tokens and logits
    of eager steps."""
    rng = np.random.default_rng(5)
    H, Hq, Hkv, I, V, L = 256, 2, 1, 384, 640, 2
    weights = tiny_model(rng, H, Hq, Hkv, I, V, L)
    prompt = dev(rng.integers(0, V, size=9).astype(np.int64))

    eager = to_device_model(pkg, weights, Hq, Hkv, max_seq=64, max_batch_tokens=16)
    eager.prefill(prompt)
    toks_e, logits_e = [], []
    for _ in range(10):
        eager.step()
        toks_e.append(int(eager.token))
        logits_e.append(eager.logits.clone())

    dec = to_device_model(pkg, weights, Hq, Hkv, max_seq=64, max_batch_tokens=16)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        dec.prefill(prompt)
        first = dec.token.clone()
        dec.step()                                # warm-up outside the capture
        s.synchronize()
        # rewind: prefill again so the captured step starts from the same state as the eager run
        dec.prefill(prompt)
        assert torch.equal(dec.token, first)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            dec.step()
        # capture does not execute: position is still 9
        s.synchronize()
        assert dec.position == 9
        for i in range(10):
            graph.replay()
            s.synchronize()
            assert int(dec.token) == toks_e[i], i
            assert torch.equal(dec.logits, logits_e[i]), i
            _ = (dec.logits * 2).sum().item()     # unrelated eager work between replays
        assert dec.position == 19


def test_decoder_prefill_replays_from_a_graph(pkg):
    """The prefill launches nothing that a capture cannot hold (no allocation, no memset; the position and the
    arrival counters of the chunked attention live in the state and are left as they were found): captured
    once for a prompt length, replayed with eager work in between, it gives the eager result every time."""
    rng = np.random.default_rng(8)
    H, Hq, Hkv, I, V, L = 256, 4, 2, 3072, 640, 2
    weights = tiny_model(rng, H, Hq, Hkv, I, V, L)
    n = 70                                        # three query blocks: the attention splits their keys
    # (the decoder lends its gate and up buffers, 2 * n * I floats, which must hold the chunks' hand-over)
    assert pkg.lib().w4a32_op_attention_prefill_scratch_bytes(n, Hq) <= 2 * n * I * 4
    prompts = [dev(rng.integers(0, V, size=n).astype(np.int64)) for _ in range(3)]

    eager = to_device_model(pkg, weights, Hq, Hkv, max_seq=128, max_batch_tokens=n)
    want = []
    for p in prompts:
        eager.prefill(p)
        want.append((int(eager.token), eager.logits.clone()))

    dec = to_device_model(pkg, weights, Hq, Hkv, max_seq=128, max_batch_tokens=n)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        buf = prompts[0].clone()                  # the captured launch reads its tokens from here
        dec.prefill(buf)                          # warm-up outside the capture
        s.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            dec.prefill(buf)
        for rep in range(2):
            for p, (tok, logits) in zip(prompts, want):
                buf.copy_(p)
                graph.replay()
                s.synchronize()
                assert int(dec.token) == tok and dec.position == n
                assert torch.equal(dec.logits, logits), rep
                _ = (dec.logits * 2).sum().item()  # unrelated eager work between replays


@pytest.mark.parametrize("K,Ns,pair", [(1536, [1536, 256, 256], False), (1536, [8960, 8960], True),
                                         (1536, [151936], False), (8960, [1536], False), (256, [640], False)])
def test_decode_linear_fusions_match_separate_operators(pkg, orc, K, Ns, pair):
    """Residual add + RMSNorm in front of the Linears and silu*mul behind them, in one launch, against
    the same operators run one by one and against the CPU oracle fed with the fused row."""
    import decoder_oracle as do

    rng = np.random.default_rng(K + len(Ns))
    x = rng.standard_normal((1, K)).astype(np.float32)
    d = rng.standard_normal((1, K)).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(K)).astype(np.float32)
    ws = [(rng.standard_normal((n, K)) * 0.02).astype(np.float32) for n in Ns]
    packed = [pkg.quant_pack_rhs(dev(w)) for w in ws]

    ys, total = pkg.decode_linear(dev(x), packed, Ns, norm_weight=dev(nw), eps=1e-6, delta=dev(d),
                                  want_sum=True, silu_pair=pair)
    torch.cuda.synchronize()
    assert torch.equal(total, dev(x) + dev(d))
    # the separate operators
    h2, xn = pkg.op_rmsnorm(dev(x), dev(nw), 1e-6, delta=dev(d))
    sep = pkg.matmul_grouped(xn, packed, Ns) if len(Ns) > 1 else [pkg.matmul(xn, packed[0], Ns[0])]
    if pair:
        sep = [pkg.op_silu_mul(sep[0], sep[1])]
    # the oracle on the normalised row
    xn_ref = do.rmsnorm((x + d).astype(np.float32), nw, 1e-6)
    want = []
    for w in ws if len(Ns) < 4 or Ns[0] < 100000 else ws:
        u4, sc = orc.quant_rhs(w)
        want.append(orc.linear(xn_ref, u4, sc))
    if pair:
        want = [do.silu_mul(want[0], want[1])]
    for got, s, ref in zip(ys, sep, want):
        assert max_abs_rel(got.cpu().numpy(), s.cpu().numpy()) < 2e-3
        assert max_abs_rel(got.cpu().numpy(), ref) < 2e-3
    # without the extras the call is the plain grouped product
    plain, _ = pkg.decode_linear(dev(x), packed, Ns)
    base = pkg.matmul_grouped(dev(x), packed, Ns) if len(Ns) > 1 else [pkg.matmul(dev(x), packed[0], Ns[0])]
    for a, b in zip(plain, base):
        assert torch.equal(a, b)


def test_full_size_decoder_properties(pkg):
    """The configuration the tokens/s figure is quoted on, at full depth: 28 layers, hidden 1536, 12 / 2
    heads, MLP 8960, vocabulary 151936, 512-token prompt, then greedy steps replayed from a captured graph.
    No CPU model finishes this in seconds, so it is held to properties: every step's logits are finite, its
    token is the first maximum of its logits, the position advances by one, and the replayed graph gives,
    bit for bit, the tokens and logits of eagerly launched steps from the same state."""
    H, Hq, Hkv, I, V, L = 1536, 12, 2, 8960, 151936, 28
    g = torch.Generator(device="cuda").manual_seed(4)
    rw = lambda n, k: pkg.quant_pack_rhs(torch.randn((n, k), generator=g, device="cuda") * 0.02)
    rb = lambda n, k: pkg.quant_pack_rhs(torch.randn((n, k), generator=g, device="cuda") * 0.02,
                                         torch.randn((n,), generator=g, device="cuda") * 0.02)
    norm = lambda: 1 + 0.1 * torch.randn((H,), generator=g, device="cuda")
    layers = [{"q": rb(Hq * 128, H), "k": rb(Hkv * 128, H), "v": rb(Hkv * 128, H), "o": rw(H, Hq * 128),
               "gate": rw(I, H), "up": rw(I, H), "down": rw(H, I), "attn_norm": norm(), "ffn_norm": norm()}
              for _ in range(L)]
    emb = torch.randn((V, H), generator=g, device="cuda")
    final_norm, lm_head = norm(), rw(V, H)
    prompt = torch.randint(0, V, (512,), generator=g, device="cuda", dtype=torch.int64)
    steps = 36

    def make():
        return pkg.Decoder(H, Hq, Hkv, I, V, layers, emb, final_norm, lm_head, max_seq=1024,
                           max_batch_tokens=512, rope_theta=1e6, rms_eps=1e-6)

    eager = make()
    eager.prefill(prompt)
    torch.cuda.synchronize()
    first_logits = eager.logits.clone()
    assert bool(torch.isfinite(first_logits).all()) and float(first_logits.abs().max()) > 0
    assert int(eager.token) == int(torch.argmax(first_logits)) and eager.position == 512
    toks, logits = [], []
    for i in range(steps):
        eager.step()
        lg = eager.logits.clone()
        assert bool(torch.isfinite(lg).all()), i
        assert int(eager.token) == int(torch.argmax(lg)), i          # torch.argmax: first maximum too
        assert eager.position == 513 + i
        toks.append(int(eager.token))
        logits.append(lg)
    assert len(set(toks)) > 1                                        # not stuck on one token

    dec = make()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        dec.prefill(prompt)
        dec.step()                                                   # warm-up outside the capture
        dec.prefill(prompt)                                          # rewind to the state the eager run started from
        s.synchronize()
        assert torch.equal(dec.logits, first_logits)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            dec.step()
        s.synchronize()
        assert dec.position == 512                                   # a capture executes nothing
        for i in range(steps):
            graph.replay()
            s.synchronize()
            assert int(dec.token) == toks[i], i
            assert torch.equal(dec.logits, logits[i]), i
            if i % 8 == 0:
                _ = (dec.logits * 2).sum().item()                    # unrelated eager work between replays
        assert dec.position == 512 + steps


def test_engine_path_operators(pkg):
    """The operators that only the engine's op-by-op path uses: SiLU then Mul equals the fused operator bit for
    bit; RoPE on one tensor equals what the fused rope + cache-append operator does to q and k; attention on a
    [keys][kv_heads][128] cache equals attention on the head-major cache; the dense matmul against torch."""
    g = torch.Generator(device="cuda").manual_seed(11)
    a = torch.randn((3, 8960), generator=g, device="cuda") * 4
    b = torch.randn((3, 8960), generator=g, device="cuda")
    assert torch.equal(pkg.op_mul(pkg.op_silu(a), b), pkg.op_silu_mul(a, b))
    assert max_abs_rel(pkg.op_silu(a).cpu().numpy(), torch.nn.functional.silu(a).cpu().numpy()) < 1e-5
    assert torch.equal(pkg.op_mul(a, b), a * b)

    Hq, Hkv, D, max_seq = 12, 2, 128, 96
    sin, cos = pkg.op_rope_table(max_seq, D, 1e6)
    for M, pos0 in [(1, 0), (1, 37), (20, 5), (64, 32)]:
        q = torch.randn((M, Hq * D), generator=g, device="cuda")
        k = torch.randn((M, Hkv * D), generator=g, device="cuda")
        v = torch.randn((M, Hkv * D), generator=g, device="cuda")
        kc = torch.randn((Hkv, max_seq, D), generator=g, device="cuda")   # earlier positions: any values
        vc = torch.randn((Hkv, max_seq, D), generator=g, device="cuda")
        q_fused = q.clone()
        pkg.op_rope_kv(q_fused, k, v, sin, cos, kc, vc, Hq, Hkv, D, pos0)
        q_rot = pkg.op_rope(q, sin, cos, Hq, D, pos0)
        k_rot = pkg.op_rope(k, sin, cos, Hkv, D, pos0)
        assert torch.equal(q_rot, q_fused)
        assert torch.equal(k_rot.view(M, Hkv, D).transpose(0, 1), kc[:, pos0:pos0 + M])
        # the same keys and values as [keys][Hkv][D]
        n_keys = pos0 + M
        k_bshd = kc[:, :n_keys].transpose(0, 1).contiguous()
        v_bshd = vc[:, :n_keys].transpose(0, 1).contiguous()
        want = pkg.op_attention(q_rot, kc, vc, Hq, Hkv, D, pos0) if M < 16 else None
        got = pkg.op_attention_bshd(q_rot, k_bshd, v_bshd, Hq, Hkv, D, pos0)
        if want is not None:
            assert torch.equal(got, want)       # the same kernel under other strides
        qh = q_rot.view(M, Hq, D).transpose(0, 1)                       # [Hq][M][D]
        kh = kc[:, :n_keys].repeat_interleave(Hq // Hkv, dim=0)
        vh = vc[:, :n_keys].repeat_interleave(Hq // Hkv, dim=0)
        mask = torch.arange(n_keys, device="cuda")[None, :] <= (pos0 + torch.arange(M, device="cuda"))[:, None]
        ref = torch.nn.functional.scaled_dot_product_attention(qh, kh, vh, attn_mask=mask)
        assert max_abs_rel(got.cpu().numpy(), ref.transpose(0, 1).reshape(M, Hq * D).cpu().numpy()) < 2e-5

    for M, K, N in [(1, 1536, 151936), (4, 1536, 1000), (8, 96, 50), (9, 64, 70), (200, 256, 300), (64, 1536, 128)]:
        x = torch.randn((M, K), generator=g, device="cuda")
        w = torch.randn((N, K), generator=g, device="cuda") * 0.05
        y = pkg.op_matmul_f32_nt(x, w)
        ref = (x.double() @ w.double().T)
        assert max_abs_rel(y.cpu().numpy(), ref.cpu().numpy()) < 1e-5, (M, K, N)


@pytest.mark.parametrize("K,N", [(8960, 1536), (6144, 256), (8992, 1000), (12288, 2048)])
def test_decode_linear_split_over_k_and_the_launch_that_reads_its_parts(pkg, orc, K, N):
    """A decode Linear with a long K and few output rows leaves its result as partial rows (its k range dealt
    to several workgroups per tile row); the next launch adds them up while it loads its row. The parts must
    add up to the unsplit Linear's output (f32 rounding apart) and match the oracle; a reader given partial
    rows must produce, bit for bit, what it produces from the row added up beforehand in the same order."""
    L = pkg.lib()
    P = L.w4a32_decode_kparts(K, N)
    assert P == 2
    assert L.w4a32_decode_kparts(1536, 1536) == 1 and L.w4a32_decode_kparts(1536, 8960) == 1
    assert L.w4a32_decode_kparts(8960, 151936) == 1 and L.w4a32_decode_kparts(100, 16) == 0
    rng = np.random.default_rng(K + N)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
    x = rng.standard_normal((1, K)).astype(np.float32)
    u4, sc = orc.quant_rhs(w)
    packed = pkg.repack_native(dev(u4), dev(sc.view(np.int16)), dev(bias), N, K)
    (parts,), _ = pkg.decode_linear(dev(x), [packed], [N], out_parts=P)
    assert parts.shape == (P, N)
    total = parts[0] + parts[1]
    whole = pkg.matmul(dev(x), packed, N)
    ref = orc.linear(x, u4, sc, bias=bias, threads=8)
    assert max_abs_rel(total.cpu().numpy()[None], whole.cpu().numpy()) < 1e-6
    assert max_abs_rel(total.cpu().numpy()[None], ref) <= 2e-5
    assert float(parts[1].abs().max()) > 0
    with pytest.raises(pkg.W4A32Error):
        pkg.decode_linear(dev(x), [packed], [N], out_parts=P + 1)        # not the library's split of this shape

    if N % 32:
        return
    # readers: Linears on a row that arrives in two or three partial rows (K of the reader = N of the producer)
    ns = [256, 64, 48]
    rd = [pkg.quant_pack_rhs(dev((rng.standard_normal((n, N)) * 0.05).astype(np.float32)),
                             dev((rng.standard_normal(n) * 0.1).astype(np.float32))) for n in ns]
    three = torch.cat([parts, dev(rng.standard_normal((1, N)).astype(np.float32) * 0.3)]).contiguous()
    h = dev(rng.standard_normal((1, N)).astype(np.float32) * 2)
    nw = dev((1 + 0.1 * rng.standard_normal(N)).astype(np.float32))
    for rows in (2, 3):
        summed = three[0] + three[1]
        if rows == 3:
            summed = summed + three[2]
        summed = summed[None].contiguous()
        for cnt in (3, 1):
            got, _ = pkg.decode_linear(three, rd[:cnt], ns[:cnt], in_parts=rows)
            want, _ = pkg.decode_linear(summed, rd[:cnt], ns[:cnt])
            assert all(torch.equal(a, b) for a, b in zip(got, want)), (rows, cnt)
        # ... and with the residual add + RMSNorm in front: the partial rows are the delta
        got, sum_got = pkg.decode_linear(h, rd, ns, norm_weight=nw, delta=three, want_sum=True, in_parts=rows)
        want, sum_want = pkg.decode_linear(h, rd, ns, norm_weight=nw, delta=summed, want_sum=True)
        assert torch.equal(sum_got, sum_want) and torch.equal(sum_got, h + summed)
        assert all(torch.equal(a, b) for a, b in zip(got, want)), rows
    # ... and an lm_head-sized reader (one wavefront per tile row): partial rows only as the delta in front of a norm
    nv = 32768 + 48
    wide = pkg.quant_pack_rhs(dev((rng.standard_normal((nv, N)) * 0.05).astype(np.float32)), None)
    for rows in (2, 3):
        summed = three[0] + three[1]
        if rows == 3:
            summed = summed + three[2]
        summed = summed[None].contiguous()
        (got,), _ = pkg.decode_linear(h, [wide], [nv], norm_weight=nw, delta=three, in_parts=rows)
        (want,), _ = pkg.decode_linear(h, [wide], [nv], norm_weight=nw, delta=summed)
        assert torch.equal(got, want), rows
    with pytest.raises(pkg.W4A32Error):
        pkg.decode_linear(three, [wide], [nv], in_parts=2)               # no norm: that kernel takes one row


def test_decoder_refuses_to_run_past_its_cache(pkg):
    # prefill checks capacity in the C ABI (its position is a host argument); the Python plumbing counts the
    # steps it issues and refuses the one that would overwrite the last cache row
    rng = np.random.default_rng(3)
    H, Hq, Hkv, I, V, L = 256, 2, 1, 384, 640, 1
    dec = to_device_model(pkg, tiny_model(rng, H, Hq, Hkv, I, V, L), Hq, Hkv, max_seq=16, max_batch_tokens=16)
    with pytest.raises(pkg.W4A32Error):
        dec.prefill(dev(rng.integers(0, V, size=14).astype(np.int64)), pos0=3)     # 3 + 14 > 16
    dec.prefill(dev(rng.integers(0, V, size=14).astype(np.int64)))
    dec.step()
    dec.step()
    torch.cuda.synchronize()
    assert dec.position == 16
    with pytest.raises(pkg.W4A32Error):
        dec.step()
    assert dec.position == 16


def test_partial_rows_whose_sum_overflows_are_clamped_by_the_reader(pkg):
    """A Linear that ran split over K leaves unclamped partial rows; the launch that adds them up clamps the sum
    to the finite f32 range, as the unsplit kernel (and the reference's matmul, kai_linear.cpp:392-396) clamps
    its output. Observed through the residual sum the reader stores: h + (p0 + p1) with h = 0."""
    K, N = 1536, 256
    big = np.float32(3e38)
    parts = np.zeros((2, K), dtype=np.float32)
    parts[:, 0] = (big, big)            # +inf as a plain sum
    parts[:, 5] = (-big, -big)          # -inf
    parts[:, 9] = (big, -big)           # cancels
    parts[:, 17] = (1.5, 2.25)
    flt_max = np.finfo(np.float32).max
    w = make_weights(N, K, seed=3)
    packed = pkg.quant_pack_rhs(dev(w))
    nw = torch.ones((K,), device="cuda")
    h = torch.zeros((1, K), device="cuda")
    _, total = pkg.decode_linear(h, [packed], [N], norm_weight=nw, delta=dev(parts), want_sum=True, in_parts=2)
    torch.cuda.synchronize()
    t = total.cpu().numpy()[0]
    assert t[0] == flt_max and t[5] == -flt_max and t[9] == 0.0 and t[17] == 3.75
    assert not t[[1, 2, 3, 4, 6, 7, 8, 10]].any()

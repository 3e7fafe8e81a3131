"""GPU: the parameters the reference's W4A32 quantizer leaves unquantised, held as it stores them.

scripts/QuantCfg/ds_qwen2/1.5B-W4A32-KAI.json:33-45 writes the three RMSNorm weights and lm_head.weight as
Fp16, and the model applies lm_head as a dense matmul with transpose_b (modeling_ds_qwen2.hpp:209-213).
Here: the f16 -> f32 widening (exact), the dense product on f16 / f32 operands against a float64 product
(1e-5 max-abs-rel: f32 products and sums, another order), the f16 and the f32 form of the same values bit for
bit, and the decoder runner with a dense lm_head against the CPU oracle."""
import numpy as np
import pytest
import torch

from conftest import max_abs_rel

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_f16_parameters_widen_exactly(pkg):
    g = torch.Generator(device="cuda").manual_seed(0)
    for n in (1, 7, 8, 1536, 1536 * 3 + 5):
        x = (torch.randn((n,), generator=g, device="cuda") * 3).half()
        assert torch.equal(pkg.op_f16_to_f32(x), x.float())
    # every finite half, the infinities included
    bits = torch.arange(0, 65536, dtype=torch.int32, device="cuda").to(torch.int16).view(torch.float16)
    out, ref = pkg.op_f16_to_f32(bits), bits.float()
    ok = torch.isnan(ref) | (out.view(torch.int32) == ref.view(torch.int32))
    assert bool(ok.all()) and bool((torch.isnan(out) == torch.isnan(ref)).all())
    # a source that is only 2-byte aligned
    base = (torch.randn((4099,), generator=g, device="cuda")).half()
    assert torch.equal(pkg.op_f16_to_f32(base[3:]), base[3:].float())


@pytest.mark.parametrize("M,K,N", [(1, 256, 100), (1, 1536, 777), (3, 1536, 640), (8, 1536, 131), (8, 96, 640),
                                   (5, 8960, 67), (2, 100, 50), (20, 128, 130), (130, 64, 64), (4, 136, 9)])
def test_dense_product_on_f16_and_f32_operands(pkg, M, K, N):
    g = torch.Generator(device="cuda").manual_seed(M * 1000 + K + N)
    a = torch.randn((M, K), generator=g, device="cuda")
    b16 = (torch.randn((N, K), generator=g, device="cuda") * 0.05).half()
    b32 = b16.float()
    ref = (a.double().cpu() @ b32.double().cpu().T).numpy()
    y16 = pkg.op_matmul_nt(a, b16)
    y32 = pkg.op_matmul_nt(a, b32)
    torch.cuda.synchronize()
    assert max_abs_rel(y16.cpu().numpy(), ref) < 1e-5
    assert max_abs_rel(y32.cpu().numpy(), ref) < 1e-5
    if M <= 8 and K % 8 == 0 and M * ((K + 127) // 128) * 512 <= 160 * 1024:
        # the streamed kernel (rows of A in LDS) takes both forms: same order, an exact widening
        assert torch.equal(y16, y32)
    assert torch.equal(pkg.op_matmul_f32_nt(a, b32), y32)


def test_dense_lm_head_at_the_model_s_size(pkg):
    V, H = 151936, 1536
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn((1, H), generator=g, device="cuda")
    w = (torch.randn((V, H), generator=g, device="cuda") * 0.02).half()
    y = pkg.op_matmul_nt(x, w)
    torch.cuda.synchronize()
    ref = torch.matmul(x, w.float().T)          # the library's f32 product ...
    ref64 = torch.matmul(x.double(), w.double().T)   # ... and the float64 one
    assert max_abs_rel(y.cpu().numpy(), ref64.cpu().numpy()) < 1e-5
    assert max_abs_rel(y.cpu().numpy(), ref.cpu().numpy()) < 1e-5


def _tiny_model(rng, H=256, Hq=2, Hkv=1, I=384, V=640, L=2):
    rw = lambda n_, k_: (rng.standard_normal((n_, k_)) * 0.05).astype(np.float32)
    f16 = lambda a: a.astype(np.float16)
    weights = {"embedding": rng.standard_normal((V, H)).astype(np.float32), "lm_head": f16(rw(V, H)),
               "final_norm": f16(1 + 0.1 * rng.standard_normal(H)), "layers": []}
    for _ in range(L):
        weights["layers"].append({"q": rw(Hq * 128, H), "k": rw(Hkv * 128, H), "v": rw(Hkv * 128, H),
                                  "o": rw(H, Hq * 128), "gate": rw(I, H), "up": rw(I, H), "down": rw(H, I),
                                  "attn_norm": f16(1 + 0.1 * rng.standard_normal(H)),
                                  "ffn_norm": f16(1 + 0.1 * rng.standard_normal(H))})
    return weights, (H, Hq, Hkv, I, V)


def _run_decoder_with_a_dense_lm_head(pkg, head_dtype):
    """Norm weights arrive as f16 and are widened on the device; lm_head stays as the file holds it (f16) or as
    its f32 widening. Prefill (separate norm + dense rows) and decode steps (residual add + norm + dense rows in
    one launch, greedy choice from the per-wavefront pairs) against the oracle, teacher-forced."""
    import decoder_oracle as do

    rng = np.random.default_rng(11)
    weights, (H, Hq, Hkv, I, V) = _tiny_model(rng)
    layers = []
    for lw in weights["layers"]:
        d = {n: pkg.quant_pack_rhs(dev(lw[n])) for n in ("q", "k", "v", "o", "gate", "up", "down")}
        d["attn_norm"] = pkg.op_f16_to_f32(dev(lw["attn_norm"]))
        d["ffn_norm"] = pkg.op_f16_to_f32(dev(lw["ffn_norm"]))
        layers.append(d)
    head = dev(weights["lm_head"])
    if head_dtype == "f32":
        head = head.float()
    dec = pkg.Decoder(H, Hq, Hkv, I, V, layers, dev(weights["embedding"]), pkg.op_f16_to_f32(dev(weights["final_norm"])),
                      head, max_seq=64, max_batch_tokens=16, lm_head_dense=True)
    ref = do.Decoder(weights, Hq, Hkv, max_seq=64, lm_head_dense=True)
    prompt = [3, 17, 100, 42, 7, 250, 611, 5, 98]
    dec.prefill(dev(np.array(prompt, dtype=np.int64)))
    want = ref.forward(prompt)
    all_logits = []
    for step in range(8):
        torch.cuda.synchronize()
        got = dec.logits.cpu().numpy().copy()
        all_logits.append(got)
        assert max_abs_rel(got, want) < 2e-3, step
        assert int(dec.token) == int(np.argmax(got)) == do.greedy(got)   # first maximum
        fed = int(dec.token)
        dec.step()
        want = ref.forward([fed])
    return all_logits


def test_decoder_runner_with_a_dense_lm_head_in_f16_and_in_f32(pkg):
    a = _run_decoder_with_a_dense_lm_head(pkg, "f16")
    b = _run_decoder_with_a_dense_lm_head(pkg, "f32")
    assert len(a) == len(b) == 8
    for x, y in zip(a, b):
        assert np.array_equal(x, y)      # an f16 element widens exactly and both forms sum in the same order


def test_dense_head_launch_matches_norm_then_product(pkg):
    """The decode step's [add + norm + dense lm_head] launch (residual in the two partial rows down_proj leaves,
    greedy choice from the per-wavefront pairs) against the prefill path's separate norm and dense product on the
    same history, at the model's widths and vocabulary."""
    H, V = 1536, 151936
    g = torch.Generator(device="cuda").manual_seed(9)
    rw = lambda n_, k_: torch.randn((n_, k_), generator=g, device="cuda") * 0.05
    layers = [{"q": pkg.quant_pack_rhs(rw(1536, H)), "k": pkg.quant_pack_rhs(rw(256, H)),
               "v": pkg.quant_pack_rhs(rw(256, H)), "o": pkg.quant_pack_rhs(rw(H, 1536)),
               "gate": pkg.quant_pack_rhs(rw(8960, H)), "up": pkg.quant_pack_rhs(rw(8960, H)),
               "down": pkg.quant_pack_rhs(rw(H, 8960)),
               "attn_norm": 1 + 0.1 * torch.randn((H,), generator=g, device="cuda"),
               "ffn_norm": 1 + 0.1 * torch.randn((H,), generator=g, device="cuda")}]
    emb = torch.randn((V, H), generator=g, device="cuda")
    head = (torch.randn((V, H), generator=g, device="cuda") * 0.02).half()
    fnorm = 1 + 0.1 * torch.randn((H,), generator=g, device="cuda")
    dec = pkg.Decoder(H, 12, 2, 8960, V, layers, emb, fnorm, head, max_seq=32, max_batch_tokens=8,
                      lm_head_dense=True)
    prompt = [5, 1000, 77]
    dec.prefill(torch.tensor(prompt, dtype=torch.int64, device="cuda"))
    torch.cuda.synchronize()
    tok1 = int(dec.token)
    assert tok1 == int(torch.argmax(dec.logits))
    dec.step()
    torch.cuda.synchronize()
    by_step = dec.logits.clone()
    assert bool(torch.isfinite(by_step).all()) and int(dec.token) == int(torch.argmax(by_step))
    dec.prefill(torch.tensor(prompt + [tok1], dtype=torch.int64, device="cuda"))
    torch.cuda.synchronize()
    by_prefill = dec.logits.clone()
    # two paths through the same model (single-row fused launches against multi-row kernels): f32 summation
    # order differs, and a last-bit difference may flip an int8 of a re-quantised row
    assert max_abs_rel(by_step.cpu().numpy(), by_prefill.cpu().numpy()) < 2e-3

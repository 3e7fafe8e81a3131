"""The C++ operator layer (mllm-advanced_amd/host): the engine-facing classes a maintainer would
drop into mllm/Backends. The GPU test runs the C++ test binary, which drives
registerBackend -> createOp -> load(.mllm) -> dispatch -> D2H and compares with the CPU oracle."""
import ctypes
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "mllm-advanced_amd", "host")
BIN = os.path.join(HOST, "tests", "hip_linear_test")
BIN_MODEL = os.path.join(HOST, "tests", "hip_qwen2_test")
BIN_OPS = os.path.join(HOST, "tests", "hip_decoder_ops_test")
LIB = os.path.join(ROOT, "mllm-advanced_amd", "libmllm_hip_backend.so")


def test_backend_library_is_built_and_loads():
    assert os.path.exists(LIB), "run __graft_entry__.build()"
    ctypes.CDLL(os.path.join(ROOT, "mllm-advanced_amd", "libw4a32_hip.so"), mode=ctypes.RTLD_GLOBAL)
    ctypes.CDLL(LIB)
    assert os.path.exists(BIN) and os.path.exists(BIN_MODEL) and os.path.exists(BIN_OPS)


def test_container_structs_have_the_on_disk_sizes():
    # head 268 bytes, descriptor 416 bytes: the header static_asserts them; check the text is there
    text = open(os.path.join(HOST, "mllm", "EngineSlice.hpp")).read()
    assert "sizeof(ParameterPackHead) == 268" in text and "sizeof(ParameterDescriptor) == 416" in text
    assert "0x519ACE0519ACE000" in text


@pytest.mark.gpu
def test_cpp_operator_tests_pass(tmp_path):
    out = subprocess.run([BIN, str(tmp_path)], capture_output=True, text=True, timeout=300)
    print(out.stdout[-4000:])
    print(out.stderr[-2000:])
    assert out.returncode == 0, out.stdout[-2000:] + out.stderr[-2000:]
    assert "[ PASSED ]" in out.stdout


@pytest.mark.gpu
def test_cpp_operator_loads_the_arm_quantizers_blob(tmp_path):
    """Writes a .mllm file that holds each test layer twice: as the interleaved blob the reference's
    Arm quantizer stores (python restatement of KleidiAI's packing: parity unpinned) and as this
    backend's row-major blob; the C++ test loads both through HipLinearOp::load and demands identical
    outputs."""
    import numpy as np

    import kai_blob
    from mllm_file import write

    params = {}
    rng = np.random.default_rng(5)
    for tile, N, K in [(5, 50, 256), (7, 56, 96), (8, 13, 64), (3, 256, 1536)]:
        nr, kr, sr = kai_blob.TILE_PARAMS[tile]
        u4 = rng.integers(0, 256, size=(N, K // 2), dtype=np.uint8)
        scales = ((rng.standard_normal((N, K // 32)) * 0.01).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        bias = rng.standard_normal(N).astype(np.float32)
        params[f"kai{tile}.weight"] = kai_blob.pack(u4, scales, bias, nr, kr, sr).view(np.int8)
        params[f"kai{tile}.bias"] = np.zeros(1, dtype=np.int8)          # KaiQuantizationPass.cpp:180-184
        native = np.concatenate([u4.ravel(), scales.ravel().view(np.uint8), bias.view(np.uint8)])
        params[f"nat{tile}.weight"] = native.view(np.int8)
        params[f"nat{tile}.bias"] = np.zeros(1, dtype=np.int8)
    write(os.path.join(str(tmp_path), "kai_layers.mllm"), "kai-blobs", params)
    out = subprocess.run([BIN, str(tmp_path)], capture_output=True, text=True, timeout=300)
    print(out.stdout[-3000:])
    print(out.stderr[-2000:])
    assert out.returncode == 0 and "[ PASSED ]" in out.stdout
    assert out.stdout.count("outputs identical") == 4 and "[ SKIP ]" not in out.stdout


@pytest.mark.gpu
def test_cpp_model_generates_what_the_oracle_generates(tmp_path):
    """The C++ model class writes a tiny Qwen2-shaped .mllm file under the reference's parameter
    names, loads it and generates greedily (prefill in two slices, first step eager, the rest from a
    HIP graph). The same file is read here and run through the numpy oracle, teacher-forced with the
    tokens the binary printed: every printed token must be the oracle's greedy choice."""
    import numpy as np

    import decoder_oracle as do
    from mllm_file import read

    out = subprocess.run([BIN_MODEL, str(tmp_path)], capture_output=True, text=True, timeout=300)
    print(out.stdout[-3000:])
    print(out.stderr[-2000:])
    assert out.returncode == 0 and "[ PASSED ]" in out.stdout
    line = [l for l in out.stdout.splitlines() if l.startswith("TOKENS:")][0]
    tokens = [int(t) for t in line.split()[1:]]
    assert len(tokens) == 14

    model_name, p = read(os.path.join(str(tmp_path), "tiny_qwen2.mllm"))
    assert model_name == "tiny-qwen2" and p["model.embed_tokens.weight"].shape == (640, 256)
    layers = []
    for i in range(2):
        b = f"model.layers.{i}."
        layers.append({
            "q": p[b + "self_attn.q_proj.weight"], "q_bias": p[b + "self_attn.q_proj.bias"],
            "k": p[b + "self_attn.k_proj.weight"], "k_bias": p[b + "self_attn.k_proj.bias"],
            "v": p[b + "self_attn.v_proj.weight"], "v_bias": p[b + "self_attn.v_proj.bias"],
            "o": p[b + "self_attn.o_proj.weight"], "gate": p[b + "mlp.gate_proj.weight"],
            "up": p[b + "mlp.up_proj.weight"], "down": p[b + "mlp.down_proj.weight"],
            "attn_norm": p[b + "input_layernorm.weight"], "ffn_norm": p[b + "post_attention_layernorm.weight"]})
    weights = {"embedding": p["model.embed_tokens.weight"], "final_norm": p["model.norm.weight"],
               "lm_head": p["lm_head.weight"], "layers": layers}
    # lm_head.weight is f32 in this file: the model class applies it as a dense matmul, as the reference does
    ref = do.Decoder(weights, 2, 1, rope_theta=1e6, max_seq=64, lm_head_dense=True)
    prompt = [3, 17, 100, 42, 7, 250, 611, 5, 98, 301, 77]
    logits = ref.forward(prompt)
    margins = []
    for i, tok in enumerate(tokens):
        top2 = np.sort(logits)[-2:]
        margins.append(float(top2[1] - top2[0]))
        # the oracle's choice, unless its two best logits are closer than the 2e-3 parity tolerance
        assert do.greedy(logits) == tok or margins[-1] < 2e-3 * float(np.abs(logits).max()), (i, tok)
        if i + 1 < len(tokens):
            logits = ref.forward([tok])
    assert max(margins) > 0.01        # the comparison was not vacuous


@pytest.mark.gpu
def test_cpp_model_loads_a_file_with_the_reference_quantizers_dtypes(tmp_path, orc):
    """One tiny model written twice under the reference's parameter names:
      A  with the dtypes of the reference's W4A32 quantizer configuration
         (scripts/QuantCfg/ds_qwen2/1.5B-W4A32-KAI.json:33-45): the three RMSNorm weights and lm_head.weight as
         Fp16, every Linear as an int8 W4 blob (this build's row-major blob, quantised here by the CPU oracle)
         with the 1-byte bias placeholder of KaiQuantizationPass.cpp:180-184, the embedding f32;
      B  all in f32, holding the values that A's Fp16 tensors widen to.
    The C++ model class loads each (lm_head applied densely, as modeling_ds_qwen2.hpp:209-213 does), generates,
    and must print the same tokens and leave the same logits, bit for bit; the tokens are the numpy oracle's
    greedy choices on A's values."""
    import numpy as np

    import decoder_oracle as do
    from mllm_file import write

    H, Hq, Hkv, I, V, L = 256, 2, 1, 384, 640, 2
    qd, kvd = Hq * 128, Hkv * 128
    rng = np.random.default_rng(77)
    f32 = np.float32
    rw = lambda n, k: (rng.standard_normal((n, k)) * 0.05).astype(f32)
    half = lambda a: a.astype(np.float16)

    A, B, layers = {}, {}, []

    def linear(name, w, bias=None):
        u4, sc = orc.quant_rhs(w)
        b = np.zeros(w.shape[0], f32) if bias is None else bias
        A[name + ".weight"] = np.concatenate([u4.ravel(), sc.ravel().view(np.uint8), b.view(np.uint8)]).view(np.int8)
        B[name + ".weight"] = w
        if bias is not None:
            A[name + ".bias"] = np.zeros(1, dtype=np.int8)
            B[name + ".bias"] = bias

    def half_param(name, a):
        A[name] = half(a)
        B[name] = half(a).astype(f32)
        return B[name]

    emb = rng.standard_normal((V, H)).astype(f32)
    A["model.embed_tokens.weight"] = B["model.embed_tokens.weight"] = emb
    for i in range(L):
        b = f"model.layers.{i}."
        lw = {"q": rw(qd, H), "q_bias": (rng.standard_normal(qd) * 0.1).astype(f32),
              "k": rw(kvd, H), "k_bias": (rng.standard_normal(kvd) * 0.1).astype(f32),
              "v": rw(kvd, H), "v_bias": (rng.standard_normal(kvd) * 0.1).astype(f32),
              "o": rw(H, qd), "gate": rw(I, H), "up": rw(I, H), "down": rw(H, I)}
        lw["attn_norm"] = half_param(b + "input_layernorm.weight", (1 + 0.1 * rng.standard_normal(H)).astype(f32))
        for n in ("q", "k", "v"):
            linear(b + f"self_attn.{n}_proj", lw[n], lw[n + "_bias"])
        linear(b + "self_attn.o_proj", lw["o"])
        lw["ffn_norm"] = half_param(b + "post_attention_layernorm.weight", (1 + 0.1 * rng.standard_normal(H)).astype(f32))
        for n in ("gate", "up", "down"):
            linear(b + f"mlp.{n}_proj", lw[n])
        layers.append(lw)
    final_norm = half_param("model.norm.weight", (1 + 0.1 * rng.standard_normal(H)).astype(f32))
    lm_head = half_param("lm_head.weight", rw(V, H))
    assert A["lm_head.weight"].dtype == np.float16 and A["model.norm.weight"].dtype == np.float16

    results = {}
    for tag, params in (("A", A), ("B", B)):
        path = os.path.join(str(tmp_path), f"tiny_{tag}.mllm")
        write(path, "tiny-qwen2", params)
        out = subprocess.run([BIN_MODEL, str(tmp_path), "--load", path], capture_output=True, text=True, timeout=300)
        print(out.stdout[-2000:])
        print(out.stderr[-2000:])
        assert out.returncode == 0 and "[ PASSED ]" in out.stdout
        line = [l for l in out.stdout.splitlines() if l.startswith("TOKENS:")][0]
        results[tag] = ([int(t) for t in line.split()[1:]], np.fromfile(path + ".logits", dtype=f32))
    assert results["A"][0] == results["B"][0] and len(results["A"][0]) == 14
    assert results["A"][1].shape == (V,) and np.array_equal(results["A"][1], results["B"][1])

    weights = {"embedding": emb, "final_norm": final_norm, "lm_head": lm_head, "layers": layers}
    ref = do.Decoder(weights, Hq, Hkv, rope_theta=1e6, max_seq=64, lm_head_dense=True)
    logits = ref.forward([3, 17, 100, 42, 7, 250, 611, 5, 98, 301, 77])
    tokens, margins = results["A"][0], []
    for i, tok in enumerate(tokens):
        top2 = np.sort(logits)[-2:]
        margins.append(float(top2[1] - top2[0]))
        assert do.greedy(logits) == tok or margins[-1] < 2e-3 * float(np.abs(logits).max()), (i, tok)
        if i + 1 < len(tokens):
            logits = ref.forward([tok])
    assert max(margins) > 0.01
    # the logits the binary left are those of its last step, which fed tokens[-2] and chose tokens[-1]
    from conftest import max_abs_rel
    assert max_abs_rel(results["A"][1], logits) < 2e-3


@pytest.mark.gpu
def test_cpp_decoder_operator_by_operator_matches_the_runner(tmp_path):
    """Every decoder operator as an op class of the HIP backend (created by its factory from the reference's
    cargo, loaded by the reference's parameter names, run through MllmEngineCtx::dispatch in the order of
    the reference's flash-attention model variant) generates what the fused runner generates; the dense MatMul
    operator matches a double-precision product; repeated steps take no new device allocation."""
    out = subprocess.run([BIN_OPS, str(tmp_path)], capture_output=True, text=True, timeout=300)
    print(out.stdout[-4000:])
    print(out.stderr[-2000:])
    assert out.returncode == 0 and "[ PASSED ]" in out.stdout
    assert "TIMING:" in out.stdout and "Trying to expand KVCache" in out.stderr

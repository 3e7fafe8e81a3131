// The decoder model class end to end: a small random Qwen2-shaped model is written to a .mllm
// file under the reference's parameter names, loaded back through ParameterLoader, and run with
// greedy generation. Checks here are the ones that need no second implementation: the decode path
// (fused launches, HIP graph replay) must continue exactly what the prefill path (separate
// operators on all rows) predicts, and generation must be reproducible. The Python test that runs
// this binary reads the same file and compares the printed tokens with the CPU oracle's.
// Needs a GPU. Usage: hip_qwen2_test <directory>
//        hip_qwen2_test <directory> --load <file.mllm>   loads that file instead (same tiny configuration),
//            generates, prints the tokens and writes the last step's logits to <file.mllm>.logits (raw f32):
//            for the Python test that writes one model twice, once with the dtypes of the reference's W4A32
//            quantizer configuration (Fp16 norm weights and lm_head, int8 W4 blobs) and once all in f32
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "mllm/Backends/HIP/HipBackend.hpp"
#include "mllm/Engine/Context.hpp"
#include "mllm/Engine/ParameterReader.hpp"
#include "mllm/Models/ds_qwen2/HipQwen2.hpp"

using namespace mllm;  // NOLINT

static int g_failed = 0;
#define EXPECT(cond)                                                   \
  do {                                                                 \
    if (!(cond)) {                                                     \
      std::printf("  EXPECT failed: %s (line %d)\n", #cond, __LINE__); \
      ++g_failed;                                                      \
    }                                                                  \
  } while (0)

static void addParam(const std::shared_ptr<ParameterLoader>& params, const std::string& name,
                     const std::vector<int32_t>& shape, std::mt19937& gen, float std_dev, float mean) {
  Tensor t = Tensor::empty(shape, kFp32, kCPU).alloc();
  std::normal_distribution<float> d(mean, std_dev);
  auto* p = t.ptr<float>();
  for (size_t i = 0; i < t.numel(); ++i) p[i] = d(gen);
  t.setName(name);
  params->insert(name, t);
}

int main(int argc, char** argv) {
  const std::string dir = argc > 1 ? argv[1] : "/tmp";
  auto& ctx = MllmEngineCtx::instance();
  ctx.registerBackend(hip::createHostBackend());
  ctx.registerBackend(hip::createHipBackend());

  models::HipQWenConfig cfg;
  cfg.num_attention_heads = 2;
  cfg.num_key_value_heads = 1;
  cfg.num_hidden_layers = 2;
  cfg.hidden_size = 256;
  cfg.intermediate_size = 384;
  cfg.vocab_size = 640;
  cfg.max_cache_length = 64;
  cfg.rope_theta = 1e6f;
  cfg.eos_token_id = -1;  // never produced: generation runs to max_length
  cfg.max_prompt_chunk = 8;  // the 11-token prompt below goes in as two slices

  const bool load_only = argc > 3 && std::string(argv[2]) == "--load";
  if (load_only) {
    std::printf("[ RUN      ] load %s, generate\n", argv[3]);
    auto file = load(argv[3]);
    models::HipQWenForCausalLM m(cfg);
    m.load(file);
    const std::vector<int64_t> prompt = {3, 17, 100, 42, 7, 250, 611, 5, 98, 301, 77};
    std::vector<int64_t> gen = m.generate(prompt, 24);
    std::printf("TOKENS:");
    for (auto t : gen) std::printf(" %lld", (long long)t);
    std::printf("\n");
    const std::vector<float> logits = m.lastLogits();
    const std::string out = std::string(argv[3]) + ".logits";
    std::FILE* f = std::fopen(out.c_str(), "wb");
    EXPECT(f != nullptr);
    if (f) {
      EXPECT(std::fwrite(logits.data(), sizeof(float), logits.size(), f) == logits.size());
      std::fclose(f);
    }
    std::printf(g_failed ? "[  FAILED  ]\n" : "[ PASSED ]\n");
    return g_failed ? 1 : 0;
  }

  // ---- write the model file under the reference's parameter names
  std::printf("[ RUN      ] write + load .mllm\n");
  const std::string path = dir + "/tiny_qwen2.mllm";
  {
    std::mt19937 gen(1234);
    auto params = std::make_shared<ParameterLoader>();
    const int H = cfg.hidden_size, I = cfg.intermediate_size, V = cfg.vocab_size;
    const int qd = 256, kvd = 128;
    addParam(params, "model.embed_tokens.weight", {V, H}, gen, 1.0f, 0.0f);
    for (int i = 0; i < cfg.num_hidden_layers; ++i) {
      const std::string b = "model.layers." + std::to_string(i) + ".";
      addParam(params, b + "input_layernorm.weight", {H}, gen, 0.1f, 1.0f);
      addParam(params, b + "self_attn.q_proj.weight", {qd, H}, gen, 0.05f, 0.0f);
      addParam(params, b + "self_attn.q_proj.bias", {qd}, gen, 0.1f, 0.0f);
      addParam(params, b + "self_attn.k_proj.weight", {kvd, H}, gen, 0.05f, 0.0f);
      addParam(params, b + "self_attn.k_proj.bias", {kvd}, gen, 0.1f, 0.0f);
      addParam(params, b + "self_attn.v_proj.weight", {kvd, H}, gen, 0.05f, 0.0f);
      addParam(params, b + "self_attn.v_proj.bias", {kvd}, gen, 0.1f, 0.0f);
      addParam(params, b + "self_attn.o_proj.weight", {H, qd}, gen, 0.05f, 0.0f);
      addParam(params, b + "post_attention_layernorm.weight", {H}, gen, 0.1f, 1.0f);
      addParam(params, b + "mlp.gate_proj.weight", {I, H}, gen, 0.05f, 0.0f);
      addParam(params, b + "mlp.up_proj.weight", {I, H}, gen, 0.05f, 0.0f);
      addParam(params, b + "mlp.down_proj.weight", {H, I}, gen, 0.05f, 0.0f);
    }
    addParam(params, "model.norm.weight", {H}, gen, 0.1f, 1.0f);
    addParam(params, "lm_head.weight", {V, H}, gen, 0.05f, 0.0f);
    write(path, params->params(), "tiny-qwen2");
  }
  auto loaded = load(path);
  EXPECT(loaded->has("model.layers.1.mlp.down_proj.weight") && loaded->has("lm_head.weight"));

  models::HipQWenForCausalLM model(cfg);
  model.load(loaded);
  std::printf("[       OK ]\n");

  // ---- generation
  std::printf("[ RUN      ] greedy generation, decode path continues what prefill predicts\n");
  const std::vector<int64_t> prompt = {3, 17, 100, 42, 7, 250, 611, 5, 98, 301, 77};
  const int total = 24;
  std::vector<int64_t> gen = model.generate(prompt, total);
  EXPECT((int)gen.size() == total - (int)prompt.size() + 1);
  EXPECT(model.position() == total);
  std::printf("TOKENS:");
  for (auto t : gen) std::printf(" %lld", (long long)t);
  std::printf("\n");
  for (auto t : gen) EXPECT(t >= 0 && t < cfg.vocab_size);

  // same prompt again: identical tokens (state fully re-initialised by position 0)
  model.reset();
  std::vector<int64_t> again = model.generate(prompt, total);
  EXPECT(again == gen);

  // teacher forcing through the prefill path: feeding prompt + the first i generated tokens as one
  // prompt must predict generated token i (separate operators on all rows vs fused single-row launches)
  int agree = 0, checked = 0;
  for (int i : {1, 4, 9}) {
    std::vector<int64_t> longer(prompt);
    longer.insert(longer.end(), gen.begin(), gen.begin() + i);
    model.reset();
    const int64_t predicted = model.prefill(longer);
    ++checked;
    if (predicted == gen[i]) ++agree;
    std::vector<float> logits = model.lastLogits();
    EXPECT((int)logits.size() == cfg.vocab_size);
    int best = 0;
    for (int v = 1; v < cfg.vocab_size; ++v) {
      if (logits[v] > logits[best]) best = v;
    }
    EXPECT(best == predicted);  // the device argmax is the first maximum of the logits it leaves
  }
  EXPECT(agree == checked);
  std::printf("[       OK ]\n");

  if (g_failed) {
    std::printf("[  FAILED  ] %d expectation(s)\n", g_failed);
    return 1;
  }
  std::printf("[ PASSED ]\n");
  return 0;
}

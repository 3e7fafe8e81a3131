// Operator-level tests of the HIP W4A32 Linear, written the way the reference tests its Arm
// kernel (tests/Arm/KaiLinearTest.hpp:387-470: build inputs, CalculateRef with the scalar model,
// Calculate through the library, Compare) but driven through the engine boundary:
// registerBackend -> createOp -> load -> dispatch (reshape/setup/forward) -> D2H.
// The scalar model is the CPU oracle (test infrastructure). Needs a GPU.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <stdexcept>
#include <string>
#include <vector>

#include "mllm/Backends/HIP/HipBackend.hpp"
#include "mllm/Backends/HIP/Ops/LinearOp.hpp"
#include "mllm/Engine/Context.hpp"
#include "mllm/Engine/ParameterReader.hpp"
#include "mllm/Utils/Log.hpp"
#include "w4a32_oracle.h"

using namespace mllm;  // NOLINT

static int g_failed = 0;
#define EXPECT(cond)                                                         \
  do {                                                                       \
    if (!(cond)) {                                                           \
      std::printf("  EXPECT failed: %s (line %d)\n", #cond, __LINE__);       \
      ++g_failed;                                                            \
    }                                                                        \
  } while (0)

static const LinearOpImplType kW4 =
    LinearOpImplType::kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp4x8_qsi4c32p4x8_8x4x32;

static Tensor hostTensor(const std::vector<int32_t>& shape, DataTypes dt, const void* src) {
  Tensor t = Tensor::empty(shape, dt, kCPU).alloc();
  if (src) std::memcpy(t.ptr<void>(), src, t.bytes());
  return t;
}

static std::vector<float> normal(size_t n, float std_dev, unsigned seed) {
  std::mt19937 gen(seed);
  std::normal_distribution<float> d(0.0f, std_dev);
  std::vector<float> v(n);
  for (auto& x : v) x = d(gen);
  return v;
}

// CalculateRef: the scalar model on the same inputs.
static std::vector<float> calculateRef(int M, int K, int N, const std::vector<float>& x,
                                       const std::vector<float>& w, const float* bias) {
  std::vector<uint8_t> u4((size_t)N * K / 2);
  std::vector<uint16_t> sc((size_t)N * K / 32);
  orc_quant_rhs_qs4c32(N, K, 32, w.data(), u4.data(), sc.data(), 0);
  std::vector<float> y((size_t)M * N);
  orc_linear_w4a32(M, N, K, x.data(), u4.data(), sc.data(), bias, y.data(), 8);
  return y;
}

static double maxAbsRel(const std::vector<float>& a, const std::vector<float>& b) {
  EXPECT(a.size() == b.size() && !a.empty());
  double num = 0, den = 0;
  for (size_t i = 0; i < a.size(); ++i) {
    num = std::max(num, std::fabs((double)a[i] - b[i]));
    den = std::max(den, std::fabs((double)b[i]));
  }
  EXPECT(den > 1e-3);  // a trivial (all-zero) reference would make any output look right
  return num / den;
}

// Calculate: through the engine boundary.
static std::vector<float> calculate(const std::shared_ptr<BaseOp>& op, const std::vector<int32_t>& in_shape,
                                    const std::vector<float>& x, std::vector<int32_t>* out_shape) {
  auto& ctx = MllmEngineCtx::instance();
  ctx.regLayerOp(op->name(), op);
  Tensor xd = hip::toDevice(hostTensor(in_shape, kFp32, x.data()));
  auto outs = ctx.dispatch(op->name(), {xd});
  D2HOpCargo d2h;  // as Tensor::cpu() fills it (mllm/Core/Tensor.cpp)
  d2h.from_device_type = outs[0].device();
  d2h.to_device_type = kCPU;
  auto host = ctx.dispatch(OpType::kD2H, d2h, {outs[0]});
  if (out_shape) *out_shape = host[0].shape();
  EXPECT(host[0].dtype() == kFp32 && host[0].device() == kCPU && outs[0].device() == kHIP);
  return std::vector<float>(host[0].ptr<float>(), host[0].ptr<float>() + host[0].numel());
}

static std::shared_ptr<BaseOp> makeLinear(const std::string& name, int K, int N, bool bias,
                                          LinearOpImplType impl = kW4) {
  LinearOpCargo cargo;
  cargo.in_channels = K;
  cargo.out_channels = N;
  cargo.bias = bias;
  cargo.impl_type_ = impl;
  auto op = MllmEngineCtx::instance().getBackend(kHIP)->createOp(OpType::kLinear, cargo);
  op->setName(name);
  return op;
}

// The reference's own test protocol: M=1, K=N=1024, uniform[-1,1] from srand(4568)/srand(4572),
// no bias, |ref - act| <= 1e-4 (tests/Arm/KaiLinearTest.hpp:391-392, 456-464, 473-476).
static void testReferenceProtocol() {
  std::printf("[ RUN ] KaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk reference protocol\n");
  const int M = 1, K = 1024, N = 1024;
  std::vector<float> x((size_t)M * K), w((size_t)N * K);
  orc_fill_uniform_random(M, K, x.data(), 4568);
  orc_fill_uniform_random(N, K, w.data(), 4572);
  auto params = std::make_shared<ParameterLoader>();
  params->insert("t0.weight", hostTensor({N, K}, kFp32, w.data()));
  auto op = makeLinear("t0", K, N, false);
  op->load(params);
  auto act = calculate(op, {M, K}, x, nullptr);
  auto ref = calculateRef(M, K, N, x, w, nullptr);
  double worst = 0;
  for (size_t i = 0; i < ref.size(); ++i) worst = std::max(worst, std::fabs((double)ref[i] - act[i]));
  std::printf("  max |ref - act| = %.3g (bar 1e-4); ref[0..2] = %g %g %g, act[0..2] = %g %g %g\n", worst,
              ref[0], ref[1], ref[2], act[0], act[1], act[2]);
  EXPECT(std::fabs(ref[0]) > 1e-3 && maxAbsRel(act, ref) <= 1e-3);
  EXPECT(worst <= 1e-4);
}

// Qwen2-1.5B shaped layers through a parameter file, f32 weights quantised at load.
static void testFromF32File(const char* dir) {
  std::printf("[ RUN ] load f32 .mllm, decode and prefill shapes\n");
  struct Case { const char* name; int K, N; bool bias; int M; double tol; };
  const Case cases[] = {{"model.layers.0.self_attn.q_proj", 1536, 1536, true, 1, 1e-3},
                        {"model.layers.0.self_attn.k_proj", 1536, 256, true, 4, 1e-3},
                        {"model.layers.0.mlp.gate_proj", 1536, 8960, false, 8, 1e-3},
                        {"model.layers.0.mlp.down_proj", 8960, 1536, false, 1, 1e-3},
                        {"model.layers.0.self_attn.v_proj", 1536, 256, true, 128, 2e-3},
                        // few output tiles, long K: the op lends the backend's scratch for split-K
                        {"model.layers.1.mlp.down_proj", 8960, 1536, false, 96, 2e-3}};
  auto params = std::make_shared<ParameterLoader>();
  std::vector<std::vector<float>> ws, bs;
  unsigned seed = 1;
  for (const auto& c : cases) {
    ws.push_back(normal((size_t)c.N * c.K, 0.02f, seed++));
    bs.push_back(normal((size_t)c.N, 0.02f, seed++));
    params->insert(std::string(c.name) + ".weight", hostTensor({c.N, c.K}, kFp32, ws.back().data()));
    if (c.bias) params->insert(std::string(c.name) + ".bias", hostTensor({c.N}, kFp32, bs.back().data()));
  }
  const std::string path = std::string(dir) + "/f32_layers.mllm";
  mllm::write(path, params->params(), "qwen2-1.5b-shapes");
  auto loaded = mllm::load(path);
  EXPECT(loaded->modelName() == "qwen2-1.5b-shapes");
  EXPECT(loaded->params().size() == params->params().size());
  for (size_t ci = 0; ci < sizeof(cases) / sizeof(cases[0]); ++ci) {
    const auto& c = cases[ci];
    auto op = makeLinear(c.name, c.K, c.N, c.bias);
    op->load(loaded);
    auto x = normal((size_t)c.M * c.K, 1.0f, 100 + ci);
    std::vector<int32_t> oshape;
    auto act = calculate(op, {1, c.M, c.K}, x, &oshape);  // [B, S, D] as the model code passes
    EXPECT((oshape == std::vector<int32_t>{1, c.M, c.N}));
    auto ref = calculateRef(c.M, c.K, c.N, x, ws[ci], c.bias ? bs[ci].data() : nullptr);
    const double err = maxAbsRel(act, ref);
    std::printf("  %-34s M=%-4d max-abs-rel %.3g (bar %.0e)\n", c.name, c.M, err, c.tol);
    EXPECT(err <= c.tol);
  }
}

// Offline quantizer -> file with int8 blob + 1-byte bias placeholder -> load -> same outputs.
static void testQuantizedFile(const char* dir) {
  std::printf("[ RUN ] quantize to file, reload, compare with quantise-at-load\n");
  const int K = 1536, N = 256, M = 3;
  auto w = normal((size_t)N * K, 0.02f, 7);
  auto b = normal((size_t)N, 0.02f, 8);
  auto x = normal((size_t)M * K, 1.0f, 9);
  Tensor wt = hostTensor({N, K}, kFp32, w.data());
  Tensor bt = hostTensor({N}, kFp32, b.data());

  auto f32_params = std::make_shared<ParameterLoader>();
  f32_params->insert("lin.weight", wt);
  f32_params->insert("lin.bias", bt);
  auto op_a = makeLinear("lin", K, N, true);
  op_a->load(f32_params);
  auto y_a = calculate(op_a, {M, K}, x, nullptr);

  Tensor blob = hip::quantizeLinearForFile(wt, bt);
  EXPECT(blob.dtype() == kInt8 && blob.numel() == hip::HipLinearOp::nativeBlobBytes(N, K));
  auto q_params = std::make_shared<ParameterLoader>();
  q_params->insert("lin.weight", blob);
  const int8_t dummy = 0;
  q_params->insert("lin.bias", hostTensor({1}, kInt8, &dummy));  // as KaiQuantizationPass.cpp:180-184
  const std::string path = std::string(dir) + "/w4_layers.mllm";
  mllm::write(path, q_params->params(), "mllm");
  auto loaded = mllm::load(path);
  EXPECT(Tensor((*loaded)["lin.weight"]).dtype() == kInt8);
  auto op_b = makeLinear("lin", K, N, true);
  op_b->load(loaded);
  auto y_b = calculate(op_b, {M, K}, x, nullptr);
  EXPECT(y_a == y_b);  // bit-identical: same nibbles, scales, bias
  auto ref = calculateRef(M, K, N, x, w, b.data());
  EXPECT(maxAbsRel(y_b, ref) <= 1e-3);
}

// A file that holds, for three of the reference's tiles, the same quantised layer twice: as the blob
// the reference's Arm quantizer would store (KleidiAI's interleaved layout, written by the python
// restatement of that layout: parity unpinned) and as this backend's row-major blob. Both must load
// to the same device weights: identical outputs.
static void testKaiFile(const char* dir) {
  const std::string path = std::string(dir) + "/kai_layers.mllm";
  if (FILE* f = std::fopen(path.c_str(), "rb")) {
    std::fclose(f);
  } else {
    std::printf("[ SKIP ] no %s\n", path.c_str());
    return;
  }
  std::printf("[ RUN ] load blobs in the Arm quantizer's layout\n");
  struct Case { int tile, N, K; };
  const Case cases[] = {{5, 50, 256}, {7, 56, 96}, {8, 13, 64}, {3, 256, 1536}};
  auto loaded = mllm::load(path);
  const int M = 3;
  for (const auto& c : cases) {
    const auto impl = static_cast<LinearOpImplType>(c.tile);
    auto op_k = makeLinear("kai" + std::to_string(c.tile), c.K, c.N, true, impl);
    auto op_n = makeLinear("nat" + std::to_string(c.tile), c.K, c.N, true, impl);
    op_k->load(loaded);
    op_n->load(loaded);
    auto x = normal((size_t)M * c.K, 1.0f, 40 + c.tile);
    auto y_k = calculate(op_k, {M, c.K}, x, nullptr);
    auto y_n = calculate(op_n, {M, c.K}, x, nullptr);
    double mx = 0;
    for (float v : y_n) mx = std::max(mx, (double)std::fabs(v));
    std::printf("  tile %d N=%d K=%d: outputs %s, max |y| %.3g\n", c.tile, c.N, c.K,
                y_k == y_n ? "identical" : "DIFFER", mx);
    EXPECT(y_k == y_n);
    EXPECT(mx > 0);
  }
}

static void testImplTypeStrings() {
  std::printf("[ RUN ] implType strings\n");
  using C = LinearOpCargo;
  EXPECT(static_cast<int>(C::parseLinearOpImplTypeStr(
             "KaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk:qai8dxp4x8_qsi4c32p4x8_8x4x32")) == 5);
  EXPECT(static_cast<int>(C::parseLinearOpImplTypeStr(
             "KaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk:qai8dxp1x8_qsi4c32p4x8_1x4x32")) == 3);
  EXPECT(static_cast<int>(C::parseLinearOpImplTypeStr(
             "KaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk:qai8dxp1x4_qsi4c32p4x4_1x4")) == 8);
  EXPECT(static_cast<int>(C::parseLinearOpImplTypeStr("KaiLinear_fp16_fp16_fp16p_mxk_kxn")) == 2);
  EXPECT(static_cast<int>(C::parseLinearOpImplTypeStr("Kai_End")) == 256);
  EXPECT(C::parseLinearOpImplTypeStr("no such impl") == LinearOpImplType::kDefault);
}

// Error paths end in MLLM_ERROR_EXIT; the handler is swapped for one that throws so they can be
// observed in-process. Nothing here launches a kernel.
static void testErrors() {
  std::printf("[ RUN ] error behaviour\n");
  auto saved = errorHandler();
  errorHandler() = [](int code, const std::string& msg) { throw std::runtime_error(std::to_string(code) + ":" + msg); };
  auto expectThrow = [](const char* what, const std::function<void()>& fn) {
    bool thrown = false;
    try { fn(); } catch (const std::runtime_error& e) { thrown = true; std::printf("  %s -> %s\n", what, e.what()); }
    EXPECT(thrown);
  };
  auto params = std::make_shared<ParameterLoader>();
  std::vector<float> w(64 * 64, 0.01f);
  params->insert("a.weight", hostTensor({64, 64}, kFp32, w.data()));
  expectThrow("default impl type", [&] { makeLinear("a", 64, 64, false, LinearOpImplType::kDefault)->load(params); });
  expectThrow("missing parameter", [&] { makeLinear("nope", 64, 64, false)->load(params); });
  expectThrow("K % 32 != 0", [&] { makeLinear("a", 48, 64, false)->load(params); });
  expectThrow("wrong weight shape", [&] { makeLinear("a", 64, 32, false)->load(params); });
  std::vector<int8_t> odd((size_t)64 * (64 / 2 + 64 / 32 * 2 + 8) + 3, 0);
  params->insert("k.weight", hostTensor({(int32_t)odd.size()}, kInt8, odd.data()));
  expectThrow("int8 blob of no known size", [&] { makeLinear("k", 64, 64, false)->load(params); });
  expectThrow("forward before load", [&] {
    auto op = makeLinear("a", 64, 64, false);
    std::vector<float> x(64, 1.0f);
    std::vector<Tensor> outs;
    Tensor xd = hip::toDevice(hostTensor({1, 64}, kFp32, x.data()));
    op->reshape({xd}, outs);
    op->setup({xd}, outs);
    op->forward({xd}, outs);
  });
  expectThrow("bad cargo type", [&] {
    try { MllmEngineCtx::instance().getBackend(kHIP)->createOp(OpType::kLinear, D2HOpCargo{}); }
    catch (const std::bad_cast&) { throw std::runtime_error("bad_cast"); }
  });
  errorHandler() = saved;
}

int main(int argc, char** argv) {
  const char* dir = argc > 1 ? argv[1] : "/tmp";
  setvbuf(stdout, nullptr, _IOLBF, 0);
  auto& ctx = MllmEngineCtx::instance();
  ctx.registerBackend(hip::createHostBackend());
  ctx.registerBackend(hip::createHipBackend());
  testImplTypeStrings();
  testErrors();
  testReferenceProtocol();
  testFromF32File(dir);
  testQuantizedFile(dir);
  testKaiFile(dir);
  hip::currentHipBackend().synchronize();
  ctx.shutdown();
  std::printf(g_failed ? "[ FAILED ] %d expectation(s)\n" : "[ PASSED ]%.0d\n", g_failed);
  return g_failed ? 1 : 0;
}

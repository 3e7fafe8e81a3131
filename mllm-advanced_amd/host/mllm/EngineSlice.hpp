// The slice of the reference engine that the HIP backend is compiled against when it is built outside the
// reference tree: device and data type keys, logging, storage and allocator, tensor, operator base classes,
// the Linear operator's abstract half, backend base, context and the parameter file reader. Inside the
// reference tree the headers of these names (the one-line files beside this one forward to here) are the
// reference's own, and this file is not used. Signatures follow the reference so that mllm/Backends/HIP and
// mllm/Models/ds_qwen2/HipQwen2.* compile unchanged against either; each part cites the file it stands for.
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <memory>
#include <string>
#include <typeinfo>
#include <unordered_map>
#include <vector>

// ====================================================================================================
// stands for mllm/Utils/Log.hpp
// ====================================================================================================
// Error convention of the engine this layer plugs into: no exceptions, no status codes; an
// unrecoverable condition prints and exits with a code (reference: mllm/Utils/Log.hpp:59-64,
// codes mllm/Utils/Common.hpp:23-30). The handler is replaceable so tests can observe it.


namespace mllm {

enum ExitCode : int {  // NOLINT
  kSuccess = 0,
  kCoreError = 1,
  kAssert = 2,
  kIOError = 3,
  kHipError = 4,
  kShapeError = 5,
};

inline std::function<void(int, const std::string&)>& errorHandler() {
  static std::function<void(int, const std::string&)> h = [](int code, const std::string& msg) {
    std::fprintf(stderr, "[mllm][ERROR] %s\n", msg.c_str());
    std::fflush(stderr);
    std::exit(code);
  };
  return h;
}

template <typename... Args>
inline std::string formatMsg(const char* fmt, Args... args) {
  char buf[1024];
  std::snprintf(buf, sizeof buf, fmt, args...);
  return std::string(buf);
}
inline std::string formatMsg(const char* fmt) { return std::string(fmt); }

}  // namespace mllm

#define MLLM_ERROR_EXIT(code, ...) ::mllm::errorHandler()((code), ::mllm::formatMsg(__VA_ARGS__))
#define MLLM_WARN(...) std::fprintf(stderr, "[mllm][WARN] %s\n", ::mllm::formatMsg(__VA_ARGS__).c_str())
#define MLLM_INFO(...) std::fprintf(stderr, "[mllm][INFO] %s\n", ::mllm::formatMsg(__VA_ARGS__).c_str())
#define MLLM_RT_ASSERT(expr)                                                                  \
  do {                                                                                        \
    if (!(expr)) MLLM_ERROR_EXIT(::mllm::kAssert, "assert failed: %s (%s:%d)", #expr, __FILE__, __LINE__); \
  } while (0)
#define MLLM_RT_ASSERT_EQ(a, b) MLLM_RT_ASSERT((a) == (b))

// ====================================================================================================
// stands for mllm/Core/DeviceTypes.hpp
// ====================================================================================================
// Device enum of the engine, with the one value this backend adds.
// Reference: mllm/Core/DeviceTypes.hpp:18-27 has kCPU, kCUDA, kOpenCL, kQNN; a backend is looked
// up by this key (mllm/Engine/Context.cpp:56-59), so a new device needs a new enumerator: kHIP.


namespace mllm {

enum DeviceTypes {  // NOLINT
  kDeviceTypes_Start = 0,
  kCPU,
  kCUDA,
  kOpenCL,
  kQNN,
  kHIP,  // added: AMD GPU through HIP (MI355X / gfx950)
  kDeviceTypes_End,
};

inline const char* deviceTypes2Str(DeviceTypes t) {
  static const char* const names[] = {"DeviceTypes_Start", "CPU", "CUDA", "OpenCL", "QNN", "HIP",
                                      "DeviceTypes_End"};
  return (t >= kDeviceTypes_Start && t <= kDeviceTypes_End) ? names[t] : "Unknown";
}

inline DeviceTypes str2DeviceType(const std::string& s) {
  for (int t = kCPU; t < kDeviceTypes_End; ++t) {
    if (s == deviceTypes2Str(static_cast<DeviceTypes>(t))) return static_cast<DeviceTypes>(t);
  }
  return kDeviceTypes_End;
}

}  // namespace mllm

// ====================================================================================================
// stands for mllm/Core/DataTypes.hpp
// ====================================================================================================
// The element types this path touches, with the numeric codes the .mllm container stores
// (reference: mllm/Core/DataTypes.hpp:19-65 - Int8 = 2, Int32 = 4, Int64 = 5, Fp16 = 8, Fp32 = 9, BF16 = 24).


namespace mllm {

enum DataTypes : uint32_t {  // NOLINT
  kInt8 = 2,
  kInt32 = 4,
  kInt64 = 5,
  kFp16 = 8,
  kFp32 = 9,
  kBF16 = 24,
};

inline size_t dataTypeSize(DataTypes t) {
  switch (t) {
    case kInt8: return 1;
    case kFp16:
    case kBF16: return 2;
    case kInt32:
    case kFp32: return 4;
    case kInt64: return 8;
  }
  return 0;
}

inline const char* dataTypes2Str(DataTypes t) {
  switch (t) {
    case kInt8: return "Int8";
    case kInt32: return "Int32";
    case kInt64: return "Int64";
    case kFp16: return "Fp16";
    case kFp32: return "Fp32";
    case kBF16: return "BF16";
  }
  return "Unknown";
}

}  // namespace mllm

// ====================================================================================================
// stands for mllm/Engine/Allocator.hpp
// ====================================================================================================
// Allocator interface a backend hands to the engine (reference: mllm/Engine/Allocator.hpp:18-32,
// same nine virtuals with the same meaning).



namespace mllm {

// reference: mllm/Core/Storage.hpp:20-37
class Storage : public std::enable_shared_from_this<Storage> {
 public:
  virtual ~Storage() = default;
  void* ptr_ = nullptr;
  size_t size_ = 0;
  DeviceTypes device_ = kCPU;
};

class Allocator {
 public:
  virtual ~Allocator() = default;
  virtual bool ctrlByMllmMemManager() = 0;
  virtual bool alloc(const std::shared_ptr<Storage>& storage) = 0;
  virtual void free(const std::shared_ptr<Storage>& storage) = 0;
  virtual void free(Storage* storage) = 0;
  virtual bool generalAlloc(void** ptr, size_t cap, size_t align) = 0;
  virtual void generalFree(void* ptr) = 0;
  virtual size_t allocSize(Storage* storage) = 0;
  virtual size_t allocSize(const std::shared_ptr<Storage>& storage) = 0;
  [[nodiscard]] virtual size_t alignSize() const = 0;
};

}  // namespace mllm

// ====================================================================================================
// stands for mllm/Core/Tensor.hpp
// ====================================================================================================
// A contiguous tensor over reference-counted storage: the slice of the engine's Tensor that an
// operator boundary needs (reference: mllm/Core/Tensor.hpp:52-140, mllm/Core/TensorImpl.hpp:43-142).
// Tensor::empty() only describes a tensor; alloc() asks the device's allocator for memory, as
// BaseOp::setup does for op outputs (mllm/Core/AOps/BaseOp.cpp:25-46).



namespace mllm {

enum TensorMemTypes : int {  // NOLINT
  kNormal = 0,  // owned: freed through the allocator when the last reference goes
  kParams = 1,  // aliases a mapped parameter file or caller memory: never freed here
};

class TensorStorage : public Storage {
 public:
  ~TensorStorage() override;
  TensorMemTypes mem_type_ = kNormal;
  std::shared_ptr<void> keep_alive_;  // e.g. the mapped file a kParams tensor aliases
};

class TensorViewImpl {
 public:
  using shape_t = std::vector<int32_t>;
  shape_t shape_;
  DataTypes dtype_ = kFp32;
  std::string name_;
  std::shared_ptr<TensorStorage> storage_;
};

class Tensor {
 public:
  using shape_t = TensorViewImpl::shape_t;

  Tensor() = default;
  explicit Tensor(const std::shared_ptr<TensorViewImpl>& impl) : impl_(impl) {}

  [[nodiscard]] bool isNil() const { return impl_ == nullptr; }
  static Tensor nil() { return {}; }

  // Describes a tensor; no memory yet.
  static Tensor empty(const shape_t& shape, DataTypes dtype = kFp32, DeviceTypes device = kCPU);
  // Wraps memory owned by someone else (a mapped file, a caller's buffer).
  static Tensor wrap(void* ptr, const shape_t& shape, DataTypes dtype, DeviceTypes device,
                     std::shared_ptr<void> keep_alive = nullptr);

  Tensor& alloc();

  [[nodiscard]] const shape_t& shape() const { return impl_->shape_; }
  [[nodiscard]] DataTypes dtype() const { return impl_->dtype_; }
  [[nodiscard]] DeviceTypes device() const { return impl_->storage_->device_; }
  [[nodiscard]] size_t numel() const;
  [[nodiscard]] size_t bytes() const { return numel() * dataTypeSize(dtype()); }
  [[nodiscard]] const std::string& name() const { return impl_->name_; }
  void setName(const std::string& n) { impl_->name_ = n; }
  [[nodiscard]] const std::shared_ptr<TensorViewImpl>& impl() const { return impl_; }

  template <typename T>
  [[nodiscard]] T* ptr() const {
    return static_cast<T*>(impl_->storage_->ptr_);
  }

 private:
  std::shared_ptr<TensorViewImpl> impl_;
};

}  // namespace mllm

// ====================================================================================================
// stands for mllm/Core/AOps/BaseOp.hpp
// ====================================================================================================
// Abstract operator API (reference: mllm/Core/AOps/BaseOp.hpp:118-234): the engine calls
// reshape -> setup -> forward on an op that a backend's factory created from a type-erased cargo.



namespace mllm {

class ParameterLoader;

// Only the values this layer uses; kLinear keeps the reference's position-independent name.
enum class OpType : int32_t {
  kOpType_Start = 0,
  kLinear,
  kD2H,
  kOpType_End,
};

inline const char* opType2Str(OpType t) {
  switch (t) {
    case OpType::kLinear: return "Linear";
    case OpType::kD2H: return "D2H";
    default: return "Unknown";
  }
}

// CRTP base of cargos (reference BaseOp.hpp:120-148): per-op thread count, default 4.
template <typename DerivedT>
class BaseOpCargo {
 public:
  [[nodiscard]] int thread() const { return threads_; }
  void setThreads(int threads) { threads_ = threads; }

 private:
  int threads_ = 4;
};

// Type-erased cargo; as<T>() throws std::bad_cast on a wrong type (reference BaseOp.hpp:151-181).
class BaseOpCargoBase {
 public:
  template <typename T>
  BaseOpCargoBase(const T& cargo) : inner_(std::make_shared<Model<T>>(cargo)) {}  // NOLINT

  template <typename T>
  const T& as() const {
    if (auto p = dynamic_cast<const Model<T>*>(inner_.get())) return p->data_;
    throw std::bad_cast();
  }

 private:
  struct Concept {
    virtual ~Concept() = default;
  };
  template <typename T>
  struct Model : Concept {
    explicit Model(const T& d) : data_(d) {}
    T data_;
  };
  std::shared_ptr<Concept> inner_;
};

class BaseOp : public std::enable_shared_from_this<BaseOp> {
 public:
  using params_t = std::unordered_map<std::string, Tensor>;

  explicit BaseOp(OpType op_type) : op_type_(op_type) {}
  virtual ~BaseOp() = default;

  virtual void load(const std::shared_ptr<ParameterLoader>& ploader) {}
  virtual void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {}
  virtual void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {}
  // Allocates every output through its device's allocator (reference BaseOp.cpp:25-46).
  virtual void setup(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs);
  virtual params_t params() { return {}; }

  [[nodiscard]] std::string name() const { return name_; }
  void setName(const std::string& name) { name_ = name; }
  [[nodiscard]] DeviceTypes device() const { return device_type_; }
  void setDeviceType(DeviceTypes d) { device_type_ = d; }
  [[nodiscard]] OpType opType() const { return op_type_; }

 private:
  DeviceTypes device_type_ = kCPU;
  std::string name_;
  OpType op_type_;
};

struct BaseOpFactory {
  virtual ~BaseOpFactory() = default;
  virtual std::shared_ptr<BaseOp> create(const BaseOpCargoBase& base_cargo) = 0;
  [[nodiscard]] virtual OpType opType() const = 0;
};

template <OpType type, typename CargoT>
class TypedOpFactory : public BaseOpFactory {
 public:
  std::shared_ptr<BaseOp> create(const BaseOpCargoBase& base_cargo) override {
    return createOpImpl(base_cargo.as<CargoT>());
  }
  [[nodiscard]] OpType opType() const override { return type; }

 protected:
  virtual std::shared_ptr<BaseOp> createOpImpl(const CargoT& cargo) = 0;
};

}  // namespace mllm

// ====================================================================================================
// stands for mllm/Core/AOps/LinearOp.hpp
// ====================================================================================================
// Linear: cargo, implementation selector and the device-independent part of the op
// (reference: mllm/Core/AOps/LinearOp.hpp:17-99, mllm/Core/AOps/LinearOp.cpp:17-106).



namespace mllm {

// Same enumerators and values as the reference (LinearOp.hpp:17-35): model configs and quantizer
// configs name an implementation by string, the op switches on the value. 3..8 are the six tile
// variants of the W4A32 family KaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk - on this backend they all
// run the same kernels (a tile only selected an Arm micro-kernel and its packed layout).
enum class LinearOpImplType {
  kDefault = 0,
  kKai_Start = 1,
  kKaiLinear_fp16_fp16_fp16p_mxk_kxn = 2,
  kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp1x8_qsi4c32p4x8_1x4x32 = 3,
  kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp1x8_qsi4c32p8x8_1x8x32 = 4,
  kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp4x8_qsi4c32p4x8_8x4x32 = 5,
  kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp4x8_qsi4c32p4x8_16x4x32 = 6,
  kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp4x8_qsi4c32p8x8_4x8x32 = 7,
  kKaiLinear_f32_qai8dxp_qsi4c32p_mxk_nxk_qai8dxp1x4_qsi4c32p4x4_1x4 = 8,
  KaiLinear_f16_qsi8d32p_qai4c32p_mxk_nxk_qsi8d32p1x8_qai4c32p4x8_1x4 = 9,
  KaiLinear_f16_qsi8d32p_qai4c32p_mxk_nxk_qsi8d32p4x4_qai4c32p4x4_8x4 = 10,
  KaiLinear_f16_qsi8d32p_qai4c32p_mxk_nxk_qsi8d32p4x8_qai4c32p4x8_8x4_i8mm = 11,
  kKai_End = 256,
};

inline bool isW4A32ImplType(LinearOpImplType t) {
  const int v = static_cast<int>(t);
  return v >= 3 && v <= 8;
}

struct LinearOpCargo : public BaseOpCargo<LinearOpCargo> {
  int32_t in_channels = 0;
  int32_t out_channels = 0;
  bool bias = true;
  bool transpose = false;
  LinearOpImplType impl_type_ = LinearOpImplType::kDefault;

  // "<family>:<tile>" -> enum; unknown strings warn and fall back to kDefault (LinearOp.cpp:53-55).
  static LinearOpImplType parseLinearOpImplTypeStr(const std::string& type_str);
};

class LinearOp : public BaseOp {
 public:
  explicit LinearOp(const LinearOpCargo& cargo) : BaseOp(OpType::kLinear), cargo_(cargo) {}

  // weight = "<name>.weight", bias = "<name>.bias" when cargo.bias (LinearOp.cpp:60-63)
  void load(const std::shared_ptr<ParameterLoader>& ploader) override;
  // output = input shape with the last dimension replaced by out_channels (LinearOp.cpp:84-94)
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  params_t params() override;

  Tensor& weight() { return weight_; }
  Tensor& bias() { return bias_; }
  [[nodiscard]] const LinearOpCargo& cargo() const { return cargo_; }

 protected:
  Tensor weight_;
  Tensor bias_;
  LinearOpCargo cargo_;
};

}  // namespace mllm

// ====================================================================================================
// stands for mllm/Engine/BackendBase.hpp
// ====================================================================================================
// What a device backend is to the engine (reference: mllm/Engine/BackendBase.hpp:20-46): a device
// key, an allocator and a table of op factories.



namespace mllm {

class BackendBase {
 public:
  explicit BackendBase(DeviceTypes device) : device_(device) {}
  virtual ~BackendBase() = default;

  template <typename... Factories>
  void regOpFactory() {
    (..., regOne<Factories>());
  }

  [[nodiscard]] std::shared_ptr<Allocator> getAllocator() const { return allocator_; }
  std::shared_ptr<BaseOp> createOp(OpType op_type, const BaseOpCargoBase& base_cargo);
  [[nodiscard]] DeviceTypes deviceType() const { return device_; }

 private:
  template <typename T>
  void regOne() {
    auto f = std::make_shared<T>();
    op_factory_table_[static_cast<int>(f->opType())] = f;
  }

 protected:
  DeviceTypes device_;
  std::unordered_map<int, std::shared_ptr<BaseOpFactory>> op_factory_table_;
  std::shared_ptr<Allocator> allocator_ = nullptr;
};

}  // namespace mllm

// ====================================================================================================
// stands for mllm/Engine/Context.hpp
// ====================================================================================================
// The engine context, reduced to what calls the Linear path (reference:
// mllm/Engine/Context.hpp:26-106, Context.cpp:56-122): a process-wide registry of backends keyed
// by device, their allocators, and eager dispatch = reshape -> setup -> forward.



namespace mllm {

class MemManager {
 public:
  void regAllocator(DeviceTypes device, const std::shared_ptr<Allocator>& a) { table_[device] = a; }
  std::shared_ptr<Allocator> allocator(DeviceTypes device) const;
  void alloc(const std::shared_ptr<Storage>& s);
  void free(Storage* s);

 private:
  std::unordered_map<int, std::shared_ptr<Allocator>> table_;
};

class MllmEngineCtx {
 public:
  static MllmEngineCtx& instance();

  void registerBackend(const std::shared_ptr<BackendBase>& backend);
  std::shared_ptr<BackendBase> getBackend(DeviceTypes device);
  [[nodiscard]] std::shared_ptr<MemManager> mem() const { return mem_; }

  // Named layers: created once (Module::reg time in the reference), dispatched by name.
  void regLayerOp(const std::string& name, const std::shared_ptr<BaseOp>& op) { layer_ops_[name] = op; }
  std::vector<Tensor> dispatch(const std::string& name, const std::vector<Tensor>& inputs);
  // Anonymous ops: created on the backend of inputs[0]'s device, then run.
  std::vector<Tensor> dispatch(OpType op_type, const BaseOpCargoBase& cargo,
                               const std::vector<Tensor>& inputs);

  void setPerf(bool on) { perf_ = on; }
  void shutdown();

 private:
  MllmEngineCtx() : mem_(std::make_shared<MemManager>()) {}
  std::vector<Tensor> run(const std::shared_ptr<BaseOp>& op, const std::vector<Tensor>& inputs,
                          const std::string& what);

  std::shared_ptr<MemManager> mem_;
  std::unordered_map<int, std::shared_ptr<BackendBase>> backends_;
  std::unordered_map<std::string, std::shared_ptr<BaseOp>> layer_ops_;
  bool perf_ = false;
};

}  // namespace mllm

// ====================================================================================================
// stands for mllm/Engine/ParameterReader.hpp
// ====================================================================================================
// The ".mllm" parameter container: 268-byte head, N x 416-byte descriptors, raw data
// (reference: mllm/Engine/ParameterReader.hpp:27-57 structs, ParameterReader.cpp:41-104 loader,
// :114-181 writer; the Python writer pads each tensor to 64 bytes, tools/convertor.py:173,207-211,
// which the offsets in the descriptors already account for).



namespace mllm {

constexpr size_t kParameterNameLen = 256;
constexpr size_t kTensorShapeMaxLen = 16;
constexpr uint64_t kParameterMagicNumber = 0x519ACE0519ACE000ULL;

struct __attribute__((packed)) ParameterDescriptor {
  uint32_t parameter_id;
  uint32_t parameter_type;   // DataTypes code
  uint64_t parameter_size;   // bytes
  uint64_t parameter_offset; // from the start of the file
  uint64_t shape_len;
  uint64_t shape[kTensorShapeMaxLen];
  char name[kParameterNameLen];
};

struct __attribute__((packed)) ParameterPackHead {
  uint64_t magic_number;
  char model_name[kParameterNameLen];
  uint32_t parameter_cnt;
};

static_assert(sizeof(ParameterPackHead) == 268, "head is 268 bytes on disk");
static_assert(sizeof(ParameterDescriptor) == 416, "descriptor is 416 bytes on disk");

class ParameterLoader {
 public:
  ParameterLoader() = default;
  explicit ParameterLoader(const std::string& file_name);  // mmaps; tensors alias the mapping

  // Exits with kIOError if the name is missing, as the reference's table lookup would.
  std::shared_ptr<TensorViewImpl> operator[](const std::string& name);
  [[nodiscard]] bool has(const std::string& name) const { return params_.count(name) != 0; }
  std::unordered_map<std::string, std::shared_ptr<TensorViewImpl>>& params() { return params_; }
  [[nodiscard]] const std::string& modelName() const { return model_name_; }

  // In-memory registration (what the quantizer does when it replaces a tensor).
  void insert(const std::string& name, const Tensor& t);

 private:
  std::shared_ptr<void> mapping_;
  std::string model_name_;
  std::unordered_map<std::string, std::shared_ptr<TensorViewImpl>> params_;
};

std::shared_ptr<ParameterLoader> load(const std::string& file_path);

// Writes host tensors in the unpadded C++ layout of the reference writer.
void write(const std::shared_ptr<ParameterLoader>& params, const std::string& file_path,
           const std::string& model_name = "mllm");

}  // namespace mllm

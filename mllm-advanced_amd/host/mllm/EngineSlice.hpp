// The slice of the reference engine that the HIP backend is compiled against when it is built outside the
// reference tree: exit codes and logging, device and data type keys, storage and allocator, tensor, operator
// base classes and the abstract operators the backend implements, backend base, memory manager, context and
// the parameter file reader. Inside the reference tree the headers of these names (the one-line files beside
// this one forward to here) are the reference's own, and this file is not used.
//
// Everything mllm/Backends/HIP and mllm/Models/ds_qwen2/HipQwen2.* use from here has the reference's name,
// signature, constness and enumerator values, so those sources compile unchanged against either tree (a test
// compiles them against the reference's headers). Members marked "stand-in only" exist for this build's own
// tests and are not used by the backend sources. Each part cites the file it stands for.
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <list>
#include <memory>
#include <sstream>
#include <string>
#include <typeinfo>
#include <unordered_map>
#include <vector>

// ====================================================================================================
// stands for mllm/Utils/Log.hpp and mllm/Utils/Common.hpp
// ====================================================================================================
// Error convention of the engine: no exceptions, no status codes; an unrecoverable condition prints and
// exits with a code (reference: mllm/Utils/Log.hpp:59-64, codes mllm/Utils/Common.hpp:23-30). Messages are
// "{}"-style, as the reference's macros pass them to fmt::format. The reference's *_EXIT macros expand to
// an `if` block followed by `exit(code)`: a caller must put them inside braces of their own.
// The exit handler is replaceable so tests can observe it (stand-in only).

namespace mllm {

enum ExitCode : int32_t {  // NOLINT
  kSuccess = 0,
  kError,
  kAssert,
  kSliceOB,
  kMemory,
  kCudaError,
};

inline std::function<void(int, const std::string&)>& errorHandler() {
  static std::function<void(int, const std::string&)> h = [](int code, const std::string& msg) {
    std::fprintf(stderr, "[mllm][ERROR] %s\n", msg.c_str());
    std::fflush(stderr);
    std::exit(code);
  };
  return h;
}

namespace detail {

template <typename T>
inline std::string showArg(const T& v) {
  std::ostringstream os;
  os << v;
  return os.str();
}

// The subset of fmt::format the backend uses: "{}" takes the next argument, "{{" and "}}" are braces.
template <typename... Args>
inline std::string braceFormat(const std::string& fmt, const Args&... args) {
  const std::vector<std::string> shown = {showArg(args)...};
  std::string out;
  size_t next = 0;
  for (size_t i = 0; i < fmt.size(); ++i) {
    if (fmt[i] == '{' && i + 1 < fmt.size() && fmt[i + 1] == '}') {
      out += next < shown.size() ? shown[next] : std::string("{}");
      ++next;
      ++i;
    } else if ((fmt[i] == '{' || fmt[i] == '}') && i + 1 < fmt.size() && fmt[i + 1] == fmt[i]) {
      out += fmt[i];
      ++i;
    } else {
      out += fmt[i];
    }
  }
  return out;
}

}  // namespace detail
}  // namespace mllm

#define MLLM_INFO(...) std::fprintf(stderr, "[INFO] %s\n", ::mllm::detail::braceFormat(__VA_ARGS__).c_str())
#define MLLM_WARN(...) std::fprintf(stderr, "[WARN] %s\n", ::mllm::detail::braceFormat(__VA_ARGS__).c_str())
#define MLLM_ERROR_EXIT(code, ...) ::mllm::errorHandler()((code), ::mllm::detail::braceFormat(__VA_ARGS__))
#define MLLM_ASSERT_EXIT(code, ...) ::mllm::errorHandler()((code), ::mllm::detail::braceFormat(__VA_ARGS__))
#define MLLM_RT_ASSERT(statement) \
  if (!(statement)) { MLLM_ASSERT_EXIT(::mllm::ExitCode::kAssert, "{}", #statement); }
#define MLLM_RT_ASSERT_EQ(statement1, statement2)                                      \
  if ((statement1) != (statement2)) {                                                  \
    MLLM_ASSERT_EXIT(::mllm::ExitCode::kAssert, "{} != {}", #statement1, #statement2); \
  }
#define NYI(...) std::fprintf(stderr, "[NYI] %s\n", ::mllm::detail::braceFormat(__VA_ARGS__).c_str())

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
// (reference: mllm/Core/DataTypes.hpp:19-65 - Int8 = 2, Int16 = 3, Int32 = 4, Int64 = 5, Fp16 = 8, Fp32 = 9,
// BF16 = 24).

namespace mllm {

enum DataTypes : uint32_t {  // NOLINT
  kDataTypes_Start = 0,
  kInt8 = 2,
  kInt16 = 3,
  kInt32 = 4,
  kInt64 = 5,
  kFp16 = 8,
  kFp32 = 9,
  kBF16 = 24,
};

inline size_t dataTypeSize(DataTypes t) {
  switch (t) {
    case kInt8: return 1;
    case kInt16:
    case kFp16:
    case kBF16: return 2;
    case kInt32:
    case kFp32: return 4;
    case kInt64: return 8;
    default: return 0;
  }
}

inline const char* dataTypes2Str(DataTypes t) {
  switch (t) {
    case kInt8: return "Int8";
    case kInt16: return "Int16";
    case kInt32: return "Int32";
    case kInt64: return "Int64";
    case kFp16: return "Fp16";
    case kFp32: return "Fp32";
    case kBF16: return "BF16";
    default: return "Unknown";
  }
}

}  // namespace mllm

// ====================================================================================================
// stands for mllm/Core/Storage.hpp and mllm/Engine/Allocator.hpp
// ====================================================================================================
// Allocator interface a backend hands to the engine (reference: mllm/Engine/Allocator.hpp:18-32, the same
// nine virtuals with the same meaning; like the reference's, the class has no virtual destructor).

namespace mllm {

// reference: mllm/Core/Storage.hpp:20-37
class Storage : public std::enable_shared_from_this<Storage> {
 public:
  virtual ~Storage() = default;
  void* ptr_ = nullptr;
  size_t size_ = 0;
  DeviceTypes device_ = kCPU;
  uint32_t custom_32bit_uuid_ = 0xFFFFFFFFu;
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
// stands for mllm/Core/TensorImpl.hpp and mllm/Core/Tensor.hpp
// ====================================================================================================
// A tensor view over reference-counted storage: the part of the engine's Tensor that an operator boundary
// needs (reference: mllm/Core/Tensor.hpp:52-140, 255-440, mllm/Core/TensorImpl.hpp:20-160). Views here are
// always dense row-major (an offset into the storage plus a shape); the reference's strided views are what
// its CPU transpose/slice produce and no HIP operator creates them.
// Tensor::empty() only describes a tensor; alloc() asks the memory manager for memory, as BaseOp::setup does
// for op outputs (mllm/Core/AOps/BaseOp.cpp:25-46).

namespace mllm {

enum TensorMemTypes : int32_t {  // NOLINT
  kTensorMemTypes_Start = 0,
  kNormal,  // owned: returned to the memory manager when the last reference goes
  kExtraInput,
  kExtraOutput,
  kManual,
  kGlobal,
  kParams,  // aliases a mapped parameter file: never freed by the tensor
  kReference,
  kQnnAppReadWrite,
  kTensorMemTypes_End,
};

class TensorStorage final : public Storage {
 public:
  ~TensorStorage() override;
  static std::shared_ptr<TensorStorage> create(const std::vector<int32_t>& shape, DataTypes dtype,
                                               DeviceTypes device);
  std::string name_;
  DataTypes dtype_ = kFp32;
  TensorMemTypes mem_type_ = kNormal;
  std::shared_ptr<void> keep_alive_;  // stand-in only: the mapped file a kParams storage aliases
};

class TensorViewImpl : public std::enable_shared_from_this<TensorViewImpl> {
 public:
  using storage_t = std::shared_ptr<TensorStorage>;
  using shape_t = std::vector<int32_t>;
  using dtype_t = DataTypes;
  using device_t = DeviceTypes;

  TensorViewImpl() = default;
  TensorViewImpl(const TensorViewImpl&) = delete;

  DataTypes dtype() const { return storage_->dtype_; }
  DeviceTypes device() const { return storage_->device_; }
  storage_t storage() const { return storage_; }
  [[nodiscard]] std::string name() const { return storage_->name_; }
  [[nodiscard]] TensorMemTypes memType() const { return storage_->mem_type_; }
  [[nodiscard]] uint32_t uuid() const { return storage_->custom_32bit_uuid_; }
  uint64_t address() const { return reinterpret_cast<uint64_t>(storage_->ptr_); }
  [[nodiscard]] void* rptr() const {
    return static_cast<char*>(storage_->ptr_) + static_cast<size_t>(storage_offset_) * dataTypeSize(dtype());
  }
  size_t size() const { return numel() * dataTypeSize(dtype()); }  // bytes, not aligned
  size_t numel() const;
  [[nodiscard]] std::vector<int32_t> shape() const { return shape_; }
  [[nodiscard]] std::vector<int32_t> stride() const;
  bool isContiguous() const { return true; }
  int32_t storageOffset() const { return storage_offset_; }

  static std::shared_ptr<TensorViewImpl> create(const std::vector<int32_t>& shape,
                                                const std::shared_ptr<TensorStorage>& storage);
  static std::shared_ptr<TensorViewImpl> create(int32_t storage_offset, const std::vector<int32_t>& shape,
                                                const std::shared_ptr<TensorStorage>& storage);

  template <typename T>
  T* ptr() {
    return static_cast<T*>(rptr());
  }

 private:
  int32_t storage_offset_ = 0;  // in elements
  shape_t shape_;
  std::shared_ptr<TensorStorage> storage_ = nullptr;
};

class Tensor {
 public:
  using shape_t = TensorViewImpl::shape_t;
  using dtype_t = TensorViewImpl::dtype_t;
  using device_t = TensorViewImpl::device_t;

  Tensor() = default;
  explicit Tensor(const std::shared_ptr<TensorViewImpl>& impl) : impl_(impl) {}

  [[nodiscard]] inline bool isNil() const { return impl_ == nullptr; }
  static inline Tensor nil() { return {}; }

  // Describes a tensor; no memory yet.
  static Tensor empty(const std::vector<int32_t>& shape, DataTypes dtype = kFp32, DeviceTypes device = kCPU);
  Tensor& alloc();

  [[nodiscard]] std::string name() const { return impl_->name(); }
  [[nodiscard]] TensorMemTypes memType() const { return impl_->memType(); }
  Tensor& setName(const std::string& name);
  Tensor& setMemType(TensorMemTypes mem_type);
  [[nodiscard]] DataTypes dtype() const { return impl_->dtype(); }
  [[nodiscard]] DeviceTypes device() const { return impl_->device(); }
  [[nodiscard]] std::vector<int32_t> shape() const { return impl_->shape(); }
  [[nodiscard]] size_t numel() const { return impl_->numel(); }
  [[nodiscard]] uint32_t uuid() const { return impl_->uuid(); }
  [[nodiscard]] bool isContiguous() const { return impl_->isContiguous(); }
  Tensor contiguous() { return *this; }
  // Same storage under another shape; goes through the backend's View operator as in the reference
  // (mllm/Core/Tensor.cpp: view() dispatches OpType::kView).
  Tensor view(const std::vector<int>& indicies);
  [[nodiscard]] inline std::shared_ptr<TensorViewImpl> impl() const { return impl_; }

  template <typename T>
  T* ptr() const {
    return impl_->ptr<T>();
  }

  size_t bytes() { return impl_->size(); }  // not const in the reference either (Tensor.hpp:439)

 private:
  std::shared_ptr<TensorViewImpl> impl_ = nullptr;
};

}  // namespace mllm

// ====================================================================================================
// stands for mllm/Engine/SymbolTable.hpp
// ====================================================================================================

namespace mllm {

// reference: mllm/Engine/SymbolTable.hpp:19-66 - registering a key twice and reading a missing key exit.
template <typename KeyT, typename ValueT>
class SymbolTable {
 public:
  void reg(const KeyT& name, const ValueT& v) {
    if (has(name)) { MLLM_ERROR_EXIT(kError, "When registing new value, found symbol table already has a value key"); }
    symbol_table_.insert({name, v});
  }
  bool has(const KeyT& name) { return symbol_table_.count(name) != 0; }
  void remove(const KeyT& name) { symbol_table_.erase(name); }
  ValueT& operator[](const KeyT& name) {
    if (!has(name)) {
      MLLM_ERROR_EXIT(kError, "When accessing symbol in symbol table. Found symbol key not in symbol table");
    }
    return symbol_table_[name];
  }
  std::unordered_map<KeyT, ValueT>& _ref_raw_data() { return symbol_table_; }

 private:
  std::unordered_map<KeyT, ValueT> symbol_table_;
};

}  // namespace mllm

// ====================================================================================================
// stands for mllm/Core/AOps/BaseOp.hpp
// ====================================================================================================
// Abstract operator API (reference: mllm/Core/AOps/BaseOp.hpp:21-234): the engine calls
// reshape -> setup -> forward on an op that a backend's factory created from a type-erased cargo.

namespace mllm {

class ParameterLoader;

// Same enumerators in the same order as the reference (BaseOp.hpp:21-77).
enum class OpType : int32_t {  // NOLINT
  kOpType_Start = 0,
  kFill,
  kAdd,
  kSub,
  kMul,
  kDiv,
  kMatMul,
  kLLMEmbeddingToken,
  kLinear,
  kRoPE,
  kSoftmax,
  kTranspose,
  kRMSNorm,
  kSiLU,
  kKVCache,
  kCausalMask,
  kCastType,
  kD2H,
  kH2D,
  kSplit,
  kView,
  kFlashAttention_2,
  kRepeat,
  kPermute,
  kConv3D,
  kConv2D,
  kConv1D,
  kGELU,
  kLayerNorm,
  kMultimodalRoPE,
  kVisionRoPE,
  kQuickGELU,
  kCopy,
  kClone,
  kNeg,
  kConcat,
  kOpType_End,
};

const char* opType2Str(OpType type);

// CRTP base of cargos (reference BaseOp.hpp:120-148): per-op thread count, default 4, and the
// inputs' / outputs' element types.
template <typename DerivedT>
class BaseOpCargo {
 public:
  BaseOpCargo() = default;
  DerivedT& setInputsDtype(size_t pos, DataTypes dtype) {
    if (pos >= inputs_dtypes_.size()) inputs_dtypes_.resize(pos + 1, kFp32);
    inputs_dtypes_[pos] = dtype;
    return *static_cast<DerivedT*>(this);
  }
  DerivedT& setOutputsDtype(size_t pos, DataTypes dtype) {
    if (pos >= outputs_dtypes_.size()) outputs_dtypes_.resize(pos + 1, kFp32);
    outputs_dtypes_[pos] = dtype;
    return *static_cast<DerivedT*>(this);
  }
  [[nodiscard]] int thread() const { return threads_; }
  void setThreads(int threads) { threads_ = threads; }

 private:
  int threads_ = 4;
  std::vector<DataTypes> inputs_dtypes_;
  std::vector<DataTypes> outputs_dtypes_;
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
  virtual void trace(void* trace_context, const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {}
  virtual void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {}
  virtual void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {}
  // Allocates every output that has no memory yet (reference BaseOp.cpp:25-46).
  virtual void setup(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs);
  virtual params_t params() { return {}; }

  [[nodiscard]] std::string name() const { return name_; }
  void setName(const std::string& name) { name_ = name; }
  [[nodiscard]] DeviceTypes device() const { return device_type_; }
  void setDeviceType(DeviceTypes d) { device_type_ = d; }

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

struct LinearOpCargo : public BaseOpCargo<LinearOpCargo> {
  int32_t in_channels = 0;
  int32_t out_channels = 0;
  bool bias = true;
  bool transpose = false;

  // "<family>:<tile>" -> enum; unknown strings warn and fall back to kDefault (LinearOp.cpp:53-55).
  static LinearOpImplType parseLinearOpImplTypeStr(const std::string& type_str);

  LinearOpImplType impl_type_ = LinearOpImplType::kDefault;
};

class LinearOp : public BaseOp {
 public:
  explicit LinearOp(const LinearOpCargo& cargo);

  // weight = "<name>.weight", bias = "<name>.bias" when cargo.bias (LinearOp.cpp:60-63)
  void load(const std::shared_ptr<ParameterLoader>& ploader) override;
  // output = input shape with the last dimension replaced by out_channels (LinearOp.cpp:84-94)
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  params_t params() override;

  inline Tensor& weight() { return weight_; }
  inline Tensor& bias() { return bias_; }
  inline const LinearOpCargo& cargo() const { return cargo_; }

 protected:
  Tensor weight_;
  Tensor bias_;
  LinearOpCargo cargo_;
};

}  // namespace mllm

// ====================================================================================================
// stands for mllm/Core/AOps/D2HOp.hpp
// ====================================================================================================

namespace mllm {

// reference: mllm/Core/AOps/D2HOp.hpp:16-38, D2HOp.cpp:15-45 (output = input's shape and type on
// cargo.to_device_type); Tensor::cpu() dispatches it (mllm/Core/Tensor.cpp).
struct D2HOpCargo : public BaseOpCargo<D2HOpCargo> {
  DeviceTypes from_device_type;
  DeviceTypes to_device_type;
};

class D2HOp : public BaseOp {
 public:
  explicit D2HOp(const D2HOpCargo& cargo);
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;

 protected:
  D2HOpCargo cargo_;
};

}  // namespace mllm

// ====================================================================================================
// stands for mllm/Core/AOps/{View,RMSNorm,RoPE,KVCache,FlashAttention2,MatMul,SiLU,Elewise,LLMEmbeddingToken}Op.hpp
// ====================================================================================================
// The abstract halves of the decoder's operators: cargos with the reference's fields and defaults, and the
// device-independent load / reshape / params of each (reference file:line at each class). The layouts are
// the ones the reference's flash-attention model variant uses (modeling_ds_qwen2_fa2_fp16.hpp:88-133):
// activations [B, S, H, D], RoPE with layout kBSHD, KV cache with layout kBSHD_NO_REPEAT.

namespace mllm {

// reference: mllm/Core/AOps/ViewOp.hpp:15-38, ViewOp.cpp:34-90 (one -1 dimension is inferred; the output
// shares the input's storage, forward does nothing)
struct ViewOpCargo : public BaseOpCargo<ViewOpCargo> {
  std::vector<int32_t> to_shape_;
};

class ViewOp : public BaseOp {
 public:
  explicit ViewOp(const ViewOpCargo& cargo);
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  void setup(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  inline std::vector<int32_t> toWhichShape() { return cargo_.to_shape_; }

 protected:
  ViewOpCargo cargo_;
};

// reference: mllm/Core/AOps/RMSNormOp.hpp:15-43, RMSNormOp.cpp (weight = "<name>.weight", output like input)
struct RMSNormOpCargo : public BaseOpCargo<RMSNormOpCargo> {
  float epsilon;
  bool add_unit_offset = false;  // Gemma
};

class RMSNormOp : public BaseOp {
 public:
  explicit RMSNormOp(const RMSNormOpCargo& cargo);
  void load(const std::shared_ptr<ParameterLoader>& ploader) override;
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  params_t params() override;

 protected:
  Tensor weight_;
  RMSNormOpCargo cargo_;
};

// reference: mllm/Core/AOps/RoPEOp.hpp:15-56
enum class RoPETypes : int32_t {
  kRoPETypes_Start = 0,
  kLlama2,
  kRoPETypes_End,
};

struct RoPEOpCargo : public BaseOpCargo<RoPEOpCargo> {
  enum RoPELayoutType {
    kBHSD = 0,  // eager attention
    kBSHD = 1,  // flash attention
  };
  RoPETypes type = RoPETypes::kLlama2;
  float theta;
  int max_position_embeddings;
  int dims;
  RoPELayoutType layout_type = kBHSD;
};

class RoPEOp : public BaseOp {
 public:
  explicit RoPEOp(const RoPEOpCargo& cargo);
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;

 protected:
  int cur_seq_cnt_ = 0;
  RoPEOpCargo cargo_;
};

// reference: mllm/Core/AOps/KVCacheOp.hpp:17-52
struct KVCacheOpCargo : public BaseOpCargo<KVCacheOpCargo> {
  enum KVCacheLayoutType {
    kBHSD_REPEAT = 0,     // eager attention
    kBSHD_NO_REPEAT = 1,  // flash attention
  };
  int32_t heads_num = 1;
  int32_t dim_per_head = 0;
  int32_t head_repeat_times = 1;
  DataTypes cached_elements_dtype = kFp32;
  int32_t pre_alloc_seq_len = 1024;
  int32_t re_alloc_multiplier = 2;
  KVCacheLayoutType layout_type = KVCacheLayoutType::kBHSD_REPEAT;
};

class KVCacheOp : public BaseOp {
 public:
  explicit KVCacheOp(const KVCacheOpCargo& cargo);

 protected:
  Tensor cache_;
  KVCacheOpCargo cargo_;
};

// reference: mllm/Core/AOps/FlashAttention2Op.hpp:15-46, FlashAttention2Op.cpp:35-44 (output like the query)
struct FlashAttn2OpCargo : public BaseOpCargo<FlashAttn2OpCargo> {
  int32_t B;
  int32_t q_head;
  int32_t kv_head;
  int32_t D;
  int32_t threads = 4;
  bool hp_exp = false;
  bool causal_mask = true;
};

class FlashAttn2Op : public BaseOp {
 public:
  explicit FlashAttn2Op(const FlashAttn2OpCargo& cargo);
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;

 protected:
  FlashAttn2OpCargo cargo_;
};

// reference: mllm/Core/AOps/MatMulOp.hpp:15-44, MatMulOp.cpp (output [..., M, N] from [..., M, K] and
// [..., K, N], either operand transposed on request)
struct MatMulOpCargo : public BaseOpCargo<MatMulOpCargo> {
  bool transpose_a = false;
  bool transpose_b = false;
};

class MatMulOp : public BaseOp {
 public:
  explicit MatMulOp(const MatMulOpCargo& cargo);
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  inline bool transposeA() { return cargo_.transpose_a; }
  inline bool transposeB() { return cargo_.transpose_b; }

 protected:
  MatMulOpCargo cargo_;
};

// reference: mllm/Core/AOps/SiLUOp.hpp:15-38
struct SiLUOpCargo : public BaseOpCargo<SiLUOpCargo> {};

class SiLUOp : public BaseOp {
 public:
  explicit SiLUOp(const SiLUOpCargo& cargo);
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;

 protected:
  SiLUOpCargo cargo_;
};

// reference: mllm/Core/AOps/ElewiseOp.hpp:15-66 (no cargo fields; output like input 0; the reference gives
// every element-wise class OpType::kAdd in its constructor, ElewiseOp.hpp:30)
struct AddOpCargo : public BaseOpCargo<AddOpCargo> {};
struct MulOpCargo : public BaseOpCargo<MulOpCargo> {};

class AddOp : public BaseOp {
 public:
  AddOp();
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
};

class MulOp : public BaseOp {
 public:
  MulOp();
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
};

// reference: mllm/Core/AOps/LLMEmbeddingTokenOp.hpp:15-45, LLMEmbeddingTokenOp.cpp (weight =
// "<name>.weight" [vocab, hidden]; ids [B, S] -> [B, S, hidden] in the weight's type)
struct LLMEmbeddingTokenOpCargo : public BaseOpCargo<LLMEmbeddingTokenOpCargo> {
  int vocab_size = 0;
  int hidden_size = 0;
};

class LLMEmbeddingTokenOp : public BaseOp {
 public:
  explicit LLMEmbeddingTokenOp(const LLMEmbeddingTokenOpCargo& cargo);
  void load(const std::shared_ptr<ParameterLoader>& ploader) override;
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  params_t params() override;

 protected:
  Tensor weight_;
  LLMEmbeddingTokenOpCargo cargo_;
};

}  // namespace mllm

// ====================================================================================================
// stands for mllm/Engine/BackendBase.hpp
// ====================================================================================================
// What a device backend is to the engine (reference: mllm/Engine/BackendBase.hpp:20-46): a device key, an
// allocator and a table of op factories. As in the reference the class has no virtual member: a backend is
// recognised by deviceType(), not by dynamic_cast, and a derived destructor is not an override.

namespace mllm {

class BackendBase {
 public:
  explicit BackendBase(DeviceTypes device) : device_(device) {}

  template <typename... Args>
  void regOpFactory() {
    (..., (_reg_one_op_factory<Args>()));
  }

  [[nodiscard]] std::shared_ptr<Allocator> getAllocator() const { return allocator_; }
  std::shared_ptr<BaseOp> createOp(OpType op_type, const BaseOpCargoBase& base_cargo);
  [[nodiscard]] DeviceTypes deviceType() const { return device_; }

 private:
  template <typename T>
  void _reg_one_op_factory() {
    auto ptr = std::make_shared<T>();
    op_factory_table_.reg(ptr->opType(), ptr);
  }

 protected:
  DeviceTypes device_;
  SymbolTable<OpType, std::shared_ptr<BaseOpFactory>> op_factory_table_;
  std::shared_ptr<Allocator> allocator_ = nullptr;
};

}  // namespace mllm

// ====================================================================================================
// stands for mllm/Engine/MemManager.hpp and mllm/Engine/Context.hpp
// ====================================================================================================
// The memory manager and the engine context, reduced to what calls this path (reference:
// mllm/Engine/MemManager.hpp:63-140, mllm/Engine/Context.hpp:26-106, Context.cpp:56-122): a process-wide
// registry of backends keyed by device, and eager dispatch = reshape -> setup -> forward.
//
// Like the reference's manager (a buddy allocator over 128 MiB segments it gets from the backend's
// allocator, MemManager.cpp:40-75, 140-160) this one does not go to the device allocator per tensor: blocks
// of a device whose allocator says ctrlByMllmMemManager() are rounded up to a size class and, when their
// tensor dies, kept in a per-device free list for the next tensor of that class. A device allocation
// (hipMalloc) and a device free (which synchronises the device) happen only when a class runs dry and in
// releaseCached(). Reuse without synchronisation is safe because a backend issues all its work on one
// stream: the new owner's kernels are ordered behind the old owner's.

namespace mllm {

class MemManager {
 public:
  ~MemManager();
  void alloc(const std::shared_ptr<Storage>& s);
  void free(Storage* s);
  void regAllocator(DeviceTypes device, const std::shared_ptr<Allocator>& allocator);

  // stand-in only
  void releaseCached();                                 // gives every cached block back to its allocator
  [[nodiscard]] size_t deviceAllocCalls() const { return device_alloc_calls_; }

 private:
  static size_t sizeClass(size_t bytes);
  SymbolTable<DeviceTypes, std::shared_ptr<Allocator>> allocators_st_;
  std::unordered_map<int, std::unordered_map<size_t, std::list<void*>>> free_blocks_;  // [device][class]
  std::unordered_map<void*, size_t> block_class_;                                        // live + cached
  size_t device_alloc_calls_ = 0;
};

class MllmEngineCtx {
 public:
  static MllmEngineCtx& instance();

  void registerBackend(const std::shared_ptr<BackendBase>& new_backend);
  std::shared_ptr<BackendBase> getBackend(DeviceTypes device);
  [[nodiscard]] std::shared_ptr<MemManager> mem() const { return main_thread_mem_; }
  uint32_t getUUID() { return custom_uuid_giver_++; }

  // Named layers: created once (Module::reg time in the reference), dispatched by name.
  std::vector<Tensor> dispatch(const std::string& name, const std::vector<Tensor>& inputs);
  // Anonymous ops: created on the backend of inputs[0]'s device, then run.
  std::vector<Tensor> dispatch(OpType op_type, const BaseOpCargoBase& base_cargo,
                               const std::vector<Tensor>& inputs);
  void shutdown();

  bool perf_ = false;

  // stand-in only: the reference keeps named layer ops in its thread object (Thread.hpp:46)
  void regLayerOp(const std::string& name, const std::shared_ptr<BaseOp>& op) { layer_ops_[name] = op; }

 private:
  MllmEngineCtx() : main_thread_mem_(std::make_shared<MemManager>()) {}
  std::vector<Tensor> run(const std::shared_ptr<BaseOp>& op, const std::vector<Tensor>& inputs,
                          const std::string& what);

  std::shared_ptr<MemManager> main_thread_mem_;
  SymbolTable<DeviceTypes, std::shared_ptr<BackendBase>> backends_table_;
  std::unordered_map<std::string, std::shared_ptr<BaseOp>> layer_ops_;
  uint32_t custom_uuid_giver_ = 0;
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

  // Exits with kError if the name is missing, as the reference's table lookup does.
  std::shared_ptr<TensorViewImpl> operator[](const std::string& name);
  std::unordered_map<std::string, std::shared_ptr<TensorViewImpl>>& params() { return params_; }

  // stand-in only
  [[nodiscard]] bool has(const std::string& name) const { return params_.count(name) != 0; }
  [[nodiscard]] const std::string& modelName() const { return model_name_; }
  void insert(const std::string& name, const Tensor& t);  // in-memory registration

 private:
  std::shared_ptr<void> mapping_;
  std::string model_name_;
  std::unordered_map<std::string, std::shared_ptr<TensorViewImpl>> params_;
};

std::shared_ptr<ParameterLoader> load(const std::string& file_path);

// Writes host tensors in the unpadded layout of the reference's C++ writer (ParameterReader.cpp:114-181),
// with the reference's signatures (ParameterReader.hpp:124-130).
void write(const std::string& file_path, const std::unordered_map<std::string, Tensor>& params,
           const std::string& model_name);
void write(const std::string& file_path,
           const std::unordered_map<std::string, std::shared_ptr<TensorViewImpl>>& params,
           const std::string& model_name);

}  // namespace mllm

// Abstract operator API (reference: mllm/Core/AOps/BaseOp.hpp:118-234): the engine calls
// reshape -> setup -> forward on an op that a backend's factory created from a type-erased cargo.
#pragma once

#include <memory>
#include <string>
#include <typeinfo>
#include <unordered_map>
#include <vector>

#include "mllm/Core/Tensor.hpp"

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

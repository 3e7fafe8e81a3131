// The engine context, reduced to what calls the Linear path (reference:
// mllm/Engine/Context.hpp:26-106, Context.cpp:56-122): a process-wide registry of backends keyed
// by device, their allocators, and eager dispatch = reshape -> setup -> forward.
#pragma once

#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "mllm/Engine/BackendBase.hpp"

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

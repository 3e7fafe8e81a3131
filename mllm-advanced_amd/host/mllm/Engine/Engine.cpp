// Engine context, memory manager, backend registry and the .mllm parameter container.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <chrono>
#include <cstring>
#include <fstream>

#include "mllm/Engine/Context.hpp"
#include "mllm/Engine/ParameterReader.hpp"
#include "mllm/Utils/Log.hpp"

namespace mllm {

// ---------------------------------------------------------------------------- memory
std::shared_ptr<Allocator> MemManager::allocator(DeviceTypes device) const {
  auto it = table_.find(device);
  if (it == table_.end()) {
    MLLM_ERROR_EXIT(kCoreError, "no allocator registered for device %s", deviceTypes2Str(device));
    return nullptr;
  }
  return it->second;
}

void MemManager::alloc(const std::shared_ptr<Storage>& s) {
  auto a = allocator(s->device_);
  if (!a || !a->alloc(s)) {
    MLLM_ERROR_EXIT(kCoreError, "allocation of %zu bytes on %s failed", s->size_,
                    deviceTypes2Str(s->device_));
  }
}

void MemManager::free(Storage* s) {
  auto it = table_.find(s->device_);
  if (it != table_.end() && s->ptr_) it->second->free(s);
  s->ptr_ = nullptr;
}

// ---------------------------------------------------------------------------- context
MllmEngineCtx& MllmEngineCtx::instance() {
  static MllmEngineCtx ctx;
  return ctx;
}

void MllmEngineCtx::registerBackend(const std::shared_ptr<BackendBase>& backend) {
  backends_[backend->deviceType()] = backend;
  mem_->regAllocator(backend->deviceType(), backend->getAllocator());
}

std::shared_ptr<BackendBase> MllmEngineCtx::getBackend(DeviceTypes device) {
  auto it = backends_.find(device);
  if (it == backends_.end()) {
    MLLM_ERROR_EXIT(kCoreError, "no backend registered for device %s", deviceTypes2Str(device));
    return nullptr;
  }
  return it->second;
}

std::vector<Tensor> MllmEngineCtx::run(const std::shared_ptr<BaseOp>& op,
                                       const std::vector<Tensor>& inputs, const std::string& what) {
  std::vector<Tensor> outputs;
  const auto t0 = std::chrono::high_resolution_clock::now();
  op->reshape(inputs, outputs);
  op->setup(inputs, outputs);
  op->forward(inputs, outputs);
  if (perf_) {
    const std::chrono::duration<double, std::milli> dt =
        std::chrono::high_resolution_clock::now() - t0;
    MLLM_INFO("perf| %s, Time:%f ms", what.c_str(), dt.count());
  }
  return outputs;
}

std::vector<Tensor> MllmEngineCtx::dispatch(const std::string& name,
                                            const std::vector<Tensor>& inputs) {
  auto it = layer_ops_.find(name);
  if (it == layer_ops_.end()) {
    MLLM_ERROR_EXIT(kCoreError, "no layer named %s", name.c_str());
    return {};
  }
  return run(it->second, inputs, "Layer: " + name);
}

std::vector<Tensor> MllmEngineCtx::dispatch(OpType op_type, const BaseOpCargoBase& cargo,
                                            const std::vector<Tensor>& inputs) {
  auto op = getBackend(inputs[0].device())->createOp(op_type, cargo);
  return run(op, inputs, std::string("Op: ") + opType2Str(op_type));
}

void MllmEngineCtx::shutdown() {
  layer_ops_.clear();
  backends_.clear();
}

std::shared_ptr<BaseOp> BackendBase::createOp(OpType op_type, const BaseOpCargoBase& base_cargo) {
  auto it = op_factory_table_.find(static_cast<int>(op_type));
  if (it == op_factory_table_.end()) {
    MLLM_ERROR_EXIT(kCoreError, "backend %s has no factory for op %s", deviceTypes2Str(device_),
                    opType2Str(op_type));
    return nullptr;
  }
  auto op = it->second->create(base_cargo);
  op->setDeviceType(device_);
  return op;
}

// ---------------------------------------------------------------------------- .mllm container
namespace {

struct Mapping {
  void* addr = nullptr;
  size_t size = 0;
  ~Mapping() {
    if (addr) munmap(addr, size);
  }
};

std::string fixedName(const char* p, size_t cap) { return std::string(p, strnlen(p, cap)); }

}  // namespace

ParameterLoader::ParameterLoader(const std::string& file_name) {
  const int fd = open(file_name.c_str(), O_RDONLY);
  if (fd < 0) {
    MLLM_ERROR_EXIT(kIOError, "cannot open %s", file_name.c_str());
    return;
  }
  struct stat st {};
  fstat(fd, &st);
  auto map = std::make_shared<Mapping>();
  map->size = static_cast<size_t>(st.st_size);
  map->addr = mmap(nullptr, map->size, PROT_READ, MAP_PRIVATE, fd, 0);
  close(fd);
  if (map->addr == MAP_FAILED) {
    map->addr = nullptr;
    MLLM_ERROR_EXIT(kIOError, "cannot map %s", file_name.c_str());
    return;
  }
  mapping_ = map;

  const auto* bytes = static_cast<const uint8_t*>(map->addr);
  if (map->size < sizeof(ParameterPackHead)) {
    MLLM_ERROR_EXIT(kIOError, "%s: shorter than a header", file_name.c_str());
    return;
  }
  const auto* head = reinterpret_cast<const ParameterPackHead*>(bytes);
  if (head->magic_number != kParameterMagicNumber) {
    MLLM_ERROR_EXIT(kIOError, "%s: bad magic number", file_name.c_str());
    return;
  }
  model_name_ = fixedName(head->model_name, kParameterNameLen);
  const size_t table_end = sizeof(ParameterPackHead) + head->parameter_cnt * sizeof(ParameterDescriptor);
  if (table_end > map->size) {
    MLLM_ERROR_EXIT(kIOError, "%s: descriptor table runs past the end", file_name.c_str());
    return;
  }
  const auto* descs = reinterpret_cast<const ParameterDescriptor*>(bytes + sizeof(ParameterPackHead));
  for (uint32_t i = 0; i < head->parameter_cnt; ++i) {
    const ParameterDescriptor& d = descs[i];
    if (d.shape_len > kTensorShapeMaxLen || d.parameter_offset + d.parameter_size > map->size) {
      MLLM_ERROR_EXIT(kIOError, "%s: descriptor %u is out of range", file_name.c_str(), i);
      return;
    }
    Tensor::shape_t shape;
    for (uint64_t k = 0; k < d.shape_len; ++k) shape.push_back(static_cast<int32_t>(d.shape[k]));
    Tensor t = Tensor::wrap(const_cast<uint8_t*>(bytes) + d.parameter_offset, shape,
                            static_cast<DataTypes>(d.parameter_type), kCPU, mapping_);
    t.setName(fixedName(d.name, kParameterNameLen));
    params_[t.name()] = t.impl();
  }
}

std::shared_ptr<TensorViewImpl> ParameterLoader::operator[](const std::string& name) {
  auto it = params_.find(name);
  if (it == params_.end()) {
    MLLM_ERROR_EXIT(kIOError, "parameter %s not found", name.c_str());
    return nullptr;
  }
  return it->second;
}

void ParameterLoader::insert(const std::string& name, const Tensor& t) {
  t.impl()->name_ = name;
  params_[name] = t.impl();
}

std::shared_ptr<ParameterLoader> load(const std::string& file_path) {
  return std::make_shared<ParameterLoader>(file_path);
}

void write(const std::shared_ptr<ParameterLoader>& params, const std::string& file_path,
           const std::string& model_name) {
  std::vector<std::pair<std::string, std::shared_ptr<TensorViewImpl>>> items(
      params->params().begin(), params->params().end());
  std::sort(items.begin(), items.end(),
            [](const auto& a, const auto& b) { return a.first < b.first; });

  ParameterPackHead head{};
  head.magic_number = kParameterMagicNumber;
  std::strncpy(head.model_name, model_name.c_str(), kParameterNameLen - 1);
  head.parameter_cnt = static_cast<uint32_t>(items.size());

  std::vector<ParameterDescriptor> descs(items.size());
  uint64_t offset = sizeof(head) + items.size() * sizeof(ParameterDescriptor);
  for (size_t i = 0; i < items.size(); ++i) {
    Tensor t(items[i].second);
    if (t.device() != kCPU) {
      MLLM_ERROR_EXIT(kIOError, "write: %s is not a host tensor", items[i].first.c_str());
      return;
    }
    ParameterDescriptor& d = descs[i];
    std::memset(&d, 0, sizeof d);
    d.parameter_id = static_cast<uint32_t>(i);
    d.parameter_type = static_cast<uint32_t>(t.dtype());
    d.parameter_size = t.bytes();
    d.parameter_offset = offset;
    d.shape_len = t.shape().size();
    for (size_t k = 0; k < t.shape().size(); ++k) d.shape[k] = static_cast<uint64_t>(t.shape()[k]);
    std::strncpy(d.name, items[i].first.c_str(), kParameterNameLen - 1);
    offset += d.parameter_size;
  }
  std::ofstream out(file_path, std::ios::binary);
  if (!out) {
    MLLM_ERROR_EXIT(kIOError, "cannot create %s", file_path.c_str());
    return;
  }
  out.write(reinterpret_cast<const char*>(&head), sizeof head);
  out.write(reinterpret_cast<const char*>(descs.data()),
            static_cast<std::streamsize>(descs.size() * sizeof(ParameterDescriptor)));
  for (auto& it : items) {
    Tensor t(it.second);
    out.write(t.ptr<char>(), static_cast<std::streamsize>(t.bytes()));
  }
}

}  // namespace mllm

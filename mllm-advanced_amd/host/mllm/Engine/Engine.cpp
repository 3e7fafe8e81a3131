// Engine context, memory manager, backend registry and the .mllm parameter container.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <chrono>
#include <cstring>
#include <fstream>

#include "mllm/Engine/Context.hpp"
#include "mllm/Engine/ParameterReader.hpp"
#include "mllm/Utils/Log.hpp"

namespace mllm {

// ---------------------------------------------------------------------------- memory
void MemManager::regAllocator(DeviceTypes device, const std::shared_ptr<Allocator>& allocator) {
  if (allocators_st_.has(device)) allocators_st_.remove(device);
  allocators_st_.reg(device, allocator);
}

// Size classes: multiples of 256 B up to 4 KiB, then four steps per power of two (at most 19 % unused).
size_t MemManager::sizeClass(size_t bytes) {
  if (bytes <= 4096) return (std::max<size_t>(bytes, 1) + 255) / 256 * 256;
  size_t p = 4096;
  while (p * 2 < bytes) p *= 2;           // p < bytes <= 2p
  const size_t step = p / 4;
  return p + (bytes - p + step - 1) / step * step;
}

void MemManager::alloc(const std::shared_ptr<Storage>& s) {
  auto& a = allocators_st_[s->device_];
  if (!a->ctrlByMllmMemManager()) {
    if (!a->alloc(s)) { MLLM_ERROR_EXIT(kMemory, "allocation of {} bytes on {} failed", s->size_, deviceTypes2Str(s->device_)); }
    return;
  }
  const size_t cls = sizeClass(a->allocSize(s));
  auto& bucket = free_blocks_[s->device_][cls];
  if (!bucket.empty()) {
    s->ptr_ = bucket.front();
    bucket.pop_front();
    return;
  }
  void* p = nullptr;
  ++device_alloc_calls_;
  if (!a->generalAlloc(&p, cls, a->alignSize()) || !p) {
    MLLM_ERROR_EXIT(kMemory, "allocation of {} bytes on {} failed", cls, deviceTypes2Str(s->device_));
  }
  block_class_[p] = cls;
  s->ptr_ = p;
}

void MemManager::free(Storage* s) {
  if (!s->ptr_ || !allocators_st_.has(s->device_)) return;
  auto& a = allocators_st_[s->device_];
  auto it = block_class_.find(s->ptr_);
  if (it == block_class_.end()) {
    a->free(s);  // not one of this manager's blocks
  } else {
    free_blocks_[s->device_][it->second].push_back(s->ptr_);
  }
  s->ptr_ = nullptr;
}

void MemManager::releaseCached() {
  for (auto& dev : free_blocks_) {
    const auto device = static_cast<DeviceTypes>(dev.first);
    if (!allocators_st_.has(device)) continue;
    auto& a = allocators_st_[device];
    for (auto& cls : dev.second) {
      for (void* p : cls.second) {
        block_class_.erase(p);
        a->generalFree(p);
      }
      cls.second.clear();
    }
  }
}

MemManager::~MemManager() { releaseCached(); }

// ---------------------------------------------------------------------------- context
MllmEngineCtx& MllmEngineCtx::instance() {
  static MllmEngineCtx ctx;
  return ctx;
}

void MllmEngineCtx::registerBackend(const std::shared_ptr<BackendBase>& new_backend) {
  if (backends_table_.has(new_backend->deviceType())) backends_table_.remove(new_backend->deviceType());
  backends_table_.reg(new_backend->deviceType(), new_backend);
  main_thread_mem_->regAllocator(new_backend->deviceType(), new_backend->getAllocator());
}

std::shared_ptr<BackendBase> MllmEngineCtx::getBackend(DeviceTypes device) { return backends_table_[device]; }

std::vector<Tensor> MllmEngineCtx::run(const std::shared_ptr<BaseOp>& op, const std::vector<Tensor>& inputs,
                                       const std::string& what) {
  std::vector<Tensor> outputs;
  const auto t0 = std::chrono::high_resolution_clock::now();
  op->reshape(inputs, outputs);
  op->setup(inputs, outputs);
  op->forward(inputs, outputs);
  if (perf_) {
    const std::chrono::duration<double, std::milli> dt = std::chrono::high_resolution_clock::now() - t0;
    MLLM_INFO("perf| {}, Time:{} ms", what, dt.count());
  }
  return outputs;
}

std::vector<Tensor> MllmEngineCtx::dispatch(const std::string& name, const std::vector<Tensor>& inputs) {
  auto it = layer_ops_.find(name);
  if (it == layer_ops_.end()) {
    MLLM_ERROR_EXIT(kError, "no layer named {}", name);
    return {};
  }
  return run(it->second, inputs, "Layer: " + name);
}

std::vector<Tensor> MllmEngineCtx::dispatch(OpType op_type, const BaseOpCargoBase& base_cargo,
                                            const std::vector<Tensor>& inputs) {
  auto op = backends_table_[inputs[0].device()]->createOp(op_type, base_cargo);
  return run(op, inputs, std::string("Op: ") + opType2Str(op_type));
}

void MllmEngineCtx::shutdown() {
  layer_ops_.clear();
  main_thread_mem_->releaseCached();
  backends_table_._ref_raw_data().clear();
}

std::shared_ptr<BaseOp> BackendBase::createOp(OpType op_type, const BaseOpCargoBase& base_cargo) {
  if (!op_factory_table_.has(op_type)) {
    MLLM_ERROR_EXIT(kError, "backend {} has no factory for op {}", deviceTypes2Str(device_), opType2Str(op_type));
    return nullptr;
  }
  auto op = op_factory_table_[op_type]->create(base_cargo);
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
    MLLM_ERROR_EXIT(kError, "cannot open {}", file_name);
    return;
  }
  struct stat st {};
  if (fstat(fd, &st) != 0 || st.st_size < 0) {
    close(fd);
    MLLM_ERROR_EXIT(kError, "cannot stat {}", file_name);
    return;
  }
  auto map = std::make_shared<Mapping>();
  map->size = static_cast<size_t>(st.st_size);
  if (map->size < sizeof(ParameterPackHead)) {
    close(fd);
    MLLM_ERROR_EXIT(kError, "{}: shorter than a header", file_name);
    return;
  }
  map->addr = mmap(nullptr, map->size, PROT_READ, MAP_PRIVATE, fd, 0);
  close(fd);
  if (map->addr == MAP_FAILED) {
    map->addr = nullptr;
    MLLM_ERROR_EXIT(kError, "cannot map {}", file_name);
    return;
  }
  mapping_ = map;

  const auto* bytes = static_cast<const uint8_t*>(map->addr);
  const auto* head = reinterpret_cast<const ParameterPackHead*>(bytes);
  if (head->magic_number != kParameterMagicNumber) {
    MLLM_ERROR_EXIT(kError, "{}: bad magic number", file_name);
    return;
  }
  model_name_ = fixedName(head->model_name, kParameterNameLen);
  const size_t room = map->size - sizeof(ParameterPackHead);
  if (head->parameter_cnt > room / sizeof(ParameterDescriptor)) {
    MLLM_ERROR_EXIT(kError, "{}: descriptor table runs past the end", file_name);
    return;
  }
  const auto* descs = reinterpret_cast<const ParameterDescriptor*>(bytes + sizeof(ParameterPackHead));
  for (uint32_t i = 0; i < head->parameter_cnt; ++i) {
    const ParameterDescriptor& d = descs[i];
    // sizes and offsets are the file's claims: compare without sums that could wrap
    if (d.shape_len > kTensorShapeMaxLen || d.parameter_size > map->size ||
        d.parameter_offset > map->size - d.parameter_size) {
      MLLM_ERROR_EXIT(kError, "{}: descriptor {} is out of range", file_name, i);
      return;
    }
    const auto dtype = static_cast<DataTypes>(d.parameter_type);
    const size_t elem = dataTypeSize(dtype);
    if (elem == 0) {
      MLLM_ERROR_EXIT(kError, "{}: descriptor {} has an element type ({}) this loader does not know", file_name, i,
                      d.parameter_type);
      return;
    }
    Tensor::shape_t shape;
    uint64_t numel = 1;
    bool fits = true;
    for (uint64_t k = 0; k < d.shape_len; ++k) {
      const uint64_t dim = d.shape[k];
      if (dim > 0x7FFFFFFFull || (dim != 0 && numel > d.parameter_size / dim)) fits = false;
      numel *= dim;
      shape.push_back(static_cast<int32_t>(dim));
    }
    // every later copy is sized from the shape, so the shape must describe exactly the payload
    if (!fits || numel * elem != d.parameter_size) {
      MLLM_ERROR_EXIT(kError, "{}: descriptor {}: shape and element type do not match {} bytes", file_name, i,
                      d.parameter_size);
      return;
    }
    auto storage = TensorStorage::create(shape, dtype, kCPU);
    storage->ptr_ = const_cast<uint8_t*>(bytes) + d.parameter_offset;
    storage->mem_type_ = kParams;
    storage->keep_alive_ = mapping_;
    storage->name_ = fixedName(d.name, kParameterNameLen);
    params_[storage->name_] = TensorViewImpl::create(shape, storage);
  }
}

std::shared_ptr<TensorViewImpl> ParameterLoader::operator[](const std::string& name) {
  auto it = params_.find(name);
  if (it == params_.end()) {
    MLLM_ERROR_EXIT(kError, "parameter {} not found", name);
    return nullptr;
  }
  return it->second;
}

void ParameterLoader::insert(const std::string& name, const Tensor& t) {
  t.impl()->storage()->name_ = name;
  params_[name] = t.impl();
}

std::shared_ptr<ParameterLoader> load(const std::string& file_path) {
  return std::make_shared<ParameterLoader>(file_path);
}

void write(const std::string& file_path,
           const std::unordered_map<std::string, std::shared_ptr<TensorViewImpl>>& params,
           const std::string& model_name) {
  std::vector<std::pair<std::string, std::shared_ptr<TensorViewImpl>>> items(params.begin(), params.end());
  std::sort(items.begin(), items.end(), [](const auto& a, const auto& b) { return a.first < b.first; });

  ParameterPackHead head{};
  head.magic_number = kParameterMagicNumber;
  const std::string shown = model_name.empty() ? std::string("<ANONYMOUS MODEL PARAMS PACKAGE>") : model_name;
  std::strncpy(head.model_name, shown.c_str(), kParameterNameLen - 1);
  head.parameter_cnt = static_cast<uint32_t>(items.size());

  std::vector<ParameterDescriptor> descs(items.size());
  uint64_t offset = sizeof(head) + items.size() * sizeof(ParameterDescriptor);
  for (size_t i = 0; i < items.size(); ++i) {
    const auto& v = items[i].second;
    if (v->device() != kCPU) {
      MLLM_ERROR_EXIT(kError, "write: {} is not a host tensor", items[i].first);
      return;
    }
    const auto shape = v->shape();
    ParameterDescriptor& d = descs[i];
    std::memset(&d, 0, sizeof d);
    d.parameter_id = static_cast<uint32_t>(i);
    d.parameter_type = static_cast<uint32_t>(v->dtype());
    d.parameter_size = v->size();
    d.parameter_offset = offset;
    d.shape_len = shape.size();
    for (size_t k = 0; k < shape.size(); ++k) d.shape[k] = static_cast<uint64_t>(shape[k]);
    std::strncpy(d.name, items[i].first.c_str(), kParameterNameLen - 1);
    offset += d.parameter_size;
  }
  std::ofstream out(file_path, std::ios::binary);
  if (!out) {
    MLLM_ERROR_EXIT(kError, "cannot create {}", file_path);
    return;
  }
  out.write(reinterpret_cast<const char*>(&head), sizeof head);
  out.write(reinterpret_cast<const char*>(descs.data()),
            static_cast<std::streamsize>(descs.size() * sizeof(ParameterDescriptor)));
  for (auto& it : items) out.write(it.second->ptr<char>(), static_cast<std::streamsize>(it.second->size()));
}

void write(const std::string& file_path, const std::unordered_map<std::string, Tensor>& params,
           const std::string& model_name) {
  std::unordered_map<std::string, std::shared_ptr<TensorViewImpl>> impls;
  for (const auto& p : params) impls.insert({p.first, p.second.impl()});
  write(file_path, impls, model_name);
}

}  // namespace mllm

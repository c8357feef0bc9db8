// Implementation of the mllm core subset (see mllm_core.hpp for what is mirrored and from where).
#include "mllm_core.hpp"

#include <dlfcn.h>

#include <cstring>
#include <stdexcept>

namespace mllm {

size_t bytesOfType(DataTypes t) {
  switch (t) {
    case kFloat32: case kInt32: case kUInt32: return 4;
    case kFloat16: case kBFloat16: case kInt16: case kUInt16: return 2;
    case kInt64: return 8;
    case kGGUF_Q4_0: return 18;  // block_q4_0, mllm/core/DataTypes.hpp:111-121
    case kGGUF_Q8_0: return 34;  // block_q8_0, :164-170
    case kInt8: case kUInt8: case kByte: case kUInt4: return 1;  // kUInt4 is a 1-byte placeholder (DataTypes.hpp:336-339)
  }
  MLLM_ERROR_EXIT(ExitCode::kCoreError, "bytesOfType: unknown dtype %d", (int)t);
}
size_t lanesOfType(DataTypes t) { return (t == kGGUF_Q4_0 || t == kGGUF_Q8_0) ? 32 : 1; }

// ---- host allocator -----------------------------------------------------------------------------------------
namespace {
class HostAllocator final : public Allocator {
 public:
  bool ctrlByMemManager() override { return false; }
  bool alloc(Storage* s) override {
    void* p = nullptr;
    if (posix_memalign(&p, 64, s->size_ ? s->size_ : 64) != 0) return false;
    s->ptr_ = p;
    return true;
  }
  bool alloc(const Storage::ptr_t& s) override { return alloc(s.get()); }
  void free(Storage* s) override { std::free(s->ptr_); s->ptr_ = nullptr; }
  void free(const Storage::ptr_t& s) override { free(s.get()); }
  bool generalAlloc(void** ptr, size_t cap, size_t align) override { return posix_memalign(ptr, align < 8 ? 8 : align, cap) == 0; }
  void generalFree(void* ptr) override { std::free(ptr); }
  size_t allocSize(Storage* s) override { return s->size_; }
  size_t allocSize(const Storage::ptr_t& s) override { return s->size_; }
  [[nodiscard]] size_t alignSize() const override { return 64; }
};
}  // namespace

Storage::~Storage() {
  if (owned_ && ptr_) Context::instance().memoryManager()->free(this);
}

void MemoryManager::alloc(Storage* s) {
  auto it = allocators_.find(s->device_);
  if (it == allocators_.end()) MLLM_ERROR_EXIT(ExitCode::kCoreError, "no allocator registered for device %d", (int)s->device_);
  if (!it->second->alloc(s)) MLLM_ERROR_EXIT(ExitCode::kCoreError, "allocation of %zu bytes failed on device %d", s->size_, (int)s->device_);
  s->owned_ = true;
}
void MemoryManager::free(Storage* s) {
  auto it = allocators_.find(s->device_);
  if (it != allocators_.end()) it->second->free(s);
  s->owned_ = false;
}
Allocator::ptr_t MemoryManager::allocator(DeviceTypes device) {
  auto it = allocators_.find(device);
  return it == allocators_.end() ? nullptr : it->second;
}

// ---- Tensor --------------------------------------------------------------------------------------------------
size_t Tensor::numel() const {
  size_t n = 1;
  for (auto d : shape_) n *= (size_t)d;
  return n;
}
Tensor Tensor::empty(const shape_t& shape, DataTypes dtype, DeviceTypes device) {
  Tensor t;
  t.shape_ = shape;
  t.dtype_ = dtype;
  t.storage_ = std::make_shared<Storage>();
  t.storage_->device_ = device;
  t.storage_->size_ = t.bytes();
  return t;
}
Tensor Tensor::fromExternal(void* ptr, const shape_t& shape, DataTypes dtype, DeviceTypes device) {
  Tensor t = empty(shape, dtype, device);
  t.storage_->ptr_ = ptr;
  return t;
}
Tensor& Tensor::alloc() {
  MLLM_RT_ASSERT(storage_ && !storage_->ptr_);
  Context::instance().memoryManager()->alloc(storage_.get());
  return *this;
}
Tensor Tensor::view(const shape_t& shape) const {
  Tensor t = *this;
  t.shape_ = shape;
  int neg = -1;
  size_t known = 1;
  for (size_t i = 0; i < shape.size(); i++) {
    if (shape[i] < 0) neg = (int)i; else known *= (size_t)shape[i];
  }
  if (neg >= 0) t.shape_[neg] = (int32_t)(numel() / known);
  MLLM_RT_ASSERT_EQ(t.numel(), numel());
  return t;
}
Tensor Tensor::to(DeviceTypes device) const {
  if (device == this->device()) return *this;
  return Context::instance().buildOpAndSubmitTask(OpTypes::kX2X, aops::X2XOpOptions{.device = device}, {*this}, device)[0];
}

Tensor ParameterFile::pull(const std::string& name) {
  auto it = data_.find(name);
  if (it == data_.end()) MLLM_ERROR_EXIT(ExitCode::kIOError, "ParameterFile: tensor '%s' not found", name.c_str());
  return it->second;
}

// ---- BaseOp / aops -----------------------------------------------------------------------------------------
void BaseOp::setup(const std::vector<Tensor>&, std::vector<Tensor>& outputs) {
  for (auto& o : outputs)
    if (!o.ptr<void>()) o.alloc();
}

namespace aops {
LinearImplTypes str2LinearImplTypes(const std::string& str) {
  static const std::unordered_map<std::string, LinearImplTypes> map = {
      {"Default", LinearImplTypes::kDefault}, {"BLAS", LinearImplTypes::kBLAS}, {"GGUF", LinearImplTypes::kGGUF},
      {"MllmBlas", LinearImplTypes::kMllmBlas}};
  auto it = map.find(str);
  return it == map.end() ? LinearImplTypes::kDefault : it->second;
}

void LinearOp::load(const ParameterFile::ptr_t& ploader) {
  weight_ = ploader->pull(getName() + ".weight");
  if (weight_.rank() != 2) weight_ = weight_.view({options_.out_channels, -1});
  if (options_.bias) {
    bias_ = ploader->pull(getName() + ".bias");
    bias_ = bias_.view({options_.out_channels});
  }
}
void LinearOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  if (options_.isRedirect()) {
    outputs.emplace_back(inputs[1]);
    return;
  }
  auto out_shape = inputs[0].shape();
  MLLM_RT_ASSERT_EQ(out_shape[out_shape.size() - 1], options_.in_channels);
  out_shape[out_shape.size() - 1] = options_.out_channels;
  outputs.emplace_back(Tensor::empty(out_shape, inputs[0].dtype(), inputs[0].device()));
}
void LinearOp::setup(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  if (options_.isRedirect()) return;
  BaseOp::setup(inputs, outputs);
}
ParameterFile::ptr_t LinearOp::getParams() {
  auto p = ParameterFile::create();
  p->push(getName() + ".weight", weight_);
  if (options_.bias) p->push(getName() + ".bias", bias_);
  return p;
}

void MatMulOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  const auto& a = inputs[0].shape();
  const auto& b = inputs[1].shape();
  MLLM_RT_ASSERT(a.size() >= 2 && b.size() >= 2);
  const int M = options_.transpose_a ? a[a.size() - 1] : a[a.size() - 2];
  const int Ka = options_.transpose_a ? a[a.size() - 2] : a[a.size() - 1];
  const int Kb = options_.transpose_b ? b[b.size() - 1] : b[b.size() - 2];
  const int N = options_.transpose_b ? b[b.size() - 2] : b[b.size() - 1];
  MLLM_RT_ASSERT_EQ(Ka, Kb);
  auto o = a;
  o[o.size() - 2] = M;
  o[o.size() - 1] = N;
  outputs.emplace_back(Tensor::empty(o, inputs[0].dtype(), inputs[0].device()));
}

void X2XOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  outputs.emplace_back(Tensor::empty(inputs[0].shape(), inputs[0].dtype(), options_.device));
}
}  // namespace aops

// ---- Backend / Context ---------------------------------------------------------------------------------------
BaseOp::ptr_t Backend::createOp(OpTypes op_type, const BaseOpOptionsBase& base_options) {
  auto it = op_factories_.find(op_type);
  if (it == op_factories_.end()) MLLM_ERROR_EXIT(ExitCode::kCoreError, "op type %d is not registered on device %d", (int)op_type, (int)device_);
  auto op = it->second->create(base_options);
  op->setDeviceType(device_);
  return op;
}

Context& Context::instance() {
  static Context ctx;
  return ctx;
}
Backend::ptr_t Context::getBackend(const DeviceTypes& device) {
  auto it = backends_.find(device);
  if (it == backends_.end()) MLLM_ERROR_EXIT(ExitCode::kCoreError, "Backend for device %d not found", (int)device);
  return it->second;
}
std::vector<Tensor> Context::buildOpAndSubmitTask(OpTypes op_type, const BaseOpOptionsBase& options, const std::vector<Tensor>& inputs,
                                                  DeviceTypes special_device) {
  DeviceTypes device = special_device != kDeviceTypes_End ? special_device : inputs[0].device();
  if (special_device != kDeviceTypes_End && special_device != inputs[0].device()) {
    const DeviceTypes in_dev = inputs[0].device();  // prefer the non-CPU side (mllm/engine/Context.cpp:54-66)
    if (special_device == kCPU && in_dev != kCPU) device = in_dev;
  }
  auto op = getBackend(device)->createOp(op_type, options);
  std::vector<Tensor> outputs;
  op->reshape(inputs, outputs);
  op->setup(inputs, outputs);
  op->forward(inputs, outputs);
  return outputs;
}
int32_t Context::registerCustomizedOp(DeviceTypes device, const std::string& name, const std::shared_ptr<BaseOpFactory>& factory) {
  const int32_t id = ++dynamic_op_type_counter_;
  factory->__forceSetType(id);
  getBackend(device)->regOpFactory(factory);
  op_name_table_[{(int32_t)device, name}] = id;
  return id;
}
int32_t Context::lookupCustomizedOpId(DeviceTypes device, const std::string& name) {
  auto it = op_name_table_.find({(int32_t)device, name});
  if (it == op_name_table_.end()) MLLM_ERROR_EXIT(ExitCode::kCoreError, "customized op '%s' not found", name.c_str());
  return it->second;
}

void initializeContext() {
  auto& ctx = Context::instance();
  if (!ctx.memoryManager()->allocator(kCPU)) ctx.memoryManager()->registerAllocator(kCPU, std::make_shared<HostAllocator>());
}

void loadOpPackage(const std::string& path) {
  void* handle = dlopen(path.c_str(), RTLD_LAZY);
  if (!handle) throw std::runtime_error("Failed to load plugin library: " + std::string(dlerror()));
  typedef void* (*DescriptorFunc)();
  auto descriptor = (DescriptorFunc)dlsym(handle, "opPackageDescriptor");
  if (!descriptor) {
    dlclose(handle);
    throw std::runtime_error("Failed to find opPackageDescriptor function in plugin: " + path);
  }
  auto* pkg = static_cast<PluginOpPackageDescriptor*>(descriptor());
  MLLM_RT_ASSERT(pkg != nullptr);
  for (int i = 0; i < pkg->op_factories_count; ++i) {
    // the host never calls the package's free function (mllm/backends/base/PluginSystem.cpp:72-76)
    std::shared_ptr<BaseOpFactory> factory((BaseOpFactory*)(pkg->op_factory_create_funcs[i]()), [](BaseOpFactory*) {});
    Context::instance().registerCustomizedOp(static_cast<DeviceTypes>(pkg->device_type), std::string(pkg->op_factories_names[i]), factory);
  }
}

}  // namespace mllm

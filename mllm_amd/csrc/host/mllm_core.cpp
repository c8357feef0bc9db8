// Implementation of the mllm core subset (see mllm_core.hpp for what is mirrored and from where).
#include "mllm_core.hpp"

#include <cstring>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <fstream>

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
    case kGGUF_Q4_K: return 144; // block_q4_K, :139-147
    case kGGUF_Q6_K: return 210; // block_q6_K, :153-160
    case kInt8: case kUInt8: case kByte: case kUInt4: return 1;  // kUInt4 is a 1-byte placeholder (DataTypes.hpp:336-339)
  }
  MLLM_ERROR_EXIT(ExitCode::kCoreError, "bytesOfType: unknown dtype %d", (int)t);
}
size_t lanesOfType(DataTypes t) { return (t == kGGUF_Q4_0 || t == kGGUF_Q8_0) ? 32 : ((t == kGGUF_Q4_K || t == kGGUF_Q6_K) ? 256 : 1); }

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

void RMSNormOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  outputs.emplace_back(Tensor::empty(inputs[0].shape(), inputs[0].dtype(), inputs[0].device()));
}
void TopKOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  auto shape = inputs[0].shape();
  const int dim = options_.dim < 0 ? options_.dim + (int)shape.size() : options_.dim;
  MLLM_RT_ASSERT(dim >= 0 && dim < (int)shape.size() && options_.k >= 1 && options_.k <= shape[dim]);
  shape[dim] = options_.k;
  outputs.emplace_back(Tensor::empty(shape, inputs[0].dtype(), inputs[0].device()));
  outputs.emplace_back(Tensor::empty(shape, kInt32, inputs[0].device()));
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

// ---- model files ---------------------------------------------------------------------------------------------
namespace {
constexpr int32_t kV1Magic = 20012;
constexpr int32_t kV2Magic = 0x519A, kV2Version = 2;
constexpr size_t kV2ModelName = 512, kV2ParamName = 256, kV2ShapeLen = 16;
struct __attribute__((packed)) V2Header {
  int32_t magic_number, version;
  char model_name[kV2ModelName];
  uint32_t num_params;
  uint64_t params_desc_offset;
};
struct __attribute__((packed)) V2Param {
  uint32_t parameter_id, parameter_type;
  uint64_t parameter_size, parameter_offset, shape_len;
  int32_t shape[kV2ShapeLen];
  char name[kV2ParamName];
};
static_assert(sizeof(V2Header) == 532 && sizeof(V2Param) == 352, "model file v2 layout");

// Offsets and lengths come from the file: every range check is written so that it cannot wrap (n > size || off > size - n),
// and nothing is allocated from a length that exceeds the file.
bool rangeInside(uint64_t off, uint64_t n, uint64_t size) { return n <= size && off <= size - n; }

template <typename T>
T take(const std::vector<char>& buf, size_t& pos) {
  MLLM_RT_ASSERT(pos <= buf.size() && sizeof(T) <= buf.size() - pos);
  T v;
  std::memcpy(&v, buf.data() + pos, sizeof(T));
  pos += sizeof(T);
  return v;
}
// bytes a tensor of this shape and type occupies, without allocating it; UINT64_MAX for a negative extent or an overflow
uint64_t shapeBytes(const Tensor::shape_t& shape, DataTypes dtype) {
  uint64_t numel = 1;
  for (int32_t d : shape) {
    if (d < 0) return UINT64_MAX;
    if (d != 0 && numel > (UINT64_MAX / 64) / (uint64_t)d) return UINT64_MAX;
    numel *= (uint64_t)d;
  }
  return numel / lanesOfType(dtype) * bytesOfType(dtype);
}
Tensor readTensor(std::ifstream& f, uint64_t file_size, const std::string& name, const Tensor::shape_t& shape, DataTypes dtype,
                  uint64_t offset, uint64_t stored_bytes) {
  const uint64_t need = shapeBytes(shape, dtype);
  if (stored_bytes < need || !rangeInside(offset, need, file_size))
    MLLM_ERROR_EXIT(ExitCode::kIOError, "model file: tensor '%s' is truncated", name.c_str());
  Tensor t = Tensor::empty(shape, dtype, kCPU).alloc();
  MLLM_RT_ASSERT(need == t.bytes());
  f.seekg((std::streamoff)offset, std::ios::beg);
  f.read(t.ptr<char>(), (std::streamsize)t.bytes());
  if (!f) MLLM_ERROR_EXIT(ExitCode::kIOError, "model file: tensor '%s' is truncated", name.c_str());
  t.setName(name);
  return t;
}
}  // namespace

// The parsing is the same for a mapped file and for one that is read tensor by tensor: `bytes(offset, n)` hands out the
// descriptor bytes, `tensor(...)` makes the tensor (a view into the mapping, or a copy read from the stream).
template <typename Bytes, typename MakeTensor>
static void parseModelFile(const std::string& file_name, ModelFileVersion version, uint64_t file_size, const ParameterFile::ptr_t& pf,
                           Bytes&& bytes, MakeTensor&& tensor) {
  if (version == ModelFileVersion::kV1) {
    int32_t magic = 0;
    uint64_t desc_bytes = 0;
    bytes(0, 4, &magic);
    bytes(4, 8, &desc_bytes);
    MLLM_RT_ASSERT_EQ(kV1Magic, magic);
    if (!rangeInside(12, desc_bytes, file_size))
      MLLM_ERROR_EXIT(ExitCode::kIOError, "model file: descriptor section truncated: %s", file_name.c_str());
    std::vector<char> buf(desc_bytes);
    bytes(12, desc_bytes, buf.data());
    struct Item { std::string name; uint64_t len, offset; int32_t dtype; };
    std::vector<Item> items;
    for (size_t pos = 0; pos < buf.size();) {
      Item it;
      const uint32_t name_len = take<uint32_t>(buf, pos);
      MLLM_RT_ASSERT(name_len <= buf.size() - pos);
      it.name.assign(buf.data() + pos, name_len);
      pos += name_len;
      it.len = take<uint64_t>(buf, pos);
      it.offset = take<uint64_t>(buf, pos);
      it.dtype = take<int32_t>(buf, pos);
      items.push_back(it);
    }
    for (const auto& it : items) {
      const auto dtype = static_cast<DataTypes>(it.dtype);
      const Tensor::shape_t shape = {(int32_t)(it.len / bytesOfType(dtype) * lanesOfType(dtype))};  // flat, as the reference
      pf->push(it.name, tensor(it.name, shape, dtype, it.offset, it.len));
    }
  } else {
    V2Header h{};
    bytes(0, sizeof(h), &h);
    MLLM_RT_ASSERT_EQ(kV2Magic, h.magic_number);
    MLLM_RT_ASSERT_EQ(kV2Version, h.version);
    if (!rangeInside(h.params_desc_offset, (uint64_t)h.num_params * sizeof(V2Param), file_size))
      MLLM_ERROR_EXIT(ExitCode::kIOError, "model file: descriptor section truncated: %s", file_name.c_str());
    std::vector<V2Param> descs(h.num_params);
    bytes(h.params_desc_offset, descs.size() * sizeof(V2Param), descs.data());  // an extra data segment in front of it is skipped
    for (const auto& d : descs) {
      const std::string name(d.name, strnlen(d.name, sizeof(d.name)));
      MLLM_RT_ASSERT(d.shape_len <= kV2ShapeLen);
      Tensor::shape_t shape(d.shape, d.shape + d.shape_len);
      pf->push(name, tensor(name, shape, static_cast<DataTypes>(d.parameter_type), d.parameter_offset, d.parameter_size));
    }
  }
  (void)file_name;
}

MappedFile::MappedFile(const std::string& filename) {
  fd_ = ::open(filename.c_str(), O_RDONLY);
  if (fd_ < 0) MLLM_ERROR_EXIT(ExitCode::kIOError, "Failed to open file for reading: %s", filename.c_str());
  struct stat st {};
  if (::fstat(fd_, &st) != 0 || st.st_size <= 0) MLLM_ERROR_EXIT(ExitCode::kIOError, "Failed to stat file: %s", filename.c_str());
  size_ = (size_t)st.st_size;
  mapping_ = ::mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
  if (mapping_ == MAP_FAILED) MLLM_ERROR_EXIT(ExitCode::kIOError, "Failed to map file: %s", filename.c_str());
}
MappedFile::~MappedFile() {
  if (mapping_ && mapping_ != MAP_FAILED) ::munmap(mapping_, size_);
  if (fd_ >= 0) ::close(fd_);
}

// mmap = true (the reference's default, mllm/mllm.hpp:210-211; mllm/core/ParameterFile.cpp:68-116): tensors are views into
// the read-only mapping -- nothing is copied into host memory, pages come in when the upload reads them, and the
// ParameterFile keeps the mapping alive.  mmap = false reads every tensor into memory of its own.
ParameterFile::ptr_t load(const std::string& file_name, ModelFileVersion version, DeviceTypes map_2_device, bool mmap) {
  if (map_2_device != kCPU || (version != ModelFileVersion::kV1 && version != ModelFileVersion::kV2))
    return ParameterFile::create();  // "return empty if not match all" (mllm/mllm.cpp:142-143)
  auto pf = ParameterFile::create(version);
  if (mmap) {
    auto mf = MappedFile::create(file_name);
    pf->setMappedFile(mf);
    char* base = static_cast<char*>(mf->data());
    const size_t size = mf->size();
    parseModelFile(
        file_name, version, size, pf,
        [&](uint64_t off, uint64_t n, void* dst) {
          if (!rangeInside(off, n, size)) MLLM_ERROR_EXIT(ExitCode::kIOError, "model file: descriptor section truncated: %s", file_name.c_str());
          std::memcpy(dst, base + off, n);
        },
        [&](const std::string& name, const Tensor::shape_t& shape, DataTypes dtype, uint64_t offset, uint64_t stored_bytes) {
          const uint64_t need = shapeBytes(shape, dtype);
          if (stored_bytes < need || !rangeInside(offset, need, size))
            MLLM_ERROR_EXIT(ExitCode::kIOError, "model file: tensor '%s' is truncated", name.c_str());
          Tensor t = Tensor::fromExternal(base + offset, shape, dtype, kCPU);
          MLLM_RT_ASSERT(need == t.bytes());
          t.setName(name);
          return t;
        });
    return pf;
  }
  std::ifstream f(file_name, std::ios::binary);
  if (!f.is_open()) MLLM_ERROR_EXIT(ExitCode::kIOError, "Failed to open file for reading: %s", file_name.c_str());
  f.seekg(0, std::ios::end);
  const uint64_t fsize = (uint64_t)std::max<std::streamoff>(0, f.tellg());
  parseModelFile(
      file_name, version, fsize, pf,
      [&](uint64_t off, uint64_t n, void* dst) {
        if (!rangeInside(off, n, fsize)) MLLM_ERROR_EXIT(ExitCode::kIOError, "model file: descriptor section truncated: %s", file_name.c_str());
        f.seekg((std::streamoff)off, std::ios::beg);
        f.read(static_cast<char*>(dst), (std::streamsize)n);
        if (!f) MLLM_ERROR_EXIT(ExitCode::kIOError, "model file: descriptor section truncated: %s", file_name.c_str());
      },
      [&](const std::string& name, const Tensor::shape_t& shape, DataTypes dtype, uint64_t offset, uint64_t stored_bytes) {
        return readTensor(f, fsize, name, shape, dtype, offset, stored_bytes);
      });
  return pf;
}

void save(const std::string& file_name, const ParameterFile::ptr_t& parameter_file, ModelFileVersion version,
          DeviceTypes map_2_device) {
  if (map_2_device != kCPU || (version != ModelFileVersion::kV1 && version != ModelFileVersion::kV2)) return;
  std::ofstream out(file_name, std::ios::binary);
  if (!out.is_open()) MLLM_ERROR_EXIT(ExitCode::kIOError, "Failed to open file for writing: %s", file_name.c_str());
  const auto& dict = parameter_file->dict();
  if (version == ModelFileVersion::kV1) {
    uint64_t desc_bytes = 0;
    for (const auto& [name, t] : dict) desc_bytes += 4 + name.size() + 8 + 8 + 4;
    out.write(reinterpret_cast<const char*>(&kV1Magic), 4);
    out.write(reinterpret_cast<const char*>(&desc_bytes), 8);
    uint64_t offset = 12 + desc_bytes;  // absolute, from the start of the file
    for (const auto& [name, t] : dict) {
      const uint32_t name_len = (uint32_t)name.size();
      const uint64_t len = t.bytes();
      const int32_t dtype = (int32_t)t.dtype();
      out.write(reinterpret_cast<const char*>(&name_len), 4);
      out.write(name.data(), name_len);
      out.write(reinterpret_cast<const char*>(&len), 8);
      out.write(reinterpret_cast<const char*>(&offset), 8);
      out.write(reinterpret_cast<const char*>(&dtype), 4);
      offset += len;
    }
  } else {
    V2Header h{};
    h.magic_number = kV2Magic;
    h.version = kV2Version;
    h.num_params = (uint32_t)dict.size();
    h.params_desc_offset = sizeof(V2Header);
    out.write(reinterpret_cast<const char*>(&h), sizeof(h));
    uint64_t offset = sizeof(V2Header) + dict.size() * sizeof(V2Param);
    uint32_t id = 0;
    for (const auto& [name, t] : dict) {
      V2Param d{};
      d.parameter_id = id++;
      d.parameter_type = (uint32_t)t.dtype();
      d.parameter_size = t.bytes();
      d.parameter_offset = offset;
      d.shape_len = t.shape().size();
      MLLM_RT_ASSERT(d.shape_len <= kV2ShapeLen);
      for (size_t i = 0; i < t.shape().size(); i++) d.shape[i] = t.shape()[i];
      std::strncpy(d.name, name.c_str(), kV2ParamName - 1);
      out.write(reinterpret_cast<const char*>(&d), sizeof(d));
      offset += t.bytes();
    }
  }
  for (const auto& [name, t] : dict) {
    MLLM_RT_ASSERT_EQ(t.device(), kCPU);
    out.write(t.ptr<char>(), (std::streamsize)t.bytes());
  }
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

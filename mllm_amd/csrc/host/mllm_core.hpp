// The slice of mllm's core / engine / backend-base API that a device backend's Linear, MatMul and X2X ops touch,
// written from scratch with the same names, argument meaning and error behaviour, so that the HIP backend sources in
// this directory compile unchanged against the real headers when dropped into an mllm checkout.
//
// Reference interfaces mirrored here (file:line under the reference checkout):
//   mllm/core/DataTypes.hpp:351-425        DataTypes ids (model-file ids: kGGUF_Q4_0 = 2, kGGUF_Q8_0 = 8, ...)
//   mllm/core/DeviceTypes.hpp:10-27        DeviceTypes; plug-in devices start at kDynamicDeviceType_Start = 4096
//   mllm/core/OpTypes.hpp:20-33            kMatMul = 6, kLinear = 8, kX2X = 19
//   mllm/core/Storage.hpp                  Storage{ptr_, size_, device_}
//   mllm/core/BaseOp.hpp:24-212            BaseOpOptions, BaseOpOptionsBase (type erased, as<T>() throws std::bad_cast),
//                                          BaseOp{load,trace,reshape,setup,forward,getParams}, TypedOpFactory
//   mllm/core/aops/LinearOp.hpp:11-201     LinearImplTypes, LinearOpOptions, LinearOp (load/reshape/setup/getParams)
//   mllm/core/aops/MatMulOp.hpp:11-68      MatMulOpOptions, MatMulOp
//   mllm/core/aops/X2XOp.hpp               X2XOpOptions, X2XOp
//   mllm/backends/base/Allocator.hpp:10-33 Allocator (10 pure virtuals)
//   mllm/backends/base/Backend.hpp:13-45   Backend{createOp, regOpFactory<...>, device, allocator, isWeightOnDevice}
//   mllm/backends/base/PluginInterface.hpp:11-52  opPackageDescriptor() / PluginOpPackageDescriptor
//   mllm/engine/Context.cpp:35-97          Context::{registerBackend, getBackend, buildOpAndSubmitTask}
//   mllm/utils/Common.hpp:42-53            MLLM_ERROR_EXIT / MLLM_RT_ASSERT terminate the process
// Everything else of the runtime (dispatchers, thread pools, IR tracing, the memory pool) is out of scope: dispatch is the
// synchronous reshape -> setup -> forward sequence of CPUDispatcher::process (mllm/backends/cpu/CPUDispatcher.cpp:56-62).
#pragma once
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <memory>
#include <string>
#include <typeinfo>
#include <unordered_map>
#include <vector>

namespace mllm {

enum class ExitCode : int32_t { kSuccess = 0, kCoreError = 1, kAssert = 2, kIOError = 3, kHIPError = 64 };

#define MLLM_ERROR_EXIT(code, ...)                                   \
  do {                                                               \
    std::fprintf(stderr, "[mllm ERROR] %s:%d ", __FILE__, __LINE__); \
    std::fprintf(stderr, __VA_ARGS__);                               \
    std::fprintf(stderr, "\n");                                      \
    std::exit(static_cast<int>(code));                               \
  } while (0)
#define MLLM_RT_ASSERT(cond)                                                            \
  do {                                                                                  \
    if (!(cond)) MLLM_ERROR_EXIT(::mllm::ExitCode::kAssert, "assertion failed: %s", #cond); \
  } while (0)
#define MLLM_RT_ASSERT_EQ(a, b) MLLM_RT_ASSERT((a) == (b))
#define NYI(...) MLLM_ERROR_EXIT(::mllm::ExitCode::kCoreError, "NYI: " __VA_ARGS__)

enum DataTypes : int32_t {
  kFloat32 = 0, kFloat16 = 1, kGGUF_Q4_0 = 2, kGGUF_Q8_0 = 8, kGGUF_Q4_K = 12, kGGUF_Q6_K = 14, kInt8 = 16, kInt16 = 17, kInt32 = 18,
  kBFloat16 = 128, kUInt8 = 129, kUInt16 = 130, kUInt32 = 131, kInt64 = 132, kByte = 134, kUInt4 = 137,
};
// bytes of one storage unit and elements ("lanes") per unit: mllm/core/DataTypes.hpp:645-648, TensorStorage.cpp:48-49
size_t bytesOfType(DataTypes t);
size_t lanesOfType(DataTypes t);

enum DeviceTypes : int32_t {
  kDeviceTypes_Start = 0, kCPU = 1, kCUDA = 2, kOpenCL = 3, kQNN = 4, kCUDAHost = 5, kAscend = 6, kAscendHost = 7,
  kDynamicDeviceType_Start = 4096,
  kHIP = kDynamicDeviceType_Start + 1,  // the id this backend registers under (DeviceTypes has no ROCm value)
  kDeviceTypes_End,
};

// values as in mllm/core/OpTypes.hpp:13-70 (only the slots this backend fills)
enum class OpTypes : int32_t {
  kOpType_Start = 0, kAdd = 2, kMul = 4, kMatMul = 6, kLinear = 8, kSoftmax = 10, kRMSNorm = 14, kSiLU = 15, kX2X = 19, kTopK = 49,
  kGraphBegin = 55, kGraphEnd = 56, kDynamicOp_Start = 4096
};

enum class ModelFileVersion : int32_t { kV1 = 1, kV2 = 2, kUserTemporary = 3 };

// ---------------------------------------------------------------------------------------------------------
class Storage : public std::enable_shared_from_this<Storage> {
 public:
  using ptr_t = std::shared_ptr<Storage>;
  virtual ~Storage();
  void* ptr_ = nullptr;
  size_t size_ = 0;
  DeviceTypes device_ = kCPU;
  bool owned_ = false;  // allocated through the memory manager (freed with it); false for borrowed / mmap'd memory
};

class Allocator {
 public:
  using ptr_t = std::shared_ptr<Allocator>;
  virtual ~Allocator() = default;
  virtual bool ctrlByMemManager() = 0;
  virtual bool alloc(Storage* storage) = 0;
  virtual bool alloc(const Storage::ptr_t& storage) = 0;
  virtual void free(Storage* storage) = 0;
  virtual void free(const Storage::ptr_t& storage) = 0;
  virtual bool generalAlloc(void** ptr, size_t cap, size_t align) = 0;
  virtual void generalFree(void* ptr) = 0;
  virtual size_t allocSize(Storage* storage) = 0;
  virtual size_t allocSize(const Storage::ptr_t& storage) = 0;
  [[nodiscard]] virtual size_t alignSize() const = 0;
};

// Value handle over shared storage; shape in elements, contiguous row-major only (all this path needs).
class Tensor {
 public:
  using shape_t = std::vector<int32_t>;
  Tensor() = default;
  static Tensor nil() { return Tensor(); }
  static Tensor empty(const shape_t& shape, DataTypes dtype = kFloat32, DeviceTypes device = kCPU);  // descriptor only
  // wraps caller-owned memory (parameter files, test inputs); never freed by the tensor
  static Tensor fromExternal(void* ptr, const shape_t& shape, DataTypes dtype, DeviceTypes device);
  Tensor& alloc();  // through Context's memory manager -> the device's Allocator
  [[nodiscard]] bool isNil() const { return !storage_; }
  explicit operator bool() const { return !isNil(); }
  [[nodiscard]] const shape_t& shape() const { return shape_; }
  [[nodiscard]] DataTypes dtype() const { return dtype_; }
  [[nodiscard]] DeviceTypes device() const { return storage_ ? storage_->device_ : kCPU; }
  [[nodiscard]] size_t numel() const;
  [[nodiscard]] size_t bytes() const { return numel() / lanesOfType(dtype_) * bytesOfType(dtype_); }
  [[nodiscard]] size_t rank() const { return shape_.size(); }
  [[nodiscard]] Tensor view(const shape_t& shape) const;
  [[nodiscard]] Tensor to(DeviceTypes device) const;  // X2X op created on the non-CPU side (mllm/core/Tensor.cpp:442-445)
  template <typename T>
  [[nodiscard]] T* ptr() const { return storage_ ? reinterpret_cast<T*>(static_cast<char*>(storage_->ptr_) + offset_bytes_) : nullptr; }
  [[nodiscard]] const Storage::ptr_t& storage() const { return storage_; }
  void setName(const std::string& n) { name_ = n; }
  [[nodiscard]] const std::string& name() const { return name_; }

 private:
  Storage::ptr_t storage_;
  shape_t shape_;
  DataTypes dtype_ = kFloat32;
  size_t offset_bytes_ = 0;
  std::string name_;
};

// A model file mapped read-only into the address space (mllm/core/MappedFile.hpp:21-44): tensors of a ParameterFile read
// with mmap = true point into the mapping, which the ParameterFile keeps alive.
class MappedFile {
 public:
  using ptr_t = std::shared_ptr<MappedFile>;
  explicit MappedFile(const std::string& filename);
  static ptr_t create(const std::string& filename) { return std::make_shared<MappedFile>(filename); }
  ~MappedFile();
  MappedFile(const MappedFile&) = delete;
  MappedFile& operator=(const MappedFile&) = delete;
  [[nodiscard]] void* data() const { return mapping_; }
  [[nodiscard]] size_t size() const { return size_; }

 private:
  int fd_ = -1;
  size_t size_ = 0;
  void* mapping_ = nullptr;
};

class ParameterFile {
 public:
  using ptr_t = std::shared_ptr<ParameterFile>;
  static ptr_t create(ModelFileVersion v = ModelFileVersion::kUserTemporary) { return std::make_shared<ParameterFile>(v); }
  explicit ParameterFile(ModelFileVersion v) : version_(v) {}
  void push(const std::string& name, const Tensor& t) { data_[name] = t; }
  Tensor pull(const std::string& name);  // a missing name terminates (mllm/core/ParameterFile.cpp:48-51)
  [[nodiscard]] bool has(const std::string& name) const { return data_.count(name) != 0; }
  [[nodiscard]] ModelFileVersion version() const { return version_; }
  [[nodiscard]] const std::map<std::string, Tensor>& dict() const { return data_; }
  void setMappedFile(const MappedFile::ptr_t& f) { mapped_file_ = f; }  // mllm/core/ParameterFile.cpp:75-78
  [[nodiscard]] const MappedFile::ptr_t& getMappedFile() const { return mapped_file_; }

 private:
  ModelFileVersion version_;
  MappedFile::ptr_t mapped_file_;
  std::map<std::string, Tensor> data_;
};

// ---------------------------------------------------------------------------------------------------------
template <typename DerivedT>
class BaseOpOptions {
 public:
  [[nodiscard]] inline int getThreads() const { return threads_; }
  inline void setThreads(int threads) { threads_ = threads; }
  inline void setInplace(bool inplace) { inplace_ = inplace; }
  [[nodiscard]] bool isInplace() const { return inplace_; }
  inline void setRedirect(bool redirect) { redirect_ = redirect; }
  [[nodiscard]] bool isRedirect() const { return redirect_; }

 private:
  bool inplace_ = false;
  bool redirect_ = false;
  int threads_ = 8;
};

class BaseOpOptionsBase {
 public:
  template <typename T>
  BaseOpOptionsBase(const T& cargo) : inner_(std::make_unique<Model<T>>(cargo)) {}  // NOLINT: implicit on purpose
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
  std::unique_ptr<Concept> inner_;
};

class BaseOp : public std::enable_shared_from_this<BaseOp> {
 public:
  using ptr_t = std::shared_ptr<BaseOp>;
  explicit BaseOp(OpTypes op_type) : op_type_(op_type) {}
  virtual ~BaseOp() = default;
  virtual void load(const ParameterFile::ptr_t&) {}
  virtual void trace(void*, const std::vector<Tensor>&, std::vector<Tensor>&) {}
  virtual void forward(const std::vector<Tensor>&, std::vector<Tensor>&) {}
  virtual void reshape(const std::vector<Tensor>&, std::vector<Tensor>&) {}
  virtual void setup(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs);  // allocates every output
  virtual ParameterFile::ptr_t getParams() { return ParameterFile::create(); }
  [[nodiscard]] std::string getName() const { return name_; }
  void setName(const std::string& name) { name_ = name; }
  [[nodiscard]] DeviceTypes getDevice() const { return device_type_; }
  void setDeviceType(DeviceTypes d) { device_type_ = d; }
  [[nodiscard]] OpTypes getOpType() const { return op_type_; }

 private:
  DeviceTypes device_type_ = kCPU;
  std::string name_;
  OpTypes op_type_;
};

struct BaseOpFactory {
  virtual ~BaseOpFactory() = default;
  virtual std::shared_ptr<BaseOp> create(const BaseOpOptionsBase& base_cargo) = 0;
  [[nodiscard]] virtual OpTypes opType() const = 0;
  inline void __forceSetType(int32_t type) { type_ = type; }
  int32_t type_ = 0;
};

template <OpTypes type, typename CargoT>
class TypedOpFactory : public BaseOpFactory {
 public:
  TypedOpFactory() { __forceSetType(static_cast<int32_t>(type)); }
  std::shared_ptr<BaseOp> create(const BaseOpOptionsBase& base_cargo) override { return createOpImpl(base_cargo.as<CargoT>()); }
  [[nodiscard]] OpTypes opType() const override { return static_cast<OpTypes>(type_); }

 protected:
  virtual std::shared_ptr<BaseOp> createOpImpl(const CargoT& cargo) = 0;
};

// ---------------------------------------------------------------------------------------------------------
namespace aops {

enum class LinearImplTypes { kLinearImplTypes_Start = 0, kDefault, kBLAS, kGGUF, kMllmBlas, kLinearImplTypes_End };
LinearImplTypes str2LinearImplTypes(const std::string& str);

struct LinearOpOptions : public BaseOpOptions<LinearOpOptions> {
  int32_t in_channels = 0;
  int32_t out_channels = 0;
  bool bias = false;
  LinearImplTypes impl_type = LinearImplTypes::kDefault;
};

class LinearOp : public BaseOp {
 public:
  explicit LinearOp(const LinearOpOptions& options) : BaseOp(OpTypes::kLinear), options_(options) {}
  void load(const ParameterFile::ptr_t& ploader) override;  // pulls "<name>.weight" (viewed [out, in]) and "<name>.bias"
  void forward(const std::vector<Tensor>&, std::vector<Tensor>&) override { NYI("LinearOp::forward not implemented in aops base."); }
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  void setup(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  ParameterFile::ptr_t getParams() override;
  inline Tensor& weight() { return weight_; }
  inline Tensor& bias() { return bias_; }
  inline LinearOpOptions& options() { return options_; }

 protected:
  Tensor weight_;
  Tensor bias_;
  LinearOpOptions options_;
};

enum class MatMulOpType { kDefault = 0, kGGUF = 1, kBLAS = 2, kMllmBlas };
struct MatMulOpOptions : public BaseOpOptions<MatMulOpOptions> {
  bool transpose_a = false;
  bool transpose_b = false;
  MatMulOpType matmul_type = MatMulOpType::kDefault;
};
class MatMulOp : public BaseOp {
 public:
  explicit MatMulOp(const MatMulOpOptions& options) : BaseOp(OpTypes::kMatMul), options_(options) {}
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  inline const MatMulOpOptions& options() const { return options_; }

 protected:
  MatMulOpOptions options_;
};

struct X2XOpOptions : public BaseOpOptions<X2XOpOptions> {
  DeviceTypes device = kCPU;
};
class X2XOp : public BaseOp {
 public:
  explicit X2XOp(const X2XOpOptions& options) : BaseOp(OpTypes::kX2X), options_(options) {}
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  inline const X2XOpOptions& options() const { return options_; }

 protected:
  X2XOpOptions options_;
};

// ---- the operators around Linear in a decoder layer (mllm/core/aops/{RMSNormOp,SiLUOp,ElewiseOps,SoftmaxOp,TopKOp}.hpp) ----
struct RMSNormOpOptions : public BaseOpOptions<RMSNormOpOptions> {
  float epsilon = 1e-6f;
  bool add_unit_offset = false;  // Gemma
};
class RMSNormOp : public BaseOp {
 public:
  explicit RMSNormOp(const RMSNormOpOptions& options) : BaseOp(OpTypes::kRMSNorm), options_(options) {}
  void load(const ParameterFile::ptr_t& ploader) override { weight_ = ploader->pull(getName() + ".weight"); }  // aops/RMSNormOp.cpp:16-30
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  inline Tensor& weight() { return weight_; }
  inline const RMSNormOpOptions& options() const { return options_; }

 protected:
  Tensor weight_;
  RMSNormOpOptions options_;
};
struct SiLUOpOptions : public BaseOpOptions<SiLUOpOptions> {};
struct AddOpOptions : public BaseOpOptions<AddOpOptions> {};
struct MulOpOptions : public BaseOpOptions<MulOpOptions> {};
// output = the first input's shape and type (no broadcasting in this backend: both inputs must have the same shape)
template <OpTypes T, typename OptT>
class SameShapeOp : public BaseOp {
 public:
  explicit SameShapeOp(const OptT& options) : BaseOp(T), options_(options) {}
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override {
    outputs.emplace_back(Tensor::empty(inputs[0].shape(), inputs[0].dtype(), inputs[0].device()));
  }

 protected:
  OptT options_;
};
using SiLUOp = SameShapeOp<OpTypes::kSiLU, SiLUOpOptions>;
using AddOp = SameShapeOp<OpTypes::kAdd, AddOpOptions>;
using MulOp = SameShapeOp<OpTypes::kMul, MulOpOptions>;
struct SoftmaxOpOptions : public BaseOpOptions<SoftmaxOpOptions> {
  int axis = -1;
};
using SoftmaxOp = SameShapeOp<OpTypes::kSoftmax, SoftmaxOpOptions>;
struct TopKOpOptions : public BaseOpOptions<TopKOpOptions> {
  int k = 0;
  int dim = -1;
  bool largest = true;
  bool sorted = true;
};
class TopKOp : public BaseOp {
 public:
  explicit TopKOp(const TopKOpOptions& options) : BaseOp(OpTypes::kTopK), options_(options) {}
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;  // values (input type), indices int32

 protected:
  TopKOpOptions options_;
};

}  // namespace aops

// ---------------------------------------------------------------------------------------------------------
class Backend {
 public:
  using ptr_t = std::shared_ptr<Backend>;
  Backend(DeviceTypes device, const Allocator::ptr_t& allocator) : device_(device), allocator_(allocator) {}
  virtual ~Backend() = default;
  BaseOp::ptr_t createOp(OpTypes op_type, const BaseOpOptionsBase& base_options);
  template <typename... Args>
  void regOpFactory() { (..., (_reg_one_op_factory<Args>())); }
  void regOpFactory(const std::shared_ptr<BaseOpFactory>& factory) { op_factories_[factory->opType()] = factory; }
  [[nodiscard]] inline DeviceTypes device() const { return device_; }
  [[nodiscard]] inline Allocator::ptr_t allocator() const { return allocator_; }
  [[nodiscard]] virtual bool isWeightOnDevice() { return true; }

 protected:
  template <typename T>
  void _reg_one_op_factory() {
    auto ptr = std::make_shared<T>();
    op_factories_[ptr->opType()] = ptr;
  }
  DeviceTypes device_ = kCPU;
  Allocator::ptr_t allocator_ = nullptr;
  std::map<OpTypes, std::shared_ptr<BaseOpFactory>> op_factories_;
};

class MemoryManager {
 public:
  void registerAllocator(DeviceTypes device, const Allocator::ptr_t& allocator) { allocators_[device] = allocator; }
  void alloc(Storage* s);
  void free(Storage* s);
  [[nodiscard]] Allocator::ptr_t allocator(DeviceTypes device);

 private:
  std::map<DeviceTypes, Allocator::ptr_t> allocators_;
};

class Context {
 public:
  static Context& instance();
  void registerBackend(const Backend::ptr_t& b) { backends_[b->device()] = b; }
  Backend::ptr_t getBackend(const DeviceTypes& device);  // terminates when the device has no backend
  [[nodiscard]] bool hasBackend(DeviceTypes device) const { return backends_.count(device) != 0; }
  MemoryManager* memoryManager() { return &mm_; }
  // create the op on `device` (default: the inputs' device), then reshape -> setup -> forward, synchronously
  std::vector<Tensor> buildOpAndSubmitTask(OpTypes op_type, const BaseOpOptionsBase& options, const std::vector<Tensor>& inputs,
                                           DeviceTypes special_device = kDeviceTypes_End);
  int32_t registerCustomizedOp(DeviceTypes device, const std::string& name, const std::shared_ptr<BaseOpFactory>& factory);
  int32_t lookupCustomizedOpId(DeviceTypes device, const std::string& name);

 private:
  std::map<DeviceTypes, Backend::ptr_t> backends_;
  MemoryManager mm_;
  int32_t dynamic_op_type_counter_ = static_cast<int32_t>(OpTypes::kDynamicOp_Start);
  std::map<std::pair<int32_t, std::string>, int32_t> op_name_table_;
};

void initializeContext();                       // registers the host (CPU) allocator: mllm/mllm.hpp:145-164
// Model files, mllm/mllm.cpp:135-154 with mllm/core/ParameterFile.cpp:68-440 and the schemas
// mllm/core/schema/ModelFileV1.hpp:36-52 (magic 20012; name, byte length, offset, dtype per tensor; shapes are flat) and
// ModelFileV2.hpp:40-62 (magic 0x519A, version 2; 352-byte descriptors with dtype, size, offset, shape, name).
// mmap = true (the reference's default): the file is mapped read-only and the tensors are views into the mapping, which the
// ParameterFile keeps alive; mmap = false: every tensor is read into host memory of its own.  Offsets and lengths read from
// the file are checked against the file size in a form that cannot wrap; a file that fails a check ends the process as any
// other load error does.
ParameterFile::ptr_t load(const std::string& file_name, ModelFileVersion version = ModelFileVersion::kV1,
                          DeviceTypes map_2_device = kCPU, bool mmap = true);
void save(const std::string& file_name, const ParameterFile::ptr_t& parameter_file,
          ModelFileVersion version = ModelFileVersion::kV1, DeviceTypes map_2_device = kCPU);
void loadOpPackage(const std::string& path);    // dlopen + opPackageDescriptor(): mllm/backends/base/PluginSystem.cpp:37-90

}  // namespace mllm

// plugin C ABI (mllm/backends/base/PluginInterface.hpp:43-52)
#define MLLM_PLUGIN_OP_PACKAGE_DESCRIPTOR_VERSION 1
#define MLLM_PLUGIN_OP_PACKAGE_NAME_LEN 256
#define MLLM_PLUGIN_OP_PACKAGE_DESCRIPTOR_LEN 256
extern "C" {
typedef void* (*OpFactoryCreateFunc)();
typedef void (*OpFactoryFreeFunc)(void*);
#pragma pack(push, 4)
struct PluginOpPackageDescriptor {
  int32_t version = MLLM_PLUGIN_OP_PACKAGE_DESCRIPTOR_VERSION;
  char name[MLLM_PLUGIN_OP_PACKAGE_NAME_LEN];
  int32_t device_type;
  int32_t op_factories_count = 0;
  char op_factories_names[MLLM_PLUGIN_OP_PACKAGE_DESCRIPTOR_LEN][MLLM_PLUGIN_OP_PACKAGE_NAME_LEN];
  OpFactoryCreateFunc op_factory_create_funcs[MLLM_PLUGIN_OP_PACKAGE_DESCRIPTOR_LEN];
  OpFactoryFreeFunc op_factory_free_funcs[MLLM_PLUGIN_OP_PACKAGE_DESCRIPTOR_LEN];
};
#pragma pack(pop)
}

// HIP backend for mllm's op-factory boundary: allocator, backend, and the Linear / MatMul / X2X ops, on top of the C ABI
// in include/mllm_hip_qlinear.h.
//
// Follows the pattern of the reference's device backends:
//   registration      mllm/backends/opencl/OpenCLBackend.cpp:32-44, mllm/backends/ascend/Register.cpp:15-42
//   factories         mllm/backends/cpu/ops/LinearOp.hpp:21-26, mllm/backends/ascend/AscendBackend.cpp:31-50
//   device allocator  mllm/backends/cuda/CudaAllocator.cpp:10-65
//   weight-side names mllm/backends/ascend/ops/AscendLinearOp.cpp:42-48 ("<name>.weight.scale")
#pragma once
#include <map>

#include "mllm_core.hpp"

namespace mllm::hip {

class HipAllocator final : public Allocator {
 public:
  bool ctrlByMemManager() override { return false; }
  bool alloc(Storage* storage) override;
  bool alloc(const Storage::ptr_t& storage) override { return alloc(storage.get()); }
  void free(Storage* storage) override;
  void free(const Storage::ptr_t& storage) override { free(storage.get()); }
  bool generalAlloc(void** ptr, size_t cap, size_t align) override;
  void generalFree(void* ptr) override;
  size_t allocSize(Storage* storage) override;
  size_t allocSize(const Storage::ptr_t& storage) override { return allocSize(storage.get()); }
  [[nodiscard]] size_t alignSize() const override { return 256; }
  // told about every free so that the backend can drop what it keeps about that memory; cleared when the backend goes
  class HipBackend* owner = nullptr;
  // true when [ptr, ptr + bytes) lies inside an allocation this allocator made through alloc() and has not freed
  [[nodiscard]] bool owns(const void* ptr, size_t bytes) const;

 private:
  std::map<const char*, size_t> live_;  // start -> size of every Storage allocation
};

// How fp16 block scales are read (see MLLM_HIP_SCALE_* in the C header): IEEE bit patterns, or the x86 reference build's
// number-valued field.  Chosen per process: environment MLLM_HIP_SCALE_MODE = "ieee" (default) | "x86".
struct HipBackendConfig {
  int weight_scale_mode = 0;
  int act_scale_mode = 0;
  int device = 0;
  // Q4_0 / Q8_0 Linear with more than 8 rows: true = matrix-core path (fp16 operands with folded block scales, a second,
  // gemm-packed copy of the weight is built at load()); false = the block-dot kernel, which keeps the reference's fp32
  // block arithmetic.  MLLM_HIP_PREFILL=blockdot selects the latter.
  bool prefill_matrix_cores = true;
  // Decode hand-over: RMSNorm and the elementwise product also write the Q8_0 image of their result (up to 8 rows), and a
  // Q4_0 / Q8_0 Linear that then reads exactly that tensor takes the image instead of quantizing in every workgroup.
  // Results are bit-identical either way.  The image is dropped as soon as any op of this backend writes to, or the
  // allocator frees, the memory it describes.  Writes that bypass the backend (another backend's op, a caller's own
  // hipMemcpy into an activation tensor) are NOT seen and would leave a stale image behind, so the hand-over is opt-in:
  // off by default, MLLM_HIP_FOLD_IMAGES=1 (or setFoldImages) turns it on for graphs in which every writer of an
  // activation tensor is an op of this backend.  Images are only kept for memory this backend's allocator handed out
  // (never for external buffers, whose lifetime it cannot see) and at most kMaxImages at a time (oldest dropped first).
  bool fold_images = false;
};

class HipBackend final : public Backend {
 public:
  explicit HipBackend(const HipBackendConfig& cfg = HipBackendConfig());
  ~HipBackend() override;
  [[nodiscard]] void* stream() const { return stream_; }  // hipStream_t; default priority
  [[nodiscard]] const HipBackendConfig& config() const { return cfg_; }
  void setScaleModes(int weight_scale_mode, int act_scale_mode) {
    cfg_.weight_scale_mode = weight_scale_mode;
    cfg_.act_scale_mode = act_scale_mode;
    images_.clear();  // images carry the activation-scale convention they were written with
  }
  void synchronize() const;
  void setFoldImages(bool on) { cfg_.fold_images = on; images_.clear(); }

  // quantized images of activation tensors (see HipBackendConfig::fold_images)
  void* newImage(const void* tensor_ptr, size_t tensor_bytes, int rows, int64_t D);  // null when not applicable
  const void* findImage(const void* tensor_ptr, int rows, int64_t D) const;
  void noteWrite(const void* ptr, size_t bytes);  // every op calls this for its outputs before it launches
  [[nodiscard]] size_t imageCount() const { return images_.size(); }
  static constexpr size_t kMaxImages = 64;

 private:
  struct Image {
    const void* tensor_ptr;
    size_t tensor_bytes;
    int rows;
    int64_t D;
    Tensor data;
  };
  HipBackendConfig cfg_;
  void* stream_ = nullptr;
  std::vector<Image> images_;
  std::vector<Tensor> image_pool_;  // buffers of dropped images, reused (no allocation in steady state)
};

// Registers backend + allocator with the Context (idempotent).  The counterpart of initOpenCLBackend() / initAscendBackend().
std::shared_ptr<HipBackend> initHipBackend();

class HipLinearOp final : public aops::LinearOp {
 public:
  explicit HipLinearOp(const aops::LinearOpOptions& options);
  void load(const ParameterFile::ptr_t& ploader) override;
  void reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
  ParameterFile::ptr_t getParams() override;

 private:
  enum class Scheme { kNone, kQ4_0, kQ8_0, kQ4_K, kQ6_K, kW8A8, kW4A16 };
  Scheme scheme_ = Scheme::kNone;
  Tensor packed_;        // the repacked device copy the kernels read (every scheme)
  Tensor gemm_packed_;   // Q4_0 / Q8_0: the matrix-core layout for more than 8 rows
  Tensor weight_scale_;  // "<name>.weight.scale": fp32 [N] (W8A8) or fp16 [N][K/group] (W4A16)
  Tensor weight_zp_;     // "<name>.weight.zero_point": uint8 [N][ceil(K/group/2)] (W4A16)
  Tensor bias_dev_;      // bias in the form the kernel takes (fp32; bf16 for W4A16)
  Tensor workspace_;
  int group_ = 0;
};
class HipLinearOpFactory final : public TypedOpFactory<OpTypes::kLinear, aops::LinearOpOptions> {
 public:
  std::shared_ptr<BaseOp> createOpImpl(const aops::LinearOpOptions& options) override { return std::make_shared<HipLinearOp>(options); }
};

class HipMatMulOp final : public aops::MatMulOp {
 public:
  explicit HipMatMulOp(const aops::MatMulOpOptions& options) : aops::MatMulOp(options) {}
  void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
};
class HipMatMulOpFactory final : public TypedOpFactory<OpTypes::kMatMul, aops::MatMulOpOptions> {
 public:
  std::shared_ptr<BaseOp> createOpImpl(const aops::MatMulOpOptions& options) override { return std::make_shared<HipMatMulOp>(options); }
};

// ---- the operators around Linear (kernels: mllm_hip_rmsnorm, mllm_hip_silu, mllm_hip_add / _mul, mllm_hip_softmax, mllm_hip_topk)
#define MLLM_HIP_SIMPLE_OP(Name, Base, Options, Type)                                                                     \
  class Name final : public aops::Base {                                                                                   \
   public:                                                                                                                 \
    explicit Name(const aops::Options& options) : aops::Base(options) {}                                                   \
    void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;                                \
  };                                                                                                                       \
  class Name##Factory final : public TypedOpFactory<OpTypes::Type, aops::Options> {                                        \
   public:                                                                                                                 \
    std::shared_ptr<BaseOp> createOpImpl(const aops::Options& options) override { return std::make_shared<Name>(options); } \
  };
MLLM_HIP_SIMPLE_OP(HipSiLUOp, SiLUOp, SiLUOpOptions, kSiLU)
MLLM_HIP_SIMPLE_OP(HipAddOp, AddOp, AddOpOptions, kAdd)
MLLM_HIP_SIMPLE_OP(HipMulOp, MulOp, MulOpOptions, kMul)
MLLM_HIP_SIMPLE_OP(HipSoftmaxOp, SoftmaxOp, SoftmaxOpOptions, kSoftmax)
MLLM_HIP_SIMPLE_OP(HipTopKOp, TopKOp, TopKOpOptions, kTopK)
#undef MLLM_HIP_SIMPLE_OP

class HipRMSNormOp final : public aops::RMSNormOp {
 public:
  explicit HipRMSNormOp(const aops::RMSNormOpOptions& options) : aops::RMSNormOp(options) {}
  void load(const ParameterFile::ptr_t& ploader) override;  // weight -> fp32 on the device
  void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
};
class HipRMSNormOpFactory final : public TypedOpFactory<OpTypes::kRMSNorm, aops::RMSNormOpOptions> {
 public:
  std::shared_ptr<BaseOp> createOpImpl(const aops::RMSNormOpOptions& options) override { return std::make_shared<HipRMSNormOp>(options); }
};

class HipX2XOp final : public aops::X2XOp {
 public:
  explicit HipX2XOp(const aops::X2XOpOptions& options) : aops::X2XOp(options) {}
  void forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) override;
};
class HipX2XOpFactory final : public TypedOpFactory<OpTypes::kX2X, aops::X2XOpOptions> {
 public:
  std::shared_ptr<BaseOp> createOpImpl(const aops::X2XOpOptions& options) override { return std::make_shared<HipX2XOp>(options); }
};

}  // namespace mllm::hip

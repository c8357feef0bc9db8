#include "HipBackend.hpp"

#include <hip/hip_runtime_api.h>

#include <cstring>

#include "mllm_hip_qlinear.h"

namespace mllm::hip {

#define MLLM_HIP_CHECK(expr)                                                                              \
  do {                                                                                                    \
    hipError_t e__ = (expr);                                                                              \
    if (e__ != hipSuccess) MLLM_ERROR_EXIT(ExitCode::kHIPError, "%s failed: %s", #expr, hipGetErrorString(e__)); \
  } while (0)
// kernels report through return codes; the op turns a failure into the runtime's fatal path
#define MLLM_HIP_KERNEL_CHECK(expr)                                                                     \
  do {                                                                                                  \
    int rc__ = (expr);                                                                                  \
    if (rc__ != 0) MLLM_ERROR_EXIT(ExitCode::kHIPError, "%s failed with code %d", #expr, rc__);          \
  } while (0)

// ---- allocator ------------------------------------------------------------------------------------------------
bool HipAllocator::alloc(Storage* storage) {
  void* p = nullptr;
  if (hipMalloc(&p, storage->size_ ? storage->size_ : 256) != hipSuccess) return false;
  storage->ptr_ = p;
  live_[static_cast<const char*>(p)] = storage->size_ ? storage->size_ : 256;
  return true;
}
bool HipAllocator::owns(const void* ptr, size_t bytes) const {
  const char* p = static_cast<const char*>(ptr);
  auto it = live_.upper_bound(p);
  if (it == live_.begin()) return false;
  --it;
  return p >= it->first && p + bytes <= it->first + it->second;
}
void HipAllocator::free(Storage* storage) {
  if (storage->ptr_ && owner) owner->noteWrite(storage->ptr_, storage->size_);
  if (storage->ptr_) {
    live_.erase(static_cast<const char*>(storage->ptr_));
    (void)hipFree(storage->ptr_);  // (waits for the device: nothing uses the memory any more)
    // the memory may have been a decode-GEMV workspace: its address gives the block of arrival counters back
    (void)mllm_hip_gemv_workspace_release(storage->ptr_);
  }
  storage->ptr_ = nullptr;
}
bool HipAllocator::generalAlloc(void** ptr, size_t cap, size_t) { return hipMalloc(ptr, cap) == hipSuccess; }
void HipAllocator::generalFree(void* ptr) { (void)hipFree(ptr); }
size_t HipAllocator::allocSize(Storage* storage) { return (storage->size_ + 255) / 256 * 256; }

// ---- backend ---------------------------------------------------------------------------------------------------
HipBackend::HipBackend(const HipBackendConfig& cfg) : Backend(kHIP, std::make_shared<HipAllocator>()), cfg_(cfg) {
  MLLM_HIP_CHECK(hipSetDevice(cfg_.device));
  MLLM_HIP_KERNEL_CHECK(mllm_hip_init(cfg_.device));
  hipStream_t st;
  MLLM_HIP_CHECK(hipStreamCreate(&st));
  stream_ = st;
  std::static_pointer_cast<HipAllocator>(allocator_)->owner = this;
  regOpFactory<HipLinearOpFactory, HipMatMulOpFactory, HipX2XOpFactory, HipRMSNormOpFactory, HipSiLUOpFactory, HipAddOpFactory,
               HipMulOpFactory, HipSoftmaxOpFactory, HipTopKOpFactory>();
}
HipBackend::~HipBackend() {
  std::static_pointer_cast<HipAllocator>(allocator_)->owner = nullptr;
  images_.clear();
  image_pool_.clear();
  if (stream_) (void)hipStreamDestroy((hipStream_t)stream_);
}
void HipBackend::synchronize() const { MLLM_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream_)); }

void* HipBackend::newImage(const void* tensor_ptr, size_t tensor_bytes, int rows, int64_t D) {
  if (!cfg_.fold_images || rows < 1 || rows > 8 || D % 32) return nullptr;
  // only for memory whose every free this backend sees; an external buffer could be reused behind its back
  if (!std::static_pointer_cast<HipAllocator>(allocator_)->owns(tensor_ptr, tensor_bytes)) return nullptr;
  if (images_.size() >= kMaxImages) {  // oldest first; its buffer goes back to the pool like any dropped image
    if (image_pool_.size() < 16) image_pool_.push_back(images_.front().data);
    images_.erase(images_.begin());
  }
  const size_t need = mllm_hip_gemv_workspace_bytes(rows, D);
  Tensor buf;
  for (size_t i = 0; i < image_pool_.size(); i++)
    if (image_pool_[i].bytes() >= need) {
      buf = image_pool_[i];
      image_pool_.erase(image_pool_.begin() + (long)i);
      break;
    }
  if (buf.isNil()) buf = Tensor::empty({(int32_t)need}, kByte, kHIP).alloc();
  images_.push_back(Image{tensor_ptr, tensor_bytes, rows, D, buf});
  return buf.ptr<void>();
}
const void* HipBackend::findImage(const void* tensor_ptr, int rows, int64_t D) const {
  for (const auto& im : images_)
    if (im.tensor_ptr == tensor_ptr && im.rows == rows && im.D == D) return im.data.ptr<void>();
  return nullptr;
}
void HipBackend::noteWrite(const void* ptr, size_t bytes) {
  const char* lo = static_cast<const char*>(ptr);
  const char* hi = lo + bytes;
  std::vector<Tensor> dropped;  // released after the loop: freeing a buffer calls back into this function
  for (size_t i = 0; i < images_.size();) {
    const char* tl = static_cast<const char*>(images_[i].tensor_ptr);
    if (tl < hi && lo < tl + images_[i].tensor_bytes) {
      dropped.push_back(images_[i].data);
      images_.erase(images_.begin() + (long)i);
    } else {
      i++;
    }
  }
  // a dropped buffer may still be read by a GEMV queued on the stream; kernels that reuse it are queued behind that one
  for (auto& t : dropped)
    if (image_pool_.size() < 16) image_pool_.push_back(t);
}

std::shared_ptr<HipBackend> initHipBackend() {
  auto& ctx = Context::instance();
  if (ctx.hasBackend(kHIP)) return std::static_pointer_cast<HipBackend>(ctx.getBackend(kHIP));
  HipBackendConfig cfg;
  if (const char* m = std::getenv("MLLM_HIP_SCALE_MODE")) {
    if (std::strcmp(m, "x86") == 0) cfg.weight_scale_mode = cfg.act_scale_mode = MLLM_HIP_SCALE_X86_REF;
  }
  if (const char* m = std::getenv("MLLM_HIP_PREFILL")) cfg.prefill_matrix_cores = std::strcmp(m, "blockdot") != 0;
  if (const char* m = std::getenv("MLLM_HIP_FOLD_IMAGES")) cfg.fold_images = std::strcmp(m, "1") == 0;
  auto backend = std::make_shared<HipBackend>(cfg);
  ctx.registerBackend(backend);
  ctx.memoryManager()->registerAllocator(kHIP, backend->allocator());
  return backend;
}

static HipBackend& backend() { return *std::static_pointer_cast<HipBackend>(Context::instance().getBackend(kHIP)); }

// ---- X2X -------------------------------------------------------------------------------------------------------
void HipX2XOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  MLLM_RT_ASSERT_EQ(inputs.size(), 1u);
  MLLM_RT_ASSERT_EQ(outputs.size(), 1u);
  const auto& in = inputs[0];
  auto& out = outputs[0];
  const size_t n = in.bytes();
  auto st = (hipStream_t)backend().stream();
  if (out.device() == kHIP) backend().noteWrite(out.ptr<void>(), out.bytes());
  if (in.device() == kCPU && out.device() == kHIP) {
    MLLM_HIP_CHECK(hipMemcpyAsync(out.ptr<void>(), in.ptr<void>(), n, hipMemcpyHostToDevice, st));
    MLLM_HIP_CHECK(hipStreamSynchronize(st));  // the host buffer may be released by the caller right after
  } else if (in.device() == kHIP && out.device() == kCPU) {
    MLLM_HIP_CHECK(hipStreamSynchronize(st));  // everything queued on the device is finished before the copy back
    MLLM_HIP_CHECK(hipMemcpy(out.ptr<void>(), in.ptr<void>(), n, hipMemcpyDeviceToHost));
  } else if (in.device() == kHIP && out.device() == kHIP) {
    if (in.ptr<void>() != out.ptr<void>()) MLLM_HIP_CHECK(hipMemcpyAsync(out.ptr<void>(), in.ptr<void>(), n, hipMemcpyDeviceToDevice, st));
  } else {
    NYI("X2X between devices %d and %d", (int)in.device(), (int)out.device());
  }
}

// ---- MatMul -----------------------------------------------------------------------------------------------------
void HipMatMulOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  const auto& a = inputs[0];
  const auto& b = inputs[1];
  auto& c = outputs[0];
  int dtype;
  switch (a.dtype()) {
    case kFloat32: dtype = MLLM_HIP_F32; break;
    case kFloat16: dtype = MLLM_HIP_F16; break;
    case kBFloat16: dtype = MLLM_HIP_BF16; break;
    default: NYI("HipMatMulOp takes fp32, fp16 or bf16 operands"); return;
  }
  if (b.dtype() != a.dtype() || c.dtype() != a.dtype()) NYI("HipMatMulOp: both operands and the output share one element type");
  backend().noteWrite(c.ptr<void>(), c.bytes());
  const auto& cs = c.shape();
  const int64_t M = cs[cs.size() - 2], N = cs[cs.size() - 1];
  const auto& as = a.shape();
  const int64_t K = options_.transpose_a ? as[as.size() - 2] : as[as.size() - 1];
  int64_t batch = 1, b_batch = 1;
  for (size_t i = 0; i + 2 < cs.size(); i++) batch *= cs[i];
  for (size_t i = 0; i + 2 < b.shape().size(); i++) b_batch *= b.shape()[i];
  // the reference wants equal batch counts (mllm/backends/cpu/ops/MatMulOp.cpp:40-44); a single right-hand matrix is
  // additionally taken as shared by every batch entry
  if (b_batch != batch && b_batch != 1) NYI("HipMatMulOp: batch counts of the operands differ");
  // the whole batch is one launch
  MLLM_HIP_KERNEL_CHECK(mllm_hip_matmul_batched(a.ptr<void>(), b.ptr<void>(), c.ptr<void>(), dtype, batch, M, N, K, M * K,
                                                b_batch == batch ? N * K : 0, M * N, options_.transpose_a, options_.transpose_b,
                                                backend().stream()));
}

// ---- Linear ------------------------------------------------------------------------------------------------------
HipLinearOp::HipLinearOp(const aops::LinearOpOptions& options) : aops::LinearOp(options) {}

static Tensor onDevice(const Tensor& t) { return t.device() == kHIP ? t : t.to(kHIP); }

void HipLinearOp::load(const ParameterFile::ptr_t& ploader) {
  aops::LinearOp::load(ploader);  // "<name>.weight" viewed [out, in], "<name>.bias"
  const int64_t N = options_.out_channels, K = options_.in_channels;
  auto& be = backend();
  switch (weight_.dtype()) {  // the weight's dtype selects the path, as the reference's device backends do
    case kGGUF_Q4_0:
    case kGGUF_Q8_0: {
      scheme_ = weight_.dtype() == kGGUF_Q4_0 ? Scheme::kQ4_0 : Scheme::kQ8_0;
      const int wt = scheme_ == Scheme::kQ4_0 ? MLLM_HIP_Q4_0 : MLLM_HIP_Q8_0;
      MLLM_RT_ASSERT_EQ((int64_t)weight_.numel(), N * K);
      const size_t pb = mllm_hip_q_packed_bytes(wt, N, K);
      if (pb == 0) MLLM_ERROR_EXIT(ExitCode::kCoreError, "Linear %s: in_channels %d is not a multiple of 32", getName().c_str(), (int)K);
      Tensor dev_blocks = onDevice(weight_);
      packed_ = Tensor::empty({(int32_t)pb}, kByte, kHIP).alloc();
      MLLM_HIP_KERNEL_CHECK(mllm_hip_q_prepack(wt, dev_blocks.ptr<void>(), be.config().weight_scale_mode, packed_.ptr<void>(), N, K, be.stream()));
      if (be.config().prefill_matrix_cores) {
        gemm_packed_ = Tensor::empty({(int32_t)mllm_hip_q_gemm_packed_bytes(wt, N, K)}, kByte, kHIP).alloc();
        MLLM_HIP_KERNEL_CHECK(mllm_hip_q_gemm_prepack(wt, dev_blocks.ptr<void>(), be.config().weight_scale_mode, gemm_packed_.ptr<void>(), N, K,
                                                      be.stream()));
      }
      be.synchronize();  // dev_blocks is released when it goes out of scope
      if (options_.bias) bias_dev_ = onDevice(bias_);
      break;
    }
    case kGGUF_Q4_K:
    case kGGUF_Q6_K: {
      scheme_ = weight_.dtype() == kGGUF_Q4_K ? Scheme::kQ4_K : Scheme::kQ6_K;
      const int wt = scheme_ == Scheme::kQ4_K ? MLLM_HIP_Q4_K : MLLM_HIP_Q6_K;
      MLLM_RT_ASSERT_EQ((int64_t)weight_.numel(), N * K);
      const size_t pb = mllm_hip_kq_packed_bytes(wt, N, K);
      if (pb == 0) MLLM_ERROR_EXIT(ExitCode::kCoreError, "Linear %s: in_channels %d is not a multiple of 256", getName().c_str(), (int)K);
      Tensor dev_blocks = onDevice(weight_);
      packed_ = Tensor::empty({(int32_t)pb}, kByte, kHIP).alloc();
      MLLM_HIP_KERNEL_CHECK(mllm_hip_kq_prepack(wt, dev_blocks.ptr<void>(), be.config().weight_scale_mode, packed_.ptr<void>(), N, K, be.stream()));
      if (be.config().prefill_matrix_cores) {
        gemm_packed_ = Tensor::empty({(int32_t)mllm_hip_kq_gemm_packed_bytes(wt, N, K)}, kByte, kHIP).alloc();
        MLLM_HIP_KERNEL_CHECK(mllm_hip_kq_gemm_prepack(wt, dev_blocks.ptr<void>(), be.config().weight_scale_mode, gemm_packed_.ptr<void>(), N, K,
                                                       be.stream()));
      }
      be.synchronize();
      if (options_.bias) bias_dev_ = onDevice(bias_);
      break;
    }
    case kInt8: {
      scheme_ = Scheme::kW8A8;
      weight_scale_ = onDevice(ploader->pull(getName() + ".weight.scale"));
      MLLM_RT_ASSERT_EQ(weight_scale_.dtype(), kFloat32);
      MLLM_RT_ASSERT_EQ((int64_t)weight_scale_.numel(), N);
      {  // the load-time repack into matrix-core operand order (the reference re-lays the weight here too)
        Tensor dev_w = onDevice(weight_);
        packed_ = Tensor::empty({(int32_t)mllm_hip_w8a8_packed_bytes(N, K)}, kByte, kHIP).alloc();
        MLLM_HIP_KERNEL_CHECK(mllm_hip_w8a8_prepack(dev_w.ptr<int8_t>(), N, K, packed_.ptr<void>(), be.stream()));
        be.synchronize();
      }
      if (options_.bias) bias_dev_ = onDevice(bias_);
      break;
    }
    case kUInt8:
    case kByte: {
      scheme_ = Scheme::kW4A16;  // two uint4 codes per byte, [N][K/2]
      MLLM_RT_ASSERT_EQ((int64_t)weight_.numel(), N * K / 2);
      weight_scale_ = onDevice(ploader->pull(getName() + ".weight.scale"));
      weight_zp_ = onDevice(ploader->pull(getName() + ".weight.zero_point"));
      MLLM_RT_ASSERT_EQ(weight_scale_.dtype(), kFloat16);
      const int64_t G = (int64_t)weight_scale_.numel() / N;
      MLLM_RT_ASSERT(G > 0 && K % G == 0);
      group_ = (int)(K / G);
      {  // codes, scales and zero-points into one packed blob (awq_marlin.py:366-410 does the Marlin repack at this point)
        Tensor dev_w = onDevice(weight_);
        const size_t pb = mllm_hip_w4a16_packed_bytes(N, K, group_);
        if (pb == 0) MLLM_ERROR_EXIT(ExitCode::kCoreError, "Linear %s: group %d must be a multiple of 64 dividing in_channels", getName().c_str(), group_);
        packed_ = Tensor::empty({(int32_t)pb}, kByte, kHIP).alloc();
        MLLM_HIP_KERNEL_CHECK(mllm_hip_w4a16_prepack(dev_w.ptr<uint8_t>(), weight_scale_.ptr<uint16_t>(), weight_zp_.ptr<uint8_t>(), N, K, group_,
                                                     packed_.ptr<void>(), be.stream()));
        be.synchronize();
      }
      if (options_.bias) {
        MLLM_RT_ASSERT_EQ(bias_.dtype(), kBFloat16);
        bias_dev_ = onDevice(bias_);
      }
      break;
    }
    default: NYI("HipLinearOp: weight dtype %d", (int)weight_.dtype());
  }
}

void HipLinearOp::reshape(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  if (options_.isRedirect()) {
    outputs.emplace_back(inputs[1]);
    return;
  }
  const auto& i = inputs[0];
  auto o_shape = i.shape();
  MLLM_RT_ASSERT_EQ(o_shape[o_shape.size() - 1], options_.in_channels);
  o_shape[o_shape.size() - 1] = options_.out_channels;
  // block-quantized weights produce fp32 like the CPU backend's kGGUF path (mllm/backends/cpu/ops/LinearOp.cpp:357-360)
  const bool blocks = scheme_ == Scheme::kQ4_0 || scheme_ == Scheme::kQ8_0 || scheme_ == Scheme::kQ4_K || scheme_ == Scheme::kQ6_K;
  const DataTypes o_dtype = blocks ? kFloat32 : kBFloat16;
  outputs.emplace_back(Tensor::empty(o_shape, o_dtype, i.device()));
}

void HipLinearOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  const auto& x = inputs[0];
  auto& y = outputs[0];
  MLLM_RT_ASSERT_EQ(x.device(), kHIP);
  const int64_t K = options_.in_channels, N = options_.out_channels;
  const int64_t M = (int64_t)x.numel() / K;  // all leading dimensions are rows
  auto& be = backend();
  void* st = be.stream();
  be.noteWrite(y.ptr<void>(), y.bytes());
  auto xdt = [&]() {
    if (x.dtype() == kFloat32) return MLLM_HIP_F32;
    if (x.dtype() == kBFloat16) return MLLM_HIP_BF16;
    MLLM_ERROR_EXIT(ExitCode::kCoreError, "HipLinearOp: activation dtype %d not supported", (int)x.dtype());
  };
  auto workspace = [&](size_t bytes) {
    if (workspace_.isNil() || workspace_.bytes() < bytes) workspace_ = Tensor::empty({(int32_t)bytes}, kByte, kHIP).alloc();
    return workspace_.ptr<void>();
  };
  const float* bias = bias_dev_.isNil() ? nullptr : bias_dev_.ptr<float>();
  switch (scheme_) {
    case Scheme::kQ4_0:
    case Scheme::kQ8_0: {
      const int wt = scheme_ == Scheme::kQ4_0 ? MLLM_HIP_Q4_0 : MLLM_HIP_Q8_0;
      // decode, and short batches as groups of eight rows over the same weights (the groups share one launch): measured on
      // the Qwen3-4B projections against the short-batch matrix-core entry (gate / down / q / o, us): 16 rows 12.0 / 12.3 /
      // 8.5 / 9.4 against 17.2 / 22.6 / 15.2 / 16.3; 48 rows 25.5 / 26.0 / 12.7 / 14.4 against 24.6 / 27.7 / 18.9 / 19.5;
      // 64 rows 34.3 / 31.8 / 16.3 / 16.8 against 25.1 / 28.3 / 19.7 / 20.5 (a layer's seven projections: a tie).  Against
      // the exact tile kernel: 128 rows 59.9 / 60.1 / 27.6 / 28.9 against 71.5 / 236.5 / 70.7 / 103.3
      if (M <= 48 || (gemm_packed_.isNil() && M <= 128)) {
        const void* image = be.findImage(x.ptr<void>(), (int)M, K);
        mllm_hip_gemv_part part{packed_.ptr<void>(), bias, y.ptr<float>(), N};
        // from three rows on: room for the partial sums of the K slices, which lets the rows run as one launch whose
        // workgroups each quantize (or copy) only their slice of the activations; the library decides
        const size_t ws_bytes = M >= 3 ? mllm_hip_gemv_splitk_workspace_bytes((int)M, K, N) : 0;
        void* ws = ws_bytes ? workspace(ws_bytes) : nullptr;
        if (image) {
          const mllm_hip_gemv_fusion fu{nullptr, ws, ws_bytes};
          MLLM_HIP_KERNEL_CHECK(mllm_hip_linear_q_gemv_fused(wt, 1, &part, ws ? &fu : nullptr, image, MLLM_HIP_Q8_IMAGE, (int)M, K,
                                                             be.config().act_scale_mode, st));
        } else {
          MLLM_HIP_KERNEL_CHECK(mllm_hip_linear_q_gemv_multi_wsn(wt, 1, &part, x.ptr<void>(), xdt(), (int)M, K,
                                                                 be.config().act_scale_mode, ws, ws_bytes, st));
        }
      } else if (!gemm_packed_.isNil()) {
        // (the short-batch entry point cuts K into ranges up to 256 rows and is the plain call beyond)
        void* ws = workspace(mllm_hip_linear_q_gemm_short_workspace_bytes(M, N, K));
        MLLM_HIP_KERNEL_CHECK(mllm_hip_linear_q_gemm_short(wt, gemm_packed_.ptr<void>(), x.ptr<void>(), xdt(), bias, y.ptr<float>(), M, N, K,
                                                           be.config().act_scale_mode, ws, st));
      } else {
        void* ws = workspace(mllm_hip_linear_q_workspace_bytes(M, K));
        MLLM_HIP_KERNEL_CHECK(mllm_hip_linear_q(wt, packed_.ptr<void>(), x.ptr<void>(), xdt(), bias, y.ptr<float>(), M, N, K,
                                                be.config().act_scale_mode, ws, st));
      }
      break;
    }
    case Scheme::kQ4_K:
    case Scheme::kQ6_K: {
      const int wt = scheme_ == Scheme::kQ4_K ? MLLM_HIP_Q4_K : MLLM_HIP_Q6_K;
      if (M > 8 && !gemm_packed_.isNil()) {  // prefill: matrix cores
        void* ws = workspace(mllm_hip_linear_kq_gemm_short_workspace_bytes(M, N, K));
        MLLM_HIP_KERNEL_CHECK(mllm_hip_linear_kq_gemm_short(wt, gemm_packed_.ptr<void>(), x.ptr<void>(), xdt(), bias, y.ptr<float>(), M, N, K, ws, st));
      } else {
        // (from three rows on: room for the quantized image of x and for the partial sums of K slices that meet in memory)
        const size_t ws_bytes = M >= 3 ? mllm_hip_kq_workspace_bytes_n(M, K, N) : 0;
        const mllm_hip_gemv_part part{packed_.ptr<void>(), bias, y.ptr<float>(), N};
        MLLM_HIP_KERNEL_CHECK(mllm_hip_linear_kq_multi_ws(wt, 1, &part, x.ptr<void>(), xdt(), M, K, ws_bytes ? workspace(ws_bytes) : nullptr,
                                                          ws_bytes, st));
      }
      break;
    }
    case Scheme::kW8A8: {
      void* ws = workspace(mllm_hip_w8a8_workspace_bytes(M, K));
      MLLM_HIP_KERNEL_CHECK(mllm_hip_w8a8_linear_packed(x.ptr<void>(), xdt(), packed_.ptr<void>(), weight_scale_.ptr<float>(), bias, y.ptr<void>(),
                                                        M, N, K, ws, st));
      break;
    }
    case Scheme::kW4A16: {
      MLLM_RT_ASSERT_EQ(x.dtype(), kBFloat16);
      MLLM_HIP_KERNEL_CHECK(mllm_hip_w4a16_gemm_packed(x.ptr<void>(), packed_.ptr<void>(), bias_dev_.isNil() ? nullptr : bias_dev_.ptr<void>(),
                                                       y.ptr<void>(), M, N, K, group_, st));
      break;
    }
    default: MLLM_ERROR_EXIT(ExitCode::kCoreError, "HipLinearOp::forward before load()");
  }
}

// ---- the operators around Linear -----------------------------------------------------------------------------------
static int actType(const Tensor& t, const char* who) {
  if (t.dtype() == kFloat32) return MLLM_HIP_F32;
  if (t.dtype() == kBFloat16) return MLLM_HIP_BF16;
  MLLM_ERROR_EXIT(ExitCode::kCoreError, "%s: dtype %d not supported (fp32 or bf16)", who, (int)t.dtype());
}
static void rowsAndWidth(const Tensor& t, int64_t& rows, int64_t& D) {
  D = t.shape().back();
  rows = (int64_t)t.numel() / D;
}

void HipRMSNormOp::load(const ParameterFile::ptr_t& ploader) {
  aops::RMSNormOp::load(ploader);
  if (weight_.dtype() != kFloat32) NYI("HipRMSNormOp: weight must be fp32 (as in the reference's x86 kernel)");
  weight_ = onDevice(weight_);
}
void HipRMSNormOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  const auto& x = inputs[0];
  auto& y = outputs[0];
  auto& be = backend();
  int64_t rows, D;
  rowsAndWidth(x, rows, D);
  MLLM_RT_ASSERT_EQ((int64_t)weight_.numel(), D);
  be.noteWrite(y.ptr<void>(), y.bytes());
  void* image = be.newImage(y.ptr<void>(), y.bytes(), (int)std::min<int64_t>(rows, 9), D);
  MLLM_HIP_KERNEL_CHECK(mllm_hip_rmsnorm(x.ptr<void>(), actType(x, "HipRMSNormOp"), weight_.ptr<float>(), y.ptr<void>(), rows, D,
                                         options_.epsilon, options_.add_unit_offset, image, be.config().act_scale_mode, be.stream()));
}
void HipSiLUOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  auto& be = backend();
  be.noteWrite(outputs[0].ptr<void>(), outputs[0].bytes());
  MLLM_HIP_KERNEL_CHECK(mllm_hip_silu(inputs[0].ptr<void>(), outputs[0].ptr<void>(), actType(inputs[0], "HipSiLUOp"),
                                      (int64_t)inputs[0].numel(), be.stream()));
}
template <typename Fn>
static void binaryForward(const char* who, Fn fn, const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs, bool want_image) {
  const auto& a = inputs[0];
  const auto& b = inputs[1];
  auto& y = outputs[0];
  if (a.shape() != b.shape() || a.dtype() != b.dtype()) NYI("%s: operands must have the same shape and type (no broadcasting)", who);
  auto& be = backend();
  int64_t rows, D;
  rowsAndWidth(a, rows, D);
  be.noteWrite(y.ptr<void>(), y.bytes());
  void* image = want_image ? be.newImage(y.ptr<void>(), y.bytes(), (int)std::min<int64_t>(rows, 9), D) : nullptr;
  MLLM_HIP_KERNEL_CHECK(fn(a.ptr<void>(), b.ptr<void>(), y.ptr<void>(), actType(a, who), rows, D, image, be.config().act_scale_mode,
                           be.stream()));
}
// the residual sum feeds the next RMSNorm, not a Linear: no image
void HipAddOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  binaryForward("HipAddOp", mllm_hip_add, inputs, outputs, false);
}
// silu(gate) * up feeds down_proj
void HipMulOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  binaryForward("HipMulOp", mllm_hip_mul, inputs, outputs, true);
}
void HipSoftmaxOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  const auto& x = inputs[0];
  const int axis = options_.axis < 0 ? options_.axis + (int)x.rank() : options_.axis;
  if (axis != (int)x.rank() - 1 || x.dtype() != kFloat32) NYI("HipSoftmaxOp: fp32 over the last axis only");
  auto& be = backend();
  int64_t rows, len;
  rowsAndWidth(x, rows, len);
  be.noteWrite(outputs[0].ptr<void>(), outputs[0].bytes());
  MLLM_HIP_KERNEL_CHECK(mllm_hip_softmax(x.ptr<float>(), outputs[0].ptr<float>(), rows, len, be.stream()));
}
void HipTopKOp::forward(const std::vector<Tensor>& inputs, std::vector<Tensor>& outputs) {
  const auto& x = inputs[0];
  const int dim = options_.dim < 0 ? options_.dim + (int)x.rank() : options_.dim;
  if (dim != (int)x.rank() - 1 || x.dtype() != kFloat32) NYI("HipTopKOp: fp32 over the last axis only");
  auto& be = backend();
  int64_t rows, len;
  rowsAndWidth(x, rows, len);
  be.noteWrite(outputs[0].ptr<void>(), outputs[0].bytes());
  be.noteWrite(outputs[1].ptr<void>(), outputs[1].bytes());
  MLLM_HIP_KERNEL_CHECK(mllm_hip_topk(x.ptr<float>(), outputs[0].ptr<float>(), outputs[1].ptr<int32_t>(), rows, len, options_.k,
                                      options_.largest, options_.sorted, be.stream()));
}

ParameterFile::ptr_t HipLinearOp::getParams() {
  auto p = aops::LinearOp::getParams();
  if (!weight_scale_.isNil()) p->push(getName() + ".weight.scale", weight_scale_);
  if (!weight_zp_.isNil()) p->push(getName() + ".weight.zero_point", weight_zp_);
  return p;
}

}  // namespace mllm::hip

// ---- out-of-tree route: the plugin C ABI (adds the ops under names; it cannot replace kLinear, see PluginSystem.cpp:82-90)
extern "C" {
static void* createHipLinearFactory() { return new mllm::hip::HipLinearOpFactory(); }
static void freeHipLinearFactory(void* f) { delete static_cast<mllm::hip::HipLinearOpFactory*>(f); }
static void* createHipMatMulFactory() { return new mllm::hip::HipMatMulOpFactory(); }
static void freeHipMatMulFactory(void* f) { delete static_cast<mllm::hip::HipMatMulOpFactory*>(f); }

__attribute__((visibility("default"))) void* opPackageDescriptor() {
  auto* pkg = new PluginOpPackageDescriptor();
  std::snprintf(pkg->name, sizeof(pkg->name), "MllmHipQLinear");
  pkg->device_type = (int32_t)mllm::kHIP;
  pkg->op_factories_count = 2;
  std::snprintf(pkg->op_factories_names[0], MLLM_PLUGIN_OP_PACKAGE_NAME_LEN, "hip_linear");
  std::snprintf(pkg->op_factories_names[1], MLLM_PLUGIN_OP_PACKAGE_NAME_LEN, "hip_matmul");
  pkg->op_factory_create_funcs[0] = createHipLinearFactory;
  pkg->op_factory_create_funcs[1] = createHipMatMulFactory;
  pkg->op_factory_free_funcs[0] = freeHipLinearFactory;
  pkg->op_factory_free_funcs[1] = freeHipMatMulFactory;
  return pkg;
}
}

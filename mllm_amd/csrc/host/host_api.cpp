// A plain-C doorway into the C++ backend for callers (and tests) that cannot include the C++ headers: runs one Linear
// through exactly the sequence mllm's runtime uses for a device op,
//   initializeContext + initHipBackend -> Backend::createOp(kLinear, LinearOpOptions) -> load(ParameterFile)
//   -> Tensor::to(kHIP) (X2X) -> reshape -> setup -> forward -> Tensor::to(kCPU)
// (mllm/nn/Layer.cpp:13-34,53-82, mllm/backends/cpu/CPUDispatcher.cpp:56-62).
#include <hip/hip_runtime_api.h>

#include <cstring>
#include <string>

#include "HipBackend.hpp"
#include "mllm_hip_qlinear.h"

using namespace mllm;

namespace {
DataTypes weight_dtype(const std::string& scheme) {
  if (scheme == "q4_0") return kGGUF_Q4_0;
  if (scheme == "q8_0") return kGGUF_Q8_0;
  if (scheme == "q4_k") return kGGUF_Q4_K;
  if (scheme == "q6_k") return kGGUF_Q6_K;
  if (scheme == "w8a8") return kInt8;
  if (scheme == "w4a16") return kUInt8;
  MLLM_ERROR_EXIT(ExitCode::kCoreError, "unknown scheme '%s'", scheme.c_str());
}
}  // namespace

extern "C" __attribute__((visibility("default"))) int mllm_hip_backend_run_linear(
    const char* scheme_c, const void* weight_host, const void* scale_host, const void* zp_host, const void* bias_host,
    const void* x_host, int x_is_bf16, void* y_host, int M, int N, int K, int group, int weight_scale_x86, int act_scale_x86, int via_plugin,
    const char* plugin_path) {
  const std::string scheme(scheme_c);
  initializeContext();
  auto be = hip::initHipBackend();
  be->setScaleModes(weight_scale_x86 ? MLLM_HIP_SCALE_X86_REF : MLLM_HIP_SCALE_IEEE,
                    act_scale_x86 ? MLLM_HIP_SCALE_X86_REF : MLLM_HIP_SCALE_IEEE);
  auto& ctx = Context::instance();

  // a parameter file holding host tensors that borrow the caller's memory
  auto params = ParameterFile::create(ModelFileVersion::kV2);
  const std::string name = "model.layers.0.proj";
  const DataTypes wdt = weight_dtype(scheme);
  if (wdt == kUInt8)
    params->push(name + ".weight", Tensor::fromExternal(const_cast<void*>(weight_host), {N, K / 2}, kUInt8, kCPU));
  else
    params->push(name + ".weight", Tensor::fromExternal(const_cast<void*>(weight_host), {N, K}, wdt, kCPU));
  if (scheme == "w8a8") params->push(name + ".weight.scale", Tensor::fromExternal(const_cast<void*>(scale_host), {N}, kFloat32, kCPU));
  if (scheme == "w4a16") {
    const int G = K / group;
    params->push(name + ".weight.scale", Tensor::fromExternal(const_cast<void*>(scale_host), {N, G}, kFloat16, kCPU));
    params->push(name + ".weight.zero_point", Tensor::fromExternal(const_cast<void*>(zp_host), {N, (G + 1) / 2}, kUInt8, kCPU));
  }
  if (bias_host)
    params->push(name + ".bias", Tensor::fromExternal(const_cast<void*>(bias_host), {N}, scheme == "w4a16" ? kBFloat16 : kFloat32, kCPU));

  aops::LinearOpOptions opts;
  opts.in_channels = K;
  opts.out_channels = N;
  opts.bias = bias_host != nullptr;
  opts.impl_type = aops::LinearImplTypes::kDefault;

  BaseOp::ptr_t op;
  if (via_plugin) {
    // out-of-tree route: the op package is looked up by name after dlopen (tests/plugin/HostTest.cpp:5-12 in the reference)
    static bool loaded = false;
    if (!loaded) {
      loadOpPackage(plugin_path);
      loaded = true;
    }
    op = ctx.getBackend(kHIP)->createOp((OpTypes)ctx.lookupCustomizedOpId(kHIP, "hip_linear"), opts);
  } else {
    op = ctx.getBackend(kHIP)->createOp(OpTypes::kLinear, opts);
  }
  op->setName(name);
  op->load(params);

  Tensor x = Tensor::fromExternal(const_cast<void*>(x_host), {1, M, K}, x_is_bf16 ? kBFloat16 : kFloat32, kCPU).to(kHIP);
  std::vector<Tensor> inputs{x}, outputs;
  op->reshape(inputs, outputs);
  op->setup(inputs, outputs);
  op->forward(inputs, outputs);
  Tensor y = outputs[0].to(kCPU);
  if ((int)y.shape().size() != 3 || y.shape()[1] != M || y.shape()[2] != N) return -10;
  std::memcpy(y_host, y.ptr<void>(), y.bytes());
  // getParams() must hand back every tensor load() needs
  auto back = op->getParams();
  if (!back->has(name + ".weight")) return -11;
  if ((scheme == "w8a8" || scheme == "w4a16") && !back->has(name + ".weight.scale")) return -12;
  return (int)y.dtype();
}

// ---- model files ---------------------------------------------------------------------------------------------------
// One tensor of a model file: dtype, shape (rank entries) and, when `data` is given, its bytes.  Returns the byte count,
// -1 if the name is missing.  Host only: touches no GPU.
extern "C" __attribute__((visibility("default"))) int64_t mllm_hip_host_file_tensor(const char* path, int version, const char* name,
                                                                                    int32_t* dtype, int32_t* rank, int32_t* shape,
                                                                                    void* data, uint64_t capacity) {
  initializeContext();
  auto pf = load(path, static_cast<ModelFileVersion>(version));
  if (!pf->has(name)) return -1;
  Tensor t = pf->pull(name);
  *dtype = (int32_t)t.dtype();
  *rank = (int32_t)t.shape().size();
  for (size_t i = 0; i < t.shape().size(); i++) shape[i] = t.shape()[i];
  if (data) {
    if (capacity < t.bytes()) return -2;
    std::memcpy(data, t.ptr<void>(), t.bytes());
  }
  return (int64_t)t.bytes();
}
// The two ways of reading a model file: 1 when, read with mmap = true, the tensor is a view into the file's mapping (nothing
// copied) AND holds the same bytes as the copy that mmap = false reads; 0 otherwise, -1 if the name is missing.
extern "C" __attribute__((visibility("default"))) int mllm_hip_host_file_tensor_is_mapped_view(const char* path, int version,
                                                                                               const char* name) {
  initializeContext();
  auto mapped = load(path, static_cast<ModelFileVersion>(version), kCPU, true);
  auto copied = load(path, static_cast<ModelFileVersion>(version), kCPU, false);
  if (!mapped->has(name) || !copied->has(name)) return -1;
  Tensor a = mapped->pull(name), b = copied->pull(name);
  const auto& mf = mapped->getMappedFile();
  if (!mf || copied->getMappedFile()) return 0;
  const char* p = a.ptr<char>();
  const char* base = static_cast<const char*>(mf->data());
  const bool inside = p >= base && p + a.bytes() <= base + mf->size();
  const bool outside = !(b.ptr<char>() >= base && b.ptr<char>() < base + mf->size());
  return inside && outside && a.bytes() == b.bytes() && std::memcmp(p, b.ptr<void>(), a.bytes()) == 0 ? 1 : 0;
}
// read in one version, write in another; returns the tensor count
extern "C" __attribute__((visibility("default"))) int mllm_hip_host_file_convert(const char* in_path, int in_version, const char* out_path,
                                                                                 int out_version) {
  initializeContext();
  auto pf = load(in_path, static_cast<ModelFileVersion>(in_version));
  save(out_path, pf, static_cast<ModelFileVersion>(out_version));
  return (int)pf->dict().size();
}
// A Linear layer straight from a model file: mllm::load -> createOp(kLinear) -> load(params) -> forward.  V1 files carry
// flat shapes; LinearOp::load views the weight as [out, in] as the reference does.
extern "C" __attribute__((visibility("default"))) int mllm_hip_backend_run_linear_file(const char* path, int version, const char* layer,
                                                                                       int in_channels, int out_channels, int has_bias,
                                                                                       const void* x_host, int x_is_bf16, void* y_host, int M,
                                                                                       int weight_scale_x86, int act_scale_x86) {
  initializeContext();
  auto be = hip::initHipBackend();
  be->setScaleModes(weight_scale_x86 ? MLLM_HIP_SCALE_X86_REF : MLLM_HIP_SCALE_IEEE,
                    act_scale_x86 ? MLLM_HIP_SCALE_X86_REF : MLLM_HIP_SCALE_IEEE);
  auto params = load(path, static_cast<ModelFileVersion>(version));
  aops::LinearOpOptions opts;
  opts.in_channels = in_channels;
  opts.out_channels = out_channels;
  opts.bias = has_bias != 0;
  opts.impl_type = aops::LinearImplTypes::kDefault;
  auto op = Context::instance().getBackend(kHIP)->createOp(OpTypes::kLinear, opts);
  op->setName(layer);
  op->load(params);
  Tensor x = Tensor::fromExternal(const_cast<void*>(x_host), {1, M, in_channels}, x_is_bf16 ? kBFloat16 : kFloat32, kCPU).to(kHIP);
  std::vector<Tensor> inputs{x}, outputs;
  op->reshape(inputs, outputs);
  op->setup(inputs, outputs);
  op->forward(inputs, outputs);
  Tensor y = outputs[0].to(kCPU);
  std::memcpy(y_host, y.ptr<void>(), y.bytes());
  return (int)y.dtype();
}

// The MLP half of a decoder layer through the op factories, operator by operator as the reference's modules call them
// (mllm/models/qwen3/modeling_qwen3_fa2.hpp:85-92 inside Qwen3Decoder::forward): h = rms_norm(x); g = gate(h); u = up(h);
// a = silu(g) * u; y = x + down(a).  Returns how many Linear inputs were handed over as quantized images (0 when
// fold_images is off); softmax / top-k run on g as a side check of those two slots (values to sm_host / tk_* when given).
extern "C" __attribute__((visibility("default"))) int mllm_hip_backend_run_decoder_mlp(
    int is_q8, const void* Wg, const void* Wu, const void* Wd, const float* norm_w, const void* x_host, int x_is_bf16, void* y_host,
    int M, int H, int I, float eps, int fold_images, float* softmax_host, int32_t* topk_idx_host, int topk) {
  initializeContext();
  auto be = hip::initHipBackend();
  be->setScaleModes(MLLM_HIP_SCALE_IEEE, MLLM_HIP_SCALE_X86_REF);
  be->setFoldImages(fold_images != 0);
  auto backend = Context::instance().getBackend(kHIP);
  const DataTypes wdt = is_q8 ? kGGUF_Q8_0 : kGGUF_Q4_0;
  auto params = ParameterFile::create(ModelFileVersion::kV2);
  params->push("l.norm.weight", Tensor::fromExternal(const_cast<float*>(norm_w), {H}, kFloat32, kCPU));
  params->push("l.gate.weight", Tensor::fromExternal(const_cast<void*>(Wg), {I, H}, wdt, kCPU));
  params->push("l.up.weight", Tensor::fromExternal(const_cast<void*>(Wu), {I, H}, wdt, kCPU));
  params->push("l.down.weight", Tensor::fromExternal(const_cast<void*>(Wd), {H, I}, wdt, kCPU));
  auto make = [&](OpTypes t, const BaseOpOptionsBase& o, const std::string& name) {
    auto op = backend->createOp(t, o);
    op->setName(name);
    op->load(params);
    return op;
  };
  auto run = [&](const BaseOp::ptr_t& op, const std::vector<Tensor>& in) {
    std::vector<Tensor> out;
    op->reshape(in, out);
    op->setup(in, out);
    op->forward(in, out);
    return out;
  };
  aops::RMSNormOpOptions no;
  no.epsilon = eps;
  aops::LinearOpOptions gu, dn;
  gu.in_channels = H;
  gu.out_channels = I;
  dn.in_channels = I;
  dn.out_channels = H;
  auto norm = make(OpTypes::kRMSNorm, no, "l.norm");
  auto gate = make(OpTypes::kLinear, gu, "l.gate");
  auto up = make(OpTypes::kLinear, gu, "l.up");
  auto down = make(OpTypes::kLinear, dn, "l.down");
  auto silu = make(OpTypes::kSiLU, aops::SiLUOpOptions{}, "l.act");
  auto mul = make(OpTypes::kMul, aops::MulOpOptions{}, "l.mul");
  auto add = make(OpTypes::kAdd, aops::AddOpOptions{}, "l.add");

  Tensor x = Tensor::fromExternal(const_cast<void*>(x_host), {M, H}, x_is_bf16 ? kBFloat16 : kFloat32, kCPU).to(kHIP);
  int handed_over = 0;
  Tensor h = run(norm, {x})[0];
  handed_over += be->findImage(h.ptr<void>(), M, H) != nullptr;
  Tensor g = run(gate, {h})[0];
  handed_over += be->findImage(h.ptr<void>(), M, H) != nullptr;  // still there for the sibling projection
  Tensor u = run(up, {h})[0];
  Tensor s = run(silu, {g})[0];
  Tensor a = run(mul, {s, u})[0];
  handed_over += be->findImage(a.ptr<void>(), M, I) != nullptr;
  Tensor d = run(down, {a})[0];
  // Linear yields fp32; the residual stream of this harness is fp32 whenever x is
  Tensor y = x_is_bf16 ? d : run(add, {d, x})[0];
  Tensor yc = y.to(kCPU);
  std::memcpy(y_host, yc.ptr<void>(), yc.bytes());
  if (softmax_host) {
    aops::SoftmaxOpOptions so;
    so.axis = -1;
    Tensor p = run(make(OpTypes::kSoftmax, so, "l.sm"), {g})[0];
    Tensor pc = p.to(kCPU);
    std::memcpy(softmax_host, pc.ptr<void>(), pc.bytes());
    if (topk_idx_host) {
      aops::TopKOpOptions to;
      to.k = topk;
      to.sorted = false;
      auto vi = run(make(OpTypes::kTopK, to, "l.topk"), {p});
      Tensor ic = vi[1].to(kCPU);
      std::memcpy(topk_idx_host, ic.ptr<void>(), ic.bytes());
    }
  }
  // an op that overwrites a tensor must drop that tensor's image
  std::vector<Tensor> reuse{h};
  norm->forward({x}, reuse);
  const bool refreshed = !fold_images || M > 8 || be->findImage(h.ptr<void>(), M, H) != nullptr;
  std::vector<Tensor> clobber{h};
  silu->forward({h}, clobber);  // writes h in place
  if (be->findImage(h.ptr<void>(), M, H) != nullptr || !refreshed) return -20;
  be->synchronize();
  return handed_over;
}

// A writer the backend cannot see: RMSNorm -> Linear, then the activation tensor is overwritten with a plain hipMemcpy
// (what another backend's op or an integrator's own kernel would do) and the Linear runs again on the same tensor.
// y1_host / y2_host receive the two Linear results; returns the number of images the backend holds for the tensor at the
// second call (with the backend's default configuration that is 0 and the second result follows the new contents),
// or a negative code.  `external` != 0 runs the Linear on a caller-owned device buffer instead of a backend tensor, with
// the hand-over switched on: no image may be made for memory the backend's allocator does not own.
extern "C" __attribute__((visibility("default"))) int mllm_hip_backend_run_rewrite_behind_backend(
    int is_q8, const void* W, const float* norm_w, const float* x_host, const float* h2_host, float* y1_host, float* y2_host, int M,
    int H, int N, int external) {
  initializeContext();
  auto be = hip::initHipBackend();
  be->setScaleModes(MLLM_HIP_SCALE_IEEE, MLLM_HIP_SCALE_X86_REF);
  be->setFoldImages(external != 0 ? true : hip::HipBackendConfig().fold_images);  // the default, whatever ran before
  auto backend = Context::instance().getBackend(kHIP);
  auto params = ParameterFile::create(ModelFileVersion::kV2);
  params->push("l.norm.weight", Tensor::fromExternal(const_cast<float*>(norm_w), {H}, kFloat32, kCPU));
  params->push("l.proj.weight", Tensor::fromExternal(const_cast<void*>(W), {N, H}, is_q8 ? kGGUF_Q8_0 : kGGUF_Q4_0, kCPU));
  aops::RMSNormOpOptions no;
  no.epsilon = 1e-6f;
  aops::LinearOpOptions lo;
  lo.in_channels = H;
  lo.out_channels = N;
  auto norm = backend->createOp(OpTypes::kRMSNorm, no);
  norm->setName("l.norm");
  norm->load(params);
  auto proj = backend->createOp(OpTypes::kLinear, lo);
  proj->setName("l.proj");
  proj->load(params);
  auto run = [&](const BaseOp::ptr_t& op, const std::vector<Tensor>& in, std::vector<Tensor> out = {}) {
    if (out.empty()) {
      op->reshape(in, out);
      op->setup(in, out);
    }
    op->forward(in, out);
    return out;
  };
  Tensor x = Tensor::fromExternal(const_cast<float*>(x_host), {M, H}, kFloat32, kCPU).to(kHIP);
  Tensor h;
  void* ext = nullptr;
  if (external) {
    if (hipMalloc(&ext, (size_t)M * H * 4) != hipSuccess) return -30;
    h = Tensor::fromExternal(ext, {M, H}, kFloat32, kHIP);
    run(norm, {x}, {h});
  } else {
    h = run(norm, {x})[0];
  }
  Tensor y1 = run(proj, {h})[0].to(kCPU);
  std::memcpy(y1_host, y1.ptr<void>(), y1.bytes());
  be->synchronize();
  if (hipMemcpy(h.ptr<void>(), h2_host, (size_t)M * H * 4, hipMemcpyHostToDevice) != hipSuccess) return -31;
  const int images = be->findImage(h.ptr<void>(), M, H) != nullptr;
  Tensor y2 = run(proj, {h})[0].to(kCPU);
  std::memcpy(y2_host, y2.ptr<void>(), y2.bytes());
  be->synchronize();
  be->setFoldImages(hip::HipBackendConfig().fold_images);
  if (ext) (void)hipFree(ext);
  return images;
}

// fp32 MatMul through the kMatMul factory slot
extern "C" __attribute__((visibility("default"))) int mllm_hip_backend_run_matmul(const float* a_host, const float* b_host, float* c_host,
                                                                                  int M, int N, int K, int transpose_b) {
  initializeContext();
  hip::initHipBackend();
  auto& ctx = Context::instance();
  Tensor a = Tensor::fromExternal(const_cast<float*>(a_host), {M, K}, kFloat32, kCPU).to(kHIP);
  Tensor b = Tensor::fromExternal(const_cast<float*>(b_host), transpose_b ? Tensor::shape_t{N, K} : Tensor::shape_t{K, N}, kFloat32, kCPU).to(kHIP);
  aops::MatMulOpOptions o;
  o.transpose_b = transpose_b != 0;
  auto outs = ctx.buildOpAndSubmitTask(OpTypes::kMatMul, o, {a, b});
  Tensor c = outs[0].to(kCPU);
  std::memcpy(c_host, c.ptr<void>(), c.bytes());
  return 0;
}

// batched MatMul of any of the three element types (mllm DataTypes id: 0 fp32, 1 fp16, 128 bf16) through the same slot;
// a is [batch][M][K] ([batch][K][M] transposed), b is [batch][K][N] ([batch][N][K] transposed) or one matrix for all
extern "C" __attribute__((visibility("default"))) int mllm_hip_backend_run_matmul_batched(const void* a_host, const void* b_host,
                                                                                          void* c_host, int dtype, int batch, int M,
                                                                                          int N, int K, int transpose_a,
                                                                                          int transpose_b, int b_batched) {
  initializeContext();
  hip::initHipBackend();
  auto& ctx = Context::instance();
  const DataTypes dt = (DataTypes)dtype;
  Tensor::shape_t sa = transpose_a ? Tensor::shape_t{batch, K, M} : Tensor::shape_t{batch, M, K};
  Tensor::shape_t sb = transpose_b ? Tensor::shape_t{N, K} : Tensor::shape_t{K, N};
  if (b_batched) sb.insert(sb.begin(), batch);
  Tensor a = Tensor::fromExternal(const_cast<void*>(a_host), sa, dt, kCPU).to(kHIP);
  Tensor b = Tensor::fromExternal(const_cast<void*>(b_host), sb, dt, kCPU).to(kHIP);
  aops::MatMulOpOptions o;
  o.transpose_a = transpose_a != 0;
  o.transpose_b = transpose_b != 0;
  auto outs = ctx.buildOpAndSubmitTask(OpTypes::kMatMul, o, {a, b});
  Tensor c = outs[0].to(kCPU);
  std::memcpy(c_host, c.ptr<void>(), c.bytes());
  return 0;
}

// error-path probe for the CPU tests: asks a backend that was never registered for an op (the runtime's behaviour is to
// terminate the process, mllm/engine/Context.cpp:37-42) -- run in a child process.
extern "C" __attribute__((visibility("default"))) int mllm_hip_backend_probe_missing_backend() {
  initializeContext();
  Context::instance().getBackend(kHIP);
  return 0;
}
// type-erased options of the wrong type must throw std::bad_cast (mllm/core/BaseOp.hpp:132-136)
extern "C" __attribute__((visibility("default"))) int mllm_hip_backend_probe_bad_cast() {
  hip::HipLinearOpFactory f;
  try {
    f.create(aops::MatMulOpOptions{});
  } catch (const std::bad_cast&) {
    return 1;
  }
  return 0;
}

// PyTorch operator binding of libwoq_hip.so: the `torch_ipex` forward ops, the `ipex_prepack` ops and
// the TorchScript custom class `__torch__.torch.classes.ipex_prepack.WoqLinearOpContext`, registered
// for tensors that live on the GPU (dispatch key CUDA, which HIP tensors carry under ROCm, plus
// AutocastCUDA), with the schemas of the reference
// (csrc/cpu/aten/Linear.cpp:1013-1112, csrc/cpu/jit/cpu/kernels/RegisterOpContextClass.cpp:127-223).
//
// Host code only: tensors in, device pointers + sizes + the current HIP stream into the C ABI of
// include/woq_hip.h, tensors out.  PyTorch supplies device memory and the stream, nothing else.
#include <ATen/ATen.h>
#include <ATen/autocast_mode.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>
#include <torch/custom_class.h>
#include <torch/library.h>

#include <atomic>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <unordered_map>

#include "../../include/woq_hip.h"

namespace woq_torch {

using at::Tensor;
using c10::optional;

constexpr int64_t kPlainFormat = 0, kGptqFormat = 1, kAwqFormat = 2;

static void check_rc(int rc, const char* what) { TORCH_CHECK(rc == 0, what, ": ", woq_hip_last_error()); }

static int act_code(at::ScalarType t) {
  switch (t) {
    case at::kFloat: return WOQ_HIP_ACT_FP32;
    case at::kHalf: return WOQ_HIP_ACT_FP16;
    case at::kBFloat16: return WOQ_HIP_ACT_BF16;
    default: TORCH_CHECK(false, "woq_linear: unsupported activation dtype ", t);
  }
  return 0;
}

static int64_t weight_dtype_of(c10::string_view name) {
  if (name == "int8") return WOQ_HIP_DTYPE_INT8;
  if (name == "int4") return WOQ_HIP_DTYPE_INT4;
  if (name == "nf4") return WOQ_HIP_DTYPE_NF4;
  if (name == "fp8") return WOQ_HIP_DTYPE_FP8;
  TORCH_CHECK(false, "Unsupported weight dtype: ", name);
  return 0;
}

// The current device while this object lives (plain HIP calls: no guard type of PyTorch is involved).
struct DeviceScope {
  int prev = -1;
  bool switched = false;
  explicit DeviceScope(const Tensor& t) {
    if (hipGetDevice(&prev) == hipSuccess && prev != t.get_device()) {
      switched = hipSetDevice(t.get_device()) == hipSuccess;
    }
  }
  ~DeviceScope() {
    if (switched) (void)hipSetDevice(prev);
  }
};

static void* current_stream(const Tensor& t) {
  return (void*)c10::hip::getCurrentHIPStream((c10::DeviceIndex)t.get_device()).stream();
}

static Tensor to_gpu(const Tensor& t, optional<c10::Device> dev = c10::nullopt) {
  if (t.is_cuda()) return t;
  int count = 0;
  TORCH_CHECK(hipGetDeviceCount(&count) == hipSuccess && count > 0,
              "WOQ linear: no GPU is available; this build runs on MI355X only and has no CPU path");
  if (dev.has_value()) return t.to(*dev);
  int cur = 0;
  (void)hipGetDevice(&cur);
  return t.to(c10::Device(c10::kCUDA, (c10::DeviceIndex)cur));
}

static void require_gpu_input(const Tensor& x, const char* name) {
  TORCH_CHECK(x.is_cuda(), name, ": the input must be on the GPU (got ", x.device(),
              "); there is no CPU implementation in this build");
}

// ---- C ABI wrappers on tensors ---------------------------------------------------------------------
static bool is_8bit(int64_t wd) { return wd == WOQ_HIP_DTYPE_INT8 || wd == WOQ_HIP_DTYPE_FP8; }

static Tensor pack_weight(const Tensor& plain_in, int64_t wd, int64_t N, int64_t K) {
  const Tensor plain = plain_in.contiguous();
  const int64_t tk = is_8bit(wd) ? WOQ_HIP_TILE_K_INT8 : WOQ_HIP_TILE_K_INT4;
  const int64_t nt = woq_hip_padded_n(N) / WOQ_HIP_TILE_N, kt = woq_hip_padded_k((int)wd, K) / tk;
  Tensor packed = at::empty({nt, kt, WOQ_HIP_TILE_BYTES}, plain.options().dtype(at::kByte));
  DeviceScope scope(plain);
  check_rc(woq_hip_pack_weight(plain.data_ptr(), (int)wd, N, K, packed.data_ptr(), current_stream(plain)),
           "pack_weight");
  return packed;
}

static Tensor unpack_weight(const Tensor& packed, int64_t wd, int64_t N, int64_t K) {
  TORCH_CHECK(packed.is_cuda(), "packed weight must live on the GPU");
  Tensor plain = wd == WOQ_HIP_DTYPE_FP8    ? at::empty({N, K}, packed.options().dtype(at::kFloat8_e4m3fn))
                 : wd == WOQ_HIP_DTYPE_INT8 ? at::empty({N, K}, packed.options().dtype(at::kChar))
                                            : at::empty({N, (K + 1) / 2}, packed.options().dtype(at::kByte));
  DeviceScope scope(packed);
  check_rc(woq_hip_unpack_weight(packed.data_ptr(), (int)wd, N, K, plain.data_ptr(), current_stream(packed)),
           "unpack_weight");
  return plain;
}

static Tensor shuffle_int4_weight(const Tensor& plain_in, int64_t N, int64_t K, const Tensor& src) {
  const Tensor plain = plain_in.contiguous();
  Tensor out = at::empty_like(plain);
  DeviceScope scope(plain);
  check_rc(woq_hip_shuffle_int4_weight(plain.data_ptr(), N, K, src.data_ptr<int32_t>(), out.data_ptr(),
                                       current_stream(plain)),
           "shuffle_int4_weight");
  return out;
}

static Tensor shuffle_activations(const Tensor& x, const Tensor& src) {
  const int64_t K = x.size(-1);
  const Tensor x2 = x.reshape({-1, K}).contiguous();
  Tensor out = at::empty_like(x2);
  DeviceScope scope(x2);
  check_rc(woq_hip_shuffle_activations(x2.data_ptr(), act_code(x.scalar_type()), x2.size(0), K,
                                       src.data_ptr<int32_t>(), out.data_ptr(), current_stream(x2)),
           "shuffle_activations");
  return out.reshape(x.sizes());
}

static Tensor dequant_weight(const Tensor& packed, int64_t wd, int64_t N, int64_t K, const Tensor& s32,
                             const optional<Tensor>& z8, int64_t G, at::ScalarType dtype) {
  Tensor out = at::empty({N, K}, packed.options().dtype(dtype));
  DeviceScope scope(packed);
  check_rc(woq_hip_dequant_weight(packed.data_ptr(), (int)wd, N, K, s32.data_ptr<float>(),
                                  z8.has_value() ? z8->data_ptr<uint8_t>() : nullptr, G, out.data_ptr(),
                                  act_code(dtype), current_stream(packed)),
           "dequant_weight");
  return out;
}

struct PackedQParams {
  Tensor s32, s16, sb16;
  optional<Tensor> z8, sz, szb;
};

static PackedQParams pack_qparams(const Tensor& scales_in, const optional<Tensor>& zeros_in, int64_t wd) {
  const Tensor scales = scales_in.to(at::kFloat).contiguous();
  const int64_t N = scales.size(0), KG = scales.size(1);
  const int64_t nt = woq_hip_padded_n(N) / WOQ_HIP_TILE_N;
  const auto opt = scales.options();
  PackedQParams q;
  q.s32 = at::empty({nt, KG, WOQ_HIP_TILE_N}, opt);
  q.s16 = at::empty({nt, KG, WOQ_HIP_TILE_N}, opt.dtype(at::kHalf));
  q.sb16 = at::empty({nt, KG, WOQ_HIP_TILE_N}, opt.dtype(at::kBFloat16));
  Tensor zeros;
  if (zeros_in.has_value()) {
    zeros = zeros_in->to(at::kFloat).contiguous();
    q.z8 = at::empty({nt, KG, WOQ_HIP_TILE_N}, opt.dtype(at::kByte));
  }
  if (!is_8bit(wd)) q.sz = at::empty({nt, KG, WOQ_HIP_TILE_N}, opt.dtype(at::kInt));
  if (wd == WOQ_HIP_DTYPE_INT4 || wd == WOQ_HIP_DTYPE_INT8) q.szb = at::empty({nt, KG, WOQ_HIP_TILE_N}, opt.dtype(at::kInt));
  DeviceScope scope(scales);
  check_rc(woq_hip_pack_qparams(scales.data_ptr<float>(), zeros.defined() ? zeros.data_ptr<float>() : nullptr, (int)wd,
                                N, KG, q.s32.data_ptr<float>(), q.s16.data_ptr(), q.sb16.data_ptr(),
                                q.z8.has_value() ? q.z8->data_ptr<uint8_t>() : nullptr,
                                q.sz.has_value() ? (uint32_t*)q.sz->data_ptr() : nullptr,
                                q.szb.has_value() ? (uint32_t*)q.szb->data_ptr() : nullptr, current_stream(scales)),
           "pack_qparams");
  return q;
}

// One zeroed counter array per (device, stream) for the kernels that share K between workgroups; none
// while a graph is being captured on a stream that has no array yet (an allocation made during capture
// belongs to the graph's pool): the call then runs without splitting K.
static optional<Tensor> split_k_counters(const Tensor& like) {
  static std::mutex& mu = *new std::mutex();
  static auto& cache = *new std::unordered_map<uint64_t, Tensor>();  // never destroyed (outlives the HIP runtime otherwise)
  const auto stream = c10::hip::getCurrentHIPStream((c10::DeviceIndex)like.get_device());
  const uint64_t key = ((uint64_t)like.get_device() << 56) ^ (uint64_t)(uintptr_t)stream.stream();
  std::lock_guard<std::mutex> lock(mu);
  auto it = cache.find(key);
  if (it != cache.end()) return it->second;
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream.stream(), &status) != hipSuccess || status != hipStreamCaptureStatusNone)
    return c10::nullopt;
  Tensor buf = at::zeros({512}, like.options().dtype(at::kInt));
  cache.emplace(key, buf);
  return buf;
}

// ---- the prepack context ----------------------------------------------------------------------------
static std::atomic<int64_t> g_next_handle{1};
// Bumped whenever a context changes or frees its device arrays (load_from_ctx, release): whoever caches the
// addresses of kernel_pointers() compares it before every use.
static std::atomic<int64_t> g_context_epoch{0};
static void unregister_context(int64_t handle);

// Prepacked weight and quantization parameters of one linear layer (ContextLinearWoq /
// IpexWoqLinearOpContext of the reference, csrc/cpu/jit/cpu/kernels/ContextLinearWoq.h:12-139,
// OpContext.cpp:364-507).  `weight` is the plain checkpoint format: uint8 [N, ceil(K/2)] for 4-bit,
// int8 [N, K] for 8-bit weights.
class WoqLinearOpContext : public torch::CustomClassHolder {
 public:
  WoqLinearOpContext(Tensor weight, int64_t weight_dtype, std::vector<int64_t> weight_shape, Tensor scales,
                     optional<Tensor> zero_points, optional<Tensor> bias, optional<Tensor> g_idx,
                     optional<int64_t> batch_size, int64_t group_size, int64_t lowp_mode, int64_t act_quant_mode,
                     bool cache_weight_for_large_batch) {
    init(std::move(weight), weight_dtype, std::move(weight_shape), std::move(scales), std::move(zero_points),
         std::move(bias), std::move(g_idx), batch_size, group_size, lowp_mode, act_quant_mode,
         cache_weight_for_large_batch);
    handle_ = g_next_handle.fetch_add(1);
  }

  // Runs when the last owner lets go (the table of live contexts holds a weak reference, so this, not the
  // destructor, is the first thing to happen): the handle stops resolving and the device memory is freed.
  void release_resources() override {
    g_context_epoch.fetch_add(1);
    unregister_context(handle_);
    packed_ = Tensor();
    q_ = PackedQParams();
    bias_f32_ = Tensor();
  }

  // ---- the reference's method surface ----
  // The packed bytes; for FP8 weights seen as float8 e4m3fn, the dtype the reference's packed weight keeps
  // (tests/cpu/test_quantization_default_recipe.py:2211-2214).
  Tensor get_weight() { return weight_dtype_ == WOQ_HIP_DTYPE_FP8 ? packed_.view(at::kFloat8_e4m3fn) : packed_; }
  optional<Tensor> get_bias() { return bias_; }
  Tensor get_scales() { return scales_plain_; }
  optional<Tensor> get_zero_points() { return zeros_plain_; }
  std::vector<int64_t> get_weight_shape() { return {N_, K_}; }
  // What a grouped launch over many contexts (the experts of a mixture-of-experts layer) needs of each: the device
  // addresses of the packed weight, the fp16 and bf16 scales, the zero points and the fp32 bias (0: none), then
  // N, K, group size, weight dtype, lowp_mode, whether the input channels are permuted (g_idx), the device index,
  // and the (fp16 scale, fp16 128 + zero) dword table of the single-row decode kernel (0: none).
  std::vector<int64_t> kernel_pointers() {
    auto addr = [](const Tensor& t) -> int64_t { return t.defined() ? (int64_t)(uintptr_t)t.data_ptr() : 0; };
    return {addr(packed_), addr(q_.s16), addr(q_.sb16), q_.z8.has_value() ? addr(*q_.z8) : 0, addr(bias_f32_),
            N_, K_, group_size_, weight_dtype_, lowp_mode_, g_src_.defined() ? 1 : 0, (int64_t)packed_.device().index(),
            q_.sz.has_value() ? addr(*q_.sz) : 0};
  }
  optional<Tensor> get_g_idx() { return g_idx_; }
  // The dequantized bf16 copy of the weight that cache_weight_for_large_batch asks for under lowp_mode BF16
  // (csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:430-486), in the operand layout of the dense kernel
  // ([K / 128][padded N / 16][4][64][8] bf16); nothing where the flag is off or no copy can be made
  // (K not a multiple of 128).  Made at prepack time, not on the first large batch: a forward call mutates nothing.
  optional<Tensor> get_cached_weight() { return dense_.defined() ? optional<Tensor>(dense_) : c10::nullopt; }
  // The reference caches the column sums of an int8 copy of the weight for lowp_mode INT8
  // (LinearWoqPacked.cpp:485-508); here the int8 MFMA kernels read the stored codes and form those sums
  // on the fly, so there is nothing to cache.
  optional<Tensor> get_cached_compensation() { return c10::nullopt; }
  // plain -> packed layout of this context (woq_linear_pack_weight of the reference)
  Tensor pack(const Tensor& plain) {
    Tensor p = to_gpu(plain, packed_.device());
    if (g_src_.defined()) p = shuffle_int4_weight(p, N_, K_, g_src_);
    return pack_weight(p, weight_dtype_, N_, K_);
  }
  // packed -> plain [N, K/2] (or [N, K]) checkpoint layout, back in the checkpoint's channel order
  // (csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:748-775)
  Tensor to_public(const Tensor& packed) {
    Tensor plain = unpack_weight(packed, weight_dtype_, N_, K_);
    if (g_dst_.defined()) plain = shuffle_int4_weight(plain, N_, K_, g_dst_);
    return plain;
  }
  // 1-element CPU int64 tensor naming this context (csrc/cpu/jit/cpu/kernels/OpContext.cpp:396-400).  A
  // key into the table of live contexts rather than the raw address: a stale handle raises instead of
  // dereferencing freed memory.
  Tensor get_data_handle() {
    Tensor h = at::empty({1}, at::TensorOptions().dtype(at::kLong));
    h.data_ptr<int64_t>()[0] = handle_;
    return h;
  }
  void load_from_ctx(const c10::intrusive_ptr<WoqLinearOpContext>& other) {
    const int64_t keep = handle_;
    g_context_epoch.fetch_add(1);
    copy_state(*other);
    handle_ = keep;
  }

  using State = std::tuple<Tensor, int64_t, std::vector<int64_t>, Tensor, optional<Tensor>, optional<Tensor>,
                           optional<Tensor>, optional<int64_t>, int64_t, int64_t, int64_t, bool>;
  // always the plain format, re-prepacked on load (csrc/cpu/jit/cpu/kernels/OpContext.h:363-403)
  State get_state() {
    auto cpu = [](const optional<Tensor>& t) -> optional<Tensor> {
      return t.has_value() ? optional<Tensor>(t->detach().cpu()) : c10::nullopt;
    };
    // float8 tensors do not pickle with every torch version: the state carries their bytes, which the
    // constructor takes as well
    Tensor w = to_public(packed_).cpu();
    if (w.scalar_type() == at::kFloat8_e4m3fn) w = w.view(at::kByte);
    return State(w, weight_dtype_, {N_, K_}, scales_plain_.detach().cpu(), cpu(zeros_plain_),
                 cpu(bias_), cpu(g_idx_), batch_size_, group_size_, lowp_mode_, act_quant_mode_, cache_weight_);
  }

  // ---- execution ----
  Tensor run(const Tensor& x_in, int64_t fusion, const std::vector<Tensor>& others) {
    TORCH_CHECK(x_in.size(-1) == K_, "WOQ linear: input and weight shapes do not match, got k = ", x_in.size(-1),
                " and ", K_, " respectively.");
    const int64_t M = x_in.numel() > 0 ? x_in.numel() / K_ : 0;
    std::vector<int64_t> out_sizes = x_in.sizes().vec();
    out_sizes.back() = N_;
    if (M == 0) return at::empty(out_sizes, x_in.options());
    Tensor x = x_in;
    if (g_src_.defined()) x = shuffle_activations(x, g_src_);
    return run_sorted(x, M, fusion, others, out_sizes);
  }

  int64_t handle() const { return handle_; }

 private:
  void init(Tensor weight, int64_t weight_dtype, std::vector<int64_t> weight_shape, Tensor scales,
            optional<Tensor> zero_points, optional<Tensor> bias, optional<Tensor> g_idx, optional<int64_t> batch_size,
            int64_t group_size, int64_t lowp_mode, int64_t act_quant_mode, bool cache_weight) {
    TORCH_CHECK(weight_dtype == WOQ_HIP_DTYPE_INT8 || weight_dtype == WOQ_HIP_DTYPE_INT4 ||
                    weight_dtype == WOQ_HIP_DTYPE_NF4 || weight_dtype == WOQ_HIP_DTYPE_FP8,
                "WOQ linear: unsupported weight dtype ", weight_dtype);
    TORCH_CHECK(!(weight_dtype == WOQ_HIP_DTYPE_NF4 && zero_points.has_value()),
                "WOQ: symmetric quantization is required for NF4 or INT8 with lowp-mode INT8");
    TORCH_CHECK(!(weight_dtype == WOQ_HIP_DTYPE_FP8 && zero_points.has_value()), "WOQ: FP8 weights take no zero points");
    TORCH_CHECK(!(weight_dtype == WOQ_HIP_DTYPE_FP8 && lowp_mode == WOQ_HIP_LOWP_INT8),
                "WOQ: lowp-mode INT8 does not take FP8 weights");
    TORCH_CHECK(weight_shape.size() == 2, "WOQ linear: weight shape must be [N, K]");
    const int64_t N = weight_shape[0], K = weight_shape[1];
    weight = to_gpu(weight);
    const auto dev = weight.device();
    if (weight_dtype == WOQ_HIP_DTYPE_FP8) {
      // float8 e4m3fn values, or their bytes
      TORCH_CHECK((weight.scalar_type() == at::kFloat8_e4m3fn || weight.scalar_type() == at::kByte) && weight.dim() == 2 &&
                      weight.size(0) == N && weight.size(1) == K,
                  "WOQ linear: fp8 weight must be float8_e4m3fn [", N, ", ", K, "]");
      weight = weight.contiguous().view(at::kByte);
    } else if (weight_dtype != WOQ_HIP_DTYPE_INT8) {
      if (weight.scalar_type() != at::kByte) weight = weight.contiguous().view(at::kByte);
      TORCH_CHECK(weight.dim() == 2 && weight.size(0) == N && weight.size(1) == (K + 1) / 2,
                  "WOQ linear: 4-bit weight has shape ", weight.sizes(), ", expected [", N, ", ", (K + 1) / 2, "]");
    } else {
      TORCH_CHECK(weight.scalar_type() == at::kChar && weight.dim() == 2 && weight.size(0) == N && weight.size(1) == K,
                  "WOQ linear: int8 weight must be int8 [", N, ", ", K, "]");
    }
    scales = to_gpu(scales, dev).to(at::kFloat);
    if (group_size > 0) {
      const int64_t KG = (K + group_size - 1) / group_size;
      scales = scales.reshape({N, -1});
      TORCH_CHECK(scales.size(1) == KG, "WOQ linear: scales have ", scales.size(1), " groups, expected ", KG,
                  " for group_size ", group_size);
    } else {
      scales = scales.reshape({N, 1});
    }
    optional<Tensor> zps;
    if (zero_points.has_value()) {
      Tensor z = to_gpu(*zero_points, dev).to(at::kFloat).reshape(scales.sizes());
      const double lo = weight_dtype == WOQ_HIP_DTYPE_INT8 ? -128 : 0, hi = 127;
      const bool ok = at::equal(z, z.round()) && z.ge(lo).all().item<bool>() && z.le(hi).all().item<bool>();
      TORCH_CHECK(ok, "WOQ linear: zero points must be integers in [", lo, ", ", hi, "] for this weight dtype");
      zps = z;
    }
    TORCH_CHECK(!(weight_dtype == WOQ_HIP_DTYPE_INT8 && lowp_mode == WOQ_HIP_LOWP_INT8 && zps.has_value()),
                "WOQ: symmetric quantization is required for NF4 or INT8 with lowp-mode INT8");

    weight_dtype_ = weight_dtype;
    N_ = N;
    K_ = K;
    group_size_ = group_size;
    lowp_mode_ = lowp_mode;
    act_quant_mode_ = act_quant_mode;
    batch_size_ = batch_size;
    cache_weight_ = cache_weight;
    // GPTQ act-order: input channel k belongs to group g_idx[k].  As the reference does for 4-bit
    // group-wise weights (LinearWoqPacked.cpp:306-316, 407-421) the weight's input channels are sorted
    // by group once here and the activations are shuffled the same way per call.
    g_idx_ = c10::nullopt;
    g_src_ = Tensor();
    g_dst_ = Tensor();
    if (g_idx.has_value() && weight_dtype == WOQ_HIP_DTYPE_INT4 && group_size > 0) {
      const Tensor g = to_gpu(*g_idx, dev).to(at::kLong).reshape({-1});
      const int64_t KG = (K + group_size - 1) / group_size;
      TORCH_CHECK(g.numel() == K, "g_idx size and weight shape mismatch");
      TORCH_CHECK(g.min().item<int64_t>() >= 0 && g.max().item<int64_t>() < KG, "WOQ linear: g_idx values must lie in [0, ",
                  KG, ")");
      Tensor want = at::full({KG}, group_size, g.options());
      want.select(0, KG - 1).fill_(K - (KG - 1) * group_size);
      TORCH_CHECK(at::equal(at::bincount(g, {}, KG), want),
                  "WOQ linear: g_idx must assign exactly group_size channels to every group");
      const Tensor src = at::argsort(g, /*stable=*/true, /*dim=*/-1, /*descending=*/false);
      g_idx_ = *g_idx;
      g_src_ = src.to(at::kInt).contiguous();
      g_dst_ = at::argsort(src).to(at::kInt).contiguous();
      weight = shuffle_int4_weight(weight, N, K, g_src_);
    }
    bias_ = bias.has_value() ? optional<Tensor>(to_gpu(*bias, dev)) : c10::nullopt;
    bias_f32_ = bias_.has_value() ? bias_->to(at::kFloat).contiguous() : Tensor();
    packed_ = pack_weight(weight, weight_dtype, N, K);
    q_ = pack_qparams(scales, zps, weight_dtype);
    dense_ = Tensor();
    if (cache_weight && lowp_mode == WOQ_HIP_LOWP_BF16) {
      if (const int64_t bytes = woq_hip_dense_weight_bytes((int32_t)weight_dtype, N, K)) {
        const int64_t nt = woq_hip_padded_n(N) / WOQ_HIP_TILE_N;
        TORCH_CHECK(bytes == K / 128 * nt * 4 * 64 * 16, "WOQ linear: unexpected size of the dense copy");
        dense_ = at::empty({K / 128, nt, 4, 64, 8}, packed_.options().dtype(at::kBFloat16));
        DeviceScope scope(packed_);
        check_rc(woq_hip_dense_weight(packed_.data_ptr(), (int32_t)weight_dtype, N, K, q_.sb16.data_ptr(),
                                      q_.z8.has_value() ? q_.z8->data_ptr<uint8_t>() : nullptr, group_size,
                                      dense_.data_ptr(), current_stream(packed_)),
                 "woq_linear_prepack");
      }
    }
    scales_plain_ = group_size > 0 ? scales : scales.reshape({N});
    zeros_plain_ = zps.has_value() ? optional<Tensor>(group_size > 0 ? *zps : zps->reshape({N})) : c10::nullopt;
  }

  void copy_state(const WoqLinearOpContext& o) {
    packed_ = o.packed_; q_ = o.q_; dense_ = o.dense_; bias_ = o.bias_; bias_f32_ = o.bias_f32_; scales_plain_ = o.scales_plain_;
    zeros_plain_ = o.zeros_plain_; g_idx_ = o.g_idx_; g_src_ = o.g_src_; g_dst_ = o.g_dst_;
    N_ = o.N_; K_ = o.K_; group_size_ = o.group_size_;
    weight_dtype_ = o.weight_dtype_; lowp_mode_ = o.lowp_mode_; act_quant_mode_ = o.act_quant_mode_;
    batch_size_ = o.batch_size_; cache_weight_ = o.cache_weight_;
  }

  // `run` behind the act-order shuffle: the input channels of x are in the order of the stored weight
  Tensor run_sorted(const Tensor& x, int64_t M, int64_t fusion, const std::vector<Tensor>& others,
                    const std::vector<int64_t>& out_sizes) {
    Tensor x2 = x.is_contiguous() ? x : x.contiguous();
    if ((uintptr_t)x2.data_ptr() % 16) x2 = x2.clone();  // the kernels read activation rows with 16-byte loads
    Tensor out = at::empty(out_sizes, x.options());
    if (lowp_mode_ == WOQ_HIP_LOWP_FP16 && x.scalar_type() == at::kBFloat16 && M > 16 && fusion == WOQ_HIP_FUSE_NONE) {
      // fp16 compute on bf16 rows beyond one row tile: the reference converts the rows to fp16 and casts
      // the fp16 result to bf16 (csrc/cpu/aten/utils/woq.h:3076-3085).  The library converts the rows once;
      // its fp16 kernels then write the bf16 output themselves.
      Tensor xh = at::empty(x2.sizes(), x2.options().dtype(at::kHalf));
      DeviceScope scope(x2);
      check_rc(woq_hip_convert_activations(x2.data_ptr(), WOQ_HIP_ACT_BF16, xh.data_ptr(), WOQ_HIP_ACT_FP16,
                                           x2.numel(), current_stream(x2)),
               "woq_linear");
      x2 = xh;
    }
    woq_hip_linear_params p;
    memset(&p, 0, sizeof(p));
    p.struct_size = sizeof(p);
    p.x = x2.data_ptr();
    p.x_dtype = act_code(x2.scalar_type());
    p.M = M; p.K = K_; p.N = N_;
    p.qweight = packed_.data_ptr();
    p.weight_dtype = (int32_t)weight_dtype_;
    p.scales_f32 = q_.s32.data_ptr<float>();
    p.scales_f16 = q_.s16.data_ptr();
    p.scales_bf16 = q_.sb16.data_ptr();
    p.zeros_u8 = q_.z8.has_value() ? q_.z8->data_ptr<uint8_t>() : nullptr;
    p.scale_zero_f16x2 = q_.sz.has_value() ? (const uint32_t*)q_.sz->data_ptr() : nullptr;
    p.scale_zero_bf16 = q_.szb.has_value() ? (const uint32_t*)q_.szb->data_ptr() : nullptr;
    p.dense_bf16 = dense_.defined() ? dense_.data_ptr() : nullptr;
    p.group_size = group_size_;
    p.bias = bias_f32_.defined() ? bias_f32_.data_ptr<float>() : nullptr;
    p.lowp_mode = (int32_t)lowp_mode_;
    p.act_quant_mode = (int32_t)act_quant_mode_;
    p.fusion = (int32_t)fusion;
    std::vector<Tensor> keep;
    for (size_t i = 0; i < others.size() && i < 2; ++i) {
      TORCH_CHECK(others[i].numel() == M * N_, "woq_linear: post-op operand must have the output's shape");
      TORCH_CHECK(others[i].is_cuda() && others[i].device() == x.device(),
                  "woq_linear: expected all tensors to be on the same device, but the post-op operand is on ",
                  others[i].device(), " and the input on ", x.device());
      keep.push_back(others[i].to(x.scalar_type()).contiguous());
      p.others[i] = keep.back().data_ptr();
    }
    p.out = out.data_ptr();
    p.out_dtype = act_code(x.scalar_type());
    DeviceScope scope(x2);
    p.stream = current_stream(x2);
    const bool int8 = lowp_mode_ == WOQ_HIP_LOWP_INT8;
    int64_t wbytes = int8 ? woq_hip_linear_workspace_bytes(M, K_, WOQ_HIP_LOWP_INT8, (int32_t)act_quant_mode_, group_size_) : 0;
    optional<Tensor> counters;
    // long K and few output tiles: scratch with which the kernels share K between workgroups, and the zeroed
    // counters of this stream (the library says for which problems it would use them)
    if (const int64_t extra = woq_hip_linear_auto_split_k_workspace_bytes(M, K_, N_, (int32_t)lowp_mode_)) {
      counters = split_k_counters(x2);
      if (counters.has_value()) wbytes = (wbytes + 255) / 256 * 256 + extra;
    }
    Tensor ws;
    if (wbytes > 0) {
      ws = at::empty({wbytes}, x.options().dtype(at::kByte));
      p.workspace = ws.data_ptr();
      p.workspace_bytes = wbytes;
      p.split_k_counters = counters.has_value() ? counters->data_ptr<int32_t>() : nullptr;
    }
    check_rc(woq_hip_linear(&p), "woq_linear");
    return out;
  }

  Tensor packed_;
  PackedQParams q_;
  Tensor dense_;  // cache_weight_for_large_batch under lowp_mode BF16: the dense bf16 copy, or undefined
  optional<Tensor> bias_;
  Tensor bias_f32_;
  Tensor scales_plain_;
  optional<Tensor> zeros_plain_;
  optional<Tensor> g_idx_;
  Tensor g_src_, g_dst_;
  int64_t N_ = 0, K_ = 0, group_size_ = -1, weight_dtype_ = 0, lowp_mode_ = 0, act_quant_mode_ = 0;
  optional<int64_t> batch_size_;
  bool cache_weight_ = false;
  int64_t handle_ = 0;
};

// Live contexts by handle: weak references, so that a handle whose context has gone is detected.  The
// table is never destroyed: contexts may outlive the static destructors of this library at process exit.
static std::mutex& ctx_mutex() {
  static std::mutex* m = new std::mutex();
  return *m;
}
static std::unordered_map<int64_t, c10::weak_intrusive_ptr<WoqLinearOpContext>>& contexts() {
  static auto* t = new std::unordered_map<int64_t, c10::weak_intrusive_ptr<WoqLinearOpContext>>();
  return *t;
}

static void unregister_context(int64_t handle) {
  std::lock_guard<std::mutex> lock(ctx_mutex());
  contexts().erase(handle);
}

static c10::intrusive_ptr<WoqLinearOpContext> context_from_handle(const Tensor& handle, const char* op) {
  TORCH_CHECK(handle.scalar_type() == at::kLong && handle.numel() == 1 && handle.is_cpu(), op,
              ": W_prepack must be the 1-element int64 tensor of get_data_handle()");
  const int64_t key = handle.data_ptr<int64_t>()[0];
  // (the ctypes twin of the Python package hands out negative handles, so that neither kind resolves as the other)
  TORCH_CHECK(key > 0, op, ": this handle does not come from a torch.classes.ipex_prepack.WoqLinearOpContext");
  c10::intrusive_ptr<WoqLinearOpContext> ctx;
  {
    std::lock_guard<std::mutex> lock(ctx_mutex());
    auto it = contexts().find(key);
    if (it != contexts().end()) ctx = it->second.lock();
  }
  TORCH_CHECK(ctx, op, ": the prepack context behind this handle no longer exists");
  return ctx;
}

template <class... Args>
static c10::intrusive_ptr<WoqLinearOpContext> make_context(Args&&... args) {
  auto ctx = c10::make_intrusive<WoqLinearOpContext>(std::forward<Args>(args)...);
  std::lock_guard<std::mutex> lock(ctx_mutex());
  contexts().emplace(ctx->handle(), c10::weak_intrusive_ptr<WoqLinearOpContext>(ctx));
  return ctx;
}

// ---- ipex_prepack ops --------------------------------------------------------------------------------
// createWoqLinearPrePackOpContext (csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:20-51)
static c10::intrusive_ptr<WoqLinearOpContext> weight_only_qlinear_prepack(
    Tensor W, int64_t W_dtype, std::vector<int64_t> W_shape, Tensor scales, optional<Tensor> zero_points,
    optional<Tensor> B, optional<Tensor> g_idx, optional<int64_t> batch_size, int64_t group_size, int64_t lowp_mode,
    int64_t act_quant_mode, bool cache_weight_for_large_batch) {
  return make_context(std::move(W), W_dtype, std::move(W_shape), std::move(scales),
                                                 std::move(zero_points), std::move(B), std::move(g_idx), batch_size,
                                                 group_size, lowp_mode, act_quant_mode, cache_weight_for_large_batch);
}

// int32 [..., C] -> int32 [..., C, 8], nibble i in the last dimension
static Tensor unpack_int32_nibbles(const Tensor& t) {
  const Tensor shifts = at::arange(0, 32, 4, t.options().dtype(at::kInt));
  return at::bitwise_and(at::bitwise_right_shift(t.unsqueeze(-1), shifts), 0xF);
}

// uint8 codes [N, K] -> plain packed [N, K/2], low nibble = even k
// (intel_extension_for_pytorch/quantization/_quantize_utils.py:1184)
static Tensor nibbles_to_plain(Tensor q) {
  q = q.to(at::kByte);
  if (q.size(1) % 2) q = at::constant_pad_nd(q, {0, 1}, 0);
  const Tensor even = q.slice(1, 0, c10::nullopt, 2), odd = q.slice(1, 1, c10::nullopt, 2);
  return at::bitwise_or(at::bitwise_left_shift(odd, 4), even).contiguous();
}

// GPTQ int32 [K/8, N]: nibble i of word [j, n] is q[8j + i, n]
// (intel_extension_for_pytorch/nn/utils/_model_convert.py:62-257, csrc/cpu/aten/kernels/WoqUtilKrnl.cpp:109-218)
static Tensor gptq_to_plain(const Tensor& qweight) {
  TORCH_CHECK(qweight.scalar_type() == at::kInt && qweight.dim() == 2, "GPTQ qweight must be int32 [K/8, N]");
  const int64_t k8 = qweight.size(0), n = qweight.size(1);
  return nibbles_to_plain(unpack_int32_nibbles(qweight).permute({1, 0, 2}).reshape({n, k8 * 8}));
}

// AWQ int32 [K, N/8]: nibble i of word [k, j] is q[k, 8j + order[i]], order = 0 2 4 6 1 3 5 7
static Tensor awq_to_plain(const Tensor& qweight) {
  TORCH_CHECK(qweight.scalar_type() == at::kInt && qweight.dim() == 2, "AWQ qweight must be int32 [K, N/8]");
  const int64_t k = qweight.size(0), n8 = qweight.size(1);
  // column c of a group of 8 sits in nibble nibble_of_col[c]
  const Tensor sel = at::tensor(std::vector<int64_t>{0, 4, 1, 5, 2, 6, 3, 7}, qweight.options().dtype(at::kLong));
  const Tensor q = unpack_int32_nibbles(qweight).index_select(-1, sel).reshape({k, n8 * 8});
  return nibbles_to_plain(q.t());
}

// INT4 checkpoint ingest (createWoqLinearPrePackOpContextInt4,
// csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:53-202): scales -> fp32, int32-compressed zero points ->
// one value per group, int32 / uint8 weight viewed as bytes, or a float weight re-quantized with the
// given parameters.
static c10::intrusive_ptr<WoqLinearOpContext> weight_only_qlinear_prepack_int4(
    Tensor W, Tensor scales, optional<Tensor> zeros, optional<Tensor> B, optional<Tensor> g_idx,
    optional<int64_t> batch_size, int64_t group_size, int64_t lowp_mode, int64_t act_quant_mode,
    bool cache_weight_for_large_batch, int64_t weight_format) {
  W = to_gpu(W);
  const auto dev = W.device();
  const Tensor scales_f32 = to_gpu(scales, dev).squeeze().to(at::kFloat);
  optional<Tensor> zp_f32;
  if (zeros.has_value()) {
    const Tensor z = to_gpu(*zeros, dev);
    if (z.scalar_type() == at::kInt && z.numel() != scales_f32.numel()) {
      TORCH_CHECK(scales_f32.dim() == 2 && z.dim() == 2 && scales_f32.size(0) == z.size(0),
                  "IPEX WOQ INT4: unexpected zero points size");
      const Tensor zc = z.contiguous();
      Tensor out = at::empty({zc.size(0), scales_f32.size(1)}, zc.options().dtype(at::kFloat));
      DeviceScope scope(zc);
      check_rc(woq_hip_unpack_int4_zeros(zc.data_ptr<int32_t>(), zc.size(0), scales_f32.size(1), zc.size(1),
                                         out.data_ptr<float>(), current_stream(zc)),
               "unpack_int4_zeros");
      zp_f32 = out;
    } else {
      TORCH_CHECK(z.numel() == scales_f32.numel(), "IPEX WOQ INT4: unexpected zero points size");
      zp_f32 = z.squeeze().to(at::kFloat);
    }
  }
  Tensor plain;
  int64_t N, K;
  if (W.scalar_type() == at::kInt || W.scalar_type() == at::kByte) {
    if (weight_format == kGptqFormat)
      plain = gptq_to_plain(W);
    else if (weight_format == kAwqFormat)
      plain = awq_to_plain(W);
    else
      plain = W.contiguous().view(at::kByte);
    N = plain.size(0);
    K = plain.size(1) * 2;
  } else if (W.scalar_type() == at::kBFloat16 || W.scalar_type() == at::kFloat || W.scalar_type() == at::kHalf) {
    N = W.size(0);
    K = W.size(1);
    const Tensor w = W.to(at::kFloat);
    Tensor q;
    if (group_size > 0) {
      q = w.view({N, K / group_size, group_size}) / scales_f32.unsqueeze(2);
      if (zp_f32.has_value()) q = q + zp_f32->unsqueeze(2);
    } else {
      q = w / scales_f32.unsqueeze(1);
      if (zp_f32.has_value()) q = q + zp_f32->unsqueeze(1);
    }
    plain = nibbles_to_plain(at::round(q).to(at::kByte).view({N, K}));
  } else {
    TORCH_CHECK(false, "IPEX WOQ INT4: unexpected weight data type: ", W.scalar_type());
  }
  return make_context(plain, (int64_t)WOQ_HIP_DTYPE_INT4, std::vector<int64_t>{N, K},
                                                 scales_f32, zp_f32, std::move(B), std::move(g_idx), batch_size,
                                                 group_size, lowp_mode, act_quant_mode, cache_weight_for_large_batch);
}

// packWoqLinearWeight (csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:212-256): (packed weight,
// [scales fp32, fp16, bf16], [zeros fp32, fp16, bf16, stored bytes] or None, [bias fp32, fp16, bf16] or None,
// compensation = None).  The lists hold the kernel layout [N/16, K/G, 16], which is what `woq_linear` takes back.
static std::tuple<Tensor, std::vector<Tensor>, optional<std::vector<Tensor>>, optional<std::vector<Tensor>>,
                  optional<Tensor>>
woq_linear_pack_weight(Tensor W, c10::string_view W_dtype, std::vector<int64_t> W_shape, Tensor scales,
                       optional<Tensor> zero_points, optional<Tensor> B, optional<Tensor> g_idx, int64_t group_size,
                       int64_t lowp_mode) {
  TORCH_CHECK(W_shape.size() == 2, "woq_linear_pack_weight: W_shape must be [N, K]");
  const int64_t wd = weight_dtype_of(W_dtype), N = W_shape[0], K = W_shape[1];
  Tensor w = to_gpu(W);
  const auto dev = w.device();
  Tensor s = to_gpu(scales, dev).to(at::kFloat);
  s = group_size > 0 ? s.reshape({N, -1}) : s.reshape({N, 1});
  optional<Tensor> z;
  if (zero_points.has_value()) z = to_gpu(*zero_points, dev).to(at::kFloat).reshape(s.sizes());
  if (wd != WOQ_HIP_DTYPE_INT8 && w.scalar_type() != at::kByte) w = w.contiguous().view(at::kByte);
  if (g_idx.has_value() && wd == WOQ_HIP_DTYPE_INT4 && group_size > 0) {
    const Tensor src = at::argsort(to_gpu(*g_idx, dev).to(at::kLong).reshape({-1}), true, -1, false).to(at::kInt).contiguous();
    w = shuffle_int4_weight(w, N, K, src);
  }
  const Tensor packed = pack_weight(w, wd, N, K);
  const PackedQParams q = pack_qparams(s, z, wd);
  (void)lowp_mode;
  optional<std::vector<Tensor>> zeros, bias;
  if (q.z8.has_value()) {
    Tensor zf = q.z8->to(at::kFloat);
    if (wd == WOQ_HIP_DTYPE_INT8) zf = zf - 128;
    zeros = std::vector<Tensor>{zf, zf.to(at::kHalf), zf.to(at::kBFloat16), *q.z8};
  }
  if (B.has_value()) {
    const Tensor b = to_gpu(*B, dev);
    bias = std::vector<Tensor>{b.to(at::kFloat), b.to(at::kHalf), b.to(at::kBFloat16)};
  }
  return {packed, {q.s32, q.s16, q.sb16}, zeros, bias, c10::nullopt};
}

// unpackWoqLinearWeight (csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:258-275)
static Tensor woq_linear_unpack_weight(Tensor W, c10::string_view W_dtype, std::vector<int64_t> W_shape,
                                       int64_t lowp_mode) {
  (void)lowp_mode;
  TORCH_CHECK(W_shape.size() == 2, "woq_linear_unpack_weight: W_shape must be [N, K]");
  return unpack_weight(W, weight_dtype_of(W_dtype), W_shape[0], W_shape[1]);
}

// ---- torch_ipex forward ops ---------------------------------------------------------------------------
static Tensor ipex_woq_linear(const Tensor& input, const Tensor& W_prepack) {
  require_gpu_input(input, "torch_ipex::ipex_woq_linear");
  return context_from_handle(W_prepack, "torch_ipex::ipex_woq_linear")->run(input, WOQ_HIP_FUSE_NONE, {});
}

template <int FUSION>
static Tensor woq_linear_unary(const Tensor& input, const Tensor& W_prepack) {
  require_gpu_input(input, "torch_ipex::woq_linear_<post-op>");
  return context_from_handle(W_prepack, "torch_ipex::woq_linear_<post-op>")->run(input, FUSION, {});
}

template <int FUSION, int NOTHERS>
static Tensor woq_linear_binary(const Tensor& input, const Tensor& W_prepack, const std::vector<Tensor>& others) {
  require_gpu_input(input, "torch_ipex::woq_linear_<post-op>");
  TORCH_CHECK((int)others.size() >= NOTHERS, "torch_ipex::woq_linear_<post-op>: expected ", NOTHERS,
              " extra input(s), got ", others.size());
  std::vector<Tensor> o(others.begin(), others.begin() + NOTHERS);
  return context_from_handle(W_prepack, "torch_ipex::woq_linear_<post-op>")->run(input, FUSION, o);
}

// ---- mixture of experts over WOQ linears (csrc/cpu/aten/MoE.cpp:260-328) -------------------------------
// One expert: gather its tokens, down(up(x) * silu(gate(x))), weighted accumulation into `output`
// (mixtral_moe_woq_kernl_impl, csrc/cpu/aten/kernels/MoEKrnl.cpp:254-284).
static Tensor moe_expert(const Tensor& hidden, const Tensor& top_x_in, const Tensor& idx_in, WoqLinearOpContext& gate,
                         WoqLinearOpContext& up, WoqLinearOpContext& down, const Tensor& routing_weights, Tensor output,
                         const char* op) {
  const auto dev = hidden.device();
  TORCH_CHECK(hidden.dim() == 2 && output.dim() == 2 && output.sizes() == hidden.sizes() && output.is_contiguous() &&
                  output.device() == dev && output.scalar_type() == hidden.scalar_type(),
              op, ": hidden_states and output must be [tokens, hidden] tensors of one dtype on one device, output contiguous");
  TORCH_CHECK(routing_weights.dim() == 2 && routing_weights.size(0) == hidden.size(0) && routing_weights.device() == dev &&
                  routing_weights.scalar_type() == hidden.scalar_type(),
              op, ": routing_weights must be [tokens, top-k] in the dtype and on the device of hidden_states");
  const Tensor x = hidden.contiguous(), rw = routing_weights.contiguous();
  const Tensor top_x = top_x_in.to(dev, at::kLong).contiguous(), idx = idx_in.to(dev, at::kLong).contiguous();
  const int64_t n = top_x.numel(), T = x.size(0), H = x.size(1);
  TORCH_CHECK(idx.numel() == n, op, ": top_x and idx differ in length");
  Tensor cur = at::empty({n, H}, x.options());
  DeviceScope scope(x);
  check_rc(woq_hip_moe_gather_rows(x.data_ptr(), act_code(x.scalar_type()), T, H, top_x.data_ptr<int64_t>(), n,
                                   cur.data_ptr(), current_stream(x)), op);
  const Tensor act = gate.run(cur, WOQ_HIP_FUSE_SILU, {});
  const Tensor out = down.run(up.run(cur, WOQ_HIP_FUSE_MUL, {act}), WOQ_HIP_FUSE_NONE, {}).contiguous();
  TORCH_CHECK(out.dim() == 2 && out.size(0) == n && out.size(1) == H, op, ": the down projection must return to the hidden width");
  check_rc(woq_hip_moe_scale_add_rows(output.data_ptr(), act_code(output.scalar_type()), T, H, out.data_ptr(), rw.data_ptr(),
                                      rw.size(1), top_x.data_ptr<int64_t>(), idx.data_ptr<int64_t>(), n, current_stream(x)),
           op);
  return output;
}

static Tensor mixtral_moe_woq(const Tensor& hidden_states, const Tensor& top_x, const Tensor& idx, const Tensor& gate_wei,
                              const Tensor& up_wei, const Tensor& down_wei, const Tensor& routing_weights, Tensor output,
                              bool is_distributed) {
  const char* op = "torch_ipex::mixtral_moe_woq";
  require_gpu_input(hidden_states, op);
  TORCH_CHECK(!is_distributed, op, ": is_distributed=True needs an all-reduce, which this one-GPU build does not have");
  if (top_x.size(0) == 0) return output;
  auto gate = context_from_handle(gate_wei, op), up = context_from_handle(up_wei, op), down = context_from_handle(down_wei, op);
  return moe_expert(hidden_states, top_x, idx, *gate, *up, *down, routing_weights, output, op);
}

// All experts of a layer: the routing table is read on the host, as the reference does (its tensors live there), and
// the experts are visited in ascending order, inside an expert the tokens in ascending order (get_expert_topx_idx,
// MoE.cpp:64-81), which fixes the order of the additions into a token's row.  The Python package puts a form without
// the host read in front of this one (grouped launches, ipex_amd/ops.py).
static Tensor deepseek_moe_woq(const Tensor& hidden_states, const Tensor& topk_ids,
                               std::vector<c10::intrusive_ptr<WoqLinearOpContext>> gate_ctx,
                               std::vector<c10::intrusive_ptr<WoqLinearOpContext>> up_ctx,
                               std::vector<c10::intrusive_ptr<WoqLinearOpContext>> down_ctx, const Tensor& routing_weights,
                               bool is_distributed) {
  const char* op = "torch_ipex::deepseek_moe_woq";
  require_gpu_input(hidden_states, op);
  TORCH_CHECK(!is_distributed, op, ": is_distributed=True needs an all-reduce, which this one-GPU build does not have");
  const int64_t experts = (int64_t)gate_ctx.size();
  TORCH_CHECK((int64_t)up_ctx.size() == experts && (int64_t)down_ctx.size() == experts, op,
              ": gate / up / down lists differ in length");
  Tensor output = at::zeros_like(hidden_states, at::MemoryFormat::Contiguous);
  const Tensor ids = topk_ids.detach().to(at::kCPU, at::kLong).contiguous();
  if (ids.numel() == 0) return output;
  TORCH_CHECK(ids.dim() == 2 && ids.size(0) == hidden_states.size(0), op, ": topk_ids must be [tokens, top-k]");
  const int64_t T = ids.size(0), topk = ids.size(1);
  const int64_t* id = ids.data_ptr<int64_t>();
  // per expert the (token, slot) entries in ascending token order; a token that names an expert more than once has
  // its k-th mention in round k (the scatter adds one row per token and call)
  std::vector<std::vector<std::vector<int64_t>>> tok(experts), slot(experts);
  for (int64_t t = 0; t < T; ++t) {
    std::vector<int64_t> mentions(0);
    for (int64_t k = 0; k < topk; ++k) {
      const int64_t e = id[t * topk + k];
      TORCH_CHECK(e >= 0 && e < experts, op, ": expert ids must lie in [0, ", experts, ")");
      int64_t round = 0;
      for (int64_t j = 0; j < k; ++j) round += id[t * topk + j] == e;
      if ((int64_t)tok[e].size() <= round) { tok[e].resize(round + 1); slot[e].resize(round + 1); }
      tok[e][round].push_back(t);
      slot[e][round].push_back(k);
    }
  }
  const auto opt = at::TensorOptions().dtype(at::kLong);
  for (int64_t e = 0; e < experts; ++e) {
    for (size_t round = 0; round < tok[e].size(); ++round) {
      if (tok[e][round].empty()) continue;
      const Tensor top_x = at::tensor(tok[e][round], opt), idx = at::tensor(slot[e][round], opt);
      moe_expert(hidden_states, top_x, idx, *gate_ctx[e], *up_ctx[e], *down_ctx[e], routing_weights, output, op);
    }
  }
  return output;
}

// Context-free forward (woq_linear_forward_v2, csrc/cpu/aten/Linear.cpp:556-617); the tensor arguments
// are the outputs of woq_linear_pack_weight.
static Tensor woq_linear_v2(const Tensor& input_in, const Tensor& qweight, c10::string_view weight_dtype,
                            std::vector<int64_t> weight_shape, std::vector<Tensor> weight_scales,
                            optional<std::vector<Tensor>> weight_zeros, optional<std::vector<Tensor>> bias,
                            optional<Tensor> g_idx, int64_t group_size, int64_t lowp_mode, int64_t act_quant_mode,
                            optional<Tensor> compensation) {
  (void)compensation;
  require_gpu_input(input_in, "torch_ipex::woq_linear");
  const int64_t wd = weight_dtype_of(weight_dtype);
  TORCH_CHECK(!weight_zeros.has_value() || weight_zeros->size() == 4, "IPEX WOQ: expect list of zeros has length 4");
  TORCH_CHECK(!bias.has_value() || bias->size() == 3, "IPEX WOQ: expect list of bias has length 3");
  TORCH_CHECK(weight_scales.size() == 3, "IPEX WOQ: expect list of scales has length 3");
  TORCH_CHECK(weight_shape.size() == 2, "IPEX WOQ: weight_shape must be [N, K]");
  const int64_t N = weight_shape[0], K = weight_shape[1];
  Tensor input = input_in;
  if (g_idx.has_value() && wd == WOQ_HIP_DTYPE_INT4 && group_size > 0) {
    // the packed weight from woq_linear_pack_weight is already sorted by group
    TORCH_CHECK(g_idx->numel() == input.size(-1), "g_idx size and weight shape mismatch");
    const Tensor src = at::argsort(g_idx->to(input.device()).to(at::kLong).reshape({-1}), true, -1, false).to(at::kInt).contiguous();
    input = shuffle_activations(input, src);
  }
  TORCH_CHECK(input.size(-1) == K, "WOQ linear: input and weight shapes do not match, got k = ", input.size(-1),
              " and ", K, " respectively.");
  // The tensor arguments go to the kernels as raw device pointers: each must live on the input's GPU and have the
  // dtype and size of woq_linear_pack_weight's outputs for [N, K] and this group size, or the kernels would read
  // host memory or past the end of an allocation.
  TORCH_CHECK(N > 0 && K > 0, "IPEX WOQ: weight_shape must be positive, got [", N, ", ", K, "]");
  auto on_input_device = [&](const Tensor& t, const char* what) {
    TORCH_CHECK(t.is_cuda() && t.device() == input.device(), "torch_ipex::woq_linear: expected all tensors to be on the "
                "same device, but ", what, " is on ", t.device(), " and the input on ", input.device());
    TORCH_CHECK(t.is_contiguous(), "torch_ipex::woq_linear: ", what, " must be contiguous");
  };
  on_input_device(qweight, "the packed weight");
  TORCH_CHECK((int64_t)qweight.nbytes() == woq_hip_packed_weight_bytes((int)wd, N, K), "torch_ipex::woq_linear: the packed "
              "weight has ", qweight.nbytes(), " bytes, expected ", woq_hip_packed_weight_bytes((int)wd, N, K), " for [", N,
              ", ", K, "] (the first output of woq_linear_pack_weight)");
  const int64_t KG = group_size > 0 ? (K + group_size - 1) / group_size : 1;
  const int64_t qcount = woq_hip_padded_n(N) / WOQ_HIP_TILE_N * KG * WOQ_HIP_TILE_N;
  static const at::ScalarType kScaleTypes[3] = {at::kFloat, at::kHalf, at::kBFloat16};
  for (int i = 0; i < 3; ++i) {
    on_input_device(weight_scales[i], "a scale tensor");
    TORCH_CHECK(weight_scales[i].scalar_type() == kScaleTypes[i] && weight_scales[i].numel() == qcount,
                "torch_ipex::woq_linear: scales[", i, "] must be ", kScaleTypes[i], " with ", qcount,
                " elements ([N/16, K/G, 16]), got ", weight_scales[i].scalar_type(), " with ", weight_scales[i].numel());
  }
  if (weight_zeros.has_value()) {
    const Tensor& z8 = (*weight_zeros)[3];
    on_input_device(z8, "the zero points");
    TORCH_CHECK(z8.scalar_type() == at::kByte && z8.numel() == qcount, "torch_ipex::woq_linear: zeros[3] must be uint8 "
                "with ", qcount, " elements ([N/16, K/G, 16]), got ", z8.scalar_type(), " with ", z8.numel());
  }
  if (bias.has_value()) {
    on_input_device((*bias)[0], "the bias");
    TORCH_CHECK((*bias)[0].numel() == N, "torch_ipex::woq_linear: bias has ", (*bias)[0].numel(), " elements, expected ", N);
  }
  Tensor x2 = input.reshape({-1, K}).contiguous();
  if ((uintptr_t)x2.data_ptr() % 16) x2 = x2.clone();
  const int64_t M = x2.size(0);
  std::vector<int64_t> out_sizes = input.sizes().vec();
  out_sizes.back() = N;
  Tensor out = at::empty(out_sizes, input.options());
  if (M == 0) return out;
  woq_hip_linear_params p;
  memset(&p, 0, sizeof(p));
  p.struct_size = sizeof(p);
  p.x = x2.data_ptr();
  p.x_dtype = act_code(input.scalar_type());
  p.M = M; p.K = K; p.N = N;
  p.qweight = qweight.data_ptr();
  p.weight_dtype = (int32_t)wd;
  p.scales_f32 = weight_scales[0].data_ptr<float>();
  p.scales_f16 = weight_scales[1].data_ptr();
  p.scales_bf16 = weight_scales[2].data_ptr();
  p.zeros_u8 = weight_zeros.has_value() ? (*weight_zeros)[3].data_ptr<uint8_t>() : nullptr;
  p.group_size = group_size;
  Tensor b32;
  if (bias.has_value()) {
    b32 = (*bias)[0].to(at::kFloat).contiguous();
    p.bias = b32.data_ptr<float>();
  }
  p.lowp_mode = (int32_t)lowp_mode;
  p.act_quant_mode = (int32_t)act_quant_mode;
  p.out = out.data_ptr();
  p.out_dtype = p.x_dtype;
  DeviceScope scope(x2);
  p.stream = current_stream(x2);
  Tensor ws;
  const int64_t wbytes = woq_hip_linear_workspace_bytes(M, K, (int32_t)lowp_mode, (int32_t)act_quant_mode, group_size);
  if (wbytes > 0) {
    ws = at::empty({wbytes}, input.options().dtype(at::kByte));
    p.workspace = ws.data_ptr();
    p.workspace_bytes = wbytes;
  }
  check_rc(woq_hip_linear(&p), "woq_linear");
  return out;
}

// NF4 codes -> dense weight: t uint8 [N, K/2] (two codes per byte, low nibble = even k), scales [N, K/G]
// (or [N]); out = table[code] * scale in out_dtype (dequantize_nf4, csrc/cpu/aten/Linear.cpp:804-811,
// csrc/cpu/aten/utils/woq_utils.h:165-262).
static Tensor dequantize_nf4(const Tensor& t_in, const Tensor& scales_in, int64_t group_size, at::ScalarType out_dtype) {
  require_gpu_input(t_in, "torch_ipex::dequantize_nf4");
  TORCH_CHECK(t_in.dim() == 2 && (t_in.scalar_type() == at::kByte || t_in.scalar_type() == at::kChar),
              "dequantize_nf4: expected a 2-D uint8 tensor of packed codes");
  TORCH_CHECK(out_dtype == at::kFloat || out_dtype == at::kHalf || out_dtype == at::kBFloat16,
              "dequantize_nf4: out_dtype must be float, half or bfloat16");
  const Tensor t = t_in.contiguous().view(at::kByte);
  const int64_t N = t.size(0), K = t.size(1) * 2;
  Tensor s = scales_in.to(t.device()).to(at::kFloat);
  s = group_size > 0 ? s.reshape({N, -1}) : s.reshape({N, 1});
  TORCH_CHECK(group_size <= 0 || s.size(1) == (K + group_size - 1) / group_size,
              "dequantize_nf4: scales do not match the group size");
  const Tensor packed = pack_weight(t, WOQ_HIP_DTYPE_NF4, N, K);
  const PackedQParams q = pack_qparams(s, c10::nullopt, WOQ_HIP_DTYPE_NF4);
  return dequant_weight(packed, WOQ_HIP_DTYPE_NF4, N, K, q.s32, c10::nullopt, group_size, out_dtype);
}

// ---- autocast (csrc/cpu/aten/Linear.cpp:874-905): the input is cast to the autocast dtype, the
// prepacked arguments are left alone ----
static Tensor autocast_input(const Tensor& input) {
  return at::autocast::cached_cast(at::autocast::get_autocast_dtype(at::kCUDA), input, at::kCUDA);
}

static Tensor ipex_woq_linear_autocast(const Tensor& input, const Tensor& W_prepack) {
  c10::impl::ExcludeDispatchKeyGuard no_autocast(c10::DispatchKey::AutocastCUDA);
  return ipex_woq_linear(autocast_input(input), W_prepack);
}

template <int FUSION>
static Tensor woq_linear_unary_autocast(const Tensor& input, const Tensor& W_prepack) {
  c10::impl::ExcludeDispatchKeyGuard no_autocast(c10::DispatchKey::AutocastCUDA);
  return woq_linear_unary<FUSION>(autocast_input(input), W_prepack);
}

template <int FUSION, int NOTHERS>
static Tensor woq_linear_binary_autocast(const Tensor& input, const Tensor& W_prepack, const std::vector<Tensor>& others) {
  c10::impl::ExcludeDispatchKeyGuard no_autocast(c10::DispatchKey::AutocastCUDA);
  return woq_linear_binary<FUSION, NOTHERS>(autocast_input(input), W_prepack, others);
}

static Tensor woq_linear_v2_autocast(const Tensor& input, const Tensor& qweight, c10::string_view weight_dtype,
                                     std::vector<int64_t> weight_shape, std::vector<Tensor> weight_scales,
                                     optional<std::vector<Tensor>> weight_zeros, optional<std::vector<Tensor>> bias,
                                     optional<Tensor> g_idx, int64_t group_size, int64_t lowp_mode,
                                     int64_t act_quant_mode, optional<Tensor> compensation) {
  c10::impl::ExcludeDispatchKeyGuard no_autocast(c10::DispatchKey::AutocastCUDA);
  return woq_linear_v2(autocast_input(input), qweight, weight_dtype, std::move(weight_shape), std::move(weight_scales),
                       std::move(weight_zeros), std::move(bias), std::move(g_idx), group_size, lowp_mode,
                       act_quant_mode, std::move(compensation));
}

}  // namespace woq_torch

using namespace woq_torch;

TORCH_LIBRARY_FRAGMENT(ipex_prepack, m) {
  m.class_<WoqLinearOpContext>("WoqLinearOpContext")
      .def_pickle(
          [](const c10::intrusive_ptr<WoqLinearOpContext>& ctx) -> WoqLinearOpContext::State {  // __getstate__
            return ctx->get_state();
          },
          [](WoqLinearOpContext::State state) -> c10::intrusive_ptr<WoqLinearOpContext> {  // __setstate__
            return weight_only_qlinear_prepack(std::move(std::get<0>(state)), std::get<1>(state),
                                               std::move(std::get<2>(state)), std::move(std::get<3>(state)),
                                               std::move(std::get<4>(state)), std::move(std::get<5>(state)),
                                               std::move(std::get<6>(state)), std::get<7>(state), std::get<8>(state),
                                               std::get<9>(state), std::get<10>(state), std::get<11>(state));
          })
      .def("get_weight", &WoqLinearOpContext::get_weight)
      .def("get_bias", &WoqLinearOpContext::get_bias)
      .def("get_scales", &WoqLinearOpContext::get_scales)
      .def("get_zero_points", &WoqLinearOpContext::get_zero_points)
      .def("get_weight_shape", &WoqLinearOpContext::get_weight_shape)
      .def("kernel_pointers", &WoqLinearOpContext::kernel_pointers)
      .def("get_g_idx", &WoqLinearOpContext::get_g_idx)
      .def("get_cached_weight", &WoqLinearOpContext::get_cached_weight)
      .def("get_cached_compensation", &WoqLinearOpContext::get_cached_compensation)
      .def("pack", &WoqLinearOpContext::pack)
      .def("to_public", &WoqLinearOpContext::to_public)
      .def("get_data_handle", &WoqLinearOpContext::get_data_handle)
      .def("load_from_ctx", &WoqLinearOpContext::load_from_ctx);
  m.def(
      "weight_only_qlinear_prepack(Tensor W, int W_dtype, int[] W_shape, Tensor scales, Tensor? zero_points, Tensor? B, "
      "Tensor? g_idx, int? batch_size, int group_size, int lowp_mode, int act_quant_mode, bool "
      "cache_weight_for_large_batch = False) -> __torch__.torch.classes.ipex_prepack.WoqLinearOpContext");
  m.def(
      "weight_only_qlinear_prepack_int4(Tensor W, Tensor scales, Tensor? zeros, Tensor? B, Tensor? g_idx, int? batch_size, "
      "int group_size, int lowp_mode, int act_quant_mode, bool cache_weight_for_large_batch = False, int weight_format = 0) "
      "-> __torch__.torch.classes.ipex_prepack.WoqLinearOpContext");
  m.def(
      "woq_linear_pack_weight(Tensor W, str W_dtype, int[] W_shape, Tensor scales, Tensor? zero_points, Tensor? B, "
      "Tensor? g_idx, int group_size, int lowp_mode) -> (Tensor, Tensor[], Tensor[]?, Tensor[]?, Tensor?)");
  m.def("woq_linear_unpack_weight(Tensor W, str W_dtype, int[] W_shape, int lowp_mode) -> Tensor");
  // no counterpart in the reference: see g_context_epoch
  m.def("woq_context_epoch() -> int", []() -> int64_t { return g_context_epoch.load(); });
}

// The prepack ops take checkpoint tensors wherever they live (the reference registers them for CPU
// tensors, RegisterOpContextClass.cpp:214-222) and put the result on the GPU.
TORCH_LIBRARY_IMPL(ipex_prepack, CompositeExplicitAutograd, m) {
  m.impl("weight_only_qlinear_prepack", TORCH_FN(weight_only_qlinear_prepack));
  m.impl("weight_only_qlinear_prepack_int4", TORCH_FN(weight_only_qlinear_prepack_int4));
  m.impl("woq_linear_pack_weight", TORCH_FN(woq_linear_pack_weight));
  m.impl("woq_linear_unpack_weight", TORCH_FN(woq_linear_unpack_weight));
}

TORCH_LIBRARY_FRAGMENT(torch_ipex, m) {
  m.def("ipex_woq_linear(Tensor input, Tensor W_prepack) -> Tensor");
  m.def("woq_linear_gelu(Tensor input, Tensor W_prepack) -> Tensor");
  m.def("woq_linear_new_gelu(Tensor input, Tensor W_prepack) -> Tensor");
  m.def("woq_linear_relu(Tensor input, Tensor W_prepack) -> Tensor");
  m.def("woq_linear_silu(Tensor input, Tensor W_prepack) -> Tensor");
  m.def("woq_linear_add(Tensor input, Tensor W_prepack, Tensor[] others) -> Tensor");
  m.def("woq_linear_add_add(Tensor input, Tensor W_prepack, Tensor[] others) -> Tensor");
  m.def("woq_linear_mul(Tensor input, Tensor W_prepack, Tensor[] others) -> Tensor");
  // the reference infers this schema from the C++ signature (csrc/utils/CustomOperatorRegistration.h:37-53):
  // positional arguments only
  m.def(
      "woq_linear(Tensor _0, Tensor _1, str _2, int[] _3, Tensor[] _4, Tensor[]? _5, Tensor[]? _6, Tensor? _7, int _8, "
      "int _9, int _10, Tensor? _11 = None) -> Tensor");
  m.def("dequantize_nf4(Tensor t, Tensor scales, int group_size, ScalarType out_dtype) -> Tensor");
  // (csrc/cpu/aten/MoE.cpp:455-472; output is accumulated into and returned)
  m.def(
      "mixtral_moe_woq(Tensor hidden_states, Tensor top_x, Tensor idx, Tensor gate_wei, Tensor up_wei, "
      "Tensor down_wei, Tensor routing_weights, Tensor(a!) output, bool is_distributed) -> Tensor(a!)");
  m.def(
      "deepseek_moe_woq(Tensor hidden_states, Tensor topk_ids, "
      "__torch__.torch.classes.ipex_prepack.WoqLinearOpContext[] gate_ctx, "
      "__torch__.torch.classes.ipex_prepack.WoqLinearOpContext[] up_ctx, "
      "__torch__.torch.classes.ipex_prepack.WoqLinearOpContext[] down_ctx, "
      "Tensor routing_weights, bool is_distributed) -> Tensor");
}

TORCH_LIBRARY_IMPL(torch_ipex, CUDA, m) {
  m.impl("ipex_woq_linear", TORCH_FN(ipex_woq_linear));
  m.impl("woq_linear_gelu", TORCH_FN(woq_linear_unary<WOQ_HIP_FUSE_GELU_ERF>));
  m.impl("woq_linear_new_gelu", TORCH_FN(woq_linear_unary<WOQ_HIP_FUSE_GELU_TANH>));
  m.impl("woq_linear_relu", TORCH_FN(woq_linear_unary<WOQ_HIP_FUSE_RELU>));
  m.impl("woq_linear_silu", TORCH_FN(woq_linear_unary<WOQ_HIP_FUSE_SILU>));
  m.impl("woq_linear_add", TORCH_FN((woq_linear_binary<WOQ_HIP_FUSE_ADD, 1>)));
  m.impl("woq_linear_add_add", TORCH_FN((woq_linear_binary<WOQ_HIP_FUSE_ADD_ADD, 2>)));
  m.impl("woq_linear_mul", TORCH_FN((woq_linear_binary<WOQ_HIP_FUSE_MUL, 1>)));
  m.impl("woq_linear", TORCH_FN(woq_linear_v2));
  m.impl("dequantize_nf4", TORCH_FN(dequantize_nf4));
  m.impl("deepseek_moe_woq", TORCH_FN(deepseek_moe_woq));
}

// The handles of mixtral_moe_woq are CPU tensors beside GPU activations, so no backend key can be computed from the
// arguments alone: registered for every backend, it checks the device of hidden_states itself.  (The Python package
// registers a CUDA kernel in front of it that also resolves the handles of its ctypes contexts.)
TORCH_LIBRARY_IMPL(torch_ipex, CompositeExplicitAutograd, m) {
  m.impl("mixtral_moe_woq", TORCH_FN(mixtral_moe_woq));
}

// Tensors on the CPU reach these kernels, whose only work is the error: this build has no CPU path.
static Tensor refuse_cpu_2(const Tensor& input, const Tensor&) {
  require_gpu_input(input, "torch_ipex::ipex_woq_linear / woq_linear_<post-op>");
  return input;
}
static Tensor refuse_cpu_3(const Tensor& input, const Tensor&, const std::vector<Tensor>&) {
  require_gpu_input(input, "torch_ipex::woq_linear_<post-op>");
  return input;
}

TORCH_LIBRARY_IMPL(torch_ipex, CPU, m) {
  for (const char* name : {"ipex_woq_linear", "woq_linear_gelu", "woq_linear_new_gelu", "woq_linear_relu", "woq_linear_silu"})
    m.impl(name, TORCH_FN(refuse_cpu_2));
  for (const char* name : {"woq_linear_add", "woq_linear_add_add", "woq_linear_mul"}) m.impl(name, TORCH_FN(refuse_cpu_3));
  m.impl("woq_linear", TORCH_FN(woq_linear_v2));      // raises on its CPU input
  m.impl("dequantize_nf4", TORCH_FN(dequantize_nf4));  // raises on its CPU input
}

TORCH_LIBRARY_IMPL(torch_ipex, AutocastCUDA, m) {
  m.impl("ipex_woq_linear", TORCH_FN(ipex_woq_linear_autocast));
  m.impl("woq_linear_gelu", TORCH_FN(woq_linear_unary_autocast<WOQ_HIP_FUSE_GELU_ERF>));
  m.impl("woq_linear_new_gelu", TORCH_FN(woq_linear_unary_autocast<WOQ_HIP_FUSE_GELU_TANH>));
  m.impl("woq_linear_relu", TORCH_FN(woq_linear_unary_autocast<WOQ_HIP_FUSE_RELU>));
  m.impl("woq_linear_silu", TORCH_FN(woq_linear_unary_autocast<WOQ_HIP_FUSE_SILU>));
  m.impl("woq_linear_add", TORCH_FN((woq_linear_binary_autocast<WOQ_HIP_FUSE_ADD, 1>)));
  m.impl("woq_linear_add_add", TORCH_FN((woq_linear_binary_autocast<WOQ_HIP_FUSE_ADD_ADD, 2>)));
  m.impl("woq_linear_mul", TORCH_FN((woq_linear_binary_autocast<WOQ_HIP_FUSE_MUL, 1>)));
  m.impl("woq_linear", TORCH_FN(woq_linear_v2_autocast));
}

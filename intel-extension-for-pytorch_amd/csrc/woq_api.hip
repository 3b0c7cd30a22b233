// extern "C" entry points: argument validation, regime / kernel selection, launches.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>

#include "woq_common.h"
#include "woq_internal.h"

namespace woq {

static thread_local char g_err[512] = "";
// name of the kernel this thread launched last (check_launch is called once per launch with it)
static thread_local const char* g_last_kernel = "";

int set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return 1;
}

int check_launch(const char* what) {
  g_last_kernel = what;
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return set_error("%s: %s", what, hipGetErrorString(err));
  return 0;
}

static bool valid_wdtype(int d) {
  return d == WOQ_HIP_DTYPE_INT8 || d == WOQ_HIP_DTYPE_INT4 || d == WOQ_HIP_DTYPE_NF4 || d == WOQ_HIP_DTYPE_FP8;
}
static bool wdtype_is_8bit(int d) { return d == WOQ_HIP_DTYPE_INT8 || d == WOQ_HIP_DTYPE_FP8; }

// Rows below which lowp_mode BF16 computes in fp16: IPEX_WOQ_SMALL_BATCH_THRESHOLD, default 5, read once
// (csrc/cpu/aten/utils/woq.h:24, used at csrc/cpu/aten/kernels/WoqLinearKrnl.cpp:77, 93).
static int small_batch_threshold() {
  static const int value = [] {
    const char* env = getenv("IPEX_WOQ_SMALL_BATCH_THRESHOLD");
    if (!env || !*env) return 5;
    char* end = nullptr;
    const long v = strtol(env, &end, 10);
    return (end && *end == '\0' && v >= 0 && v <= 1 << 20) ? (int)v : 5;
  }();
  return value;
}

// Rows from which lowp_mode BF16 uses the dense copy of the weight when the caller holds one:
// IPEX_WOQ_WEIGHT_CACHE_BATCH_THRESHOLD, default 64, read once (csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:17-18, 517).
static int weight_cache_batch_threshold() {
  static const int value = [] {
    const char* env = getenv("IPEX_WOQ_WEIGHT_CACHE_BATCH_THRESHOLD");
    if (!env || !*env) return 64;
    char* end = nullptr;
    const long v = strtol(env, &end, 10);
    return (end && *end == '\0' && v >= 0 && v <= 1 << 20) ? (int)v : 64;
  }();
  return value;
}

}  // namespace woq

using namespace woq;

extern "C" {

const char* woq_hip_last_error(void) { return g_err; }

int woq_hip_abi_version(void) { return 3; }

int woq_hip_weight_cache_batch_threshold(void) { return weight_cache_batch_threshold(); }

int64_t woq_hip_dense_weight_bytes(int32_t weight_dtype, int64_t N, int64_t K) {
  if (!valid_wdtype(weight_dtype) || N <= 0 || K <= 0 || K % 128 != 0) return 0;
  const int64_t bytes = woq_hip_padded_n(N) * K * 2;
  return bytes < (int64_t)1 << 31 ? bytes : 0;
}

int woq_hip_dense_weight(const void* qweight, int32_t weight_dtype, int64_t N, int64_t K, const void* scales_bf16,
                         const uint8_t* zeros_u8, int64_t group_size, void* dense, void* stream) {
  if (!valid_wdtype(weight_dtype)) return set_error("dense_weight: unsupported weight dtype %d", weight_dtype);
  if (woq_hip_dense_weight_bytes(weight_dtype, N, K) == 0)
    return set_error("dense_weight: no dense copy for N=%lld K=%lld (K must be a multiple of 128, the copy below 2 GiB)",
                     (long long)N, (long long)K);
  if (!qweight || !scales_bf16 || !dense) return set_error("dense_weight: null pointer");
  if (group_size > 0 && group_size % 32 != 0) return set_error("dense_weight: group_size must be a multiple of 32");
  const int64_t G = group_size > 0 ? group_size : woq_hip_padded_k(weight_dtype, K);
  return launch_dense_weight(qweight, weight_dtype, N, K, (const uint16_t*)scales_bf16, zeros_u8, G, dense,
                             (hipStream_t)stream);
}

int woq_hip_small_batch_threshold(void) { return small_batch_threshold(); }

const char* woq_hip_last_kernel(void) { return g_last_kernel; }

int64_t woq_hip_padded_n(int64_t N) { return (N + kTileN - 1) / kTileN * kTileN; }

int64_t woq_hip_padded_k(int weight_dtype, int64_t K) {
  const int tk = wdtype_is_8bit(weight_dtype) ? kTileK8 : kTileK4;
  return (K + tk - 1) / tk * tk;
}

int64_t woq_hip_packed_weight_bytes(int weight_dtype, int64_t N, int64_t K) {
  const int tk = wdtype_is_8bit(weight_dtype) ? kTileK8 : kTileK4;
  return woq_hip_padded_n(N) / kTileN * (woq_hip_padded_k(weight_dtype, K) / tk) * kTileBytes;
}

int woq_hip_pack_weight(const void* plain, int weight_dtype, int64_t N, int64_t K, void* packed,
                        void* stream) {
  if (!valid_wdtype(weight_dtype)) return set_error("pack_weight: unsupported weight dtype %d", weight_dtype);
  if (N < 0 || K < 0) return set_error("pack_weight: negative shape");
  if ((N > 0 && K > 0) && (!plain || !packed)) return set_error("pack_weight: null pointer");
  return launch_pack_weight(plain, weight_dtype, N, K, packed, (hipStream_t)stream);
}

int woq_hip_unpack_weight(const void* packed, int weight_dtype, int64_t N, int64_t K, void* plain,
                          void* stream) {
  if (!valid_wdtype(weight_dtype)) return set_error("unpack_weight: unsupported weight dtype %d", weight_dtype);
  if (N < 0 || K < 0) return set_error("unpack_weight: negative shape");
  if ((N > 0 && K > 0) && (!plain || !packed)) return set_error("unpack_weight: null pointer");
  return launch_unpack_weight(packed, weight_dtype, N, K, plain, (hipStream_t)stream);
}

int woq_hip_pack_qparams(const float* scales, const float* zeros, int weight_dtype, int64_t N, int64_t KG,
                         float* scales_f32, void* scales_f16, void* scales_bf16, uint8_t* zeros_u8,
                         uint32_t* scale_zero_f16x2, uint32_t* scale_zero_bf16, void* stream) {
  if (!valid_wdtype(weight_dtype)) return set_error("pack_qparams: unsupported weight dtype %d", weight_dtype);
  if (N < 0 || KG < 1) return set_error("pack_qparams: bad shape N=%lld KG=%lld", (long long)N, (long long)KG);
  if (N > 0 && (!scales || !scales_f32 || !scales_f16 || !scales_bf16))
    return set_error("pack_qparams: null scales pointer");
  if (zeros && !zeros_u8) return set_error("pack_qparams: zeros given but zeros_u8 is null");
  return launch_pack_qparams(scales, zeros, weight_dtype, N, KG, scales_f32, scales_f16, scales_bf16, zeros_u8,
                             scale_zero_f16x2, scale_zero_bf16, (hipStream_t)stream);
}

int woq_hip_unpack_int4_zeros(const int32_t* zp32, int64_t rows, int64_t cols, int64_t cols_zp32, float* out,
                              void* stream) {
  if (rows < 0 || cols < 0 || cols_zp32 * 8 < cols)
    return set_error("unpack_int4_zeros: bad shape rows=%lld cols=%lld cols_zp32=%lld", (long long)rows,
                     (long long)cols, (long long)cols_zp32);
  return launch_unpack_int4_zeros(zp32, rows, cols, cols_zp32, out, (hipStream_t)stream);
}

int woq_hip_dynamic_quant(const void* x, int x_dtype, int64_t M, int64_t K, int64_t quant_block_k,
                          int act_quant_mode, void* q, float* scales, int32_t* zps, void* stream) {
  if (act_quant_mode < 0 || act_quant_mode > 7) return set_error("dynamic_quant: bad act_quant_mode %d", act_quant_mode);
  if (x_dtype < 0 || x_dtype > 2) return set_error("dynamic_quant: bad x_dtype %d", x_dtype);
  if (K % 8 != 0) return set_error("dynamic_quant: K (%lld) must be a multiple of 8", (long long)K);
  if (act_quant_mode < 4 && !zps) return set_error("dynamic_quant: asymmetric mode needs a zps buffer");
  return launch_dynamic_quant(x, x_dtype, M, K, K, quant_block_k, act_quant_mode, q, scales, zps,
                              (hipStream_t)stream);
}

int64_t woq_hip_int8_block_k(int64_t group_size, int64_t K) {
  int64_t bk = group_size > 0 ? (group_size < 128 ? group_size : 128) : 128;
  while (bk > 0 && K % bk != 0) bk /= 2;
  return bk;
}

int64_t woq_hip_linear_workspace_bytes(int64_t M, int64_t K, int32_t lowp_mode, int32_t act_quant_mode,
                                       int64_t group_size) {
  if (lowp_mode != WOQ_HIP_LOWP_INT8) return 0;
  (void)act_quant_mode;
  const int64_t kp = (K + 127) / 128 * 128;
  const int64_t qbytes = (M * kp + 255) / 256 * 256;
  int64_t qbk = group_size > 0 ? group_size : woq_hip_int8_block_k(-1, K);
  if (qbk <= 0) qbk = 1;
  const int64_t Kc = (K + qbk - 1) / qbk;
  return qbytes + (M * Kc + 64) * 8;
}

int64_t woq_hip_linear_split_k_workspace_bytes(int64_t M, int64_t N) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64) {
    // prefill GEMM, 64 x 128 tiles, up to four workgroups per tile while the tiles alone fill less than
    // half of the chip
    const int64_t tiles = ((M + 63) / 64) * ((woq_hip_padded_n(N) + 127) / 128);
    return tiles <= 128 ? 4 * tiles * 64 * 128 * (int64_t)sizeof(float) : 0;
  }
  if (M > 32) return 0;
  const int64_t NT = woq_hip_padded_n(N) / kTileN;
  if (NT > 4 * kSplitKCounters) return 0;
  return decode_dq_splitk_bytes(M, NT, kSplitKMax);
}

int64_t woq_hip_linear_auto_split_k_workspace_bytes(int64_t M, int64_t K, int64_t N, int32_t lowp_mode) {
  const bool int8 = lowp_mode == WOQ_HIP_LOWP_INT8;
  // the dequantizing decode kernel (launch_decode_dq) and the 64 x 128 tiles of the prefill GEMMs (pick_splits)
  const bool decode = !int8 && M >= 5 && M <= 32 && K >= 8192 && N <= 4096;
  const bool prefill = M > 64 && K >= 4096 && M * N <= 1048576;
  return decode || prefill ? woq_hip_linear_split_k_workspace_bytes(M, N) : 0;
}

int woq_hip_linear(const woq_hip_linear_params* p) {
  if (!p) return set_error("woq_linear: null params");
  if (p->struct_size != sizeof(woq_hip_linear_params))
    return set_error("woq_linear: struct_size %u does not match this library (%zu)", p->struct_size,
                     sizeof(woq_hip_linear_params));
  if (!valid_wdtype(p->weight_dtype)) return set_error("woq_linear: unsupported weight dtype %d", p->weight_dtype);
  if (p->M < 0 || p->K <= 0 || p->N <= 0)
    return set_error("woq_linear: bad shape M=%lld K=%lld N=%lld", (long long)p->M, (long long)p->K, (long long)p->N);
  if (p->x_dtype != WOQ_HIP_ACT_BF16 && p->x_dtype != WOQ_HIP_ACT_FP16 && p->x_dtype != WOQ_HIP_ACT_FP32)
    return set_error("woq_linear: bad x_dtype %d", p->x_dtype);
  if (p->out_dtype != p->x_dtype && p->out_dtype != WOQ_HIP_ACT_FP32) {
    const bool both16 = p->x_dtype != WOQ_HIP_ACT_FP32 &&
                        (p->out_dtype == WOQ_HIP_ACT_FP16 || p->out_dtype == WOQ_HIP_ACT_BF16);
    if (!both16 || p->fusion != WOQ_HIP_FUSE_NONE)
      return set_error("woq_linear: out_dtype must equal x_dtype or be fp32 (without a post-op it may be the "
                       "other 16-bit type)");
  }
  if (p->lowp_mode < 0 || p->lowp_mode > 3) return set_error("woq_linear: bad lowp_mode %d", p->lowp_mode);
  if (p->M == 0) return 0;
  if (!p->x || !p->qweight || !p->out || !p->scales_f32 || !p->scales_f16 || !p->scales_bf16)
    return set_error("woq_linear: null pointer argument");
  if (p->group_size > 0 && p->group_size % 32 != 0)
    return set_error("woq_linear: group_size %lld must be a multiple of 32 (or <= 0 for per-channel)",
                     (long long)p->group_size);
  switch (p->fusion) {
    case WOQ_HIP_FUSE_NONE: case WOQ_HIP_FUSE_GELU_ERF: case WOQ_HIP_FUSE_GELU_TANH:
    case WOQ_HIP_FUSE_RELU: case WOQ_HIP_FUSE_SILU:
      break;
    case WOQ_HIP_FUSE_ADD: case WOQ_HIP_FUSE_MUL:
      if (!p->others[0]) return set_error("woq_linear: fusion 0x%x needs others[0]", p->fusion);
      break;
    case WOQ_HIP_FUSE_ADD_ADD:
      if (!p->others[0] || !p->others[1]) return set_error("woq_linear: add_add needs two others");
      break;
    default:
      return set_error("woq_linear: unexpected fusion type 0x%x", p->fusion);
  }
  if (p->out_dtype == WOQ_HIP_ACT_FP32 && p->x_dtype != WOQ_HIP_ACT_FP32 && p->fusion != WOQ_HIP_FUSE_NONE)
    return set_error("woq_linear: the fp32 accumulator output does not take a post-op");

  const int wbits = wdtype_is_8bit(p->weight_dtype) ? 8 : 4;
  const int tk = wbits == 4 ? kTileK4 : kTileK8;
  const int64_t NT = woq_hip_padded_n(p->N) / kTileN;
  const int64_t KT = woq_hip_padded_k(p->weight_dtype, p->K) / tk;
  const int64_t Kpad = KT * tk;
  const int64_t G = p->group_size > 0 ? p->group_size : Kpad;
  const int64_t KG = p->group_size > 0 ? (p->K + G - 1) / G : 1;
  hipStream_t st = (hipStream_t)p->stream;

  const bool nf4 = p->weight_dtype == WOQ_HIP_DTYPE_NF4;
  if (nf4 && p->zeros_u8) return set_error("woq_linear: symmetric quantization is required for NF4 weights");
  const bool fp8 = p->weight_dtype == WOQ_HIP_DTYPE_FP8;
  if (fp8 && p->zeros_u8) return set_error("woq_linear: FP8 weights take no zero points");
  if (fp8 && p->lowp_mode == WOQ_HIP_LOWP_INT8)
    return set_error("woq_linear: lowp_mode INT8 does not take FP8 weights");
  int lowp = p->lowp_mode;
  if (lowp == WOQ_HIP_LOWP_INT8) {
    const int64_t bk = woq_hip_int8_block_k(p->group_size, p->K);
    const bool blocks_ok = bk == 32 || bk == 64 || bk == 128;
    const bool mode_ok = p->act_quant_mode >= WOQ_HIP_QUANT_A_PER_TENSOR &&
                         p->act_quant_mode <= WOQ_HIP_QUANT_A_PER_M_K_BLOCK_SYM;
    if (p->weight_dtype == WOQ_HIP_DTYPE_INT8 && p->zeros_u8)
      return set_error("woq_linear: symmetric quantization is required for INT8 weights with lowp_mode INT8");
    if (p->x_dtype == WOQ_HIP_ACT_FP32 || !blocks_ok) {
      // Shapes the blocked int8 kernel does not take run unquantized in the activation dtype,
      // which is what the reference's fallback does for lowp_mode INT8
      // (csrc/cpu/aten/kernels/WoqInt8GemmAPerMKrnl.cpp:143-169).
      lowp = WOQ_HIP_LOWP_NONE;
    } else if (!mode_ok) {
      return set_error("woq_linear: lowp_mode INT8 needs an act_quant_mode in 0..7, got %d", p->act_quant_mode);
    } else {
      Int8Args a;
      a.x = p->x; a.x_dtype = p->x_dtype; a.M = p->M; a.K = p->K; a.N = p->N; a.NT = NT; a.KT = KT;
      a.qweight = (const uint8_t*)p->qweight; a.wbits = wbits; a.scales = p->scales_f32;
      a.zeros = p->zeros_u8; a.G = G; a.KG = KG; a.bias = p->bias; a.act_quant_mode = p->act_quant_mode;
      a.fusion = p->fusion; a.other0 = p->others[0]; a.other1 = p->others[1]; a.out = p->out;
      a.out_dtype = p->out_dtype; a.workspace = p->workspace; a.workspace_bytes = p->workspace_bytes;
      a.split_k_counters = p->split_k_counters;
      a.debug_block_sums = p->debug_block_sums;
      a.nf4 = nf4 ? 1 : 0;
      a.group_size = p->group_size;
      return launch_int8_linear(a, st);
    }
  }

  // Floating-point regimes (csrc/cpu/aten/kernels/WoqLinearKrnl.cpp:75-112; the small-batch threshold
  // is the environment's IPEX_WOQ_SMALL_BATCH_THRESHOLD, 5 by default, csrc/cpu/aten/utils/woq.h:24).
  int regime;
  if (lowp == WOQ_HIP_LOWP_FP16 || (lowp == WOQ_HIP_LOWP_NONE && p->x_dtype == WOQ_HIP_ACT_FP16) ||
      (lowp == WOQ_HIP_LOWP_BF16 && p->M < small_batch_threshold())) {
    regime = kRegimeF16;
  } else if ((lowp == WOQ_HIP_LOWP_NONE && p->x_dtype == WOQ_HIP_ACT_BF16) || lowp == WOQ_HIP_LOWP_BF16) {
    regime = kRegimeBF16;
  } else if (lowp == WOQ_HIP_LOWP_NONE && p->x_dtype == WOQ_HIP_ACT_FP32) {
    // fp32 compute (csrc/cpu/aten/kernels/WoqLinearKrnl.cpp:142-158)
    if (p->force_kernel != 0) return set_error("woq_linear: fp32 compute has one kernel; force_kernel must be 0");
    Fp32Args a;
    a.x = (const float*)p->x; a.M = p->M; a.K = p->K; a.N = p->N; a.NT = NT; a.KT = KT;
    a.qweight = (const uint8_t*)p->qweight; a.scales = p->scales_f32; a.zeros = p->zeros_u8;
    a.G = G; a.KG = KG; a.bias = p->bias; a.fusion = p->fusion;
    a.other0 = p->others[0]; a.other1 = p->others[1]; a.out = p->out; a.nf4 = nf4 ? 1 : 0;
    a.fp8 = fp8 ? 1 : 0;
    return launch_fp32(a, wbits, st);
  } else {
    return set_error("woq_linear: lowp_mode %d does not take x_dtype %d", lowp, p->x_dtype);
  }

  FpArgs f;
  f.x = p->x; f.x_dtype = p->x_dtype; f.M = p->M; f.K = p->K; f.N = p->N; f.NT = NT; f.KT = KT;
  f.qweight = (const uint8_t*)p->qweight;
  f.scales = (const uint16_t*)(regime == kRegimeF16 ? p->scales_f16 : p->scales_bf16);
  f.zeros = p->zeros_u8; f.G = G; f.KG = KG; f.bias = p->bias; f.fusion = p->fusion;
  f.other0 = p->others[0]; f.other1 = p->others[1]; f.out = p->out; f.out_dtype = p->out_dtype;
  f.nf4 = nf4 ? 1 : 0;
  f.fp8 = fp8 ? 1 : 0;
  f.szb = (regime == kRegimeBF16 && !nf4 && !fp8) ? p->scale_zero_bf16 : nullptr;
  SplitKScratch scratch;
  if (p->split_k_counters && p->workspace && p->workspace_bytes > 0) {
    scratch.partial = (float*)p->workspace;
    scratch.bytes = p->workspace_bytes;
    scratch.counters = p->split_k_counters;
  }

  int kernel = p->force_kernel;
  // The dense copy (cache_weight_for_large_batch, csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:511-526: lowp_mode
  // BF16, at least the threshold's rows): same operands into the same MFMAs as the kernels below, so same results.
  if (kernel >= 23 && kernel <= 26) {
    if (!p->dense_bf16 || regime != kRegimeBF16 || !gemm_dense_applies(f))
      return set_error("woq_linear: the dense kernel takes dense_bf16, bf16 compute on bf16 activations and "
                       "K %% 128 == 0");
    return launch_gemm_dense(f, p->dense_bf16, wbits, st, kernel == 23 ? 0 : kernel == 24 ? 7 : kernel == 25 ? 4 : 2);
  }
  if (kernel == 0 && p->dense_bf16 && lowp == WOQ_HIP_LOWP_BF16 && regime == kRegimeBF16 &&
      p->M >= weight_cache_batch_threshold() && p->M > 64 && gemm_dense_applies(f)) {
    // ... where it is the faster kernel: against the prefill kernel that dequantizes in registers (a quarter of the
    // bytes for the same MFMAs, and shapes of 64 rows) by the two cost models; weights that kernel does not take
    // (NF4, groups that split a lane's K values) run on the general tiled kernel, which the dense one always beats
    if (!gemm_w4_applies(f, wbits, regime) || gemm_dense_cost(f) < 0.97 * gemm_w4_cost(f, wbits))
      return launch_gemm_dense(f, p->dense_bf16, wbits, st, 0);
  }
  if (nf4) {
    // table lookups instead of the integer decode: the dequantizing decode kernel and the two
    // general kernels carry them
    if (kernel == 0) kernel = decode_dq_applies(f, wbits, regime) ? 7 : (p->M <= 64 ? 1 : 2);
    if (kernel != 1 && kernel != 2 && (kernel < 7 || kernel > 9) && kernel != 13 && kernel != 14 && kernel != 16)
      return set_error("woq_linear: NF4 weights run on kernels 1, 2, 7..9, 13, 14 and 16 only");
  }
  if (kernel == 0 && decode_kernel_applies(f, wbits, regime, p->scale_zero_f16x2))
    return launch_decode(f, p->scale_zero_f16x2, st);
  // 33..64 rows: the decode kernel with four row tiles while its workgroups of four row-blocks fit one
  // generation (up to 1024 row-blocks), the prefill kernel's 64 x 128 tiles beyond (M = 64, 4096 -> 14336 /
  // 16384: 20.7 / 21.2 us against 29 us; 4096 -> 22016 / 28672: 38.5 / 39.3 us against 29.7 / 30.9 us)
  const bool w4 = gemm_w4_applies(f, wbits, regime);
  if (kernel == 0 && decode_dq_applies(f, wbits, regime) && !(p->M > 32 && w4 && p->N > 16384)) kernel = 7;
  if (kernel >= 7 && kernel <= 10) {
    if (!decode_dq_applies(f, wbits, regime))
      return set_error("woq_linear: the dequantizing decode kernel takes M <= 64, K a multiple of the weight tile, a "
                       "power-of-two or per-channel group size and activations in the compute dtype");
    // 7: row-blocks per workgroup and K splits by shape; 8..10: that many row-blocks, K not split
    return launch_decode_dq(f, wbits, regime, st, kernel == 10 ? 4 : kernel - 7, kernel == 7 ? 0 : 1, &scratch);
  }
  if (kernel == 22) {  // three row-blocks per workgroup (they need not divide the row-blocks), K not split
    if (!decode_dq_applies(f, wbits, regime))
      return set_error("woq_linear: the dequantizing decode kernel does not take this problem");
    return launch_decode_dq(f, wbits, regime, st, 3, 1, &scratch);
  }
  if (kernel >= 13 && kernel <= 17) {
    static const int kNtw[5] = {1, 2, 4, 2, 4}, kSplits[5] = {2, 2, 2, 4, 4};
    if (!decode_dq_applies(f, wbits, regime))
      return set_error("woq_linear: the dequantizing decode kernel does not take this problem");
    return launch_decode_dq(f, wbits, regime, st, kNtw[kernel - 13], kSplits[kernel - 13], &scratch);
  }
  if (kernel == 0) {
    if (p->M <= 64)
      kernel = (p->M > 32 && w4 && p->N >= 8192) ? 3 : 1;
    else
      kernel = w4 ? 3 : 2;
  }
  if (kernel == 1 && p->M > 64) return set_error("woq_linear: the small-M kernel takes M <= 64");
  if (kernel == 21) {
    if (!gemm_w4s_applies(f, wbits, regime))
      return set_error("woq_linear: the prefill kernel with the dequantized tile in LDS takes 4-bit integer weights, "
                       "K %% 128 == 0, a power-of-two or per-channel group size and activations in the compute dtype");
    return launch_gemm_w4s(f, regime, st);
  }
  const int w4_shape = kernel == 4 ? 7 : kernel == 5 ? 4 : kernel == 6 ? 2 : kernel == 11 ? 163
                       : (kernel == 12 || kernel == 19 || kernel == 20) ? 42 : 0;
  // forced shapes run unsplit, 19 / 20 split K in two / four; the automatic choice may split
  const int w4_splits = kernel == 19 ? 2 : kernel == 20 ? 4 : kernel == 3 || kernel == 0 ? 0 : 1;
  if ((kernel >= 4 && kernel <= 6) || kernel == 11 || kernel == 12 || kernel == 19 || kernel == 20) kernel = 3;
  if (kernel == 3 && !gemm_w4_applies(f, wbits, regime))
    return set_error("woq_linear: the prefill kernel takes 4-bit integer weights (or 8-bit ones with groups of at "
                     "least 128), K %% 128 == 0, a power-of-two or per-channel group size and activations in the "
                     "compute dtype");
  if (kernel == 1) return launch_small_m(f, wbits, regime, st);
  return kernel == 3 ? launch_gemm_w4(f, wbits, regime, st, w4_shape, w4_splits, &scratch)
                     : launch_gemm(f, wbits, regime, st);
}

int woq_hip_linear_grouped(const woq_hip_linear_params* p, const void* group, int64_t slots) {
  if (!p || !group) return set_error("woq_linear_grouped: null params or group table");
  if (p->struct_size != sizeof(woq_hip_linear_params))
    return set_error("woq_linear_grouped: struct_size %u does not match this library (%zu)", p->struct_size,
                     sizeof(woq_hip_linear_params));
  if (p->weight_dtype != WOQ_HIP_DTYPE_INT4 && p->weight_dtype != WOQ_HIP_DTYPE_INT8)
    return set_error("woq_linear_grouped: INT4 and INT8 weights, got dtype %d", p->weight_dtype);
  if (p->M < 1 || p->M > 64 || p->K <= 0 || p->N <= 0)
    return set_error("woq_linear_grouped: 1..64 rows per slot, got M=%lld K=%lld N=%lld", (long long)p->M, (long long)p->K,
                     (long long)p->N);
  if (p->x_dtype != WOQ_HIP_ACT_BF16 && p->x_dtype != WOQ_HIP_ACT_FP16)
    return set_error("woq_linear_grouped: bf16 or fp16 rows, got x_dtype %d", p->x_dtype);
  if (p->out_dtype != p->x_dtype) return set_error("woq_linear_grouped: out_dtype must equal x_dtype");
  if (p->lowp_mode < 0 || p->lowp_mode > 2) return set_error("woq_linear_grouped: lowp_mode NONE, FP16 or BF16, got %d", p->lowp_mode);
  if (!p->x || !p->out) return set_error("woq_linear_grouped: null pointer argument");
  if (p->group_size > 0 && p->group_size % 32 != 0)
    return set_error("woq_linear_grouped: group_size %lld must be a multiple of 32 (or <= 0 for per-channel)",
                     (long long)p->group_size);
  if (p->fusion != WOQ_HIP_FUSE_NONE && p->fusion != WOQ_HIP_FUSE_SILU && p->fusion != WOQ_HIP_FUSE_MUL)
    return set_error("woq_linear_grouped: post-op none, silu or mul, got 0x%x", p->fusion);
  if (p->fusion == WOQ_HIP_FUSE_MUL && !p->others[0]) return set_error("woq_linear_grouped: mul needs others[0]");
  const int wbits = p->weight_dtype == WOQ_HIP_DTYPE_INT8 ? 8 : 4;
  const int tk = wbits == 4 ? kTileK4 : kTileK8;
  const int64_t NT = woq_hip_padded_n(p->N) / kTileN;
  const int64_t KT = woq_hip_padded_k(p->weight_dtype, p->K) / tk;
  const int64_t G = p->group_size > 0 ? p->group_size : KT * tk;
  const int64_t KG = p->group_size > 0 ? (p->K + G - 1) / G : 1;
  // the regimes of woq_hip_linear (csrc/cpu/aten/kernels/WoqLinearKrnl.cpp:75-112), with M the bound on a slot's rows
  int regime;
  if (p->lowp_mode == WOQ_HIP_LOWP_FP16 || (p->lowp_mode == WOQ_HIP_LOWP_NONE && p->x_dtype == WOQ_HIP_ACT_FP16) ||
      (p->lowp_mode == WOQ_HIP_LOWP_BF16 && p->M < small_batch_threshold()))
    regime = kRegimeF16;
  else
    regime = kRegimeBF16;
  FpArgs f;
  f.x = p->x; f.x_dtype = p->x_dtype; f.M = p->M; f.K = p->K; f.N = p->N; f.NT = NT; f.KT = KT;
  f.qweight = nullptr; f.scales = nullptr; f.zeros = nullptr;  // per expert, from the group table
  f.szb = nullptr;
  f.G = G; f.KG = KG; f.bias = nullptr; f.fusion = p->fusion;
  f.other0 = p->others[0]; f.other1 = nullptr; f.out = p->out; f.out_dtype = p->out_dtype;
  f.nf4 = 0; f.fp8 = 0;
  if (p->scale_zero_f16x2) {
    // up to four routed rows per slot on the integer-weight decode kernels: the group's scales table holds the
    // experts' (fp16 scale, fp16 128 + zero) dword tables
    if (p->M > 4) return set_error("woq_linear_grouped: (scale, zero) dword tables go with at most four rows per slot (M <= 4)");
    f.scales = nullptr;
    if (!decode_kernel_applies(f, wbits, regime, (const uint32_t*)p->scale_zero_f16x2))
      return set_error("woq_linear_grouped: the integer-weight decode kernels take 4-bit weights in groups of 32, 64 or "
                       "128 x 2^k, fp16 compute and K a multiple of 256");
    return launch_decode_grouped(f, (const MoeGroup*)group, slots, (hipStream_t)p->stream);
  }
  return launch_decode_dq_grouped(f, wbits, regime, (const MoeGroup*)group, slots, (hipStream_t)p->stream);
}

int woq_hip_dequant_weight(const void* qweight, int weight_dtype, int64_t N, int64_t K, const float* scales_f32,
                           const uint8_t* zeros_u8, int64_t group_size, void* out, int out_dtype, void* stream) {
  if (!valid_wdtype(weight_dtype)) return set_error("dequant_weight: unsupported weight dtype %d", weight_dtype);
  if (out_dtype < 0 || out_dtype > 2) return set_error("dequant_weight: bad out_dtype %d", out_dtype);
  if (N > 0 && K > 0 && (!qweight || !scales_f32 || !out)) return set_error("dequant_weight: null pointer");
  return launch_dequant_weight(qweight, weight_dtype, N, K, scales_f32, zeros_u8, group_size, out, out_dtype,
                               (hipStream_t)stream);
}

int woq_hip_convert_activations(const void* src, int src_dtype, void* dst, int dst_dtype, int64_t count,
                                void* stream) {
  if (src_dtype < 0 || src_dtype > 2 || dst_dtype < 0 || dst_dtype > 2)
    return set_error("convert_activations: bad dtype %d -> %d", src_dtype, dst_dtype);
  if (count < 0) return set_error("convert_activations: bad count %lld", (long long)count);
  if (count == 0) return 0;
  if (!src || !dst) return set_error("convert_activations: null pointer argument");
  return launch_convert_activations(src, src_dtype, dst, dst_dtype, count, (hipStream_t)stream);
}

int woq_hip_shuffle_activations(const void* x, int x_dtype, int64_t M, int64_t K, const int32_t* src, void* out,
                                void* stream) {
  if (x_dtype < 0 || x_dtype > 2) return set_error("shuffle_activations: bad x_dtype %d", x_dtype);
  if (M < 0 || K < 0) return set_error("shuffle_activations: bad shape M=%lld K=%lld", (long long)M, (long long)K);
  if (M > 0 && K > 0 && (!x || !src || !out)) return set_error("shuffle_activations: null pointer");
  if (x == out && M > 0) return set_error("shuffle_activations: in-place shuffling is not supported");
  return launch_shuffle_activations(x, x_dtype, M, K, src, out, (hipStream_t)stream);
}

int woq_hip_shuffle_int4_weight(const void* plain, int64_t N, int64_t K, const int32_t* src, void* out,
                                void* stream) {
  if (N < 0 || K < 0) return set_error("shuffle_int4_weight: bad shape N=%lld K=%lld", (long long)N, (long long)K);
  if (N > 0 && K > 0 && (!plain || !src || !out)) return set_error("shuffle_int4_weight: null pointer");
  if (plain == out && N > 0) return set_error("shuffle_int4_weight: in-place shuffling is not supported");
  return launch_shuffle_int4_weight(plain, N, K, src, out, (hipStream_t)stream);
}

int woq_hip_moe_gather_rows(const void* x, int x_dtype, int64_t T, int64_t H, const int64_t* rows, int64_t n,
                            void* out, void* stream) {
  if (x_dtype < 0 || x_dtype > 2) return set_error("moe_gather_rows: bad x_dtype %d", x_dtype);
  if (T < 0 || H < 0 || n < 0) return set_error("moe_gather_rows: negative size");
  if (n > 0 && H > 0 && (!x || !rows || !out)) return set_error("moe_gather_rows: null pointer");
  if (n > 0 && T == 0) return set_error("moe_gather_rows: rows requested from an empty tensor");
  return launch_moe_gather_rows(x, x_dtype, T, H, rows, n, out, (hipStream_t)stream);
}

int woq_hip_moe_scale_add_rows(void* out, int dtype, int64_t T, int64_t H, const void* expert_out,
                               const void* routing_weights, int64_t topk, const int64_t* top_x, const int64_t* idx,
                               int64_t n, void* stream) {
  if (dtype < 0 || dtype > 2) return set_error("moe_scale_add_rows: bad dtype %d", dtype);
  if (T < 0 || H < 0 || n < 0 || topk <= 0) return set_error("moe_scale_add_rows: bad size");
  if (n > 0 && H > 0 && (!out || !expert_out || !routing_weights || !top_x || !idx))
    return set_error("moe_scale_add_rows: null pointer");
  if (n > T) return set_error("moe_scale_add_rows: %lld rows for %lld tokens (a token may appear once)", (long long)n,
                              (long long)T);
  return launch_moe_scale_add_rows(out, dtype, T, H, expert_out, routing_weights, topk, top_x, idx, n,
                                   (hipStream_t)stream);
}

int woq_hip_moe_route(const int64_t* topk_ids, int64_t T, int64_t topk, int64_t experts, int64_t split_lo,
                      int64_t split_mid, int use_single, int64_t S, int64_t* x_row, int32_t* slots, int32_t* row_of,
                      int32_t* slot_of, void* stream) {
  if (T < 0 || topk <= 0 || experts <= 0) return set_error("moe_route: bad size");
  if (T * topk > WOQ_HIP_MOE_ROUTE_MAX)
    return set_error("moe_route: at most %d (token, slot) entries, got %lld", WOQ_HIP_MOE_ROUTE_MAX, (long long)(T * topk));
  if (use_single < 0 || use_single > 2) return set_error("moe_route: use_single is 0, 1 or 2");
  // experts that can have tokens; with a slot per sorted position, the positions
  const int64_t need = use_single == 2 ? T * topk : (T * topk < experts ? T * topk : experts);
  if (S < need) return set_error("moe_route: slot tables of %lld entries, %lld experts can have tokens", (long long)S, (long long)need);
  if (T > 0 && (!topk_ids || !x_row || !slots || !row_of || !slot_of)) return set_error("moe_route: null pointer");
  return launch_moe_route(topk_ids, T, topk, experts, split_lo, split_mid, use_single, S, x_row, slots, row_of, slot_of,
                          (hipStream_t)stream);
}

int woq_hip_moe_combine_rows(void* out, int dtype, int64_t T, int64_t H, const void* expert_out,
                             const void* routing_weights, int64_t topk, const int32_t* row_of, const int32_t* slot_of,
                             int accumulate, void* stream) {
  if (dtype < 0 || dtype > 2) return set_error("moe_combine_rows: bad dtype %d", dtype);
  if (T < 0 || H < 0 || topk <= 0) return set_error("moe_combine_rows: bad size");
  if (T > 0 && H > 0 && (!out || !expert_out || !routing_weights || !row_of || !slot_of))
    return set_error("moe_combine_rows: null pointer");
  return launch_moe_combine_rows(out, dtype, T, H, expert_out, routing_weights, topk, row_of, slot_of, accumulate,
                                 (hipStream_t)stream);
}

// ---- woq_hip_linear for callers that cannot allocate ----------------------------------------------
// One array per GPU, resident until the process ends: 512 split-K counters, then the workspace.
constexpr int64_t kNoAllocCounterBytes = kSplitKCounters * (int64_t)sizeof(int32_t);
constexpr int64_t kNoAllocWorkspaceBytes = WOQ_HIP_NOALLOC_MAX_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char scratch[kNoAllocCounterBytes + kNoAllocWorkspaceBytes];

// `scratch` above is a host-side stand-in, not a device address: the address of each GPU's copy comes
// from hipGetSymbolAddress with that GPU current, once per device.
constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static unsigned char* g_scratch_ptr[kMaxDevices] = {};

static int scratch_of_current_device(unsigned char** out, hipStream_t stream) {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return set_error("woq_linear_noalloc: hipGetDevice: %s", hipGetErrorString(err));
  if (dev < 0 || dev >= kMaxDevices) return set_error("woq_linear_noalloc: device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    // The address is looked up once per device, and not under stream capture (the lookup may load the code
    // object, which a capturing stream does not allow): the first call on a device must come before the capture.
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &status) != hipSuccess || status != hipStreamCaptureStatusNone)
      return set_error("woq_linear_noalloc: the first call on a device looks up the resident scratch and cannot be "
                       "captured; call woq_hip_linear_noalloc once on this device before capturing");
    void* ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || !ptr)
      return set_error("woq_linear_noalloc: hipGetSymbolAddress: %s", hipGetErrorString(err));
    g_scratch_ptr[dev] = (unsigned char*)ptr;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

static __global__ void woq_zero_counters_kernel(int32_t* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

int woq_hip_linear_noalloc(const woq_hip_linear_params* p) {
  if (!p) return set_error("woq_linear_noalloc: null params");
  if (p->struct_size != sizeof(woq_hip_linear_params))
    return set_error("woq_linear_noalloc: struct_size %u does not match this library (%zu)", p->struct_size,
                     sizeof(woq_hip_linear_params));
  if (p->workspace || p->workspace_bytes != 0 || p->split_k_counters)
    return set_error("woq_linear_noalloc: workspace and split_k_counters must be null; the library's resident "
                     "scratch takes their place");
  if (p->M < 0 || p->K <= 0 || p->N <= 0)
    return set_error("woq_linear_noalloc: bad shape M=%lld K=%lld N=%lld", (long long)p->M, (long long)p->K,
                     (long long)p->N);
  if (p->M == 0) return woq_hip_linear(p);
  const bool int8 = p->lowp_mode == WOQ_HIP_LOWP_INT8;
  int64_t need = woq_hip_linear_workspace_bytes(p->M, p->K, p->lowp_mode, p->act_quant_mode, p->group_size);
  if (need > kNoAllocWorkspaceBytes)
    return set_error("woq_linear_noalloc: M=%lld K=%lld under lowp_mode INT8 needs %lld bytes of workspace, the "
                     "resident scratch holds %lld; use woq_hip_linear with a workspace of your own",
                     (long long)p->M, (long long)p->K, (long long)need, (long long)kNoAllocWorkspaceBytes);
  // Sharing K between workgroups is an option, not a need: offered for the problems it pays for (few
  // output tiles and a long K) while its scratch fits behind the quantized activations.
  bool split = false;
  {
    const int64_t extra = woq_hip_linear_auto_split_k_workspace_bytes(p->M, p->K, p->N, p->lowp_mode);
    const int64_t base = (need + 255) / 256 * 256;
    if (extra > 0 && base + extra <= kNoAllocWorkspaceBytes) {
      need = base + extra;
      split = true;
    }
  }
  woq_hip_linear_params q = *p;
  if (need > 0) {
    unsigned char* ptr = nullptr;
    if (int rc = scratch_of_current_device(&ptr, (hipStream_t)p->stream)) return rc;
    q.workspace = ptr + kNoAllocCounterBytes;
    q.workspace_bytes = need;
    if (split) {
      // every finished launch leaves the counters at zero; a fill kernel (not a memset node, so that the
      // call can be captured into a HIP graph) makes that hold whatever ran before
      q.split_k_counters = (int32_t*)ptr;
      woq_zero_counters_kernel<<<(kSplitKCounters + 255) / 256, 256, 0, (hipStream_t)p->stream>>>(q.split_k_counters,
                                                                                                  kSplitKCounters);
      if (int rc = check_launch("woq_zero_counters_kernel")) return rc;
    }
  }
  return woq_hip_linear(&q);
}

}  // extern "C"

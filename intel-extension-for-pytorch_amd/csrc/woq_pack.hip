// Weight prepack / unpack and quantization-parameter layout kernels.
//
// The reference blocks weights for AVX-512 / AMX as [N/32][K/Kb][Kb][16] bytes
// (csrc/cpu/aten/kernels/WoqUtilKrnl.cpp:32-249).  Here the unit is what one wave64 fetches
// with a single global_load_dwordx4 per lane: a 1 KiB tile of 16 output rows.  Both
// directions are integer-exact and invertible, as the reference's pack / unpack pair is
// (tests/cpu/test_quantization_default_recipe.py:1848-1854).
#include "woq_common.h"
#include "woq_internal.h"

namespace woq {

// One thread per packed dword.
__global__ void pack_int4_kernel(const uint8_t* __restrict__ plain, uint32_t* __restrict__ packed,
                                 int64_t N, int64_t K, int64_t KT, int64_t total_dwords) {
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= total_dwords) return;
  const int j = gid & 3;
  const int lane = (gid >> 2) & 63;
  const int64_t tile = gid >> 8;
  const int64_t nt = tile / KT, kt = tile % KT;
  const int r = lane & 15, c = lane >> 4;
  const int64_t n = nt * kTileN + r;
  const int64_t kbase = kt * kTileK4 + c * 32 + j * 8;
  const int64_t row_bytes = (K + 1) / 2;
  uint32_t out = 0;
  if (n < N) {
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int64_t k = kbase + 2 * b;
      if (k < K) {
        const uint32_t byte = plain[n * row_bytes + (k >> 1)];
        out |= (byte & 0xFu) << (4 * b);
        if (k + 1 < K) out |= (byte >> 4) << (16 + 4 * b);
      }
    }
  }
  packed[gid] = out;
}

// One thread per plain byte (two K elements).
__global__ void unpack_int4_kernel(const uint32_t* __restrict__ packed, uint8_t* __restrict__ plain,
                                   int64_t N, int64_t K, int64_t KT) {
  const int64_t row_bytes = (K + 1) / 2;
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= N * row_bytes) return;
  const int64_t n = gid / row_bytes, kb = gid % row_bytes;
  const int64_t k = kb * 2;
  const int64_t nt = n / kTileN, kt = k / kTileK4;
  const int r = n % kTileN;
  const int koff = k % kTileK4;
  const int c = koff / 32, j = (koff % 32) / 8, b = (koff % 8) / 2;
  const uint32_t d = packed[((nt * KT + kt) * 64 + (r + 16 * c)) * 4 + j];
  const uint32_t lo = (d >> (4 * b)) & 0xFu;
  const uint32_t hi = (d >> (16 + 4 * b)) & 0xFu;
  plain[gid] = (uint8_t)(lo | (hi << 4));
}

// One thread per packed dword (4 K elements of one row).
// flip = 0x80: int8 values become offset-binary bytes (q + 128), padding is the byte of zero; flip = 0: float8
// bytes are stored as they are, padding is +0.
__global__ void pack_int8_kernel(const int8_t* __restrict__ plain, uint32_t* __restrict__ packed,
                                 int64_t N, int64_t K, int64_t KT, int64_t total_dwords, uint32_t flip) {
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= total_dwords) return;
  const int j = gid & 3;
  const int lane = (gid >> 2) & 63;
  const int64_t tile = gid >> 8;
  const int64_t nt = tile / KT, kt = tile % KT;
  const int r = lane & 15, c = lane >> 4;
  const int64_t n = nt * kTileN + r;
  const int64_t kbase = kt * kTileK8 + c * 16 + j * 4;
  uint32_t out = flip * 0x01010101u;  // the stored byte of zero, four times
  if (n < N) {
    out = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int64_t k = kbase + i;
      const uint32_t u = (k < K) ? ((uint32_t)(uint8_t)plain[n * K + k] ^ flip) : flip;
      out |= u << (8 * i);
    }
  }
  packed[gid] = out;
}

__global__ void unpack_int8_kernel(const uint8_t* __restrict__ packed, int8_t* __restrict__ plain,
                                   int64_t N, int64_t K, int64_t KT, uint32_t flip) {
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= N * K) return;
  const int64_t n = gid / K, k = gid % K;
  const int64_t nt = n / kTileN, kt = k / kTileK8;
  const int r = n % kTileN;
  const int koff = k % kTileK8;
  const int c = koff / 16, i = koff % 16;
  const uint8_t u = packed[((nt * KT + kt) * 64 + (r + 16 * c)) * 16 + i];
  plain[gid] = (int8_t)(u ^ flip);
}

__global__ void pack_qparams_kernel(const float* __restrict__ scales, const float* __restrict__ zeros,
                                    int weight_dtype, int64_t N, int64_t Np, int64_t KG,
                                    float* __restrict__ s32, uint16_t* __restrict__ s16,
                                    uint16_t* __restrict__ sb16, uint8_t* __restrict__ z8,
                                    uint32_t* __restrict__ sz, uint32_t* __restrict__ szb) {
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= Np * KG) return;
  const int r = gid % kTileN;
  const int64_t g = (gid / kTileN) % KG;
  const int64_t nt = gid / (kTileN * KG);
  const int64_t n = nt * kTileN + r;
  float s = 1.0f, z = 0.0f;
  if (n < N) {
    s = scales[n * KG + g];
    if (zeros) z = zeros[n * KG + g];
  }
  s32[gid] = s;
  s16[gid] = f32_to_f16_bits(s);
  sb16[gid] = f32_to_bf16_bits(s);
  if (z8) {
    int zi = (int)z;
    if (weight_dtype == WOQ_HIP_DTYPE_INT8) zi += 128;
    z8[gid] = (uint8_t)zi;
  }
  if (sz) {
    const float zz = 128.0f + (zeros ? z : (n < N ? 8.0f : 0.0f));
    sz[gid] = (uint32_t)f32_to_f16_bits(s) | ((uint32_t)f32_to_f16_bits(zz) << 16);
  }
  if (szb) {
    // what the bf16 kernels subtract from the stored code: the zero point byte as stored (8-bit weights:
    // offset-binary), the code of zero for symmetric weights; 4-bit weights get the 1024 of the fp16 number
    // 1024 + q that their nibbles are read as
    const bool w8 = weight_dtype == WOQ_HIP_DTYPE_INT8;
    const float zc = zeros ? z + (w8 ? 128.0f : 0.0f) : (w8 ? 128.0f : 8.0f);
    szb[gid] = ((uint32_t)f32_to_bf16_bits(s) << 16) | (uint32_t)f32_to_f16_bits(zc + (w8 ? 0.0f : 1024.0f));
  }
}

__global__ void unpack_int4_zeros_kernel(const uint32_t* __restrict__ zp32, int64_t rows, int64_t cols,
                                         int64_t cols_zp32, float* __restrict__ out) {
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= rows * cols) return;
  const int64_t i = gid / cols, j = gid % cols;
  out[gid] = (float)((zp32[i * cols_zp32 + j / 8] >> ((j % 8) * 4)) & 0xFu);
}

// Dense dequantization of a packed weight: one thread per (n, 8 consecutive k).
__global__ void dequant_weight_kernel(const uint8_t* __restrict__ packed, int weight_dtype, int64_t N,
                                      int64_t K, int64_t KT, const float* __restrict__ s32,
                                      const uint8_t* __restrict__ z8, int64_t G, int64_t KG,
                                      void* __restrict__ out, int out_dtype) {
  const int64_t K8 = (K + 7) / 8;
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= N * K8) return;
  const int64_t n = gid / K8, k0 = (gid % K8) * 8;
  const int64_t nt = n / kTileN;
  const int r = n % kTileN;
  const bool fp8 = weight_dtype == WOQ_HIP_DTYPE_FP8;
  const bool w4 = weight_dtype != WOQ_HIP_DTYPE_INT8 && !fp8;
  const int tile_k = w4 ? kTileK4 : kTileK8;
  const int64_t kt = k0 / tile_k;
  const int koff = k0 % tile_k;
  int64_t g = G > 0 ? k0 / G : 0;
  if (g >= KG) g = KG - 1;
  const float s = s32[(nt * KG + g) * kTileN + r];
  float z = 0.0f;
  if (z8)
    z = (float)z8[(nt * KG + g) * kTileN + r];
  else
    z = w4 ? 8.0f : 128.0f;  // symmetric: INT4 stored +8, INT8 bytes are offset-binary
  float w[8];
  if (w4) {
    const int c = koff / 32, j = (koff % 32) / 8;
    const uint32_t d = ((const uint32_t*)packed)[((nt * KT + kt) * 64 + (r + 16 * c)) * 4 + j];
#pragma unroll
    for (int e = 0; e < 8; ++e) w[e] = (float)((d >> (4 * nibble_pos(e))) & 0xFu);
  } else {
    const int c = koff / 16, i0 = koff % 16;
    const uint8_t* p = packed + ((nt * KT + kt) * 64 + (r + 16 * c)) * 16 + i0;
#pragma unroll
    for (int e = 0; e < 8; ++e) w[e] = fp8 ? fp8_e4m3fn_to_f32(p[e]) : (float)p[e];
  }
  const bool nf4 = weight_dtype == WOQ_HIP_DTYPE_NF4;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int64_t k = k0 + e;
    if (k >= K) break;
    // (q - z) first, then the scale, each in fp32 (woq_utils.h:147-161); NF4: table value times
    // scale (woq_utils.h:165-262)
    // float8: the converted byte times the scale (woq.h:728-741)
    const float v = nf4 ? __fmul_rn(kNf4Values[(int)w[e]], s) : fp8 ? __fmul_rn(w[e], s) : __fmul_rn(__fsub_rn(w[e], z), s);
    store_act(out, out_dtype, n * K + k, v);
  }
}

static inline unsigned blocks_for(int64_t n, int bs) { return (unsigned)((n + bs - 1) / bs); }

int launch_pack_weight(const void* plain, int weight_dtype, int64_t N, int64_t K, void* packed,
                       hipStream_t st) {
  const int64_t Np = woq_hip_padded_n(N), Kp = woq_hip_padded_k(weight_dtype, K);
  const bool w8 = weight_dtype == WOQ_HIP_DTYPE_INT8 || weight_dtype == WOQ_HIP_DTYPE_FP8;
  const int tile_k = w8 ? kTileK8 : kTileK4;
  const int64_t KT = Kp / tile_k;
  const int64_t total = (Np / kTileN) * KT * (kTileBytes / 4);
  if (total == 0) return 0;
  if (w8)
    pack_int8_kernel<<<blocks_for(total, 256), 256, 0, st>>>((const int8_t*)plain, (uint32_t*)packed, N, K, KT, total,
                                                             weight_dtype == WOQ_HIP_DTYPE_FP8 ? 0u : 0x80u);
  else
    pack_int4_kernel<<<blocks_for(total, 256), 256, 0, st>>>((const uint8_t*)plain, (uint32_t*)packed,
                                                             N, K, KT, total);
  return check_launch("pack_weight");
}

int launch_unpack_weight(const void* packed, int weight_dtype, int64_t N, int64_t K, void* plain,
                         hipStream_t st) {
  const int64_t Kp = woq_hip_padded_k(weight_dtype, K);
  if (N == 0 || K == 0) return 0;
  if (weight_dtype == WOQ_HIP_DTYPE_INT8 || weight_dtype == WOQ_HIP_DTYPE_FP8) {
    unpack_int8_kernel<<<blocks_for(N * K, 256), 256, 0, st>>>((const uint8_t*)packed, (int8_t*)plain, N, K,
                                                               Kp / kTileK8,
                                                               weight_dtype == WOQ_HIP_DTYPE_FP8 ? 0u : 0x80u);
  } else {
    const int64_t total = N * ((K + 1) / 2);
    unpack_int4_kernel<<<blocks_for(total, 256), 256, 0, st>>>((const uint32_t*)packed, (uint8_t*)plain,
                                                               N, K, Kp / kTileK4);
  }
  return check_launch("unpack_weight");
}

int launch_pack_qparams(const float* scales, const float* zeros, int weight_dtype, int64_t N, int64_t KG,
                        float* s32, void* s16, void* sb16, uint8_t* z8, uint32_t* sz, uint32_t* szb, hipStream_t st) {
  const int64_t Np = woq_hip_padded_n(N);
  const int64_t total = Np * KG;
  if (total == 0) return 0;
  pack_qparams_kernel<<<blocks_for(total, 256), 256, 0, st>>>(scales, zeros, weight_dtype, N, Np, KG, s32,
                                                              (uint16_t*)s16, (uint16_t*)sb16,
                                                              zeros ? z8 : nullptr, sz, szb);
  return check_launch("pack_qparams");
}

int launch_unpack_int4_zeros(const int32_t* zp32, int64_t rows, int64_t cols, int64_t cols_zp32,
                             float* out, hipStream_t st) {
  const int64_t total = rows * cols;
  if (total == 0) return 0;
  unpack_int4_zeros_kernel<<<blocks_for(total, 256), 256, 0, st>>>((const uint32_t*)zp32, rows, cols,
                                                                   cols_zp32, out);
  return check_launch("unpack_int4_zeros");
}

int launch_dequant_weight(const void* qweight, int weight_dtype, int64_t N, int64_t K, const float* s32,
                          const uint8_t* z8, int64_t G, void* out, int out_dtype, hipStream_t st) {
  if (N == 0 || K == 0) return 0;
  const int64_t Kp = woq_hip_padded_k(weight_dtype, K);
  const int tile_k = (weight_dtype == WOQ_HIP_DTYPE_INT8 || weight_dtype == WOQ_HIP_DTYPE_FP8) ? kTileK8 : kTileK4;
  const int64_t KG = G > 0 ? (K + G - 1) / G : 1;
  const int64_t total = N * ((K + 7) / 8);
  dequant_weight_kernel<<<blocks_for(total, 256), 256, 0, st>>>((const uint8_t*)qweight, weight_dtype, N,
                                                                K, Kp / tile_k, s32, z8, G, KG, out,
                                                                out_dtype);
  return check_launch("dequant_weight");
}

// ---- dense bf16 copy for large batches --------------------------------------------------------
// The weight as the bf16 kernels would dequantize it, w = bf16((q - z) * s) with s the bf16 scale
// (csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:430-486 caches the same values, blocked for its GEMM), laid out as
// the MFMA operands of woq_gemm_dense_kernel: [K / 128][NT][4][64] fragments of 16 bytes, fragment (kt, nt, j, lane)
// holding row 16 nt + lane % 16 and the eight K values 128 kt + 8 chunk .. + 7, chunk = 4 (lane / 16) + j for 4-bit
// codes and 8 (j / 2) + 2 (lane / 16) + j % 2 for bytes -- the K values that the same lane and K sub-step of
// woq_gemm_w4_kernel take from the packed tile, so that the two kernels feed identical operands to identical
// instructions.  One thread per fragment.
__global__ void dense_weight_kernel(const uint8_t* __restrict__ packed, int weight_dtype, int64_t NT, int64_t KT128,
                                    int64_t KT, const uint16_t* __restrict__ sb16, const uint8_t* __restrict__ z8,
                                    int64_t G, int64_t KG, u4* __restrict__ out) {
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= KT128 * NT * 256) return;
  const int lane = (int)(gid & 63), j = (int)((gid >> 6) & 3);
  const int64_t nt = (gid >> 8) % NT, kt128 = (gid >> 8) / NT;
  const int r = lane & 15, c = lane >> 4;
  const bool fp8 = weight_dtype == WOQ_HIP_DTYPE_FP8;
  const bool w4 = weight_dtype != WOQ_HIP_DTYPE_INT8 && !fp8;
  const bool nf4 = weight_dtype == WOQ_HIP_DTYPE_NF4;
  const int chunk = w4 ? 4 * c + j : 8 * (j / 2) + 2 * c + (j % 2);
  const int64_t k0 = kt128 * 128 + chunk * 8;
  int64_t g = G > 0 ? k0 / G : 0;
  if (g >= KG) g = KG - 1;
  const float s = bf16_bits_to_f32(sb16[(nt * KG + g) * kTileN + r]);
  const float z = z8 ? (float)z8[(nt * KG + g) * kTileN + r] : (w4 ? 8.0f : 128.0f);
  float w[8];
  if (w4) {
    const uint32_t d = ((const uint32_t*)packed)[((nt * KT + kt128) * 64 + lane) * 4 + j];
#pragma unroll
    for (int e = 0; e < 8; ++e) w[e] = (float)((d >> (4 * nibble_pos(e))) & 0xFu);
  } else {
    const int64_t kt = k0 / kTileK8;
    const int koff = (int)(k0 % kTileK8);
    const uint8_t* p = packed + ((nt * KT + kt) * 64 + (r + 16 * (koff / 16))) * 16 + koff % 16;
#pragma unroll
    for (int e = 0; e < 8; ++e) w[e] = fp8 ? fp8_e4m3fn_to_f32(p[e]) : (float)p[e];
  }
  uint32_t o[4];
#pragma unroll
  for (int e = 0; e < 8; e += 2) {
    float v[2];
#pragma unroll
    for (int h = 0; h < 2; ++h)
      v[h] = nf4 ? __fmul_rn(kNf4Values[(int)w[e + h]], s)
                 : fp8 ? __fmul_rn(w[e + h], s) : __fmul_rn(__fsub_rn(w[e + h], z), s);
    o[e / 2] = (uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
  }
  out[gid] = u4{o[0], o[1], o[2], o[3]};
}

int launch_dense_weight(const void* qweight, int weight_dtype, int64_t N, int64_t K, const uint16_t* sb16,
                        const uint8_t* z8, int64_t G, void* out, hipStream_t st) {
  if (N == 0 || K == 0) return 0;
  if (K % 128 != 0) return set_error("dense_weight: K = %lld is not a multiple of 128", (long long)K);
  const bool w8 = weight_dtype == WOQ_HIP_DTYPE_INT8 || weight_dtype == WOQ_HIP_DTYPE_FP8;
  const int64_t NT = (N + kTileN - 1) / kTileN, KT128 = K / 128;
  const int64_t KT = woq_hip_padded_k(weight_dtype, K) / (w8 ? kTileK8 : kTileK4);
  const int64_t KG = G > 0 ? (K + G - 1) / G : 1;
  const int64_t total = KT128 * NT * 256;
  dense_weight_kernel<<<blocks_for(total, 256), 256, 0, st>>>((const uint8_t*)qweight, weight_dtype, NT, KT128, KT,
                                                              sb16, z8, G, KG, (u4*)out);
  return check_launch("dense_weight");
}

// ---- GPTQ act-order (g_idx): channel shuffles -------------------------------------------------
// Reference: woq_shuffle_tensor_by_group_idx / woq_shuffle_weight_back_by_group_idx
// (csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:777-954).  Channel j moves to position
// g_idx[j] * group_size + (number of earlier channels of the same group); `src` is that map
// read backwards (src[p] = the channel that lands at position p), which serves both directions.
template <typename T>
__global__ void shuffle_activations_kernel(const T* __restrict__ x, int64_t M, int64_t K,
                                           const int32_t* __restrict__ src, T* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= M * K) return;
  const int64_t m = i / K, p = i - m * K;
  out[i] = x[m * K + src[p]];
}

// plain int4 rows (two values per byte, low nibble first): one thread per output byte
__global__ void shuffle_int4_weight_kernel(const uint8_t* __restrict__ plain, int64_t N, int64_t K,
                                           const int32_t* __restrict__ src, uint8_t* __restrict__ out) {
  const int64_t stride = (K + 1) / 2;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= N * stride) return;
  const int64_t n = i / stride, b = i - n * stride;
  uint8_t v = 0;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int64_t pos = 2 * b + h;
    if (pos < K) {
      const int64_t j = src[pos];
      const uint8_t byte = plain[n * stride + j / 2];
      v |= (uint8_t)(((j & 1) ? byte >> 4 : byte & 15) << (4 * h));
    }
  }
  out[i] = v;
}

// Element-wise conversion between the activation dtypes, eight elements per thread where both
// pointers allow 16-byte accesses of the narrower type.
__global__ void convert_activations_kernel(const void* __restrict__ src, int src_dtype, void* __restrict__ dst,
                                           int dst_dtype, int64_t count) {
  const int64_t i0 = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 8;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int64_t i = i0 + e;
    if (i < count) store_act(dst, dst_dtype, i, load_act(src, src_dtype, i));
  }
}
__global__ void convert_bf16_to_f16_kernel(const u4* __restrict__ src, u4* __restrict__ dst, int64_t chunks) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= chunks) return;
  const u4 v = __builtin_nontemporal_load(src + i);
  u4 o;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float lo = bitcast<float>(v[e] << 16), hi = bitcast<float>(v[e] & 0xFFFF0000u);
    o[e] = (uint32_t)f32_to_f16_bits(lo) | ((uint32_t)f32_to_f16_bits(hi) << 16);
  }
  dst[i] = o;
}

int launch_convert_activations(const void* src, int src_dtype, void* dst, int dst_dtype, int64_t count,
                               hipStream_t st) {
  if (count == 0) return 0;
  if (src_dtype == WOQ_HIP_ACT_BF16 && dst_dtype == WOQ_HIP_ACT_FP16 && count % 8 == 0 &&
      (((uintptr_t)src | (uintptr_t)dst) & 15) == 0) {
    convert_bf16_to_f16_kernel<<<blocks_for(count / 8, 256), 256, 0, st>>>((const u4*)src, (u4*)dst, count / 8);
  } else {
    convert_activations_kernel<<<blocks_for((count + 7) / 8, 256), 256, 0, st>>>(src, src_dtype, dst, dst_dtype,
                                                                                 count);
  }
  return check_launch("convert_activations");
}

int launch_shuffle_activations(const void* x, int x_dtype, int64_t M, int64_t K, const int32_t* src, void* out,
                               hipStream_t st) {
  const int64_t total = M * K;
  if (total == 0) return 0;
  if (x_dtype == WOQ_HIP_ACT_FP32)
    shuffle_activations_kernel<uint32_t><<<blocks_for(total, 256), 256, 0, st>>>((const uint32_t*)x, M, K, src,
                                                                                   (uint32_t*)out);
  else
    shuffle_activations_kernel<uint16_t><<<blocks_for(total, 256), 256, 0, st>>>((const uint16_t*)x, M, K, src,
                                                                                   (uint16_t*)out);
  return check_launch("shuffle_activations");
}

int launch_shuffle_int4_weight(const void* plain, int64_t N, int64_t K, const int32_t* src, void* out,
                               hipStream_t st) {
  const int64_t total = N * ((K + 1) / 2);
  if (total == 0) return 0;
  shuffle_int4_weight_kernel<<<blocks_for(total, 256), 256, 0, st>>>((const uint8_t*)plain, N, K, src,
                                                                     (uint8_t*)out);
  return check_launch("shuffle_int4_weight");
}

}  // namespace woq

// Shared device helpers for the gfx950 WOQ linear kernels: vector types, the packed
// tile geometry, nibble decoding and the rounding helpers every kernel uses.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/woq_hip.h"

namespace woq {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef __bf16 b2 __attribute__((ext_vector_type(2)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef float f2 __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef int i4 __attribute__((ext_vector_type(4)));
typedef int i16v __attribute__((ext_vector_type(16)));
typedef unsigned u2 __attribute__((ext_vector_type(2)));
typedef unsigned u4 __attribute__((ext_vector_type(4)));

constexpr int kTileN = WOQ_HIP_TILE_N;
constexpr int kTileBytes = WOQ_HIP_TILE_BYTES;
constexpr int kTileK4 = WOQ_HIP_TILE_K_INT4;
constexpr int kTileK8 = WOQ_HIP_TILE_K_INT8;

// Compute regimes of the floating-point kernels.  The reference picks fp16 for
// lowp_mode FP16, for NONE with half activations and for BF16 with M < 5, and bf16 for
// NONE with bf16 activations and for BF16 with M >= 5
// (csrc/cpu/aten/kernels/WoqLinearKrnl.cpp:75-112).
enum Regime { kRegimeF16 = 0, kRegimeBF16 = 1 };

template <typename T, typename U>
__device__ __forceinline__ T bitcast(U u) {
  static_assert(sizeof(T) == sizeof(U), "size mismatch");
  return __builtin_bit_cast(T, u);
}

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
  return bitcast<float>((uint32_t)b << 16);
}

// fp32 -> bf16, round to nearest even (NaN kept quiet); v_cvt_pk_bf16_f32 on gfx950.
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  __bf16 b = (__bf16)f;
  return bitcast<uint16_t>(b);
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;
  return bitcast<uint16_t>(h);
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) {
  return (float)bitcast<_Float16>(b);
}

// Nibble position of K-element e (0..7) inside one dword of the packed INT4 layout.
__host__ __device__ __forceinline__ constexpr int nibble_pos(int e) {
  return (e & 1) ? 4 + (e >> 1) : (e >> 1);
}

// ---- workgroup -> tile, by XCD ------------------------------------------------------------------
// Workgroups are handed to the eight XCDs round robin in dispatch order (x fastest), and each XCD has an L2 of
// its own.  With a grid whose width is no multiple of eight, the tiles of one XCD would be scattered over every
// column block, and every L2 would fetch the whole weight.  This maps the dispatch order onto tiles so that an XCD
// works on a contiguous range of them: tiles are numbered in bands of four column blocks (x fastest inside a band,
// then y, then the next band), XCD k takes the k-th eighth of that numbering.  For a width that is a multiple of
// 32 and any height this is what the hardware order gives anyway (four column blocks per XCD, rows in order).
__device__ __forceinline__ void xcd_tile(int& tx, int& ty) {
  const int gx = (int)gridDim.x, gy = (int)gridDim.y;
  const int total = gx * gy;
  const int id = (int)(blockIdx.y * gridDim.x + blockIdx.x);
  const int xcd = id & 7, slot = id >> 3;
  const int lin = xcd * (total >> 3) + (xcd < (total & 7) ? xcd : (total & 7)) + slot;
  const int band = lin / (4 * gy);
  const int within = lin - band * (4 * gy);
  const int bw = gx - 4 * band < 4 ? gx - 4 * band : 4;
  ty = within / bw;
  tx = 4 * band + within - ty * bw;
}

// ---- 4-bit decode -------------------------------------------------------------------
// (d >> 4v) & 0x000F000F | 0x6400_6400 is the fp16 pair (1024 + q[2v], 1024 + q[2v+1]).
__device__ __forceinline__ h2 nib_pair_f16(uint32_t d, int v, uint32_t mask, uint32_t magic) {
  return bitcast<h2>(((d >> (4 * v)) & mask) | magic);
}

// fp16 regime: w = fp16((q - z) * s).  nz = -(1024 + z) (exact in fp16 for integral z < 1024),
// so the add is exact and the product is rounded once, which is fp16((q - z) * s) whenever s
// is an fp16 value (csrc/cpu/aten/utils/woq_utils.h:79-163 followed by .to(half),
// csrc/cpu/aten/utils/woq.h:3565-3567).
__device__ __forceinline__ h8 dequant8_f16(uint32_t d, h2 nz, h2 s2) {
  const uint32_t mask = 0x000F000Fu, magic = 0x64006400u;
  h8 r;
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    h2 h = nib_pair_f16(d, v, mask, magic);
    h = (h + nz) * s2;
    r[2 * v] = h[0];
    r[2 * v + 1] = h[1];
  }
  return r;
}

// bf16 regime: w = bf16((q - z) * s) with s a bf16 value held in fp32.  c = -(1024 + z) * s is
// exact in fp32 (11 bits x 8 bits), and fma(1024 + q, s, c) has the exactly representable
// value (q - z) * s, so the only rounding is the final RNE to bf16
// (csrc/cpu/aten/utils/woq.h:1495-1581: separate sub and mul in fp32, then store as bf16).
__device__ __forceinline__ b8 dequant8_bf16(uint32_t d, float s, float c) {
  const uint32_t mask = 0x000F000Fu, magic = 0x64006400u;
  b8 r;
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    h2 h = nib_pair_f16(d, v, mask, magic);
    f2 f;
    f[0] = __builtin_fmaf((float)h[0], s, c);
    f[1] = __builtin_fmaf((float)h[1], s, c);
    b2 b = __builtin_convertvector(f, b2);
    r[2 * v] = b[0];
    r[2 * v + 1] = b[1];
  }
  return r;
}

// ---- 8-bit decode (bytes are offset-binary: stored = q + 128) ---------------------------
// 8 consecutive K elements live in two dwords.
// float8 e4m3fn byte (1 sign, 4 exponent bits with bias 7, 3 mantissa bits) -> fp32 the way the reference's
// weight-only kernels convert it (convert_fp8_e4m3_to_fp32, csrc/cpu/aten/utils/woq.h:465-485): the 7 low bits
// shifted to the fp32 exponent / mantissa boundary plus the bias difference (127 - 7) << 23, zero when those
// bits are zero, then the sign.  Every code is read as a normal number: that is the float8 value for
// exponents 1..15 and for +-0; the subnormal codes 0x01..0x07 give (8 + m) * 2^-10 where float8 means
// m * 2^-9, and the NaN codes 0x7F / 0xFF give +-480.  Kept, so that a checkpoint gives the reference's numbers.
__device__ __forceinline__ float fp8_e4m3fn_to_f32(uint32_t byte) {
  const uint32_t mag = byte & 0x7Fu;
  const uint32_t bits = mag ? (mag << 20) + (120u << 23) : 0u;
  return bitcast<float>(bits | ((byte & 0x80u) << 24));
}

// The same conversion for two bytes at once, to fp16, where every one of its values is exact: v holds the bytes in
// bits 15..8 and 31..24; the 7 low bits of each land on fp16's exponent / mantissa boundary (>> 1), the bias
// difference (15 - 7) << 10 is added unless they are zero, the sign bit stays where it is.
// (min(t, 1) * 0x2000 + t on 16-bit halves; written as the two packed instructions because the compiler turns the
// same expression into a compare and a select per half.)
__device__ __forceinline__ h2 fp8x2_to_f16x2(uint32_t v) {
  const uint32_t t = (v & 0x7F007F00u) >> 1;
  uint32_t nz, r;
  asm("v_pk_min_u16 %0, %1, %2" : "=v"(nz) : "v"(t), "v"(0x00010001u));
  asm("v_pk_mad_u16 %0, %1, %2, %3" : "=v"(r) : "v"(nz), "v"(0x20002000u), "v"(t));
  return bitcast<h2>(r | (v & 0x80008000u));
}

// 8-bit weights as fp8: w = cd(fp8(byte) * s), one rounding (load_dequant_fp8, csrc/cpu/aten/utils/woq.h:728-741:
// the converted value times the scale in the compute type).  fp16: the fp16 product of two fp16 numbers is that
// rounding.  bf16: the product is exact in fp32 (4 x 8 significant bits) and rounded once.
__device__ __forceinline__ h8 dequant8_f16_fp8(uint32_t d0, uint32_t d1, float s) {
  const h2 sh = {(_Float16)s, (_Float16)s};  // exact: the fp16 regime reads fp16 scales
  const h2 p0 = fp8x2_to_f16x2(__builtin_amdgcn_perm(0u, d0, 0x010c000cu)) * sh;
  const h2 p1 = fp8x2_to_f16x2(__builtin_amdgcn_perm(0u, d0, 0x030c020cu)) * sh;
  const h2 p2 = fp8x2_to_f16x2(__builtin_amdgcn_perm(0u, d1, 0x010c000cu)) * sh;
  const h2 p3 = fp8x2_to_f16x2(__builtin_amdgcn_perm(0u, d1, 0x030c020cu)) * sh;
  return h8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
}
// fp32(fp16 half of v) * s in one mixed-precision instruction (a zero product comes out as +0)
__device__ __forceinline__ f2 f16x2_times_f32(h2 v, float s) {
  f2 r;
  asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel_hi:[1,0,0]" : "=v"(r[0]) : "v"(bitcast<uint32_t>(v)), "v"(s));
  asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(r[1]) : "v"(bitcast<uint32_t>(v)), "v"(s));
  return r;
}
__device__ __forceinline__ b8 dequant8_bf16_fp8(uint32_t d0, uint32_t d1, float s) {
  const b2 p0 = __builtin_convertvector(f16x2_times_f32(fp8x2_to_f16x2(__builtin_amdgcn_perm(0u, d0, 0x010c000cu)), s), b2);
  const b2 p1 = __builtin_convertvector(f16x2_times_f32(fp8x2_to_f16x2(__builtin_amdgcn_perm(0u, d0, 0x030c020cu)), s), b2);
  const b2 p2 = __builtin_convertvector(f16x2_times_f32(fp8x2_to_f16x2(__builtin_amdgcn_perm(0u, d1, 0x010c000cu)), s), b2);
  const b2 p3 = __builtin_convertvector(f16x2_times_f32(fp8x2_to_f16x2(__builtin_amdgcn_perm(0u, d1, 0x030c020cu)), s), b2);
  return b8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
}

// 8-bit integer weights (offset-binary bytes u, zero point uz): w = cd((u - uz) * s), one rounding.  Two bytes at a
// time become the fp16 numbers 1024 + u (v_perm_b32 places each byte under the constant 0x64: exponent 2^10, mantissa
// step 1); one mixed-precision fma per weight, (1024 + u) * s - (1024 + uz) * s, gives the exact product in fp32
// (at most 11 x 11 significant bits, and the constant term, c - 1024 s with c = -uz * s, is exact too), which is
// rounded once to the compute type.  2 instructions per weight instead of 2.5 with a byte-to-float conversion each.
__device__ __forceinline__ f2 w8_pair(uint32_t d, uint32_t sel, float s, float c2) {
  const h2 h = bitcast<h2>(__builtin_amdgcn_perm(0x64646464u, d, sel));
  f2 f;
  f[0] = __builtin_fmaf((float)h[0], s, c2);
  f[1] = __builtin_fmaf((float)h[1], s, c2);
  return f;
}
__device__ __forceinline__ h8 dequant8_f16_w8(uint32_t d0, uint32_t d1, float s, float c) {
  const float c2 = __builtin_fmaf(-1024.0f, s, c);
  const h2 p0 = __builtin_convertvector(w8_pair(d0, 0x04010400u, s, c2), h2);
  const h2 p1 = __builtin_convertvector(w8_pair(d0, 0x04030402u, s, c2), h2);
  const h2 p2 = __builtin_convertvector(w8_pair(d1, 0x04010400u, s, c2), h2);
  const h2 p3 = __builtin_convertvector(w8_pair(d1, 0x04030402u, s, c2), h2);
  return h8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
}
__device__ __forceinline__ b8 dequant8_bf16_w8(uint32_t d0, uint32_t d1, float s, float c) {
  const float c2 = __builtin_fmaf(-1024.0f, s, c);
  const b2 p0 = __builtin_convertvector(w8_pair(d0, 0x04010400u, s, c2), b2);
  const b2 p1 = __builtin_convertvector(w8_pair(d0, 0x04030402u, s, c2), b2);
  const b2 p2 = __builtin_convertvector(w8_pair(d1, 0x04010400u, s, c2), b2);
  const b2 p3 = __builtin_convertvector(w8_pair(d1, 0x04030402u, s, c2), b2);
  return b8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
}

// Output rounding of one accumulator.
//   fp16 regime: the reference GEMM result is an fp16 tensor, the fp16 bias is added in
//   fp16, and the result is cast to the activation dtype
//   (csrc/cpu/aten/utils/woq.h:3569-3576, 3612).
//   bf16 regime: fp32 accumulator initialised with the fp32 bias, one rounding to the
//   output dtype (csrc/cpu/aten/utils/woq.h:3298-3310, 3452).
template <int REGIME>
__device__ __forceinline__ float finalize_acc(float acc, bool has_bias, float bias) {
  if (REGIME == kRegimeF16) {
    _Float16 h = (_Float16)acc;
    if (has_bias) h = (_Float16)((float)h + (float)(_Float16)bias);
    return (float)h;
  } else {
    return has_bias ? acc + bias : acc;
  }
}

__device__ __forceinline__ float gelu_erf(float x) {
  return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}
__device__ __forceinline__ float gelu_tanh(float x) {
  const float k0 = 0.7978845608028654f, k1 = 0.044715f;
  return 0.5f * x * (1.0f + tanhf(k0 * (x + k1 * x * x * x)));
}
__device__ __forceinline__ float silu(float x) { return x / (1.0f + __expf(-x)); }

__device__ __forceinline__ float load_act(const void* p, int dtype, int64_t i) {
  if (dtype == WOQ_HIP_ACT_BF16) return bf16_bits_to_f32(((const uint16_t*)p)[i]);
  if (dtype == WOQ_HIP_ACT_FP16) return f16_bits_to_f32(((const uint16_t*)p)[i]);
  return ((const float*)p)[i];
}

// Round v to the activation dtype and return it as fp32 (the reference applies post-ops on
// the output-dtype tile, csrc/cpu/aten/utils/woq.h:2924-2967).
__device__ __forceinline__ float round_to_act(float v, int dtype) {
  if (dtype == WOQ_HIP_ACT_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(v));
  if (dtype == WOQ_HIP_ACT_FP16) return f16_bits_to_f32(f32_to_f16_bits(v));
  return v;
}

__device__ __forceinline__ void store_act(void* p, int dtype, int64_t i, float v) {
  if (dtype == WOQ_HIP_ACT_BF16)
    ((uint16_t*)p)[i] = f32_to_bf16_bits(v);
  else if (dtype == WOQ_HIP_ACT_FP16)
    ((uint16_t*)p)[i] = f32_to_f16_bits(v);
  else
    ((float*)p)[i] = v;
}

// Epilogue shared by every kernel: bias + regime rounding, optional post-op, store.
struct Epilogue {
  const float* bias;
  int fusion;
  const void* other0;
  const void* other1;
  void* out;
  int out_dtype;  // WOQ_HIP_ACT_*; fp32 means "raw accumulator + bias"
  int act_dtype;  // dtype post-ops round through
  int64_t N;      // logical N (row stride of out / others)
};

template <int REGIME>
__device__ __forceinline__ void epilogue_store(const Epilogue& e, int64_t m, int64_t n, float acc) {
  const bool hb = e.bias != nullptr;
  const float b = hb ? e.bias[n] : 0.0f;
  const int64_t idx = m * e.N + n;
  if (e.out_dtype == WOQ_HIP_ACT_FP32 && e.act_dtype != WOQ_HIP_ACT_FP32) {
    ((float*)e.out)[idx] = hb ? acc + b : acc;
    return;
  }
  float y = finalize_acc<REGIME>(acc, hb, b);
  if (e.fusion != WOQ_HIP_FUSE_NONE) {
    y = round_to_act(y, e.act_dtype);
    switch (e.fusion) {
      case WOQ_HIP_FUSE_GELU_ERF: y = gelu_erf(y); break;
      case WOQ_HIP_FUSE_GELU_TANH: y = gelu_tanh(y); break;
      case WOQ_HIP_FUSE_RELU: y = y > 0.0f ? y : 0.0f; break;
      case WOQ_HIP_FUSE_SILU: y = silu(y); break;
      case WOQ_HIP_FUSE_ADD: y = y + load_act(e.other0, e.act_dtype, idx); break;
      case WOQ_HIP_FUSE_ADD_ADD:
        y = round_to_act(y + load_act(e.other0, e.act_dtype, idx), e.act_dtype);
        y = y + load_act(e.other1, e.act_dtype, idx);
        break;
      case WOQ_HIP_FUSE_MUL: y = y * load_act(e.other0, e.act_dtype, idx); break;
      default: break;
    }
  }
  store_act(e.out, e.out_dtype, idx, y);
}

// a pointer every lane of the wave loaded from the same address, moved to scalar registers
template <typename T>
__device__ __forceinline__ T* dq_uniform(T* p) {
  const uint64_t v = (uint64_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (T*)(((uint64_t)hi << 32) | lo);
}

// ---- 4-bit weights as MFMA operands: one packed dword (8 weights of one row) -> 8 bf16 / fp16 ----
// Per-lane dequantization constants of one weight row and quantization group.
template <int REGIME>
struct G4Consts;
// bf16 regime: w = bf16((q - z) * s).  The fp16 value 1024 + q (or 1024 + 16 q for a nibble taken
// in place at bits 4..7) times s (or s / 16) plus c is the exact product (q - z) * s in fp32: one
// fma, then one round-to-nearest-even to bf16.
template <>
struct G4Consts<kRegimeBF16> {
  float s, c, s16, c16;
  __device__ __forceinline__ void set(uint16_t sbits, float z) {
    s = bf16_bits_to_f32(sbits);
    c = -((1024.0f + z) * s);
    s16 = s * 0.0625f;
    c16 = -((64.0f + z) * s);
  }
};
// fp16 regime: w = fp16((q - z) * s): exact subtraction, one rounding in the product.
template <>
struct G4Consts<kRegimeF16> {
  h2 nz, s2;
  __device__ __forceinline__ void set(uint16_t sbits, float z) {
    const _Float16 s = bitcast<_Float16>(sbits);
    const _Float16 n = (_Float16)(-(1024.0f + z));
    nz = h2{n, n};
    s2 = h2{s, s};
  }
};

// Chunk swizzle of an LDS row of 128 bytes (8 chunks of 16 bytes; chunk q of row m is kept at q ^ swz_row128(m)):
// distinct over any 8 consecutive rows, and over the even and the odd rows of 16, so that a fragment read -- 16
// rows x one chunk per lane column -- touches every 16-byte bank group once whether the LDS serves 8 lanes x
// 128 bytes or 16 lanes x 256 bytes at a time.  (The prefill kernel with the dequantized tile in LDS reads its bf16
// tiles this way with the bank-conflict counter at zero; the int8 kernels' fragment reads -- chunk 2 c + j instead of
// 4 s + c -- still count four conflict cycles each, as they did with (m / 2) % 8, behind vector work that bounds them.)
__device__ __forceinline__ int swz_row128(int row) { return ((row >> 1) & 3) | (((row ^ (row >> 3)) & 1) << 2); }

struct G4Masks {
  uint32_t lo, hi, magic;  // 0x000F000F, 0x00F000F0, fp16 1024 twice
};

__device__ __forceinline__ f2 g4_fma_pair(uint32_t hbits, float s, float c) {
  const h2 h = bitcast<h2>(hbits);
  f2 f;
  f[0] = __builtin_fmaf((float)h[0], s, c);
  f[1] = __builtin_fmaf((float)h[1], s, c);
  return f;
}
__device__ __forceinline__ uint32_t g4_cvt_pair(f2 f) { return bitcast<uint32_t>(__builtin_convertvector(f, b2)); }

// One packed dword (8 weights of one row) -> MFMA B operand.  Written so that no conversion
// directly follows the fma that feeds it: v_cvt_pk_bf16_f32 one instruction behind its producer
// costs a wait state.
__device__ __forceinline__ u4 g4_dequant(uint32_t d, const G4Masks& k, const G4Consts<kRegimeBF16>& q) {
  u4 r;
  const f2 f0 = g4_fma_pair((d & k.lo) | k.magic, q.s, q.c);
  const f2 f1 = g4_fma_pair((d & k.hi) | k.magic, q.s16, q.c16);
  r[0] = g4_cvt_pair(f0);
  const uint32_t d8 = d >> 8;
  const f2 f2_ = g4_fma_pair((d8 & k.lo) | k.magic, q.s, q.c);
  r[1] = g4_cvt_pair(f1);
  const f2 f3 = g4_fma_pair((d8 & k.hi) | k.magic, q.s16, q.c16);
  r[2] = g4_cvt_pair(f2_);
  r[3] = g4_cvt_pair(f3);
  return r;
}
__device__ __forceinline__ u4 g4_dequant(uint32_t d, const G4Masks& k, const G4Consts<kRegimeF16>& q) {
  u4 r;
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    h2 h = bitcast<h2>(((d >> (4 * v)) & k.lo) | k.magic);
    h = (h + q.nz) * q.s2;
    r[v] = bitcast<uint32_t>(h);
  }
  return r;
}

// ---- NF4 weights: 4-bit codes into a fixed table of 16 values in [-1, 1] ----------------------
// The table of csrc/cpu/aten/utils/woq_utils.h:34-51 (the NormalFloat4 code book); w = table[q] *
// scale, the product rounded to fp32 and then once to the compute dtype
// (csrc/cpu/aten/utils/woq_utils.h:165-262).
static __constant__ const float kNf4Values[16] = {
    -1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f,
    -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
    0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f, 0.33791524171829224f,
    0.44070982933044434f, 0.5626170039176941f, 0.7229568362236023f, 1.0f};

// One packed dword (8 codes of one row) -> 8 compute-dtype weights in K order.  `lut` is the pair
// table in LDS (nf4_fill_lut): entry b holds the table values of the two codes in byte b, so a dword
// takes four 8-byte reads instead of eight 4-byte ones and half the address arithmetic.  Byte b of the
// dword carries the codes of nibble positions 2 b and 2 b + 1; output dword v pairs the positions v and
// v + 4 (K elements 2 v and 2 v + 1).
constexpr int kNf4LutEntries = 256;
__device__ __forceinline__ void nf4_fill_lut(f2* lut, int tid, int nthreads) {
  for (int i = tid; i < kNf4LutEntries; i += nthreads) lut[i] = f2{kNf4Values[i & 15], kNf4Values[i >> 4]};
}
template <int REGIME>
__device__ __forceinline__ u4 nf4_dequant(uint32_t d, const f2* lut, float s) {
  const f2 p0 = lut[d & 0xFFu], p1 = lut[(d >> 8) & 0xFFu], p2 = lut[(d >> 16) & 0xFFu], p3 = lut[d >> 24];
  const float lo[4] = {__fmul_rn(p0[0], s), __fmul_rn(p0[1], s), __fmul_rn(p1[0], s), __fmul_rn(p1[1], s)};
  const float hi[4] = {__fmul_rn(p2[0], s), __fmul_rn(p2[1], s), __fmul_rn(p3[0], s), __fmul_rn(p3[1], s)};
  u4 r;
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    if constexpr (REGIME == kRegimeF16)
      r[v] = (uint32_t)f32_to_f16_bits(lo[v]) | ((uint32_t)f32_to_f16_bits(hi[v]) << 16);
    else
      r[v] = g4_cvt_pair(f2{lo[v], hi[v]});
  }
  return r;
}

}  // namespace woq

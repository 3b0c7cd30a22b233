// lowp_mode = INT8: dynamic activation quantization and int8 x int8 -> int32 MFMA kernels.
//
// Reference counterparts:
//   dynamic_quantize_per_block (csrc/cpu/aten/utils/woq_dynamic_quant.h:1526-1750)
//   Dequantize<int8_t> + BrgemmTPP<int8,int32> + fp32 epilogue (csrc/cpu/aten/utils/woq.h:1664-1734,
//   2133-2199), small-M VNNI micro-kernel (woq.h:953-1127).
//
// Arithmetic contract (bit-exact parts): q_a = clamp(rint(x / s_a + zp_a)), B = q_w - z_w as int8,
// qC[m, n, kb] = sum over the K block kb of q_a * B in int32.  Float epilogue, blocks in ascending
// K order inside a wave: C += (float(qC) * s_a) * s_w  (woq.h:2172-2186, unfused mul, mul, add).
#include "woq_common.h"
#include "woq_internal.h"

// The fp32 epilogue `C += (float(sum) * s_a) * s_w` keeps three separate roundings
// (csrc/cpu/aten/utils/woq.h:2172-2186).  hipcc contracts a multiply feeding an add into one fused
// multiply-add by default, also through the __fmul_rn / __fadd_rn helpers (header functions built
// under the command line's mode), so contraction is switched off for the operators of this file.
#pragma clang fp contract(off)

namespace woq {

__host__ __device__ inline bool quant_a_is_sym(int mode) { return mode >= WOQ_HIP_QUANT_A_PER_TENSOR_SYM; }
__host__ __device__ inline bool quant_a_per_m(int mode) {
  return mode == WOQ_HIP_QUANT_A_PER_M || mode == WOQ_HIP_QUANT_A_PER_M_K_BLOCK ||
         mode == WOQ_HIP_QUANT_A_PER_M_SYM || mode == WOQ_HIP_QUANT_A_PER_M_K_BLOCK_SYM;
}
__host__ __device__ inline bool quant_a_per_k(int mode) {
  return mode == WOQ_HIP_QUANT_A_PER_K_BLOCK || mode == WOQ_HIP_QUANT_A_PER_M_K_BLOCK ||
         mode == WOQ_HIP_QUANT_A_PER_K_BLOCK_SYM || mode == WOQ_HIP_QUANT_A_PER_M_K_BLOCK_SYM;
}

// ---- statistics: one workgroup per quantization group -------------------------------------
// group id -> (row range, k range); writes scale (and zero point for asymmetric modes).
__global__ __launch_bounds__(256) void act_stats_kernel(const void* __restrict__ x, int x_dtype, int64_t M,
                                                        int64_t K, int64_t qbk, int64_t Kc, int mode,
                                                        float* __restrict__ scales, int32_t* __restrict__ zps) {
  const int64_t gid = blockIdx.x;
  const bool per_m = quant_a_per_m(mode), per_k = quant_a_per_k(mode);
  int64_t m_lo = 0, m_hi = M, k_lo = 0, k_hi = K;
  if (per_m && per_k) {
    m_lo = gid / Kc;
    m_hi = m_lo + 1;
    k_lo = (gid % Kc) * qbk;
    k_hi = k_lo + qbk < K ? k_lo + qbk : K;
  } else if (per_m) {
    m_lo = gid;
    m_hi = gid + 1;
  } else if (per_k) {
    k_lo = gid * qbk;
    k_hi = k_lo + qbk < K ? k_lo + qbk : K;
  }
  const int64_t kw = k_hi - k_lo;
  const int64_t total = (m_hi - m_lo) * kw;
  float mn = __builtin_inff(), mx = -__builtin_inff();
  for (int64_t i = threadIdx.x; i < total; i += blockDim.x) {
    const int64_t m = m_lo + i / kw, k = k_lo + i % kw;
    const float v = load_act(x, x_dtype, m * K + k);
    mn = fminf(mn, v);
    mx = fmaxf(mx, v);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    mn = fminf(mn, __shfl_xor(mn, off));
    mx = fmaxf(mx, __shfl_xor(mx, off));
  }
  __shared__ float smn[4], smx[4];
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
    smn[wave] = mn;
    smx[wave] = mx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w) {
      mn = fminf(mn, smn[w]);
      mx = fmaxf(mx, smx[w]);
    }
    if (quant_a_is_sym(mode)) {
      scales[gid] = __fdiv_rn(fmaxf(fabsf(mx), fabsf(mn)), 127.0f);
    } else {
      const float s = __fdiv_rn(__fsub_rn(mx, mn), 255.0f);
      scales[gid] = s;
      zps[gid] = (int32_t)(-rintf(__fdiv_rn(mn, s)));
    }
  }
}

// ---- statistics of groups that span all rows (per-tensor, per-K-block modes) ----------------
// One workgroup per group would scan M * K (or M * qbk) elements alone.  Instead many workgroups
// scan 8 rows x one K range each and combine through integer atomics on an order-preserving key
// of the float (min / max are exact in any order, so the result is deterministic).  The keys live
// in the output arrays themselves: max (or max |x| for the symmetric modes) in `scales`, min in
// `zps`; a last pass turns them into scale and zero point in place.
__device__ __forceinline__ int32_t float_key(float f) {
  const int32_t b = bitcast<int32_t>(f);
  return b ^ ((b >> 31) & 0x7fffffff);
}
__device__ __forceinline__ float key_float(int32_t k) { return bitcast<float>(k ^ ((k >> 31) & 0x7fffffff)); }

__global__ void act_stats_init_kernel(int64_t groups, int32_t* __restrict__ maxk, int32_t* __restrict__ mink) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= groups) return;
  maxk[i] = float_key(-__builtin_inff());
  if (mink) mink[i] = float_key(__builtin_inff());
}

constexpr int kStatRows = 8, kStatChunk = 2048;

__global__ __launch_bounds__(256) void act_stats_partial_kernel(const void* __restrict__ x, int x_dtype, int64_t M,
                                                                int64_t K, int64_t qbk, int per_k, int sym,
                                                                int32_t* __restrict__ maxk,
                                                                int32_t* __restrict__ mink) {
  // blockIdx.x: K range (a quantization block, or a chunk of the row for per-tensor), blockIdx.y: 8 rows
  const int64_t kw = per_k ? qbk : kStatChunk;
  const int64_t k_lo = (int64_t)blockIdx.x * kw;
  const int64_t k_hi = k_lo + kw < K ? k_lo + kw : K;
  const int64_t m_lo = (int64_t)blockIdx.y * kStatRows;
  const int64_t m_hi = m_lo + kStatRows < M ? m_lo + kStatRows : M;
  const int64_t w = k_hi - k_lo, total = (m_hi - m_lo) * w;
  float mn = __builtin_inff(), mx = -__builtin_inff();
  for (int64_t i = threadIdx.x; i < total; i += blockDim.x) {
    const float v = load_act(x, x_dtype, (m_lo + i / w) * K + k_lo + i % w);
    mn = fminf(mn, v);
    mx = fmaxf(mx, v);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    mn = fminf(mn, __shfl_xor(mn, off));
    mx = fmaxf(mx, __shfl_xor(mx, off));
  }
  if ((threadIdx.x & 63) == 0 && mx >= mn) {  // a wave that saw no element still holds (+inf, -inf)
    const int64_t g = per_k ? blockIdx.x : 0;
    if (sym) {
      atomicMax(maxk + g, float_key(fmaxf(fabsf(mx), fabsf(mn))));
    } else {
      atomicMax(maxk + g, float_key(mx));
      atomicMin(mink + g, float_key(mn));
    }
  }
}

__global__ void act_stats_finalize_kernel(int64_t groups, int sym, float* __restrict__ scales,
                                          int32_t* __restrict__ zps) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= groups) return;
  const float mx = key_float(bitcast<int32_t>(scales[i]));
  if (sym) {
    scales[i] = __fdiv_rn(mx, 127.0f);
  } else {
    const float mn = key_float(zps[i]);
    const float s = __fdiv_rn(__fsub_rn(mx, mn), 255.0f);
    scales[i] = s;
    zps[i] = (int32_t)(-rintf(__fdiv_rn(mn, s)));
  }
}

// ---- quantize: one thread per 8 consecutive K elements -------------------------------------
// ldq: row stride of q in bytes (>= K, the tail is zero-filled up to ldq).
// permute: store each group of 8 as [e0 e4 e1 e5 e2 e6 e3 e7], the byte order the 4-bit decode
// produces, so the int8 kernels can use the activations without a shuffle.  Padding bytes up to
// ldq hold 0 (symmetric) or, with offset128, whatever: the weights there are padded with q = z.
__global__ void act_quant_kernel(const void* __restrict__ x, int x_dtype, int64_t M, int64_t K, int64_t ldq,
                                 int64_t qbk, int64_t Kc, int mode, const float* __restrict__ scales,
                                 const int32_t* __restrict__ zps, uint8_t* __restrict__ q, int permute,
                                 int offset128) {
  const int64_t g8 = ldq / 8;
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= M * g8) return;
  const int64_t m = gid / g8, k0 = (gid % g8) * 8;
  const bool per_m = quant_a_per_m(mode), per_k = quant_a_per_k(mode), sym = quant_a_is_sym(mode);
  uint8_t o[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int64_t k = k0 + e;
    uint8_t b = 0;
    if (k < K) {
      const int64_t gi = (per_m ? m * (per_k ? Kc : 1) : 0) + (per_k ? k / qbk : 0);
      const float s = scales[gi];
      const float zp = sym ? 0.0f : (float)zps[gi];
      const float v = load_act(x, x_dtype, m * K + k);
      float t = __fadd_rn(__fdiv_rn(v, s), zp);
      t = rintf(t);
      const float lo = sym ? -128.0f : 0.0f, hi = sym ? 127.0f : 255.0f;
      t = fminf(fmaxf(t, lo), hi);
      if (s == 0.0f || t != t) t = sym ? 0.0f : zp;  // all-zero group: the reference divides 0 by 0
      // offset128: the asymmetric value 0..255 stored as the int8 number q - 128 for the signed MFMA
      b = sym ? (uint8_t)(int8_t)(int)t : (uint8_t)((int)t ^ (offset128 ? 0x80 : 0));
    }
    o[e] = b;
  }
  uint32_t d0, d1;
  if (permute) {
    d0 = o[0] | (o[4] << 8) | (o[1] << 16) | ((uint32_t)o[5] << 24);
    d1 = o[2] | (o[6] << 8) | (o[3] << 16) | ((uint32_t)o[7] << 24);
  } else {
    d0 = o[0] | (o[1] << 8) | (o[2] << 16) | ((uint32_t)o[3] << 24);
    d1 = o[4] | (o[5] << 8) | (o[6] << 16) | ((uint32_t)o[7] << 24);
  }
  *(u2*)(q + m * ldq + k0) = u2{d0, d1};
}

static int64_t num_quant_groups(int64_t M, int64_t Kc, int mode) {
  const bool per_m = quant_a_per_m(mode), per_k = quant_a_per_k(mode);
  return (per_m ? M : 1) * (per_k ? Kc : 1);
}

static int launch_quant_impl(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldq, int64_t qbk,
                             int mode, void* q, float* scales, int32_t* zps, int permute, int offset128,
                             hipStream_t st) {
  if (M == 0 || K == 0) return 0;
  if (qbk <= 0) qbk = K;
  const int64_t Kc = (K + qbk - 1) / qbk;
  const int64_t groups = num_quant_groups(M, Kc, mode);
  // whole rows from a wave's registers where a row fits them; otherwise the general statistics and quantization
  if (act_quant_rows_applies(x, x_dtype, K, q, ldq, qbk, quant_a_per_m(mode), quant_a_per_k(mode)))
    return launch_act_quant_rows(x, x_dtype, M, K, ldq, qbk, Kc, quant_a_per_m(mode), quant_a_per_k(mode),
                                 quant_a_is_sym(mode), q, scales, zps, permute, offset128, st);
  if (quant_a_per_m(mode)) {
    act_stats_kernel<<<(unsigned)groups, 256, 0, st>>>(x, x_dtype, M, K, qbk, Kc, mode, scales, zps);
    if (int rc = check_launch("act_stats_kernel")) return rc;
  } else {
    const int sym = quant_a_is_sym(mode), per_k = quant_a_per_k(mode);
    if (!sym && zps == nullptr) return set_error("dynamic_quant: asymmetric modes need a zero-point array");
    int32_t* maxk = (int32_t*)scales;
    int32_t* mink = sym ? nullptr : zps;
    act_stats_init_kernel<<<(unsigned)((groups + 255) / 256), 256, 0, st>>>(groups, maxk, mink);
    if (int rc = check_launch("act_stats_init_kernel")) return rc;
    dim3 grid((unsigned)(per_k ? Kc : (K + kStatChunk - 1) / kStatChunk), (unsigned)((M + kStatRows - 1) / kStatRows));
    act_stats_partial_kernel<<<grid, 256, 0, st>>>(x, x_dtype, M, K, qbk, per_k, sym, maxk, mink);
    if (int rc = check_launch("act_stats_partial_kernel")) return rc;
    act_stats_finalize_kernel<<<(unsigned)((groups + 255) / 256), 256, 0, st>>>(groups, sym, scales, zps);
    if (int rc = check_launch("act_stats_finalize_kernel")) return rc;
  }
  const int64_t total = M * (ldq / 8);
  act_quant_kernel<<<(unsigned)((total + 255) / 256), 256, 0, st>>>(x, x_dtype, M, K, ldq, qbk, Kc, mode,
                                                                    scales, zps, (uint8_t*)q, permute, offset128);
  return check_launch("act_quant_kernel");
}

int launch_dynamic_quant(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldq, int64_t qbk, int mode,
                         void* q, float* scales, int32_t* zps, hipStream_t st) {
  return launch_quant_impl(x, x_dtype, M, K, ldq, qbk, mode, q, scales, zps, 0, 0, st);
}

// ---- weight nibbles / bytes -> int8 (q - z) --------------------------------------------------
// Four bytes at once: ((b | 0x80808080) - z * 0x01010101) ^ 0x80808080 never borrows across bytes
// for |q - z| < 128 and leaves q - z in two's complement.
__device__ __forceinline__ uint32_t sub_bytes(uint32_t b, uint32_t z4) {
  return ((b | 0x80808080u) - z4) ^ 0x80808080u;
}

// NF4 under lowp_mode INT8: the code's table value times 127, rounded, as int8 (load_nf4_as_int8,
// csrc/cpu/aten/utils/woq.h:628-669).  Four codes in the bytes of b: two byte permutes over the halves
// of the table (codes 0..7 and 8..15), merged on bit 3 of each code.
__device__ __forceinline__ uint32_t nf4_codes_to_i8(uint32_t b) {
  // -127 -88 -67 -50 | -36 -23 -12 0 | 10 20 31 43 | 56 71 92 127, least significant byte first
  const uint32_t t0 = 0xCEBDA881u, t1 = 0x00F4E9DCu, t2 = 0x2B1F140Au, t3 = 0x7F5C4738u;
  const uint32_t sel = b & 0x07070707u;
  const uint32_t lo = __builtin_amdgcn_perm(t1, t0, sel);
  const uint32_t hi = __builtin_amdgcn_perm(t3, t2, sel);
  const uint32_t m = ((b >> 3) & 0x01010101u) * 0xFFu;
  return (hi & m) | (lo & ~m);
}

// 16 K elements of one lane for one 16x16x64 MFMA, from two packed dwords (4-bit) or four
// dwords (8-bit); 4-bit yields the permuted order [e0 e4 e1 e5][e2 e6 e3 e7].
template <int WBITS>
__device__ __forceinline__ i4 decode16_i8(const uint32_t* d, uint32_t z4, bool nf4 = false) {
  i4 r;
  if (WBITS == 4 && nf4) {
    r[0] = (int)nf4_codes_to_i8(d[0] & 0x0F0F0F0Fu);
    r[1] = (int)nf4_codes_to_i8((d[0] >> 4) & 0x0F0F0F0Fu);
    r[2] = (int)nf4_codes_to_i8(d[1] & 0x0F0F0F0Fu);
    r[3] = (int)nf4_codes_to_i8((d[1] >> 4) & 0x0F0F0F0Fu);
  } else if (WBITS == 4) {
    r[0] = (int)sub_bytes(d[0] & 0x0F0F0F0Fu, z4);
    r[1] = (int)sub_bytes((d[0] >> 4) & 0x0F0F0F0Fu, z4);
    r[2] = (int)sub_bytes(d[1] & 0x0F0F0F0Fu, z4);
    r[3] = (int)sub_bytes((d[1] >> 4) & 0x0F0F0F0Fu, z4);
  } else {
    // offset-binary bytes u = q + 128 and zero uz = z + 128: (u - uz) needs 9 bits when both are
    // extreme; the reference restricts 8-bit weights to symmetric (z = 0) in this mode
    // (csrc/cpu/aten/kernels/WoqInt8GemmAPerMKrnl.cpp:69-73), where it is exact.
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = (int)(d[i] ^ 0x80808080u);
  }
  return r;
}

struct Int8KArgs {
  Int8Args a;
  const uint8_t* xq;   // [M][ldq]
  int64_t ldq;
  const float* sa;     // activation scales
  const int32_t* za;   // activation zero points (asymmetric modes), indexed like sa
  int64_t sa_m_stride, sa_k_stride, qbk;
  int sa_kc;           // activation-scale groups along K (1 unless the mode is per K block)
  int64_t block_k;     // K block of the int32 accumulation
  int W;
  int64_t Kpad;
};

// Small-M int8 kernel; same work decomposition as the floating-point small-M kernel.
template <int WBITS, int MT, int KPW, int NTW, bool NF4>
__global__ __launch_bounds__(1024) void woq_small_m_i8_kernel(const Int8KArgs p) {
  static_assert(!NF4 || WBITS == 4, "NF4 codes are 4 bits wide");
  constexpr int TK = WBITS == 4 ? kTileK4 : kTileK8;
  constexpr int STEPS = WBITS == 4 ? 2 : 1;  // 16x16x64 MFMAs per tile
  constexpr int CK = TK / 4;
  extern __shared__ __align__(16) uint8_t smem[];
  const Int8Args& a = p.a;
  const int W = p.W;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, c = lane >> 4;
  const int64_t nt0 = (int64_t)blockIdx.x * NTW;
  const int64_t KC = (int64_t)W * KPW * TK;
  f4* red = (f4*)smem;

  f4 acc[NTW][MT];
#pragma unroll
  for (int t = 0; t < NTW; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f4{0.f, 0.f, 0.f, 0.f};

  // blocks per tile (block_k <= TK) or tiles per block (block_k > TK, 8-bit only: 128 / 64)
  const int bpt = p.block_k <= TK ? (int)(TK / p.block_k) : 1;

  for (int64_t kc0 = 0; kc0 < p.Kpad; kc0 += KC) {
    const int64_t ktw = kc0 / TK + (int64_t)wave * KPW;
    u4 wreg[NTW][KPW];
    uint8_t zreg[NTW][KPW];
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
      const int64_t nt = nt0 + t;
#pragma unroll
      for (int i = 0; i < KPW; ++i) {
        // unconditional loads from clamped indices; a clamped tile is replaced by the zero
        // encoding (q == z) afterwards
        const int64_t ktr = ktw + i;
        const bool live = nt < a.NT && ktr < a.KT;
        const int64_t ntc = nt < a.NT ? nt : a.NT - 1;
        const int64_t kt = ktr < a.KT ? ktr : a.KT - 1;
        const u4 wv = __builtin_nontemporal_load((const u4*)(a.qweight + ((ntc * a.KT + kt) * 64 + lane) * 16));
        uint8_t zb = WBITS == 4 ? 8 : 128;
        if (a.zeros) {
          int64_t g = (kt * TK + c * CK) / a.G;
          if (g >= a.KG) g = a.KG - 1;
          zb = a.zeros[(ntc * a.KG + g) * kTileN + r];
        }
        // a tile past the end contributes zeros: q = z = 0, offset-binary 128, or NF4 code 7
        const uint32_t dead = WBITS == 4 ? (NF4 ? 0x77777777u : 0u) : 0x80808080u;
        wreg[t][i] = live ? wv : u4{dead, dead, dead, dead};
        zreg[t][i] = live ? zb : (uint8_t)(WBITS == 4 ? 0 : 128);
      }
    }
    i4 xb[KPW][STEPS][MT];
#pragma unroll
    for (int i = 0; i < KPW; ++i)
#pragma unroll
      for (int j = 0; j < STEPS; ++j) {
        const int64_t k = (ktw + i) * TK + c * CK + j * 16;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const int64_t row = mt * 16 + r;
          const bool ok = row < a.M && k < p.ldq;
          const i4 v0 = *(const i4*)(p.xq + (row < a.M ? row : a.M - 1) * p.ldq + (k < p.ldq ? k : 0));
          const i4 v = ok ? v0 : i4{0, 0, 0, 0};
          xb[i][j][mt] = v;
        }
      }

#pragma unroll
    for (int t = 0; t < NTW; ++t) {
      const int64_t nt = nt0 + t;
      i4 qc[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) qc[mt] = i4{0, 0, 0, 0};
#pragma unroll
      for (int i = 0; i < KPW; ++i) {
        const int64_t kt = ktw + i;
        const uint32_t z4 = (uint32_t)zreg[t][i] * 0x01010101u;
#pragma unroll
        for (int j = 0; j < STEPS; ++j) {
          const uint32_t* d = (const uint32_t*)&wreg[t][i] + (WBITS == 4 ? 2 * j : 0);
          const i4 aop = decode16_i8<WBITS>(d, z4, NF4);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            qc[mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop, xb[i][j][mt], qc[mt], 0, 0, 0);
          // a K block ends here when the K extent accumulated so far is a multiple of block_k
          const int64_t kend = kt * TK + (WBITS == 4 ? (j + 1) * 64 : 64);
          const bool flush = (kend % p.block_k) == 0 || (i == KPW - 1 && j == STEPS - 1);
          if (flush) {
            const int64_t kb = (kend - 1) / p.block_k;          // block index
            const int64_t kq = kb * p.block_k;                   // first k of the block
            int64_t g = kq / a.G;
            if (g >= a.KG) g = a.KG - 1;
            const bool live = nt < a.NT && kt < a.KT;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
              const int64_t m = mt * 16 + (lane & 15);
              const float sa = (m < a.M && live) ? p.sa[m * p.sa_m_stride + (kq / p.qbk) * p.sa_k_stride] : 0.0f;
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const int64_t n = nt * kTileN + 4 * (lane >> 4) + e;
                float sw = live ? a.scales[(nt * a.KG + g) * kTileN + 4 * (lane >> 4) + e] : 0.0f;
                if (NF4) sw = sw * (1.0f / 127.0f);
                const float cterm = ((float)qc[mt][e] * sa) * sw;
                acc[t][mt][e] = acc[t][mt][e] + cterm;
                if (a.debug_block_sums && live && m < a.M && n < a.N)
                  a.debug_block_sums[(m * a.N + n) * (p.Kpad / p.block_k) + kb] = qc[mt][e];
              }
              qc[mt] = i4{0, 0, 0, 0};
            }
          }
        }
      }
    }
  }
  (void)bpt;

#pragma unroll
  for (int t = 0; t < NTW; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[((t * MT + mt) * W + wave) * 64 + lane] = acc[t][mt];
  __syncthreads();

  Epilogue e{a.bias, a.fusion, a.other0, a.other1, a.out, a.out_dtype, a.x_dtype, a.N};
  for (int idx = threadIdx.x; idx < NTW * MT * 64; idx += blockDim.x) {
    const int ln = idx & 63, tm = idx >> 6;
    const int t = tm / MT, mt = tm % MT;
    f4 s = red[(tm * W) * 64 + ln];
    for (int w = 1; w < W; ++w) {
      const f4 v = red[(tm * W + w) * 64 + ln];
      s[0] = __fadd_rn(s[0], v[0]);
      s[1] = __fadd_rn(s[1], v[1]);
      s[2] = __fadd_rn(s[2], v[2]);
      s[3] = __fadd_rn(s[3], v[3]);
    }
    const int64_t m = mt * 16 + (ln & 15);
    const int64_t n = (nt0 + t) * kTileN + 4 * (ln >> 4);
    if (m < a.M) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n + i < a.N) epilogue_store<kRegimeBF16>(e, m, n + i, s[i]);
    }
  }
}

// ---- tiled int8 GEMM for large M -------------------------------------------------------------
// 128 x 128 output tile, K step 128 bytes, 4 waves (2 x 2), v_mfma_i32_32x32x32_i8.
constexpr int IBM = 128, IBN = 128, IBK = 128;
constexpr int ILDS = IBK + 16;

// ASYM: asymmetric activations (uint8 q_a with zero point zp_a; csrc/cpu/aten/utils/woq.h:2172-2186).
// The activations arrive as int8 q_a - 128, the zero points are used as zp_a - 128, and the weight
// column sums of the K block ("compensation") come from one more MFMA against a row of ones:
// (sum (q_a - 128) B) - (zp_a - 128) sum B = sum q_a B - zp_a sum B, exactly the reference's integer.
template <int WBITS, int BLOCK_K, bool PER_K, bool DEBUG, bool ASYM, bool NF4 = false>
__global__ __launch_bounds__(256) void woq_gemm_i8_kernel(const Int8KArgs p) {
  static_assert(!NF4 || WBITS == 4, "NF4 codes are 4 bits wide");
  static_assert(!ASYM || PER_K, "the asymmetric variant reloads scales and zero points per K block");
  constexpr int TK = WBITS == 4 ? kTileK4 : kTileK8;
  const Int8Args& a = p.a;
  __shared__ __align__(16) uint8_t sA[IBM * ILDS];
  __shared__ __align__(16) uint8_t sB[IBN * ILDS];
  // activation scales of the K blocks of one step (per-K-block modes): [IBK / BLOCK_K][IBM]
  __shared__ __align__(16) float sSA[PER_K ? (IBK / BLOCK_K) * IBM : 4];
  __shared__ __align__(16) int32_t sZA[ASYM ? (IBK / BLOCK_K) * IBM : 4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int64_t m0 = (int64_t)blockIdx.y * IBM, n0 = (int64_t)blockIdx.x * IBN;
  const int64_t nt0 = n0 / kTileN;

  f16v acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  constexpr int sub_blocks = IBK / BLOCK_K;  // BLOCK_K in {32, 64, 128}

  // rows / columns of this lane's accumulator elements: m = mrow0 + 32 i + 8 (e / 4) + e % 4,
  // n = ncol0 + 32 j
  const int mrow0 = (int)m0 + wm * 64 + 4 * (lane >> 5);
  const int ncol0 = (int)n0 + wn * 64 + (lane & 31);
  // activation scales of those rows; constant over K unless the mode is per K block
  float sa_reg[2][16];
  int za_reg[ASYM ? 2 : 1][16];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int m = mrow0 + i * 32 + 8 * (e >> 2) + (e & 3);
      sa_reg[i][e] = p.sa[(int64_t)(m < (int)a.M ? m : (int)a.M - 1) * p.sa_m_stride];
    }

  for (int64_t k0 = 0; k0 < p.Kpad; k0 += IBK) {
    // activations: 128 rows x 128 bytes = 1024 x 16 B -> 4 per thread
    u4 xa[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = (tid >> 3) + 32 * i;
      const int64_t m = m0 + row, k = k0 + (tid & 7) * 16;
      xa[i] = u4{0u, 0u, 0u, 0u};
      if (m < a.M && k < p.ldq) xa[i] = *(const u4*)(p.xq + m * p.ldq + k);
    }
    // weights: 8 row blocks x 128 K.  4-bit: one tile per row block -> 512 lane slots;
    // 8-bit: two tiles per row block -> 1024 lane slots.
    constexpr int WL = WBITS == 4 ? 2 : 4;
    u4 wo[WL][WBITS == 4 ? 2 : 1];
    int wrow[WL], wcol[WL];
#pragma unroll
    for (int q = 0; q < WL; ++q) {
      const int slot = tid + 256 * q;
      int ntl, li, kt_off;
      if (WBITS == 4) {
        ntl = slot >> 6;
        li = slot & 63;
        kt_off = 0;
      } else {
        ntl = slot >> 7;
        kt_off = (slot >> 6) & 1;
        li = slot & 63;
      }
      const int r = li & 15, c = li >> 4;
      wrow[q] = ntl * 16 + r;
      wcol[q] = WBITS == 4 ? c * 32 : kt_off * 64 + c * 16;
      const int64_t nt = nt0 + ntl, kt = k0 / TK + kt_off;
      const uint32_t dead = WBITS == 4 ? (NF4 ? 0x77777777u : 0u) : 0x80808080u;
      u4 wv = u4{dead, dead, dead, dead};
      uint32_t z = WBITS == 4 ? 8u : 128u;
      if (nt < a.NT && kt < a.KT) {
        wv = *(const u4*)(a.qweight + ((nt * a.KT + kt) * 64 + li) * 16);
        if (a.zeros) {
          int64_t g = (kt * TK + c * (TK / 4)) / a.G;
          if (g >= a.KG) g = a.KG - 1;
          z = a.zeros[(nt * a.KG + g) * kTileN + r];
        }
      } else if (WBITS == 4) {
        z = 0;
      }
      const uint32_t z4 = z * 0x01010101u;
      if (WBITS == 4) {
        const i4 lo = decode16_i8<4>((const uint32_t*)&wv, z4, NF4);
        const i4 hi = decode16_i8<4>((const uint32_t*)&wv + 2, z4, NF4);
        wo[q][0] = bitcast<u4>(lo);
        wo[q][WBITS == 4 ? 1 : 0] = bitcast<u4>(hi);
      } else {
        wo[q][0] = bitcast<u4>(decode16_i8<8>((const uint32_t*)&wv, z4));
      }
    }
    // per-K-block activation scales of this step: one coalesced pass into LDS instead of 32
    // strided loads per thread and block
    float sa_stage[PER_K ? (IBK / BLOCK_K) * IBM / 256 + 1 : 1];
    int32_t za_stage[ASYM ? (IBK / BLOCK_K) * IBM / 256 + 1 : 1];
    if (PER_K) {
#pragma unroll
      for (int q = 0; q * 256 < (IBK / BLOCK_K) * IBM; ++q) {
        const int idx = tid + 256 * q;
        const int sb = idx / IBM, row = idx % IBM;
        const int64_t m = m0 + row < a.M ? m0 + row : a.M - 1;
        int kcol = (int)((unsigned)((int)k0 + sb * BLOCK_K) / (unsigned)p.qbk);
        kcol = kcol < p.sa_kc ? kcol : p.sa_kc - 1;  // K blocks of the padding past K
        sa_stage[q] = idx < (IBK / BLOCK_K) * IBM ? p.sa[m * p.sa_m_stride + kcol] : 0.0f;
        if (ASYM) za_stage[q] = idx < (IBK / BLOCK_K) * IBM ? p.za[m * p.sa_m_stride + kcol] - 128 : 0;
      }
    }
    __syncthreads();
    if (PER_K) {
#pragma unroll
      for (int q = 0; q * 256 < (IBK / BLOCK_K) * IBM; ++q)
        if (tid + 256 * q < (IBK / BLOCK_K) * IBM) {
          sSA[tid + 256 * q] = sa_stage[q];
          if (ASYM) sZA[tid + 256 * q] = za_stage[q];
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = (tid >> 3) + 32 * i;
      *(u4*)(sA + row * ILDS + (tid & 7) * 16) = xa[i];
    }
#pragma unroll
    for (int q = 0; q < WL; ++q) {
      *(u4*)(sB + wrow[q] * ILDS + wcol[q]) = wo[q][0];
      if (WBITS == 4) *(u4*)(sB + wrow[q] * ILDS + wcol[q] + 16) = wo[q][WBITS == 4 ? 1 : 0];
    }
    __syncthreads();

#pragma unroll
    for (int sb = 0; sb < sub_blocks; ++sb) {
      i16v qc[2][2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) qc[i][j][e] = 0;
      i16v qcomp[2];  // column sums of the weights of this K block (every row of the tile alike)
      if (ASYM) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) qcomp[j][e] = 0;
      }
      const int ones1 = 0x01010101;
      const i4 ones = i4{ones1, ones1, ones1, ones1};
      const int kbeg = sb * BLOCK_K;
#pragma unroll
      for (int ks = 0; ks < BLOCK_K; ks += 32) {
        i4 af[2], bf[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          af[i] = *(const i4*)(sA + (wm * 64 + i * 32 + (lane & 31)) * ILDS + kbeg + ks + (lane >> 5) * 16);
          bf[i] = *(const i4*)(sB + (wn * 64 + i * 32 + (lane & 31)) * ILDS + kbeg + ks + (lane >> 5) * 16);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            qc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], qc[i][j], 0, 0, 0);
        if (ASYM) {
          // padded K positions hold weights q = 0, not q = z: keep them out of the column sums
          const bool in_k = (int)k0 + kbeg + ks + (lane >> 5) * 16 < (int)a.K;
          const i4 ones_k = in_k ? ones : i4{0, 0, 0, 0};
#pragma unroll
          for (int j = 0; j < 2; ++j)
            qcomp[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ones_k, bf[j], qcomp[j], 0, 0, 0);
        }
      }
      // fp32 epilogue of this K block: C += (float(qC) * s_a[m]) * s_w[n, g]
      const int kq = (int)k0 + kbeg;
      int g = (int)((unsigned)kq / (unsigned)a.G);
      if (g >= (int)a.KG) g = (int)a.KG - 1;
      if (PER_K) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int e4 = 0; e4 < 4; ++e4) {
            // rows wm * 64 + 32 i + 8 e4 + 4 (lane / 32) + 0..3 of the workgroup tile
            const f4 v = *(const f4*)(sSA + sb * IBM + wm * 64 + i * 32 + 8 * e4 + 4 * (lane >> 5));
#pragma unroll
            for (int e = 0; e < 4; ++e) sa_reg[i][4 * e4 + e] = v[e];
            if (ASYM) {
              const i4 z = *(const i4*)(sZA + sb * IBM + wm * 64 + i * 32 + 8 * e4 + 4 * (lane >> 5));
#pragma unroll
              for (int e = 0; e < 4; ++e) za_reg[i][4 * e4 + e] = z[e];
            }
          }
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int n = ncol0 + j * 32;  // < NT * 16 by construction of the grid? clamp below
        const int nc = n < (int)a.NT * kTileN ? n : (int)a.NT * kTileN - 1;
        float sw = a.scales[((nc >> 4) * (int)a.KG + g) * kTileN + (nc & 15)];
        if (NF4) sw = sw * (1.0f / 127.0f);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int qv = ASYM ? qc[i][j][e] - qcomp[j][e] * za_reg[i][e] : qc[i][j][e];
            const float cterm = ((float)qv * sa_reg[i][e]) * sw;
            acc[i][j][e] = acc[i][j][e] + cterm;
            if (DEBUG) {
              // the block sum as the reference defines it: unsigned activations times weights
              const int64_t m = mrow0 + i * 32 + 8 * (e >> 2) + (e & 3);
              if (m < a.M && n < a.N && kq < (int)p.Kpad)  // (a K step may end past the padded K)
                a.debug_block_sums[(m * a.N + n) * (p.Kpad / BLOCK_K) + kq / BLOCK_K] =
                    ASYM ? qc[i][j][e] + 128 * qcomp[j][e] : qc[i][j][e];
            }
          }
        }
      }
    }
  }

  Epilogue ep{a.bias, a.fusion, a.other0, a.other1, a.out, a.out_dtype, a.x_dtype, a.N};
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t n = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int64_t m = m0 + wm * 64 + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
        if (m < a.M && n < a.N) epilogue_store<kRegimeBF16>(ep, m, n, acc[i][j][e]);
      }
    }
}

template <int WBITS, int MT, int KPW, int NTW>
static int launch_small_i8_cfg(Int8KArgs& p, hipStream_t st) {
  const size_t smem = (size_t)NTW * MT * p.W * 64 * sizeof(f4);
  auto kern = woq_small_m_i8_kernel<WBITS, MT, KPW, NTW, false>;
  if constexpr (WBITS == 4) {
    if (p.a.nf4) kern = woq_small_m_i8_kernel<WBITS, MT, KPW, NTW, true>;
  }
  if (smem > 64 * 1024) {
    hipError_t err = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (err != hipSuccess) return set_error("hipFuncSetAttribute: %s", hipGetErrorString(err));
  }
  const unsigned grid = (unsigned)((p.a.NT + NTW - 1) / NTW);
  kern<<<grid, p.W * 64, smem, st>>>(p);
  return check_launch("woq_small_m_i8_kernel");
}

template <int WBITS>
static int dispatch_small_i8(Int8KArgs& p, hipStream_t st) {
  const int64_t KT = p.a.KT, NT = p.a.NT, M = p.a.M;
  auto pick_w = [&](int kpw) {
    int64_t w = (KT + kpw - 1) / kpw;
    if (w > 16) {
      const int64_t rounds = (KT + 16 * kpw - 1) / (16 * kpw);
      w = (KT + rounds * kpw - 1) / (rounds * kpw);
    }
    return (int)(w < 1 ? 1 : w);
  };
  if (M <= 16) {
    p.W = pick_w(2);
    if (NT >= 512) return launch_small_i8_cfg<WBITS, 1, 2, 2>(p, st);
    return launch_small_i8_cfg<WBITS, 1, 2, 1>(p, st);
  } else if (M <= 32) {
    p.W = pick_w(2);
    if (NT >= 512) return launch_small_i8_cfg<WBITS, 2, 2, 2>(p, st);
    return launch_small_i8_cfg<WBITS, 2, 2, 1>(p, st);
  }
  p.W = pick_w(2);
  if (NT >= 512) return launch_small_i8_cfg<WBITS, 4, 2, 2>(p, st);
  return launch_small_i8_cfg<WBITS, 4, 2, 1>(p, st);
}

int launch_int8_linear(const Int8Args& a, hipStream_t st) {
  const int mode = a.act_quant_mode;
  if (mode < WOQ_HIP_QUANT_A_PER_TENSOR || mode > WOQ_HIP_QUANT_A_PER_M_K_BLOCK_SYM)
    return set_error("lowp_mode INT8: bad act_quant_mode %d", mode);
  const bool asym = !quant_a_is_sym(mode);
  const int TK = a.wbits == 4 ? kTileK4 : kTileK8;
  Int8KArgs p;
  p.a = a;
  p.Kpad = a.KT * TK;
  p.ldq = p.Kpad;
  const int64_t G = a.G;
  // Group-wise even when a single group covers all of K: the activation blocks then follow the
  // group size, not the K block (quant_w_mode, csrc/cpu/aten/Linear.cpp:511-513).
  const bool per_channel = a.group_size <= 0;
  p.block_k = woq_hip_int8_block_k(per_channel ? -1 : G, a.K);
  if (p.block_k % 32 != 0 || 128 % p.block_k != 0)
    return set_error("lowp_mode INT8: K block %lld (from group_size / K) must be 32, 64 or 128",
                     (long long)p.block_k);
  p.qbk = per_channel ? p.block_k : G;
  const int64_t Kc = (a.K + p.qbk - 1) / p.qbk;
  const bool per_m = quant_a_per_m(mode), per_k = quant_a_per_k(mode);
  p.sa_m_stride = per_m ? (per_k ? Kc : 1) : 0;
  p.sa_k_stride = per_k ? 1 : 0;
  if (!per_k) p.qbk = p.Kpad + 1;  // k / qbk == 0 for every k
  p.sa_kc = per_k ? (int)Kc : 1;

  // workspace: q [M][ldq] | scales [groups] | zero points [groups] (asymmetric modes)
  const int64_t qbytes = (a.M * p.ldq + 255) / 256 * 256;
  const int64_t groups = (per_m ? a.M : 1) * (per_k ? Kc : 1);
  const int64_t need = qbytes + groups * (int64_t)(sizeof(float) + (asym ? sizeof(int32_t) : 0));
  if (a.workspace == nullptr || a.workspace_bytes < need)
    return set_error("lowp_mode INT8: workspace too small (%lld < %lld bytes)", (long long)a.workspace_bytes,
                     (long long)need);
  uint8_t* xq = (uint8_t*)a.workspace;
  float* sa = (float*)((uint8_t*)a.workspace + qbytes);
  int32_t* za = asym ? (int32_t*)(sa + groups) : nullptr;
  p.xq = xq;
  p.sa = sa;
  p.za = za;
  const int64_t qbk_quant = per_k ? (per_channel ? p.block_k : G) : a.K;
  if (int rc = launch_quant_impl(a.x, a.x_dtype, a.M, a.K, p.ldq, qbk_quant, mode, xq, sa, za,
                                 a.wbits == 4 ? 1 : 0, asym ? 1 : 0, st))
    return rc;

  // Large M, 4-bit weights, one activation scale per row or tensor: the kernel that feeds the
  // decoded dwords straight to the MFMA
  if (gemm_w4i8_applies(a, p.block_k, qbk_quant, per_k, asym)) {
    // what the caller gave beyond the quantized activations and their parameters serves as scratch for
    // sharing K between workgroups (with the caller's counters)
    SplitKScratch scratch;
    const int64_t used = (need + 255) / 256 * 256;
    if (a.split_k_counters && a.workspace_bytes > used) {
      scratch.partial = (float*)((uint8_t*)a.workspace + used);
      scratch.bytes = a.workspace_bytes - used;
      scratch.counters = a.split_k_counters;
    }
    return launch_gemm_w4i8(a, xq, p.ldq, sa, p.sa_m_stride, p.sa_k_stride, qbk_quant, st, &scratch, za);
  }

  // The small-M kernel accumulates whole tiles per MFMA, so it needs K blocks that are whole
  // tiles; finer blocks (group_size 32 / 64 with 4-bit weights) go through the tiled kernel,
  // which re-lays the weights in LDS in plain K order.
  // Asymmetric activations that the kernels above do not take (8-bit or NF4 weights, groups below 128)
  // take the tiled kernel.
  if (!asym && a.M <= 64 && p.block_k % TK == 0)
    return a.wbits == 4 ? dispatch_small_i8<4>(p, st) : dispatch_small_i8<8>(p, st);
  dim3 grid((unsigned)((a.NT * kTileN + IBN - 1) / IBN), (unsigned)((a.M + IBM - 1) / IBM));
  const bool dbg = a.debug_block_sums != nullptr;
#define WOQ_I8_GEMM_B(WB, BK)                                                            \
  if (asym && dbg)                                                                       \
    woq_gemm_i8_kernel<WB, BK, true, true, true><<<grid, 256, 0, st>>>(p);               \
  else if (asym)                                                                         \
    woq_gemm_i8_kernel<WB, BK, true, false, true><<<grid, 256, 0, st>>>(p);              \
  else if (dbg)                                                                          \
    woq_gemm_i8_kernel<WB, BK, true, true, false><<<grid, 256, 0, st>>>(p);              \
  else if (per_k)                                                                        \
    woq_gemm_i8_kernel<WB, BK, true, false, false><<<grid, 256, 0, st>>>(p);             \
  else                                                                                   \
    woq_gemm_i8_kernel<WB, BK, false, false, false><<<grid, 256, 0, st>>>(p);
#define WOQ_I8_GEMM(WB)                                   \
  switch (p.block_k) {                                    \
    case 32: { WOQ_I8_GEMM_B(WB, 32) } break;             \
    case 64: { WOQ_I8_GEMM_B(WB, 64) } break;             \
    default: { WOQ_I8_GEMM_B(WB, 128) } break;            \
  }
  // NF4 codes: the same kernel with the table decode and the scale / 127 (no debug-less / per-K
  // split: the per-K-block form covers every mode)
#define WOQ_I8_GEMM_NF4(BK)                                                                   \
  if (asym && dbg)                                                                            \
    woq_gemm_i8_kernel<4, BK, true, true, true, true><<<grid, 256, 0, st>>>(p);               \
  else if (asym)                                                                              \
    woq_gemm_i8_kernel<4, BK, true, false, true, true><<<grid, 256, 0, st>>>(p);              \
  else if (dbg)                                                                               \
    woq_gemm_i8_kernel<4, BK, true, true, false, true><<<grid, 256, 0, st>>>(p);              \
  else                                                                                        \
    woq_gemm_i8_kernel<4, BK, true, false, false, true><<<grid, 256, 0, st>>>(p);
  if (a.wbits == 4 && a.nf4) {
    switch (p.block_k) {
      case 32: { WOQ_I8_GEMM_NF4(32) } break;
      case 64: { WOQ_I8_GEMM_NF4(64) } break;
      default: { WOQ_I8_GEMM_NF4(128) } break;
    }
  } else if (a.wbits == 4) {
    WOQ_I8_GEMM(4)
  } else {
    WOQ_I8_GEMM(8)
  }
#undef WOQ_I8_GEMM_NF4
#undef WOQ_I8_GEMM
#undef WOQ_I8_GEMM_B
  return check_launch("woq_gemm_i8_kernel");
}

}  // namespace woq

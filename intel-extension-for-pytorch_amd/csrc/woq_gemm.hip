// Tiled MFMA GEMM for large M (prefill): y[M, N] = x[M, K] * dequant(W)[N, K]^T.
//
// Reference counterpart: DequantGemmTPP (dequantize a [Kb x 32] weight block to a stack
// buffer, then libxsmm BRGEMM) driven by qlinear_woq_affine_impl
// (csrc/cpu/aten/utils/woq.h:1847-1944, 3104-3477).  There the block is re-dequantized for
// every M block; here a workgroup dequantizes its weight slice once per K step into LDS and all
// of its waves consume it from there.
//
// Workgroup tile BM x BN = 128 x 128, K step 64, 4 waves in a 2 x 2 grid, each wave owning a
// 64 x 64 output block as 2 x 2 v_mfma_f32_32x32x16 tiles (A = activations, B = weights, so a
// lane's accumulator registers hold consecutive n for coalesced stores).
#include "woq_common.h"
#include "woq_internal.h"

namespace woq {

template <int REGIME>
struct GemmTraits;
template <>
struct GemmTraits<kRegimeF16> {
  using vec8 = h8;
  static constexpr int act_dtype = WOQ_HIP_ACT_FP16;
  static __device__ __forceinline__ f16v mfma(h8 a, h8 b, f16v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint16_t from_f32(float f) { return f32_to_f16_bits(f); }
};
template <>
struct GemmTraits<kRegimeBF16> {
  using vec8 = b8;
  static constexpr int act_dtype = WOQ_HIP_ACT_BF16;
  static __device__ __forceinline__ f16v mfma(b8 a, b8 b, f16v c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint16_t from_f32(float f) { return f32_to_bf16_bits(f); }
};

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDS_STRIDE = BK + 8;  // elements; 16-byte pad against bank conflicts

template <int WBITS, int REGIME, bool CONV, bool NF4>
__global__ __launch_bounds__(256) void woq_gemm_kernel(const FpArgs f) {
  static_assert(!NF4 || WBITS == 4, "NF4 codes are 4 bits wide");
  using T = GemmTraits<REGIME>;
  using vec8 = typename T::vec8;
  constexpr int TK = WBITS == 4 ? kTileK4 : kTileK8;

  __shared__ __align__(16) uint16_t sA[BM * LDS_STRIDE];
  __shared__ __align__(16) uint16_t sB[BN * LDS_STRIDE];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int64_t m0 = (int64_t)blockIdx.y * BM;
  const int64_t n0 = (int64_t)blockIdx.x * BN;
  const int64_t nt0 = n0 / kTileN;
  const int64_t Kpad = f.KT * TK;

  __shared__ f2 sNf4[NF4 ? kNf4LutEntries : 1];
  constexpr bool nf4 = NF4;  // a template parameter: a runtime flag in the decode loop is not free
  if (nf4) {
    nf4_fill_lut(sNf4, (int)tid, (int)blockDim.x);
    __syncthreads();
  }

  f16v acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  for (int64_t k0 = 0; k0 < Kpad; k0 += BK) {
    // ---- global -> registers ----
    u4 xa[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = (tid >> 3) + 32 * i;
      const int64_t k = k0 + (tid & 7) * 8;
      const int64_t m = m0 + row;
      xa[i] = u4{0u, 0u, 0u, 0u};
      if (m < f.M && k < f.K) {
        if (CONV) {
          uint16_t v[8];
#pragma unroll
          for (int e = 0; e < 8; ++e)
            v[e] = (k + e < f.K) ? T::from_f32(load_act(f.x, f.x_dtype, m * f.K + k + e)) : (uint16_t)0;
#pragma unroll
          for (int e = 0; e < 4; ++e) xa[i][e] = (uint32_t)v[2 * e] | ((uint32_t)v[2 * e + 1] << 16);
        } else {
          xa[i] = *(const u4*)((const uint16_t*)f.x + m * f.K + k);
        }
      }
    }

    // weights: WBITS == 4: one dwordx4 per thread (half a tile row block: 32 K values of one
    // row); WBITS == 8: two dwordx4 per thread (16 K values each).
    constexpr int WLOADS = WBITS == 4 ? 1 : 2;
    u4 wv[WLOADS];
    vec8 wd[4];
    int wrow[WLOADS], wcol[WLOADS];
#pragma unroll
    for (int q = 0; q < WLOADS; ++q) {
      int ntl, r, c;
      if (WBITS == 4) {
        ntl = tid >> 5;  // 8 row blocks of 16
        const int li = tid & 31;
        r = li & 15;
        c = (int)((k0 % TK) / 32) + (li >> 4);
        wcol[q] = (li >> 4) * 32;
      } else {
        const int slot = tid + 256 * q;  // 512 lane slots
        ntl = slot >> 6;
        const int li = slot & 63;
        r = li & 15;
        c = li >> 4;
        wcol[q] = c * 16;
      }
      wrow[q] = ntl * 16 + r;
      const int64_t nt = nt0 + ntl, kt = k0 / TK;
      wv[q] = u4{0u, 0u, 0u, 0u};
      uint16_t sbits = 0;
      uint8_t zb = 0;
      const bool valid = nt < f.NT;
      if (valid) {
        wv[q] = *(const u4*)(f.qweight + ((nt * f.KT + kt) * 64 + (r + 16 * c)) * 16);
        int64_t g = (kt * TK + c * (TK / 4)) / f.G;
        if (g >= f.KG) g = f.KG - 1;
        const int64_t qi = (nt * f.KG + g) * kTileN + r;
        sbits = f.scales[qi];
        if (f.zeros) zb = f.zeros[qi];
      }
      const float z = f.zeros ? (float)zb : (WBITS == 4 ? 8.0f : 128.0f);
      if (nf4) {
        const float s = REGIME == kRegimeF16 ? f16_bits_to_f32(sbits) : bf16_bits_to_f32(sbits);
#pragma unroll
        for (int j = 0; j < 4; ++j) wd[j] = bitcast<vec8>(nf4_dequant<REGIME>(wv[q][j], sNf4, s));
      } else if (WBITS == 4) {
        if constexpr (REGIME == kRegimeF16) {
          const _Float16 s = bitcast<_Float16>(sbits);
          const _Float16 nz = (_Float16)(-(1024.0f + z));
#pragma unroll
          for (int j = 0; j < 4; ++j) wd[j] = dequant8_f16(wv[q][j], h2{nz, nz}, h2{s, s});
        } else {
          const float s = bf16_bits_to_f32(sbits);
          const float cc = -((1024.0f + z) * s);
#pragma unroll
          for (int j = 0; j < 4; ++j) wd[j] = dequant8_bf16(wv[q][j], s, cc);
        }
      } else {
        const float s = REGIME == kRegimeF16 ? f16_bits_to_f32(sbits) : bf16_bits_to_f32(sbits);
        const float cc = -(z * s);
        if (f.fp8) {  // (uniform) float8 e4m3fn bytes
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            if constexpr (REGIME == kRegimeF16)
              wd[2 * q + j] = dequant8_f16_fp8(wv[q][2 * j], wv[q][2 * j + 1], s);
            else
              wd[2 * q + j] = dequant8_bf16_fp8(wv[q][2 * j], wv[q][2 * j + 1], s);
          }
        } else {
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            if constexpr (REGIME == kRegimeF16)
              wd[2 * q + j] = dequant8_f16_w8(wv[q][2 * j], wv[q][2 * j + 1], s, cc);
            else
              wd[2 * q + j] = dequant8_bf16_w8(wv[q][2 * j], wv[q][2 * j + 1], s, cc);
          }
        }
      }
    }

    __syncthreads();  // previous step's MFMA reads are done
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = (tid >> 3) + 32 * i;
      *(u4*)(sA + row * LDS_STRIDE + (tid & 7) * 8) = xa[i];
    }
    if (WBITS == 4) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        *(vec8*)(sB + wrow[0] * LDS_STRIDE + wcol[0] + j * 8) = wd[j];
    } else {
#pragma unroll
      for (int q = 0; q < WLOADS; ++q)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          *(vec8*)(sB + wrow[q] * LDS_STRIDE + wcol[q] + j * 8) = wd[2 * q + j];
    }
    __syncthreads();

    // ---- MFMA over the K step ----
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      vec8 af[2], bf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int row = wm * 64 + i * 32 + (lane & 31);
        af[i] = *(const vec8*)(sA + row * LDS_STRIDE + ks * 16 + (lane >> 5) * 8);
        const int col = wn * 64 + i * 32 + (lane & 31);
        bf[i] = *(const vec8*)(sB + col * LDS_STRIDE + ks * 16 + (lane >> 5) * 8);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = T::mfma(af[i], bf[j], acc[i][j]);
    }
  }

  // ---- epilogue: D[m][n], lane holds n = lane % 32, m = 8*(e/4) + 4*(lane/32) + e%4 ----
  Epilogue ep{f.bias, f.fusion, f.other0, f.other1, f.out, f.out_dtype, f.x_dtype, f.N};
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t n = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int64_t m = m0 + wm * 64 + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
        if (m < f.M && n < f.N) epilogue_store<REGIME>(ep, m, n, acc[i][j][e]);
      }
    }
}

template <int WBITS, int REGIME>
static int launch_gemm_cfg(const FpArgs& f, bool conv, hipStream_t st) {
  dim3 grid((unsigned)((f.NT * kTileN + BN - 1) / BN), (unsigned)((f.M + BM - 1) / BM));
  auto kern = conv ? woq_gemm_kernel<WBITS, REGIME, true, false> : woq_gemm_kernel<WBITS, REGIME, false, false>;
  if constexpr (WBITS == 4) {
    if (f.nf4) kern = conv ? woq_gemm_kernel<WBITS, REGIME, true, true> : woq_gemm_kernel<WBITS, REGIME, false, true>;
  }
  kern<<<grid, 256, 0, st>>>(f);
  return check_launch("woq_gemm_kernel");
}

int launch_gemm(const FpArgs& f, int wbits, int regime, hipStream_t st) {
  const int want = regime == kRegimeF16 ? WOQ_HIP_ACT_FP16 : WOQ_HIP_ACT_BF16;
  const bool conv = f.x_dtype != want || (f.K % 8) != 0;
  if (wbits == 4)
    return regime == kRegimeF16 ? launch_gemm_cfg<4, kRegimeF16>(f, conv, st)
                                : launch_gemm_cfg<4, kRegimeBF16>(f, conv, st);
  return regime == kRegimeF16 ? launch_gemm_cfg<8, kRegimeF16>(f, conv, st)
                              : launch_gemm_cfg<8, kRegimeBF16>(f, conv, st);
}

}  // namespace woq

// Decode kernel for the fp16 regime (M < 5 under lowp_mode BF16 or FP16) with 4-bit weights and
// group sizes that are multiples of 128: HBM-bound weight streaming.
//
// Reference counterpart: the small-batch FMA micro-kernel, which keeps the weights as exact small
// integers and applies the group scale to the block sum (csrc/cpu/aten/utils/woq.h:775-951:
// vc = sum a_k * (q_k - z), then C = fma(s, vc, C)).  The same algebra is used here, with fp32
// instead of fp16 accumulators:
//     y[m, n] = sum_g s[n, g] * ( sum_{k in g} x[m, k] * (c + q[n, k])  -  (c + z[n, g]) * sum_{k in g} x[m, k] )
// c = 128 (bf16 activations) or 1024 (fp16 activations) is the magic constant that turns a nibble
// into a bf16 / fp16 value with a single v_and_or_b32 per pair: 0x4300 | q is the bf16 number
// 128 + q.  The products x * (c + q) are exact in the MFMA and the sums are accumulated in fp32;
// sum_k x comes from one extra MFMA whose B operand is the constant -1, shared by every weight
// tile of the same K range.
//
// Mapping: v_mfma_f32_16x16x32 with A = activations (row m = lane % 16) and B = weights (column
// n = lane % 16), so a lane's four accumulator registers are rows m = 4 * (lane / 16) + e of its
// own output column and one (scale, zero) dword per lane and tile serves the epilogue.
// A workgroup owns NTW weight tiles (16 rows each) and all of K; its W waves split K in rounds of
// W * 2 K-tiles.  Every global load is unconditional (indices are clamped and the contribution
// of an out-of-range tile is cancelled by a zero scale) so that the compiler can count
// outstanding loads and start on the first tile while the rest are in flight.  Each wave keeps
// its own slice of the activations in a private LDS region: no workgroup barrier before the
// final cross-wave sum, which is done in wave order (deterministic).
#include "woq_common.h"
#include "woq_internal.h"

namespace woq {

constexpr int kDecodeKPW = 2;

// (a & mask) | magic with both constants held in registers (their values are hidden from the
// optimizer), which the compiler selects as one v_and_or_b32 instead of a literal AND plus a
// literal OR.
__device__ __forceinline__ uint32_t v_and_or(uint32_t a, uint32_t mask, uint32_t orv) { return (a & mask) | orv; }

__device__ __forceinline__ float fma_f16lo(float a, uint32_t h, float c) {
  return __builtin_fmaf(a, (float)bitcast<h2>(h)[0], c);
}
__device__ __forceinline__ float fma_f16hi(float a, uint32_t h, float c) {
  return __builtin_fmaf(a, (float)bitcast<h2>(h)[1], c);
}

template <bool XF16>
__device__ __forceinline__ f4 mfma16(u4 a, u4 b, f4 c) {
  if constexpr (XF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(bitcast<h8>(a), bitcast<h8>(b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(bitcast<b8>(a), bitcast<b8>(b), c, 0, 0, 0);
}

template <bool XF16, int NTW, int MAXM, bool ONE_ROUND>
__global__ __launch_bounds__(1024, 8) void woq_decode_kernel(const DecodeArgs a) {
  constexpr int KPW = kDecodeKPW;
  constexpr int SLICE = KPW * kTileK4;  // K elements of one wave per round
  extern __shared__ __align__(16) uint8_t smem[];
  const int W = a.W;
  const int lane = threadIdx.x & 63;
  // the wave index is uniform: keeping it in an SGPR moves the tile / group address arithmetic to
  // the scalar unit and leaves one VGPR offset per stream
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int r = lane & 15, c = lane >> 4;
  const int64_t nt0 = (int64_t)blockIdx.x * NTW;

  uint16_t* sx = (uint16_t*)smem + (size_t)wave * MAXM * SLICE;            // private [MAXM][SLICE]
  f4* red = (f4*)(smem + (size_t)W * MAXM * SLICE * sizeof(uint16_t));     // [NTW][W][16]

  uint32_t mask, magic;
  asm volatile("s_mov_b32 %0, 0x000F000F" : "=s"(mask));
  if (XF16)
    asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic));
  else
    asm volatile("v_mov_b32 %0, 0x43004300" : "=v"(magic));
  const uint32_t n1 = XF16 ? 0xBC00BC00u : 0xBF80BF80u;  // -1 in every slot
  const u4 neg1 = u4{n1, n1, n1, n1};

  f4 acc[NTW];
#pragma unroll
  for (int t = 0; t < NTW; ++t) acc[t] = f4{0.f, 0.f, 0.f, 0.f};

  const int NT = (int)a.NT, KT = (int)a.KT, KG = (int)a.KG;
  const int tpg_shift = a.tpg_shift;  // log2(tiles per group)
  const int xlane = lane & (KPW * 16 - 1);  // lanes 32..63 mirror 0..31
  (void)NT;
  const int xrow = r < MAXM ? r : 0;

  // 32-bit offsets from uniform base pointers keep the per-lane address state in one VGPR each
  // (the packed weight, its parameters and the activations are each far below 4 GiB)
  const int K = (int)a.K, M = (int)a.M;
  // ONE_ROUND: the W waves cover K exactly once (K == W * KPW * 128), the common decode case
  const int rounds = ONE_ROUND ? 1 : (KT + W * KPW - 1) / (W * KPW);
#pragma unroll 1
  for (int rd = 0; rd < rounds; ++rd) {
    const int ktw = (rd * W + wave) * KPW;
    // The launcher guarantees K % (KPW * 128) == 0 and NT % NTW == 0, so a wave either has a
    // full slice of work or none: no clamped addresses, no selects between the loads.
    if (!ONE_ROUND && ktw >= KT) break;

    // ---- this wave's slice of the activations: issued first, so it is the first to return ----
    u4 xs[MAXM];
    const uint8_t* xbase = (const uint8_t*)a.x + (size_t)ktw * kTileK4 * 2;  // uniform
#pragma unroll
    for (int m = 0; m < MAXM; ++m) {
      const int mm = m < M ? m : M - 1;
      xs[m] = *(const u4*)(xbase + (size_t)mm * K * 2 + (uint32_t)xlane * 16u);
    }

    // ---- the weight stream of this round, in the order it is consumed: one KiB tile per load,
    // all in flight together; uniform bases + one per-lane offset ----
    u4 wreg[NTW][KPW];
    uint32_t szreg[NTW][KPW];
#pragma unroll
    for (int i = 0; i < KPW; ++i) {
      const int kt = ktw + i;
      int g = kt >> tpg_shift;
      g = g < KG ? g : KG - 1;
#pragma unroll
      for (int t = 0; t < NTW; ++t) {
        const size_t nt = (size_t)nt0 + t;
        const uint8_t* wb = a.qweight + (nt * KT + kt) * kTileBytes;                      // uniform
        const uint8_t* sb = (const uint8_t*)a.sz + (nt * KG + g) * (kTileN * sizeof(uint32_t));  // uniform
        wreg[t][i] = __builtin_nontemporal_load((const u4*)(wb + (uint32_t)lane * 16u));
        szreg[t][i] = *(const uint32_t*)(sb + (uint32_t)r * 4u);
      }
    }

    // Every load of the round stays ahead of the first use: the scheduler would otherwise sink
    // some of them below the first s_waitcnt to save registers, exposing a full memory round
    // trip in the middle of the round.
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < MAXM; ++m) *(u4*)(sx + m * SLICE + xlane * 8) = xs[m];

#pragma unroll
    for (int i = 0; i < KPW; ++i) {
      // -sum_k x of this K tile (shared by the NTW weight tiles)
      f4 d1 = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const u4 xa = *(const u4*)(sx + xrow * SLICE + i * kTileK4 + c * 32 + j * 8);
        d1 = mfma16<XF16>(xa, neg1, d1);
      }
#pragma unroll
      for (int t = 0; t < NTW; ++t) {
        f4 dw = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const u4 xa = *(const u4*)(sx + xrow * SLICE + i * kTileK4 + c * 32 + j * 8);
          const uint32_t d = wreg[t][i][j];
          u4 bop;
          bop[0] = v_and_or(d, mask, magic);
          bop[1] = v_and_or(d >> 4, mask, magic);
          bop[2] = v_and_or(d >> 8, mask, magic);
          bop[3] = v_and_or(d >> 12, mask, magic);
          dw = mfma16<XF16>(xa, bop, dw);
        }
        // dw = sum x (c + q), d1 = -sum x;  group term = s * (dw + (128 + z) * d1 [+ 896 * d1])
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float base = dw[e];
          if (XF16) base = __builtin_fmaf(d1[e], 896.0f, base);
          const float tsum = fma_f16hi(d1[e], szreg[t][i], base);
          acc[t][e] = fma_f16lo(tsum, szreg[t][i], acc[t][e]);
        }
      }
    }
  }

  // ---- combine the waves' partial sums in wave order, then bias / rounding / store ----
  // Only lanes 0..15 hold rows m = 0..3 (M <= 4); they publish their four accumulators.
  if (c == 0) {
#pragma unroll
    for (int t = 0; t < NTW; ++t) red[(t * W + wave) * 16 + r] = acc[t];
  }
  __syncthreads();

  Epilogue ep{a.bias, a.fusion, a.other0, a.other1, a.out, a.out_dtype, a.x_dtype, a.N};
  const float* redf = (const float*)red;
  // one thread per output element (tile, column, row); its W <= 16 partial sums are fetched with
  // independent LDS reads (a rolled loop would pay one LDS round trip per wave) and added in wave
  // order
  for (int idx = threadIdx.x; idx < NTW * 64; idx += blockDim.x) {
    const int e = idx & 3, col = (idx >> 2) & 15, t = idx >> 6;
    const int64_t n = (nt0 + t) * kTileN + col;
    if (e >= M || n >= a.N) continue;
    float part[16];
#pragma unroll
    for (int w = 0; w < 16; ++w) part[w] = w < W ? redf[((t * W + w) * 16 + col) * 4 + e] : 0.0f;
    float s = part[0];
#pragma unroll
    for (int w = 1; w < 16; ++w) s += part[w];
    // plain case first: bf16 in / out, no bias, no post-op -> fp16 rounding then bf16 store
    if (a.fusion == WOQ_HIP_FUSE_NONE && a.bias == nullptr && a.out_dtype == WOQ_HIP_ACT_BF16)
      ((uint16_t*)a.out)[(int64_t)e * a.N + n] = f32_to_bf16_bits((float)(_Float16)s);
    else
      epilogue_store<kRegimeF16>(ep, e, n, s);
  }
}

template <bool XF16, int NTW, int MAXM, bool ONE_ROUND>
static int launch_decode_cfg(const DecodeArgs& a, hipStream_t st) {
  const size_t smem = (size_t)NTW * a.W * 16 * sizeof(f4) +
                      (size_t)a.W * MAXM * kDecodeKPW * kTileK4 * sizeof(uint16_t);
  auto kern = woq_decode_kernel<XF16, NTW, MAXM, ONE_ROUND>;
  if (smem > 64 * 1024) {
    hipError_t err = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (err != hipSuccess) return set_error("hipFuncSetAttribute: %s", hipGetErrorString(err));
  }
  const unsigned grid = (unsigned)((a.NT + NTW - 1) / NTW);
  kern<<<grid, a.W * 64, smem, st>>>(a);
  return check_launch("woq_decode_kernel");
}

bool decode_kernel_applies(const FpArgs& f, int wbits, int regime, const uint32_t* sz) {
  const int64_t tpg = f.G / kTileK4;
  return sz != nullptr && wbits == 4 && regime == kRegimeF16 && f.M <= 4 && (f.G % kTileK4) == 0 &&
         (tpg & (tpg - 1)) == 0 && (f.K % (kDecodeKPW * kTileK4)) == 0 && (f.x_dtype == WOQ_HIP_ACT_BF16 || f.x_dtype == WOQ_HIP_ACT_FP16);
}

int launch_decode(const FpArgs& f, const uint32_t* sz, hipStream_t st) {
  DecodeArgs a;
  a.x = (const uint16_t*)f.x;
  a.x_dtype = f.x_dtype;
  a.M = f.M; a.K = f.K; a.N = f.N; a.NT = f.NT; a.KT = f.KT;
  a.qweight = f.qweight;
  a.sz = sz;
  a.G = f.G; a.KG = f.KG;
  a.bias = f.bias; a.fusion = f.fusion; a.other0 = f.other0; a.other1 = f.other1;
  a.out = f.out; a.out_dtype = f.out_dtype;
  a.Kpad = f.KT * kTileK4;
  a.tpg_shift = 0;
  while ((int64_t)kTileK4 << (a.tpg_shift + 1) <= f.G && a.tpg_shift < 30) ++a.tpg_shift;
  // waves per workgroup: cover K in as few equal rounds as possible, at most 16 waves
  int64_t w = (f.KT + kDecodeKPW - 1) / kDecodeKPW;
  if (w > 16) {
    const int64_t rounds = (w + 15) / 16;
    w = (w + rounds - 1) / rounds;
  }
  a.W = (int)w;
  const bool xf16 = f.x_dtype == WOQ_HIP_ACT_FP16;
  const bool two = f.NT >= 512 && f.NT % 2 == 0;
  const bool one_row = f.M == 1;
  const bool one_round = f.KT == (int64_t)a.W * kDecodeKPW;
#define WOQ_DECODE(XF, NTW)                                                                             \
  (one_row ? (one_round ? launch_decode_cfg<XF, NTW, 1, true>(a, st) : launch_decode_cfg<XF, NTW, 1, false>(a, st)) \
           : (one_round ? launch_decode_cfg<XF, NTW, 4, true>(a, st) : launch_decode_cfg<XF, NTW, 4, false>(a, st)))
  if (xf16) return two ? WOQ_DECODE(true, 2) : WOQ_DECODE(true, 1);
  return two ? WOQ_DECODE(false, 2) : WOQ_DECODE(false, 1);
#undef WOQ_DECODE
}

}  // namespace woq

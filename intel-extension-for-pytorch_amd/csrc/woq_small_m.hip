// Small-M (decode) kernel: streams the packed weight from HBM exactly once and feeds MFMA.
//
// Reference counterpart: the M < 5 FMA micro-kernel and the small-M BRGEMM calls of
// qlinear_woq_affine_impl (csrc/cpu/aten/utils/woq.h:775-951, 1847-1944, 2748-3509).
//
// Mapping to the machine:
//   * a workgroup owns NTW consecutive 16-row weight tiles and the whole K extent; its W
//     waves split K, each wave taking KPW consecutive K-tiles per round of W*KPW tiles;
//   * one global_load_dwordx4 per lane fetches a whole 1 KiB tile (16 rows x 128 int4 or
//     16 rows x 64 int8); nibbles are decoded in registers into the MFMA A operand;
//   * the activations of the wave's K range are the MFMA B operand; they are loaded once per
//     round and stay in registers while the wave walks over its NTW weight tiles, so the
//     weight stream is the only per-tile memory traffic;
//   * v_mfma_f32_16x16x32_{f16,bf16}: D[n][m] += W[n][k] * X[m][k], fp32 accumulate;
//   * the W partial results are summed through LDS in a fixed order (deterministic), then
//     bias / rounding / post-op / store.
#include "woq_common.h"
#include "woq_internal.h"

namespace woq {

template <int REGIME>
struct RegimeTraits;
template <>
struct RegimeTraits<kRegimeF16> {
  using vec8 = h8;
  static constexpr int act_dtype = WOQ_HIP_ACT_FP16;
  static __device__ __forceinline__ f4 mfma(h8 a, h8 b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint16_t from_f32(float f) { return f32_to_f16_bits(f); }
};
template <>
struct RegimeTraits<kRegimeBF16> {
  using vec8 = b8;
  static constexpr int act_dtype = WOQ_HIP_ACT_BF16;
  static __device__ __forceinline__ f4 mfma(b8 a, b8 b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint16_t from_f32(float f) { return f32_to_bf16_bits(f); }
};

// Per-lane dequantization parameters of one tile.
template <int WBITS, int REGIME>
struct LaneQ {
  // fp16 regime, 4-bit: nz = -(1024 + z) and s as fp16 pairs.  Everything else: s and
  // c = -(offset + z) * s in fp32.
  h2 nz, s2;
  float s, c;
};

template <int WBITS, int REGIME>
__device__ __forceinline__ LaneQ<WBITS, REGIME> make_laneq(uint16_t sbits, bool has_z, uint8_t zbyte) {
  LaneQ<WBITS, REGIME> q;
  // symmetric: INT4 is stored +8 (quantize_per_block, _quantize_utils.py:1141), INT8 bytes are
  // offset-binary, so the implied zero is 8 / 128.
  const float z = has_z ? (float)zbyte : (WBITS == 4 ? 8.0f : 128.0f);
  if (REGIME == kRegimeF16) {
    const _Float16 s = bitcast<_Float16>(sbits);
    if (WBITS == 4) {
      const _Float16 nz = (_Float16)(-(1024.0f + z));
      q.nz = h2{nz, nz};
      q.s2 = h2{s, s};
    }
    q.s = (float)s;
    q.c = -(z * q.s);
  } else {
    q.s = bf16_bits_to_f32(sbits);
    q.c = WBITS == 4 ? -((1024.0f + z) * q.s) : -(z * q.s);
  }
  return q;
}

template <int WBITS, int REGIME>
__device__ __forceinline__ void dequant_tile(const u4& w, const LaneQ<WBITS, REGIME>& q,
                                             typename RegimeTraits<REGIME>::vec8 (&a)[WBITS == 4 ? 4 : 2],
                                             bool fp8 = false) {
  if (WBITS == 4) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if constexpr (REGIME == kRegimeF16)
        a[j] = dequant8_f16(w[j], q.nz, q.s2);
      else
        a[j] = dequant8_bf16(w[j], q.s, q.c);
    }
  } else if (fp8) {  // (uniform) float8 e4m3fn bytes
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if constexpr (REGIME == kRegimeF16)
        a[j] = dequant8_f16_fp8(w[2 * j], w[2 * j + 1], q.s);
      else
        a[j] = dequant8_bf16_fp8(w[2 * j], w[2 * j + 1], q.s);
    }
  } else {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if constexpr (REGIME == kRegimeF16)
        a[j] = dequant8_f16_w8(w[2 * j], w[2 * j + 1], q.s, q.c);
      else
        a[j] = dequant8_bf16_w8(w[2 * j], w[2 * j + 1], q.s, q.c);
    }
  }
}

struct SmallMArgs {
  FpArgs f;
  int W;          // waves per workgroup
  int64_t Kpad;   // KT * tile_k
};

template <int WBITS, int REGIME, int MT, int KPW, int NTW, bool CONV, bool NF4>
__global__ __launch_bounds__(1024) void woq_small_m_kernel(const SmallMArgs a) {
  static_assert(!NF4 || WBITS == 4, "NF4 codes are 4 bits wide");
  using T = RegimeTraits<REGIME>;
  using vec8 = typename T::vec8;
  constexpr int TK = WBITS == 4 ? kTileK4 : kTileK8;
  constexpr int STEPS = WBITS == 4 ? 4 : 2;
  constexpr int CK = TK / 4;  // K elements per lane column c

  extern __shared__ __align__(16) uint8_t smem[];
  const int W = a.W;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, c = lane >> 4;
  const int64_t nt0 = (int64_t)blockIdx.x * NTW;
  const int64_t KC = (int64_t)W * KPW * TK;  // K elements per round
  const FpArgs& f = a.f;

  f4* red = (f4*)smem;                                                 // [NTW][MT][W][64]
  uint16_t* sx = (uint16_t*)(smem + (size_t)NTW * MT * W * 64 * sizeof(f4));  // [rows][KC]
  const int rows = (int)(f.M < MT * 16 ? f.M : MT * 16);

  __shared__ f2 sNf4[NF4 ? kNf4LutEntries : 1];
  constexpr bool nf4 = NF4;  // a template parameter: a runtime flag in the decode loop is not free
  if (nf4) {
    nf4_fill_lut(sNf4, (int)threadIdx.x, (int)blockDim.x);
    __syncthreads();
  }

  f4 acc[NTW][MT];
#pragma unroll
  for (int t = 0; t < NTW; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f4{0.f, 0.f, 0.f, 0.f};

  for (int64_t kc0 = 0; kc0 < a.Kpad; kc0 += KC) {
    const int64_t ktw = kc0 / TK + (int64_t)wave * KPW;  // first K-tile of this wave

    // ---- issue the weight stream of this round first: it has the longest latency ----
    u4 wreg[NTW][KPW];
    uint16_t sreg[NTW][KPW];
    uint8_t zreg[NTW][KPW];
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
      const int64_t nt = nt0 + t;
#pragma unroll
      for (int i = 0; i < KPW; ++i) {
        // unconditional loads from clamped indices: the compiler can then count outstanding
        // loads and start on the first tile while the others are in flight; a zero scale
        // cancels a clamped tile
        const int64_t ktr = ktw + i;
        const bool live = nt < f.NT && ktr < f.KT;
        const int64_t ntc = nt < f.NT ? nt : f.NT - 1;
        const int64_t kt = ktr < f.KT ? ktr : f.KT - 1;
        wreg[t][i] = __builtin_nontemporal_load((const u4*)(f.qweight + ((ntc * f.KT + kt) * 64 + lane) * 16));
        int64_t g = (kt * TK + c * CK) / f.G;
        if (g >= f.KG) g = f.KG - 1;
        const int64_t qi = (ntc * f.KG + g) * kTileN + r;
        const uint16_t sb = f.scales[qi];
        sreg[t][i] = live ? sb : (uint16_t)0;
        zreg[t][i] = f.zeros ? f.zeros[qi] : (uint8_t)0;
      }
    }

    // ---- activations of this wave's K range -> B operands ----
    if (CONV) {
      __syncthreads();  // readers of the previous round are done
      const int64_t n8 = (int64_t)rows * (KC / 8);
      for (int64_t idx = threadIdx.x; idx < n8; idx += blockDim.x) {
        const int64_t row = idx / (KC / 8), k = kc0 + (idx % (KC / 8)) * 8;
        uint16_t v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e)
          v[e] = (k + e < f.K) ? T::from_f32(load_act(f.x, f.x_dtype, row * f.K + k + e)) : (uint16_t)0;
        u4 pk;
#pragma unroll
        for (int e = 0; e < 4; ++e) pk[e] = (uint32_t)v[2 * e] | ((uint32_t)v[2 * e + 1] << 16);
        *(u4*)(sx + row * KC + (k - kc0)) = pk;
      }
      __syncthreads();
    }
    vec8 xb[KPW][STEPS][MT];
#pragma unroll
    for (int i = 0; i < KPW; ++i) {
#pragma unroll
      for (int j = 0; j < STEPS; ++j) {
        const int64_t k = (ktw + i) * TK + c * CK + j * 8;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const int64_t row = mt * 16 + r;
          const bool ok = row < f.M && k < f.K;
          const int64_t rowc = row < f.M ? row : f.M - 1;
          const int64_t kc = k < f.K ? k : 0;
          u4 v;
          if (CONV)
            v = *(const u4*)(sx + (rowc < rows ? rowc : 0) * KC + (ok ? k - kc0 : 0));
          else
            v = *(const u4*)((const uint16_t*)f.x + rowc * f.K + kc);
          v = ok ? v : u4{0u, 0u, 0u, 0u};
          xb[i][j][mt] = bitcast<vec8>(v);
        }
      }
    }

    // ---- decode + MFMA ----
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
#pragma unroll
      for (int i = 0; i < KPW; ++i) {
        const LaneQ<WBITS, REGIME> q = make_laneq<WBITS, REGIME>(sreg[t][i], f.zeros != nullptr, zreg[t][i]);
        vec8 aop[STEPS];
        if (nf4) {
          const float s = REGIME == kRegimeF16 ? f16_bits_to_f32(sreg[t][i]) : bf16_bits_to_f32(sreg[t][i]);
#pragma unroll
          for (int j = 0; j < STEPS; ++j) aop[j] = bitcast<vec8>(nf4_dequant<REGIME>(wreg[t][i][j], sNf4, s));
        } else {
          dequant_tile<WBITS, REGIME>(wreg[t][i], q, aop, WBITS == 8 && f.fp8);
        }
#pragma unroll
        for (int j = 0; j < STEPS; ++j)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) acc[t][mt] = T::mfma(aop[j], xb[i][j][mt], acc[t][mt]);
      }
    }
  }

  // ---- cross-wave reduction in wave order, then epilogue ----
  if (CONV) __syncthreads();
#pragma unroll
  for (int t = 0; t < NTW; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[((t * MT + mt) * W + wave) * 64 + lane] = acc[t][mt];
  __syncthreads();

  Epilogue e{f.bias, f.fusion, f.other0, f.other1, f.out, f.out_dtype, f.x_dtype, f.N};
  for (int idx = threadIdx.x; idx < NTW * MT * 64; idx += blockDim.x) {
    const int ln = idx & 63, tm = idx >> 6;
    const int t = tm / MT, mt = tm % MT;
    f4 s = red[(tm * W) * 64 + ln];
    for (int w = 1; w < W; ++w) {
      const f4 v = red[(tm * W + w) * 64 + ln];
      s[0] += v[0];
      s[1] += v[1];
      s[2] += v[2];
      s[3] += v[3];
    }
    const int64_t m = mt * 16 + (ln & 15);
    const int64_t n = (nt0 + t) * kTileN + 4 * (ln >> 4);
    if (m < f.M) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n + i < f.N) epilogue_store<REGIME>(e, m, n + i, s[i]);
    }
  }
}

template <int WBITS, int REGIME, int MT, int KPW, int NTW, bool CONV>
static int launch_cfg(SmallMArgs& a, hipStream_t st) {
  constexpr int TK = WBITS == 4 ? kTileK4 : kTileK8;
  auto smem_for = [&](int W) {
    size_t smem = (size_t)NTW * MT * W * 64 * sizeof(f4);
    if (CONV) {
      const int64_t rows = a.f.M < MT * 16 ? a.f.M : MT * 16;
      smem += (size_t)rows * W * KPW * TK * sizeof(uint16_t);
    }
    return smem;
  };
  // the staging buffer of converted activations grows with W: fewer waves, more rounds
  while (a.W > 1 && smem_for(a.W) > 96 * 1024) a.W = (a.W + 1) / 2;
  const int W = a.W;
  const size_t smem = smem_for(W);
  auto kern = woq_small_m_kernel<WBITS, REGIME, MT, KPW, NTW, CONV, false>;
  if constexpr (WBITS == 4) {
    if (a.f.nf4) kern = woq_small_m_kernel<WBITS, REGIME, MT, KPW, NTW, CONV, true>;
  }
  if (smem > 160 * 1024) return set_error("small-M kernel: LDS request %zu exceeds 160 KiB", smem);
  if (smem > 64 * 1024) {
    hipError_t err = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)smem);
    if (err != hipSuccess) return set_error("hipFuncSetAttribute: %s", hipGetErrorString(err));
  }
  const unsigned grid = (unsigned)((a.f.NT + NTW - 1) / NTW);
  kern<<<grid, W * 64, smem, st>>>(a);
  return check_launch("woq_small_m_kernel");
}

template <int WBITS, int REGIME, bool CONV>
static int dispatch_shape(SmallMArgs& a, hipStream_t st) {
  constexpr int TK = WBITS == 4 ? kTileK4 : kTileK8;
  const int64_t M = a.f.M, KT = a.f.KT, NT = a.f.NT;
  // Waves per workgroup: enough to cover K in few rounds, at most 16.
  auto pick_w = [&](int kpw) {
    int64_t w = (KT + kpw - 1) / kpw;
    if (w > 16) {
      // spread K-tiles evenly over the rounds
      const int64_t rounds = (KT + 16 * kpw - 1) / (16 * kpw);
      w = (KT + rounds * kpw - 1) / (rounds * kpw);
    }
    return (int)(w < 1 ? 1 : w);
  };
  (void)TK;
  if (M <= 16) {
    // two weight tiles per workgroup once there are enough tiles to fill the chip twice over
    if (NT >= 512) {
      a.W = pick_w(2);
      return launch_cfg<WBITS, REGIME, 1, 2, 2, CONV>(a, st);
    }
    a.W = pick_w(2);
    return launch_cfg<WBITS, REGIME, 1, 2, 1, CONV>(a, st);
  } else if (M <= 32) {
    a.W = pick_w(2);
    if (NT >= 512) return launch_cfg<WBITS, REGIME, 2, 2, 2, CONV>(a, st);
    return launch_cfg<WBITS, REGIME, 2, 2, 1, CONV>(a, st);
  } else {
    a.W = pick_w(1);
    if (NT >= 512) return launch_cfg<WBITS, REGIME, 4, 1, 2, CONV>(a, st);
    return launch_cfg<WBITS, REGIME, 4, 1, 1, CONV>(a, st);
  }
}

int launch_small_m(const FpArgs& f, int wbits, int regime, hipStream_t st) {
  if (f.M > 64) return set_error("small-M kernel supports M <= 64, got %lld", (long long)f.M);
  SmallMArgs a;
  a.f = f;
  a.W = 1;
  a.Kpad = f.KT * (wbits == 4 ? kTileK4 : kTileK8);
  const int want = regime == kRegimeF16 ? WOQ_HIP_ACT_FP16 : WOQ_HIP_ACT_BF16;
  const bool conv = f.x_dtype != want || (f.K % 8) != 0;
#define WOQ_DISPATCH(WB, RG)                                            \
  (conv ? dispatch_shape<WB, RG, true>(a, st) : dispatch_shape<WB, RG, false>(a, st))
  if (wbits == 4)
    return regime == kRegimeF16 ? WOQ_DISPATCH(4, kRegimeF16) : WOQ_DISPATCH(4, kRegimeBF16);
  return regime == kRegimeF16 ? WOQ_DISPATCH(8, kRegimeF16) : WOQ_DISPATCH(8, kRegimeBF16);
#undef WOQ_DISPATCH
}

}  // namespace woq

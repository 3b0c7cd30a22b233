// Decode kernel for the fp16 regime (M < 5 under lowp_mode BF16 or FP16) with 4-bit weights and
// group sizes that are multiples of 128, or 64, or 32: HBM-bound weight streaming.
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

// GPT = 4 or 2 groups per K tile (groups of 32 or 64 input channels): a lane column's 32 K values of a tile belong to
// one group, but an MFMA sums over the four lane columns.  The rows of the A operand keep the groups apart: row
// 4 g + m carries activation row m in the lane columns of group g only and zeros elsewhere (read from a zeroed LDS
// slice), so lane column c accumulates the sums over group c alone for the four activation rows and applies that
// group's (scale, zero) dword; the lane columns are added at the end.
// GROUPED (mixture of experts): the workgroups with blockIdx.z = s serve slot s, up to four routed rows of one expert,
// whose packed weight, (scale, zero) table and bias come from pointer tables in device memory; an empty slot exits.
template <bool XF16, int NTW, int MAXM, bool ONE_ROUND, int GPT, bool GROUPED, int KPW = kDecodeKPW>
__global__ __launch_bounds__(1024, KPW == 2 ? 8 : 4) void woq_decode_kernel(const DecodeArgs a_in) {
  static_assert(GPT == 1 || GPT == 2 || GPT == 4, "groups of 128 x 2^k, 64 or 32");
  DecodeArgs ag;
  int64_t xr[MAXM];  // GROUPED: the rows of x that the slot's rows read
  if constexpr (GROUPED) {
    const MoeGroup& g = *a_in.grp;
    const int slot = (int)blockIdx.z;
    const int e = __builtin_amdgcn_readfirstlane(g.slot_expert[slot]);
    if (e < 0) return;  // the whole workgroup, before anything is synchronized
    const int64_t row0 = __builtin_amdgcn_readfirstlane(g.slot_row0[slot]);
    const int rows = __builtin_amdgcn_readfirstlane(g.slot_rows[slot]);
    ag = a_in;
    ag.M = rows < MAXM ? rows : MAXM;
    ag.qweight = dq_uniform((const uint8_t*)g.qweight[e]);
    ag.sz = dq_uniform((const uint32_t*)g.scales[e]);
    ag.bias = g.bias ? dq_uniform(g.bias[e]) : nullptr;
    ag.out = (uint8_t*)a_in.out + row0 * a_in.N * 2;
    if (a_in.other0) ag.other0 = (const uint8_t*)a_in.other0 + row0 * a_in.N * 2;
#pragma unroll
    for (int m = 0; m < MAXM; ++m) {
      const int64_t row = row0 + (m < (int)ag.M ? m : (int)ag.M - 1);
      xr[m] = g.x_row ? (int64_t)__builtin_amdgcn_readfirstlane((int)g.x_row[row]) : row;
    }
  }
  const DecodeArgs& a = GROUPED ? ag : a_in;
  constexpr bool G32 = GPT > 1;  // the groups of a tile are kept apart
  static_assert(!G32 || MAXM == 4, "four activation rows times up to four groups fill the 16 rows of the A operand");
  static_assert(KPW == 2 || KPW == 8, "two K tiles per wave and round, or eight in one round");
  constexpr int XL = KPW * 16 > 64 ? KPW * 16 / 64 : 1;  // 16-byte pieces of a row's slice per lane
  constexpr int SLICE = KPW * kTileK4;  // K elements of one wave per round
  constexpr int XROWS = MAXM + (G32 ? 1 : 0);  // LDS rows of a wave: its activation slices (and one of zeros)
  extern __shared__ __align__(16) uint8_t smem[];
  const int W = a.W;
  const int lane = threadIdx.x & 63;
  // the wave index is uniform: keeping it in an SGPR moves the tile / group address arithmetic to
  // the scalar unit and leaves one VGPR offset per stream
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int r = lane & 15, c = lane >> 4;
  const int64_t nt0 = (int64_t)blockIdx.x * NTW;

  uint16_t* sx = (uint16_t*)smem + (size_t)wave * XROWS * SLICE;           // private [MAXM][SLICE] (+ zeros)
  f4* red = (f4*)(smem + (size_t)W * XROWS * SLICE * sizeof(uint16_t));    // [NTW][W][16]
  if constexpr (G32) {
#pragma unroll
    for (int o = 0; o < SLICE; o += 512)
      if (o + lane * 8 < SLICE) *(u4*)(sx + MAXM * SLICE + o + lane * 8) = u4{0u, 0u, 0u, 0u};
  }

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

  const int KT = (int)a.KT, KG = (int)a.KG;
  const int tpg_shift = a.tpg_shift;  // log2(tiles per group)
  const int xlane = lane & (KPW * 16 - 1);  // lanes 32..63 mirror 0..31
  // row of the A operand -> LDS row: the activation row itself (rows past MAXM mirror row 0), or with G32 row r % 4
  // in lane column r / 4 and the zero slice in the others
  const int xrow = G32 ? ((r >> 2) < GPT && (c >> (GPT == 2 ? 1 : 0)) == (r >> 2) ? (r & 3) : MAXM) : (r < MAXM ? r : 0);
  const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc((void*)a.qweight, 0, (int)a.wbytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t srs = __builtin_amdgcn_make_buffer_rsrc((void*)a.sz, 0, (int)a.szbytes, 0x00020000);

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
    u4 xs[MAXM][XL];
    const uint8_t* xbase = (const uint8_t*)a.x + (size_t)ktw * kTileK4 * 2;  // uniform
#pragma unroll
    for (int m = 0; m < MAXM; ++m) {
      const int64_t mm = GROUPED ? xr[m] : (int64_t)(m < M ? m : M - 1);
#pragma unroll
      for (int l = 0; l < XL; ++l) xs[m][l] = *(const u4*)(xbase + (size_t)mm * K * 2 + (uint32_t)(xlane + 64 * l) * 16u);
    }

    // ---- the weight stream of this round, in the order it is consumed: one KiB tile per load,
    // all in flight together.  Buffer loads: the resource, one VGPR offset shared by every load and a
    // wave-uniform 32-bit offset in a scalar register, so the address arithmetic runs on the scalar
    // unit (decode_kernel_applies keeps weights of 4 GiB and more away) ----
    u4 wreg[NTW][KPW];
    uint32_t szreg[NTW][KPW];
    // (several groups per tile: lane column c takes the dword of group GPT kt + c % GPT, 64 bytes per group)
    const int lane16 = lane * 16, r4 = ((c & (GPT - 1)) * 16 + r) * 4;
#pragma unroll
    for (int i = 0; i < KPW; ++i) {
#pragma unroll
      for (int t = 0; t < NTW; ++t) {
        const uint32_t nt = (uint32_t)nt0 + t;
        const int woff = (int)((nt * (uint32_t)KT + (uint32_t)(ktw + i)) * (uint32_t)kTileBytes);
        const uint32_t grp = G32 ? (uint32_t)(ktw + i) * (uint32_t)GPT : (uint32_t)(ktw + i) >> tpg_shift;
        const int soff = (int)((nt * (uint32_t)KG + grp) * (uint32_t)(kTileN * sizeof(uint32_t)));
        wreg[t][i] = __builtin_amdgcn_raw_buffer_load_b128(wrs, lane16, woff, 2);  // non-temporal
        szreg[t][i] = __builtin_amdgcn_raw_buffer_load_b32(srs, r4, soff, 0);
      }
    }

    // Every load of the round stays ahead of the first use: the scheduler would otherwise sink
    // some of them below the first s_waitcnt to save registers, exposing a full memory round
    // trip in the middle of the round.
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < MAXM; ++m)
#pragma unroll
      for (int l = 0; l < XL; ++l) *(u4*)(sx + m * SLICE + (xlane + 64 * l) * 8) = xs[m][l];

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
  // several groups per tile: a lane column holds the terms of its own groups (columns without a group hold
  // zeros); they are added here
  if constexpr (G32) {
#pragma unroll
    for (int t = 0; t < NTW; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        acc[t][e] += __shfl_xor(acc[t][e], 16);
        if constexpr (GPT == 4) acc[t][e] += __shfl_xor(acc[t][e], 32);
      }
  }
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

// One row (M = 1), the single-stream decode step: the same decomposition with fewer VALU instructions
// per weight, which is what the kernel above spends its time on once the data has arrived (every wave of
// a SIMD gets its tiles at about the same time, and their decode then queues on the one VALU).
//   * the row is converted to fp16 on its way into LDS (the reference's M < 5 path computes in fp16 and
//     converts bf16 rows the same way, csrc/cpu/aten/utils/woq.h:3076-3079, 3369-3375) and the MFMA is
//     the fp16 one: the 10-bit fp16 mantissa holds a nibble in place at bits 0..3 AND at bits 4..7 --
//     0x6400 | q is 1024 + q and 0x5400 | (q << 4) is 64 + q -- so a packed dword becomes the four
//     operand dwords with one shift and four v_and_or_b32 (5 instructions instead of 7 for 8 weights);
//   * sum_k x (q - z) = sum_k x (c_k + q) - sum_k (c_k - 128) x - (128 + z) sum_k x with c_k = 1024 or 64
//     by position: the middle sum is one more MFMA per K chunk against the constants (-896, +64), whose
//     result is the C input of the weight MFMAs (no VALU instruction at all); the last is the MFMA
//     against -1 as above;
//   * every row of the A operand is the one activation row, so every row of D is the result: a lane
//     scales and accumulates one element per tile instead of four.
// GROUPED (mixture of experts): the workgroups with blockIdx.z = s serve slot s, one routed row of one expert, whose
// packed weight, (scale, zero) table and bias come from pointer tables in device memory; an empty slot exits.
// GPT = 4 or 2 groups per K tile (groups of 32 or 64 input channels): a lane column's 32 K values of a tile belong to
// one group, but an MFMA sums over the four lane columns.  The 15 spare rows of the A operand keep the groups apart:
// row m carries the activations of the lane columns of one group only -- the group of lane column m / 4 -- and zeros
// elsewhere (read from a zeroed LDS slice, no instruction more), so D[4 c][n] -- the accumulator register the kernel
// uses anyway -- is the sum over the group of lane column c alone, and that lane column applies the group's
// (scale, zero) dword; one lane column per group is added at the end.
template <bool XBF16, int NTW, int KPW, bool ONE_ROUND, bool GROUPED, int GPT>
__global__ __launch_bounds__(KPW == 4 ? 512 : 1024, KPW == 2 ? 8 : 4) void woq_decode_m1_kernel(const DecodeArgs a_in) {
  static_assert(GPT == 1 || GPT == 2 || GPT == 4, "groups of 128 x 2^k, 64 or 32");
  constexpr bool G32 = GPT > 1;       // the groups of a tile are kept apart
  constexpr int CS = GPT == 2 ? 1 : 0;  // lane columns per group, as a shift
  DecodeArgs ag;
  if constexpr (GROUPED) {
    const MoeGroup& g = *a_in.grp;
    const int slot = (int)blockIdx.z;
    const int e = __builtin_amdgcn_readfirstlane(g.slot_expert[slot]);
    if (e < 0) return;  // the whole workgroup, before anything is synchronized
    const int64_t row = __builtin_amdgcn_readfirstlane(g.slot_row0[slot]);
    const int64_t xr = g.x_row ? (int64_t)__builtin_amdgcn_readfirstlane((int)g.x_row[row]) : row;
    ag = a_in;
    ag.qweight = dq_uniform((const uint8_t*)g.qweight[e]);
    ag.sz = dq_uniform((const uint32_t*)g.scales[e]);
    ag.bias = g.bias ? dq_uniform(g.bias[e]) : nullptr;
    ag.x = a_in.x + xr * a_in.K;
    ag.out = (uint8_t*)a_in.out + row * a_in.N * 2;
    if (a_in.other0) ag.other0 = (const uint8_t*)a_in.other0 + row * a_in.N * 2;
  }
  const DecodeArgs& a = GROUPED ? ag : a_in;
  constexpr int SLICE = KPW * kTileK4;  // K elements of one wave per round
  extern __shared__ __align__(16) uint8_t smem[];
  const int W = a.W;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int r = lane & 15, c = lane >> 4;
  const int64_t nt0 = (int64_t)blockIdx.x * NTW;

  // this wave's fp16 slice of the row (G32: followed by a slice of zeros)
  uint16_t* sx = (uint16_t*)smem + (size_t)wave * SLICE * (G32 ? 2 : 1);
  float* red = (float*)(smem + (size_t)W * SLICE * (G32 ? 2 : 1) * sizeof(uint16_t));  // [NTW][16 columns][16 waves]
  if constexpr (G32) {
#pragma unroll
    for (int o = 0; o < SLICE; o += 512)
      if (o + lane * 8 < SLICE) *(u4*)(sx + SLICE + o + lane * 8) = u4{0u, 0u, 0u, 0u};
  }

  // buffer resources over the packed weight and its parameters: a load then takes the resource, one
  // VGPR offset shared by all loads, a wave-uniform offset in a scalar register and an immediate, so
  // the address arithmetic of the whole kernel runs on the scalar unit (offsets are 32 bits wide: the
  // launcher sends larger weights elsewhere); reads past the end return zero
  const __amdgpu_buffer_rsrc_t wrs = __builtin_amdgcn_make_buffer_rsrc((void*)a.qweight, 0, (int)a.wbytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t srs = __builtin_amdgcn_make_buffer_rsrc((void*)a.sz, 0, (int)a.szbytes, 0x00020000);

  uint32_t mask_lo, mask_hi, magic_a, magic_b;
  asm volatile("s_mov_b32 %0, 0x000F000F" : "=s"(mask_lo));
  asm volatile("s_mov_b32 %0, 0x00F000F0" : "=s"(mask_hi));
  asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(magic_a));
  asm volatile("v_mov_b32 %0, 0x54005400" : "=v"(magic_b));
  // One MFMA chain gives both correction sums: output columns 0..7 see the constant -1 (their D is
  // -sum x), columns 8..15 the constants -(1024 - 128), -(64 - 128) (their D is -sum (c - 128) x); a lane
  // takes the sum it does not hold from the lane eight columns over (a rotation inside its row of 16).
  const bool low_cols = r < 8;
  const u4 kcorr = low_cols ? u4{0xBC00BC00u, 0xBC00BC00u, 0xBC00BC00u, 0xBC00BC00u}
                            : u4{0xE300E300u, 0x54005400u, 0xE300E300u, 0x54005400u};

  float acc[NTW];
#pragma unroll
  for (int t = 0; t < NTW; ++t) acc[t] = 0.f;

  const int KT = (int)a.KT, KG = (int)a.KG;
  const int tpg_shift = a.tpg_shift;
  static_assert(KPW == 2 || KPW == 4 || KPW == 8, "two, four or eight K tiles per wave and round");
  constexpr int XL = KPW * 16 > 64 ? KPW * 16 / 64 : 1;  // 16-byte pieces of the slice per lane
  const int xlane = lane & (KPW * 16 - 1);  // (two tiles: lanes 32..63 mirror 0..31)
  // What the last instructions of the kernel need from the argument block, loaded with the rest of it
  // and kept in scalar registers: left to itself the compiler reads them behind the barrier, one
  // dependent scalar load after the other in the only part of the kernel that nothing overlaps.
  // (pinned behind the first round's requests, so that their own loads do not delay those)
  uint32_t out_lo = 0, out_hi = 0;
  int n_cols = 0, plain = 0;
  const int rounds = ONE_ROUND ? 1 : (KT + W * KPW - 1) / (W * KPW);
#pragma unroll 1
  for (int rd = 0; rd < rounds; ++rd) {
    const int ktw = (rd * W + wave) * KPW;
    if (!ONE_ROUND && ktw >= KT) break;

    const uint8_t* xbase = (const uint8_t*)a.x + (uint32_t)ktw * (kTileK4 * 2);  // uniform
    u4 xs[XL];
#pragma unroll
    for (int l = 0; l < XL; ++l) xs[l] = *(const u4*)(xbase + (uint32_t)(xlane + 64 * l) * 16u);

    u4 wreg[NTW][KPW];
    uint32_t szreg[NTW][KPW];
    // (several groups per tile: lane column c takes the dword of its group GPT kt + c / (4 / GPT), 64 bytes per group)
    const int lane16 = lane * 16, r4 = G32 ? ((c >> CS) * 16 + r) * 4 : r * 4;
    // requested in the order of use: K tile by K tile, row-block by row-block, each tile with its parameters
#pragma unroll
    for (int i = 0; i < KPW; ++i) {
#pragma unroll
      for (int t = 0; t < NTW; ++t) {
        const uint32_t nt = (uint32_t)nt0 + t;
        const int woff = (int)((nt * (uint32_t)KT + (uint32_t)(ktw + i)) * (uint32_t)kTileBytes);
        const uint32_t grp = G32 ? (uint32_t)(ktw + i) * (uint32_t)GPT : (uint32_t)(ktw + i) >> tpg_shift;
        const int soff = (int)((nt * (uint32_t)KG + grp) * (uint32_t)(kTileN * sizeof(uint32_t)));
        wreg[t][i] = __builtin_amdgcn_raw_buffer_load_b128(wrs, lane16, woff, 2);  // non-temporal
        szreg[t][i] = __builtin_amdgcn_raw_buffer_load_b32(srs, r4, soff, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (ONE_ROUND || rd == 0) {
      out_lo = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)a.out);
      out_hi = __builtin_amdgcn_readfirstlane((uint32_t)((uintptr_t)a.out >> 32));
      n_cols = __builtin_amdgcn_readfirstlane((int)a.N);
      plain = __builtin_amdgcn_readfirstlane(
          (int)(a.fusion == WOQ_HIP_FUSE_NONE && a.bias == nullptr && a.out_dtype == WOQ_HIP_ACT_BF16));
      asm volatile("" : "+s"(out_lo), "+s"(out_hi), "+s"(n_cols), "+s"(plain));
    }
    __builtin_amdgcn_sched_barrier(0);

#pragma unroll
    for (int l = 0; l < XL; ++l) {
      u4 xh = xs[l];
      if constexpr (XBF16) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const float lo = bitcast<float>(xs[l][v] << 16), hi = bitcast<float>(xs[l][v] & 0xFFFF0000u);
          xh[v] = bitcast<uint32_t>(__builtin_amdgcn_cvt_pkrtz(lo, hi));  // exact for every fp16-normal value
        }
      }
      *(u4*)(sx + (xlane + 64 * l) * 8) = xh;
    }

#pragma unroll
    for (int i = 0; i < KPW; ++i) {
      u4 xa[4];
      // (several groups per tile: row r of the A operand carries the lane columns of the group of lane column r / 4
      // only; the other lanes read the zero slice)
      const uint16_t* const xsrc = (!G32 || (c >> CS) == (r >> (2 + CS))) ? sx : sx + SLICE;
#pragma unroll
      for (int j = 0; j < 4; ++j) xa[j] = *(const u4*)(xsrc + i * kTileK4 + c * 32 + j * 8);
      f4 dk = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 4; ++j) dk = mfma16<true>(xa[j], kcorr, dk);
      const float mine = dk[0];
      const float theirs = bitcast<float>(__builtin_amdgcn_mov_dpp(bitcast<int>(mine), 0x128, 0xf, 0xf, true));  // row_ror:8
      const float d1 = low_cols ? mine : theirs;                    // -sum x
      const f4 dc = f4{low_cols ? theirs : mine, 0.f, 0.f, 0.f};   // -sum (c - 128) x; rows 1..3 are not used
#pragma unroll
      for (int t = 0; t < NTW; ++t) {
        f4 dw = dc;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t d = wreg[t][i][j], d8 = d >> 8;
          u4 bop;
          bop[0] = v_and_or(d, mask_lo, magic_a);
          bop[1] = v_and_or(d, mask_hi, magic_b);
          bop[2] = v_and_or(d8, mask_lo, magic_a);
          bop[3] = v_and_or(d8, mask_hi, magic_b);
          dw = mfma16<true>(xa[j], bop, dw);
        }
        // dw = sum x (c + q) - sum (c - 128) x, d1 = -sum x;  group term = s * (dw + (128 + z) * d1)
        const float tsum = fma_f16hi(d1, szreg[t][i], dw[0]);
        acc[t] = fma_f16lo(tsum, szreg[t][i], acc[t]);
      }
    }
  }

  // the partial sums of waves that do not exist read as zero
  if (W < 16 && threadIdx.x < NTW * 16) {
    for (int w = W; w < 16; ++w) red[threadIdx.x * 16 + w] = 0.f;
  }
  // several groups per tile: a lane column holds the terms of its own group (with two groups, lane columns c and
  // c + 1 the same ones); one lane column per group is added here
  if constexpr (G32) {
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
      if constexpr (GPT == 4) acc[t] += __shfl_xor(acc[t], 16);
      acc[t] += __shfl_xor(acc[t], 32);
    }
  }
  // every lane column holds the same sums; column 0 publishes them
  if (c == 0) {
#pragma unroll
    for (int t = 0; t < NTW; ++t) red[(t * 16 + r) * 16 + wave] = acc[t];
  }
  __syncthreads();

  if (threadIdx.x < NTW * 16) {
    const int col = threadIdx.x & 15, t = threadIdx.x >> 4;
    const int n = ((int)nt0 + t) * kTileN + col;
    // the 16 partial sums of this output in four reads, added pairwise in a fixed order
    const f4* mine = (const f4*)(red + threadIdx.x * 16);
    const f4 p0 = mine[0], p1 = mine[1], p2 = mine[2], p3 = mine[3];
    const float s = (((p0[0] + p0[1]) + (p0[2] + p0[3])) + ((p1[0] + p1[1]) + (p1[2] + p1[3]))) +
                    (((p2[0] + p2[1]) + (p2[2] + p2[3])) + ((p3[0] + p3[1]) + (p3[2] + p3[3])));
    if (n < n_cols) {
      if (plain) {
        typedef __attribute__((address_space(1))) uint16_t* global_u16_ptr;  // a global store, not a flat one
        global_u16_ptr out = (global_u16_ptr)(((uintptr_t)out_hi << 32) | out_lo);
        out[n] = f32_to_bf16_bits((float)(_Float16)s);
      } else {
        Epilogue ep{a.bias, a.fusion, a.other0, a.other1, a.out, a.out_dtype, a.x_dtype, a.N};
        epilogue_store<kRegimeF16>(ep, 0, n, s);
      }
    }
  }
}

template <bool XBF16, int NTW, int KPW, bool ONE_ROUND>
static int launch_decode_m1_cfg(const DecodeArgs& a, hipStream_t st, int slots = 0) {
  const bool apart = a.G == 32 || a.G == 64;  // several groups per K tile
  const size_t smem = (size_t)NTW * 16 * 16 * sizeof(float) + (size_t)a.W * KPW * kTileK4 * sizeof(uint16_t) * (apart ? 2 : 1);
  const unsigned grid = (unsigned)((a.NT + NTW - 1) / NTW);
  const dim3 ggrid(grid, 1, (unsigned)(slots > 0 ? slots : 1));
  if (slots > 0 && a.G == 32)
    woq_decode_m1_kernel<XBF16, NTW, KPW, ONE_ROUND, true, 4><<<ggrid, a.W * 64, smem, st>>>(a);
  else if (slots > 0 && a.G == 64)
    woq_decode_m1_kernel<XBF16, NTW, KPW, ONE_ROUND, true, 2><<<ggrid, a.W * 64, smem, st>>>(a);
  else if (slots > 0)
    woq_decode_m1_kernel<XBF16, NTW, KPW, ONE_ROUND, true, 1><<<ggrid, a.W * 64, smem, st>>>(a);
  else if (a.G == 32)
    woq_decode_m1_kernel<XBF16, NTW, KPW, ONE_ROUND, false, 4><<<grid, a.W * 64, smem, st>>>(a);
  else if (a.G == 64)
    woq_decode_m1_kernel<XBF16, NTW, KPW, ONE_ROUND, false, 2><<<grid, a.W * 64, smem, st>>>(a);
  else
    woq_decode_m1_kernel<XBF16, NTW, KPW, ONE_ROUND, false, 1><<<grid, a.W * 64, smem, st>>>(a);
  return check_launch("woq_decode_m1_kernel");
}

template <bool XF16, int NTW, int MAXM, bool ONE_ROUND, int GPT, bool GROUPED, int KPW = kDecodeKPW>
static int launch_decode_cfg_g(const DecodeArgs& a, hipStream_t st, int slots) {
  const size_t smem = (size_t)NTW * a.W * 16 * sizeof(f4) +
                      (size_t)a.W * (MAXM + (GPT > 1 ? 1 : 0)) * KPW * kTileK4 * sizeof(uint16_t);
  auto kern = woq_decode_kernel<XF16, NTW, MAXM, ONE_ROUND, GPT, GROUPED, KPW>;
  if (smem > 64 * 1024) {
    hipError_t err = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (err != hipSuccess) return set_error("hipFuncSetAttribute: %s", hipGetErrorString(err));
  }
  const dim3 grid((unsigned)((a.NT + NTW - 1) / NTW), 1, (unsigned)(GROUPED ? slots : 1));
  kern<<<grid, a.W * 64, smem, st>>>(a);
  return check_launch("woq_decode_kernel");
}

template <bool XF16, int NTW, int MAXM, bool ONE_ROUND>
static int launch_decode_cfg(const DecodeArgs& a, hipStream_t st, int slots = 0) {
  if (slots > 0)
    return a.G == 32   ? launch_decode_cfg_g<XF16, NTW, MAXM, ONE_ROUND, 4, true>(a, st, slots)
           : a.G == 64 ? launch_decode_cfg_g<XF16, NTW, MAXM, ONE_ROUND, 2, true>(a, st, slots)
                       : launch_decode_cfg_g<XF16, NTW, MAXM, ONE_ROUND, 1, true>(a, st, slots);
  return a.G == 32   ? launch_decode_cfg_g<XF16, NTW, MAXM, ONE_ROUND, 4, false>(a, st, 0)
         : a.G == 64 ? launch_decode_cfg_g<XF16, NTW, MAXM, ONE_ROUND, 2, false>(a, st, 0)
                     : launch_decode_cfg_g<XF16, NTW, MAXM, ONE_ROUND, 1, false>(a, st, 0);
}

bool decode_kernel_applies(const FpArgs& f, int wbits, int regime, const uint32_t* sz) {
  const int64_t tpg = f.G / kTileK4;
  // the kernels address the packed weight and its parameters with 32-bit offsets
  if (f.NT * f.KT * kTileBytes >= ((int64_t)1 << 32) || f.NT * f.KG * kTileN * 4 >= ((int64_t)1 << 32)) return false;
  // groups of 128 x 2^k, of 64 or of 32
  const bool groups = ((f.G % kTileK4) == 0 && (tpg & (tpg - 1)) == 0) || f.G == 32 || f.G == 64;
  return sz != nullptr && wbits == 4 && regime == kRegimeF16 && f.M <= 4 && groups &&
         (f.K % (kDecodeKPW * kTileK4)) == 0 && (f.x_dtype == WOQ_HIP_ACT_BF16 || f.x_dtype == WOQ_HIP_ACT_FP16);
}

static int launch_decode_impl(const FpArgs& f, const uint32_t* sz, hipStream_t st, const MoeGroup* grp, int slots);

int launch_decode(const FpArgs& f, const uint32_t* sz, hipStream_t st) { return launch_decode_impl(f, sz, st, nullptr, 0); }

int launch_decode_grouped(const FpArgs& f, const MoeGroup* grp, int64_t slots, hipStream_t st) {
  if (!grp || slots < 1 || slots > 65535) return set_error("woq_linear_grouped: 1..65535 slots and a group table");
  if (f.M < 1 || f.M > 4) return set_error("woq_linear_grouped: the integer-weight decode kernels take up to four rows per slot");
  return launch_decode_impl(f, nullptr, st, grp, (int)slots);
}

static int launch_decode_impl(const FpArgs& f, const uint32_t* sz, hipStream_t st, const MoeGroup* grp, int slots) {
  DecodeArgs a;
  a.grp = grp;
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
  // Two row-blocks per workgroup from 512 row-blocks on; a single row only above 768: up to there one
  // row-block per workgroup spreads more evenly over the 256 CUs (M = 1: 8192 -> 10240 9.6 us against
  // 11.7 us, 4096 -> 8192 5.2 against 5.4 us, 4096 -> 11008 6.5 against 6.7 us; 4096 -> 14336 the other
  // way round, 7.1 against 7.8 us; M = 4, 4096 -> 11008: 7.4 us with two against 7.7 us).
  const bool two = f.NT % 2 == 0 && (f.M == 1 ? f.NT > 768 : f.NT >= 512);
  a.wbytes = (uint32_t)(f.NT * f.KT * kTileBytes);  // below 4 GiB (decode_kernel_applies)
  a.szbytes = (uint32_t)(f.NT * f.KG * kTileN * (int64_t)sizeof(uint32_t));
  const bool one_row = f.M == 1;
  const bool one_round = f.KT == (int64_t)a.W * kDecodeKPW;
  if (one_row && !one_round && f.KT % 8 == 0 && f.KT / 8 <= 16 && f.G != 32 && f.G != 64) {
    // A long K in one round: eight K tiles per wave (8 KiB in flight per wave, a budget of 128 registers) instead of
    // several rounds of two, each of which waits for its own requests (M = 1, 14336 -> 4096: 7.48 against 7.71 us,
    // 8192 -> 8192 8.04 against 8.39 us; with groups of 32 the larger zeroed slice makes it a loss, 8.6 against 8.2 us).
    a.W = (int)(f.KT / 8);
    if (xf16) return two ? launch_decode_m1_cfg<false, 2, 8, true>(a, st, slots) : launch_decode_m1_cfg<false, 1, 8, true>(a, st, slots);
    return two ? launch_decode_m1_cfg<true, 2, 8, true>(a, st, slots) : launch_decode_m1_cfg<true, 1, 8, true>(a, st, slots);
  }
  if (one_row) {
    // Four K tiles per wave (half the waves, each with twice the bytes in flight) where two tiles per
    // wave would leave at most two waves per SIMD anyway: the per-wave overhead then weighs more than
    // the occupancy (M = 1, 2048 -> 8192: 3.8 us against 4.6 us; 4096 -> 14336, seven waves per SIMD:
    // 7.4 us against 7.1 us the other way round).
    const int64_t waves2 = (f.NT / (two ? 2 : 1)) * ((f.KT + 1) / 2);
    if (waves2 <= 2048 && f.KT % 4 == 0 && f.KT / 4 <= 8) {
      a.W = (int)(f.KT / 4);
      if (xf16) return two ? launch_decode_m1_cfg<false, 2, 4, true>(a, st, slots) : launch_decode_m1_cfg<false, 1, 4, true>(a, st, slots);
      return two ? launch_decode_m1_cfg<true, 2, 4, true>(a, st, slots) : launch_decode_m1_cfg<true, 1, 4, true>(a, st, slots);
    }
#define WOQ_DECODE_M1(XB, NTW) \
  (one_round ? launch_decode_m1_cfg<XB, NTW, 2, true>(a, st, slots) : launch_decode_m1_cfg<XB, NTW, 2, false>(a, st, slots))
    if (xf16) return two ? WOQ_DECODE_M1(false, 2) : WOQ_DECODE_M1(false, 1);
    return two ? WOQ_DECODE_M1(true, 2) : WOQ_DECODE_M1(true, 1);
#undef WOQ_DECODE_M1
  }
  if (!one_round && f.KT % 8 == 0 && f.KT / 8 <= 16 && f.G != 32 && f.G != 64 && !two) {
    // a long K in one round of eight K tiles per wave, as for one row above (M = 4, 14336 -> 4096: 8.9 against 9.2 us)
    a.W = (int)(f.KT / 8);
    if (slots > 0)
      return xf16 ? launch_decode_cfg_g<true, 1, 4, true, 1, true, 8>(a, st, slots)
                  : launch_decode_cfg_g<false, 1, 4, true, 1, true, 8>(a, st, slots);
    return xf16 ? launch_decode_cfg_g<true, 1, 4, true, 1, false, 8>(a, st, 0)
                : launch_decode_cfg_g<false, 1, 4, true, 1, false, 8>(a, st, 0);
  }
#define WOQ_DECODE(XF, NTW) \
  (one_round ? launch_decode_cfg<XF, NTW, 4, true>(a, st, slots) : launch_decode_cfg<XF, NTW, 4, false>(a, st, slots))
  if (xf16) return two ? WOQ_DECODE(true, 2) : WOQ_DECODE(true, 1);
  return two ? WOQ_DECODE(false, 2) : WOQ_DECODE(false, 1);
#undef WOQ_DECODE
}

}  // namespace woq

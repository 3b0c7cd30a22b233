// Decode kernel with per-weight dequantization: 4- or 8-bit weights, M <= 64, HBM-bound weight
// streaming.
//
// Reference counterpart: the M >= 5 path of lowp_mode BF16 -- Dequantize<bfloat16> into a bf16
// block, then a bf16 x bf16 -> fp32 BRGEMM (csrc/cpu/aten/utils/woq.h:1495-1581, 1847-1944) -- at
// the batch sizes of a decode step.  Each weight becomes w = bf16((q - z) * s) with the scale read
// as bf16 (fp16 regime: w = fp16((q - z) * s)), exactly as there; the products accumulate in fp32.
//
// Same decomposition as the integer-weight decode kernel: a workgroup owns NTW weight row-blocks
// (16 output columns each) and all of K, its W <= 8 waves take one K tile each per round, the
// partial sums meet in LDS and are added in wave order.  v_mfma_f32_16x16x32 with A = activations
// (row m = lane % 16) and B = weights (column n = lane % 16): the dequantized registers of one
// packed dword are the B operand.
// The dequantization is ~17 VALU instructions per packed dword, about as much time chip-wide as
// the weight stream itself, so the rounds are software pipelined: the requests of round r + 1
// (tiles and parameters into registers, activations into the other LDS buffer) are issued before
// round r is computed.
// Activations: a wave copies the rows of its K tile (16, 32 or 64 rows x 256 bytes for 4-bit weights,
// x 128 bytes for 8-bit ones) straight into its private slice of LDS (global_load_lds_dwordx4:
// fully coalesced, no registers) and reads the operand fragments from there; chunk p of row m sits
// at p ^ m (p ^ swz_row128(m) for the 128-byte rows) so the fragment reads are conflict-free.  Reading
// the fragments from global memory directly costs the same number of instructions but each one
// gathers 64 separate 16-byte pieces, which made the texture addresser the bottleneck (M = 16:
// 19.7 us against 13.9 us at M = 8 for the same weights).  Rows past M re-read row M - 1 and their
// results are dropped.  The at most 64 KiB of slices (up to 32 rows; 128 KiB and four waves for
// 33..64 rows) are reused for the cross-wave sum; up to 32 rows two workgroups fit on a CU.
// Split K: every workgroup streams the activations of all the K tiles it owns, so a layer with few
// output columns (few row-blocks, hence one row-block per workgroup to fill the chip) reads the
// activations once per 16 columns -- M = 32, 14336 -> 4096: 235 MB through LDS against 29 MB of
// weights.  With gridDim.y = S > 1 a workgroup owns more row-blocks and 1 / S of the K tiles; it
// writes its fp32 partial tile to scratch memory, and the workgroup that arrives last at the
// row-block set's counter (no workgroup ever waits) adds the S partial tiles in split order and runs
// the epilogue.  The sum order is fixed, so the result does not depend on the arrival order.
#include <type_traits>

#include "woq_common.h"
#include "woq_internal.h"

namespace woq {

constexpr int kDqMaxWaves = 8;

struct DecodeDqArgs {
  FpArgs f;
  int W;        // waves per workgroup
  int g_shift;  // log2(group size); 30 for per-channel
  int KTs;      // K tiles per workgroup row (gridDim.y workgroups share the K tiles of a row-block set)
  float* partial;  // split K: [gridDim.y][gridDim.x] fp32 partial tiles
  int* counters;   // split K: [gridDim.x], zero between launches
  // GROUPED instances (mixture of experts): the workgroups with blockIdx.z = s serve slot s, whose expert, first
  // routed row and row count they read from device memory; the expert's tensors come from pointer tables.
  const MoeGroup* grp;
};



template <int REGIME>
__device__ __forceinline__ f4 dq_mfma(u4 a, u4 b, f4 c) {
  if constexpr (REGIME == kRegimeF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(bitcast<h8>(a), bitcast<h8>(b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(bitcast<b8>(a), bitcast<b8>(b), c, 0, 0, 0);
}

typedef __attribute__((address_space(3))) void* dq_lds_ptr_t;
typedef const __attribute__((address_space(1))) void* dq_global_ptr_t;

// Geometry of one K tile (1 KiB of packed weights: 16 rows x 128 int4 or x 64 int8) and of the
// activation slice that goes with it.
template <int WBITS, int MT>
struct DqGeom {
  static constexpr int TK = WBITS == 4 ? kTileK4 : kTileK8;
  static constexpr int ROWB = TK * 2;             // bytes of one activation row of the tile
  static constexpr int LPR = ROWB / 16;           // lanes (16-byte chunks) per row
  static constexpr int RPI = 64 / LPR;            // rows per LDS-load instruction
  static constexpr int SLICE = MT * 16 * ROWB;    // one buffer of one wave
  static constexpr int NX = SLICE / 1024;         // LDS-load instructions per buffer
  static constexpr int NJ = TK / 32;              // MFMAs (32 K values each) per tile
  static __device__ __forceinline__ int swz(int row) { return WBITS == 4 ? (row & 15) : swz_row128(row); }
};

// 8-bit weights: per-lane scale and offset of one row, c = -(128 + z) * s for the offset-binary
// bytes (symmetric: z = 0).
struct G8Consts {
  float s, c;
};

// NF4: the 4-bit codes index the NormalFloat4 table (a copy in LDS) and there are no zero points.
// XCONV (fp16 regime, one row tile): the activations are bf16 and become fp16 on the way in, as the
// reference's fp16 kernel converts them per K block (csrc/cpu/aten/utils/woq.h:3076-3079) -- the common
// case of a bf16 model under lowp_mode BF16 with fewer than five rows.  The rows then travel through
// registers (16-byte loads, conversion, ds_write to the same swizzled places) instead of the LDS DMA.
// Constants of one (row, group) from its merged dword, bf16 scale << 16 | an fp16 number: 4-bit weights
// w = (1024 + q) * s + c = (64 + q) * s + c64 with the fp16 number 1024 + z (a nibble is read as 1024 + q, or as
// 64 + q in place at bits 4..7); 8-bit weights w = u * s + c with the fp16 number the stored zero byte.  All exact
// in fp32, so the one rounding is the conversion to bf16, as with separate scale and zero point.
struct DqConstsM {
  float s, c, c64;
  template <int WBITS>
  __device__ __forceinline__ void set(uint32_t pd) {
    s = bitcast<float>(pd & 0xFFFF0000u);
    const _Float16 h = bitcast<_Float16>((uint16_t)(pd & 0xFFFFu));
    c = -((float)h * s);
    if constexpr (WBITS == 4) c64 = __builtin_fmaf(960.0f, s, c);
  }
};
__device__ __forceinline__ u4 dq_dequant_m(uint32_t d, const G4Masks& k, uint32_t magic64, const DqConstsM& q) {
  u4 r;
  const f2 f0 = g4_fma_pair((d & k.lo) | k.magic, q.s, q.c);
  const f2 f1 = g4_fma_pair((d & k.hi) | magic64, q.s, q.c64);
  r[0] = g4_cvt_pair(f0);
  const uint32_t d8 = d >> 8;
  const f2 f2_ = g4_fma_pair((d8 & k.lo) | k.magic, q.s, q.c);
  r[1] = g4_cvt_pair(f1);
  const f2 f3 = g4_fma_pair((d8 & k.hi) | magic64, q.s, q.c64);
  r[2] = g4_cvt_pair(f2_);
  r[3] = g4_cvt_pair(f3);
  return r;
}

// SZB (bf16 compute, integer weights, not GROUPED): scale and zero point of a (row, group) come as one dword
// (f.szb): one request and three vector instructions per row-block and round instead of two and eight.
template <int REGIME, int WBITS, int MT, int NTW, bool NF4, bool XCONV, bool FP8, bool GROUPED, bool SZB = false>
__global__ __launch_bounds__(512, (MT * NTW > 8 ? 2 : 4)) void woq_decode_dq_kernel(const DecodeDqArgs a) {
  static_assert(!XCONV || (REGIME == kRegimeF16 && MT == 1), "bf16 -> fp16 rows: fp16 regime, one row tile");
  static_assert(!SZB || (REGIME == kRegimeBF16 && !NF4 && !FP8 && !GROUPED), "merged parameters: bf16 compute, integer weights");
  using Geo = DqGeom<WBITS, MT>;
  constexpr int TK = Geo::TK, NJ = Geo::NJ, NX = Geo::NX, SLICE = Geo::SLICE;
  static_assert(!NF4 || WBITS == 4, "NF4 codes are 4 bits wide");
  static_assert(!FP8 || WBITS == 8, "float8 weights are bytes");
  extern __shared__ __align__(1024) uint8_t smem[];
  __shared__ f2 sNf4[NF4 ? kNf4LutEntries : 1];
  if constexpr (NF4) {
    nf4_fill_lut(sNf4, (int)threadIdx.x, (int)blockDim.x);
    __syncthreads();
  }
  FpArgs fg;                      // GROUPED: this slot's problem
  const int64_t* xrow = nullptr;  // GROUPED: routed row -> row of x, from xrow0 on
  int64_t xrow0 = 0;
  if constexpr (GROUPED) {
    // every workgroup of a slot takes the same path, and nothing has been synchronized yet
    const MoeGroup& g = *a.grp;
    const int slot = (int)blockIdx.z;
    const int e = __builtin_amdgcn_readfirstlane(g.slot_expert[slot]);
    if (e < 0) return;
    const int64_t row0 = __builtin_amdgcn_readfirstlane(g.slot_row0[slot]);
    const int rows = __builtin_amdgcn_readfirstlane(g.slot_rows[slot]);
    fg = a.f;
    fg.M = rows < (int)fg.M ? rows : fg.M;
    fg.qweight = dq_uniform((const uint8_t*)g.qweight[e]);
    fg.scales = dq_uniform((const uint16_t*)g.scales[e]);
    fg.zeros = g.zeros ? dq_uniform(g.zeros[e]) : nullptr;
    fg.bias = g.bias ? dq_uniform(g.bias[e]) : nullptr;
    const int64_t out_elt = fg.out_dtype == WOQ_HIP_ACT_FP32 ? 4 : 2, x_elt = 2;  // rows are 16-bit here
    fg.out = (uint8_t*)fg.out + row0 * fg.N * out_elt;
    if (fg.other0) fg.other0 = (const uint8_t*)fg.other0 + row0 * fg.N * x_elt;
    if (fg.other1) fg.other1 = (const uint8_t*)fg.other1 + row0 * fg.N * x_elt;
    if (g.x_row) {
      xrow = g.x_row;
      xrow0 = row0;
    } else {
      fg.x = (const uint8_t*)fg.x + row0 * fg.K * x_elt;
    }
  }
  const FpArgs& f = GROUPED ? fg : a.f;
  const int W = a.W;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int r = lane & 15, c = lane >> 4;
  const int M = (int)f.M, K = (int)f.K, KT = (int)f.KT, KG = (int)f.KG;
  const int64_t nt0 = (int64_t)blockIdx.x * NTW;
  uint8_t* const sx = smem + wave * (2 * SLICE);  // this wave's two activation buffers
  f4* const red = (f4*)smem;                      // [NTW * MT][W][64], after the K loop

  G4Masks km;
  asm volatile("s_mov_b32 %0, 0x000F000F" : "=s"(km.lo));
  asm volatile("s_mov_b32 %0, 0x00F000F0" : "=s"(km.hi));
  asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(km.magic));
  uint32_t magic64 = 0;  // fp16 64 twice
  if constexpr (SZB && WBITS == 4) asm volatile("v_mov_b32 %0, 0x54005400" : "=v"(magic64));

  f4 acc[NTW][MT];
#pragma unroll
  for (int t = 0; t < NTW; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f4{0.f, 0.f, 0.f, 0.f};

  // wave-uniform bases + one 32-bit per-lane offset per stream.
  // Activation load i fills LDS bytes [1024 i, +1024) of a buffer: rows RPI * i + lane / LPR,
  // physical chunk lane % LPR = logical chunk ^ swz(row).
  uint32_t xoff[NX];
#pragma unroll
  for (int i = 0; i < NX; ++i) {
    const int row = Geo::RPI * i + lane / Geo::LPR;
    int rowc = row < M ? row : M - 1;
    if constexpr (GROUPED) {
      if (xrow) rowc = (int)xrow[xrow0 + rowc];  // (the host bounds rows of x * K * 2 below 2^31)
    }
    const int chunk = ((lane % Geo::LPR) ^ Geo::swz(row)) & (Geo::LPR - 1);
    xoff[i] = (uint32_t)(rowc * K + chunk * 8) * 2u;
  }
  uint32_t rdo[NJ];  // fragment j of this lane in row tile 0: row r, logical chunk NJ c + j
#pragma unroll
  for (int j = 0; j < NJ; ++j) rdo[j] = (uint32_t)(r * Geo::ROWB + (((c * NJ + j) ^ Geo::swz(r)) << 4));
  const uint32_t woff = (uint32_t)lane * 16u;
  const bool has_z = f.zeros != nullptr;
  const uint8_t* wbase[NTW];
  const uint8_t* sbase[NTW];
  const uint8_t* zbase[NTW];
#pragma unroll
  for (int t = 0; t < NTW; ++t) {
    // the row-blocks per workgroup need not divide the row-blocks: the last workgroup reads its
    // missing ones from the last real row-block, and the store below drops their columns (n >= N)
    const int64_t nt = nt0 + t < f.NT ? nt0 + t : f.NT - 1;
    wbase[t] = f.qweight + (size_t)nt * KT * kTileBytes;
    if constexpr (SZB) {
      sbase[t] = (const uint8_t*)f.szb + (size_t)nt * KG * (kTileN * 4);
      zbase[t] = sbase[t];
    } else {
      sbase[t] = (const uint8_t*)(f.scales + (size_t)nt * KG * kTileN);
      zbase[t] = has_z ? f.zeros + (size_t)nt * KG * kTileN : sbase[t];
    }
  }

  // Two register sets for the tiles and parameters in flight: round i computes from set i % 2 while the
  // requests of round i + 1 fill the other, so nothing is copied between rounds.
  u4 wq[2][NTW];
  uint16_t sq[2][SZB ? 1 : NTW];
  uint8_t zq[2][SZB ? 1 : NTW];
  uint32_t mq[2][SZB ? NTW : 1];
  u4 xnext[XCONV ? NX : 1];  // XCONV: the next round's activation rows, still bf16
  // every request of one round: activations into LDS buffer `buf`, tiles and parameters into register set `buf`
  auto request = [&](int kt, auto bufc) {
    constexpr int buf = decltype(bufc)::value;
    // uniform base + 32-bit offset; instructions whose rows lie entirely past M are skipped
    // (their LDS bytes stay undefined: an MFMA output row depends on its own A row only)
    const uint32_t ko = (uint32_t)kt * Geo::ROWB;
#pragma unroll
    for (int i = 0; i < NX; ++i)
      if (Geo::RPI * i < M) {
        if constexpr (XCONV)
          xnext[i] = *(const u4*)((const uint8_t*)f.x + (uint32_t)(xoff[i] + ko));
        else
          __builtin_amdgcn_global_load_lds((dq_global_ptr_t)((const uint8_t*)f.x + (uint32_t)(xoff[i] + ko)),
                                           (dq_lds_ptr_t)(sx + buf * SLICE + i * 1024), 16, 0, 0);
      }
    int g = (kt * TK + c * (TK / 4)) >> a.g_shift;
    g = g < KG ? g : KG - 1;
    const uint32_t qoff = (uint32_t)(g * kTileN + r);
    const uint32_t wo = (uint32_t)kt * kTileBytes + woff;
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
      wq[buf][t] = __builtin_nontemporal_load((const u4*)(wbase[t] + wo));
      if constexpr (SZB) {
        mq[buf][t] = *(const uint32_t*)(sbase[t] + (uint32_t)(qoff * 4u));
      } else {
        sq[buf][t] = *(const uint16_t*)(sbase[t] + (uint32_t)(qoff * 2u));
        zq[buf][t] = *(zbase[t] + qoff);  // raw: any use here would wait for the load inside the request
      }
    }
  };

  // Rounds: wave w takes K tiles kt0 + w, kt0 + w + W, ... of this workgroup's range [kt0, kt1); a
  // wave with no tile left idles until the sum.
  const int kt0 = (int)blockIdx.y * a.KTs;
  const int kt1 = kt0 + a.KTs < KT ? kt0 + a.KTs : KT;
  using Buf0 = std::integral_constant<int, 0>;
  using Buf1 = std::integral_constant<int, 1>;
  if (kt0 + wave < kt1) request(kt0 + wave, Buf0{});
  // one round: K tile kt from register set and LDS buffer `buf`
  auto round = [&](const int kt, auto bufc) {
    constexpr int buf = decltype(bufc)::value;
    const u4 (&wreg)[NTW] = wq[buf];
    G4Consts<REGIME> qc4[WBITS == 4 && !SZB ? NTW : 1];
    G8Consts qc8[WBITS == 8 || NF4 ? NTW : 1];
    DqConstsM qm[SZB ? NTW : 1];
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
      if constexpr (SZB) {
        qm[t].template set<WBITS>(mq[buf][t]);
        if constexpr (WBITS == 8) {
          qc8[t].s = qm[t].s;
          qc8[t].c = qm[t].c;
        }
      } else if constexpr (NF4) {
        qc8[t].s = REGIME == kRegimeF16 ? f16_bits_to_f32(sq[buf][t]) : bf16_bits_to_f32(sq[buf][t]);
      } else if constexpr (WBITS == 4) {
        qc4[t].set(sq[buf][t], has_z ? (float)zq[buf][t] : 8.0f);
      } else {
        qc8[t].s = REGIME == kRegimeF16 ? f16_bits_to_f32(sq[buf][t]) : bf16_bits_to_f32(sq[buf][t]);
        qc8[t].c = -((has_z ? (float)zq[buf][t] : 128.0f) * qc8[t].s);
      }
    }
    // The compiler does not order LDS reads after the LDS-writing loads: wait for them here.
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    if constexpr (XCONV) {
      // bf16 -> fp16 (exact inside the fp16 range, round to nearest even below it) into this wave's
      // slice; a wave's LDS accesses complete in order, so the fragment reads below see the rows
#pragma unroll
      for (int i = 0; i < NX; ++i)
        if (Geo::RPI * i < M) {
          u4 h;
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const float lo = bitcast<float>(xnext[i][v] << 16), hi = bitcast<float>(xnext[i][v] & 0xFFFF0000u);
            h[v] = (uint32_t)f32_to_f16_bits(lo) | ((uint32_t)f32_to_f16_bits(hi) << 16);
          }
          *(u4*)(sx + buf * SLICE + i * 1024 + lane * 16) = h;
        }
    }
    if (kt + W < kt1) request(kt + W, std::integral_constant<int, buf ^ 1>{});
    __builtin_amdgcn_sched_barrier(0);

#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      u4 xa[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) xa[mt] = *(const u4*)(sx + buf * SLICE + mt * 16 * Geo::ROWB + rdo[j]);
#pragma unroll
      for (int t = 0; t < NTW; ++t) {
        u4 bop;
        if constexpr (NF4) {
          bop = nf4_dequant<REGIME>(wreg[t][j], sNf4, qc8[t].s);
        } else if constexpr (WBITS == 4 && SZB) {
          bop = dq_dequant_m(wreg[t][j], km, magic64, qm[t]);
        } else if constexpr (WBITS == 4) {
          bop = g4_dequant(wreg[t][j], km, qc4[t]);
        } else if constexpr (FP8) {
          if constexpr (REGIME == kRegimeF16)
            bop = bitcast<u4>(dequant8_f16_fp8(wreg[t][2 * j], wreg[t][2 * j + 1], qc8[t].s));
          else
            bop = bitcast<u4>(dequant8_bf16_fp8(wreg[t][2 * j], wreg[t][2 * j + 1], qc8[t].s));
        } else if constexpr (REGIME == kRegimeF16) {
          bop = bitcast<u4>(dequant8_f16_w8(wreg[t][2 * j], wreg[t][2 * j + 1], qc8[t].s, qc8[t].c));
        } else {
          bop = bitcast<u4>(dequant8_bf16_w8(wreg[t][2 * j], wreg[t][2 * j + 1], qc8[t].s, qc8[t].c));
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[t][mt] = dq_mfma<REGIME>(xa[mt], bop, acc[t][mt]);
      }
    }
  };
#pragma unroll 1
  for (int kt = kt0 + wave; kt < kt1; kt += 2 * W) {
    round(kt, Buf0{});
    if (kt + W < kt1) round(kt + W, Buf1{});
  }

  // ---- combine the waves' partial sums in wave order, then bias / rounding / store ----
  __syncthreads();  // every wave is done with its activation slices: the region becomes `red`
#pragma unroll
  for (int t = 0; t < NTW; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[((t * MT + mt) * W + wave) * 64 + lane] = acc[t][mt];
  __syncthreads();

  Epilogue ep{f.bias, f.fusion, f.other0, f.other1, f.out, f.out_dtype, f.x_dtype, f.N};
  const float* redf = (const float*)red;
  const bool plain = REGIME == kRegimeBF16 && f.fusion == WOQ_HIP_FUSE_NONE && f.bias == nullptr &&
                     f.out_dtype == WOQ_HIP_ACT_BF16;
  // one thread per output element, consecutive threads on consecutive columns; D[m][n] of a row
  // tile sits in lane n + 16 (m / 4), register m % 4
  constexpr int kTileElems = NTW * MT * 256;
  auto wave_sum = [&](int idx) {
    const int col = idx & 15, m16 = (idx >> 4) & 15, tm = idx >> 8;
    const int slot = (col + 16 * (m16 >> 2)) * 4 + (m16 & 3);
    float part[kDqMaxWaves];
#pragma unroll
    for (int w = 0; w < kDqMaxWaves; ++w) part[w] = w < W ? redf[(tm * W + w) * 256 + slot] : 0.0f;
    float s = part[0];
#pragma unroll
    for (int w = 1; w < kDqMaxWaves; ++w) s += part[w];
    return s;
  };
  auto store = [&](int idx, float s) {
    const int col = idx & 15, m16 = (idx >> 4) & 15, tm = idx >> 8;
    const int t = tm / MT, mt = tm - t * MT;
    const int m = mt * 16 + m16;
    const int64_t n = (nt0 + t) * kTileN + col;
    if (m >= M || n >= f.N) return;
    if (plain)
      ((uint16_t*)f.out)[(int64_t)m * f.N + n] = f32_to_bf16_bits(s);
    else
      epilogue_store<REGIME>(ep, m, n, s);
  };
  const int S = (int)gridDim.y;
  if (S == 1) {
    for (int idx = threadIdx.x; idx < kTileElems; idx += blockDim.x) store(idx, wave_sum(idx));
    return;
  }
  // ---- split K: partial tile to scratch, then the last workgroup of this row-block set sums ----
  // Every access to the scratch is a relaxed atomic at device scope: such stores write through to
  // the point where the other XCDs see them and such loads do not hit a stale cache line, so no
  // cache-wide write-back or invalidation (what a device-scope fence costs) is needed.  Order: a
  // thread's stores have completed at its vmcnt(0), the barrier collects all threads, then thread 0
  // moves the counter; the last workgroup reads only after it has seen the final count.
  float* const mine = a.partial + ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * kTileElems;
  for (int idx = threadIdx.x; idx < kTileElems; idx += blockDim.x)
    __hip_atomic_store(mine + idx, wave_sum(idx), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  __syncthreads();
  __shared__ int s_last;
  if (threadIdx.x == 0)
    s_last = __hip_atomic_fetch_add(a.counters + blockIdx.x, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == S - 1;
  __syncthreads();
  if (!s_last) return;
  const float* const all = a.partial + (size_t)blockIdx.x * kTileElems;
  for (int idx = threadIdx.x; idx < kTileElems; idx += blockDim.x) {
    float s = __hip_atomic_load(all + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (int k = 1; k < S; ++k)
      s += __hip_atomic_load(all + (size_t)k * gridDim.x * kTileElems + idx, __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
    store(idx, s);
  }
  // the counter is back at zero for the next launch that uses it
  if (threadIdx.x == 0) __hip_atomic_store(a.counters + blockIdx.x, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int REGIME, int WBITS, int MT, int NTW, bool NF4, bool XCONV, bool FP8, bool GROUPED, bool SZB>
static int launch_dq_cfg_impl(DecodeDqArgs a, int splits, hipStream_t st, int slots) {
  using Geo = DqGeom<WBITS, MT>;
  if (MT > 2 && splits > 1) return set_error("woq_decode_dq_kernel: split K takes at most 32 rows");
  // At most 64 KiB of activation buffers per workgroup, so that two workgroups share a CU -- unless
  // there is at most one workgroup per CU anyway: then two row tiles (17..32 rows, 16 KiB per wave for
  // 4-bit weights) take 128 KiB and keep eight waves instead of four (M = 32, 4096 -> 14336, four
  // row-blocks per workgroup: 13.9 us against 15.7 us; 14336 -> 4096: 19.1 us against 25.1 us).  With
  // four row tiles (33..64 rows) a wave's two buffers are 32 KiB and one workgroup of four waves takes
  // 128 KiB.  Sixteen waves of one row tile measured no faster than eight.
  constexpr int kLdsMax = 131072;
  const dim3 grid((unsigned)((a.f.NT + NTW - 1) / NTW), (unsigned)splits, (unsigned)slots);
  const bool alone = MT == 2 && grid.x * grid.y <= 256;
  const int lds_cap = (MT > 2 || alone) ? kLdsMax : 65536;
  const int max_w = lds_cap / (2 * Geo::SLICE);
  a.KTs = (int)((a.f.KT + splits - 1) / splits);
  a.W = a.KTs < max_w ? a.KTs : max_w;
  if (a.W > kDqMaxWaves) a.W = kDqMaxWaves;
  size_t smem = (size_t)a.W * 2 * Geo::SLICE;
  const size_t red = (size_t)NTW * MT * a.W * 64 * sizeof(f4);
  if (red > smem) smem = red;
  auto kern = woq_decode_dq_kernel<REGIME, WBITS, MT, NTW, NF4, XCONV, FP8, GROUPED, SZB>;
  if (MT >= 2) {
    // more than 64 KiB of LDS per workgroup needs an opt-in (once per kernel and process)
    static const hipError_t lds_optin =
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsMax);
    if (lds_optin != hipSuccess)
      return set_error("woq_decode_dq_kernel: LDS opt-in failed: %s", hipGetErrorString(lds_optin));
  }
  kern<<<grid, a.W * 64, smem, st>>>(a);
  return check_launch("woq_decode_dq_kernel");
}

template <int REGIME, int WBITS, int MT, int NTW, bool NF4 = false, bool XCONV = false, bool FP8 = false, bool GROUPED = false>
static int launch_dq_cfg(DecodeDqArgs a, int splits, hipStream_t st, int slots = 1) {
  if constexpr (REGIME == kRegimeBF16 && !NF4 && !FP8 && !GROUPED && !XCONV) {
    // the caller's merged (scale, zero) dword table: one parameter request per row-block and round
    if (a.f.szb) return launch_dq_cfg_impl<REGIME, WBITS, MT, NTW, NF4, XCONV, FP8, GROUPED, true>(a, splits, st, slots);
  }
  return launch_dq_cfg_impl<REGIME, WBITS, MT, NTW, NF4, XCONV, FP8, GROUPED, false>(a, splits, st, slots);
}

// At most 64 rows already in the compute dtype (or up to 16 bf16 rows for fp16 compute), whole K tiles, and (4-bit) a group size whose
// boundaries never split a lane's 32 consecutive K values (8-bit: 16).
bool decode_dq_applies(const FpArgs& f, int wbits, int regime) {
  const int want = regime == kRegimeF16 ? WOQ_HIP_ACT_FP16 : WOQ_HIP_ACT_BF16;
  const int tk = wbits == 4 ? kTileK4 : kTileK8;
  // bf16 rows under the fp16 regime are converted on the way in, up to one row tile
  const bool converts = regime == kRegimeF16 && f.x_dtype == WOQ_HIP_ACT_BF16 && f.M <= 16;
  if (f.M > 64 || (f.x_dtype != want && !converts) || ((uintptr_t)f.x & 15) != 0) return false;
  if (f.K % tk != 0 || f.M * f.K * 2 >= (int64_t)1 << 31) return false;
  if (f.G >= f.KT * tk) return true;
  return f.G >= (wbits == 4 ? 32 : 16) && (f.G & (f.G - 1)) == 0;
}

template <int REGIME, int WBITS, bool FP8 = false>
static int launch_dq_regime(const DecodeDqArgs& a, int ntw, int splits, hipStream_t st) {
  const int mt = a.f.M > 32 ? 4 : a.f.M > 16 ? 2 : 1;
  if constexpr (REGIME == kRegimeF16) {
    if (a.f.x_dtype == WOQ_HIP_ACT_BF16) {  // one row tile, rows converted to fp16 on the way in
      if (ntw == 4) return launch_dq_cfg<REGIME, WBITS, 1, 4, false, true, FP8>(a, splits, st);
      if (ntw == 3) {
        if constexpr (FP8)
          return set_error("woq_decode_dq_kernel: FP8 weights take 1, 2 or 4 row-blocks per workgroup");
        else
          return launch_dq_cfg<REGIME, WBITS, 1, 3, false, true>(a, splits, st);
      }
      if (ntw == 2) return launch_dq_cfg<REGIME, WBITS, 1, 2, false, true, FP8>(a, splits, st);
      return launch_dq_cfg<REGIME, WBITS, 1, 1, false, true, FP8>(a, splits, st);
    }
  }
  if (mt == 4) {
    // 33..64 rows: one, two or (integer weights: 16 accumulator tiles, so two waves per SIMD at most, which
    // is what the 128 KiB of activation buffers of four waves allow anyway) four row-blocks per workgroup
    if (ntw == 3 || (ntw == 4 && FP8))
      return set_error("woq_decode_dq_kernel: 33..64 rows take 1, 2 or (integer weights) 4 row-blocks per workgroup");
    if constexpr (!FP8) {
      if (ntw == 4) return launch_dq_cfg<REGIME, WBITS, 4, 4>(a, splits, st);
    }
    return ntw == 2 ? launch_dq_cfg<REGIME, WBITS, 4, 2, false, false, FP8>(a, splits, st) : launch_dq_cfg<REGIME, WBITS, 4, 1, false, false, FP8>(a, splits, st);
  }
  const bool two_rows = mt == 2;
  if (ntw == 3) {
    if constexpr (FP8)
      return set_error("woq_decode_dq_kernel: FP8 weights take 1, 2 or 4 row-blocks per workgroup");
    else
      return two_rows ? launch_dq_cfg<REGIME, WBITS, 2, 3>(a, splits, st) : launch_dq_cfg<REGIME, WBITS, 1, 3>(a, splits, st);
  }
  if (ntw == 4) return two_rows ? launch_dq_cfg<REGIME, WBITS, 2, 4, false, false, FP8>(a, splits, st) : launch_dq_cfg<REGIME, WBITS, 1, 4, false, false, FP8>(a, splits, st);
  if (ntw == 2) return two_rows ? launch_dq_cfg<REGIME, WBITS, 2, 2, false, false, FP8>(a, splits, st) : launch_dq_cfg<REGIME, WBITS, 1, 2, false, false, FP8>(a, splits, st);
  return two_rows ? launch_dq_cfg<REGIME, WBITS, 2, 1, false, false, FP8>(a, splits, st) : launch_dq_cfg<REGIME, WBITS, 1, 1, false, false, FP8>(a, splits, st);
}

// NF4: one or two row-blocks per workgroup.
template <int REGIME>
static int launch_dq_nf4(const DecodeDqArgs& a, int ntw, int splits, hipStream_t st) {
  if constexpr (REGIME == kRegimeF16) {
    if (a.f.x_dtype == WOQ_HIP_ACT_BF16)
      return ntw == 2 ? launch_dq_cfg<REGIME, 4, 1, 2, true, true>(a, splits, st)
                      : launch_dq_cfg<REGIME, 4, 1, 1, true, true>(a, splits, st);
  }
  if (a.f.M > 32)  // four row tiles
    return ntw == 2 ? launch_dq_cfg<REGIME, 4, 4, 2, true>(a, splits, st) : launch_dq_cfg<REGIME, 4, 4, 1, true>(a, splits, st);
  const bool two_rows = a.f.M > 16;
  if (ntw == 2) return two_rows ? launch_dq_cfg<REGIME, 4, 2, 2, true>(a, splits, st) : launch_dq_cfg<REGIME, 4, 1, 2, true>(a, splits, st);
  return two_rows ? launch_dq_cfg<REGIME, 4, 2, 1, true>(a, splits, st) : launch_dq_cfg<REGIME, 4, 1, 1, true>(a, splits, st);
}

// Grouped launch over the slots of a mixture-of-experts layer: INT4 / INT8 weights, two row-blocks per workgroup, one
// row tile (up to 16 rows per slot) or four (up to 64), K never split.  f describes one expert's problem with M = the
// bound on a slot's rows; the slots' experts, rows and tensors come from grp (device memory).
template <int REGIME, int WBITS>
static int launch_dq_grouped_regime(const DecodeDqArgs& a, int slots, hipStream_t st) {
  const bool four = a.f.M > 16;
  if constexpr (REGIME == kRegimeF16) {
    if (a.f.x_dtype == WOQ_HIP_ACT_BF16) {
      if (four) return set_error("woq_linear_grouped: bf16 rows under fp16 compute take at most 16 rows per slot");
      return launch_dq_cfg<REGIME, WBITS, 1, 2, false, true, false, true>(a, 1, st, slots);
    }
  }
  return four ? launch_dq_cfg<REGIME, WBITS, 4, 2, false, false, false, true>(a, 1, st, slots)
              : launch_dq_cfg<REGIME, WBITS, 1, 2, false, false, false, true>(a, 1, st, slots);
}

int launch_decode_dq_grouped(const FpArgs& f, int wbits, int regime, const MoeGroup* grp, int64_t slots, hipStream_t st) {
  if (!grp || slots < 1 || slots > 65535) return set_error("woq_linear_grouped: 1..65535 slots and a group table");
  if (f.nf4 || f.fp8) return set_error("woq_linear_grouped: INT4 and INT8 weights");
  if (f.NT % 2 != 0) return set_error("woq_linear_grouped: an even number of row-blocks (N a multiple of 32 after padding)");
  if (!decode_dq_applies(f, wbits, regime))
    return set_error("woq_linear_grouped: at most 64 rows per slot, K a multiple of the weight tile, a power-of-two or "
                     "per-channel group size and rows in the compute dtype (bf16 rows under fp16 compute: 16 per slot)");
  DecodeDqArgs a;
  a.f = f;
  a.partial = nullptr;
  a.counters = nullptr;
  a.grp = grp;
  a.W = 1;
  a.KTs = (int)f.KT;
  a.g_shift = 30;
  if (f.G < f.KT * (wbits == 4 ? kTileK4 : kTileK8)) {
    a.g_shift = 0;
    while (((int64_t)1 << a.g_shift) < f.G) ++a.g_shift;
  }
  if (wbits == 4)
    return regime == kRegimeF16 ? launch_dq_grouped_regime<kRegimeF16, 4>(a, (int)slots, st)
                                : launch_dq_grouped_regime<kRegimeBF16, 4>(a, (int)slots, st);
  return regime == kRegimeF16 ? launch_dq_grouped_regime<kRegimeF16, 8>(a, (int)slots, st)
                              : launch_dq_grouped_regime<kRegimeBF16, 8>(a, (int)slots, st);
}

int64_t decode_dq_splitk_bytes(int64_t M, int64_t NT, int splits) {
  return (int64_t)splits * NT * (M > 16 ? 2 : 1) * 256 * (int64_t)sizeof(float);
}

int launch_decode_dq(const FpArgs& f, int wbits, int regime, hipStream_t st, int ntw, int splits,
                     const SplitKScratch* scratch) {
  DecodeDqArgs a;
  a.f = f;
  a.partial = scratch ? scratch->partial : nullptr;
  a.counters = scratch ? scratch->counters : nullptr;
  a.grp = nullptr;
  a.W = 1;
  a.KTs = (int)f.KT;
  a.g_shift = 30;
  if (f.G < f.KT * (wbits == 4 ? kTileK4 : kTileK8)) {
    a.g_shift = 0;
    while (((int64_t)1 << a.g_shift) < f.G) ++a.g_shift;
  }
  if (ntw < 0 || ntw > 4)
    return set_error("woq_decode_dq_kernel: 1 to 4 row-blocks per workgroup, got %d", ntw);
  if (ntw == 3 && splits > 1) return set_error("woq_decode_dq_kernel: three row-blocks per workgroup run unsplit");
  if (ntw != 0 && ntw != 3 && f.NT % ntw != 0)
    return set_error("woq_decode_dq_kernel: %d row-blocks per workgroup do not divide %lld", ntw, (long long)f.NT);
  // More row-blocks per workgroup re-read the activations less often (every workgroup streams all
  // of x through LDS); fewer make more workgroups, which small N needs to fill the chip.  Measured at
  // M = 16 / 32: 4096 -> 14336 (896 row-blocks) 14.4 / 11.4 / 10.7 us with 1 / 2 / 4, 4096 -> 6144 (384)
  // 8.5 / 7.0 / 9.7 us, 14336 -> 4096 (256) 12.9 / 15.5 / 24.5 us.  33..64 rows (four row tiles, no
  // variant with four row-blocks) have four times the activation bytes per workgroup.
  // Up to 32 rows: the count with the shortest schedule -- generations of 256 workgroups (one per CU and
  // round; a second workgroup on a CU shares its vector pipes) times a workgroup's length, which is its
  // row-blocks plus a fixed part for streaming the activations (about half a row-block's worth, from the
  // 1 / 2 / 4 figures above); ties go to the larger count.  That gives 1 up to 256 row-blocks, 2 up to 512
  // (288 row-blocks, M = 16 / 32: 6.9 / 8.4 us against 8.3 / 10.9 us with one), 3 up to 768 (4096 -> 11008, 688
  // row-blocks: INT4 G = 128 at M = 8 / 16 / 32 8.4 / 8.8 / 10.8 us against 9.9 / 10.2 / 12.5 us with four, INT8
  // per channel at M = 32 12.8 against 14.5 us), 4 up to 1024 (at 832 row-blocks three make 278 workgroups
  // and lose, 17.3 against 12.7 us), then whichever of 3 and 4 wastes less of the last generation (1376
  // row-blocks: three).  A count that does not divide the row-blocks is fine: the last workgroup repeats
  // the last row-block.
  const bool auto_ntw = ntw == 0;
  if (ntw == 0) {
    if (f.M <= 32 && !f.nf4) {
      double best = 0.0;
      for (int cand = 1; cand <= 4; ++cand) {
        if (cand == 3 && f.fp8) continue;  // no such instances
        const int64_t wgs = (f.NT + cand - 1) / cand;
        const double cost = (double)((wgs + 255) / 256) * (cand * 1.9 + 1.0);
        if (ntw == 0 || cost <= best) {
          best = cost;
          ntw = cand;
        }
      }
    } else if (f.M > 32 && !f.nf4 && !f.fp8) {
      // four row tiles: streaming 33..64 activation rows is the larger part of a workgroup's time (256
      // workgroups of one / two row-blocks at M = 64: 11.7 / 14.3 us), so the same rule with that fixed part
      double best = 0.0;
      for (int cand = 1; cand <= 4; cand *= 2) {
        const int64_t wgs = (f.NT + cand - 1) / cand;
        const double cost = (double)((wgs + 255) / 256) * (cand * 2.5 + 7.0);
        if (ntw == 0 || cost <= best) {
          best = cost;
          ntw = cand;
        }
      }
    } else {
      ntw = f.NT > 256 ? 2 : 1;  // 288 row-blocks, M = 64: 13.9 us against 20.6 us with one
    }
  }
  // Few output columns and a long K: one row-block per workgroup fills the chip but re-reads the
  // activations once per 16 columns.  Two workgroups per row-block set, each with half of the K tiles
  // and twice the row-blocks, halve that traffic: 14336 -> 4096 (256 row-blocks), G = 128, takes
  // 10.8 / 11.2 / 15.1 us at M = 8 / 16 / 32 against 12.7 / 13.6 / 19.1 us unsplit (four splits of four
  // row-blocks: 13.3 / 13.4 / 17.1 us); at K = 4096 the unsplit form stays faster (4096 -> 4096, M = 16:
  // 6.0 against 7.0 us).
  if (splits == 0) {
    splits = 1;
    const bool have = scratch && scratch->partial && scratch->counters &&
                      scratch->bytes >= decode_dq_splitk_bytes(f.M, f.NT, 2);
    if (have && auto_ntw && f.M >= 5 && f.M <= 32 && f.K >= 8192 && f.NT <= 256) {
      splits = 2;
      ntw = (f.NT > 128 && f.NT % 2 == 0) ? 2 : 1;
    }
  }
  if (splits != 1 && splits != 2 && splits != 4)
    return set_error("woq_decode_dq_kernel: 1, 2 or 4 K splits, got %d", splits);
  if (splits > 1) {
    if (f.M > 32) return set_error("woq_decode_dq_kernel: split K takes at most 32 rows");
    if (!a.partial || !a.counters)
      return set_error("woq_decode_dq_kernel: split K needs the partial-tile workspace and the counter array");
    if (scratch->bytes < decode_dq_splitk_bytes(f.M, f.NT, splits))
      return set_error("woq_decode_dq_kernel: split K needs %lld bytes of workspace, got %lld",
                       (long long)decode_dq_splitk_bytes(f.M, f.NT, splits), (long long)scratch->bytes);
    if (f.NT / ntw > kSplitKCounters)
      return set_error("woq_decode_dq_kernel: split K takes at most %d row-block sets", kSplitKCounters);
  }
  if (f.nf4) {
    if (wbits != 4 || f.zeros) return set_error("woq_decode_dq_kernel: NF4 weights are 4-bit and symmetric");

    if (ntw > 2) return set_error("woq_decode_dq_kernel: NF4 weights take 1 or 2 row-blocks per workgroup");
    return regime == kRegimeF16 ? launch_dq_nf4<kRegimeF16>(a, ntw, splits, st)
                                : launch_dq_nf4<kRegimeBF16>(a, ntw, splits, st);
  }
  if (wbits == 4)
    return regime == kRegimeF16 ? launch_dq_regime<kRegimeF16, 4>(a, ntw, splits, st)
                                : launch_dq_regime<kRegimeBF16, 4>(a, ntw, splits, st);
  if (f.fp8) {  // float8 bytes: own instances, so that the integer ones keep their registers
    if (wbits != 8 || f.zeros) return set_error("woq_decode_dq_kernel: FP8 weights are bytes without zero points");
    return regime == kRegimeF16 ? launch_dq_regime<kRegimeF16, 8, true>(a, ntw, splits, st)
                                : launch_dq_regime<kRegimeBF16, 8, true>(a, ntw, splits, st);
  }
  return regime == kRegimeF16 ? launch_dq_regime<kRegimeF16, 8>(a, ntw, splits, st)
                              : launch_dq_regime<kRegimeBF16, 8>(a, ntw, splits, st);
}

}  // namespace woq

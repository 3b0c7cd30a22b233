// int8 MFMA kernels for 4-bit weights under lowp_mode INT8: the GEMM form for large M (prefill,
// below) and the decode form for up to 32 rows (further down); symmetric activation quantization
// (per tensor, per row, per K block or per row and K block), K blocks of 128.
//
// Reference counterpart: Dequantize<int8_t> of a [128 x 32] weight block, int8 BRGEMM into int32,
// then the fp32 epilogue C += (float(sum) * s_a[m]) * s_w[n, g] per K block
// (csrc/cpu/aten/utils/woq.h:1664-1734, 2133-2199; driver woq.h:3298-3452).
//
// Same decomposition as the bf16 prefill kernel: v_mfma_i32_16x16x64_i8 with A = quantized
// activations (row m = lane % 16, 16 K values per lane) and B = weights (column n = lane % 16);
// the two packed dwords of a lane, decoded to sixteen int8 (q - z), ARE the B operand, so every
// weight is decoded once per 64 rows by exactly one wave and never stored.  The activations
// (already quantized, each group of eight in the order the nibble decode produces) and the packed
// tiles go from global memory straight into LDS (global_load_lds_dwordx4), two K steps ahead; 16-byte
// chunk p of activation row m sits at chunk p ^ swz_row128(m), which makes the fragment reads
// conflict-free for 128-byte rows.
// The int32 sums of a K step (128 K values = the reference's K block) are scaled into fp32
// accumulators right away: four VALU instructions per output element and step, which is what
// bounds the kernel.  A workgroup is 64 rows x 128 columns so that three fit on a CU (152 registers,
// 48 KiB of LDS): with 128 rows and one wave per SIMD the LDS reads, the barrier and the MFMAs of a
// step all sat exposed between its VALU work (452 us for M = 2048, 4096 -> 14336, against 245 us).
#include "woq_common.h"
#include "woq_internal.h"

// the three roundings of the epilogue stay separate (see woq_int8.hip)
#pragma clang fp contract(off)

namespace woq {

constexpr int W8_WAVES = 4;
constexpr int W8_MT = 4;    // 16-row tiles: 64 rows per workgroup
constexpr int W8_NTW = 2;   // weight row-blocks per wave: 128 columns per workgroup
constexpr int W8_BM = 16 * W8_MT;
constexpr int W8_BN = W8_WAVES * W8_NTW * kTileN;
constexpr int W8_XBYTES = W8_BM * kTileK4;                     // one activation buffer (int8)
constexpr int W8_XLOADS = W8_XBYTES / (W8_WAVES * 1024);       // LDS loads per wave and buffer
constexpr int W8_WSTAGE = W8_WAVES * W8_NTW * kTileBytes;      // one weight stage (4-bit codes)
constexpr int W8_NBUF = 3;    // activation buffers and weight stages: requests run two K steps ahead
constexpr int W8_LDS_BYTES = W8_NBUF * (W8_XBYTES + W8_WSTAGE + W8_BM * (int)sizeof(float));
// 8-bit weights: two packed tiles (64 K values each) per row-block and K step
constexpr int W8_LDS_BYTES_W8 = W8_NBUF * (W8_XBYTES + 2 * W8_WSTAGE + W8_BM * (int)sizeof(float));

struct W4I8Args {
  const uint8_t* xq;       // [M][ldq] int8, groups of eight in nibble-decode order
  int64_t ldq;
  const float* sa;         // activation scales: sa[m * sa_m_stride + (kt >> q_shift) * sa_k_stride]
  int64_t sa_m_stride;     // per row: scales per row (1 or the K blocks per row), else 0
  int64_t sa_k_stride;     // per K block: 1, else 0
  int q_shift;             // K tile kt belongs to activation K block kt >> q_shift
  const int32_t* za;       // asymmetric activations: zero points, indexed like sa; xq then holds q_a - 128
  int64_t M, N, NT, KT, KG;
  const uint8_t* qweight;
  const float* scales;     // fp32 [NT][KG][16]
  const uint8_t* zeros;    // [NT][KG][16] or nullptr (symmetric: codes stand for code - 8)
  int g_shift;             // K tile kt belongs to group kt >> g_shift
  Epilogue ep;
  // GEMM form with gridDim.z > 1: K steps per workgroup, fp32 partial tiles, one counter per tile
  int kts;
  float* sk_partial;
  int* sk_counters;
};

typedef __attribute__((address_space(3))) void* w8_lds_ptr_t;
typedef const __attribute__((address_space(1))) void* w8_global_ptr_t;

// Four bytes at once: ((b | 0x80808080) - z4) ^ 0x80808080 never borrows across bytes for
// |q - z| < 128 and leaves q - z in two's complement.
__device__ __forceinline__ uint32_t w8_sub_bytes(uint32_t b, uint32_t z4) {
  return ((b | 0x80808080u) - z4) ^ 0x80808080u;
}
// sixteen K values of one lane from two packed dwords, in the order [e0 e4 e1 e5][e2 e6 e3 e7] per dword
__device__ __forceinline__ i4 w8_decode16(uint32_t d0, uint32_t d1, uint32_t z4) {
  i4 r;
  r[0] = (int)w8_sub_bytes(d0 & 0x0F0F0F0Fu, z4);
  r[1] = (int)w8_sub_bytes((d0 >> 4) & 0x0F0F0F0Fu, z4);
  r[2] = (int)w8_sub_bytes(d1 & 0x0F0F0F0Fu, z4);
  r[3] = (int)w8_sub_bytes((d1 >> 4) & 0x0F0F0F0Fu, z4);
  return r;
}

// One K block's int32 sum into the fp32 accumulator.  The reference computes
// C += (float(sum) * s_a) * s_w per block (csrc/cpu/aten/utils/woq.h:2172-2186; its compiler is free to
// contract the last multiply and the addition).  PER_K: exactly that, with the contraction: convert,
// multiply, fused multiply-add.  Otherwise s_a is the same for every block of a row and is applied
// once after the K loop, C = (sum over blocks of float(sum) * s_w) * s_a: convert and one fused
// multiply-add per block, a third fewer VALU instructions in a loop that they bound; the results
// differ from the per-block order by fp32 rounding only (~1e-7 relative).
template <bool PER_K>
__device__ __forceinline__ float w8_accumulate(int sum, float s_a, float s_w, float acc) {
  if constexpr (PER_K)
    return __builtin_fmaf((float)sum * s_a, s_w, acc);
  else
    return __builtin_fmaf((float)sum, s_w, acc);
}

// Asymmetric activations (uint8 q_a with zero point z_a; csrc/cpu/aten/utils/woq.h:2172-2186): the
// reference's block integer is sum q_a B - z_a sum B.  The activations arrive as the int8 numbers
// q_a - 128, so it equals (sum (q_a - 128) B) + (128 - z_a) sum B, with the column sums of the block's
// weights ("compensation") from one more pair of MFMAs against rows of ones: every row of that D tile
// is the same, so register 0 of a lane is the sum of its column n = lane % 16.
__device__ __forceinline__ int w8_column_sums(i4 bq0, i4 bq1) {
  const i4 ones = i4{0x01010101, 0x01010101, 0x01010101, 0x01010101};
  i4 cv = __builtin_amdgcn_mfma_i32_16x16x64_i8(ones, bq0, i4{0, 0, 0, 0}, 0, 0, 0);
  cv = __builtin_amdgcn_mfma_i32_16x16x64_i8(ones, bq1, cv, 0, 0, 0);
  return cv[0];
}

// NF4 codes under lowp_mode INT8: the code's table value times 127, rounded, as int8
// (load_nf4_as_int8, csrc/cpu/aten/utils/woq.h:628-669): two byte permutes over the halves of the
// table (codes 0..7 and 8..15), merged on bit 3 of each code; the weight scale carries the 1 / 127.
__device__ __forceinline__ uint32_t w8_nf4_codes_to_i8(uint32_t b) {
  // -127 -88 -67 -50 | -36 -23 -12 0 | 10 20 31 43 | 56 71 92 127, least significant byte first
  const uint32_t t0 = 0xCEBDA881u, t1 = 0x00F4E9DCu, t2 = 0x2B1F140Au, t3 = 0x7F5C4738u;
  const uint32_t sel = b & 0x07070707u;
  const uint32_t lo = __builtin_amdgcn_perm(t1, t0, sel);
  const uint32_t hi = __builtin_amdgcn_perm(t3, t2, sel);
  const uint32_t m = ((b >> 3) & 0x01010101u) * 0xFFu;
  return (hi & m) | (lo & ~m);
}
__device__ __forceinline__ i4 w8_decode16_nf4(uint32_t d0, uint32_t d1) {
  i4 r;
  r[0] = (int)w8_nf4_codes_to_i8(d0 & 0x0F0F0F0Fu);
  r[1] = (int)w8_nf4_codes_to_i8((d0 >> 4) & 0x0F0F0F0Fu);
  r[2] = (int)w8_nf4_codes_to_i8(d1 & 0x0F0F0F0Fu);
  r[3] = (int)w8_nf4_codes_to_i8((d1 >> 4) & 0x0F0F0F0Fu);
  return r;
}

// PER_K: the activation scales change with the K block; they reach the lanes through LDS.
// ASYM: asymmetric activations (w8_column_sums); the zero points travel like the scales.
// WBITS 8: symmetric 8-bit weights, stored offset-binary: a K step of 128 takes two packed tiles per
// row-block (one MFMA each), the lane's 16 bytes with the sign bit flipped are the B operand, and the A
// fragment of tile u is chunk 4 u + c of the 128-byte row (the activations keep their plain byte order).
// The doubled weight stages leave two workgroups per CU instead of three.
// NF4: the codes index the int8 NormalFloat4 table (no zero points; scale / 127).
// GSUB > 1: groups of 64 or 32 input channels, i.e. 2 or 4 K blocks per packed tile, each computed with
// the other blocks' lane columns of the B operand zeroed (see woq_decode_w4i8_kernel) and scaled on its
// own: GSUB times the MFMAs and the fp32 scalings of a step.
// (their extra scales and the second set of int32 sums do not fit the registers of three workgroups per
// CU: two).
template <bool PER_K, bool ASYM = false, int WBITS = 4, bool NF4 = false, int GSUB = 1>
__global__ __launch_bounds__(256, (GSUB > 1 ? 2 : 3)) void woq_gemm_w4i8_kernel(const W4I8Args a) {
  static_assert(GSUB == 1 || (WBITS == 4 && !ASYM && !NF4), "K blocks inside a tile: 4-bit integer codes, symmetric activations");
  static_assert(WBITS == 4 || (WBITS == 8 && !ASYM), "8-bit weights: symmetric activations only");
  static_assert(!NF4 || (WBITS == 4 && !ASYM), "NF4 codes: 4 bits wide, symmetric activations only");
  constexpr int TPS = WBITS / 4;  // packed tiles per row-block and K step
  constexpr int WSTAGE = TPS * W8_WSTAGE;
  // the activation buffers, then the weight stages, then the activation scales (and, ASYM, zero points)
  // of a step's rows
  extern __shared__ __align__(1024) uint8_t sX[];
  uint8_t* const sW = sX + W8_NBUF * W8_XBYTES;
  float* const sSA = (float*)(sW + W8_NBUF * WSTAGE);
  int32_t* const sZA = (int32_t*)(sSA + W8_NBUF * GSUB * W8_BM);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, c = lane >> 4;
  const int M = (int)a.M, NT = (int)a.NT, KTW = (int)a.KT / TPS, KG = (int)a.KG;
  // K steps (of 128 values) of this workgroup: [kt_lo, KT).  gridDim.z > 1 (few tiles, long K): the workgroups of a tile
  // share K; each writes its fp32 accumulators to scratch and the one that arrives last at the tile's
  // counter adds the partial tiles in z order and stores -- the scheme of the bf16 prefill kernel.
  const int kt_lo = (int)blockIdx.z * a.kts;
  const int KT = KTW < kt_lo + a.kts ? KTW : kt_lo + a.kts;
  const int m0 = blockIdx.y * W8_BM;
  const int nt0 = (blockIdx.x * W8_WAVES + wave) * W8_NTW;

  f4 acc[W8_MT][W8_NTW];
#pragma unroll
  for (int mt = 0; mt < W8_MT; ++mt)
#pragma unroll
    for (int t = 0; t < W8_NTW; ++t) acc[mt][t] = f4{0.f, 0.f, 0.f, 0.f};

  // activation scales of this lane's accumulator rows m = 16 mt + 4 c + e: constant over K, or
  // (PER_K) read from LDS at the top of every step, where wave 0 put them a step earlier
  f4 sa[W8_MT];
  if (!PER_K) {
#pragma unroll
    for (int mt = 0; mt < W8_MT; ++mt)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int m = m0 + mt * 16 + 4 * c + e;
        sa[mt][e] = a.sa[(int64_t)(m < M ? m : M - 1) * a.sa_m_stride];
      }
  }
  const int sa_row = m0 + tid < M ? m0 + tid : M - 1;  // wave 0: the row whose scale this thread fetches
  const float* const sa_mine = a.sa + (int64_t)sa_row * a.sa_m_stride;
  float sa_next[GSUB];
  // activation K block of scale g of K step kt
  auto sa_block = [&](int kt, int g) { return GSUB == 1 ? (int64_t)(kt >> a.q_shift) : (int64_t)kt * GSUB + g; };
  const int my_block = c / (4 / GSUB);  // K block of the tile this lane column's weights belong to
  // 128 - z_a of the same rows
  i4 zoff[ASYM ? W8_MT : 1];
  if (ASYM && !PER_K) {
#pragma unroll
    for (int mt = 0; mt < (ASYM ? W8_MT : 1); ++mt)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int m = m0 + mt * 16 + 4 * c + e;
        zoff[mt][e] = 128 - a.za[(int64_t)(m < M ? m : M - 1) * a.sa_m_stride];
      }
  }
  const int32_t* const za_mine = ASYM ? a.za + (int64_t)sa_row * a.sa_m_stride : nullptr;
  int32_t za_next = 0;

  // ---- activations: load i of wave w fills LDS KiB number w * XLOADS + i of a buffer: rows
  // 8 (w * XLOADS + i) + lane / 8, physical chunk lane % 8 = logical chunk ^ swz_row128(row).
  // Rows past M re-read row M - 1; their results are never stored. ----
  uint32_t xoff[W8_XLOADS];
#pragma unroll
  for (int i = 0; i < W8_XLOADS; ++i) {
    const int rowl = (wave * W8_XLOADS + i) * 8 + (lane >> 3);
    const int rowc = m0 + rowl < M ? rowl : M - 1 - m0;
    const int chunk = (lane & 7) ^ swz_row128(rowl);
    xoff[i] = (uint32_t)(rowc * (int)a.ldq + chunk * 16);
  }
  const uint8_t* xbase = a.xq + (int64_t)m0 * a.ldq;
  auto load_x = [&](int kt, int buf) {
    const uint32_t ko = (uint32_t)kt * kTileK4;
#pragma unroll
    for (int i = 0; i < W8_XLOADS; ++i)
      __builtin_amdgcn_global_load_lds((w8_global_ptr_t)(xbase + (uint32_t)(xoff[i] + ko)),
                                       (w8_lds_ptr_t)(sX + buf * W8_XBYTES + (wave * W8_XLOADS + i) * 1024), 16, 0,
                                       0);
  };
  // A fragment of row tile mt, MFMA j: row 16 mt + r, logical chunk 2 c + j
  uint32_t rd[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
    rd[j] = (uint32_t)(r * 128 + (((WBITS == 4 ? 2 * c + j : 4 * j + c) ^ swz_row128(r)) << 4));

  // ---- weights ----
  const bool has_z = a.zeros != nullptr;
  const uint8_t* wbase[W8_NTW];
  const float* sbase[W8_NTW];
  const uint8_t* zbase[W8_NTW];
#pragma unroll
  for (int t = 0; t < W8_NTW; ++t) {
    const int nt = nt0 + t < NT ? nt0 + t : NT - 1;
    wbase[t] = a.qweight + (size_t)nt * KTW * (TPS * kTileBytes);
    sbase[t] = a.scales + (size_t)nt * KG * kTileN;
    zbase[t] = has_z ? a.zeros + (size_t)nt * KG * kTileN : (const uint8_t*)sbase[t];
  }
  const uint32_t woff = (uint32_t)lane * 16u;
  uint8_t* const wmine = sW + wave * (W8_NTW * TPS * kTileBytes);
  auto dma_w = [&](int kt, int stage) {
    const uint32_t wo = (uint32_t)kt * (TPS * kTileBytes) + woff;
#pragma unroll
    for (int t = 0; t < W8_NTW; ++t)
#pragma unroll
      for (int u = 0; u < TPS; ++u)
        __builtin_amdgcn_global_load_lds((w8_global_ptr_t)(wbase[t] + (uint32_t)(wo + u * kTileBytes)),
                                         (w8_lds_ptr_t)(wmine + stage * WSTAGE + (t * TPS + u) * kTileBytes), 16,
                                         0, 0);
  };
  // scale and zero point of this lane's accumulator column n = r... the D tile of an MFMA has column
  // n = lane % 16 in every lane, so one scale per row-block and lane; the B operand's column is the
  // same n, so the zero point is per lane too.
  auto load_q = [&](int kt, float (&s)[W8_NTW][GSUB], uint8_t (&z)[W8_NTW]) {
    // first group of the tile (GSUB == 1: the tile's only one, shared by 2^g_shift tiles)
    int g = GSUB == 1 ? (kt >> a.g_shift) : kt * GSUB;
    g = g < KG ? g : KG - 1;
    const uint32_t qoff = (uint32_t)(g * kTileN + r);
#pragma unroll
    for (int t = 0; t < W8_NTW; ++t) {
#pragma unroll
      for (int gg = 0; gg < GSUB; ++gg) s[t][gg] = sbase[t][qoff + gg * kTileN];
      // raw: any use here would wait for the load inside the request
      z[t] = *(zbase[t] + qoff + (GSUB == 1 ? 0 : my_block) * kTileN);
    }
  };
  // NF4: the table holds round(127 value), the scale carries the 1 / 127 (applied where a step's scales
  // become current, after their load has landed)
  auto current = [&](float v) { return NF4 ? v * (1.0f / 127.0f) : v; };

  constexpr int kVmcnt0 = 0x0F70;
  // all but the youngest request of activations and tiles (one K step's worth) have landed
  constexpr int kVmcntStep = 0x0F70 | (W8_XLOADS + W8_NTW * TPS);

  u4 wr[W8_NTW][TPS];
  float sw[W8_NTW][GSUB], swn[W8_NTW][GSUB];
  uint8_t zq[W8_NTW], zqn[W8_NTW];

  // A K step here is short (about 2000 cycles: 32 MFMAs and the fp32 epilogue of 64 sums per lane),
  // shorter than the round trip of a request, so activations and tiles are requested two steps ahead
  // into three buffers; the scales and zero points of the next step ride in registers.
  load_x(kt_lo, 0);
  dma_w(kt_lo, 0);
  load_x(KT > kt_lo + 1 ? kt_lo + 1 : kt_lo, 1);
  dma_w(KT > kt_lo + 1 ? kt_lo + 1 : kt_lo, 1);
  load_q(kt_lo, sw, zq);
  __builtin_amdgcn_s_waitcnt(kVmcnt0);
#pragma unroll
  for (int t = 0; t < W8_NTW; ++t)
#pragma unroll
    for (int g = 0; g < GSUB; ++g) sw[t][g] = current(sw[t][g]);
  __syncthreads();
#pragma unroll
  for (int t = 0; t < W8_NTW; ++t)
#pragma unroll
    for (int u = 0; u < TPS; ++u) wr[t][u] = *(const u4*)(wmine + (t * TPS + u) * kTileBytes + woff);

  if (PER_K && tid < W8_BM) {
#pragma unroll
    for (int g = 0; g < GSUB; ++g) sSA[g * W8_BM + tid] = sa_mine[sa_block(kt_lo, g) * a.sa_k_stride];
  }
  if (PER_K && ASYM && tid < W8_BM) sZA[tid] = za_mine[(int64_t)(kt_lo >> a.q_shift) * a.sa_k_stride];
  __syncthreads();

  // Per K step: the MFMAs of row-block 0, then those of row-block 1 with the fp32 epilogue of
  // row-block 0 between them, then the epilogue of row-block 1.  What stays exposed in one wave (the
  // fragment reads, the first MFMAs, the barrier) is covered by the other two workgroups of the CU.
  int b0 = 0, b1 = 1, b2 = 2;  // buffers of steps kt, kt + 1, kt + 2
  for (int kt = kt_lo; kt < KT; ++kt) {
    const uint8_t* xs = sX + b0 * W8_XBYTES;
    const int kt1 = kt + 1 < KT ? kt + 1 : KT - 1;
    const int kt2 = kt + 2 < KT ? kt + 2 : KT - 1;
    // requests, oldest first: parameters of step kt + 1, then activations and tiles of step kt + 2
    // into the buffers of step kt - 1, which every wave left before the last barrier
    load_q(kt1, swn, zqn);
    if (PER_K && tid < W8_BM) {
#pragma unroll
      for (int g = 0; g < GSUB; ++g) sa_next[g] = sa_mine[sa_block(kt1, g) * a.sa_k_stride];
    }
    if (PER_K && ASYM && tid < W8_BM) za_next = za_mine[(int64_t)(kt1 >> a.q_shift) * a.sa_k_stride];
    __builtin_amdgcn_sched_barrier(0);  // the parameter loads stay the oldest requests of the step
    load_x(kt2, b2);
    dma_w(kt2, b2);
    __builtin_amdgcn_sched_barrier(0);

    if (PER_K && GSUB == 1) {
#pragma unroll
      for (int mt = 0; mt < W8_MT; ++mt) sa[mt] = *(const f4*)(sSA + b0 * W8_BM + mt * 16 + 4 * c);
      if constexpr (ASYM) {
#pragma unroll
        for (int mt = 0; mt < W8_MT; ++mt)
          zoff[mt] = i4{128, 128, 128, 128} - *(const i4*)(sZA + b0 * W8_BM + mt * 16 + 4 * c);
      }
    }
    // A fragments of the step: 2 MFMAs x MT row tiles
    i4 xa[2][W8_MT];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int mt = 0; mt < W8_MT; ++mt) xa[j][mt] = *(const i4*)(xs + mt * 2048 + rd[j]);

    if constexpr (GSUB > 1) {
      // units (row-block t, K block g): the MFMAs of a unit with the fp32 scaling of the unit before
      // between them, the B operand masked to the lane columns of block g
      constexpr int NU = W8_NTW * GSUB;
      i4 qcu[2][W8_MT];
      i4 bqt0 = i4{0, 0, 0, 0}, bqt1 = i4{0, 0, 0, 0};
      f4 sap[W8_MT];  // PER_K: activation scales of the previous unit's K block
#pragma unroll
      for (int u = 0; u < NU; ++u) {
        const int t = u / GSUB, g = u % GSUB;
        if (g == 0) {
          const uint32_t z4 = (has_z ? (uint32_t)zq[t] : 8u) * 0x01010101u;
          bqt0 = w8_decode16(wr[t][0][0], wr[t][0][1], z4);
          bqt1 = w8_decode16(wr[t][0][2], wr[t][0][3], z4);
        }
        const bool mine = my_block == g;
        const i4 bm0 = mine ? bqt0 : i4{0, 0, 0, 0};
        const i4 bm1 = mine ? bqt1 : i4{0, 0, 0, 0};
        if (PER_K && u > 0) {
#pragma unroll
          for (int mt = 0; mt < W8_MT; ++mt)
            sap[mt] = *(const f4*)(sSA + (b0 * GSUB + (u - 1) % GSUB) * W8_BM + mt * 16 + 4 * c);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 2 * W8_MT; ++i) {
          const int mt = i % W8_MT;
          if (i < W8_MT)
            qcu[u & 1][mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xa[0][mt], bm0, i4{0, 0, 0, 0}, 0, 0, 0);
          else
            qcu[u & 1][mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xa[1][mt], bm1, qcu[u & 1][mt], 0, 0, 0);
          if (u > 0) {
            const int tp = (u - 1) / GSUB, gp = (u - 1) % GSUB;
#pragma unroll
            for (int w = 0; w < 2; ++w) {
              const int q = 2 * i + w, pm = q / 4, pe = q % 4;
              acc[pm][tp][pe] = w8_accumulate<PER_K>(qcu[(u - 1) & 1][pm][pe], PER_K ? sap[pm][pe] : 0.0f, sw[tp][gp],
                                                     acc[pm][tp][pe]);
            }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      if (PER_K) {
#pragma unroll
        for (int mt = 0; mt < W8_MT; ++mt)
          sap[mt] = *(const f4*)(sSA + (b0 * GSUB + GSUB - 1) * W8_BM + mt * 16 + 4 * c);
      }
#pragma unroll
      for (int mt = 0; mt < W8_MT; ++mt)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          acc[mt][W8_NTW - 1][e] = w8_accumulate<PER_K>(qcu[(NU - 1) & 1][mt][e], PER_K ? sap[mt][e] : 0.0f,
                                                        sw[W8_NTW - 1][GSUB - 1], acc[mt][W8_NTW - 1][e]);
    } else {
      i4 qc[W8_NTW][W8_MT];
      int cm[W8_NTW];  // ASYM: column sum of the block's weights, row-block t
  #pragma unroll
      for (int t = 0; t < W8_NTW; ++t) {
        i4 bq0, bq1;
        if constexpr (WBITS == 8) {
          // offset-binary bytes: flipping the sign bit leaves the two's complement weight
          bq0 = bitcast<i4>(wr[t][0] ^ u4{0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u});
          bq1 = bitcast<i4>(wr[t][TPS - 1] ^ u4{0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u});
        } else if constexpr (NF4) {
          bq0 = w8_decode16_nf4(wr[t][0][0], wr[t][0][1]);
          bq1 = w8_decode16_nf4(wr[t][0][2], wr[t][0][3]);
        } else {
          const uint32_t z4 = (has_z ? (uint32_t)zq[t] : 8u) * 0x01010101u;
          bq0 = w8_decode16(wr[t][0][0], wr[t][0][1], z4);
          bq1 = w8_decode16(wr[t][0][2], wr[t][0][3], z4);
        }
        cm[t] = ASYM ? w8_column_sums(bq0, bq1) : 0;
        __builtin_amdgcn_sched_barrier(0);
        // one MFMA, then (second row-block) the fp32 epilogue of two sums of the first:
        // C += (float(sum) * s_a[m]) * s_w[n, g]; each pair is fenced so that the order stands
  #pragma unroll
        for (int i = 0; i < 2 * W8_MT; ++i) {
          const int mt = i % W8_MT;
          if (i < W8_MT)
            qc[t][mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xa[0][mt], bq0, i4{0, 0, 0, 0}, 0, 0, 0);
          else
            qc[t][mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xa[1][mt], bq1, qc[t][mt], 0, 0, 0);
          if (t > 0) {
  #pragma unroll
            for (int u = 0; u < 2; ++u) {
              const int q = 2 * i + u, pm = q / 4, pe = q % 4;
              const int qv = ASYM ? qc[t - 1][pm][pe] + cm[t - 1] * zoff[ASYM ? pm : 0][pe] : qc[t - 1][pm][pe];
              acc[pm][t - 1][pe] = w8_accumulate<PER_K>(qv, sa[pm][pe], sw[t - 1][0], acc[pm][t - 1][pe]);
            }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
  #pragma unroll
      for (int mt = 0; mt < W8_MT; ++mt)
  #pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int qv = ASYM ? qc[W8_NTW - 1][mt][e] + cm[W8_NTW - 1] * zoff[ASYM ? mt : 0][e] : qc[W8_NTW - 1][mt][e];
          acc[mt][W8_NTW - 1][e] = w8_accumulate<PER_K>(qv, sa[mt][e], sw[W8_NTW - 1][0], acc[mt][W8_NTW - 1][e]);
        }

    }

    // Next step: its activations and tiles (requested a step ago) must have landed -- every wave
    // waits for its own requests, the barrier covers the others' -- and every wave must be done
    // reading this step's buffer.  Written as an instruction: before the barrier builtin the
    // compiler waits for every outstanding load, the requests for step kt + 2 included.
    if (PER_K) {
      if (tid < W8_BM) {
#pragma unroll
        for (int g = 0; g < GSUB; ++g) sSA[(b1 * GSUB + g) * W8_BM + tid] = sa_next[g];
      }
      if (ASYM && tid < W8_BM) sZA[b1 * W8_BM + tid] = za_next;
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the LDS write is done before the barrier
    }
    __builtin_amdgcn_s_waitcnt(kVmcntStep);
    asm volatile("s_barrier" ::: "memory");
#pragma unroll
    for (int t = 0; t < W8_NTW; ++t) {
#pragma unroll
      for (int u = 0; u < TPS; ++u)
        wr[t][u] = *(const u4*)(wmine + b1 * WSTAGE + (t * TPS + u) * kTileBytes + woff);
#pragma unroll
      for (int g = 0; g < GSUB; ++g) sw[t][g] = current(swn[t][g]);
      zq[t] = zqn[t];
    }
    const int b = b0;
    b0 = b1;
    b1 = b2;
    b2 = b;
  }
  // the requests past the last step are still writing LDS: drain them before the workgroup can end
  __builtin_amdgcn_s_waitcnt(kVmcnt0);

  if (gridDim.z > 1) {
    const int nsplit = (int)gridDim.z, z = (int)blockIdx.z;
    const int tiles = (int)(gridDim.x * gridDim.y), tile = (int)(blockIdx.y * gridDim.x + blockIdx.x);
    constexpr int kWaveFloats = W8_MT * W8_NTW * 256;
    float* const mine = a.sk_partial + ((size_t)(z * tiles + tile) * W8_WAVES + wave) * kWaveFloats + lane * 4;
#pragma unroll
    for (int mt = 0; mt < W8_MT; ++mt)
#pragma unroll
      for (int t = 0; t < W8_NTW; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          __hip_atomic_store(mine + (mt * W8_NTW + t) * 256 + e, acc[mt][t][e], __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_s_waitcnt(kVmcnt0);  // this thread's stores have completed
    __syncthreads();
    __shared__ int s_last;
    if (tid == 0)
      s_last = __hip_atomic_fetch_add(a.sk_counters + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == nsplit - 1;
    __syncthreads();
    if (!s_last) return;
    // the other workgroups' partial tiles, one after the other in z order: all loads of one in flight
    // together, then the additions (this workgroup's own tile comes from its registers, in its turn)
    f4 total[W8_MT][W8_NTW];
#pragma unroll 1
    for (int zz = 0; zz < nsplit; ++zz) {
      f4 v[W8_MT][W8_NTW];
      const float* const other = a.sk_partial + ((size_t)(zz * tiles + tile) * W8_WAVES + wave) * kWaveFloats + lane * 4;
#pragma unroll
      for (int mt = 0; mt < W8_MT; ++mt)
#pragma unroll
        for (int t = 0; t < W8_NTW; ++t) {
          v[mt][t] = acc[mt][t];
          if (zz != z) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              v[mt][t][e] = __hip_atomic_load(other + (mt * W8_NTW + t) * 256 + e, __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
          }
        }
#pragma unroll
      for (int mt = 0; mt < W8_MT; ++mt)
#pragma unroll
        for (int t = 0; t < W8_NTW; ++t) {
          if (zz == 0) {
            total[mt][t] = v[mt][t];
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) total[mt][t][e] = total[mt][t][e] + v[mt][t][e];
          }
        }
    }
#pragma unroll
    for (int mt = 0; mt < W8_MT; ++mt)
#pragma unroll
      for (int t = 0; t < W8_NTW; ++t) acc[mt][t] = total[mt][t];
    // the counter is back at zero for the next launch that uses it
    if (tid == 0) __hip_atomic_store(a.sk_counters + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  // ---- store: D[m][n], lane (n = r, c) holds rows m = 16 mt + 4 c + e ----
#pragma unroll
  for (int mt = 0; mt < W8_MT; ++mt)
#pragma unroll
    for (int t = 0; t < W8_NTW; ++t) {
      const int64_t n = (int64_t)(nt0 + t) * kTileN + r;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int64_t m = m0 + mt * 16 + 4 * c + e;
        const float y = PER_K ? acc[mt][t][e] : acc[mt][t][e] * sa[mt][e];
        if (m < M && n < a.N && nt0 + t < NT) epilogue_store<kRegimeBF16>(a.ep, m, n, y);
      }
    }
}

// ---- at most 16 rows (decode): the weight stream bounds the kernel -------------------------------
// Same work decomposition as the floating-point decode kernels: a workgroup owns NTW weight
// row-blocks and all of K, its W <= 8 waves take one K tile (= one K block of 128) each per round,
// the fp32 partial sums meet in LDS and are added in wave order.  Per tile and row-block: two
// v_mfma_i32_16x16x64_i8 on the decoded dwords, then the four sums of a lane go into its fp32
// accumulators as in the prefill kernel.  The quantized rows of a tile (16 x 128 bytes) are copied
// into the wave's own LDS slice (global_load_lds, swizzled as in the prefill kernel); requests run
// one round ahead.
// GSUB > 1: groups of 64 or 32 input channels, i.e. 2 or 4 K blocks per tile.  A lane column c holds
// the K values 32 c .. 32 c + 31 of the tile, all of one group, but an MFMA sums over the four lane
// columns; block g is therefore computed with the activation fragments of the other blocks' lane
// columns zeroed (GSUB times the MFMAs, which a decode step has to spare), and scaled with its own
// weight and activation scales.
struct DecodeW4I8Args {
  W4I8Args k;
  int W;  // waves per workgroup
};

// MT: 16-row tiles (one, two or four).  The forms with many K blocks and row tiles keep GSUB x MT sets of
// activation scales in flight and get the registers of two waves per SIMD instead of four.
// NF4: the codes index the int8 NormalFloat4 table (no zero points; scale / 127).
// WBITS 8: symmetric 8-bit weights, stored offset-binary; a packed tile is 16 rows x 64 K values, so a
// round takes two tiles per row-block (one MFMA each) and the lane's 16 bytes are the B operand as they
// are, sign bit flipped; the A fragment of tile u is chunk 4 u + c of the 128-byte row.
// ASYM: asymmetric activations (w8_column_sums), for 4-bit integer codes with one K block per tile.
template <bool PER_K, int MT, int NTW, int GSUB, bool NF4, int WBITS = 4, bool ASYM = false>
__global__ __launch_bounds__(512, (GSUB * MT > 4 ? 2 : 4)) void woq_decode_w4i8_kernel(const DecodeW4I8Args a) {
  static_assert(WBITS == 4 || (WBITS == 8 && GSUB == 1 && !NF4), "8-bit weights: one K block per round");
  static_assert(!ASYM || (WBITS == 4 && GSUB == 1 && !NF4), "asymmetric activations: 4-bit codes, one K block per tile");
  constexpr int TPR = WBITS / 4;  // packed tiles per row-block and round of 128 K values
  constexpr int SLICE = MT * 16 * kTileK4;  // one buffer of one wave: 16 MT rows x 128 bytes
  constexpr int NX = 2 * MT;                // activation loads per tile (eight rows each)
  extern __shared__ __align__(1024) uint8_t smem[];
  const W4I8Args& k = a.k;
  const int W = a.W;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int r = lane & 15, c = lane >> 4;
  const int M = (int)k.M, KTW = (int)k.KT, KG = (int)k.KG;
  const int KT = KTW / TPR;  // rounds of 128 K values
  const int64_t nt0 = (int64_t)blockIdx.x * NTW;
  uint8_t* const sx = smem + wave * (2 * SLICE);
  f4* const red = (f4*)smem;  // [NTW * MT][W][64], after the K loop

  f4 acc[NTW][MT];
#pragma unroll
  for (int t = 0; t < NTW; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f4{0.f, 0.f, 0.f, 0.f};

  // activation load i fills LDS bytes [1024 i, +1024) of a buffer: rows 8 i + lane / 8, physical
  // chunk lane % 8 = logical chunk ^ swz_row128(row); rows past M re-read row M - 1
  uint32_t xoff[NX];
#pragma unroll
  for (int i = 0; i < NX; ++i) {
    const int row = 8 * i + (lane >> 3);
    const int rowc = row < M ? row : M - 1;
    const int chunk = (lane & 7) ^ swz_row128(row);
    xoff[i] = (uint32_t)(rowc * (int)k.ldq + chunk * 16);
  }
  uint32_t rd[2];  // A fragment of MFMA j in row tile 0: row r, logical chunk 2 c + j (8-bit weights: 4 j + c)
#pragma unroll
  for (int j = 0; j < 2; ++j)
    rd[j] = (uint32_t)(r * 128 + ((((WBITS == 4 ? 2 * c + j : 4 * j + c)) ^ swz_row128(r)) << 4));

  const bool has_z = k.zeros != nullptr;
  const uint8_t* wbase[NTW];
  const float* sbase[NTW];
  const uint8_t* zbase[NTW];
#pragma unroll
  for (int t = 0; t < NTW; ++t) {
    wbase[t] = k.qweight + (size_t)(nt0 + t) * KTW * kTileBytes;
    sbase[t] = k.scales + (size_t)(nt0 + t) * KG * kTileN;
    zbase[t] = has_z ? k.zeros + (size_t)(nt0 + t) * KG * kTileN : (const uint8_t*)sbase[t];
  }
  const uint32_t woff = (uint32_t)lane * 16u;

  // activation scales of this lane's accumulator rows m = 16 mt + 4 c + e: one per row for the whole
  // K (applied after the sum over the waves), or (PER_K) one per row and K block, requested with the tile
  u4 wnext[NTW][TPR];
  float snext[NTW][GSUB];
  uint8_t znext[NTW];
  f4 sanext[PER_K ? GSUB : 1][PER_K ? MT : 1];
  i4 zanext[PER_K && ASYM ? MT : 1];
  // 128 - z_a of the accumulator rows: fixed (one zero point per row or tensor) or per K block
  i4 zoff[ASYM ? MT : 1];
  if constexpr (ASYM && !PER_K) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int m = 16 * mt + 4 * c + e;
        zoff[mt][e] = 128 - k.za[(int64_t)(m < M ? m : M - 1) * k.sa_m_stride];
      }
  }
  const int my_block = c / (4 / GSUB);  // K block of the tile this lane column's weights belong to
  auto request = [&](int kt, int buf) {
    const uint32_t ko = (uint32_t)kt * kTileK4;
#pragma unroll
    for (int i = 0; i < NX; ++i)
      if (8 * i < M)
        __builtin_amdgcn_global_load_lds((w8_global_ptr_t)(k.xq + (uint32_t)(xoff[i] + ko)),
                                         (w8_lds_ptr_t)(sx + buf * SLICE + i * 1024), 16, 0, 0);
    // first group of the tile (GSUB == 1: the tile's only one, shared by 2^g_shift tiles)
    int g0 = GSUB == 1 ? (kt >> k.g_shift) : kt * GSUB;
    g0 = g0 < KG ? g0 : KG - 1;
    const uint32_t wo = (uint32_t)kt * (TPR * kTileBytes) + woff;
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
#pragma unroll
      for (int u = 0; u < TPR; ++u)
        wnext[t][u] = __builtin_nontemporal_load((const u4*)(wbase[t] + (uint32_t)(wo + u * kTileBytes)));
#pragma unroll
      for (int g = 0; g < GSUB; ++g) snext[t][g] = sbase[t][(uint32_t)((g0 + g) * kTileN + r)];
      // raw: any use here would wait for the load inside the request
      znext[t] = *(zbase[t] + (uint32_t)((g0 + (GSUB == 1 ? 0 : my_block)) * kTileN + r));
    }
    if constexpr (PER_K) {
#pragma unroll
      for (int g = 0; g < GSUB; ++g)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int m = 16 * mt + 4 * c + e;
            const int64_t kb = GSUB == 1 ? (int64_t)(kt >> k.q_shift) : (int64_t)kt * GSUB + g;
            sanext[g][mt][e] = k.sa[(int64_t)(m < M ? m : M - 1) * k.sa_m_stride + kb * k.sa_k_stride];
            if constexpr (ASYM)
              zanext[mt][e] = k.za[(int64_t)(m < M ? m : M - 1) * k.sa_m_stride + kb * k.sa_k_stride];
          }
    }
  };

  if (wave < KT) request(wave, 0);
#pragma unroll 1
  for (int kt = wave, buf = 0; kt < KT; kt += W, buf ^= 1) {
    u4 wreg[NTW][TPR];
    float sw[NTW][GSUB];
    uint32_t z4[NTW];
    f4 sa[PER_K ? GSUB : 1][PER_K ? MT : 1];
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
#pragma unroll
      for (int u = 0; u < TPR; ++u) wreg[t][u] = wnext[t][u];
#pragma unroll
      for (int g = 0; g < GSUB; ++g) sw[t][g] = NF4 ? snext[t][g] * (1.0f / 127.0f) : snext[t][g];
      z4[t] = (has_z ? (uint32_t)znext[t] : 8u) * 0x01010101u;
    }
    if constexpr (PER_K) {
#pragma unroll
      for (int g = 0; g < GSUB; ++g)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) sa[g][mt] = sanext[g][mt];
      if constexpr (ASYM) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) zoff[mt] = i4{128, 128, 128, 128} - zanext[mt];
      }
    }
    // the compiler does not order LDS reads after the LDS-writing loads: wait for them here
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    if (kt + W < KT) request(kt + W, buf ^ 1);
    __builtin_amdgcn_sched_barrier(0);

    i4 xa[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < 2; ++j) xa[mt][j] = *(const i4*)(sx + buf * SLICE + mt * 2048 + rd[j]);
#pragma unroll
    for (int t = 0; t < NTW; ++t) {
      i4 bq0, bq1;
      if constexpr (WBITS == 8) {
        // offset-binary bytes: flipping the sign bit leaves the two's complement weight
        bq0 = bitcast<i4>(wreg[t][0] ^ u4{0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u});
        bq1 = bitcast<i4>(wreg[t][TPR - 1] ^ u4{0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u});
      } else if constexpr (NF4) {
        bq0 = w8_decode16_nf4(wreg[t][0][0], wreg[t][0][1]);
        bq1 = w8_decode16_nf4(wreg[t][0][2], wreg[t][0][3]);
      } else {
        bq0 = w8_decode16(wreg[t][0][0], wreg[t][0][1], z4[t]);
        bq1 = w8_decode16(wreg[t][0][2], wreg[t][0][3], z4[t]);
      }
      const int cm = ASYM ? w8_column_sums(bq0, bq1) : 0;
#pragma unroll
      for (int g = 0; g < GSUB; ++g) {
        // activation fragments of K block g: the lane columns of the other blocks contribute zeros
        // (masked again for every row-block: holding GSUB masked copies costs more registers than
        // the selects cost time)
        const bool mine = GSUB == 1 || my_block == g;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const i4 xg0 = mine ? xa[mt][0] : i4{0, 0, 0, 0};
          const i4 xg1 = mine ? xa[mt][1] : i4{0, 0, 0, 0};
          i4 qc = __builtin_amdgcn_mfma_i32_16x16x64_i8(xg0, bq0, i4{0, 0, 0, 0}, 0, 0, 0);
          qc = __builtin_amdgcn_mfma_i32_16x16x64_i8(xg1, bq1, qc, 0, 0, 0);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int qv = ASYM ? qc[e] + cm * zoff[ASYM ? mt : 0][e] : qc[e];
            acc[t][mt][e] = w8_accumulate<PER_K>(qv, PER_K ? sa[g][mt][e] : 0.0f, sw[t][g], acc[t][mt][e]);
          }
        }
      }
    }
  }

  // ---- combine the waves' partial sums in wave order, then scale / bias / rounding / store ----
  __syncthreads();  // every wave is done with its activation slices: the region becomes `red`
#pragma unroll
  for (int t = 0; t < NTW; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[((t * MT + mt) * W + wave) * 64 + lane] = acc[t][mt];
  __syncthreads();
  const float* redf = (const float*)red;
  // one thread per output element, consecutive threads on consecutive columns; D[m][n] of a row
  // tile sits in lane n + 16 (m / 4), register m % 4
  for (int idx = threadIdx.x; idx < NTW * MT * 256; idx += blockDim.x) {
    const int col = idx & 15, m16 = (idx >> 4) & 15, tm = idx >> 8;
    const int t = tm / MT, mt = tm - t * MT;
    const int m = 16 * mt + m16;
    const int64_t n = (nt0 + t) * kTileN + col;
    if (m >= M || n >= k.N) continue;
    const int slot = (col + 16 * (m16 >> 2)) * 4 + (m16 & 3);
    float part[8];
#pragma unroll
    for (int w = 0; w < 8; ++w) part[w] = w < W ? redf[(tm * W + w) * 256 + slot] : 0.0f;
    float s = part[0];
#pragma unroll
    for (int w = 1; w < 8; ++w) s = s + part[w];
    if (!PER_K) s = s * k.sa[(int64_t)m * k.sa_m_stride];
    epilogue_store<kRegimeBF16>(k.ep, m, n, s);
  }
}

// Rows the decode form takes: up to 32 for groups of at least 128 (from 33 rows the 64-row tiles of the
// GEMM form are as fast), and for groups of 64 / 32, which the GEMM form does not take, up to 64 / 32
// (four row tiles times four K blocks of activation scales do not fit the registers).
static int decode_w4i8_max_rows(int64_t group_size) { return group_size == 64 ? 64 : 32; }

// K blocks of 128 that are whole weight tiles and a group size of 128 * 2^s (or one group), so that a K
// tile has one scale: 4-bit integer codes (any activation mode), NF4 codes and symmetric 8-bit weights
// (symmetric activation modes).  Groups of 32 / 64: the decode form only.
// Up to 32 rows run on the decode form (woq_decode_w4i8_kernel; M = 32: 14 us), from 33 rows on the
// 64-row tiles of the MFMA GEMM, which with a single row tile still beats the general small-M kernel
// (4096 -> 14336, per-row scales, M = 48 / 64: 34 / 36 us against 157 / 162 us).
bool gemm_w4i8_applies(const Int8Args& a, int64_t block_k, int64_t qbk, bool per_k, bool asym) {
  if (a.debug_block_sums) return false;
  if (a.K % 128 != 0) return false;
  // asymmetric activations: 4-bit integer codes with groups of at least 128
  if (asym && (a.wbits != 4 || a.nf4 || block_k != 128)) return false;
  if (a.wbits == 8) {
    // symmetric 8-bit weights, symmetric activations, one scale per channel or per 128 * 2^s input channels
    if (a.zeros || asym || block_k != 128) return false;
    // two workgroups per CU: from 512 rows on, with one scale per row, the general tiled kernel is level
    // or ahead (4096 -> 11008, M = 2048: 249 us against 260 us here; per (row, K block): 268 against 252)
    if (a.M > 512 && !per_k) return false;
    if (a.group_size > 0 && (a.G % 128 != 0 || ((a.G / 128) & (a.G / 128 - 1)) != 0)) return false;
    if (per_k && (qbk % 128 != 0 || ((qbk / 128) & (qbk / 128 - 1)) != 0)) return false;
    return a.M * a.K < ((int64_t)1 << 31);
  }
  if (a.wbits != 4) return false;
  // NF4 codes: no zero points; above two row tiles the 64 x 128 tiles, which take K blocks of 128 only
  if (a.nf4 && (a.zeros || (a.M > 32 && block_k != 128))) return false;
  if (block_k == 32 || block_k == 64) {
    // groups of 32 / 64 (K blocks inside a tile), activation blocks = groups; above the rows of the decode
    // form: the 64 x 128 tiles, for 4-bit integer codes and symmetric activations
    // (not groups of 32 with per-(row, K block) scales: four sets of activation scales on top of the
    // second set of sums spill, and a reload waits behind the requests of two steps -- 4096 -> 14336,
    // M = 128: 257 us against 62 us with per-row scales; the general kernel keeps that case)
    if (a.M > decode_w4i8_max_rows(a.group_size) && (a.nf4 || asym || (block_k == 32 && per_k))) return false;
    return a.group_size == block_k && (!per_k || qbk == block_k) && a.M * a.K < ((int64_t)1 << 31);
  }
  if (block_k != 128) return false;
  if (a.group_size > 0 && (a.G % 128 != 0 || ((a.G / 128) & (a.G / 128 - 1)) != 0)) return false;
  // activation K blocks of 128 * 2^s as well (they follow the group size, or the K block)
  if (per_k && (qbk % 128 != 0 || ((qbk / 128) & (qbk / 128 - 1)) != 0)) return false;
  return a.M * a.K < ((int64_t)1 << 31);
}

int launch_gemm_w4i8(const Int8Args& a, const uint8_t* xq, int64_t ldq, const float* sa, int64_t sa_m_stride,
                     int64_t sa_k_stride, int64_t qbk, hipStream_t st, const SplitKScratch* scratch,
                     const int32_t* za) {
  constexpr int kLdsAsym = W8_LDS_BYTES + W8_NBUF * W8_BM * (int)sizeof(int32_t);
  static const hipError_t lds_optin[4] = {
      hipFuncSetAttribute(reinterpret_cast<const void*>(&woq_gemm_w4i8_kernel<false, false>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, W8_LDS_BYTES),
      hipFuncSetAttribute(reinterpret_cast<const void*>(&woq_gemm_w4i8_kernel<true, false>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, W8_LDS_BYTES),
      hipFuncSetAttribute(reinterpret_cast<const void*>(&woq_gemm_w4i8_kernel<false, true>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, kLdsAsym),
      hipFuncSetAttribute(reinterpret_cast<const void*>(&woq_gemm_w4i8_kernel<true, true>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, kLdsAsym)};
  for (int i = 0; i < 4; ++i)
    if (lds_optin[i] != hipSuccess)
      return set_error("woq_gemm_w4i8_kernel: LDS opt-in failed: %s", hipGetErrorString(lds_optin[i]));
  static const hipError_t lds_optin_w8[4] = {
      hipFuncSetAttribute(reinterpret_cast<const void*>(&woq_gemm_w4i8_kernel<false, false, 8>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, W8_LDS_BYTES_W8),
      hipFuncSetAttribute(reinterpret_cast<const void*>(&woq_gemm_w4i8_kernel<true, false, 8>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, W8_LDS_BYTES_W8),
      hipFuncSetAttribute(reinterpret_cast<const void*>(&woq_gemm_w4i8_kernel<false, false, 4, true>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, W8_LDS_BYTES),
      hipFuncSetAttribute(reinterpret_cast<const void*>(&woq_gemm_w4i8_kernel<true, false, 4, true>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, W8_LDS_BYTES)};
  for (int i = 0; i < 4; ++i)
    if (lds_optin_w8[i] != hipSuccess)
      return set_error("woq_gemm_w4i8_kernel: LDS opt-in failed: %s", hipGetErrorString(lds_optin_w8[i]));
  static const hipError_t lds_optin_gsub[3] = {
      hipFuncSetAttribute(reinterpret_cast<const void*>(&woq_gemm_w4i8_kernel<false, false, 4, false, 2>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, W8_LDS_BYTES + W8_NBUF * W8_BM * 4),
      hipFuncSetAttribute(reinterpret_cast<const void*>(&woq_gemm_w4i8_kernel<true, false, 4, false, 2>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, W8_LDS_BYTES + W8_NBUF * W8_BM * 4),
      hipFuncSetAttribute(reinterpret_cast<const void*>(&woq_gemm_w4i8_kernel<false, false, 4, false, 4>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, W8_LDS_BYTES + W8_NBUF * 3 * W8_BM * 4)};
  for (int i = 0; i < 3; ++i)
    if (lds_optin_gsub[i] != hipSuccess)
      return set_error("woq_gemm_w4i8_kernel: LDS opt-in failed: %s", hipGetErrorString(lds_optin_gsub[i]));
  const bool asym = za != nullptr;
  W4I8Args k;
  k.xq = xq; k.ldq = ldq; k.sa = sa; k.sa_m_stride = sa_m_stride; k.sa_k_stride = sa_k_stride;
  k.za = za;
  k.q_shift = 0;
  while (sa_k_stride != 0 && ((int64_t)128 << k.q_shift) < qbk) ++k.q_shift;
  k.M = a.M; k.N = a.N; k.NT = a.NT; k.KT = a.KT; k.KG = a.KG;
  k.qweight = a.qweight; k.scales = a.scales; k.zeros = a.zeros;
  k.g_shift = 30;
  if (a.group_size > 0) {
    k.g_shift = 0;
    while (((int64_t)128 << k.g_shift) < a.G) ++k.g_shift;
  }
  k.ep = Epilogue{a.bias, a.fusion, a.other0, a.other1, a.out, a.out_dtype, a.x_dtype, a.N};
  const int64_t ksteps = a.KT / (a.wbits / 4);  // K steps of 128 values
  k.kts = (int)ksteps;
  k.sk_partial = nullptr;
  k.sk_counters = nullptr;
  if (a.M <= decode_w4i8_max_rows(a.group_size)) {
    // decode form; 2 row-blocks per workgroup while that leaves at least 256 workgroups and the
    // registers allow it, else 1
    DecodeW4I8Args d;
    d.k = k;
    const int gsub = a.group_size == 32 ? 4 : a.group_size == 64 ? 2 : 1;
    const int mt = a.M > 32 ? 4 : a.M > 16 ? 2 : 1;
    // (up to four rows: only above 768 row-blocks; below, single row-blocks spread more evenly over the
    // CUs -- M = 1 with its activation quantization, 4096 -> 11008: 8.9 against 10.1 us, 8192 -> 10240: 13.8
    // against 15.3 us; 16 and 32 rows measured the same either way)
    // (17..32 rows: from 258 row-blocks on -- 288..512 row-blocks at M = 32: 10.5-10.9 us against 11.6-12.0 us)
    const int ntw = (gsub * mt <= 2 && a.NT >= (a.M <= 4 ? 769 : a.M > 16 ? 258 : 512) && a.NT % 2 == 0) ? 2 : 1;
    const int slice = mt * 16 * kTileK4;
    int w = 65536 / (2 * slice);  // at most 64 KiB of activation slices
    if (w > 8) w = 8;
    const int64_t rounds = a.KT / (a.wbits / 4);
    d.W = (int)(rounds < w ? rounds : w);
    size_t smem = (size_t)d.W * 2 * slice;
    const size_t red = (size_t)ntw * mt * d.W * 64 * sizeof(f4);
    if (red > smem) smem = red;
    const unsigned dgrid = (unsigned)(a.NT / ntw);
    const bool per_k = sa_k_stride != 0;
#define WOQ_DECODE_W4I8(MTV, NTWV, GS)                                                         \
  do {                                                                                         \
    if (per_k)                                                                                 \
      woq_decode_w4i8_kernel<true, MTV, NTWV, GS, false><<<dgrid, d.W * 64, smem, st>>>(d);    \
    else                                                                                       \
      woq_decode_w4i8_kernel<false, MTV, NTWV, GS, false><<<dgrid, d.W * 64, smem, st>>>(d);   \
  } while (0)
#define WOQ_DECODE_W4I8_NF4(MTV, NTWV, GS)                                                     \
  do {                                                                                         \
    if (per_k)                                                                                 \
      woq_decode_w4i8_kernel<true, MTV, NTWV, GS, true><<<dgrid, d.W * 64, smem, st>>>(d);     \
    else                                                                                       \
      woq_decode_w4i8_kernel<false, MTV, NTWV, GS, true><<<dgrid, d.W * 64, smem, st>>>(d);    \
  } while (0)
    if (asym) {  // 4-bit integer codes, one K block per tile, at most two row tiles (gemm_w4i8_applies)
#define WOQ_DECODE_W4I8_ASYM(MTV, NTWV)                                                                  \
  do {                                                                                                   \
    if (per_k)                                                                                           \
      woq_decode_w4i8_kernel<true, MTV, NTWV, 1, false, 4, true><<<dgrid, d.W * 64, smem, st>>>(d);      \
    else                                                                                                 \
      woq_decode_w4i8_kernel<false, MTV, NTWV, 1, false, 4, true><<<dgrid, d.W * 64, smem, st>>>(d);     \
  } while (0)
      if (mt == 2 && ntw == 2) WOQ_DECODE_W4I8_ASYM(2, 2);
      else if (mt == 2) WOQ_DECODE_W4I8_ASYM(2, 1);
      else if (ntw == 2) WOQ_DECODE_W4I8_ASYM(1, 2);
      else WOQ_DECODE_W4I8_ASYM(1, 1);
#undef WOQ_DECODE_W4I8_ASYM
      return check_launch("woq_decode_w4i8_kernel");
    }
    if (a.wbits == 8) {  // at most two row tiles, one K block per round (gemm_w4i8_applies)
#define WOQ_DECODE_W8I8(MTV, NTWV)                                                                  \
  do {                                                                                              \
    if (per_k)                                                                                      \
      woq_decode_w4i8_kernel<true, MTV, NTWV, 1, false, 8><<<dgrid, d.W * 64, smem, st>>>(d);       \
    else                                                                                            \
      woq_decode_w4i8_kernel<false, MTV, NTWV, 1, false, 8><<<dgrid, d.W * 64, smem, st>>>(d);      \
  } while (0)
      if (mt == 2 && ntw == 2) WOQ_DECODE_W8I8(2, 2);
      else if (mt == 2) WOQ_DECODE_W8I8(2, 1);
      else if (ntw == 2) WOQ_DECODE_W8I8(1, 2);
      else WOQ_DECODE_W8I8(1, 1);
#undef WOQ_DECODE_W8I8
      return check_launch("woq_decode_w4i8_kernel");
    }
    if (a.nf4) {  // at most two row tiles (gemm_w4i8_applies)
      if (mt == 2) {
        if (gsub == 4) WOQ_DECODE_W4I8_NF4(2, 1, 4);
        else if (gsub == 2) WOQ_DECODE_W4I8_NF4(2, 1, 2);
        else if (ntw == 2) WOQ_DECODE_W4I8_NF4(2, 2, 1);
        else WOQ_DECODE_W4I8_NF4(2, 1, 1);
      } else {
        if (gsub == 4) WOQ_DECODE_W4I8_NF4(1, 1, 4);
        else if (gsub == 2 && ntw == 2) WOQ_DECODE_W4I8_NF4(1, 2, 2);
        else if (gsub == 2) WOQ_DECODE_W4I8_NF4(1, 1, 2);
        else if (ntw == 2) WOQ_DECODE_W4I8_NF4(1, 2, 1);
        else WOQ_DECODE_W4I8_NF4(1, 1, 1);
      }
      return check_launch("woq_decode_w4i8_kernel");
    }
    if (gsub == 4) {
      if (mt == 2) WOQ_DECODE_W4I8(2, 1, 4);
      else WOQ_DECODE_W4I8(1, 1, 4);
    } else if (gsub == 2) {
      if (mt == 4) WOQ_DECODE_W4I8(4, 1, 2);
      else if (mt == 2) WOQ_DECODE_W4I8(2, 1, 2);
      else if (ntw == 2) WOQ_DECODE_W4I8(1, 2, 2);
      else WOQ_DECODE_W4I8(1, 1, 2);
    } else {
      if (mt == 2 && ntw == 2) WOQ_DECODE_W4I8(2, 2, 1);
      else if (mt == 2) WOQ_DECODE_W4I8(2, 1, 1);
      else if (ntw == 2) WOQ_DECODE_W4I8(1, 2, 1);
      else WOQ_DECODE_W4I8(1, 1, 1);
    }
#undef WOQ_DECODE_W4I8
#undef WOQ_DECODE_W4I8_NF4
    return check_launch("woq_decode_w4i8_kernel");
  }
  dim3 grid((unsigned)((a.NT * kTileN + W8_BN - 1) / W8_BN), (unsigned)((a.M + W8_BM - 1) / W8_BM));
  // few tiles and a long K: 4 or 2 workgroups per tile while that stays within 256 workgroups, leaves
  // each at least 16 K steps and the caller's scratch suffices
  const int64_t tiles = (int64_t)grid.x * grid.y;
  if (scratch && scratch->partial && scratch->counters && tiles <= kSplitKCounters) {
    for (int s = 4; s >= 2; s -= 2) {
      const int64_t need = (int64_t)s * tiles * W8_BM * W8_BN * (int64_t)sizeof(float);
      const int kts = (int)((ksteps + s - 1) / s);
      if (tiles * s <= 256 && ksteps / s >= 16 && scratch->bytes >= need && (int64_t)(s - 1) * kts < ksteps) {
        grid.z = (unsigned)s;
        k.kts = kts;
        k.sk_partial = scratch->partial;
        k.sk_counters = scratch->counters;
        break;
      }
    }
  }
  if (a.group_size == 64 && sa_k_stride != 0)
    woq_gemm_w4i8_kernel<true, false, 4, false, 2><<<grid, 256, W8_LDS_BYTES + W8_NBUF * W8_BM * 4, st>>>(k);
  else if (a.group_size == 64)
    woq_gemm_w4i8_kernel<false, false, 4, false, 2><<<grid, 256, W8_LDS_BYTES + W8_NBUF * W8_BM * 4, st>>>(k);
  else if (a.group_size == 32 && sa_k_stride != 0)
    return set_error("woq_gemm_w4i8_kernel: groups of 32 with per-(row, K block) scales are not taken here");
  else if (a.group_size == 32)
    woq_gemm_w4i8_kernel<false, false, 4, false, 4><<<grid, 256, W8_LDS_BYTES + W8_NBUF * 3 * W8_BM * 4, st>>>(k);
  else if (a.wbits == 8 && sa_k_stride != 0)
    woq_gemm_w4i8_kernel<true, false, 8><<<grid, 256, W8_LDS_BYTES_W8, st>>>(k);
  else if (a.wbits == 8)
    woq_gemm_w4i8_kernel<false, false, 8><<<grid, 256, W8_LDS_BYTES_W8, st>>>(k);
  else if (a.nf4 && sa_k_stride != 0)
    woq_gemm_w4i8_kernel<true, false, 4, true><<<grid, 256, W8_LDS_BYTES, st>>>(k);
  else if (a.nf4)
    woq_gemm_w4i8_kernel<false, false, 4, true><<<grid, 256, W8_LDS_BYTES, st>>>(k);
  else if (asym && sa_k_stride != 0)
    woq_gemm_w4i8_kernel<true, true><<<grid, 256, kLdsAsym, st>>>(k);
  else if (asym)
    woq_gemm_w4i8_kernel<false, true><<<grid, 256, kLdsAsym, st>>>(k);
  else if (sa_k_stride != 0)
    woq_gemm_w4i8_kernel<true><<<grid, 256, W8_LDS_BYTES, st>>>(k);
  else
    woq_gemm_w4i8_kernel<false><<<grid, 256, W8_LDS_BYTES, st>>>(k);
  return check_launch("woq_gemm_w4i8_kernel");
}

}  // namespace woq

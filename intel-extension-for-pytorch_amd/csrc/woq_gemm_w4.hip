// MFMA GEMM for 4-bit weights and large M (prefill): y[M, N] = x[M, K] * dequant(W)[N, K]^T.
//
// Reference counterpart: DequantGemmTPP (dequantize a [Kb x 32] weight block to a stack
// buffer, then libxsmm BRGEMM) driven by qlinear_woq_affine_impl
// (csrc/cpu/aten/utils/woq.h:1847-1944, 3104-3477).  There the block is re-dequantized for
// every M block of 64 rows; here a wave dequantizes a weight tile once per 128 rows.
//
//   * v_mfma_f32_16x16x32 with A = activations and B = weights, as in the decode kernel: the
//     dequantized registers of one packed dword ARE the B operand, so weights never touch LDS
//     in dequantized form and every weight is dequantized by exactly one wave;
//   * a workgroup is 4 waves, one per SIMD with the whole 512-entry register file; wave w owns NTW
//     weight row-blocks (16 columns each) for all 16 * MT rows of the workgroup, i.e. MT x NTW
//     accumulator tiles.  The shape built is 128 x 448 (MT 8, NTW 7: 224 accumulator registers;
//     14336 / 448 = 32 and 2048 / 128 = 16 give 512 workgroups = two full generations on 256 CUs).
//     One wave hides about two VALU instructions behind each MFMA (measured: 16.4 cycles per MFMA
//     with 0..2 independent VALU instructions in between, +4 cycles for each further one); a
//     dequantized dword costs 17 and feeds MT = 8 MFMAs, so the loop is VALU-issue-bound;
//   * per K step of 128 (one packed tile per row-block) the activations of the rows go from global
//     memory straight into LDS (global_load_lds_dwordx4, no staging registers), double buffered;
//     16-byte chunk p of row m is stored at chunk p ^ (m % 16), which makes the A-fragment reads
//     (16 rows, one chunk) conflict-free without padding.  The packed tiles take the same route
//     into a per-wave LDS stage two steps ahead and are read into registers during the last K
//     sub-step of the step before;
//   * the step is software pipelined over its 4 K sub-steps and NTW row-blocks: while the MT MFMAs
//     of one (sub-step, row-block) run, the VALU dequantizes the dword of the next one;
//   * 8-bit weights (WBITS 8; per-channel or groups of at least 128) run through the same loop: a K
//     step of 128 is then two packed tiles per row-block (a tile is 16 rows x 64 bytes), sub-step j
//     takes dwords 2 (j % 2), 2 (j % 2) + 1 of tile j / 2 -- the K offsets 64 (j / 2) + 16 c + 8 (j % 2)
//     of lane column c -- and the A fragment is read from the matching 16-byte chunk; 20 VALU
//     instructions per B operand (byte -> float, fma, pack) against 17;
//   * MERGED instances (4-bit weights, bf16 compute, when the caller passes the table): the scale and the
//     zero point of a (row, group) come as one dword, bf16 scale << 16 | fp16 (1024 + zero), and the two
//     nibble positions are read as the fp16 numbers 1024 + q and 64 + q, so that one scale serves both:
//     7 instead of 14 parameter requests and 21 instead of 56 vector instructions per K step and wave
//     (M = 2048, 4096 -> 14336: 198 against 202-206 us on the same boxes; same bits out).
#include <algorithm>

#include "woq_common.h"
#include "woq_internal.h"

namespace woq {

constexpr int G4_WAVES = 4;
template <int MT_, int NTW_>
struct G4Shape {
  static constexpr int MT = MT_;                        // 16-row accumulator tiles
  static constexpr int NTW = NTW_;                      // weight row-blocks (16 columns) per wave
  static constexpr int BM = 16 * MT;                    // rows per workgroup
  static constexpr int BN = G4_WAVES * NTW * kTileN;    // columns per workgroup
  static constexpr int XBYTES = BM * kTileK4 * 2;       // one activation buffer
  static constexpr int XLOADS = XBYTES / (G4_WAVES * 1024);  // LDS loads per wave and buffer
  static constexpr int WSTAGE = G4_WAVES * NTW * kTileBytes;  // one weight stage of 4-bit tiles (8-bit: two)
  static constexpr int LDS_BYTES = 2 * XBYTES + 2 * WSTAGE;   // 4-bit weights; lds_bytes() below
  static constexpr int SSTRIDE = NTW * kTileN + 4;      // fp32 row stride of the epilogue staging tile
  // Row-block during whose MFMAs the A fragments of the next K sub-step are read from LDS.  One
  // block ahead of their first use needs a second set of MT fragment registers; with 16 row tiles
  // a block is long enough (256 cycles) to read them in the last block, each into the registers of
  // the fragment whose last MFMA has just been issued.
  static constexpr int XA_SETS = MT >= 16 ? 1 : 2;
  static constexpr int FETCH_T = XA_SETS == 1 ? NTW - 1 : NTW - 2;
};

template <class S, int WBITS>
constexpr int g4_lds_bytes() {
  return 2 * S::XBYTES + 2 * S::WSTAGE * (WBITS / 4);
}

template <int REGIME>
__device__ __forceinline__ f4 g4_mfma(u4 a, u4 b, f4 c) {
  if constexpr (REGIME == kRegimeF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(bitcast<h8>(a), bitcast<h8>(b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(bitcast<b8>(a), bitcast<b8>(b), c, 0, 0, 0);
}

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* global_ptr_t;

// gridDim.z > 1 (small M x N with a long K, where the tiles alone leave most CUs idle): workgroup z
// of a tile takes the K steps [z * kts, (z + 1) * kts), writes its accumulators to scratch memory as they
// lie in the registers, and the workgroup that arrives last at the tile's counter adds the partial
// tiles in z order (its own from the registers) and runs the epilogue.  Nobody waits; the order of
// the sum is fixed.  All scratch accesses are relaxed device-scope atomics, as in the decode kernel.
// Constants of one (row, group) from its merged dword: w = (1024 + q) * s + c = (64 + q) * s + c64, both
// exact in fp32 (an 11-bit integer times an 8-bit significand), so the fma result is the exact product
// (q - z) * s and the one rounding is the conversion to bf16, as with separate scale and zero point.
struct G4ConstsM {
  float s, c, c64;
  __device__ __forceinline__ void set(uint32_t pd) {
    s = bitcast<float>(pd & 0xFFFF0000u);
    const _Float16 h = bitcast<_Float16>((uint16_t)(pd & 0xFFFFu));
    c = -((float)h * s);
    c64 = __builtin_fmaf(960.0f, s, c);
  }
};
__device__ __forceinline__ u4 g4_dequant_m(uint32_t d, const G4Masks& k, uint32_t magic64, const G4ConstsM& q) {
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

template <int REGIME, class S, int WBITS, bool FP8, bool MERGED = false>
__global__ __launch_bounds__(256) void woq_gemm_w4_kernel(const FpArgs f, const int g_shift, float* const sk_partial,
                                                          int* const sk_counters, const int kts) {
  constexpr int TPS = WBITS / 4;  // packed tiles per row-block and K step of 128
  constexpr int G4_MT = S::MT, G4_NTW = S::NTW, G4_BM = S::BM, G4_XBYTES = S::XBYTES, G4_XLOADS = S::XLOADS,
                G4_WSTAGE = S::WSTAGE * TPS, G4_SSTRIDE = S::SSTRIDE;
  // two activation buffers, then two weight stages of 4 waves x NTW tiles x 1 KiB
  extern __shared__ __align__(1024) uint8_t sX[];
  uint8_t* const sW = sX + 2 * G4_XBYTES;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, c = lane >> 4;
  const int M = (int)f.M, K = (int)f.K, NT = (int)f.NT, KG = (int)f.KG;
  const int KTW = (int)f.KT;   // packed tiles along K of a row-block
  // K steps of 128 of this workgroup: [kt_lo, KT); kts is even, so the buffer parity of a step is
  // that of its number whatever the split
  const int kt_lo = (int)blockIdx.z * kts;
  const int KT = KTW / TPS < kt_lo + kts ? KTW / TPS : kt_lo + kts;
  int bx, by;  // this workgroup's tile, by XCD (xcd_tile)
  xcd_tile(bx, by);
  const int m0 = by * G4_BM;
  const int nt0 = (bx * G4_WAVES + wave) * G4_NTW;  // first row-block of this wave

  G4Masks km;
  asm volatile("s_mov_b32 %0, 0x000F000F" : "=s"(km.lo));
  asm volatile("s_mov_b32 %0, 0x00F000F0" : "=s"(km.hi));
  asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(km.magic));
  uint32_t magic64;  // fp16 64 twice: a nibble in place at bits 4..7 reads as 64 + q
  asm volatile("v_mov_b32 %0, 0x54005400" : "=v"(magic64));

  f4 acc[G4_MT][G4_NTW];
#pragma unroll
  for (int mt = 0; mt < G4_MT; ++mt)
#pragma unroll
    for (int t = 0; t < G4_NTW; ++t) acc[mt][t] = f4{0.f, 0.f, 0.f, 0.f};

  // ---- activations: load i of wave w fills LDS KiB number w * XLOADS + i of a buffer: rows
  // 4 (w * XLOADS + i) + lane / 16, physical chunk lane % 16 = logical chunk ^ (row % 16).  Rows
  // past M re-read row M - 1; their results are never stored.
  uint32_t xoff[G4_XLOADS];
#pragma unroll
  for (int i = 0; i < G4_XLOADS; ++i) {
    const int rowl = (wave * G4_XLOADS + i) * 4 + c;
    const int rowc = m0 + rowl < M ? rowl : M - 1 - m0;
    // (4-bit weights: the chunk 4 c + j of lane column c and sub-step j is kept at slot 4 j + c, so that the four
    // lane columns of a row read slots that differ in their low bits: chunks 8 apart share their banks)
    const int slot = r ^ (rowl & 15);
    const int chunk = WBITS == 4 ? ((slot & 3) << 2) | (slot >> 2) : slot;
    xoff[i] = (uint32_t)(rowc * K + chunk * 8) * 2u;
  }
  // All global addresses are a wave-uniform 64-bit base plus a 32-bit per-lane byte offset that
  // carries the K step, which keeps the bases in scalar registers.
  const uint8_t* xbase = (const uint8_t*)f.x + (int64_t)m0 * K * 2;
  auto load_x = [&](int kt, int buf) {
    const uint32_t ko = (uint32_t)kt * (kTileK4 * 2);
#pragma unroll
    for (int i = 0; i < G4_XLOADS; ++i)
      __builtin_amdgcn_global_load_lds((global_ptr_t)(xbase + (uint32_t)(xoff[i] + ko)),
                                       (lds_ptr_t)(sX + buf * G4_XBYTES + (wave * G4_XLOADS + i) * 1024), 16, 0,
                                       0);
  };
  // A fragment of row tile mt, sub-step j: row 16 mt + r, logical chunk 4 c + j (8-bit weights:
  // 8 (j / 2) + 2 c + j % 2, the K offsets of the lane column's bytes in tile j / 2)
  uint32_t rd[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int slot = WBITS == 4 ? j * 4 + c : 8 * (j / 2) + 2 * c + (j % 2);
    rd[j] = (uint32_t)(r * 256 + ((slot ^ r) << 4));
  }

  // ---- weights of one K tile: one dwordx4 + one (scale, zero) per row-block and lane.  Symmetric
  // weights carry no zero points: scale bytes are read (and ignored) instead of branching. ----
  const bool has_z = f.zeros != nullptr;
  const uint8_t* wbase[G4_NTW];
  const uint8_t* sbase[G4_NTW];
  const uint8_t* zbase[G4_NTW];
  const uint8_t* mbase[G4_NTW];
#pragma unroll
  for (int t = 0; t < G4_NTW; ++t) {
    const int nt = nt0 + t < NT ? nt0 + t : NT - 1;
    wbase[t] = f.qweight + (size_t)nt * KTW * kTileBytes;
    sbase[t] = (const uint8_t*)(f.scales + (size_t)nt * KG * kTileN);
    zbase[t] = has_z ? f.zeros + (size_t)nt * KG * kTileN : sbase[t];
    mbase[t] = (const uint8_t*)f.szb + (size_t)nt * KG * (kTileN * 4);
  }
  const uint32_t woff = (uint32_t)lane * 16u;
  auto load_q = [&](int kt, uint16_t (&s)[G4_NTW], uint8_t (&z)[G4_NTW]) {
    int g = (kt * kTileK4 + c * 32) >> g_shift;
    g = g < KG ? g : KG - 1;
    const uint32_t qoff = (uint32_t)(g * kTileN + r);
#pragma unroll
    for (int t = 0; t < G4_NTW; ++t) {
      s[t] = *(const uint16_t*)(sbase[t] + (uint32_t)(qoff * 2u));
      const uint8_t zb = *(zbase[t] + qoff);
      z[t] = has_z ? zb : (uint8_t)(WBITS == 4 ? 8 : 128);  // symmetric: the stored code of zero
    }
  };
  auto load_m = [&](int kt, uint32_t (&p)[G4_NTW]) {
    int g = (kt * kTileK4 + c * 32) >> g_shift;
    g = g < KG ? g : KG - 1;
    const uint32_t qoff = (uint32_t)(g * kTileN + r) * 4u;
#pragma unroll
    for (int t = 0; t < G4_NTW; ++t) p[t] = *(const uint32_t*)(mbase[t] + qoff);
  };
  // The packed tiles of a K step travel global -> LDS -> registers: the LDS stage costs no
  // registers while the load is in flight, which lets the tiles be requested two steps ahead.
  // Each wave fills and reads only its own NTW KiB of a stage.
  uint8_t* const wmine = sW + wave * (G4_NTW * TPS * kTileBytes);
  auto dma_w = [&](int kt, int stage) {
    const uint32_t wo = (uint32_t)kt * (TPS * kTileBytes) + woff;
#pragma unroll
    for (int t = 0; t < G4_NTW; ++t)
#pragma unroll
      for (int u = 0; u < TPS; ++u)
        __builtin_amdgcn_global_load_lds((global_ptr_t)(wbase[t] + (uint32_t)(wo + u * kTileBytes)),
                                         (lds_ptr_t)(wmine + stage * G4_WSTAGE + (t * TPS + u) * kTileBytes), 16, 0,
                                         0);
  };
  auto read_w = [&](int stage, int t, int u) {
    return *(const u4*)(wmine + stage * G4_WSTAGE + (t * TPS + u) * kTileBytes + woff);
  };

  u4 wr[G4_NTW][TPS];
  uint16_t sr[G4_NTW];
  uint8_t zr[G4_NTW];
  G4Consts<REGIME> qc[WBITS == 4 ? G4_NTW : 1];
  G4ConstsM qm[G4_NTW];
  uint32_t mr[G4_NTW];
  float q8s[WBITS == 8 ? G4_NTW : 1], q8c[WBITS == 8 ? G4_NTW : 1];  // 8-bit: scale, -(128 + z) * scale
  auto set_q = [&](int t, uint16_t sbits, float z) {
    if constexpr (MERGED) {
      qm[t].set(mr[t]);
    } else if constexpr (WBITS == 4) {
      qc[t].set(sbits, z);
    } else {
      q8s[t] = REGIME == kRegimeF16 ? f16_bits_to_f32(sbits) : bf16_bits_to_f32(sbits);
      q8c[t] = -(z * q8s[t]);
    }
  };
  // B operand of row-block t, K sub-step j
  auto deq = [&](int t, int j) -> u4 {
    if constexpr (MERGED) {
      return g4_dequant_m(wr[t][0][j], km, magic64, qm[t]);
    } else if constexpr (WBITS == 4) {
      return g4_dequant(wr[t][0][j], km, qc[t]);
    } else {
      const uint32_t d0 = wr[t][j / 2][2 * (j % 2)], d1 = wr[t][j / 2][2 * (j % 2) + 1];
      if constexpr (FP8 && REGIME == kRegimeF16)  // float8 e4m3fn bytes
        return bitcast<u4>(dequant8_f16_fp8(d0, d1, q8s[t]));
      else if constexpr (FP8)
        return bitcast<u4>(dequant8_bf16_fp8(d0, d1, q8s[t]));
      else if constexpr (REGIME == kRegimeF16)
        return bitcast<u4>(dequant8_f16_w8(d0, d1, q8s[t], q8c[t]));
      else
        return bitcast<u4>(dequant8_bf16_w8(d0, d1, q8s[t], q8c[t]));
    }
  };
  u4 bop[2];        // B operand in use / being dequantized
  u4 xa[S::XA_SETS][G4_MT];  // A fragments of the sub-step in use (/ of the next one)

  // s_waitcnt immediates (vmcnt in bits 3:0 and 15:14; expcnt 6:4 and lgkmcnt 11:8 left at maximum)
  constexpr int kVmcnt0 = 0x0F70, kLgkmcnt0 = 0xC07F;
  constexpr int kVmcntW = 0x0F70 | (G4_NTW * TPS);  // all but the last loads (one weight stage) have landed
  // everything older than one whole step of loads (2 NTW parameter loads -- merged: NTW --, XLOADS + NTW * TPS
  // LDS loads)
  constexpr int kStepLoads = ((MERGED ? 1 : 2) + TPS) * G4_NTW + G4_XLOADS;
  static_assert(kStepLoads < 64 && G4_NTW * TPS < 16, "s_waitcnt vmcnt is a 6-bit field");
  constexpr int kVmcntStep = 0x0F70 | (kStepLoads & 15) | ((kStepLoads >> 4) << 14);

  // With one set of fragment registers (16 row tiles) a wave reads the 16 fragments of the next sub-step in one block,
  // and four waves that do so at the same moment queue at the LDS: a ds_read_b128 issued next to vector work costs
  // 10 clocks alone and about 40 when the three other waves issue theirs with it.  The waves therefore meet at the
  // barrier in different blocks of the last sub-step -- wave w in block FETCH_T - w, the same moment for all -- and so
  // reach the fetching block one block apart, in every sub-step (M = 2048, 4096 -> 6144: 92 us against 99 us).
  constexpr int STAG_MAX = S::XA_SETS == 1 ? (S::FETCH_T < 3 ? S::FETCH_T : 3) : 0;
  const int bar_t = S::FETCH_T - (wave < STAG_MAX ? wave : STAG_MAX);
  load_x(kt_lo, 0);
  dma_w(kt_lo, 0);
  dma_w(KT > kt_lo + 1 ? kt_lo + 1 : kt_lo, 1);
  if constexpr (MERGED) load_m(kt_lo, mr); else load_q(kt_lo, sr, zr);
  __builtin_amdgcn_s_waitcnt(kVmcnt0);
  __syncthreads();
#pragma unroll
  for (int t = 0; t < G4_NTW; ++t) {
#pragma unroll
    for (int u = 0; u < TPS; ++u) wr[t][u] = read_w(0, t, u);
    set_q(t, sr[t], (float)zr[t]);
  }
  bop[0] = deq(0, 0);
#pragma unroll
  for (int mt = 0; mt < G4_MT; ++mt) xa[0][mt] = *(const u4*)(sX + mt * 4096 + rd[0]);

  // The accumulator tiles pass through an opaque statement on both sides of the K loop: without it
  // the optimizer splits each loop-carried vector into four scalars (the epilogue reads single
  // elements), and the tiles are then copied between registers in every iteration.
#pragma unroll
  for (int mt = 0; mt < G4_MT; ++mt)
#pragma unroll
    for (int t = 0; t < G4_NTW; ++t) asm volatile("" : "+a"(acc[mt][t]));

  for (int kt = kt_lo; kt < KT; ++kt) {
    const uint8_t* xs = sX + (kt & 1) * G4_XBYTES;
    const uint8_t* xsn = sX + ((kt & 1) ^ 1) * G4_XBYTES;
    // ---- requests, in this order (s_waitcnt vmcnt counts from the youngest): parameters and
    // activations of step kt + 1, then (behind the first MFMA block) the weight tiles of step
    // kt + 2 into the stage that held step kt.  Past the end the last step is requested again. ----
    const int kt1 = kt + 1 < KT ? kt + 1 : KT - 1;
    const int kt2 = kt + 2 < KT ? kt + 2 : KT - 1;
    if constexpr (MERGED) load_m(kt1, mr); else load_q(kt1, sr, zr);
    load_x(kt1, (kt & 1) ^ 1);
    __builtin_amdgcn_sched_barrier(0);

    // 4 NTW blocks of MT MFMAs (one row-block t of one K sub-step j against the MT row tiles); the VALU
    // dequantizes the B operand of the next block meanwhile.  Block FETCH_T of a sub-step also
    // fetches the A fragments of the next sub-step; in the last sub-step these come from the other
    // buffer, so that block starts with the wait for this step's activations and the barrier.  Block t of the last sub-step reads the
    // tile of row-block t for the next step from LDS; its registers were last used one block before.
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int t = 0; t < G4_NTW; ++t) {
        const int cur = (j * G4_NTW + t) & 1;
        const bool last_t = t == G4_NTW - 1;
        const bool fetch_t = t == S::FETCH_T;
        if (j == 0 && t == 1) {
          // the LDS reads of the previous step's last blocks have returned: their stage is free
          __builtin_amdgcn_s_waitcnt(kLgkmcnt0);
          dma_w(kt2, kt & 1);
          __builtin_amdgcn_sched_barrier(0);
        }
        if (j == 3 && t == 0) __builtin_amdgcn_s_waitcnt(kVmcntStep);  // tiles of step kt + 1 are in LDS
        if constexpr (STAG_MAX == 0) {
          if (fetch_t && j == 3) {
            // Written as an instruction, not as the barrier builtin: before that one the compiler
            // waits for every outstanding load, the tiles requested for step kt + 2 included.
            __builtin_amdgcn_s_waitcnt(kVmcntW);
            asm volatile("s_barrier" ::: "memory");
          }
        } else {
          // this wave's meeting block (see bar_t)
          if (j == 3 && t <= S::FETCH_T && t >= S::FETCH_T - STAG_MAX && bar_t == t) {
            __builtin_amdgcn_s_waitcnt(kVmcntW);
            __builtin_amdgcn_s_barrier();
          }
        }
        if (last_t && j == 3) {
#pragma unroll
          for (int u = 0; u < G4_NTW; ++u) set_q(u, sr[u], (float)zr[u]);
          bop[cur ^ 1] = deq(0, 0);
        } else if (last_t) {
          bop[cur ^ 1] = deq(0, j + 1);
        } else {
          bop[cur ^ 1] = deq(t + 1, j);
        }
#pragma unroll
        for (int mt = 0; mt < G4_MT; ++mt) {
          acc[mt][t] = g4_mfma<REGIME>(bop[cur], xa[(j & 1) % S::XA_SETS][mt], acc[mt][t]);
          if (fetch_t)
            xa[((j & 1) ^ 1) % S::XA_SETS][mt] = j == 3 ? *(const u4*)(xsn + mt * 4096 + rd[0])
                                         : *(const u4*)(xs + mt * 4096 + rd[j + 1]);
        }
        if (j == 3) {
#pragma unroll
          for (int u = 0; u < TPS; ++u) wr[t][u] = read_w((kt & 1) ^ 1, t, u);
        }
#pragma unroll
        for (int mt = 0; mt < G4_MT; ++mt) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (fetch_t) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // The requests past the last step are still writing LDS: drain them before the workgroup can end.
  __builtin_amdgcn_s_waitcnt(kVmcnt0);
#pragma unroll
  for (int mt = 0; mt < G4_MT; ++mt)
#pragma unroll
    for (int t = 0; t < G4_NTW; ++t) asm volatile("" : "+a"(acc[mt][t]));

  // (built for the 64 x 128 shape only, the one that is ever launched with gridDim.z > 1: with more
  // accumulator tiles the second copy of them would not fit the registers)
  if constexpr (G4_MT * G4_NTW <= 8) if (gridDim.z > 1) {
    const int nsplit = (int)gridDim.z, z = (int)blockIdx.z;
    const int tiles = (int)(gridDim.x * gridDim.y), tile = (int)(blockIdx.y * gridDim.x + blockIdx.x);
    constexpr int kWaveFloats = G4_MT * G4_NTW * 256;
    float* const mine = sk_partial + ((size_t)(z * tiles + tile) * G4_WAVES + wave) * kWaveFloats + lane * 4;
#pragma unroll
    for (int mt = 0; mt < G4_MT; ++mt)
#pragma unroll
      for (int t = 0; t < G4_NTW; ++t)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          __hip_atomic_store(mine + (mt * G4_NTW + t) * 256 + e, acc[mt][t][e], __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_s_waitcnt(kVmcnt0);  // this thread's stores have completed
    __syncthreads();
    __shared__ int s_last;
    if (tid == 0)
      s_last = __hip_atomic_fetch_add(sk_counters + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == nsplit - 1;
    __syncthreads();
    if (!s_last) return;
    // the other workgroups' partial tiles, one after the other in z order: all loads of one in flight
    // together, then the additions (this workgroup's own tile comes from its registers, in its turn)
    f4 total[G4_MT][G4_NTW];
#pragma unroll 1
    for (int zz = 0; zz < nsplit; ++zz) {
      f4 v[G4_MT][G4_NTW];
      const float* const other = sk_partial + ((size_t)(zz * tiles + tile) * G4_WAVES + wave) * kWaveFloats + lane * 4;
#pragma unroll
      for (int mt = 0; mt < G4_MT; ++mt)
#pragma unroll
        for (int t = 0; t < G4_NTW; ++t) {
          v[mt][t] = acc[mt][t];
          if (zz != z) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              v[mt][t][e] = __hip_atomic_load(other + (mt * G4_NTW + t) * 256 + e, __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
          }
        }
#pragma unroll
      for (int mt = 0; mt < G4_MT; ++mt)
#pragma unroll
        for (int t = 0; t < G4_NTW; ++t) {
          if (zz == 0) {
            total[mt][t] = v[mt][t];
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) total[mt][t][e] = total[mt][t][e] + v[mt][t][e];
          }
        }
    }
#pragma unroll
    for (int mt = 0; mt < G4_MT; ++mt)
#pragma unroll
      for (int t = 0; t < G4_NTW; ++t) acc[mt][t] = total[mt][t];
    // the counter is back at zero for the next launch that uses it
    if (tid == 0) __hip_atomic_store(sk_counters + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  // ---- epilogue.  The weights are the first MFMA operand and the activations the second, so the
  // accumulator tile is D[n][m]: lane (r, c) holds row m = 16 mt + r and the four consecutive columns
  // n = 16 t + 4 c + e.  In the plain case (no post-op, output in the activation dtype) a lane rounds
  // its four values and stores them as 8 bytes straight from the registers: the four lane columns of a
  // row write 32 contiguous bytes, the NTW row-blocks of a wave follow each other in the row, and
  // nothing waits on LDS.  Post-ops go through a per-wave LDS tile (the activation buffers are idle
  // after the last barrier) so that the element-wise tail sees consecutive columns in consecutive lanes. ----
  const int64_t ncol0 = (int64_t)nt0 * kTileN;
  // (the output may be the other 16-bit type than the activations: fp16 rows converted from a bf16 tensor)
  const bool out_f16 = f.out_dtype == WOQ_HIP_ACT_FP16;
  const bool fast = f.fusion == WOQ_HIP_FUSE_NONE && (out_f16 || f.out_dtype == WOQ_HIP_ACT_BF16) && (f.N % 4) == 0 &&
                    (((uintptr_t)f.out & 7) | ((uintptr_t)f.bias & 15)) == 0;
  const bool hb = f.bias != nullptr;
  if (fast) {
    f4 bias4[G4_NTW];
#pragma unroll
    for (int t = 0; t < G4_NTW; ++t)
      bias4[t] = hb && ncol0 + t * kTileN + 4 * c < f.N ? *(const f4*)(f.bias + ncol0 + t * kTileN + 4 * c)
                                                        : f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int mt = 0; mt < G4_MT; ++mt) {
      const int m = m0 + mt * 16 + r;
      if (m < M) {
        uint16_t* const row = (uint16_t*)f.out + (int64_t)m * f.N + ncol0 + 4 * c;
#pragma unroll
        for (int t = 0; t < G4_NTW; ++t) {
          const float y0 = finalize_acc<REGIME>(acc[mt][t][0], hb, bias4[t][0]);
          const float y1 = finalize_acc<REGIME>(acc[mt][t][1], hb, bias4[t][1]);
          const float y2 = finalize_acc<REGIME>(acc[mt][t][2], hb, bias4[t][2]);
          const float y3 = finalize_acc<REGIME>(acc[mt][t][3], hb, bias4[t][3]);
          u2 o;
          if (out_f16) {
            o[0] = (uint32_t)f32_to_f16_bits(y0) | ((uint32_t)f32_to_f16_bits(y1) << 16);
            o[1] = (uint32_t)f32_to_f16_bits(y2) | ((uint32_t)f32_to_f16_bits(y3) << 16);
          } else {
            o[0] = bitcast<uint32_t>(__builtin_convertvector(f2{y0, y1}, b2));
            o[1] = bitcast<uint32_t>(__builtin_convertvector(f2{y2, y3}, b2));
          }
          if (ncol0 + t * kTileN + 4 * c < f.N) *(u2*)(row + t * kTileN) = o;  // (N % 4 == 0: all four or none)
        }
      }
    }
    return;
  }
  float* stage = (float*)sX + wave * (16 * G4_SSTRIDE);
  Epilogue ep{f.bias, f.fusion, f.other0, f.other1, f.out, f.out_dtype, f.x_dtype, f.N};
#pragma unroll
  for (int mt = 0; mt < G4_MT; ++mt) {
#pragma unroll
    for (int t = 0; t < G4_NTW; ++t) *(f4*)(stage + r * G4_SSTRIDE + t * kTileN + 4 * c) = acc[mt][t];
#pragma unroll 1
    for (int it = 0; it < 16 * G4_NTW * kTileN / 64; ++it) {
      const int idx = it * 64 + lane;
      const int row = idx / (G4_NTW * kTileN), col = idx - row * (G4_NTW * kTileN);
      const int m = m0 + mt * 16 + row;
      const int64_t n = ncol0 + col;
      if (m < M && n < f.N) epilogue_store<REGIME>(ep, m, n, stage[row * G4_SSTRIDE + col]);
    }
  }
}

// The kernel needs whole K steps of 128, activations already in the regime's dtype, and a group size
// whose boundaries never split a lane's 32 consecutive K values (8-bit weights: a K step, so groups of
// at least 128 or one scale per channel).  NF4 codes are not taken.
bool gemm_w4_applies(const FpArgs& f, int wbits, int regime) {
  const int want = regime == kRegimeF16 ? WOQ_HIP_ACT_FP16 : WOQ_HIP_ACT_BF16;
  if ((wbits != 4 && wbits != 8) || f.nf4 || f.x_dtype != want || ((uintptr_t)f.x & 15) != 0) return false;
  if (f.K % kTileK4 != 0 || f.K * 256 * 2 >= (int64_t)1 << 31) return false;
  if (f.G >= f.KT * (wbits == 4 ? kTileK4 : kTileK8)) return true;  // per-channel: one group
  return f.G >= (wbits == 4 ? 32 : 128) && (f.G & (f.G - 1)) == 0;
}

template <int REGIME, class S, int WBITS = 4, bool FP8 = false>
static int launch_shape(const FpArgs& f, int g_shift, hipStream_t st, int splits = 1,
                        const SplitKScratch* scratch = nullptr) {
  constexpr int kLds = g4_lds_bytes<S, WBITS>();
  static_assert(kLds <= 160 * 1024, "a workgroup's LDS");
  // more than 64 KiB of LDS per workgroup needs an opt-in (once per kernel and process)
  static const hipError_t lds_optin =
      hipFuncSetAttribute(reinterpret_cast<const void*>(&woq_gemm_w4_kernel<REGIME, S, WBITS, FP8>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
  if (lds_optin != hipSuccess)
    return set_error("woq_gemm_w4_kernel: LDS opt-in failed: %s", hipGetErrorString(lds_optin));
  dim3 grid((unsigned)((f.NT * kTileN + S::BN - 1) / S::BN), (unsigned)((f.M + S::BM - 1) / S::BM),
            (unsigned)splits);
  const int ksteps = (int)(f.KT / (WBITS / 4));
  int kts = ksteps;
  if (splits > 1) {
    if (S::MT * S::NTW > 8) return set_error("woq_gemm_w4_kernel: K is split for the 64 x 128 shape only");
    kts = ((ksteps + splits - 1) / splits + 1) & ~1;  // even, so that every workgroup starts on buffer 0
    const int64_t tiles = (int64_t)grid.x * grid.y;
    const int64_t need = (int64_t)splits * tiles * S::BM * S::BN * (int64_t)sizeof(float);
    if ((int64_t)(splits - 1) * kts >= ksteps)
      return set_error("woq_gemm_w4_kernel: %d K steps are too few for %d splits", ksteps, splits);
    if (!scratch || !scratch->partial || !scratch->counters || scratch->bytes < need || tiles > kSplitKCounters)
      return set_error("woq_gemm_w4_kernel: split K needs %lld bytes of workspace, the counter array and at most %d "
                       "tiles", (long long)need, kSplitKCounters);
  }
  if constexpr (REGIME == kRegimeBF16 && WBITS == 4) {
    if (f.szb) {  // scale and zero point of a (row, group) in one dword
      static const hipError_t lds_optin_m =
          hipFuncSetAttribute(reinterpret_cast<const void*>(&woq_gemm_w4_kernel<REGIME, S, WBITS, FP8, true>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
      if (lds_optin_m != hipSuccess)
        return set_error("woq_gemm_w4_kernel: LDS opt-in failed: %s", hipGetErrorString(lds_optin_m));
      woq_gemm_w4_kernel<REGIME, S, WBITS, FP8, true><<<grid, 256, kLds, st>>>(
          f, g_shift, splits > 1 ? scratch->partial : nullptr, splits > 1 ? scratch->counters : nullptr, kts);
      return check_launch("woq_gemm_w4_kernel");
    }
  }
  woq_gemm_w4_kernel<REGIME, S, WBITS, FP8><<<grid, 256, kLds, st>>>(f, g_shift, splits > 1 ? scratch->partial : nullptr,
                                                                 splits > 1 ? scratch->counters : nullptr, kts);
  return check_launch("woq_gemm_w4_kernel");
}

// Relative time of a shape: generations of 256 workgroups times the length of one K step, which
// is proportional to the row-blocks per wave plus a fixed part (requests, barrier, pipeline fill).
template <class S>
static double shape_cost(const FpArgs& f) {
  const double wgs = (double)((f.NT * kTileN + S::BN - 1) / S::BN) * (double)((f.M + S::BM - 1) / S::BM);
  return (double)(int64_t)((wgs + 255) / 256) * (S::NTW + 1.0);
}

// K splits of the 64 x 128 shape: 4 or 2 workgroups per tile while that stays within 256 workgroups,
// leaves each at least 16 K steps and the caller's scratch suffices (14336 -> 4096, M = 128: 64 tiles).
static int pick_splits(const FpArgs& f, int wbits, int64_t tiles, const SplitKScratch* scratch) {
  if (!scratch || !scratch->partial || !scratch->counters || tiles > kSplitKCounters) return 1;
  const int64_t ksteps = f.KT / (wbits / 4);
  for (int s = 4; s >= 2; s -= 2) {
    const int64_t need = (int64_t)s * tiles * 64 * 128 * (int64_t)sizeof(float);
    if (tiles * s <= 256 && ksteps / s >= 16 && scratch->bytes >= need) return s;
  }
  return 1;
}

// 8-bit weights of one shape: integers or float8 bytes, fp16 or bf16 compute
template <class S>
static int launch8(const FpArgs& f, int regime, int g_shift, hipStream_t st, int splits = 1,
                   const SplitKScratch* scratch = nullptr) {
  if (f.fp8)
    return regime == kRegimeF16 ? launch_shape<kRegimeF16, S, 8, true>(f, g_shift, st, splits, scratch)
                                : launch_shape<kRegimeBF16, S, 8, true>(f, g_shift, st, splits, scratch);
  return regime == kRegimeF16 ? launch_shape<kRegimeF16, S, 8>(f, g_shift, st, splits, scratch)
                              : launch_shape<kRegimeBF16, S, 8>(f, g_shift, st, splits, scratch);
}

// Estimated time of the automatic choice below, in microseconds, for the comparison with the dense kernel
// (gemm_dense_cost): per 4096 input channels a generation of 256 workgroups measured 92 / 58 / 37 us with 7 / 4 / 2
// row-blocks per wave, the 64 x 128 shape 27 us while it fits one generation; the 128 x 128 shape beyond 512
// workgroups (two share a CU) 68 us per 512 and 24-68 us for the rest; 8-bit weights a fifth more.
double gemm_w4_cost(const FpArgs& f, int wbits) {
  auto wgs = [&](int bm, int bn) { return ((f.NT * kTileN + bn - 1) / bn) * ((f.M + bm - 1) / bm); };
  auto gens = [](int64_t w) { return (double)((w + 255) / 256); };
  const int64_t w42 = wgs(64, 128), w2 = wgs(128, 128);
  double c;
  if (w42 <= 256) {
    c = 27.0;
  } else {
    const int64_t rem = w2 % 512;
    const double c2 = w2 <= 512 ? gens(w2) * 37.0 : 68.0 * (double)(w2 / 512) + (rem ? 24.0 + 44.0 * (double)rem / 512.0 : 0.0);
    c = std::min(gens(wgs(128, 256)) * 58.0, c2);
    if (wbits == 4) c = std::min(c, gens(wgs(128, 448)) * 92.0);
  }
  return c * (wbits == 8 ? 1.2 : 1.0) * (double)f.K / 4096.0;
}

int launch_gemm_w4(const FpArgs& f, int wbits, int regime, hipStream_t st, int shape, int splits,
                   const SplitKScratch* scratch) {
  int g_shift = 30;
  if (f.G < f.KT * (wbits == 4 ? kTileK4 : kTileK8)) {
    g_shift = 0;
    while (((int64_t)1 << g_shift) < f.G) ++g_shift;
  }
  // 128 rows x 448, 256 or 128 columns per workgroup: the widest shape does the most work per
  // activation fragment, the narrower ones make enough workgroups to fill the chip when M * N is
  // small (e.g. N = 4096: 10 column blocks of 448 but 16 of 256).
  // 256 rows x 192 columns (MT 16, NTW 3: 192 accumulator registers) dequantizes half as much per
  // MFMA but measured no faster per output (a workgroup takes 95-120 us for K = 4096 against 103 us
  // for the 17 % larger 128 x 448 one); it is chosen only where it tiles the problem into whole
  // generations of 256 workgroups and the others do not (N = 6144, M = 2048: 93 us against 138 us).
  // A 256 x 256 shape would need all 256 accumulator registers; the register allocator then
  // copies accumulators through VGPRs and scratch, it measured slower and is not built.
  using S7 = G4Shape<8, 7>;
  using S4 = G4Shape<8, 4>;
  using S2 = G4Shape<8, 2>;
  using ST = G4Shape<16, 3>;
  using S42 = G4Shape<4, 2>;
  if (wbits == 8) {
    // 8-bit weights: twice the tile bytes per K step, so at most four row-blocks per wave fit the LDS
    // (128 x 256, 128 x 128 and 64 x 128 workgroup tiles), chosen like the 4-bit ones
    if (shape != 0 && shape != 4 && shape != 2 && shape != 42)
      return set_error("woq_gemm_w4_kernel: 8-bit weights take the 128 x 256, 128 x 128 and 64 x 128 shapes");
    const int64_t wgs42 = ((f.NT * kTileN + S42::BN - 1) / S42::BN) * ((f.M + S42::BM - 1) / S42::BM);
    if (shape == 0) shape = wgs42 <= 256 ? 42 : (shape_cost<S4>(f) <= shape_cost<S2>(f) ? 4 : 2);
    if (shape == 42) {
      if (splits == 0) splits = pick_splits(f, 8, wgs42, scratch);
      return launch8<S42>(f, regime, g_shift, st, splits, scratch);
    }
    if (splits > 1) return set_error("woq_gemm_w4_kernel: K is split for the 64 x 128 shape only");
    if (shape == 4)
      return launch8<S4>(f, regime, g_shift, st);
    return launch8<S2>(f, regime, g_shift, st);
  }
  if (shape == 0) {
    // Small M x N: 64 x 128 tiles at four waves per SIMD (79 + 32 registers, 48 KiB of LDS).  While
    // every workgroup has a CU to itself the K loop is one memory round trip per step whatever the
    // tile, and the small tile's steps are the shortest: M = 128, 4096 -> 14336 takes 27.7 us against
    // 37.2 us with 128 x 128 tiles, 14336 -> 4096 80.8 us against 112.5 us.
    const int64_t wgs42 = ((f.NT * kTileN + S42::BN - 1) / S42::BN) * ((f.M + S42::BM - 1) / S42::BM);
    if (wgs42 <= 256) shape = 42;
  }
  if (shape == 42) {
    const int64_t wgs42 = ((f.NT * kTileN + S42::BN - 1) / S42::BN) * ((f.M + S42::BM - 1) / S42::BM);
    if (splits == 0) splits = pick_splits(f, 4, wgs42, scratch);
    return regime == kRegimeF16 ? launch_shape<kRegimeF16, S42>(f, g_shift, st, splits, scratch)
                                : launch_shape<kRegimeBF16, S42>(f, g_shift, st, splits, scratch);
  }
  if (splits > 1) return set_error("woq_gemm_w4_kernel: K is split for the 64 x 128 shape only");
  const double c7 = shape_cost<S7>(f), c4 = shape_cost<S4>(f);
  // 128 x 128 tiles of 4-bit weights: two workgroups share a CU, so beyond two generations the CUs stay
  // evenly loaded (fractional generations), and a generation measured 0.53 of a 128 x 256 one (37 against
  // 70 us at K = 4096).  M = 1024, 4096 -> 11008 (688 workgroups): 101 us against 124 us with 128 x 448
  // tiles (200 workgroups); M = 1024 / 2048, 8192 -> 10240: 180 / 313 us against 207 / 329 us.
  const double wgs2 = (double)((f.NT * kTileN + S2::BN - 1) / S2::BN) * (double)((f.M + S2::BM - 1) / S2::BM);
  const double c2 = wgs2 <= 512 ? shape_cost<S2>(f) : wgs2 / 256.0 * 2.7;
  if (shape == 0) {
    shape = (c7 <= c4 && c7 <= c2) ? 7 : (c4 <= c2 ? 4 : 2);
    const int64_t wgs_t = ((f.NT * kTileN + ST::BN - 1) / ST::BN) * ((f.M + ST::BM - 1) / ST::BM);
    const double ct = (double)(wgs_t / 256) * 7.4;
    if (wgs_t % 256 == 0 && ct < c7 && ct < c4 && ct < c2) shape = 163;
  }
  if (shape == 163)
    return regime == kRegimeF16 ? launch_shape<kRegimeF16, ST>(f, g_shift, st)
                                : launch_shape<kRegimeBF16, ST>(f, g_shift, st);
  if (shape == 7)
    return regime == kRegimeF16 ? launch_shape<kRegimeF16, S7>(f, g_shift, st)
                                : launch_shape<kRegimeBF16, S7>(f, g_shift, st);
  if (shape == 4)
    return regime == kRegimeF16 ? launch_shape<kRegimeF16, S4>(f, g_shift, st)
                                : launch_shape<kRegimeBF16, S4>(f, g_shift, st);
  return regime == kRegimeF16 ? launch_shape<kRegimeF16, S2>(f, g_shift, st)
                              : launch_shape<kRegimeBF16, S2>(f, g_shift, st);
}

}  // namespace woq

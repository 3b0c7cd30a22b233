// MFMA GEMM for 4-bit weights and large M with the dequantized weights shared through LDS:
// y[M, N] = x[M, K] * dequant(W)[N, K]^T on 256 x 224 workgroup tiles, two waves per SIMD.
//
// Reference counterpart: DequantGemmTPP (dequantize a [Kb x 32] weight block to a buffer, then a
// BRGEMM over it) driven by qlinear_woq_affine_impl (csrc/cpu/aten/utils/woq.h:1847-1944,
// 3104-3477): the same two stages, the buffer being a tile in LDS here.
//
//   * a workgroup is 8 waves in a 4 x 2 grid; a wave owns 64 rows x 112 columns = 4 x 7 accumulator
//     tiles of v_mfma_f32_16x16x32 (112 accumulator registers, so two waves fit a SIMD and the
//     vector and LDS instructions of one run under the MFMAs of the other);
//   * per K step of 64 every weight of the workgroup's 224 columns is dequantized once, by one lane:
//     a wave takes the two half tiles (16 rows x 64 K, 512 packed bytes) of two row-blocks, one
//     16-byte piece per lane -> 4 packed dwords -> 4 x 8 values in the compute dtype, written to the
//     LDS tile.  That is 17 vector instructions per 16 MFMAs against 40 when every wave dequantizes
//     the operands of its own 128 rows in registers (woq_gemm_w4.hip);
//   * the activations of the 256 rows go from global memory straight into LDS (global_load_lds);
//     both LDS tiles keep a row's 64 K values as 8 chunks of 16 bytes, chunk q stored at q ^ gs_swz(row): the
//     fragment reads (16 rows x 1 chunk) then touch every 16-byte bank group once, whether the LDS serves 8
//     lanes x 128 bytes or 16 lanes x 256 bytes at a time, and the four lane columns of a row read slots that
//     differ in their low bits (the bank-conflict counter reads zero);
//   * both tiles are double buffered with ONE barrier per K step, after the MFMAs of the first
//     row-block of the second K sub-step: by then a wave has read all its fragments of the step, so
//     behind the barrier the step's buffers are free and are refilled for the step after next
//     (activations requested, weights dequantized during the following blocks), and the fragments
//     of the next step, complete since before the barrier, are read from the other buffers;
//   * a wave holds the 7 weight and 4 activation fragments of both K sub-steps (88 registers) and reads those
//     of the next sub-step during the first blocks of the one in use.
//
// Where it stands (M = 2048, 4096 -> 14336, groups of 128): within a few percent of woq_gemm_w4_kernel (202-215 us
// against 199-207 us on the same boxes), so it is reached through force_kernel only.  Half the vector work per MFMA
// and two waves per SIMD do pay -- without its global requests the loop takes 183 us -- but a 256 x 224 tile
// requests twice the activation bytes per MFMA of a 128 x 448 one, and the issue of those requests, not their
// latency, is what the loop pays for (requests issued and never waited for cost the same 18 us; the eight waves
// pass the barrier together and queue at the address unit, which is why each block behind it issues at most one).
#include "woq_common.h"
#include "woq_internal.h"

namespace woq {

namespace {
constexpr int GS_MT = 4, GS_NTW = 7;          // accumulator tiles of a wave: 16-row tiles x row-blocks
constexpr int GS_NB = 2 * GS_NTW;             // row-blocks (16 columns) of a workgroup
constexpr int GS_BM = 4 * GS_MT * 16, GS_BN = GS_NB * kTileN;
constexpr int GS_KS = 64;                     // K step
constexpr int GS_XBYTES = GS_BM * GS_KS * 2, GS_BBYTES = GS_BN * GS_KS * 2;
constexpr int GS_LDS = 2 * (GS_XBYTES + GS_BBYTES);
constexpr int GS_SSTRIDE = GS_NTW * kTileN + 4;  // fp32 row stride of the epilogue staging tile
static_assert(GS_LDS <= 160 * 1024 && 8 * 16 * GS_SSTRIDE * 4 <= GS_LDS, "a workgroup's LDS");

typedef __attribute__((address_space(3))) void* gs_lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gs_global_ptr_t;

__device__ __forceinline__ int gs_swz(int row) { return swz_row128(row); }

template <int REGIME>
__device__ __forceinline__ f4 gs_mfma(u4 a, u4 b, f4 c) {
  if constexpr (REGIME == kRegimeF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(bitcast<h8>(a), bitcast<h8>(b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(bitcast<b8>(a), bitcast<b8>(b), c, 0, 0, 0);
}
}  // namespace

template <int REGIME>
__global__ __launch_bounds__(512) void woq_gemm_w4s_kernel(const FpArgs f, const int g_shift) {
  extern __shared__ __align__(1024) uint8_t smem[];
  uint8_t* const sX = smem;                  // two activation buffers [256 rows][8 chunks]
  uint8_t* const sB = smem + 2 * GS_XBYTES;  // two weight buffers [224 columns][8 chunks]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, c = lane >> 4;
  const int wr = wave >> 1, wc = wave & 1;  // the wave's 64 rows and 112 columns
  const int M = (int)f.M, K = (int)f.K, NT = (int)f.NT, KG = (int)f.KG;
  const int KS = K / GS_KS;
  const int m0 = blockIdx.y * GS_BM;
  const int nb0 = blockIdx.x * GS_NB;

  G4Masks km;
  asm volatile("s_mov_b32 %0, 0x000F000F" : "=s"(km.lo));
  asm volatile("s_mov_b32 %0, 0x00F000F0" : "=s"(km.hi));
  asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(km.magic));

  f4 acc[GS_MT][GS_NTW];
#pragma unroll
  for (int mt = 0; mt < GS_MT; ++mt)
#pragma unroll
    for (int t = 0; t < GS_NTW; ++t) acc[mt][t] = f4{0.f, 0.f, 0.f, 0.f};

  // ---- activations: load i of wave w fills KiB number 4 w + i of a buffer = rows 8 (4 w + i) + lane / 8,
  // physical chunk lane % 8.  Rows past M re-read row M - 1; their results are never stored.
  uint32_t xoff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int rowl = (wave * 4 + i) * 8 + (lane >> 3);
    const int rowc = m0 + rowl < M ? rowl : M - 1 - m0;
    const int chunk = (lane & 7) ^ gs_swz(rowl);
    xoff[i] = (uint32_t)(rowc * K + chunk * 8) * 2u;
  }
  const uint8_t* const xbase = (const uint8_t*)f.x + (int64_t)m0 * K * 2;
  auto load_x1 = [&](int ks, int buf, int i) {
    const uint32_t ko = (uint32_t)ks * (GS_KS * 2);
    __builtin_amdgcn_global_load_lds((gs_global_ptr_t)(xbase + (uint32_t)(xoff[i] + ko)),
                                     (gs_lds_ptr_t)(sX + buf * GS_XBYTES + (wave * 4 + i) * 1024), 16, 0, 0);
  };
  auto load_x = [&](int ks, int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i) load_x1(ks, buf, i);
  };
  // fragment of K sub-step s: 16 rows (or columns) r, chunk 4 s + c
  uint32_t rd[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) rd[s] = (uint32_t)(r * 128 + (((4 * s + c) ^ gs_swz(r)) << 4));
  const uint8_t* const xfrag = sX + wr * (64 * 128);
  const uint8_t* const wfrag = sB + wc * (GS_NTW * 16 * 128);

  // ---- this lane's share of the dequantization: row r of row-block 2 w + lane / 32 of the workgroup, the
  // 32 K values (lane / 16) % 2 of the step's 64: one 16-byte piece of the packed tile = 4 dwords of 8 values.
  // The eighth wave repeats the work of the seventh (same values to the same addresses).
  const int dw = wave < 7 ? wave : 6;
  const int rbl = 2 * dw + (c >> 1), ch = c & 1;
  const int ntq = nb0 + rbl < NT ? nb0 + rbl : NT - 1;
  const uint8_t* const qbase = f.qweight + (size_t)ntq * (size_t)f.KT * kTileBytes + (r + 16 * ch) * 16;
  const uint16_t* const sbase = f.scales + (size_t)ntq * KG * kTileN + r;
  const bool has_z = f.zeros != nullptr;
  const uint8_t* const zbase = has_z ? f.zeros + (size_t)ntq * KG * kTileN + r : (const uint8_t*)sbase;
  uint32_t wb[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) wb[j] = (uint32_t)((16 * rbl + r) * 128 + (((4 * ch + j) ^ gs_swz(r)) << 4));
  auto load_q = [&](int ks) { return *(const u4*)(qbase + (uint32_t)ks * 512u); };
  auto load_s = [&](int ks, uint16_t& s, uint8_t& z) {
    int g = (ks * GS_KS + 32 * ch) >> g_shift;
    g = g < KG ? g : KG - 1;
    s = sbase[g * kTileN];
    z = zbase[g * kTileN];  // symmetric weights: a scale byte, replaced by the code of zero when the constants are set
  };
  // (the choice between the loaded byte and 8 is made here, a step after the load, so that nothing waits for it)
  G4Consts<REGIME> qc;
  auto set_q = [&](uint16_t s, uint8_t z) { qc.set(s, has_z ? (float)z : 8.0f); };
  auto put = [&](int buf, int j, uint32_t d) {
    *(u4*)(sB + buf * GS_BBYTES + wb[j]) = g4_dequant(d, km, qc);
  };
  auto clampk = [&](int ks) { return ks < KS ? ks : KS - 1; };

  // ---- prologue: steps 0 and 1 into the buffers (dword 3 of step 1 is left to the first block of the loop),
  // the packed piece of step 2 into registers ----
  u4 wq, wqn;
  uint16_t sn;
  uint8_t zn;
  {
    uint16_t s0, s1;
    uint8_t z0, z1;
    const u4 w0 = load_q(0);
    load_s(0, s0, z0);
    load_x(0, 0);
    wq = load_q(clampk(1));
    load_s(clampk(1), s1, z1);
    load_x(clampk(1), 1);
    wqn = load_q(clampk(2));
    load_s(clampk(2), sn, zn);
    set_q(s0, z0);
#pragma unroll
    for (int j = 0; j < 4; ++j) put(0, j, w0[j]);
    set_q(s1, z1);
#pragma unroll
    for (int j = 0; j < 3; ++j) put(1, j, wq[j]);
  }
  __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
  __syncthreads();

  // fragments of both K sub-steps: while one set is in use the other is read
  u4 wf[2][GS_NTW], xa[2][GS_MT];
#pragma unroll
  for (int t = 0; t < GS_NTW; ++t) wf[0][t] = *(const u4*)(wfrag + t * 2048 + rd[0]);
#pragma unroll
  for (int mt = 0; mt < GS_MT; ++mt) xa[0][mt] = *(const u4*)(xfrag + mt * 2048 + rd[0]);

  // (the accumulator tiles pass through an opaque statement on both sides of the K loop, which keeps each a
  // whole vector in the loop)
#pragma unroll
  for (int mt = 0; mt < GS_MT; ++mt)
#pragma unroll
    for (int t = 0; t < GS_NTW; ++t) asm volatile("" : "+v"(acc[mt][t]));

  // A K step is 14 blocks of 4 MFMAs: block b = 7 s + t takes row-block t of K sub-step s against the four row
  // tiles.  Scheduling regions of 8 MFMAs: blocks (0, 1), (2, 3), (4, 5), (6 and the MFMAs of 7), then the
  // barrier, (the rest of 7, 8, 9), (10, 11), (12, 13); in each the MFMAs alternate with the LDS accesses, at most
  // one global request and up to three vector instructions.
  auto region_end = [&]() {
#pragma unroll
    for (int i = 0; i < 2 * GS_MT; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  auto mfmas = [&](const int b) {
    const int s = b / GS_NTW, t = b % GS_NTW;
#pragma unroll
    for (int mt = 0; mt < GS_MT; ++mt) acc[mt][t] = gs_mfma<REGIME>(wf[s][t], xa[s][mt], acc[mt][t]);
    if (b == GS_NTW) region_end();
  };
  // What block b of step ks (buffers cur = ks % 2) does besides its MFMAs.  Sub-step 0 reads the fragments of
  // sub-step 1 from the step's buffers -- all of them before block 6, so that they have returned when the wave
  // reaches the barrier -- and sub-step 1, behind the barrier, those of the next step from the other buffers.
  auto rest = [&](const int ks, const int cur, const int b) {
    const int s = b / GS_NTW, t = b % GS_NTW;
    const int from = s == 0 ? cur : cur ^ 1;
    const uint8_t* const xsrc = xfrag + from * GS_XBYTES;
    const uint8_t* const wsrc = wfrag + from * GS_BBYTES;
    if (t == 0) wf[s ^ 1][0] = *(const u4*)(wsrc + rd[s ^ 1]);
    if (t < GS_NTW - 1) wf[s ^ 1][t + 1] = *(const u4*)(wsrc + (t + 1) * 2048 + rd[s ^ 1]);
    if (t < GS_MT) xa[s ^ 1][t] = *(const u4*)(xsrc + t * 2048 + rd[s ^ 1]);
    // the requests for the coming steps, one block each behind the barrier (all waves of the workgroup pass it
    // together: seven requests each in one burst would queue at the address unit)
    if (b == 8) {
      wqn = load_q(clampk(ks + 3));
      load_s(clampk(ks + 3), sn, zn);
    }
    if (b >= 9 && b <= 12) load_x1(clampk(ks + 2), cur, b - 9);
    // dequantization: dword 3 of the next step in block 0, dwords 0..2 of the step after next behind the barrier
    if (b == 0) put(cur ^ 1, 3, wq[3]);
    if (b == 8) put(cur, 0, wq[0]);
    if (b == 10) put(cur, 1, wq[1]);
    if (b == 12) put(cur, 2, wq[2]);
    if (b % 2 == 1 && b != GS_NTW) region_end();
  };
  // Behind the MFMAs of block 7: every fragment of step ks has been read and has returned, the activations of step
  // ks + 1 have landed.  Behind the barrier the buffers of step ks are refilled for step ks + 2.
  auto sync = [&]() {
    __builtin_amdgcn_s_waitcnt(0x0070);
    __builtin_amdgcn_s_barrier();
    // the packed piece requested one step ago moves on, as instructions, so that this is where the wait for it
    // stands, and its registers take the request for the step after
#pragma unroll
    for (int i = 0; i < 4; ++i) asm volatile("v_mov_b32 %0, %1" : "=v"(wq[i]) : "v"(wqn[i]));
    set_q(sn, zn);
    __builtin_amdgcn_sched_barrier(0);
  };

  // The loop turns at the barrier, where the wave has nothing in flight anyway: blocks 0..7 of step 0 first, then
  // per turn the second half of a step and the first half of the next, at last the second half of the last step,
  // whose fragments are in registers.
#pragma unroll
  for (int b = 0; b < GS_NTW; ++b) {
    mfmas(b);
    rest(0, 0, b);
  }
  mfmas(GS_NTW);
  for (int ks = 0; ks < KS - 1; ++ks) {
    const int cur = ks & 1;
    sync();
    rest(ks, cur, GS_NTW);
#pragma unroll
    for (int b = GS_NTW + 1; b < 2 * GS_NTW; ++b) {
      mfmas(b);
      rest(ks, cur, b);
    }
#pragma unroll
    for (int b = 0; b < GS_NTW; ++b) {
      mfmas(b);
      rest(ks + 1, cur ^ 1, b);
    }
    mfmas(GS_NTW);
  }
#pragma unroll
  for (int b = GS_NTW + 1; b < 2 * GS_NTW; ++b) mfmas(b);

  // the requests past the last step are still writing LDS: drain them before the buffers are reused or the
  // workgroup ends
  __builtin_amdgcn_s_waitcnt(0x0070);
  __syncthreads();
#pragma unroll
  for (int mt = 0; mt < GS_MT; ++mt)
#pragma unroll
    for (int t = 0; t < GS_NTW; ++t) asm volatile("" : "+v"(acc[mt][t]));

  // ---- epilogue.  The weights are the first MFMA operand and the activations the second, so the accumulator
  // tile is D[n][m]: lane (r, c) holds row m = 16 mt + r and the four consecutive columns n = 16 t + 4 c + e. ----
  const int nt0 = nb0 + wc * GS_NTW;
  const int mw = m0 + wr * 64;
  const int64_t ncol0 = (int64_t)nt0 * kTileN;
  const bool out_f16 = f.out_dtype == WOQ_HIP_ACT_FP16;
  const bool fast = f.fusion == WOQ_HIP_FUSE_NONE && (out_f16 || f.out_dtype == WOQ_HIP_ACT_BF16) && (f.N % 4) == 0 &&
                    ncol0 + GS_NTW * kTileN <= f.N && (((uintptr_t)f.out & 7) | ((uintptr_t)f.bias & 15)) == 0;
  const bool hb = f.bias != nullptr;
  if (fast) {
    f4 bias4[GS_NTW];
#pragma unroll
    for (int t = 0; t < GS_NTW; ++t)
      bias4[t] = hb ? *(const f4*)(f.bias + ncol0 + t * kTileN + 4 * c) : f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int mt = 0; mt < GS_MT; ++mt) {
      const int m = mw + mt * 16 + r;
      if (m < M) {
        uint16_t* const row = (uint16_t*)f.out + (int64_t)m * f.N + ncol0 + 4 * c;
#pragma unroll
        for (int t = 0; t < GS_NTW; ++t) {
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
          *(u2*)(row + t * kTileN) = o;
        }
      }
    }
    return;
  }
  // post-ops go through a per-wave LDS tile (the buffers are idle: every wave's last requests have landed) so
  // that the element-wise tail sees consecutive columns in consecutive lanes
  float* const stage = (float*)smem + wave * (16 * GS_SSTRIDE);
  Epilogue ep{f.bias, f.fusion, f.other0, f.other1, f.out, f.out_dtype, f.x_dtype, f.N};
#pragma unroll
  for (int mt = 0; mt < GS_MT; ++mt) {
#pragma unroll
    for (int t = 0; t < GS_NTW; ++t) *(f4*)(stage + r * GS_SSTRIDE + t * kTileN + 4 * c) = acc[mt][t];
#pragma unroll 1
    for (int it = 0; it < 16 * GS_NTW * kTileN / 64; ++it) {
      const int idx = it * 64 + lane;
      const int row = idx / (GS_NTW * kTileN), col = idx - row * (GS_NTW * kTileN);
      const int m = mw + mt * 16 + row;
      const int64_t n = ncol0 + col;
      if (m < M && n < f.N) epilogue_store<REGIME>(ep, m, n, stage[row * GS_SSTRIDE + col]);
    }
  }
}

// What the register-resident prefill kernel takes, 4-bit integer weights only.
bool gemm_w4s_applies(const FpArgs& f, int wbits, int regime) { return wbits == 4 && gemm_w4_applies(f, wbits, regime); }

template <int REGIME>
static int launch_w4s(const FpArgs& f, int g_shift, hipStream_t st) {
  static const hipError_t lds_optin = hipFuncSetAttribute(reinterpret_cast<const void*>(&woq_gemm_w4s_kernel<REGIME>),
                                                          hipFuncAttributeMaxDynamicSharedMemorySize, GS_LDS);
  if (lds_optin != hipSuccess)
    return set_error("woq_gemm_w4s_kernel: LDS opt-in failed: %s", hipGetErrorString(lds_optin));
  dim3 grid((unsigned)((f.NT + GS_NB - 1) / GS_NB), (unsigned)((f.M + GS_BM - 1) / GS_BM));
  woq_gemm_w4s_kernel<REGIME><<<grid, 512, GS_LDS, st>>>(f, g_shift);
  return check_launch("woq_gemm_w4s_kernel");
}

int launch_gemm_w4s(const FpArgs& f, int regime, hipStream_t st) {
  int g_shift = 30;
  if (f.G < f.KT * kTileK4) {
    g_shift = 0;
    while (((int64_t)1 << g_shift) < f.G) ++g_shift;
  }
  return regime == kRegimeF16 ? launch_w4s<kRegimeF16>(f, g_shift, st) : launch_w4s<kRegimeBF16>(f, g_shift, st);
}

}  // namespace woq

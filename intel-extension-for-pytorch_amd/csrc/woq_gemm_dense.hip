// MFMA GEMM on the dense bf16 copy of a weight (large batches with cache_weight_for_large_batch):
// y[M, N] = x[M, K] * W[N, K]^T, W already dequantized to bf16 and laid out as MFMA operands.
//
// Reference counterpart: the cached-weight branch of the weight-only linear
// (csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:430-486 builds the copy, :511-526 runs a dense bf16 GEMM on it
// for at least IPEX_WOQ_WEIGHT_CACHE_BATCH_THRESHOLD rows).  There the copy is blocked for the CPU GEMM; here it is
// the operand stream of woq_gemm_w4_kernel with the dequantization already done (dense_weight_kernel writes it):
//
//   * same workgroup as woq_gemm_w4_kernel -- 4 waves, one per SIMD, wave w owns NTW weight row-blocks for all
//     16 MT rows; the activations travel global -> LDS (two to four buffers, swizzled) -> A fragments exactly as
//     there, and the MFMAs see the same operands in the same order, so the results are bit-identical to the
//     kernel that dequantizes on the fly;
//   * a weight fragment (16 rows x 8 K values per lane = 1 KiB per wave) is private to its wave, so it goes from
//     global memory straight into the registers that feed the MFMA: one global_load_dwordx4 per MT MFMAs and
//     nothing else -- no LDS stage, no vector ALU work.  The 4 NTW fragments of a K step form a ring: the
//     registers of the block just finished are refilled for the next step, which leaves a whole K step (about
//     1.8 us) for the load to arrive;
//   * the refills are written as instructions with their own s_waitcnt: the compiler's wait counting would
//     drain every outstanding load at the loop's back edge, the manual counts wait for exactly the fragment
//     that the next block needs (loads return in order: 4 NTW - 1 refills and the XLOADS activation loads of a
//     step are younger than it).
//
// M = 2048, 4096 -> 14336: 166-176 us with one weight copy (cache-resident between launches) and 185-194 us when every
// launch reads a fresh 117 MB copy from HBM, where woq_gemm_w4_kernel takes 192-205 and 204-215 us.  Stand-alone builds
// with one part removed at a time (from HBM, 185 us): the MFMAs with barrier and epilogue alone 134 us, the A fragments
// from LDS 9 us, the weight loads 18 us when they hit in L2 and 12 us more from HBM (the dense copy is four times the
// packed bytes), the activation loads 9 + 2 us.
// A lone, partly filled generation of the narrow shapes is bound by what one CU can pull in (64 KiB per K step of the
// narrowest shape, about 70 GB/s per CU): 4096 input channels take 30 us on 128-column tiles with the activations
// three steps ahead (35 us one step ahead) where the MFMAs need 14 us, and a deeper fragment ring in registers on
// top of that changes nothing; woq_gemm_w4_kernel moves a quarter of the weight bytes and takes 24-28 us there, so
// the copy pays from about 256 rows up, not below.
//
// The inline loads write their registers when the data arrives, not where the instruction stands: a load whose value
// the program never reads would leave its registers free for the compiler to reuse while it is still in flight.
// Every load here is therefore followed, on every path, by a wait that is tied to its registers.
#include <algorithm>

#include "woq_common.h"
#include "woq_internal.h"

namespace woq {

namespace {

constexpr int GD_WAVES = 4;
template <int MT_, int NTW_>
struct GdShape {
  static constexpr int MT = MT_;
  static constexpr int NTW = NTW_;
  static constexpr int BM = 16 * MT;
  static constexpr int BN = GD_WAVES * NTW * kTileN;
  static constexpr int XBYTES = BM * 128 * 2;                 // one activation buffer: BM rows x 128 K values
  static constexpr int XLOADS = XBYTES / (GD_WAVES * 1024);   // LDS loads per wave and buffer
  static constexpr int SSTRIDE = NTW * kTileN + 4;            // fp32 row stride of the epilogue staging tile
  static constexpr int FETCH_T = NTW >= 2 ? NTW - 2 : 0;      // block that reads the next sub-step's A fragments
  static constexpr int NBLK = 4 * NTW;                        // blocks (row-block x K sub-step) of a K step
};

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* global_ptr_t;

struct GdArgs {
  FpArgs f;
  const uint8_t* dense;  // [K / 128][NT][4][64][16 bytes]
  int kmap8;             // the copy was made from 8-bit weights: their assignment of K values to lanes
};

// One weight fragment: 16 bytes per lane at base + off (+ 1 KiB per K sub-step j).
template <int J>
__device__ __forceinline__ u4 gd_load_b(const uint8_t* base, uint32_t off) {
  u4 v;
  if constexpr (J == 0) asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(v) : "v"(off), "s"(base) : "memory");
  if constexpr (J == 1)
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:1024" : "=v"(v) : "v"(off), "s"(base) : "memory");
  if constexpr (J == 2)
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:2048" : "=v"(v) : "v"(off), "s"(base) : "memory");
  if constexpr (J == 3)
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:3072" : "=v"(v) : "v"(off), "s"(base) : "memory");
  return v;
}

// XD: how many K steps ahead the activations are requested (XD + 1 buffers in LDS).  Because loads return in order,
// the barrier's wait for the activations of the next step also retires every fragment requested before them: XD
// bounds how long any load may take.  One step of the widest shape (28 blocks of 8 MFMAs) is long enough; one of the
// narrowest (8 blocks) is not, and when its workgroups are too few for two to share a CU (which hides the same
// latency with half the LDS each) it runs with XD = 3.
template <class S, int XD>
__global__ __launch_bounds__(256) void woq_gemm_dense_kernel(const GdArgs a) {
  constexpr int MT = S::MT, NTW = S::NTW, BM = S::BM, XBYTES = S::XBYTES, XLOADS = S::XLOADS, NBLK = S::NBLK,
                SSTRIDE = S::SSTRIDE;
  constexpr int kRegime = kRegimeBF16;
  extern __shared__ __align__(1024) uint8_t sX[];
  const FpArgs& f = a.f;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, c = lane >> 4;
  const int M = (int)f.M, K = (int)f.K, NT = (int)f.NT;
  const int KT = K / 128;
  int bx, by;
  xcd_tile(bx, by);
  const int m0 = by * BM;
  const int nt0 = (bx * GD_WAVES + wave) * NTW;
  const bool k8 = a.kmap8 != 0;

  f4 acc[MT][NTW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NTW; ++t) acc[mt][t] = f4{0.f, 0.f, 0.f, 0.f};

  // ---- activations, as in woq_gemm_w4_kernel: load i of wave w fills LDS KiB number w * XLOADS + i of a buffer
  // (rows 4 (w * XLOADS + i) + lane / 16), 16-byte chunk of K values kept at physical slot = logical slot ^ (row % 16);
  // the logical slot of chunk 4 c + j is 4 j + c for 4-bit weights and the chunk itself for bytes.  Rows past M
  // re-read row M - 1; their results are never stored.
  uint32_t xoff[XLOADS];
#pragma unroll
  for (int i = 0; i < XLOADS; ++i) {
    const int rowl = (wave * XLOADS + i) * 4 + c;
    const int rowc = m0 + rowl < M ? rowl : M - 1 - m0;
    const int slot = r ^ (rowl & 15);
    const int chunk = k8 ? slot : ((slot & 3) << 2) | (slot >> 2);
    xoff[i] = (uint32_t)(rowc * K + chunk * 8) * 2u;
  }
  const uint8_t* xbase = (const uint8_t*)f.x + (int64_t)m0 * K * 2;
  auto load_x = [&](int kt, int buf) {
    const uint32_t ko = (uint32_t)kt * 256u;
#pragma unroll
    for (int i = 0; i < XLOADS; ++i)
      __builtin_amdgcn_global_load_lds((global_ptr_t)(xbase + (uint32_t)(xoff[i] + ko)),
                                       (lds_ptr_t)(sX + buf * XBYTES + (wave * XLOADS + i) * 1024), 16, 0, 0);
  };
  uint32_t rd[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int slot = k8 ? 8 * (j / 2) + 2 * c + (j % 2) : j * 4 + c;
    rd[j] = (uint32_t)(r * 256 + ((slot ^ r) << 4));
  }

  // ---- weight fragments: wave-uniform base per row-block, per-lane offset that carries the K step
  const uint8_t* bbase[NTW];
#pragma unroll
  for (int t = 0; t < NTW; ++t) {
    const int nt = nt0 + t < NT ? nt0 + t : NT - 1;
    bbase[t] = a.dense + (size_t)nt * 4096;
  }
  const uint32_t boff = (uint32_t)lane * 16u;
  const uint32_t kstride = (uint32_t)NT * 4096u;

  u4 bf[4][NTW];
  u4 xa[2][MT];
  constexpr int kVmcnt0 = 0x0F70;
  // barrier block: the activation loads of the next step (issued at the top of step kt + 1 - XD) have landed when at
  // most the loads issued since are outstanding (XD - 1 whole steps' and this step's refills so far); two fewer than
  // were issued, for slack
  constexpr int NXB = XD + 1;
  constexpr int BARB = (XD - 1) * (NBLK + XLOADS) + 3 * NTW + S::FETCH_T;
  constexpr int NBAR = BARB >= 2 ? BARB - 2 : 0;
  static_assert(NBAR < 64, "s_waitcnt vmcnt is a 6-bit field");
  constexpr int kVmcntBar = 0x0F70 | (NBAR & 15) | ((NBAR >> 4) << 14);
  static_assert(NBLK - 1 + XLOADS < 64, "s_waitcnt vmcnt is a 6-bit field");

  // Prologue: the activations of the first XD steps, then the fragments of step 0 in the order the blocks use them -- all but
  // the last block's, which block 0 of the loop requests like in every later step (a load whose value nothing reads
  // would leave its registers free for other uses while it is still in flight).  Only the activations are waited
  // for here; the loop's per-block waits cover the fragments (the loads behind fragment b -- the rest of the
  // prologue, the activations requested at the top of step 0, the refills up to block b -- are as many as in a later
  // step), so the first MFMAs start when the first fragments are there, not the last.
#pragma unroll
  for (int st = 0; st < XD; ++st) load_x(st < KT ? st : KT - 1, st);
#pragma unroll
  for (int t = 0; t < NTW; ++t) bf[0][t] = gd_load_b<0>(bbase[t], boff);
#pragma unroll
  for (int t = 0; t < NTW; ++t) bf[1][t] = gd_load_b<1>(bbase[t], boff);
#pragma unroll
  for (int t = 0; t < NTW; ++t) bf[2][t] = gd_load_b<2>(bbase[t], boff);
#pragma unroll
  for (int t = 0; t + 1 < NTW; ++t) bf[3][t] = gd_load_b<3>(bbase[t], boff);
  {
    constexpr int kVmcntX = 0x0F70 | ((NBLK - 1) & 15) | (((NBLK - 1) >> 4) << 14);  // all but the fragment loads
    __builtin_amdgcn_s_waitcnt(kVmcntX);
    asm volatile("s_barrier" ::: "memory");
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) xa[0][mt] = *(const u4*)(sX + mt * 4096 + rd[0]);
  // (the accumulators pass through an opaque statement on both sides of the loop so that they stay whole vectors)
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NTW; ++t) asm volatile("" : "+a"(acc[mt][t]));

  int xb = 0;  // the activation buffer of step kt: kt % NXB
  for (int kt = 0; kt < KT; ++kt) {
    const int xbn = xb + 1 == NXB ? 0 : xb + 1, xbp = xb == 0 ? NXB - 1 : xb - 1;
    const uint8_t* xs = sX + xb * XBYTES;
    const uint8_t* xsn = sX + xbn * XBYTES;
    const int kt1 = kt + 1 < KT ? kt + 1 : KT - 1;  // past the end the last step is requested again
    // step kt + XD goes into the buffer of step kt - 1, which every wave has left (that step's barrier stands behind
    // its last read of it)
    load_x(kt + XD < KT ? kt + XD : KT - 1, xbp);
    xb = xbn;
    const uint32_t bko0 = boff + (uint32_t)kt * kstride;
    const uint32_t bko1 = boff + (uint32_t)kt1 * kstride;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int t = 0; t < NTW; ++t) {
        constexpr int kLastJ = 3, kLastT = NTW - 1;
        const bool fetch_t = t == S::FETCH_T;
        if (fetch_t && j == 3) {
          __builtin_amdgcn_s_waitcnt(kVmcntBar);
          asm volatile("s_barrier" ::: "memory");
        }
        // refill the registers of the block just finished with its fragment of the next step (block 0: the last
        // block's fragment of this step, whose registers the previous step has just left)
        if (j == 0 && t == 0) bf[kLastJ][kLastT] = gd_load_b<3>(bbase[kLastT], bko0);
        else if (t == 0) {
          if (j == 1) bf[0][kLastT] = gd_load_b<0>(bbase[kLastT], bko1);
          if (j == 2) bf[1][kLastT] = gd_load_b<1>(bbase[kLastT], bko1);
          if (j == 3) bf[2][kLastT] = gd_load_b<2>(bbase[kLastT], bko1);
        } else {
          if (j == 0) bf[0][t - 1] = gd_load_b<0>(bbase[t - 1], bko1);
          if (j == 1) bf[1][t - 1] = gd_load_b<1>(bbase[t - 1], bko1);
          if (j == 2) bf[2][t - 1] = gd_load_b<2>(bbase[t - 1], bko1);
          if (j == 3) bf[3][t - 1] = gd_load_b<3>(bbase[t - 1], bko1);
        }
        // this block's fragment has arrived: everything but the loads issued after it
        if (j == kLastJ && t == kLastT) asm volatile("s_waitcnt vmcnt(%1)" : "+v"(bf[j][t]) : "n"(NBLK - 1));
        else asm volatile("s_waitcnt vmcnt(%1)" : "+v"(bf[j][t]) : "n"(NBLK - 1 + XLOADS));
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bitcast<b8>(bf[j][t]), bitcast<b8>(xa[j & 1][mt]),
                                                               acc[mt][t], 0, 0, 0);
          if (fetch_t)
            xa[(j & 1) ^ 1][mt] = j == 3 ? *(const u4*)(xsn + mt * 4096 + rd[0]) : *(const u4*)(xs + mt * 4096 + rd[j + 1]);
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (fetch_t) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  // the requests past the last step are still in flight: drain them before the registers and LDS are reused
  __builtin_amdgcn_s_waitcnt(kVmcnt0);
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int t = 0; t < NTW; ++t) asm volatile("" : "+v"(bf[j][t]));
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NTW; ++t) asm volatile("" : "+a"(acc[mt][t]));

  // ---- epilogue, as in woq_gemm_w4_kernel: lane (r, c) holds row 16 mt + r and columns 16 t + 4 c + e
  const int64_t ncol0 = (int64_t)nt0 * kTileN;
  const bool out_f16 = f.out_dtype == WOQ_HIP_ACT_FP16;
  const bool fast = f.fusion == WOQ_HIP_FUSE_NONE && (out_f16 || f.out_dtype == WOQ_HIP_ACT_BF16) && (f.N % 4) == 0 &&
                    (((uintptr_t)f.out & 7) | ((uintptr_t)f.bias & 15)) == 0;
  const bool hb = f.bias != nullptr;
  if (fast) {
    f4 bias4[NTW];
#pragma unroll
    for (int t = 0; t < NTW; ++t)
      bias4[t] = hb && ncol0 + t * kTileN + 4 * c < f.N ? *(const f4*)(f.bias + ncol0 + t * kTileN + 4 * c)
                                                        : f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = m0 + mt * 16 + r;
      if (m < M) {
        uint16_t* const row = (uint16_t*)f.out + (int64_t)m * f.N + ncol0 + 4 * c;
#pragma unroll
        for (int t = 0; t < NTW; ++t) {
          const float y0 = finalize_acc<kRegime>(acc[mt][t][0], hb, bias4[t][0]);
          const float y1 = finalize_acc<kRegime>(acc[mt][t][1], hb, bias4[t][1]);
          const float y2 = finalize_acc<kRegime>(acc[mt][t][2], hb, bias4[t][2]);
          const float y3 = finalize_acc<kRegime>(acc[mt][t][3], hb, bias4[t][3]);
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
  // (staging tiles in the activation buffers: behind the last barrier the waves only repeat reads whose values
  // nothing uses)
  float* stage = (float*)sX + wave * (16 * SSTRIDE);
  Epilogue ep{f.bias, f.fusion, f.other0, f.other1, f.out, f.out_dtype, f.x_dtype, f.N};
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int t = 0; t < NTW; ++t) *(f4*)(stage + r * SSTRIDE + t * kTileN + 4 * c) = acc[mt][t];
#pragma unroll 1
    for (int it = 0; it < 16 * NTW * kTileN / 64; ++it) {
      const int idx = it * 64 + lane;
      const int row = idx / (NTW * kTileN), col = idx - row * (NTW * kTileN);
      const int m = m0 + mt * 16 + row;
      const int64_t n = ncol0 + col;
      if (m < M && n < f.N) epilogue_store<kRegime>(ep, m, n, stage[row * SSTRIDE + col]);
    }
  }
}

template <class S, int XD>
int launch_dense_shape_xd(const GdArgs& a, dim3 grid, hipStream_t st) {
  constexpr int LDS_BYTES = (XD + 1) * S::XBYTES;
  static_assert(LDS_BYTES <= 160 * 1024 && GD_WAVES * 16 * S::SSTRIDE * 4 <= LDS_BYTES, "a workgroup's LDS");
  static const hipError_t lds_optin =
      hipFuncSetAttribute(reinterpret_cast<const void*>(&woq_gemm_dense_kernel<S, XD>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
  if (lds_optin != hipSuccess)
    return set_error("woq_gemm_dense_kernel: LDS opt-in failed: %s", hipGetErrorString(lds_optin));
  woq_gemm_dense_kernel<S, XD><<<grid, 256, LDS_BYTES, st>>>(a);
  return check_launch("woq_gemm_dense_kernel");
}

template <class S>
int launch_dense_shape(const GdArgs& a, hipStream_t st) {
  dim3 grid((unsigned)((a.f.NT * kTileN + S::BN - 1) / S::BN), (unsigned)((a.f.M + S::BM - 1) / S::BM));
  // the narrowest shape with one workgroup per CU at most (256 CUs): deeper prefetch instead of a second workgroup
  if constexpr (S::NTW <= 2) {
    if ((int64_t)grid.x * grid.y <= 256) return launch_dense_shape_xd<S, 3>(a, grid, st);
  }
  return launch_dense_shape_xd<S, 1>(a, grid, st);
}

// Estimated time of a shape, in microseconds per 4096 input channels, from measurements: a full generation of 256
// workgroups takes 88 / 54 / 40 us with 7 / 4 / 2 row-blocks per wave; a partial one, alone or behind full ones, is bound
// by the latency of its weight loads rather than by the chip and takes 66 / 43 / 34 us when nearly empty, rising
// (with the square of its fill) to the full figure (so the narrow shapes are far from proportional, and two workgroups past a generation
// cost almost a whole one).  The narrowest shape alone on the chip (256 workgroups at most, deeper prefetch) takes
// 29.5 us nearly empty and 34.5 us full.
template <class S>
double dense_shape_cost(const FpArgs& f) {
  const int64_t wgs = ((f.NT * kTileN + S::BN - 1) / S::BN) * ((f.M + S::BM - 1) / S::BM);
  const double t_full = S::NTW == 7 ? 88.0 : S::NTW == 4 ? 54.0 : 40.0;
  const double t_low = S::NTW == 7 ? 66.0 : S::NTW == 4 ? 43.0 : 34.0;
  const int64_t full = wgs / 256, rem = wgs % 256;
  const double fill = (double)rem / 256.0;
  if (S::NTW <= 2 && wgs <= 256) return 29.5 + 5.0 * (double)wgs / 256.0 * (double)wgs / 256.0;
  return t_full * (double)full + (rem ? t_low + (t_full - t_low) * fill * fill : 0.0);
}

}  // namespace

// Whole K steps of 128, bf16 activations on a 16-byte boundary, 32-bit byte offsets into a row block of
// activations and into one K step of the copy.
bool gemm_dense_applies(const FpArgs& f) {
  if (f.x_dtype != WOQ_HIP_ACT_BF16 || ((uintptr_t)f.x & 15) != 0 || f.M <= 0) return false;
  if (f.K % 128 != 0 || f.K * 256 * 2 >= (int64_t)1 << 31) return false;
  return f.NT * (f.K / 128) * 4096 < (int64_t)1 << 31;
}

double gemm_dense_cost(const FpArgs& f) {
  const double c = std::min(dense_shape_cost<GdShape<8, 7>>(f),
                            std::min(dense_shape_cost<GdShape<8, 4>>(f), dense_shape_cost<GdShape<8, 2>>(f)));
  return c * (double)f.K / 4096.0;
}

int launch_gemm_dense(const FpArgs& f, const void* dense, int wbits, hipStream_t st, int shape) {
  if (!gemm_dense_applies(f)) return set_error("woq_gemm_dense_kernel: shape or activations not supported");
  GdArgs a{f, (const uint8_t*)dense, wbits == 8 ? 1 : 0};
  using S7 = GdShape<8, 7>;
  using S4 = GdShape<8, 4>;
  using S2 = GdShape<8, 2>;
  if (shape == 0) {
    const double c7 = dense_shape_cost<S7>(f), c4 = dense_shape_cost<S4>(f), c2 = dense_shape_cost<S2>(f);
    shape = (c7 <= c4 && c7 <= c2) ? 7 : (c4 <= c2 ? 4 : 2);
  }
  if (shape == 7) return launch_dense_shape<S7>(a, st);
  if (shape == 4) return launch_dense_shape<S4>(a, st);
  if (shape == 2) return launch_dense_shape<S2>(a, st);
  return set_error("woq_gemm_dense_kernel: shapes are 7, 4 and 2 row-blocks per wave");
}

}  // namespace woq

// fp32 compute: lowp_mode NONE with fp32 activations (also what lowp_mode INT8 falls back to for
// fp32 activations).
//
// Reference counterpart: woq_gemm_fp32 -> qlinear_woq_affine_impl<float, float, float, float, float,
// float> (csrc/cpu/aten/kernels/WoqLinearKrnl.cpp:142-158): fp32 scales and zero points,
// w = (q - z) * s as a subtraction and a product in fp32 (csrc/cpu/aten/utils/woq.h:183-186,
// 703-708; NF4: table[q] * s), fp32 x fp32 products accumulated in fp32 on top of the fp32 bias,
// post-op and store in fp32.
//
// y[M, N] = x[M, K] * w[N, K]^T on v_mfma_f32_32x32x2_f32: workgroup tile 128 x 128, K step 32,
// 4 waves in a 2 x 2 grid, each owning 64 x 64 as 2 x 2 MFMA tiles (A = activations, B = weights:
// a lane's accumulator registers hold consecutive rows of its own output column); up to 64 rows
// (SMALL) the tile is 32 x 128 and a wave owns one 32 x 32 MFMA tile, a quarter of the MFMA work
// per K step.  Weights are dequantized once per workgroup and K step into LDS.  One MFMA consumes the K pair (2t, 2t + 1),
// lanes 0..31 the even element and lanes 32..63 the odd one; both LDS tiles keep the even elements
// of a row in floats 0..15 and the odd ones in floats 16..31, so that a lane reads the operands of
// four MFMAs with one 16-byte load.
#include "woq_common.h"
#include "woq_internal.h"

namespace woq {

namespace {
constexpr int F_BM = 128, F_BN = 128, F_BK = 32;
constexpr int F_STRIDE = F_BK + 4;  // floats; keeps 16-byte alignment, spreads rows over the banks
}  // namespace

template <int WBITS, bool NF4, bool SMALL>
__global__ __launch_bounds__(256) void woq_fp32_kernel(const Fp32Args f) {
  static_assert(!NF4 || WBITS == 4, "NF4 codes are 4 bits wide");
  constexpr int TK = WBITS == 4 ? kTileK4 : kTileK8;
  constexpr int BM = SMALL ? 32 : F_BM;
  constexpr int XI = BM / 32;         // 16-byte activation pieces per thread and K step
  constexpr int TM = SMALL ? 1 : 2;   // MFMA tiles per wave along M and N
  constexpr int TN = SMALL ? 1 : 2;
  __shared__ __align__(16) float sA[BM * F_STRIDE];
  __shared__ __align__(16) float sB[F_BN * F_STRIDE];
  __shared__ float sTab[16];

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int row0 = SMALL ? 0 : (wave >> 1) * 64;             // first row / column of this wave
  const int col0 = SMALL ? wave * 32 : (wave & 1) * 64;
  const int64_t m0 = (int64_t)blockIdx.y * BM;
  const int64_t n0 = (int64_t)blockIdx.x * F_BN;
  const int64_t nt0 = n0 / kTileN;
  const int64_t Kpad = f.KT * TK;
  const bool xvec = (f.K % 4) == 0;

  if (NF4) {
    if (tid < 16) sTab[tid] = kNf4Values[tid];
    __syncthreads();
  }

  f16v acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // weight slot of this thread: row-block ntl of the workgroup's eight, row r, and 16 of the 32 K
  // values of the step
  const int ntl = tid >> 5, r = tid & 15, hh = (tid >> 4) & 1;
  const int64_t nt = nt0 + ntl;
  const bool wvalid = nt < f.NT;

  // raw operands of one K step in registers: requested one step ahead, so that they travel
  // during the MFMAs of the step before
  f4 xa[XI];
  uint32_t d[4] = {0u, 0u, 0u, 0u};
  float s = 1.0f, z = 0.0f;
  auto request = [&](int64_t k0) {
    // ---- activations: BM rows x 32 floats, one 16-byte piece per thread and 32 rows ----
#pragma unroll
    for (int i = 0; i < XI; ++i) {
      const int64_t m = m0 + (tid >> 3) + 32 * i;
      const int64_t k = k0 + (tid & 7) * 4;
      xa[i] = f4{0.f, 0.f, 0.f, 0.f};
      if (m < f.M) {
        if (xvec) {
          if (k < f.K) xa[i] = *(const f4*)(f.x + m * f.K + k);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (k + e < f.K) xa[i][e] = f.x[m * f.K + k + e];
        }
      }
    }
    // ---- weights: 16 values of one row with their scale and zero point ----
    if (wvalid) {
      const int64_t kt = k0 / TK;
      int64_t g = k0 / f.G;
      if (g >= f.KG) g = f.KG - 1;
      const int64_t qi = (nt * f.KG + g) * kTileN + r;
      s = f.scales[qi];
      z = f.zeros ? (float)f.zeros[qi] : (WBITS == 4 ? 8.0f : 128.0f);
      if (WBITS == 4) {
        const int c = (int)((k0 % TK) / 32);
        const uint32_t* p = (const uint32_t*)(f.qweight + ((nt * f.KT + kt) * 64 + (r + 16 * c)) * 16) + 2 * hh;
        d[0] = p[0];
        d[1] = p[1];
      } else {
        const int c = (int)((k0 % TK) / 16) + hh;
        const u4 v = *(const u4*)(f.qweight + ((nt * f.KT + kt) * 64 + (r + 16 * c)) * 16);
        d[0] = v[0]; d[1] = v[1]; d[2] = v[2]; d[3] = v[3];
      }
    }
  };

  if (Kpad > 0) request(0);
  for (int64_t k0 = 0; k0 < Kpad; k0 += F_BK) {
    // ---- dequantize to fp32 ----
    float w[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      float q;
      if (WBITS == 4)
        q = (float)((d[e >> 3] >> (4 * nibble_pos(e & 7))) & 0xFu);
      else
        q = (float)((d[e >> 2] >> (8 * (e & 3))) & 0xFFu);
      if (NF4)
        w[e] = wvalid ? __fmul_rn(sTab[(int)q], s) : 0.0f;
      else if (WBITS == 8 && f.fp8)  // float8 e4m3fn bytes: w = fp8(byte) * s (woq.h:728-741)
        w[e] = wvalid ? __fmul_rn(fp8_e4m3fn_to_f32((d[e >> 2] >> (8 * (e & 3))) & 0xFFu), s) : 0.0f;
      else
        w[e] = wvalid ? __fmul_rn(__fsub_rn(q, z), s) : 0.0f;
    }

    __syncthreads();  // the previous step's LDS reads are done
#pragma unroll
    for (int i = 0; i < XI; ++i) {
      float* row = sA + ((tid >> 3) + 32 * i) * F_STRIDE;
      const int kl = (tid & 7) * 4;  // elements kl .. kl + 3: two even, two odd
      *(f2*)(row + (kl >> 1)) = f2{xa[i][0], xa[i][2]};
      *(f2*)(row + 16 + (kl >> 1)) = f2{xa[i][1], xa[i][3]};
    }
    {
      float* row = sB + (ntl * 16 + r) * F_STRIDE + hh * 8;  // elements 16 hh .. 16 hh + 15
      *(f4*)(row) = f4{w[0], w[2], w[4], w[6]};
      *(f4*)(row + 4) = f4{w[8], w[10], w[12], w[14]};
      *(f4*)(row + 16) = f4{w[1], w[3], w[5], w[7]};
      *(f4*)(row + 20) = f4{w[9], w[11], w[13], w[15]};
    }
    __syncthreads();
    if (k0 + F_BK < Kpad) request(k0 + F_BK);

    // ---- 16 K pairs: lane half h supplies element 2 t + h of pair t ----
    const int h = lane >> 5;
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      f4 af[TM], bf[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[i] = *(const f4*)(sA + (row0 + i * 32 + (lane & 31)) * F_STRIDE + h * 16 + q4 * 4);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        bf[j] = *(const f4*)(sB + (col0 + j * 32 + (lane & 31)) * F_STRIDE + h * 16 + q4 * 4);
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][t], bf[j][t], acc[i][j], 0, 0, 0);
    }
  }

  // ---- epilogue: D[m][n], lane holds n = lane % 32, m = 8 * (e / 4) + 4 * (lane / 32) + e % 4 ----
  Epilogue ep{f.bias, f.fusion, f.other0, f.other1, f.out, WOQ_HIP_ACT_FP32, WOQ_HIP_ACT_FP32, f.N};
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int64_t n = n0 + col0 + j * 32 + (lane & 31);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int64_t m = m0 + row0 + i * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
        if (m < f.M && n < f.N) epilogue_store<kRegimeBF16>(ep, m, n, acc[i][j][e]);
      }
    }
}

int launch_fp32(const Fp32Args& f, int wbits, hipStream_t st) {
  if (f.G <= 0 || f.G % F_BK != 0) return set_error("woq_linear: fp32 compute needs groups that are multiples of 32");
  const bool small = f.M <= 64;
  const int bm = small ? 32 : F_BM;
  dim3 grid((unsigned)((f.NT * kTileN + F_BN - 1) / F_BN), (unsigned)((f.M + bm - 1) / bm));
#define WOQ_FP32(WB, NF)                                          \
  (small ? woq_fp32_kernel<WB, NF, true><<<grid, 256, 0, st>>>(f) \
         : woq_fp32_kernel<WB, NF, false><<<grid, 256, 0, st>>>(f))
  if (wbits == 8)
    WOQ_FP32(8, false);
  else if (f.nf4)
    WOQ_FP32(4, true);
  else
    WOQ_FP32(4, false);
#undef WOQ_FP32
  return check_launch("woq_fp32_kernel");
}

}  // namespace woq

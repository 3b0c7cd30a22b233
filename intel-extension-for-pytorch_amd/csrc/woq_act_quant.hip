// Dynamic activation quantization of whole rows in one pass: statistics and quantization from
// registers, for the modes with one scale per row or per (row, K block).
//
// Reference counterpart: dynamic_quantize_per_block (csrc/cpu/aten/utils/woq_dynamic_quant.h:1526-1750):
// symmetric s = max(|max|, |min|) / 127, q = clamp(rint(x / s), -128, 127); asymmetric
// s = (max - min) / 255, zp = -rint(min / s), q = clamp(rint(x / s + zp), 0, 255), all in IEEE fp32.
//
// The two-kernel form (one workgroup per quantization group for the statistics, then one thread per
// 8 elements) reads the activations twice and, for per-(row, K block) scales, starts one workgroup
// per 128 elements.  Here a wave owns a row: it loads the row once (16 bytes per lane and 512-element
// chunk, kept as the raw 16-bit values), reduces min / max over the wave (or over the lanes of a K
// block), and quantizes from the registers.  Same arithmetic, expression by expression, as the
// two-kernel form, so the bytes and the scales are identical.
#include "woq_common.h"
#include "woq_internal.h"

// every rounding of the reference's expressions is kept: no multiply-add contraction in this file
#pragma clang fp contract(off)

namespace woq {

namespace {

// lane's eight values of one chunk
__device__ __forceinline__ void aq_unpack(u4 raw, bool bf16, float (&v)[8]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint16_t lo = (uint16_t)(raw[i] & 0xFFFFu), hi = (uint16_t)(raw[i] >> 16);
    v[2 * i] = bf16 ? bf16_bits_to_f32(lo) : f16_bits_to_f32(lo);
    v[2 * i + 1] = bf16 ? bf16_bits_to_f32(hi) : f16_bits_to_f32(hi);
  }
}

struct AqParams {
  float s, zp;
};

__device__ __forceinline__ AqParams aq_params(float mn, float mx, bool sym, int32_t* zp_out) {
  AqParams p;
  if (sym) {
    p.s = __fdiv_rn(fmaxf(fabsf(mx), fabsf(mn)), 127.0f);
    p.zp = 0.0f;
  } else {
    p.s = __fdiv_rn(__fsub_rn(mx, mn), 255.0f);
    const int32_t z = (int32_t)(-rintf(__fdiv_rn(mn, p.s)));
    p.zp = (float)z;
    if (zp_out) *zp_out = z;
  }
  return p;
}

__device__ __forceinline__ uint8_t aq_quant(float v, AqParams p, bool sym, bool offset128) {
  float t = __fadd_rn(__fdiv_rn(v, p.s), p.zp);
  t = rintf(t);
  const float lo = sym ? -128.0f : 0.0f, hi = sym ? 127.0f : 255.0f;
  t = fminf(fmaxf(t, lo), hi);
  if (p.s == 0.0f || t != t) t = sym ? 0.0f : p.zp;  // all-zero group: the reference divides 0 by 0
  return sym ? (uint8_t)(int8_t)(int)t : (uint8_t)((int)t ^ (offset128 ? 0x80 : 0));
}

struct AqArgs {
  const uint16_t* x;
  int bf16;
  int64_t M, K, ldq;
  int block_lanes_log2;  // per-(row, K block) scales: log2(block / 8); -1: one scale per row
  int block_shift;       // log2(block)
  int64_t Kc;
  int sym;
  float* scales;
  int32_t* zps;
  uint8_t* q;
  int permute, offset128;
  int given;  // the scales (and zero points) are inputs, shared by all rows: one per tensor or per K block
};

// NCH: 512-element chunks of a (padded) row that one wave holds.  SPLIT: the four waves of a
// workgroup share one row (wave w takes chunks w, w + 4, ...), for the few rows of a decode step,
// where a single wave per row would be one long dependent chain (M = 1, K = 4096: 6.5 us).
template <int NCH, bool SPLIT>
__global__ __launch_bounds__(256) void act_quant_rows_kernel(const AqArgs a) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t m = SPLIT ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * 4 + wave;
  if (m >= a.M) return;
  // chunk held in register slot c
  auto chunk_of = [&](int c) { return SPLIT ? wave + 4 * c : c; };
  const uint16_t* const row = a.x + m * a.K;
  const bool bf16 = a.bf16 != 0, sym = a.sym != 0, per_k = a.block_lanes_log2 >= 0;

  // K % 8 == 0: a lane's eight elements are all inside the row or all outside
  u4 raw[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int64_t k0 = (int64_t)chunk_of(c) * 512 + lane * 8;
    raw[c] = k0 < a.K ? *(const u4*)(row + k0) : u4{0u, 0u, 0u, 0u};
  }

  const bool given = a.given != 0;
  float mn[NCH], mx[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    mn[c] = __builtin_inff();
    mx[c] = -__builtin_inff();
    if (!given && (int64_t)chunk_of(c) * 512 + lane * 8 < a.K) {
      float v[8];
      aq_unpack(raw[c], bf16, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        mn[c] = fminf(mn[c], v[e]);
        mx[c] = fmaxf(mx[c], v[e]);
      }
    }
  }
  if (given) {
    // nothing to reduce
  } else if (!per_k) {
#pragma unroll
    for (int c = 1; c < NCH; ++c) {
      mn[0] = fminf(mn[0], mn[c]);
      mx[0] = fmaxf(mx[0], mx[c]);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      mn[0] = fminf(mn[0], __shfl_xor(mn[0], off));
      mx[0] = fmaxf(mx[0], __shfl_xor(mx[0], off));
    }
    if constexpr (SPLIT) {
      // the four waves' extremes meet in LDS (every wave of the workgroup is here: same row)
      __shared__ float smn[4], smx[4];
      if (lane == 0) {
        smn[wave] = mn[0];
        smx[wave] = mx[0];
      }
      __syncthreads();
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        mn[0] = fminf(mn[0], smn[w]);
        mx[0] = fmaxf(mx[0], smx[w]);
      }
    }
  } else {
    // the lanes of one K block are 2^block_lanes_log2 consecutive lanes, aligned
#pragma unroll
    for (int c = 0; c < NCH; ++c)
      for (int step = 0; step < a.block_lanes_log2; ++step) {
        mn[c] = fminf(mn[c], __shfl_xor(mn[c], 1 << step));
        mx[c] = fmaxf(mx[c], __shfl_xor(mx[c], 1 << step));
      }
  }

  AqParams row_p;
  if (given) {
    row_p.s = a.scales[0];
    row_p.zp = sym ? 0.0f : (float)a.zps[0];
  } else if (!per_k) {
    int32_t z = 0;
    row_p = aq_params(mn[0], mx[0], sym, &z);
    if (lane == 0 && (!SPLIT || wave == 0)) {
      a.scales[m] = row_p.s;
      if (!sym) a.zps[m] = z;
    }
  }
  uint8_t* const qrow = a.q + m * a.ldq;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int64_t k0 = (int64_t)chunk_of(c) * 512 + lane * 8;
    if (k0 >= a.ldq) continue;
    u2 out = u2{0u, 0u};  // the tail of a padded row is zero
    if (k0 < a.K) {
      AqParams p = row_p;
      if (given && per_k) {
        p.s = a.scales[k0 >> a.block_shift];
        p.zp = sym ? 0.0f : (float)a.zps[k0 >> a.block_shift];
      } else if (per_k) {
        int32_t z = 0;
        p = aq_params(mn[c], mx[c], sym, &z);
        if ((lane & ((1 << a.block_lanes_log2) - 1)) == 0) {
          const int64_t gi = m * a.Kc + (k0 >> a.block_shift);
          a.scales[gi] = p.s;
          if (!sym) a.zps[gi] = z;
        }
      }
      float v[8];
      aq_unpack(raw[c], bf16, v);
      uint32_t o[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = aq_quant(v[e], p, sym, a.offset128 != 0);
      if (a.permute) {
        out[0] = o[0] | (o[4] << 8) | (o[1] << 16) | (o[5] << 24);
        out[1] = o[2] | (o[6] << 8) | (o[3] << 16) | (o[7] << 24);
      } else {
        out[0] = o[0] | (o[1] << 8) | (o[2] << 16) | (o[3] << 24);
        out[1] = o[4] | (o[5] << 8) | (o[6] << 16) | (o[7] << 24);
      }
    }
    *(u2*)(qrow + k0) = out;
  }
}

// ---- scales shared by all rows (one per tensor, or one per K block) ----
// The extremes travel as integer keys whose order is the order of the floats, so that workgroups can
// merge them with integer atomics: one atomic per workgroup and scale (per wave or per element, every
// update of a per-tensor scale would queue at one address).
__device__ __forceinline__ int32_t aq_float_key(float f) {
  const int32_t b = __builtin_bit_cast(int32_t, f);
  return b ^ ((b >> 31) & 0x7fffffff);
}
__device__ __forceinline__ float aq_key_float(int32_t k) {
  return __builtin_bit_cast(float, k ^ ((k >> 31) & 0x7fffffff));
}

__global__ void aq_shared_init_kernel(int groups, int32_t* maxk, int32_t* mink) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= groups) return;
  maxk[i] = aq_float_key(-__builtin_inff());
  if (mink) mink[i] = aq_float_key(__builtin_inff());
}

// Wave w of a workgroup takes rows w, w + 4, ... of the workgroup's rows_per_wg rows; slot c of a lane
// sees the same eight K offsets in every row, so per-K-block extremes accumulate in registers over the
// rows, then over the lanes of a block; the four waves merge theirs with LDS atomics, and the workgroup
// reports each scale's extremes once.
template <int NCH>
__global__ __launch_bounds__(256) void act_stats_shared_kernel(const AqArgs a, int rows_per_wg, int32_t* maxk,
                                                               int32_t* mink) {
  // one entry per scale: a K block has at least eight elements, a lane's share of a chunk
  __shared__ int32_t kmax[NCH * 64], kmin[NCH * 64];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const bool bf16 = a.bf16 != 0, sym = a.sym != 0, per_k = a.block_lanes_log2 >= 0;
  const int groups = per_k ? (int)a.Kc : 1;
  for (int t = threadIdx.x; t < groups; t += 256) {
    kmax[t] = aq_float_key(-__builtin_inff());
    kmin[t] = aq_float_key(__builtin_inff());
  }
  __syncthreads();
  const int64_t m_lo = (int64_t)blockIdx.x * rows_per_wg;
  const int64_t m_hi = m_lo + rows_per_wg < a.M ? m_lo + rows_per_wg : a.M;
  float mn[NCH], mx[NCH];
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    mn[c] = __builtin_inff();
    mx[c] = -__builtin_inff();
  }
  for (int64_t m = m_lo + wave; m < m_hi; m += 4) {
    const uint16_t* const row = a.x + m * a.K;
    u4 raw[NCH];
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int64_t k0 = (int64_t)c * 512 + lane * 8;
      raw[c] = k0 < a.K ? *(const u4*)(row + k0) : u4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      if ((int64_t)c * 512 + lane * 8 < a.K) {
        float v[8];
        aq_unpack(raw[c], bf16, v);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          mn[c] = fminf(mn[c], v[e]);
          mx[c] = fmaxf(mx[c], v[e]);
        }
      }
    }
  }
  if (!per_k) {
#pragma unroll
    for (int c = 1; c < NCH; ++c) {
      mn[0] = fminf(mn[0], mn[c]);
      mx[0] = fmaxf(mx[0], mx[c]);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      mn[0] = fminf(mn[0], __shfl_xor(mn[0], off));
      mx[0] = fmaxf(mx[0], __shfl_xor(mx[0], off));
    }
    if (lane == 0) {
      atomicMax(&kmax[0], aq_float_key(mx[0]));
      atomicMin(&kmin[0], aq_float_key(mn[0]));
    }
  } else {
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      for (int step = 0; step < a.block_lanes_log2; ++step) {
        mn[c] = fminf(mn[c], __shfl_xor(mn[c], 1 << step));
        mx[c] = fmaxf(mx[c], __shfl_xor(mx[c], 1 << step));
      }
      const int64_t k0 = (int64_t)c * 512 + lane * 8;
      // the first lane of a K block reports it
      if ((lane & ((1 << a.block_lanes_log2) - 1)) == 0 && k0 < a.K) {
        atomicMax(&kmax[k0 >> a.block_shift], aq_float_key(mx[c]));
        atomicMin(&kmin[k0 >> a.block_shift], aq_float_key(mn[c]));
      }
    }
  }
  __syncthreads();
  for (int t = threadIdx.x; t < groups; t += 256) {
    const float hi = aq_key_float(kmax[t]), lo = aq_key_float(kmin[t]);
    if (hi < lo) continue;  // a workgroup that saw no element still holds (-inf, +inf)
    if (sym) {
      atomicMax(maxk + t, aq_float_key(fmaxf(fabsf(hi), fabsf(lo))));
    } else {
      atomicMax(maxk + t, aq_float_key(hi));
      atomicMin(mink + t, aq_float_key(lo));
    }
  }
}

// keys -> scale (and zero point), in place
__global__ void aq_shared_finalize_kernel(int groups, int sym, float* scales, int32_t* zps) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= groups) return;
  const float mx = aq_key_float(__builtin_bit_cast(int32_t, scales[i]));
  int32_t z = 0;
  const AqParams p = sym ? aq_params(-mx, mx, true, &z) : aq_params(aq_key_float(zps[i]), mx, false, &z);
  scales[i] = p.s;
  if (!sym) zps[i] = z;
}

template <int NCH, bool SPLIT>
void aq_launch_rows(const AqArgs& a, unsigned grid, hipStream_t st) {
  act_quant_rows_kernel<NCH, SPLIT><<<grid, 256, 0, st>>>(a);
}

// the quantization pass over whole rows, for scales computed here or given
void aq_launch_quant(const AqArgs& a, hipStream_t st) {
  const int64_t chunks = (a.ldq + 511) / 512;
  if (a.M <= 64) {
    // few rows: a workgroup per row, a quarter of the chunks per wave
    if (chunks <= 8)
      aq_launch_rows<2, true>(a, (unsigned)a.M, st);
    else if (chunks <= 16)
      aq_launch_rows<4, true>(a, (unsigned)a.M, st);
    else
      aq_launch_rows<8, true>(a, (unsigned)a.M, st);
    return;
  }
  const unsigned grid = (unsigned)((a.M + 3) / 4);
  if (chunks <= 8)
    aq_launch_rows<8, false>(a, grid, st);
  else if (chunks <= 16)
    aq_launch_rows<16, false>(a, grid, st);
  else
    aq_launch_rows<32, false>(a, grid, st);
}

}  // namespace

// Rows of 16-bit activations that fit a wave's registers (padded row <= 16384 elements), one scale per
// row or per (row, K block of 8 * 2^j <= 512 elements).
bool act_quant_rows_applies(const void* x, int x_dtype, int64_t K, const void* q, int64_t ldq, int64_t qbk,
                            bool per_m, bool per_k) {
  (void)per_m;  // scales per row: one pass; shared by all rows: statistics, then the same pass with given scales
  if (x_dtype != WOQ_HIP_ACT_BF16 && x_dtype != WOQ_HIP_ACT_FP16) return false;
  if (((uintptr_t)x & 15) != 0 || ((uintptr_t)q & 7) != 0) return false;
  if (K % 8 != 0 || ldq % 8 != 0 || ldq < K || ldq > 16384) return false;
  if (per_k && (qbk < 8 || qbk > 512 || (qbk & (qbk - 1)) != 0)) return false;
  return true;
}

int launch_act_quant_rows(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldq, int64_t qbk, int64_t Kc,
                          bool per_m, bool per_k, bool sym, void* q, float* scales, int32_t* zps, int permute,
                          int offset128, hipStream_t st) {
  if (!sym && zps == nullptr) return set_error("dynamic_quant: asymmetric modes need a zero-point array");
  AqArgs a;
  a.x = (const uint16_t*)x;
  a.bf16 = x_dtype == WOQ_HIP_ACT_BF16;
  a.M = M; a.K = K; a.ldq = ldq;
  a.block_lanes_log2 = -1;
  a.block_shift = 0;
  if (per_k) {
    while (((int64_t)1 << a.block_shift) < qbk) ++a.block_shift;
    a.block_lanes_log2 = a.block_shift - 3;
  }
  a.Kc = Kc;
  a.sym = sym;
  a.scales = scales; a.zps = zps; a.q = (uint8_t*)q;
  a.permute = permute; a.offset128 = offset128;
  a.given = 0;
  // one row: its statistics are the tensor's
  if (per_m || M == 1) {
    aq_launch_quant(a, st);
    return check_launch("act_quant_rows_kernel");
  }
  const int groups = per_k ? (int)Kc : 1;
  int32_t* const maxk = (int32_t*)scales;
  int32_t* const mink = sym ? nullptr : zps;
  aq_shared_init_kernel<<<(unsigned)((groups + 255) / 256), 256, 0, st>>>(groups, maxk, mink);
  if (int rc = check_launch("aq_shared_init_kernel")) return rc;
  // about 512 workgroups at 2048 rows and more; at least one row per wave
  const int rows_per_wg = 4 * (int)((M + 2047) / 2048);
  const unsigned grid = (unsigned)((M + rows_per_wg - 1) / rows_per_wg);
  const int64_t chunks = (K + 511) / 512;
  if (chunks <= 8)
    act_stats_shared_kernel<8><<<grid, 256, 0, st>>>(a, rows_per_wg, maxk, mink);
  else if (chunks <= 16)
    act_stats_shared_kernel<16><<<grid, 256, 0, st>>>(a, rows_per_wg, maxk, mink);
  else
    act_stats_shared_kernel<32><<<grid, 256, 0, st>>>(a, rows_per_wg, maxk, mink);
  if (int rc = check_launch("act_stats_shared_kernel")) return rc;
  aq_shared_finalize_kernel<<<(unsigned)((groups + 255) / 256), 256, 0, st>>>(groups, sym ? 1 : 0, scales, zps);
  if (int rc = check_launch("aq_shared_finalize_kernel")) return rc;
  a.given = 1;
  aq_launch_quant(a, st);
  return check_launch("act_quant_rows_kernel");
}

}  // namespace woq

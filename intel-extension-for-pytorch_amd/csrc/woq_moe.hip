// Token gather / weighted scatter around the expert linears of a mixture-of-experts layer whose
// experts are weight-only-quantized linears.
//
// Reference counterparts (csrc/cpu/aten/kernels/MoEKrnl.cpp): fuse_index_unsqueeze (:123-160) copies
// the rows of the tokens routed to one expert into a dense [n, H] tensor; after the expert's
// gate / up / down linears, fuse_index_mul_index_add (:31-121) does
//   output[top_x[i], :] += routing_weights[top_x[i], idx[i]] * expert_out[i, :]
// with the sum formed in fp32 and rounded once for bf16 (:96-110), in fp32 for fp32 (:60-61), and
// as an fp16 product followed by an fp16 add for any other dtype (:277-280).
// Both are HBM-bound row copies: one 16-byte chunk per thread where rows allow it.
#include "woq_common.h"
#include "woq_internal.h"

// The multiply and the add below are separate roundings; hipcc would otherwise contract them into
// one fused multiply-add (for fp16 even into v_pk_fma_f16, which skips the rounding of the product).
// The pragma covers operators written in this file only: the __fmul_rn / __fadd_rn helpers are
// header functions compiled under the command line's contraction mode and fuse all the same.
#pragma clang fp contract(off)

namespace woq {

// out[i, :] = x[rows[i], :]; a row is `chunks` units of T.  The indices come from the caller's routing
// tensors: a row outside [0, tokens) reads nothing and leaves zeros (an out-of-bounds access would be a
// device fault, not an error the host can report).
template <typename T>
__global__ void moe_gather_rows_kernel(const T* __restrict__ x, const int64_t* __restrict__ rows, int64_t n,
                                       int64_t chunks, int64_t tokens, T* __restrict__ out) {
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= n * chunks) return;
  const int64_t i = g / chunks, c = g - i * chunks;
  const int64_t row = rows[i];
  out[g] = (uint64_t)row < (uint64_t)tokens ? x[row * chunks + c] : T{};
}

template <int DTYPE>
__device__ __forceinline__ float moe_accumulate(float o, float v, float w) {
  if constexpr (DTYPE == WOQ_HIP_ACT_FP16) {
    const float p = f16_bits_to_f32(f32_to_f16_bits(v * w));  // product rounded to fp16 first
    return o + p;
  } else {
    const float p = v * w;  // separate multiply and add, as the vector code does
    return o + p;
  }
}

// One thread per (i, 8 consecutive columns) for the 16-bit dtypes, per (i, 4 columns) for fp32.
template <int DTYPE>
__global__ void moe_scale_add_rows_kernel(void* __restrict__ out, const void* __restrict__ cur,
                                          const void* __restrict__ rw, int64_t topk, const int64_t* __restrict__ top_x,
                                          const int64_t* __restrict__ idx, int64_t n, int64_t H, int64_t tokens,
                                          bool vec) {
  constexpr int PER = DTYPE == WOQ_HIP_ACT_FP32 ? 4 : 8;
  const int64_t chunks = (H + PER - 1) / PER;
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= n * chunks) return;
  const int64_t i = g / chunks, j0 = (g - i * chunks) * PER;
  const int64_t t = top_x[i], slot = idx[i];
  // a token or a top-k slot out of range is skipped: nothing is read or written for it
  if ((uint64_t)t >= (uint64_t)tokens || (uint64_t)slot >= (uint64_t)topk) return;
  const float w = load_act(rw, DTYPE, t * topk + slot);
  const int64_t ob = t * H + j0, cb = i * H + j0;
  if (vec) {
    if constexpr (DTYPE == WOQ_HIP_ACT_FP32) {
      f4 o = *(const f4*)((const float*)out + ob);
      const f4 v = *(const f4*)((const float*)cur + cb);
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = moe_accumulate<DTYPE>(o[e], v[e], w);
      *(f4*)((float*)out + ob) = o;
    } else {
      u4 o = *(const u4*)((const uint16_t*)out + ob);
      const u4 v = *(const u4*)((const uint16_t*)cur + cb);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        uint32_t r = 0;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const uint16_t ob16 = (uint16_t)(o[e] >> (16 * h)), vb16 = (uint16_t)(v[e] >> (16 * h));
          const float of = DTYPE == WOQ_HIP_ACT_BF16 ? bf16_bits_to_f32(ob16) : f16_bits_to_f32(ob16);
          const float vf = DTYPE == WOQ_HIP_ACT_BF16 ? bf16_bits_to_f32(vb16) : f16_bits_to_f32(vb16);
          const float s = moe_accumulate<DTYPE>(of, vf, w);
          r |= (uint32_t)(DTYPE == WOQ_HIP_ACT_BF16 ? f32_to_bf16_bits(s) : f32_to_f16_bits(s)) << (16 * h);
        }
        o[e] = r;
      }
      *(u4*)((uint16_t*)out + ob) = o;
    }
  } else {
    for (int e = 0; e < PER && j0 + e < H; ++e)
      store_act(out, DTYPE, ob + e, moe_accumulate<DTYPE>(load_act(out, DTYPE, ob + e), load_act(cur, DTYPE, cb + e), w));
  }
}

static inline unsigned moe_blocks(int64_t n) { return (unsigned)((n + 255) / 256); }

int launch_moe_gather_rows(const void* x, int x_dtype, int64_t T, int64_t H, const int64_t* rows, int64_t n, void* out,
                           hipStream_t st) {
  if (n == 0 || H == 0) return 0;
  const int64_t row_bytes = H * (x_dtype == WOQ_HIP_ACT_FP32 ? 4 : 2);
  if (row_bytes % 16 == 0 && (((uintptr_t)x | (uintptr_t)out) & 15) == 0) {
    const int64_t chunks = row_bytes / 16;
    moe_gather_rows_kernel<u4><<<moe_blocks(n * chunks), 256, 0, st>>>((const u4*)x, rows, n, chunks, T, (u4*)out);
  } else if (x_dtype == WOQ_HIP_ACT_FP32) {
    moe_gather_rows_kernel<uint32_t><<<moe_blocks(n * H), 256, 0, st>>>((const uint32_t*)x, rows, n, H, T, (uint32_t*)out);
  } else {
    moe_gather_rows_kernel<uint16_t><<<moe_blocks(n * H), 256, 0, st>>>((const uint16_t*)x, rows, n, H, T, (uint16_t*)out);
  }
  return check_launch("moe_gather_rows");
}

int launch_moe_scale_add_rows(void* out, int dtype, int64_t T, int64_t H, const void* cur, const void* rw, int64_t topk,
                              const int64_t* top_x, const int64_t* idx, int64_t n, hipStream_t st) {
  if (n == 0 || H == 0) return 0;
  const int per = dtype == WOQ_HIP_ACT_FP32 ? 4 : 8;
  const bool vec = H % per == 0 && (((uintptr_t)out | (uintptr_t)cur) & 15) == 0;
  const unsigned blocks = moe_blocks(n * ((H + per - 1) / per));
  if (dtype == WOQ_HIP_ACT_BF16)
    moe_scale_add_rows_kernel<WOQ_HIP_ACT_BF16><<<blocks, 256, 0, st>>>(out, cur, rw, topk, top_x, idx, n, H, T, vec);
  else if (dtype == WOQ_HIP_ACT_FP16)
    moe_scale_add_rows_kernel<WOQ_HIP_ACT_FP16><<<blocks, 256, 0, st>>>(out, cur, rw, topk, top_x, idx, n, H, T, vec);
  else
    moe_scale_add_rows_kernel<WOQ_HIP_ACT_FP32><<<blocks, 256, 0, st>>>(out, cur, rw, topk, top_x, idx, n, H, T, vec);
  return check_launch("moe_scale_add_rows");
}

}  // namespace woq

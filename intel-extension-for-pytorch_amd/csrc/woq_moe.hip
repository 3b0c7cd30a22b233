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

// Routing of a whole layer on the device, for the grouped launches: one workgroup sorts the R = tokens x top-k
// (token, slot) entries by expert -- stable, so that inside an expert the tokens ascend, the order of
// get_expert_topx_idx (csrc/cpu/aten/MoE.cpp:64-81) -- and writes
//   x_row[p]        token of the entry at sorted position p (the row of the hidden states it reads),
//   slots           [4 classes][expert, first row, rows][S]: the experts that have tokens, densely from index 0 and in
//                   ascending expert order, by size class -- 0: fewer than split_lo rows, 1: at most split_mid,
//                   2: more, 3 (use_single 1): exactly one row (taken out of class 0) -- unused entries expert -1;
//                   use_single 2: every sorted position p is a slot of one row in class 3, at index p (an expert
//                   named twice then has two slots; for a single token, where that costs nothing),
//   row_of[t, i]    sorted position of token t's i-th contribution in ascending expert order (-1: none),
//   slot_of[t, i]   its top-k slot.
// An expert id outside [0, experts) contributes nothing.  R <= kMoeRouteMax entries, compared pairwise from LDS.
constexpr int kMoeRouteMax = WOQ_HIP_MOE_ROUTE_MAX;
constexpr int kMoeSlotRowsMax = 64;
__global__ __launch_bounds__(256) void moe_route_kernel(const int64_t* __restrict__ ids, int R, int topk, int experts,
                                                        int split_lo, int split_mid, int use_single, int S,
                                                        int64_t* __restrict__ x_row, int32_t* __restrict__ slots,
                                                        int32_t* __restrict__ row_of, int32_t* __restrict__ slot_of) {
  __shared__ int se[kMoeRouteMax];
  __shared__ int8_t cls_of[kMoeRouteMax];  // size class of the expert whose first sorted position this is, or -1
  for (int i = threadIdx.x; i < R; i += blockDim.x) {
    const int64_t e = ids[i];
    se[i] = (e >= 0 && e < experts) ? (int)e : -1;
    cls_of[i] = -1;
    row_of[i] = -1;
    slot_of[i] = 0;
  }
  for (int i = threadIdx.x; i < 12 * S; i += blockDim.x) slots[i] = (i / S) % 3 == 0 ? -1 : 0;
  __syncthreads();
  int my_p[kMoeRouteMax / 256], my_e[kMoeRouteMax / 256], my_n[kMoeRouteMax / 256];
#pragma unroll
  for (int u = 0; u < kMoeRouteMax / 256; ++u) {
    my_p[u] = -1;
    const int i = (int)threadIdx.x + u * 256;
    if (i >= R) continue;
    const int e = se[i];
    if (e < 0) continue;
    int before = 0, rank = 0, count = 0;
    for (int k = 0; k < R; ++k) {
      const int ek = se[k];
      before += (ek >= 0 && ek < e) ? 1 : 0;
      rank += (ek == e && k < i) ? 1 : 0;
      count += (ek == e) ? 1 : 0;
    }
    const int p = before + rank;
    const int t = i / topk, j = i - t * topk;
    x_row[p] = t;
    if (use_single == 2) {
      if (p < S) {
        int32_t* const tab = slots + (size_t)3 * 3 * S;
        tab[p] = e;
        tab[S + p] = p;
        tab[2 * S + p] = 1;
      }
    } else if (rank == 0) {
      const int cls = (use_single && count == 1) ? 3 : count < split_lo ? 0 : count <= split_mid ? 1 : 2;
      cls_of[p] = (int8_t)cls;
      my_p[u] = p;
      my_e[u] = e;
      my_n[u] = count < kMoeSlotRowsMax ? count : kMoeSlotRowsMax;
    }
    // a slot holds at most 64 rows (an expert gets more only if a token names it twice): the rest contribute nothing
    if (rank >= kMoeSlotRowsMax) continue;
    int ord = 0;
    for (int jj = 0; jj < topk; ++jj) {
      const int ek = se[t * topk + jj];
      ord += (ek >= 0 && (ek < e || (ek == e && jj < j))) ? 1 : 0;
    }
    row_of[t * topk + ord] = p;
    slot_of[t * topk + ord] = j;
  }
  __syncthreads();
  // dense index of an expert inside its class: the experts of that class at earlier sorted positions
#pragma unroll
  for (int u = 0; u < kMoeRouteMax / 256; ++u) {
    const int p = my_p[u];
    if (p < 0) continue;
    const int cls = cls_of[p];
    int idx = 0;
    for (int k = 0; k < p; ++k) idx += cls_of[k] == cls ? 1 : 0;
    if (idx < S) {
      int32_t* const tab = slots + (size_t)cls * 3 * S;
      tab[idx] = my_e[u];
      tab[S + idx] = p;
      tab[2 * S + idx] = my_n[u];
    }
  }
  // positions past the valid entries read token 0 (never used: no slot covers them)
  int valid = 0;
  for (int k = 0; k < R; ++k) valid += se[k] >= 0 ? 1 : 0;
  for (int i = valid + threadIdx.x; i < R; i += blockDim.x) x_row[i] = 0;
}

// out[t, :] accumulates token t's contributions in the order row_of gives (ascending expert), each step rounded to the
// output dtype -- what one moe_scale_add_rows launch per expert leaves in memory between the experts.
template <int DTYPE>
__global__ void moe_combine_rows_kernel(void* __restrict__ out, const void* __restrict__ cur, const void* __restrict__ rw,
                                        int64_t topk, const int32_t* __restrict__ row_of,
                                        const int32_t* __restrict__ slot_of, int64_t T, int64_t H, int64_t R,
                                        bool accumulate) {
  constexpr int PER = DTYPE == WOQ_HIP_ACT_FP32 ? 4 : 8;
  const int64_t chunks = (H + PER - 1) / PER;
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= T * chunks) return;
  const int64_t t = g / chunks, j0 = (g - t * chunks) * PER;
  float o[PER];
  for (int e = 0; e < PER; ++e) o[e] = (accumulate && j0 + e < H) ? load_act(out, DTYPE, t * H + j0 + e) : 0.0f;
  // the contributions in groups of eight: all rows of a group are requested before the first addition, the additions
  // then run in order
  for (int64_t i0 = 0; i0 < topk; i0 += 8) {
    float v[8][PER], w[8];
    bool have[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int64_t r = i0 + i < topk ? (int64_t)row_of[t * topk + i0 + i] : -1;
      have[i] = (uint64_t)r < (uint64_t)R;
      w[i] = have[i] ? load_act(rw, DTYPE, t * topk + slot_of[t * topk + i0 + i]) : 0.0f;
#pragma unroll
      for (int e = 0; e < PER; ++e) v[i][e] = (have[i] && j0 + e < H) ? load_act(cur, DTYPE, r * H + j0 + e) : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (!have[i]) continue;
#pragma unroll
      for (int e = 0; e < PER; ++e) {
        const float s = moe_accumulate<DTYPE>(o[e], v[i][e], w[i]);
        o[e] = DTYPE == WOQ_HIP_ACT_BF16   ? bf16_bits_to_f32(f32_to_bf16_bits(s))
               : DTYPE == WOQ_HIP_ACT_FP16 ? f16_bits_to_f32(f32_to_f16_bits(s))
                                           : s;
      }
    }
  }
  for (int e = 0; e < PER && j0 + e < H; ++e) store_act(out, DTYPE, t * H + j0 + e, o[e]);
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

int launch_moe_route(const int64_t* ids, int64_t T, int64_t topk, int64_t experts, int64_t split_lo, int64_t split_mid,
                     int use_single, int64_t S, int64_t* x_row, int32_t* slots, int32_t* row_of, int32_t* slot_of,
                     hipStream_t st) {
  const int64_t R = T * topk;
  if (R == 0) return 0;
  if (R > kMoeRouteMax) return set_error("moe_route: at most %d (token, slot) entries, got %lld", kMoeRouteMax, (long long)R);
  moe_route_kernel<<<1, 256, 0, st>>>(ids, (int)R, (int)topk, (int)experts, (int)split_lo, (int)split_mid, use_single, (int)S,
                                       x_row, slots, row_of, slot_of);
  return check_launch("moe_route");
}

int launch_moe_combine_rows(void* out, int dtype, int64_t T, int64_t H, const void* cur, const void* rw, int64_t topk,
                            const int32_t* row_of, const int32_t* slot_of, int accumulate, hipStream_t st) {
  if (T == 0 || H == 0 || topk == 0) return 0;
  const int per = dtype == WOQ_HIP_ACT_FP32 ? 4 : 8;
  const unsigned blocks = moe_blocks(T * ((H + per - 1) / per));
  const int64_t R = T * topk;
  if (dtype == WOQ_HIP_ACT_BF16)
    moe_combine_rows_kernel<WOQ_HIP_ACT_BF16><<<blocks, 256, 0, st>>>(out, cur, rw, topk, row_of, slot_of, T, H, R, accumulate != 0);
  else if (dtype == WOQ_HIP_ACT_FP16)
    moe_combine_rows_kernel<WOQ_HIP_ACT_FP16><<<blocks, 256, 0, st>>>(out, cur, rw, topk, row_of, slot_of, T, H, R, accumulate != 0);
  else
    moe_combine_rows_kernel<WOQ_HIP_ACT_FP32><<<blocks, 256, 0, st>>>(out, cur, rw, topk, row_of, slot_of, T, H, R, accumulate != 0);
  return check_launch("moe_combine_rows");
}

}  // namespace woq

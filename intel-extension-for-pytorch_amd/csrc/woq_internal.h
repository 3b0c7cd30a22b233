// Host-side declarations shared by the translation units of libwoq_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/woq_hip.h"

namespace woq {

// Records msg as the thread's last error and returns 1.
int set_error(const char* fmt, ...);
// hipGetLastError() after a launch; records and returns non-zero on failure.
int check_launch(const char* what);

struct Epilogue;

// Arguments common to the floating-point kernels (small-M streaming and tiled GEMM).
// Device-side description of a grouped launch over the experts of a mixture-of-experts layer (woq_hip_moe_group).
struct MoeGroup {
  const int32_t* slot_expert;  // [slots] expert of the slot, or -1: nothing to do
  const int32_t* slot_row0;    // [slots] first routed row of the slot
  const int32_t* slot_rows;    // [slots] its number of rows
  const int64_t* x_row;        // [routed rows] row of x a routed row reads, or null: the routed row itself
  const void* const* qweight;  // [experts] packed weights
  const void* const* scales;   // [experts] scales in the regime's dtype
  const uint8_t* const* zeros; // [experts] or null
  const float* const* bias;    // [experts] or null
};

struct FpArgs {
  const void* x;
  int x_dtype;
  int64_t M, K, N;       // logical sizes
  int64_t NT, KT;        // tiles along N and K of the packed weight
  const uint8_t* qweight;
  const uint16_t* scales;  // fp16 bits (fp16 regime) or bf16 bits (bf16 regime), [NT][KG][16]
  const uint8_t* zeros;    // [NT][KG][16] or nullptr
  // bf16 regime, integer weights, optional: [NT][KG][16] dwords, bf16 scale << 16 | fp16 (1024 + zero) (4-bit
  // weights) or fp16 (stored zero byte) (8-bit weights): one load instead of two per (row, group)
  const uint32_t* szb;
  int64_t G;               // group size in K elements (per-channel: >= padded K)
  int64_t KG;
  const float* bias;
  int fusion;
  const void* other0;
  const void* other1;
  void* out;
  int out_dtype;
  int nf4;  // 4-bit codes index the NF4 table instead of standing for integers (zeros == nullptr)
  int fp8;  // 8-bit weights are float8 e4m3fn bytes, not offset-binary integers (zeros == nullptr)
};

// Split-K scratch of the dequantizing decode kernel: fp32 partial tiles, and one counter per
// row-block set that is zero between launches.
struct SplitKScratch {
  float* partial = nullptr;
  int64_t bytes = 0;
  int* counters = nullptr;
};
// Entries the caller's split-K counter array must have, and the largest number of K splits.
constexpr int kSplitKCounters = 512;
constexpr int kSplitKMax = 4;

int launch_pack_weight(const void* plain, int weight_dtype, int64_t N, int64_t K, void* packed,
                       hipStream_t st);
int launch_unpack_weight(const void* packed, int weight_dtype, int64_t N, int64_t K, void* plain,
                         hipStream_t st);
int launch_pack_qparams(const float* scales, const float* zeros, int weight_dtype, int64_t N, int64_t KG,
                        float* s32, void* s16, void* sb16, uint8_t* z8, uint32_t* sz, uint32_t* szb, hipStream_t st);
int launch_unpack_int4_zeros(const int32_t* zp32, int64_t rows, int64_t cols, int64_t cols_zp32,
                             float* out, hipStream_t st);
int launch_convert_activations(const void* src, int src_dtype, void* dst, int dst_dtype, int64_t count, hipStream_t st);
int launch_shuffle_activations(const void* x, int x_dtype, int64_t M, int64_t K, const int32_t* src, void* out,
                               hipStream_t st);
int launch_shuffle_int4_weight(const void* plain, int64_t N, int64_t K, const int32_t* src, void* out,
                               hipStream_t st);
int launch_moe_gather_rows(const void* x, int x_dtype, int64_t T, int64_t H, const int64_t* rows, int64_t n, void* out,
                           hipStream_t st);
int launch_moe_scale_add_rows(void* out, int dtype, int64_t T, int64_t H, const void* cur, const void* rw, int64_t topk,
                              const int64_t* top_x, const int64_t* idx, int64_t n, hipStream_t st);
int launch_moe_route(const int64_t* ids, int64_t T, int64_t topk, int64_t experts, int64_t split_lo, int64_t split_mid,
                     int use_single, int64_t S, int64_t* x_row, int32_t* slots, int32_t* row_of, int32_t* slot_of,
                     hipStream_t st);
int launch_moe_combine_rows(void* out, int dtype, int64_t T, int64_t H, const void* cur, const void* rw, int64_t topk,
                            const int32_t* row_of, const int32_t* slot_of, int accumulate, hipStream_t st);
int launch_dequant_weight(const void* qweight, int weight_dtype, int64_t N, int64_t K, const float* s32,
                          const uint8_t* z8, int64_t G, void* out, int out_dtype, hipStream_t st);

// Arguments of the fp16-regime decode kernel (4-bit weights, groups that are multiples of 128).
struct DecodeArgs {
  const uint16_t* x;
  int x_dtype;
  int64_t M, K, N, NT, KT, Kpad;
  const uint8_t* qweight;
  const uint32_t* sz;  // [NT][KG][16]: fp16 scale | fp16 (128 + zero) << 16
  int64_t G, KG;
  const float* bias;
  int fusion;
  const void* other0;
  const void* other1;
  void* out;
  int out_dtype;
  int W;
  int tpg_shift;  // log2(G / 128)
  uint32_t wbytes, szbytes;  // extents of qweight and sz: the single-row kernel addresses them with 32-bit offsets
  const MoeGroup* grp;       // GROUPED instances of the single-row kernel: one routed row per slot (blockIdx.z)
};
bool decode_kernel_applies(const FpArgs& f, int wbits, int regime, const uint32_t* sz);
int launch_decode(const FpArgs& f, const uint32_t* sz, hipStream_t st);
// One routed row per slot, the experts' (scale, zero) dword tables in grp->scales.
int launch_decode_grouped(const FpArgs& f, const MoeGroup* grp, int64_t slots, hipStream_t st);

// fp32 compute (woq_fp32.hip): lowp_mode NONE with fp32 activations; fp32 scales, one-byte zero
// points, fp32 output.
struct Fp32Args {
  const float* x;
  int64_t M, K, N, NT, KT;
  const uint8_t* qweight;
  const float* scales;   // [NT][KG][16]
  const uint8_t* zeros;  // [NT][KG][16] or null (symmetric)
  int64_t G, KG;
  const float* bias;
  int fusion;
  const void* other0;
  const void* other1;
  void* out;
  int nf4;
  int fp8;  // 8-bit weights are float8 e4m3fn bytes (symmetric)
};
int launch_fp32(const Fp32Args& f, int wbits, hipStream_t st);

// Decode kernel with per-weight dequantization (woq_decode_dq.hip): 4- or 8-bit weights, M <= 64.
// ntw: weight row-blocks per workgroup (1, 2 or 4), 0 = automatic;
// splits: workgroups that share the K tiles of a row-block set (1, 2 or 4; more than 1 needs the
// scratch and at most 32 rows), 0 = automatic (only together with ntw = 0)
bool decode_dq_applies(const FpArgs& f, int wbits, int regime);
int launch_decode_dq_grouped(const FpArgs& f, int wbits, int regime, const MoeGroup* grp, int64_t slots, hipStream_t st);
int launch_decode_dq(const FpArgs& f, int wbits, int regime, hipStream_t st, int ntw = 0, int splits = 1,
                     const SplitKScratch* scratch = nullptr);
// Bytes of partial-tile scratch that `splits` workgroups per row-block set need.
int64_t decode_dq_splitk_bytes(int64_t M, int64_t NT, int splits);

// regime: 0 = fp16, 1 = bf16 (woq::Regime)
int launch_small_m(const FpArgs& a, int wbits, int regime, hipStream_t st);
int launch_gemm(const FpArgs& a, int wbits, int regime, hipStream_t st);
// Prefill GEMM with register-resident dequantization (woq_gemm_w4.hip): 4-bit integer weights, or
// 8-bit weights with one scale per channel or per group of at least 128
bool gemm_w4_applies(const FpArgs& f, int wbits, int regime);
// shape: row-blocks per wave (7, 4 or 2: 448, 256 or 128 columns per workgroup), 163 / 42 = 256 x 192 /
// 64 x 128 tiles, 0 = by cost model; 8-bit weights: 4, 2, 42 or 0
// splits: workgroups that share the K steps of a tile (64 x 128 shape only; 2 or 4 need the scratch),
// 0 = by problem size, 1 = none
bool gemm_w4s_applies(const FpArgs& f, int wbits, int regime);
int launch_gemm_w4s(const FpArgs& f, int regime, hipStream_t st);
int launch_gemm_w4(const FpArgs& f, int wbits, int regime, hipStream_t st, int shape = 0, int splits = 0,
                   const SplitKScratch* scratch = nullptr);
// Dense bf16 GEMM on the fragment-laid copy that launch_dense_weight writes (woq_gemm_dense.hip): bf16 activations,
// K % 128 == 0; wbits selects the assignment of K values to lanes that the copy was written with;
// shape: row-blocks per wave (7, 4 or 2), 0 = by cost model
bool gemm_dense_applies(const FpArgs& f);
// estimated microseconds of the dense kernel / of launch_gemm_w4's automatic choice on this problem
double gemm_dense_cost(const FpArgs& f);
double gemm_w4_cost(const FpArgs& f, int wbits);
int launch_gemm_dense(const FpArgs& f, const void* dense, int wbits, hipStream_t st, int shape = 0);
int launch_dense_weight(const void* qweight, int weight_dtype, int64_t N, int64_t K, const uint16_t* sb16,
                        const uint8_t* z8, int64_t G, void* out, hipStream_t st);

struct Int8Args {
  const void* x;
  int x_dtype;
  int64_t M, K, N;
  int64_t NT, KT;
  const uint8_t* qweight;
  int wbits;
  const float* scales;   // fp32 [NT][KG][16]
  const uint8_t* zeros;  // [NT][KG][16] or nullptr
  int64_t G, KG;
  int64_t group_size;    // as the caller gave it: <= 0 means one scale per output channel
  const float* bias;
  int act_quant_mode;
  int fusion;
  const void* other0;
  const void* other1;
  void* out;
  int out_dtype;
  void* workspace;
  int64_t workspace_bytes;
  int32_t* split_k_counters;  // optional; with workspace bytes beyond the quantized activations: split K
  int32_t* debug_block_sums;
  int nf4;  // 4-bit codes index the NF4 int8 table; the weight scale is multiplied by fp32(1 / 127)
};

// int8 MFMA kernels that feed the stored codes to the MFMA (woq_gemm_w4i8.hip);
// sa[m * sa_m_stride + (k / qbk) * sa_k_stride] is the activation scale of row m at k, za (asymmetric
// modes, else nullptr) the zero point at the same index, the quantized activations then being q_a - 128.
bool gemm_w4i8_applies(const Int8Args& a, int64_t block_k, int64_t qbk, bool per_k, bool asym);
int launch_gemm_w4i8(const Int8Args& a, const uint8_t* xq, int64_t ldq, const float* sa, int64_t sa_m_stride,
                     int64_t sa_k_stride, int64_t qbk, hipStream_t st, const SplitKScratch* scratch = nullptr,
                     const int32_t* za = nullptr);
// Quantization of whole rows from registers (woq_act_quant.hip): 16-bit activations, padded rows of at
// most 16384 elements.  per_m (one scale per row or per (row, K block)): one pass; scales shared by all
// rows: a statistics pass, then the same kernel with the scales given.  Same bytes and scales as the
// general form in woq_int8.hip.
bool act_quant_rows_applies(const void* x, int x_dtype, int64_t K, const void* q, int64_t ldq, int64_t qbk,
                            bool per_m, bool per_k);
int launch_act_quant_rows(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldq, int64_t qbk, int64_t Kc,
                          bool per_m, bool per_k, bool sym, void* q, float* scales, int32_t* zps, int permute,
                          int offset128, hipStream_t st);
int launch_dynamic_quant(const void* x, int x_dtype, int64_t M, int64_t K, int64_t ldq, int64_t qbk,
                         int mode, void* q, float* scales, int32_t* zps, hipStream_t st);
int launch_int8_linear(const Int8Args& a, hipStream_t st);

}  // namespace woq

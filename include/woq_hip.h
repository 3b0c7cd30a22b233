/*
 * woq_hip.h -- C ABI of the MI355X (gfx950) weight-only-quantized linear library.
 *
 * Every entry point takes plain device pointers, sizes and a hipStream_t (passed as
 * void*).  Nothing here allocates device memory: callers own every buffer, including
 * the workspace that lowp_mode=INT8 needs.  All work is enqueued on the given stream;
 * no entry point synchronises the host.
 *
 * Return value: 0 on success, non-zero on error; woq_hip_last_error() then returns a
 * description (thread-local).  Argument errors are reported before anything is
 * launched, mirroring the TORCH_CHECK behaviour of the reference op
 * (csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:537-543, csrc/cpu/aten/Linear.cpp:574-577).
 *
 * Reference interfaces replaced (paths relative to the reference tree):
 *   woq_hip_pack_weight      <- woq_linear_pack_weight / qlinear_woq_pack
 *                               (csrc/cpu/aten/Linear.cpp:379-438,
 *                                csrc/cpu/aten/kernels/WoqUtilKrnl.cpp:32-249)
 *   woq_hip_unpack_weight    <- woq_linear_unpack_weight / qlinear_woq_unpack
 *                               (csrc/cpu/aten/Linear.cpp:464-495,
 *                                csrc/cpu/aten/kernels/WoqUtilKrnl.cpp:251-324)
 *   woq_hip_pack_qparams     <- ContextLinearWoq constructor: dtype copies and the
 *                               [N, K/G] -> [N/Nb, K/G, Nb] permutation of scales / zero
 *                               points (csrc/cpu/jit/cpu/kernels/ContextLinearWoq.h:37-133)
 *   woq_hip_unpack_int4_zeros<- int32-compressed zero points -> one value per group
 *                               (csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:98-103)
 *   woq_hip_dynamic_quant    <- dynamic_quantize_per_block
 *                               (csrc/cpu/aten/utils/woq_dynamic_quant.h:1526-1750)
 *   woq_hip_linear           <- woq_linear_kernel -> qlinear_woq_affine
 *                               (csrc/cpu/aten/Linear.cpp:499-546,
 *                                csrc/cpu/aten/kernels/WoqLinearKrnl.cpp:56-161) including the
 *                               fused post-ops of woq_linear_unary_kernel /
 *                               woq_linear_binary_kernel (csrc/cpu/aten/Linear.cpp:619-801)
 *   woq_hip_dequant_weight   <- dequantize_woq_weight (csrc/cpu/aten/utils/woq_utils.h:79-163)
 *   woq_hip_convert_activations<- the conversion of bf16 activation rows to the fp16 compute type in front
 *                               of the fp16 kernels (csrc/cpu/aten/utils/woq.h:3076-3079)
 *   woq_hip_shuffle_activations, woq_hip_shuffle_int4_weight
 *                            <- woq_shuffle_tensor_by_group_idx /
 *                               woq_shuffle_weight_back_by_group_idx, the channel shuffles of
 *                               GPTQ act-order (csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:407-421,
 *                               777-954)
 *   woq_hip_moe_gather_rows, woq_hip_moe_scale_add_rows
 *                            <- fuse_index_unsqueeze / fuse_index_mul_index_add, the token gather
 *                               and weighted scatter around the expert linears of mixtral_moe_woq
 *                               (csrc/cpu/aten/kernels/MoEKrnl.cpp:31-160, 254-284)
 */
#ifndef WOQ_HIP_H_
#define WOQ_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* weight dtype, csrc/cpu/aten/utils/woq_defines.h:6-9.  NF4: 4-bit codes into the NormalFloat4 table
 * (csrc/cpu/aten/utils/woq_utils.h:34-51), packed like INT4, symmetric only; under
 * WOQ_HIP_LOWP_INT8 the codes become the int8 table of csrc/cpu/aten/utils/woq.h:628-669. */
#define WOQ_HIP_DTYPE_INT8 1
#define WOQ_HIP_DTYPE_INT4 2
#define WOQ_HIP_DTYPE_NF4 3
/* FP8: float8 e4m3fn bytes, no zero points, not under WOQ_HIP_LOWP_INT8: w = conv(byte) * scale rounded once to
 * the compute type (load_dequant_fp8, csrc/cpu/aten/utils/woq.h:728-741).  conv is the reference kernels'
 * conversion (convert_fp8_e4m3_to_fp32, woq.h:465-485): the float8 value on +-0 and every normal code,
 * (8 + m) * 2^-10 on the subnormal codes 0x01..0x07 (float8: m * 2^-9), +-480 on the NaN codes 0x7F / 0xFF. */
#define WOQ_HIP_DTYPE_FP8 4

/* lowp_mode, csrc/cpu/aten/utils/woq_defines.h:21-24 */
#define WOQ_HIP_LOWP_NONE 0
#define WOQ_HIP_LOWP_FP16 1
#define WOQ_HIP_LOWP_BF16 2
#define WOQ_HIP_LOWP_INT8 3

/* act_quant_mode, csrc/cpu/aten/utils/woq_defines.h:11-19 */
#define WOQ_HIP_QUANT_A_NONE (-1)
#define WOQ_HIP_QUANT_A_PER_TENSOR 0
#define WOQ_HIP_QUANT_A_PER_K_BLOCK 1
#define WOQ_HIP_QUANT_A_PER_M 2
#define WOQ_HIP_QUANT_A_PER_M_K_BLOCK 3
#define WOQ_HIP_QUANT_A_PER_TENSOR_SYM 4
#define WOQ_HIP_QUANT_A_PER_K_BLOCK_SYM 5
#define WOQ_HIP_QUANT_A_PER_M_SYM 6
#define WOQ_HIP_QUANT_A_PER_M_K_BLOCK_SYM 7

/* fused post-op, csrc/cpu/aten/utils/woq_defines.h:27-36 */
#define WOQ_HIP_FUSE_NONE 0x0
#define WOQ_HIP_FUSE_GELU_ERF 0x1
#define WOQ_HIP_FUSE_GELU_TANH 0x2
#define WOQ_HIP_FUSE_RELU 0x3
#define WOQ_HIP_FUSE_SILU 0x4
#define WOQ_HIP_FUSE_ADD 0x10
#define WOQ_HIP_FUSE_ADD_ADD 0x20
#define WOQ_HIP_FUSE_MUL 0x30

/* element types of activations / outputs */
#define WOQ_HIP_ACT_FP32 0
#define WOQ_HIP_ACT_FP16 1
#define WOQ_HIP_ACT_BF16 2

/* Tile geometry of the packed layouts (see woq_hip_pack_weight). */
#define WOQ_HIP_TILE_N 16      /* output rows per tile                     */
#define WOQ_HIP_TILE_BYTES 1024 /* one tile = one dwordx4 load per lane of a wave64 */
#define WOQ_HIP_TILE_K_INT4 128 /* K values per tile row, 4-bit weights    */
#define WOQ_HIP_TILE_K_INT8 64  /* K values per tile row, 8-bit weights    */

const char* woq_hip_last_error(void);

/* ABI version; bumped whenever a struct or a layout below changes. */
int woq_hip_abi_version(void);

/* Rows below which lowp_mode BF16 computes in fp16 (the reference's fp16 kernel) instead of bf16: the value of the
 * environment's IPEX_WOQ_SMALL_BATCH_THRESHOLD when the library first needed it, 5 by default
 * (csrc/cpu/aten/utils/woq.h:24, csrc/cpu/aten/kernels/WoqLinearKrnl.cpp:77, 93). */
int woq_hip_small_batch_threshold(void);

/* Name of the kernel the calling thread enqueued last through any entry point below ("" before the
 * first launch), e.g. "woq_gemm_w4i8_kernel": lets a test or a profile script state which kernel served
 * a call.  No counterpart in the reference, whose kernel choice is visible only in its dispatch code
 * (csrc/cpu/aten/kernels/WoqLinearKrnl.cpp:56-161). */
const char* woq_hip_last_kernel(void);

/* Padded extents of the packed layout: N up to a multiple of 16, K up to a multiple of
 * the tile K extent.  packed bytes = Np/16 * Kp/tile_k * 1024. */
int64_t woq_hip_padded_n(int64_t N);
int64_t woq_hip_padded_k(int weight_dtype, int64_t K);
int64_t woq_hip_packed_weight_bytes(int weight_dtype, int64_t N, int64_t K);

/*
 * Plain -> packed.
 *   INT4 / NF4: plain is uint8 [N, ceil(K/2)], byte j of a row holds element 2j in the
 *               low nibble and 2j+1 in the high nibble
 *               (intel_extension_for_pytorch/quantization/_quantize_utils.py:1184).
 *   INT8:       plain is int8 [N, K].
 *   FP8:        plain is the float8 e4m3fn bytes [N, K].
 * Packed layout (the same bytes serve the small-M kernel, the MFMA GEMM and the int8 path):
 *   tiles [Np/16][Kp/tile_k], 1024 bytes each, K-tiles of one row block contiguous.
 *   Lane l = r + 16*c of a wave64 owns bytes [16*l, 16*l+16) of a tile: output row
 *   n0 + r, and
 *     INT4: K offsets 32*c .. 32*c+31 as 4 dwords; dword j holds offsets 8*j .. 8*j+7 with
 *           element e stored in nibble position (e even ? e/2 : 4 + e/2), so that
 *           (dword >> 4*v) & 0x000F000F yields elements (2v, 2v+1) in the two 16-bit halves;
 *     INT8: K offsets 16*c .. 16*c+15, one per byte, stored offset-binary (value + 128).
 *     FP8:  the same places, the bytes as they are.
 *   Padding rows / columns hold zero-weight encodings and never contribute.
 */
int woq_hip_pack_weight(const void* plain, int weight_dtype, int64_t N, int64_t K,
                        void* packed, void* stream);

/* Exact inverse of woq_hip_pack_weight (padding dropped). */
int woq_hip_unpack_weight(const void* packed, int weight_dtype, int64_t N, int64_t K,
                          void* plain, void* stream);

/*
 * Quantization parameters -> kernel layout.
 *   scales: fp32 [N, KG] (KG = number of K groups; 1 for per-channel)
 *   zeros : fp32 [N, KG] or NULL (symmetric).  Must be integral, in [0,127] for 4-bit and
 *           [-128,127] for 8-bit weights (checked by the host wrapper).
 * Outputs are laid out [Np/16][KG][16] (row-in-tile fastest):
 *   scales_f32 / scales_f16 / scales_bf16: the three roundings the reference keeps
 *   (ContextLinearWoq.h:104-106); zeros_u8: zero point as one byte, the value itself for
 *   4-bit weights and value + 128 for 8-bit weights (the same offset-binary shift as the
 *   weight bytes, so stored_weight - stored_zero == q - z in both cases).
 *   scale_zero_f16x2 (may be NULL): one dword per (row, group) for the decode kernel, low half =
 *   fp16 scale, high half = fp16 (128 + zero point) (symmetric 4-bit weights: 128 + 8); only
 *   meaningful for 4-bit weights.
 *   scale_zero_bf16 (may be NULL): one dword per (row, group) for the bf16 kernels on integer weights
 *   (INT4, INT8), so that they load a group's parameters with one request: high half = bf16 scale (the
 *   rounding of scales_bf16), low half = an fp16 number, 1024 + zero point for 4-bit weights (symmetric:
 *   1024 + 8; the kernels read a nibble q as the fp16 number 1024 + q), the stored byte of zeros_u8 for
 *   8-bit weights (symmetric: 128).  No counterpart in the reference, which keeps scales and zero points
 *   in separate tensors (ContextLinearWoq.h:104-133).
 * Padding rows get scale 1, zero 0 (LinearWoqPacked.cpp:344-361).
 */
int woq_hip_pack_qparams(const float* scales, const float* zeros, int weight_dtype, int64_t N,
                         int64_t KG, float* scales_f32, void* scales_f16, void* scales_bf16,
                         uint8_t* zeros_u8, uint32_t* scale_zero_f16x2, uint32_t* scale_zero_bf16,
                         void* stream);

/* zp[i][j] = (zp32[i][j/8] >> (4*(j%8))) & 0xf, written as fp32 [rows, cols]. */
int woq_hip_unpack_int4_zeros(const int32_t* zp32, int64_t rows, int64_t cols,
                              int64_t cols_zp32, float* out, void* stream);

/*
 * Dynamic activation quantization.
 *   x: [M, K] (x_dtype), q: int8 (symmetric modes 4..7) or uint8 (asymmetric 0..3) [M, K],
 *   scales: fp32, zps: int32 (asymmetric only, may be NULL for symmetric modes); shapes
 *   per mode: per-tensor [1], per-K-block [Kc], per-M [M], per-M-K-block [M, Kc] with
 *   Kc = ceil(K / quant_block_k).
 *   scale = max(|max|,|min|)/127 (sym) or (max-min)/255 (asym); q = clamp(rint(x/scale + zp)).
 */
int woq_hip_dynamic_quant(const void* x, int x_dtype, int64_t M, int64_t K,
                          int64_t quant_block_k, int act_quant_mode, void* q, float* scales,
                          int32_t* zps, void* stream);

typedef struct woq_hip_linear_params {
  uint32_t struct_size; /* sizeof(woq_hip_linear_params), checked */

  /* activations, row-major [M, K], 16-byte aligned rows (K % 8 == 0) */
  const void* x;
  int32_t x_dtype; /* WOQ_HIP_ACT_* */
  int64_t M, K, N;

  /* packed weight + parameters (woq_hip_pack_weight / woq_hip_pack_qparams) */
  const void* qweight;
  int32_t weight_dtype; /* WOQ_HIP_DTYPE_* */
  const float* scales_f32;
  const void* scales_f16;
  const void* scales_bf16;
  const uint8_t* zeros_u8; /* NULL: symmetric weights */
  const uint32_t* scale_zero_f16x2; /* from woq_hip_pack_qparams; NULL disables the decode kernel */
  const uint32_t* scale_zero_bf16;  /* from woq_hip_pack_qparams, optional: with it the bf16 kernels on INT4 /
                                     * INT8 weights load one dword per (row, group) instead of a scale and a zero
                                     * point; results are the same bit for bit */
  const void* dense_bf16;   /* from woq_hip_dense_weight, optional (cache_weight_for_large_batch): with it, lowp_mode
                             * BF16 on bf16 activations runs batches of at least woq_hip_weight_cache_batch_threshold()
                             * rows on the dense copy where that is the faster kernel; same results */
  int64_t group_size;       /* <= 0: per output channel */
  const float* bias;        /* fp32 [N] or NULL */

  int32_t lowp_mode;      /* WOQ_HIP_LOWP_* */
  int32_t act_quant_mode; /* WOQ_HIP_QUANT_A_*, used when lowp_mode == INT8 */

  /* fused post-op; others[i] is [M, N] in x_dtype */
  int32_t fusion;
  const void* others[2];

  /* output [M, N]; out_dtype = x_dtype, or WOQ_HIP_ACT_FP32 to receive the fp32
   * accumulator (bias added, no output rounding, no post-op) for parity checks, or -- without a
   * post-op -- the other 16-bit type: the result in the compute type's rounding, cast to it (fp16 rows
   * made by woq_hip_convert_activations from a bf16 tensor under lowp_mode FP16, bf16 output) */
  void* out;
  int32_t out_dtype;

  /* workspace: for lowp_mode == INT8 the quantized activations (size from
   * woq_hip_linear_workspace_bytes), optionally followed by split-K scratch (round that size up to a
   * multiple of 256 and add woq_hip_linear_split_k_workspace_bytes); for the other modes, optional
   * split-K scratch alone (size from woq_hip_linear_split_k_workspace_bytes).  Contents undefined
   * before and after the call */
  void* workspace;
  int64_t workspace_bytes;

  /* optional, with the split-K scratch: 512 int32 counters that are zero when the call is enqueued
   * and are zero again when its work has finished (allocate and zero them once; calls that may run
   * at the same time, e.g. on different streams, need arrays of their own).  NULL: K is never split
   * across workgroups.  No counterpart in the reference, whose threads share the activations in cache. */
  int32_t* split_k_counters;

  /* optional, lowp_mode == INT8 only: receives the exact int32 sum of every
   * (m, n, K-block) as int32 [M, N, Kp/block_k] (tests only, small shapes) */
  int32_t* debug_block_sums;

  /* force_kernel: 0 = automatic; 1 = small-M streaming kernel; 2 = tiled MFMA GEMM (any shape);
   * 3 = prefill GEMM with register-resident dequantization (4-bit integer weights, or 8-bit weights with
   * groups of at least 128; K % 128 == 0, power-of-two or per-channel groups, x in the compute dtype),
   * workgroup shape by cost model; 4 / 5 / 6 = the same kernel with 448 / 256 / 128 columns per workgroup;
   * 7 = dequantizing decode kernel (M <= 64, K % 128 == 0 for 4-bit and K % 64 == 0 for 8-bit weights, x in the
   * compute dtype), 8 / 9 / 10 = the same with one / two / four weight row-blocks per workgroup;
   * 11 / 12 = the same prefill GEMM with 256 rows x 192 columns / 64 rows x 128 columns per workgroup
   * (8-bit weights: 5, 6 and 12 only);
   * 13..17 = the dequantizing decode kernel (M <= 32) with (row-blocks per workgroup, K splits) =
   * (1, 2), (2, 2), (4, 2), (2, 4), (4, 4): needs workspace and split_k_counters;
   * 19 / 20 = the prefill GEMM with 64 x 128 tiles and K shared by two / four workgroups per tile (same needs);
   * 21 = prefill GEMM that dequantizes each weight once per workgroup into an LDS tile (256 rows x 224 columns,
   * 8 waves; 4-bit integer weights, otherwise the conditions of 3);
   * 22 = the dequantizing decode kernel (M <= 32, INT4 / INT8 weights) with three weight row-blocks per workgroup,
   * which need not divide the row-blocks;
   * 23 = dense bf16 GEMM on dense_bf16 (lowp_mode BF16, bf16 activations, K % 128 == 0; any M), workgroup shape by
   * cost model; 24 / 25 / 26 = the same with 448 / 256 / 128 columns per workgroup.
   * NF4 weights: 0, 1, 2, 7, 8, 9, 13, 14, 16 and 23..26 only.
   * fp32 compute (lowp_mode NONE with fp32 activations, csrc/cpu/aten/kernels/WoqLinearKrnl.cpp:142-158;
   * also lowp_mode INT8 on fp32 activations) has one kernel of its own and takes 0 only */
  int32_t force_kernel;

  void* stream;
} woq_hip_linear_params;

int64_t woq_hip_linear_workspace_bytes(int64_t M, int64_t K, int32_t lowp_mode,
                                       int32_t act_quant_mode, int64_t group_size);

/* Scratch bytes that let woq_hip_linear split K across workgroups for M rows and N output columns
 * in the floating-point modes (decode kernel up to 32 rows; prefill GEMM when its 64 x 128 tiles are
 * at most 128); 0 where it never does.  No counterpart in the reference. */
int64_t woq_hip_linear_split_k_workspace_bytes(int64_t M, int64_t N);

/* The same size for the problems on which woq_hip_linear shares K between workgroups BY ITSELF (force_kernel 0):
 * few output tiles and a long K -- 5..32 rows with K >= 8192 and N <= 4096 in the floating-point modes, more than
 * 64 rows with K >= 4096 and M * N <= 2^20 in every mode -- and 0 for every other problem, where scratch and
 * counters would go unused.  A caller that allocates per call asks this function; there is no second copy of the
 * rule to keep in step.  No counterpart in the reference. */
int64_t woq_hip_linear_auto_split_k_workspace_bytes(int64_t M, int64_t K, int64_t N, int32_t lowp_mode);

/* K-block of the int8 path: min(group_size, 128), per-channel -> 128
 * (get_block_k, csrc/cpu/aten/Linear.cpp:362-376). */
int64_t woq_hip_int8_block_k(int64_t group_size, int64_t K);

int woq_hip_linear(const woq_hip_linear_params* p);

/* woq_hip_linear for callers that cannot allocate and hold no workspace: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference, whose kernels
 * take their temporaries from the CPU heap.  Same arguments and results as woq_hip_linear, except that
 * workspace, workspace_bytes and split_k_counters must be NULL / 0: the quantized activations of
 * lowp_mode INT8 and the split-K scratch live in an array that the library keeps resident on every GPU it
 * runs on (WOQ_HIP_NOALLOC_MAX_WORKSPACE_BYTES plus 2 KiB of counters, until the process ends).  A call
 * whose workspace need (woq_hip_linear_workspace_bytes) exceeds that maximum is rejected with an error
 * before anything is launched; K is shared between workgroups only while that scratch fits as well.
 * Allocates nothing, on the device or through any library.  All calls on one GPU share the array: calls
 * that may overlap in time on one GPU (different streams, concurrent graph launches) race and must be
 * serialised by the caller.  The first call on a device that needs the array looks up its address, which cannot
 * happen under stream capture: such a call is rejected, so make one call on the device before capturing. */
#define WOQ_HIP_NOALLOC_MAX_WORKSPACE_BYTES (12 * 1024 * 1024)
int woq_hip_linear_noalloc(const woq_hip_linear_params* p);

/* Packed weight -> dense [N, K] in out_dtype (fp32: (q - z) * s exactly; fp16 / bf16: that
 * value rounded to nearest even).  Used by the weight cache and by tests. */
int woq_hip_dequant_weight(const void* qweight, int weight_dtype, int64_t N, int64_t K,
                           const float* scales_f32, const uint8_t* zeros_u8,
                           int64_t group_size, void* out, int out_dtype, void* stream);

/* Dense bf16 copy of a packed weight for large batches: what the reference caches under
 * cache_weight_for_large_batch with lowp_mode BF16 (csrc/cpu/jit/cpu/kernels/LinearWoqPacked.cpp:430-486: the weight
 * dequantized with the bf16 scales, w = bf16((q - z) * s), blocked for its GEMM; :511-526 uses it for at least
 * IPEX_WOQ_WEIGHT_CACHE_BATCH_THRESHOLD rows).  Here the copy is laid out as the MFMA operands of the dense kernel
 * ([K / 128][padded N / 16][4][64] fragments of 16 bytes), four times the packed 4-bit bytes.
 * woq_hip_dense_weight_bytes: size of the copy, or 0 where none can be made (K not a multiple of 128, or a copy of
 * 2 GiB and more).  woq_hip_dense_weight: writes it from the packed weight, the bf16 scales and the zero point
 * bytes of woq_hip_pack_qparams.  woq_hip_weight_cache_batch_threshold: rows from which woq_hip_linear uses the
 * copy, the environment's IPEX_WOQ_WEIGHT_CACHE_BATCH_THRESHOLD when the library first needed it, 64 by default
 * (LinearWoqPacked.cpp:17-18). */
int64_t woq_hip_dense_weight_bytes(int32_t weight_dtype, int64_t N, int64_t K);
int woq_hip_dense_weight(const void* qweight, int32_t weight_dtype, int64_t N, int64_t K, const void* scales_bf16,
                         const uint8_t* zeros_u8, int64_t group_size, void* dense, void* stream);
int woq_hip_weight_cache_batch_threshold(void);

/* dst[i] = src[i] converted, round to nearest even; dtypes WOQ_HIP_ACT_*; count elements.  With it a
 * caller runs lowp_mode FP16 on a bf16 tensor of any number of rows through the fp16 kernels: convert
 * the rows once, call woq_hip_linear with x_dtype FP16 and out_dtype BF16 (up to 16 rows woq_hip_linear
 * converts on the way into LDS by itself). */
int woq_hip_convert_activations(const void* src, int src_dtype, void* dst, int dst_dtype, int64_t count,
                                void* stream);

/* GPTQ act-order.  src[p] (int32, K entries, a permutation of 0..K-1) is the input channel that
 * belongs at position p once the channels are sorted by group (stable in the channel index).
 *   shuffle_activations: out[m, p] = x[m, src[p]], x and out [M, K] in x_dtype.
 *   shuffle_int4_weight: the same on plain int4 rows [N, (K + 1) / 2] (low nibble = even index);
 *   with the inverse permutation it restores the checkpoint order. */
int woq_hip_shuffle_activations(const void* x, int x_dtype, int64_t M, int64_t K, const int32_t* src,
                                void* out, void* stream);
int woq_hip_shuffle_int4_weight(const void* plain, int64_t N, int64_t K, const int32_t* src, void* out,
                                void* stream);

/* Mixture of experts over WOQ linears (csrc/cpu/aten/kernels/MoEKrnl.cpp:254-284): the rows of the
 * tokens routed to one expert, and the weighted accumulation of the expert's output.
 *   gather_rows:    out[i, :] = x[rows[i], :], x [T, H] and out [n, H] in x_dtype, rows int64 on the device.
 *   scale_add_rows: out[top_x[i], :] += routing_weights[top_x[i], idx[i]] * expert_out[i, :] for i < n;
 *                   out [T, H], expert_out [n, H], routing_weights [T, topk], all in `dtype`; bf16 and
 *                   fp32 form product and sum in fp32 (one rounding), fp16 rounds the product first.
 *                   The entries of top_x must be distinct (a token reaches an expert at most once: two rows
 *                   for one token would race on its output row).
 * Indices outside [0, T) (rows, top_x) or [0, topk) (idx) are not an error the kernels can report: such a
 * row is skipped -- gather_rows leaves zeros, scale_add_rows adds nothing -- instead of faulting. */
int woq_hip_moe_gather_rows(const void* x, int x_dtype, int64_t T, int64_t H, const int64_t* rows, int64_t n,
                            void* out, void* stream);
int woq_hip_moe_scale_add_rows(void* out, int dtype, int64_t T, int64_t H, const void* expert_out,
                               const void* routing_weights, int64_t topk, const int64_t* top_x, const int64_t* idx,
                               int64_t n, void* stream);

/*
 * A whole mixture-of-experts layer without reading the routing on the host (deepseek_moe_woq, csrc/cpu/aten/MoE.cpp:290-328,
 * whose expert loop runs on the host because its tensors live there).
 *
 * woq_hip_moe_route: topk_ids int64 [T, topk] on the device -> the (token, slot) entries sorted by expert, stable, so
 *   that inside an expert the tokens ascend (get_expert_topx_idx, MoE.cpp:64-81).  x_row[p] (T * topk entries, at most
 *   WOQ_HIP_MOE_ROUTE_MAX) = token of the entry at sorted position p.  slots: int32 [4][3][S], S >= min(T * topk, experts):
 *   per size class the experts that have tokens, densely from index 0 in ascending expert order, as three arrays --
 *   expert id (-1: unused entry), first sorted position, number of rows (at most 64).  Classes: 0 fewer than split_lo
 *   rows, 1 at most split_mid, 2 more, 3 (use_single = 1) exactly one row, taken out of class 0.  use_single = 2:
 *   every sorted position is a slot of one row in class 3, at its own index (S >= T * topk; for a single token).
 *   row_of[t, i] / slot_of[t, i] = sorted position and top-k slot of token t's i-th contribution in ascending expert
 *   order (row_of -1: none).  An expert id outside [0, experts) contributes nothing, and neither do an expert's entries
 *   beyond its first 64 (a slot holds at most 64 rows).
 * woq_hip_linear_grouped: one linear of every expert that has a slot, in one launch.  p describes one expert's problem
 *   (all experts share N, K, group size, weight dtype INT4 or INT8, lowp_mode NONE / FP16 / BF16, post-op none / silu /
 *   mul) with M = the bound on a slot's rows (1..64; it selects the compute type like woq_hip_linear's M, so a layer
 *   under lowp_mode BF16 takes one call with M = 4 on the slots of experts with fewer than five rows and one with a
 *   larger M on the others; M <= 16 and M > 16 also select a kernel with one or four row tiles, hence the size classes); p's weight, scale, zero
 *   point and bias pointers are ignored -- except that a non-NULL scale_zero_f16x2 says that the group's scales table
 *   holds the experts' (fp16 scale, fp16 128 + zero) dword tables: the call then runs the single-row decode kernel
 *   (M must be at most 4: the classes of experts with exactly one row and with fewer than five; 4-bit weights in groups of 32, 64 or 128 * 2^k, K a multiple of 256,
 *   fp16 compute).  x: the rows the slots read, out / others[0]: [routed rows, N].  group: DEVICE
 *   pointer to a woq_hip_moe_group.  Rows of a slot are row0 .. row0 + rows - 1 of out; they read row x_row[row] of x,
 *   or the same row when x_row is NULL.  Needs what the dequantizing decode kernel needs: K a multiple of the weight tile,
 *   a power-of-two or per-channel group size, an even number of 16-column blocks, rows in the compute type (bf16 rows
 *   under fp16 compute: at most 16 per slot).
 * woq_hip_moe_combine_rows: out[t, :] (accumulate != 0: its value; else zero) plus token t's contributions in row_of's order of
 *   routing_weights[t, slot] * expert_out[row, :], added in row_of's order and rounded to the dtype after every addition: bit for bit what one
 *   woq_hip_moe_scale_add_rows call per expert, experts ascending, leaves.
 */
#define WOQ_HIP_MOE_ROUTE_MAX 2048
typedef struct woq_hip_moe_group {
  const int32_t* slot_expert;      /* [slots] expert of the slot or -1 */
  const int32_t* slot_row0;        /* [slots] */
  const int32_t* slot_rows;        /* [slots] */
  const int64_t* x_row;            /* [routed rows] or NULL */
  const void* const* qweight;      /* [experts] packed weights */
  const void* const* scales;       /* [experts] scales in the compute type of the call (fp16 or bf16 layout of woq_hip_pack_qparams) */
  const uint8_t* const* zeros_u8;  /* [experts] or NULL (symmetric) */
  const float* const* bias;        /* [experts] or NULL */
} woq_hip_moe_group;
int woq_hip_moe_route(const int64_t* topk_ids, int64_t T, int64_t topk, int64_t experts, int64_t split_lo,
                      int64_t split_mid, int use_single, int64_t S, int64_t* x_row, int32_t* slots, int32_t* row_of,
                      int32_t* slot_of, void* stream);
int woq_hip_linear_grouped(const woq_hip_linear_params* p, const void* group, int64_t slots);
int woq_hip_moe_combine_rows(void* out, int dtype, int64_t T, int64_t H, const void* expert_out,
                             const void* routing_weights, int64_t topk, const int32_t* row_of, const int32_t* slot_of,
                             int accumulate, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* WOQ_HIP_H_ */

/* llmk.h -- C ABI of libllmk_gfx950.so: MI355X (gfx950) kernels for the quantized-GEMM
 * path of Jzz24/LLM_Kernels.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless stated; the library never allocates,
 *     frees or synchronises; work is enqueued on `stream` (a hipStream_t, NULL = default).
 *   - return value: 0 on success, negative LLMK_ERR_* otherwise; llmk_last_error()
 *     gives a thread-local message.
 *   - matrices are row-major and contiguous.  dtype codes: LLMK_F32/F16/BF16.
 *   - "ref:" comments cite the file:line of the reference interface each entry replaces.
 */
#ifndef LLMK_H
#define LLMK_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LLMK_OK          0
#define LLMK_ERR_SHAPE  (-1)   /* shape / alignment precondition violated                */
#define LLMK_ERR_DTYPE  (-2)   /* unsupported dtype / mode code                          */
#define LLMK_ERR_LAUNCH (-3)   /* hipGetLastError() reported a launch failure            */
#define LLMK_ERR_ARG    (-4)   /* null pointer or inconsistent argument                  */

#define LLMK_F32  0
#define LLMK_F16  1
#define LLMK_BF16 2

/* rounding rules of the three reference quantizers */
#define LLMK_ROUND_HALF_AWAY 0 /* libdevice.round   ref: quantization/int8_kernel.py:27,84          */
#define LLMK_ROUND_HALF_UP   1 /* floor(v + 0.5)    ref: quantization/w4a8_kernel.py:164,222        */

/* element kinds of the grouped GEMM */
#define LLMK_KIND_I8   0       /* int8 x int8, 128x128 / 1x128 block scales (fp16 or fp32 scales)    */
#define LLMK_KIND_FP8  1       /* e4m3 x e4m3, block scales fp32                                      */
#define LLMK_KIND_F16  2       /* fp16 x fp16, no scales                                              */
#define LLMK_KIND_BF16 3       /* bf16 x bf16, no scales                                              */

int         llmk_version(void);
const char* llmk_last_error(void);
/* Bytes of scratch llmk_gemm_fp8_block / _i8_block / _w4a8 / llmk_grouped_gemm can use for this shape
 * (0 = none; M = all rows of a grouped launch).  The scratch is optional: without it, or with less of it, a
 * slower kernel variant runs.  For M > 512 and K >= 8192 it ends with 64 MiB for the partial sums of a split
 * last round of tiles (shorter K is never split there). */
int64_t     llmk_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);

/* ------------------------------------------------------------------ bit packing
 * ref: quantization/bitpack.py:228-293 (pack rows), :84-149 (pack cols),
 *      :308-373 (unpack rows), :163-226 (unpack cols); aliases :376-379.
 * in_bytes: element size of the unpacked matrix (1, 2, 4 or 8; little endian integers).
 * pack_bits in {8,16,32,64}, nbits in {1,2,4,8}; e = pack_bits / nbits.
 * pack rows:  out[r, c] = OR_i (in[r*e+i, c] << i*nbits), in [rows_out*e, cols]
 * pack cols:  out[r, c] = OR_i (in[r, c*e+i] << i*nbits), in [rows, cols_out*e]
 * unpack:     (packed >> i*nbits) & mask, written as out_bytes-wide integers.      */
int llmk_pack_rows(const void* in, int in_bytes, void* out, int64_t rows_out, int64_t cols,
                   int nbits, int pack_bits, void* stream);
int llmk_pack_cols(const void* in, int in_bytes, void* out, int64_t rows, int64_t cols_out,
                   int nbits, int pack_bits, void* stream);
int llmk_unpack_rows(const void* packed, int pack_bits, void* out, int out_bytes,
                     int64_t rows_packed, int64_t cols, int nbits, int e, void* stream);
int llmk_unpack_cols(const void* packed, int pack_bits, void* out, int out_bytes,
                     int64_t rows, int64_t cols_packed, int nbits, int e, void* stream);

/* ------------------------------------------------------------------ quantizers
 * 1 x block activation groups (block = 128 in every reference call).
 * ref: quantization/fp8_kernel.py:9-52   -> llmk_act_quant_fp8  (s fp32 [n_groups])
 *      quantization/int8_kernel.py:9-56  -> llmk_act_quant_i8, LLMK_ROUND_HALF_AWAY (s fp16)
 *      quantization/w4a8_kernel.py:145-193 -> llmk_act_quant_i8, LLMK_ROUND_HALF_UP          */
int llmk_act_quant_fp8(const void* x, int x_dtype, void* y_e4m3, float* s, int64_t n_groups,
                       int block, void* stream);
int llmk_act_quant_i8(const void* x, int x_dtype, int8_t* y, void* s_f16, int64_t n_groups,
                      int block, int round_mode, void* stream);

/* One group per row of x [rows, cols] (any cols >= 1): s[row] = max|x[row]| / 127 in fp32 (stored fp32),
 * y = round-half-away(x / s) int8.  The per-token activation / per-output-channel weight quantizer of the
 * W8A8 scheme with one scale per row; the reference has no function of this shape, its nearest relative is
 * the 1 x 128 group kernel quantization/int8_kernel.py:9-31 (same arithmetic, group = whole row). */
int llmk_quant_i8_rowwise(const void* x, int x_dtype, int8_t* y, float* s, int64_t rows, int64_t cols,
                          void* stream);

/* block x block weight quantizers over W [M, N].
 * ref: quantization/int8_kernel.py:59-113 (qmax 127, half-away, no clamp)
 *      quantization/w4a8_kernel.py:196-225 (qmax 119, half-up, clamp +-119)
 * fp8: s = blockmax/448 fp32; the reference has no fp8 weight quantizer (analogue of the above). */
int llmk_weight_quant_i8_block(const void* x, int x_dtype, int8_t* y, void* s_f16, int64_t M,
                               int64_t N, int block, float qmax, int round_mode, int clamp,
                               void* stream);
int llmk_weight_quant_fp8_block(const void* x, int x_dtype, void* y_e4m3, float* s, int64_t M,
                                int64_t N, int block, void* stream);
/* second level of the w4a8 weight quantizer, in place on the int8 matrix y [M,N]:
 * per (row, group): s4 = floor((max-min)/15+.5), z4 = floor(-min/s4+.5),
 * y <- clamp(floor(y/s4+.5)+z4, 0, 15).   ref: quantization/w4a8_kernel.py:228-262 */
int llmk_weight_quant_w4a8_level2(int8_t* y, int8_t* s4, int8_t* z4, int64_t M, int64_t N,
                                  int group, void* stream);

/* dequantizers: y = fp32(x) * s[block]  ref: fp8_kernel.py:55-105, int8_kernel.py:116-166 */
int llmk_weight_dequant_fp8_block(const void* x_e4m3, const float* s, void* y, int y_dtype,
                                  int64_t M, int64_t N, int block, void* stream);
int llmk_weight_dequant_i8_block(const int8_t* x, const void* s, int s_dtype, void* y, int y_dtype,
                                 int64_t M, int64_t N, int block, void* stream);
/* packed [N/8, K] int32 (8 rows per word) -> fp16 [N, K]: ((q - z4) * s4 in int8) * s
 * ref: quantization/w4a8_kernel.py:16-142 */
int llmk_weight_dequant_w4a8(const int32_t* packed, const void* s_f16, const int8_t* s4,
                             const int8_t* z4, void* y_f16, int64_t N, int64_t K, int block,
                             int group, void* stream);

/* ------------------------------------------------------------------ dense quantized GEMMs
 * C[M,N] = sum_kb dot_kb(A, B) * a_s[m, kb] * b_s[n / 128, kb], K % 128 == 0, any M, N >= 1.
 * A [M,K], B [N,K] both K-contiguous.  c_dtype selects the epilogue (torch default dtype).
 * workspace/workspace_bytes: optional scratch of llmk_gemm_workspace_bytes(M, N, K) bytes (fp32 activation
 * scales for large M, fp32 partial sums of the split-K / K-range variants); NULL/0 -> single-pass variants.
 * ref: quantization/fp8_kernel.py:113-191 (a_s, b_s fp32)                                   */
int llmk_gemm_fp8_block(const void* a_e4m3, const float* a_s, const void* b_e4m3, const float* b_s,
                        void* c, int c_dtype, int64_t M, int64_t N, int64_t K,
                        void* workspace, int64_t workspace_bytes, void* stream);
/* llmk_gemm_fp8_block for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same operands as
 * llmk_gemm_fp8_block, but the scratch is a device array built into the library (LLMK_STATIC_SCRATCH_BYTES per
 * GPU, held until the process ends); the call itself allocates and frees nothing.  The array serves the
 * activation scales / split-K / K-range partial sums, not the optional 64 MiB of a split last round of tiles:
 * results equal llmk_gemm_fp8_block with a workspace of llmk_gemm_workspace_bytes(M, N, K) bytes bit for bit
 * whenever that size holds no such 64 MiB (M <= 512 or K < 8192); beyond that the workspace entry may split its
 * last round of tiles along K and the two differ in the fp32 summation order only (same tolerance against the
 * oracle).  Shapes whose scratch exceeds the array fail with LLMK_ERR_SHAPE.  All calls on one GPU share
 * the array: calls that may overlap on different streams of that GPU race, issue them on one stream. */
#define LLMK_STATIC_SCRATCH_BYTES (32 << 20)
int llmk_gemm_fp8_block_static(const void* a_e4m3, const float* a_s, const void* b_e4m3, const float* b_s,
                               void* c, int c_dtype, int64_t M, int64_t N, int64_t K, void* stream);
/* ref: quantization/int8_kernel.py:174-257 (scales fp16 in the reference; s_dtype F16/BF16/F32) */
int llmk_gemm_i8_block(const int8_t* a, const void* a_s, const int8_t* b, const void* b_s,
                       int s_dtype, void* c, int c_dtype, int64_t M, int64_t N, int64_t K,
                       void* workspace, int64_t workspace_bytes, void* stream);
/* per-token x per-channel W8A8 with one full-K int32 accumulation (a scheme with
 * no counterpart function in the reference).  c may be NULL; c_i32 (raw accumulators) may be NULL.
 * M <= 64 streams the weights once; larger M runs on the MFMA tile kernels (int32 accumulation inside
 * the MFMA, c = float(acc) * a_s[m] * b_s[n] in the epilogue of either path).  With a workspace of
 * llmk_gemm_workspace_bytes(M, N, K), shapes with few tiles and a long K are split along K; the slices' int32 sums
 * are added as integers before the scaling, so c and c_i32 do not depend on the split. */
int llmk_gemm_i8_rowcol(const int8_t* a, const float* a_s, const int8_t* b, const float* b_s,
                        void* c, int c_dtype, int32_t* c_i32, int64_t M, int64_t N, int64_t K,
                        void* workspace, int64_t workspace_bytes, void* stream);
/* b packed [N/8, K] int32, nibble (n % 8) of word [n/8, k]; b8 = int8((q - z4[n,kg]) * s4[n,kg]).
 * ref: quantization/w4a8_kernel.py:317-448 */
/* workspace: llmk_gemm_w4a8_workspace_bytes(M, N, K, group_int4) bytes, 16-byte aligned, is what the path
 * chosen for the shape uses (0 for decode-size calls with K <= 4096: small M, group_int4 == 128, 16-byte aligned a
 * and b_packed run one fused kernel that reads the packed words once; fp32 partial sums of its K ranges,
 * ceil(K / 4096) * M * N * 4 bytes, for K > 4096; otherwise the expanded int8 weights, round16(N*K), and behind
 * them llmk_gemm_workspace_bytes(M,N,K) for the int8 tile kernels). */
int64_t llmk_gemm_w4a8_workspace_bytes(int64_t M, int64_t N, int64_t K, int group_int4);
int llmk_gemm_w4a8(const int8_t* a, const void* a_s, const int32_t* b_packed, const void* b_s,
                   int s_dtype, const int8_t* b_s4, const int8_t* b_z4, void* c, int c_dtype,
                   int64_t M, int64_t N, int64_t K, int group_int4,
                   void* workspace, int64_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ W4A16
 * C[M,N] (fp16) = A[M,K] (fp16) x ((nibble - 8) * s[k / groupsize, n]); B and s in the
 * simple-Marlin packed layout produced by QuantUtils.pack (B int32 [K/16, 2N], s fp16 [K/g, N]
 * permuted per 64 columns).  M, N, K % 16 == 0 (rc -1 otherwise, as the reference launcher),
 * additionally N % 64 == 0 and groupsize % 16 == 0.
 * ref: fast_dequant/simple_marlin/marlin_w4a16_gemm.cu:283-326 (simple_marlin_cuda),
 *      marlin_w4a16_gemm.cpp:23-111 (mul).                                                    */
/* bytes of scratch llmk_gemm_w4a16_marlin uses for this shape (0 = none): fp32 split-K partial sums, and for
 * M > 64 room for the fp16 copy of W that the two-pass path of large M multiplies.  Without it (workspace
 * NULL / too small) the kernels run with fewer K slices, large M on the weight-streaming kernel. */
int64_t llmk_gemm_w4a16_marlin_workspace_bytes(int64_t M, int64_t N, int64_t K);
int llmk_gemm_w4a16_marlin(const void* a_f16, const int32_t* b, void* c_f16, const void* s_f16,
                           int64_t M, int64_t N, int64_t K, int groupsize,
                           void* workspace, int64_t workspace_bytes, void* stream);
/* Quantiser of the [N, K] bit-packed W4A16 layout (the reference states this rule only in its benchmark
 * configuration: groups along K, s = absmax / 7 as fp16, q = clamp(rne(w / s), -8, 7) + 8, 8 K-consecutive nibbles
 * per int32 as quantization/bitpack.py:38-145 packs columns).  w fp32 / fp16 / bf16 [N, K], 16-byte aligned;
 * packed int32 [N, K/8]; scales fp16 [N, K/group]; q (optional, 8-byte aligned) uint8 [N, K]; group a power
 * of two in 8..512 dividing K. */
int llmk_quant_w4_nk(const void* w, int w_dtype, int32_t* packed, void* scales_f16, uint8_t* q, int64_t N,
                     int64_t K, int group, void* stream);
/* Same product for W stored [N, K/8] int32 by pack_weights_over_cols (nibble i of a word = k*8+i)
 * with s fp16 [N, K/g]; a/c fp16 or bf16 (ac_dtype; bf16: M <= 64 with 128-wide groups streams the weights,
 * every other bf16 call multiplies a bf16 copy of W and needs the N*K*2-byte workspace).  workspace is optional for fp16:
 * M > 512 with N*K*2 bytes (16-byte aligned) runs as dequantise + tiled MFMA GEMM; 64 < M <= 512 (and
 * 32 < M <= 64 with large weights) runs on tile kernels that expand the packed words themselves and use
 * up to 8*M*N*4 bytes for split-K partial sums; M <= 64, K > 4096 with ceil(K/4096)*M*N*4 bytes runs as
 * K ranges with fp32 partial sums. */
int llmk_gemm_w4a16_nk(const void* a, const int32_t* b_packed, void* c, const void* s_f16,
                       int ac_dtype, int64_t M, int64_t N, int64_t K, int groupsize,
                       void* workspace, int64_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ converters and the one-tile MFMA GEMM
 * ref: fast_dequant/fast_dtype_convert/fast_uint4_to_fp16.cu:21-109,112-127 (out[i] = nibble_i - 8, nibble i
 *      of word w at bits 4i; the natural order of the reference's "simple" kernel),
 *      fast_uint8_to_fp16.cu:8-73 and fast_uint8_to_bf16.cu:8-70 (out[i] = in[i] - 128),
 *      fast_dequant/simple_marlin/mma_fp16.cu (C fp16 [M,N] = A fp16 [M,K] x B fp16 [K,N], row-major). */
int llmk_convert_u4_to_f16(const uint32_t* packed, void* out_f16, int64_t n, void* stream);
int llmk_convert_u8_to_f16(const uint8_t* in, void* out_f16, int64_t n, void* stream);
int llmk_convert_u8_to_bf16(const uint8_t* in, void* out_bf16, int64_t n, void* stream);
int llmk_gemm_f16_simple(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K,
                         void* stream);

/* ------------------------------------------------------------------ communication payload quantizers
 * ref: quant_communication/quant_utils.py:9-58 (int8, block 32: llmk_act_quant_i8 with
 *      LLMK_ROUND_HALF_UP), :61-113 and :158-205 (dequant: the product is formed and rounded in the
 *      scale dtype), :116-155 (e4m3, block 128, scale stored as fp16). */
int llmk_comm_quant_fp8(const void* x, int x_dtype, void* y_e4m3, void* s, int s_dtype,
                        int64_t n_groups, int block, void* stream);
int llmk_comm_dequant(const void* y, int kind, const void* s, int s_dtype, void* x, int x_dtype,
                      int64_t n_groups, int block, void* stream);

/* ------------------------------------------------------------------ MoE (one GPU's experts)
 * ref: moe/group_gemm_kernel.py:19-45 (segment pointers, src2dst), :81-117 (pre_reorder),
 *      :120-235 (silu/gelu and mul), :238-288 (post_reorder), :291-513 (grouped GEMM).       */
int llmk_moe_seg_indptr(const int64_t* sorted_ids, int64_t* seg_indptr, int64_t num_toks,
                        int num_experts, void* stream);
int llmk_moe_src2dst(const int64_t* reorder_ids, int32_t* src2dst, int64_t num_toks, void* stream);
/* ref: moe/group_gemm_kernel.py:48-78 (run_moe_ep_preproess) in one launch: stable sort of the num_toks
 * flattened expert ids (int32 / int64 by ids_bytes; sorted_ids has the same type), src2dst[i] = position of
 * id i in the sorted order, seg_indptr[e + 1] = number of ids <= e.  Every workgroup places 1024 ids and
 * reads the whole id list to do so: the entry point is for the id counts of one forward pass and fails
 * beyond the limits below;
 * ids outside [0, num_experts) are ordered as one leading (negative) and one trailing group. */
#define LLMK_MOE_PREPROCESS_MAX_EXPERTS 512
#define LLMK_MOE_PREPROCESS_MAX_IDS 32768
int llmk_moe_ep_preprocess(const void* topk_ids, int ids_bytes, int64_t num_toks, int num_experts,
                           void* sorted_ids, int32_t* src2dst, int64_t* seg_indptr, void* stream);
/* ids_bytes: 4 or 8 (topk_ids int32 / int64).  a1_scales may be NULL (fp32 per expert). */
int llmk_moe_pre_reorder(const void* x, int x_dtype, void* out, int out_dtype, const int32_t* src2dst,
                         const void* topk_ids, int ids_bytes, const float* a1_scales,
                         int start_expert, int end_expert, int topk, int64_t T, int64_t hidden,
                         void* stream);
/* act: 0 silu, 1 tanh-gelu.  gateup [M, 2I] -> out [M, I]; scales may be NULL. */
int llmk_moe_act_and_mul(const void* gateup, int in_dtype, void* out, int out_dtype,
                         const void* reorder_topk_ids, int ids_bytes, const float* scales,
                         int start_expert, int end_expert, int64_t M, int64_t two_i, int act,
                         void* stream);
/* Fused variants (the reference marks them as TODO: moe/sglang_moe_all_gather_all_reduce.py:295-296,365,
 * 407-408): the gated activation, resp. the token permutation, followed by the 1 x 128 activation quantizer
 * of the grouped GEMM in one pass.  kind: LLMK_KIND_FP8 (q e4m3, s fp32) or LLMK_KIND_I8 (q int8, s fp16,
 * round_mode as in llmk_act_quant_i8).  q_out [M, I] resp. [T*topk, hidden]; s_out one scale per 128
 * elements of a row.  Results equal llmk_moe_act_and_mul / llmk_moe_pre_reorder followed by
 * llmk_act_quant_fp8 / _i8 bit for bit.  fp16 / bf16 inputs; I resp. hidden a multiple of 128. */
int llmk_moe_act_and_mul_quant(const void* gateup, int in_dtype, void* q_out, void* s_out, int kind,
                               int round_mode, const void* reorder_topk_ids, int ids_bytes,
                               const float* scales, int start_expert, int end_expert, int64_t M,
                               int64_t two_i, int act, void* stream);
int llmk_moe_pre_reorder_quant(const void* x, int x_dtype, void* q_out, void* s_out, int kind,
                               int round_mode, const int32_t* src2dst, const void* topk_ids,
                               int ids_bytes, const float* a1_scales, int start_expert, int end_expert,
                               int topk, int64_t T, int64_t hidden, void* stream);
/* Grouped gate / up projection with the gated activation and the 1 x 128 quantiser of the down projection in its
 * epilogue: q_out, s_out = llmk_moe_act_and_mul_quant(llmk_grouped_gemm(a, b) rounded to mid_dtype), bit for bit, without
 * the [M, 2I] tensor in between (the reference runs grouped_gemm_triton, silu_and_mul_triton_kernel and the activation
 * quantiser of the next grouped_gemm_triton one after the other: moe/sglang_moe_all_gather_all_reduce.py:330-408).
 * a [M, K] and b [E, 2I, K] (gate rows first) in the operand type of `kind` (LLMK_KIND_FP8 or LLMK_KIND_I8) with block
 * scales scale_a [M, K/128], scale_b [E, 2I/128, K/128] of s_dtype; mid_dtype LLMK_F16 or LLMK_BF16 = the dtype the
 * separate GEMM would have written; act 0 silu, 1 tanh-gelu; q_out [M, I], s_out [M, I/128] as in
 * llmk_moe_act_and_mul_quant (no per-expert scales).  Rows outside every segment are left unwritten.  16-bit scales
 * need M * K/128 * 4 bytes of workspace.  Taken only for shapes that run on the 256-column tile kernel:
 * llmk_grouped_gemm_swiglu_quant_fused returns 1 for those, 0 otherwise (then run the three calls), and the fused entry
 * fails with LLMK_ERR_SHAPE on a shape it does not take. */
int llmk_grouped_gemm_swiglu_quant_fused(int kind, int E, int64_t M, int64_t two_i, int64_t K);
int llmk_grouped_gemm_swiglu_quant(const void* a, const void* b, void* q_out, void* s_out, int kind,
                                   int mid_dtype, int round_mode, int E, int64_t M, int64_t two_i, int64_t K,
                                   const int64_t* seg_indptr, const int64_t* weight_indices,
                                   const void* scale_a, const void* scale_b, int s_dtype, int act,
                                   void* workspace, int64_t workspace_bytes, void* stream);
/* w_dtype: dtype code of topk_weights. */
int llmk_moe_post_reorder(const void* down_out, void* out, int dtype, const int32_t* src2dst,
                          const void* topk_ids, int ids_bytes, const void* topk_weights, int w_dtype,
                          int start_expert, int end_expert, int topk, int64_t T, int64_t hidden,
                          void* stream);
/* Per-expert scalar scales (the `use_fp8_w8a8` branch without block_shape that the reference keeps commented
 * out, moe/group_gemm_kernel.py:417-420) written in the block-scale layout of llmk_grouped_gemm, in one launch
 * and without reading anything back: scale_a[r, 0:K/128] = sa[e] for the rows r of segment e (0 for rows
 * outside every segment), scale_b[w, :, :] = sb[w] for the Eb weight matrices.  sa [E], sb [Eb] fp32. */
int llmk_moe_expert_scales(const float* sa, const float* sb, const int64_t* seg_indptr, int E, int Eb,
                           int64_t M, int64_t N, int64_t K, void* scale_a, void* scale_b, int s_dtype,
                           void* stream);
/* C[seg[e]:seg[e+1], :] = A[seg[e]:seg[e+1], :] x B[weight_indices[e]]^T  for e < E.
 * a [M,K], b [E,N,K], c [M,N]; scale_a [M,K/128], scale_b [E,ceil(N/128),K/128] for the
 * block-scaled kinds (s_dtype = dtype code of both), NULL otherwise.  workspace: optional scratch of
 * llmk_gemm_workspace_bytes(M, N, K) bytes. */
int llmk_grouped_gemm(const void* a, const void* b, void* c, int kind, int c_dtype, int E,
                      int64_t M, int64_t N, int64_t K, const int64_t* seg_indptr,
                      const int64_t* weight_indices, const void* scale_a, const void* scale_b,
                      int s_dtype, void* workspace, int64_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ calibration (benchmark harness only)
 * No counterpart in the reference and not on the product path: what the chip sustains on the two resources the
 * GEMMs are priced against, for the same process that times them.
 * llmk_calib_mfma: `workgroups` workgroups of eight waves, each wave `iters` x 32 matrix instructions of `kind`
 * (LLMK_KIND_FP8: 16x16x128, LLMK_KIND_I8: 16x16x64, LLMK_KIND_F16 / BF16: 16x16x32) on register operands
 * taken from `operands` (64 KiB of finite values of the operand type) into 32 independent accumulator tiles;
 * out: workgroups * 512 floats (keeps the loop alive); clocks (optional): two int64, the s_memtime and the
 * s_memrealtime (100 MHz) ticks the loop of one wave took.
 * llmk_calib_read: reads nbytes (whole 64 KiB tiles) with no arithmetic, pattern 0 = linear stream, 1 = the
 * address pattern of the weight-streaming GEMM kernels (16-row tiles of 4096-byte rows). */
int llmk_calib_mfma(int kind, int iters, const void* operands, float* out, int workgroups, long long* clocks,
                    void* stream);
int llmk_calib_read(const void* src, int64_t nbytes, int pattern, int* sink, int workgroups, void* stream);
/* llmk_gemm_fp8_block (same operands, M > 512) whose first workgroup also reports the shader clock it ran at:
 * clocks[0] = s_memtime ticks, clocks[1] = s_memrealtime (100 MHz) ticks between its first and its last instruction. */
int llmk_calib_gemm_fp8_clock(const void* a_e4m3, const float* a_s, const void* b_e4m3, const float* b_s, void* c,
                              int c_dtype, int64_t M, int64_t N, int64_t K, void* workspace, int64_t workspace_bytes,
                              long long* clocks, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LLMK_H */

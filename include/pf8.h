/*
 * pf8.h -- C ABI of libpf8.so: MI355X (gfx950) kernels for the PaddleFormers FP8 block-quant /
 * block-scaled GEMM path.
 *
 * Every entry point replaces one third-party operator the reference resolves at call time
 * (paddle.incubate.nn.functional.* and paddlefleet_ops.deep_gemm.*); the comment on each
 * declaration cites the reference call site (paths relative to the PaddleFormers checkout).
 *
 * Conventions
 *   - plain pointers to DEVICE memory and sizes; no framework types.  bf16 = uint16_t bit pattern,
 *     e4m3 = uint8_t OCP float8_e4m3fn code, scales = float (decode scale: x ~= q * s).
 *   - every function returns 0 on success or a negative PF8_E* code; pf8_last_error() gives the
 *     thread-local message.  Nothing throws, nothing allocates device memory, nothing synchronises.
 *   - `stream` is a hipStream_t (NULL = the null stream).  Launches are asynchronous.
 *   - zero-sized problems are legal and return 0 without launching (the reference short-circuits
 *     them: transformers/fp8_utils.py:185,202,308,945,998,1208,1256).
 *   - scale_layout: 0 = row-major [rows, K/128] (output_scale_transpose=False),
 *                   1 = [K/128, rows]          (output_scale_transpose=True, the layout the GEMMs
 *                       consume as `.T`, transformers/fp8_utils.py:278,941).
 *                   2 = [K/128, rows] UE8M0 exponent bytes (uint8 behind the float* argument, scale =
 *                       2^(byte - 127); needs pow2): what the *_ue8m0 GEMMs read as `sa`, the scale format of
 *                       use_ue8m0 (transformers/configuration_utils.py:454-459).  Taken by pf8_quant_1x128 and
 *                       pf8_swiglu_weighted_quant; pf8_quant_and_transpose_split writes its row scales this
 *                       way with pow2_rows = 2, pf8_transpose_split_quant reads such scales with xs_layout = 2.
 *   - pow2: 0 = s = amax/448 (cli/train/deepseek_v3_pretrain/kernel.py:44);
 *           1 = s rounded up to a power of two (utils/upcast_downcast_triton.py:71-85).
 *     An all-zero tile gets s = 1 and zero bytes.
 *   - all base pointers must be 16-byte aligned; K (the quantised axis) must be a multiple of 128.
 */
#ifndef PF8_H
#define PF8_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PF8_OK 0
#define PF8_EINVAL (-1)    /* bad shape, alignment, flag or null pointer */
#define PF8_ELAUNCH (-2)   /* HIP reported an error at launch */
#define PF8_ENODEV (-3)    /* no gfx950 device / wrong architecture */

typedef void* pf8_stream_t; /* hipStream_t */

int pf8_version(void);
const char* pf8_last_error(void);

/* deep_gemm.set_num_sms(get_sm_num()) -- transformers/fp8_utils.py:42,54-55,277: caps the number of
 * compute units the GEMM grids are sized for (0 = all).  Returns the previous value. */
int pf8_set_num_cus(int n);
int pf8_get_num_cus(void);
/* The budget in force on the current device: min(pf8_set_num_cus value, the device's compute units). */
int pf8_effective_num_cus(void);

/* fp8_quant_blockwise(x, quant_method="1x128", input_transpose=False, output_scale_transpose=...)
 * transformers/fp8_utils.py:262-268, 938-941; cli/train/deepseek_v3_pretrain/kernel.py:29-70.
 * x bf16 [M,K] with row stride ldx (elements) -> q [M,K], s per scale_layout. */
int pf8_quant_1x128(const uint16_t* x, int64_t M, int64_t K, int64_t ldx, uint8_t* q, float* s,
                    int scale_layout, int pow2, pf8_stream_t stream);

/* fp8_quant_blockwise(w, quant_method="128x128", output_scale_transpose=False, input_transpose=...,
 * return_transpose_only=...) -- transformers/fp8_utils.py:105-131, 628-665.
 * w bf16 [R,C] -> q [R,C], s [R/128,C/128] and/or q_t [C,R], s_t [C/128,R/128]; either pair may be
 * NULL (return_transpose_only=True passes q = s = NULL). */
int pf8_quant_128x128(const uint16_t* w, int64_t R, int64_t C, uint8_t* q, float* s, uint8_t* q_t,
                      float* s_t, int pow2, pf8_stream_t stream);

/* fp8_quant_blockwise(x, quant_method="1x128", input_transpose=True[, return_transpose_only=True])
 * transformers/fp8_utils.py:155-174, 380-382, 585-587, 725-727: one pass that emits the row-scaled
 * copy q [M,K] (+ s) and the column-scaled transposed copy q_t [K,M] (+ s_t: layout 1 ->
 * [M/128,K], layout 0 -> [K,M/128]).  M and K multiples of 128.  q = s = NULL skips the row copy. */
int pf8_quant_transpose(const uint16_t* x, int64_t M, int64_t K, uint8_t* q, float* s, uint8_t* q_t,
                        float* s_t, int scale_layout, int pow2, pf8_stream_t stream);

/* fused_stack_transpose_quant(weight_list, transpose) -- transformers/fp8_utils.py:91-102;
 * un-fused definition ernie token_dispatcher/fp8_utils.py:276-287.  w_list is a HOST array of E
 * device pointers to bf16 [R,C] weights.  transpose=0: q [E*R, C], s [E*R/128, C/128];
 * transpose=1: q [E*C, R], s [E*C/128, R/128]. */
int pf8_stack_transpose_quant(const uint16_t* const* w_list, int E, int64_t R, int64_t C,
                              int transpose, uint8_t* q, float* s, int pow2, pf8_stream_t stream);

/* Both orientations of fused_stack_transpose_quant from ONE read of the weights: what
 * DeepseekV2MoE.fp8_quant_weight(quant_transpose=None) asks for with two calls per weight list
 * (cli/train/deepseek_v3_pretrain/modeling.py:506-567, driven once per optimizer step by
 * FP8QuantWeightCallback, trainer/trainer_callback.py:727-765).  q [E*R, C] + s [E*R/128, C/128]
 * and q_t [E*C, R] + s_t [E*C/128, R/128]; byte-identical to the two separate calls. */
int pf8_stack_quant_both(const uint16_t* const* w_list, int E, int64_t R, int64_t C, uint8_t* q,
                         float* s, uint8_t* q_t, float* s_t, int pow2, pf8_stream_t stream);

/* pf8_stack_quant_both with the fragment-major copies of its two outputs made in the same pass (no counterpart in the
 * reference, whose FP8 weight cache is read by deep_gemm only): q_fm / q_t_fm receive the bytes of q / q_t in the order
 * pf8_weight_to_fragment_major gives them, what the *_fm GEMMs read.  Either may be NULL (an orientation whose shape those
 * GEMMs do not take), not both.  Saves the two re-ordering passes per cached weight and optimizer step. */
int pf8_stack_quant_both_fm(const uint16_t* const* w_list, int E, int64_t R, int64_t C, uint8_t* q, float* s,
                            uint8_t* q_t, float* s_t, uint8_t* q_fm, uint8_t* q_t_fm, int pow2,
                            pf8_stream_t stream);

/* fused_weighted_swiglu_act_quant(o1, probs, using_pow2_scaling) -- transformers/fp8_utils.py:981-987;
 * un-fused definition ernie token_dispatcher/fp8_utils.py:996-1004.  o1 bf16 [M,2I] (gate first),
 * probs fp32 [M] or NULL -> q [M,I], s per scale_layout.  o2 (bf16 [M,I]) optionally receives the
 * pre-quant activations (NULL to skip). */
int pf8_swiglu_weighted_quant(const uint16_t* o1, const float* probs, int64_t M, int64_t I,
                              uint8_t* q, float* s, uint16_t* o2, int scale_layout, int pow2,
                              pf8_stream_t stream);

/* fused_transpose_split_quant(x, scale, tokens_per_expert, pow_2_scales) --
 * transformers/fp8_utils.py:1096-1100; un-fused definition ernie token_dispatcher/fp8_utils.py:1199-1210.
 * x: bf16 [Mtot,K] (x_is_fp8=0) or e4m3 [Mtot,K] with fp32 scales xs (x_is_fp8=1; xs_layout 0 =
 * [Mtot,K/128] row-major, 1 = [K/128,Mtot] -- the cached input_scale of the MoE node is the latter).
 * rows_per_expert: HOST array of E counts, each a multiple of 128, summing to Mtot.
 * Outputs are packed: expert e's q_t [K, M_e] starts at q_t + K*off_e and its s_t [M_e/128, K] at
 * s_t + (off_e/128)*K, off_e = rows of the experts before e. */
int pf8_transpose_split_quant(const void* x, const float* xs, int x_is_fp8, int xs_layout,
                              const int64_t* rows_per_expert, int E, int64_t K, uint8_t* q_t, float* s_t,
                              int pow2, pf8_stream_t stream);

/* pf8_transpose_split_quant with the row copy of UnZipNode.forward / ZipNode.backward (moe_utils.py:141-186, 217-261)
 * folded into the read: row r of the expert-sorted input is row src_row[r] of tokens [T, K] -- bf16 (x_is_fp8 = 0), or
 * e4m3 with that row's scales (xs_layout 0 = [T, K/128], 1 = [K/128, T], 2 = UE8M0 bytes [K/128, T]); src_row[r] < 0 is a
 * row of zeros.  src_row int32 [sum rows_per_expert], 16-byte aligned, entries below T.  Outputs bit-identical to
 * pf8_transpose_split_quant on the rows pf8_moe_permute copies out. */
int pf8_transpose_split_quant_gather(const void* tokens, const float* token_scales, int x_is_fp8, int xs_layout,
                                     int64_t T, const int32_t* src_row, const int64_t* rows_per_expert, int E,
                                     int64_t K, uint8_t* q_t, float* s_t, int pow2, pf8_stream_t stream);

/* The two quantizations the MoE node's backward applies to the SAME bf16 gradient, from one read:
 * fp8_quant_blockwise(x, quant_method="1x128", output_scale_transpose=True, using_pow2_scale=pow2_rows)
 * for the dgrad GEMM and fused_transpose_split_quant(x, None, tokens_per_expert, pow2_t) for the wgrad
 * GEMM -- out_grad at transformers/fp8_utils.py:1030-1036 and :1115, do1 at :1073-1079 and :1168.  q e4m3 [Mtot,K], s fp32 [K/128,Mtot]; q_t / s_t packed as pf8_transpose_split_quant
 * writes them.  Every output is bit-identical to the separate calls'. */
int pf8_quant_and_transpose_split(const uint16_t* x, const int64_t* rows_per_expert, int E, int64_t K,
                                  uint8_t* q, float* s, int pow2_rows, uint8_t* q_t, float* s_t,
                                  int pow2_t, pf8_stream_t stream);

/* fused_act_dequant(q, s) -- transformers/fp8_utils.py:136-138, 779.  1x128 dequant to bf16. */
int pf8_act_dequant(const uint8_t* q, const float* s, int scale_layout, int64_t M, int64_t K,
                    uint16_t* out, pf8_stream_t stream);

/* weight_dequant(x, s) -- cli/train/deepseek_v3_pretrain/kernel.py:73-118;
 * quantization/checkpoint_dequant.py:148-174,277-292.  128x128 dequant to bf16; R and C arbitrary
 * (s is [ceil(R/128), ceil(C/128)], trailing partial blocks cropped). */
int pf8_weight_dequant(const uint8_t* q, const float* s, int64_t R, int64_t C, uint16_t* out,
                       pf8_stream_t stream);

/* FP8BlockCheckpointDequantizer.dequantize -- quantization/checkpoint_dequant.py:277-292 with
 * _decode_e4m3 / _decode_ue8m0 / _expand_scale_grid (:76-176): out = cast(e4m3(q) * scale), q raw
 * e4m3 bytes viewed as [B, R, C], scale [B, ceil(R/block_r), ceil(C/block_c)] (an axis that is not
 * blocked has block size 1), partial trailing blocks cropped.  scale_format 0 = fp32, 1 = UE8M0
 * exponent bytes (2^(e-127), 255 -> inf), 2 = bf16, 3 = fp16.  out is bf16 (out_f32 = 0) or fp32. */
int pf8_block_dequant(const uint8_t* q, const void* scale, int scale_format, int64_t B, int64_t R,
                      int64_t C, int64_t block_r, int64_t block_c, void* out, int out_f32,
                      pf8_stream_t stream);

/* paddle.nn.functional.moe_permute(hidden_states, scale, expert_routemap_topk, expert_prob_topk,
 * num_experts, tokens_per_expert, padding_alignment) as UnZipNode.forward / ZipNode.backward call it
 * (cli/train/deepseek_v3_pretrain/moe_utils.py:141-186, 217-261; ernie twin
 * models/moe/token_dispatcher/moe_utils.py:222, 349).  x [T,H] bf16 (x_is_fp8 = 0) or e4m3 bytes with
 * xs fp32 [T,H/128]; routemap int32 [T,topk] (expert id, negative = unused slot), probs fp32 [T,topk]
 * or NULL; tokens_per_expert: HOST array of E routed-row counts.  Outputs: out_x [Mpad,H] with every
 * expert's segment padded to a multiple of padding_alignment (zero rows), rowmap int32 [T,E] (row of
 * token t in expert e's segment, -1 = not routed; tokens keep their order inside a segment),
 * out_probs fp32 [Mpad] (0 on padding rows; NULL to skip), out_xs fp32 [Mpad,H/128] (with xs).
 * *overflow (device int32, cleared by the caller): bit 0 is set when a token is routed to an expert whose
 * tokens_per_expert count is already used up (such copies are dropped), bit 1 when an expert receives
 * fewer tokens than its count says (the rows left over are written as zeros, like padding rows). */
int pf8_moe_permute(const void* x, int x_is_fp8, const float* xs, const int32_t* routemap,
                    const float* probs, int64_t T, int64_t H, int topk, int E,
                    const int64_t* tokens_per_expert, int padding_alignment, void* out_x,
                    int32_t* rowmap, float* out_probs, float* out_xs, int32_t* overflow,
                    pf8_stream_t stream);

/* The same reordering as pf8_moe_permute with no row copied: src_row int32 [Mpad] receives, for every row of the
 * expert-sorted padded layout, the index of the token that pf8_moe_permute would have copied there (-1 for a padding row
 * and for the rows left over when an expert receives fewer tokens than its count says); rowmap, out_probs and *overflow
 * are what pf8_moe_permute writes.  The consumers that take (tokens, src_row) in place of the copied rows
 * (pf8_grouped_gemm_nt_contiguous_fm_gather, pf8_transpose_split_quant_gather) read a -1 row as zeros, which is what
 * the copy holds there; UnZipNode.forward's token copy (moe_utils.py:141-186) then never exists in memory. */
int pf8_moe_permute_map(const int32_t* routemap, const float* probs, int64_t T, int topk, int E,
                        const int64_t* tokens_per_expert, int padding_alignment, int32_t* rowmap,
                        int32_t* src_row, float* out_probs, int32_t* overflow, pf8_stream_t stream);

/* paddle.nn.functional.moe_unpermute(hidden_states_unzipped, zipped_expertwise_rowmap,
 * expert_routemap_topk, token_prob_unzipped, total_zipped_tokens, num_experts) as ZipNode.forward /
 * UnZipNode.backward call it (moe_utils.py:188-215): out[t] = bf16(sum over the token's used slots,
 * in slot order, fp32) of unzipped[rowmap[t, routemap[t,k]]]; out_probs[t,k] = probs_unzipped of
 * that row (0 for an unused slot; NULL to skip). */
int pf8_moe_unpermute(const uint16_t* unzipped, const int32_t* rowmap, const int32_t* routemap,
                      const float* probs_unzipped, int64_t T, int64_t H, int topk, int E,
                      uint16_t* out, float* out_probs, pf8_stream_t stream);

/* paddle.incubate.nn.functional.fused_rms_norm_ext(x, norm_w, eps) -> (y, invvar) and its gradient
 * paddle._C_ops.fused_rms_norm_ext_grad(x, norm_w, invvar, dy, eps) -> (dx, dw), the norm that
 * FusedNormFP8MLPFunction recomputes (transformers/fp8_utils.py:470-475, 520-541, 687-741).
 * x, dy, y, dx bf16 [M,H], w bf16 [H], invar fp32 [M] = 1/sqrt(mean(x^2)+eps); y = bf16(x*invar*w).
 * dw fp32 [H] is ADDED to (the caller zeroes it).  ws: DEVICE scratch of ws_rows x H floats, 16-byte
 * aligned (1024 rows use the whole device); each workgroup leaves its share of dw in a row of it
 * and a second kernel adds the rows up in order.  ws == NULL: the shares go to dw by atomics
 * (several times slower at training sizes, and the rounding then depends on the order). */
int pf8_rms_norm_fwd(const uint16_t* x, const uint16_t* w, float eps, int64_t M, int64_t H,
                     uint16_t* y, float* invar, pf8_stream_t stream);
int pf8_rms_norm_bwd(const uint16_t* x, const uint16_t* w, const float* invar, const uint16_t* dy,
                     int64_t M, int64_t H, uint16_t* dx, float* dw, float* ws, int64_t ws_rows,
                     pf8_stream_t stream);

/* fused_swiglu_weighted_bwd(o1, do2_s, probs) -- transformers/fp8_utils.py:1049-1052; un-fused
 * definition ernie token_dispatcher/fp8_utils.py:1088-1092.  -> do1 bf16 [M,2I], probs_grad fp32 [M],
 * o2_s bf16 [M,I]. */
int pf8_swiglu_weighted_bwd(const uint16_t* o1, const uint16_t* do2_s, const float* probs, int64_t M,
                            int64_t I, uint16_t* do1, float* probs_grad, uint16_t* o2_s,
                            pf8_stream_t stream);

/* The SwiGLU backward of the MoE node (transformers/fp8_utils.py:1049-1052) together with the quantizations its results
 * go through before their next use: do1 [M,2I] row-wise for the dgrad GEMM (fp8_quant_blockwise "1x128" with
 * output_scale_transpose, :1073-1079) and transposed per expert for the weight gradient (fused_transpose_split_quant,
 * :1168), o2_s [M,I] transposed per expert (:1115).  One kernel reads o1 [M,2I], do2_s [M,I] (bf16) and probs fp32 [M]
 * and writes only the quantized forms; M = sum of rows_per_expert (HOST array of E multiples of 128, E <= 256).
 * do1_q e4m3 [M,2I]; do1_s fp32 [M,2I/128] (scale_layout 0) or [2I/128,M] (scale_layout 1), exact (pow2_rows = 0) or
 * powers of two (1), or UE8M0 bytes [2I/128,M] (pow2_rows = 2, scale_layout 1);
 * do1_q_t / do1_s_t and o2s_q_t / o2s_s_t: the experts' [2I,Me] / [I,Me] blocks and [Me/128,2I] / [Me/128,I] scales
 * packed back to back, as pf8_transpose_split_quant lays them out.  All of these equal, byte for byte, what
 * pf8_quant_and_transpose_split and pf8_transpose_split_quant make of pf8_swiglu_weighted_bwd's outputs.  probs_grad
 * fp32 [M] is summed per 128-column tile and then over the tiles, so it agrees with pf8_swiglu_weighted_bwd's to
 * rounding only.  pg_partial: DEVICE scratch of (I/128) x M floats. */
int pf8_swiglu_weighted_bwd_quant(const uint16_t* o1, const uint16_t* do2_s, const float* probs,
                                  const int64_t* rows_per_expert, int E, int64_t I, uint8_t* do1_q, float* do1_s,
                                  int scale_layout, int pow2_rows, uint8_t* do1_q_t, float* do1_s_t, uint8_t* o2s_q_t,
                                  float* o2s_s_t, int pow2_t, float* probs_grad, float* pg_partial, pf8_stream_t stream);

/* deep_gemm.fp8_gemm_nt((a, sa), (b, sb), out) -- transformers/fp8_utils.py:278, 368;
 * cli/train/deepseek_v3_pretrain/kernel.py:129-220.  a e4m3 [M,K], sa per sa_layout, b e4m3 [N,K],
 * sb fp32 [ceil(N/128), K/128] -> out bf16 [M,N] (row stride ldo elements). */
int pf8_gemm_nt(const uint8_t* a, const float* sa, int sa_layout, const uint8_t* b, const float* sb,
                int64_t M, int64_t N, int64_t K, uint16_t* out, int64_t ldo, pf8_stream_t stream);

/* fp8_gemm_blockwise(..., is_a_1d_scaled=True, is_b_1d_scaled=True) / deep_gemm.fp8_gemm_nt(...,
 * recipe=(1,1,128)) -- transformers/fp8_utils.py:176-221 (kitchen_gemm).  Weight-gradient GEMM:
 * out[Kin,N] (+)= a_t[Kin,M] . b_t[N,M]^T, a_t/b_t e4m3, sa_t fp32 [M/128,Kin], sb_t fp32 [M/128,N],
 * out fp32, accumulate != 0 adds to the existing contents.  M multiple of 128. */
int pf8_gemm_nt_1d1d_f32(const uint8_t* a_t, const float* sa_t, const uint8_t* b_t, const float* sb_t,
                         int64_t Kin, int64_t N, int64_t M, float* out, int accumulate,
                         pf8_stream_t stream);

/* deep_gemm.m_grouped_fp8_gemm_nt_contiguous((a, sa), (b, sb), out, m_indices) --
 * transformers/fp8_utils.py:906-911, 949-954, 1002-1007, 1042-1047, 1087-1092.  a [Mtot,K] rows sorted
 * by expert, every expert segment a multiple of 128 rows; b [E,N,K]; sb [E,ceil(N/128),K/128];
 * m_indices DEVICE int32 [Mtot] (expert of each row; negative = skip the 128-row tile).
 * Mtot multiple of 128. */
int pf8_grouped_gemm_nt_contiguous(const uint8_t* a, const float* sa, int sa_layout, const uint8_t* b,
                                   const float* sb, int E, int64_t Mtot, int64_t N, int64_t K,
                                   const int32_t* m_indices, uint16_t* out, pf8_stream_t stream);

/* Fragment-major copy of a quantized weight, the operand form of the *_fm GEMMs below.  The reference keeps its FP8
 * weights as plain [N, K] tensors that only deep_gemm reads (cache_fp8_weight / fp8_quant_weight,
 * transformers/fp8_utils.py:97-137, 403-437); this library's GEMMs take the same bytes re-ordered into the order in which
 * a wavefront's matrix instructions consume them: w e4m3 [E][N, K] row-major ->
 *     wf[e][n / 64][k / 128][pf 0..1][kh 0..1][h 0..1][lane 0..63][16 bytes],
 * the 16 bytes being k = 128 (k / 128) + 64 kh + 32 (lane / 32) + 16 h .. + 15 of row n = 64 (n / 64) + 32 pf + lane % 32
 * (the A-operand fragments of v_mfma_f32_32x32x64_f8f6f4, in the order a wavefront consumes them).
 * A permutation of the same E * N * K bytes (no re-quantization; scales are shared with the plain form).
 * N multiple of 64, K multiple of 128. */
int pf8_weight_to_fragment_major(const uint8_t* w, int E, int64_t N, int64_t K, uint8_t* wf, pf8_stream_t stream);

/* 1 when the *_fm GEMMs take this shape (M % 128 == 0, N % 128 == 0 and N >= 256, K % 128 == 0, K >= 384), else 0.  No device access. */
int pf8_gemm_fm_supported(int64_t M, int64_t N, int64_t K);

/* deep_gemm.fp8_gemm_nt / m_grouped_fp8_gemm_nt_contiguous (transformers/fp8_utils.py:289-302, 949-954, 1002-1007) on a
 * fragment-major weight b_fm (pf8_weight_to_fragment_major of the [N, K] / [E, N, K] operand); everything else as in
 * pf8_gemm_nt / pf8_grouped_gemm_nt_contiguous (same scale factors, same order of the K blocks; a block's product is formed
 * by two chained 32x32x64 matrix instructions instead of one 16x16x128, so results agree with theirs to the matrix pipe's
 * precision, within the same bars against the reference formulation).  Shapes outside
 * pf8_gemm_fm_supported are rejected (the caller keeps the plain weight for those). */
int pf8_gemm_nt_fm(const uint8_t* a, const float* sa, int sa_layout, const uint8_t* b_fm, const float* sb, int64_t M,
                   int64_t N, int64_t K, uint16_t* out, int64_t ldo, pf8_stream_t stream);
int pf8_grouped_gemm_nt_contiguous_fm(const uint8_t* a, const float* sa, int sa_layout, const uint8_t* b_fm,
                                      const float* sb, int E, int64_t Mtot, int64_t N, int64_t K,
                                      const int32_t* m_indices, uint16_t* out, pf8_stream_t stream);

/* pf8_grouped_gemm_nt_contiguous_fm with the row copy of UnZipNode.forward / ZipNode.backward (moe_utils.py:141-186,
 * 217-261) folded into the read of the activation operand: row r of the expert-sorted operand is row src_row[r] of
 * tokens [T, K] (e4m3); src_row[r] < 0 (see pf8_moe_permute_map) is a row of zeros.  sa holds the scales of the
 * EXPERT-SORTED rows, [Mtot, K/128] in either layout, as pf8_gather_row_scales makes them from the token scales (zero
 * for a negative src_row).  out is bit-identical to pf8_grouped_gemm_nt_contiguous_fm on the rows pf8_moe_permute copies
 * out.  src_row: int32 [Mtot], 16-byte aligned, every entry below T; tokens below 2 GiB. */
int pf8_grouped_gemm_nt_contiguous_fm_gather(const uint8_t* tokens, int64_t T, const int32_t* src_row, const float* sa,
                                             int sa_layout, const uint8_t* b_fm, const float* sb, int E, int64_t Mtot,
                                             int64_t N, int64_t K, const int32_t* m_indices, uint16_t* out,
                                             pf8_stream_t stream);

/* out[r, kb] = xs[src_row[r], kb] (0 for a negative src_row): the 1x128 scales of rows that are read through a source map,
 * gathered on their own.  xs fp32 [T, KB] row-major; out [rows, KB] row-major (out_layout 0) or [KB, rows] (1). */
int pf8_gather_row_scales(const float* xs, int64_t T, int64_t KB, const int32_t* src_row, int64_t rows, float* out,
                          int out_layout, pf8_stream_t stream);

/* The up+gate grouped GEMM with the activation quantizer of the down projection in its epilogue: the two calls of
 * FP8GroupGemmMlpFunctionNode.forward -- deep_gemm.m_grouped_fp8_gemm_nt_contiguous (transformers/fp8_utils.py:949-954)
 * and fused_weighted_swiglu_act_quant(o1, probs, using_pow2_scaling) (:981-987; un-fused definition ernie
 * token_dispatcher/fp8_utils.py:996-1004) -- as one launch.  a, sa, m_indices as in pf8_grouped_gemm_nt_contiguous;
 * b e4m3 [E, 2I, K] with every expert's gate rows first and its up rows after them (the stacked [H, 2I] weight
 * transposed, as fused_stack_transpose_quant(..., transpose=True) writes it), sb fp32 [E, 2I/128, K/128]; probs fp32
 * [Mtot] or NULL.  Outputs: q e4m3 [Mtot, I] and s fp32 [Mtot, I/128] of
 * quant_1x128( bf16( bf16(silu(o1[:, :I]) * o1[:, I:]) * probs ) ), bit-identical to the two separate calls, and,
 * when o1 is not NULL, the bf16 GEMM result o1 [Mtot, 2I] itself (the node keeps it for backward unless
 * recompute_fwd_gate_up is set, :1263-1267).  pow2: bit 0 = power-of-two scales, bit 1 = s is stored [I/128, Mtot] (the
 * layout the down GEMM reads fastest, scale_layout 1).  Mtot and I multiples of 128, K a multiple of 128 and >= 384;
 * other shapes return PF8_EINVAL (make the two calls). */
int pf8_grouped_gemm_swiglu_quant_nt_contiguous(const uint8_t* a, const float* sa, int sa_layout, const uint8_t* b,
                                                const float* sb, int E, int64_t Mtot, int64_t I, int64_t K,
                                                const int32_t* m_indices, const float* probs, uint16_t* o1,
                                                uint8_t* q, float* s, int pow2, pf8_stream_t stream);

/* The same two GEMMs with power-of-two scales held as UE8M0 exponent bytes (scale = 2^(byte-127)),
 * the form `use_ue8m0` selects for deep_gemm (transformers/configuration_utils.py:454-459; byte
 * format quantization/checkpoint_dequant.py:121-131).  Both operands must have been quantized with
 * pow2 scales (using_pow2_scale=True).  sa u8 [K/128, ldsa] (1x128 scales, K-block major, ldsa >= M
 * and a multiple of 8, base 8-byte aligned); sb u8 [N/128, K/128] ([E, N/128, K/128] grouped).
 * M (Mtot) multiple of 128, N multiple of 128 and >= 256, K multiple of 128 and >= 384, ldo multiple
 * of 8; other shapes return PF8_EINVAL (decode the scales and use the fp32-scale entry points).
 * items: the list pf8_grouped_items_build made for this m_indices (two 128-row blocks of one expert
 * per 256-row work item); with it the call also weighs the expert load and, when N is a multiple of
 * 256, hands a GEMM whose experts are too small for 256-row tiles to the 128-row-tile kernel (with
 * N = 256 t + 128 the paired tiles always run; the last column tile is then half empty).  NULL makes
 * the call walk aligned 256-row tiles and visit those that hold two experts twice. */
int pf8_gemm_nt_ue8m0(const uint8_t* a, const uint8_t* sa, int64_t ldsa, const uint8_t* b,
                      const uint8_t* sb, int64_t M, int64_t N, int64_t K, uint16_t* out, int64_t ldo,
                      pf8_stream_t stream);
int pf8_grouped_gemm_nt_contiguous_ue8m0(const uint8_t* a, const uint8_t* sa, int64_t ldsa,
                                         const uint8_t* b, const uint8_t* sb, int E, int64_t Mtot,
                                         int64_t N, int64_t K, const int32_t* m_indices,
                                         const int32_t* items, uint16_t* out, pf8_stream_t stream);

/* Work-item list of the call above for one m_indices (the same list serves every GEMM that shares
 * it: up+gate, down and the dgrad GEMMs of an MoE step): pairs the 128-row blocks of each expert
 * into 256-row tiles, skipping padding blocks.  items: DEVICE buffer of 4 + 4 * Mtot/128 int32,
 * 16-byte aligned.  No counterpart in the reference, whose deep_gemm schedules inside the binary. */
int pf8_grouped_items_build(const int32_t* m_indices, int64_t Mtot, int32_t* items,
                            pf8_stream_t stream);

/* pf8_grouped_gemm_nt_contiguous_ue8m0 for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same arguments without `items`: the work-item list is built by the call itself, on `stream`, into a
 * 131,088-byte array that is part of the library's device image (one copy per GPU, held until the process
 * ends), and the GEMM then runs exactly as with a caller-built list, so `out` is bit-identical to
 * pf8_grouped_items_build + pf8_grouped_gemm_nt_contiguous_ue8m0.  The call allocates and frees nothing.
 * Mtot is limited to 1,048,576 rows (PF8_EINVAL beyond).  All calls on one GPU share that array: calls
 * that may overlap on one GPU (different streams, different threads) race on it and must be serialised
 * by the caller.  The first call on a device looks the array's address up (hipGetSymbolAddress); make
 * that call outside any stream capture. */
int pf8_grouped_gemm_nt_contiguous_ue8m0_noalloc(const uint8_t* a, const uint8_t* sa, int64_t ldsa,
                                                 const uint8_t* b, const uint8_t* sb, int E, int64_t Mtot,
                                                 int64_t N, int64_t K, const int32_t* m_indices,
                                                 uint16_t* out, pf8_stream_t stream);

/* fp32 scales that are powers of two -> UE8M0 exponent bytes, elementwise (any layout).  not_pow2,
 * when non-null, is a DEVICE int the kernel adds the number of scales to that are negative, zero,
 * non-finite or not a power of two (the caller zeroes it).  Scale side of `use_ue8m0`
 * (transformers/configuration_utils.py:454-459). */
int pf8_scales_to_ue8m0(const float* s, int64_t n, uint8_t* out, int* not_pow2, pf8_stream_t stream);

/* deep_gemm.m_grouped_fp8_gemm_nt_masked((a, sa), (b, sb), out, masked_m, expected_m) --
 * ernie token_dispatcher/fp8_utils.py:227-233.  a [E,Mmax,K], sa [E,Mmax,K/128] row-major,
 * b [E,N,K], sb [E,ceil(N/128),K/128], masked_m DEVICE int32 [E] valid rows -> out [E,Mmax,N];
 * rows >= masked_m[e] are not written. */
int pf8_grouped_gemm_nt_masked(const uint8_t* a, const float* sa, const uint8_t* b, const float* sb,
                               int E, int64_t Mmax, int64_t N, int64_t K, const int32_t* masked_m,
                               int expected_m, uint16_t* out, pf8_stream_t stream);

/* Per-expert weight-gradient loop -- transformers/fp8_utils.py:1102-1134 (bwd_down_weight),
 * 1136-1189 (bwd_gate_up_weight): for each expert e with rows_per_expert[e] > 0,
 * out[e] [Kin,N] (+)= a_t[e] . b_t[e]^T as in pf8_gemm_nt_1d1d_f32, in ONE launch.  a_t/sa_t and
 * b_t/sb_t use the packed layout written by pf8_transpose_split_quant; out is fp32 [E,Kin,N].
 * rows_per_expert is a HOST array (E <= 256). */
int pf8_grouped_wgrad(const uint8_t* a_t, const float* sa_t, const uint8_t* b_t, const float* sb_t,
                      const int64_t* rows_per_expert, int E, int64_t Kin, int64_t N, float* out,
                      int accumulate, pf8_stream_t stream);

/* pf8_gemm_nt_1d1d_f32 / pf8_grouped_wgrad for operands whose scales are ALL powers of two -- what
 * fused_transpose_split_quant(..., pow_2_scales=True) emits, which is how the weight-gradient
 * operands of the MoE node are quantized (transformers/fp8_utils.py:1096-1100, 1117-1129,
 * 1170-1182): both scales go into the block-scaled MFMA (their exponent fields are its UE8M0
 * bytes) and the matrix pipe accumulates the K blocks itself.  Same arguments and layouts; a
 * scale that is not a power of two is NOT detected (its mantissa is dropped). */
int pf8_gemm_nt_1d1d_f32_pow2(const uint8_t* a_t, const float* sa_t, const uint8_t* b_t,
                              const float* sb_t, int64_t Kin, int64_t N, int64_t M, float* out,
                              int accumulate, pf8_stream_t stream);
int pf8_grouped_wgrad_pow2(const uint8_t* a_t, const float* sa_t, const uint8_t* b_t,
                           const float* sb_t, const int64_t* rows_per_expert, int E, int64_t Kin,
                           int64_t N, float* out, int accumulate, pf8_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* PF8_H */

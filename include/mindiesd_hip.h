/*
 * C ABI of libmindiesd_hip.so: the MI355X (gfx950) kernels behind the attention hot path of MindIE-SD.
 *
 * Every entry point takes plain device pointers, sizes, element strides and a HIP stream; nothing is
 * allocated inside (scratch memory, where needed, is an explicit workspace argument with a
 * *_workspace_size companion, mirroring the aclnnXxxGetWorkspaceSize / aclnnXxx pairs the reference
 * resolves with dlsym, csrc/plugin/pytorch_npu_helper.h:612-659).  Kernels are enqueued
 * asynchronously on `stream`; there is no implicit synchronisation.  Inputs are never modified.
 *
 * Return value: 0 on success, otherwise
 *   1  bad argument (null / misaligned pointer, non-positive size, unknown dtype code)
 *   2  unsupported shape or option (head_dim the entry point does not take, offsets beyond 32 bits, ...)
 *   3  workspace too small
 *   4  HIP launch failure
 * (the reference checks the aclnn status the same way: TORCH_CHECK(apiRet == 0, ...),
 * pytorch_npu_helper.h:646-649).
 *
 * dtype codes: 0 = bf16, 1 = fp16.  All tensors have head_dim D contiguous in memory: D = 128 everywhere,
 * except that the three dense entry points (mindiesd_flash_attention_fwd, mindiesd_flash_attention_general_fwd,
 * mindiesd_flash_attention_packed_fwd) also take every multiple of 8 up to 256 (kernels of their own at 64, up to
 * 128 and up to 256, narrower head dims computed at the next of these widths; the reference's own
 * attention_forward tests run head_dim 64, tests/layers/flash_attn/test_attn_forward.py:31-169).  Pointers must
 * be 16-byte aligned and every stride a multiple of 8 elements.  "strides" are element strides of the
 * (batch, head, token) dimensions, so BNSD and BSND tensors are both passed without a copy.
 */
#ifndef MINDIESD_HIP_H
#define MINDIESD_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* hipStream_t;

/* ---- dense attention -------------------------------------------------------------------------------
 * out = softmax(scale * Q K^T) V per (batch, head); N % Nkv == 0 (grouped-query heads).
 * lse: optional [B][N][Sq] fp32 log-sum-exp of the scaled scores (may be NULL).
 * Replaces the fused kernels behind attention_forward
 * (mindiesd/layers/flash_attn/attention_forward.py:24-89: torch_npu.npu_prompt_flash_attention
 * prompt_flash_attn.py:48, npu_fusion_attention fused_attn_score.py:48, torch.ops.mindiesd.la
 * csrc/plugin/la.cpp:27-58). */
int mindiesd_flash_attention_fwd(const void* q, const void* k, const void* v, void* out, float* lse, int dtype,
                                 int B, int N, int Nkv, int Sq, int Skv, int D,
                                 long long q_sb, long long q_sn, long long q_ss,
                                 long long k_sb, long long k_sn, long long k_ss,
                                 long long v_sb, long long v_sn, long long v_ss,
                                 long long o_sb, long long o_sn, long long o_ss,
                                 float scale, hipStream_t stream);

/* Dense attention with the options of the reference's vendor kernels that the entry point above leaves
 * out:
 *   seq_meta != NULL: packed variable-length sequences (layout "TND").  q/out are [Tq][N][128], k/v
 *     [Tk][Nkv][128] (pass batch strides 0); B = number of sequences, Sq / Skv = the longest query / key
 *     count; seq_meta is a device array int32 [B][4] = {first query token, query count, first key token,
 *     key count}.  Replaces torch_npu.npu_fusion_attention(input_layout="TND", actual_seq_qlen,
 *     actual_seq_kvlen) as called by attention_forward_varlen
 *     (mindiesd/layers/flash_attn/attention_forward_varlen.py:141-149).  lse and mask must be NULL.
 *   causal != 0: key j is visible to query i iff j <= i + (Skv - Sq), the lower triangle aligned to the
 *     bottom-right corner (the vendor kernel's sparse_mode = 3, attention_forward_varlen.py:134-136).
 *   mask != NULL: boolean mask, one byte per (query, key), non-zero = attend, keys contiguous, element
 *     strides m_sb / m_sn (0 = broadcast over batch / heads) and m_sq (>= Skv, or 0 = one row for all queries).
 *     Replaces the atten_mask argument
 *     of the fused wrappers (prompt_flash_attn.py:46-52, fused_attn_score.py:46-52; they pass the
 *     inverted mask, this entry point takes it as the caller of attention_forward gives it).
 * A query row without any visible key gives zeros (and lse = -inf). */
int mindiesd_flash_attention_general_fwd(const void* q, const void* k, const void* v, void* out, float* lse, int dtype,
                                         int B, int N, int Nkv, int Sq, int Skv, int D,
                                         long long q_sb, long long q_sn, long long q_ss,
                                         long long k_sb, long long k_sn, long long k_ss,
                                         long long v_sb, long long v_sn, long long v_ss,
                                         long long o_sb, long long o_sn, long long o_ss,
                                         float scale, const int* seq_meta, int causal,
                                         const unsigned char* mask, long long m_sb, long long m_sn, long long m_sq,
                                         hipStream_t stream);

/* Packed sequences whose lengths only the device knows (cu_seqlens given as device tensors to
 * attention_forward_varlen, mindiesd/layers/flash_attn/attention_forward_varlen.py:45-149; the reference hands
 * them to torch_npu.npu_fusion_attention as actual_seq_qlen / actual_seq_kvlen, :141-149): q, out
 * [total_q][N][D], k, v [total_k][Nkv][D] with element strides of head and token, seq_meta int32 [B][4] as in
 * mindiesd_flash_attention_general_fwd.  The grid is sized from the token totals (at most ceil(total_q / 128) + B
 * query tiles per head exist whatever the lengths are) and every workgroup finds its sequence in the table; the
 * general entry point with Sq = total_q as the only bound launches B times as many.  The query counts of the table
 * must not add up to more than total_q: tiles beyond the bound are not computed.  causal as above. */
int mindiesd_flash_attention_packed_fwd(const void* q, const void* k, const void* v, void* out, int dtype,
                                        int B, int N, int Nkv, int total_q, int total_k, int D,
                                        long long q_sn, long long q_ss, long long k_sn, long long k_ss,
                                        long long v_sn, long long v_ss, long long o_sn, long long o_ss,
                                        float scale, const int* seq_meta, int causal, hipStream_t stream);

/* cu_seqlens_q / cu_seqlens_k as attention_forward_varlen receives them (device arrays, int32, B + 1 entries each;
 * mindiesd/layers/flash_attn/attention_forward_varlen.py:86-89) -> the seq_meta table [B][4] of the two entry points
 * above, built on the device without a host read-back: first tokens are clamped to [0, total], counts to what lies
 * behind them and to max_q / max_k (pass the token totals when the longest sequence is not known).  seq_meta must be
 * 16-byte aligned. */
int mindiesd_varlen_meta(const int* cu_seqlens_q, const int* cu_seqlens_k, int B, int total_q, int total_k,
                         int max_q, int max_k, int* seq_meta, hipStream_t stream);

/* ---- block-sparse attention ------------------------------------------------------------------------
 * Query block i (128 rows) of (b, n) attends to the 128-key blocks blk_idx[b][n][i][0 .. blk_cnt[b][n][i])
 * (ascending ids, int32, row pitch kb_stride); an empty list gives zeros.  `order` (optional,
 * [B*N*ceil(Sq/128)], a permutation of the query block numbers (b*N + n)*ceil(Sq/128) + i) is the sequence
 * in which query blocks are dispatched: workgroup j takes block order[j].
 * Replaces aclnnBlockSparseAttention / aclnnRainFusionAttention behind
 * torch.ops.mindiesd.block_sparse_attention / rainfusionattention
 * (csrc/plugin/block_sparse_attention.cpp:31-121, csrc/plugin/rainfusionattention.cpp:27-64). */
int mindiesd_block_sparse_attention_fwd(const void* q, const void* k, const void* v, void* out, float* lse, int dtype,
                                        int B, int N, int Nkv, int Sq, int Skv, int D,
                                        long long q_sb, long long q_sn, long long q_ss,
                                        long long k_sb, long long k_sn, long long k_ss,
                                        long long v_sb, long long v_sn, long long v_ss,
                                        long long o_sb, long long o_sn, long long o_ss,
                                        float scale, const int* blk_idx, const int* blk_cnt, int kb_stride,
                                        const int* order, hipStream_t stream);

/* The same with the query side addressed through a table (self-attention, S tokens): query position i - the
 * position that the block lists and the rows of k and v refer to - is row token_order[i] of q and of out
 * (every row exactly once).  With the table of mindiesd_rf_token_order, k and v permuted by
 * mindiesd_rf_rearrange_pool and q, out in their original order, this is attention on
 * rearrange_with_remaining(q) followed by inv_rearrange_with_remaining of the result
 * (mindiesd/layers/flash_attn/sparse_flash_attn_rf_v2.py:137-289, sparse_flash_attn_rf_v3.py:22-97, 248-295)
 * without the permuted copy of q and without the inverse pass. */
int mindiesd_block_sparse_attention_gather_fwd(const void* q, const void* k, const void* v, void* out, float* lse,
                                               int dtype, int B, int N, int Nkv, int S, int D,
                                               long long q_sb, long long q_sn, long long q_ss,
                                               long long k_sb, long long k_sn, long long k_ss,
                                               long long v_sb, long long v_sn, long long v_ss,
                                               long long o_sb, long long o_sn, long long o_ss,
                                               float scale, const int* blk_idx, const int* blk_cnt, int kb_stride,
                                               const int* token_order, hipStream_t stream);

/* Block-sparse attention with per-sequence lengths (the actual_seq_lengths / actual_seq_lengths_kv arguments of
 * aclnnBlockSparseAttention, csrc/plugin/block_sparse_attention.cpp:42-66, 100-121): seq_meta int32 [B][4] =
 * {first query token, query count, first key token, key count} as in mindiesd_flash_attention_general_fwd.  Layout
 * "TND": packed [T][N][128] tensors, batch strides 0; layout "BNSD" with shorter sequences: ordinary batch strides,
 * first tokens 0.  Sq / Skv = the longest counts; blk_idx / blk_cnt are per (batch, head, query block) of that
 * length.  lse (optional): [B][N][Sq], or with lse_token_major != 0 [T][N].  Query rows past a sequence's count
 * are not written.  causal != 0: key j visible to query i iff j <= i + (key count - query count). */
int mindiesd_block_sparse_attention_general_fwd(const void* q, const void* k, const void* v, void* out, float* lse,
                                                int dtype, int B, int N, int Nkv, int Sq, int Skv, int D,
                                                long long q_sb, long long q_sn, long long q_ss,
                                                long long k_sb, long long k_sn, long long k_ss,
                                                long long v_sb, long long v_sn, long long v_ss,
                                                long long o_sb, long long o_sn, long long o_ss,
                                                float scale, const int* blk_idx, const int* blk_cnt, int kb_stride,
                                                const int* seq_meta, int lse_token_major, int causal,
                                                hipStream_t stream);

/* Block-sparse attention driven by the int8 mask itself (mask [B][N][ceil(Sq/128)][ceil(Skv/128)], non-zero =
 * attend), over PAIRED query blocks: query blocks of a head whose mask rows overlap most are paired on the device;
 * one 256-row workgroup per pair first walks the key blocks both partners selected (each K/V tile is fetched once for
 * both, the dense kernel's inner loop), then each partner's four waves walk the key blocks only it selected, in
 * 64-key sub-tiles, the running softmax going on.  Same semantics as mindiesd_block_sparse_attention_fwd on the lists
 * of the mask; results differ by the order of the accumulation only, well
 * inside the reference kernels' 2^-6 rule; replaces the same reference kernels.  token_order (optional, self-attention): as in the gather entry
 * point above.  workspace: mindiesd_block_sparse_attention_paired_workspace_size bytes, 16-byte aligned.
 * Returns 2 when the mask is too large for the pairing kernels (more than 2048 key blocks, or mask rows of one
 * head beyond about 150 KiB of bits); the caller then uses the list entry points. */
size_t mindiesd_block_sparse_attention_paired_workspace_size(int B, int N, int Sq, int Skv);
int mindiesd_block_sparse_attention_paired_fwd(const void* q, const void* k, const void* v, void* out, float* lse,
                                               int dtype, int B, int N, int Nkv, int Sq, int Skv, int D,
                                               long long q_sb, long long q_sn, long long q_ss,
                                               long long k_sb, long long k_sn, long long k_ss,
                                               long long v_sb, long long v_sn, long long v_ss,
                                               long long o_sb, long long o_sn, long long o_ss,
                                               float scale, const signed char* mask, const int* token_order,
                                               void* workspace, size_t ws_bytes, hipStream_t stream);

/* token_order[i] (int32, S entries) = row of the original [text | image (t,h,w)] sequence that holds the
 * token at position i of RainFusion's [image in 8x8-window order | text] sequence (the index map behind
 * rearrange_with_remaining, sparse_flash_attn_rf_v2.py:137-196, 297-312). */
int mindiesd_rf_token_order(int* token_order, int S, int t, int h, int w, int txt_len, hipStream_t stream);

/* ---- adaptive block-sparse attention (mask estimate + attention) ------------------------------------------
 * Block-sparse attention as above (queries and keys of equal length S) with an optional causal mask inside
 * the selected blocks: key j is visible to query i iff j <= i.  Replaces aclnnAdaBlockSparseAttention behind
 * torch.ops.mindiesd.ada_block_sparse_attention (csrc/plugin/ada_block_sparse_attention.cpp:27-57); the
 * int8 sparse_mask is turned into lists with mindiesd_mask_to_index first. */
int mindiesd_ada_block_sparse_attention_fwd(const void* q, const void* k, const void* v, void* out, int dtype,
                                            int B, int N, int Nkv, int S, int D,
                                            long long q_sb, long long q_sn, long long q_ss,
                                            long long k_sb, long long k_sn, long long k_ss,
                                            long long v_sb, long long v_sn, long long v_ss,
                                            long long o_sb, long long o_sn, long long o_ss,
                                            float scale, const int* blk_idx, const int* blk_cnt, int kb_stride,
                                            int causal, hipStream_t stream);

/* Mask estimate: aclnnSparseBlockEstimate (csrc/plugin/sparse_block_estimate.cpp:27-85,
 * csrc/ops/sparse_block_estimate/op_kernel/sparse_block_estimate.h; numpy statement
 * tests/plugin/test_sparseblockestimate.py:49-145) in two calls.
 * mindiesd_sbe_scores: q [B][N][S][128], k [B][Nkv][S][128] (element strides as above) -> scores fp32
 *   [B * N][NB][NB], NB = ceil(S / 128): scores[bn][I][J] = sum over the 16 x 16 block (I, J) of
 *   softmax_j(scale * P'), with the anti-diagonal strided products P'[i][j] = sum_{s<8} q[8i+7-s] . k[8j+s]
 *   (tokens past S count as zeros; the caller passes scale = softmax scale / 8).  P' is never stored.
 *   workspace: mindiesd_sbe_scores_workspace_size(B * N, S) bytes, or less - any size that holds one head works,
 *   the heads are then processed in groups.
 *   causal != 0 (test_sparseblockestimate.py:71-78): the rows of one step of 1024 query tokens see the strided
 *   columns below min(S / 8, 128 * (step + 1)); scores beyond are zero.
 * mindiesd_sbe_select (sparse_block_estimate.h:947-1078): per block row, the key blocks take part that the row may
 *   see (all NB, or with causal the first I + 1; causal rows with at most 2 keep them all).  The last of them (if
 *   keep_recent or not causal) and the first (if keep_sink) are left out of the ranking and forced afterwards; the
 *   others are kept in descending score order until their running sum reaches threshold * their total
 *   (threshold >= 1 keeps all), at most row_sparse * blocks of them when at least 10 take part; block 0 is always
 *   kept.  mask int8 [BN][NB][pitch] (pitch >= NB, zero padded; the reference uses NB rounded up to 32), count
 *   int32 [BN][NB]. */
size_t mindiesd_sbe_scores_workspace_size(int heads, int S);
int mindiesd_sbe_scores(const void* q, const void* k, float* scores, int dtype, int B, int N, int Nkv, int S, int D,
                        long long q_sb, long long q_sn, long long q_ss, long long k_sb, long long k_sn, long long k_ss,
                        float scale, int causal, void* workspace, size_t ws_bytes, hipStream_t stream);
int mindiesd_sbe_select(const float* scores, signed char* mask, int* count, int BN, int NB, int pitch,
                        float threshold, float row_sparse, int keep_sink, int keep_recent, int causal,
                        hipStream_t stream);

/* ---- RainFusion2.0 mask pipeline ---------------------------------------------------------------------
 * Token permutation into 8x8 spatial windows (+ optional block mean pooling) of up to three tensors
 * of one shape; replaces rearrange_with_remaining / avgpool / do_tensor_rearrange_pooling /
 * inv_rearrange_with_remaining (mindiesd/layers/flash_attn/sparse_flash_attn_rf_v2.py:24-73,
 * :137-317).  The sequence is [txt_len text tokens | t*h*w image tokens]; the permuted sequence is
 * [image in window order | text].  t == 0 selects the identity order (pooling only).  inverse != 0
 * undoes the permutation.  q_out/k_out/v_out may be NULL (pool only); pool may be NULL (permute only).
 * pool: 16-bit [n_tensors][B][N][blocks][128] addressed with strides p_st (tensor), p_sb, p_sn,
 * p_sblk; blocks = ceil(image/128) + ceil(text/128), each block averaged over its own length. */
int mindiesd_rf_rearrange_pool(const void* q, const void* k, const void* v, void* q_out, void* k_out, void* v_out,
                               void* pool, int dtype, int B, int N, int S, int D,
                               long long s_sb, long long s_sn, long long s_ss,
                               long long d_sb, long long d_sn, long long d_ss,
                               long long p_st, long long p_sb, long long p_sn, long long p_sblk,
                               int t, int h, int w, int txt_len, int inverse, int n_tensors, hipStream_t stream);

/* Block mask from pooled q/k (get_blockwise_mask + get_mask_index, sparse_flash_attn_rf_v2.py:76-134):
 * keep[b][n][i][j] = softmax_j(q_pool_i . k_pool_j * scale) >= keep_len-th largest of row i,
 * OR i/j inside the last txt_blocks or the first ff_blocks blocks, OR (keep_diag and i == j);
 * scores and probabilities are rounded to the 16-bit input type at the reference's rounding points.
 * Outputs (each optional): mask int8 [B][N][NB][NB]; blk_idx int32 [B][N][NB][kb_stride] ascending,
 * -1 padded, with blk_cnt int32 [B][N][NB]; select_idx int64 [NB][N][NB] / select_num int64 [NB][N]
 * (batch 0, the reference's layout). */
int mindiesd_rf_block_mask(const void* q_pool, const void* k_pool, int dtype, int B, int N, int NB, int D,
                           long long p_sb, long long p_sn, long long p_sblk, float scale, int keep_len,
                           int txt_blocks, int ff_blocks, int keep_diag, signed char* mask, int* blk_idx,
                           int* blk_cnt, int kb_stride, long long* select_idx, long long* select_num,
                           hipStream_t stream);

/* int8 mask [BN][QB][KB] (non-zero = attend) -> ascending index lists + counts (the form
 * mindiesd_block_sparse_attention_fwd consumes). */
int mindiesd_mask_to_index(const signed char* mask, int BN, int QB, int KB, int* blk_idx, int* blk_cnt,
                           int kb_stride, hipStream_t stream);

/* ---- FP8 attention -----------------------------------------------------------------------------------
 * Block quantisation of one attention operand: x [B][N][S][128] 16-bit (strided) ->
 * q [B][N][S][128] E4M3 bytes + scale fp32 [B][N][ceil(S/block_size)], scale = amax/448 per block of
 * block_size (128/256/512) tokens x 128 channels.  Replaces torch_npu.npu_dynamic_block_quant as
 * called by fa_block_quant_preprocess (mindiesd/layers/quant/block_quant.py:19-48) with prescale 1 and
 * pow2_scale 0.  prescale (> 0) multiplies x before the quantisation; pow2_scale != 0 rounds the scale up to a
 * power of two (no counterpart in the reference: the recipe of the log2-domain attention kernel below). */
int mindiesd_fa_block_quant(const void* x, void* q, float* scale, int dtype, int B, int N, int S, int D,
                            long long x_sb, long long x_sn, long long x_ss, int block_size, float prescale,
                            int pow2_scale, hipStream_t stream);

/* Rotation fused into the quantisation pass: y = x @ rot ([128][128], passed transposed as rot_t, same
 * 16-bit type as x), y rounded to the 16-bit type, then quantised as above with block_size 128.  Replaces
 * torch.matmul(query, self.q_rot) / torch.matmul(key, self.k_rot) followed by fa_block_quant_preprocess in
 * FP8RotateQuantFA.forward (mindiesd/quantization/layer.py:283-296). */
int mindiesd_fa_rot_block_quant(const void* x, const void* rot_t, void* q, float* scale, int dtype, int B, int N, int S,
                                int D, long long x_sb, long long x_sn, long long x_ss, float prescale, int pow2_scale,
                                hipStream_t stream);

/* V for the FP8 kernel: per-(batch, head, channel) scale = amax/448 over the sequence, codes written
 * transposed ([B][N][128][S rounded up to 128], zero padded, keys permuted inside groups of 64 into
 * the order the matrix instruction consumes).  workspace: mindiesd_fp8_v_quant_workspace_size bytes. */
size_t mindiesd_fp8_v_quant_workspace_size(int B, int N);
int mindiesd_fp8_v_quant(const void* v, void* v8t, float* v_scale, int dtype, int B, int N, int S, int D,
                         long long v_sb, long long v_sn, long long v_ss, void* workspace, size_t ws_bytes,
                         hipStream_t stream);

/* mindiesd_fp8_v_quant for callers that cannot allocate (code under HIP graph capture, serving loops and
 * harnesses that forbid hipMalloc); it has no counterpart in the reference.  Same inputs, outputs and results,
 * no workspace argument: the per-channel maxima live in a fixed device array inside the library (2 MiB per GPU,
 * held until the process ends), which limits B * N to mindiesd_fp8_v_quant_static_max_heads() = 4096 (beyond
 * that: return code 3).  Nothing is allocated or freed, no stream is synchronised.  All calls on one GPU share
 * that array: calls that overlap on one GPU (different streams or threads) race and must be serialised by the
 * caller. */
int mindiesd_fp8_v_quant_static_max_heads(void);
int mindiesd_fp8_v_quant_static(const void* v, void* v8t, float* v_scale, int dtype, int B, int N, int S, int D,
                                long long v_sb, long long v_sn, long long v_ss, hipStream_t stream);

/* FP8 flash attention on operands produced by the two functions above (Q/K with block_size 128).
 * Replaces torch_npu.npu_fused_infer_attention_score_v2 with per-block dequantisation scales as
 * called by FP8RotateQuantFA.forward (mindiesd/quantization/layer.py:304-316).
 * flags (bits, 0 = the default):
 *   MSD_FP8_LOG2_DOMAIN  q_scale and k_scale hold powers of two and the query was quantised with
 *                        prescale = softmax scale * log2(e) (pow2_scale quantisation above); the scales are then
 *                        applied by the matrix instruction's exponent operands and `scale` is not used.
 *   MSD_FP8_P_EXP2       the probabilities of a tile are 2^(score - reference) by the exponential instruction, rounded
 *                        to E4M3 (the older, slower rule).  Default: the E4M3 code of a probability is computed
 *                        directly as round(8 * (score - reference) + const), i.e. the exponential with its mantissa
 *                        interpolated linearly between powers of two; the denominator is summed from the same codes.
 *   MSD_FP8_K_BLOCK_256  k_scale holds one scale per 256 keys ([B][N][ceil(Skv/256)], mindiesd_fa_block_quant with
 *                        block_size 256 - the K recipe of FP8RotateQuantFA, mindiesd/quantization/layer.py:297-302)
 *                        instead of one per 128. */
#define MSD_FP8_LOG2_DOMAIN 1
#define MSD_FP8_P_EXP2 2
#define MSD_FP8_K_BLOCK_256 4
int mindiesd_fp8_attention_fwd(const void* q8, const void* k8, const void* v8t, const float* q_scale,
                               const float* k_scale, const float* v_scale, void* out, int out_dtype, int B, int N,
                               int Sq, int Skv, int D, long long o_sb, long long o_sn, long long o_ss, float scale,
                               int flags, hipStream_t stream);

/* ---- MXFP8 linear layer --------------------------------------------------------------------------------
 * x [M][K] 16-bit (row stride x_stride elements) -> q [M][K] E4M3 + e8m0 [M][K/32]
 * (OCP MX: shared scale 2^(floor(log2(amax)) - 8) per 32 elements).  Replaces
 * torch_npu.npu_dynamic_mx_quant (mindiesd/quantization/layer.py:338-341). */
int mindiesd_mx_quant(const void* x, void* q, void* e8m0, int dtype, long long M, int K, long long x_stride,
                      hipStream_t stream);

/* out[M][Nout] = act(X W^T + bias) on MX-quantised operands (a [M][K], a_scale [M][K/32], w [Nw][K],
 * w_scale [Nw][K/32], bias fp32 [Nw] or NULL).  swiglu == 0: Nout = Nw.  swiglu != 0: W holds
 * [gate rows | up rows], Nout = Nw/2 and out = silu(gate) * up, computed on the accumulators.
 * Replaces torch_npu.npu_quant_matmul(..., group_sizes=[1,1,32]) (mindiesd/quantization/layer.py:351-361);
 * the fused SwiGLU has no counterpart in the reference, which applies nn.SiLU afterwards
 * (mindiesd/layers/activation.py:34-61). */
int mindiesd_mxfp8_gemm(const void* a, const void* a_scale, const void* w, const void* w_scale, const float* bias,
                        void* out, int out_dtype, int M, int K, int Nw, int swiglu, hipStream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MINDIESD_HIP_H */

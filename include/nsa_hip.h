/* C ABI of libnsa_hip.so: MI355X (gfx950) kernels for the Native-Sparse-Attention hot path.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless stated otherwise; tensors are bf16 unless stated otherwise;
 *   - strides are in ELEMENTS; "_st" = token/row stride, "_sh" = head stride; the channel dim is contiguous;
 *   - packed variable-length batches: x_cu [B+1] int32 token offsets, y_cu [B+1] int32 compressed-row offsets
 *     (y_len = max((L-kernel)/stride+1, 0) per sequence);
 *   - `stream` is a hipStream_t passed as void*; kernels are enqueued, never synchronised;
 *   - return value: 0 = ok, otherwise an error code; nsa_last_error() gives the message (thread local);
 *   - log-sum-exp outputs are in log2 units (m + log2(l)), as upstream stores them.
 * Citations name the upstream (mdy666/Scalable-Flash-Native-Sparse-Attention) interface each entry replaces.
 */
#ifndef NSA_HIP_H
#define NSA_HIP_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

const char* nsa_last_error(void);
int nsa_abi_version(void);
/* Overrides one of the library's launch heuristics for this process (experiments and tests; nothing is read from
 * the environment): name (host string) = "fwd_variant", "dq_min_blocks", "dkdv_key_blocks" or "topk_seg_blocks"
 * (selection blocks per segment of the block selector: -1 = from the LDS budget, 0 = never segment).
 * nsa_reset_tuning restores every default.  No upstream counterpart. */
int nsa_set_tuning(const char* name, int value);
int nsa_reset_tuning(void);

/* flash_nsa/ops/compress_kv.py:335-366 mean_pooling_fwd */
int nsa_mean_pool_fwd(const void* x, int64_t x_st, int64_t x_sh, void* y, int64_t y_st, int64_t y_sh,
                      const int32_t* x_cu, const int32_t* y_cu, int B, int y_maxlen, int H, int D, int kernel_size,
                      int stride, void* stream);
/* flash_nsa/ops/compress_kv.py:368-399 mean_pooling_bwd; dx fp32 (optionally accumulated into) or bf16 */
int nsa_mean_pool_bwd(const void* dy, int64_t dy_st, int64_t dy_sh, void* dx, int64_t dx_st, int64_t dx_sh,
                      int dx_is_f32, int accumulate, const int32_t* x_cu, const int32_t* y_cu, int B, int x_maxlen,
                      int H, int D, int kernel_size, int stride, void* stream);
/* flash_nsa/ops/compress_kv.py:126-170 construct_block_fwd; y contiguous [y_len,H,kernel,D] */
int nsa_construct_block_fwd(const void* x, int64_t x_st, int64_t x_sh, void* y, const int32_t* x_cu,
                            const int32_t* y_cu, int B, int y_maxlen, int H, int D, int kernel_size, int stride,
                            void* stream);
/* flash_nsa/ops/compress_kv.py:172-218 construct_block_bwd */
int nsa_construct_block_bwd(const void* dblock, void* dx, int64_t dx_st, int64_t dx_sh, int dx_is_f32,
                            int accumulate, const int32_t* x_cu, const int32_t* y_cu, int B, int x_maxlen, int H,
                            int D, int kernel_size, int stride, void* stream);
/* flash_nsa/ops/act.py:175-208 sigmoid_mul_fwd/bwd (act 0) and :60-100 swiglu_fwd/bwd (act 1);
 * x [N,2d] = gate|up, y [N,d], dx [N,2d] = dgate|dup (dx may alias x) */
int nsa_glu_fwd(const void* x, void* y, int64_t N, int d, int act, void* stream);
int nsa_glu_bwd(const void* x, const void* dy, void* dx, int64_t N, int d, int act, void* stream);

/* flash_nsa/ops/combine.py:114-144 combine_fwd */
int nsa_combine_fwd(const void* a, const void* b, const void* c, int64_t i_st, int64_t i_sh, const void* w,
                    int64_t w_st, int64_t w_sh, void* o, int64_t o_st, int64_t o_sh, int64_t T, int H, int D,
                    void* stream);
/* flash_nsa/ops/combine.py:146-177 combine_bwd; da/db/dc contiguous [T,H,D], dw [T,H,3];
 * delta3 (optional, fp32 [3,T,H]) receives rowsum(x_k * dx_k) for the three branches */
int nsa_combine_bwd(const void* a, const void* b, const void* c, int64_t i_st, int64_t i_sh, const void* w,
                    int64_t w_st, int64_t w_sh, const void* dy, int64_t dy_st, int64_t dy_sh, void* da, void* db,
                    void* dc, void* dw, float* delta3, int64_t T, int H, int D, void* stream);
/* flash_nsa/ops/compress_attn.py:160-184 _bwd_preprocess: delta[T,H] fp32 = rowsum(o*do) */
int nsa_delta(const void* o, int64_t o_st, int64_t o_sh, const void* dO, int64_t d_st, int64_t d_sh, float* delta,
              int64_t T, int H, int D, void* stream);

/* flash_nsa/ops/compress_attn.py:531-592 cmp_attn_fwd; lse addressed tok*lse_st + head*lse_sh */
int nsa_cmp_attn_fwd(const void* q, int64_t q_st, int64_t q_sh, const void* ck, int64_t ck_sr, int64_t ck_sh,
                     const void* cv, int64_t cv_sr, int64_t cv_sh, void* o, int64_t o_st, int64_t o_sh, float* lse,
                     int64_t lse_st, int64_t lse_sh, const int32_t* x_cu, const int32_t* y_cu, int B, int x_maxlen,
                     int QH, int KH, int D, int VD, int kernel_size, int stride, float sm_scale, void* stream);
/* flash_nsa/ops/sliding_window_attention.py:42-95 swa_fwd (FlashAttention varlen, window=(W,-1), causal) */
int nsa_swa_fwd(const void* q, int64_t q_st, int64_t q_sh, const void* k, int64_t k_sr, int64_t k_sh,
                const void* v, int64_t v_sr, int64_t v_sh, void* o, int64_t o_st, int64_t o_sh, float* lse,
                int64_t lse_st, int64_t lse_sh, const int32_t* x_cu, int B, int x_maxlen, int QH, int KH, int D,
                int VD, int window, float sm_scale, void* stream);
/* flash_nsa/ops/topk.py:630-775 slc_topk_indices; topk int32 addressed kh*tk_sh + tok*tk_st + slot;
 * imp_out optional fp32 block scores [KH, T, imp_cols] */
int nsa_topk_select(const void* q, int64_t q_st, int64_t q_sh, const void* ck, int64_t ck_sr, int64_t ck_sh,
                    const float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk, int64_t tk_sh, int64_t tk_st,
                    float* imp_out, int64_t imp_sh, int64_t imp_st, int imp_cols, const int32_t* x_cu,
                    const int32_t* y_cu, int B, int x_maxlen, int QH, int KH, int D, int kernel_size, int stride,
                    int block_size, int top_n, int num_init, int num_local, int ignore_index, float sm_scale,
                    void* stream);
/* The same selection in two launches, the fp32 block scores between them in `workspace` (upstream keeps them in its
 * slc_probs tensor between its two kernels, flash_nsa/ops/topk.py:226-425, 498-560): scoring then runs at twice the
 * occupancy of the one-launch kernel, which keeps the scores of its tokens in LDS.  total_tokens = tokens of the packed
 * batch (x_cu[B]).  nsa_topk_workspace_bytes(total_tokens, max_blocks, KH), max_blocks = selection blocks of the
 * longest sequence, is what one pass over all tokens needs; a smaller workspace makes the call work in chunks of as
 * many tokens as it holds (identical results).  workspace NULL, or a shape the two launches do not take (more than 16
 * q-heads per kv head, more than 2048 selection blocks, block sizes that are not 1..64 strides in powers of two):
 * the one-launch kernel runs, as in nsa_topk_select.  The workspace is scratch: nothing is kept between calls. */
int64_t nsa_topk_workspace_bytes(int total_tokens, int max_blocks, int KH);
int nsa_topk_select_ws(const void* q, int64_t q_st, int64_t q_sh, const void* ck, int64_t ck_sr, int64_t ck_sh,
                       const float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk, int64_t tk_sh, int64_t tk_st,
                       float* imp_out, int64_t imp_sh, int64_t imp_st, int imp_cols, const int32_t* x_cu,
                       const int32_t* y_cu, int B, int x_maxlen, int QH, int KH, int D, int kernel_size, int stride,
                       int block_size, int top_n, int num_init, int num_local, int ignore_index, float sm_scale,
                       int total_tokens, void* workspace, int64_t workspace_bytes, void* stream);
/* flash_nsa/ops/select_attn.py:439-507 slc_attn_fwd */
int nsa_slc_attn_fwd(const void* q, int64_t q_st, int64_t q_sh, const void* k, int64_t k_sr, int64_t k_sh,
                     const void* v, int64_t v_sr, int64_t v_sh, const int32_t* topk, int64_t tk_sh, int64_t tk_st,
                     void* o, int64_t o_st, int64_t o_sh, float* lse, int64_t lse_st, int64_t lse_sh,
                     const int32_t* x_cu, int B, int x_maxlen, int QH, int KH, int D, int VD, int block_size,
                     int top_n, float sm_scale, void* stream);

/* ---- backward ----
 * dq_mode: 0 = store bf16, 1 = store fp32, 2 = add into an existing fp32 buffer (single writer per element).
 * delta = rowsum(o * do) of the branch, fp32; lse as produced by the matching forward. */

/* flash_nsa/ops/compress_attn.py:701-736 (_cmp_dq_kernel launch) */
int nsa_cmp_attn_bwd_dq(const void* q, int64_t q_st, int64_t q_sh, const void* ck, int64_t ck_sr, int64_t ck_sh,
                        const void* cv, int64_t cv_sr, int64_t cv_sh, const void* dO, int64_t do_st, int64_t do_sh,
                        const float* lse, int64_t lse_st, int64_t lse_sh, const float* delta, int64_t delta_st,
                        int64_t delta_sh, void* dq, int64_t dq_st, int64_t dq_sh, int dq_mode, const int32_t* x_cu,
                        const int32_t* y_cu, int B, int x_maxlen, int QH, int KH, int D, int VD, int kernel_size,
                        int stride, float sm_scale, void* stream);
/* Same kernel as nsa_cmp_attn_bwd_dq, as the LAST branch of the fused backward
 * (flash_nsa/modules/megatron_level_nsa.py:129-159 accumulates the three branches' dq and returns it in q's dtype):
 * dq [T,QH,D] bf16 = this branch's dq + dq_partial (fp32, the sum of the other branches), which saves the fp32
 * read-modify-write and the separate cast pass. */
int nsa_cmp_attn_bwd_dq_final(const void* q, int64_t q_st, int64_t q_sh, const void* ck, int64_t ck_sr,
                              int64_t ck_sh, const void* cv, int64_t cv_sr, int64_t cv_sh, const void* dO,
                              int64_t do_st, int64_t do_sh, const float* lse, int64_t lse_st, int64_t lse_sh,
                              const float* delta, int64_t delta_st, int64_t delta_sh, const float* dq_partial,
                              int64_t dqp_st, int64_t dqp_sh, void* dq, int64_t dq_st, int64_t dq_sh,
                              const int32_t* x_cu, const int32_t* y_cu, int B, int x_maxlen, int QH, int KH, int D,
                              int VD, int kernel_size, int stride, float sm_scale, void* stream);
/* flash_nsa/ops/compress_attn.py:650-690 (_cmp_dkdv_kernel launch, dkdv_repeat=False): fp32 atomic adds into
 * dck/dcv [y_len,KH,*], which the caller zero-fills; queries are cut into chunks of q_chunk_tokens
 * (<= 0: chosen from the sizes so that short batches still fill the GPU) */
int nsa_cmp_attn_bwd_dkdv(const void* q, int64_t q_st, int64_t q_sh, const void* ck, int64_t ck_sr, int64_t ck_sh,
                          const void* cv, int64_t cv_sr, int64_t cv_sh, const void* dO, int64_t do_st,
                          int64_t do_sh, const float* lse, int64_t lse_st, int64_t lse_sh, const float* delta,
                          int64_t delta_st, int64_t delta_sh, float* dck, int64_t dck_sr, int64_t dck_sh,
                          float* dcv, int64_t dcv_sr, int64_t dcv_sh, const int32_t* x_cu, const int32_t* y_cu,
                          int B, int x_maxlen, int y_maxlen, int QH, int KH, int D, int VD, int kernel_size,
                          int stride, int q_chunk_tokens, float sm_scale, void* stream);
/* The same with a summation order that does not depend on the run (upstream's dkdv_repeat=True: per-head buffers and a
 * final sum, flash_nsa/ops/compress_attn.py:594-598,691-693; here the q-heads of a group are summed inside the matrix
 * accumulators and what remains to be ordered are the query chunks): every work item stores its fp32 partial result
 * in its own slot of `workspace` (nsa_cmp_attn_bwd_dkdv_det_bytes(...) bytes, same sizes and q_chunk_tokens as the
 * call), a second launch sums the slots of a key in ascending chunk order and stores dck / dcv (no zero-fill needed
 * for the keys it writes; keys no query sees keep what the buffers held). */
int64_t nsa_cmp_attn_bwd_dkdv_det_bytes(int B, int x_maxlen, int y_maxlen, int QH, int KH, int D, int VD,
                                        int kernel_size, int stride, int q_chunk_tokens);
int nsa_cmp_attn_bwd_dkdv_det(const void* q, int64_t q_st, int64_t q_sh, const void* ck, int64_t ck_sr,
                              int64_t ck_sh, const void* cv, int64_t cv_sr, int64_t cv_sh, const void* dO,
                              int64_t do_st, int64_t do_sh, const float* lse, int64_t lse_st, int64_t lse_sh,
                              const float* delta, int64_t delta_st, int64_t delta_sh, float* dck, int64_t dck_sr,
                              int64_t dck_sh, float* dcv, int64_t dcv_sr, int64_t dcv_sh, const int32_t* x_cu,
                              const int32_t* y_cu, int B, int x_maxlen, int y_maxlen, int QH, int KH, int D, int VD,
                              int kernel_size, int stride, int q_chunk_tokens, float sm_scale, void* workspace,
                              int64_t workspace_bytes, void* stream);
/* flash_nsa/ops/sliding_window_attention.py:98-157 swa_bwd (FlashAttention varlen backward) */
int nsa_swa_bwd_dq(const void* q, int64_t q_st, int64_t q_sh, const void* k, int64_t k_sr, int64_t k_sh,
                   const void* v, int64_t v_sr, int64_t v_sh, const void* dO, int64_t do_st, int64_t do_sh,
                   const float* lse, int64_t lse_st, int64_t lse_sh, const float* delta, int64_t delta_st,
                   int64_t delta_sh, void* dq, int64_t dq_st, int64_t dq_sh, int dq_mode, const int32_t* x_cu,
                   int B, int x_maxlen, int QH, int KH, int D, int VD, int window, float sm_scale, void* stream);
/* same upstream site; dk/dv are stored (every key row has exactly one writer), bf16 or fp32 */
int nsa_swa_bwd_dkdv(const void* q, int64_t q_st, int64_t q_sh, const void* k, int64_t k_sr, int64_t k_sh,
                     const void* v, int64_t v_sr, int64_t v_sh, const void* dO, int64_t do_st, int64_t do_sh,
                     const float* lse, int64_t lse_st, int64_t lse_sh, const float* delta, int64_t delta_st,
                     int64_t delta_sh, void* dk, int64_t dk_sr, int64_t dk_sh, void* dv, int64_t dv_sr,
                     int64_t dv_sh, int dkv_is_f32, const int32_t* x_cu, int B, int x_maxlen, int QH, int KH, int D,
                     int VD, int window, float sm_scale, void* stream);
/* flash_nsa/ops/select_attn.py:650-695 (_dq_kernel launch) */
int nsa_slc_attn_bwd_dq(const void* q, int64_t q_st, int64_t q_sh, const void* k, int64_t k_sr, int64_t k_sh,
                        const void* v, int64_t v_sr, int64_t v_sh, const void* dO, int64_t do_st, int64_t do_sh,
                        const float* lse, int64_t lse_st, int64_t lse_sh, const float* delta, int64_t delta_st,
                        int64_t delta_sh, const int32_t* topk, int64_t tk_sh, int64_t tk_st, void* dq,
                        int64_t dq_st, int64_t dq_sh, int dq_mode, const int32_t* x_cu, int B, int x_maxlen, int QH,
                        int KH, int D, int VD, int block_size, int top_n, float sm_scale, void* stream);
/* flash_nsa/ops/topk.py:889-945 get_bind_from_find: inverse of the selection as a CSR.
 *   csr_off  [KH][nblk_total+1] absolute start of each (kv head, global block) list inside csr_tok
 *   csr_tok  [KH*T*top_n]       query tokens (index local to their sequence), ascending within a list
 *   item_off [KH][nblk_total+1] prefix count of list chunks of chunk_tokens tokens (work items of the dk/dv pass)
 *   workspace: int32 scratch of nsa_inverse_index_workspace_elems(T,KH,nblk_total) elements
 * nsa_slc_bwd_chunk_tokens: the chunk_tokens this library suggests for a batch of T tokens (1024 for long batches,
 * less when that would leave the dk/dv pass too few work items); any positive value is valid as long as the
 * builder and nsa_slc_attn_bwd_dkdv get the same one */
int64_t nsa_inverse_index_workspace_elems(int T, int KH, int nblk_total);
int nsa_slc_bwd_chunk_tokens(int T, int KH, int top_n);
int nsa_build_inverse_index(const int32_t* topk, int64_t tk_sh, int64_t tk_st, int top_n, const int32_t* x_cu,
                            const int32_t* kblk_cu, int B, int T, int KH, int nblk_total, int block_size,
                            int chunk_tokens, int32_t* csr_off, int32_t* csr_tok, int32_t* item_off,
                            int32_t* workspace, int64_t workspace_elems, void* stream);
/* flash_nsa/ops/select_attn.py:593-637 (_dkdv_kernel launch): fp32 atomic adds into dk/dv [T,KH,*];
 * blk_seq [nblk_total] = sequence of each global block; n_items_bound >= max over kv heads of item_off[kh][nblk_total] */
int nsa_slc_attn_bwd_dkdv(const void* q, int64_t q_st, int64_t q_sh, const void* k, int64_t k_sr, int64_t k_sh,
                          const void* v, int64_t v_sr, int64_t v_sh, const void* dO, int64_t do_st,
                          int64_t do_sh, const float* lse, int64_t lse_st, int64_t lse_sh, const float* delta,
                          int64_t delta_st, int64_t delta_sh, float* dk, int64_t dk_sr, int64_t dk_sh, float* dv,
                          int64_t dv_sr, int64_t dv_sh, const int32_t* x_cu, const int32_t* kblk_cu,
                          const int32_t* blk_seq, const int32_t* csr_off, const int32_t* csr_tok,
                          const int32_t* item_off, int nblk_total, int chunk_tokens, int n_items_bound, int B,
                          int QH, int KH, int D, int VD, int block_size, float sm_scale, void* stream);
/* The same with a run-independent summation order (upstream's dkdv_repeat=True, flash_nsa/ops/select_attn.py:528-531,
 * 639-641): every work item (a chunk of a block's token list) stores its partial result in its own slot of
 * `workspace` (nsa_slc_attn_bwd_dkdv_det_bytes(...) bytes), a second launch adds the slots of a block to dk / dv in
 * ascending chunk order, one thread per element. */
int64_t nsa_slc_attn_bwd_dkdv_det_bytes(int n_items_bound, int KH, int D, int VD, int block_size);
int nsa_slc_attn_bwd_dkdv_det(const void* q, int64_t q_st, int64_t q_sh, const void* k, int64_t k_sr, int64_t k_sh,
                              const void* v, int64_t v_sr, int64_t v_sh, const void* dO, int64_t do_st,
                              int64_t do_sh, const float* lse, int64_t lse_st, int64_t lse_sh, const float* delta,
                              int64_t delta_st, int64_t delta_sh, float* dk, int64_t dk_sr, int64_t dk_sh,
                              float* dv, int64_t dv_sr, int64_t dv_sh, const int32_t* x_cu, const int32_t* kblk_cu,
                              const int32_t* blk_seq, const int32_t* csr_off, const int32_t* csr_tok,
                              const int32_t* item_off, int nblk_total, int chunk_tokens, int n_items_bound, int B,
                              int QH, int KH, int D, int VD, int block_size, float sm_scale, void* workspace,
                              int64_t workspace_bytes, void* stream);

/* ---- paged KV (inference).  Caches are [num_pages, page_size, KH, D]; *_sr is the stride of a flat row
 * (page*page_size + offset), *_sh the head stride.  Request b's raw token n lives at flat row
 * block_tables[b][n/page]*page + n%page; its compressed row i at cmp_block_tables[b][i/page]*page + i%page of the
 * SAME pool.  x_cu counts only the new query tokens; query n of request b sits at absolute position
 * n + context_lens[b] - x_len[b].  page_size must be a multiple of 64. */

/* flash_nsa/inference/compress_attn.py:486-538 cmp_attn_prefill (and, with one query per request, :540-667 decode) */
int nsa_paged_cmp_attn_fwd(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr,
                           int64_t k_sh, const void* v_cache, int64_t v_sr, int64_t v_sh, void* o, int64_t o_st,
                           int64_t o_sh, float* lse, int64_t lse_st, int64_t lse_sh, const int32_t* x_cu,
                           const int32_t* context_lens, const int32_t* cmp_block_tables, int table_stride,
                           int page_size, int B, int x_maxlen, int QH, int KH, int D, int VD, int kernel_size,
                           int stride, float sm_scale, void* stream);
/* flash_nsa/inference/__init__.py:125-155 (FlashAttention with page table and window) */
int nsa_paged_swa_fwd(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr, int64_t k_sh,
                      const void* v_cache, int64_t v_sr, int64_t v_sh, void* o, int64_t o_st, int64_t o_sh,
                      float* lse, int64_t lse_st, int64_t lse_sh, const int32_t* x_cu, const int32_t* context_lens,
                      const int32_t* block_tables, int table_stride, int page_size, int B, int x_maxlen, int QH,
                      int KH, int D, int VD, int window, float sm_scale, void* stream);
/* flash_nsa/inference/topk.py:184-298 topk_prefill / :495-623 topk_decode (causality is masked per row here) */
int nsa_paged_topk_select(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr,
                          int64_t k_sh, const float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk,
                          int64_t tk_sh, int64_t tk_st, const int32_t* x_cu, const int32_t* context_lens,
                          const int32_t* cmp_block_tables, int table_stride, int page_size, int B, int x_maxlen,
                          int fixed_num_slc_blocks, int QH, int KH, int D, int kernel_size, int stride,
                          int block_size, int top_n, int num_init, int num_local, int ignore_index, float sm_scale,
                          void* stream);
/* nsa_paged_topk_select in two launches with a workspace, as nsa_topk_select_ws (max_blocks = fixed_num_slc_blocks) */
int nsa_paged_topk_select_ws(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr,
                             int64_t k_sh, const float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk,
                             int64_t tk_sh, int64_t tk_st, const int32_t* x_cu, const int32_t* context_lens,
                             const int32_t* cmp_block_tables, int table_stride, int page_size, int B, int x_maxlen,
                             int fixed_num_slc_blocks, int QH, int KH, int D, int kernel_size, int stride,
                             int block_size, int top_n, int num_init, int num_local, int ignore_index,
                             float sm_scale, int total_tokens, void* workspace, int64_t workspace_bytes,
                             void* stream);
/* flash_nsa/inference/select_attn.py:103-166 slc_attn_prefill */
int nsa_paged_slc_attn_fwd(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr,
                           int64_t k_sh, const void* v_cache, int64_t v_sr, int64_t v_sh, const int32_t* topk,
                           int64_t tk_sh, int64_t tk_st, void* o, int64_t o_st, int64_t o_sh, float* lse,
                           int64_t lse_st, int64_t lse_sh, const int32_t* x_cu, const int32_t* context_lens,
                           const int32_t* block_tables, int table_stride, int page_size, int B, int x_maxlen,
                           int QH, int KH, int D, int VD, int block_size, int top_n, float sm_scale, void* stream);

/* flash_nsa/inference/compress_kv.py:191-220 mean_pooling_prefill (in-pool write at flat row slot) */
int nsa_paged_pool_prefill(void* cache, int64_t c_sr, int64_t c_sh, const int32_t* y_cu, const int32_t* block_tables,
                           int table_stride, const int32_t* cmp_slot_mapping, int B, int y_maxlen, int page_size,
                           int H, int D, int kernel_size, int stride, void* stream);
/* flash_nsa/inference/compress_kv.py:253-287 kv_mean_pooling_decode */
int nsa_paged_pool_decode(void* k_cache, int64_t k_sr, int64_t k_sh, int Dk, void* v_cache, int64_t v_sr,
                          int64_t v_sh, int Dv, const int32_t* context_lens, const int32_t* block_tables,
                          int table_stride, const int32_t* cmp_slot_mapping, int B, int page_size, int H,
                          int kernel_size, int stride, void* stream);

/* ---- the layer around the core ----
 * flash_nsa/ops/rope.py:13-232 fused_apply_rope: rotate-half RoPE of q [B,N,QH,D] and k [B,N,KH,D] (element strides
 * per batch / token / head, last dim contiguous) with cos / sin [B,N,D] (bf16, or fp32 when cos_is_fp32; a batch
 * stride of 0 broadcasts one table); qe / ke may alias q / k (in place).  backward != 0 applies the inverse
 * rotation to incoming gradients. */
int nsa_rope(const void* q, int64_t q_sb, int64_t q_sn, int64_t q_sh, const void* k, int64_t k_sb, int64_t k_sn,
             int64_t k_sh, void* qe, int64_t qe_sb, int64_t qe_sn, int64_t qe_sh, void* ke, int64_t ke_sb,
             int64_t ke_sn, int64_t ke_sh, const void* cos, const void* sin, int64_t c_sb, int64_t c_sn,
             int cos_is_fp32, int B, int N, int QH, int KH, int D, int backward, void* stream);

/* ---- KV-cache writer (the caller side of the paged entry points) ----
 * nano-vllm/nanovllm/layers/attention.py:123-153 store_kvcache: row n of key / value (k_row_elems = KH*D contiguous
 * elements, row stride k_st) is copied to flat pool row slot_mapping[n] of k_cache / v_cache (row stride kc_sr);
 * negative slots are skipped. */
int nsa_store_kvcache(const void* key, int64_t k_st, const void* value, int64_t v_st, void* k_cache, int64_t kc_sr,
                      void* v_cache, int64_t vc_sr, const int32_t* slot_mapping, int N, int k_row_elems,
                      int v_row_elems, void* stream);
/* One launch for a prefill chunk: store_kvcache of the chunk's new tokens (key / value [t,KH,D] packed by x_cu,
 * slot_mapping [t]) + mean pooling of the compressed rows listed in cmp_slot_mapping (as nsa_paged_pool_prefill,
 * flash_nsa/inference/compress_kv.py:191-220, for K and V).  Source rows of a pooled window are taken from the
 * chunk when they are new (position >= context_lens[b] - new tokens of b) and from the pool otherwise. */
int nsa_paged_store_pool_prefill(const void* key, int64_t k_st, int64_t k_sh, int Dk, const void* value, int64_t v_st,
                                 int64_t v_sh, int Dv, void* k_cache, int64_t kc_sr, int64_t kc_sh, void* v_cache,
                                 int64_t vc_sr, int64_t vc_sh, const int32_t* x_cu, const int32_t* context_lens,
                                 const int32_t* slot_mapping, const int32_t* y_cu, const int32_t* cmp_slot_mapping,
                                 const int32_t* block_tables, int table_stride, int B, int x_maxlen, int y_maxlen,
                                 int page_size, int H, int kernel_size, int stride, void* stream);

/* ---- fused decode step (one query token per request; q [B,QH,D], at most 16 q-heads per kv head) ----
 * Replaces flash_nsa/inference/compress_attn.py:540-667 (cmp_attn_decode) + inference/topk.py:495-623 (topk_decode):
 * compressed attention (cmp_o [B,QH,VD], optional lse addressed b*lse_st + head*lse_sh) and the top-n selection
 * topk[kh*tk_sh + b*tk_st + slot]; call after nsa_paged_pool_decode. */
int nsa_decode_cmp_topk(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr, int64_t k_sh,
                        const void* v_cache, int64_t v_sr, int64_t v_sh, void* cmp_o, int64_t co_st, int64_t co_sh,
                        float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk, int64_t tk_sh, int64_t tk_st,
                        const int32_t* context_lens, const int32_t* cmp_block_tables, int cmp_table_stride,
                        int page_size, int B, int QH, int KH, int D, int VD, int fixed_y_maxlen,
                        int fixed_num_slc_blocks, int kernel_size, int stride, int block_size, int top_n,
                        int num_init, int num_local, int ignore_index, float sm_scale, void* stream);
/* Split variant of the compressed branch for batches whose context lengths differ widely (two launches, grid
 * B x KH x nsplit): partial attention per key-interleaved split, then merge (cmp_o, lse) + head-summed probabilities
 * pg [B,KH,fixed_y_maxlen] fp32 of every compressed key.  Scratch (fp32): sp_m, sp_l [B,KH,nsplit,16],
 * sp_o [B,KH,nsplit,16,VD].  The selection itself then runs in the prologue of nsa_decode_slc_swa_combine. */
int nsa_decode_cmp_split(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr, int64_t k_sh,
                         const void* v_cache, int64_t v_sr, int64_t v_sh, void* cmp_o, int64_t co_st, int64_t co_sh,
                         float* lse, int64_t lse_st, int64_t lse_sh, float* pg, float* sp_m, float* sp_l, float* sp_o,
                         int nsplit, const int32_t* context_lens, const int32_t* cmp_block_tables,
                         int cmp_table_stride, int page_size, int B, int QH, int KH, int D, int VD,
                         int fixed_y_maxlen, int kernel_size, int stride, float sm_scale, void* stream);
/* The decode step of flash_nsa/inference/__init__.py:207-257 for small batches of long contexts, in two launches:
 * (1) the compressed branch cut into nsplit key-interleaved parts per (request, kv head) -- partial (m, l, o) and the
 * un-normalised fp16 probabilities of every compressed key go to scratch; (2) per (request, kv head): merge of the
 * parts, block scores, selection, selected-block + window attention, gated combine.  cmp_slot_mapping [B] (-1: no
 * compressed row completes at this step) makes launch (1) pool the newest compressed row, as nsa_paged_pool_decode
 * would; null: the row must be in the pool already.  Scratch, all caller-allocated, contents undefined:
 *   sp_m, sp_l [B,KH,nsplit,16] fp32; sp_o [B,KH,nsplit,16,VD] fp32;
 *   sp_keep_p [B,KH,Y/32,16,32] fp16 and sp_keep_m [B,KH,Y/32,16] fp32 with Y = fixed_y_maxlen rounded up to 32.
 * cmp_o / slc_o / swa_o / lse / topk are optional outputs (null: not written).
 * nsa_decode_split_fits: 1 when fixed_y_maxlen / fixed_num_slc_blocks / the raw table width fit the LDS of (2). */
int nsa_decode_split_fits(int D, int VD, int fixed_y_maxlen, int fixed_num_slc_blocks, int table_stride);
/* LDS bytes of launch (2), dynamic + statically declared, for these capacities; 0 when they do not fit 160 KB */
int nsa_decode_split_lds_total(int D, int VD, int fixed_y_maxlen, int fixed_num_slc_blocks, int table_stride);
int nsa_decode_split(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr, int64_t k_sh,
                     const void* v_cache, int64_t v_sr, int64_t v_sh, const void* w, int64_t w_st, int64_t w_sh,
                     void* out, int64_t o_st, int64_t o_sh, void* cmp_o, void* slc_o, void* swa_o, int64_t co_st,
                     int64_t co_sh, float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk, int64_t tk_sh,
                     int64_t tk_st, float* sp_m, float* sp_l, float* sp_o, void* sp_keep_p, float* sp_keep_m,
                     int nsplit, const int32_t* cmp_slot_mapping, const int32_t* context_lens,
                     const int32_t* block_tables, int table_stride, const int32_t* cmp_block_tables,
                     int cmp_table_stride, int page_size, int B, int QH, int KH, int D, int VD, int fixed_y_maxlen,
                     int fixed_num_slc_blocks, int kernel_size, int stride, int block_size, int top_n, int num_init,
                     int num_local, int ignore_index, int window, float sm_scale, void* stream);
/* nsa_decode_split with launch (2) cut as well: upstream's slc_num_splits (flash_nsa/inference/__init__.py:195-196,
 * inference/select_attn.py:329-331,492-498 -- the selected blocks of one token dealt over several programs, merged
 * through fp32 partials).  Here slc_nsplit workgroups per (request, kv head) share the window units and the selected
 * blocks (every one of them repeats the merge of the compressed parts and the selection), and a third launch merges
 * their partial results and applies the gates.  Worth it only when B x KH workgroups leave most of the GPU idle.
 * slc_nsplit in [1,16]; 1 = nsa_decode_split.  Extra scratch (caller-allocated, contents undefined):
 *   sp2_ml [B,KH,slc_nsplit,2,2,16] fp32, sp2_o [B,KH,slc_nsplit,2,16,VD] fp32, cmp_tmp [B,QH,VD] bf16 addressed with
 *   co_st / co_sh. */
int nsa_decode_split_parts(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr,
                           int64_t k_sh, const void* v_cache, int64_t v_sr, int64_t v_sh, const void* w, int64_t w_st,
                           int64_t w_sh, void* out, int64_t o_st, int64_t o_sh, void* cmp_o, void* slc_o, void* swa_o,
                           int64_t co_st, int64_t co_sh, float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk,
                           int64_t tk_sh, int64_t tk_st, float* sp_m, float* sp_l, float* sp_o, void* sp_keep_p,
                           float* sp_keep_m, int nsplit, const int32_t* cmp_slot_mapping,
                           const int32_t* context_lens, const int32_t* block_tables, int table_stride,
                           const int32_t* cmp_block_tables, int cmp_table_stride, int page_size, int B, int QH,
                           int KH, int D, int VD, int fixed_y_maxlen, int fixed_num_slc_blocks, int kernel_size,
                           int stride, int block_size, int top_n, int num_init, int num_local, int ignore_index,
                           int window, float sm_scale, int slc_nsplit, float* sp2_ml, float* sp2_o, void* cmp_tmp,
                           void* stream);
/* nsa_decode_split without any allocation.  No counterpart upstream: it is for callers that cannot allocate device
 * memory around the call (code under graph capture, tight serving loops, harnesses that forbid hipMalloc).  The
 * arguments are those of nsa_decode_split minus the five scratch buffers, which are carved out of one file-scope
 * device array of nsa_decode_split_static_capacity() bytes (32 MiB, held by every GPU the library runs on until the
 * process ends).  nsa_decode_split_static_bytes gives the bytes a call needs (e.g. 22.1 MB for 16 requests x 4 kv
 * heads x 8 parts at fixed_y_maxlen 8192); a call that needs more is refused with NSA_ERR_UNSUPPORTED.  All calls on
 * one GPU share the array: calls that overlap there (other streams or threads) race.  Neither this entry point nor
 * anything below it calls hipMalloc / hipFree. */
int64_t nsa_decode_split_static_capacity(void);
int64_t nsa_decode_split_static_bytes(int B, int KH, int VD, int nsplit, int fixed_y_maxlen);
int nsa_decode_split_static(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr,
                            int64_t k_sh, const void* v_cache, int64_t v_sr, int64_t v_sh, const void* w,
                            int64_t w_st, int64_t w_sh, void* out, int64_t o_st, int64_t o_sh, void* cmp_o,
                            void* slc_o, void* swa_o, int64_t co_st, int64_t co_sh, float* lse, int64_t lse_st,
                            int64_t lse_sh, int32_t* topk, int64_t tk_sh, int64_t tk_st, int nsplit,
                            const int32_t* cmp_slot_mapping, const int32_t* context_lens,
                            const int32_t* block_tables, int table_stride, const int32_t* cmp_block_tables,
                            int cmp_table_stride, int page_size, int B, int QH, int KH, int D, int VD,
                            int fixed_y_maxlen, int fixed_num_slc_blocks, int kernel_size, int stride,
                            int block_size, int top_n, int num_init, int num_local, int ignore_index, int window,
                            float sm_scale, void* stream);
/* Replaces flash_nsa/inference/select_attn.py:655-787 (fused_slc_swa_attn_decode) + inference/combine.py:104-127
 * (combine_decode): selected-block and window attention; slc_o / swa_o (optional, same strides as cmp_o) receive the
 * branch outputs; out (optional) = cmp_o*sig(w0) + slc_o*sig(w1) + swa_o*sig(w2).
 * pg == NULL: topk is an input.  pg != NULL (from nsa_decode_cmp_split): the block scores are folded from pg and
 * the selection (inference/topk.py:433-493) runs in the kernel's prologue; topk is then an output. */
int nsa_decode_slc_swa_combine(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr,
                               int64_t k_sh, const void* v_cache, int64_t v_sr, int64_t v_sh, const void* w,
                               int64_t w_st, int64_t w_sh, int32_t* topk, int64_t tk_sh, int64_t tk_st,
                               const float* pg, int fixed_y_maxlen, int fixed_num_slc_blocks, int kernel_size,
                               int stride, int num_init, int num_local, int ignore_index, const void* cmp_o,
                               void* slc_o, void* swa_o, int64_t co_st, int64_t co_sh, void* out, int64_t o_st,
                               int64_t o_sh, const int32_t* context_lens, const int32_t* block_tables,
                               int table_stride, int page_size, int B, int QH, int KH, int D, int VD, int block_size,
                               int top_n, int window, float sm_scale, void* stream);

/* The whole decode step in ONE launch (one workgroup per request and kv head):
 * replaces flash_nsa/inference/__init__.py:207-257 (cmp_attn_decode, topk_decode, fused_slc_swa_attn_decode,
 * combine_decode).  out [B,QH,VD] is required; cmp_o / slc_o / swa_o (shared strides co_st, co_sh), lse and topk
 * are optional outputs (NULL to skip).  cmp_slot_mapping [B] (optional): when given, the kernel also pools the
 * compressed K and V row that the newest token completes (flat pool row, -1: none), i.e. it includes
 * nsa_paged_pool_decode (flash_nsa/inference/compress_kv.py:253-287) and the step is a single launch.
 * new_k / new_v [B,KH,D] / [B,KH,VD] + slot_mapping [B] (optional, all three or none): the newest token's K and V
 * rows are first written to flat pool row slot_mapping[b] (-1: skip), i.e. the kernel also includes
 * store_kvcache (nano-vllm/nanovllm/layers/attention.py:123-153).
 * Needs fixed_y_maxlen / fixed_num_slc_blocks / table_stride small enough for
 * 160 KB of LDS (nsa_decode_fused_fits returns 1; e.g. contexts up to 32K tokens at kernel 32 / stride 16);
 * otherwise use nsa_decode_cmp_topk + nsa_decode_slc_swa_combine. */
int nsa_decode_fused_fits(int D, int VD, int fixed_y_maxlen, int fixed_num_slc_blocks, int table_stride,
                          int page_size);
int nsa_decode_fused(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr, int64_t k_sh,
                     const void* v_cache, int64_t v_sr, int64_t v_sh, const void* w, int64_t w_st, int64_t w_sh,
                     void* out, int64_t o_st, int64_t o_sh, void* cmp_o, void* slc_o, void* swa_o, int64_t co_st,
                     int64_t co_sh, float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk, int64_t tk_sh,
                     int64_t tk_st, const int32_t* context_lens, const int32_t* block_tables, int table_stride,
                     const int32_t* cmp_block_tables, int cmp_table_stride,
                     const int32_t* cmp_slot_mapping, const void* new_k, int64_t nk_st, int64_t nk_sh,
                     const void* new_v, int64_t nv_st, int64_t nv_sh, const int32_t* slot_mapping, int page_size, int B, int QH, int KH,
                     int D, int VD, int fixed_y_maxlen, int fixed_num_slc_blocks, int kernel_size, int stride,
                     int block_size, int top_n, int num_init, int num_local, int ignore_index, int window,
                     float sm_scale, void* stream);

#ifdef __cplusplus
}
#endif
#endif

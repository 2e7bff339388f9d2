// Parameter blocks handed (by value) to the attention kernels and the internal launch functions the C entry
// points in nsa_api.hip dispatch to.  Strides are in elements; pointers are device pointers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "nsa_common.h"

struct NsaFwdTileParams {
  const bf16_t* q; int64_t q_st, q_sh;      // [tokens, QH, D]
  const bf16_t* k; int64_t k_sr, k_sh;      // key rows [rows, KH, D]
  const bf16_t* v; int64_t v_sr, v_sh;      // value rows [rows, KH, VD]
  bf16_t* o; int64_t o_st, o_sh;            // [tokens, QH, VD]
  float* lse; int64_t lse_st, lse_sh;       // log2-domain log-sum-exp, addressed tok*lse_st + head*lse_sh
  const int32_t* x_cu;                      // [B+1] query-token offsets
  const int32_t* k_cu;                      // [B+1] compressed-row offsets (contiguous compressed mode)
  const int32_t* ctx_lens;                  // [B] total context length (paged)
  const int32_t* table; int table_stride; int page_size;  // paged: block table of the key rows
  int G, KH;
  float scale_log2;
  int kernel_size, stride, window;
};

struct NsaSlcParams {
  const bf16_t* q; int64_t q_st, q_sh;
  const bf16_t* k; int64_t k_sr, k_sh;
  const bf16_t* v; int64_t v_sr, v_sh;
  bf16_t* o; int64_t o_st, o_sh;
  float* lse; int64_t lse_st, lse_sh;
  const int32_t* topk; int64_t tk_sh, tk_st;  // [KH, tokens, top_n]
  const int32_t* x_cu;
  const int32_t* ctx_lens;
  const int32_t* table; int table_stride; int page_size;
  int G, KH, top_n, block_size;
  float scale_log2;
};

struct NsaTopkParams {
  const bf16_t* q; int64_t q_st, q_sh;
  const bf16_t* ck; int64_t ck_sr, ck_sh;
  const float* lse; int64_t lse_st, lse_sh;
  int32_t* topk; int64_t tk_sh, tk_st;
  float* imp_out; int64_t imp_sh, imp_st; int imp_cols;  // optional fp32 block scores [KH, tokens, imp_cols]
  const int32_t* x_cu;
  const int32_t* y_cu;
  const int32_t* ctx_lens;
  const int32_t* table; int table_stride; int page_size;
  int G, KH;
  float scale_log2;
  int kernel_size, stride, block_size, top_n, num_init, num_local, ignore_index;
  int nb_max;  // selection blocks of the longest context
  int seg_blocks;  // set by the launcher: 0 = an LDS score row holds all nb_max blocks; else blocks per segment
};

int nsa_fwd_tile_launch(const NsaFwdTileParams& p, int mode, bool paged, int B, int max_q_len, int D, int VD,
                        hipStream_t stream);
int nsa_slc_fwd_launch(const NsaSlcParams& p, bool paged, int B, int max_q_len, int D, int VD, hipStream_t stream);
int nsa_topk_launch(const NsaTopkParams& p, bool paged, int B, int max_q_len, int D, hipStream_t stream);
// two launches with the block scores in a workspace (nsa_topk_two_pass.hip)
bool nsa_topk_two_pass_supported(const NsaTopkParams& p, int D);
int64_t nsa_topk_two_pass_bytes_per_token(int KH, int nb_max);
int nsa_topk_two_pass_launch(const NsaTopkParams& p, bool paged, int B, int max_q_len, int total_tokens, int D,
                             void* workspace, int64_t workspace_bytes, hipStream_t stream);

// backward of the range-keyed branches and of the gathered (selected) branch
struct NsaBwdTileParams {
  const bf16_t* q; int64_t q_st, q_sh;
  const bf16_t* k; int64_t k_sr, k_sh;
  const bf16_t* v; int64_t v_sr, v_sh;
  const bf16_t* dO; int64_t do_st, do_sh;
  const float* lse; int64_t lse_st, lse_sh;
  const float* delta; int64_t delta_st, delta_sh;
  void* dq; int64_t dq_st, dq_sh; int dq_mode;      // 0: store bf16, 1: store fp32, 2: add into fp32,
                                                    // 3 (dq tile kernel): bf16 store of (result + fp32 dq_partial)
  const float* dq_partial; int64_t dqp_st, dqp_sh;
  void* dk; int64_t dk_sr, dk_sh;                   // dkdv kernels
  void* dv; int64_t dv_sr, dv_sh;
  int dkv_mode;                                     // 0: store bf16, 1: store fp32, 3: atomic add into fp32,
                                                    // 4: fp32 store into the workgroup's own slot of part_dk / part_dv
  float* part_dk; float* part_dv;                   // dkv_mode 4: [slots][keys per workgroup][D | VD]
  const int32_t* x_cu;
  const int32_t* k_cu;
  // gathered (selected-attention) row lists: CSR over (kv head, global selection block)
  const int32_t* csr_off;      // [KH][nblk_total + 1] absolute positions into csr_tok
  const int32_t* csr_tok;      // [KH * T * top_n] local token index inside its sequence, ascending per list
  const int32_t* item_off;     // [KH][nblk_total + 1] prefix of work items (list chunks)
  const int32_t* blk_seq;      // [nblk_total] sequence id of a global block
  const int32_t* kblk_cu;      // [B+1] selection-block offsets
  int nblk_total, chunk_tokens, block_size;
  int G, KH;
  float scale_log2, sm_scale;
  int kernel_size, stride, window;
  int q_chunk_tokens;          // compressed dkdv: query tokens per grid.x chunk
  int grid_chunks;             // compressed dkdv: chunks per key tile in grid.x (set by the launcher)
};

int nsa_bwd_dq_tile_launch(const NsaBwdTileParams& p, int mode, int B, int max_q_len, int D, int VD,
                           hipStream_t stream);
int nsa_bwd_dkdv_launch(const NsaBwdTileParams& p, int mode, int B, int max_q_len, int max_k_len, int D, int VD,
                        int n_items_bound, hipStream_t stream);
// deterministic dk / dv (dkv_mode 4): slots a launch writes, and the ordered sums over them (nsa_dkdv_reduce.hip)
int64_t nsa_bwd_dkdv_cmp_slots(int B, int KH, int max_q_len, int max_k_len, int q_chunk_tokens, int kernel_size,
                               int stride);
int64_t nsa_bwd_dkdv_slc_slots(int KH, int n_items_bound, int block_size);
int nsa_bwd_dkdv_slot_keys(int mode, int block_size);
int nsa_dkdv_reduce_cmp_launch(const NsaBwdTileParams& p, int B, int max_q_len, int max_k_len, int D, int VD,
                               hipStream_t stream);
int nsa_dkdv_reduce_slc_launch(const NsaBwdTileParams& p, int n_items_bound, int D, int VD, hipStream_t stream);

struct NsaSlcBwdDqParams {
  const bf16_t* q; int64_t q_st, q_sh;
  const bf16_t* k; int64_t k_sr, k_sh;
  const bf16_t* v; int64_t v_sr, v_sh;
  const bf16_t* dO; int64_t do_st, do_sh;
  const float* lse; int64_t lse_st, lse_sh;
  const float* delta; int64_t delta_st, delta_sh;
  void* dq; int64_t dq_st, dq_sh; int dq_mode;
  const int32_t* topk; int64_t tk_sh, tk_st;
  const int32_t* x_cu;
  int G, KH, top_n, block_size;
  float scale_log2, sm_scale;
};
int nsa_slc_bwd_dq_launch(const NsaSlcBwdDqParams& p, int B, int max_q_len, int D, int VD, hipStream_t stream);

// fused paged decode (one query token per request)
struct NsaDecodeParams {
  const bf16_t* q; int64_t q_st, q_sh;          // [B, QH, D]
  const bf16_t* k; int64_t k_sr, k_sh;          // pool, flat rows
  const bf16_t* v; int64_t v_sr, v_sh;
  const bf16_t* w; int64_t w_st, w_sh;          // gates [B, QH, 3]
  bf16_t* cmp_o; bf16_t* slc_o; bf16_t* swa_o; int64_t co_st, co_sh;  // branch outputs [B, QH, VD] (slc/swa optional)
  bf16_t* out; int64_t o_st, o_sh;              // final output (optional)
  float* lse_out; int64_t lse_st, lse_sh;       // compressed-branch lse (optional)
  int32_t* topk; int64_t tk_sh, tk_st;          // [KH, B, top_n]
  const int32_t* ctx_lens;
  const int32_t* table; int table_stride;       // raw block tables
  const int32_t* cmp_table; int cmp_table_stride;
  const int32_t* cmp_slots;                     // one-launch kernel: flat row of the compressed row completed now (-1: none), or null
  const bf16_t* new_k; int64_t nk_st, nk_sh;    // one-launch kernel: K / V of the newest token [B, KH, D] to be written
  const bf16_t* new_v; int64_t nv_st, nv_sh;    // to flat pool row raw_slots[b] first (null: the caller stored them)
  const int32_t* raw_slots;
  int page_size;
  int G, KH;
  float scale_log2;
  int kernel_size, stride, block_size, window, top_n, num_init, num_local, ignore_index;
  int y_cap, nb_cap;                            // fixed_y_maxlen, fixed_num_slc_blocks
  // split compressed branch: fp32 scratch [B,KH,nsplit,16] (m, l), [B,KH,nsplit,16,VD] (o), pg [B,KH,y_cap]
  float* sp_m; float* sp_l; float* sp_o; float* pg;
  // two-launch split path: the partial kernel also spills, per (request, kv head), the un-normalised fp16
  // probabilities [16][ceil32(y_cap)] and the maxima they refer to [ceil32(y_cap)/32][16]; the final kernel merges
  // the nsplit parts, folds the probabilities into block scores and selects
  _Float16* sp_keep_p; float* sp_keep_m; int nsplit;
  // two-launch split path with the window and selected branches cut as well (slc_nsplit > 1 parts per request and kv
  // head): every part writes its un-normalised (m, l, o) of both branches, part 0 the merged compressed-branch
  // output, and a third launch merges and combines.  sp2_ml [B,KH,slc_nsplit,2 branches,2 (m,l),16],
  // sp2_o [B,KH,slc_nsplit,2,16,VD] fp32, cmp_tmp [B,QH,VD] bf16
  int slc_nsplit; float* sp2_ml; float* sp2_o; bf16_t* cmp_tmp;
};
int nsa_decode_cmp_topk_launch(const NsaDecodeParams& p, int B, int D, int VD, hipStream_t stream);
int nsa_decode_slc_swa_launch(const NsaDecodeParams& p, int B, int D, int VD, hipStream_t stream);
int nsa_decode_fused_launch(const NsaDecodeParams& p, int B, int D, int VD, hipStream_t stream);
int nsa_decode_fused_lds_bytes(const NsaDecodeParams& p, int D, int VD);  // 0: does not fit
int nsa_decode_cmp_split_launch(const NsaDecodeParams& p, int B, int nsplit, int D, int VD, hipStream_t stream);
int nsa_decode_split_launch(const NsaDecodeParams& p, int B, int D, int VD, hipStream_t stream);
int nsa_decode_split_lds_bytes(const NsaDecodeParams& p, int D, int VD);  // final kernel, dynamic part; 0: does not fit
int nsa_decode_split_static_lds_bytes();                                   // final kernel, statically declared part

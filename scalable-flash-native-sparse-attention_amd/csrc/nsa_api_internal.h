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
  int nb_max;  // selection blocks of the longest context (length of an LDS score row)
};

int nsa_fwd_tile_launch(const NsaFwdTileParams& p, int mode, bool paged, int B, int max_q_len, int D, int VD,
                        hipStream_t stream);
int nsa_slc_fwd_launch(const NsaSlcParams& p, bool paged, int B, int max_q_len, int D, int VD, hipStream_t stream);
int nsa_topk_launch(const NsaTopkParams& p, bool paged, int B, int max_q_len, int D, hipStream_t stream);

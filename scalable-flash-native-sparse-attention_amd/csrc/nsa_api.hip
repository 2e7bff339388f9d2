// C entry points for the attention stages plus the library's error plumbing.  Argument checks live here so
// that a kernel is never launched on shapes its tiling does not cover.
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <math.h>
#include <string.h>
#include <atomic>
#include "nsa_common.h"
#include "nsa_api_internal.h"

static thread_local char g_err[512] = "";

void nsa_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

// Tuning values that a caller may override through nsa_set_tuning (never read from the environment).
namespace {
struct Knob {
  const char* name;
  std::atomic<int> value;
  std::atomic<bool> is_set;
};
Knob g_knobs[] = {
    {"fwd_variant", {0}, {false}},      // forward tile kernel: staging / rows per wave variant
    {"dq_min_blocks", {0}, {false}},    // workgroups per CU of the dense dq kernel
    {"dkdv_key_blocks", {0}, {false}},  // 32-key blocks per wave of the dense dk/dv kernel
    {"topk_seg_blocks", {0}, {false}},  // selection blocks per segment of the block selector
    {"topk_two_pass", {0}, {false}},    // 0: the one-launch selector even when a workspace is given
};
Knob* find_knob(const char* name) {
  for (Knob& k : g_knobs)
    if (strcmp(k.name, name) == 0) return &k;
  return nullptr;
}
}  // namespace

int nsa_tuning_knob(const char* name, int default_value) {
  Knob* k = find_knob(name);
  return (k && k->is_set.load()) ? k->value.load() : default_value;
}

int nsa_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    nsa_set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return NSA_ERR_LAUNCH;
  }
  return NSA_OK;
}

static int check_heads(const char* who, int QH, int KH, int D, int VD) {
  NSA_REQUIRE(QH > 0 && KH > 0 && QH % KH == 0, NSA_ERR_BAD_ARG, "%s: q heads %d must be a multiple of kv heads %d",
              who, QH, KH);
  NSA_REQUIRE(D % 32 == 0 && VD % 32 == 0, NSA_ERR_BAD_ARG, "%s: head dims %d/%d must be multiples of 32", who, D, VD);
  return NSA_OK;
}
static int check_nsa_sizes(const char* who, int kernel_size, int stride, int block_size) {
  NSA_REQUIRE(stride > 0 && (stride & (stride - 1)) == 0, NSA_ERR_BAD_ARG, "%s: stride %d must be a power of 2", who,
              stride);
  NSA_REQUIRE(kernel_size % stride == 0 && kernel_size >= stride, NSA_ERR_BAD_ARG,
              "%s: kernel_size %d must be a multiple of stride %d", who, kernel_size, stride);
  if (block_size > 0) {
    NSA_REQUIRE(block_size >= kernel_size && block_size % stride == 0, NSA_ERR_BAD_ARG,
                "%s: block_size %d must be >= kernel_size %d and a multiple of stride %d", who, block_size,
                kernel_size, stride);
  }
  return NSA_OK;
}

extern "C" {

const char* nsa_last_error(void) { return g_err; }
int nsa_abi_version(void) { return 1; }

int nsa_set_tuning(const char* name, int value) {
  Knob* k = name ? find_knob(name) : nullptr;
  NSA_REQUIRE(k != nullptr, NSA_ERR_BAD_ARG, "set_tuning: unknown name '%s' (fwd_variant, dq_min_blocks, "
              "dkdv_key_blocks, topk_seg_blocks, topk_two_pass)", name ? name : "(null)");
  k->value.store(value);
  k->is_set.store(true);
  return NSA_OK;
}
int nsa_reset_tuning(void) {
  for (Knob& k : g_knobs) k.is_set.store(false);
  return NSA_OK;
}

int nsa_cmp_attn_fwd(const void* q, int64_t q_st, int64_t q_sh, const void* ck, int64_t ck_sr, int64_t ck_sh,
                     const void* cv, int64_t cv_sr, int64_t cv_sh, void* o, int64_t o_st, int64_t o_sh, float* lse,
                     int64_t lse_st, int64_t lse_sh, const int32_t* x_cu, const int32_t* y_cu, int B, int x_maxlen,
                     int QH, int KH, int D, int VD, int kernel_size, int stride, float sm_scale, void* stream) {
  int rc = check_heads("cmp_attn_fwd", QH, KH, D, VD);
  if (rc) return rc;
  rc = check_nsa_sizes("cmp_attn_fwd", kernel_size, stride, 0);
  if (rc) return rc;
  NsaFwdTileParams p{};
  p.q = (const bf16_t*)q; p.q_st = q_st; p.q_sh = q_sh;
  p.k = (const bf16_t*)ck; p.k_sr = ck_sr; p.k_sh = ck_sh;
  p.v = (const bf16_t*)cv; p.v_sr = cv_sr; p.v_sh = cv_sh;
  p.o = (bf16_t*)o; p.o_st = o_st; p.o_sh = o_sh;
  p.lse = lse; p.lse_st = lse_st; p.lse_sh = lse_sh;
  p.x_cu = x_cu; p.k_cu = y_cu;
  p.G = QH / KH; p.KH = KH;
  p.scale_log2 = sm_scale * NSA_LOG2E;
  p.kernel_size = kernel_size; p.stride = stride; p.window = 0;
  return nsa_fwd_tile_launch(p, 0, false, B, x_maxlen, D, VD, (hipStream_t)stream);
}

int nsa_swa_fwd(const void* q, int64_t q_st, int64_t q_sh, const void* k, int64_t k_sr, int64_t k_sh,
                const void* v, int64_t v_sr, int64_t v_sh, void* o, int64_t o_st, int64_t o_sh, float* lse,
                int64_t lse_st, int64_t lse_sh, const int32_t* x_cu, int B, int x_maxlen, int QH, int KH, int D,
                int VD, int window, float sm_scale, void* stream) {
  int rc = check_heads("swa_fwd", QH, KH, D, VD);
  if (rc) return rc;
  NSA_REQUIRE(window >= 0, NSA_ERR_BAD_ARG, "swa_fwd: window %d must be >= 0", window);
  NsaFwdTileParams p{};
  p.q = (const bf16_t*)q; p.q_st = q_st; p.q_sh = q_sh;
  p.k = (const bf16_t*)k; p.k_sr = k_sr; p.k_sh = k_sh;
  p.v = (const bf16_t*)v; p.v_sr = v_sr; p.v_sh = v_sh;
  p.o = (bf16_t*)o; p.o_st = o_st; p.o_sh = o_sh;
  p.lse = lse; p.lse_st = lse_st; p.lse_sh = lse_sh;
  p.x_cu = x_cu; p.k_cu = x_cu;
  p.G = QH / KH; p.KH = KH;
  p.scale_log2 = sm_scale * NSA_LOG2E;
  p.kernel_size = 1; p.stride = 1; p.window = window;
  return nsa_fwd_tile_launch(p, 1, false, B, x_maxlen, D, VD, (hipStream_t)stream);
}

static int topk_select_impl(const void* q, int64_t q_st, int64_t q_sh, const void* ck, int64_t ck_sr, int64_t ck_sh,
                            const float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk, int64_t tk_sh,
                            int64_t tk_st, float* imp_out, int64_t imp_sh, int64_t imp_st, int imp_cols,
                            const int32_t* x_cu, const int32_t* y_cu, int B, int x_maxlen, int QH, int KH, int D,
                            int kernel_size, int stride, int block_size, int top_n, int num_init, int num_local,
                            int ignore_index, float sm_scale, int total_tokens, void* workspace,
                            int64_t workspace_bytes, void* stream) {
  int rc = check_heads("topk_select", QH, KH, D, 32);
  if (rc) return rc;
  rc = check_nsa_sizes("topk_select", kernel_size, stride, block_size);
  if (rc) return rc;
  NSA_REQUIRE(top_n >= 1 && top_n <= 64, NSA_ERR_BAD_ARG, "topk_select: top_n %d must be in [1,64]", top_n);
  NSA_REQUIRE(num_init >= 0 && num_local >= 0 && num_init + num_local <= top_n, NSA_ERR_BAD_ARG,
              "topk_select: num_init %d + num_local %d must be <= top_n %d", num_init, num_local, top_n);
  NsaTopkParams p{};
  p.q = (const bf16_t*)q; p.q_st = q_st; p.q_sh = q_sh;
  p.ck = (const bf16_t*)ck; p.ck_sr = ck_sr; p.ck_sh = ck_sh;
  p.lse = lse; p.lse_st = lse_st; p.lse_sh = lse_sh;
  p.topk = topk; p.tk_sh = tk_sh; p.tk_st = tk_st;
  p.imp_out = imp_out; p.imp_sh = imp_sh; p.imp_st = imp_st; p.imp_cols = imp_cols;
  p.x_cu = x_cu; p.y_cu = y_cu;
  p.G = QH / KH; p.KH = KH;
  p.scale_log2 = sm_scale * NSA_LOG2E;
  p.kernel_size = kernel_size; p.stride = stride; p.block_size = block_size;
  p.top_n = top_n; p.num_init = num_init; p.num_local = num_local; p.ignore_index = ignore_index;
  p.nb_max = (x_maxlen + block_size - 1) / block_size;
  if (p.nb_max < 1) p.nb_max = 1;
  if (workspace != nullptr && nsa_tuning_knob("topk_two_pass", 1) != 0 && nsa_topk_two_pass_supported(p, D))
    return nsa_topk_two_pass_launch(p, false, B, x_maxlen, total_tokens, D, workspace, workspace_bytes,
                                    (hipStream_t)stream);
  return nsa_topk_launch(p, false, B, x_maxlen, D, (hipStream_t)stream);
}

int nsa_topk_select(const void* q, int64_t q_st, int64_t q_sh, const void* ck, int64_t ck_sr, int64_t ck_sh,
                    const float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk, int64_t tk_sh, int64_t tk_st,
                    float* imp_out, int64_t imp_sh, int64_t imp_st, int imp_cols, const int32_t* x_cu,
                    const int32_t* y_cu, int B, int x_maxlen, int QH, int KH, int D, int kernel_size, int stride,
                    int block_size, int top_n, int num_init, int num_local, int ignore_index, float sm_scale,
                    void* stream) {
  return topk_select_impl(q, q_st, q_sh, ck, ck_sr, ck_sh, lse, lse_st, lse_sh, topk, tk_sh, tk_st, imp_out, imp_sh,
                          imp_st, imp_cols, x_cu, y_cu, B, x_maxlen, QH, KH, D, kernel_size, stride, block_size,
                          top_n, num_init, num_local, ignore_index, sm_scale, 0, nullptr, 0, stream);
}

int64_t nsa_topk_workspace_bytes(int total_tokens, int max_blocks, int KH) {
  if (total_tokens <= 0 || max_blocks <= 0 || KH <= 0) return 0;
  return (int64_t)total_tokens * nsa_topk_two_pass_bytes_per_token(KH, max_blocks) + 512;
}

int nsa_topk_select_ws(const void* q, int64_t q_st, int64_t q_sh, const void* ck, int64_t ck_sr, int64_t ck_sh,
                       const float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk, int64_t tk_sh, int64_t tk_st,
                       float* imp_out, int64_t imp_sh, int64_t imp_st, int imp_cols, const int32_t* x_cu,
                       const int32_t* y_cu, int B, int x_maxlen, int QH, int KH, int D, int kernel_size, int stride,
                       int block_size, int top_n, int num_init, int num_local, int ignore_index, float sm_scale,
                       int total_tokens, void* workspace, int64_t workspace_bytes, void* stream) {
  NSA_REQUIRE(total_tokens >= 0 && (workspace == nullptr || workspace_bytes > 0), NSA_ERR_BAD_ARG,
              "topk_select_ws: bad token count %d or workspace size %lld", total_tokens, (long long)workspace_bytes);
  return topk_select_impl(q, q_st, q_sh, ck, ck_sr, ck_sh, lse, lse_st, lse_sh, topk, tk_sh, tk_st, imp_out, imp_sh,
                          imp_st, imp_cols, x_cu, y_cu, B, x_maxlen, QH, KH, D, kernel_size, stride, block_size,
                          top_n, num_init, num_local, ignore_index, sm_scale, total_tokens, workspace,
                          workspace_bytes, stream);
}

int nsa_slc_attn_fwd(const void* q, int64_t q_st, int64_t q_sh, const void* k, int64_t k_sr, int64_t k_sh,
                     const void* v, int64_t v_sr, int64_t v_sh, const int32_t* topk, int64_t tk_sh, int64_t tk_st,
                     void* o, int64_t o_st, int64_t o_sh, float* lse, int64_t lse_st, int64_t lse_sh,
                     const int32_t* x_cu, int B, int x_maxlen, int QH, int KH, int D, int VD, int block_size,
                     int top_n, float sm_scale, void* stream) {
  int rc = check_heads("slc_attn_fwd", QH, KH, D, VD);
  if (rc) return rc;
  NSA_REQUIRE(block_size % 32 == 0 && block_size > 0, NSA_ERR_UNSUPPORTED,
              "slc_attn_fwd: block_size %d must be a multiple of 32", block_size);
  NSA_REQUIRE(top_n >= 1 && top_n <= 64, NSA_ERR_BAD_ARG, "slc_attn_fwd: top_n %d must be in [1,64]", top_n);
  NsaSlcParams p{};
  p.q = (const bf16_t*)q; p.q_st = q_st; p.q_sh = q_sh;
  p.k = (const bf16_t*)k; p.k_sr = k_sr; p.k_sh = k_sh;
  p.v = (const bf16_t*)v; p.v_sr = v_sr; p.v_sh = v_sh;
  p.o = (bf16_t*)o; p.o_st = o_st; p.o_sh = o_sh;
  p.lse = lse; p.lse_st = lse_st; p.lse_sh = lse_sh;
  p.topk = topk; p.tk_sh = tk_sh; p.tk_st = tk_st;
  p.x_cu = x_cu;
  p.G = QH / KH; p.KH = KH; p.top_n = top_n; p.block_size = block_size;
  p.scale_log2 = sm_scale * NSA_LOG2E;
  return nsa_slc_fwd_launch(p, false, B, x_maxlen, D, VD, (hipStream_t)stream);
}

}  // extern "C"

// ------------------------------------------------------------------------------------------------ backward
namespace {
struct BwdCommon {
  const void* q; int64_t q_st, q_sh;
  const void* k; int64_t k_sr, k_sh;
  const void* v; int64_t v_sr, v_sh;
  const void* dO; int64_t do_st, do_sh;
  const float* lse; int64_t lse_st, lse_sh;
  const float* delta; int64_t delta_st, delta_sh;
};
NsaBwdTileParams make_bwd(const BwdCommon& c, int QH, int KH, float sm_scale) {
  NsaBwdTileParams p{};
  p.q = (const bf16_t*)c.q; p.q_st = c.q_st; p.q_sh = c.q_sh;
  p.k = (const bf16_t*)c.k; p.k_sr = c.k_sr; p.k_sh = c.k_sh;
  p.v = (const bf16_t*)c.v; p.v_sr = c.v_sr; p.v_sh = c.v_sh;
  p.dO = (const bf16_t*)c.dO; p.do_st = c.do_st; p.do_sh = c.do_sh;
  p.lse = c.lse; p.lse_st = c.lse_st; p.lse_sh = c.lse_sh;
  p.delta = c.delta; p.delta_st = c.delta_st; p.delta_sh = c.delta_sh;
  p.G = QH / KH; p.KH = KH;
  p.scale_log2 = sm_scale * NSA_LOG2E; p.sm_scale = sm_scale;
  p.kernel_size = 1; p.stride = 1; p.window = 0;
  return p;
}
}  // namespace

extern "C" {

static int cmp_bwd_dq_impl(const char* who, const BwdCommon& c, void* dq, int64_t dq_st, int64_t dq_sh, int dq_mode,
                           const float* dq_partial, int64_t dqp_st, int64_t dqp_sh, const int32_t* x_cu,
                           const int32_t* y_cu, int B, int x_maxlen, int QH, int KH, int D, int VD, int kernel_size,
                           int stride, float sm_scale, void* stream) {
  int rc = check_heads(who, QH, KH, D, VD);
  if (rc) return rc;
  rc = check_nsa_sizes(who, kernel_size, stride, 0);
  if (rc) return rc;
  NsaBwdTileParams p = make_bwd(c, QH, KH, sm_scale);
  p.dq = dq; p.dq_st = dq_st; p.dq_sh = dq_sh; p.dq_mode = dq_mode;
  p.dq_partial = dq_partial; p.dqp_st = dqp_st; p.dqp_sh = dqp_sh;
  p.x_cu = x_cu; p.k_cu = y_cu;
  p.kernel_size = kernel_size; p.stride = stride;
  return nsa_bwd_dq_tile_launch(p, 0, B, x_maxlen, D, VD, (hipStream_t)stream);
}

int nsa_cmp_attn_bwd_dq(const void* q, int64_t q_st, int64_t q_sh, const void* ck, int64_t ck_sr, int64_t ck_sh,
                        const void* cv, int64_t cv_sr, int64_t cv_sh, const void* dO, int64_t do_st, int64_t do_sh,
                        const float* lse, int64_t lse_st, int64_t lse_sh, const float* delta, int64_t delta_st,
                        int64_t delta_sh, void* dq, int64_t dq_st, int64_t dq_sh, int dq_mode, const int32_t* x_cu,
                        const int32_t* y_cu, int B, int x_maxlen, int QH, int KH, int D, int VD, int kernel_size,
                        int stride, float sm_scale, void* stream) {
  NSA_REQUIRE(dq_mode >= 0 && dq_mode <= 2, NSA_ERR_BAD_ARG, "cmp_attn_bwd_dq: dq_mode %d not in {0,1,2}", dq_mode);
  BwdCommon c{q, q_st, q_sh, ck, ck_sr, ck_sh, cv, cv_sr, cv_sh, dO, do_st, do_sh, lse, lse_st, lse_sh, delta,
              delta_st, delta_sh};
  return cmp_bwd_dq_impl("cmp_attn_bwd_dq", c, dq, dq_st, dq_sh, dq_mode, nullptr, 0, 0, x_cu, y_cu, B, x_maxlen, QH,
                         KH, D, VD, kernel_size, stride, sm_scale, stream);
}

int nsa_cmp_attn_bwd_dq_final(const void* q, int64_t q_st, int64_t q_sh, const void* ck, int64_t ck_sr,
                              int64_t ck_sh, const void* cv, int64_t cv_sr, int64_t cv_sh, const void* dO,
                              int64_t do_st, int64_t do_sh, const float* lse, int64_t lse_st, int64_t lse_sh,
                              const float* delta, int64_t delta_st, int64_t delta_sh, const float* dq_partial,
                              int64_t dqp_st, int64_t dqp_sh, void* dq, int64_t dq_st, int64_t dq_sh,
                              const int32_t* x_cu, const int32_t* y_cu, int B, int x_maxlen, int QH, int KH, int D,
                              int VD, int kernel_size, int stride, float sm_scale, void* stream) {
  NSA_REQUIRE(dq_partial != nullptr && dq != nullptr, NSA_ERR_BAD_ARG, "cmp_attn_bwd_dq_final: null dq buffers");
  BwdCommon c{q, q_st, q_sh, ck, ck_sr, ck_sh, cv, cv_sr, cv_sh, dO, do_st, do_sh, lse, lse_st, lse_sh, delta,
              delta_st, delta_sh};
  return cmp_bwd_dq_impl("cmp_attn_bwd_dq_final", c, dq, dq_st, dq_sh, 3, dq_partial, dqp_st, dqp_sh, x_cu, y_cu, B,
                         x_maxlen, QH, KH, D, VD, kernel_size, stride, sm_scale, stream);
}

// Query tokens per work item of the compressed dk/dv kernel when the caller leaves the choice to the library.
static int cmp_dkdv_q_chunk(int q_chunk_tokens, int B, int x_maxlen, int y_maxlen, int QH, int KH, int D, int VD,
                            int kernel_size, int stride) {
  if (q_chunk_tokens <= 0) {
    // The kernel keeps one workgroup per CU, so a launch takes about
    //   ceil(workgroups / CUs) * (fixed cost of a workgroup + its 64-row tiles * time per tile);
    // a workgroup is one (128-key tile, query chunk that sees it, kv head, sequence).  The chunk (a power of two in
    // [128, 2048]) that minimises this for the longest sequence is taken.  The constants (90 us, 2.4 us per tile
    // at d = dv = 128) were fitted on MI355X to sweeps over one to eight sequences of 4K to 64K tokens, where the
    // choice is within 1 % of the best chunk.
    static int num_cus = 0;
    if (num_cus == 0) {
      int dev = 0;
      hipDeviceProp_t prop;
      num_cus = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
                 prop.multiProcessorCount > 0) ? prop.multiProcessorCount : 256;
    }
    const double tile_us = 2.4 * (D + VD) / 256.0, fixed_us = 90.0;
    const int G = QH / KH;
    double best = 0.0;
    for (int chunk = 128; chunk <= 2048; chunk *= 2) {
      const int64_t nch = (x_maxlen + chunk - 1) / chunk;
      int64_t wgs = 0;
      for (int64_t kt = 0; kt * 128 < y_maxlen; kt++) {
        const int64_t fc = ((int64_t)stride * kt * 128 + kernel_size - 1) / chunk;
        wgs += nch - (fc < nch ? fc : nch);
      }
      wgs *= (int64_t)B * KH;
      const double rounds = (double)((wgs + num_cus - 1) / num_cus);
      const double cost = rounds * (fixed_us + (double)chunk * G / 64.0 * tile_us);
      if (q_chunk_tokens <= 0 || cost < best) { best = cost; q_chunk_tokens = chunk; }
    }
  }
  return q_chunk_tokens;
}

static int cmp_attn_bwd_dkdv_impl(const void* q, int64_t q_st, int64_t q_sh, const void* ck, int64_t ck_sr,
                                  int64_t ck_sh, const void* cv, int64_t cv_sr, int64_t cv_sh, const void* dO,
                                  int64_t do_st, int64_t do_sh, const float* lse, int64_t lse_st, int64_t lse_sh,
                                  const float* delta, int64_t delta_st, int64_t delta_sh, float* dck, int64_t dck_sr,
                                  int64_t dck_sh, float* dcv, int64_t dcv_sr, int64_t dcv_sh, const int32_t* x_cu,
                                  const int32_t* y_cu, int B, int x_maxlen, int y_maxlen, int QH, int KH, int D,
                                  int VD, int kernel_size, int stride, int q_chunk_tokens, float sm_scale,
                                  bool deterministic, void* workspace, int64_t workspace_bytes, void* stream) {
  int rc = check_heads("cmp_attn_bwd_dkdv", QH, KH, D, VD);
  if (rc) return rc;
  rc = check_nsa_sizes("cmp_attn_bwd_dkdv", kernel_size, stride, 0);
  if (rc) return rc;
  q_chunk_tokens = cmp_dkdv_q_chunk(q_chunk_tokens, B, x_maxlen, y_maxlen, QH, KH, D, VD, kernel_size, stride);
  BwdCommon c{q, q_st, q_sh, ck, ck_sr, ck_sh, cv, cv_sr, cv_sh, dO, do_st, do_sh, lse, lse_st, lse_sh, delta,
              delta_st, delta_sh};
  NsaBwdTileParams p = make_bwd(c, QH, KH, sm_scale);
  p.dk = dck; p.dk_sr = dck_sr; p.dk_sh = dck_sh;
  p.dv = dcv; p.dv_sr = dcv_sr; p.dv_sh = dcv_sh;
  p.dkv_mode = 3;
  p.x_cu = x_cu; p.k_cu = y_cu;
  p.kernel_size = kernel_size; p.stride = stride;
  p.q_chunk_tokens = q_chunk_tokens;
  if (!deterministic) return nsa_bwd_dkdv_launch(p, 0, B, x_maxlen, y_maxlen, D, VD, 0, (hipStream_t)stream);
  if (B <= 0 || y_maxlen <= 0) return NSA_OK;
  // every work item stores into its own slot, then one pass sums the slots of a key in ascending chunk order
  const int64_t slots = nsa_bwd_dkdv_cmp_slots(B, KH, x_maxlen, y_maxlen, q_chunk_tokens, kernel_size, stride);
  const int64_t kw = nsa_bwd_dkdv_slot_keys(0, 0);
  const int64_t dk_bytes = (slots * kw * D * 4 + 255) & ~(int64_t)255;
  const int64_t need = dk_bytes + slots * kw * VD * 4;
  NSA_REQUIRE(workspace != nullptr && workspace_bytes >= need, NSA_ERR_WORKSPACE,
              "cmp_attn_bwd_dkdv_det: workspace of %lld bytes, %lld needed", (long long)workspace_bytes,
              (long long)need);
  p.dkv_mode = 4;
  p.part_dk = (float*)workspace;
  p.part_dv = (float*)((char*)workspace + dk_bytes);
  rc = nsa_bwd_dkdv_launch(p, 0, B, x_maxlen, y_maxlen, D, VD, 0, (hipStream_t)stream);
  if (rc) return rc;
  return nsa_dkdv_reduce_cmp_launch(p, B, x_maxlen, y_maxlen, D, VD, (hipStream_t)stream);
}

int nsa_cmp_attn_bwd_dkdv(const void* q, int64_t q_st, int64_t q_sh, const void* ck, int64_t ck_sr, int64_t ck_sh,
                          const void* cv, int64_t cv_sr, int64_t cv_sh, const void* dO, int64_t do_st,
                          int64_t do_sh, const float* lse, int64_t lse_st, int64_t lse_sh, const float* delta,
                          int64_t delta_st, int64_t delta_sh, float* dck, int64_t dck_sr, int64_t dck_sh,
                          float* dcv, int64_t dcv_sr, int64_t dcv_sh, const int32_t* x_cu, const int32_t* y_cu,
                          int B, int x_maxlen, int y_maxlen, int QH, int KH, int D, int VD, int kernel_size,
                          int stride, int q_chunk_tokens, float sm_scale, void* stream) {
  return cmp_attn_bwd_dkdv_impl(q, q_st, q_sh, ck, ck_sr, ck_sh, cv, cv_sr, cv_sh, dO, do_st, do_sh, lse, lse_st,
                                lse_sh, delta, delta_st, delta_sh, dck, dck_sr, dck_sh, dcv, dcv_sr, dcv_sh, x_cu,
                                y_cu, B, x_maxlen, y_maxlen, QH, KH, D, VD, kernel_size, stride, q_chunk_tokens,
                                sm_scale, false, nullptr, 0, stream);
}

int64_t nsa_cmp_attn_bwd_dkdv_det_bytes(int B, int x_maxlen, int y_maxlen, int QH, int KH, int D, int VD,
                                        int kernel_size, int stride, int q_chunk_tokens) {
  if (B <= 0 || x_maxlen <= 0 || y_maxlen <= 0 || KH <= 0 || QH <= 0 || stride <= 0) return 0;
  q_chunk_tokens = cmp_dkdv_q_chunk(q_chunk_tokens, B, x_maxlen, y_maxlen, QH, KH, D, VD, kernel_size, stride);
  const int64_t slots = nsa_bwd_dkdv_cmp_slots(B, KH, x_maxlen, y_maxlen, q_chunk_tokens, kernel_size, stride);
  const int64_t kw = nsa_bwd_dkdv_slot_keys(0, 0);
  return ((slots * kw * D * 4 + 255) & ~(int64_t)255) + slots * kw * VD * 4;
}

int nsa_cmp_attn_bwd_dkdv_det(const void* q, int64_t q_st, int64_t q_sh, const void* ck, int64_t ck_sr,
                              int64_t ck_sh, const void* cv, int64_t cv_sr, int64_t cv_sh, const void* dO,
                              int64_t do_st, int64_t do_sh, const float* lse, int64_t lse_st, int64_t lse_sh,
                              const float* delta, int64_t delta_st, int64_t delta_sh, float* dck, int64_t dck_sr,
                              int64_t dck_sh, float* dcv, int64_t dcv_sr, int64_t dcv_sh, const int32_t* x_cu,
                              const int32_t* y_cu, int B, int x_maxlen, int y_maxlen, int QH, int KH, int D, int VD,
                              int kernel_size, int stride, int q_chunk_tokens, float sm_scale, void* workspace,
                              int64_t workspace_bytes, void* stream) {
  return cmp_attn_bwd_dkdv_impl(q, q_st, q_sh, ck, ck_sr, ck_sh, cv, cv_sr, cv_sh, dO, do_st, do_sh, lse, lse_st,
                                lse_sh, delta, delta_st, delta_sh, dck, dck_sr, dck_sh, dcv, dcv_sr, dcv_sh, x_cu,
                                y_cu, B, x_maxlen, y_maxlen, QH, KH, D, VD, kernel_size, stride, q_chunk_tokens,
                                sm_scale, true, workspace, workspace_bytes, stream);
}



int nsa_slc_bwd_chunk_tokens(int T, int KH, int top_n) {
  // list chunk (tokens per work item of the selected-attention dk/dv pass): 1024 for long batches, smaller when
  // that would leave fewer than about 2048 two-wave work items; below 256 the fp32 atomic additions of the many
  // items cost more than the idle CUs
  const int64_t want = (int64_t)KH * T * top_n / 2048;
  int c = 256;
  while (c < 1024 && c * 2 <= want) c *= 2;
  return c;
}

int nsa_swa_bwd_dq(const void* q, int64_t q_st, int64_t q_sh, const void* k, int64_t k_sr, int64_t k_sh,
                   const void* v, int64_t v_sr, int64_t v_sh, const void* dO, int64_t do_st, int64_t do_sh,
                   const float* lse, int64_t lse_st, int64_t lse_sh, const float* delta, int64_t delta_st,
                   int64_t delta_sh, void* dq, int64_t dq_st, int64_t dq_sh, int dq_mode, const int32_t* x_cu,
                   int B, int x_maxlen, int QH, int KH, int D, int VD, int window, float sm_scale, void* stream) {
  int rc = check_heads("swa_bwd_dq", QH, KH, D, VD);
  if (rc) return rc;
  NSA_REQUIRE(dq_mode >= 0 && dq_mode <= 2, NSA_ERR_BAD_ARG, "swa_bwd_dq: dq_mode %d not in {0,1,2}", dq_mode);
  BwdCommon c{q, q_st, q_sh, k, k_sr, k_sh, v, v_sr, v_sh, dO, do_st, do_sh, lse, lse_st, lse_sh, delta, delta_st,
              delta_sh};
  NsaBwdTileParams p = make_bwd(c, QH, KH, sm_scale);
  p.dq = dq; p.dq_st = dq_st; p.dq_sh = dq_sh; p.dq_mode = dq_mode;
  p.x_cu = x_cu; p.k_cu = x_cu;
  p.window = window;
  return nsa_bwd_dq_tile_launch(p, 1, B, x_maxlen, D, VD, (hipStream_t)stream);
}

int nsa_swa_bwd_dkdv(const void* q, int64_t q_st, int64_t q_sh, const void* k, int64_t k_sr, int64_t k_sh,
                     const void* v, int64_t v_sr, int64_t v_sh, const void* dO, int64_t do_st, int64_t do_sh,
                     const float* lse, int64_t lse_st, int64_t lse_sh, const float* delta, int64_t delta_st,
                     int64_t delta_sh, void* dk, int64_t dk_sr, int64_t dk_sh, void* dv, int64_t dv_sr,
                     int64_t dv_sh, int dkv_is_f32, const int32_t* x_cu, int B, int x_maxlen, int QH, int KH, int D,
                     int VD, int window, float sm_scale, void* stream) {
  int rc = check_heads("swa_bwd_dkdv", QH, KH, D, VD);
  if (rc) return rc;
  BwdCommon c{q, q_st, q_sh, k, k_sr, k_sh, v, v_sr, v_sh, dO, do_st, do_sh, lse, lse_st, lse_sh, delta, delta_st,
              delta_sh};
  NsaBwdTileParams p = make_bwd(c, QH, KH, sm_scale);
  p.dk = dk; p.dk_sr = dk_sr; p.dk_sh = dk_sh;
  p.dv = dv; p.dv_sr = dv_sr; p.dv_sh = dv_sh;
  p.dkv_mode = dkv_is_f32 ? 1 : 0;
  p.x_cu = x_cu; p.k_cu = x_cu;
  p.window = window;
  return nsa_bwd_dkdv_launch(p, 1, B, x_maxlen, x_maxlen, D, VD, 0, (hipStream_t)stream);
}

int nsa_slc_attn_bwd_dq(const void* q, int64_t q_st, int64_t q_sh, const void* k, int64_t k_sr, int64_t k_sh,
                        const void* v, int64_t v_sr, int64_t v_sh, const void* dO, int64_t do_st, int64_t do_sh,
                        const float* lse, int64_t lse_st, int64_t lse_sh, const float* delta, int64_t delta_st,
                        int64_t delta_sh, const int32_t* topk, int64_t tk_sh, int64_t tk_st, void* dq,
                        int64_t dq_st, int64_t dq_sh, int dq_mode, const int32_t* x_cu, int B, int x_maxlen, int QH,
                        int KH, int D, int VD, int block_size, int top_n, float sm_scale, void* stream) {
  int rc = check_heads("slc_attn_bwd_dq", QH, KH, D, VD);
  if (rc) return rc;
  NSA_REQUIRE(block_size % 32 == 0 && block_size > 0, NSA_ERR_UNSUPPORTED,
              "slc_attn_bwd_dq: block_size %d must be a multiple of 32", block_size);
  NSA_REQUIRE(top_n >= 1 && top_n <= 64, NSA_ERR_BAD_ARG, "slc_attn_bwd_dq: top_n %d must be in [1,64]", top_n);
  NSA_REQUIRE(dq_mode >= 0 && dq_mode <= 2, NSA_ERR_BAD_ARG, "slc_attn_bwd_dq: dq_mode %d not in {0,1,2}", dq_mode);
  NsaSlcBwdDqParams p{};
  p.q = (const bf16_t*)q; p.q_st = q_st; p.q_sh = q_sh;
  p.k = (const bf16_t*)k; p.k_sr = k_sr; p.k_sh = k_sh;
  p.v = (const bf16_t*)v; p.v_sr = v_sr; p.v_sh = v_sh;
  p.dO = (const bf16_t*)dO; p.do_st = do_st; p.do_sh = do_sh;
  p.lse = lse; p.lse_st = lse_st; p.lse_sh = lse_sh;
  p.delta = delta; p.delta_st = delta_st; p.delta_sh = delta_sh;
  p.dq = dq; p.dq_st = dq_st; p.dq_sh = dq_sh; p.dq_mode = dq_mode;
  p.topk = topk; p.tk_sh = tk_sh; p.tk_st = tk_st;
  p.x_cu = x_cu;
  p.G = QH / KH; p.KH = KH; p.top_n = top_n; p.block_size = block_size;
  p.scale_log2 = sm_scale * NSA_LOG2E; p.sm_scale = sm_scale;
  return nsa_slc_bwd_dq_launch(p, B, x_maxlen, D, VD, (hipStream_t)stream);
}

static int slc_attn_bwd_dkdv_impl(const void* q, int64_t q_st, int64_t q_sh, const void* k, int64_t k_sr, int64_t k_sh,
                          const void* v, int64_t v_sr, int64_t v_sh, const void* dO, int64_t do_st,
                          int64_t do_sh, const float* lse, int64_t lse_st, int64_t lse_sh, const float* delta,
                          int64_t delta_st, int64_t delta_sh, float* dk, int64_t dk_sr, int64_t dk_sh, float* dv,
                          int64_t dv_sr, int64_t dv_sh, const int32_t* x_cu, const int32_t* kblk_cu,
                          const int32_t* blk_seq, const int32_t* csr_off, const int32_t* csr_tok,
                          const int32_t* item_off, int nblk_total, int chunk_tokens, int n_items_bound, int B,
                          int QH, int KH, int D, int VD, int block_size, float sm_scale, bool deterministic,
                          void* workspace, int64_t workspace_bytes, void* stream) {
  int rc = check_heads("slc_attn_bwd_dkdv", QH, KH, D, VD);
  if (rc) return rc;
  NSA_REQUIRE(block_size % 32 == 0 && block_size > 0, NSA_ERR_UNSUPPORTED,
              "slc_attn_bwd_dkdv: block_size %d must be a multiple of 32", block_size);
  BwdCommon c{q, q_st, q_sh, k, k_sr, k_sh, v, v_sr, v_sh, dO, do_st, do_sh, lse, lse_st, lse_sh, delta, delta_st,
              delta_sh};
  NsaBwdTileParams p = make_bwd(c, QH, KH, sm_scale);
  p.dk = dk; p.dk_sr = dk_sr; p.dk_sh = dk_sh;
  p.dv = dv; p.dv_sr = dv_sr; p.dv_sh = dv_sh;
  p.dkv_mode = 3;
  p.x_cu = x_cu; p.k_cu = x_cu;
  p.csr_off = csr_off; p.csr_tok = csr_tok; p.item_off = item_off; p.blk_seq = blk_seq; p.kblk_cu = kblk_cu;
  p.nblk_total = nblk_total; p.chunk_tokens = chunk_tokens; p.block_size = block_size;
  if (!deterministic) return nsa_bwd_dkdv_launch(p, 2, B, 0, 0, D, VD, n_items_bound, (hipStream_t)stream);
  if (n_items_bound <= 0) return NSA_OK;
  const int64_t slots = nsa_bwd_dkdv_slc_slots(KH, n_items_bound, block_size);
  const int64_t kw = nsa_bwd_dkdv_slot_keys(2, block_size);
  const int64_t dk_bytes = (slots * kw * D * 4 + 255) & ~(int64_t)255;
  const int64_t need = dk_bytes + slots * kw * VD * 4;
  NSA_REQUIRE(workspace != nullptr && workspace_bytes >= need, NSA_ERR_WORKSPACE,
              "slc_attn_bwd_dkdv_det: workspace of %lld bytes, %lld needed", (long long)workspace_bytes,
              (long long)need);
  p.dkv_mode = 4;
  p.part_dk = (float*)workspace;
  p.part_dv = (float*)((char*)workspace + dk_bytes);
  rc = nsa_bwd_dkdv_launch(p, 2, B, 0, 0, D, VD, n_items_bound, (hipStream_t)stream);
  if (rc) return rc;
  return nsa_dkdv_reduce_slc_launch(p, n_items_bound, D, VD, (hipStream_t)stream);
}

int nsa_slc_attn_bwd_dkdv(const void* q, int64_t q_st, int64_t q_sh, const void* k, int64_t k_sr, int64_t k_sh,
                          const void* v, int64_t v_sr, int64_t v_sh, const void* dO, int64_t do_st,
                          int64_t do_sh, const float* lse, int64_t lse_st, int64_t lse_sh, const float* delta,
                          int64_t delta_st, int64_t delta_sh, float* dk, int64_t dk_sr, int64_t dk_sh, float* dv,
                          int64_t dv_sr, int64_t dv_sh, const int32_t* x_cu, const int32_t* kblk_cu,
                          const int32_t* blk_seq, const int32_t* csr_off, const int32_t* csr_tok,
                          const int32_t* item_off, int nblk_total, int chunk_tokens, int n_items_bound, int B,
                          int QH, int KH, int D, int VD, int block_size, float sm_scale, void* stream) {
  return slc_attn_bwd_dkdv_impl(q, q_st, q_sh, k, k_sr, k_sh, v, v_sr, v_sh, dO, do_st, do_sh, lse, lse_st, lse_sh,
                                delta, delta_st, delta_sh, dk, dk_sr, dk_sh, dv, dv_sr, dv_sh, x_cu, kblk_cu, blk_seq,
                                csr_off, csr_tok, item_off, nblk_total, chunk_tokens, n_items_bound, B, QH, KH, D, VD,
                                block_size, sm_scale, false, nullptr, 0, stream);
}

int64_t nsa_slc_attn_bwd_dkdv_det_bytes(int n_items_bound, int KH, int D, int VD, int block_size) {
  if (n_items_bound <= 0 || KH <= 0 || block_size <= 0) return 0;
  const int64_t slots = nsa_bwd_dkdv_slc_slots(KH, n_items_bound, block_size);
  const int64_t kw = nsa_bwd_dkdv_slot_keys(2, block_size);
  return ((slots * kw * D * 4 + 255) & ~(int64_t)255) + slots * kw * VD * 4;
}

int nsa_slc_attn_bwd_dkdv_det(const void* q, int64_t q_st, int64_t q_sh, const void* k, int64_t k_sr, int64_t k_sh,
                              const void* v, int64_t v_sr, int64_t v_sh, const void* dO, int64_t do_st,
                              int64_t do_sh, const float* lse, int64_t lse_st, int64_t lse_sh, const float* delta,
                              int64_t delta_st, int64_t delta_sh, float* dk, int64_t dk_sr, int64_t dk_sh,
                              float* dv, int64_t dv_sr, int64_t dv_sh, const int32_t* x_cu, const int32_t* kblk_cu,
                              const int32_t* blk_seq, const int32_t* csr_off, const int32_t* csr_tok,
                              const int32_t* item_off, int nblk_total, int chunk_tokens, int n_items_bound, int B,
                              int QH, int KH, int D, int VD, int block_size, float sm_scale, void* workspace,
                              int64_t workspace_bytes, void* stream) {
  return slc_attn_bwd_dkdv_impl(q, q_st, q_sh, k, k_sr, k_sh, v, v_sr, v_sh, dO, do_st, do_sh, lse, lse_st, lse_sh,
                                delta, delta_st, delta_sh, dk, dk_sr, dk_sh, dv, dv_sr, dv_sh, x_cu, kblk_cu, blk_seq,
                                csr_off, csr_tok, item_off, nblk_total, chunk_tokens, n_items_bound, B, QH, KH, D, VD,
                                block_size, sm_scale, true, workspace, workspace_bytes, stream);
}



}  // extern "C"

// ------------------------------------------------------------------------------------------------ paged KV
namespace {
int check_page(const char* who, int page_size) {
  NSA_REQUIRE(page_size > 0 && page_size % 64 == 0, NSA_ERR_BAD_ARG, "%s: page_size %d must be a multiple of 64", who,
              page_size);
  return NSA_OK;
}
}  // namespace

extern "C" {

int nsa_paged_cmp_attn_fwd(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr,
                           int64_t k_sh, const void* v_cache, int64_t v_sr, int64_t v_sh, void* o, int64_t o_st,
                           int64_t o_sh, float* lse, int64_t lse_st, int64_t lse_sh, const int32_t* x_cu,
                           const int32_t* context_lens, const int32_t* cmp_block_tables, int table_stride,
                           int page_size, int B, int x_maxlen, int QH, int KH, int D, int VD, int kernel_size,
                           int stride, float sm_scale, void* stream) {
  int rc = check_heads("paged_cmp_attn_fwd", QH, KH, D, VD);
  if (rc) return rc;
  rc = check_nsa_sizes("paged_cmp_attn_fwd", kernel_size, stride, 0);
  if (rc) return rc;
  rc = check_page("paged_cmp_attn_fwd", page_size);
  if (rc) return rc;
  NsaFwdTileParams p{};
  p.q = (const bf16_t*)q; p.q_st = q_st; p.q_sh = q_sh;
  p.k = (const bf16_t*)k_cache; p.k_sr = k_sr; p.k_sh = k_sh;
  p.v = (const bf16_t*)v_cache; p.v_sr = v_sr; p.v_sh = v_sh;
  p.o = (bf16_t*)o; p.o_st = o_st; p.o_sh = o_sh;
  p.lse = lse; p.lse_st = lse_st; p.lse_sh = lse_sh;
  p.x_cu = x_cu; p.ctx_lens = context_lens;
  p.table = cmp_block_tables; p.table_stride = table_stride; p.page_size = page_size;
  p.G = QH / KH; p.KH = KH;
  p.scale_log2 = sm_scale * NSA_LOG2E;
  p.kernel_size = kernel_size; p.stride = stride; p.window = 0;
  return nsa_fwd_tile_launch(p, 0, true, B, x_maxlen, D, VD, (hipStream_t)stream);
}

int nsa_paged_swa_fwd(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr, int64_t k_sh,
                      const void* v_cache, int64_t v_sr, int64_t v_sh, void* o, int64_t o_st, int64_t o_sh,
                      float* lse, int64_t lse_st, int64_t lse_sh, const int32_t* x_cu, const int32_t* context_lens,
                      const int32_t* block_tables, int table_stride, int page_size, int B, int x_maxlen, int QH,
                      int KH, int D, int VD, int window, float sm_scale, void* stream) {
  int rc = check_heads("paged_swa_fwd", QH, KH, D, VD);
  if (rc) return rc;
  rc = check_page("paged_swa_fwd", page_size);
  if (rc) return rc;
  NsaFwdTileParams p{};
  p.q = (const bf16_t*)q; p.q_st = q_st; p.q_sh = q_sh;
  p.k = (const bf16_t*)k_cache; p.k_sr = k_sr; p.k_sh = k_sh;
  p.v = (const bf16_t*)v_cache; p.v_sr = v_sr; p.v_sh = v_sh;
  p.o = (bf16_t*)o; p.o_st = o_st; p.o_sh = o_sh;
  p.lse = lse; p.lse_st = lse_st; p.lse_sh = lse_sh;
  p.x_cu = x_cu; p.ctx_lens = context_lens;
  p.table = block_tables; p.table_stride = table_stride; p.page_size = page_size;
  p.G = QH / KH; p.KH = KH;
  p.scale_log2 = sm_scale * NSA_LOG2E;
  p.kernel_size = 1; p.stride = 1; p.window = window;
  return nsa_fwd_tile_launch(p, 1, true, B, x_maxlen, D, VD, (hipStream_t)stream);
}

static int paged_topk_select_impl(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr,
                          int64_t k_sh, const float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk,
                          int64_t tk_sh, int64_t tk_st, const int32_t* x_cu, const int32_t* context_lens,
                          const int32_t* cmp_block_tables, int table_stride, int page_size, int B, int x_maxlen,
                          int fixed_num_slc_blocks, int QH, int KH, int D, int kernel_size, int stride,
                          int block_size, int top_n, int num_init, int num_local, int ignore_index, float sm_scale,
                          int total_tokens, void* workspace, int64_t workspace_bytes, void* stream) {
  int rc = check_heads("paged_topk_select", QH, KH, D, 32);
  if (rc) return rc;
  rc = check_nsa_sizes("paged_topk_select", kernel_size, stride, block_size);
  if (rc) return rc;
  rc = check_page("paged_topk_select", page_size);
  if (rc) return rc;
  NSA_REQUIRE(top_n >= 1 && top_n <= 64, NSA_ERR_BAD_ARG, "paged_topk_select: top_n %d must be in [1,64]", top_n);
  NSA_REQUIRE(num_init >= 0 && num_local >= 0 && num_init + num_local <= top_n, NSA_ERR_BAD_ARG,
              "paged_topk_select: num_init %d + num_local %d must be <= top_n %d", num_init, num_local, top_n);
  NSA_REQUIRE(fixed_num_slc_blocks >= 1, NSA_ERR_BAD_ARG, "paged_topk_select: fixed_num_slc_blocks must be >= 1");
  NsaTopkParams p{};
  p.q = (const bf16_t*)q; p.q_st = q_st; p.q_sh = q_sh;
  p.ck = (const bf16_t*)k_cache; p.ck_sr = k_sr; p.ck_sh = k_sh;
  p.lse = lse; p.lse_st = lse_st; p.lse_sh = lse_sh;
  p.topk = topk; p.tk_sh = tk_sh; p.tk_st = tk_st;
  p.x_cu = x_cu; p.ctx_lens = context_lens;
  p.table = cmp_block_tables; p.table_stride = table_stride; p.page_size = page_size;
  p.G = QH / KH; p.KH = KH;
  p.scale_log2 = sm_scale * NSA_LOG2E;
  p.kernel_size = kernel_size; p.stride = stride; p.block_size = block_size;
  p.top_n = top_n; p.num_init = num_init; p.num_local = num_local; p.ignore_index = ignore_index;
  p.nb_max = fixed_num_slc_blocks;
  if (workspace != nullptr && nsa_tuning_knob("topk_two_pass", 1) != 0 && nsa_topk_two_pass_supported(p, D))
    return nsa_topk_two_pass_launch(p, true, B, x_maxlen, total_tokens, D, workspace, workspace_bytes,
                                    (hipStream_t)stream);
  return nsa_topk_launch(p, true, B, x_maxlen, D, (hipStream_t)stream);
}

int nsa_paged_topk_select(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr,
                          int64_t k_sh, const float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk,
                          int64_t tk_sh, int64_t tk_st, const int32_t* x_cu, const int32_t* context_lens,
                          const int32_t* cmp_block_tables, int table_stride, int page_size, int B, int x_maxlen,
                          int fixed_num_slc_blocks, int QH, int KH, int D, int kernel_size, int stride,
                          int block_size, int top_n, int num_init, int num_local, int ignore_index, float sm_scale,
                          void* stream) {
  return paged_topk_select_impl(q, q_st, q_sh, k_cache, k_sr, k_sh, lse, lse_st, lse_sh, topk, tk_sh, tk_st, x_cu,
                                context_lens, cmp_block_tables, table_stride, page_size, B, x_maxlen,
                                fixed_num_slc_blocks, QH, KH, D, kernel_size, stride, block_size, top_n, num_init,
                                num_local, ignore_index, sm_scale, 0, nullptr, 0, stream);
}

int nsa_paged_topk_select_ws(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr,
                             int64_t k_sh, const float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk,
                             int64_t tk_sh, int64_t tk_st, const int32_t* x_cu, const int32_t* context_lens,
                             const int32_t* cmp_block_tables, int table_stride, int page_size, int B, int x_maxlen,
                             int fixed_num_slc_blocks, int QH, int KH, int D, int kernel_size, int stride,
                             int block_size, int top_n, int num_init, int num_local, int ignore_index,
                             float sm_scale, int total_tokens, void* workspace, int64_t workspace_bytes,
                             void* stream) {
  NSA_REQUIRE(total_tokens >= 0 && (workspace == nullptr || workspace_bytes > 0), NSA_ERR_BAD_ARG,
              "paged_topk_select_ws: bad token count %d or workspace size %lld", total_tokens,
              (long long)workspace_bytes);
  return paged_topk_select_impl(q, q_st, q_sh, k_cache, k_sr, k_sh, lse, lse_st, lse_sh, topk, tk_sh, tk_st, x_cu,
                                context_lens, cmp_block_tables, table_stride, page_size, B, x_maxlen,
                                fixed_num_slc_blocks, QH, KH, D, kernel_size, stride, block_size, top_n, num_init,
                                num_local, ignore_index, sm_scale, total_tokens, workspace, workspace_bytes, stream);
}

int nsa_paged_slc_attn_fwd(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr,
                           int64_t k_sh, const void* v_cache, int64_t v_sr, int64_t v_sh, const int32_t* topk,
                           int64_t tk_sh, int64_t tk_st, void* o, int64_t o_st, int64_t o_sh, float* lse,
                           int64_t lse_st, int64_t lse_sh, const int32_t* x_cu, const int32_t* context_lens,
                           const int32_t* block_tables, int table_stride, int page_size, int B, int x_maxlen,
                           int QH, int KH, int D, int VD, int block_size, int top_n, float sm_scale, void* stream) {
  int rc = check_heads("paged_slc_attn_fwd", QH, KH, D, VD);
  if (rc) return rc;
  rc = check_page("paged_slc_attn_fwd", page_size);
  if (rc) return rc;
  NSA_REQUIRE(block_size % 32 == 0 && block_size > 0, NSA_ERR_UNSUPPORTED,
              "paged_slc_attn_fwd: block_size %d must be a multiple of 32", block_size);
  NSA_REQUIRE(top_n >= 1 && top_n <= 64, NSA_ERR_BAD_ARG, "paged_slc_attn_fwd: top_n %d must be in [1,64]", top_n);
  NsaSlcParams p{};
  p.q = (const bf16_t*)q; p.q_st = q_st; p.q_sh = q_sh;
  p.k = (const bf16_t*)k_cache; p.k_sr = k_sr; p.k_sh = k_sh;
  p.v = (const bf16_t*)v_cache; p.v_sr = v_sr; p.v_sh = v_sh;
  p.o = (bf16_t*)o; p.o_st = o_st; p.o_sh = o_sh;
  p.lse = lse; p.lse_st = lse_st; p.lse_sh = lse_sh;
  p.topk = topk; p.tk_sh = tk_sh; p.tk_st = tk_st;
  p.x_cu = x_cu; p.ctx_lens = context_lens;
  p.table = block_tables; p.table_stride = table_stride; p.page_size = page_size;
  p.G = QH / KH; p.KH = KH; p.top_n = top_n; p.block_size = block_size;
  p.scale_log2 = sm_scale * NSA_LOG2E;
  return nsa_slc_fwd_launch(p, true, B, x_maxlen, D, VD, (hipStream_t)stream);
}

}  // extern "C"

// ------------------------------------------------------------------------------------------------ fused decode
extern "C" {

int nsa_decode_cmp_topk(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr, int64_t k_sh,
                        const void* v_cache, int64_t v_sr, int64_t v_sh, void* cmp_o, int64_t co_st, int64_t co_sh,
                        float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk, int64_t tk_sh, int64_t tk_st,
                        const int32_t* context_lens, const int32_t* cmp_block_tables, int cmp_table_stride,
                        int page_size, int B, int QH, int KH, int D, int VD, int fixed_y_maxlen,
                        int fixed_num_slc_blocks, int kernel_size, int stride, int block_size, int top_n,
                        int num_init, int num_local, int ignore_index, float sm_scale, void* stream) {
  int rc = check_heads("decode_cmp_topk", QH, KH, D, VD);
  if (rc) return rc;
  rc = check_nsa_sizes("decode_cmp_topk", kernel_size, stride, block_size);
  if (rc) return rc;
  rc = check_page("decode_cmp_topk", page_size);
  if (rc) return rc;
  NSA_REQUIRE(QH / KH <= 16, NSA_ERR_UNSUPPORTED, "decode_cmp_topk: at most 16 q-heads per kv head (got %d)", QH / KH);
  NSA_REQUIRE(top_n >= 1 && top_n <= 64 && num_init >= 0 && num_local >= 0 && num_init + num_local <= top_n,
              NSA_ERR_BAD_ARG, "decode_cmp_topk: bad top_n/num_init/num_local %d/%d/%d", top_n, num_init, num_local);
  NSA_REQUIRE(fixed_y_maxlen >= 1 && fixed_num_slc_blocks >= 1, NSA_ERR_BAD_ARG,
              "decode_cmp_topk: fixed_y_maxlen and fixed_num_slc_blocks must be positive");
  NsaDecodeParams p{};
  p.q = (const bf16_t*)q; p.q_st = q_st; p.q_sh = q_sh;
  p.k = (const bf16_t*)k_cache; p.k_sr = k_sr; p.k_sh = k_sh;
  p.v = (const bf16_t*)v_cache; p.v_sr = v_sr; p.v_sh = v_sh;
  p.cmp_o = (bf16_t*)cmp_o; p.co_st = co_st; p.co_sh = co_sh;
  p.lse_out = lse; p.lse_st = lse_st; p.lse_sh = lse_sh;
  p.topk = topk; p.tk_sh = tk_sh; p.tk_st = tk_st;
  p.ctx_lens = context_lens;
  p.cmp_table = cmp_block_tables; p.cmp_table_stride = cmp_table_stride; p.page_size = page_size;
  p.G = QH / KH; p.KH = KH;
  p.scale_log2 = sm_scale * NSA_LOG2E;
  p.kernel_size = kernel_size; p.stride = stride; p.block_size = block_size;
  p.top_n = top_n; p.num_init = num_init; p.num_local = num_local; p.ignore_index = ignore_index;
  p.y_cap = fixed_y_maxlen; p.nb_cap = fixed_num_slc_blocks;
  return nsa_decode_cmp_topk_launch(p, B, D, VD, (hipStream_t)stream);
}

int nsa_decode_cmp_split(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr, int64_t k_sh,
                         const void* v_cache, int64_t v_sr, int64_t v_sh, void* cmp_o, int64_t co_st, int64_t co_sh,
                         float* lse, int64_t lse_st, int64_t lse_sh, float* pg, float* sp_m, float* sp_l, float* sp_o,
                         int nsplit, const int32_t* context_lens, const int32_t* cmp_block_tables,
                         int cmp_table_stride, int page_size, int B, int QH, int KH, int D, int VD,
                         int fixed_y_maxlen, int kernel_size, int stride, float sm_scale, void* stream) {
  int rc = check_heads("decode_cmp_split", QH, KH, D, VD);
  if (rc) return rc;
  rc = check_nsa_sizes("decode_cmp_split", kernel_size, stride, 0);
  if (rc) return rc;
  rc = check_page("decode_cmp_split", page_size);
  if (rc) return rc;
  NSA_REQUIRE(QH / KH <= 16, NSA_ERR_UNSUPPORTED, "decode_cmp_split: at most 16 q-heads per kv head (got %d)", QH / KH);
  NSA_REQUIRE(nsplit >= 1 && nsplit <= 64, NSA_ERR_BAD_ARG, "decode_cmp_split: nsplit %d must be in [1,64]", nsplit);
  NSA_REQUIRE(fixed_y_maxlen >= 1 && fixed_y_maxlen <= 32768, NSA_ERR_BAD_ARG,
              "decode_cmp_split: fixed_y_maxlen %d must be in [1,32768]", fixed_y_maxlen);
  NsaDecodeParams p{};
  p.q = (const bf16_t*)q; p.q_st = q_st; p.q_sh = q_sh;
  p.k = (const bf16_t*)k_cache; p.k_sr = k_sr; p.k_sh = k_sh;
  p.v = (const bf16_t*)v_cache; p.v_sr = v_sr; p.v_sh = v_sh;
  p.cmp_o = (bf16_t*)cmp_o; p.co_st = co_st; p.co_sh = co_sh;
  p.lse_out = lse; p.lse_st = lse_st; p.lse_sh = lse_sh;
  p.pg = pg; p.sp_m = sp_m; p.sp_l = sp_l; p.sp_o = sp_o;
  p.ctx_lens = context_lens;
  p.cmp_table = cmp_block_tables; p.cmp_table_stride = cmp_table_stride; p.page_size = page_size;
  p.G = QH / KH; p.KH = KH;
  p.scale_log2 = sm_scale * NSA_LOG2E;
  p.kernel_size = kernel_size; p.stride = stride;
  p.y_cap = fixed_y_maxlen;
  return nsa_decode_cmp_split_launch(p, B, nsplit, D, VD, (hipStream_t)stream);
}

static void fill_decode_split(NsaDecodeParams& p, int fixed_y_maxlen, int fixed_num_slc_blocks, int table_stride) {
  p.y_cap = fixed_y_maxlen; p.nb_cap = fixed_num_slc_blocks; p.table_stride = table_stride;
}

int nsa_decode_split_fits(int D, int VD, int fixed_y_maxlen, int fixed_num_slc_blocks, int table_stride) {
  NsaDecodeParams p{};
  fill_decode_split(p, fixed_y_maxlen, fixed_num_slc_blocks, table_stride);
  return nsa_decode_split_lds_bytes(p, D, VD) > 0 ? 1 : 0;
}

int nsa_decode_split_lds_total(int D, int VD, int fixed_y_maxlen, int fixed_num_slc_blocks, int table_stride) {
  NsaDecodeParams p{};
  fill_decode_split(p, fixed_y_maxlen, fixed_num_slc_blocks, table_stride);
  const int dyn = nsa_decode_split_lds_bytes(p, D, VD);
  return dyn > 0 ? dyn + nsa_decode_split_static_lds_bytes() : 0;
}

static int decode_split_impl(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr, int64_t k_sh,
                     const void* v_cache, int64_t v_sr, int64_t v_sh, const void* w, int64_t w_st, int64_t w_sh,
                     void* out, int64_t o_st, int64_t o_sh, void* cmp_o, void* slc_o, void* swa_o, int64_t co_st,
                     int64_t co_sh, float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk, int64_t tk_sh,
                     int64_t tk_st, float* sp_m, float* sp_l, float* sp_o, void* sp_keep_p, float* sp_keep_m,
                     int nsplit, const int32_t* cmp_slot_mapping, const int32_t* context_lens,
                     const int32_t* block_tables, int table_stride, const int32_t* cmp_block_tables,
                     int cmp_table_stride, int page_size, int B, int QH, int KH, int D, int VD, int fixed_y_maxlen,
                     int fixed_num_slc_blocks, int kernel_size, int stride, int block_size, int top_n, int num_init,
                     int num_local, int ignore_index, int window, float sm_scale, int slc_nsplit, float* sp2_ml,
                     float* sp2_o, void* cmp_tmp, void* stream) {
  int rc = check_heads("decode_split", QH, KH, D, VD);
  if (rc) return rc;
  rc = check_nsa_sizes("decode_split", kernel_size, stride, block_size);
  if (rc) return rc;
  rc = check_page("decode_split", page_size);
  if (rc) return rc;
  NSA_REQUIRE(QH / KH <= 16, NSA_ERR_UNSUPPORTED, "decode_split: at most 16 q-heads per kv head (got %d)", QH / KH);
  NSA_REQUIRE(nsplit >= 1 && nsplit <= 64, NSA_ERR_BAD_ARG, "decode_split: nsplit %d must be in [1,64]", nsplit);
  NSA_REQUIRE(block_size % 32 == 0, NSA_ERR_UNSUPPORTED, "decode_split: block_size %d must be a multiple of 32",
              block_size);
  NSA_REQUIRE(top_n >= 1 && top_n <= 64 && num_init >= 0 && num_local >= 0 && num_init + num_local <= top_n,
              NSA_ERR_BAD_ARG, "decode_split: bad top_n %d / num_init %d / num_local %d", top_n, num_init, num_local);
  NSA_REQUIRE(fixed_y_maxlen >= 1 && fixed_num_slc_blocks >= 1, NSA_ERR_BAD_ARG,
              "decode_split: fixed_y_maxlen %d and fixed_num_slc_blocks %d must be positive", fixed_y_maxlen,
              fixed_num_slc_blocks);
  NSA_REQUIRE(out && w && sp_m && sp_l && sp_o && sp_keep_p && sp_keep_m, NSA_ERR_BAD_ARG,
              "decode_split: out, w and the five scratch buffers are required");
  NSA_REQUIRE(slc_nsplit >= 1 && slc_nsplit <= 16, NSA_ERR_BAD_ARG, "decode_split: slc_nsplit %d must be in [1,16]",
              slc_nsplit);
  NSA_REQUIRE(slc_nsplit == 1 || (sp2_ml && sp2_o && cmp_tmp), NSA_ERR_BAD_ARG,
              "decode_split: slc_nsplit > 1 needs the three buffers of the window / selected parts");
  NsaDecodeParams p{};
  p.slc_nsplit = slc_nsplit; p.sp2_ml = sp2_ml; p.sp2_o = sp2_o; p.cmp_tmp = (bf16_t*)cmp_tmp;
  p.q = (const bf16_t*)q; p.q_st = q_st; p.q_sh = q_sh;
  p.k = (const bf16_t*)k_cache; p.k_sr = k_sr; p.k_sh = k_sh;
  p.v = (const bf16_t*)v_cache; p.v_sr = v_sr; p.v_sh = v_sh;
  p.w = (const bf16_t*)w; p.w_st = w_st; p.w_sh = w_sh;
  p.out = (bf16_t*)out; p.o_st = o_st; p.o_sh = o_sh;
  p.cmp_o = (bf16_t*)cmp_o; p.slc_o = (bf16_t*)slc_o; p.swa_o = (bf16_t*)swa_o; p.co_st = co_st; p.co_sh = co_sh;
  p.lse_out = lse; p.lse_st = lse_st; p.lse_sh = lse_sh;
  p.topk = topk; p.tk_sh = tk_sh; p.tk_st = tk_st;
  p.sp_m = sp_m; p.sp_l = sp_l; p.sp_o = sp_o;
  p.sp_keep_p = (_Float16*)sp_keep_p; p.sp_keep_m = sp_keep_m; p.nsplit = nsplit;
  p.ctx_lens = context_lens;
  p.cmp_slots = cmp_slot_mapping;
  p.table = block_tables;
  p.cmp_table = cmp_block_tables; p.cmp_table_stride = cmp_table_stride; p.page_size = page_size;
  p.G = QH / KH; p.KH = KH;
  p.scale_log2 = sm_scale * NSA_LOG2E;
  p.kernel_size = kernel_size; p.stride = stride; p.block_size = block_size; p.window = window; p.top_n = top_n;
  p.num_init = num_init; p.num_local = num_local; p.ignore_index = ignore_index;
  fill_decode_split(p, fixed_y_maxlen, fixed_num_slc_blocks, table_stride);
  return nsa_decode_split_launch(p, B, D, VD, (hipStream_t)stream);
}

int nsa_decode_split(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr, int64_t k_sh,
                     const void* v_cache, int64_t v_sr, int64_t v_sh, const void* w, int64_t w_st, int64_t w_sh,
                     void* out, int64_t o_st, int64_t o_sh, void* cmp_o, void* slc_o, void* swa_o, int64_t co_st,
                     int64_t co_sh, float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk, int64_t tk_sh,
                     int64_t tk_st, float* sp_m, float* sp_l, float* sp_o, void* sp_keep_p, float* sp_keep_m,
                     int nsplit, const int32_t* cmp_slot_mapping, const int32_t* context_lens,
                     const int32_t* block_tables, int table_stride, const int32_t* cmp_block_tables,
                     int cmp_table_stride, int page_size, int B, int QH, int KH, int D, int VD, int fixed_y_maxlen,
                     int fixed_num_slc_blocks, int kernel_size, int stride, int block_size, int top_n, int num_init,
                     int num_local, int ignore_index, int window, float sm_scale, void* stream) {
  return decode_split_impl(q, q_st, q_sh, k_cache, k_sr, k_sh, v_cache, v_sr, v_sh, w, w_st, w_sh, out, o_st, o_sh, cmp_o, slc_o,
                           swa_o, co_st, co_sh, lse, lse_st, lse_sh, topk, tk_sh, tk_st, sp_m, sp_l, sp_o, sp_keep_p,
                           sp_keep_m, nsplit, cmp_slot_mapping, context_lens, block_tables, table_stride,
                           cmp_block_tables, cmp_table_stride, page_size, B, QH, KH, D, VD, fixed_y_maxlen,
                           fixed_num_slc_blocks, kernel_size, stride, block_size, top_n, num_init, num_local,
                           ignore_index, window, sm_scale, 1, nullptr, nullptr, nullptr, stream);
}

int nsa_decode_split_parts(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr, int64_t k_sh,
                     const void* v_cache, int64_t v_sr, int64_t v_sh, const void* w, int64_t w_st, int64_t w_sh,
                     void* out, int64_t o_st, int64_t o_sh, void* cmp_o, void* slc_o, void* swa_o, int64_t co_st,
                     int64_t co_sh, float* lse, int64_t lse_st, int64_t lse_sh, int32_t* topk, int64_t tk_sh,
                     int64_t tk_st, float* sp_m, float* sp_l, float* sp_o, void* sp_keep_p, float* sp_keep_m,
                     int nsplit, const int32_t* cmp_slot_mapping, const int32_t* context_lens,
                     const int32_t* block_tables, int table_stride, const int32_t* cmp_block_tables,
                     int cmp_table_stride, int page_size, int B, int QH, int KH, int D, int VD, int fixed_y_maxlen,
                     int fixed_num_slc_blocks, int kernel_size, int stride, int block_size, int top_n, int num_init,
                     int num_local, int ignore_index, int window, float sm_scale, int slc_nsplit, float* sp2_ml,
                     float* sp2_o, void* cmp_tmp, void* stream) {
  return decode_split_impl(q, q_st, q_sh, k_cache, k_sr, k_sh, v_cache, v_sr, v_sh, w, w_st, w_sh, out, o_st, o_sh, cmp_o, slc_o,
                           swa_o, co_st, co_sh, lse, lse_st, lse_sh, topk, tk_sh, tk_st, sp_m, sp_l, sp_o, sp_keep_p,
                           sp_keep_m, nsplit, cmp_slot_mapping, context_lens, block_tables, table_stride,
                           cmp_block_tables, cmp_table_stride, page_size, B, QH, KH, D, VD, fixed_y_maxlen,
                           fixed_num_slc_blocks, kernel_size, stride, block_size, top_n, num_init, num_local,
                           ignore_index, window, sm_scale, slc_nsplit, sp2_ml, sp2_o, cmp_tmp, stream);
}

int nsa_decode_slc_swa_combine(const void* q, int64_t q_st, int64_t q_sh, const void* k_cache, int64_t k_sr,
                               int64_t k_sh, const void* v_cache, int64_t v_sr, int64_t v_sh, const void* w,
                               int64_t w_st, int64_t w_sh, int32_t* topk, int64_t tk_sh, int64_t tk_st,
                               const float* pg, int fixed_y_maxlen, int fixed_num_slc_blocks, int kernel_size,
                               int stride, int num_init, int num_local, int ignore_index, const void* cmp_o,
                               void* slc_o, void* swa_o, int64_t co_st, int64_t co_sh, void* out, int64_t o_st,
                               int64_t o_sh, const int32_t* context_lens, const int32_t* block_tables,
                               int table_stride, int page_size, int B, int QH, int KH, int D, int VD, int block_size,
                               int top_n, int window, float sm_scale, void* stream) {
  int rc = check_heads("decode_slc_swa_combine", QH, KH, D, VD);
  if (rc) return rc;
  rc = check_page("decode_slc_swa_combine", page_size);
  if (rc) return rc;
  NSA_REQUIRE(QH / KH <= 16, NSA_ERR_UNSUPPORTED, "decode_slc_swa_combine: at most 16 q-heads per kv head (got %d)",
              QH / KH);
  NSA_REQUIRE(block_size % 32 == 0 && block_size > 0, NSA_ERR_UNSUPPORTED,
              "decode_slc_swa_combine: block_size %d must be a multiple of 32", block_size);
  NSA_REQUIRE(top_n >= 1 && top_n <= 64, NSA_ERR_BAD_ARG, "decode_slc_swa_combine: top_n %d must be in [1,64]", top_n);
  NSA_REQUIRE(out == nullptr || (w != nullptr && cmp_o != nullptr), NSA_ERR_BAD_ARG,
              "decode_slc_swa_combine: the combined output needs the gates and the compressed-branch output");
  if (pg != nullptr) {
    rc = check_nsa_sizes("decode_slc_swa_combine", kernel_size, stride, block_size);
    if (rc) return rc;
    NSA_REQUIRE(num_init >= 0 && num_local >= 0 && num_init + num_local <= top_n, NSA_ERR_BAD_ARG,
                "decode_slc_swa_combine: num_init %d + num_local %d must be <= top_n %d", num_init, num_local, top_n);
    NSA_REQUIRE(fixed_num_slc_blocks >= 1 && fixed_num_slc_blocks <= 8192 && fixed_y_maxlen >= 1, NSA_ERR_BAD_ARG,
                "decode_slc_swa_combine: fixed_num_slc_blocks %d must be in [1,8192]", fixed_num_slc_blocks);
  }
  NsaDecodeParams p{};
  p.q = (const bf16_t*)q; p.q_st = q_st; p.q_sh = q_sh;
  p.k = (const bf16_t*)k_cache; p.k_sr = k_sr; p.k_sh = k_sh;
  p.v = (const bf16_t*)v_cache; p.v_sr = v_sr; p.v_sh = v_sh;
  p.w = (const bf16_t*)w; p.w_st = w_st; p.w_sh = w_sh;
  p.topk = topk; p.tk_sh = tk_sh; p.tk_st = tk_st;
  p.pg = const_cast<float*>(pg);
  p.y_cap = fixed_y_maxlen; p.nb_cap = fixed_num_slc_blocks;
  p.kernel_size = kernel_size; p.stride = stride;
  p.num_init = num_init; p.num_local = num_local; p.ignore_index = ignore_index;
  p.cmp_o = (bf16_t*)const_cast<void*>(cmp_o); p.slc_o = (bf16_t*)slc_o; p.swa_o = (bf16_t*)swa_o;
  p.co_st = co_st; p.co_sh = co_sh;
  p.out = (bf16_t*)out; p.o_st = o_st; p.o_sh = o_sh;
  p.ctx_lens = context_lens;
  p.table = block_tables; p.table_stride = table_stride; p.page_size = page_size;
  p.G = QH / KH; p.KH = KH;
  p.scale_log2 = sm_scale * NSA_LOG2E;
  p.block_size = block_size; p.window = window; p.top_n = top_n;
  return nsa_decode_slc_swa_launch(p, B, D, VD, (hipStream_t)stream);
}

int nsa_decode_fused_fits(int D, int VD, int fixed_y_maxlen, int fixed_num_slc_blocks, int table_stride,
                          int page_size) {
  if (fixed_y_maxlen < 1 || fixed_num_slc_blocks < 1 || table_stride < 1 || page_size < 1) return 0;
  NsaDecodeParams p{};
  p.y_cap = fixed_y_maxlen; p.nb_cap = fixed_num_slc_blocks; p.table_stride = table_stride; p.page_size = page_size;
  return nsa_decode_fused_lds_bytes(p, D, VD) > 0 ? 1 : 0;
}

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
                     float sm_scale, void* stream) {
  int rc = check_heads("decode_fused", QH, KH, D, VD);
  if (rc) return rc;
  rc = check_nsa_sizes("decode_fused", kernel_size, stride, block_size);
  if (rc) return rc;
  rc = check_page("decode_fused", page_size);
  if (rc) return rc;
  NSA_REQUIRE(QH / KH <= 16, NSA_ERR_UNSUPPORTED, "decode_fused: at most 16 q-heads per kv head (got %d)", QH / KH);
  NSA_REQUIRE(block_size % 32 == 0, NSA_ERR_UNSUPPORTED, "decode_fused: block_size %d must be a multiple of 32",
              block_size);
  NSA_REQUIRE(o_st % 4 == 0 && o_sh % 4 == 0 && co_st % 4 == 0 && co_sh % 4 == 0, NSA_ERR_BAD_ARG,
              "decode_fused: output strides must be multiples of 4 elements (8-byte stores)");
  NSA_REQUIRE(top_n >= 1 && top_n <= 64 && num_init >= 0 && num_local >= 0 && num_init + num_local <= top_n,
              NSA_ERR_BAD_ARG, "decode_fused: bad top_n/num_init/num_local %d/%d/%d", top_n, num_init, num_local);
  NSA_REQUIRE(fixed_y_maxlen >= 1 && fixed_num_slc_blocks >= 1 && table_stride >= 1 && cmp_table_stride >= 1,
              NSA_ERR_BAD_ARG, "decode_fused: fixed_y_maxlen, fixed_num_slc_blocks and the table widths must be positive");
  NSA_REQUIRE(out != nullptr && w != nullptr, NSA_ERR_BAD_ARG, "decode_fused: out and w are required");
  NSA_REQUIRE(window >= 0, NSA_ERR_BAD_ARG, "decode_fused: window %d must be >= 0", window);
  NsaDecodeParams p{};
  p.q = (const bf16_t*)q; p.q_st = q_st; p.q_sh = q_sh;
  p.k = (const bf16_t*)k_cache; p.k_sr = k_sr; p.k_sh = k_sh;
  p.v = (const bf16_t*)v_cache; p.v_sr = v_sr; p.v_sh = v_sh;
  p.w = (const bf16_t*)w; p.w_st = w_st; p.w_sh = w_sh;
  p.out = (bf16_t*)out; p.o_st = o_st; p.o_sh = o_sh;
  p.cmp_o = (bf16_t*)cmp_o; p.slc_o = (bf16_t*)slc_o; p.swa_o = (bf16_t*)swa_o; p.co_st = co_st; p.co_sh = co_sh;
  p.lse_out = lse; p.lse_st = lse_st; p.lse_sh = lse_sh;
  p.topk = topk; p.tk_sh = tk_sh; p.tk_st = tk_st;
  p.ctx_lens = context_lens;
  p.table = block_tables; p.table_stride = table_stride;
  p.cmp_table = cmp_block_tables; p.cmp_table_stride = cmp_table_stride; p.page_size = page_size;
  p.cmp_slots = cmp_slot_mapping;
  NSA_REQUIRE((new_k == nullptr) == (new_v == nullptr) && (new_k == nullptr) == (slot_mapping == nullptr),
              NSA_ERR_BAD_ARG, "decode_fused: new_k, new_v and slot_mapping must be given together");
  p.new_k = (const bf16_t*)new_k; p.nk_st = nk_st; p.nk_sh = nk_sh;
  p.new_v = (const bf16_t*)new_v; p.nv_st = nv_st; p.nv_sh = nv_sh;
  p.raw_slots = slot_mapping;
  p.G = QH / KH; p.KH = KH;
  p.scale_log2 = sm_scale * NSA_LOG2E;
  p.kernel_size = kernel_size; p.stride = stride; p.block_size = block_size; p.window = window;
  p.top_n = top_n; p.num_init = num_init; p.num_local = num_local; p.ignore_index = ignore_index;
  p.y_cap = fixed_y_maxlen; p.nb_cap = fixed_num_slc_blocks;
  return nsa_decode_fused_launch(p, B, D, VD, (hipStream_t)stream);
}

}  // extern "C"

// nsa_decode_split_static: the two-launch split decode step for callers that cannot allocate device memory
// (code under graph capture, tight serving loops).  Same kernels as nsa_decode_split; the five scratch buffers that
// entry point takes from its caller are carved out of one file-scope device array instead.
//
// The array exists once per GPU and keeps the contents of the last call.  The kernels overwrite every element they
// later read (the parts' statistics and outputs, the probabilities and maxima of every unit below the request's own
// compressed length), so nothing has to be cleared between calls; two calls that overlap on one GPU (different
// streams, or different threads) race on it.
#include <mutex>
#include "nsa_common.h"
#include "nsa_api_internal.h"

namespace {

constexpr size_t STATIC_SCRATCH_BYTES = (size_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
std::mutex g_lock;
unsigned char* g_scratch_ptr[MAX_DEVICES] = {};  // device address of `scratch` on each GPU, resolved on first use

// Device address of the array's copy on the GPU that owns `dev_ptr` (the array's name is only a host-side handle, and
// every GPU has its own copy at its own address).  The GPU is taken from the output pointer, not from the calling
// thread's current device, so a caller whose current device differs from the one its tensors and stream live on
// still gets the right copy; the first call for a GPU makes it current for the duration of the lookup.
int scratch_base(const void* dev_ptr, unsigned char** base) {
  int dev = -1;
  hipPointerAttribute_t attr;
  hipError_t e = hipPointerGetAttributes(&attr, dev_ptr);
  if (e == hipSuccess) {
    dev = attr.device;
  } else {
    (void)hipGetLastError();
    e = hipGetDevice(&dev);
  }
  if (e != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    nsa_set_error("decode_split_static: cannot tell the GPU of the output buffer (device %d): %s", dev,
                  hipGetErrorString(e));
    return NSA_ERR_LAUNCH;
  }
  std::lock_guard<std::mutex> guard(g_lock);
  if (g_scratch_ptr[dev] == nullptr) {
    int cur = -1;
    (void)hipGetDevice(&cur);
    if (cur != dev && hipSetDevice(dev) != hipSuccess) {
      nsa_set_error("decode_split_static: hipSetDevice(%d) failed", dev);
      return NSA_ERR_LAUNCH;
    }
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (cur != dev && cur >= 0) (void)hipSetDevice(cur);
    if (e != hipSuccess || ptr == nullptr) {
      nsa_set_error("decode_split_static: hipGetSymbolAddress(scratch) failed on device %d: %s", dev,
                    hipGetErrorString(e));
      return NSA_ERR_LAUNCH;
    }
    g_scratch_ptr[dev] = (unsigned char*)ptr;
  }
  *base = g_scratch_ptr[dev];
  return NSA_OK;
}

size_t round256(size_t n) { return (n + 255) & ~(size_t)255; }

struct ScratchLayout {
  size_t m, l, o, keep_p, keep_m, total;
};

ScratchLayout layout(int B, int KH, int VD, int nsplit, int fixed_y_maxlen) {
  const size_t pairs = (size_t)B * KH;
  const size_t ycap32 = ((size_t)fixed_y_maxlen + 31) / 32 * 32;
  ScratchLayout s{};
  size_t at = 0;
  s.m = at; at += round256(pairs * nsplit * 16 * sizeof(float));
  s.l = at; at += round256(pairs * nsplit * 16 * sizeof(float));
  s.o = at; at += round256(pairs * nsplit * 16 * VD * sizeof(float));
  s.keep_p = at; at += round256(pairs * 16 * ycap32 * sizeof(_Float16));
  s.keep_m = at; at += round256(pairs * (ycap32 / 32) * 16 * sizeof(float));
  s.total = at;
  return s;
}

}  // namespace

extern "C" {

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

int64_t nsa_decode_split_static_capacity(void) { return (int64_t)STATIC_SCRATCH_BYTES; }

int64_t nsa_decode_split_static_bytes(int B, int KH, int VD, int nsplit, int fixed_y_maxlen) {
  if (B < 0 || KH <= 0 || VD <= 0 || nsplit <= 0 || fixed_y_maxlen <= 0) return -1;
  return (int64_t)layout(B, KH, VD, nsplit, fixed_y_maxlen).total;
}

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
                            float sm_scale, void* stream) {
  NSA_REQUIRE(B >= 0 && KH > 0 && VD > 0 && nsplit >= 1 && nsplit <= 64 && fixed_y_maxlen >= 1, NSA_ERR_BAD_ARG,
              "decode_split_static: bad sizes B %d, kv heads %d, VD %d, nsplit %d, fixed_y_maxlen %d", B, KH, VD,
              nsplit, fixed_y_maxlen);
  const ScratchLayout s = layout(B, KH, VD, nsplit, fixed_y_maxlen);
  NSA_REQUIRE(s.total <= STATIC_SCRATCH_BYTES, NSA_ERR_UNSUPPORTED,
              "decode_split_static: B %d x kv heads %d x nsplit %d at fixed_y_maxlen %d needs %zu bytes of scratch, "
              "the static buffer holds %zu; use nsa_decode_split with caller-allocated scratch",
              B, KH, nsplit, fixed_y_maxlen, s.total, STATIC_SCRATCH_BYTES);
  if (B == 0) return NSA_OK;
  unsigned char* base = nullptr;
  int rc = scratch_base(out, &base);
  if (rc) return rc;
  return nsa_decode_split(q, q_st, q_sh, k_cache, k_sr, k_sh, v_cache, v_sr, v_sh, w, w_st, w_sh, out, o_st, o_sh,
                          cmp_o, slc_o, swa_o, co_st, co_sh, lse, lse_st, lse_sh, topk, tk_sh, tk_st,
                          (float*)(base + s.m), (float*)(base + s.l), (float*)(base + s.o), base + s.keep_p,
                          (float*)(base + s.keep_m), nsplit, cmp_slot_mapping, context_lens, block_tables,
                          table_stride, cmp_block_tables, cmp_table_stride, page_size, B, QH, KH, D, VD,
                          fixed_y_maxlen, fixed_num_slc_blocks, kernel_size, stride, block_size, top_n, num_init,
                          num_local, ignore_index, window, sm_scale, stream);
}

}  // extern "C"

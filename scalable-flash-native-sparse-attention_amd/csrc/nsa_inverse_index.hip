// Inverse of the top-n selection: for every (kv head, selection block) the ascending list of query tokens that
// selected the block, as a CSR (offsets + token ids), plus the prefix of fixed-size list chunks that the dK/dV
// kernel uses as its work items.  Built by a deterministic counting sort: per-token-chunk histograms,
// a scan over chunks and blocks, then an in-order fill, so no sort and no dense (block x token) scratch.
// Upstream: flash_nsa/ops/topk.py:782-945 (get_bind_from_find, dense scatter + per-row sort).
#include "nsa_common.h"
#include "nsa_api_internal.h"

namespace {

// Tokens per counting chunk: short chunks give the serial in-order fill more parallelism, long ones keep the
// [KH][chunks][blocks] histogram workspace small for very long batches.
__host__ __device__ inline int counting_chunk(int T) { return T <= 131072 ? 256 : 1024; }

__device__ __forceinline__ int find_seq(const int32_t* x_cu, int B, int tok) {
  int lo = 0, hi = B;  // last b with x_cu[b] <= tok
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (x_cu[mid] <= tok) lo = mid; else hi = mid;
  }
  return lo;
}

// grid (nchunks, KH), 256 threads, dynamic LDS nblk ints
__global__ void csr_count_kernel(const int32_t* topk, int64_t tk_sh, int64_t tk_st, int top_n, const int32_t* x_cu,
                                 const int32_t* kblk_cu, int B, int T, int nblk, int block_size, int32_t* chunk_cnt) {
  extern __shared__ int hist[];
  const int chunk = blockIdx.x, kh = blockIdx.y;
  for (int i = threadIdx.x; i < nblk; i += blockDim.x) hist[i] = 0;
  __syncthreads();
  const int CT = counting_chunk(T);
  const int t0 = chunk * CT;
  const int t1 = min(T, t0 + CT);
  for (int idx = threadIdx.x; idx < (t1 - t0) * top_n; idx += blockDim.x) {
    int tok = t0 + idx / top_n;
    int s = idx % top_n;
    int b = find_seq(x_cu, B, tok);
    int n = tok - x_cu[b];
    if (s < min(top_n, n / block_size + 1)) {
      int j = topk[(int64_t)kh * tk_sh + (int64_t)tok * tk_st + s];
      int nb = kblk_cu[b + 1] - kblk_cu[b];
      if (j >= 0 && j < nb) atomicAdd(&hist[kblk_cu[b] + j], 1);
    }
  }
  __syncthreads();
  int32_t* dst = chunk_cnt + ((int64_t)kh * gridDim.x + chunk) * nblk;
  for (int i = threadIdx.x; i < nblk; i += blockDim.x) dst[i] = hist[i];
}

// grid (KH), 1024 threads: chunk counts -> chunk bases (in place), list offsets, work-item offsets
__global__ __launch_bounds__(1024) void csr_scan_kernel(int32_t* chunk_cnt, int nchunks, int nblk, int64_t list_cap,
                                                        int chunk_tokens, int32_t* csr_off, int32_t* item_off) {
  __shared__ int part_a[1024];
  __shared__ int part_b[1024];
  const int kh = blockIdx.x;
  const int tid = threadIdx.x;
  int32_t* cnt = chunk_cnt + (int64_t)kh * nchunks * nblk;
  const int per = (nblk + 1023) / 1024;
  const int j0 = tid * per, j1 = min(nblk, j0 + per);
  int sum_a = 0, sum_b = 0;
  for (int j = j0; j < j1; j++) {
    int base = 0;
    for (int c = 0; c < nchunks; c++) {
      int v = cnt[(int64_t)c * nblk + j];
      cnt[(int64_t)c * nblk + j] = base;
      base += v;
    }
    // totals are parked in the output arrays and replaced by their prefixes below
    csr_off[(int64_t)kh * (nblk + 1) + j] = base;
    sum_a += base;
    sum_b += (base + chunk_tokens - 1) / chunk_tokens;
  }
  // exclusive scan of the per-thread sums (Hillis-Steele over the 1024 threads)
  part_a[tid] = sum_a;
  part_b[tid] = sum_b;
  __syncthreads();
  for (int d = 1; d < 1024; d <<= 1) {
    const int a = tid >= d ? part_a[tid - d] : 0, bb = tid >= d ? part_b[tid - d] : 0;
    __syncthreads();
    part_a[tid] += a;
    part_b[tid] += bb;
    __syncthreads();
  }
  part_a[tid] -= sum_a;
  part_b[tid] -= sum_b;
  int ra = part_a[tid] + (int)((int64_t)kh * list_cap), rb = part_b[tid];
  for (int j = j0; j < j1; j++) {
    int total = csr_off[(int64_t)kh * (nblk + 1) + j];
    csr_off[(int64_t)kh * (nblk + 1) + j] = ra;
    item_off[(int64_t)kh * (nblk + 1) + j] = rb;
    ra += total;
    rb += (total + chunk_tokens - 1) / chunk_tokens;
  }
  if (j0 < j1 && j1 == nblk) {  // the owner of the last block also writes the end markers
    csr_off[(int64_t)kh * (nblk + 1) + nblk] = ra;
    item_off[(int64_t)kh * (nblk + 1) + nblk] = rb;
  }
}

// grid (nchunks, KH), 64 threads: in-order fill
__global__ __launch_bounds__(64) void csr_fill_kernel(const int32_t* topk, int64_t tk_sh, int64_t tk_st, int top_n,
                                                      const int32_t* x_cu, const int32_t* kblk_cu, int B, int T,
                                                      int nblk, int block_size, const int32_t* chunk_base,
                                                      const int32_t* csr_off, int32_t* csr_tok) {
  extern __shared__ int cursor[];
  const int chunk = blockIdx.x, kh = blockIdx.y;
  const int lane = threadIdx.x;
  const int32_t* base = chunk_base + ((int64_t)kh * gridDim.x + chunk) * nblk;
  for (int i = lane; i < nblk; i += 64) cursor[i] = base[i] + csr_off[(int64_t)kh * (nblk + 1) + i];
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const int CT = counting_chunk(T);
  const int t0 = chunk * CT;
  const int t1 = min(T, t0 + CT);
  if (t0 >= t1) return;
  // The list positions depend on the order of the tokens, so the wave walks them one by one; the selection rows
  // do not, and are fetched a batch ahead so that the walk never waits for memory.
  constexpr int PF = 16;
  int b = find_seq(x_cu, B, t0);
  int x_begin = x_cu[b], x_end = x_cu[b + 1], kb_begin = kblk_cu[b], nb = kblk_cu[b + 1] - kb_begin;
  const int32_t* row0 = topk + (int64_t)kh * tk_sh;
  int nxt[PF], cur[PF];
  auto fetch = [&](int tb) {
#pragma unroll
    for (int u = 0; u < PF; u++)
      nxt[u] = (tb + u < t1 && lane < top_n) ? row0[(int64_t)(tb + u) * tk_st + lane] : -1;
  };
  fetch(t0);
  for (int tb = t0; tb < t1; tb += PF) {
#pragma unroll
    for (int u = 0; u < PF; u++) cur[u] = nxt[u];
    if (tb + PF < t1) fetch(tb + PF);
#pragma unroll
    for (int u = 0; u < PF; u++) {
      const int tok = tb + u;
      if (tok >= t1) break;
      if (tok >= x_end) {  // next (non-empty) sequence: the only loads inside the walk
        do { b++; } while (tok >= x_cu[b + 1]);
        x_begin = x_cu[b], x_end = x_cu[b + 1], kb_begin = kblk_cu[b], nb = kblk_cu[b + 1] - kb_begin;
      }
      const int n = tok - x_begin;
      const int nvalid = min(top_n, n / block_size + 1);
      if (lane < nvalid) {
        const int j = cur[u];
        if (j >= 0 && j < nb) {
          const int jb = kb_begin + j;
          const int pos = cursor[jb];
          cursor[jb] = pos + 1;
          csr_tok[pos] = n;
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  }
}

}  // namespace

extern "C" {

int64_t nsa_inverse_index_workspace_elems(int T, int KH, int nblk_total) {
  const int CT = counting_chunk(T);
  int64_t nchunks = (T + CT - 1) / CT;
  return (int64_t)KH * nchunks * nblk_total;
}

int nsa_build_inverse_index(const int32_t* topk, int64_t tk_sh, int64_t tk_st, int top_n, const int32_t* x_cu,
                            const int32_t* kblk_cu, int B, int T, int KH, int nblk_total, int block_size,
                            int chunk_tokens, int32_t* csr_off, int32_t* csr_tok, int32_t* item_off,
                            int32_t* workspace, int64_t workspace_elems, void* stream) {
  if (T <= 0 || B <= 0 || nblk_total <= 0) return NSA_OK;
  NSA_REQUIRE(top_n >= 1 && top_n <= 64, NSA_ERR_BAD_ARG, "build_inverse_index: top_n %d must be in [1,64]", top_n);
  NSA_REQUIRE(chunk_tokens >= 1, NSA_ERR_BAD_ARG, "build_inverse_index: chunk_tokens must be positive");
  NSA_REQUIRE(nblk_total * 4 <= 64 * 1024, NSA_ERR_UNSUPPORTED,
              "build_inverse_index: %d selection blocks exceed the LDS histogram (16384)", nblk_total);
  NSA_REQUIRE((int64_t)KH * T * top_n < 0x7fffffffLL, NSA_ERR_UNSUPPORTED,
              "build_inverse_index: KH*T*top_n exceeds int32 positions");
  NSA_REQUIRE(workspace_elems >= nsa_inverse_index_workspace_elems(T, KH, nblk_total), NSA_ERR_WORKSPACE,
              "build_inverse_index: workspace of %lld ints is too small", (long long)workspace_elems);
  hipStream_t s = (hipStream_t)stream;
  const int CT = counting_chunk(T);
  int nchunks = (T + CT - 1) / CT;
  size_t lds = (size_t)nblk_total * sizeof(int);
  dim3 grid(nchunks, KH);
  csr_count_kernel<<<grid, 256, lds, s>>>(topk, tk_sh, tk_st, top_n, x_cu, kblk_cu, B, T, nblk_total, block_size,
                                          workspace);
  int rc = nsa_check_launch("csr_count_kernel");
  if (rc) return rc;
  csr_scan_kernel<<<KH, 1024, 0, s>>>(workspace, nchunks, nblk_total, (int64_t)T * top_n, chunk_tokens, csr_off,
                                      item_off);
  rc = nsa_check_launch("csr_scan_kernel");
  if (rc) return rc;
  csr_fill_kernel<<<grid, 64, lds, s>>>(topk, tk_sh, tk_st, top_n, x_cu, kblk_cu, B, T, nblk_total, block_size,
                                        workspace, csr_off, csr_tok);
  return nsa_check_launch("csr_fill_kernel");
}

}  // extern "C"

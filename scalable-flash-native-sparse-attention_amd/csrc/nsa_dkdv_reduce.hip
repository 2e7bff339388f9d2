// Deterministic dK / dV: the dk/dv kernels store every workgroup's fp32 partial result in its own slot instead of
// adding it with atomics, and the kernels here sum the slots of a key in a fixed (ascending work-item) order.
// Upstream's counterpart is dkdv_repeat=True: per-q-head buffers followed by a sum over the heads
// (flash_nsa/ops/compress_attn.py:594-598,691-693, flash_nsa/ops/select_attn.py:528-531,639-641); here the q-heads of
// a group are already summed inside the MFMA accumulators, and what is left to order are the query chunks.
#include "nsa_common.h"
#include "nsa_api_internal.h"

namespace {

// compressed branch: grid (key tiles, B, KH).  The work items of a key tile are consecutive in the dk/dv kernel's
// grid.x (key-tile major), one per query chunk that sees the tile.
template <int KW>
__global__ __launch_bounds__(256) void cmp_dkdv_reduce_kernel(NsaBwdTileParams p, int D, int VD, int grid_x_items) {
  const int ktile = blockIdx.x, b = blockIdx.y, kh = blockIdx.z;
  const int x0 = p.x_cu[b];
  const int xl = p.x_cu[b + 1] - x0;
  const int kbase = p.k_cu[b];
  const int nkeys = p.k_cu[b + 1] - kbase;
  const int key0 = ktile * KW;
  if (key0 >= nkeys) return;
  // the enumeration of bwd_dkdv_kernel MODE_CMP
  const int nch = cdiv_i(xl, p.q_chunk_tokens);
  int start = 0;
  for (int kt = 0; kt < ktile; kt++)
    start += nch - min(nch, (p.stride * kt * KW + p.kernel_size - 1) / p.q_chunk_tokens);
  const int fc = min(nch, (p.stride * key0 + p.kernel_size - 1) / p.q_chunk_tokens);
  const int first = p.stride * key0 + p.kernel_size - 1;
  const int n4k = D / 4, n4v = VD / 4;
  const int per_key = n4k + n4v;
  const int nk_here = min(KW, nkeys - key0);
  for (int e = threadIdx.x; e < nk_here * per_key; e += 256) {
    const int kl = e / per_key, c4 = e - kl * per_key;
    const bool is_v = c4 >= n4k;
    const int d = (is_v ? c4 - n4k : c4) * 4;
    const int W = is_v ? VD : D;
    const float* part = is_v ? p.part_dv : p.part_dk;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int ch = fc; ch < nch; ch++) {
      // chunks without a visible row wrote nothing
      if (max(ch * p.q_chunk_tokens, first) >= min((ch + 1) * p.q_chunk_tokens, xl)) continue;
      const int64_t slot = ((int64_t)b * grid_x_items + start + (ch - fc)) * p.KH + kh;
      const f32x4 x = *reinterpret_cast<const f32x4*>(part + (slot * KW + kl) * W + d);
      acc[0] += x[0]; acc[1] += x[1]; acc[2] += x[2]; acc[3] += x[3];
    }
    float* dst = is_v ? (float*)p.dv + ((int64_t)kbase + key0 + kl) * p.dv_sr + (int64_t)kh * p.dv_sh + d
                      : (float*)p.dk + ((int64_t)kbase + key0 + kl) * p.dk_sr + (int64_t)kh * p.dk_sh + d;
    *reinterpret_cast<f32x4*>(dst) = acc;
  }
}

// selected branch: grid (selection blocks, sub-blocks, KH).  The work items of a block are the chunks of its token
// list, consecutive in the dk/dv kernel's grid.x; their sum is added to what dk / dv already hold (the window
// branch's result), one thread per element.
template <int KW>
__global__ __launch_bounds__(256) void slc_dkdv_reduce_kernel(NsaBwdTileParams p, int D, int VD, int grid_x_items,
                                                              int grid_y) {
  const int jb = blockIdx.x, sy = blockIdx.y, kh = blockIdx.z;
  const int32_t* ioff = p.item_off + (int64_t)kh * (p.nblk_total + 1);
  const int w0 = ioff[jb], w1 = ioff[jb + 1];
  if (w0 >= w1) return;
  const int b = p.blk_seq[jb];
  const int x0 = p.x_cu[b];
  const int xl = p.x_cu[b + 1] - x0;
  const int key0 = (jb - p.kblk_cu[b]) * p.block_size + sy * KW;
  const int nkeys = min(xl, (key0 / p.block_size + 1) * p.block_size);
  if (key0 >= nkeys) return;
  const int n4k = D / 4, n4v = VD / 4;
  const int per_key = n4k + n4v;
  const int nk_here = min(KW, nkeys - key0);
  for (int e = threadIdx.x; e < nk_here * per_key; e += 256) {
    const int kl = e / per_key, c4 = e - kl * per_key;
    const bool is_v = c4 >= n4k;
    const int d = (is_v ? c4 - n4k : c4) * 4;
    const int W = is_v ? VD : D;
    const float* part = is_v ? p.part_dv : p.part_dk;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int w = w0; w < w1; w++) {
      const int64_t slot = ((int64_t)kh * grid_x_items + w) * grid_y + sy;
      const f32x4 x = *reinterpret_cast<const f32x4*>(part + (slot * KW + kl) * W + d);
      acc[0] += x[0]; acc[1] += x[1]; acc[2] += x[2]; acc[3] += x[3];
    }
    float* dst = is_v ? (float*)p.dv + ((int64_t)x0 + key0 + kl) * p.dv_sr + (int64_t)kh * p.dv_sh + d
                      : (float*)p.dk + ((int64_t)x0 + key0 + kl) * p.dk_sr + (int64_t)kh * p.dk_sh + d;
    f32x4 cur = *reinterpret_cast<f32x4*>(dst);
    cur[0] += acc[0]; cur[1] += acc[1]; cur[2] += acc[2]; cur[3] += acc[3];
    *reinterpret_cast<f32x4*>(dst) = cur;
  }
}

}  // namespace

int nsa_dkdv_reduce_cmp_launch(const NsaBwdTileParams& p, int B, int max_q_len, int max_k_len, int D, int VD,
                               hipStream_t stream) {
  if (B <= 0 || max_k_len <= 0) return NSA_OK;
  const int KW = nsa_bwd_dkdv_slot_keys(0, 0);
  const int grid_x_items = (int)(nsa_bwd_dkdv_cmp_slots(1, 1, max_q_len, max_k_len, p.q_chunk_tokens, p.kernel_size,
                                                         p.stride));
  if (grid_x_items <= 0) return NSA_OK;
  dim3 grid(cdiv_i(max_k_len, KW), B, p.KH);
  if (KW == 128) cmp_dkdv_reduce_kernel<128><<<grid, 256, 0, stream>>>(p, D, VD, grid_x_items);
  else cmp_dkdv_reduce_kernel<256><<<grid, 256, 0, stream>>>(p, D, VD, grid_x_items);
  return nsa_check_launch("cmp_dkdv_reduce_kernel");
}

int nsa_dkdv_reduce_slc_launch(const NsaBwdTileParams& p, int n_items_bound, int D, int VD, hipStream_t stream) {
  if (n_items_bound <= 0 || p.nblk_total <= 0) return NSA_OK;
  const int KW = nsa_bwd_dkdv_slot_keys(2, p.block_size);
  const int grid_y = p.block_size <= 64 ? 1 : cdiv_i(p.block_size, 128);
  dim3 grid(p.nblk_total, grid_y, p.KH);
  if (KW == 64) slc_dkdv_reduce_kernel<64><<<grid, 256, 0, stream>>>(p, D, VD, n_items_bound, grid_y);
  else slc_dkdv_reduce_kernel<128><<<grid, 256, 0, stream>>>(p, D, VD, n_items_bound, grid_y);
  return nsa_check_launch("slc_dkdv_reduce_kernel");
}

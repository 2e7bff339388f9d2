// Selected-block attention forward: one wave per (query token, kv head); the MFMA M dimension is the group of
// (up to 16) q-heads that share the kv head, N is 16 keys, v_mfma_f32_16x16x32_bf16.
// Upstream: flash_nsa/ops/select_attn.py:21-108 (training), flash_nsa/inference/select_attn.py:21-100 (paged).
//
// K fragments are loaded straight from global memory into the A operand (the contraction index d is contiguous
// in a key row); V is staged row-major in a wave-private LDS region and read back through
// ds_read_b64_tr_b16, which delivers the key-contraction slices.  Keys are gathered by the per-token block
// list topk[kh, t, 0 .. min(top_n, t/block+1)).
#include "nsa_common.h"
#include "nsa_api_internal.h"

namespace {

template <int D, int VD, bool PAGED>
__global__ __launch_bounds__(256) void slc_fwd_kernel(NsaSlcParams p) {
  constexpr int VLD = VD + 8;
  __shared__ __attribute__((aligned(16))) bf16_t Vs_all[4 * 64 * VLD];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  bf16_t* Vs = Vs_all + wave * 64 * VLD;
  const int l16 = lane & 15;
  const int kq = lane >> 4;
  const int b = blockIdx.y;
  const int n_hc = (p.G + 15) / 16;
  const int kh = blockIdx.z / n_hc;
  const int hc = blockIdx.z - kh * n_hc;

  const int x0 = p.x_cu[b];
  const int xl = p.x_cu[b + 1] - x0;
  const int n = blockIdx.x * 4 + wave;
  if (n >= xl) return;
  const int ctx = PAGED ? p.ctx_lens[b] : xl;
  const int t = n + (ctx - xl);
  const int64_t tok = x0 + n;
  const int32_t* table = PAGED ? p.table + (int64_t)b * p.table_stride : nullptr;
  const int Bs = p.block_size;
  const int nvalid = min(p.top_n, t / Bs + 1);

  int g = hc * 16 + l16;
  const bool head_ok = g < p.G;
  if (!head_ok) g = p.G - 1;
  const int head = kh * p.G + g;

  bf16x8 qf[D / 32];
  {
    const bf16_t* qp = p.q + tok * p.q_st + (int64_t)head * p.q_sh + kq * 8;
#pragma unroll
    for (int kc = 0; kc < D / 32; kc++) qf[kc] = ld_global_b128(qp + kc * 32);
  }
  int my_blk = 0;
  if (lane < nvalid) my_blk = p.topk[(int64_t)kh * p.tk_sh + tok * p.tk_st + lane];

  f32x4 oacc[VD / 16];
#pragma unroll
  for (int dt = 0; dt < VD / 16; dt++) oacc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = NSA_NEG_INF, l_run = 0.f;
  const float sc = p.scale_log2;
  const int subs = Bs / 64;

  for (int slot = 0; slot < nvalid; slot++) {
    const int blk = __shfl(my_blk, slot, 64);
    for (int sub = 0; sub < subs; sub++) {
      const int key0 = blk * Bs + sub * 64;
      if (key0 > t || key0 < 0) continue;  // nothing visible (also guards ignore values)
      int64_t row0;
      if (PAGED) {
        int pg = table[key0 / p.page_size];
        row0 = (int64_t)pg * p.page_size + (key0 % p.page_size);
      } else {
        row0 = (int64_t)x0 + key0;
      }
      const int kmax = min(ctx - 1, t) - key0;  // last usable key offset inside this tile (>= 0)

      // ---- V tile -> registers (issued early), K fragments -> registers ----
      bf16x8 vreg[(64 * (VD / 8)) / 64];
#pragma unroll
      for (int j = 0; j < (VD / 8); j++) {
        int pc = lane + j * 64;
        int kr = pc / (VD / 8), dp = pc - kr * (VD / 8);
        int krc = min(kr, kmax);
        vreg[j] = ld_global_b128(p.v + (row0 + krc) * p.v_sr + (int64_t)kh * p.v_sh + dp * 8);
      }
      f32x4 sacc[4];
#pragma unroll
      for (int jt = 0; jt < 4; jt++) {
        sacc[jt] = f32x4{0.f, 0.f, 0.f, 0.f};
        int kr = min(jt * 16 + l16, kmax);
        const bf16_t* kp = p.k + (row0 + kr) * p.k_sr + (int64_t)kh * p.k_sh + kq * 8;
#pragma unroll
        for (int kc = 0; kc < D / 32; kc++) {
          bf16x8 kf = ld_global_b128(kp + kc * 32);
          sacc[jt] = mfma16(kf, qf[kc], sacc[jt]);
        }
      }
      // ---- softmax over this tile ----
      float tmax = NSA_NEG_INF;
#pragma unroll
      for (int jt = 0; jt < 4; jt++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
          int ko = jt * 16 + kq * 4 + i;
          float s = ko <= kmax ? sacc[jt][i] * sc : NSA_NEG_INF;
          sacc[jt][i] = s;
          tmax = fmaxf(tmax, s);
        }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      float m_new = fmaxf(m_run, tmax);  // finite: key0 <= t guarantees at least one visible key
      float alpha = fast_exp2(m_run - m_new);
      m_run = m_new;
      float psum = 0.f;
#pragma unroll
      for (int jt = 0; jt < 4; jt++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
          float pv = fast_exp2(sacc[jt][i] - m_new);
          sacc[jt][i] = pv;
          psum += pv;
        }
      l_run = l_run * alpha + psum;
#pragma unroll
      for (int dt = 0; dt < VD / 16; dt++) oacc[dt] *= alpha;

      // ---- V registers -> wave-private LDS ----
#pragma unroll
      for (int j = 0; j < (VD / 8); j++) {
        int pc = lane + j * 64;
        int kr = pc / (VD / 8), dp = pc - kr * (VD / 8);
        *reinterpret_cast<bf16x8*>(&Vs[kr * VLD + dp * 8]) = vreg[j];
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

      // ---- O^T += V^T P^T ----
#pragma unroll
      for (int c = 0; c < 2; c++) {
        bf16x8 pf = pack8(sacc[2 * c][0], sacc[2 * c][1], sacc[2 * c][2], sacc[2 * c][3], sacc[2 * c + 1][0],
                          sacc[2 * c + 1][1], sacc[2 * c + 1][2], sacc[2 * c + 1][3]);
        const int kb0 = (2 * c) * 16 + kq * 4 + (l16 >> 2);
        const int kb1 = kb0 + 16;
#pragma unroll
        for (int dt = 0; dt < VD / 16; dt++) {
          const int col = dt * 16 + 4 * (l16 & 3);
          bf16x4 v0 = lds_read_tr(&Vs[kb0 * VLD + col]);
          bf16x4 v1 = lds_read_tr(&Vs[kb1 * VLD + col]);
          oacc[dt] = mfma16(cat4(v0, v1), pf, oacc[dt]);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
  }

  float l_tot = l_run + __shfl_xor(l_run, 16, 64);
  l_tot += __shfl_xor(l_tot, 32, 64);
  if (!head_ok) return;
  float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  bf16_t* op = p.o + tok * p.o_st + (int64_t)head * p.o_sh + kq * 4;
#pragma unroll
  for (int dt = 0; dt < VD / 16; dt++) {
    bf16x4 w = pack4(oacc[dt][0] * inv, oacc[dt][1] * inv, oacc[dt][2] * inv, oacc[dt][3] * inv);
    *reinterpret_cast<bf16x4*>(op + dt * 16) = w;
  }
  if (kq == 0 && p.lse != nullptr) {
    p.lse[tok * p.lse_st + (int64_t)head * p.lse_sh] = l_tot > 0.f ? m_run + fast_log2(l_tot) : 0.f;
  }
}

template <int D, int VD, bool PAGED>
int launch_slc(const NsaSlcParams& p, int B, int max_q_len, hipStream_t stream) {
  if (B <= 0 || max_q_len <= 0) return NSA_OK;
  dim3 grid(cdiv_i(max_q_len, 4), B, p.KH * ((p.G + 15) / 16));
  slc_fwd_kernel<D, VD, PAGED><<<grid, 256, 0, stream>>>(p);
  return nsa_check_launch("slc_fwd_kernel");
}

template <bool PAGED>
int dispatch_slc(const NsaSlcParams& p, int B, int max_q_len, int D, int VD, hipStream_t stream) {
  if (D == 128 && VD == 128) return launch_slc<128, 128, PAGED>(p, B, max_q_len, stream);
  if (D == 64 && VD == 64) return launch_slc<64, 64, PAGED>(p, B, max_q_len, stream);
  if (D == 192 && VD == 128) return launch_slc<192, 128, PAGED>(p, B, max_q_len, stream);
  nsa_set_error("selected attention forward: unsupported head dims D=%d VD=%d", D, VD);
  return NSA_ERR_UNSUPPORTED;
}

}  // namespace

int nsa_slc_fwd_launch(const NsaSlcParams& p, bool paged, int B, int max_q_len, int D, int VD, hipStream_t stream) {
  return paged ? dispatch_slc<true>(p, B, max_q_len, D, VD, stream)
               : dispatch_slc<false>(p, B, max_q_len, D, VD, stream);
}

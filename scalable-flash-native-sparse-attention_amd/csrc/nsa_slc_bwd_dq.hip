// dQ of selected-block attention: one wave per (query token, kv head), 16 q-heads as the MFMA N dimension.
//   S^T = K Q^T,  P^T = exp2(S^T*c - lse),  dP^T = V dO^T,  dS^T = P^T o (dP^T - delta),  dQ^T += K^T dS^T
// K is staged row-major in a wave-private LDS region (read both as row fragments and, transposed, through
// ds_read_b64_tr_b16); V fragments are loaded straight from global memory.
// Upstream: flash_nsa/ops/select_attn.py:336-437 (_dq_kernel).
#include "nsa_common.h"
#include "nsa_api_internal.h"

namespace {

template <int D, int VD>
__global__ __launch_bounds__(256) void slc_dq_kernel(NsaSlcBwdDqParams p) {
  constexpr int KLD = D + NSA_LDS_PAD;
  __shared__ __attribute__((aligned(16))) bf16_t Ks_all[4 * 64 * KLD];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  bf16_t* Ks = Ks_all + wave * 64 * KLD;
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
  const int t = n;
  const int64_t tok = x0 + n;
  const int Bs = p.block_size;
  const int nvalid = min(p.top_n, t / Bs + 1);

  int g = hc * 16 + l16;
  const bool head_ok = g < p.G;
  if (!head_ok) g = p.G - 1;
  const int head = kh * p.G + g;

  bf16x8 qf[D / 32], dof[VD / 32];
  {
    const bf16_t* qp = p.q + tok * p.q_st + (int64_t)head * p.q_sh + kq * 8;
#pragma unroll
    for (int kc = 0; kc < D / 32; kc++) qf[kc] = ld_global_b128(qp + kc * 32);
    const bf16_t* dp = p.dO + tok * p.do_st + (int64_t)head * p.do_sh + kq * 8;
#pragma unroll
    for (int kc = 0; kc < VD / 32; kc++) dof[kc] = ld_global_b128(dp + kc * 32);
  }
  const float lse = p.lse[tok * p.lse_st + (int64_t)head * p.lse_sh];
  const float delta = p.delta[tok * p.delta_st + (int64_t)head * p.delta_sh];
  int my_blk = 0;
  if (lane < nvalid) my_blk = p.topk[(int64_t)kh * p.tk_sh + tok * p.tk_st + lane];

  f32x4 dqacc[D / 16];
#pragma unroll
  for (int dt = 0; dt < D / 16; dt++) dqacc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float sc = p.scale_log2;
  const int subs = Bs / 64;

  for (int slot = 0; slot < nvalid; slot++) {
    const int blk = __shfl(my_blk, slot, 64);
    for (int sub = 0; sub < subs; sub++) {
      const int key0 = blk * Bs + sub * 64;
      if (key0 > t || key0 < 0) continue;
      const int64_t row0 = (int64_t)x0 + key0;
      const int kmax = min(xl - 1, t) - key0;

      // K tile -> registers -> wave-private LDS
      bf16x8 kreg[D / 8];
#pragma unroll
      for (int j = 0; j < (D / 8); j++) {
        int pc = lane + j * 64;
        int kr = pc / (D / 8), dp = pc - kr * (D / 8);
        int krc = min(kr, kmax);
        kreg[j] = ld_global_b128(p.k + (row0 + krc) * p.k_sr + (int64_t)kh * p.k_sh + dp * 8);
      }
      // dP^T = V dO^T with V fragments from global
      f32x4 pacc[4];
#pragma unroll
      for (int jt = 0; jt < 4; jt++) {
        pacc[jt] = f32x4{0.f, 0.f, 0.f, 0.f};
        int kr = min(jt * 16 + l16, kmax);
        const bf16_t* vp = p.v + (row0 + kr) * p.v_sr + (int64_t)kh * p.v_sh + kq * 8;
#pragma unroll
        for (int kc = 0; kc < VD / 32; kc++) pacc[jt] = mfma16(ld_global_b128(vp + kc * 32), dof[kc], pacc[jt]);
      }
#pragma unroll
      for (int j = 0; j < (D / 8); j++) {
        int pc = lane + j * 64;
        int kr = pc / (D / 8), dp = pc - kr * (D / 8);
        *reinterpret_cast<bf16x8*>(&Ks[kr * KLD + dp * 8]) = kreg[j];
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

      f32x4 sacc[4];
#pragma unroll
      for (int jt = 0; jt < 4; jt++) {
        sacc[jt] = f32x4{0.f, 0.f, 0.f, 0.f};
        const bf16_t* kp = &Ks[(jt * 16 + l16) * KLD + kq * 8];
#pragma unroll
        for (int kc = 0; kc < D / 32; kc++)
          sacc[jt] = mfma16(*reinterpret_cast<const bf16x8*>(kp + kc * 32), qf[kc], sacc[jt]);
      }
#pragma unroll
      for (int jt = 0; jt < 4; jt++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
          int ko = jt * 16 + kq * 4 + i;
          float pv = ko <= kmax ? fast_exp2(sacc[jt][i] * sc - lse) : 0.f;
          sacc[jt][i] = pv * (pacc[jt][i] - delta);
        }
#pragma unroll
      for (int c = 0; c < 2; c++) {
        bf16x8 df = pack8(sacc[2 * c][0], sacc[2 * c][1], sacc[2 * c][2], sacc[2 * c][3], sacc[2 * c + 1][0],
                          sacc[2 * c + 1][1], sacc[2 * c + 1][2], sacc[2 * c + 1][3]);
        const int kb0 = (2 * c) * 16 + kq * 4 + (l16 >> 2);
        const int kb1 = kb0 + 16;
#pragma unroll
        for (int dt = 0; dt < D / 16; dt++) {
          const int col = dt * 16 + 4 * (l16 & 3);
          bf16x4 a0 = lds_read_tr(&Ks[kb0 * KLD + col]);
          bf16x4 a1 = lds_read_tr(&Ks[kb1 * KLD + col]);
          dqacc[dt] = mfma16(cat4(a0, a1), df, dqacc[dt]);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
  }

  if (!head_ok) return;
  const float osc = p.sm_scale;
  const int64_t off = tok * p.dq_st + (int64_t)head * p.dq_sh + kq * 4;
#pragma unroll
  for (int dt = 0; dt < D / 16; dt++) {
    f32x4 val = dqacc[dt] * osc;
    if (p.dq_mode == 0) {
      *reinterpret_cast<bf16x4*>((bf16_t*)p.dq + off + dt * 16) = pack4(val[0], val[1], val[2], val[3]);
    } else {
      float* dst = (float*)p.dq + off + dt * 16;
      if (p.dq_mode == 2) val += *reinterpret_cast<f32x4*>(dst);
      *reinterpret_cast<f32x4*>(dst) = val;
    }
  }
}

}  // namespace

int nsa_slc_bwd_dq_launch(const NsaSlcBwdDqParams& p, int B, int max_q_len, int D, int VD, hipStream_t stream) {
  if (B <= 0 || max_q_len <= 0) return NSA_OK;
  dim3 grid(cdiv_i(max_q_len, 4), B, p.KH * ((p.G + 15) / 16));
  if (D == 128 && VD == 128) slc_dq_kernel<128, 128><<<grid, 256, 0, stream>>>(p);
  else if (D == 64 && VD == 64) slc_dq_kernel<64, 64><<<grid, 256, 0, stream>>>(p);
  else if (D == 192 && VD == 128) slc_dq_kernel<192, 128><<<grid, 256, 0, stream>>>(p);
  else {
    nsa_set_error("selected attention dq: unsupported head dims D=%d VD=%d", D, VD);
    return NSA_ERR_UNSUPPORTED;
  }
  return nsa_check_launch("slc_dq_kernel");
}

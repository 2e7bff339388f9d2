// dQ of selected-block attention: one wave per (query token, kv head), 16 q-heads as the MFMA N dimension.
//   S^T = K Q^T,  P^T = exp2(S^T*c - lse),  dP^T = V dO^T,  dS^T = P^T o (dP^T - delta),  dQ^T += K^T dS^T
// K rows are staged row-major in a wave-private LDS region (K is read both as row fragments and, transposed,
// through ds_read_b64_tr_b16); V is only read as row fragments and comes from global memory in that layout.
// Upstream: flash_nsa/ops/select_attn.py:336-437 (_dq_kernel).
#include "nsa_common.h"
#include "nsa_api_internal.h"

namespace {

template <int D, int VD>
__global__ __launch_bounds__(256, 2) void slc_dq_kernel(NsaSlcBwdDqParams p) {
  // Work unit = 32 keys.  The K and V rows of unit u+1 are fetched (coalesced 16-byte-per-lane row loads) into
  // registers while unit u is computed out of wave-private LDS.
  constexpr int UK = 32;
  constexpr int KLD = D + NSA_LDS_PAD;
  constexpr int KC = D / 32, VC = VD / 32;
  constexpr int KJ = (UK * (D / 8)) / 64, VJ = 2 * VC;
  __shared__ __attribute__((aligned(16))) bf16_t Ks_all[4 * UK * KLD];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  bf16_t* Ks = Ks_all + wave * UK * KLD;
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
  const int upb = Bs / UK;
  const int nu = nvalid * upb;
  const int key_last = min(xl - 1, t);

  int g = hc * 16 + l16;
  const bool head_ok = g < p.G;
  if (!head_ok) g = p.G - 1;
  const int head = kh * p.G + g;

  bf16x8 qf[KC], dof[VC];
  {
    const bf16_t* qp = p.q + tok * p.q_st + (int64_t)head * p.q_sh + kq * 8;
#pragma unroll
    for (int kc = 0; kc < KC; kc++) qf[kc] = ld_global_b128(qp + kc * 32);
    const bf16_t* dp = p.dO + tok * p.do_st + (int64_t)head * p.do_sh + kq * 8;
#pragma unroll
    for (int kc = 0; kc < VC; kc++) dof[kc] = ld_global_b128(dp + kc * 32);
  }
  const float lse = p.lse[tok * p.lse_st + (int64_t)head * p.lse_sh];
  const float delta = p.delta[tok * p.delta_st + (int64_t)head * p.delta_sh];
  int my_blk = 0;
  if (lane < nvalid) my_blk = p.topk[(int64_t)kh * p.tk_sh + tok * p.tk_st + lane];

  f32x4 dqacc[D / 16];
#pragma unroll
  for (int dt = 0; dt < D / 16; dt++) dqacc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float sc = p.scale_log2;

  auto unit_key0 = [&](int u) {  // wave-uniform; -1: nothing to attend in this unit
    int slot = u / upb;
    int blk = __builtin_amdgcn_readlane(my_blk, slot);
    int key0 = blk * Bs + (u - slot * upb) * UK;
    return (blk < 0 || key0 > key_last) ? -1 : key0;
  };
  int64_t koff[KJ], voff[VJ];
#pragma unroll
  for (int j = 0; j < KJ; j++) {
    int pc = lane + j * 64;
    koff[j] = (int64_t)(pc / (D / 8)) * p.k_sr + (pc % (D / 8)) * 8;
  }
  // V is only needed as row fragments (dP^T = V dO^T): its rows are loaded straight in MFMA operand layout, lane
  // (l16, kq) taking 16 bytes of row jt*16 + l16 at column kq*8 + kc*32 (16 rows x 64 contiguous bytes per load)
#pragma unroll
  for (int j = 0; j < VJ; j++) voff[j] = (int64_t)((j / VC) * 16 + l16) * p.v_sr + kq * 8 + (j % VC) * 32;
  auto issue = [&](int key0, bf16x8 (&kr)[KJ], bf16x8 (&vr)[VJ]) {
    if (key0 < 0) return;
    const int64_t row0 = (int64_t)x0 + key0;
    const bf16_t* kb = p.k + row0 * p.k_sr + (int64_t)kh * p.k_sh;
    const bf16_t* vb = p.v + row0 * p.v_sr + (int64_t)kh * p.v_sh;
    const int kmax = key_last - key0;
    if (kmax >= UK - 1) {
#pragma unroll
      for (int j = 0; j < KJ; j++) kr[j] = ld_global_b128(kb + koff[j]);
#pragma unroll
      for (int j = 0; j < VJ; j++) vr[j] = ld_global_b128(vb + voff[j]);
    } else {  // causal boundary unit: rows past the boundary are replaced by the boundary row (masked later)
#pragma unroll
      for (int j = 0; j < KJ; j++) {
        int pc = lane + j * 64;
        kr[j] = ld_global_b128(kb + (int64_t)min(pc / (D / 8), kmax) * p.k_sr + (pc % (D / 8)) * 8);
      }
#pragma unroll
      for (int j = 0; j < VJ; j++)
        vr[j] = ld_global_b128(vb + (int64_t)min((j / VC) * 16 + l16, kmax) * p.v_sr + kq * 8 + (j % VC) * 32);
    }
  };
  auto compute = [&](int key0, bf16x8 (&kr)[KJ], bf16x8 (&vr)[VJ]) {
    if (key0 < 0) return;
#pragma unroll
    for (int j = 0; j < KJ; j++) {
      int pc = lane + j * 64;
      *reinterpret_cast<bf16x8*>(&Ks[(pc / (D / 8)) * KLD + (pc % (D / 8)) * 8]) = kr[j];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    f32x4 sacc[2], pacc[2];
#pragma unroll
    for (int jt = 0; jt < 2; jt++) {
      sacc[jt] = f32x4{0.f, 0.f, 0.f, 0.f};
      pacc[jt] = f32x4{0.f, 0.f, 0.f, 0.f};
      const bf16_t* kp = &Ks[(jt * 16 + l16) * KLD + kq * 8];
#pragma unroll
      for (int kc = 0; kc < KC; kc++)
        sacc[jt] = mfma16(*reinterpret_cast<const bf16x8*>(kp + kc * 32), qf[kc], sacc[jt]);
#pragma unroll
      for (int kc = 0; kc < VC; kc++) pacc[jt] = mfma16(vr[jt * VC + kc], dof[kc], pacc[jt]);
    }
    const int kmax = key_last - key0;
#pragma unroll
    for (int jt = 0; jt < 2; jt++)
#pragma unroll
      for (int i = 0; i < 4; i++) sacc[jt][i] = fast_exp2(__builtin_fmaf(sacc[jt][i], sc, -lse));
    if (kmax < UK - 1) {  // wave-uniform
#pragma unroll
      for (int jt = 0; jt < 2; jt++)
#pragma unroll
        for (int i = 0; i < 4; i++)
          if (jt * 16 + kq * 4 + i > kmax) sacc[jt][i] = 0.f;
    }
#pragma unroll
    for (int jt = 0; jt < 2; jt++)
#pragma unroll
      for (int i = 0; i < 4; i++) sacc[jt][i] *= (pacc[jt][i] - delta);
    bf16x8 df = pack8(sacc[0][0], sacc[0][1], sacc[0][2], sacc[0][3], sacc[1][0], sacc[1][1], sacc[1][2], sacc[1][3]);
    const int kb0 = kq * 4 + (l16 >> 2);
    const int kb1 = kb0 + 16;
#pragma unroll
    for (int dt = 0; dt < D / 16; dt++) {
      const int col = dt * 16 + 4 * (l16 & 3);
      bf16x4 a0 = lds_read_tr(&Ks[kb0 * KLD + col]);
      bf16x4 a1 = lds_read_tr(&Ks[kb1 * KLD + col]);
      dqacc[dt] = mfma16(cat4(a0, a1), df, dqacc[dt]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  };

  bf16x8 krA[KJ], krB[KJ], vrA[VJ], vrB[VJ];
  int keyA = 0, keyB = 0;
  if (nu > 0) { keyA = unit_key0(0); issue(keyA, krA, vrA); }
  for (int u = 0; u < nu; u += 2) {
    if (u + 1 < nu) { keyB = unit_key0(u + 1); issue(keyB, krB, vrB); }
    compute(keyA, krA, vrA);
    if (u + 1 < nu) {
      if (u + 2 < nu) { keyA = unit_key0(u + 2); issue(keyA, krA, vrA); }
      compute(keyB, krB, vrB);
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
  else if (D == 256 && VD == 256) slc_dq_kernel<256, 256><<<grid, 256, 0, stream>>>(p);
  else if (D == 32 && VD == 32) slc_dq_kernel<32, 32><<<grid, 256, 0, stream>>>(p);
  else {
    nsa_set_error("selected attention dq: unsupported head dims D=%d VD=%d", D, VD);
    return NSA_ERR_UNSUPPORTED;
  }
  return nsa_check_launch("slc_dq_kernel");
}

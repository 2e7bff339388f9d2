// dQ of the two range-keyed branches (compressed attention, sliding window): same row/lane ownership as the
// forward tile kernel.  Per key tile:  S^T = K Q^T,  P^T = exp2(S^T*c - lse),  dP^T = V dO^T,
// dS^T = P^T o (dP^T - delta),  dQ^T += K^T dS^T  (K^T fragments via ds_read_b64_tr_b16).
// Upstream: flash_nsa/ops/compress_attn.py:385-528 (_cmp_dq_kernel); the window branch upstream is
// FlashAttention's backward (flash_nsa/ops/sliding_window_attention.py:98-157).
#include "nsa_common.h"
#include "nsa_api_internal.h"

namespace {

constexpr int MODE_CMP = 0;
constexpr int MODE_SWA = 1;

template <int D, int VD, int MODE, int MINB, bool DO_LDS>
__global__ __launch_bounds__(256, MINB) void bwd_dq_tile_kernel(NsaBwdTileParams p) {
  constexpr int ROWS_W = 32;
  constexpr int ROWS_WG = 4 * ROWS_W;
  constexpr int KT = 64;
  constexpr int KLD = D + NSA_LDS_PAD;
  constexpr int VLD = VD + NSA_LDS_PAD;
  __shared__ __attribute__((aligned(16))) bf16_t Ks[KT * KLD];
  __shared__ __attribute__((aligned(16))) bf16_t Vs[KT * VLD];
  // with DO_LDS the dO fragments of a wave's 32 rows live in a wave-private LDS region instead of 32 registers,
  // which brings the kernel under 256 registers (two workgroups per CU)
  __shared__ __attribute__((aligned(16))) bf16_t dOs[DO_LDS ? 4 * 32 * VLD : 8];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int hl = lane >> 5;
  const int b = blockIdx.y;
  const int kh = blockIdx.z;
  const int G = p.G;

  const int x0 = p.x_cu[b];
  const int xl = p.x_cu[b + 1] - x0;
  const int rows_total = xl * G;
  const int r0 = blockIdx.x * ROWS_WG;
  if (r0 >= rows_total) return;
  int nkeys, kbase;
  if (MODE == MODE_CMP) {
    kbase = p.k_cu[b];
    nkeys = p.k_cu[b + 1] - kbase;
  } else {
    kbase = x0;
    nkeys = xl;
  }

  const int r = r0 + wave * ROWS_W + l32;
  const bool valid = r < rows_total;
  const int rr = valid ? r : rows_total - 1;
  const int n = rr / G;
  const int g = rr - n * G;
  const int t = n;
  const int64_t tok = x0 + n;
  const int head = kh * G + g;

  bf16x8 qf[D / 16], dof[DO_LDS ? 1 : VD / 16];
  {
    const bf16_t* qp = p.q + tok * p.q_st + (int64_t)head * p.q_sh + hl * 8;
#pragma unroll
    for (int kc = 0; kc < D / 16; kc++) qf[kc] = ld_global_b128(qp + kc * 16);
    const bf16_t* dp = p.dO + tok * p.do_st + (int64_t)head * p.do_sh + hl * 8;
#pragma unroll
    for (int kc = 0; kc < VD / 16; kc++) {
      bf16x8 t8 = ld_global_b128(dp + kc * 16);
      if (DO_LDS) *reinterpret_cast<bf16x8*>(&dOs[(wave * 32 + l32) * VLD + hl * 8 + kc * 16]) = t8;
      else dof[kc] = t8;
    }
  }
  const float lse = p.lse[tok * p.lse_st + (int64_t)head * p.lse_sh];
  const float delta = p.delta[tok * p.delta_st + (int64_t)head * p.delta_sh];

  const int rw_lo = r0 + wave * ROWS_W;
  const int rw_hi = min(rw_lo + ROWS_W - 1, rows_total - 1);
  const bool wave_active = rw_lo < rows_total;
  const int tw_lo = wave_active ? rw_lo / G : 0;
  const int tw_hi = wave_active ? rw_hi / G : 0;
  const int t_lo = r0 / G;
  const int t_hi = min(r0 + ROWS_WG - 1, rows_total - 1) / G;

  int key_begin, key_end;
  if (MODE == MODE_CMP) {
    key_begin = 0;
    key_end = t_hi >= p.kernel_size - 1 ? min((t_hi - p.kernel_size + 1) / p.stride + 1, nkeys) : 0;
  } else {
    key_begin = (max(0, t_lo - p.window) / KT) * KT;
    key_end = min(t_hi + 1, nkeys);
  }

  f32x16 dqacc[D / 32];
#pragma unroll
  for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
    for (int i = 0; i < 16; i++) dqacc[dt][i] = 0.f;
  const float sc = p.scale_log2;
  const int g16 = lane >> 4, i16 = lane & 15;

  // software pipeline: next tile's global loads fly while the current tile is computed; rows past the end of
  // the key range are replaced by the last valid row (their probabilities are masked to zero)
  constexpr int KP = D / 8, VP = VD / 8;
  constexpr int KJ = (KT * KP) / 256, VJ = (KT * VP) / 256;
  bf16x8 kreg[KJ], vreg[VJ];
  auto gload = [&](int kt) {
    const int last = key_end - 1 - kt;
#pragma unroll
    for (int j = 0; j < KJ; j++) {
      int pc = tid + j * 256;
      int kr = min(pc / KP, last), dp = pc % KP;
      kreg[j] = ld_global_b128(p.k + ((int64_t)kbase + kt + kr) * p.k_sr + (int64_t)kh * p.k_sh + dp * 8);
    }
#pragma unroll
    for (int j = 0; j < VJ; j++) {
      int pc = tid + j * 256;
      int kr = min(pc / VP, last), dp = pc % VP;
      vreg[j] = ld_global_b128(p.v + ((int64_t)kbase + kt + kr) * p.v_sr + (int64_t)kh * p.v_sh + dp * 8);
    }
  };
  if (key_begin < key_end) gload(key_begin);

  for (int kt = key_begin; kt < key_end; kt += KT) {
    __syncthreads();
#pragma unroll
    for (int j = 0; j < KJ; j++) {
      int pc = tid + j * 256;
      *reinterpret_cast<bf16x8*>(&Ks[(pc / KP) * KLD + (pc % KP) * 8]) = kreg[j];
    }
#pragma unroll
    for (int j = 0; j < VJ; j++) {
      int pc = tid + j * 256;
      *reinterpret_cast<bf16x8*>(&Vs[(pc / VP) * VLD + (pc % VP) * 8]) = vreg[j];
    }
    __syncthreads();
    if (kt + KT < key_end) gload(kt + KT);
    if (!wave_active) continue;
    bool any_vis, full_vis;
    if (MODE == MODE_CMP) {
      any_vis = tw_hi >= p.stride * kt + p.kernel_size - 1;
      full_vis = (tw_lo >= p.stride * (kt + KT - 1) + p.kernel_size - 1) && (kt + KT <= nkeys);
    } else {
      any_vis = (kt <= tw_hi) && (kt + KT - 1 >= tw_lo - p.window);
      full_vis = (kt + KT - 1 <= tw_lo) && (kt >= tw_hi - p.window);
    }
    if (!any_vis) continue;

    f32x16 sacc[2], pacc[2];
#pragma unroll
    for (int i = 0; i < 16; i++) { sacc[0][i] = 0.f; sacc[1][i] = 0.f; pacc[0][i] = 0.f; pacc[1][i] = 0.f; }
    {
      const bf16_t* kp0 = &Ks[l32 * KLD + hl * 8];
      const bf16_t* kp1 = kp0 + 32 * KLD;
#pragma unroll
      for (int kc = 0; kc < D / 16; kc++) {
        sacc[0] = mfma32(*reinterpret_cast<const bf16x8*>(kp0 + kc * 16), qf[kc], sacc[0]);
        sacc[1] = mfma32(*reinterpret_cast<const bf16x8*>(kp1 + kc * 16), qf[kc], sacc[1]);
      }
      const bf16_t* vp0 = &Vs[l32 * VLD + hl * 8];
      const bf16_t* vp1 = vp0 + 32 * VLD;
#pragma unroll
      for (int kc = 0; kc < VD / 16; kc++) {
        bf16x8 df = DO_LDS ? *reinterpret_cast<const bf16x8*>(&dOs[(wave * 32 + l32) * VLD + hl * 8 + kc * 16]) : dof[kc];
        pacc[0] = mfma32(*reinterpret_cast<const bf16x8*>(vp0 + kc * 16), df, pacc[0]);
        pacc[1] = mfma32(*reinterpret_cast<const bf16x8*>(vp1 + kc * 16), df, pacc[1]);
      }
    }
    const float lsc = lse;
#pragma unroll
    for (int nt = 0; nt < 2; nt++)
#pragma unroll
      for (int i = 0; i < 16; i++) sacc[nt][i] = fast_exp2(__builtin_fmaf(sacc[nt][i], sc, -lsc));
    if (!full_vis) {  // wave-uniform
#pragma unroll
      for (int nt = 0; nt < 2; nt++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          int key = kt + nt * 32 + (i >> 2) * 8 + hl * 4 + (i & 3);
          bool vis;
          if (MODE == MODE_CMP) vis = (key < nkeys) && (t >= p.stride * key + p.kernel_size - 1);
          else vis = (key <= t) && (key >= t - p.window);
          sacc[nt][i] = vis ? sacc[nt][i] : 0.f;
        }
    }
#pragma unroll
    for (int nt = 0; nt < 2; nt++)
#pragma unroll
      for (int i = 0; i < 16; i++) sacc[nt][i] *= (pacc[nt][i] - delta);  // dS^T (without the softmax scale)
#pragma unroll
    for (int c = 0; c < 4; c++) {
      const int nt = c >> 1, ch = c & 1;
      bf16x8 df = pack8(sacc[nt][ch * 8 + 0], sacc[nt][ch * 8 + 1], sacc[nt][ch * 8 + 2], sacc[nt][ch * 8 + 3],
                        sacc[nt][ch * 8 + 4], sacc[nt][ch * 8 + 5], sacc[nt][ch * 8 + 6], sacc[nt][ch * 8 + 7]);
      const int kb0 = nt * 32 + (2 * ch) * 8 + hl * 4;
      const int kb1 = kb0 + 8;
#pragma unroll
      for (int dt = 0; dt < D / 32; dt++) {
        const int col = dt * 32 + (g16 & 1) * 16 + 4 * (i16 & 3);
        bf16x4 a0 = lds_read_tr(&Ks[(kb0 + (i16 >> 2)) * KLD + col]);
        bf16x4 a1 = lds_read_tr(&Ks[(kb1 + (i16 >> 2)) * KLD + col]);
        dqacc[dt] = mfma32(cat4(a0, a1), df, dqacc[dt]);
      }
    }
  }

  if (!valid) return;
  const float osc = p.sm_scale;
  const int64_t off = tok * p.dq_st + (int64_t)head * p.dq_sh;
#pragma unroll
  for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
    for (int i4 = 0; i4 < 4; i4++) {
      int d = dt * 32 + i4 * 8 + hl * 4;
      f32x4 val = {dqacc[dt][i4 * 4 + 0] * osc, dqacc[dt][i4 * 4 + 1] * osc, dqacc[dt][i4 * 4 + 2] * osc,
                   dqacc[dt][i4 * 4 + 3] * osc};
      if (p.dq_mode == 0) {
        *reinterpret_cast<bf16x4*>((bf16_t*)p.dq + off + d) = pack4(val[0], val[1], val[2], val[3]);
      } else if (p.dq_mode == 3) {
        val += *reinterpret_cast<const f32x4*>(p.dq_partial + tok * p.dqp_st + (int64_t)head * p.dqp_sh + d);
        *reinterpret_cast<bf16x4*>((bf16_t*)p.dq + off + d) = pack4(val[0], val[1], val[2], val[3]);
      } else {
        float* dst = (float*)p.dq + off + d;
        if (p.dq_mode == 2) val += *reinterpret_cast<f32x4*>(dst);
        *reinterpret_cast<f32x4*>(dst) = val;
      }
    }
}

template <int MODE>
int dispatch(const NsaBwdTileParams& p, int B, int max_q_len, int D, int VD, hipStream_t stream) {
  if (B <= 0 || max_q_len <= 0) return NSA_OK;
  dim3 grid(cdiv_i(max_q_len * p.G, 128), B, p.KH);
  const int minb = nsa_tuning_knob("dq_min_blocks", 2);
  if (D == 128 && VD == 128) {
    if (minb == 2) bwd_dq_tile_kernel<128, 128, MODE, 2, true><<<grid, 256, 0, stream>>>(p);
    else bwd_dq_tile_kernel<128, 128, MODE, 1, false><<<grid, 256, 0, stream>>>(p);
  } else if (D == 64 && VD == 64) bwd_dq_tile_kernel<64, 64, MODE, 2, false><<<grid, 256, 0, stream>>>(p);
  else if (D == 192 && VD == 128) bwd_dq_tile_kernel<192, 128, MODE, 1, false><<<grid, 256, 0, stream>>>(p);
  else if (D == 256 && VD == 256) bwd_dq_tile_kernel<256, 256, MODE, 1, false><<<grid, 256, 0, stream>>>(p);
  else if (D == 32 && VD == 32) bwd_dq_tile_kernel<32, 32, MODE, 2, false><<<grid, 256, 0, stream>>>(p);
  else {
    nsa_set_error("attention dq: unsupported head dims D=%d VD=%d", D, VD);
    return NSA_ERR_UNSUPPORTED;
  }
  return nsa_check_launch("bwd_dq_tile_kernel");
}

}  // namespace

int nsa_bwd_dq_tile_launch(const NsaBwdTileParams& p, int mode, int B, int max_q_len, int D, int VD,
                           hipStream_t stream) {
  return mode == MODE_CMP ? dispatch<MODE_CMP>(p, B, max_q_len, D, VD, stream)
                          : dispatch<MODE_SWA>(p, B, max_q_len, D, VD, stream);
}

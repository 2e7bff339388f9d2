// Selected-block attention forward: one wave per (query token, kv head); the MFMA M dimension is the group of
// (up to 16) q-heads that share the kv head, N is 16 keys, v_mfma_f32_16x16x32_bf16.
// Upstream: flash_nsa/ops/select_attn.py:21-108 (training), flash_nsa/inference/select_attn.py:21-100 (paged).
//
// The keys of the selected blocks are processed in units of 32.  The K and V rows of a unit are fetched as whole
// coalesced rows (16 lanes x 16 bytes per row) into registers one unit ahead, pass through wave-private LDS
// regions, and are read back as MFMA fragments (K row-major, V through ds_read_b64_tr_b16, which delivers the
// key-contraction slices).  Keys are gathered by the per-token block list topk[kh, t, 0 .. min(top_n, t/block+1)).
#include "nsa_common.h"
#include "nsa_api_internal.h"

namespace {

template <int D, int VD, bool PAGED>
__global__ __launch_bounds__(256, 2) void slc_fwd_kernel(NsaSlcParams p) {
  // Work unit = 32 keys (half of a 64-key tile).  The K fragments and the V rows of unit u+1 are loaded into
  // registers while unit u is computed, so the gather latency overlaps the MFMAs of the previous unit.
  constexpr int VLD = VD + NSA_LDS_PAD;
  constexpr int UK = 32;                      // keys per unit
  constexpr int KC = D / 32;                  // K fragments per 16-key tile
  constexpr int VJ = (UK * (VD / 8)) / 64;    // 16-byte V loads per lane and unit
  constexpr int KJ = (UK * (D / 8)) / 64;     // 16-byte K loads per lane and unit
  constexpr int KLD = D + NSA_LDS_PAD;
  __shared__ __attribute__((aligned(16))) bf16_t Vs_all[4 * UK * VLD];
  __shared__ __attribute__((aligned(16))) bf16_t Ks_all[4 * UK * KLD];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  bf16_t* Vs = Vs_all + wave * UK * VLD;
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
  const int ctx = PAGED ? p.ctx_lens[b] : xl;
  const int t = n + (ctx - xl);
  const int64_t tok = x0 + n;
  const int32_t* table = PAGED ? p.table + (int64_t)b * p.table_stride : nullptr;
  const int Bs = p.block_size;
  const int nvalid = t >= 0 ? min(p.top_n, t / Bs + 1) : 0;  // t < 0: padded request, output row = 0
  const int upb = Bs / UK;                    // units per selection block
  const int nu = nvalid * upb;
  const int key_last = min(ctx - 1, t);       // last key this token may attend

  int g = hc * 16 + l16;
  const bool head_ok = g < p.G;
  if (!head_ok) g = p.G - 1;
  const int head = kh * p.G + g;

  bf16x8 qf[KC];
  {
    const bf16_t* qp = p.q + tok * p.q_st + (int64_t)head * p.q_sh + kq * 8;
#pragma unroll
    for (int kc = 0; kc < KC; kc++) qf[kc] = ld_global_b128(qp + kc * 32);
  }
  int my_blk = 0;
  if (lane < nvalid) my_blk = p.topk[(int64_t)kh * p.tk_sh + tok * p.tk_st + lane];

  f32x4 oacc[VD / 16];
#pragma unroll
  for (int dt = 0; dt < VD / 16; dt++) oacc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = NSA_NEG_INF, l_run = 0.f;
  const float sc = p.scale_log2;

  // first key of unit u; wave-uniform.  Units that start past the last attendable key (second half of the current
  // block) and ignore values (negative ids) are reported as -1 and skipped.
  auto unit_key0 = [&](int u) {
    int slot = u / upb;
    int blk = __builtin_amdgcn_readlane(my_blk, slot);
    int key0 = blk * Bs + (u - slot * upb) * UK;
    return (blk < 0 || key0 > key_last) ? -1 : key0;
  };
  // per-lane element offsets inside a unit are the same for every unit: the loads are (uniform base) + offset
  // K and V rows are fetched as whole 16-byte-per-lane coalesced rows (every cache line is requested once and used
  // completely) and go through wave-private LDS; the MFMA fragments are read from there
  int64_t koff[KJ], voff[VJ];
#pragma unroll
  for (int j = 0; j < KJ; j++) {
    int pc = lane + j * 64;
    koff[j] = (int64_t)(pc / (D / 8)) * p.k_sr + (pc % (D / 8)) * 8;
  }
#pragma unroll
  for (int j = 0; j < VJ; j++) {
    int pc = lane + j * 64;
    voff[j] = (int64_t)(pc / (VD / 8)) * p.v_sr + (pc % (VD / 8)) * 8;
  }
  auto issue = [&](int key0, bf16x8 (&kf)[KJ], bf16x8 (&vr)[VJ]) {
    if (key0 < 0) return;
    int64_t row0;  // flat row of the unit's first key (a unit never straddles a page)
    if (PAGED) row0 = (int64_t)__builtin_amdgcn_readfirstlane(table[key0 / p.page_size]) * p.page_size + (key0 % p.page_size);
    else row0 = (int64_t)x0 + key0;
    const bf16_t* kb = p.k + row0 * p.k_sr + (int64_t)kh * p.k_sh;
    const bf16_t* vb = p.v + row0 * p.v_sr + (int64_t)kh * p.v_sh;
    const int kmax = key_last - key0;  // >= 0
    if (kmax >= UK - 1) {
#pragma unroll
      for (int j = 0; j < KJ; j++) kf[j] = ld_global_b128(kb + koff[j]);
#pragma unroll
      for (int j = 0; j < VJ; j++) vr[j] = ld_global_b128(vb + voff[j]);
    } else {  // the unit holding the causal boundary: rows past it are replaced by the boundary row (masked later)
#pragma unroll
      for (int j = 0; j < KJ; j++) {
        int pc = lane + j * 64;
        kf[j] = ld_global_b128(kb + (int64_t)min(pc / (D / 8), kmax) * p.k_sr + (pc % (D / 8)) * 8);
      }
#pragma unroll
      for (int j = 0; j < VJ; j++) {
        int pc = lane + j * 64;
        vr[j] = ld_global_b128(vb + (int64_t)min(pc / (VD / 8), kmax) * p.v_sr + (pc % (VD / 8)) * 8);
      }
    }
  };
  auto compute = [&](int key0, bf16x8 (&kf)[KJ], bf16x8 (&vr)[VJ]) {
    if (key0 < 0) return;
#pragma unroll
    for (int j = 0; j < KJ; j++) {
      int pc = lane + j * 64;
      *reinterpret_cast<bf16x8*>(&Ks[(pc / (D / 8)) * KLD + (pc % (D / 8)) * 8]) = kf[j];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    f32x4 sacc[2];
#pragma unroll
    for (int jt = 0; jt < 2; jt++) {
      sacc[jt] = f32x4{0.f, 0.f, 0.f, 0.f};
      const bf16_t* kp = &Ks[(jt * 16 + l16) * KLD + kq * 8];
#pragma unroll
      for (int kc = 0; kc < KC; kc++) sacc[jt] = mfma16(*reinterpret_cast<const bf16x8*>(kp + kc * 32), qf[kc], sacc[jt]);
    }
    // V rows -> wave-private LDS (previous unit's transpose reads are complete: LDS ops of a wave are in order)
#pragma unroll
    for (int j = 0; j < VJ; j++) {
      int pc = lane + j * 64;
      *reinterpret_cast<bf16x8*>(&Vs[(pc / (VD / 8)) * VLD + (pc % (VD / 8)) * 8]) = vr[j];
    }
    const int kmax = key_last - key0;  // last usable key offset inside this unit
    if (kmax < UK - 1) {               // wave-uniform: only the unit holding the causal boundary is masked
#pragma unroll
      for (int jt = 0; jt < 2; jt++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
          int ko = jt * 16 + kq * 4 + i;
          if (ko > kmax) sacc[jt][i] = NSA_NEG_INF;
        }
    }
    float tmax = fmaxf(fmaxf(fmaxf(sacc[0][0], sacc[0][1]), fmaxf(sacc[0][2], sacc[0][3])),
                       fmaxf(fmaxf(sacc[1][0], sacc[1][1]), fmaxf(sacc[1][2], sacc[1][3])));
    tmax = xrow_max(tmax);
    tmax = xhalf_max(tmax);
    const float m_old = m_run;
    const float m_new = fmaxf(m_old, tmax);
    const float m_safe = (m_new == NSA_NEG_INF) ? 0.f : m_new;
    const float msc = m_safe * sc;
    m_run = m_new;
    float psum = 0.f;
#pragma unroll
    for (int jt = 0; jt < 2; jt++)
#pragma unroll
      for (int i = 0; i < 4; i++) {
        float pv = fast_exp2(__builtin_fmaf(sacc[jt][i], sc, -msc));
        sacc[jt][i] = pv;
        psum += pv;
      }
    if (__builtin_amdgcn_ballot_w64(m_new != m_old) != 0) {
      const float alpha = fast_exp2((m_old - m_safe) * sc);
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < VD / 16; dt++) oacc[dt] *= alpha;
    }
    l_run += psum;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // O^T += V^T P^T over the 32 keys of the unit
    bf16x8 pf = pack8(sacc[0][0], sacc[0][1], sacc[0][2], sacc[0][3], sacc[1][0], sacc[1][1], sacc[1][2], sacc[1][3]);
    const int kb0 = kq * 4 + (l16 >> 2);
    const int kb1 = kb0 + 16;
#pragma unroll
    for (int dt = 0; dt < VD / 16; dt++) {
      const int col = dt * 16 + 4 * (l16 & 3);
      bf16x4 v0 = lds_read_tr(&Vs[kb0 * VLD + col]);
      bf16x4 v1 = lds_read_tr(&Vs[kb1 * VLD + col]);
      oacc[dt] = mfma16(cat4(v0, v1), pf, oacc[dt]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  };

  bf16x8 kfA[KJ], kfB[KJ], vrA[VJ], vrB[VJ];
  int keyA = 0, keyB = 0;
  if (nu > 0) { keyA = unit_key0(0); issue(keyA, kfA, vrA); }
  for (int u = 0; u < nu; u += 2) {
    if (u + 1 < nu) { keyB = unit_key0(u + 1); issue(keyB, kfB, vrB); }
    compute(keyA, kfA, vrA);
    if (u + 1 < nu) {
      if (u + 2 < nu) { keyA = unit_key0(u + 2); issue(keyA, kfA, vrA); }
      compute(keyB, kfB, vrB);
    }
  }

  float l_tot = xrow_sum(l_run);
  l_tot = xhalf_sum(l_tot);
  if (!head_ok) return;
  float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  bf16_t* op = p.o + tok * p.o_st + (int64_t)head * p.o_sh + kq * 4;
#pragma unroll
  for (int dt = 0; dt < VD / 16; dt++) {
    bf16x4 w = pack4(oacc[dt][0] * inv, oacc[dt][1] * inv, oacc[dt][2] * inv, oacc[dt][3] * inv);
    *reinterpret_cast<bf16x4*>(op + dt * 16) = w;
  }
  if (kq == 0 && p.lse != nullptr) {
    p.lse[tok * p.lse_st + (int64_t)head * p.lse_sh] = l_tot > 0.f ? m_run * sc + fast_log2(l_tot) : 0.f;
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
  if (D == 256 && VD == 256) return launch_slc<256, 256, PAGED>(p, B, max_q_len, stream);
  if (D == 32 && VD == 32) return launch_slc<32, 32, PAGED>(p, B, max_q_len, stream);
  nsa_set_error("selected attention forward: unsupported head dims D=%d VD=%d", D, VD);
  return NSA_ERR_UNSUPPORTED;
}

}  // namespace

int nsa_slc_fwd_launch(const NsaSlcParams& p, bool paged, int B, int max_q_len, int D, int VD, hipStream_t stream) {
  return paged ? dispatch_slc<true>(p, B, max_q_len, D, VD, stream)
               : dispatch_slc<false>(p, B, max_q_len, D, VD, stream);
}

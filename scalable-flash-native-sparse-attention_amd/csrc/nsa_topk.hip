// Block-importance scoring fused with the top-n block selector.
// Upstream: flash_nsa/ops/topk.py:18-218 (general two-kernel path), :226-425 (32/16/64 fast path),
//           flash_nsa/inference/topk.py:17-182 (paged prefill; the device path masks causality per row).
//
// For a tile of query tokens of one kv-head group the kernel recomputes the compressed-attention
// probabilities p = exp2(q.ck*scale*log2e - lse) with v_mfma_f32_32x32x16_bf16 (S = Q CK^T, so that a lane
// holds 16 q-rows of one compressed key and the sum over the G heads of a token is an in-register reduction),
// folds them into per-token selection-block scores held in LDS (overlap weights area/stride, added in
// ascending compressed-key order), and then picks blocks: forced initial and local blocks first, then repeated
// arg-max (lowest index on ties) -- only the int32 indices leave the CU (plus the fp32 scores on request).
#include "nsa_common.h"
#include "nsa_api_internal.h"

namespace {

template <int GP>
struct SlotMap {
  static constexpr int NSLOT = GP >= 8 ? 32 / GP : 16 / GP;
  static constexpr bool CROSS = GP >= 8;
  NSA_DEVICE static constexpr int slot_of(int i) { return GP >= 8 ? i / (GP / 2) : i / GP; }
  // token (local to the wave) of a slot for lane-half hl
  NSA_DEVICE static int token_of(int slot, int hl) {
    if (GP >= 8) return slot;
    int i = slot * GP;
    int row = (i >> 2) * 8 + hl * 4 + (i & 3);
    return row / GP;
  }
};

template <int D, int GP, bool PAGED>
__global__ __launch_bounds__(256) void topk_kernel(NsaTopkParams p) {
  constexpr int KT = 64;
  constexpr int KLD = D + NSA_LDS_PAD;
  constexpr int TPW = 32 / GP;  // tokens per wave
  constexpr int TWG = 4 * TPW;  // tokens per workgroup
  constexpr int PLD = KT + 1;
  using SM = SlotMap<GP>;
  __shared__ __attribute__((aligned(16))) bf16_t Ks[KT * KLD];
  __shared__ float Pst[4 * TPW * PLD];
  extern __shared__ float imp_all[];  // [TWG][nb_max]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int hl = lane >> 5;
  const int b = blockIdx.y;
  const int kh = blockIdx.z;
  const int G = p.G;
  const int n_hc = (G + 31) / 32;

  const int x0 = p.x_cu[b];
  const int xl = p.x_cu[b + 1] - x0;
  const int n0 = blockIdx.x * TWG;
  if (n0 >= xl) return;
  const int ctx = PAGED ? p.ctx_lens[b] : xl;
  const int qoff = ctx - xl;
  const int nkeys = ctx >= p.kernel_size ? (ctx - p.kernel_size) / p.stride + 1 : 0;
  const int kbase = PAGED ? 0 : p.y_cu[b];
  const int32_t* table = PAGED ? p.table + (int64_t)b * p.table_stride : nullptr;
  const int nb_max = p.nb_max;
  const int Bs = p.block_size, Kz = p.kernel_size, St = p.stride;

  float* imp_w = imp_all + (wave * TPW) * nb_max;  // this wave's token rows
  for (int i = lane; i < TPW * nb_max; i += 64) imp_w[i] = 0.f;
  float* pst_w = Pst + wave * TPW * PLD;

  // A-operand row of this lane
  const int tokl_a = l32 / GP;
  const int nw0 = n0 + wave * TPW;
  const int n_a = min(nw0 + tokl_a, xl - 1);
  const int t_hi_wg = min(n0 + TWG - 1, xl - 1) + qoff;
  const int key_end = t_hi_wg >= Kz - 1 ? min((t_hi_wg - Kz + 1) / St + 1, nkeys) : 0;
  const int tw_hi = min(nw0 + TPW - 1, xl - 1) + qoff;
  const bool wave_active = nw0 < xl;

  // per-lane C-layout rows: lse and positions
  float lse_r[16];
  int t_r[16];
  bf16x8 qf[D / 16];

  auto load_rows = [&](int hc) {
    int g = hc * 32 + (l32 % GP);
    if (g >= G) g = G - 1;
    const bf16_t* qp = p.q + (int64_t)(x0 + n_a) * p.q_st + (int64_t)(kh * G + g) * p.q_sh + hl * 8;
#pragma unroll
    for (int kc = 0; kc < D / 16; kc++) qf[kc] = ld_global_b128(qp + kc * 16);
#pragma unroll
    for (int i = 0; i < 16; i++) {
      int row = (i >> 2) * 8 + hl * 4 + (i & 3);
      int gg = hc * 32 + (row % GP);
      int nn = nw0 + row / GP;
      bool ok = (gg < G) && (nn < xl);
      t_r[i] = ok ? nn + qoff : -1;  // -1: nothing visible
      lse_r[i] = ok ? p.lse[(int64_t)(x0 + nn) * p.lse_st + (int64_t)(kh * G + gg) * p.lse_sh] : 0.f;
    }
  };
  if (n_hc == 1) load_rows(0);

  for (int kt = 0; kt < key_end; kt += KT) {
    __syncthreads();
    {
      int64_t page_row0 = 0;
      if (PAGED) {
        int pg = table[kt / p.page_size];
        page_row0 = (int64_t)pg * p.page_size + (kt % p.page_size);
      }
      constexpr int KP = D / 8;
#pragma unroll
      for (int j = 0; j < (KT * KP) / 256; j++) {
        int pc = tid + j * 256;
        int kr = pc / KP, dp = pc - kr * KP;
        bf16x8 val = zero_bf16x8();
        if (kt + kr < key_end) {
          int64_t row = PAGED ? page_row0 + kr : (int64_t)kbase + kt + kr;
          val = ld_global_b128(p.ck + row * p.ck_sr + (int64_t)kh * p.ck_sh + dp * 8);
        }
        *reinterpret_cast<bf16x8*>(&Ks[kr * KLD + dp * 8]) = val;
      }
    }
    __syncthreads();
    if (!wave_active) continue;
    if (tw_hi < St * kt + Kz - 1) continue;  // tile invisible to every token of this wave

    for (int hc = 0; hc < n_hc; hc++) {
      if (n_hc > 1) load_rows(hc);
#pragma unroll
      for (int nt = 0; nt < 2; nt++) {
        f32x16 sacc;
#pragma unroll
        for (int i = 0; i < 16; i++) sacc[i] = 0.f;
        const bf16_t* kp = &Ks[(nt * 32 + l32) * KLD + hl * 8];
#pragma unroll
        for (int kc = 0; kc < D / 16; kc++) {
          bf16x8 kf = *reinterpret_cast<const bf16x8*>(kp + kc * 16);
          sacc = mfma32(qf[kc], kf, sacc);
        }
        const int key = kt + nt * 32 + l32;
        const int vis_from = St * key + Kz - 1;  // first position that sees this key
        float ps[SM::NSLOT];
#pragma unroll
        for (int s = 0; s < SM::NSLOT; s++) ps[s] = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
          bool vis = (key < nkeys) && (t_r[i] >= vis_from);
          float pv = vis ? fast_exp2(sacc[i] * p.scale_log2 - lse_r[i]) : 0.f;
          ps[SM::slot_of(i)] += pv;
        }
#pragma unroll
        for (int s = 0; s < SM::NSLOT; s++) {
          float v = ps[s];
          if (SM::CROSS) v += __shfl_xor(v, 32, 64);
          if (!SM::CROSS || hl == 0) {
            int tk = SM::token_of(s, hl);
            float* dst = &pst_w[tk * PLD + nt * 32 + l32];
            *dst = (hc == 0) ? v : *dst + v;
          }
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // ---- fold the 64 compressed keys of this tile into selection-block scores ----
    {
      const int nloops = (Bs + Kz - St) / St;
      const int j_lo = (St * kt) / Bs;
      const int j_hi = min((St * (kt + KT - 1) + Kz - 1) / Bs, nb_max - 1);
      const int nj = j_hi - j_lo + 1;
      for (int it = lane; it < TPW * nj; it += 64) {
        int tk = it / nj;
        int j = j_lo + (it - tk * nj);
        int i0 = (j * Bs - Kz) / St + 1;  // exact: block and kernel sizes are multiples of the stride
        float acc = imp_w[tk * nb_max + j];
        int cs = St - Kz;
        for (int r = 0; r < nloops; r++, cs += St) {
          int i = i0 + r;
          if (i >= kt && i < kt + KT) {
            int area = min(cs + Kz, Bs) - max(cs, 0);
            acc += pst_w[tk * PLD + (i - kt)] * ((float)area / (float)St);
          }
        }
        imp_w[tk * nb_max + j] = acc;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  if (!wave_active) return;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

  // ---- selection, one token at a time ----
  for (int tk = 0; tk < TPW; tk++) {
    const int n = nw0 + tk;
    if (n >= xl) break;
    const int t = n + qoff;
    const int nk = t / Bs;
    float* imp = imp_w + tk * nb_max;
    const int64_t tok = x0 + n;
    if (p.imp_out != nullptr) {
      for (int j = lane; j < p.imp_cols; j += 64)
        p.imp_out[(int64_t)kh * p.imp_sh + tok * p.imp_st + j] = j < nb_max ? imp[j] : 0.f;
    }
    int result = p.ignore_index;
    __builtin_amdgcn_wave_barrier();
    if (lane == 0) {
      for (int s = 0; s < p.num_init; s++)
        if (s < nb_max) imp[s] = -1.f;
      for (int i = 0; i < p.num_local; i++)
        if (nk - i >= 0 && nk - i < nb_max) imp[nk - i] = -1.f;
    }
    if (lane < p.num_init) {
      if (lane <= nk) result = lane;
    } else if (lane < p.num_init + p.num_local) {
      if (lane <= nk) result = nk - (lane - p.num_init);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int nsel = min(p.top_n, nk + 1);
    const int jmax = min(nk, nb_max - 1);
    for (int slot = p.num_init + p.num_local; slot < nsel; slot++) {
      float best = -2.f;
      int bj = 0x7fffffff;
      for (int j = lane; j <= jmax; j += 64) {
        float v = imp[j];
        if (v > best) { best = v; bj = j; }
      }
      bj = wave_argmax_lowest(best, bj, bj != 0x7fffffff);
      if (lane == slot) result = bj;
      if (lane == 0 && bj <= jmax) imp[bj] = -1.f;
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    if (lane < p.top_n) p.topk[(int64_t)kh * p.tk_sh + tok * p.tk_st + lane] = result;
  }
}

template <int D, int GP, bool PAGED>
int launch_topk(const NsaTopkParams& p, int B, int max_q_len, hipStream_t stream) {
  constexpr int TWG = 4 * (32 / GP);
  size_t dyn = (size_t)TWG * p.nb_max * sizeof(float);
  size_t stat = 64 * (D + NSA_LDS_PAD) * 2 + 4 * (32 / GP) * 65 * 4;
  if (dyn + stat > 160 * 1024) {
    nsa_set_error("top-k: %d selection blocks x %d tokens per workgroup do not fit LDS", p.nb_max, TWG);
    return NSA_ERR_UNSUPPORTED;
  }
  auto kern = topk_kernel<D, GP, PAGED>;
  if (dyn + stat > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn);
    if (e != hipSuccess) {
      nsa_set_error("top-k: hipFuncSetAttribute(%zu) failed: %s", dyn, hipGetErrorString(e));
      return NSA_ERR_LAUNCH;
    }
  }
  dim3 grid(cdiv_i(max_q_len, TWG), B, p.KH);
  kern<<<grid, 256, dyn, stream>>>(p);
  return nsa_check_launch("topk_kernel");
}

template <int D, bool PAGED>
int dispatch_gp(const NsaTopkParams& p, int B, int max_q_len, hipStream_t stream) {
  int G = p.G;
  if (G > 16) return launch_topk<D, 32, PAGED>(p, B, max_q_len, stream);
  if (G > 8) return launch_topk<D, 16, PAGED>(p, B, max_q_len, stream);
  if (G > 4) return launch_topk<D, 8, PAGED>(p, B, max_q_len, stream);
  if (G > 2) return launch_topk<D, 4, PAGED>(p, B, max_q_len, stream);
  if (G > 1) return launch_topk<D, 2, PAGED>(p, B, max_q_len, stream);
  return launch_topk<D, 1, PAGED>(p, B, max_q_len, stream);
}

}  // namespace

int nsa_topk_launch(const NsaTopkParams& p, bool paged, int B, int max_q_len, int D, hipStream_t stream) {
  if (B <= 0 || max_q_len <= 0) return NSA_OK;
  if (D == 128) return paged ? dispatch_gp<128, true>(p, B, max_q_len, stream) : dispatch_gp<128, false>(p, B, max_q_len, stream);
  if (D == 64) return paged ? dispatch_gp<64, true>(p, B, max_q_len, stream) : dispatch_gp<64, false>(p, B, max_q_len, stream);
  if (D == 192) return paged ? dispatch_gp<192, true>(p, B, max_q_len, stream) : dispatch_gp<192, false>(p, B, max_q_len, stream);
  nsa_set_error("top-k: unsupported head dim D=%d", D);
  return NSA_ERR_UNSUPPORTED;
}

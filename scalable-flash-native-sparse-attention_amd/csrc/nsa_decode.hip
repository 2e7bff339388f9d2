// Paged-KV decode (one query token per request): two fused kernels after the pooling of the newest compressed row.
//   decode_cmp_topk_kernel      compressed attention (o, lse) + block importance + top-n selection
//   decode_slc_swa_kernel       selected-block attention + sliding-window attention + gated combine with the
//                               compressed-branch output -> final o
// Upstream runs this step as 7 launches (flash_nsa/inference/__init__.py:207-257: cmp_attn_decode stage1/2,
// topk_decode probs/select, fused_slc_swa_attn_decode stage1/2, combine_decode).
//
// One workgroup of 8 waves per (request, kv head); the G <= 16 q-heads of the group are the MFMA N dimension
// (v_mfma_f32_16x16x32_bf16, S^T = K Q^T so that softmax statistics are per-lane).  The key range is cut in units
// of 32 keys dealt round-robin to the waves; every wave runs an online softmax over its units with the K
// fragments and V rows of the next unit in flight (register double buffering), and the partial (m, l, o) of the
// waves are merged through LDS.  The step is HBM-bound: every K/V row is read once per pass straight from the
// pool through the block tables.
#include "nsa_common.h"
#include "nsa_api_internal.h"
#include <type_traits>
#include "nsa_select.h"

namespace {

constexpr int DEC_WAVES = 8;
// static LDS of decode_slc_swa_kernel (statistics and weights of up to 64 parts of the compressed branch); the host
// adds it to the dynamic size when it decides whether a launch fits the 160 KB of a CU
constexpr size_t SLC_SWA_STATIC_LDS = (3 * 16 + 64 * 16) * sizeof(float);
constexpr int UK = 32;  // keys per unit
constexpr int SEL_INTS = 192;  // LDS words of a selecting wave: 64 selected blocks + candidate list (64 scores, 64 indices)

// One wave's flash-attention state over units of 32 keys for the 16 heads of a kv group.
// K and V rows of a unit are fetched as whole rows (16 lanes x 16 bytes per row: every cache line is requested once
// and used completely), held in registers while the previous unit is computed, and pass through one wave-private
// LDS slot: first the K rows (read back as MFMA A fragments), then the V rows (read back transposed).
// With KEEP the un-normalised probabilities exp2((s - m_unit) * c) of every unit are kept in LDS as fp16 together
// with the m_unit they refer to, so that the importance pass needs no second pass over the keys.
template <int D, int VD>
struct UnitFlash {
  static constexpr int KC = D / 32;
  static constexpr int KJ = (UK * (D / 8)) / 64;
  static constexpr int VJ = (UK * (VD / 8)) / 64;
  static constexpr int KLD = D + NSA_LDS_PAD;
  static constexpr int VLD = VD + NSA_LDS_PAD;
  static constexpr int SLOT = UK * (KLD > VLD ? KLD : VLD);  // bf16 elements of a wave's staging slot
  // row stride (floats) of a published partial output [16 heads][OLD]: with VD floats the 16 rows that one
  // 16-byte store instruction writes would all start in the same LDS bank (a 16-way conflict); 4 more floats
  // spread them over all 64 banks
  static constexpr int OLD = VD + 4;
  bf16x8 qf[KC];
  f32x4 oacc[VD / 16];
  float m_run, l_run;
  float sc;
  int l16, kq, lane;
  bf16_t* Ss;          // wave-private staging slot
  _Float16* keep_p;    // [16][keep_ld] (keep_ld > 0), [units][16][UK] (keep_ld == 0: whole units contiguous), or null
  float* keep_m;       // [units][16]
  int keep_ld;

  NSA_DEVICE void init(const bf16_t* qrow, float scale_log2, int lane_, bf16_t* slot) {
    lane = lane_;
    l16 = lane & 15;
    kq = lane >> 4;
    sc = scale_log2;
    Ss = slot;
    keep_p = nullptr;
    keep_m = nullptr;
    keep_ld = 0;
#pragma unroll
    for (int kc = 0; kc < KC; kc++) qf[kc] = ld_global_b128(qrow + kq * 8 + kc * 32);
#pragma unroll
    for (int dt = 0; dt < VD / 16; dt++) oacc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    m_run = NSA_NEG_INF;
    l_run = 0.f;
  }
  // start another branch with the same q fragments
  NSA_DEVICE void reset() {
#pragma unroll
    for (int dt = 0; dt < VD / 16; dt++) oacc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    m_run = NSA_NEG_INF;
    l_run = 0.f;
    keep_p = nullptr;
  }
  // loads of the unit starting at key0 (wave-uniform); keys outside [klo, khi] are replaced by a clamped key
  // (masked later).  A unit spans at most two pages: the page of its first usable key is looked up once.
  NSA_DEVICE void issue(int key0, int klo, int khi, const int* tab_s, int page, const bf16_t* kbase, int64_t k_sr,
                        const bf16_t* vbase, int64_t v_sr, bf16x8 (&kf)[KJ], bf16x8 (&vr)[VJ]) {
    const int ks = __builtin_amdgcn_readfirstlane(max(klo, min(key0, khi)));
    const int pi = ks / page;
    const int rem0 = ks - pi * page;
    if constexpr (64 % (D / 8) == 0 && 64 % (VD / 8) == 0) {
      // A unit that lies inside [klo, khi] and inside one page (nearly all of them) is UK consecutive pool rows:
      // one wave-uniform row address per group of 64 lanes' rows, and a per-lane byte offset that never changes.
      const int k0 = __builtin_amdgcn_readfirstlane(key0);
      if (k0 >= klo && k0 + UK - 1 <= khi && rem0 + UK <= page && k_sr > 0 && v_sr > 0 && k_sr < (1 << 28) &&
          v_sr < (1 << 28)) {
        const int64_t row0 = (int64_t)__builtin_amdgcn_readfirstlane(tab_s[pi]) * page + rem0;
        const char* kp = reinterpret_cast<const char*>(kbase + row0 * k_sr);
        const char* vp = reinterpret_cast<const char*>(vbase + row0 * v_sr);
        const uint32_t koff = (uint32_t)(lane / (D / 8)) * (uint32_t)k_sr * 2u + (uint32_t)(lane % (D / 8)) * 16u;
        const uint32_t voff = (uint32_t)(lane / (VD / 8)) * (uint32_t)v_sr * 2u + (uint32_t)(lane % (VD / 8)) * 16u;
#pragma unroll
        for (int j = 0; j < KJ; j++)
          kf[j] = *reinterpret_cast<const bf16x8*>(kp + (int64_t)(j * (64 / (D / 8))) * k_sr * 2 + koff);
#pragma unroll
        for (int j = 0; j < VJ; j++)
          vr[j] = *reinterpret_cast<const bf16x8*>(vp + (int64_t)(j * (64 / (VD / 8))) * v_sr * 2 + voff);
        return;
      }
    }
    const int64_t base0 = (int64_t)tab_s[pi] * page;
    const int64_t base1 = (rem0 + UK > page && (int64_t)(pi + 1) * page <= khi) ? (int64_t)tab_s[pi + 1] * page - page : base0;
#pragma unroll
    for (int j = 0; j < KJ; j++) {
      int pc = lane + j * 64;
      int r = rem0 + max(klo, min(key0 + pc / (D / 8), khi)) - ks;
      int64_t row = (r >= page ? base1 : base0) + r;
      kf[j] = ld_global_b128(kbase + row * k_sr + (pc % (D / 8)) * 8);
    }
#pragma unroll
    for (int j = 0; j < VJ; j++) {
      int pc = lane + j * 64;
      int r = rem0 + max(klo, min(key0 + pc / (VD / 8), khi)) - ks;
      int64_t row = (r >= page ? base1 : base0) + r;
      vr[j] = ld_global_b128(vbase + row * v_sr + (pc % (VD / 8)) * 8);
    }
  }
  NSA_DEVICE void compute(int key0, int klo, int khi, bf16x8 (&kf)[KJ], bf16x8 (&vr)[VJ]) {
#pragma unroll
    for (int j = 0; j < KJ; j++) {
      int pc = lane + j * 64;
      *reinterpret_cast<bf16x8*>(&Ss[(pc / (D / 8)) * KLD + (pc % (D / 8)) * 8]) = kf[j];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    f32x4 sacc[2];
#pragma unroll
    for (int jt = 0; jt < 2; jt++) {
      sacc[jt] = f32x4{0.f, 0.f, 0.f, 0.f};
      const bf16_t* kp = &Ss[(jt * 16 + l16) * KLD + kq * 8];
#pragma unroll
      for (int kc = 0; kc < KC; kc++)
        sacc[jt] = mfma16(*reinterpret_cast<const bf16x8*>(kp + kc * 32), qf[kc], sacc[jt]);
    }
    // the K fragments are consumed (LDS operations of a wave complete in order): the slot now takes the V rows
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int j = 0; j < VJ; j++) {
      int pc = lane + j * 64;
      *reinterpret_cast<bf16x8*>(&Ss[(pc / (VD / 8)) * VLD + (pc % (VD / 8)) * 8]) = vr[j];
    }
    if (key0 < klo || key0 + UK - 1 > khi) {  // wave-uniform: only boundary units are masked
#pragma unroll
      for (int jt = 0; jt < 2; jt++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
          int key = key0 + jt * 16 + kq * 4 + i;
          if (key < klo || key > khi) sacc[jt][i] = NSA_NEG_INF;
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
    if (keep_p != nullptr) {
      typedef _Float16 h4 __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int jt = 0; jt < 2; jt++) {
        h4 hv = {(_Float16)sacc[jt][0], (_Float16)sacc[jt][1], (_Float16)sacc[jt][2], (_Float16)sacc[jt][3]};
        const int at = keep_ld > 0 ? l16 * keep_ld + key0 + jt * 16 + kq * 4
                                   : (key0 / UK) * (16 * UK) + l16 * UK + jt * 16 + kq * 4;
        *reinterpret_cast<h4*>(&keep_p[at]) = hv;
      }
      if (kq == 0) keep_m[(key0 / UK) * 16 + l16] = m_safe;
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
    bf16x8 pf = pack8(sacc[0][0], sacc[0][1], sacc[0][2], sacc[0][3], sacc[1][0], sacc[1][1], sacc[1][2], sacc[1][3]);
    const int kb0 = kq * 4 + (l16 >> 2);
    const int kb1 = kb0 + 16;
#pragma unroll
    for (int dt = 0; dt < VD / 16; dt++) {
      const int col = dt * 16 + 4 * (l16 & 3);
      bf16x4 v0 = lds_read_tr(&Ss[kb0 * VLD + col]);
      bf16x4 v1 = lds_read_tr(&Ss[kb1 * VLD + col]);
      oacc[dt] = mfma16(cat4(v0, v1), pf, oacc[dt]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  // Loads of the first unit of the next run(), issued early (before a serial section of the kernel that does not
  // touch the staging slot) so that their latency is hidden behind it; the next run() must be called with the same
  // arguments.
  bf16x8 pre_k[KJ], pre_v[VJ];
  int pre_key;
  template <class KeyFn>
  NSA_DEVICE void prefetch(int first, int nu, int klo, int khi, KeyFn key0_of, const int* tab_s, int page,
                           const bf16_t* kbase, int64_t k_sr, const bf16_t* vbase, int64_t v_sr) {
    if (first < nu) { pre_key = key0_of(first); issue(pre_key, klo, khi, tab_s, page, kbase, k_sr, vbase, v_sr, pre_k, pre_v); }
  }
  // pipelined loop over units u = first, first+step, ... < nu ; key0_of(u) gives the unit's first key
  // USE_PRE: the first unit was fetched by prefetch() with the same arguments.  Only the call that consumes the
  // prefetched registers is instantiated with it, so that they are dead everywhere else.
  template <bool USE_PRE = false, class KeyFn>
  NSA_DEVICE void run(int first, int step, int nu, int klo, int khi, KeyFn key0_of, const int* tab_s, int page,
                      const bf16_t* kbase, int64_t k_sr, const bf16_t* vbase, int64_t v_sr) {
    bf16x8 kfA[KJ], kfB[KJ], vrA[VJ], vrB[VJ];
    int keyA = 0, keyB = 0;
    if (USE_PRE) {
      keyA = pre_key;
#pragma unroll
      for (int j = 0; j < KJ; j++) kfA[j] = pre_k[j];
#pragma unroll
      for (int j = 0; j < VJ; j++) vrA[j] = pre_v[j];
    } else if (first < nu) {
      keyA = key0_of(first);
      issue(keyA, klo, khi, tab_s, page, kbase, k_sr, vbase, v_sr, kfA, vrA);
    }
    for (int u = first; u < nu; u += 2 * step) {
      const bool hasB = u + step < nu;
      if (hasB) { keyB = key0_of(u + step); issue(keyB, klo, khi, tab_s, page, kbase, k_sr, vbase, v_sr, kfB, vrB); }
      compute(keyA, klo, khi, kfA, vrA);
      if (hasB) {
        if (u + 2 * step < nu) {
          keyA = key0_of(u + 2 * step);
          issue(keyA, klo, khi, tab_s, page, kbase, k_sr, vbase, v_sr, kfA, vrA);
        }
        compute(keyB, klo, khi, kfB, vrB);
      }
    }
  }
  // wave partial -> LDS slot: m (raw units), l, o[16 heads][VD]
  NSA_DEVICE void publish(float* pm, float* pl, float* po) {
    float l_tot = xrow_sum(l_run);
    l_tot = xhalf_sum(l_tot);
    if (kq == 0) { pm[l16] = m_run; pl[l16] = l_tot; }
#pragma unroll
    for (int dt = 0; dt < VD / 16; dt++)
      *reinterpret_cast<f32x4*>(&po[l16 * OLD + dt * 16 + kq * 4]) = oacc[dt];
  }
};

// Merge of n wave partials (m in raw score units, l, un-normalised o) in two steps, so that the exponentials are
// evaluated once per (part, head) and not once per output channel:
//   merge_weights: one thread per head turns the l of every part into its normalised weight
//                  exp2((m_part - m) * c) / l_total, in place, and returns lse2 (0 when nothing was visible);
//   merge_value:   after a barrier, o[head][d] = sum over parts of weight * o_part.
NSA_DEVICE float merge_weights(const float* pm, float* pl, int nparts, int part_stride_ml, int head, float sc) {
  float m = NSA_NEG_INF;
  for (int w = 0; w < nparts; w++) m = fmaxf(m, pm[w * part_stride_ml + head]);
  if (m == NSA_NEG_INF) {
    for (int w = 0; w < nparts; w++) pl[w * part_stride_ml + head] = 0.f;
    return 0.f;
  }
  float l = 0.f;
  for (int w = 0; w < nparts; w++) {
    const float mw = pm[w * part_stride_ml + head];
    const float a = (mw == NSA_NEG_INF) ? 0.f : fast_exp2((mw - m) * sc);
    l += a * pl[w * part_stride_ml + head];
    pl[w * part_stride_ml + head] = a;
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
  for (int w = 0; w < nparts; w++) pl[w * part_stride_ml + head] *= inv;
  return l > 0.f ? m * sc + fast_log2(l) : 0.f;
}
NSA_DEVICE float merge_value(const float* wgt, const float* po, int nparts, int part_stride_ml, int part_stride_o,
                             int head, int d, int row_ld) {
  float o = 0.f;
  for (int w = 0; w < nparts; w++) o += wgt[w * part_stride_ml + head] * po[w * part_stride_o + head * row_ld + d];
  return o;
}

// four consecutive channels at once (16-byte LDS reads; same summation order over the parts as merge_value)
NSA_DEVICE f32x4 merge_value4(const float* wgt, const float* po, int nparts, int part_stride_ml, int part_stride_o,
                              int head, int d, int row_ld) {
  f32x4 o = {0.f, 0.f, 0.f, 0.f};
  for (int w = 0; w < nparts; w++) {
    const float a = wgt[w * part_stride_ml + head];
    const f32x4 x = *reinterpret_cast<const f32x4*>(&po[w * part_stride_o + head * row_ld + d]);
    o[0] += a * x[0]; o[1] += a * x[1]; o[2] += a * x[2]; o[3] += a * x[3];
  }
  return o;
}
// The same merge without the shared weights: every thread evaluates the weights of its own head in registers
// (the same operations in the same order as merge_weights, so the results are bit-identical) -- 2 * NP broadcast
// LDS reads and NP exponentials per thread buy one barrier and a serial 16-thread step less.
template <int NP>
NSA_DEVICE float merge_weights_local(const float* pm, const float* pl, int part_stride_ml, int head, float sc,
                                     float (&wgt)[NP]) {
  float mw[NP];
  float m = NSA_NEG_INF;
#pragma unroll
  for (int w = 0; w < NP; w++) { mw[w] = pm[w * part_stride_ml + head]; m = fmaxf(m, mw[w]); }
  if (m == NSA_NEG_INF) {
#pragma unroll
    for (int w = 0; w < NP; w++) wgt[w] = 0.f;
    return 0.f;
  }
  float l = 0.f;
#pragma unroll
  for (int w = 0; w < NP; w++) {
    const float a = (mw[w] == NSA_NEG_INF) ? 0.f : fast_exp2((mw[w] - m) * sc);
    l += a * pl[w * part_stride_ml + head];
    wgt[w] = a;
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int w = 0; w < NP; w++) wgt[w] *= inv;
  return l > 0.f ? m * sc + fast_log2(l) : 0.f;
}
template <int NP>
NSA_DEVICE f32x4 merge_value4_local(const float (&wgt)[NP], const float* po, int part_stride_o, int head, int d, int row_ld) {
  f32x4 o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int w = 0; w < NP; w++) {
    const float a = wgt[w];
    const f32x4 x = *reinterpret_cast<const f32x4*>(&po[w * part_stride_o + head * row_ld + d]);
    o[0] += a * x[0]; o[1] += a * x[1]; o[2] += a * x[2]; o[3] += a * x[3];
  }
  return o;
}
NSA_DEVICE f32x4 round_bf16x4(f32x4 x) {
  return f32x4{(float)(bf16_t)x[0], (float)(bf16_t)x[1], (float)(bf16_t)x[2], (float)(bf16_t)x[3]};
}

// head-summed probabilities of the compressed keys -> scores of the selection blocks (ascending key order per
// block); all threads of the workgroup
NSA_DEVICE void fold_block_scores(const float* pg, float* imp, int y, int nb, int nb_cap, const NsaDecodeParams& p,
                                  int tid, int nthreads) {
  // stride is a power of two and divides kernel_size and block_size: block j covers the compressed keys
  // j*Bs/St - Kz/St + 1 + r, r = 0 .. (Bs+Kz-St)/St - 1, with overlap area (in positions) / St as the weight
  const int Bs = p.block_size, Kz = p.kernel_size, St = p.stride;
  const int bps = Bs / St, kps = Kz / St;
  const int nloops = bps + kps - 1;
  const float inv_st = 1.f / (float)St;
  for (int j = tid; j < nb_cap; j += nthreads) {
    float acc = 0.f;
    if (j < nb) {
      const int i0 = j * bps - kps + 1;
      int cs = St - Kz;
      for (int r = 0; r < nloops; r++, cs += St) {
        const int i = i0 + r;
        if (i >= 0 && i < y) {
          const int area = min(cs + Kz, Bs) - max(cs, 0);
          acc += pg[i] * ((float)area * inv_st);
        }
      }
    }
    imp[j] = acc;
  }
}

// more than 2048 blocks: the same selection with the scores rescanned in LDS every round (taken scores are
// overwritten with -1)
NSA_DEVICE int select_blocks_lds(float* imp, int t, int nb_cap, const NsaDecodeParams& p, int lane) {
  const int nk = t >= 0 ? t / p.block_size : -1;
  int result = p.ignore_index;
  if (lane == 0) {
    for (int s = 0; s < p.num_init; s++)
      if (s < nb_cap) imp[s] = -1.f;
    for (int i = 0; i < p.num_local; i++)
      if (nk - i >= 0 && nk - i < nb_cap) imp[nk - i] = -1.f;
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
  const int jmax = min(nk, nb_cap - 1);
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
  return result;
}

// cand_v / cand_i: 64 floats + 64 ints of LDS private to the selecting wave
NSA_DEVICE int select_blocks_wave(float* imp, int t, int nb_cap, const NsaDecodeParams& p, int lane, float* cand_v,
                                  int* cand_i) {
  if (nb_cap <= 512) return select_blocks_short_list<8>(imp, t, nb_cap, p, lane, cand_v, cand_i);
  if (nb_cap <= 1024) return select_blocks_short_list<16>(imp, t, nb_cap, p, lane, cand_v, cand_i);
  if (nb_cap <= 2048) return select_blocks_short_list<32>(imp, t, nb_cap, p, lane, cand_v, cand_i);
  return select_blocks_lds(imp, t, nb_cap, p, lane);
}

template <int D, int VD, bool KEEP>
__global__ __launch_bounds__(DEC_WAVES * 64) void decode_cmp_topk_kernel(NsaDecodeParams p) {
  using UF = UnitFlash<D, VD>;
  constexpr int NW = DEC_WAVES;
  // dynamic LDS: [staging slot per wave (reused for the wave's partial o, then for pg)] [m][l][lse] [imp] [table]
  //              KEEP: [un-normalised p, fp16 [16][keep_ld]] [m of every unit [units][16]]
  //              else: [pg]
  extern __shared__ __attribute__((aligned(16))) unsigned char dyn_raw[];
  constexpr int SLOT = UF::SLOT;
  static_assert(SLOT * 2 >= 16 * UF::OLD * 4, "a wave's slot must hold its partial output");
  bf16_t* Vs_all = reinterpret_cast<bf16_t*>(dyn_raw);
  float* part_m = reinterpret_cast<float*>(dyn_raw + (size_t)NW * SLOT * 2);
  float* part_l = part_m + NW * 16;
  float* lse_s = part_l + NW * 16;
  float* imp = lse_s + 16;
  int* tab_s = reinterpret_cast<int*>(imp + p.nb_cap);  // the request's compressed-row page table
  const int ntab = (p.y_cap + p.page_size - 1) / p.page_size;
  const int n_units_cap = (p.y_cap + UK - 1) / UK;
  const int keep_ld = n_units_cap * UK + 8;  // +8 halves: the 16 head rows start in different banks
  float* after_tab = reinterpret_cast<float*>(tab_s + ((ntab + 3) & ~3));
  float* keep_m = after_tab;                                               // KEEP
  _Float16* keep_p = reinterpret_cast<_Float16*>(keep_m + n_units_cap * 16);  // KEEP
  float* pg = KEEP ? reinterpret_cast<float*>(dyn_raw) : after_tab;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = blockIdx.x, kh = blockIdx.y;
  const int G = p.G;
  const int L = p.ctx_lens[b];
  const int t = L - 1;
  const int y = L >= p.kernel_size ? min((L - p.kernel_size) / p.stride + 1, p.y_cap) : 0;
  const int nb = min(L > 0 ? (L - 1) / p.block_size + 1 : 0, p.nb_cap);
  const int32_t* ctab = p.cmp_table + (int64_t)b * p.cmp_table_stride;
  const int page = p.page_size;
  // page-table entries go to LDS first: a table lookup in global memory in front of every gather would serialise
  // the pipelined K/V loads behind it (memory operations of a wave retire in order)
  for (int i = tid; i < (y + page - 1) / page; i += NW * 64) tab_s[i] = ctab[i];
  __syncthreads();
  const bf16_t* kbase = p.k + (int64_t)kh * p.k_sh;
  const bf16_t* vbase = p.v + (int64_t)kh * p.v_sh;
  const int l16 = lane & 15, kq = lane >> 4;
  const int g = min(l16, G - 1);
  const int head = kh * G + g;

  UF uf;
  uf.init(p.q + (int64_t)b * p.q_st + (int64_t)head * p.q_sh, p.scale_log2, lane, Vs_all + wave * SLOT);
  if (KEEP) {
    uf.keep_p = keep_p;
    uf.keep_m = keep_m;
    uf.keep_ld = keep_ld;
  }
  const int nu = (y + UK - 1) / UK;

  // ---- phase A: compressed attention, units dealt round-robin to the waves ----
  uf.run(wave, NW, nu, 0, y - 1, [&](int u) { return u * UK; }, tab_s, page, kbase, p.k_sr, vbase, p.v_sr);
  uf.publish(part_m + wave * 16, part_l + wave * 16, reinterpret_cast<float*>(Vs_all + wave * SLOT));
  __syncthreads();
  if (tid < 16) {
    const float lse2 = merge_weights(part_m, part_l, NW, 16, tid, p.scale_log2);
    lse_s[tid] = tid < G ? lse2 : 0.f;
    if (tid < G && p.lse_out) p.lse_out[(int64_t)b * p.lse_st + (kh * G + tid) * p.lse_sh] = lse2;
  }
  __syncthreads();
  for (int idx = tid; idx < G * VD; idx += NW * 64) {
    int h = idx / VD, d = idx - h * VD;
    float o = merge_value(part_l, reinterpret_cast<const float*>(Vs_all), NW, 16, SLOT / 2, h, d, UF::OLD);
    p.cmp_o[(int64_t)b * p.co_st + (int64_t)(kh * G + h) * p.co_sh + d] = (bf16_t)o;
  }
  __syncthreads();

  // ---- phase B: p = exp2(s*c - lse) summed over the heads of the group, per compressed key ----
  if (KEEP) {
    // p = kept exp2((s - m_unit)*c) * exp2(m_unit*c - lse): turn the m table into these factors, then one thread per key
    for (int i = tid; i < nu * 16; i += NW * 64) {
      int h = i & 15;
      keep_m[i] = h < G ? fast_exp2(__builtin_fmaf(keep_m[i], p.scale_log2, -lse_s[h])) : 0.f;
    }
    __syncthreads();
    for (int key = tid; key < y; key += NW * 64) {
      const float* fac = keep_m + (key / UK) * 16;
      float acc = 0.f;
#pragma unroll
      for (int h = 0; h < 16; h++) acc += (float)keep_p[h * keep_ld + key] * fac[h];
      pg[key] = acc;
    }
  } else {
    // second pass over the compressed keys: S[head][key] = Q K^T, lane holds key = l16, heads kq*4 .. +3
    auto row_of = [&](int key) -> int64_t { return (int64_t)tab_s[key / page] * page + (key % page); };
    float lse4[4];
#pragma unroll
    for (int i = 0; i < 4; i++) lse4[i] = lse_s[kq * 4 + i];
    bf16x8 kf[2][UF::KC];
    for (int u = wave; u < nu; u += NW) {
      const int key0 = u * UK;
#pragma unroll
      for (int jt = 0; jt < 2; jt++) {
        int key = min(key0 + jt * 16 + l16, y - 1);
        const bf16_t* kp = kbase + row_of(key) * p.k_sr + kq * 8;
#pragma unroll
        for (int kc = 0; kc < UF::KC; kc++) kf[jt][kc] = ld_global_b128(kp + kc * 32);
      }
#pragma unroll
      for (int jt = 0; jt < 2; jt++) {
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kc = 0; kc < UF::KC; kc++) s = mfma16(uf.qf[kc], kf[jt][kc], s);
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < 4; i++)
          if (kq * 4 + i < G) acc += fast_exp2(__builtin_fmaf(s[i], p.scale_log2, -lse4[i]));
        acc = xrow_sum(acc);
        acc = xhalf_sum(acc);
        int key = key0 + jt * 16 + l16;
        if (kq == 0 && key < y) pg[key] = acc;
      }
    }
  }
  __syncthreads();
  fold_block_scores(pg, imp, y, nb, p.nb_cap, p, tid, NW * 64);
  __syncthreads();
  if (wave != 0) return;
  // the waves' partial statistics are consumed: their space is the selector's candidate list
  const int result = select_blocks_wave(imp, t, p.nb_cap, p, lane, part_m, reinterpret_cast<int*>(part_l));
  if (lane < p.top_n) p.topk[(int64_t)kh * p.tk_sh + (int64_t)b * p.tk_st + lane] = result;
}

// ---- split variant of the compressed branch: requests are cut in NSPLIT key-interleaved parts so that long
// contexts do not leave most CUs idle; partial (m, l, o) go through a small fp32 scratch in global memory.
constexpr int SPLIT_WAVES = 4;

// grid (B, KH, nsplit): compressed attention over the units u = s*4 + wave (mod 4*nsplit)
template <int D, int VD>
__global__ __launch_bounds__(SPLIT_WAVES * 64) void decode_cmp_partial_kernel(NsaDecodeParams p) {
  using UF = UnitFlash<D, VD>;
  constexpr int NW = SPLIT_WAVES;
  constexpr int SLOT = UF::SLOT;
  extern __shared__ __attribute__((aligned(16))) unsigned char dyn_raw[];
  bf16_t* Vs_all = reinterpret_cast<bf16_t*>(dyn_raw);
  float* part_m = reinterpret_cast<float*>(dyn_raw + (size_t)NW * SLOT * 2);
  float* part_l = part_m + NW * 16;
  int* tab_s = reinterpret_cast<int*>(part_l + NW * 16);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = blockIdx.x, kh = blockIdx.y, sp = blockIdx.z;
  const int nsplit = gridDim.z;
  const int G = p.G;
  const int L = p.ctx_lens[b];
  const int y = L >= p.kernel_size ? min((L - p.kernel_size) / p.stride + 1, p.y_cap) : 0;
  const int32_t* ctab = p.cmp_table + (int64_t)b * p.cmp_table_stride;
  const int page = p.page_size;
  for (int i = tid; i < (y + page - 1) / page; i += NW * 64) tab_s[i] = ctab[i];
  // The compressed row that the newest token completes (mean of the last kernel_size raw rows, fp32 sums in row
  // order like nsa_paged_pool_decode; flash_nsa/inference/compress_kv.py:253-287 upstream) is written by the part
  // that attends it -- the one whose waves own the last unit -- wave 0 for K and wave 1 for V, one 16-byte piece per
  // lane.  Only this workgroup reads it back in this launch, so a workgroup-scope release and the barrier suffice.
  {
    const int cmp_slot = p.cmp_slots != nullptr ? p.cmp_slots[b] : -1;
    const int last_unit = y > 0 ? (y - 1) / UK : 0;
    if (cmp_slot >= 0 && L >= p.kernel_size && sp == (last_unit % (NW * nsplit)) / NW && wave < 2) {
      bf16_t* cache = const_cast<bf16_t*>(wave == 0 ? p.k : p.v);
      const int64_t c_sr = wave == 0 ? p.k_sr : p.v_sr, c_sh = wave == 0 ? p.k_sh : p.v_sh;
      if (lane < (wave == 0 ? D : VD) / 8) {
        const int32_t* tab = p.table + (int64_t)b * p.table_stride;
        const int st = ((L - p.kernel_size) / p.stride) * p.stride;
        float a[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int r = 0; r < p.kernel_size; r++) {
          const int n = st + r;
          const int64_t row = (int64_t)tab[n / page] * page + (n % page);
          const bf16x8 x = ld_global_b128(cache + row * c_sr + (int64_t)kh * c_sh + lane * 8);
#pragma unroll
          for (int e = 0; e < 8; e++) a[e] += (float)x[e];
        }
        const float inv = 1.f / (float)p.kernel_size;
        *reinterpret_cast<bf16x8*>(cache + (int64_t)cmp_slot * c_sr + (int64_t)kh * c_sh + lane * 8) =
            pack8(a[0] * inv, a[1] * inv, a[2] * inv, a[3] * inv, a[4] * inv, a[5] * inv, a[6] * inv, a[7] * inv);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    }
  }
  __syncthreads();
  const bf16_t* kbase = p.k + (int64_t)kh * p.k_sh;
  const bf16_t* vbase = p.v + (int64_t)kh * p.v_sh;
  const int l16 = lane & 15;
  const int head = kh * G + min(l16, G - 1);

  UF uf;
  uf.init(p.q + (int64_t)b * p.q_st + (int64_t)head * p.q_sh, p.scale_log2, lane, Vs_all + wave * SLOT);
  if (p.sp_keep_p != nullptr) {  // spill the un-normalised probabilities of every unit for the final kernel
    const int nuc = (p.y_cap + UK - 1) / UK;
    uf.keep_ld = 0;  // unit-major: a wave writes the 1 KB of a unit as whole cache lines
    uf.keep_p = p.sp_keep_p + ((int64_t)b * p.KH + kh) * 16 * nuc * UK;
    uf.keep_m = p.sp_keep_m + ((int64_t)b * p.KH + kh) * nuc * 16;
  }
  const int nu = (y + UK - 1) / UK;
  uf.run(sp * NW + wave, NW * nsplit, nu, 0, y - 1, [&](int u) { return u * UK; }, tab_s, page, kbase, p.k_sr,
         vbase, p.v_sr);
  uf.publish(part_m + wave * 16, part_l + wave * 16, reinterpret_cast<float*>(Vs_all + wave * SLOT));
  __syncthreads();
  // merge the 4 waves; store the split's un-normalised partial
  const int64_t base = (((int64_t)b * p.KH + kh) * nsplit + sp) * 16;
  const float* po = reinterpret_cast<const float*>(Vs_all);
  for (int idx = tid; idx < 16 * VD; idx += NW * 64) {
    int h = idx / VD, d = idx - h * VD;
    float m = NSA_NEG_INF;
    for (int w = 0; w < NW; w++) m = fmaxf(m, part_m[w * 16 + h]);
    float l = 0.f, o = 0.f;
    if (m != NSA_NEG_INF) {
      for (int w = 0; w < NW; w++) {
        float mw = part_m[w * 16 + h];
        float a = (mw == NSA_NEG_INF) ? 0.f : fast_exp2((mw - m) * p.scale_log2);
        l += a * part_l[w * 16 + h];
        o += a * po[w * (SLOT / 2) + h * UF::OLD + d];
      }
    }
    p.sp_o[(base + h) * VD + d] = o;
    if (d == 0) { p.sp_m[base + h] = m; p.sp_l[base + h] = l; }
  }
}

// grid (B, KH, nsplit): merge the splits (lse; split 0 also writes cmp_o), then the head-summed probabilities of
// this split's compressed keys -> pg [B, KH, y_cap] fp32
template <int D, int VD>
__global__ __launch_bounds__(SPLIT_WAVES * 64) void decode_importance_kernel(NsaDecodeParams p) {
  constexpr int NW = SPLIT_WAVES;
  constexpr int KC = D / 32;
  __shared__ float lse_s[16];
  __shared__ float m_s[16], l_s[16];
  extern __shared__ int tab_dyn[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = blockIdx.x, kh = blockIdx.y, sp = blockIdx.z;
  const int nsplit = gridDim.z;
  const int G = p.G;
  const int L = p.ctx_lens[b];
  const int y = L >= p.kernel_size ? min((L - p.kernel_size) / p.stride + 1, p.y_cap) : 0;
  const int32_t* ctab = p.cmp_table + (int64_t)b * p.cmp_table_stride;
  const int page = p.page_size;
  for (int i = tid; i < (y + page - 1) / page; i += NW * 64) tab_dyn[i] = ctab[i];
  const int64_t base = ((int64_t)b * p.KH + kh) * nsplit * 16;
  if (tid < 16) {
    float m = NSA_NEG_INF;
    for (int s2 = 0; s2 < nsplit; s2++) m = fmaxf(m, p.sp_m[base + s2 * 16 + tid]);
    float l = 0.f;
    if (m != NSA_NEG_INF)
      for (int s2 = 0; s2 < nsplit; s2++) {
        float ms = p.sp_m[base + s2 * 16 + tid];
        if (ms != NSA_NEG_INF) l += fast_exp2((ms - m) * p.scale_log2) * p.sp_l[base + s2 * 16 + tid];
      }
    m_s[tid] = m;
    l_s[tid] = l;
    float lse2 = (m != NSA_NEG_INF && l > 0.f) ? m * p.scale_log2 + fast_log2(l) : 0.f;
    lse_s[tid] = lse2;
    if (sp == 0 && tid < G && p.lse_out) p.lse_out[(int64_t)b * p.lse_st + (kh * G + tid) * p.lse_sh] = lse2;
  }
  __syncthreads();
  if (sp == 0) {
    for (int idx = tid; idx < G * VD; idx += NW * 64) {
      int h = idx / VD, d = idx - h * VD;
      float m = m_s[h], l = l_s[h], o = 0.f;
      if (m != NSA_NEG_INF && l > 0.f) {
        for (int s2 = 0; s2 < nsplit; s2++) {
          float ms = p.sp_m[base + s2 * 16 + h];
          if (ms != NSA_NEG_INF) o += fast_exp2((ms - m) * p.scale_log2) * p.sp_o[(base + s2 * 16 + h) * VD + d];
        }
        o /= l;
      }
      p.cmp_o[(int64_t)b * p.co_st + (int64_t)(kh * G + h) * p.co_sh + d] = (bf16_t)o;
    }
  }
  // S[head][key] = Q K^T : lane holds key = l16, heads kq*4 .. +3
  auto row_of = [&](int key) -> int64_t { return (int64_t)tab_dyn[key / page] * page + (key % page); };
  const bf16_t* kbase = p.k + (int64_t)kh * p.k_sh;
  const int l16 = lane & 15, kq = lane >> 4;
  const int head = kh * G + min(l16, G - 1);
  bf16x8 qf[KC];
  {
    const bf16_t* qp = p.q + (int64_t)b * p.q_st + (int64_t)head * p.q_sh + kq * 8;
#pragma unroll
    for (int kc = 0; kc < KC; kc++) qf[kc] = ld_global_b128(qp + kc * 32);
  }
  float lse4[4];
#pragma unroll
  for (int i = 0; i < 4; i++) lse4[i] = lse_s[kq * 4 + i];
  float* pg = p.pg + ((int64_t)b * p.KH + kh) * p.y_cap;
  const int nu = (y + UK - 1) / UK;
  const int step = NW * nsplit;
  bf16x8 kfA[2][KC], kfB[2][KC];
  auto issue = [&](int u, bf16x8 (&kf)[2][KC]) {
#pragma unroll
    for (int jt = 0; jt < 2; jt++) {
      int key = min(u * UK + jt * 16 + l16, y - 1);
      const bf16_t* kp = kbase + row_of(key) * p.k_sr + kq * 8;
#pragma unroll
      for (int kc = 0; kc < KC; kc++) kf[jt][kc] = ld_global_b128(kp + kc * 32);
    }
  };
  auto compute = [&](int u, bf16x8 (&kf)[2][KC]) {
#pragma unroll
    for (int jt = 0; jt < 2; jt++) {
      f32x4 sv = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kc = 0; kc < KC; kc++) sv = mfma16(qf[kc], kf[jt][kc], sv);
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < 4; i++)
        if (kq * 4 + i < G) acc += fast_exp2(__builtin_fmaf(sv[i], p.scale_log2, -lse4[i]));
      acc = xrow_sum(acc);
      acc = xhalf_sum(acc);
      int key = u * UK + jt * 16 + l16;
      if (kq == 0 && key < y) pg[key] = acc;
    }
  };
  const int first = sp * NW + wave;
  if (first < nu) issue(first, kfA);
  for (int u = first; u < nu; u += 2 * step) {
    const bool hasB = u + step < nu;
    if (hasB) issue(u + step, kfB);
    compute(u, kfA);
    if (hasB) {
      if (u + 2 * step < nu) issue(u + 2 * step, kfA);
      compute(u + step, kfB);
    }
  }
}

template <int D, int VD>
__global__ __launch_bounds__(DEC_WAVES * 64) void decode_slc_swa_kernel(NsaDecodeParams p) {
  using UF = UnitFlash<D, VD>;
  constexpr int NW = DEC_WAVES;
  constexpr int NT = NW * 64;
  extern __shared__ __attribute__((aligned(16))) unsigned char dyn_raw[];
  constexpr int SLOT = UF::SLOT;
  static_assert(SLOT * 2 >= 16 * UF::OLD * 4, "a wave's slot must hold its partial output");
  bf16_t* Vs_all = reinterpret_cast<bf16_t*>(dyn_raw);
  float* part_m = reinterpret_cast<float*>(dyn_raw + (size_t)NW * SLOT * 2);
  float* part_l = part_m + NW * 16;
  int* blk_s = reinterpret_cast<int*>(part_l + NW * 16);
  float* cand_v = reinterpret_cast<float*>(blk_s + 64);  // the selector's candidate list (64 scores + 64 indices)
  int* cand_i = blk_s + 128;
  int* tab_s = blk_s + SEL_INTS;  // the request's raw page table

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = blockIdx.x, kh = blockIdx.y;
  // the window and selected units of a (request, kv head) may be cut into gridDim.z parts (every part repeats the
  // prologue and the selection, which all of them need, and writes partial results for a merging launch)
  const int part = blockIdx.z, nparts = gridDim.z;
  const int G = p.G;
  const int L = p.ctx_lens[b];
  const int t = L - 1;
  const int32_t* tab = p.table + (int64_t)b * p.table_stride;
  const int page = p.page_size;
  for (int i = tid; i < (L + page - 1) / page; i += NT) tab_s[i] = tab[i];
  const bf16_t* kbase = p.k + (int64_t)kh * p.k_sh;
  const bf16_t* vbase = p.v + (int64_t)kh * p.v_sh;
  const int l16 = lane & 15;
  const int g = min(l16, G - 1);
  const int head = kh * G + g;
  const int Bs = p.block_size;
  const int nvalid = t >= 0 ? min(p.top_n, t / Bs + 1) : 0;
  const int nb = min(L > 0 ? (L - 1) / Bs + 1 : 0, p.nb_cap);
  __shared__ float sp_lse_s[16], sp_m_s[16], sp_l_s[16];
  __shared__ float sp_w_s[64 * 16];  // weights of the parts of the compressed branch (nsplit <= 64)
  static_assert(sizeof(sp_lse_s) + sizeof(sp_m_s) + sizeof(sp_l_s) + sizeof(sp_w_s) == SLC_SWA_STATIC_LDS,
                "the host-side LDS budget must count this kernel's static arrays");
  constexpr int OPT = 16 * VD / NT;  // output values per thread
  static_assert((16 * VD) % NT == 0, "output values must divide over the threads");
  float ocmp_pre[OPT];               // split path: merged compressed-branch output of this thread's values
  float* imp = nullptr;              // block scores, when the selection runs here
  const bool select_here = p.sp_keep_p != nullptr || p.pg != nullptr;
  if (p.sp_keep_p != nullptr) {
    // Prologue of the two-launch split path: merge the statistics of the parts of the compressed branch, turn the
    // spilled fp16 probabilities into head-summed probabilities (over the not-yet-used staging slots) and fold them
    // into block scores.  The same arithmetic as the one-launch kernel.
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    const int y = L >= p.kernel_size ? min((L - p.kernel_size) / p.stride + 1, p.y_cap) : 0;
    const int nuc = (p.y_cap + UK - 1) / UK, keep_ld = nuc * UK;
    const int nsplit = p.nsplit;
    float* pgs = reinterpret_cast<float*>(Vs_all);
    imp = reinterpret_cast<float*>(tab_s + ((p.table_stride + 3) & ~3));
    float* fac = imp + ((p.nb_cap + 3) & ~3);
    const int64_t sp_base = ((int64_t)b * p.KH + kh) * nsplit * 16;
    const _Float16* keep_p = p.sp_keep_p + ((int64_t)b * p.KH + kh) * 16 * keep_ld;
    const float* keep_m = p.sp_keep_m + ((int64_t)b * p.KH + kh) * nuc * 16;
    // all (m, l) of the parts in one round trip, then one thread per head
    float* st_m = fac;
    float* st_l = fac + 64 * 16;
    for (int i = tid; i < nsplit * 16; i += NT) { st_m[i] = p.sp_m[sp_base + i]; st_l[i] = p.sp_l[sp_base + i]; }
    __syncthreads();
    if (tid < 16) {
      float m = NSA_NEG_INF;
      for (int s2 = 0; s2 < nsplit; s2++) m = fmaxf(m, st_m[s2 * 16 + tid]);
      float l = 0.f;
      for (int s2 = 0; s2 < nsplit; s2++) {
        const float ms = st_m[s2 * 16 + tid];
        const float a = (ms == NSA_NEG_INF) ? 0.f : fast_exp2((ms - m) * p.scale_log2);
        sp_w_s[s2 * 16 + tid] = a;
        l += a * st_l[s2 * 16 + tid];
      }
      const float inv = l > 0.f ? 1.f / l : 0.f;
      for (int s2 = 0; s2 < nsplit; s2++) sp_w_s[s2 * 16 + tid] *= inv;
      const float lse2 = (m != NSA_NEG_INF && l > 0.f) ? m * p.scale_log2 + fast_log2(l) : 0.f;
      sp_lse_s[tid] = lse2;
      if (tid < G && p.lse_out) p.lse_out[(int64_t)b * p.lse_st + (kh * G + tid) * p.lse_sh] = lse2;
    }
    __syncthreads();
    // merge of the parts' outputs: independent loads, issued here so that they overlap the rest of the prologue
#pragma unroll
    for (int r = 0; r < OPT; r++) {
      const int idx = tid + r * NT;
      const int h = idx / VD, d = idx - h * VD;
      float o = 0.f;
      for (int s2 = 0; s2 < nsplit; s2++) o += sp_w_s[s2 * 16 + h] * p.sp_o[(sp_base + s2 * 16 + h) * VD + d];
      ocmp_pre[r] = o;
    }
    const int nu = (y + UK - 1) / UK;
    for (int i = tid; i < nu * 16; i += NT) {
      const int h = i & 15;
      fac[i] = h < G ? fast_exp2(__builtin_fmaf(keep_m[i], p.scale_log2, -sp_lse_s[h])) : 0.f;
    }
    __syncthreads();
    for (int k4 = tid * 4; k4 < y; k4 += NT * 4) {
      const float* f = fac + (k4 / UK) * 16;
      h4 v[16];
#pragma unroll
      for (int h = 0; h < 16; h++)
        v[h] = *reinterpret_cast<const h4*>(keep_p + (k4 / UK) * (16 * UK) + h * UK + (k4 % UK));
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int h = 0; h < 16; h++)
#pragma unroll
        for (int e = 0; e < 4; e++) acc[e] += (float)v[h][e] * f[h];
      *reinterpret_cast<f32x4*>(pgs + k4) = acc;
    }
    __syncthreads();
    fold_block_scores(pgs, imp, y, nb, nb, p, tid, NT);
  } else if (p.pg != nullptr) {
    // fold the head-summed probabilities of the compressed keys (computed by the importance kernel) into block
    // scores; they live behind the page table, the staging slots belong to the window waves
    imp = reinterpret_cast<float*>(tab_s + ((p.table_stride + 3) & ~3));
    const float* pg = p.pg + ((int64_t)b * p.KH + kh) * p.y_cap;
    const int y = L >= p.kernel_size ? min((L - p.kernel_size) / p.stride + 1, p.y_cap) : 0;
    fold_block_scores(pg, imp, y, nb, nb, p, tid, NT);
  } else if (tid < 64) {
    blk_s[tid] = tid < nvalid ? max(p.topk[(int64_t)kh * p.tk_sh + (int64_t)b * p.tk_st + tid], 0) : 0;
  }
  __syncthreads();

  // ---- window attention; when the selection runs here, wave 0 selects meanwhile ----
  UF uf;
  uf.init(p.q + (int64_t)b * p.q_st + (int64_t)head * p.q_sh, p.scale_log2, lane, Vs_all + wave * SLOT);
  const int w_first = select_here ? 1 : 0;
  if (wave < w_first) {
    const int result = select_blocks_wave(imp, t, nb, p, lane, cand_v, cand_i);
    blk_s[lane] = lane < nvalid ? max(result, 0) : 0;
    if (p.topk && part == 0 && lane < p.top_n) p.topk[(int64_t)kh * p.tk_sh + (int64_t)b * p.tk_st + lane] = result;
  } else {
    if (t >= 0) {
      const int klo = max(0, t - p.window);
      const int k0 = (klo / UK) * UK;
      const int nu = (t - k0) / UK + 1;
      uf.run(part * (NW - w_first) + wave - w_first, nparts * (NW - w_first), nu, klo, t,
             [&](int u) { return k0 + u * UK; }, tab_s, page, kbase, p.k_sr, vbase, p.v_sr);
    }
    uf.publish(part_m + wave * 16, part_l + wave * 16, reinterpret_cast<float*>(Vs_all + wave * SLOT));
  }
  __syncthreads();
  const float* part_o = reinterpret_cast<const float*>(Vs_all);
  // parts: the un-normalised (m, l, o) of this part's waves, one thread per output value (same arithmetic as the
  // partial kernel of the compressed branch)
  auto spill_part = [&](int branch, int w0, int nw) {
    const int64_t base = ((((int64_t)b * p.KH + kh) * nparts + part) * 2 + branch);
    for (int idx = tid; idx < 16 * VD; idx += NT) {
      const int h = idx / VD, d = idx - h * VD;
      float m = NSA_NEG_INF;
      for (int w = w0; w < w0 + nw; w++) m = fmaxf(m, part_m[w * 16 + h]);
      float l = 0.f, o = 0.f;
      if (m != NSA_NEG_INF) {
        for (int w = w0; w < w0 + nw; w++) {
          const float mw = part_m[w * 16 + h];
          const float a = (mw == NSA_NEG_INF) ? 0.f : fast_exp2((mw - m) * p.scale_log2);
          l += a * part_l[w * 16 + h];
          o += a * part_o[w * (SLOT / 2) + h * UF::OLD + d];
        }
      }
      p.sp2_o[(base * 16 + h) * VD + d] = o;
      if (d == 0) { p.sp2_ml[(base * 2 + 0) * 16 + h] = m; p.sp2_ml[(base * 2 + 1) * 16 + h] = l; }
    }
  };
  if (nparts > 1) {
    spill_part(1, w_first, NW - w_first);
    __syncthreads();  // the slots are staging space again
    uf.reset();
    if (t >= 0) {
      const int upb = Bs / UK;
      uf.run(part * NW + wave, nparts * NW, nvalid * upb, 0, t,
             [&](int u) { int slot = u / upb; return blk_s[slot] * Bs + (u - slot * upb) * UK; }, tab_s, page, kbase,
             p.k_sr, vbase, p.v_sr);
    }
    uf.publish(part_m + wave * 16, part_l + wave * 16, reinterpret_cast<float*>(Vs_all + wave * SLOT));
    __syncthreads();
    spill_part(0, 0, NW);
    if (part == 0 && p.sp_keep_p != nullptr) {  // the compressed branch's output, merged in the prologue
#pragma unroll
      for (int r = 0; r < OPT; r++) {
        const int idx = tid + r * NT;
        const int h = idx / VD, d = idx - h * VD;
        if (h < G) p.cmp_tmp[(int64_t)b * p.co_st + (int64_t)(kh * G + h) * p.co_sh + d] = (bf16_t)ocmp_pre[r];
      }
    }
    return;
  }
  if (tid < 16) merge_weights(part_m + w_first * 16, part_l + w_first * 16, NW - w_first, 16, tid, p.scale_log2);
  __syncthreads();
  float o_swa_pre[OPT];
#pragma unroll
  for (int r = 0; r < OPT; r++) {
    const int idx = tid + r * NT;
    const int h = idx / VD, d = idx - h * VD;
    o_swa_pre[r] = merge_value(part_l + w_first * 16, part_o + w_first * (SLOT / 2), NW - w_first, 16, SLOT / 2, h, d, UF::OLD);
  }
  __syncthreads();  // the slots are staging space again

  // ---- selected blocks, all waves ----
  uf.reset();
  if (t >= 0) {
    const int upb = Bs / UK;
    uf.run(wave, NW, nvalid * upb, 0, t,
           [&](int u) { int slot = u / upb; return blk_s[slot] * Bs + (u - slot * upb) * UK; }, tab_s, page, kbase,
           p.k_sr, vbase, p.v_sr);
  }
  uf.publish(part_m + wave * 16, part_l + wave * 16, reinterpret_cast<float*>(Vs_all + wave * SLOT));
  __syncthreads();
  if (tid < 16) merge_weights(part_m, part_l, NW, 16, tid, p.scale_log2);
  __syncthreads();
#pragma unroll
  for (int r = 0; r < OPT; r++) {
    const int idx = tid + r * NT;
    const int h = idx / VD, d = idx - h * VD;
    if (h >= G) continue;
    const int hq = kh * G + h;
    float o_slc = merge_value(part_l, part_o, NW, 16, SLOT / 2, h, d, UF::OLD);
    // branch outputs are rounded to bf16 before the gated sum, as the three-kernel path stores them
    o_slc = (float)(bf16_t)o_slc;
    const float o_swa = (float)(bf16_t)o_swa_pre[r];
    if (p.slc_o) p.slc_o[(int64_t)b * p.co_st + (int64_t)hq * p.co_sh + d] = (bf16_t)o_slc;
    if (p.swa_o) p.swa_o[(int64_t)b * p.co_st + (int64_t)hq * p.co_sh + d] = (bf16_t)o_swa;
    if (p.out) {
      const bf16_t* wp = p.w + (int64_t)b * p.w_st + (int64_t)hq * p.w_sh;
      float s0 = 1.f / (1.f + __expf(-(float)wp[0]));
      float s1 = 1.f / (1.f + __expf(-(float)wp[1]));
      float s2 = 1.f / (1.f + __expf(-(float)wp[2]));
      float o_cmp;
      if (p.sp_keep_p != nullptr) {  // merged in the prologue
        const float o = ocmp_pre[r];
        if (p.cmp_o) p.cmp_o[(int64_t)b * p.co_st + (int64_t)hq * p.co_sh + d] = (bf16_t)o;
        o_cmp = (float)(bf16_t)o;
      } else {
        o_cmp = (float)p.cmp_o[(int64_t)b * p.co_st + (int64_t)hq * p.co_sh + d];
      }
      p.out[(int64_t)b * p.o_st + (int64_t)hq * p.o_sh + d] = (bf16_t)(o_cmp * s0 + o_slc * s1 + o_swa * s2);
    }
  }
}

// grid (B, KH): merges the parts written by decode_slc_swa_kernel when it ran with several parts per (request, kv
// head) and applies the gates -> final output (and the branch outputs on request)
template <int VD>
__global__ __launch_bounds__(256) void decode_split_final_kernel(NsaDecodeParams p) {
  const int b = blockIdx.x, kh = blockIdx.y, tid = threadIdx.x;
  const int G = p.G, S = p.slc_nsplit;
  for (int idx = tid; idx < G * (VD / 4); idx += 256) {
    const int h = idx / (VD / 4), d = (idx - h * (VD / 4)) * 4;
    const int hq = kh * G + h;
    f32x4 res[2];
#pragma unroll
    for (int br = 0; br < 2; br++) {
      const int64_t base0 = (((int64_t)b * p.KH + kh) * S) * 2 + br;
      float m = NSA_NEG_INF;
      for (int s2 = 0; s2 < S; s2++) m = fmaxf(m, p.sp2_ml[((base0 + s2 * 2) * 2 + 0) * 16 + h]);
      float l = 0.f;
      f32x4 o = {0.f, 0.f, 0.f, 0.f};
      if (m != NSA_NEG_INF) {
        for (int s2 = 0; s2 < S; s2++) {
          const int64_t base = base0 + s2 * 2;
          const float ms = p.sp2_ml[(base * 2 + 0) * 16 + h];
          const float a = (ms == NSA_NEG_INF) ? 0.f : fast_exp2((ms - m) * p.scale_log2);
          l += a * p.sp2_ml[(base * 2 + 1) * 16 + h];
          const f32x4 x = *reinterpret_cast<const f32x4*>(p.sp2_o + (base * 16 + h) * VD + d);
          o[0] += a * x[0]; o[1] += a * x[1]; o[2] += a * x[2]; o[3] += a * x[3];
        }
      }
      const float inv = l > 0.f ? 1.f / l : 0.f;
      // branch outputs are rounded to bf16 before the gated sum, as the other decode paths store them
      res[br] = round_bf16x4(f32x4{o[0] * inv, o[1] * inv, o[2] * inv, o[3] * inv});
    }
    const int64_t co = (int64_t)b * p.co_st + (int64_t)hq * p.co_sh + d;
    if (p.slc_o) *reinterpret_cast<bf16x4*>(p.slc_o + co) = pack4(res[0][0], res[0][1], res[0][2], res[0][3]);
    if (p.swa_o) *reinterpret_cast<bf16x4*>(p.swa_o + co) = pack4(res[1][0], res[1][1], res[1][2], res[1][3]);
    const bf16x4 c4 = *reinterpret_cast<const bf16x4*>(p.cmp_tmp + co);
    if (p.cmp_o) *reinterpret_cast<bf16x4*>(p.cmp_o + co) = c4;
    const bf16_t* wp = p.w + (int64_t)b * p.w_st + (int64_t)hq * p.w_sh;
    const float s0 = 1.f / (1.f + __expf(-(float)wp[0]));
    const float s1 = 1.f / (1.f + __expf(-(float)wp[1]));
    const float s2g = 1.f / (1.f + __expf(-(float)wp[2]));
    *reinterpret_cast<bf16x4*>(p.out + (int64_t)b * p.o_st + (int64_t)hq * p.o_sh + d) =
        pack4((float)c4[0] * s0 + res[0][0] * s1 + res[1][0] * s2g, (float)c4[1] * s0 + res[0][1] * s1 + res[1][1] * s2g,
              (float)c4[2] * s0 + res[0][2] * s1 + res[1][2] * s2g, (float)c4[3] * s0 + res[0][3] * s1 + res[1][3] * s2g);
  }
}

// ---- the whole decode step of one (request, kv head) in one workgroup ------------------------------------------
// compressed attention -> block scores -> [wave 0: selection | waves 1..7: window attention] -> selected-block
// attention -> gated combine.  Nothing but the final output (and, on request, topk / the branch outputs) goes
// back to global memory; the compressed-branch output stays in registers, the window partials in the LDS region
// that held the fp16 probabilities.
template <int D, int VD>
__global__ __launch_bounds__(DEC_WAVES * 64) void decode_fused_kernel(NsaDecodeParams p) {
  using UF = UnitFlash<D, VD>;
  constexpr int NW = DEC_WAVES;
  constexpr int SLOT = UF::SLOT;
  constexpr int NTHREADS = NW * 64;
  constexpr int NV4 = 16 * VD / 4;                             // groups of four merged output values
  constexpr int OPT4 = (NV4 + NTHREADS - 1) / NTHREADS;        // groups per thread
  static_assert(SLOT * 2 >= 16 * UF::OLD * 4, "a wave's slot must hold its partial output");
  extern __shared__ __attribute__((aligned(16))) unsigned char dyn_raw[];
  bf16_t* slots = reinterpret_cast<bf16_t*>(dyn_raw);
  float* part_m = reinterpret_cast<float*>(dyn_raw + (size_t)NW * SLOT * 2);
  float* part_l = part_m + NW * 16;
  float* swa_m = part_l + NW * 16;
  float* swa_l = swa_m + NW * 16;
  float* lse_s = swa_l + NW * 16;
  float* imp = lse_s + 16;
  int* blk_s = reinterpret_cast<int*>(imp + ((p.nb_cap + 3) & ~3));
  float* cand_v = reinterpret_cast<float*>(blk_s + 64);  // the selector's candidate list (64 scores + 64 indices)
  int* cand_i = blk_s + 128;
  int* ctab_s = blk_s + SEL_INTS;
  const int ntab_c = (p.y_cap + p.page_size - 1) / p.page_size;
  int* tab_s = ctab_s + ((ntab_c + 3) & ~3);
  const int n_units_cap = (p.y_cap + UK - 1) / UK;
  const int keep_ld = n_units_cap * UK + 8;
  float* keep_m = reinterpret_cast<float*>(tab_s + ((p.table_stride + 3) & ~3));
  _Float16* keep_p = reinterpret_cast<_Float16*>(keep_m + n_units_cap * 16);
  float* swa_o = reinterpret_cast<float*>(keep_p);  // [NW-1][16][VD], after the probabilities are consumed
  float* pg = reinterpret_cast<float*>(dyn_raw);    // over the staging slots, between the phases

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = blockIdx.x, kh = blockIdx.y;
  const int G = p.G;
  const int L = p.ctx_lens[b];
  const int t = L - 1;
  const int y = L >= p.kernel_size ? min((L - p.kernel_size) / p.stride + 1, p.y_cap) : 0;
  const int Bs = p.block_size;
  const int nb = min(L > 0 ? (L - 1) / Bs + 1 : 0, p.nb_cap);
  const int page = p.page_size;
  {
    const int32_t* ctab = p.cmp_table + (int64_t)b * p.cmp_table_stride;
    const int32_t* tab = p.table + (int64_t)b * p.table_stride;
    // whole table rows (their widths are the capacity, the entries past a request's pages are never used), so that
    // these loads do not wait for the context length and both round trips overlap
    const int nc = min(ntab_c, p.cmp_table_stride), nr = p.table_stride;
    for (int i = tid; i < nc + nr; i += NTHREADS) {
      if (i < nc) ctab_s[i] = ctab[i];
      else tab_s[i - nc] = tab[i - nc];
    }
  }
  // Cache maintenance of this (request, kv head), wave 0 for K and wave 1 for V, one 16-byte piece per lane:
  //  * the newest token's row goes to its pool row (upstream store_kvcache,
  //    nano-vllm/nanovllm/layers/attention.py:123-153), when the caller passes it;
  //  * the compressed row that the newest token completes = mean of the last kernel_size raw rows, summed in
  //    row order in fp32 like nsa_paged_pool_decode (flash_nsa/inference/compress_kv.py:253-287 upstream).
  // Both are written to the pool and read back by the attention phases of this workgroup after a fence and a
  // barrier.  The compressed phase only needs the pooled row, so when nothing is pooled at this step the store
  // runs after the first barrier and its fence is covered by the barriers that separate the phases.
  const int raw_slot = (p.raw_slots != nullptr && L > 0) ? p.raw_slots[b] : -1;
  const int cmp_slot = p.cmp_slots != nullptr ? p.cmp_slots[b] : -1;
  const bool pool_now = cmp_slot >= 0 && L >= p.kernel_size;
  auto maintain = [&]() {
    bf16_t* cache = const_cast<bf16_t*>(wave == 0 ? p.k : p.v);
    const int64_t c_sr = wave == 0 ? p.k_sr : p.v_sr, c_sh = wave == 0 ? p.k_sh : p.v_sh;
    const int C = (wave == 0 ? D : VD) / 8;
    if (lane < C) {
      bf16x8 newest = zero_bf16x8();
      if (raw_slot >= 0) {
        const bf16_t* src = wave == 0 ? p.new_k + (int64_t)b * p.nk_st + (int64_t)kh * p.nk_sh
                                      : p.new_v + (int64_t)b * p.nv_st + (int64_t)kh * p.nv_sh;
        newest = ld_global_b128(src + lane * 8);
        *reinterpret_cast<bf16x8*>(cache + (int64_t)raw_slot * c_sr + (int64_t)kh * c_sh + lane * 8) = newest;
      }
      if (pool_now) {
        const int32_t* tab = p.table + (int64_t)b * p.table_stride;
        const int st = ((L - p.kernel_size) / p.stride) * p.stride;
        float a[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int r = 0; r < p.kernel_size; r++) {
          const int n = st + r;
          bf16x8 x;
          if (raw_slot >= 0 && n == L - 1) {
            x = newest;  // the row just stored: taken from the register, not read back
          } else {
            const int64_t row = (int64_t)tab[n / page] * page + (n % page);
            x = ld_global_b128(cache + row * c_sr + (int64_t)kh * c_sh + lane * 8);
          }
#pragma unroll
          for (int e = 0; e < 8; e++) a[e] += (float)x[e];
        }
        const float inv = 1.f / (float)p.kernel_size;
        *reinterpret_cast<bf16x8*>(cache + (int64_t)cmp_slot * c_sr + (int64_t)kh * c_sh + lane * 8) =
            pack8(a[0] * inv, a[1] * inv, a[2] * inv, a[3] * inv, a[4] * inv, a[5] * inv, a[6] * inv, a[7] * inv);
      }
    }
    // the rows are read back only by waves of this workgroup (same CU, same vector L1): a workgroup-scope release
    // is enough, and much cheaper than a device-scope fence, which writes back the L2 slice of the XCD
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  };
  if (pool_now && wave < 2) maintain();
  __syncthreads();
  if (!pool_now && raw_slot >= 0 && wave < 2) maintain();
  const bf16_t* kbase = p.k + (int64_t)kh * p.k_sh;
  const bf16_t* vbase = p.v + (int64_t)kh * p.v_sh;
  const int l16 = lane & 15;
  const int head = kh * G + min(l16, G - 1);

  UF uf;
  uf.init(p.q + (int64_t)b * p.q_st + (int64_t)head * p.q_sh, p.scale_log2, lane, slots + wave * SLOT);
  uf.keep_p = keep_p;
  uf.keep_m = keep_m;
  uf.keep_ld = keep_ld;
  const int nu = (y + UK - 1) / UK;

  // ---- compressed attention, units dealt round-robin to the waves ----
  uf.run(wave, NW, nu, 0, y - 1, [&](int u) { return u * UK; }, ctab_s, page, kbase, p.k_sr, vbase, p.v_sr);
  uf.publish(part_m + wave * 16, part_l + wave * 16, reinterpret_cast<float*>(slots + wave * SLOT));
  // the window branch does not depend on anything computed here: the waves that will run it fetch their first
  // unit now, behind the merge of the compressed branch, the block scores and the selection
  const int swa_klo = max(0, t - p.window);
  const int swa_k0 = (swa_klo / UK) * UK;
  const int swa_nu = t >= 0 ? (t - swa_k0) / UK + 1 : 0;
  auto swa_key = [&](int u) { return swa_k0 + u * UK; };
  constexpr bool PREFETCH_SWA = true;
  // When the newest token's row was stored by waves 0 / 1 after the first barrier (nothing pooled at this step),
  // only the next barrier orders that store before other waves' reads of the row, and the window's last unit holds
  // it: the prefetch then waits for the barrier (workgroup-uniform condition).
  const bool stored_late = !pool_now && raw_slot >= 0;
  if (PREFETCH_SWA && !stored_late && wave != 0 && t >= 0)
    uf.prefetch(wave - 1, swa_nu, swa_klo, t, swa_key, tab_s, page, kbase, p.k_sr, vbase, p.v_sr);
  __syncthreads();
  if (PREFETCH_SWA && stored_late && wave != 0 && t >= 0)
    uf.prefetch(wave - 1, swa_nu, swa_klo, t, swa_key, tab_s, page, kbase, p.k_sr, vbase, p.v_sr);
  // every thread merges four consecutive channels of one head (16-byte LDS reads, 8-byte stores) with weights it
  // evaluates itself; the thread that holds channel 0 of a head also publishes the head's lse
  f32x4 o_cmp[OPT4];
#pragma unroll
  for (int r = 0; r < OPT4; r++) {
    const int idx = tid + r * NTHREADS;
    const int h = min(idx / (VD / 4), 15), d = (idx % (VD / 4)) * 4;
    float wgt[NW];
    const float lse2 = merge_weights_local<NW>(part_m, part_l, 16, h, p.scale_log2, wgt);
    if (idx < NV4 && d == 0) {
      lse_s[h] = h < G ? lse2 : 0.f;
      if (h < G && p.lse_out) p.lse_out[(int64_t)b * p.lse_st + (kh * G + h) * p.lse_sh] = lse2;
    }
    // the staged path stores the branch output as bf16 before the gated sum
    o_cmp[r] = round_bf16x4(merge_value4_local<NW>(wgt, reinterpret_cast<const float*>(slots), SLOT / 2, h, d, UF::OLD));
    if (idx < NV4 && h < G && p.cmp_o)
      *reinterpret_cast<bf16x4*>(p.cmp_o + (int64_t)b * p.co_st + (int64_t)(kh * G + h) * p.co_sh + d) =
          pack4(o_cmp[r][0], o_cmp[r][1], o_cmp[r][2], o_cmp[r][3]);
  }
  __syncthreads();
  // ---- probabilities p = kept exp2((s - m_unit)*c) * exp2(m_unit*c - lse), summed over the heads; a thread takes
  // four consecutive keys (one unit, so one set of 16 per-head factors) ----
  for (int key = tid * 4; key < y; key += NTHREADS * 4) {
    const float* um = keep_m + (key / UK) * 16;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int h = 0; h < 16; h++) {
      const float fac = h < G ? fast_exp2(__builtin_fmaf(um[h], p.scale_log2, -lse_s[h])) : 0.f;
      typedef _Float16 h4 __attribute__((ext_vector_type(4)));
      const h4 kp = *reinterpret_cast<const h4*>(&keep_p[h * keep_ld + key]);
      acc[0] += (float)kp[0] * fac; acc[1] += (float)kp[1] * fac;
      acc[2] += (float)kp[2] * fac; acc[3] += (float)kp[3] * fac;
    }
    *reinterpret_cast<f32x4*>(&pg[key]) = acc;
  }
  __syncthreads();
  fold_block_scores(pg, imp, y, nb, p.nb_cap, p, tid, NTHREADS);
  __syncthreads();

  // ---- wave 0 selects the blocks while the other waves run the window ----
  const int nvalid = t >= 0 ? min(p.top_n, t / Bs + 1) : 0;
  uf.reset();
  if (wave == 0) {
    const int result = select_blocks_wave(imp, t, p.nb_cap, p, lane, cand_v, cand_i);
    blk_s[lane] = lane < nvalid ? max(result, 0) : 0;
    if (p.topk && lane < p.top_n) p.topk[(int64_t)kh * p.tk_sh + (int64_t)b * p.tk_st + lane] = result;
  } else {
    if (t >= 0)
      uf.template run<PREFETCH_SWA>(wave - 1, NW - 1, swa_nu, swa_klo, t, swa_key, tab_s, page, kbase, p.k_sr, vbase,
                                    p.v_sr);
    uf.publish(swa_m + wave * 16, swa_l + wave * 16, swa_o + (wave - 1) * 16 * UF::OLD);
  }
  __syncthreads();

  // ---- selected blocks, all waves ----
  uf.reset();
  if (t >= 0) {
    const int upb = Bs / UK;
    uf.run(wave, NW, nvalid * upb, 0, t,
           [&](int u) { int slot = u / upb; return blk_s[slot] * Bs + (u - slot * upb) * UK; }, tab_s, page, kbase,
           p.k_sr, vbase, p.v_sr);
  }
  uf.publish(part_m + wave * 16, part_l + wave * 16, reinterpret_cast<float*>(slots + wave * SLOT));
  __syncthreads();
#pragma unroll
  for (int r = 0; r < OPT4; r++) {
    const int idx = tid + r * NTHREADS;
    const int h = idx / (VD / 4), d = (idx % (VD / 4)) * 4;
    if (idx >= NV4 || h >= G) continue;
    const int hq = kh * G + h;
    float w_slc[NW], w_swa[NW - 1];
    merge_weights_local<NW>(part_m, part_l, 16, h, p.scale_log2, w_slc);
    merge_weights_local<NW - 1>(swa_m + 16, swa_l + 16, 16, h, p.scale_log2, w_swa);
    const f32x4 o_slc =
        round_bf16x4(merge_value4_local<NW>(w_slc, reinterpret_cast<const float*>(slots), SLOT / 2, h, d, UF::OLD));
    const f32x4 o_swa = round_bf16x4(merge_value4_local<NW - 1>(w_swa, swa_o, 16 * UF::OLD, h, d, UF::OLD));
    const int64_t co = (int64_t)b * p.co_st + (int64_t)hq * p.co_sh + d;
    if (p.slc_o) *reinterpret_cast<bf16x4*>(p.slc_o + co) = pack4(o_slc[0], o_slc[1], o_slc[2], o_slc[3]);
    if (p.swa_o) *reinterpret_cast<bf16x4*>(p.swa_o + co) = pack4(o_swa[0], o_swa[1], o_swa[2], o_swa[3]);
    const bf16_t* wp = p.w + (int64_t)b * p.w_st + (int64_t)hq * p.w_sh;
    const float s0 = 1.f / (1.f + __expf(-(float)wp[0]));
    const float s1 = 1.f / (1.f + __expf(-(float)wp[1]));
    const float s2 = 1.f / (1.f + __expf(-(float)wp[2]));
    *reinterpret_cast<bf16x4*>(p.out + (int64_t)b * p.o_st + (int64_t)hq * p.o_sh + d) =
        pack4(o_cmp[r][0] * s0 + o_slc[0] * s1 + o_swa[0] * s2, o_cmp[r][1] * s0 + o_slc[1] * s1 + o_swa[1] * s2,
              o_cmp[r][2] * s0 + o_slc[2] * s1 + o_swa[2] * s2, o_cmp[r][3] * s0 + o_slc[3] * s1 + o_swa[3] * s2);
  }
}

}  // namespace

template <class K>
static int launch_dyn(K kern, dim3 grid, size_t dyn, const NsaDecodeParams& p, hipStream_t stream, const char* name,
                      size_t static_lds = 0) {
  if (dyn + static_lds > 160 * 1024) {
    nsa_set_error("%s: %zu bytes of LDS needed (fixed_y_maxlen / fixed_num_slc_blocks too large)", name,
                  dyn + static_lds);
    return NSA_ERR_UNSUPPORTED;
  }
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)dyn);
  if (e != hipSuccess) {
    nsa_set_error("%s: hipFuncSetAttribute(%zu) failed: %s", name, dyn, hipGetErrorString(e));
    return NSA_ERR_LAUNCH;
  }
  kern<<<grid, DEC_WAVES * 64, dyn, stream>>>(p);
  return nsa_check_launch(name);
}

template <int D, int VD>
static size_t slot_bytes() { return (size_t)DEC_WAVES * UnitFlash<D, VD>::SLOT * 2; }

// LDS of the fused compressed-attention + selection kernel; `keep` adds the fp16 probabilities of every compressed
// key and the per-unit maxima (no second pass over the keys) and drops the separate pg array
static size_t cmp_topk_lds(size_t slots, const NsaDecodeParams& p, bool keep) {
  const size_t ntab = (size_t)(p.y_cap + p.page_size - 1) / p.page_size;
  const size_t units = (size_t)(p.y_cap + UK - 1) / UK;
  size_t n = slots + (size_t)(2 * DEC_WAVES * 16 + 16 + p.nb_cap + ((ntab + 3) & ~(size_t)3)) * sizeof(float);
  if (keep) n += units * 16 * sizeof(float) + 16 * (units * UK + 8) * sizeof(_Float16);
  else n += (size_t)p.y_cap * sizeof(float);
  return n;
}

template <int D, int VD>
static int launch_cmp_topk(const NsaDecodeParams& p, dim3 grid, hipStream_t stream) {
  const size_t keep_bytes = cmp_topk_lds(slot_bytes<D, VD>(), p, true);
  if (keep_bytes <= 160 * 1024)
    return launch_dyn(decode_cmp_topk_kernel<D, VD, true>, grid, keep_bytes, p, stream, "decode_cmp_topk_kernel");
  return launch_dyn(decode_cmp_topk_kernel<D, VD, false>, grid, cmp_topk_lds(slot_bytes<D, VD>(), p, false), p, stream,
                    "decode_cmp_topk_kernel");
}

int nsa_decode_cmp_topk_launch(const NsaDecodeParams& p, int B, int D, int VD, hipStream_t stream) {
  if (B <= 0) return NSA_OK;
  dim3 grid(B, p.KH);
  if (D == 128 && VD == 128) return launch_cmp_topk<128, 128>(p, grid, stream);
  if (D == 64 && VD == 64) return launch_cmp_topk<64, 64>(p, grid, stream);
  nsa_set_error("decode: unsupported head dims D=%d VD=%d (built: 128/128, 64/64)", D, VD);
  return NSA_ERR_UNSUPPORTED;
}

int nsa_decode_slc_swa_launch(const NsaDecodeParams& p, int B, int D, int VD, hipStream_t stream) {
  if (B <= 0) return NSA_OK;
  dim3 grid(B, p.KH);
  size_t extra = (size_t)(2 * DEC_WAVES * 16 + SEL_INTS + ((p.table_stride + 3) & ~3)) * sizeof(float);
  if (p.pg != nullptr) extra += (size_t)((p.nb_cap + 3) & ~3) * sizeof(float);  // block scores
  if (D == 128 && VD == 128)
    return launch_dyn(decode_slc_swa_kernel<128, 128>, grid, slot_bytes<128, 128>() + extra, p, stream,
                      "decode_slc_swa_kernel", SLC_SWA_STATIC_LDS);
  if (D == 64 && VD == 64)
    return launch_dyn(decode_slc_swa_kernel<64, 64>, grid, slot_bytes<64, 64>() + extra, p, stream,
                      "decode_slc_swa_kernel", SLC_SWA_STATIC_LDS);
  nsa_set_error("decode: unsupported head dims D=%d VD=%d (built: 128/128, 64/64)", D, VD);
  return NSA_ERR_UNSUPPORTED;
}

int nsa_decode_cmp_split_launch(const NsaDecodeParams& p, int B, int nsplit, int D, int VD, hipStream_t stream) {
  if (B <= 0) return NSA_OK;
  dim3 grid(B, p.KH, nsplit);
  int ntab = (p.y_cap + p.page_size - 1) / p.page_size;
  size_t dyn1 = (size_t)SPLIT_WAVES * (D == 128 ? UnitFlash<128, 128>::SLOT : UnitFlash<64, 64>::SLOT) * 2 +
                (size_t)(2 * SPLIT_WAVES * 16 + ntab) * 4;
  size_t dyn2 = (size_t)ntab * 4;
  if (!((D == 128 && VD == 128) || (D == 64 && VD == 64))) {
    nsa_set_error("decode: unsupported head dims D=%d VD=%d (built: 128/128, 64/64)", D, VD);
    return NSA_ERR_UNSUPPORTED;
  }
  if (D == 128) {
    decode_cmp_partial_kernel<128, 128><<<grid, SPLIT_WAVES * 64, dyn1, stream>>>(p);
    int rc = nsa_check_launch("decode_cmp_partial_kernel");
    if (rc) return rc;
    decode_importance_kernel<128, 128><<<grid, SPLIT_WAVES * 64, dyn2, stream>>>(p);
  } else {
    decode_cmp_partial_kernel<64, 64><<<grid, SPLIT_WAVES * 64, dyn1, stream>>>(p);
    int rc = nsa_check_launch("decode_cmp_partial_kernel");
    if (rc) return rc;
    decode_importance_kernel<64, 64><<<grid, SPLIT_WAVES * 64, dyn2, stream>>>(p);
  }
  return nsa_check_launch("decode_importance_kernel");
}

// ---- two-launch split path: partial kernel with the probability spill, then the final kernel ----
template <int D, int VD>
static size_t split_final_lds(const NsaDecodeParams& p) {
  const size_t slots = slot_bytes<D, VD>();
  if ((size_t)((p.y_cap + UK - 1) / UK) * UK * 4 > slots) return 0;  // head-summed probabilities overlay the slots
  const size_t nuc = (size_t)(p.y_cap + UK - 1) / UK;
  const size_t total = slots + (size_t)(2 * DEC_WAVES * 16 + SEL_INTS + ((p.table_stride + 3) & ~3)) * 4 +
                       (size_t)(((p.nb_cap + 3) & ~3) + (nuc * 16 > 2 * 64 * 16 ? nuc * 16 : 2 * 64 * 16)) * 4;  // factors, or the parts' (m, l)
  return total + SLC_SWA_STATIC_LDS <= 160 * 1024 ? total : 0;
}

int nsa_decode_split_lds_bytes(const NsaDecodeParams& p, int D, int VD) {
  if (D == 128 && VD == 128) return (int)split_final_lds<128, 128>(p);
  if (D == 64 && VD == 64) return (int)split_final_lds<64, 64>(p);
  return 0;
}

int nsa_decode_split_static_lds_bytes() { return (int)SLC_SWA_STATIC_LDS; }

int nsa_decode_split_launch(const NsaDecodeParams& p, int B, int D, int VD, hipStream_t stream) {
  if (B <= 0) return NSA_OK;
  const int lds2 = nsa_decode_split_lds_bytes(p, D, VD);
  if (lds2 == 0) {
    nsa_set_error("decode_split: head dims %d/%d or fixed_y_maxlen %d / fixed_num_slc_blocks %d / table width %d do "
                  "not fit the final kernel's LDS", D, VD, p.y_cap, p.nb_cap, p.table_stride);
    return NSA_ERR_UNSUPPORTED;
  }
  const int S = p.slc_nsplit > 1 ? p.slc_nsplit : 1;
  dim3 grid1(B, p.KH, p.nsplit), grid2(B, p.KH, S);
  const int ntab = (p.y_cap + p.page_size - 1) / p.page_size;
  const size_t dyn1 = (size_t)SPLIT_WAVES * (D == 128 ? UnitFlash<128, 128>::SLOT : UnitFlash<64, 64>::SLOT) * 2 +
                      (size_t)(2 * SPLIT_WAVES * 16 + ntab) * 4;
  if (D == 128) {
    decode_cmp_partial_kernel<128, 128><<<grid1, SPLIT_WAVES * 64, dyn1, stream>>>(p);
    int rc = nsa_check_launch("decode_cmp_partial_kernel");
    if (rc) return rc;
    rc = launch_dyn(decode_slc_swa_kernel<128, 128>, grid2, (size_t)lds2, p, stream, "decode_slc_swa_kernel",
                    SLC_SWA_STATIC_LDS);
    if (rc || S == 1) return rc;
    decode_split_final_kernel<128><<<dim3(B, p.KH), 256, 0, stream>>>(p);
    return nsa_check_launch("decode_split_final_kernel");
  }
  decode_cmp_partial_kernel<64, 64><<<grid1, SPLIT_WAVES * 64, dyn1, stream>>>(p);
  int rc = nsa_check_launch("decode_cmp_partial_kernel");
  if (rc) return rc;
  rc = launch_dyn(decode_slc_swa_kernel<64, 64>, grid2, (size_t)lds2, p, stream, "decode_slc_swa_kernel",
                  SLC_SWA_STATIC_LDS);
  if (rc || S == 1) return rc;
  decode_split_final_kernel<64><<<dim3(B, p.KH), 256, 0, stream>>>(p);
  return nsa_check_launch("decode_split_final_kernel");
}

// LDS of the one-launch decode kernel; 0 when it does not fit (the caller then takes the two-launch path)
template <int D, int VD>
static size_t fused_lds(const NsaDecodeParams& p) {
  const size_t ntab_c = (size_t)(p.y_cap + p.page_size - 1) / p.page_size;
  const size_t units = (size_t)(p.y_cap + UK - 1) / UK;
  size_t region = 16 * (units * UK + 8) * sizeof(_Float16);
  const size_t swa_part = (size_t)(DEC_WAVES - 1) * 16 * UnitFlash<D, VD>::OLD * sizeof(float);
  if (region < swa_part) region = swa_part;
  region = (region + 15) & ~(size_t)15;
  size_t n = slot_bytes<D, VD>() +
             (size_t)(4 * DEC_WAVES * 16 + 16 + (((size_t)p.nb_cap + 3) & ~(size_t)3) + SEL_INTS + ((ntab_c + 3) & ~(size_t)3) +
                      (((size_t)p.table_stride + 3) & ~(size_t)3) + units * 16) * sizeof(float) + region;
  if ((size_t)p.y_cap * sizeof(float) > slot_bytes<D, VD>()) return 0;
  return n <= 160 * 1024 ? n : 0;
}

int nsa_decode_fused_lds_bytes(const NsaDecodeParams& p, int D, int VD) {
  if (D == 128 && VD == 128) return (int)fused_lds<128, 128>(p);
  if (D == 64 && VD == 64) return (int)fused_lds<64, 64>(p);
  return 0;
}

int nsa_decode_fused_launch(const NsaDecodeParams& p, int B, int D, int VD, hipStream_t stream) {
  if (B <= 0) return NSA_OK;
  dim3 grid(B, p.KH);
  const int dyn = nsa_decode_fused_lds_bytes(p, D, VD);
  if (dyn == 0) {
    nsa_set_error("decode_fused: head dims %d/%d or fixed_y_maxlen %d / fixed_num_slc_blocks %d / table width %d do "
                  "not fit the one-launch kernel (160 KB of LDS); use the two-launch path", D, VD, p.y_cap, p.nb_cap,
                  p.table_stride);
    return NSA_ERR_UNSUPPORTED;
  }
  if (D == 128) return launch_dyn(decode_fused_kernel<128, 128>, grid, (size_t)dyn, p, stream, "decode_fused_kernel");
  return launch_dyn(decode_fused_kernel<64, 64>, grid, (size_t)dyn, p, stream, "decode_fused_kernel");
}

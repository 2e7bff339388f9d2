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
#include <type_traits>

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

// Picks the blocks of one token from its score row imp[0 .. nb_max) (one wave): forced initial and local blocks
// first, then repeated arg-max (lowest index on ties).  Returns the block of slot `lane`.
// With REGS the candidates of a lane (blocks lane, lane+64, ...) sit in 16 registers (nb_max <= 1024) and only the
// winner's lane rescans; otherwise every round rescans the LDS row.
template <bool REGS>
NSA_DEVICE int select_row(float* imp, int t, int nb_max, const NsaTopkParams& p, int lane) {
  const int nk = t / p.block_size;
  const int jmax = min(nk, nb_max - 1);
  const int nsel = min(p.top_n, nk + 1);
  int result = p.ignore_index;
  if (lane < p.num_init) {
    if (lane <= nk) result = lane;
  } else if (lane < p.num_init + p.num_local) {
    if (lane <= nk) result = nk - (lane - p.num_init);
  }
  if (REGS) {
    // candidates in two groups of 8 registers with their best kept aside: a round marks and rescans only the group
    // the winner came from (its number is wave-uniform)
    float v[16];
#pragma unroll
    for (int k = 0; k < 16; k++) {
      const int j = lane + 64 * k;
      float x = j <= jmax ? imp[min(j, nb_max - 1)] : -3.f;
      if (j <= jmax && (j < p.num_init || j > nk - p.num_local)) x = -1.f;
      v[k] = x;
    }
    float gbest[2];
    int gidx[2];
    auto rescan = [&](auto g_tag) {
      constexpr int g = decltype(g_tag)::value;
      float bs = -2.f;
      int bi = 0x7fffffff;
#pragma unroll
      for (int k = g * 8; k < g * 8 + 8; k++)
        if (v[k] > bs) { bs = v[k]; bi = lane + 64 * k; }
      gbest[g] = bs;
      gidx[g] = bi;
    };
    rescan(std::integral_constant<int, 0>{});
    rescan(std::integral_constant<int, 1>{});
    for (int slot = p.num_init + p.num_local; slot < nsel; slot++) {
      const bool second = gbest[1] > gbest[0];
      const int w = wave_argmax_lowest(second ? gbest[1] : gbest[0], second ? gidx[1] : gidx[0],
                                       (second ? gidx[1] : gidx[0]) != 0x7fffffff);
      if (lane == slot) result = w;
      if (w > jmax) continue;  // wave-uniform: no candidate left
      const bool mine = (w & 63) == lane;
      const int kk = w >> 6;
      auto take = [&](auto g_tag) {
        constexpr int g = decltype(g_tag)::value;
#pragma unroll
        for (int k = g * 8; k < g * 8 + 8; k++)
          if (mine && k == kk) v[k] = -1.f;
        rescan(g_tag);
      };
      if (kk < 8) take(std::integral_constant<int, 0>{});
      else take(std::integral_constant<int, 1>{});
    }
    return result;
  }
  if (lane == 0) {
    for (int s = 0; s < p.num_init; s++)
      if (s < nb_max) imp[s] = -1.f;
    for (int i = 0; i < p.num_local; i++)
      if (nk - i >= 0 && nk - i < nb_max) imp[nk - i] = -1.f;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  for (int slot = p.num_init + p.num_local; slot < nsel; slot++) {
    float best = -2.f;
    int bj = 0x7fffffff;
    for (int j = lane; j <= jmax; j += 64) {
      float x = imp[j];
      if (x > best) { best = x; bj = j; }
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

// Segmented selection, for contexts whose score rows do not fit LDS.  The LDS row of a token holds the scores of one
// segment of selection blocks (row[jj] = block j0 + jj); once the compressed keys of the segment are folded, its
// `count` finished blocks are merged with the winners of the earlier segments (cand_s / cand_i, `ncand` slots in
// LDS, empty slots have index 0x7fffffff) by the same repeated arg-max, lowest index on ties -- so the list after
// the last segment is the list the one-pass selector produces.  Forced blocks never enter the list.  On return
// lane r < ncand holds the r-th winner (index, or 0x7fffffff) and the LDS list is updated.
NSA_DEVICE int merge_segment(float* row, int count, int j0, float* cand_s, int* cand_i, int ncand, bool first, int t,
                             int nb_max, const NsaTopkParams& p, int lane) {
  const int nk = t / p.block_size;
  const int jmax = min(nk, nb_max - 1);
  for (int jj = lane; jj < count; jj += 64) {
    const int j = j0 + jj;
    if (j > jmax || j < p.num_init || j > nk - p.num_local) row[jj] = -3.f;
  }
  if (first && lane < ncand) cand_i[lane] = 0x7fffffff;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  float my_s = -3.f;
  int my_i = 0x7fffffff;
  for (int r = 0; r < ncand; r++) {
    float best = -2.f;
    int bj = 0x7fffffff;
    for (int jj = lane; jj < count; jj += 64) {
      const float x = row[jj];
      if (x > best) { best = x; bj = j0 + jj; }
    }
    if (lane < ncand) {  // winners of earlier segments: lower block numbers, so they win ties
      const int ci = cand_i[lane];
      const float x = cand_s[lane];
      if (ci != 0x7fffffff && (x > best || (x == best && ci < bj))) { best = x; bj = ci; }
    }
    float ws;
    const int w = wave_argmax_lowest_score(best, bj, bj != 0x7fffffff, ws);
    if (w == 0x7fffffff) break;  // wave-uniform: nothing left
    if (lane == r) { my_s = ws; my_i = w; }
    if (w >= j0) {
      if (lane == 0) row[w - j0] = -3.f;
    } else if (lane < ncand && cand_i[lane] == w) {
      cand_i[lane] = 0x7fffffff;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  if (lane < ncand) { cand_s[lane] = my_s; cand_i[lane] = my_i; }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  return my_i;
}

// Workgroup = 4 waves on the same 64 (token, head) rows (two MFMA row blocks); the compressed keys are cut in units
// of 32 that are dealt to the waves (wave w takes unit 4*tile + w of every 128-key tile).  A wave stages the rows of
// its unit in a private LDS slot (coalesced whole-row loads, one tile ahead through registers), reads each K
// fragment once and uses it for both row blocks; the head-summed probabilities go to a double-buffered LDS tile,
// and after the one barrier per tile all threads fold that tile into the block scores in ascending key order.
template <int D, int GP, bool PAGED>
__global__ __launch_bounds__(256, 2) void topk_kernel(NsaTopkParams p) {
  constexpr int UK = 32;            // keys per unit
  constexpr int KT = 4 * UK;        // keys per tile
  constexpr int RB = 2;             // 32-row blocks per workgroup
  constexpr int KLD = D + NSA_LDS_PAD;
  constexpr int TPB = 32 / GP;      // tokens per row block
  constexpr int TWG = RB * TPB;     // tokens per workgroup
  constexpr int PLD = KT + 4;
  constexpr int KP = D / 8;
  constexpr int KJ = (UK * KP) / 64;
  using SM = SlotMap<GP>;
  __shared__ __attribute__((aligned(16))) bf16_t Ks_all[4 * UK * KLD];
  __shared__ float Pst[2 * TWG * PLD];
  extern __shared__ float imp_all[];  // [TWG][W] scores, then (segmented mode) [TWG][ncand] scores + indices

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int hl = lane >> 5;
  const int b = blockIdx.y;
  const int kh = blockIdx.z;
  const int G = p.G;
  const int n_hc = GP < 32 ? 1 : (G + 31) / 32;  // chunks of 32 q-heads (more than one only for G > 32)

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
  // segmented mode: a score row covers blocks [j0, j0 + seg] plus the block a segment's last tile only starts
  const int seg = p.seg_blocks;
  const int W = seg > 0 ? seg + 1 : nb_max;
  const int ncand = max(p.top_n - p.num_init - p.num_local, 0);
  float* cand_s_all = imp_all + TWG * W;
  int* cand_i_all = reinterpret_cast<int*>(cand_s_all + TWG * ncand);
  const int tiles_per_seg = seg > 0 ? seg / ((St * KT) / Bs) : 0x7fffffff;
  int j0 = 0;

  for (int i = tid; i < TWG * W; i += 256) imp_all[i] = 0.f;
  bf16_t* Ks = Ks_all + wave * UK * KLD;

  const int t_hi_wg = min(n0 + TWG - 1, xl - 1) + qoff;
  const int key_end = t_hi_wg >= Kz - 1 ? min((t_hi_wg - Kz + 1) / St + 1, nkeys) : 0;
  const int ntiles = (key_end + KT - 1) / KT;

  // A-operand rows of this lane (row l32 of each block) and the lse of its C-layout rows
  bf16x8 qf[RB][D / 16];
  float lse_r[RB][16];
  bool rows_full[RB];
  auto load_rows = [&](int hc) {
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
      int g = hc * 32 + (l32 % GP);
      if (g >= G) g = G - 1;
      const int n_a = min(n0 + rb * TPB + l32 / GP, xl - 1);
      const bf16_t* qp = p.q + (int64_t)(x0 + n_a) * p.q_st + (int64_t)(kh * G + g) * p.q_sh + hl * 8;
#pragma unroll
      for (int kc = 0; kc < D / 16; kc++) qf[rb][kc] = ld_global_b128(qp + kc * 16);
      bool mine = true;
#pragma unroll
      for (int i = 0; i < 16; i++) {
        int row = (i >> 2) * 8 + hl * 4 + (i & 3);
        int gg = hc * 32 + (row % GP);
        int nn = n0 + rb * TPB + row / GP;
        bool ok = (gg < G) && (nn < xl);
        mine = mine && ok;
        lse_r[rb][i] = ok ? p.lse[(int64_t)(x0 + nn) * p.lse_st + (int64_t)(kh * G + gg) * p.lse_sh] : 0.f;
      }
      rows_full[rb] = __builtin_amdgcn_ballot_w64(!mine) == 0;
    }
  };
  if (GP < 32 || n_hc == 1) load_rows(0);

  // fold constants: a tile covers a whole number of selection blocks, so the blocks a tile touches, the offsets of
  // their compressed keys inside the tile and the overlap weights are the same for every tile
  const int f_nloops = (Bs + Kz - St) / St;
  const int f_nj = (St * (KT - 1) + Kz - 1) / Bs + 1;
  const bool fold_fast = (St * KT) % Bs == 0 && TWG * f_nj <= 256 && f_nloops <= 8;
  const int f_tk = tid / f_nj, f_jj = tid - f_tk * f_nj;
  const bool f_on = tid < TWG * f_nj;
  const int f_rel0 = (f_jj * Bs - Kz) / St + 1;
  float f_w[8];
  {
    int cs = St - Kz;
#pragma unroll
    for (int r = 0; r < 8; r++, cs += St) {
      f_w[r] = (float)(min(cs + Kz, Bs) - max(cs, 0)) / (float)St;
      asm volatile("" : "+v"(f_w[r]));  // keep the quotient in a register: the division must not sink into the loop
    }
  }

  // rows of the wave's unit of the next tile travel through registers while the current one is computed
  bf16x8 kreg[KJ];
  uint32_t kboff[KJ];  // byte offset of the lane's 16-byte pieces inside a unit (same for every unit)
#pragma unroll
  for (int j = 0; j < KJ; j++) {
    int pc = lane + j * 64;
    kboff[j] = (uint32_t)(((int64_t)(pc / KP) * p.ck_sr + (pc % KP) * 8) * 2);
  }
  auto issue = [&](int key0) {
    int64_t row0;
    if (PAGED) row0 = (int64_t)table[key0 / p.page_size] * p.page_size + (key0 % p.page_size);
    else row0 = (int64_t)kbase + key0;
    const char* kb = reinterpret_cast<const char*>(p.ck + row0 * p.ck_sr + (int64_t)kh * p.ck_sh);
    const int last = key_end - 1 - key0;
    if (last >= UK - 1) {
#pragma unroll
      for (int j = 0; j < KJ; j++) kreg[j] = *reinterpret_cast<const bf16x8*>(kb + kboff[j]);
    } else {  // the last unit: rows past the last visible key repeat it (masked below)
#pragma unroll
      for (int j = 0; j < KJ; j++) {
        int pc = lane + j * 64;
        int kr = min(pc / KP, last);
        kreg[j] = ld_global_b128(p.ck + (row0 + kr) * p.ck_sr + (int64_t)kh * p.ck_sh + (pc % KP) * 8);
      }
    }
  };
  if (wave * UK < key_end) issue(wave * UK);
  __syncthreads();  // score rows are zeroed

  for (int tile = 0; tile < ntiles; tile++) {
    const int key0 = tile * KT + wave * UK;
    float* pst = Pst + (tile & 1) * TWG * PLD;
    if (key0 < key_end) {
#pragma unroll
      for (int j = 0; j < KJ; j++) {
        int pc = lane + j * 64;
        *reinterpret_cast<bf16x8*>(&Ks[(pc / KP) * KLD + (pc % KP) * 8]) = kreg[j];
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      if (key0 + KT < key_end) issue(key0 + KT);
      bf16x8 kf[D / 16];
#pragma unroll
      for (int kc = 0; kc < D / 16; kc++)
        kf[kc] = *reinterpret_cast<const bf16x8*>(&Ks[l32 * KLD + hl * 8 + kc * 16]);
      const int key = key0 + l32;
      const int vis_from = St * key + Kz - 1;  // first position that sees this key
      for (int hc = 0; hc < n_hc; hc++) {
        if (GP == 32 && n_hc > 1) load_rows(hc);
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
          f32x16 sacc;
#pragma unroll
          for (int i = 0; i < 16; i++) sacc[i] = 0.f;
#pragma unroll
          for (int kc = 0; kc < D / 16; kc++) sacc = mfma32(qf[rb][kc], kf[kc], sacc);
          float ps[SM::NSLOT];
#pragma unroll
          for (int s2 = 0; s2 < SM::NSLOT; s2++) ps[s2] = 0.f;
          // wave-uniform: away from the causal boundary every (row, key) pair of the unit is visible
          const bool all_vis = rows_full[rb] && key0 + UK <= nkeys &&
                               n0 + rb * TPB + qoff >= St * (key0 + UK - 1) + Kz - 1;
          if (all_vis) {
#pragma unroll
            for (int i = 0; i < 16; i++)
              ps[SM::slot_of(i)] += fast_exp2(__builtin_fmaf(sacc[i], p.scale_log2, -lse_r[rb][i]));
          } else {
#pragma unroll
            for (int i = 0; i < 16; i++) {
              int row = (i >> 2) * 8 + hl * 4 + (i & 3);
              int nn = n0 + rb * TPB + row / GP;
              bool vis = (hc * 32 + (row % GP) < G) && (nn < xl) && (key < nkeys) && (nn + qoff >= vis_from);
              float pv = vis ? fast_exp2(__builtin_fmaf(sacc[i], p.scale_log2, -lse_r[rb][i])) : 0.f;
              ps[SM::slot_of(i)] += pv;
            }
          }
#pragma unroll
          for (int s2 = 0; s2 < SM::NSLOT; s2++) {
            float v = ps[s2];
            if (SM::CROSS) v = xhalf_sum(v);
            if (!SM::CROSS || hl == 0) {
              int tk = rb * TPB + SM::token_of(s2, hl);
              float* dst = &pst[tk * PLD + wave * UK + l32];
              *dst = (hc == 0) ? v : *dst + v;
            }
          }
        }
      }
    } else {
      for (int i = lane; i < TWG * UK; i += 64) pst[(i / UK) * PLD + wave * UK + (i % UK)] = 0.f;
    }
    __syncthreads();
    // ---- fold the 128 compressed keys of this tile into selection-block scores ----
    const int kt = tile * KT;
    if (fold_fast) {
      const int j = (St * kt) / Bs + f_jj;
      if (f_on && j < nb_max) {
        float* cell = &imp_all[f_tk * W + (j - j0)];  // j - j0 <= seg: a tile stays inside its segment
        float acc = *cell;
#pragma unroll
        for (int r = 0; r < 8; r++) {
          const int i = f_rel0 + r;
          if (r < f_nloops && i >= 0 && i < KT) acc += pst[f_tk * PLD + i] * f_w[r];
        }
        *cell = acc;
      }
    } else {
      const int j_lo = (St * kt) / Bs;
      const int j_hi = min((St * (kt + KT - 1) + Kz - 1) / Bs, nb_max - 1);
      const int nj = j_hi - j_lo + 1;
      for (int it = tid; it < TWG * nj; it += 256) {
        int tk = it / nj;
        int j = j_lo + (it - tk * nj);
        int i0 = (j * Bs - Kz) / St + 1;  // exact: block and kernel sizes are multiples of the stride
        float acc = imp_all[tk * nb_max + j];
        int cs = St - Kz;
        for (int r = 0; r < f_nloops; r++, cs += St) {
          int i = i0 + r;
          if (i >= kt && i < kt + KT) {
            int area = min(cs + Kz, Bs) - max(cs, 0);
            acc += pst[tk * PLD + (i - kt)] * ((float)area / (float)St);
          }
        }
        imp_all[tk * nb_max + j] = acc;
      }
    }
    // ---- segmented mode: at the end of a segment merge its finished blocks into the running winners ----
    if (seg > 0 && ((tile + 1) % tiles_per_seg == 0 || tile == ntiles - 1)) {
      const bool last = tile == ntiles - 1;
      const int count = last ? W : seg;
      __syncthreads();  // the fold of this tile is complete
      for (int tk = wave; tk < TWG; tk += 4) {
        const int n = n0 + tk;
        if (n >= xl) break;
        float* row = imp_all + tk * W;
        const int64_t tok = x0 + n;
        if (p.imp_out != nullptr) {
          float* dst = p.imp_out + (int64_t)kh * p.imp_sh + tok * p.imp_st;
          for (int jj = lane; jj < count; jj += 64)
            if (j0 + jj < p.imp_cols) dst[j0 + jj] = j0 + jj < nb_max ? row[jj] : 0.f;
          if (last)
            for (int j = j0 + count + lane; j < p.imp_cols; j += 64) dst[j] = 0.f;
        }
        const float carry = row[seg];
        const int win = merge_segment(row, count, j0, cand_s_all + tk * ncand, cand_i_all + tk * ncand, ncand, j0 == 0,
                                      n + qoff, nb_max, p, lane);
        if (last) {
          const int t = n + qoff, nk = t / Bs;
          const int nsel = min(p.top_n, nk + 1), forced = p.num_init + p.num_local;
          int result = p.ignore_index;
          if (lane < p.num_init) {
            if (lane <= nk) result = lane;
          } else if (lane < forced) {
            if (lane <= nk) result = nk - (lane - p.num_init);
          }
          const int from_list = __shfl(win, max(lane - forced, 0));
          if (lane >= forced && lane < nsel) result = from_list;
          if (lane < p.top_n) p.topk[(int64_t)kh * p.tk_sh + tok * p.tk_st + lane] = result;
        } else {  // next segment: its first block keeps what this segment's last tile already added to it
          for (int jj = lane; jj < W; jj += 64) row[jj] = jj == 0 ? carry : 0.f;
        }
      }
      j0 += seg;
      __syncthreads();
    }
  }
  __syncthreads();
  if (seg > 0) {
    // a workgroup without any visible compressed key: forced blocks only
    if (ntiles == 0)
      for (int tk = wave; tk < TWG; tk += 4) {
        const int n = n0 + tk;
        if (n >= xl) break;
        const int nk = (n + qoff) / Bs;
        int result = p.ignore_index;
        if (lane < p.num_init) {
          if (lane <= nk) result = lane;
        } else if (lane < p.num_init + p.num_local) {
          if (lane <= nk) result = nk - (lane - p.num_init);
        }
        const int64_t tok = x0 + n;
        if (lane < p.top_n) p.topk[(int64_t)kh * p.tk_sh + tok * p.tk_st + lane] = result;
        if (p.imp_out != nullptr)
          for (int j = lane; j < p.imp_cols; j += 64) p.imp_out[(int64_t)kh * p.imp_sh + tok * p.imp_st + j] = 0.f;
      }
    return;
  }

  // ---- selection: the tokens of the workgroup are dealt to the waves ----
  for (int tk = wave; tk < TWG; tk += 4) {
    const int n = n0 + tk;
    if (n >= xl) break;
    const int t = n + qoff;
    float* imp = imp_all + tk * nb_max;
    const int64_t tok = x0 + n;
    if (p.imp_out != nullptr) {
      for (int j = lane; j < p.imp_cols; j += 64)
        p.imp_out[(int64_t)kh * p.imp_sh + tok * p.imp_st + j] = j < nb_max ? imp[j] : 0.f;
    }
    const int result = nb_max <= 1024 ? select_row<true>(imp, t, nb_max, p, lane) : select_row<false>(imp, t, nb_max, p, lane);
    if (lane < p.top_n) p.topk[(int64_t)kh * p.tk_sh + tok * p.tk_st + lane] = result;
  }
}

template <int D, int GP, bool PAGED>
int launch_topk(const NsaTopkParams& p_in, int B, int max_q_len, hipStream_t stream) {
  constexpr int TWG = 2 * (32 / GP);
  NsaTopkParams p = p_in;
  const size_t stat = 128 * (D + NSA_LDS_PAD) * 2 + 2 * TWG * 132 * 4;
  // One pass while the score rows of all blocks leave room for two workgroups per CU; else segments of the largest
  // whole number of key tiles that does.  The tuning value topk_seg_blocks forces a segment length (0 = never segment).
  const int forced_seg = nsa_tuning_knob("topk_seg_blocks", -1);
  const size_t budget = 80 * 1024;
  size_t dyn = (size_t)TWG * p.nb_max * sizeof(float);
  p.seg_blocks = 0;
  const int tile_span = p.stride * 128;  // positions covered by a 128-key tile
  const bool aligned = tile_span % p.block_size == 0 && (p.block_size + p.kernel_size - p.stride) / p.stride <= 8 &&
                       TWG * ((p.stride * 127 + p.kernel_size - 1) / p.block_size + 1) <= 256;
  const bool want_seg = forced_seg > 0 || (forced_seg < 0 && dyn + stat > budget);
  if (want_seg && aligned) {
    const int bpt = tile_span / p.block_size;  // selection blocks per key tile
    const int ncand = p.top_n - p.num_init - p.num_local > 0 ? p.top_n - p.num_init - p.num_local : 0;
    const size_t fixed = stat + (size_t)TWG * ncand * 8 + (size_t)TWG * 4;
    int seg = forced_seg > 0 ? forced_seg : (fixed < budget ? (int)((budget - fixed) / (TWG * 4)) : bpt);
    seg = seg / bpt * bpt;
    if (seg < bpt) seg = bpt;
    if (seg < p.nb_max) {
      p.seg_blocks = seg;
      dyn = (size_t)TWG * (seg + 1) * sizeof(float) + (size_t)TWG * ncand * 8;
    }
  }
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
  if (D == 256) return paged ? dispatch_gp<256, true>(p, B, max_q_len, stream) : dispatch_gp<256, false>(p, B, max_q_len, stream);
  if (D == 32) return paged ? dispatch_gp<32, true>(p, B, max_q_len, stream) : dispatch_gp<32, false>(p, B, max_q_len, stream);
  nsa_set_error("top-k: unsupported head dim D=%d", D);
  return NSA_ERR_UNSUPPORTED;
}

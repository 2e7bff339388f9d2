// dK / dV of all three attention branches.  A workgroup owns NW*32 keys (each wave 32 keys whose K and V
// fragments stay in registers as MFMA B operands) and streams tiles of 64 query rows through LDS; a "row" is a
// (query token, q-head) pair of the kv-head group, so the GQA reduction over heads happens in the accumulators.
//   S = Q K^T,  P = exp2(S*c - lse),  dP = dO V^T,  dS = P o (dP - delta),
//   dV^T += dO^T P,  dK^T += Q^T dS      (Q^T / dO^T fragments via ds_read_b64_tr_b16)
// MODE_CMP: rows are all later queries of the sequence, split in chunks over grid.x, fp32 atomics
//           (upstream flash_nsa/ops/compress_attn.py:193-376)
// MODE_SWA: rows are the <= W+NW*32 queries whose window contains the keys, plain stores
//           (upstream: FlashAttention backward, flash_nsa/ops/sliding_window_attention.py:98-157)
// MODE_SLC: rows are gathered through the inverse index (selection block -> tokens that selected it), lists are
//           cut into chunks over grid.x, fp32 atomics (upstream flash_nsa/ops/select_attn.py:147-328)
#include "nsa_common.h"
#include "nsa_api_internal.h"

namespace {

constexpr int MODE_CMP = 0;
constexpr int MODE_SWA = 1;
constexpr int MODE_SLC = 2;

template <int D, int VD, int MODE, int NW, int KB>
__global__ __launch_bounds__(NW * 64) void bwd_dkdv_kernel(NsaBwdTileParams p) {
  constexpr int NT = NW * 64;
  constexpr int KPW = 32 * KB;   // keys per wave: KB blocks of 32, every Q / dO fragment read from LDS serves KB MFMAs
  constexpr int KW = NW * KPW;
  constexpr int RT = KB > 1 ? 32 : 64;  // query rows per tile
  constexpr int QLD = D + NSA_LDS_PAD;
  constexpr int OLD = VD + NSA_LDS_PAD;
  constexpr int T_INVALID = -0x40000000;
  __shared__ __attribute__((aligned(16))) bf16_t Qs[RT * QLD];
  __shared__ __attribute__((aligned(16))) bf16_t dOs[RT * OLD];
  __shared__ __attribute__((aligned(16))) float lse_s[RT];
  __shared__ __attribute__((aligned(16))) float delta_s[RT];
  __shared__ __attribute__((aligned(16))) int t_s[RT];
  // KB > 1: the V rows of the workgroup's keys live in LDS (dP = dO V^T reads its B fragments from there), which
  // leaves the registers to the 2*KB accumulator blocks and the K fragments
  constexpr bool V_LDS = KB > 1;
  __shared__ __attribute__((aligned(16))) bf16_t Vk[V_LDS ? KW * OLD : 8];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int hl = lane >> 5;
  const int g16 = lane >> 4, i16 = lane & 15;
  const int kh = blockIdx.z;
  const int G = p.G;
  const int gshift = (G & (G - 1)) == 0 ? __builtin_ctz(G) : -1;  // power-of-two groups avoid the division

  int b, key0, row_begin, row_end;  // rows in the group-row space of sequence b (MODE_SLC: positions in the list)
  const int32_t* list = nullptr;
  if (MODE == MODE_SLC) {
    const int32_t* ioff = p.item_off + (int64_t)kh * (p.nblk_total + 1);
    const int w = blockIdx.x;
    if (w >= ioff[p.nblk_total]) return;
    int lo = 0, hi = p.nblk_total;  // last jb with ioff[jb] <= w
    while (hi - lo > 1) {
      int mid = (lo + hi) >> 1;
      if (ioff[mid] <= w) lo = mid; else hi = mid;
    }
    const int jb = lo;
    const int c = w - ioff[jb];
    b = p.blk_seq[jb];
    // a selection block wider than the workgroup's NW*32 keys is cut into sub-blocks over grid.y (same token list)
    key0 = (jb - p.kblk_cu[b]) * p.block_size + blockIdx.y * (NW * 32 * KB);
    const int s0 = p.csr_off[(int64_t)kh * (p.nblk_total + 1) + jb];
    const int s1 = p.csr_off[(int64_t)kh * (p.nblk_total + 1) + jb + 1];
    const int a = s0 + c * p.chunk_tokens;
    list = p.csr_tok + a;
    row_begin = 0;
    row_end = (min(s1, a + p.chunk_tokens) - a) * G;
  } else {
    b = blockIdx.y;
  }
  const int x0 = p.x_cu[b];
  const int xl = p.x_cu[b + 1] - x0;
  int nkeys, kbase;
  if (MODE == MODE_CMP) {
    kbase = p.k_cu[b];
    nkeys = p.k_cu[b + 1] - kbase;
    // blockIdx.x enumerates only the (key tile, query chunk) pairs that have visible rows, key-tile major, so
    // that consecutive workgroups (which the dispatcher deals round-robin to the XCDs) carry equal work
    const int nch = cdiv_i(xl, p.q_chunk_tokens);
    int rem = blockIdx.x, ktile = 0, ch = -1;
    for (; ktile * KW < nkeys; ktile++) {
      const int fc = min(nch, (p.stride * ktile * KW + p.kernel_size - 1) / p.q_chunk_tokens);
      const int cnt = nch - fc;
      if (rem < cnt) { ch = fc + rem; break; }
      rem -= cnt;
    }
    if (ch < 0) return;
    key0 = ktile * KW;
    const int first = p.stride * key0 + p.kernel_size - 1;
    const int ta = max(ch * p.q_chunk_tokens, first);
    const int tb = min((ch + 1) * p.q_chunk_tokens, xl);
    if (ta >= tb) return;
    row_begin = ta * G;
    row_end = tb * G;
  } else {
    kbase = x0;
    nkeys = xl;
    // MODE_SLC: the workgroup's keys end with its selection block (a block narrower than NW*32 keys, or the last
    // sub-block of a wide one, leaves the upper waves without keys)
    if (MODE == MODE_SLC) nkeys = min(xl, (key0 / p.block_size + 1) * p.block_size);
    if (MODE == MODE_SWA) {
      key0 = blockIdx.x * KW;
      if (key0 >= nkeys) return;
      row_begin = key0 * G;
      row_end = min(xl, key0 + KW + p.window) * G;
    } else if (key0 >= nkeys) {
      return;
    }
  }
  if (row_begin >= row_end) return;

  // ---- this wave's keys: K and V fragments as B operands ----
  const int kw0 = key0 + wave * KPW;
  bf16x8 kf[KB][D / 16], vf[V_LDS ? 1 : KB][VD / 16];
#pragma unroll
  for (int kb = 0; kb < KB; kb++) {
    const int kr = min(kw0 + kb * 32 + l32, nkeys - 1);
    const bf16_t* kp = p.k + ((int64_t)kbase + kr) * p.k_sr + (int64_t)kh * p.k_sh + hl * 8;
#pragma unroll
    for (int kc = 0; kc < D / 16; kc++) kf[kb][kc] = ld_global_b128(kp + kc * 16);
    if (!V_LDS) {
      const bf16_t* vp = p.v + ((int64_t)kbase + kr) * p.v_sr + (int64_t)kh * p.v_sh + hl * 8;
#pragma unroll
      for (int kc = 0; kc < VD / 16; kc++) vf[kb][kc] = ld_global_b128(vp + kc * 16);
    }
  }
  if (V_LDS) {
    constexpr int VP = VD / 8;
    for (int pc = tid; pc < KW * VP; pc += NT) {
      const int kr = min(key0 + pc / VP, nkeys - 1);
      *reinterpret_cast<bf16x8*>(&Vk[(pc / VP) * OLD + (pc % VP) * 8]) =
          ld_global_b128(p.v + ((int64_t)kbase + kr) * p.v_sr + (int64_t)kh * p.v_sh + (pc % VP) * 8);
    }
  }
  f32x16 dkacc[KB][D / 32], dvacc[KB][VD / 32];
#pragma unroll
  for (int kb = 0; kb < KB; kb++) {
#pragma unroll
    for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
      for (int i = 0; i < 16; i++) dkacc[kb][dt][i] = 0.f;
#pragma unroll
    for (int dt = 0; dt < VD / 32; dt++)
#pragma unroll
      for (int i = 0; i < 16; i++) dvacc[kb][dt][i] = 0.f;
  }
  const float sc = p.scale_log2;
  const bool wave_has_keys = kw0 < nkeys;

  // ---- software pipeline over 64-row tiles: registers hold the next tile while the current one is computed.
  // Rows past the end of the range are replaced by the last valid row and flagged with an invalid position,
  // which zeroes their probabilities.
  constexpr int QP = D / 8, OP = VD / 8;
  constexpr int QJ = (RT * QP) / NT, OJ = (RT * OP) / NT;
  bf16x8 qreg[QJ], oreg[OJ];
  float lse_reg = 0.f, delta_reg = 0.f;
  int t_reg = T_INVALID;
  // Per-thread row bookkeeping.  A thread stages the same tile-relative rows every iteration, so when G is a power
  // of two dividing 64 its (token index, head) pairs advance by a constant per tile and no division is needed in
  // the loop; other group sizes recompute the pair each time.
  const bool fastG = gshift >= 0 && G <= RT;
  const int n_step = fastG ? (RT >> gshift) : 0;
  const int row_last = row_end - 1;
  auto split_row = [&](int rr, int& n, int& g) {
    if (gshift >= 0) { n = rr >> gshift; g = rr & (G - 1); }
    else { n = rr / G; g = rr - n * G; }
  };
  int n_lastrow, g_lastrow;
  split_row(row_last, n_lastrow, g_lastrow);
  int qn[QJ], on[OJ], sn;                 // token index (MODE_SLC: list position) of the thread's rows, current tile
  int64_t qoffs[QJ], ooffs[OJ];           // head + channel offsets (elements)
  int sg;
#pragma unroll
  for (int j = 0; j < QJ; j++) {
    int pc = tid + j * NT, g;
    split_row(row_begin + pc / QP, qn[j], g);
    qoffs[j] = (int64_t)(kh * G + g) * p.q_sh + (pc % QP) * 8;
  }
#pragma unroll
  for (int j = 0; j < OJ; j++) {
    int pc = tid + j * NT, g;
    split_row(row_begin + pc / OP, on[j], g);
    ooffs[j] = (int64_t)(kh * G + g) * p.do_sh + (pc % OP) * 8;
  }
  split_row(row_begin + (tid & (RT - 1)), sn, sg);
  const int64_t qoff_last = (int64_t)(kh * G + g_lastrow) * p.q_sh;
  const int64_t ooff_last = (int64_t)(kh * G + g_lastrow) * p.do_sh;
  // (token index or list position, head+channel offset) of tile-relative row `rowrel` for the tile starting at rt0
  auto locate = [&](int rt0, int rowrel, int n_inc, int64_t off_inc, int64_t off_last, int chan, int64_t hstride,
                    int& n, int64_t& off) {
    if (!fastG) {
      int g;
      split_row(min(rt0 + rowrel, row_last), n, g);
      off = (int64_t)(kh * G + g) * hstride + chan;
    } else if (rt0 + rowrel > row_last) {
      n = n_lastrow;
      off = off_last + chan;
    } else {
      n = n_inc;
      off = off_inc;
    }
  };
  // MODE_SLC: tokens of the NEXT tile to load, fetched from the inverse-index list one tile ahead of their use so
  // that the dependent (list -> row) lookups never stall the pipeline
  int tq[QJ], to[OJ], tsn = 0;
  // When a thread's rows of one load step (NT / QP consecutive rows) never straddle a token, the token of load step
  // j is the same for every thread of the workgroup: the list entries become scalar loads, the row addresses one
  // scalar base per step plus a per-thread byte offset that never changes, and the (list position -> token -> 64-bit
  // address) arithmetic leaves the vector unit.
  // (the per-thread offsets are kept as 32-bit byte offsets: head strides beyond that take the general path)
  const bool off32 = ((int64_t)(kh * G + G) * p.q_sh + D) * 2 < ((int64_t)1 << 32) &&
                     ((int64_t)(kh * G + G) * p.do_sh + VD) * 2 < ((int64_t)1 << 32) && p.q_sh >= 0 && p.do_sh >= 0;
  // (a head dim of 192 has 24 chunks per row, which do not divide the thread count: its load steps straddle tokens)
  constexpr bool steps_whole_rows = (NT % QP == 0) && (NT % OP == 0);
  const bool tok_uniform = MODE == MODE_SLC && steps_whole_rows && fastG && (NT / QP) <= G && G % (NT / QP) == 0 &&
                           (NT / OP) <= G && G % (NT / OP) == 0 && off32;
  uint32_t qoff_b[QJ], ooff_b[OJ];
#pragma unroll
  for (int j = 0; j < QJ; j++) qoff_b[j] = (uint32_t)(qoffs[j] * 2);
#pragma unroll
  for (int j = 0; j < OJ; j++) ooff_b[j] = (uint32_t)(ooffs[j] * 2);
  auto fetch_tokens = [&](int rt0) {
    if (MODE != MODE_SLC) return;
    if (tok_uniform) {
      const int n0 = rt0 >> gshift;
#pragma unroll
      for (int j = 0; j < QJ; j++)
        tq[j] = __builtin_amdgcn_readfirstlane(list[min(n0 + ((j * (NT / QP)) >> gshift), n_lastrow)]);
      if (QP != OP) {
#pragma unroll
        for (int j = 0; j < OJ; j++)
          to[j] = __builtin_amdgcn_readfirstlane(list[min(n0 + ((j * (NT / OP)) >> gshift), n_lastrow)]);
      }
      if (tid < RT) tsn = list[min(n0 + (tid >> gshift), n_lastrow)];
      return;
    }
#pragma unroll
    for (int j = 0; j < QJ; j++) {
      int pc = tid + j * NT, n;
      int64_t off;
      locate(rt0, pc / QP, qn[j], 0, 0, 0, 0, n, off);
      tq[j] = list[n];
    }
    if (QP != OP) {
#pragma unroll
      for (int j = 0; j < OJ; j++) {
        int pc = tid + j * NT, n;
        int64_t off;
        locate(rt0, pc / OP, on[j], 0, 0, 0, 0, n, off);
        to[j] = list[n];
      }
    }
    if (tid < RT) {
      int n;
      int64_t off;
      locate(rt0, tid, sn, 0, 0, 0, 0, n, off);
      tsn = list[n];
    }
  };
  // Range-keyed modes with a power-of-two group: a thread's rows advance by a whole number of tokens per tile, so
  // its global addresses advance by a constant; the loop then needs one 64-bit add per load instead of the
  // (token, head) -> address arithmetic.  Partial tiles (only the last one) take the general path.
  const bool ptr_mode = (MODE != MODE_SLC) && fastG;
  const bf16_t* qptr[QJ];
  const bf16_t* optr[OJ];
  const float* lptr = p.lse;
  const float* dptr = p.delta;
  if (ptr_mode) {
#pragma unroll
    for (int j = 0; j < QJ; j++) qptr[j] = p.q + (int64_t)(x0 + qn[j]) * p.q_st + qoffs[j];
#pragma unroll
    for (int j = 0; j < OJ; j++) optr[j] = p.dO + (int64_t)(x0 + on[j]) * p.do_st + ooffs[j];
    lptr = p.lse + (int64_t)(x0 + sn) * p.lse_st + (int64_t)(kh * G + sg) * p.lse_sh;
    dptr = p.delta + (int64_t)(x0 + sn) * p.delta_st + (int64_t)(kh * G + sg) * p.delta_sh;
  }
  const int64_t q_step = (int64_t)n_step * p.q_st, o_step = (int64_t)n_step * p.do_st;
  const int64_t l_step = (int64_t)n_step * p.lse_st, d_step = (int64_t)n_step * p.delta_st;
  auto gload = [&](int rt0) {
    if (ptr_mode && rt0 + RT <= row_end) {
#pragma unroll
      for (int j = 0; j < QJ; j++) qreg[j] = ld_global_b128(qptr[j]);
#pragma unroll
      for (int j = 0; j < OJ; j++) oreg[j] = ld_global_b128(optr[j]);
      if (tid < RT) {
        lse_reg = *lptr;
        delta_reg = *dptr;
        t_reg = sn;
      }
    } else if (tok_uniform) {
#pragma unroll
      for (int j = 0; j < QJ; j++)
        qreg[j] = *reinterpret_cast<const bf16x8*>(
            reinterpret_cast<const char*>(p.q + (int64_t)(x0 + tq[j]) * p.q_st) + qoff_b[j]);
#pragma unroll
      for (int j = 0; j < OJ; j++)
        oreg[j] = *reinterpret_cast<const bf16x8*>(
            reinterpret_cast<const char*>(p.dO + (int64_t)(x0 + ((QP == OP) ? tq[j] : to[j])) * p.do_st) + ooff_b[j]);
      if (tid < RT) {
        const bool ok = rt0 + tid <= row_last;
        const int64_t tok = x0 + tsn;
        const int64_t hoff = kh * G + (tid & (G - 1));
        lse_reg = p.lse[tok * p.lse_st + hoff * p.lse_sh];
        delta_reg = p.delta[tok * p.delta_st + hoff * p.delta_sh];
        t_reg = ok ? tsn : T_INVALID;
      }
    } else {
#pragma unroll
      for (int j = 0; j < QJ; j++) {
        int pc = tid + j * NT, n;
        int64_t off;
        locate(rt0, pc / QP, qn[j], qoffs[j], qoff_last, (pc % QP) * 8, p.q_sh, n, off);
        if (MODE == MODE_SLC) n = tq[j];
        qreg[j] = ld_global_b128(p.q + (int64_t)(x0 + n) * p.q_st + off);
      }
#pragma unroll
      for (int j = 0; j < OJ; j++) {
        int pc = tid + j * NT, n;
        int64_t off;
        locate(rt0, pc / OP, on[j], ooffs[j], ooff_last, (pc % OP) * 8, p.do_sh, n, off);
        if (MODE == MODE_SLC) n = (QP == OP) ? tq[j] : to[j];
        oreg[j] = ld_global_b128(p.dO + (int64_t)(x0 + n) * p.do_st + off);
      }
      if (tid < RT) {
        const bool ok = rt0 + tid <= row_last;
        int n;
        int64_t hoff;
        locate(rt0, tid, sn, (int64_t)(kh * G + sg), (int64_t)(kh * G + g_lastrow), 0, 1, n, hoff);
        if (MODE == MODE_SLC) n = tsn;
        const int64_t tok = x0 + n;
        lse_reg = p.lse[tok * p.lse_st + hoff * p.lse_sh];
        delta_reg = p.delta[tok * p.delta_st + hoff * p.delta_sh];
        t_reg = ok ? n : T_INVALID;
      }
    }
    // advance the bookkeeping to the next tile, then start fetching that tile's tokens
#pragma unroll
    for (int j = 0; j < QJ; j++) qn[j] += n_step;
#pragma unroll
    for (int j = 0; j < OJ; j++) on[j] += n_step;
    sn += n_step;
    if (ptr_mode) {
#pragma unroll
      for (int j = 0; j < QJ; j++) qptr[j] += q_step;
#pragma unroll
      for (int j = 0; j < OJ; j++) optr[j] += o_step;
      lptr += l_step;
      dptr += d_step;
    }
    if (rt0 + RT < row_end) fetch_tokens(rt0 + RT);
  };
  fetch_tokens(row_begin);
  gload(row_begin);

  for (int rt0 = row_begin; rt0 < row_end; rt0 += RT) {
    __syncthreads();
#pragma unroll
    for (int j = 0; j < QJ; j++) {
      int pc = tid + j * NT;
      *reinterpret_cast<bf16x8*>(&Qs[(pc / QP) * QLD + (pc % QP) * 8]) = qreg[j];
    }
#pragma unroll
    for (int j = 0; j < OJ; j++) {
      int pc = tid + j * NT;
      *reinterpret_cast<bf16x8*>(&dOs[(pc / OP) * OLD + (pc % OP) * 8]) = oreg[j];
    }
    if (tid < RT) {
      lse_s[tid] = lse_reg;
      delta_s[tid] = delta_reg;
      t_s[tid] = t_reg;
    }
    __syncthreads();
    if (rt0 + RT < row_end) gload(rt0 + RT);
    if (!wave_has_keys) continue;

    // tile position range (rows ascend in position for all three modes); scalar values
    const int n_in = min(RT, row_end - rt0);
    const int t_min = __builtin_amdgcn_readfirstlane(t_s[0]);
    const int t_max = __builtin_amdgcn_readfirstlane(t_s[n_in - 1]);
    bool any_vis, full_vis;
    constexpr int KL = KPW - 1;  // offset of the wave's last key
    if (MODE == MODE_CMP) {
      any_vis = t_max >= p.stride * kw0 + p.kernel_size - 1;
      full_vis = (n_in == RT) && (t_min >= p.stride * (kw0 + KL) + p.kernel_size - 1) && (kw0 + KL < nkeys);
    } else if (MODE == MODE_SWA) {
      any_vis = (kw0 <= t_max) && (kw0 + KL >= t_min - p.window);
      full_vis = (n_in == RT) && (kw0 + KL <= t_min) && (kw0 >= t_max - p.window) && (kw0 + KL < nkeys);
    } else {
      any_vis = kw0 <= t_max;
      full_vis = (n_in == RT) && (kw0 + KL <= t_min) && (kw0 + KL < nkeys);
    }
    if (!any_vis) continue;

#pragma unroll
    for (int mt = 0; mt < RT / 32; mt++) {
      f32x16 sacc[KB], pacc[KB];
#pragma unroll
      for (int kb = 0; kb < KB; kb++)
#pragma unroll
        for (int i = 0; i < 16; i++) { sacc[kb][i] = 0.f; pacc[kb][i] = 0.f; }
      const bf16_t* qp = &Qs[(mt * 32 + l32) * QLD + hl * 8];
      const bf16_t* dp = &dOs[(mt * 32 + l32) * OLD + hl * 8];
#pragma unroll
      for (int kc = 0; kc < D / 16; kc++) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(qp + kc * 16);
#pragma unroll
        for (int kb = 0; kb < KB; kb++) sacc[kb] = mfma32(a, kf[kb][kc], sacc[kb]);
      }
#pragma unroll
      for (int kc = 0; kc < VD / 16; kc++) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(dp + kc * 16);
#pragma unroll
        for (int kb = 0; kb < KB; kb++) {
          if (V_LDS) {
            const bf16x8 bv =
                *reinterpret_cast<const bf16x8*>(&Vk[(wave * KPW + kb * 32 + l32) * OLD + hl * 8 + kc * 16]);
            pacc[kb] = mfma32(a, bv, pacc[kb]);
          } else {
            pacc[kb] = mfma32(a, vf[kb][kc], pacc[kb]);
          }
        }
      }
      // P = exp2(S*c - lse);  dS = P o (dP - delta)
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        const int rbase = mt * 32 + i4 * 8 + hl * 4;
        f32x4 l4 = *reinterpret_cast<const f32x4*>(&lse_s[rbase]);
#pragma unroll
        for (int kb = 0; kb < KB; kb++)
#pragma unroll
          for (int ii = 0; ii < 4; ii++)
            sacc[kb][i4 * 4 + ii] = fast_exp2(__builtin_fmaf(sacc[kb][i4 * 4 + ii], sc, -l4[ii]));
      }
      if (!full_vis) {  // wave-uniform: only tiles that straddle a visibility boundary pay for the mask
#pragma unroll
        for (int i4 = 0; i4 < 4; i4++) {
          const int rbase = mt * 32 + i4 * 8 + hl * 4;
#pragma unroll
          for (int ii = 0; ii < 4; ii++) {
            int tr = t_s[rbase + ii];
#pragma unroll
            for (int kb = 0; kb < KB; kb++) {
              const int my_key = kw0 + kb * 32 + l32;
              bool vis;
              if (MODE == MODE_CMP) vis = (my_key < nkeys) && (tr >= p.stride * my_key + p.kernel_size - 1);
              else if (MODE == MODE_SWA) vis = (my_key <= tr) && (my_key >= tr - p.window) && (my_key < nkeys);
              else vis = (my_key <= tr) && (my_key < nkeys);
              sacc[kb][i4 * 4 + ii] = vis ? sacc[kb][i4 * 4 + ii] : 0.f;
            }
          }
        }
      }
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        const int rbase = mt * 32 + i4 * 8 + hl * 4;
        f32x4 d4 = *reinterpret_cast<const f32x4*>(&delta_s[rbase]);
#pragma unroll
        for (int kb = 0; kb < KB; kb++)
#pragma unroll
          for (int ii = 0; ii < 4; ii++)
            pacc[kb][i4 * 4 + ii] = sacc[kb][i4 * 4 + ii] * (pacc[kb][i4 * 4 + ii] - d4[ii]);
      }
#pragma unroll
      for (int c = 0; c < 2; c++) {
        bf16x8 pf[KB], df[KB];
#pragma unroll
        for (int kb = 0; kb < KB; kb++) {
          pf[kb] = pack8(sacc[kb][c * 8 + 0], sacc[kb][c * 8 + 1], sacc[kb][c * 8 + 2], sacc[kb][c * 8 + 3],
                         sacc[kb][c * 8 + 4], sacc[kb][c * 8 + 5], sacc[kb][c * 8 + 6], sacc[kb][c * 8 + 7]);
          df[kb] = pack8(pacc[kb][c * 8 + 0], pacc[kb][c * 8 + 1], pacc[kb][c * 8 + 2], pacc[kb][c * 8 + 3],
                         pacc[kb][c * 8 + 4], pacc[kb][c * 8 + 5], pacc[kb][c * 8 + 6], pacc[kb][c * 8 + 7]);
        }
        const int rb0 = mt * 32 + (2 * c) * 8 + hl * 4 + (i16 >> 2);
        const int rb1 = rb0 + 8;
#pragma unroll
        for (int dt = 0; dt < VD / 32; dt++) {
          const int col = dt * 32 + (g16 & 1) * 16 + 4 * (i16 & 3);
          bf16x4 a0 = lds_read_tr(&dOs[rb0 * OLD + col]);
          bf16x4 a1 = lds_read_tr(&dOs[rb1 * OLD + col]);
#pragma unroll
          for (int kb = 0; kb < KB; kb++) dvacc[kb][dt] = mfma32(cat4(a0, a1), pf[kb], dvacc[kb][dt]);
        }
#pragma unroll
        for (int dt = 0; dt < D / 32; dt++) {
          const int col = dt * 32 + (g16 & 1) * 16 + 4 * (i16 & 3);
          bf16x4 a0 = lds_read_tr(&Qs[rb0 * QLD + col]);
          bf16x4 a1 = lds_read_tr(&Qs[rb1 * QLD + col]);
#pragma unroll
          for (int kb = 0; kb < KB; kb++) dkacc[kb][dt] = mfma32(cat4(a0, a1), df[kb], dkacc[kb][dt]);
        }
      }
    }
  }

  const float osc = p.sm_scale;
  // dkv_mode 4: the workgroup's own slot of the partial buffers (summed in a fixed order by a second kernel)
  int64_t slot = 0;
  if (MODE == MODE_CMP) slot = ((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * p.KH + kh;
  else if (MODE == MODE_SLC) slot = ((int64_t)kh * gridDim.x + blockIdx.x) * gridDim.y + blockIdx.y;
  auto emit = [&](void* base, int64_t off, f32x4 val) {
    if (p.dkv_mode == 0) {
      *reinterpret_cast<bf16x4*>((bf16_t*)base + off) = pack4(val[0], val[1], val[2], val[3]);
    } else if (p.dkv_mode == 1 || p.dkv_mode == 4) {
      *reinterpret_cast<f32x4*>((float*)base + off) = val;
    } else {
      float* dst = (float*)base + off;
#pragma unroll
      for (int e = 0; e < 4; e++) unsafeAtomicAdd(dst + e, val[e]);
    }
  };
#pragma unroll
  for (int kb = 0; kb < KB; kb++) {
    const int my_key = kw0 + kb * 32 + l32;
    if (my_key >= nkeys) continue;
    int64_t koff = ((int64_t)kbase + my_key) * p.dk_sr + (int64_t)kh * p.dk_sh;
    int64_t voff = ((int64_t)kbase + my_key) * p.dv_sr + (int64_t)kh * p.dv_sh;
    void* dk_base = p.dk;
    void* dv_base = p.dv;
    if (p.dkv_mode == 4) {
      koff = (slot * KW + (my_key - key0)) * D;
      voff = (slot * KW + (my_key - key0)) * VD;
      dk_base = p.part_dk;
      dv_base = p.part_dv;
    }
#pragma unroll
    for (int dt = 0; dt < D / 32; dt++)
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        int d = dt * 32 + i4 * 8 + hl * 4;
        emit(dk_base, koff + d, f32x4{dkacc[kb][dt][i4 * 4 + 0] * osc, dkacc[kb][dt][i4 * 4 + 1] * osc,
                                   dkacc[kb][dt][i4 * 4 + 2] * osc, dkacc[kb][dt][i4 * 4 + 3] * osc});
      }
#pragma unroll
    for (int dt = 0; dt < VD / 32; dt++)
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        int d = dt * 32 + i4 * 8 + hl * 4;
        emit(dv_base, voff + d, f32x4{dvacc[kb][dt][i4 * 4 + 0], dvacc[kb][dt][i4 * 4 + 1], dvacc[kb][dt][i4 * 4 + 2],
                                   dvacc[kb][dt][i4 * 4 + 3]});
      }
  }
}

template <int D, int VD>
int launch(const NsaBwdTileParams& p0, int mode, int B, int max_q_len, int max_k_len, int n_items_bound,
           hipStream_t stream) {
  NsaBwdTileParams p = p0;
  // the variant with two 32-key blocks per wave exists for the head dims it was measured on
  constexpr bool KB2_BUILT = D >= 64 && D <= 192;
  const int kb_cmp = KB2_BUILT ? nsa_tuning_knob("dkdv_key_blocks", 1) : 1;  // 32-key blocks per wave (cmp / swa)
  if (mode == MODE_CMP) {
    if (B <= 0 || max_k_len <= 0) return NSA_OK;
    const int KW = 4 * 32 * (kb_cmp == 2 ? 2 : 1);
    const int nch = cdiv_i(max_q_len, p.q_chunk_tokens);
    int total = 0;
    for (int kt = 0; kt * KW < max_k_len; kt++) {
      const int fc = (p.stride * kt * KW + p.kernel_size - 1) / p.q_chunk_tokens;
      total += nch - (nch < fc ? nch : fc);
    }
    if (total <= 0) return NSA_OK;
    dim3 grid(total, B, p.KH);
    if constexpr (KB2_BUILT) {
      if (kb_cmp == 2) bwd_dkdv_kernel<D, VD, MODE_CMP, 4, 2><<<grid, 256, 0, stream>>>(p);
      else bwd_dkdv_kernel<D, VD, MODE_CMP, 4, 1><<<grid, 256, 0, stream>>>(p);
    } else {
      bwd_dkdv_kernel<D, VD, MODE_CMP, 4, 1><<<grid, 256, 0, stream>>>(p);
    }
  } else if (mode == MODE_SWA) {
    if (B <= 0 || max_k_len <= 0) return NSA_OK;
    if constexpr (KB2_BUILT) {
      if (kb_cmp == 2) {
        dim3 grid(cdiv_i(max_k_len, 256), B, p.KH);
        bwd_dkdv_kernel<D, VD, MODE_SWA, 4, 2><<<grid, 256, 0, stream>>>(p);
        return nsa_check_launch("bwd_dkdv_kernel");
      }
    }
    dim3 grid(cdiv_i(max_k_len, 128), B, p.KH);
    bwd_dkdv_kernel<D, VD, MODE_SWA, 4, 1><<<grid, 256, 0, stream>>>(p);
  } else {
    if (n_items_bound <= 0) return NSA_OK;
    if (p.block_size <= 0 || p.block_size % 32 != 0) {
      nsa_set_error("selected attention dk/dv: block_size %d must be a multiple of 32", p.block_size);
      return NSA_ERR_UNSUPPORTED;
    }
    // a workgroup owns 64 keys (blocks of 32 or 64) or 128 keys (wider blocks, cut into sub-blocks over grid.y);
    // waves whose 32 keys lie past the end of the block only help staging the query rows
    if (p.block_size <= 64) {
      dim3 grid(n_items_bound, 1, p.KH);
      bwd_dkdv_kernel<D, VD, MODE_SLC, 2, 1><<<grid, 128, 0, stream>>>(p);
    } else {
      dim3 grid(n_items_bound, cdiv_i(p.block_size, 128), p.KH);
      bwd_dkdv_kernel<D, VD, MODE_SLC, 4, 1><<<grid, 256, 0, stream>>>(p);
    }
  }
  return nsa_check_launch("bwd_dkdv_kernel");
}

}  // namespace

// workgroups (= slots of the partial buffers) of a compressed-branch launch: grid.x * B * KH, as launch() sizes it
int64_t nsa_bwd_dkdv_cmp_slots(int B, int KH, int max_q_len, int max_k_len, int q_chunk_tokens, int kernel_size,
                               int stride) {
  const int KW = nsa_bwd_dkdv_slot_keys(0, 0);
  const int nch = cdiv_i(max_q_len, q_chunk_tokens);
  int64_t total = 0;
  for (int kt = 0; kt * KW < max_k_len; kt++) {
    const int fc = (stride * kt * KW + kernel_size - 1) / q_chunk_tokens;
    total += nch - (nch < fc ? nch : fc);
  }
  return total * B * KH;
}
int64_t nsa_bwd_dkdv_slc_slots(int KH, int n_items_bound, int block_size) {
  return (int64_t)KH * n_items_bound * (block_size <= 64 ? 1 : cdiv_i(block_size, 128));
}
// keys of one slot
int nsa_bwd_dkdv_slot_keys(int mode, int block_size) {
  if (mode == MODE_SLC) return block_size <= 64 ? 64 : 128;
  return 4 * 32 * (nsa_tuning_knob("dkdv_key_blocks", 1) == 2 ? 2 : 1);
}

int nsa_bwd_dkdv_launch(const NsaBwdTileParams& p, int mode, int B, int max_q_len, int max_k_len, int D, int VD,
                        int n_items_bound, hipStream_t stream) {
  if (D == 128 && VD == 128) return launch<128, 128>(p, mode, B, max_q_len, max_k_len, n_items_bound, stream);
  if (D == 64 && VD == 64) return launch<64, 64>(p, mode, B, max_q_len, max_k_len, n_items_bound, stream);
  if (D == 192 && VD == 128) return launch<192, 128>(p, mode, B, max_q_len, max_k_len, n_items_bound, stream);
  if (D == 256 && VD == 256) return launch<256, 256>(p, mode, B, max_q_len, max_k_len, n_items_bound, stream);
  if (D == 32 && VD == 32) return launch<32, 32>(p, mode, B, max_q_len, max_k_len, n_items_bound, stream);
  nsa_set_error("attention dk/dv: unsupported head dims D=%d VD=%d", D, VD);
  return NSA_ERR_UNSUPPORTED;
}

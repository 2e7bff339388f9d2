// Block-importance scoring and top-n block selection as two launches with the block scores in a caller-provided
// workspace (upstream keeps them in a [KH, T, blocks] tensor between its two kernels too: flash_nsa/ops/topk.py:226-425
// `slc_probs`; here fp32, and only for the tokens of one chunk).
//
//   topk_score_kernel  a workgroup of 4 waves owns 128 (token, q-head) rows of one kv-head group, 32 per wave, and
//                      walks the compressed keys in tiles of 64 that all four waves share (global -> LDS directly,
//                      double-buffered, one barrier per tile).  S = Q CK^T with v_mfma_f32_32x32x16_bf16 (a lane
//                      holds 16 rows of one key, so the sum over the heads of a token is an in-register add),
//                      p = exp2(s*c - lse); the head-summed probabilities of a tile go to a wave-private LDS strip,
//                      are folded into the scores of the selection blocks the tile completes (overlap weights
//                      area/stride, ascending key order) and stored.  128 registers: four waves per SIMD.
//   topk_pick_kernel   one wave per (kv head, token): the visible scores of the row in registers, forced initial and
//                      local blocks first, then repeated arg-max (lowest index on ties).
//
// The one-launch kernel of nsa_topk.hip keeps the scores of its tokens in LDS, which holds it at two waves per SIMD;
// it remains the path for shapes this one does not take (more than 16 q-heads per kv head, selection blocks that are
// not a power-of-two number of strides up to 64, more than 2048 selection blocks) and for callers without a
// workspace.
#include "nsa_common.h"
#include "nsa_api_internal.h"
#include "nsa_select.h"

namespace {

typedef __attribute__((address_space(1))) const void* nsa_gptr_t;
typedef __attribute__((address_space(3))) void* nsa_lptr_t;

constexpr int KT = 64;    // compressed keys per tile
constexpr int HALO = 8;   // head-summed probabilities kept from the previous tile (>= kernel_size / stride - 1)

template <int CP>
NSA_DEVICE constexpr int swz(int r) { return CP % 16 == 0 ? (r & 15) : ((r >> 1) & 7); }

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

struct ScoreWs {
  float* imp;      // [KH][ntok][row_stride] block scores of the chunk's tokens
  int32_t* pos;    // [ntok] absolute position of the token in its context, -1: token not in this launch
  int tok_lo, tok_hi, row_stride;
};

#ifndef NSA_TOPK_SCORE_WAVES
#define NSA_TOPK_SCORE_WAVES 4
#endif
template <int D, int GP, bool PAGED>
__global__ __launch_bounds__(256, NSA_TOPK_SCORE_WAVES) void topk_score_kernel(NsaTopkParams p, ScoreWs ws) {
  constexpr int TPW = 32 / GP;      // tokens per wave
  constexpr int TWG = 4 * TPW;      // tokens per workgroup
  constexpr int KP = D / 8;         // 16-byte chunks per key row
  constexpr int KJ = (KT * KP) / 256;
  constexpr int PLD = HALO + KT + 8;  // a fold may look up to 7 entries past its last key
  using SM = SlotMap<GP>;
  // two separate arrays, addressed with compile-time buffer numbers: the compiler then knows that the LDS reads of
  // the tile being computed do not alias the direct-to-LDS loads of the next tile, and does not wait for those
  __shared__ __attribute__((aligned(16))) bf16_t Ks_a[KT * D];
  __shared__ __attribute__((aligned(16))) bf16_t Ks_b[KT * D];
  __shared__ float pg_all[4 * TPW * PLD];

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
  const int n0 = blockIdx.x * TWG;
  if (n0 >= xl) return;
  // tokens outside this launch's chunk of the packed token range are left to the other launches
  if (x0 + n0 >= ws.tok_hi || x0 + min(n0 + TWG, xl) <= ws.tok_lo) return;
  const int ctx = PAGED ? p.ctx_lens[b] : xl;
  const int qoff = ctx - xl;
  const int nkeys = ctx >= p.kernel_size ? (ctx - p.kernel_size) / p.stride + 1 : 0;
  const int kbase = PAGED ? 0 : p.y_cu[b];
  const int32_t* table = PAGED ? p.table + (int64_t)b * p.table_stride : nullptr;
  const int Bs = p.block_size, Kz = p.kernel_size, St = p.stride;
  const int bps = Bs / St, kps = Kz / St;
  const int BPT = KT / bps;         // selection blocks completed per tile
  const int nloops = bps + kps - 1; // compressed keys that overlap a block

  // workgroup: keys that its last token sees, tiles to score and tiles to fold (every block up to the last token's)
  const int t_hi_wg = min(n0 + TWG - 1, xl - 1) + qoff;
  const int key_end = t_hi_wg >= Kz - 1 ? min((t_hi_wg - Kz + 1) / St + 1, nkeys) : 0;
  const int n_score = (key_end + KT - 1) / KT;
  const int n_fold = (t_hi_wg / Bs) / BPT + 1;
  const int ntiles = max(n_score, n_fold);

  // wave: its tokens
  const int nw0 = n0 + wave * TPW;
  const bool wave_active = nw0 < xl;
  const int tw_lo = nw0 + qoff;
  const int tw_hi = min(nw0 + TPW - 1, xl - 1) + qoff;
  float* pgw = pg_all + wave * TPW * PLD;

  // A-operand rows of this lane (row l32) and the lse of its C-layout rows
  bf16x8 qf[D / 16];
  float lse_r[16];
  bool rows_full;
  {
    int g = l32 % GP;
    if (g >= G) g = G - 1;
    const int n_a = min(nw0 + l32 / GP, xl - 1);
    const bf16_t* qp = p.q + (int64_t)(x0 + n_a) * p.q_st + (int64_t)(kh * G + g) * p.q_sh + hl * 8;
#pragma unroll
    for (int kc = 0; kc < D / 16; kc++) qf[kc] = ld_global_b128(qp + kc * 16);
    bool mine = true;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int row = (i >> 2) * 8 + hl * 4 + (i & 3);
      const int gg = row % GP, nn = nw0 + row / GP;
      const bool ok = (gg < G) && (nn < xl);
      mine = mine && ok;
      lse_r[i] = ok ? p.lse[(int64_t)(x0 + nn) * p.lse_st + (int64_t)(kh * G + gg) * p.lse_sh] : 0.f;
    }
    rows_full = __builtin_amdgcn_ballot_w64(!mine) == 0;
  }
  for (int i = lane; i < TPW * PLD; i += 64) pgw[i] = 0.f;

  // overlap weights of the keys of a block (the same for every block)
  float f_w[8];
  {
    int cs = St - Kz;
#pragma unroll
    for (int r = 0; r < 8; r++, cs += St) {
      const float w = r < nloops ? (float)(min(cs + Kz, Bs) - max(cs, 0)) / (float)St : 0.f;
      // wave-uniform: kept in a scalar register, so that the division does not sink into the loop
      f_w[r] = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, w)));
    }
  }

  // K tile staging, global -> LDS: lane L of a wave's j-th load fills LDS piece j*256 + wave*64 + L (row = piece /
  // chunks per row, position = piece % chunks per row) with the chunk that the row swizzle puts at that position
  int goffk[KJ];
#pragma unroll
  for (int j = 0; j < KJ; j++) {
    const int pc = tid + j * 256, row = pc / KP;
    goffk[j] = (int)((row * p.ck_sr + ((pc % KP) ^ swz<KP>(row)) * 8) * 2);
  }
  auto stage = [&](int kt, auto buf_tag) {
    bf16_t* Kdst = decltype(buf_tag)::value == 0 ? Ks_a : Ks_b;
    int64_t row0;
    if (PAGED) row0 = (int64_t)table[kt / p.page_size] * p.page_size + (kt % p.page_size);
    else row0 = (int64_t)kbase + kt;
    const int last = key_end - 1 - kt;  // >= 0; rows past it repeat it (masked)
    const char* kb = reinterpret_cast<const char*>(p.ck + row0 * p.ck_sr + (int64_t)kh * p.ck_sh);
    if (last >= KT - 1) {
#pragma unroll
      for (int j = 0; j < KJ; j++)
        __builtin_amdgcn_global_load_lds((nsa_gptr_t)(kb + goffk[j]), (nsa_lptr_t)&Kdst[(j * 256 + wave * 64) * 8], 16, 0, 0);
    } else {
#pragma unroll
      for (int j = 0; j < KJ; j++) {
        const int pc = tid + j * 256;
        const int row = pc / KP, c = (pc % KP) ^ swz<KP>(row);
        __builtin_amdgcn_global_load_lds((nsa_gptr_t)(kb + ((int64_t)min(row, last) * p.ck_sr + c * 8) * 2),
                                         (nsa_lptr_t)&Kdst[(j * 256 + wave * 64) * 8], 16, 0, 0);
      }
    }
  };
  // B-operand fragment of key row l32 + 32*half: chunk 2*kc + hl
  auto kfrag = [&](const bf16_t* Ks, int half, int kc) -> bf16x8 {
    const int row = l32 + 32 * half;
    return *reinterpret_cast<const bf16x8*>(Ks + (row * KP + ((2 * kc + hl) ^ swz<KP>(row))) * 8);
  };

  if (n_score > 0) stage(0, std::integral_constant<int, 0>{});
  auto do_tile = [&](int tile, auto buf_tag) {
    constexpr int BUF = decltype(buf_tag)::value;
    const int kt = tile * KT;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's pieces of the tile have landed
    __syncthreads();  // the tile is visible; nobody reads the other buffer any more
    if (tile + 1 < n_score) stage(kt + KT, std::integral_constant<int, 1 - BUF>{});
    if (!wave_active) return;
    const bf16_t* Ks = BUF == 0 ? Ks_a : Ks_b;
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const int key0 = kt + u * 32;
      float ps[SM::NSLOT];
#pragma unroll
      for (int s2 = 0; s2 < SM::NSLOT; s2++) ps[s2] = 0.f;
      // wave-uniform: does any / every (row, key) pair of this unit see its key
      const bool any_vis = key0 < key_end && tw_hi >= St * key0 + Kz - 1;
      if (any_vis) {
        f32x16 sacc;
#pragma unroll
        for (int i = 0; i < 16; i++) sacc[i] = 0.f;
        bf16x8 kf[D / 16];  // all fragments of the unit in flight before the first product
#pragma unroll
        for (int kc = 0; kc < D / 16; kc++) kf[kc] = kfrag(Ks, u, kc);
#pragma unroll
        for (int kc = 0; kc < D / 16; kc++) sacc = mfma32(qf[kc], kf[kc], sacc);
        const bool all_vis = rows_full && key0 + 32 <= nkeys && tw_lo >= St * (key0 + 31) + Kz - 1;
        if (all_vis) {
#pragma unroll
          for (int i = 0; i < 16; i++)
            ps[SM::slot_of(i)] += fast_exp2(__builtin_fmaf(sacc[i], p.scale_log2, -lse_r[i]));
        } else {
          const int key = key0 + l32;
          const int vis_from = St * key + Kz - 1;  // first position that sees this key
#pragma unroll
          for (int i = 0; i < 16; i++) {
            const int row = (i >> 2) * 8 + hl * 4 + (i & 3);
            const int nn = nw0 + row / GP;
            const bool vis = (row % GP < G) && (nn < xl) && (key < nkeys) && (nn + qoff >= vis_from);
            const float pv = vis ? fast_exp2(__builtin_fmaf(sacc[i], p.scale_log2, -lse_r[i])) : 0.f;
            ps[SM::slot_of(i)] += pv;
          }
        }
      }
#pragma unroll
      for (int s2 = 0; s2 < SM::NSLOT; s2++) {
        float v = ps[s2];
        if (SM::CROSS) v = xhalf_sum(v);
        if (!SM::CROSS || hl == 0) pgw[SM::token_of(s2, hl) * PLD + HALO + u * 32 + l32] = v;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // ---- fold: the blocks this tile completes, (token, block) pairs dealt to the lanes.  All 8 weights are applied
    // (those past the block's last key are 0 and meet finite entries of the strip), so the loop has no branches ----
    auto fold_one = [&](int it) {
      const int tk = it / BPT, jj = it - tk * BPT;
      const int n = nw0 + tk;
      const int j = tile * BPT + jj;
      const float* src = pgw + tk * PLD + HALO + jj * bps - kps + 1;
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < 8; r++) acc += src[r] * f_w[r];
      const int64_t tok = (int64_t)x0 + n;
      if (n < xl && tok >= ws.tok_lo && tok < ws.tok_hi && j < ws.row_stride)
        ws.imp[((int64_t)kh * (ws.tok_hi - ws.tok_lo) + (tok - ws.tok_lo)) * ws.row_stride + j] = acc;
    };
    if (TPW * BPT <= 64) {
      if (lane < TPW * BPT) fold_one(lane);
    } else {
      for (int it = lane; it < TPW * BPT; it += 64) fold_one(it);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // the last keys of this tile are the halo of the next
    for (int i = lane; i < TPW * HALO; i += 64) {
      const int tk = i / HALO, h = i - tk * HALO;
      pgw[tk * PLD + h] = pgw[tk * PLD + KT + h];
    }
  };
  for (int tile = 0; tile < ntiles; tile += 2) {
    do_tile(tile, std::integral_constant<int, 0>{});
    if (tile + 1 < ntiles) do_tile(tile + 1, std::integral_constant<int, 1>{});
  }
  // positions of the workgroup's tokens, for the pick kernel (kv head 0 writes them)
  if (kh == 0 && tid < TWG) {
    const int n = n0 + tid;
    const int64_t tok = (int64_t)x0 + n;
    if (n < xl && tok >= ws.tok_lo && tok < ws.tok_hi) ws.pos[tok - ws.tok_lo] = n + qoff;
  }
}

struct PickParams {
  const float* imp;      // [KH][ntok][row_stride]
  const int32_t* pos;    // [ntok]
  int32_t* topk; int64_t tk_sh, tk_st;
  float* imp_out; int64_t imp_sh, imp_st; int imp_cols;
  int ntok, tok_lo, row_stride, nb_max, KH;
  int block_size, top_n, num_init, num_local, ignore_index;
};

__global__ __launch_bounds__(256) void topk_pick_kernel(PickParams p) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t r = (int64_t)blockIdx.x * 4 + wave;
  if (r >= (int64_t)p.KH * p.ntok) return;
  const int kh = (int)(r / p.ntok);
  const int tr = (int)(r - (int64_t)kh * p.ntok);
  const int t = __builtin_amdgcn_readfirstlane(p.pos[tr]);
  if (t < 0) return;
  const float* imp = p.imp + r * p.row_stride;
  const int64_t tok = (int64_t)p.tok_lo + tr;
  const int nk = t / p.block_size;
  const int jmax = min(nk, p.nb_max - 1);
  if (p.imp_out != nullptr) {
    float* dst = p.imp_out + (int64_t)kh * p.imp_sh + tok * p.imp_st;
    for (int j = lane; j < p.imp_cols; j += 64) dst[j] = j <= jmax ? imp[j] : 0.f;
  }
  // candidates per lane sized by the row's own number of visible blocks (wave-uniform)
  const int cap = min(p.nb_max, p.row_stride);
  __shared__ float cand_v[4][64];
  __shared__ int cand_i[4][64];
  int result;
  if (jmax < 512) result = select_blocks_short_list<8>(imp, t, min(cap, 512), p, lane, cand_v[wave], cand_i[wave]);
  else if (jmax < 1024) result = select_blocks_short_list<16>(imp, t, min(cap, 1024), p, lane, cand_v[wave], cand_i[wave]);
  else result = select_blocks_short_list<32>(imp, t, min(cap, 2048), p, lane, cand_v[wave], cand_i[wave]);
  if (lane < p.top_n) p.topk[(int64_t)kh * p.tk_sh + tok * p.tk_st + lane] = result;
}

__global__ void fill_i32_kernel(int32_t* dst, int n, int32_t value) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = value;
}

template <int D, int GP, bool PAGED>
void launch_score(const NsaTopkParams& p, const ScoreWs& ws, int B, int max_q_len, hipStream_t stream) {
  constexpr int TWG = 4 * (32 / GP);
  dim3 grid(cdiv_i(max_q_len, TWG), B, p.KH);
  topk_score_kernel<D, GP, PAGED><<<grid, 256, 0, stream>>>(p, ws);
}

template <int D, bool PAGED>
void dispatch_score(const NsaTopkParams& p, const ScoreWs& ws, int B, int max_q_len, hipStream_t stream) {
  const int G = p.G;
  if (G > 8) launch_score<D, 16, PAGED>(p, ws, B, max_q_len, stream);
  else if (G > 4) launch_score<D, 8, PAGED>(p, ws, B, max_q_len, stream);
  else if (G > 2) launch_score<D, 4, PAGED>(p, ws, B, max_q_len, stream);
  else if (G > 1) launch_score<D, 2, PAGED>(p, ws, B, max_q_len, stream);
  else launch_score<D, 1, PAGED>(p, ws, B, max_q_len, stream);
}

int64_t row_stride_of(int nb_max) { return ((int64_t)nb_max + 63) / 64 * 64; }

}  // namespace

// does the two-pass selector take this shape
bool nsa_topk_two_pass_supported(const NsaTopkParams& p, int D) {
  if (p.G > 16 || !(D == 64 || D == 128 || D == 192)) return false;
  if (p.block_size % p.stride != 0 || p.kernel_size % p.stride != 0) return false;
  const int bps = p.block_size / p.stride, kps = p.kernel_size / p.stride;
  if (bps < 1 || KT % bps != 0 || bps + kps - 1 > 8 || kps - 1 > HALO) return false;
  return p.nb_max <= 2048;
}

// bytes per token of the chunk: its score rows for every kv head and its position
int64_t nsa_topk_two_pass_bytes_per_token(int KH, int nb_max) { return (int64_t)KH * row_stride_of(nb_max) * 4 + 4; }

int nsa_topk_two_pass_launch(const NsaTopkParams& p, bool paged, int B, int max_q_len, int total_tokens, int D,
                             void* workspace, int64_t workspace_bytes, hipStream_t stream) {
  if (B <= 0 || max_q_len <= 0 || total_tokens <= 0) return NSA_OK;
  const int64_t per_tok = nsa_topk_two_pass_bytes_per_token(p.KH, p.nb_max);
  int64_t chunk = (workspace_bytes - 256) / per_tok;
  if (workspace == nullptr || chunk < 1) {
    nsa_set_error("top-k: a workspace of %lld bytes holds no token (%lld bytes per token)", (long long)workspace_bytes,
                  (long long)per_tok);
    return NSA_ERR_WORKSPACE;
  }
  if (chunk > total_tokens) chunk = total_tokens;
  const int rs = (int)row_stride_of(p.nb_max);
  for (int64_t lo = 0; lo < total_tokens; lo += chunk) {
    const int ntok = (int)min((int64_t)total_tokens - lo, chunk);
    ScoreWs ws;
    ws.imp = (float*)workspace;
    ws.pos = (int32_t*)((char*)workspace + (((int64_t)p.KH * ntok * rs * 4 + 255) & ~(int64_t)255));
    ws.tok_lo = (int)lo; ws.tok_hi = (int)lo + ntok; ws.row_stride = rs;
    fill_i32_kernel<<<cdiv_i(ntok, 256), 256, 0, stream>>>(ws.pos, ntok, -1);
    if (D == 128) paged ? dispatch_score<128, true>(p, ws, B, max_q_len, stream) : dispatch_score<128, false>(p, ws, B, max_q_len, stream);
    else if (D == 64) paged ? dispatch_score<64, true>(p, ws, B, max_q_len, stream) : dispatch_score<64, false>(p, ws, B, max_q_len, stream);
    else paged ? dispatch_score<192, true>(p, ws, B, max_q_len, stream) : dispatch_score<192, false>(p, ws, B, max_q_len, stream);
    int rc = nsa_check_launch("topk_score_kernel");
    if (rc) return rc;
    PickParams pp{};
    pp.imp = ws.imp; pp.pos = ws.pos;
    pp.topk = p.topk; pp.tk_sh = p.tk_sh; pp.tk_st = p.tk_st;
    pp.imp_out = p.imp_out; pp.imp_sh = p.imp_sh; pp.imp_st = p.imp_st; pp.imp_cols = p.imp_cols;
    pp.ntok = ntok; pp.tok_lo = (int)lo; pp.row_stride = rs; pp.nb_max = p.nb_max; pp.KH = p.KH;
    pp.block_size = p.block_size; pp.top_n = p.top_n; pp.num_init = p.num_init; pp.num_local = p.num_local;
    pp.ignore_index = p.ignore_index;
    const int64_t rows = (int64_t)p.KH * ntok;
    topk_pick_kernel<<<(unsigned)((rows + 3) / 4), 256, 0, stream>>>(pp);
    rc = nsa_check_launch("topk_pick_kernel");
    if (rc) return rc;
  }
  return NSA_OK;
}

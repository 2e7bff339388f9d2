// Dense-tile flash forward for the two branches whose key set is a contiguous range per query:
//   MODE_CMP: compressed attention, key i visible to absolute query position t iff t >= stride*i + kernel-1
//             (upstream flash_nsa/ops/compress_attn.py:17-153; paged: flash_nsa/inference/compress_attn.py:19-149)
//   MODE_SWA: causal sliding window, keys max(0,t-W) <= j <= t
//             (upstream flash_nsa/ops/sliding_window_attention.py:26-95, which calls FlashAttention)
//
// Work decomposition: a "row" is one (query token, q-head) pair of one kv-head group, rows ordered
// token-major / head-minor so that the G heads sharing K/V sit next to each other.  A workgroup of 4 waves
// owns 4*32*RS consecutive rows; every lane owns RS rows (lane l and l+32 share a row and split its keys), so
// the online-softmax statistics are per-lane scalars.  Key tiles of 64 rows are staged in LDS (row-major) and
// shared by the 4 waves.  S^T = K Q^T and O^T = V^T P^T are computed with v_mfma_f32_32x32x16_bf16; the V^T
// operand comes from ds_read_b64_tr_b16 so V never needs an explicit transpose.
#include "nsa_common.h"
#include "nsa_api_internal.h"
#include <type_traits>

namespace {

constexpr int MODE_CMP = 0;
constexpr int MODE_SWA = 1;

typedef __attribute__((address_space(1))) const void* nsa_gptr_t;
typedef __attribute__((address_space(3))) void* nsa_lptr_t;

// position swizzle of the 16-byte chunks of row r in an unpadded LDS tile with CP chunks per row: chunk c sits at
// position c ^ swz(r), which spreads the rows that a fragment read touches over all banks
template <int CP>
NSA_DEVICE constexpr int swz(int r) { return CP % 16 == 0 ? (r & 15) : ((r >> 1) & 7); }
// the same for the V tile, whose transposed reads fetch 32 bytes (two chunks) from each of four consecutive rows
// per group of 16 lanes: the swizzle moves whole chunk pairs, so that the rows of a group (and of the wave's other
// groups) land in different 32-byte bank slots (measured: 108 bytes/clk/CU against 61 with swz above)
template <int CP>
NSA_DEVICE constexpr int swzv(int r) { return CP % 16 == 0 ? ((r & 7) << 1) : (((r >> 1) & 3) << 1); }

// ASYNC: the K/V tiles go from global memory straight into LDS (global_load_lds, 16 bytes per lane, no staging
// registers, no ds_write); the tiles are then unpadded and swizzled instead of padded.
template <int D, int VD, int MODE, bool PAGED, int RS, int MINB, bool ASYNC>
__global__ __launch_bounds__(256, MINB) void fwd_tile_kernel(NsaFwdTileParams p) {
  static_assert(RS == 1 || RS == 2, "one or two 32-row sets per wave");
  constexpr int ROWS_W = 32 * RS;
  constexpr int ROWS_WG = 4 * ROWS_W;
  constexpr int KT = 64;
  constexpr int KLD = ASYNC ? D : D + NSA_LDS_PAD;
  constexpr int VLD = ASYNC ? VD : VD + NSA_LDS_PAD;
  // two K/V tile buffers: the tile after the one being computed is stored while the other waves may still read the
  // current one, so a tile costs one barrier
  __shared__ __attribute__((aligned(16))) bf16_t Ks2[2][KT * KLD];
  __shared__ __attribute__((aligned(16))) bf16_t Vs2[2][KT * VLD];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31;
  const int hl = lane >> 5;
  const int g16 = lane >> 4, i16 = lane & 15;
  const int b = blockIdx.y;
  const int kh = blockIdx.z;
  const int G = p.G;

  const int x0 = p.x_cu[b];
  const int xl = p.x_cu[b + 1] - x0;
  const int rows_total = xl * G;
  const int r0 = blockIdx.x * ROWS_WG;
  if (r0 >= rows_total) return;
  const int ctx = PAGED ? p.ctx_lens[b] : xl;
  const int qoff = ctx - xl;
  int nkeys, kbase = 0;
  if (MODE == MODE_CMP) {
    nkeys = ctx >= p.kernel_size ? (ctx - p.kernel_size) / p.stride + 1 : 0;
    if (!PAGED) kbase = p.k_cu[b];
  } else {
    nkeys = ctx;
    if (!PAGED) kbase = x0;
  }
  const int32_t* table = PAGED ? p.table + (int64_t)b * p.table_stride : nullptr;

  // ---- per-lane rows ----
  int t_row[RS];
  bool valid[RS];
  int64_t tok[RS];
  int head[RS];
  bf16x8 qf[RS][D / 16];
#pragma unroll
  for (int rs = 0; rs < RS; rs++) {
    int r = r0 + wave * ROWS_W + rs * 32 + l32;
    valid[rs] = r < rows_total;
    int rr = valid[rs] ? r : rows_total - 1;
    int n = rr / G;
    int g = rr - n * G;
    t_row[rs] = n + qoff;
    tok[rs] = x0 + n;
    head[rs] = kh * G + g;
    const bf16_t* qp = p.q + tok[rs] * p.q_st + (int64_t)head[rs] * p.q_sh + hl * 8;
#pragma unroll
    for (int kc = 0; kc < D / 16; kc++) qf[rs][kc] = ld_global_b128(qp + kc * 16);
  }
  // wave-uniform position range (scalar registers)
  const int rw_lo = r0 + wave * ROWS_W;
  const int rw_hi = min(rw_lo + ROWS_W - 1, rows_total - 1);
  const bool wave_active = rw_lo < rows_total;
  const int tw_lo = (wave_active ? rw_lo / G : 0) + qoff;
  const int tw_hi = (wave_active ? rw_hi / G : 0) + qoff;
  const int t_lo = r0 / G + qoff;
  const int t_hi = min(r0 + ROWS_WG - 1, rows_total - 1) / G + qoff;

  int key_begin, key_end;
  if (MODE == MODE_CMP) {
    key_begin = 0;
    key_end = t_hi >= p.kernel_size - 1 ? min((t_hi - p.kernel_size + 1) / p.stride + 1, nkeys) : 0;
  } else {
    key_begin = (max(0, t_lo - p.window) / KT) * KT;
    key_end = min(t_hi + 1, nkeys);
  }

  f32x16 oacc[RS][VD / 32];
  float m_run[RS], l_run[RS];
#pragma unroll
  for (int rs = 0; rs < RS; rs++) {
    m_run[rs] = NSA_NEG_INF;
    l_run[rs] = 0.f;
#pragma unroll
    for (int dt = 0; dt < VD / 32; dt++)
#pragma unroll
      for (int i = 0; i < 16; i++) oacc[rs][dt][i] = 0.f;
  }
  const float sc = p.scale_log2;

  // software pipeline: the next tile's global loads are in flight while the current tile is computed.
  // Rows past the end of the key range are replaced by the last valid row; their scores are masked, so the
  // duplicated data never contributes.
  constexpr int KP = D / 8, VP = VD / 8;
  constexpr int KJ = (KT * KP) / 256, VJ = (KT * VP) / 256;
  bf16x8 kreg[KJ], vreg[VJ];
  auto gload = [&](int kt) {
    int64_t page_row0 = 0;
    if (PAGED) {
      int pg = table[kt / p.page_size];
      page_row0 = (int64_t)pg * p.page_size + (kt % p.page_size);
    }
    const int last = key_end - 1 - kt;  // >= 0
#pragma unroll
    for (int j = 0; j < KJ; j++) {
      int pc = tid + j * 256;
      int kr = min(pc / KP, last), dp = pc % KP;
      int64_t row = PAGED ? page_row0 + kr : (int64_t)kbase + kt + kr;
      kreg[j] = ld_global_b128(p.k + row * p.k_sr + (int64_t)kh * p.k_sh + dp * 8);
    }
#pragma unroll
    for (int j = 0; j < VJ; j++) {
      int pc = tid + j * 256;
      int kr = min(pc / VP, last), dp = pc % VP;
      int64_t row = PAGED ? page_row0 + kr : (int64_t)kbase + kt + kr;
      vreg[j] = ld_global_b128(p.v + row * p.v_sr + (int64_t)kh * p.v_sh + dp * 8);
    }
  };

  // one 64-key tile for one row set
  // Fragment addresses.  Padded tiles: row * stride + column, the compiler folds everything but the lane part into
  // immediates.  Swizzled tiles with a power-of-two row size: byte address = lane part XOR (index << 5 or 6) +
  // compile-time row offset, with the lane parts computed once (kx, vxa, vxb), so a read costs at most one v_xor.
  constexpr bool POW2 = (D == 64 || D == 128) && (VD == 64 || VD == 128);
  int kx = 0, vxa = 0, vxb = 0;
  if constexpr (ASYNC && POW2) {
    const int s0 = swz<D / 8>(l32);
    kx = (l32 * D * 2 + ((hl ^ (s0 & 1)) << 4)) ^ ((s0 >> 1) << 5);
    const int sl = hl * 4 + (i16 >> 2);                 // row of the fragment inside its group of 16 rows
    const int cl = (g16 & 1) * 2 + ((i16 & 3) >> 1);    // chunk inside its group of 4 chunks
    const int sa = swzv<VD / 8>(sl), sb = swzv<VD / 8>(sl + 8);
    vxa = (sl * VD * 2 + ((cl ^ (sa & 3)) << 4) + (i16 & 1) * 8) ^ ((sa >> 2) << 6);
    vxb = ((sl + 8) * VD * 2 + ((cl ^ (sb & 3)) << 4) + (i16 & 1) * 8) ^ ((sb >> 2) << 6);
  }
  // K fragment: rows l32 + 32*half, chunk 2*kc + hl
  auto kfrag = [&](const bf16_t* Ks, int half, int kc) -> bf16x8 {
    if constexpr (ASYNC && POW2)
      return *reinterpret_cast<const bf16x8*>(reinterpret_cast<const char*>(Ks) + half * 32 * D * 2 + (kx ^ (kc << 5)));
    else if constexpr (ASYNC)
      return *reinterpret_cast<const bf16x8*>(
          Ks + ((l32 + 32 * half) * (D / 8) + ((2 * kc + hl) ^ swz<D / 8>(l32))) * 8);
    else
      return *reinterpret_cast<const bf16x8*>(Ks + (l32 + 32 * half) * KLD + (2 * kc + hl) * 8);
  };
  // transposed V fragment piece: row kb + (i16 >> 2) (kb a multiple of 16, plus 8 for the second piece), columns
  // dt*32 + (g16&1)*16 + 4*(i16&3) ..
  auto vfrag = [&](const bf16_t* Vs, int kb16, int second, int dt) -> bf16x4 {
    if constexpr (ASYNC && POW2) {
      const int x = (second ? vxb : vxa) ^ (dt << 6);
      return lds_read_tr(reinterpret_cast<const bf16_t*>(reinterpret_cast<const char*>(Vs) + kb16 * VD * 2 + x));
    } else {
      const int row = kb16 + second * 8 + hl * 4 + (i16 >> 2);
      const int col = dt * 32 + (g16 & 1) * 16 + 4 * (i16 & 3);
      if constexpr (ASYNC) return lds_read_tr(Vs + (row * (VD / 8) + ((col >> 3) ^ swzv<VD / 8>(row))) * 8 + (col & 7));
      else return lds_read_tr(Vs + row * VLD + col);
    }
  };
  auto process = [&](bool masked, auto rs_tag, int kt, const bf16_t* Ks, const bf16_t* Vs) {
    constexpr int rs = decltype(rs_tag)::value;
    // ---- S^T = K Q^T : two 32-key sub tiles, interleaved accumulators ----
    f32x16 sacc[2];
#pragma unroll
    for (int i = 0; i < 16; i++) { sacc[0][i] = 0.f; sacc[1][i] = 0.f; }
#pragma unroll
    for (int kc = 0; kc < D / 16; kc++) {
      bf16x8 k0 = kfrag(Ks, 0, kc);
      bf16x8 k1 = kfrag(Ks, 1, kc);
      sacc[0] = mfma32(k0, qf[rs][kc], sacc[0]);
      sacc[1] = mfma32(k1, qf[rs][kc], sacc[1]);
    }
    // ---- mask, online softmax (running max in raw score units; scale folded into the exp2 fma) ----
    if (masked) {  // wave-uniform: only tiles that straddle a visibility boundary pay for the mask
      const int t = t_row[rs];
#pragma unroll
      for (int nt = 0; nt < 2; nt++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          int key = kt + nt * 32 + (i >> 2) * 8 + hl * 4 + (i & 3);
          bool vis;
          if (MODE == MODE_CMP) vis = (key < nkeys) && (t >= p.stride * key + p.kernel_size - 1);
          else vis = (key <= t) && (key >= t - p.window);
          sacc[nt][i] = vis ? sacc[nt][i] : NSA_NEG_INF;
        }
    }
    float tmax = NSA_NEG_INF;
#pragma unroll
    for (int nt = 0; nt < 2; nt++)
#pragma unroll
      for (int i = 0; i < 16; i++) tmax = fmaxf(tmax, sacc[nt][i]);
    tmax = xhalf_max(tmax);
    const float m_old = m_run[rs];
    const float m_new = fmaxf(m_old, tmax);
    const float m_safe = (m_new == NSA_NEG_INF) ? 0.f : m_new;
    const float msc = m_safe * sc;
    m_run[rs] = m_new;
    float psum = 0.f;
#pragma unroll
    for (int nt = 0; nt < 2; nt++)
#pragma unroll
      for (int i = 0; i < 16; i++) {
        float pv = fast_exp2(__builtin_fmaf(sacc[nt][i], sc, -msc));
        sacc[nt][i] = pv;
        psum += pv;
      }
    if (__builtin_amdgcn_ballot_w64(m_new != m_old) != 0) {  // rescale only when some row's max moved
      const float alpha = fast_exp2((m_old - m_safe) * sc);
      l_run[rs] *= alpha;
#pragma unroll
      for (int dt = 0; dt < VD / 32; dt++)
#pragma unroll
        for (int i = 0; i < 16; i++) oacc[rs][dt][i] *= alpha;
    }
    l_run[rs] += psum;

    // ---- O^T += V^T P^T ----
#pragma unroll
    for (int c = 0; c < 4; c++) {
      const int nt = c >> 1, ch = c & 1;
      bf16x8 pf = pack8(sacc[nt][ch * 8 + 0], sacc[nt][ch * 8 + 1], sacc[nt][ch * 8 + 2], sacc[nt][ch * 8 + 3],
                        sacc[nt][ch * 8 + 4], sacc[nt][ch * 8 + 5], sacc[nt][ch * 8 + 6], sacc[nt][ch * 8 + 7]);
      const int kb16 = nt * 32 + ch * 16;  // the lane's rows: kb16 + hl*4 + (i16>>2) and 8 further
#pragma unroll
      for (int dt = 0; dt < VD / 32; dt++) {
        bf16x4 v0 = vfrag(Vs, kb16, 0, dt);
        bf16x4 v1 = vfrag(Vs, kb16, 1, dt);
        oacc[rs][dt] = mfma32(cat4(v0, v1), pf, oacc[rs][dt]);
      }
    }
  };

  auto stage = [&](int buf) {
#pragma unroll
    for (int j = 0; j < KJ; j++) {
      int pc = tid + j * 256;
      *reinterpret_cast<bf16x8*>(&Ks2[buf][(pc / KP) * KLD + (pc % KP) * 8]) = kreg[j];
    }
#pragma unroll
    for (int j = 0; j < VJ; j++) {
      int pc = tid + j * 256;
      *reinterpret_cast<bf16x8*>(&Vs2[buf][(pc / VP) * VLD + (pc % VP) * 8]) = vreg[j];
    }
  };
  // ASYNC staging: lane L of a wave's j-th load fills LDS piece j*256 + wave*64 + L (row = piece / chunks per row,
  // position = piece % chunks per row), i.e. it fetches the chunk that the swizzle puts at that position
  // per-lane byte offsets of its pieces from the first row of a tile (the same for every full tile)
  int goffk[KJ], goffv[VJ];
  if constexpr (ASYNC) {
#pragma unroll
    for (int j = 0; j < KJ; j++) {
      const int pc = tid + j * 256, row = pc / KP;
      goffk[j] = (int)((row * p.k_sr + ((pc % KP) ^ swz<KP>(row)) * 8) * 2);
    }
#pragma unroll
    for (int j = 0; j < VJ; j++) {
      const int pc = tid + j * 256, row = pc / VP;
      goffv[j] = (int)((row * p.v_sr + ((pc % VP) ^ swzv<VP>(row)) * 8) * 2);
    }
  }
  auto stage_async = [&](int kt, int buf) {
    int64_t row0;
    if (PAGED) row0 = (int64_t)table[kt / p.page_size] * p.page_size + (kt % p.page_size);
    else row0 = (int64_t)kbase + kt;
    const int last = key_end - 1 - kt;  // >= 0; rows past it repeat it (masked)
    const char* kb = reinterpret_cast<const char*>(p.k + row0 * p.k_sr + (int64_t)kh * p.k_sh);
    const char* vb = reinterpret_cast<const char*>(p.v + row0 * p.v_sr + (int64_t)kh * p.v_sh);
    if (last >= KT - 1) {  // wave-uniform
#pragma unroll
      for (int j = 0; j < KJ; j++)
        __builtin_amdgcn_global_load_lds((nsa_gptr_t)(kb + goffk[j]),
                                         (nsa_lptr_t)&Ks2[buf][(j * 256 + wave * 64) * 8], 16, 0, 0);
#pragma unroll
      for (int j = 0; j < VJ; j++)
        __builtin_amdgcn_global_load_lds((nsa_gptr_t)(vb + goffv[j]),
                                         (nsa_lptr_t)&Vs2[buf][(j * 256 + wave * 64) * 8], 16, 0, 0);
    } else {
#pragma unroll
      for (int j = 0; j < KJ; j++) {
        const int pc = tid + j * 256;
        const int row = pc / KP, c = (pc % KP) ^ swz<KP>(row);
        __builtin_amdgcn_global_load_lds((nsa_gptr_t)(kb + ((int64_t)min(row, last) * p.k_sr + c * 8) * 2),
                                         (nsa_lptr_t)&Ks2[buf][(j * 256 + wave * 64) * 8], 16, 0, 0);
      }
#pragma unroll
      for (int j = 0; j < VJ; j++) {
        const int pc = tid + j * 256;
        const int row = pc / VP, c = (pc % VP) ^ swzv<VP>(row);
        __builtin_amdgcn_global_load_lds((nsa_gptr_t)(vb + ((int64_t)min(row, last) * p.v_sr + c * 8) * 2),
                                         (nsa_lptr_t)&Vs2[buf][(j * 256 + wave * 64) * 8], 16, 0, 0);
      }
    }
  };
  if (key_begin < key_end) {
    if constexpr (ASYNC) {
      stage_async(key_begin, 0);
    } else {
      gload(key_begin);
      stage(0);
      if (key_begin + KT < key_end) gload(key_begin + KT);
    }
  }

  int buf = 0;
  for (int kt = key_begin; kt < key_end; kt += KT, buf ^= 1) {
    if constexpr (ASYNC) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's pieces of tile kt have landed
    __syncthreads();  // tile kt is visible; nobody reads the other buffer (tile kt - KT) any more
    if (kt + KT < key_end) {
      if constexpr (ASYNC) {
        stage_async(kt + KT, buf ^ 1);
      } else {
        stage(buf ^ 1);
        if (kt + 2 * KT < key_end) gload(kt + 2 * KT);
      }
    }
    if (!wave_active) continue;

    // wave-uniform visibility classification of this tile
    bool any_vis, full_vis;
    if (MODE == MODE_CMP) {
      any_vis = tw_hi >= p.stride * kt + p.kernel_size - 1;
      full_vis = (tw_lo >= p.stride * (kt + KT - 1) + p.kernel_size - 1) && (kt + KT <= nkeys);
    } else {
      any_vis = (kt <= tw_hi) && (kt + KT - 1 >= tw_lo - p.window);
      full_vis = (kt + KT - 1 <= tw_lo) && (kt >= tw_hi - p.window);
    }
    if (!any_vis) continue;
    process(!full_vis, std::integral_constant<int, 0>{}, kt, Ks2[buf], Vs2[buf]);
    if constexpr (RS > 1) process(!full_vis, std::integral_constant<int, RS - 1>{}, kt, Ks2[buf], Vs2[buf]);
  }

  // ---- epilogue ----
#pragma unroll
  for (int rs = 0; rs < RS; rs++) {
    float l_tot = xhalf_sum(l_run[rs]);
    if (!valid[rs]) continue;
    float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    bf16_t* op = p.o + tok[rs] * p.o_st + (int64_t)head[rs] * p.o_sh;
#pragma unroll
    for (int dt = 0; dt < VD / 32; dt++)
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        int d = dt * 32 + i4 * 8 + hl * 4;
        bf16x4 w = pack4(oacc[rs][dt][i4 * 4 + 0] * inv, oacc[rs][dt][i4 * 4 + 1] * inv,
                         oacc[rs][dt][i4 * 4 + 2] * inv, oacc[rs][dt][i4 * 4 + 3] * inv);
        *reinterpret_cast<bf16x4*>(op + d) = w;
      }
    if (hl == 0 && p.lse != nullptr) {
      float lse2 = l_tot > 0.f ? m_run[rs] * sc + fast_log2(l_tot) : 0.f;
      p.lse[tok[rs] * p.lse_st + (int64_t)head[rs] * p.lse_sh] = lse2;
    }
  }
}

template <int D, int VD, int MODE, bool PAGED>
int launch_fwd_tile(const NsaFwdTileParams& p, int B, int max_q_len, hipStream_t stream) {
  if (B <= 0 || max_q_len <= 0) return NSA_OK;
  // 0 (default): direct-to-LDS staging for the compressed branch with power-of-two head dims (4.5 % faster there;
  // the window branch, with its short key loops, and d=192, whose swizzled addresses cost registers, are faster with
  // register staging); 1..4 force one variant for experiments
  const int variant = nsa_tuning_knob("fwd_variant", 0);
  constexpr bool pow2 = (D == 64 || D == 128) && (VD == 64 || VD == 128);
  const bool async = variant == 4 || (variant == 0 && MODE == MODE_CMP && pow2);
  if constexpr (D > 192 || VD > 128) {
    // head dims of 256: the output accumulators alone take 128 registers, one workgroup per CU
    dim3 grid(cdiv_i(max_q_len * p.G, 128), B, p.KH);
    fwd_tile_kernel<D, VD, MODE, PAGED, 1, 1, false><<<grid, 256, 0, stream>>>(p);
    return nsa_check_launch("fwd_tile_kernel");
  } else if (variant == 2) {
    dim3 grid(cdiv_i(max_q_len * p.G, 256), B, p.KH);
    fwd_tile_kernel<D, VD, MODE, PAGED, 2, 1, false><<<grid, 256, 0, stream>>>(p);
  } else if (variant == 3) {
    dim3 grid(cdiv_i(max_q_len * p.G, 128), B, p.KH);
    fwd_tile_kernel<D, VD, MODE, PAGED, 1, 1, false><<<grid, 256, 0, stream>>>(p);
  } else if (async) {
    dim3 grid(cdiv_i(max_q_len * p.G, 128), B, p.KH);
    fwd_tile_kernel<D, VD, MODE, PAGED, 1, 2, true><<<grid, 256, 0, stream>>>(p);
  } else {
    dim3 grid(cdiv_i(max_q_len * p.G, 128), B, p.KH);
    fwd_tile_kernel<D, VD, MODE, PAGED, 1, 2, false><<<grid, 256, 0, stream>>>(p);
  }
  return nsa_check_launch("fwd_tile_kernel");
}

template <int MODE, bool PAGED>
int dispatch_fwd_tile(const NsaFwdTileParams& p, int B, int max_q_len, int D, int VD, hipStream_t stream) {
  if (D == 128 && VD == 128) return launch_fwd_tile<128, 128, MODE, PAGED>(p, B, max_q_len, stream);
  if (D == 64 && VD == 64) return launch_fwd_tile<64, 64, MODE, PAGED>(p, B, max_q_len, stream);
  if (D == 192 && VD == 128) return launch_fwd_tile<192, 128, MODE, PAGED>(p, B, max_q_len, stream);
  if (D == 256 && VD == 256) return launch_fwd_tile<256, 256, MODE, PAGED>(p, B, max_q_len, stream);
  if (D == 32 && VD == 32) return launch_fwd_tile<32, 32, MODE, PAGED>(p, B, max_q_len, stream);
  nsa_set_error("attention forward: unsupported head dims D=%d VD=%d (built: 128/128, 64/64, 192/128, 256/256, 32/32)", D, VD);
  return NSA_ERR_UNSUPPORTED;
}

}  // namespace

int nsa_fwd_tile_launch(const NsaFwdTileParams& p, int mode, bool paged, int B, int max_q_len, int D, int VD,
                        hipStream_t stream) {
  if (mode == MODE_CMP) {
    return paged ? dispatch_fwd_tile<MODE_CMP, true>(p, B, max_q_len, D, VD, stream)
                 : dispatch_fwd_tile<MODE_CMP, false>(p, B, max_q_len, D, VD, stream);
  }
  return paged ? dispatch_fwd_tile<MODE_SWA, true>(p, B, max_q_len, D, VD, stream)
               : dispatch_fwd_tile<MODE_SWA, false>(p, B, max_q_len, D, VD, stream);
}

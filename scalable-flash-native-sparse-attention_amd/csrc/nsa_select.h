// Block selection of one token by one wave, with the candidates in registers; shared by the decode kernels and the
// two-pass block selector of the training / prefill path.
#pragma once
#include <type_traits>
#include "nsa_common.h"

// one wave: forced initial and local blocks, then repeated arg-max over imp[0 .. min(t/block, nb_cap-1)] (lowest
// index on ties).  Returns the block of slot `lane`.
// The candidates of a lane (blocks lane, lane+64, ...) are read once into NV registers; after every round only the
// winner's lane rescans its registers, so a round costs one wave reduction instead of a dependent chain of LDS reads.
template <int NV, class P>
NSA_DEVICE int select_blocks_regs(const float* imp, int t, int nb_cap, const P& p, int lane) {
  static_assert(NV % 8 == 0, "candidates per lane come in groups of 8");
  constexpr int NG = NV / 8;
  const int nk = t >= 0 ? t / p.block_size : -1;
  int result = p.ignore_index;
  if (lane < p.num_init) {
    if (lane <= nk) result = lane;
  } else if (lane < p.num_init + p.num_local) {
    if (lane <= nk) result = nk - (lane - p.num_init);
  }
  const int nsel = min(p.top_n, nk + 1);
  const int jmax = min(nk, nb_cap - 1);
  float v[NV];
#pragma unroll
  for (int k = 0; k < NV; k++) {
    const int j = lane + 64 * k;
    float x = j <= jmax ? imp[min(j, nb_cap - 1)] : -3.f;
    if (j <= jmax && (j < p.num_init || j > nk - p.num_local)) x = -1.f;  // forced blocks: behind every real score
    v[k] = x;
  }
  // best candidate of every group of 8 registers; a round only rescans the group the winner came from (the group
  // number is wave-uniform, so that is one uniform branch)
  float gbest[NG];
  int gidx[NG];
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
  auto for_group = [&](int g, auto&& fn) {
    if constexpr (NG == 1) { fn(std::integral_constant<int, 0>{}); }
    else if constexpr (NG == 2) { if (g == 0) fn(std::integral_constant<int, 0>{}); else fn(std::integral_constant<int, 1>{}); }
    else {
      static_assert(NG == 4, "8, 16 or 32 candidates per lane");
      if (g == 0) fn(std::integral_constant<int, 0>{});
      else if (g == 1) fn(std::integral_constant<int, 1>{});
      else if (g == 2) fn(std::integral_constant<int, 2>{});
      else fn(std::integral_constant<int, 3>{});
    }
  };
#pragma unroll
  for (int g = 0; g < NG; g++) for_group(g, rescan);
  for (int slot = p.num_init + p.num_local; slot < nsel; slot++) {
    float best = -2.f;
    int bj = 0x7fffffff;
#pragma unroll
    for (int g = 0; g < NG; g++)
      if (gbest[g] > best) { best = gbest[g]; bj = gidx[g]; }
    const int w = wave_argmax_lowest(best, bj, bj != 0x7fffffff);
    if (lane == slot) result = w;
    if (w > jmax) continue;  // wave-uniform: no candidate left
    const bool mine = (w & 63) == lane;
    const int kk = w >> 6;
    for_group(kk >> 3, [&](auto g_tag) {  // take the winner out of its group, then rescan that group only
      constexpr int g = decltype(g_tag)::value;
#pragma unroll
      for (int k = g * 8; k < g * 8 + 8; k++)
        if (mine && k == kk) v[k] = -1.f;
      rescan(g_tag);
    });
  }
  return result;
}


// wave-wide maximum of a float on the DPP crossbar, the same value in every lane
NSA_DEVICE float wave_fmax_uniform(float x) {
  float m = x;
  m = dpp_fmax_step<0x111, 0xf>(m);  // row_shr:1
  m = dpp_fmax_step<0x112, 0xf>(m);  // row_shr:2
  m = dpp_fmax_step<0x114, 0xf>(m);  // row_shr:4
  m = dpp_fmax_step<0x118, 0xf>(m);  // row_shr:8
  m = dpp_fmax_step<0x142, 0xa>(m);  // row_bcast:15
  m = dpp_fmax_step<0x143, 0xc>(m);  // row_bcast:31 -> lane 63 holds the wave maximum
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, m), 63));
}

// The same selection as select_blocks_regs, with the repeated arg-max run over a short list instead of the NV
// registers of every lane: the R-th largest of the 64 lane maxima is a lower bound of the R-th largest score (R =
// number of arg-max rounds), so only the scores at or above it can be selected; they are compacted (ballot + prefix
// count) into a wave-private list of at most 64 entries in LDS (cand_v / cand_i), one per lane, and a round is one
// wave reduction plus one compare.  The picks and their order are those of select_blocks_regs (descending score,
// lowest index on ties); rows with more than 64 scores at the bound (many equal values) take that function.
template <int NV, class P>
NSA_DEVICE int select_blocks_short_list(const float* imp, int t, int nb_cap, const P& p, int lane, float* cand_v,
                                        int* cand_i) {
  const int nk = t >= 0 ? t / p.block_size : -1;
  const int forced = p.num_init + p.num_local;
  const int nsel = min(p.top_n, nk + 1);
  const int rounds = nsel - forced;
  int result = p.ignore_index;
  if (lane < p.num_init) {
    if (lane <= nk) result = lane;
  } else if (lane < forced) {
    if (lane <= nk) result = nk - (lane - p.num_init);
  }
  if (rounds <= 0) return result;
  const int jmax = min(nk, nb_cap - 1);
  float v[NV];
  float m = -3.f;
#pragma unroll
  for (int k = 0; k < NV; k++) {
    const int j = lane + 64 * k;
    float x = j <= jmax ? imp[min(j, nb_cap - 1)] : -3.f;
    if (j <= jmax && (j < p.num_init || j > nk - p.num_local)) x = -1.f;  // forced blocks: behind every real score
    v[k] = x;
    m = fmaxf(m, x);
  }
  // bound: the lane maxima in descending order until `rounds` lanes are counted
  float theta = -1.f;
  int counted = 0;
  for (int r = 0; r < rounds; r++) {
    const float mx = wave_fmax_uniform(m);
    if (mx < -1.f) { theta = -1.f; break; }  // fewer lanes than rounds hold a candidate: everything is listed
    theta = mx;
    const bool hit = m == mx;
    counted += __builtin_popcountll(__builtin_amdgcn_ballot_w64(hit));
    if (hit) m = -4.f;
    if (counted >= rounds) break;
  }
  // compaction of the scores >= theta, register by register (ascending block number within a register)
  int base = 0;
#pragma unroll
  for (int k = 0; k < NV; k++) {
    const bool q = v[k] >= theta;
    const uint64_t mask = __builtin_amdgcn_ballot_w64(q);
    const int pos = base + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
    if (q && pos < 64) { cand_v[pos] = v[k]; cand_i[pos] = lane + 64 * k; }
    base += __builtin_popcountll(mask);
  }
  if (base > 64) return select_blocks_regs<NV>(imp, t, nb_cap, p, lane);  // wave-uniform
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  float cv = lane < base ? cand_v[lane] : -3.f;
  int ci = lane < base ? cand_i[lane] : 0x7fffffff;
  for (int slot = forced; slot < nsel; slot++) {
    const int w = wave_argmax_lowest(cv, ci, ci != 0x7fffffff);
    if (lane == slot) result = w;
    if (ci == w) ci = 0x7fffffff;
  }
  return result;
}

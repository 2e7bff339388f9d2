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


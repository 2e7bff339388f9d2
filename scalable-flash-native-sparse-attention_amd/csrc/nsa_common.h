// Shared device helpers for the gfx950 (CDNA4) Native-Sparse-Attention kernels.
//
// MFMA operand layouts used throughout (wave64, verified on hardware):
//   v_mfma_f32_32x32x16_bf16:  A[m][k]: lane l holds m = l%32, k = (l/32)*8 .. +7
//                              B[k][n]: lane l holds n = l%32, k = (l/32)*8 .. +7
//                              C[m][n]: lane l holds n = l%32, m = (i/4)*8 + (l/32)*4 + i%4, i = 0..15
//   v_mfma_f32_16x16x32_bf16:  A[m][k]: lane l holds m = l%16, k = (l/16)*8 .. +7
//                              B[k][n]: lane l holds n = l%16, k = (l/16)*8 .. +7
//                              C[m][n]: lane l holds n = l%16, m = (l/16)*4 + i, i = 0..3
// A C-tile can be fed back as the B operand of a following MFMA whose contraction runs over the C-tile's
// m index: the lane's accumulator values i = 8c .. 8c+7 are the k-slice of "virtual" k-chunk c, as long as the
// A operand of that MFMA is gathered with the same m -> k permutation (see frag_tr_* below).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define NSA_DEVICE __device__ __forceinline__
#define LDS_PTR(T) __attribute__((address_space(3))) T*

// Row padding (bf16 elements) of LDS tiles.  With 128-wide rows the stride is 76 dwords = 12 mod 64 banks: the
// 16-byte row-fragment reads of 16 consecutive rows and the 4-row x 32-byte groups of the transpose reads both
// land on distinct banks.
constexpr int NSA_LDS_PAD = 24;

constexpr float NSA_LOG2E = 1.4426950408889634f;
constexpr float NSA_LN2 = 0.6931471805599453f;
constexpr float NSA_NEG_INF = -__builtin_huge_valf();

NSA_DEVICE f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
NSA_DEVICE f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

NSA_DEVICE float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
NSA_DEVICE float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
NSA_DEVICE float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

NSA_DEVICE float bf16_bits_to_f32(uint32_t hi16) { return __builtin_bit_cast(float, hi16 << 16); }

// 16-byte global load of 8 bf16
NSA_DEVICE bf16x8 ld_global_b128(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }
NSA_DEVICE bf16x8 zero_bf16x8() {
  u32x4 z = {0, 0, 0, 0};
  return __builtin_bit_cast(bf16x8, z);
}

// pack 8 floats to bf16x8 (round to nearest even via the hardware convert)
NSA_DEVICE bf16x8 pack8(float a0, float a1, float a2, float a3, float a4, float a5, float a6, float a7) {
  bf16x8 r;
  r[0] = (bf16_t)a0; r[1] = (bf16_t)a1; r[2] = (bf16_t)a2; r[3] = (bf16_t)a3;
  r[4] = (bf16_t)a4; r[5] = (bf16_t)a5; r[6] = (bf16_t)a6; r[7] = (bf16_t)a7;
  return r;
}
NSA_DEVICE bf16x4 pack4(float a0, float a1, float a2, float a3) {
  bf16x4 r;
  r[0] = (bf16_t)a0; r[1] = (bf16_t)a1; r[2] = (bf16_t)a2; r[3] = (bf16_t)a3;
  return r;
}

// LDS transpose read (gfx950 ds_read_b64_tr_b16).  Within each group of 16 lanes, lane i receives
// element (i%4) of the 4-element rows addressed by lanes (i/4), (i/4)+4, (i/4)+8, (i/4)+12 of the group.
// With lane s of a group pointing at &M[row0 + s/4][col0 + 4*(s%4)] of a row-major bf16 matrix in LDS, lane i
// gets M[row0+0..3][col0 + i]: four consecutive rows of one column, i.e. a k-slice for an operand whose
// contraction index is the LDS row.
NSA_DEVICE bf16x4 lds_read_tr(const bf16_t* p) {
  s16x4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))p);
  return __builtin_bit_cast(bf16x4, r);
}
NSA_DEVICE bf16x8 cat4(bf16x4 a, bf16x4 b) {
  return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
}

// exchange between the two 32-lane halves of a wave on the VALU (v_permlane32_swap), no LDS crossbar round trip
NSA_DEVICE float xhalf_max(float v) {
  uint32_t b = __builtin_bit_cast(uint32_t, v);
  auto r = __builtin_amdgcn_permlane32_swap(b, b, false, false);
  return fmaxf(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
}
NSA_DEVICE float xhalf_sum(float v) {
  uint32_t b = __builtin_bit_cast(uint32_t, v);
  auto r = __builtin_amdgcn_permlane32_swap(b, b, false, false);
  return __builtin_bit_cast(float, (uint32_t)r[0]) + __builtin_bit_cast(float, (uint32_t)r[1]);
}

// exchange between neighbouring 16-lane rows (lane l <-> lane l ^ 16) on the VALU (v_permlane16_swap)
NSA_DEVICE float xrow_max(float v) {
  uint32_t b = __builtin_bit_cast(uint32_t, v);
  auto r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
  return fmaxf(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
}
NSA_DEVICE float xrow_sum(float v) {
  uint32_t b = __builtin_bit_cast(uint32_t, v);
  auto r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
  return __builtin_bit_cast(float, (uint32_t)r[0]) + __builtin_bit_cast(float, (uint32_t)r[1]);
}

NSA_DEVICE float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
NSA_DEVICE float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// ---- wave-wide arg-max over (score, index) pairs with "lowest index wins ties", on the DPP crossbar (no LDS
// traffic).  Scores must be finite.  A 32-bit float maximum is reduced first; the lanes that hold it are found with
// one ballot, and only when several lanes tie is a second reduction (minimum index) needed.  Returns the winning
// index in every lane (0x7fffffff if no lane had a candidate) and, on request, the winning score.
template <int CTRL, int ROW_MASK>
NSA_DEVICE float dpp_fmax_step(float x) {
  const int xi = __builtin_bit_cast(int, x);
  return fmaxf(x, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(xi, xi, CTRL, ROW_MASK, 0xf, false)));
}
template <int CTRL, int ROW_MASK>
NSA_DEVICE int dpp_imin_step(int x) {
  return min(x, __builtin_amdgcn_update_dpp(x, x, CTRL, ROW_MASK, 0xf, false));
}
NSA_DEVICE int wave_argmax_lowest_score(float score, int index, bool has_candidate, float& win_score) {
  float s = has_candidate ? score : -__builtin_inff();
  float m = s;
  m = dpp_fmax_step<0x111, 0xf>(m);  // row_shr:1
  m = dpp_fmax_step<0x112, 0xf>(m);  // row_shr:2
  m = dpp_fmax_step<0x114, 0xf>(m);  // row_shr:4
  m = dpp_fmax_step<0x118, 0xf>(m);  // row_shr:8   -> lane 15 of every row holds the row maximum
  m = dpp_fmax_step<0x142, 0xa>(m);  // row_bcast:15 into rows 1 and 3
  m = dpp_fmax_step<0x143, 0xc>(m);  // row_bcast:31 into rows 2 and 3 -> lane 63 holds the wave maximum
  m = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, m), 63));
  win_score = m;
  const uint64_t tied = __builtin_amdgcn_ballot_w64(has_candidate && s == m);
  if (tied == 0) return 0x7fffffff;
  if ((tied & (tied - 1)) == 0)  // one lane holds the maximum
    return __builtin_amdgcn_readlane(index, (int)__builtin_ctzll(tied));
  int i = (has_candidate && s == m) ? index : 0x7fffffff;
  i = dpp_imin_step<0x111, 0xf>(i);
  i = dpp_imin_step<0x112, 0xf>(i);
  i = dpp_imin_step<0x114, 0xf>(i);
  i = dpp_imin_step<0x118, 0xf>(i);
  i = dpp_imin_step<0x142, 0xa>(i);
  i = dpp_imin_step<0x143, 0xc>(i);
  return __builtin_amdgcn_readlane(i, 63);
}
NSA_DEVICE int wave_argmax_lowest(float score, int index, bool has_candidate) {
  float unused;
  return wave_argmax_lowest_score(score, index, has_candidate, unused);
}

__host__ __device__ inline int cdiv_i(int a, int b) { return (a + b - 1) / b; }

// error codes returned by the C entry points
enum {
  NSA_OK = 0,
  NSA_ERR_BAD_ARG = 1,
  NSA_ERR_UNSUPPORTED = 2,
  NSA_ERR_LAUNCH = 3,
  NSA_ERR_WORKSPACE = 4,
};

void nsa_set_error(const char* fmt, ...);
int nsa_tuning_knob(const char* name, int default_value);  // value given to nsa_set_tuning for this name, else the default
int nsa_check_launch(const char* what);

#define NSA_REQUIRE(cond, code, ...)        \
  do {                                      \
    if (!(cond)) {                          \
      nsa_set_error(__VA_ARGS__);           \
      return (code);                        \
    }                                       \
  } while (0)

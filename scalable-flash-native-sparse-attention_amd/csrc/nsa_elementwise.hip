// Bandwidth-bound kernels of the path: KV mean pooling (contiguous and paged), im2col of compression
// windows, the sigmoid-mul / swiglu activations, the sigmoid-gated combine and the delta pre-pass.
// Every thread moves 16-byte vectors; reductions over a head's channels run across the D/8 lanes that share
// a (token, head) pair.
// Upstream: flash_nsa/ops/compress_kv.py:17-426, flash_nsa/ops/act.py:13-208, flash_nsa/ops/combine.py:15-177,
//           flash_nsa/ops/compress_attn.py:160-184, flash_nsa/inference/compress_kv.py:13-287,
//           flash_nsa/inference/combine.py:16-127.
#include "nsa_common.h"
#include "nsa_api_internal.h"

namespace {

NSA_DEVICE void acc8(float* a, bf16x8 v) {
#pragma unroll
  for (int e = 0; e < 8; e++) a[e] += (float)v[e];
}
NSA_DEVICE float sigmoidf_(float x) { return 1.f / (1.f + __expf(-x)); }

// ------------------------------------------------------------------------------------------ mean pooling fwd
// grid (cdiv(y_maxlen*H*D/8, 256), B)
__global__ void mean_pool_fwd_kernel(const bf16_t* x, int64_t x_st, int64_t x_sh, bf16_t* y, int64_t y_st,
                                     int64_t y_sh, const int32_t* x_cu, const int32_t* y_cu, int H, int D, int K,
                                     int S) {
  const int b = blockIdx.y;
  const int x0 = x_cu[b], y0 = y_cu[b];
  const int yl = y_cu[b + 1] - y0;
  const int C = D / 8;
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)yl * H * C) return;
  int c = idx % C;
  int h = (idx / C) % H;
  int i = idx / ((int64_t)C * H);
  float a[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  const bf16_t* xp = x + (int64_t)(x0 + (int64_t)S * i) * x_st + (int64_t)h * x_sh + c * 8;
  for (int r = 0; r < K; r++) acc8(a, ld_global_b128(xp + r * x_st));
  float inv = 1.f / (float)K;
  *reinterpret_cast<bf16x8*>(y + (int64_t)(y0 + i) * y_st + (int64_t)h * y_sh + c * 8) =
      pack8(a[0] * inv, a[1] * inv, a[2] * inv, a[3] * inv, a[4] * inv, a[5] * inv, a[6] * inv, a[7] * inv);
}

// ------------------------------------------------------------------------------------------ mean pooling bwd
// dx[n] (+)= sum over windows containing n of dy[i]/K.  grid (cdiv(x_maxlen*H*D/8, 256), B)
template <bool DX_F32, bool ACCUM>
__global__ void mean_pool_bwd_kernel(const bf16_t* dy, int64_t dy_st, int64_t dy_sh, void* dxv, int64_t dx_st,
                                     int64_t dx_sh, const int32_t* x_cu, const int32_t* y_cu, int H, int D, int K,
                                     int S) {
  const int b = blockIdx.y;
  const int x0 = x_cu[b], y0 = y_cu[b];
  const int xl = x_cu[b + 1] - x0, yl = y_cu[b + 1] - y0;
  const int C = D / 8;
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)xl * H * C) return;
  int c = idx % C;
  int h = (idx / C) % H;
  int n = idx / ((int64_t)C * H);
  int i_lo = n - K + 1 <= 0 ? 0 : (n - K + 1 + S - 1) / S;
  int i_hi = min(n / S, yl - 1);
  float a[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int i = i_lo; i <= i_hi; i++)
    acc8(a, ld_global_b128(dy + (int64_t)(y0 + i) * dy_st + (int64_t)h * dy_sh + c * 8));
  float inv = 1.f / (float)K;
  int64_t off = (int64_t)(x0 + n) * dx_st + (int64_t)h * dx_sh + c * 8;
  if (DX_F32) {
    float* dx = (float*)dxv + off;
    f32x4 lo = {a[0] * inv, a[1] * inv, a[2] * inv, a[3] * inv};
    f32x4 hi = {a[4] * inv, a[5] * inv, a[6] * inv, a[7] * inv};
    if (ACCUM) {
      if (i_lo > i_hi) return;
      lo += *reinterpret_cast<f32x4*>(dx);
      hi += *reinterpret_cast<f32x4*>(dx + 4);
    }
    *reinterpret_cast<f32x4*>(dx) = lo;
    *reinterpret_cast<f32x4*>(dx + 4) = hi;
  } else {
    bf16_t* dx = (bf16_t*)dxv + off;
    *reinterpret_cast<bf16x8*>(dx) =
        pack8(a[0] * inv, a[1] * inv, a[2] * inv, a[3] * inv, a[4] * inv, a[5] * inv, a[6] * inv, a[7] * inv);
  }
}

// ------------------------------------------------------------------------------------------ im2col fwd / bwd
// y[i,h,r,:] = x[S*i+r,h,:]   grid (cdiv(y_maxlen*H*K*D/8,256), B); y contiguous [y_len,H,K,D]
__global__ void construct_block_fwd_kernel(const bf16_t* x, int64_t x_st, int64_t x_sh, bf16_t* y,
                                           const int32_t* x_cu, const int32_t* y_cu, int H, int D, int K, int S) {
  const int b = blockIdx.y;
  const int x0 = x_cu[b], y0 = y_cu[b];
  const int yl = y_cu[b + 1] - y0;
  const int C = D / 8;
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)yl * H * K * C) return;
  int c = idx % C;
  int r = (idx / C) % K;
  int h = (idx / ((int64_t)C * K)) % H;
  int i = idx / ((int64_t)C * K * H);
  bf16x8 v = ld_global_b128(x + (int64_t)(x0 + (int64_t)S * i + r) * x_st + (int64_t)h * x_sh + c * 8);
  *reinterpret_cast<bf16x8*>(y + (((int64_t)(y0 + i) * H + h) * K + r) * D + c * 8) = v;
}

// dx[n,h,:] (+)= sum_i dblock[i,h,n-S*i,:]
template <bool DX_F32, bool ACCUM>
__global__ void construct_block_bwd_kernel(const bf16_t* dyb, void* dxv, int64_t dx_st, int64_t dx_sh,
                                           const int32_t* x_cu, const int32_t* y_cu, int H, int D, int K, int S) {
  const int b = blockIdx.y;
  const int x0 = x_cu[b], y0 = y_cu[b];
  const int xl = x_cu[b + 1] - x0, yl = y_cu[b + 1] - y0;
  const int C = D / 8;
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)xl * H * C) return;
  int c = idx % C;
  int h = (idx / C) % H;
  int n = idx / ((int64_t)C * H);
  int i_lo = n - K + 1 <= 0 ? 0 : (n - K + 1 + S - 1) / S;
  int i_hi = min(n / S, yl - 1);
  float a[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int i = i_lo; i <= i_hi; i++)
    acc8(a, ld_global_b128(dyb + (((int64_t)(y0 + i) * H + h) * K + (n - S * i)) * D + c * 8));
  int64_t off = (int64_t)(x0 + n) * dx_st + (int64_t)h * dx_sh + c * 8;
  if (DX_F32) {
    float* dx = (float*)dxv + off;
    f32x4 lo = {a[0], a[1], a[2], a[3]};
    f32x4 hi = {a[4], a[5], a[6], a[7]};
    if (ACCUM) {
      if (i_lo > i_hi) return;
      lo += *reinterpret_cast<f32x4*>(dx);
      hi += *reinterpret_cast<f32x4*>(dx + 4);
    }
    *reinterpret_cast<f32x4*>(dx) = lo;
    *reinterpret_cast<f32x4*>(dx + 4) = hi;
  } else {
    *reinterpret_cast<bf16x8*>((bf16_t*)dxv + off) = pack8(a[0], a[1], a[2], a[3], a[4], a[5], a[6], a[7]);
  }
}

// ------------------------------------------------------------------------------------------ gated activations
// x [N, 2*d] (gate | up) -> y [N, d];  ACT 0: sigmoid(gate)*up, 1: silu(gate)*up
template <int ACT>
__global__ void glu_fwd_kernel(const bf16_t* x, bf16_t* y, int64_t N, int d) {
  const int C = d / 8;
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= N * C) return;
  int c = idx % C;
  int64_t n = idx / C;
  bf16x8 g = ld_global_b128(x + n * 2 * d + c * 8);
  bf16x8 u = ld_global_b128(x + n * 2 * d + d + c * 8);
  float o[8];
#pragma unroll
  for (int e = 0; e < 8; e++) {
    float gf = (float)g[e], uf = (float)u[e];
    float s = sigmoidf_(gf);
    o[e] = (ACT == 0 ? s : s * gf) * uf;
  }
  *reinterpret_cast<bf16x8*>(y + n * d + c * 8) = pack8(o[0], o[1], o[2], o[3], o[4], o[5], o[6], o[7]);
}
// dx [N, 2*d] = [dgate | dup]; may alias x (each thread reads its inputs before writing)
template <int ACT>
__global__ void glu_bwd_kernel(const bf16_t* x, const bf16_t* dy, bf16_t* dx, int64_t N, int d) {
  const int C = d / 8;
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= N * C) return;
  int c = idx % C;
  int64_t n = idx / C;
  bf16x8 g = ld_global_b128(x + n * 2 * d + c * 8);
  bf16x8 u = ld_global_b128(x + n * 2 * d + d + c * 8);
  bf16x8 go = ld_global_b128(dy + n * d + c * 8);
  float dg[8], du[8];
#pragma unroll
  for (int e = 0; e < 8; e++) {
    float gf = (float)g[e], uf = (float)u[e], d0 = (float)go[e];
    float s = sigmoidf_(gf);
    if (ACT == 0) {
      du[e] = d0 * s;
      dg[e] = d0 * uf * s * (1.f - s);
    } else {
      du[e] = d0 * s * gf;
      dg[e] = d0 * uf * (s + gf * s * (1.f - s));
    }
  }
  *reinterpret_cast<bf16x8*>(dx + n * 2 * d + c * 8) = pack8(dg[0], dg[1], dg[2], dg[3], dg[4], dg[5], dg[6], dg[7]);
  *reinterpret_cast<bf16x8*>(dx + n * 2 * d + d + c * 8) =
      pack8(du[0], du[1], du[2], du[3], du[4], du[5], du[6], du[7]);
}

// ------------------------------------------------------------------------------------------ combine
// o = a*sig(w0) + b*sig(w1) + c*sig(w2).  One thread per 8 channels; grid cdiv(T*H*D/8, 256)
__global__ void combine_fwd_kernel(const bf16_t* a, const bf16_t* bb, const bf16_t* c, int64_t i_st, int64_t i_sh,
                                   const bf16_t* w, int64_t w_st, int64_t w_sh, bf16_t* o, int64_t o_st,
                                   int64_t o_sh, int64_t T, int H, int D) {
  const int C = D / 8;
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= T * H * C) return;
  int cc = idx % C;
  int h = (idx / C) % H;
  int64_t t = idx / ((int64_t)C * H);
  const bf16_t* wp = w + t * w_st + (int64_t)h * w_sh;
  float s0 = sigmoidf_((float)wp[0]), s1 = sigmoidf_((float)wp[1]), s2 = sigmoidf_((float)wp[2]);
  int64_t off = t * i_st + (int64_t)h * i_sh + cc * 8;
  bf16x8 va = ld_global_b128(a + off), vb = ld_global_b128(bb + off), vc = ld_global_b128(c + off);
  float r[8];
#pragma unroll
  for (int e = 0; e < 8; e++) r[e] = (float)va[e] * s0 + (float)vb[e] * s1 + (float)vc[e] * s2;
  *reinterpret_cast<bf16x8*>(o + t * o_st + (int64_t)h * o_sh + cc * 8) =
      pack8(r[0], r[1], r[2], r[3], r[4], r[5], r[6], r[7]);
}

// backward: da,db,dc = dy*sig(w_k); dw_k = sig_k(1-sig_k) * sum_d dy*x_k; optional delta_k = rowsum(x_k * d x_k)
// with the stored (bf16) d x_k, the softmax-backward correction term of branch k, written as delta[k][T][H] fp32.
// D/8 consecutive lanes share one (t,h); D/8 must be a power of two <= 64.
__global__ void combine_bwd_kernel(const bf16_t* a, const bf16_t* bb, const bf16_t* c, int64_t i_st, int64_t i_sh,
                                   const bf16_t* w, int64_t w_st, int64_t w_sh, const bf16_t* dy, int64_t dy_st,
                                   int64_t dy_sh, bf16_t* da, bf16_t* db, bf16_t* dc, bf16_t* dw, float* delta,
                                   int64_t T, int H, int D) {
  const int C = D / 8;
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  bool ok = idx < T * H * C;
  if (!ok) idx = T * H * C - 1;
  int cc = idx % C;
  int h = (idx / C) % H;
  int64_t t = idx / ((int64_t)C * H);
  const bf16_t* wp = w + t * w_st + (int64_t)h * w_sh;
  float s0 = sigmoidf_((float)wp[0]), s1 = sigmoidf_((float)wp[1]), s2 = sigmoidf_((float)wp[2]);
  int64_t off = t * i_st + (int64_t)h * i_sh + cc * 8;
  bf16x8 va = ld_global_b128(a + off), vb = ld_global_b128(bb + off), vc = ld_global_b128(c + off);
  bf16x8 g = ld_global_b128(dy + t * dy_st + (int64_t)h * dy_sh + cc * 8);
  // p_k = sum_d dy * x_k (gate gradient); q_k = sum_d round(dy * sig_k) * x_k: the correction term is formed from
  // the ROUNDED branch gradient, the one the attention backward kernels read, so that dP - delta cancels exactly
  // where a row's probabilities are one-hot (upstream forms it the same way from the stored bf16 tensors,
  // flash_nsa/ops/compress_attn.py:160-184)
  float p0 = 0.f, p1 = 0.f, p2 = 0.f, q0 = 0.f, q1 = 0.f, q2 = 0.f;
  bf16x8 ra, rb, rc;
#pragma unroll
  for (int e = 0; e < 8; e++) {
    float gf = (float)g[e];
    float xa = (float)va[e], xb = (float)vb[e], xc = (float)vc[e];
    ra[e] = (bf16_t)(gf * s0); rb[e] = (bf16_t)(gf * s1); rc[e] = (bf16_t)(gf * s2);
    p0 += gf * xa; p1 += gf * xb; p2 += gf * xc;
    q0 += (float)ra[e] * xa; q1 += (float)rb[e] * xb; q2 += (float)rc[e] * xc;
  }
  for (int o = C >> 1; o > 0; o >>= 1) {
    p0 += __shfl_xor(p0, o, 64); p1 += __shfl_xor(p1, o, 64); p2 += __shfl_xor(p2, o, 64);
    q0 += __shfl_xor(q0, o, 64); q1 += __shfl_xor(q1, o, 64); q2 += __shfl_xor(q2, o, 64);
  }
  if (!ok) return;
  int64_t ooff = (t * H + h) * (int64_t)D + cc * 8;  // grads are contiguous [T,H,D]
  *reinterpret_cast<bf16x8*>(da + ooff) = ra;
  *reinterpret_cast<bf16x8*>(db + ooff) = rb;
  *reinterpret_cast<bf16x8*>(dc + ooff) = rc;
  if (cc == 0) {
    bf16_t* dwp = dw + (t * H + h) * 3;
    dwp[0] = (bf16_t)(s0 * (1.f - s0) * p0);
    dwp[1] = (bf16_t)(s1 * (1.f - s1) * p1);
    dwp[2] = (bf16_t)(s2 * (1.f - s2) * p2);
    if (delta != nullptr) {
      int64_t TH = T * H;
      delta[0 * TH + t * H + h] = q0;
      delta[1 * TH + t * H + h] = q1;
      delta[2 * TH + t * H + h] = q2;
    }
  }
}

// delta[t,h] = sum_d o*do   (fp32, contiguous [T,H])
__global__ void delta_kernel(const bf16_t* o, int64_t o_st, int64_t o_sh, const bf16_t* dO, int64_t d_st,
                             int64_t d_sh, float* delta, int64_t T, int H, int D) {
  const int C = D / 8;
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  bool ok = idx < T * H * C;
  if (!ok) idx = T * H * C - 1;
  int cc = idx % C;
  int h = (idx / C) % H;
  int64_t t = idx / ((int64_t)C * H);
  bf16x8 vo = ld_global_b128(o + t * o_st + (int64_t)h * o_sh + cc * 8);
  bf16x8 vd = ld_global_b128(dO + t * d_st + (int64_t)h * d_sh + cc * 8);
  float s = 0.f;
#pragma unroll
  for (int e = 0; e < 8; e++) s += (float)vo[e] * (float)vd[e];
  for (int o2 = C >> 1; o2 > 0; o2 >>= 1) s += __shfl_xor(s, o2, 64);
  if (ok && cc == 0) delta[t * H + h] = s;
}

// ------------------------------------------------------------------------------------------ paged pooling
// prefill: one compressed row per (entry e, head, chunk); rows read through the raw block table, written to flat
// pool row slot[e] unless slot[e] < 0.   grid (cdiv(y_maxlen*H*C,256), B)
__global__ void paged_pool_prefill_kernel(bf16_t* cache, int64_t c_sr, int64_t c_sh, const int32_t* y_cu,
                                          const int32_t* table, int table_stride, const int32_t* slots,
                                          int page, int H, int D, int K, int S) {
  const int b = blockIdx.y;
  const int y0 = y_cu[b];
  const int yl = y_cu[b + 1] - y0;
  const int C = D / 8;
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)yl * H * C) return;
  int c = idx % C;
  int h = (idx / C) % H;
  int i = idx / ((int64_t)C * H);
  int slot = slots[y0 + i];
  if (slot < 0) return;
  const int32_t* tb = table + (int64_t)b * table_stride;
  float a[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int r = 0; r < K; r++) {
    int n = S * i + r;
    int64_t row = (int64_t)tb[n / page] * page + (n % page);
    acc8(a, ld_global_b128(cache + row * c_sr + (int64_t)h * c_sh + c * 8));
  }
  float inv = 1.f / (float)K;
  *reinterpret_cast<bf16x8*>(cache + (int64_t)slot * c_sr + (int64_t)h * c_sh + c * 8) =
      pack8(a[0] * inv, a[1] * inv, a[2] * inv, a[3] * inv, a[4] * inv, a[5] * inv, a[6] * inv, a[7] * inv);
}

// decode: per request, pool the last complete window of K (blockIdx.z = 0) and V (= 1) if slot >= 0 and len >= K.
// grid (cdiv(H*C, 64), B, 2), block 64
__global__ void paged_pool_decode_kernel(bf16_t* kc, int64_t k_sr, int64_t k_sh, int Dk, bf16_t* vc, int64_t v_sr,
                                         int64_t v_sh, int Dv, const int32_t* ctx_lens, const int32_t* table,
                                         int table_stride, const int32_t* slots, int page, int H, int K, int S) {
  const int b = blockIdx.y;
  const int slot = slots[b];
  const int L = ctx_lens[b];
  if (slot < 0 || L < K) return;
  bf16_t* cache = blockIdx.z == 0 ? kc : vc;
  const int64_t c_sr = blockIdx.z == 0 ? k_sr : v_sr, c_sh = blockIdx.z == 0 ? k_sh : v_sh;
  const int D = blockIdx.z == 0 ? Dk : Dv;
  const int C = D / 8;
  int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= H * C) return;
  int c = idx % C, h = idx / C;
  const int st = ((L - K) / S) * S;
  const int32_t* tb = table + (int64_t)b * table_stride;
  float a[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  if (K <= page) {
    // the window touches at most two pages: both table entries are read up front, then the rows are fetched eight at
    // a time (independent loads) and added in row order
    const int p0 = st / page, r0 = st - p0 * page;
    const int64_t base0 = (int64_t)tb[p0] * page + r0;
    const int64_t base1 = r0 + K > page ? (int64_t)tb[p0 + 1] * page + r0 - page : base0;
    const bf16_t* col = cache + (int64_t)h * c_sh + c * 8;
    for (int r = 0; r < K; r += 8) {
      bf16x8 x[8];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int rr = min(r + u, K - 1);
        x[u] = ld_global_b128(col + ((r0 + rr < page ? base0 : base1) + rr) * c_sr);
      }
#pragma unroll
      for (int u = 0; u < 8; u++)
        if (r + u < K) acc8(a, x[u]);
    }
  } else {
    for (int r = 0; r < K; r++) {
      int n = st + r;
      int64_t row = (int64_t)tb[n / page] * page + (n % page);
      acc8(a, ld_global_b128(cache + row * c_sr + (int64_t)h * c_sh + c * 8));
    }
  }
  float inv = 1.f / (float)K;
  *reinterpret_cast<bf16x8*>(cache + (int64_t)slot * c_sr + (int64_t)h * c_sh + c * 8) =
      pack8(a[0] * inv, a[1] * inv, a[2] * inv, a[3] * inv, a[4] * inv, a[5] * inv, a[6] * inv, a[7] * inv);
}

// ------------------------------------------------------------------------------------------ KV-cache writer
// store_kvcache (upstream nano-vllm/nanovllm/layers/attention.py:123-153): row n of key / value goes to flat pool
// row slot[n] (skipped when negative).  grid (cdiv(N*max(Wk,Wv)/8, 256), 2): y = 0 copies K, y = 1 copies V.
__global__ void store_kvcache_kernel(const bf16_t* key, int64_t k_st, const bf16_t* value, int64_t v_st,
                                     bf16_t* kc, int64_t kc_sr, bf16_t* vc, int64_t vc_sr, const int32_t* slots,
                                     int N, int Wk, int Wv) {
  const bool is_v = blockIdx.y == 1;
  const int C = (is_v ? Wv : Wk) / 8;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)N * C) return;
  const int n = idx / C, c = idx - (int64_t)n * C;
  const int slot = slots[n];
  if (slot < 0) return;
  if (is_v) *reinterpret_cast<bf16x8*>(vc + (int64_t)slot * vc_sr + c * 8) = ld_global_b128(value + n * v_st + c * 8);
  else *reinterpret_cast<bf16x8*>(kc + (int64_t)slot * kc_sr + c * 8) = ld_global_b128(key + n * k_st + c * 8);
}

// Prefill chunk in one launch: scatter the chunk's new K/V rows into the pool AND pool the compressed rows that the
// chunk completes.  A pooled row reads a source row from the chunk itself when that row is new (position >=
// context - new tokens) and from the pool otherwise, so the two halves of the kernel do not depend on each other.
// grid (cdiv(max(new_max, y_max)*H*C, 256), B, 2): z = 0 K, z = 1 V.
__global__ void paged_store_pool_prefill_kernel(const bf16_t* key, int64_t k_st, int64_t k_sh, int Dk,
                                                const bf16_t* value, int64_t v_st, int64_t v_sh, int Dv,
                                                bf16_t* kc, int64_t kc_sr, int64_t kc_sh, bf16_t* vc, int64_t vc_sr,
                                                int64_t vc_sh, const int32_t* x_cu, const int32_t* ctx_lens,
                                                const int32_t* slots, const int32_t* y_cu, const int32_t* cmp_slots,
                                                const int32_t* table, int table_stride, int page, int H, int K,
                                                int S) {
  const bool is_v = blockIdx.z == 1;
  const bf16_t* src = is_v ? value : key;
  const int64_t s_st = is_v ? v_st : k_st, s_sh = is_v ? v_sh : k_sh;
  bf16_t* cache = is_v ? vc : kc;
  const int64_t c_sr = is_v ? vc_sr : kc_sr, c_sh = is_v ? vc_sh : kc_sh;
  const int D = is_v ? Dv : Dk;
  const int C = D / 8;
  const int b = blockIdx.y;
  const int x0 = x_cu[b], xl = x_cu[b + 1] - x0;
  const int y0 = y_cu[b], yl = y_cu[b + 1] - y0;
  const int cached = ctx_lens[b] - xl;  // tokens of the request that are in the pool already
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int c = idx % C;
  const int h = (idx / C) % H;
  const int i = idx / ((int64_t)C * H);
  if (i < xl) {  // scatter new token i of the request
    const int slot = slots[x0 + i];
    if (slot >= 0)
      *reinterpret_cast<bf16x8*>(cache + (int64_t)slot * c_sr + (int64_t)h * c_sh + c * 8) =
          ld_global_b128(src + (int64_t)(x0 + i) * s_st + (int64_t)h * s_sh + c * 8);
  }
  if (i < yl) {  // compressed row i of the request
    const int slot = cmp_slots[y0 + i];
    if (slot < 0) return;
    const int32_t* tb = table + (int64_t)b * table_stride;
    float a[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int r = 0; r < K; r++) {
      const int n = S * i + r;
      if (n >= cached) {
        acc8(a, ld_global_b128(src + (int64_t)(x0 + n - cached) * s_st + (int64_t)h * s_sh + c * 8));
      } else {
        const int64_t row = (int64_t)tb[n / page] * page + (n % page);
        acc8(a, ld_global_b128(cache + row * c_sr + (int64_t)h * c_sh + c * 8));
      }
    }
    const float inv = 1.f / (float)K;
    *reinterpret_cast<bf16x8*>(cache + (int64_t)slot * c_sr + (int64_t)h * c_sh + c * 8) =
        pack8(a[0] * inv, a[1] * inv, a[2] * inv, a[3] * inv, a[4] * inv, a[5] * inv, a[6] * inv, a[7] * inv);
  }
}

// ------------------------------------------------------------------------------------------ rotary embedding
// Rotate-half RoPE of q and k of one token in one pass (upstream flash_nsa/ops/rope.py:13-124): with H = D/2,
//   out[:H] = x[:H]*cos[:H] - x[H:]*sin[:H],   out[H:] = x[H:]*cos[H:] + x[:H]*sin[H:]
// and for the backward the inverse rotation (sin halves swapped and negated).  A thread owns 8 channels of the
// first half and the matching 8 of the second half, so in-place operation is safe; it reads its slice of the
// token's tables once and walks the heads (q heads, then k heads) in batches whose loads are all issued before
// the first store.
// grid (N, B), block 256: thread = (head slot, channel octet), 256 / (D/16) head slots
__device__ inline void load_table8(const float* p, float (&v)[8]) {
  const float4 lo = *reinterpret_cast<const float4*>(p), hi = *reinterpret_cast<const float4*>(p + 4);
  v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w, v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
}
__device__ inline void load_table8(const bf16_t* p, float (&v)[8]) {
  const bf16x8 t = ld_global_b128(p);
#pragma unroll
  for (int e = 0; e < 8; e++) v[e] = (float)t[e];
}

template <typename CS>
__global__ __launch_bounds__(256) void rope_kernel(
    const bf16_t* q, int64_t q_sb, int64_t q_sn, int64_t q_sh, const bf16_t* k, int64_t k_sb, int64_t k_sn,
    int64_t k_sh, bf16_t* qe, int64_t qe_sb, int64_t qe_sn, int64_t qe_sh, bf16_t* ke, int64_t ke_sb, int64_t ke_sn,
    int64_t ke_sh, const CS* cos_, const CS* sin_, int64_t c_sb, int64_t c_sn, int QH, int KH, int D, int backward) {
  constexpr int U = 3;
  const int H2 = D / 2, C = H2 / 8, HT = QH + KH, slots = 256 / C;
  const int c = threadIdx.x % C, hs = threadIdx.x / C;
  if (hs >= slots) return;
  const int64_t n = blockIdx.x, b = blockIdx.y;
  float c1[8], c2[8], s1[8], s2[8];
  {
    const CS* cp = cos_ + b * c_sb + n * c_sn + c * 8;
    const CS* sp = sin_ + b * c_sb + n * c_sn + c * 8;
    load_table8(cp, c1), load_table8(cp + H2, c2);
    if (backward) {
      load_table8(sp + H2, s1), load_table8(sp, s2);
#pragma unroll
      for (int e = 0; e < 8; e++) s1[e] = -s1[e], s2[e] = -s2[e];
    } else {
      load_table8(sp, s1), load_table8(sp + H2, s2);
    }
  }
  const bf16_t* qrow = q + b * q_sb + n * q_sn + c * 8;
  const bf16_t* krow = k + b * k_sb + n * k_sn + c * 8;
  bf16_t* qerow = qe + b * qe_sb + n * qe_sn + c * 8;
  bf16_t* kerow = ke + b * ke_sb + n * ke_sn + c * 8;
  for (int h0 = hs; h0 < HT; h0 += U * slots) {
    bf16x8 x1[U], x2[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int h = h0 + u * slots;
      if (h < HT) {
        const bf16_t* src = h >= QH ? krow + (int64_t)(h - QH) * k_sh : qrow + (int64_t)h * q_sh;
        x1[u] = ld_global_b128(src), x2[u] = ld_global_b128(src + H2);
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      const int h = h0 + u * slots;
      if (h < HT) {
        float o1[8], o2[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
          const float a = (float)x1[u][e], bb = (float)x2[u][e];
          o1[e] = a * c1[e] - bb * s1[e];
          o2[e] = bb * c2[e] + a * s2[e];
        }
        bf16_t* dst = h >= QH ? kerow + (int64_t)(h - QH) * ke_sh : qerow + (int64_t)h * qe_sh;
        *reinterpret_cast<bf16x8*>(dst) = pack8(o1[0], o1[1], o1[2], o1[3], o1[4], o1[5], o1[6], o1[7]);
        *reinterpret_cast<bf16x8*>(dst + H2) = pack8(o2[0], o2[1], o2[2], o2[3], o2[4], o2[5], o2[6], o2[7]);
      }
    }
  }
}

inline unsigned blocks_for(int64_t n, int bs) { return (unsigned)((n + bs - 1) / bs); }

}  // namespace

// ============================================================================================== C entry points
extern "C" {

int nsa_mean_pool_fwd(const void* x, int64_t x_st, int64_t x_sh, void* y, int64_t y_st, int64_t y_sh,
                      const int32_t* x_cu, const int32_t* y_cu, int B, int y_maxlen, int H, int D, int kernel_size,
                      int stride, void* stream) {
  NSA_REQUIRE(D % 8 == 0 && D > 0, NSA_ERR_BAD_ARG, "mean_pool_fwd: head dim %d must be a multiple of 8", D);
  if (B <= 0 || y_maxlen <= 0) return NSA_OK;
  dim3 grid(blocks_for((int64_t)y_maxlen * H * (D / 8), 256), B);
  mean_pool_fwd_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const bf16_t*)x, x_st, x_sh, (bf16_t*)y, y_st, y_sh,
                                                              x_cu, y_cu, H, D, kernel_size, stride);
  return nsa_check_launch("mean_pool_fwd");
}

int nsa_mean_pool_bwd(const void* dy, int64_t dy_st, int64_t dy_sh, void* dx, int64_t dx_st, int64_t dx_sh,
                      int dx_is_f32, int accumulate, const int32_t* x_cu, const int32_t* y_cu, int B, int x_maxlen,
                      int H, int D, int kernel_size, int stride, void* stream) {
  NSA_REQUIRE(D % 8 == 0 && D > 0, NSA_ERR_BAD_ARG, "mean_pool_bwd: head dim %d must be a multiple of 8", D);
  NSA_REQUIRE(dx_is_f32 || !accumulate, NSA_ERR_BAD_ARG, "mean_pool_bwd: accumulation needs an fp32 dx");
  if (B <= 0 || x_maxlen <= 0) return NSA_OK;
  dim3 grid(blocks_for((int64_t)x_maxlen * H * (D / 8), 256), B);
  hipStream_t s = (hipStream_t)stream;
  const bf16_t* g = (const bf16_t*)dy;
  if (dx_is_f32 && accumulate)
    mean_pool_bwd_kernel<true, true><<<grid, 256, 0, s>>>(g, dy_st, dy_sh, dx, dx_st, dx_sh, x_cu, y_cu, H, D, kernel_size, stride);
  else if (dx_is_f32)
    mean_pool_bwd_kernel<true, false><<<grid, 256, 0, s>>>(g, dy_st, dy_sh, dx, dx_st, dx_sh, x_cu, y_cu, H, D, kernel_size, stride);
  else
    mean_pool_bwd_kernel<false, false><<<grid, 256, 0, s>>>(g, dy_st, dy_sh, dx, dx_st, dx_sh, x_cu, y_cu, H, D, kernel_size, stride);
  return nsa_check_launch("mean_pool_bwd");
}

int nsa_construct_block_fwd(const void* x, int64_t x_st, int64_t x_sh, void* y, const int32_t* x_cu,
                            const int32_t* y_cu, int B, int y_maxlen, int H, int D, int kernel_size, int stride,
                            void* stream) {
  NSA_REQUIRE(D % 8 == 0 && D > 0, NSA_ERR_BAD_ARG, "construct_block_fwd: head dim %d must be a multiple of 8", D);
  if (B <= 0 || y_maxlen <= 0) return NSA_OK;
  dim3 grid(blocks_for((int64_t)y_maxlen * H * kernel_size * (D / 8), 256), B);
  construct_block_fwd_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const bf16_t*)x, x_st, x_sh, (bf16_t*)y, x_cu,
                                                                    y_cu, H, D, kernel_size, stride);
  return nsa_check_launch("construct_block_fwd");
}

int nsa_construct_block_bwd(const void* dblock, void* dx, int64_t dx_st, int64_t dx_sh, int dx_is_f32,
                            int accumulate, const int32_t* x_cu, const int32_t* y_cu, int B, int x_maxlen, int H,
                            int D, int kernel_size, int stride, void* stream) {
  NSA_REQUIRE(D % 8 == 0 && D > 0, NSA_ERR_BAD_ARG, "construct_block_bwd: head dim %d must be a multiple of 8", D);
  NSA_REQUIRE(dx_is_f32 || !accumulate, NSA_ERR_BAD_ARG, "construct_block_bwd: accumulation needs an fp32 dx");
  if (B <= 0 || x_maxlen <= 0) return NSA_OK;
  dim3 grid(blocks_for((int64_t)x_maxlen * H * (D / 8), 256), B);
  hipStream_t s = (hipStream_t)stream;
  const bf16_t* g = (const bf16_t*)dblock;
  if (dx_is_f32 && accumulate)
    construct_block_bwd_kernel<true, true><<<grid, 256, 0, s>>>(g, dx, dx_st, dx_sh, x_cu, y_cu, H, D, kernel_size, stride);
  else if (dx_is_f32)
    construct_block_bwd_kernel<true, false><<<grid, 256, 0, s>>>(g, dx, dx_st, dx_sh, x_cu, y_cu, H, D, kernel_size, stride);
  else
    construct_block_bwd_kernel<false, false><<<grid, 256, 0, s>>>(g, dx, dx_st, dx_sh, x_cu, y_cu, H, D, kernel_size, stride);
  return nsa_check_launch("construct_block_bwd");
}

int nsa_glu_fwd(const void* x, void* y, int64_t N, int d, int act, void* stream) {
  NSA_REQUIRE(d % 8 == 0 && d > 0, NSA_ERR_BAD_ARG, "glu_fwd: width %d must be a multiple of 8", d);
  NSA_REQUIRE(act == 0 || act == 1, NSA_ERR_BAD_ARG, "glu_fwd: act must be 0 (sigmoid-mul) or 1 (swiglu)");
  if (N <= 0) return NSA_OK;
  unsigned g = blocks_for(N * (d / 8), 256);
  if (act == 0) glu_fwd_kernel<0><<<g, 256, 0, (hipStream_t)stream>>>((const bf16_t*)x, (bf16_t*)y, N, d);
  else glu_fwd_kernel<1><<<g, 256, 0, (hipStream_t)stream>>>((const bf16_t*)x, (bf16_t*)y, N, d);
  return nsa_check_launch("glu_fwd");
}

int nsa_glu_bwd(const void* x, const void* dy, void* dx, int64_t N, int d, int act, void* stream) {
  NSA_REQUIRE(d % 8 == 0 && d > 0, NSA_ERR_BAD_ARG, "glu_bwd: width %d must be a multiple of 8", d);
  NSA_REQUIRE(act == 0 || act == 1, NSA_ERR_BAD_ARG, "glu_bwd: act must be 0 (sigmoid-mul) or 1 (swiglu)");
  if (N <= 0) return NSA_OK;
  unsigned g = blocks_for(N * (d / 8), 256);
  if (act == 0) glu_bwd_kernel<0><<<g, 256, 0, (hipStream_t)stream>>>((const bf16_t*)x, (const bf16_t*)dy, (bf16_t*)dx, N, d);
  else glu_bwd_kernel<1><<<g, 256, 0, (hipStream_t)stream>>>((const bf16_t*)x, (const bf16_t*)dy, (bf16_t*)dx, N, d);
  return nsa_check_launch("glu_bwd");
}

int nsa_combine_fwd(const void* a, const void* b, const void* c, int64_t i_st, int64_t i_sh, const void* w,
                    int64_t w_st, int64_t w_sh, void* o, int64_t o_st, int64_t o_sh, int64_t T, int H, int D,
                    void* stream) {
  NSA_REQUIRE(D % 8 == 0 && D > 0, NSA_ERR_BAD_ARG, "combine_fwd: head dim %d must be a multiple of 8", D);
  if (T <= 0) return NSA_OK;
  combine_fwd_kernel<<<blocks_for(T * H * (D / 8), 256), 256, 0, (hipStream_t)stream>>>(
      (const bf16_t*)a, (const bf16_t*)b, (const bf16_t*)c, i_st, i_sh, (const bf16_t*)w, w_st, w_sh, (bf16_t*)o, o_st,
      o_sh, T, H, D);
  return nsa_check_launch("combine_fwd");
}

int nsa_combine_bwd(const void* a, const void* b, const void* c, int64_t i_st, int64_t i_sh, const void* w,
                    int64_t w_st, int64_t w_sh, const void* dy, int64_t dy_st, int64_t dy_sh, void* da, void* db,
                    void* dc, void* dw, float* delta3, int64_t T, int H, int D, void* stream) {
  int C = D / 8;
  NSA_REQUIRE(D % 8 == 0 && C > 0 && C <= 64 && (C & (C - 1)) == 0, NSA_ERR_BAD_ARG,
              "combine_bwd: head dim %d must be 8 * a power of two <= 512", D);
  if (T <= 0) return NSA_OK;
  combine_bwd_kernel<<<blocks_for(T * H * C, 256), 256, 0, (hipStream_t)stream>>>(
      (const bf16_t*)a, (const bf16_t*)b, (const bf16_t*)c, i_st, i_sh, (const bf16_t*)w, w_st, w_sh, (const bf16_t*)dy,
      dy_st, dy_sh, (bf16_t*)da, (bf16_t*)db, (bf16_t*)dc, (bf16_t*)dw, delta3, T, H, D);
  return nsa_check_launch("combine_bwd");
}

int nsa_delta(const void* o, int64_t o_st, int64_t o_sh, const void* dO, int64_t d_st, int64_t d_sh, float* delta,
              int64_t T, int H, int D, void* stream) {
  int C = D / 8;
  NSA_REQUIRE(D % 8 == 0 && C > 0 && C <= 64 && (C & (C - 1)) == 0, NSA_ERR_BAD_ARG,
              "delta: head dim %d must be 8 * a power of two <= 512", D);
  if (T <= 0) return NSA_OK;
  delta_kernel<<<blocks_for(T * H * C, 256), 256, 0, (hipStream_t)stream>>>((const bf16_t*)o, o_st, o_sh,
                                                                            (const bf16_t*)dO, d_st, d_sh, delta, T, H, D);
  return nsa_check_launch("delta");
}

int nsa_paged_pool_prefill(void* cache, int64_t c_sr, int64_t c_sh, const int32_t* y_cu, const int32_t* block_tables,
                           int table_stride, const int32_t* cmp_slot_mapping, int B, int y_maxlen, int page_size,
                           int H, int D, int kernel_size, int stride, void* stream) {
  NSA_REQUIRE(D % 8 == 0 && D > 0, NSA_ERR_BAD_ARG, "paged_pool_prefill: head dim %d must be a multiple of 8", D);
  if (B <= 0 || y_maxlen <= 0) return NSA_OK;
  dim3 grid(blocks_for((int64_t)y_maxlen * H * (D / 8), 256), B);
  paged_pool_prefill_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((bf16_t*)cache, c_sr, c_sh, y_cu, block_tables,
                                                                   table_stride, cmp_slot_mapping, page_size, H, D,
                                                                   kernel_size, stride);
  return nsa_check_launch("paged_pool_prefill");
}

int nsa_paged_pool_decode(void* k_cache, int64_t k_sr, int64_t k_sh, int Dk, void* v_cache, int64_t v_sr,
                          int64_t v_sh, int Dv, const int32_t* context_lens, const int32_t* block_tables,
                          int table_stride, const int32_t* cmp_slot_mapping, int B, int page_size, int H,
                          int kernel_size, int stride, void* stream) {
  NSA_REQUIRE(Dk % 8 == 0 && Dv % 8 == 0, NSA_ERR_BAD_ARG, "paged_pool_decode: head dims must be multiples of 8");
  if (B <= 0) return NSA_OK;
  int mx = Dk > Dv ? Dk : Dv;
  dim3 grid(blocks_for((int64_t)H * (mx / 8), 64), B, 2);
  paged_pool_decode_kernel<<<grid, 64, 0, (hipStream_t)stream>>>((bf16_t*)k_cache, k_sr, k_sh, Dk, (bf16_t*)v_cache,
                                                                 v_sr, v_sh, Dv, context_lens, block_tables,
                                                                 table_stride, cmp_slot_mapping, page_size, H,
                                                                 kernel_size, stride);
  return nsa_check_launch("paged_pool_decode");
}

int nsa_store_kvcache(const void* key, int64_t k_st, const void* value, int64_t v_st, void* k_cache, int64_t kc_sr,
                      void* v_cache, int64_t vc_sr, const int32_t* slot_mapping, int N, int k_row_elems,
                      int v_row_elems, void* stream) {
  NSA_REQUIRE(k_row_elems > 0 && v_row_elems > 0 && k_row_elems % 8 == 0 && v_row_elems % 8 == 0, NSA_ERR_BAD_ARG,
              "store_kvcache: row widths %d / %d must be positive multiples of 8", k_row_elems, v_row_elems);
  NSA_REQUIRE(k_st >= k_row_elems && v_st >= v_row_elems && kc_sr >= k_row_elems && vc_sr >= v_row_elems,
              NSA_ERR_BAD_ARG, "store_kvcache: a row stride is smaller than the row");
  if (N <= 0) return NSA_OK;
  const int mx = k_row_elems > v_row_elems ? k_row_elems : v_row_elems;
  dim3 grid(blocks_for((int64_t)N * (mx / 8), 256), 2);
  store_kvcache_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const bf16_t*)key, k_st, (const bf16_t*)value, v_st,
                                                              (bf16_t*)k_cache, kc_sr, (bf16_t*)v_cache, vc_sr,
                                                              slot_mapping, N, k_row_elems, v_row_elems);
  return nsa_check_launch("store_kvcache");
}

int nsa_paged_store_pool_prefill(const void* key, int64_t k_st, int64_t k_sh, int Dk, const void* value, int64_t v_st,
                                 int64_t v_sh, int Dv, void* k_cache, int64_t kc_sr, int64_t kc_sh, void* v_cache,
                                 int64_t vc_sr, int64_t vc_sh, const int32_t* x_cu, const int32_t* context_lens,
                                 const int32_t* slot_mapping, const int32_t* y_cu, const int32_t* cmp_slot_mapping,
                                 const int32_t* block_tables, int table_stride, int B, int x_maxlen, int y_maxlen,
                                 int page_size, int H, int kernel_size, int stride, void* stream) {
  NSA_REQUIRE(Dk % 8 == 0 && Dv % 8 == 0 && Dk > 0 && Dv > 0, NSA_ERR_BAD_ARG,
              "paged_store_pool_prefill: head dims %d / %d must be positive multiples of 8", Dk, Dv);
  NSA_REQUIRE(page_size > 0 && H > 0 && kernel_size > 0 && stride > 0, NSA_ERR_BAD_ARG,
              "paged_store_pool_prefill: page_size, H, kernel_size and stride must be positive");
  if (B <= 0 || (x_maxlen <= 0 && y_maxlen <= 0)) return NSA_OK;
  const int rows = x_maxlen > y_maxlen ? x_maxlen : y_maxlen;
  const int mx = Dk > Dv ? Dk : Dv;
  dim3 grid(blocks_for((int64_t)rows * H * (mx / 8), 256), B, 2);
  paged_store_pool_prefill_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(
      (const bf16_t*)key, k_st, k_sh, Dk, (const bf16_t*)value, v_st, v_sh, Dv, (bf16_t*)k_cache, kc_sr, kc_sh,
      (bf16_t*)v_cache, vc_sr, vc_sh, x_cu, context_lens, slot_mapping, y_cu, cmp_slot_mapping, block_tables,
      table_stride, page_size, H, kernel_size, stride);
  return nsa_check_launch("paged_store_pool_prefill");
}

int nsa_rope(const void* q, int64_t q_sb, int64_t q_sn, int64_t q_sh, const void* k, int64_t k_sb, int64_t k_sn,
             int64_t k_sh, void* qe, int64_t qe_sb, int64_t qe_sn, int64_t qe_sh, void* ke, int64_t ke_sb,
             int64_t ke_sn, int64_t ke_sh, const void* cos, const void* sin, int64_t c_sb, int64_t c_sn,
             int cos_is_fp32, int B, int N, int QH, int KH, int D, int backward, void* stream) {
  NSA_REQUIRE(D > 0 && D % 16 == 0 && D <= 4096, NSA_ERR_BAD_ARG,
              "rope: head dim %d must be a positive multiple of 16, at most 4096", D);
  NSA_REQUIRE(QH >= 0 && KH >= 0 && QH + KH > 0, NSA_ERR_BAD_ARG, "rope: bad head counts %d / %d", QH, KH);
  if (B <= 0 || N <= 0) return NSA_OK;
  NSA_REQUIRE(B <= 65535, NSA_ERR_BAD_ARG, "rope: batch %d exceeds the grid limit 65535", B);
  // every row is moved in 16-byte pieces
  const int64_t strides[] = {q_sb, q_sn, q_sh, k_sb, k_sn, k_sh, qe_sb, qe_sn, qe_sh, ke_sb, ke_sn, ke_sh};
  for (int64_t st : strides)
    NSA_REQUIRE(st % 8 == 0, NSA_ERR_BAD_ARG, "rope: stride %lld is not a multiple of 8 elements", (long long)st);
  const int tab_align = cos_is_fp32 ? 4 : 8;
  NSA_REQUIRE(c_sb % tab_align == 0 && c_sn % tab_align == 0, NSA_ERR_BAD_ARG,
              "rope: table strides %lld / %lld must be multiples of %d elements", (long long)c_sb, (long long)c_sn,
              tab_align);
  const void* ptrs[] = {q, k, qe, ke, cos, sin};
  for (const void* ptr : ptrs)
    NSA_REQUIRE(((uintptr_t)ptr & 15) == 0, NSA_ERR_BAD_ARG, "rope: pointer %p is not 16-byte aligned", ptr);
  dim3 grid((unsigned)N, (unsigned)B);
  if (cos_is_fp32)
    rope_kernel<float><<<grid, 256, 0, (hipStream_t)stream>>>(
        (const bf16_t*)q, q_sb, q_sn, q_sh, (const bf16_t*)k, k_sb, k_sn, k_sh, (bf16_t*)qe, qe_sb, qe_sn, qe_sh,
        (bf16_t*)ke, ke_sb, ke_sn, ke_sh, (const float*)cos, (const float*)sin, c_sb, c_sn, QH, KH, D, backward);
  else
    rope_kernel<bf16_t><<<grid, 256, 0, (hipStream_t)stream>>>(
        (const bf16_t*)q, q_sb, q_sn, q_sh, (const bf16_t*)k, k_sb, k_sn, k_sh, (bf16_t*)qe, qe_sb, qe_sn, qe_sh,
        (bf16_t*)ke, ke_sb, ke_sn, ke_sh, (const bf16_t*)cos, (const bf16_t*)sin, c_sb, c_sn, QH, KH, D, backward);
  return nsa_check_launch("rope");
}

}  // extern "C"

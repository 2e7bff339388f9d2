"""CPU oracle for the Native-Sparse-Attention hot path.  TEST INFRASTRUCTURE ONLY.

This module is a naive, dense PyTorch restatement of the algorithm that the HIP
kernels in this repository implement.  It exists to *check* the GPU path (tests,
the smoke entry and the CPU-baseline leg of the benchmark); nothing in the shipped
package imports it and it must never be used as a fallback.

Every function cites the reference file:line whose behaviour it restates
(paths relative to the upstream repository root):

* lengths               flash_nsa/utils.py:228-244
* construct_block       flash_nsa/ops/torch_ref.py:7-30, flash_nsa/ops/compress_kv.py:17-60
* mean_pooling          flash_nsa/ops/compress_kv.py:226-264
* compress (learned)    flash_nsa/modules/hf_level_nsa.py:33-60, flash_nsa/ops/act.py:129-144
* cmp_attn              flash_nsa/ops/torch_ref.py:41-62, flash_nsa/ops/compress_attn.py:94-153
* importance / select   flash_nsa/ops/torch_ref.py:64-105, flash_nsa/ops/topk.py:119-218, 353-425
* slc_attn              flash_nsa/ops/torch_ref.py:108-134, flash_nsa/ops/select_attn.py:87-108
* swa                   flash_nsa/ops/sliding_window_attention.py:26-37 (FlashAttention window=(W,-1), causal),
                        mask restated at flash_nsa/inference/select_attn.py:353-354
* combine               flash_nsa/ops/torch_ref.py:185-188, flash_nsa/ops/combine.py:42-46
* nsa_forward           flash_nsa/modules/hf_level_nsa.py:128-140
* paged prefill/decode  flash_nsa/inference/__init__.py:21-257, flash_nsa/inference/compress_kv.py:13-61,123-188

Pinning status (see tests/test_oracle_*.py):
  mean_pooling / construct_block  closed forms (unfold, avg_pool1d), hand cases
  cmp_attn / slc_attn / swa       torch scaled_dot_product_attention with explicit masks, brute force
  select_blocks                   golden vectors of the upstream torch_topk (tests/golden) + brute force
  combine / activations           closed forms
  gradients                       torch.autograd of this dense restatement + fp64 gradcheck
  nsa_forward_backward,           with no rounding: equal to torch.autograd through nsa_forward / cmp_attn /
  branch_forward_backward         slc_attn / swa (fp64)
  paged_pool_decode               last row of mean_pooling on the gathered sequence
  topk_mismatch_report            hand-built cases (identical, tie-excused, wrong, out-of-range)
  swa                             parity unpinned against upstream: the upstream delegates to the external
                                  FlashAttention wheel and holds no vectors for it; pinned by the textbook
                                  band-mask definition only.

All functions are dtype-preserving (run them in fp32 or fp64) and differentiable.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch
import torch.nn.functional as F

LOG2E = 1.4426950408889634


@dataclass
class OracleConfig:
    kernel_size: int = 32
    stride: int = 16
    block_size: int = 64
    top_n: int = 16
    num_init_blocks: int = 1
    num_local_blocks: int = 2
    window_size: int = 512
    cmp_k_method: str = "mean"
    cmp_v_method: str = "mean"


def cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


# ----------------------------------------------------------------------------------------------
# lengths  (flash_nsa/utils.py:228-244)
# ----------------------------------------------------------------------------------------------
def seq_lengths(cu_seqlens, kernel_size=32, stride=16, block_size=64):
    """Per-sequence token / compressed-row / selection-block counts and their cumulative sums."""
    cu = [int(c) for c in (cu_seqlens.tolist() if hasattr(cu_seqlens, "tolist") else cu_seqlens)]
    x = [cu[i + 1] - cu[i] for i in range(len(cu) - 1)]
    y = [max((l - kernel_size) // stride + 1, 0) for l in x]
    k = [cdiv(l, block_size) for l in x]

    def cs(v):
        out = [0]
        for e in v:
            out.append(out[-1] + e)
        return out

    return dict(x_seqlens=x, y_seqlens=y, k_seqlens=k, x_cu=cu, y_cu=cs(y), k_cu=cs(k))


# ----------------------------------------------------------------------------------------------
# compression
# ----------------------------------------------------------------------------------------------
def construct_block(x, cu_seqlens, kernel_size=32, stride=16):
    """im2col: [T,H,D] -> [y_len,H,kernel,D]; window i of a sequence = tokens [stride*i, stride*i+kernel)."""
    meta = seq_lengths(cu_seqlens, kernel_size, stride)
    outs = []
    for b, L in enumerate(meta["x_seqlens"]):
        y = meta["y_seqlens"][b]
        xs = x[meta["x_cu"][b]: meta["x_cu"][b + 1]]
        if y == 0:
            outs.append(x.new_zeros(0, x.shape[1], kernel_size, x.shape[2]))
            continue
        idx = (torch.arange(y)[:, None] * stride + torch.arange(kernel_size)[None, :])  # [y, K]
        blk = xs[idx]  # [y, K, H, D]
        outs.append(blk.permute(0, 2, 1, 3))
    return torch.cat(outs, 0)


def mean_pooling(x, cu_seqlens, kernel_size=32, stride=16):
    """[T,H,D] -> [y_len,H,D], mean over each window."""
    return construct_block(x, cu_seqlens, kernel_size, stride).mean(-2)


def sigmoid_mul(h):
    gate, up = h.chunk(2, -1)
    return torch.sigmoid(gate) * up


def swiglu(h):
    gate, up = h.chunk(2, -1)
    return F.silu(gate) * up


def compress(x, cu_seqlens, method="mean", weight=None, kernel_size=32, stride=16):
    """KV compression.  weight: [out, kernel*D] (no bias); flatten order = (position-in-window, channel)."""
    if method == "mean":
        return mean_pooling(x, cu_seqlens, kernel_size, stride)
    blk = construct_block(x, cu_seqlens, kernel_size, stride)  # [y,H,K,D]
    hid = blk.flatten(-2, -1) @ weight.t()
    if method == "linear":
        return hid
    if method == "sigmoid-mul":
        return sigmoid_mul(hid)
    if method == "swiglu":
        return swiglu(hid)
    raise ValueError(method)


# ----------------------------------------------------------------------------------------------
# compressed attention
# ----------------------------------------------------------------------------------------------
def _cmp_probs_one_seq(q, ck, kernel_size, stride, scale, q_offset=0):
    """q [L,QH,D], ck [y,KH,D] -> (P [QH,L,y] with invisible entries = 0, lse2 [QH,L])."""
    L, QH, D = q.shape
    y, KH, _ = ck.shape
    G = QH // KH
    if y == 0:
        return q.new_zeros(QH, L, 0), q.new_zeros(QH, L)
    kk = ck.repeat_interleave(G, 1)
    s = torch.einsum("nhd,mhd->hnm", q, kk) * scale
    t = torch.arange(L) + q_offset
    vis = t[:, None] >= (torch.arange(y) * stride + kernel_size - 1)[None, :]
    s = s.masked_fill(~vis[None], float("-inf"))
    has = vis.any(-1)  # rows with at least one visible compressed key
    lse = torch.logsumexp(s, -1)
    lse = torch.where(has[None], lse, torch.zeros_like(lse))
    p = torch.exp(s - lse[..., None])
    p = torch.where(has[None, :, None], p, torch.zeros_like(p))
    return p, lse * LOG2E


def cmp_attn(q, ck, cv, cu_seqlens, kernel_size=32, stride=16, scale=None):
    """Compressed attention.  Returns o [T,QH,VD] and lse in log2 units, layout [QH,T]; rows with no
    visible compressed key give o = 0, lse = 0."""
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    meta = seq_lengths(cu_seqlens, kernel_size, stride)
    G = q.shape[1] // ck.shape[1]
    os_, ls_ = [], []
    for b in range(len(meta["x_seqlens"])):
        qs = q[meta["x_cu"][b]: meta["x_cu"][b + 1]]
        cks = ck[meta["y_cu"][b]: meta["y_cu"][b + 1]]
        cvs = cv[meta["y_cu"][b]: meta["y_cu"][b + 1]]
        p, lse2 = _cmp_probs_one_seq(qs, cks, kernel_size, stride, scale)
        o = torch.einsum("hnm,mhd->nhd", p, cvs.repeat_interleave(G, 1))
        os_.append(o)
        ls_.append(lse2)
    return torch.cat(os_, 0), torch.cat(ls_, 1)


# ----------------------------------------------------------------------------------------------
# block importance + selection
# ----------------------------------------------------------------------------------------------
def overlap_weights(kernel_size=32, stride=16, block_size=64):
    """Weights w_r and the first compressed index offset for selection block j:
    compressed index i = (j*block - kernel)//stride + 1 + r, r = 0..len(w)-1  (topk.py:179-194)."""
    n = (block_size + kernel_size - stride) // stride
    w = []
    cs = stride - kernel_size
    for _ in range(n):
        ce = cs + kernel_size
        w.append((min(ce, block_size) - max(cs, 0)) / stride)
        cs += stride
    return w


def importance_one_seq(p, KH, kernel_size, stride, block_size, L):
    """p [QH,L,y] compressed-attention probabilities -> imp [KH,L,nb] (sum over the G heads of a group,
    then overlap-weighted map onto selection blocks)."""
    QH, Lq, y = p.shape
    G = QH // KH
    nb = cdiv(L, block_size)
    pg = p.reshape(KH, G, Lq, y).sum(1)
    w = overlap_weights(kernel_size, stride, block_size)
    imp = p.new_zeros(KH, Lq, nb)
    j = torch.arange(nb)
    i0 = (j * block_size - kernel_size) // stride + 1
    for r, wr in enumerate(w):
        i = i0 + r
        ok = (i >= 0) & (i < y)
        if y > 0 and ok.any():
            imp[:, :, ok] += wr * pg[:, :, i[ok]]
    return imp


def select_blocks(imp, t_abs, block_size, top_n, num_init, num_local, ignore_index):
    """imp [KH,Lq,nb], t_abs [Lq] absolute positions.  Slot order (topk.py:203-218 / 408-425):
    slots [0,I): block s (if s <= nk); slots I+i: block nk-i (if I+i <= nk); remaining slots up to
    min(top_n, nk+1): repeated argmax (lowest index on ties) over the scores with forced blocks removed."""
    KH, Lq, nb = imp.shape
    out = torch.full((KH, Lq, top_n), ignore_index, dtype=torch.int32)
    if Lq == 0:
        return out
    nk = (t_abs // block_size).to(torch.int64)  # [Lq]
    work = imp.detach().clone()
    cols = torch.arange(nb)
    for s in range(num_init):
        if s < top_n:
            ok = s <= nk
            out[:, ok, s] = s
        work[:, :, cols == s] = -1.0
    for i in range(num_local):
        slot = num_init + i
        ok = slot <= nk
        if slot < top_n:
            out[:, ok, slot] = (nk - i)[ok].to(torch.int32)
        tgt = nk - i
        m = (cols[None, :] == tgt[:, None])  # [Lq, nb]
        work = torch.where(m[None], torch.full_like(work, -1.0), work)
    order = torch.sort(work, dim=-1, descending=True, stable=True)[1]  # ties -> lowest index first
    nfree = top_n - num_init - num_local
    for r in range(max(nfree, 0)):
        slot = num_init + num_local + r
        if r >= nb:
            break
        ok = slot <= nk
        out[:, ok, slot] = order[:, ok, r].to(torch.int32)
    return out


def slc_topk(q, ck, lse2, cu_seqlens, cfg: OracleConfig = OracleConfig(), scale=None, ignore_index=None,
             return_importance=False):
    """Top-n selection-block indices per kv head, [KH,T,top_n] int32.  lse2 is accepted for interface parity
    but the probabilities are recomputed exactly (they equal exp2(s*log2e - lse2))."""
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    meta = seq_lengths(cu_seqlens, cfg.kernel_size, cfg.stride, cfg.block_size)
    KH = ck.shape[1]
    if ignore_index is None:
        ignore_index = cdiv(max(meta["x_seqlens"]), cfg.block_size)
    outs, imps = [], []
    for b, L in enumerate(meta["x_seqlens"]):
        qs = q[meta["x_cu"][b]: meta["x_cu"][b + 1]]
        cks = ck[meta["y_cu"][b]: meta["y_cu"][b + 1]]
        p, _ = _cmp_probs_one_seq(qs, cks, cfg.kernel_size, cfg.stride, scale)
        imp = importance_one_seq(p, KH, cfg.kernel_size, cfg.stride, cfg.block_size, L)
        outs.append(select_blocks(imp, torch.arange(L), cfg.block_size, cfg.top_n, cfg.num_init_blocks,
                                  cfg.num_local_blocks, ignore_index))
        imps.append(imp)
    topk = torch.cat(outs, 1)
    if return_importance:
        return topk, imps
    return topk


# ----------------------------------------------------------------------------------------------
# selected attention
# ----------------------------------------------------------------------------------------------
def _slc_mask_one_seq(topk, t_abs, Lk, block_size):
    """topk [KH,Lq,N] (block ids local to the sequence), -> bool mask [KH,Lq,Lk] of attended keys."""
    KH, Lq, N = topk.shape
    nb = cdiv(Lk, block_size)
    nk = (t_abs // block_size).to(torch.int64)
    nvalid = torch.clamp(nk + 1, max=N)  # first min(N, nk+1) slots are consumed (select_attn.py:69-71)
    slot_ok = torch.arange(N)[None, :] < nvalid[:, None]  # [Lq,N]
    idx = topk.to(torch.int64).clamp(min=0, max=nb)  # ignore values land in the spill column nb
    idx = torch.where(slot_ok[None], idx, torch.full_like(idx, nb))
    bm = torch.zeros(KH, Lq, nb + 1, dtype=torch.bool)
    bm.scatter_(-1, idx, True)
    bm = bm[..., :nb]
    km = bm.repeat_interleave(block_size, -1)[..., :Lk]
    causal = t_abs[:, None] >= torch.arange(Lk)[None, :]
    return km & causal[None]


def _masked_attn(q, k, v, mask, scale):
    """q [Lq,QH,D], k [Lk,KH,D], v [Lk,KH,VD], mask [KH,Lq,Lk] bool -> o [Lq,QH,VD], lse2 [Lq,QH]."""
    Lq, QH, D = q.shape
    KH = k.shape[1]
    G = QH // KH
    s = torch.einsum("nhd,mhd->hnm", q, k.repeat_interleave(G, 1)) * scale
    m = mask.repeat_interleave(G, 0)
    s = s.masked_fill(~m, float("-inf"))
    has = m.any(-1)
    lse = torch.logsumexp(s, -1)
    lse = torch.where(has, lse, torch.zeros_like(lse))
    p = torch.exp(s - lse[..., None])
    p = torch.where(has[..., None], p, torch.zeros_like(p))
    o = torch.einsum("hnm,mhd->nhd", p, v.repeat_interleave(G, 1))
    return o, (lse * LOG2E).transpose(0, 1)


def slc_attn(q, k, v, topk, cu_seqlens, block_size=64, scale=None):
    """Selected-block attention.  Returns o [T,QH,VD], lse2 [T,QH]."""
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    cu = [int(c) for c in (cu_seqlens.tolist() if hasattr(cu_seqlens, "tolist") else cu_seqlens)]
    os_, ls_ = [], []
    for b in range(len(cu) - 1):
        a, e = cu[b], cu[b + 1]
        L = e - a
        mask = _slc_mask_one_seq(topk[:, a:e], torch.arange(L), L, block_size)
        o, l2 = _masked_attn(q[a:e], k[a:e], v[a:e], mask, scale)
        os_.append(o)
        ls_.append(l2)
    return torch.cat(os_, 0), torch.cat(ls_, 0)


# ----------------------------------------------------------------------------------------------
# sliding window attention
# ----------------------------------------------------------------------------------------------
def swa(q, k, v, cu_seqlens, window_size=512, scale=None):
    """Causal sliding window: query t attends keys max(0,t-W) <= j <= t.  Returns o, lse2 [T,QH]."""
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    cu = [int(c) for c in (cu_seqlens.tolist() if hasattr(cu_seqlens, "tolist") else cu_seqlens)]
    KH = k.shape[1]
    os_, ls_ = [], []
    for b in range(len(cu) - 1):
        a, e = cu[b], cu[b + 1]
        L = e - a
        t = torch.arange(L)
        d = t[:, None] - t[None, :]
        mask = ((d >= 0) & (d <= window_size))[None].expand(KH, L, L)
        o, l2 = _masked_attn(q[a:e], k[a:e], v[a:e], mask, scale)
        os_.append(o)
        ls_.append(l2)
    return torch.cat(os_, 0), torch.cat(ls_, 0)


# ----------------------------------------------------------------------------------------------
# combine and composition
# ----------------------------------------------------------------------------------------------
def combine(a, b, c, w):
    g = torch.sigmoid(w)
    return a * g[..., 0:1] + b * g[..., 1:2] + c * g[..., 2:3]


def nsa_forward(q, k, v, w, cu_seqlens, cfg: OracleConfig = OracleConfig(), wk=None, wv=None, scale=None,
                topk=None, return_parts=False, round_dtype: Optional[torch.dtype] = None):
    """Composed NSA forward (hf_level_nsa.py:128-140).  If `topk` is given it is used instead of the oracle's
    own selection (lets a test feed the device's indices so that near-ties cannot change the output).
    round_dtype: round the three branch outputs (and compressed K/V) to this dtype before they are consumed,
    as the device path stores them (combine.py reads bf16 branches)."""
    scale = q.shape[-1] ** -0.5 if scale is None else scale

    def rnd(x):
        return x.to(round_dtype).to(x.dtype) if round_dtype is not None else x

    ck = rnd(compress(k, cu_seqlens, cfg.cmp_k_method, wk, cfg.kernel_size, cfg.stride))
    cv = rnd(compress(v, cu_seqlens, cfg.cmp_v_method, wv, cfg.kernel_size, cfg.stride))
    cmp_o, cmp_lse = cmp_attn(q, ck, cv, cu_seqlens, cfg.kernel_size, cfg.stride, scale)
    if topk is None:
        topk = slc_topk(q, ck, cmp_lse, cu_seqlens, cfg, scale)
    slc_o, slc_lse = slc_attn(q, k, v, topk, cu_seqlens, cfg.block_size, scale)
    swa_o, swa_lse = swa(q, k, v, cu_seqlens, cfg.window_size, scale)
    o = combine(rnd(cmp_o), rnd(slc_o), rnd(swa_o), w)
    if return_parts:
        return o, dict(cmp_k=ck, cmp_v=cv, cmp_o=cmp_o, cmp_lse=cmp_lse, topk=topk, slc_o=slc_o, slc_lse=slc_lse,
                       swa_o=swa_o, swa_lse=swa_lse)
    return o


# ----------------------------------------------------------------------------------------------
# forward + backward with the rounding points of a half-precision pipeline
# ----------------------------------------------------------------------------------------------
class _RoundBothWays(torch.autograd.Function):
    """y = round(x) on the way forward, dx = round(dy) on the way back (a tensor that a pipeline stores in
    half precision in both directions)."""

    @staticmethod
    def forward(ctx, x, dtype):
        ctx.dtype = dtype
        return x.to(dtype).to(x.dtype)

    @staticmethod
    def backward(ctx, g):
        return g.to(ctx.dtype).to(g.dtype), None


def _branch_backward(p, q, k, v, d_o, delta, scale, r_mma=lambda x: x):
    """Softmax-attention backward of one branch of one sequence from its probabilities.
    p [QH,L,M], q [L,QH,D], k [M,KH,D], v [M,KH,VD], d_o [L,QH,VD], delta [L,QH]
    -> dq [L,QH,D], dk [M,KH,D], dv [M,KH,VD]   (dS = P * (dP - delta), the form every flash backward uses:
    flash_nsa/ops/compress_attn.py:187-332, flash_nsa/ops/select_attn.py:142-330 upstream).
    r_mma rounds the two computed matrix operands, P (for dV) and dS (for dQ and dK), the way a half-precision
    matrix unit receives them (upstream casts them with .to(dtype) before tl.dot at the same places)."""
    QH, KH = q.shape[1], k.shape[1]
    G = QH // KH
    M = k.shape[0]
    ke, ve = k.repeat_interleave(G, 1), v.repeat_interleave(G, 1)
    dp = torch.einsum("nhd,mhd->hnm", d_o, ve)
    ds = r_mma(p * (dp - delta.transpose(0, 1)[..., None]))
    dq = scale * torch.einsum("hnm,mhd->nhd", ds, ke)
    dk = scale * torch.einsum("hnm,nhd->mhd", ds, q).reshape(M, KH, G, q.shape[-1]).sum(2)
    dv = torch.einsum("hnm,nhd->mhd", r_mma(p), d_o).reshape(M, KH, G, d_o.shape[-1]).sum(2)
    return dq, dk, dv


def _masked_probs(q, k, mask, scale):
    """q [Lq,QH,D], k [Lk,KH,D], mask [KH,Lq,Lk] -> softmax probabilities [QH,Lq,Lk] (rows without a key: 0)."""
    G = q.shape[1] // k.shape[1]
    s = torch.einsum("nhd,mhd->hnm", q, k.repeat_interleave(G, 1)) * scale
    m = mask.repeat_interleave(G, 0)
    s = s.masked_fill(~m, float("-inf"))
    has = m.any(-1)
    p = torch.softmax(torch.where(has[..., None], s, torch.zeros_like(s)), -1)
    return torch.where(has[..., None], p, torch.zeros_like(p))


def _branch_probs(kind, qs, ks, cfg, scale, topk_seq=None):
    """Probabilities [QH,L,M] of one branch for one sequence; ks = compressed keys for "cmp", raw keys otherwise."""
    L, KH = qs.shape[0], ks.shape[1]
    t = torch.arange(L)
    if kind == "cmp":
        return _cmp_probs_one_seq(qs, ks, cfg.kernel_size, cfg.stride, scale)[0]
    if kind == "slc":
        return _masked_probs(qs, ks, _slc_mask_one_seq(topk_seq, t, L, cfg.block_size), scale)
    d = t[:, None] - t[None, :]
    return _masked_probs(qs, ks, ((d >= 0) & (d <= cfg.window_size))[None].expand(KH, L, L), scale)


def branch_forward_backward(kind, q, k, v, d_o, cu_seqlens, cfg: OracleConfig = OracleConfig(), topk=None,
                            scale=None, round_dtype: Optional[torch.dtype] = None, round_mma=False):
    """One attention branch ("cmp": k, v are the compressed rows; "slc"; "swa") forward and backward the way a
    flash backward computes it: o stored rounded, delta = rowsum(round(o) * d_o), dS = P (dP - delta), optionally
    with P and dS rounded before the matrix products.  Without rounding it equals torch.autograd through
    cmp_attn / slc_attn / swa.  -> dict(o, dq, dk, dv), gradients unrounded."""
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    r = (lambda x: x) if round_dtype is None else (lambda x: x.to(round_dtype).to(x.dtype))
    meta = seq_lengths(cu_seqlens, cfg.kernel_size, cfg.stride, cfg.block_size)
    G = q.shape[1] // k.shape[1]
    o = torch.zeros(q.shape[0], q.shape[1], v.shape[-1], dtype=q.dtype)
    dq, dk, dv = torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)
    for b, L in enumerate(meta["x_seqlens"]):
        if L == 0:
            continue
        a, e = meta["x_cu"][b], meta["x_cu"][b + 1]
        ka, ke = (meta["y_cu"][b], meta["y_cu"][b + 1]) if kind == "cmp" else (a, e)
        p = _branch_probs(kind, q[a:e], k[ka:ke], cfg, scale, None if topk is None else topk[:, a:e])
        o[a:e] = r(torch.einsum("hnm,mhd->nhd", p, v[ka:ke].repeat_interleave(G, 1)))
        delta = (d_o[a:e] * o[a:e]).sum(-1)
        dq[a:e], dk_i, dv_i = _branch_backward(p, q[a:e], k[ka:ke], v[ka:ke], d_o[a:e], delta, scale,
                                               r if round_mma else (lambda x: x))
        dk[ka:ke] += dk_i
        dv[ka:ke] += dv_i
    return dict(o=o, dq=dq, dk=dk, dv=dv)


def nsa_forward_backward(q, k, v, w, d_out, cu_seqlens, cfg: OracleConfig = OracleConfig(), topk=None, wk=None,
                         wv=None, scale=None, round_dtype: Optional[torch.dtype] = None, round_mma=False):
    """Composed NSA forward and a hand-written backward that keeps the rounding points of the fused training node
    (flash_nsa/modules/megatron_level_nsa.py:87-159 upstream stores exactly these tensors in q's dtype between
    kernels): compressed K/V, the three branch outputs, the three branch output gradients d o_k = round(dy sig_k),
    the correction term delta_k = rowsum(round(o_k) * round(d o_k)), the compressed-row gradients handed to the
    compression backward, the learned compression's pre-activation and its gradient, and the final dq / dk / dv /
    dw / dW.  Everything else is computed in the dtype of the inputs (fp32 or fp64); with round_mma the
    probabilities and dS of the backward are rounded as well before they enter a matrix product.
    With round_dtype=None nothing is rounded and the result must equal torch.autograd through nsa_forward: that
    identity pins the backward formulas.
    -> dict(o, dq, dk, dv, dw, dwk, dwv)"""
    assert topk is not None, "pass the selection so that both sides attend the same blocks"
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    r = (lambda x: x) if round_dtype is None else (lambda x: x.to(round_dtype).to(x.dtype))
    rb = (lambda x: x) if round_dtype is None else (lambda x: _RoundBothWays.apply(x, round_dtype))
    meta = seq_lengths(cu_seqlens, cfg.kernel_size, cfg.stride, cfg.block_size)
    KH = k.shape[1]

    # compression through autograd, with the tensors the pipeline stores rounded both ways
    def compress_graph(x, weight, method):
        xl = x.detach().clone().requires_grad_()
        if method == "mean":
            return xl, None, rb(mean_pooling(xl, cu_seqlens, cfg.kernel_size, cfg.stride))
        wl = weight.detach().clone().requires_grad_()
        win = rb(construct_block(xl, cu_seqlens, cfg.kernel_size, cfg.stride).flatten(-2, -1))
        hid = rb(win @ wl.t())
        out = hid if method == "linear" else rb(sigmoid_mul(hid) if method == "sigmoid-mul" else swiglu(hid))
        return xl, wl, out

    k_leaf, wk_leaf, ck_g = compress_graph(k, wk, cfg.cmp_k_method)
    v_leaf, wv_leaf, cv_g = compress_graph(v, wv, cfg.cmp_v_method)
    ck, cv = ck_g.detach(), cv_g.detach()

    g = torch.sigmoid(w)
    o = torch.zeros(q.shape[0], q.shape[1], v.shape[-1], dtype=q.dtype)
    dq = torch.zeros_like(q)
    dk = torch.zeros_like(k)
    dv = torch.zeros_like(v)
    dw = torch.zeros_like(w)
    dck = torch.zeros_like(ck)
    dcv = torch.zeros_like(cv)
    for b, L in enumerate(meta["x_seqlens"]):
        if L == 0:
            continue
        a, e = meta["x_cu"][b], meta["x_cu"][b + 1]
        ya, ye = meta["y_cu"][b], meta["y_cu"][b + 1]
        qs, ks, vs, gs, dys = q[a:e], k[a:e], v[a:e], g[a:e], d_out[a:e]
        G = qs.shape[1] // KH
        branches = (
            (_branch_probs("cmp", qs, ck[ya:ye], cfg, scale), ck[ya:ye], cv[ya:ye]),
            (_branch_probs("slc", qs, ks, cfg, scale, topk[:, a:e]), ks, vs),
            (_branch_probs("swa", qs, ks, cfg, scale), ks, vs),
        )
        for i, (p, kk, vv) in enumerate(branches):
            o_i = r(torch.einsum("hnm,mhd->nhd", p, vv.repeat_interleave(G, 1)))
            o[a:e] += o_i * gs[..., i:i + 1]
            dw[a:e, :, i] = gs[..., i] * (1 - gs[..., i]) * (dys * o_i).sum(-1)
            d_oi = r(dys * gs[..., i:i + 1])
            delta = (d_oi * o_i).sum(-1)
            dq_i, dk_i, dv_i = _branch_backward(p, qs, kk, vv, d_oi, delta, scale, r if round_mma else (lambda x: x))
            dq[a:e] += dq_i
            if i == 0:
                dck[ya:ye] += dk_i
                dcv[ya:ye] += dv_i
            else:
                dk[a:e] += dk_i
                dv[a:e] += dv_i
    grads_k = torch.autograd.grad(ck_g, [k_leaf] + ([wk_leaf] if wk_leaf is not None else []), dck,
                                  allow_unused=True) if ck.numel() else (torch.zeros_like(k), None)
    grads_v = torch.autograd.grad(cv_g, [v_leaf] + ([wv_leaf] if wv_leaf is not None else []), dcv,
                                  allow_unused=True) if cv.numel() else (torch.zeros_like(v), None)
    dk = dk + (grads_k[0] if grads_k[0] is not None else 0)
    dv = dv + (grads_v[0] if grads_v[0] is not None else 0)

    def wgrad(leaf, grads):
        if leaf is None:
            return None
        gw = grads[1] if len(grads) > 1 and grads[1] is not None else torch.zeros_like(leaf)
        return r(gw)

    return dict(o=r(o), dq=r(dq), dk=r(dk), dv=r(dv), dw=r(dw), dwk=wgrad(wk_leaf, grads_k),
                dwv=wgrad(wv_leaf, grads_v))


# ----------------------------------------------------------------------------------------------
# paged KV (inference)
# ----------------------------------------------------------------------------------------------
def _acc(x):
    """accumulation dtype: fp32 for half/bf16/fp32 inputs, fp64 stays fp64"""
    return x if x.dtype == torch.float64 else x.float()


def gather_rows(cache, table_row, n):
    """cache [P,page,H,D]; rows 0..n-1 of a request live at table_row[r//page]*page + r%page."""
    P, page, H, D = cache.shape
    flat = cache.reshape(P * page, H, D)
    r = torch.arange(n)
    pages = table_row.to(torch.int64)[r // page]
    return flat[pages * page + r % page]


def rope(x, cos, sin):
    """Rotate-half rotary embedding of x [..., s, h, d] with cos / sin [..., s, d] (flash_nsa/ops/rope.py:84-97
    upstream): out[:H] = x[:H]*cos[:H] - x[H:]*sin[:H], out[H:] = x[H:]*cos[H:] + x[:H]*sin[H:], H = d/2."""
    H = x.size(-1) // 2
    c, s_ = cos.unsqueeze(-2), sin.unsqueeze(-2)
    x1, x2 = x[..., :H], x[..., H:]
    return torch.cat([x1 * c[..., :H] - x2 * s_[..., :H], x2 * c[..., H:] + x1 * s_[..., H:]], -1)


def store_kvcache(key, value, k_cache, v_cache, slot_mapping):
    """Cache writer (nano-vllm/nanovllm/layers/attention.py:123-153 upstream): row n of key / value is copied to
    flat pool row slot_mapping[n]; negative slots are skipped.  In place on the [pages, page, KH, *] pools."""
    kf = k_cache.view(-1, *k_cache.shape[2:])
    vf = v_cache.view(-1, *v_cache.shape[2:])
    for n, slot in enumerate(slot_mapping.tolist()):
        if slot >= 0:
            kf[slot] = key[n].to(kf.dtype)
            vf[slot] = value[n].to(vf.dtype)


def paged_pool_prefill(cache, y_cu_seqlens, context_lens, block_tables, cmp_slot_mapping, kernel_size=32,
                       stride=16):
    """In-place: for every compressed row with slot != -1, write mean of its window (read through the raw block
    table) to flat pool row `slot`  (inference/compress_kv.py:13-61)."""
    P, page, H, D = cache.shape
    flat = cache.view(P * page, H, D)
    ycu = [int(c) for c in y_cu_seqlens.tolist()]
    for b in range(len(ycu) - 1):
        L = int(context_lens[b])
        xs = _acc(gather_rows(cache, block_tables[b], L))
        for i in range(ycu[b + 1] - ycu[b]):
            slot = int(cmp_slot_mapping[ycu[b] + i])
            if slot < 0:
                continue
            flat[slot] = xs[i * stride: i * stride + kernel_size].mean(0).to(cache.dtype)


def paged_pool_decode(cache, context_lens, block_tables, cmp_slot_mapping, kernel_size=32, stride=16):
    """In-place: per request with slot != -1 and len >= kernel, pool the last complete window
    [stride*((len-kernel)//stride), +kernel)  (inference/compress_kv.py:123-188)."""
    P, page, H, D = cache.shape
    flat = cache.view(P * page, H, D)
    for b in range(len(context_lens)):
        slot = int(cmp_slot_mapping[b])
        L = int(context_lens[b])
        if slot < 0 or L < kernel_size:
            continue
        st = ((L - kernel_size) // stride) * stride
        xs = _acc(gather_rows(cache, block_tables[b], L))
        flat[slot] = xs[st: st + kernel_size].mean(0).to(cache.dtype)


def nsa_paged_forward(q, k_cache, v_cache, w, x_cu_seqlens, context_lens, block_tables, cmp_block_tables,
                      cfg: OracleConfig = OracleConfig(), scale=None, ignore_index=-1, topk=None,
                      round_dtype: Optional[torch.dtype] = None, return_parts=False):
    """Paged prefill / decode forward AFTER pooling has been written into the pool.  q holds only the new
    tokens of each request; request b's query n sits at absolute position n + (context_len - x_len).
    Compressed rows are read from the pool through cmp_block_tables.  Decode = x_len 1 per request."""
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    xcu = [int(c) for c in x_cu_seqlens.tolist()]
    KH = k_cache.shape[2]
    f = lambda x: x.to(q.dtype)

    def rnd(x):
        return x.to(round_dtype).to(x.dtype) if round_dtype is not None else x

    outs, parts = [], []
    for b in range(len(xcu) - 1):
        a, e = xcu[b], xcu[b + 1]
        xl = e - a
        L = int(context_lens[b])
        c = L - xl
        qs = q[a:e]
        if xl == 0:
            continue
        y = max((L - cfg.kernel_size) // cfg.stride + 1, 0)
        ks = f(gather_rows(k_cache, block_tables[b], L))
        vs = f(gather_rows(v_cache, block_tables[b], L))
        cks = f(gather_rows(k_cache, cmp_block_tables[b], y)) if y > 0 else ks.new_zeros(0, KH, ks.shape[-1])
        cvs = f(gather_rows(v_cache, cmp_block_tables[b], y)) if y > 0 else vs.new_zeros(0, KH, vs.shape[-1])
        G = q.shape[1] // KH
        t_abs = torch.arange(xl) + c
        p, lse2 = _cmp_probs_one_seq(qs, cks, cfg.kernel_size, cfg.stride, scale, q_offset=c)
        cmp_o = torch.einsum("hnm,mhd->nhd", p, cvs.repeat_interleave(G, 1))
        imp = importance_one_seq(p, KH, cfg.kernel_size, cfg.stride, cfg.block_size, L)
        if topk is None:
            tk = select_blocks(imp, t_abs, cfg.block_size, cfg.top_n, cfg.num_init_blocks, cfg.num_local_blocks,
                               ignore_index)
        else:
            tk = topk[:, a:e]
        mask = _slc_mask_one_seq(tk, t_abs, L, cfg.block_size)
        slc_o, _ = _masked_attn(qs, ks, vs, mask, scale)
        d = t_abs[:, None] - torch.arange(L)[None, :]
        wmask = ((d >= 0) & (d <= cfg.window_size))[None].expand(KH, xl, L)
        swa_o, _ = _masked_attn(qs, ks, vs, wmask, scale)
        outs.append(combine(rnd(cmp_o), rnd(slc_o), rnd(swa_o), w[a:e]))
        parts.append(dict(cmp_o=cmp_o, lse2=lse2, topk=tk, imp=imp, slc_o=slc_o, swa_o=swa_o))
    o = torch.cat(outs, 0) if outs else q.new_zeros(0, q.shape[1], v_cache.shape[-1])
    if return_parts:
        return o, parts
    return o


# ----------------------------------------------------------------------------------------------
# comparison helper for index parity with ties
# ----------------------------------------------------------------------------------------------
def topk_mismatch_report(topk_a, topk_b, imps: List[torch.Tensor], cu_seqlens, block_size=64, top_n=16,
                         tie_tol=1e-3, t_offsets=None):
    """Compare two [KH,T,N] index tensors as per-row sets over the first min(N, nk+1) slots.  A row whose sets
    differ is excused only if every block in the symmetric difference has an importance within tie_tol
    (relative to the row maximum of 1.0-scale probabilities, i.e. absolute) of the row's selection
    threshold.  Returns (n_rows, n_differing_rows, n_unexcused_rows)."""
    cu = [int(c) for c in (cu_seqlens.tolist() if hasattr(cu_seqlens, "tolist") else cu_seqlens)]
    KH = topk_a.shape[0]
    n_rows = n_diff = n_bad = 0
    for b in range(len(cu) - 1):
        a, e = cu[b], cu[b + 1]
        off = 0 if t_offsets is None else int(t_offsets[b])
        imp = imps[b]
        for kh in range(KH):
            ta = topk_a[kh, a:e].to(torch.int64)
            tb = topk_b[kh, a:e].to(torch.int64)
            for n in range(e - a):
                nk = (n + off) // block_size
                nv = min(top_n, nk + 1)
                sa = set(ta[n, :nv].tolist())
                sb = set(tb[n, :nv].tolist())
                n_rows += 1
                if sa == sb:
                    continue
                n_diff += 1
                diff = sa ^ sb
                if any((j < 0 or j > nk) for j in diff):
                    n_bad += 1
                    continue
                vals = torch.stack([imp[kh, n, j] for j in sorted(diff)])
                if float(vals.max() - vals.min()) > tie_tol:
                    n_bad += 1
    return n_rows, n_diff, n_bad

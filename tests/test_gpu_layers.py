"""The layer around the core: fused rotary embedding and the two demo layers (projections -> RoPE -> core ->
output projection)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import nsa_oracle as O
from gpu_util import assert_close, make_cu, randn_bf16

pytestmark = pytest.mark.gpu


def tables(b, s, d, dtype, seed=0, distinct_halves=False):
    inv = 1.0 / (10000 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    ang = (torch.arange(s, dtype=torch.float32)[:, None] + seed) * inv[None]
    cos, sin = torch.cat([ang.cos(), ang.cos()], -1), torch.cat([ang.sin(), ang.sin()], -1)
    if distinct_halves:  # the kernel treats the two halves of the tables independently, as upstream's does
        g = torch.Generator().manual_seed(seed)
        cos, sin = torch.randn(s, d, generator=g), torch.randn(s, d, generator=g)
    return cos.expand(b, s, d).to(dtype).contiguous(), sin.expand(b, s, d).to(dtype).contiguous()


@pytest.mark.parametrize("b,s,QH,KH,D", [(1, 300, 16, 2, 128), (3, 65, 4, 4, 64), (2, 17, 8, 1, 192)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("inplace", [False, True])
def test_rope_forward_and_backward(device, b, s, QH, KH, D, dtype, inplace):
    from flash_nsa import fused_apply_rope
    q, k = randn_bf16(b, s, QH, D, seed=1), randn_bf16(b, s, KH, D, seed=2)
    cos, sin = tables(b, s, D, dtype, seed=3, distinct_halves=(D == 64))
    rq, rk = O.rope(q.float(), cos.float(), sin.float()), O.rope(k.float(), cos.float(), sin.float())
    qd, kd = q.to(device).requires_grad_(), k.to(device).requires_grad_()
    # a leaf cannot be modified in place: rotate a product of it, as a layer rotates the output of a projection
    qe, ke = fused_apply_rope(qd * 1, kd * 1, cos.to(device), sin.to(device), inplace=inplace)
    # fp32 arithmetic, one rounding to bf16: equal to the rounded oracle up to the last bit (the absolute term
    # covers x*cos ~ y*sin, where a fused multiply-add and a separate one differ by an fp32 ulp of the products)
    assert_close(qe, rq.to(torch.bfloat16).float(), "qe", atol=2e-6, rtol=8e-3)
    assert_close(ke, rk.to(torch.bfloat16).float(), "ke", atol=2e-6, rtol=8e-3)
    dq, dk = randn_bf16(b, s, QH, D, seed=4), randn_bf16(b, s, KH, D, seed=5)
    torch.autograd.backward([qe, ke], [dq.to(device), dk.to(device)])
    ql, kl = q.float().requires_grad_(), k.float().requires_grad_()
    torch.autograd.backward([O.rope(ql, cos.float(), sin.float()), O.rope(kl, cos.float(), sin.float())],
                            [dq.float(), dk.float()])
    assert_close(qd.grad, ql.grad.to(torch.bfloat16).float(), "dq", atol=2e-6, rtol=8e-3)
    assert_close(kd.grad, kl.grad.to(torch.bfloat16).float(), "dk", atol=2e-6, rtol=8e-3)


def test_rope_strided_views_and_broadcast_table(device):
    """q / k as slices of one fused projection output (token stride larger than the row) and a [1,s,d] table."""
    from flash_nsa import fused_apply_rope
    b, s, QH, KH, D = 2, 40, 8, 2, 128
    fused = randn_bf16(b, s, (QH + KH) * D + 24, seed=7).to(device)
    q = fused[..., :QH * D].view(b, s, QH, D)
    k = fused[..., QH * D:(QH + KH) * D].view(b, s, KH, D)
    cos, sin = tables(1, s, D, torch.float32)
    want_q, want_k = O.rope(q.float().cpu(), cos, sin), O.rope(k.float().cpu(), cos, sin)
    tail = fused[..., (QH + KH) * D:].clone()
    qe, ke = fused_apply_rope(q, k, cos.to(device), sin.to(device), inplace=True)
    assert qe.data_ptr() == q.data_ptr() and torch.equal(fused[..., (QH + KH) * D:], tail)
    assert_close(qe, want_q.to(torch.bfloat16).float(), "qe", atol=2e-6, rtol=8e-3)
    assert_close(ke, want_k.to(torch.bfloat16).float(), "ke", atol=2e-6, rtol=8e-3)


def _layer_reference(x, cos, sin, weights, cfg_kw, cu, QH, KH, D, topk, d_out):
    """Forward and backward of the layer on the CPU in fp32 with the pipeline's rounding points: every tensor the
    device stores in bf16 between two stages (projection outputs, rotated q / k, the core's output and gradients,
    the gradients handed back through RoPE and the projections) is rounded, the arithmetic in between is fp32.
    -> (layer output, d hidden_states)"""
    wq, wk, wv, ww, wo = weights
    r = lambda t: t.to(torch.bfloat16).float()
    b, s, _ = x.shape
    q = r(F.linear(x, wq)).view(b, s, QH, D)
    k = r(F.linear(x, wk)).view(b, s, KH, D)
    v = r(F.linear(x, wv)).view(b, s, KH, D)
    w = r(F.linear(x, ww)).view(b, s, QH, 3)
    ql, kl = q.clone().requires_grad_(), k.clone().requires_grad_()
    qe, ke = O.rope(ql, cos, sin), O.rope(kl, cos, sin)
    d_core = r(d_out @ wo).view(b * s, QH, D)
    core = O.nsa_forward_backward(r(qe.detach()).flatten(0, 1), r(ke.detach()).flatten(0, 1), v.flatten(0, 1),
                                  w.flatten(0, 1), d_core, cu, O.OracleConfig(**cfg_kw), topk=topk,
                                  round_dtype=torch.bfloat16, round_mma=True)
    out = F.linear(core["o"].view(b, s, -1), wo)
    dq, dk = torch.autograd.grad([qe, ke], [ql, kl], [core["dq"].view_as(qe), core["dk"].view_as(ke)])
    gx = (r(dq).flatten(2) @ wq + r(dk).flatten(2) @ wk + core["dv"].view(b, s, -1) @ wv +
          core["dw"].view(b, s, -1) @ ww)
    return out, gx


@pytest.mark.parametrize("kind", ["hf", "megatron"])
def test_attention_layers_forward_backward(device, kind):
    from flash_nsa import NSAConfig, HFNSA, NSA, NSAHelper
    from flash_nsa.ops.compress_kv import mean_pooling_fwd
    from flash_nsa.ops.compress_attn import cmp_attn_fwd
    from flash_nsa.ops.topk import slc_topk_indices
    from flash_nsa import fused_apply_rope
    b, s, hidden, QH, KH, D = 2, 260, 256, 8, 2, 64
    cfg_kw = dict(top_n=6, window_size=96)
    cfg = NSAConfig(hidden_size=hidden, head_dim=D, num_heads=QH, num_kv_heads=KH, **cfg_kw)
    torch.manual_seed(0)
    layer = (HFNSA(cfg) if kind == "hf" else NSA(cfg)).to(device=device, dtype=torch.bfloat16)
    x = (randn_bf16(b, s, hidden, seed=11) * 0.5)
    cos, sin = tables(b, s, D, torch.float32)
    cu = make_cu([s] * b)
    if kind == "hf":
        weights = [m.weight.detach().float().cpu() for m in
                   (layer.q_proj, layer.k_proj, layer.v_proj, layer.combine_proj, layer.o_proj)]
        xd = x.to(device).requires_grad_()
        out = layer(xd, (cos.to(device), sin.to(device)), cu.to(device))
    else:
        wq, wk, wv, ww, _ = layer.qkv_proj.weight.detach().float().cpu().split(layer.split_size, 0)
        weights = [wq, wk, wv, ww, layer.o_proj.weight.detach().float().cpu()]
        xd = x.to(device).transpose(0, 1).contiguous().requires_grad_()       # sequence first
        out = layer(xd, (cos.to(device), sin.to(device)), {"cu_seqlens": cu.to(device)}).transpose(0, 1)
    # the device's own block selection, so that a near-tie cannot change which keys the two sides attend
    with torch.no_grad():
        r = lambda t: t.to(torch.bfloat16)
        xq = x.to(device)
        qd = F.linear(xq, r(weights[0]).to(device)).view(b, s, QH, D)
        kd = F.linear(xq, r(weights[1]).to(device)).view(b, s, KH, D)
        qd, kd = fused_apply_rope(qd, kd, cos.to(device), sin.to(device))
        NSAHelper.set_hyperparameters(**cfg_kw)
        NSAHelper.init_cu_seqlens(cu.to(device))
        ck = mean_pooling_fwd(kd.flatten(0, 1))
        _, lse = cmp_attn_fwd(qd.flatten(0, 1), ck, ck)
        topk, _ = slc_topk_indices(qd.flatten(0, 1), ck, lse)
    do = randn_bf16(b, s, hidden, seed=12)
    ref_out, ref_gx = _layer_reference(x.float(), cos, sin, weights, cfg_kw, cu, QH, KH, D, topk.cpu(), do.float())
    assert_close(out, ref_out, "layer output")
    out.backward(do.to(device))
    gx = xd.grad if kind == "hf" else xd.grad.transpose(0, 1)
    assert_close(gx, ref_gx, "d hidden_states")
    NSAHelper.set_hyperparameters()

"""R11 at its own size (benchmark configuration 5): the attention sub-chain of one DiT block at 720p,
x [1, 86400, 4096] bf16, weights ~ N(0, 0.02), 32 heads x 128, latent grid 24 x 45 x 80, density 1/16
(longcat_video/modules/attention.py:107-147).

The whole chain is far too large for the CPU oracle, so every stage is checked on samples against the oracle
fed with the GPU's own inputs of that stage:
  * the two projections at M = 86 400 (N = 12 288 and N = 4 096, bias, residual): sampled rows against an fp32
    matmul, with the output and the GEMM workspace placed inside one larger allocation whose guard regions must
    survive (a GEMM library handed less workspace than it uses once wrote past it at exactly this size);
  * per-head RMSNorm + 3-D RoPE and the move into per-head tensors: sampled tokens;
  * the operator on the module's q, k, v: selection bit-exact given the scores, sampled query blocks of two
    heads against the gathered fp32 oracle;
  * the module's forward and `attention_block_forward` against the staged evaluation.
"""
import math

import numpy as np
import pytest
import torch

from oracle import bsa_oracle as O
from test_gpu_e2e import check_against_oracle

pytestmark = pytest.mark.gpu

BF16_ULP = 2.0 ** -7
SHAPE = (24, 45, 80)
N_TOK, DIM, HEADS = 86400, 4096, 32
GUARD = 1 << 20
SENTINEL = 0xA5


def M():
    from longcat_video_amd.modules import attention
    return attention


def guarded(sizes):
    """One uint8 allocation filled with a sentinel, holding slices of the given byte sizes (256-byte aligned)
    with a guard region before, between and behind them.  Returns (whole buffer, slices, guard ranges)."""
    offs, off, guards = [], 0, []
    for n in sizes:
        guards.append((off, off + GUARD))
        off += GUARD
        offs.append(off)
        off += (n + 255) // 256 * 256
    guards.append((off, off + GUARD))
    off += GUARD
    buf = torch.full((off,), SENTINEL, dtype=torch.uint8, device="cuda")
    return buf, [buf[o:o + n] for o, n in zip(offs, sizes)], guards


def assert_guards(buf, guards, what):
    for lo, hi in guards:
        assert bool((buf[lo:hi] == SENTINEL).all()), "%s: bytes %d..%d next to a GEMM buffer were overwritten" % (what, lo, hi)


def sampled_rows(n, count, seed):
    g = torch.Generator().manual_seed(seed)
    rows = torch.randint(0, n, (count,), generator=g)
    rows[0], rows[1] = 0, n - 1
    return rows


@pytest.fixture(scope="module")
def c5():
    g = torch.Generator(device="cuda").manual_seed(4)
    x = torch.randn(1, N_TOK, DIM, generator=g, device="cuda").bfloat16()
    m = M().Attention(DIM, HEADS, enable_bsa=True,
                      bsa_params=dict(sparsity=0.9375, cdf_threshold=None, chunk_3d_shape_q=[4, 4, 4], chunk_3d_shape_k=[4, 4, 4]),
                      cp_split_hw=[1, 1])
    cg = torch.Generator().manual_seed(5)
    with torch.no_grad():
        for p in (m.qkv.weight, m.proj.weight, m.qkv.bias, m.proj.bias):
            p.copy_(torch.randn(p.shape, generator=cg) * 0.02)
        m.q_norm.weight.copy_(1 + 0.1 * torch.randn(128, generator=cg))
        m.k_norm.weight.copy_(1 + 0.1 * torch.randn(128, generator=cg))
    return x, m.to(torch.bfloat16).cuda()


@pytest.mark.parametrize("n_out,with_residual", [(3 * DIM, False), (DIM, True)])
def test_projection_at_720p_size_stays_inside_its_buffers(c5, n_out, with_residual):
    x, m = c5
    layer = m.qkv if n_out == 3 * DIM else m.proj
    out_bytes, ws_bytes = N_TOK * n_out * 2, 64 << 20
    buf, (ws, out_raw), guards = guarded([ws_bytes, out_bytes])
    out = out_raw.view(torch.bfloat16).view(N_TOK, n_out)
    res = None
    if with_residual:
        res = torch.randn(1, N_TOK, n_out, generator=torch.Generator(device="cuda").manual_seed(6), device="cuda").bfloat16()
    y = M().linear_bf16(x, layer.weight, layer.bias, residual=res, workspace=ws, out=out)
    torch.cuda.synchronize()
    assert y.data_ptr() == out.data_ptr()
    assert_guards(buf, guards, "linear %d -> %d" % (DIM, n_out))
    rows = sampled_rows(N_TOK, 48, 7)
    want = x[0, rows].float().cpu() @ layer.weight.float().cpu().t() + layer.bias.float().cpu()
    if with_residual:
        want = want + res[0, rows].float().cpu()
    got = out[rows].float().cpu()
    assert torch.all((got - want).abs() <= want.abs() * BF16_ULP + 4e-3), float((got - want).abs().max())
    assert torch.isfinite(out.float()).all()


def test_module_stages_at_720p_size(c5):
    x, m = c5
    att = M()
    B, N, C, Hn, D = 1, N_TOK, DIM, HEADS, 128
    eps = m.q_norm.eps
    # ---- projection, as Attention._project_qkv does it
    qs, ks, vs = m._project_qkv(x)
    # ---- norm + RoPE + move, as Attention.forward does it
    new = lambda: torch.empty(B, Hn, N, D, dtype=x.dtype, device=x.device)
    q = att.norm_rope(qs, new(), m.q_norm.weight, SHAPE, eps=eps)
    k = att.norm_rope(ks, new(), m.k_norm.weight, SHAPE, eps=eps)
    v = att.norm_rope(vs, new())
    torch.cuda.synchronize()
    assert torch.equal(v, vs)                                            # a plain move
    toks = sampled_rows(N, 96, 8)
    ang = O.rope_3d_angles(SHAPE, D)[toks]
    for got, src, w in ((q, qs, m.q_norm.weight), (k, ks, m.k_norm.weight)):
        s = src[:, :, toks].cpu()                                        # [1, H, n, D]
        want = O.rope_3d_apply(O.rms_norm_fp32(s, w.cpu()), ang)
        d = (got[:, :, toks].cpu().float() - want.float()).abs()
        assert torch.all(d <= want.float().abs() * 3 * BF16_ULP + 0.02), float(d.max())
        assert (d > 0).float().mean() < 0.05
    # ---- the operator on the module's own q, k, v
    from longcat_video_amd.block_sparse_attention import bsa_interface as bi
    o = torch.empty(B, N, Hn, D, dtype=x.dtype, device=x.device)
    ov = o.permute(0, 2, 1, 3)
    _, idx, lens, score = bi._bsa_3d(q, k, v, SHAPE, SHAPE, 0.9375, (4, 4, 4), (4, 4, 4), True, out=ov)
    torch.cuda.synchronize()
    assert idx.shape == (1, 32, 1440, 90)
    heads = [3, 30]
    check_against_oracle(q.cpu(), k.cpu(), v.cpu(), SHAPE, SHAPE, 0.9375, ov, idx, lens, score,
                         q_blocks=[0, 77, 1000, 1439], heads=heads)
    assert torch.isfinite(o.float()).all()
    # ---- output projection with the residual fused
    y = att.linear_bf16(o.view(B, N, C), m.proj.weight, m.proj.bias, residual=x)
    rows = sampled_rows(N, 48, 9)
    want = o.view(N, C)[rows].float().cpu() @ m.proj.weight.float().cpu().t() + m.proj.bias.float().cpu() + x[0, rows].float().cpu()
    got = y[0, rows].float().cpu()
    assert torch.all((got - want).abs() <= want.abs() * BF16_ULP + 2e-2), float((got - want).abs().max())
    # ---- the module's forward is this sequence
    y_mod = m(x, shape=SHAPE, residual=x)
    torch.cuda.synchronize()
    assert torch.equal(y_mod, y)


def test_engine_projections_at_720p_size(c5):
    """The engine's own GEMM at the two projection shapes of the module: the fused QKV projection (norm, rotation,
    head split in the epilogue) against the hipBLASLt route's q, k, v on sampled tokens and against the oracle's
    chain on fp32 products of sampled rows; the output projection with bias and residual against fp32."""
    x, m = c5
    att = M()
    B, N, C, Hn, D = 1, N_TOK, DIM, HEADS, 128
    q, k, v = att.qkv_projection(x, m.qkv.weight, m.qkv.bias, m.q_norm.weight, m.k_norm.weight, SHAPE, Hn, eps=m.q_norm.eps)
    torch.cuda.synchronize()
    assert q.shape == (B, Hn, N, D) and torch.isfinite(q.float()).all() and torch.isfinite(k.float()).all()
    toks = torch.cat([sampled_rows(N, 64, 12), torch.tensor([255, 256, N - 129, N - 128])])   # tile edges and the half tile at the end
    rows = x[0, toks].float().cpu() @ m.qkv.weight.float().cpu().t() + m.qkv.bias.float().cpu()      # [n, 3C] in fp32
    qkv = rows.bfloat16().view(len(toks), 3, Hn, D).permute(1, 2, 0, 3)[:, None]                    # [3, 1, H, n, D]
    ang = O.rope_3d_angles(SHAPE, D)[toks]
    assert torch.all((v[:, :, toks].cpu().float() - qkv[2].float()).abs() <= qkv[2].float().abs() * BF16_ULP + 4e-3)
    for got, src, w in ((q, qkv[0], m.q_norm.weight), (k, qkv[1], m.k_norm.weight)):
        want = O.rope_3d_apply(O.rms_norm_fp32(src, w.cpu()), ang)
        d = (got[:, :, toks].cpu().float() - want.float()).abs()
        # the projection feeding the norm may differ by one rounding from the fp32 one: a few ulps after the norm
        assert torch.all(d <= want.float().abs() * 4 * BF16_ULP + 0.03), float(d.max())
        assert (d > want.float().abs() * BF16_ULP + 1e-3).float().mean() < 0.02
    # the module's two routes agree closely (different summation orders inside the GEMMs)
    y_lt = m(x, shape=SHAPE, residual=x)
    m.projection_backend = "engine"
    try:
        y_en = m(x, shape=SHAPE, residual=x)
    finally:
        m.projection_backend = "hipblaslt"
    torch.cuda.synchronize()
    assert torch.isfinite(y_en.float()).all()
    d = (y_en.float() - y_lt.float()).abs()
    assert d.mean() <= 4e-3 and (d > 0.25).float().mean() < 1e-3, (float(d.mean()), float(d.max()))
    # output projection
    o = torch.randn(N, C, generator=torch.Generator(device="cuda").manual_seed(13), device="cuda").bfloat16()
    y = att.gemm_bf16(o, m.proj.weight, m.proj.bias, residual=x[0])
    rows = sampled_rows(N, 48, 14)
    want = o[rows].float().cpu() @ m.proj.weight.float().cpu().t() + m.proj.bias.float().cpu() + x[0, rows].float().cpu()
    assert torch.all((y[rows].float().cpu() - want).abs() <= want.abs() * BF16_ULP + 2e-2)


def test_attention_block_forward_at_720p_size(c5):
    """RMSNorm -> module -> residual (benchmark configuration 5 as worded): finite, deterministic, and the
    pre-norm agrees with the oracle on sampled rows; the module behind it is covered stage by stage above."""
    x, m = c5
    att = M()
    wn = (1 + 0.1 * torch.randn(DIM, generator=torch.Generator().manual_seed(10))).bfloat16().cuda()
    y = att.attention_block_forward(x, wn, m, SHAPE)
    torch.cuda.synchronize()
    assert y.shape == x.shape and y.dtype == torch.bfloat16 and torch.isfinite(y.float()).all()
    rows = sampled_rows(N_TOK, 32, 11)
    xn = att.rms_norm(x, wn, 1e-6)
    want = O.rms_norm_fp32(x[0, rows].cpu(), wn.cpu())
    assert torch.all((xn[0, rows].cpu().float() - want.float()).abs() <= want.float().abs() * 2 * BF16_ULP + 1e-6)
    y2 = m(xn, shape=SHAPE, residual=x)
    torch.cuda.synchronize()
    assert torch.equal(y, y2)

"""R10/R11 on the GPU: the attention-module glue (linear layers, RMSNorm, QK-norm +
3-D RoPE), the conditioning/noise split, and the whole module against the oracle."""
import math

import numpy as np
import pytest
import torch

from oracle import bsa_oracle as O

pytestmark = pytest.mark.gpu

BF16_ULP = 2.0 ** -7


def M():
    from longcat_video_amd.modules import attention
    return attention


def make_module(dim=512, heads=4, sparsity=0.5, seed=0):
    g = torch.Generator().manual_seed(seed)
    m = M().Attention(dim, heads, enable_bsa=True,
                      bsa_params=dict(sparsity=sparsity, cdf_threshold=None, chunk_3d_shape_q=[4, 4, 4], chunk_3d_shape_k=[4, 4, 4]),
                      cp_split_hw=[1, 1])
    with torch.no_grad():
        for p in (m.qkv.weight, m.proj.weight):
            p.copy_(torch.randn(p.shape, generator=g) * 0.02)
        m.qkv.bias.copy_(torch.randn(m.qkv.bias.shape, generator=g) * 0.02)
        m.proj.bias.copy_(torch.randn(m.proj.bias.shape, generator=g) * 0.02)
        m.q_norm.weight.copy_(1 + 0.1 * torch.randn(128, generator=g))
        m.k_norm.weight.copy_(1 + 0.1 * torch.randn(128, generator=g))
    return m.to(torch.bfloat16)


def test_state_dict_names_match_the_reference_module():
    m = M().Attention(512, 4, enable_bsa=True, bsa_params={}, cp_split_hw=[1, 1])
    assert sorted(m.state_dict()) == ["k_norm.weight", "proj.bias", "proj.weight", "q_norm.weight", "qkv.bias", "qkv.weight"]
    assert m.qkv.weight.shape == (1536, 512) and m.q_norm.weight.shape == (128,)


def test_row_rmsnorm():
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(3, 37, 4096, generator=g) * 3).bfloat16()
    w = (1 + 0.2 * torch.randn(4096, generator=g)).bfloat16()
    got = M().rms_norm(x.cuda(), w.cuda(), 1e-6).cpu()
    want = O.rms_norm_fp32(x, w)
    assert got.dtype == torch.bfloat16
    assert torch.all((got.float() - want.float()).abs() <= want.float().abs() * 2 * BF16_ULP + 1e-6)
    assert (got.float() - want.float()).abs().mean() < 1e-3


def test_linear_with_bias_and_residual():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(2, 100, 512, generator=g).bfloat16()
    w = (torch.randn(384, 512, generator=g) * 0.05).bfloat16()
    b = torch.randn(384, generator=g).bfloat16()
    r = torch.randn(2, 100, 384, generator=g).bfloat16()
    want = x.float() @ w.float().t() + b.float()
    got = M().linear_bf16(x.cuda(), w.cuda(), b.cuda()).cpu()
    assert got.shape == (2, 100, 384)
    assert torch.all((got.float() - want).abs() <= want.abs() * BF16_ULP + 2e-3)
    got_r = M().linear_bf16(x.cuda(), w.cuda(), b.cuda(), residual=r.cuda()).cpu()
    assert torch.all((got_r.float() - (want + r.float())).abs() <= (want + r.float()).abs() * BF16_ULP + 2e-2)
    got_nb = M().linear_bf16(x.cuda(), w.cuda(), None).cpu()
    assert torch.all((got_nb.float() - (want - b.float())).abs() <= (want - b.float()).abs() * BF16_ULP + 2e-3)


def test_qk_norm_rope_against_the_oracle():
    grid = (3, 5, 7)
    S = 105
    g = torch.Generator().manual_seed(3)
    qkv = (torch.randn(2, S, 3, 4, 128, generator=g) * 2).bfloat16()
    qw = (1 + 0.1 * torch.randn(128, generator=g)).bfloat16()
    kw = (1 + 0.1 * torch.randn(128, generator=g)).bfloat16()
    q, k, v = qkv.permute(2, 0, 3, 1, 4).unbind(0)
    ang = O.rope_3d_angles(grid, 128)
    want_q = O.rope_3d_apply(O.rms_norm_fp32(q, qw), ang)
    want_k = O.rope_3d_apply(O.rms_norm_fp32(k, kw), ang)
    dev = qkv.cuda()
    dq, dk, dv = dev.permute(2, 0, 3, 1, 4).unbind(0)
    M().qk_norm_rope_(dq, dk, qw.cuda(), kw.cuda(), grid)
    for got, want in ((dq.cpu(), want_q), (dk.cpu(), want_k)):
        d = (got.float() - want.float()).abs()
        # three roundings (norm, weight, rotation): a couple of ulps at most, almost always none
        assert torch.all(d <= want.float().abs() * 3 * BF16_ULP + 0.02)
        assert (d > 0).float().mean() < 0.05
    assert torch.equal(dv.cpu(), v)                       # v is untouched
    # rotation keeps the norm of the normalised vector
    n_in = O.rms_norm_fp32(q, qw).float().norm(dim=-1)
    assert torch.allclose(dq.cpu().float().norm(dim=-1), n_in, rtol=2e-2)


def module_reference(m, x, shape, num_cond=0):
    """Oracle evaluation of the module on the CPU with the module's own weights."""
    sd = {k: v.detach().cpu() for k, v in m.state_dict().items()}
    prm = dict(sparsity=m.bsa_params["sparsity"], chunk_3d_shape_q=tuple(m.bsa_params["chunk_3d_shape_q"]),
               chunk_3d_shape_k=tuple(m.bsa_params["chunk_3d_shape_k"]))
    return O.attention_module_forward(x, sd["qkv.weight"], sd["qkv.bias"], sd["proj.weight"], sd["proj.bias"],
                                      sd["q_norm.weight"], sd["k_norm.weight"], shape, m.num_heads, prm, num_cond)


@pytest.mark.parametrize("sparsity", [0.0, 0.5])
def test_module_forward_matches_the_oracle(sparsity):
    shape = (4, 8, 8)
    m = make_module(sparsity=sparsity)
    x = torch.randn(1, 256, 512, generator=torch.Generator().manual_seed(4)).bfloat16()
    want = module_reference(m, x, shape)
    got = m.cuda()(x.cuda(), shape=shape).cpu()
    assert got.shape == (1, 256, 512) and got.dtype == torch.bfloat16
    d = (got.float() - want.float()).abs()
    assert d.max() <= 2e-2 and d.mean() <= 2e-3, (d.max(), d.mean())


def test_cond_noise_split():
    """attention.py:124-135: conditioning rows only see conditioning tokens."""
    shape, cond = (8, 8, 8), 4
    m = make_module(sparsity=0.5, seed=5)
    x = torch.randn(1, 512, 512, generator=torch.Generator().manual_seed(6)).bfloat16()
    want = module_reference(m, x, shape, num_cond=cond)
    mc = m.cuda()
    got = mc(x.cuda(), shape=shape, num_cond_latents=cond).cpu()
    d = (got.float() - want.float()).abs()
    assert d.max() <= 2e-2 and d.mean() <= 2e-3, (d.max(), d.mean())
    # perturbing noise tokens must leave the conditioning rows bit-identical
    x2 = x.clone()
    x2[:, 256:] += 1.0
    got2 = mc(x2.cuda(), shape=shape, num_cond_latents=cond).cpu()
    assert torch.equal(got[:, :256], got2[:, :256]) and not torch.equal(got[:, 256:], got2[:, 256:])


def test_attention_block_with_pre_norm_and_residual():
    shape = (4, 8, 8)
    m = make_module(sparsity=0.5, seed=7)
    g = torch.Generator().manual_seed(8)
    x = torch.randn(1, 256, 512, generator=g).bfloat16()
    wn = (1 + 0.1 * torch.randn(512, generator=g)).bfloat16()
    y = O.rms_norm_fp32(x, wn)
    want = (x.float() + module_reference(m, y, shape).float())
    got = M().attention_block_forward(x.cuda(), wn.cuda(), m.cuda(), shape).cpu()
    d = (got.float() - want).abs()
    assert d.max() <= 4e-2 and d.mean() <= 4e-3, (d.max(), d.mean())


def test_unbuilt_branches_raise():
    m = make_module().cuda()
    x = torch.zeros(1, 256, 512, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(NotImplementedError):
        m(x, shape=(4, 8, 8), return_kv=True)
    with pytest.raises(NotImplementedError):
        m.forward_with_kv_cache(x)
    m.enable_bsa = False
    with pytest.raises(NotImplementedError):
        m(x, shape=(4, 8, 8))

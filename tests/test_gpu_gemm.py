"""R11 on the GPU: the engine's own MFMA GEMM (bsa_gemm_bf16) against an fp32 matrix product, and the QKV
projection with its fused epilogue (bsa_qkv_projection) against the oracle's Linear -> RMSNorm -> RoPE chain
(attention.py:111-121)."""
import pytest
import torch

from oracle import bsa_oracle as O

pytestmark = pytest.mark.gpu

BF16_ULP = 2.0 ** -7


def M():
    from longcat_video_amd.modules import attention
    return attention


@pytest.mark.parametrize("m,n,k", [(256, 256, 64), (300, 256, 192), (77, 128, 64), (1000, 384, 4096), (5000, 1280, 1024)])
def test_gemm_against_an_fp32_product(m, n, k):
    """Ragged row counts, a feature count that fills only half of the last tile, one k block and many; with
    bias, and with bias and residual.  One rounding at the end: equal to the rounded fp32 product except where
    the fp32 sums, taken in another order, fall on the other side of a rounding boundary."""
    g = torch.Generator().manual_seed(m + n + k)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.05).bfloat16()
    b = torch.randn(n, generator=g).bfloat16()
    r = torch.randn(m, n, generator=g).bfloat16()
    ref = x.cuda().float() @ w.cuda().float().T
    for bias, res in ((None, None), (b, None), (b, r)):
        got = M().gemm_bf16(x.cuda(), w.cuda(), None if bias is None else bias.cuda(), None if res is None else res.cuda())
        want = ref + (0 if bias is None else bias.cuda().float()) + (0 if res is None else res.cuda().float())
        assert got.shape == (m, n) and got.dtype == torch.bfloat16
        d = (got.float() - want).abs()
        assert torch.all(d <= want.abs() * BF16_ULP + 1e-3 * (k / 64) ** 0.5)
        assert (got == want.bfloat16()).float().mean() > 0.995


def test_gemm_is_exact_on_integers():
    """Small integers: every product and every partial sum is exact in fp32, so a dropped k block, a swapped
    fragment or a wrong row shows as a wrong integer."""
    g = torch.Generator().manual_seed(5)
    m, n, k = 515, 384, 320
    x = torch.randint(-3, 4, (m, k), generator=g).bfloat16()
    w = torch.randint(-2, 3, (n, k), generator=g).bfloat16()
    b = torch.randint(-4, 5, (n,), generator=g).bfloat16()
    got = M().gemm_bf16(x.cuda(), w.cuda(), b.cuda()).cpu()
    want = (x.double() @ w.double().T + b.double()).to(torch.bfloat16)
    assert torch.equal(got, want)


def test_gemm_with_row_strides():
    """Operands and output as column slices of wider tensors (row strides above K and N)."""
    g = torch.Generator().manual_seed(6)
    m, n, k = 333, 256, 128
    xw = torch.randn(m, k + 64, generator=g).bfloat16().cuda()
    ww = (torch.randn(n, k + 8, generator=g) * 0.1).bfloat16().cuda()
    outw = torch.full((m, n + 128), 7.0, dtype=torch.bfloat16).cuda()
    got = M().gemm_bf16(xw[:, :k], ww[:, :k], None, out=outw[:, :n])
    want = xw[:, :k].float() @ ww[:, :k].float().T
    assert torch.all((got.float() - want).abs() <= want.abs() * BF16_ULP + 2e-3)
    assert torch.all(outw[:, n:] == 7.0)                                   # nothing written beside the slice


def test_gemm_rejects_bad_arguments():
    x = torch.zeros(64, 96, dtype=torch.bfloat16).cuda()
    w = torch.zeros(128, 96, dtype=torch.bfloat16).cuda()
    with pytest.raises(NotImplementedError):                                 # K is not a multiple of 64
        M().gemm_bf16(x, w, None)
    with pytest.raises(NotImplementedError):                                 # N is not a multiple of 128
        M().gemm_bf16(torch.zeros(64, 64, dtype=torch.bfloat16).cuda(), torch.zeros(72, 64, dtype=torch.bfloat16).cuda(), None)


@pytest.mark.parametrize("grid,batch,heads", [((3, 5, 7), 2, 4), ((2, 16, 17), 1, 2)])
def test_qkv_projection_against_the_oracle(grid, batch, heads):
    """Linear, head split, RMSNorm of q and k, RoPE; ragged token counts (105 and 544 per batch entry, so a
    256-token tile spans two batch entries in the first case)."""
    S = grid[0] * grid[1] * grid[2]
    C = heads * 128
    g = torch.Generator().manual_seed(S)
    x = torch.randn(batch, S, C, generator=g).bfloat16()
    w = (torch.randn(3 * C, C, generator=g) * C ** -0.5 * 2).bfloat16()
    b = (torch.randn(3 * C, generator=g) * 0.1).bfloat16()
    qw = (1 + 0.1 * torch.randn(128, generator=g)).bfloat16()
    kw = (1 + 0.1 * torch.randn(128, generator=g)).bfloat16()
    q, k, v = M().qkv_projection(x.cuda(), w.cuda(), b.cuda(), qw.cuda(), kw.cuda(), grid, heads)
    assert q.shape == (batch, heads, S, 128) and q.is_contiguous() and k.is_contiguous() and v.is_contiguous()
    # the projection itself, as the plain entry point computes it (bit-equal accumulation order)
    qkv = M().gemm_bf16(x.cuda(), w.cuda(), b.cuda()).cpu()
    ref = (x.double() @ w.double().T + b.double()).float()
    assert torch.all((qkv.float() - ref).abs() <= ref.abs() * BF16_ULP + 4e-3)
    qs, ks, vs = qkv.view(batch, S, 3, heads, 128).permute(2, 0, 3, 1, 4).unbind(0)
    assert torch.equal(v.cpu(), vs)
    ang = O.rope_3d_angles(grid, 128)
    for got, src, nw in ((q.cpu(), qs, qw), (k.cpu(), ks, kw)):
        want = O.rope_3d_apply(O.rms_norm_fp32(src, nw), ang)
        d = (got.float() - want.float()).abs()
        # three roundings (norm, weight, rotation): a couple of ulps at most, almost always none
        assert torch.all(d <= want.float().abs() * 3 * BF16_ULP + 0.02)
        assert (d > 0).float().mean() < 0.05
    # and against the engine's separate pass, which rounds at the same points
    sep = M().norm_rope(qs.cuda(), torch.empty_like(q), qw.cuda(), grid)
    assert (sep != q).float().mean() < 0.01


def test_qkv_projection_frame_offset():
    """Tokens that are frames 2.. of a larger grid take the rotation angles of those frames."""
    grid, full = (2, 4, 8), (4, 4, 8)
    heads, C = 2, 256
    S = grid[0] * grid[1] * grid[2]
    g = torch.Generator().manual_seed(11)
    x = torch.randn(1, S, C, generator=g).bfloat16().cuda()
    w = (torch.randn(3 * C, C, generator=g) * 0.1).bfloat16().cuda()
    qw = torch.ones(128).bfloat16().cuda()
    q_off, k_off, _ = M().qkv_projection(x, w, None, qw, qw, grid, heads, t_offset=2, table_grid=full)
    xx = torch.cat([torch.zeros_like(x), x], dim=1)
    q_full, k_full, _ = M().qkv_projection(xx, w, None, qw, qw, full, heads)
    assert torch.equal(q_off, q_full[:, :, S:]) and torch.equal(k_off, k_full[:, :, S:])

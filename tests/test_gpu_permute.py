"""R0/R1/R7 on the GPU: the HIP permute / unpermute kernels are bit-exact against
the oracle, including padded grids, strided sources and the fused pooled mean."""
import numpy as np
import pytest
import torch

from oracle import bsa_oracle as O

pytestmark = pytest.mark.gpu

GRIDS = [
    ((4, 8, 8), (4, 4, 4)),
    ((8, 8, 8), (4, 4, 8)),
    ((5, 6, 7), (4, 4, 4)),
    ((4, 9, 13), (4, 4, 4)),
    ((3, 4, 8), (2, 2, 2)),
    ((1, 1, 1), (4, 4, 4)),
]


def I():
    from longcat_video_amd.block_sparse_attention import bsa_interface
    return bsa_interface


@pytest.mark.parametrize("latent,chunk", GRIDS)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_permute_and_unpermute_bit_exact(latent, chunk, dtype):
    S = int(np.prod(latent))
    x = torch.randn(2, 3, S, 128, generator=torch.Generator().manual_seed(1)).to(dtype)
    Nt, Nh, Nw = O.block_grid(latent, chunk)
    got = I().rearrange_THW_to_3d_block(x.cuda(), Nt, Nh, Nw, *chunk, 128, latent_shape=latent)
    want = O.rearrange_thw_to_3d_block(x, latent, chunk)
    assert got.is_contiguous() and torch.equal(got.cpu().view(torch.uint8), want.view(torch.uint8))
    back = I().rearrange_3d_block_to_THW(got, Nt, Nh, Nw, *chunk, 128, latent_shape=latent)
    assert torch.equal(back.cpu().view(torch.uint8), x.view(torch.uint8))


def test_permute_of_strided_qkv_views():
    """q, k, v as the attention module hands them over: slices of one
    [B, N, 3, H, D] GEMM output viewed as [B, H, N, D] (attention.py:113-115)."""
    latent, chunk = (4, 6, 10), (4, 4, 4)
    N = 240
    qkv = torch.randn(2, N, 3, 4, 128, generator=torch.Generator().manual_seed(2)).bfloat16()
    dev = qkv.cuda().permute(2, 0, 3, 1, 4)
    for i in range(3):
        src = dev[i]
        assert not src.is_contiguous()
        got = I()._permute(src, latent, chunk)[0]
        want = O.rearrange_thw_to_3d_block(qkv.permute(2, 0, 3, 1, 4)[i], latent, chunk)
        assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16))


def test_unpermute_into_token_major_layout():
    """The destination may be a [B, S, H, D] buffer viewed as [B, H, S, D], which
    makes the transpose of attention.py:140-141 free."""
    from longcat_video_amd import _capi
    latent, chunk = (4, 5, 8), (4, 4, 4)
    S = 160
    x = torch.randn(1, 3, S, 128, generator=torch.Generator().manual_seed(3)).bfloat16()
    blocked = O.rearrange_thw_to_3d_block(x, latent, chunk).cuda()
    dst = torch.zeros(1, S, 3, 128, dtype=torch.bfloat16, device="cuda")
    view = dst.permute(0, 2, 1, 3)
    lib = _capi.load()
    rc = lib.bsa_unpermute_blocks_to_thw(blocked.data_ptr(), dst.data_ptr(), _capi.strides3(view.stride()[:3]),
                                         1, 3, *latent, *chunk, 128, _capi.BSA_BF16,
                                         torch.cuda.current_stream().cuda_stream)
    _capi.check(rc)
    torch.cuda.synchronize()
    assert torch.equal(dst.cpu(), x.transpose(1, 2).contiguous())


@pytest.mark.parametrize("latent,chunk", GRIDS[:4])
def test_fused_pool_and_tile_validity(latent, chunk):
    S = int(np.prod(latent))
    bs = int(np.prod(chunk))
    x = torch.randn(1, 2, S, 128, generator=torch.Generator().manual_seed(4)).bfloat16()
    blocked, pooled, valid = I()._permute(x.cuda(), latent, chunk, want_pooled=True, want_valid=True)
    want_blocked = O.rearrange_thw_to_3d_block(x, latent, chunk)
    want_pooled = O.mean_pooling_compression(want_blocked, bs)
    # same fp32 sum up to ordering, one rounding: at most one bf16 ulp apart
    diff = (pooled.cpu().float() - want_pooled.float()).abs()
    assert torch.all(diff <= want_pooled.float().abs() * 2.0 ** -7 + 1e-6)
    assert torch.equal(pooled, I().mean_pooling_compression(blocked, bs))      # the two kernels agree bit for bit
    bits = valid.cpu().numpy().view(np.uint64)
    slot_ok = O.slot_validity(latent, chunk)
    got = ((bits[:, None] >> np.arange(64, dtype=np.uint64)[None, :]) & np.uint64(1)).astype(bool).reshape(-1)
    assert np.array_equal(got, slot_ok)


def test_pool_exact_on_representable_inputs():
    x = (torch.arange(1, 7).repeat_interleave(64).view(1, 1, 384, 1) * torch.ones(1, 2, 1, 128)).contiguous()
    for dt in (torch.bfloat16, torch.float16, torch.float32):
        got = I().mean_pooling_compression(x.to(dt).cuda(), 64)
        assert torch.equal(got.cpu(), O.mean_pooling_compression(x.to(dt), 64))
    ragged = torch.ones(1, 1, 96, 128, dtype=torch.bfloat16)
    got = I().mean_pooling_compression(ragged.cuda(), 64).cpu()
    assert torch.equal(got, O.mean_pooling_compression(ragged, 64)) and float(got[0, 0, 1, 0]) == 0.5


def test_full_size_720p_round_trip_and_checksum():
    """benchmark configuration 3 shape, all 32 heads: size-independent properties."""
    latent, chunk = (24, 45, 80), (4, 4, 4)
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(1, 32, 86400, 128, generator=g, device="cuda", dtype=torch.bfloat16)
    blocked, pooled, valid = I()._permute(x, latent, chunk, want_pooled=True, want_valid=True)
    assert blocked.shape == (1, 32, 92160, 128)
    # permutation + zero fill preserves the multiset: compare integer checksums of the bit patterns
    assert int(blocked.view(torch.int16).long().sum()) == int(x.view(torch.int16).long().sum())
    assert int((blocked.view(torch.int16) != 0).sum()) == int((x.view(torch.int16) != 0).sum())
    back = I().rearrange_3d_block_to_THW(blocked, 6, 12, 20, 4, 4, 4, 128, latent_shape=latent)
    assert torch.equal(back, x)
    # spot-check one head against the oracle
    want = O.rearrange_thw_to_3d_block(x[:, 7:8].cpu(), latent, chunk)
    assert torch.equal(blocked[:, 7:8].cpu(), want)
    assert int(valid.cpu().numpy().view(np.uint64).astype(object).sum()) > 0
    ok = torch.from_numpy(O.slot_validity(latent, chunk)).cuda()
    assert torch.all(blocked[0, 3][~ok] == 0)

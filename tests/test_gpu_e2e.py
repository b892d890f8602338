"""R8/R9 on the GPU: the whole operator through flash_attn_bsa_3d, from the
benchmark configurations at reduced head count up to the full 720p shape."""
import math

import numpy as np
import pytest
import torch

from oracle import bsa_oracle as O
from conftest import seeded_qkv

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 2e-2, 2e-3
CH = dict(chunk_3d_shape_q=[4, 4, 4], chunk_3d_shape_k=[4, 4, 4])


def I():
    from longcat_video_amd.block_sparse_attention import bsa_interface
    return bsa_interface


def check_against_oracle(q, k, v, latent_q, latent_k, sparsity, o, idx, lens, score, q_blocks, heads=None,
                         chunk=(4, 4, 4)):
    """Selection: bit-exact given the GPU's scores.  Pooled scores: one ulp from the
    oracle's.  Output: tolerance against the fp32 oracle evaluated with the
    GPU's selection, on the sampled query blocks."""
    bs = int(np.prod(chunk))
    heads = list(range(q.shape[1])) if heads is None else heads
    qh, kh, vh = q[:, heads], k[:, heads], v[:, heads]
    qp = O.rearrange_thw_to_3d_block(qh, latent_q, chunk)
    kp = O.rearrange_thw_to_3d_block(kh, latent_k, chunk)
    vp = O.rearrange_thw_to_3d_block(vh, latent_k, chunk)
    want_score = O.cal_score(O.mean_pooling_compression(qp, bs), O.mean_pooling_compression(kp, bs))
    s_gpu = score[:, heads].cpu()
    tol = 2.0 ** -6 if q.dtype != torch.float32 else 1e-5     # pooled means and the score are each one rounding
    assert torch.all((s_gpu.float() - want_score.float()).abs() <= want_score.float().abs() * tol + 1e-3)
    k_sel = O.num_selected(sparsity, s_gpu.shape[-1])
    want_idx, _ = O.select_topk(s_gpu, k_sel)
    assert torch.equal(idx[:, heads].cpu().long(), want_idx), "selection differs from the oracle on identical scores"
    assert torch.all(lens.cpu() == k_sel)
    kvalid = torch.from_numpy(O.slot_validity(latent_k, chunk))
    want_o, _ = O.gathered_attention(qp, kp, vp, want_idx, lens[:, heads].cpu(), bs, bs, 1 / math.sqrt(q.shape[-1]),
                                     key_valid=kvalid, q_blocks=q_blocks)
    got_p = O.rearrange_thw_to_3d_block(o[:, heads].cpu(), latent_q, chunk)
    qvalid = torch.from_numpy(O.slot_validity(latent_q, chunk))
    for m in q_blocks:
        rows = torch.arange(m * bs, (m + 1) * bs)[qvalid[m * bs:(m + 1) * bs]]
        d = (got_p[:, :, rows].float() - want_o[:, :, rows]).abs()
        if q.dtype == torch.float32:
            assert d.max() <= 2e-5
        else:
            assert d.max() <= MAX_ABS and d.mean() <= MEAN_ABS, (m, d.max(), d.mean())


def test_config1_fp32_plumbing():
    q, k, v = seeded_qkv(0, 1, 4, 256, 256, 128, torch.float32)
    o, idx, lens, score = I()._bsa_3d(q.cuda(), k.cuda(), v.cuda(), (4, 8, 8), (4, 8, 8), 0.5, (4, 4, 4), (4, 4, 4), True)
    want, want_idx, _, want_score = O.flash_attn_bsa_3d(q, k, v, (4, 8, 8), (4, 8, 8), 0.5, (4, 4, 4), (4, 4, 4))
    assert torch.allclose(score.cpu(), want_score, atol=1e-5)
    assert torch.equal(idx.cpu().long(), want_idx)
    assert (o.cpu() - want).abs().max() <= 2e-5
    pub = I().flash_attn_bsa_3d(q.cuda(), k.cuda(), v.cuda(), (4, 8, 8), (4, 8, 8), sparsity=0.5, **CH)
    assert torch.equal(pub, o) and pub.is_contiguous()


def test_config1_in_bf16():
    q, k, v = seeded_qkv(0, 1, 4, 256, 256, 128, torch.bfloat16)
    o, idx, lens, score = I()._bsa_3d(q.cuda(), k.cuda(), v.cuda(), (4, 8, 8), (4, 8, 8), 0.5, (4, 4, 4), (4, 4, 4), True)
    check_against_oracle(q, k, v, (4, 8, 8), (4, 8, 8), 0.5, o, idx, lens, score, q_blocks=range(4))


@pytest.mark.parametrize("latent,sparsity", [((4, 6, 5), 0.5), ((5, 9, 13), 0.75), ((8, 30, 52), 0.9375)])
def test_padded_grids(latent, sparsity):
    S = int(np.prod(latent))
    q, k, v = seeded_qkv(31, 1, 2, S, S, 128, torch.bfloat16)
    o, idx, lens, score = I()._bsa_3d(q.cuda(), k.cuda(), v.cuda(), latent, latent, sparsity, (4, 4, 4), (4, 4, 4), True)
    nb = int(np.prod(O.block_grid(latent, (4, 4, 4))))
    check_against_oracle(q, k, v, latent, latent, sparsity, o, idx, lens, score, q_blocks=sorted({0, 1, nb // 2, nb - 1}))
    assert torch.isfinite(o.float()).all()


def test_default_chunk_4x4x8():
    latent = (8, 8, 16)
    q, k, v = seeded_qkv(32, 1, 2, 1024, 1024, 128, torch.bfloat16)
    o, idx, lens, score = I()._bsa_3d(q.cuda(), k.cuda(), v.cuda(), latent, latent, 0.5, (4, 4, 8), (4, 4, 8), True)
    check_against_oracle(q, k, v, latent, latent, 0.5, o, idx, lens, score, q_blocks=range(8), chunk=(4, 4, 8))
    pub = I().flash_attn_bsa_3d(q.cuda(), k.cuda(), v.cuda(), latent, latent, sparsity=0.5)   # reference defaults
    assert torch.equal(pub, o)


@pytest.mark.parametrize("latent,chunk", [
    ((5, 6, 12), (4, 4, 8)),     # 128-slot chunks on a ragged grid: one 64-slot tile of the last layer is padding only
    ((3, 9, 20), (2, 8, 4)),     # tiles of two (h, w) planes
    ((6, 5, 36), (1, 4, 16)),    # one plane per tile, long runs along w, ragged h
    ((4, 8, 6), (4, 8, 2)),      # runs of 2 tokens: k and v go through blocked copies
    ((6, 7, 9), (4, 2, 8)),      # four planes of two runs per tile
    ((2, 40, 8), (1, 32, 4)),    # a 64-slot tile is half a plane: blocked copies again
])
def test_chunk_shapes_on_ragged_grids(latent, chunk):
    S = int(np.prod(latent))
    q, k, v = seeded_qkv(36, 1, 2, S, S, 128, torch.bfloat16)
    o, idx, lens, score = I()._bsa_3d(q.cuda(), k.cuda(), v.cuda(), latent, latent, 0.5, chunk, chunk, True)
    nb = int(np.prod(O.block_grid(latent, chunk)))
    check_against_oracle(q, k, v, latent, latent, 0.5, o, idx, lens, score, q_blocks=range(nb), chunk=chunk)
    assert torch.isfinite(o.float()).all()


@pytest.mark.parametrize("latent,chunk", [
    ((8, 16, 16), (4, 8, 8)),    # 256 tokens per chunk: the case the reference gives to its second kernel
    ((9, 10, 11), (8, 8, 4)),    # the same on a grid that is ragged in every direction
    ((8, 16, 16), (8, 8, 8)),    # 512 tokens per chunk
    ((5, 12, 20), (2, 12, 8)),   # 192 tokens: a multiple of 64 that is no power of two
])
def test_chunks_above_128_tokens(latent, chunk):
    """The reference switches to another kernel when a KV chunk holds more than 128 tokens
    (bsa_interface.py:311-313, flash_attn_bsa_varlen_mask.py:35-153: the chunk in steps of BLOCK_N keys, same
    arithmetic).  Here the same kernels take every chunk that is a multiple of 64 tokens."""
    S = int(np.prod(latent))
    q, k, v = seeded_qkv(38, 1, 2, S, S, 128, torch.bfloat16)
    o, idx, lens, score = I()._bsa_3d(q.cuda(), k.cuda(), v.cuda(), latent, latent, 0.5, chunk, chunk, True)
    nb = int(np.prod(O.block_grid(latent, chunk)))
    check_against_oracle(q, k, v, latent, latent, 0.5, o, idx, lens, score, q_blocks=range(nb), chunk=chunk)
    assert torch.isfinite(o.float()).all()
    pub = I().flash_attn_bsa_3d(q.cuda(), k.cuda(), v.cuda(), latent, latent, sparsity=0.5,
                                chunk_3d_shape_q=list(chunk), chunk_3d_shape_k=list(chunk))
    assert torch.equal(pub, o)


def test_strided_inputs_on_a_ragged_grid():
    """q, k, v as views of one [B, S, 3, H, D] projection output and o written into a [B, S, H, D]
    buffer, on a grid with padded chunks in every direction."""
    latent = (5, 9, 13)
    S = int(np.prod(latent))
    qkv = torch.randn(1, S, 3, 2, 128, generator=torch.Generator().manual_seed(37)).bfloat16().cuda()
    dq, dk, dv = qkv.permute(2, 0, 3, 1, 4).unbind(0)
    out = torch.full((1, S, 2, 128), float("nan"), dtype=torch.bfloat16, device="cuda")
    I()._bsa_3d(dq, dk, dv, latent, latent, 0.75, (4, 4, 4), (4, 4, 4), out=out.permute(0, 2, 1, 3))
    ref = I()._bsa_3d(dq.contiguous(), dk.contiguous(), dv.contiguous(), latent, latent, 0.75, (4, 4, 4), (4, 4, 4))
    assert torch.equal(out.permute(0, 2, 1, 3), ref)


def test_rectangular_query_and_key_grids():
    """Tq != Tk, as in the noise half of the cond/noise split (attention.py:132-133)."""
    lq, lk = (4, 8, 8), (8, 8, 8)
    q, _, _ = seeded_qkv(33, 1, 2, 256, 256, 128, torch.bfloat16)
    _, k, v = seeded_qkv(34, 1, 2, 512, 512, 128, torch.bfloat16)
    o, idx, lens, score = I()._bsa_3d(q.cuda(), k.cuda(), v.cuda(), lq, lk, 0.5, (4, 4, 4), (4, 4, 4), True)
    assert idx.shape == (1, 2, 4, 4) and score.shape == (1, 2, 4, 8)
    check_against_oracle(q, k, v, lq, lk, 0.5, o, idx, lens, score, q_blocks=range(4))


def test_strided_inputs_from_a_qkv_projection():
    latent = (4, 8, 8)
    qkv = torch.randn(1, 256, 3, 2, 128, generator=torch.Generator().manual_seed(35)).bfloat16()
    q, k, v = qkv.permute(2, 0, 3, 1, 4).unbind(0)
    dq, dk, dv = qkv.cuda().permute(2, 0, 3, 1, 4).unbind(0)
    o = I().flash_attn_bsa_3d(dq, dk, dv, latent, latent, sparsity=0.5, **CH)
    o2 = I().flash_attn_bsa_3d(dq.contiguous(), dk.contiguous(), dv.contiguous(), latent, latent, sparsity=0.5, **CH)
    assert torch.equal(o, o2)
    assert torch.equal(dq.cpu(), q)      # inputs are not modified


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("token_major", [False, True])
def test_the_operator_scores_equal_the_standalone_route(dtype, token_major):
    """The operator takes q's chunk means in a read-only pass of its own and k's in the pass that writes the fragment
    order; permute + pool + score through the separate entry points (bsa_interface.py:547-548, 650-652 as
    the reference runs them) must give the same score bits and the same selection, on a grid with padding on two
    axes, for head-major tensors and for the token-major views a QKV projection leaves."""
    latent, B, H = (6, 10, 13), 2, 3
    S = latent[0] * latent[1] * latent[2]
    g = torch.Generator().manual_seed(71)
    if token_major:
        qkv = torch.randn(B, S, 3, H, 128, generator=g).to(dtype).cuda()
        q, k, v = qkv.permute(2, 0, 3, 1, 4).unbind(0)
    else:
        q, k, v = (torch.randn(B, H, S, 128, generator=g).to(dtype).cuda() for _ in range(3))
    bi = I()
    o, idx, lens, score = bi._bsa_3d(q, k, v, latent, latent, 0.75, (4, 4, 4), (4, 4, 4), True)
    _, q_cmp, _ = bi._permute(q, latent, (4, 4, 4), want_pooled=True)
    _, k_cmp, _ = bi._permute(k, latent, (4, 4, 4), want_pooled=True)
    idx2, lens2, score2 = bi._score_topk(q_cmp, k_cmp, idx.shape[-1])
    assert torch.equal(score.view(torch.int16), score2.view(torch.int16))
    assert torch.equal(idx, idx2) and torch.equal(lens, lens2)


def test_480p_two_heads():
    latent = (24, 30, 52)
    q, k, v = seeded_qkv(1, 1, 2, 37440, 37440, 128, torch.bfloat16)
    o, idx, lens, score = I()._bsa_3d(q.cuda(), k.cuda(), v.cuda(), latent, latent, 0.9375, (4, 4, 4), (4, 4, 4), True)
    assert idx.shape == (1, 2, 624, 39)
    check_against_oracle(q, k, v, latent, latent, 0.9375, o, idx, lens, score, q_blocks=[0, 12, 300, 611, 623])


def test_long_video_continuation_two_heads():
    """benchmark configuration 4 geometry with 2 heads: grid 48x30x52, the first 12 latent frames are
    conditioning tokens.  Two operator calls as in attention.py:124-135: conditioning queries
    against conditioning keys (312 blocks, 39 kept), noise queries against all keys
    (936 x 1248 blocks, 156 kept)."""
    T, Hh, W, cond = 48, 30, 52, 12
    S, n = T * Hh * W, cond * Hh * W
    q, k, v = seeded_qkv(3, 1, 2, S, S, 128, torch.bfloat16)
    dq, dk, dv = q.cuda(), k.cuda(), v.cuda()
    out = torch.empty(1, S, 2, 128, dtype=torch.bfloat16, device="cuda").permute(0, 2, 1, 3)
    o_c, idx_c, lens_c, score_c = I()._bsa_3d(dq[:, :, :n], dk[:, :, :n], dv[:, :, :n], (cond, Hh, W), (cond, Hh, W),
                                              0.875, (4, 4, 4), (4, 4, 4), True, out=out[:, :, :n])
    o_n, idx_n, lens_n, score_n = I()._bsa_3d(dq[:, :, n:], dk, dv, (T - cond, Hh, W), (T, Hh, W),
                                              0.875, (4, 4, 4), (4, 4, 4), True, out=out[:, :, n:])
    assert idx_c.shape == (1, 2, 312, 39) and idx_n.shape == (1, 2, 936, 156)
    check_against_oracle(q[:, :, :n], k[:, :, :n], v[:, :, :n], (cond, Hh, W), (cond, Hh, W), 0.875,
                         out[:, :, :n], idx_c, lens_c, score_c, q_blocks=[0, 155, 311])
    check_against_oracle(q[:, :, n:], k, v, (T - cond, Hh, W), (T, Hh, W), 0.875,
                         out[:, :, n:], idx_n, lens_n, score_n, q_blocks=[0, 500, 935])


def test_720p_full_shape_sampled():
    """benchmark configuration 3 at full size (32 heads, 86 400 tokens, RMS-normalised q/k,
    density 1/16): two heads are checked against the oracle on sampled query
    blocks; all heads for finiteness, determinism and row-stochastic bounds."""
    latent = (24, 45, 80)
    g = torch.Generator(device="cuda").manual_seed(2)
    q = torch.randn(1, 32, 86400, 128, generator=g, device="cuda")
    k = torch.randn(1, 32, 86400, 128, generator=g, device="cuda")
    v = torch.randn(1, 32, 86400, 128, generator=g, device="cuda").bfloat16()
    q = (q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + 1e-6)).bfloat16()
    k = (k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + 1e-6)).bfloat16()
    o, idx, lens, score = I()._bsa_3d(q, k, v, latent, latent, 0.9375, (4, 4, 4), (4, 4, 4), True)
    assert idx.shape == (1, 32, 1440, 90) and torch.all(lens == 90)
    assert torch.isfinite(o.float()).all()
    # a convex combination of value rows cannot leave their range
    assert float(o.float().abs().max()) <= float(v.float().abs().max())
    heads = [5, 31]
    check_against_oracle(q.cpu(), k.cpu(), v.cpu(), latent, latent, 0.9375, o, idx, lens, score,
                         q_blocks=[0, 19, 700, 1439], heads=heads)
    o2 = I().flash_attn_bsa_3d(q, k, v, latent, latent, sparsity=0.9375, **CH)
    assert torch.equal(o, o2)


def gpu_qkv(seed, heads, tokens):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return tuple(torch.randn(1, heads, tokens, 128, generator=g, device="cuda").bfloat16() for _ in range(3))


def all_heads_properties(o, v_rows):
    assert torch.isfinite(o.float()).all()
    # a convex combination of value rows cannot leave their range, in any head
    assert bool((o.float().abs().amax(dim=(0, 2, 3)) <= v_rows.float().abs().amax(dim=(0, 2, 3))).all())


def test_480p_all_heads():
    """benchmark configuration 2 at full size (32 heads, 37 440 tokens, 624 blocks, 39 kept): 19 968 work items are
    19 full rounds of 1 024 and one of 512, and a head's 624 items never fill a round, so every round crosses a head
    boundary.  All heads: finiteness, range, determinism; heads on both sides of round boundaries: the oracle on
    sampled query blocks (the last block of a head and the first of the next lie in one round)."""
    latent = (24, 30, 52)
    q, k, v = gpu_qkv(1, 32, 37440)
    o, idx, lens, score = I()._bsa_3d(q, k, v, latent, latent, 0.9375, (4, 4, 4), (4, 4, 4), True)
    assert idx.shape == (1, 32, 624, 39) and torch.all(lens == 39)
    all_heads_properties(o, v)
    # item 1023 | 1024 is block 399 | 400 of head 1; item 19 455 | 19 456 (the half round begins) is block 111 | 112 of head 31
    check_against_oracle(q.cpu(), k.cpu(), v.cpu(), latent, latent, 0.9375, o, idx, lens, score,
                         q_blocks=[0, 111, 112, 399, 400, 623], heads=[0, 1, 31])
    assert torch.equal(o, I().flash_attn_bsa_3d(q, k, v, latent, latent, sparsity=0.9375, **CH))


def test_long_video_continuation_all_heads():
    """benchmark configuration 4 at full size (32 heads, grid 48x30x52, 12 conditioning frames): both operator calls of
    attention.py:124-135 into one output buffer - 32 x 312 work items of 39 tiles, then 32 x 936 of 156."""
    T, Hh, W, cond = 48, 30, 52, 12
    S, n = T * Hh * W, cond * Hh * W
    q, k, v = gpu_qkv(3, 32, S)
    out = torch.empty(1, S, 32, 128, dtype=torch.bfloat16, device="cuda").permute(0, 2, 1, 3)
    bi = I()
    call = lambda: (bi._bsa_3d(q[:, :, :n], k[:, :, :n], v[:, :, :n], (cond, Hh, W), (cond, Hh, W), 0.875, (4, 4, 4), (4, 4, 4), True,
                               out=out[:, :, :n]),
                    bi._bsa_3d(q[:, :, n:], k, v, (T - cond, Hh, W), (T, Hh, W), 0.875, (4, 4, 4), (4, 4, 4), True, out=out[:, :, n:]))
    (_, idx_c, lens_c, score_c), (_, idx_n, lens_n, score_n) = call()
    assert idx_c.shape == (1, 32, 312, 39) and idx_n.shape == (1, 32, 936, 156)
    all_heads_properties(out, v)
    first = out.clone()
    heads = [0, 3, 31]               # item 1023 | 1024 of the conditioning call: block 87 | 88 of head 3; of the noise call: block 87 | 88 of head 1
    qc, kc, vc = q.cpu(), k.cpu(), v.cpu()
    check_against_oracle(qc[:, :, :n], kc[:, :, :n], vc[:, :, :n], (cond, Hh, W), (cond, Hh, W), 0.875,
                         out[:, :, :n], idx_c, lens_c, score_c, q_blocks=[0, 87, 88, 311], heads=heads)
    check_against_oracle(qc[:, :, n:], kc, vc, (T - cond, Hh, W), (T, Hh, W), 0.875,
                         out[:, :, n:], idx_n, lens_n, score_n, q_blocks=[0, 87, 88, 935], heads=[1, 31])
    call()
    assert torch.equal(out, first)


@pytest.mark.parametrize("sparsity", [None, 0.75])
def test_operator_with_cdf_selection(sparsity):
    """flash_attn_bsa_3d with cdf_threshold (bsa_interface.py:268-277, 555): rows keep different numbers of
    blocks; the output is judged against the oracle evaluated with the GPU's own selection."""
    latent = (5, 8, 12)
    S = int(np.prod(latent))
    q, k, v = seeded_qkv(51, 1, 2, S, S, 128, torch.bfloat16)
    q = q * 3                                               # sharper pooled scores: a wider spread of list lengths
    o, idx, lens, score = I()._bsa_3d(q.cuda(), k.cuda(), v.cuda(), latent, latent, sparsity, (4, 4, 4), (4, 4, 4), True,
                                      cdf_threshold=0.6)
    nb = int(np.prod(O.block_grid(latent, (4, 4, 4))))
    assert idx.shape == (1, 2, nb, nb)
    k_min = 0 if sparsity is None else O.num_selected(sparsity, nb)
    want_idx, want_lens, cdf = O.select_cdf(score.cpu(), 0.6, 1 / math.sqrt(128), k_min=k_min)
    near = (cdf - float(np.float32(0.6))).abs().min(-1).values < 1e-5
    assert torch.equal(lens.cpu().long()[~near], want_lens.long()[~near])
    assert int(lens.min()) >= k_min and int(lens.min()) < int(lens.max())
    qp = O.rearrange_thw_to_3d_block(q, latent, (4, 4, 4))
    kp = O.rearrange_thw_to_3d_block(k, latent, (4, 4, 4))
    vp = O.rearrange_thw_to_3d_block(v, latent, (4, 4, 4))
    kvalid = torch.from_numpy(O.slot_validity(latent, (4, 4, 4)))
    want_o, _ = O.gathered_attention(qp, kp, vp, idx.cpu().long().clamp(min=0), lens.cpu(), 64, 64, 1 / math.sqrt(128),
                                     key_valid=kvalid, q_blocks=range(nb))
    got_p = O.rearrange_thw_to_3d_block(o.cpu(), latent, (4, 4, 4))
    qvalid = torch.from_numpy(O.slot_validity(latent, (4, 4, 4)))
    d = (got_p[:, :, qvalid].float() - want_o[:, :, qvalid]).abs()
    assert d.max() <= MAX_ABS and d.mean() <= MEAN_ABS
    pub = I().flash_attn_bsa_3d(q.cuda(), k.cuda(), v.cuda(), latent, latent, sparsity=sparsity, cdf_threshold=0.6, **CH)
    assert torch.equal(pub, o)


def test_operator_with_cdf_rows_of_more_than_1024_blocks():
    """A grid of 1 152 blocks and a threshold that keeps nearly all of them: rows of more than 1 024 blocks go
    through selection, visiting order and the attention kernel at their full length (the reference keeps however
    many blocks fall under the threshold, bsa_interface.py:233-243)."""
    latent = (36, 32, 64)
    S = int(np.prod(latent))
    q, k, v = seeded_qkv(53, 1, 1, S, S, 128, torch.bfloat16)
    o, idx, lens, score = I()._bsa_3d(q.cuda(), k.cuda(), v.cuda(), latent, latent, None, (4, 4, 4), (4, 4, 4), True,
                                      cdf_threshold=0.97)
    nb = 1152
    assert idx.shape == (1, 1, nb, nb) and int(lens.max()) > 1024
    want_idx, want_lens, cdf = O.select_cdf(score.cpu(), 0.97, 1 / math.sqrt(128))
    near = (cdf - float(np.float32(0.97))).abs().min(-1).values < 1e-5
    assert torch.equal(lens.cpu().long()[~near], want_lens.long()[~near])
    long_rows = torch.nonzero(lens[0, 0].cpu() > 1024).flatten().tolist()
    sample = long_rows[:2] + [long_rows[-1], 0]
    qp, kp, vp = (O.rearrange_thw_to_3d_block(t, latent, (4, 4, 4)) for t in (q, k, v))
    want_o, _ = O.gathered_attention(qp, kp, vp, idx.cpu().long().clamp(min=0), lens.cpu(), 64, 64, 1 / math.sqrt(128),
                                     q_blocks=sample)
    got_p = O.rearrange_thw_to_3d_block(o.cpu(), latent, (4, 4, 4))
    for m in sample:
        d = (got_p[:, :, m * 64:(m + 1) * 64].float() - want_o[:, :, m * 64:(m + 1) * 64]).abs()
        assert d.max() <= MAX_ABS and d.mean() <= MEAN_ABS, (m, float(d.max()))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_two_batches_on_a_ragged_grid(dtype):
    """Batch and head strides of the direct (T,H,W)-order path: B = 2, three heads, every axis ragged."""
    latent = (5, 9, 13)
    S = int(np.prod(latent))
    q, k, v = seeded_qkv(52, 2, 3, S, S, 128, dtype)
    o, idx, lens, score = I()._bsa_3d(q.cuda(), k.cuda(), v.cuda(), latent, latent, 0.75, (4, 4, 4), (4, 4, 4), True)
    nb = int(np.prod(O.block_grid(latent, (4, 4, 4))))
    for b in range(2):
        check_against_oracle(q[b:b + 1], k[b:b + 1], v[b:b + 1], latent, latent, 0.75, o[b:b + 1], idx[b:b + 1],
                             lens[b:b + 1], score[b:b + 1], q_blocks=[0, nb // 3, nb - 1])
    # each batch entry on its own gives the same bits
    o0 = I()._bsa_3d(q[1:].cuda(), k[1:].cuda(), v[1:].cuda(), latent, latent, 0.75, (4, 4, 4), (4, 4, 4))
    assert torch.equal(o0, o[1:])


@pytest.mark.parametrize("cdf", [None, 0.6])
def test_operator_replays_from_a_hip_graph(cdf):
    """The operator makes no allocation, host wait or memset of its own, so a captured stream replays it.  The
    graph is replayed three times with eager work and synchronisations in between and new input values each
    time; every replay must equal the eager result on the same values bit for bit."""
    latent = (5, 9, 13)                                   # ragged in every axis: edge copies, masks, tables
    q, k, v = (t.cuda() for t in seeded_qkv(40, 1, 2, 5 * 9 * 13, 5 * 9 * 13, 128, torch.bfloat16))
    sq, sk, sv = q.clone(), k.clone(), v.clone()          # static inputs of the graph
    run = lambda: I().flash_attn_bsa_3d(sq, sk, sv, latent, latent, sparsity=0.5, cdf_threshold=cdf, **CH)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()                                             # warm-up outside the capture (library handles, caches)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = run()
    for step in range(3):
        scale = 1.0 + 0.5 * step
        sq.copy_(q * scale); sk.copy_(k.roll(step, dims=2)); sv.copy_(v * (1 - 0.25 * step))
        g.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = run()                                      # eager, same values
        torch.cuda.synchronize()
        assert torch.equal(got, want), "replay %d differs from the eager result" % step
        assert got.abs().sum() > 0


def _random_case(rnd):
    chunks = [(4, 4, 4), (4, 4, 8), (2, 8, 4), (1, 4, 16), (4, 2, 8), (2, 4, 8), (8, 2, 4), (1, 8, 8), (4, 8, 2), (2, 2, 16)]
    chunk = rnd.choice(chunks)
    nb = [rnd.randint(1, 3), rnd.randint(1, 5), rnd.randint(1, 5)]
    lq = tuple(max(1, c * b - rnd.randint(0, c - 1)) for c, b in zip(chunk, nb))        # ragged in any axis
    rect = rnd.random() < 0.25
    lk = (lq[0] + rnd.randint(1, chunk[0] * 2), lq[1], lq[2]) if rect else lq            # more key frames than query frames
    return dict(chunk=chunk, lq=lq, lk=lk, H=rnd.choice([1, 2, 3]), B=rnd.choice([1, 1, 2]),
                dtype=rnd.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32]),
                sparsity=rnd.choice([0.0, 0.25, 0.5, 0.75, 0.9]), strided=(not rect) and rnd.random() < 0.3)


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes_against_the_oracle(seed):
    """Seeded random draws over chunk shapes, ragged and rectangular grids, batch and head counts, storage types,
    sparsities and strided views of one projection output; every query block of every case is checked."""
    import random
    c = _random_case(random.Random(7000 + seed))
    Sq, Sk = int(np.prod(c["lq"])), int(np.prod(c["lk"]))
    g = torch.Generator().manual_seed(7000 + seed)
    if c["strided"]:
        qkv = torch.randn(c["B"], Sq, 3, c["H"], 128, generator=g).to(c["dtype"])
        q, k, v = qkv.permute(2, 0, 3, 1, 4).unbind(0)
        gq, gk, gv = qkv.cuda().permute(2, 0, 3, 1, 4).unbind(0)
    else:
        q, k, v = (torch.randn(c["B"], c["H"], s, 128, generator=g).to(c["dtype"]) for s in (Sq, Sk, Sk))
        gq, gk, gv = q.cuda(), k.cuda(), v.cuda()
    o, idx, lens, score = I()._bsa_3d(gq, gk, gv, c["lq"], c["lk"], c["sparsity"], c["chunk"], c["chunk"], True)
    nbq = int(np.prod(O.block_grid(c["lq"], c["chunk"])))
    for b in range(c["B"]):
        check_against_oracle(q[b:b + 1], k[b:b + 1], v[b:b + 1], c["lq"], c["lk"], c["sparsity"], o[b:b + 1], idx[b:b + 1],
                             lens[b:b + 1], score[b:b + 1], q_blocks=range(nbq), chunk=c["chunk"])
    assert torch.isfinite(o.float()).all(), c


@pytest.mark.parametrize("spread", ["wide", "narrow"])
def test_cdf_lists_of_unequal_length_schedule(spread):
    """With the CDF rule the operator enqueues two schedules of the attention kernel (rounds of equal work items,
    and one launch whose workgroups draw the items longest list first) and picks one on the device from the list
    lengths.  Whatever it picks, the output must equal, bit for bit, what the kernel gives in plain rounds on the
    same lists in the same visiting order (ThwAttention), here with more work items (640) than one round holds: 'wide' has lists from a few
    blocks to most of them, 'narrow' lists of nearly equal length."""
    latent, heads = (8, 32, 32), 5
    S = int(np.prod(latent))
    g = torch.Generator().manual_seed(52)
    q = torch.randn(1, heads, S, 128, generator=g)
    k = torch.randn(1, heads, S, 128, generator=g)
    v = torch.randn(1, heads, S, 128, generator=g).bfloat16()
    if spread == "wide":
        # chunks whose queries all point the same way (peaked pooled scores, short lists) next to chunks of
        # independent queries (flat scores, long lists)
        pos = torch.arange(S)
        chunk_id = ((pos // (32 * 32)) // 4) * 64 + (((pos // 32) % 32) // 4) * 8 + (pos % 32) // 4
        peaked = (chunk_id % 10 != 0)      # nine short lists for every long one: the draw-from-a-counter schedule wins
        common = torch.randn(1, heads, S // 64, 128, generator=g).repeat_interleave(64, dim=2)   # one direction per 64 tokens
        chunk_dir = torch.zeros_like(q)
        order = torch.argsort(chunk_id, stable=True)                 # tokens grouped by chunk: 64 each
        chunk_dir[:, :, order] = common
        q[:, :, peaked] = 3 * chunk_dir[:, :, peaked] + 0.1 * q[:, :, peaked]
        k[:, :, peaked] = 3 * chunk_dir[:, :, peaked] + 0.1 * k[:, :, peaked]
    q, k = q.bfloat16(), k.bfloat16()
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    o, idx, lens, score = I()._bsa_3d(qg, kg, vg, latent, latent, None, (4, 4, 4), (4, 4, 4), True, cdf_threshold=0.5)
    lens_c = lens.cpu()
    if spread == "wide":
        assert int(lens_c.max()) > 4 * max(int(lens_c.min()), 1)
    else:
        assert int(lens_c.max()) <= 2 * max(int(lens_c.min()), 1)
    big = idx.shape[-1] + 1
    asc = torch.where(idx < 0, torch.full_like(idx, big), idx).sort(dim=-1).values
    asc = torch.where(asc == big, torch.zeros_like(asc), asc)
    asc = I().visit_order(asc.int(), lens, int(np.prod(O.block_grid(latent, (4, 4, 4)))))      # the operator's visiting order
    rounds = I().ThwAttention(kg, vg, latent, latent, (4, 4, 4), (4, 4, 4))(qg, asc, lens)
    assert torch.equal(o, rounds)
    # the same choice of schedule for a caller's own lists
    either = I().ThwAttention(kg, vg, latent, latent, (4, 4, 4), (4, 4, 4), unequal_lengths=True)(qg, asc, lens)
    assert torch.equal(either, rounds)
    # and both agree with the oracle on a few query blocks of every head
    qp, kp, vp = (O.rearrange_thw_to_3d_block(t, latent, (4, 4, 4)) for t in (q, k, v))
    blocks = [0, 37, 127]
    want_o, _ = O.gathered_attention(qp, kp, vp, asc.cpu().long(), lens_c, 64, 64, 1 / math.sqrt(128), q_blocks=blocks)
    got_p = O.rearrange_thw_to_3d_block(o.cpu(), latent, (4, 4, 4))
    for m in blocks:
        d = (got_p[:, :, 64 * m:64 * m + 64].float() - want_o[:, :, 64 * m:64 * m + 64]).abs()
        assert d.max() <= MAX_ABS and d.mean() <= MEAN_ABS


def test_keys_beyond_one_buffer_span():
    """6 batches x 32 heads at the 720p grid: K in fragment order is 4.5 GB, more than the 4 GB one buffer resource of the
    attention kernel spans, so the launches are cut at head boundaries and each addresses K and V from its own first
    head.  The last batch must come out as when it is given alone (another kernel variant: the tolerance between two
    summation orders), and equal to the oracle on sampled blocks."""
    latent = (24, 45, 80)
    B, H, S = 6, 32, 86400
    g = torch.Generator(device="cuda").manual_seed(11)
    q, k, v = (torch.randn(B, H, S, 128, generator=g, device="cuda").bfloat16() for _ in range(3))
    bi = I()
    o = bi.flash_attn_bsa_3d(q, k, v, latent, latent, sparsity=0.9375, **CH)
    assert torch.isfinite(o.float()).all()
    for b in (0, B - 1):
        one, idx, lens, score = bi._bsa_3d(q[b:b + 1], k[b:b + 1], v[b:b + 1], latent, latent, 0.9375, (4, 4, 4), (4, 4, 4), True)
        d = (o[b:b + 1].float() - one.float()).abs()
        assert float(d.max()) <= 1.6e-2 and float(d.mean()) <= 1e-3, (b, float(d.max()), float(d.mean()))
    check_against_oracle(q[B - 1:].cpu(), k[B - 1:].cpu(), v[B - 1:].cpu(), latent, latent, 0.9375, o[B - 1:], idx, lens, score,
                         q_blocks=[0, 733, 1439], heads=[0, 31])


def test_query_rows_too_far_apart_for_32_bit_offsets():
    """q as a view whose token rows lie 1.2 MB apart (4.9 GB from first to last): the LDS DMA that prepares the next
    work item's Q rows cannot address them, so every item fetches its own; the result must not change."""
    latent = (4, 32, 32)
    S = 4096
    g = torch.Generator(device="cuda").manual_seed(12)
    qc, k, v = (torch.randn(1, 1, S, 128, generator=g, device="cuda").bfloat16() for _ in range(3))
    wide = torch.empty(1, 1, S, 600000, dtype=torch.bfloat16, device="cuda")        # 4096 rows x 1.2 MB
    q = wide[..., :128]
    q.copy_(qc)
    assert q.stride(2) * 2 * S > 2 ** 32 and not q.is_contiguous()
    bi = I()
    got = bi.flash_attn_bsa_3d(q, k, v, latent, latent, sparsity=0.75, **CH)
    want = bi.flash_attn_bsa_3d(qc, k, v, latent, latent, sparsity=0.75, **CH)
    assert torch.equal(got, want)

"""Pins the oracle's attention (R6, R8-R10) through special cases that reduce to
library routines, through invariants, and through agreement between its two
independent formulations."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import bsa_oracle as O
from conftest import seeded_qkv


def full_lists(B, H, nbq, nbk):
    idx = torch.arange(nbk).view(1, 1, 1, nbk).expand(B, H, nbq, nbk).contiguous()
    lens = torch.full((B, H, nbq), nbk, dtype=torch.int32)
    return idx, lens


def test_dense_special_case_equals_sdpa():
    q, k, v = seeded_qkv(10, 1, 2, 128, 192, 128, torch.float32)
    idx, lens = full_lists(1, 2, 2, 3)
    mask = O.block_mask_from_indices(idx, lens, 3)
    scale = 1 / math.sqrt(128)
    o, lse = O.masked_dense_attention(q, k, v, mask, 64, 64, scale)
    want = F.scaled_dot_product_attention(q, k, v, scale=scale)
    assert torch.allclose(o, want, atol=2e-6, rtol=1e-5)
    want_lse = torch.logsumexp(torch.einsum("bhmd,bhnd->bhmn", q, k) * scale, -1)
    assert torch.allclose(lse, want_lse, atol=1e-5)
    o2, lse2 = O.gathered_attention(q, k, v, idx, lens, 64, 64, scale)
    assert torch.allclose(o2, want, atol=2e-6, rtol=1e-5) and torch.allclose(lse2, want_lse, atol=1e-5)


def test_single_block_is_a_plain_softmax_over_its_keys():
    q, k, v = seeded_qkv(11, 1, 1, 64, 256, 128, torch.float32)
    idx = torch.tensor([2]).view(1, 1, 1, 1)
    lens = torch.ones(1, 1, 1, dtype=torch.int32)
    scale = 0.3
    o, _ = O.masked_dense_attention(q, k, v, O.block_mask_from_indices(idx, lens, 4), 64, 64, scale)
    ks, vs = k[0, 0, 128:192], v[0, 0, 128:192]
    want = torch.softmax(q[0, 0] @ ks.t() * scale, -1) @ vs
    assert torch.allclose(o[0, 0], want, atol=2e-6, rtol=1e-5)


@pytest.mark.parametrize("dtype,atol", [(torch.float32, 5e-6), (torch.bfloat16, 1.6e-2)])
def test_blockwise_restatement_agrees_with_masked_dense(dtype, atol):
    q, k, v = seeded_qkv(12, 1, 2, 128, 320, 128, dtype)
    g = torch.Generator().manual_seed(12)
    idx = torch.stack([torch.randperm(5, generator=g)[:3] for _ in range(4)]).view(1, 2, 2, 3)
    lens = torch.tensor([[[3, 2], [1, 3]]], dtype=torch.int32)
    scale = 1 / math.sqrt(128)
    o_b, lse_b = O.blockwise_attention(q, k, v, idx, lens, 64, 64, scale)
    o_d, lse_d = O.masked_dense_attention(q, k, v, O.block_mask_from_indices(idx, lens, 5), 64, 64, scale)
    assert o_b.dtype == dtype
    assert (o_b.float() - o_d).abs().max() <= atol
    assert torch.allclose(lse_b, lse_d, atol=1e-4)
    o_g, lse_g = O.gathered_attention(q, k, v, idx, lens, 64, 64, scale)
    assert torch.allclose(o_g, o_d, atol=5e-6) and torch.allclose(lse_g, lse_d, atol=1e-5)


def test_empty_list_gives_zero_output_and_minus_inf():
    q, k, v = seeded_qkv(13, 1, 1, 64, 64, 128, torch.float32)
    idx = torch.zeros(1, 1, 1, 1, dtype=torch.int64)
    lens = torch.zeros(1, 1, 1, dtype=torch.int32)
    for fn in (lambda: O.blockwise_attention(q, k, v, idx, lens, 64, 64, 0.1),
               lambda: O.masked_dense_attention(q, k, v, O.block_mask_from_indices(idx, lens, 1), 64, 64, 0.1)):
        o, lse = fn()
        assert torch.all(o == 0) and torch.all(torch.isinf(lse) & (lse < 0))


def test_lse_merge_identity_and_order_invariance():
    q, k, v = seeded_qkv(14, 1, 1, 64, 384, 128, torch.float32)
    lst = [4, 0, 3, 5]
    lens_n = lambda n: torch.full((1, 1, 1), n, dtype=torch.int32)
    t = lambda l: torch.tensor(l).view(1, 1, 1, -1)
    scale = 1 / math.sqrt(128)
    o, lse = O.blockwise_attention(q, k, v, t(lst), lens_n(4), 64, 64, scale)
    oa, la = O.blockwise_attention(q, k, v, t(lst[:2]), lens_n(2), 64, 64, scale)
    ob, lb = O.blockwise_attention(q, k, v, t(lst[2:]), lens_n(2), 64, 64, scale)
    om, lm = O.merge_partial_attention(oa, la, ob, lb)
    assert torch.allclose(om, o, atol=2e-6) and torch.allclose(lm, lse, atol=1e-5)
    o_rev, lse_rev = O.blockwise_attention(q, k, v, t(lst[::-1]), lens_n(4), 64, 64, scale)
    assert torch.allclose(o_rev, o, atol=2e-6) and torch.allclose(lse_rev, lse, atol=1e-5)


def test_padded_keys_are_ignored():
    q, k, v = seeded_qkv(15, 1, 1, 64, 128, 128, torch.float32)
    valid = torch.ones(128, dtype=torch.bool)
    valid[70:] = False
    idx, lens = full_lists(1, 1, 1, 2)
    scale = 0.2
    o, lse = O.blockwise_attention(q, k, v, idx, lens, 64, 64, scale, key_valid=valid)
    want = torch.softmax(q[0, 0] @ k[0, 0, :70].t() * scale, -1) @ v[0, 0, :70]
    assert torch.allclose(o[0, 0], want, atol=2e-6)
    o2, _ = O.masked_dense_attention(q, k, v, O.block_mask_from_indices(idx, lens, 2), 64, 64, scale, key_valid=valid)
    assert torch.allclose(o2[0, 0], want, atol=2e-6)


def test_config1_end_to_end_on_cpu():
    """benchmark configuration 1: B=1, 4 heads, D=128, grid 4x8x8, chunk 4x4x4, top-2 of 4, fp32."""
    q, k, v = seeded_qkv(0, 1, 4, 256, 256, 128, torch.float32)
    out, idx, lens, score = O.flash_attn_bsa_3d(q, k, v, (4, 8, 8), (4, 8, 8), sparsity=0.5,
                                                chunk_3d_shape_q=(4, 4, 4), chunk_3d_shape_k=(4, 4, 4))
    assert out.shape == (1, 4, 256, 128) and idx.shape == (1, 4, 4, 2) and torch.all(lens == 2)
    # independent evaluation: token-level mask in THW order, one dense softmax
    pm = torch.from_numpy(O.permute_index_map((4, 8, 8), (4, 4, 4)))
    blk_of_token = torch.empty(256, dtype=torch.long)
    blk_of_token[pm] = torch.arange(256) // 64
    bmask = O.block_mask_from_indices(idx, lens, 4)
    for h in range(4):
        tok_mask = bmask[0, h][blk_of_token][:, blk_of_token]
        logits = (q[0, h] @ k[0, h].t()) / math.sqrt(128)
        want = torch.softmax(logits.masked_fill(~tok_mask, -math.inf), -1) @ v[0, h]
        assert torch.allclose(out[0, h], want, atol=5e-6)


def test_padded_grid_end_to_end_matches_token_level_mask():
    latent, chunk = (4, 6, 5), (4, 4, 4)          # H and W ragged: 2x2 blocks of 64 slots
    S = 4 * 6 * 5
    q, k, v = seeded_qkv(16, 1, 2, S, S, 128, torch.float32)
    out, idx, lens, _ = O.flash_attn_bsa_3d(q, k, v, latent, latent, sparsity=0.5,
                                            chunk_3d_shape_q=chunk, chunk_3d_shape_k=chunk)
    pm = O.permute_index_map(latent, chunk)
    blk_of_token = torch.empty(S, dtype=torch.long)
    real = pm >= 0
    blk_of_token[torch.from_numpy(pm[real])] = torch.from_numpy(np.nonzero(real)[0] // 64)
    bmask = O.block_mask_from_indices(idx, lens, 4)
    for h in range(2):
        tok_mask = bmask[0, h][blk_of_token][:, blk_of_token]
        logits = (q[0, h] @ k[0, h].t()) / math.sqrt(128)
        want = torch.softmax(logits.masked_fill(~tok_mask, -math.inf), -1) @ v[0, h]
        assert torch.allclose(out[0, h], want, atol=5e-6)


def test_cond_noise_split_composition():
    T, Hh, W, c = 8, 4, 4, 4
    S = T * Hh * W
    q, k, v = seeded_qkv(17, 1, 1, S, S, 128, torch.float32)
    prm = dict(sparsity=0.5, chunk_3d_shape_q=(4, 4, 4), chunk_3d_shape_k=(4, 4, 4))
    out = O.cond_noise_split_attention(q, k, v, (T, Hh, W), c, **prm)
    n = c * Hh * W
    # conditioning rows never see noise keys: perturbing noise k/v leaves them unchanged
    k2, v2 = k.clone(), v.clone()
    k2[:, :, n:] += 1.0
    v2[:, :, n:] -= 2.0
    out2 = O.cond_noise_split_attention(q, k2, v2, (T, Hh, W), c, **prm)
    assert torch.equal(out[:, :, :n], out2[:, :, :n]) and not torch.equal(out[:, :, n:], out2[:, :, n:])
    want_noise, *_ = O.flash_attn_bsa_3d(q[:, :, n:], k, v, (T - c, Hh, W), (T, Hh, W), **prm)
    assert torch.equal(out[:, :, n:], want_noise)

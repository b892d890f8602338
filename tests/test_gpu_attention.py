"""R5/R6 on the GPU: the block-sparse flash-attention kernel against the oracle.

Tolerances (bf16 / fp16 outputs vs the fp32 masked-dense oracle): max-abs 2e-2,
mean-abs 2e-3; fp32 kernel: 2e-5.  lse: 2e-3 absolute."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import bsa_oracle as O
from conftest import seeded_qkv

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 2e-2, 2e-3


def I():
    from longcat_video_amd.block_sparse_attention import bsa_interface
    return bsa_interface


KERNEL = {"name": None}


@pytest.fixture(autouse=True, params=["fragment", "lds"])
def attention_kernel(request):
    """Every test that goes through run() is made with both attention kernels of the blocked-order boundary: the
    operator's fragment-order kernel (bsa_fwd_fragment) and the LDS-tiled one (bsa_fwd).  fp32 has one kernel."""
    KERNEL["name"] = request.param
    yield request.param
    KERNEL["name"] = None


def run(q, k, v, idx, lens, bs_q=64, bs_k=64, scale=None, valid_bits=None):
    scale = 1 / math.sqrt(q.shape[-1]) if scale is None else scale
    tv = None if valid_bits is None else torch.from_numpy(valid_bits.view(np.int64)).cuda()
    kern = None if q.dtype == torch.float32 else KERNEL["name"]
    o, lse = I().attn_fwd_bsa_varlen(q.cuda(), k.cuda(), v.cuda(), scale, idx.cuda(), lens.cuda(), bs_q, bs_k,
                                     tile_valid=tv, kernel=kern)
    torch.cuda.synchronize()
    return o.cpu(), lse.cpu()


def close(o, want, dtype):
    d = (o.float() - want).abs()
    if dtype == torch.float32:
        assert d.max() <= 2e-5, d.max()
    else:
        assert d.max() <= MAX_ABS and d.mean() <= MEAN_ABS, (d.max(), d.mean())


def random_lists(seed, B, H, nbq, nbk, k_sel):
    g = torch.Generator().manual_seed(seed)
    idx = torch.stack([torch.randperm(nbk, generator=g)[:k_sel] for _ in range(B * H * nbq)]).view(B, H, nbq, k_sel)
    return idx, torch.full((B, H, nbq), k_sel, dtype=torch.int32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_small_random_lists(dtype):
    q, k, v = seeded_qkv(20, 1, 3, 192, 448, 128, dtype)
    idx, lens = random_lists(20, 1, 3, 3, 7, 4)
    o, lse = run(q, k, v, idx, lens)
    assert o.dtype == dtype
    want, want_lse = O.masked_dense_attention(q, k, v, O.block_mask_from_indices(idx, lens, 7), 64, 64, 1 / math.sqrt(128))
    close(o, want, dtype)
    assert torch.allclose(lse, want_lse, atol=2e-3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_matches_the_step_by_step_kernel_restatement(dtype):
    q, k, v = seeded_qkv(21, 2, 2, 128, 256, 128, dtype)
    idx, lens = random_lists(21, 2, 2, 2, 4, 3)
    o, lse = run(q, k, v, idx, lens)
    want, want_lse = O.blockwise_attention(q, k, v, idx, lens, 64, 64, 1 / math.sqrt(128))
    d = (o.float() - want.float()).abs()
    assert d.max() <= (2e-5 if dtype == torch.float32 else 1.6e-2)     # at most a couple of bf16 ulps at |o| <= 2
    assert torch.allclose(lse, want_lse, atol=2e-3)


def test_dense_special_case_equals_sdpa():
    q, k, v = seeded_qkv(22, 1, 2, 256, 256, 128, torch.bfloat16)
    idx = torch.arange(4).view(1, 1, 1, 4).expand(1, 2, 4, 4).contiguous()
    lens = torch.full((1, 2, 4), 4, dtype=torch.int32)
    o, _ = run(q, k, v, idx, lens)
    want = F.scaled_dot_product_attention(q.float(), k.float(), v.float())
    close(o, want, torch.bfloat16)


def test_variable_lengths_and_empty_rows():
    q, k, v = seeded_qkv(23, 1, 2, 256, 384, 128, torch.bfloat16)
    idx, _ = random_lists(23, 1, 2, 4, 6, 5)
    lens = torch.tensor([[[5, 0, 1, 3], [2, 4, 0, 5]]], dtype=torch.int32)
    o, lse = run(q, k, v, idx, lens)
    want, want_lse = O.masked_dense_attention(q, k, v, O.block_mask_from_indices(idx, lens, 6), 64, 64, 1 / math.sqrt(128))
    close(o, want, torch.bfloat16)
    empty = (lens == 0).repeat_interleave(64, dim=-1)
    assert torch.all(o[empty] == 0) and torch.all(torch.isinf(lse[empty]) & (lse[empty] < 0))
    assert torch.allclose(lse[~empty], want_lse[~empty], atol=2e-3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_malformed_lists_are_clamped(dtype):
    """Block indices outside [0, nbk) and lengths outside [0, list width] are clamped by the kernels, so a bad list
    costs wrong numbers for that query block and never an access outside k and v."""
    q, k, v = seeded_qkv(27, 1, 2, 192, 320, 128, dtype)
    idx, _ = random_lists(27, 1, 2, 3, 5, 3)
    bad = idx.clone()                      # rows chosen so that the clamped lists hold no block twice
    bad[0, 0, 0] = torch.tensor([-1, 2, 3])
    bad[0, 0, 1] = torch.tensor([1, 2, 5])
    bad[0, 1, 2] = torch.tensor([0, 2 ** 30, 1])
    lens = torch.tensor([[[3, 3, 99], [-4, 3, 3]]], dtype=torch.int32)
    o, lse = run(q, k, v, bad, lens)
    mask = O.block_mask_from_indices(bad.clamp(0, 4), lens.clamp(0, 3), 5)
    want, want_lse = O.masked_dense_attention(q, k, v, mask, 64, 64, 1 / math.sqrt(128))
    close(o, want, dtype)
    assert torch.all(o[0, 1, :64] == 0)
    ok = ~torch.isinf(want_lse)
    assert torch.allclose(lse[ok], want_lse[ok], atol=2e-3)


@pytest.mark.parametrize("pattern", ["tail", "first16", "second_half", "sparse"])
def test_padded_keys_are_masked(pattern):
    q, k, v = seeded_qkv(24, 1, 1, 128, 256, 128, torch.bfloat16)
    valid = torch.ones(256, dtype=torch.bool)
    if pattern == "tail":
        valid[200:] = False
    elif pattern == "first16":                # a T-padded chunk: only slots 0..15 of each tile are real
        valid.view(4, 64)[:, 16:] = False
    elif pattern == "second_half":
        valid.view(4, 64)[1:3, :32] = False
    else:
        valid[torch.randperm(256, generator=torch.Generator().manual_seed(1))[:150]] = False
        valid[::64] = True                    # every block keeps a real key
    bits = np.packbits(valid.numpy().reshape(-1, 64), axis=1, bitorder="little").view(np.uint64).reshape(-1)
    idx, lens = random_lists(24, 1, 1, 2, 4, 3)
    o, lse = run(q, k, v, idx, lens, valid_bits=bits)
    want, want_lse = O.masked_dense_attention(q, k, v, O.block_mask_from_indices(idx, lens, 4), 64, 64,
                                              1 / math.sqrt(128), key_valid=valid)
    close(o, want, torch.bfloat16)
    assert torch.allclose(lse, want_lse, atol=2e-3)


def test_128_token_chunks():
    """The reference's default 4x4x8 chunk: 128-token query and key blocks."""
    q, k, v = seeded_qkv(25, 1, 2, 256, 640, 128, torch.bfloat16)
    idx, lens = random_lists(25, 1, 2, 2, 5, 2)
    o, lse = run(q, k, v, idx, lens, bs_q=128, bs_k=128)
    want, want_lse = O.masked_dense_attention(q, k, v, O.block_mask_from_indices(idx, lens, 5), 128, 128, 1 / math.sqrt(128))
    close(o, want, torch.bfloat16)
    assert torch.allclose(lse, want_lse, atol=2e-3)


def test_lse_merge_identity_and_determinism():
    q, k, v = seeded_qkv(26, 1, 1, 64, 512, 128, torch.bfloat16)
    full = torch.tensor([5, 1, 7, 2, 0, 6]).view(1, 1, 1, 6)
    n = lambda c: torch.full((1, 1, 1), c, dtype=torch.int32)
    o, lse = run(q, k, v, full, n(6))
    oa, la = run(q, k, v, full[..., :3].contiguous(), n(3))
    ob, lb = run(q, k, v, full[..., 3:].contiguous(), n(3))
    om, lm = O.merge_partial_attention(oa, la, ob, lb)
    assert (om - o.float()).abs().max() <= 1.6e-2 and torch.allclose(lm, lse, atol=2e-3)
    o2, lse2 = run(q, k, v, full, n(6))
    assert torch.equal(o, o2) and torch.equal(lse, lse2)
    o_rev, _ = run(q, k, v, full.flip(-1).contiguous(), n(6))
    assert (o_rev.float() - o.float()).abs().max() <= 1.6e-2


def test_large_logits_do_not_overflow():
    q, k, v = seeded_qkv(27, 1, 1, 64, 128, 128, torch.bfloat16)
    q = (q.float() * 30).bfloat16()
    idx, lens = random_lists(27, 1, 1, 1, 2, 2)
    o, lse = run(q, k, v, idx, lens)
    want, want_lse = O.masked_dense_attention(q, k, v, O.block_mask_from_indices(idx, lens, 2), 64, 64, 1 / math.sqrt(128))
    assert torch.isfinite(o.float()).all()
    close(o, want, torch.bfloat16)
    assert torch.allclose(lse, want_lse, rtol=1e-4, atol=2e-3)


def test_480p_two_heads_sampled_rows():
    """benchmark configuration 2 geometry with 2 heads: 624 blocks, 39 selected per row,
    checked on sampled query blocks against the gathered fp32 oracle."""
    nb, ks = 624, 39
    q, k, v = seeded_qkv(1, 1, 2, nb * 64, nb * 64, 128, torch.bfloat16)
    idx, lens = random_lists(28, 1, 2, nb, nb, ks)
    o, lse = run(q, k, v, idx, lens)
    rows = [0, 1, 311, 622, 623]
    want, want_lse = O.gathered_attention(q, k, v, idx, lens, 64, 64, 1 / math.sqrt(128), q_blocks=rows)
    for m in rows:
        sl = slice(m * 64, (m + 1) * 64)
        close(o[:, :, sl], want[:, :, sl], torch.bfloat16)
        assert torch.allclose(lse[:, :, sl], want_lse[:, :, sl], atol=2e-3)


@pytest.mark.parametrize("latent,chunk", [
    ((5, 9, 13), (4, 4, 4)),     # padded chunks in t, h and w
    ((5, 6, 12), (4, 4, 8)),     # 128-slot chunks, one 64-slot tile of padding only
    ((4, 8, 6), (4, 8, 2)),      # chunk shape without gathering: k and v copied in full
])
def test_thw_attention_equals_permute_attend_unpermute(latent, chunk):
    """attn_fwd_bsa_thw reads q/k/v and writes o/lse in (T,H,W) order; the blocked-order kernel between
    a permute and an unpermute (bsa_interface.py:650-659) must give the same result, also for lists
    of different lengths (an empty one included) in arbitrary order.  With the LDS-tiled kernel on the blocked-order
    route the two routes run different kernels
    (one online softmax over 32-key steps on fragment-order K/V against two 32-key halves per tile merged at the
    end), so P is rounded to bf16 relative to different running maxima and the sums run in different orders: the results
    agree to a couple of bf16 ulps of the value rows (max-abs 1.6e-2, mean-abs 1e-3), like either against the oracle."""
    bi = I()
    S = int(np.prod(latent))
    bs = int(np.prod(chunk))
    q, k, v = (x.cuda() for x in seeded_qkv(41, 1, 2, S, S, 128, torch.bfloat16))
    nb = int(np.prod(O.block_grid(latent, chunk)))
    gen = torch.Generator().manual_seed(42)
    n = max(nb // 2, 1)
    idx = torch.stack([torch.randperm(nb, generator=gen)[:n] for _ in range(2 * nb)]).view(1, 2, nb, n).int().cuda()
    lens = torch.randint(0, n + 1, (1, 2, nb), generator=gen).int().cuda()
    lens[0, 0, 0] = 0
    lens[0, 1, nb - 1] = n
    qp, _, _ = bi._permute(q, latent, chunk)
    kp, _, valid = bi._permute(k, latent, chunk, want_valid=True)
    vp, _, _ = bi._permute(v, latent, chunk)
    padded = any(a % c for a, c in zip(latent, chunk))
    op, lse_p = bi.attn_fwd_bsa_varlen(qp, kp, vp, 0.11, idx, lens, bs, bs, tile_valid=valid if padded else None,
                                       kernel=KERNEL["name"])
    grid = O.block_grid(latent, chunk)
    want = bi.rearrange_3d_block_to_THW(op, *grid, *chunk, 128, latent_shape=latent)
    want_lse = O.rearrange_3d_block_to_thw(lse_p.cpu().unsqueeze(-1), latent, chunk)[..., 0]
    got, lse = bi.attn_fwd_bsa_thw(q, k, v, latent, latent, chunk, chunk, idx, lens, sm_scale=0.11, return_lse=True)
    d = (got.float() - want.float()).abs()
    assert d.max() <= 1.6e-2 and d.mean() <= 1e-3, (float(d.max()), float(d.mean()))
    if KERNEL["name"] == "fragment":
        # the same kernel on both routes, reading q and writing o through a row table on one of them: the same bits
        assert torch.equal(got, want) and torch.equal(lse.cpu(), want_lse)
    # rows of empty lists and their lse are exact on both routes
    assert torch.equal(got == 0, want == 0)
    assert torch.allclose(lse.cpu(), want_lse, atol=1e-4, rtol=1e-5)
    assert torch.equal(torch.isinf(lse.cpu()), torch.isinf(want_lse))


@pytest.mark.parametrize("seed", range(16))
def test_random_lists_lengths_and_masks(seed):
    """Seeded random draws: 64- and 128-token blocks, list widths, lengths from 0 to the width, lists in random
    order, validity masks that blank random keys, whole tiles, whole 32-key halves or a tail, every storage type."""
    import random
    rnd = random.Random(6000 + seed)
    B, H = rnd.choice([1, 1, 2]), rnd.choice([1, 2, 3])
    bs_q, bs_k = rnd.choice([64, 64, 128]), rnd.choice([64, 64, 128])
    nbq, nbk = rnd.randint(1, 6), rnd.randint(1, 12)
    width = rnd.randint(1, nbk)
    dtype = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
    Sq, Sk = nbq * bs_q, nbk * bs_k
    g = torch.Generator().manual_seed(6000 + seed)
    q, k, v = (torch.randn(B, H, s, 128, generator=g).to(dtype) for s in (Sq, Sk, Sk))
    idx = torch.stack([torch.randperm(nbk, generator=g)[:width] for _ in range(B * H * nbq)]).view(B, H, nbq, width)
    lens = torch.randint(0, width + 1, (B, H, nbq), generator=g, dtype=torch.int32)
    valid, bits = None, None
    mode = rnd.choice(["none", "rand", "tiles", "halves", "tail"])
    if mode != "none":
        valid = torch.ones(Sk, dtype=torch.bool)
        if mode == "rand":
            valid = torch.rand(Sk, generator=g) < 0.6
        elif mode == "tiles":
            valid.view(-1, 64)[torch.rand(Sk // 64, generator=g) < 0.4] = False
        elif mode == "halves":
            valid.view(-1, 32)[torch.rand(Sk // 32, generator=g) < 0.5] = False
        else:
            valid[rnd.randint(0, Sk - 1):] = False
        bits = np.packbits(valid.numpy().reshape(-1, 64), axis=1, bitorder="little").view(np.uint64).reshape(-1)
    o, lse = run(q, k, v, idx, lens, bs_q, bs_k, valid_bits=bits)
    want, want_lse = O.masked_dense_attention(q, k, v, O.block_mask_from_indices(idx, lens, nbk), bs_q, bs_k,
                                              1 / math.sqrt(128), key_valid=valid)
    close(o, want, dtype)
    fin = torch.isfinite(want_lse)
    assert torch.allclose(lse[fin], want_lse[fin], atol=2e-3)
    assert torch.all(torch.isinf(lse[~fin]) & (lse[~fin] < 0)) and torch.all(o[~fin] == 0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_items_with_and_without_a_norm_bound_side_by_side(dtype):
    """The fragment-order kernel runs a launch's work items several per workgroup, each prepared by the one before it,
    without row maxima where |q| |k| bounds the logits; an item without such a bound is left to a last launch of the
    exact kernel, and the item after it starts from scratch.  6 400 work items (every workgroup runs six or seven), of
    which every third query block has rows 40 times the usual size, some lists are empty and some are short: against
    the LDS-tiled kernel on every row (a different summation order: 1.6e-2 / 1e-3) and against the oracle on sampled
    query blocks of both kinds."""
    bi = I()
    H, nbq, nbk, width = 5, 1280, 96, 6
    g = torch.Generator().manual_seed(61)
    q = torch.randn(1, H, nbq * 64, 128, generator=g)
    k = torch.randn(1, H, nbk * 64, 128, generator=g)
    v = torch.randn(1, H, nbk * 64, 128, generator=g)
    big = (torch.arange(nbq) % 3 == 1).repeat_interleave(64).view(1, 1, -1, 1)
    q = torch.where(big, q * 40.0, q).to(dtype)
    k, v = k.to(dtype), v.to(dtype)
    idx = torch.stack([torch.randperm(nbk, generator=g)[:width].sort().values for _ in range(H * nbq)]).view(1, H, nbq, width).int()
    lens = torch.full((1, H, nbq), width, dtype=torch.int32)
    lens[:, :, 5::17] = 0
    lens[:, :, 7::23] = 2
    outs = {}
    for kern in ("fragment", "lds"):
        o, lse = bi.attn_fwd_bsa_varlen(q.cuda(), k.cuda(), v.cuda(), 1 / math.sqrt(128), idx.cuda(), lens.cuda(), 64, 64, kernel=kern)
        torch.cuda.synchronize()
        outs[kern] = (o.cpu(), lse.cpu())
    o, lse = outs["fragment"]
    o2, lse2 = outs["lds"]
    assert torch.isfinite(o.float()).all()
    d = (o.float() - o2.float()).abs()
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10       # a nearly one-hot row gives one row of v: one ulp of its size
    assert bool((d <= 1.6e-2 + ulp * o2.float().abs()).all()) and float(d.mean()) <= 1e-3, (float(d.max()), float(d.mean()))
    fin = torch.isfinite(lse2)
    assert torch.equal(torch.isfinite(lse), fin) and torch.allclose(lse[fin], lse2[fin], rtol=1e-4, atol=2e-3)
    empty = (lens == 0).repeat_interleave(64, dim=-1)
    assert torch.all(o[empty] == 0)
    # the oracle on a few query blocks of each kind, first and last work items included
    for h, m in ((0, 0), (0, 1), (1, 4), (2, 640), (3, 1024), (4, 1278), (4, 1279), (2, 7), (1, 5)):
        rows = slice(64 * m, 64 * m + 64)
        want, want_lse = O.masked_dense_attention(q[:, h:h + 1, rows], k[:, h:h + 1], v[:, h:h + 1],
                                                  O.block_mask_from_indices(idx[:, h:h + 1, m:m + 1].long(), lens[:, h:h + 1, m:m + 1], nbk),
                                                  64, 64, 1 / math.sqrt(128))
        close(o[:, h:h + 1, rows], want, dtype)
        f = torch.isfinite(want_lse)
        assert torch.allclose(lse[:, h:h + 1, rows][f], want_lse[f], rtol=1e-4, atol=2e-3)


@pytest.mark.parametrize("case", ["scaled", "late", "late_within_bound", "nan_free_zero_keys"])
def test_thw_kernel_keeps_its_exponentials_finite(case):
    """The (T,H,W)-order kernel raises its running maximum lazily and rescales its accumulators a quarter of a step
    after the maximum has moved.  Inputs that drive that path hard: logits scaled far beyond the usual range; a list
    whose first blocks give tiny logits and whose last blocks give huge ones (the maximum moves late and far); the same
    with a milder slope; all-zero keys."""
    bi = I()
    latent, chunk = (8, 8, 16), (4, 4, 4)
    S, nb = 1024, 16
    q, k, v = seeded_qkv(90, 1, 2, S, S, 128, torch.bfloat16)
    kp = O.rearrange_thw_to_3d_block(k, latent, chunk).float()
    if case == "scaled":
        q = (q.float() * 30).bfloat16()
    elif case in ("late", "late_within_bound"):
        # keys of the low blocks shrink, keys of the high blocks grow: ascending lists meet the large logits last
        gain = torch.linspace(-6, 5 if case == "late" else 1.5, nb).exp2().repeat_interleave(64).view(1, 1, -1, 1)
        k = O.rearrange_3d_block_to_thw((kp * gain).bfloat16(), latent, chunk)
        q = (q.float() * (6 if case == "late" else 1)).bfloat16()
    else:
        k = torch.zeros_like(k)
    g = torch.Generator().manual_seed(91)
    idx = torch.stack([torch.randperm(nb, generator=g)[:8].sort().values for _ in range(2 * nb)]).view(1, 2, nb, 8)
    lens = torch.full((1, 2, nb), 8, dtype=torch.int32)
    o, lse = bi.attn_fwd_bsa_thw(q.cuda(), k.cuda(), v.cuda(), latent, latent, chunk, chunk, idx.int().cuda(), lens.cuda(),
                                 return_lse=True)
    qp = O.rearrange_thw_to_3d_block(q, latent, chunk)
    kp = O.rearrange_thw_to_3d_block(k, latent, chunk)
    vp = O.rearrange_thw_to_3d_block(v, latent, chunk)
    want, want_lse = O.masked_dense_attention(qp, kp, vp, O.block_mask_from_indices(idx, lens, nb), 64, 64, 1 / math.sqrt(128))
    got = O.rearrange_thw_to_3d_block(o.cpu(), latent, chunk)
    got_lse = O.rearrange_thw_to_3d_block(lse.cpu().unsqueeze(-1), latent, chunk)[..., 0]
    assert torch.isfinite(got.float()).all() and torch.isfinite(got_lse).all()
    close(got, want, torch.bfloat16)
    assert torch.allclose(got_lse, want_lse, rtol=1e-4, atol=2e-3)

"""R5/R6/R9 on the GPU at the edges of the kernel's list handling and chunk sizes:

* chunks of 256 tokens (4x8x8, 8x4x8, 8x8x4), which the reference sends to its second kernel
  (`_attn_fwd_bsa_varlen`, flash_attn_bsa_varlen_mask.py:35-153, dispatched at bsa_interface.py:310-335);
* index lists longer than the 256 tiles that are staged before the list length has arrived, and longer than
  the 1 024 tiles staged at a time (the route the CDF rule takes on large grids);
* `torch.compile(fullgraph=True)` of a caller (run_demo_text_to_video.py:57-58 compiles the transformer).

Tolerances as everywhere: bf16 outputs within max-abs 2e-2 / mean-abs 2e-3 of the fp32 oracle, lse 2e-3."""
import math

import numpy as np
import pytest
import torch

from oracle import bsa_oracle as O
from conftest import seeded_qkv
from test_gpu_e2e import check_against_oracle

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 2e-2, 2e-3


def I():
    from longcat_video_amd.block_sparse_attention import bsa_interface
    return bsa_interface


def close(o, want):
    d = (o.float() - want).abs()
    assert d.max() <= MAX_ABS and d.mean() <= MEAN_ABS, (float(d.max()), float(d.mean()))


# ------------------------------------------------------------------ 256-token chunks
@pytest.mark.parametrize("latent,chunk", [
    ((8, 16, 16), (4, 8, 8)),      # even grid, one (h, w) plane per 64-slot tile, four tiles per chunk
    ((16, 8, 16), (8, 4, 8)),      # two planes per tile
    ((16, 16, 8), (8, 8, 4)),      # runs of 4 tokens, two planes per tile
    ((6, 13, 20), (4, 8, 8)),      # ragged in t, h and w: whole tiles of a chunk are padding
    ((11, 6, 21), (8, 4, 8)),
    ((9, 20, 7), (8, 8, 4)),
])
def test_operator_with_256_token_chunks(latent, chunk):
    S = int(np.prod(latent))
    q, k, v = seeded_qkv(50, 1, 2, S, S, 128, torch.bfloat16)
    o, idx, lens, score = I()._bsa_3d(q.cuda(), k.cuda(), v.cuda(), latent, latent, 0.5, chunk, chunk, True)
    nb = int(np.prod(O.block_grid(latent, chunk)))
    assert idx.shape == (1, 2, nb, nb // 2)
    check_against_oracle(q, k, v, latent, latent, 0.5, o, idx, lens, score, q_blocks=range(nb), chunk=chunk)
    assert torch.isfinite(o.float()).all()
    pub = I().flash_attn_bsa_3d(q.cuda(), k.cuda(), v.cuda(), latent, latent, sparsity=0.5,
                                chunk_3d_shape_q=list(chunk), chunk_3d_shape_k=list(chunk))
    assert torch.equal(pub, o)


@pytest.mark.parametrize("bs_q,bs_k", [(256, 256), (64, 256), (256, 128)])
def test_blocked_order_kernel_with_256_token_blocks(bs_q, bs_k):
    nbq, nbk, width = 3, 7, 4
    q, k, v = seeded_qkv(51, 1, 2, nbq * bs_q, nbk * bs_k, 128, torch.bfloat16)
    g = torch.Generator().manual_seed(51)
    idx = torch.stack([torch.randperm(nbk, generator=g)[:width] for _ in range(2 * nbq)]).view(1, 2, nbq, width)
    lens = torch.tensor([[[4, 1, 3], [0, 4, 2]]], dtype=torch.int32)
    o, lse = I().attn_fwd_bsa_varlen(q.cuda(), k.cuda(), v.cuda(), 1 / math.sqrt(128), idx.cuda(), lens.cuda(), bs_q, bs_k)
    want, want_lse = O.masked_dense_attention(q, k, v, O.block_mask_from_indices(idx, lens, nbk), bs_q, bs_k, 1 / math.sqrt(128))
    close(o.cpu(), want)
    fin = torch.isfinite(want_lse)
    assert torch.allclose(lse.cpu()[fin], want_lse[fin], atol=2e-3)
    assert torch.all(o.cpu()[~fin] == 0)


@pytest.mark.parametrize("latent,chunk", [((6, 13, 20), (4, 8, 8)), ((9, 20, 7), (8, 8, 4))])
def test_thw_attention_with_256_token_chunks_equals_the_blocked_route(latent, chunk):
    bi = I()
    S, bs = int(np.prod(latent)), int(np.prod(chunk))
    q, k, v = (x.cuda() for x in seeded_qkv(52, 1, 2, S, S, 128, torch.bfloat16))
    nb = int(np.prod(O.block_grid(latent, chunk)))
    gen = torch.Generator().manual_seed(52)
    n = max(nb // 2, 1)
    idx = torch.stack([torch.randperm(nb, generator=gen)[:n] for _ in range(2 * nb)]).view(1, 2, nb, n).int().cuda()
    lens = torch.randint(0, n + 1, (1, 2, nb), generator=gen).int().cuda()
    qp, _, _ = bi._permute(q, latent, chunk)
    kp, _, valid = bi._permute(k, latent, chunk, want_valid=True)
    vp, _, _ = bi._permute(v, latent, chunk)
    op, _ = bi.attn_fwd_bsa_varlen(qp, kp, vp, 0.09, idx, lens, bs, bs, tile_valid=valid)
    want = bi.rearrange_3d_block_to_THW(op, *O.block_grid(latent, chunk), *chunk, 128, latent_shape=latent)
    got = bi.attn_fwd_bsa_thw(q, k, v, latent, latent, chunk, chunk, idx, lens, sm_scale=0.09)
    # two kernels: P rounded relative to different running maxima, sums in different orders
    d = (got.float() - want.float()).abs()
    assert d.max() <= 1.6e-2 and d.mean() <= 1e-3, (float(d.max()), float(d.mean()))
    assert torch.equal(got == 0, want == 0)


# ------------------------------------------------------------------ long index lists
def lists_with_lengths(seed, H, nbq, nbk, width, forced):
    """Random lists of `width` distinct blocks per row, lengths uniform in [0, width] with some rows forced."""
    g = torch.Generator().manual_seed(seed)
    idx = torch.stack([torch.randperm(nbk, generator=g)[:width] for _ in range(H * nbq)]).view(1, H, nbq, width)
    lens = torch.randint(0, width + 1, (1, H, nbq), generator=g, dtype=torch.int32)
    flat = lens.view(-1)
    for i, n in enumerate(forced):
        flat[i % flat.numel()] = n
    return idx, lens


@pytest.mark.parametrize("bs_k,width", [
    (64, 300),       # 300 tiles: the list length is awaited, one staging chunk
    (64, 1025),      # two staging chunks, the second of one tile (odd tail)
    (64, 1500),      # two chunks, even tail
    (128, 520),      # 1 040 tiles of 64: the chunk boundary falls between two blocks
    (128, 1000),     # 2 000 tiles
])
def test_blocked_order_kernel_with_long_lists(bs_k, width):
    H, nbq = 2, 6
    nbk = width + 37
    nsub = bs_k // 64
    q, k, v = seeded_qkv(60 + width, 1, H, nbq * 64, nbk * bs_k, 128, torch.bfloat16)
    cap = 1024 // nsub
    forced = [width, 0, 1, min(cap, width), min(cap + 1, width), min(cap - 1, width), max(width - 1, 0), 256 // nsub + 1]
    idx, lens = lists_with_lengths(60 + width, H, nbq, nbk, width, forced)
    o, lse = I().attn_fwd_bsa_varlen(q.cuda(), k.cuda(), v.cuda(), 1 / math.sqrt(128), idx.cuda(), lens.cuda(), 64, bs_k)
    rows = range(nbq)
    want, want_lse = O.gathered_attention(q, k, v, idx, lens, 64, bs_k, 1 / math.sqrt(128), q_blocks=rows)
    close(o.cpu(), want)
    fin = torch.isfinite(want_lse)
    assert torch.allclose(lse.cpu()[fin], want_lse[fin], atol=2e-3)
    assert torch.all(o.cpu()[~fin] == 0) and torch.all(torch.isinf(lse.cpu()[~fin]))


@pytest.mark.parametrize("unequal", [False, True])
@pytest.mark.parametrize("chunk,width", [((4, 4, 4), 300), ((4, 4, 4), 1100), ((4, 4, 8), 560)])
def test_thw_attention_with_long_lists(chunk, width, unequal):
    """ThwAttention (bsa_fwd_thw) with lists beyond 256 and beyond 1 024 tiles, as rounds and, with
    `unequal_lengths`, with the schedule chosen on the device."""
    bi = I()
    latent = (36, 32, 64)
    S, bs = int(np.prod(latent)), int(np.prod(chunk))
    nb = int(np.prod(O.block_grid(latent, chunk)))
    assert width <= nb
    H = 2
    q, k, v = seeded_qkv(70 + width, 1, H, S, S, 128, torch.bfloat16)
    cap = 1024 // (bs // 64)
    g = torch.Generator().manual_seed(70 + width)
    idx = torch.stack([torch.randperm(nb, generator=g)[:width] for _ in range(H * nb)]).view(1, H, nb, width)
    lens = torch.randint(0, width + 1, (1, H, nb), generator=g, dtype=torch.int32)
    sample = [0, 1, 2, 3, nb // 2, nb - 1]
    for m, n in zip(sample, [width, 0, min(cap, width), min(cap + 1, width), 1, width]):
        lens[0, :, m] = n
    att = bi.ThwAttention(k.cuda(), v.cuda(), latent, latent, chunk, chunk, unequal_lengths=unequal)
    o, lse = att(q.cuda(), idx.int().cuda(), lens.cuda(), return_lse=True)
    qp = O.rearrange_thw_to_3d_block(q, latent, chunk)
    kp = O.rearrange_thw_to_3d_block(k, latent, chunk)
    vp = O.rearrange_thw_to_3d_block(v, latent, chunk)
    more = [int(x) for x in torch.randint(0, nb, (6,), generator=g)]
    rows = sorted(set(sample + more))
    want, want_lse = O.gathered_attention(qp, kp, vp, idx, lens, bs, bs, 1 / math.sqrt(128), q_blocks=rows)
    got = O.rearrange_thw_to_3d_block(o.cpu(), latent, chunk)
    got_lse = O.rearrange_thw_to_3d_block(lse.cpu().unsqueeze(-1), latent, chunk)[..., 0]
    for m in rows:
        sl = slice(m * bs, (m + 1) * bs)
        if int(lens[0, 0, m]) == 0:
            assert torch.all(got[:, 0, sl] == 0)
        close(got[:, :, sl], want[:, :, sl])
        fin = torch.isfinite(want_lse[:, :, sl])
        assert torch.allclose(got_lse[:, :, sl][fin], want_lse[:, :, sl][fin], atol=2e-3)
    assert torch.isfinite(o.float()).all()


# ------------------------------------------------------------------ torch.compile of a caller
@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
def test_torch_compile_of_a_caller_does_not_graph_break(backend):
    """A caller shaped like Attention._process_attn (attention.py:58-67) compiled with fullgraph=True: Dynamo
    must trace through the custom op (a graph break would raise), and the result must equal eager.  The
    reference compiles with the default backend (run_demo_text_to_video.py:57-58); aot_eager checks the trace
    and the fake kernel without any code generation."""
    bi = I()
    latent = (4, 8, 8)
    prm = dict(sparsity=0.5, cdf_threshold=None, chunk_3d_shape_q=[4, 4, 4], chunk_3d_shape_k=[4, 4, 4])

    def caller(q, k, v):
        x = bi.flash_attn_bsa_3d(q * 1.0, k, v, latent, latent, **prm)
        return x.transpose(1, 2).reshape(q.shape[0], q.shape[2], -1) + 1.0

    q, k, v = (t.cuda() for t in seeded_qkv(80, 1, 2, 256, 256, 128, torch.bfloat16))
    torch._dynamo.reset()
    with torch.no_grad():
        want = caller(q, k, v)
        got = torch.compile(caller, fullgraph=True, backend=backend)(q, k, v)
        torch.cuda.synchronize()
        assert got.shape == want.shape
        assert torch.allclose(got.float(), want.float(), atol=1e-2)     # the elementwise tail may fuse differently
        # the operator itself is the same kernel in both: compare it alone, bit for bit
        op_only = torch.compile(lambda a, b, c: bi.flash_attn_bsa_3d(a, b, c, latent, latent, **prm),
                                fullgraph=True, backend=backend)
        assert torch.equal(op_only(q, k, v), bi.flash_attn_bsa_3d(q, k, v, latent, latent, **prm))

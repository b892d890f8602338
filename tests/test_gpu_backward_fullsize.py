"""The backward (bsa_bwd through the C-ABI) at the sizes of the benchmark configurations and beyond one round of
work items: every launch span of the dQ kernel, the XCD remap of later rounds, the longest-first order of the dK / dV
kernel over many (batch, head).  At these sizes the oracle's restatement of the reference backward
(flash_attn_bsa_varlen_mask.py:288-360, 428-500; bsa_interface.py:343-461) is evaluated on sampled query blocks (all
pairs of each) and sampled KV blocks (all query blocks that selected each); tolerances as in test_gpu_backward.py."""
import math

import numpy as np
import pytest
import torch

from oracle import bsa_oracle as O

pytestmark = pytest.mark.gpu


def I():
    from longcat_video_amd.block_sparse_attention import bsa_interface
    return bsa_interface


def close_to_restatement(got, want, name):
    ulp = 2.0 ** -7 if got.dtype == torch.bfloat16 else 2.0 ** -10
    g, w = got.float(), want.float()
    assert torch.isfinite(g).all(), name
    err = (g - w).abs()
    assert float(err.max()) <= 4 * ulp * float(w.abs().max()) + 1e-6, (name, float(err.max()), float(w.abs().max()))
    assert float(err.mean()) <= 0.5 * ulp * float(w.abs().mean()) + 1e-7, (name, float(err.mean()), float(w.abs().mean()))


def backward_twice(bi, qp, kp, vp, do, sm, idx, lens, valid):
    o, lse = bi.attn_fwd_bsa_varlen(qp, kp, vp, sm, idx, lens, 64, 64, tile_valid=valid)
    runs = []
    for _ in range(2):
        dq, dk, dv = (torch.full(t.shape, float("nan"), dtype=t.dtype, device="cuda") for t in (qp, kp, vp))
        bi.attn_bwd_bsa_varlen(do, qp, kp, vp, o, dq, dk, dv, sm, lse, idx, lens, 64, 64, tile_valid=valid)
        runs.append((dq, dk, dv))
    torch.cuda.synchronize()
    for a, b, name in zip(runs[0], runs[1], ("dq", "dk", "dv")):
        assert torch.isfinite(a.float()).all(), name
        assert torch.equal(a, b), name + " differs between two runs"
    return o, lse, runs[0]


def check_sampled(qp, kp, vp, do, o, lse, grads, idx, lens, sm, q_items, kv_items, key_valid=None):
    """q_items / kv_items: (batch, head, block) triples.  One (batch, head) at a time goes to the host."""
    dq, dk, dv = grads
    pairs = sorted(set((b, h) for b, h, _ in q_items) | set((b, h) for b, h, _ in kv_items))
    for b, h in pairs:
        qb = [m for bb, hh, m in q_items if (bb, hh) == (b, h)]
        kb = [j for bb, hh, j in kv_items if (bb, hh) == (b, h)]
        one = lambda t: t[b:b + 1, h:h + 1].cpu()
        wq, wk, wv = O.blockwise_attention_backward(one(qp), one(kp), one(vp), one(o), one(do), one(lse), one(idx).long(), one(lens),
                                                    64, 64, sm, key_valid=key_valid, q_blocks=qb, kv_blocks=kb)
        rows = lambda blocks: torch.cat([torch.arange(64 * m, 64 * m + 64) for m in blocks]) if blocks else None
        if qb:
            r = rows(qb)
            close_to_restatement(one(dq)[:, :, r], wq[:, :, r], "dq of (b=%d, h=%d), query blocks %s" % (b, h, qb))
        if kb:
            r = rows(kb)
            close_to_restatement(one(dk)[:, :, r], wk[:, :, r], "dk of (b=%d, h=%d), KV blocks %s" % (b, h, kb))
            close_to_restatement(one(dv)[:, :, r], wv[:, :, r], "dv of (b=%d, h=%d), KV blocks %s" % (b, h, kb))


@pytest.mark.parametrize("name,latent,sparsity,seed,rms", [("c3", (24, 45, 80), 0.9375, 2, True), ("c2", (24, 30, 52), 0.9375, 1, False)])
def test_backward_at_a_benchmark_geometry(name, latent, sparsity, seed, rms):
    """32 heads on the padded grid of benchmark configuration 3 (1 440 blocks, 90 per row) and 2 (624 blocks, 39 per
    row), lists from the operator's own gating: 46 080 / 19 968 query tiles are 23 / 10 launches of two rounds of the
    dQ kernel, and as many KV tiles in groups of 1 024 for the dK / dV kernel."""
    bi = I()
    H, chunk = 32, (4, 4, 4)
    S = int(np.prod(latent))
    g = torch.Generator(device="cuda").manual_seed(seed)
    thw = []
    for i in range(4):                                                  # q, k, v, dO in (T, H, W) order
        x = torch.randn(1, H, S, 128, generator=g, device="cuda")
        if rms and i < 2:
            x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)
        thw.append(x.bfloat16())
        del x
    qp, _, _ = bi._permute(thw[0], latent, chunk)
    kp, _, valid = bi._permute(thw[1], latent, chunk, want_valid=True)
    vp, _, _ = bi._permute(thw[2], latent, chunk)
    do, _, _ = bi._permute(thw[3], latent, chunk)                       # padded query rows: a zero gradient comes in
    del thw
    nb = qp.shape[2] // 64
    sm = 1 / math.sqrt(128)
    idx, lens = bi._select_blocked(qp, kp, 64, 64, sparsity, None)
    k_sel = O.num_selected(sparsity, nb)
    assert idx.shape == (1, H, nb, k_sel) and bool((lens == k_sel).all())
    o, lse, grads = backward_twice(bi, qp, kp, vp, do, sm, idx, lens, valid)
    key_valid = torch.from_numpy(O.slot_validity(latent, chunk))
    assert int((~key_valid).sum()) > 0
    # padded keys receive no gradient, in any head
    pad = (~key_valid).cuda()
    assert bool((grads[1][:, :, pad] == 0).all()) and bool((grads[2][:, :, pad] == 0).all())
    # query tiles: first and last of the layer, both sides of the first head boundary, both sides of launch
    # boundaries (2 048 tiles per launch) and of a round boundary inside a launch (1 024), and a few anywhere
    total = H * nb
    rnd = np.random.default_rng(seed)
    tiles = sorted(set([0, nb - 1, nb, 1023, 1024, 2047, 2048, (total // 2048) * 2048 - 1, min((total // 2048) * 2048, total - 1), total - 1]
                       + [int(x) for x in rnd.integers(0, total, 4)]))
    q_items = [(0, t // nb, t % nb) for t in tiles]
    # KV blocks: the most and the least selected of two heads, and a few anywhere
    kv_items = []
    for h in (0, H - 1):
        counts = torch.bincount(idx[0, h].flatten().long(), minlength=nb).cpu()
        kv_items += [(0, h, int(counts.argmax())), (0, h, int(counts.argmin()))]
    kv_items += [(0, int(rnd.integers(0, H)), int(rnd.integers(0, nb))) for _ in range(3)]
    check_sampled(qp, kp, vp, do, o, lse, grads, idx, lens, sm, q_items, kv_items, key_valid=key_valid)


def test_backward_over_two_batches_and_many_rounds():
    """B = 2, 7 heads, 321 query blocks against 150 KV blocks, lists of 0 to 4 blocks: 4 494 query tiles (four full rounds of
    1 024 and one of 398, not a multiple of 8) and 2 100 KV tiles whose lists hold 0 to about 20 query blocks,
    all of it against the oracle."""
    bi = I()
    B, H, nbq, nbk, width = 2, 7, 321, 150, 4
    g = torch.Generator().manual_seed(77)
    q = torch.randn(B, H, nbq * 64, 128, generator=g).bfloat16()
    k = torch.randn(B, H, nbk * 64, 128, generator=g).bfloat16()
    v = torch.randn(B, H, nbk * 64, 128, generator=g).bfloat16()
    do = torch.randn(B, H, nbq * 64, 128, generator=g).bfloat16()
    idx = torch.stack([torch.randperm(nbk, generator=g)[:width] for _ in range(B * H * nbq)]).view(B, H, nbq, width).int()
    lens = torch.randint(0, width + 1, (B, H, nbq), generator=g, dtype=torch.int32)
    lens[:, :, ::3] = width
    sm = 1 / math.sqrt(128)
    o, lse, grads = backward_twice(bi, q.cuda(), k.cuda(), v.cuda(), do.cuda(), sm, idx.cuda(), lens.cuda(), None)
    wq, wk, wv = O.blockwise_attention_backward(q, k, v, o.cpu(), do, lse.cpu(), idx.long(), lens, 64, 64, sm)
    for got, want, name in zip(grads, (wq, wk, wv), ("dq", "dk", "dv")):
        for b in range(B):
            for h in range(H):
                close_to_restatement(got[b, h].cpu(), want[b, h], "%s of (b=%d, h=%d)" % (name, b, h))
    empty = (lens == 0).repeat_interleave(64, dim=-1)
    assert torch.all(grads[0].cpu()[empty] == 0)

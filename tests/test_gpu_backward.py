"""Backward of the block-sparse attention on the GPU (bsa_bwd through the C-ABI, and autograd through the host
mirror).  Two references: the oracle's restatement of the reference backward with the same rounding points
(tight tolerance: only summation order, exp2 and the forward's own o / lse differ), and torch.autograd through
fp32 masked-dense attention (the roundings of a 16-bit backward apart)."""
import math

import numpy as np
import pytest
import torch

from oracle import bsa_oracle as O

pytestmark = pytest.mark.gpu


def I():
    from longcat_video_amd.block_sparse_attention import bsa_interface
    return bsa_interface


def make_case(seed, H, nbq, nbk, width, dtype, bs_q=64, bs_k=64, min_len=0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(1, H, nbq * bs_q, 128, generator=g).to(dtype)
    k = torch.randn(1, H, nbk * bs_k, 128, generator=g).to(dtype)
    v = torch.randn(1, H, nbk * bs_k, 128, generator=g).to(dtype)
    do = torch.randn(1, H, nbq * bs_q, 128, generator=g).to(dtype)
    idx = torch.stack([torch.randperm(nbk, generator=g)[:width] for _ in range(H * nbq)]).view(1, H, nbq, width).int()
    lens = torch.randint(min_len, width + 1, (1, H, nbq), generator=g, dtype=torch.int32)
    lens[0, :, 0] = width
    return q, k, v, do, idx, lens


def run_gpu(q, k, v, do, idx, lens, bs_q, bs_k, sm, valid_words=None):
    bi = I()
    tv = None if valid_words is None else valid_words.cuda()
    o, lse = bi.attn_fwd_bsa_varlen(q.cuda(), k.cuda(), v.cuda(), sm, idx.cuda(), lens.cuda(), bs_q, bs_k, tile_valid=tv)
    dq, dk, dv = (torch.full(t.shape, float("nan"), dtype=t.dtype, device="cuda") for t in (q, k, v))
    bi.attn_bwd_bsa_varlen(do.cuda(), q.cuda(), k.cuda(), v.cuda(), o, dq, dk, dv, sm, lse, idx.cuda(), lens.cuda(), bs_q, bs_k,
                           tile_valid=tv)
    torch.cuda.synchronize()
    return o.cpu(), lse.cpu(), dq.cpu(), dk.cpu(), dv.cpu()


def close_to_restatement(got, want, name):
    """Same rounding points: an element differs where a rounding of p, ds or of the result fell the other way."""
    ulp = 2.0 ** -7 if got.dtype == torch.bfloat16 else 2.0 ** -10
    g, w = got.float(), want.float()
    assert torch.isfinite(g).all(), name
    err = (g - w).abs()
    scale = float(w.abs().mean())
    assert float(err.max()) <= 4 * ulp * float(w.abs().max()) + 1e-6, (name, float(err.max()), float(w.abs().max()))
    assert float(err.mean()) <= 0.5 * ulp * scale + 1e-7, (name, float(err.mean()), scale)


def words_of(valid):
    """bool [Sk] -> one int64 word per 64 keys, bit i = key i of the tile."""
    bits = valid.view(-1, 64).to(torch.int64)
    w = torch.zeros(bits.shape[0], dtype=torch.int64)
    for i in range(64):
        w |= bits[:, i] << i if i < 63 else torch.where(bits[:, i] > 0, torch.tensor(-2 ** 63), torch.tensor(0))
    return w


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("bs_q,bs_k,nbq,nbk,width", [(64, 64, 9, 14, 5), (128, 64, 4, 11, 4), (64, 128, 6, 5, 3), (128, 128, 3, 4, 2),
                                                       (256, 64, 3, 9, 4), (64, 256, 7, 3, 2), (64, 64, 40, 6, 3), (64, 64, 1, 5, 5)])
def test_against_the_restated_reference_backward(dtype, bs_q, bs_k, nbq, nbk, width):
    sm = 1 / math.sqrt(128)
    q, k, v, do, idx, lens = make_case(nbq * 100 + nbk, 2, nbq, nbk, width, dtype, bs_q, bs_k)
    o, lse, dq, dk, dv = run_gpu(q, k, v, do, idx, lens, bs_q, bs_k, sm)
    wq, wk, wv = O.blockwise_attention_backward(q, k, v, o, do, lse, idx.long(), lens, bs_q, bs_k, sm)
    for got, want, name in ((dq, wq, "dq"), (dk, wk, "dk"), (dv, wv, "dv")):
        close_to_restatement(got, want, name)
    # query blocks with an empty list get a zero gradient, KV blocks nobody selected too
    empty_q = (lens[0] == 0).repeat_interleave(bs_q, dim=-1)
    assert torch.all(dq[0][empty_q] == 0)
    mask = O.block_mask_from_indices(idx.long(), lens, nbk)
    unused = (~mask.any(dim=2))[0].repeat_interleave(bs_k, dim=-1)
    assert torch.all(dk[0][unused] == 0) and torch.all(dv[0][unused] == 0)


def test_padded_keys_and_rows_without_keys():
    sm = 1 / math.sqrt(128)
    q, k, v, do, idx, lens = make_case(7, 2, 5, 8, 3, torch.bfloat16, min_len=1)
    valid = torch.ones(8 * 64, dtype=torch.bool)
    valid[64 * 3 + 17:64 * 4] = False                        # a partly padded block
    valid[64 * 6:64 * 7] = False                             # a block without a real key
    idx[0, 0, 2, 0] = 6
    lens[0, 0, 2] = 1                                        # query block 2 of head 0 sees no real key at all
    idx[0, 1, 3, :2] = torch.tensor([3, 6])
    lens[0, 1, 3] = 2
    o, lse, dq, dk, dv = run_gpu(q, k, v, do, idx, lens, 64, 64, sm, words_of(valid))
    assert torch.all(torch.isinf(lse[0, 0, 128:192])) and torch.all(o[0, 0, 128:192] == 0)
    wq, wk, wv = O.blockwise_attention_backward(q, k, v, o, do, torch.where(torch.isinf(lse), torch.full_like(lse, float("inf")), lse),
                                                idx.long(), lens, 64, 64, sm, key_valid=valid)
    for got, want, name in ((dq, wq, "dq"), (dk, wk, "dk"), (dv, wv, "dv")):
        close_to_restatement(got, want, name)
    assert torch.all(dk[0, :, ~valid] == 0) and torch.all(dv[0, :, ~valid] == 0)
    assert torch.all(dq[0, 0, 128:192] == 0)


def test_medium_case_against_autograd():
    """40 x 40 blocks, density 1/4: against the gradients of fp32 masked-dense attention."""
    sm = 1 / math.sqrt(128)
    q, k, v, do, idx, lens = make_case(8, 2, 40, 40, 10, torch.bfloat16, min_len=10)
    o, lse, dq, dk, dv = run_gpu(q, k, v, do, idx, lens, 64, 64, sm)
    mask = O.block_mask_from_indices(idx.long(), lens, 40)
    wq, wk, wv = O.masked_dense_attention_autograd(q, k, v, do, mask, 64, 64, sm)
    for got, want, name in ((dq, wq, "dq"), (dk, wk, "dk"), (dv, wv, "dv")):
        err = (got.float() - want).abs()
        assert float(err.max()) <= 2.0 ** -6 * 4 * float(want.abs().max()), (name, float(err.max()))
        assert float(err.mean()) <= 2.0 ** -6 * float(want.abs().mean()), (name, float(err.mean()))


def test_autograd_through_the_blocked_order_operator():
    bi = I()
    g = torch.Generator().manual_seed(9)
    q, k, v = (torch.randn(1, 2, 16 * 64, 128, generator=g).bfloat16().cuda().requires_grad_(True) for _ in range(3))
    do = torch.randn(1, 2, 16 * 64, 128, generator=g).bfloat16().cuda()
    sm = 1 / math.sqrt(128)
    o = bi.flash_attn_bsa(q, k, v, 64, 64, 0.75, None, sm)
    o.backward(do)
    idx, lens = bi._select_blocked(q.detach(), k.detach(), 64, 64, 0.75, None)
    mask = O.block_mask_from_indices(idx.cpu().long(), lens.cpu(), 16)
    want = O.masked_dense_attention_autograd(q.detach().cpu(), k.detach().cpu(), v.detach().cpu(), do.cpu(), mask, 64, 64, sm)
    for t, w in zip((q, k, v), want):
        err = (t.grad.cpu().float() - w).abs()
        assert float(err.max()) <= 2.0 ** -6 * 4 * float(w.abs().max()) and float(err.mean()) <= 2.0 ** -6 * float(w.abs().mean())
    # without gradients the same call gives the same output
    with torch.no_grad():
        assert torch.equal(bi.flash_attn_bsa(q, k, v, 64, 64, 0.75, None, sm), o)


@pytest.mark.parametrize("shape", [(8, 8, 16), (6, 10, 14), (9, 13, 22)])
def test_autograd_through_the_operator_on_a_grid(shape):
    """flash_attn_bsa_3d with inputs that require a gradient, on a grid with and without padded chunks: gradients in
    (T, H, W) order against autograd through fp32 attention with the token-level mask of the GPU's own selection."""
    bi = I()
    S = int(np.prod(shape))
    chunk = (4, 4, 4)
    g = torch.Generator().manual_seed(10)
    q, k, v = (torch.randn(1, 2, S, 128, generator=g).bfloat16().cuda().requires_grad_(True) for _ in range(3))
    do = torch.randn(1, 2, S, 128, generator=g).bfloat16().cuda()
    o = bi.flash_attn_bsa_3d(q, k, v, shape, shape, sparsity=0.5, chunk_3d_shape_q=list(chunk), chunk_3d_shape_k=list(chunk))
    o.backward(do)
    with torch.no_grad():
        o_plain = bi.flash_attn_bsa_3d(q, k, v, shape, shape, sparsity=0.5, chunk_3d_shape_q=list(chunk), chunk_3d_shape_k=list(chunk))
    assert torch.equal(o.detach(), o_plain)                                # one forward kernel with and without grad (bsa:538-568)
    # the oracle in blocked order on the GPU's selection
    qp, kp, vp, dop = (O.rearrange_thw_to_3d_block(t.detach().cpu(), shape, chunk) for t in (q, k, v, do))
    idx, lens = bi._select_blocked(qp.cuda(), kp.cuda(), 64, 64, 0.5, None)
    nb = qp.shape[2] // 64
    mask = O.block_mask_from_indices(idx.cpu().long(), lens.cpu(), nb)
    valid = torch.from_numpy(O.slot_validity(shape, chunk))
    wq, wk, wv = O.masked_dense_attention_autograd(qp, kp, vp, dop, mask, 64, 64, 1 / math.sqrt(128), key_valid=valid)
    for t, w in zip((q, k, v), (wq, wk, wv)):
        w_thw = O.rearrange_3d_block_to_thw(w, shape, chunk)
        err = (t.grad.cpu().float() - w_thw).abs()
        assert float(err.max()) <= 2.0 ** -6 * 4 * float(w_thw.abs().max()), float(err.max())
        assert float(err.mean()) <= 2.0 ** -6 * float(w_thw.abs().mean())


def test_autograd_through_the_operator_with_the_cdf_rule():
    """Lists of unequal length (bsa_interface.py:226-266 feeding :570-596) on a padded grid: gradients in (T, H, W) order
    against autograd through fp32 attention with the token-level mask of the GPU's own selection."""
    bi = I()
    shape, chunk = (6, 10, 14), (4, 4, 4)
    S = int(np.prod(shape))
    g = torch.Generator().manual_seed(12)
    q, k, v = (torch.randn(1, 2, S, 128, generator=g) for _ in range(3))
    # a common direction whose weight varies over the grid: the pooled scores then differ from row to row by more than
    # noise, and so do the numbers of blocks the rule keeps
    pos = torch.arange(S).view(1, 1, S, 1).float()
    q = q + 0.6 * torch.sin(pos / 37.0) * torch.ones(128)
    k = k + 0.6 * torch.cos(pos / 53.0) * torch.ones(128)
    q, k, v = (t.bfloat16().cuda().requires_grad_(True) for t in (q, k, v))
    do = torch.randn(1, 2, S, 128, generator=g).bfloat16().cuda()
    prm = dict(sparsity=0.75, cdf_threshold=0.6, chunk_3d_shape_q=list(chunk), chunk_3d_shape_k=list(chunk))
    o = bi.flash_attn_bsa_3d(q, k, v, shape, shape, **prm)
    o.backward(do)
    with torch.no_grad():
        o_plain, idx, lens, _ = bi._bsa_3d(q, k, v, shape, shape, 0.75, chunk, chunk, want_selection=True, cdf_threshold=0.6)
    assert torch.equal(o.detach(), o_plain)
    lens_c = lens.cpu()
    assert int(lens_c.min()) < int(lens_c.max())                          # the rule did give lists of unequal length
    qp, kp, vp, dop = (O.rearrange_thw_to_3d_block(t.detach().cpu(), shape, chunk) for t in (q, k, v, do))
    nb = qp.shape[2] // 64
    mask = O.block_mask_from_indices(idx.cpu().long().clamp(min=0), lens_c, nb)
    valid = torch.from_numpy(O.slot_validity(shape, chunk))
    wq, wk, wv = O.masked_dense_attention_autograd(qp, kp, vp, dop, mask, 64, 64, 1 / math.sqrt(128), key_valid=valid)
    for t, w in zip((q, k, v), (wq, wk, wv)):
        w_thw = O.rearrange_3d_block_to_thw(w, shape, chunk)
        err = (t.grad.cpu().float() - w_thw).abs()
        assert float(err.max()) <= 2.0 ** -6 * 4 * float(w_thw.abs().max()), float(err.max())
        assert float(err.mean()) <= 2.0 ** -6 * float(w_thw.abs().mean())


@pytest.mark.parametrize("dtype,lq,lk,chunk_q,chunk_k,token_major", [
    (torch.bfloat16, (8, 8, 16), (8, 8, 16), (4, 4, 4), (4, 4, 4), False),      # no padding
    (torch.bfloat16, (6, 10, 13), (6, 10, 13), (4, 4, 4), (4, 4, 4), True),     # padding on all axes, views of a projection
    (torch.float16, (5, 9, 14), (5, 9, 14), (4, 4, 4), (4, 4, 4), False),
    (torch.bfloat16, (4, 8, 12), (8, 8, 12), (4, 4, 4), (4, 4, 8), False),      # fewer queries than keys, 128-token key chunks
    (torch.bfloat16, (7, 9, 17), (7, 9, 17), (4, 4, 8), (4, 4, 8), True),
])
def test_the_token_order_backward_equals_the_rearranging_route(dtype, lq, lk, chunk_q, chunk_k, token_major):
    """bsa_bwd_3d reads o, dO, lse and k through the row tables and stores the gradients at their tokens; five
    rearrangements (bsa_interface.py:650-652 and their like), bsa_bwd and three rearrangements back run the same kernels on
    the same values, so the two must agree bit for bit - on padded grids, strided views, two batches."""
    bi = I()
    B, H = 2, 3
    Sq, Sk = int(np.prod(lq)), int(np.prod(lk))
    g = torch.Generator().manual_seed(11)
    if token_major and Sq == Sk:
        qkv = torch.randn(B, Sq, 3, H, 128, generator=g).to(dtype).cuda()
        q, k, v = qkv.permute(2, 0, 3, 1, 4).unbind(0)
    else:
        q = torch.randn(B, H, Sq, 128, generator=g).to(dtype).cuda()
        k, v = (torch.randn(B, H, Sk, 128, generator=g).to(dtype).cuda() for _ in range(2))
    do = torch.randn(B, Sq, H, 128, generator=g).to(dtype).cuda().transpose(1, 2)          # a view, as a reshape upstream leaves it
    o, walk, lens, lse = bi._bsa_3d(q, k, v, lq, lk, 0.5, chunk_q, chunk_k, for_backward=True)
    args = (do, q, k, v, o, lse, walk, lens, lq, lk, chunk_q, chunk_k, 1 / math.sqrt(128))
    got = bi._bsa_3d_backward(*args)
    want = bi._bsa_3d_backward_by_rearranging(*args)
    for a, b, name in zip(got, want, ("dq", "dk", "dv")):
        assert a.shape == b.shape and a.is_contiguous()
        assert torch.isfinite(a.float()).all(), name
        assert torch.equal(a, b), (name, float((a.float() - b.float()).abs().max()))
    again = bi._bsa_3d_backward(*args)
    for a, b in zip(got, again):
        assert torch.equal(a, b)


@pytest.mark.parametrize("seed", range(8))
def test_random_grids_through_both_backward_routes(seed):
    """Random grids, chunk shapes, batch and head counts, selection rules and storage types: bsa_bwd_3d against the
    rearranging route, bit for bit, and both finite."""
    bi = I()
    rnd = np.random.default_rng(100 + seed)
    chunk_q = [(4, 4, 4), (2, 4, 8), (4, 4, 8), (1, 8, 8)][rnd.integers(0, 4)]
    chunk_k = [(4, 4, 4), (2, 4, 8), (4, 4, 8)][rnd.integers(0, 3)]
    lq = tuple(int(rnd.integers(c, 4 * c + 2)) for c in chunk_q)
    lk = lq if rnd.integers(0, 2) else tuple(int(rnd.integers(c, 4 * c + 2)) for c in chunk_k)
    B, H = int(rnd.integers(1, 3)), int(rnd.integers(1, 4))
    dtype = [torch.bfloat16, torch.float16][rnd.integers(0, 2)]
    sparsity = [0.0, 0.5, 0.8][rnd.integers(0, 3)]
    cdf = None if rnd.integers(0, 3) else 0.7
    g = torch.Generator().manual_seed(200 + seed)
    Sq, Sk = int(np.prod(lq)), int(np.prod(lk))
    q = torch.randn(B, H, Sq, 128, generator=g).to(dtype).cuda()
    k, v = (torch.randn(B, H, Sk, 128, generator=g).to(dtype).cuda() for _ in range(2))
    do = torch.randn(B, H, Sq, 128, generator=g).to(dtype).cuda()
    o, walk, lens, lse = bi._bsa_3d(q, k, v, lq, lk, sparsity, chunk_q, chunk_k, cdf_threshold=cdf, for_backward=True)
    if walk.shape[3] == 0:
        pytest.skip("no block selected at this size")
    args = (do, q, k, v, o, lse, walk, lens, lq, lk, chunk_q, chunk_k, 1 / math.sqrt(128))
    got = bi._bsa_3d_backward(*args)
    want = bi._bsa_3d_backward_by_rearranging(*args)
    for a, b, name in zip(got, want, ("dq", "dk", "dv")):
        assert torch.isfinite(a.float()).all(), (name, lq, lk, chunk_q, chunk_k)
        assert torch.equal(a, b), (name, lq, lk, chunk_q, chunk_k, float((a.float() - b.float()).abs().max()))


def test_argument_checks():
    from longcat_video_amd import _capi
    lib = _capi.load()
    assert lib.bsa_bwd_workspace_bytes(1, 2, 640, 640, 128, 64, 64, 5, _capi.BSA_BF16) > 2 * 640 * 128 * 2          # the scaled K and the small tables
    assert lib.bsa_bwd_workspace_bytes(1, 2, 640, 640, 128, 64, 64, 5, _capi.BSA_F32) == 0          # 16-bit types only
    assert lib.bsa_bwd_workspace_bytes(1, 2, 640, 650, 128, 64, 64, 5, _capi.BSA_BF16) == 0
    t = torch.zeros(1, 1, 64, 128, dtype=torch.bfloat16, device="cuda")
    f = torch.zeros(1, 1, 64, dtype=torch.float32, device="cuda")
    i = torch.zeros(1, 1, 1, 1, dtype=torch.int32, device="cuda")
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    p = lambda x: x.data_ptr()
    args = [p(t)] * 5 + [p(f), p(i), p(i), None] + [p(t)] * 3
    assert lib.bsa_bwd(*args, 1, 1, 64, 64, 128, 64, 64, 1, 0.1, _capi.BSA_BF16, p(ws), 16, None) == _capi.BSA_ERR_WORKSPACE
    assert lib.bsa_bwd(*args, 1, 1, 64, 64, 96, 64, 64, 1, 0.1, _capi.BSA_BF16, p(ws), 1 << 20, None) == _capi.BSA_ERR_UNSUPPORTED
    args[0] = None
    assert lib.bsa_bwd(*args, 1, 1, 64, 64, 128, 64, 64, 1, 0.1, _capi.BSA_BF16, p(ws), 1 << 20, None) == _capi.BSA_ERR_BAD_ARG
    # the token-order entry point
    import ctypes as C
    prm = _capi.Bsa3dParams(1, 1, 128, _capi.BSA_BF16, 4, 4, 4, 4, 4, 4, 4, 4, 4, 4, 4, 4, 0, 0.1, 0.0)
    need = lib.bsa_bwd_3d_workspace_bytes(C.byref(prm), 1)
    assert need > 3 * 64 * 128 * 2
    bad = _capi.Bsa3dParams(1, 1, 128, _capi.BSA_F32, 4, 4, 4, 4, 4, 4, 4, 4, 4, 4, 4, 4, 0, 0.1, 0.0)
    assert lib.bsa_bwd_3d_workspace_bytes(C.byref(bad), 1) == 0
    assert lib.bsa_bwd_3d_workspace_bytes(C.byref(prm), 0) == 0
    st = _capi.strides3((64 * 128, 64 * 128, 128))
    call = lambda first, ws_bytes: lib.bsa_bwd_3d(C.byref(prm), first, st, p(t), st, p(t), st, p(t), st, p(t), st, p(f), p(i), p(i), 1,
                                                  p(t), st, p(t), st, p(t), st, p(ws), ws_bytes, None)
    assert call(p(t), 16) == _capi.BSA_ERR_WORKSPACE
    assert call(None, 1 << 20) == _capi.BSA_ERR_BAD_ARG

"""Pins the oracle's restatement of the reference backward (blockwise_attention_backward, inverse_block_lists)
against an independent derivation: torch.autograd through an fp32 masked-dense softmax attention."""
import math

import numpy as np
import pytest
import torch

from oracle import bsa_oracle as O


def case(seed, H, nbq, nbk, width, dtype, bs=64, D=128, scale_in=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(1, H, nbq * bs, D, generator=g) * scale_in).to(dtype)
    k = (torch.randn(1, H, nbk * bs, D, generator=g) * scale_in).to(dtype)
    v = torch.randn(1, H, nbk * bs, D, generator=g).to(dtype)
    do = torch.randn(1, H, nbq * bs, D, generator=g).to(dtype)
    idx = torch.stack([torch.randperm(nbk, generator=g)[:width] for _ in range(H * nbq)]).view(1, H, nbq, width)
    lens = torch.randint(0, width + 1, (1, H, nbq), generator=g, dtype=torch.int32)
    lens[0, :, 0] = width
    return q, k, v, do, idx, lens


def test_inverse_lists_against_a_loop():
    _, _, _, _, idx, lens = case(1, 2, 5, 7, 4, torch.float32)
    inv, n = O.inverse_block_lists(idx, lens, 7)
    for h in range(2):
        for j in range(7):
            want = [m for m in range(5) if j in idx[0, h, m, :int(lens[0, h, m])].tolist()]
            assert inv[0, h, j, :int(n[0, h, j])].tolist() == want and int(n[0, h, j]) == len(want)
            assert torch.all(inv[0, h, j, int(n[0, h, j]):] == 5)


@pytest.mark.parametrize("with_padding", [False, True])
def test_fp32_backward_equals_autograd_to_rounding(with_padding):
    sm = 1 / math.sqrt(128)
    q, k, v, do, idx, lens = case(2, 2, 3, 6, 3, torch.float32)
    valid = None
    if with_padding:
        valid = torch.ones(6 * 64, dtype=torch.bool)
        valid[64 * 2 + 40:64 * 3] = False
        valid[-64:] = False                                  # a KV block with no real key
    mask = O.block_mask_from_indices(idx, lens, 6)
    o, lse = O.masked_dense_attention(q, k, v, mask, 64, 64, sm, key_valid=valid)
    dq, dk, dv = O.blockwise_attention_backward(q, k, v, o, do, lse, idx, lens, 64, 64, sm, key_valid=valid)
    wq, wk, wv = O.masked_dense_attention_autograd(q, k, v, do, mask, 64, 64, sm, key_valid=valid)
    for got, want in ((dq, wq), (dk, wk), (dv, wv)):
        assert torch.allclose(got, want, rtol=2e-4, atol=2e-5), float((got - want).abs().max())
    if with_padding:
        assert torch.all(dk[0, :, ~valid] == 0) and torch.all(dv[0, :, ~valid] == 0)
    # rows with an empty list: no gradient into q
    empty = (lens[0] == 0).repeat_interleave(64, dim=-1)
    assert torch.all(dq[0][empty] == 0)


@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, 2.0 ** -6), (torch.float16, 2.0 ** -9)])
def test_16_bit_backward_is_within_its_roundings_of_autograd(dtype, tol):
    sm = 1 / math.sqrt(128)
    q, k, v, do, idx, lens = case(3, 2, 4, 8, 3, dtype)
    mask = O.block_mask_from_indices(idx, lens, 8)
    o32, lse = O.masked_dense_attention(q, k, v, mask, 64, 64, sm)
    o = o32.to(dtype)
    dq, dk, dv = O.blockwise_attention_backward(q, k, v, o, do, lse, idx, lens, 64, 64, sm)
    assert dq.dtype == dtype
    wq, wk, wv = O.masked_dense_attention_autograd(q, k, v, do, mask, 64, 64, sm)
    for got, want in ((dq, wq), (dk, wk), (dv, wv)):
        err = (got.float() - want).abs()
        # a few roundings of p, ds, k_s and the result: relative to the gradient's own scale
        assert float(err.max()) <= tol * float(want.abs().max()) * 4, float(err.max())
        assert float(err.mean()) <= tol * float(want.abs().mean())


def test_finite_differences_on_a_tiny_case():
    sm = 0.3
    g = torch.Generator().manual_seed(4)
    q = torch.randn(1, 1, 64, 128, generator=g, dtype=torch.float64)
    k = torch.randn(1, 1, 128, 128, generator=g, dtype=torch.float64)
    v = torch.randn(1, 1, 128, 128, generator=g, dtype=torch.float64)
    do = torch.randn(1, 1, 64, 128, generator=g, dtype=torch.float64)
    idx = torch.tensor([[[[1, 0]]]])
    lens = torch.tensor([[[2]]], dtype=torch.int32)

    def loss(qq, kk, vv):
        p = torch.softmax((qq @ kk.transpose(-1, -2)) * sm, dim=-1)
        return ((p @ vv) * do).sum()

    o = torch.softmax((q @ k.transpose(-1, -2)) * sm, dim=-1) @ v
    lse = torch.logsumexp((q @ k.transpose(-1, -2)) * sm, dim=-1)
    dq, dk, dv = O.blockwise_attention_backward(q.float(), k.float(), v.float(), o.float(), do.float(), lse.float(), idx, lens, 64, 64, sm)
    eps = 1e-5
    rng = np.random.default_rng(5)
    for which, grad, t in (("q", dq, q), ("k", dk, k), ("v", dv, v)):
        for _ in range(5):
            pos = tuple(int(rng.integers(0, n)) for n in t.shape)
            tp, tm = t.clone(), t.clone()
            tp[pos] += eps
            tm[pos] -= eps
            args_p = {"q": (tp, k, v), "k": (q, tp, v), "v": (q, k, tp)}[which]
            args_m = {"q": (tm, k, v), "k": (q, tm, v), "v": (q, k, tm)}[which]
            fd = float((loss(*args_p) - loss(*args_m)) / (2 * eps))
            assert abs(float(grad[pos]) - fd) <= 2e-4 * max(1.0, abs(fd)), (which, pos, float(grad[pos]), fd)


def test_block_subsets_equal_the_rows_of_the_full_evaluation():
    """q_blocks / kv_blocks: the named rows bit for bit as in the full evaluation (same pairs, same order), every other
    row zero; the query blocks of a KV block found column by column are those of inverse_block_lists."""
    sm = 1 / math.sqrt(128)
    q, k, v, do, idx, lens = case(6, 2, 7, 9, 4, torch.bfloat16)
    mask = O.block_mask_from_indices(idx, lens, 9)
    o32, lse = O.masked_dense_attention(q, k, v, mask, 64, 64, sm)
    o = o32.bfloat16()
    full = O.blockwise_attention_backward(q, k, v, o, do, lse, idx, lens, 64, 64, sm)
    qb, kb = [0, 5, 6], [2, 8]
    part = O.blockwise_attention_backward(q, k, v, o, do, lse, idx, lens, 64, 64, sm, q_blocks=qb, kv_blocks=kb)
    rows = lambda blocks, n: torch.isin(torch.arange(n * 64) // 64, torch.tensor(blocks))
    rq, rk = rows(qb, 7), rows(kb, 9)
    assert torch.equal(part[0][:, :, rq], full[0][:, :, rq]) and torch.all(part[0][:, :, ~rq] == 0)
    for got, want in ((part[1], full[1]), (part[2], full[2])):
        assert torch.equal(got[:, :, rk], want[:, :, rk]) and torch.all(got[:, :, ~rk] == 0)
    assert float(full[1][:, :, rk].abs().max()) > 0              # the sampled KV blocks were selected by someone
    # an empty subset computes nothing
    none = O.blockwise_attention_backward(q, k, v, o, do, lse, idx, lens, 64, 64, sm, q_blocks=[], kv_blocks=[])
    assert all(torch.all(t == 0) for t in none)

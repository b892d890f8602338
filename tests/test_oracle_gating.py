"""Pins the oracle's gating functions (R2-R4): pooling, scores, k_sel, top-k,
block mask."""
import numpy as np
import pytest
import torch

from oracle import bsa_oracle as O


def test_pool_closed_form_on_representable_inputs():
    # rows of block b are all (b+1): the mean is b+1 exactly, in any dtype
    x = torch.arange(1, 5).repeat_interleave(64).view(1, 1, 256, 1).expand(1, 2, 256, 8).contiguous()
    for dt in (torch.float32, torch.bfloat16, torch.float16):
        p = O.mean_pooling_compression(x.to(dt), 64)
        assert p.dtype == dt and p.shape == (1, 2, 4, 8)
        assert torch.equal(p.float(), torch.arange(1, 5).float().view(1, 1, 4, 1).expand(1, 2, 4, 8))


def test_pool_ragged_tail_divides_by_block_size():
    x = torch.ones(1, 1, 96, 4)
    p = O.mean_pooling_compression(x, 64)
    assert p.shape == (1, 1, 2, 4)
    assert torch.equal(p[0, 0, 0], torch.ones(4)) and torch.equal(p[0, 0, 1], torch.full((4,), 0.5))


def test_pool_rounds_once_from_fp32():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(1, 1, 128, 16, generator=g).bfloat16()
    want = x.double().view(1, 1, 2, 64, 16).mean(3)
    got = O.mean_pooling_compression(x, 64)
    # one bf16 rounding of the exact mean: at most half an ulp (2^-9 relative) away
    assert torch.all((got.double() - want).abs() <= want.abs() * 2.0 ** -8 + 1e-30)


def test_score_exact_on_integer_inputs_and_unscaled():
    g = torch.Generator().manual_seed(2)
    q = torch.randint(-3, 4, (1, 2, 5, 128), generator=g).float()
    k = torch.randint(-3, 4, (1, 2, 7, 128), generator=g).float()
    want = torch.einsum("bhmd,bhnd->bhmn", q.double(), k.double())
    for dt in (torch.float32, torch.bfloat16):
        got = O.cal_score(q.to(dt), k.to(dt))
        assert got.shape == (1, 2, 5, 7) and got.dtype == dt
        assert torch.equal(got.double(), want.to(dt).double())     # no 1/sqrt(D) anywhere


@pytest.mark.parametrize("sparsity,n,want", [
    (0.875, 8, 1), (0.9375, 1440, 90), (0.9375, 624, 39), (0.875, 1248, 156), (0.875, 312, 39),
    (0.5, 4, 2), (0.9, 10, 0),          # (1-0.9)*10 = 0.9999999999999998 truncates to 0
    (0.0, 7, 7), (1.0, 7, 0), (0.3, 10, 7),
])
def test_num_selected_is_the_literal_expression(sparsity, n, want):
    assert O.num_selected(sparsity, n) == want == int((1 - sparsity) * n)


def brute_topk(row, k):
    return sorted(range(len(row)), key=lambda i: (-row[i], i))[:k]


def test_topk_brute_force_with_heavy_ties():
    g = torch.Generator().manual_seed(3)
    score = torch.randint(-2, 3, (2, 2, 6, 37), generator=g).float().bfloat16()   # 5 distinct values
    idx, lens = O.select_topk(score, 9)
    assert idx.dtype == torch.int64 and lens.dtype == torch.int32 and torch.all(lens == 9)
    s = score.float().numpy()
    for b in range(2):
        for h in range(2):
            for m in range(6):
                assert idx[b, h, m].tolist() == brute_topk(s[b, h, m].tolist(), 9)


def test_topk_values_equal_torch_topk_values():
    g = torch.Generator().manual_seed(4)
    score = torch.randn(1, 3, 11, 200, generator=g).bfloat16()
    idx, _ = O.select_topk(score, 25)
    got = torch.gather(score.float(), -1, idx)
    want = torch.topk(score.float(), 25).values
    assert torch.equal(got, want)      # descending, same multiset whatever torch's tie order


def test_topk_signed_zero_ties_and_edges():
    score = torch.tensor([[[[0.0, -0.0, 1.0, -0.0, 0.0]]]])
    idx, _ = O.select_topk(score, 3)
    assert idx.flatten().tolist() == [2, 0, 1]
    idx0, lens0 = O.select_topk(score, 0)
    assert idx0.shape == (1, 1, 1, 0) and int(lens0) == 0
    idx5, _ = O.select_topk(score, 5)
    assert idx5.flatten().tolist() == [2, 0, 1, 3, 4]
    with pytest.raises(ValueError):
        O.select_topk(torch.tensor([[[[0.0, float("nan")]]]]), 1)


def test_block_mask_brute_force():
    g = torch.Generator().manual_seed(5)
    idx = torch.stack([torch.randperm(9, generator=g)[:4] for _ in range(2 * 3)]).view(1, 2, 3, 4)
    lens = torch.tensor([[[4, 2, 0], [1, 4, 3]]], dtype=torch.int32)
    mask = O.block_mask_from_indices(idx, lens, 9)
    for h in range(2):
        for m in range(3):
            want = torch.zeros(9, dtype=torch.bool)
            for j in range(int(lens[0, h, m])):
                want[idx[0, h, m, j]] = True
            assert torch.equal(mask[0, h, m], want)


# ---------------------------------------------------------------------------
# selection by cumulative attention mass (bsa_interface.py:233-266)
# ---------------------------------------------------------------------------
def test_cdf_rule_closed_forms():
    # equal scores: equal weights 1/n, cdf_j = j/n, ties in index order
    score = torch.zeros(1, 1, 2, 8)
    idx, lens, cdf = O.select_cdf(score, 0.5, 0.3)
    assert torch.equal(idx[0, 0, 0], torch.arange(8)) and lens.tolist() == [[[4, 4]]]
    assert torch.allclose(cdf[0, 0, 0], torch.arange(1, 9).double() / 8)
    # one dominant column outweighs the threshold alone: nothing is kept, unless a minimum is asked for
    score = torch.tensor([[[[0.0, 50.0, 1.0, 2.0]]]])
    idx, lens, _ = O.select_cdf(score, 0.9, 1.0)
    assert idx[0, 0, 0].tolist() == [1, 3, 2, 0] and int(lens) == 0
    assert int(O.select_cdf(score, 0.9, 1.0, k_min=2)[1]) == 2
    # a threshold above one keeps every column; cap limits it
    assert int(O.select_cdf(score, 1.5, 1.0)[1]) == 4 and int(O.select_cdf(score, 1.5, 1.0, cap=3)[1]) == 3
    # two columns of weight 1/4 each and one of 1/2: log-weights as scores with scale 1
    score = torch.log(torch.tensor([[[[0.25, 0.5, 0.25]]]]))
    assert int(O.select_cdf(score, 0.5, 1.0)[1]) == 1 and int(O.select_cdf(score, 0.76, 1.0)[1]) == 2
    assert O.select_cdf(score, 0.76, 1.0)[0][0, 0, 0].tolist() == [1, 0, 2]


def test_cdf_rule_against_a_python_loop_and_the_library_pipeline():
    g = torch.Generator().manual_seed(7)
    score = torch.randn(2, 3, 5, 37, generator=g) * 3
    thr, scale = 0.8, 0.7
    idx, lens, cdf = O.select_cdf(score, thr, scale)
    for b, h, m in [(0, 0, 0), (1, 2, 4), (0, 1, 3)]:
        row = score[b, h, m].tolist()
        order = sorted(range(37), key=lambda j: (-row[j], j))
        mx = max(row)
        e = [float(np.float32(np.exp(np.float32((row[j] - mx) * scale)))) for j in order]
        z = sum(e)
        run, n = 0.0, 0
        for x in e:
            run += x / z
            if run <= thr:
                n += 1
        assert idx[b, h, m].tolist() == order
        assert abs(int(lens[b, h, m]) - n) <= (1 if min(abs(c - thr) for c in cdf[b, h, m].tolist()) < 1e-5 else 0)
    # the reference's own sequence of library calls (bsa:234-241) on tie-free fp32 scores
    weights = torch.softmax(score * scale, dim=-1)
    ws = torch.sort(weights, dim=-1, descending=True)
    ref_cdf = torch.cumsum(ws.values, dim=-1)
    ref_n = torch.searchsorted(ref_cdf, torch.full(score.shape[:3] + (1,), thr), right=True).squeeze(-1)
    clear = (cdf - thr).abs().min(-1).values > 1e-5
    assert clear.float().mean() > 0.9
    assert torch.equal(ref_n[clear], lens.long()[clear])
    assert torch.equal(ws.indices, idx)
    # cdf + top-k: never fewer than the top-k count
    lens2 = O.select_cdf(score, thr, scale, k_min=9)[1]
    assert torch.equal(lens2, torch.clamp(lens, min=9))

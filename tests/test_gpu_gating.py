"""R2-R4 on the GPU: pooled scores and top-k selection.  Selection is bit-exact
against the oracle's (-score, index) order given the same scores."""
import numpy as np
import pytest
import torch

from oracle import bsa_oracle as O

pytestmark = pytest.mark.gpu


def I():
    from longcat_video_amd.block_sparse_attention import bsa_interface
    return bsa_interface


def topk_gpu(score, k_sel, sorted_too=False):
    """Calls the C-ABI top-k directly with an explicit k_sel."""
    from longcat_video_amd import _capi
    B, H, nbq, nbk = score.shape
    s = score.cuda().contiguous()
    idx = torch.full((B * H * nbq * max(k_sel, 1),), -7, dtype=torch.int32, device="cuda")
    lens = torch.empty(B, H, nbq, dtype=torch.int32, device="cuda")
    code = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}[score.dtype]
    srt = torch.full_like(idx, -7) if sorted_too else None
    _capi.check(_capi.load().bsa_topk_from_score(s.data_ptr(), idx.data_ptr(), None if srt is None else srt.data_ptr(),
                                                  lens.data_ptr(), B, H, nbq, nbk, k_sel, code,
                                                  torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    out = idx[: B * H * nbq * k_sel].view(B, H, nbq, k_sel).cpu().long()
    if sorted_too:
        return out, lens.cpu(), srt[: B * H * nbq * k_sel].view(B, H, nbq, k_sel).cpu().long()
    return out, lens.cpu()


def test_score_exact_on_integer_inputs():
    g = torch.Generator().manual_seed(1)
    q = torch.randint(-3, 4, (1, 2, 70, 128), generator=g).float()
    k = torch.randint(-3, 4, (1, 2, 131, 128), generator=g).float()
    for dt in (torch.bfloat16, torch.float16, torch.float32):
        got = I().cal_score(q.to(dt).cuda(), k.to(dt).cuda()).cpu()
        assert torch.equal(got, O.cal_score(q.to(dt), k.to(dt)))


@pytest.mark.parametrize("dtype,ulp", [(torch.bfloat16, 2.0 ** -7), (torch.float16, 2.0 ** -10), (torch.float32, 2.0 ** -20)])
def test_score_random_within_one_ulp(dtype, ulp):
    g = torch.Generator().manual_seed(2)
    q = torch.randn(2, 3, 97, 128, generator=g).to(dtype)
    k = torch.randn(2, 3, 160, 128, generator=g).to(dtype)
    got = I().cal_score(q.cuda(), k.cuda()).cpu().float()
    want64 = torch.einsum("bhmd,bhnd->bhmn", q.double(), k.double())
    assert torch.all((got.double() - want64).abs() <= want64.abs() * ulp + 1e-4)


@pytest.mark.parametrize("nbq,nbk,k_sel", [(4, 4, 2), (5, 37, 9), (3, 64, 64), (2, 65, 1), (7, 200, 0), (3, 624, 39),
                                             (2, 1440, 90), (2, 1248, 156), (1, 2047, 300), (1, 4096, 1024), (5, 4096, 3000)])
def test_topk_bit_exact_with_ties(nbq, nbk, k_sel):
    g = torch.Generator().manual_seed(nbk)
    # few distinct values => many exact ties, resolved towards the lowest index
    score = (torch.randint(-6, 7, (1, 2, nbq, nbk), generator=g).float() / 4).bfloat16()
    got, lens = topk_gpu(score, k_sel)
    want, want_lens = O.select_topk(score, k_sel)
    assert torch.equal(lens, want_lens)
    assert torch.equal(got, want)


def topk_block_order_only_gpu(score, k_sel):
    """The C-ABI top-k asked for the ascending-block-order list alone (what the operator asks for): for 16-bit scores
    with a multiple of 8 columns this takes the kernel that holds 8 consecutive columns per lane."""
    from longcat_video_amd import _capi
    B, H, nbq, nbk = score.shape
    s = score.cuda().contiguous()
    srt = torch.full((B * H * nbq * max(k_sel, 1),), -7, dtype=torch.int32, device="cuda")
    lens = torch.empty(B, H, nbq, dtype=torch.int32, device="cuda")
    code = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}[score.dtype]
    _capi.check(_capi.load().bsa_topk_from_score(s.data_ptr(), None, srt.data_ptr(), lens.data_ptr(), B, H, nbq, nbk, k_sel, code,
                                                  torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return srt[: B * H * nbq * k_sel].view(B, H, nbq, k_sel).cpu().long(), lens.cpu()


@pytest.mark.parametrize("nbq,nbk,k_sel", [(4, 8, 2), (5, 40, 9), (3, 64, 64), (7, 200, 0), (3, 624, 39), (2, 520, 17), (2, 512, 511),
                                             (2, 1440, 90), (2, 1248, 156), (1, 2048, 300), (3, 2056, 1500), (1, 4096, 1024),
                                             (5, 4096, 3000), (2, 3080, 77), (3, 37, 9), (2, 585, 36)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_topk_block_order_list_alone(nbq, nbk, k_sel, dtype):
    g = torch.Generator().manual_seed(nbk + k_sel)
    # few distinct values => ties that the selection has to cut at the lowest indices; then plain random scores
    for score in ((torch.randint(-6, 7, (1, 2, nbq, nbk), generator=g).float() / 4).to(dtype),
                  torch.randn(1, 2, nbq, nbk, generator=g).to(dtype)):
        got, lens = topk_block_order_only_gpu(score, k_sel)
        want, want_lens = O.select_topk(score, k_sel)
        assert torch.equal(lens, want_lens)
        assert torch.equal(got, torch.sort(want, dim=-1).values)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_topk_random_scores_all_dtypes(dtype):
    g = torch.Generator().manual_seed(7)
    score = torch.randn(2, 2, 9, 333, generator=g).to(dtype)
    got, _ = topk_gpu(score, 41)
    want, _ = O.select_topk(score, 41)
    assert torch.equal(got, want)
    vals = torch.gather(score.float(), -1, got)
    assert torch.equal(vals, torch.topk(score.float(), 41).values)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_topk_rows_on_both_sides_of_the_histogram_window(dtype):
    """For 16-bit scores the kernel first looks for the k-th largest value within 254 codes below the row maximum
    (a histogram) and otherwise searches bit by bit.  Rows built from bit patterns so that the k-th largest value
    lies 0, 1, 253, 254, 255, 256 and thousands of codes below the maximum, with ties at the threshold, across
    zero, and with a maximum so small that its distance to the padding code would fit the window."""
    nbk, k = 333, 20
    base = 0x3C00 if dtype == torch.float16 else 0x3F80          # 1.0
    rows = []
    for gap in (0, 1, 253, 254, 255, 256, 5000):
        codes = np.full(nbk, base - gap - 300, dtype=np.int64)       # the crowd, far below
        codes[5:5 + k - 4] = base                                    # k - 4 columns at the maximum
        codes[100:110] = base - gap                                  # ten tied columns of which four win (lowest index)
        rows.append(codes)
    # positive and negative values around zero: codes of -x sort below every positive code
    mixed = np.full(nbk, 0x8000 | (base - 7), dtype=np.int64)        # about -1
    mixed[::17] = 3                                                  # tiny positives: the winners, all tied
    rows.append(mixed)
    # a row of tiny values: maximum = code 2 (a denormal), the rest zero or negative zero
    tiny = np.zeros(nbk, dtype=np.int64)
    tiny[50] = 2
    tiny[51::3] = 0x8000
    rows.append(tiny)
    bits = torch.from_numpy(np.stack(rows).astype(np.uint16).view(np.int16))
    score = bits.view(dtype).view(1, 1, len(rows), nbk)
    for kk in (k, 1, 150):
        got, lens = topk_gpu(score, kk)
        want, want_lens = O.select_topk(score, kk)
        assert torch.equal(lens, want_lens)
        assert torch.equal(got, want), kk


def test_topk_long_lists_of_fp32_scores():
    """2 500 of 4 096 columns of fp32 scores in score order: the ranking keeps 64-bit keys of four rows in LDS,
    more than the 64 KB a kernel gets without asking."""
    g = torch.Generator().manual_seed(13)
    score = torch.randn(1, 1, 6, 4096, generator=g)
    score[0, 0, 2] = (score[0, 0, 2] * 4).round() / 4                  # a row full of ties
    got, lens = topk_gpu(score, 2500)
    want, want_lens = O.select_topk(score, 2500)
    assert torch.equal(lens, want_lens) and torch.equal(got, want)


def test_block_ordered_list_is_the_same_set_in_ascending_order():
    g = torch.Generator().manual_seed(8)
    score = (torch.randint(-6, 7, (1, 2, 5, 700), generator=g).float() / 4).bfloat16()
    got, _, srt = topk_gpu(score, 77, sorted_too=True)
    assert torch.equal(torch.sort(got, dim=-1).values, srt)
    idx_b, lens_b, _ = I()._score_topk(torch.randn(1, 2, 9, 128, generator=g).bfloat16().cuda(),
                                       torch.randn(1, 2, 300, 128, generator=g).bfloat16().cuda(), 40, order="block")
    assert torch.all(idx_b[..., 1:] > idx_b[..., :-1]) and torch.all(lens_b == 40)


def test_topk_special_values():
    inf = float("inf")
    row = torch.tensor([0.0, -0.0, 1.0, -inf, inf, -0.0, 0.0, -1.0, inf, 3.0])
    for dt in (torch.bfloat16, torch.float32):
        score = row.to(dt).view(1, 1, 1, -1)
        for k in (1, 3, 6, 10):
            got, _ = topk_gpu(score, k)
            want, _ = O.select_topk(score, k)
            assert got.flatten().tolist() == want.flatten().tolist()


def test_topk_special_values_block_order_list_alone():
    inf = float("inf")
    row = torch.tensor([0.0, -0.0, 1.0, -inf, inf, -0.0, 0.0, -1.0, inf, 3.0, 2.0, -2.0, 0.0, -0.0, 5.0, -inf])
    for dt in (torch.bfloat16, torch.float16):
        score = row.to(dt).view(1, 1, 1, -1)
        for k in (1, 3, 6, 10, 16):
            got, _ = topk_block_order_only_gpu(score, k)
            want, _ = O.select_topk(score, k)
            assert got.flatten().tolist() == sorted(want.flatten().tolist())


def test_score_topk_pipeline_matches_oracle_given_gpu_scores():
    g = torch.Generator().manual_seed(9)
    qc = torch.randn(1, 4, 312, 128, generator=g).bfloat16() * 0.2
    kc = torch.randn(1, 4, 1248, 128, generator=g).bfloat16() * 0.2
    idx, lens, score = I()._score_topk(qc.cuda(), kc.cuda(), 156)      # rectangular, config-4 noise shape
    want, _ = O.select_topk(score.cpu(), 156)
    assert torch.equal(idx.cpu().long(), want) and torch.all(lens.cpu() == 156)
    idx64, lens2 = I().get_select_indices_topk(qc.cuda(), kc.cuda(), 0.875)
    assert idx64.dtype == torch.int64 and torch.equal(idx64.cpu(), want)


def test_full_size_720p_selection():
    """32 heads x 1440 x 1440 bf16 scores: every row has k_sel distinct indices, the
    selected values are exactly torch.topk's values, and sampled heads are
    bit-exact against the oracle."""
    g = torch.Generator(device="cuda").manual_seed(11)
    qc = torch.randn(1, 32, 1440, 128, generator=g, device="cuda").bfloat16() * 0.125
    kc = torch.randn(1, 32, 1440, 128, generator=g, device="cuda").bfloat16() * 0.125
    idx, lens, score = I()._score_topk(qc, kc, 90)
    assert torch.all(lens == 90)
    srt = torch.sort(idx.long(), dim=-1).values
    assert torch.all(srt[..., 1:] > srt[..., :-1]) and int(srt.min()) >= 0 and int(srt.max()) < 1440
    vals = torch.gather(score.float(), -1, idx.long())
    assert torch.equal(vals, torch.topk(score.float(), 90).values)
    for h in (0, 13, 31):
        want, _ = O.select_topk(score[:, h:h + 1].cpu(), 90)
        assert torch.equal(idx[:, h:h + 1].cpu().long(), want)
    idx2, _, _ = I()._score_topk(qc, kc, 90)
    assert torch.equal(idx, idx2)


# ---------------------------------------------------------------------------
# selection by cumulative attention mass (bsa_interface.py:226-266)
# ---------------------------------------------------------------------------
def check_cdf_selection(score, idx, lens, thr, scale, k_min=0):
    """idx/lens from the GPU against the oracle on the same scores: the count may only differ where the
    running sum comes within rounding of the threshold; given the count, the list is the oracle's order."""
    nbk = score.shape[-1]
    cap = nbk                                           # a row may keep every block
    want_idx, want_lens, cdf = O.select_cdf(score, thr, scale, k_min=k_min, cap=cap)
    lens = lens.cpu().long()
    near = (cdf - float(np.float32(thr))).abs().min(-1).values < 1e-5
    assert torch.equal(lens[~near], want_lens.long()[~near])
    assert (lens - want_lens.long()).abs().max() <= 1
    assert near.float().mean() < 0.05
    idx = idx.cpu().long()
    assert idx.shape[-1] == cap
    pos = torch.arange(cap).expand_as(idx)
    used = pos < lens.unsqueeze(-1)
    assert torch.equal(idx[used], want_idx[..., :cap][used])
    assert torch.all(idx[~used] == -1)
    return lens


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_cdf_selection_from_score(dtype):
    g = torch.Generator().manual_seed(21)
    score = (torch.randn(1, 2, 33, 200, generator=g) * 4).to(dtype)
    for thr, scale in [(0.5, 1.0), (0.9, 0.25), (0.999, 0.0883883)]:
        idx, lens = I().get_select_indices_cdf_from_score(score.cuda(), thr, scale)
        assert idx.dtype == torch.int64 and lens.dtype == torch.int32
        got = check_cdf_selection(score, idx, lens, thr, scale)
        assert got.min() < got.max()                       # rows keep different numbers of blocks
    # with a top-k floor (bsa_interface.py:252-266)
    idx, lens = I().get_select_indices_cdf_topk_from_score(score.cuda(), 0.9, 0.5, 1.0)
    check_cdf_selection(score, idx, lens, 0.5, 1.0, k_min=O.num_selected(0.9, 200))
    assert int(lens.min()) >= O.num_selected(0.9, 200) == 19      # int((1 - 0.9) * 200) truncates 19.999...


def test_cdf_selection_edge_cases():
    score = torch.zeros(1, 1, 4, 130)
    score[0, 0, 1, 7] = 60.0                                # one column holds all the mass
    score[0, 0, 2, :] = torch.arange(130).float() * 0.01
    idx, lens = I().get_select_indices_cdf_from_score(score.cuda(), 0.5, 1.0)
    assert lens.cpu().tolist() == [[[65, 0, int(O.select_cdf(score, 0.5, 1.0)[1][0, 0, 2]), 65]]]
    assert torch.equal(idx[0, 0, 0, :65].cpu(), torch.arange(65))          # ties: lowest index first
    assert int(idx[0, 0, 1, 0]) == -1
    idx, lens = I().get_select_indices_cdf_from_score(score.cuda(), 2.0, 1.0)   # threshold above one: everything
    assert torch.all(lens == 130)
    big = torch.randn(1, 1, 3, 1440, generator=torch.Generator().manual_seed(22)).bfloat16()
    idx, lens = I().get_select_indices_cdf_from_score(big.cuda(), 0.95, 1.0)
    check_cdf_selection(big, idx, lens, 0.95, 1.0)
    assert idx.shape[-1] == 1440 and 1024 < int(lens.max()) <= 1440        # rows that keep more than 1 024 blocks


def test_cdf_selection_from_pooled_vectors_and_dispatch():
    g = torch.Generator().manual_seed(23)
    q = torch.randn(1, 2, 24, 128, generator=g).bfloat16()
    k = torch.randn(1, 2, 96, 128, generator=g).bfloat16()
    score = I().cal_score(q.cuda(), k.cuda()).cpu()
    idx, lens = I().get_select_indices(q.cuda(), k.cuda(), None, 0.7)
    check_cdf_selection(score, idx, lens, 0.7, 1 / 128 ** 0.5)
    idx2, lens2 = I().get_select_indices(q.cuda(), k.cuda(), 0.75, 0.7)
    check_cdf_selection(score, idx2, lens2, 0.7, 1 / 128 ** 0.5, k_min=24)
    idx3, lens3 = I().get_select_indices_from_score(score.cuda(), None, 0.7)
    assert torch.equal(idx3, idx) and torch.equal(lens3, lens)

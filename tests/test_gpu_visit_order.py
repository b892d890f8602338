"""The visiting order of the selected KV blocks on the GPU (bsa_visit_order): bit-exact against the oracle,
and the operator's attention kernel run on its own with that order reproduces the operator's output."""
import numpy as np
import pytest
import torch

from oracle import bsa_oracle as O

pytestmark = pytest.mark.gpu


def I():
    from longcat_video_amd.block_sparse_attention import bsa_interface
    return bsa_interface


def random_lists(rows, nbk, stride, lens, seed):
    rng = np.random.default_rng(seed)
    idx = np.full((rows, stride), -1, dtype=np.int32)
    for r in range(rows):
        idx[r, :lens[r]] = np.sort(rng.choice(nbk, lens[r], replace=False))
    return idx


@pytest.mark.parametrize("nbk,stride,fixed", [(1440, 90, True), (624, 39, True), (1170, 146, True), (64, 64, True),
                                              (1440, 1024, False), (4096, 4096, False), (40, 8, True), (300, 9, False),
                                              (5000, 70, False)])
def test_matches_the_oracle_bit_for_bit(nbk, stride, fixed):
    rows = 37 if stride > 1000 else 301
    rng = np.random.default_rng(stride)
    lens = np.full(rows, stride) if fixed else rng.integers(0, min(stride, nbk) + 1, rows)
    lens = np.minimum(lens, nbk).astype(np.int32)
    if not fixed:
        lens[:4] = (0, 1, min(stride, nbk), 8)
    idx = random_lists(rows, nbk, stride, lens, seed=nbk + stride)
    got = I().visit_order(torch.from_numpy(idx).cuda(), torch.from_numpy(lens).cuda(), nbk).cpu().numpy()
    for r in range(rows):
        want = O.paced_visit_order(idx[r, :lens[r]], nbk)
        assert np.array_equal(got[r, :lens[r]], want), (r, lens[r])
        assert np.array_equal(got[r, lens[r]:], idx[r, lens[r]:])          # the unused tail is carried over


def test_in_place_and_leading_dimensions():
    from longcat_video_amd import _capi
    nbk, n = 1440, 90
    lens = np.full(2 * 3 * 5, n, dtype=np.int32)
    idx = random_lists(30, nbk, n, lens, seed=9)
    t = torch.from_numpy(idx).cuda().view(2, 3, 5, n)
    ln = torch.from_numpy(lens).cuda().view(2, 3, 5)
    want = I().visit_order(t, ln, nbk)
    assert want.shape == t.shape
    buf = t.clone()
    _capi.check(_capi.load().bsa_visit_order(buf.data_ptr(), ln.data_ptr(), buf.data_ptr(), 30, nbk, n,
                                             torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert torch.equal(buf, want)


def test_malformed_lists_give_a_permutation_of_the_clamped_blocks():
    nbk, n, rows = 200, 40, 64
    rng = np.random.default_rng(11)
    idx = rng.integers(-5, nbk + 5, (rows, n)).astype(np.int32)         # unsorted, repeated, out of range
    lens = np.full(rows, n, dtype=np.int32)
    lens[0] = 1000                                                     # longer than the row: clamped to it
    got = I().visit_order(torch.from_numpy(idx).cuda(), torch.from_numpy(lens).cuda(), nbk).cpu().numpy()
    clamped = np.clip(idx, 0, nbk - 1)
    assert np.array_equal(np.sort(got, axis=1), np.sort(clamped, axis=1))


def test_argument_checks():
    from longcat_video_amd import _capi
    lib = _capi.load()
    t = torch.zeros(4, 8, dtype=torch.int32, device="cuda")
    ln = torch.zeros(4, dtype=torch.int32, device="cuda")
    assert lib.bsa_visit_order(None, ln.data_ptr(), t.data_ptr(), 4, 10, 8, None) == _capi.BSA_ERR_BAD_ARG
    assert lib.bsa_visit_order(t.data_ptr(), ln.data_ptr(), t.data_ptr(), 4, 10, 5000, None) == _capi.BSA_ERR_BAD_ARG
    assert lib.bsa_visit_order(t.data_ptr(), ln.data_ptr(), t.data_ptr(), 4, 0, 8, None) == _capi.BSA_ERR_BAD_ARG
    assert lib.bsa_visit_order(t.data_ptr(), ln.data_ptr(), t.data_ptr(), 0, 10, 8, None) == _capi.BSA_OK


@pytest.mark.parametrize("shape,sparsity", [((8, 12, 16), 0.25), ((6, 10, 14), 0.5), ((16, 16, 16), 0.75)])
def test_operator_equals_its_attention_kernel_on_the_visiting_order(shape, sparsity):
    """bsa_fwd_3d = selection, visiting order, attention kernel: running the kernel alone on
    visit_order(ascending selection) gives the operator's output bit for bit (the same kernel on the same
    lists), for a grid without and with padded chunks."""
    bi = I()
    S = shape[0] * shape[1] * shape[2]
    g = torch.Generator(device="cuda").manual_seed(12)
    q, k, v = (torch.randn(1, 4, S, 128, generator=g, device="cuda").bfloat16() for _ in range(3))
    o, idx, lens, _ = bi._bsa_3d(q, k, v, shape, shape, sparsity, (4, 4, 4), (4, 4, 4), want_selection=True)
    nbk = int(np.prod([-(-n // 4) for n in shape]))
    asc = idx.sort(dim=-1).values.int().contiguous()
    paced = bi.visit_order(asc, lens, nbk)
    assert idx.shape[-1] > 8 and not torch.equal(paced, asc)
    attend = bi.ThwAttention(k, v, shape, shape, (4, 4, 4), (4, 4, 4))
    assert torch.equal(attend(q, paced, lens), o)
    # and the ascending order gives the same attention up to rounding
    d = (attend(q, asc, lens).float() - o.float()).abs()
    assert float(d.max()) <= 1.6e-2 and float(d.mean()) <= 1e-3

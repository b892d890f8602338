"""Pins the oracle's 3-D chunk permutation (R0, R1, R7) by brute force and by
an independent view/permute evaluation; no reference code is imported."""
import itertools

import numpy as np
import pytest
import torch

from oracle import bsa_oracle as O

GRIDS = [
    ((4, 8, 8), (4, 4, 4)),     # config 1
    ((8, 8, 8), (4, 4, 8)),     # the reference's default chunk
    ((2, 3, 5), (2, 2, 2)),     # ragged on H and W
    ((5, 6, 7), (4, 4, 4)),     # ragged on all axes
    ((1, 1, 1), (4, 4, 4)),     # a single token
    ((4, 4, 4), (1, 1, 1)),     # chunk of one token: identity
]


def brute_force_map(latent, chunk):
    T, H, W = latent
    t, h, w = chunk
    Nt, Nh, Nw = -(-T // t), -(-H // h), -(-W // w)
    out = []
    for nt, nh, nw, ti, hi, wi in itertools.product(range(Nt), range(Nh), range(Nw), range(t), range(h), range(w)):
        tt, hh, ww = nt * t + ti, nh * h + hi, nw * w + wi
        out.append((tt * H + hh) * W + ww if (tt < T and hh < H and ww < W) else -1)
    return np.array(out, dtype=np.int64)


@pytest.mark.parametrize("latent,chunk", GRIDS)
def test_index_map_matches_brute_force(latent, chunk):
    assert np.array_equal(O.permute_index_map(latent, chunk), brute_force_map(latent, chunk))


@pytest.mark.parametrize("latent,chunk", GRIDS)
def test_index_map_is_a_bijection_on_real_tokens(latent, chunk):
    m = O.permute_index_map(latent, chunk)
    real = m[m >= 0]
    assert np.array_equal(np.sort(real), np.arange(int(np.prod(latent))))
    Nt, Nh, Nw = O.block_grid(latent, chunk)
    assert m.size == Nt * Nh * Nw * int(np.prod(chunk))


@pytest.mark.parametrize("latent,chunk", [g for g in GRIDS if all(n % c == 0 for n, c in zip(*g))])
def test_divisible_grids_equal_view_permute(latent, chunk):
    """On divisible grids the oracle must equal the view -> permute -> contiguous
    formulation of the operator (bsa_interface.py:600-604), written out here."""
    T, H, W = latent
    t, h, w = chunk
    Nt, Nh, Nw = T // t, H // h, W // w
    x = torch.arange(2 * 3 * T * H * W * 5, dtype=torch.float32).view(2, 3, T * H * W, 5)
    want = x.view(2, 3, Nt, t, Nh, h, Nw, w, 5).permute(0, 1, 2, 4, 6, 3, 5, 7, 8).contiguous().view(2, 3, -1, 5)
    got = O.rearrange_thw_to_3d_block(x, latent, chunk)
    assert torch.equal(got, want)
    back = want.view(2, 3, Nt, Nh, Nw, t, h, w, 5).permute(0, 1, 2, 5, 3, 6, 4, 7, 8).contiguous().view(2, 3, -1, 5)
    assert torch.equal(O.rearrange_3d_block_to_thw(want, latent, chunk), back)
    assert torch.equal(back, x)


@pytest.mark.parametrize("latent,chunk", GRIDS)
def test_round_trip_and_zero_padding(latent, chunk):
    S = int(np.prod(latent))
    x = torch.randn(1, 2, S, 4, generator=torch.Generator().manual_seed(0)) + 10.0   # no zeros
    p = O.rearrange_thw_to_3d_block(x, latent, chunk)
    valid = torch.from_numpy(O.slot_validity(latent, chunk))
    assert torch.all(p[:, :, ~valid] == 0)
    assert torch.all(p[:, :, valid] != 0)
    assert torch.equal(O.rearrange_3d_block_to_thw(p, latent, chunk), x)


def test_every_block_is_a_spatial_cube():
    latent, chunk = (8, 8, 12), (4, 4, 4)
    m = O.permute_index_map(latent, chunk).reshape(-1, 64)
    T, H, W = latent
    for blk in m:
        tt, hh, ww = blk // (H * W), (blk // W) % H, blk % W
        assert tt.max() - tt.min() == 3 and hh.max() - hh.min() == 3 and ww.max() - ww.min() == 3


def test_every_padded_block_keeps_a_real_token():
    for latent, chunk in GRIDS + [((24, 45, 80), (4, 4, 4)), ((24, 30, 52), (4, 4, 4))]:
        v = O.slot_validity(latent, chunk).reshape(-1, int(np.prod(chunk)))
        assert v.any(axis=1).all()


def test_baseline_grid_sizes():
    assert O.permute_index_map((24, 45, 80), (4, 4, 4)).size == 92160
    assert O.block_grid((24, 45, 80), (4, 4, 4)) == (6, 12, 20)
    assert O.permute_index_map((24, 30, 52), (4, 4, 4)).size == 39936
    assert O.permute_index_map((48, 30, 52), (4, 4, 4)).size == 79872

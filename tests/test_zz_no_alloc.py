"""The entry point that allocates nothing: bsa_fwd_3d_static keeps its scratch memory in a buffer built into the
library.  It has no counterpart in the reference.  It runs the compact route of the operator (k and v gathered
where they lie), bsa_fwd_3d the route that rewrites k and v in fragment order: the same pooling, score and
selection kernels, so scores and selection must agree bit for bit, and two attention kernels that agree to fp32
summation order (fp32 inputs take one route in both).  Checked on calls in a row, the later ones smaller, which
find the earlier calls' leftovers in the buffer; a problem that does not fit must be rejected."""
import ctypes as C

import numpy as np
import pytest
import torch

from conftest import seeded_qkv

pytestmark = pytest.mark.gpu


def I():
    from longcat_video_amd.block_sparse_attention import bsa_interface
    return bsa_interface


def both(seed, heads, latent, sparsity, chunk, dtype=torch.bfloat16, cdf=None):
    S = int(np.prod(latent))
    q, k, v = (t.cuda() for t in seeded_qkv(seed, 1, heads, S, S, 128, dtype))
    got = I()._bsa_3d(q, k, v, latent, latent, sparsity, chunk, chunk, True, cdf_threshold=cdf, static_scratch=True)
    torch.cuda.synchronize()
    want = I()._bsa_3d(q, k, v, latent, latent, sparsity, chunk, chunk, True, cdf_threshold=cdf)
    torch.cuda.synchronize()
    return got, want


def same(got, want):
    o, idx, lens, score = got
    o2, idx2, lens2, score2 = want
    assert torch.equal(score, score2)
    assert torch.equal(idx, idx2) and torch.equal(lens, lens2)          # integer results: bit-exact
    if o.dtype == torch.float32:
        assert torch.equal(o, o2)                                       # one route, the same kernels
    else:
        d = (o.float() - o2.float()).abs()                              # two attention kernels: a couple of bf16 ulps
        assert d.max() <= 1.6e-2 and d.mean() <= 1e-3, (float(d.max()), float(d.mean()))
    assert torch.isfinite(o.float()).all()


def test_two_calls_in_a_row_the_second_smaller():
    same(*both(90, 4, (9, 18, 26), 0.75, (4, 4, 4)))      # padded in t, h and w: edge copies, validity words, tables
    same(*both(91, 2, (4, 8, 8), 0.5, (4, 4, 4)))         # smaller: every piece of the buffer sits at a lower offset
    same(*both(92, 3, (5, 6, 12), 0.5, (4, 4, 8)))        # 128-token chunks
    same(*both(93, 2, (4, 8, 8), 0.5, (4, 4, 4), dtype=torch.float32))   # fp32 route: blocked copies in the buffer
    same(*both(94, 2, (5, 8, 12), 0.75, (4, 4, 4), cdf=0.6))             # lists of unequal length: order + queue words


def test_matches_the_oracle_directly():
    """Not only equal to the other entry point: the static route is held to the oracle on its own."""
    from test_gpu_e2e import check_against_oracle
    latent = (5, 9, 13)
    S = int(np.prod(latent))
    q, k, v = seeded_qkv(95, 1, 2, S, S, 128, torch.bfloat16)
    o, idx, lens, score = I()._bsa_3d(q.cuda(), k.cuda(), v.cuda(), latent, latent, 0.75, (4, 4, 4), (4, 4, 4), True,
                                      static_scratch=True)
    check_against_oracle(q, k, v, latent, latent, 0.75, o, idx, lens, score, q_blocks=range(24))


def test_a_problem_beyond_the_buffer_is_rejected_before_any_launch():
    from longcat_video_amd import _capi
    lib = _capi.load()
    latent = (24, 30, 52)                                 # 480p at 32 heads needs 118 MB of scratch memory
    prm = _capi.Bsa3dParams(1, 32, 128, _capi.BSA_BF16, *latent, *latent, 4, 4, 4, 4, 4, 4, 39, 128 ** -0.5, 0.0)
    assert lib.bsa_workspace_bytes(C.byref(prm)) > _capi.BSA_STATIC_SCRATCH_BYTES
    one = torch.zeros(16, dtype=torch.bfloat16, device="cuda")           # never read: the size check comes first
    st = _capi.strides3((0, 0, 128))
    rc = lib.bsa_fwd_3d_static(C.byref(prm), one.data_ptr(), st, one.data_ptr(), st, one.data_ptr(), st, one.data_ptr(), st,
                               None, None, None, None)
    assert rc == _capi.BSA_ERR_WORKSPACE
    assert "scratch" in _capi.last_error()
    torch.cuda.synchronize()


def _direct_call(lib, prm, q, k, v, o, stream):
    """bsa_fwd_3d_static through the C-ABI with tensors that exist already: the Python side allocates nothing either."""
    from longcat_video_amd import _capi
    st = lambda t: _capi.strides3(t.stride()[:3])
    return lib.bsa_fwd_3d_static(C.byref(prm), q.data_ptr(), st(q), k.data_ptr(), st(k), v.data_ptr(), st(v), o.data_ptr(), st(o),
                                 None, None, None, C.c_void_p(stream.cuda_stream))


def _problem(seed, heads, latent, k_sel):
    from longcat_video_amd import _capi
    S = int(np.prod(latent))
    q, k, v = (t.cuda() for t in seeded_qkv(seed, 1, heads, S, S, 128, torch.bfloat16))
    prm = _capi.Bsa3dParams(1, heads, 128, _capi.BSA_BF16, *latent, *latent, 4, 4, 4, 4, 4, 4, k_sel, 128 ** -0.5, 0.0)
    return prm, q, k, v, torch.empty_like(q)


def test_a_call_leaves_the_free_device_memory_as_it_was():
    """What the entry point is for: after one warm call (which looks up the buffer's address) a call through the
    C-ABI with existing tensors changes neither the driver's free memory nor what torch's allocator holds."""
    from longcat_video_amd import _capi
    lib = _capi.load()
    prm, q, k, v, o = _problem(96, 2, (5, 9, 13), 6)
    stream = torch.cuda.current_stream()
    assert _direct_call(lib, prm, q, k, v, o, stream) == _capi.BSA_OK       # warm: symbol lookup, event creation
    torch.cuda.synchronize()
    want = o.clone()
    o.zero_()
    free_before, reserved_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
    for _ in range(3):
        assert _direct_call(lib, prm, q, k, v, o, stream) == _capi.BSA_OK
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_reserved() == reserved_before
    assert torch.equal(o, want)


def test_a_captured_call_replays():
    """Under stream capture the call records kernels only (no allocation, no memset node); every replay, with eager
    work and synchronisations between them, gives the eager result."""
    from longcat_video_amd import _capi
    lib = _capi.load()
    prm, q, k, v, o = _problem(97, 2, (4, 8, 12), 6)
    assert _direct_call(lib, prm, q, k, v, o, torch.cuda.current_stream()) == _capi.BSA_OK
    torch.cuda.synchronize()
    want = o.clone()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph, stream=side):
        assert _direct_call(lib, prm, q, k, v, o, torch.cuda.current_stream()) == _capi.BSA_OK
    for r in range(3):
        o.fill_(float(r))
        (q.float().sum() + r).item()                     # eager work and a synchronisation between replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(o, want), r


def test_a_call_while_another_stream_still_uses_the_buffer_is_refused():
    """Two streams: the second call arrives while the first one's kernels run and must come back with BSA_ERR_BUSY,
    having launched nothing; once the first has finished, the same call goes through.  One stream never refuses."""
    from longcat_video_amd import _capi
    lib = _capi.load()
    prm, q, k, v, o = _problem(98, 6, (24, 45, 80), 90)                      # the largest 720p share that fits: ~2 ms
    o2 = torch.full_like(o, 7.0)
    a, b = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    assert _direct_call(lib, prm, q, k, v, o, a) == _capi.BSA_OK
    assert _direct_call(lib, prm, q, k, v, o, a) == _capi.BSA_OK             # same stream: in order, never refused
    rc = _direct_call(lib, prm, q, k, v, o2, b)
    assert rc == _capi.BSA_ERR_BUSY and "another stream" in _capi.last_error()
    torch.cuda.synchronize()
    assert bool((o2 == 7.0).all())                                           # nothing ran
    assert _direct_call(lib, prm, q, k, v, o2, b) == _capi.BSA_OK
    torch.cuda.synchronize()
    assert torch.equal(o2, o)

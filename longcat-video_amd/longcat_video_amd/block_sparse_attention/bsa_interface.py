"""Host side of the block-sparse attention operator.

Mirrors the call surface of the reference module
``longcat_video/block_sparse_attention/bsa_interface.py`` (names, argument
order and meaning, error types) so that ``Attention._process_attn``
(longcat_video/modules/attention.py:58-67) can call it unchanged.  Every
function here only validates, allocates torch tensors and calls the C-ABI of
the gfx950 engine; there is no eager or CPU implementation behind it.

Differences from the reference, all supersets:
  * grids that are not chunk multiples are padded at the high end (zeros,
    padded keys masked, padded query rows dropped) instead of raising; pass
    ``allow_padding=False`` for the reference's AssertionError
    (bsa_interface.py:639-640);
  * block indices are int32 inside the engine; the helpers that the reference
    returns int64 from (torch.topk) convert on the way out;
  * gradients flow for bf16 / fp16 inputs (the reference's backward, bsa_interface.py:570-596); fp32 inputs that
    require a gradient are rejected while grad mode is on;
  * the CDF selection rule (bsa_interface.py:226-266) keeps its weights in fp32 and its running sum in double
    for every storage type, and ``get_select_indices_from_score`` takes the ``sm_scale`` the reference forgets
    to pass on (bsa_interface.py:283, 285).
"""
from __future__ import annotations

import ctypes as C
import math
import threading
from typing import Optional, Sequence, Tuple

import torch

from .. import _capi

_DTYPES = {torch.bfloat16: _capi.BSA_BF16, torch.float16: _capi.BSA_F16, torch.float32: _capi.BSA_F32}


def _code(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise NotImplementedError("dtype %s is not supported (bf16, fp16, fp32)" % t.dtype)


def _need_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("the block-sparse attention engine runs on the GPU only; got a %s tensor" % t.device)


def _stream(t: torch.Tensor) -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _ptr(t: Optional[torch.Tensor]) -> C.c_void_p:
    return C.c_void_p(None if t is None else t.data_ptr())


def _rows_ok(t: torch.Tensor) -> torch.Tensor:
    """[B,H,S,D] with a contiguous, 16-byte aligned D axis; anything else is copied."""
    es = t.element_size()
    ok = t.stride(3) == 1 and t.data_ptr() % 16 == 0 and all((t.stride(i) * es) % 16 == 0 for i in range(3))
    return t if ok else t.contiguous()


_WORKSPACES: dict = {}


def _workspace(nbytes: int, device: torch.device) -> torch.Tensor:
    """The engine's scratch memory for a call on the current stream of `device`: one uint8 buffer per (device,
    stream, host thread), grown when a call needs more and otherwise reused, so that a steady-state call allocates
    nothing.  Calls that one thread enqueues on one stream run in order and may share a buffer; another stream or
    another thread gets its own.  Under stream capture the buffer is a fresh allocation from the graph's own pool
    (it then lives as long as the graph does, and a later regrowth here cannot pull it from under a replay)."""
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)
    key = (device.index if device.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(device).cuda_stream, threading.get_ident())
    buf = _WORKSPACES.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)
        _WORKSPACES[key] = buf
    return buf


def release_workspaces() -> None:
    """Drops the cached scratch buffers (they are re-created on demand)."""
    _WORKSPACES.clear()


def num_selected(sparsity: float, n_kv_blocks: int) -> int:
    """bsa_interface.py:214: ``int((1 - sparsity) * n_blocks)`` in Python doubles."""
    return int((1 - sparsity) * n_kv_blocks)


# ---------------------------------------------------------------------------
# R1 / R7: 3-D chunk permute and its inverse
# ---------------------------------------------------------------------------
def _permute(x, latent_shape, chunk, want_pooled=False, want_valid=False):
    _need_gpu(x)
    B, H, S, D = x.shape
    T, Hh, W = (int(v) for v in latent_shape)
    t, h, w = (int(v) for v in chunk)
    assert T * Hh * W == S, "latent shape %s does not match %d tokens" % ((T, Hh, W), S)
    x = _rows_ok(x)
    lib = _capi.load()
    Sp = lib.bsa_padded_tokens(T, Hh, W, t, h, w)
    nb = Sp // (t * h * w)
    out = torch.empty(B, H, Sp, D, dtype=x.dtype, device=x.device)
    pooled = torch.empty(B, H, nb, D, dtype=x.dtype, device=x.device) if want_pooled else None
    valid = torch.empty(Sp // 64, dtype=torch.int64, device=x.device) if want_valid else None
    with torch.cuda.device(x.device):
        _capi.check(lib.bsa_permute_thw_to_blocks(
            _ptr(x), _capi.strides3(x.stride()[:3]), _ptr(out), _ptr(pooled), _ptr(valid),
            B, H, T, Hh, W, t, h, w, D, _code(x), _stream(x)), "permute")
    return out, pooled, valid


def rearrange_THW_to_3d_block(x, Nt, Nh, Nw, t, h, w, D=None, latent_shape=None):
    """bsa_interface.py:600-604.  ``latent_shape`` (T,H,W) may be given when the
    grid is not a chunk multiple; it defaults to (Nt*t, Nh*h, Nw*w)."""
    if latent_shape is None:
        latent_shape = (Nt * t, Nh * h, Nw * w)
    return _permute(x, latent_shape, (t, h, w))[0]


def rearrange_3d_block_to_THW(x, Nt, Nh, Nw, t, h, w, D=None, latent_shape=None):
    """bsa_interface.py:606-610; padded slots are dropped."""
    _need_gpu(x)
    if latent_shape is None:
        latent_shape = (Nt * t, Nh * h, Nw * w)
    T, Hh, W = (int(v) for v in latent_shape)
    B, H, Sp, Dd = x.shape
    assert Sp == Nt * Nh * Nw * t * h * w, "blocked tensor has %d slots, expected %d" % (Sp, Nt * Nh * Nw * t * h * w)
    x = x.contiguous()
    out = torch.empty(B, H, T * Hh * W, Dd, dtype=x.dtype, device=x.device)
    lib = _capi.load()
    with torch.cuda.device(x.device):
        _capi.check(lib.bsa_unpermute_blocks_to_thw(
            _ptr(x), _ptr(out), _capi.strides3(out.stride()[:3]), B, H, T, Hh, W, t, h, w, Dd, _code(x),
            _stream(x)), "unpermute")
    return out


# ---------------------------------------------------------------------------
# R2 - R4: gating
# ---------------------------------------------------------------------------
def mean_pooling_compression(x: torch.Tensor, block_size: int) -> torch.Tensor:
    """bsa_interface.py:168-178."""
    _need_gpu(x)
    B, H, S, D = x.shape
    x = x.contiguous()
    nb = math.ceil(S / block_size)
    out = torch.empty(B, H, nb, D, dtype=x.dtype, device=x.device)
    lib = _capi.load()
    with torch.cuda.device(x.device):
        _capi.check(lib.bsa_mean_pool(_ptr(x), _ptr(out), B, H, S, int(block_size), D, _code(x), _stream(x)), "mean_pool")
    return out


def _score_topk(q_cmp, k_cmp, k_sel, order="score"):
    """order: "score" = descending score (the reference's torch.topk order), "block" = ascending block index."""
    _need_gpu(q_cmp, k_cmp)
    B, H, nbq, D = q_cmp.shape
    nbk = k_cmp.shape[2]
    assert k_cmp.shape[0] == B and k_cmp.shape[1] == H and k_cmp.shape[3] == D
    q_cmp, k_cmp = q_cmp.contiguous(), k_cmp.contiguous()
    score = torch.empty(B, H, nbq, nbk, dtype=q_cmp.dtype, device=q_cmp.device)
    buf = torch.empty(B * H * nbq * max(k_sel, 1), dtype=torch.int32, device=q_cmp.device)   # non-null even for k_sel == 0
    idx = buf[: B * H * nbq * k_sel].view(B, H, nbq, k_sel)
    lens = torch.empty(B, H, nbq, dtype=torch.int32, device=q_cmp.device)
    lib = _capi.load()
    with torch.cuda.device(q_cmp.device):
        by_score = order == "score"
        _capi.check(lib.bsa_score_topk(_ptr(q_cmp), _ptr(k_cmp), _ptr(buf) if by_score else None,
                                       None if by_score else _ptr(buf), _ptr(lens), _ptr(score),
                                       B, H, nbq, nbk, D, k_sel, _code(q_cmp), _stream(q_cmp)), "score_topk")
    return idx, lens, score


def visit_order(idx_sorted: torch.Tensor, lens: torch.Tensor, n_kv_blocks: int) -> torch.Tensor:
    """The operator's visiting order for lists given in ascending block order (bsa_visit_order): [..., rows, width]
    int32 lists with lens[...] entries in use.  No counterpart in the reference, whose kernel visits the blocks in
    list order; attention depends on the order only through rounding."""
    _need_gpu(idx_sorted, lens)
    assert idx_sorted.dtype == torch.int32 and lens.dtype == torch.int32 and idx_sorted.shape[:-1] == lens.shape
    idx_sorted, lens = idx_sorted.contiguous(), lens.contiguous()
    out = torch.empty_like(idx_sorted)
    if idx_sorted.numel() == 0:
        return out
    lib = _capi.load()
    with torch.cuda.device(idx_sorted.device):
        _capi.check(lib.bsa_visit_order(_ptr(idx_sorted), _ptr(lens), _ptr(out), lens.numel(), int(n_kv_blocks),
                                        idx_sorted.shape[-1], _stream(idx_sorted)), "visit_order")
    return out


def cal_score(q: torch.Tensor, k: torch.Tensor) -> torch.Tensor:
    """bsa_interface.py:180-184: unscaled ``q @ k^T`` in the input dtype."""
    return _score_topk(q, k, 0)[2]


def get_select_indices_topk_from_score(score: torch.Tensor, sparsity: float):
    """bsa_interface.py:212-224.  Indices int64, descending score, ties towards
    the lowest index; lens int32, all ``num_selected``."""
    _need_gpu(score)
    B, H, nbq, nbk = score.shape
    k_sel = num_selected(sparsity, nbk)
    score = score.contiguous()
    buf = torch.empty(B * H * nbq * max(k_sel, 1), dtype=torch.int32, device=score.device)
    idx = buf[: B * H * nbq * k_sel].view(B, H, nbq, k_sel)
    lens = torch.empty(B, H, nbq, dtype=torch.int32, device=score.device)
    lib = _capi.load()
    with torch.cuda.device(score.device):
        _capi.check(lib.bsa_topk_from_score(_ptr(score), _ptr(buf), None, _ptr(lens), B, H, nbq, nbk, k_sel,
                                            _code(score), _stream(score)), "topk")
    return idx.long(), lens


def get_select_indices_topk(q: torch.Tensor, k: torch.Tensor, sparsity: float):
    """bsa_interface.py:206-210."""
    idx, lens, _ = _score_topk(q, k, num_selected(sparsity, k.shape[2]))
    return idx.long(), lens


def _cdf_width(nbk: int) -> int:
    return min(int(nbk), 4096)       # columns kept per row at most: all of them (the engine's lists hold 4096 entries)


def _select_cdf(score, q_cmp, k_cmp, cdf_threshold, sm_scale, k_min, order="score"):
    """CDF rule on a given score tensor, or on pooled q/k (score is then computed too)."""
    lib = _capi.load()
    if score is not None:
        _need_gpu(score)
        score = score.contiguous()
        B, H, nbq, nbk = score.shape
        dev, dt = score.device, score
    else:
        _need_gpu(q_cmp, k_cmp)
        q_cmp, k_cmp = q_cmp.contiguous(), k_cmp.contiguous()
        B, H, nbq, D = q_cmp.shape
        nbk = k_cmp.shape[2]
        dev, dt = q_cmp.device, q_cmp
        score = torch.empty(B, H, nbq, nbk, dtype=q_cmp.dtype, device=dev)
    width = _cdf_width(nbk)
    idx = torch.empty(B, H, nbq, width, dtype=torch.int32, device=dev)
    lens = torch.empty(B, H, nbq, dtype=torch.int32, device=dev)
    a, b = (_ptr(idx), None) if order == "score" else (None, _ptr(idx))
    with torch.cuda.device(dev):
        if q_cmp is None:
            _capi.check(lib.bsa_cdf_from_score(_ptr(score), a, b, _ptr(lens), B, H, nbq, nbk, float(cdf_threshold),
                                               float(sm_scale), int(k_min), width, _code(dt), _stream(dt)), "cdf")
        else:
            _capi.check(lib.bsa_score_cdf(_ptr(q_cmp), _ptr(k_cmp), a, b, _ptr(lens), _ptr(score), B, H, nbq, nbk,
                                          q_cmp.shape[3], float(cdf_threshold), float(sm_scale), int(k_min), width,
                                          _code(dt), _stream(dt)), "score_cdf")
    return idx, lens, score


def get_select_indices_cdf_from_score(score: torch.Tensor, cdf_threshold: float, sm_scale: float):
    """bsa_interface.py:233-243.  Indices int64 [B,H,nbq,nbk]: row m holds its selection in
    descending score order up to lens[m] and -1 behind (the reference returns all nbk sorted columns, of
    which only the first lens[m] are ever read); lens int32."""
    idx, lens, _ = _select_cdf(score, None, None, cdf_threshold, sm_scale, 0)
    return idx.long(), lens


def get_select_indices_cdf(q: torch.Tensor, k: torch.Tensor, cdf_threshold: float):
    """bsa_interface.py:226-231."""
    idx, lens, _ = _select_cdf(None, q, k, cdf_threshold, 1 / q.shape[-1] ** 0.5, 0)
    return idx.long(), lens


def get_select_indices_cdf_topk_from_score(score: torch.Tensor, sparsity: float, cdf_threshold: float, sm_scale: float):
    """bsa_interface.py:252-266: the CDF rule, but never fewer blocks than top-k would keep."""
    idx, lens, _ = _select_cdf(score, None, None, cdf_threshold, sm_scale,
                               min(num_selected(sparsity, score.shape[-1]), _cdf_width(score.shape[-1])))
    return idx.long(), lens


def get_select_indices_cdf_topk(q: torch.Tensor, k: torch.Tensor, sparsity: float, cdf_threshold: float):
    """bsa_interface.py:245-250."""
    idx, lens, _ = _select_cdf(None, q, k, cdf_threshold, 1 / q.shape[-1] ** 0.5,
                               min(num_selected(sparsity, k.shape[2]), _cdf_width(k.shape[2])))
    return idx.long(), lens


def get_select_indices(q, k, sparsity, cdf_threshold):
    """bsa_interface.py:268-277."""
    if sparsity is not None and cdf_threshold is None:
        return get_select_indices_topk(q, k, sparsity)
    if sparsity is None and cdf_threshold is not None:
        return get_select_indices_cdf(q, k, cdf_threshold)
    if sparsity is not None and cdf_threshold is not None:
        return get_select_indices_cdf_topk(q, k, sparsity, cdf_threshold)
    raise ValueError


def get_select_indices_from_score(score, sparsity, cdf_threshold, sm_scale=None):
    """bsa_interface.py:279-288.  The reference forgets to pass sm_scale to its CDF helpers there (a TypeError
    at :283 and :285); here it is an argument, defaulting to 1/sqrt(128)."""
    sm_scale = 1 / 128 ** 0.5 if sm_scale is None else sm_scale
    if sparsity is not None and cdf_threshold is None:
        return get_select_indices_topk_from_score(score, sparsity)
    if sparsity is None and cdf_threshold is not None:
        return get_select_indices_cdf_from_score(score, cdf_threshold, sm_scale)
    if sparsity is not None and cdf_threshold is not None:
        return get_select_indices_cdf_topk_from_score(score, sparsity, cdf_threshold, sm_scale)
    raise ValueError


# ---------------------------------------------------------------------------
# R5 / R6: the attention kernel on blocked-order tensors
# ---------------------------------------------------------------------------
def attn_fwd_bsa_varlen(q, k, v, sm_scale, block_indices, block_indices_lens, chunk_size_q, chunk_size_k,
                        sparsity=None, tile_valid: Optional[torch.Tensor] = None, kernel: Optional[str] = None):
    """bsa_interface.py:290-341 (attn_fwd_bsa_varlen_triton).  Returns ``(o, lse)``
    with ``lse`` the natural-log sum-exp, fp32 [B,H,S].  ``kernel``: "fragment" (bsa_fwd_fragment: the
    operator's attention kernel, with k and v rewritten once into its operand order; bf16 / fp16, the default
    for them) or "lds" (bsa_fwd: the LDS-tiled kernel, no workspace; the only one for fp32)."""
    _need_gpu(q, k, v, block_indices, block_indices_lens)
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    assert k.shape == v.shape and k.shape[0] == B and k.shape[1] == H and k.shape[3] == D
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    idx = block_indices.to(torch.int32).contiguous()
    lens = block_indices_lens.to(torch.int32).contiguous()
    assert idx.shape[:3] == (B, H, Sq // chunk_size_q) and lens.shape == idx.shape[:3]
    if kernel is None:
        kernel = "lds" if q.dtype == torch.float32 or idx.shape[3] > 4096 else "fragment"
    assert kernel in ("fragment", "lds")
    o = torch.empty_like(q)
    lse = torch.empty(B, H, Sq, dtype=torch.float32, device=q.device)
    lib = _capi.load()
    with torch.cuda.device(q.device):
        if kernel == "fragment":
            need = lib.bsa_fwd_fragment_workspace_bytes(B, H, Sq, Sk, D, _code(q))
            if need == 0:
                raise NotImplementedError("bsa_fwd_fragment: " + _capi.last_error())
            ws = _workspace(need, q.device)
            _capi.check(lib.bsa_fwd_fragment(_ptr(q), _ptr(k), _ptr(v), _ptr(idx), _ptr(lens), _ptr(tile_valid), _ptr(o),
                                             _ptr(lse), B, H, Sq, Sk, D, int(chunk_size_q), int(chunk_size_k), idx.shape[3],
                                             float(sm_scale), _code(q), _ptr(ws), need, _stream(q)), "bsa_fwd_fragment")
        else:
            _capi.check(lib.bsa_fwd(_ptr(q), _ptr(k), _ptr(v), _ptr(idx), _ptr(lens), _ptr(tile_valid), _ptr(o), _ptr(lse),
                                    B, H, Sq, Sk, D, int(chunk_size_q), int(chunk_size_k), idx.shape[3],
                                    float(sm_scale), _code(q), _stream(q)), "bsa_fwd")
    return o, lse


attn_fwd_bsa_varlen_triton = attn_fwd_bsa_varlen   # the reference's name for the same entry


def attn_bwd_bsa_varlen(do, q, k, v, o, dq, dk, dv, sm_scale, M, block_indices, block_indices_lens, chunk_size_q,
                        chunk_size_k, sparsity=None, tile_valid: Optional[torch.Tensor] = None):
    """bsa_interface.py:343-461 (attn_bwd_bsa_varlen_triton): gradients of the blocked-order attention into the
    caller's ``dq``, ``dk``, ``dv``.  ``M`` is the natural-log sum-exp the forward returned.  bf16 / fp16."""
    _need_gpu(do, q, k, v, o, dq, dk, dv, M, block_indices, block_indices_lens)
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    if q.dtype == torch.float32:
        raise NotImplementedError("the backward is built for bf16 and fp16")
    for t, like in ((do, q), (o, q), (dq, q), (dk, k), (dv, k), (v, k)):
        assert t.shape == like.shape and t.dtype == q.dtype
    for t in (dq, dk, dv):
        assert t.is_contiguous(), "dq, dk, dv are written in place and must be contiguous"
    do, q, k, v, o = (t.contiguous() for t in (do, q, k, v, o))
    lse = M.to(torch.float32).contiguous()
    idx = block_indices.to(torch.int32).contiguous()
    lens = block_indices_lens.to(torch.int32).contiguous()
    assert idx.shape[:3] == (B, H, Sq // chunk_size_q) and lens.shape == idx.shape[:3] and lse.shape == (B, H, Sq)
    lib = _capi.load()
    need = lib.bsa_bwd_workspace_bytes(B, H, Sq, Sk, D, int(chunk_size_q), int(chunk_size_k), idx.shape[3], _code(q))
    if need == 0:
        raise RuntimeError("bsa_bwd: " + lib.bsa_last_error().decode())
    ws = _workspace(need, q.device)
    with torch.cuda.device(q.device):
        _capi.check(lib.bsa_bwd(_ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(do), _ptr(lse), _ptr(idx), _ptr(lens),
                                _ptr(tile_valid), _ptr(dq), _ptr(dk), _ptr(dv), B, H, Sq, Sk, D, int(chunk_size_q),
                                int(chunk_size_k), idx.shape[3], float(sm_scale), _code(q), _ptr(ws), need, _stream(q)),
                    "bsa_bwd")


attn_bwd_bsa_varlen_triton = attn_bwd_bsa_varlen   # the reference's name for the same entry


def _select_blocked(q, k, chunk_size_q, chunk_size_k, sparsity, cdf_threshold):
    """Gating of the blocked-order operator (bsa_interface.py:546-549): lists in ascending block order."""
    D = q.shape[-1]
    q_cmp = mean_pooling_compression(q, chunk_size_q)
    k_cmp = mean_pooling_compression(k, chunk_size_k)
    if sparsity is None and cdf_threshold is None:
        raise ValueError
    if cdf_threshold is not None:
        k_min = 0 if sparsity is None else min(num_selected(sparsity, k_cmp.shape[2]), _cdf_width(k_cmp.shape[2]))
        idx, lens, _ = _select_cdf(None, q_cmp, k_cmp, cdf_threshold, 1 / D ** 0.5, k_min, order="block")   # bsa:229, 248
    else:
        idx, lens, _ = _score_topk(q_cmp, k_cmp, num_selected(sparsity, k_cmp.shape[2]), order="block")
    return idx, lens


class _AttentionBsa(torch.autograd.Function):
    """bsa_interface.py:535-596 (``_attention_bsa``): the blocked-order operator with its backward.  The gating
    (pooling, scores, selection) gets no gradient, as in the reference."""

    @staticmethod
    def forward(ctx, q, k, v, chunk_size_q, chunk_size_k, sparsity, cdf_threshold, sm_scale, tile_valid):
        idx, lens = _select_blocked(q, k, chunk_size_q, chunk_size_k, sparsity, cdf_threshold)
        o, lse = attn_fwd_bsa_varlen(q, k, v, sm_scale, idx, lens, chunk_size_q, chunk_size_k, sparsity, tile_valid)
        ctx.save_for_backward(q, k, v, o, lse, idx, lens)
        ctx.args = (sm_scale, chunk_size_q, chunk_size_k, sparsity, tile_valid)
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, lse, idx, lens = ctx.saved_tensors
        sm_scale, chunk_size_q, chunk_size_k, sparsity, tile_valid = ctx.args
        dq, dk, dv = (torch.empty(t.shape, dtype=t.dtype, device=t.device) for t in (q, k, v))
        attn_bwd_bsa_varlen(do, q, k, v, o, dq, dk, dv, sm_scale, lse, idx, lens, chunk_size_q, chunk_size_k, sparsity,
                            tile_valid)
        return dq, dk, dv, None, None, None, None, None, None


def _wants_grad(*tensors: torch.Tensor) -> bool:
    return torch.is_grad_enabled() and any(t.requires_grad for t in tensors)


def flash_attn_bsa(q, k, v, chunk_size_q, chunk_size_k, sparsity, cdf_threshold, sm_scale,
                   tile_valid: Optional[torch.Tensor] = None):
    """bsa_interface.py:535-568, 598 (``_attention_bsa.apply``) on blocked-order
    tensors: pool, score, top-k, attention.  Returns ``o`` only, like the reference.  With inputs that
    require a gradient (bf16 / fp16) the call is recorded for autograd."""
    if _wants_grad(q, k, v):
        return _AttentionBsa.apply(q, k, v, chunk_size_q, chunk_size_k, sparsity, cdf_threshold, sm_scale, tile_valid)
    D = q.shape[-1]
    assert D == k.shape[-1] and D == v.shape[-1]
    assert D in {16, 32, 64, 128, 256}
    idx, lens = _select_blocked(q, k, chunk_size_q, chunk_size_k, sparsity, cdf_threshold)
    o, _ = attn_fwd_bsa_varlen(q, k, v, sm_scale, idx, lens, chunk_size_q, chunk_size_k, sparsity, tile_valid)
    return o


# ---------------------------------------------------------------------------
# R9: the operator
# ---------------------------------------------------------------------------
def _bsa_3d(q, k, v, latent_shape_q, latent_shape_k, sparsity, chunk_q, chunk_k, want_selection=False, out=None,
            cdf_threshold=None, static_scratch=False, qk_norm=None, for_backward=False):
    """`out`: optional [B,H,Sq,D] view (any B/H/S strides, contiguous D) to write into.  `sparsity` may be
    None when `cdf_threshold` is given (bsa_interface.py:268-277).  `static_scratch`: run through
    bsa_fwd_3d_static, which keeps its scratch memory in a buffer built into the library instead of a
    workspace tensor (problems beyond that buffer raise; calls on one GPU must not overlap).
    `qk_norm` = (q_weight, k_weight, rope_table, table_T, t_offset_q, t_offset_k, eps): q and k are the raw
    projections and are normalised per head and rotated inside the operator's own passes (bsa_fwd_3d_qknorm;
    bf16 / fp16 and 64-token chunks only).  `for_backward`: the same kernels through bsa_fwd_3d_lse; returns
    (o, lists in the kernel's visiting order, lens, lse in token order) for the backward."""
    _need_gpu(q, k, v)
    B, H, Sq, D = q.shape
    Tq, Hq, Wq = (int(x) for x in latent_shape_q)
    Tk, Hk, Wk = (int(x) for x in latent_shape_k)
    tq, hq, wq = (int(x) for x in chunk_q)
    tk, hk, wk = (int(x) for x in chunk_k)
    lib = _capi.load()
    q, k, v = _rows_ok(q), _rows_ok(k), _rows_ok(v)
    if k.stride(2) != v.stride(2) or max(1, 64 // (wk * hk)) * Hk * Wk * k.stride(2) * k.element_size() >= 2 ** 32:
        # the engine gathers k and v tiles with one set of in-tile offsets (32 bits); views that
        # do not fit are copied once
        k, v = k.contiguous(), v.contiguous()
    nbk = lib.bsa_padded_tokens(Tk, Hk, Wk, tk, hk, wk) // (tk * hk * wk)
    nbq = lib.bsa_padded_tokens(Tq, Hq, Wq, tq, hq, wq) // (tq * hq * wq)
    k_sel = 0 if sparsity is None else num_selected(sparsity, nbk)
    width = k_sel
    if cdf_threshold is not None:
        width = _cdf_width(nbk)
        k_sel = min(k_sel, width)
    prm = _capi.Bsa3dParams(B, H, D, _code(q), Tq, Hq, Wq, Tk, Hk, Wk, tq, hq, wq, tk, hk, wk, k_sel,
                            1.0 / D ** 0.5, 0.0 if cdf_threshold is None else float(cdf_threshold))
    need = lib.bsa_workspace_bytes(C.byref(prm))
    if need == 0:
        _capi.check(lib.bsa_fwd_3d(C.byref(prm), None, None, None, None, None, None, None, None, None, 0,
                                   None, None, None, None), "flash_attn_bsa_3d")
    ws = None if static_scratch else _workspace(need, q.device)
    o = torch.empty(B, H, Sq, D, dtype=q.dtype, device=q.device) if out is None else out
    assert o.shape == (B, H, Sq, D) and o.dtype == q.dtype and o.stride(3) == 1
    idx = lens = score = None
    if want_selection:
        idx = torch.empty(B, H, nbq, width, dtype=torch.int32, device=q.device)
        lens = torch.empty(B, H, nbq, dtype=torch.int32, device=q.device)
        score = torch.empty(B, H, nbq, nbk, dtype=q.dtype, device=q.device)
    if for_backward:
        walk = torch.empty(B, H, nbq, max(width, 1), dtype=torch.int32, device=q.device)[..., :width]
        lens = torch.empty(B, H, nbq, dtype=torch.int32, device=q.device)
        lse = torch.empty(B, H, Sq, dtype=torch.float32, device=q.device)
        with torch.cuda.device(q.device):
            _capi.check(lib.bsa_fwd_3d_lse(
                C.byref(prm), _ptr(q), _capi.strides3(q.stride()[:3]), _ptr(k), _capi.strides3(k.stride()[:3]),
                _ptr(v), _capi.strides3(v.stride()[:3]), _ptr(o), _capi.strides3(o.stride()[:3]),
                _ptr(lse), _ptr(walk), _ptr(lens), _ptr(ws), need, _stream(q)), "flash_attn_bsa_3d (with lse)")
        return o, walk, lens, lse
    with torch.cuda.device(q.device):
        if qk_norm is not None:
            qw, kw, tab, table_T, t_off_q, t_off_k, eps = qk_norm
            qw, kw = qw.to(q.dtype).contiguous(), kw.to(q.dtype).contiguous()
            q_normed = torch.empty(B, H, Sq, D, dtype=q.dtype, device=q.device)
            n = _capi.BsaQkNorm(_ptr(qw), _ptr(kw), _ptr(tab), int(table_T), int(t_off_q), int(t_off_k), float(eps))
            _capi.check(lib.bsa_fwd_3d_qknorm(
                C.byref(prm), C.byref(n), _ptr(q), _capi.strides3(q.stride()[:3]), _ptr(q_normed),
                _capi.strides3(q_normed.stride()[:3]), _ptr(k), _capi.strides3(k.stride()[:3]),
                _ptr(v), _capi.strides3(v.stride()[:3]), _ptr(o), _capi.strides3(o.stride()[:3]),
                _ptr(ws), need, _ptr(idx), _ptr(lens), _ptr(score), _stream(q)), "flash_attn_bsa_3d (q/k norm inside)")
        elif static_scratch:
            _capi.check(lib.bsa_fwd_3d_static(
                C.byref(prm), _ptr(q), _capi.strides3(q.stride()[:3]), _ptr(k), _capi.strides3(k.stride()[:3]),
                _ptr(v), _capi.strides3(v.stride()[:3]), _ptr(o), _capi.strides3(o.stride()[:3]),
                _ptr(idx), _ptr(lens), _ptr(score), _stream(q)), "flash_attn_bsa_3d (static scratch)")
        else:
            _capi.check(lib.bsa_fwd_3d(
                C.byref(prm), _ptr(q), _capi.strides3(q.stride()[:3]), _ptr(k), _capi.strides3(k.stride()[:3]),
                _ptr(v), _capi.strides3(v.stride()[:3]), _ptr(o), _capi.strides3(o.stride()[:3]),
                _ptr(ws), need, _ptr(idx), _ptr(lens), _ptr(score), _stream(q)), "flash_attn_bsa_3d")
    return (o, idx, lens, score) if want_selection else o


class ThwAttention:
    """Block-sparse attention over (T,H,W)-ordered tensors with a caller-supplied selection, in two
    steps: the constructor prepares what depends on k and v (bsa_thw_prepare), every call runs the
    attention kernel alone (bsa_fwd_thw).  bf16 / fp16."""

    def __init__(self, k, v, latent_shape_q, latent_shape_k, chunk_3d_shape_q, chunk_3d_shape_k, sm_scale=None,
                 unequal_lengths=False):
        _need_gpu(k, v)
        B, H, Sk, D = k.shape
        self.gq = tuple(int(x) for x in latent_shape_q) + tuple(int(x) for x in chunk_3d_shape_q)
        Tq, Hq, Wq, tq, hq, wq = self.gq
        Tk, Hk, Wk = (int(x) for x in latent_shape_k)
        tk, hk, wk = (int(x) for x in chunk_3d_shape_k)
        assert Tk * Hk * Wk == Sk and v.shape == k.shape and v.dtype == k.dtype
        self.lib = lib = _capi.load()
        k, v = _rows_ok(k), _rows_ok(v)
        if k.stride(2) != v.stride(2) or max(1, 64 // (wk * hk)) * Hk * Wk * k.stride(2) * k.element_size() >= 2 ** 32:
            k, v = k.contiguous(), v.contiguous()      # one set of 32-bit in-tile offsets serves both
        self.k, self.v = k, v
        self.nbq = lib.bsa_padded_tokens(Tq, Hq, Wq, tq, hq, wq) // (tq * hq * wq)
        scale = 1.0 / D ** 0.5 if sm_scale is None else float(sm_scale)
        # unequal_lengths: the lists of later calls may differ in length (enqueue both schedules, choose on the device)
        self.prm = _capi.Bsa3dParams(B, H, D, _code(k), Tq, Hq, Wq, Tk, Hk, Wk, tq, hq, wq, tk, hk, wk, 0, scale,
                                     1.0 if unequal_lengths else 0.0)
        self.need = lib.bsa_workspace_bytes(C.byref(self.prm))
        self.ws = torch.empty(max(self.need, 1), dtype=torch.uint8, device=k.device)
        self.ks, self.vs = _capi.strides3(k.stride()[:3]), _capi.strides3(v.stride()[:3])
        with torch.cuda.device(k.device):
            _capi.check(lib.bsa_thw_prepare(C.byref(self.prm), _ptr(k), self.ks, _ptr(v), self.vs, _ptr(self.ws),
                                            self.need, _stream(k)), "bsa_thw_prepare")

    def __call__(self, q, block_indices, block_indices_lens, return_lse=False, out=None):
        _need_gpu(q)
        B, H, Sq, D = q.shape
        Tq, Hq, Wq = self.gq[:3]
        assert Tq * Hq * Wq == Sq and (B, H, D) == (self.k.shape[0], self.k.shape[1], self.k.shape[3]) and q.dtype == self.k.dtype
        q = _rows_ok(q)
        idx = block_indices.to(torch.int32).contiguous()
        lens = block_indices_lens.to(torch.int32).contiguous()
        assert idx.shape[:3] == (B, H, self.nbq) and lens.shape == (B, H, self.nbq)
        o = torch.empty(B, H, Sq, D, dtype=q.dtype, device=q.device) if out is None else out
        assert o.shape == (B, H, Sq, D) and o.dtype == q.dtype and o.stride(3) == 1
        lse = torch.empty(B, H, Sq, dtype=torch.float32, device=q.device) if return_lse else None
        with torch.cuda.device(q.device):
            _capi.check(self.lib.bsa_fwd_thw(
                C.byref(self.prm), _ptr(q), _capi.strides3(q.stride()[:3]), _ptr(self.k), self.ks, _ptr(self.v), self.vs,
                _ptr(o), _capi.strides3(o.stride()[:3]), _ptr(idx), _ptr(lens), idx.shape[3], _ptr(lse),
                _ptr(self.ws), self.need, _stream(q)), "bsa_fwd_thw")
        return (o, lse) if return_lse else o


def attn_fwd_bsa_thw(q, k, v, latent_shape_q, latent_shape_k, chunk_3d_shape_q, chunk_3d_shape_k,
                     block_indices, block_indices_lens, sm_scale=None, return_lse=False, out=None):
    """What the reference does with three rearrange_THW_to_3d_block calls, attn_fwd_bsa_varlen_triton
    and rearrange_3d_block_to_THW (bsa_interface.py:650-659, 290-341), without the permuted copies.
    block_indices [B,H,nbq,n] / block_indices_lens [B,H,nbq] count chunks of the padded grids.
    Returns o [B,H,Sq,D] (and lse [B,H,Sq] fp32, natural log, with return_lse)."""
    return ThwAttention(k, v, latent_shape_q, latent_shape_k, chunk_3d_shape_q, chunk_3d_shape_k, sm_scale)(
        q, block_indices, block_indices_lens, return_lse, out)


_SLOT_TOKENS: dict = {}


def _slot_tokens(latent_shape, chunk, device) -> torch.Tensor:
    """Token index of every slot of the blocked order of a (T, H, W) grid cut into chunks (bsa_interface.py:600-604
    on the padded grid), -1 for padding.  int64 [padded slots]; kept per (grid, chunk, device)."""
    key = (tuple(latent_shape), tuple(chunk), str(device))
    m = _SLOT_TOKENS.get(key)
    if m is None:
        (T, Hh, W), (t, h, w) = latent_shape, chunk
        Nt, Nh, Nw = -(-T // t), -(-Hh // h), -(-W // w)
        ar = lambda n: torch.arange(n, device=device)
        tt = (ar(Nt).view(Nt, 1, 1, 1, 1, 1) * t + ar(t).view(1, 1, 1, t, 1, 1)).expand(Nt, Nh, Nw, t, h, w)
        hh = (ar(Nh).view(1, Nh, 1, 1, 1, 1) * h + ar(h).view(1, 1, 1, 1, h, 1)).expand(Nt, Nh, Nw, t, h, w)
        ww = (ar(Nw).view(1, 1, Nw, 1, 1, 1) * w + ar(w).view(1, 1, 1, 1, 1, w)).expand(Nt, Nh, Nw, t, h, w)
        tok = (tt * Hh + hh) * W + ww
        m = torch.where((tt < T) & (hh < Hh) & (ww < W), tok, torch.full_like(tok, -1)).reshape(-1).contiguous()
        _SLOT_TOKENS[key] = m
    return m


class _Bsa3dWithGrad(torch.autograd.Function):
    """The operator for inputs that require a gradient.  The forward is the forward of every other call - the same
    kernels on the same lists, the same bits (bsa_interface.py:538-568 runs one kernel with and without grad) - and
    keeps the log-sum-exp and the lists it walked.  The backward (bsa_bwd_3d) takes and returns token-order tensors."""

    @staticmethod
    def forward(ctx, q, k, v, latent_shape_q, latent_shape_k, sparsity, cdf_threshold, chunk_q, chunk_k):
        o, walk, lens, lse = _bsa_3d(q, k, v, latent_shape_q, latent_shape_k, sparsity, chunk_q, chunk_k,
                                     cdf_threshold=cdf_threshold, for_backward=True)
        ctx.save_for_backward(q, k, v, o, lse, walk, lens)
        ctx.args = (tuple(latent_shape_q), tuple(latent_shape_k), tuple(chunk_q), tuple(chunk_k), 1 / q.shape[-1] ** 0.5)
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, o, lse, walk, lens = ctx.saved_tensors
        latent_q, latent_k, chunk_q, chunk_k, sm_scale = ctx.args
        return _bsa_3d_backward(do, q, k, v, o, lse, walk, lens, latent_q, latent_k, chunk_q, chunk_k, sm_scale) + (None,) * 6


def _bsa_3d_backward(do, q, k, v, o, lse, walk, lens, latent_q, latent_k, chunk_q, chunk_k, sm_scale):
    """bsa_bwd_3d: dq, dk, dv in token order from token-order tensors (bsa_interface.py:570-596 between the
    rearrangements of :650-652 and :659, of which only those of q and v are made, inside the call)."""
    _need_gpu(do, q, k, v, o)
    B, H, Sq, D = q.shape
    lib = _capi.load()
    q, k, v, o, do = (_rows_ok(t) for t in (q, k, v, o, do))
    prm = _capi.Bsa3dParams(B, H, D, _code(q), *latent_q, *latent_k, *chunk_q, *chunk_k, 0, float(sm_scale), 0.0)
    width = walk.shape[3]
    need = lib.bsa_bwd_3d_workspace_bytes(C.byref(prm), width)
    if need == 0:        # the call itself names what is wrong with the shape
        _capi.check(lib.bsa_bwd_3d(C.byref(prm), *([None] * 10), None, None, None, width, *([None] * 6), None, 0, None), "bsa_bwd_3d")
        raise RuntimeError("bsa_bwd_3d: no workspace size for this problem")
    ws = _workspace(need, q.device)
    dq, dk, dv = (torch.empty(t.shape, dtype=t.dtype, device=t.device) for t in (q, k, v))
    lse, walk, lens = lse.contiguous(), walk.contiguous(), lens.contiguous()
    st = lambda t: _capi.strides3(t.stride()[:3])
    with torch.cuda.device(q.device):
        _capi.check(lib.bsa_bwd_3d(C.byref(prm), _ptr(q), st(q), _ptr(k), st(k), _ptr(v), st(v), _ptr(o), st(o), _ptr(do), st(do),
                                   _ptr(lse), _ptr(walk), _ptr(lens), width, _ptr(dq), st(dq), _ptr(dk), st(dk), _ptr(dv), st(dv),
                                   _ptr(ws), need, _stream(q)), "bsa_bwd_3d")
    return dq, dk, dv


def _bsa_3d_backward_by_rearranging(do, q, k, v, o, lse, walk, lens, latent_q, latent_k, chunk_q, chunk_k, sm_scale):
    """The same gradients the way a caller of the blocked-order entry points gets them: five rearrangements in
    (bsa_interface.py:650-652 and their like for o and dO), bsa_bwd, three out.  Kept for the tests."""
    bs_q, bs_k = int(math.prod(chunk_q)), int(math.prod(chunk_k))
    qp, _, _ = _permute(q, latent_q, chunk_q)
    kp, _, valid = _permute(k, latent_k, chunk_k, want_valid=True)
    vp, _, _ = _permute(v, latent_k, chunk_k)
    op, _, _ = _permute(o, latent_q, chunk_q)
    dop, _, _ = _permute(do, latent_q, chunk_q)                      # padded slots get a zero gradient
    padded_k = kp.shape[2] != k.shape[2]
    # lse in blocked order; a padded query slot has no keys as far as the backward is concerned (its p is 0)
    slots = _slot_tokens(latent_q, chunk_q, q.device)
    lse_p = torch.where(slots >= 0, lse[..., slots.clamp(min=0)], torch.full((), float("-inf"), device=q.device))
    dqp, dkp, dvp = (torch.empty_like(t) for t in (qp, kp, vp))
    attn_bwd_bsa_varlen(dop, qp, kp, vp, op, dqp, dkp, dvp, sm_scale, lse_p, walk, lens, bs_q, bs_k, None,
                        valid if padded_k else None)
    return _unpermute(dqp, latent_q, chunk_q), _unpermute(dkp, latent_k, chunk_k), _unpermute(dvp, latent_k, chunk_k)


def _unpermute(xp, latent_shape, chunk):
    T, Hh, W = (int(x) for x in latent_shape)
    t, h, w = (int(x) for x in chunk)
    return rearrange_3d_block_to_THW(xp, -(-T // t), -(-Hh // h), -(-W // w), t, h, w, xp.shape[-1], latent_shape=latent_shape)


@torch.library.custom_op("longcat_video_amd::flash_attn_bsa_3d", mutates_args=())
def _bsa_3d_op(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, latent_shape_q: Sequence[int],
               latent_shape_k: Sequence[int], sparsity: float, cdf_threshold: float, chunk_3d_shape_q: Sequence[int],
               chunk_3d_shape_k: Sequence[int]) -> torch.Tensor:
    # a negative sparsity / cdf_threshold stands for None (operator schemas have no optional floats here)
    return _bsa_3d(q, k, v, latent_shape_q, latent_shape_k, None if sparsity < 0 else sparsity, chunk_3d_shape_q,
                   chunk_3d_shape_k, cdf_threshold=None if cdf_threshold < 0 else cdf_threshold)


@_bsa_3d_op.register_fake
def _(q, k, v, latent_shape_q, latent_shape_k, sparsity, cdf_threshold, chunk_3d_shape_q, chunk_3d_shape_k):
    return q.new_empty(q.shape)


def flash_attn_bsa_3d(
    q: torch.Tensor,  # [B, H, Sq, D]
    k: torch.Tensor,  # [B, H, Skv, D]
    v: torch.Tensor,  # [B, H, Skv, D]
    latent_shape_q,
    latent_shape_k,
    # bsa_params
    sparsity=0.875,
    cdf_threshold=None,
    chunk_3d_shape_q=[4, 4, 8],
    chunk_3d_shape_k=[4, 4, 8],
    allow_padding: bool = True,
) -> torch.Tensor:
    """Drop-in for bsa_interface.py:612-660.  q [B,H,Sq,D], k/v [B,H,Skv,D] in
    (T,H,W) token order, any strides with a contiguous D axis; returns a fresh
    contiguous [B,H,Sq,D] tensor of the same dtype."""
    _, _, Sq, head_dim_q = q.shape
    _, _, Sk, head_dim_k = k.shape
    assert head_dim_q == head_dim_k
    assert v.shape == k.shape and k.shape[:2] == q.shape[:2] and q.dtype == k.dtype == v.dtype
    Tq, Hq, Wq = latent_shape_q
    Tk, Hk, Wk = latent_shape_k
    assert Tq * Hq * Wq == Sq
    assert Tk * Hk * Wk == Sk
    tq, hq, wq = chunk_3d_shape_q
    tk, hk, wk = chunk_3d_shape_k
    if not allow_padding:
        assert Tq % tq == 0 and Hq % hq == 0 and Wq % wq == 0
        assert Tk % tk == 0 and Hk % hk == 0 and Wk % wk == 0
    assert head_dim_q in {16, 32, 64, 128, 256}
    if sparsity is None and cdf_threshold is None:
        raise ValueError
    if _wants_grad(q, k, v):
        if q.dtype == torch.float32:
            raise NotImplementedError("the backward is built for bf16 and fp16")
        return _Bsa3dWithGrad.apply(q, k, v, [int(x) for x in latent_shape_q], [int(x) for x in latent_shape_k], sparsity,
                                    cdf_threshold, [int(x) for x in chunk_3d_shape_q], [int(x) for x in chunk_3d_shape_k])
    return _bsa_3d_op(q, k, v, [int(x) for x in latent_shape_q], [int(x) for x in latent_shape_k],
                      -1.0 if sparsity is None else float(sparsity), -1.0 if cdf_threshold is None else float(cdf_threshold),
                      [int(x) for x in chunk_3d_shape_q], [int(x) for x in chunk_3d_shape_k])

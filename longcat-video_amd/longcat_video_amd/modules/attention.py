"""Self-attention module of the LongCat-Video DiT on the MI355X engine.

Mirrors ``Attention`` of the reference (longcat_video/modules/attention.py:14-181):
same constructor arguments, same parameter names (``qkv``, ``q_norm.weight``,
``k_norm.weight``, ``proj``) so a reference state dict loads unchanged, same
``forward(x, shape, num_cond_latents)`` contract.  Every stage runs through the
C-ABI of the engine:

    qkv = Linear(x)                      bsa_linear_bf16   (attention.py:111)
    q, k = RMSNorm(q), RMSNorm(k); RoPE  bsa_norm_rope     (attention.py:116, :121)
    block-sparse attention               bsa_fwd_3d        (attention.py:58-67, :124-137)
    x = Linear(o)                        bsa_linear_bf16   (attention.py:139-142)

q is moved from the token-major projection output into a per-head contiguous
tensor by the same pass that normalises and rotates it (the attention kernel
fetches query rows tile by tile); k is normalised and rotated where it lies and
v is used where it lies, since the operator reads both exactly once, to rewrite
them in the attention kernel's fragment order.  The attention output is written
token-major, so none of
the reference's ``.contiguous()`` / ``cat`` / transpose copies (attention.py:127-135,
:140-141, :166-171) exist here.  Only the block-sparse branch is built: dense back
ends (flash-attn, xformers) raise ``NotImplementedError``.
"""
from __future__ import annotations

import ctypes as C
from typing import List, Optional

import torch
import torch.nn as nn

from .. import _capi
from ..block_sparse_attention.bsa_interface import _bsa_3d, _ptr, _stream


class RMSNorm_FP32(nn.Module):
    """Parameter holder with the reference's name and layout (blocks.py:42-53);
    ``forward`` normalises rows of ``dim`` elements with the engine's kernel."""

    def __init__(self, dim: int, eps: float):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return rms_norm(x, self.weight, self.eps)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    if not x.is_cuda:
        raise RuntimeError("the engine runs on the GPU only")
    x = x.contiguous()
    w = weight.to(x.dtype).contiguous()
    out = torch.empty_like(x)
    dim = x.shape[-1]
    code = {torch.bfloat16: _capi.BSA_BF16, torch.float16: _capi.BSA_F16}.get(x.dtype)
    if code is None:
        raise NotImplementedError("rms_norm: dtype %s is not built (bf16, fp16)" % x.dtype)
    with torch.cuda.device(x.device):
        _capi.check(_capi.load().bsa_rmsnorm(_ptr(x), _ptr(w), _ptr(out), x.numel() // dim, dim, float(eps), code,
                                             _stream(x)), "rmsnorm")
    return out


class _Bounded(dict):
    """A dict that forgets its oldest entry beyond `limit` (insertion order): the caches below are keyed by stream or
    by grid, and a long-lived process that keeps creating streams or changing resolutions must not grow them forever."""

    def __init__(self, limit: int):
        super().__init__()
        self.limit = limit

    def __setitem__(self, key, value):
        if key not in self and len(self) >= self.limit:
            del self[next(iter(self))]
        super().__setitem__(key, value)


_GEMM_WORKSPACES = _Bounded(16)          # 64 MiB each


def _gemm_workspace(device) -> torch.Tensor:
    """64 MiB per device and stream, kept: calls on one stream run one after the other."""
    key = (str(device), torch.cuda.current_stream(device).cuda_stream)
    ws = _GEMM_WORKSPACES.get(key)
    if ws is None:
        ws = _GEMM_WORKSPACES[key] = torch.empty(64 << 20, dtype=torch.uint8, device=device)
    return ws


def linear_bf16(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                residual: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x @ weight.T + bias (+ residual)`` for bf16 tensors, weight in nn.Linear layout [out, in]."""
    if not x.is_cuda:
        raise RuntimeError("the engine runs on the GPU only")
    if x.dtype != torch.bfloat16:
        raise NotImplementedError("linear: only bf16 is built")
    K = x.shape[-1]
    N = weight.shape[0]
    assert weight.shape[1] == K
    x2 = x.reshape(-1, K).contiguous()
    w = weight.to(torch.bfloat16).contiguous()
    b = None if bias is None else bias.to(torch.bfloat16).contiguous()
    if out is None:
        out = torch.empty(x2.shape[0], N, dtype=torch.bfloat16, device=x.device)
    assert out.shape == (x2.shape[0], N) and out.dtype == torch.bfloat16 and out.is_contiguous()
    r = None
    if residual is not None:
        r = residual.reshape(-1, N).contiguous()
        assert r.shape == out.shape and r.dtype == torch.bfloat16
    if workspace is None:
        workspace = _gemm_workspace(x.device)
    with torch.cuda.device(x.device):
        _capi.check(_capi.load().bsa_linear_bf16(_ptr(x2), _ptr(w), _ptr(b), _ptr(r), _ptr(out), x2.shape[0], N, K,
                                                 _ptr(workspace), workspace.numel(), _stream(x)), "linear")
    return out.view(*x.shape[:-1], N)


def tune_linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], residual: bool = False,
                workspace: Optional[torch.Tensor] = None):
    """One-time choice of the GEMM algorithm for ``linear_bf16`` calls of this shape (rows of x, weight shape, bias and
    residual presence): times what hipBLASLt proposes and keeps the fastest for the rest of the process.  Waits for
    the stream; call at set-up.  Returns (algorithms timed, ms of the default choice, ms of the chosen one)."""
    if not x.is_cuda:
        raise RuntimeError("the engine runs on the GPU only")
    K, N = x.shape[-1], weight.shape[0]
    x2 = x.reshape(-1, K).contiguous()
    w = weight.to(torch.bfloat16).contiguous()
    b = None if bias is None else bias.to(torch.bfloat16).contiguous()
    out = torch.empty(x2.shape[0], N, dtype=torch.bfloat16, device=x.device)
    r = torch.zeros_like(out) if residual else None
    if workspace is None:
        workspace = _gemm_workspace(x.device)
    d, best = C.c_float(0), C.c_float(0)
    with torch.cuda.device(x.device):
        n = _capi.load().bsa_linear_bf16_tune(_ptr(x2), K, _ptr(w), K, _ptr(b), _ptr(r), _ptr(out), N, x2.shape[0], N, K,
                                              _ptr(workspace), workspace.numel(), _stream(x), C.byref(d), C.byref(best))
    if n <= 0:
        _capi.check(n if n < 0 else _capi.BSA_ERR_HIP, "linear tune")
    return n, d.value, best.value


def gemm_bf16(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
              residual: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x @ weight.T + bias (+ residual)`` through the engine's own MFMA GEMM (no workspace, nothing allocated by
    the library).  weight [N, K] with N a multiple of 128 and K of 64."""
    if not x.is_cuda:
        raise RuntimeError("the engine runs on the GPU only")
    if x.dtype != torch.bfloat16:
        raise NotImplementedError("gemm: only bf16 is built")
    K, N = x.shape[-1], weight.shape[0]
    assert weight.shape[1] == K
    x2 = x.reshape(-1, K)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    w = weight.to(torch.bfloat16)
    if w.stride(1) != 1:
        w = w.contiguous()
    b = None if bias is None else bias.to(torch.bfloat16).contiguous()
    if out is None:
        out = torch.empty(x2.shape[0], N, dtype=torch.bfloat16, device=x.device)
    assert out.shape == (x2.shape[0], N) and out.dtype == torch.bfloat16 and out.stride(1) == 1
    r, ldr = None, 0
    if residual is not None:
        r = residual.reshape(-1, N)
        assert r.shape == out.shape and r.dtype == torch.bfloat16 and r.stride(1) == 1
        ldr = r.stride(0)
    with torch.cuda.device(x.device):
        _capi.check(_capi.load().bsa_gemm_bf16(_ptr(x2), x2.stride(0), _ptr(w), w.stride(0), _ptr(b), _ptr(r), ldr, _ptr(out),
                                               out.stride(0), x2.shape[0], N, K, _stream(x)), "gemm")
    return out.view(*x.shape[:-1], N)


def qkv_projection(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], q_weight: torch.Tensor,
                   k_weight: torch.Tensor, grid_size, num_heads: int, eps: float = 1e-6, t_offset: int = 0,
                   table_grid=None):
    """attention.py:111-121 in one kernel: the QKV Linear, the split into heads, RMSNorm of q and k per head and
    the 3-D RoPE.  x [B, T*H*W, C]; returns q, k, v as contiguous [B, heads, T*H*W, 128] tensors."""
    if not x.is_cuda:
        raise RuntimeError("the engine runs on the GPU only")
    if x.dtype != torch.bfloat16:
        raise NotImplementedError("qkv_projection: only bf16 is built")
    B, S, K = x.shape
    T, Hg, Wg = (int(g) for g in grid_size)
    assert S == T * Hg * Wg and weight.shape == (3 * num_heads * 128, K)
    table_grid = tuple(int(g) for g in (table_grid if table_grid is not None else grid_size))
    assert table_grid[1:] == (Hg, Wg)
    tab = rope_table(table_grid, 128, x.device)
    x2 = x.reshape(B * S, K)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    w = weight.to(torch.bfloat16)
    if w.stride(1) != 1:
        w = w.contiguous()
    b = None if bias is None else bias.to(torch.bfloat16).contiguous()
    qw, kw = q_weight.to(torch.bfloat16).contiguous(), k_weight.to(torch.bfloat16).contiguous()
    qkv = torch.empty(3, B, num_heads, S, 128, dtype=torch.bfloat16, device=x.device)
    with torch.cuda.device(x.device):
        _capi.check(_capi.load().bsa_qkv_projection(
            _ptr(x2), x2.stride(0), _ptr(w), w.stride(0), _ptr(b), _ptr(qw), _ptr(kw), _ptr(tab), _ptr(qkv[0]), _ptr(qkv[1]),
            _ptr(qkv[2]), _capi.strides3(qkv[0].stride()[:3]), B, num_heads, T, Hg, Wg, int(t_offset), table_grid[0], 128, K,
            float(eps), _stream(x)), "qkv_projection")
    return qkv[0], qkv[1], qkv[2]


_ROPE_TABLES = _Bounded(32)


def rope_table(grid_size, head_dim: int, device, base: float = 10000.0) -> torch.Tensor:
    """cos/sin of position x frequency per axis and rotation pair, following
    rope_3d.py:68-87 (axis dims D-4*(D//6), 2*(D//6), 2*(D//6); frequency i of an
    axis = base^(-2i/dim_axis); integer grid positions), evaluated in fp32 on the
    device like the reference (rope_3d.py:112-115).  Layout: cos_t, sin_t, cos_h,
    sin_h, cos_w, sin_w, each [positions, pairs]."""
    key = (tuple(int(g) for g in grid_size), head_dim, str(device), base)
    tab = _ROPE_TABLES.get(key)
    if tab is None:
        dims = (head_dim - 4 * (head_dim // 6), 2 * (head_dim // 6), 2 * (head_dim // 6))
        parts = []
        for n, dim in zip(key[0], dims):
            freqs = 1.0 / (base ** (torch.arange(0, dim, 2)[: dim // 2].float() / dim))
            ang = (torch.arange(n, dtype=torch.float32)[:, None] * freqs[None, :]).to(device)
            parts += [ang.cos().reshape(-1), ang.sin().reshape(-1)]
        tab = torch.cat(parts).contiguous()
        _ROPE_TABLES[key] = tab
    return tab


def qk_norm_rope_(q: torch.Tensor, k: torch.Tensor, q_weight, k_weight, grid_size, eps: float = 1e-6) -> None:
    """In place on q and k ([B,H,S,128] views, contiguous D): per-head RMSNorm then 3-D RoPE."""
    B, H, S, D = q.shape
    T, Hg, Wg = (int(g) for g in grid_size)
    assert k.shape == q.shape and S == T * Hg * Wg and q.stride(3) == 1 and k.stride(3) == 1
    code = {torch.bfloat16: _capi.BSA_BF16, torch.float16: _capi.BSA_F16}.get(q.dtype)
    if code is None:
        raise NotImplementedError("qk_norm_rope: dtype %s is not built (bf16, fp16)" % q.dtype)
    tab = rope_table(grid_size, D, q.device)
    qw, kw = q_weight.to(q.dtype).contiguous(), k_weight.to(q.dtype).contiguous()
    with torch.cuda.device(q.device):
        _capi.check(_capi.load().bsa_qk_norm_rope(
            _ptr(q), _capi.strides3(q.stride()[:3]), _ptr(k), _capi.strides3(k.stride()[:3]), _ptr(qw), _ptr(kw),
            _ptr(tab), B, H, T, Hg, Wg, D, float(eps), code, _stream(q)), "qk_norm_rope")


def norm_rope(src: torch.Tensor, dst: torch.Tensor, weight=None, grid_size=None, eps: float = 1e-6,
              t_offset: int = 0, table_grid=None) -> torch.Tensor:
    """dst = rope(norm(src)) on [B,H,S,128] tensors or views (contiguous D); `weight` None skips the RMSNorm,
    `grid_size` None skips the rotation, both None copies.  `table_grid`: the grid the rotation angles are
    laid out on when src covers only the frames t_offset .. t_offset + T of it."""
    B, H, S, D = src.shape
    assert dst.shape == src.shape and dst.dtype == src.dtype and src.stride(3) == 1 and dst.stride(3) == 1
    code = {torch.bfloat16: _capi.BSA_BF16, torch.float16: _capi.BSA_F16}.get(src.dtype)
    if code is None:
        raise NotImplementedError("norm_rope: dtype %s is not built (bf16, fp16)" % src.dtype)
    tab, T, Hg, Wg, table_T = None, S, 1, 1, S
    if grid_size is not None:
        T, Hg, Wg = (int(g) for g in grid_size)
        assert S == T * Hg * Wg
        table_grid = tuple(int(g) for g in (table_grid if table_grid is not None else grid_size))
        assert table_grid[1:] == (Hg, Wg)
        tab, table_T = rope_table(table_grid, D, src.device), table_grid[0]
    w = None if weight is None else weight.to(src.dtype).contiguous()
    with torch.cuda.device(src.device):
        _capi.check(_capi.load().bsa_norm_rope(
            _ptr(src), _capi.strides3(src.stride()[:3]), _ptr(dst), _capi.strides3(dst.stride()[:3]), _ptr(w), _ptr(tab),
            B, H, T, Hg, Wg, int(t_offset), table_T, D, float(eps), code, _stream(src)), "norm_rope")
    return dst


class Attention(nn.Module):
    def __init__(
        self,
        dim: int,
        num_heads: int,
        enable_flashattn3: bool = False,
        enable_flashattn2: bool = False,
        enable_xformers: bool = False,
        enable_bsa: bool = False,
        bsa_params: dict = None,
        cp_split_hw: Optional[List[int]] = None,
    ) -> None:
        super().__init__()
        assert dim % num_heads == 0, "dim should be divisible by num_heads"
        self.dim = dim
        self.num_heads = num_heads
        self.head_dim = dim // num_heads
        self.scale = self.head_dim ** -0.5
        self.enable_flashattn3 = enable_flashattn3
        self.enable_flashattn2 = enable_flashattn2
        self.enable_xformers = enable_xformers
        self.enable_bsa = enable_bsa
        self.bsa_params = bsa_params
        self.cp_split_hw = cp_split_hw if cp_split_hw is not None else [1, 1]

        self.qkv = nn.Linear(dim, dim * 3, bias=True)
        self.q_norm = RMSNorm_FP32(self.head_dim, eps=1e-6)
        self.k_norm = RMSNorm_FP32(self.head_dim, eps=1e-6)
        self.proj = nn.Linear(dim, dim)
        # LoRA side branches (lists of modules.lora.LoRABranch), as enable_loras attaches them to
        # `attn.qkv` and `attn.proj` (longcat_video_dit.py:211-232); empty = the plain Linear
        self.qkv_loras = []
        self.proj_loras = []
        # "hipblaslt": the projections through bsa_linear_bf16, norm and rotation as separate passes (the faster
        # route at the 720p shapes); "engine": bsa_qkv_projection (GEMM with norm, rotation and head split in its
        # epilogue) and bsa_gemm_bf16.  Both round at the same points.
        self.projection_backend = "hipblaslt"

    def _linear(self, x, layer, loras, residual=None):
        if any(b.use_lora for b in loras):
            from .lora import lora_linear
            y = lora_linear(x, layer.weight, layer.bias, loras)
            return y if residual is None else y + residual
        if self.projection_backend == "engine" and layer.weight.shape[0] % 128 == 0 and layer.weight.shape[1] % 64 == 0:
            return gemm_bf16(x, layer.weight, layer.bias, residual=residual)
        return linear_bf16(x, layer.weight, layer.bias, residual=residual)

    def _fused_projection(self, x, shape, return_kv):
        """True when the QKV GEMM with the fused epilogue applies: engine backend, no LoRA branch on qkv, no
        k cache wanted (the cache holds k before the rotation, which the fused epilogue does not keep)."""
        return (self.projection_backend == "engine" and not return_kv and self.head_dim == 128 and x.shape[-1] % 64 == 0
                and not any(b.use_lora for b in self.qkv_loras))

    @torch.no_grad()
    def tune(self, x: torch.Tensor, residual: bool = False):
        """Picks the GEMM algorithms of the two projections for inputs shaped like x ([B, N, C]); see tune_linear."""
        a = tune_linear(x, self.qkv.weight, self.qkv.bias)
        b = tune_linear(x, self.proj.weight, self.proj.bias, residual=residual)
        return a, b

    def _process_attn(self, q, k, v, shape, out=None, qk_norm=None):
        """attention.py:50-105, block-sparse branch; writes into `out` ([B,H,SQ,D] view) if given.  `qk_norm`: q and
        k are the raw projections, normalised and rotated inside the operator (see _bsa_3d)."""
        B, H, SQ, D = q.shape
        SKV = k.shape[2]
        if not (self.enable_bsa and shape[0] > 1):
            raise NotImplementedError("only the block-sparse branch (enable_bsa, more than one latent frame) is built")
        assert self.bsa_params is not None
        _, Hh, W = shape
        if self.cp_split_hw[0] * self.cp_split_hw[1] != 1:
            raise NotImplementedError("context parallelism is not built: one GPU holds every head and token")
        Tq, Tk = SQ // (Hh * W), SKV // (Hh * W)
        prm = dict(sparsity=0.875, cdf_threshold=None, chunk_3d_shape_q=[4, 4, 8], chunk_3d_shape_k=[4, 4, 8])
        prm.update(self.bsa_params)
        if prm["sparsity"] is None and prm["cdf_threshold"] is None:
            raise ValueError
        return _bsa_3d(q, k, v, (Tq, Hh, W), (Tk, Hh, W), prm["sparsity"], prm["chunk_3d_shape_q"],
                       prm["chunk_3d_shape_k"], out=out, cdf_threshold=prm["cdf_threshold"], qk_norm=qk_norm)

    def _norm_inside_operator(self, x, shape, num_cond_latents, return_kv):
        """True when q and k can go to the operator as projected: its passes over them (chunk means of q, k into
        the attention kernel's operand order) then apply the norm and the rotation, and the two stand-alone passes
        drop out.  One operator call over the whole grid, 64-token chunks, no k cache wanted."""
        if return_kv or (num_cond_latents is not None and num_cond_latents > 0) or self.head_dim != 128:
            return False
        if not (self.enable_bsa and shape[0] > 1) or x.dtype not in (torch.bfloat16, torch.float16):
            return False
        prm = dict(chunk_3d_shape_q=[4, 4, 8], chunk_3d_shape_k=[4, 4, 8])
        prm.update(self.bsa_params or {})
        fits = lambda c: int(c[0]) * int(c[1]) * int(c[2]) == 64 and max(int(e) for e in c) <= 8
        return fits(prm["chunk_3d_shape_q"]) and fits(prm["chunk_3d_shape_k"])

    def _project_qkv(self, x):
        B, N, C = x.shape
        qkv = self._linear(x, self.qkv, self.qkv_loras)                           # [B, N, 3C]
        return qkv.view(B, N, 3, self.num_heads, self.head_dim).permute(2, 0, 3, 1, 4).unbind(0)   # strided [B,H,N,D] views

    @torch.no_grad()
    def forward(self, x: torch.Tensor, shape=None, num_cond_latents=None, return_kv=False,
                residual: Optional[torch.Tensor] = None):
        """attention.py:107-147.  `residual` (extension): added to the projection output inside the GEMM."""
        B, N, C = x.shape
        Hn, D = self.num_heads, self.head_dim
        eps = self.q_norm.eps
        new = lambda: torch.empty(B, Hn, N, D, dtype=x.dtype, device=x.device)
        if self._fused_projection(x, shape, return_kv):
            q, k, v = qkv_projection(x, self.qkv.weight, self.qkv.bias, self.q_norm.weight, self.k_norm.weight, shape,
                                     Hn, eps=eps)
        elif self._norm_inside_operator(x, shape, num_cond_latents, return_kv):
            # q, k, v stay where the projection left them: the operator's pass over q (chunk means) normalises and
            # rotates it into a per-head tensor of its own, its pass over k (fragment order) does the same on the way
            qs, ks, v = self._project_qkv(x)
            o = torch.empty(B, N, Hn, D, dtype=x.dtype, device=x.device)
            tab = rope_table(shape, D, x.device)
            self._process_attn(qs, ks, v, shape, out=o.permute(0, 2, 1, 3),
                               qk_norm=(self.q_norm.weight, self.k_norm.weight, tab, int(shape[0]), 0, 0, eps))
            return self._linear(o.view(B, N, C), self.proj, self.proj_loras, residual=residual)
        else:
            # q moves into a per-head tensor on the way (the attention kernel fetches its rows tile by tile); k is
            # normed and rotated where it lies and v stays where it is: the operator reads both once, to rewrite
            # them in its fragment order, and a strided read costs that pass less than a separate move costs
            qs, ks, v = self._project_qkv(x)
            q = norm_rope(qs, new(), self.q_norm.weight, shape, eps=eps)
            if return_kv:
                k_cache = norm_rope(ks, new(), self.k_norm.weight, eps=eps)       # attention.py:118-119
                k = norm_rope(k_cache, new(), None, shape)
            else:
                k = norm_rope(ks, ks, self.k_norm.weight, shape, eps=eps)

        o = torch.empty(B, N, Hn, D, dtype=x.dtype, device=x.device)             # token-major: reshape below is free
        ov = o.permute(0, 2, 1, 3)                                                # [B, H, N, D] view
        if num_cond_latents is not None and num_cond_latents > 0:
            n = num_cond_latents * (N // shape[0])
            self._process_attn(q[:, :, :n], k[:, :, :n], v[:, :, :n], shape, out=ov[:, :, :n])   # attention.py:127-130
            self._process_attn(q[:, :, n:], k, v, shape, out=ov[:, :, n:])                       # attention.py:132-133
        else:
            self._process_attn(q, k, v, shape, out=ov)
        y = self._linear(o.view(B, N, C), self.proj, self.proj_loras, residual=residual)
        if return_kv:
            return y, (k_cache, v.contiguous())
        return y

    @torch.no_grad()
    def forward_with_kv_cache(self, x: torch.Tensor, shape=None, num_cond_latents=None, kv_cache=None,
                              residual: Optional[torch.Tensor] = None) -> torch.Tensor:
        """attention.py:149-181: the new tokens attend to the cached conditioning keys/values followed by
        their own.  The cache holds keys after the norm and before the rotation; cached and new keys are
        rotated together on a grid of T + num_cond_latents frames, the queries sit at its last T frames."""
        B, N, C = x.shape
        Hn, D = self.num_heads, self.head_dim
        T, Hg, Wg = (int(g) for g in shape)
        k_cache, v_cache = kv_cache
        assert k_cache.shape[0] == v_cache.shape[0] and k_cache.shape[0] in [1, B]
        if not (num_cond_latents is not None and num_cond_latents > 0):
            # the reference leaves k_full undefined on this path (attention.py:165-173)
            raise ValueError("forward_with_kv_cache needs num_cond_latents > 0")
        n_c = k_cache.shape[2]
        assert n_c == num_cond_latents * Hg * Wg and N == T * Hg * Wg
        qs, ks, vs = self._project_qkv(x)
        eps = self.q_norm.eps
        grid_full = (T + num_cond_latents, Hg, Wg)
        k_full = torch.empty(B, Hn, n_c + N, D, dtype=x.dtype, device=x.device)
        v_full = torch.empty_like(k_full)
        kc = k_cache.to(x.device).expand(B, -1, -1, -1)                            # attention.py:162-164
        vc = v_cache.to(x.device).expand(B, -1, -1, -1)
        # cached keys: rotation only, frames 0 .. num_cond; new keys: norm + rotation at frames num_cond ..
        norm_rope(kc, k_full[:, :, :n_c], None, (num_cond_latents, Hg, Wg), table_grid=grid_full)
        norm_rope(ks, k_full[:, :, n_c:], self.k_norm.weight, shape, eps=eps, t_offset=num_cond_latents, table_grid=grid_full)
        norm_rope(vc, v_full[:, :, :n_c])
        norm_rope(vs, v_full[:, :, n_c:])
        q = norm_rope(qs, torch.empty(B, Hn, N, D, dtype=x.dtype, device=x.device), self.q_norm.weight, shape, eps=eps,
                      t_offset=num_cond_latents, table_grid=grid_full)
        o = torch.empty(B, N, Hn, D, dtype=x.dtype, device=x.device)
        self._process_attn(q, k_full, v_full, shape, out=o.permute(0, 2, 1, 3))
        return self._linear(o.view(B, N, C), self.proj, self.proj_loras, residual=residual)


@torch.no_grad()
def attention_block_forward(x: torch.Tensor, pre_norm_weight: torch.Tensor, attn: Attention, shape,
                            num_cond_latents=None, eps: float = 1e-6) -> torch.Tensor:
    """RMSNorm -> QKV projection -> QK RMSNorm -> 3-D RoPE -> block-sparse attention -> out projection
    -> residual: the attention sub-chain of one DiT block as benchmark configuration 5 words it."""
    y = rms_norm(x, pre_norm_weight, eps)
    return attn(y, shape=shape, num_cond_latents=num_cond_latents, residual=x)


# ---------------------------------------------------------------------------
# adaLN wrapper of the self-attention branch of a DiT block
# ---------------------------------------------------------------------------
def _frames(x: torch.Tensor, mod: torch.Tensor, name: str):
    B, N, C = x.shape
    assert mod.dtype == torch.float32, "%s must be fp32 (blocks.py:129)" % name
    assert mod.dim() == 4 and mod.shape[0] == B and mod.shape[2] == 1 and mod.shape[3] == C, \
        "%s must be [B, T, 1, C]" % name
    T = mod.shape[1]
    assert N % T == 0
    return mod.contiguous(), N // T


def layernorm_modulate(x: torch.Tensor, shift: torch.Tensor, scale: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """modulate_fp32(LayerNorm_FP32(no affine), x.view(B,T,-1,C), shift, scale).view(B,N,C)
    (blocks.py:56-69, 126-134 as called at longcat_video_dit.py:88).  x [B,N,C] bf16/fp16; shift, scale [B,T,1,C] fp32."""
    if not x.is_cuda:
        raise RuntimeError("the engine runs on the GPU only")
    code = {torch.bfloat16: _capi.BSA_BF16, torch.float16: _capi.BSA_F16}.get(x.dtype)
    if code is None:
        raise NotImplementedError("layernorm_modulate: dtype %s is not built (bf16, fp16)" % x.dtype)
    shift, per = _frames(x, shift, "shift")
    scale, _ = _frames(x, scale, "scale")
    x = x.contiguous()
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        _capi.check(_capi.load().bsa_layernorm_modulate(_ptr(x), _ptr(shift), _ptr(scale), _ptr(out), x.shape[0] * x.shape[1],
                                                        per, x.shape[2], float(eps), code, _stream(x)), "layernorm_modulate")
    return out


def gated_residual(x: torch.Tensor, gate: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """(x + gate * y.view(B,-1,N//T,C)).to(x.dtype) of longcat_video_dit.py:101-103; gate [B,T,1,C] fp32."""
    if not x.is_cuda:
        raise RuntimeError("the engine runs on the GPU only")
    code = {torch.bfloat16: _capi.BSA_BF16, torch.float16: _capi.BSA_F16}.get(x.dtype)
    if code is None:
        raise NotImplementedError("gated_residual: dtype %s is not built (bf16, fp16)" % x.dtype)
    gate, per = _frames(x, gate, "gate")
    assert y.shape == x.shape and y.dtype == x.dtype
    x, y = x.contiguous(), y.contiguous()
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        _capi.check(_capi.load().bsa_gated_residual(_ptr(x), _ptr(y), _ptr(gate), _ptr(out), x.shape[0] * x.shape[1], per,
                                                    x.shape[2], code, _stream(x)), "gated_residual")
    return out


@torch.no_grad()
def dit_self_attention_branch(x: torch.Tensor, shift_msa: torch.Tensor, scale_msa: torch.Tensor, gate_msa: torch.Tensor,
                              attn: Attention, latent_shape, num_cond_latents=None, return_kv=False, kv_cache=None):
    """The self-attention branch of LongCatSingleStreamBlock.forward (longcat_video_dit.py:88-103):
    x + gate * attn(modulate(LayerNorm(x), shift, scale)), with the block's three attention routes
    (plain / return_kv / kv_cache).  The modulation vectors come from the caller (adaLN_modulation is a
    small fp32 linear layer outside this path)."""
    x_m = layernorm_modulate(x, shift_msa, scale_msa)
    new_cache = None
    if kv_cache is not None:
        x_s = attn.forward_with_kv_cache(x_m, shape=latent_shape, num_cond_latents=num_cond_latents, kv_cache=kv_cache)
    elif return_kv:
        x_s, new_cache = attn(x_m, shape=latent_shape, num_cond_latents=num_cond_latents, return_kv=True)
    else:
        x_s = attn(x_m, shape=latent_shape, num_cond_latents=num_cond_latents)
    out = gated_residual(x, gate_msa, x_s)
    return (out, new_cache) if return_kv else out

"""LoRA side branches of the attention module's linear layers.

The reference patches the forward of every Linear a LoRA file names (longcat_video_dit.py:211-249):
``org_forward(x) + sum_i lora_up_i(lora_down_i(x)) * multiplier_i * alpha_scale_i``.  ``lora_up`` is either one
Linear or, for fused projections such as qkv, one Linear per equal slice of the output features, each fed its own
slice of the rank axis (lora_utils.py:12-21, 47-53).  Here the three GEMMs go to hipBLASLt through the C ABI (the
sliced up-projection with row strides, in place) and one elementwise pass applies the scaling and the sums with the
eager expression's roundings.
"""
from typing import List, Optional, Sequence

import torch

from .. import _capi
from .attention import _gemm_workspace, _ptr, _stream, linear_bf16

MAX_BRANCHES = 4


class LoRABranch:
    """The tensors of one LoRAModule (lora_utils.py:23-66): ``lora_down.weight`` [n_sep * rank, in],
    ``lora_up`` weights (one [out, rank] matrix, or n_sep matrices [out / n_sep, rank]), the multiplier and
    ``alpha_scale = alpha / rank`` (a buffer the reference casts to the model dtype, longcat_video_dit.py:221)."""

    def __init__(self, lora_down: torch.Tensor, lora_up: Sequence[torch.Tensor], multiplier: float = 1.0,
                 alpha: Optional[float] = None):
        lora_up = list(lora_up) if isinstance(lora_up, (list, tuple)) else [lora_up]
        n = len(lora_up)
        assert n >= 1 and lora_down.shape[0] % n == 0
        self.rank = lora_down.shape[0] // n
        assert all(u.shape == lora_up[0].shape and u.shape[1] == self.rank for u in lora_up)
        self.lora_down = lora_down
        self.lora_up = lora_up
        self.multiplier = multiplier
        alpha = self.rank if alpha is None or alpha == 0 else alpha                 # lora_utils.py:56
        self.alpha_scale = float(alpha) / self.rank
        self.use_lora = True

    @property
    def out_features(self) -> int:
        return self.lora_up[0].shape[0] * len(self.lora_up)

    def to(self, device=None, dtype=None):
        self.lora_down = self.lora_down.to(device=device, dtype=dtype)
        self.lora_up = [u.to(device=device, dtype=dtype) for u in self.lora_up]
        return self


def _up_projection(lx: torch.Tensor, branch: LoRABranch, workspace: torch.Tensor) -> torch.Tensor:
    """lora_up(lx): one GEMM, or one per output slice writing its columns of the result in place."""
    n = len(branch.lora_up)
    if n == 1:
        return linear_bf16(lx, branch.lora_up[0], None, workspace=workspace)
    M, r = lx.shape[0], branch.rank
    per = branch.lora_up[0].shape[0]
    out = torch.empty(M, n * per, dtype=torch.bfloat16, device=lx.device)
    lib = _capi.load()
    with torch.cuda.device(lx.device):
        for i, w in enumerate(branch.lora_up):
            w = w.contiguous()
            _capi.check(lib.bsa_linear_bf16_ld(lx.data_ptr() + 2 * i * r, n * r, _ptr(w), r, None, None,
                                               out.data_ptr() + 2 * i * per, n * per, M, per, r,
                                               _ptr(workspace), workspace.numel(), _stream(lx)), "lora up projection")
    return out


@torch.no_grad()
def lora_linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                loras: Optional[List[LoRABranch]] = None, workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The patched forward of longcat_video_dit.py:234-249 for a bf16 Linear."""
    org = linear_bf16(x, weight, bias, workspace=workspace)
    active = [b for b in (loras or []) if b.use_lora]
    if not active:
        return org                                 # `org_output + 0`
    if len(active) > MAX_BRANCHES:
        raise NotImplementedError("at most %d LoRA branches per Linear are built" % MAX_BRANCHES)
    if workspace is None:
        workspace = _gemm_workspace(x.device)
    N = weight.shape[0]
    x2 = x.reshape(-1, x.shape[-1])
    ups = []
    for b in active:
        assert b.out_features == N and b.lora_down.shape[1] == x.shape[-1]
        if b.lora_down.dtype != torch.bfloat16:
            raise NotImplementedError("LoRA weights must be bf16 (the reference moves them to the model dtype)")
        lx = linear_bf16(x2, b.lora_down, None, workspace=workspace)              # [M, n_sep * rank]
        ups.append(_up_projection(lx, b, workspace))
    import ctypes as C
    n = len(ups)
    up_ptrs = (C.c_void_p * n)(*[u.data_ptr() for u in ups])
    mult = (C.c_float * n)(*[float(b.multiplier) for b in active])
    # alpha_scale lives in a bf16 buffer in the reference
    alpha = (C.c_float * n)(*[float(torch.tensor(b.alpha_scale, dtype=torch.bfloat16)) for b in active])
    out2 = org.view(-1, N)
    with torch.cuda.device(x.device):
        _capi.check(_capi.load().bsa_lora_add(_ptr(out2), up_ptrs, mult, alpha, n, _ptr(out2), out2.numel(),
                                              _capi.BSA_BF16, _stream(x)), "lora_add")
    return org

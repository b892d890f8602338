"""CPU oracle for the LongCat-Video block-sparse attention (BSA) forward path.

THIS FILE IS TEST INFRASTRUCTURE.  It restates, on the CPU, the arithmetic of
the reference's BSA forward so that the HIP engine can be checked against it.
Only tests, the smoke check and the benchmark's CPU-baseline leg may import it;
the product path never does.

Every function names the reference lines it follows (paths relative to the
reference checkout):

  bsa   = longcat_video/block_sparse_attention/bsa_interface.py
  vmask = longcat_video/block_sparse_attention/flash_attn_bsa_varlen_mask.py
  attn  = longcat_video/modules/attention.py
  blocks= longcat_video/modules/blocks.py
  rope  = longcat_video/modules/rope_3d.py

How each function is pinned (the reference ships no tests, golden vectors or
fixtures for this path, so the pins are mathematical; see tests/test_oracle_*):

  permute_index_map / rearrange_*   brute-force triple loop on tiny grids, a
                                    view/permute/contiguous evaluation written
                                    with plain torch ops, bijection + round trip
  mean_pooling_compression          closed form on exactly representable inputs
  cal_score                         integer-valued inputs (exact in fp32)
  num_selected                      literal Python expression incl. the
                                    int((1-0.9)*10)==0 truncation case
  select_topk                       brute-force sorted() on (-score, index),
                                    value multiset equal to torch.topk values
  block_mask_from_indices           brute-force loop
  masked_dense_attention            torch scaled_dot_product_attention on the
                                    dense special case; single-block softmax
  blockwise_attention               agreement with masked_dense_attention;
                                    LSE-merge identity; order invariance
  rms_norm / rope_3d_*              norm preservation, relative-position
                                    property, closed-form frequencies
  select_cdf                        closed forms (equal scores, one dominant
                                    column, log-weights), a Python loop, and
                                    the reference's own library sequence
                                    (softmax, sort, cumsum, searchsorted) on
                                    tie-free fp32 scores
  attention_module_forward_with_kv_cache / attention_module_kv
                                    equality with the noise rows of the split
                                    forward over all frames
  layernorm_modulate_fp32 / gated_residual_fp32
                                    torch F.layer_norm, closed forms
  lora_linear                       zero up-weights (the initial state) give the
                                    plain Linear bit for bit; integer-valued
                                    inputs give the merged weight
                                    W + m*a*U.D exactly; split up-projection ==
                                    one block-diagonal matrix; torch F.linear

  inverse_block_lists               brute-force loop over the mask
  blockwise_attention_backward      torch.autograd through an fp32 masked-dense
                                    softmax attention written with plain torch
                                    ops (an independent derivation): equal to
                                    rounding in fp32, within the stated bf16
                                    tolerance otherwise; finite differences on
                                    a tiny case; delta == rowsum(o * do)
  paced_visit_order                 (no reference counterpart: the reference
                                    visits the selected blocks in list order,
                                    and the result does not depend on that
                                    order beyond rounding) permutation
                                    property, identity on evenly spread lists,
                                    a hand-worked example, a brute-force
                                    sequential restatement

What no CPU check can pin ("parity unpinned", because the reference executes
them inside un-vendored third parties - Triton and ATen/Inductor of torch 2.6 -
and holds no recorded outputs): torch.topk's order among exactly tied scores,
Inductor's summation order inside the pooled mean (last-ulp bf16 flips), the
bit-level output of the Triton attention kernel, and for the CDF rule the order
of torch.sort among equal weights, the fp32 rounding of torch.cumsum next to
the threshold and the storage type of the weights (the reference's bf16 route
does not run).  For those the build rule is
stated in the function's docstring.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import numpy as np
import torch

LOG2E = 1.44269504          # vmask:247, the literal the kernel multiplies sm_scale by
LN2 = 0.6931471824645996    # bsa:338


# --------------------------------------------------------------------------
# R0: shape contract and the padded-grid extension
# --------------------------------------------------------------------------
def ceil_div(a: int, b: int) -> int:
    return -(-a // b)


def block_grid(latent_shape: Sequence[int], chunk: Sequence[int]) -> Tuple[int, int, int]:
    """Number of chunks per axis.  The reference requires divisibility
    (bsa:639-640) and uses exact quotients (bsa:642-648); the build pads each
    axis up at its high end, so the counts are ceilings."""
    return tuple(ceil_div(int(n), int(c)) for n, c in zip(latent_shape, chunk))


def permute_index_map(latent_shape: Sequence[int], chunk: Sequence[int]) -> np.ndarray:
    """Source token index for every destination slot of the blocked order.

    Destination slot order is (Nt, Nh, Nw, t, h, w) and the source order is
    (T, H, W), exactly the view/permute of bsa:600-604; slots that fall outside
    the real grid (padding, an extension the reference does not have) map to -1.
    """
    T, H, W = (int(x) for x in latent_shape)
    t, h, w = (int(x) for x in chunk)
    Nt, Nh, Nw = block_grid(latent_shape, chunk)
    nt, nh, nw, ti, hi, wi = np.meshgrid(
        np.arange(Nt), np.arange(Nh), np.arange(Nw), np.arange(t), np.arange(h), np.arange(w),
        indexing="ij")
    tt = nt * t + ti
    hh = nh * h + hi
    ww = nw * w + wi
    src = (tt * H + hh) * W + ww
    src = np.where((tt < T) & (hh < H) & (ww < W), src, -1)
    return src.reshape(-1).astype(np.int64)


def rearrange_thw_to_3d_block(x: torch.Tensor, latent_shape, chunk) -> torch.Tensor:
    """bsa:600-604 (rearrange_THW_to_3d_block) plus zero-filled padding slots.
    x: [B, H, S, D] -> [B, H, S_padded, D]."""
    idx = torch.from_numpy(permute_index_map(latent_shape, chunk))
    safe = idx.clamp(min=0)
    out = x[:, :, safe, :].clone()
    out[:, :, idx < 0, :] = 0
    return out.contiguous()


def rearrange_3d_block_to_thw(x: torch.Tensor, latent_shape, chunk) -> torch.Tensor:
    """bsa:606-610 (rearrange_3d_block_to_THW); padding slots are dropped.
    x: [B, H, S_padded, D] -> [B, H, S, D]."""
    idx = torch.from_numpy(permute_index_map(latent_shape, chunk))
    S = int(np.prod([int(v) for v in latent_shape]))
    out = torch.empty(x.shape[0], x.shape[1], S, x.shape[3], dtype=x.dtype)
    real = idx >= 0
    out[:, :, idx[real], :] = x[:, :, real, :]
    return out


def slot_validity(latent_shape, chunk) -> np.ndarray:
    """bool per blocked slot: True where the slot holds a real token."""
    return permute_index_map(latent_shape, chunk) >= 0


# --------------------------------------------------------------------------
# R2-R4: gating (pool, score, top-k)
# --------------------------------------------------------------------------
def mean_pooling_compression(x: torch.Tensor, block_size: int) -> torch.Tensor:
    """bsa:168-178.  Zero-pads S to a block multiple, then the mean over each
    block, returned in the input dtype.  The sum is taken in fp32 and rounded
    once; the order of the fp32 sum is not fixed by the reference (Inductor
    picks it), so for non-representable inputs the last bf16 bit is unpinned."""
    B, H, S, D = x.shape
    nb = math.ceil(S / block_size)
    xf = x.float()
    if S % block_size != 0:
        xf = torch.nn.functional.pad(xf, (0, 0, 0, nb * block_size - S))
    return xf.view(B, H, nb, block_size, D).mean(dim=3).to(x.dtype)


def cal_score(q_cmp: torch.Tensor, k_cmp: torch.Tensor) -> torch.Tensor:
    """bsa:180-184.  Unscaled q_cmp @ k_cmp^T, fp32 accumulate, one rounding to
    the input dtype."""
    return torch.matmul(q_cmp.float(), k_cmp.float().transpose(-1, -2)).to(q_cmp.dtype)


def num_selected(sparsity: float, n_kv_blocks: int) -> int:
    """bsa:214, evaluated in Python doubles with truncation."""
    return int((1 - sparsity) * n_kv_blocks)


def select_topk(score: torch.Tensor, k_sel: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """bsa:212-224.  Returns (indices int64 [B,H,nbq,k_sel] in descending score
    order, lens int32 [B,H,nbq] all equal to k_sel).  torch.topk leaves the order
    among equal scores unspecified; the build rule is: ties go to the lowest
    index, i.e. the order key is (-score, index).  NaN scores are rejected."""
    s = score.float().numpy()
    if np.isnan(s).any():
        raise ValueError("NaN score")
    order = np.argsort(-s, axis=-1, kind="stable")       # stable => lowest index first among ties
    idx = torch.from_numpy(np.ascontiguousarray(order[..., :k_sel]).astype(np.int64))
    lens = torch.full(score.shape[:3], k_sel, dtype=torch.int32)
    return idx, lens


def select_cdf(score: torch.Tensor, cdf_threshold: float, sm_scale: float, k_min: int = 0, cap: int = None):
    """bsa:233-243 (and bsa:252-266 with k_min = the top-k count): weights = softmax(score * sm_scale),
    columns sorted by descending weight, cdf = cumsum, lens = searchsorted(cdf, threshold, right=True) = the
    number of cdf entries <= threshold, raised to k_min.  Returns (indices int64 [B,H,nbq,nbk] in the full
    sorted order, lens int32, cdf float64 in sorted order).
    Build rules where the reference leaves freedom or cannot run: the sort key is (-score, index) (torch.sort
    leaves ties unspecified; the softmax is monotone in the score); the weights are fp32 for every score
    dtype (the reference's bf16 route stops at a dtype check inside torch.searchsorted, bsa:236-241); the
    running sum is kept in float64, so a row can differ from an fp32 running sum only where that sum comes
    within rounding of the threshold.  `cap` limits lens (the engine's own entry points take a list width)."""
    s = score.float()
    w = torch.softmax(s * sm_scale, dim=-1)
    order = np.argsort(-s.numpy(), axis=-1, kind="stable")
    idx = torch.from_numpy(np.ascontiguousarray(order).astype(np.int64))
    cdf = torch.cumsum(torch.gather(w, -1, idx).double(), dim=-1)
    lens = (cdf <= float(np.float32(cdf_threshold))).sum(-1)
    lens = torch.clamp(lens, min=int(k_min))
    if cap is not None:
        lens = torch.clamp(lens, max=int(cap))
    return idx, lens.to(torch.int32), cdf


def block_mask_from_indices(idx: torch.Tensor, lens: torch.Tensor, n_cols: int) -> torch.Tensor:
    """bsa:131-149 (create_mask_from_indices_varlen), restricted to the first
    lens[b,h,m] entries of each row as the forward kernel does (vmask:250-252)."""
    B, H, M, K = idx.shape
    mask = torch.zeros(B, H, M, n_cols, dtype=torch.bool)
    pos = torch.arange(K).view(1, 1, 1, K)
    use = (pos < lens.unsqueeze(-1).long()) & (idx < n_cols) & (idx >= 0)
    b, h, m, j = torch.nonzero(use, as_tuple=True)
    mask[b, h, m, idx[b, h, m, j].long()] = True
    return mask


# --------------------------------------------------------------------------
# R6: attention itself
# --------------------------------------------------------------------------
def masked_dense_attention(q, k, v, block_mask, bs_q: int, bs_k: int, sm_scale: float,
                           key_valid: Optional[torch.Tensor] = None,
                           heads: Optional[Sequence[int]] = None,
                           q_blocks: Optional[Sequence[int]] = None):
    """The tolerance oracle: fp32 softmax(Q K^T * sm_scale + mask) V over the
    blocked layout, one query block at a time.

    q [B,H,Sq,D], k/v [B,H,Sk,D] in blocked order; block_mask [B,H,nbq,nbk];
    key_valid [Sk] bool (False = padded slot, gets -inf).  Returns
    (o fp32 [B,H,Sq,D], lse fp32 [B,H,Sq], natural log).  Rows of query blocks
    not in `q_blocks` / heads not in `heads` are left at zero / -inf.
    A row with no admissible key gives o = 0 and lse = -inf, which is what the
    kernel's initial state m=-inf, l=1, acc=0 produces (vmask:242-244, 281-282).
    """
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    nbq, nbk = Sq // bs_q, Sk // bs_k
    o = torch.zeros(B, H, Sq, D, dtype=torch.float32)
    lse = torch.full((B, H, Sq), -math.inf, dtype=torch.float32)
    heads = range(H) if heads is None else heads
    q_blocks = range(nbq) if q_blocks is None else q_blocks
    for b in range(B):
        for h in heads:
            kf = k[b, h].float()
            vf = v[b, h].float()
            for m in q_blocks:
                qs = q[b, h, m * bs_q:(m + 1) * bs_q].float()
                logits = (qs @ kf.t()) * sm_scale
                allow = block_mask[b, h, m].repeat_interleave(bs_k)
                if key_valid is not None:
                    allow = allow & key_valid
                logits = logits.masked_fill(~allow.unsqueeze(0), -math.inf)
                row_lse = torch.logsumexp(logits, dim=-1)
                p = torch.exp(logits - torch.where(torch.isinf(row_lse), torch.zeros_like(row_lse), row_lse).unsqueeze(-1))
                p = torch.where(allow.unsqueeze(0), p, torch.zeros_like(p))
                o[b, h, m * bs_q:(m + 1) * bs_q] = p @ vf
                lse[b, h, m * bs_q:(m + 1) * bs_q] = row_lse
    return o, lse


def gathered_attention(q, k, v, idx, lens, bs_q: int, bs_k: int, sm_scale: float,
                       key_valid: Optional[torch.Tensor] = None,
                       heads: Optional[Sequence[int]] = None,
                       q_blocks: Optional[Sequence[int]] = None):
    """Same mathematics as masked_dense_attention, evaluated only over the
    selected key blocks (masked entries contribute exactly zero, so the two are
    equal up to fp32 summation order).  Used where the dense form is too large."""
    B, H, Sq, D = q.shape
    nbq = Sq // bs_q
    o = torch.zeros(B, H, Sq, D, dtype=torch.float32)
    lse = torch.full((B, H, Sq), -math.inf, dtype=torch.float32)
    heads = range(H) if heads is None else heads
    q_blocks = range(nbq) if q_blocks is None else q_blocks
    ar = torch.arange(bs_k)
    for b in range(B):
        for h in heads:
            for m in q_blocks:
                n = int(lens[b, h, m])
                if n == 0:
                    continue
                blocks = torch.unique(idx[b, h, m, :n].long())      # a mask has no duplicates
                rows = (blocks.unsqueeze(1) * bs_k + ar.unsqueeze(0)).reshape(-1)
                if key_valid is not None:
                    rows = rows[key_valid[rows]]
                if rows.numel() == 0:
                    continue
                qs = q[b, h, m * bs_q:(m + 1) * bs_q].float()
                logits = (qs @ k[b, h, rows].float().t()) * sm_scale
                row_lse = torch.logsumexp(logits, dim=-1)
                p = torch.exp(logits - row_lse.unsqueeze(-1))
                o[b, h, m * bs_q:(m + 1) * bs_q] = p @ v[b, h, rows].float()
                lse[b, h, m * bs_q:(m + 1) * bs_q] = row_lse
    return o, lse


def blockwise_attention(q, k, v, idx, lens, bs_q: int, bs_k: int, sm_scale: float,
                        key_valid: Optional[torch.Tensor] = None):
    """Step-by-step restatement of the forward kernel's numerics, vmask:242-285:
    one selected key block per iteration in list order, logits from an fp32
    accumulate, scale sm_scale*LOG2E applied after the dot, exp2, running max
    and sum in fp32 starting from m=-inf, l=1, P rounded to the input dtype
    before P@V, epilogue acc/l and M = m + log2(l).  Returns (o in the input
    dtype, lse = M*LN2 fp32 as bsa:338-339).  Padded keys (extension) get -inf."""
    B, H, Sq, D = q.shape
    nbq = Sq // bs_q
    dt = q.dtype
    o = torch.empty(B, H, Sq, D, dtype=dt)
    M = torch.empty(B, H, Sq, dtype=torch.float32)
    qk_scale = sm_scale * LOG2E
    for b in range(B):
        for h in range(H):
            for mblk in range(nbq):
                qs = q[b, h, mblk * bs_q:(mblk + 1) * bs_q].float()
                m_i = torch.full((bs_q,), -math.inf)
                l_i = torch.ones(bs_q)
                acc = torch.zeros(bs_q, D)
                for i in range(int(lens[b, h, mblk])):
                    j = int(idx[b, h, mblk, i])
                    ks = k[b, h, j * bs_k:(j + 1) * bs_k].float()
                    vs = v[b, h, j * bs_k:(j + 1) * bs_k]
                    qk = qs @ ks.t()
                    if key_valid is not None:
                        kvld = key_valid[j * bs_k:(j + 1) * bs_k]
                        qk = qk.masked_fill(~kvld.unsqueeze(0), -math.inf)
                    m_ij = torch.maximum(m_i, qk.max(dim=1).values * qk_scale)
                    safe = torch.where(torch.isinf(m_ij), torch.zeros_like(m_ij), m_ij)
                    p = torch.exp2(qk * qk_scale - safe.unsqueeze(1))
                    alpha = torch.exp2(m_i - safe)
                    l_ij = p.sum(dim=1)
                    acc = acc * alpha.unsqueeze(1) + p.to(dt).float() @ vs.float()
                    l_i = l_i * alpha + l_ij
                    m_i = m_ij
                M[b, h, mblk * bs_q:(mblk + 1) * bs_q] = m_i + torch.log2(l_i)
                o[b, h, mblk * bs_q:(mblk + 1) * bs_q] = (acc / l_i.unsqueeze(1)).to(dt)
    return o, M * LN2


# --------------------------------------------------------------------------
# backward (bsa:341-461, vmask:288-945)
# --------------------------------------------------------------------------
RCP_LN2 = 1.4426950408889634     # bsa:359, 369


def inverse_block_lists(idx: torch.Tensor, lens: torch.Tensor, n_kv_blocks: int):
    """create_indices_k_from_indices_q_varlen, bsa:152-165: for every KV block the query blocks that selected it,
    ascending.  Returns (lists [B,H,nbk,nbq] int64 padded with nbq, counts [B,H,nbk])."""
    mask = block_mask_from_indices(idx, lens, n_kv_blocks)              # [B,H,nbq,nbk]
    B, H, nbq, nbk = mask.shape
    mk = mask.permute(0, 1, 3, 2)
    ids = torch.arange(nbq).view(1, 1, 1, -1).expand_as(mk)
    lists = torch.where(mk, ids, torch.full_like(ids, nbq)).sort(dim=-1).values
    return lists, (lists < nbq).sum(dim=-1)


def blockwise_attention_backward(q, k, v, o, do, lse, idx, lens, bs_q: int, bs_k: int, sm_scale: float,
                                 key_valid: Optional[torch.Tensor] = None, q_blocks=None, kv_blocks=None):
    """Restatement of the reference backward's numerics (bsa:341-461; kernels vmask:288-360, 428-462, wrappers
    vmask:630-642, 943-945):
      M2 = lse * RCP_LN2 (fp32); k_s = k * (sm_scale * RCP_LN2) in k's dtype (one rounding, bsa:369-370);
      delta = rowsum(o * do) in fp32 (common.py:105-109);
      per (query block, selected KV block): s = q . k_s^T (fp32), p = exp2(s - M2), dp = do . v^T (fp32),
      ds = p * (dp - delta) rounded to the storage type, p rounded to the storage type for dV;
      dV = sum p^T do, dK = (sum ds^T q) * sm_scale, dQ = (sum ds k_s) * LN2, fp32 accumulators, one final rounding.
    dQ walks a row's blocks in list order, dK / dV walk the query blocks of a KV block in ascending order
    (bsa:389-392); fp32 summation order inside a product is free.  Padded keys (extension) have p = 0.  Lists name
    a block at most once (a selection does); the reference gives a repeated block no consistent meaning.
    q_blocks / kv_blocks (optional, for problems too large to evaluate in full): only the dQ rows of these query
    blocks and the dK / dV rows of these KV blocks are computed, each from all of its pairs; every other row of
    the result stays zero.
    Returns (dq, dk, dv) in the input dtype."""
    B, H, Sq, D = q.shape
    Sk = k.shape[2]
    nbq, nbk = Sq // bs_q, Sk // bs_k
    dt = q.dtype
    ln2 = 0.6931471824645996                                  # vmask:943 (tl.constexpr LN2)
    m2 = lse.float() * RCP_LN2
    k_s = k * (sm_scale * RCP_LN2)                            # stays in k's dtype
    delta = (o.float() * do.float()).sum(-1)
    dq = torch.zeros(B, H, Sq, D, dtype=torch.float32)
    dk = torch.zeros(B, H, Sk, D, dtype=torch.float32)
    dv = torch.zeros(B, H, Sk, D, dtype=torch.float32)
    q_todo = range(nbq) if q_blocks is None else sorted(set(int(m) for m in q_blocks))
    kv_todo = range(nbk) if kv_blocks is None else sorted(set(int(j) for j in kv_blocks))

    def selectors(b, h, j):
        """Query blocks of (b, h) whose list names KV block j, ascending (bsa:152-165 for one column)."""
        live = torch.arange(idx.shape[-1]).unsqueeze(0) < lens[b, h].long().unsqueeze(1)
        return torch.nonzero(((idx[b, h] == j) & live).any(dim=1)).flatten().tolist()

    def pair(b, h, m, j):
        qs = q[b, h, m * bs_q:(m + 1) * bs_q]
        ks = k_s[b, h, j * bs_k:(j + 1) * bs_k]
        vs = v[b, h, j * bs_k:(j + 1) * bs_k]
        dos = do[b, h, m * bs_q:(m + 1) * bs_q]
        s = qs.float() @ ks.float().t()
        p = torch.exp2(s - m2[b, h, m * bs_q:(m + 1) * bs_q].unsqueeze(1))
        if key_valid is not None:
            p = torch.where(key_valid[j * bs_k:(j + 1) * bs_k].unsqueeze(0), p, torch.zeros_like(p))
        dp = dos.float() @ vs.float().t()
        ds = (p * (dp - delta[b, h, m * bs_q:(m + 1) * bs_q].unsqueeze(1))).to(dt)
        return qs, ks, dos, p.to(dt), ds

    for b in range(B):
        for h in range(H):
            for m in q_todo:                                                # dQ: list order (vmask:469-499)
                for i in range(int(lens[b, h, m])):
                    j = int(idx[b, h, m, i])
                    qs, ks, dos, p, ds = pair(b, h, m, j)
                    dq[b, h, m * bs_q:(m + 1) * bs_q] += ds.float() @ ks.float()
            for j in kv_todo:                                               # dK, dV: ascending query blocks (vmask:327-356)
                for m in selectors(b, h, j):
                    qs, ks, dos, p, ds = pair(b, h, m, j)
                    dv[b, h, j * bs_k:(j + 1) * bs_k] += p.float().t() @ dos.float()
                    dk[b, h, j * bs_k:(j + 1) * bs_k] += ds.float().t() @ qs.float()
    return (dq * ln2).to(dt), (dk * sm_scale).to(dt), dv.to(dt)


def masked_dense_attention_autograd(q, k, v, do, block_mask, bs_q: int, bs_k: int, sm_scale: float,
                                    key_valid: Optional[torch.Tensor] = None):
    """The tolerance oracle of the backward: gradients of fp32 softmax(Q K^T * sm_scale + mask) V by
    torch.autograd.  Returns (dq, dk, dv) fp32."""
    qf, kf, vf = (t.detach().float().requires_grad_(True) for t in (q, k, v))
    allow = block_mask.repeat_interleave(bs_q, dim=2).repeat_interleave(bs_k, dim=3)
    if key_valid is not None:
        allow = allow & key_valid.view(1, 1, 1, -1)
    logits = (qf @ kf.transpose(-1, -2)) * sm_scale
    logits = logits.masked_fill(~allow, -math.inf)
    none = ~allow.any(-1, keepdim=True)
    p = torch.softmax(logits.masked_fill(none, 0.0), dim=-1)
    p = torch.where(allow, p, torch.zeros_like(p))
    out = p @ vf
    out.backward(do.float())
    return qf.grad, kf.grad, vf.grad


PACE_WIDTH = 8


def paced_visit_order(blocks: np.ndarray, n_kv_blocks: int, width: int = PACE_WIDTH) -> np.ndarray:
    """Order in which the engine's attention kernel visits one query block's selected KV blocks.  The
    reference visits them in list order (vmask:249-285) and softmax(QK^T)V does not depend on the
    order beyond fp rounding, so the engine is free to choose one; it chooses the order that keeps
    the query blocks that run side by side on the GPU at the same place of the KV sequence, which is
    what lets them share K/V tiles in the L2 cache.

    `blocks`: the n selected block indices in ascending order.  Visit slots are cut into groups of
    `width`; group g belongs to the blocks whose index b falls in the g-th n/width-th of the KV
    sequence, g = min(b*n // (n_kv_blocks*width), groups-1).  A group takes its own blocks in
    ascending order up to its number of slots; the blocks over that number, in ascending order over
    the whole list, fill the slots that groups with too few blocks leave empty, in ascending slot
    order; finally every group's slots are put in ascending block order.  Lists of at most `width`
    blocks stay as they are."""
    blocks = np.asarray(blocks)
    n = len(blocks)
    if n <= width:
        return blocks.copy()
    groups = -(-n // width)
    g = np.minimum(blocks.astype(np.int64) * n // (n_kv_blocks * width), groups - 1)
    slots = np.full(n, -1, dtype=np.int64)
    spare = []
    for grp in range(groups):
        own = blocks[g == grp]
        room = min(width, n - grp * width)
        slots[grp * width:grp * width + min(len(own), room)] = own[:room]
        spare.extend(own[room:])
    slots[slots < 0] = spare
    for grp in range(groups):
        slots[grp * width:(grp + 1) * width] = np.sort(slots[grp * width:(grp + 1) * width])
    return slots.astype(blocks.dtype)


def merge_partial_attention(o_a, lse_a, o_b, lse_b):
    """The LSE-merge identity of bsa:490-527 (softmax_lse_correction and
    out_correction): lse = logaddexp(lse_a, lse_b), o = sum_i o_i*exp(lse_i-lse)."""
    lse = torch.logaddexp(lse_a, lse_b)
    safe = torch.where(torch.isinf(lse), torch.zeros_like(lse), lse)
    wa = torch.exp(lse_a - safe).unsqueeze(-1)
    wb = torch.exp(lse_b - safe).unsqueeze(-1)
    return o_a.float() * wa + o_b.float() * wb, lse


# --------------------------------------------------------------------------
# R8/R9: the operator
# --------------------------------------------------------------------------
def flash_attn_bsa(q, k, v, chunk_size_q, chunk_size_k, sparsity, sm_scale,
                   key_valid: Optional[torch.Tensor] = None, exact_kernel_numerics: bool = False):
    """bsa:535-568 forward with cdf_threshold=None: pool, score, top-k, attention.
    Returns (o fp32 or input dtype, lse, idx, lens, score)."""
    q_cmp = mean_pooling_compression(q, chunk_size_q)
    k_cmp = mean_pooling_compression(k, chunk_size_k)
    score = cal_score(q_cmp, k_cmp)
    k_sel = num_selected(sparsity, score.shape[-1])
    idx, lens = select_topk(score, k_sel)
    if exact_kernel_numerics:
        o, lse = blockwise_attention(q, k, v, idx, lens, chunk_size_q, chunk_size_k, sm_scale, key_valid)
    else:
        mask = block_mask_from_indices(idx, lens, score.shape[-1])
        o, lse = masked_dense_attention(q, k, v, mask, chunk_size_q, chunk_size_k, sm_scale, key_valid)
    return o, lse, idx, lens, score


def flash_attn_bsa_3d(q, k, v, latent_shape_q, latent_shape_k, sparsity=0.875,
                      chunk_3d_shape_q=(4, 4, 8), chunk_3d_shape_k=(4, 4, 8)):
    """bsa:612-660 with cdf_threshold=None, extended to grids that are not chunk
    multiples (pad high, zero tokens, padded keys masked, padded queries dropped).
    Returns o fp32 [B,H,Sq,D] in (T,H,W) order plus the selection for inspection."""
    D = q.shape[-1]
    assert int(np.prod(latent_shape_q)) == q.shape[2] and int(np.prod(latent_shape_k)) == k.shape[2]
    qp = rearrange_thw_to_3d_block(q, latent_shape_q, chunk_3d_shape_q)
    kp = rearrange_thw_to_3d_block(k, latent_shape_k, chunk_3d_shape_k)
    vp = rearrange_thw_to_3d_block(v, latent_shape_k, chunk_3d_shape_k)
    kvalid = torch.from_numpy(slot_validity(latent_shape_k, chunk_3d_shape_k))
    cs_q = int(np.prod(chunk_3d_shape_q))
    cs_k = int(np.prod(chunk_3d_shape_k))
    o, lse, idx, lens, score = flash_attn_bsa(qp, kp, vp, cs_q, cs_k, sparsity, 1 / D ** 0.5,
                                              key_valid=None if bool(kvalid.all()) else kvalid)
    out = rearrange_3d_block_to_thw(o, latent_shape_q, chunk_3d_shape_q)
    return out, idx, lens, score


# --------------------------------------------------------------------------
# R10: conditioning / noise split
# --------------------------------------------------------------------------
def cond_noise_split_attention(q, k, v, shape, num_cond_latents, **bsa_params):
    """attn:124-135: conditioning queries attend within the conditioning tokens,
    noise queries attend to all tokens; outputs concatenated along S."""
    T, Hh, W = shape
    n = num_cond_latents * Hh * W
    o_c, *_ = flash_attn_bsa_3d(q[:, :, :n], k[:, :, :n], v[:, :, :n],
                                (num_cond_latents, Hh, W), (num_cond_latents, Hh, W), **bsa_params)
    o_n, *_ = flash_attn_bsa_3d(q[:, :, n:], k, v, (T - num_cond_latents, Hh, W), (T, Hh, W), **bsa_params)
    return torch.cat([o_c, o_n], dim=2)


# --------------------------------------------------------------------------
# R11: glue of the attention module
# --------------------------------------------------------------------------
def rms_norm_fp32(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """blocks:42-53: fp32 x*rsqrt(mean(x^2)+eps), cast to x.dtype, times weight."""
    xf = x.float()
    y = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype)
    return y * weight


def rope_3d_angles(grid_size, head_dim: int = 128, base: float = 10000.0) -> torch.Tensor:
    """rope:68-97.  Angle table [T*H*W, head_dim] in fp32; per-axis dims
    dim_t = D - 4*(D//6), dim_h = dim_w = 2*(D//6); frequency i of an axis is
    base^(-2i/dim_axis); every frequency is repeated for its (even, odd) pair;
    the three axes are concatenated as (t, h, w) along D."""
    T, Hh, W = grid_size
    dim_t = head_dim - 4 * (head_dim // 6)
    dim_h = 2 * (head_dim // 6)
    dim_w = 2 * (head_dim // 6)

    def axis(n, dim):
        freqs = 1.0 / (base ** (torch.arange(0, dim, 2)[: dim // 2].float() / dim))
        pos = torch.arange(n, dtype=torch.float32)
        return torch.repeat_interleave(pos[:, None] * freqs[None, :], 2, dim=-1)

    ft, fh, fw = axis(T, dim_t), axis(Hh, dim_h), axis(W, dim_w)
    ang = torch.cat([
        ft[:, None, None, :].expand(T, Hh, W, dim_t),
        fh[None, :, None, :].expand(T, Hh, W, dim_h),
        fw[None, None, :, :].expand(T, Hh, W, dim_w)], dim=-1)
    return ang.reshape(T * Hh * W, head_dim)


def rope_3d_apply(x: torch.Tensor, angles: torch.Tensor) -> torch.Tensor:
    """rope:34-38, 112-120: x*cos + rotate_half(x)*sin in fp32 with interleaved
    pairs (x0,x1)->(-x1,x0), cast back to x.dtype.  x: [B,H,S,D]."""
    xf = x.float()
    cos, sin = angles.cos()[None, None], angles.sin()[None, None]
    x1, x2 = xf[..., 0::2], xf[..., 1::2]
    rot = torch.stack((-x2, x1), dim=-1).reshape(xf.shape)
    return (xf * cos + rot * sin).to(x.dtype)


def attention_module_forward(x, w_qkv, b_qkv, w_proj, b_proj, q_norm_w, k_norm_w, shape,
                             num_heads: int, bsa_params: dict, num_cond_latents: int = 0,
                             qkv_loras=(), proj_loras=()):
    """attn:107-147 (Attention.forward) with the BSA branch of attn:58-67.
    x [B,N,C]; weights in nn.Linear layout [out,in].  Linear layers accumulate in
    fp32 and round once to x.dtype, as a bf16 GEMM does.  qkv_loras / proj_loras: side
    branches on the two Linears in the form lora_linear takes."""
    B, N, C = x.shape
    D = C // num_heads
    dt = x.dtype
    qkv = lora_linear(x.reshape(B * N, C), w_qkv, b_qkv, qkv_loras).view(B, N, 3 * C)
    qkv = qkv.view(B, N, 3, num_heads, D).permute(2, 0, 3, 1, 4)
    q, k, v = qkv.unbind(0)
    q, k = rms_norm_fp32(q, q_norm_w), rms_norm_fp32(k, k_norm_w)
    ang = rope_3d_angles(shape, D)
    q, k = rope_3d_apply(q, ang), rope_3d_apply(k, ang)
    if num_cond_latents:
        o = cond_noise_split_attention(q, k, v, shape, num_cond_latents, **bsa_params)
    else:
        o, *_ = flash_attn_bsa_3d(q, k, v, shape, shape, **bsa_params)
    o = o.to(dt).transpose(1, 2).reshape(B, N, C)
    return lora_linear(o.reshape(B * N, C), w_proj, b_proj, proj_loras).view(B, N, C)


def attention_module_kv(x, w_qkv, b_qkv, q_norm_w, k_norm_w, num_heads: int):
    """attn:110-119 with return_kv: the cache holds k after the RMSNorm and before the rotation, and v."""
    B, N, C = x.shape
    D = C // num_heads
    qkv = (x.float() @ w_qkv.float().t() + b_qkv.float()).to(x.dtype)
    _, k, v = qkv.view(B, N, 3, num_heads, D).permute(2, 0, 3, 1, 4).unbind(0)
    return rms_norm_fp32(k, k_norm_w).clone(), v.clone()


def attention_module_forward_with_kv_cache(x, w_qkv, b_qkv, w_proj, b_proj, q_norm_w, k_norm_w, shape,
                                           num_heads: int, bsa_params: dict, num_cond_latents: int, kv_cache):
    """attn:149-181 (Attention.forward_with_kv_cache), BSA branch.  x holds the T*H*W new tokens; the
    cache holds num_cond_latents frames.  Keys: cat(cache, new) rotated on a grid of T + num_cond frames
    (attn:166-170); queries: the last N positions of that grid (attn:168-171); attention with
    Tq = T and Tk = T + num_cond (attn:173, 60-61)."""
    B, N, C = x.shape
    D = C // num_heads
    dt = x.dtype
    T, Hh, W = shape
    qkv = (x.float() @ w_qkv.float().t() + b_qkv.float()).to(dt)
    q, k, v = qkv.view(B, N, 3, num_heads, D).permute(2, 0, 3, 1, 4).unbind(0)
    q, k = rms_norm_fp32(q, q_norm_w), rms_norm_fp32(k, k_norm_w)
    k_cache, v_cache = kv_cache
    if k_cache.shape[0] == 1:
        k_cache, v_cache = k_cache.repeat(B, 1, 1, 1), v_cache.repeat(B, 1, 1, 1)
    k_full = torch.cat([k_cache, k], dim=2)
    v_full = torch.cat([v_cache, v], dim=2)
    ang = rope_3d_angles((T + num_cond_latents, Hh, W), D)
    k_full = rope_3d_apply(k_full, ang)
    q = rope_3d_apply(q, ang[-N:])
    o, *_ = flash_attn_bsa_3d(q, k_full, v_full, (T, Hh, W), (T + num_cond_latents, Hh, W), **bsa_params)
    o = o.to(dt).transpose(1, 2).reshape(B, N, C)
    return (o.float() @ w_proj.float().t() + b_proj.float()).to(dt)


def layernorm_modulate_fp32(x: torch.Tensor, shift: torch.Tensor, scale: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """modulate_fp32 (blocks.py:126-134) around LayerNorm_FP32 without affine parameters (blocks.py:56-69), as
    called at longcat_video_dit.py:88: x [B,N,C] viewed as [B,T,N/T,C]; shift, scale [B,T,1,C] fp32; the
    statistics, the product with (scale + 1) and the sum are fp32, one rounding to x.dtype."""
    B, N, C = x.shape
    T = shift.shape[1]
    xf = x.float().view(B, T, N // T, C)
    mean = xf.mean(-1, keepdim=True)
    var = ((xf - mean) ** 2).mean(-1, keepdim=True)
    n = (xf - mean) * torch.rsqrt(var + eps)
    return (n * (scale.float() + 1) + shift.float()).to(x.dtype).view(B, N, C)


def gated_residual_fp32(x: torch.Tensor, gate: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """longcat_video_dit.py:101-103: x + gate * y in fp32 (gate [B,T,1,C] fp32), one rounding to x.dtype."""
    B, N, C = x.shape
    T = gate.shape[1]
    out = x.float().view(B, T, N // T, C) + gate.float() * y.float().view(B, T, N // T, C)
    return out.view(B, N, C).to(x.dtype)


def lora_linear(x, weight, bias, loras):
    """The patched Linear forward of longcat_video_dit.py:234-249: org_output + sum over the active branches of
    lora_up(lora_down(x)) * multiplier * alpha_scale, every tensor op rounding to x.dtype (GEMMs accumulate
    in fp32 and round once; the two scalings and the sums round one by one; `0 + first` is exact).
    loras: sequence of (lora_down [n*r, in], [lora_up_i [out/n, r]] * n, multiplier, alpha_scale); the up
    projection of a fused layer is one Linear per chunk of the rank axis, results concatenated
    (lora_utils.py:12-21).  alpha_scale is held in x.dtype (longcat_video_dit.py:221 casts the buffer)."""
    dt = x.dtype
    lin = lambda a, w: (a.float() @ w.float().t()).to(dt)
    org = (x.float() @ weight.float().t() + (0 if bias is None else bias.float())).to(dt)
    total = None
    for down, ups, multiplier, alpha_scale in loras:
        lx = lin(x, down)
        chunks = torch.chunk(lx, len(ups), dim=-1)
        lx = torch.cat([lin(c, u) for c, u in zip(chunks, ups)], dim=-1)
        a = torch.tensor(alpha_scale, dtype=dt).float()
        term = ((lx.float() * float(torch.tensor(multiplier, dtype=torch.float32))).to(dt).float() * a).to(dt)
        total = term if total is None else (total.float() + term.float()).to(dt)
    return org if total is None else (org.float() + total.float()).to(dt)


"""Benchmark of the block-sparse attention forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c2|c4|c5]

A step is one pass of the whole operator (chunk mean pooling of q and k, pooled
scores, top-k, block-sparse flash attention that gathers its tiles from the
(T,H,W) token order and writes the output back in that order) over one
synthetic attention layer that is already resident in HBM.  Rank 0 prints ONE
JSON line.  `value` is the sparse-actual TFLOP/s of the whole operator (only the
FLOPs of the selected block pairs are counted; everything else in the step is
overhead that lowers it).  `roofline` covers the dominant kernel, timed on its
own with HIP events on the launch stream; `cpu_baseline` times the CPU oracle's
masked-dense evaluation on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "longcat-video_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_BF16_TFLOPS = 2500.0      # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E

WORKLOADS = {
    # name: (latent grid, sparsity, seed, rms-normalised q/k, description)
    "c2": ((24, 30, 52), 0.9375, 1, False, "480p layer: 32 heads x 128, grid 24x30x52 (37440 tokens), density 1/16"),
    "c3": ((24, 45, 80), 0.9375, 2, True, "720p layer: 32 heads x 128, grid 24x45x80 (86400 tokens), density 1/16"),
}
# Bytes that leave L2 per layer in the attention kernel (all of its launches), from rocprofv3 --pmc
# FETCH_SIZE (x2) and WRITE_SIZE (x1) as recorded in profiles/bsa_operator_c3_720p.md: 45 launches
# x (1286.6 MB + 15.7 MB).  Re-measure after kernel changes.
ATTENTION_TRAFFIC_BYTES = {"c3": 45 * (1286.6e6 + 15.7e6)}
CHUNK = (4, 4, 4)
HEADS, D = 32, 128


def make_inputs(torch, latent, seed, rms):
    S = latent[0] * latent[1] * latent[2]
    g = torch.Generator(device="cuda").manual_seed(seed)
    out = []
    for i in range(3):
        x = torch.randn(1, HEADS, S, D, generator=g, device="cuda")
        if rms and i < 2:
            x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)
        out.append(x.bfloat16())
        del x
    return out


def make_coherent_inputs(torch, latent, seed):
    """q = k = smooth functions of the grid position plus noise (per-head random low frequencies), v random:
    pooled scores then fall off with distance, so neighbouring query blocks select largely the same KV blocks,
    as attention over real video does.  Not the headline workload; shows the kernel when tiles are shared."""
    T, H, W = latent
    g = torch.Generator(device="cuda").manual_seed(seed)
    ax = lambda n, shape: torch.arange(n, device="cuda").view(shape).expand(T, H, W).reshape(-1, 1).float() / 4
    pos = torch.cat([ax(T, (T, 1, 1)), ax(H, (1, H, 1)), ax(W, (1, 1, W))], 1)          # in chunks
    q = torch.empty(1, HEADS, T * H * W, D, dtype=torch.bfloat16, device="cuda")
    for h in range(HEADS):
        freq = torch.randn(3, D, generator=g, device="cuda") * 0.3
        phase = torch.rand(1, D, generator=g, device="cuda") * 2 * math.pi
        x = torch.cos(pos @ freq + phase) * math.sqrt(2) + torch.randn(pos.shape[0], D, generator=g, device="cuda")
        q[0, h] = (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6)).bfloat16()
    v = torch.randn(1, HEADS, T * H * W, D, generator=g, device="cuda").bfloat16()
    return q, q.clone(), v


def time_events(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps      # ms per call


def cpu_baseline(torch, latent, sparsity, seed, rms, budget_s):
    """The oracle's masked-dense evaluation of the same layer on the host cores:
    pool -> score -> top-k -> block mask -> fp32 softmax(QK^T/sqrt(D) + mask)V.
    One head is prepared in full; query blocks are evaluated until the time
    budget is spent, then scaled linearly to all heads and query blocks."""
    from oracle import bsa_oracle as O
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    S = latent[0] * latent[1] * latent[2]
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(1, 1, S, D, generator=g) for _ in range(3))
    if rms:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + 1e-6)
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + 1e-6)
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    t0 = time.perf_counter()
    qp = O.rearrange_thw_to_3d_block(q, latent, CHUNK)
    kp = O.rearrange_thw_to_3d_block(k, latent, CHUNK)
    vp = O.rearrange_thw_to_3d_block(v, latent, CHUNK)
    score = O.cal_score(O.mean_pooling_compression(qp, 64), O.mean_pooling_compression(kp, 64))
    nbq, nbk = score.shape[-2:]
    k_sel = O.num_selected(sparsity, nbk)
    idx, lens = O.select_topk(score, k_sel)
    mask = O.block_mask_from_indices(idx, lens, nbk)
    kvalid = torch.from_numpy(O.slot_validity(latent, CHUNK))
    t_head_setup = time.perf_counter() - t0
    done, t_attn = 0, 0.0
    O.masked_dense_attention(qp, kp, vp, mask, 64, 64, 1 / math.sqrt(D), key_valid=kvalid, q_blocks=[0])   # warm-up
    while done < nbq and t_attn < budget_s:
        blocks = list(range(done, min(done + 8, nbq)))
        t0 = time.perf_counter()
        O.masked_dense_attention(qp, kp, vp, mask, 64, 64, 1 / math.sqrt(D), key_valid=kvalid, q_blocks=blocks)
        t_attn += time.perf_counter() - t0
        done += len(blocks)
    layer_s = HEADS * (t_head_setup + t_attn * nbq / done)
    flop = HEADS * nbq * k_sel * 4 * 64 * 64 * D
    return {
        "value": flop / layer_s / 1e12, "unit": "TFLOP/s (sparse-actual)", "cores": cores, "kind": "port",
        "ms_per_layer": layer_s * 1e3,
        "sample": "1 of %d heads: permute+pool+score+top-k in full (%.2f s), masked-dense fp32 attention on %d of %d "
                  "query blocks against all keys (%.2f s); scaled linearly to %d heads x %d query blocks"
                  % (HEADS, t_head_setup, done, nbq, t_attn, HEADS, nbq),
    }


def run_c4(torch, args):
    """benchmark configuration 4: long-video continuation, grid 48x30x52 with 12 conditioning frames.  Two operator
    calls per layer as in attention.py:124-135, writing into one output buffer."""
    from longcat_video_amd.block_sparse_attention import bsa_interface as I
    T, Hh, W, cond = 48, 30, 52, 12
    S, n = T * Hh * W, cond * Hh * W
    q, k, v = make_inputs(torch, (T, Hh, W), 3, False)
    out = torch.empty(1, S, HEADS, D, dtype=torch.bfloat16, device="cuda").permute(0, 2, 1, 3)

    def step():
        I._bsa_3d(q[:, :, :n], k[:, :, :n], v[:, :, :n], (cond, Hh, W), (cond, Hh, W), 0.875, CHUNK, CHUNK, out=out[:, :, :n])
        I._bsa_3d(q[:, :, n:], k, v, (T - cond, Hh, W), (T, Hh, W), 0.875, CHUNK, CHUNK, out=out[:, :, n:])
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    pairs = HEADS * (312 * 39 + 936 * 156)
    flop = pairs * 4 * 64 * 64 * D
    print(json.dumps({
        "metric": "BSA fwd ms/layer + sparse TFLOPS, long-video continuation (cond/noise split)", "value": round(flop / ms / 1e9, 2),
        "unit": "TFLOP/s (sparse-actual, both operator calls)", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic N(0,1) q/k/v, seeded on the GPU",
        "config": {"workload": "c4: 32 heads x 128, grid 48x30x52 (74880 tokens), 12 conditioning frames, density 1/8",
                   "block_pairs": pairs},
        "pct_of_bf16_peak_whole_operator": round(100 * flop / ms / 1e9 / PEAK_BF16_TFLOPS, 2)}))


def run_c5(torch, args):
    """benchmark configuration 5: the attention sub-chain of one DiT block at 720p: RMSNorm -> QKV projection ->
    per-head RMSNorm + 3-D RoPE -> block-sparse attention -> output projection + residual (dim 4096)."""
    from longcat_video_amd.modules import attention as M
    latent = WORKLOADS["c3"][0]
    N, C = latent[0] * latent[1] * latent[2], HEADS * D
    g = torch.Generator(device="cuda").manual_seed(4)
    x = torch.randn(1, N, C, generator=g, device="cuda").bfloat16()
    attn = M.Attention(C, HEADS, enable_bsa=True,
                       bsa_params=dict(sparsity=0.9375, chunk_3d_shape_q=list(CHUNK), chunk_3d_shape_k=list(CHUNK))).cuda().bfloat16()
    for prm in attn.parameters():
        prm.data = (torch.randn(prm.shape, generator=g, device="cuda") * 0.02).bfloat16() if prm.dim() > 1 else torch.zeros_like(prm)
    attn.q_norm.weight.data.fill_(1.0)
    attn.k_norm.weight.data.fill_(1.0)
    w_pre = torch.ones(C, dtype=torch.bfloat16, device="cuda")
    # one-time set-up: GEMM algorithm choice per projection shape (skipped under a profiler to keep its tables short)
    tuned = ((0, 0.0, 0.0), (0, 0.0, 0.0)) if args.no_gemm_tuning else attn.tune(x, residual=True)
    for _ in range(args.warmup):
        M.attention_block_forward(x, w_pre, attn, latent)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        y = M.attention_block_forward(x, w_pre, attn, latent)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    assert torch.isfinite(y.float()).all()
    bsa_flop = HEADS * 1440 * 90 * 4 * 64 * 64 * D
    gemm_flop = 2 * N * C * 3 * C + 2 * N * C * C
    ms_qkv = time_events(torch, lambda: M.linear_bf16(x, attn.qkv.weight, attn.qkv.bias), 5, 2)
    print(json.dumps({
        "metric": "attention sub-chain of a DiT block, ms/layer + TFLOPS (GEMMs + sparse-actual attention)",
        "value": round((bsa_flop + gemm_flop) / ms / 1e9, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic N(0,1) activations, N(0,0.02) weights, zero biases, unit norm weights",
        "config": {"workload": "c5: x [1, 86400, 4096] bf16, 32 heads x 128, grid 24x45x80, density 1/16"},
        "qkv_gemm_ms": round(ms_qkv, 4), "qkv_gemm_tflops": round(2 * N * C * 3 * C / ms_qkv / 1e9, 1),
        "gemm_tuning": {"qkv": {"algorithms_timed": tuned[0][0], "default_ms": round(tuned[0][1], 4), "chosen_ms": round(tuned[0][2], 4)},
                        "proj": {"algorithms_timed": tuned[1][0], "default_ms": round(tuned[1][1], 4), "chosen_ms": round(tuned[1][2], 4)}},
        "pct_of_bf16_peak": round(100 * (bsa_flop + gemm_flop) / ms / 1e9 / PEAK_BF16_TFLOPS, 2)}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS) + ["c4", "c5"],
                    help="c3 is the headline (default); c2 the same operator at 480p; c4 and c5 print a reduced line "
                         "for the cond/noise split and for the attention module")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="time budget of the CPU baseline's attention sample")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-gemm-tuning", action="store_true", help="c5: leave the GEMM algorithm choice to hipBLASLt's first proposal")
    ap.add_argument("--data", default="random", choices=["random", "coherent"],
                    help="random (the benchmark's definition) or spatially coherent q/k (c2, c3 only; no CPU baseline)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (the operator shards over heads; "
                 "run one process per GPU on its own heads). Use --gpus 1.")

    import torch
    from longcat_video_amd.block_sparse_attention import bsa_interface as I

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (there is no CPU path to measure)")
    torch.cuda.set_device(0)
    if args.workload == "c4":
        return run_c4(torch, args)
    if args.workload == "c5":
        return run_c5(torch, args)
    latent, sparsity, seed, rms, desc = WORKLOADS[args.workload]
    coherent = args.data == "coherent"
    q, k, v = make_coherent_inputs(torch, latent, seed) if coherent else make_inputs(torch, latent, seed, rms)
    prm = dict(sparsity=sparsity, chunk_3d_shape_q=list(CHUNK), chunk_3d_shape_k=list(CHUNK))

    # ---- whole operator: warm-up, then exactly K timed steps between synchronisations ----
    for _ in range(args.warmup):
        I.flash_attn_bsa_3d(q, k, v, latent, latent, **prm)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        o = I.flash_attn_bsa_3d(q, k, v, latent, latent, **prm)
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # ---- per-kernel timing with events on the launch stream ----
    # the attention kernel exactly as the operator runs it: same lists (ascending block order), same
    # THW-order addressing, workspace prepared once outside the timed region
    _, idx_score, lens, _ = I._bsa_3d(q, k, v, latent, latent, sparsity, CHUNK, CHUNK, want_selection=True)
    idx = idx_score.sort(dim=-1).values.contiguous()
    del idx_score
    nbq, k_sel = idx.shape[2], idx.shape[3]
    ksteps, kwarm = max(args.steps, 5), max(min(args.warmup, 3), 1)
    attend = I.ThwAttention(k, v, latent, latent, CHUNK, CHUNK)
    o_buf = torch.empty_like(q)
    ms_attn = time_events(torch, lambda: attend(q, idx, lens, out=o_buf), ksteps, kwarm)
    assert torch.equal(o_buf, o), "the separately timed attention kernel must reproduce the operator's output"
    del attend, o_buf
    # the other entry points on their own (the permutes are no longer part of the operator for bf16)
    qp, q_cmp, _ = I._permute(q, latent, CHUNK, want_pooled=True)
    _, k_cmp, _ = I._permute(k, latent, CHUNK, want_pooled=True)
    nbk = k_cmp.shape[2]
    ms_permute = time_events(torch, lambda: I._permute(k, latent, CHUNK, want_pooled=True), ksteps, kwarm)
    ms_unpermute = time_events(torch, lambda: I.rearrange_3d_block_to_THW(qp, *[-(-n // c) for n, c in zip(latent, CHUNK)], *CHUNK, D, latent_shape=latent), ksteps, kwarm)
    ms_select = time_events(torch, lambda: I._score_topk(q_cmp, k_cmp, k_sel, order="block"), ksteps, kwarm)   # as the operator runs it

    S = q.shape[2]
    Sp = qp.shape[2]
    pairs = HEADS * nbq * k_sel
    flop = pairs * 4 * 64 * 64 * D
    dense_flop = 4 * HEADS * S * S * D
    tflops_step = flop / (ms_step * 1e-3) / 1e12
    tflops_attn = flop / (ms_attn * 1e-3) / 1e12
    es = 2
    permute_bytes = HEADS * (S + Sp) * D * es

    result = {
        "metric": "BSA fwd ms/layer + sparse TFLOPS (% bf16 MFMA peak) at " + ("720p 86.4k tokens" if args.workload == "c3" else "480p 37.4k tokens"),
        "value": round(tflops_step, 2),
        "unit": "TFLOP/s (sparse-actual, whole operator)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16",
        "data": ("synthetic, spatially coherent q = k (smooth in the grid position + noise, RMS-normalised), random v, seeded on the GPU"
                 if coherent else
                 "synthetic N(0,1) q/k/v%s, seeded on the GPU" % (" with per-head RMS-normalised q/k" if rms else "")),
        "config": {"workload": "%s: %s" % (args.workload, desc), "chunk": list(CHUNK), "kv_blocks": nbk, "k_sel": k_sel,
                   "block_pairs": pairs, "padded_tokens": Sp},
        "ms_per_layer": round(ms_step, 4),
        "pct_of_bf16_peak_whole_operator": round(100 * tflops_step / PEAK_BF16_TFLOPS, 2),
        "dense_equivalent_tflops": round(dense_flop / (ms_step * 1e-3) / 1e12, 1),
        "kernels_ms": {"attention": round(ms_attn, 4), "score_topk": round(ms_select, 4),
                       "pool_q_k_and_edge_copies (step - attention - score_topk)": round(ms_step - ms_attn - ms_select, 4)},
        "standalone_ms": {"permute_pool_one_tensor": round(ms_permute, 4), "unpermute": round(ms_unpermute, 4)},
        "permute_gbs": round(permute_bytes / (ms_permute * 1e-3) / 1e9, 1),
        "roofline": {"kernel": "fwd_mfma_kernel<bf16> (all launches of one layer)", "bound": "mfma", "achieved": round(tflops_attn, 2),
                     "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(tflops_attn / PEAK_BF16_TFLOPS, 4),
                     "traffic": None if coherent else ATTENTION_TRAFFIC_BYTES.get(args.workload), "ms": round(ms_attn, 4)},
    }
    del o
    if not args.no_cpu_baseline and not coherent:
        result["cpu_baseline"] = cpu_baseline(torch, latent, sparsity, seed, rms, args.cpu_seconds)
        result["cpu_baseline"]["value"] = round(result["cpu_baseline"]["value"], 5)
        result["cpu_baseline"]["ms_per_layer"] = round(result["cpu_baseline"]["ms_per_layer"], 1)
    print(json.dumps(result))


if __name__ == "__main__":
    main()

"""Benchmark of the block-sparse attention forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c2|c4|c5|bwd]

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
ATTENTION_KERNEL = "fwd_frag_kernel<bf16> (all launches of one layer)"
# what the attention kernel's traffic depends on: the kernel and its helpers, the visiting order of the lists it walks,
# and the layer that decides rounds per launch and whether the visiting order runs
ATTENTION_SOURCES = [os.path.join(ROOT, "longcat-video_amd", "csrc", f)
                     for f in ("bsa_fwd_frag.hip", "bsa_select.hip", "bsa_mfma.h", "bsa_common.h", "bsa_capi.hip")]


def source_sha16(paths=ATTENTION_SOURCES):
    import hashlib
    h = hashlib.sha256()
    for path in paths:
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


BACKWARD_SOURCES = [os.path.join(ROOT, "longcat-video_amd", "csrc", "bsa_bwd.hip")]


def recorded_traffic(workload, summaries="bsa_operator_%s_*.md", sources=ATTENTION_SOURCES):
    """HBM-side bytes per layer of the workload's dominant kernels (rocprofv3 FETCH_SIZE / WRITE_SIZE, scaled as the
    profile summary says), as recorded in a summary under profiles/ on a line
    `traffic_record: {"workload": ..., "source_sha16": ..., "bytes_per_layer": ...}` - or None when there is no
    record for this workload or the kernel source has changed since it was taken (a stale figure is not reported)."""
    import glob
    for path in glob.glob(os.path.join(ROOT, "profiles", summaries % workload if "%s" in summaries else summaries)):
        with open(path) as f:
            for line in f:
                if line.startswith("traffic_record:"):
                    rec = json.loads(line[len("traffic_record:"):])
                    if rec.get("workload") == workload and rec.get("source_sha16") == source_sha16(sources):
                        return float(rec["bytes_per_layer"])
    return None


CHUNK = (4, 4, 4)
HEADS, D = 32, 128
DRAWN = {"host": "drawn in fp32 by torch's CPU generator (seeded) and moved to the GPU", "device": "drawn in fp32 by the GPU's generator (seeded)"}


def kv_blocks(latent):
    return math.prod(-(-n // c) for n, c in zip(latent, CHUNK))


def operator_lists(I, idx_score_order, lens, latent_k):
    """The lists as the operator hands them to its attention kernel: ascending block order, then its visiting order."""
    return I.visit_order(idx_score_order.sort(dim=-1).values.int().contiguous(), lens, kv_blocks(latent_k))


def make_inputs(torch, latent, seed, rms, where="device"):
    """q, k, v ~ N(0, 1) in fp32 from one seeded generator, q and k optionally RMS-normalised per head, cast to bf16.
    where = "host": drawn by torch's CPU generator (the same numbers on every machine) and moved to the GPU;
    "device": drawn by the GPU's generator (seconds faster; used for the side figures)."""
    S = latent[0] * latent[1] * latent[2]
    g = torch.Generator(device="cuda" if where == "device" else "cpu").manual_seed(seed)
    out = []
    for i in range(3):
        if where == "device":
            x = torch.randn(1, HEADS, S, D, generator=g, device="cuda")
        else:
            x = torch.randn(1, HEADS, S, D, generator=g).cuda()
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


def time_events(torch, fn, steps, warmup, settle_s=0.0):
    """Average ms per call over `steps` calls between two events on the current stream, after `warmup` calls.
    settle_s > 0: keep warming up until that much wall time has passed and time at least that long as well, so that
    a kernel of a millisecond or two is measured at the clock it settles at, not on the ramp after an idle phase."""
    t0 = time.perf_counter()
    done = 0
    while done < warmup or time.perf_counter() - t0 < settle_s:
        fn()
        done += 1
        if done % 8 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    if settle_s > 0 and done > 0:
        per_call = (time.perf_counter() - t0) / done
        steps = max(steps, int(settle_s / max(per_call, 1e-6)) + 1)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps      # ms per call


def cpu_attention_sample(torch, q, k, v, latent_q, latent_k, sparsity, budget_s):
    """One head of one operator call on the host cores through the oracle: permute, pool, score, top-k in full,
    then masked-dense fp32 attention on as many query blocks as the time budget allows.  q [1,1,Sq,D], k, v
    [1,1,Sk,D].  Returns (seconds for the whole head, extrapolated linearly over its query blocks; set-up seconds;
    attention seconds spent; query blocks evaluated; query blocks in all; blocks kept per row)."""
    from oracle import bsa_oracle as O
    t0 = time.perf_counter()
    qp = O.rearrange_thw_to_3d_block(q, latent_q, CHUNK)
    kp = O.rearrange_thw_to_3d_block(k, latent_k, CHUNK)
    vp = O.rearrange_thw_to_3d_block(v, latent_k, CHUNK)
    score = O.cal_score(O.mean_pooling_compression(qp, 64), O.mean_pooling_compression(kp, 64))
    nbq, nbk = score.shape[-2:]
    k_sel = O.num_selected(sparsity, nbk)
    idx, lens = O.select_topk(score, k_sel)
    mask = O.block_mask_from_indices(idx, lens, nbk)
    kvalid = torch.from_numpy(O.slot_validity(latent_k, CHUNK))
    t_setup = time.perf_counter() - t0
    done, t_attn = 0, 0.0
    O.masked_dense_attention(qp, kp, vp, mask, 64, 64, 1 / math.sqrt(D), key_valid=kvalid, q_blocks=[0])   # warm-up
    while done < nbq and t_attn < budget_s:
        blocks = list(range(done, min(done + 8, nbq)))
        t0 = time.perf_counter()
        O.masked_dense_attention(qp, kp, vp, mask, 64, 64, 1 / math.sqrt(D), key_valid=kvalid, q_blocks=blocks)
        t_attn += time.perf_counter() - t0
        done += len(blocks)
    return t_setup + t_attn * nbq / done, t_setup, t_attn, done, nbq, k_sel


def host_inputs(torch, S, seed, rms):
    """One head of q, k, v drawn on the host: the same distribution as the GPU leg's inputs, a separate draw."""
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(1, 1, S, D, generator=g) for _ in range(3))
    if rms:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + 1e-6)
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + 1e-6)
    return q.bfloat16(), k.bfloat16(), v.bfloat16()


def cpu_baseline(torch, latent, sparsity, seed, rms, budget_s):
    """The oracle's masked-dense evaluation of the same layer on the host cores:
    pool -> score -> top-k -> block mask -> fp32 softmax(QK^T/sqrt(D) + mask)V.
    One head is prepared in full; query blocks are evaluated until the time
    budget is spent, then scaled linearly to all heads and query blocks."""
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    q, k, v = host_inputs(torch, latent[0] * latent[1] * latent[2], seed, rms)
    head_s, t_setup, t_attn, done, nbq, k_sel = cpu_attention_sample(torch, q, k, v, latent, latent, sparsity, budget_s)
    layer_s = HEADS * head_s
    flop = HEADS * nbq * k_sel * 4 * 64 * 64 * D
    return {
        "value": round(flop / layer_s / 1e12, 5), "unit": "TFLOP/s (sparse-actual)", "cores": cores, "kind": "port",
        "ms_per_layer": round(layer_s * 1e3, 1),
        "sample": "1 of %d heads, inputs drawn on the host from the same distribution as the GPU leg's (a separate "
                  "draw, not the same tensors): permute+pool+score+top-k in full (%.2f s), masked-dense fp32 attention "
                  "on %d of %d query blocks against all keys (%.2f s); scaled linearly to %d heads x %d query blocks"
                  % (HEADS, t_setup, done, nbq, t_attn, HEADS, nbq),
    }


def attention_roofline(flop, ms, workload, coherent=False):
    tflops = flop / (ms * 1e-3) / 1e12
    return {"kernel": ATTENTION_KERNEL, "bound": "mfma", "achieved": round(tflops, 2), "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s", "frac": round(tflops / PEAK_BF16_TFLOPS, 4),
            "traffic": None if coherent else recorded_traffic(workload), "ms": round(ms, 4)}


def measure_c4(torch, steps, warmup, settle, where):
    """Both operator calls of configuration 4 (attention.py:124-135) into one output buffer: ms per layer of the operator
    and of its attention kernel alone (the operator's own lists; its output is asserted to be reproduced)."""
    from longcat_video_amd.block_sparse_attention import bsa_interface as I
    T, Hh, W, cond = 48, 30, 52, 12
    S, n = T * Hh * W, cond * Hh * W
    q, k, v = make_inputs(torch, (T, Hh, W), 3, False, where)
    out = torch.empty(1, S, HEADS, D, dtype=torch.bfloat16, device="cuda").permute(0, 2, 1, 3)
    calls = [((q[:, :, :n], k[:, :, :n], v[:, :, :n]), (cond, Hh, W), (cond, Hh, W), out[:, :, :n]),
             ((q[:, :, n:], k, v), (T - cond, Hh, W), (T, Hh, W), out[:, :, n:])]

    def step():
        for (a, b, c), lq, lk, o in calls:
            I._bsa_3d(a, b, c, lq, lk, 0.875, CHUNK, CHUNK, out=o)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    want = out.clone()
    # the attention kernel of both calls on its own, with the operator's lists
    ms_attn = 0.0
    for (a, b, c), lq, lk, o in calls:
        _, idx, lens, _ = I._bsa_3d(a, b, c, lq, lk, 0.875, CHUNK, CHUNK, want_selection=True)
        idx = operator_lists(I, idx, lens, lk)
        attend = I.ThwAttention(b, c, lq, lk, CHUNK, CHUNK)
        ms_attn += time_events(torch, lambda: attend(a, idx, lens, out=o), max(steps, 20), 5, settle_s=settle)
        del attend
    assert torch.equal(out, want), "the separately timed attention kernel must reproduce the operator's output"
    pairs = HEADS * (312 * 39 + 936 * 156)
    return ms, ms_attn, pairs, (T, Hh, W, cond, S, n)


def sample_clocks(torch, fn, seconds=3.0):
    """Runs fn back to back for `seconds` while a thread asks `rocm-smi` (a child process) for the shader clock every
    0.3 s: what the kernel settles at once the power controller has acted."""
    import re
    import subprocess
    import threading
    samples, stop = [], threading.Event()

    def sampler():
        while not stop.is_set():
            try:
                text = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=10).stdout
                sclk = re.findall(r"sclk clock level: \d+: \((\d+)Mhz\)", text)
                samples.append(int(sclk[0]) if sclk else None)
            except Exception:
                samples.append(None)
            stop.wait(0.3)
    th = threading.Thread(target=sampler)
    t0, calls = time.perf_counter(), 0
    th.start()
    while time.perf_counter() - t0 < seconds:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()
        calls += 8
    ms = (time.perf_counter() - t0) * 1e3 / calls
    stop.set()
    th.join()
    samples = samples[1:] or samples                # the first reading may precede the load
    return {"ms_per_call_in_this_loop": round(ms, 4), "sclk_mhz": samples, "nominal_sclk_mhz": 2400,
            "how": "rocm-smi --showclocks every 0.3 s while the attention kernel runs back to back"}


def measure_operator(torch, workload, steps, warmup, settle, where, coherent=False, clocks=None):
    """One of the single-call workloads: ms per layer of the whole operator over exactly `steps` timed calls, and of its
    attention kernel alone exactly as the operator runs it (same lists in the same visiting order, same (T, H, W)
    addressing, workspace prepared outside the timed region; its output is asserted equal to the operator's)."""
    from longcat_video_amd.block_sparse_attention import bsa_interface as I
    latent, sparsity, seed, rms, desc = WORKLOADS[workload]
    q, k, v = make_coherent_inputs(torch, latent, seed) if coherent else make_inputs(torch, latent, seed, rms, where)
    prm = dict(sparsity=sparsity, chunk_3d_shape_q=list(CHUNK), chunk_3d_shape_k=list(CHUNK))
    for _ in range(warmup):
        I.flash_attn_bsa_3d(q, k, v, latent, latent, **prm)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        o = I.flash_attn_bsa_3d(q, k, v, latent, latent, **prm)
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / steps
    _, idx_score, lens, _ = I._bsa_3d(q, k, v, latent, latent, sparsity, CHUNK, CHUNK, want_selection=True)
    idx = operator_lists(I, idx_score, lens, latent)
    del idx_score
    attend = I.ThwAttention(k, v, latent, latent, CHUNK, CHUNK)
    o_buf = torch.empty_like(q)
    ms_attn = time_events(torch, lambda: attend(q, idx, lens, out=o_buf), max(steps, 20), max(warmup, 5), settle_s=settle)
    assert torch.equal(o_buf, o), "the separately timed attention kernel must reproduce the operator's output"
    if clocks is not None:
        clocks.update(sample_clocks(torch, lambda: attend(q, idx, lens, out=o_buf)))
    del attend, o_buf, o
    return ms_step, ms_attn, idx.shape[2], idx.shape[3], (q, k, v)


def other_configurations(torch, args):
    """The attention kernel (and the operator around it) at the other operator configurations, for the default line:
    a few seconds of GPU time each, inputs drawn on the device, no CPU leg."""
    out = {}
    ms_step, ms_attn, nbq, k_sel, qkv = measure_operator(torch, "c2", 10, 3, args.settle, "device")
    del qkv
    flop = HEADS * nbq * k_sel * 4 * 64 * 64 * D
    out["c2"] = {"workload": WORKLOADS["c2"][4], "operator_ms": round(ms_step, 4), "attention_ms": round(ms_attn, 4),
                 "attention_tflops": round(flop / ms_attn / 1e9, 1), "attention_frac_of_bf16_peak": round(flop / ms_attn / 1e9 / PEAK_BF16_TFLOPS, 4),
                 "block_pairs": HEADS * nbq * k_sel}
    torch.cuda.empty_cache()
    ms, ms_attn, pairs, _ = measure_c4(torch, 5, 2, args.settle, "device")
    flop = pairs * 4 * 64 * 64 * D
    out["c4"] = {"workload": "32 heads x 128, grid 48x30x52 (74880 tokens), 12 conditioning frames, density 1/8, two operator calls",
                 "operator_ms": round(ms, 4), "attention_ms": round(ms_attn, 4), "attention_tflops": round(flop / ms_attn / 1e9, 1),
                 "attention_frac_of_bf16_peak": round(flop / ms_attn / 1e9 / PEAK_BF16_TFLOPS, 4), "block_pairs": pairs}
    torch.cuda.empty_cache()
    return out


def run_c4(torch, args):
    """benchmark configuration 4: long-video continuation, grid 48x30x52 with 12 conditioning frames.  Two operator
    calls per layer as in attention.py:124-135, writing into one output buffer."""
    from longcat_video_amd.block_sparse_attention import bsa_interface as I
    ms, ms_attn, pairs, (T, Hh, W, cond, S, n) = measure_c4(torch, args.steps, args.warmup, args.settle, args.inputs)
    pairs = HEADS * (312 * 39 + 936 * 156)
    flop = pairs * 4 * 64 * 64 * D
    result = {
        "metric": "BSA fwd ms/layer + sparse TFLOPS, long-video continuation (cond/noise split)", "value": round(flop / ms / 1e9, 2),
        "unit": "TFLOP/s (sparse-actual, both operator calls)", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic N(0,1) q/k/v, " + DRAWN[args.inputs],
        "config": {"workload": "c4: 32 heads x 128, grid 48x30x52 (74880 tokens), 12 conditioning frames, density 1/8",
                   "block_pairs": pairs},
        "pct_of_bf16_peak_whole_operator": round(100 * flop / ms / 1e9 / PEAK_BF16_TFLOPS, 2),
        "kernels_ms": {"attention (both calls)": round(ms_attn, 4), "everything else (step - attention)": round(ms - ms_attn, 4)},
        "roofline": attention_roofline(flop, ms_attn, "c4")}
    if not args.no_cpu_baseline:
        cores = os.cpu_count() or 1
        torch.set_num_threads(cores)
        hq, hk, hv = host_inputs(torch, S, 3, False)
        half = args.cpu_seconds / 2
        a = cpu_attention_sample(torch, hq[:, :, :n], hk[:, :, :n], hv[:, :, :n], (cond, Hh, W), (cond, Hh, W), 0.875, half)
        b = cpu_attention_sample(torch, hq[:, :, n:], hk, hv, (T - cond, Hh, W), (T, Hh, W), 0.875, half)
        layer_s = HEADS * (a[0] + b[0])
        result["cpu_baseline"] = {
            "value": round(flop / layer_s / 1e12, 5), "unit": "TFLOP/s (sparse-actual)", "cores": cores, "kind": "port",
            "ms_per_layer": round(layer_s * 1e3, 1),
            "sample": "1 of %d heads, inputs drawn on the host from the same distribution (a separate draw): both operator "
                      "calls with permute+pool+score+top-k in full (%.2f s + %.2f s) and masked-dense fp32 attention on %d of %d "
                      "conditioning and %d of %d noise query blocks (%.2f s + %.2f s); scaled linearly to all query blocks and %d heads"
                      % (HEADS, a[1], b[1], a[3], a[4], b[3], b[4], a[2], b[2], HEADS)}
    print(json.dumps(result))


def run_bwd(torch, args):
    """Backward of the blocked-order operator (bsa_bwd) at the c3 geometry: 32 heads x 128, 1440 query and KV blocks of
    64 tokens, 90 selected blocks per row from the operator's own gating.  A step is one backward pass (row sums,
    scaled k, bit matrix, seven fragment-order passes, dQ kernel, dK/dV kernel); the forward is not in it."""
    from longcat_video_amd.block_sparse_attention import bsa_interface as I
    latent, sparsity, seed, rms, desc = WORKLOADS["c3"]
    q, k, v = make_inputs(torch, latent, seed, rms, args.inputs)
    qp, kp, vp = (I._permute(t, latent, CHUNK)[0] for t in (q, k, v))
    # ---- first the operator as a training step sees it: flash_attn_bsa_3d on inputs that require a gradient (the
    # forward of every other call, which also keeps lse and the lists it walked) and autograd's backward through it
    # (permutes into blocked order, bsa_bwd, permutes back)
    prm = dict(sparsity=sparsity, chunk_3d_shape_q=list(CHUNK), chunk_3d_shape_k=list(CHUNK))
    for t in (q, k, v):
        t.requires_grad_(True)
    d_o = torch.randn(q.shape, generator=torch.Generator(device="cuda").manual_seed(seed + 100), device="cuda").bfloat16()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    ms_tf, ms_tb = [], []
    for rep in range(3):
        for t in (q, k, v):
            t.grad = None
        ev[0].record()
        o_t = I.flash_attn_bsa_3d(q, k, v, latent, latent, **prm)
        ev[1].record()
        o_t.backward(d_o)
        ev[2].record()
        torch.cuda.synchronize()
        ms_tf.append(ev[0].elapsed_time(ev[1]))
        ms_tb.append(ev[1].elapsed_time(ev[2]))
    with torch.no_grad():
        assert torch.equal(o_t, I.flash_attn_bsa_3d(q, k, v, latent, latent, **prm)), "one forward with and without grad"
    assert all(bool(torch.isfinite(t.grad.float()).all()) for t in (q, k, v))
    through_autograd = {"forward_with_grad_ms": round(min(ms_tf), 4), "backward_ms": round(min(ms_tb), 4),
                        "note": "flash_attn_bsa_3d in (T,H,W) order on inputs that require a gradient; best of 3"}
    for t in (q, k, v):
        t.grad = None
    del q, k, v, o_t, d_o
    torch.cuda.empty_cache()
    sm = 1 / math.sqrt(D)
    idx, lens = I._select_blocked(qp, kp, 64, 64, sparsity, None)
    o, lse = I.attn_fwd_bsa_varlen(qp, kp, vp, sm, idx, lens, 64, 64)
    do = torch.randn(o.shape, generator=torch.Generator(device="cuda").manual_seed(seed + 100), device="cuda").bfloat16()
    dq, dk, dv = (torch.empty_like(t) for t in (qp, kp, vp))
    step = lambda: I.attn_bwd_bsa_varlen(do, qp, kp, vp, o, dq, dk, dv, sm, lse, idx, lens, 64, 64)
    for _ in range(min(args.warmup, 2)):
        step()
    torch.cuda.synchronize()
    steps = min(args.steps, 5)
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    assert all(bool(torch.isfinite(t.float()).all()) for t in (dq, dk, dv))
    pairs = HEADS * idx.shape[2] * idx.shape[3]
    flop = pairs * 7 * 2 * 64 * 64 * D       # q.k_s and do.v (each in both kernels), dV, dK, dQ
    tflops = flop / ms / 1e9
    result = {
        "metric": "BSA bwd ms/layer + TFLOPS at 720p 86.4k tokens (blocked order)", "value": round(tflops, 2),
        "unit": "TFLOP/s (seven 64x64x128 products per selected block pair)", "n_gpus": 1, "steps": steps, "warmup": min(args.warmup, 2),
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic N(0,1) q/k/v with per-head RMS-normalised q/k, " + DRAWN[args.inputs] + "; N(0,1) output gradient drawn on the GPU",
        "config": {"workload": "bwd: backward of the c3 layer in blocked order, 32 heads x 128, 1440 x 1440 blocks of 64, 90 per row",
                   "block_pairs": pairs},
        "through_autograd": through_autograd,
        "roofline": {"kernel": "bwd_dq_lds_kernel<bf16> + bwd_dkdv_kernel<bf16> (with the passes before them)", "bound": "mfma",
                     "achieved": round(tflops, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / PEAK_BF16_TFLOPS, 4),
                     "traffic": recorded_traffic("bwd", "bsa_backward_*.md", BACKWARD_SOURCES), "ms": round(ms, 4)}}
    if not args.no_cpu_baseline:
        from oracle import bsa_oracle as O
        cores = os.cpu_count() or 1
        torch.set_num_threads(cores)
        hq, hk, hv = host_inputs(torch, qp.shape[2], seed, rms)
        hdo = torch.randn(hq.shape, generator=torch.Generator().manual_seed(seed + 100)).bfloat16()
        score = O.cal_score(O.mean_pooling_compression(hq, 64), O.mean_pooling_compression(hk, 64))
        hidx, hlens = O.select_topk(score, idx.shape[3])
        nq = 128                                                         # query blocks of the sample
        mask = O.block_mask_from_indices(hidx[:, :, :nq], hlens[:, :, :nq], score.shape[-1])
        ho, hlse = O.masked_dense_attention(hq[:, :, :nq * 64], hk, hv, mask, 64, 64, sm)
        t0 = time.perf_counter()
        O.blockwise_attention_backward(hq[:, :, :nq * 64], hk, hv, ho.bfloat16(), hdo[:, :, :nq * 64], hlse, hidx[:, :, :nq], hlens[:, :, :nq],
                                       64, 64, sm)
        sec = time.perf_counter() - t0
        layer_s = sec * pairs / (nq * idx.shape[3])
        # the checker's other job in this leg: the timed call's own gradients against the oracle on sampled blocks of
        # the first head (all pairs of three query blocks; every query block that selected two KV blocks)
        one = lambda t: t[:, :1].cpu()
        nb = idx.shape[2]
        counts = torch.bincount(idx[0, 0].flatten().long(), minlength=nb).cpu()
        qb, kb = [0, nb // 2, nb - 1], [int(counts.argmax()), int(counts.argmin())]
        wq, wk, wv = O.blockwise_attention_backward(one(qp), one(kp), one(vp), one(o), one(do), one(lse), one(idx).long(), one(lens),
                                                    64, 64, sm, q_blocks=qb, kv_blocks=kb)
        rows = lambda blocks: torch.cat([torch.arange(64 * b, 64 * b + 64) for b in blocks])
        worst = 0.0
        for got, want, r in ((dq, wq, rows(qb)), (dk, wk, rows(kb)), (dv, wv, rows(kb))):
            g, w = one(got)[:, :, r].float(), want[:, :, r].float()
            err = float((g - w).abs().max()) / max(float(w.abs().max()), 1e-30)
            assert err <= 4 * 2.0 ** -7, "sampled gradient blocks differ from the oracle (%.3g of the largest entry)" % err
            worst = max(worst, err)
        result["sampled_parity"] = {"query_blocks": qb, "kv_blocks": kb, "max_error_over_largest_entry": round(worst, 6), "bound": 4 * 2.0 ** -7}
        result["cpu_baseline"] = {
            "value": round(flop / layer_s / 1e12, 5), "unit": "TFLOP/s", "cores": cores, "kind": "port", "ms_per_layer": round(layer_s * 1e3, 1),
            "sample": "1 of %d heads, inputs drawn on the host from the same distribution (a separate draw): the oracle's backward "
                      "of %d of 1440 query blocks with their %d selected blocks each (%.2f s), scaled linearly to all block pairs"
                      % (HEADS, nq, idx.shape[3], sec)}
    print(json.dumps(result))


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
    # ---- the module's kernels on their own, on the module's own tensors
    ms_qkv = time_events(torch, lambda: M.linear_bf16(x, attn.qkv.weight, attn.qkv.bias), 5, 2)
    ms_proj = time_events(torch, lambda: M.linear_bf16(x, attn.proj.weight, attn.proj.bias, residual=x), 5, 2)
    qs, ks, vs = attn._project_qkv(M.rms_norm(x, w_pre, 1e-6))
    new = lambda: torch.empty(1, HEADS, N, D, dtype=x.dtype, device=x.device)
    qd, kd, vd = new(), new(), new()
    ms_norm_rope = time_events(torch, lambda: M.norm_rope(qs, qd, attn.q_norm.weight, latent), 5, 2)
    M.norm_rope(ks, kd, attn.k_norm.weight, latent)
    M.norm_rope(vs, vd)
    from longcat_video_amd.block_sparse_attention import bsa_interface as I
    _, idx, lens, _ = I._bsa_3d(qd, kd, vd, latent, latent, 0.9375, CHUNK, CHUNK, want_selection=True)
    idx = operator_lists(I, idx, lens, latent)
    attend = I.ThwAttention(kd, vd, latent, latent, CHUNK, CHUNK)
    o_buf = torch.empty(1, N, HEADS, D, dtype=x.dtype, device=x.device).permute(0, 2, 1, 3)
    ms_attn = time_events(torch, lambda: attend(qd, idx, lens, out=o_buf), 20, 5, settle_s=args.settle)
    del attend
    # ---- the engine's own GEMM: QKV projection with norm, rotation and head split in its epilogue, and the output
    # projection; and the module with both (projection_backend = "engine")
    xn = M.rms_norm(x, w_pre, 1e-6)
    ms_eng_qkv = time_events(torch, lambda: M.qkv_projection(xn, attn.qkv.weight, attn.qkv.bias, attn.q_norm.weight,
                                                             attn.k_norm.weight, latent, HEADS), 5, 2)
    ms_eng_proj = time_events(torch, lambda: M.gemm_bf16(x, attn.proj.weight, attn.proj.bias, residual=x), 5, 2)
    attn.projection_backend = "engine"
    ms_eng_step = time_events(torch, lambda: M.attention_block_forward(x, w_pre, attn, latent), max(args.steps // 2, 3), 2)
    attn.projection_backend = "hipblaslt"
    eng_tflops = 2 * N * C * 3 * C / ms_eng_qkv / 1e9
    qkv_tflops = 2 * N * C * 3 * C / ms_qkv / 1e9
    norm_rope_gbs = 2 * N * C * 2 / ms_norm_rope / 1e6          # one tensor: 708 MB read + 708 MB written
    result = {
        "metric": "attention sub-chain of a DiT block, ms/layer + TFLOPS (GEMMs + sparse-actual attention)",
        "value": round((bsa_flop + gemm_flop) / ms / 1e9, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic N(0,1) activations, N(0,0.02) weights, zero biases, unit norm weights",
        "config": {"workload": "c5: x [1, 86400, 4096] bf16, 32 heads x 128, grid 24x45x80, density 1/16"},
        "kernels_ms": {"attention": round(ms_attn, 4), "qkv_gemm": round(ms_qkv, 4), "proj_gemm_with_residual": round(ms_proj, 4),
                       "norm_rope_move_one_tensor": round(ms_norm_rope, 4),
                       "engine_qkv_projection_with_norm_rope_epilogue": round(ms_eng_qkv, 4),
                       "engine_proj_gemm_with_residual": round(ms_eng_proj, 4)},
        "ms_per_step_with_engine_projections": round(ms_eng_step, 4),
        "qkv_gemm_ms": round(ms_qkv, 4), "qkv_gemm_tflops": round(qkv_tflops, 1),
        "gemm_tuning": {"qkv": {"algorithms_timed": tuned[0][0], "default_ms": round(tuned[0][1], 4), "chosen_ms": round(tuned[0][2], 4)},
                        "proj": {"algorithms_timed": tuned[1][0], "default_ms": round(tuned[1][1], 4), "chosen_ms": round(tuned[1][2], 4)}},
        "pct_of_bf16_peak": round(100 * (bsa_flop + gemm_flop) / ms / 1e9 / PEAK_BF16_TFLOPS, 2),
        # the dominant kernel of the module is still the attention kernel; the other two kinds of kernel beside it
        "roofline": attention_roofline(bsa_flop, ms_attn, "c5"),
        "roofline_qkv_gemm": {"kernel": "hipBLASLt bf16 GEMM [86400,4096]x[4096,12288]^T + bias (library kernel)", "bound": "mfma",
                              "achieved": round(qkv_tflops, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                              "frac": round(qkv_tflops / PEAK_BF16_TFLOPS, 4), "traffic": None, "ms": round(ms_qkv, 4)},
        "roofline_engine_gemm": {"kernel": "gemm_nt_kernel<qkv epilogue> [86400,4096]x[4096,12288]^T + bias, per-head RMSNorm, RoPE, head split",
                                 "bound": "mfma", "achieved": round(eng_tflops, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                                 "frac": round(eng_tflops / PEAK_BF16_TFLOPS, 4), "traffic": None, "ms": round(ms_eng_qkv, 4)},
        "roofline_norm_rope": {"kernel": "norm_rope_kernel<bf16> (per-head RMSNorm + 3-D RoPE + move of one tensor)", "bound": "hbm",
                               "achieved": round(norm_rope_gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                               "frac": round(norm_rope_gbs / PEAK_HBM_GBS, 4), "traffic": None, "ms": round(ms_norm_rope, 4)},
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline_c5(torch, latent, N, C, args.cpu_seconds, bsa_flop + gemm_flop)
    print(json.dumps(result))


def cpu_baseline_c5(torch, latent, N, C, budget_s, flop):
    """The module on the host cores through the oracle, on a bounded sample: both projections in fp32 on a slice of the
    tokens (with the pre-norm, the per-head norm and the rotation of that slice), and the attention of one head as in
    cpu_baseline; each part scaled linearly to the layer."""
    from oracle import bsa_oracle as O
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(4)
    n_tok = 1024
    x = torch.randn(1, n_tok, C, generator=g).bfloat16()
    w_qkv = (torch.randn(3 * C, C, generator=g) * 0.02).bfloat16()
    w_proj = (torch.randn(C, C, generator=g) * 0.02).bfloat16()
    t0 = time.perf_counter()
    y = O.rms_norm_fp32(x, torch.ones(C, dtype=torch.bfloat16))
    qkv = (y.reshape(n_tok, C).float() @ w_qkv.float().t()).bfloat16().view(1, n_tok, 3, HEADS, D).permute(2, 0, 3, 1, 4)
    qh, kh = O.rms_norm_fp32(qkv[0], torch.ones(D, dtype=torch.bfloat16)), O.rms_norm_fp32(qkv[1], torch.ones(D, dtype=torch.bfloat16))
    ang = O.rope_3d_angles(latent, D)[:n_tok]
    qh, kh = O.rope_3d_apply(qh, ang), O.rope_3d_apply(kh, ang)
    o = qkv[2].transpose(1, 2).reshape(n_tok, C)
    _ = (o.float() @ w_proj.float().t() + x.reshape(n_tok, C).float()).bfloat16()
    t_glue = time.perf_counter() - t0
    hq, hk, hv = host_inputs(torch, N, 2, True)
    head_s, t_setup, t_attn, done, nbq, _ = cpu_attention_sample(torch, hq, hk, hv, latent, latent, 0.9375, budget_s)
    layer_s = t_glue * N / n_tok + HEADS * head_s
    return {"value": round(flop / layer_s / 1e12, 5), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "ms_per_layer": round(layer_s * 1e3, 1),
            "sample": "inputs drawn on the host from the same distributions (separate draws): pre-norm, both projections in fp32, "
                      "per-head norm and rotation on %d of %d tokens (%.2f s, scaled linearly); attention of 1 of %d heads with "
                      "permute+pool+score+top-k in full (%.2f s) and masked-dense fp32 attention on %d of %d query blocks (%.2f s), "
                      "scaled linearly to all query blocks and heads" % (n_tok, N, t_glue, HEADS, t_setup, done, nbq, t_attn)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS) + ["c4", "c5", "bwd"],
                    help="c3 is the headline (default); c2 the same operator at 480p; c4 the cond/noise split of a long "
                         "video; c5 the attention module around the operator; bwd the backward of the c3 layer")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="time budget of the CPU baseline's attention sample")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--settle", type=float, default=0.3,
                    help="seconds of warm-up, and at least as many of timing, for the kernel-alone measurements (0: fixed "
                         "call counts, for runs under a profiler whose per-dispatch averages must weigh every call alike)")
    ap.add_argument("--no-gemm-tuning", action="store_true", help="c5: leave the GEMM algorithm choice to hipBLASLt's first proposal")
    ap.add_argument("--inputs", default="host", choices=["host", "device"],
                    help="where q, k, v of the timed workload are drawn: torch's CPU generator (the same numbers on every "
                         "machine; half a minute at 720p) or the GPU's")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="c3: leave out the attention-kernel figures of c2 and c4 that the default line carries beside its own")
    ap.add_argument("--clocks", action="store_true",
                    help="c2, c3: also run the attention kernel back to back for three seconds and report the shader clock "
                         "that rocm-smi shows meanwhile")
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
    if args.workload == "bwd":
        return run_bwd(torch, args)
    latent, sparsity, seed, rms, desc = WORKLOADS[args.workload]
    coherent = args.data == "coherent"
    # ---- whole operator: warm-up, then exactly K timed steps between synchronisations; then the attention kernel alone
    clocks = {} if args.clocks else None
    ms_step, ms_attn, nbq, k_sel, (q, k, v) = measure_operator(torch, args.workload, args.steps, args.warmup, args.settle, args.inputs, coherent, clocks)
    ksteps, kwarm = max(args.steps, 20), max(args.warmup, 5)      # kernels alone: enough calls for a steady clock
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
                 "synthetic N(0,1) q/k/v%s, %s" % (" with per-head RMS-normalised q/k" if rms else "", DRAWN[args.inputs])),
        "config": {"workload": "%s: %s" % (args.workload, desc), "chunk": list(CHUNK), "kv_blocks": nbk, "k_sel": k_sel,
                   "block_pairs": pairs, "padded_tokens": Sp},
        "ms_per_layer": round(ms_step, 4),
        "pct_of_bf16_peak_whole_operator": round(100 * tflops_step / PEAK_BF16_TFLOPS, 2),
        "dense_equivalent_tflops": round(dense_flop / (ms_step * 1e-3) / 1e12, 1),
        "kernels_ms": {"attention": round(ms_attn, 4), "score_topk": round(ms_select, 4),
                       "pool_q_and_fragment_order_k_v (step - attention - score_topk)": round(ms_step - ms_attn - ms_select, 4)},
        "standalone_ms": {"permute_pool_one_tensor": round(ms_permute, 4), "unpermute": round(ms_unpermute, 4)},
        "permute_gbs": round(permute_bytes / (ms_permute * 1e-3) / 1e9, 1),
        "roofline": attention_roofline(flop, ms_attn, args.workload, coherent),
    }
    if clocks:
        result["clocks_under_the_attention_kernel"] = clocks
    del q, k, v, qp, q_cmp, k_cmp
    torch.cuda.empty_cache()
    if args.workload == "c3" and not coherent and not args.no_other_configs:
        result["other_configs"] = other_configurations(torch, args)
    if not args.no_cpu_baseline and not coherent:
        result["cpu_baseline"] = cpu_baseline(torch, latent, sparsity, seed, rms, args.cpu_seconds)
    print(json.dumps(result))


if __name__ == "__main__":
    main()

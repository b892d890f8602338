"""R10/R11 on the GPU: the attention-module glue (linear layers, RMSNorm, QK-norm +
3-D RoPE), the conditioning/noise split, and the whole module against the oracle."""
import math

import numpy as np
import pytest
import torch

from oracle import bsa_oracle as O

pytestmark = pytest.mark.gpu

BF16_ULP = 2.0 ** -7


def M():
    from longcat_video_amd.modules import attention
    return attention


def make_module(dim=512, heads=4, sparsity=0.5, seed=0):
    g = torch.Generator().manual_seed(seed)
    m = M().Attention(dim, heads, enable_bsa=True,
                      bsa_params=dict(sparsity=sparsity, cdf_threshold=None, chunk_3d_shape_q=[4, 4, 4], chunk_3d_shape_k=[4, 4, 4]),
                      cp_split_hw=[1, 1])
    with torch.no_grad():
        for p in (m.qkv.weight, m.proj.weight):
            p.copy_(torch.randn(p.shape, generator=g) * 0.02)
        m.qkv.bias.copy_(torch.randn(m.qkv.bias.shape, generator=g) * 0.02)
        m.proj.bias.copy_(torch.randn(m.proj.bias.shape, generator=g) * 0.02)
        m.q_norm.weight.copy_(1 + 0.1 * torch.randn(128, generator=g))
        m.k_norm.weight.copy_(1 + 0.1 * torch.randn(128, generator=g))
    return m.to(torch.bfloat16)


def test_state_dict_names_match_the_reference_module():
    m = M().Attention(512, 4, enable_bsa=True, bsa_params={}, cp_split_hw=[1, 1])
    assert sorted(m.state_dict()) == ["k_norm.weight", "proj.bias", "proj.weight", "q_norm.weight", "qkv.bias", "qkv.weight"]
    assert m.qkv.weight.shape == (1536, 512) and m.q_norm.weight.shape == (128,)


def test_row_rmsnorm():
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(3, 37, 4096, generator=g) * 3).bfloat16()
    w = (1 + 0.2 * torch.randn(4096, generator=g)).bfloat16()
    got = M().rms_norm(x.cuda(), w.cuda(), 1e-6).cpu()
    want = O.rms_norm_fp32(x, w)
    assert got.dtype == torch.bfloat16
    assert torch.all((got.float() - want.float()).abs() <= want.float().abs() * 2 * BF16_ULP + 1e-6)
    assert (got.float() - want.float()).abs().mean() < 1e-3


def test_linear_with_bias_and_residual():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(2, 100, 512, generator=g).bfloat16()
    w = (torch.randn(384, 512, generator=g) * 0.05).bfloat16()
    b = torch.randn(384, generator=g).bfloat16()
    r = torch.randn(2, 100, 384, generator=g).bfloat16()
    want = x.float() @ w.float().t() + b.float()
    got = M().linear_bf16(x.cuda(), w.cuda(), b.cuda()).cpu()
    assert got.shape == (2, 100, 384)
    assert torch.all((got.float() - want).abs() <= want.abs() * BF16_ULP + 2e-3)
    got_r = M().linear_bf16(x.cuda(), w.cuda(), b.cuda(), residual=r.cuda()).cpu()
    assert torch.all((got_r.float() - (want + r.float())).abs() <= (want + r.float()).abs() * BF16_ULP + 2e-2)
    got_nb = M().linear_bf16(x.cuda(), w.cuda(), None).cpu()
    assert torch.all((got_nb.float() - (want - b.float())).abs() <= (want - b.float()).abs() * BF16_ULP + 2e-3)


def test_linear_from_several_threads_on_their_own_streams():
    """Linear layers called from four host threads at once, each on its own stream and with its own shapes, give
    what they give when called alone (the GEMM wrapper keeps one library handle per thread and shares only its
    table of chosen algorithms)."""
    import threading
    g = torch.Generator().manual_seed(40)
    jobs = []
    for n_out, rows in ((384, 200), (512, 333), (640, 128), (384, 200)):
        x = torch.randint(-2, 3, (rows, 512), generator=g).bfloat16().cuda()          # small integers: exact
        w = torch.randint(-2, 3, (n_out, 512), generator=g).bfloat16().cuda()
        b = torch.randint(-2, 3, (n_out,), generator=g).bfloat16().cuda()
        jobs.append((x, w, b, M().linear_bf16(x, w, b)))
    torch.cuda.synchronize()
    failures = []

    def worker(job):
        x, w, b, want = job
        stream = torch.cuda.Stream()
        try:
            with torch.cuda.stream(stream):
                for _ in range(25):
                    got = M().linear_bf16(x, w, b)
                    stream.synchronize()
                    if not torch.equal(got, want):
                        failures.append("mismatch")
                        return
        except Exception as exc:                                       # noqa: BLE001 - reported through the list
            failures.append(repr(exc))

    threads = [threading.Thread(target=worker, args=(j,)) for j in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
    assert not failures, failures
    assert all(not t.is_alive() for t in threads)


def test_qk_norm_rope_against_the_oracle():
    grid = (3, 5, 7)
    S = 105
    g = torch.Generator().manual_seed(3)
    qkv = (torch.randn(2, S, 3, 4, 128, generator=g) * 2).bfloat16()
    qw = (1 + 0.1 * torch.randn(128, generator=g)).bfloat16()
    kw = (1 + 0.1 * torch.randn(128, generator=g)).bfloat16()
    q, k, v = qkv.permute(2, 0, 3, 1, 4).unbind(0)
    ang = O.rope_3d_angles(grid, 128)
    want_q = O.rope_3d_apply(O.rms_norm_fp32(q, qw), ang)
    want_k = O.rope_3d_apply(O.rms_norm_fp32(k, kw), ang)
    dev = qkv.cuda()
    dq, dk, dv = dev.permute(2, 0, 3, 1, 4).unbind(0)
    M().qk_norm_rope_(dq, dk, qw.cuda(), kw.cuda(), grid)
    for got, want in ((dq.cpu(), want_q), (dk.cpu(), want_k)):
        d = (got.float() - want.float()).abs()
        # three roundings (norm, weight, rotation): a couple of ulps at most, almost always none
        assert torch.all(d <= want.float().abs() * 3 * BF16_ULP + 0.02)
        assert (d > 0).float().mean() < 0.05
    assert torch.equal(dv.cpu(), v)                       # v is untouched
    # rotation keeps the norm of the normalised vector
    n_in = O.rms_norm_fp32(q, qw).float().norm(dim=-1)
    assert torch.allclose(dq.cpu().float().norm(dim=-1), n_in, rtol=2e-2)


def module_reference(m, x, shape, num_cond=0):
    """Oracle evaluation of the module on the CPU with the module's own weights."""
    sd = {k: v.detach().cpu() for k, v in m.state_dict().items()}
    prm = dict(sparsity=m.bsa_params["sparsity"], chunk_3d_shape_q=tuple(m.bsa_params["chunk_3d_shape_q"]),
               chunk_3d_shape_k=tuple(m.bsa_params["chunk_3d_shape_k"]))
    return O.attention_module_forward(x, sd["qkv.weight"], sd["qkv.bias"], sd["proj.weight"], sd["proj.bias"],
                                      sd["q_norm.weight"], sd["k_norm.weight"], shape, m.num_heads, prm, num_cond)


@pytest.mark.parametrize("sparsity", [0.0, 0.5])
def test_module_forward_matches_the_oracle(sparsity):
    shape = (4, 8, 8)
    m = make_module(sparsity=sparsity)
    x = torch.randn(1, 256, 512, generator=torch.Generator().manual_seed(4)).bfloat16()
    want = module_reference(m, x, shape)
    got = m.cuda()(x.cuda(), shape=shape).cpu()
    assert got.shape == (1, 256, 512) and got.dtype == torch.bfloat16
    d = (got.float() - want.float()).abs()
    assert d.max() <= 2e-2 and d.mean() <= 2e-3, (d.max(), d.mean())


def test_module_forward_with_the_engine_projections():
    """projection_backend = "engine": QKV GEMM with the fused norm / rotation / head-split epilogue and the
    engine GEMM for the output projection, against the oracle and against the default route."""
    shape = (4, 8, 8)
    m = make_module(sparsity=0.5)
    x = torch.randn(1, 256, 512, generator=torch.Generator().manual_seed(4)).bfloat16()
    want = module_reference(m, x, shape)
    m = m.cuda()
    base = m(x.cuda(), shape=shape).cpu()
    m.projection_backend = "engine"
    got = m(x.cuda(), shape=shape).cpu()
    d = (got.float() - want.float()).abs()
    assert d.max() <= 2e-2 and d.mean() <= 2e-3, (d.max(), d.mean())
    assert (got.float() - base.float()).abs().max() <= 2e-2
    r = torch.randn(1, 256, 512, generator=torch.Generator().manual_seed(5)).bfloat16().cuda()
    with_res = m(x.cuda(), shape=shape, residual=r).cpu()
    assert torch.all((with_res.float() - (got.float() + r.cpu().float())).abs() <= (got.float().abs() + r.cpu().float().abs()) * BF16_ULP + 1e-3)
    # the k cache path keeps the separate passes (the cache holds k before the rotation)
    y_kv, (kc, vc) = m(x.cuda(), shape=shape, return_kv=True)
    assert (y_kv.cpu().float() - got.float()).abs().max() <= 2e-2 and kc.shape == (1, 4, 256, 128)


def test_cond_noise_split():
    """attention.py:124-135: conditioning rows only see conditioning tokens."""
    shape, cond = (8, 8, 8), 4
    m = make_module(sparsity=0.5, seed=5)
    x = torch.randn(1, 512, 512, generator=torch.Generator().manual_seed(6)).bfloat16()
    want = module_reference(m, x, shape, num_cond=cond)
    mc = m.cuda()
    got = mc(x.cuda(), shape=shape, num_cond_latents=cond).cpu()
    d = (got.float() - want.float()).abs()
    assert d.max() <= 2e-2 and d.mean() <= 2e-3, (d.max(), d.mean())
    # perturbing noise tokens must leave the conditioning rows bit-identical
    x2 = x.clone()
    x2[:, 256:] += 1.0
    got2 = mc(x2.cuda(), shape=shape, num_cond_latents=cond).cpu()
    assert torch.equal(got[:, :256], got2[:, :256]) and not torch.equal(got[:, 256:], got2[:, 256:])


def test_attention_block_with_pre_norm_and_residual():
    shape = (4, 8, 8)
    m = make_module(sparsity=0.5, seed=7)
    g = torch.Generator().manual_seed(8)
    x = torch.randn(1, 256, 512, generator=g).bfloat16()
    wn = (1 + 0.1 * torch.randn(512, generator=g)).bfloat16()
    y = O.rms_norm_fp32(x, wn)
    want = (x.float() + module_reference(m, y, shape).float())
    got = M().attention_block_forward(x.cuda(), wn.cuda(), m.cuda(), shape).cpu()
    d = (got.float() - want).abs()
    assert d.max() <= 4e-2 and d.mean() <= 4e-3, (d.max(), d.mean())


def test_return_kv_and_forward_with_kv_cache():
    """attention.py:118-119 and :149-181: a first pass over the conditioning frames returns the cache
    (keys after the norm, before the rotation); a second pass over the new frames attends to cache + new."""
    cond, T, Hh, W = 4, 8, 8, 8
    m = make_module(sparsity=0.5, seed=9)
    g = torch.Generator().manual_seed(10)
    x_cond = torch.randn(1, cond * Hh * W, 512, generator=g).bfloat16()
    x_new = torch.randn(2, T * Hh * W, 512, generator=g).bfloat16()      # the cache of batch 1 serves batch 2
    sd = {k: v.detach().cpu() for k, v in m.state_dict().items()}
    prm = dict(sparsity=0.5, chunk_3d_shape_q=(4, 4, 4), chunk_3d_shape_k=(4, 4, 4))
    mc = m.cuda()
    y, (k_cache, v_cache) = mc(x_cond.cuda(), shape=(cond, Hh, W), return_kv=True)
    assert torch.equal(y, mc(x_cond.cuda(), shape=(cond, Hh, W)))          # the cache is a by-product
    want_k, want_v = O.attention_module_kv(x_cond, sd["qkv.weight"], sd["qkv.bias"], sd["q_norm.weight"],
                                           sd["k_norm.weight"], m.num_heads)
    assert k_cache.shape == (1, 4, cond * Hh * W, 128) and k_cache.is_contiguous()
    dk = (k_cache.cpu().float() - want_k.float()).abs()
    assert torch.all(dk <= want_k.float().abs() * 3 * BF16_ULP + 0.02) and (dk > 0).float().mean() < 0.05
    dv = (v_cache.cpu().float() - want_v.float()).abs()
    assert torch.all(dv <= want_v.float().abs() * BF16_ULP + 2e-3)
    # second pass: judged against the oracle fed with the GPU's own cache
    want = O.attention_module_forward_with_kv_cache(
        x_new, sd["qkv.weight"], sd["qkv.bias"], sd["proj.weight"], sd["proj.bias"], sd["q_norm.weight"],
        sd["k_norm.weight"], (T, Hh, W), m.num_heads, prm, cond, (k_cache.cpu(), v_cache.cpu()))
    got = mc.forward_with_kv_cache(x_new.cuda(), shape=(T, Hh, W), num_cond_latents=cond, kv_cache=(k_cache, v_cache)).cpu()
    assert got.shape == (2, T * Hh * W, 512)
    d = (got.float() - want.float()).abs()
    assert d.max() <= 2e-2 and d.mean() <= 2e-3, (d.max(), d.mean())


def test_norm_rope_steps_and_frame_offset():
    """bsa_norm_rope: each step alone, the move into another layout, and rotation of a slice of frames on
    a larger grid (the position a new token gets in forward_with_kv_cache)."""
    g = torch.Generator().manual_seed(11)
    B, H, grid = 2, 3, (6, 4, 5)
    S = grid[0] * grid[1] * grid[2]
    x = torch.randn(B, S, H, 128, generator=g).bfloat16().permute(0, 2, 1, 3)     # token-major storage
    w = (1 + 0.1 * torch.randn(128, generator=g)).bfloat16()
    dx = x.cuda()
    new = lambda: torch.empty(B, H, S, 128, dtype=torch.bfloat16, device="cuda")
    moved = M().norm_rope(dx, new())
    assert moved.is_contiguous() and torch.equal(moved.cpu(), x)
    normed = M().norm_rope(dx, new(), w.cuda())
    want_n = O.rms_norm_fp32(x, w)
    assert torch.all((normed.cpu().float() - want_n.float()).abs() <= want_n.float().abs() * BF16_ULP + 1e-6)
    ang = O.rope_3d_angles(grid, 128)
    roped = M().norm_rope(normed, new(), None, grid)
    want_r = O.rope_3d_apply(normed.cpu(), ang)
    assert torch.all((roped.cpu().float() - want_r.float()).abs() <= want_r.float().abs() * BF16_ULP + 1e-2)
    both = M().norm_rope(dx, new(), w.cuda(), grid)
    assert torch.equal(both, roped)                          # the fused pass rounds at the same points
    # frames 2..6 of the grid, handed over as a tensor of 4 frames
    part = normed[:, :, 2 * 20:].contiguous()
    off = M().norm_rope(part, torch.empty_like(part), None, (4, 4, 5), t_offset=2, table_grid=grid)
    assert torch.equal(off, roped[:, :, 2 * 20:])
    with pytest.raises(AssertionError):
        M().norm_rope(part, torch.empty_like(part), None, (4, 4, 5), t_offset=3, table_grid=grid)


def test_layernorm_modulate_and_gated_residual():
    g = torch.Generator().manual_seed(12)
    B, T, per, C = 2, 3, 40, 512
    x = (torch.randn(B, T * per, C, generator=g) * 2 + 0.5).bfloat16()
    y = torch.randn(B, T * per, C, generator=g).bfloat16()
    shift = torch.randn(B, T, 1, C, generator=g)
    scale = torch.randn(B, T, 1, C, generator=g) * 0.2
    gate = torch.randn(B, T, 1, C, generator=g)
    got = M().layernorm_modulate(x.cuda(), shift.cuda(), scale.cuda()).cpu()
    want = O.layernorm_modulate_fp32(x, shift, scale)
    d = (got.float() - want.float()).abs()
    assert torch.all(d <= want.float().abs() * BF16_ULP + 1e-6) and (d > 0).float().mean() < 0.01   # fp32 statistics differ in the last bit at most
    assert torch.equal(M().gated_residual(x.cuda(), gate.cuda(), y.cuda()).cpu(), O.gated_residual_fp32(x, gate, y))
    wide = torch.randn(1, 8, 4096, generator=g).bfloat16()                     # the model's width
    z = torch.zeros(1, 2, 1, 4096)
    got = M().layernorm_modulate(wide.cuda(), z.cuda(), z.cuda()).cpu()
    want = O.layernorm_modulate_fp32(wide, z, z)
    assert torch.all((got.float() - want.float()).abs() <= want.float().abs() * BF16_ULP + 1e-6)
    with pytest.raises(AssertionError):
        M().layernorm_modulate(x.cuda(), shift.cuda().bfloat16(), scale.cuda())


def test_dit_self_attention_branch():
    """longcat_video_dit.py:88-103: LayerNorm + modulate, attention, gated residual."""
    shape = (4, 8, 8)
    m = make_module(sparsity=0.5, seed=13)
    g = torch.Generator().manual_seed(14)
    x = torch.randn(1, 256, 512, generator=g).bfloat16()
    shift = torch.randn(1, 4, 1, 512, generator=g) * 0.1
    scale = torch.randn(1, 4, 1, 512, generator=g) * 0.1
    gate = torch.randn(1, 4, 1, 512, generator=g)
    x_m = O.layernorm_modulate_fp32(x, shift, scale)
    want = O.gated_residual_fp32(x, gate, module_reference(m, x_m, shape))
    got = M().dit_self_attention_branch(x.cuda(), shift.cuda(), scale.cuda(), gate.cuda(), m.cuda(), shape).cpu()
    d = (got.float() - want.float()).abs()
    assert d.max() <= 6e-2 and d.mean() <= 4e-3, (d.max(), d.mean())


def L():
    from longcat_video_amd.modules import lora
    return lora


def _branch(g, K, N, r, n_sep, multiplier, alpha, scale=0.05, integers=False):
    if integers:
        rnd = lambda *s: torch.randint(-2, 3, s, generator=g).bfloat16()
    else:
        rnd = lambda *s: (torch.randn(*s, generator=g) * scale).bfloat16()
    down = rnd(n_sep * r, K)
    ups = [rnd(N // n_sep, r) for _ in range(n_sep)]
    return L().LoRABranch(down, ups, multiplier, alpha), (down, ups, multiplier, alpha / r)


def test_lora_linear_integer_inputs_are_exact():
    """Small integers make every GEMM, scaling and sum exact, so the three GEMMs (one of them with row
    strides, in three column slices), and the combining pass must reproduce the oracle bit for bit."""
    g = torch.Generator().manual_seed(30)
    K, N, r = 256, 384, 128
    x = torch.randint(-2, 3, (200, K), generator=g).bfloat16()
    w = torch.randint(-2, 3, (N, K), generator=g).bfloat16()
    b = torch.randint(-2, 3, (N,), generator=g).bfloat16()
    br1, t1 = _branch(g, K, N, r, 3, 2.0, 64, integers=True)        # alpha_scale 0.5
    br2, t2 = _branch(g, K, N, r, 1, 0.5, 32, integers=True)        # alpha_scale 0.25
    for brs, terms in (([br1], [t1]), ([br1, br2], [t1, t2])):
        want = O.lora_linear(x, w, b, terms)
        for br in brs:
            br.to("cuda")
        got = L().lora_linear(x.cuda(), w.cuda(), b.cuda(), brs).cpu()
        assert torch.equal(got, want)
    br1.use_lora = br2.use_lora = False                            # set_use_lora(False): plain Linear
    assert torch.equal(L().lora_linear(x.cuda(), w.cuda(), b.cuda(), [br1, br2]).cpu(), O.lora_linear(x, w, b, []))


def test_lora_linear_random_inputs():
    g = torch.Generator().manual_seed(31)
    K, N, r = 512, 1536, 128
    x = torch.randn(300, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) * 0.05).bfloat16()
    b = torch.randn(N, generator=g).bfloat16()
    br, term = _branch(g, K, N, r, 3, 0.8, 64)
    want = O.lora_linear(x, w, b, [term]).float()
    plain = O.lora_linear(x, w, b, []).float()
    got = L().lora_linear(x.cuda(), w.cuda(), b.cuda(), [br.to("cuda")]).cpu().float()
    # GEMM summation order differs from the oracle's: an ulp of each rounded term
    assert torch.all((got - want).abs() <= 3 * BF16_ULP * (want.abs() + plain.abs() + 0.05))
    assert (want - plain).abs().mean() > 10 * (got - want).abs().mean()      # the side branch is not lost in the tolerance


def test_module_forward_with_lora_branches():
    """longcat_video_dit.py:211-249: LoRA branches on attn.qkv (up-projection split in three) and attn.proj."""
    shape = (4, 8, 8)
    m = make_module(sparsity=0.5)
    g = torch.Generator().manual_seed(32)
    x = torch.randn(1, 256, 512, generator=g).bfloat16()
    bq, tq = _branch(g, 512, 1536, 128, 3, 1.0, 64, scale=0.02)
    bp, tp = _branch(g, 512, 512, 128, 1, 1.0, 64, scale=0.02)
    sd = {k: v.detach().cpu() for k, v in m.state_dict().items()}
    prm = dict(sparsity=0.5, chunk_3d_shape_q=(4, 4, 4), chunk_3d_shape_k=(4, 4, 4))
    args = (x, sd["qkv.weight"], sd["qkv.bias"], sd["proj.weight"], sd["proj.bias"], sd["q_norm.weight"],
            sd["k_norm.weight"], shape, m.num_heads, prm, 0)
    want = O.attention_module_forward(*args, qkv_loras=[tq], proj_loras=[tp])
    plain = O.attention_module_forward(*args)
    m = m.cuda()
    m.qkv_loras, m.proj_loras = [bq.to("cuda")], [bp.to("cuda")]
    got = m(x.cuda(), shape=shape).cpu()
    d = (got.float() - want.float()).abs()
    assert d.max() <= 2e-2 and d.mean() <= 2e-3, (d.max(), d.mean())
    assert (want.float() - plain.float()).abs().mean() > 5 * d.mean()        # the branches change the result visibly
    r = torch.randn(1, 256, 512, generator=g).bfloat16()
    got_r = m(x.cuda(), shape=shape, residual=r.cuda()).cpu()
    assert torch.equal(got_r, got + r)


def test_unbuilt_branches_raise():
    m = make_module().cuda()
    x = torch.zeros(1, 256, 512, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        m.forward_with_kv_cache(x, shape=(4, 8, 8), kv_cache=(x.view(1, 4, 256, 128), x.view(1, 4, 256, 128)))
    m.enable_bsa = False
    with pytest.raises(NotImplementedError):
        m(x, shape=(4, 8, 8))


def test_linear_tuning_keeps_results_and_is_remembered():
    """bsa_linear_bf16_tune times hipBLASLt's candidates for a shape and later calls of that shape use the winner;
    the product stays the same GEMM (fp32 accumulation, one rounding; summation order may differ by an ulp)."""
    g = torch.Generator().manual_seed(33)
    x = torch.randn(1, 640, 512, generator=g).bfloat16().cuda()
    w = (torch.randn(768, 512, generator=g) * 0.05).bfloat16().cuda()
    b = torch.randn(768, generator=g).bfloat16().cuda()
    before = M().linear_bf16(x, w, b).cpu()
    n, default_ms, best_ms = M().tune_linear(x, w, b)
    assert n >= 1 and best_ms > 0 and (default_ms == 0 or best_ms <= default_ms * 1.001)
    after = M().linear_bf16(x, w, b).cpu()
    want = x.cpu().float() @ w.cpu().float().t() + b.cpu().float()
    for got in (before, after):
        assert torch.all((got.float() - want).abs() <= want.abs() * BF16_ULP + 2e-3)
    assert torch.equal(after, M().linear_bf16(x, w, b).cpu())          # the remembered choice is deterministic


@pytest.mark.parametrize("grid,dtype", [((4, 8, 8), torch.bfloat16), ((3, 6, 10), torch.bfloat16), ((2, 9, 8), torch.float16)])
def test_operator_with_the_norm_inside_equals_the_separate_passes(grid, dtype):
    """bsa_fwd_3d_qknorm (q and k normalised and rotated inside the operator's own passes) against bsa_norm_rope
    followed by bsa_fwd_3d: same selection, same output bits; a grid of whole chunks and a ragged one; q and k as
    strided views into a token-major projection output."""
    from longcat_video_amd.block_sparse_attention import bsa_interface as bi
    S = grid[0] * grid[1] * grid[2]
    g = torch.Generator().manual_seed(S)
    qkv = (torch.randn(2, S, 3, 4, 128, generator=g) * 2).to(dtype).cuda()
    qw = (1 + 0.1 * torch.randn(128, generator=g)).to(dtype).cuda()
    kw = (1 + 0.1 * torch.randn(128, generator=g)).to(dtype).cuda()
    qs, ks, vs = qkv.permute(2, 0, 3, 1, 4).unbind(0)
    att = M()
    tab = att.rope_table(grid, 128, qkv.device)
    got, idx, lens, score = bi._bsa_3d(qs, ks, vs, grid, grid, 0.5, (4, 4, 4), (4, 4, 4), True,
                                       qk_norm=(qw, kw, tab, grid[0], 0, 0, 1e-6))
    q = att.norm_rope(qs, torch.empty(2, 4, S, 128, dtype=dtype, device="cuda"), qw, grid)
    k = att.norm_rope(ks, torch.empty(2, 4, S, 128, dtype=dtype, device="cuda"), kw, grid)
    want, idx2, lens2, score2 = bi._bsa_3d(q, k, vs, grid, grid, 0.5, (4, 4, 4), (4, 4, 4), True)
    assert torch.equal(score, score2) and torch.equal(idx, idx2) and torch.equal(lens, lens2)
    assert torch.equal(got, want)
    # 128-token chunks are not built for this entry point
    with pytest.raises(NotImplementedError):
        bi._bsa_3d(qs, ks, vs, grid, grid, 0.5, (4, 4, 8), (4, 4, 8), qk_norm=(qw, kw, tab, grid[0], 0, 0, 1e-6))

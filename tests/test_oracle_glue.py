"""Pins the oracle's glue functions (R11): RMSNorm and 3-D RoPE."""
import math

import torch

from oracle import bsa_oracle as O


def test_rms_norm_unit_rms_and_weight():
    x = torch.randn(2, 3, 5, 128, generator=torch.Generator().manual_seed(0)) * 7
    y = O.rms_norm_fp32(x, torch.ones(128))
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(2, 3, 5), atol=1e-4)
    w = torch.linspace(0.5, 2, 128)
    assert torch.allclose(O.rms_norm_fp32(x, w), y * w)
    yb = O.rms_norm_fp32(x.bfloat16(), torch.ones(128, dtype=torch.bfloat16))
    assert yb.dtype == torch.bfloat16


def test_rope_axis_split_and_frequencies():
    ang = O.rope_3d_angles((3, 4, 5), 128)
    assert ang.shape == (60, 128)
    # dims: t = 128 - 4*21 = 44, h = w = 42
    tok = lambda t, h, w: (t * 4 + h) * 5 + w
    a = ang[tok(2, 3, 4)]
    for i in range(22):
        assert math.isclose(a[2 * i].item(), 2 * 10000 ** (-2 * i / 44), rel_tol=1e-5)
        assert a[2 * i].item() == a[2 * i + 1].item()
    for i in range(21):
        assert math.isclose(a[44 + 2 * i].item(), 3 * 10000 ** (-2 * i / 42), rel_tol=1e-5)
        assert math.isclose(a[86 + 2 * i].item(), 4 * 10000 ** (-2 * i / 42), rel_tol=1e-5)
    assert torch.all(ang[0] == 0)


def test_rope_preserves_norm_and_relative_position():
    grid = (2, 3, 6)
    ang = O.rope_3d_angles(grid, 128)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(1, 1, 36, 128, generator=g)
    y = O.rope_3d_apply(x, ang)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), rtol=1e-5)
    assert torch.equal(y[0, 0, 0], x[0, 0, 0])           # position (0,0,0) is the identity
    # same content at every token: q.k depends only on the offset between positions
    qv, kv = torch.randn(128, generator=g), torch.randn(128, generator=g)
    q = O.rope_3d_apply(qv.expand(1, 1, 36, 128), ang)[0, 0]
    k = O.rope_3d_apply(kv.expand(1, 1, 36, 128), ang)[0, 0]
    tok = lambda t, h, w: (t * 3 + h) * 6 + w
    d1 = q[tok(0, 1, 2)] @ k[tok(1, 2, 5)]
    d2 = q[tok(0, 0, 0)] @ k[tok(1, 1, 3)]
    assert math.isclose(d1.item(), d2.item(), rel_tol=1e-4, abs_tol=1e-4)


def test_rope_pairs_are_interleaved():
    ang = torch.zeros(1, 4)
    ang[0, :2] = math.pi / 2
    x = torch.tensor([1.0, 2.0, 3.0, 4.0]).view(1, 1, 1, 4)
    y = O.rope_3d_apply(x, ang)
    assert torch.allclose(y.flatten(), torch.tensor([-2.0, 1.0, 3.0, 4.0]), atol=1e-6)


def test_kv_cache_forward_equals_the_noise_rows_of_the_split_forward():
    """attn:149-181 against attn:107-147: running the conditioning frames first (return_kv) and the new
    frames against the cache must reproduce, bit for bit, the noise rows of one forward over all frames
    with num_cond_latents set: the same keys are normalised, rotated at the same grid positions and
    selected from the same pooled scores in both routes."""
    g = torch.Generator().manual_seed(3)
    heads, C, cond, T, Hh, W = 2, 256, 4, 4, 4, 8
    n_c, n_new = cond * Hh * W, T * Hh * W
    x = torch.randn(1, n_c + n_new, C, generator=g).bfloat16()
    w_qkv = (torch.randn(3 * C, C, generator=g) * 0.05).bfloat16()
    b_qkv = (torch.randn(3 * C, generator=g) * 0.05).bfloat16()
    w_proj = (torch.randn(C, C, generator=g) * 0.05).bfloat16()
    b_proj = (torch.randn(C, generator=g) * 0.05).bfloat16()
    qw = (1 + 0.1 * torch.randn(128, generator=g)).bfloat16()
    kw = (1 + 0.1 * torch.randn(128, generator=g)).bfloat16()
    prm = dict(sparsity=0.5, chunk_3d_shape_q=(4, 4, 4), chunk_3d_shape_k=(4, 4, 4))
    full = O.attention_module_forward(x, w_qkv, b_qkv, w_proj, b_proj, qw, kw, (T + cond, Hh, W), heads, prm, cond)
    cache = O.attention_module_kv(x[:, :n_c], w_qkv, b_qkv, qw, kw, heads)
    assert cache[0].shape == (1, heads, n_c, 128)
    got = O.attention_module_forward_with_kv_cache(x[:, n_c:], w_qkv, b_qkv, w_proj, b_proj, qw, kw, (T, Hh, W), heads,
                                                   prm, cond, cache)
    assert torch.equal(got, full[:, n_c:])
    # the cache is position-free: its keys are not rotated yet
    k_plain = O.rms_norm_fp32((x[:, :n_c].float() @ w_qkv.float().t() + b_qkv.float()).bfloat16()
                              .view(1, n_c, 3, heads, 128)[:, :, 1].transpose(1, 2), kw)
    assert torch.equal(cache[0], k_plain)


def test_layernorm_modulate_against_the_library_routine():
    """The oracle's LayerNorm must be torch's F.layer_norm (what LayerNorm_FP32 calls, blocks.py:60-66); the
    modulation is checked on closed forms: zero shift/scale is the plain norm, and a constant row maps to shift."""
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(5)
    B, T, per, C = 2, 3, 5, 64
    x = (torch.randn(B, T * per, C, generator=g) * 3 + 1).bfloat16()
    shift = torch.randn(B, T, 1, C, generator=g)
    scale = torch.randn(B, T, 1, C, generator=g) * 0.1
    zero = torch.zeros(B, T, 1, C)
    plain = O.layernorm_modulate_fp32(x, zero, zero)
    assert torch.equal(plain, F.layer_norm(x.float(), (C,), None, None, 1e-6).to(torch.bfloat16))
    want = (F.layer_norm(x.float(), (C,), None, None, 1e-6).view(B, T, per, C) * (scale + 1) + shift).to(torch.bfloat16)
    assert torch.equal(O.layernorm_modulate_fp32(x, shift, scale), want.view(B, T * per, C))
    const = torch.full((B, T * per, C), 2.5).bfloat16()
    assert torch.equal(O.layernorm_modulate_fp32(const, shift, scale),
                       shift.expand(B, T, per, C).reshape(B, T * per, C).to(torch.bfloat16))
    # every frame uses its own row of shift / scale
    s2 = shift.clone()
    s2[:, 1] += 1.0
    d = (O.layernorm_modulate_fp32(x, s2, scale).float() - O.layernorm_modulate_fp32(x, shift, scale).float()).view(B, T, per, C)
    assert torch.all(d[:, 0] == 0) and torch.all(d[:, 2] == 0) and torch.all((d[:, 1] - 1).abs() < 0.05)


def test_gated_residual_closed_forms():
    g = torch.Generator().manual_seed(6)
    B, T, per, C = 1, 2, 4, 32
    x = torch.randn(B, T * per, C, generator=g).bfloat16()
    y = torch.randn(B, T * per, C, generator=g).bfloat16()
    assert torch.equal(O.gated_residual_fp32(x, torch.zeros(B, T, 1, C), y), x)
    assert torch.equal(O.gated_residual_fp32(torch.zeros_like(x), torch.ones(B, T, 1, C), y), y)
    gate = torch.randn(B, T, 1, C, generator=g)
    want = (x.float() + gate.expand(B, T, per, C).reshape(B, T * per, C) * y.float()).bfloat16()
    assert torch.equal(O.gated_residual_fp32(x, gate, y), want)


# ---------------------------------------------------------------- LoRA side branches
def _lora_case(seed, M=12, K=16, N=24, r=4, n_sep=1, integers=False, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    if integers:
        rnd = lambda *s: torch.randint(-2, 3, s, generator=g).to(dtype)
    else:
        rnd = lambda *s: torch.randn(*s, generator=g).to(dtype)
    x, w, b = rnd(M, K), rnd(N, K), rnd(N)
    down = rnd(n_sep * r, K)
    ups = [rnd(N // n_sep, r) for _ in range(n_sep)]
    return x, w, b, down, ups


def test_lora_with_zero_up_weights_is_the_plain_linear():
    # the state right after LoRAModule.__init__ (lora_utils.py:60-65: lora_up zero-initialised)
    x, w, b, down, ups = _lora_case(0, n_sep=3)
    plain = torch.nn.functional.linear(x.float(), w.float(), b.float()).bfloat16()
    got = O.lora_linear(x, w, b, [(down, [torch.zeros_like(u) for u in ups], 1.0, 0.5)])
    assert torch.equal(got, plain)
    assert torch.equal(O.lora_linear(x, w, b, []), plain)


def test_lora_on_integers_equals_the_merged_weight():
    # small integers: every product, sum and rounding is exact, so the side branch must equal the
    # textbook merged form x (W + m a U D)^T + b
    x, w, b, down, ups = _lora_case(1, integers=True)
    m, a = 2.0, 0.5
    merged = w.double() + m * a * (ups[0].double() @ down.double())
    want = x.double() @ merged.t() + b.double()
    got = O.lora_linear(x, w, b, [(down, ups, m, a)])
    assert torch.equal(got.double(), want)


def test_lora_split_up_projection_is_block_diagonal():
    x, w, b, down, ups = _lora_case(2, n_sep=3, integers=True)
    r = 4
    full = torch.zeros(24, 12, dtype=torch.bfloat16)
    for i, u in enumerate(ups):
        full[8 * i:8 * i + 8, r * i:r * i + r] = u
    a = O.lora_linear(x, w, b, [(down, ups, 1.0, 1.0)])
    c = O.lora_linear(x, w, b, [(down, [full], 1.0, 1.0)])
    assert torch.equal(a, c)
    # and a transposed or shifted block assignment would not
    wrong = torch.zeros_like(full)
    for i, u in enumerate(ups):
        wrong[8 * i:8 * i + 8, r * ((i + 1) % 3):r * ((i + 1) % 3) + r] = u
    assert not torch.equal(a, O.lora_linear(x, w, b, [(down, [wrong], 1.0, 1.0)]))


def test_lora_rounding_chain_and_two_branches():
    # against the eager expression of longcat_video_dit.py:239-247 written with torch's own bf16 ops
    # (scalar products and sums of bf16 tensors round once per op); the GEMMs are taken in fp32 and rounded
    x, w, b, down, ups = _lora_case(3, n_sep=1)
    _, _, _, down2, ups2 = _lora_case(4, n_sep=3)
    lin = lambda t, wt: (t.float() @ wt.float().t()).bfloat16()
    org = (x.float() @ w.float().t() + b.float()).bfloat16()
    total = 0
    for d, u, m, a in ((down, ups, 0.7, 0.5), (down2, ups2, 1.3, 0.25)):
        lx = lin(x, d)
        lx = torch.cat([lin(c, ui) for c, ui in zip(torch.chunk(lx, len(u), dim=-1), u)], dim=-1)
        total = total + lx * m * torch.tensor(a, dtype=torch.bfloat16)
    want = org + total
    got = O.lora_linear(x, w, b, [(down, ups, 0.7, 0.5), (down2, ups2, 1.3, 0.25)])
    assert want.dtype == torch.bfloat16 and torch.equal(got, want)

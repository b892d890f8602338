"""The C-ABI library loads without a GPU, exports every symbol the header
declares, and rejects bad arguments on the host before anything is launched."""
import ctypes as C
import os
import re

import pytest

from longcat_video_amd import _capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "bsa_mi355x.h")
FAKE = C.c_void_p(0x10000)          # never dereferenced: validation fails first


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    return sorted(set(re.findall(r"\b(bsa_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _capi.load()
    names = declared_functions()
    assert "bsa_fwd_3d" in names and "bsa_permute_thw_to_blocks" in names and len(names) >= 12
    for n in names:
        assert hasattr(lib, n), "library lacks %s" % n
        assert n in _capi.SIGNATURES, "binding lacks %s" % n
    assert sorted(_capi.SIGNATURES) == names


def test_version_and_error_string():
    lib = _capi.load()
    assert lib.bsa_version() >= 100
    assert isinstance(_capi.last_error(), str)


@pytest.mark.parametrize("sparsity,n", [(0.875, 8), (0.9375, 1440), (0.9, 10), (0.0, 7), (1.0, 7), (0.3, 10), (0.9375, 624)])
def test_num_selected_matches_python_doubles(sparsity, n):
    assert _capi.load().bsa_num_selected(sparsity, n) == int((1 - sparsity) * n)


def test_padded_tokens():
    lib = _capi.load()
    assert lib.bsa_padded_tokens(24, 45, 80, 4, 4, 4) == 92160
    assert lib.bsa_padded_tokens(24, 30, 52, 4, 4, 4) == 39936
    assert lib.bsa_padded_tokens(4, 8, 8, 4, 4, 4) == 256
    assert lib.bsa_padded_tokens(0, 8, 8, 4, 4, 4) == -1


def test_permute_rejects_bad_arguments():
    lib = _capi.load()
    st = _capi.strides3([256 * 128, 256 * 128, 128])
    ok_tail = (1, 1, 4, 8, 8, 4, 4, 4, 128, _capi.BSA_BF16, None)
    assert lib.bsa_permute_thw_to_blocks(None, st, FAKE, None, None, *ok_tail) == _capi.BSA_ERR_BAD_ARG
    assert "null" in _capi.last_error()
    assert lib.bsa_permute_thw_to_blocks(FAKE, None, FAKE, None, None, *ok_tail) == _capi.BSA_ERR_BAD_ARG
    bad_dtype = ok_tail[:9] + (7, None)
    assert lib.bsa_permute_thw_to_blocks(FAKE, st, FAKE, None, None, *bad_dtype) == _capi.BSA_ERR_UNSUPPORTED
    odd_d = ok_tail[:8] + (100, _capi.BSA_BF16, None)     # 200-byte rows
    assert lib.bsa_permute_thw_to_blocks(FAKE, st, FAKE, None, None, *odd_d) == _capi.BSA_ERR_UNSUPPORTED
    zero = (1, 1, 0, 8, 8, 4, 4, 4, 128, _capi.BSA_BF16, None)
    assert lib.bsa_permute_thw_to_blocks(FAKE, st, FAKE, None, None, *zero) == _capi.BSA_ERR_BAD_ARG
    misaligned = C.c_void_p(0x10002)
    assert lib.bsa_permute_thw_to_blocks(misaligned, st, FAKE, None, None, *ok_tail) == _capi.BSA_ERR_BAD_ARG
    bad_stride = _capi.strides3([256 * 128, 256 * 128, 100])
    assert lib.bsa_permute_thw_to_blocks(FAKE, bad_stride, FAKE, None, None, *ok_tail) == _capi.BSA_ERR_BAD_ARG
    small_chunk = (1, 1, 4, 8, 8, 2, 2, 2, 128, _capi.BSA_BF16, None)   # 8-token chunk: no 64-slot tiles
    assert lib.bsa_permute_thw_to_blocks(FAKE, st, FAKE, None, FAKE, *small_chunk) == _capi.BSA_ERR_UNSUPPORTED


def test_topk_rejects_bad_arguments():
    lib = _capi.load()
    assert lib.bsa_topk_from_score(FAKE, FAKE, None, FAKE, 1, 1, 4, 4, 5, _capi.BSA_BF16, None) == _capi.BSA_ERR_SHAPE
    assert lib.bsa_topk_from_score(FAKE, FAKE, None, FAKE, 1, 1, 4, 5000, 5, _capi.BSA_BF16, None) == _capi.BSA_ERR_UNSUPPORTED
    assert lib.bsa_topk_from_score(FAKE, FAKE, None, FAKE, 1, 1, 4, 4096, 4097, _capi.BSA_BF16, None) == _capi.BSA_ERR_SHAPE
    assert lib.bsa_topk_from_score(None, FAKE, None, FAKE, 1, 1, 4, 4, 2, _capi.BSA_BF16, None) == _capi.BSA_ERR_BAD_ARG
    assert lib.bsa_score_topk(FAKE, FAKE, FAKE, None, FAKE, FAKE, 1, 1, 4, 4, 100, 2, _capi.BSA_BF16, None) == _capi.BSA_ERR_UNSUPPORTED
    assert lib.bsa_score_topk(FAKE, FAKE, FAKE, None, FAKE, None, 1, 1, 4, 4, 128, 2, _capi.BSA_BF16, None) == _capi.BSA_ERR_BAD_ARG
    assert lib.bsa_score_topk(FAKE, FAKE, None, None, FAKE, FAKE, 1, 1, 4, 4, 128, 2, _capi.BSA_BF16, None) == _capi.BSA_ERR_BAD_ARG


def test_fwd_rejects_bad_arguments():
    lib = _capi.load()
    ptrs = [FAKE] * 5 + [None, FAKE, None]

    def call(B=1, Hn=1, Sq=256, Sk=256, D=128, bs_q=64, bs_k=64, stride=2, scale=0.088, dtype=_capi.BSA_BF16, p=ptrs):
        return lib.bsa_fwd(*p, B, Hn, Sq, Sk, D, bs_q, bs_k, stride, scale, dtype, None)

    assert call(D=64) == _capi.BSA_ERR_UNSUPPORTED and "128" in _capi.last_error()
    assert call(bs_q=48) == _capi.BSA_ERR_UNSUPPORTED
    assert call(Sq=200) == _capi.BSA_ERR_SHAPE
    assert call(Sk=100) == _capi.BSA_ERR_SHAPE
    assert call(scale=0.0) == _capi.BSA_ERR_BAD_ARG
    assert call(scale=float("nan")) == _capi.BSA_ERR_BAD_ARG
    assert call(dtype=9) == _capi.BSA_ERR_UNSUPPORTED
    assert call(B=0) == _capi.BSA_ERR_BAD_ARG
    assert call(p=[None] + ptrs[1:]) == _capi.BSA_ERR_BAD_ARG


def test_fwd_fragment_and_bwd_shape_limits():
    """The blocked-order entry on the fragment-order kernel and the backward reject what they cannot run before any
    launch (no GPU is touched: every check comes before the first HIP call)."""
    lib = _capi.load()
    need = lib.bsa_fwd_fragment_workspace_bytes(1, 2, 640, 1280, 128, _capi.BSA_BF16)
    assert need >= 2 * 2 * 1280 * 128 * 2 and need % 256 == 0                      # K and V in fragment order, two tables
    assert lib.bsa_fwd_fragment_workspace_bytes(1, 2, 640, 1280, 128, _capi.BSA_F32) == 0
    assert lib.bsa_fwd_fragment_workspace_bytes(1, 2, 640, 1290, 128, _capi.BSA_BF16) == 0
    ptrs = [FAKE] * 5 + [None, FAKE, None]

    def call(Sq=640, Sk=1280, D=128, bs_q=64, bs_k=64, stride=3, dtype=_capi.BSA_BF16, ws=FAKE, ws_bytes=1 << 30):
        return lib.bsa_fwd_fragment(*ptrs, 1, 2, Sq, Sk, D, bs_q, bs_k, stride, 0.088, dtype, ws, ws_bytes, None)

    assert call(dtype=_capi.BSA_F32) == _capi.BSA_ERR_UNSUPPORTED
    assert call(D=64) == _capi.BSA_ERR_UNSUPPORTED
    assert call(Sq=650) == _capi.BSA_ERR_SHAPE
    assert call(stride=5000) == _capi.BSA_ERR_UNSUPPORTED and "4096" in _capi.last_error()
    assert call(ws=None) == _capi.BSA_ERR_BAD_ARG
    assert call(ws_bytes=need - 1) == _capi.BSA_ERR_WORKSPACE
    # the backward stages a KV block's query blocks in LDS: more query blocks than fit are refused, with the number
    assert lib.bsa_bwd_workspace_bytes(1, 1, 64 * 23552, 64, 128, 64, 64, 1, _capi.BSA_BF16) > 0
    assert lib.bsa_bwd_workspace_bytes(1, 1, 64 * 23553, 64, 128, 64, 64, 1, _capi.BSA_BF16) == 0
    assert "23552" in _capi.last_error()


def test_fwd_3d_plan_and_workspace():
    lib = _capi.load()
    prm = _capi.Bsa3dParams(1, 32, 128, _capi.BSA_BF16, 24, 45, 80, 24, 45, 80, 4, 4, 4, 4, 4, 4, 90, 0.0883883)
    need = lib.bsa_workspace_bytes(C.byref(prm))
    # q and o are used where they lie; k and v are rewritten once, in fragment order, at their padded size;
    # plus pooled vectors, the score matrix and the lists
    kv = 2 * 32 * 92160 * 128 * 2
    assert need > kv and need < kv + 300 * 2 ** 20
    prm32 = _capi.Bsa3dParams(1, 32, 128, _capi.BSA_F32, 24, 45, 80, 24, 45, 80, 4, 4, 4, 4, 4, 4, 90, 0.0883883)
    assert lib.bsa_workspace_bytes(C.byref(prm32)) > 4 * 32 * 92160 * 128 * 4     # fp32: blocked copies of all four
    st = _capi.strides3([32 * 86400 * 128, 86400 * 128, 128])
    args = (FAKE, st, FAKE, st, FAKE, st, FAKE, st)
    ws = C.c_void_p(0x100000)
    assert lib.bsa_fwd_3d(C.byref(prm), *args, ws, need - 1, None, None, None, None) == _capi.BSA_ERR_WORKSPACE
    assert lib.bsa_fwd_3d(C.byref(prm), *args, C.c_void_p(0x100010), need, None, None, None, None) == _capi.BSA_ERR_BAD_ARG
    prm.k_sel = 2000
    assert lib.bsa_workspace_bytes(C.byref(prm)) == 0
    assert lib.bsa_fwd_3d(C.byref(prm), *args, ws, need, None, None, None, None) == _capi.BSA_ERR_SHAPE
    prm.k_sel, prm.D = 90, 64
    assert lib.bsa_fwd_3d(C.byref(prm), *args, ws, need, None, None, None, None) == _capi.BSA_ERR_UNSUPPORTED
    prm.D, prm.tq = 128, 2                          # 32-token query chunks
    assert lib.bsa_fwd_3d(C.byref(prm), *args, ws, need, None, None, None, None) == _capi.BSA_ERR_UNSUPPORTED
    assert lib.bsa_fwd_3d(None, *args, ws, need, None, None, None, None) == _capi.BSA_ERR_BAD_ARG


def test_gemm_and_qkv_projection_reject_bad_arguments():
    lib = _capi.load()

    def gemm(x=FAKE, ldx=256, w=FAKE, ldw=256, bias=None, res=None, ldr=0, out=FAKE, ldo=256, M=300, N=256, K=256):
        return lib.bsa_gemm_bf16(x, ldx, w, ldw, bias, res, ldr, out, ldo, M, N, K, None)

    assert gemm(x=None) == _capi.BSA_ERR_BAD_ARG
    assert gemm(out=None) == _capi.BSA_ERR_BAD_ARG
    assert gemm(K=96, ldx=96, ldw=96) == _capi.BSA_ERR_UNSUPPORTED and "64" in _capi.last_error()
    assert gemm(N=200, ldo=200) == _capi.BSA_ERR_UNSUPPORTED and "128" in _capi.last_error()
    assert gemm(ldx=128) == _capi.BSA_ERR_BAD_ARG                   # row stride below K
    assert gemm(ldo=128) == _capi.BSA_ERR_BAD_ARG                   # row stride below N
    assert gemm(res=FAKE, ldr=100) == _capi.BSA_ERR_BAD_ARG
    assert gemm(M=0) == _capi.BSA_ERR_BAD_ARG
    assert gemm(x=C.c_void_p(0x10008)) == _capi.BSA_ERR_BAD_ARG     # 16-byte alignment
    assert gemm(ldx=1 << 23) == _capi.BSA_ERR_UNSUPPORTED

    st = _capi.strides3([4 * 256 * 128, 256 * 128, 128])

    def qkv(x=FAKE, q=FAKE, tab=FAKE, qw=FAKE, B=1, Hn=4, T=4, H=8, W=8, t0=0, table_T=4, D=128, K=512, eps=1e-6, strides=st):
        return lib.bsa_qkv_projection(x, K, FAKE, K, None, qw, FAKE, tab, q, FAKE, FAKE, strides, B, Hn, T, H, W, t0, table_T, D, K, eps, None)

    assert qkv(D=64) == _capi.BSA_ERR_UNSUPPORTED
    assert qkv(x=None) == _capi.BSA_ERR_BAD_ARG
    assert qkv(q=None) == _capi.BSA_ERR_BAD_ARG
    assert qkv(tab=None) == _capi.BSA_ERR_BAD_ARG
    assert qkv(qw=None) == _capi.BSA_ERR_BAD_ARG
    assert qkv(T=0) == _capi.BSA_ERR_BAD_ARG
    assert qkv(t0=2) == _capi.BSA_ERR_SHAPE                         # frames 2..6 of a table of 4
    assert qkv(K=100) == _capi.BSA_ERR_UNSUPPORTED
    assert qkv(eps=-1.0) == _capi.BSA_ERR_BAD_ARG
    assert qkv(strides=_capi.strides3([4 * 256 * 128, 256 * 128, 100])) == _capi.BSA_ERR_BAD_ARG


def test_fwd_3d_qknorm_rejects_bad_arguments():
    lib = _capi.load()
    prm = _capi.Bsa3dParams(1, 4, 128, _capi.BSA_BF16, 4, 8, 8, 4, 8, 8, 4, 4, 4, 4, 4, 4, 2, 0.0883883)
    need = lib.bsa_workspace_bytes(C.byref(prm))
    st = _capi.strides3([4 * 256 * 128, 256 * 128, 128])
    ws = C.c_void_p(0x100000)

    def call(p=prm, n=None, qn=FAKE, q_weight=FAKE, tab=FAKE, table_T=4, t_q=0, t_k=0, eps=1e-6):
        norm = _capi.BsaQkNorm(q_weight, FAKE, tab, table_T, t_q, t_k, eps) if n is None else n
        return lib.bsa_fwd_3d_qknorm(C.byref(p), C.byref(norm) if norm is not False else None, FAKE, st, qn, st, FAKE, st, FAKE, st,
                                     FAKE, st, ws, need, None, None, None, None)

    assert call(n=False) == _capi.BSA_ERR_BAD_ARG
    assert call(qn=None) == _capi.BSA_ERR_BAD_ARG
    assert call(q_weight=None) == _capi.BSA_ERR_BAD_ARG
    assert call(tab=None) == _capi.BSA_ERR_BAD_ARG
    assert call(table_T=3) == _capi.BSA_ERR_SHAPE
    assert call(t_k=1) == _capi.BSA_ERR_SHAPE
    assert call(eps=-1.0) == _capi.BSA_ERR_BAD_ARG
    assert call(q_weight=C.c_void_p(0x10008)) == _capi.BSA_ERR_BAD_ARG
    big = _capi.Bsa3dParams(1, 4, 128, _capi.BSA_BF16, 4, 8, 8, 4, 8, 8, 4, 4, 8, 4, 4, 8, 1, 0.0883883)      # 128-token chunks
    assert call(p=big) == _capi.BSA_ERR_UNSUPPORTED and "64-token" in _capi.last_error()
    f32 = _capi.Bsa3dParams(1, 4, 128, _capi.BSA_F32, 4, 8, 8, 4, 8, 8, 4, 4, 4, 4, 4, 4, 2, 0.0883883)
    assert call(p=f32) == _capi.BSA_ERR_UNSUPPORTED
    long_axis = _capi.Bsa3dParams(1, 4, 128, _capi.BSA_BF16, 4, 8, 16, 4, 8, 16, 1, 4, 16, 1, 4, 16, 2, 0.0883883)  # 16 positions on one axis
    assert call(p=long_axis) == _capi.BSA_ERR_UNSUPPORTED


def test_status_to_exception_mapping():
    lib = _capi.load()
    rc = lib.bsa_topk_from_score(FAKE, FAKE, None, FAKE, 1, 1, 4, 4, 5, _capi.BSA_BF16, None)
    with pytest.raises(AssertionError):
        _capi.check(rc)
    rc = lib.bsa_topk_from_score(None, FAKE, None, FAKE, 1, 1, 4, 4, 2, _capi.BSA_BF16, None)
    with pytest.raises(ValueError):
        _capi.check(rc)
    rc = lib.bsa_topk_from_score(FAKE, FAKE, None, FAKE, 1, 1, 4, 5000, 5, _capi.BSA_BF16, None)
    with pytest.raises(NotImplementedError):
        _capi.check(rc)
    _capi.check(0)


def test_header_and_library_from_a_plain_c_program(tmp_path):
    """include/bsa_mi355x.h is C, and the library needs no Python or torch around it."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no C compiler")
    exe = str(tmp_path / "capi_from_c")
    src = os.path.join(ROOT, "tests", "capi_from_c.c")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), src, "-o", exe, "-ldl"], check=True)
    _capi.load()                       # raises with the build hint if the library is missing
    out = subprocess.run([exe, _capi.LIB_PATH], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and out.stdout.startswith("ok"), (out.returncode, out.stdout, out.stderr)

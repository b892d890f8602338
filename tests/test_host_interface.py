"""Host-side mirror of the reference call surface: names, signature, and the
errors raised before any GPU work (runs without a GPU)."""
import inspect

import pytest
import torch

from longcat_video_amd.block_sparse_attention import bsa_interface as I


def test_reference_names_exist():
    for name in ("flash_attn_bsa_3d", "flash_attn_bsa", "rearrange_THW_to_3d_block", "rearrange_3d_block_to_THW",
                 "mean_pooling_compression", "cal_score", "get_select_indices", "get_select_indices_topk",
                 "get_select_indices_topk_from_score", "attn_fwd_bsa_varlen_triton"):
        assert callable(getattr(I, name))


def test_flash_attn_bsa_3d_signature_matches_the_reference():
    sig = inspect.signature(I.flash_attn_bsa_3d)
    names = list(sig.parameters)
    assert names[:9] == ["q", "k", "v", "latent_shape_q", "latent_shape_k", "sparsity", "cdf_threshold",
                         "chunk_3d_shape_q", "chunk_3d_shape_k"]
    assert sig.parameters["sparsity"].default == 0.875
    assert sig.parameters["cdf_threshold"].default is None
    assert sig.parameters["chunk_3d_shape_q"].default == [4, 4, 8]
    assert sig.parameters["chunk_3d_shape_k"].default == [4, 4, 8]


def qkv(S=256, D=128, H=2):
    return [torch.zeros(1, H, S, D, dtype=torch.bfloat16) for _ in range(3)]


def test_shape_violations_raise_assertion_error():
    q, k, v = qkv()
    prm = dict(chunk_3d_shape_q=[4, 4, 4], chunk_3d_shape_k=[4, 4, 4])
    with pytest.raises(AssertionError):
        I.flash_attn_bsa_3d(q, k, v, (4, 8, 9), (4, 8, 8), **prm)            # T*H*W != S
    with pytest.raises(AssertionError):
        I.flash_attn_bsa_3d(q, k[..., :64], v[..., :64], (4, 8, 8), (4, 8, 8), **prm)   # head dims differ
    with pytest.raises(AssertionError):
        I.flash_attn_bsa_3d(q, k, v, (4, 8, 8), (4, 8, 8), chunk_3d_shape_q=[4, 4, 3], chunk_3d_shape_k=[4, 4, 4],
                            allow_padding=False)                               # reference divisibility assert
    q96 = [t[..., :96] for t in (q, k, v)]
    with pytest.raises(AssertionError):
        I.flash_attn_bsa_3d(*q96, (4, 8, 8), (4, 8, 8), **prm)                # head dim outside {16..256}


def test_selection_mode_errors():
    q, k, v = qkv()
    with pytest.raises(ValueError):
        I.flash_attn_bsa_3d(q, k, v, (4, 8, 8), (4, 8, 8), sparsity=None, cdf_threshold=None)
    with pytest.raises(RuntimeError, match="GPU only"):          # the CDF rule is built: CPU tensors get as far as the engine
        I.flash_attn_bsa_3d(q, k, v, (4, 8, 8), (4, 8, 8), sparsity=None, cdf_threshold=0.9)
    with pytest.raises(ValueError):
        I.get_select_indices(q, k, None, None)
    with pytest.raises(ValueError):
        I.get_select_indices_from_score(q, None, None)


def test_no_cpu_fallback_with_or_without_gradients():
    q, k, v = qkv()
    with pytest.raises(RuntimeError, match="GPU only"):
        I.flash_attn_bsa_3d(q, k, v, (4, 8, 8), (4, 8, 8), chunk_3d_shape_q=[4, 4, 4], chunk_3d_shape_k=[4, 4, 4])
    with pytest.raises(RuntimeError, match="GPU only"):
        I.mean_pooling_compression(q, 64)
    q.requires_grad_(True)                       # the differentiable route runs on the GPU only as well
    with pytest.raises(RuntimeError, match="GPU only"):
        I.flash_attn_bsa_3d(q, k, v, (4, 8, 8), (4, 8, 8), chunk_3d_shape_q=[4, 4, 4], chunk_3d_shape_k=[4, 4, 4])
    with pytest.raises(NotImplementedError, match="bf16 and fp16"):
        I.flash_attn_bsa_3d(q.float().requires_grad_(True), k.float(), v.float(), (4, 8, 8), (4, 8, 8),
                            chunk_3d_shape_q=[4, 4, 4], chunk_3d_shape_k=[4, 4, 4])


def test_num_selected():
    assert I.num_selected(0.9375, 1440) == 90 and I.num_selected(0.9, 10) == 0


def test_module_caches_are_bounded():
    """The per-stream GEMM workspaces and the per-grid rotation tables forget their oldest entry beyond a limit."""
    from longcat_video_amd.modules import attention as A
    d = A._Bounded(3)
    for i in range(5):
        d[i] = i
    assert list(d) == [2, 3, 4]
    d[3] = 30                                    # rewriting a key evicts nothing
    assert list(d) == [2, 3, 4] and d[3] == 30
    assert isinstance(A._GEMM_WORKSPACES, A._Bounded) and isinstance(A._ROPE_TABLES, A._Bounded)

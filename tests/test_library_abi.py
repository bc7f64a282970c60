"""CPU-side checks of the C-ABI library: it loads and exports every symbol the header
declares; argument structs have the layout the header gives them; the host-side
validation of the binding raises before anything touches a GPU."""
import ctypes
import os
import re

import pytest
import torch

from flash_moba import flash_moba_hip as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_functions():
    src = open(os.path.join(ROOT, "include", "flash_moba_hip.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(fmoba_[a-z_0-9]+)\s*\(", src)))


def test_header_declares_the_expected_entry_points():
    fns = header_functions()
    for need in ("fmoba_mean_pool", "fmoba_fused_topk", "fmoba_varlen_sort", "fmoba_attn_fwd", "fmoba_attn_bwd",
                 "fmoba_last_error", "fmoba_version", "fmoba_check_device"):
        assert need in fns


def test_library_loads_and_exports_every_declared_symbol():
    lib = H.load_library()
    for fn in header_functions():
        assert hasattr(lib, fn), fn
        assert fn in H.EXPORTS, f"{fn} is declared in the header but not bound"
    assert lib.fmoba_version() >= 100
    assert lib.fmoba_last_error() is not None


def test_workspace_queries_are_pure_host_functions():
    lib = H.load_library()
    # selection bits: heads * ceil(maxC/32) * total_q words; counts: batch*heads*nseg*maxC words
    b = lib.fmoba_fused_topk_workspace_bytes(8, 65536, 16, 14336, 14336, 64)
    assert b >= 16 * 7 * 65536 * 4 + 8 * 16 * 28 * 224 * 4  # 512-row counting segments at this size
    assert lib.fmoba_fused_topk_workspace_bytes(0, 0, 0, 0, 0, 0) == 0
    # `total` int32, then 256 bytes of notes on a 256-byte boundary
    assert lib.fmoba_varlen_sort_workspace_bytes(1000) == 4096 + 256
    assert lib.fmoba_varlen_sort_workspace_bytes(0) == 0
    a = H.AttnBwdArgs()
    a.total_q, a.heads, a.head_dim, a.batch, a.total_k, a.lg_block_n, a.max_visits_per_row, a.num_row_indices = 1024, 4, 128, 1, 1024, 64, 8, 32768
    a.dq_mode = 2
    assert lib.fmoba_attn_bwd_workspace_bytes(ctypes.byref(a)) >= 1024 * 4 * 8 * 128 * 2
    a.dq_mode = 1
    assert lib.fmoba_attn_bwd_workspace_bytes(ctypes.byref(a)) >= 32768 * 64 * 2
    f = H.AttnFwdArgs()
    f.total_q, f.heads, f.heads_k, f.head_dim, f.batch, f.total_k, f.lg_block_n, f.max_visits_per_row = 1024, 4, 4, 128, 1, 1024, 64, 8
    f.max_seqlen_q = f.max_seqlen_k = 1024
    f.max_cols, f.is_causal = 16, 1
    f.fwd_mode = 1  # columns: one partial row + header per visit
    assert lib.fmoba_attn_fwd_uses_row_blocks(ctypes.byref(f)) == 0
    assert lib.fmoba_attn_fwd_workspace_bytes(ctypes.byref(f)) >= 1024 * 4 * 8 * (128 * 2 + 16)
    f.fwd_mode = 2  # row blocks: one selection bit per (row, head, chunk)
    assert lib.fmoba_attn_fwd_uses_row_blocks(ctypes.byref(f)) == 1
    assert 1024 * 4 * 4 <= lib.fmoba_attn_fwd_workspace_bytes(ctypes.byref(f)) < 1024 * 4 * 4 + 1024
    f.fwd_mode = 0  # 8 of at most 16 chunks per row: dense enough for row blocks
    assert lib.fmoba_attn_fwd_uses_row_blocks(ctypes.byref(f)) == 1
    f.total_k = f.max_seqlen_k = 1 << 20  # 16384 chunks: columns
    f.max_cols = 16384
    assert lib.fmoba_attn_fwd_uses_row_blocks(ctypes.byref(f)) == 0
    assert lib.fmoba_attn_fwd_key_block(64) == 64 and lib.fmoba_attn_fwd_key_block(128) == 128 and lib.fmoba_attn_fwd_key_block(192) == 64


@pytest.mark.parametrize("lens,chunk,topk,fwd_rows,dq_partials", [
    ([8192], 128, 8, 0, 1),           # a row selects 8 of 32 visible 128-key chunks: columns, partials
    ([4096, 4096], 128, 8, 1, 0),     # 8 of 16: row blocks in both passes
    ([32768], 128, 16, 0, 1),         # 16 of 128
    ([8192] * 8, 64, 32, 1, 0),       # the headline density, 32 of 64 visible 64-key chunks: row blocks
    ([8192, 8192], 64, 16, 1, 0),     # 16 of 64: still row blocks with 64-key blocks
    ([8192, 8192], 64, 8, 0, 0),      # 8 of 64: column forward, but the row-block dQ until a tenth
    ([262144], 128, 16, 0, 1),
])
def test_form_choice_follows_the_measured_break_even_points(lens, chunk, topk, fwd_rows, dq_partials):
    lib = H.load_library()
    T, L = sum(lens), max(lens)
    f = H.AttnFwdArgs()
    f.total_q = f.total_k = T
    f.heads = f.heads_k = 16
    f.head_dim, f.batch, f.lg_block_n, f.is_causal = 128, len(lens), chunk, 1
    f.max_seqlen_q = f.max_seqlen_k = L
    f.max_cols = (L + chunk - 1) // chunk
    f.max_visits_per_row = topk * (chunk // lib.fmoba_attn_fwd_key_block(chunk))
    assert lib.fmoba_attn_fwd_uses_row_blocks(ctypes.byref(f)) == fwd_rows
    a = H.AttnBwdArgs()
    a.total_q = a.total_k = T
    a.heads = a.heads_k = 16
    a.head_dim, a.batch, a.lg_block_n, a.is_causal = 128, len(lens), chunk, 1
    a.max_seqlen_q = a.max_seqlen_k = L
    a.max_visits_per_row = topk * (chunk // 64)
    assert lib.fmoba_attn_bwd_uses_partials(ctypes.byref(a)) == dq_partials


def test_struct_sizes_match_the_header_layout():
    # pointers and int64 are 8 bytes, int32/float 4; sizes follow from the field lists
    assert ctypes.sizeof(H.MeanPoolArgs) == 4 * 8 + 6 * 4 + 4 * 8
    assert ctypes.sizeof(H.FusedTopkArgs) == 11 * 8 + 8 + 11 * 4 + 4 + 4 * 8
    assert ctypes.sizeof(H.AttnFwdArgs) % 8 == 0
    assert ctypes.sizeof(H.AttnBwdArgs) % 8 == 0


def test_null_args_are_rejected_with_a_message():
    lib = H.load_library()
    assert lib.fmoba_mean_pool(None, None) != 0
    assert b"null" in lib.fmoba_last_error()
    assert lib.fmoba_fused_topk(None, None) != 0
    assert lib.fmoba_attn_fwd(None, None) != 0
    assert lib.fmoba_attn_bwd(None, None) != 0


def test_host_validation_needs_no_gpu():
    q = torch.zeros(4, 2, 8)          # fp32, CPU
    cu = torch.tensor([0, 4], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="fp16 and bf16"):
        H.moba_fused_topk(q, q, cu, cu, cu, 4, 4, 2, 2, True)
    with pytest.raises(RuntimeError, match="on CUDA"):
        H.moba_fused_topk(q.half(), q.half(), cu, cu, cu, 4, 4, 2, 2, True)
    with pytest.raises(RuntimeError, match="int64"):
        H.varlen_sort(cu, cu, cu)


def test_public_api_signatures_are_the_reference_ones():
    import inspect

    import flash_moba
    from flash_moba import flash_moba_interface as I

    assert list(inspect.signature(flash_moba.flash_moba_varlen_func).parameters) == [
        "q", "k", "v", "cu_seqlens_q", "cu_seqlens_k", "max_seqlen_q", "max_seqlen_k", "moba_chunk_size", "moba_topk", "causal"]
    assert inspect.signature(flash_moba.flash_moba_varlen_func).parameters["causal"].default is True
    assert list(inspect.signature(flash_moba.flash_topk_varlen_func).parameters) == [
        "q", "k", "cu_seqlens_q", "cu_seqlens_k", "max_seqlen_q", "max_seqlen_k", "moba_topk", "moba_chunk_size", "causal"]
    assert inspect.signature(flash_moba.flash_topk_varlen_func).parameters["causal"].default is False
    p = inspect.signature(flash_moba.flash_moba_attn_varlen_func).parameters
    assert list(p) == ["q", "k", "v", "cu_seqlens_q", "cu_seqlens_k", "max_seqlen_q", "max_seqlen_k",
                       "moba_col_offsets", "moba_col_nnz", "moba_row_indices", "lg_block_m", "lg_block_n", "dropout_p",
                       "softmax_scale", "causal", "softcap", "alibi_slopes", "deterministic", "return_attn_probs"]
    assert (p["lg_block_m"].default, p["lg_block_n"].default, p["causal"].default) == (64, 64, False)
    for op in ("_moba_fused_topk", "_varlen_sort", "_flash_moba_attn_varlen_forward", "_flash_moba_attn_varlen_backward"):
        assert hasattr(torch.ops.flash_moba, op)
    assert I.decide_lg_block_m(8, 128, 8192, True) == 512
    from flash_moba.triton_mean_pool import flash_topk_mean_pool  # import path of the reference
    assert callable(flash_topk_mean_pool)


def test_fake_shape_functions():
    from torch._subclasses.fake_tensor import FakeTensorMode

    import flash_moba  # noqa: F401  (registers the ops)

    with FakeTensorMode():
        q = torch.empty(100, 4, 64, dtype=torch.bfloat16, device="cuda")
        km = torch.empty(10, 4, 64, dtype=torch.bfloat16, device="cuda")
        cu = torch.empty(3, dtype=torch.int32, device="cuda")
        co, cn, ind = torch.ops.flash_moba._moba_fused_topk(q, km, cu, cu, cu, 60, 60, 3, 16, True)
        assert co.shape == (2, 4, 4) and co.dtype == torch.int64
        assert cn.shape == (2, 4, 4) and cn.dtype == torch.int32
        assert ind.shape == (100 * 4 * 3,) and ind.dtype == torch.int32
        out, lse, p, rng = torch.ops.flash_moba._flash_moba_attn_varlen_forward(
            q, q, q, cu, cu, 60, 60, co, cn, ind, 128, 64, 0.0, 0.125, True)
        assert out.shape == q.shape and lse.shape == (4, 100) and p.shape == (0,) and rng.shape == (2,)
        sd = torch.ops.flash_moba._flash_moba_attn_varlen_backward(
            q, q, q, q, out, lse, None, None, None, cu, cu, 60, 60, co, cn, ind, 128, 64, 0.0, 0.125, True, 0.0, None, False)
        assert sd.shape == (4, 100 + 128 * 2)
        # the private ops of the fused path: the visits bound and the selection bits are ordinary arguments
        km2, cu_km = torch.ops.flash_moba._mean_pool(q, cu, 60, 16)
        assert km2.shape == (100 // 16 + 2, 4, 64) and cu_km.dtype == torch.int32 and cu_km.shape == cu.shape
        co, cn, ind, sel = torch.ops.flash_moba._gated_topk(q, km, cu, cu, cu, 60, 60, 3, 16, True)
        assert sel.shape == (4, 1, 100) and sel.dtype == torch.int32 and ind.shape == (100 * 4 * 3,)
        out, lse, p, rng = torch.ops.flash_moba._attn_varlen_forward_bounded(
            q, q, q, cu, cu, 60, 60, co, cn, ind, 128, 64, 0.125, True, 3, sel)
        assert out.shape == q.shape and lse.shape == (4, 100) and p.shape == (0,) and rng.shape == (2,)
        dq = torch.empty_like(q)
        sd = torch.ops.flash_moba._attn_varlen_backward_bounded(
            q, q, q, q, out, lse, dq, dq, dq, cu, cu, 60, 60, co, cn, ind, 128, 64, 0.125, True, False, 3)
        assert sd.shape == (4, 100 + 128 * 2)


def test_fused_path_traces_end_to_end_on_fake_tensors():
    # flash_moba_varlen_func touches the GPU only through custom ops with fake-shape functions: on fake tensors the
    # whole forward runs without a device and without any state outside the op arguments
    from torch._subclasses.fake_tensor import FakeTensorMode

    import flash_moba

    with FakeTensorMode():
        q, k, v = (torch.empty(700, 4, 72, dtype=torch.bfloat16, device="cuda", requires_grad=True) for _ in range(3))
        cu = torch.empty(3, dtype=torch.int32, device="cuda")
        out = flash_moba.flash_moba_varlen_func(q, k, v, cu, cu, 400, 400, 64, 3, causal=True)
        assert out.shape == q.shape and out.dtype == q.dtype
        assert out.grad_fn is not None  # (running the backward needs the autograd engine's device thread: GPU test)


def test_key_block_rule_of_the_host_code_matches_the_library():
    from flash_moba import flash_moba_interface as I

    lib = H.load_library()
    for n in (64, 128, 192, 256, 320, 1024):
        assert I._fwd_key_block(n) == H.fwd_key_block(n) == lib.fmoba_attn_fwd_key_block(n)


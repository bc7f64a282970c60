"""Thin binding over the C ABI of libflash_moba_hip.so (include/flash_moba_hip.h).

This module plays the role of the reference's compiled module ``flash_moba_cuda``
(csrc/flash_moba_binding.cpp:6-10): it exposes the same four callables with the same
positional signatures and return lists

    moba_fused_topk   csrc/flash_topk/flash_topk_api.cpp:130-140,257
    varlen_sort       csrc/flash_topk/src/varlen_sort.cu:127-161
    moba_varlen_fwd   csrc/flash_moba/flash_moba_api.cpp:375-398,595
    moba_varlen_bwd   csrc/flash_moba/flash_moba_api.cpp:610-637,847

plus ``mean_pool`` (the kernel the reference launches from
flash_moba/triton_mean_pool.py:146).  It validates arguments the way the reference's host
code does (same conditions, RuntimeError), allocates outputs and scratch with torch on the
tensors' device, and passes raw device pointers, sizes and the current HIP stream to the
library.  PyTorch is used for device memory and streams only; there is no CPU or eager
fallback: if the library is missing or the device is not a gfx950 part, calls fail.
"""
from __future__ import annotations

import contextlib
import ctypes
import threading
import os
from typing import List, Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libflash_moba_hip.so")

c_i32, c_i64, c_f32, c_vp, c_sz = ctypes.c_int32, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t


class MeanPoolArgs(ctypes.Structure):
    _fields_ = [("k", c_vp), ("km", c_vp), ("cu_seqlens_k", c_vp), ("cu_seqlens_km", c_vp),
                ("batch", c_i32), ("max_chunks", c_i32), ("heads_k", c_i32), ("head_dim", c_i32),
                ("chunk", c_i32), ("dtype", c_i32),
                ("k_row_stride", c_i64), ("k_head_stride", c_i64), ("km_row_stride", c_i64), ("km_head_stride", c_i64)]


class FusedTopkArgs(ctypes.Structure):
    _fields_ = [("q", c_vp), ("km", c_vp), ("cu_seqlens_q", c_vp), ("cu_seqlens_k", c_vp), ("cu_seqlens_km", c_vp),
                ("col_offsets", c_vp), ("col_nnz", c_vp), ("flat_indices", c_vp), ("raw_indices", c_vp),
                ("raw_values", c_vp), ("workspace", c_vp), ("workspace_bytes", c_sz),
                ("batch", c_i32), ("total_q", c_i32), ("heads", c_i32), ("heads_k", c_i32), ("head_dim", c_i32),
                ("max_seqlen_q", c_i32), ("max_seqlen_k", c_i32),
                ("topk", c_i32), ("chunk", c_i32), ("is_causal", c_i32), ("dtype", c_i32),
                ("q_row_stride", c_i64), ("q_head_stride", c_i64), ("km_row_stride", c_i64), ("km_head_stride", c_i64)]


class AttnFwdArgs(ctypes.Structure):
    _fields_ = [("q", c_vp), ("k", c_vp), ("v", c_vp), ("out", c_vp), ("softmax_lse", c_vp),
                ("col_offsets", c_vp), ("col_nnz", c_vp), ("row_indices", c_vp),
                ("cu_seqlens_q", c_vp), ("cu_seqlens_k", c_vp), ("selection_bits", c_vp),
                ("workspace", c_vp), ("workspace_bytes", c_sz),
                ("batch", c_i32), ("total_q", c_i32), ("total_k", c_i32), ("heads", c_i32), ("heads_k", c_i32),
                ("head_dim", c_i32), ("max_seqlen_q", c_i32), ("max_seqlen_k", c_i32), ("max_cols", c_i32),
                ("lg_block_m", c_i32), ("lg_block_n", c_i32), ("is_causal", c_i32), ("dtype", c_i32),
                ("max_visits_per_row", c_i32), ("fwd_mode", c_i32), ("softmax_scale", c_f32),
                ("q_row_stride", c_i64), ("q_head_stride", c_i64), ("k_row_stride", c_i64), ("k_head_stride", c_i64),
                ("v_row_stride", c_i64), ("v_head_stride", c_i64), ("o_row_stride", c_i64), ("o_head_stride", c_i64),
                ("visits_overflow", c_vp)]


class AttnBwdArgs(ctypes.Structure):
    _fields_ = [("dout", c_vp), ("q", c_vp), ("k", c_vp), ("v", c_vp), ("out", c_vp), ("softmax_lse", c_vp),
                ("dq", c_vp), ("dk", c_vp), ("dv", c_vp), ("softmax_d", c_vp),
                ("col_offsets", c_vp), ("col_nnz", c_vp), ("row_indices", c_vp),
                ("cu_seqlens_q", c_vp), ("cu_seqlens_k", c_vp),
                ("workspace", c_vp), ("workspace_bytes", c_sz), ("num_row_indices", c_i64),
                ("batch", c_i32), ("total_q", c_i32), ("total_k", c_i32), ("heads", c_i32), ("heads_k", c_i32),
                ("head_dim", c_i32), ("max_seqlen_q", c_i32), ("max_seqlen_k", c_i32), ("max_cols", c_i32),
                ("lg_block_m", c_i32), ("lg_block_n", c_i32), ("is_causal", c_i32), ("dtype", c_i32),
                ("deterministic", c_i32), ("max_visits_per_row", c_i32), ("dq_mode", c_i32), ("softmax_scale", c_f32),
                ("q_row_stride", c_i64), ("q_head_stride", c_i64), ("k_row_stride", c_i64), ("k_head_stride", c_i64),
                ("v_row_stride", c_i64), ("v_head_stride", c_i64), ("o_row_stride", c_i64), ("o_head_stride", c_i64),
                ("do_row_stride", c_i64), ("do_head_stride", c_i64),
                ("dq_row_stride", c_i64), ("dq_head_stride", c_i64), ("dk_row_stride", c_i64), ("dk_head_stride", c_i64),
                ("dv_row_stride", c_i64), ("dv_head_stride", c_i64), ("visits_overflow", c_vp)]


EXPORTS = {
    "fmoba_version": (c_i32, []),
    "fmoba_last_error": (ctypes.c_char_p, []),
    "fmoba_check_device": (c_i32, []),
    "fmoba_mean_pool": (c_i32, [ctypes.POINTER(MeanPoolArgs), c_vp]),
    "fmoba_chunk_offsets": (c_i32, [c_vp, c_vp, c_i32, c_i32, c_vp]),
    "fmoba_fused_topk_workspace_bytes": (c_sz, [c_i32, c_i32, c_i32, c_i32, c_i32, c_i32]),
    "fmoba_fused_topk": (c_i32, [ctypes.POINTER(FusedTopkArgs), c_vp]),
    "fmoba_fused_topk_static": (c_i32, [ctypes.POINTER(FusedTopkArgs), c_vp]),
    "fmoba_varlen_sort_workspace_bytes": (c_sz, [c_i64]),
    "fmoba_varlen_sort": (c_i32, [c_vp, c_vp, c_i64, c_vp, c_vp, c_i64, c_vp, c_sz, c_vp]),
    "fmoba_attn_fwd_key_block": (c_i32, [c_i32]),
    "fmoba_attn_fwd_workspace_bytes": (c_sz, [ctypes.POINTER(AttnFwdArgs)]),
    "fmoba_attn_fwd_uses_row_blocks": (c_i32, [ctypes.POINTER(AttnFwdArgs)]),
    "fmoba_csc_max_row_visits": (c_i32, [ctypes.POINTER(AttnFwdArgs), c_vp, c_vp, c_vp]),
    "fmoba_attn_fwd": (c_i32, [ctypes.POINTER(AttnFwdArgs), c_vp]),
    "fmoba_attn_fwd_phases": (c_i32, [ctypes.POINTER(AttnFwdArgs), c_i32, c_vp]),
    "fmoba_attn_bwd_workspace_bytes": (c_sz, [ctypes.POINTER(AttnBwdArgs)]),
    "fmoba_attn_bwd_uses_partials": (c_i32, [ctypes.POINTER(AttnBwdArgs)]),
    "fmoba_attn_bwd": (c_i32, [ctypes.POINTER(AttnBwdArgs), c_vp]),
    "fmoba_attn_bwd_phases": (c_i32, [ctypes.POINTER(AttnBwdArgs), c_i32, c_vp]),
}

_lib = None
_device_ok = set()


def load_library() -> ctypes.CDLL:
    """dlopen the kernel library (once) and declare every exported symbol."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python flash-moba_amd/build.py` "
                "(hipcc --offload-arch=gfx950).  There is no fallback path.")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in EXPORTS.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def _check(rc: int):
    if rc != 0:
        raise RuntimeError(load_library().fmoba_last_error().decode())


def _require(cond: bool, msg: str):
    if not cond:
        raise RuntimeError(msg)


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dt(t: torch.Tensor) -> int:
    return 1 if t.dtype == torch.bfloat16 else 0


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


@contextlib.contextmanager
def _device_guard(t: torch.Tensor):
    """Makes the tensor's device current for the call and checks once that it is a gfx950 part."""
    _require(t.is_cuda, "tensor must be on a GPU device")
    with torch.cuda.device(t.device):
        if t.device.index not in _device_ok:
            _check(load_library().fmoba_check_device())
            _device_ok.add(t.device.index)
        yield


def _check_cu(name: str, t: torch.Tensor, batch: int):
    _require(t.is_cuda, f"{name} must be on CUDA")
    _require(t.dtype == torch.int32, f"{name} must be int32")
    _require(t.is_contiguous(), f"{name} must be contiguous")
    _require(tuple(t.shape) == (batch + 1,), f"{name} must have shape (batch_size + 1)")


# --------------------------------------------------------------------------------------
# mean-pool (kernel behind flash_topk_mean_pool)
# --------------------------------------------------------------------------------------
def mean_pool(k: torch.Tensor, km: torch.Tensor, cu_seqlens_k: torch.Tensor, cu_seqlens_km: torch.Tensor,
              max_chunks: int, chunk: int) -> None:
    _require(k.dtype in (torch.float16, torch.bfloat16), "mean-pool only supports fp16 and bf16")
    _require(km.dtype == k.dtype, "k and km must have the same dtype")
    _require(k.dim() == 3 and km.dim() == 3, "k and km must be (rows, heads, head_dim)")
    _require(k.stride(-1) == 1 and km.stride(-1) == 1, "k and km must be contiguous on the last dim")
    batch = cu_seqlens_k.numel() - 1
    _check_cu("cu_seqlens_k", cu_seqlens_k, batch)
    _check_cu("cu_seqlens_km", cu_seqlens_km, batch)
    with _device_guard(k):
        a = MeanPoolArgs(k.data_ptr(), km.data_ptr(), cu_seqlens_k.data_ptr(), cu_seqlens_km.data_ptr(),
                         batch, int(max_chunks), k.shape[1], k.shape[2], int(chunk), _dt(k),
                         k.stride(0), k.stride(1), km.stride(0), km.stride(1))
        _check(load_library().fmoba_mean_pool(ctypes.byref(a), _stream()))


def chunk_offsets(cu_seqlens: torch.Tensor, chunk: int) -> torch.Tensor:
    """cu_seqlens of the pooled sequences: cumsum(ceil(len / chunk)) with a leading zero, int32, one launch
    (the tensor expressions of flash_moba/triton_mean_pool.py:132-139)."""
    batch = cu_seqlens.numel() - 1
    _require(batch > 0, "batch size must be positive")
    _check_cu("cu_seqlens", cu_seqlens, batch)
    _require(chunk > 0, "chunk size must be positive")
    with _device_guard(cu_seqlens):
        out = torch.empty_like(cu_seqlens)
        _check(load_library().fmoba_chunk_offsets(cu_seqlens.data_ptr(), out.data_ptr(), batch, int(chunk), _stream()))
    return out


# --------------------------------------------------------------------------------------
# moba_fused_topk
# --------------------------------------------------------------------------------------
def moba_fused_topk(q: torch.Tensor, km: torch.Tensor, cu_seqlens_q: torch.Tensor, cu_seqlens_k: torch.Tensor,
                    cu_seqlens_km: torch.Tensor, max_seqlen_q: int, max_seqlen_k: int, moba_topk: int,
                    moba_chunk_size: int, is_causal: bool, return_raw: bool = True,
                    return_selection: bool = False) -> List[Optional[torch.Tensor]]:
    """Returns [col_offsets, col_nnz, flat_indices, values, indices]
    (csrc/flash_topk/flash_topk_api.cpp:257).  `flat_indices` already holds each column's
    rows in ascending order.  With return_raw=False the ordered per-row lists are not
    produced and the last two entries are None.  With return_selection=True a sixth entry
    follows: the same pattern as one bit per (row, head, chunk), int32 words of shape
    (heads, ceil(max_cols / 32), total_q) -- the head of the call's workspace, which the
    row-block forward can read instead of deriving the bits from the lists."""
    dtype = q.dtype
    _require(dtype in (torch.float16, torch.bfloat16), "FlashMoBA only supports fp16 and bf16 data types")
    _require(km.dtype == dtype, "q and km must have the same dtype")
    _require(q.is_cuda, "q must be on CUDA")
    _require(km.is_cuda, "km must be on CUDA")
    _require(q.dim() == 3 and km.dim() == 3, "q and km must be (rows, heads, head_size)")
    _require(q.stride(-1) == 1, "q must be contiguous on the last dim")
    _require(km.stride(-1) == 1, "km must be contiguous on the last dim")
    batch = cu_seqlens_q.numel() - 1
    _require(batch > 0, "batch size must be positive")
    _check_cu("cu_seqlens_q", cu_seqlens_q, batch)
    _check_cu("cu_seqlens_k", cu_seqlens_k, batch)
    _check_cu("cu_seqlens_km", cu_seqlens_km, batch)
    _require(moba_topk <= 64, "moba_topk must be <= 64")
    _require(moba_topk >= 1, "moba_topk must be >= 1")
    total_q, heads, d = q.shape
    heads_k = km.shape[1]
    _require(d <= 256, "head_size must be <= 256")
    _require(d % 8 == 0, "head_size must be multiple of 8")
    _require(km.shape[2] == d, "km must have shape (total_km, num_heads_k, head_size)")
    _require(heads % heads_k == 0, "#heads in key/value must divide #heads in query")
    max_cols = (max_seqlen_k + moba_chunk_size - 1) // moba_chunk_size
    kr = (moba_topk + 15) // 16 * 16
    with _device_guard(q):
        dev = q.device
        col_offsets = torch.empty((batch, heads, max_cols), dtype=torch.int64, device=dev)
        col_nnz = torch.empty((batch, heads, max_cols), dtype=torch.int32, device=dev)
        flat = torch.empty((total_q * heads * moba_topk,), dtype=torch.int32, device=dev)
        values = indices = None
        if return_raw:
            indices = torch.empty((total_q, heads, kr), dtype=torch.int32, device=dev)
            values = torch.empty((total_q, heads, kr), dtype=torch.float32, device=dev)
        lib = load_library()
        ws_bytes = lib.fmoba_fused_topk_workspace_bytes(batch, total_q, heads, max_seqlen_q, max_seqlen_k, moba_chunk_size)
        ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=dev)
        a = FusedTopkArgs(q.data_ptr(), km.data_ptr(), cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(),
                          cu_seqlens_km.data_ptr(), col_offsets.data_ptr(), col_nnz.data_ptr(), flat.data_ptr(),
                          _ptr(indices), _ptr(values), ws.data_ptr(), ws_bytes,
                          batch, total_q, heads, heads_k, d, int(max_seqlen_q), int(max_seqlen_k),
                          int(moba_topk), int(moba_chunk_size), int(bool(is_causal)), _dt(q),
                          q.stride(0), q.stride(1), km.stride(0), km.stride(1))
        _check(lib.fmoba_fused_topk(ctypes.byref(a), _stream()))
        res = [col_offsets, col_nnz, flat, values, indices]
        if return_selection:
            # the selection bits sit at the first 256-byte boundary of the workspace: (heads, ceil(max_cols/32), total_q) words
            words = (max_cols + 31) // 32
            off = (-ws.data_ptr()) % 256
            nbytes = heads * words * total_q * 4
            if max_cols == 0 or max_seqlen_k == 0 or ws_bytes < off + nbytes:  # (no keys: nothing was written)
                res.append(torch.zeros((heads, words, total_q), dtype=torch.int32, device=dev))
            else:
                res.append(ws[off:off + nbytes].view(torch.int32).view(heads, words, total_q))
    return res


# --------------------------------------------------------------------------------------
# varlen_sort
# --------------------------------------------------------------------------------------
def varlen_sort(cu_seq_starts: torch.Tensor, cu_seq_ends: torch.Tensor, src: torch.Tensor) -> torch.Tensor:
    _require(cu_seq_starts.dtype == torch.int64, "only support int64 cu_seq_starts data type")
    _require(cu_seq_ends.dtype == torch.int64, "only support int64 cu_seq_ends data type")
    _require(src.dtype == torch.int32, "only support int32 src data type")
    _require(cu_seq_starts.is_cuda, "cu_seq_starts must be on CUDA")
    _require(cu_seq_ends.is_cuda, "cu_seq_ends must be on CUDA")
    _require(src.is_cuda, "src must be on CUDA")
    _require(cu_seq_starts.dim() == 1 and cu_seq_ends.dim() == 1, "cu_seq_starts / cu_seq_lens must be 1-D")
    _require(cu_seq_starts.numel() == cu_seq_ends.numel(), "seq_starts and seq_lens must have the same length")
    _require(cu_seq_starts.is_contiguous(), "cu_seq_starts must be contiguous")
    _require(cu_seq_ends.is_contiguous(), "cu_seq_ends must be contiguous")
    _require(src.is_contiguous(), "src must be contiguous")
    with _device_guard(src):
        dst = torch.empty_like(src)
        total = src.numel()
        if total:
            lib = load_library()
            ws_bytes = lib.fmoba_varlen_sort_workspace_bytes(total)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=src.device)
            _check(lib.fmoba_varlen_sort(cu_seq_starts.data_ptr(), cu_seq_ends.data_ptr(), cu_seq_starts.numel(),
                                         src.data_ptr(), dst.data_ptr(), total, ws.data_ptr(), ws_bytes, _stream()))
        return dst


# --------------------------------------------------------------------------------------
# moba_varlen_fwd
# --------------------------------------------------------------------------------------
def _check_csc(col_offsets, col_nnz, row_indices, batch, heads):
    _require(col_offsets.dtype == torch.int64, "moba_col_offsets must have dtype int64 (index_t)")
    _require(col_nnz.dtype == torch.int32, "moba_col_nnz must have dtype int32")
    _require(row_indices.dtype == torch.int32, "moba_row_indices must have dtype int32")
    for name, t in (("moba_col_offsets", col_offsets), ("moba_col_nnz", col_nnz), ("moba_row_indices", row_indices)):
        _require(t.is_cuda, f"{name} must be on CUDA")
        _require(t.is_contiguous(), f"{name} must be contiguous")
    _require(col_offsets.dim() == 3, "moba_col_offsets must have shape (batch_size, num_heads, max_lg_col_num)")
    max_cols = col_offsets.shape[2]
    _require(tuple(col_offsets.shape) == (batch, heads, max_cols), "moba_col_offsets must have shape (batch_size, num_heads, max_lg_col_num)")
    _require(tuple(col_nnz.shape) == (batch, heads, max_cols), "moba_col_nnz must have shape (batch_size, num_heads, max_lg_col_num)")
    return max_cols


def _reject_unsupported(p_dropout, softcap, alibi_slopes, seqused_k=None, leftpad_k=None, return_softmax=False):
    _require(p_dropout < 1.0, "p_dropout must be < 1")
    _require(p_dropout == 0.0, "attention dropout is not supported by FlashMoBA (dropout_p must be 0.0)")
    _require(not (softcap > 0.0), "softcap is not supported by FlashMoBA (softcap must be 0.0)")
    _require(alibi_slopes is None, "ALiBi is not supported by FlashMoBA (alibi_slopes must be None)")
    _require(seqused_k is None, "seqused_k is not supported")
    _require(leftpad_k is None, "leftpad_k is not supported")
    _require(not return_softmax, "return_softmax is only supported when p_dropout > 0.0, which FlashMoBA does not support")


# What the last forward / backward call of this thread ran.  Read-only diagnostics for tests and benchmarks: nothing
# in here influences a later call (bounds and selection bits are explicit arguments).
_last = threading.local()


def last_fwd_visits():
    """The visits bound the last forward call of this thread used, in forward key blocks."""
    return getattr(_last, "fwd_visits", None)


def last_fwd_row_blocks():
    """1 if the last forward of this thread ran the row-block form, 0 for the column form."""
    return int(getattr(_last, "fwd_row_blocks", 0))


def last_bwd_partials():
    """1 if the last backward of this thread formed dQ from per-visit partials, 0 for the row-block form."""
    return int(getattr(_last, "bwd_partials", 0))


def fwd_key_block(n_lg_block_dim: int) -> int:
    """Keys per forward visit (fmoba_attn_fwd_key_block): 128 for columns of a multiple of 128 keys, else 64."""
    return 128 if int(n_lg_block_dim) % 128 == 0 else 64


def _count_visits(lib, q, moba_col_offsets, moba_col_nnz, moba_row_indices, cu_seqlens_q, cu_seqlens_k, batch, total_q, total_k,
                  heads, heads_k, d, max_seqlen_q, max_seqlen_k, max_cols, m_lg_block_dim, n_lg_block_dim):
    """Largest number of (row, forward key block) visits of any (row, head) of the pattern: one pass + one read."""
    if total_q == 0 or total_k == 0 or max_cols == 0:
        return 1
    counts = torch.empty((total_q * heads + 1,), dtype=torch.int32, device=q.device)
    a0 = AttnFwdArgs(None, None, None, None, None,
                     moba_col_offsets.data_ptr(), moba_col_nnz.data_ptr(), moba_row_indices.data_ptr(),
                     cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), None, None, 0,
                     batch, total_q, total_k, heads, heads_k, d, int(max_seqlen_q), int(max_seqlen_k), max_cols,
                     int(m_lg_block_dim), int(n_lg_block_dim), 0, _dt(q), 0, 0, 1.0, 0, 0, 0, 0, 0, 0, 0, 0, None)
    _check(lib.fmoba_csc_max_row_visits(ctypes.byref(a0), counts.data_ptr(), counts[total_q * heads:].data_ptr(), _stream()))
    return max(1, int(counts[total_q * heads].item()))


def count_max_visits(q, moba_col_offsets, moba_col_nnz, moba_row_indices, cu_seqlens_q, cu_seqlens_k, total_k, heads_k,
                     max_seqlen_q, max_seqlen_k, n_lg_block_dim) -> int:
    """Largest number of (row, forward key block) visits of any (row, head) of a CSC pattern: the bound the attention
    entry points need for a pattern that does not come from the gating.  One pass over the lists + one device-to-host
    read."""
    _require(q.is_cuda and q.dim() == 3, "q must be a (total_q, heads, head_size) tensor on CUDA")
    batch = cu_seqlens_q.numel() - 1
    _require(batch > 0, "batch size must be positive")
    _check_cu("cu_seqlens_q", cu_seqlens_q, batch)
    _check_cu("cu_seqlens_k", cu_seqlens_k, batch)
    total_q, heads, d = q.shape
    _check_csc(moba_col_offsets, moba_col_nnz, moba_row_indices, batch, heads)
    _require(n_lg_block_dim % 64 == 0 and n_lg_block_dim > 0, "n_lg_block_dim must be a multiple of 64")
    with _device_guard(q):
        return _count_visits(load_library(), q, moba_col_offsets, moba_col_nnz, moba_row_indices, cu_seqlens_q, cu_seqlens_k,
                             batch, total_q, int(total_k), heads, heads_k, d, max_seqlen_q, max_seqlen_k,
                             moba_col_offsets.shape[2], 128, n_lg_block_dim)


def moba_varlen_fwd(q, k, v, out_, moba_col_offsets, moba_col_nnz, moba_row_indices, cu_seqlens_q, cu_seqlens_k,
                    seqused_k, leftpad_k, alibi_slopes, max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale,
                    zero_tensors, is_causal, softcap, return_softmax, m_lg_block_dim, n_lg_block_dim, gen=None, _phases=None,
                    _fwd_mode=0, _max_visits=None, _selection=None, _overflow=None):
    """Returns [out, softmax_lse (H, total_q) fp32, p (empty), rng_state (2,) int64].

    Beyond the reference's arguments: _max_visits, a bound on the (row, forward key block) visits of any (row, head)
    -- a gated pattern has top-k * lg_block_n / fwd_key_block(lg_block_n); None or a value below 1 makes the call count
    them from the pattern (one device-to-host read) -- and _selection, the int32 selection words of the gating call that
    produced exactly this pattern (moba_fused_topk(return_selection=True)); _overflow, a zeroed int32 tensor of one
    element that a form with per-visit partial results raises to the visit count of a row that exceeds the bound."""
    dtype = q.dtype
    _require(dtype in (torch.float16, torch.bfloat16), "FlashMoBA only support fp16 and bf16 data type")
    _require(k.dtype == dtype, "query and key must have the same dtype")
    _require(v.dtype == dtype, "query and value must have the same dtype")
    for name, t in (("q", q), ("k", k), ("v", v)):
        _require(t.is_cuda, f"{name} must be on CUDA")
        _require(t.dim() == 3, f"{name} must be (total, heads, head_size)")
        _require(t.stride(-1) == 1, "Input tensor must have contiguous last dimension")
    batch = cu_seqlens_q.numel() - 1
    _require(batch > 0, "batch size must be positive")
    _check_cu("cu_seqlens_q", cu_seqlens_q, batch)
    _check_cu("cu_seqlens_k", cu_seqlens_k, batch)
    total_q, heads, d = q.shape
    total_k, heads_k = k.shape[0], k.shape[1]
    max_cols = _check_csc(moba_col_offsets, moba_col_nnz, moba_row_indices, batch, heads)
    _reject_unsupported(p_dropout, softcap, alibi_slopes, seqused_k, leftpad_k, return_softmax)
    if max_seqlen_q == 1:
        is_causal = False  # flash_moba_api.cpp:450
    _require(d <= 256, "FlashMoBA forward only supports head dimension at most 256")
    _require(d % 8 == 0, "query, key, value, and out_ must have a head_size that is a multiple of 8")
    _require(heads % heads_k == 0, "Number of heads in key/value must divide number of heads in query")
    _require(128 <= m_lg_block_dim <= 1024, "m_lg_block_dim must be at least 128 and at most 1024")
    _require(m_lg_block_dim % 64 == 0, "m_lg_block_dim must be a multiple of 64")
    _require(n_lg_block_dim % 64 == 0 and n_lg_block_dim > 0, "n_lg_block_dim must be a multiple of 64")
    _require(tuple(k.shape) == (total_k, heads_k, d), "k must have shape (total_k, num_heads_k, head_size)")
    _require(tuple(v.shape) == (total_k, heads_k, d), "v must have shape (total_k, num_heads_k, head_size)")
    with _device_guard(q):
        if out_ is not None:
            out = out_
            _require(out.dtype == dtype, "Output must have the same dtype as inputs")
            _require(out.is_cuda, "out must be on CUDA")
            _require(out.stride(-1) == 1, "Output tensor must have contiguous last dimension")
            _require(tuple(out.shape) == (total_q, heads, d), "out must have shape (total_q, num_heads, head_size)")
        else:
            out = torch.empty_like(q)
        lse = torch.empty((heads, total_q), dtype=torch.float32, device=q.device)
        p = torch.empty((0,), dtype=dtype, device=q.device)
        rng_state = torch.zeros((2,), dtype=torch.int64, device=q.device)
        lib = load_library()
        sel_ptr = None
        if _selection is not None and max_cols > 0 and total_q > 0:
            _require(_selection.dtype == torch.int32 and _selection.is_cuda and _selection.device == q.device and _selection.is_contiguous()
                     and tuple(_selection.shape) == (heads, (max_cols + 31) // 32, total_q),
                     "selection bits must be a contiguous int32 tensor of shape (num_heads, ceil(max_lg_col_num / 32), total_q) on q's device")
            sel_ptr = _selection.data_ptr()

        def args(ws_ptr, ws_bytes, visits):
            return AttnFwdArgs(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
                               moba_col_offsets.data_ptr(), moba_col_nnz.data_ptr(), moba_row_indices.data_ptr(),
                               cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), sel_ptr, ws_ptr, ws_bytes,
                               batch, total_q, total_k, heads, heads_k, d, int(max_seqlen_q), int(max_seqlen_k), max_cols,
                               int(m_lg_block_dim), int(n_lg_block_dim), int(bool(is_causal)), _dt(q), visits,
                               int(_fwd_mode), float(softmax_scale),
                               q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1),
                               out.stride(0), out.stride(1), _ptr(_overflow))

        visits = _max_visits
        if visits is None or int(visits) < 1:
            visits = _count_visits(lib, q, moba_col_offsets, moba_col_nnz, moba_row_indices, cu_seqlens_q, cu_seqlens_k, batch,
                                   total_q, total_k, heads, heads_k, d, max_seqlen_q, max_seqlen_k, max_cols,
                                   m_lg_block_dim, n_lg_block_dim)
        visits = max(1, int(visits))
        _last.fwd_visits = visits
        a = args(None, 0, visits)
        ws_bytes = lib.fmoba_attn_fwd_workspace_bytes(ctypes.byref(a))
        _last.fwd_row_blocks = int(lib.fmoba_attn_fwd_uses_row_blocks(ctypes.byref(a)))
        ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=q.device)
        a = args(ws.data_ptr(), ws_bytes, visits)
        if _phases is None:
            _check(lib.fmoba_attn_fwd(ctypes.byref(a), _stream()))
        else:  # measurement hook: callable(run) receives run(mask) launching the chosen phases
            _phases(lambda mask: _check(lib.fmoba_attn_fwd_phases(ctypes.byref(a), mask, _stream())))
    return [out, lse, p, rng_state]


# --------------------------------------------------------------------------------------
# moba_varlen_bwd
# --------------------------------------------------------------------------------------
def moba_varlen_bwd(dout, q, k, v, out, softmax_lse, dq_, dk_, dv_, moba_col_offsets, moba_col_nnz, moba_row_indices,
                    cu_seqlens_q, cu_seqlens_k, alibi_slopes, max_seqlen_q, max_seqlen_k, p_dropout, softmax_scale,
                    zero_tensors, is_causal, softcap, deterministic, m_lg_block_dim, n_lg_block_dim, gen=None,
                    rng_state=None, _phases=None, _dq_mode=0, _max_visits=None, _overflow=None):
    """Returns [dq, dk, dv, softmax_d (H, total_q + 128*batch) fp32].

    Beyond the reference's arguments: _max_visits, a bound on the visits of any (row, head) in 64-KEY blocks (a gated
    pattern has top-k * lg_block_n / 64); None or a value below 1 makes the call count them from the pattern (one
    device-to-host read)."""
    dtype = q.dtype
    _require(dtype in (torch.float16, torch.bfloat16), "FlashMoBA only support fp16 and bf16 data type")
    _require(k.dtype == dtype, "query and key must have the same dtype")
    _require(v.dtype == dtype, "query and value must have the same dtype")
    _require(out.dtype == dtype, "query and out must have the same dtype")
    _require(dout.dtype == dtype, "query and dout must have the same dtype")
    for name, t in (("q", q), ("k", k), ("v", v), ("out", out), ("dout", dout)):
        _require(t.is_cuda, f"{name} must be on CUDA")
        _require(t.dim() == 3, f"{name} must be (total, heads, head_size)")
    _require(softmax_lse.is_cuda, "softmax_lse must be on CUDA")
    _require(q.stride(-1) == 1 and k.stride(-1) == 1 and v.stride(-1) == 1, "Input tensor must have contiguous last dimension")
    _require(out.stride(-1) == 1, "out tensor must have contiguous last dimension")
    _require(dout.stride(-1) == 1, "dout tensor must have contiguous last dimension")
    batch = cu_seqlens_q.numel() - 1
    _require(batch > 0, "batch size must be positive")
    _check_cu("cu_seqlens_q", cu_seqlens_q, batch)
    _check_cu("cu_seqlens_k", cu_seqlens_k, batch)
    total_q, heads, d = q.shape
    total_k, heads_k = k.shape[0], k.shape[1]
    max_cols = _check_csc(moba_col_offsets, moba_col_nnz, moba_row_indices, batch, heads)
    _reject_unsupported(p_dropout, softcap, alibi_slopes)
    if max_seqlen_q == 1:
        is_causal = False  # keep forward and backward masks identical (flash_moba_api.cpp:450)
    _require(d % 8 == 0, "head_size should be a multiple of 8")
    _require(d <= 256, "FlashMoBA backward only supports head dimension at most 256")
    _require(heads % heads_k == 0, "Number of heads in key/value must divide number of heads in query")
    _require(m_lg_block_dim % 64 == 0, "m_lg_block_dim must be a multiple of 64")
    _require(n_lg_block_dim % 64 == 0 and n_lg_block_dim > 0, "n_lg_block_dim must be a multiple of 64")
    _require(tuple(k.shape) == (total_k, heads_k, d) and tuple(v.shape) == (total_k, heads_k, d), "k, v must have shape (total_k, num_heads_k, head_size)")
    _require(tuple(out.shape) == (total_q, heads, d) and tuple(dout.shape) == (total_q, heads, d), "out, dout must have shape (total_q, num_heads, head_size)")
    _require(softmax_lse.dtype == torch.float32 and tuple(softmax_lse.shape) == (heads, total_q) and softmax_lse.is_contiguous(),
             "softmax_lse must be a contiguous fp32 tensor of shape (num_heads, total_q)")

    def _grad(t, like, name, shape):
        if t is None:
            return torch.empty_like(like)
        _require(t.dtype == dtype, f"{name} must have the same dtype as q")
        _require(t.is_cuda, f"{name} must be on CUDA")
        _require(t.stride(-1) == 1, f"{name} must have contiguous last dimension")
        _require(tuple(t.shape) == shape, f"{name} has the wrong shape")
        return t

    with _device_guard(q):
        dq = _grad(dq_, q, "dq", (total_q, heads, d))
        dk = _grad(dk_, k, "dk", (total_k, heads_k, d))
        dv = _grad(dv_, v, "dv", (total_k, heads_k, d))
        dev = q.device
        softmax_d = torch.empty((heads, total_q + 128 * batch), dtype=torch.float32, device=dev)
        if heads_k != heads:  # MQA / GQA: per-query-head gradients, summed below (flash_moba_api.cpp:764-771,842-845)
            dk_e = torch.empty((total_k, heads, d), dtype=dtype, device=dev)
            dv_e = torch.empty((total_k, heads, d), dtype=dtype, device=dev)
        else:
            dk_e, dv_e = dk, dv
        lib = load_library()
        visits = _max_visits
        if visits is None or int(visits) < 1:
            kb = fwd_key_block(n_lg_block_dim)
            visits = (kb // 64) * _count_visits(lib, q, moba_col_offsets, moba_col_nnz, moba_row_indices, cu_seqlens_q,
                                                cu_seqlens_k, batch, total_q, total_k, heads, heads_k, d, max_seqlen_q,
                                                max_seqlen_k, max_cols, 128, n_lg_block_dim)
        visits = max(1, int(visits))
        a = AttnBwdArgs(dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), softmax_lse.data_ptr(),
                        dq.data_ptr(), dk_e.data_ptr(), dv_e.data_ptr(), softmax_d.data_ptr(),
                        moba_col_offsets.data_ptr(), moba_col_nnz.data_ptr(), moba_row_indices.data_ptr(),
                        cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), None, 0, int(moba_row_indices.numel()),
                        batch, total_q, total_k, heads, heads_k, d, int(max_seqlen_q), int(max_seqlen_k), max_cols,
                        int(m_lg_block_dim), int(n_lg_block_dim), int(bool(is_causal)), _dt(q), int(bool(deterministic)),
                        visits, int(_dq_mode), float(softmax_scale),
                        q.stride(0), q.stride(1), k.stride(0), k.stride(1), v.stride(0), v.stride(1),
                        out.stride(0), out.stride(1), dout.stride(0), dout.stride(1),
                        dq.stride(0), dq.stride(1), dk_e.stride(0), dk_e.stride(1), dv_e.stride(0), dv_e.stride(1), _ptr(_overflow))
        ws_bytes = lib.fmoba_attn_bwd_workspace_bytes(ctypes.byref(a))
        _last.bwd_partials = int(lib.fmoba_attn_bwd_uses_partials(ctypes.byref(a)))
        ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=dev)
        a.workspace, a.workspace_bytes = ws.data_ptr(), ws_bytes
        if _phases is None:
            _check(lib.fmoba_attn_bwd(ctypes.byref(a), _stream()))
        else:  # measurement hook: callable(run) receives run(mask) launching the chosen phases
            _phases(lambda mask: _check(lib.fmoba_attn_bwd_phases(ctypes.byref(a), mask, _stream())))
        if heads_k != heads:
            grp = heads // heads_k
            torch.sum(dk_e.view(total_k, heads_k, grp, d), dim=2, out=dk)
            torch.sum(dv_e.view(total_k, heads_k, grp, d), dim=2, out=dv)
    return [dq, dk, dv, softmax_d]

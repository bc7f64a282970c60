"""Public Python API of FlashMoBA on MI355X.

Drop-in for flash_moba/flash_moba_interface.py of the reference: the three public functions
(flash_topk_varlen_func :517, flash_moba_attn_varlen_func :578, flash_moba_varlen_func :688),
the four ``flash_moba::`` custom ops with their fake-shape functions (:83-396) and the
autograd function (:400-513) keep their names, argument order, defaults and the meaning of
col_offsets / col_nnz / indices.  The compiled module behind them is
``flash_moba.flash_moba_hip`` (ctypes over the C ABI of libflash_moba_hip.so) instead of
``flash_moba_cuda``.

Differences a caller can observe, all within the reference's contract:
  * the row lists returned by ``_moba_fused_topk`` are already ascending (the reference
    returns them in nondeterministic order and sorts afterwards); ``flash_topk_varlen_func``
    therefore does not need the extra sort pass, ``_varlen_sort`` stays available;
  * dropout, softcap, ALiBi, seqused_k and leftpad_k raise an error instead of being
    silently unsupported (the reference's README lists them as unsupported).
"""
from typing import Optional, Tuple

import torch

from flash_moba import flash_moba_hip as flash_moba_gpu
from flash_moba.mean_pool import flash_topk_mean_pool, mean_pool_nosync  # noqa: F401


def round_multiple(x: int, m: int) -> int:
    return (x + m - 1) // m * m


def decide_lg_block_m(top_k: int, chunk_size: int, seqlen: int, causal: bool = False) -> int:
    """Query-block heuristic of the reference (flash_moba_interface.py:20-48), kept because
    lg_block_m is an API argument.  The HIP forward kernel always works on 128-row
    superblocks held in LDS and accepts any valid value.  The reference's cap for sm86/sm89
    parts has no counterpart on gfx950."""
    budget = top_k * chunk_size
    density = (2 * budget * seqlen - budget ** 2) / (seqlen ** 2) if causal else budget / seqlen
    sparsity = 1 - density
    for bound, lg in ((0.5, 128), (0.7, 256), (0.8, 512), (0.9, 768)):
        if sparsity <= bound:
            return lg
    return 1024


def maybe_contiguous(x):
    return x.contiguous() if x is not None and x.stride(-1) != 1 else x


def _pad8(*ts):
    """Pad the head dimension to a multiple of 8 (flash_moba_interface.py:431-435,550-553)."""
    d = ts[0].size(-1)
    if d % 8 == 0:
        return ts
    return tuple(torch.nn.functional.pad(t, [0, 8 - d % 8]) for t in ts)


# --------------------------------------------------------------------------------------
# custom ops (names, schemas and fake-shape functions as in the reference)
# --------------------------------------------------------------------------------------
@torch.library.custom_op("flash_moba::_moba_fused_topk", mutates_args=(), device_types="cuda")
def _moba_fused_topk(
    q: torch.Tensor,
    km: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    cu_seqlens_km: torch.Tensor,
    max_seqlen_q: int,
    max_seqlen_k: int,
    moba_topk: int,
    moba_chunk_size: int,
    causal: bool = True,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    q, km = maybe_contiguous(q), maybe_contiguous(km)
    col_offsets, col_nnz, indices, _, _ = flash_moba_gpu.moba_fused_topk(
        q, km, cu_seqlens_q, cu_seqlens_k, cu_seqlens_km, max_seqlen_q, max_seqlen_k,
        moba_topk, moba_chunk_size, causal, return_raw=False)
    return col_offsets, col_nnz, indices


@torch.library.register_fake("flash_moba::_moba_fused_topk")
def _moba_fused_topk_fake(q, km, cu_seqlens_q, cu_seqlens_k, cu_seqlens_km, max_seqlen_q, max_seqlen_k,
                          moba_topk, moba_chunk_size, causal=True):
    batch = cu_seqlens_q.numel() - 1
    total_q, heads, _ = q.shape
    cols = (max_seqlen_k + moba_chunk_size - 1) // moba_chunk_size
    return (torch.empty((batch, heads, cols), device=q.device, dtype=torch.int64),
            torch.empty((batch, heads, cols), device=q.device, dtype=torch.int32),
            torch.empty((total_q * heads * moba_topk,), device=q.device, dtype=torch.int32))


@torch.library.custom_op("flash_moba::_varlen_sort", mutates_args=(), device_types="cuda")
def _varlen_sort(col_offsets: torch.Tensor, col_nnz: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    starts = col_offsets.reshape(-1)
    return flash_moba_gpu.varlen_sort(starts, starts + col_nnz.reshape(-1), indices)


@torch.library.register_fake("flash_moba::_varlen_sort")
def _varlen_sort_fake(col_offsets, col_nnz, indices):
    return torch.empty_like(indices)


@torch.library.custom_op("flash_moba::_flash_moba_attn_varlen_forward", mutates_args=(), device_types="cuda")
def _flash_moba_attn_varlen_forward(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    max_seqlen_q: int,
    max_seqlen_k: int,
    moba_col_offsets: torch.Tensor,
    moba_col_nnz: torch.Tensor,
    moba_row_indices: torch.Tensor,
    lg_block_m: int,
    lg_block_n: int,
    dropout_p: float,
    softmax_scale: float,
    causal: bool,
    softcap: float = 0.0,
    alibi_slopes: Optional[torch.Tensor] = None,
    return_softmax: bool = False,
    leftpad_k: Optional[torch.Tensor] = None,
    seqused_k: Optional[torch.Tensor] = None,
    zero_tensors: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    q, k, v = (maybe_contiguous(x) for x in (q, k, v))
    csc = [maybe_contiguous(x) for x in (moba_col_offsets, moba_col_nnz, moba_row_indices)]
    out, softmax_lse, S_dmask, rng_state = flash_moba_gpu.moba_varlen_fwd(
        q, k, v, None, csc[0], csc[1], csc[2], cu_seqlens_q, cu_seqlens_k, seqused_k, leftpad_k, alibi_slopes,
        max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale, zero_tensors, causal, softcap, return_softmax,
        lg_block_m, lg_block_n, None)
    return out, softmax_lse, S_dmask, rng_state


@torch.library.register_fake("flash_moba::_flash_moba_attn_varlen_forward")
def _flash_moba_attn_varlen_forward_fake(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                                         moba_col_offsets, moba_col_nnz, moba_row_indices, lg_block_m, lg_block_n,
                                         dropout_p, softmax_scale, causal, softcap=0.0, alibi_slopes=None,
                                         return_softmax=False, leftpad_k=None, seqused_k=None, zero_tensors=False):
    batch = cu_seqlens_q.numel() - 1
    total_q, heads, _ = q.shape
    out = torch.empty_like(maybe_contiguous(q))
    lse = torch.empty((heads, total_q), dtype=torch.float32, device=q.device)
    if return_softmax:
        p = torch.empty((batch, heads, round_multiple(max_seqlen_q, 128), round_multiple(max_seqlen_k, 128)),
                        dtype=q.dtype, device=q.device)
    else:
        p = torch.empty((0,), dtype=q.dtype, device=q.device)
    return out, lse, p, torch.empty((2,), dtype=torch.int64, device=q.device)


@torch.library.custom_op("flash_moba::_flash_moba_attn_varlen_backward", mutates_args=("dq", "dk", "dv"), device_types="cuda")
def _flash_moba_attn_varlen_backward(
    dout: torch.Tensor,
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    out: torch.Tensor,
    softmax_lse: torch.Tensor,
    dq: Optional[torch.Tensor],
    dk: Optional[torch.Tensor],
    dv: Optional[torch.Tensor],
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    max_seqlen_q: int,
    max_seqlen_k: int,
    moba_col_offsets: torch.Tensor,
    moba_col_nnz: torch.Tensor,
    moba_row_indices: torch.Tensor,
    lg_block_m: int,
    lg_block_n: int,
    dropout_p: float,
    softmax_scale: float,
    causal: bool,
    softcap: float,
    alibi_slopes: Optional[torch.Tensor],
    deterministic: bool,
    rng_state: Optional[torch.Tensor] = None,
    zero_tensors: bool = False,
) -> torch.Tensor:
    dout, q, k, v, out = (maybe_contiguous(x) for x in (dout, q, k, v, out))
    _, _, _, softmax_d = flash_moba_gpu.moba_varlen_bwd(
        dout, q, k, v, out, softmax_lse, dq, dk, dv, moba_col_offsets, moba_col_nnz, moba_row_indices,
        cu_seqlens_q, cu_seqlens_k, alibi_slopes, max_seqlen_q, max_seqlen_k, dropout_p, softmax_scale,
        zero_tensors, causal, softcap, deterministic, lg_block_m, lg_block_n, None, rng_state)
    return softmax_d


@torch.library.register_fake("flash_moba::_flash_moba_attn_varlen_backward")
def _flash_moba_attn_varlen_backward_fake(dout, q, k, v, out, softmax_lse, dq, dk, dv, cu_seqlens_q, cu_seqlens_k,
                                          max_seqlen_q, max_seqlen_k, moba_col_offsets, moba_col_nnz, moba_row_indices,
                                          lg_block_m, lg_block_n, dropout_p, softmax_scale, causal, softcap,
                                          alibi_slopes, deterministic, rng_state=None, zero_tensors=False):
    batch = cu_seqlens_q.numel() - 1
    total_q, heads, _ = q.shape
    return torch.empty((heads, total_q + 128 * batch), device=q.device, dtype=torch.float32)


# --------------------------------------------------------------------------------------
# private ops of the fused path.  The reference's four ops above keep their schemas; these carry, as ordinary
# arguments, what the MI355X kernels need beyond them -- the bound on a row's (row, key block) visits, which sizes
# the partial-result workspace and selects the kernel form, and the gating's selection bits -- so that a traced or
# compiled graph carries them too (the reference has no counterpart: its row-wise scratch needs no bound).
# --------------------------------------------------------------------------------------
@torch.library.custom_op("flash_moba::_mean_pool", mutates_args=(), device_types="cuda")
def _mean_pool(k: torch.Tensor, cu_seqlens_k: torch.Tensor, max_seqlen_k: int, chunk: int) -> Tuple[torch.Tensor, torch.Tensor]:
    km, cu_km, _ = mean_pool_nosync(k, cu_seqlens_k, max_seqlen_k, chunk)
    return km, cu_km


@torch.library.register_fake("flash_moba::_mean_pool")
def _mean_pool_fake(k, cu_seqlens_k, max_seqlen_k, chunk):
    batch = cu_seqlens_k.numel() - 1
    return (torch.empty((k.shape[0] // chunk + batch, k.shape[1], k.shape[2]), dtype=k.dtype, device=k.device),
            torch.empty(cu_seqlens_k.shape, dtype=torch.int32, device=k.device))


@torch.library.custom_op("flash_moba::_gated_topk", mutates_args=(), device_types="cuda")
def _gated_topk(
    q: torch.Tensor,
    km: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    cu_seqlens_km: torch.Tensor,
    max_seqlen_q: int,
    max_seqlen_k: int,
    moba_topk: int,
    moba_chunk_size: int,
    causal: bool,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """_moba_fused_topk plus the selection as one bit per (row, head, chunk): int32 (heads, ceil(cols/32), total_q)."""
    q, km = maybe_contiguous(q), maybe_contiguous(km)
    col_offsets, col_nnz, indices, _, _, selection = flash_moba_gpu.moba_fused_topk(
        q, km, cu_seqlens_q, cu_seqlens_k, cu_seqlens_km, max_seqlen_q, max_seqlen_k,
        moba_topk, moba_chunk_size, causal, return_raw=False, return_selection=True)
    return col_offsets, col_nnz, indices, selection


@torch.library.register_fake("flash_moba::_gated_topk")
def _gated_topk_fake(q, km, cu_seqlens_q, cu_seqlens_k, cu_seqlens_km, max_seqlen_q, max_seqlen_k,
                     moba_topk, moba_chunk_size, causal):
    co, cn, ind = _moba_fused_topk_fake(q, km, cu_seqlens_q, cu_seqlens_k, cu_seqlens_km, max_seqlen_q, max_seqlen_k,
                                        moba_topk, moba_chunk_size, causal)
    total_q, heads, _ = q.shape
    return co, cn, ind, torch.empty((heads, (co.shape[2] + 31) // 32, total_q), device=q.device, dtype=torch.int32)


@torch.library.custom_op("flash_moba::_attn_varlen_forward_bounded", mutates_args=(), device_types="cuda")
def _attn_varlen_forward_bounded(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    max_seqlen_q: int,
    max_seqlen_k: int,
    moba_col_offsets: torch.Tensor,
    moba_col_nnz: torch.Tensor,
    moba_row_indices: torch.Tensor,
    lg_block_m: int,
    lg_block_n: int,
    softmax_scale: float,
    causal: bool,
    max_visits: int,
    selection_bits: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """_flash_moba_attn_varlen_forward with the visits bound (in forward key blocks; below 1 = count them from the
    pattern) and, optionally, the gating's selection bits as arguments."""
    q, k, v = (maybe_contiguous(x) for x in (q, k, v))
    csc = [maybe_contiguous(x) for x in (moba_col_offsets, moba_col_nnz, moba_row_indices)]
    out, softmax_lse, S_dmask, rng_state = flash_moba_gpu.moba_varlen_fwd(
        q, k, v, None, csc[0], csc[1], csc[2], cu_seqlens_q, cu_seqlens_k, None, None, None,
        max_seqlen_q, max_seqlen_k, 0.0, softmax_scale, False, causal, 0.0, False,
        lg_block_m, lg_block_n, None, _max_visits=max_visits, _selection=selection_bits)
    return out, softmax_lse, S_dmask, rng_state


@torch.library.register_fake("flash_moba::_attn_varlen_forward_bounded")
def _attn_varlen_forward_bounded_fake(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                                      moba_col_offsets, moba_col_nnz, moba_row_indices, lg_block_m, lg_block_n,
                                      softmax_scale, causal, max_visits, selection_bits=None):
    return _flash_moba_attn_varlen_forward_fake(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                                                moba_col_offsets, moba_col_nnz, moba_row_indices, lg_block_m, lg_block_n,
                                                0.0, softmax_scale, causal)


@torch.library.custom_op("flash_moba::_attn_varlen_backward_bounded", mutates_args=("dq", "dk", "dv"), device_types="cuda")
def _attn_varlen_backward_bounded(
    dout: torch.Tensor,
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    out: torch.Tensor,
    softmax_lse: torch.Tensor,
    dq: torch.Tensor,
    dk: torch.Tensor,
    dv: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    max_seqlen_q: int,
    max_seqlen_k: int,
    moba_col_offsets: torch.Tensor,
    moba_col_nnz: torch.Tensor,
    moba_row_indices: torch.Tensor,
    lg_block_m: int,
    lg_block_n: int,
    softmax_scale: float,
    causal: bool,
    deterministic: bool,
    max_visits: int,
) -> torch.Tensor:
    """_flash_moba_attn_varlen_backward with the visits bound (in 64-key blocks; below 1 = count them) as an argument."""
    dout, q, k, v, out = (maybe_contiguous(x) for x in (dout, q, k, v, out))
    _, _, _, softmax_d = flash_moba_gpu.moba_varlen_bwd(
        dout, q, k, v, out, softmax_lse, dq, dk, dv, moba_col_offsets, moba_col_nnz, moba_row_indices,
        cu_seqlens_q, cu_seqlens_k, None, max_seqlen_q, max_seqlen_k, 0.0, softmax_scale,
        False, causal, 0.0, deterministic, lg_block_m, lg_block_n, None, None, _max_visits=max_visits)
    return softmax_d


@torch.library.register_fake("flash_moba::_attn_varlen_backward_bounded")
def _attn_varlen_backward_bounded_fake(dout, q, k, v, out, softmax_lse, dq, dk, dv, cu_seqlens_q, cu_seqlens_k,
                                       max_seqlen_q, max_seqlen_k, moba_col_offsets, moba_col_nnz, moba_row_indices,
                                       lg_block_m, lg_block_n, softmax_scale, causal, deterministic, max_visits):
    batch = cu_seqlens_q.numel() - 1
    total_q, heads, _ = q.shape
    return torch.empty((heads, total_q + 128 * batch), device=q.device, dtype=torch.float32)


_wrapped_moba_fused_topk = torch.ops.flash_moba._moba_fused_topk
_wrapped_varlen_sort = torch.ops.flash_moba._varlen_sort
_wrapped_flash_moba_attn_varlen_forward = torch.ops.flash_moba._flash_moba_attn_varlen_forward
_wrapped_flash_moba_attn_varlen_backward = torch.ops.flash_moba._flash_moba_attn_varlen_backward
_wrapped_mean_pool = torch.ops.flash_moba._mean_pool
_wrapped_gated_topk = torch.ops.flash_moba._gated_topk
_wrapped_attn_varlen_forward_bounded = torch.ops.flash_moba._attn_varlen_forward_bounded
_wrapped_attn_varlen_backward_bounded = torch.ops.flash_moba._attn_varlen_backward_bounded


def _fwd_key_block(lg_block_n: int) -> int:
    """Keys per visit of the forward's column form (fmoba_attn_fwd_key_block of the library, as plain arithmetic so
    that a traced graph can fold it)."""
    return 128 if lg_block_n % 128 == 0 else 64


# --------------------------------------------------------------------------------------
# autograd
# --------------------------------------------------------------------------------------
class FlashMobaAttnVarlenFunc(torch.autograd.Function):
    """Forward/backward over a given CSC pattern (flash_moba_interface.py:400-513).

    Two trailing arguments beyond the reference's twenty, both optional: max_visits, the bound on a row's visits in
    forward key blocks when the caller knows it (a gated pattern: top-k * lg_block_n / key block), and the gating's
    selection bits.  Without a bound it is counted from the pattern once, here (eager mode; one device-to-host read)
    or inside each op (while a graph is being traced or captured, where a data-dependent integer cannot leave an op).
    A caller's bound without selection bits is checked against the pattern in eager mode and raises if a row has more
    visits; under tracing or capture it is taken as given."""

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                moba_col_offsets, moba_col_nnz, moba_row_indices, lg_block_m, lg_block_n,
                dropout_p, softmax_scale, causal, softcap, alibi_slopes, deterministic,
                return_softmax, is_grad_enabled, max_visits=None, selection_bits=None):
        needs_grad = is_grad_enabled and any(x.requires_grad for x in (q, k, v))
        if softmax_scale is None:
            softmax_scale = q.shape[-1] ** (-0.5)
        flash_moba_gpu._reject_unsupported(dropout_p, softcap, alibi_slopes, None, None, return_softmax and dropout_p > 0)
        head_size_og = q.size(2)
        q, k, v = _pad8(q, k, v)
        def can_read_back():  # a device-to-host read is possible: not while tracing (fake tensors) or capturing a graph
            if torch.compiler.is_compiling() or torch._subclasses.fake_tensor.is_fake(q) or not q.is_cuda:
                return False
            return not torch.cuda.is_current_stream_capturing()

        if max_visits is None:
            if lg_block_n <= 0 or lg_block_n % 64 != 0 or not can_read_back():
                max_visits = -1  # counted inside the ops (a malformed lg_block_n is reported there)
            else:
                max_visits = flash_moba_gpu.count_max_visits(
                    q, moba_col_offsets, moba_col_nnz, moba_row_indices, cu_seqlens_q, cu_seqlens_k, k.shape[0], k.shape[1],
                    max_seqlen_q, max_seqlen_k, lg_block_n)
        elif selection_bits is None and lg_block_n > 0 and lg_block_n % 64 == 0 and can_read_back():
            # A bound of the caller's own for a pattern of the caller's own (the gated path hands its selection bits
            # along, and its bound, top-k, cannot be exceeded): visits beyond it would be dropped, so it is checked
            # against the pattern here (one device-to-host read).  While a graph is traced or captured nothing can be
            # read back: there the caller answers for the bound (the raw entry points report a violation through
            # their visits_overflow word).
            actual = flash_moba_gpu.count_max_visits(
                q, moba_col_offsets, moba_col_nnz, moba_row_indices, cu_seqlens_q, cu_seqlens_k, k.shape[0], k.shape[1],
                max_seqlen_q, max_seqlen_k, lg_block_n)
            if actual > max_visits:
                raise RuntimeError(f"max_visits = {max_visits}, but a row of the pattern has {actual} (row, key block) visits")
        out_padded, softmax_lse, S_dmask, rng_state = _wrapped_attn_varlen_forward_bounded(
            q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
            moba_col_offsets, moba_col_nnz, moba_row_indices, lg_block_m, lg_block_n,
            softmax_scale, causal, max_visits, selection_bits)
        if needs_grad:
            # the same bound in the backward's 64-key blocks
            ctx.bwd_visits = max_visits * (_fwd_key_block(lg_block_n) // 64) if max_visits > 0 else -1
            ctx.save_for_backward(q, k, v, out_padded, softmax_lse, cu_seqlens_q, cu_seqlens_k,
                                  moba_col_offsets, moba_col_nnz, moba_row_indices)
            ctx.cfg = (max_seqlen_q, max_seqlen_k, lg_block_m, lg_block_n, softmax_scale, causal, deterministic)
        out = out_padded[..., :head_size_og]
        return out if not return_softmax else (out, softmax_lse, S_dmask)

    @staticmethod
    def backward(ctx, dout, *args):
        (q, k, v, out, softmax_lse, cu_seqlens_q, cu_seqlens_k, col_offsets, col_nnz, row_indices) = ctx.saved_tensors
        (max_seqlen_q, max_seqlen_k, lg_block_m, lg_block_n, softmax_scale, causal, deterministic) = ctx.cfg
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        (dout_padded,) = _pad8(dout)
        _wrapped_attn_varlen_backward_bounded(
            dout_padded, q, k, v, out, softmax_lse, dq, dk, dv, cu_seqlens_q, cu_seqlens_k,
            max_seqlen_q, max_seqlen_k, col_offsets, col_nnz, row_indices, lg_block_m, lg_block_n,
            softmax_scale, causal, deterministic, ctx.bwd_visits)
        d = dout.shape[-1]  # the head dimension may have been padded
        return (dq[..., :d], dk[..., :d], dv[..., :d]) + (None,) * 19


# --------------------------------------------------------------------------------------
# public functions
# --------------------------------------------------------------------------------------
def flash_topk_varlen_func(q, k, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                           moba_topk, moba_chunk_size, causal=False):
    """Top-k key-chunk selection for MoBA on packed variable-length sequences.

    q: (total_q, num_heads, head_size), k: (total_k, num_heads_k, head_size), fp16/bf16;
    cu_seqlens_*: (batch + 1,) int32.  Every query scores the mean of every key chunk of
    `moba_chunk_size` keys, keeps the `moba_topk` best (causal: only chunks that lie
    entirely before it, plus its own chunk, which is always kept).

    Returns (col_offsets, col_nnz, indices): for sequence b, head h and key chunk c,
    ``indices[col_offsets[b,h,c] : col_offsets[b,h,c] + col_nnz[b,h,c]]`` are the query
    rows (local to the sequence, ascending) that attend to chunk c.
    col_offsets: (batch, num_heads, ceil(max_seqlen_k / chunk)) int64, col_nnz: same shape
    int32, indices: (total_q * num_heads * moba_topk,) int32.
    """
    q, k = _pad8(q, k)
    km, cu_seqlens_km = _wrapped_mean_pool(maybe_contiguous(k), cu_seqlens_k, max_seqlen_k, moba_chunk_size)
    # The row lists come back ascending, so the reference's second step
    # (_wrapped_varlen_sort, flash_moba_interface.py:570-572) has nothing left to do.
    return _wrapped_moba_fused_topk(q, km, cu_seqlens_q, cu_seqlens_k, cu_seqlens_km,
                                    max_seqlen_q, max_seqlen_k, moba_topk, moba_chunk_size, causal=causal)


def flash_moba_attn_varlen_func(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                                moba_col_offsets, moba_col_nnz, moba_row_indices,
                                lg_block_m=64, lg_block_n=64, dropout_p=0.0, softmax_scale=None,
                                causal=False, softcap=0.0, alibi_slopes=None, deterministic=False,
                                return_attn_probs=False):
    """Block-sparse attention over a column-wise (CSC) pattern, with autograd.

    q: (total_q, nheads, headdim); k, v: (total_k, nheads_k, headdim) with nheads % nheads_k
    == 0 (MQA/GQA: query head h reads kv head h // (nheads / nheads_k)).  The pattern says,
    per (sequence, head, key block of `lg_block_n` keys), which query rows attend to the
    block (see flash_topk_varlen_func; row lists must be ascending, without duplicates).
    causal=True additionally masks key j for query i unless j <= i + seqlen_k - seqlen_q
    (bottom-right aligned).  Rows that see no key produce 0.

    lg_block_m must be in [128, 1024] and a multiple of 64, lg_block_n a multiple of 64.
    dropout_p, softcap and alibi_slopes must stay at their defaults.  softmax_scale defaults
    to headdim ** -0.5.  Returns out (total_q, nheads, headdim), or with
    return_attn_probs=True the triple (out, softmax_lse (nheads, total_q) fp32, S_dmask
    (empty)).
    """
    return FlashMobaAttnVarlenFunc.apply(
        q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
        moba_col_offsets, moba_col_nnz, moba_row_indices, lg_block_m, lg_block_n,
        dropout_p, softmax_scale, causal, softcap, alibi_slopes, deterministic,
        return_attn_probs, torch.is_grad_enabled())


def flash_moba_varlen_func(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                           moba_chunk_size, moba_topk, causal=True):
    """MoBA attention end to end: gate (mean-pool + top-k + CSC), then sparse attention."""
    qp, kp = _pad8(q, k)
    km, cu_seqlens_km = _wrapped_mean_pool(maybe_contiguous(kp), cu_seqlens_k, max_seqlen_k, moba_chunk_size)
    col_offsets, col_nnz, indices, selection = _wrapped_gated_topk(
        qp, km, cu_seqlens_q, cu_seqlens_k, cu_seqlens_km, max_seqlen_q, max_seqlen_k, moba_topk, moba_chunk_size, causal)
    lg_block_m = decide_lg_block_m(moba_topk, moba_chunk_size, max_seqlen_k, causal)
    max_visits = None
    if moba_chunk_size > 0 and moba_chunk_size % 64 == 0:
        # a gated row visits at most top-k chunks: the forward needs no pass over the pattern to size its scratch,
        # and the gating's own selection bits spare its row-block form the pass that derives them from the lists
        max_visits = moba_topk * (moba_chunk_size // _fwd_key_block(moba_chunk_size))
    return FlashMobaAttnVarlenFunc.apply(
        q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
        col_offsets, col_nnz, indices, lg_block_m, moba_chunk_size,
        0.0, None, causal, 0.0, None, False, False, torch.is_grad_enabled(), max_visits, selection)

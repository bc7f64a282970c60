"""Per-chunk key mean-pool for variable-length batches (host side).

Mirrors ``flash_topk_mean_pool`` of the reference (flash_moba/triton_mean_pool.py:112-157):
same arguments, same return triple ``(km, cu_seqlens_km, max_chunks)``, output of exactly
``sum(ceil(len_b / chunk))`` rows in the input dtype.
"""
import torch

from flash_moba import flash_moba_hip as _hip


def chunk_cu_seqlens(cu_seqlens: torch.Tensor, chunk: int) -> torch.Tensor:
    """cu_seqlens of the pooled sequences: cumsum(ceil(len / chunk)), int32, on the same device."""
    if cu_seqlens.is_cuda and cu_seqlens.dtype == torch.int32 and cu_seqlens.is_contiguous() and cu_seqlens.numel() > 1 and chunk > 0:
        return _hip.chunk_offsets(cu_seqlens, chunk)  # one launch instead of six
    lens = cu_seqlens[1:] - cu_seqlens[:-1]
    chunks = torch.div(lens + (chunk - 1), chunk, rounding_mode="floor")
    out = torch.zeros_like(cu_seqlens, dtype=torch.int32)
    out[1:] = torch.cumsum(chunks, dim=0)
    return out


def _pool_into(k: torch.Tensor, cu_seqlens_k: torch.Tensor, cu_seqlens_km: torch.Tensor, rows: int,
               max_chunks: int, chunk: int) -> torch.Tensor:
    km = torch.empty((rows, k.shape[1], k.shape[2]), dtype=k.dtype, device=k.device)
    if rows and max_chunks:
        _hip.mean_pool(k, km, cu_seqlens_k, cu_seqlens_km, max_chunks, chunk)
    return km


def flash_topk_mean_pool(input, cu_seqlens_input, max_seqlen_input, pool_block_size):
    """Mean over non-overlapping windows of `pool_block_size` rows inside every sequence.

    input: (total_seqlen, num_heads, head_dim) fp16/bf16; cu_seqlens_input: (batch + 1,) int32.
    Returns (output (total_blocks, num_heads, head_dim), cu_seqlens_output int32, max_blocks).
    The exact output size needs the last entry of cu_seqlens_output on the host (one
    device-to-host read, as in the reference, triton_mean_pool.py:140).
    """
    if input.stride(-1) != 1:
        input = input.contiguous()
    max_chunks = (max_seqlen_input + pool_block_size - 1) // pool_block_size
    cu_km = chunk_cu_seqlens(cu_seqlens_input, pool_block_size)
    total_blocks = int(cu_km[-1].item())
    km = _pool_into(input, cu_seqlens_input.to(torch.int32), cu_km, total_blocks, max_chunks, pool_block_size)
    return km, cu_km, max_chunks


def mean_pool_nosync(k: torch.Tensor, cu_seqlens_k: torch.Tensor, max_seqlen_k: int, chunk: int):
    """Same pooling without the device-to-host read: the output is sized by the bound
    total_k // chunk + batch >= sum(ceil(len_b / chunk)); rows past cu_km[-1] are never
    read by the gating kernel.  Used on the hot path of flash_topk_varlen_func."""
    if k.stride(-1) != 1:
        k = k.contiguous()
    batch = cu_seqlens_k.numel() - 1
    max_chunks = (max_seqlen_k + chunk - 1) // chunk
    cu_km = chunk_cu_seqlens(cu_seqlens_k, chunk)
    rows = k.shape[0] // chunk + batch
    return _pool_into(k, cu_seqlens_k, cu_km, rows, max_chunks, chunk), cu_km, max_chunks

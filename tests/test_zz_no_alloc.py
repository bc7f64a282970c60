"""fmoba_fused_topk_static (the gating + CSC build for callers that cannot allocate device memory) against
fmoba_fused_topk, through the C ABI: two calls in a row on one device, the second with a smaller input, so
that what the first call left in the library's fixed scratch array must not leak into the second."""
import ctypes

import pytest
import torch

from flash_moba import flash_moba_hip as H
from flash_moba.mean_pool import flash_topk_mean_pool
from oracle import moba_oracle as O

pytestmark = pytest.mark.gpu


def _gate(entry, q, km, cu, cu_km, max_len, topk, chunk, with_workspace, outputs=None, sync=True):
    lib = H.load_library()
    T, heads, d = q.shape
    batch = cu.numel() - 1
    max_cols = (max_len + chunk - 1) // chunk
    if outputs is None:
        co = torch.full((batch, heads, max_cols), -7, dtype=torch.int64, device=q.device)
        cn = torch.full((batch, heads, max_cols), -7, dtype=torch.int32, device=q.device)
        flat = torch.full((T * heads * topk,), -7, dtype=torch.int32, device=q.device)
    else:
        co, cn, flat = outputs
    ws_bytes = lib.fmoba_fused_topk_workspace_bytes(batch, T, heads, max_len, max_len, chunk)
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=q.device) if with_workspace else None
    a = H.FusedTopkArgs(q.data_ptr(), km.data_ptr(), cu.data_ptr(), cu.data_ptr(), cu_km.data_ptr(),
                        co.data_ptr(), cn.data_ptr(), flat.data_ptr(), None, None,
                        ws.data_ptr() if with_workspace else None, ws_bytes if with_workspace else 0,
                        batch, T, heads, km.shape[1], d, max_len, max_len, topk, chunk, 1, 1,
                        q.stride(0), q.stride(1), km.stride(0), km.stride(1))
    rc = getattr(lib, entry)(ctypes.byref(a), torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.fmoba_last_error().decode()
    if sync:
        torch.cuda.synchronize()
    return co, cn, flat, ws_bytes


def test_static_scratch_gating_matches_the_workspace_entry_point_twice_in_a_row():
    # first call: 3 ragged sequences, 5 selection words per row; second: smaller in every dimension
    cases = [([2500, 4133, 9000], 8, 128, 64, 12, 21), ([700, 333], 2, 64, 64, 3, 22)]
    sizes = []
    for lens, heads, d, chunk, topk, seed in cases:
        q, k, _, cu = O.make_inputs(lens, heads, d, chunk, seed, torch.bfloat16)
        q, k, cu = q.cuda(), k.cuda(), cu.cuda()
        km, cu_km, _ = flash_topk_mean_pool(k, cu, max(lens), chunk)
        ref = _gate("fmoba_fused_topk", q, km, cu, cu_km, max(lens), topk, chunk, True)
        got = _gate("fmoba_fused_topk_static", q, km, cu, cu_km, max(lens), topk, chunk, False)
        for name, x, y in zip(("col_offsets", "col_nnz", "flat_indices"), got, ref):
            assert torch.equal(x, y), f"{name} differs for lens={lens}"
        assert int(ref[1].sum()) > 0
        sizes.append(ref[3])
    assert sizes[1] < sizes[0]


def test_static_scratch_gating_rejects_what_its_buffer_cannot_hold():
    lib = H.load_library()
    a = H.FusedTopkArgs()
    a.batch, a.total_q, a.heads, a.heads_k, a.head_dim = 1, 262144, 16, 16, 128
    a.max_seqlen_q = a.max_seqlen_k = 262144
    a.topk, a.chunk, a.is_causal, a.dtype = 16, 128, 1, 1
    assert lib.fmoba_fused_topk_workspace_bytes(1, 262144, 16, 262144, 262144, 128) > (32 << 20)
    assert lib.fmoba_fused_topk_static(ctypes.byref(a), None) != 0
    assert b"fixed buffer" in lib.fmoba_last_error()


def test_static_scratch_gating_allocates_nothing_and_replays_from_a_graph():
    # the callers the entry point is for: code under HIP graph capture.  After one call outside any capture (the
    # first call on a device looks the array's address up), the call is recorded on a capturing stream, replayed on
    # new inputs written into the captured tensors, and compared with the workspace entry point every time; torch's
    # allocator sees no change across the recorded call (its outputs are allocated before).
    lens, heads, d, chunk, topk = [3000, 1700, 650], 4, 128, 64, 9
    data = []
    for seed in (31, 32, 33):
        q, k, _, cu = O.make_inputs(lens, heads, d, chunk, seed, torch.bfloat16)
        q, k, cu = q.cuda(), k.cuda(), cu.cuda()
        km, cu_km, _ = flash_topk_mean_pool(k, cu, max(lens), chunk)
        data.append((q, km))
    _gate("fmoba_fused_topk_static", data[0][0], data[0][1], cu, cu_km, max(lens), topk, chunk, False)  # warm-up, eager
    qs, kms = data[0][0].clone(), data[0][1].clone()
    T, max_cols = qs.shape[0], (max(lens) + chunk - 1) // chunk
    outs = (torch.empty((len(lens), heads, max_cols), dtype=torch.int64, device="cuda"),
            torch.empty((len(lens), heads, max_cols), dtype=torch.int32, device="cuda"),
            torch.empty((T * heads * topk,), dtype=torch.int32, device="cuda"))
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        before = torch.cuda.memory_allocated()
        _gate("fmoba_fused_topk_static", qs, kms, cu, cu_km, max(lens), topk, chunk, False, outputs=outs, sync=False)
        assert torch.cuda.memory_allocated() == before
    for q, km in data:
        ref = _gate("fmoba_fused_topk", q, km, cu, cu_km, max(lens), topk, chunk, True)  # eager work between the replays
        qs.copy_(q)
        kms.copy_(km)
        for t in outs:
            t.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        for name, x, y in zip(("col_offsets", "col_nnz", "flat_indices"), outs, ref):
            assert torch.equal(x, y), name

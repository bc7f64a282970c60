"""GPU parity tests: every stage of the HIP path (called through the C-ABI binding)
against the CPU oracle on the same seeded inputs.

Bars: bit-exact for integer artefacts (CSC triple, sorted keys) wherever the oracle's
score gap between the last kept and first rejected chunk exceeds 1e-3 relative;
2e-2 abs / 1e-2 rel for bf16/fp16 attention outputs and gradients; 1e-2 abs for the
mean-pool (the reference's own tolerance, tests/test_triton_mean_pool.py:63-64), tightened
here to one ulp of the output dtype.
"""
import math

import numpy as np
import pytest
import torch

from oracle import moba_oracle as O
from gpu_utils import assert_close, csc_structure_ok, selection_sets

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fm():
    import flash_moba
    from flash_moba import flash_moba_hip, flash_moba_interface, mean_pool

    class NS:
        pass

    ns = NS()
    ns.api = flash_moba
    ns.hip = flash_moba_hip
    ns.iface = flash_moba_interface
    ns.pool = mean_pool
    return ns


# ------------------------------------------------------------------------ mean-pool
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("batch,max_seqlen,heads,d,pool", [
    (1, 512, 4, 64, 32), (8, 2048, 12, 128, 64), (8, 512, 4, 256, 128), (1, 2048, 12, 64, 512),
    (8, 2048, 4, 128, 256), (4, 128, 4, 32, 256), (16, 8, 4, 32, 4), (3, 777, 5, 72, 48),
])
def test_mean_pool_matches_oracle(fm, batch, max_seqlen, heads, d, pool, dtype):
    g = torch.Generator().manual_seed(42)
    seqlens = torch.randint(0, max_seqlen, (batch,), generator=g)
    cu = torch.cat([torch.zeros(1, dtype=torch.int64), torch.cumsum(seqlens, 0)]).to(torch.int32)
    x = torch.randn((int(seqlens.sum()), heads, d), generator=g).to(dtype)
    km, cu_km, maxc = fm.pool.flash_topk_mean_pool(x.cuda(), cu.cuda(), max_seqlen, pool)
    ref, cu_ref = O.mean_pool(x, cu, pool)
    assert km.shape == ref.shape and km.dtype == dtype
    assert torch.equal(cu_km.cpu(), cu_ref) and cu_km.dtype == torch.int32
    assert maxc == (max_seqlen + pool - 1) // pool
    # fp32 accumulation in a different order: at most one ulp of the 16-bit result
    ulp = (ref.float().abs() * (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10)).clamp_min(1e-6)
    assert ((km.cpu().float() - ref.float()).abs() <= ulp).all()
    assert torch.allclose(km.cpu().float(), ref.float(), atol=1e-2, rtol=0)


def test_mean_pool_all_empty_and_strided(fm):
    cu = torch.zeros(9, dtype=torch.int32).cuda()
    km, cu_km, _ = fm.pool.flash_topk_mean_pool(torch.zeros((0, 12, 128), dtype=torch.bfloat16).cuda(), cu, 0, 128)
    assert km.shape == (0, 12, 128) and cu_km.tolist() == [0] * 9
    # k taken as a strided view of a packed qkv tensor
    g = torch.Generator().manual_seed(1)
    qkv = torch.randn((300, 3, 4, 64), generator=g).to(torch.bfloat16)
    cu = torch.tensor([0, 100, 300], dtype=torch.int32)
    k = qkv[:, 1]
    km, _, _ = fm.pool.flash_topk_mean_pool(qkv.cuda()[:, 1], cu.cuda(), 200, 64)
    ref, _ = O.mean_pool(k.contiguous(), cu, 64)
    assert torch.allclose(km.cpu().float(), ref.float(), atol=1e-2)


@pytest.mark.parametrize("batch,chunk", [(1, 64), (3, 128), (8, 64), (255, 1), (256, 7), (257, 64), (1000, 33), (5000, 128)])
def test_chunk_offsets_match_the_tensor_expression(fm, batch, chunk):
    # flash_moba/triton_mean_pool.py:132-139: lengths, ceil-division, cumulative sum, a leading zero
    rng = np.random.RandomState(batch * 131 + chunk)
    lens = rng.randint(0, 700, batch)
    lens[rng.randint(0, batch, max(1, batch // 7))] = 0
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    want = torch.zeros(batch + 1, dtype=torch.int32)
    want[1:] = torch.cumsum(torch.div(cu[1:] - cu[:-1] + (chunk - 1), chunk, rounding_mode="floor"), 0)
    got = fm.hip.chunk_offsets(cu.cuda(), chunk)
    assert got.dtype == torch.int32 and torch.equal(got.cpu(), want)


# ------------------------------------------------------------------------ gating + CSC
def _gate_case(fm, seed, lens_q, lens_k, H, Hk, D, chunk, topk, causal, dtype=torch.bfloat16, integer=False):
    g = torch.Generator().manual_seed(seed)
    Tq, Tk = sum(lens_q), sum(lens_k)
    if integer:
        q = torch.randint(-2, 3, (Tq, H, D), generator=g).to(dtype)
        k = torch.randint(-1, 2, (Tk, Hk, D), generator=g).to(dtype)
    else:
        q = torch.randn((Tq, H, D), generator=g).to(dtype)
        k = torch.randn((Tk, Hk, D), generator=g)
        # per-chunk bias so that scores separate
        pos = 0
        for L in lens_k:
            C = (L + chunk - 1) // chunk
            if C:
                k[pos:pos + L] += (0.5 * torch.randn((C, Hk, D), generator=g)).repeat_interleave(chunk, 0)[:L]
            pos += L
        k = k.to(dtype)
    cuq = torch.tensor([0] + list(np.cumsum(lens_q)), dtype=torch.int32)
    cuk = torch.tensor([0] + list(np.cumsum(lens_k)), dtype=torch.int32)
    return q, k, cuq, cuk


def _check_gating(fm, q, k, cuq, cuk, chunk, topk, causal, integer=False):
    H = q.shape[1]
    max_q, max_k = int((cuq[1:] - cuq[:-1]).max()), int((cuk[1:] - cuk[:-1]).max())
    maxC = (max_k + chunk - 1) // chunk
    # chunk means from the HIP kernel feed both sides, so that only the gating is compared
    km_gpu, cu_km, _ = fm.pool.flash_topk_mean_pool(k.cuda(), cuk.cuda(), max_k, chunk)
    if integer:
        km_gpu = (km_gpu.float() * chunk).round().to(k.dtype)   # integer-valued chunk sums: scores tie exactly
    co, cn, flat, values, indices = fm.hip.moba_fused_topk(
        q.cuda(), km_gpu, cuq.cuda(), cuk.cuda(), cu_km, max_q, max_k, topk, chunk, causal)
    torch.cuda.synchronize()
    idx_ref, val_ref, gates = O.fused_topk(q, km_gpu.cpu(), cuq, cuk, cu_km.cpu(), topk, chunk, causal, return_gate=True)
    co_ref, cn_ref, flat_ref = O.csc_from_topk(idx_ref, cuq, topk, maxC)
    assert co.dtype == torch.int64 and cn.dtype == torch.int32 and flat.dtype == torch.int32
    assert co.shape == co_ref.shape and cn.shape == cn_ref.shape and flat.shape == flat_ref.shape
    csc_structure_ok(co, cn, flat, cuq, H, topk)
    unamb = O.topk_gap_mask(gates, cuq, topk, 1e-3) if any(g is not None for g in gates) else None
    n_amb = 0 if unamb is None else int((~unamb).sum())
    if n_amb == 0 or integer:
        # no near-tie anywhere (or exact integer arithmetic): everything must be bit-exact
        assert torch.equal(cn.cpu(), cn_ref)
        assert torch.equal(co.cpu(), co_ref)
        assert torch.equal(flat.cpu(), flat_ref)
    else:
        # rows away from near-ties must select exactly the oracle's chunk set
        cuq_np = cuq.numpy()
        for b in range(len(cuq_np) - 1):
            Lq = int(cuq_np[b + 1] - cuq_np[b])
            for h in range(H):
                got = selection_sets(co, cn, flat, b, h, Lq, maxC)
                ref = selection_sets(co_ref, cn_ref, flat_ref, b, h, Lq, maxC)
                ok_rows = unamb[int(cuq_np[b]):int(cuq_np[b + 1]), h].numpy()
                assert (got[ok_rows] == ref[ok_rows]).all()
                assert (got.sum(1) == ref.sum(1)).all()       # same number of chunks everywhere
    # ordered per-row lists (auxiliary outputs): same sets as the CSC, descending scores
    kr = (topk + 15) // 16 * 16
    assert indices.shape == (q.shape[0], H, kr) and values.shape == indices.shape
    mism = (indices.cpu() != idx_ref).float().mean().item()
    assert mism < 0.005 or integer, mism        # the reference's own bar (tests/test_fused_topk.py:251-254)
    if integer:
        assert torch.equal(indices.cpu(), idx_ref)
        assert torch.equal(values.cpu(), val_ref)
    # the ordered lists name exactly the chunks whose columns hold the row, near-ties included (one selection feeds both)
    ic = indices.cpu().numpy()
    cuq_np = cuq.numpy()
    for b in range(len(cuq_np) - 1):
        s0, Lq = int(cuq_np[b]), int(cuq_np[b + 1] - cuq_np[b])
        for h in range(H):
            got = selection_sets(co, cn, flat, b, h, Lq, maxC)
            raw = np.zeros_like(got)
            rows, slots = np.nonzero(ic[s0:s0 + Lq, h] >= 0)
            raw[rows, ic[s0:s0 + Lq, h][rows, slots]] = True
            assert (raw == got).all(), (b, h)


@pytest.mark.parametrize("topk", [1, 2, 4, 8, 16, 24, 32, 33, 64])
@pytest.mark.parametrize("chunk", [1, 16, 32])
@pytest.mark.parametrize("causal", [True, False])
def test_gating_reference_grid(fm, topk, chunk, causal):
    # (b, h, s) grid of tests/test_fused_topk.py:119-122 limited to <= 256 chunks per sequence
    for (b, h, s, d, dt) in [(1, 4, 128, 64, torch.float16), (2, 8, 256, 128, torch.bfloat16), (4, 4, 512, 256, torch.bfloat16)]:
        if (s + chunk - 1) // chunk > 256:
            continue
        q, k, cuq, cuk = _gate_case(fm, 0, [s] * b, [s] * b, h, h, d, chunk, topk, causal, dt)
        _check_gating(fm, q, k, cuq, cuk, chunk, topk, causal)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("topk,chunk", [(3, 16), (8, 32), (5, 64)])
def test_gating_exact_ties_prefer_higher_chunk(fm, topk, chunk, causal):
    q, k, cuq, cuk = _gate_case(fm, 7, [300, 0, 513], [300, 0, 513], 4, 2, 64, chunk, topk, causal, integer=True)
    _check_gating(fm, q, k, cuq, cuk, chunk, topk, causal, integer=True)


@pytest.mark.parametrize("causal", [True, False])
def test_gating_ragged_varlen_gqa_and_len_q_ne_len_k(fm, causal):
    q, k, cuq, cuk = _gate_case(fm, 11, [200, 77, 0, 1, 640], [333, 50, 0, 130, 640], 6, 2, 72, 64, 4, causal)
    _check_gating(fm, q, k, cuq, cuk, 64, 4, causal)


def test_gating_headline_shape_small(fm):
    # the headline configuration's shape parameters (d=128, chunk 64, top-k 32) at 2 x ~3K tokens
    q, k, cuq, cuk = _gate_case(fm, 5, [3072, 2112], [3072, 2112], 4, 4, 128, 64, 32, True)
    _check_gating(fm, q, k, cuq, cuk, 64, 32, True)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("topk", [1, 4, 16, 33, 40, 64])
def test_gating_more_than_256_chunks_per_sequence(fm, topk, causal):
    # the grouped gate: 550 and 500/175 chunks per sequence, (b, h, s) in the spirit of tests/test_fused_topk.py:119-122
    # (running lists of 16, 32 and -- top-k above 33 -- 64 winners per row)
    q, k, cuq, cuk = _gate_case(fm, 3, [1100], [1100], 2, 2, 64, 2, topk, causal, torch.float16)
    _check_gating(fm, q, k, cuq, cuk, 2, topk, causal)
    q, k, cuq, cuk = _gate_case(fm, 4, [2000, 0, 700], [2000, 0, 700], 4, 2, 128, 4, topk, causal)
    _check_gating(fm, q, k, cuq, cuk, 4, topk, causal)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("topk", [5, 16, 40])
def test_gating_more_than_256_chunks_len_q_ne_len_k(fm, topk, causal):
    # fewer queries than keys (the queries are the last rows of the sequence), ragged batch, grouped heads
    q, k, cuq, cuk = _gate_case(fm, 21, [700, 33, 0, 1500], [2600, 700, 90, 1500], 4, 2, 64, 4, topk, causal)
    _check_gating(fm, q, k, cuq, cuk, 4, topk, causal)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("topk", [16, 33, 64])
def test_gating_reference_grid_point_1024_chunks(fm, topk, causal):
    # (b, h, s) = (8, 2, 1024) with chunk size 1 of tests/test_fused_topk.py:115-122: 1024 chunks per sequence
    q, k, cuq, cuk = _gate_case(fm, 0, [1024] * 8, [1024] * 8, 2, 2, 64, 1, topk, causal, torch.bfloat16)
    _check_gating(fm, q, k, cuq, cuk, 1, topk, causal)
    # head_dim 256 takes the variants with the smallest groups
    q, k, cuq, cuk = _gate_case(fm, 1, [1024], [1024], 2, 1, 256, 2, topk, causal, torch.float16)
    _check_gating(fm, q, k, cuq, cuk, 2, topk, causal)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("topk", [6, 12, 17])
def test_gating_more_than_256_chunks_exact_ties(fm, topk, causal):
    # (up to 16 running winners per row: the lanes hold four or eight of them each)
    q, k, cuq, cuk = _gate_case(fm, 9, [900, 1300], [900, 1300], 2, 1, 64, 4, topk, causal, integer=True)
    _check_gating(fm, q, k, cuq, cuk, 4, topk, causal, integer=True)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("topk", [3, 9, 16])
def test_gating_thousands_of_chunks_exact_ties(fm, topk, causal):
    # dozens of groups per row, scores from a small set of integers: many scores equal the weakest winner, rows get
    # more entrants than a list holds, exact zeros of both signs occur
    q, k, cuq, cuk = _gate_case(fm, 12, [3000, 700], [3000, 700], 2, 2, 64, 1, topk, causal, integer=True)
    _check_gating(fm, q, k, cuq, cuk, 1, topk, causal, integer=True)


@pytest.mark.parametrize("causal", [True, False])
def test_gating_more_than_256_chunks_exact_ties_long_lists(fm, causal):
    q, k, cuq, cuk = _gate_case(fm, 10, [1500], [1500], 2, 1, 64, 4, 50, causal, integer=True)
    _check_gating(fm, q, k, cuq, cuk, 4, 50, causal, integer=True)


@pytest.mark.parametrize("topk", [8, 33, 64])
@pytest.mark.parametrize("lens", [[4096], [4500, 300], [8192]])
def test_gating_4096_to_8192_chunks_exact_ties(fm, topk, lens):
    # the chunk counts of the reference's own 2 x 524288-token benchmark point (4096) and beyond: the grouped gates
    # write their selection words and counts out in several passes; top-k 8 keeps a row's winners in registers, 33 and
    # 64 take the variants with 32 and 64 running winners per row
    q, k, cuq, cuk = _gate_case(fm, 31, lens, lens, 2, 1, 64, 1, topk, True, integer=True)
    _check_gating(fm, q, k, cuq, cuk, 1, topk, True, integer=True)


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("topk", [40, 64])
def test_gating_long_lists_3000_chunks_every_head_dim(fm, D, topk):
    # 64 running winners per row with thousands of chunks, at every width of the chunk-mean tile
    q, k, cuq, cuk = _gate_case(fm, 32, [3000], [3000], 2, 2, D, 1, topk, True, integer=True)
    _check_gating(fm, q, k, cuq, cuk, 1, topk, True, integer=True)
    q, k, cuq, cuk = _gate_case(fm, 33, [2900, 200], [2900, 200], 2, 1, D, 1, topk, False, torch.float16)
    _check_gating(fm, q, k, cuq, cuk, 1, topk, False)


def test_gating_rejects_more_chunks_than_supported(fm):
    # chunk indices are 16-bit fields inside the kernels: the call fails on the host, before anything is launched
    T = 65536 + 8
    q = torch.zeros((T, 1, 8), dtype=torch.bfloat16).cuda()
    cu = torch.tensor([0, T], dtype=torch.int32).cuda()
    with pytest.raises(RuntimeError, match="at most 65535 are supported"):
        fm.hip.moba_fused_topk(q, q, cu, cu, cu, T, T, 4, 1, True, return_raw=False)


def test_gating_no_keys(fm):
    q = torch.randn(10, 2, 64).to(torch.bfloat16).cuda()
    km = torch.zeros(0, 2, 64, dtype=torch.bfloat16).cuda()
    cuq = torch.tensor([0, 10], dtype=torch.int32).cuda()
    z = torch.tensor([0, 0], dtype=torch.int32).cuda()
    co, cn, flat, val, idx = fm.hip.moba_fused_topk(q, km, cuq, z, z, 10, 0, 4, 16, True)
    assert co.shape == (1, 2, 0) and (flat == -1).all() and (idx == -1).all() and torch.isinf(val).all()


def test_gating_rejects_bad_arguments(fm):
    q = torch.zeros(8, 2, 64, dtype=torch.bfloat16).cuda()
    cu = torch.tensor([0, 8], dtype=torch.int32).cuda()
    with pytest.raises(RuntimeError, match="moba_topk must be <= 64"):
        fm.hip.moba_fused_topk(q, q, cu, cu, cu, 8, 8, 65, 4, True)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        fm.hip.moba_fused_topk(q[..., :60].contiguous(), q[..., :60].contiguous(), cu, cu, cu, 8, 8, 2, 4, True)
    with pytest.raises(RuntimeError, match="int32"):
        fm.hip.moba_fused_topk(q, q, cu.long(), cu, cu, 8, 8, 2, 4, True)
    with pytest.raises(RuntimeError, match="same dtype"):
        fm.hip.moba_fused_topk(q, q.half(), cu, cu, cu, 8, 8, 2, 4, True)


# ------------------------------------------------------------------------ segmented sort
@pytest.mark.parametrize("segments,seed,maxlen", [(1, 3, 2 ** 18), (17, 11, 2 ** 16), (128, 47, 2 ** 14), (1024, 97, 4096), (4096, 233, 512)])
def test_varlen_sort_random(fm, segments, seed, maxlen):
    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(0, maxlen, (segments,), generator=g)
    ends = torch.cumsum(lens, 0).to(torch.int64)
    starts = ends - lens
    total = int(ends[-1])
    src = torch.randint(0, 2 ** 31 - 1, (total,), generator=g, dtype=torch.int64).to(torch.int32)
    out = fm.hip.varlen_sort(starts.cuda(), ends.cuda(), src.cuda())
    ref = O.varlen_sort(starts, ends, src)
    assert torch.equal(out.cpu(), ref)


def test_varlen_sort_extremes_gaps_and_small_ranges(fm):
    i32 = torch.iinfo(torch.int32)
    vals = torch.tensor([i32.max, i32.min] * 32, dtype=torch.int32)
    starts = torch.tensor([0, 16, 32, 48], dtype=torch.int64)
    ends = starts + 16
    out = fm.hip.varlen_sort(starts.cuda(), ends.cuda(), vals.cuda())
    assert torch.equal(out.cpu(), O.varlen_sort(starts, ends, vals))
    # gaps between segments stay zero; negative keys; a long segment of row-index-like keys
    g = torch.Generator().manual_seed(5)
    src = torch.randint(-50000, 50000, (100000,), generator=g, dtype=torch.int64).to(torch.int32)
    starts = torch.tensor([5, 1000, 30000, 99990], dtype=torch.int64)
    ends = torch.tensor([900, 1000, 90000, 100000], dtype=torch.int64)
    out = fm.hip.varlen_sort(starts.cuda(), ends.cuda(), src.cuda())
    assert torch.equal(out.cpu(), O.varlen_sort(starts, ends, src))
    out = fm.hip.varlen_sort(starts[:0].cuda(), ends[:0].cuda(), src.cuda())
    assert (out == 0).all()


def test_varlen_sort_size_classes(fm):
    # segment lengths on both sides of every size class of the kernel (2048, 8192, 16384 keys), mixed in one call,
    # with gaps, keys of both signs and a segment of equal keys
    lens = [2048, 1, 2049, 0, 8192, 63, 8193, 64, 16384, 65, 16385, 2047, 300, 40000]
    g = torch.Generator().manual_seed(21)
    starts, ends, pos = [], [], 3
    for n in lens:
        starts.append(pos)
        ends.append(pos + n)
        pos += n + 5
    src = torch.randint(-2 ** 31, 2 ** 31 - 1, (pos,), generator=g, dtype=torch.int64).to(torch.int32)
    src[starts[12]:ends[12]] = -7
    src[starts[4]:ends[4]] = torch.randint(0, 70000, (8192,), generator=g, dtype=torch.int64).to(torch.int32)
    starts, ends = torch.tensor(starts, dtype=torch.int64), torch.tensor(ends, dtype=torch.int64)
    out = fm.hip.varlen_sort(starts.cuda(), ends.cuda(), src.cuda())
    assert torch.equal(out.cpu(), O.varlen_sort(starts, ends, src))


def test_varlen_sort_keys_without_repeats_and_with_one(fm):
    # segments of distinct keys in a narrow range take the bitmap shortcut of the kernel, one repeated key sends a
    # segment back to the radix passes: every size class, lengths up to 300000 (through HBM), ranges on both sides of
    # what the bitmaps hold (32 x 2048, 32 x 8192, 32 x 16384 and 64 x 16384 keys), keys of both signs
    g = torch.Generator().manual_seed(77)
    cases = [(1, 1, 0), (2, 2, -1), (63, 64, 5), (2048, 2048, -1000), (2048, 65536, 0), (2047, 65537, -7), (1500, 65535, 100),
             (2049, 3000, 0), (8192, 262144, -3), (8000, 262145, 0), (8193, 10000, 2 ** 31 - 10001), (16384, 524288, -2 ** 31),
             (16000, 524289, 0), (16385, 16385, -16000), (40000, 1048576, -500000), (40000, 1048577, 0), (300000, 300000, 0),
             (300000, 600000, -300000), (5000, 14336, 0)]
    chunks, starts, ends, pos = [], [], [], 2
    for n, span, lo in cases:
        for repeat in (False, True):
            keys = torch.randperm(span, generator=g)[:n] + lo
            if repeat and n > 1:
                keys[int(torch.randint(0, n - 1, (1,), generator=g))] = keys[n - 1]
            chunks.append((pos, keys))
            starts.append(pos)
            ends.append(pos + n)
            pos += n + 3
    src = torch.full((pos,), 12345, dtype=torch.int32)
    for at, keys in chunks:
        src[at:at + keys.numel()] = keys.to(torch.int32)
    starts, ends = torch.tensor(starts, dtype=torch.int64), torch.tensor(ends, dtype=torch.int64)
    out = fm.hip.varlen_sort(starts.cuda(), ends.cuda(), src.cuda())
    assert torch.equal(out.cpu(), O.varlen_sort(starts, ends, src))


def test_varlen_sort_tiny_segments_at_every_alignment(fm):
    # lengths 0 .. 13 starting at every offset modulo four (the bitmap launch reads whole 16-byte vectors between up to
    # three keys before and after them), distinct keys and keys with a repeat, one call
    g = torch.Generator().manual_seed(13)
    starts, ends, pieces, pos = [], [], [], 0
    for n in range(14):
        for shift in range(4):
            for repeat in (False, True):
                while pos % 4 != shift:
                    pos += 1
                keys = torch.randperm(40, generator=g)[:n] - 20
                if repeat and n > 1:
                    keys[0] = keys[n - 1]
                starts.append(pos)
                ends.append(pos + n)
                pieces.append((pos, keys))
                pos += n
    src = torch.full((pos + 2,), -99, dtype=torch.int32)
    for at, keys in pieces:
        src[at:at + keys.numel()] = keys.to(torch.int32)
    starts, ends = torch.tensor(starts, dtype=torch.int64), torch.tensor(ends, dtype=torch.int64)
    out = fm.hip.varlen_sort(starts.cuda(), ends.cuda(), src.cuda())
    assert torch.equal(out.cpu(), O.varlen_sort(starts, ends, src))
    # the same keys behind an odd offset of the buffers themselves (a view that starts one int32 into an allocation)
    src1 = torch.cat([torch.zeros(1, dtype=torch.int32), src]).cuda()[1:]
    out1 = fm.hip.varlen_sort(starts.cuda(), ends.cuda(), src1)
    assert torch.equal(out1.cpu(), out.cpu())


def test_varlen_sort_with_a_workspace_of_total_int32_only(fm):
    # the C entry point also takes a workspace of exactly `total` int32 (then it always clears the whole output first);
    # segments that tile the buffer and segments with gaps, ascending and not, both ways, into an output full of 77s
    lib = fm.hip.load_library()
    g = torch.Generator().manual_seed(9)
    for gaps, reverse in ((False, False), (True, False), (True, True), (False, True)):
        lens = torch.randint(0, 3000, (40,), generator=g)
        ends = torch.cumsum(lens + (7 if gaps else 0), 0).to(torch.int64)
        starts = ends - lens
        total = int(ends[-1]) + (5 if gaps else 0)
        if reverse:  # the segments need not come in ascending order
            starts, ends = starts.flip(0).contiguous(), ends.flip(0).contiguous()
        src = torch.randint(-10 ** 6, 10 ** 6, (total,), generator=g, dtype=torch.int64).to(torch.int32)
        ref = O.varlen_sort(starts, ends, src)
        sd, ed, xd = starts.cuda(), ends.cuda(), src.cuda()
        for ws_bytes in (total * 4, lib.fmoba_varlen_sort_workspace_bytes(total)):
            dst = torch.full((total,), 77, dtype=torch.int32, device="cuda")
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
            rc = lib.fmoba_varlen_sort(sd.data_ptr(), ed.data_ptr(), sd.numel(), xd.data_ptr(), dst.data_ptr(), total, ws.data_ptr(),
                                       ws_bytes, torch.cuda.current_stream().cuda_stream)
            assert rc == 0, lib.fmoba_last_error()
            assert torch.equal(dst.cpu(), ref)


def test_varlen_sort_restores_a_shuffled_csc(fm):
    # the op as the reference pipeline uses it: shuffle each column list, sort it back
    q, k, cuq, cuk = _gate_case(fm, 3, [700, 300], [700, 300], 4, 4, 64, 32, 6, True)
    co, cn, flat = fm.api.flash_topk_varlen_func(q.cuda(), k.cuda(), cuq.cuda(), cuk.cuda(), 700, 700, 6, 32, causal=True)
    f = flat.cpu().clone()
    g = torch.Generator().manual_seed(0)
    for s, n in zip(co.flatten().tolist(), cn.flatten().tolist()):
        if n > 1:
            f[s:s + n] = f[s:s + n][torch.randperm(n, generator=g)]
    back = torch.ops.flash_moba._varlen_sort(co, cn, f.cuda())
    assert torch.equal(back, flat)


# ------------------------------------------------------------------------ attention
def _random_csc(seed, lens_q, lens_k, H, lg_n, topk, causal):
    """Random block pattern in the spirit of generate_moba_sparse_mask_topk
    (flash_moba/moba_test_utils.py:61-96) with the gap-free running offsets of
    generate_moba_params_from_sparse_mask (:169-191)."""
    rng = np.random.RandomState(seed)
    nb = len(lens_q)
    maxC = (max(lens_k) + lg_n - 1) // lg_n
    co = np.zeros((nb, H, maxC), dtype=np.int64)
    cn = np.zeros((nb, H, maxC), dtype=np.int32)
    rows_all = []
    offset = 0
    for b in range(nb):
        Lq, Lk = lens_q[b], lens_k[b]
        for h in range(H):
            lists = [[] for _ in range(maxC)]
            for r in range(Lq):
                end_col = Lk - (Lq - r - 1) if causal else Lk
                nblk = max(0, math.ceil(end_col / lg_n))
                if nblk > 0:
                    sel = set(rng.permutation(nblk - 1)[: min(topk - 1, nblk - 1)].tolist()) | {nblk - 1}
                    for c in sel:
                        lists[c].append(r)
            for c in range(maxC):
                co[b, h, c] = offset
                cn[b, h, c] = len(lists[c])
                rows_all.extend(lists[c])
                offset += len(lists[c])
    ind = np.array(rows_all if rows_all else [0], dtype=np.int32)
    return torch.from_numpy(co), torch.from_numpy(cn), torch.from_numpy(ind)


def _attn_inputs(seed, lens_q, lens_k, H, Hk, D, dtype):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((sum(lens_q), H, D), generator=g).to(dtype)
    k = torch.randn((sum(lens_k), Hk, D), generator=g).to(dtype)
    v = torch.randn((sum(lens_k), Hk, D), generator=g).to(dtype)
    dout = torch.randn((sum(lens_q), H, D), generator=g).to(dtype)
    cuq = torch.tensor([0] + list(np.cumsum(lens_q)), dtype=torch.int32)
    cuk = torch.tensor([0] + list(np.cumsum(lens_k)), dtype=torch.int32)
    return q, k, v, dout, cuq, cuk


def _check_attention(fm, q, k, v, dout, cuq, cuk, co, cn, ind, lg_n, causal, scale=None, lg_m=128, check_grads=True):
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    max_q, max_k = int((cuq[1:] - cuq[:-1]).max()), int((cuk[1:] - cuk[:-1]).max())
    out, lse, _ = fm.api.flash_moba_attn_varlen_func(
        qg, kg, vg, cuq.cuda(), cuk.cuda(), max_q, max_k, co.cuda(), cn.cuda(), ind.cuda(),
        lg_m, lg_n, softmax_scale=scale, causal=causal, return_attn_probs=True)
    o_ref, lse_ref, dq_ref, dk_ref, dv_ref = O.attn_fwd_bwd(q, k, v, dout, cuq, cuk, co, cn, ind, lg_n, scale, causal)
    assert out.dtype == q.dtype and out.shape == q.shape
    assert lse.dtype == torch.float32 and lse.shape == (q.shape[1], q.shape[0])
    assert_close("out", out, o_ref, 2e-2, 1e-2)
    fin = torch.isfinite(lse_ref)
    assert torch.equal(torch.isfinite(lse.cpu()), fin)
    assert (lse.cpu()[~fin] == float("inf")).all()
    assert_close("lse", lse.cpu()[fin], lse_ref[fin], 2e-2, 1e-2)
    if check_grads:
        dq, dk, dv = torch.autograd.grad(out, (qg, kg, vg), dout.cuda())
        assert dq.dtype == q.dtype and dk.shape == k.shape and dv.shape == v.shape
        assert_close("dq", dq, dq_ref, 2e-2, 1e-2)
        assert_close("dk", dk, dk_ref, 2e-2 * max(1, q.shape[1] // k.shape[1]), 1e-2)
        assert_close("dv", dv, dv_ref, 2e-2 * max(1, q.shape[1] // k.shape[1]), 1e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("mha", ["mha", "gqa", "mqa"])
@pytest.mark.parametrize("d", [64, 128, 96, 59])
@pytest.mark.parametrize("sq,sk", [(113, 203), (128, 217), (256, 512), (512, 256), (1023, 1024)])
def test_attention_random_pattern(fm, sq, sk, d, mha, causal, dtype):
    H = 6
    Hk = {"mha": 6, "gqa": 2, "mqa": 1}[mha]
    # padded batch in the spirit of tests/test_moba_attn.py:103-104: lengths a little below the maximum
    rng = np.random.RandomState(sq + sk)
    lens_q = [max(1, sq - int(x)) for x in rng.randint(0, 20, 3)]
    lens_k = [max(1, sk - int(x)) for x in rng.randint(0, 20, 3)]
    q, k, v, dout, cuq, cuk = _attn_inputs(0, lens_q, lens_k, H, Hk, d, dtype)
    co, cn, ind = _random_csc(1, lens_q, lens_k, H, 64, 4, causal)
    _check_attention(fm, q, k, v, dout, cuq, cuk, co, cn, ind, 64, causal)


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("d,mha,dtype", [(64, "mha", torch.bfloat16), (128, "gqa", torch.bfloat16), (128, "mqa", torch.float16), (80, "mha", torch.float16)])
@pytest.mark.parametrize("sq,sk", [(1, 147), (113, 211), (108, 256), (1024, 1024), (1024, 1023), (2048, 2048), (4096, 4096)])
def test_attention_random_pattern_remaining_reference_shapes(fm, sq, sk, d, mha, causal, dtype):
    # the other shapes of tests/test_moba_attn.py:52-65; a batch whose longest query sequence has ONE row takes the
    # "max_seqlen_q == 1 => not causal" rule of csrc/flash_moba/flash_moba_api.cpp:450 (the oracle applies it too)
    big = max(sq, sk) >= 2048
    H = 4 if big else 6
    Hk = {"mha": H, "gqa": 2, "mqa": 1}[mha]
    rng = np.random.RandomState(sq * 3 + sk)
    nb = 2 if big else 3
    lens_q = [max(1, sq - int(x)) for x in rng.randint(0, 20, nb)]
    lens_k = [max(1, sk - int(x)) for x in rng.randint(0, 20, nb)]
    q, k, v, dout, cuq, cuk = _attn_inputs(sq, lens_q, lens_k, H, Hk, d, dtype)
    eff_causal = causal and max(lens_q) > 1
    co, cn, ind = _random_csc(4, lens_q, lens_k, H, 64, 4, eff_causal)
    _check_attention(fm, q, k, v, dout, cuq, cuk, co, cn, ind, 64, causal)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("mha", ["mha", "gqa"])
@pytest.mark.parametrize("d", [32, 80, 111, 160, 192, 224, 256])
@pytest.mark.parametrize("sq,sk", [(113, 203), (256, 512), (1023, 1024)])
def test_attention_random_pattern_more_head_dims(fm, sq, sk, d, mha, causal, dtype):
    # the rest of the head dimensions tests/test_moba_attn.py:48-49 sweeps (32 .. 256, odd ones padded to a multiple
    # of 8 by the interface); above 128 the forward runs its row-block form and the backward its feature-split kernels
    H = 4
    Hk = {"mha": 4, "gqa": 2}[mha]
    rng = np.random.RandomState(sq + sk + d)
    lens_q = [max(1, sq - int(x)) for x in rng.randint(0, 20, 2)]
    lens_k = [max(1, sk - int(x)) for x in rng.randint(0, 20, 2)]
    q, k, v, dout, cuq, cuk = _attn_inputs(d, lens_q, lens_k, H, Hk, d, dtype)
    co, cn, ind = _random_csc(3, lens_q, lens_k, H, 64, 4, causal)
    _check_attention(fm, q, k, v, dout, cuq, cuk, co, cn, ind, 64, causal)


def test_attention_head_dim_256_on_gated_patterns_with_wide_chunks(fm):
    # chunk 128 (two 64-key blocks per column) and the fused path at head dimension 256 / 192
    for d, chunk, topk in ((256, 128, 3), (192, 64, 5)):
        lens = [700, 130, 0, 1300]
        q, k, v, cu, dout = O.make_inputs(lens, 2, d, chunk, 23, torch.bfloat16, with_dout=True)
        qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
        out = fm.api.flash_moba_varlen_func(qg, kg, vg, cu.cuda(), cu.cuda(), max(lens), max(lens), chunk, topk, causal=True)
        out.backward(dout.cuda())
        co, cn, ind = fm.api.flash_topk_varlen_func(q.cuda(), k.cuda(), cu.cuda(), cu.cuda(), max(lens), max(lens), topk, chunk, causal=True)
        o_ref, _, dq_ref, dk_ref, dv_ref = O.attn_fwd_bwd(q, k, v, dout, cu, cu, co.cpu(), cn.cpu(), ind.cpu(), chunk, None, True)
        assert_close("out", out, o_ref, 2e-2, 1e-2)
        assert_close("dq", qg.grad, dq_ref, 2e-2, 1e-2)
        assert_close("dk", kg.grad, dk_ref, 2e-2, 1e-2)
        assert_close("dv", vg.grad, dv_ref, 2e-2, 1e-2)


@pytest.mark.parametrize("form", [1, 2])
@pytest.mark.parametrize("sq,sk,d,Hk,chunk,topk,causal,dtype", [
    (300, 300, 128, 4, 64, 3, True, torch.bfloat16),
    (1023, 1024, 128, 4, 64, 6, True, torch.bfloat16),
    (513, 700, 64, 2, 64, 4, True, torch.bfloat16),      # len_k > len_q, GQA
    (700, 513, 96, 1, 64, 4, True, torch.float16),       # len_q > len_k: leading rows see nothing; MQA; padded head dim
    (384, 640, 128, 4, 128, 2, True, torch.bfloat16),    # 128-key chunks: two 64-key steps per chunk
    (257, 390, 128, 4, 64, 3, False, torch.bfloat16),    # non-causal
    (129, 1, 64, 4, 64, 1, False, torch.float16),
])
def test_forward_both_forms(fm, form, sq, sk, d, Hk, chunk, topk, causal, dtype):
    # the library picks the forward form (columns / row blocks) by the density of the pattern; both are
    # checked here whatever it would pick
    H = 4
    rng = np.random.RandomState(sq * 7 + sk)
    lens_q = [max(1, sq - int(x)) for x in rng.randint(0, 150, 3)]
    lens_k = [max(1, sk - int(x)) for x in rng.randint(0, 150, 3)] if sk > 1 else [1, 1, 1]
    q, k, v, dout, cuq, cuk = _attn_inputs(5, lens_q, lens_k, H, Hk, d, dtype)
    co, cn, ind = _random_csc(2, lens_q, lens_k, H, chunk, topk, causal)
    scale = d ** -0.5
    dp = (8 - d % 8) % 8
    pad = (lambda t: torch.nn.functional.pad(t, (0, dp))) if dp else (lambda t: t)
    out, lse, _, _ = fm.hip.moba_varlen_fwd(pad(q).cuda(), pad(k).cuda(), pad(v).cuda(), None, co.cuda(), cn.cuda(), ind.cuda(),
                                            cuq.cuda(), cuk.cuda(), None, None, None, max(lens_q), max(lens_k), 0.0, scale,
                                            False, causal, 0.0, False, 128, chunk, None, _fwd_mode=form)
    o_ref, lse_ref, _, _, _ = O.attn_fwd_bwd(q, k, v, dout, cuq, cuk, co, cn, ind, chunk, scale, causal)
    assert_close("out", out[..., :d], o_ref, 2e-2, 1e-2)
    fin = torch.isfinite(lse_ref)
    assert torch.equal(torch.isfinite(lse.cpu()), fin)
    assert (lse.cpu()[~fin] == float("inf")).all()
    assert_close("lse", lse.cpu()[fin], lse_ref[fin], 2e-2, 1e-2)
    out2, lse2, _, _ = fm.hip.moba_varlen_fwd(pad(q).cuda(), pad(k).cuda(), pad(v).cuda(), None, co.cuda(), cn.cuda(), ind.cuda(),
                                              cuq.cuda(), cuk.cuda(), None, None, None, max(lens_q), max(lens_k), 0.0, scale,
                                              False, causal, 0.0, False, 128, chunk, None, _fwd_mode=form)
    assert torch.equal(out, out2) and torch.equal(lse, lse2)


def test_autograd_function_checks_a_callers_visit_bound(fm):
    # FlashMobaAttnVarlenFunc takes an optional bound on a row's visits; one that is too small for the caller's own
    # pattern would drop visits, so eager calls check it against the pattern
    lens = [700, 300]
    q, k, v, dout, cuq, cuk = _attn_inputs(2, lens, lens, 2, 2, 64, torch.bfloat16)
    co, cn, ind = _random_csc(5, lens, lens, 2, 64, 4, True)
    args = (q.cuda(), k.cuda(), v.cuda(), cuq.cuda(), cuk.cuda(), 700, 700, co.cuda(), cn.cuda(), ind.cuda(), 128, 64,
            0.0, None, True, 0.0, None, False, False, False)
    ref = fm.iface.FlashMobaAttnVarlenFunc.apply(*args)
    assert torch.equal(fm.iface.FlashMobaAttnVarlenFunc.apply(*args, 4), ref)
    with pytest.raises(RuntimeError, match="max_visits = 2, but a row of the pattern has 4"):
        fm.iface.FlashMobaAttnVarlenFunc.apply(*args, 2)


@pytest.mark.parametrize("lens,chunk,topk,Hk", [([640, 1, 0, 1300], 64, 6, 4), ([2100, 900], 128, 5, 2), ([300 * 64 + 17], 64, 33, 1)])
def test_fused_path_hands_the_gating_selection_to_the_forward(fm, lens, chunk, topk, Hk):
    # flash_moba_varlen_func passes the gating's selection bits on; the attention entry point alone derives them from
    # the lists: same bits, same result
    H, D = 4, 128
    g = torch.Generator().manual_seed(9)
    T = sum(lens)
    q = torch.randn((T, H, D), generator=g).to(torch.bfloat16).cuda()
    k = torch.randn((T, Hk, D), generator=g).to(torch.bfloat16).cuda()
    v = torch.randn((T, Hk, D), generator=g).to(torch.bfloat16).cuda()
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32).cuda()
    out = fm.api.flash_moba_varlen_func(q, k, v, cu, cu, max(lens), max(lens), chunk, topk, causal=True)
    assert fm.hip.last_fwd_row_blocks() == 1
    co, cn, ind = fm.api.flash_topk_varlen_func(q, k, cu, cu, max(lens), max(lens), topk, chunk, causal=True)
    lg_m = fm.iface.decide_lg_block_m(topk, chunk, max(lens), True)
    out2 = fm.api.flash_moba_attn_varlen_func(q, k, v, cu, cu, max(lens), max(lens), co, cn, ind, lg_m, chunk, causal=True)
    assert fm.hip.last_fwd_row_blocks() == 1
    assert torch.equal(out, out2)


def test_row_block_forms_over_many_columns(fm):
    # more than 32 chunks (several selection words per row) in the forward, more than 256 columns (several column
    # batches per row block) in the row-block dQ pass
    lens = [300 * 64 + 40, 2500]
    H, D, chunk, topk = 2, 64, 64, 5
    q, k, v, cu, dout = O.make_inputs(lens, H, D, chunk, 41, torch.bfloat16, with_dout=True)
    Q, K, V, CU, DO = q.cuda(), k.cuda(), v.cuda(), cu.cuda(), dout.cuda()
    co, cn, ind = fm.api.flash_topk_varlen_func(Q, K, CU, CU, max(lens), max(lens), topk, chunk, causal=True)
    scale = D ** -0.5
    out, lse, _, _ = fm.hip.moba_varlen_fwd(Q, K, V, None, co, cn, ind, CU, CU, None, None, None, max(lens), max(lens), 0.0, scale,
                                            False, True, 0.0, False, 128, chunk, None, _fwd_mode=2)
    assert fm.hip.last_fwd_row_blocks() == 1
    dq, dk, dv, _ = fm.hip.moba_varlen_bwd(DO, Q, K, V, out, lse, None, None, None, co, cn, ind, CU, CU, None, max(lens), max(lens),
                                           0.0, scale, False, True, 0.0, False, 128, chunk, None, None, _dq_mode=1)
    assert fm.hip.last_bwd_partials() == 0
    # the column form / the partials form of the same call as the reference: they are checked against the oracle elsewhere
    out1, lse1, _, _ = fm.hip.moba_varlen_fwd(Q, K, V, None, co, cn, ind, CU, CU, None, None, None, max(lens), max(lens), 0.0, scale,
                                              False, True, 0.0, False, 128, chunk, None, _fwd_mode=1)
    dq2, dk2, dv2, _ = fm.hip.moba_varlen_bwd(DO, Q, K, V, out, lse, None, None, None, co, cn, ind, CU, CU, None, max(lens), max(lens),
                                              0.0, scale, False, True, 0.0, False, 128, chunk, None, None, _dq_mode=2)
    assert_close("out", out, out1.float().cpu(), 2e-2, 1e-2)
    assert_close("lse", lse, lse1.float().cpu(), 2e-2, 1e-2)
    assert_close("dq", dq, dq2.float().cpu(), 2e-2, 1e-2)
    assert torch.equal(dk, dk2) and torch.equal(dv, dv2)


@pytest.mark.parametrize("dq_mode", [1, 2])
# (128, 128), (96, 128), (128, 256): columns of a multiple of 128 keys with head_dim > 64, where the dK/dV pass works
# on 128-key blocks (one or two per column; 96: a wave without features of its own in the dQ products)
@pytest.mark.parametrize("d,chunk", [(128, 64), (64, 128), (96, 64), (128, 128), (96, 128), (128, 256)])
def test_backward_both_dq_forms(fm, dq_mode, d, chunk):
    # the library picks the dQ form by shape; both are checked here whatever it would pick
    lens = [300, 0, 77, 650]
    q, k, v, cu, dout = O.make_inputs(lens, 4, d, chunk, 33, torch.bfloat16, with_dout=True)
    Q, K, V, CU, DO = q.cuda(), k.cuda(), v.cuda(), cu.cuda(), dout.cuda()
    co, cn, ind = fm.api.flash_topk_varlen_func(Q, K, CU, CU, max(lens), max(lens), 3, chunk, causal=True)
    scale = d ** -0.5
    out, lse, _, _ = fm.hip.moba_varlen_fwd(Q, K, V, None, co, cn, ind, CU, CU, None, None, None, max(lens), max(lens), 0.0, scale,
                                            False, True, 0.0, False, 128, chunk, None)
    dq, dk, dv, _ = fm.hip.moba_varlen_bwd(DO, Q, K, V, out, lse, None, None, None, co, cn, ind, CU, CU, None, max(lens), max(lens),
                                           0.0, scale, False, True, 0.0, False, 128, chunk, None, None, _dq_mode=dq_mode)
    _, _, dq_ref, dk_ref, dv_ref = O.attn_fwd_bwd(q, k, v, dout, cu, cu, co.cpu(), cn.cpu(), ind.cpu(), chunk, None, True)
    assert_close("dq", dq, dq_ref, 2e-2, 1e-2)
    assert_close("dk", dk, dk_ref, 2e-2, 1e-2)
    assert_close("dv", dv, dv_ref, 2e-2, 1e-2)
    # no floating-point atomics in either form: a second run gives the same bits
    dq2, dk2, dv2, _ = fm.hip.moba_varlen_bwd(DO, Q, K, V, out, lse, None, None, None, co, cn, ind, CU, CU, None, max(lens), max(lens),
                                              0.0, scale, False, True, 0.0, False, 128, chunk, None, None, _dq_mode=dq_mode)
    assert torch.equal(dq, dq2) and torch.equal(dk, dk2) and torch.equal(dv, dv2)


@pytest.mark.parametrize("d,chunk", [(128, 64), (64, 64), (128, 128)])
@pytest.mark.parametrize("dq_mode", [1, 2])
def test_backward_with_rows_far_apart(fm, dq_mode, d, chunk):
    # The dK/dV pass fetches the rows of a list with a 32-bit byte offset per lane where a sequence's rows lie within
    # 4 GB of its first one, and with 64-bit addresses otherwise (a kernel form of its own, chosen by the host, for
    # each head dimension and key-block width): q and dout as views with a row stride of 2^22 elements (8 MB) take the
    # second way and must give the bits of the packed tensors.
    lens = [200, 90] if chunk == 64 else [300, 140]
    heads = 2
    q, k, v, cu, dout = O.make_inputs(lens, heads, d, chunk, 35, torch.bfloat16, with_dout=True)
    Q, K, V, CU, DO = q.cuda(), k.cuda(), v.cuda(), cu.cuda(), dout.cuda()
    co, cn, ind = fm.api.flash_topk_varlen_func(Q, K, CU, CU, max(lens), max(lens), 2, chunk, causal=True)
    scale = d ** -0.5
    out, lse, _, _ = fm.hip.moba_varlen_fwd(Q, K, V, None, co, cn, ind, CU, CU, None, None, None, max(lens), max(lens), 0.0, scale,
                                            False, True, 0.0, False, 128, chunk, None)
    ref = fm.hip.moba_varlen_bwd(DO, Q, K, V, out, lse, None, None, None, co, cn, ind, CU, CU, None, max(lens), max(lens),
                                 0.0, scale, False, True, 0.0, False, 128, chunk, None, None, _dq_mode=dq_mode)[:3]
    total = sum(lens)
    wide = 1 << 22

    def far_apart(t):
        big = torch.zeros((total, wide), dtype=t.dtype, device=t.device)
        view = big[:, :heads * d].view(total, heads, d)
        view.copy_(t)
        assert view.stride(0) == wide and view.stride(1) == d
        return view

    got = fm.hip.moba_varlen_bwd(far_apart(DO), far_apart(Q), K, V, out, lse, None, None, None, co, cn, ind, CU, CU, None,
                                 max(lens), max(lens), 0.0, scale, False, True, 0.0, False, 128, chunk, None, None, _dq_mode=dq_mode)[:3]
    for name, x, y in zip(("dq", "dk", "dv"), ref, got):
        assert torch.equal(x, y), name


@pytest.mark.parametrize("chunk,topk,visits", [(64, 40, 40), (128, 24, 24), (256, 10, 20)])
def test_partial_forms_are_bitwise_repeatable_beyond_16_visits_per_row(fm, chunk, topk, visits):
    # Column forward and partial-sum dQ hand out a row's partial slots from a counter, in whatever order the
    # workgroups arrive; the merge must not depend on it: ranks are taken over ALL of a row's visits (here 20 to 40
    # per row, more than one batch of 16), so repeated runs give the same bits, and both agree with the oracle.
    lens = [chunk * 50 + 17, 900]
    q, k, v, cu, dout = O.make_inputs(lens, 4, 128, chunk, 62, torch.bfloat16, with_dout=True)
    Q, K, V, CU, DO = q.cuda(), k.cuda(), v.cuda(), cu.cuda(), dout.cuda()
    co, cn, ind = fm.api.flash_topk_varlen_func(Q, K, CU, CU, max(lens), max(lens), topk, chunk, causal=True)
    scale = 128 ** -0.5
    runs = []
    for _ in range(3):  # (no hints: the visit bounds are counted from the pattern)
        out, lse, _, _ = fm.hip.moba_varlen_fwd(Q, K, V, None, co, cn, ind, CU, CU, None, None, None, max(lens), max(lens), 0.0, scale,
                                                False, True, 0.0, False, 128, chunk, None, _fwd_mode=1)
        assert fm.hip.last_fwd_row_blocks() == 0 and fm.hip.last_fwd_visits() == visits
        dq, dk, dv, _ = fm.hip.moba_varlen_bwd(DO, Q, K, V, out, lse, None, None, None, co, cn, ind, CU, CU, None, max(lens), max(lens),
                                               0.0, scale, False, True, 0.0, False, 128, chunk, None, None, _dq_mode=2)
        assert fm.hip.last_bwd_partials() == 1
        runs.append((out, lse, dq, dk, dv))
    for other in runs[1:]:
        for x, y in zip(runs[0], other):
            assert torch.equal(x, y)
    o_ref, _, dq_ref, dk_ref, dv_ref = O.attn_fwd_bwd(q, k, v, dout, cu, cu, co.cpu(), cn.cpu(), ind.cpu(), chunk, None, True)
    assert_close("out", runs[0][0], o_ref, 2e-2, 1e-2)
    assert_close("dq", runs[0][2], dq_ref, 2e-2, 1e-2)
    assert_close("dk", runs[0][3], dk_ref, 2e-2, 1e-2)
    assert_close("dv", runs[0][4], dv_ref, 2e-2, 1e-2)


@pytest.mark.parametrize("chunk,topk", [(64, 4), (128, 3), (64, 32)])
def test_attention_on_gated_pattern(fm, chunk, topk):
    lens = [640, 1, 0, 1300]
    q, k, v, cu, dout = O.make_inputs(lens, 4, 128, chunk, 21, torch.bfloat16, with_dout=True)
    co, cn, ind = fm.api.flash_topk_varlen_func(q.cuda(), k.cuda(), cu.cuda(), cu.cuda(), max(lens), max(lens), topk, chunk, causal=True)
    _check_attention(fm, q, k, v, dout, cu, cu, co.cpu(), cn.cpu(), ind.cpu(), chunk, True, lg_m=256)


def test_attention_dense_special_case_matches_sdpa(fm):
    # top-k >= number of chunks: plain causal attention
    L, H, D, chunk = 512, 2, 128, 64
    q, k, v, cu = O.make_inputs([L], H, D, chunk, 3, torch.bfloat16)
    out = fm.api.flash_moba_varlen_func(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), cu.cuda(), L, L, chunk, 16, causal=True)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.float().transpose(0, 1), k.float().transpose(0, 1), v.float().transpose(0, 1), is_causal=True).transpose(0, 1)
    assert_close("out", out, ref, 2e-2, 1e-2)


def test_attention_rows_without_keys_and_no_keys_at_all(fm):
    # len_q > len_k, causal: leading rows see nothing -> out 0, lse +inf, zero gradients
    q, k, v, dout, cuq, cuk = _attn_inputs(4, [200], [130], 2, 2, 64, torch.bfloat16)
    co, cn, ind = fm.api.flash_topk_varlen_func(q.cuda(), k.cuda(), cuq.cuda(), cuk.cuda(), 200, 130, 2, 64, causal=True)
    _check_attention(fm, q, k, v, dout, cuq, cuk, co.cpu(), cn.cpu(), ind.cpu(), 64, True)
    z = torch.zeros(2, dtype=torch.int32).cuda()
    out, lse, _, _ = fm.hip.moba_varlen_fwd(
        q.cuda(), k[:0].cuda(), v[:0].cuda(), None, torch.zeros((1, 2, 0), dtype=torch.int64).cuda(),
        torch.zeros((1, 2, 0), dtype=torch.int32).cuda(), torch.zeros((0,), dtype=torch.int32).cuda(), cuq.cuda(), z,
        None, None, None, 200, 0, 0.0, 0.125, False, True, 0.0, False, 128, 64, None)
    assert (out == 0).all() and (lse == float("inf")).all()


def test_a_visits_bound_that_is_too_small_is_reported(fm):
    # a caller's own bound on a row's visits sizes the partial-result buffers; visits beyond it are dropped, and the
    # optional status word then holds the largest visit count seen (0 when the bound held)
    lens = [900]
    q, k, v, cu, dout = O.make_inputs(lens, 2, 128, 64, 13, torch.bfloat16, with_dout=True)
    Q, K, V, CU, DO = q.cuda(), k.cuda(), v.cuda(), cu.cuda(), dout.cuda()
    co, cn, ind = fm.api.flash_topk_varlen_func(Q, K, CU, CU, 900, 900, 6, 64, causal=True)
    for bound, want in ((6, 0), (4, 6)):
        st = torch.zeros(2, dtype=torch.int32, device="cuda")
        out, lse, _, _ = fm.hip.moba_varlen_fwd(Q, K, V, None, co, cn, ind, CU, CU, None, None, None, 900, 900, 0.0, 128 ** -0.5, False, True,
                                                0.0, False, 128, 64, None, _fwd_mode=1, _max_visits=bound, _overflow=st[0:1])
        fm.hip.moba_varlen_bwd(DO, Q, K, V, out, lse, None, None, None, co, cn, ind, CU, CU, None, 900, 900, 0.0, 128 ** -0.5, False, True,
                               0.0, False, 128, 64, None, None, _dq_mode=2, _max_visits=bound, _overflow=st[1:2])
        assert st.tolist() == [want, want]


def test_attention_rejects_unsupported_options(fm):
    q, k, v, dout, cuq, cuk = _attn_inputs(4, [128], [128], 2, 2, 64, torch.bfloat16)
    co, cn, ind = _random_csc(1, [128], [128], 2, 64, 2, True)
    args = [t.cuda() for t in (q, k, v, cuq, cuk)] + [128, 128] + [t.cuda() for t in (co, cn, ind)]
    with pytest.raises(RuntimeError, match="dropout"):
        fm.api.flash_moba_attn_varlen_func(*args, 128, 64, dropout_p=0.1)
    with pytest.raises(RuntimeError, match="softcap"):
        fm.api.flash_moba_attn_varlen_func(*args, 128, 64, softcap=30.0)
    with pytest.raises(RuntimeError, match="ALiBi"):
        fm.api.flash_moba_attn_varlen_func(*args, 128, 64, alibi_slopes=torch.ones(2).cuda())
    with pytest.raises(RuntimeError, match="m_lg_block_dim"):
        fm.api.flash_moba_attn_varlen_func(*args, 64, 64)
    with pytest.raises(RuntimeError, match="n_lg_block_dim"):
        fm.api.flash_moba_attn_varlen_func(*args, 128, 32)
    with pytest.raises(RuntimeError, match="int64"):
        fm.api.flash_moba_attn_varlen_func(*args[:7], co.int().cuda(), cn.cuda(), ind.cuda(), 128, 64)


# ------------------------------------------------------------------------ end to end
def test_end_to_end_config1_shape_against_dense_reference(fm):
    # BASELINE config 1 (lengths [1024, 2048], 8 heads, d=64, chunk 128, top-k 4) evaluated by the HIP
    # path in bf16 against the CPU reference path in fp32 on the same (bf16-rounded) inputs
    lens = [1024, 2048]
    q, k, v, cu = O.make_inputs(lens, 8, 64, 128, 1001, torch.bfloat16)
    out = fm.api.flash_moba_varlen_func(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), cu.cuda(), 2048, 2048, 128, 4, causal=True)
    ref = O.moba_dense_ref(q.float(), k.float(), v.float(), cu, cu, 128, 4, True)
    # gating uses bf16-rounded chunk means; a near-tie may flip a chunk for a few rows
    err = (out.float().cpu() - ref).abs()
    bad_rows = (err > 2e-2 + 1e-2 * ref.abs()).any(-1)
    assert bad_rows.float().mean().item() < 0.005


def test_end_to_end_backward_runs_through_autograd(fm):
    lens = [512, 384]
    q, k, v, cu, dout = O.make_inputs(lens, 4, 128, 64, 77, torch.bfloat16, with_dout=True)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    out = fm.api.flash_moba_varlen_func(qg, kg, vg, cu.cuda(), cu.cuda(), 512, 512, 64, 3, causal=True)
    out.backward(dout.cuda())
    co, cn, ind = fm.api.flash_topk_varlen_func(q.cuda(), k.cuda(), cu.cuda(), cu.cuda(), 512, 512, 3, 64, causal=True)
    _, _, dq_ref, dk_ref, dv_ref = O.attn_fwd_bwd(q, k, v, dout, cu, cu, co.cpu(), cn.cpu(), ind.cpu(), 64, None, True)
    assert_close("dq", qg.grad, dq_ref, 2e-2, 1e-2)
    assert_close("dk", kg.grad, dk_ref, 2e-2, 1e-2)
    assert_close("dv", vg.grad, dv_ref, 2e-2, 1e-2)

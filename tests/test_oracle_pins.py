"""Pins the CPU oracle (oracle/moba_oracle.py) against closed forms, library routines,
brute force and independent formulations, so that a plausible mistake (dropped term,
wrong sign or index, transposed operand) fails at least one check."""
import math

import numpy as np
import pytest
import torch

from oracle import moba_oracle as O


# ------------------------------------------------------------------ mean-pool
def test_mean_pool_constant_keys_is_identity():
    cu = torch.tensor([0, 70, 70, 200], dtype=torch.int32)
    row = torch.randn(3, 16)
    k = row[None].expand(200, 3, 16).contiguous().to(torch.bfloat16)
    km, cu_km = O.mean_pool(k, cu, 32)
    assert cu_km.tolist() == [0, 3, 3, 8] and cu_km.dtype == torch.int32
    assert km.shape == (8, 3, 16)
    assert torch.equal(km, k[:8])


def test_mean_pool_chunk_one_is_copy():
    k = torch.randn(37, 2, 8).to(torch.float16)
    cu = torch.tensor([0, 10, 37], dtype=torch.int32)
    km, cu_km = O.mean_pool(k, cu, 1)
    assert torch.equal(km, k) and cu_km.tolist() == [0, 10, 37]


def test_mean_pool_tail_divides_by_real_length_and_matches_f64():
    torch.manual_seed(1)
    k = torch.randn(100, 2, 8)
    cu = torch.tensor([0, 100], dtype=torch.int32)
    km, _ = O.mean_pool(k, cu, 64)
    ref0 = k[:64].double().mean(0)
    ref1 = k[64:100].double().sum(0) / 36.0
    assert torch.allclose(km[0].double(), ref0, atol=1e-6)
    assert torch.allclose(km[1].double(), ref1, atol=1e-6)
    # a wrong divisor (64 instead of 36) would be off by a factor 0.5625
    assert not torch.allclose(km[1].double(), k[64:100].double().sum(0) / 64.0, atol=1e-3)


def test_mean_pool_pool_larger_than_seq_and_empty():
    k = torch.randn(5, 1, 8)
    km, cu_km = O.mean_pool(k, torch.tensor([0, 0, 5], dtype=torch.int32), 256)
    assert km.shape == (1, 1, 8) and cu_km.tolist() == [0, 0, 1]
    assert torch.allclose(km[0], k.mean(0), atol=1e-6)
    km, cu_km = O.mean_pool(torch.zeros(0, 2, 8), torch.tensor([0, 0, 0], dtype=torch.int32), 16)
    assert km.shape == (0, 2, 8) and cu_km.tolist() == [0, 0, 0]


# ------------------------------------------------------------------ gating / top-k
def _rand_case(seed, lens_q, lens_k, H, Hk, D, integer=False, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    Tq, Tk = sum(lens_q), sum(lens_k)
    if integer:  # integer-valued operands: scores tie exactly and are exact in fp32
        q = torch.randint(-2, 3, (Tq, H, D), generator=g).to(dtype)
        k = torch.randint(-1, 2, (Tk, Hk, D), generator=g).to(dtype)
    else:
        q = torch.randn((Tq, H, D), generator=g).to(dtype)
        k = torch.randn((Tk, Hk, D), generator=g).to(dtype)
    cuq = torch.tensor([0] + list(np.cumsum(lens_q)), dtype=torch.int32)
    cuk = torch.tensor([0] + list(np.cumsum(lens_k)), dtype=torch.int32)
    return q, k, cuq, cuk


@pytest.mark.parametrize("integer", [False, True])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("topk,chunk", [(1, 4), (3, 4), (4, 8), (8, 4), (17, 2)])
def test_topk_three_formulations_agree(integer, causal, topk, chunk):
    q, k, cuq, cuk = _rand_case(3 + topk, [37, 0, 64], [37, 0, 64], 2, 1, 8, integer)
    km, cu_km = O.mean_pool(k, cuk, chunk)
    if integer:
        # keep km integer-valued too: use chunk sums instead of means (still a valid km input)
        km = (km.float() * chunk).round().to(k.dtype)
    i1, v1 = O.fused_topk(q, km, cuq, cuk, cu_km, topk, chunk, causal)
    i2, v2 = O.fused_topk_literal(q, km, cuq, cuk, cu_km, topk, chunk, causal)
    assert torch.equal(i1, i2)
    assert torch.equal(v1, v2)
    if integer:
        # ties must exist for the test to bite
        fin = torch.isfinite(v1)
        if topk >= 3:
            assert (v1[..., :-1][fin[..., 1:] & fin[..., :-1]] == v1[..., 1:][fin[..., 1:] & fin[..., :-1]]).any()
        # among equal finite scores the higher chunk index comes first
        same = (v1[..., :-1] == v1[..., 1:]) & fin[..., 1:] & fin[..., :-1]
        assert (i1[..., :-1][same] > i1[..., 1:][same]).all()


def test_topk_invariants_causal_with_offset():
    # len_q != len_k: bottom-right aligned; rows with r + off < 0 select nothing
    q, k, cuq, cuk = _rand_case(11, [20, 9], [12, 30], 2, 2, 8)
    chunk, topk = 4, 3
    km, cu_km = O.mean_pool(k, cuk, chunk)
    idx, val = O.fused_topk(q, km, cuq, cuk, cu_km, topk, chunk, True)
    assert idx.shape == (29, 2, 16)
    for b, (Lq, Lk) in enumerate([(20, 12), (9, 30)]):
        off = Lk - Lq
        for r in range(Lq):
            row = idx[int(cuq[b]) + r]
            for h in range(2):
                sel = row[h][row[h] >= 0].tolist()
                s = r + off
                if s < 0:
                    assert sel == []
                    continue
                p = s // chunk
                assert row[h, 0].item() == p                  # slot 0 = own chunk
                assert len(sel) == min(topk, p + 1)           # min(k, visible chunks)
                assert all(c <= p for c in sel) and len(set(sel)) == len(sel)
    assert (idx[..., topk:] == -1).all() and torch.isinf(val[..., topk:]).all()


def test_topk_matches_bruteforce_selection_set():
    q, k, cuq, cuk = _rand_case(5, [50], [50], 1, 1, 16, dtype=torch.float32)
    chunk, topk = 5, 4
    km, cu_km = O.mean_pool(k, cuk, chunk)
    idx, _ = O.fused_topk(q, km, cuq, cuk, cu_km, topk, chunk, True)
    gate = (q[:, 0].double() @ km[:, 0].double().T)
    for r in range(50):
        p = r // chunk
        cands = sorted(range(p), key=lambda c: (-gate[r, c].item(), -c))[: topk - 1]
        assert set(idx[r, 0][idx[r, 0] >= 0].tolist()) == set(cands) | {p}


# ------------------------------------------------------------------ CSC + sort
def test_csc_matches_rowwalk_and_invariants():
    q, k, cuq, cuk = _rand_case(7, [33, 0, 48], [33, 0, 48], 3, 1, 8)
    chunk, topk = 4, 3
    km, cu_km = O.mean_pool(k, cuk, chunk)
    idx, _ = O.fused_topk(q, km, cuq, cuk, cu_km, topk, chunk, True)
    maxC = (48 + chunk - 1) // chunk
    co, cn, flat = O.csc_from_topk(idx, cuq, topk, maxC)
    flat2, cn2 = O.csc_from_topk_rowwalk(idx, cuq, topk, co)
    assert torch.equal(flat, flat2) and torch.equal(cn, cn2)
    assert co.dtype == torch.int64 and cn.dtype == torch.int32 and flat.dtype == torch.int32
    assert flat.numel() == 81 * 3 * topk
    assert int(cn.sum()) == int((idx[..., :topk] >= 0).sum())
    lens = [33, 0, 48]
    for b in range(3):
        for h in range(3):
            base = (int(cuq[b]) * 3 + lens[b] * h) * topk
            assert co[b, h, 0] == base
            ends = co[b, h] + cn[b, h]
            assert (co[b, h, 1:] == ends[:-1]).all()
            assert ends[-1] <= base + lens[b] * topk
            for c in range(maxC):
                seg = flat[int(co[b, h, c]):int(ends[c])]
                assert (seg[1:] > seg[:-1]).all()
                assert (seg >= 0).all() and (seg < max(lens[b], 1)).all()
            # columns past the sequence's own chunk count are empty
            assert (cn[b, h, (lens[b] + chunk - 1) // chunk:] == 0).all()


def test_varlen_sort_library_and_extremes():
    g = torch.Generator().manual_seed(3)
    lens = torch.randint(0, 50, (17,), generator=g)
    ends = torch.cumsum(lens, 0).to(torch.int64)
    starts = ends - lens
    src = torch.randint(-2 ** 31, 2 ** 31 - 1, (int(ends[-1]),), generator=g, dtype=torch.int64).to(torch.int32)
    out = O.varlen_sort(starts, ends, src)
    for s, e in zip(starts.tolist(), ends.tolist()):
        assert torch.equal(out[s:e], torch.sort(src[s:e])[0])
    vals = torch.tensor([2 ** 31 - 1, -2 ** 31] * 8, dtype=torch.int32)
    out = O.varlen_sort(torch.tensor([0, 8]), torch.tensor([8, 12]), vals)
    assert out[:4].tolist() == [-2 ** 31] * 4 and out[4:8].tolist() == [2 ** 31 - 1] * 4
    assert out[12:].tolist() == [0, 0, 0, 0]        # zeros outside every segment


# ------------------------------------------------------------------ attention
def _pattern(seed, lens, H, Hk, D, chunk, topk, causal=True, dtype=torch.float32):
    q, k, v, cu = O.make_inputs(lens, H, D, chunk, seed, dtype, Hk)
    co, cn, ind = O.flash_topk_ref(q, k, cu, cu, max(lens), max(lens), topk, chunk, causal)
    return q, k, v, cu, co, cn, ind


def test_attention_topk_covers_everything_equals_dense_causal_sdpa():
    lens, H, D, chunk = [96, 40], 2, 16, 8
    q, k, v, cu, co, cn, ind = _pattern(1, lens, H, H, D, chunk, topk=64)
    out, lse = O.attn_fwd(q, k, v, cu, cu, co, cn, ind, chunk, None, True)
    for b, L in enumerate(lens):
        s = int(cu[b])
        ref = torch.nn.functional.scaled_dot_product_attention(
            q[s:s + L].transpose(0, 1), k[s:s + L].transpose(0, 1), v[s:s + L].transpose(0, 1), is_causal=True)
        assert torch.allclose(out[s:s + L].transpose(0, 1), ref, atol=2e-5, rtol=1e-5)
        sc = torch.einsum("hqd,hkd->hqk", q[s:s + L].transpose(0, 1), k[s:s + L].transpose(0, 1)) / math.sqrt(D)
        sc = sc.masked_fill(~torch.ones(L, L, dtype=torch.bool).tril(), float("-inf"))
        assert torch.allclose(lse[:, s:s + L], torch.logsumexp(sc, -1), atol=2e-5)


def test_attention_topk1_is_block_diagonal_causal():
    lens, H, D, chunk = [50], 1, 8, 8
    q, k, v, cu, co, cn, ind = _pattern(2, lens, H, H, D, chunk, topk=1)
    out, _ = O.attn_fwd(q, k, v, cu, cu, co, cn, ind, chunk, None, True)
    for r in range(50):
        lo = (r // chunk) * chunk
        w = torch.softmax((q[r, 0] @ k[lo:r + 1, 0].T) / math.sqrt(D), -1)
        assert torch.allclose(out[r, 0], w @ v[lo:r + 1, 0], atol=1e-5)


def test_attention_csc_path_equals_independent_dense_mask_path():
    lens, H, Hk, D, chunk, topk = [80, 33], 4, 2, 16, 8, 3
    q, k, v, cu, co, cn, ind = _pattern(3, lens, H, Hk, D, chunk, topk)
    out, _ = O.attn_fwd(q, k, v, cu, cu, co, cn, ind, chunk, None, True)
    out2 = O.moba_dense_ref(q, k, v, cu, cu, chunk, topk, True, row_block=32)
    assert torch.allclose(out, out2, atol=1e-5)
    # sparsity is real: differs from dense causal attention
    dense = O.moba_dense_ref(q, k, v, cu, cu, chunk, 64, True)
    assert (out - dense).abs().max() > 1e-3


def test_attention_empty_rows_and_noncausal_offsets():
    # len_q > len_k, causal: the first rows see no key -> out 0, lse +inf
    g = torch.Generator().manual_seed(4)
    q = torch.randn(12, 1, 8, generator=g); k = torch.randn(8, 1, 8, generator=g); v = torch.randn(8, 1, 8, generator=g)
    cuq = torch.tensor([0, 12], dtype=torch.int32); cuk = torch.tensor([0, 8], dtype=torch.int32)
    co, cn, ind = O.flash_topk_ref(q, k, cuq, cuk, 12, 8, 2, 4, True)
    out, lse = O.attn_fwd(q, k, v, cuq, cuk, co, cn, ind, 4, None, True)
    assert torch.isinf(lse[0, :4]).all() and (lse[0, :4] > 0).all() and (out[:4] == 0).all()
    assert torch.isfinite(lse[0, 4:]).all()
    # row 4 (r + off = 0) sees exactly key 0
    assert torch.allclose(out[4, 0], v[0, 0], atol=1e-6)


def test_attention_backward_gradcheck_f64():
    lens, H, Hk, D, chunk, topk = [24], 2, 1, 4, 4, 2
    q, k, v, cu, co, cn, ind = _pattern(5, lens, H, Hk, D, chunk, topk, dtype=torch.float64)

    def f(q_, k_, v_):
        return O.attn_fwd(q_, k_, v_, cu, cu, co, cn, ind, chunk, 0.37, True, dtype=torch.float64)[0]

    q.requires_grad_(True); k.requires_grad_(True); v.requires_grad_(True)
    assert torch.autograd.gradcheck(f, (q, k, v), eps=1e-6, atol=1e-5)


def test_attention_backward_matches_closed_form():
    # dV = P^T dO, dS = P*(dP - delta), dQ = scale dS K, dK = scale dS^T Q  (flash_bwd_kernel.h:627-686,812)
    lens, H, D, chunk, topk = [40], 1, 8, 8, 2
    q, k, v, cu, co, cn, ind = _pattern(6, lens, H, H, D, chunk, topk)
    g = torch.Generator().manual_seed(9)
    dout = torch.randn(q.shape, generator=g)
    out, lse, dq, dk, dv = O.attn_fwd_bwd(q, k, v, dout, cu, cu, co, cn, ind, chunk, None, True)
    scale = D ** -0.5
    bm = O.csc_to_block_mask(co, cn, ind, 0, 0, 40, 5)
    tm = O.token_mask(bm, chunk, 40, 40, True)
    S = (q[:, 0] @ k[:, 0].T) * scale
    P = torch.where(tm, torch.exp(S - lse[0][:, None]), torch.zeros(()))
    delta = (dout[:, 0] * out[:, 0]).sum(-1)
    dP = dout[:, 0] @ v[:, 0].T
    dS = P * (dP - delta[:, None])
    assert torch.allclose(dv[:, 0], P.T @ dout[:, 0], atol=1e-5)
    assert torch.allclose(dq[:, 0], scale * dS @ k[:, 0], atol=1e-5)
    assert torch.allclose(dk[:, 0], scale * dS.T @ q[:, 0], atol=1e-5)


def test_decide_lg_block_m_table():
    assert O.decide_lg_block_m(4, 128, 2048, True) == 256
    assert O.decide_lg_block_m(8, 128, 8192, True) == 512
    assert O.decide_lg_block_m(16, 128, 32768, True) == 768
    assert O.decide_lg_block_m(16, 128, 262144, True) == 1024
    assert O.decide_lg_block_m(8, 64, 1024, False) == 128


def test_headline_seqlens_and_pairs_formula():
    lens = O.headline_seqlens()
    assert sum(lens) == 65536 and len(lens) == 8 and all(l % 64 == 0 for l in lens)
    # pairs closed form for one causal sequence of C full chunks
    C, B, kk, H = 12, 8, 4, 2
    q, k, v, cu, co, cn, ind = _pattern(8, [C * B], H, H, 8, B, kk)
    pairs = O.count_pairs(cu, cu, cn, B, True, H)
    closed = H * (C * B * (B + 1) // 2 + B * B * sum(min(kk - 1, c) for c in range(C)))
    assert pairs == closed

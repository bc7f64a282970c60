"""Parity at BASELINE's full sizes through size-independent properties and sampled dense checks.

The CPU oracle cannot evaluate 64K-token configurations in seconds, so these tests use
  * structural invariants of the CSC triple that hold for ANY input (ascending lists, offsets =
    exclusive scan of the counts from the region base, closed-form number of kept chunks);
  * linearity of attention in V and of the backward in dO for a fixed pattern;
  * a dense fp32 evaluation of sampled (sequence, head) pairs with plain torch ops on the GPU over the
    kernel's own pattern (out, dQ, dK, dV under the bf16 tolerance 2e-2 abs / 1e-2 rel, every element),
    and that pattern against an fp32 re-gating wherever the selection is unambiguous.
"""
import numpy as np
import pytest
import torch

from gpu_utils import csc_selection_one_head, dense_ref_one_head

pytestmark = pytest.mark.gpu


def _inputs(seqlens, H, D, chunk, seed, dtype=torch.bfloat16):
    g = torch.Generator(device="cuda").manual_seed(seed)
    T = sum(seqlens)
    q = torch.randn((T, H, D), generator=g, device="cuda")
    k = torch.randn((T, H, D), generator=g, device="cuda")
    v = torch.randn((T, H, D), generator=g, device="cuda")
    dout = torch.randn((T, H, D), generator=g, device="cuda")
    pos = 0
    for L in seqlens:
        C = (L + chunk - 1) // chunk
        k[pos:pos + L] += (0.5 * torch.randn((C, H, D), generator=g, device="cuda")).repeat_interleave(chunk, 0)[:L]
        pos += L
    cu = torch.tensor([0] + list(np.cumsum(seqlens)), dtype=torch.int32, device="cuda")
    return q.to(dtype), k.to(dtype), v.to(dtype), dout.to(dtype), cu


def _check_csc(co, cn, ind, seqlens, H, chunk, topk):
    nb, _, maxC = co.shape
    cu = np.concatenate([[0], np.cumsum(seqlens)])
    # closed form: row r keeps min(topk, r // chunk + 1) chunks
    want = sum(H * int(np.minimum(topk, np.arange(L) // chunk + 1).sum()) for L in seqlens)
    assert int(cn.sum()) == want
    ends = co + cn
    assert bool((co[:, :, 1:] == ends[:, :, :-1]).all())
    for b, L in enumerate(seqlens):
        base = (int(cu[b]) * H + L * torch.arange(H, device=co.device)) * topk
        assert bool((co[b, :, 0] == base).all())
        assert bool((ends[b, :, -1] <= base + L * topk).all())
        C = (L + chunk - 1) // chunk
        assert bool((cn[b, :, C:] == 0).all())
    # ascending lists: inside a segment every entry exceeds its predecessor
    seg_id = torch.zeros(ind.numel() + 1, dtype=torch.int32, device=ind.device)
    starts = co.flatten()[cn.flatten() > 0]
    seg_id.index_add_(0, starts, torch.ones_like(starts, dtype=torch.int32))
    seg_id = torch.cumsum(seg_id[:-1], 0)
    used = torch.zeros(ind.numel() + 1, dtype=torch.int32, device=ind.device)
    used.index_add_(0, starts, torch.ones_like(starts, dtype=torch.int32))
    used.index_add_(0, ends.flatten()[cn.flatten() > 0], -torch.ones_like(starts, dtype=torch.int32))
    used = torch.cumsum(used[:-1], 0) > 0
    same_seg = (seg_id[1:] == seg_id[:-1]) & used[1:] & used[:-1]
    assert bool((ind[1:][same_seg] > ind[:-1][same_seg]).all())
    assert bool((ind[~used] == 0).all())


def _sampled_dense_check(api, pool, q, k, v, dout, cu, seqlens, chunk, topk, samples, grads, csc):
    """Sampled (sequence, head) pairs against a dense fp32 evaluation.  The dense mask is the kernel's OWN pattern
    (`csc`, the triple the same gating call produces: the gating is deterministic), so every row is comparable and
    out, dQ, dK and dV are asserted without exception; the pattern itself is compared with an fp32 re-gating on
    every row whose selection is unambiguous (gap between the last kept and the first rejected score above 1e-3
    relative)."""
    max_len = max(seqlens)
    co, cn, ind = csc
    qg, kg, vg = (t.clone().requires_grad_(grads) for t in (q, k, v))
    out = api.flash_moba_varlen_func(qg, kg, vg, cu, cu, max_len, max_len, chunk, topk, causal=True)
    if grads:
        out.backward(dout)
    km, cu_km, _ = pool.flash_topk_mean_pool(k, cu, max_len, chunk)
    cun = cu.cpu().numpy()
    for (b, h) in samples:
        s, e = int(cun[b]), int(cun[b + 1])
        sel_kernel = csc_selection_one_head(co, cn, ind, b, h, e - s)
        o_ref, dq_ref, dk_ref, dv_ref, sel, gate = dense_ref_one_head(
            q[s:e, h], k[s:e, h], v[s:e, h], dout[s:e, h], km[int(cu_km[b]):int(cu_km[b + 1]), h], chunk, topk,
            sel_override=sel_kernel)
        C = gate.shape[1]
        assert not bool(sel_kernel[:, C:].any()), "a column past the sequence's last chunk has rows"
        ok = torch.ones(e - s, dtype=torch.bool, device=q.device)
        if C > topk:
            sv, _ = torch.sort(gate, dim=-1, descending=True)
            a_, b_ = sv[:, topk - 1], sv[:, topk]
            fin = torch.isfinite(a_) & torch.isfinite(b_)
            ok = ~(fin & ((a_ - b_).abs() <= 1e-3 * torch.maximum(a_.abs(), b_.abs())))
        assert int(ok.sum()) > 0.9 * (e - s)
        differs = (sel_kernel[:, :C] != sel).any(-1)
        assert not bool((differs & ok).any()), f"selection differs from the fp32 gating at (b={b}, h={h}): {int((differs & ok).sum())} unambiguous rows"
        # every row keeps min(topk, visible chunks) chunks, ambiguous or not
        assert torch.equal(sel_kernel.sum(-1), sel.sum(-1))
        named = [("out", out[s:e, h], o_ref)]
        if grads:
            named += [("dq", qg.grad[s:e, h], dq_ref), ("dk", kg.grad[s:e, h], dk_ref), ("dv", vg.grad[s:e, h], dv_ref)]
        for name, got, ref in named:
            err = (got.float() - ref).abs()
            nbad = int((err > 2e-2 + 1e-2 * ref.abs()).sum())
            assert nbad == 0, (name, b, h, nbad, err.max().item())
    return out


@pytest.fixture(scope="module")
def mods():
    import flash_moba
    from flash_moba import mean_pool
    return flash_moba, mean_pool


def test_config2_forward_8k(mods):
    api, pool = mods
    seqlens, H, D, chunk, topk = [8192], 16, 128, 128, 8
    q, k, v, dout, cu = _inputs(seqlens, H, D, chunk, 1002)
    co, cn, ind = api.flash_topk_varlen_func(q, k, cu, cu, 8192, 8192, topk, chunk, causal=True)
    _check_csc(co, cn, ind, seqlens, H, chunk, topk)
    _sampled_dense_check(api, pool, q, k, v, dout, cu, seqlens, chunk, topk, [(0, 0), (0, 7), (0, 15)], grads=False, csc=(co, cn, ind))


def test_config3_fwd_bwd_32k(mods):
    api, pool = mods
    seqlens, H, D, chunk, topk = [32768], 32, 128, 128, 16
    q, k, v, dout, cu = _inputs(seqlens, H, D, chunk, 1003)
    co, cn, ind = api.flash_topk_varlen_func(q, k, cu, cu, 32768, 32768, topk, chunk, causal=True)
    _check_csc(co, cn, ind, seqlens, H, chunk, topk)
    _sampled_dense_check(api, pool, q, k, v, dout, cu, seqlens, chunk, topk, [(0, 5), (0, 17), (0, 31)], grads=True, csc=(co, cn, ind))


def test_sweep_point_2x16k_fp16_fwd_bwd(mods):
    # a point of the reference's own sweep (benchmarks/bench_flash_moba.py:66-78: batch 2, 16 heads of 128, fp16, chunk 128, top-k 8)
    api, pool = mods
    seqlens, H, D, chunk, topk = [16384, 16384], 16, 128, 128, 8
    q, k, v, dout, cu = _inputs(seqlens, H, D, chunk, 1006, torch.float16)
    co, cn, ind = api.flash_topk_varlen_func(q, k, cu, cu, 16384, 16384, topk, chunk, causal=True)
    _check_csc(co, cn, ind, seqlens, H, chunk, topk)
    _sampled_dense_check(api, pool, q, k, v, dout, cu, seqlens, chunk, topk, [(0, 3), (1, 12)], grads=True, csc=(co, cn, ind))


def test_config4_headline_fwd_bwd_64k(mods):
    api, pool = mods
    import bench
    seqlens = bench.headline_seqlens()
    assert sum(seqlens) == 65536 and len(seqlens) == 8 and all(L % 64 == 0 for L in seqlens)
    H, D, chunk, topk = 16, 128, 64, 32
    q, k, v, dout, cu = _inputs(seqlens, H, D, chunk, 1004)
    max_len = max(seqlens)
    co, cn, ind = api.flash_topk_varlen_func(q, k, cu, cu, max_len, max_len, topk, chunk, causal=True)
    _check_csc(co, cn, ind, seqlens, H, chunk, topk)
    # determinism of the integer artefacts: a second run gives the same bits
    co2, cn2, ind2 = api.flash_topk_varlen_func(q, k, cu, cu, max_len, max_len, topk, chunk, causal=True)
    assert torch.equal(co, co2) and torch.equal(cn, cn2) and torch.equal(ind, ind2)
    # the standalone sort is idempotent on the (already ascending) lists
    assert torch.equal(torch.ops.flash_moba._varlen_sort(co, cn, ind), ind)
    out = _sampled_dense_check(api, pool, q, k, v, dout, cu, seqlens, chunk, topk, [(0, 3), (5, 12), (1, 0)], grads=True, csc=(co, cn, ind))
    # linearity in V for a fixed pattern: attn(v1 + v2) = attn(v1) + attn(v2)
    v2 = torch.randn_like(v)
    lg = api.flash_moba_interface.decide_lg_block_m(topk, chunk, max_len, True)
    f = lambda vv: api.flash_moba_attn_varlen_func(q, k, vv, cu, cu, max_len, max_len, co, cn, ind, lg, chunk, causal=True).float()
    lhs, rhs = f(v + v2), f(v) + f(v2)
    assert bool(((lhs - rhs).abs() <= 4e-2 + 2e-2 * rhs.abs()).all())
    assert torch.equal(f(v).to(torch.bfloat16), out.detach())      # forward is deterministic


def _row_reference(q, k, v, dout, km, chunk, topk, r, h, scale):
    """fp32 gate -> top-k (own chunk forced, ties to the higher chunk) -> masked softmax attention of ONE
    query row of a single self-attention sequence, with its dQ (flash_moba/moba_test_utils naive path, row-wise)."""
    L = q.shape[0]
    own = r // chunk
    gate = km[:own, h].float() @ q[r, h].float()
    sel = torch.zeros((L + chunk - 1) // chunk, dtype=torch.bool, device=q.device)
    sel[own] = True
    gap_ok = True
    if own > 0 and topk > 1:
        kk = min(topk - 1, own)
        # total order (score desc, chunk desc): stable sort of the reversed list
        order = torch.argsort(gate.flip(0), descending=True, stable=True)
        idx = own - 1 - order
        sel[idx[:kk]] = True
        if own > kk:
            a_, b_ = gate[idx[kk - 1]], gate[idx[kk]]
            gap_ok = bool((a_ - b_).abs() > 1e-3 * torch.maximum(a_.abs(), b_.abs()))
    mask = sel.repeat_interleave(chunk)[:L] & (torch.arange(L, device=q.device) <= r)
    kk_, vv_ = k[mask, h].float(), v[mask, h].float()
    s = (kk_ @ q[r, h].float()) * scale
    p = torch.softmax(s, 0)
    o = p @ vv_
    dp = vv_ @ dout[r, h].float()
    ds = p * (dp - (dout[r, h].float() * o).sum())
    dq = scale * (ds @ kk_)
    return o, dq, gap_ok


def test_config5_long_context_262k(mods):
    api, pool = mods
    L, H, D, chunk, topk = 262144, 16, 128, 128, 16
    q, k, v, dout, cu = _inputs([L], H, D, chunk, 1005)
    co, cn, ind = api.flash_topk_varlen_func(q, k, cu, cu, L, L, topk, chunk, causal=True)
    assert co.shape == (1, H, 2048) and co.dtype == torch.int64
    _check_csc(co, cn, ind, [L], H, chunk, topk)
    # the last list ends where the last head's region ends minus the slots the first topk-1 chunks leave unused
    assert int(co[0, -1, -1]) + int(cn[0, -1, -1]) == L * H * topk - chunk * (topk * (topk - 1) // 2)
    qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
    out = api.flash_moba_varlen_func(qg, kg, vg, cu, cu, L, L, chunk, topk, causal=True)
    out.backward(dout)
    torch.cuda.synchronize()
    km, cu_km, _ = pool.flash_topk_mean_pool(k, cu, L, chunk)
    scale = D ** -0.5
    checked = 0
    for h in (0, 9):
        for r in (0, 1, 127, 128, 129, 4999, 65536, 131071, 200000, 262143):
            o_ref, dq_ref, gap_ok = _row_reference(q, k, v, dout, km, chunk, topk, r, h, scale)
            if not gap_ok:
                continue
            checked += 1
            assert bool(((out[r, h].float() - o_ref).abs() <= 2e-2 + 1e-2 * o_ref.abs()).all()), (r, h)
            assert bool(((qg.grad[r, h].float() - dq_ref).abs() <= 2e-2 + 1e-2 * dq_ref.abs()).all()), (r, h)
    assert checked >= 16
    # dK and dV of three key chunks (first, middle, last) of two heads, in fp32 from the kernel's own lists and LSE:
    #   P = exp(scale q k^T - lse), dV_j = sum_r P_rj dO_r, dS = P o (dO v^T - delta), dK_j = scale sum_r dS_rj q_r
    lg = api.flash_moba_interface.decide_lg_block_m(topk, chunk, L, True)
    _, lse, _ = api.flash_moba_attn_varlen_func(q, k, v, cu, cu, L, L, co, cn, ind, lg, chunk, causal=True, return_attn_probs=True)
    for h in (3, 14):
        for c in (0, 1023, 2047):
            n, o0 = int(cn[0, h, c]), int(co[0, h, c])
            assert n >= chunk
            rows = ind[o0:o0 + n].long()
            keys = torch.arange(c * chunk, (c + 1) * chunk, device=q.device)
            qr, dor = q[rows, h].float(), dout[rows, h].float()
            kc, vc = k[keys, h].float(), v[keys, h].float()
            p_ = torch.exp(scale * (qr @ kc.T) - lse[h, rows][:, None])
            p_ = torch.where(keys[None, :] <= rows[:, None], p_, torch.zeros_like(p_))
            delta = (dor * out[rows, h].float()).sum(-1, keepdim=True)
            ds = p_ * (dor @ vc.T - delta)
            dv_ref, dk_ref = p_.T @ dor, scale * (ds.T @ qr)
            for name, got, ref in (("dv", vg.grad[keys, h].float(), dv_ref), ("dk", kg.grad[keys, h].float(), dk_ref)):
                nbad = int(((got - ref).abs() > 2e-2 + 1e-2 * ref.abs()).sum())
                assert nbad == 0, (name, h, c, nbad, (got - ref).abs().max().item())
    # every probability row sums to one: sum_j dV_j = sum_r dO_r, per head and feature
    lhs, rhs = vg.grad.float().sum(0), dout.float().sum(0)
    assert bool(((lhs - rhs).abs() <= 2e-2 * rhs.abs().max()).all()), (lhs - rhs).abs().max().item()
    # S = scale * Q K^T is bilinear: sum_r <q_r, dQ_r> = sum_j <k_j, dK_j>, per head.  Both gradients are rounded to
    # bf16 (relative 2^-9 per element, independent), so the two sums differ by about 2^-9 * sqrt(sum of squared terms).
    tq, tk = qg.grad.float() * q.float(), kg.grad.float() * k.float()
    eq, ek = tq.sum((0, 2)), tk.sum((0, 2))
    noise = 2.0 ** -9 * torch.sqrt((tq * tq).sum((0, 2)) + (tk * tk).sum((0, 2)))
    assert bool(((eq - ek).abs() <= 8 * noise + 1e-3 * eq.abs()).all()), (eq, ek, noise)

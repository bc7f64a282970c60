"""CPU restatement of the reference's MoBA hot path.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only ``tests/``,
``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import it.
The shipped package (``flash-moba_amd/flash_moba``) never imports it and has no CPU
fallback.

Every function restates one stage of the reference pipeline in plain PyTorch (CPU,
fp32/fp64) or numpy and cites the reference file:line it follows (paths relative to
the reference checkout):

  stage                     reference
  ------------------------  ---------------------------------------------------------
  mean_pool                 flash_moba/triton_mean_pool.py:74-109,112-157
                            tests/test_triton_mean_pool.py:6-26
  gate_scores               tests/test_fused_topk.py:68-72
  fused_topk                csrc/flash_topk/src/flash_topk_kernel.h:203-295
                            tests/test_fused_topk.py:18-37,40-111
  fused_topk_literal        csrc/flash_topk/src/flash_topk_kernel.h:246-295 (loop, verbatim order)
  csc_from_topk             csrc/flash_topk/src/flash_topk_kernel.h:375-402,406-478
                            tests/test_fused_topk_epilogue.py:19-73
  varlen_sort               csrc/flash_topk/src/varlen_sort.cu:127-162
                            tests/test_varlen_sort.py:11-18
  csc_to_block_mask / attn  flash_moba/moba_test_utils.py:142-196,644-748
                            csrc/flash_moba/src/softmax.h:306-326 (LSE, empty rows)
  attn_bwd                  tests/test_moba_attn.py:288-297 (autograd through the fp32 path)
  decide_lg_block_m         flash_moba/flash_moba_interface.py:20-48

How each function is pinned (tests/test_oracle_pins.py):
  * mean_pool: closed forms (constant keys, chunk size 1, ragged tail divides by its
    real length), and a float64 brute force.
  * fused_topk: three independent formulations agree on random and tie-heavy integer
    inputs (vectorised lexicographic sort, the reference test's stable-sort form, the
    kernel's literal insertion loop); invariants (slot 0 = own chunk in causal mode,
    min(k, visible) valid slots, -inf slots -> -1).
  * csc_from_topk: row-walk formulation of the reference epilogue test, plus
    invariants (sum nnz = valid slots, lists strictly ascending, region bounds).
  * varlen_sort: per-segment library sort, INT32_MIN/MAX, zeros outside segments.
  * attn_fwd: k >= #chunks reduces to dense causal softmax attention
    (torch.nn.functional.scaled_dot_product_attention); k = 1 reduces to
    block-diagonal causal attention; an independent mask path (selection mask
    expanded to tokens, as moba_test_utils.py:644-650) agrees with the CSC path.
  * attn_bwd: torch.autograd.gradcheck in float64 on tiny shapes.
No function here is "parity unpinned".
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch

NEG_INF = float("-inf")


# --------------------------------------------------------------------------------------
# helpers
# --------------------------------------------------------------------------------------
def _lens(cu: torch.Tensor) -> np.ndarray:
    c = cu.detach().cpu().numpy().astype(np.int64)
    return c[1:] - c[:-1]


def round_up(x: int, m: int) -> int:
    return (x + m - 1) // m * m


def decide_lg_block_m(top_k: int, chunk_size: int, seqlen: int, causal: bool = False) -> int:
    """flash_moba/flash_moba_interface.py:20-48 (without the sm86/sm89 cap, which cannot
    fire on a ROCm device)."""
    budget = top_k * chunk_size
    if causal:
        density = (2 * (budget * seqlen) - budget ** 2) / (seqlen ** 2)
    else:
        density = budget / seqlen
    sparsity = 1 - density
    if sparsity <= 0.5:
        return 128
    if sparsity <= 0.7:
        return 256
    if sparsity <= 0.8:
        return 512
    if sparsity <= 0.9:
        return 768
    return 1024


# --------------------------------------------------------------------------------------
# 1. mean-pool
# --------------------------------------------------------------------------------------
def chunk_counts(cu_seqlens_k: torch.Tensor, chunk: int) -> Tuple[np.ndarray, torch.Tensor]:
    """cu_seqlens_km = cumsum(ceil(len / chunk)), int32 (triton_mean_pool.py:134-138)."""
    lens = _lens(cu_seqlens_k)
    c = (lens + chunk - 1) // chunk
    cu = np.zeros(len(c) + 1, dtype=np.int64)
    np.cumsum(c, out=cu[1:])
    return c, torch.from_numpy(cu.astype(np.int32))


def mean_pool(k: torch.Tensor, cu_seqlens_k: torch.Tensor, chunk: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """km[cu_km[b] + c] = cast(sum_fp32(K[cu_k[b] + c*B : +n]) / n), n = min(B, len_b - c*B).

    triton_mean_pool.py:86 (actual_block_size), :105 (divide by it), :142 (zero-initialised
    output of exactly sum(C_b) rows); tests/test_triton_mean_pool.py:19-24."""
    cuk = cu_seqlens_k.detach().cpu().numpy().astype(np.int64)
    counts, cu_km = chunk_counts(cu_seqlens_k, chunk)
    total = int(counts.sum())
    _, hk, d = k.shape
    out = torch.zeros((total, hk, d), dtype=k.dtype)
    kc = k.detach().cpu()
    pos = 0
    for b in range(len(counts)):
        s, e = int(cuk[b]), int(cuk[b + 1])
        L = e - s
        if L <= 0:
            continue
        nfull = L // chunk
        if nfull:
            blk = kc[s:s + nfull * chunk].to(torch.float32).reshape(nfull, chunk, hk, d)
            out[pos:pos + nfull] = blk.mean(dim=1).to(k.dtype)
        if L % chunk:
            tail = kc[s + nfull * chunk:e].to(torch.float32)
            out[pos + nfull] = tail.mean(dim=0).to(k.dtype)
        pos += int(counts[b])
    return out, cu_km


# --------------------------------------------------------------------------------------
# 2. gating + top-k
# --------------------------------------------------------------------------------------
def gate_scores(q_seq: torch.Tensor, km_seq: torch.Tensor) -> torch.Tensor:
    """(H, Lq, C) fp32 scores from dtype-rounded operands (tests/test_fused_topk.py:68-72).
    km_seq has H_k heads; q head h reads kv head h // (H // H_k) (flash_topk_kernel.h:86)."""
    H = q_seq.shape[1]
    Hk = km_seq.shape[1]
    g = H // Hk
    kmf = km_seq.to(torch.float32)
    if g > 1:
        kmf = kmf.repeat_interleave(g, dim=1)
    return torch.einsum("shd,nhd->hsn", q_seq.to(torch.float32), kmf)


def _causal_gate(gate: torch.Tensor, chunk: int, off: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Apply the kernel's rule (flash_topk_kernel.h:203-214,264-267):
    own chunk p=(r+off)//B forced (+inf) iff r+off >= 0; chunk c is a candidate iff
    (c+1)*B - 1 < r + off.  Returns (gate_with_inf, self_chunk[Lq] or -1)."""
    H, Lq, C = gate.shape
    r = torch.arange(Lq, dtype=torch.int64) + off
    cidx = torch.arange(C, dtype=torch.int64)
    cand = ((cidx[None, :] + 1) * chunk - 1) < r[:, None]            # (Lq, C)
    p = torch.div(r, chunk, rounding_mode="floor")
    has_self = r >= 0
    g = gate.clone()
    g.masked_fill_(~cand[None], NEG_INF)
    selfmask = (cidx[None, :] == p[:, None]) & has_self[:, None]
    g.masked_fill_(selfmask[None], float("inf"))
    return g, torch.where(has_self, p, torch.full_like(p, -1))


def _topk_desc_highidx(g: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Top-k by (score desc, index desc) along the last dim via one lexicographic sort."""
    C = g.shape[-1]
    # stable ascending sort on score keeps lower indices first among ties; taking the
    # last k and flipping puts the higher index first (tests/test_fused_topk.py:27-37).
    sv, si = torch.sort(g, dim=-1, descending=False, stable=True)
    kk = min(k, C)
    return sv[..., C - kk:].flip(-1), si[..., C - kk:].flip(-1)


def fused_topk(q: torch.Tensor, km: torch.Tensor, cu_seqlens_q: torch.Tensor,
               cu_seqlens_k: torch.Tensor, cu_seqlens_km: torch.Tensor,
               moba_topk: int, moba_chunk_size: int, causal: bool,
               return_gate: bool = False):
    """Ordered per-row top-k lists: indices (T,H,k_r) int32, values (T,H,k_r) fp32,
    k_r = round_up(k,16), unfilled = (-1, -inf)  (flash_topk_api.cpp:213-214,246-247).
    Ordering/tie rule: flash_topk_kernel.h:217,261,269 (descending chunk scan, strict >)."""
    cuq = cu_seqlens_q.cpu().numpy().astype(np.int64)
    cuk = cu_seqlens_k.cpu().numpy().astype(np.int64)
    cukm = cu_seqlens_km.cpu().numpy().astype(np.int64)
    T, H, _ = q.shape
    kr = round_up(moba_topk, 16)
    idx_out = torch.full((T, H, kr), -1, dtype=torch.int32)
    val_out = torch.full((T, H, kr), NEG_INF, dtype=torch.float32)
    gates = []
    for b in range(len(cuq) - 1):
        sq, eq = int(cuq[b]), int(cuq[b + 1])
        Lq, Lk = eq - sq, int(cuk[b + 1] - cuk[b])
        C = int(cukm[b + 1] - cukm[b])
        if Lq == 0:
            gates.append(None)
            continue
        if C == 0 or Lk == 0:
            gates.append(None)
            continue
        gate = gate_scores(q[sq:eq].cpu(), km[int(cukm[b]):int(cukm[b + 1])].cpu())
        if causal:
            g, _ = _causal_gate(gate, moba_chunk_size, Lk - Lq)
        else:
            g = gate
        vals, inds = _topk_desc_highidx(g, moba_topk)
        inds = inds.to(torch.int32)
        inds[vals == NEG_INF] = -1
        kk = vals.shape[-1]
        idx_out[sq:eq, :, :kk] = inds.permute(1, 0, 2)
        val_out[sq:eq, :, :kk] = vals.permute(1, 0, 2)
        gates.append(g if return_gate else None)
    if return_gate:
        return idx_out, val_out, gates
    return idx_out, val_out


def fused_topk_literal(q, km, cu_seqlens_q, cu_seqlens_k, cu_seqlens_km,
                       moba_topk: int, moba_chunk_size: int, causal: bool):
    """Literal (slow, python-loop) transcription of the selection semantics of
    flash_topk_kernel.h:203-214 (forced own chunk) and :246-295 (descending scan,
    insert on strict '>', bubble on strict '>').  Small inputs only."""
    cuq = cu_seqlens_q.cpu().numpy().astype(np.int64)
    cuk = cu_seqlens_k.cpu().numpy().astype(np.int64)
    cukm = cu_seqlens_km.cpu().numpy().astype(np.int64)
    T, H, _ = q.shape
    kr = round_up(moba_topk, 16)
    idx_out = np.full((T, H, kr), -1, dtype=np.int32)
    val_out = np.full((T, H, kr), -np.inf, dtype=np.float32)
    B = moba_chunk_size
    for b in range(len(cuq) - 1):
        sq, eq = int(cuq[b]), int(cuq[b + 1])
        Lq, Lk = eq - sq, int(cuk[b + 1] - cuk[b])
        C = int(cukm[b + 1] - cukm[b])
        if Lq == 0 or C == 0:
            continue
        gate = gate_scores(q[sq:eq].cpu(), km[int(cukm[b]):int(cukm[b + 1])].cpu()).numpy()
        for h in range(H):
            for r in range(Lq):
                vals = [-np.inf] * moba_topk
                inds = [-1] * moba_topk
                self_idx = r + Lk - Lq
                if causal and self_idx >= 0:
                    inds[0] = self_idx // B
                    vals[0] = np.inf
                for c in range(C - 1, -1, -1):
                    if causal and not ((c + 1) * B - 1 < self_idx):
                        continue
                    v = gate[h, r, c]
                    if v > vals[moba_topk - 1]:
                        vals[moba_topk - 1] = v
                        inds[moba_topk - 1] = c
                        for kk in range(moba_topk - 1, 0, -1):
                            if vals[kk] > vals[kk - 1]:
                                vals[kk], vals[kk - 1] = vals[kk - 1], vals[kk]
                                inds[kk], inds[kk - 1] = inds[kk - 1], inds[kk]
                idx_out[sq + r, h, :moba_topk] = inds
                val_out[sq + r, h, :moba_topk] = vals
    return torch.from_numpy(idx_out), torch.from_numpy(val_out)


# --------------------------------------------------------------------------------------
# 3. CSC build + segmented sort
# --------------------------------------------------------------------------------------
def csc_from_topk(indices: torch.Tensor, cu_seqlens_q: torch.Tensor, moba_topk: int,
                  max_lg_col_num: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """col_offsets (b,H,maxC) int64, col_nnz (b,H,maxC) int32, flat indices (T*H*k,) int32.

    base(b,h) = (cu_q[b]*H + len_q_b*h)*k (flash_topk_kernel.h:396); offsets are an
    exclusive scan of nnz over ALL maxC columns (:397-401); each column's list holds the
    sequence-local rows that selected it (:468-477), here already ascending, which is what
    the reference obtains after its segmented sort; unused slots are 0
    (flash_topk_api.cpp:217)."""
    idx = indices.cpu().numpy()
    cuq = cu_seqlens_q.cpu().numpy().astype(np.int64)
    T, H, _ = idx.shape
    nb = len(cuq) - 1
    col_offsets = np.zeros((nb, H, max_lg_col_num), dtype=np.int64)
    col_nnz = np.zeros((nb, H, max_lg_col_num), dtype=np.int32)
    flat = np.zeros((T * H * moba_topk,), dtype=np.int32)
    for b in range(nb):
        sq, eq = int(cuq[b]), int(cuq[b + 1])
        Lq = eq - sq
        for h in range(H):
            base = (sq * H + Lq * h) * moba_topk
            sel = idx[sq:eq, h, :moba_topk]                      # (Lq, k)
            valid = sel >= 0
            cols = sel[valid].astype(np.int64)
            rows = np.broadcast_to(np.arange(Lq, dtype=np.int32)[:, None], sel.shape)[valid]
            nnz = np.bincount(cols, minlength=max_lg_col_num).astype(np.int64)
            col_nnz[b, h] = nnz.astype(np.int32)
            excl = np.concatenate([[0], np.cumsum(nnz)[:-1]])
            col_offsets[b, h] = base + excl
            order = np.argsort(cols, kind="stable")              # rows stay ascending per column
            flat[base:base + len(order)] = rows[order]
    return torch.from_numpy(col_offsets), torch.from_numpy(col_nnz), torch.from_numpy(flat)


def csc_from_topk_rowwalk(indices, cu_seqlens_q, moba_topk, col_offsets):
    """Row-walk formulation used by the reference's epilogue test
    (tests/test_fused_topk_epilogue.py:19-37): rows ascending, slots ascending, append
    row_local at col_offsets[col] + running count.  Slow; small inputs only."""
    idx = indices.cpu().numpy()
    cuq = cu_seqlens_q.cpu().numpy().astype(np.int64)
    co = col_offsets.cpu().numpy()
    T, H, _ = idx.shape
    nb, _, maxC = co.shape
    flat = np.zeros((T * H * moba_topk,), dtype=np.int32)
    nnz = np.zeros((nb, H, maxC), dtype=np.int32)
    for b in range(nb):
        for h in range(H):
            for j in range(int(cuq[b]), int(cuq[b + 1])):
                for s in range(moba_topk):
                    c = int(idx[j, h, s])
                    if c >= 0:
                        flat[co[b, h, c] + nnz[b, h, c]] = j - int(cuq[b])
                        nnz[b, h, c] += 1
    return torch.from_numpy(flat), torch.from_numpy(nnz)


def varlen_sort(starts: torch.Tensor, ends: torch.Tensor, src: torch.Tensor) -> torch.Tensor:
    """Ascending signed-int32 sort inside each [start, end); zeros elsewhere
    (varlen_sort.cu:154 allocates the output with zeros_like)."""
    s = starts.cpu().numpy().astype(np.int64)
    e = ends.cpu().numpy().astype(np.int64)
    x = src.cpu().numpy()
    out = np.zeros_like(x)
    for a, b in zip(s, e):
        if b > a:
            out[a:b] = np.sort(x[a:b], kind="stable")
    return torch.from_numpy(out)


def flash_topk_ref(q, k, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k,
                   moba_topk, moba_chunk_size, causal=False):
    """flash_moba_interface.py:517-574 on the CPU: pool -> gate/top-k -> CSC (sorted)."""
    d = q.shape[-1]
    if d % 8:
        q = torch.nn.functional.pad(q, [0, 8 - d % 8])
        k = torch.nn.functional.pad(k, [0, 8 - d % 8])
    km, cu_km = mean_pool(k, cu_seqlens_k, moba_chunk_size)
    idx, _ = fused_topk(q, km, cu_seqlens_q, cu_seqlens_k, cu_km, moba_topk, moba_chunk_size, causal)
    maxC = (max_seqlen_k + moba_chunk_size - 1) // moba_chunk_size
    return csc_from_topk(idx, cu_seqlens_q, moba_topk, maxC)


# --------------------------------------------------------------------------------------
# 4. attention over a CSC pattern
# --------------------------------------------------------------------------------------
def csc_to_block_mask(col_offsets, col_nnz, indices, b: int, h: int, Lq: int, nblk: int) -> torch.Tensor:
    """(Lq, nblk) bool: row r attends key block c iff r is listed in column c."""
    co = col_offsets.cpu().numpy()
    cn = col_nnz.cpu().numpy()
    ind = indices.cpu().numpy()
    m = np.zeros((Lq, nblk), dtype=bool)
    for c in range(min(nblk, co.shape[2])):
        n = int(cn[b, h, c])
        if n:
            rows = ind[int(co[b, h, c]):int(co[b, h, c]) + n]
            m[rows, c] = True
    return torch.from_numpy(m)


def token_mask(block_mask: torch.Tensor, lg_block_n: int, Lq: int, Lk: int, causal: bool) -> torch.Tensor:
    """Expand a (Lq, nblk) block mask to tokens and crop (moba_test_utils.py:644-650);
    causal is bottom-right aligned: key j visible iff j <= r + Lk - Lq
    (flash_moba_interface.py:606-616, mask.h:147-175)."""
    m = block_mask.repeat_interleave(lg_block_n, dim=1)[:, :Lk]
    if m.shape[1] < Lk:
        m = torch.nn.functional.pad(m, [0, Lk - m.shape[1]])
    if causal:
        r = torch.arange(Lq)[:, None] + (Lk - Lq)
        j = torch.arange(Lk)[None, :]
        m = m & (j <= r)
    return m


def masked_attention(qh: torch.Tensor, kh: torch.Tensor, vh: torch.Tensor, mask: torch.Tensor,
                     scale: float, round_p_to: Optional[torch.dtype] = None):
    """One (sequence, head): qh (Lq,D), kh/vh (Lk,D), mask (Lq,Lk) True = visible.
    Returns out (Lq,D), lse (Lq,) with lse=+inf / out=0 for rows that see no key
    (softmax.h:317-319).  Differentiable."""
    s = (qh @ kh.transpose(0, 1)) * scale
    s = s.masked_fill(~mask, NEG_INF)
    any_vis = mask.any(dim=1)
    m = torch.where(any_vis, s.max(dim=1).values, torch.zeros_like(s[:, 0]))
    p = torch.exp(s - m[:, None])                     # masked entries -> exp(-inf) = 0
    l = p.sum(dim=1)
    l_safe = torch.where(any_vis, l, torch.ones_like(l))
    pn = p / l_safe[:, None]
    if round_p_to is not None:
        pn = pn.to(round_p_to).to(qh.dtype)
    out = pn @ vh
    lse = torch.where(any_vis, m + torch.log(l_safe), torch.full_like(m, float("inf")))
    return out, lse


def attn_fwd(q, k, v, cu_seqlens_q, cu_seqlens_k, col_offsets, col_nnz, indices,
             lg_block_n: int, softmax_scale: Optional[float] = None, causal: bool = False,
             dtype=torch.float32):
    """Sparse attention forward over a CSC pattern, evaluated densely with masks
    (moba_test_utils.py:653-748 upcast path).  out (T,H,D) `dtype`, lse (H,T) `dtype`.
    Keeps the autograd graph when q/k/v require grad."""
    cuq = cu_seqlens_q.cpu().numpy().astype(np.int64)
    cuk = cu_seqlens_k.cpu().numpy().astype(np.int64)
    T, H, D = q.shape
    Hk = k.shape[1]
    g = H // Hk
    scale = softmax_scale if softmax_scale is not None else D ** (-0.5)
    qf, kf, vf = q.to(dtype), k.to(dtype), v.to(dtype)
    outs = []
    lses = []
    for b in range(len(cuq) - 1):
        sq, eq, sk, ek = int(cuq[b]), int(cuq[b + 1]), int(cuk[b]), int(cuk[b + 1])
        Lq, Lk = eq - sq, ek - sk
        nblk = (Lk + lg_block_n - 1) // lg_block_n
        ob = []
        lb = []
        for h in range(H):
            if Lq == 0:
                continue
            if Lk == 0:
                ob.append(torch.zeros((Lq, D), dtype=dtype))
                lb.append(torch.full((Lq,), float("inf"), dtype=dtype))
                continue
            bm = csc_to_block_mask(col_offsets, col_nnz, indices, b, h, Lq, nblk)
            tm = token_mask(bm, lg_block_n, Lq, Lk, causal)
            o, l = masked_attention(qf[sq:eq, h], kf[sk:ek, h // g], vf[sk:ek, h // g], tm, scale)
            ob.append(o)
            lb.append(l)
        if Lq:
            outs.append(torch.stack(ob, dim=1))        # (Lq,H,D)
            lses.append(torch.stack(lb, dim=0))        # (H,Lq)
    out = torch.cat(outs, dim=0) if outs else torch.zeros((0, H, D), dtype=dtype)
    lse = torch.cat(lses, dim=1) if lses else torch.zeros((H, 0), dtype=dtype)
    return out, lse


def attn_fwd_bwd(q, k, v, dout, cu_seqlens_q, cu_seqlens_k, col_offsets, col_nnz, indices,
                 lg_block_n, softmax_scale=None, causal=False, dtype=torch.float32):
    """Forward + autograd backward in `dtype` (tests/test_moba_attn.py:288-297).
    Returns out, lse, dq, dk, dv (all `dtype`)."""
    qf = q.detach().to(dtype).requires_grad_(True)
    kf = k.detach().to(dtype).requires_grad_(True)
    vf = v.detach().to(dtype).requires_grad_(True)
    out, lse = attn_fwd(qf, kf, vf, cu_seqlens_q, cu_seqlens_k, col_offsets, col_nnz, indices,
                        lg_block_n, softmax_scale, causal, dtype)
    dq, dk, dv = torch.autograd.grad(out, (qf, kf, vf), dout.to(dtype))
    return out.detach(), lse.detach(), dq, dk, dv


# --------------------------------------------------------------------------------------
# 5. the reference's PyTorch MoBA path, end to end (what the CPU baseline times)
# --------------------------------------------------------------------------------------
def moba_dense_ref(q, k, v, cu_seqlens_q, cu_seqlens_k, moba_chunk_size: int, moba_topk: int,
                   causal: bool = True, softmax_scale: Optional[float] = None,
                   dtype=torch.float32, row_block: int = 1024, heads=None, seqs=None):
    """per-chunk mean -> einsum gate -> causal/own-chunk rule -> top-k -> block mask
    expanded to tokens -> dense-masked softmax attention, evaluated `row_block` query rows
    at a time (tests/test_fused_topk.py:40-111 + moba_test_utils.py:653-748,825-829).
    Independent of the CSC code path.  `heads` / `seqs` restrict the evaluation to a subset
    (other entries of the result stay zero).  Returns out (T,H,D) `dtype`."""
    cuq = cu_seqlens_q.cpu().numpy().astype(np.int64)
    cuk = cu_seqlens_k.cpu().numpy().astype(np.int64)
    T, H, D = q.shape
    Hk = k.shape[1]
    g = H // Hk
    B = moba_chunk_size
    scale = softmax_scale if softmax_scale is not None else D ** (-0.5)
    km, cu_km = mean_pool(k, cu_seqlens_k, B)
    cukm = cu_km.numpy().astype(np.int64)
    out = torch.zeros((T, H, D), dtype=dtype)
    for b in (range(len(cuq) - 1) if seqs is None else seqs):
        sq, eq, sk, ek = int(cuq[b]), int(cuq[b + 1]), int(cuk[b]), int(cuk[b + 1])
        Lq, Lk = eq - sq, ek - sk
        C = int(cukm[b + 1] - cukm[b])
        if Lq == 0 or Lk == 0:
            continue
        off = Lk - Lq
        km_b = km[int(cukm[b]):int(cukm[b + 1])]
        for h in (range(H) if heads is None else heads):
            kh = k[sk:ek, h // g].to(dtype)
            vh = v[sk:ek, h // g].to(dtype)
            for r0 in range(0, Lq, row_block):
                r1 = min(Lq, r0 + row_block)
                qh = q[sq + r0:sq + r1, h]
                gate = qh.to(torch.float32) @ km_b[:, h // g].to(torch.float32).transpose(0, 1)  # (R,C)
                rr = torch.arange(r0, r1, dtype=torch.int64) + off
                cidx = torch.arange(C, dtype=torch.int64)
                if causal:
                    cand = ((cidx[None, :] + 1) * B - 1) < rr[:, None]
                    gate = gate.masked_fill(~cand, NEG_INF)
                    selfm = (cidx[None, :] == torch.div(rr, B, rounding_mode="floor")[:, None]) & (rr >= 0)[:, None]
                    gate = gate.masked_fill(selfm, float("inf"))
                vals, inds = _topk_desc_highidx(gate, moba_topk)
                bm = torch.zeros((r1 - r0, C), dtype=torch.bool)
                bm.scatter_(1, inds, vals > NEG_INF)
                tm = bm.repeat_interleave(B, dim=1)[:, :Lk]
                if causal:
                    tm = tm & (torch.arange(Lk)[None, :] <= rr[:, None])
                o, _ = masked_attention(qh.to(dtype), kh, vh, tm, scale)
                out[sq + r0:sq + r1, h] = o
    return out


# --------------------------------------------------------------------------------------
# 6. acceptance rule for near-ties
# --------------------------------------------------------------------------------------
def topk_gap_mask(gates, cu_seqlens_q, moba_topk: int, rel: float = 1e-3) -> torch.Tensor:
    """(T,H) bool: True where the row's selection is unambiguous, i.e. the gap between the
    last selected and the first rejected candidate score exceeds `rel` relative
    (BASELINE north_star: "bit-exact wherever the reference score gap exceeds 1e-3
    relative"; moba_test_utils.py:835-843 uses the same idea with an absolute eps).
    `gates` is the list returned by fused_topk(..., return_gate=True)."""
    cuq = cu_seqlens_q.cpu().numpy().astype(np.int64)
    H = next(g.shape[0] for g in gates if g is not None) if any(g is not None for g in gates) else 0
    T = int(cuq[-1])
    ok = torch.ones((T, H), dtype=torch.bool)
    for b, g in enumerate(gates):
        if g is None:
            continue
        C = g.shape[-1]
        if C <= moba_topk:
            continue
        sv, _ = torch.sort(g, dim=-1, descending=True)
        kth, nxt = sv[..., moba_topk - 1], sv[..., moba_topk]
        finite = torch.isfinite(kth) & torch.isfinite(nxt)
        gap = (kth - nxt).abs()
        thr = rel * torch.maximum(kth.abs(), nxt.abs())
        amb = finite & (gap <= thr)
        ok[int(cuq[b]):int(cuq[b + 1])] = (~amb).transpose(0, 1)
    return ok


# --------------------------------------------------------------------------------------
# 7. seeded inputs of the benchmark configurations
# --------------------------------------------------------------------------------------
def make_inputs(seqlens, H: int, D: int, chunk: int, seed: int, dtype=torch.float32, Hk: Optional[int] = None,
                with_dout: bool = False):
    """q, v ~ N(0,1); k = N(0,1) + a per-(sequence, chunk, head) bias vector ~ N(0, 0.5)
    shared by the tokens of a chunk, so that gating scores separate.  Generated in fp32
    on the CPU from a seeded generator, then cast, so the CPU oracle and the GPU see the
    same bits."""
    Hk = Hk or H
    gen = torch.Generator().manual_seed(seed)
    T = int(sum(seqlens))
    q = torch.randn((T, H, D), generator=gen)
    k = torch.randn((T, Hk, D), generator=gen)
    v = torch.randn((T, Hk, D), generator=gen)
    pos = 0
    for L in seqlens:
        C = (L + chunk - 1) // chunk
        if C:
            bias = 0.5 * torch.randn((C, Hk, D), generator=gen)
            k[pos:pos + L] += bias.repeat_interleave(chunk, dim=0)[:L]
        pos += L
    cu = torch.tensor([0] + list(np.cumsum(seqlens)), dtype=torch.int32)
    res = [q.to(dtype), k.to(dtype), v.to(dtype), cu]
    if with_dout:
        res.append(torch.randn((T, H, D), generator=gen).to(dtype))
    return res


def headline_seqlens(seed: int = 1004, n: int = 8, total: int = 65536, lo: int = 2048, hi: int = 14336,
                     mult: int = 64):
    """8 lengths ~ U[lo,hi] from a seeded RNG, rescaled to sum to `total`, rounded to
    multiples of `mult`, the last one fixed so that the sum is exact."""
    rng = np.random.RandomState(seed)
    raw = rng.uniform(lo, hi, size=n)
    scaled = raw / raw.sum() * total
    lens = [int(round(x / mult)) * mult for x in scaled]
    lens[-1] = total - sum(lens[:-1])
    assert all(l > 0 and l % mult == 0 for l in lens), lens
    return lens


def count_pairs(cu_seqlens_q, cu_seqlens_k, col_nnz, lg_block_n: int, causal: bool, H: int) -> int:
    """Unmasked (query,key) pairs for a gating-produced pattern with len_q == len_k and
    full chunks: every listed (row, chunk) pair contributes `chunk` keys except the row's
    own chunk, which contributes (r mod chunk) + 1."""
    cuq = cu_seqlens_q.cpu().numpy().astype(np.int64)
    nn = col_nnz.cpu().numpy().astype(np.int64)
    total = int(nn.sum()) * lg_block_n
    if causal:
        for b in range(len(cuq) - 1):
            L = int(cuq[b + 1] - cuq[b])
            r = np.arange(L)
            total -= H * int((lg_block_n - (r % lg_block_n) - 1).sum())
    return total

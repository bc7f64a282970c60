"""Helpers shared by the GPU parity tests (the HIP path is always called through the
package's C-ABI binding; the oracle runs on the CPU)."""
import numpy as np
import torch

from oracle import moba_oracle as O


def dev(*ts):
    return [t.cuda() if isinstance(t, torch.Tensor) else t for t in ts]


def csc_structure_ok(co, cn, flat, cu_q, H, topk):
    """Invariants every CSC triple produced by gating must satisfy."""
    co, cn, flat = co.cpu().numpy(), cn.cpu().numpy(), flat.cpu().numpy()
    cuq = cu_q.cpu().numpy().astype(np.int64)
    nb, _, maxC = co.shape
    for b in range(nb):
        Lq = int(cuq[b + 1] - cuq[b])
        for h in range(H):
            base = (int(cuq[b]) * H + Lq * h) * topk
            ends = co[b, h] + cn[b, h]
            assert co[b, h, 0] == base, (b, h)
            assert (co[b, h, 1:] == ends[:-1]).all(), (b, h)
            assert ends[-1] <= base + Lq * topk
            region = flat[base:base + Lq * topk]
            used = int(cn[b, h].sum())
            assert (region[used:] == 0).all(), "unused slots must be zero"
            for c in range(maxC):
                seg = flat[co[b, h, c]:ends[c]]
                assert (np.diff(seg) > 0).all(), (b, h, c)
                if len(seg):
                    assert seg[0] >= 0 and seg[-1] < Lq


def selection_sets(co, cn, flat, b, h, Lq, maxC):
    """(Lq, maxC) bool selection matrix of one (sequence, head) from a CSC triple."""
    return O.csc_to_block_mask(co, cn, flat, b, h, Lq, maxC).numpy()


def assert_close(name, got, ref, atol, rtol):
    got, ref = got.float().cpu(), ref.float().cpu()
    err = (got - ref).abs()
    tol = atol + rtol * ref.abs()
    bad = err > tol
    assert not bad.any(), f"{name}: {int(bad.sum())} / {bad.numel()} elements out of tolerance, max err {err.max().item():.4e}"


def csc_selection_one_head(co, cn, ind, b, h, L):
    """(L, maxC) bool selection of one (sequence, head) read from a CSC triple on its device: the lists of a
    (sequence, head) are consecutive (offsets = exclusive scan of the counts), so one slice holds them all."""
    maxC = co.shape[2]
    counts = cn[b, h].long()
    start = int(co[b, h, 0])
    rows = ind[start:start + int(counts.sum())].long()
    cols = torch.repeat_interleave(torch.arange(maxC, device=co.device), counts)
    sel = torch.zeros((L, maxC), dtype=torch.bool, device=co.device)
    sel[rows, cols] = True
    return sel


def dense_ref_one_head(q, k, v, dout, km, chunk, topk, row_block=2048, sel_override=None):
    """fp32 dense-masked MoBA of ONE (sequence, head) evaluated with plain torch ops on the
    tensors' device (test reference for sizes the CPU oracle cannot finish in seconds).
    q, k, v, dout: (L, D); km: (C, D) chunk means in the storage dtype.  Returns out, dq, dk, dv
    (fp32), the boolean (L, C) selection of its own fp32 gating and the gate values.  With
    sel_override (L, >= C) the attention uses that selection instead of the re-gated one (the
    re-gated selection and the gates are still returned)."""
    L, D = q.shape
    C = km.shape[0]
    dev = q.device
    qf = q.float().requires_grad_(True)
    kf = k.float().requires_grad_(True)
    vf = v.float().requires_grad_(True)
    gate = q.float() @ km.float().T
    r = torch.arange(L, device=dev)
    c = torch.arange(C, device=dev)
    cand = ((c[None] + 1) * chunk - 1) < r[:, None]
    gate = gate.masked_fill(~cand, float("-inf"))
    own = c[None] == (r // chunk)[:, None]
    gate = gate.masked_fill(own, float("inf"))
    sv, si = torch.sort(gate, dim=-1, descending=False, stable=True)
    kk = min(topk, C)
    tv, ti = sv[:, C - kk:], si[:, C - kk:]
    sel = torch.zeros((L, C), dtype=torch.bool, device=dev)
    sel.scatter_(1, ti, tv > float("-inf"))
    use = sel if sel_override is None else sel_override[:, :C]
    outs = []
    scale = D ** -0.5
    for r0 in range(0, L, row_block):
        r1 = min(L, r0 + row_block)
        m = use[r0:r1].repeat_interleave(chunk, dim=1)[:, :L] & (torch.arange(L, device=dev)[None] <= r[r0:r1, None])
        s = (qf[r0:r1] @ kf.T) * scale
        s = s.masked_fill(~m, float("-inf"))
        outs.append(torch.softmax(s, -1) @ vf)
    out = torch.cat(outs)
    dq, dk, dv = torch.autograd.grad(out, (qf, kf, vf), dout.float())
    return out.detach(), dq, dk, dv, sel, gate

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

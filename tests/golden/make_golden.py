"""Writes the committed golden fixtures (small .npz files: inputs + expected outputs).

    python tests/golden/make_golden.py

Every expected output comes from the CPU oracle (oracle/moba_oracle.py), whose functions are
pinned by tests/test_oracle_pins.py against closed forms, library routines and brute force; the
reference repository holds no golden data of its own (its tests compare against in-file PyTorch
oracles on CUDA-seeded inputs, which do not transfer to another device).  The reference's Python
is neither imported nor run here.

Fixtures:
  c1_plumbing.npz     BASELINE config 1: lengths [1024, 2048], 8 heads, d=64, chunk 128, top-k 4, fp32,
                      causal; inputs are regenerated from the seed (checksummed), outputs stored:
                      CSC triple and the forward output at every 37th row.
  ties.npz            integer-valued q/k so that gating scores tie exactly (tie rule: higher chunk wins).
  ragged_gqa.npz      ragged tails (len % chunk != 0), len_q != len_k, an empty sequence, GQA (6 q heads,
                      2 kv heads), top-k larger than the number of chunks; CSC + forward output + gradients.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import moba_oracle as O  # noqa: E402


def checksum(*ts):
    return float(sum(t.double().abs().sum().item() for t in ts))


def c1():
    lens, H, D, chunk, topk = [1024, 2048], 8, 64, 128, 4
    q, k, v, cu = O.make_inputs(lens, H, D, chunk, 1001, torch.float32)
    co, cn, ind = O.flash_topk_ref(q, k, cu, cu, max(lens), max(lens), topk, chunk, True)
    out = O.moba_dense_ref(q, k, v, cu, cu, chunk, topk, True)
    out2, lse = O.attn_fwd(q, k, v, cu, cu, co, cn, ind, chunk, None, True)
    assert torch.allclose(out, out2, atol=2e-5)
    np.savez_compressed(os.path.join(HERE, "c1_plumbing.npz"), seqlens=np.array(lens), heads=H, head_dim=D, chunk=chunk,
                        topk=topk, seed=1001, input_checksum=checksum(q, k, v), col_offsets=co.numpy(), col_nnz=cn.numpy(),
                        indices=ind.numpy(), out_rows=np.arange(0, sum(lens), 37), out=out[::37].numpy(), lse=lse[:, ::37].numpy())


def ties():
    g = torch.Generator().manual_seed(5)
    lens_q, lens_k, H, Hk, D, chunk, topk = [96, 40], [96, 40], 4, 2, 16, 8, 3
    q = torch.randint(-2, 3, (sum(lens_q), H, D), generator=g).float()
    k = torch.randint(-1, 2, (sum(lens_k), Hk, D), generator=g).float()
    km_sum = torch.cat([k[s:s + L].reshape(-1, chunk, Hk, D).sum(1) for s, L in ((0, 96), (96, 40))])  # integer "means" x chunk
    cu = torch.tensor([0, 96, 136], dtype=torch.int32)
    cu_km = torch.tensor([0, 12, 17], dtype=torch.int32)
    res = {}
    for causal in (True, False):
        idx, val = O.fused_topk(q, km_sum, cu, cu, cu_km, topk, chunk, causal)
        co, cn, ind = O.csc_from_topk(idx, cu, topk, 12)
        tag = "causal" if causal else "full"
        res.update({f"idx_{tag}": idx.numpy(), f"val_{tag}": val.numpy(), f"co_{tag}": co.numpy(), f"cn_{tag}": cn.numpy(),
                    f"ind_{tag}": ind.numpy()})
    np.savez_compressed(os.path.join(HERE, "ties.npz"), q=q.numpy(), km=km_sum.numpy(), cu=cu.numpy(), cu_km=cu_km.numpy(),
                        chunk=chunk, topk=topk, **res)


def ragged():
    g = torch.Generator().manual_seed(9)
    lens_q, lens_k, H, Hk, D, chunk, topk = [70, 0, 33, 150], [100, 0, 33, 130], 6, 2, 32, 64, 4
    q = torch.randn((sum(lens_q), H, D), generator=g)
    k = torch.randn((sum(lens_k), Hk, D), generator=g)
    v = torch.randn((sum(lens_k), Hk, D), generator=g)
    dout = torch.randn((sum(lens_q), H, D), generator=g)
    # round to bf16 so that a bf16 kernel sees exactly these values
    q, k, v, dout = (t.to(torch.bfloat16).float() for t in (q, k, v, dout))
    cuq = torch.tensor([0] + list(np.cumsum(lens_q)), dtype=torch.int32)
    cuk = torch.tensor([0] + list(np.cumsum(lens_k)), dtype=torch.int32)
    km, cu_km = O.mean_pool(k.to(torch.bfloat16), cuk, chunk)
    idx, val = O.fused_topk(q.to(torch.bfloat16), km, cuq, cuk, cu_km, topk, chunk, True)
    co, cn, ind = O.csc_from_topk(idx, cuq, topk, 3)
    out, lse, dq, dk, dv = O.attn_fwd_bwd(q, k, v, dout, cuq, cuk, co, cn, ind, chunk, None, True)
    np.savez_compressed(os.path.join(HERE, "ragged_gqa.npz"), q=q.numpy(), k=k.numpy(), v=v.numpy(), dout=dout.numpy(),
                        cuq=cuq.numpy(), cuk=cuk.numpy(), chunk=chunk, topk=topk, km=km.float().numpy(), cu_km=cu_km.numpy(),
                        idx=idx.numpy(), co=co.numpy(), cn=cn.numpy(), ind=ind.numpy(), out=out.numpy(), lse=lse.numpy(),
                        dq=dq.numpy(), dk=dk.numpy(), dv=dv.numpy())


if __name__ == "__main__":
    c1()
    ties()
    ragged()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")

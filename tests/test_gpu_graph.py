"""The fused path under HIP graph capture: the library allocates nothing, never synchronises and clears its scratch
memory with fill kernels, and the Python host of the gated path reads nothing back from the device, so the whole
forward + backward (mean-pool, gating, CSC build, attention, gradients) can be recorded once and replayed.  A replay is
checked bit for bit against the eager result, several times, on new inputs written into the captured tensors, with
eager work and synchronisations of the program's own between the replays."""
import pytest
import torch

from oracle import moba_oracle as O

pytestmark = pytest.mark.gpu


def _eager(fn, q, k, v, dout, *args, **kw):
    qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
    out = fn(qg, kg, vg, *args, **kw)
    dq, dk, dv = torch.autograd.grad(out, (qg, kg, vg), dout)
    return out.detach(), dq, dk, dv


@pytest.mark.parametrize("lens,H,D,chunk,topk", [([1536, 700, 2100], 4, 128, 64, 6), ([4000, 1100], 2, 64, 128, 3)])
def test_fused_path_replays_from_a_graph(lens, H, D, chunk, topk):
    import flash_moba

    fn = flash_moba.flash_moba_varlen_func
    inputs = []
    for seed in (11, 12, 13, 14):
        q, k, v, cu, dout = O.make_inputs(lens, H, D, chunk, seed, torch.bfloat16, with_dout=True)
        inputs.append(tuple(t.cuda() for t in (q, k, v, dout)))
    cu = cu.cuda()
    args = (cu, cu, max(lens), max(lens), chunk, topk)

    # the captured tensors; warm-up on a side stream as torch asks for before a capture
    qs, ks, vs = (t.clone().requires_grad_(True) for t in inputs[0][:3])
    ds = inputs[0][3].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            out = fn(qs, ks, vs, *args, causal=True)
            torch.autograd.grad(out, (qs, ks, vs), ds)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_s = fn(qs, ks, vs, *args, causal=True)
        dq_s, dk_s, dv_s = torch.autograd.grad(out_s, (qs, ks, vs), ds)

    for i, (q, k, v, dout) in enumerate(inputs):
        want = _eager(fn, q, k, v, dout, *args, causal=True)  # eager work between the replays
        torch.cuda.synchronize()
        with torch.no_grad():
            qs.copy_(q)
            ks.copy_(k)
            vs.copy_(v)
            ds.copy_(dout)
        graph.replay()
        torch.cuda.synchronize()
        for name, x, y in zip(("out", "dq", "dk", "dv"), (out_s, dq_s, dk_s, dv_s), want):
            assert torch.equal(x, y), (i, name)

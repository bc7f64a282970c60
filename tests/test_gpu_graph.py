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


def test_attention_over_a_given_pattern_replays_from_a_graph():
    """A caller's own CSC pattern: with the bound on a row's visits given (the trailing argument of the autograd
    function) nothing is read back from the device, so forward + backward capture as well."""
    import flash_moba
    from flash_moba.flash_moba_interface import FlashMobaAttnVarlenFunc

    lens, H, D, chunk, topk = [1100, 2300], 4, 128, 64, 5
    inputs = []
    for seed in (21, 22, 23):
        q, k, v, cu, dout = O.make_inputs(lens, H, D, chunk, seed, torch.bfloat16, with_dout=True)
        inputs.append(tuple(t.cuda() for t in (q, k, v, dout)))
    cu = cu.cuda()
    with torch.no_grad():  # one pattern for every input (from the first one's gate)
        co, cn, ind = flash_moba.flash_topk_varlen_func(inputs[0][0], inputs[0][1], cu, cu, max(lens), max(lens), topk, chunk, causal=True)

    def fn(q, k, v):
        return FlashMobaAttnVarlenFunc.apply(q, k, v, cu, cu, max(lens), max(lens), co, cn, ind, 128, chunk, 0.0, None, True,
                                             0.0, None, False, False, True, topk, None)

    qs, ks, vs = (t.clone().requires_grad_(True) for t in inputs[0][:3])
    ds = inputs[0][3].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        torch.autograd.grad(fn(qs, ks, vs), (qs, ks, vs), ds)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_s = fn(qs, ks, vs)
        grads_s = torch.autograd.grad(out_s, (qs, ks, vs), ds)
    for i, (q, k, v, dout) in enumerate(inputs):
        qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
        out = flash_moba.flash_moba_attn_varlen_func(qg, kg, vg, cu, cu, max(lens), max(lens), co, cn, ind, 128, chunk, causal=True)
        want = (out.detach(),) + torch.autograd.grad(out, (qg, kg, vg), dout)
        torch.cuda.synchronize()
        with torch.no_grad():
            qs.copy_(q)
            ks.copy_(k)
            vs.copy_(v)
            ds.copy_(dout)
        graph.replay()
        torch.cuda.synchronize()
        for name, x, y in zip(("out", "dq", "dk", "dv"), (out_s,) + tuple(grads_s), want):
            assert torch.equal(x, y), (i, name)

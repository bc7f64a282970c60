"""torch.compile through the public functions (the reference registers fake-shape functions for exactly that,
flash_moba/flash_moba_interface.py:113-137,157-165,233-270,349-391).  The graphs are captured with fullgraph=True,
so nothing may fall back to Python between the ops, and run through AOT autograd on fake tensors (backend
"aot_eager": the compiled graph then calls the same HIP kernels as eager mode and must give the same bits; no
generated device code is involved)."""
import numpy as np
import pytest
import torch

from oracle import moba_oracle as O

pytestmark = pytest.mark.gpu


def _fwd_bwd(fn, q, k, v, dout, *args, **kw):
    qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
    out = fn(qg, kg, vg, *args, **kw)
    out.backward(dout)
    return out.detach(), qg.grad, kg.grad, vg.grad


@pytest.mark.parametrize("lens,H,D,chunk,topk", [([640, 300, 1300], 4, 128, 64, 4), ([2100, 900], 2, 72, 128, 5)])
def test_compiled_fused_path_equals_eager_bit_for_bit(lens, H, D, chunk, topk):
    import flash_moba

    q, k, v, cu, dout = O.make_inputs(lens, H, D, chunk, 5, torch.bfloat16, with_dout=True)
    q, k, v, cu, dout = (t.cuda() for t in (q, k, v, cu, dout))
    args = (cu, cu, max(lens), max(lens), chunk, topk)
    eager = _fwd_bwd(flash_moba.flash_moba_varlen_func, q, k, v, dout, *args, causal=True)
    torch._dynamo.reset()
    compiled = torch.compile(flash_moba.flash_moba_varlen_func, fullgraph=True, backend="aot_eager")
    for _ in range(2):  # second call: the cached graph
        got = _fwd_bwd(compiled, q, k, v, dout, *args, causal=True)
        for name, x, y in zip(("out", "dq", "dk", "dv"), got, eager):
            assert torch.equal(x, y), name


def test_compiled_attention_over_a_user_pattern_equals_eager():
    import flash_moba

    lens = [513, 700]
    q, k, v, cu, dout = O.make_inputs(lens, 4, 64, 64, 6, torch.bfloat16, with_dout=True)
    q, k, v, cu, dout = (t.cuda() for t in (q, k, v, cu, dout))
    with torch.no_grad():
        co, cn, ind = flash_moba.flash_topk_varlen_func(q, k, cu, cu, max(lens), max(lens), 3, 64, causal=True)
    args = (cu, cu, max(lens), max(lens), co, cn, ind, 128, 64)
    eager = _fwd_bwd(flash_moba.flash_moba_attn_varlen_func, q, k, v, dout, *args, causal=True)
    torch._dynamo.reset()
    compiled = torch.compile(flash_moba.flash_moba_attn_varlen_func, fullgraph=True, backend="aot_eager")
    got = _fwd_bwd(compiled, q, k, v, dout, *args, causal=True)
    for name, x, y in zip(("out", "dq", "dk", "dv"), got, eager):
        assert torch.equal(x, y), name
    # the gating alone
    topk_c = torch.compile(flash_moba.flash_topk_varlen_func, fullgraph=True, backend="aot_eager")
    co2, cn2, ind2 = topk_c(q, k, cu, cu, max(lens), max(lens), 3, 64, causal=True)
    assert torch.equal(co, co2) and torch.equal(cn, cn2) and torch.equal(ind, ind2)

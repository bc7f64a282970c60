#!/usr/bin/env python3
"""Benchmark of the MoBA hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config headline|c2|c3]

A step is one pass of the hot path over one batch of synthetic input with everything
already resident in HBM: mean-pool -> fused top-k gating -> CSC build -> sparse attention
forward -> sparse attention backward (``flash_moba_varlen_func`` + ``.backward``).  The
default workload is the headline configuration: a packed batch of 8 sequences totalling
65536 tokens, bf16, causal, 16 heads, head_dim 128, chunk 64, top-k 32.

Prints ONE JSON line: the metric (effective sparse TFLOP/s of fwd+bwd attention over the
step time), ms per step, per-stage times with their roofline fractions, a ``roofline``
object for the dominant kernel (timed alone with events on the launch stream) and a
``cpu_baseline`` object (the CPU restatement of the reference's PyTorch MoBA path timed on
the host cores on a bounded sample of the same inputs).
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "flash-moba_amd"))
sys.path.insert(0, ROOT)

# MI355X published peaks used for every roofline fraction printed here
PEAK_HBM_GBS = 8000.0          # GB/s
PEAK_BF16_TFLOPS = 2500.0      # dense bf16 MFMA, TFLOP/s

CONFIGS = {
    # name: (seqlens or None for the seeded headline rule, heads, head_dim, chunk, topk, backward)
    "headline": (None, 16, 128, 64, 32, True),
    "c2": ([8192], 16, 128, 128, 8, False),
    "c3": ([32768], 32, 128, 128, 16, True),
    "c5": ([262144], 16, 128, 128, 16, True),
    # two points of the reference's own sequence-length sweep (benchmarks/bench_flash_moba.py): batch 2, chunk 128, top-k 8, fp16
    "sweep16k": ([16384, 16384], 16, 128, 128, 8, True),
    "sweep64k": ([65536, 65536], 16, 128, 128, 8, True),
}
# the arithmetic type of the 16-bit inputs: bf16 as BASELINE.json's configs say, fp16 where the reference's own sweep uses it
CONFIG_DTYPE = {"sweep16k": "fp16", "sweep64k": "fp16"}


def headline_seqlens(seed=1004, n=8, total=65536, lo=2048, hi=14336, mult=64):
    """8 lengths ~ U[lo, hi] from a seeded RNG, rescaled to sum to `total`, rounded to multiples
    of `mult`, the last one fixed so that the sum is exact."""
    rng = np.random.RandomState(seed)
    raw = rng.uniform(lo, hi, size=n)
    lens = [int(round(x / raw.sum() * total / mult)) * mult for x in raw]
    lens[-1] = total - sum(lens[:-1])
    return lens


def make_inputs(seqlens, H, D, chunk, seed, device, dtype=torch.bfloat16):
    """q, v, dout ~ N(0,1); k = N(0,1) + per-(sequence, chunk, head) bias ~ N(0, 0.5)."""
    g = torch.Generator(device=device).manual_seed(seed)
    T = sum(seqlens)
    q = torch.randn((T, H, D), generator=g, device=device)
    k = torch.randn((T, H, D), generator=g, device=device)
    v = torch.randn((T, H, D), generator=g, device=device)
    dout = torch.randn((T, H, D), generator=g, device=device)
    pos = 0
    for L in seqlens:
        C = (L + chunk - 1) // chunk
        bias = 0.5 * torch.randn((C, H, D), generator=g, device=device)
        k[pos:pos + L] += bias.repeat_interleave(chunk, dim=0)[:L]
        pos += L
    cu = torch.tensor([0] + list(np.cumsum(seqlens)), dtype=torch.int32, device=device)
    return q.to(dtype), k.to(dtype), v.to(dtype), dout.to(dtype), cu


def count_pairs(seqlens, col_nnz, chunk, H):
    """Unmasked (query, key) pairs of a causal, gating-produced pattern (len_q == len_k): every
    listed (row, chunk) pair contributes `chunk` keys, except a row's own chunk, which
    contributes (row mod chunk) + 1."""
    total = int(col_nnz.sum().item()) * chunk
    for L in seqlens:
        r = np.arange(L)
        total -= H * int((chunk - (r % chunk) - 1).sum())
    return total


def time_events(fn, iters, warmup=1):
    """Average milliseconds of fn() over `iters` runs, measured with events recorded on the
    stream the kernels are launched on (torch's current stream)."""
    for _ in range(warmup):
        fn()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) / iters


# HBM-side bytes per launch, per workload: rocprofv3 FETCH_SIZE + WRITE_SIZE per dispatch, each scaled by what the
# same counter reads for a plain 1 GiB copy (the summaries of those runs are kept under profiles/, one per workload).
# Counter runs cannot be made from inside this script, so the figures are the committed measurement.
MEASURED_TRAFFIC_BYTES = {
    ("headline", "attn_fwd_rows_kernel"): 1.278e9,
    ("headline", "attn_bwd_dkdv_kernel"): 6.697e9,
    ("headline", "attn_bwd_dq_kernel"): 5.135e9,
    ("c2", "attn_fwd_col_kernel"): 4.421e8,
    ("c3", "attn_fwd_col_kernel"): 8.239e9,
    ("c3", "attn_bwd_dkdv_kernel"): 1.295e10,
    ("c5", "attn_fwd_col_kernel"): 3.995e10,
    ("c5", "attn_bwd_dkdv_kernel"): 6.686e10,
    ("sweep16k", "attn_fwd_col_kernel"): 1.942e9,
    ("sweep16k", "attn_bwd_dkdv_kernel"): 2.939e9,
    ("sweep64k", "attn_fwd_col_kernel"): 9.662e9,
    ("sweep64k", "attn_bwd_dkdv_kernel"): 1.551e10,
}


def cpu_baseline(q, k, v, cu, seqlens, chunk, topk, budget_s=12.0):
    """Times the CPU restatement of the reference's PyTorch MoBA path (chunk means -> gate ->
    top-k -> block mask -> dense-masked softmax attention, fp32) on (longest sequence,
    heads 0..n) of the same inputs, adding heads until ~budget_s of CPU work has been done."""
    from oracle import moba_oracle as O  # checker only: never on the product path

    torch.set_num_threads(os.cpu_count())
    H, D = q.shape[1], q.shape[2]
    order = sorted(range(len(seqlens)), key=lambda i: -seqlens[i])  # longest sequences first
    t0 = time.perf_counter()
    pairs, done = 0, []
    for b in order:
        L, start = seqlens[b], sum(seqlens[:b])
        qs, ks, vs = (t[start:start + L].float().cpu() for t in (q, k, v))
        cu0 = torch.tensor([0, L], dtype=torch.int32)
        C = (L + chunk - 1) // chunk
        per_head = (sum(min(chunk, L - c * chunk) * (min(chunk, L - c * chunk) + 1) // 2 for c in range(C))
                    + chunk * chunk * sum(min(topk - 1, c) for c in range(C)))
        # a head of a very long sequence alone would exceed the budget: take its last rows only (the keys stay whole)
        R = L if L <= 32768 else 4096
        if R < L:
            qs = qs[L - R:]
            per_head = sum((p % chunk + 1) + chunk * min(topk - 1, p // chunk) for p in range(L - R, L))
        cuq0 = torch.tensor([0, R], dtype=torch.int32)
        heads = 0
        while heads < H and (time.perf_counter() - t0) < budget_s:
            O.moba_dense_ref(qs[:, heads:heads + 1], ks[:, heads:heads + 1], vs[:, heads:heads + 1], cuq0, cu0, chunk, topk, True,
                             row_block=1024)
            heads += 1
            pairs += per_head
        if heads:
            done.append(f"sequence {b} ({L} tokens{'' if R == L else f', its last {R} query rows'}) x {heads} heads")
        if (time.perf_counter() - t0) >= budget_s:
            break
    dt = time.perf_counter() - t0
    flops = 4.0 * D * pairs
    return {
        "value": flops / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": os.cpu_count(),
        "kind": "port",
        "sample": "forward only, fp32, row-blocked dense-masked attention on " + ", ".join(done)
                  + f"; {dt:.1f} s of CPU time; effective sparse FLOPs / time",
        "seconds": dt,
    }


def dense_sdpa_ms(cfg, dev, iters=3):
    """Forward + backward of dense causal attention (torch scaled_dot_product_attention, fp16) on a sweep shape: the
    baseline benchmarks/bench_flash_moba.py of the reference compares with."""
    seqlens, H, D, _, _, _ = cfg
    B, L = len(seqlens), seqlens[0]
    q, k, v = (torch.randn((B, H, L, D), device=dev, dtype=torch.float16, requires_grad=True) for _ in range(3))
    g = torch.randn((B, H, L, D), device=dev, dtype=torch.float16)

    def step():
        q.grad = k.grad = v.grad = None
        torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True).backward(g)

    return time_events(step, iters)


def graph_replay_ms(q, k, v, dout, cu, max_len, chunk, topk, backward, steps):
    """The same step recorded once as a HIP graph (torch.cuda.CUDAGraph) and replayed `steps` times: what a serving or
    training loop pays per step when it keeps the launches of the hot path in a graph.  Reported beside `ms_per_step`
    (which stays the eager loop); None if the capture fails."""
    import flash_moba

    try:
        qs, ks, vs = (t.detach().clone().requires_grad_(backward) for t in (q, k, v))

        def once():
            out = flash_moba.flash_moba_varlen_func(qs, ks, vs, cu, cu, max_len, max_len, chunk, topk, causal=True)
            return (out,) + (torch.autograd.grad(out, (qs, ks, vs), dout) if backward else ())

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            once()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            keep = once()
        graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            graph.replay()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        del graph, keep
        return ms
    except Exception as e:  # the eager measurement does not depend on this one
        print(f"bench.py: graph replay not measured: {e}", file=sys.stderr)
        return None


def run_config(name, steps, warmup, args, dev, cpu_budget_s):
    """Measures one configuration: K timed steps, then per-stage and per-kernel timings, the roofline object of its
    dominant kernel and (cpu_budget_s > 0) the CPU leg on a bounded sample of the same inputs."""
    import flash_moba
    from flash_moba import flash_moba_hip as hip
    from flash_moba.mean_pool import mean_pool_nosync

    seqlens, H, D, chunk, topk, backward = CONFIGS[name]
    if seqlens is None:
        seqlens = headline_seqlens()
    T, nb, max_len = sum(seqlens), len(seqlens), max(seqlens)
    dtype_name = CONFIG_DTYPE.get(name, "bf16")
    q, k, v, dout, cu = make_inputs(seqlens, H, D, chunk, 1000 + len(seqlens), dev,
                                    torch.float16 if dtype_name == "fp16" else torch.bfloat16)
    q.requires_grad_(backward), k.requires_grad_(backward), v.requires_grad_(backward)

    def step():
        out = flash_moba.flash_moba_varlen_func(q, k, v, cu, cu, max_len, max_len, chunk, topk, causal=True)
        if backward:
            q.grad = k.grad = v.grad = None
            out.backward(dout)
        return out

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / steps
    graph_ms = graph_replay_ms(q, k, v, dout, cu, max_len, chunk, topk, backward, steps)

    # ---- algorithmic work -------------------------------------------------------------
    with torch.no_grad():
        # as flash_moba_varlen_func does: the forward may use the gating's selection bits
        km0, cu_km0, _ = mean_pool_nosync(k.detach(), cu, max_len, chunk)
        co, cn, ind, _, _, selection = hip.moba_fused_topk(q.detach(), km0, cu, cu, cu_km0, max_len, max_len, topk, chunk, True,
                                                           return_raw=False, return_selection=True)
        del km0
    pairs = count_pairs(seqlens, cn, chunk, H)
    fwd_flops = 4.0 * D * pairs
    bwd_flops = 2.5 * fwd_flops
    step_flops = fwd_flops + (bwd_flops if backward else 0.0)
    sumC = sum((L + chunk - 1) // chunk for L in seqlens)
    maxC = (max_len + chunk - 1) // chunk
    pool_bytes = (T + sumC) * H * D * 2
    gate_bytes = T * H * D * 2 + sumC * H * D * 2 + T * H * topk * 4 + nb * H * maxC * 12

    # ---- per-stage times (events on the launch stream) ----------------------------------
    it = max(3, min(steps, 20))
    lg_m = flash_moba.flash_moba_interface.decide_lg_block_m(topk, chunk, max_len, True)
    scale = D ** -0.5
    qd, kd, vd = q.detach(), k.detach(), v.detach()
    km, cu_km, _ = mean_pool_nosync(kd, cu, max_len, chunk)
    t_pool = time_events(lambda: mean_pool_nosync(kd, cu, max_len, chunk), it)
    t_gate = time_events(lambda: hip.moba_fused_topk(qd, km, cu, cu, cu_km, max_len, max_len, topk, chunk, True, return_raw=False), it)
    visits = topk * (chunk // hip.fwd_key_block(chunk))  # the bound the gated path hands to the forward

    def fwd(**kw):
        return hip.moba_varlen_fwd(qd, kd, vd, None, co, cn, ind, cu, cu, None, None, None, max_len, max_len, 0.0, scale,
                                   False, True, 0.0, False, lg_m, chunk, None, _fwd_mode=args.fwd_mode, _max_visits=visits,
                                   _selection=selection, **kw)

    fwd_phase_ms = {}
    fwd()
    row_blocks = bool(hip.last_fwd_row_blocks())  # which of the two forward forms the library picks for this shape
    fwd_names = ("selection_bits", "row_blocks") if row_blocks else ("columns", "combine")

    def run_fwd_phases(run):
        run(3)
        for name, mask in zip(fwd_names, (1, 2)):
            fwd_phase_ms[name] = time_events(lambda: run(mask), it)

    fwd(_phases=run_fwd_phases)

    out, lse, _, _ = fwd()
    t_fwd = time_events(fwd, it)
    stages = {
        "mean_pool": {"ms": t_pool, "GBps": pool_bytes / t_pool / 1e6, "frac_hbm": pool_bytes / t_pool / 1e6 / PEAK_HBM_GBS},
        "topk_csc": {"ms": t_gate, "GBps": gate_bytes / t_gate / 1e6, "frac_hbm": gate_bytes / t_gate / 1e6 / PEAK_HBM_GBS},
        "attn_fwd": {"ms": t_fwd, "TFLOPs": fwd_flops / t_fwd / 1e9, "frac_mfma": fwd_flops / t_fwd / 1e9 / PEAK_BF16_TFLOPS,
                     "phases_ms": fwd_phase_ms},
    }
    # Compulsory HBM bytes of a launch: the tensors it has to read and write, once each (q, k, v, out, dout, dq, dk, dv of
    # T*H*D*2 bytes, the selection bits or the CSC lists); rows that a kernel gathers again per visit count once.  What a
    # form of a kernel writes or reads per list entry on top of that (partial results, dS tiles) is the implementation's
    # own scratch traffic and is reported beside it, not inside it.
    entries = int(cn.sum().item())
    qkv_once = T * H * D * 2
    list_bytes = entries * 4
    fwd_visits = entries * (chunk // hip.fwd_key_block(chunk))
    # kernels[name] = (ms, FLOP, compulsory bytes, scratch bytes)
    # one kernel runs both forward GEMMs: the row-block pass, or the column pass (its combine only merges partial rows)
    if row_blocks:
        kernels = {"attn_fwd_rows_kernel": (fwd_phase_ms["row_blocks"], fwd_flops, 4 * qkv_once + T * H * ((maxC + 31) // 32) * 4, 0)}
    else:
        kernels = {"attn_fwd_col_kernel": (fwd_phase_ms["columns"], fwd_flops, 3 * qkv_once + list_bytes, fwd_visits * (D * 2 + 16))}
    if backward:
        dq, dk, dv = torch.empty_like(qd), torch.empty_like(kd), torch.empty_like(vd)
        phase_ms = {}

        def run_phases(run):
            run(7)  # make the buffers consistent first
            for name, mask in (("prep", 1), ("dkdv", 2), ("dq", 4)):
                phase_ms[name] = time_events(lambda: run(mask), it)

        bwd_visits = visits * (hip.fwd_key_block(chunk) // 64)

        def bwd(**kw):
            return hip.moba_varlen_bwd(dout, qd, kd, vd, out, lse, dq, dk, dv, co, cn, ind, cu, cu, None, max_len, max_len, 0.0,
                                       scale, False, True, 0.0, False, lg_m, chunk, None, None, _dq_mode=args.dq_mode,
                                       _max_visits=bwd_visits, **kw)

        bwd(_phases=run_phases)
        t_bwd = time_events(bwd, it)
        stages["attn_bwd"] = {"ms": t_bwd, "TFLOPs": bwd_flops / t_bwd / 1e9, "frac_mfma": bwd_flops / t_bwd / 1e9 / PEAK_BF16_TFLOPS,
                              "phases_ms": phase_ms}
        # the dK/dV kernel runs four of the five backward GEMMs (S, dP, dV, dK) and writes the dS tiles for the dQ
        # kernel; when the library picks the partial-sum form of dQ (long sequences) the fifth GEMM is in it as well and
        # it writes one dQ partial row per visit instead
        if hip.last_bwd_partials():
            bwd_kb = 128 if (chunk % 128 == 0 and D > 64) else 64
            kernels["attn_bwd_dkdv_kernel"] = (phase_ms["dkdv"], 10.0 * D * pairs, 6 * qkv_once + list_bytes, entries * (chunk // bwd_kb) * (D * 2 + 4))
        else:
            kernels["attn_bwd_dkdv_kernel"] = (phase_ms["dkdv"], 8.0 * D * pairs, 6 * qkv_once + list_bytes, entries * chunk * 2)
            kernels["attn_bwd_dq_kernel"] = (phase_ms["dq"], 2.0 * D * pairs, 2 * qkv_once + list_bytes, entries * chunk * 2)
    # sort alone, on the CSC the gating produced (already sorted input; same traffic)
    t_sort = time_events(lambda: torch.ops.flash_moba._varlen_sort(co, cn, ind), it)
    sort_bytes = 2 * int(cn.sum().item()) * 4 + 2 * cn.numel() * 8
    stages["varlen_sort"] = {"ms": t_sort, "GBps": sort_bytes / t_sort / 1e6, "frac_hbm": sort_bytes / t_sort / 1e6 / PEAK_HBM_GBS}

    # ---- roofline of the dominant kernel ---------------------------------------------------
    # The bound is the roof that lies lower for this launch: the larger of flops / MFMA peak and bytes / HBM peak.
    dom = max(kernels, key=lambda n: kernels[n][0])
    d_ms, d_flops, d_bytes, d_scratch = kernels[dom]
    t_mfma_ms = d_flops / (PEAK_BF16_TFLOPS * 1e9)
    t_hbm_ms = d_bytes / (PEAK_HBM_GBS * 1e6)
    if t_hbm_ms > t_mfma_ms:
        roofline = {"kernel": dom, "bound": "hbm", "achieved": d_bytes / d_ms / 1e6, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": d_bytes / d_ms / 1e6 / PEAK_HBM_GBS}
    else:
        roofline = {"kernel": dom, "bound": "mfma", "achieved": d_flops / d_ms / 1e9, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                    "frac": d_flops / d_ms / 1e9 / PEAK_BF16_TFLOPS}
    roofline.update({"traffic": MEASURED_TRAFFIC_BYTES.get((name, dom)), "traffic_unit": "bytes/launch", "avg_launch_ms": d_ms,
                     "flops_per_launch": d_flops, "bytes_per_launch": d_bytes, "scratch_bytes_per_launch": d_scratch,
                     "frac_mfma": d_flops / d_ms / 1e9 / PEAK_BF16_TFLOPS, "frac_hbm": d_bytes / d_ms / 1e6 / PEAK_HBM_GBS})

    result = {
        "metric": "moba_fwd_bwd_effective_sparse_tflops" if backward else "moba_fwd_effective_sparse_tflops",
        "value": step_flops / ms_per_step / 1e9,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": ms_per_step,
        "graph_replay_ms_per_step": graph_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype_name,
        "data": "synthetic",
        "config": {"workload": f"{name}: varlen packed batch, {nb} sequences totalling {T} tokens "
                               f"(lengths {seqlens}), causal, {H} heads, head_dim {D}, chunk {chunk}, top-k {topk}, "
                               + ("fwd+bwd" if backward else "fwd only"),
                   "tokens": T, "heads": H, "head_dim": D, "chunk": chunk, "topk": topk},
        "frac_of_bf16_mfma_peak": step_flops / ms_per_step / 1e9 / PEAK_BF16_TFLOPS,
        "pairs": pairs,
        "flops_per_step": step_flops,
        "topk_csc_ms": t_gate,
        "stages": stages,
        "roofline": roofline,
    }
    if cpu_budget_s > 0:
        result["cpu_baseline"] = cpu_baseline(qd, kd, vd, cu, seqlens, chunk, topk, budget_s=cpu_budget_s)
    return result


def stage_summary(r):
    """The per-stage and per-kernel milliseconds of one configuration as one flat object (what a reader of the tail of
    the line looks for first)."""
    st = r["stages"]
    out = {"workload": r["config"]["workload"].split(":")[0], "dtype": r["dtype"], "ms_per_step": round(r["ms_per_step"], 4),
           "effective_sparse_tflops": round(r["value"], 1), "frac_of_bf16_mfma_peak": round(r["frac_of_bf16_mfma_peak"], 4),
           "mean_pool_ms": round(st["mean_pool"]["ms"], 4), "mean_pool_frac_hbm": round(st["mean_pool"]["frac_hbm"], 4),
           "topk_csc_ms": round(st["topk_csc"]["ms"], 4), "topk_csc_frac_hbm": round(st["topk_csc"]["frac_hbm"], 4),
           "attn_fwd_ms": round(st["attn_fwd"]["ms"], 4), "attn_fwd_frac_mfma": round(st["attn_fwd"]["frac_mfma"], 4)}
    for k, v in st["attn_fwd"]["phases_ms"].items():
        out["fwd_" + k + "_ms"] = round(v, 4)
    if "attn_bwd" in st:
        out["attn_bwd_ms"] = round(st["attn_bwd"]["ms"], 4)
        out["attn_bwd_frac_mfma"] = round(st["attn_bwd"]["frac_mfma"], 4)
        for k, v in st["attn_bwd"]["phases_ms"].items():
            out["bwd_" + k + "_ms"] = round(v, 4)
    out["varlen_sort_ms"] = round(st["varlen_sort"]["ms"], 4)
    out["varlen_sort_frac_hbm"] = round(st["varlen_sort"]["frac_hbm"], 4)
    return out



def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="headline", choices=sorted(CONFIGS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline legs")
    ap.add_argument("--no-configs", action="store_true",
                    help="headline run only: skip the `configs` array (the other BASELINE configs, measured after the headline)")
    ap.add_argument("--dq-mode", type=int, default=0, choices=(0, 1, 2),
                    help="dQ form of the per-stage timings: 0 = the library's choice (what the timed steps run), 1 = row blocks, 2 = partials")
    ap.add_argument("--fwd-mode", type=int, default=0, choices=(0, 1, 2),
                    help="forward form of the per-stage timings: 0 = the library's choice (what the timed steps run), 1 = columns, 2 = row blocks")
    ap.add_argument("--calib-copy", action="store_true",
                    help="run one plain 1 GiB device copy first, so that a counter run has a kernel of known traffic to scale by")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; --gpus N with N > 1 is not supported", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.calib_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
    result = run_config(args.config, args.steps, args.warmup, args, dev, 0.0 if args.no_cpu else 12.0)
    if args.config == "headline" and not args.no_configs:
        # every other BASELINE config that runs on the GPU, a few steps each, same measurements
        result["configs"] = []
        for name, k_steps, cpu_s in (("c2", 20, 4.0), ("c3", 10, 4.0), ("c5", 3, 4.0), ("sweep16k", 10, 0.0), ("sweep64k", 5, 0.0)):
            torch.cuda.empty_cache()
            r = run_config(name, k_steps, 2, args, dev, 0.0 if args.no_cpu else cpu_s)
            if name == "sweep16k":
                r["dense_sdpa_fwd_bwd_ms"] = dense_sdpa_ms(CONFIGS[name], dev)  # the dense baseline of the reference's benchmark
            keep = ("metric", "value", "unit", "dtype", "ms_per_step", "graph_replay_ms_per_step", "steps", "warmup", "frac_of_bf16_mfma_peak", "pairs", "flops_per_step",
                    "topk_csc_ms", "stages", "roofline", "cpu_baseline", "dense_sdpa_fwd_bwd_ms")
            entry = {"name": name, "workload": r["config"]["workload"]}
            entry.update({k: r[k] for k in keep if k in r})
            result["configs"].append(entry)
    # last keys of the line: the other configurations' stage and kernel times as flat objects, then those of the configuration that was asked for
    if "configs" in result:
        result["configs_stages_flat"] = [stage_summary({**c, "config": {"workload": c["name"] + ":"}}) for c in result["configs"]]
    result["stages_flat"] = stage_summary(result)
    result["topk_csc_ms"] = result.pop("topk_csc_ms")
    print(json.dumps(result))


if __name__ == "__main__":
    main()

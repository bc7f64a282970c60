"""Sequence-length sweep of flash_moba_varlen_func against dense causal attention.

Mirrors the reference's benchmarks/bench_flash_moba.py (batch 2, 16 heads of 128, fp16, causal,
chunk 128, top-k 8, sequence lengths 4K ... 512K, forward and backward timed separately, TFLOP/s
counted on the DENSE causal work of the same shape so that the two methods share one axis) and its
benchmarks/bench_flash_moba_memory.py (peak device memory of one forward + backward per point).  The
dense baseline is torch's scaled_dot_product_attention (its flash kernel on ROCm) where the
reference uses flash_attn_varlen_func.

    python flash-moba_amd/benchmarks/bench_flash_moba.py [--max-seqlen 524288] [--dense-max-seqlen 65536]

Prints one line per (method, sequence length) and a JSON line per sequence length.
"""
import argparse
import json
import math
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
from flash_moba import flash_moba_varlen_func  # noqa: E402


def dense_flops(batch, seqlen, headdim, nheads, causal, mode="fwd"):
    f = 4 * batch * seqlen ** 2 * nheads * headdim // (2 if causal else 1)
    return f if mode == "fwd" else (2.5 * f if mode == "bwd" else 3.5 * f)


def time_fwd_bwd(fn, inputs, repeats):
    """Mean milliseconds of the forward and of the backward alone (events on the current stream)."""
    out = fn()
    grad = torch.randn_like(out)
    torch.autograd.grad(out, inputs, grad)
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    tf = tb = 0.0
    for _ in range(repeats):
        s.record()
        out = fn()
        e.record()
        e.synchronize()
        tf += s.elapsed_time(e)
        s.record()
        torch.autograd.grad(out, inputs, grad)
        e.record()
        e.synchronize()
        tb += s.elapsed_time(e)
    return tf / repeats, tb / repeats


def peak_memory_mb(fn, inputs):
    """Peak device memory (MiB, torch.cuda.max_memory_allocated) of one forward + backward after one warm-up pass, as
    the reference's benchmarks/bench_flash_moba_memory.py:104-143 measures it: inputs and the upstream gradient included."""
    out = fn()
    grad = torch.randn_like(out)
    torch.autograd.grad(out, inputs, grad)
    del out
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    torch.cuda.reset_peak_memory_stats()
    out = fn()
    torch.autograd.grad(out, inputs, grad)
    torch.cuda.synchronize()
    return torch.cuda.max_memory_allocated() / 1024 ** 2


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--max-seqlen", type=int, default=524288)
    ap.add_argument("--dense-max-seqlen", type=int, default=65536, help="longest sequence the dense baseline is timed on")
    ap.add_argument("--chunk", type=int, default=128)
    ap.add_argument("--topk", type=int, default=8)
    ap.add_argument("--dtype", default="fp16", choices=("fp16", "bf16"))
    args = ap.parse_args()
    if not torch.cuda.is_available():
        print("no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    dtype = torch.float16 if args.dtype == "fp16" else torch.bfloat16
    batch, headdim, nheads, causal = 2, 128, 16, True
    print(f"chunk = {args.chunk}, top_k = {args.topk}, batch = {batch}, heads = {nheads}, head_dim = {headdim}, {args.dtype}")
    for seqlen in (4096, 8192, 16384, 32768, 65536, 131072, 262144, 524288):
        if seqlen > args.max_seqlen:
            break
        repeats = 2 if seqlen >= 262144 else (5 if seqlen >= 65536 else 30)
        g = torch.Generator(device=dev).manual_seed(seqlen)
        q, k, v = (torch.randn((batch * seqlen, nheads, headdim), device=dev, dtype=dtype, generator=g).requires_grad_(True)
                   for _ in range(3))
        cu = torch.arange(0, (batch + 1) * seqlen, step=seqlen, dtype=torch.int32, device=dev)
        row = {"seqlen": seqlen}
        f, b = time_fwd_bwd(lambda: flash_moba_varlen_func(q, k, v, cu, cu, seqlen, seqlen, args.chunk, args.topk, causal=causal),
                            (q, k, v), repeats)
        row["FlashMoBA"] = {"fwd_ms": f, "bwd_ms": b}
        row["FlashMoBA"]["peak_mb"] = peak_memory_mb(
            lambda: flash_moba_varlen_func(q, k, v, cu, cu, seqlen, seqlen, args.chunk, args.topk, causal=causal), (q, k, v))
        if seqlen <= args.dense_max_seqlen:
            qd, kd, vd = (t.detach().view(batch, seqlen, nheads, headdim).transpose(1, 2).requires_grad_(True) for t in (q, k, v))
            f2, b2 = time_fwd_bwd(lambda: torch.nn.functional.scaled_dot_product_attention(qd, kd, vd, is_causal=causal),
                                  (qd, kd, vd), repeats)
            row["SDPA"] = {"fwd_ms": f2, "bwd_ms": b2}
            row["SDPA"]["peak_mb"] = peak_memory_mb(lambda: torch.nn.functional.scaled_dot_product_attention(qd, kd, vd, is_causal=causal), (qd, kd, vd))
        print(f"### causal={causal}, headdim={headdim}, batch_size={batch}, seqlen={seqlen} ###")
        for method in ("FlashMoBA", "SDPA"):
            if method not in row:
                continue
            tf, tb = row[method]["fwd_ms"], row[method]["bwd_ms"]
            eff = lambda mode, ms: dense_flops(batch, seqlen, headdim, nheads, causal, mode) / (ms * 1e-3) / 1e12
            print(f"{method} fwd: {eff('fwd', tf):.2f} TFLOPs/s, time: {tf:.2f} ms, bwd: {eff('bwd', tb):.2f} TFLOPs/s, time: {tb:.2f} ms, "
                  f"fwd + bwd: {eff('fwd_bwd', tf + tb):.2f} TFLOPs/s, time: {tf + tb:.2f} ms, peak memory: {row[method]['peak_mb'] / 1024:.2f} GiB")
        if "SDPA" in row:
            row["speedup_fwd_bwd"] = (row["SDPA"]["fwd_ms"] + row["SDPA"]["bwd_ms"]) / (f + b)
        print(json.dumps(row), flush=True)
        del q, k, v
        torch.cuda.empty_cache()


if __name__ == "__main__":
    main()

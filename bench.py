"""Benchmark of the NSA hot path on one MI355X: topk_sparse_attention forward + backward.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--seqlen N] [--topk k]

A step is one forward plus one backward of topk_sparse_attention on a synthetic bf16
batch that is already resident in HBM: a single sequence of N tokens, 64 query heads,
4 KV heads, head_dim 128, 64-token blocks, top-16 causal block selection (block 0 and
the two local blocks forced, the rest uniform).  Prints ONE JSON line.

`value` is TFLOP/s on selected-block FLOPs: 4*d*block*G per valid (kv-head, token, block)
entry for the forward, 2.5x that for the backward (five matmuls).
"""
import argparse
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "native-sparse-attention-triton_amd"))

PEAK_BF16_TFLOPS = 2500.0        # MI355X dense bf16 MFMA
HQ, HKV, D, BS = 64, 4, 128, 64
# reference-published Triton timings for this exact workload (its README.md:219,229): H100 fwd + bwd, ms
H100_FWD_BWD_MS = 12.417 + 15.154


def _events_ms(fn, iters):
    """Average duration of fn() on torch's current stream (the stream the kernels are launched on)."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) / iters


def cpu_baseline():
    """Oracle (pure PyTorch restatement) on the host cores: the reference's CPU-runnable case -
    varlen [512, 1024, 512], 16 q heads / 1 kv head, d=64, block 64, top-8, fp32, forward."""
    sys.path.insert(0, ROOT)
    import oracle
    from native_sparse_attention.testing import cu_from_lens, make_topk_idx

    torch.manual_seed(0)
    cu = cu_from_lens([512, 1024, 512])
    q, k, v = torch.randn(2048, 16, 64), torch.randn(2048, 1, 64), torch.randn(2048, 1, 64)
    idx = make_topk_idx(cu, 64, 8, 1, seed=0, local_blocks=1)
    flops = 4 * 64 * 64 * 16 * int((idx >= 0).sum())
    oracle.topk_sparse_attention(q, k, v, idx, 64, cu)
    times = []
    t_end = time.perf_counter() + 15.0
    while len(times) < 5 or (time.perf_counter() < t_end and len(times) < 50):
        t0 = time.perf_counter()
        oracle.topk_sparse_attention(q, k, v, idx, 64, cu)
        times.append(time.perf_counter() - t0)
    med = statistics.median(times)
    return {
        "value": flops / med / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
        "ms": med * 1e3,
        "sample": "oracle forward fp32, cu_seqlens=[0,512,1536,2048], 16q/1kv heads, d=64, block 64, top-8; median of %d runs" % len(times),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--seqlen", type=int, default=32768)
    ap.add_argument("--topk", type=int, default=16)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: the operator path has no multi-GPU part (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    from native_sparse_attention.ops.topk_sparse_attention import _topk_sparse_attention_bwd, _topk_sparse_attention_fwd
    from native_sparse_attention.testing import cu_from_lens, make_topk_idx
    from native_sparse_attention import _lib

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    N, topk = args.seqlen, args.topk
    G = HQ // HKV
    g = torch.Generator(device=dev).manual_seed(0)
    cu = cu_from_lens([N], dev)
    q = torch.randn(N, HQ, D, generator=g, device=dev).bfloat16()
    k = torch.randn(N, HKV, D, generator=g, device=dev).bfloat16()
    v = torch.randn(N, HKV, D, generator=g, device=dev).bfloat16()
    do = torch.randn(N, HQ, D, generator=g, device=dev).bfloat16()
    idx = make_topk_idx(cu, BS, topk, HKV, seed=0, local_blocks=2)
    sm = D ** -0.5
    f_fwd = 4.0 * D * BS * G * int((idx >= 0).sum())
    f_total = 3.5 * f_fwd

    def step():
        o, lse = _topk_sparse_attention_fwd(q, k, v, idx, BS, cu, cu, N, N, sm)
        return _topk_sparse_attention_bwd(o, do, lse, q, k, v, idx, BS, cu, cu, N, N, sm)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # per-kernel durations, HIP events on the launch stream; single passes re-run on filled workspaces
    lib = _lib.load()
    ws_f = _lib.workspace(lib.nsa_topk_attn_fwd_workspace_bytes(N, 1, HKV, D), dev)
    ws_b = _lib.workspace(lib.nsa_topk_attn_bwd_workspace_bytes(N, 1, HQ, HKV, D, topk, BS), dev)
    o, lse = _topk_sparse_attention_fwd(q, k, v, idx, BS, cu, cu, N, N, sm, workspace=ws_f)
    grads = _topk_sparse_attention_bwd(o, do, lse, q, k, v, idx, BS, cu, cu, N, N, sm, workspace=ws_b)
    it = max(3, min(args.steps, 20))
    fwd = lambda ph: _topk_sparse_attention_fwd(q, k, v, idx, BS, cu, cu, N, N, sm, workspace=ws_f, phases=ph, out=(o, lse))
    bwd = lambda ph: _topk_sparse_attention_bwd(o, do, lse, q, k, v, idx, BS, cu, cu, N, N, sm, workspace=ws_b, phases=ph, out=grads)
    kern = {
        "fwd_attend": (_events_ms(lambda: fwd(2), it), 1.0 * f_fwd),        # QK^T, PV
        "bwd_prep": (_events_ms(lambda: bwd(1), it), 0.0),                  # delta + reverse index (HBM / integer)
        "bwd_dkdv": (_events_ms(lambda: bwd(2), it), 2.0 * f_fwd),          # QK^T, dO V^T, P^T dO, dS^T Q
        "bwd_dq": (_events_ms(lambda: bwd(4), it), 0.5 * f_fwd),            # dS K (its recomputed QK^T, dO V^T are not counted)
    }
    fwd_ms = _events_ms(lambda: fwd(3), it)
    bwd_ms = _events_ms(lambda: bwd(7), it)
    dom = max((n for n in kern if kern[n][1] > 0), key=lambda n: kern[n][0])
    dom_ms, dom_flops = kern[dom]
    achieved = dom_flops / dom_ms / 1e9
    line = {
        "metric": "topk_sparse_attn fwd+bwd TFLOP/s on selected-block FLOPs (N=%d, top%d)" % (N, topk),
        "value": f_total / ms_per_step / 1e9, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": (H100_FWD_BWD_MS / ms_per_step) if (N, topk) == (32768, 16) else None,
        "dtype": "bf16", "data": "synthetic",
        "config": {
            "workload": "topk_sparse_attention fwd+bwd, single sequence N=%d, 64 q / 4 kv heads, d=128, block 64, top-%d, "
                        "causal topk_idx with block 0 and two local blocks forced" % (N, topk),
            "baseline": "H100 Triton fwd+bwd ms published in the reference README (12.417 + 15.154)",
            "fwd_ms": fwd_ms, "bwd_ms": bwd_ms, "frac_of_bf16_peak": f_total / ms_per_step / 1e9 / PEAK_BF16_TFLOPS,
            "kernel_ms": {n: kern[n][0] for n in kern},
        },
        "roofline": {
            "bound": "mfma", "kernel": dom, "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
            "frac": achieved / PEAK_BF16_TFLOPS, "traffic": None,
        },
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline()
    print(json.dumps(line))


if __name__ == "__main__":
    main()

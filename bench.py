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
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "native-sparse-attention-triton_amd"))

PEAK_BF16_TFLOPS = 2500.0        # MI355X dense bf16 MFMA
PEAK_HBM_GBPS = 8000.0           # MI355X HBM3E
HQ, HKV, D, BS = 64, 4, 128, 64
# reference-published Triton timings for this exact workload (its README.md:219,229): H100 fwd + bwd, ms
H100_FWD_BWD_MS = 12.417 + 15.154
# memory-side traffic per launch at the default workload (N=32768, top16), bytes: rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE, scaled by what the same counters read for a plain 1 GiB copy (x2.0 and x1.0); see profiles/
MEASURED_TRAFFIC = {"topk_fwd_sweep_kernel": 8.38 * 2**30, "dq_sweep_kernel": 9.71 * 2**30, "dkdv_kernel": 16.15 * 2**30}


def _paced(N, topk):
    """Whether the forward and the dQ pass of a sequence of N tokens run their paced schedule (pace_pays in csrc/pace.h:
    at least 8 blocks per token and K/V rows of a kv-head that reach 12 MiB), i.e. which kernel name a profile shows."""
    return topk >= 8 and N * D * 4 >= 12 << 20


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
    """The oracle (this repository's restatement of the reference's ops/torch/topk_sparse_attention.py:19-83) on the
    host cores, on the reference's CPU-runnable configuration: fp32, cu_seqlens = [0, 512, 1536, 2048], 16 query heads,
    1 KV head, head_dim 64, block 64, top-8 with block 0 and the query's own block forced, q / k / v drawn in that order
    from torch.manual_seed(0); forward only, one warm-up, median of 7 runs, every host core torch was given.  `value`
    is in the unit of the headline metric (TFLOP/s on selected-block FLOPs)."""
    sys.path.insert(0, ROOT)
    import statistics

    import oracle
    from native_sparse_attention.testing import cu_from_lens, make_topk_idx

    torch.manual_seed(0)
    cu = cu_from_lens([512, 1024, 512])
    q, k, v = torch.randn(2048, 16, 64), torch.randn(2048, 1, 64), torch.randn(2048, 1, 64)
    idx = make_topk_idx(cu, 64, 8, 1, seed=0, local_blocks=1)
    flops = 4.0 * 64 * 64 * 16 * int((idx >= 0).sum())
    times = []
    with torch.no_grad():
        for i in range(8):
            t0 = time.perf_counter()
            oracle.topk_sparse_attention(q, k, v, idx, 64, cu)
            if i > 0:
                times.append(time.perf_counter() - t0)
    med = statistics.median(times)
    out = {
        "value": flops / med / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port", "ms": med * 1e3,
        "sample": "oracle forward, fp32, cu_seqlens=[0,512,1536,2048], 16 q / 1 kv heads, d=64, block 64, top-8 "
                  "(block 0 and own block forced), seed 0; 1 warm-up, median of 7 runs",
    }
    if torch.cuda.is_available():
        # the same inputs (cast to bf16) through the HIP operator, for the record beside the host figure
        from native_sparse_attention.ops import topk_sparse_attention
        dev = torch.device("cuda:0")
        qg, kg, vg, ig, cg = q.bfloat16().to(dev), k.bfloat16().to(dev), v.bfloat16().to(dev), idx.to(dev), cu.to(dev)
        with torch.no_grad():
            for _ in range(3):
                topk_sparse_attention(qg, kg, vg, ig, 64, cg)
            torch.cuda.synchronize()
            gpu_ms = _events_ms(lambda: topk_sparse_attention(qg, kg, vg, ig, 64, cg), 20)
        out["gpu_ms_same_inputs_bf16"] = gpu_ms
        out["gpu_over_cpu"] = med * 1e3 / gpu_ms
    return out


def _mfma_roofline(ops, whole_tflops):
    """roofline object for a workload made of several operators: ops = [(name, ms, algorithmic FLOPs)]; the entry is the
    MFMA-bound operator that takes the most time."""
    rows = [{"kernel": n, "ms": ms, "algorithmic_flops": f, "tflops": f / ms / 1e9 if f else None,
             "frac": f / ms / 1e9 / PEAK_BF16_TFLOPS if f else None} for n, ms, f in ops]
    dom = max((r for r in rows if r["algorithmic_flops"]), key=lambda r: r["ms"])
    return {"bound": "mfma", "kernel": dom["kernel"], "achieved": dom["tflops"], "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
            "frac": dom["frac"], "traffic": None, "step_frac": whole_tflops / PEAK_BF16_TFLOPS, "kernels": rows}


def _time_ms(fn, iters, warm=2):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    return _events_ms(fn, iters)


def bench_pipeline(args, dev):
    """Pipeline benchmark: linear_compress -> compressed_attention (+selection) -> topk_sparse_attention, forward, bf16."""
    from native_sparse_attention.ops import compressed_attention, linear_compress, topk_sparse_attention
    from native_sparse_attention.ops.compressed_attention import _compressed_attention_fwd, _select_blocks
    from native_sparse_attention.testing import cu_from_lens

    g = torch.Generator(device=dev).manual_seed(0)
    cu = cu_from_lens([1024, 7168, 8192], dev)
    T, ks, st, bs, topk = 16384, 32, 16, 64, 16
    q = torch.randn(T, HQ, D, generator=g, device=dev).bfloat16()
    k = torch.randn(T, HKV, D, generator=g, device=dev).bfloat16()
    v = torch.randn(T, HKV, D, generator=g, device=dev).bfloat16()
    wk = (torch.randn(HKV, ks * D, D, generator=g, device=dev) / (ks * D) ** 0.5).bfloat16()
    wv = (torch.randn(HKV, ks * D, D, generator=g, device=dev) / (ks * D) ** 0.5).bfloat16()
    pe = (0.02 * torch.randn(HKV, ks, D, generator=g, device=dev)).bfloat16()
    it = args.steps
    with torch.no_grad():
        ck, cuk = linear_compress(k, wk, cu, ks, st, pe)
        cv, _ = linear_compress(v, wv, cu, ks, st)
        o_c, idx = compressed_attention(q, ck, cv, ks, st, bs, topk, cu, cuk, 8192, 511)
        o_c2, lse = _compressed_attention_fwd(q, ck, cv, ks, st, cu, cuk, 8192, 511, D ** -0.5)
        t_lin = _time_ms(lambda: (linear_compress(k, wk, cu, ks, st, pe), linear_compress(v, wv, cu, ks, st)), it)
        t_cmp = _time_ms(lambda: _compressed_attention_fwd(q, ck, cv, ks, st, cu, cuk, 8192, 511, D ** -0.5), it)
        t_sel = _time_ms(lambda: _select_blocks(q, ck, lse, ks, st, bs, topk, cu, cuk, 8192, 1, 2, D ** -0.5), it)
        t_top = _time_ms(lambda: topk_sparse_attention(q, k, v, idx, bs, cu), it)

        def whole():
            a, c = linear_compress(k, wk, cu, ks, st, pe)
            b, _ = linear_compress(v, wv, cu, ks, st)
            _, i2 = compressed_attention(q, a, b, ks, st, bs, topk, cu, c, 8192, 511)
            return topk_sparse_attention(q, k, v, i2, bs, cu)
        t_all = _time_ms(whole, it)
    lens = [1024, 7168, 8192]
    pairs = sum(sum((i - ks + 1) // st + 1 for i in range(ks - 1, L)) for L in lens)
    f_lin = 2 * 2.0 * int(cuk[-1]) * ks * D * D * HKV
    f_cmp = 4.0 * D * HQ * pairs
    f_top = 4.0 * D * bs * (HQ // HKV) * int((idx >= 0).sum())
    ops = [("linear_compress (K and V: lin_fwd_kernel, two launches)", t_lin, f_lin),
           ("compressed_attention forward (cmp_fwd_kernel)", t_cmp, f_cmp),
           ("block selection (cmp_select_kernel; recomputes the scores: no algorithmic FLOPs of its own)", t_sel, 0.0),
           ("topk_sparse_attention forward (retile_pair_kernel + topk_fwd_kernel)", t_top, f_top)]
    roof = _mfma_roofline(ops, (f_lin + f_cmp + f_top) / t_all / 1e9)
    return {
        "roofline": roof,
        "metric": "NSA op pipeline forward ms (linear_compress x2 + compressed_attention w/ selection + topk_sparse_attention)",
        "value": t_all, "unit": "ms", "n_gpus": 1, "steps": it, "warmup": 2, "ms_per_step": t_all, "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "cu_seqlens=[0,1024,8192,16384], 64q/4kv heads, d=128, kernel 32 stride 16, block 64, top-16",
                   "ms": {"linear_compress_kv": t_lin, "compressed_attention_fwd": t_cmp, "block_selection": t_sel, "topk_sparse_attention_fwd": t_top},
                   "tflops": {"linear_compress_kv": f_lin / t_lin / 1e9, "compressed_attention_fwd": f_cmp / t_cmp / 1e9,
                              "topk_sparse_attention_fwd": f_top / t_top / 1e9}},
    }


def bench_compressed(args, dev):
    """Long-sequence benchmark: weightedpool compression + compressed_attention forward+backward, N=65536, 32q/2kv."""
    from native_sparse_attention.ops import compressed_attention, weightedpool_compress
    from native_sparse_attention.ops.compressed_attention import _compressed_attention_bwd, _compressed_attention_fwd, _select_blocks
    from native_sparse_attention.testing import cu_from_lens

    N, ks, st, bs, topk = 65536, 32, 16, 64, 16
    Hq, Hkv = (64, 4) if args.readme_heads else (32, 2)
    g = torch.Generator(device=dev).manual_seed(0)
    cu = cu_from_lens([N], dev)
    q = torch.randn(N, Hq, D, generator=g, device=dev).bfloat16().requires_grad_()
    k = torch.randn(N, Hkv, D, generator=g, device=dev).bfloat16().requires_grad_()
    v = torch.randn(N, Hkv, D, generator=g, device=dev).bfloat16().requires_grad_()
    wk = torch.softmax(torch.randn(Hkv, ks, generator=g, device=dev), -1).bfloat16().requires_grad_()
    wv = torch.softmax(torch.randn(Hkv, ks, generator=g, device=dev), -1).bfloat16().requires_grad_()
    do = torch.randn(N, Hq, D, generator=g, device=dev).bfloat16()
    it = max(2, min(args.steps, 5))

    def step():
        ck, cuk = weightedpool_compress(k, wk, cu, ks, st)
        cv, _ = weightedpool_compress(v, wv, cu, ks, st)
        o, idx = compressed_attention(q, ck, cv, ks, st, bs, topk, cu, cuk, N, 4095)
        o.backward(do)
        return idx
    t_all = _time_ms(step, it, warm=1)
    with torch.no_grad():
        ck, cuk = weightedpool_compress(k, wk, cu, ks, st)
        cv, _ = weightedpool_compress(v, wv, cu, ks, st)
        o, lse = _compressed_attention_fwd(q, ck, cv, ks, st, cu, cuk, N, 4095, D ** -0.5)
        t_pool = _time_ms(lambda: weightedpool_compress(k, wk, cu, ks, st), it)
        t_fwd = _time_ms(lambda: _compressed_attention_fwd(q, ck, cv, ks, st, cu, cuk, N, 4095, D ** -0.5), it)
        t_sel = _time_ms(lambda: _select_blocks(q, ck, lse, ks, st, bs, topk, cu, cuk, N, 1, 2, D ** -0.5), it)
        t_bwd = _time_ms(lambda: _compressed_attention_bwd(o, do, lse, q, ck, cv, ks, st, cu, cuk, N, 4095, D ** -0.5), it)
    pairs = sum((i - ks + 1) // st + 1 for i in range(ks - 1, N))
    f_fwd = 4.0 * D * Hq * pairs
    pool_bytes = (N * Hkv * D + 4095 * Hkv * D) * 2
    ops = [("compressed_attention forward (cmp_fwd_kernel)", t_fwd, f_fwd),
           ("block selection (cmp_select_kernel; recomputes the scores: no algorithmic FLOPs of its own)", t_sel, 0.0),
           ("compressed_attention backward (dkdv_kernel over query ranges + dkdv_reduce_kernel + cmp_dq_kernel)", t_bwd, 2.5 * f_fwd)]
    roof = _mfma_roofline(ops, 3.5 * f_fwd / t_all / 1e9)
    roof["hbm_kernels"] = [{"kernel": "weightedpool forward, one tensor (pool_fwd_split_kernel; wrapper time, includes the length bookkeeping launch)",
                            "ms": t_pool, "algorithmic_bytes": pool_bytes, "GBps": pool_bytes / t_pool / 1e6, "peak": PEAK_HBM_GBPS,
                            "frac": pool_bytes / t_pool / 1e6 / PEAK_HBM_GBPS}]
    return {
        "roofline": roof,
        "metric": "weightedpool + compressed_attention fwd+bwd ms (N=65536)", "value": t_all, "unit": "ms", "n_gpus": 1, "steps": it,
        "warmup": 1, "ms_per_step": t_all, "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "single sequence N=65536, %dq/%dkv heads, d=128, kernel 32 stride 16, block 64, top-16" % (Hq, Hkv),
                   # H100 Triton, 64q/4kv, N=65536 (reference README): forward with scoring 53.009, without 16.134, backward 46.054
                   "h100_triton_ms_64q4kv": {"fwd_with_selection": 53.009, "fwd_without_selection": 16.134, "bwd": 46.054},
                   "ms": {"weightedpool_fwd_one_tensor": t_pool, "compressed_attention_fwd": t_fwd, "block_selection": t_sel,
                          "compressed_attention_bwd": t_bwd},
                   "tflops": {"compressed_attention_fwd": f_fwd / t_fwd / 1e9, "compressed_attention_bwd": 2.5 * f_fwd / t_bwd / 1e9},
                   "gbps": {"weightedpool_fwd": pool_bytes / t_pool / 1e6}},
    }


def bench_decode(args, dev):
    """Decode benchmark: one NSA decode step over the cache slabs (three branches + sigmoid gates)."""
    from native_sparse_attention.infer import nsa_infer
    from native_sparse_attention.module import NSACache
    from native_sparse_attention.ops import weightedpool_compress
    from native_sparse_attention.testing import cu_from_lens

    Hq, Hkv, ks, st, bs, topk, W = 32, 2, 32, 16, 64, 8, 512
    lens = [2048, 4096, 6144, 8192]
    B = len(lens)
    g = torch.Generator(device=dev).manual_seed(0)
    cu = cu_from_lens(lens, dev)
    T = int(cu[-1])
    q = torch.randn(T, Hq, D, generator=g, device=dev).bfloat16()
    k = torch.randn(T, Hkv, D, generator=g, device=dev).bfloat16()
    v = torch.randn(T, Hkv, D, generator=g, device=dev).bfloat16()
    gate = torch.sigmoid(torch.randn(T, Hq, 3, generator=g, device=dev)).bfloat16()
    wk = torch.softmax(torch.randn(Hkv, ks, generator=g, device=dev), -1).bfloat16()
    wv = torch.softmax(torch.randn(Hkv, ks, generator=g, device=dev), -1).bfloat16()
    from native_sparse_attention.module import RopeConfig, RotaryEmbedding
    rope = RotaryEmbedding(RopeConfig(head_dim=D), device=dev)  # llama3 rotary embedding, as the layer applies it
    steps = max(4, args.steps)
    cache = NSACache(B, max(lens) + 3 * steps + 16, Hkv, D, ks, st, W, torch.bfloat16, dev)
    fargs = (rope, cache, (wk, wv), (weightedpool_compress, weightedpool_compress), None, ks, st, bs, topk, 1, 2, W)
    with torch.no_grad():
        nsa_infer(cu, 0, q, k, v, gate, *fargs)
        qd = torch.randn(B, Hq, D, generator=g, device=dev).bfloat16()
        kd = torch.randn(B, Hkv, D, generator=g, device=dev).bfloat16()
        vd = torch.randn(B, Hkv, D, generator=g, device=dev).bfloat16()
        gd = torch.sigmoid(torch.randn(B, Hq, 3, generator=g, device=dev)).bfloat16()
        nsa_infer(cu, 1, qd, kd, vd, gd, *fargs)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for s in range(2, steps + 2):
            nsa_infer(cu, s, qd, kd, vd, gd, *fargs)
        torch.cuda.synchronize()
        us_eager = (time.perf_counter() - t0) * 1e6 / steps
        # the same step recorded once in a HIP graph and replayed (inputs copied into the graph's buffers)
        from native_sparse_attention.infer import NSADecodeGraph
        graph = NSADecodeGraph(cu, Hq, *fargs)
        for _ in range(2):
            graph.step(qd, kd, vd, gd)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            graph.step(qd, kd, vd, gd)
        torch.cuda.synchronize()
        us = (time.perf_counter() - t0) * 1e6 / steps
        # a caller whose projections write straight into the graph's input buffers skips the four copies
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            graph.replay()
        torch.cuda.synchronize()
        us_inplace = (time.perf_counter() - t0) * 1e6 / steps
        # the three attention kernels alone, on the final cache state
        from native_sparse_attention.ops import compressed_attention_decode, flash_attention_decode, topk_sparse_attention_decode
        seqlens = cache.sparse_kv_len[:B].clone()
        rows = int(cache.compress_kv_len[:B].max())
        o1, idx = compressed_attention_decode(qd, cache.compress_kv_cache[0, :B, :rows], cache.compress_kv_cache[1, :B, :rows],
                                              seqlens, cache.compress_kv_len[:B], ks, st, bs, topk)
        t_c = _time_ms(lambda: compressed_attention_decode(qd, cache.compress_kv_cache[0, :B, :rows], cache.compress_kv_cache[1, :B, :rows],
                                                           seqlens, cache.compress_kv_len[:B], ks, st, bs, topk), 20)
        t_s = _time_ms(lambda: topk_sparse_attention_decode(qd, cache.sparse_kv_cache[0, :B], cache.sparse_kv_cache[1, :B], idx, bs, seqlens), 20)
        wl = torch.clamp(cache.sliding_kv_len[:B], max=W)
        t_w = _time_ms(lambda: flash_attention_decode(qd, cache.sliding_kv_cache[0, :B], cache.sliding_kv_cache[1, :B], wl), 20)
    key_rows = int(cache.compress_kv_len[:B].sum()) + 64 * int((idx >= 0).sum()) // Hkv + B * W
    alg_bytes = 2 * Hkv * D * 2 * key_rows
    step_bytes = alg_bytes + 2 * B * (Hq + 2 * Hkv) * D * 2 + B * Hq * 3 * 2       # keys and values read + q, k, v, gate in and the output
    roof = {"bound": "hbm", "kernel": "whole decode step (5 dependent launches, replayed from a HIP graph)", "achieved": step_bytes / us / 1e3,
            "peak": PEAK_HBM_GBPS, "unit": "GB/s", "frac": step_bytes / us / 1e3 / PEAK_HBM_GBPS, "traffic": None, "algorithmic_bytes": step_bytes,
            "note": "a decode step moves a few MiB: it is bound by the latency of its dependent launches, not by bandwidth",
            "kernels": [{"kernel": n, "us": t * 1e3, "GBps": bts / t / 1e6} for n, t, bts in (
                ("compressed_attention_decode (decode_partial_kernel + decode_score_select_kernel)", t_c, 2 * Hkv * D * 2 * int(cache.compress_kv_len[:B].sum())),
                ("topk_sparse_attention_decode (decode_partial_kernel + decode_merge_kernel)", t_s, 2 * Hkv * D * 2 * 64 * int((idx >= 0).sum()) // Hkv),
                ("flash_attention_decode over the window (decode_partial_kernel + decode_merge_kernel)", t_w, 2 * Hkv * D * 2 * B * W))]}
    return {
        "roofline": roof,
        "metric": "NSA decode step latency (us, cache update + compression + rope + three branches + gate), B=4, cached lens 2K..8K", "value": us, "unit": "us", "n_gpus": 1, "steps": steps,
        "warmup": 2, "ms_per_step": us / 1e3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "32q/2kv heads, d=128, weightedpool kernel 32 stride 16, block 64, top-8, window 512, sigmoid gates",
                   "us": {"full_step_graph_replay": us, "full_step_graph_replay_inputs_in_place": us_inplace,
                          "full_step_eager_launches": us_eager,
                          "compressed_decode_with_selection": t_c * 1e3,
                          "topk_decode": t_s * 1e3, "window_decode": t_w * 1e3},
                   "algorithmic_kv_bytes": alg_bytes, "gbps_three_kernels": alg_bytes / ((t_c + t_s + t_w) * 1e-3) / 1e9},
    }


def bench_layer(args, dev):
    """Layer benchmark of the reference's test/test_nsa_module.py:20-60,103-150: NativeSparseAttention against the dense
    SelfAttention layer, hidden 8192, 64q/4kv heads, d=128, one sequence of --seqlen tokens; forward (no grad) and
    forward + backward.  The projections are rocBLAS GEMMs (plumbing); everything else runs on this library's kernels."""
    from native_sparse_attention.module import NativeSparseAttention, RopeConfig, SelfAttention

    rope = RopeConfig(max_position_embeddings=131072, head_dim=D, rope_theta=500000,
                      rope_scaling={"factor": 8.0, "high_freq_factor": 4.0, "low_freq_factor": 1.0,
                                    "original_max_position_embeddings": 8192, "rope_type": "llama3"})
    torch.manual_seed(42)
    nsa = NativeSparseAttention(compress_type="avgpool", hidden_size=8192, num_q_heads=HQ, num_kv_heads=HKV, head_dim=D,
                                kernel_size=32, kernel_stride=16, block_size=BS, topk=16, init_blocks=1, local_blocks=2,
                                window_size=512, rope_config=rope).to(dev).to(torch.bfloat16)
    dense = SelfAttention(hidden_size=8192, num_q_heads=HQ, num_kv_heads=HKV, head_dim=D, rope_config=rope).to(dev).to(torch.bfloat16)
    N = args.seqlen
    x = torch.randn(N, 8192, device=dev, dtype=torch.bfloat16)
    cu = torch.tensor([0, N], device=dev, dtype=torch.int32)
    xg = x.clone().requires_grad_()
    it = max(2, min(args.steps, 5))

    def fwd_bwd(layer):
        y = layer(xg, cu)
        (y * y).sum().backward()
    with torch.no_grad():
        t_nsa_f = _time_ms(lambda: nsa(x, cu), it)
        t_dense_f = _time_ms(lambda: dense(x, cu), it)
    t_nsa = _time_ms(lambda: fwd_bwd(nsa), it)
    t_dense = _time_ms(lambda: fwd_bwd(dense), it)
    return {
        "metric": "NSA attention layer forward+backward ms (hidden 8192, N=%d)" % N, "value": t_nsa, "unit": "ms", "n_gpus": 1,
        "steps": it, "warmup": 2, "ms_per_step": t_nsa, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "NativeSparseAttention layer, hidden 8192, 64q/4kv heads, d=128, avgpool kernel 32 stride 16, block 64, "
                               "top-16, window 512, one sequence of %d tokens" % N,
                   "ms": {"nsa_forward": t_nsa_f, "nsa_forward_backward": t_nsa, "dense_self_attention_forward": t_dense_f,
                          "dense_self_attention_forward_backward": t_dense}},
    }


def measure_topk(N, topk, steps, warmup, dev, per_kernel):
    """One point of the top-k sweep: forward + backward of topk_sparse_attention on a single sequence of N tokens (64 q / 4 kv
    heads, d=128, block 64), inputs resident in HBM.  ms_per_step: wall clock over `steps` steps after `warmup`; fwd_ms /
    bwd_ms and (per_kernel) the duration of every kernel of the step: HIP events on the launch stream, single passes
    re-run on filled workspaces."""
    from native_sparse_attention import _lib
    from native_sparse_attention.ops.topk_sparse_attention import _topk_sparse_attention_bwd, _topk_sparse_attention_fwd
    from native_sparse_attention.testing import cu_from_lens, make_topk_idx

    G = HQ // HKV
    g = torch.Generator(device=dev).manual_seed(0)
    cu = cu_from_lens([N], dev)
    q = torch.randn(N, HQ, D, generator=g, device=dev).bfloat16()
    k = torch.randn(N, HKV, D, generator=g, device=dev).bfloat16()
    v = torch.randn(N, HKV, D, generator=g, device=dev).bfloat16()
    do = torch.randn(N, HQ, D, generator=g, device=dev).bfloat16()
    idx = make_topk_idx(cu, BS, topk, HKV, seed=0, local_blocks=2)
    sm = D ** -0.5
    n_pairs = int((idx >= 0).sum())
    f_fwd = 4.0 * D * BS * G * n_pairs

    def step():
        o, lse = _topk_sparse_attention_fwd(q, k, v, idx, BS, cu, cu, N, N, sm)
        return _topk_sparse_attention_bwd(o, do, lse, q, k, v, idx, BS, cu, cu, N, N, sm)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / steps

    lib = _lib.load()
    ws_f = _lib.workspace(lib.nsa_topk_attn_fwd_workspace_bytes(N, 1, HKV, D), dev)
    ws_b = _lib.workspace(lib.nsa_topk_attn_bwd_workspace_bytes(N, 1, HQ, HKV, D, topk, BS), dev)
    o, lse = _topk_sparse_attention_fwd(q, k, v, idx, BS, cu, cu, N, N, sm, workspace=ws_f)
    grads = _topk_sparse_attention_bwd(o, do, lse, q, k, v, idx, BS, cu, cu, N, N, sm, workspace=ws_b)
    it = max(3, min(steps, 20))
    fwd = lambda ph: _topk_sparse_attention_fwd(q, k, v, idx, BS, cu, cu, N, N, sm, workspace=ws_f, phases=ph, out=(o, lse))
    bwd = lambda ph: _topk_sparse_attention_bwd(o, do, lse, q, k, v, idx, BS, cu, cu, N, N, sm, workspace=ws_b, phases=ph, out=grads)
    out = {"f_fwd": f_fwd, "ms_per_step": ms_per_step, "fwd_ms": _events_ms(lambda: fwd(3), it), "bwd_ms": _events_ms(lambda: bwd(7), it)}
    if per_kernel:
        qb, kvb = q.numel() * 2, k.numel() * 2                 # bytes of one [N,64,128] and of one [N,4,128] tensor
        small = idx.numel() * 4 + 2 * HQ * N * 4               # block ids, lse / delta
        out["kernels"] = {
            # name: (ms, algorithmic FLOPs per launch, bytes the kernel must read or write at least once)
            "topk_fwd_sweep_kernel" if _paced(N, topk) else "topk_fwd_kernel": (_events_ms(lambda: fwd(2), it), 1.0 * f_fwd, 2 * qb + 2 * kvb + small),   # QK^T, PV
            "dq_sweep_kernel" if _paced(N, topk) else "dq_kernel": (_events_ms(lambda: bwd(4), it), 0.5 * f_fwd, 4 * qb + 2 * kvb + small),            # dS K (recomputed QK^T, dO V^T not counted)
            "dkdv_kernel": (_events_ms(lambda: bwd(2), it), 2.0 * f_fwd, 2 * qb + 4 * kvb + small),       # QK^T, dO V^T, P^T dO, dS^T Q
            "reverse_index": (_events_ms(lambda: bwd(1), it) , 0.0, None),   # run alone this phase also holds the stand-alone delta pass
        }
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--seqlen", type=int, default=32768)
    ap.add_argument("--topk", type=int, default=16)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-sweep", action="store_true", help="skip the N x top-k sweep table (config.sweep)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three plain 1 GiB device copies (reference point for FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--readme-heads", action="store_true",
                    help="compressed workload with the 64q/4kv head layout of the reference README tables instead of config 3's 32q/2kv")
    ap.add_argument("--workload", default="topk", choices=["topk", "pipeline", "compressed", "decode", "layer"],
                    help="topk = the headline metric (default); the others time the pipeline, long-sequence compressed-attention, decode and whole-layer benchmarks")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: the operator path has no multi-GPU part (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import __graft_entry__
    __graft_entry__.ensure_built()  # uses the library that is built; compiles only when it is missing or older than its sources
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.workload != "topk":
        fn = {"pipeline": bench_pipeline, "compressed": bench_compressed, "decode": bench_decode, "layer": bench_layer}[args.workload]
        print(json.dumps(fn(args, dev)))
        return
    N, topk = args.seqlen, args.topk
    r = measure_topk(N, topk, args.steps, args.warmup, dev, per_kernel=True)
    f_fwd, ms_per_step, kern = r["f_fwd"], r["ms_per_step"], r["kernels"]
    f_total = 3.5 * f_fwd
    headline = (N, topk) == (32768, 16)
    kernels = []
    for name, (ms, flops, unique) in kern.items():
        traffic = MEASURED_TRAFFIC.get(name) if headline else None
        kernels.append({
            "kernel": name, "ms": ms, "algorithmic_flops": flops, "tflops": flops / ms / 1e9 if flops else None,
            "frac": flops / ms / 1e9 / PEAK_BF16_TFLOPS if flops else None,
            "unique_bytes": unique, "traffic": traffic, "traffic_over_unique": traffic / unique if traffic and unique else None,
        })
    mfma = [x for x in kernels if x["algorithmic_flops"]]
    dom = max(mfma, key=lambda x: x["ms"])   # the kernel that takes the most time
    line = {
        "metric": "topk_sparse_attn fwd+bwd TFLOP/s on selected-block FLOPs (N=%d, top%d)" % (N, topk),
        "value": f_total / ms_per_step / 1e9, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": (H100_FWD_BWD_MS / ms_per_step) if headline else None,
        "dtype": "bf16", "data": "synthetic",
        "config": {
            "workload": "topk_sparse_attention fwd+bwd, single sequence N=%d, 64 q / 4 kv heads, d=128, block 64, top-%d, "
                        "causal topk_idx with block 0 and two local blocks forced" % (N, topk),
            "baseline": "H100 Triton fwd+bwd ms published in the reference README (12.417 + 15.154)",
            "fwd_ms": r["fwd_ms"], "bwd_ms": r["bwd_ms"], "frac_of_bf16_peak": f_total / ms_per_step / 1e9 / PEAK_BF16_TFLOPS,
        },
        "roofline": {
            "bound": "mfma", "kernel": dom["kernel"], "achieved": dom["tflops"], "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
            "frac": dom["frac"], "traffic": dom["traffic"], "unique_bytes": dom["unique_bytes"],
            "traffic_over_unique": dom["traffic_over_unique"],
            "note": "kernel = the MFMA kernel with the largest measured duration; achieved = its algorithmic FLOPs per launch / "
                    "its duration (HIP events on the launch stream); traffic = L2<->memory-side bytes per launch from rocprofv3 "
                    "--pmc FETCH_SIZE / WRITE_SIZE (profiles/), unique_bytes = what the kernel must read and write at least once",
            "step_frac": f_total / ms_per_step / 1e9 / PEAK_BF16_TFLOPS,
            "kernels": kernels,
        },
    }
    if not args.no_sweep:
        sweep = []
        for n in (2048, 4096, 8192, 16384, 32768, 65536, 131072):
            for kk in (8, 16):
                m = r if (n, kk) == (N, topk) else measure_topk(n, kk, max(3, min(args.steps, 10)), 2, dev, per_kernel=False)
                sweep.append({"N": n, "topk": kk, "fwd_ms": round(m["fwd_ms"], 4), "bwd_ms": round(m["bwd_ms"], 4),
                              "fwd_bwd_ms": round(m["ms_per_step"], 4), "tflops": round(3.5 * m["f_fwd"] / m["ms_per_step"] / 1e9, 1)})
        line["config"]["sweep"] = sweep
    if args.calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)  # 1 GiB read + 1 GiB written per launch
        torch.cuda.synchronize()
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline()
    print(json.dumps(line))


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Benchmark of the paged-KV decode attention hot path on one MI355X.

Workload (BASELINE.json configs[1]): one Llama-3-8B-shaped attention layer in decode,
batch 64, 32 query / 8 KV heads, head_dim 128, block_size 64, context lengths
U[3584, 4608], int8 KV cache with per-channel scales, block tables a random
permutation over a 6000-block pool.  A "step" is one decode-attention pass over the
batch (split-KV kernel + merge kernel); inputs are resident in HBM.

Prints ONE JSON line.  `value` is microseconds per layer for the whole op;
`roofline` prices the dominant (split-KV) kernel against the 8 TB/s HBM peak with
the algorithmic bytes of the pass; `cpu_baseline` is the CPU oracle timed on this
host's cores on the same workload.
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes per algorithmic byte of one decode_c8_kernel launch on this workload, from the TCC counters (rocprofv3
# --pmc FETCH_SIZE, then WRITE_SIZE, each scaled by a 1 GiB copy in the same run): the summary file below holds the
# figures; the counters cannot be read from inside this script, so the ratio measured there is applied to this
# run's algorithmic bytes.
TRAFFIC_PROFILE = "profiles/decode_c8_kernel_configs1_b64_ctx4k.md"
TRAFFIC_PER_ALGORITHMIC_BYTE = 1.0089
# The same profile's kernel trace holds this script's one-by-one launches too (each follows an idle queue): the median of
# the profiler's own begin-to-end durations of those launches, as a fraction of the HBM peak over configs[1]'s bytes.
ISOLATED_PROFILE = TRAFFIC_PROFILE + ": decode_c8_kernel launches that follow an idle queue, profiler's durations, median 83.19 us"
ISOLATED_FRAC_PROFILED = 0.8034


def time_events(fn, steps, warmup):
    """Average milliseconds per call over `steps` back-to-back calls on torch's current stream
    (the stream the kernels are launched on), bracketed by HIP events and device syncs."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def time_each(fn, steps):
    """The same launches with an event between every two of them (still back to back on the stream, no host sync
    inside): the per-launch durations in milliseconds, for the median and the minimum beside the mean."""
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    torch.cuda.synchronize()
    ev[0].record()
    for i in range(steps):
        fn()
        ev[i + 1].record()
    torch.cuda.synchronize()
    return sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(steps))


def pick_context_lengths(batch, lo, hi, target_mean, tol=0.01):
    """ctx ~ U{lo..hi} from the first seed whose draw has a mean within tol of the configuration's mean (a draw of 64
    lengths is off by up to 3 %, which would flatter or penalise the microseconds per layer)."""
    for seed in range(1000):
        lens = torch.randint(lo, hi + 1, (batch,), generator=torch.Generator().manual_seed(seed)).tolist()
        if abs(sum(lens) / batch - target_mean) <= tol * target_mean:
            return lens, seed
    raise RuntimeError("no seed gives a mean within %g of %g" % (tol, target_mean))


def time_graph(fn, steps, per_graph=10):
    """The same average with the host taken out: `per_graph` calls captured in one HIP graph, replayed
    steps / per_graph times.  For ops whose kernels are shorter than the Python call that launches them."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(per_graph):
            fn()
    n = max(steps // per_graph, 2)
    return time_events(graph.replay, n, 2) / per_graph


def other_workloads(args):
    """The rows of the path that are not the headline metric (configs[2], [3], [4]): one JSON line each
    with the kernel time and its roofline fraction.  Not part of the default run."""
    import fastdeploy_amd as fd
    from fastdeploy_amd import synthetic as syn
    dev = "cuda:0"
    res = []
    g = torch.Generator(device=dev).manual_seed(0)

    def line(name, ms, bound, work, peak, unit, extra=None):
        ach = work / (ms * 1e-3) / (1e9 if unit == "GB/s" else 1e12)
        d = {"workload": name, "us": round(ms * 1e3, 2),
             "roofline": {"bound": bound, "achieved": round(ach, 1), "peak": peak, "unit": unit, "frac": round(ach / peak, 4)}}
        if extra:
            d.update(extra)
        print(json.dumps(d))
        res.append(d)

    if args.workload in ("write_decode", "all"):
        # configs[2]: 256 new tokens, positions U{0..8191}, RoPE theta 500000, int8 write, then decode over ctx = pos + 1
        c = syn.write_case(num_seqs=256, max_pos=8192, seed=0, device=dev, blocks_per_seq=128)
        rot = (c["rope_cos"], c["rope_sin"])
        ws = fd.decode_workspace(256, 32, 8, 128, 128, dev)

        def wr():
            return fd.write_cache_kv(c["qkv"], c["key_cache"], c["value_cache"], c["cache_k_scale"], c["cache_v_scale"],
                                     c["block_tables"], c["seq_lens_encoder"], c["seq_lens_decoder"], c["seq_lens_this_time"],
                                     c["cu_seqlens_q"], rot, num_heads=32, kv_num_heads=8)
        q = wr()[0]
        ms = time_events(wr, args.steps, args.warmup)
        line("configs[2] cache write (256 tokens, RoPE + int8)", ms, "hbm", 256 * (48 * 128 * 2 + 2 * 8 * 128 + 32 * 128 * 2),
             HBM_PEAK_GBPS, "GB/s", {"note": "5.8 MB of traffic: bound by the Python call that launches it",
                                     "us_from_a_hip_graph": round(time_graph(wr, args.steps) * 1e3, 2)})
        # the same kernel at prefill size: 2 sequences x 2048 new tokens behind 8192 cached ones (configs[4]'s write),
        # with the rotated K and the V handed on for the append attention - large enough to be HBM-bound
        cw = syn.write_case(num_seqs=2, max_pos=8192 + 2048, seed=1, device=dev, chunk=2048, blocks_per_seq=160)
        cw["seq_lens_decoder"].fill_(8192)
        rotw = (cw["rope_cos"], cw["rope_sin"])

        def wr_big():
            return fd.write_cache_kv(cw["qkv"], cw["key_cache"], cw["value_cache"], cw["cache_k_scale"], cw["cache_v_scale"],
                                     cw["block_tables"], cw["seq_lens_encoder"], cw["seq_lens_decoder"], cw["seq_lens_this_time"],
                                     cw["cu_seqlens_q"], rotw, num_heads=32, kv_num_heads=8, want_kv_out=True)
        ms = time_events(wr_big, args.steps, args.warmup)
        # per token: qkv read 48*128*2, q/k/v out (32+8+8)*128*2, cache bytes 2*8*128, cos/sin 2*64*4
        line("configs[4] cache write (4096 tokens, RoPE + int8, q/k/v handed on)", ms, "hbm",
             4096 * (48 * 128 * 2 * 2 + 2 * 8 * 128 + 2 * 64 * 4), HBM_PEAK_GBPS, "GB/s")
        del cw
        lens = (c["seq_lens_decoder"] + 1).tolist()

        def dec():
            fd.decode_attention(q, c["key_cache"], c["value_cache"], c["cache_k_scale"], c["cache_v_scale"],
                                c["block_tables"], c["seq_lens_decoder"], c["seq_lens_this_time"], num_heads=32, workspace=ws)
        ms = time_events(dec, args.steps, args.warmup)
        line("configs[2] decode (batch 256, ctx = pos+1, mean 4k)", ms, "hbm", syn.decode_algorithmic_bytes(lens, 256),
             HBM_PEAK_GBPS, "GB/s")
        # the same two pieces as ONE library call (the cache keeps being rewritten at the same positions)
        sws = fd.append_attention_workspace(256, 256, 32, 8, 128, 128, dev)
        sout = torch.empty((256, 32 * 128), dtype=torch.bfloat16, device=dev)

        def fused():
            fd.append_attention(c["qkv"], c["key_cache"], c["value_cache"], c["seq_lens_encoder"], c["seq_lens_decoder"],
                                c["seq_lens_this_time"], c["block_tables"], rot, c["cache_k_scale"], c["cache_v_scale"],
                                num_heads=32, kv_num_heads=8, max_chunk=0, cu_seqlens_q=c["cu_seqlens_q"], workspace=sws,
                                out=sout)
        ms = time_events(fused, args.steps, args.warmup)
        line("configs[2] fused step: cache write + decode in one call", ms, "hbm",
             syn.decode_algorithmic_bytes(lens, 256) + 256 * (48 * 128 * 2 + 2 * 8 * 128 + 32 * 128 * 2), HBM_PEAK_GBPS, "GB/s")

    if args.workload in ("sqattn", "all"):
        # configs[3]: batch 16, ctx 32768, fp8 KV, top-64 of 512 blocks per KV head
        c = syn.decode_case(batch=16, ctx=32768, quant=2, seed=0, device=dev, salient=0.05)   # K ~ N(0,1), 5 % of blocks x4
        sel = lambda: fd.sqattn_select(c["q"], c["key_cache"], c["cache_k_scale"], c["block_tables"], c["seq_lens_decoder"],
                                       num_heads=32, top_k=64, cache_quant_type="cache_fp8")
        kept, cnt = sel()
        ms = time_events(sel, max(args.steps // 10, 5), 2)
        line("configs[3] SQAttn selector (scores + top-64 of 512)", ms, "hbm", 16 * 32768 * 8 * 128, HBM_PEAK_GBPS, "GB/s")
        ws = fd.decode_workspace(16, 32, 8, 128, 512, dev)
        sp = lambda: fd.decode_attention_sparse(c["q"], c["key_cache"], c["value_cache"], c["cache_k_scale"], c["cache_v_scale"],
                                                c["block_tables"], c["seq_lens_decoder"], kept_blocks=kept, kept_counts=cnt,
                                                num_heads=32, cache_quant_type="cache_fp8", workspace=ws)
        ms = time_events(sp, args.steps, args.warmup)
        line("configs[3] sparse decode (64 of 512 blocks)", ms, "hbm", 16 * 8 * 64 * 64 * 128 * 2, HBM_PEAK_GBPS, "GB/s",
             {"us_from_a_hip_graph": round(time_graph(sp, args.steps) * 1e3, 2)})
        de = lambda: fd.decode_attention(c["q"], c["key_cache"], c["value_cache"], c["cache_k_scale"], c["cache_v_scale"],
                                         c["block_tables"], c["seq_lens_decoder"], num_heads=32, cache_quant_type="cache_fp8", workspace=ws)
        ms = time_events(de, max(args.steps // 4, 5), 3)
        line("configs[3] dense fp8 decode, for comparison", ms, "hbm", 16 * 32768 * 8 * 128 * 2, HBM_PEAK_GBPS, "GB/s")
        # the same as ONE library call per step: write the 16 new tokens (the last of each 32768), select, sparse decode
        from fastdeploy_amd.rope import rope_table
        g = torch.Generator(device=dev).manual_seed(5)
        qkv = torch.randn((16, 48 * 128), generator=g, device=dev).to(torch.bfloat16)
        zeros, ones = torch.zeros(16, dtype=torch.int32, device=dev), torch.ones(16, dtype=torch.int32, device=dev)
        cu = torch.arange(17, dtype=torch.int32, device=dev)
        cached = c["seq_lens_decoder"] - 1
        rot = rope_table(32768, 128, 500000.0, dev)
        sws = fd.append_attention_workspace(16, 16, 32, 8, 128, 512, dev)
        sout = torch.empty((16, 32 * 128), dtype=torch.bfloat16, device=dev)

        def sparse_step():
            fd.append_attention(qkv, c["key_cache"], c["value_cache"], zeros, cached, ones, c["block_tables"], rot,
                                c["cache_k_scale"], c["cache_v_scale"], num_heads=32, kv_num_heads=8, max_chunk=0,
                                cache_quant_type="cache_fp8", cu_seqlens_q=cu, workspace=sws, out=sout, sqattn_top_k=64)
        ms = time_events(sparse_step, max(args.steps // 4, 5), 3)
        line("configs[3] as one call per step: cache write + selector + sparse decode", ms, "hbm",
             16 * 32768 * 8 * 128 + 16 * 8 * 64 * 64 * 128 * 2, HBM_PEAK_GBPS, "GB/s",
             {"us_from_a_hip_graph": round(time_graph(sparse_step, args.steps) * 1e3, 2)})

    if args.workload in ("prefill", "prefill_configs4", "all"):
        # configs[4]: batch 2, 2048 new tokens on 8192 cached (int8 paged: N(0,1) activations quantised with
        # max-abs / 127 scales, as the configuration states), causal
        c = syn.decode_case(batch=2, ctx=8192, seed=0, device=dev, extra_blocks=8)
        T = 4096
        q = torch.randn((T, 4096), generator=g, device=dev).to(torch.bfloat16)
        k = torch.randn((T, 1024), generator=g, device=dev).to(torch.bfloat16)
        v = torch.randn((T, 1024), generator=g, device=dev).to(torch.bfloat16)
        cu = torch.tensor([0, 2048, 4096], dtype=torch.int32, device=dev)
        out = torch.empty_like(q)
        pf = lambda: fd.append_attention_prefill(q, k, v, c["key_cache"], c["value_cache"], c["cache_k_scale"], c["cache_v_scale"],
                                                 c["block_tables"], c["seq_lens_decoder"], cu, num_heads=32, max_chunk=2048, out=out)
        # 30 launches of warm-up: the first ~20 ms of an MFMA-bound kernel after idle run slower (clock ramp)
        ms = time_events(pf, max(args.steps // 5, 20), 30)
        # the second yardstick beside the nominal 2.5 PFLOP/s: what a plain bf16 GEMM of the library reaches on this box
        ga = torch.randn((8192, 8192), device=dev, dtype=torch.bfloat16)
        gb = torch.randn((8192, 8192), device=dev, dtype=torch.bfloat16)
        gemm_ms = time_events(lambda: torch.matmul(ga, gb), 20, 10)
        gemm_tflops = 2 * 8192 ** 3 / (gemm_ms * 1e-3) / 1e12
        del ga, gb
        fl = 2 * syn.prefill_flops(8192, 2048)
        line("configs[4] append attention (2 x 2048 new on 8192 cached, int8-quantised N(0,1) prefix)", ms, "mfma", fl,
             2500.0, "TFLOP/s", {"measured_bf16_gemm_8192_tflops": round(gemm_tflops, 1),
                                 "frac_of_measured_gemm": round(fl / (ms * 1e-3) / 1e12 / gemm_tflops, 4)})
        # the same shape where the hand-scheduled kernel does not apply: other head sizes and block sizes (the MFMA
        # kernel for head_dim 64 / 128 / 256 at any block size), and the first chunk of two fresh prompts
        # ("prefill_configs4" stops here: configs[4]'s launches alone, for a profiler run)
        others = args.workload != "prefill_configs4"
        pf0 = lambda: fd.append_attention_prefill(q, k, v, c["key_cache"], c["value_cache"], c["cache_k_scale"], c["cache_v_scale"],
                                                  c["block_tables"], zeros2, cu, num_heads=32, max_chunk=2048, out=out)
        zeros2 = torch.zeros(2, dtype=torch.int32, device=dev)
        if others:
            ms = time_events(pf0, max(args.steps // 5, 20), 30)
            line("2 x 2048 new tokens on an empty cache (the first chunk of two prompts)", ms, "mfma", 2 * syn.prefill_flops(0, 2048),
                 2500.0, "TFLOP/s")
        del c, q, k, v, out
        for hd, bsz in ((64, 64), (128, 16), (256, 64)) if others else ():
            c2 = syn.decode_case(batch=2, ctx=8192, seed=0, device=dev, extra_blocks=8, d=hd, bs=bsz)
            q2 = torch.randn((T, 32 * hd), generator=g, device=dev).to(torch.bfloat16)
            k2 = torch.randn((T, 8 * hd), generator=g, device=dev).to(torch.bfloat16)
            v2 = torch.randn((T, 8 * hd), generator=g, device=dev).to(torch.bfloat16)
            out2 = torch.empty_like(q2)
            pf2 = lambda: fd.append_attention_prefill(q2, k2, v2, c2["key_cache"], c2["value_cache"], c2["cache_k_scale"],
                                                      c2["cache_v_scale"], c2["block_tables"], c2["seq_lens_decoder"], cu,
                                                      num_heads=32, max_chunk=2048, out=out2)
            ms = time_events(pf2, max(args.steps // 5, 20), 30)
            line("configs[4]'s shape at head_dim %d, block_size %d (the MFMA kernel for any block size)" % (hd, bsz), ms, "mfma",
                 2 * syn.prefill_flops(8192, 2048, d=hd), 2500.0, "TFLOP/s")
            del c2, q2, k2, v2, out2
    if args.workload in ("mixed", "all"):
        # a serving step: 63 decode rows (ctx U[3584,4608]) and one prefill row appending 512 tokens to 8192 cached ones,
        # in ONE call (cache write, decode rows, prefill row); without and with the host's hint that one row is a prefill row
        from fastdeploy_amd.rope import rope_table
        gm = torch.Generator().manual_seed(3)
        lens = torch.randint(3584, 4609, (63,), generator=gm).tolist() + [8192]
        c = syn.decode_case(batch=64, ctx=[n + 1 for n in lens[:63]] + [8192 + 512], seed=2, device=dev, direct_bytes=True)
        enc = torch.tensor([0] * 63 + [512], dtype=torch.int32, device=dev)
        dec = torch.tensor(lens, dtype=torch.int32, device=dev)
        this = torch.tensor([1] * 63 + [512], dtype=torch.int32, device=dev)
        cu = torch.tensor([0] + list(range(1, 64)) + [63 + 512], dtype=torch.int32, device=dev)
        T = 63 + 512
        qkv = torch.randn((T, 48 * 128), generator=g, device=dev).to(torch.bfloat16)
        rot = rope_table(16384, 128, 500000.0, dev)
        mb = c["block_tables"].shape[1]
        outm = torch.empty((T, 32 * 128), dtype=torch.bfloat16, device=dev)
        for rows in (None, 1):
            splits = fd.prefill_auto_splits(rows or 1, 32, 512)  # without the hint the kernel counts the prefill rows itself
            wsm = fd.append_attention_workspace(T, 64, 32, 8, 128, mb, dev, prefill_splits=splits)
            stepm = lambda: fd.append_attention(qkv, c["key_cache"], c["value_cache"], enc, dec, this, c["block_tables"], rot,
                                                c["cache_k_scale"], c["cache_v_scale"], num_heads=32, kv_num_heads=8,
                                                max_chunk=512, cu_seqlens_q=cu, workspace=wsm, out=outm, prefill_rows=rows)
            ms = time_events(stepm, max(args.steps // 4, 5), 3)
            kvb = syn.decode_kv_bytes([n + 1 for n in lens[:63]])
            line("mixed step: 63 decode rows + 1 prefill row (512 new on 8192 cached), one call%s" %
                 (", prefill_rows hint -> %d key splits" % splits if rows else ", no hint (the prefill rows counted on the GPU)"), ms, "hbm", kvb, HBM_PEAK_GBPS, "GB/s",
                 {"note": "roofline counts the decode rows' K/V bytes only; the prefill row adds %.1f GFLOP" %
                          (syn.prefill_flops(8192, 512) / 1e9)})
        del c
    if args.workload in ("speculative", "all"):
        # a speculative step: the 64 sequences of configs[1] bring 2 tokens each (the last two of their ctx), one call;
        # as decode rows of two tokens (one pass of the decode kernel) and as prefill rows of two tokens
        from fastdeploy_amd.rope import rope_table
        lens = torch.randint(3584, 4609, (64,), generator=torch.Generator().manual_seed(0)).tolist()
        c = syn.decode_case(batch=64, ctx=lens, pool_blocks=6000, seed=0, device=dev, direct_bytes=True, max_blocks=72)
        g = torch.Generator(device=dev).manual_seed(5)
        qkv = torch.randn((128, 48 * 128), generator=g, device=dev).to(torch.bfloat16)
        zeros = torch.zeros(64, dtype=torch.int32, device=dev)
        twos = torch.full((64,), 2, dtype=torch.int32, device=dev)
        cu = torch.arange(0, 129, 2, dtype=torch.int32, device=dev)
        cached = c["seq_lens_decoder"] - 2
        rot = rope_table(8192, 128, 500000.0, dev)
        sws = fd.append_attention_workspace(128, 64, 32, 8, 128, 72, dev)
        sout = torch.empty((128, 32 * 128), dtype=torch.bfloat16, device=dev)

        def spec(enc, **kw):
            fd.append_attention(qkv, c["key_cache"], c["value_cache"], enc, cached, twos, c["block_tables"], rot,
                                c["cache_k_scale"], c["cache_v_scale"], num_heads=32, kv_num_heads=8,
                                cu_seqlens_q=cu, workspace=sws, out=sout, **kw)
        nbytes = syn.decode_algorithmic_bytes(lens, 64) + 128 * (48 * 128 * 2 + 2 * 8 * 128) + 64 * 32 * 128 * 2 * 2
        ms = time_events(lambda: spec(zeros, max_chunk=0, decode_tokens=2), args.steps, args.warmup)
        line("speculative step, 64 x 2 tokens on ctx ~4k as decode rows of two tokens (write + one decode pass)", ms,
             "hbm", nbytes, HBM_PEAK_GBPS, "GB/s")
        ms = time_events(lambda: spec(twos, max_chunk=2), args.steps, 30)
        line("the same step as prefill rows of two tokens (write + packed append attention)", ms, "hbm", nbytes,
             HBM_PEAK_GBPS, "GB/s")
        # the rows of two tokens block-sparse (16 of their ~64 blocks kept): one list per row, scored by both tokens in
        # one pass over K, then a list per token (selector and sparse decode over tokens as rows: K is streamed per token)
        sparse_bytes = sum(lens) * 8 * 128 + 64 * 8 * 16 * 64 * 128 * 2
        for per_token in (False, True):
            swsx = fd.append_attention_workspace(128, 128 if per_token else 64, 32, 8, 128, 72, dev)
            ms = time_events(lambda: fd.append_attention(qkv, c["key_cache"], c["value_cache"], zeros, cached, twos,
                                                         c["block_tables"], rot, c["cache_k_scale"], c["cache_v_scale"],
                                                         num_heads=32, kv_num_heads=8, cu_seqlens_q=cu, workspace=swsx,
                                                         out=sout, max_chunk=0, decode_tokens=2, sqattn_top_k=16,
                                                         sqattn_per_token=per_token), args.steps, args.warmup)
            line("speculative step, 64 x 2 tokens on ctx ~4k, block-sparse (16 blocks kept per KV head): %s"
                 % ("a list per token" if per_token else "one list per row"), ms, "hbm", sparse_bytes, HBM_PEAK_GBPS, "GB/s")
        # the same sequences with 4 tokens each (16 (token, head) pairs per KV head: the step hands such rows to the
        # fp16-MFMA decode kernel, whose 16 columns they fill)
        qkv4 = torch.randn((256, 48 * 128), generator=g, device=dev).to(torch.bfloat16)
        fours = torch.full((64,), 4, dtype=torch.int32, device=dev)
        cu4 = torch.arange(0, 257, 4, dtype=torch.int32, device=dev)
        cached4 = c["seq_lens_decoder"] - 4
        sws4 = fd.append_attention_workspace(256, 64, 32, 8, 128, 72, dev)
        sout4 = torch.empty((256, 32 * 128), dtype=torch.bfloat16, device=dev)
        spec4 = lambda: fd.append_attention(qkv4, c["key_cache"], c["value_cache"], zeros, cached4, fours, c["block_tables"],
                                            rot, c["cache_k_scale"], c["cache_v_scale"], num_heads=32, kv_num_heads=8,
                                            cu_seqlens_q=cu4, workspace=sws4, out=sout4, max_chunk=0, decode_tokens=4)
        nbytes4 = syn.decode_algorithmic_bytes(lens, 64) + 256 * (48 * 128 * 2 + 2 * 8 * 128) + 4 * 64 * 32 * 128 * 2 * 2
        ms = time_events(spec4, args.steps, args.warmup)
        line("speculative step, 64 x 4 tokens on ctx ~4k as decode rows of four tokens (write + one decode pass)", ms,
             "hbm", nbytes4, HBM_PEAK_GBPS, "GB/s")
        del c
    if args.workload in ("dynamic", "all"):
        # the formats with one scale per stored row: configs[1]'s decode (two pools rotated, as the headline run) and
        # the prefill-sized cache write; the scale caches add 2 x 4 B per token and KV head to the bytes moved
        lens = torch.randint(3584, 4609, (64,), generator=torch.Generator().manual_seed(0)).tolist()
        for name in ("cache_int8_dynamic", "cache_fp8_dynamic", "cache_int8_block", "cache_fp8_block"):
            cs = [syn.decode_case(batch=64, ctx=lens, pool_blocks=6000, seed=sd, device=dev, direct_bytes=True,
                                  max_blocks=72, quant=name) for sd in range(2)]
            ws = fd.decode_workspace(64, 32, 8, 128, 72, dev)
            out = torch.empty((64, 32 * 128), dtype=torch.bfloat16, device=dev)
            n = [0]

            def dec_dyn():
                c = cs[n[0] % 2]
                n[0] += 1
                fd.decode_attention(c["q"], c["key_cache"], c["value_cache"], c["cache_k_scale"], c["cache_v_scale"],
                                    c["block_tables"], c["seq_lens_decoder"], num_heads=32, cache_quant_type=name,
                                    out=out, workspace=ws)
            ms = time_events(dec_dyn, args.steps, args.warmup)
            per_tile = name.endswith("_block")
            scales = sum((n_ + 63) // 64 for n_ in lens) if per_tile else sum(lens)
            work = syn.decode_algorithmic_bytes(lens, 64) - 2 * 8 * 128 * 4 + scales * 8 * 2 * 4
            line("configs[1] decode over the %s cache (one scale per %s)" % (name, "tile" if per_tile else "stored row"),
                 ms, "hbm", work, HBM_PEAK_GBPS, "GB/s")
            del cs
        # configs[3]'s selector over the fp8 dynamic format
        cs = syn.decode_case(batch=16, ctx=32768, quant="cache_fp8_dynamic", seed=0, device=dev, direct_bytes=True)
        sel = lambda: fd.sqattn_select(cs["q"], cs["key_cache"], cs["cache_k_scale"], cs["block_tables"],
                                       cs["seq_lens_decoder"], num_heads=32, top_k=64, cache_quant_type="cache_fp8_dynamic")
        ms = time_events(sel, max(args.steps // 4, 5), 3)
        line("configs[3] SQAttn selector over the cache_fp8_dynamic cache", ms, "hbm",
             16 * 32768 * 8 * (128 + 4) + 16 * 4096 * 2, HBM_PEAK_GBPS, "GB/s")
        del cs
        for wname in ("cache_int8_dynamic", "cache_int8_block"):
            cw = syn.write_case(num_seqs=2, max_pos=8192 + 2048, seed=1, device=dev, chunk=2048, blocks_per_seq=160,
                                quant=wname)
            cw["seq_lens_decoder"].fill_(8192)
            rotw = (cw["rope_cos"], cw["rope_sin"])

            def wr_dyn():
                return fd.write_cache_kv(cw["qkv"], cw["key_cache"], cw["value_cache"], cw["cache_k_scale"], cw["cache_v_scale"],
                                         cw["block_tables"], cw["seq_lens_encoder"], cw["seq_lens_decoder"], cw["seq_lens_this_time"],
                                         cw["cu_seqlens_q"], rotw, num_heads=32, kv_num_heads=8, want_kv_out=True,
                                         cache_quant_type=wname)
            ms = time_events(wr_dyn, args.steps, args.warmup)
            # (the per-block format reads the chunk's K and V rows a second and third time, from the L2)
            line("configs[4] cache write, %s (4096 tokens, q/k/v handed on)" % wname, ms, "hbm",
                 4096 * (48 * 128 * 2 * 2 + 2 * 8 * 128 + 2 * 64 * 4 + (2 * 8 * 4 if wname.endswith("dynamic") else 0)),
                 HBM_PEAK_GBPS, "GB/s")
            del cw
        # a decode step's write (256 sequences, one token each) in the per-block format: one launch (the token kernel keeps
        # the tiles' scales itself when a step brings no more tokens than sequences)
        cw = syn.write_case(num_seqs=256, max_pos=8192, seed=1, device=dev, blocks_per_seq=128, quant="cache_int8_block")
        rotw = (cw["rope_cos"], cw["rope_sin"])
        wr_blk = lambda: fd.write_cache_kv(cw["qkv"], cw["key_cache"], cw["value_cache"], cw["cache_k_scale"], cw["cache_v_scale"],
                                           cw["block_tables"], cw["seq_lens_encoder"], cw["seq_lens_decoder"],
                                           cw["seq_lens_this_time"], cw["cu_seqlens_q"], rotw, num_heads=32, kv_num_heads=8,
                                           cache_quant_type="cache_int8_block")
        ms = time_events(wr_blk, args.steps, args.warmup)
        line("configs[2] cache write, cache_int8_block (256 tokens; prior rows are requantised where a scale grows)", ms,
             "hbm", 256 * (48 * 128 * 2 + 32 * 128 * 2 + 2 * 8 * 128), HBM_PEAK_GBPS, "GB/s",
             {"us_from_a_hip_graph": round(time_graph(wr_blk, args.steps) * 1e3, 2)})
        del cw
        for name in ("cache_int8_dynamic", "cache_fp8_dynamic", "cache_int8_block"):
            c = syn.decode_case(batch=2, ctx=8192, seed=0, device=dev, direct_bytes=True, extra_blocks=8, quant=name)
            q = torch.randn((4096, 4096), generator=g, device=dev).to(torch.bfloat16)
            k = torch.randn((4096, 1024), generator=g, device=dev).to(torch.bfloat16)
            v = torch.randn((4096, 1024), generator=g, device=dev).to(torch.bfloat16)
            cu = torch.tensor([0, 2048, 4096], dtype=torch.int32, device=dev)
            out = torch.empty_like(q)
            pf = lambda: fd.append_attention_prefill(q, k, v, c["key_cache"], c["value_cache"], c["cache_k_scale"],
                                                     c["cache_v_scale"], c["block_tables"], c["seq_lens_decoder"], cu,
                                                     num_heads=32, max_chunk=2048, out=out, cache_quant_type=name)
            ms = time_events(pf, max(args.steps // 5, 20), 30)
            line("configs[4] append attention over the %s cache" % name, ms, "mfma", 2 * syn.prefill_flops(8192, 2048),
                 2500.0, "TFLOP/s")

    if args.workload in ("shapes", "all"):
        # configs[1]'s batch at the shapes the int8-MFMA decode kernel does not take: the fp16-MFMA kernel for head_dim
        # 64 / 128 / 256 at any block size (what the dispatch picks), with the vector-ALU kernel beside it
        lens, _ = pick_context_lengths(64, 3584, 4608, 4096.0)
        for hd, bsz in ((64, 64), (128, 16), (256, 64)):
            mb = (4608 + bsz - 1) // bsz
            c = syn.decode_case(batch=64, ctx=lens, seed=3, device=dev, d=hd, bs=bsz, max_blocks=mb, direct_bytes=True)
            ws = fd.decode_workspace(64, 32, 8, hd, mb, dev)
            out = torch.empty((64, 32 * hd), dtype=torch.bfloat16, device=dev)
            t = {}
            for impl in ("auto", "generic"):
                dec = lambda: fd.decode_attention(c["q"], c["key_cache"], c["value_cache"], c["cache_k_scale"], c["cache_v_scale"],
                                                  c["block_tables"], c["seq_lens_decoder"], num_heads=32, out=out, workspace=ws,
                                                  impl=impl)
                t[impl] = time_events(dec, max(args.steps // 4, 10), 5)
            line("configs[1]'s batch at head_dim %d, block_size %d (the fp16-MFMA decode kernel for any block size)" % (hd, bsz),
                 t["auto"], "hbm", syn.decode_algorithmic_bytes(lens, 64, d=hd, bs=bsz), HBM_PEAK_GBPS, "GB/s",
                 {"us_on_the_vector_alu_kernel": round(t["generic"] * 1e3, 2)})
            del c, ws, out
        # configs[3]'s selector (batch 16, 32k tokens, fp8, top-64) at two of these shapes: scores and bounds from the
        # fp16-MFMA kernel's K half, with the all-fp64 selector beside it
        for hd, bsz in ((128, 16), (64, 64)):
            mb = 32768 // bsz
            c = syn.decode_case(batch=16, ctx=32768, quant=2, seed=0, device=dev, d=hd, bs=bsz, max_blocks=mb, direct_bytes=True)
            t = {}
            for impl in ("auto", "exact"):
                sel = lambda: fd.sqattn_select(c["q"], c["key_cache"], c["cache_k_scale"], c["block_tables"], c["seq_lens_decoder"],
                                               num_heads=32, top_k=64 * 64 // bsz, cache_quant_type=2, impl=impl)
                t[impl] = time_events(sel, max(args.steps // 4, 10), 5)
            line("configs[3]'s selector at head_dim %d, block_size %d, top-%d of %d blocks (scores on the fp16 MFMAs)" % (hd, bsz, 64 * 64 // bsz, mb),
                 t["auto"], "hbm", 16 * 32768 * 8 * hd, HBM_PEAK_GBPS, "GB/s", {"us_all_fp64": round(t["exact"] * 1e3, 2)})
            del c
        # a speculative step at one of these shapes: the 64 sequences with 4 new tokens each as decode rows of four
        # tokens, head_dim 256 (16 (token, head) columns per KV head), one call: cache write + one decode pass
        from fastdeploy_amd.rope import rope_table
        hd = 256
        c = syn.decode_case(batch=64, ctx=lens, seed=4, device=dev, d=hd, bs=64, max_blocks=72, direct_bytes=True)
        qkv4 = torch.randn((256, 48 * hd), generator=g, device=dev).to(torch.bfloat16)
        zeros = torch.zeros(64, dtype=torch.int32, device=dev)
        fours = torch.full((64,), 4, dtype=torch.int32, device=dev)
        cu4 = torch.arange(0, 257, 4, dtype=torch.int32, device=dev)
        cached4 = c["seq_lens_decoder"] - 4
        rot = rope_table(8192, hd, 500000.0, dev)
        sws4 = fd.append_attention_workspace(256, 64, 32, 8, hd, 72, dev)
        sout4 = torch.empty((256, 32 * hd), dtype=torch.bfloat16, device=dev)
        spec4 = lambda: fd.append_attention(qkv4, c["key_cache"], c["value_cache"], zeros, cached4, fours, c["block_tables"],
                                            rot, c["cache_k_scale"], c["cache_v_scale"], num_heads=32, kv_num_heads=8,
                                            cu_seqlens_q=cu4, workspace=sws4, out=sout4, max_chunk=0, decode_tokens=4)
        nbytes4 = (syn.decode_algorithmic_bytes(lens, 64, d=hd) + 256 * (48 * hd * 2 + 2 * 8 * hd) + 4 * 64 * 32 * hd * 2 * 2)
        ms = time_events(spec4, max(args.steps // 4, 10), 5)
        line("speculative step at head_dim 256, 64 x 4 tokens on ctx ~4k as decode rows of four tokens (write + one decode pass)",
             ms, "hbm", nbytes4, HBM_PEAK_GBPS, "GB/s")
        del c
    if args.workload in ("kv_wire", "all"):
        # the sequences of configs[1] leave the cache in wire form and enter another one: HBM copies (read + write)
        from fastdeploy_amd import kv_wire
        c = syn.decode_case(batch=64, ctx=(3584, 4608), pool_blocks=6000, seed=0, device=dev, direct_bytes=True)
        plan = kv_wire.WirePlan(c["seq_lens_decoder"].tolist(), 8, 128, 64, dev)
        wire = torch.empty(plan.total, dtype=torch.uint8, device=dev)
        kc2, vc2 = torch.empty_like(c["key_cache"]), torch.empty_like(c["value_cache"])
        status = torch.zeros(2, dtype=torch.int32, device=dev)
        ex = lambda: kv_wire.kv_export(c["key_cache"], c["value_cache"], c["cache_k_scale"], c["cache_v_scale"],
                                       c["block_tables"], plan, wire=wire)
        im = lambda: kv_wire.kv_import(wire, kc2, vc2, c["block_tables"], plan, cache_k_scale=c["cache_k_scale"],
                                       cache_v_scale=c["cache_v_scale"], status=status)
        ms = time_events(ex, max(args.steps // 4, 5), 3)
        line("KV export to wire form (64 sequences of configs[1])", ms, "hbm", 2 * plan.total, HBM_PEAK_GBPS, "GB/s")
        ms = time_events(im, max(args.steps // 4, 5), 3)
        line("KV import from wire form (64 sequences of configs[1])", ms, "hbm", 2 * plan.total, HBM_PEAK_GBPS, "GB/s",
             {"status": status.tolist()})
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-baseline leg")
    ap.add_argument("--pools", type=int, default=2, help="distinct cache pools rotated between steps")
    ap.add_argument("--workload", default="decode", choices=["decode", "write_decode", "sqattn", "prefill", "prefill_configs4", "mixed", "speculative", "dynamic", "shapes", "kv_wire", "all"],
                    help="decode = the headline metric (default); the others print one line per kernel of that row")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (the path shards by KV head or by sequence with no "
                 "exchange; nothing here uses a second device). Run with --gpus 1.")

    import fastdeploy_amd as fd
    from fastdeploy_amd import synthetic as syn

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = "cuda:0"
    torch.cuda.set_device(0)
    if args.workload != "decode":
        other_workloads(args)
        return
    B = 64
    # distinct pools so that consecutive steps do not re-read the same bytes out of the
    # last-level cache; every pool has its own block table permutation and contents
    lens, ctx_seed = pick_context_lengths(B, 3584, 4608, 4096.0)
    cases = [syn.decode_case(batch=B, ctx=lens, pool_blocks=6000, seed=s, device=dev, direct_bytes=True,
                             max_blocks=72) for s in range(args.pools)]
    from fastdeploy_amd import _lib
    assert fd.decode_uses_mfma(32, 8, 128, 64, "cache_int8")
    ws = fd.decode_workspace(B, 32, 8, 128, 72, dev)
    outs = [torch.empty((B, 32 * 128), dtype=torch.bfloat16, device=dev) for _ in cases]

    def run(i, impl):
        c = cases[i % len(cases)]
        fd.decode_attention(c["q"], c["key_cache"], c["value_cache"], c["cache_k_scale"], c["cache_v_scale"],
                            c["block_tables"], c["seq_lens_decoder"], num_heads=32, cache_quant_type="cache_int8",
                            out=outs[i % len(cases)], workspace=ws, impl=impl)

    counter = [0]

    def step(impl="auto"):
        run(counter[0], impl)
        counter[0] += 1

    chunks_per_pair = _lib.lib().fdattn_decode_chunks_per_sequence(B, 8, 72)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ms_op = time_events(lambda: step("auto"), args.steps, args.warmup)
    wall = time.perf_counter() - t0
    each = time_each(lambda: step("auto"), args.steps)
    if chunks_per_pair == 1:
        # every (sequence, KV head) list is one chunk: the op IS one launch of decode_c8_kernel (no merge kernel), so
        # the roofline prices the kernel with the very loop `value` comes from - the events bracket the launches and
        # the gaps between them, i.e. an upper bound of the kernel's own duration
        ms_main, ms_merge, kernel_timing = ms_op, 0.0, "the timed region of `value` (one kernel per step)"
    else:
        # the dominant kernel alone (the same launches without the merge), timed in one loop with the whole op so that
        # both see the same clocks and cache state: step 2 i is the whole op, step 2 i + 1 the main kernel only
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2 * args.steps + 1)]
        torch.cuda.synchronize()
        ev[0].record()
        for i in range(args.steps):
            step("auto")
            ev[2 * i + 1].record()
            step("partials")
            ev[2 * i + 2].record()
        torch.cuda.synchronize()
        ms_op2 = sum(ev[2 * i].elapsed_time(ev[2 * i + 1]) for i in range(args.steps)) / args.steps
        ms_main = sum(ev[2 * i + 1].elapsed_time(ev[2 * i + 2]) for i in range(args.steps)) / args.steps
        ms_main = min(ms_main, ms_op)
        ms_merge, kernel_timing = max(ms_op2 - ms_main, 0.0), "events around alternating whole-op and main-kernel-only launches"

    # single launches timed one by one (event pair each): the spread behind the average
    singles = []
    for _ in range(min(args.steps, 100)):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        step("partials")
        e1.record()
        e1.synchronize()
        singles.append(e0.elapsed_time(e1) * 1e3)
    singles.sort()
    # what the same event pair reads around a one-workgroup fill kernel: the part of a single launch's reading that
    # is the two event packets and the dispatch between them, not the kernel (a profiler's begin/end stamps of a
    # launch that follows an idle queue are the kernel's own duration in isolation)
    tiny, floor = torch.zeros(64, dtype=torch.float32, device=dev), []
    for _ in range(min(args.steps, 100)):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        tiny.zero_()
        e1.record()
        e1.synchronize()
        floor.append(e0.elapsed_time(e1) * 1e3)
    floor.sort()

    # yardstick of the same run: a plain 1 GiB device copy (reads 1 GiB, writes 1 GiB) - what the
    # memory system of this box gives a trivial kernel, beside the nominal 8 TB/s
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    ms_copy = time_events(lambda: dst.copy_(src), 10, 3)
    copy_gbps = 2.0 * (1 << 30) / (ms_copy * 1e-3) / 1e9
    del src, dst

    alg_bytes = syn.decode_algorithmic_bytes(lens, B)
    kv_bytes = syn.decode_kv_bytes(lens)
    achieved = alg_bytes / (ms_main * 1e-3) / 1e9
    us_layer = ms_op * 1e3
    result = {
        "metric": "decode_attn_us_per_layer", "value": round(us_layer, 3), "unit": "us/layer",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_op, 6),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "int8", "data": "synthetic",
        "config": {"workload": "configs[1]: Llama-3-8B decode attention, 1 layer, batch 64, 32q/8kv heads, "
                               "head_dim 128, block_size 64, ctx U[3584,4608], int8 paged KV, 6000-block pool",
                   "batch": B, "mean_ctx": sum(lens) / B, "ctx_seed": ctx_seed, "kv_bytes": kv_bytes,
                   "pools_rotated": len(cases)},
        "us_per_layer_median": round(each[len(each) // 2] * 1e3, 3), "us_per_layer_min": round(each[0] * 1e3, 3),
        "achieved_hbm_gbps_whole_op": round(alg_bytes / (ms_op * 1e-3) / 1e9, 1),
        "pct_hbm_peak_whole_op": round(100 * alg_bytes / (ms_op * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2),
        "tokens_per_s_1_layer": round(B / (ms_op * 1e-3), 1),
        "tokens_per_s_32_layers_attention_only": round(B / (32 * ms_op * 1e-3), 1),
        # chunks per (sequence, KV head): 1 = every pair is finished by the main kernel, no merge kernel is launched
        # (the merge-only call then measures an empty call: host overhead of the timing loop)
        "chunks_per_pair": chunks_per_pair,
        "kernel_us": {"decode_c8_kernel": round(ms_main * 1e3, 3), "merge_kernel": round(ms_merge * 1e3, 3),
                      "timed_by": kernel_timing},
        "roofline": {"bound": "hbm", "kernel": "decode_c8_kernel<int8,dense>", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "algorithmic_bytes": alg_bytes, "traffic": int(alg_bytes * TRAFFIC_PER_ALGORITHMIC_BYTE),
                     "traffic_source": "%s: FETCH_SIZE + WRITE_SIZE per dispatch / algorithmic bytes = %.4f, applied "
                                       "to this run's algorithmic bytes" % (TRAFFIC_PROFILE, TRAFFIC_PER_ALGORITHMIC_BYTE),
                     "device_copy_gbps_same_run": round(copy_gbps, 1),
                     "frac_of_device_copy": round(achieved / copy_gbps, 4),
                     # the same bytes over the median of launches timed ONE BY ONE (an event pair and a device sync
                     # each): no next launch fills the tail of this one.  The reading holds the event pair's own cost
                     # (event_pair_around_a_fill_kernel below); ISOLATED_PROFILE has the kernel's own duration in
                     # such launches from the profiler's stamps.
                     "frac_isolated": round(alg_bytes / (singles[len(singles) // 2] * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                     "frac_isolated_kernel_only": ISOLATED_FRAC_PROFILED,
                     "frac_isolated_kernel_only_source": ISOLATED_PROFILE},
        "kernel_us_single_launches": {"min": round(singles[0], 2), "median": round(singles[len(singles) // 2], 2),
                                      "max": round(singles[-1], 2), "n": len(singles),
                                      "event_pair_around_a_fill_kernel": {"min": round(floor[0], 2),
                                                                          "median": round(floor[len(floor) // 2], 2)}},
    }

    if not args.no_cpu:
        from oracle import oracle
        import numpy as np
        c = {k: (v.cpu() if isinstance(v, torch.Tensor) else v) for k, v in cases[0].items()}
        qb = c["q"].view(torch.int16).numpy().view(np.uint16)
        a = [qb, c["key_cache"].numpy(), c["value_cache"].numpy(), c["cache_k_scale"].numpy(),
             c["cache_v_scale"].numpy(), c["block_tables"].numpy(), c["seq_lens_decoder"].numpy(), 32, 8, 128, 1]
        cores = len(os.sched_getaffinity(0))
        cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
        oracle.decode_attention(*a)                      # warm-up pass (page-in, thread start)
        reps, t = 0, time.perf_counter()
        while True:
            ref = oracle.decode_attention(*a)
            reps += 1
            if time.perf_counter() - t > 10.0 or reps >= 5:
                break
        cpu_s = (time.perf_counter() - t) / reps
        result["cpu_baseline"] = {
            "value": round(cpu_s * 1e6, 1), "unit": "us/layer", "cores": cores, "kind": "port",
            "sample": "the whole configs[1] workload (pool 0), %d timed passes of the C oracle "
                      "(fp32, OpenMP over sequence x head); the reference has no CPU attention path" % reps,
            "gpu_speedup": round(cpu_s * 1e6 / us_layer, 1)}
        # cross-check of the CPU figure: PyTorch's own CPU SDPA on the dequantised, gathered K / V of a bounded sample
        # (the first 8 sequences; dequantising and gathering are outside the timed region), scaled to the batch
        nseq = 8
        kc, vc = c["key_cache"].view(torch.int8), c["value_cache"].view(torch.int8)
        t_sdpa = 0.0
        for b in range(nseq):
            n = int(c["seq_lens_decoder"][b])
            blk = c["block_tables"][b, :(n + 63) // 64].long()
            kd = (kc[blk].float() * c["cache_k_scale"][None, :, None, :]).permute(1, 0, 2, 3).reshape(8, -1, 128)[:, :n]
            vd = (vc[blk].float() * c["cache_v_scale"][None, :, None, :]).permute(1, 0, 2, 3).reshape(8, -1, 128)[:, :n]
            qf = c["q"][b].float().view(8, 4, 128)
            torch.nn.functional.scaled_dot_product_attention(qf, kd, vd)      # warm-up
            t1 = time.perf_counter()
            torch.nn.functional.scaled_dot_product_attention(qf, kd, vd)
            t_sdpa += time.perf_counter() - t1
        result["cpu_baseline"]["torch_cpu_sdpa_us_per_layer"] = round(t_sdpa / nseq * B * 1e6, 1)
        result["cpu_baseline"]["torch_cpu_sdpa_sample"] = ("torch.nn.functional.scaled_dot_product_attention, fp32, on the "
                                                           "dequantised gathered K/V of the first %d of %d sequences, "
                                                           "scaled to the batch; %d torch threads" % (nseq, B, torch.get_num_threads()))
        # and the run doubles as a full-size parity check of pool 0
        got = outs[0].cpu().view(torch.int16).numpy().view(np.uint16)
        run(0, "auto")
        torch.cuda.synchronize()
        got = outs[0].cpu().view(torch.int16).numpy().view(np.uint16)
        gf = (got.astype(np.uint32) << 16).view(np.float32)
        rf = (ref.astype(np.uint32) << 16).view(np.float32)
        d = np.abs(gf - rf)
        bad = (d > 2e-3) & (d / np.maximum(np.maximum(np.abs(gf), np.abs(rf)), 1e-30) > 1e-2)
        result["parity_full_size"] = {"max_abs_diff": float(d.max()), "out_of_tolerance": int(bad.sum()),
                                      "tolerance": "abs 2e-3 OR rel 1e-2"}
    result["wall_s_timed_region"] = round(wall, 3)
    print(json.dumps(result))


if __name__ == "__main__":
    main()

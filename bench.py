#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

A "step" is one pass of paged-KV decode attention (split-K pass + combine) over the
whole batch of configs[3]: bf16 KV cache, batch 128, 32 query / 8 kv heads, head_dim
128, block 16, ragged context lengths ~ U[512, 16384] (seeded), physical blocks a
random permutation of a pool sized 1.1x.  Inputs are resident in HBM before timing.
`value` is algorithmic bytes / wall time per step.  The same JSON line also carries
the prefill measurement at configs[2] (bf16, packed varlen, B8, 32/8 heads, D128,
S4096, causal) and the fp8-KV decode at configs[4], each with its own roofline.

The CPU baseline is the oracle (a restatement of the reference's PyTorch attention)
timed on the host cores over a bounded sample of the same inputs; its outputs also
check the GPU results of that sample.

The line is kept short (the driver keeps only the end of stdout): the contract's fields for configs[3], then the
fp8 decode, then one {ms, frac} pair per auxiliary leg under "legs", and the configs[2] `prefill` object LAST.
`--full` prints every leg's whole object instead; `--detail PATH` writes that verbose form to a file.

usage: python bench.py [--gpus 1] [--steps K=200] [--warmup W=50] [--seed S]
                       [--only decode|prefill|small|few|fp8|backward|producers|layer|loop] [--no-cpu] [--full] [--detail PATH]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "llm-systems-from-scratch_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
METRIC = "paged-decode attn HBM GB/s (% of 8 TB/s) + prefill attn TFLOP/s (% MFMA peak)"


def _traffic(key):
    """HBM bytes per launch measured with rocprofv3 --pmc (kept as data under profiles/)."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get(key)
    except (OSError, ValueError):
        return None


def _prefill_kernel(head_dim):
    """Name of the kernel a causal, unsplit prefill of this head_dim runs on."""
    return "prefill_fwd_w64_kernel<causal>" if head_dim == 128 else "prefill_fwd_kernel<%d, causal>" % head_dim


BURN_MS = 40.0      # untimed launches for about this long in front of the warm-up of every leg but the two decode legs
                    # (disclosed in the JSON line)


def timed(fn, steps, warmup, burn_ms=0.0):
    """Returns (wall ms/step, device ms/step): K launches between two syncs, HIP events on the launch stream.
    `burn_ms`: untimed launches for about that long come first.  A short warm-up leaves a short kernel inside the
    clocks' transient: the shader clock needs some tens of milliseconds of MFMA load to leave its idle state, and a
    0.15 ms streaming kernel runs its launches 10 to 50 about 10 % slower than the ones before and after."""
    import torch
    if burn_ms > 0:
        fn()
        torch.cuda.synchronize()
        t = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        one_ms = max((time.perf_counter() - t) * 1e3, 0.01)
        for _ in range(min(int(burn_ms / one_ms) + 1, 1000)):
            fn()
    for _ in range(warmup):
        fn()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps, e0.elapsed_time(e1) / steps


CPU_SAMPLE_SEQS = 128      # sequences of a decode configuration that the CPU oracle is run (and timed) on


def bench_decode(cfg, args, with_cpu=False):
    import torch
    import mi355_attn
    from mi355_attn import workloads

    case = workloads.decode_config(cfg, seed=args.seed, keep_bf16_seqs=CPU_SAMPLE_SEQS if with_cpu else 0)
    B, Hq, D = case.q.shape
    ws = mi355_attn.paged_decode_workspace(B, Hq, D, case.max_context, case.q.device)
    out = torch.empty_like(case.q)

    def step():
        mi355_attn.paged_attention_decode(case.q, case.k_cache, case.v_cache, case.block_tables, case.context_lens,
                                          k_scale=case.k_scale, v_scale=case.v_scale, max_context=case.max_context,
                                          workspace=ws, out=out)

    wall_ms, dev_ms = timed(step, args.steps, args.warmup)
    nbytes = case.algorithmic_bytes()
    res = {
        "value": nbytes / wall_ms / 1e6,
        "unit": "GB/s",
        "ms_per_step": wall_ms,
        "tokens": case.tokens,
        "algorithmic_bytes": nbytes,
        "roofline": {
            "bound": "hbm", "kernel": "paged_decode_split_kernel (+ combine, same launch sequence)",
            "achieved": nbytes / dev_ms / 1e6, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": nbytes / dev_ms / 1e6 / HBM_PEAK_GBPS, "device_ms": dev_ms,
            "traffic": _traffic(f"decode_cfg{cfg}"),
        },
    }
    return res, (case, out)


def bench_prefill_backward(cfg, args):
    """dq, dk, dv at configs[cfg] (the two backward launches: dq with delta, then dk and dv).  FLOPs by the usual
    convention: 2.5 x the forward's (five GEMMs against two), causal = half."""
    import torch
    from mi355_attn import ops, workloads

    case = workloads.prefill_config(cfg, seed=args.seed)
    S = case.seqlen
    if case.cu_seqlens is not None:
        out, lse = ops._varlen(case.q, case.k, case.v, case.cu_seqlens, case.cu_seqlens, S, S, True, None, want_lse=True)
        cu = case.cu_seqlens
    else:
        out, lse = ops._dense(case.q, case.k, case.v, None, 1, None, want_lse=True)
        cu = None
    g = torch.Generator(device=case.q.device).manual_seed(args.seed + 1)
    dout = torch.randn(out.shape, device=out.device, generator=g).to(torch.bfloat16)
    scale = 1.0 / (case.q.shape[-1] ** 0.5)
    wall_ms, dev_ms = timed(lambda: ops._prefill_backward(case.q, case.k, case.v, out, dout, lse, cu, cu, S, S, scale, 1),
                            args.steps, args.warmup, BURN_MS)
    flops = case.flops() * 5 // 2
    return {
        "value": flops / wall_ms / 1e9, "unit": "TFLOP/s", "ms_per_step": wall_ms, "dtype": "bf16",
        "algorithmic_flops": flops,
        "config": {"workload": f"configs[{cfg}] backward: dq, dk, dv of the causal prefill (seed {args.seed})"},
        "roofline": {"bound": "mfma", "kernel": "bwd_dq_kernel + bwd_dkv_kernel",
                     "achieved": flops / dev_ms / 1e9, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": flops / dev_ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, "device_ms": dev_ms,
                     "traffic": _traffic(f"prefill_bwd_cfg{cfg}")},
    }


def bench_producers(args):
    """The two cache producers at the shapes the attention configs imply: RoPE + cache write for the
    32768 packed tokens of configs[2], and fp8 quantisation of a K pool of configs[4]'s size."""
    import torch
    import mi355_attn

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(args.seed)
    res = {}
    # --- rope_and_cache: T = 8 x 4096 tokens, 32 q / 8 kv heads, head_dim 128, blocks dealt as a random permutation
    B, S, Hq, Hkv, D = 8, 4096, 32, 8, 128
    T = B * S
    q = torch.randn(T, Hq, D, device=dev, generator=g).mul_(0.5).to(torch.bfloat16)
    k = torch.randn(T, Hkv, D, device=dev, generator=g).mul_(0.5).to(torch.bfloat16)
    v = torch.randn(T, Hkv, D, device=dev, generator=g).mul_(0.5).to(torch.bfloat16)
    n_blocks = T // 16
    perm = torch.randperm(n_blocks, device=dev, generator=g)
    slots = (perm.repeat_interleave(16) * 16 + torch.arange(16, device=dev).repeat(n_blocks)).to(torch.int64)
    pos = torch.arange(S, device=dev, dtype=torch.int32).repeat(B)
    freq = mi355_attn.build_rope_cache(S, D, 10000.0, dev)
    k_cache = torch.zeros(n_blocks, Hkv, 16, D, dtype=torch.bfloat16, device=dev)
    v_cache = torch.zeros_like(k_cache)
    q_out = torch.empty_like(q)
    wall_ms, dev_ms = timed(lambda: mi355_attn.rope_and_cache(q, k, v, pos, freq, k_cache, v_cache, slots, out=q_out),
                            args.steps, args.warmup, BURN_MS)
    nbytes = 2 * (q.numel() + k.numel() + v.numel()) * 2 + T * 12 + freq.numel() * 4
    res["rope_and_cache"] = {
        "value": nbytes / wall_ms / 1e6, "unit": "GB/s", "ms_per_step": wall_ms, "dtype": "bf16 (fp32 rotation)",
        "config": {"workload": "RoPE + paged cache write of configs[2]'s 32768 packed tokens (32 q / 8 kv heads, "
                               "head_dim 128), blocks a random permutation", "algorithmic_bytes": nbytes},
        "roofline": {"bound": "hbm", "kernel": "rope_and_cache_kernel", "achieved": nbytes / dev_ms / 1e6,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": nbytes / dev_ms / 1e6 / HBM_PEAK_GBPS,
                     "device_ms": dev_ms, "traffic": _traffic("rope_and_cache")},
    }
    del k_cache, v_cache
    # --- rope_and_cache_fp8: the same tokens into an fp8 pool with per-(block, kv head) scales (two launches:
    # queries, then keys/values; 16 tokens per block arrive together, so no row is re-expressed)
    k8 = torch.zeros(n_blocks, Hkv, 16, D, dtype=torch.uint8, device=dev)
    v8 = torch.zeros_like(k8)
    ks = torch.ones(n_blocks, Hkv, dtype=torch.float32, device=dev)
    vs = torch.ones_like(ks)
    wall_ms, dev_ms = timed(lambda: mi355_attn.rope_and_cache_fp8(q, k, v, pos, freq, k8, v8, ks, vs, slots, out=q_out),
                            args.steps, args.warmup, BURN_MS)
    nbytes = 2 * q.numel() * 2 + (k.numel() + v.numel()) * 3 + 2 * ks.numel() * 4 + T * 12 + freq.numel() * 4
    res["rope_and_cache_fp8"] = {
        "value": nbytes / wall_ms / 1e6, "unit": "GB/s", "ms_per_step": wall_ms, "dtype": "bf16 -> fp8-e4m3 (fp32 rotation)",
        "config": {"workload": "RoPE + quantising write into an fp8 paged cache of configs[2]'s 32768 packed tokens "
                               "(32 q / 8 kv heads, head_dim 128), blocks a random permutation", "algorithmic_bytes": nbytes},
        "roofline": {"bound": "hbm", "kernel": "rope_and_cache_fp8_fused_kernel",
                     "achieved": nbytes / dev_ms / 1e6, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": nbytes / dev_ms / 1e6 / HBM_PEAK_GBPS, "device_ms": dev_ms,
                     "traffic": _traffic("rope_and_cache_fp8")},
    }
    # --- gather_kv_fp8: the way back for a prompt chunk over an fp8 cache: the 8 sequences' 4096 tokens each out of that
    # pool, dequantised, as packed bf16 rows
    tables = perm.view(B, S // 16).to(torch.int32)
    lens = torch.full((B,), S, dtype=torch.int32, device=dev)
    cu_k = (torch.arange(B + 1, device=dev) * S).to(torch.int32)
    k_lin = torch.empty(T, Hkv, D, dtype=torch.bfloat16, device=dev)
    v_lin = torch.empty_like(k_lin)
    wall_ms, dev_ms = timed(lambda: mi355_attn.gather_kv_fp8(k8, v8, ks, vs, tables, lens, total_context=T, cu_seqlens_k=cu_k,
                                                             out=(k_lin, v_lin)), args.steps, args.warmup, BURN_MS)
    nbytes = (k.numel() + v.numel()) * 3 + 2 * ks.numel() * 4 + tables.numel() * 4
    res["gather_kv_fp8"] = {
        "value": nbytes / wall_ms / 1e6, "unit": "GB/s", "ms_per_step": wall_ms, "dtype": "fp8-e4m3 -> bf16",
        "config": {"workload": "gather + dequantise 8 sequences of 4096 tokens out of an fp8 paged cache into packed bf16 "
                               "rows (8 kv heads, head_dim 128), blocks a random permutation", "algorithmic_bytes": nbytes},
        "roofline": {"bound": "hbm", "kernel": "gather_kv_fp8_kernel", "achieved": nbytes / dev_ms / 1e6,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": nbytes / dev_ms / 1e6 / HBM_PEAK_GBPS,
                     "device_ms": dev_ms, "traffic": None},
    }
    del q, k, v, q_out, k8, v8, k_lin, v_lin
    # --- quantize_kv_fp8: a pool of configs[4]'s size (about 103k blocks x 8 kv heads x 16 x 128)
    nb = 103_000
    pool = torch.randn(nb, Hkv, 16, D, device=dev, generator=g).to(torch.bfloat16)
    out8 = torch.empty(nb, Hkv, 16, D, dtype=torch.uint8, device=dev)
    scale = torch.empty(nb, Hkv, dtype=torch.float32, device=dev)
    wall_ms, dev_ms = timed(lambda: mi355_attn.quantize_kv_cache_fp8(pool, out=(out8, scale)), args.steps, args.warmup, BURN_MS)
    nbytes = pool.numel() * 3 + scale.numel() * 4
    res["quantize_kv_fp8"] = {
        "value": nbytes / wall_ms / 1e6, "unit": "GB/s", "ms_per_step": wall_ms, "dtype": "bf16 -> fp8-e4m3",
        "config": {"workload": f"per-(block, kv head) fp8 quantisation of a {nb}-block bf16 pool (8 kv heads, block 16, "
                               "head_dim 128)", "algorithmic_bytes": nbytes},
        "roofline": {"bound": "hbm", "kernel": "quantize_kv_fp8_kernel", "achieved": nbytes / dev_ms / 1e6,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": nbytes / dev_ms / 1e6 / HBM_PEAK_GBPS,
                     "device_ms": dev_ms, "traffic": _traffic("quantize_kv_fp8")},
    }
    return res


def bench_layer_ops(args):
    """RMSNorm (with the fused residual add) and silu(gate)*up on the activations of configs[2]'s
    32768 tokens at d_model 4096 (32 heads x 128) and d_ff 11008."""
    import torch
    import mi355_attn

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(args.seed)
    T, d, ff = 32768, 4096, 11008
    res = {}
    x = torch.randn(T, d, device=dev, generator=g).to(torch.bfloat16)
    r = torch.randn(T, d, device=dev, generator=g).to(torch.bfloat16)
    w = torch.ones(d, device=dev)
    wall_ms, dev_ms = timed(lambda: mi355_attn.rms_norm(x, w, 1e-5, residual=r, return_sum=True), args.steps, args.warmup, BURN_MS)
    nbytes = 4 * T * d * 2 + d * 4                   # read x, residual; write y, sum
    res["rms_norm_residual"] = {
        "value": nbytes / wall_ms / 1e6, "unit": "GB/s", "ms_per_step": wall_ms, "dtype": "bf16 (fp32 math)",
        "config": {"workload": f"y, h = rms_norm(x + residual): {T} rows x {d} bf16, fp32 weight", "algorithmic_bytes": nbytes},
        "roofline": {"bound": "hbm", "kernel": "rms_norm_rows_kernel<8>", "achieved": nbytes / dev_ms / 1e6,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": nbytes / dev_ms / 1e6 / HBM_PEAK_GBPS,
                     "device_ms": dev_ms, "traffic": _traffic("rms_norm_residual")},
    }
    del x, r
    gu = torch.randn(T, 2 * ff, device=dev, generator=g).to(torch.bfloat16)
    wall_ms, dev_ms = timed(lambda: mi355_attn.silu_mul(gu[:, :ff], gu[:, ff:]), args.steps, args.warmup, BURN_MS)
    nbytes = 3 * T * ff * 2
    res["silu_mul"] = {
        "value": nbytes / wall_ms / 1e6, "unit": "GB/s", "ms_per_step": wall_ms, "dtype": "bf16 (fp32 silu)",
        "config": {"workload": f"silu(gate) * up on the two halves of a ({T}, {2 * ff}) bf16 projection output",
                   "algorithmic_bytes": nbytes},
        "roofline": {"bound": "hbm", "kernel": "silu_mul_vec8_kernel", "achieved": nbytes / dev_ms / 1e6,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": nbytes / dev_ms / 1e6 / HBM_PEAK_GBPS,
                     "device_ms": dev_ms, "traffic": _traffic("silu_mul")},
    }
    return res


def bench_decode_few_sequences(args):
    """Decode attention of a few long sequences (the reference's `generate` is batch 1): too few (sequence, kv head)
    pairs for the compute units at the chunk size of a large batch, so the split-K pass runs with shorter chunks.
    Timed in a HIP graph of ten steps (the host takes longer to issue one eager step than the GPU to run it)."""
    import torch
    import mi355_attn
    from mi355_attn import workloads

    out = {}
    for name, batch, ctx in (("one_sequence_8192", 1, 8192), ("one_sequence_32768", 1, 32768), ("four_sequences_8192", 4, 8192)):
        case = workloads.make_decode_case(batch=batch, n_q_heads=32, n_kv_heads=8, head_dim=128, ctx_kind="fixed", ctx_lo=ctx,
                                          ctx_hi=ctx, pool_factor=1.1, seed=args.seed)
        B, Hq, D = case.q.shape
        ws = mi355_attn.paged_decode_workspace(B, Hq, D, case.max_context, case.q.device)
        res = torch.empty_like(case.q)

        def step():
            mi355_attn.paged_attention_decode(case.q, case.k_cache, case.v_cache, case.block_tables, case.context_lens,
                                              max_context=case.max_context, workspace=ws, out=res)

        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            step()
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=side):
                for _ in range(10):
                    step()
        wall_ms, dev_ms = timed(graph.replay, max(1, args.steps // 2), args.warmup, BURN_MS)
        nbytes = case.algorithmic_bytes()
        out[name] = {
            "us_per_step": dev_ms * 100.0, "algorithmic_bytes": nbytes,
            "chunk_tokens": mi355_attn.decode_chunk_tokens(B, Hq, 8, case.max_context),
            "config": {"workload": "paged decode attention, bf16 KV, %d sequence(s) of %d tokens, 32 q / 8 kv heads, "
                                   "head_dim 128, ten steps per graph launch" % (batch, ctx)},
            "roofline": {"bound": "hbm", "kernel": "paged_decode_split_kernel + paged_decode_combine_kernel",
                         "achieved": nbytes / (dev_ms / 10.0) / 1e6, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": nbytes / (dev_ms / 10.0) / 1e6 / HBM_PEAK_GBPS, "device_ms": dev_ms / 10.0, "traffic": None},
        }
    return out


def bench_decode_loop(args):
    """Decode steps of the KV-cached decoder at the reference's sample model (configures/sample.yaml:
    vocab 10000, context 256, d_model 512, 4 layers, 16 heads, d_ff 1344; random weights), batch 8:
    launched eagerly (about ten launches per layer from Python) and replayed from a captured HIP graph."""
    import torch
    import mi355_attn

    cfg = dict(vocab_size=10000, context_length=256, d_model=512, num_layers=4, num_heads=16, d_ff=1344,
               rope_theta=10000.0)
    g = torch.Generator().manual_seed(args.seed)
    d, ff, V = cfg["d_model"], cfg["d_ff"], cfg["vocab_size"]

    def w(*shape, std):
        return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16)

    sd = {"token_embeddings.weight": w(V, d, std=1.0), "lm_head.weight": w(V, d, std=d ** -0.5),
          "final_norm.weight": torch.ones(d)}
    for i in range(cfg["num_layers"]):
        pre = f"layers.{i}."
        for n in ("q_proj", "k_proj", "v_proj", "output_proj"):
            sd[pre + f"attn.{n}.weight"] = w(d, d, std=d ** -0.5)
        sd[pre + "ffn.gate_proj.weight"] = w(ff, d, std=d ** -0.5)
        sd[pre + "ffn.up_proj.weight"] = w(ff, d, std=d ** -0.5)
        sd[pre + "ffn.down_proj.weight"] = w(d, ff, std=ff ** -0.5)
        sd[pre + "attn_norm.weight"] = torch.ones(d)
        sd[pre + "ffn_norm.weight"] = torch.ones(d)
    B, prompt_len, n_steps = 8, 32, min(200, cfg["context_length"] - 33)
    res = {"config": {"workload": f"decode steps of the KV-cached decoder, reference sample model {cfg}, batch {B}, "
                                  f"prompt {prompt_len}, {n_steps} timed steps, greedy tokens fed back through the host",
                       "weights": "random"}}
    for name, graphs in (("eager", False), ("hip_graph", True)):
        model = mi355_attn.CachedTransformerLM(cfg, sd, max_batch=B, decode_graphs=graphs)
        sids = [model.new_sequence() for _ in range(B)]
        prompts = [torch.randint(0, V, (prompt_len,), generator=g) for _ in range(B)]
        logits = model.prefill(sids, prompts)
        toks = logits.argmax(-1).tolist()
        for _ in range(5):                                   # warm-up steps (the first graphed one captures)
            toks = model.decode(sids, toks).argmax(-1).tolist()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n_steps):
            toks = model.decode(sids, toks).argmax(-1).tolist()     # .tolist() synchronises: a real sampling loop
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / n_steps
        res[name] = {"ms_per_step": dt * 1e3, "tokens_per_s": B / dt}
        del model
    res["speedup"] = res["eager"]["ms_per_step"] / res["hip_graph"]["ms_per_step"]
    return res


def _timed_repeats(fn, min_seconds=10.0, max_reps=20):
    """Run fn until min_seconds of wall time have been spent; returns (last result, seconds per call, calls)."""
    total, reps, out = 0.0, 0, None
    while total < min_seconds and reps < max_reps:
        t0 = time.perf_counter()
        out = fn()
        total += time.perf_counter() - t0
        reps += 1
    return out, total / reps, reps


# Quantisation-error bound of the fp8-KV decode against a bf16-KV fp32-math reference (e4m3 rounds with relative
# error <= 2^-4): per element |out - ref| <= 0.15 + 2^-4 |ref|, and rms(out - ref) <= 6 % of rms(ref).
FP8_ATOL, FP8_RTOL, FP8_RMS = 0.15, 2.0 ** -4, 0.06


def cpu_decode(case, gpu_out, cfg, n_seq=CPU_SAMPLE_SEQS):
    """Oracle on the host cores over the first n_seq sequences; also checks the GPU result of those."""
    import torch
    from oracle import attention_oracle as orc

    n_seq = min(n_seq, case.q.shape[0])
    ctx = case.context_lens_host[:n_seq]
    nblk = (ctx + 15) // 16
    ids = torch.cat([case.block_tables[b, :int(nblk[b])] for b in range(n_seq)]).long()
    kc = case.k_cache[ids].cpu()
    vc = case.v_cache[ids].cpu()
    ks = case.k_scale[ids].cpu() if case.k_scale is not None else None
    vs = case.v_scale[ids].cpu() if case.v_scale is not None else None
    bt = torch.zeros(n_seq, int(nblk.max()), dtype=torch.int32)
    off = 0
    for b in range(n_seq):
        bt[b, :int(nblk[b])] = torch.arange(off, off + int(nblk[b]), dtype=torch.int32)
        off += int(nblk[b])
    q = case.q[:n_seq].cpu()
    torch.set_num_threads(min(os.cpu_count() or 1, 16))
    ref, dt, reps = _timed_repeats(lambda: orc.paged_decode_reference(q, kc, vc, bt, ctx, k_scale=ks, v_scale=vs))
    per_token = 2 * kc.shape[1] * kc.shape[3] * kc.element_size() + (8 * kc.shape[1] / 16 if ks is not None else 0)
    sample_bytes = int(ctx.sum()) * per_token
    got = gpu_out[:n_seq].float().cpu()
    err = (got - ref).abs()
    bound = 2e-2 + 1e-2 * ref.abs()
    base = {"value": sample_bytes / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "seconds_per_pass": dt, "passes": reps,
            "sample": f"configs[{cfg}] first {n_seq} of {case.q.shape[0]} sequences ({int(ctx.sum())} tokens), "
                      f"{reps} passes of oracle paged_decode_reference, torch CPU fp32"}
    parity = {"checked_sequences": n_seq, "max_abs_err": float(err.max()),
              "within_2e-2_abs_1e-2_rel": bool((err <= bound).all())}
    if ks is not None:
        parity["reference"] = "oracle on the dequantised fp8 cache (kernel parity)"
    extra = None
    if case.k_bf16_sample is not None and case.bf16_sample_seqs >= n_seq:
        # the configuration's own error metric: fp8-KV result against fp32 math on the bf16 cache it was quantised from
        n_ids = int(nblk.sum())
        ref16 = orc.paged_decode_reference(q, case.k_bf16_sample[:n_ids].cpu(), case.v_bf16_sample[:n_ids].cpu(), bt, ctx)
        e16 = (got - ref16).abs()
        rms = float((got - ref16).pow(2).mean().sqrt() / ref16.pow(2).mean().sqrt())
        extra = {"reference": "oracle (fp32 math) on the bf16 cache before quantisation", "checked_sequences": n_seq,
                 "max_abs_err": float(e16.max()), "rms_err_over_rms_ref": rms,
                 "bound": f"|err| <= {FP8_ATOL} + 2^-4 |ref| and rms ratio <= {FP8_RMS}",
                 "within_bound": bool((e16 <= FP8_ATOL + FP8_RTOL * ref16.abs()).all()) and rms <= FP8_RMS}
    return base, parity, extra


def cpu_config0(args):
    """configs[0] is the reference's own CPU-runnable case (fp32, B4, 8 = 8 heads, D64, ctx 256): the oracle is timed
    on it (1 warm-up, best of 3) and the HIP kernel is run on the same (bf16-rounded) inputs as a parity and latency
    figure; the working set is cache-resident on the GPU, so no roofline is claimed for it."""
    import torch
    import mi355_attn
    from oracle import attention_oracle as orc

    q, kc, vc, bt, cl = orc.make_paged_case(batch=4, n_q_heads=8, n_kv_heads=8, head_dim=64, block_size=16,
                                            context_lens=[256] * 4, seed=args.seed, dtype=torch.float32)
    torch.set_num_threads(min(os.cpu_count() or 1, 16))
    orc.paged_decode_reference(q, kc, vc, bt, cl)
    best = float("inf")
    for _ in range(3):
        t0 = time.perf_counter()
        ref = orc.paged_decode_reference(q, kc, vc, bt, cl)
        best = min(best, time.perf_counter() - t0)
    nbytes = int(cl.sum()) * 2 * 8 * 64 * 4
    dev = "cuda:0"
    qb, kb, vb = (t.to(torch.bfloat16) for t in (q, kc, vc))
    args_gpu = [t.to(dev) for t in (qb, kb, vb, bt, cl)]
    ws = mi355_attn.paged_decode_workspace(4, 8, 64, 256, dev)
    out = torch.empty_like(args_gpu[0])
    wall_ms, dev_ms = timed(lambda: mi355_attn.paged_attention_decode(*args_gpu, max_context=256, workspace=ws, out=out),
                            args.steps, args.warmup)
    ref16 = orc.paged_decode_reference(qb, kb, vb, bt, cl)
    err = (out.float().cpu() - ref16).abs()
    return {"config": {"workload": "configs[0]: paged decode, fp32 on the CPU path, batch 4, 8 q = 8 kv heads, head_dim 64, "
                                   "block 16, ctx 256, 64-block pool permuted, seed %d" % args.seed,
                       "algorithmic_bytes": nbytes},
            "cpu_baseline": {"value": nbytes / best / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
                             "kind": "port", "seconds_per_pass": best,
                             "sample": "whole configuration, 1 warm-up + best of 3 passes of oracle "
                                       "paged_decode_reference, torch CPU fp32"},
            "gpu": {"ms_per_step": wall_ms, "device_ms": dev_ms, "dtype": "bf16", "note": "cache-resident: latency figure, "
                    "no roofline claim"},
            "parity": {"max_abs_err": float(err.max()), "within_2e-2_abs_1e-2_rel": bool((err <= 2e-2 + 1e-2 * ref16.abs()).all()),
                       "max_abs_diff_bf16_inputs_vs_fp32_inputs": float((ref16 - ref).abs().max())}}


def bench_prefill(cfg, args):
    import torch
    import mi355_attn
    from mi355_attn import workloads

    case = workloads.prefill_config(cfg, seed=args.seed)
    holder = {}

    if case.cu_seqlens is not None:
        def step():
            holder["out"] = mi355_attn.flash_attn_varlen_prefill(case.q, case.k, case.v, case.cu_seqlens,
                                                                 case.cu_seqlens, case.seqlen, case.seqlen, causal=True)
    else:
        def step():
            holder["out"] = mi355_attn.flash_attn_prefill(case.q, case.k, case.v, causal=True)

    wall_ms, dev_ms = timed(step, args.steps, args.warmup, BURN_MS)
    flops = case.flops()
    res = {
        "value": flops / wall_ms / 1e9,
        "unit": "TFLOP/s",
        "ms_per_step": wall_ms,
        "algorithmic_flops": flops,
        "roofline": {
            "bound": "mfma", "kernel": _prefill_kernel(case.q.shape[-1]),
            "achieved": flops / dev_ms / 1e9, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": flops / dev_ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, "device_ms": dev_ms,
            "traffic": _traffic(f"prefill_cfg{cfg}"),
        },
    }
    return res, (case, holder["out"])


def bench_prefill_small(args, with_cpu):
    """The two small prefill shapes: configs[1] (dense, batch 4, 16 heads, head_dim 64, 1024 tokens) and the attention
    call of the reference's sample model (configures/sample.yaml:2-12: batch 64, 16 heads of head_dim 32, context 256,
    through the slot at llm-core/llm_core/model.py:382 with V as the strided view of its projection).  A few
    microseconds of MFMA work each: the figures are launch-bound latencies, reported with their roofline fraction
    but not part of the target.  CPU baseline: the oracle on the whole shape, 1 warm-up + best of 3 passes."""
    import torch
    import mi355_attn
    from mi355_attn import workloads

    out = {}
    case = workloads.prefill_config(1, seed=args.seed)
    B, H, S, D = 64, 16, 256, 32
    g = torch.Generator(device="cuda").manual_seed(args.seed + 3)
    qs = (torch.randn(B, H, S, D, generator=g, device="cuda") * 0.5).to(torch.bfloat16)
    ks = (torch.randn(B, H, S, D, generator=g, device="cuda") * 0.5).to(torch.bfloat16)
    vs = (torch.randn(B, S, H * D, generator=g, device="cuda") * 0.5).to(torch.bfloat16).view(B, S, H, D).permute(0, 2, 1, 3)
    for name, (q, k, v), what in (
            ("prefill_cfg1", (case.q, case.k, case.v),
             "configs[1]: causal prefill forward, bf16, dense, batch 4, 16 heads, head_dim 64, seq 1024, seed %d" % args.seed),
            ("prefill_sample_model", (qs, ks, vs),
             "the reference sample model's attention call (sample.yaml: batch 64, 16 heads, head_dim 32, context 256), "
             "V a strided view, through sdpa_slot")):
        holder = {}

        def step():
            holder["out"] = mi355_attn.sdpa_slot(q, k, v, is_causal=True)

        # Launched one by one from Python the call is bound by the host (about 20 us per call through ctypes, whatever
        # the shape): the roofline figure is taken from a HIP graph of ten calls, the eager time is reported beside it.
        _, eager_ms = timed(step, args.steps, args.warmup, BURN_MS)
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            step()
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=side):
                for _ in range(10):
                    step()
        wall_ms, dev_ms = timed(graph.replay, max(1, args.steps // 2), args.warmup, BURN_MS)
        wall_ms, dev_ms = wall_ms / 10.0, dev_ms / 10.0
        b, h, n, d = q.shape
        flops = 4 * b * h * d * n * n // 2
        nbytes = 4 * b * h * n * d * 2                  # q, k, v read and out written once, bf16
        # which roofline binds: S/4 flops per byte (causal) against the part's 312 -- at these sizes the HBM one
        if nbytes / HBM_PEAK_GBPS / 1e9 >= flops / MFMA_BF16_PEAK_TFLOPS / 1e12:
            roof = {"bound": "hbm", "kernel": _prefill_kernel(d), "achieved": nbytes / dev_ms / 1e6, "peak": HBM_PEAK_GBPS,
                    "unit": "GB/s", "frac": nbytes / dev_ms / 1e6 / HBM_PEAK_GBPS}
        else:
            roof = {"bound": "mfma", "kernel": _prefill_kernel(d), "achieved": flops / dev_ms / 1e9,
                    "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": flops / dev_ms / 1e9 / MFMA_BF16_PEAK_TFLOPS}
        roof.update({"device_ms": dev_ms, "traffic": None, "algorithmic_bytes": nbytes,
                     "mfma_frac": flops / dev_ms / 1e9 / MFMA_BF16_PEAK_TFLOPS,
                     "note": "a few microseconds of work at either peak per call, ten calls per graph launch: a latency figure"})
        res = {
            "value": flops / wall_ms / 1e9, "unit": "TFLOP/s", "ms_per_step": wall_ms, "dtype": "bf16",
            "algorithmic_flops": flops, "config": {"workload": what}, "eager_ms_per_call": eager_ms,
            "roofline": roof,
        }
        if with_cpu:
            from oracle import attention_oracle as orc
            qc, kc, vc = q.cpu(), k.cpu(), v.cpu()
            torch.set_num_threads(min(os.cpu_count() or 1, 16))
            ref = orc.prefill_reference(qc, kc, vc, causal=True, head_chunk=h)
            best = float("inf")
            for _ in range(3):
                t0 = time.perf_counter()
                ref = orc.prefill_reference(qc, kc, vc, causal=True, head_chunk=h)
                best = min(best, time.perf_counter() - t0)
            err = (holder["out"].float().cpu() - ref).abs()
            res["cpu_baseline"] = {"value": flops / best / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
                                   "kind": "port", "seconds_per_pass": best,
                                   "sample": "whole shape, 1 warm-up + best of 3 passes of oracle prefill_reference, "
                                             "torch CPU fp32, causal-convention FLOPs"}
            res["parity"] = {"max_abs_err": float(err.max()),
                             "within_2e-2_abs_1e-2_rel": bool((err <= 2e-2 + 1e-2 * ref.abs()).all())}
        out[name] = res
    return out


def bench_prefill_few_sequences(args):
    """Prefill of ONE sequence (what a per-request prefill of `generate` produces): whole long prompts, whose query
    tiles alone fill the GPU, and a chunk of a prompt over a long cached context, where they do not and the keys
    are split over workgroups (mi355_prefill_fwd_splitkv).  Then one packed batch of very different lengths."""
    import torch
    import mi355_attn

    Hq, Hkv, D = 32, 8, 128
    g = torch.Generator(device="cuda").manual_seed(args.seed + 7)

    def rnd(*shape):
        return (torch.randn(*shape, generator=g, device="cuda") * 0.5).to(torch.bfloat16)

    out = {}
    steps, warmup = max(1, args.steps // 2), args.warmup
    for name, Sq, Sk in (("prompt_8192", 8192, 8192), ("prompt_16384", 16384, 16384), ("prompt_2048", 2048, 2048),
                         ("chunk_256_over_16384", 256, 16384)):
        q, k, v = rnd(1, Hq, Sq, D), rnd(1, Hkv, Sk, D), rnd(1, Hkv, Sk, D)
        flops = 4.0 * Hq * D * (Sq * (Sk - Sq) + Sq * Sq / 2.0)          # causal convention, bottom-right diagonal
        n_split = mi355_attn.suggest_kv_splits(1, Hq, D, Sq, Sk, Sq, True, q.device)
        ws = mi355_attn.prefill_splitkv_workspace(Sq, Hq, D, n_split, q.device) if n_split > 1 else None
        wall_ms, dev_ms = timed(lambda: mi355_attn.flash_attn_prefill(q, k, v, causal=True, kv_splits=n_split, workspace=ws),
                                steps, warmup, BURN_MS)
        res = {
            "value": flops / wall_ms / 1e9, "unit": "TFLOP/s", "ms_per_step": wall_ms, "dtype": "bf16",
            "algorithmic_flops": flops, "kv_splits": n_split,
            "config": {"workload": "causal prefill forward of one sequence, %d query rows over %d keys, 32 q / 8 kv heads, "
                                   "head_dim 128, dense layout" % (Sq, Sk)},
            "roofline": {"bound": "mfma",
                         "kernel": "prefill_fwd_w64_kernel<causal>" if n_split == 1 else
                                   "prefill_fwd_w64_kernel<causal> (keys split %d ways) + prefill_merge_kernel" % n_split,
                         "achieved": flops / dev_ms / 1e9, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": flops / dev_ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, "device_ms": dev_ms, "traffic": None},
        }
        if n_split > 1:
            _, one_ms = timed(lambda: mi355_attn.flash_attn_prefill(q, k, v, causal=True, kv_splits=1), steps, warmup, BURN_MS)
            res["unsplit_device_ms"] = one_ms
            res["speedup_over_unsplit"] = one_ms / dev_ms
        out[name] = res
    # A packed batch of sequences of very different lengths (what a serving step's batched prefill looks like): the
    # kernel deals its (sequence, head, query tile) jobs by cost, so the rate should stay near that of equal lengths.
    import math
    import random
    rng = random.Random(args.seed + 11)
    lens = [int(round(math.exp(rng.uniform(math.log(256), math.log(8192))))) for _ in range(16)]
    T, longest = sum(lens), max(lens)
    cu = torch.tensor([0] + [sum(lens[:i + 1]) for i in range(len(lens))], dtype=torch.int32, device="cuda")
    q, k, v = rnd(T, Hq, D), rnd(T, Hkv, D), rnd(T, Hkv, D)
    flops = sum(4.0 * Hq * D * n * n / 2.0 for n in lens)
    wall_ms, dev_ms = timed(lambda: mi355_attn.flash_attn_varlen_prefill(q, k, v, cu, cu, longest, longest, causal=True, kv_splits=1),
                            steps, warmup, BURN_MS)
    out["ragged_batch_16"] = {
        "value": flops / wall_ms / 1e9, "unit": "TFLOP/s", "ms_per_step": wall_ms, "dtype": "bf16",
        "algorithmic_flops": flops, "kv_splits": 1,
        "config": {"workload": "causal prefill forward of 16 packed sequences, lengths log-uniform in [256, 8192] "
                               "(%d tokens, longest %d), 32 q / 8 kv heads, head_dim 128" % (T, longest)},
        "roofline": {"bound": "mfma", "kernel": "prefill_fwd_w64_kernel<causal>",
                     "achieved": flops / dev_ms / 1e9, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": flops / dev_ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, "device_ms": dev_ms, "traffic": None},
    }
    # Chunks of prompts over context that is already in the paged cache (4 sequences, 2048 new rows each over 8192
    # tokens of context, chunk included), keys and values read through the block table: a bf16 cache by the prefill
    # kernel itself, an fp8 cache through the gather-and-dequantise pass in front of it.
    B, chunk, ctx = 4, 2048, 8192
    nblk = ctx // 16
    g2 = torch.Generator(device="cuda").manual_seed(args.seed + 12)
    pool = B * nblk + 7
    kc = (torch.randn(pool, Hkv, 16, D, device="cuda", generator=g2) * 0.5).to(torch.bfloat16)
    vc = (torch.randn(pool, Hkv, 16, D, device="cuda", generator=g2) * 0.5).to(torch.bfloat16)
    table = torch.randperm(pool, device="cuda", generator=g2)[:B * nblk].view(B, nblk).to(torch.int32)
    lens = torch.full((B,), ctx, dtype=torch.int32, device="cuda")
    cu = (torch.arange(B + 1, device="cuda") * chunk).to(torch.int32)
    q = rnd(B * chunk, Hq, D)
    k8, ks = mi355_attn.quantize_kv_cache_fp8(kc)
    v8, vs = mi355_attn.quantize_kv_cache_fp8(vc)
    flops = 4.0 * Hq * D * B * (chunk * (ctx - chunk) + chunk * chunk / 2.0)
    for name, fn, kernel in (
            ("paged_chunks_4x2048_over_8192",
             lambda: mi355_attn.flash_attn_paged_prefill(q, kc, vc, cu, table, lens, chunk, kv_splits=1),
             "prefill_fwd_w64_kernel<causal, block table>"),
            ("paged_chunks_4x2048_over_8192_fp8",
             lambda: mi355_attn.flash_attn_paged_prefill(q, k8, v8, cu, table, lens, chunk, k_scale=ks, v_scale=vs,
                                                         total_context=B * ctx, kv_splits=1),
             "gather_kv_fp8_kernel + prefill_fwd_w64_kernel<causal>")):
        wall_ms, dev_ms = timed(fn, steps, warmup, BURN_MS)
        out[name] = {
            "value": flops / wall_ms / 1e9, "unit": "TFLOP/s", "ms_per_step": wall_ms, "dtype": "bf16",
            "algorithmic_flops": flops, "kv_splits": 1,
            "config": {"workload": "causal prefill of 4 chunks of 2048 rows over 8192 tokens of paged context each, "
                                   "32 q / 8 kv heads, head_dim 128, block 16" + (", fp8-e4m3 cache" if name.endswith("fp8") else "")},
            "roofline": {"bound": "mfma", "kernel": kernel, "achieved": flops / dev_ms / 1e9, "peak": MFMA_BF16_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": flops / dev_ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, "device_ms": dev_ms,
                         "traffic": None},
        }
    return out


def cpu_prefill(case, gpu_out, cfg, n_heads=8):
    import torch
    from oracle import attention_oracle as orc

    S = case.seqlen
    if case.cu_seqlens is not None:          # packed (T, H, D): sequence 0, first n_heads query heads
        Hq, Hkv = case.q.shape[1], case.k.shape[1]
        n_heads = min(n_heads, Hq)
        n_kv = max(1, n_heads * Hkv // Hq)
        q = case.q[:S, :n_heads].transpose(0, 1)[None].cpu()
        k = case.k[:S, :n_kv].transpose(0, 1)[None].cpu()
        v = case.v[:S, :n_kv].transpose(0, 1)[None].cpu()
        got = gpu_out[:S, :n_heads].transpose(0, 1)[None].float().cpu()
    else:
        n_heads = min(n_heads, case.q.shape[1])
        q, k, v = (t[:1, :n_heads].cpu() for t in (case.q, case.k, case.v))
        got = gpu_out[:1, :n_heads].float().cpu()
    torch.set_num_threads(min(os.cpu_count() or 1, 16))
    ref, dt, reps = _timed_repeats(lambda: orc.prefill_reference(q, k, v, causal=True, head_chunk=4))
    flops = 4 * n_heads * q.shape[-1] * S * S // 2
    err = (got - ref).abs()
    bound = 2e-2 + 1e-2 * ref.abs()
    base = {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "seconds_per_pass": dt, "passes": reps,
            "sample": f"configs[{cfg}] sequence 0, query heads 0..{n_heads - 1} (S={S}), {reps} passes of oracle "
                      "prefill_reference, torch CPU fp32, causal-convention FLOPs"}
    parity = {"checked_heads": n_heads, "max_abs_err": float(err.max()),
              "within_2e-2_abs_1e-2_rel": bool((err <= bound).all())}
    return base, parity


LINE_BUDGET = 7000        # characters of the printed line
PREFILL_TAIL = 1800       # the `prefill` object must sit inside this many last characters


def _sig(x, digits=5):
    """Floats cut to `digits` significant digits (the line is read by people and kept short); the rest unchanged."""
    if isinstance(x, float):
        return float(f"{x:.{digits}g}")
    if isinstance(x, dict):
        return {k: _sig(v, digits) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return [_sig(v, digits) for v in x]
    return x


def _short_cpu(c):
    return None if c is None else {k: c[k] for k in ("value", "unit", "cores", "kind", "sample") if k in c}


def _leg(o):
    """One auxiliary leg as {ms, frac[, cpu]}: device time per launch and the fraction of its roofline."""
    r = o.get("roofline", {})
    d = {"ms": r.get("device_ms", o.get("ms_per_step")), "frac": r.get("frac"), "bound": r.get("bound")}
    if "kv_splits" in o and o["kv_splits"] != 1:
        d["kv_splits"] = o["kv_splits"]
    if "eager_ms_per_call" in o:
        d["eager_ms"] = o["eager_ms_per_call"]
    if "cpu_baseline" in o:
        c = o["cpu_baseline"]
        d["cpu"] = {"value": c["value"], "unit": c["unit"], "cores": c["cores"]}
        d["parity_ok"] = o.get("parity", {}).get("within_2e-2_abs_1e-2_rel")
    return d


def compact_line(full):
    """The printed form of the line: headline fields untouched (floats shortened), auxiliary legs as {ms, frac}
    under "legs", the configs[2] prefill object last and whole (value, ms_per_step, roofline, cpu_baseline, parity)."""
    out = {}
    groups = ("prefill_few_sequences", "prefill_small_shapes", "cache_producers", "layer_ops", "decode_few_sequences")
    tail_keys = ("decode_fp8", "prefill")
    for k, v in full.items():
        if k in groups or k in tail_keys or k in ("prefill_backward", "decode_loop", "config0"):
            continue
        out[k] = v
    if "cpu_baseline" in out:
        out["cpu_baseline"] = _short_cpu(out["cpu_baseline"])
    legs = {}
    for gname in groups:
        for name, o in full.get(gname, {}).items():
            legs[name] = _leg(o)
    if "prefill_backward" in full:
        legs["prefill_backward_cfg2"] = _leg(full["prefill_backward"])
    if "decode_loop" in full:
        dl = full["decode_loop"]
        legs["decode_loop_sample_model"] = {"eager_ms": dl["eager"]["ms_per_step"], "hip_graph_ms": dl["hip_graph"]["ms_per_step"]}
    if "config0" in full:
        c0 = full["config0"]
        legs["config0"] = {"cpu": {"value": c0["cpu_baseline"]["value"], "unit": c0["cpu_baseline"]["unit"],
                                   "cores": c0["cpu_baseline"]["cores"]},
                           "gpu_ms": c0["gpu"]["device_ms"], "parity_ok": c0["parity"]["within_2e-2_abs_1e-2_rel"]}
    if legs:
        out["legs"] = legs
    for k in tail_keys:
        if k in full:
            o = dict(full[k])
            if "cpu_baseline" in o:
                o["cpu_baseline"] = _short_cpu(o["cpu_baseline"])
            o.pop("algorithmic_bytes", None)
            out[k] = o
    return {k: (v if isinstance(v, float) else _sig(v)) for k, v in out.items()}     # headline floats stay exact


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--only", choices=["decode", "prefill", "small", "few", "fp8", "backward", "producers", "layer", "loop"],
                    default=None)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--full", action="store_true", help="print every leg's whole object (a line of about 10 KB)")
    ap.add_argument("--detail", default=None, metavar="PATH", help="also write the verbose form to this file")
    ap.add_argument("--calibrate", action="store_true",
                    help="only run the 1 GiB plain copy kernel (yardstick for rocprofv3 --pmc FETCH_SIZE/WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (attention needs no exchange between GPUs: it shards "
              "by sequences or by kv heads, one process per GPU). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    import mi355_attn
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    mi355_attn.load()
    torch.cuda.set_device(0)
    with_cpu = not args.no_cpu
    if args.calibrate:
        from mi355_attn import _lib
        n = 1 << 30
        a = torch.full((n,), 1, dtype=torch.uint8, device="cuda:0")
        b = torch.empty_like(a)
        for _ in range(max(1, args.steps)):
            _lib.check(_lib.load().mi355_calib_copy(a.data_ptr(), b.data_ptr(), n,
                                                    torch.cuda.current_stream().cuda_stream), "mi355_calib_copy")
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "mi355_calib_copy", "bytes_read": n, "bytes_written": n}))
        return

    line = {
        "metric": METRIC, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "data": "synthetic (seeded)",
    }
    # Every GPU leg runs first, back to back (the shader clock then stays in its loaded state: a GPU that idles
    # through a CPU leg starts the next kernel at a low clock); the CPU oracle legs follow on the kept outputs.
    line["burn_in_ms_before_every_leg_but_decode"] = BURN_MS
    dec = pre = f8 = None
    kept = {}
    if args.only in (None, "decode"):
        dec, kept["decode"] = bench_decode(3, args, with_cpu)
        line.update({
            "value": dec["value"], "unit": "GB/s", "ms_per_step": dec["ms_per_step"], "dtype": "bf16",
            "config": {"workload": "configs[3]: paged decode attention, bf16 KV cache, batch 128, 32 q / 8 kv heads, "
                                   "head_dim 128, block 16, ctx ~ U[512,16384], pool 1.1x, seed %d" % args.seed,
                       "tokens": dec["tokens"], "algorithmic_bytes": dec["algorithmic_bytes"]},
            "roofline": dec["roofline"],
        })
    if args.only in (None, "prefill"):
        pre, kept["prefill"] = bench_prefill(2, args)
        pre["config"] = {"workload": "configs[2]: causal prefill forward, bf16, packed varlen, batch 8, 32 q / 8 kv "
                                     "heads, head_dim 128, seq 4096, seed %d" % args.seed}
        pre["dtype"] = "bf16"
        if args.only == "prefill":
            line.update({"value": pre["value"], "unit": "TFLOP/s", "ms_per_step": pre["ms_per_step"], "dtype": "bf16",
                         "config": pre["config"], "roofline": pre["roofline"]})
    if args.only in (None, "few"):
        line["prefill_few_sequences"] = bench_prefill_few_sequences(args)
    if args.only in (None, "small"):
        line["prefill_small_shapes"] = bench_prefill_small(args, with_cpu)
    if args.only in (None, "backward"):
        line["prefill_backward"] = bench_prefill_backward(2, args)
    if args.only in (None, "fp8"):
        f8, kept["fp8"] = bench_decode(4, args, with_cpu)
        f8["config"] = {"workload": "configs[4]: paged decode attention, fp8-e4m3 KV cache + per-(block, kv head) fp32 "
                                    "scales, batch 256, 64 q / 8 kv heads, head_dim 128, block 16, ctx log-uniform "
                                    "[128,32768], seed %d" % args.seed}
        f8["dtype"] = "fp8 KV / bf16 math"
        line["decode_fp8"] = f8
        if args.only == "fp8":
            line.update({"value": f8["value"], "unit": "GB/s", "ms_per_step": f8["ms_per_step"],
                         "dtype": f8["dtype"], "config": f8["config"], "roofline": f8["roofline"]})
    if args.only in (None, "producers"):
        line["cache_producers"] = bench_producers(args)
    if args.only in (None, "layer"):
        line["layer_ops"] = bench_layer_ops(args)
    if args.only in (None, "loop"):
        line["decode_few_sequences"] = bench_decode_few_sequences(args)
        line["decode_loop"] = bench_decode_loop(args)

    if with_cpu:
        if dec is not None:
            dec["cpu_baseline"], dec["parity"], _ = cpu_decode(*kept.pop("decode"), 3)
            line["cpu_baseline"], line["parity"] = dec["cpu_baseline"], dec["parity"]
        if pre is not None:
            pre["cpu_baseline"], pre["parity"] = cpu_prefill(*kept.pop("prefill"), 2)
            if args.only == "prefill":
                line["cpu_baseline"] = pre["cpu_baseline"]
        if f8 is not None:
            f8["cpu_baseline"], f8["parity"], f8["parity_vs_bf16_kv"] = cpu_decode(*kept.pop("fp8"), 4)
            if args.only == "fp8":
                line["cpu_baseline"] = f8["cpu_baseline"]
        if args.only in (None, "decode"):
            line["config0"] = cpu_config0(args)
    if pre is not None:
        line["prefill"] = pre                     # last key of the line: the other half of the metric
    if args.detail:
        with open(args.detail, "w") as f:
            json.dump(line, f, indent=1)
    print(json.dumps(line if args.full else compact_line(line)))


if __name__ == "__main__":
    main()

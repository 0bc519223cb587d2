#!/usr/bin/env python
"""Decode throughput of the LFM2.5-1.2B-shaped FP8 model at 256 ragged concurrent sequences on one MI355X.

A step is one decode token for every sequence of the batch: HIP-graph replay of the fused decode step
(FP8 W8A8 linears, e4m3 KV cache), on-device sampling and the record kernel.  Prompts (uniform lengths in
[256, 2048], uniform token ids, seed 0) are prefilled before the timed region, so inputs are resident in
HBM when timing starts.  Prints ONE JSON line with the throughput, the roofline of the dominant kernel
(ragged GQA decode attention over the e4m3 cache, timed with device timestamps inside the replayed step) and the CPU
baseline (the oracle's restatement of the reference CPU engine, bf16, on a bounded sample of the same workload).
"""
from __future__ import annotations

import argparse
import itertools
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def fp8_requested(args):
    return args.precision == "fp8"


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=64)
    p.add_argument("--warmup", type=int, default=8)
    p.add_argument("--batch", type=int, default=256)
    p.add_argument("--prompt-low", type=int, default=256)
    p.add_argument("--prompt-high", type=int, default=2048)
    p.add_argument("--max-model-len", type=int, default=8192)
    p.add_argument("--precision", choices=("fp8", "bf16"), default="fp8")
    p.add_argument("--cpu-seqs", type=int, default=4, help="sequences of the workload the CPU baseline runs (0 = skip)")
    p.add_argument("--cpu-steps", type=int, default=16)
    p.add_argument("--attn-samples", type=int, default=20, help="timed launches of the decode-attention kernel per layer")
    p.add_argument("--mid-job-advance", type=int, default=2048,
                   help="second timed point: the same batch with every context this many tokens longer (0 = skip)")
    p.add_argument("--top-k", type=int, default=0, help="top-k filter of the sampler (0: full support)")
    p.add_argument("--top-p", type=float, default=1.0, help="top-p filter of the sampler (1: off)")
    p.add_argument("--workload", choices=("decode", "attention", "gemm", "prefill", "serve", "hbm-ceiling", "mfma-ceiling"), default="decode",
                   help="decode: the model's decode step (the headline metric); attention: the decode-attention call alone "
                        "on 256 sequences of U[128, 8192] history tokens, dense and paged (block 16), e4m3 and bf16; "
                        "gemm: the W8A8 projection shapes at 1..4096 rows; prefill: causal varlen attention over a packed "
                        "4096-token chunk; serve: --requests requests through one session with continuous admit/retire; "
                        "hbm-ceiling: the loads-only streaming read (every CU reading, 8 GiB per launch); mfma-ceiling: the "
                        "register-operand fp8 MFMA loop (every SIMD multiplying, no memory traffic)")
    p.add_argument("--rows", type=str, default="1,8,64,256,1024,4096", help="gemm workload: row counts, comma separated")
    p.add_argument("--shapes", type=str, default="w13,conv_in,qkv,out,w2", help="gemm workload: projection shapes to run")
    p.add_argument("--plain-launches", action="store_true",
                   help="gemm workload: launch every product directly instead of replaying a graph, the fused MLP variants "
                        "left out, and one 256 MiB copy for counter calibration at the end (for `rocprofv3 --pmc` runs)")
    p.add_argument("--adaptive-batching", action="store_true",
                   help="compact graphs (16, 32, 64 ... rows) for a batch that has thinned out, as the reference's switch of that name")
    p.add_argument("--requests", type=int, default=1024, help="requests of the serve workload")
    p.add_argument("--output-low", type=int, default=64, help="serve workload: shortest output, tokens")
    p.add_argument("--output-high", type=int, default=256, help="serve workload: longest output, tokens")
    return p.parse_args()


def gemm_workload(args):
    """The W8A8 product `y = (xq * xs) (Wq * ws)^T` on the model's five projection shapes at 1 to 4096 rows:
    activations N(0,1) with 1 % of the entries scaled by 20 and quantised per token, weights N(0, 0.02) quantised per
    output channel, bf16 out.  Each shape cycles through enough weight copies (>= 1 GiB) that they stream from HBM.
    Every product is checked against the fp32 matmul of the dequantised operands (1e-2 relative, Frobenius)."""
    from climbing_gym_amd import ops
    shapes = {"w13": (11264, 2048), "conv_in": (6144, 2048), "qkv": (3072, 2048), "out": (2048, 2048), "w2": (2048, 5632)}
    shapes = {name: shapes[name] for name in args.shapes.split(",")}
    rows_list = tuple(int(r) for r in args.rows.split(","))
    gen = torch.Generator(device="cuda").manual_seed(0)
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    stream = torch.cuda.current_stream()
    table, worst = {}, 0.0
    for name, (n, k) in shapes.items():
        copies = -(-(1 << 30) // (n * k))
        packs = [ops.PackedFP8Weight.from_weight((torch.randn(n, k, device="cuda", generator=gen) * 0.02).bfloat16())
                 for _ in range(copies)]
        for m in rows_list:
            x = torch.randn(m, k, device="cuda", generator=gen)
            x = torch.where(torch.rand(m, k, device="cuda", generator=gen) < 0.01, x * 20, x).bfloat16()
            xq, xs = ops.quantize_rows(x)
            got = packs[0].linear_quantized(xq, xs).float()
            want = (xq.float() * xs[:, None]) @ (packs[0].values.float() * packs[0].scales[:, None]).t()
            err = float((got - want).norm() / want.norm())
            worst = max(worst, err)
            if not err < 1e-2:
                raise SystemExit(f"W8A8 product differs from the dequantised matmul: {name} rows {m}: {err:.3e}")
            repeats = max(1, 64 // copies)
            def body():
                for _ in range(repeats):
                    for p in packs:
                        p.linear_quantized(xq, xs)
            body()
            torch.cuda.synchronize()
            if args.plain_launches:
                begin.record(stream)
                for _ in range(args.steps):
                    body()
                end.record(stream)
                end.synchronize()
                graph = None
            else:
                side, graph = torch.cuda.Stream(), torch.cuda.CUDAGraph()
                with torch.cuda.stream(side), torch.cuda.graph(graph, stream=side):
                    body()
                torch.cuda.synchronize()
                graph.replay()
                begin.record(stream)
                for _ in range(args.steps):
                    graph.replay()
                end.record(stream)
                end.synchronize()
            sec = begin.elapsed_time(end) / 1000 / (args.steps * repeats * copies)
            moved = n * k + 4 * n + m * k + 4 * m + 2 * m * n
            table[f"{name} n{n} k{k} m{m}"] = {"us": round(sec * 1e6, 2), "GBps": round(moved / sec / 1e9, 1),
                                               "TFLOPs": round(2 * m * n * k / sec / 1e12, 1), "algorithmic_bytes": moved}
            del graph
            if name == "w13" and m in (256, 4096) and not args.plain_launches:
                # the MLP's first half as the engine runs it: projection, SwiGLU and per-token e4m3 rows for the down
                # projection; with the SwiGLU in the product's epilogue, and as projection + SwiGLU launch
                def timed(step):
                    def body():
                        for _ in range(repeats):
                            for p in packs:
                                step(p)
                    body()
                    torch.cuda.synchronize()
                    side, graph = torch.cuda.Stream(), torch.cuda.CUDAGraph()
                    with torch.cuda.stream(side), torch.cuda.graph(graph, stream=side):
                        body()
                    torch.cuda.synchronize()
                    graph.replay()
                    begin.record(stream)
                    for _ in range(args.steps):
                        graph.replay()
                    end.record(stream)
                    end.synchronize()
                    return begin.elapsed_time(end) * 1000 / (args.steps * repeats * copies)
                fused = timed(lambda p: p.linear_swiglu_quantized(xq, xs))
                apart = timed(lambda p: ops.swiglu_fp8(p.linear_quantized(xq, xs)))
                a, b = packs[0].linear_swiglu_quantized(xq, xs), ops.swiglu_fp8(packs[0].linear_quantized(xq, xs))
                if not (torch.equal(a[0].view(torch.uint8), b[0].view(torch.uint8)) and torch.equal(a[1], b[1])):
                    raise SystemExit(f"fused gate+up projection differs from the two launches at {m} rows")
                table[f"w13 + swiglu + quantise m{m}"] = {"fused_us": round(fused, 2), "two_launches_us": round(apart, 2),
                                                          "fused_TFLOPs": round(2 * m * n * k / fused / 1e6, 1)}
        del packs
        torch.cuda.empty_cache()
    if args.plain_launches:
        calibration_copy()
    products = [r for r in table.values() if "GBps" in r]
    big = table.get("w13 n11264 k2048 m4096") or max(products, key=lambda r: r["TFLOPs"])
    small = table.get("w13 n11264 k2048 m256") or max(products, key=lambda r: r["GBps"])
    mfma_peak, mfma_details = measure_mfma_peak(repeats=2)
    print(json.dumps({
        "metric": "W8A8 FP8 GEMM, gate+up projection (N 11264, K 2048) at 4096 rows", "value": big["TFLOPs"],
        "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": 1, "ms_per_step": round(big["us"] / 1000, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp8_e4m3 (fp32 accumulate, bf16 out)",
        "data": "synthetic",
        "config": {"workload": f"W8A8 products of the LFM2.5-1.2B projection shapes {args.shapes} at {args.rows} rows, "
                               "per-token and per-channel scales, weights streamed from HBM",
                   "worst_relative_error": round(worst, 6), "shapes": table},
        "roofline": {"kernel": "gemm_nt_kernel on the tile of the default plan (256x256 of sixteen waves for the gate+up product "
                               "at 4096 rows)", "bound": "mfma", "achieved": big["TFLOPs"],
                     "peak": 5000.0, "unit": "TFLOP/s", "frac": round(big["TFLOPs"] / 5000.0, 4), "traffic": None,
                     "measured_peak": {"TFLOPs": mfma_peak, "by_occupancy": mfma_details,
                                       "what": "register-operand loop of v_mfma_f32_16x16x128_f8f6f4 on every SIMD (lfm2_mfma_fp8_peak)"},
                     "frac_of_measured_peak": round(big["TFLOPs"] / mfma_peak, 4),
                     "decode_rows_256": {"bound": "hbm", "achieved": small["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                         "frac": round(small["GBps"] / HBM_PEAK_GBS, 4)}},
        "cpu_baseline": None}))


def prefill_workload(args):
    """Causal GQA attention over one packed prefill chunk: sequences of U[64, 2048] tokens drawn until they fill 4096
    tokens (the last one cut), 32 query heads over 8 KV heads of 64 dims, bf16.  Checked per sequence against fp32
    softmax attention (2e-2 absolute on N(0,1) inputs)."""
    from climbing_gym_amd import ops
    heads, kv_heads, dim, budget = 32, 8, 64, 4096
    gen = torch.Generator().manual_seed(0)
    lengths = []
    while sum(lengths) < budget:
        lengths.append(min(int(torch.randint(64, 2049, (1,), generator=gen)), budget - sum(lengths)))
    cu = torch.tensor([0] + list(itertools.accumulate(lengths)), dtype=torch.int32, device="cuda")
    torch.manual_seed(0)
    q = torch.randn(budget, heads, dim, device="cuda", dtype=torch.bfloat16)
    k = torch.randn(budget, kv_heads, dim, device="cuda", dtype=torch.bfloat16)
    v = torch.randn(budget, kv_heads, dim, device="cuda", dtype=torch.bfloat16)
    call = lambda: ops.prefill_attention(q, k, v, cu, max(lengths))
    out = call().float()
    worst = 0.0
    for first, n in zip(cu.tolist(), lengths):
        qs = q[first:first + n].float().transpose(0, 1)
        ks = k[first:first + n].float().transpose(0, 1).repeat_interleave(heads // kv_heads, 0)
        vs = v[first:first + n].float().transpose(0, 1).repeat_interleave(heads // kv_heads, 0)
        want = torch.nn.functional.scaled_dot_product_attention(qs, ks, vs, is_causal=True).transpose(0, 1)
        worst = max(worst, float((out[first:first + n] - want).abs().max()))
    if not worst < 2e-2:
        raise SystemExit(f"varlen prefill attention differs from fp32 softmax attention: {worst:.3e}")
    for _ in range(max(args.warmup, 1)):
        call()
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    stream = torch.cuda.current_stream()
    begin.record(stream)
    for _ in range(args.steps):
        call()
    end.record(stream)
    end.synchronize()
    sec = begin.elapsed_time(end) / 1000 / args.steps
    flops = sum(4 * heads * dim * n * (n + 1) // 2 for n in lengths)   # QK^T and PV over the causal triangle
    moved = (2 * budget * heads * dim + 2 * budget * kv_heads * dim) * 2
    print(json.dumps({
        "metric": "causal varlen prefill attention, 4096 packed tokens", "value": round(budget / sec, 1), "unit": "tok/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(sec * 1000, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16 (fp32 softmax and accumulate)",
        "data": "synthetic",
        "config": {"workload": f"one packed chunk of {len(lengths)} sequences, lengths {lengths}, 32 query / 8 KV heads x 64",
                   "worst_abs_error": round(worst, 5), "algorithmic_bytes": moved},
        "roofline": {"kernel": "prefill_attn_kernel", "bound": "mfma", "achieved": round(flops / sec / 1e12, 1), "peak": 2500.0,
                     "unit": "TFLOP/s", "frac": round(flops / sec / 1e12 / 2500.0, 4), "traffic": None},
        "cpu_baseline": None}))


def attention_workload(args):
    """One ragged GQA decode-attention call (one workgroup per row and KV head, finished rows) on 256 sequences with U[128, 8192] history tokens,
    32 query heads over 8 KV heads of 64 dims: history stored dense (each head's tokens contiguous) and in 16-token
    pages reached through a shuffled block table (pages token-major and head-major), e4m3 with scales and bf16.
    Paged results must equal the dense ones bit for bit."""
    from climbing_gym_amd import ops
    rows, kv_heads, heads, dim, capacity, page = 256, 8, 32, 64, 8192, 16
    lengths = torch.randint(128, capacity + 1, (rows,), generator=torch.Generator().manual_seed(0))
    positions = (lengths - 1).to(torch.int32).cuda()
    torch.manual_seed(0)
    q = torch.randn(rows, 1, heads, dim, device="cuda", dtype=torch.bfloat16)
    schedule = ops.decode_schedule(positions, None, None, capacity=capacity)
    tokens = int(lengths.sum())
    results = {}

    def timed(name, bytes_per_token, call):
        for _ in range(max(1, args.warmup // 4)):
            call()
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        begin.record()
        for _ in range(args.steps):
            call()
        end.record()
        end.synchronize()
        us = begin.elapsed_time(end) * 1000 / args.steps
        alg = tokens * bytes_per_token + 2 * rows * heads * dim * 2
        results[name] = {"us_per_call": round(us, 2), "GB/s": round(alg / us / 1e3, 1), "algorithmic_bytes": alg}

    blocks = capacity // page
    order = torch.randperm(rows * blocks, device="cuda")
    table = order.view(rows, blocks).to(torch.int32)

    def to_pages(t):   # [rows, capacity, ...] -> pool [pages, page, ...] under the block table
        src = t.contiguous().reshape(rows * blocks, page, *t.shape[2:])
        pool = torch.empty_like(src)
        if t.dtype == torch.float8_e4m3fn:
            pool.view(torch.uint8)[order] = src.view(torch.uint8)
        else:
            pool[order] = src
        return pool

    def head_major(t):   # the same pages with each head's tokens contiguous inside a page
        rest = range(3, t.ndim)
        return t.permute(0, 2, 1, *rest).contiguous().permute(0, 2, 1, *rest)

    for fp8 in (True, False):
        name = "e4m3" if fp8 else "bf16"
        shape = (rows, kv_heads, capacity, dim)
        if fp8:
            make = lambda: torch.randint(0, 120, shape, device="cuda", dtype=torch.uint8).view(torch.float8_e4m3fn).permute(0, 2, 1, 3)
            k, v = make(), make()
            ks, vs = ((torch.rand(shape[:3], device="cuda") * 0.01).permute(0, 2, 1) for _ in range(2))
        else:
            k, v = (torch.randn(shape, device="cuda", dtype=torch.bfloat16).permute(0, 2, 1, 3) for _ in range(2))
            ks = vs = None
        per_token = 2 * kv_heads * dim * (1 if fp8 else 2) + (2 * kv_heads * 4 if fp8 else 0)
        timed(f"{name} dense", per_token, lambda: ops.attend(q, k, v, ks, vs, positions, schedule=schedule))
        dense = ops.attend(q, k, v, ks, vs, positions, schedule=schedule)
        pk, pv = to_pages(k), to_pages(v)
        pks, pvs = (None, None) if ks is None else (to_pages(ks), to_pages(vs))
        del k, v
        paged = lambda: ops.attend(q, pk, pv, pks, pvs, positions, block_table=table, page=page, schedule=schedule)
        timed(f"{name} paged, token-major pages", per_token, paged)
        same = torch.equal(paged(), dense)
        pk, pv = head_major(pk), head_major(pv)
        if pks is not None:
            pks, pvs = head_major(pks), head_major(pvs)
        timed(f"{name} paged, head-major pages", per_token, paged)
        same = same and torch.equal(paged(), dense)
        if not same:
            raise SystemExit(f"paged {name} attention differs from dense")
        del pk, pv, pks, pvs
        torch.cuda.empty_cache()
    head = results["e4m3 dense"]
    print(json.dumps({
        "metric": "decode attention algorithmic GB/s @256 ragged seqs, history U[128,8192], e4m3 KV", "value": head["GB/s"],
        "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": max(1, args.warmup // 4),
        "ms_per_step": round(head["us_per_call"] / 1000, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8_e4m3 history, bf16 queries, fp32 accumulate", "data": "synthetic",
        "config": {"workload": "one decode-attention call: 256 sequences, history U[128,8192] tokens, 32 query / 8 KV heads x 64, "
                               "dense and 16-token pages, e4m3 + scales and bf16", "context_tokens": tokens, "variants": results},
        "roofline": {"kernel": "decode_attn_mfma_kernel (one workgroup per row and KV head) + quantize_kernel", "bound": "hbm", "achieved": head["GB/s"],
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(head["GB/s"] / HBM_PEAK_GBS, 4), "traffic": None},
        "cpu_baseline": None}))


def serve_workload(args):
    """Continuous admit/retire: `--requests` requests (prompts U[prompt-low, prompt-high], output lengths
    U[output-low, output-high], seed 0) flow through one session of `--batch` slots; a finished request frees its slot, and waiting requests are
    admitted (prefilled) as soon as 16 slots are free or nothing is running.  The figure is whole-job generated tokens
    per second, prefill and host bookkeeping included."""
    import collections
    from climbing_gym_amd.config import LFM25SamplingConfig
    from climbing_gym_amd.synthetic import LFM2_1P2B, random_prompts, random_state_dict
    state = random_state_dict(**LFM2_1P2B, seed=0)
    prompts = random_prompts(args.requests, args.prompt_low, args.prompt_high, LFM2_1P2B["vocab"], seed=0)
    lengths = torch.randint(args.output_low, args.output_high + 1, (args.requests,), generator=torch.Generator().manual_seed(1)).tolist()
    engine, _ = build_engine(args, state)
    sampling = [LFM25SamplingConfig(temperature=1.0, seed=1000 + i, max_new_tokens=n, ignore_eos=True, top_k=args.top_k,
                                    top_p=args.top_p) for i, n in enumerate(lengths)]
    with engine.generation_session(max_batch_size=8, max_new_tokens=args.output_high, cache_len=args.max_model_len) as session:
        session.admit(prompts[:8], sampling[:8])     # loads code objects and warms the allocator
    waiting = collections.deque(range(args.requests))
    running = generated = polls = admissions = 0
    owner = {}
    with engine.generation_session(max_batch_size=args.batch, max_new_tokens=args.output_high, cache_len=args.max_model_len) as session:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while waiting or running:
            free = args.batch - running
            if waiting and (free >= 16 or running == 0):
                take = [waiting.popleft() for _ in range(min(free, len(waiting)))]
                slots = session.admit([prompts[i] for i in take], [sampling[i] for i in take])
                owner.update(zip(slots, take))
                running += len(take)
                admissions += 1
            for result in session.poll():
                if len(result.token_ids) != lengths[owner[result.handle.slot]]:
                    raise SystemExit("a request finished at the wrong length")
                generated += len(result.token_ids)
                session.release(result.handle)
                running -= 1
            polls += 1
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        stats = dict(session.stats)
    if generated != sum(lengths):
        raise SystemExit(f"generated {generated} tokens, expected {sum(lengths)}")
    steps = stats["decode_steps"]
    print(json.dumps({
        "metric": "whole-job output tok/s, continuous admit/retire", "value": round(generated / elapsed, 1), "unit": "tok/s",
        "n_gpus": 1, "steps": steps, "warmup": 0, "ms_per_step": round(elapsed / steps * 1000, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8_e4m3 (W8A8, fp32 accumulate; bf16 activations)" if fp8_requested(args) else "bf16", "data": "synthetic",
        "config": {"workload": f"{args.requests} requests through {args.batch} slots, prompts U[{args.prompt_low},"
                               f"{args.prompt_high}], output lengths U[{args.output_low},{args.output_high}], temperature 1"
                               f"{'' if args.top_k == 0 and args.top_p == 1.0 else f', top-k {args.top_k}, top-p {args.top_p}'}, "
                               f"LFM2.5-1.2B shape, {args.precision} linears and KV cache",
                   "generated_tokens": generated, "prompt_tokens": sum(map(len, prompts)), "seconds": round(elapsed, 3),
                   "admissions": admissions, "polls": polls, "decode_steps": steps,
                   "prompt_plus_output_tok_per_s": round((generated + sum(map(len, prompts))) / elapsed, 1),
                   "mean_compute_rows_per_step": round(stats["decode_row_steps"] / max(steps, 1), 1),
                   "slot_refills": stats["slot_refills"], "adaptive_batching": bool(args.adaptive_batching),
                   "steps_by_compute_rows": dict(stats["decode_batches"])},
        "roofline": None, "cpu_baseline": None}))


def build_engine(args, state):
    from climbing_gym_amd.config import LFM2Config
    from climbing_gym_amd.engine import LFM25Engine
    from climbing_gym_amd.synthetic import LFM2_1P2B
    cfg = LFM2Config(vocab_size=LFM2_1P2B["vocab"], hidden_size=LFM2_1P2B["hidden"], mlp_hidden_size=LFM2_1P2B["mlp_hidden"],
                     num_hidden_layers=16, num_attention_heads=32, num_key_value_heads=8,
                     layer_types=LFM2_1P2B["layer_types"], max_position_embeddings=128000)
    engine = LFM25Engine.from_state_dict(cfg, state, device="cuda", dtype=torch.bfloat16, max_model_len=args.max_model_len)
    fp8 = args.precision == "fp8"
    engine.enable_cuda_graphs(max_graphs=1, max_prefill_tokens=4096, fp8_mlp=fp8, fp8_kv=fp8, fp8_lm_head=fp8, fp8_operators=fp8,
                              adaptive_batching=args.adaptive_batching)
    return engine, cfg


def time_decode_attention(engine, session, samples):
    """Average duration (s) of one decode-attention call in the decode step's form (the attention kernel, one
    workgroup per row and KV head over the schedule the step shares between its layers, plus the row quantiser when the
    out projection is W8A8) at the batch's current context lengths, from HIP events recorded on the launch stream around
    back-to-back launches, and the algorithmic bytes of one call."""
    from climbing_gym_amd import ops
    cfg, cache = engine.config, session.entry.cache
    rows = session.batch_size
    q = torch.randn((rows, 1, cfg.num_attention_heads, cfg.head_dim), device="cuda", dtype=torch.bfloat16)
    positions = (cache.seq_lens - 1).clamp_min(0).contiguous()
    active = torch.ones(rows, device="cuda", dtype=torch.bool)
    schedule = ops.decode_schedule(positions, active, capacity=cache.max_seq_len) if cache.fp8 else None
    # the decode step's form of the call: rows come back e4m3-quantised when the out projection is W8A8
    attention_ops = [l.attention for l in engine.weights.layers if l.attention is not None]
    quantized = bool(cache.fp8 and attention_ops and id(attention_ops[0].out_weight) in engine._fp8()
                     and -(-cfg.num_attention_heads // 16) * -(-cfg.head_dim // 64) <= 4)
    stream = torch.cuda.current_stream()
    layers = cache.k_cache.size(0)
    call_args = [(q, cache.k_cache[layer], cache.v_cache[layer],
                  None if cache.k_scales is None else cache.k_scales[layer],
                  None if cache.v_scales is None else cache.v_scales[layer], positions) for layer in range(layers)]
    run = lambda args: ops.attend(*args, active=active, scale=engine._scaling, schedule=schedule, quantized=quantized)
    for args in call_args:
        run(args)   # warm
    # consecutive calls walk the layers' caches as the decode step does, so every call streams its history from HBM
    # (six layers' histories do not fit the memory-side cache).  One pair of events around the whole run of calls,
    # replayed as a graph like the decode step: kernels of one stream do not overlap, so elapsed / calls is the kernels'
    # durations plus the dispatch gaps between them (an event pair per call would add about 5 us of idle stream to each)
    launches = samples * layers
    side = torch.cuda.Stream()   # captured and replayed as one graph: the host's launch cost stays out of the figure
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side), torch.cuda.graph(graph, stream=side):
        for index in range(launches):
            run(call_args[index % layers])
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    begin.record(stream)
    graph.replay()
    end.record(stream)
    end.synchronize()
    total_ms = begin.elapsed_time(end)
    del graph
    tokens = int((positions.long() + 1).sum())
    kv_token = cfg.num_key_value_heads * cfg.head_dim * 2 * (1 if cache.fp8 else 2) + (cfg.num_key_value_heads * 2 * 4 if cache.fp8 else 0)
    bytes_per_call = tokens * kv_token + 2 * rows * cfg.num_attention_heads * cfg.head_dim * 2
    return total_ms / 1000 / launches, bytes_per_call, tokens


def time_attention_in_step(engine, session, replays):
    """Duration (s) of one decode-attention call (attention kernel + row quantiser) INSIDE the replayed decode step: the
    step is recorded once more with a timestamp kernel (one lane storing the device's constant-rate wall clock) before
    and after each attention layer's call, replayed `replays` times, and the stamps are read after each replay.  This
    is the time the call takes where it runs, after the QKV projection and with the other layers' traffic in the
    caches.  A pair of adjacent stamps costs one dispatch gap, measured in a graph of adjacent pairs and subtracted, so
    the figure holds the two kernels and the gaps between and after them like the back-to-back loop's elapsed / calls."""
    from climbing_gym_amd import ops
    layers = session.entry.cache.k_cache.size(0)
    hz = ops.timestamp_rate_hz()
    stamps = torch.zeros((layers, 2), device="cuda", dtype=torch.int64)
    empty = torch.zeros((16, 2), device="cuda", dtype=torch.int64)
    side, bracket = torch.cuda.Stream(), torch.cuda.CUDAGraph()
    ops.timestamp(empty[0, 0])
    torch.cuda.synchronize()
    with torch.cuda.stream(side), torch.cuda.graph(bracket, stream=side):
        for pair in range(16):
            ops.timestamp(empty[pair, 0])
            ops.timestamp(empty[pair, 1])
    torch.cuda.synchronize()
    bracket.replay()
    bracket.replay()
    torch.cuda.synchronize()
    gap_ticks = float((empty[:, 1] - empty[:, 0]).double().median())
    graph = engine._cuda_decoder.capture_probed_step(session.entry, lambda kind, index, phase: ops.timestamp(stamps[index, phase]))
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    per_layer = torch.zeros(layers, dtype=torch.float64)
    for _ in range(replays):
        graph.replay()
        torch.cuda.synchronize()
        per_layer += (stamps[:, 1] - stamps[:, 0]).double().cpu() - gap_ticks
    del graph, bracket
    per_layer_s = per_layer / replays / hz
    return float(per_layer_s.mean()), {"us_by_layer": [round(v * 1e6, 2) for v in per_layer_s.tolist()],
                                       "bracket_us": round(gap_ticks / hz * 1e6, 2)}


def measure_hbm_ceiling(gib=8, repeats=3):
    """GB/s of the loads-only streaming read (`lfm2_hbm_stream_read`): `gib` GiB per launch, far beyond the 256 MB
    memory-side cache, 2048 workgroups (eight per CU) each streaming a private contiguous region, and the same bytes
    swept by the whole grid together; HIP events around `repeats` launches of each.  Returns (best, {layout: GB/s})."""
    from climbing_gym_amd import ops
    buffer = torch.empty(gib << 28, device="cuda", dtype=torch.int32)
    buffer.zero_()
    buffer[1] = 5     # read by lane 0 of workgroup 0 in both layouts
    groups = 2048
    sink = torch.empty(groups * 256, device="cuda", dtype=torch.int32)
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    stream = torch.cuda.current_stream()
    rates = {}
    for layout, name in ((0, "private_regions"), (1, "grid_sweep")):
        read = ops.hbm_stream_read(buffer, sink, workgroups=groups, layout=layout)
        torch.cuda.synchronize()
        begin.record(stream)
        for _ in range(repeats):
            ops.hbm_stream_read(buffer, sink, workgroups=groups, layout=layout)
        end.record(stream)
        end.synchronize()
        rates[name] = round(read * repeats / (begin.elapsed_time(end) / 1000) / 1e9, 1)
    # every lane folds what it read into one word: the single non-zero word of the buffer must come out, once
    if int(sink[0]) != 5 or int(sink.count_nonzero()) != 1:
        raise SystemExit("the streaming read did not fold what it read")
    del buffer
    torch.cuda.empty_cache()
    return max(rates.values()), rates


def measure_mfma_peak(iterations=20000, repeats=3):
    """TFLOP/s of the register-operand loop of v_mfma_f32_16x16x128_f8f6f4 (`lfm2_mfma_fp8_peak`) with one, two and four
    waves per SIMD on all 256 CUs, HIP events around `repeats` launches of each, and the core clock the loop ran at (its
    cycle counter against the constant-rate clock, median over the workgroups).  Returns (best, details)."""
    from climbing_gym_amd import ops
    props = torch.cuda.get_device_properties(0)
    cus = props.multi_processor_count
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    stream = torch.cuda.current_stream()
    tick_hz = ops.timestamp_rate_hz()
    details = {}
    for waves in (4, 8, 16):
        sink = torch.empty(cus * waves * 64, device="cuda", dtype=torch.float32)
        clock = torch.zeros(2 * cus, device="cuda", dtype=torch.int64)
        flops = ops.mfma_fp8_peak(sink, clock, workgroups=cus, waves=waves, iterations=iterations)
        torch.cuda.synchronize()
        begin.record(stream)
        for _ in range(repeats):
            ops.mfma_fp8_peak(sink, clock, workgroups=cus, waves=waves, iterations=iterations)
        end.record(stream)
        end.synchronize()
        pairs = clock.view(cus, 2).double().cpu()
        ghz = float((pairs[:, 0] / pairs[:, 1].clamp_min(1)).median()) * tick_hz / 1e9
        if not bool(torch.isfinite(sink).all()) or float(sink.abs().max()) == 0.0:
            raise SystemExit("the MFMA loop left no finite result")
        details[f"{waves // 4}_waves_per_simd"] = {"TFLOPs": round(flops * repeats / (begin.elapsed_time(end) / 1000) / 1e12, 1),
                                                   "core_clock_GHz": round(ghz, 3)}
    best = max(v["TFLOPs"] for v in details.values())
    return best, details


def mfma_ceiling_workload(args):
    """What the matrix units deliver with nothing else in the way: the figure the prefill products are held against."""
    best, details = measure_mfma_peak(repeats=max(args.steps, 3))
    print(json.dumps({
        "metric": "dense fp8 MFMA rate, register operands only", "value": best, "unit": "TFLOP/s", "n_gpus": 1,
        "steps": max(args.steps, 3), "warmup": 1, "ms_per_step": None, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "fp8_e4m3 (fp32 accumulate)", "data": "synthetic",
        "config": {"workload": "mfma_fp8_peak_kernel: one workgroup per CU, 20000 rounds of eight independent "
                               "v_mfma_f32_16x16x128_f8f6f4 per wave, no memory traffic in the loop", "by_occupancy": details},
        "roofline": {"kernel": "mfma_fp8_peak_kernel", "bound": "mfma", "achieved": best, "peak": 5000.0, "unit": "TFLOP/s",
                     "frac": round(best / 5000.0, 4), "traffic": None},
        "cpu_baseline": None}))


def ceiling_workload(args):
    """The chip's streaming read rate as this library can measure it: every CU issuing 16-byte loads, nothing else."""
    best, rates = measure_hbm_ceiling(gib=8, repeats=max(args.steps, 3))
    src = torch.ones(64 << 20, device="cuda", dtype=torch.int32)
    dst = torch.empty_like(src)
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.mul(src, 1, out=dst)
    begin.record()
    for _ in range(10):
        torch.mul(src, 1, out=dst)
    end.record()
    end.synchronize()
    copy_rate = round(2 * src.numel() * 4 * 10 / (begin.elapsed_time(end) / 1000) / 1e9, 1)
    print(json.dumps({
        "metric": "HBM streaming read, loads only, 8 GiB per launch", "value": best, "unit": "GB/s", "n_gpus": 1,
        "steps": max(args.steps, 3), "warmup": 1, "ms_per_step": round((8 << 30) / best / 1e6, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u8 (16-byte loads)", "data": "synthetic",
        "config": {"workload": "hbm_stream_kernel: 2048 workgroups x 256 lanes, eight 16-byte loads in flight per lane, 8 GiB "
                               "read once per launch", "layouts_GBps": rates, "elementwise_copy_256MiB_read_plus_write_GBps": copy_rate},
        "roofline": {"kernel": "hbm_stream_kernel", "bound": "hbm", "achieved": best, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(best / HBM_PEAK_GBS, 4), "traffic": None},
        "cpu_baseline": None}))


def time_gemms(engine, rows=256, prefill_rows=4096, repeats=5):
    """Secondary figures: the W8A8 projections at the decode batch size, cycling through the layers' weights so they
    stream from HBM (GB/s of weight bytes; HBM-bound regime), and the fused gate+up projection at a prefill chunk of
    4096 tokens (TFLOP/s against the 5.0 PFLOP/s dense fp8 MFMA peak).  HIP events on the launch stream."""
    from climbing_gym_amd import ops
    fp8 = engine._fp8()
    layers = engine.weights.layers
    groups = {"w13": [fp8.get(id(l.w13_weight)) for l in layers], "w2": [fp8.get(id(l.w2_weight)) for l in layers],
              "qkv": [fp8.get(id(l.attention.qkv_weight)) for l in layers if l.attention is not None],
              "conv_in": [fp8.get(id(l.conv.in_weight)) for l in layers if l.conv is not None],
              "out": [fp8.get(id((l.attention or l.conv).out_weight)) for l in layers]}
    stream = torch.cuda.current_stream()
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    out = {"decode_rows": rows, "decode": {}, "prefill_rows": prefill_rows}

    def run(packs, m):
        width = packs[0].values.size(1)
        x = torch.randn(m, width, device="cuda", dtype=torch.bfloat16)
        xq, xs = ops.quantize_rows(x)
        def body():
            for _ in range(repeats):
                for p in packs:
                    p.linear_quantized(xq, xs)
        body()
        torch.cuda.synchronize()
        side = torch.cuda.Stream()   # captured and replayed as one graph: host launch cost stays out of the figure
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side), torch.cuda.graph(graph, stream=side):
            body()
        torch.cuda.synchronize()
        graph.replay()
        begin.record(stream)
        graph.replay()
        end.record(stream)
        end.synchronize()
        return begin.elapsed_time(end) / 1000 / (repeats * len(packs))
    for name, packs in groups.items():
        if any(p is None for p in packs) or not packs:
            continue
        n, k = packs[0].values.shape
        sec = run(packs, rows)
        out["decode"][name] = {"n": n, "k": k, "us": round(sec * 1e6, 2), "weight_GBps": round(n * k / sec / 1e9, 1),
                               "TFLOPs": round(2 * rows * n * k / sec / 1e12, 1)}
    packs = groups["w13"]
    if packs and packs[0] is not None:
        n, k = packs[0].values.shape
        sec = run(packs[:4], prefill_rows)
        tflops = 2 * prefill_rows * n * k / sec / 1e12
        peak, _ = measure_mfma_peak(repeats=2)
        out["prefill"] = {"name": "w13", "n": n, "k": k, "us": round(sec * 1e6, 1), "TFLOPs": round(tflops, 1),
                          "mfma_fp8_frac_of_5PF": round(tflops / 5000, 4), "measured_mfma_peak_TFLOPs": peak,
                          "mfma_fp8_frac_of_measured_peak": round(tflops / peak, 4)}
    return out


def calibration_copy():
    """One plain elementwise copy of known size (256 MiB read, 256 MiB written).  It costs nothing measurable in a
    normal run; under `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` its counter reading gives the factor that turns
    the decode-attention kernel's counter readings into bytes."""
    src = torch.ones(64 << 20, device="cuda", dtype=torch.int32)
    dst = torch.empty_like(src)
    torch.mul(src, 1, out=dst)
    torch.cuda.synchronize()


def measured_traffic(args, attn_bytes):
    """HBM bytes per decode-attention call: the ratio of counter-measured to algorithmic bytes in the committed
    FETCH_SIZE / WRITE_SIZE summary (taken on this workload a few decode steps earlier or later), applied to this
    run's algorithmic bytes.  None when the summary is absent or was taken on another workload."""
    path = os.path.join(ROOT, "profiles", "decode_attention_hbm_traffic.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        rec = json.load(f)
    same = (rec.get("batch") == args.batch and rec.get("precision") == args.precision
            and rec.get("prompt_range") == [args.prompt_low, args.prompt_high])
    return int(rec["ratio"] * attn_bytes) if same else None


def cpu_baseline(args, state, prompts):
    """The oracle (restatement of the reference CPU engine) on the first `cpu_seqs` sequences of the workload, with
    bf16 weights and activations as the reference's engine holds a 1.2B model: one untimed warm-up (a short prompt and
    two steps), then two repeats of prefill + `cpu_steps` greedy decode steps, both phases timed, on all host threads;
    the medians are reported, `value` being the decode rate (the metric is decode output tok/s)."""
    from climbing_gym_amd.synthetic import LFM2_1P2B
    from oracle.lfm2_oracle import OracleConfig, OracleEngine
    torch.set_num_threads(max(1, min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))))
    ocfg = OracleConfig(vocab_size=LFM2_1P2B["vocab"], hidden_size=LFM2_1P2B["hidden"], mlp_hidden_size=LFM2_1P2B["mlp_hidden"],
                        num_hidden_layers=16, num_attention_heads=32, num_key_value_heads=8,
                        layer_types=LFM2_1P2B["layer_types"])
    oracle = OracleEngine(ocfg, state, torch.bfloat16, max_model_len=args.max_model_len)
    sample = prompts[:args.cpu_seqs]
    slots = torch.arange(len(sample))
    decode_rates, prefill_rates = [], []
    with torch.inference_mode():
        cache, logits = oracle.prefill([sample[0][:64]], cap=72)
        for _ in range(2):
            logits = oracle.append_tokens(cache, torch.arange(1), logits.argmax(-1))
        for _ in range(2):
            start = time.perf_counter()
            cache, logits = oracle.prefill(sample, cap=max(map(len, sample)) + args.cpu_steps + 1)
            tokens = logits.argmax(-1)
            middle = time.perf_counter()
            for _ in range(args.cpu_steps):
                logits = oracle.append_tokens(cache, slots, tokens)
                tokens = logits.argmax(-1)
            done = time.perf_counter()
            prefill_rates.append(sum(map(len, sample)) / (middle - start))
            decode_rates.append(len(sample) * args.cpu_steps / (done - middle))
    median = lambda xs: sorted(xs)[len(xs) // 2] if len(xs) % 2 else sum(sorted(xs)[len(xs) // 2 - 1:len(xs) // 2 + 1]) / 2
    return {"value": round(median(decode_rates), 3), "unit": "tok/s", "cores": torch.get_num_threads(), "kind": "port",
            "prefill_tok_per_s": round(median(prefill_rates), 1),
            "sample": f"first {len(sample)} of the {args.batch} sequences ({sum(map(len, sample))} prompt tokens), bf16 weights and "
                      f"activations, one warm-up, then the median of 2 repeats of prefill (timed apart) + {args.cpu_steps} greedy "
                      "decode steps; a bounded sample because the whole batch would take hours on the host"}


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one MI355X; --gpus {args.gpus} is not supported in this build "
              "(the path shards by slots across independent engines with no collective in the step).", file=sys.stderr)
        sys.exit(2)
    if args.workload != "decode":
        with torch.inference_mode():
            {"attention": attention_workload, "gemm": gemm_workload, "prefill": prefill_workload,
             "serve": serve_workload, "hbm-ceiling": ceiling_workload, "mfma-ceiling": mfma_ceiling_workload}[args.workload](args)
        return
    from climbing_gym_amd.config import LFM25SamplingConfig
    from climbing_gym_amd.synthetic import LFM2_1P2B, random_prompts, random_state_dict

    state = random_state_dict(**LFM2_1P2B, seed=0)
    prompts = random_prompts(args.batch, args.prompt_low, args.prompt_high, LFM2_1P2B["vocab"], seed=0)
    engine, cfg = build_engine(args, state)
    new_tokens = min(4096, args.max_model_len - max(map(len, prompts)))
    sampling = [LFM25SamplingConfig(temperature=1.0, seed=1000 + i, max_new_tokens=new_tokens, ignore_eos=True,
                                    top_k=args.top_k, top_p=args.top_p) for i in range(args.batch)]
    # a first admission of a few prompts into a throw-away session: kernel code objects and the allocator's blocks are
    # loaded once per process, and the prefill rate reported is that of an engine that has served before
    with torch.inference_mode(), engine.generation_session(max_batch_size=8, max_new_tokens=new_tokens,
                                                            cache_len=args.max_model_len) as session:
        session.admit(prompts[:8], sampling[:8])
    with torch.inference_mode(), engine.generation_session(max_batch_size=args.batch, max_new_tokens=new_tokens,
                                                            cache_len=args.max_model_len) as session:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        session.admit(prompts, sampling)
        torch.cuda.synchronize()
        prefill_s = time.perf_counter() - t0
        prefill_plan = dict(engine.last_prefill)
        session.poll(steps=max(args.warmup, 1))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        finished = session.poll(steps=args.steps)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        assert not finished, "no sequence may finish inside the timed region"
        attn_s, attn_bytes, ctx_tokens = time_decode_attention(engine, session, args.attn_samples)
        in_step_s, in_step_layers = time_attention_in_step(engine, session, max(args.attn_samples // 2, 4))
        kv_token = 6 * (attn_bytes - 2 * args.batch * 32 * 64 * 2) // max(ctx_tokens, 1)
        # the same batch later in the job: every row's context longer by `--mid-job-advance` tokens (the cache is
        # written by the steps that follow; what the history holds does not change what the step costs)
        mid = None
        # every position a step of this run will write must lie inside the cache: the steps timed so far, the probed
        # replays, then 2 + steps more at the advanced lengths, and the probed replays there
        cache = session.entry.cache
        headroom = cache.max_seq_len - int(cache.seq_lens.max()) - (2 + args.steps + 2 * args.attn_samples + 16)
        advance = min(args.mid_job_advance, headroom)
        if 0 < advance < args.mid_job_advance:
            print(f"--mid-job-advance {args.mid_job_advance} does not fit the {cache.max_seq_len}-token cache behind the "
                  f"longest row: advancing by {advance}", file=sys.stderr)
        if advance > 0:
            cache.seq_lens.add_(advance)   # the skipped span holds the zeros the cache was allocated with
            session.poll(steps=2)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            finished = session.poll(steps=args.steps)
            torch.cuda.synchronize()
            mid_elapsed = time.perf_counter() - t0
            assert not finished, "no sequence may finish inside the timed region"
            mid_attn_s, mid_attn_bytes, mid_tokens = time_decode_attention(engine, session, max(args.attn_samples // 2, 2))
            mid_in_step_s, _ = time_attention_in_step(engine, session, max(args.attn_samples // 4, 3))
            mid = (mid_elapsed, mid_attn_s, mid_attn_bytes, mid_tokens, mid_in_step_s, advance)
        calibration_copy()
        gemms = time_gemms(engine) if fp8_requested(args) else None
        ceiling, ceiling_layouts = measure_hbm_ceiling()
    fp8 = args.precision == "fp8"
    weights = sum(w.numel() for w in set(engine.weights.linear_matrices())) * (1 if fp8 else 2)
    fixed_bytes = weights + args.batch * 122880 * 2 + args.batch * cfg.vocab_size * 2 * 2
    step_bytes = fixed_bytes + ctx_tokens * kv_token
    ms_per_step = elapsed / args.steps * 1000
    # the roofline figure is the call's time INSIDE the replayed step; the back-to-back loop over the layers' caches
    # (faster: no other kernel's traffic between the calls) is reported next to it
    loop_achieved = attn_bytes / attn_s / 1e9
    launch_s = in_step_s if in_step_s is not None else attn_s
    achieved = attn_bytes / launch_s / 1e9
    mid_job = None
    if mid is not None:
        mid_elapsed, mid_attn_s, mid_attn_bytes, mid_tokens, mid_in_step_s, advance = mid
        mid_ms = mid_elapsed / args.steps * 1000
        mid_bytes = fixed_bytes + mid_tokens * kv_token
        mid_launch_s = mid_in_step_s if mid_in_step_s is not None else mid_attn_s
        mid_job = {"advance": advance, "context_tokens": mid_tokens, "ms_per_step": round(mid_ms, 4),
                   "tok_per_s": round(args.batch * args.steps / mid_elapsed, 1), "step_algorithmic_bytes": mid_bytes,
                   "step_hbm_fraction": round(mid_bytes / (mid_ms / 1000) / 1e9 / HBM_PEAK_GBS, 4),
                   "attention_us_per_call": round(mid_launch_s * 1e6, 2),
                   "attention_GBps": round(mid_attn_bytes / mid_launch_s / 1e9, 1),
                   "attention_frac": round(mid_attn_bytes / mid_launch_s / 1e9 / HBM_PEAK_GBS, 4),
                   "attention_frac_of_measured_ceiling": round(mid_attn_bytes / mid_launch_s / 1e9 / ceiling, 4),
                   "attention_loop_us_per_call": round(mid_attn_s * 1e6, 2)}
    line = {
        "metric": "decode output tok/s @256 ragged seqs, LFM2.5-1.2B FP8; % HBM roofline",
        "value": round(args.batch * args.steps / elapsed, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "fp8_e4m3 (W8A8, fp32 accumulate; bf16 activations)" if fp8 else "bf16",
        "data": "synthetic",
        "config": {"workload": f"LFM2.5-1.2B-shaped random-init model, {args.precision} linears and KV cache, {args.batch} "
                               f"concurrent sequences, prompts U[{args.prompt_low},{args.prompt_high}] tokens, temperature 1"
                               f"{'' if args.top_k == 0 and args.top_p == 1.0 else f', top-k {args.top_k}, top-p {args.top_p}'}, "
                               f"max_model_len {args.max_model_len}, HIP-graph decode step",
                   "context_tokens": ctx_tokens, "prefill_tok_per_s": round(sum(map(len, prompts)) / prefill_s, 1),
                   "prefill_chunks": prefill_plan.get("chunks"), "prefill_chunk_fill": round(prefill_plan.get("fill", 0.0), 4),
                   "gemm": gemms, "step_algorithmic_bytes": step_bytes,
                   "step_hbm_fraction": round(step_bytes / (ms_per_step / 1000) / 1e9 / HBM_PEAK_GBS, 4),
                   "step_fraction_of_measured_ceiling": round(step_bytes / (ms_per_step / 1000) / 1e9 / ceiling, 4),
                   "mid_job": mid_job},
        "roofline": {"kernel": "decode_attn_mfma_kernel, one workgroup per row and KV head, + quantize_kernel (one ragged GQA decode-attention call, e4m3 KV, rows quantised for the W8A8 out projection as in the decode step)"
                               if fp8 else "decode_attn_mfma_kernel, one workgroup per row and KV head (one ragged GQA decode-attention call, bf16 KV)",
                     "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": measured_traffic(args, attn_bytes),
                     "timed": "device timestamps recorded before and after the call inside the replayed decode step",
                     "avg_launch_us": round(launch_s * 1e6, 2), "in_step": in_step_layers,
                     "algorithmic_bytes_per_launch": attn_bytes,
                     "back_to_back_loop": {"avg_launch_us": round(attn_s * 1e6, 2), "achieved": round(loop_achieved, 1),
                                           "frac": round(loop_achieved / HBM_PEAK_GBS, 4)},
                     "measured_ceiling": {"GBps": ceiling, "layouts_GBps": ceiling_layouts,
                                          "what": "loads-only streaming read of 8 GiB by 2048 workgroups (lfm2_hbm_stream_read)"},
                     "frac_of_measured_ceiling": round(achieved / ceiling, 4)},
    }
    del session
    engine.disable_cuda_graphs()
    torch.cuda.empty_cache()
    line["cpu_baseline"] = cpu_baseline(args, state, prompts) if args.cpu_seqs > 0 else None
    print(json.dumps(line))


if __name__ == "__main__":
    main()

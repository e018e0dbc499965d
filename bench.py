#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, with random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--shape 0.6b|8b|32b] [--batch B] ...

The default run has the layer sizes of the Qwen3-0.6B shape (28 layers, hidden 1024, 16 query
heads, 8 key/value heads, head_dim 128, intermediate 3072, vocabulary 151936, tied head), a
batch of 8 requests with 1,024-token prompts inside a 4,096-token context limit, bfloat16. A
"step" is one decode step of the whole engine (schedule, run the batch from a HIP graph,
sample, update). W warm-up steps, then exactly K timed steps between synchronisations; such
regions of K steps follow each other until half a second has been timed, and the median region
is the one reported (``timed_regions`` says how many there were). One JSON line is printed:

  value        decoded tokens per second at the default batch
  prefill      one 2,048-token prompt run whole: tokens/s, ms, and its share of the bf16 MFMA peak
  roofline     bytes the decode step has to read (every weight once, the live requests' cache)
               divided by its time, against 8 TB/s of HBM
  points       decode tokens/s at batch 1 and batch 64

``--emit-kernels CSV`` measures nothing: it takes the kernel trace that rocprofv3 wrote for a run
with the same options and prints one row per kernel of the step with its time, the bytes it has to
move, its operations and the share of the HBM and MFMA peaks these amount to.

``--only floor`` times a replayed graph of empty kernels: what every dependent launch of a decode step
costs before it computes anything.

``--only graphs`` records every decode graph the configuration can ask for ahead of serving and prints
their number, the time and the device memory they took.

``--only serve`` runs a continuous-batching workload instead (``--requests`` requests, 256 by
default, with prompt lengths uniform in 128..2048 and ``--gen-len`` generated tokens each, all
submitted at once under a budget of ``--token-budget`` tokens a step) and prints its own line:
generated tokens per second over the whole run, with the time of the run and the number of steps.

Weights are seeded random tensors of the named shape and prompts are seeded uniform token ids
(there is no network for checkpoints or datasets). The reference publishes no number for this
metric, so ``vs_baseline`` is null.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from minivllm_amd.config.shapes import QWEN3_SHAPES

SHAPES = {k: v for k, v in QWEN3_SHAPES.items() if k != "tiny"}
MIN_TIMED_SECONDS = 0.5
MAX_REGIONS = 101
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}


def model_numbers(c, layers):
    h, I, V = c["hidden_size"], c["intermediate_size"], c["vocab_size"]
    q, kv = c["num_attention_heads"] * c["head_dim"], c["num_key_value_heads"] * c["head_dim"]
    layer_params = h * (q + 2 * kv) + q * h + 3 * h * I + 2 * h + 2 * c["head_dim"]
    matrix_params = layers * (h * (q + 2 * kv) + q * h + 3 * h * I)
    return dict(layer_params=layer_params, step_params=layers * layer_params + h + V * h,
                matrix_params=matrix_params, kv_bytes_per_token=layers * 2 * kv)


def build_llm(args, shape, layers, max_seqs=None, token_budget=None, num_pages=None):
    import torch
    from minivllm_amd import LLM
    from minivllm_amd.config import EngineConfig
    from minivllm_amd.models import config_from_dict, expected_tensors
    from minivllm_amd.weights.device_random import DeviceRandomSource

    raw = dict(shape, architectures=["Qwen3ForCausalLM"], num_hidden_layers=layers,
               max_position_embeddings=40960, torch_dtype=args.dtype)
    arch, cfg = config_from_dict(raw)
    dev = torch.device("cuda:0")
    stored = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    source = DeviceRandomSource(expected_tensors(arch, cfg), args.seed, stored, dev)
    pages_per_seq = -(-args.context // args.block_size)
    ec = EngineConfig(model="", dtype=args.dtype, max_model_len=args.context,
                      max_num_batched_tokens=token_budget or max(args.prefill_tokens, 2048),
                      max_num_batched_seqs=max_seqs or max(64, args.batch),
                      kv_cache_block_size=args.block_size,
                      kv_cache_num_blocks=num_pages or max(64, args.batch) * pages_per_seq + 16,
                      use_cuda_graph=not args.no_graph, num_scheduler_steps=args.scheduler_steps, seed=args.seed)
    if getattr(args, "launch_ahead", None) is not None:
        ec.launch_ahead = bool(args.launch_ahead)
    return LLM(config=ec, model_source=(arch, cfg, source)), cfg


def random_prompt(vocab, n, seed):
    import numpy as np
    return [int(t) for t in np.random.default_rng(seed).integers(0, vocab, size=n)]


def measure_decode(llm, vocab, batch, prompt_len, steps, warmup, seed):
    """Tokens per second over ``steps`` decode steps (tokens per request) at ``batch`` after the
    prompts are in the cache. One call of ``llm.step()`` may run several decode steps in a row on
    the device; what is counted is what the requests received."""
    import torch
    from minivllm_amd import SamplingParams
    # room for what the first requests decode while the last prompts are still being read
    sp = SamplingParams(temperature=0.0, max_tokens=llm.config.max_model_len - prompt_len - 1, ignore_eos=True)
    reqs = [llm.submit(random_prompt(vocab, prompt_len, seed + i), sp) for i in range(batch)]
    while any(r.num_completion_tokens == 0 for r in reqs):          # prompts in, first token drawn
        llm.step()
    ahead = llm.config.launch_ahead

    def run(n):
        target = min(r.num_completion_tokens for r in reqs) + n
        try:
            while min(r.num_completion_tokens for r in reqs) < target:
                # the steps that reach the target are not followed by steps launched ahead: the timed
                # region then holds exactly n steps and nothing runs on when its clock is read
                to_go = target - min(r.num_completion_tokens for r in reqs)
                llm.config.launch_ahead = ahead and to_go > llm.config.num_scheduler_steps
                if llm.step() is None or any(r.finished for r in reqs):
                    raise RuntimeError("a request of the benchmark ended before the timed steps were over; "
                                       "give it a longer --context")
        finally:
            llm.config.launch_ahead = ahead
    run(warmup)
    # Regions of exactly ``steps`` steps, each between synchronisations, one after the other until
    # MIN_TIMED_SECONDS have been timed (or the context limit is near): the median region is reported,
    # so that a short region (20 steps are 30 ms) does not stand on one sample.
    regions = []
    margin = steps + 2 * llm.config.num_scheduler_steps + 2
    while True:
        torch.cuda.synchronize()
        before = sum(r.num_completion_tokens for r in reqs)
        ctx_before = prompt_len + min(r.num_completion_tokens for r in reqs)
        t0 = time.perf_counter()
        run(steps)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        tokens = sum(r.num_completion_tokens for r in reqs) - before
        regions.append((dt / (tokens / batch), tokens, dt, ctx_before + tokens / batch / 2.0))
        longest = prompt_len + max(r.num_completion_tokens for r in reqs)
        if sum(r[2] for r in regions) >= MIN_TIMED_SECONDS or longest + margin >= llm.config.max_model_len \
                or len(regions) >= MAX_REGIONS:
            break
    regions.sort()
    per_step, tokens, dt, mean_ctx = regions[len(regions) // 2]
    done_steps = tokens / batch
    # finish and free
    for r in reqs:
        r.sampling_params.max_tokens = r.num_completion_tokens
    while llm.has_unfinished():
        llm.step()
    return tokens / dt, per_step * 1e3, mean_ctx, int(round(done_steps)), len(regions)


def measure_prefill(llm, vocab, tokens, repeats, seed):
    import torch
    from minivllm_amd import SamplingParams
    times = []
    for i in range(repeats + 1):
        r = llm.submit(random_prompt(vocab, tokens, seed + 100 + i), SamplingParams(temperature=0.0, max_tokens=1,
                                                                                     ignore_eos=True))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while not r.finished:
            llm.step()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    return min(times[1:]) if repeats else times[0]


def measure_serve(llm, vocab, requests, gen_len, seed, prompt_min=128, prompt_max=2048):
    """All requests submitted at once; returns (seconds, generated tokens, prompt tokens, steps, preemptions)."""
    import numpy as np
    import torch
    from minivllm_amd import SamplingParams
    rng = np.random.default_rng(seed)
    prompts = [[int(t) for t in rng.integers(0, vocab, size=int(n))]
               for n in rng.integers(prompt_min, prompt_max + 1, size=requests)]
    # a few requests through every kind of step first (graphs are captured on first use)
    llm.generate(prompts[:4], SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True), use_tqdm=False)
    torch.cuda.synchronize()
    sp = SamplingParams(temperature=0.0, max_tokens=gen_len, ignore_eos=True)
    before = llm.scheduler.num_preemptions
    reqs = [llm.submit(p, sp) for p in prompts]
    steps = 0
    t0 = time.perf_counter()
    while llm.has_unfinished():
        llm.step()
        steps += 1
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    return (dt, sum(r.num_completion_tokens for r in reqs), sum(len(p) for p in prompts), steps,
            llm.scheduler.num_preemptions - before)


def measure_floor(args) -> int:
    """What a dependent kernel launch costs inside a replayed graph, whatever the kernel does: a graph of
    ``--nodes`` empty kernels in a row (170 by default, about the nodes of a decode step of the default
    shape before fusion), replayed; microseconds per node at several launch sizes."""
    import torch
    from minivllm_amd.kernels.ops import dtype_from_name, get_ops
    ops = get_ops(dtype_from_name(args.dtype))
    buf = torch.zeros(16, device="cuda:0")
    points = {}
    for grid, block in ((1, 64), (256, 64), (256, 256), (256, 512), (1024, 256)):
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            launch = lambda: ops.lib.call("mv_launch_empty", grid, block, buf.data_ptr(), torch.cuda.current_stream().cuda_stream)
            launch()
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                for _ in range(args.nodes):
                    launch()
            for _ in range(3):
                g.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(200):
                g.replay()
            torch.cuda.synchronize()
            points[f"{grid}x{block}"] = round((time.perf_counter() - t0) / 200 / args.nodes * 1e6, 3)
    print(json.dumps({"metric": "microseconds per dependent empty kernel in a replayed graph of %d" % args.nodes,
                      "value": points["256x256"], "unit": "us", "n_gpus": 1, "higher_is_better": False,
                      "points": points, "nodes": args.nodes}))
    return 0


def emit_kernels(llm, cfg, args) -> int:
    """Prints, for the step kinds of this run, a table of their kernels: time from the rocprofv3
    kernel trace ``args.emit_kernels``, bytes and operations from what the engine launches."""
    from minivllm_amd import SamplingParams
    from minivllm_amd.engine import roofline
    vocab = cfg.vocab_size
    ex = llm.executor
    if args.only in ("all", "decode"):
        k = llm.config.num_scheduler_steps
        sp = SamplingParams(temperature=0.0, max_tokens=llm.config.max_model_len - args.prompt_len - 1, ignore_eos=True)
        reqs = [llm.submit(random_prompt(vocab, args.prompt_len, args.seed + i), sp) for i in range(args.batch)]
        while any(r.num_completion_tokens == 0 for r in reqs):          # prompts in, first token drawn
            llm.step()
        for _ in range(3):                                               # the whole batch decodes: its graphs are recorded
            llm.step()
        for r in reqs:
            r.sampling_params.max_tokens = r.num_completion_tokens
        while llm.has_unfinished():
            llm.step()
        rows = [key for key in ex.graph_ledger if len(key) == 3 and key[0] >= args.batch]
        single = [key for key in ex.graph_ledger if len(key) == 2 and key[0] >= args.batch]
        if not rows and not single:
            print("bench.py: no decode graph was recorded for this batch (graphs off?); nothing to price")
            return 2
        key = max(rows, key=lambda t: (-t[0], t[2])) if rows else min(single)
        ledger = roofline.one_step(roofline.launches(ex.graph_ledger[key]))
        ctx = args.prompt_len + (args.warmup + args.steps) // 2
        title = (f"decode step, qwen3-{args.shape} shape, batch {args.batch}, priced at a context of {ctx} tokens "
                 f"(graph for {key[0]} sequences, contexts up to {key[1]})")
        print(roofline.kernel_table(args.emit_kernels, ledger, args.dtype, keys=args.batch * ctx, pairs=args.batch * ctx,
                                    title=title, wall_ms=args.step_ms))
    if args.only in ("all", "prefill"):
        if args.only == "all":
            print()
        sp = SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True)
        llm.submit(random_prompt(vocab, args.prefill_tokens, args.seed + 100), sp)
        before = set(ex.graph_ledger)
        ex.ops.ledger = []
        try:
            while llm.has_unfinished():
                llm.step()
            # a prompt step that is replayed from a graph leaves its launches with the graph it recorded
            recorded = [k for k in ex.graph_ledger if k not in before and k and k[0] == "mixed"]
            lines = ex.graph_ledger[recorded[-1]] if recorded else ex.ops.ledger
            ledger = roofline.launches(lines)
        finally:
            ex.ops.ledger = None
        title = f"prefill of one {args.prefill_tokens}-token prompt, qwen3-{args.shape} shape"
        print(roofline.kernel_table(args.emit_kernels, ledger, args.dtype, title=title,
                                    wall_ms=args.step_ms if args.only == "prefill" else None))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--shape", choices=sorted(SHAPES), default="0.6b")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (named in the record)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=1024)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--no-graph", action="store_true")
    ap.add_argument("--scheduler-steps", type=int, default=4,
                    help="decode steps run in a row on the device before the host looks at the tokens")
    ap.add_argument("--launch-ahead", type=int, choices=[0, 1], default=None,
                    help="launch the next decode steps before the running ones' tokens are read (default: the engine's)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and batch 64 points")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--only", "--mode", dest="only", choices=["all", "decode", "prefill", "serve", "floor", "graphs"],
                    default="all",
                    help="measure one phase alone (for profiling); the line then lacks the other's fields. "
                         "'serve': the continuous-batching workload; 'floor': what a dependent launch costs in a graph; "
                         "'graphs': time and device memory of recording every decode graph ahead of serving "
                         "(--max-seqs sequences, contexts up to --context)")
    ap.add_argument("--nodes", type=int, default=170, help="kernels in the graph of --only floor")
    ap.add_argument("--requests", type=int, default=256, help="requests of the serve workload")
    ap.add_argument("--gen-len", type=int, default=256, help="generated tokens per request of the serve workload")
    ap.add_argument("--token-budget", type=int, default=8192, help="tokens per step of the serve workload")
    ap.add_argument("--prompt-min", type=int, default=128, help="shortest prompt of the serve workload")
    ap.add_argument("--prompt-max", type=int, default=2048, help="longest prompt of the serve workload")
    ap.add_argument("--max-seqs", type=int, default=256, help="most requests in one step of the serve workload")
    ap.add_argument("--emit-kernels", metavar="CSV", default=None,
                    help="measure nothing; read the *_kernel_trace.csv that `rocprofv3 --kernel-trace --output-format csv` "
                         "wrote for a run with the same options and print a table of the step's kernels: time, bytes, "
                         "operations, share of the HBM and MFMA peaks")
    ap.add_argument("--step-ms", type=float, default=None,
                    help="with --emit-kernels: the step's time on the clock (ms_per_step of the measured line), to "
                         "show the time between kernels")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    if args.prompt_len + args.warmup + args.steps + 16 > args.context:
        print(f"bench.py: prompt {args.prompt_len} + {args.warmup + args.steps} steps exceed the context {args.context}")
        return 2

    import torch
    if args.only == "floor":
        return measure_floor(args)
    shape = SHAPES[args.shape]
    layers_full = shape["num_hidden_layers"]
    layers = args.layers or layers_full
    if args.only == "serve":
        if not 1 <= args.prompt_min <= args.prompt_max or args.prompt_max + args.gen_len > args.context:
            print(f"bench.py: prompts of {args.prompt_min}..{args.prompt_max} tokens + {args.gen_len} generated "
                  f"do not fit the context {args.context}")
            return 2
        live = min(args.max_seqs, args.requests)
        pages = live * (-(-(args.prompt_max + args.gen_len) // args.block_size) + 1) + 64
        llm, cfg = build_llm(args, shape, layers, max_seqs=live, token_budget=args.token_budget, num_pages=pages)
        dt, gen, prompt, steps, preempted = measure_serve(llm, cfg.vocab_size, args.requests, args.gen_len, args.seed,
                                                          args.prompt_min, args.prompt_max)
        print(json.dumps({
            "metric": "generated tok/s, continuous batching (%d requests, prompts %d..%d, %d generated each)"
                      % (args.requests, args.prompt_min, args.prompt_max, args.gen_len),
            "value": round(gen / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": 0,
            "ms_per_step": round(dt / steps * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
            "config": {"model": f"qwen3-{args.shape}-shape-random", "layers": layers, "layers_full": layers_full,
                       "requests": args.requests, "gen_len": args.gen_len, "token_budget": args.token_budget,
                       "max_seqs": live, "prompt_min": args.prompt_min, "prompt_max": args.prompt_max,
                       "seq_len": args.context, "block_size": args.block_size, "graph": not args.no_graph,
                       "scheduler_steps": args.scheduler_steps, "launch_ahead": bool(llm.config.launch_ahead),
                       "parallelism": "single-gpu"},
            "seconds": round(dt, 3), "prompt_tokens": prompt, "generated_tokens": gen,
            "total_tok_s": round((gen + prompt) / dt, 1), "preemptions": preempted}))
        return 0
    if args.only == "graphs":
        live = args.max_seqs
        llm, cfg = build_llm(args, shape, layers, max_seqs=live, num_pages=live + 64)
        ex = llm.executor
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        t0 = time.perf_counter()
        made = ex.capture_graphs()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        used = free0 - torch.cuda.mem_get_info()[0]
        print(json.dumps({"metric": "decode graphs recorded ahead of serving", "value": made, "unit": "graphs", "n_gpus": 1,
                          "seconds": round(dt, 2), "device_bytes": int(used), "ms_per_graph": round(dt / max(made, 1) * 1e3, 1),
                          "config": {"model": f"qwen3-{args.shape}-shape-random", "layers": layers, "max_seqs": live,
                                     "seq_len": args.context, "scheduler_steps": args.scheduler_steps,
                                     "block_size": args.block_size}}))
        return 0
    llm, cfg = build_llm(args, shape, layers)
    if args.emit_kernels:
        return emit_kernels(llm, cfg, args)
    nums = model_numbers(shape, layers)
    item = 2 if args.dtype == "bfloat16" else 4

    prefill = None
    if args.only in ("all", "prefill"):
        prefill_s = measure_prefill(llm, cfg.vocab_size, args.prefill_tokens, repeats=3, seed=args.seed)
        T = args.prefill_tokens
        attn_flops = layers * 2 * cfg.num_attention_heads * cfg.head_dim * T * T   # causal half of 4 H D T^2
        prefill_flops = 2 * T * nums["matrix_params"] + attn_flops + 2 * cfg.vocab_size * cfg.hidden_size
        prefill = {"value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 3),
                   "frac": round(prefill_flops / prefill_s / PEAK_FLOPS[args.dtype], 4)}

    tok_s = ms_step = roofline = None
    ran = regions = 0
    if args.only in ("all", "decode"):
        tok_s, ms_step, mean_ctx, ran, regions = measure_decode(llm, cfg.vocab_size, args.batch, args.prompt_len,
                                                                args.steps, args.warmup, args.seed)
        step_bytes = nums["step_params"] * item + args.batch * mean_ctx * nums["kv_bytes_per_token"] * item
        achieved = step_bytes / (ms_step * 1e-3) / 1e9
        roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": round(achieved / PEAK_HBM_GBS, 4)}

    points = {}
    if not args.no_points and args.only == "all":
        for b, key in ((1, "decode_b1"), (64, "decode_b64")):
            n = min(args.steps, 128)
            v = measure_decode(llm, cfg.vocab_size, b, args.prompt_len, n, min(args.warmup, 8), args.seed + b)[0]
            points[key] = round(v, 1)

    config = {"model": f"qwen3-{args.shape}-shape-random", "layers": layers, "layers_full": layers_full,
              "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
              "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
              "tied_head": cfg.tie_word_embeddings, "global_batch": args.batch, "seq_len": args.context,
              "prompt_len": args.prompt_len, "block_size": args.block_size, "graph": not args.no_graph,
              "scheduler_steps": args.scheduler_steps, "launch_ahead": bool(llm.config.launch_ahead),
              "parallelism": "single-gpu"}
    line = {"metric": "decode tok/s (batch %d, %d-token prompts)" % (args.batch, args.prompt_len),
            "value": round(tok_s, 1) if tok_s is not None else None, "unit": "tokens/s", "n_gpus": 1, "steps": ran if ran else args.steps, "warmup": args.warmup,
            "ms_per_step": round(ms_step, 4) if ms_step is not None else None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic", "config": config,
            "timed_regions": regions, "prefill": prefill, "roofline": roofline, "points": points}
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())

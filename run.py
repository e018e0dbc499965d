#!/usr/bin/env python3
"""Generates completions for a few prompts, in the manner of the reference's ``run.py``.

Reference: run.py:11-46 — four fixed questions go through the model's chat template
(``enable_thinking=True``), ``Engine.generate`` runs them with ``max_tokens=1024`` and the
prompts and completions are printed. The reference takes no options and reads
``~/huggingface/Qwen3-0.6B/``; that is the default here too, and every setting is an option.
A model folder without a tokenizer (a random-weights model) is driven with ``--prompt-ids``.

    python run.py --model ~/huggingface/Qwen3-0.6B/
    python run.py --random-model 0.6b --seed 0 --prompt-ids 1,2,3 --prompt-ids 7,8 --max-tokens 16
"""
import argparse
import logging
import os
import sys
import tempfile

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

DEFAULT_PROMPTS = [
    "What is the meaning of life?",
    "What is the difference between GPT and ChatGPT?",
    "How do I get started with LLMs?",
    "How to build a LLM inference engine from scratch?",
]


def add_engine_options(ap: argparse.ArgumentParser) -> None:
    ap.add_argument("--model", default=os.path.expanduser("~/huggingface/Qwen3-0.6B/"),
                    help="folder with config.json and safetensors (and a tokenizer for text prompts)")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default=None, help="default: the model's own")
    ap.add_argument("--max-model-len", type=int, default=4096)
    ap.add_argument("--max-num-batched-tokens", type=int, default=16384)
    ap.add_argument("--max-num-batched-seqs", type=int, default=512)
    ap.add_argument("--prefill-chunk", type=int, default=None)
    ap.add_argument("--kv-cache-block-size", type=int, default=16)
    ap.add_argument("--kv-cache-num-blocks", type=int, default=None)
    ap.add_argument("--gpu-memory-utilization", type=float, default=0.5)
    ap.add_argument("--enable-prefix-caching", action="store_true")
    ap.add_argument("--no-cuda-graph", action="store_true", help="run decode steps eagerly (no HIP graph)")
    ap.add_argument("--num-scheduler-steps", type=int, default=4,
                    help="decode-only steps run this many times in a row on the device (1: one token per step)")
    ap.add_argument("--no-launch-ahead", action="store_true",
                    help="read the tokens of a row of decode steps before the next row is launched")
    ap.add_argument("--capture-graphs-at-start", action="store_true",
                    help="record every decode graph before the first request instead of at its first use")
    ap.add_argument("--debug-poison-pages", action="store_true",
                    help="debugging: fill cache pages with NaN whenever they change hands")
    ap.add_argument("--seed", type=int, default=0)


def add_sampling_options(ap: argparse.ArgumentParser) -> None:
    ap.add_argument("--max-tokens", type=int, default=1024)
    ap.add_argument("--temperature", type=float, default=1.0)
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--ignore-eos", action="store_true")
    ap.add_argument("--sampling-seed", type=int, default=None)


def engine_config_from(args):
    from minivllm_amd import EngineConfig
    return EngineConfig(model=args.model, dtype=args.dtype, max_model_len=args.max_model_len,
                        max_num_batched_tokens=args.max_num_batched_tokens,
                        max_num_batched_seqs=args.max_num_batched_seqs, prefill_chunk=args.prefill_chunk,
                        kv_cache_block_size=args.kv_cache_block_size, kv_cache_num_blocks=args.kv_cache_num_blocks,
                        gpu_memory_utilization=args.gpu_memory_utilization,
                        enable_prefix_caching=args.enable_prefix_caching, use_cuda_graph=not args.no_cuda_graph,
                        num_scheduler_steps=args.num_scheduler_steps, launch_ahead=not args.no_launch_ahead,
                        capture_graphs_at_start=args.capture_graphs_at_start,
                        debug_poison_pages=args.debug_poison_pages, seed=args.seed)


def sampling_params_from(args):
    from minivllm_amd import SamplingParams
    return SamplingParams(temperature=args.temperature, max_tokens=args.max_tokens, ignore_eos=args.ignore_eos,
                          top_k=args.top_k, top_p=args.top_p, seed=args.sampling_seed)


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    add_engine_options(ap)
    add_sampling_options(ap)
    ap.add_argument("--prompt", action="append", default=None, help="a text prompt (repeatable)")
    ap.add_argument("--prompt-ids", action="append", default=None, help="a prompt as comma-separated token ids")
    ap.add_argument("--no-chat-template", action="store_true", help="encode text prompts as they are")
    ap.add_argument("--random-model", default=None, metavar="SHAPE",
                    help="write a random-weights model of this named shape (tiny, 0.6b, ...) to a temporary folder "
                         "and run it; the architecture is the one the shape's config names")
    args = ap.parse_args()
    logging.basicConfig(format="%(asctime)s: %(message)s", level=logging.INFO, datefmt="%m-%d-%Y %H:%M:%S")

    from minivllm_amd import LLM
    tmp = None
    if args.random_model:
        from minivllm_amd.config import named_shape, named_shapes
        from minivllm_amd.models import config_from_dict
        from minivllm_amd.weights import write_model_folder
        if args.random_model not in named_shapes():
            ap.error(f"--random-model: unknown shape {args.random_model!r} (known: {sorted(named_shapes())})")
        arch, cfg = config_from_dict(named_shape(args.random_model))       # the registry picks the architecture
        tmp = tempfile.TemporaryDirectory()
        args.model = write_model_folder(os.path.join(tmp.name, "model"), cfg, seed=args.seed)
        logging.info("wrote a random %s model to %s", args.random_model, args.model)

    llm = LLM(config=engine_config_from(args))
    sp = sampling_params_from(args)
    if args.prompt_ids:
        prompts = [[int(t) for t in p.split(",") if t.strip()] for p in args.prompt_ids]
    else:
        if llm.tokenizer is None:
            print("this model folder has no tokenizer: give prompts with --prompt-ids", file=sys.stderr)
            return 2
        texts = args.prompt or DEFAULT_PROMPTS
        if args.no_chat_template:
            prompts = [llm.tokenizer.encode(t) for t in texts]
        else:
            prompts = [llm.tokenizer.apply_chat_template([{"role": "user", "content": t}], tokenize=True,
                                                         add_generation_prompt=True, enable_thinking=True)
                       for t in texts]
    outputs = llm.generate(prompts, sp)
    for out in outputs:
        print("=" * 50)
        print("Prompt:\n", out.prompt if out.prompt is not None else out.prompt_token_ids)
        print("Completion:\n", out.text if out.text is not None else out.token_ids)
    s = llm.metrics.stats()
    logging.info("prefill %.0f tok/s, decode %.0f tok/s, %d requests, %d steps, %d preemptions",
                 s.prefill_throughput, s.decode_throughput, s.finished_requests, s.steps, s.preemptions)
    if tmp is not None:
        tmp.cleanup()
    return 0


if __name__ == "__main__":
    sys.exit(main())

"""The command lines: the reference's option names and chat commands."""
import argparse
import subprocess
import sys
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_run_options_map_to_the_engine_config():
    import run
    ap = argparse.ArgumentParser()
    run.add_engine_options(ap)
    run.add_sampling_options(ap)
    args = ap.parse_args(["--model", "/m", "--max-num-batched-tokens", "2048", "--max-num-batched-seqs", "128",
                          "--gpu-memory-utilization", "0.4", "--kv-cache-block-size", "32", "--no-cuda-graph",
                          "--temperature", "0.5", "--top-k", "7", "--top-p", "0.9", "--max-tokens", "33",
                          "--ignore-eos", "--prefill-chunk", "256", "--enable-prefix-caching"])
    ec = run.engine_config_from(args)
    assert (ec.model, ec.max_num_batched_tokens, ec.max_num_batched_seqs) == ("/m", 2048, 128)
    assert ec.gpu_memory_utilization == 0.4 and ec.kv_cache_block_size == 32 and ec.use_cuda_graph is False
    assert ec.prefill_chunk == 256 and ec.enable_prefix_caching is True
    assert ec.launch_ahead is True
    assert run.engine_config_from(ap.parse_args(["--model", "/m", "--no-launch-ahead"])).launch_ahead is False
    sp = run.sampling_params_from(args)
    assert (sp.temperature, sp.top_k, sp.top_p, sp.max_tokens, sp.ignore_eos) == (0.5, 7, 0.9, 33, True)
    # the reference's defaults (run.py:12,36)
    d = ap.parse_args([])
    assert d.model.endswith("huggingface/Qwen3-0.6B/") and d.max_tokens == 1024


def test_chat_requires_model():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "chat.py")], capture_output=True, text=True)
    assert proc.returncode != 0 and "--model" in proc.stderr


def test_chat_commands(capsys):
    import chat
    from minivllm_amd import SamplingParams
    s = chat.ChatSession(llm=None, system_prompt="Be brief.", sampling_params=SamplingParams())
    assert s.history == [{"role": "system", "content": "Be brief."}]
    s.run_command("/maxtokens", ["77"]); assert s.sampling_params.max_tokens == 77
    s.run_command("/maxtokens", ["x"]); assert s.sampling_params.max_tokens == 77
    s.run_command("/top-k", ["5"]); assert s.sampling_params.top_k == 5
    s.run_command("/top-p", ["0.8"]); assert s.sampling_params.top_p == 0.8
    s.run_command("/top-p", ["7"]); assert s.sampling_params.top_p == 0.8
    s.run_command("/temperature", ["0.3"]); assert s.sampling_params.temperature == 0.3
    s.history.append({"role": "user", "content": "hi"})
    s.run_command("/system", ["You", "are", "terse."])
    assert s.system_prompt == "You are terse." and s.history == [{"role": "system", "content": "You are terse."}]
    s.history.append({"role": "user", "content": "hi"})
    s.run_command("/reset", []); assert len(s.history) == 1
    s.run_command("/clear", []); assert s.history == []
    s.run_command("/settings", []); s.run_command("/help", []); s.run_command("/history", []); s.run_command("/nope", [])
    out = capsys.readouterr().out
    for needle in ("Max Tokens: 77", "/temperature <float>", "No conversation history", "Unknown command: /nope"):
        assert needle in out


def test_bench_refuses_more_than_one_gpu():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert proc.returncode == 2 and "one GPU" in proc.stdout
    assert len(proc.stdout.strip().splitlines()) == 1

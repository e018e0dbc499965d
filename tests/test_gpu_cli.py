"""The command lines on the GPU: ``run.py`` from a model folder to printed tokens, as a program, and
the chat session's streaming loop with a stand-in tokenizer (a random-weights model has none).

Reference: run.py:32-42 (generate, then print prompt and completion of every request) and
chat.py:163-181 (submit, step until the request has finished, yield the text of what each step
added)."""
import ast
import builtins
import os
import re
import subprocess
import sys

import numpy as np
import pytest
import torch

from helpers import TINY, make_weights, plain_logits, random_tokens, write_model_dir

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    cfg = TINY["A"]
    w = make_weights(cfg, seed=12, stored=torch.float32, qk_gain=1.5)
    return cfg, w, write_model_dir(str(tmp_path_factory.mktemp("cli") / "A"), cfg, w)


def greedy_continuation(cfg, w, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(np.argmax(plain_logits(cfg, w, toks)[-1])))
    return toks[len(prompt):]


def test_run_py_from_a_model_folder_to_printed_tokens(model):
    cfg, w, path = model
    prompts = [random_tokens(cfg, n, seed=40 + n) for n in (9, 3)]
    cmd = [sys.executable, os.path.join(ROOT, "run.py"), "--model", path, "--dtype", "float32", "--temperature", "0",
           "--max-tokens", "6", "--ignore-eos", "--max-model-len", "64", "--kv-cache-num-blocks", "16",
           "--max-num-batched-tokens", "64", "--max-num-batched-seqs", "4"]
    for p in prompts:
        cmd += ["--prompt-ids", ",".join(map(str, p))]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    # the reference's layout: a rule, "Prompt:", the prompt, "Completion:", the completion (run.py:38-42)
    blocks = proc.stdout.split("=" * 50)[1:]
    assert len(blocks) == 2
    for block, prompt in zip(blocks, prompts):
        m = re.search(r"Prompt:\s*(\[.*?\])\s*Completion:\s*(\[.*?\])", block, re.S)
        assert m, block
        assert ast.literal_eval(m.group(1)) == prompt
        assert ast.literal_eval(m.group(2)) == greedy_continuation(cfg, w, prompt, 6)


def test_run_py_with_a_random_model(model):
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "run.py"), "--random-model", "tiny", "--seed", "3",
                           "--prompt-ids", "5,17,3", "--prompt-ids", "200", "--max-tokens", "5", "--temperature", "0",
                           "--ignore-eos", "--max-model-len", "64", "--kv-cache-num-blocks", "16",
                           "--max-num-batched-tokens", "64", "--max-num-batched-seqs", "4",
                           "--capture-graphs-at-start"], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-3000:]
    completions = re.findall(r"Completion:\s*(\[.*?\])", proc.stdout, re.S)
    assert len(completions) == 2 and all(len(ast.literal_eval(c)) == 5 for c in completions)
    assert "recorded" in proc.stderr and "decode graphs ahead of serving" in proc.stderr


class StubTokenizer:
    """Words are token ids written in letters: enough of a tokenizer for the chat loop."""

    def __init__(self, vocab):
        self.vocab = vocab
        self.templated = []

    def apply_chat_template(self, messages, tokenize=True, add_generation_prompt=True, enable_thinking=True):
        self.templated.append([dict(m) for m in messages])
        ids = []
        for m in messages:
            ids.append({"system": 1, "user": 2, "assistant": 3}[m["role"]])
            ids += [sum(map(ord, word)) % self.vocab for word in m["content"].split()]
        return ids + [3]

    def decode(self, ids, skip_special_tokens=True):
        return "".join(f" t{int(i)}" for i in ids)


def test_chat_session_streams_what_every_step_adds(model, monkeypatch, capsys):
    import chat
    from minivllm_amd import LLM, SamplingParams
    cfg, w, path = model
    llm = LLM(model=path, dtype="float32", kv_cache_num_blocks=32, max_model_len=128, max_num_batched_tokens=64,
              max_num_batched_seqs=4, num_scheduler_steps=4)
    llm.tokenizer = StubTokenizer(cfg["vocab_size"])
    session = chat.ChatSession(llm, system_prompt="Be brief.",
                               sampling_params=SamplingParams(temperature=0.0, max_tokens=11, ignore_eos=True))
    # the streaming loop by itself (chat.py:163-181): the pieces are the tokens in order, several per step
    # once the request decodes in rows of four steps
    prompt = session.build_model_input_tokens("hello there")
    assert prompt[:2] == [1, sum(map(ord, "Be")) % cfg["vocab_size"]] and prompt[-1] == 3
    pieces = list(session.generate(prompt))
    want = greedy_continuation(cfg, w, prompt, 11)
    assert "".join(pieces) == "".join(f" t{t}" for t in want)
    assert 1 < len(pieces) < 11 and any(p.count(" t") == 4 for p in pieces)
    llm.manager.check_invariants()
    assert all(p.num_free == p.num_pages for p in llm.manager.pools)

    # the whole loop: two turns, a command in between, then /exit; the second turn's prompt holds the first turn
    lines = iter(["hello there", "/maxtokens 5", "and again", "/exit"])
    monkeypatch.setattr(builtins, "input", lambda prompt="": next(lines))
    session.start()
    out = capsys.readouterr().out
    assert out.count("Assistant: ") == 2 and "[Max tokens set to 5]" in out and "Goodbye!" in out
    first = "".join(f" t{t}" for t in want)
    assert [m["role"] for m in session.history] == ["system", "user", "assistant", "user", "assistant"]
    assert session.history[2]["content"] == first.strip() and first in out
    second_prompt = llm.tokenizer.templated[-1]
    assert [m["content"] for m in second_prompt] == ["Be brief.", "hello there", first.strip(), "and again"]
    assert len(session.history[4]["content"].split()) == 5

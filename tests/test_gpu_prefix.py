"""Prefix reuse against the plain model: requests that share their first 16 tokens, cache pages of
8, prompt portions of 7, on a pool so small that the shared pages are given back, taken up again
by a later request and finally overwritten; every (request, position) row is compared with the
plain model, in float32 and in bfloat16. Then the same through the entry point: seeded drawing at
temperature 0.8, requests arriving over the steps, a forced preemption (the victim is admitted
again through the prefix lookup), rows of decode steps launched ahead.

Reference: minivllm/kvcache/block_manager.py:54-87 (a hit needs an equal hash and equal tokens; a
hit on a page in use adds a holder, one on a page given back takes that page up again;
after the first miss everything misses) and its test tests/test_block_manager.py:19-28."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import trace_tools
from helpers import (TINY, TOL_F32, bf16_tolerance, make_weights, plain_logits, plain_logits_bf16, random_tokens,
                     rel_err, write_model_dir)
from test_gpu_generate import check_against_plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PAGE, PORTION, SHARED = 8, 7, 16


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    cfg = TINY["B0"]
    w = make_weights(cfg, seed=1, stored=torch.float32, qk_gain=2.0)
    path = write_model_dir(str(tmp_path_factory.mktemp("prefix") / "B0"), cfg, w)
    shared = random_tokens(cfg, SHARED, seed=50)
    reqs = {
        "a": shared + random_tokens(cfg, 20, seed=51),            # computes the shared pages, then ends
        "b": shared + random_tokens(cfg, 22, seed=52),            # takes them up again from the free pages
        "c": shared + random_tokens(cfg, 25, seed=53),            # shares them with b while b lives
        "f1": random_tokens(cfg, 64, seed=54),                    # two requests that fill the whole pool:
        "f2": random_tokens(cfg, 64, seed=55),                    # the shared pages are overwritten
        "d": shared + random_tokens(cfg, 9, seed=56),             # finds nothing and computes them again
        "e": shared[:8] + random_tokens(cfg, 30, seed=57),        # shares d's first page only
    }
    want = {rid: plain_logits(cfg, w, t) for rid, t in reqs.items()}
    emulated = {rid: plain_logits_bf16(cfg, w, t) for rid, t in reqs.items()}
    bf16_err = max(rel_err(emulated[r][p], want[r][p]) for r, t in reqs.items() for p in range(len(t)))
    return cfg, w, path, reqs, want, bf16_err


def prefix_trace(reqs):
    """Steps in which a request's first entry holds its known prefix and one portion (logits
    wanted for the portion only, so the prefix may come from the cache); then portions of 7."""
    known = {"a": 0, "b": SHARED, "c": SHARED, "f1": 0, "f2": 0, "d": SHARED, "e": 8}
    steps = []
    done = {rid: 0 for rid in reqs}

    def entry(rid):
        toks, p = reqs[rid], done[rid]
        n = min(PORTION, len(toks) - p - (known[rid] if p == 0 else 0))
        first = known[rid] if p == 0 else 0
        if len(toks) - (p + first + n) == 1:
            n += 1
        chunk = toks[p:p + first + n]
        done[rid] = p + len(chunk)
        return {"id": rid, "tokens": chunk, "want": list(range(first, len(chunk)))}

    def run(live, until_done):
        while any(done[r] < len(reqs[r]) for r in until_done):
            entries = [entry(r) for r in live if done[r] < len(reqs[r])]
            ended = [e["id"] for e in entries if done[e["id"]] == len(reqs[e["id"]])]
            steps.append({"step": len(steps), "entries": entries, "end": ended})

    run(["a"], ["a"])                     # a alone, then it ends: its pages are free but keep their content
    steps.append({"step": len(steps), "entries": [entry("b")], "end": []})     # b takes two of them up again
    run(["b", "c"], ["b", "c"])           # c shares them with b, which is still running
    run(["f1", "f2"], ["f1", "f2"])       # the pool is filled: nothing of the shared prefix is left
    run(["d"], ["d"])
    run(["e"], ["e"])
    return steps, known


def check_rows(got, reqs, want, known, tol):
    assert set(got) == {(r, p) for r, t in reqs.items() for p in range(known[r], len(t))}
    return max(rel_err(row, want[rid][pos]) for (rid, pos), row in got.items())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefix_hits_give_the_plain_models_logits(model, dtype):
    from minivllm_amd.engine.trace import TraceRunner
    cfg, w, path, reqs, want, bf16_err = model
    steps, known = prefix_trace(reqs)
    tol = TOL_F32 if dtype == "float32" else bf16_tolerance(bf16_err)
    # the pool holds exactly the two fillers: 128 tokens = 16 pages
    assert trace_tools.max_live_tokens(steps) == 128
    runner = TraceRunner(path, dtype, 128, page_size=PAGE, enable_prefix_caching=True)
    assert runner.manager.prefix_caching and runner.manager.pools[0].num_pages == 16
    reused = {}
    real_admit = runner.manager.admit

    def admit(rid, tokens=None):
        seq = real_admit(rid, tokens)
        reused[rid] = (seq.num_cached, [list(p) for p in seq.pages])
        return seq

    runner.manager.admit = admit
    got = trace_tools.collect(steps, runner.run_step)
    worst = check_rows(got, reqs, want, known, tol)
    print(f"prefix reuse [{dtype}]: {len(got)} rows, worst relative error {worst:.3e} (allowed {tol:.3e}), "
          f"reused {({r: n for r, (n, _) in reused.items()})}")
    assert worst <= tol
    # what was reused, and from where: b revives a's two pages, c shares them while b holds them, the
    # fillers overwrite them so that d misses, e shares d's first page only
    assert {r: n for r, (n, _) in reused.items()} == {"a": 0, "b": 16, "c": 16, "f1": 0, "f2": 0, "d": 0, "e": 8}
    assert reused["b"][1] == reused["c"][1] and len(reused["b"][1][0]) == 2
    assert runner.num_reused_tokens == 40
    runner.manager.check_invariants()
    assert not runner.manager.seqs and all(p.num_free == p.num_pages for p in runner.manager.pools)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_wrong_page_in_a_hit_shows(model, dtype):
    """The check above is able to fail: when the block tables of b and c name the first shared page
    in the place of the second as well, their rows are far from the plain model's. (Two shared pages
    in the wrong order would not show: attention does not care where a key it sees is stored.)"""
    from minivllm_amd.engine.trace import TraceRunner
    cfg, w, path, reqs, want, bf16_err = model
    steps, known = prefix_trace(reqs)
    tol = TOL_F32 if dtype == "float32" else bf16_tolerance(bf16_err)
    runner = TraceRunner(path, dtype, 128, page_size=PAGE, enable_prefix_caching=True)
    real_step = runner.executor.step
    slots = {}

    def step(seqs):
        for s in seqs:
            if s.state_slot in slots:
                s.block_tables = [[t[0], t[0]] + list(t[2:]) for t in s.block_tables]
        return real_step(seqs)

    real_admit = runner.manager.admit

    def admit(rid, tokens=None):
        seq = real_admit(rid, tokens)
        slots.pop(seq.state_slot, None)
        if seq.num_cached == 16:
            slots[seq.state_slot] = rid
        return seq

    runner.executor.step = step
    runner.manager.admit = admit
    got = trace_tools.collect(steps, runner.run_step)
    bad = max(rel_err(row, want[rid][pos]) for (rid, pos), row in got.items() if rid in ("b", "c"))
    good = max(rel_err(row, want[rid][pos]) for (rid, pos), row in got.items() if rid not in ("b", "c"))
    print(f"a wrong page in the hits [{dtype}]: b and c {bad:.3e}, the others {good:.3e} (allowed {tol:.3e})")
    assert bad > 3 * tol and good <= tol


def test_trace_run_program_with_prefix_caching(model, tmp_path):
    cfg, w, path, reqs, want, bf16_err = model
    steps, known = prefix_trace(reqs)
    out = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", path, "--dtype", "float32",
         "--out", str(out), "--max-tokens", "128", "--block-size", str(PAGE), "--enable-prefix-caching"],
        input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-4000:]

    def read(step):
        n = sum(len(e["want"]) for e in step["entries"])
        return np.fromfile(out / f"{step['step']}.f32", dtype="<f4").reshape(n, cfg["vocab_size"]) if n else None

    got = trace_tools.collect(steps, read)
    assert check_rows(got, reqs, want, known, TOL_F32) <= TOL_F32


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generation_with_prefix_reuse_preemption_and_launch_ahead(model, dtype):
    """The workload of the second tiny configuration: six prompts of 1 to 40 tokens arriving over
    the steps, two sharing their first 16 tokens, pages of 8, portions of 7, temperature 0.8 with
    seeds, 12 new tokens each; here on so few pages that a request is preempted and admitted again
    through the prefix lookup, with rows of four decode steps launched ahead. Every drawn token is
    the plain model's draw at its position."""
    from minivllm_amd import LLM, SamplingParams
    cfg, w, path, reqs, want, bf16_err = model
    shared = reqs["a"][:SHARED]
    lengths = [1, 40, 9, 23, 31]
    prompts = [random_tokens(cfg, n, seed=600 + n) for n in lengths]
    prompts[1] = shared + prompts[1][SHARED:]
    prompts[4] = shared + prompts[4][SHARED:]
    prompts.append(shared + random_tokens(cfg, 5, seed=77))          # a third one, arriving last
    # 12 new tokens each, as the workload says; the two that arrive last go on to 40, so that they
    # end up decoding alone, in rows of four steps with the next row launched ahead
    params = [SamplingParams(temperature=0.8, max_tokens=12 if i < 4 else 40, ignore_eos=True, seed=2000 + i)
              for i in range(len(prompts))]
    llm = LLM(model=path, dtype=dtype, kv_cache_block_size=PAGE, kv_cache_num_blocks=15, max_model_len=80,
              max_num_batched_tokens=24, max_num_batched_seqs=4, prefill_chunk=PORTION, seed=3,
              enable_prefix_caching=True, num_scheduler_steps=4, launch_ahead=True)
    assert llm.manager.prefix_caching
    cached, preempted, after_preemption = {}, [], {}
    real_admit, real_preempt = llm.manager.admit, llm.scheduler.preempt

    def admit(rid, tokens=None):
        seq = real_admit(rid, tokens)
        cached.setdefault(rid, []).append(seq.num_cached)
        if rid in preempted:
            after_preemption[rid] = max(after_preemption.get(rid, 0), seq.num_cached)
        return seq

    def preempt(req):
        preempted.append(req.id)
        return real_preempt(req)

    llm.manager.admit, llm.scheduler.preempt = admit, preempt
    reqs_in, pending, launched = [], list(zip(prompts, params)), 0
    while pending or llm.has_unfinished():
        if pending:
            p, sp = pending.pop(0)
            reqs_in.append(llm.submit(p, sp))
        llm.step()
        launched += llm._in_flight is not None
    llm.drain()
    outs = [llm._output(r) for r in reqs_in]
    assert [len(o.token_ids) for o in outs] == [sp.max_tokens for sp in params]
    check_against_plain(cfg, w, outs, params, dtype, seeds=[2000 + i for i in range(len(prompts))])
    first = reqs_in[0].id
    print(f"prefix reuse through the entry point [{dtype}]: preempted {[r - first for r in preempted]}, found again "
          f"{({r - first: n for r, n in after_preemption.items()})}, rows launched ahead {launched}, cached tokens at "
          f"admission {({r - first: v for r, v in cached.items()})}")
    assert preempted, "the pool was not tight enough to preempt"
    assert cached[reqs_in[4].id][0] == SHARED and cached[reqs_in[5].id][0] == SHARED      # the shared prefix
    assert any(n > 0 for n in after_preemption.values()), \
        "no preempted request found pages of its own when it was admitted again"
    assert launched > 0, "no row of decode steps was launched ahead"
    llm.manager.check_invariants()
    assert all(p.num_free == p.num_pages for p in llm.manager.pools)
    # the same requests without prefix reuse on a roomy pool give the same tokens in float32
    if dtype == "float32":
        roomy = LLM(model=path, dtype=dtype, kv_cache_block_size=PAGE, kv_cache_num_blocks=64, max_model_len=80,
                    max_num_batched_tokens=24, max_num_batched_seqs=4, prefill_chunk=PORTION, seed=3)
        again = roomy.generate(prompts, params, use_tqdm=False)
        assert [o.token_ids for o in again] == [o.token_ids for o in outs]

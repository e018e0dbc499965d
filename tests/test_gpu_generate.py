"""Generation through the Python entry point against the plain model: greedy and seeded
temperature sampling, chunked prompts, few pages (preemption), prefix reuse, graphs."""
import numpy as np
import pytest
import torch

from helpers import (TINY, TOL_F32, bf16_tolerance, make_weights, plain_logits, plain_logits_bf16, random_tokens,
                     rel_err, write_model_dir)
from plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("gen_models")
    out = {}
    for name, stored in (("A", torch.float32), ("B", torch.bfloat16)):
        cfg = TINY[name]
        w = make_weights(cfg, seed=40 + ord(name), stored=stored, qk_gain=1.5)
        out[name] = (cfg, w, write_model_dir(str(tmp / name), cfg, w))
    return out


def check_against_plain(cfg, w, outputs, params, dtype, seeds=None):
    """Every generated token must be the plain model's choice at its position, given the tokens
    before it, unless the plain model's first and second choice lie closer together than twice the
    error bound of a logit (then either may win). Returns (tokens decided by a clear margin, near ties)."""
    clear = near = 0
    for i, out in enumerate(outputs):
        seq = list(out.prompt_token_ids) + list(out.token_ids)
        logits = plain_logits(cfg, w, seq)
        tol = TOL_F32 if dtype == "float32" else bf16_tolerance(
            max(rel_err(plain_logits_bf16(cfg, w, seq)[p], logits[p]) for p in range(len(seq))))
        sp = params[i]
        for t, tok in enumerate(out.token_ids):
            row = logits[len(out.prompt_token_ids) + t - 1]
            slack = 2 * tol * float(np.abs(row).max()) / max(sp.temperature, 1.0 if sp.temperature == 0 else 1e-3)
            seed = 0 if seeds is None else seeds[i]
            want, score = plain.sample_token(row, sp.temperature, sp.top_k, sp.top_p, seed=seed, counter=t)
            if sp.temperature == 0:
                mine = row[tok]
            else:
                # the engine's filters see its own logits: a token within the slack of the kept
                # set's lowest member may be kept by the engine though the plain model drops it
                z = row.astype(np.float32) / np.float32(sp.temperature)
                kept = plain.kept_set(z, sp.top_k, sp.top_p)
                assert z[tok] >= z[kept].min() - slack, f"request {i} token {t}: {tok} is outside the kept set"
                u = plain.uniform23(seed, t, tok)
                mine = z[tok] - np.log(-np.log(u))
            assert mine >= score[want] - slack, \
                f"request {i} token {t}: engine drew {tok} (score {mine}), plain {want} (score {score[want]})"
            # a clear winner must be the engine's token too (a token that only the engine's filters kept,
            # within the slack of the kept set's edge, competes outside the plain model's kept set)
            if float(score[want]) - float(np.partition(score, -2)[-2]) > slack and np.isfinite(score[tok]):
                assert tok == want
                clear += 1
            else:
                near += 1
    return clear, near


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_tiny_a(models, dtype):
    from minivllm_amd import LLM, SamplingParams
    cfg, w, path = models["A"]
    llm = LLM(model=path, dtype=dtype, kv_cache_block_size=16, kv_cache_num_blocks=32, max_model_len=128,
              max_num_batched_tokens=64, max_num_batched_seqs=8)
    prompts = [random_tokens(cfg, n, seed=n) for n in (5, 17, 33, 1)]
    sp = SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True)
    outs = llm.generate(prompts, sp, use_tqdm=False)
    assert [o.prompt_token_ids for o in outs] == prompts
    assert all(len(o.token_ids) == 8 and o.finish_reason == "length" for o in outs)
    assert outs[0]["tokens"] == outs[0].token_ids          # the reference's record keys
    clear, near = check_against_plain(cfg, w, outs, [sp] * 4, dtype)
    print(f"greedy tiny A [{dtype}]: {clear} tokens decided by a clear margin, {near} near ties")
    assert clear > near                   # a tied head repeats its input by a wide margin: the check has teeth
    llm.manager.check_invariants()
    assert all(p.num_free == p.num_pages for p in llm.manager.pools)
    # the same prompts again, each alone: identical tokens whatever the batch was
    for p, o in zip(prompts, outs):
        alone = llm.generate([p], sp, use_tqdm=False)[0]
        if dtype == "float32":
            assert alone.token_ids == o.token_ids


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sampled_generation_tiny_b_chunked(models, dtype):
    """Block size 8, prompt portions of 7, requests arriving over the steps, temperature 0.8
    with seeds, top-k/top-p on some."""
    from minivllm_amd import LLM, SamplingParams
    cfg, w, path = models["B"]
    llm = LLM(model=path, dtype=dtype, kv_cache_block_size=8, kv_cache_num_blocks=40, max_model_len=96,
              max_num_batched_tokens=24, max_num_batched_seqs=4, prefill_chunk=7, seed=5)
    lengths = [1, 40, 9, 23, 16, 31]
    prompts = [random_tokens(cfg, n, seed=200 + n) for n in lengths]
    params = [SamplingParams(temperature=0.8, max_tokens=12, ignore_eos=True, seed=1000 + i,
                             top_k=(20 if i % 3 == 1 else 0), top_p=(0.9 if i % 3 == 2 else 1.0))
              for i in range(len(prompts))]
    reqs = []
    pending = list(zip(prompts, params))
    while pending or llm.has_unfinished():
        if pending:                                    # one new request per step
            p, sp = pending.pop(0)
            reqs.append(llm.submit(p, sp))
        llm.step()
    outs = [llm._output(r) for r in reqs]
    assert all(len(o.token_ids) == 12 for o in outs)
    check_against_plain(cfg, w, outs, params, dtype, seeds=[1000 + i for i in range(len(prompts))])
    # requests arrived while others ran: some steps held prompt portions beside decoded tokens, and no
    # portion was longer than the chunk
    assert llm.metrics.steps > len(prompts) + 12 and llm.scheduler.num_preemptions == 0
    # a request's draws do not depend on the batch: alone it gives the same tokens
    if dtype == "float32":
        for p, sp, o in zip(prompts, params, outs):
            assert llm.generate([p], sp, use_tqdm=False)[0].token_ids == o.token_ids


def test_preemption_gives_the_same_tokens(models):
    from minivllm_amd import LLM, SamplingParams
    cfg, w, path = models["A"]
    prompts = [random_tokens(cfg, n, seed=300 + n) for n in (30, 25, 20, 28, 12)]
    sp = SamplingParams(temperature=0.0, max_tokens=30, ignore_eos=True)
    roomy = LLM(model=path, dtype="float32", kv_cache_block_size=4, kv_cache_num_blocks=200, max_model_len=64,
                max_num_batched_tokens=48, max_num_batched_seqs=8)
    want = [o.token_ids for o in roomy.generate(prompts, sp, use_tqdm=False)]
    assert roomy.scheduler.num_preemptions == 0
    tight = LLM(model=path, dtype="float32", kv_cache_block_size=4, kv_cache_num_blocks=34, max_model_len=64,
                max_num_batched_tokens=48, max_num_batched_seqs=8)
    got = [o.token_ids for o in tight.generate(prompts, sp, use_tqdm=False)]
    assert tight.scheduler.num_preemptions > 0, "the pool was not tight enough to preempt"
    assert got == want
    tight.manager.check_invariants()


def test_prefix_reuse_gives_the_same_tokens(models):
    from minivllm_amd import LLM, SamplingParams
    cfg, w, path = models["A"]
    shared = random_tokens(cfg, 16, seed=1)
    prompts = [shared + random_tokens(cfg, n, seed=400 + n) for n in (3, 9)] + [shared]
    sp = SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True)
    plain_llm = LLM(model=path, dtype="float32", kv_cache_block_size=16, kv_cache_num_blocks=32, max_model_len=64)
    want = [o.token_ids for o in plain_llm.generate(prompts, sp, use_tqdm=False)]
    llm = LLM(model=path, dtype="float32", kv_cache_block_size=16, kv_cache_num_blocks=32, max_model_len=64,
              enable_prefix_caching=True)
    first = llm.generate(prompts[:1], sp, use_tqdm=False)
    rest = llm.generate(prompts[1:], sp, use_tqdm=False)
    assert [o.token_ids for o in first + rest] == want
    assert llm.manager.prefix_caching
    assert llm.metrics.prefill_tokens < plain_llm.metrics.prefill_tokens      # the shared page was not run again


def test_pool_sized_from_the_memory_left(models):
    """Without a page count the pool is what the memory share leaves after a dry step of a full
    token budget, never more than every request at full length can use; a share below what is
    already in use is refused with the numbers."""
    from minivllm_amd import LLM, SamplingParams
    cfg, w, path = models["B"]
    llm = LLM(model=path, dtype="bfloat16", kv_cache_block_size=8, max_model_len=96, max_num_batched_tokens=256,
              max_num_batched_seqs=6, gpu_memory_utilization=0.3)
    assert llm.executor.num_pages == 6 * 12 and llm.manager.pools[0].num_pages == 72
    assert all(t.shape[0] == 72 for pages in llm.executor.kv_pages.values() for t in pages.values())
    prompts = [random_tokens(cfg, n, seed=70 + n) for n in (30, 3, 11)]
    sp = SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True)
    outs = llm.generate(prompts, sp, use_tqdm=False)
    check_against_plain(cfg, w, outs, [sp] * 3, "bfloat16")
    with pytest.raises(RuntimeError, match="no memory left for the cache"):
        LLM(model=path, dtype="bfloat16", max_model_len=96, max_num_batched_tokens=64, max_num_batched_seqs=4,
            gpu_memory_utilization=1e-6)


def test_eos_and_max_model_len(models):
    from minivllm_amd import LLM, SamplingParams
    cfg, w, path = models["A"]
    llm = LLM(model=path, dtype="float32", kv_cache_num_blocks=16, max_model_len=40)
    p = random_tokens(cfg, 10, seed=9)
    free_run = llm.generate([p], SamplingParams(temperature=0.0, max_tokens=30, ignore_eos=True), use_tqdm=False)[0]
    assert len(free_run.token_ids) == 30 and free_run.finish_reason == "length"
    stop_at = free_run.token_ids[4]
    llm2 = LLM(model=path, dtype="float32", kv_cache_num_blocks=16, max_model_len=40, eos_token_ids=(stop_at,))
    stopped = llm2.generate([p], SamplingParams(temperature=0.0, max_tokens=30), use_tqdm=False)[0]
    n = free_run.token_ids.index(stop_at) + 1
    assert stopped.token_ids == free_run.token_ids[:n] and stopped.finish_reason == "stop"   # the end token stays
    with pytest.raises(ValueError, match="max_model_len"):
        llm.submit(random_tokens(cfg, 40, seed=1))
    with pytest.raises(ValueError, match="token ids"):
        llm.submit([cfg["vocab_size"]])


def test_graph_replays_match_eager(models):
    """A captured decode graph is replayed many times, with eager steps of other shapes and
    synchronisations in between; every replay must give what the eager step gives."""
    from minivllm_amd.engine.trace import TraceRunner
    cfg, w, path = models["B"]
    toks = {f"g{i}": random_tokens(cfg, 60 + 5 * i, seed=500 + i) for i in range(3)}
    for dtype in ("float32", "bfloat16"):
        runs = {}
        for use_graph in (False, True):
            r = TraceRunner(path, dtype, 512, page_size=16, use_graph=use_graph)
            rows = []
            for rid, t in toks.items():
                r.run_step({"step": 0, "entries": [{"id": rid, "tokens": t[:20], "want": []}], "end": []})
            for p in range(20, 60):
                out = r.run_step({"step": p, "entries": [{"id": rid, "tokens": [t[p]], "want": [0]}
                                                          for rid, t in toks.items()], "end": []})
                rows.append(out.copy())
                if p % 7 == 0:          # eager work of another shape between the replays
                    r.run_step({"step": 1000 + p, "entries": [{"id": f"x{p}", "tokens": toks["g0"][:p % 11 + 2],
                                                               "want": [0]}], "end": [f"x{p}"]})
                    torch.cuda.synchronize()
            runs[use_graph] = np.stack(rows)
        if dtype == "float32":
            assert np.array_equal(runs[True], runs[False])
        else:
            assert rel_err(runs[True], runs[False]) <= 2e-2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_in_a_row_give_the_same_tokens(models, dtype):
    """Decode-only steps run four times in a row on the device (one graph, tokens fed back on the
    device) or one by one: the same tokens, with greedy and seeded drawing, requests of different
    lengths, one arriving late, and an end token in the middle of a run."""
    from minivllm_amd import LLM, SamplingParams
    cfg, w, path = models["B"]
    prompts = [random_tokens(cfg, n, seed=70 + n) for n in (9, 30, 4, 17)]
    params = [SamplingParams(temperature=0.0, max_tokens=21, ignore_eos=True),
              SamplingParams(temperature=0.8, max_tokens=14, ignore_eos=True, seed=5),
              SamplingParams(temperature=1.0, top_k=20, top_p=0.9, max_tokens=9, ignore_eos=True, seed=6),
              SamplingParams(temperature=0.0, max_tokens=18, ignore_eos=True)]

    def run(steps, graph, eos=None):
        llm = LLM(model=path, dtype=dtype, kv_cache_block_size=8, kv_cache_num_blocks=48, max_model_len=96,
                  max_num_batched_tokens=64, max_num_batched_seqs=8, num_scheduler_steps=steps, use_cuda_graph=graph,
                  eos_token_ids=eos)
        sps = [SamplingParams(**{**p.__dict__, "ignore_eos": eos is None}) for p in params]
        reqs = [llm.submit(p, sp) for p, sp in zip(prompts[:3], sps[:3])]
        n, repeats = 0, []
        while llm.has_unfinished():
            st = llm.step()
            repeats.append(st.repeat)
            n += 1
            if n == 5:
                reqs.append(llm.submit(prompts[3], sps[3]))
        llm.manager.check_invariants()
        assert all(p.num_free == p.num_pages for p in llm.manager.pools)
        return [list(r.completion_tokens) for r in reqs], [r.finish_reason for r in reqs], repeats

    one, why_one, rep_one = run(1, True)
    assert set(rep_one) == {1}
    four, why_four, rep_four = run(4, True)
    assert max(rep_four) == 4
    host, _, rep_host = run(4, False)                  # the same schedule, run by run from the host
    assert max(rep_host) == 4
    assert four == one and why_four == why_one
    if dtype == "float32":                             # without graphs bfloat16 steps round differently
        assert host == one
    # an end token: what the device ran past it is dropped
    stop = one[0][6]
    cut, why_cut, _ = run(4, True, eos=(stop,))
    ref, why_ref, _ = run(1, True, eos=(stop,))
    assert cut == ref and why_cut == why_ref and "stop" in why_cut


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_launching_ahead_gives_the_same_tokens(models, dtype):
    """Rows of decode steps launched before the tokens of the running row are read: the same tokens
    as without, for greedy and drawn tokens, requests that end on an end token in the middle of a
    row (what ran on for them is dropped), different lengths, and a late arrival."""
    from minivllm_amd import LLM, SamplingParams
    cfg, w, path = models["B"]
    prompts = [random_tokens(cfg, n, seed=300 + n) for n in (5, 21, 40, 3, 17, 9)]
    params = [SamplingParams(temperature=0.0, max_tokens=37, ignore_eos=True),
              SamplingParams(temperature=0.8, top_k=20, max_tokens=50, ignore_eos=True, seed=11),
              SamplingParams(temperature=0.0, max_tokens=64),
              SamplingParams(temperature=1.0, top_p=0.9, max_tokens=29, seed=12),
              SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True),
              SamplingParams(temperature=0.7, max_tokens=45, seed=13)]

    def run(ahead, eos_ids):
        llm = LLM(model=path, dtype=dtype, kv_cache_block_size=8, kv_cache_num_blocks=64, max_model_len=128,
                  max_num_batched_tokens=64, max_num_batched_seqs=8, num_scheduler_steps=4, launch_ahead=ahead,
                  eos_token_ids=eos_ids, seed=5)
        reqs = [llm.submit(p, sp) for p, sp in zip(prompts[:5], params[:5])]
        steps = launched = 0
        while not llm.finished:
            llm.step()
            steps += 1
            launched += llm._in_flight is not None
            if steps == 7:
                reqs.append(llm.submit(prompts[5], params[5]))
        assert ahead == (launched > 0)
        llm.drain()                                   # a row that may still be in flight is waited for
        assert llm._in_flight is None
        llm.manager.check_invariants()
        assert all(p.num_free == p.num_pages for p in llm.manager.pools)
        return [list(r.completion_tokens) for r in reqs]

    never = (cfg["vocab_size"] - 1,)
    base = run(False, never)
    assert base == run(True, never)
    # an end token that the greedy request 2 meets in the middle of a row of four
    stop = base[2][13]
    ends_at = base[2].index(stop)
    off = run(False, (stop,))
    assert off == run(True, (stop,))
    assert off[2] == base[2][:ends_at + 1] and off[0] == base[0]      # request 0 ignores end tokens


def test_graphs_of_many_sequences_hold_library_products_and_no_memset_node(models, monkeypatch):
    """Decode steps of more than 64 sequences: their products go to the library, inside graphs too.
    Every recorded graph is looked at: it may hold no memset node (such nodes replay wrongly on this
    platform); replays must give what eager steps give."""
    from minivllm_amd.engine.trace import TraceRunner
    from minivllm_amd.kernels.library import KernelLibrary
    cfg, w, path = models["B"]
    S = 70
    toks = {f"s{i}": random_tokens(cfg, 12 + i % 5, seed=900 + i) for i in range(S)}
    recorded = {"library": 0}
    real_offer = KernelLibrary.offer

    def offer(self, name, *args):
        if name == "mv_gemm_lt" and torch.cuda.is_current_stream_capturing():
            recorded["library"] += 1
        return real_offer(self, name, *args)

    monkeypatch.setattr(KernelLibrary, "offer", offer)
    runs = {}
    for use_graph in (False, True):
        r = TraceRunner(path, "bfloat16", 64 * S, page_size=16, use_graph=use_graph, max_live=128)
        for rid, t in toks.items():
            r.run_step({"step": 0, "entries": [{"id": rid, "tokens": t[:8], "want": []}], "end": []})
        rows = []
        for p in range(8, 12):
            out = r.run_step({"step": p, "entries": [{"id": rid, "tokens": [t[p]], "want": [0]}
                                                      for rid, t in toks.items()], "end": []})
            rows.append(out.copy())
            torch.cuda.synchronize()
        runs[use_graph] = np.stack(rows)
        if use_graph:
            census = dict(r.executor.graph_census)
        del r
    assert rel_err(runs[True], runs[False]) <= 2e-2
    assert recorded["library"] > 0, "no library product was recorded into the graph"
    assert census and all(c["memset"] == 0 and c["kernel"] > 0 for c in census.values()), census
    print(f"graphs of {S} sequences: {recorded['library']} library products recorded, nodes {census}")


def test_a_graph_with_a_memset_node_is_recorded_again_without_library_products(models, monkeypatch):
    """Should a library product leave a memset node in a graph, the graph is thrown away and recorded
    again with the engine's own products only (after one eager run of them, outside any capture). No
    library product has ever done so here, so the census is made to report one on the first look:
    the second recording must hold no library product and replay to the logits of eager steps."""
    from minivllm_amd.engine.trace import TraceRunner
    from minivllm_amd.kernels.library import KernelLibrary
    from minivllm_amd.kernels.ops import Ops
    cfg, w, path = models["B"]
    S = 70
    toks = {f"s{i}": random_tokens(cfg, 12 + i % 5, seed=300 + i) for i in range(S)}
    looks, in_capture = {"n": 0}, {"library": 0}
    real_census, real_offer = Ops.graph_census, KernelLibrary.offer

    def census(self, raw_graph):
        counts = real_census(self, raw_graph)
        looks["n"] += 1
        if looks["n"] == 1:
            counts = dict(counts, memset=1)
        return counts

    def offer(self, name, *args):
        if name == "mv_gemm_lt" and torch.cuda.is_current_stream_capturing():
            in_capture["library"] += 1
        return real_offer(self, name, *args)

    runs = {}
    for use_graph in (False, True):
        if use_graph:
            monkeypatch.setattr(Ops, "graph_census", census)
            monkeypatch.setattr(KernelLibrary, "offer", offer)
        r = TraceRunner(path, "bfloat16", 64 * S, page_size=16, use_graph=use_graph, max_live=128)
        r.executor.config.prompt_graph_max_tokens = 0          # the decode graph is the first one recorded
        for rid, t in toks.items():
            r.run_step({"step": 0, "entries": [{"id": rid, "tokens": t[:8], "want": []}], "end": []})
        rows = []
        for p in range(8, 11):
            out = r.run_step({"step": p, "entries": [{"id": rid, "tokens": [t[p]], "want": [0]}
                                                      for rid, t in toks.items()], "end": []})
            rows.append(out.copy())
            torch.cuda.synchronize()
        runs[use_graph] = np.stack(rows)
        if use_graph:
            assert looks["n"] == 2 and r.executor.graph_census[(80, 1024)]["memset"] == 0
            first_pass = in_capture["library"]
            assert first_pass > 0
        del r
    assert rel_err(runs[True], runs[False]) <= 2e-2
    # nothing of the library's went into the second recording (the counter saw the first pass only)
    assert in_capture["library"] == first_pass


def test_graphs_recorded_when_the_engine_starts(models):
    """With ``capture_graphs_at_start`` every decode graph the configuration can ask for exists before
    the first request; serving then records nothing, and gives the tokens it gives without."""
    from minivllm_amd import LLM, SamplingParams
    cfg, w, path = models["B"]
    prompts = [random_tokens(cfg, n, seed=800 + n) for n in (9, 30, 4, 17, 22)]
    params = [SamplingParams(temperature=0.0 if i % 2 else 0.8, max_tokens=15 + i, ignore_eos=True, seed=i)
              for i in range(len(prompts))]
    opts = dict(model=path, dtype="bfloat16", kv_cache_block_size=8, kv_cache_num_blocks=64, max_model_len=96,
                max_num_batched_tokens=64, max_num_batched_seqs=6, num_scheduler_steps=4)
    early = LLM(capture_graphs_at_start=True, **opts)
    ex = early.executor
    # buckets 1, 2, 4, 8 (the first that holds 6), one context cap (max_model_len), single steps and whole rows of 4
    assert sorted(ex._graphs) == [(1, 96), (2, 96), (4, 96), (8, 96)]
    assert sorted(ex._repeat_graphs) == [(b, 96, 4) for b in (1, 2, 4, 8)]   # a row is whole or one step
    assert all(c["memset"] == 0 for c in ex.graph_census.values())
    before = (sorted(ex._graphs), sorted(ex._repeat_graphs), {k: id(v[0]) for k, v in ex._repeat_graphs.items()})
    got = [o.token_ids for o in early.generate(prompts, params, use_tqdm=False)]
    # nothing was recorded while serving
    assert (sorted(ex._graphs), sorted(ex._repeat_graphs), {k: id(v[0]) for k, v in ex._repeat_graphs.items()}) == before
    late = LLM(**opts)
    assert not late.executor._graphs
    assert [o.token_ids for o in late.generate(prompts, params, use_tqdm=False)] == got


def test_engine_starts_with_one_sequence_per_step_and_default_budgets(models):
    """max_num_batched_seqs = 1 with the default token budget (16384) and max_model_len (4096 > the
    model's 2048 here, so 2048): the dry step that sizes the cache holds no more tokens of a request
    than a request may have."""
    from minivllm_amd import LLM, SamplingParams
    cfg, w, path = models["B"]
    llm = LLM(model=path, dtype="bfloat16", max_num_batched_seqs=1, max_model_len=2048, gpu_memory_utilization=0.1)
    assert llm.executor.num_pages == 2048 // 16
    out = llm.generate([random_tokens(cfg, 30, seed=5)], SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True),
                       use_tqdm=False)[0]
    assert len(out.token_ids) == 4


D128 = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 256,
        "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 128, "intermediate_size": 512,
        "vocab_size": 1000, "max_position_embeddings": 4096, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
        "tie_word_embeddings": True, "attention_bias": False, "hidden_act": "silu", "torch_dtype": "bfloat16"}


@pytest.mark.parametrize("page_size", [64, 256])
def test_generation_with_large_pages(tmp_path, page_size):
    """Pages of 64 and of 256 slots (the reference's default block size) with the MFMA attention
    kernels: prompts that end inside a page, cross a page's edge while decoding, and share the step."""
    from minivllm_amd import LLM, SamplingParams
    cfg = D128
    w = make_weights(cfg, seed=78, stored=torch.bfloat16, qk_gain=1.5)
    path = write_model_dir(str(tmp_path / "d128p"), cfg, w)
    prompts = [random_tokens(cfg, n, seed=700 + n) for n in (250, 40, 7, 300, 129)]
    sp = SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True)
    llm = LLM(model=path, dtype="bfloat16", kv_cache_block_size=page_size, kv_cache_num_blocks=4096 // page_size,
              max_model_len=512, max_num_batched_tokens=192, max_num_batched_seqs=8)
    outs = llm.generate(prompts, sp, use_tqdm=False)
    check_against_plain(cfg, w, outs, [sp] * len(prompts), "bfloat16")
    llm.manager.check_invariants()


def test_generation_with_head_size_128(tmp_path):
    """A small model with the head size the MFMA kernels serve (128; hidden 256, two kv heads, K =
    256/512): decode steps take the fused attention and products, alone, in graphs and four in a
    row; the tokens are the plain model's, and the same however the steps are run."""
    from minivllm_amd import LLM, SamplingParams
    cfg = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 256,
           "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 128, "intermediate_size": 512,
           "vocab_size": 1000, "max_position_embeddings": 4096, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
           "tie_word_embeddings": True, "attention_bias": False, "hidden_act": "silu", "torch_dtype": "bfloat16"}
    w = make_weights(cfg, seed=77, stored=torch.bfloat16, qk_gain=1.5)
    path = write_model_dir(str(tmp_path / "d128"), cfg, w)
    prompts = [random_tokens(cfg, n, seed=300 + n) for n in (150, 40, 7, 300)]
    sp = SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True)
    results = {}
    for name, opts in (("graphs of four", dict(num_scheduler_steps=4)), ("graphs of one", dict(num_scheduler_steps=1)),
                       ("eager", dict(use_cuda_graph=False, num_scheduler_steps=1))):
        llm = LLM(model=path, dtype="bfloat16", kv_cache_block_size=16, kv_cache_num_blocks=128, max_model_len=512,
                  max_num_batched_tokens=256, max_num_batched_seqs=8, **opts)
        outs = llm.generate(prompts, sp, use_tqdm=False)
        results[name] = [o.token_ids for o in outs]
        if name == "graphs of four":
            check_against_plain(cfg, w, outs, [sp] * len(prompts), "bfloat16")
        llm.manager.check_invariants()
        del llm
        torch.cuda.empty_cache()
    assert results["graphs of four"] == results["graphs of one"]
    # eager steps split the keys differently and round differently: the same tokens but for near ties
    same = sum(a == b for a, b in zip(results["eager"], results["graphs of one"]))
    assert same >= len(prompts) - 1


def test_generation_with_wide_layers_leaves_partial_sums_to_the_norms(tmp_path, monkeypatch):
    """Two layers as wide as a large model's (output and down projections of 16 Mi elements): with
    ten sequences decoding, these products split K over workgroups and leave their partial sums to
    the norm that follows. The tokens are the plain model's, and the same as when every product
    adds its sums up itself."""
    from minivllm_amd import LLM, SamplingParams
    cfg = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 2048,
           "num_attention_heads": 64, "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 8192,
           "vocab_size": 1000, "max_position_embeddings": 4096, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
           "tie_word_embeddings": False, "attention_bias": False, "hidden_act": "silu", "torch_dtype": "bfloat16"}
    w = make_weights(cfg, seed=91, stored=torch.bfloat16, qk_gain=1.5)
    path = write_model_dir(str(tmp_path / "wide"), cfg, w)
    prompts = [random_tokens(cfg, n, seed=500 + n) for n in (3, 20, 7, 12, 5, 9, 16, 4, 11, 8)]
    sp = SamplingParams(temperature=0.0, max_tokens=5, ignore_eos=True)
    calls = {"split": 0}
    from minivllm_amd.kernels.library import KernelLibrary
    real_call = KernelLibrary.call

    def counting_call(self, name, *args):
        if name == "mv_add_rmsnorm_split":
            calls["split"] += 1
        return real_call(self, name, *args)

    monkeypatch.setattr(KernelLibrary, "call", counting_call)
    results = {}
    for name in ("deferred", "added up"):
        if name == "added up":
            real_has = KernelLibrary.has
            monkeypatch.setattr(KernelLibrary, "has", lambda self, n: n != "mv_add_rmsnorm_split" and real_has(self, n))
        llm = LLM(model=path, dtype="bfloat16", kv_cache_block_size=16, kv_cache_num_blocks=64, max_model_len=64,
                  max_num_batched_tokens=256, max_num_batched_seqs=16, use_cuda_graph=(name == "deferred"))
        outs = llm.generate(prompts, sp, use_tqdm=False)
        results[name] = [o.token_ids for o in outs]
        if name == "deferred":
            assert calls["split"] > 0, "no product left its sums to a norm"
            check_against_plain(cfg, w, outs[:3], [sp] * 3, "bfloat16")
            seen = calls["split"]
        else:
            assert calls["split"] == seen
        del llm
        torch.cuda.empty_cache()
    assert results["deferred"] == results["added up"]

"""Configurations drawn at random (head sizes in steps of 16, any number of heads and groups,
widths and vocabularies that are no power of two, with and without window, bias and tied head,
pages of 4 to 64 slots): for each, mixed steps on few pages against the plain model, in float32
and in bfloat16. Whatever kernels a configuration is served by, the logits must be right."""
import numpy as np
import pytest
import torch

import trace_tools
from helpers import (TOL_F32, bf16_tolerance, make_weights, plain_logits, plain_logits_bf16, random_tokens, rel_err,
                     write_model_dir)

pytestmark = pytest.mark.gpu


def draw_config(seed: int):
    rng = np.random.default_rng(1000 + seed)
    head_dim = int(rng.choice([16, 32, 48, 64, 64, 80, 96, 112, 128, 128]))
    kv_heads = int(rng.choice([1, 2, 3, 5]))
    group = int(rng.choice([1, 2, 3, 4, 8, 16]))
    layers = int(rng.choice([1, 2, 3]))
    window = int(rng.choice([0, 0, 9, 20, 33]))
    cfg = {
        "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
        "num_hidden_layers": layers, "hidden_size": int(rng.choice([40, 72, 96, 100, 160, 192, 224, 264, 320])),
        "num_attention_heads": kv_heads * group, "num_key_value_heads": kv_heads, "head_dim": head_dim,
        "intermediate_size": int(rng.choice([56, 96, 100, 160, 264, 288])), "vocab_size": int(rng.choice([97, 300, 1001])),
        "max_position_embeddings": 512, "rope_theta": float(rng.choice([1e4, 5e4, 1e6])),
        "rms_norm_eps": float(rng.choice([1e-6, 1e-5, 3e-5])), "tie_word_embeddings": bool(rng.integers(2)),
        "attention_bias": bool(rng.integers(2)), "hidden_act": "silu",
        "torch_dtype": str(rng.choice(["float32", "bfloat16"])), "eos_token_id": 1,
    }
    if window:
        cfg.update(use_sliding_window=True, sliding_window=window, max_window_layers=int(rng.integers(0, layers)))
    page_size = int(rng.choice([4, 8, 16, 16, 32, 64]))
    lengths = [int(n) for n in rng.integers(2, 90, size=4)]
    return cfg, page_size, lengths


@pytest.mark.parametrize("seed", range(16))
def test_random_configuration_against_the_plain_model(tmp_path, seed):
    from minivllm_amd.engine.trace import TraceRunner
    cfg, page_size, lengths = draw_config(seed)
    stored = torch.float32 if cfg["torch_dtype"] == "float32" else torch.bfloat16
    weights = make_weights(cfg, seed=seed, stored=stored, qk_gain=2.0)
    path = write_model_dir(str(tmp_path / "model"), cfg, weights)
    reqs = {f"r{i}": random_tokens(cfg, n, seed=10 * seed + i) for i, n in enumerate(lengths)}
    want = {rid: plain_logits(cfg, weights, toks) for rid, toks in reqs.items()}
    emulated = {rid: plain_logits_bf16(cfg, weights, toks) for rid, toks in reqs.items()}
    bf16_error = max(rel_err(emulated[rid][p], want[rid][p]) for rid, toks in reqs.items() for p in range(len(toks)))
    prompt_lens = {rid: max(2, len(t) - 9) if len(t) > 3 else len(t) for rid, t in reqs.items()}
    steps = trace_tools.mixed(reqs, prompt_lens, max_live=3, seed=seed)
    what = (f"seed {seed}: D={cfg['head_dim']} H={cfg['num_attention_heads']} Hkv={cfg['num_key_value_heads']} "
            f"h={cfg['hidden_size']} I={cfg['intermediate_size']} V={cfg['vocab_size']} L={cfg['num_hidden_layers']} "
            f"window={cfg.get('sliding_window')} bias={cfg['attention_bias']} page={page_size}")
    for dtype in ("float32", "bfloat16"):
        runner = TraceRunner(path, dtype, trace_tools.max_live_tokens(steps), page_size=page_size)
        got = trace_tools.collect(steps, runner.run_step)
        assert len(got) == sum(len(t) for t in reqs.values())
        worst = max(rel_err(row, want[rid][pos]) for (rid, pos), row in got.items())
        tol = TOL_F32 if dtype == "float32" else bf16_tolerance(bf16_error)
        print(f"{what} [{dtype}]: worst relative error {worst:.3e} (allowed {tol:.3e})")
        assert worst <= tol, f"{what} [{dtype}]: {worst:.3e} exceeds {tol:.1e}"
        runner.manager.check_invariants()
        assert all(pool.num_free == pool.num_pages for pool in runner.manager.pools)

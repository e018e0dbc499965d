"""A toy architecture defined here, in the test: a mixer with a state of its own (a running
mean, carried per request in a state slot), an order of layers that runs one layer twice and
lets another read an earlier call's cache. It is registered, built and stepped through the
engine's executor, cache manager and kernels without touching the framework's files, and is
compared with a plain whole-sequence computation, cut in several ways."""
from dataclasses import dataclass
from typing import ClassVar, Dict, Optional

import numpy as np
import pytest
import torch

from helpers import rel_err

pytestmark = pytest.mark.gpu


def define_toy():
    from minivllm_amd.config.model_config import ModelConfig
    from minivllm_amd.models.registry import Architecture, register_architecture
    from minivllm_amd.parts import (AttentionSpec, Call, EmbeddingSpec, HeadSpec, LayerPlan, Mixer, ModelPlan,
                                    PartSpec, PreNormBlockSpec, RMSNormSpec, RotarySpec, SwiGLUSpec, TensorDecl,
                                    MIXERS, register_mixer)

    @dataclass(frozen=True)
    class RunningMeanSpec(PartSpec):
        kind: ClassVar[str] = "toy_running_mean"
        hidden_size: int = 0

    class RunningMean(Mixer):
        """y_t = W mean(x_0 .. x_t); the running sum lives in the request's state slot."""

        @classmethod
        def tensors(cls, spec):
            return {"w": TensorDecl((spec.hidden_size, spec.hidden_size))}

        @classmethod
        def state_shape(cls, spec):
            return (spec.hidden_size,), torch.float32

        def __init__(self, spec, tensors, rt):
            self.spec, self.rt, self.w = spec, rt, tensors["w"]

        def forward(self, x, ctx, call):
            state = ctx.state(call)
            y = torch.zeros_like(x)
            base = 0
            for n, start, slot in zip(ctx.q_lens, ctx.starts, ctx.host_state_slots):
                rows = slice(base, base + n)
                sums = state[slot][None, :] + torch.cumsum(x[rows].float(), dim=0)
                counts = torch.arange(start + 1, start + n + 1, device=x.device, dtype=torch.float32)[:, None]
                y[rows] = ((sums / counts) @ self.w.float().T).to(x.dtype)
                state[slot] = sums[-1]
                base += n
            return y

    if "toy_running_mean" not in MIXERS.kinds():
        register_mixer(RunningMeanSpec.kind, RunningMean)

    @dataclass(frozen=True)
    class ToyConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyStateLM"
        vocab_size: int = 50
        hidden_size: int = 48
        max_position_embeddings: int = 256
        dtype: str = "float32"

        @classmethod
        def from_dict(cls, d, where="config.json"):
            return cls(vocab_size=d["vocab_size"], hidden_size=d["hidden_size"])

    def plan(cfg):
        h = cfg.hidden_size
        norm = RMSNormSpec(size=h, eps=1e-5)
        rope = RotarySpec(rotary_dim=8, theta=100.0)          # rotates half of each head only
        attn = AttentionSpec(hidden_size=h, num_heads=3, num_kv_heads=1, head_dim=16, scale=0.25, qk_norm=False,
                             position=rope)
        reader = AttentionSpec(hidden_size=h, num_heads=3, num_kv_heads=1, head_dim=16, scale=0.25, qk_norm=False,
                               position=rope, shares_kv=True)
        ffn = SwiGLUSpec(hidden_size=h, intermediate_size=40)
        norms = (("mixer", norm), ("ffn", norm))
        layers = (LayerPlan(PreNormBlockSpec(), attn, ffn, norms),
                  LayerPlan(PreNormBlockSpec(), RunningMeanSpec(hidden_size=h), ffn, norms),
                  LayerPlan(PreNormBlockSpec(), reader, ffn, norms))
        # layer 0 runs twice (two caches), layer 2 reads the cache of the first call
        calls = (Call(0), Call(1), Call(0), Call(2, cache_from=0))
        return ModelPlan(hidden_size=h, vocab_size=cfg.vocab_size, max_positions=cfg.max_position_embeddings,
                         embedding=EmbeddingSpec(cfg.vocab_size, h), layers=layers, calls=calls, final_norm=norm,
                         head=HeadSpec(cfg.vocab_size, h, tied=True))

    def tensor_name(cfg, loc):
        if loc.layer is None:
            return "embed" if loc.role in ("embedding", "head") else f"{loc.role}.{loc.name}"
        return f"layers.{loc.layer}.{loc.role}.{loc.name}"

    arch = Architecture("ToyStateLM", ToyConfig, plan, tensor_name)
    register_architecture(arch, replace=True)
    return arch, ToyConfig()


def toy_plain(w: Dict[str, torch.Tensor], tokens):
    """The toy model on a whole sequence in float64."""
    w = {k: v.double() for k, v in w.items()}
    n = len(tokens)
    x = w["embed"][torch.tensor(tokens)]
    pos = torch.arange(n, dtype=torch.float64)

    def norm(v, name):
        return v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + 1e-5) * w[name]

    def rope(t):                       # [n, heads, 16], the first 8 of each head rotate in halves of 4
        inv = 1.0 / (100.0 ** (torch.arange(0, 8, 2, dtype=torch.float) / 8)).double()
        ang = pos[:, None] * inv[None, :]
        c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
        a, b = t[..., :4], t[..., 4:8]
        return torch.cat([a * c - b * s, b * c + a * s, t[..., 8:]], dim=-1)

    def attention(q, k, v):
        out = torch.zeros(n, 3, 16, dtype=torch.float64)
        mask = torch.tril(torch.ones(n, n, dtype=torch.bool))
        for h in range(3):
            sc = (q[:, h] @ k[:, 0].T) * 0.25
            out[:, h] = torch.softmax(sc.masked_fill(~mask, float("-inf")), -1) @ v[:, 0]
        return out.reshape(n, 48)

    def ffn(v, i):
        p = f"layers.{i}.ffn."
        g, u = v @ w[p + "gate"].T, v @ w[p + "up"].T
        return (g * torch.sigmoid(g) * u) @ w[p + "down"].T

    kv0 = None
    for call, layer in enumerate([0, 1, 0, 2]):
        p = f"layers.{layer}."
        hcur = norm(x, p + "norm.mixer.weight")
        if layer == 1:
            mean = torch.cumsum(hcur, 0) / (pos[:, None] + 1)
            y = mean @ w[p + "mixer.w"].T
        else:
            q = rope((hcur @ w[p + "mixer.q"].T).view(n, 3, 16))
            if layer == 0:
                k = rope((hcur @ w[p + "mixer.k"].T).view(n, 1, 16))
                v = (hcur @ w[p + "mixer.v"].T).view(n, 1, 16)
                if call == 0:
                    kv0 = (k, v)
            else:
                k, v = kv0
            y = attention(q, k, v) @ w[p + "mixer.o"].T
        x = x + y
        x = x + ffn(norm(x, p + "norm.ffn.weight"), layer)
    return (norm(x, "final_norm.weight") @ w["embed"].T).numpy()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_model_with_state_steps_through_the_engine(dtype):
    from minivllm_amd.config import EngineConfig
    from minivllm_amd.engine.executor import Executor
    from minivllm_amd.engine.step import SeqStep
    from minivllm_amd.models import expected_tensors
    from minivllm_amd.weights import DictSource

    arch, cfg = define_toy()
    g = torch.Generator().manual_seed(3)
    weights = {}
    for name, decl in expected_tensors(arch, cfg).items():
        t = torch.randn(decl.shape, generator=g) * 0.1
        weights[name] = (t + 1.0) if decl.init == "ones_normal" else t
    ex = Executor(EngineConfig(model="", dtype=dtype, max_model_len=128, kv_cache_block_size=8,
                               kv_cache_num_blocks=24, max_num_batched_seqs=4, use_cuda_graph=False),
                  model=(arch, cfg, DictSource(weights)))
    assert ex.has_state and len(ex.groups) == 1 and ex.groups[0].calls == (0, 2)      # calls 0 and 2 keep caches
    assert sorted(ex.state_tensors) == [1] and sorted(ex.kv_pages) == [0, 2]
    mgr = ex.new_cache_manager(enable_prefix_caching=True)
    assert not mgr.prefix_caching                              # state forbids prefix reuse
    rng = np.random.default_rng(0)
    reqs = {r: [int(t) for t in rng.integers(0, 50, size=n)] for r, n in (("a", 37), ("b", 21), ("c", 30))}
    want = {r: toy_plain(weights, t) for r, t in reqs.items()}
    tol = 3e-5 if dtype == "float32" else 6e-2

    def run(entries):
        seqs = []
        for rid, toks in entries:
            if rid not in mgr:
                mgr.admit(rid)
            mgr.reserve(rid, len(toks))
            s = mgr.sequence(rid)
            seqs.append(SeqStep(toks, s.num_computed, [mgr.block_table(rid, 0)], s.state_slot,
                                list(range(len(toks)))))
        out = ex.step(seqs).cpu().numpy()
        for rid, toks in entries:
            mgr.commit(rid, len(toks))
        return out

    # whole
    for rid, toks in reqs.items():
        assert rel_err(run([(rid, toks)]), want[rid]) <= tol
        mgr.release(rid)
    # portions of changing size, three requests interleaved, then one token at a time; the slots
    # of ended requests are taken again and must start from zero
    done = {r: 0 for r in reqs}
    sizes = [5, 2, 9, 3, 1, 1, 7, 2]
    k = 0
    while any(done[r] < len(reqs[r]) for r in reqs):
        entries = []
        for r in reqs:
            if done[r] < len(reqs[r]):
                n = min(sizes[k % len(sizes)], len(reqs[r]) - done[r]); k += 1
                entries.append((r, reqs[r][done[r]:done[r] + n]))
        out = run(entries)
        row = 0
        for r, toks in entries:
            assert rel_err(out[row:row + len(toks)], want[r][done[r]:done[r] + len(toks)]) <= tol, (r, done[r])
            row += len(toks); done[r] += len(toks)
    for r in reqs:
        mgr.release(r)
    mgr.check_invariants()
    assert rel_err(run([("again", reqs["b"])]), want["b"]) <= tol

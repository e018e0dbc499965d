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
        graph_safe = False            # the loop below follows host-side values of the step

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
                               kv_cache_num_blocks=24, max_num_batched_seqs=4),
                  model=(arch, cfg, DictSource(weights)))
    assert not ex.model.graph_safe and not ex.can_repeat(1)     # the toy mixer forbids graphs: every step is eager
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


def define_routed_toy():
    """A second toy architecture: a feed-forward that routes every token to one of four experts,
    and a position encoding with a learned table of its own that is added to queries and keys."""
    from minivllm_amd.config.model_config import ModelConfig
    from minivllm_amd.models.registry import Architecture, register_architecture
    from minivllm_amd.parts import (AttentionSpec, Call, EmbeddingSpec, FeedForward, HeadSpec, LayerPlan, ModelPlan,
                                    PartSpec, PositionEncoding, PreNormBlockSpec, RMSNormSpec, RotarySpec, SwiGLUSpec,
                                    TensorDecl, FEED_FORWARDS, POSITION_ENCODINGS, register_feed_forward,
                                    register_position_encoding)

    @dataclass(frozen=True)
    class RoutedSpec(PartSpec):
        kind: ClassVar[str] = "toy_routed"
        hidden_size: int = 0
        experts: int = 0
        inner: int = 0

    class Routed(FeedForward):
        """y = p_e (relu(x A_e^T) B_e^T) for the expert e with the largest router logit; p = softmax
        of the router logits in float32."""

        @classmethod
        def tensors(cls, spec):
            return {"router": TensorDecl((spec.experts, spec.hidden_size)),
                    "a": TensorDecl((spec.experts, spec.inner, spec.hidden_size)),
                    "b": TensorDecl((spec.experts, spec.hidden_size, spec.inner))}

        def __init__(self, spec, tensors, rt):
            self.spec, self.t = spec, tensors

        def forward(self, x, ctx):
            xf = x.float()
            p = torch.softmax(xf @ self.t["router"].float().T, dim=-1)
            top = p.argmax(dim=-1)
            y = torch.zeros_like(xf)
            for e in range(self.spec.experts):
                rows = (top == e).nonzero().flatten()
                if rows.numel():
                    hid = torch.relu(xf[rows] @ self.t["a"][e].float().T)
                    y[rows] = p[rows, e:e + 1] * (hid @ self.t["b"][e].float().T)
            return y.to(x.dtype)

    @dataclass(frozen=True)
    class LearnedSpec(PartSpec):
        kind: ClassVar[str] = "toy_learned_positions"
        positions: int = 0
        head_dim: int = 0

    class Learned(PositionEncoding):
        """q and k of position p get table[p] added (every head the same)."""

        @classmethod
        def tensors(cls, spec):
            return {"table": TensorDecl((spec.positions, spec.head_dim))}

        def __init__(self, spec, tensors, rt):
            self.table = tensors["table"]

        def apply(self, q, k, ctx):
            add = self.table[ctx.positions[:q.shape[0]].long()].to(q.dtype)[:, None, :]
            q += add
            if k is not None:
                k += add

    if RoutedSpec.kind not in FEED_FORWARDS.kinds():
        register_feed_forward(RoutedSpec.kind, Routed)
    if LearnedSpec.kind not in POSITION_ENCODINGS.kinds():
        register_position_encoding(LearnedSpec.kind, Learned)

    @dataclass(frozen=True)
    class RoutedConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyRoutedLM"
        vocab_size: int = 61
        hidden_size: int = 40
        max_position_embeddings: int = 96
        dtype: str = "float32"

        @classmethod
        def from_dict(cls, d, where="config.json"):
            return cls(vocab_size=d["vocab_size"], hidden_size=d["hidden_size"])

    def plan(cfg):
        h = cfg.hidden_size
        norm = RMSNormSpec(size=h, eps=1e-6)
        learned = LearnedSpec(positions=cfg.max_position_embeddings, head_dim=20)
        a0 = AttentionSpec(hidden_size=h, num_heads=2, num_kv_heads=2, head_dim=20, scale=20 ** -0.5, qk_norm=False,
                           position=learned)
        a1 = AttentionSpec(hidden_size=h, num_heads=2, num_kv_heads=1, head_dim=20, scale=20 ** -0.5, qk_norm=True,
                           position=RotarySpec(rotary_dim=20, theta=50.0))
        norms = (("mixer", norm), ("ffn", norm))
        layers = (LayerPlan(PreNormBlockSpec(), a0, RoutedSpec(hidden_size=h, experts=4, inner=24), norms),
                  LayerPlan(PreNormBlockSpec(), a1, SwiGLUSpec(hidden_size=h, intermediate_size=56), norms))
        return ModelPlan(hidden_size=h, vocab_size=cfg.vocab_size, max_positions=cfg.max_position_embeddings,
                         embedding=EmbeddingSpec(cfg.vocab_size, h), layers=layers, calls=(Call(0), Call(1)),
                         final_norm=norm, head=HeadSpec(cfg.vocab_size, h, tied=False))

    def tensor_name(cfg, loc):
        if loc.layer is None:
            return f"{loc.role}.{loc.name}"
        return f"layers.{loc.layer}.{loc.role}.{loc.name}"

    arch = Architecture("ToyRoutedLM", RoutedConfig, plan, tensor_name)
    register_architecture(arch, replace=True)
    return arch, RoutedConfig()


def routed_plain(w: Dict[str, torch.Tensor], tokens):
    """The routed toy model on a whole sequence in float64."""
    w = {k: v.double() for k, v in w.items()}
    n = len(tokens)
    x = w["embedding.weight"][torch.tensor(tokens)]
    pos = torch.arange(n)
    mask = torch.tril(torch.ones(n, n, dtype=torch.bool))

    def norm(v, weight, eps=1e-6):
        return v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * weight

    def attend(q, k, v, groups):
        out = torch.zeros(n, 2, 20, dtype=torch.float64)
        for h in range(2):
            sc = (q[:, h] @ k[:, h // groups].T) * 20 ** -0.5
            out[:, h] = torch.softmax(sc.masked_fill(~mask, float("-inf")), -1) @ v[:, h // groups]
        return out.reshape(n, 40)

    # layer 0: learned additive positions, two kv heads, routed feed-forward
    p = "layers.0."
    hcur = norm(x, w[p + "norm.mixer.weight"])
    add = w["position.toy_learned_positions.table"][pos][:, None, :]
    q = (hcur @ w[p + "mixer.q"].T).view(n, 2, 20) + add
    k = (hcur @ w[p + "mixer.k"].T).view(n, 2, 20) + add
    v = (hcur @ w[p + "mixer.v"].T).view(n, 2, 20)
    x = x + attend(q, k, v, 1) @ w[p + "mixer.o"].T
    hcur = norm(x, w[p + "norm.ffn.weight"])
    prob = torch.softmax(hcur @ w[p + "ffn.router"].T, dim=-1)
    top = prob.argmax(-1)
    y = torch.zeros_like(hcur)
    for t in range(n):
        e = int(top[t])
        y[t] = prob[t, e] * (torch.relu(hcur[t] @ w[p + "ffn.a"][e].T) @ w[p + "ffn.b"][e].T)
    x = x + y
    # layer 1: q/k norm, rotation over the whole head, one kv head, SwiGLU
    p = "layers.1."
    hcur = norm(x, w[p + "norm.mixer.weight"])
    inv = 1.0 / (50.0 ** (torch.arange(0, 20, 2, dtype=torch.float) / 20)).double()
    ang = pos.double()[:, None] * inv[None, :]
    c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]

    def rope(t):
        a, b = t[..., :10], t[..., 10:]
        return torch.cat([a * c - b * s, b * c + a * s], dim=-1)

    q = rope(norm((hcur @ w[p + "mixer.q"].T).view(n, 2, 20), w[p + "mixer.q_norm"]))
    k = rope(norm((hcur @ w[p + "mixer.k"].T).view(n, 1, 20), w[p + "mixer.k_norm"]))
    v = (hcur @ w[p + "mixer.v"].T).view(n, 1, 20)
    x = x + attend(q, k, v, 2) @ w[p + "mixer.o"].T
    hcur = norm(x, w[p + "norm.ffn.weight"])
    g, u = hcur @ w[p + "ffn.gate"].T, hcur @ w[p + "ffn.up"].T
    x = x + (g * torch.sigmoid(g) * u) @ w[p + "ffn.down"].T
    return (norm(x, w["final_norm.weight"]) @ w["head.weight"].T).numpy(), top.numpy()


def test_toy_routed_feed_forward_and_learned_positions():
    """A routed feed-forward and a position encoding with a tensor of its own, defined here and
    registered without touching the framework's files, through the executor in float32: whole,
    in portions beside another request, and token by token."""
    from minivllm_amd.config import EngineConfig
    from minivllm_amd.engine.executor import Executor
    from minivllm_amd.engine.step import SeqStep
    from minivllm_amd.models import expected_tensors
    from minivllm_amd.weights import DictSource

    arch, cfg = define_routed_toy()
    decls = expected_tensors(arch, cfg)
    assert "position.toy_learned_positions.table" in decls and "layers.0.ffn.router" in decls
    g = torch.Generator().manual_seed(4)
    weights = {}
    for name, decl in decls.items():
        t = torch.randn(decl.shape, generator=g) * 0.2
        weights[name] = (t + 1.0) if decl.init == "ones_normal" else t
    weights["layers.0.ffn.router"] *= 8.0                   # clear routing decisions
    ex = Executor(EngineConfig(model="", dtype="float32", max_model_len=96, kv_cache_block_size=8,
                               kv_cache_num_blocks=30, max_num_batched_seqs=4, use_cuda_graph=False),
                  model=(arch, cfg, DictSource(weights)))
    mgr = ex.new_cache_manager()
    rng = np.random.default_rng(1)
    reqs = {r: [int(t) for t in rng.integers(0, 61, size=n)] for r, n in (("a", 41), ("b", 26))}
    want, routes = {}, {}
    for r, t in reqs.items():
        want[r], routes[r] = routed_plain(weights, t)
    assert len(set(routes["a"].tolist())) >= 3              # several experts are in use

    def run(entries):
        seqs = []
        for rid, toks in entries:
            if rid not in mgr:
                mgr.admit(rid)
            mgr.reserve(rid, len(toks))
            s = mgr.sequence(rid)
            seqs.append(SeqStep(toks, s.num_computed, [mgr.block_table(rid, g) for g in range(len(ex.groups))],
                                s.state_slot, list(range(len(toks)))))
        out = ex.step(seqs).cpu().numpy()
        for rid, toks in entries:
            mgr.commit(rid, len(toks))
        return out

    for rid, toks in reqs.items():
        assert rel_err(run([(rid, toks)]), want[rid]) <= 3e-5
        mgr.release(rid)
    done = {r: 0 for r in reqs}
    sizes = [6, 2, 11, 1, 1, 4]
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
            assert rel_err(out[row:row + len(toks)], want[r][done[r]:done[r] + len(toks)]) <= 3e-5, (r, done[r])
            row += len(toks); done[r] += len(toks)
    for r in reqs:
        mgr.release(r)
    mgr.check_invariants()


def define_chunk_toy():
    """A third toy architecture. Its mixer caches one tensor per token (the mixer's input itself, no
    keys and values) and keeps it by a rule of its own: a query sees its own chunk of tokens (12 in
    the first layer, 20 in the second, which also pages its tensor in float32 whatever the activation
    type: two cache groups with pools of their own sizes), every page before that chunk goes back to
    the pool. Its layers have no feed-forward (a block
    arrangement defined here wires a norm and a mixer only), its norm centres the row (not an RMS
    norm, so no kernel may fuse it as one), and its head caps the logits."""
    from minivllm_amd.config.model_config import ModelConfig
    from minivllm_amd.models.registry import Architecture, register_architecture
    from minivllm_amd.parts import (BLOCKS, HEADS, MIXERS, NORMS, Block, CacheNeed, Call, EmbeddingSpec, Head, LayerPlan,
                                    Mixer, ModelPlan, Norm, PartSpec, Retention, TensorDecl, register_block,
                                    register_head, register_mixer, register_norm)

    @dataclass(frozen=True)
    class KeepChunk(Retention):
        chunk: int = 1

        def first_kept_page(self, next_position, page_size):
            return (next_position // self.chunk) * self.chunk // page_size

        def most_pages_held(self, length, page_size, portion):
            # the chunk of the portion's first token up to the portion's last token
            return min(-(-length // page_size), (self.chunk + portion) // page_size + 2)

    @dataclass(frozen=True)
    class InputCacheNeed(CacheNeed):
        retention: Retention
        hidden_size: int
        in_float32: bool = False

        def page_shapes(self, page_size):
            return {"x": (page_size, self.hidden_size)}

        def page_dtypes(self, activation_dtype):
            return {"x": torch.float32 if self.in_float32 else activation_dtype}

    @dataclass(frozen=True)
    class ChunkMeanSpec(PartSpec):
        kind: ClassVar[str] = "toy_chunk_mean"
        hidden_size: int = 0
        chunk: int = 1
        in_float32: bool = False

    class ChunkMean(Mixer):
        """y_t = W mean(x_s : chunk start <= s <= t), the x_s read back from the paged cache."""
        graph_safe = False

        @classmethod
        def tensors(cls, spec):
            return {"w": TensorDecl((spec.hidden_size, spec.hidden_size))}

        @classmethod
        def cache_need(cls, spec):
            return InputCacheNeed(KeepChunk(spec.chunk), spec.hidden_size, spec.in_float32)

        def __init__(self, spec, tensors, rt):
            self.spec, self.w = spec, tensors["w"]

        def forward(self, x, ctx, call):
            view = ctx.kv(call)
            assert set(view.pages) == {"x"}
            pages, ps, C = view.pages["x"], view.page_size, self.spec.chunk
            y = torch.zeros_like(x)
            base = 0
            for i, (n, start) in enumerate(zip(ctx.q_lens, ctx.starts)):
                table = view.block_table[i].long()
                pos = torch.arange(start, start + n, device=x.device)
                pages[table[pos // ps], pos % ps] = x[base:base + n].to(pages.dtype)
                for j in range(n):
                    p = start + j
                    seen = torch.arange((p // C) * C, p + 1, device=x.device)
                    ids = table[seen // ps]
                    assert int(ids.min()) >= 0, "a page the query needs was given back"
                    mean = pages[ids, seen % ps].float().mean(dim=0)
                    y[base + j] = (mean @ self.w.float().T).to(x.dtype)
                base += n
            return y

    @dataclass(frozen=True)
    class CentredNormSpec(PartSpec):
        kind: ClassVar[str] = "toy_centred_norm"
        size: int = 0
        eps: float = 1e-5

    class CentredNorm(Norm):
        """(x - mean) / sqrt(var + eps) * w: it declares no RMS form, so it always runs by itself."""

        @classmethod
        def tensors(cls, spec):
            return {"weight": TensorDecl((spec.size,), init="ones_normal")}

        def __init__(self, spec, tensors, rt):
            self.spec, self.rt, self.weight = spec, rt, tensors["weight"]

        def forward(self, stream, ctx, rows=None, tag="normed"):
            delta = stream.delta
            if delta is not None and not isinstance(delta, torch.Tensor):
                delta = delta.materialize()
            x = stream.resid if delta is None else stream.resid + delta.float()
            if rows is None:
                stream.resid, stream.delta = x, None
            else:
                x = x[rows.long()]
            c = x - x.mean(-1, keepdim=True)
            return (c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + self.spec.eps) * self.weight.float()).to(self.rt.dtype)

    @dataclass(frozen=True)
    class MixerOnlySpec(PartSpec):
        kind: ClassVar[str] = "toy_mixer_only"

    class MixerOnly(Block):
        """x = x + mixer(norm(x)); the layer has no feed-forward."""
        norm_slots = ("mixer",)

        def __init__(self, spec, norms, mixer, ffn):
            assert ffn is None
            self.norm, self.mixer = norms["mixer"], mixer

        def forward(self, stream, ctx, call):
            stream.delta = self.mixer.forward(self.norm.forward(stream, ctx), ctx, call)

    @dataclass(frozen=True)
    class CappedHeadSpec(PartSpec):
        kind: ClassVar[str] = "toy_capped_head"
        vocab_size: int = 0
        hidden_size: int = 0
        cap: float = 1.0

    class CappedHead(Head):
        """logits = cap * tanh(h W^T / cap), in float32."""

        @classmethod
        def tensors(cls, spec):
            return {"weight": TensorDecl((spec.vocab_size, spec.hidden_size))}

        def __init__(self, spec, tensors, rt):
            self.spec, self.rt, self.weight = spec, rt, tensors["weight"]

        def forward(self, h, ctx):
            raw = torch.empty((h.shape[0], self.spec.vocab_size), dtype=torch.float32, device=h.device)
            self.rt.ops.gemm(h, self.weight, raw)             # the engine's product, then the cap
            return self.spec.cap * torch.tanh(raw / self.spec.cap)

    for registry, register, spec, cls in ((MIXERS, register_mixer, ChunkMeanSpec, ChunkMean),
                                          (NORMS, register_norm, CentredNormSpec, CentredNorm),
                                          (BLOCKS, register_block, MixerOnlySpec, MixerOnly),
                                          (HEADS, register_head, CappedHeadSpec, CappedHead)):
        registry.unregister(spec.kind)
        register(spec.kind, cls)

    @dataclass(frozen=True)
    class ChunkConfig(ModelConfig):
        architecture: ClassVar[str] = "ToyChunkLM"
        vocab_size: int = 70
        hidden_size: int = 64
        max_position_embeddings: int = 128
        dtype: str = "float32"

        @classmethod
        def from_dict(cls, d, where="config.json"):
            return cls(vocab_size=d["vocab_size"], hidden_size=d["hidden_size"])

    def plan(cfg):
        h = cfg.hidden_size
        norm = CentredNormSpec(size=h, eps=1e-5)
        first = LayerPlan(MixerOnlySpec(), ChunkMeanSpec(hidden_size=h, chunk=12), None, (("mixer", norm),))
        second = LayerPlan(MixerOnlySpec(), ChunkMeanSpec(hidden_size=h, chunk=20, in_float32=True), None, (("mixer", norm),))
        return ModelPlan(hidden_size=h, vocab_size=cfg.vocab_size, max_positions=cfg.max_position_embeddings,
                         embedding=EmbeddingSpec(cfg.vocab_size, h), layers=(first, second), calls=(Call(0), Call(1)),
                         final_norm=norm, head=CappedHeadSpec(cfg.vocab_size, h, cap=3.0))

    def tensor_name(cfg, loc):
        return f"{loc.role}.{loc.name}" if loc.layer is None else f"layers.{loc.layer}.{loc.role}.{loc.name}"

    arch = Architecture("ToyChunkLM", ChunkConfig, plan, tensor_name)
    register_architecture(arch, replace=True)
    return arch, ChunkConfig()


def chunk_plain(w: Dict[str, torch.Tensor], tokens, chunks=(12, 20), cap=3.0):
    w = {k: v.double() for k, v in w.items()}
    x = w["embedding.weight"][torch.tensor(tokens)]
    n = len(tokens)

    def norm(v, weight):
        c = v - v.mean(-1, keepdim=True)
        return c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + 1e-5) * weight

    for layer, chunk in enumerate(chunks):
        hcur = norm(x, w[f"layers.{layer}.norm.mixer.weight"])
        y = torch.stack([hcur[(t // chunk) * chunk:t + 1].mean(0) for t in range(n)])
        x = x + y @ w[f"layers.{layer}.mixer.w"].T
    return (cap * torch.tanh(norm(x, w["final_norm.weight"]) @ w["head.weight"].T / cap)).numpy()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_one_tensor_cache_with_its_own_retention_norm_block_and_head(dtype):
    """A mixer with a one-tensor cache and a third retention rule, a layer without feed-forward, a
    norm that is no RMS norm and a head that caps its logits: all defined in this file, built and
    stepped through the engine without a change to it; two requests beside each other in portions
    and token by token, on pools that hold them only because pages behind a chunk come back. The two
    layers keep chunks of different lengths, so they are two cache groups, each with a pool of its
    own size, and the second pages its tensor in float32 whatever the activation type."""
    from minivllm_amd.config import EngineConfig
    from minivllm_amd.engine.executor import Executor
    from minivllm_amd.engine.step import SeqStep
    from minivllm_amd.models import expected_tensors
    from minivllm_amd.weights import DictSource

    arch, cfg = define_chunk_toy()
    g = torch.Generator().manual_seed(8)
    weights = {}
    for name, decl in expected_tensors(arch, cfg).items():
        t = torch.randn(decl.shape, generator=g) * 0.3
        weights[name] = (t + 1.0) if decl.init == "ones_normal" else t
    assert sorted(weights) == ["embedding.weight", "final_norm.weight", "head.weight", "layers.0.mixer.w",
                               "layers.0.norm.mixer.weight", "layers.1.mixer.w", "layers.1.norm.mixer.weight"]
    ex = Executor(EngineConfig(model="", dtype=dtype, max_model_len=128, kv_cache_block_size=8,
                               kv_cache_num_blocks=(8, 9), max_num_batched_seqs=2),
                  model=(arch, cfg, DictSource(weights)))
    assert [g.retention.key() for g in ex.groups] == [("KeepChunk", ("chunk", 12)), ("KeepChunk", ("chunk", 20))]
    assert {n: tuple(t.shape) for n, t in ex.kv_pages[0].items()} == {"x": (8, 8, 64)}
    assert {n: tuple(t.shape) for n, t in ex.kv_pages[1].items()} == {"x": (9, 8, 64)}
    assert ex.kv_pages[0]["x"].dtype == ex.dtype and ex.kv_pages[1]["x"].dtype == torch.float32
    assert ex.bytes_per_page(1) == 8 * 64 * 4
    mgr = ex.new_cache_manager(enable_prefix_caching=True)
    assert not mgr.prefix_caching                      # the rule does not keep everything
    rng = np.random.default_rng(2)
    reqs = {r: [int(t) for t in rng.integers(0, 70, size=n)] for r, n in (("a", 61), ("b", 47))}
    want = {r: chunk_plain(weights, t) for r, t in reqs.items()}
    tol = 3e-5 if dtype == "float32" else 4e-2

    def run(entries):
        seqs = []
        for rid, toks in entries:
            if rid not in mgr:
                mgr.admit(rid)
            mgr.reserve(rid, len(toks))
            s = mgr.sequence(rid)
            seqs.append(SeqStep(toks, s.num_computed, [mgr.block_table(rid, 0), mgr.block_table(rid, 1)], s.state_slot,
                                list(range(len(toks)))))
        out = ex.step(seqs).cpu().numpy()
        for rid, toks in entries:
            mgr.commit(rid, len(toks))
        mgr.check_invariants()
        return out

    assert [p.num_pages for p in mgr.pools] == [8, 9]
    assert rel_err(run([("a", reqs["a"])]), want["a"]) <= tol           # whole: all 8 pages for one request
    mgr.release("a")
    done = {r: 0 for r in reqs}
    sizes = [5, 2, 9, 3, 1, 1, 7, 2]
    k = most_used = 0
    while any(done[r] < len(reqs[r]) for r in reqs):
        entries = []
        for r in reqs:
            if done[r] < len(reqs[r]):
                n = min(sizes[k % len(sizes)], len(reqs[r]) - done[r]); k += 1
                entries.append((r, reqs[r][done[r]:done[r] + n]))
        out = run(entries)
        most_used = max(most_used, mgr.pools[0].num_used)
        row = 0
        for r, toks in entries:
            assert rel_err(out[row:row + len(toks)], want[r][done[r]:done[r] + len(toks)]) <= tol, (r, done[r])
            row += len(toks); done[r] += len(toks)
    # 108 tokens went through a pool of 64 slots: pages behind the chunks were given back and used again
    assert most_used <= 8 and sum(len(t) for t in reqs.values()) > 8 * 8
    for r in reqs:
        mgr.release(r)
    assert [p.num_free for p in mgr.pools] == [8, 9]
    # pools sized from the memory left: no group gets more pages than its live requests can hold at a
    # time (two requests; steps of up to 16 tokens: a chunk and a portion, and the pages their ends touch)
    auto = Executor(EngineConfig(model="", dtype=dtype, max_model_len=128, kv_cache_block_size=8, max_num_batched_seqs=2,
                                 max_num_batched_tokens=16, gpu_memory_utilization=0.3),
                    model=(arch, cfg, DictSource(weights)))
    assert auto.group_pages == [2 * ((12 + 16) // 8 + 2), 2 * ((20 + 16) // 8 + 2)]
    assert [p.num_pages for p in auto.new_cache_manager().pools] == auto.group_pages

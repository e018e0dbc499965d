"""Each part alone (norm, position encoding, attention mixer, feed-forward, block
arrangement), built from its spec through the registries and run on a hand-made step, against
the plain functions."""
import numpy as np
import pytest
import torch

from helpers import TINY_B, make_weights, rel_err
from plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu
TOL = {"float32": 2e-5, "bfloat16": 3e-2}


def runtime(dtype_name, max_positions=256):
    from minivllm_amd.kernels.ops import dtype_from_name, get_ops
    from minivllm_amd.parts import Runtime, Workspace
    dt = dtype_from_name(dtype_name)
    dev = torch.device("cuda:0")
    return Runtime(device=dev, dtype=dt, ops=get_ops(dt), workspace=Workspace(dev), max_positions=max_positions)


def hand_made_step(rt, portions, page_size, kv_shapes):
    """portions: list of (sequence index, start, n). Pages are handed out in a scrambled order."""
    from minivllm_amd.engine.step import KVView, StepContext
    n_seqs = max(s for s, _, _ in portions) + 1
    ends = [0] * n_seqs
    for s, start, n in portions:
        ends[s] = max(ends[s], start + n)
    pages_per = [-(-e // page_size) for e in ends]
    order = np.random.default_rng(0).permutation(sum(pages_per) + 3).tolist()
    tables, cur = [], 0
    for p in pages_per:
        tables.append(order[cur:cur + p]); cur += p
    width = max(pages_per)
    return tables, width, sum(pages_per) + 3


class Ctx:
    """The few fields of a step context that parts read."""
    def __init__(self, rt, seq_of_token, positions, tables, width, page_size, kv):
        from minivllm_amd.engine.step import KVView
        dev = rt.device
        self.n_tokens = len(positions)
        self.positions = torch.tensor(positions, dtype=torch.int32, device=dev)
        self.token_seq = torch.tensor(seq_of_token, dtype=torch.int32, device=dev)
        bt = torch.full((len(tables), width), -1, dtype=torch.int32)
        for i, t in enumerate(tables):
            bt[i, :len(t)] = torch.tensor(t, dtype=torch.int32)
        self.block_table = bt.to(dev)
        self.attention_plan = None
        self._kv = KVView({"k": kv[0], "v": kv[1]}, self.block_table, page_size)

    def kv(self, call):
        return self._kv


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_norm_part(dtype):
    from minivllm_amd.parts import NORMS, HiddenStream, RMSNormSpec
    rt = runtime(dtype)
    spec = RMSNormSpec(size=72, eps=1e-5)
    g = torch.Generator().manual_seed(0)
    w = 1 + 0.1 * torch.randn(72, generator=g)
    part = NORMS.get(spec.kind)(spec, {"weight": w.to(rt.device)}, rt)
    assert list(NORMS.get(spec.kind).tensors(spec)) == ["weight"]
    resid = torch.randn(6, 72, generator=g)
    delta = torch.randn(6, 72, generator=g).to(rt.dtype)
    stream = HiddenStream(resid.to(rt.device).clone())
    stream.delta = delta.to(rt.device)
    out = part.forward(stream, None)
    want_sum = resid.double() + delta.double()
    assert stream.delta is None
    assert rel_err(stream.resid.cpu().numpy(), want_sum.numpy()) <= 1e-7
    assert rel_err(out.float().cpu().numpy(), plain.rms_norm(want_sum, w.double(), 1e-5).numpy()) <= TOL[dtype]


def test_rotary_part_table():
    from minivllm_amd.parts import POSITION_ENCODINGS, RotarySpec
    rt = runtime("float32", max_positions=300)
    spec = RotarySpec(rotary_dim=32, theta=1e6)
    part = POSITION_ENCODINGS.get(spec.kind)(spec, {}, rt)
    table, interleaved = part.rotary()
    cos, sin = plain.rope_cos_sin(torch.arange(300), 32, 1e6)
    assert not interleaved and table.shape == (300, 32)
    assert float((table.cpu().double() - torch.cat([cos, sin], -1)).abs().max()) <= 3e-7


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_feed_forward_part(dtype):
    from minivllm_amd.parts import FEED_FORWARDS, SwiGLUSpec
    rt = runtime(dtype)
    spec = SwiGLUSpec(hidden_size=40, intermediate_size=56)
    g = torch.Generator().manual_seed(1)
    t = {"gate": torch.randn(56, 40, generator=g) * 0.3, "up": torch.randn(56, 40, generator=g) * 0.3,
         "down": torch.randn(40, 56, generator=g) * 0.3}
    stored = {k: v.to(rt.dtype) for k, v in t.items()}
    part = FEED_FORWARDS.get(spec.kind)(spec, {k: v.to(rt.device) for k, v in stored.items()}, rt)
    x = torch.randn(9, 40, generator=g).to(rt.dtype)
    y = part.forward(x.to(rt.device), None)
    want = plain.swiglu_mlp(x.double(), *(stored[k].double() for k in ("gate", "up", "down")))
    assert rel_err(y.float().cpu().numpy(), want.numpy()) <= TOL[dtype]


def _attention_case(dtype, layer):
    """Layer ``layer`` of tiny B (bias, q/k norm, rotary; layer 1 has a window of 21) on two
    sequences: one whole (50 tokens), one whose first 30 tokens are already in the cache."""
    from minivllm_amd.models import config_from_dict
    rt = runtime(dtype)
    cfg = TINY_B
    arch, typed = config_from_dict(dict(cfg))
    plan = arch.plan(typed)
    w = make_weights(cfg, 11, stored=torch.float32 if dtype == "float32" else torch.bfloat16, qk_gain=2.0)
    spec = plan.layers[layer].mixer
    return rt, cfg, arch, typed, plan, w, spec


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("layer", [0, 1])
def test_attention_part_and_block(dtype, layer):
    from minivllm_amd.parts import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, HiddenStream
    from minivllm_amd.parts.plan import TensorLocation
    rt, cfg, arch, typed, plan, w, spec = _attention_case(dtype, layer)
    dev = rt.device
    ps = 8

    def tensors(role, decls):
        return {n: w[arch.tensor_name(typed, TensorLocation(layer, role, n))].to(dev) for n in decls}

    rope = POSITION_ENCODINGS.get(spec.position.kind)(spec.position, {}, rt)
    mixer_cls = MIXERS.get(spec.kind)
    mixer = mixer_cls(spec, tensors("mixer", mixer_cls.tensors(spec)), rt, position=rope)
    need = mixer_cls.cache_need(spec)
    from minivllm_amd.parts import KeepAll, KeepWindow
    assert need.retention == (KeepAll() if layer == 0 else KeepWindow(20))

    g = torch.Generator().manual_seed(2)
    lens = [50, 44]
    x_all = [torch.randn(n, cfg["hidden_size"], generator=g).to(rt.dtype) for n in lens]
    # plain: whole sequences
    wd = {k: v.double() for k, v in w.items()}
    want = [plain.attention_block(cfg, wd, layer, x.double(), torch.arange(x.shape[0])) for x in x_all]

    tables, width, n_pages = hand_made_step(rt, [(0, 0, 50), (1, 0, 44)], ps, None)
    shapes = need.page_shapes(ps)
    assert list(shapes) == ["k", "v"]
    k_shape, v_shape = shapes["k"], shapes["v"]
    kv = (torch.full((n_pages,) + k_shape, float("nan"), dtype=rt.dtype, device=dev),
          torch.full((n_pages,) + v_shape, float("nan"), dtype=rt.dtype, device=dev))
    # step 1: the first 30 tokens of sequence 1 alone
    ctx = Ctx(rt, [1] * 30, list(range(30)), tables, width, ps, kv)
    y = mixer.forward(x_all[1][:30].to(dev), ctx, 0)
    assert rel_err(y.float().cpu().numpy(), want[1][:30].numpy()) <= TOL[dtype]
    # step 2: sequence 0 whole beside the rest of sequence 1
    ctx = Ctx(rt, [0] * 50 + [1] * 14, list(range(50)) + list(range(30, 44)), tables, width, ps, kv)
    x = torch.cat([x_all[0], x_all[1][30:]]).to(dev)
    y = mixer.forward(x, ctx, 0).float().cpu()
    assert rel_err(y[:50].numpy(), want[0].numpy()) <= TOL[dtype]
    assert rel_err(y[50:].numpy(), want[1][30:].numpy()) <= TOL[dtype]

    # the whole block arrangement around the same mixer
    lp = plan.layers[layer]
    norms = {}
    for slot, nspec in lp.norms:
        cls = NORMS.get(nspec.kind)
        norms[slot] = cls(nspec, tensors(f"norm.{slot}", cls.tensors(nspec)), rt)
    ffn_cls = FEED_FORWARDS.get(lp.ffn.kind)
    ffn = ffn_cls(lp.ffn, tensors("ffn", ffn_cls.tensors(lp.ffn)), rt)
    block = BLOCKS.get(lp.block.kind)(lp.block, norms, mixer, ffn)
    kv[0].fill_(float("nan")); kv[1].fill_(float("nan"))
    ctx = Ctx(rt, [0] * 50, list(range(50)), tables, width, ps, kv)
    stream = HiddenStream(x_all[0].float().to(dev).clone())
    block.forward(stream, ctx, 0)
    got = stream.resid.cpu().double() + stream.delta.float().cpu().double()
    want_block = plain.decoder_layer(cfg, wd, layer, x_all[0].double(), torch.arange(50))
    assert rel_err(got.numpy(), want_block.numpy()) <= TOL[dtype]

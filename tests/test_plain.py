"""Pins the plain implementation by what fixes it beside the reference's text: special cases
that reduce to a library routine, invariants, and hand-made vectors; each chosen so that a
plausible mistake (a wrong sign or pairing, a norm in the wrong place, an off-by-one window)
fails it. The reference holds no numeric vectors for these parts (its only test is the block
manager's), so there is no reference output to compare with: parity with the reference's own
kernels is unpinned beyond these checks."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import TINY_A, TINY_B, make_weights, random_tokens
from plain import qwen3_plain as P

torch.manual_seed(0)
D64 = torch.float64


def test_rms_norm_is_the_library_routine():
    x = torch.randn(5, 3, 48, dtype=D64)
    w = torch.randn(48, dtype=D64)
    assert torch.allclose(P.rms_norm(x, w, 1e-5), F.rms_norm(x, (48,), w, 1e-5), atol=1e-14)
    # with unit weight the mean square of the output is 1 / (1 + eps / ms)
    y = P.rms_norm(x, torch.ones(48, dtype=D64), 1e-2)
    ms = x.pow(2).mean(-1)
    assert torch.allclose(y.pow(2).mean(-1), 1 / (1 + 1e-2 / ms), atol=1e-12)
    # scale invariance up to eps; the weight multiplies (it is not 1 + w)
    assert torch.allclose(P.rms_norm(7 * x, w, 1e-12), P.rms_norm(x, w, 1e-12), atol=1e-9)
    assert torch.equal(P.rms_norm(x, torch.zeros(48, dtype=D64), 1e-6), torch.zeros_like(x))


def test_rope_is_complex_multiplication_of_half_split_pairs():
    n, H, d, theta = 9, 3, 16, 10000.0
    x = torch.randn(n, H, d, dtype=D64)
    pos = torch.tensor([0, 1, 2, 3, 10, 50, 51, 400, 1000])
    cos, sin = P.rope_cos_sin(pos, d, theta)
    y = P.apply_rope(x, cos, sin)
    # pairs are (i, i + d/2): (x1 + i x2) * exp(i * ang)   [a wrong sign or an interleaved pairing fails here]
    z = torch.complex(x[..., :d // 2], x[..., d // 2:]) * torch.polar(torch.ones_like(cos), torch.atan2(sin, cos))[:, None, :]
    assert torch.allclose(y[..., :d // 2], z.real, atol=1e-12) and torch.allclose(y[..., d // 2:], z.imag, atol=1e-12)
    assert torch.allclose(y[0], x[0], atol=0)                               # position 0 is the identity
    assert torch.allclose(y.pow(2).sum(-1), x.pow(2).sum(-1), atol=1e-10)   # a rotation keeps the norm
    # inv_freq_0 = 1: the first pair turns by exactly `position` radians; the last by pos * theta^-(d-2)/d
    assert torch.allclose(cos[:, 0], torch.cos(pos.double()), atol=1e-6)
    inv_last = theta ** (-(d - 2) / d)
    assert torch.allclose(sin[:, -1], torch.sin(pos.double() * inv_last), atol=1e-6)


def test_rope_scores_depend_on_distance_only():
    d, theta = 32, 1e6
    q, k = torch.randn(1, 1, d, dtype=D64), torch.randn(1, 1, d, dtype=D64)
    def score(m, n):
        cm, sm = P.rope_cos_sin(torch.tensor([m]), d, theta)
        cn, sn = P.rope_cos_sin(torch.tensor([n]), d, theta)
        return float((P.apply_rope(q, cm, sm) * P.apply_rope(k, cn, sn)).sum())
    assert abs(score(7, 3) - score(107, 103)) < 1e-4        # angles are float32, as in the reference
    assert abs(score(7, 3) - score(3, 7)) > 1e-3            # but the sign of the distance matters


def test_attention_is_the_library_routine_without_window():
    n, H, Hkv, d = 13, 6, 2, 16
    q, k, v = torch.randn(n, H, d, dtype=D64), torch.randn(n, Hkv, d, dtype=D64), torch.randn(n, Hkv, d, dtype=D64)
    got = P.causal_attention(q, k, v, d ** -0.5)
    kr, vr = k.repeat_interleave(H // Hkv, dim=1), v.repeat_interleave(H // Hkv, dim=1)   # head h reads h // group
    want = F.scaled_dot_product_attention(q.transpose(0, 1), kr.transpose(0, 1), vr.transpose(0, 1),
                                          is_causal=True, scale=d ** -0.5).transpose(0, 1)
    assert torch.allclose(got, want, atol=1e-12)
    assert torch.allclose(got[0], vr[0], atol=1e-14)                   # the first token sees only itself
    # with as many kv heads as heads it is plain multi-head attention
    got_mha = P.causal_attention(q, kr, vr, d ** -0.5)
    assert torch.allclose(got_mha, got, atol=1e-14)


def test_attention_window_counts_tokens_to_the_left():
    """window = number of tokens to the left a query may attend to besides itself
    (minivllm/models/layers/attention.py:56-60)."""
    n, d = 8, 4
    q = torch.zeros(n, 1, d, dtype=D64)                 # equal scores: the output is the mean of the visible values
    k = torch.zeros(n, 1, d, dtype=D64)
    v = torch.arange(n, dtype=D64)[:, None, None].expand(n, 1, d).clone()
    out = P.causal_attention(q, k, v, 1.0, window=2)[:, 0, 0]
    want = torch.tensor([0, 0.5, 1, 2, 3, 4, 5, 6], dtype=D64)     # mean of positions max(0, p-2) .. p
    assert torch.allclose(out, want, atol=1e-14)
    assert torch.allclose(P.causal_attention(q, k, v, 1.0, window=0)[:, 0, 0], torch.arange(n, dtype=D64))
    assert torch.allclose(P.causal_attention(q, k, v, 1.0, window=100), P.causal_attention(q, k, v, 1.0))


def test_swiglu_is_the_library_routine():
    x = torch.randn(4, 10, dtype=D64)
    g, u, dn = torch.randn(14, 10, dtype=D64), torch.randn(14, 10, dtype=D64), torch.randn(10, 14, dtype=D64)
    want = (F.silu(x @ g.T) * (x @ u.T)) @ dn.T
    assert torch.allclose(P.swiglu_mlp(x, g, u, dn), want, atol=1e-12)


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B])
def test_model_invariants(cfg):
    w = make_weights(cfg, 5, qk_gain=2.0)
    toks = random_tokens(cfg, 40, 9)
    full = P.forward(cfg, w, toks)
    assert full.shape == (40, cfg["vocab_size"])
    # causal: the logits at a position do not depend on later tokens
    assert torch.allclose(P.forward(cfg, w, toks[:23]), full[:23], atol=1e-10)
    other = toks[:23] + random_tokens(cfg, 17, 10)
    assert torch.allclose(P.forward(cfg, w, other)[:23], full[:23], atol=1e-10)
    assert not torch.allclose(P.forward(cfg, w, other)[30], full[30], atol=1e-3)
    # only distances count: shifting every position leaves the logits (angles are float32)
    assert torch.allclose(P.forward(cfg, w, toks, first_position=64), full, atol=2e-4)
    # the order of tokens matters (a missing rotary embedding would pass the line above vacuously)
    swapped = list(toks); swapped[3], swapped[11] = swapped[11], swapped[3]
    assert not torch.allclose(P.forward(cfg, w, swapped)[-1], full[-1], atol=1e-3)


def test_tied_and_untied_heads():
    w = make_weights(TINY_A, 1)
    toks = random_tokens(TINY_A, 6, 0)
    base = P.forward(TINY_A, w, toks)
    w2 = dict(w); w2["model.embed_tokens.weight"] = w["model.embed_tokens.weight"] * 2
    # tied: doubling the table doubles the logits' head side (the input side is normalised away only partly)
    assert not torch.allclose(P.forward(TINY_A, w2, toks), base)
    wb = make_weights(TINY_B, 1)
    tb = random_tokens(TINY_B, 6, 0)
    wb2 = dict(wb); wb2["lm_head.weight"] = wb["lm_head.weight"] * 2
    assert torch.allclose(P.forward(TINY_B, wb2, tb), 2 * P.forward(TINY_B, wb, tb), atol=1e-12)


def test_window_layers_of_the_tiny_config():
    assert [P.layer_window(TINY_B, i) for i in range(3)] == [None, 20, 20]
    assert [P.layer_window(TINY_A, i) for i in range(2)] == [None, None]
    # the window changes the result once the sequence is longer than it
    w = make_weights(TINY_B, 2, qk_gain=2.0)
    toks = random_tokens(TINY_B, 40, 3)
    no_window = {**TINY_B, "use_sliding_window": False}
    a, b = P.forward(TINY_B, w, toks), P.forward(no_window, w, toks)
    # sliding_window 21: position 20 still sees keys 0..20 (21 of them), position 21 is the first to lose key 0
    assert torch.allclose(a[:21], b[:21], atol=1e-12) and not torch.allclose(a[21], b[21], atol=1e-6)
    assert not torch.allclose(a[30:], b[30:], atol=1e-4)


def test_sampling_rule():
    z = np.array([2.0, 1.0, 3.0, 0.5, 3.0, -1.0], dtype=np.float32)
    assert P.sample_token(z, 0.0)[0] == 2                                   # arg-max, ties to the lowest id
    assert P.kept_set(z, 2, 1.0).tolist() == [False, False, True, False, True, False]
    assert P.kept_set(z, 3, 1.0).tolist() == [True, False, True, False, True, False]
    p = np.exp(z - z.max()); p /= p.sum()
    # top-p: the smallest set of most likely tokens with mass >= p (ties come together)
    assert P.kept_set(z, 0, float(p[2] + p[4]) - 1e-6).tolist() == [False, False, True, False, True, False]
    assert P.kept_set(z, 0, float(p[2] + p[4]) + 1e-3).tolist() == [True, False, True, False, True, False]
    # draws are reproducible, differ between counters, and never leave the kept set
    toks = [P.sample_token(z, 0.7, top_k=3, seed=11, counter=c)[0] for c in range(50)]
    assert toks == [P.sample_token(z, 0.7, top_k=3, seed=11, counter=c)[0] for c in range(50)]
    assert set(toks) <= {0, 2, 4} and len(set(toks)) > 1
    u = [float(P.uniform23(1, c, i)) for c in range(20) for i in range(20)]
    assert 0 < min(u) and max(u) < 1 and abs(np.mean(u) - 0.5) < 0.05

"""A plain, slow Qwen3 forward pass: whole sequences, no cache, one function per part.

Written from the reference's formulas (each function cites file:line under the reference's
root); it imports nothing from the engine. Everything runs on the CPU in the dtype of the
inputs (tests use float64, or float32 to mirror the reference's own arithmetic).

``weights`` maps the names on disk (``model.layers.0.self_attn.q_proj.weight`` ...) to
tensors; ``cfg`` is the raw dictionary of ``config.json``.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import numpy as np
import torch


# ---------------------------------------------------------------------------------------
# parts
# ---------------------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """minivllm/models/models/qwen3.py:18-23 — x * rsqrt(mean(x^2) + eps), then * weight.
    (The model uses nn.RMSNorm with the same eps, qwen3.py:134-139,64-65,176.)"""
    variance = x.pow(2).mean(-1, keepdim=True)
    return weight * (x * torch.rsqrt(variance + eps))


def rope_cos_sin(positions: torch.Tensor, rotary_dim: int, theta: float, dtype=torch.float64):
    """minivllm/models/layers/rotary.py:35-46 — inv_freq = 1 / theta^(arange(0, d, 2) / d),
    freqs = position (outer) inv_freq, table = cat(cos, sin). The reference evaluates inv_freq
    and the angles in float32 (``dtype=torch.float``, rotary.py:35,38); so does this, and then
    takes cosine and sine of those float32 angles in ``dtype``. Returns (cos, sin), each
    [n, rotary_dim / 2]."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float) / rotary_dim))
    freqs = torch.einsum("i,j->ij", positions.to(torch.float), inv_freq.to(positions.device))
    return freqs.to(dtype).cos(), freqs.to(dtype).sin()


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """minivllm/models/layers/rotary.py:6-14 — split the head in two halves x1 | x2;
    y1 = x1 cos - x2 sin, y2 = x2 cos + x1 sin; x is [n, heads, d], cos/sin [n, d/2]
    (broadcast over heads, rotary.py:63-65)."""
    x1, x2 = torch.chunk(x, 2, dim=-1)
    c, s = cos.unsqueeze(1), sin.unsqueeze(1)
    return torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), dim=-1)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                     window: Optional[int] = None) -> torch.Tensor:
    """minivllm/models/layers/attention.py:78-92 with scale = head_dim^-0.5
    (minivllm/models/models/qwen3.py:32): causal softmax attention of one sequence; query head
    h reads key/value head h // (H / Hkv). ``window`` = how many tokens to the left a query may
    attend to besides itself (attention.py:56-60); None = all.
    q [n, H, d], k, v [n, Hkv, d] -> [n, H, d]."""
    n, H, d = q.shape
    Hkv = k.shape[1]
    group = H // Hkv
    out = torch.empty_like(q)
    idx = torch.arange(n, device=q.device)
    allowed = idx[None, :] <= idx[:, None]
    if window is not None:
        allowed &= idx[None, :] >= idx[:, None] - window
    for h in range(H):
        kh = h // group
        scores = (q[:, h, :] @ k[:, kh, :].T) * scale
        scores = scores.masked_fill(~allowed, float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        out[:, h, :] = probs @ v[:, kh, :]
    return out


def swiglu_mlp(x: torch.Tensor, gate_w: torch.Tensor, up_w: torch.Tensor, down_w: torch.Tensor,
               rnd=None) -> torch.Tensor:
    """minivllm/models/models/qwen3.py:116-121 — down(silu(gate(x)) * up(x)), no biases."""
    rnd = rnd or (lambda t: t)
    gate = rnd(x @ gate_w.T)
    up = rnd(x @ up_w.T)
    return rnd(rnd(gate * torch.sigmoid(gate) * up) @ down_w.T)


def layer_window(cfg: Dict, layer: int) -> Optional[int]:
    """Window of a layer from config.json, as ``causal_attention`` counts it (tokens to the left
    besides the query, minivllm/models/layers/attention.py:56-60). With ``use_sliding_window`` the
    layers from ``max_window_layers`` on see ``sliding_window`` keys, the query's own among them
    (the meaning of the key where it comes from), hence ``sliding_window - 1`` to the left. The
    reference's Qwen3 never hands a window to its attention (minivllm/models/models/qwen3.py:66-71):
    no file of the reference pins this rule."""
    if cfg.get("use_sliding_window") and layer >= cfg.get("max_window_layers", cfg["num_hidden_layers"]):
        return cfg["sliding_window"] - 1
    return None


def _identity(x: torch.Tensor) -> torch.Tensor:
    return x


def round_to_bfloat16(x: torch.Tensor) -> torch.Tensor:
    """What storing an activation in bfloat16 does to it."""
    return x.to(torch.bfloat16).to(x.dtype)


def attention_block(cfg: Dict, w: Dict[str, torch.Tensor], i: int, x: torch.Tensor,
                    positions: torch.Tensor, rnd=_identity) -> torch.Tensor:
    """minivllm/models/models/qwen3.py:73-101 — q/k/v projections, view as heads, RMSNorm of q
    and k over head_dim with one weight per projection (qwen3.py:64-65,89-90), rotary embedding
    (qwen3.py:92), attention, output projection."""
    H, Hkv = cfg["num_attention_heads"], cfg.get("num_key_value_heads", cfg["num_attention_heads"])
    d = cfg.get("head_dim") or cfg["hidden_size"] // H
    eps = cfg.get("rms_norm_eps", 1e-6)
    p = f"model.layers.{i}.self_attn."
    q = x @ w[p + "q_proj.weight"].T
    k = x @ w[p + "k_proj.weight"].T
    v = x @ w[p + "v_proj.weight"].T
    if cfg.get("attention_bias"):
        q = q + w[p + "q_proj.bias"]
        k = k + w[p + "k_proj.bias"]
        v = v + w[p + "v_proj.bias"]
    q, k, v = rnd(q), rnd(k), rnd(v)
    n = x.shape[0]
    q = q.view(n, H, d)
    k = k.view(n, Hkv, d)
    v = v.view(n, Hkv, d)
    q = rms_norm(q, w[p + "q_norm.weight"], eps)
    k = rms_norm(k, w[p + "k_norm.weight"], eps)
    cos, sin = rope_cos_sin(positions, d, cfg.get("rope_theta", 10000.0), dtype=x.dtype)
    q = rnd(apply_rope(q, cos, sin))
    k = rnd(apply_rope(k, cos, sin))
    o = rnd(causal_attention(q, k, v, d ** -0.5, layer_window(cfg, i)))
    o = o.reshape(n, H * d) @ w[p + "o_proj.weight"].T
    if cfg.get("attention_bias"):
        o = o + w[p + "o_proj.bias"]
    return rnd(o)


def decoder_layer(cfg: Dict, w: Dict[str, torch.Tensor], i: int, x: torch.Tensor,
                  positions: torch.Tensor, rnd=_identity) -> torch.Tensor:
    """minivllm/models/models/qwen3.py:141-156 — x += attn(input_layernorm(x));
    x += mlp(post_attention_layernorm(x))."""
    eps = cfg.get("rms_norm_eps", 1e-6)
    p = f"model.layers.{i}."
    x = x + attention_block(cfg, w, i, rnd(rms_norm(x, w[p + "input_layernorm.weight"], eps)), positions, rnd)
    h = rnd(rms_norm(x, w[p + "post_attention_layernorm.weight"], eps))
    x = x + swiglu_mlp(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                       w[p + "mlp.down_proj.weight"], rnd)
    return x


def forward(cfg: Dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64,
            first_position: int = 0, rnd=_identity, device=None) -> torch.Tensor:
    """minivllm/models/models/qwen3.py:178-190,206-220 — embed, layers, final norm, head (tied
    to the embedding when ``tie_word_embeddings``, qwen3.py:203-204). Returns the logits of every
    position, [n, vocab]. ``first_position`` shifts all positions (for invariance tests).
    ``rnd`` is applied to every activation a reduced-precision implementation would store
    (outputs of projections, norms, rotary embedding, attention, activation); with
    ``round_to_bfloat16`` the result shows how far bfloat16 storage alone moves the logits of
    this model and input, which is what an engine's bfloat16 error is measured against.
    ``device``: where these tensor operations run (the CPU unless a test of very long sequences
    says otherwise: a square of scores per head is slow there); the result is on the CPU."""
    w = {k: v.to(device=device, dtype=dtype) for k, v in weights.items()}
    ids = torch.tensor(tokens, dtype=torch.long, device=device)
    positions = torch.arange(first_position, first_position + len(tokens), device=device)
    x = w["model.embed_tokens.weight"][ids]
    for i in range(cfg["num_hidden_layers"]):
        x = decoder_layer(cfg, w, i, x, positions, rnd)
    x = rnd(rms_norm(x, w["model.norm.weight"], cfg.get("rms_norm_eps", 1e-6)))
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings") else w["lm_head.weight"]
    return (x @ head.T).cpu()


# ---------------------------------------------------------------------------------------
# sampling (the engine's documented rule, computed here with numpy)
# ---------------------------------------------------------------------------------------
_M64 = (1 << 64) - 1


def _mix64(x: int) -> int:
    x &= _M64
    x ^= x >> 30
    x = (x * 0xBF58476D1CE4E5B9) & _M64
    x ^= x >> 27
    x = (x * 0x94D049BB133111EB) & _M64
    x ^= x >> 31
    return x


def uniform23(seed: int, counter: int, index: int) -> np.float32:
    """The engine's counter-based uniform number in (0, 1) for (seed, counter, index)."""
    x = _mix64((seed + 0x9E3779B97F4A7C15 * (counter + 1)) & _M64)
    x = _mix64(x ^ ((0xD1B54A32D192ED03 * (index + 1)) & _M64))
    return (np.float32(x >> 41) + np.float32(0.5)) * np.float32(1.0 / 8388608.0)


def kept_set(z: np.ndarray, top_k: int, top_p: float) -> np.ndarray:
    """Boolean mask of the tokens that stay after top-k (every z >= the k-th largest), then
    top-p over the kept ones (every z >= t, t the largest value whose upper set holds at least
    top_p of the kept probability mass). minivllm/models/layers/sampler.py:18-27 hands both
    filters to a library; this is the rule the engine documents for them."""
    keep = np.ones(z.shape, dtype=bool)
    V = z.shape[0]
    if 0 < top_k < V:
        kth = np.sort(z)[::-1][top_k - 1]
        keep &= z >= kth
    if top_p < 1.0:
        zk = np.where(keep, z.astype(np.float64), -np.inf)
        w = np.exp(zk - zk.max())
        total = w.sum()
        order = np.argsort(-zk, kind="stable")
        csum = np.cumsum(w[order])
        cut = int(np.searchsorted(csum, top_p * total, side="left"))
        cut = min(cut, V - 1)
        t = zk[order[cut]]
        keep &= zk >= t
    return keep


def sample_token(logits: np.ndarray, temperature: float, top_k: int = 0, top_p: float = 1.0,
                 seed: int = 0, counter: int = 0):
    """minivllm/models/layers/sampler.py:15-31 — divide by the temperature, filter, draw. The
    draw is the engine's Gumbel-max rule: argmax z_i - log(-log(u_i)). Returns (token, perturbed
    scores) so that a test can allow for a near tie."""
    logits = logits.astype(np.float32)
    if temperature == 0:
        return int(np.argmax(logits)), logits
    z = logits / np.float32(temperature)
    keep = kept_set(z, top_k, top_p)
    u = np.array([uniform23(seed, counter, i) for i in range(z.shape[0])], dtype=np.float32)
    g = -np.log(-np.log(u))
    score = np.where(keep, z + g.astype(np.float32), -np.inf).astype(np.float32)
    return int(np.argmax(score)), score

"""A plain, slow Llama 3 decoder: whole sequences, no cache, one function per part.

Written from the formulas of the reference (paths are relative to the reference
checkout); it shares no code with ``yalis_amd``. Everything is computed in
float32 (float64 on request) on the CPU.  ``rounder`` lets a caller emulate a
reduced-precision engine by rounding activations where such an engine stores them.

The weights are a dict keyed by the tensor names of a Hugging Face Llama checkpoint
(``model.embed_tokens.weight``, ``model.layers.{i}.self_attn.q_proj.weight`` ...),
the configuration is the plain dict of ``config.json``.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, Optional, Sequence

import numpy as np
import torch

Rounder = Callable[[torch.Tensor], torch.Tensor]


def _identity(x: torch.Tensor) -> torch.Tensor:
    return x


def bf16_round(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.bfloat16).to(x.dtype)


# --------------------------------------------------------------------------- norm
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """yalis/external/model.py:979-986: float32, mean of squares over the last
    dim, rsqrt(ms + eps), times the weight in float32, one rounding at the end."""
    xf = x.to(torch.float32) if x.dtype != torch.float64 else x
    ms = torch.mean(xf * xf, dim=-1, keepdim=True)
    return xf * torch.rsqrt(ms + eps) * weight.to(xf.dtype)


# --------------------------------------------------------------------------- rope
def rope_inv_freq(head_dim: int, theta: float, scaling: Optional[dict]) -> torch.Tensor:
    """yalis/external/model.py:786-807: inverse frequencies, with the llama3
    adjustment when ``scaling`` (config.json's rope_scaling) is given."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2).float() / head_dim))
    if scaling is not None:
        orig = scaling["original_max_position_embeddings"]
        factor = scaling["factor"]
        low = scaling["low_freq_factor"]
        high = scaling["high_freq_factor"]
        wavelen = 2 * torch.pi / inv
        ratio = orig / wavelen
        smooth = torch.clamp((ratio - low) / (high - low), min=0.0, max=1.0)
        inv = (1 - smooth) * (inv / factor) + smooth * inv
    return inv


def rope_cos_sin(positions: torch.Tensor, inv_freq: torch.Tensor):
    """yalis/external/model.py:809-820: angle[p, i] = p * theta_i in float32, the
    table has head_dim/2 columns (the flash layout; the sdpa one repeats it)."""
    ang = torch.outer(positions.to(torch.float32), inv_freq.to(torch.float32))
    return torch.cos(ang), torch.sin(ang)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """yalis/external/model.py:894-909: half-split pairs (i, i + D/2):
    out = x * cos + cat(-x2, x1) * sin.  x: [T, heads, D]; cos, sin: [T, D/2]."""
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    c = cos[:, None, :].to(x.dtype)
    s = sin[:, None, :].to(x.dtype)
    return torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), dim=-1)


# ---------------------------------------------------------------------- attention
def causal_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    scale: float,
    q_positions: Optional[torch.Tensor] = None,
    k_positions: Optional[torch.Tensor] = None,
    window: Optional[int] = None,
    round_p: Rounder = _identity,
) -> torch.Tensor:
    """yalis/attention/backend_impl/sdpa_and_flex.py:59-90 and :300-312: query
    head h reads key/value head h // (H / G); scores times ``scale``; key j is
    visible to the query at position p iff j <= p (and p - j < window when a
    window is given); softmax in float32; P @ V.
    q: [Tq, H, D]; k, v: [Tk, G, D].  Returns [Tq, H, D]."""
    tq, n_head, _ = q.shape
    tk, n_group, _ = k.shape
    qpk = n_head // n_group
    if q_positions is None:
        q_positions = torch.arange(tq)
    if k_positions is None:
        k_positions = torch.arange(tk)
    visible = k_positions[None, :] <= q_positions[:, None]
    if window is not None:
        visible &= (q_positions[:, None] - k_positions[None, :]) < window
    out = torch.empty_like(q)
    for h in range(n_head):
        g = h // qpk
        s = (q[:, h, :] @ k[:, g, :].T) * scale
        s = s.masked_fill(~visible, float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[:, h, :] = round_p(p) @ v[:, g, :]
    return out


# -------------------------------------------------------------------- feed-forward
def swiglu_mlp(x, w_gate, w_up, w_down, rounder: Rounder = _identity):
    """yalis/external/model.py:740-744: silu(gate(x)) * up(x), then down.  The
    reference keeps gate and up rows interleaved in one matrix; with separate
    matrices the arithmetic is the same."""
    g = rounder(x @ w_gate.T)
    u = rounder(x @ w_up.T)
    a = rounder(g * torch.sigmoid(g) * u)
    return rounder(a @ w_down.T)


# ---------------------------------------------------------------------- the model
def layer_forward(
    cfg: dict,
    weights: Dict[str, torch.Tensor],
    layer: int,
    x: torch.Tensor,
    positions: torch.Tensor,
    rounder: Rounder = _identity,
    window: Optional[int] = None,
    residual_rounder: Rounder = _identity,
) -> torch.Tensor:
    """yalis/external/model.py:414-439 (pre-norm, sequential residuals) around
    :525-608 (attention) and :740-744 (feed-forward).  x: [T, C] residual.
    ``residual_rounder`` rounds the residual stream after each sum: the reference in bfloat16
    keeps the stream in bfloat16 (every tensor of :437-438 is), an engine may keep it wider."""
    n_head = cfg["num_attention_heads"]
    n_group = cfg.get("num_key_value_heads") or n_head
    head_dim = cfg.get("head_dim") or cfg["hidden_size"] // n_head
    eps = cfg["rms_norm_eps"]
    p = f"model.layers.{layer}."
    w = lambda n: weights[p + n].to(x.dtype)
    t = x.shape[0]

    h = rounder(rms_norm(x, w("input_layernorm.weight"), eps))
    q = rounder(h @ w("self_attn.q_proj.weight").T).view(t, n_head, head_dim)
    k = rounder(h @ w("self_attn.k_proj.weight").T).view(t, n_group, head_dim)
    v = rounder(h @ w("self_attn.v_proj.weight").T).view(t, n_group, head_dim)
    inv = rope_inv_freq(head_dim, cfg.get("rope_theta", 10000.0), cfg.get("rope_scaling"))
    cos, sin = rope_cos_sin(positions, inv)
    q = rounder(apply_rope(q, cos, sin))
    k = rounder(apply_rope(k, cos, sin))
    a = causal_attention(
        q, k, v, 1.0 / math.sqrt(head_dim), positions, positions, window, round_p=rounder
    )
    a = rounder(a).reshape(t, n_head * head_dim)
    x = residual_rounder(x + rounder(a @ w("self_attn.o_proj.weight").T))

    h = rounder(rms_norm(x, w("post_attention_layernorm.weight"), eps))
    x = residual_rounder(x + swiglu_mlp(
        h, w("mlp.gate_proj.weight"), w("mlp.up_proj.weight"), w("mlp.down_proj.weight"), rounder
    ))
    return x


def forward(
    cfg: dict,
    weights: Dict[str, torch.Tensor],
    tokens: Sequence[int],
    rounder: Rounder = _identity,
    first_position: int = 0,
    dtype: torch.dtype = torch.float32,
    n_layers: Optional[int] = None,
    residual_rounder: Rounder = _identity,
) -> torch.Tensor:
    """yalis/external/model.py:122-197: embedding, the blocks, final norm, head.
    Returns logits [T, V].  ``first_position`` shifts every position (only
    distances matter to rotary attention)."""
    ids = torch.as_tensor(list(tokens), dtype=torch.long)
    x = weights["model.embed_tokens.weight"].to(dtype)[ids]
    positions = torch.arange(first_position, first_position + len(ids))
    n = cfg["num_hidden_layers"] if n_layers is None else n_layers
    for layer in range(n):
        x = layer_forward(cfg, weights, layer, x, positions, rounder, residual_rounder=residual_rounder)
    h = rounder(rms_norm(x, weights["model.norm.weight"].to(dtype), cfg["rms_norm_eps"]))
    if cfg.get("tie_word_embeddings", False):
        head = weights["model.embed_tokens.weight"]
    else:
        head = weights["lm_head.weight"]
    return h @ head.to(dtype).T


# ----------------------------------------------------------------------- sampling
def top_k_filter(logits: torch.Tensor, top_k: int) -> torch.Tensor:
    """yalis/external/sampling.py:51-62: keep the k largest, others to -inf."""
    k = min(top_k, logits.shape[-1])
    kth = torch.topk(logits, k, dim=-1).values[..., -1:]
    return logits.masked_fill(logits < kth, float("-inf"))


def top_p_filter(logits: torch.Tensor, top_p: float) -> torch.Tensor:
    """yalis/external/sampling.py:16-38: sort descending, cumulative softmax,
    remove where the cumulative sum (own mass included) exceeds top_p; rank 0 is
    always kept."""
    sorted_logits, order = torch.sort(logits, descending=True, dim=-1)
    cum = torch.softmax(sorted_logits, dim=-1).cumsum(dim=-1)
    remove_sorted = cum > top_p
    remove_sorted[..., 0] = False
    remove = remove_sorted.scatter(-1, order, remove_sorted)
    return logits.masked_fill(remove, float("-inf"))


def filtered_probs(logits, temperature: float, top_k: Optional[int], top_p: float):
    """yalis/external/sampling.py:41-72 up to the draw: top-k, then temperature,
    then top-p, then a float32 softmax."""
    logits = logits.to(torch.float32)
    if top_k is not None:
        logits = top_k_filter(logits, top_k)
    if temperature > 0.0:
        logits = logits / temperature
    if top_p < 1.0:
        logits = top_p_filter(logits, top_p)
    return torch.softmax(logits, dim=-1)


MASK64 = (1 << 64) - 1


def _mix64(z: int) -> int:
    """The splitmix64 finaliser (public-domain constant set of Steele/Vigna)."""
    z = (z + 0x9E3779B97F4A7C15) & MASK64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK64
    return z ^ (z >> 31)


def race_uniforms(seed: int, draw: int, vocab: int) -> np.ndarray:
    """The engine's documented stream of uniforms: for token i of draw number
    ``draw`` of a request seeded with ``seed``,
    u = (top 23 bits of mix64(mix64(seed * 2^32 + draw) + i) + 0.5) / 2^23
    (exact in float32)."""
    base = _mix64(((seed & 0xFFFFFFFF) << 32) | (draw & 0xFFFFFFFF))
    idx = np.arange(vocab, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = np.uint64(base) + idx
        z = z + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    top = (z >> np.uint64(41)).astype(np.float64)
    return ((top + 0.5) / float(1 << 23)).astype(np.float32)


def sample_token(logits, temperature, top_k, top_p, seed: int, draw: int) -> int:
    """yalis/external/sampling.py:5-13, 64-74: greedy when temperature is 0,
    else draw by the exponential race argmax(p_i / e_i), e_i = -log(u_i)."""
    if temperature == 0.0:
        return int(torch.argmax(logits.to(torch.float32), dim=-1))
    probs = filtered_probs(logits, temperature, top_k, top_p)
    u = torch.from_numpy(race_uniforms(seed, draw, logits.shape[-1]))
    e = -torch.log(u)
    return int(torch.argmax(probs / e, dim=-1))


def greedy_generate(cfg, weights, prompt: Sequence[int], n_new: int, rounder=_identity):
    """Whole-sequence recomputation at every step (no cache)."""
    toks = list(prompt)
    out = []
    for _ in range(n_new):
        logits = forward(cfg, weights, toks, rounder)[-1]
        nxt = int(torch.argmax(logits))
        out.append(nxt)
        toks.append(nxt)
    return out


def sampled_generate(cfg, weights, prompt, n_new, temperature, top_k, top_p, seed):
    toks = list(prompt)
    out = []
    for draw in range(n_new):
        logits = forward(cfg, weights, toks)[-1]
        nxt = sample_token(logits, temperature, top_k, top_p, seed, draw)
        out.append(nxt)
        toks.append(nxt)
    return out


# ------------------------------------------------------------------ random weights
def random_weights(cfg: dict, seed: int, dtype=torch.float32) -> Dict[str, torch.Tensor]:
    """Matrices N(0, 0.02) (yalis/external/model.py:113-120), norm weights
    1 + N(0, 0.1) so that the norm's multiply shows.  Test-side generator: it
    does not have to agree with the framework's own."""
    g = torch.Generator().manual_seed(seed)
    c = cfg["hidden_size"]
    n_head = cfg["num_attention_heads"]
    n_group = cfg.get("num_key_value_heads") or n_head
    d = cfg.get("head_dim") or c // n_head
    inter = cfg["intermediate_size"]
    v = cfg["vocab_size"]

    def mat(*shape):
        return (torch.randn(*shape, generator=g) * 0.02).to(dtype)

    def norm():
        return (1.0 + 0.1 * torch.randn(c, generator=g)).to(dtype)

    w = {"model.embed_tokens.weight": mat(v, c)}
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        w[p + "input_layernorm.weight"] = norm()
        w[p + "self_attn.q_proj.weight"] = mat(n_head * d, c)
        w[p + "self_attn.k_proj.weight"] = mat(n_group * d, c)
        w[p + "self_attn.v_proj.weight"] = mat(n_group * d, c)
        w[p + "self_attn.o_proj.weight"] = mat(c, n_head * d)
        w[p + "post_attention_layernorm.weight"] = norm()
        w[p + "mlp.gate_proj.weight"] = mat(inter, c)
        w[p + "mlp.up_proj.weight"] = mat(inter, c)
        w[p + "mlp.down_proj.weight"] = mat(c, inter)
    w["model.norm.weight"] = norm()
    if not cfg.get("tie_word_embeddings", False):
        w["lm_head.weight"] = mat(v, c)
    return w

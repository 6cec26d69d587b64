"""A plain, slow Qwen3 dense decoder: whole sequences, no cache, one function per part.

Written from the reference's formulas (cited per function as file:line under the
reference's root); it shares no code with ``dryft_amd``. Everything runs in one floating
dtype (float32 by default, float64 to bound its own rounding) with library routines
(``torch.softmax``, ``F.silu``, ``@``), on the CPU unless the weights it is handed sit on
another device (layers of a real model's sizes take minutes in float64 on a CPU). Inputs are
the raw ``config.json`` dictionary and a dictionary of checkpoint tensors by name.
"""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """engine/dryft_qwen3/model.py:28-32: y = w * (x * rsqrt(mean(x^2) + eps)); plain multiplier weight."""
    var = x.pow(2).mean(-1, keepdim=True)
    return weight * (x * torch.rsqrt(var + eps))


def rope_tables(head_dim: int, theta: float, length: int, dtype=torch.float32):
    """engine/dryft_qwen3/model.py:49-57: inv_freq = 1/theta^(2i/d) (float32), angles = pos * inv_freq,
    tables = cos/sin of cat(angles, angles), shape [length, head_dim]. The reference computes the
    angles in float32; so does this, whatever ``dtype`` the result is returned in."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.int64).to(torch.float32) / head_dim))
    pos = torch.arange(length, dtype=torch.float32)
    freqs = pos[:, None] * inv_freq[None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """engine/dryft_qwen3/model.py:35-37: cat(-x[d/2:], x[:d/2])."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """engine/dryft_qwen3/model.py:40-41: x*cos + rotate_half(x)*sin; x [T, heads, d], tables [T, d]."""
    return x * cos[:, None, :] + rotate_half(x) * sin[:, None, :]


def causal_gqa_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                         window: int | None = None) -> torch.Tensor:
    """engine/dryft_qwen3/model.py:172-177 and kernels/attn_decode.py:180-196: query head h uses kv head
    h // group; scores (q.k)*scale; key j visible to query i iff j <= i (and i - j < window if a window is
    given); softmax over keys; weighted sum of values. q [T, nH, d]; k, v [T, nKV, d] -> [T, nH, d]."""
    T, n_heads, _ = q.shape
    group = n_heads // k.shape[1]
    k = k.repeat_interleave(group, dim=1)      # [T, nH, d]
    v = v.repeat_interleave(group, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, k) * scale
    i = torch.arange(T, device=q.device)[:, None]
    j = torch.arange(T, device=q.device)[None, :]
    visible = j <= i
    if window is not None:
        visible = visible & (i - j < window)
    scores = scores.masked_fill(~visible[None], float("-inf"))
    p = torch.softmax(scores, dim=-1)
    return torch.einsum("hij,jhd->ihd", p, v)


def attention_block(h: torch.Tensor, w: dict, prefix: str, cfg: dict, cos, sin) -> torch.Tensor:
    """engine/dryft_qwen3/model.py:153-179 (unfused path 162-171): projections without bias, per-head
    q_norm/k_norm over head_dim before the rotation, rotation of q and k, causal GQA attention with
    scale 1/sqrt(head_dim) (model.py:65), heads concatenated in order, output projection."""
    T = h.shape[0]
    n_heads, n_kv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d = cfg.get("head_dim") or cfg["hidden_size"] // n_heads
    eps = cfg["rms_norm_eps"]
    q = (h @ w[prefix + "self_attn.q_proj.weight"].T).view(T, n_heads, d)
    k = (h @ w[prefix + "self_attn.k_proj.weight"].T).view(T, n_kv, d)
    v = (h @ w[prefix + "self_attn.v_proj.weight"].T).view(T, n_kv, d)
    q = rms_norm(q, w[prefix + "self_attn.q_norm.weight"], eps)
    k = rms_norm(k, w[prefix + "self_attn.k_norm.weight"], eps)
    q = apply_rope(q, cos[:T], sin[:T])
    k = apply_rope(k, cos[:T], sin[:T])
    o = causal_gqa_attention(q, k, v, 1.0 / math.sqrt(d))
    return o.reshape(T, n_heads * d) @ w[prefix + "self_attn.o_proj.weight"].T


def swiglu(h: torch.Tensor, w: dict, prefix: str) -> torch.Tensor:
    """engine/dryft_qwen3/model.py:44-46, 180: down( silu(gate(h)) * up(h) ), no bias."""
    g = h @ w[prefix + "mlp.gate_proj.weight"].T
    u = h @ w[prefix + "mlp.up_proj.weight"].T
    return (F.silu(g) * u) @ w[prefix + "mlp.down_proj.weight"].T


def decoder_layer(x: torch.Tensor, w: dict, i: int, cfg: dict, cos, sin) -> torch.Tensor:
    """engine/dryft_qwen3/model.py:151, 179-184: x += attn(norm(x)); x += mlp(norm(x)); residual adds
    outside the normed branches."""
    p = f"model.layers.{i}."
    eps = cfg["rms_norm_eps"]
    x = x + attention_block(rms_norm(x, w[p + "input_layernorm.weight"], eps), w, p, cfg, cos, sin)
    x = x + swiglu(rms_norm(x, w[p + "post_attention_layernorm.weight"], eps), w, p)
    return x


def forward(cfg: dict, weights: dict, tokens, dtype=torch.float32) -> torch.Tensor:
    """Logits [T, vocab] at every position of one whole sequence.
    engine/dryft_qwen3/model.py:132 (embedding gather), 152 (layers in order), 185-186 (final norm, head);
    weights.py:47-49 (a tied head is the embedding)."""
    w = {k: v.to(dtype) for k, v in weights.items()}
    device = w["model.embed_tokens.weight"].device
    ids = torch.as_tensor(tokens, dtype=torch.long).to(device)
    n_heads = cfg["num_attention_heads"]
    d = cfg.get("head_dim") or cfg["hidden_size"] // n_heads
    cos, sin = (t.to(device) for t in rope_tables(d, cfg["rope_theta"], len(ids), dtype))
    x = w["model.embed_tokens.weight"][ids]
    for i in range(cfg["num_hidden_layers"]):
        x = decoder_layer(x, w, i, cfg, cos, sin)
    x = rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return x @ head.T


def greedy(logits: torch.Tensor) -> int:
    """engine/dryft_qwen3/model.py:187, 262 and AGENTS.md:174-175: argmax, lowest index on ties."""
    return int(torch.argmax(logits, dim=-1))


def sample_with_temperature(logits: torch.Tensor, temperature: float, u: float) -> int:
    """This library's own rule (the reference has none): p = softmax(logits / T); the token is the first
    index whose cumulative probability exceeds u."""
    p = torch.softmax(logits.double() / temperature, dim=-1)
    cdf = torch.cumsum(p, dim=-1)
    idx = int(torch.searchsorted(cdf, torch.tensor(u, dtype=cdf.dtype), right=True))
    return min(idx, logits.numel() - 1)


def cdf_margin(logits: torch.Tensor, temperature: float, u: float) -> float:
    """Distance of u from the nearest boundary of the cumulative distribution."""
    p = torch.softmax(logits.double() / temperature, dim=-1)
    cdf = torch.cumsum(p, dim=-1)
    return float((cdf - u).abs().min())


def generate(cfg: dict, weights: dict, prompt, max_new_tokens: int, choose=greedy, dtype=torch.float32,
             stop_token_ids=()):
    """The starter loop's semantics (agent/verify.py:83-97), one sequence, every step re-running the whole
    sequence: returns (tokens, logits of each step)."""
    seq = list(prompt)
    out, all_logits = [], []
    for t in range(max_new_tokens):
        logits = forward(cfg, weights, seq, dtype)[-1]
        tok = choose(logits) if choose is greedy else choose(logits, t)
        out.append(tok)
        all_logits.append(logits)
        seq.append(tok)
        if tok in stop_token_ids:
            break
    return out, all_logits

"""A plain, slow Qwen3 dense decoder: whole sequences, no cache, double precision.

Written from the reference's formulas (file:line cited at each function; paths
are relative to the reference's root).  It shares no code with the engine: it
has its own weight access (a dictionary of tensors keyed by checkpoint name)
and one function per part.  Everything is torch on the CPU in float64.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

F64 = torch.float64


def embedding(table: torch.Tensor, tokens) -> torch.Tensor:
    """x[r] = E[token_r]; no scale, no position term (crates/leone/src/runtime.rs:7380-7386,
    crates/leone/src/cpu.rs:1258-1263)."""
    return table.to(F64)[torch.as_tensor(tokens, dtype=torch.long)]


def rms_norm(x: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x * gain / sqrt(mean(x^2) + eps), eps inside the root, gain multiplies directly
    (crates/leone/src/cpu.rs:1642-1663)."""
    x = x.to(F64)
    mean_square = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x * gain.to(F64) / torch.sqrt(mean_square + eps)


def linear(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """out_r = sum_c W[r, c] x_c, no bias (crates/leone/src/cpu.rs:1379-1405)."""
    return x.to(F64) @ weight.to(F64).T


def rope_half_split(x: torch.Tensor, positions, theta: float) -> torch.Tensor:
    """x: [tokens, heads, D].  Pair i is (x[i], x[i + D/2]); angle = pos * theta^(-2i/D);
    first' = a cos - b sin, second' = a sin + b cos (crates/leone/src/cpu.rs:1721-1779,
    pairing HalfSplit for this architecture: crates/leone/src/model.rs:299-304)."""
    x = x.to(F64)
    tokens, heads, dim = x.shape
    half = dim // 2
    out = torch.empty_like(x)
    for t in range(tokens):
        pos = float(int(positions[t]))
        for i in range(half):
            angle = pos * (float(theta) ** (-2.0 * i / dim))
            c, s = math.cos(angle), math.sin(angle)
            a, b = x[t, :, i], x[t, :, i + half]
            out[t, :, i] = a * c - b * s
            out[t, :, i + half] = a * s + b * c
    return out


def rope_pairs(x: torch.Tensor, positions, theta: float, rotary_dim: int, pairing: str) -> torch.Tensor:
    """The rotation with its shape as parameters: of a head's first ``rotary_dim`` = R elements, pair i is
    (x[i], x[i + R/2]) ("half_split") or (x[2i], x[2i + 1]) ("adjacent"), angle = pos * theta^(-2i/R); the
    elements from R on are left as they are (the pairing switch of crates/leone/src/cpu.rs:1765-1774, the
    frequencies of :1721-1743 with the rotated width in the exponent)."""
    x = x.to(F64)
    out = x.clone()
    half = rotary_dim // 2
    for t in range(x.shape[0]):
        pos = float(int(positions[t]))
        for i in range(half):
            angle = pos * (float(theta) ** (-2.0 * i / rotary_dim))
            c, s = math.cos(angle), math.sin(angle)
            first, second = (i, i + half) if pairing == "half_split" else (2 * i, 2 * i + 1)
            a, b = x[t, :, first], x[t, :, second]
            out[t, :, first] = a * c - b * s
            out[t, :, second] = a * s + b * c
    return out


def attend_one(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: Optional[int] = None) -> torch.Tensor:
    """One query [Hq, D] at position t = len(k) - 1 over the keys and values [t + 1, Hkv, D] of its
    sequence.  Query head h uses kv head h // (Hq/Hkv); score = (q . k) / sqrt(D), scale after the
    dot (crates/leone/src/cpu.rs:2299-2357).  Two-pass softmax, not the running recurrence.
    ``window`` keeps only the last `window` keys (t - window < j <= t)."""
    q, k, v = q.to(F64), k.to(F64), v.to(F64)
    q_heads, dim = q.shape
    group = q_heads // k.shape[1]
    t = k.shape[0] - 1
    lo = 0 if window is None else max(0, t - window + 1)
    out = torch.zeros_like(q)
    for h in range(q_heads):
        scores = (k[lo:, h // group] @ q[h]) / math.sqrt(dim)
        weights = torch.exp(scores - scores.max())
        out[h] = (weights / weights.sum()) @ v[lo:, h // group]
    return out


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: Optional[int] = None) -> torch.Tensor:
    """q: [T, Hq, D], k and v: [T, Hkv, D] of one sequence from position 0.  Query t sees keys 0..t:
    the mask is the loop bound `j <= pos` (crates/leone/src/cpu.rs:2359-2421, :2372)."""
    return torch.stack([attend_one(q[t], k[:t + 1], v[:t + 1], window) for t in range(q.shape[0])])


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """a = gate / (1 + exp(-gate)) * up (crates/leone/src/cpu.rs:892-907)."""
    gate, up = gate.to(F64), up.to(F64)
    return gate / (1.0 + torch.exp(-gate)) * up


def attention_block(y: torch.Tensor, weights: Dict[str, torch.Tensor], prefix: str, config: dict,
                    positions) -> torch.Tensor:
    """Projections, per-head q/k norm (same formula and eps as the layer norms, gain shared by all heads,
    not applied to v, before the rotation: crates/leone/src/runtime.rs:7388-7389, 9227-9241;
    crates/leone/src/backend.rs:2182-2208), rotation of q and k, attention, output projection."""
    heads, kv_heads, dim = config["num_attention_heads"], config["num_key_value_heads"], config["head_dim"]
    tokens = y.shape[0]
    q = linear(y, weights[f"{prefix}.q_proj.weight"]).view(tokens, heads, dim)
    k = linear(y, weights[f"{prefix}.k_proj.weight"]).view(tokens, kv_heads, dim)
    v = linear(y, weights[f"{prefix}.v_proj.weight"]).view(tokens, kv_heads, dim)
    q = rms_norm(q, weights[f"{prefix}.q_norm.weight"], config["rms_norm_eps"])
    k = rms_norm(k, weights[f"{prefix}.k_norm.weight"], config["rms_norm_eps"])
    if "rotary_dim" in config or "rope_pairing" in config:      # another shape of rotation than this architecture's
        shape = (config.get("rotary_dim", dim), config.get("rope_pairing", "half_split"))
        q, k = (rope_pairs(t, positions, config["rope_theta"], *shape) for t in (q, k))
    else:
        q = rope_half_split(q, positions, config["rope_theta"])
        k = rope_half_split(k, positions, config["rope_theta"])
    attended = causal_attention(q, k, v).reshape(tokens, heads * dim)
    return linear(attended, weights[f"{prefix}.o_proj.weight"])


def feed_forward(y: torch.Tensor, weights: Dict[str, torch.Tensor], prefix: str) -> torch.Tensor:
    """down(swiglu(gate y, up y)), no bias (crates/leone/src/runtime.rs:9283-9319)."""
    gate = linear(y, weights[f"{prefix}.gate_proj.weight"])
    up = linear(y, weights[f"{prefix}.up_proj.weight"])
    return linear(swiglu(gate, up), weights[f"{prefix}.down_proj.weight"])


def forward(weights: Dict[str, torch.Tensor], config: dict, tokens) -> torch.Tensor:
    """Logits [T, vocab] for a whole sequence starting at position 0.

    Layer order x -> norm -> attention -> +x -> norm -> feed-forward -> +x
    (crates/leone/src/runtime.rs:9019-9050); final norm and head, the head being the embedding
    table when tied (crates/leone/src/runtime.rs:7428-7453, crates/leone/src/model.rs:459-470)."""
    config = dict(config)
    config.setdefault("head_dim", config["hidden_size"] // config["num_attention_heads"])
    config.setdefault("num_key_value_heads", config["num_attention_heads"])
    positions = list(range(len(tokens)))
    x = embedding(weights["model.embed_tokens.weight"], tokens)
    for layer in range(config["num_hidden_layers"]):
        p = f"model.layers.{layer}"
        y = rms_norm(x, weights[f"{p}.input_layernorm.weight"], config["rms_norm_eps"])
        x = x + attention_block(y, weights, f"{p}.self_attn", config, positions)
        y = rms_norm(x, weights[f"{p}.post_attention_layernorm.weight"], config["rms_norm_eps"])
        x = x + feed_forward(y, weights, f"{p}.mlp")
    y = rms_norm(x, weights["model.norm.weight"], config["rms_norm_eps"])
    head = weights["model.embed_tokens.weight"] if config.get("tie_word_embeddings", False) else weights["lm_head.weight"]
    return linear(y, head)


def rope_half_split_at_once(x: torch.Tensor, positions, theta: float) -> torch.Tensor:
    """``rope_half_split`` for a hundred thousand positions: the same angles and pairs as array arithmetic
    (``tests/test_plain.py`` holds the two against each other)."""
    x = x.to(F64)
    dim = x.shape[-1]
    half = dim // 2
    rates = torch.tensor([float(theta) ** (-2.0 * i / dim) for i in range(half)], dtype=F64)
    angles = torch.as_tensor(positions, dtype=F64)[:, None] * rates[None, :]
    c, s = torch.cos(angles)[:, None, :], torch.sin(angles)[:, None, :]
    a, b = x[..., :half], x[..., half:]
    return torch.cat([a * c - b * s, a * s + b * c], dim=-1)


def forward_rows_of_one_layer(weights: Dict[str, torch.Tensor], config: dict, tokens, rows) -> torch.Tensor:
    """Logits [len(rows), vocab] at the positions ``rows`` only, for a model of ONE layer: there the keys and
    values of every position come straight from the embeddings, so a context of 100,000 tokens costs what its
    length costs, not its square.  The same part functions in the same order as ``forward``."""
    config = dict(config)
    if config["num_hidden_layers"] != 1:
        raise ValueError("only a model of one layer can be evaluated row by row")
    config.setdefault("head_dim", config["hidden_size"] // config["num_attention_heads"])
    config.setdefault("num_key_value_heads", config["num_attention_heads"])
    heads, kv_heads, dim = config["num_attention_heads"], config["num_key_value_heads"], config["head_dim"]
    eps, theta = config["rms_norm_eps"], config["rope_theta"]
    count = len(tokens)
    p, a = "model.layers.0", "model.layers.0.self_attn"
    x = embedding(weights["model.embed_tokens.weight"], tokens)
    y = rms_norm(x, weights[f"{p}.input_layernorm.weight"], eps)
    k = rms_norm(linear(y, weights[f"{a}.k_proj.weight"]).view(count, kv_heads, dim), weights[f"{a}.k_norm.weight"], eps)
    k = rope_half_split_at_once(k, list(range(count)), theta)
    v = linear(y, weights[f"{a}.v_proj.weight"]).view(count, kv_heads, dim)
    head = weights["model.embed_tokens.weight"] if config.get("tie_word_embeddings", False) else weights["lm_head.weight"]
    out = []
    for t in rows:
        q = rms_norm(linear(y[t:t + 1], weights[f"{a}.q_proj.weight"]).view(1, heads, dim), weights[f"{a}.q_norm.weight"], eps)
        q = rope_half_split(q, [t], theta)
        attended = attend_one(q[0], k[:t + 1], v[:t + 1]).reshape(1, heads * dim)
        xt = x[t:t + 1] + linear(attended, weights[f"{a}.o_proj.weight"])
        xt = xt + feed_forward(rms_norm(xt, weights[f"{p}.post_attention_layernorm.weight"], eps), weights, f"{p}.mlp")
        out.append(linear(rms_norm(xt, weights["model.norm.weight"], eps), head)[0])
    return torch.stack(out)

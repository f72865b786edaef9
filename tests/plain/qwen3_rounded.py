"""The plain Qwen3 decoder with the bfloat16 engine's roundings put in: every tensor the engine stores in
bfloat16 is rounded here at the same point of the formula, everything between is double.  What is left between
this and the engine is the order of float sums, a bfloat16 value that falls the other way when those sums
differ in the last place.  The softmax weights are rounded too: the attention kernels compute them as powers of
two against a whole-number reference, so their bfloat16 significant bits do not depend on the reference, and
the row sum is the sum of the rounded weights.

Where the engine rounds depends on how many rows a step has (crates/leone-cuda/tests/gpu.rs:287-386 rounds the
oracle's inputs like the kernel under test does; crates/leone/src/cpu.rs:205-235, 2583-2602 is the reference's
oracle with quantised activations).  ``few``: a step of at most ``few_rows`` rows folds the norms into the
products, so the product's operand is bf16(x * gain) and the factor 1/rms is applied to the float result; more
rows normalise first and round bf16(x * gain / rms).  ``many``: a step of more than ``many_rows`` rows rounds
gate and up before the activation (the library's product stores them), fewer rows apply the activation to the
float results.  The final norm and head go by the number of wanted rows of the step instead.
"""
from __future__ import annotations

import math
from typing import Dict, Sequence

import torch

from . import qwen3_plain as plain

F64 = torch.float64


def r(x: torch.Tensor) -> torch.Tensor:
    """Round to bfloat16 (nearest even), back in double."""
    return x.to(torch.float32).to(torch.bfloat16).to(F64)


def attend_one_rounded(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """plain.attend_one with weights 2^(t - m), t = score / sqrt(D) * log2(e), m the maximum rounded up, rounded to
    bfloat16 before they weight the values and before they are summed."""
    q, k, v = q.to(F64), k.to(F64), v.to(F64)
    q_heads, dim = q.shape
    group = q_heads // k.shape[1]
    out = torch.zeros_like(q)
    for h in range(q_heads):
        t = (k[:, h // group] @ q[h]) * r_f32(torch.tensor((1.0 / math.sqrt(dim)) * 1.4426950408889634, dtype=F64))
        p = r(torch.exp2(t - torch.ceil(t.max())))
        out[h] = (p @ v[:, h // group]) / p.sum()
    return out


def normed_product(x, gain, eps, weight, few: torch.Tensor):
    """rows of x through norm and product, each row in its step's way.  few: bool [rows]."""
    x = x.to(F64)
    inv = 1.0 / torch.sqrt((x * x).sum(dim=-1, keepdim=True) / x.shape[-1] + eps)
    g = gain.to(F64)
    folded = plain.linear(r(x * g), weight) * inv
    whole = plain.linear(r(r_f32(x * g) * inv), weight)
    return torch.where(few[:, None], folded, whole)


def r_f32(x: torch.Tensor) -> torch.Tensor:
    """A float product as the kernels form it before the next operation."""
    return x.to(torch.float32).to(F64)


def forward(weights: Dict[str, torch.Tensor], config: dict, tokens, step_rows: Sequence[int],
            wanted_rows: Sequence[int], few_rows: int, many_rows: int) -> torch.Tensor:
    """Logits [T, vocab] as the bfloat16 engine rounds them.  step_rows[t]: rows of the step that ran position
    t; wanted_rows[t]: rows of that step whose logits were asked for."""
    config = dict(config)
    config.setdefault("head_dim", config["hidden_size"] // config["num_attention_heads"])
    heads, kv_heads, dim = config["num_attention_heads"], config["num_key_value_heads"], config["head_dim"]
    eps, theta = config["rms_norm_eps"], config["rope_theta"]
    n = len(tokens)
    positions = list(range(n))
    few = torch.tensor([s <= few_rows for s in step_rows])
    many = torch.tensor([s > many_rows for s in step_rows])
    x = plain.embedding(weights["model.embed_tokens.weight"], tokens)
    for layer in range(config["num_hidden_layers"]):
        p = f"model.layers.{layer}"
        a = f"{p}.self_attn"
        w_qkv = torch.cat([weights[f"{a}.{name}_proj.weight"] for name in "qkv"], dim=0)
        qkv = r(normed_product(x, weights[f"{p}.input_layernorm.weight"], eps, w_qkv, few))
        q = qkv[:, :heads * dim].view(n, heads, dim)
        k = qkv[:, heads * dim:(heads + kv_heads) * dim].view(n, kv_heads, dim)
        v = qkv[:, (heads + kv_heads) * dim:].view(n, kv_heads, dim)
        q = r(plain.rope_half_split(plain.rms_norm(q, weights[f"{a}.q_norm.weight"], eps), positions, theta))
        k = r(plain.rope_half_split(plain.rms_norm(k, weights[f"{a}.k_norm.weight"], eps), positions, theta))
        attended = r(torch.stack([attend_one_rounded(q[t], k[:t + 1], v[:t + 1]) for t in range(n)]).reshape(n, heads * dim))
        x = x + plain.linear(attended, weights[f"{a}.o_proj.weight"])
        m = f"{p}.mlp"
        w_gu = torch.cat([weights[f"{m}.gate_proj.weight"], weights[f"{m}.up_proj.weight"]], dim=0)
        gu = normed_product(x, weights[f"{p}.post_attention_layernorm.weight"], eps, w_gu, few)
        gu = torch.where(many[:, None], r(gu), gu)
        ffn = gu.shape[1] // 2
        act = r(plain.swiglu(gu[:, :ffn], gu[:, ffn:]))
        x = x + plain.linear(act, weights[f"{m}.down_proj.weight"])
    head = weights["model.embed_tokens.weight"] if config.get("tie_word_embeddings", False) else weights["lm_head.weight"]
    few_wanted = torch.tensor([w <= few_rows for w in wanted_rows])
    return normed_product(x, weights["model.norm.weight"], eps, head, few_wanted)


def step_sizes(steps, requests) -> Dict[str, tuple]:
    """request -> (rows of the step that ran each position, wanted rows of that step), from trace records."""
    out = {rid: ([], []) for rid in requests}
    for s in steps:
        rows = sum(len(e["tokens"]) for e in s["entries"])
        wanted = sum(len(e["want"]) for e in s["entries"])
        for e in s["entries"]:
            out[e["id"]][0].extend([rows] * len(e["tokens"]))
            out[e["id"]][1].extend([wanted] * len(e["tokens"]))
    return out

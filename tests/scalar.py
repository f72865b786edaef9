"""The host library's scalar single-precision reference (csrc/host/scalar_reference.cpp), bound for the tests:
numpy arrays in, numpy arrays out, and a whole Qwen3 model put together from those functions over a paged
cache.  Test code only: the package never loads these functions."""
from __future__ import annotations

import ctypes
from ctypes import POINTER, c_double, c_float, c_int, c_long

import numpy as np

from leone_amd import hostlib

PF, PI, PD = POINTER(c_float), POINTER(c_int), POINTER(c_double)
_PROTOTYPES = {
    "leone_ref_embed": [PF, PI, PF, c_int, c_int, c_int],
    "leone_ref_add_rmsnorm": [PF, PF, c_int, c_long, PF, c_float, PF, PI, c_int, c_int],
    "leone_ref_rope_table": [PF, PF, c_double, c_int, c_int],
    "leone_ref_qk_norm_rope_write": [PF, c_int, c_long, PF, PF, PF, PF, PF, c_float, PF, PF, c_int, c_int, c_int, PI, PI, PI, c_int,
                                     c_int, c_int, c_int, c_int, c_int, c_int],
    "leone_ref_attention": [PF, PF, PF, PF, PI, PI, PI, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int],
    "leone_ref_gemm": [PF, PF, PF, c_int, c_int, c_int],
    "leone_ref_swiglu": [PF, PF, c_int, c_int],
    "leone_ref_argmax": [PF, PI, c_int, c_int],
    "leone_ref_sample_temperature": [PF, PD, PD, PI, c_int, c_int],
}
_ready = False


def _lib():
    global _ready
    lib = hostlib.library()
    if not _ready:
        for name, argtypes in _PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.argtypes, fn.restype = argtypes, c_int
        _ready = True
    return lib


def _f(a):
    return None if a is None else a.ctypes.data_as(PF)


def _i(a):
    return None if a is None else a.ctypes.data_as(PI)


def f32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def i32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.int32))


def _check(status: int, what: str) -> None:
    if status != 0:
        raise ValueError(f"{what}: the scalar reference refused its arguments ({status})")


def embed(table, tokens):
    table, tokens = f32(table), i32(tokens)
    out = np.empty((tokens.size, table.shape[1]), dtype=np.float32)
    _check(_lib().leone_ref_embed(_f(table), _i(tokens), _f(out), tokens.size, table.shape[1], table.shape[0]), "embed")
    return out


def add_rmsnorm(x, delta, gain, eps, rows=None):
    """x (float32 [n, hidden], changed in place when ``rows`` is None) += delta ([n, hidden] or planes
    [p, n, hidden]); returns the normalised rows."""
    assert x.dtype == np.float32 and x.flags.c_contiguous
    n, hidden = x.shape
    delta = None if delta is None else f32(delta)
    planes = 1 if delta is None or delta.ndim == 2 else delta.shape[0]
    rows = None if rows is None else i32(rows)
    n_out = n if rows is None else rows.size
    y = np.empty((n_out, hidden), dtype=np.float32)
    _check(_lib().leone_ref_add_rmsnorm(_f(x), _f(delta), planes, n * hidden, _f(f32(gain)), eps, _f(y), _i(rows), n_out,
                                        hidden), "add_rmsnorm")
    return y


def rope_table(theta, rotary_dim, positions):
    cos = np.empty((positions, rotary_dim // 2), dtype=np.float32)
    sin = np.empty_like(cos)
    _check(_lib().leone_ref_rope_table(_f(cos), _f(sin), float(theta), rotary_dim, positions), "rope_table")
    return cos, sin


def qk_norm_rope_write(qkv, q_heads, kv_heads, head_dim, q_gain, k_gain, eps, cos, sin, positions, row_entry,
                       block_table, k_pool, v_pool, write_cache=True, pairing=0):
    """The rotation covers the first 2 * (the tables' width) elements of a head; ``pairing`` 0 half split, 1 adjacent."""
    qkv = f32(qkv)
    planes = 1 if qkv.ndim == 2 else qkv.shape[0]
    rows, width = qkv.shape[-2:]
    q_out = np.empty((rows, q_heads * head_dim), dtype=np.float32)
    q_gain, k_gain = (None if q_gain is None else f32(q_gain)), (None if k_gain is None else f32(k_gain))
    positions, row_entry, block_table = i32(positions), i32(row_entry), i32(block_table)
    page_tokens = k_pool.shape[3] if k_pool is not None else 0
    _check(_lib().leone_ref_qk_norm_rope_write(
        _f(qkv), planes, rows * width, _f(q_out), _f(k_pool), _f(v_pool), _f(q_gain), _f(k_gain), eps, _f(cos), _f(sin),
        0 if cos is None else cos.shape[0], 0 if cos is None else 2 * cos.shape[1], pairing, _i(positions), _i(row_entry), _i(block_table), block_table.shape[1], rows,
        q_heads, kv_heads, head_dim, page_tokens, 1 if write_cache else 0), "qk_norm_rope_write")
    return q_out


def attention(q, k_pool, v_pool, positions, row_entry, block_table, q_heads, scale, window=0):
    q = f32(q)
    _, kv_heads, d8, page_tokens, _ = k_pool.shape
    positions, row_entry, block_table = i32(positions), i32(row_entry), i32(block_table)
    out = np.empty_like(q)
    _check(_lib().leone_ref_attention(_f(q), _f(out), _f(k_pool), _f(v_pool), _i(positions), _i(row_entry),
                                      _i(block_table), block_table.shape[1], q.shape[0], q_heads, kv_heads, d8 * 8,
                                      page_tokens, scale, window), "attention")
    return out


def gemm(a, b):
    a, b = f32(a), f32(b)
    c = np.empty((a.shape[0], b.shape[0]), dtype=np.float32)
    _check(_lib().leone_ref_gemm(_f(a), _f(b), _f(c), a.shape[0], b.shape[0], a.shape[1]), "gemm")
    return c


def swiglu(gate_up):
    gate_up = f32(gate_up)
    out = np.empty((gate_up.shape[0], gate_up.shape[1] // 2), dtype=np.float32)
    _check(_lib().leone_ref_swiglu(_f(gate_up), _f(out), gate_up.shape[0], gate_up.shape[1] // 2), "swiglu")
    return out


def argmax(logits):
    logits = f32(logits)
    out = np.empty(logits.shape[0], dtype=np.int32)
    _check(_lib().leone_ref_argmax(_f(logits), _i(out), logits.shape[0], logits.shape[1]), "argmax")
    return out


def sample_temperature(logits, temperature, uniform):
    logits = f32(logits)
    temperature = np.ascontiguousarray(temperature, dtype=np.float64)
    uniform = np.ascontiguousarray(uniform, dtype=np.float64)
    out = np.empty(logits.shape[0], dtype=np.int32)
    _check(_lib().leone_ref_sample_temperature(_f(logits), temperature.ctypes.data_as(PD), uniform.ctypes.data_as(PD),
                                               _i(out), logits.shape[0], logits.shape[1]), "sample_temperature")
    return out


def interleave_gate_up(gate, up):
    """8 gate rows, their 8 up rows, and so on: the order the gated product and ``swiglu`` expect."""
    ffn, hidden = gate.shape
    return np.stack([gate.reshape(ffn // 8, 8, hidden), up.reshape(ffn // 8, 8, hidden)], axis=1).reshape(2 * ffn, hidden)


class ScalarQwen3:
    """A whole Qwen3 decoder over a paged cache, every operation one call of the scalar reference: float32,
    on the host, one request.  ``pages`` names the pages the request's blocks lie on, in order."""

    def __init__(self, weights, config, pages, page_tokens=16):
        self.c = dict(config)
        self.c.setdefault("head_dim", self.c["hidden_size"] // self.c["num_attention_heads"])
        self.w = {k: f32(v.float().numpy()) for k, v in weights.items()}
        c = self.c
        self.layers = []
        for layer in range(c["num_hidden_layers"]):
            p = f"model.layers.{layer}"
            self.layers.append(dict(
                norm1=self.w[f"{p}.input_layernorm.weight"], norm2=self.w[f"{p}.post_attention_layernorm.weight"],
                qkv=np.concatenate([self.w[f"{p}.self_attn.{n}_proj.weight"] for n in "qkv"], axis=0),
                o=self.w[f"{p}.self_attn.o_proj.weight"], q_gain=self.w[f"{p}.self_attn.q_norm.weight"],
                k_gain=self.w[f"{p}.self_attn.k_norm.weight"],
                gate_up=f32(interleave_gate_up(self.w[f"{p}.mlp.gate_proj.weight"], self.w[f"{p}.mlp.up_proj.weight"])),
                down=self.w[f"{p}.mlp.down_proj.weight"]))
        self.page_tokens = page_tokens
        self.table = i32([list(pages)])
        n_pages, kv, d = max(pages) + 1, c["num_key_value_heads"], c["head_dim"]
        self.pools = [(np.full((n_pages, kv, d // 8, page_tokens, 8), np.nan, dtype=np.float32),
                       np.full((n_pages, kv, page_tokens // 8, d, 8), np.nan, dtype=np.float32))
                      for _ in range(c["num_hidden_layers"])]
        self.cos, self.sin = rope_table(c["rope_theta"], d, c["max_position_embeddings"])
        self.length = 0

    def step(self, tokens):
        """Feeds the next tokens of the request; returns the logits of all of them, float32 [n, vocab]."""
        c = self.c
        n = len(tokens)
        positions = np.arange(self.length, self.length + n, dtype=np.int32)
        entry = np.zeros(n, dtype=np.int32)
        heads, kv, d, eps = c["num_attention_heads"], c["num_key_value_heads"], c["head_dim"], c["rms_norm_eps"]
        x = embed(self.w["model.embed_tokens.weight"], tokens)
        pending = None
        for layer, (k_pool, v_pool) in zip(self.layers, self.pools):
            y = add_rmsnorm(x, pending, layer["norm1"], eps)
            q = qk_norm_rope_write(gemm(y, layer["qkv"]), heads, kv, d, layer["q_gain"], layer["k_gain"], eps, self.cos,
                                   self.sin, positions, entry, self.table, k_pool, v_pool)
            attended = attention(q, k_pool, v_pool, positions, entry, self.table, heads, 1.0 / np.sqrt(np.float32(d)))
            y = add_rmsnorm(x, gemm(attended, layer["o"]), layer["norm2"], eps)
            pending = gemm(swiglu(gemm(y, layer["gate_up"])), layer["down"])
        y = add_rmsnorm(x, pending, self.w["model.norm.weight"], eps)
        head = self.w["model.embed_tokens.weight"] if c.get("tie_word_embeddings", False) else self.w["lm_head.weight"]
        self.length += n
        return gemm(y, head)

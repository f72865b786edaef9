"""Tensor-level wrappers over the HIP entry points.

Each wrapper checks device, type, shape and contiguity on the host before the
launch, because a kernel that reads outside its operands can take the whole
GPU down.  Tensors must live on the GPU: there is no CPU path.
"""
from __future__ import annotations

from typing import Optional

import functools
import math
import threading
import weakref

import numpy as np
import torch

from . import profile
from .library import KernelError, call, library

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}


def _code(t: torch.Tensor, what: str) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise KernelError(f"{what}: element type {t.dtype} is not float32 or bfloat16") from None


def _dev(t: Optional[torch.Tensor], what: str, dtype=None, shape=None) -> int:
    """Checks one operand and returns its device address (0 for None)."""
    if t is None:
        return 0
    if not t.is_cuda:
        raise KernelError(f"{what}: tensor is on {t.device}; the kernels run on the GPU only")
    if not t.is_contiguous():
        raise KernelError(f"{what}: tensor must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{what}: expected {dtype}, found {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{what}: expected shape {tuple(shape)}, found {tuple(t.shape)}")
    return t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


_held = threading.local()                # .stream inside ``one_stream``: the handle that was current when it began


def _stream() -> int:
    """The current stream's handle.  Asked for before every launch, so the short way is taken where this
    torch has it (a tenth of the time of building a Stream object); within ``one_stream`` it was asked for once."""
    held = getattr(_held, "stream", None)
    if held is not None:
        return held
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


class one_stream:
    """Within this context every launch of this thread goes to the stream that is current at its beginning: the
    few hundred launches of a step need not ask for it one by one (0.4 ms of the 4 ms the host takes to issue a
    step of the 8B shape).  Whoever changes the current stream inside (a graph capture does) opens a context of
    its own.  The handle is kept per thread, as torch keeps the current stream: engines that step side by side
    in threads of their own, each on its stream, do not see each other's."""

    def __enter__(self):
        self._before = getattr(_held, "stream", None)
        _held.stream = None
        _held.stream = _stream()
        return self

    def __exit__(self, *exc):
        _held.stream = self._before
        return False


def cache_dims(k_pool: torch.Tensor, v_pool: torch.Tensor):
    """(pages, kv_heads, page_tokens, head_dim) of a key/value pool pair in the packed cache layout:
    keys ``[pages, kv_heads, head_dim/8, page_tokens, 8]``, values ``[pages, kv_heads, page_tokens/8, head_dim, 8]``."""
    if k_pool.dim() != 5 or k_pool.shape[4] != 8:
        raise KernelError(f"key pool must be [pages, kv_heads, head_dim/8, page_tokens, 8], found {tuple(k_pool.shape)}")
    pages, kv_heads, d8, page_tokens, _ = k_pool.shape
    if page_tokens % 8 or tuple(v_pool.shape) != (pages, kv_heads, page_tokens // 8, d8 * 8, 8):
        raise KernelError(f"value pool must be [pages, kv_heads, page_tokens/8, head_dim, 8] matching the key pool "
                          f"{tuple(k_pool.shape)}, found {tuple(v_pool.shape)}")
    return pages, kv_heads, page_tokens, d8 * 8


def pack_keys(k: torch.Tensor) -> torch.Tensor:
    """[..., tokens, head_dim] -> the packed page layout [..., head_dim/8, tokens, 8]."""
    *lead, tokens, dim = k.shape
    return k.reshape(*lead, tokens, dim // 8, 8).transpose(-3, -2).contiguous()


def pack_values(v: torch.Tensor) -> torch.Tensor:
    """[..., tokens, head_dim] -> the packed page layout [..., tokens/8, head_dim, 8]."""
    *lead, tokens, dim = v.shape
    return v.reshape(*lead, tokens // 8, 8, dim).transpose(-2, -1).contiguous()


def embed(table: torch.Tensor, tokens: torch.Tensor, out: Optional[torch.Tensor] = None,
          scale: float = 1.0) -> torch.Tensor:
    """out[r] = table[tokens[r]] * scale as float32.  Token ids must have been checked against the table."""
    vocab, hidden = table.shape
    rows = tokens.numel()
    if out is None:
        out = torch.empty((rows, hidden), dtype=torch.float32, device=table.device)
    call("leone_embed", _dev(table, "embed table"), _code(table, "embed table"),
         _dev(tokens, "embed tokens", torch.int32, (rows,)), _dev(out, "embed out", torch.float32, (rows, hidden)),
         rows, hidden, vocab, float(scale), _stream())
    return out


def soft_cap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x = cap * tanh(x / cap), in place (float32)."""
    call("leone_soft_cap", _dev(x, "soft_cap values", torch.float32), x.numel(), float(cap), _stream())
    return x


def add_rmsnorm(x: torch.Tensor, delta: Optional[torch.Tensor], gain: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None, prepare: bool = False):
    """x += delta, then y = rmsnorm(x) * gain; with ``rows``, y[i] comes from row rows[i] and x is not written.
    ``delta`` is [n, hidden] or a stack of planes [p, n, hidden] whose sum, taken in order, is meant (the
    parts of a product whose inner dimension was cut, see ``linear``).  With ``prepare`` the norm is left for
    the product that consumes it to finish: ``PreparedRows`` comes back (the operand x * gain, and the rows'
    sums of squares), which rounds where the product with the norm folded in rounds."""
    n, hidden = x.shape
    n_out = n if rows is None else rows.numel()
    if out is None:
        out = torch.empty((n_out, hidden), dtype=out_dtype, device=x.device)
    squares = torch.empty((n_out, -(-hidden // 16)), dtype=torch.float32, device=x.device) if prepare else None
    delta_code = _code(delta, "add_rmsnorm delta") if delta is not None else _CODES[out_dtype]
    stacked = delta is not None and delta.dim() == 3
    planes = delta.shape[0] if stacked else 1
    if not 1 <= planes <= 16:
        raise KernelError(f"add_rmsnorm: {planes} planes of what is to be added")
    call("leone_add_rmsnorm", _dev(x, "add_rmsnorm x", torch.float32),
         _dev(delta, "add_rmsnorm delta", None, (planes, n, hidden) if stacked else (n, hidden)), delta_code, planes,
         n * hidden,
         _dev(gain, "add_rmsnorm gain", None, (hidden,)), _code(gain, "add_rmsnorm gain"), float(eps),
         _dev(out, "add_rmsnorm out", out_dtype, (n_out, hidden)), _CODES[out_dtype],
         _dev(rows, "add_rmsnorm rows", torch.int32), n_out, hidden, _dev(squares, "add_rmsnorm sums"), _stream())
    return PreparedRows(x, gain, eps, out_dtype, out, squares, rows) if prepare else out


def swiglu(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    rows, twice = gate_up.shape
    if twice % 2:
        raise KernelError("swiglu: input width must be even (gate columns, then up columns)")
    ffn = twice // 2
    if out is None:
        out = torch.empty((rows, ffn), dtype=gate_up.dtype, device=gate_up.device)
    call("leone_swiglu", _dev(gate_up, "swiglu in"), _dev(out, "swiglu out", gate_up.dtype, (rows, ffn)),
         _code(gate_up, "swiglu in"), rows, ffn, _stream())
    return out


def rope_table(theta: float, rotary_dim: int, positions: int, device) -> tuple[torch.Tensor, torch.Tensor]:
    cos = torch.empty((positions, rotary_dim // 2), dtype=torch.float32, device=device)
    sin = torch.empty_like(cos)
    call("leone_rope_table", _dev(cos, "rope cos"), _dev(sin, "rope sin"), float(theta), rotary_dim, positions,
         _stream())
    return cos, sin


PAIRINGS = {"half_split": 0, "adjacent": 1}   # which two elements of a head a rotation turns together


def _rotation_shape(what: str, head_dim: int, cos, sin, pairing: str):
    """(table positions, rotary_dim, pairing code) of a rotation given as cos/sin tables ``[positions,
    rotary_dim / 2]``: the head's first ``rotary_dim`` elements are rotated, in pairs (i, i + rotary_dim / 2)
    ("half_split") or (2 i, 2 i + 1) ("adjacent") (crates/leone/src/cpu.rs:1765-1774); the rest is left as it is."""
    if pairing not in PAIRINGS:
        raise KernelError(f"{what}: unknown pairing {pairing!r}; known: {', '.join(PAIRINGS)}")
    if cos is None:
        return 0, 0, PAIRINGS[pairing]
    if sin is None or sin.shape != cos.shape or cos.dim() != 2:
        raise KernelError(f"{what}: cos and sin tables must both be [positions, rotary_dim / 2]")
    rotary_dim = 2 * cos.shape[1]
    if not 0 < rotary_dim <= head_dim:
        raise KernelError(f"{what}: the rotary tables cover {rotary_dim} elements, a head has {head_dim}")
    return cos.shape[0], rotary_dim, PAIRINGS[pairing]


def decode_projected_supported(head_dim: int, rotary_dim: int = 0, pairing: str = "half_split") -> bool:
    """Whether ``attention_decode_projected`` takes this head and rotation: head sizes that are multiples of
    64, no rotation (``rotary_dim`` 0) or the half-split one over the whole head."""
    return head_dim % 64 == 0 and (rotary_dim == 0 or (rotary_dim == head_dim and pairing == "half_split"))


def qk_norm_rope_write(qkv: torch.Tensor, q_heads: int, kv_heads: int, head_dim: int,
                       q_gain: Optional[torch.Tensor], k_gain: Optional[torch.Tensor], eps: float,
                       cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], positions: torch.Tensor,
                       row_entry: Optional[torch.Tensor], block_table: Optional[torch.Tensor],
                       k_pool: Optional[torch.Tensor], v_pool: Optional[torch.Tensor], write_cache: bool = True,
                       out: Optional[torch.Tensor] = None, out_dtype: Optional[torch.dtype] = None,
                       pairing: str = "half_split") -> torch.Tensor:
    """Splits the fused projection, normalises and rotates q and k heads, writes k and v into the cache.
    ``qkv`` is ``[rows, width]`` of the cache's type, or float32 (also as planes ``[p, rows, width]`` whose
    sum, in order, is meant: a product cut along K) with ``out_dtype`` naming the type of q and the cache.
    The rotation's shape comes with its tables (``_rotation_shape``): their width says how much of a head is
    rotated, ``pairing`` which elements go together."""
    planes = qkv.shape[0] if qkv.dim() == 3 else 1
    rows, width = qkv.shape[-2:]
    kind = out_dtype or qkv.dtype
    if qkv.dtype != kind and qkv.dtype != torch.float32:
        raise KernelError(f"qk_norm_rope_write: input {qkv.dtype} for outputs of {kind}")
    if width != (q_heads + 2 * kv_heads) * head_dim:
        raise KernelError(f"qk_norm_rope_write: width {width} is not ({q_heads}+2*{kv_heads})*{head_dim}")
    if out is None:
        out = torch.empty((rows, q_heads * head_dim), dtype=kind, device=qkv.device)
    max_blocks = page_tokens = 0
    if write_cache:
        if k_pool is None or v_pool is None or block_table is None or row_entry is None:
            raise KernelError("qk_norm_rope_write: a cache write needs pools, a block table and a row map")
        pages, pool_heads, page_tokens, pool_dim = cache_dims(k_pool, v_pool)
        if (pool_heads, pool_dim) != (kv_heads, head_dim):
            raise KernelError(f"qk_norm_rope_write: pool shape {tuple(k_pool.shape)} does not fit "
                              f"{kv_heads} heads of {head_dim}")
        max_blocks = block_table.shape[1]
    table_positions, rotary_dim, pairing_code = _rotation_shape("qk_norm_rope_write", head_dim, cos, sin, pairing)
    gain_code = _code(q_gain, "q gain") if q_gain is not None else F32
    if q_gain is not None and (k_gain is None or k_gain.dtype != q_gain.dtype):
        raise KernelError("qk_norm_rope_write: q and k gains must come together in one type")
    call("leone_qk_norm_rope_write", _dev(qkv, "qkv"), _code(qkv, "qkv"), planes, rows * width,
         _dev(out, "q out", kind),
         _dev(k_pool if write_cache else None, "k pool", kind),
         _dev(v_pool if write_cache else None, "v pool", kind), _CODES[kind],
         _dev(q_gain, "q gain", None, (head_dim,)), _dev(k_gain, "k gain", None, (head_dim,)), gain_code,
         float(eps), _dev(cos, "rope cos", torch.float32), _dev(sin, "rope sin", torch.float32), table_positions,
         rotary_dim, pairing_code, _dev(positions, "positions", torch.int32, (rows,)),
         _dev(row_entry if write_cache else None, "row map", torch.int32, (rows,)),
         _dev(block_table if write_cache else None, "block table", torch.int32), max_blocks, rows, q_heads,
         kv_heads, head_dim, page_tokens, 1 if write_cache else 0, _stream())
    return out


def attention_rows(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, positions: torch.Tensor,
                   row_entry: torch.Tensor, block_table: torch.Tensor, q_heads: int, scale: float,
                   window: int = 0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Each query row attends its request's cached keys up to its own position."""
    rows = q.shape[0]
    pages, kv_heads, page_tokens, head_dim = cache_dims(k_pool, v_pool)
    if q.shape[1] != q_heads * head_dim:
        raise KernelError(f"attention: query width {q.shape[1]} is not {q_heads}*{head_dim}")
    if out is None:
        out = torch.empty_like(q)
    call("leone_attention_rows", _dev(q, "attention q"), _dev(out, "attention out", q.dtype, q.shape),
         _dev(k_pool, "k pool", q.dtype), _dev(v_pool, "v pool", q.dtype), _code(q, "attention q"),
         _dev(positions, "positions", torch.int32, (rows,)), _dev(row_entry, "row map", torch.int32, (rows,)),
         _dev(block_table, "block table", torch.int32), block_table.shape[1], rows, q_heads, kv_heads, head_dim,
         page_tokens, float(scale), int(window), _stream())
    return out


def decode_attention_supported(dtype: torch.dtype, head_dim: int, page_tokens: int, group: int = 1,
                               max_blocks: int = 0) -> bool:
    """Whether the matrix-core kernel takes this case; otherwise ``attention_rows`` does."""
    cols = min(group, 16)
    shared = (4 * cols * head_dim + 8 * cols) * 4 + 4 * max_blocks   # the four waves' partial results, page ids
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= 256 and shared <= 64 * 1024
            and page_tokens >= 16 and page_tokens & (page_tokens - 1) == 0)


DECODE_SPLIT_START_TILES = 8   # what starting a workgroup of the split-KV kernel costs, in 32-key tiles


def choose_splits(rows: int, kv_heads: int, group: int, max_context: int, units: int = 256) -> int:
    """Into how many parts the keys of a row are cut: the number (up to 32, at least four 32-key tiles a part,
    one for each of a workgroup's waves) for which the compute unit with the most workgroups has the least to
    do: ceil(workgroups / units) x (tiles a part + a start worth 8 tiles).  Measured in whole decode steps at
    8,192 keys, 1 to 48 rows, against a fixed aim of one or two workgroups a unit: level where those do well
    (1, 8, 12, 17 rows) and up to 15 % of a step better where their workgroup counts leave units idle or a few
    with one workgroup more than the rest (24 rows: 8.67 ms against 9.18, 40 rows: 11.8 against 13.9)."""
    blocks = rows * kv_heads * ((group + 15) // 16)
    tiles = (max_context + 31) // 32
    best = None
    for splits in range(1, min(32, max(1, tiles // 4)) + 1):
        cost = (-(-blocks * splits // units) * (-(-tiles // splits) + DECODE_SPLIT_START_TILES), splits)
        if best is None or cost < best:
            best = cost
    return best[1]


def attention_decode(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, positions: torch.Tensor,
                     row_entry: torch.Tensor, block_table: torch.Tensor, q_heads: int, scale: float,
                     window: int = 0, max_context: int = 1, splits: Optional[int] = None,
                     out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Split-KV attention on the matrix cores (bfloat16).  ``max_context`` only steers the number of splits."""
    rows = q.shape[0]
    pages, kv_heads, page_tokens, head_dim = cache_dims(k_pool, v_pool)
    if q.shape[1] != q_heads * head_dim:
        raise KernelError(f"attention: query width {q.shape[1]} is not {q_heads}*{head_dim}")
    if splits is None:
        splits = choose_splits(rows, kv_heads, q_heads // kv_heads, max_context, compute_units(q.device))
    if out is None:
        out = torch.empty_like(q)
    part_acc = part_ml = None
    if splits > 1:
        part_acc = torch.empty((rows * q_heads * splits * head_dim,), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((rows * q_heads * splits * 2,), dtype=torch.float32, device=q.device)
    call("leone_attention_decode", _dev(q, "attention q", torch.bfloat16),
         _dev(out, "attention out", torch.bfloat16, q.shape), _dev(k_pool, "k pool", torch.bfloat16),
         _dev(v_pool, "v pool", torch.bfloat16), _dev(positions, "positions", torch.int32, (rows,)),
         _dev(row_entry, "row map", torch.int32, (rows,)), _dev(block_table, "block table", torch.int32),
         block_table.shape[1], _dev(part_acc, "partials"), _dev(part_ml, "partial sums"), rows, q_heads, kv_heads,
         head_dim, page_tokens, float(scale), int(window), int(splits), _stream())
    return out


def attention_decode_projected(qkv: torch.Tensor, q_heads: int, kv_heads: int, head_dim: int,
                               q_gain: Optional[torch.Tensor], k_gain: Optional[torch.Tensor], eps: float,
                               cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], k_pool: torch.Tensor,
                               v_pool: torch.Tensor, positions: torch.Tensor, row_entry: torch.Tensor,
                               block_table: torch.Tensor, scale: float, window: int = 0, max_context: int = 1,
                               splits: Optional[int] = None, write_cache: bool = True,
                               pairing: str = "half_split") -> torch.Tensor:
    """``qk_norm_rope_write`` and ``attention_decode`` in one launch, for a step in which every row is another
    request (single decoded tokens): the kernel takes the fused q/k/v projection (bfloat16 ``[rows, width]``, or
    float32 planes ``[p, rows, width]``), makes queries and the new key itself and writes key and value into
    the cache before it reads the keys.  Head sizes that are multiples of 64."""
    planes = qkv.shape[0] if qkv.dim() == 3 else 1
    rows, width = qkv.shape[-2:]
    pages, pool_heads, page_tokens, pool_dim = cache_dims(k_pool, v_pool)
    if (pool_heads, pool_dim) != (kv_heads, head_dim) or width != (q_heads + 2 * kv_heads) * head_dim:
        raise KernelError(f"attention_decode_projected: width {width} and pool {tuple(k_pool.shape)} do not fit "
                          f"{q_heads}+2*{kv_heads} heads of {head_dim}")
    if head_dim % 64:
        raise KernelError(f"attention_decode_projected: head size {head_dim} is no multiple of 64")
    table_positions, rotary_dim, pairing_code = _rotation_shape("attention_decode_projected", head_dim, cos, sin, pairing)
    if not decode_projected_supported(head_dim, rotary_dim, pairing):
        raise KernelError(f"attention_decode_projected: the kernel rotates whole heads in half-split pairs, not "
                          f"{rotary_dim} of {head_dim} elements in {pairing} pairs (qk_norm_rope_write and "
                          f"attention_decode take those)")
    if q_gain is not None and (k_gain is None or k_gain.dtype != q_gain.dtype):
        raise KernelError("attention_decode_projected: q and k gains must come together in one type")
    if splits is None:
        splits = choose_splits(rows, kv_heads, q_heads // kv_heads, max_context, compute_units(qkv.device))
    out = torch.empty((rows, q_heads * head_dim), dtype=torch.bfloat16, device=qkv.device)
    part_acc = part_ml = None
    if splits > 1:
        part_acc = torch.empty((rows * q_heads * splits * head_dim,), dtype=torch.float32, device=qkv.device)
        part_ml = torch.empty((rows * q_heads * splits * 2,), dtype=torch.float32, device=qkv.device)
    call("leone_attention_decode_projected", _dev(qkv, "qkv"), _code(qkv, "qkv"), planes, rows * width,
         _dev(q_gain, "q gain", None, (head_dim,)), _dev(k_gain, "k gain", None, (head_dim,)),
         _code(q_gain, "q gain") if q_gain is not None else F32, float(eps),
         _dev(cos, "rope cos", torch.float32), _dev(sin, "rope sin", torch.float32), table_positions, rotary_dim,
         pairing_code, _dev(out, "attention out"), _dev(k_pool, "k pool", torch.bfloat16), _dev(v_pool, "v pool", torch.bfloat16),
         1 if write_cache else 0, _dev(positions, "positions", torch.int32, (rows,)),
         _dev(row_entry, "row map", torch.int32, (rows,)), _dev(block_table, "block table", torch.int32),
         block_table.shape[1], _dev(part_acc, "partials"), _dev(part_ml, "partial sums"), rows, q_heads, kv_heads,
         head_dim, page_tokens, float(scale), int(window), int(splits), _stream())
    return out


PREFILL_TILE_ROWS = 32       # rows of one request a wave of the prompt kernel takes (checked against the library)
PREFILL_GROUP_TILES = 4      # tiles of one request a workgroup of the prompt kernel takes (likewise)
PREFILL_MIN_ROWS = 16        # shorter portions go through the split-KV kernel row by row
PREFILL_MAX_SPLITS = 32      # most key ranges the prompt kernel takes (checked against the library)
PREFILL_SPLIT_MIN_STAGES = 4 # a key range of the prompt kernel keeps at least this many 64-key stages
PREFILL_SPLIT_START_STAGES = 8   # what a workgroup of the prompt kernel costs before its first stage, in stages
PREFILL_SPLIT_MERGE_STAGES = 6   # what writing and merging a range's partial results adds, in stages


def prefill_attention_supported(dtype: torch.dtype, head_dim: int, page_tokens: int, max_blocks: int = 0) -> bool:
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= 128
            and 16 * max_blocks <= 64 * 1024                      # the page ids of four waves' keys
            and page_tokens >= 16 and page_tokens & (page_tokens - 1) == 0)


def choose_prefill_splits(groups: int, q_heads: int, mean_keys: int, window: int = 0, units: int = 256) -> int:
    """How many ranges the keys of a prompt workgroup are cut into, where a row sees ``mean_keys`` keys: the
    number (a range keeps at least PREFILL_SPLIT_MIN_STAGES stages of 64 keys) for which the rounds of
    workgroups over the chip (two fit a compute unit) x (stages a range + the start, + the merge where there
    is more than one range) come out least.  Measured in whole
    steps on portions of 128 to 1,536 rows after 30,720 positions against a fixed aim of two workgroups a unit:
    level for 256, 512 and 1,024 rows, 28.9 against 30.2 ms for 768 rows, 51.3 against 54.4 for 1,536.  (A
    prompt from position 0 gains nothing from ranges, its early rows see few keys: without the merge's term
    the rule took two ranges for 1,024 and 3,072 rows and lost 3 and 4 % of the step by it.)"""
    reach = PREFILL_GROUP_TILES * PREFILL_TILE_ROWS
    keys = min(mean_keys, window + reach) if window > 0 else mean_keys
    stages = -(-keys // 64)
    blocks = max(1, groups * q_heads)
    best = None
    for splits in range(1, min(PREFILL_MAX_SPLITS, max(1, stages // PREFILL_SPLIT_MIN_STAGES)) + 1):
        each = -(-stages // splits) + PREFILL_SPLIT_START_STAGES + (PREFILL_SPLIT_MERGE_STAGES if splits > 1 else 0)
        cost = (-(-blocks * splits // (2 * units)) * each, splits)
        if best is None or cost < best:
            best = cost
    return best[1]


def attention_prefill(q: torch.Tensor, out: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                      positions: torch.Tensor, tiles: torch.Tensor, block_table: torch.Tensor, q_heads: int,
                      scale: float, window: int = 0, mean_keys: int = 1, splits: Optional[int] = None,
                      covered_rows: Optional[int] = None) -> torch.Tensor:
    """Attention for the rows that ``tiles`` covers; writes into ``out``.

    ``tiles`` is int32 [n, 3]: (entry, first row, rows) with at most PREFILL_TILE_ROWS consecutive rows of one
    request each, PREFILL_GROUP_TILES to a group, all tiles of a group of the same entry, unused places with
    0 rows (``prefill_tiles`` builds such a list).  ``mean_keys`` (keys a row sees on average) only steers
    the number of key ranges (``splits``); ``covered_rows``: one more than the last row a tile names, if the
    caller knows it."""
    if (library().leone_attention_prefill_tile_rows() != PREFILL_TILE_ROWS
            or library().leone_attention_prefill_group_tiles() != PREFILL_GROUP_TILES
            or library().leone_attention_prefill_max_splits() != PREFILL_MAX_SPLITS):
        raise KernelError("the kernel library was built for another prompt tile size")
    rows = q.shape[0]
    pages, kv_heads, page_tokens, head_dim = cache_dims(k_pool, v_pool)
    if q.shape[1] != q_heads * head_dim:
        raise KernelError(f"attention: query width {q.shape[1]} is not {q_heads}*{head_dim}")
    if tiles.dim() != 2 or tiles.shape[1] != 3 or tiles.shape[0] % PREFILL_GROUP_TILES:
        raise KernelError(f"attention_prefill: tiles must be int32 [n, 3] with n a multiple of {PREFILL_GROUP_TILES}")
    groups = tiles.shape[0] // PREFILL_GROUP_TILES
    if splits is None:
        splits = choose_prefill_splits(groups, q_heads, mean_keys, window, compute_units(q.device))
    part_acc = part_ml = None
    if splits > 1:
        covered = rows if covered_rows is None else covered_rows
        if not 0 < covered <= rows:
            raise KernelError(f"attention_prefill: {covered} covered rows of {rows}")
        part_acc = torch.empty((covered * q_heads * splits * head_dim,), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((covered * q_heads * splits * 2,), dtype=torch.float32, device=q.device)
    call("leone_attention_prefill", _dev(q, "attention q", torch.bfloat16),
         _dev(out, "attention out", torch.bfloat16, q.shape), _dev(k_pool, "k pool", torch.bfloat16),
         _dev(v_pool, "v pool", torch.bfloat16), _dev(positions, "positions", torch.int32, (rows,)),
         _dev(tiles, "tiles", torch.int32), groups, _dev(block_table, "block table", torch.int32),
         block_table.shape[1], q_heads, kv_heads, head_dim, page_tokens, float(scale), int(window),
         _dev(part_acc, "partials"), _dev(part_ml, "partial sums"), int(splits), _stream())
    return out


def prefill_tiles(portions) -> torch.Tensor:
    """The tile list of ``attention_prefill`` for portions given as (entry, first row, rows): tiles in order,
    every portion's last group filled up with unused places (as the native step layout lists a step's own)."""
    tiles = []
    for entry, first_row, rows in portions:
        mine = [(entry, first_row + at, min(PREFILL_TILE_ROWS, rows - at)) for at in range(0, rows, PREFILL_TILE_ROWS)]
        mine += [(entry, first_row, 0)] * (-len(mine) % PREFILL_GROUP_TILES)
        tiles += mine
    return torch.tensor(tiles, dtype=torch.int32).view(-1, 3)


def gemm_f32(a: torch.Tensor, b: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """a[M,K] . b[N,K]^T in true single precision."""
    m, k = a.shape
    n, k2 = b.shape
    if k != k2:
        raise KernelError(f"gemm_f32: inner sizes {k} and {k2} differ")
    if out is None:
        out = torch.empty((m, n), dtype=torch.float32, device=a.device)
    with profile.span("gemm f32", b):
        call("leone_gemm_f32", _dev(a, "gemm a", torch.float32), _dev(b, "gemm b", torch.float32),
             _dev(out, "gemm out", torch.float32, (m, n)), m, n, k, _stream())
    return out


# Up to here norm, gate and residual are folded into the weight-streaming kernel for few rows; beyond, the
# multi-row kernel runs with the row-wise kernels between.  Measured in whole decode steps at the 8B layer sizes
# with the second copies of the weights (ms a step, folded : multi-row): 5.98 : 6.40 at 11 rows, 6.17 : 6.47 at
# 12, 6.51 : 6.66 at 14, level at 16, which is all the kernel takes.  (With row-major weights only, the folded
# kernel's reads of X weighed more and the two crossed between 10 and 11 rows.)
FUSED_ROWS = 16
FUSED_NORM_WEIGHT_ROWS = 1024   # a norm is folded into the product only for weights of at most this many rows


class NormedRows:
    """Rows of the float32 stream that are to be RMS-normalised: a norm not yet carried out, so that
    the product that consumes it can fold it in.  ``rows`` (int32 indices) picks rows of ``x``."""

    def __init__(self, x: torch.Tensor, gain: torch.Tensor, eps: float, dtype: torch.dtype,
                 rows: Optional[torch.Tensor] = None):
        self.x, self.gain, self.eps, self.dtype, self.rows = x, gain, float(eps), dtype, rows
        self.shape = (x.shape[0] if rows is None else rows.numel(), x.shape[1])

    def materialize(self) -> torch.Tensor:
        return add_rmsnorm(self.x, None, self.gain, self.eps, self.dtype, self.rows)

    def prepare(self) -> "PreparedRows":
        """The norm kernel runs, but leaves the scaling to the product (see ``add_rmsnorm``)."""
        return add_rmsnorm(self.x, None, self.gain, self.eps, self.dtype, self.rows, prepare=True)


class PreparedRows(NormedRows):
    """A norm of the stream ``x`` (of its rows ``rows``) whose operand lies ready: ``operand`` is
    bf16(x * gain), ``squares`` float32 ``[rows, ceil(hidden / 16)]`` partial sums of x^2.  The product before
    leaves them behind (``linear(..., next_norm=)``), so that the product that consumes them needs no norm
    kernel and no second read of the stream; or the norm kernel does (``add_rmsnorm(..., prepare=True)``).  The stream itself is
    up to date: any other consumer normalises it in the usual way (``materialize``)."""

    def __init__(self, x: torch.Tensor, gain: torch.Tensor, eps: float, dtype: torch.dtype,
                 operand: torch.Tensor, squares: torch.Tensor, rows: Optional[torch.Tensor] = None):
        super().__init__(x, gain, eps, dtype, rows)
        self.operand, self.squares = operand, squares


def prepared_fits(rows: int, hidden: int) -> bool:
    """Whether ``gemm_fused`` takes rows of this width as ``PreparedRows`` (its sums of squares travel in
    16-byte runs, at most 2,048 of them)."""
    return hidden % 64 == 0 and rows * (hidden // 64) <= 2048


def materialize(x) -> torch.Tensor:
    return x.materialize() if isinstance(x, NormedRows) else x


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """The fused gate/up weight: 8 gate rows, the 8 up rows that belong to them, and so on; the order in
    which ``swiglu`` and the gated product expect the columns of the product."""
    ffn, hidden = gate.shape
    if ffn % 8 or up.shape != gate.shape:
        raise KernelError(f"gate and up must both be [F, H] with F a multiple of 8, found {tuple(gate.shape)}")
    return torch.stack([gate.view(ffn // 8, 8, hidden), up.view(ffn // 8, 8, hidden)], dim=1).reshape(2 * ffn, hidden)


def tile_weight(weight: torch.Tensor) -> torch.Tensor:
    """The copy of ``weight[N, K]`` (bfloat16, K a multiple of 64) that the weight-streaming products read
    fastest: rows in tiles of 16 (the last filled up with zero rows), K in steps of 64, a step in two halves;
    element e of lane 16 g + c in half h of step s of tile t is ``weight[16 t + c][64 s + 16 g + 8 h + e]``, so
    ``[tiles, K / 64, 2, 4, 16, 8]``.  Each load of a wave is then 1 KB in one piece."""
    n, k = weight.shape
    if weight.dtype != torch.bfloat16 or k % 64:
        raise KernelError(f"tile_weight: a bfloat16 matrix with K a multiple of 64 is needed, not {weight.dtype} with K {k}")
    tiles = -(-n // 16)
    if tiles * 16 != n:
        weight = torch.cat([weight, weight.new_zeros((tiles * 16 - n, k))])
    return weight.view(tiles, 16, k // 64, 4, 2, 8).permute(0, 2, 4, 3, 1, 5).contiguous()


_streamed: dict = {}         # (address, shape) of a weight -> (weak reference to the weight, its tiled copy)


def keep_streamed_copy(weight: torch.Tensor) -> int:
    """Makes and keeps the tiled copy of a weight; the products take it from then on whenever they are given
    this weight, and it is dropped when the weight is.  Returns the copy's bytes (0 if the weight's shape or
    type has no tiled form)."""
    if weight.dtype != torch.bfloat16 or weight.dim() != 2 or weight.shape[1] % 64 or not weight.is_cuda:
        return 0
    key = (weight.data_ptr(), tuple(weight.shape))
    held = _streamed.get(key)
    if held is None or held[0]() is not weight:
        def forget(_, key=key):
            _streamed.pop(key, None)
        _streamed[key] = (weakref.ref(weight, forget), tile_weight(weight))
    return _streamed[key][1].numel() * 2


def streamed_copy(weight: torch.Tensor) -> Optional[torch.Tensor]:
    held = _streamed.get((weight.data_ptr(), tuple(weight.shape)))
    return None if held is None or held[0]() is not weight else held[1]


def drop_streamed_copies() -> None:
    _streamed.clear()


def gemm_fused(x, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
               residual: Optional[torch.Tensor] = None, gated: bool = False, next_norm=None):
    """The product for at most 16 rows with its neighbours folded in: ``x`` may be ``NormedRows`` or
    ``PreparedRows``; with ``residual`` the product is added into that float32 tensor and None is returned;
    with ``gated`` the weight is an interleaved gate/up weight and silu(gate) * up comes out.  With
    ``residual`` and ``next_norm = (gain, eps, dtype)`` the kernel also leaves the operand of that norm
    behind and ``PreparedRows`` is returned (the residual has been added)."""
    m, k = x.shape
    n, k2 = weight.shape
    if k != k2:
        raise KernelError(f"gemm_fused: inner sizes {k} and {k2} differ")
    prepared = isinstance(x, PreparedRows)
    normed = isinstance(x, NormedRows) and not prepared
    if residual is not None and gated:
        raise KernelError("gemm_fused: a gated product cannot also be added into the stream")
    if next_norm is not None and residual is None:
        raise KernelError("gemm_fused: the next norm can only be prepared from the stream the product is added into")
    operand = squares = None
    if residual is not None:
        out, mode, out_dtype = residual, 1, torch.float32
        if next_norm is not None:
            mode = 3
            operand = torch.empty((m, n), dtype=torch.bfloat16, device=weight.device)
            squares = torch.empty((m, -(-n // 16)), dtype=torch.float32, device=weight.device)
    elif gated:
        out, mode, out_dtype = torch.empty((m, n // 2), dtype=torch.bfloat16, device=weight.device), 2, torch.bfloat16
    else:
        out, mode = torch.empty((m, n), dtype=out_dtype, device=weight.device), 0
    if prepared:
        source, in_mode = _dev(x.operand, "prepared operand", torch.bfloat16, (m, k)), 2
        _dev(x.squares, "prepared sums", torch.float32, (m, -(-k // 16)))
    elif normed:
        source, in_mode = _dev(x.x, "stream", torch.float32), 1
    else:
        source, in_mode = _dev(x, "gemm x", torch.bfloat16, (m, k)), 0
    tiles = streamed_copy(weight) if _streamed else None
    with profile.span("gemv fused", weight):
        call("leone_gemm_fused_bf16", source, in_mode, _dev(x.rows, "rows", torch.int32) if normed else 0,
             _dev(x.gain, "gain", None, (k,)) if normed else 0, _code(x.gain, "gain") if normed else 0,
             x.eps if (normed or prepared) else 0.0,
             _dev(weight if tiles is None else tiles, "gemm weight", torch.bfloat16), 0 if tiles is None else 1,
             _dev(out, "gemm out", out_dtype, (m, n // 2 if gated else n)), mode, _CODES[out_dtype], m, n, k,
             x.squares.data_ptr() if prepared else 0, _dev(operand, "operand out"), _dev(squares, "sums out"),
             _dev(next_norm[0], "next gain", None, (n,)) if next_norm is not None else 0,
             _code(next_norm[0], "next gain") if next_norm is not None else 0, _stream())
    if next_norm is not None:
        return PreparedRows(residual, next_norm[0], next_norm[1], next_norm[2], operand, squares)
    return None if residual is not None else out


ROWS_MAX = 128               # most rows the multi-row weight-streaming product takes (checked against the library)
ROWS_WAVES = (4, 6, 8)       # workgroup sizes it is built for, in waves (16 weight rows each)
_UNITS = {}


def compute_units(device) -> int:
    index = torch.device(device).index or 0
    if index not in _UNITS:
        _UNITS[index] = torch.cuda.get_device_properties(index).multi_processor_count if torch.cuda.is_available() else 256
    return _UNITS[index]


def rows_plan(m: int, n: int, k: int, may_split: bool, units: int = 256) -> tuple[int, int]:
    """(waves, splits) for ``gemm_rows``: how many waves (tiles of 16 weight rows) a workgroup gets and into
    how many ranges K is cut.  The kernel is fastest with one workgroup on every compute unit and none
    waiting for a second round (6,144 x 4,096 at 64 rows: 18 us with 256 workgroups, 22 with 480, 24 with
    288), so the plan minimises rounds x the longest workgroup's traffic, where a chunk of K costs a
    workgroup its waves' weight tiles plus half of X's tiles (those come from the cache) and starting up
    costs as much as 3,072 elements of K; ties go to fewer ranges, then fewer waves.  The constants were set
    in whole decode steps of 17 to 128 rows at the layer sizes of the 8B, 14B and 32B models (a start of 768
    or 1,536 elements cuts long K's into too many ranges: 8B 8.05 : 7.91 ms a step at 64 rows; a fixed choice
    for matrices of many rows gave the 32B gate/up product 4 waves and four rounds where 8 waves need two:
    21.7 : 20.3 ms at 64 rows)."""
    return _rows_plan(m, n, k, bool(may_split), units, library().leone_gemm_rows_chunk(m), tuple(ROWS_WAVES))


@functools.lru_cache(maxsize=4096)
def _rows_plan(m: int, n: int, k: int, may_split: bool, units: int, chunk: int, waves_offered: tuple) -> tuple[int, int]:
    # the same few problems come back a few hundred times a step: 0.8 ms of a step's 4 on the host without this
    chunks = -(-k // chunk)
    tiles = -(-n // 16)
    x_tiles = -(-m // 16)
    best = None
    for waves in waves_offered:
        groups = -(-tiles // waves)
        for splits in range(1, (min(chunks, 16) if may_split else 1) + 1):
            per = -(-chunks // splits)
            if per * (splits - 1) >= chunks:            # a range would be empty
                continue
            rounds = -(-groups * splits // units)
            cost = (rounds * (per + 3072 // chunk) * (waves + 0.5 * x_tiles), splits, waves)
            if best is None or cost < best:
                best = cost
    return best[2], best[1]


ROWS_WAYS = 2                # most waves that share a tile of the weight in ``gemm_rows``


def rows_ways(m: int, waves: int) -> int:
    """How many waves share each tile of the weight in ``gemm_rows`` (each takes its share of a chunk's units of
    K; their sums are added up in a fixed order at the end): the most the kernel is built with for this many
    rows and tiles, up to ROWS_WAYS."""
    ways = ROWS_WAYS
    while ways > 1 and not library().leone_gemm_rows_shape_built(m, waves, ways):
        ways //= 2
    return ways


def gemm_rows(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
              residual: Optional[torch.Tensor] = None, gated: bool = False, splits: Optional[int] = None,
              waves: Optional[int] = None, may_split: bool = True, ways: Optional[int] = None) -> Optional[torch.Tensor]:
    """The weight-streaming product for up to ROWS_MAX rows of bfloat16 ``x``.  With ``residual`` and one
    range of K the product is added into that float32 tensor (None returned); with ``gated`` the weight is
    an interleaved gate/up weight and silu(gate) * up comes out.  With more than one range of K (``splits``;
    by default what ``rows_plan`` finds best, one if ``may_split`` is false or the product is gated) float32
    planes ``[splits, M, N]`` are returned whose sum, in order, is the product (with ``residual``: for the
    caller to add)."""
    m, k = x.shape
    n, k2 = weight.shape
    if k != k2:
        raise KernelError(f"gemm_rows: inner sizes {k} and {k2} differ")
    if library().leone_gemm_rows_max_rows() != ROWS_MAX:
        raise KernelError("the kernel library was built for another number of rows")
    if not 1 <= m <= ROWS_MAX:
        raise KernelError(f"gemm_rows: {m} rows, the kernel takes 1..{ROWS_MAX}")
    if residual is not None and gated:
        raise KernelError("gemm_rows: a gated product cannot also be added into the stream")
    if splits is None or waves is None:
        plan = rows_plan(m, n, k, may_split and not gated, compute_units(weight.device))
        waves = plan[0] if waves is None else waves
        splits = plan[1] if splits is None else splits
    if ways is None:
        ways = rows_ways(m, int(waves))
    chunks = -(-k // library().leone_gemm_rows_chunk(m))
    splits = max(1, min(int(splits), chunks))
    splits = -(-chunks // -(-chunks // splits))        # no range of K may be empty
    if gated:
        splits = 1
    plane = 0
    if splits > 1:
        out, mode, kind = torch.empty((splits, m, n), dtype=torch.float32, device=weight.device), 3, torch.float32
        plane = m * n
    elif residual is not None:
        out, mode, kind = residual, 1, torch.float32
        _dev(out, "gemm_rows stream", torch.float32, (m, n))
    elif gated:
        out, mode, kind = torch.empty((m, n // 2), dtype=torch.bfloat16, device=weight.device), 2, torch.bfloat16
    else:
        out, mode, kind = torch.empty((m, n), dtype=out_dtype, device=weight.device), 0, out_dtype
    tiles = streamed_copy(weight) if _streamed else None
    with profile.span("gemm rows", weight):
        call("leone_gemm_rows_bf16", _dev(x, "gemm x", torch.bfloat16, (m, k)),
             _dev(weight if tiles is None else tiles, "gemm weight", torch.bfloat16), 0 if tiles is None else 1,
             _dev(out, "gemm out", kind), mode, _CODES[kind], m, n, k,
             splits, plane, int(waves), int(ways), _stream())
    return None if (residual is not None and splits == 1) else out


def inner_parts(rows: int, n: int, k: int) -> int:
    """Into how many parts the inner dimension of x[rows, k] . w[n, k]^T is cut when the result goes into the
    float32 stream.  The library's product does badly with a few hundred rows, few columns and a long inner
    dimension (the down projection of a prompt portion: 81 us whole against 64 in four parts for 512 x 4096 x
    12288, 171 against 97 for 512 x 5120 x 17408, 55 against 32 for 96 x 4096 x 12288); beyond 1,024 rows
    and up to 64 it is best left whole."""
    if not (64 < rows <= 1024 and k >= 8192 and k >= 2 * n):
        return 1
    for parts in ((4, 2) if rows <= 512 else (2,)):
        if k % (64 * parts) == 0:
            return parts
    return 1


# ---- the vendor library's product with a measured choice of its algorithm -------------------------------------
_tuned_products: set = set()     # (device index, m, n, k, output code, accumulate) of the problems tuned
_recorded_products = None        # while ``record_library_products`` runs: problem -> weights it was asked with


class record_library_products:
    """Within this context ``linear`` notes every product that it hands to the vendor library: the problem
    (rows, weight rows, inner size, output type, whether it adds into the stream) and the weights it came with.
    ``problems`` maps each problem to its weights afterwards."""

    def __enter__(self):
        global _recorded_products
        self.problems: dict = {}
        self._before = _recorded_products
        _recorded_products = self.problems
        return self

    def __exit__(self, *exc):
        global _recorded_products
        _recorded_products = self._before
        return False


def _library_problem(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype, accumulate: bool):
    return (x.device.index or 0, x.shape[0], weight.shape[0], weight.shape[1], F32 if out_dtype == torch.float32 else BF16,
            1 if accumulate else 0)


def library_product_available() -> bool:
    return bool(library().leone_library_product_available())


def tune_library_product(rows: int, weights, out_dtype: torch.dtype, accumulate: bool, candidates: int = 256,
                         thorough: bool = False) -> dict:
    """Times the vendor library's algorithms for ``[rows, K] . W^T`` on ``weights`` (matrices of one shape, taken
    in turn as a model's layers are; ``candidates`` from the library's heuristic, with ``thorough`` every
    algorithm the library has) and keeps the fastest for ``linear`` to use on exactly this problem, after
    checking its result against a float32 product: it must be no further from it than twice what the library's
    ordinary call is.  Returns the problem, the microseconds of the library's own choice and of the winner, and
    how many algorithms were timed; ``kept`` is False if the winner failed the check and was dropped."""
    weights = list(weights)
    weight = weights[0]
    n, k = weight.shape
    if any(w.shape != weight.shape or w.dtype != torch.bfloat16 or not w.is_contiguous() for w in weights):
        raise KernelError("tune_library_product: the weights must be contiguous bfloat16 matrices of one shape")
    if accumulate and out_dtype != torch.float32:
        raise KernelError("tune_library_product: adding into the stream is a float32 product")
    generator = torch.Generator(device=weight.device).manual_seed(rows * 31 + n)
    x = torch.randn((rows, k), device=weight.device, generator=generator).to(torch.bfloat16)
    y = torch.zeros((rows, n), dtype=out_dtype, device=weight.device)
    import ctypes
    pointers = (ctypes.c_void_p * len(weights))(*[w.data_ptr() for w in weights])
    first, best, timed = ctypes.c_float(), ctypes.c_float(), ctypes.c_int()
    out_code = F32 if out_dtype == torch.float32 else BF16
    call("leone_library_product_tune", _dev(x, "x", torch.bfloat16), pointers, len(weights), _dev(y, "y"), rows, n, k,
         out_code, 1 if accumulate else 0, int(candidates), 1 if thorough else 0, ctypes.byref(first), ctypes.byref(best),
         ctypes.byref(timed), _stream())
    problem = _library_problem(x, weight, out_dtype, accumulate)
    # the check: the winner and the library's ordinary call against a float32 product, from a zero stream
    exact = torch.mm(x.float(), weight.float().t())
    y.zero_()
    call("leone_library_product", _dev(x, "x"), _dev(weight, "w"), _dev(y, "y"), rows, n, k, out_code,
         1 if accumulate else 0, _stream())
    usual = torch.mm(x, weight.t(), out_dtype=torch.float32) if out_dtype == torch.float32 else torch.nn.functional.linear(x, weight)
    off = (y.float() - exact).abs().max().item()
    usual_off = (usual.float() - exact).abs().max().item()
    kept = bool(off <= 2.0 * usual_off + 1e-6 * exact.abs().max().item())
    if kept:
        # An algorithm that reduces over K with atomics (split-K, stream-K) need not repeat bit for bit, and
        # then neither would the logits of a replayed trace: the winner runs again from the same zero stream,
        # and once more with the rows of x in reverse order (a row's bits must not depend on the other rows).
        again = torch.zeros_like(y)
        call("leone_library_product", _dev(x, "x"), _dev(weight, "w"), _dev(again, "y"), rows, n, k, out_code,
             1 if accumulate else 0, _stream())
        turned, x_turned = torch.zeros_like(y), x.flip(0).contiguous()
        call("leone_library_product", _dev(x_turned, "x"), _dev(weight, "w"), _dev(turned, "y"), rows, n, k, out_code,
             1 if accumulate else 0, _stream())
        kept = bool(torch.equal(again, y) and torch.equal(turned.flip(0), y))
    if kept:
        _tuned_products.add(problem)
    else:
        call("leone_library_product_forget", rows, n, k, out_code, 1 if accumulate else 0)
    return {"problem": problem, "rows": rows, "weight_rows": n, "inner": k, "float_out": out_dtype == torch.float32,
            "adds": bool(accumulate),
            "library_us": round(first.value, 1), "tuned_us": round(best.value, 1), "timed": timed.value, "kept": kept,
            "off": off, "library_off": usual_off}      # ``kept`` False: too far off, or not the same bits twice


def forget_tuned_products(problems=None) -> None:
    """Gives the named problems (all, if none are named) back to the library's heuristic."""
    for problem in list(_tuned_products if problems is None else problems):
        device, m, n, k, out_code, accumulate = problem
        with torch.cuda.device(device):
            call("leone_library_product_forget", m, n, k, out_code, accumulate)
        _tuned_products.discard(problem)


def _library_product(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype,
                     residual: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    """The vendor library's product for many rows: bfloat16 or float32 out, or added into the float32 stream
    (then nothing comes back).  A problem that was tuned runs with the algorithm that won; any other goes
    through torch's call of the same library."""
    problem = _library_problem(x, weight, out_dtype, residual is not None)
    if _recorded_products is not None:
        known = _recorded_products.setdefault(problem[1:], [])
        if all(w is not weight for w in known):
            known.append(weight)
    if problem in _tuned_products and x.is_contiguous() and weight.is_contiguous():
        y = residual if residual is not None else torch.empty((x.shape[0], weight.shape[0]), dtype=out_dtype, device=x.device)
        call("leone_library_product", _dev(x, "x", torch.bfloat16), _dev(weight, "w", torch.bfloat16),
             _dev(y, "y", out_dtype, (x.shape[0], weight.shape[0])), x.shape[0], weight.shape[0], weight.shape[1],
             problem[4], problem[5], _stream())
        return None if residual is not None else y
    if residual is not None:
        # the library adds into the stream itself (float product plus float stream, the same bits as adding the
        # product afterwards), which saves the next norm's kernel the read of the product: 27.2 against 27.8 ms
        # for a prompt of 2,048 tokens
        torch.addmm(residual, x, weight.t(), out_dtype=torch.float32, out=residual)
        return None
    if out_dtype == torch.float32:
        return torch.mm(x, weight.t(), out_dtype=torch.float32)
    return torch.nn.functional.linear(x, weight)    # float accumulation


def linear(x, weight: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
           residual: Optional[torch.Tensor] = None, gated: bool = False,
           planes_ok: bool = False, next_norm=None):
    """x[R,K] . weight[N,K]^T, with optional neighbours.

    ``x`` is a tensor or ``NormedRows`` (a norm still to be done).  ``gated``: the weight is an
    interleaved gate/up weight and the result is silu(gate) * up, ``[R, N/2]``.  ``residual``: the caller
    wants the product added into this float32 tensor; if the kernel in use can do that, it does and None
    is returned, otherwise the product is returned for the caller to add later, as float32 ``[R, N]`` or
    as a stack of planes ``[p, R, N]`` whose sum is meant (``add_rmsnorm`` takes either).

    ``next_norm`` = (gain, eps, dtype) with ``residual``: the caller will normalise the stream with this
    gain next; the kernel may leave that norm's operand behind, and then ``PreparedRows`` is returned
    instead of None.  ``planes_ok``: the caller also takes a plain product as float32 planes ``[p, R, N]`` whose sum, in
    order, is meant (``qk_norm_rope_write`` does).

    float32 runs the single-precision kernel.  bfloat16 accumulates in float: up to FUSED_ROWS rows on the
    weight-streaming kernel with everything folded in, up to ROWS_MAX rows (a decode step of many requests)
    on the multi-row weight-streaming kernel, more rows (prompt portions) through the library's matrix
    product, with float32 output for logits and for what goes into the stream.
    """
    dtype = x.dtype if isinstance(x, NormedRows) else x.dtype
    if dtype != weight.dtype:
        raise KernelError(f"linear: activations are {dtype} but the weight is {weight.dtype}")
    out_dtype = out_dtype or dtype
    rows, k = x.shape
    if dtype == torch.bfloat16 and weight.is_cuda and k % 8 == 0 and rows <= FUSED_ROWS \
            and (not gated or weight.shape[0] % 16 == 0):
        # Every workgroup (16 weight rows) would redo a folded norm for its own use: that pays only for
        # matrices with few rows; for the others the norm kernel runs once and the product reads its result.
        if isinstance(x, NormedRows) and not isinstance(x, PreparedRows) and weight.shape[0] > FUSED_NORM_WEIGHT_ROWS:
            # rounds where the folded norm rounds, whatever the weight's size
            x = x.prepare() if prepared_fits(rows, k) else x.materialize()
        if next_norm is not None and (residual is None or not prepared_fits(rows, weight.shape[0])
                                      or next_norm[2] != torch.bfloat16):
            next_norm = None
        return gemm_fused(x, weight, out_dtype, residual, gated, next_norm)
    x = materialize(x)
    if dtype == torch.bfloat16 and weight.is_cuda and k % 8 == 0 and rows <= ROWS_MAX \
            and (not gated or weight.shape[0] % 16 == 0):
        return gemm_rows(x, weight, out_dtype, residual, gated, may_split=planes_ok or residual is not None)
    if dtype == torch.float32:
        if out_dtype != torch.float32:
            raise KernelError("linear: the float32 path produces float32")
        y = gemm_f32(x, weight)
    elif not x.is_cuda:
        raise KernelError("linear: tensor is not on the GPU")
    elif out_dtype == torch.float32 or (residual is not None and not gated):
        # float32 results for many rows, from the library's product with float output: logits, and what is
        # to be added into the float32 stream, which the kernel for few rows adds unrounded as well
        parts = inner_parts(rows, weight.shape[0], k) if residual is not None else 1
        with profile.span(profile.LIBRARY_PRODUCT, weight):
            if parts > 1:
                # [parts, rows, N]: the planes are summed, in order, by the norm kernel that adds them
                y = torch.bmm(x.view(rows, parts, k // parts).transpose(0, 1),
                              weight.view(weight.shape[0], parts, k // parts).permute(1, 2, 0), out_dtype=torch.float32)
            elif residual is not None:
                return _library_product(x, weight, torch.float32, residual)
            else:
                y = _library_product(x, weight, torch.float32, None)
    else:
        with profile.span(profile.LIBRARY_PRODUCT, weight):
            y = _library_product(x, weight, torch.bfloat16, None)
        if out_dtype != y.dtype:
            y = y.to(out_dtype)
    return swiglu(y) if gated else y


def argmax(logits: torch.Tensor) -> torch.Tensor:
    rows, vocab = logits.shape
    chunks = -(-vocab // library().leone_argmax_chunk())
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    part_value = torch.empty((rows * chunks,), dtype=torch.float32, device=logits.device)
    part_index = torch.empty((rows * chunks,), dtype=torch.int32, device=logits.device)
    call("leone_argmax", _dev(logits, "argmax logits", torch.float32), _dev(out, "argmax out"),
         _dev(part_value, "argmax partial values"), _dev(part_index, "argmax partial indices"), rows, vocab,
         _stream())
    return out


def sample_temperature(logits: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor) -> torch.Tensor:
    """One token a row by its temperature (float64 [rows], positive) and uniform value (float64 [rows] in
    [0, 1)); -1 for a row without a finite logit."""
    rows, vocab = logits.shape
    chunks = -(-vocab // library().leone_argmax_chunk())
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    part_value = torch.empty((rows * chunks,), dtype=torch.float32, device=logits.device)
    part_index = torch.empty((rows * (chunks + 1),), dtype=torch.int32, device=logits.device)   # and the best of each row
    sums = torch.empty((rows * chunks,), dtype=torch.float64, device=logits.device)
    call("leone_sample_temperature", _dev(logits, "sample logits", torch.float32),
         _dev(temperature, "sample temperature", torch.float64, (rows,)),
         _dev(uniform, "sample uniform", torch.float64, (rows,)), _dev(out, "sample out"),
         _dev(part_value, "sample partial values"), _dev(part_index[:rows * chunks], "sample partial indices"),
         _dev(part_index[rows * chunks:], "sample best"), _dev(sums, "sample sums"), rows, vocab, _stream())
    return out


TOP_CANDIDATES_MAX = 256     # most candidates a row the selection kernel gives (checked against the library)


def top_candidates(logits: torch.Tensor, wanted) -> tuple:
    """The ``wanted[row]`` best finite logits of every row in the sampler's order (higher first, the lower
    id on a tie), selected on the device and brought to the host in one copy.

    Returns numpy arrays: values float32 [rows, TOP_CANDIDATES_MAX], ids int32 likewise, counts int32
    [rows]; row r is filled up to counts[r] (fewer than it wanted only if it has fewer finite logits)."""
    if library().leone_top_candidates_max() != TOP_CANDIDATES_MAX:
        raise KernelError("the kernel library was built for another number of candidates")
    rows, vocab = logits.shape
    wanted = [int(k) for k in wanted]
    if len(wanted) != rows or not all(1 <= k <= TOP_CANDIDATES_MAX for k in wanted):
        raise KernelError(f"top_candidates: one count in 1..{TOP_CANDIDATES_MAX} for each of {rows} rows, found {wanted}")
    room = rows * TOP_CANDIDATES_MAX
    flat = torch.empty((rows + 2 * room,), dtype=torch.int32, device=logits.device)   # counts | values | ids
    # The kernel selects the largest count for every row, best first: a row that wants fewer takes the first.
    call("leone_top_candidates", _dev(logits, "candidate logits", torch.float32),
         _dev(flat[rows:rows + room], "candidate values"), _dev(flat[rows + room:], "candidate ids"),
         _dev(flat[:rows], "candidate counts"), rows, vocab, max(wanted), _stream())
    host = flat.cpu().numpy()
    counts = np.where(host[:rows] < 0, -1, np.minimum(host[:rows], np.asarray(wanted, dtype=np.int32)))
    return (host[rows:rows + room].view("float32").reshape(rows, TOP_CANDIDATES_MAX),
            host[rows + room:].reshape(rows, TOP_CANDIDATES_MAX), counts)


TRUNCATED_STAGES = 8         # most truncation stages of a row that is drawn on the device (checked against the library)
TRUNCATION_KINDS = {"top_k": 0, "top_p": 1, "min_p": 2}


def truncated_draw_supported(stages) -> bool:
    """Whether ``sample_truncated`` serves a row with these (stage, value) pairs: top-k first with k at most
    TOP_CANDIDATES_MAX, then top-k, top-p and min-p in any order, TRUNCATED_STAGES at most in all."""
    stages = list(stages)
    return (0 < len(stages) <= TRUNCATED_STAGES and all(name in TRUNCATION_KINDS for name, _ in stages)
            and stages[0][0] == "top_k" and 1 <= int(stages[0][1]) <= TOP_CANDIDATES_MAX)


def truncated_rows(draws) -> np.ndarray:
    """The parameters of ``sample_truncated`` as a host array, float64 [rows, 3 + 2 * TRUNCATED_STAGES]: ``draws``
    holds for each row either None (the row is skipped and gets -1) or (temperature, uniform value,
    [(stage, value), ...]) with stages that ``truncated_draw_supported`` accepts."""
    lib = library()
    if (lib.leone_sample_truncated_stages() != TRUNCATED_STAGES or lib.leone_top_candidates_max() != TOP_CANDIDATES_MAX
            or lib.leone_sample_truncated_params() != 3 + 2 * TRUNCATED_STAGES):
        raise KernelError("the kernel library was built for another table of truncation stages")
    draws = list(draws)
    table = np.zeros((len(draws), 3 + 2 * TRUNCATED_STAGES), dtype=np.float64)
    for r, draw in enumerate(draws):
        if draw is None:
            continue
        temperature, uniform, stages = draw
        stages = list(stages)
        if not truncated_draw_supported(stages):
            raise KernelError(f"sample_truncated: row {r}: stages {stages} are not drawn on the device")
        if not (math.isfinite(temperature) and temperature > 0.0 and 0.0 <= uniform < 1.0):
            raise KernelError(f"sample_truncated: row {r}: temperature {temperature} or uniform value {uniform} out of range")
        for name, value in stages:
            if name == "top_k" and not (value >= 1 and int(value) == value) or name != "top_k" and not 0.0 < value <= 1.0:
                raise KernelError(f"sample_truncated: row {r}: {name} {value} out of range")
        table[r, 0], table[r, 1], table[r, 2] = temperature, uniform, len(stages)
        for s, (name, value) in enumerate(stages):
            # top-k beyond every vocabulary keeps everything: the value only has to stay a number the kernel can compare
            table[r, 3 + 2 * s], table[r, 4 + 2 * s] = TRUNCATION_KINDS[name], min(float(value), 2.0 ** 31)
    return table


def truncated_table(draws, device) -> torch.Tensor:
    """``truncated_rows`` on the device."""
    return torch.from_numpy(truncated_rows(draws)).to(device)


def sample_truncated(logits: torch.Tensor, draws) -> torch.Tensor:
    """One token a row (int32 on the device) by temperature sampling with truncation stages, top-k first:
    selection, stages and draw in one launch, nothing comes to the host.  ``draws``: what ``truncated_table``
    takes, or the table it made (float64 on the device).  -1 for a skipped row and for a row without a finite
    logit."""
    rows, vocab = logits.shape
    params = draws if isinstance(draws, torch.Tensor) else truncated_table(draws, logits.device)
    if params.shape != (rows, 3 + 2 * TRUNCATED_STAGES):
        raise KernelError(f"sample_truncated: {rows} rows of logits, a table of {tuple(params.shape)}")
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    call("leone_sample_truncated", _dev(logits, "sample logits", torch.float32),
         _dev(params, "sample stages", torch.float64), _dev(out, "sample out"), rows, vocab, _stream())
    return out


__all__ = [name for name in dir() if not name.startswith("_")]

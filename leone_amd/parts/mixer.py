"""Token mixers."""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from .. import ops
from ..weights.loader import MATRIX, VECTOR, TensorSpec
from .base import MIXERS, KvNeed, Part, PartSpec, RowTiling
from .context import KvCacheView, StepContext
from .position import rotation_of


@MIXERS.register("gqa_attention")
class GqaAttention(Part):
    """Grouped-query causal attention over a paged key/value cache.

    q = Wq y, k = Wk y, v = Wv y (no bias); optional per-head RMSNorm of q and
    k over head_dim, then the position encoding on q and k; k and v go into the
    cache; each row attends the keys of its own request up to its position
    (within ``window`` if set) with scale 1/sqrt(head_dim); out = Wo o.
    Reference: crates/leone/src/runtime.rs:9104-9157 (decode order),
    crates/leone/src/backend.rs:2182-2208 (per-head norm),
    crates/leone/src/cpu.rs:2299-2357 (attention).

    Parameters: ``hidden``, ``q_heads``, ``kv_heads``, ``head_dim``, ``qk_norm_eps``
    (None: no q/k norm), ``window`` (None: all keys), ``position`` (name of a
    position part) and tensor names ``q``, ``k``, ``v``, ``o``, ``q_norm``, ``k_norm``.
    """

    graph_safe = True

    def __init__(self, spec: PartSpec, positions: Optional[dict] = None, **_):
        p = spec.params
        self.hidden = int(p["hidden"])
        self.q_heads = int(p["q_heads"])
        self.kv_heads = int(p["kv_heads"])
        self.head_dim = int(p["head_dim"])
        if self.q_heads % self.kv_heads:
            raise ValueError(f"{self.q_heads} query heads cannot be grouped over {self.kv_heads} kv heads")
        self.qk_norm_eps = p.get("qk_norm_eps")
        self.window = p.get("window")
        self.scale = float(p.get("scale", 1.0 / math.sqrt(self.head_dim)))
        self.names = {k: p[k] for k in ("q", "k", "v", "o")}
        if self.qk_norm_eps is not None:
            self.names.update(q_norm=p["q_norm"], k_norm=p["k_norm"])
        self.position = (positions or {}).get(p.get("position")) if p.get("position") else None
        if p.get("position") and self.position is None:
            raise ValueError(f"attention names position part {p.get('position')!r}, which the model does not define")
        self.w_qkv = self.w_o = self.q_gain = self.k_gain = None

    def cache_need(self) -> KvNeed:
        return KvNeed(self.kv_heads, self.head_dim, self.window)

    def row_tiling(self) -> RowTiling:
        """The tiles of the prompt-attention kernel."""
        return RowTiling(ops.PREFILL_TILE_ROWS, ops.PREFILL_GROUP_TILES, ops.PREFILL_MIN_ROWS)

    def tensor_specs(self) -> List[TensorSpec]:
        qw, kvw = self.q_heads * self.head_dim, self.kv_heads * self.head_dim
        specs = [TensorSpec(self.names["q"], (qw, self.hidden), MATRIX),
                 TensorSpec(self.names["k"], (kvw, self.hidden), MATRIX),
                 TensorSpec(self.names["v"], (kvw, self.hidden), MATRIX),
                 TensorSpec(self.names["o"], (self.hidden, qw), MATRIX)]
        if self.qk_norm_eps is not None:
            specs += [TensorSpec(self.names["q_norm"], (self.head_dim,), VECTOR),
                      TensorSpec(self.names["k_norm"], (self.head_dim,), VECTOR)]
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        # One product for q, k and v: a pure re-layout of the three matrices.
        self.w_qkv = torch.cat([tensors.pop(self.names["q"]), tensors.pop(self.names["k"]),
                                tensors.pop(self.names["v"])], dim=0).contiguous()
        self.w_o = tensors.pop(self.names["o"]).contiguous()
        if self.qk_norm_eps is not None:
            self.q_gain = tensors.pop(self.names["q_norm"]).contiguous()
            self.k_gain = tensors.pop(self.names["k_norm"]).contiguous()
            if self.q_gain.dtype != self.k_gain.dtype:
                self.q_gain, self.k_gain = self.q_gain.float(), self.k_gain.float()

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_qkv, self.w_o]

    fused_io = True
    prepares_next = True

    def forward(self, y, step: StepContext, cache: KvCacheView,
                residual: Optional[torch.Tensor] = None, next_norm=None):
        """``y`` may be a norm still to be done; with ``residual`` the result may be added there (None returned),
        and with ``next_norm`` the norm that follows may come back prepared (see ``ops.linear``)."""
        qkv = ops.linear(y, self.w_qkv, planes_ok=True)
        # How much of a head is rotated and in which pairs is the position part's affair; the kernels are told.
        rotation = rotation_of(self.position)
        cos, sin = rotation.cos, rotation.sin
        if cos is not None and step.max_position >= cos.shape[0]:
            raise ValueError(f"position {step.max_position} is beyond the rotary table of {cos.shape[0]} positions")
        kernels = self.attention_kernels(step.dtype, cache.page_tokens, cache.block_table.shape[1])
        if step.decode_only and kernels["decode"] == "projected":
            # Single decoded tokens, every row another request: the attention kernel makes the heads itself.
            attended = ops.attention_decode_projected(
                qkv, self.q_heads, self.kv_heads, self.head_dim, self.q_gain, self.k_gain,
                self.qk_norm_eps if self.qk_norm_eps is not None else 1.0, cos, sin, cache.k_pool, cache.v_pool,
                step.positions, step.row_entry, cache.block_table, self.scale, int(self.window or 0),
                max_context=step.max_position + 1, write_cache=cache.writes, pairing=rotation.pairing)
            return ops.linear(attended, self.w_o, residual=residual, next_norm=next_norm)
        q = ops.qk_norm_rope_write(qkv, self.q_heads, self.kv_heads, self.head_dim, self.q_gain, self.k_gain,
                                   self.qk_norm_eps if self.qk_norm_eps is not None else 1.0, cos, sin,
                                   step.positions, step.row_entry, cache.block_table, cache.k_pool, cache.v_pool,
                                   write_cache=cache.writes, out_dtype=step.dtype, pairing=rotation.pairing)
        attended = self._attend(q, step, cache)
        return ops.linear(attended, self.w_o, residual=residual, next_norm=next_norm)

    def attention_kernels(self, dtype: torch.dtype, page_tokens: int, max_blocks: int = 0) -> Dict[str, str]:
        """Which kernels this shape gets, by kind of work: ``decode`` (steps of single tokens): "projected" (the
        split-KV matrix-core kernel that also makes the heads and writes the cache), "split_kv" (the same
        kernel behind the norm/rotation/write kernel) or "rows" (the float kernel for any shape and type);
        ``prompt`` (portions of at least ``ops.PREFILL_MIN_ROWS`` rows): "flash" (the matrix-core prompt
        kernel), else what single tokens get."""
        group = self.q_heads // self.kv_heads
        if not ops.decode_attention_supported(dtype, self.head_dim, page_tokens, group, max_blocks):
            return {"decode": "rows", "prompt": "rows"}
        rotation = rotation_of(self.position)
        projected = ops.decode_projected_supported(self.head_dim, rotation.rotary_dim, rotation.pairing)
        return {"decode": "projected" if projected else "split_kv",
                "prompt": "flash" if ops.prefill_attention_supported(dtype, self.head_dim, page_tokens, max_blocks) else "split_kv"}

    def _attend(self, q: torch.Tensor, step: StepContext, cache: KvCacheView) -> torch.Tensor:
        """Long prompt portions through the prompt kernel, the other rows through the split-KV kernel; the
        row kernel takes what the matrix-core kernels refuse (float32, odd sizes)."""
        window = int(self.window or 0)
        group = self.q_heads // self.kv_heads
        max_blocks = cache.block_table.shape[1]
        if not ops.decode_attention_supported(q.dtype, self.head_dim, cache.page_tokens, group, max_blocks):
            return ops.attention_rows(q, cache.k_pool, cache.v_pool, step.positions, step.row_entry,
                                      cache.block_table, self.q_heads, self.scale, window)
        first = 0
        out = torch.empty_like(q)
        tiled = step.tiled.get(self.row_tiling())
        if (tiled is not None and tiled.rows
                and ops.prefill_attention_supported(q.dtype, self.head_dim, cache.page_tokens, max_blocks)):
            ops.attention_prefill(q, out, cache.k_pool, cache.v_pool, step.positions, tiled.tiles,
                                  cache.block_table, self.q_heads, self.scale, window,
                                  mean_keys=tiled.mean_keys or step.max_position + 1, covered_rows=tiled.rows)
            first = tiled.rows
        if first < step.rows:
            ops.attention_decode(q[first:], cache.k_pool, cache.v_pool, step.positions[first:],
                                 step.row_entry[first:], cache.block_table, self.q_heads, self.scale, window,
                                 max_context=step.max_position + 1, out=out[first:])
        return out

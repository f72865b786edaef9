"""A decoder model as data (``ModelSpec``) and the object built from it."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import torch

from .. import ops
from ..weights.loader import MATRIX, TensorSpec
from .base import BLOCKS, NORMS, POSITIONS, PartSpec
from .context import CacheView, StepContext


@dataclass(frozen=True)
class LayerRun:
    """One entry of the execution order.

    ``layer`` indexes ``ModelSpec.layers`` (a layer may be named more than
    once).  ``cache`` is the cache slot the run works on; two runs that name the
    same slot share it, and only runs with ``writes`` put new keys, values or
    state there.
    """
    layer: int
    cache: Optional[int]
    writes: bool = True


@dataclass
class ModelSpec:
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: str                                  # tensor name of the token table [vocab, hidden]
    layers: List[PartSpec]                          # block specs
    schedule: List[LayerRun]
    final_norm: PartSpec
    head: Optional[str]                             # tensor name [vocab, hidden]; None = tied to the embedding
    positions: Dict[str, PartSpec] = field(default_factory=dict)
    ignore_tensors: Sequence[str] = ()              # names a file may hold that the model does not use
    embedding_scale: Optional[float] = None         # the stream starts as table row * scale
    logit_cap: Optional[float] = None               # logits = cap * tanh(logits / cap)


def default_schedule(n_layers: int) -> List[LayerRun]:
    return [LayerRun(i, i, True) for i in range(n_layers)]


class DecoderModel:
    """Embedding, the scheduled layer runs, final norm and the output head."""

    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"engine type must be float32 or bfloat16, found {dtype}")
        self.spec = spec
        self.dtype = dtype
        self.device = torch.device(device)
        self.positions = {name: POSITIONS.build(s) for name, s in spec.positions.items()}
        self.layers = [BLOCKS.build(s, positions=self.positions) for s in spec.layers]
        self.final_norm = NORMS.build(spec.final_norm)
        self.schedule = list(spec.schedule)
        for run in self.schedule:
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"schedule names layer {run.layer}, the model has {len(self.layers)}")
        self.embedding: Optional[torch.Tensor] = None
        self.head: Optional[torch.Tensor] = None
        self.streamed_copy_bytes: Optional[int] = None    # None: not decided yet (``keep_streamed_copies``)

    @property
    def graph_safe(self) -> bool:
        """Whether a step of this model can be recorded once and replayed (see ``Part.graph_safe``)."""
        return (all(getattr(layer, "graph_safe", False) for layer in self.layers)
                and getattr(self.final_norm, "graph_safe", False))

    # ---- weights -------------------------------------------------------------
    def tensor_specs(self) -> List[TensorSpec]:
        specs = [TensorSpec(self.spec.embedding, (self.spec.vocab_size, self.spec.hidden_size), MATRIX)]
        for layer in self.layers:
            specs += layer.tensor_specs()
        specs += self.final_norm.tensor_specs()
        if self.spec.head is not None:
            specs.append(TensorSpec(self.spec.head, (self.spec.vocab_size, self.spec.hidden_size), MATRIX))
        return specs

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        tensors = dict(tensors)
        self.embedding = tensors.pop(self.spec.embedding).contiguous()
        self.head = tensors.pop(self.spec.head).contiguous() if self.spec.head is not None else self.embedding
        for layer in self.layers:
            layer.bind(tensors)
        self.final_norm.bind(tensors)
        for position in self.positions.values():
            position.prepare(self.spec.max_positions, self.device)

    # Auto: keep the second copies if they take at most this share of the device's memory and of what is free.
    STREAMED_SHARE_OF_DEVICE = 0.25
    STREAMED_SHARE_OF_FREE = 0.5

    def streamed_weights(self) -> List[torch.Tensor]:
        """Every matrix a decode step streams through ``ops.linear``: the layers' and the head."""
        found = [w for layer in self.layers if hasattr(layer, "streamed_weights") for w in layer.streamed_weights()]
        if self.head is not None:
            found.append(self.head)
        return found

    def keep_streamed_copies(self, wanted: Optional[bool] = None) -> int:
        """Keeps, beside every matrix that decode steps stream through, a second copy in the order in which
        the weight-streaming kernels read it fastest (``ops.tile_weight``; the row-major one stays for the
        library's products of prompt portions and for the token table).  The results are the same bit for
        bit; a decode step of few rows takes a sixth less time; the weights take twice the memory.
        ``wanted`` None decides by room: yes if the copies take at most a quarter of the device's memory
        and half of what is free.  Returns the bytes the copies take (0: none kept).  Asked again, it
        answers what it did the first time."""
        if self.streamed_copy_bytes is not None:
            return self.streamed_copy_bytes
        self.streamed_copy_bytes = 0
        weights = self.streamed_weights() if (self.dtype == torch.bfloat16 and wanted is not False) else []
        weights = [w for w in weights if w.is_cuda and w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] % 64 == 0]
        if not weights:
            return 0
        if wanted is None:
            needed = sum(-(-w.shape[0] // 16) * 16 * w.shape[1] * 2 for w in weights)
            free, total = torch.cuda.mem_get_info(weights[0].device)
            if needed > self.STREAMED_SHARE_OF_DEVICE * total or needed > self.STREAMED_SHARE_OF_FREE * free:
                return 0
        self.streamed_copy_bytes = sum(ops.keep_streamed_copy(w) for w in weights)
        return self.streamed_copy_bytes

    def row_tilings(self) -> list:
        """Every distinct tiling a part of the model declares, in a fixed order (``RowTiling``)."""
        found = []
        for layer in self.layers:
            for tiling in (layer.row_tilings() if hasattr(layer, "row_tilings") else []):
                if tiling is not None and tiling not in found:
                    found.append(tiling)
        return found

    # ---- bytes ---------------------------------------------------------------
    def weight_accounting(self, nbytes=None, rows: int = 1) -> Dict[str, object]:
        """Bytes of the model's tensors by class, as they lie in memory (``resident``) and as a decode step
        of ``rows`` rows reads them (``decode``): of the token table only the rows' own rows, and the whole
        table once more as the head if the head is tied to it (the reference's accounting,
        crates/leone/src/model.rs:306-366).  ``nbytes(spec)`` gives a tensor's size; by default its element
        count in this model's type."""
        size = 2 if self.dtype == torch.bfloat16 else 4
        if nbytes is None:
            def nbytes(spec):
                count = 1
                for extent in spec.shape:
                    count *= extent
                return count * size
        resident: Dict[str, int] = {"embed": 0, "head": 0}
        table = TensorSpec(self.spec.embedding, (self.spec.vocab_size, self.spec.hidden_size), MATRIX)
        resident["embed"] = nbytes(table)
        if self.spec.head is not None:
            resident["head"] = nbytes(TensorSpec(self.spec.head, (self.spec.vocab_size, self.spec.hidden_size), MATRIX))
        for layer in self.layers:
            for part in (layer.parts() if hasattr(layer, "parts") else (layer,)):
                family = getattr(part, "family", "layer")
                resident[family] = resident.get(family, 0) + sum(nbytes(s) for s in part.tensor_specs())
        resident["norm"] = resident.get("norm", 0) + sum(nbytes(s) for s in self.final_norm.tensor_specs())
        decode = dict(resident)
        decode["embed"] = resident["embed"] // self.spec.vocab_size * rows
        if self.spec.head is None:
            decode["head"] = resident["embed"]
        return {"tensor_bytes": sum(resident.values()), "resident": resident, "decode": decode,
                "streamed_copy_bytes": self.streamed_copy_bytes or 0}

    def weight_bytes(self) -> int:
        """Bytes of all tensors of the model."""
        return self.weight_accounting()["tensor_bytes"]

    def decode_step_weight_bytes(self, rows: int = 1) -> int:
        """Weight bytes a decode step of ``rows`` rows has to read: every weight it uses, once."""
        return sum(self.weight_accounting(rows=rows)["decode"].values())

    # ---- cache ---------------------------------------------------------------
    def cache_needs(self) -> Dict[int, object]:
        """Cache slot -> what the layer runs on it need (one need per slot)."""
        needs: Dict[int, object] = {}
        writers: Dict[int, int] = {}
        for run in self.schedule:
            need = self.layers[run.layer].cache_need()
            if need is None:
                if run.cache is not None:
                    raise ValueError(f"layer {run.layer} keeps no cache but its run names slot {run.cache}")
                continue
            if run.cache is None:
                raise ValueError(f"layer {run.layer} needs a cache but its run names none")
            if run.cache in needs and needs[run.cache] != need:
                raise ValueError(f"cache slot {run.cache} is shared by layers with different needs")
            needs[run.cache] = need
            writers[run.cache] = writers.get(run.cache, 0) + (1 if run.writes else 0)
        for slot, count in writers.items():
            if count != 1:
                raise ValueError(f"cache slot {slot} must have exactly one writing run, found {count}")
        return needs

    # ---- forward ---------------------------------------------------------------
    def forward(self, tokens: torch.Tensor, step: StepContext, caches: Dict[int, CacheView]) -> Optional[torch.Tensor]:
        """Runs the step's rows through every scheduled layer; returns float32 logits of the wanted rows."""
        x = ops.embed(self.embedding, tokens, scale=self.spec.embedding_scale or 1.0)
        pending = None
        for at, run in enumerate(self.schedule):
            cache = caches.get(run.cache) if run.cache is not None else None
            if cache is not None and cache.writes != run.writes:
                cache = type(cache)(**{**cache.__dict__, "writes": run.writes})
            layer = self.layers[run.layer]
            # A block that can do so leaves the first norm of the block that runs next prepared.
            after = self.layers[self.schedule[at + 1].layer] if at + 1 < len(self.schedule) else None
            next_norm = after.entry_norm(step.dtype) if hasattr(after, "entry_norm") else None
            if next_norm is not None and getattr(layer, "prepares_next", False):
                pending = layer.forward(x, pending, step, cache, next_norm=next_norm)
            else:
                pending = layer.forward(x, pending, step, cache)
        if step.want_rows is None or step.want_rows.numel() == 0:
            if pending is not None:
                pass  # nothing reads the last delta when no logits are wanted
            return None
        if isinstance(pending, ops.PreparedRows):
            pending = None                    # prepared for a norm that never ran: the stream is up to date
        if hasattr(self.final_norm, "lazy"):
            y = self.final_norm.lazy(x, pending, self.dtype, rows=step.want_rows)
        else:
            y = self.final_norm.add_norm(x, pending, self.dtype, rows=step.want_rows)
        logits = ops.linear(y, self.head, out_dtype=torch.float32)
        return ops.soft_cap(logits, self.spec.logit_cap) if self.spec.logit_cap else logits

"""The step function: a batch of (request, its next tokens) through the model, from the cache.

The reference has three entry points for this work: one token of one request
(crates/leone/src/runtime.rs:7293), a prompt portion of one request
(crates/leone/src/runtime.rs:6638) and one token each of several requests
(crates/leone/src/runtime.rs:7461).  Here one ``step`` takes any mixture: each
entry brings the next tokens of one request, prompt portions beside single
decoded tokens, cut anywhere.  Only the given tokens are run; everything
earlier comes from the cache.  A step is a transaction on the cache: pages are
reserved first, written by the kernels, and committed only if the step succeeds
(crates/leone/src/kv.rs:326-370, 856-927).
"""
from __future__ import annotations

import ctypes
import math
import time
from ctypes import c_int, c_int64, c_long
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from .. import hostlib, ops
from ..ops import profile
from ..cache.manager import CacheManager
from ..cache.pools import DevicePools
from ..parts.context import TiledRows, EntryInfo, StepContext
from ..parts.model import DecoderModel


@dataclass
class StepEntry:
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()       # indices into ``tokens`` whose logits are asked for


@dataclass
class StepOutput:
    logits: Optional[torch.Tensor]                 # float32 [wanted, vocab] on the device, or None
    rows: List[tuple] = field(default_factory=list)  # (request, index into its tokens) per logits row


class StepError(ValueError):
    """A step was refused before anything ran; the cache is unchanged."""


class PackedStep:
    """One step's metadata as the native layout routine wrote it into a host buffer (int32 words):
    tokens, positions, row -> entry, state slots, wanted rows, one tile list per row tiling, one block table
    per cache group."""

    def __init__(self, cache: CacheManager, vocab_size: int, entries: Sequence[StepEntry], all_rows_wanted: bool = False,
                 host=None, tilings: Sequence = ()):
        """``host``: nothing (a buffer is made), a buffer to write into (it must be large enough), or a
        callable that is given the number of words and returns one.  ``tilings``: the ``RowTiling`` of the
        model's parts; each gets a tile list."""
        n = len(entries)
        lib = hostlib.library()
        requests = (c_int64 * max(1, n))()
        counts, want_counts = (c_int * max(1, n))(), (c_int * max(1, n))()
        flat_tokens: List[int] = []
        flat_wants: List[int] = []
        for i, e in enumerate(entries):
            key = cache.keys.key(e.request)
            if key is None:
                raise StepError(f"request {e.request!r} is not admitted")
            requests[i], counts[i], want_counts[i] = key, len(e.tokens), len(e.want)
            flat_tokens.extend(e.tokens)
            flat_wants.extend(e.want)
        try:
            tokens = np.asarray(flat_tokens, dtype=np.int64)
            wants = np.asarray(flat_wants, dtype=np.int64)
        except (TypeError, ValueError, OverflowError) as error:
            raise StepError(f"tokens and wanted places must be integers: {error}") from None
        limit = np.iinfo(np.int32)
        if tokens.size and (tokens.min() < limit.min or tokens.max() > limit.max):
            raise StepError(f"a token lies outside the vocabulary of {vocab_size}")
        if wants.size and (wants.min() < limit.min or wants.max() > limit.max):
            raise StepError("a wanted place lies outside its entry")
        tokens, wants = tokens.astype(np.int32), wants.astype(np.int32)
        tilings = list(tilings)
        flat = [v for t in tilings for v in (t.tile_rows, t.min_rows, t.group_tiles)]
        shape = (c_int * (3 + len(flat)))(vocab_size, int(all_rows_wanted), len(tilings), *flat)
        sections = (c_long * (6 + len(tilings) + len(cache.groups)))()
        summary, placed = (c_int * (4 + 2 * len(tilings)))(), (c_int * (5 * max(1, n)))()
        as_i32 = lambda a: a.ctypes.data_as(hostlib.PI32)
        args = (cache.handle, n, requests, counts, want_counts, as_i32(tokens), as_i32(wants), shape)
        total = lib.leone_step_pack(*args, None, 0, sections, None, None)
        if total >= 0:
            if host is None:
                host = torch.empty(max(1, total), dtype=torch.int32)
            elif callable(host):
                host = host(max(1, total))                  # the caller hands out a buffer of that many words
            elif host.numel() < total:
                raise StepError("the step does not fit the recorded layout")
            total = lib.leone_step_pack(*args, ctypes.cast(host.data_ptr(), hostlib.PI32), host.numel(), sections,
                                        summary, placed)
        if total < 0:
            raise StepError(cache.keys.named(hostlib.last_error()))
        self.host = host
        self.total = int(total)
        self.offsets = list(sections)
        self.rows, self.max_position, self.wanted = summary[0], summary[1], summary[2]
        self.decode_only = bool(summary[3])
        self.tilings = tilings
        self.tiled = [(summary[4 + 2 * i], summary[5 + 2 * i]) for i in range(len(tilings))]   # (rows, tiles) of each
        self.first_table = 5 + len(tilings)      # index of the first block table among the pieces
        # Entries in the order they run in: (index in the caller's list, slot, first row, rows, start).
        self.placed = [tuple(placed[5 * i:5 * i + 5]) for i in range(n)]

    def pieces(self, packed: torch.Tensor) -> List[torch.Tensor]:
        return [packed[self.offsets[i]:self.offsets[i + 1]] for i in range(len(self.offsets) - 1)]


DECODE_BUCKET_MIN = 256      # the smallest context range a decode step is recorded for


def context_bucket(positions: int, max_context: int) -> int:
    """The context range a decode step whose longest request holds ``positions`` tokens is recorded for: the
    next power of two from DECODE_BUCKET_MIN on, at most the engine's ``max_context``."""
    bucket = DECODE_BUCKET_MIN
    while bucket < positions:
        bucket *= 2
    return min(bucket, max_context)


class _DecodeGraph:
    """Recorded decode steps for one batch size: static metadata buffers and, for every context range
    (``context_bucket``) that came up, a graph and its logits.

    The step's metadata (tokens, positions, state slots, block tables) lives in one device buffer
    that is refilled before each replay; the recorded kernels read everything through it, so one
    recording serves every step of that batch size whose contexts lie in its range.  What a recording fixes
    beside the batch size is what the parts derive from ``StepContext.max_position`` on the host (into how
    many parts the attention kernel cuts a row's keys), hence one recording a range: a chat of 300 tokens on
    an engine built for 40,960 is cut as for 512, not as for 40,960 (the reference replays one decode graph per
    context bucket with a device-resident position, crates/leone/src/runtime.rs:3555-3615, 4991-5013).
    """

    def __init__(self, engine: "Engine", rows: int):
        groups = len(engine.cache.groups)
        widths = [engine.cache.max_blocks(g) for g in range(groups)]
        tilings = engine.tilings
        sizes = [rows] * 5 + [0] * len(tilings) + [rows * w for w in widths]   # tokens, positions, row_entry, slots, want, tiles, tables
        self.offsets = [int(v) for v in np.cumsum([0] + sizes)]
        total = self.offsets[-1]
        self.host = torch.empty(total, dtype=torch.int32).pin_memory()
        self.dev = torch.zeros(total, dtype=torch.int32, device=engine.device)
        pieces = [self.dev[self.offsets[i]:self.offsets[i + 1]] for i in range(len(sizes))]
        self.tokens = pieces[0]
        self.rows = rows
        self._pieces, self._tables = pieces, {g: pieces[5 + len(tilings) + g].view(rows, widths[g]) for g in range(groups)}
        self._engine_type = (engine.dtype, engine.device)
        self.recordings: Dict[int, tuple] = {}        # context range -> (graph, its logits)
        self.copied = torch.cuda.Event()

    def context(self, bucket: int) -> StepContext:
        """The step as the parts see it when it is recorded for contexts of up to ``bucket`` positions."""
        pieces = self._pieces
        return StepContext(
            rows=self.rows, dtype=self._engine_type[0], device=self._engine_type[1], positions=pieces[1],
            row_entry=pieces[2], entries=[], entry_slots=pieces[3], want_rows=pieces[4],
            block_tables=self._tables, max_position=bucket - 1, decode_only=True)

    def fill(self, engine: "Engine", entries: Sequence[StepEntry]) -> PackedStep:
        self.copied.synchronize()                     # the last upload has left the pinned buffer
        packed = PackedStep(engine.cache, engine.vocab_size, entries, all_rows_wanted=True, host=self.host,
                            tilings=engine.tilings)
        if packed.offsets != self.offsets:
            raise StepError("the step does not fit the recorded layout")
        self.dev.copy_(self.host, non_blocking=True)
        self.copied.record()
        return packed


class Engine:
    def __init__(self, model: DecoderModel, *, num_pages: Optional[int] = None, max_tokens: Optional[int] = None,
                 page_tokens: int = 64, max_requests: int = 64, max_context: Optional[int] = None,
                 poison_freed: bool = False, graphs: bool = True, streamed_weights: Optional[bool] = None):
        if model.embedding is None:
            raise ValueError("the model has no weights bound")
        if not torch.cuda.is_available() or model.device.type != "cuda":
            raise RuntimeError("the engine runs on a GPU only; there is no CPU path")
        # A second copy of the matrices in the order the decode kernels read fastest: by default if there is
        # ample room (``DecoderModel.keep_streamed_copies``); before the pools take their memory.
        model.keep_streamed_copies(streamed_weights)
        self.model = model
        self.device = model.device
        self.dtype = model.dtype
        self.page_tokens = page_tokens
        self.max_context = min(max_context or model.spec.max_positions, model.spec.max_positions)
        if num_pages is None:
            if max_tokens is None:
                raise ValueError("give num_pages or max_tokens")
            num_pages = (max_tokens + page_tokens - 1) // page_tokens
        self.pools = DevicePools(model.cache_needs(), self.dtype, self.device, num_pages, page_tokens, max_requests)
        self.cache = CacheManager(self.pools.group_specs, max_requests, self.max_context)
        # With poison_freed every page is filled with NaN when its last holder lets go of it, whoever frees it
        # (this engine, a scheduler on the same cache manager, a window that has passed): the manager notes
        # such pages and they are overwritten before the next kernel runs.
        self.poison_freed = poison_freed
        if poison_freed:
            self.cache.log_freed(True)
        self.vocab_size = model.spec.vocab_size
        self.tilings = model.row_tilings()      # what the parts want long portions cut into
        # Steps of single decoded tokens are recorded once per batch size and replayed.
        self.graphs = bool(graphs) and model.graph_safe
        self._decode_graphs: Dict[int, _DecodeGraph] = {}
        self._graph_pool = torch.cuda.graph_pool_handle() if self.graphs else None
        self._staging: List[Optional[tuple]] = [None, None]
        self._staging_turn = 0

    # ---- requests -----------------------------------------------------------------
    def admit(self, request: Hashable) -> int:
        slot = self.cache.admit(request)
        self.pools.zero_state(slot)
        return slot

    def release(self, request: Hashable) -> None:
        self.cache.release(request)
        self.poison_freed_pages()

    def poison_freed_pages(self) -> None:
        """Overwrites the pages that became free since the last call (nothing unless ``poison_freed``).  A page
        that was handed out again meanwhile has not been written by its new holder: no kernel ran in between."""
        if self.poison_freed:
            for g in range(len(self.cache.groups)):
                self.pools.poison_pages(g, self.cache.drain_freed(g))

    def length(self, request: Hashable) -> int:
        return self.cache.length(request)

    def fork(self, parent: Hashable, child: Hashable, tokens: Optional[int] = None) -> int:
        """A new request that shares the full cache pages of ``parent``'s first ``tokens`` tokens.  Returns the
        number of tokens the child holds (a page boundary); the caller feeds it whatever comes after."""
        if not self.pools.state:
            return self.cache.fork(parent, child, tokens)
        # Per-request state exists only for the parent's latest position: the share point has to be there, and
        # the child gets a copy of the state as it is now (pages are shared by reference, state by value).
        length = self.cache.length(parent)
        if tokens is not None and tokens < length:
            raise StepError(f"a model with per-request state shares a prefix only at the parent's latest position "
                            f"({length} tokens), where its state is; asked for {tokens}")
        unit = math.lcm(*[group.page_tokens for group in self.cache.groups]) if self.cache.groups else 1
        if length % unit:
            raise StepError(f"a model with per-request state shares a prefix only at the parent's latest position "
                            f"({length} tokens), and pages are shared whole: every {unit} tokens")
        held = self.cache.fork(parent, child, tokens)
        assert held == length
        self.pools.copy_state(self.cache.slot(parent), self.cache.slot(child))
        return held

    def truncate(self, request: Hashable, position: int) -> None:
        """Cuts a request back to its first ``position`` tokens.  Per-request state cannot be wound back: a model
        that has some can only be cut back to nothing (the state starts from zero again) or not at all."""
        if self.pools.state and position not in (0, self.cache.length(request)):
            raise StepError("a model with per-request state cannot be cut back to a position in between: its state "
                            "exists only for the latest position")
        self.cache.truncate(request, position)
        if self.pools.state and position == 0:
            self.pools.zero_state(self.cache.slot(request))

    # ---- the vendor library's products ---------------------------------------------------
    def tune_products(self, rows: int, candidates: int = 256, thorough: bool = False,
                      keep_only_faster_steps: bool = True) -> List[dict]:
        """Lets the vendor library's products of a step of ``rows`` prompt tokens (the portion size a scheduler
        cuts long prompts into) be run with the fastest of the library's algorithms instead of the one its
        heuristic names.  A trial step of that size on a request of its own shows which products reach the
        library; ``ops.tune_library_product`` times the candidates for each on the model's own matrices; and a
        winner is kept only if the whole trial step is faster with it than without (a product timed by itself
        says too little: at 1,024 rows of the 8B shape the winners of the four products made the step 3 %
        slower; ``keep_only_faster_steps=False`` skips this).  Takes a few seconds (``thorough``: every algorithm of the library, not only the heuristic's
        list); steps of other sizes are not affected.  Needs room for ``rows`` tokens and a free request slot in
        the cache for the moment (without them nothing is tuned).  Returns a record for every product; ``kept``
        says whether its winner is in use."""
        if not ops.library_product_available():
            return []
        rows = min(int(rows), self.max_context)
        request = ("tune products", id(self))
        tokens = [(i * 7919) % self.vocab_size for i in range(rows)]      # varied, as a prompt's are

        def trial_step_ms(repeats: int = 3) -> float:
            best = float("inf")
            for _ in range(repeats):
                torch.cuda.synchronize(self.device)
                started = time.perf_counter()
                self.step([StepEntry(request, tokens, [rows - 1])])
                torch.cuda.synchronize(self.device)
                best = min(best, (time.perf_counter() - started) * 1e3)
                self.release(request)
            return best

        from ..cache.manager import OutOfPages, OutOfSlots
        records = []
        try:
            try:
                with ops.record_library_products() as recorded:
                    trial_step_ms(1)
            except (OutOfPages, OutOfSlots):
                return []                                   # no room for the trial step now: nothing is tuned
            step_ms = trial_step_ms()
            for (m, n, k, out_code, accumulate), weights in recorded.problems.items():
                out_dtype = torch.float32 if out_code == ops.F32 else torch.bfloat16
                record = ops.tune_library_product(m, weights, out_dtype, bool(accumulate), candidates, thorough)
                records.append(record)
                if record["kept"] and keep_only_faster_steps:
                    with_it = trial_step_ms()
                    record["step_ms"], record["step_ms_before"] = round(with_it, 3), round(step_ms, 3)
                    if with_it < step_ms * 0.998:
                        step_ms = with_it
                    else:
                        ops.forget_tuned_products([record["problem"]])
                        record["kept"] = False
        except BaseException:
            # whatever failed, the engine is left as it was found: no winner of this call stays in use
            ops.forget_tuned_products([r["problem"] for r in records if r["kept"]])
            raise
        finally:
            if self.cache.has(request):                     # a trial step that failed half way still holds its request
                self.release(request)
        return records

    # ---- the step --------------------------------------------------------------------
    def _validate(self, entries: Sequence[StepEntry]) -> None:
        """Refuses a malformed step before anything is reserved (the layout routine checks again)."""
        if not entries:
            raise StepError("a step needs at least one entry")
        seen = set()
        for e in entries:
            if e.request in seen:
                raise StepError(f"request {e.request!r} appears twice in one step")
            seen.add(e.request)
            if len(e.tokens) == 0:
                raise StepError(f"request {e.request!r} brings no tokens")
            if len(e.tokens) <= 4:                      # decoded tokens: not worth an array
                fine = all(isinstance(t, (int, np.integer)) and not isinstance(t, bool) and 0 <= t < self.vocab_size
                           for t in e.tokens)
            else:
                tokens = np.asarray(e.tokens)
                fine = tokens.dtype.kind in "iu" and tokens.min() >= 0 and tokens.max() < self.vocab_size
            if not fine:
                raise StepError(f"request {e.request!r}: a token is outside the vocabulary of {self.vocab_size}")
            for w in e.want:
                if not 0 <= int(w) < len(e.tokens):
                    raise StepError(f"request {e.request!r}: wanted place {w} is outside its {len(e.tokens)} tokens")

    def step(self, entries: Sequence[StepEntry], device_tokens: Optional[torch.Tensor] = None) -> StepOutput:
        """Admits unknown requests, reserves pages, runs the tokens and commits.  All or nothing.
        ``device_tokens``: see ``run_reserved``."""
        self._validate(entries)
        admitted, reserved = [], []
        try:
            for e in entries:
                if not self.cache.has(e.request):
                    self.admit(e.request)
                    admitted.append(e.request)
                self.cache.reserve(e.request, len(e.tokens))
                reserved.append(e.request)
        except Exception:
            for request in reserved:
                self.cache.rollback(request)
            for request in admitted:
                self.cache.release(request)
            raise
        return self.run_reserved(entries, device_tokens)

    def run_reserved(self, entries: Sequence[StepEntry], device_tokens: Optional[torch.Tensor] = None) -> StepOutput:
        """Runs a step whose pages the caller has reserved; commits on success, rolls back on failure.

        ``device_tokens`` (int32 ``[entries]`` on the device, for a step of one token an entry): the rows' tokens
        are these, not the entries' (which only stand in): the tokens an earlier step has chosen and that have
        not left the device yet, so that this step can be issued before the host has seen them.  Everything is
        ordered on the stream; a value outside the vocabulary (a row that found no finite logit gives -1) is
        run as the nearest token, for the caller to throw away."""
        if device_tokens is not None:
            if any(len(e.tokens) != 1 for e in entries):
                raise StepError("tokens can be taken from the device only for a step of one token an entry")
            if (device_tokens.dtype != torch.int32 or device_tokens.device != self.device
                    or tuple(device_tokens.shape) != (len(entries),)):
                raise StepError(f"device tokens must be int32 [{len(entries)}] on {self.device}")
        self.poison_freed_pages()              # what a scheduler on the same manager has freed since the last step
        # A failed step gives its pages back (rollback) and leaves per-request state as it found it.
        saved_state = self.pools.snapshot_state([self.cache.slot(e.request) for e in entries])
        try:
            for e in entries:
                if self.cache.length(e.request) == 0:
                    self.pools.zero_state(self.cache.slot(e.request))   # a request's state starts from zero
            # A step that is being profiled runs call by call: a replayed recording has no calls to time.
            if self.graphs and not profile.recording() and all(len(e.tokens) == 1 for e in entries):
                logits, rows = self._run_decode_graph(entries, device_tokens)
            else:
                tokens, context, rows = self._build_context(entries)
                if device_tokens is not None:
                    # entries run in the order the layout gives them: rows of one token each keep the caller's
                    torch.clamp(device_tokens, 0, self.vocab_size - 1, out=tokens)
                caches = self.pools.views(context.block_tables)
                with ops.one_stream():
                    logits = self.model.forward(tokens, context, caches)
        except Exception:
            for e in entries:
                if self.cache.has(e.request):
                    self.cache.rollback(e.request)
            self.pools.restore_state(saved_state)
            raise
        for e in entries:
            self.cache.commit(e.request, len(e.tokens))
        self.poison_freed_pages()              # pages a window has passed
        return StepOutput(logits, rows)

    def _run_decode_graph(self, entries: Sequence[StepEntry], device_tokens: Optional[torch.Tensor] = None):
        """One decoded token for each entry, replayed from the recording for this batch size."""
        state = self._decode_graphs.get(len(entries))
        if state is None:
            state = self._decode_graphs[len(entries)] = _DecodeGraph(self, len(entries))
        packed = state.fill(self, entries)
        if device_tokens is not None:                 # after the upload, on the same stream
            torch.clamp(device_tokens, 0, self.vocab_size - 1, out=state.tokens)
        bucket = context_bucket(packed.max_position + 1, self.max_context)
        recording = state.recordings.get(bucket)
        if recording is None:
            # First step of this size and context range: run it for real on the static buffers, then record
            # the same calls for later steps.  Recording executes nothing, so the cache is written once.
            context = state.context(bucket)
            caches = self.pools.views(context.block_tables)
            with ops.one_stream():
                logits = self.model.forward(state.tokens, context, caches)
            graph = torch.cuda.CUDAGraph()
            # one pool of memory for all recordings: they run one after the other on one stream, and what a
            # replay leaves in its logits is copied out before the next replay begins
            # (errors of the capture are this thread's: an engine in another thread goes on with its own work)
            with torch.cuda.graph(graph, pool=self._graph_pool, capture_error_mode="thread_local"), ops.one_stream():
                recorded_logits = self.model.forward(state.tokens, context, caches)
            state.recordings[bucket] = (graph, recorded_logits)
        else:
            recording[0].replay()
            logits = recording[1]
        wanted, rows_map = [], []
        for i, e in enumerate(entries):
            for w in e.want:
                wanted.append(i)
                rows_map.append((e.request, int(w)))
        if not wanted:
            return None, rows_map
        if wanted == list(range(len(entries))):
            return logits.clone(), rows_map                   # the recording's buffer is reused by the next replay
        index = torch.tensor(wanted, dtype=torch.long, device=self.device)
        return logits.index_select(0, index), rows_map

    def _staging_buffer(self, words: int) -> torch.Tensor:
        """A pinned host buffer for one step's metadata.  Two take turns, each guarded by an event, so that
        the upload need not be waited for and the host can prepare the next step while this one runs."""
        self._staging_turn ^= 1
        held = self._staging[self._staging_turn]
        if held is None or held[0].numel() < words:
            grown = max(words, 4096, 2 * held[0].numel() if held is not None else 0)
            held = (torch.empty(grown, dtype=torch.int32).pin_memory(), torch.cuda.Event())
            self._staging[self._staging_turn] = held
        else:
            held[1].synchronize()                       # its last upload has left the buffer
        return held[0]

    def _build_context(self, entries: Sequence[StepEntry]):
        """The step's metadata, laid out by the native routine and uploaded in one copy."""
        packed = PackedStep(self.cache, self.vocab_size, entries, host=self._staging_buffer, tilings=self.tilings)
        device = torch.empty(max(1, packed.total), dtype=torch.int32, device=self.device)
        device.copy_(packed.host[:max(1, packed.total)], non_blocking=True)
        self._staging[self._staging_turn][1].record()
        pieces = packed.pieces(device)
        infos = [EntryInfo(entries[given].request, slot, first_row, count, start)
                 for given, slot, first_row, count, start in packed.placed]
        rows_map = [(e.request, int(w)) for e in entries for w in e.want]
        n_groups = len(self.cache.groups)
        tiled = {}
        for i, (tiling, (tiled_rows, tiles)) in enumerate(zip(packed.tilings, packed.tiled)):
            if not tiles:
                continue
            cut = [(count, start) for _, _, first_row, count, start in packed.placed if first_row < tiled_rows]
            mean_keys = sum(count * (start + (count + 1) // 2) for count, start in cut) // max(1, sum(c for c, _ in cut))
            tiled[tiling] = TiledRows(tiled_rows, pieces[5 + i].view(-1, 3), mean_keys)
        context = StepContext(
            rows=packed.rows, dtype=self.dtype, device=self.device, positions=pieces[1], row_entry=pieces[2],
            entries=infos, entry_slots=pieces[3], want_rows=pieces[4] if packed.wanted else None,
            block_tables={g: pieces[packed.first_table + g].view(len(entries), -1) for g in range(n_groups)},
            max_position=packed.max_position, decode_only=packed.decode_only, tiled=tiled)
        return pieces[0], context, rows_map

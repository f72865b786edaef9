"""Each part alone against the plain functions, and the generality of the assembly: a toy mixer with
state of its own, a windowed layer without rotation, a layer that runs twice and a run that reads
another run's cache, all defined here and registered without touching the framework's files."""
import json
import math
import os
from dataclasses import dataclass

import numpy as np
import pytest
import torch

from tests import schedules
from tests.plain import qwen3_plain as plain
from tests.util import random_tokens

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def step_context(rows_meta, dtype, tables=None):
    """A StepContext for rows [(entry, position)], in the order given."""
    from leone_amd.parts.context import EntryInfo, StepContext
    positions = torch.tensor([p for _, p in rows_meta], dtype=torch.int32, device=DEV)
    row_entry = torch.tensor([e for e, _ in rows_meta], dtype=torch.int32, device=DEV)
    n_entries = max(e for e, _ in rows_meta) + 1
    infos, row = [], 0
    for e in range(n_entries):
        mine = [p for ee, p in rows_meta if ee == e]
        infos.append(EntryInfo(e, e, row, len(mine), mine[0]))
        row += len(mine)
    return StepContext(rows=len(rows_meta), dtype=dtype, device=torch.device(DEV), positions=positions,
                       row_entry=row_entry, entries=infos,
                       entry_slots=torch.arange(n_entries, dtype=torch.int32, device=DEV), want_rows=None,
                       block_tables=tables or {}, max_position=max(p for _, p in rows_meta))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(dtype):
    from leone_amd.parts import NORMS, PartSpec
    norm = NORMS.build(PartSpec("rmsnorm", {"size": 80, "eps": 3e-6, "weight": "g"}))
    assert [(s.name, s.shape) for s in norm.tensor_specs()] == [("g", (80,))]
    gain = 1 + 0.1 * torch.randn(80)
    norm.bind({"g": gain.to(DEV)})
    x = torch.randn(5, 80, device=DEV)
    delta = torch.randn(5, 80, device=DEV).to(dtype)
    want = plain.rms_norm(x.cpu().double() + delta.cpu().double(), gain, 3e-6)
    y = norm.add_norm(x, delta, dtype)
    tol = 2e-5 if dtype == torch.float32 else 1e-2
    assert (y.cpu().double() - want).abs().max() < tol * (1 + want.abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_part(dtype):
    from leone_amd.parts import FEED_FORWARDS, PartSpec
    ffn = FEED_FORWARDS.build(PartSpec("swiglu", {"hidden": 80, "intermediate": 176, "gate": "g", "up": "u", "down": "d"}))
    assert [(s.name, s.shape) for s in ffn.tensor_specs()] == [("g", (176, 80)), ("u", (176, 80)), ("d", (80, 176))]
    w = {"g": torch.randn(176, 80) * 0.1, "u": torch.randn(176, 80) * 0.1, "d": torch.randn(80, 176) * 0.1}
    w = {k: v.to(dtype) for k, v in w.items()}
    ffn.bind({k: v.to(DEV) for k, v in w.items()})
    y = torch.randn(9, 80).to(dtype)
    out = ffn.forward(y.to(DEV), step_context([(0, i) for i in range(9)], dtype))
    want = plain.feed_forward(y.float(), {f"p.{k}_proj.weight": v.float() for k, v in
                                          (("gate", w["g"]), ("up", w["u"]), ("down", w["d"]))}, "p")
    tol = 1e-5 if dtype == torch.float32 else 3e-2
    assert (out.cpu().double() - want).abs().max() < tol * (1 + want.abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_part_with_portions_and_two_requests(dtype):
    """Two requests; the second is fed in two calls (a portion, then one token).  Scores are sharpened
    by a large q/k gain so that one key dominates each row: a misplaced key changes the result by
    far more than bfloat16 rounding."""
    from leone_amd.parts import MIXERS, POSITIONS, PartSpec
    from leone_amd.parts.context import KvCacheView
    hidden, q_heads, kv_heads, dim, page = 96, 6, 2, 32, 16
    rope = POSITIONS.build(PartSpec("rope_half_split", {"rotary_dim": dim, "theta": 1e4}))
    rope.prepare(256, DEV)
    names = {k: k for k in ("q", "k", "v", "o", "q_norm", "k_norm")}
    mixer = MIXERS.build(PartSpec("gqa_attention", dict(hidden=hidden, q_heads=q_heads, kv_heads=kv_heads, head_dim=dim,
                                                        qk_norm_eps=1e-5, window=None, position="rope", **names)),
                         positions={"rope": rope})
    torch.manual_seed(3)
    w = {"q": torch.randn(q_heads * dim, hidden) * 0.1, "k": torch.randn(kv_heads * dim, hidden) * 0.1,
         "v": torch.randn(kv_heads * dim, hidden) * 0.1, "o": torch.randn(hidden, q_heads * dim) * 0.1,
         "q_norm": torch.full((dim,), 3.0), "k_norm": torch.full((dim,), 3.0)}
    w = {k: v.to(dtype) for k, v in w.items()}
    mixer.bind({k: v.to(DEV) for k, v in w.items()})
    assert mixer.cache_need().kv_heads == kv_heads
    lengths = [40, 21]
    ys = [torch.randn(n, hidden).to(dtype) for n in lengths]
    pw = {f"a.{k}_proj.weight": w[k].float() for k in ("q", "k", "v", "o")}
    pw.update({"a.q_norm.weight": w["q_norm"].float(), "a.k_norm.weight": w["k_norm"].float()})
    cfg = dict(num_attention_heads=q_heads, num_key_value_heads=kv_heads, head_dim=dim, rms_norm_eps=1e-5, rope_theta=1e4)
    want = [plain.attention_block(y.float(), pw, "a", cfg, list(range(len(y)))) for y in ys]
    k_pool = torch.full((8, kv_heads, dim // 8, page, 8), float("nan"), dtype=dtype, device=DEV)
    v_pool = torch.full((8, kv_heads, page // 8, dim, 8), float("nan"), dtype=dtype, device=DEV)
    table = torch.tensor([[5, 0, 3, -1], [7, 2, -1, -1]], dtype=torch.int32, device=DEV)
    cache = KvCacheView(writes=True, k_pool=k_pool, v_pool=v_pool, block_table=table, page_tokens=page)
    # call 1: all of request 0 and the first 20 tokens of request 1
    meta = [(0, p) for p in range(40)] + [(1, p) for p in range(20)]
    out1 = mixer.forward(torch.cat([ys[0], ys[1][:20]]).to(DEV), step_context(meta, dtype, {0: table}), cache)
    # call 2: the last token of request 1 alone, as entry 0 of its step
    cache2 = KvCacheView(writes=True, k_pool=k_pool, v_pool=v_pool, block_table=table[1:2].contiguous(), page_tokens=page)
    out2 = mixer.forward(ys[1][20:21].to(DEV), step_context([(0, 20)], dtype, {0: table[1:2]}), cache2)
    have = [out1[:40], torch.cat([out1[40:], out2])]
    tol = 2e-5 if dtype == torch.float32 else 4e-2
    for r in range(2):
        err = (have[r].cpu().double() - want[r]).abs().max(dim=1).values
        assert float(err.max()) < tol * (1 + float(want[r].abs().max())), (r, int(err.argmax()), float(err.max()))


@pytest.mark.parametrize("position_kind, rotary_dim", [("rope_half_split", 32), ("rope_adjacent", 64), ("rope_half_split", 64)])
def test_attention_part_takes_the_rotation_shape_from_its_position_part(position_kind, rotary_dim):
    """The mixer assumes no shape of rotation: a position part that rotates half a head, or adjacent pairs,
    is handed to the kernels as it is.  At head size 64 in bfloat16 the decode kernel that makes the heads
    itself only knows the whole head in half-split pairs; for the other shapes the mixer must take the two
    kernels instead, and says which it takes.  A prompt portion, then single tokens of two requests."""
    from leone_amd.parts import MIXERS, POSITIONS, PartSpec
    from leone_amd.parts.context import KvCacheView
    dtype = torch.bfloat16
    hidden, q_heads, kv_heads, dim, page = 64, 4, 2, 64, 16
    rope = POSITIONS.build(PartSpec(position_kind, {"rotary_dim": rotary_dim, "theta": 1e4}))
    rope.prepare(128, DEV)
    pairing = "adjacent" if position_kind == "rope_adjacent" else "half_split"
    assert rope.rotation().pairing == pairing and rope.rotation().rotary_dim == rotary_dim
    names = {k: k for k in ("q", "k", "v", "o", "q_norm", "k_norm")}
    mixer = MIXERS.build(PartSpec("gqa_attention", dict(hidden=hidden, q_heads=q_heads, kv_heads=kv_heads, head_dim=dim,
                                                        qk_norm_eps=1e-5, window=None, position="rope", **names)),
                         positions={"rope": rope})
    whole = rotary_dim == dim and pairing == "half_split"
    assert mixer.attention_kernels(dtype, page) == {"decode": "projected" if whole else "split_kv", "prompt": "flash"}
    torch.manual_seed(4)
    w = {"q": torch.randn(q_heads * dim, hidden) * 0.1, "k": torch.randn(kv_heads * dim, hidden) * 0.1,
         "v": torch.randn(kv_heads * dim, hidden) * 0.1, "o": torch.randn(hidden, q_heads * dim) * 0.1,
         "q_norm": torch.full((dim,), 3.0), "k_norm": torch.full((dim,), 3.0)}
    w = {k: v.to(dtype) for k, v in w.items()}
    mixer.bind({k: v.to(DEV) for k, v in w.items()})
    lengths = [37, 22]
    ys = [torch.randn(n, hidden).to(dtype) for n in lengths]
    pw = {f"a.{k}_proj.weight": w[k].float() for k in ("q", "k", "v", "o")}
    pw.update({"a.q_norm.weight": w["q_norm"].float(), "a.k_norm.weight": w["k_norm"].float()})
    cfg = dict(num_attention_heads=q_heads, num_key_value_heads=kv_heads, head_dim=dim, rms_norm_eps=1e-5, rope_theta=1e4,
               rotary_dim=rotary_dim, rope_pairing=pairing)
    want = [plain.attention_block(y.float(), pw, "a", cfg, list(range(len(y)))) for y in ys]
    other = plain.attention_block(ys[0].float(), pw, "a", dict(cfg, rotary_dim=dim, rope_pairing="half_split"), list(range(lengths[0])))
    assert whole or (other - want[0]).abs().max() > 0.2 * want[0].abs().max()       # the shapes can be told apart
    k_pool = torch.full((8, kv_heads, dim // 8, page, 8), float("nan"), dtype=dtype, device=DEV)
    v_pool = torch.full((8, kv_heads, page // 8, dim, 8), float("nan"), dtype=dtype, device=DEV)
    table = torch.tensor([[5, 0, 3, -1], [7, 2, -1, -1]], dtype=torch.int32, device=DEV)
    cache = KvCacheView(writes=True, k_pool=k_pool, v_pool=v_pool, block_table=table, page_tokens=page)
    meta = [(0, p) for p in range(33)] + [(1, p) for p in range(18)]
    out = mixer.forward(torch.cat([ys[0][:33], ys[1][:18]]).to(DEV), step_context(meta, dtype, {0: table}), cache)
    have = [[out[:33]], [out[33:]]]
    for i in range(4):                                  # single tokens of both requests: a decode-only step
        context = step_context([(0, 33 + i), (1, 18 + i)], dtype, {0: table})
        context.decode_only = True
        step = mixer.forward(torch.stack([ys[0][33 + i], ys[1][18 + i]]).to(DEV), context, cache)
        have[0].append(step[0:1])
        have[1].append(step[1:2])
    for r in range(2):
        got = torch.cat(have[r]).cpu().double()
        err = (got - want[r]).abs().max(dim=1).values
        assert float(err.max()) < 4e-2 * (1 + float(want[r].abs().max())), (r, int(err.argmax()), float(err.max()))


# ---- a toy architecture assembled from the framework's parts and one part defined here --------------

DECAY = 0.75


def register_toy():
    from leone_amd.architectures import register_architecture
    from leone_amd.config.base import FieldReader
    from leone_amd.parts import MIXERS, Part, PartSpec, RowTiling, StateNeed
    from leone_amd.parts.context import CacheView
    from leone_amd.parts.model import LayerRun, ModelSpec
    from leone_amd.weights.loader import MATRIX, TensorSpec
    from leone_amd import ops

    class DecayMixer(Part):
        """s_t = decay * s_{t-1} + y_t per request; out_t = W s_t.  Its state lives in the per-request slot."""

        def __init__(self, spec, **_):
            self.hidden, self.decay, self.name = spec["hidden"], spec["decay"], spec["weight"]

        def tensor_specs(self):
            return [TensorSpec(self.name, (self.hidden, self.hidden), MATRIX)]

        def bind(self, tensors):
            self.weight = tensors.pop(self.name).contiguous()

        def cache_need(self):
            return StateNeed((self.hidden,), torch.float32)

        def forward(self, y, step, cache):
            states = torch.empty((step.rows, self.hidden), dtype=torch.float32, device=y.device)
            for entry in step.entries:
                s = cache.state[entry.slot].clone()
                for r in range(entry.first_row, entry.first_row + entry.count):
                    s = self.decay * s + y[r].float()
                    states[r] = s
                if cache.writes:
                    cache.state[entry.slot] = s
            return ops.linear(states.to(y.dtype), self.weight)

    @dataclass(frozen=True)
    class VectorNeed:
        """A kind of cache the framework does not have: one float32 vector per token, in pages of its own size."""
        width: int
        page_tokens: int = 4
        window = None
        paged = True

        def group_key(self):
            return self

        def allocate(self, pages, page_tokens, dtype, device):
            return torch.zeros((pages, page_tokens, self.width), dtype=torch.float32, device=device)

        def view(self, storage, block_table, page_tokens):
            view = CacheView(writes=True)
            view.vectors, view.block_table, view.page_tokens = storage, block_table, page_tokens
            return view

        def poison(self, storage, index):
            storage.index_fill_(0, index, float("nan"))

        def bytes_per_token(self, element_size):
            return 4 * self.width

    class PrefixMeanMixer(Part):
        """out_t = W mean(y_0 .. y_t) per request: every y is kept in the cache (a ``VectorNeed``), so that a
        later step finds the earlier ones.  It has a row kernel of its own, as it were: portions of 6 rows and
        more it takes tile by tile (tiles of 8 rows, two to a group), the other rows one by one."""

        TILING = RowTiling(tile_rows=8, group_tiles=2, min_rows=6)

        def __init__(self, spec, **_):
            self.hidden, self.name = spec["hidden"], spec["weight"]
            self.tiles_seen = []

        def tensor_specs(self):
            return [TensorSpec(self.name, (self.hidden, self.hidden), MATRIX)]

        def bind(self, tensors):
            self.weight = tensors.pop(self.name).contiguous()

        def cache_need(self):
            return VectorNeed(self.hidden)

        def row_tiling(self):
            return self.TILING

        def forward(self, y, step, cache):
            assert cache.page_tokens == 4
            table = cache.block_table.cpu()
            positions, row_entry = step.positions.cpu().tolist(), step.row_entry.cpu().tolist()
            for r in range(step.rows):                                   # every row's vector into its page
                page = int(table[row_entry[r], positions[r] // 4])
                cache.vectors[page, positions[r] % 4] = y[r].float()
            means = torch.empty((step.rows, self.hidden), dtype=torch.float32, device=y.device)

            def mean_of(r):
                pages = table[row_entry[r], :positions[r] // 4 + 1].to(y.device).long()
                return cache.vectors[pages].reshape(-1, self.hidden)[:positions[r] + 1].mean(dim=0)

            tiled = step.tiled.get(self.TILING)
            covered = 0
            if tiled is not None:
                listed = tiled.tiles.cpu().tolist()
                assert len(listed) % 2 == 0
                self.tiles_seen.append(listed)
                for entry, first_row, rows in listed:
                    assert rows <= 8 and all(row_entry[r] == entry for r in range(first_row, first_row + rows))
                    for r in range(first_row, first_row + rows):
                        means[r] = mean_of(r)
                covered = tiled.rows
                assert sum(rows for _, _, rows in listed) == covered
            for info in step.entries:                                    # the layout's promise about the rest
                assert (info.first_row < covered) == (info.count >= 6)
            for r in range(covered, step.rows):
                means[r] = mean_of(r)
            return ops.linear(means.to(y.dtype), self.weight)

    if "toy_decay" not in MIXERS.kinds():
        MIXERS.register("toy_decay", DecayMixer)
        MIXERS.register("toy_prefix_mean", PrefixMeanMixer)

    @dataclass(frozen=True)
    class ToyConfig:
        architecture: str
        hidden: int
        heads: int
        kv_heads: int
        head_dim: int
        ffn: int
        vocab: int
        window: int
        eps: float
        max_positions: int

        @classmethod
        def from_dict(cls, raw):
            r = FieldReader(raw)
            return cls("ToyForCausalLM", r.positive_int("hidden"), r.positive_int("heads"), r.positive_int("kv_heads"),
                       r.positive_int("head_dim"), r.positive_int("ffn"), r.positive_int("vocab"),
                       r.positive_int("window"), r.positive_float("eps"), r.positive_int("max_positions"))

    def spec(c):
        def norm(name):
            return PartSpec("rmsnorm", {"size": c.hidden, "eps": c.eps, "weight": name})

        def ffn(p):
            return PartSpec("swiglu", {"hidden": c.hidden, "intermediate": c.ffn, "gate": f"{p}.gate", "up": f"{p}.up",
                                       "down": f"{p}.down"})

        def attention(p, window, rope, qk_norm):
            params = dict(hidden=c.hidden, q_heads=c.heads, kv_heads=c.kv_heads, head_dim=c.head_dim,
                          qk_norm_eps=c.eps if qk_norm else None, window=window, position="rope" if rope else None,
                          q=f"{p}.q", k=f"{p}.k", v=f"{p}.v", o=f"{p}.o")
            if qk_norm:
                params.update(q_norm=f"{p}.qn", k_norm=f"{p}.kn")
            return PartSpec("gqa_attention", params)

        layers = [
            PartSpec("prenorm", {"norm1": norm("l0.n1"), "mixer": attention("l0", None, True, True),
                                 "norm2": norm("l0.n2"), "feed_forward": ffn("l0")}),
            PartSpec("prenorm", {"norm1": norm("l1.n1"),
                                 "mixer": PartSpec("toy_decay", {"hidden": c.hidden, "decay": DECAY, "weight": "l1.w"}),
                                 "norm2": norm("l1.n2"), "feed_forward": ffn("l1")}),
            PartSpec("prenorm", {"norm1": norm("l2.n1"), "mixer": attention("l2", c.window, False, False),
                                 "norm2": norm("l2.n2"), "feed_forward": ffn("l2")}),
            PartSpec("prenorm", {"norm1": norm("l3.n1"),
                                 "mixer": PartSpec("toy_prefix_mean", {"hidden": c.hidden, "weight": "l3.w"}),
                                 "norm2": norm("l3.n2"), "feed_forward": ffn("l3")}),
        ]
        # layer 1 runs twice, each run with state of its own; the last run is layer 0 again, reading the
        # keys and values its first run wrote, writing none
        order = [LayerRun(0, 0), LayerRun(1, 1), LayerRun(2, 2), LayerRun(3, 4), LayerRun(1, 3),
                 LayerRun(0, 0, writes=False)]
        return ModelSpec(hidden_size=c.hidden, vocab_size=c.vocab, max_positions=c.max_positions, embedding="emb",
                         layers=layers, schedule=order, final_norm=norm("final"), head="head",
                         positions={"rope": PartSpec("rope_half_split", {"rotary_dim": c.head_dim, "theta": 5000.0})})

    register_architecture("ToyForCausalLM", ToyConfig.from_dict, spec)


TOY = dict(architectures=["ToyForCausalLM"], hidden=48, heads=3, kv_heads=1, head_dim=16, ffn=80, vocab=301, window=11,
           eps=1e-5, max_positions=256)


def toy_plain(w, tokens):
    """The toy model with the plain functions, whole sequence."""
    c = TOY
    n = len(tokens)
    positions = list(range(n))

    def ffn(x, p):
        y = plain.rms_norm(x, w[f"{p}.n2"], c["eps"])
        return x + plain.linear(plain.swiglu(plain.linear(y, w[f"{p}.gate"]), plain.linear(y, w[f"{p}.up"])), w[f"{p}.down"])

    def heads(y, name, count):
        return plain.linear(y, w[name]).view(n, count, c["head_dim"])

    x = plain.embedding(w["emb"], tokens)
    # run 1: layer 0, full attention with q/k norm and rotation; its keys and values are kept
    y = plain.rms_norm(x, w["l0.n1"], c["eps"])
    k0 = plain.rope_half_split(plain.rms_norm(heads(y, "l0.k", 1), w["l0.kn"], c["eps"]), positions, 5000.0)
    v0 = heads(y, "l0.v", 1)
    q = plain.rope_half_split(plain.rms_norm(heads(y, "l0.q", 3), w["l0.qn"], c["eps"]), positions, 5000.0)
    x = ffn(x + plain.linear(plain.causal_attention(q, k0, v0).reshape(n, -1), w["l0.o"]), "l0")

    def decay_layer(x):
        y = plain.rms_norm(x, w["l1.n1"], c["eps"])
        s, rows = torch.zeros(c["hidden"], dtype=torch.float64), []
        for t in range(n):
            s = DECAY * s + y[t]
            rows.append(s)
        return ffn(x + plain.linear(torch.stack(rows), w["l1.w"]), "l1")

    x = decay_layer(x)
    # run 3: layer 2, window of 11 keys, no q/k norm, no rotation
    y = plain.rms_norm(x, w["l2.n1"], c["eps"])
    att = plain.causal_attention(heads(y, "l2.q", 3), heads(y, "l2.k", 1), heads(y, "l2.v", 1), window=c["window"])
    x = ffn(x + plain.linear(att.reshape(n, -1), w["l2.o"]), "l2")
    # run 4: layer 3, the mean of everything so far
    y = plain.rms_norm(x, w["l3.n1"], c["eps"])
    means = torch.cumsum(y, dim=0) / torch.arange(1, n + 1, dtype=torch.float64)[:, None]
    x = ffn(x + plain.linear(means, w["l3.w"]), "l3")
    x = decay_layer(x)                      # run 5: layer 1 again, state of its own, starting from zero
    # run 6: layer 0 again: new queries over the keys and values of run 1
    y = plain.rms_norm(x, w["l0.n1"], c["eps"])
    q = plain.rope_half_split(plain.rms_norm(heads(y, "l0.q", 3), w["l0.qn"], c["eps"]), positions, 5000.0)
    x = ffn(x + plain.linear(plain.causal_attention(q, k0, v0).reshape(n, -1), w["l0.o"]), "l0")
    return plain.linear(plain.rms_norm(x, w["final"], c["eps"]), w["head"])


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_toy_architecture_with_state_window_repeat_and_shared_cache(tmp_path, dtype_name):
    from leone_amd.architectures import config_from_dict, model_spec_for, unregister_architecture
    from leone_amd.engine.engine import Engine, StepEntry
    from leone_amd.parts import MIXERS
    from leone_amd.parts.model import DecoderModel
    from leone_amd.runtime import load_model
    from leone_amd.weights.random_init import host_tensors
    from leone_amd.weights.safetensors_io import write_file

    register_toy()
    try:
        dtype = torch.float32 if dtype_name == "float32" else torch.bfloat16
        folder = str(tmp_path / "toy")
        os.makedirs(folder)
        json.dump(TOY, open(os.path.join(folder, "config.json"), "w"))
        config = config_from_dict(TOY)
        specs = DecoderModel(model_spec_for(config), torch.float32, "cpu").tensor_specs()
        assert len({s.name for s in specs}) == len(specs)
        tensors = host_tensors(specs, 77, dtype)
        for name in tensors:
            if name.endswith(".w"):
                tensors[name] = (tensors[name].float() * 0.3).to(dtype)     # keep the decaying sum's output small
        write_file(os.path.join(folder, "model.safetensors"), tensors)
        model = load_model(folder, dtype_name)
        needs = model.cache_needs()
        assert sorted(needs) == [0, 1, 2, 3, 4]
        engine = Engine(model, num_pages=36, page_tokens=8, max_requests=3, poison_freed=True)
        # three groups: all keys, a window of 11, and the toy's own kind of cache with pages of 4 tokens
        assert [(g.window or 0, g.page_tokens) for g in engine.cache.groups] == [(0, 8), (11, 8), (0, 4)]
        # two tilings: the attention mixer's and the toy's
        assert len(engine.tilings) == 2 and {t.tile_rows for t in engine.tilings} == {8, 32}
        requests = {f"t{i}": random_tokens(900 + i, n, TOY["vocab"]) for i, n in enumerate([45, 30, 9, 38])}
        weights = {k: v.float() for k, v in tensors.items()}
        expected = {rid: toy_plain(weights, toks).numpy() for rid, toks in requests.items()}
        tol = 1e-4 if dtype_name == "float32" else 4e-2
        for mode in ("whole", "portions", "mixed"):
            steps = getattr(schedules, mode)(requests, **({"max_live": 3} if mode == "mixed" else {}))
            outputs = {}
            for s in steps:
                out = engine.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
                outputs[s["step"]] = out.logits.cpu().numpy()
                for rid in s["end"]:
                    engine.release(rid)
                engine.cache.check()
            got = schedules.collect(steps, outputs)
            for rid, rows in got.items():
                err = np.abs(np.stack(rows) - expected[rid]).max(axis=1)
                assert np.isfinite(err).all() and err.max() <= tol, (mode, rid, int(err.argmax()), float(err.max()))
            # the windowed group never holds more than ceil((window - 1 + longest portion) / page) + 1 pages a request
            assert all(engine.cache.free_pages(g) == 36 for g in range(3))
        assert any(len(listed) > 2 for listed in model.layers[3].mixer.tiles_seen)        # the toy's tiles were used
        # A step that fails half way leaves pages and per-request state as they were: the first half of a
        # request, then its second half fails after the state mixers have run; run again it gives the same
        # logits as if nothing had happened.
        tokens = requests["t0"]
        engine.step([StepEntry("f", tokens[:20], [])])
        state_before = {slot: tensor.clone() for slot, tensor in engine.pools.state.items()}
        free_before = [engine.cache.free_pages(g) for g in range(3)]
        last = model.layers[0].feed_forward
        real = last.forward
        calls = []

        def failing(*args, **kwargs):
            calls.append(1)
            if len(calls) == 2:                     # layer 0 runs twice a step: its second run comes last
                raise RuntimeError("injected")
            return real(*args, **kwargs)
        last.forward = failing
        try:
            with pytest.raises(RuntimeError, match="injected"):
                engine.step([StepEntry("f", tokens[20:], list(range(len(tokens) - 20)))])
        finally:
            last.forward = real
        assert engine.cache.length("f") == 20 and [engine.cache.free_pages(g) for g in range(3)] == free_before
        for slot, tensor in engine.pools.state.items():
            assert torch.equal(tensor, state_before[slot])
        out = engine.step([StepEntry("f", tokens[20:], list(range(len(tokens) - 20)))])
        err = np.abs(out.logits.cpu().numpy() - expected["t0"][20:]).max()
        assert err <= tol, err
        engine.release("f")
        engine.cache.check()
        # A prefix is shared at the parent's latest position, where its state is: the child gets the pages by
        # reference and a copy of the state, and both go on with tokens of their own.  Anywhere else it is refused
        # and nothing is left behind; a request with state is cut back to nothing or not at all.
        from leone_amd.engine.engine import StepError
        first, second = requests["t0"], requests["t3"]
        other = first[:24] + second[:14]
        want_other = toy_plain(weights, other).numpy()
        engine.step([StepEntry("p", first[:20], [])])
        with pytest.raises(StepError, match="latest position"):
            engine.fork("p", "c")                          # 20 tokens: pages are shared whole, 16 could be
        with pytest.raises(StepError, match="latest position"):
            engine.fork("p", "c", 16)
        assert not engine.cache.has("c")
        engine.step([StepEntry("p", first[20:24], [])])
        assert engine.fork("p", "c") == 24 and engine.cache.shared_pages(0) > 0
        out_child = engine.step([StepEntry("c", other[24:], list(range(14)))]).logits.cpu().numpy()
        out_parent = engine.step([StepEntry("p", first[24:], list(range(len(first) - 24)))]).logits.cpu().numpy()
        assert np.abs(out_child - want_other[24:]).max() <= tol and np.abs(out_parent - expected["t0"][24:]).max() <= tol
        with pytest.raises(StepError, match="in between"):
            engine.truncate("c", 8)
        engine.truncate("c", 0)                            # its state starts from zero again
        again = engine.step([StepEntry("c", second, list(range(len(second))))]).logits.cpu().numpy()
        assert np.abs(again - expected["t3"]).max() <= tol
        engine.release("p"), engine.release("c")
        engine.cache.check()
        assert all(engine.cache.free_pages(g) == 36 for g in range(3))
        # The generation loop on this model (state, a window, pages of two sizes; no recording, one of its parts is
        # not safe to record): steps issued ahead of the tokens give the tokens that steps one by one give, and
        # the plain implementation's greedy choice in float32.
        from leone_amd.engine.generate import Generator
        from leone_amd.engine.scheduler import SchedulerPolicy
        assert not engine.graphs
        prompts = [requests["t0"][:19], requests["t1"][:7], requests["t3"][:30]]
        outcomes = []
        for look_ahead in (False, True):
            generator = Generator(engine, SchedulerPolicy(max_live_requests=3, prefill_chunk_tokens=8, max_step_tokens=16))
            generator.look_ahead = look_ahead
            for i, prompt in enumerate(prompts):
                generator.submit(i, prompt, 12, None, None)
            finished = {f.id: f.tokens for f in generator.run()}
            outcomes.append([finished[i] for i in range(len(prompts))])
            assert (generator.stats.steps_ahead > 5) == look_ahead
            engine.cache.check()
        assert outcomes[0] == outcomes[1]
        if dtype_name == "float32":
            for prompt, tokens in zip(prompts, outcomes[1]):
                history = list(prompt)
                for token in tokens:
                    assert int(toy_plain(weights, history)[-1].argmax()) == token
                    history.append(token)
    finally:
        unregister_architecture("ToyForCausalLM")
        MIXERS.unregister("toy_decay")
        MIXERS.unregister("toy_prefix_mean")


# ---- a second toy: a feed-forward that routes rows to experts, and another position encoding -------------

SLOW = 4.0          # the second half of the rotary pairs turns this much slower
TOY2 = dict(architectures=["ToyRoutedForCausalLM"], hidden=32, heads=2, kv_heads=2, head_dim=16, ffn=24, experts=3,
            vocab=97, eps=1e-5, max_positions=128)


def register_routed_toy():
    from leone_amd.architectures import register_architecture
    from leone_amd.config.base import FieldReader
    from leone_amd.parts import FEED_FORWARDS, POSITIONS, Part, PartSpec
    from leone_amd.parts.model import ModelSpec, default_schedule
    from leone_amd.weights.loader import MATRIX, TensorSpec

    class TopOneExperts(Part):
        """Every row goes to the expert with the highest router logit (float32; the lowest index on a tie):
        out = down_e(relu(up_e y)).  Rows are grouped by expert inside; nothing outside knows."""

        def __init__(self, spec, **_):
            self.hidden, self.ffn, self.experts, self.prefix = spec["hidden"], spec["ffn"], spec["experts"], spec["prefix"]

        def tensor_specs(self):
            specs = [TensorSpec(f"{self.prefix}.router", (self.experts, self.hidden), MATRIX)]
            for e in range(self.experts):
                specs += [TensorSpec(f"{self.prefix}.up{e}", (self.ffn, self.hidden), MATRIX),
                          TensorSpec(f"{self.prefix}.down{e}", (self.hidden, self.ffn), MATRIX)]
            return specs

        def bind(self, tensors):
            self.router = tensors.pop(f"{self.prefix}.router").float()
            self.up = [tensors.pop(f"{self.prefix}.up{e}") for e in range(self.experts)]
            self.down = [tensors.pop(f"{self.prefix}.down{e}") for e in range(self.experts)]

        def forward(self, y, step):
            choice = (y.float() @ self.router.t()).argmax(dim=1)          # first of equal maxima
            out = torch.zeros((y.shape[0], self.hidden), dtype=y.dtype, device=y.device)
            for e in range(self.experts):
                rows = (choice == e).nonzero().flatten()
                if rows.numel():
                    hidden = torch.relu(torch.nn.functional.linear(y[rows], self.up[e]))
                    out[rows] = torch.nn.functional.linear(hidden, self.down[e])
            return out

    class TwoSpeedRotary(Part):
        """Half-split rotary pairs whose second half turns SLOW times slower (a per-pair frequency factor,
        the reference's hook at crates/leone/src/cpu.rs:1739-1742).  It hands the mixer tables like the
        framework's own rotary part."""
        graph_safe = True

        def __init__(self, spec, **_):
            self.dim, self.theta = spec["rotary_dim"], spec["theta"]

        def prepare(self, max_positions, device):
            half = self.dim // 2
            inv = torch.tensor([self.theta ** (-2.0 * i / self.dim) / (SLOW if i >= half // 2 else 1.0)
                                for i in range(half)], dtype=torch.float64)
            angles = torch.arange(max_positions, dtype=torch.float64)[:, None] * inv[None, :]
            self.cos, self.sin = angles.cos().float().to(device), angles.sin().float().to(device)

        def tables(self):
            return self.cos, self.sin

    if "toy_top_one" not in FEED_FORWARDS.kinds():
        FEED_FORWARDS.register("toy_top_one", TopOneExperts)
    if "toy_two_speed" not in POSITIONS.kinds():
        POSITIONS.register("toy_two_speed", TwoSpeedRotary)

    @dataclass(frozen=True)
    class Config:
        architecture: str
        raw: tuple

        @classmethod
        def from_dict(cls, raw):
            r = FieldReader(raw)
            keys = ("hidden", "heads", "kv_heads", "head_dim", "ffn", "experts", "vocab", "max_positions")
            return cls("ToyRoutedForCausalLM", tuple((k, r.positive_int(k)) for k in keys) + (("eps", r.positive_float("eps")),))

    def spec(config):
        c = dict(config.raw)

        def norm(name):
            return PartSpec("rmsnorm", {"size": c["hidden"], "eps": c["eps"], "weight": name})

        layers = []
        for l in range(2):
            attention = PartSpec("gqa_attention", dict(
                hidden=c["hidden"], q_heads=c["heads"], kv_heads=c["kv_heads"], head_dim=c["head_dim"], qk_norm_eps=None,
                window=None, position="slow", q=f"l{l}.q", k=f"l{l}.k", v=f"l{l}.v", o=f"l{l}.o"))
            experts = PartSpec("toy_top_one", dict(hidden=c["hidden"], ffn=c["ffn"], experts=c["experts"], prefix=f"l{l}.moe"))
            layers.append(PartSpec("prenorm", {"norm1": norm(f"l{l}.n1"), "mixer": attention, "norm2": norm(f"l{l}.n2"),
                                               "feed_forward": experts}))
        return ModelSpec(hidden_size=c["hidden"], vocab_size=c["vocab"], max_positions=c["max_positions"], embedding="emb",
                         layers=layers, schedule=default_schedule(2), final_norm=norm("final"), head="head",
                         positions={"slow": PartSpec("toy_two_speed", {"rotary_dim": c["head_dim"], "theta": 300.0})})

    register_architecture("ToyRoutedForCausalLM", Config.from_dict, spec)


def routed_plain(w, tokens):
    c, n = TOY2, len(tokens)
    x = plain.embedding(w["emb"], tokens)

    def rotate(t):                                                     # [n, heads, D], the toy's own angles
        out, half = t.clone(), c["head_dim"] // 2
        for pos in range(n):
            for i in range(half):
                angle = pos * 300.0 ** (-2.0 * i / c["head_dim"]) / (SLOW if i >= half // 2 else 1.0)
                a, b = t[pos, :, i], t[pos, :, i + half]
                out[pos, :, i] = a * math.cos(angle) - b * math.sin(angle)
                out[pos, :, i + half] = a * math.sin(angle) + b * math.cos(angle)
        return out

    for l in range(2):
        y = plain.rms_norm(x, w[f"l{l}.n1"], c["eps"])
        q, k, v = (plain.linear(y, w[f"l{l}.{m}"]).view(n, 2, c["head_dim"]) for m in "qkv")
        x = x + plain.linear(plain.causal_attention(rotate(q), rotate(k), v).reshape(n, -1), w[f"l{l}.o"])
        y = plain.rms_norm(x, w[f"l{l}.n2"], c["eps"])
        rows = []
        for t in range(n):
            logits = plain.linear(y[t:t + 1], w[f"l{l}.moe.router"])[0]
            e = int(logits.argmax())
            hidden = torch.clamp(plain.linear(y[t:t + 1], w[f"l{l}.moe.up{e}"]), min=0.0)
            rows.append(plain.linear(hidden, w[f"l{l}.moe.down{e}"])[0])
        x = x + torch.stack(rows)
    return plain.linear(plain.rms_norm(x, w["final"], c["eps"]), w["head"])


def test_toy_architecture_with_routed_feed_forward_and_another_position_encoding(tmp_path):
    """Float32 only: a router's choice between two nearly equal experts is not stable under bfloat16
    rounding, and a different choice is not a rounding difference."""
    from leone_amd.architectures import config_from_dict, model_spec_for, unregister_architecture
    from leone_amd.engine.engine import Engine, StepEntry
    from leone_amd.parts import FEED_FORWARDS, POSITIONS
    from leone_amd.parts.model import DecoderModel
    from leone_amd.runtime import load_model
    from leone_amd.weights.random_init import host_tensors
    from leone_amd.weights.safetensors_io import write_file

    register_routed_toy()
    try:
        folder = str(tmp_path / "routed")
        os.makedirs(folder)
        json.dump(TOY2, open(os.path.join(folder, "config.json"), "w"))
        specs = DecoderModel(model_spec_for(config_from_dict(TOY2)), torch.float32, "cpu").tensor_specs()
        tensors = host_tensors(specs, 5, torch.float32)
        for name in tensors:
            if name.endswith("router"):
                tensors[name] = tensors[name] * 40.0                    # clear choices, all experts in use
        write_file(os.path.join(folder, "model.safetensors"), tensors)
        model = load_model(folder, "float32")
        engine = Engine(model, num_pages=12, page_tokens=8, max_requests=3, poison_freed=True)
        assert not engine.graphs                                        # the routed part does not claim to be graph-safe
        requests = {f"r{i}": random_tokens(40 + i, n, TOY2["vocab"]) for i, n in enumerate([33, 21, 40])}
        expected = {rid: routed_plain({k: v.double() for k, v in tensors.items()}, toks).numpy()
                    for rid, toks in requests.items()}
        used = set()
        for toks in requests.values():
            x = plain.rms_norm(plain.embedding(tensors["emb"].double(), toks), tensors["l0.n1"].double(), TOY2["eps"])
            used |= set(plain.linear(x, tensors["l0.moe.router"].double()).argmax(dim=1).tolist())
        assert len(used) >= 2
        for mode in ("whole", "tail_decoded", "portions", "mixed"):
            kwargs = {"max_live": 3} if mode == "mixed" else {"tail": 8} if mode == "tail_decoded" else {}
            steps = getattr(schedules, mode)(requests, **kwargs)
            outputs = {}
            for s in steps:
                out = engine.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
                if out.logits is not None:
                    outputs[s["step"]] = out.logits.cpu().numpy()
                for rid in s["end"]:
                    engine.release(rid)
            for rid, rows in schedules.collect(steps, outputs).items():
                err = np.abs(np.stack(rows) - expected[rid]).max(axis=1)
                assert np.isfinite(err).all() and err.max() <= 1e-4, (mode, rid, int(err.argmax()), float(err.max()))
            assert engine.cache.free_pages(0) == 12
    finally:
        unregister_architecture("ToyRoutedForCausalLM")
        FEED_FORWARDS.unregister("toy_top_one")
        POSITIONS.unregister("toy_two_speed")


def test_position_part():
    from leone_amd.parts import POSITIONS, PartSpec
    rope = POSITIONS.build(PartSpec("rope_half_split", {"rotary_dim": 48, "theta": 50000.0}))
    rope.prepare(300, DEV)
    cos, sin = rope.tables()
    assert cos.shape == (300, 24) and cos.dtype == torch.float32
    for pos in (0, 1, 77, 299):
        for i in (0, 5, 23):
            angle = pos * 50000.0 ** (-2.0 * i / 48)
            assert abs(float(cos[pos, i]) - math.cos(angle)) < 5e-7 and abs(float(sin[pos, i]) - math.sin(angle)) < 5e-7
    none = POSITIONS.build(PartSpec("none", {}))
    none.prepare(10, DEV)
    assert none.tables() == (None, None)
    with pytest.raises(ValueError):
        POSITIONS.build(PartSpec("rope_half_split", {"rotary_dim": 15, "theta": 1e4}))
    with pytest.raises(ValueError):
        POSITIONS.build(PartSpec("alibi", {}))


@pytest.mark.parametrize("rows", [9, 40])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_block_part(dtype, rows):
    """One pre-norm block alone: x1 = x + attention(norm1 x), x2 = x1 + feed_forward(norm2 x1).  With few
    rows the bfloat16 products add into the stream themselves; with many the block hands back a delta."""
    from leone_amd import ops
    from leone_amd.parts import BLOCKS, POSITIONS, PartSpec
    from leone_amd.parts.context import KvCacheView
    hidden, heads, kv, dim, ffn, page = 64, 4, 2, 16, 96, 16
    rope = POSITIONS.build(PartSpec("rope_half_split", {"rotary_dim": dim, "theta": 1e4}))
    rope.prepare(64, DEV)
    spec = PartSpec("prenorm", {
        "norm1": PartSpec("rmsnorm", {"size": hidden, "eps": 1e-5, "weight": "n1"}),
        "mixer": PartSpec("gqa_attention", dict(hidden=hidden, q_heads=heads, kv_heads=kv, head_dim=dim, qk_norm_eps=1e-5,
                                                window=None, position="rope", q="a.q_proj.weight", k="a.k_proj.weight",
                                                v="a.v_proj.weight", o="a.o_proj.weight", q_norm="a.q_norm.weight",
                                                k_norm="a.k_norm.weight")),
        "norm2": PartSpec("rmsnorm", {"size": hidden, "eps": 1e-5, "weight": "n2"}),
        "feed_forward": PartSpec("swiglu", {"hidden": hidden, "intermediate": ffn, "gate": "f.gate_proj.weight",
                                            "up": "f.up_proj.weight", "down": "f.down_proj.weight"})})
    block = BLOCKS.build(spec, positions={"rope": rope})
    torch.manual_seed(12)
    w = {s.name: (torch.randn(s.shape) * 0.08 if len(s.shape) == 2 else 1 + 0.1 * torch.randn(s.shape)).to(dtype)
         for s in block.tensor_specs()}
    assert len(w) == 11
    block.bind({k: v.to(DEV) for k, v in w.items()})
    x0 = torch.randn(rows, hidden)
    k_pool = torch.zeros((4, kv, dim // 8, page, 8), dtype=dtype, device=DEV)
    v_pool = torch.zeros((4, kv, page // 8, dim, 8), dtype=dtype, device=DEV)
    table = torch.tensor([[2, 0, 3, 1]], dtype=torch.int32, device=DEV)
    cache = KvCacheView(writes=True, k_pool=k_pool, v_pool=v_pool, block_table=table, page_tokens=page)
    step = step_context([(0, i) for i in range(rows)], dtype, {0: table})
    x = x0.to(DEV)
    pending = block.forward(x, None, step, cache)
    if pending is not None and pending.dim() == 3:
        pending = pending.double().sum(0)
    got = x.cpu().double() + (0 if pending is None else pending.cpu().double())
    if dtype == torch.bfloat16:
        # the weight-streaming kernels add into the stream themselves (the inner sizes here are one chunk of K)
        assert (pending is None) == (rows <= ops.ROWS_MAX)
    wf = {k: v.float() for k, v in w.items()}
    cfg = dict(num_attention_heads=heads, num_key_value_heads=kv, head_dim=dim, rms_norm_eps=1e-5, rope_theta=1e4)
    x1 = x0.double() + plain.attention_block(plain.rms_norm(x0, wf["n1"], 1e-5), wf, "a", cfg, list(range(rows)))
    want = x1 + plain.feed_forward(plain.rms_norm(x1, wf["n2"], 1e-5), wf, "f")
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    assert (got - want).abs().max() < tol


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_model_spec_with_embedding_scale_and_logit_cap(tmp_path, dtype_name):
    """Two things a model description may ask for around the layers: the stream starts as table row * scale,
    and logits pass through cap * tanh(logits / cap).  Checked on the Qwen3 parts with a spec changed here:
    the plain side gets the scale through a scaled table (the head is not tied) and the cap applied after."""
    import dataclasses
    from leone_amd.architectures import config_from_dict, model_spec_for
    from leone_amd.engine.engine import Engine, StepEntry
    from leone_amd.parts.model import DecoderModel
    from leone_amd.weights import loader
    from tests.util import TINY, make_model_dir, read_weights
    dtype = torch.float32 if dtype_name == "float32" else torch.bfloat16
    folder = make_model_dir(str(tmp_path / "m"), TINY["B"], 5, dtype)
    spec = dataclasses.replace(model_spec_for(config_from_dict(TINY["B"])), embedding_scale=4.0, logit_cap=0.5)
    model = DecoderModel(spec, dtype, DEV)
    model.bind(loader.load_from_dir(folder, model.tensor_specs(), dtype, torch.device(DEV)))
    weights = {k: v.float() for k, v in read_weights(folder).items()}
    tokens = random_tokens(3, 50, TINY["B"]["vocab_size"])
    scaled = dict(weights)
    scaled["model.embed_tokens.weight"] = weights["model.embed_tokens.weight"] * 4.0
    want = 0.5 * torch.tanh(plain.forward(scaled, TINY["B"], tokens) / 0.5)
    engine = Engine(model, max_tokens=64, page_tokens=16, max_requests=2)
    out = engine.step([StepEntry("a", tokens[:37], list(range(37)))]).logits
    out = torch.cat([out, engine.step([StepEntry("a", tokens[37:], list(range(13)))]).logits]).cpu().double()
    assert float(want.abs().max()) > 0.3                                  # the cap bites
    assert (out - want).abs().max() < (1e-4 if dtype_name == "float32" else 3e-2)

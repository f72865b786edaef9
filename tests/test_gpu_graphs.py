"""Decode steps replayed from a recorded graph against the same steps run call by call."""
import numpy as np
import pytest
import torch

from tests.util import TINY, make_model_dir, random_tokens

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_replayed_decode_steps_equal_eager_ones(tmp_path, dtype_name):
    """Every replay is checked, with eager work (prompt portions of other requests, synchronisation,
    releases that hand pages to new requests) between the replays."""
    from leone_amd.engine.engine import Engine, StepEntry
    from leone_amd.runtime import load_model

    folder = make_model_dir(str(tmp_path / "m"), TINY["B"], 5,
                            torch.float32 if dtype_name == "float32" else torch.bfloat16)
    model = load_model(folder, dtype_name)
    assert model.graph_safe
    engines = [Engine(model, num_pages=24, page_tokens=16, max_requests=4, graphs=flag) for flag in (True, False)]
    assert engines[0].graphs and not engines[1].graphs
    vocab = TINY["B"]["vocab_size"]
    prompts = {rid: random_tokens(300 + i, n, vocab) for i, (rid, n) in enumerate([("a", 30), ("b", 5), ("c", 47)])}
    feed = {rid: random_tokens(400 + i, 40, vocab) for i, rid in enumerate(prompts)}

    def both(entries):
        outs = [e.step([StepEntry(*x) for x in entries]).logits for e in engines]
        torch.cuda.synchronize()
        return [None if o is None else o.cpu().numpy() for o in outs]

    both([("a", prompts["a"], [29]), ("b", prompts["b"], [4])])
    replays = 0
    for i in range(40):
        entries = [("a", [feed["a"][i]], [0]), ("b", [feed["b"][i]], [0])]
        if i == 12:
            both([("c", prompts["c"][:20], [])])          # eager work between replays
        if i == 13:
            both([("c", prompts["c"][20:], [26])])
        if i >= 14:
            entries.append(("c", [feed["c"][i]], [] if i % 3 == 0 else [0]))   # another batch size, some rows unwanted
        graph_out, eager_out = both(entries)
        assert graph_out.shape == eager_out.shape
        if dtype_name == "float32":
            assert np.array_equal(graph_out, eager_out), f"step {i}"
        else:   # the number of key splits differs between the two, which moves sums by rounding only
            assert np.abs(graph_out - eager_out).max() < 2e-2, f"step {i}"
        replays += 1
        if i == 25:
            for e in engines:
                e.release("b")
            both([("b", prompts["b"], [])])               # its pages and slot are handed out again
            feed["b"] = feed["b"][:26] + random_tokens(77, 14, vocab)
    assert len(engines[0]._decode_graphs) == 2 and all(g.recordings for g in engines[0]._decode_graphs.values())
    for e in engines:
        e.cache.check()


def test_a_part_that_is_not_graph_safe_keeps_the_model_eager(tmp_path):
    """A model one of whose parts does not declare itself safe to record is never replayed: the engine stays
    eager, records nothing, and its decode steps still agree with the plain implementation."""
    import dataclasses

    from leone_amd.architectures import config_from_dir, model_spec_for
    from leone_amd.engine.engine import Engine, StepEntry
    from leone_amd.parts import MIXERS, Part
    from leone_amd.parts.base import PartSpec
    from leone_amd.parts.mixer import GqaAttention
    from leone_amd.parts.model import DecoderModel
    from leone_amd.weights import loader
    from tests.plain import qwen3_plain
    from tests.util import read_config, read_weights, tolerance

    class HostDependent(GqaAttention):
        graph_safe = False

    assert not Part.graph_safe and GqaAttention.graph_safe and not HostDependent.graph_safe
    folder = make_model_dir(str(tmp_path / "m"), TINY["B"], 9, torch.float32)
    spec = model_spec_for(config_from_dir(folder))
    MIXERS.register("host_dependent_attention", HostDependent)
    try:
        spec = dataclasses.replace(spec, layers=[
            PartSpec(layer.kind, {**layer.params, "mixer": PartSpec("host_dependent_attention", layer["mixer"].params)})
            if i == 1 else layer for i, layer in enumerate(spec.layers)])
        model = DecoderModel(spec, torch.float32, "cuda:0")
        model.bind(loader.load_from_dir(folder, model.tensor_specs(), model.dtype, model.device))
        assert not model.graph_safe
        engine = Engine(model, num_pages=16, page_tokens=16, max_requests=2, graphs=True)
        assert engine.graphs is False
        tokens = random_tokens(31, 40, TINY["B"]["vocab_size"])
        expected = qwen3_plain.forward(read_weights(folder), read_config(folder), tokens).numpy()
        engine.step([StepEntry("a", tokens[:30], [])])
        for at in range(30, 40):
            logits = engine.step([StepEntry("a", [tokens[at]], [0])]).logits.cpu().numpy()
            assert np.abs(logits[0] - expected[at]).max() <= tolerance("float32"), at
        assert not engine._decode_graphs
    finally:
        MIXERS.unregister("host_dependent_attention")


@pytest.mark.parametrize("n", [20, 150])
def test_replayed_decode_steps_of_many_rows_agree_with_plain(tmp_path, n):
    """Decode steps of many requests, recorded and replayed, against the plain implementation: 20 rows take
    the multi-row weight-streaming product, 150 rows (more than it takes) the vendor library's products and
    the separate activation kernel inside the recording.  The recording is replayed several times, with eager
    steps between, and every replay is compared."""
    from leone_amd import ops
    from leone_amd.engine.engine import Engine, StepEntry
    from leone_amd.runtime import load_model
    from tests.plain import qwen3_plain
    from tests.util import read_config, read_weights, tolerance

    folder = make_model_dir(str(tmp_path / "m"), TINY["M"], 6, torch.bfloat16)
    model = load_model(folder, "bfloat16")
    engines = [Engine(model, num_pages=n * 2 + 8, page_tokens=16, max_requests=n + 1, graphs=flag) for flag in (True, False)]
    vocab = TINY["M"]["vocab_size"]
    steps = 5
    sequences = [random_tokens(700 + i, 3 + (i * 7) % 19 + steps, vocab) for i in range(n)]
    weights, config = read_weights(folder), read_config(folder)
    expected = [qwen3_plain.forward(weights, config, s).numpy()[-steps:] for s in sequences]
    for e in engines:
        e.step([StepEntry(i, sequences[i][:-steps], []) for i in range(n)])
    for step in range(steps):
        entries = [StepEntry(i, [sequences[i][step - steps]], [0]) for i in range(n)]
        with ops.record_library_products() as recorded:
            outs = [e.step(entries).logits.cpu().numpy() for e in engines]
        assert bool(recorded.problems) == (n > ops.ROWS_MAX)        # (a replay hands nothing to ``linear``)
        want = np.stack([expected[i][step] for i in range(n)])
        for which, out in zip(("replayed", "eager"), outs):
            assert np.isfinite(out).all()
            assert np.abs(out - want).max() <= tolerance("bfloat16"), f"{which} step {step}"
        if step % 2 == 0:                                      # eager work between the replays
            for e in engines:
                e.step([StepEntry("other", random_tokens(900 + step, 21, vocab), [20])])
                e.release("other")
    assert engines[0]._decode_graphs[n].recordings and not engines[1]._decode_graphs


def test_decode_steps_are_recorded_for_the_context_range_they_run_in(tmp_path):
    """An engine built for 40,960 positions records a decode step at context 300 for the range up to 512, not
    for its largest context: the attention kernel then cuts the keys as an engine built for 512 positions
    does, and the step takes the same time (within 5 %); as requests grow into the next range a further
    recording is made; every replay equals the eager engine and the plain implementation."""
    from leone_amd import ops
    from leone_amd.engine.engine import Engine, StepEntry, context_bucket
    from leone_amd.runtime import load_model
    from tests.plain import qwen3_plain
    from tests.util import read_config, read_weights, tolerance

    assert [context_bucket(n, 40960) for n in (1, 256, 257, 512, 513, 40000, 40960)] == [256, 256, 512, 512, 1024, 40960, 40960]
    assert context_bucket(300, 384) == 384
    config = dict(TINY["M"], max_position_embeddings=40960)
    folder = make_model_dir(str(tmp_path / "m"), config, 8, torch.bfloat16)
    model = load_model(folder, "bfloat16")
    wide = Engine(model, num_pages=40, page_tokens=16, max_requests=2, graphs=True)
    narrow = Engine(model, num_pages=40, page_tokens=16, max_requests=2, graphs=True, max_context=512)
    eager = Engine(model, num_pages=40, page_tokens=16, max_requests=2, graphs=False)
    assert wide.max_context == 40960 and narrow.max_context == 512
    chosen = []
    choose = ops.choose_splits
    ops.choose_splits = lambda rows, kv_heads, group, max_context, units=256: chosen.append(max_context) or choose(rows, kv_heads, group, max_context, units)
    try:
        vocab = config["vocab_size"]
        tokens = {"a": random_tokens(1, 300, vocab), "b": random_tokens(2, 236, vocab)}
        expected = {r: qwen3_plain.forward(read_weights(folder), read_config(folder), t).numpy() for r, t in tokens.items()}
        engines = (wide, narrow, eager)
        for e in engines:
            e.step([StepEntry("a", tokens["a"][:270], []), StepEntry("b", tokens["b"][:206], [])])
        chosen.clear()
        for i in range(30):
            entries = [StepEntry("a", [tokens["a"][270 + i]], [0]), StepEntry("b", [tokens["b"][206 + i]], [0])]
            outs = [e.step(entries).logits.cpu().numpy() for e in engines]
            want = np.stack([expected["a"][270 + i], expected["b"][206 + i]])
            for which, out in zip(("wide", "narrow", "eager"), outs):
                assert np.abs(out - want).max() <= tolerance("bfloat16"), f"{which} step {i}"
            assert np.array_equal(outs[0], outs[1]), f"step {i}: the two recordings cut the keys differently"
        # contexts 271..300 and 207..236: one range (up to 512) for both engines, cut as for 512 positions
        assert set(wide._decode_graphs[2].recordings) == {512} and set(narrow._decode_graphs[2].recordings) == {512}
        assert 40960 not in chosen and 512 in chosen
        # the same steps again, timed: replays of the wide engine's recording against the narrow one's
        def replay_ms(engine):
            entries = [StepEntry("a", [5], [0]), StepEntry("b", [7], [0])]
            best = float("inf")
            first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            for _ in range(5):
                first.record()
                for _ in range(20):
                    engine._decode_graphs[2].recordings[512][0].replay()
                last.record()
                torch.cuda.synchronize()
                best = min(best, first.elapsed_time(last) / 20)
            return best
        assert replay_ms(wide) <= 1.05 * replay_ms(narrow)
        # growing past 512 positions makes a second recording, which still agrees with the eager engine
        long_tokens = random_tokens(3, 520, vocab)
        for e in (wide, eager):
            e.release("a"), e.release("b")
            e.step([StepEntry("c", long_tokens[:505], [])])
        for i in range(505, 520):
            outs = [e.step([StepEntry("c", [long_tokens[i]], [0])]).logits.cpu().numpy() for e in (wide, eager)]
            assert np.abs(outs[0] - outs[1]).max() < 2e-2, i
        assert set(wide._decode_graphs[1].recordings) == {512, 1024}
    finally:
        ops.choose_splits = choose

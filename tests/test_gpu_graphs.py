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
    assert len(engines[0]._decode_graphs) == 2 and all(g.graph is not None for g in engines[0]._decode_graphs.values())
    for e in engines:
        e.cache.check()


def test_a_part_that_is_not_graph_safe_keeps_the_model_eager(tmp_path):
    from leone_amd.parts import MIXERS, Part
    from leone_amd.parts.mixer import GqaAttention

    class HostDependent(GqaAttention):
        graph_safe = False

    assert not Part.graph_safe and GqaAttention.graph_safe and not HostDependent.graph_safe


def test_replay_with_many_rows_uses_the_library_product_inside_the_graph(tmp_path):
    """More than 16 decode rows take the library's matrix product; a recording that holds it is
    replayed several times, with eager steps between, and every replay is compared with the eager engine."""
    from leone_amd.engine.engine import Engine, StepEntry
    from leone_amd.runtime import load_model

    folder = make_model_dir(str(tmp_path / "m"), TINY["M"], 6, torch.bfloat16)
    model = load_model(folder, "bfloat16")
    engines = [Engine(model, num_pages=64, page_tokens=16, max_requests=24, graphs=flag) for flag in (True, False)]
    vocab = TINY["M"]["vocab_size"]
    n = 20
    prompts = [random_tokens(700 + i, 3 + (i * 7) % 19, vocab) for i in range(n)]
    for e in engines:
        e.step([StepEntry(i, prompts[i], []) for i in range(n)])
    for step in range(6):
        tokens = random_tokens(800 + step, n, vocab)
        outs = [e.step([StepEntry(i, [tokens[i]], [0]) for i in range(n)]).logits.cpu().numpy() for e in engines]
        assert np.isfinite(outs[0]).all()
        assert np.abs(outs[0] - outs[1]).max() < 3e-2, f"replay {step}"
        if step % 2 == 0:                                      # eager work between the replays
            for e in engines:
                e.step([StepEntry("other", random_tokens(900 + step, 21, vocab), [20])])
                e.release("other")
    assert engines[0]._decode_graphs[n].graph is not None

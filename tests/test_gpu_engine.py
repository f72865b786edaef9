"""The engine against the plain implementation, under every way of cutting the work."""
import numpy as np
import pytest
import torch

from tests import schedules
from tests.plain import qwen3_plain
from tests.util import REAL_8B_ONE_LAYER, TINY, make_model_dir, random_tokens, read_config, read_weights, tolerance

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [1, 7, 33, 64, 100, 18, 47], "B": [5, 40, 130, 66, 90], "C": [70, 150, 35, 81, 3],
           "M": [300, 45, 170, 129, 20], "D": [90, 17, 64, 2]}
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    """(config name, dtype name) -> model folder, requests and the plain logits of each request."""
    cache = {}

    def get(name, dtype_name):
        key = (name, dtype_name)
        if key not in cache:
            folder = str(tmp_path_factory.mktemp(f"model_{name}_{dtype_name}"))
            # float32: q/k gains doubled, so scores spread (std ~4) and a misplaced key moves the logits
            # far beyond 1e-4.  bfloat16: gains as drawn; sharper scores would only amplify the 2^-9
            # rounding of q and k, which is no fault (misplaced keys in bfloat16 are pinned by the
            # kernel tests, where one key dominates).
            sharpen = 2.0 if dtype_name == "float32" else 1.0
            make_model_dir(folder, TINY[name], seed=11 + len(cache), dtype=DTYPES[dtype_name], sharpen=sharpen)
            config, weights = read_config(folder), read_weights(folder)
            requests = {f"r{i}": random_tokens(100 * i + 7, n, config["vocab_size"])
                        for i, n in enumerate(LENGTHS[name])}
            expected = {rid: qwen3_plain.forward(weights, config, toks).numpy() for rid, toks in requests.items()}
            cache[key] = (folder, requests, expected)
        return cache[key]

    return get


def run_steps(engine, steps):
    from leone_amd.engine.engine import StepEntry

    outputs = {}
    for s in steps:
        out = engine.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        if out.logits is not None:
            outputs[s["step"]] = out.logits.float().cpu().numpy()
        for rid in s["end"]:
            engine.release(rid)
        engine.cache.check()
    return outputs


def compare(steps, outputs, expected, tol, what):
    got = schedules.collect(steps, outputs)
    assert set(got) == set(expected)
    for rid, rows in got.items():
        have = np.stack(rows)
        want = expected[rid]
        assert have.shape == want.shape, (what, rid, have.shape, want.shape)
        assert np.isfinite(have).all(), f"{what}: request {rid} has non-finite logits"
        err = np.abs(have - want).max(axis=1)
        worst = int(err.argmax())
        assert err[worst] <= tol, (f"{what}: request {rid} first wrong position "
                                   f"{int(np.argmax(err > tol))} of {len(err)}, worst {worst}: {err[worst]:.3e} > {tol}")


SCHEDULES = {
    "whole": schedules.whole,
    "tail_decoded": schedules.tail_decoded,
    "portions": schedules.portions,
    "mixed": schedules.mixed,
}


@pytest.mark.parametrize("page_tokens", [16, 64])
@pytest.mark.parametrize("schedule", list(SCHEDULES))
@pytest.mark.parametrize("dtype_name", list(DTYPES))
@pytest.mark.parametrize("name", list(TINY))
def test_engine_matches_plain(cases, name, dtype_name, schedule, page_tokens):
    from leone_amd.engine.engine import Engine
    from leone_amd.runtime import load_model

    folder, requests, expected = cases(name, dtype_name)
    steps = SCHEDULES[schedule](requests)
    # As few pages as the schedule can live with, so that pages given back are used again.
    pool_tokens = schedules.max_live_tokens(steps, round_to=page_tokens)
    model = load_model(folder, dtype_name)
    engine = Engine(model, num_pages=pool_tokens // page_tokens, page_tokens=page_tokens, max_requests=4,
                    poison_freed=True)
    outputs = run_steps(engine, steps)
    compare(steps, outputs, expected, tolerance(dtype_name), f"{name}/{dtype_name}/{schedule}/page{page_tokens}")
    assert not engine.cache.live_requests()
    assert all(engine.cache.free_pages(g) == engine.cache.groups[g].num_pages for g in range(len(engine.cache.groups)))


@pytest.mark.parametrize("schedule", ["whole", "portions", "mixed"])
@pytest.mark.parametrize("name", ["M", "C"])
def test_prompt_key_ranges_agree_with_plain(cases, monkeypatch, name, schedule):
    """The prompt kernel cuts a workgroup's keys into ranges when rows are few and keys many; here every
    64-key stage may be a range of its own and ranges cost nothing, so that the tiny prompts go that way too."""
    from leone_amd import ops
    from leone_amd.engine.engine import Engine
    from leone_amd.runtime import load_model

    chosen = []
    choose = ops.choose_prefill_splits

    def recording(*args, **kwargs):
        chosen.append(choose(*args, **kwargs))
        return chosen[-1]

    monkeypatch.setattr(ops, "PREFILL_SPLIT_MIN_STAGES", 1)
    monkeypatch.setattr(ops, "PREFILL_SPLIT_START_STAGES", 0)
    monkeypatch.setattr(ops, "PREFILL_SPLIT_MERGE_STAGES", 0)
    monkeypatch.setattr(ops, "choose_prefill_splits", recording)
    folder, requests, expected = cases(name, "bfloat16")
    steps = SCHEDULES[schedule](requests)
    model = load_model(folder, "bfloat16")
    engine = Engine(model, num_pages=schedules.max_live_tokens(steps, round_to=16) // 16, page_tokens=16,
                    max_requests=4, poison_freed=True)
    outputs = run_steps(engine, steps)
    assert max(chosen) >= 2, "no step took the key-range path"
    compare(steps, outputs, expected, tolerance("bfloat16"), f"{name}/key ranges/{schedule}")


def test_tuned_library_products_agree_with_plain(cases):
    """After ``Engine.tune_products`` the prompt portions of that size run the vendor library's products with
    the algorithms that were fastest when timed: the logits still agree with the plain implementation, for a
    prompt of the tuned size and for one of another size, and every tuned product is used."""
    from leone_amd import ops
    from leone_amd.engine.engine import Engine
    from leone_amd.runtime import load_model

    folder, requests, expected = cases("M", "bfloat16")
    name, tokens = max(requests.items(), key=lambda item: len(item[1]))
    rows = len(tokens) - 7
    assert rows > ops.ROWS_MAX, "the prompt is too short to reach the vendor library"
    model = load_model(folder, "bfloat16")
    engine = Engine(model, max_tokens=2 * len(tokens) + 64, page_tokens=16, max_requests=2)
    try:
        records = engine.tune_products(rows, keep_only_faster_steps=False)    # tiny products: no step would be faster
        assert len(records) >= 3 and all(r["kept"] and r["rows"] == rows for r in records), records
        assert not engine.cache.live_requests()
        with ops.record_library_products() as seen:
            steps = [{"step": 0, "entries": [{"id": name, "tokens": tokens[:rows], "want": list(range(rows))}], "end": []},
                     {"step": 1, "entries": [{"id": name, "tokens": tokens[rows:], "want": list(range(7))}], "end": [name]},
                     {"step": 2, "entries": [{"id": "again", "tokens": tokens[:rows - 3], "want": list(range(rows - 3))}], "end": ["again"]}]
            outputs = run_steps(engine, steps)
        mine = {r["problem"] for r in records}
        assert mine <= ops._tuned_products and mine <= {(0,) + problem for problem in seen.problems}    # all are in use
        assert any(problem[0] == rows for problem in seen.problems) and any(problem[0] == rows - 3 for problem in seen.problems)
        compare(steps[:2], outputs, {name: expected[name]}, tolerance("bfloat16"), "tuned products")
        again = {"again": expected[name][:rows - 3]}
        compare(steps[2:], {2: outputs[2]}, again, tolerance("bfloat16"), "beside tuned products")
        # without room for the trial step nothing is tuned and nothing is left behind
        tight = Engine(model, max_tokens=64, page_tokens=16, max_requests=1)
        assert tight.tune_products(rows) == [] and not tight.cache.live_requests()
        assert tight.cache.free_pages(0) == tight.cache.groups[0].num_pages
    finally:
        ops.forget_tuned_products()


def test_late_portions_of_a_long_request(tmp_path):
    """One request of 2,200 tokens at the large models' head shape: a long first portion, then portions of
    changing size far into the context, where the prompt kernel cuts the keys into ranges by its own rule,
    then single tokens."""
    from leone_amd import ops
    from leone_amd.engine.engine import Engine
    from leone_amd.runtime import load_model

    folder = make_model_dir(str(tmp_path / "long"), dict(TINY["M"], max_position_embeddings=4096), seed=77,
                            dtype=torch.bfloat16)
    config, weights = read_config(folder), read_weights(folder)
    tokens = random_tokens(4242, 2200, config["vocab_size"])
    expected = {"long": qwen3_plain.forward(weights, config, tokens).numpy()}
    cuts = [1200, 300, 150, 64, 40, 17, 200, 200] + [1] * 29
    assert sum(cuts) == len(tokens)
    steps, at = [], 0
    for n, size in enumerate(cuts):
        steps.append({"step": n, "entries": [{"id": "long", "tokens": tokens[at:at + size], "want": list(range(size))}],
                      "end": ["long"] if at + size == len(tokens) else []})
        at += size
    chosen = []
    choose = ops.choose_prefill_splits
    ops.choose_prefill_splits = lambda *a, **k: chosen.append(choose(*a, **k)) or chosen[-1]
    try:
        engine = Engine(load_model(folder, "bfloat16"), max_tokens=2240, page_tokens=64, max_requests=1)
        outputs = run_steps(engine, steps)
    finally:
        ops.choose_prefill_splits = choose
    assert chosen[0] == 1 and max(chosen) >= 2, chosen
    compare(steps, outputs, expected, tolerance("bfloat16"), "long request in late portions")


def test_a_hundred_thousand_tokens_cut_three_ways(tmp_path):
    """A context far beyond what the plain implementation can check: block tables of 1,500 pages, key
    ranges in both attention kernels.  The last prompt token's logits and those of eight decoded tokens
    must not depend on how the prompt was cut."""
    from leone_amd.engine.engine import Engine, StepEntry
    from leone_amd.runtime import load_model

    config = dict(TINY["M"], max_position_embeddings=131072)
    folder = make_model_dir(str(tmp_path / "far"), config, seed=9, dtype=torch.bfloat16)
    model = load_model(folder, "bfloat16")
    n = 100_000
    tokens = random_tokens(5, n + 8, config["vocab_size"])
    results = []
    for chunk in (2048, 1000, 333):
        engine = Engine(model, max_tokens=n + 64, page_tokens=64, max_requests=1, max_context=n + 64)
        at = 0
        while at < n:
            size = min(chunk, n - at)
            out = engine.step([StepEntry("r", tokens[at:at + size], [size - 1] if at + size == n else [])])
            at += size
        rows = [out.logits[0].float().cpu()]
        for i in range(8):
            rows.append(engine.step([StepEntry("r", [tokens[n + i]], [0])]).logits[0].float().cpu())
        results.append(torch.stack(rows))
        engine.release("r")
        engine.cache.check()
    assert all(torch.isfinite(r).all() for r in results)
    assert float(results[0].abs().max()) > 0.5                    # the logits are not all alike
    for other in results[1:]:
        assert float((other - results[0]).abs().max()) <= tolerance("bfloat16")


def test_a_hundred_thousand_tokens_against_the_plain_implementation(tmp_path):
    """The same length against the plain implementation: a model of ONE layer, whose keys and values come
    straight from the embeddings, can be evaluated at single positions for what the length costs.  Scores are
    sharpened (q/k gains doubled in float32: the softmax of 100,000 keys then rests on the few hundred best,
    which lie anywhere in the context; in the plain implementation a sixteenth of the keys left out moves these
    logits by 0.4, a single page by 0.004 to 0.02; measured from the plain implementation: float32 6e-5,
    bfloat16 1.3e-2).  The last prompt
    position (the prompt kernel with key ranges, the last portion's rows over 98,000 earlier keys) and eight
    decoded tokens (the split-KV kernel over 1,563 pages), in bfloat16 and float32."""
    from leone_amd.engine.engine import Engine, StepEntry
    from leone_amd.runtime import load_model

    config = dict(TINY["M"], num_hidden_layers=1, max_position_embeddings=131072)
    n = 100_000
    tokens = random_tokens(6, n + 8, config["vocab_size"])
    # bfloat16 with gains times 1.5: its own rounding of sharper scores comes close to its tolerance
    for dtype_name, chunk, sharpen in (("bfloat16", 2048, 1.5), ("float32", 4096, 2.0)):
        folder = make_model_dir(str(tmp_path / dtype_name), config, seed=10, dtype=DTYPES[dtype_name], sharpen=sharpen)
        weights = read_weights(folder)
        want = qwen3_plain.forward_rows_of_one_layer(weights, read_config(folder), tokens, list(range(n - 1, n + 8))).float()
        engine = Engine(load_model(folder, dtype_name), max_tokens=n + 64, page_tokens=64, max_requests=1, max_context=n + 64)
        at = 0
        while at < n:
            size = min(chunk, n - at)
            out = engine.step([StepEntry("r", tokens[at:at + size], [size - 1] if at + size == n else [])])
            at += size
        rows = [out.logits[0].float().cpu()]
        for i in range(8):
            rows.append(engine.step([StepEntry("r", [tokens[n + i]], [0])]).logits[0].float().cpu())
        got = torch.stack(rows)
        engine.release("r")
        engine.cache.check()
        worst = float((got - want).abs().max())
        assert float(want.abs().max()) > 0.5
        print(f"100,000 tokens, {dtype_name}: {worst:.3e} from the plain implementation")
        assert worst <= tolerance(dtype_name), f"{dtype_name}: {worst:.3e} from the plain implementation at 100,000 tokens"


@pytest.mark.parametrize("schedule", ["whole", "portions", "mixed"])
def test_a_wide_feed_forward_whose_down_projection_is_cut(tmp_path, schedule):
    """An intermediate size of 8,192 over a width of 64: for steps of more than 128 rows the down projection
    runs in parts on the library, for 17 to 128 on the multi-row weight-streaming kernel with K cut into
    ranges; either way the next norm adds up the planes, and the last block's planes go to the final norm."""
    from leone_amd import ops
    from leone_amd.engine.engine import Engine
    from leone_amd.runtime import load_model

    config = dict(TINY["A"], intermediate_size=8192, max_position_embeddings=512)
    folder = make_model_dir(str(tmp_path / "wide"), config, seed=23, dtype=torch.bfloat16)
    weights = read_weights(folder)
    requests = {f"w{i}": random_tokens(900 + i, n, config["vocab_size"]) for i, n in enumerate([330, 90, 70, 200])}
    expected = {rid: qwen3_plain.forward(weights, read_config(folder), toks).numpy() for rid, toks in requests.items()}
    steps = (schedules.portions(requests, sizes=(100, 66, 7, 157)) if schedule == "portions"
             else schedules.mixed(requests, sizes=(70, 3, 120)) if schedule == "mixed" else schedules.whole(requests))
    taken = []
    real = ops.inner_parts
    ops.inner_parts = lambda *a: taken.append(real(*a)) or taken[-1]
    try:
        engine = Engine(load_model(folder, "bfloat16"), num_pages=schedules.max_live_tokens(steps, round_to=16) // 16,
                        page_tokens=16, max_requests=4, poison_freed=True)
        outputs = run_steps(engine, steps)
    finally:
        ops.inner_parts = real
    assert max(taken) == 4 and min(taken) == 1
    compare(steps, outputs, expected, tolerance("bfloat16"), f"wide feed-forward/{schedule}")


def test_a_malformed_step_is_refused_and_changes_nothing(cases):
    from leone_amd.engine.engine import Engine, StepEntry, StepError
    from leone_amd.runtime import load_model

    folder, requests, expected = cases("A", "float32")
    engine = Engine(load_model(folder, "float32"), max_tokens=256, page_tokens=16, max_requests=4)
    vocab = TINY["A"]["vocab_size"]
    tokens = requests["r3"]
    engine.step([StepEntry("kept", tokens[:10], [])])
    free = engine.cache.free_pages(0)
    bad = [[], [StepEntry("a", [1, 2], []), StepEntry("a", [3], [])], [StepEntry("a", [], [])],
           [StepEntry("a", [vocab], [0])], [StepEntry("a", [-1], [0])], [StepEntry("a", [1, 2, 3, 4, 5, vocab], [0])],
           [StepEntry("a", [True], [0])], [StepEntry("a", [1.5], [0])], [StepEntry("a", [1, 2], [2])],
           [StepEntry("a", [1, 2], [-1])], [StepEntry("kept", [5], [0]), StepEntry("b", [1, vocab + 7], [])]]
    for entries in bad:
        with pytest.raises(StepError):
            engine.step(entries)
        assert engine.cache.free_pages(0) == free and engine.cache.length("kept") == 10
        assert not engine.cache.has("a") and not engine.cache.has("b")
        engine.cache.check()
    out = engine.step([StepEntry("kept", tokens[10:20], list(range(10)))])
    assert np.abs(out.logits.float().cpu().numpy() - expected["r3"][10:20]).max() <= tolerance("float32")


@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_rerun_is_bitwise_identical(cases, dtype_name):
    from leone_amd.engine.engine import Engine
    from leone_amd.runtime import load_model

    folder, requests, _ = cases("B", dtype_name)
    steps = schedules.mixed(requests)
    model = load_model(folder, dtype_name)
    results = []
    for _ in range(2):
        engine = Engine(model, max_tokens=schedules.max_live_tokens(steps, 16), page_tokens=16, max_requests=4)
        results.append(run_steps(engine, steps))
    for step in results[0]:
        assert np.array_equal(results[0][step], results[1][step]), f"step {step} differs between two runs"


@pytest.mark.parametrize("dtype_name", list(DTYPES))
def test_forked_requests_share_prefix_pages_and_agree_with_plain(cases, dtype_name):
    """A second request takes over the full pages of the first one's prefix, computes only what lies
    beyond, and both go on independently; cutting a request back and feeding other tokens likewise."""
    from leone_amd.engine.engine import Engine, StepEntry
    from leone_amd.runtime import load_model

    folder, _, _ = cases("B", dtype_name)
    config, weights = read_config(folder), read_weights(folder)
    vocab, tol = config["vocab_size"], tolerance(dtype_name)
    model = load_model(folder, dtype_name)
    engine = Engine(model, num_pages=16, page_tokens=16, max_requests=3, poison_freed=True)
    a = random_tokens(1, 90, vocab)
    b = a[:64] + random_tokens(2, 45, vocab)                    # the same first four pages, then its own way
    want_a = qwen3_plain.forward(weights, config, a).numpy()
    want_b = qwen3_plain.forward(weights, config, b).numpy()

    def feed(rid, tokens, start, want):
        out = engine.step([StepEntry(rid, tokens, list(range(len(tokens))))]).logits.cpu().numpy()
        err = np.abs(out - want[start:start + len(tokens)]).max()
        assert np.isfinite(out).all() and err <= tol, (rid, start, float(err))

    feed("a", a[:70], 0, want_a)
    free_before = engine.cache.free_pages(0)
    assert engine.fork("a", "b") == 64 and engine.cache.free_pages(0) == free_before
    assert engine.cache.shared_pages(0) == 4
    feed("b", b[64:100], 64, want_b)                             # a portion right after the shared pages
    feed("a", a[70:71], 70, want_a)                              # the parent decodes on in its own tail
    feed("b", b[100:], 100, want_b)
    engine.release("a")                                          # its private pages are poisoned, the shared ones live on
    engine.cache.check()
    c = b[:80] + random_tokens(3, 20, vocab)
    want_c = qwen3_plain.forward(weights, config, c).numpy()
    engine.truncate("b", 80)
    feed("b", c[80:], 80, want_c)
    engine.release("b")
    engine.cache.check()
    assert engine.cache.free_pages(0) == 16


def drawn_config(seed: int) -> dict:
    """A configuration drawn at random: head sizes in steps of 16, any number of heads and groups, widths
    and vocabularies that are multiples of nothing in particular."""
    gen = np.random.default_rng(seed)
    kv_heads = int(gen.integers(1, 5))
    group = int(gen.integers(1, 8))
    head_dim = int(gen.choice([16, 32, 48, 64, 80, 96, 112, 128, 144, 256]))
    return dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=int(gen.integers(1, 4)),
                hidden_size=int(gen.integers(5, 40)) * int(gen.choice([2, 4, 8])), num_attention_heads=kv_heads * group,
                num_key_value_heads=kv_heads, head_dim=head_dim, intermediate_size=int(gen.integers(9, 200)),
                vocab_size=int(gen.integers(40, 1500)), max_position_embeddings=512,
                rope_theta=float(gen.choice([1e4, 5e5, 1e6, 123456.0])), rms_norm_eps=float(gen.choice([1e-6, 1e-5, 3e-5])),
                tie_word_embeddings=bool(gen.integers(0, 2)))


@pytest.mark.parametrize("dtype_name", list(DTYPES))
@pytest.mark.parametrize("seed", range(10))
def test_drawn_configurations(tmp_path, seed, dtype_name):
    """Whatever sizes a configuration allows run, whole and cut up, and agree with the plain implementation."""
    from leone_amd.engine.engine import Engine
    from leone_amd.runtime import load_model
    raw = drawn_config(1000 + seed)
    folder = make_model_dir(str(tmp_path / "m"), raw, seed=seed, dtype=DTYPES[dtype_name],
                            sharpen=2.0 if dtype_name == "float32" else 1.0)
    config, weights = read_config(folder), read_weights(folder)
    gen = np.random.default_rng(seed)
    requests = {f"r{i}": random_tokens(50 * seed + i, int(n), config["vocab_size"])
                for i, n in enumerate(gen.integers(1, 160, size=3))}
    expected = {rid: qwen3_plain.forward(weights, config, toks).numpy() for rid, toks in requests.items()}
    plans = {name: SCHEDULES[name](requests, **({"max_live": 3} if name == "mixed" else {}))
             for name in ("whole", "portions", "mixed")}
    engine = Engine(load_model(folder, dtype_name), page_tokens=16, max_requests=4, poison_freed=True,
                    max_tokens=max(schedules.max_live_tokens(steps, 16) for steps in plans.values()))
    for name, steps in plans.items():
        compare(steps, run_steps(engine, steps), expected, tolerance(dtype_name), f"{raw} {name}")


# Against the oracle that rounds where the engine rounds: largest mean |difference| over all logits of a run,
# and largest single difference.  Measured: means 1e-6 to 3e-4 on A, B, C and 1.3e-3 on M, where the plain
# implementation without roundings is 1e-3 to 2.4e-3 and 5.7e-3 away; single logits up to 1.1e-2 (3.4e-2 on M).
ROUNDED_MEAN = {"A": 6e-4, "B": 6e-4, "C": 6e-4, "M": 2.5e-3}
ROUNDED_MAX = {"A": 2e-2, "B": 2e-2, "C": 2e-2, "M": 5e-2}


@pytest.mark.parametrize("schedule", list(SCHEDULES))
@pytest.mark.parametrize("name", ["A", "B", "C", "M"])
def test_bfloat16_engine_against_the_oracle_that_rounds_where_it_rounds(tmp_path, name, schedule):
    """Sharpened scores (q/k gains doubled, so that a misplaced or missing key moves the logits) in bfloat16.
    The oracle rounds every tensor the engine stores, softmax weights included, at the engine's place for a
    step of that many rows.  Most positions then agree to 1e-7; what is left are single bfloat16 values that
    fall the other way because a float sum differs from the double one in its last place, most visibly a
    softmax weight of a key that dominates its row, and whatever later positions take over from such a
    position through the cache.  Those are sparse, so the mean difference is held to a fraction of what
    bfloat16 itself does to the logits: a fault that moves one layer's attention by a few percent moves
    every position and does not fit under it."""
    from leone_amd import ops
    from leone_amd.engine.engine import Engine
    from leone_amd.runtime import load_model
    from tests.plain import qwen3_rounded

    folder = make_model_dir(str(tmp_path / "m"), TINY[name], seed=61, dtype=torch.bfloat16, sharpen=2.0)
    config, weights = read_config(folder), read_weights(folder)
    requests = {f"r{i}": random_tokens(100 * i + 9, n, config["vocab_size"]) for i, n in enumerate(LENGTHS[name])}
    steps = SCHEDULES[schedule](requests)
    sizes = qwen3_rounded.step_sizes(steps, requests)
    expected = {rid: qwen3_rounded.forward(weights, config, toks, sizes[rid][0], sizes[rid][1], ops.FUSED_ROWS,
                                           ops.ROWS_MAX).numpy() for rid, toks in requests.items()}
    engine = Engine(load_model(folder, "bfloat16"), num_pages=schedules.max_live_tokens(steps, round_to=16) // 16,
                    page_tokens=16, max_requests=4, poison_freed=True)
    outputs = run_steps(engine, steps)
    compare(steps, outputs, expected, ROUNDED_MAX[name], f"{name}/rounded oracle/{schedule}")
    got = schedules.collect(steps, outputs)
    differences = np.concatenate([np.abs(np.stack(got[rid]) - expected[rid]).ravel() for rid in requests])
    assert differences.mean() <= ROUNDED_MEAN[name], f"{name}/{schedule}: mean difference {differences.mean():.2e}"
    # The first position of a request sees one key, whose weight is exactly 1: only the other roundings are left
    # there, and the oracle reproduces them: most first positions agree to the last bits of a float.  One in a
    # few has a single bfloat16 value of the first layers fall the other way (which one depends on the order
    # in which a kernel's waves add up K), and then nearly every logit of that position moves by up to 3e-3.
    firsts = sorted(float(np.abs(got[rid][0] - expected[rid][0]).max()) for rid in requests)
    assert firsts[(len(firsts) - 1) // 2] <= 1e-5, f"{name}/{schedule}: first positions differ by {firsts}"
    assert firsts[-1] <= 5e-3, f"{name}/{schedule}: a first position differs by {firsts[-1]:.2e}"


# ---- the layer sizes of the large models ----------------------------------------------------------------
_REAL_BASE = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", rope_theta=1000000.0, rms_norm_eps=1e-6,
                  tie_word_embeddings=False, max_position_embeddings=1024, vocab_size=8200)
REAL = {
    # one and two layers of the 8B widths, one of the 32B head shape (64 query heads of 128 over a width of 5,120)
    "8b-1": REAL_8B_ONE_LAYER,
    "8b-2": dict(_REAL_BASE, num_hidden_layers=2, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
                 head_dim=128, intermediate_size=12288),
    "32b-1": dict(_REAL_BASE, num_hidden_layers=1, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8,
                  head_dim=128, intermediate_size=25600),
}
REAL_LENGTHS = {"8b-1": [150, 600], "8b-2": [300, 160], "32b-1": [200, 330]}
REAL_SCHEDULES = dict(SCHEDULES, portions=lambda requests: schedules.portions(
    requests, sizes=(16, 17, 64, 65, 128, 129, 2, 40)))      # both sides of every change of kernel


@pytest.fixture(scope="module")
def real_cases(tmp_path_factory):
    cache = {}

    def get(name):
        if name not in cache:
            folder = make_model_dir(str(tmp_path_factory.mktemp(f"real_{name}")), REAL[name], seed=71, dtype=torch.bfloat16)
            config, weights = read_config(folder), read_weights(folder)
            requests = {f"r{i}": random_tokens(100 * i + 9, n, config["vocab_size"]) for i, n in enumerate(REAL_LENGTHS[name])}
            expected = {rid: qwen3_plain.forward(weights, config, toks).numpy() for rid, toks in requests.items()}
            cache[name] = (folder, requests, expected, config, weights)
        return cache[name]

    return get


@pytest.mark.parametrize("schedule", list(REAL_SCHEDULES))
@pytest.mark.parametrize("dtype_name", list(DTYPES))
@pytest.mark.parametrize("name", list(REAL))
def test_layers_of_the_large_models_match_plain(real_cases, name, dtype_name, schedule):
    """The widths at which the products' plans, the cuts of K and the changes of kernel at 16/17, 64/65 and
    128/129 rows were chosen (crates/leone-cuda/tests/gpu.rs:653-711 tests at the model's own shapes).
    Logits reach 7.5 here, so the bounds are taken relative to the largest logit: float32 as everywhere
    (measured 4e-5), bfloat16 1.5 % for a single logit and 0.25 % on average (measured 0.9 % and 0.16 %)."""
    from leone_amd import ops
    from leone_amd.engine.engine import Engine
    from leone_amd.runtime import load_model

    folder, requests, expected, config, weights = real_cases(name)
    steps = REAL_SCHEDULES[schedule](requests)
    engine = Engine(load_model(folder, dtype_name), num_pages=schedules.max_live_tokens(steps, round_to=64) // 64,
                    page_tokens=64, max_requests=4, poison_freed=True)
    outputs = run_steps(engine, steps)
    scale = max(float(np.abs(v).max()) for v in expected.values())
    assert scale > 3.0
    if dtype_name == "float32":
        compare(steps, outputs, expected, tolerance("float32"), f"{name}/float32/{schedule}")
        return
    compare(steps, outputs, expected, 1.5e-2 * scale, f"{name}/bfloat16/{schedule}")
    got = schedules.collect(steps, outputs)
    mean = np.mean([np.abs(np.stack(got[rid]) - expected[rid]).mean() for rid in requests])
    assert mean <= 2.5e-3 * scale, f"{name}/{schedule}: mean difference {mean:.2e} of logits up to {scale:.2f}"
    if schedule == "mixed":
        from tests.plain import qwen3_rounded
        sizes = qwen3_rounded.step_sizes(steps, requests)
        rounded = {rid: qwen3_rounded.forward(weights, config, toks, sizes[rid][0], sizes[rid][1], ops.FUSED_ROWS,
                                              ops.ROWS_MAX).numpy() for rid, toks in requests.items()}
        mean = np.mean([np.abs(np.stack(got[rid]) - rounded[rid]).mean() for rid in requests])
        assert mean <= 1e-3 * scale, f"{name}: mean difference from the rounding oracle {mean:.2e}"


@pytest.mark.parametrize("dtype_name", list(DTYPES))
@pytest.mark.parametrize("name", ["B", "M"])
def test_many_live_requests_decoding_side_by_side(tmp_path, name, dtype_name):
    """Up to 28 live requests, most of them decoding: steps of 17 to 28 rows of single tokens beside short
    portions, which is where the multi-row weight-streaming products and the split-KV kernel serve many
    requests at once; few pages, so that finished requests' pages are used again."""
    from leone_amd import ops
    from leone_amd.engine.engine import Engine
    from leone_amd.runtime import load_model

    folder = make_model_dir(str(tmp_path / "m"), TINY[name], seed=81, dtype=DTYPES[dtype_name],
                            sharpen=2.0 if dtype_name == "float32" else 1.0)
    config, weights = read_config(folder), read_weights(folder)
    gen = np.random.default_rng(5)
    requests = {f"d{i}": random_tokens(900 + i, int(gen.integers(18, 60)), config["vocab_size"]) for i in range(40)}
    expected = {rid: qwen3_plain.forward(weights, config, toks).numpy() for rid, toks in requests.items()}
    steps = schedules.mixed(requests, max_live=28, prompt_fraction=0.3, sizes=(5, 2, 9, 3))
    decode_rows = [sum(1 for e in s["entries"] if len(e["tokens"]) == 1) for s in steps]
    assert max(decode_rows) >= 20 and sum(1 for n in decode_rows if n > ops.FUSED_ROWS) >= 20
    engine = Engine(load_model(folder, dtype_name), num_pages=schedules.max_live_tokens(steps, round_to=16) // 16,
                    page_tokens=16, max_requests=28, poison_freed=True)
    outputs = run_steps(engine, steps)
    compare(steps, outputs, expected, tolerance(dtype_name), f"{name}/{dtype_name}/many live")


@pytest.mark.parametrize("name", ["A", "M", "B"])
def test_second_copies_of_the_weights_change_no_bit(tmp_path, name):
    """With a second copy of every matrix in the decode kernels' order (kept by default where the widths allow
    it and memory is ample) the engine gives the logits it gives without, bit for bit, over a mixed schedule;
    the model's accounting names the copies' bytes; a matrix whose inner size is no multiple of 64 gets none."""
    from leone_amd.engine.engine import Engine
    from leone_amd.runtime import load_model

    folder = make_model_dir(str(tmp_path / "m"), TINY[name], seed=83, dtype=torch.bfloat16)
    config = read_config(folder)
    requests = {f"s{i}": random_tokens(300 + i, 50 + 17 * i, config["vocab_size"]) for i in range(6)}
    steps = schedules.mixed(requests, max_live=4, prompt_fraction=0.4, sizes=(11, 2, 30, 5))
    pages = schedules.max_live_tokens(steps, round_to=16) // 16
    outputs = {}
    for wanted in (False, None):
        model = load_model(folder, "bfloat16")
        engine = Engine(model, num_pages=pages, page_tokens=16, max_requests=4, streamed_weights=wanted)
        copies = model.weight_accounting()["streamed_copy_bytes"]
        if wanted is None:                            # every matrix whose inner size allows it, and no other
            fitting = [w for w in model.streamed_weights() if w.shape[1] % 64 == 0]
            assert copies == sum(-(-w.shape[0] // 16) * 16 * w.shape[1] * 2 for w in fitting) > 0
            assert (len(fitting) == len(model.streamed_weights())) == (config["hidden_size"] % 64 == 0)
        else:
            assert copies == 0
        outputs[wanted] = run_steps(engine, steps)
    assert outputs[False].keys() == outputs[None].keys()
    for step, logits in outputs[False].items():
        assert np.array_equal(logits, outputs[None][step]), f"step {step} differs"


@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_many_groups_of_prompt_tiles_at_few_heads(tmp_path, name):
    """Four prompt portions of 40 tokens in one step (a group of tiles each), then a prompt of 420 tokens whole
    (four groups of one request), at 4, 6 and 2 query heads: head counts at which the prompt kernel's numbering
    of workgroups by die once left heads out.  bfloat16 with sharpened scores against the oracle that rounds
    where the engine rounds (a width that is no multiple of 8 takes other kernels: against the plain one)."""
    from leone_amd import ops
    from leone_amd.engine.engine import Engine, StepEntry
    from leone_amd.runtime import load_model
    from tests.plain import qwen3_rounded

    raw = dict(TINY[name], max_position_embeddings=512)
    runs_of_8 = raw["hidden_size"] % 8 == 0  # the oracle knows the roundings of the 16-byte-run kernels only
    folder = make_model_dir(str(tmp_path / "m"), raw, seed=91, dtype=torch.bfloat16, sharpen=2.0 if runs_of_8 else 1.0)
    config, weights = read_config(folder), read_weights(folder)
    requests = {f"g{i}": random_tokens(40 + i, 40, config["vocab_size"]) for i in range(4)}
    requests["long"] = random_tokens(50, 420, config["vocab_size"])
    steps = [{"step": 0, "entries": [{"id": f"g{i}", "tokens": requests[f"g{i}"], "want": list(range(40))} for i in range(4)],
              "end": [f"g{i}" for i in range(4)]},
             {"step": 1, "entries": [{"id": "long", "tokens": requests["long"], "want": list(range(420))}], "end": ["long"]}]
    engine = Engine(load_model(folder, "bfloat16"), max_tokens=448, page_tokens=16, max_requests=4, poison_freed=True)
    outputs = run_steps(engine, steps)
    if not runs_of_8:
        expected = {rid: qwen3_plain.forward(weights, config, toks).numpy() for rid, toks in requests.items()}
        compare(steps, outputs, expected, tolerance("bfloat16"), f"{name}/groups of tiles")
        return
    sizes = qwen3_rounded.step_sizes(steps, requests)
    rounded = {rid: qwen3_rounded.forward(weights, config, toks, sizes[rid][0], sizes[rid][1], ops.FUSED_ROWS,
                                          ops.ROWS_MAX).numpy() for rid, toks in requests.items()}
    compare(steps, outputs, rounded, ROUNDED_MAX[name], f"{name}/groups of tiles")
    got = schedules.collect(steps, outputs)
    mean = np.mean([np.abs(np.stack(got[rid]) - rounded[rid]).mean() for rid in requests])
    assert mean <= ROUNDED_MEAN[name], f"{name}: mean difference from the rounding oracle {mean:.2e}"


def test_two_engines_step_side_by_side_in_threads_on_streams_of_their_own(cases):
    """Nothing a step relies on is kept for the process: two engines on one model, each in a thread with a
    stream of its own, give bit for bit what they give one after the other."""
    import threading

    from leone_amd.engine.engine import Engine
    from leone_amd.runtime import load_model

    folder, requests, expected = cases("B", "float32")
    model = load_model(folder, "float32")
    halves = [dict(list(requests.items())[:3]), dict(list(requests.items())[2:])]
    plans = [schedules.mixed(half, max_live=2) for half in halves]

    def run(which, results, stream=None):
        engine = Engine(model, num_pages=schedules.max_live_tokens(plans[which], 16) // 16 + 1, page_tokens=16, max_requests=2)
        if stream is None:
            results[which] = run_steps(engine, plans[which])
            return
        with torch.cuda.stream(stream):
            for _ in range(3):                        # several times over, so that the two really overlap
                results[which] = run_steps(engine, plans[which])
            stream.synchronize()

    alone, together = {}, {}
    for which in range(2):
        run(which, alone)
    threads = [threading.Thread(target=run, args=(which, together, torch.cuda.Stream())) for which in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for which in range(2):
        assert set(alone[which]) == set(together[which])
        for step in alone[which]:
            assert np.array_equal(alone[which][step], together[which][step]), (which, step)
        compare(plans[which], together[which], {r: expected[r] for r in halves[which]}, tolerance("float32"), "side by side")

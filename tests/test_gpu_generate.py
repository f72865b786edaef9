"""Generation through the entry points: greedy against the plain implementation, temperature against
the slow sampler oracle, device sampling kernels against the double-precision sampler, the CLI."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests.plain import qwen3_plain, sampler_plain
from tests.util import TINY, make_model_dir, random_tokens, read_config, read_weights

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: make_model_dir(str(tmp_path_factory.mktemp(f"gen{name}")), TINY[name], 21, torch.float32, 2.0)
            for name in ("A", "B")}


def plain_greedy(weights, config, prompt, n):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(qwen3_plain.forward(weights, config, tokens)[-1].argmax()))
    return tokens[len(prompt):]


def test_greedy_generation_matches_plain(folders):
    """Config A's workload: prompts of 1, 7, 33 and 64 tokens, 16 greedy tokens each, all live together."""
    from leone_amd.api import Runtime
    folder = folders["A"]
    weights, config = read_weights(folder), read_config(folder)
    prompts = [random_tokens(40 + i, n, config["vocab_size"]) for i, n in enumerate([1, 7, 33, 64])]
    runtime = Runtime.load(folder, "float32", max_tokens=4 * 96, page_tokens=16, max_requests=4)
    results = runtime.generate_tokens(prompts, 16, eos_token_id=None)
    for prompt, result in zip(prompts, results):
        assert result.tokens == plain_greedy(weights, config, prompt, 16)
        assert result.finish_reason == "length"
    assert runtime.last_stats.emitted_tokens == 64
    assert not runtime.engine.cache.live_requests()


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_long_decoding_and_preemption_keep_the_tokens(folders, tmp_path, dtype_name):
    """Few pages: requests are preempted and recomputed, and still produce what they produce alone.  Every
    page is filled with NaN when it is given back, also by the scheduler (a preempted or finished request), so
    that a row that read a page no longer its own would show.  In bfloat16 a batch rounds differently from a
    request alone, so there the tokens may part where the two best logits of the run alone lie closer than the
    type resolves; up to there, and in float32 everywhere, they are the same."""
    from leone_amd.api import Runtime
    from leone_amd.engine.scheduler import SchedulerPolicy
    folder = folders["A"] if dtype_name == "float32" else make_model_dir(str(tmp_path / "m"), TINY["A"], 29, torch.bfloat16)
    weights, config = read_weights(folder), read_config(folder)
    prompts = [random_tokens(60 + i, n, config["vocab_size"]) for i, n in enumerate([20, 35, 9])]
    alone = Runtime.load(folder, dtype_name, max_tokens=256, page_tokens=16, max_requests=1)
    expect, margins = [], []
    for p in prompts:
        seen = {}

        def note(request, position, row, seen=seen):
            best = torch.topk(row.float(), 2).values
            seen[position] = float(best[0] - best[1])
        expect.append(alone.generate_tokens([p], 120, eos_token_id=None, logit_observer=note)[0].tokens)
        margins.append(seen)
    if dtype_name == "float32":
        assert expect[2][:24] == plain_greedy(weights, config, prompts[2], 24)
    tight = Runtime.load(folder, dtype_name, num_pages=14, page_tokens=16, max_requests=3, poison_freed=True,
                         policy=SchedulerPolicy(max_live_requests=3, prefill_chunk_tokens=16, max_step_tokens=24))
    finite = []
    results = tight.generate_tokens(prompts, 120, eos_token_id=None,
                                    logit_observer=lambda request, position, row: finite.append(bool(torch.isfinite(row).all())))
    assert finite and all(finite)
    assert tight.last_stats.preemptions >= 1
    tight.engine.cache.check()
    for i, (result, want) in enumerate(zip(results, expect)):
        assert len(result.tokens) == 120 and all(0 <= t < config["vocab_size"] for t in result.tokens)
        if result.tokens != want:
            assert dtype_name == "bfloat16"
            at = next(j for j, (a, b) in enumerate(zip(result.tokens, want)) if a != b)
            assert margins[i][len(prompts[i]) + at - 1] < 3e-2, (i, at, margins[i][len(prompts[i]) + at - 1])


def test_greedy_generation_at_the_widths_of_the_large_models(tmp_path):
    """Scheduler, step and device sampler together at one layer of the 8B widths in bfloat16 (where the
    products' plans, the cuts of K and the changes of kernel were chosen): four requests, prompts in portions
    of 64 beside decoded tokens, so few pages that a request is preempted and recomputed.  Every token the
    engine picks must be, for the plain implementation on the same (bfloat16) weights fed the same tokens,
    the best one or within the type's noise of it: 1.5 % of the largest logit, the bound the step itself is
    held to at these widths."""
    from leone_amd.api import Runtime
    from leone_amd.engine.scheduler import SchedulerPolicy
    from tests.util import REAL_8B_ONE_LAYER

    folder = make_model_dir(str(tmp_path / "m"), REAL_8B_ONE_LAYER, seed=73, dtype=torch.bfloat16)
    weights, config = read_weights(folder), read_config(folder)
    prompts = [random_tokens(50 + i, n, config["vocab_size"]) for i, n in enumerate([120, 60, 180, 50])]
    new = 20        # every request grows over a page's edge while it decodes: 7 pages at first, 11 at the end, 8 there are
    runtime = Runtime.load(folder, "bfloat16", num_pages=8, page_tokens=64, max_requests=4, poison_freed=True,
                           policy=SchedulerPolicy(max_live_requests=4, prefill_chunk_tokens=64, max_step_tokens=96))
    results = runtime.generate_tokens(prompts, new, eos_token_id=None)
    runtime.engine.cache.check()
    assert runtime.last_stats.emitted_tokens == new * len(prompts)
    assert runtime.last_stats.preemptions >= 1
    assert not runtime.engine.cache.live_requests()
    for prompt, result in zip(prompts, results):
        assert len(result.tokens) == new and result.finish_reason == "length"
        logits = qwen3_plain.forward(weights, config, list(prompt) + result.tokens).numpy()
        scale = float(np.abs(logits).max())
        assert scale > 3.0
        for i, token in enumerate(result.tokens):
            row = logits[len(prompt) + i - 1]
            assert row[token] >= row.max() - 1.5e-2 * scale, (i, token, float(row[token]), float(row.max()))


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("temperature,top_k", [(None, None), (0.9, None), (1.3, 20)])
def test_steps_issued_ahead_of_the_tokens_give_the_same_tokens(folders, tmp_path, dtype_name, temperature, top_k):
    """Where device kernels choose the tokens, the next decode step is issued before the last step's tokens have
    reached the host (they are fed from the device): the same tokens as step by step, with requests that end
    on an end token at different times (their row in the step ahead is thrown away), with so few pages that
    requests are preempted, greedy, with a temperature, and with top-k and top-p behind it; the decision log
    still shows a sound run."""
    from leone_amd.api import Runtime, sampling_params
    from leone_amd.engine import trace_check
    from leone_amd.engine.generate import Generator
    from leone_amd.engine.scheduler import SchedulerPolicy
    folder = folders["B"] if dtype_name == "float32" else make_model_dir(str(tmp_path / "m"), TINY["B"], 33, torch.bfloat16)
    config = read_config(folder)
    prompts = [random_tokens(70 + i, n, config["vocab_size"]) for i, n in enumerate([12, 31, 5, 44, 20])]
    params = sampling_params(temperature=temperature, seed=99, top_k=top_k, top_p=0.95 if top_k else None)
    policy = SchedulerPolicy(max_live_requests=4, prefill_chunk_tokens=16, max_step_tokens=32)
    runtime = Runtime.load(folder, dtype_name, num_pages=10, page_tokens=16, max_requests=4, poison_freed=True, policy=policy)
    plain_run = runtime.generate_tokens(prompts, 40, params, eos_token_id=None, look_ahead=False)
    assert runtime.last_stats.steps_ahead == 0 and runtime.last_stats.preemptions >= 1
    ahead_run = runtime.generate_tokens(prompts, 40, params, eos_token_id=None)          # ahead by default
    assert runtime.last_stats.steps_ahead > 10 and runtime.last_stats.preemptions >= 1
    assert [r.tokens for r in ahead_run] == [r.tokens for r in plain_run]
    # an end token that some requests meet early, some late and some never
    seen = [t for r in plain_run for t in r.tokens[5:30]]
    eos = max(set(seen), key=seen.count)
    results = {}
    for look_ahead in (False, True):
        generator = Generator(runtime.engine, policy)
        generator.look_ahead = look_ahead
        for i, prompt in enumerate(prompts):
            generator.submit(i, prompt, 40, params, eos)
        finished = {f.id: f for f in generator.run()}
        results[look_ahead] = [(finished[i].tokens, finished[i].reason) for i in range(len(prompts))]
        report = trace_check.verify_events(generator.scheduler.events, trace_check.figures_of(generator.scheduler))
        assert report.steps == generator.scheduler.stats.steps
        assert (generator.stats.steps_ahead > 10) == look_ahead
        assert any(kind == "ahead" for kind, *_ in generator.scheduler.events) == look_ahead
        runtime.engine.cache.check()
        assert not runtime.engine.cache.live_requests()
    if dtype_name == "float32":
        assert results[True] == results[False]
    else:
        # A request that has met its end token still rides along in the step ahead: that step has one row more
        # than the step-by-step run's, other kernels may take it, and bfloat16 logits differ in their rounding,
        # which a draw close to a boundary shows.  Until the first end token the two runs are the same steps.
        assert [tokens[:5] for tokens, _ in results[True]] == [tokens[:5] for tokens, _ in results[False]]
    for run in results.values():
        assert {reason for _, reason in run} == {"eos", "length"}
        assert any(tokens[-1] == eos and len(tokens) < 40 for tokens, _ in run)


def test_temperature_sampling_matches_oracle_and_ignores_batching(folders):
    """Config B's workload: prompts 5/40/130, portions of 32, 24 tokens at temperature 0.8, seeded."""
    from leone_amd.api import Runtime, sampling_params
    from leone_amd.engine.scheduler import SchedulerPolicy
    folder = folders["B"]
    weights, config = read_weights(folder), read_config(folder)
    prompts = [random_tokens(80 + i, n, config["vocab_size"]) for i, n in enumerate([5, 40, 130])]
    params = sampling_params(temperature=0.8, seed=1234)
    together = Runtime.load(folder, "float32", max_tokens=3 * 192, page_tokens=16, max_requests=3,
                            policy=SchedulerPolicy(max_live_requests=3, prefill_chunk_tokens=32))
    results = together.generate_tokens(prompts, 24, params, eos_token_id=None)
    alone = Runtime.load(folder, "float32", max_tokens=192, page_tokens=64, max_requests=1)
    for prompt, result in zip(prompts, results):
        assert alone.generate_tokens([prompt], 24, params, eos_token_id=None)[0].tokens == result.tokens
    # the first request against the oracle: plain logits, slow double-precision distribution, same draws
    tokens = list(prompts[0])
    for _ in range(24):
        logits = qwen3_plain.forward(weights, config, tokens)[-1].float().tolist()
        probs = sampler_plain.distribution(logits, 0.8)
        tokens.append(sampler_plain.select(probs, sampler_plain.uniform(1234, len(tokens) - 1)))
    assert results[0].tokens == tokens[len(prompts[0]):]
    # truncation stages take the host path; top-k 1 is the argmax whatever the draw
    greedy = together.generate_tokens(prompts[:1], 8, eos_token_id=None)[0].tokens
    top1 = together.generate_tokens(prompts[:1], 8, sampling_params(temperature=1.3, seed=5, top_k=1),
                                    eos_token_id=None)[0].tokens
    assert top1 == greedy


def test_mirostat_and_dry_generation_matches_oracle(folders):
    """The controller's bound and the repeated-suffix penalty follow a request through portions and a batch."""
    from leone_amd.api import Runtime, sampling_params
    from leone_amd.engine.scheduler import SchedulerPolicy
    folder = folders["A"]
    weights, config = read_weights(folder), read_config(folder)
    # a prompt that repeats itself, so that the penalty has something to act on
    prompts = [random_tokens(60, 9, config["vocab_size"]) * 3, random_tokens(61, 21, config["vocab_size"])]
    params = sampling_params(temperature=1.1, seed=77, mirostat=(2.5, 0.4), dry_multiplier=0.8, dry_base=1.5,
                             dry_allowed_length=2, dry_window=32)
    runtime = Runtime.load(folder, "float32", max_tokens=256, page_tokens=16, max_requests=2,
                           policy=SchedulerPolicy(max_live_requests=2, prefill_chunk_tokens=8))
    results = runtime.generate_tokens(prompts, 16, params, eos_token_id=None)
    for prompt, result in zip(prompts, results):
        tokens, bound = list(prompt), 5.0
        for _ in range(16):
            logits = qwen3_plain.forward(weights, config, tokens)[-1].float().tolist()
            logits = np.array(sampler_plain.dry(logits, tokens, 0.8, 1.5, 2, 32), dtype=np.float32).tolist()
            probs = sampler_plain.distribution(logits, 1.1)
            token, bound = sampler_plain.mirostat(probs, bound, 2.5, 0.4, sampler_plain.uniform(77, len(tokens) - 1))
            tokens.append(token)
        assert result.tokens == tokens[len(prompt):]


def test_cycle_and_zero_models(tmp_path):
    """Two models whose output is known without any arithmetic (the reference's fixtures,
    crates/leone/src/runtime.rs:11567-11608 and crates/leone/tests/common/cpu_fixture.rs:67-105): one-hot
    embedding, silent layers and a head shifted by one make token t answer t + 1; all-zero weights make
    every logit 0, and the lowest id wins the tie."""
    from leone_amd.api import Runtime
    from leone_amd.weights.safetensors_io import write_file
    size = 16
    raw = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2, hidden_size=size,
               num_attention_heads=1, num_key_value_heads=1, head_dim=16, intermediate_size=8, vocab_size=size,
               max_position_embeddings=64, rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=False)
    for kind in ("cycle", "zero"):
        folder = make_model_dir(str(tmp_path / kind), raw, 1, torch.float32)
        tensors = {name: torch.zeros_like(t) for name, t in read_weights(folder).items()}
        if kind == "cycle":
            for name in tensors:
                if name.endswith("norm.weight") or name.endswith("layernorm.weight"):
                    tensors[name] += 1.0
            tensors["model.embed_tokens.weight"] = torch.eye(size)
            tensors["lm_head.weight"] = torch.roll(torch.eye(size), 1, dims=0)       # row t + 1 reads column t
        write_file(os.path.join(folder, "model.safetensors"), tensors)
        for dtype in ("float32", "bfloat16"):
            runtime = Runtime.load(folder, dtype, max_tokens=128, page_tokens=16, max_requests=2)
            out = runtime.generate_tokens([[3], [14, 2, 9]], 6, eos_token_id=None)
            if kind == "cycle":
                assert out[0].tokens == [4, 5, 6, 7, 8, 9] and out[1].tokens == [10, 11, 12, 13, 14, 15]
            else:
                assert out[0].tokens == [0] * 6 and out[1].tokens == [0] * 6


def test_eos_stops_generation(folders):
    from leone_amd.api import Runtime
    folder = folders["A"]
    runtime = Runtime.load(folder, "float32", max_tokens=128, page_tokens=16, max_requests=1)
    prompt = random_tokens(99, 12, 512)
    free = runtime.generate_tokens([prompt], 10, eos_token_id=None)[0].tokens
    stopped = runtime.generate_tokens([prompt], 10, eos_token_id=free[3])[0]
    assert stopped.tokens == free[:free.index(free[3]) + 1] and stopped.finish_reason == "eos"


def test_cancellation_ends_every_request_with_what_it_has(folders):
    """The cancellation flag (Ctrl-C on the command line) is looked at before every step: the requests end
    as cancelled with the tokens generated so far, which are the tokens of an undisturbed run, and nothing
    stays live."""
    from leone_amd.api import Runtime
    folder = folders["A"]
    config = read_config(folder)
    prompts = [random_tokens(300 + i, n, config["vocab_size"]) for i, n in enumerate([12, 30])]
    runtime = Runtime.load(folder, "float32", max_tokens=256, page_tokens=16, max_requests=2)
    whole = runtime.generate_tokens(prompts, 20, eos_token_id=None)
    steps = []
    cut = runtime.generate_tokens(prompts, 20, eos_token_id=None, on_token=lambda request, token: steps.append(request),
                                  cancelled=lambda: len(steps) >= 10)
    for full, part in zip(whole, cut):
        assert part.finish_reason == "cancelled" and 0 < len(part.tokens) < 20
        assert full.tokens[:len(part.tokens)] == part.tokens
    assert not runtime.engine.cache.live_requests()
    runtime.engine.cache.check()
    assert runtime.generate_tokens(prompts, 20, eos_token_id=None)[0].tokens == whole[0].tokens


def test_device_sampling_kernels_against_the_double_precision_sampler():
    from leone_amd import ops
    from leone_amd.sampling.sampler import SamplingParams, distribution, select
    gen = np.random.default_rng(7)
    for vocab in (1, 2, 777, 1024, 1025, 151936):
        rows = 6
        logits = (gen.standard_normal((rows, vocab)) * 3).astype(np.float32)
        if vocab > 2:
            logits[1, vocab // 2] = np.nan
            logits[2, 0] = -np.inf
            logits[3, :] = logits[3, 0]                      # all equal: uniform distribution
        temps = np.array([0.8, 1.0, 0.3, 1.0, 5.0, 0.05])
        draws = gen.random(rows)
        draws[4] = 0.0
        got = ops.sample_temperature(torch.from_numpy(logits).cuda(), torch.from_numpy(temps).cuda(),
                                     torch.from_numpy(draws).cuda()).cpu().tolist()
        for r in range(rows):
            probs = distribution(logits[r], SamplingParams(temperature=float(temps[r])))
            want = select(probs, float(draws[r]))
            if got[r] != want:   # only a draw within rounding of a boundary may differ, and then by one neighbour
                cumulative = np.cumsum(probs)
                assert abs(cumulative[min(got[r], want)] - draws[r]) < 1e-9, (vocab, r, got[r], want)
    nothing = torch.full((1, 50), float("nan"), device="cuda")
    assert ops.sample_temperature(nothing, torch.ones(1, dtype=torch.float64, device="cuda"),
                                  torch.zeros(1, dtype=torch.float64, device="cuda")).tolist() == [-1]


def best_in_sampler_order(row, k):
    """Ids of the k best finite logits: the higher first, the lower id on a tie."""
    ids = [i for i in range(len(row)) if np.isfinite(row[i])]
    ids.sort(key=lambda i: (-float(row[i]), i))
    return ids[:k]


def test_top_candidates_kernel():
    """The device's selection of a row's k best logits against a plain sort: ties, values that are not
    finite, fewer finite values than k, vocabularies smaller and larger than a workgroup, and a row laid
    out against the deal of ids to threads, which the kernel hands back."""
    from leone_amd import ops
    gen = np.random.default_rng(11)
    for vocab in (1, 5, 300, 1024, 4097, 151936):
        rows = 7
        logits = (gen.standard_normal((rows, vocab)) * 3).astype(np.float32)
        logits[1] = np.round(logits[1])                                  # many ties
        logits[2, ::3] = np.nan
        logits[2, 1::7] = -np.inf
        logits[3] = 0.0                                                  # all equal, +0 and -0 alike: the lowest ids win
        logits[3, ::2] = -0.0
        logits[4, vocab // 3:] = np.inf                                  # few finite values
        logits[5] = np.sort(logits[5])                                   # ascending: the best come last
        logits[6] = -np.sort(-logits[6])
        wanted = [40, 256, 17, 9, 50, 1, 255]
        values, ids, counts = ops.top_candidates(torch.from_numpy(logits).cuda(), wanted)
        for r in range(rows):
            want = best_in_sampler_order(logits[r], wanted[r])
            assert counts[r] == len(want), (vocab, r, counts[r], len(want))
            assert ids[r, :counts[r]].tolist() == want, (vocab, r)
            assert np.array_equal(values[r, :counts[r]], logits[r, want]), (vocab, r)
    # 39 cells own nothing but large values: the bound falls among the small ones and the large ones
    # (39 * 592) do not fit the kernel's room.
    against = np.full((2, 151936), -5.0, dtype=np.float32)
    against[0, :] = gen.standard_normal(151936).astype(np.float32)
    owner = (np.arange(151936) // 16) % 256                   # the cell (four threads, four ids each a turn) that owns an id
    for t in range(39):
        against[1, owner == t] = 50.0 + t
    values, ids, counts = ops.top_candidates(torch.from_numpy(against).cuda(), [40, 40])
    assert counts.tolist() == [40, 40]
    for r in range(2):
        assert ids[r, :40].tolist() == best_in_sampler_order(against[r], 40)
        assert np.array_equal(values[r, :40], against[r, ids[r, :40]])
    with pytest.raises(ops.KernelError):
        ops.top_candidates(torch.from_numpy(against).cuda(), [40, 257])


def test_truncated_sampling_kernel_against_the_double_precision_sampler():
    """Selection, stages and draw in one launch against the plain sampler over the whole row: stages in every
    order behind the first top-k, ties across the cut, values that are not finite, rows with fewer finite values
    than k (the whole row's sum counts then), k of 1 and of 256, a uniform value of 0, rows that are skipped, a
    row laid out against the selection's deal of ids to threads."""
    from leone_amd import ops
    from leone_amd.sampling.sampler import SamplingParams, distribution, select
    gen = np.random.default_rng(23)
    checked = 0
    for vocab in (1, 3, 50, 777, 4097, 151936):
        for case in range(6 if vocab > 10000 else 12):
            rows = 8
            logits = (gen.standard_normal((rows, vocab)) * gen.choice([0.3, 2.0, 8.0])).astype(np.float32)
            logits[1] = np.round(logits[1])                                      # ties, also across the cut
            logits[2, ::2] = np.nan
            logits[3, 1::5] = -np.inf
            logits[4] = 1.5
            if vocab > 1024:
                logits[5, :] = -5.0
                owner = (np.arange(vocab) // 16) % 256        # the cell that owns an id
                for t in range(39):
                    logits[5, owner == t] = 50.0 + t * 0.01
            draws = []
            for r in range(rows):
                later = [(str(name), float(gen.integers(1, 300)) if name == "top_k" else float(gen.uniform(0.02, 1.0)))
                         for name in gen.permutation(["top_p", "min_p", "top_k", "top_p"])[:int(gen.integers(0, 5))]]
                k = float(gen.choice([1, 2, 12, 40, 255, 256]))
                u = 0.0 if r == 6 and case == 0 else float(gen.random())
                draws.append((float(gen.choice([0.3, 0.8, 1.0, 2.5])), u, [("top_k", k)] + later))
            draws[7] = None
            got = ops.sample_truncated(torch.from_numpy(logits).cuda(), draws).cpu().tolist()
            assert got[7] == -1
            for r in range(7):
                t, u, stages = draws[r]
                if not np.isfinite(logits[r]).any():
                    assert got[r] == -1
                    continue
                probs = distribution(logits[r], SamplingParams(temperature=t, truncations=stages))
                want = select(probs, u)
                if got[r] != want:      # only a draw within rounding of a boundary may differ, and then by one neighbour
                    eligible = np.nonzero(probs > 0.0)[0]
                    cumulative = np.cumsum(probs[eligible])
                    edge = cumulative[np.searchsorted(eligible, min(got[r], want))]
                    assert probs[got[r]] > 0.0 and abs(edge - u) < 1e-9, (vocab, case, r, got[r], want)
                checked += 1
    assert checked > 300
    nothing = torch.full((2, 50), float("nan"), device="cuda")
    assert ops.sample_truncated(nothing, [(1.0, 0.5, [("top_k", 5.0)])] * 2).tolist() == [-1, -1]
    for bad in ([("top_p", 0.9)], [("top_k", 257.0)], [("top_k", 5.0), ("tfs", 0.5)], [("top_k", 5.0)] * 9, []):
        assert not ops.truncated_draw_supported(bad)
        with pytest.raises(ops.KernelError):
            ops.sample_truncated(nothing, [(1.0, 0.5, bad), None])
    with pytest.raises(ops.KernelError):
        ops.sample_truncated(nothing, [(0.0, 0.5, [("top_k", 5.0)]), None])
    with pytest.raises(ops.KernelError):
        ops.sample_truncated(nothing, [(1.0, 1.0, [("top_k", 5.0)]), None])


def test_truncated_sampling_on_the_device_matches_the_whole_row_on_the_host(folders, monkeypatch):
    """top-k first: the device selects, cuts and draws; the tokens are those of the host sampler over whole rows,
    alone, in a batch, beside greedy and plain-temperature requests, and with steps issued ahead."""
    from leone_amd import ops
    from leone_amd.api import Runtime, sampling_params
    folder = folders["B"]
    config = read_config(folder)
    prompts = [random_tokens(90 + i, n, config["vocab_size"]) for i, n in enumerate([9, 33, 70])]
    params = sampling_params(temperature=0.9, seed=4321, top_k=12, top_p=0.85, min_p=0.02)
    mixed = [params, None, sampling_params(temperature=1.1, seed=5)]
    runtime = Runtime.load(folder, "float32", max_tokens=3 * 128, page_tokens=16, max_requests=3)
    calls = []
    real = ops.sample_truncated
    monkeypatch.setattr(ops, "sample_truncated", lambda *a: calls.append(1) or real(*a))
    narrow = [r.tokens for r in runtime.generate_tokens(prompts, 20, params, eos_token_id=None)]
    assert len(calls) >= 20 and runtime.last_stats.steps_ahead >= 15
    one_by_one = [r.tokens for r in runtime.generate_tokens(prompts, 20, params, eos_token_id=None, look_ahead=False)]
    assert one_by_one == narrow and runtime.last_stats.steps_ahead == 0
    beside = [r.tokens for r in runtime.generate_tokens(prompts, 20, mixed, eos_token_id=None)]
    assert beside[0] == narrow[0] and runtime.last_stats.steps_ahead >= 15
    calls.clear()
    monkeypatch.setattr(ops, "truncated_draw_supported", lambda stages: False)      # everything the long way
    whole = [r.tokens for r in runtime.generate_tokens(prompts, 20, params, eos_token_id=None)]
    assert not calls and whole == narrow and runtime.last_stats.steps_ahead == 0
    assert [r.tokens for r in runtime.generate_tokens(prompts, 20, mixed, eos_token_id=None)] == beside


def test_command_line_generate(folders, tmp_path):
    folder = folders["A"]
    weights, config = read_weights(folder), read_config(folder)
    prompt = random_tokens(123, 11, config["vocab_size"])
    tokens_file, logits_file = tmp_path / "tokens.json", tmp_path / "logits.txt"
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "leone"), "generate", "-m", folder,
                          "--prompt-tokens", ",".join(map(str, prompt)), "-n", "8", "--dtype", "float32",
                          "--debug-tokens", str(tokens_file), "--debug-logits", str(logits_file),
                          "--profile-decode"],
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    assert "decode profile: 7 evaluations" in run.stderr
    expect = plain_greedy(weights, config, prompt, 8)
    assert json.load(open(tokens_file)) == expect
    assert [int(t) for t in run.stdout.split()] == expect
    assert "decode:" in run.stderr and "prefill:" in run.stderr and "tokens emitted: 8" in run.stderr
    lines = open(logits_file).read().strip().splitlines()
    assert len(lines) == 8 and int(lines[0].split()[0].split(":")[0]) == expect[0]


def test_decode_profile_counts_operations_and_keeps_tokens(folders):
    """Profiled decode steps run call by call between replayed ones: same tokens, and what was counted is
    what one decode step of this model launches."""
    from leone_amd.api import Runtime
    folder = folders["B"]
    config = read_config(folder)
    prompt = random_tokens(77, 19, config["vocab_size"])
    for dtype in ("float32", "bfloat16"):
        runtime = Runtime.load(folder, dtype, max_tokens=128, page_tokens=16, max_requests=1)
        expect = runtime.generate_tokens([prompt], 12, eos_token_id=None)[0].tokens
        assert runtime.last_decode_profile is None
        assert runtime.generate_tokens([prompt], 12, eos_token_id=None, profile_decode_steps=5)[0].tokens == expect
        profile = runtime.last_decode_profile
        layers = config["num_hidden_layers"]
        assert profile.steps == 5 and profile.tokens == 5
        assert profile.launches % 5 == 0 and profile.launches // 5 >= 5 * layers
        assert 0 < profile.gpu_seconds <= profile.wall_seconds
        assert {"embed", "attention", "qknorm rope kv", "argmax"} <= set(profile.seconds_by_operation)
        # every layer's four products and the head, five times each
        assert sum(t.calls for t in profile.products.values()) == 5 * (4 * layers + 1)
        head = [t for (name, rows, columns, size), t in profile.products.items() if rows == config["vocab_size"]]
        assert sum(t.calls for t in head) == 5
        text = "\n".join(profile.lines())
        assert "decode profile: 5 evaluations" in text and "host gap" in text and "weight GB/s" in text
        from leone_amd.ops import profile as recording
        assert not recording.recording()


def test_command_line_eval_and_doctor(folders, tmp_path):
    """`leone eval`: windows of W tokens with stride W-1, a fresh cache per window, the row after token i
    scores token i+1 (crates/leone/src/runtime.rs:1673-1996); here against the plain logits of each window."""
    folder = folders["B"]
    weights, config = read_weights(folder), read_config(folder)
    tokens = random_tokens(5, 70, config["vocab_size"])
    tokens_file, logits_file, meta_file = tmp_path / "t.bin", tmp_path / "l.bin", tmp_path / "m.json"
    np.asarray(tokens, dtype="<u4").tofile(tokens_file)
    for chunk in (None, 7):
        cmd = [sys.executable, os.path.join(ROOT, "bin", "leone"), "eval", "-m", folder, "--tokens", str(tokens_file),
               "--logits", str(logits_file), "--window", "32", "--dtype", "float32", "--metadata", str(meta_file)]
        if chunk:
            cmd += ["--prefill-chunk", str(chunk)]
        run = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
        assert run.returncode == 0, run.stderr
        rows = np.fromfile(logits_file, dtype="<f4").reshape(-1, config["vocab_size"])
        expect = []
        start = 0
        while start < len(tokens) - 1:
            window = tokens[start:start + 32]
            expect.append(qwen3_plain.forward(weights, config, window).numpy()[:len(window) - 1])
            start += 31
        expect = np.concatenate(expect)
        assert rows.shape == expect.shape and np.abs(rows - expect).max() < 1e-4
        assert json.load(open(meta_file))["rows"] == rows.shape[0]
    doctor = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "leone"), "doctor", "-m", folder, "--probe"],
                            capture_output=True, text=True, timeout=300)
    assert doctor.returncode == 0, doctor.stdout + doctor.stderr
    assert "Qwen3ForCausalLM" in doctor.stdout and "tensor names and shapes: ok" in doctor.stdout

"""The double-precision sampler against a slow oracle and the reference's own test vectors."""
import math

import numpy as np
import pytest

from leone_amd.sampling import rng
from leone_amd.sampling.sampler import (SamplerError, SamplingParams, apply_penalties, argmax, distribution, sample,
                                        select)
from tests.plain import sampler_plain as oracle


def test_greedy_ties_and_nan():
    # crates/leone/src/sampler/tests.rs:521-537
    assert argmax(np.array([1, 4, 4, np.nan], dtype=np.float32)) == 1
    assert argmax(np.array([np.nan, np.inf, -np.inf], dtype=np.float32)) == -1
    with pytest.raises(SamplerError):
        sample(np.array([np.nan, np.nan], dtype=np.float32), SamplingParams(), 0)


def test_invalid_parameters():
    # crates/leone/src/sampler/tests.rs:659-668
    for bad in (0.0, float("nan"), -1.0, float("inf")):
        with pytest.raises(SamplerError):
            SamplingParams(temperature=bad).validate()
    with pytest.raises(SamplerError):
        SamplingParams(temperature=1.0, truncations=[("top_p", 0.0)]).validate()
    with pytest.raises(SamplerError):
        SamplingParams(temperature=1.0, truncations=[("top_k", 0)]).validate()


def test_rng_is_pure_and_in_range():
    # crates/leone/src/sampler/tests.rs:746-760
    seen = set()
    for seed in (0, 1, 2**63 + 5):
        for position in range(50):
            u = rng.uniform(seed, position)
            assert 0.0 <= u < 1.0
            assert u == rng.uniform(seed, position) == oracle.uniform(seed, position)
            seen.add(u)
    assert len(seen) == 150
    assert rng.uniform(3, 7, rng.PURPOSE_SELECT) != rng.uniform(3, 7, rng.PURPOSE_ACCEPT)


def test_top_k_keeps_exactly_k_and_min_p_cases():
    # crates/leone/src/sampler/tests.rs:539-548
    logits = np.array([0.1, 2.0, 1.5, -1.0, 0.7], dtype=np.float32)
    d = distribution(logits, SamplingParams(temperature=1.0, truncations=[("top_k", 3)]))
    assert (d > 0).sum() == 3 and abs(d.sum() - 1) < 1e-12
    peaked = np.array([10.0, 0.0, 0.0, 0.0], dtype=np.float32)
    flat = np.array([1.0, 1.0, 1.0, 1.0], dtype=np.float32)
    assert (distribution(peaked, SamplingParams(temperature=1.0, truncations=[("min_p", 0.5)])) > 0).sum() == 1
    assert (distribution(flat, SamplingParams(temperature=1.0, truncations=[("min_p", 0.5)])) > 0).sum() == 4


def test_low_temperature_concentrates_on_argmax():
    logits = np.random.default_rng(0).standard_normal(100).astype(np.float32)
    d = distribution(logits, SamplingParams(temperature=1e-3))
    assert d[argmax(logits)] > 0.999


def test_differential_against_slow_oracle():
    """Random rows, temperatures and stage pipelines: probabilities within 1e-12, same token
    (the reference's differential test, crates/leone/src/sampler/tests.rs:453-500)."""
    gen = np.random.default_rng(1234)
    for case in range(400):
        n = int(gen.integers(1, 60))
        logits = (gen.standard_normal(n) * gen.choice([0.1, 1.0, 5.0, 30.0])).astype(np.float32)
        if gen.random() < 0.3:
            logits[gen.integers(0, n)] = gen.choice([np.nan, np.inf, -np.inf])
        if gen.random() < 0.2 and n > 2:
            logits[1] = logits[0]
        if not np.isfinite(logits).any():
            continue
        t = float(gen.choice([0.05, 0.5, 0.8, 1.0, 1.7, 10.0]))
        stages = []
        for name in gen.permutation(["top_k", "top_p", "min_p"])[:int(gen.integers(0, 4))]:
            stages.append((str(name), float(gen.integers(1, 8)) if name == "top_k" else float(gen.uniform(0.05, 1.0))))
        params = SamplingParams(temperature=t, truncations=stages, seed=int(gen.integers(0, 2**62)))
        have = distribution(logits, params)
        want = oracle.distribution(logits.tolist(), t, stages)
        assert np.abs(have - np.array(want)).max() <= 1e-12, (case, stages)
        position = int(gen.integers(0, 10000))
        u = oracle.uniform(params.seed, position)
        assert sample(logits, params, position) == oracle.select(want, u) == select(have, u)


def test_penalties():
    # positive logits divided, negative multiplied, presence once, frequency per occurrence
    # (crates/leone/src/penalty.rs:160-196)
    logits = np.array([2.0, -2.0, 1.0, 0.5], dtype=np.float32)
    params = SamplingParams(repeat_penalty=2.0, presence_penalty=0.25, frequency_penalty=0.5, penalty_window=3)
    out = apply_penalties(logits, [3, 0, 1, 1], params)   # window keeps [0, 1, 1]
    assert out.tolist() == [2.0 / 2 - 0.25 - 0.5, -2.0 * 2 - 0.25 - 1.0, 1.0, 0.5]
    assert apply_penalties(logits, [0, 1], SamplingParams()) is logits
    assert not SamplingParams(repeat_penalty=2.0, penalty_window=0).penalties_active


def _dry_params(**kw):
    base = dict(dry_multiplier=1.0, dry_base=2.0, dry_allowed_length=2, dry_window=64)
    base.update(kw)
    return SamplingParams(**base)


def test_dry_reference_vectors():
    # crates/leone/src/penalty.rs:440-505: the expected values of the reference's own tests.
    zeros = np.zeros(8, dtype=np.float32)
    out = apply_penalties(zeros, [1, 2, 3, 4, 9, 1, 2, 3], _dry_params())
    assert out[4] == -2.0 and np.count_nonzero(out) == 1
    out = apply_penalties(zeros, [7, 1, 2, 3, 4, 9, 7, 1, 2, 3], _dry_params())
    assert out[4] == -4.0
    out = apply_penalties(zeros, [1, 2, 3, 4, 9, 1, 2, 3], _dry_params(dry_allowed_length=4))
    assert not out.any()
    out = apply_penalties(zeros, [1, 9, 2, 3, 5, 1, 9, 2], _dry_params(dry_breakers=(9,)))
    assert not out.any()
    with pytest.raises(SamplerError):
        _dry_params(dry_base=0.0).validate()


def test_dry_against_slow_oracle():
    gen = np.random.default_rng(11)
    for _ in range(400):
        vocab = int(gen.integers(1, 12))
        history = gen.integers(0, vocab, size=int(gen.integers(1, 40))).tolist()
        logits = gen.uniform(-8, 8, size=vocab).astype(np.float32)
        breakers = (int(gen.integers(0, vocab)),) if gen.random() < 0.3 else ()
        params = _dry_params(dry_multiplier=float(gen.uniform(0.1, 2)), dry_base=float(gen.uniform(1, 3)),
                             dry_allowed_length=int(gen.integers(1, 5)), dry_window=int(gen.integers(1, 48)),
                             dry_breakers=breakers)
        want = oracle.dry(logits, history, params.dry_multiplier, params.dry_base, params.dry_allowed_length,
                         params.dry_window, breakers)
        got = apply_penalties(logits, history, params)
        np.testing.assert_allclose(got, np.array(want, dtype=np.float32), rtol=1e-6, atol=1e-6)


def test_mirostat_controller():
    from leone_amd.sampling.sampler import MirostatState
    probs = np.array([0.5, 0.25, 0.125, 0.125, 0.0])
    # A generous bound keeps everything: the draw is the plain one and the bound moves by the error.
    state = MirostatState(1.0, 0.5, maximum_surprise=10.0)
    assert state.select(probs, 0.6) == 1
    assert state.maximum_surprise == pytest.approx(10.0 - 0.5 * (-np.log(0.25) - 1.0))
    # A bound below every surprise leaves the most likely token alone, whatever the draw.
    state = MirostatState(1.0, 1.0, maximum_surprise=0.1)
    assert state.select(probs, 0.99) == 0
    # The bound cuts the tail: with ln 4 < bound < ln 8 the two rarest tokens are gone and the rest renormalised.
    state = MirostatState(3.0, 0.1, maximum_surprise=1.5)
    assert state.select(probs, 0.7) == 1          # cumulative 2/3, 1 over {0.5, 0.25} / 0.75
    assert MirostatState(2.0, 0.1).maximum_surprise == 4.0
    with pytest.raises(SamplerError):
        SamplingParams(temperature=1.0, mirostat=(0.0, 0.1)).validate()
    with pytest.raises(SamplerError):
        SamplingParams(temperature=1.0, mirostat=(1.0, 1.5)).validate()
    # Against the loop oracle over a run of draws.
    gen = np.random.default_rng(5)
    state, bound = MirostatState(2.0, 0.3), 4.0
    for step in range(200):
        p = gen.dirichlet(np.full(9, 0.3))
        u = float(gen.random())
        token, bound = oracle.mirostat(p.tolist(), bound, 2.0, 0.3, u)
        assert state.select(p, u) == token
        assert state.maximum_surprise == pytest.approx(bound, rel=1e-12)


def test_native_rows_against_the_general_sampler_and_the_oracle():
    """The host library's sampler (selection instead of a full sort) draws what the general sampler draws:
    small rows against the slow oracle, full-vocabulary rows (peaked, flat, with ties, NaN and infinities)
    against the general sampler, and top-p 1.0, which has to look at everything."""
    from leone_amd.sampling.sampler import native_eligible, sample_rows_native
    gen = np.random.default_rng(4321)
    for case in range(300):
        n = int(gen.integers(1, 60))
        logits = (gen.standard_normal(n) * gen.choice([0.1, 1.0, 5.0, 30.0])).astype(np.float32)
        if gen.random() < 0.3:
            logits[gen.integers(0, n)] = gen.choice([np.nan, np.inf, -np.inf])
        if gen.random() < 0.2 and n > 2:
            logits[1] = logits[0]
        if not np.isfinite(logits).any():
            continue
        t = float(gen.choice([0.05, 0.5, 0.8, 1.0, 1.7, 10.0]))
        stages = [(str(name), float(gen.integers(1, 8)) if name == "top_k" else float(gen.uniform(0.05, 1.0)))
                  for name in gen.permutation(["top_k", "top_p", "min_p"])[:int(gen.integers(0, 4))]]
        params = SamplingParams(temperature=t, truncations=stages, seed=int(gen.integers(0, 2**62)))
        assert native_eligible(params)
        position = int(gen.integers(0, 10000))
        want = oracle.select(oracle.distribution(logits.tolist(), t, stages), oracle.uniform(params.seed, position))
        assert sample_rows_native(logits[None, :], [params], [position]) == [want], (case, stages)
    for vocab, spread in ((50000, 6.0), (151936, 3.0), (30000, 0.01)):
        rows = 5
        logits = (gen.standard_normal((rows, vocab)) * spread).astype(np.float32)
        logits[1, 17] = np.nan
        logits[2, :200] = logits[2, 0]                               # ties at the top
        logits[3, 5] = np.inf
        policies = [SamplingParams(temperature=0.8, truncations=[("top_k", 40), ("top_p", 0.9)], seed=3),
                    SamplingParams(temperature=1.3, truncations=[("top_p", 0.95)], seed=4),
                    SamplingParams(temperature=0.7, truncations=[("min_p", 0.02), ("top_k", 2000)], seed=5),
                    SamplingParams(temperature=1.0, truncations=[("top_p", 1.0)], seed=6),
                    SamplingParams(temperature=0.5, truncations=[("top_k", 100000)], seed=7)]
        positions = [11, 12, 13, 14, 15]
        got = sample_rows_native(logits, policies, positions)
        for r in range(rows):
            u = rng.uniform(policies[r].seed, positions[r])
            assert got[r] == select(distribution(logits[r], policies[r]), u), (vocab, r)
    assert not native_eligible(SamplingParams(temperature=1.0, truncations=[("tfs", 0.9)]))
    assert sample_rows_native(np.full((1, 7), np.nan, dtype=np.float32), [SamplingParams(temperature=1.0)], [0]) == [-1]

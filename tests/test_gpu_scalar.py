"""The float32 kernels and the float32 engine against the host library's scalar reference, which computes the
same formulas in the same precision with every sum left to right: what is left is the order of the sums
(the reference's kernels are held against its scalar backend in the same way, docs/oracle.md:16-21)."""
import math

import numpy as np
import pytest
import torch

from tests import scalar, schedules
from tests.util import TINY, make_model_dir, random_tokens, read_config, read_weights

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    return (t if dtype is None else t.to(dtype)).to(DEV)


def worst(have, want):
    return float(np.abs(have.float().cpu().numpy() - want).max())


def test_rowwise_kernels_and_products():
    from leone_amd import ops
    rng = np.random.default_rng(5)
    table = rng.standard_normal((300, 96)).astype(np.float32)
    tokens = [7, 299, 0, 150]
    assert np.array_equal(ops.embed(dev(table), dev(np.array(tokens, dtype=np.int32))).cpu().numpy(), scalar.embed(table, tokens))
    for hidden in (80, 1000, 4096):
        x = rng.standard_normal((6, hidden)).astype(np.float32) * 2
        delta = rng.standard_normal((3, 6, hidden)).astype(np.float32)
        gain = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
        xs = x.copy()
        want = scalar.add_rmsnorm(xs, delta, gain, 1e-6)
        xd = dev(x)
        got = ops.add_rmsnorm(xd, dev(delta), dev(gain), 1e-6, torch.float32)
        assert np.array_equal(xd.cpu().numpy(), xs)                       # the same additions in the same order
        assert worst(got, want) < 2e-6 * math.sqrt(hidden)
        rows = np.array([5, 0, 2], dtype=np.int32)
        assert worst(ops.add_rmsnorm(xd, dev(delta[0]), dev(gain), 1e-6, torch.float32, dev(rows)),
                     scalar.add_rmsnorm(xs, delta[0], gain, 1e-6, rows=rows)) < 2e-6 * math.sqrt(hidden)
    for m, n, k in [(5, 64, 64), (67, 1000, 333), (1, 777, 80)]:
        a, b = rng.standard_normal((m, k)).astype(np.float32), rng.standard_normal((n, k)).astype(np.float32)
        assert worst(ops.gemm_f32(dev(a), dev(b)), scalar.gemm(a, b)) < 2e-6 * k
    gate_up = rng.standard_normal((9, 2 * 88)).astype(np.float32) * 3
    assert worst(ops.swiglu(dev(gate_up)), scalar.swiglu(gate_up)) < 2e-6
    cos, sin = ops.rope_table(1e6, 64, 4096, DEV)
    want_cos, want_sin = scalar.rope_table(1e6, 64, 4096)
    assert worst(cos, want_cos) < 1e-7 and worst(sin, want_sin) < 1e-7    # both from double angles


@pytest.mark.parametrize("shape", [(4, 2, 16, 16), (6, 1, 32, 64), (5, 5, 48, 16), (8, 2, 128, 32)])
def test_cache_write_and_attention(shape):
    """The same scattered pages on both sides: the pools agree to rounding everywhere, also where nothing was
    written, and attention over them agrees for a window and without."""
    from leone_amd import ops
    q_heads, kv_heads, dim, page = shape
    rng = np.random.default_rng(6)
    rows_meta = [(0, p) for p in range(70)] + [(1, p) for p in range(3, 40)]      # (entry, position)
    n = len(rows_meta)
    width = (q_heads + 2 * kv_heads) * dim
    qkv = rng.standard_normal((n, width)).astype(np.float32)
    q_gain, k_gain = (1 + 0.1 * rng.standard_normal((2, dim))).astype(np.float32)
    blocks = -(-70 // page)
    pages = rng.permutation(2 * blocks + 2)
    table = np.full((2, blocks), -1, dtype=np.int32)
    table[0] = pages[:blocks]
    table[1, :-(-40 // page)] = pages[blocks:blocks + -(-40 // page)]
    k_pool = np.zeros((2 * blocks + 2, kv_heads, dim // 8, page, 8), dtype=np.float32)
    v_pool = np.zeros((2 * blocks + 2, kv_heads, page // 8, dim, 8), dtype=np.float32)
    # request 1 starts at position 3: its first three keys come from an earlier step
    k_pool[table[1, 0]], v_pool[table[1, 0]] = rng.standard_normal(k_pool[0].shape), rng.standard_normal(v_pool[0].shape)
    positions = np.array([p for _, p in rows_meta], dtype=np.int32)
    entry = np.array([e for e, _ in rows_meta], dtype=np.int32)
    cos, sin = scalar.rope_table(1e4, dim, 128)
    kd, vd = dev(k_pool), dev(v_pool)
    want_q = scalar.qk_norm_rope_write(qkv, q_heads, kv_heads, dim, q_gain, k_gain, 1e-5, cos, sin, positions, entry,
                                       table, k_pool, v_pool)
    got_q = ops.qk_norm_rope_write(dev(qkv), q_heads, kv_heads, dim, dev(q_gain), dev(k_gain), 1e-5, dev(cos), dev(sin),
                                   dev(positions), dev(entry), dev(table), kd, vd)
    assert worst(got_q, want_q) < 5e-6 and worst(kd, k_pool) < 5e-6 and np.array_equal(vd.cpu().numpy(), v_pool)
    for window in (0, 9):
        want = scalar.attention(want_q, k_pool, v_pool, positions, entry, table, q_heads, 1 / math.sqrt(dim), window)
        got = ops.attention_rows(got_q, kd, vd, dev(positions), dev(entry), dev(table), q_heads, 1 / math.sqrt(dim), window)
        assert worst(got, want) < 2e-5


def test_token_selection():
    from leone_amd import ops
    rng = np.random.default_rng(7)
    logits = rng.standard_normal((5, 9001)).astype(np.float32) * 4
    logits[0, 4097] = logits[0, 12] = logits[0].max() + 1
    logits[1] = np.nan
    logits[2, 100] = np.inf
    assert np.array_equal(ops.argmax(dev(logits)).cpu().numpy(), scalar.argmax(logits))
    temperature, uniform = np.array([0.7, 1.0, 1.3, 0.2, 2.0]), rng.random(5)
    got = ops.sample_temperature(dev(logits), dev(temperature), dev(uniform)).cpu().numpy()
    assert np.array_equal(got, scalar.sample_temperature(logits, temperature, uniform))


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_float32_engine_against_the_scalar_model(tmp_path, name):
    """Mixed steps with page reuse on the device, each request whole on the host: rounding only."""
    from leone_amd.engine.engine import Engine, StepEntry
    from leone_amd.runtime import load_model
    folder = make_model_dir(str(tmp_path / "m"), TINY[name], 51, torch.float32, sharpen=2.0)
    weights, config = read_weights(folder), read_config(folder)
    requests = {f"s{i}": random_tokens(300 + i, n, config["vocab_size"]) for i, n in enumerate([60, 33, 90, 17, 48])}
    steps = schedules.mixed(requests)
    engine = Engine(load_model(folder, "float32"), num_pages=schedules.max_live_tokens(steps, 16) // 16, page_tokens=16,
                    max_requests=4, poison_freed=True)
    outputs = {}
    for s in steps:
        out = engine.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        outputs[s["step"]] = out.logits.cpu().numpy()
        for rid in s["end"]:
            engine.release(rid)
    got = schedules.collect(steps, outputs)
    for rid, tokens in requests.items():
        pages = list(range(-(-len(tokens) // 16)))
        want = scalar.ScalarQwen3(weights, config, pages, 16).step(tokens)
        err = np.abs(np.stack(got[rid]) - want).max()
        assert err < 2e-5, (rid, err)

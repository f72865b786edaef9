"""The scalar single-precision reference in the host library against the double-precision plain implementation,
one operation at a time and as a whole model; and a paged cache against a contiguous one, bit for bit
(crates/leone/tests/cpu_kv_span_attention_oracle.rs: paged equals contiguous)."""
import math

import numpy as np
import pytest
import torch

from tests import scalar
from tests.plain import qwen3_plain as plain, sampler_plain
from tests.util import TINY, make_model_dir, random_tokens, read_config, read_weights


def test_embed_norm_product_and_activation():
    rng = np.random.default_rng(1)
    table = rng.standard_normal((50, 24)).astype(np.float32)
    out = scalar.embed(table, [3, 49, 0, 50, -1])
    assert np.array_equal(out[:3], table[[3, 49, 0]]) and np.isnan(out[3:]).all()
    x = rng.standard_normal((5, 72)).astype(np.float32) * 3
    delta = rng.standard_normal((3, 5, 72)).astype(np.float32)
    gain = (1 + 0.1 * rng.standard_normal(72)).astype(np.float32)
    before = x.copy()
    y = scalar.add_rmsnorm(x, delta, gain, 1e-5)
    total = ((before + delta[0]) + delta[1]) + delta[2]
    assert np.array_equal(x, total)                                       # planes in order, in float
    want = plain.rms_norm(torch.from_numpy(total), torch.from_numpy(gain), 1e-5).numpy()
    assert np.abs(y - want).max() < 5e-6
    rows = [4, 0, 4]
    kept = x.copy()
    picked = scalar.add_rmsnorm(x, delta[0], gain, 1e-5, rows=rows)
    assert np.array_equal(x, kept)                                        # rows given: the stream stays
    assert np.abs(picked - plain.rms_norm(torch.from_numpy((kept + delta[0])[rows]), torch.from_numpy(gain), 1e-5).numpy()).max() < 5e-6
    a, b = rng.standard_normal((7, 130)).astype(np.float32), rng.standard_normal((33, 130)).astype(np.float32)
    assert np.abs(scalar.gemm(a, b) - a.astype(np.float64) @ b.astype(np.float64).T).max() < 1e-4
    gate, up = rng.standard_normal((4, 24)).astype(np.float32) * 4, rng.standard_normal((4, 24)).astype(np.float32)
    mixed = np.stack([gate.reshape(4, 3, 8), up.reshape(4, 3, 8)], axis=2).reshape(4, 48)
    assert np.abs(scalar.swiglu(mixed) - plain.swiglu(torch.from_numpy(gate), torch.from_numpy(up)).numpy()).max() < 1e-6


@pytest.mark.parametrize("shape", [(4, 2, 16, 16), (6, 1, 32, 8), (5, 5, 48, 16)])
def test_rotation_cache_write_and_attention(shape):
    q_heads, kv_heads, dim, page = shape
    rng = np.random.default_rng(2)
    n, theta, eps = 37, 1e4, 1e-5
    width = (q_heads + 2 * kv_heads) * dim
    qkv = rng.standard_normal((n, width)).astype(np.float32)
    q_gain, k_gain = (1 + 0.1 * rng.standard_normal((2, dim))).astype(np.float32)
    blocks = -(-n // page)
    pages = rng.permutation(blocks + 3)[:blocks]
    table = np.array([pages], dtype=np.int32)
    k_pool = np.full((blocks + 3, kv_heads, dim // 8, page, 8), np.nan, dtype=np.float32)
    v_pool = np.full((blocks + 3, kv_heads, page // 8, dim, 8), np.nan, dtype=np.float32)
    cos, sin = scalar.rope_table(theta, dim, 64)
    positions, entry = np.arange(n), np.zeros(n)
    q = scalar.qk_norm_rope_write(qkv, q_heads, kv_heads, dim, q_gain, k_gain, eps, cos, sin, positions, entry, table,
                                  k_pool, v_pool)
    t = torch.from_numpy(qkv)
    tq = t[:, :q_heads * dim].view(n, q_heads, dim)
    tk = t[:, q_heads * dim:(q_heads + kv_heads) * dim].view(n, kv_heads, dim)
    tv = t[:, (q_heads + kv_heads) * dim:].view(n, kv_heads, dim)
    want_q = plain.rope_half_split(plain.rms_norm(tq, torch.from_numpy(q_gain), eps), positions, theta)
    want_k = plain.rope_half_split(plain.rms_norm(tk, torch.from_numpy(k_gain), eps), positions, theta)
    assert np.abs(q.reshape(n, q_heads, dim) - want_q.numpy()).max() < 1e-5
    keys = k_pool.transpose(0, 1, 3, 2, 4).reshape(-1, kv_heads, page, dim)       # [page][head][token][element]
    values = v_pool.transpose(0, 1, 2, 4, 3).reshape(-1, kv_heads, page, dim)
    for i in range(n):
        assert np.abs(keys[pages[i // page], :, i % page] - want_k[i].numpy()).max() < 1e-5
        assert np.array_equal(values[pages[i // page], :, i % page], tv[i].numpy())
    for window in (0, 5):
        out = scalar.attention(q, k_pool, v_pool, positions, entry, table, q_heads, 1 / math.sqrt(dim), window)
        want = plain.causal_attention(want_q, want_k, tv, window or None)
        assert np.abs(out.reshape(n, q_heads, dim) - want.numpy()).max() < 2e-5
    # planes of a product cut along K are added up first
    parts = np.stack([qkv * 0.75, qkv * 0.25])
    again = scalar.qk_norm_rope_write(parts, q_heads, kv_heads, dim, q_gain, k_gain, eps, cos, sin, positions, entry,
                                      table, k_pool.copy(), v_pool.copy())
    assert np.abs(again - q).max() < 1e-6
    # a key without a page is reported, never read
    table[0, 0] = -1
    assert np.isnan(scalar.attention(q[:1], k_pool, v_pool, [0], [0], table, q_heads, 1.0)).all()


def test_token_selection_follows_the_sampler_oracle():
    rng = np.random.default_rng(3)
    logits = rng.standard_normal((6, 300)).astype(np.float32) * 3
    logits[0, 17] = logits[0, 5] = logits[0].max() + 1          # a tie: the lower index wins
    logits[1, :] = np.nan
    logits[2, 40] = np.inf                                       # infinities never win
    picked = scalar.argmax(logits)
    assert picked[0] == 5 and picked[1] == -1 and picked[2] != 40
    for r in range(2, 6):
        assert picked[r] == sampler_plain.greedy(logits[r].tolist())
    temperature, uniform = np.array([0.7, 1.0, 1.3, 0.2, 2.0, 1.0]), rng.random(6)
    drawn = scalar.sample_temperature(logits, temperature, uniform)
    assert drawn[1] == -1
    for r in (0, 2, 3, 4, 5):
        probs = sampler_plain.distribution(logits[r].tolist(), float(temperature[r]))
        assert drawn[r] == sampler_plain.select(probs, float(uniform[r]))


@pytest.mark.parametrize("name", ["A", "B"])
def test_scalar_model_against_plain_and_paged_against_contiguous(tmp_path, name):
    """The whole model built from the scalar functions equals the double-precision plain implementation at
    float rounding; fed in portions over scattered pages it gives the same bits as whole over pages in order."""
    folder = make_model_dir(str(tmp_path / "m"), TINY[name], 41, torch.float32, sharpen=2.0)
    weights, config = read_weights(folder), read_config(folder)
    tokens = random_tokens(77, 45, config["vocab_size"])
    want = plain.forward(weights, config, tokens).numpy()
    whole = scalar.ScalarQwen3(weights, config, pages=[0, 1, 2], page_tokens=16).step(tokens)
    assert np.abs(whole - want).max() < 1e-4
    paged = scalar.ScalarQwen3(weights, config, pages=[5, 0, 3], page_tokens=16)
    rows, at = [], 0
    for size in (7, 2, 16, 1, 1, 18):
        rows.append(paged.step(tokens[at:at + size]))
        at += size
    assert at == len(tokens) and np.array_equal(np.concatenate(rows), whole)

"""Pins the plain implementation by what fixes it beside the reference's text: the vectors the
reference's own tests hold, special cases that reduce to a library routine, and invariants, each
chosen so that a plausible mistake (a wrong sign or pairing, a norm in the wrong place) fails."""
import math

import pytest
import torch

from tests.plain import qwen3_plain as plain
from tests.util import TINY_A, TINY_B, make_model_dir, random_tokens, read_config, read_weights

F64 = torch.float64


def test_rms_norm_reference_vector_and_closed_form():
    # rows [1,2],[3,4], gain [1,0.5], eps 1e-6: the largest output is index 2 (crates/leone/src/cpu.rs:2781-2807)
    y = plain.rms_norm(torch.tensor([[1.0, 2.0], [3.0, 4.0]]), torch.tensor([1.0, 0.5]), 1e-6)
    assert int(y.flatten().argmax()) == 2
    assert abs(float(y[0, 0]) - 1.0 / math.sqrt(2.5 + 1e-6)) < 1e-15
    x = torch.randn(5, 37, dtype=F64)
    unit = plain.rms_norm(x, torch.ones(37), 0.0)
    assert torch.allclose((unit * unit).mean(dim=-1), torch.ones(5, dtype=F64))      # output RMS is 1
    assert torch.allclose(plain.rms_norm(7.0 * x, torch.ones(37), 0.0), unit)        # scale invariance
    # eps is added to the mean inside the root, not to the root and not to the sum
    one = plain.rms_norm(torch.tensor([[2.0, 2.0]]), torch.tensor([1.0, 1.0]), 5.0)
    assert abs(float(one[0, 0]) - 2.0 / 3.0) < 1e-15
    # the gain multiplies directly: a zero gain gives zero (it is not 1 + gain)
    assert float(plain.rms_norm(x, torch.zeros(37), 1e-6).abs().max()) == 0.0


def test_rope_pairs_signs_and_frequencies():
    dim, theta = 16, 10000.0
    x = torch.randn(6, 3, dim, dtype=F64)
    positions = [0, 1, 2, 17, 2048, 8000]
    y = plain.rope_half_split(x, positions, theta)
    assert torch.equal(y[0], x[0])                                               # position 0 is the identity
    half = dim // 2
    assert torch.allclose(y[..., :half] ** 2 + y[..., half:] ** 2, x[..., :half] ** 2 + x[..., half:] ** 2)
    # a unit vector e_i moves only into slots i and i + D/2 (half-split, not adjacent pairs),
    # by the angle pos * theta^(-2i/D), counter-clockwise: (cos, +sin)
    for i in (0, 3, 7):
        e = torch.zeros(1, 1, dim, dtype=F64)
        e[0, 0, i] = 1.0
        r = plain.rope_half_split(e, [5], theta)[0, 0]
        angle = 5 * theta ** (-2.0 * i / dim)
        expect = torch.zeros(dim, dtype=F64)
        expect[i], expect[i + half] = math.cos(angle), math.sin(angle)
        assert torch.allclose(r, expect, atol=1e-15)
    # equals complex multiplication of (a + ib) by e^{i angle}: a library routine
    z = torch.complex(x[..., :half], x[..., half:])
    angles = torch.tensor([[p * theta ** (-2.0 * i / dim) for i in range(half)] for p in positions], dtype=F64)
    w = z * torch.polar(torch.ones_like(angles), angles)[:, None, :]
    assert torch.allclose(y, torch.cat([w.real, w.imag], dim=-1), atol=1e-12)
    # 16 elements a head mean 8 inverse frequencies, the first 1, the last theta^(-14/16) (crates/leone/src/cpu.rs:2752-2762)
    e = torch.zeros(1, 1, dim, dtype=F64); e[0, 0, 7] = 1.0
    assert abs(float(plain.rope_half_split(e, [1], theta)[0, 0, 7]) - math.cos(theta ** (-14.0 / 16.0))) < 1e-15


def test_rope_scores_depend_only_on_distance():
    q, k = torch.randn(1, 1, 32, dtype=F64), torch.randn(1, 1, 32, dtype=F64)

    def score(m, n):
        return float((plain.rope_half_split(q, [m], 1e6) * plain.rope_half_split(k, [n], 1e6)).sum())
    assert abs(score(10, 3) - score(110, 103)) < 1e-9
    assert abs(score(10, 3) - score(10, 4)) > 1e-6


def test_rotation_with_its_shape_as_parameters():
    """``rope_pairs`` pinned by what fixes it: over the whole head in half-split pairs it is ``rope_half_split``;
    the adjacent pairing is the same rotation on a permuted head (element 2i <-> i, 2i + 1 <-> i + R/2); elements
    beyond rotary_dim come through untouched and the rotated ones do not depend on them; scores depend on
    distances only, whatever the shape."""
    dim, theta = 24, 5000.0
    x = torch.randn(5, 2, dim, dtype=F64)
    positions = [0, 3, 9, 100, 4000]
    assert torch.equal(plain.rope_pairs(x, positions, theta, dim, "half_split"), plain.rope_half_split(x, positions, theta))
    for rotary in (8, 16, 24):
        half = rotary // 2
        split = plain.rope_pairs(x, positions, theta, rotary, "half_split")
        assert torch.equal(split[..., rotary:], x[..., rotary:])
        assert torch.equal(split[..., :rotary], plain.rope_half_split(x[..., :rotary], positions, theta))
        order = [2 * i for i in range(half)] + [2 * i + 1 for i in range(half)]     # adjacent slot of each half-split slot
        permuted = x.clone()
        permuted[..., order] = x[..., :rotary]
        adjacent = plain.rope_pairs(permuted, positions, theta, rotary, "adjacent")
        assert torch.allclose(adjacent[..., order], split[..., :rotary], atol=1e-14)
        assert torch.equal(adjacent[..., rotary:], x[..., rotary:])
        # a unit vector at slot 2 of an adjacent pairing moves into slots 2 and 3 by angle pos * theta^(-2/R)
        e = torch.zeros(1, 1, dim, dtype=F64); e[0, 0, 2] = 1.0
        r = plain.rope_pairs(e, [7], theta, rotary, "adjacent")[0, 0]
        angle = 7 * theta ** (-2.0 / rotary)
        assert abs(float(r[2]) - math.cos(angle)) < 1e-15 and abs(float(r[3]) - math.sin(angle)) < 1e-15
        q, k = torch.randn(1, 1, dim, dtype=F64), torch.randn(1, 1, dim, dtype=F64)
        for pairing in ("half_split", "adjacent"):
            score = lambda m, n: float((plain.rope_pairs(q, [m], theta, rotary, pairing) * plain.rope_pairs(k, [n], theta, rotary, pairing)).sum())
            assert abs(score(10, 3) - score(510, 503)) < 1e-9


def test_attention_reference_vector():
    # 2 heads, 1 kv head, D=2; K rows [1,0],[0,1]; V rows [2,4],[6,8]; q [1,0] for head 0, [0,1] for head 1
    # (crates/leone/src/cpu.rs:2850-2898)
    k = torch.tensor([[[1.0, 0.0]], [[0.0, 1.0]]])
    v = torch.tensor([[[2.0, 4.0]], [[6.0, 8.0]]])
    q = torch.tensor([[[1.0, 0.0], [0.0, 1.0]], [[1.0, 0.0], [0.0, 1.0]]])
    out = plain.causal_attention(q, k, v).reshape(2, 4)
    h = math.exp(1.0 / math.sqrt(2.0))
    want = torch.tensor([[2.0, 4.0, 2.0, 4.0],
                         [(h * 2 + 6) / (h + 1), (h * 4 + 8) / (h + 1), (2 + h * 6) / (h + 1), (4 + h * 8) / (h + 1)]],
                        dtype=F64)
    assert torch.allclose(out, want, atol=1e-12)


def test_attention_special_cases_and_library_routine():
    torch.manual_seed(0)
    q, k, v = torch.randn(9, 6, 8, dtype=F64), torch.randn(9, 2, 8, dtype=F64), torch.randn(9, 2, 8, dtype=F64)
    out = plain.causal_attention(q, k, v)
    assert torch.allclose(out[0], v[0].repeat_interleave(3, dim=0))              # one key: that value row
    zero_q = plain.causal_attention(torch.zeros_like(q), k, v)
    assert torch.allclose(zero_q[4, 0], v[:5, 0].mean(dim=0))                    # equal scores: the mean
    # library scaled-dot-product attention with kv heads repeated: head h uses kv head h // 3
    lib = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.repeat_interleave(3, 1).transpose(0, 1)[None],
        v.repeat_interleave(3, 1).transpose(0, 1)[None], is_causal=True)[0].transpose(0, 1)
    assert torch.allclose(out, lib, atol=1e-12)
    # later tokens never change earlier rows
    k2, v2 = k.clone(), v.clone()
    k2[6:], v2[6:] = 9.0, -9.0
    assert torch.equal(plain.causal_attention(q, k2, v2)[:6], out[:6])
    # a window of w keeps keys t-w+1 .. t
    w3 = plain.causal_attention(q, k, v, window=3)
    assert torch.allclose(w3[:3], out[:3]) and not torch.allclose(w3[5], out[5])
    assert torch.allclose(w3[8], plain.attend_one(q[8], k[6:9], v[6:9]))


def test_swiglu_is_silu_times_up():
    g, u = torch.linspace(-8, 8, 101, dtype=F64), torch.linspace(-2, 2, 101, dtype=F64)
    assert torch.allclose(plain.swiglu(g, u), torch.nn.functional.silu(g) * u, atol=1e-15)
    assert float(plain.swiglu(torch.zeros(3), torch.ones(3)).abs().max()) == 0.0
    assert abs(float(plain.swiglu(torch.tensor([30.0]), torch.tensor([2.0]))) - 60.0) < 1e-9
    assert abs(float(plain.swiglu(torch.tensor([-30.0]), torch.tensor([2.0])))) < 1e-10


@pytest.fixture(scope="module")
def tiny(tmp_path_factory):
    out = {}
    for name, raw in (("A", TINY_A), ("B", TINY_B)):
        folder = make_model_dir(str(tmp_path_factory.mktemp(name)), raw, 3, torch.float32)
        out[name] = (read_weights(folder), read_config(folder))
    return out


def test_whole_model_invariants(tiny):
    weights, config = tiny["B"]
    tokens = random_tokens(1, 24, config["vocab_size"])
    logits = plain.forward(weights, config, tokens)
    assert logits.shape == (24, config["vocab_size"])
    # causal: a row does not depend on later tokens
    other = tokens[:10] + random_tokens(2, 14, config["vocab_size"])
    assert torch.equal(plain.forward(weights, config, other)[:10], logits[:10])
    assert not torch.allclose(plain.forward(weights, config, other)[10:], logits[10:])
    # untied: the head is lm_head, not the embedding
    swapped = dict(weights, **{"lm_head.weight": weights["model.embed_tokens.weight"]})
    assert not torch.allclose(plain.forward(swapped, config, tokens), logits)
    tied = plain.forward(weights, dict(config, tie_word_embeddings=True), tokens)
    assert torch.equal(tied, plain.forward(swapped, config, tokens))               # tied == untied copy of E


def test_zero_layers_is_head_of_norm_of_embedding(tiny):
    # the reference's zero-layer toy runtime (crates/leone/src/runtime.rs:11497-11565)
    weights, config = tiny["A"]
    tokens = [5, 9, 5]
    logits = plain.forward(weights, dict(config, num_hidden_layers=0), tokens)
    e = weights["model.embed_tokens.weight"].double()
    want = plain.rms_norm(e[tokens], weights["model.norm.weight"], config["rms_norm_eps"]) @ e.T
    assert torch.allclose(logits, want, atol=1e-14)
    assert torch.equal(logits[0], logits[2])                                       # no position term at all


def test_residuals_and_norm_placement(tiny):
    """With the output projections zeroed each block adds nothing, so the logits equal the zero-layer
    model's: the residual path carries x unnormalised (a norm applied to the stream itself would show)."""
    weights, config = tiny["A"]
    tokens = random_tokens(3, 7, config["vocab_size"])
    muted = dict(weights)
    for name in weights:
        if name.endswith("o_proj.weight") or name.endswith("down_proj.weight"):
            muted[name] = torch.zeros_like(weights[name])
    assert torch.allclose(plain.forward(muted, config, tokens),
                          plain.forward(weights, dict(config, num_hidden_layers=0), tokens), atol=1e-14)
    # only the feed-forward muted: x1 = x + attention(norm(x)); scaling the input gain of a layer changes
    # the attention input only through the norm, never the residual itself
    only_attention = dict(weights)
    for name in weights:
        if name.endswith("down_proj.weight"):
            only_attention[name] = torch.zeros_like(weights[name])
    a = plain.forward(only_attention, dict(config, num_hidden_layers=1), tokens)
    x = plain.embedding(weights["model.embed_tokens.weight"], tokens)
    y = plain.rms_norm(x, weights["model.layers.0.input_layernorm.weight"], config["rms_norm_eps"])
    x1 = x + plain.attention_block(y, weights, "model.layers.0.self_attn", config, list(range(len(tokens))))
    want = plain.rms_norm(x1, weights["model.norm.weight"], config["rms_norm_eps"]) @ weights["model.embed_tokens.weight"].double().T
    assert torch.allclose(a, want, atol=1e-13)


def test_q_and_k_norm_come_before_the_rotation_and_skip_v(tiny):
    weights, config = tiny["B"]
    tokens = random_tokens(4, 6, config["vocab_size"])
    # inputs large enough that eps is negligible beside the mean square of a projected head
    x = plain.embedding(weights["model.embed_tokens.weight"], tokens) * 1000.0
    base = plain.attention_block(x, weights, "model.layers.0.self_attn", config, list(range(6)))
    # doubling Wq or Wk changes nothing (the per-head norm removes the scale); doubling Wv doubles the output
    for name, factor in (("q_proj", 1.0), ("k_proj", 1.0), ("v_proj", 2.0)):
        scaled = dict(weights)
        scaled[f"model.layers.0.self_attn.{name}.weight"] = weights[f"model.layers.0.self_attn.{name}.weight"] * 2
        out = plain.attention_block(x, scaled, "model.layers.0.self_attn", config, list(range(6)))
        assert torch.allclose(out, base * factor, rtol=1e-5, atol=1e-5), name
    # shifting every position by the same amount changes nothing: only distances count
    shifted = plain.attention_block(x, weights, "model.layers.0.self_attn", config, list(range(100, 106)))
    assert torch.allclose(shifted, base, atol=1e-8)


def test_gate_is_the_activated_projection_by_numbers():
    """silu goes on gate_proj's result, up_proj's multiplies it (crates/leone/src/cpu.rs:892-907 with the
    operands of crates/leone/src/runtime.rs:9283-9319).  One input, one unit each: gate 2, up 3 gives
    2 / (1 + e^-2) * 3 = 5.2847...; the other way round it would be 3 / (1 + e^-3) * 2 = 5.7154..."""
    weights = {"f.gate_proj.weight": torch.tensor([[2.0]]), "f.up_proj.weight": torch.tensor([[3.0]]),
               "f.down_proj.weight": torch.tensor([[1.0]])}
    out = plain.feed_forward(torch.tensor([[1.0]]), weights, "f")
    assert abs(float(out) - 5.284782467867294) < 1e-12
    assert abs(float(out) - 5.715445096562234) > 0.4


def test_head_norms_use_the_layer_norms_eps_by_numbers():
    """q and k are normalised with rms_norm_eps (crates/leone/src/runtime.rs:9227-9241 passes the model's one
    epsilon).  Activations small enough for eps to matter: q = (3e-3, 4e-3), mean square 1.25e-5, eps 1e-5:
    q / sqrt(2.25e-5) = (0.63246, 0.84327); with another eps (1e-6) it would be (0.81650, 1.08866).  One head
    of size 2, one position, so rotation by angle 0 and attention over one key change nothing: the output is v."""
    config = dict(num_attention_heads=1, num_key_value_heads=1, head_dim=2, rms_norm_eps=1e-5, rope_theta=1e4)
    eye = torch.eye(2)
    weights = {"a.q_proj.weight": eye, "a.k_proj.weight": eye, "a.v_proj.weight": eye, "a.o_proj.weight": eye,
               "a.q_norm.weight": torch.ones(2), "a.k_norm.weight": torch.ones(2)}
    y = torch.tensor([[3e-3, 4e-3]])
    normed = plain.rms_norm(y.view(1, 1, 2), weights["a.q_norm.weight"], config["rms_norm_eps"])
    assert torch.allclose(normed.view(2), torch.tensor([0.6324555320336759, 0.8432740427115678], dtype=torch.float64), atol=1e-12)
    # and through the block, two positions: the second attends both keys with weights that depend on q . k,
    # which depends on that factor: softmax over (q1.k0, q1.k1) / sqrt(2)
    y2 = torch.tensor([[3e-3, 4e-3], [4e-3, -3e-3]])
    out = plain.attention_block(y2, weights, "a", config, [0, 0])       # both at position 0: no rotation
    n0, n1 = [v / math.sqrt((v * v).sum() / 2 + 1e-5) for v in (y2[0].double(), y2[1].double())]
    scores = torch.stack([n1 @ n0, n1 @ n1]) / math.sqrt(2)
    w = torch.softmax(scores, dim=0)
    assert torch.allclose(out[1], w[0] * y2[0].double() + w[1] * y2[1].double(), atol=1e-12)
    wrong = [v / math.sqrt((v * v).sum() / 2 + 1e-6) for v in (y2[0].double(), y2[1].double())]
    wrong_w = torch.softmax(torch.stack([wrong[1] @ wrong[0], wrong[1] @ wrong[1]]) / math.sqrt(2), dim=0)
    assert (wrong_w - w).abs().max() > 0.02


def test_rows_of_one_layer_equal_the_whole_forward():
    """The row-by-row evaluation of a one-layer model (used where the whole forward would cost the square of
    100,000 tokens) gives what ``forward`` gives at those rows."""
    torch.manual_seed(3)
    config = dict(num_hidden_layers=1, hidden_size=48, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
                  intermediate_size=80, vocab_size=97, rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=False)
    names = {"model.embed_tokens.weight": (97, 48), "lm_head.weight": (97, 48), "model.norm.weight": (48,),
             "model.layers.0.input_layernorm.weight": (48,), "model.layers.0.post_attention_layernorm.weight": (48,),
             "model.layers.0.self_attn.q_proj.weight": (64, 48), "model.layers.0.self_attn.k_proj.weight": (32, 48),
             "model.layers.0.self_attn.v_proj.weight": (32, 48), "model.layers.0.self_attn.o_proj.weight": (48, 64),
             "model.layers.0.self_attn.q_norm.weight": (16,), "model.layers.0.self_attn.k_norm.weight": (16,),
             "model.layers.0.mlp.gate_proj.weight": (80, 48), "model.layers.0.mlp.up_proj.weight": (80, 48),
             "model.layers.0.mlp.down_proj.weight": (48, 80)}
    weights = {name: torch.randn(shape) * (1.0 if len(shape) == 1 else 0.3) for name, shape in names.items()}
    tokens = [int(t) for t in torch.randint(0, 97, (40,))]
    whole = plain.forward(weights, config, tokens)
    rows = [0, 7, 38, 39]
    assert torch.allclose(plain.forward_rows_of_one_layer(weights, config, tokens, rows), whole[rows], rtol=0, atol=1e-12)
    x = torch.randn(9, 3, 16, dtype=torch.float64)
    positions = [0, 1, 2, 77, 1000, 31000, 99999, 5, 100007]
    assert torch.allclose(plain.rope_half_split_at_once(x, positions, 1e6), plain.rope_half_split(x, positions, 1e6), rtol=0, atol=1e-12)

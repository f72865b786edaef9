"""Each HIP kernel alone against a plain float64 computation, at sizes other than the engine's."""
import math

import numpy as np
import pytest
import torch

from tests.plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def close(have, want, atol, rtol, what=""):
    have, want = have.double().cpu(), want.double().cpu()
    err = (have - want).abs()
    bound = atol + rtol * want.abs()
    bad = err > bound
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.numel()} off, worst {float((err - bound).max()):.3e} over"


def tol(dtype):
    # float32: a few ulps of sums over up to thousands of terms; bfloat16: one rounding of the output (2^-8).
    return (2e-5, 2e-5) if dtype == torch.float32 else (1e-2, 1e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(dtype):
    from leone_amd import ops
    torch.manual_seed(0)
    table = torch.randn(777, 80, device=DEV).to(dtype)
    tokens = torch.tensor([0, 776, 5, 5, 123], dtype=torch.int32, device=DEV)
    out = ops.embed(table, tokens)
    assert out.dtype == torch.float32
    assert torch.equal(out, table.float()[tokens.long()])
    assert torch.equal(ops.embed(table, tokens, scale=3.0), table.float()[tokens.long()] * 3.0)
    values = torch.randn(7, 333, device=DEV) * 40
    capped = ops.soft_cap(values.clone(), 30.0)
    close(capped, 30.0 * torch.tanh(values.double() / 30.0), 1e-5, 1e-6, "soft cap")


@pytest.mark.parametrize("hidden", [80, 1000, 4096, 5120])
@pytest.mark.parametrize("dtype", DTYPES)
def test_add_rmsnorm(dtype, hidden):
    from leone_amd import ops
    torch.manual_seed(1)
    x = torch.randn(7, hidden, device=DEV) * 3
    delta = torch.randn(7, hidden, device=DEV).to(dtype)
    gain = (1 + 0.1 * torch.randn(hidden, device=DEV))
    eps = 1e-5
    x0 = x.clone()
    y = ops.add_rmsnorm(x, delta, gain, eps, dtype)
    want_x = x0.double() + delta.double()
    assert torch.equal(x, (x0 + delta.float()))          # the stream is updated in float
    close(y, plain.rms_norm(want_x.cpu(), gain.cpu(), eps), *tol(dtype), "add_rmsnorm")
    # without a delta the stream is untouched
    x1 = x.clone()
    y2 = ops.add_rmsnorm(x, None, gain.to(dtype), eps, dtype)
    assert torch.equal(x, x1)
    close(y2, plain.rms_norm(x1.cpu(), gain.to(dtype).cpu(), eps), *tol(dtype), "rmsnorm")
    # gathered rows: x stays, only the chosen rows come out
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device=DEV)
    y3 = ops.add_rmsnorm(x, delta, gain, eps, torch.float32, rows=rows)
    assert torch.equal(x, x1)
    close(y3, plain.rms_norm((x1.double() + delta.double())[rows.long()].cpu(), gain.cpu(), eps), 2e-5, 2e-5, "gather")


@pytest.mark.parametrize("hidden", [80, 4096, 9000])
def test_add_rmsnorm_takes_what_is_added_in_planes(hidden):
    """The parts of a product whose inner dimension was cut come as planes; their sum in order is added."""
    from leone_amd import ops
    torch.manual_seed(3)
    rows = 7
    x = torch.randn(rows, hidden, device=DEV)
    planes = torch.randn(3, rows, hidden, device=DEV)
    gain = 1 + 0.1 * torch.randn(hidden, device=DEV)
    whole = ((x + planes[0]) + planes[1]) + planes[2]                 # the planes are added one after the other
    want_y = ops.add_rmsnorm(whole.clone(), None, gain, 1e-5, torch.float32)
    mine = x.clone()
    got_y = ops.add_rmsnorm(mine, planes, gain, 1e-5, torch.float32)
    assert torch.equal(mine, whole) and torch.equal(got_y, want_y)
    picked = torch.tensor([5, 0, 5, 2], dtype=torch.int32, device=DEV)
    untouched = x.clone()
    got = ops.add_rmsnorm(untouched, planes, gain, 1e-5, torch.bfloat16, picked)
    assert torch.equal(untouched, x)
    assert torch.equal(got, ops.add_rmsnorm(whole.clone(), None, gain, 1e-5, torch.bfloat16, picked))
    with pytest.raises(ops.KernelError):
        ops.add_rmsnorm(x.clone(), torch.zeros(17, rows, hidden, device=DEV), gain, 1e-5, torch.float32)


def test_linear_cuts_a_long_inner_dimension_for_a_few_hundred_rows():
    """A product that goes into the stream with a few hundred rows, few columns and a long inner dimension
    comes back in planes, which the next norm adds up: the same stream as with the product whole."""
    from leone_amd import ops
    torch.manual_seed(4)
    rows, n, k = 300, 64, 8192
    assert ops.inner_parts(rows, n, k) == 4 and ops.inner_parts(1000, n, k) == 2
    assert ops.inner_parts(2048, n, k) == 1 and ops.inner_parts(64, n, k) == 1 and ops.inner_parts(rows, 8192, 8192) == 1
    assert ops.inner_parts(65, n, k) == 4
    assert ops.inner_parts(rows, n, 8192 + 64) == 1          # no part would be whole steps of 64
    x = (torch.randn(rows, k, device=DEV) * 0.5).bfloat16()
    w = (torch.randn(n, k, device=DEV) * 0.05).bfloat16()
    stream = torch.randn(rows, n, device=DEV)
    delta = ops.linear(x, w, residual=stream)
    assert delta.shape == (4, rows, n) and delta.dtype == torch.float32
    gain = torch.ones(n, device=DEV)
    after = stream.clone()
    ops.add_rmsnorm(after, delta, gain, 1e-6, torch.bfloat16)
    want = stream.double() + x.double() @ w.double().T
    close(after, want, 2e-6 * k, 1e-5, "stream after a product in parts")
    # without a stream to go into, the product stays whole and bfloat16
    assert ops.linear(x, w).shape == (rows, n)


def test_rmsnorm_reference_vector():
    """rows [1,2],[3,4], gain [1,0.5], eps 1e-6: the largest of the four outputs is index 2
    (crates/leone/src/cpu.rs:2781-2807)."""
    from leone_amd import ops
    x = torch.tensor([[1.0, 2.0], [3.0, 4.0]], device=DEV)
    y = ops.add_rmsnorm(x, None, torch.tensor([1.0, 0.5], device=DEV), 1e-6, torch.float32)
    assert int(y.flatten().argmax()) == 2
    assert int(ops.argmax(y.reshape(1, 4))[0]) == 2


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu(dtype):
    """gate in [-8, 8], up in [-2, 2], about 12,289 elements (crates/leone-cuda/tests/gpu.rs:1851-1867).  The input
    holds 8 gate values, then their 8 up values, and so on, as the fused gate/up weight orders its rows."""
    from leone_amd import ops
    torch.manual_seed(2)
    n = 12296
    gate = (torch.rand(3, n, device=DEV) * 16 - 8).to(dtype)
    up = (torch.rand(3, n, device=DEV) * 4 - 2).to(dtype)
    gu = torch.stack([gate.view(3, n // 8, 8), up.view(3, n // 8, 8)], dim=2).reshape(3, 2 * n).contiguous()
    out = ops.swiglu(gu)
    want = plain.swiglu(gate.cpu(), up.cpu())
    atol, rtol = (2e-6, 3e-6) if dtype == torch.float32 else (1e-2, 1e-2)
    close(out, want, atol, rtol, "swiglu")
    # the same order as rows of a weight: interleave_gate_up(Wg, Wu) @ x gives the layout above
    wg, wu = torch.randn(16, 5), torch.randn(16, 5)
    x = torch.randn(5)
    fused = ops.interleave_gate_up(wg, wu) @ x
    assert torch.equal(fused.view(2, 2, 8)[:, 0].reshape(-1), wg @ x) and torch.equal(fused.view(2, 2, 8)[:, 1].reshape(-1), wu @ x)


def test_rope_table():
    """positions {0, 17, 2048, 8000}, theta 1e6, D 128 within 5e-7 of double (crates/leone-cuda/tests/gpu.rs:1468-1488)."""
    from leone_amd import ops
    cos, sin = ops.rope_table(1e6, 128, 8192, DEV)
    for pos in (0, 17, 2048, 8000):
        for i in (0, 1, 31, 63):
            angle = pos * (1e6 ** (-2.0 * i / 128))
            assert abs(float(cos[pos, i]) - math.cos(angle)) < 5e-7
            assert abs(float(sin[pos, i]) - math.sin(angle)) < 5e-7
    # far positions and a small base: angles of 10^5 radians, which single precision could not reduce
    cos, sin = ops.rope_table(1e4, 48, 131072, DEV)
    for pos in (65535, 100000, 131071):
        for i in (0, 1, 7, 23):
            angle = pos * (1e4 ** (-2.0 * i / 48))
            assert abs(float(cos[pos, i]) - math.cos(angle)) < 5e-7
            assert abs(float(sin[pos, i]) - math.sin(angle)) < 5e-7


def paged_setup(lengths, kv_heads, head_dim, page_tokens, dtype, seed, extra_pages=3):
    """Random keys/values for several requests scattered over shuffled pages."""
    g = torch.Generator().manual_seed(seed)
    blocks = [(n + page_tokens - 1) // page_tokens for n in lengths]
    n_pages = sum(blocks) + extra_pages
    order = torch.randperm(n_pages, generator=g).tolist()
    max_blocks = max(blocks) + 1
    table = torch.full((len(lengths), max_blocks), -1, dtype=torch.int32)
    # plain [page][head][token][element] first, NaN where nothing lives; packed into the cache layout at the end
    k_pool = torch.full((n_pages, kv_heads, page_tokens, head_dim), float("nan"))
    v_pool = torch.full((n_pages, kv_heads, page_tokens, head_dim), float("nan"))
    keys, values = [], []
    at = 0
    for r, n in enumerate(lengths):
        k = torch.randn(n, kv_heads, head_dim, generator=g).to(dtype).float()
        v = torch.randn(n, kv_heads, head_dim, generator=g).to(dtype).float()
        keys.append(k)
        values.append(v)
        for b in range(blocks[r]):
            page = order[at]
            at += 1
            table[r, b] = page
            lo, hi = b * page_tokens, min(n, (b + 1) * page_tokens)
            k_pool[page, :, :hi - lo] = k[lo:hi].transpose(0, 1)
            v_pool[page, :, :hi - lo] = v[lo:hi].transpose(0, 1)
    from leone_amd import ops
    k_pool, v_pool = ops.pack_keys(k_pool), ops.pack_values(v_pool)
    return table, k_pool.to(dtype), v_pool.to(dtype), keys, values


@pytest.mark.parametrize("window", [0, 5, 37])
@pytest.mark.parametrize("shape", [(4, 2, 16, 16), (6, 1, 32, 64), (5, 5, 48, 16), (8, 2, 128, 32), (3, 3, 256, 16)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_rows(dtype, shape, window):
    """Rows of several requests, portions and single tokens, over scattered pages; unmapped
    slots hold NaN and must never be read (crates/leone/tests/cpu_kv_span_attention_oracle.rs:303-309)."""
    from leone_amd import ops
    q_heads, kv_heads, head_dim, page_tokens = shape
    lengths = [1, 17, 70, 130]
    table, k_pool, v_pool, keys, values = paged_setup(lengths, kv_heads, head_dim, page_tokens, dtype, seed=3)
    # request 0: its only token; request 1: last token (decode); request 2: rows 40..69 (a portion);
    # request 3: every row.
    rows = [(0, 0)] + [(1, 16)] + [(2, p) for p in range(40, 70)] + [(3, p) for p in range(130)]
    g = torch.Generator().manual_seed(4)
    q = torch.randn(len(rows), q_heads, head_dim, generator=g).to(dtype)
    positions = torch.tensor([p for _, p in rows], dtype=torch.int32)
    row_entry = torch.tensor([r for r, _ in rows], dtype=torch.int32)
    scale = 1.0 / math.sqrt(head_dim)
    out = ops.attention_rows(q.reshape(len(rows), -1).to(DEV), k_pool.to(DEV), v_pool.to(DEV), positions.to(DEV),
                             row_entry.to(DEV), table.to(DEV), q_heads, scale, window)
    assert torch.isfinite(out.float()).all()
    want = torch.empty(len(rows), q_heads, head_dim, dtype=torch.float64)
    for i, (r, p) in enumerate(rows):
        want[i] = plain.attend_one(q[i].float(), keys[r][:p + 1], values[r][:p + 1], window or None)
    atol, rtol = (3e-5, 3e-4) if dtype == torch.float32 else (2e-2, 2e-2)
    close(out.reshape(len(rows), q_heads, head_dim), want, atol, rtol, "attention")


def test_attention_reference_vector():
    """2 heads, 1 kv head, D=2, K rows [1,0],[0,1], V rows [2,4],[6,8], q [1,0] and [0,1] per token
    (crates/leone/src/cpu.rs:2850-2898)."""
    from leone_amd import ops
    # head_dim 2 there; here the heads are padded with zeros to 8, which changes no score as the scale is given
    k = torch.zeros(1, 1, 16, 8)
    v = torch.zeros(1, 1, 16, 8)
    k[0, 0, 0, :2] = torch.tensor([1.0, 0.0]); k[0, 0, 1, :2] = torch.tensor([0.0, 1.0])
    v[0, 0, 0, :2] = torch.tensor([2.0, 4.0]); v[0, 0, 1, :2] = torch.tensor([6.0, 8.0])
    q = torch.zeros(2, 2, 8)
    q[:, 0, 0] = 1.0
    q[:, 1, 1] = 1.0
    out = ops.attention_rows(q.reshape(2, 16).to(DEV), ops.pack_keys(k).to(DEV), ops.pack_values(v).to(DEV),
                             torch.tensor([0, 1], dtype=torch.int32, device=DEV),
                             torch.zeros(2, dtype=torch.int32, device=DEV),
                             torch.zeros(1, 1, dtype=torch.int32, device=DEV), 2, 1.0 / math.sqrt(2.0))
    out = out.view(2, 2, 8)[:, :, :2].reshape(2, 4)
    h = math.exp(1.0 / math.sqrt(2.0))
    want = torch.tensor([[2.0, 4.0, 2.0, 4.0],
                         [(h * 2 + 6) / (h + 1), (h * 4 + 8) / (h + 1), (2 + h * 6) / (h + 1), (4 + h * 8) / (h + 1)]])
    close(out, want, 1e-6, 1e-6, "reference vector")


@pytest.mark.parametrize("shape", [(4, 2, 16, 16), (6, 1, 32, 64), (5, 5, 48, 16), (32, 8, 128, 64)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_qk_norm_rope_write(dtype, shape):
    from leone_amd import ops
    q_heads, kv_heads, head_dim, page_tokens = shape
    torch.manual_seed(5)
    rows_meta = [(0, 3), (0, 4), (1, 16), (1, 17), (2, 8000)]  # (entry, position): page edges and a far position
    n = len(rows_meta)
    width = (q_heads + 2 * kv_heads) * head_dim
    qkv = torch.randn(n, width).to(dtype)
    q_gain = (1 + 0.1 * torch.randn(head_dim))
    k_gain = (1 + 0.1 * torch.randn(head_dim))
    eps, theta = 1e-5, 1e6
    max_blocks = 8000 // page_tokens + 1
    n_pages = 6
    table = torch.full((3, max_blocks), -1, dtype=torch.int32)
    table[0, 0] = 4
    table[1, 16 // page_tokens] = 2
    table[1, 17 // page_tokens] = 2 if 16 // page_tokens == 17 // page_tokens else 5
    table[2, 8000 // page_tokens] = 1
    k_pool = torch.full((n_pages, kv_heads, head_dim // 8, page_tokens, 8), 7.0).to(dtype)
    v_pool = torch.full((n_pages, kv_heads, page_tokens // 8, head_dim, 8), 7.0).to(dtype)

    def unpack(kp, vp):
        """Packed pools back to [page][head][token][element]."""
        return (kp.cpu().transpose(2, 3).reshape(n_pages, kv_heads, page_tokens, head_dim),
                vp.cpu().transpose(3, 4).reshape(n_pages, kv_heads, page_tokens, head_dim))
    cos, sin = ops.rope_table(theta, head_dim, 8192, DEV)
    positions = torch.tensor([p for _, p in rows_meta], dtype=torch.int32)
    row_entry = torch.tensor([e for e, _ in rows_meta], dtype=torch.int32)
    kp, vp = k_pool.to(DEV), v_pool.to(DEV)
    q_out = ops.qk_norm_rope_write(qkv.to(DEV), q_heads, kv_heads, head_dim, q_gain.to(DEV), k_gain.to(DEV), eps,
                                   cos, sin, positions.to(DEV), row_entry.to(DEV), table.to(DEV), kp, vp)
    x = qkv.float()
    q = x[:, :q_heads * head_dim].view(n, q_heads, head_dim)
    k = x[:, q_heads * head_dim:(q_heads + kv_heads) * head_dim].view(n, kv_heads, head_dim)
    v = x[:, (q_heads + kv_heads) * head_dim:].view(n, kv_heads, head_dim)
    want_q = plain.rope_half_split(plain.rms_norm(q, q_gain, eps), positions, theta)
    want_k = plain.rope_half_split(plain.rms_norm(k, k_gain, eps), positions, theta)
    atol, rtol = (5e-6, 2e-5) if dtype == torch.float32 else (2e-2, 1e-2)
    close(q_out.view(n, q_heads, head_dim), want_q, atol, rtol, "q")
    touched = torch.zeros(n_pages, page_tokens, dtype=torch.bool)
    k_plain, v_plain = unpack(kp, vp)
    for i, (e, p) in enumerate(rows_meta):
        page, off = int(table[e, p // page_tokens]), p % page_tokens
        touched[page, off] = True
        close(k_plain[page, :, off], want_k[i], atol, rtol, f"k row {i}")
        assert torch.equal(v_plain[page, :, off], v[i].to(dtype))          # values are copied unchanged
    # every other slot is untouched
    untouched = ~touched[:, None, :].expand(-1, kv_heads, -1)
    assert (k_plain[untouched] == 7.0).all() and (v_plain[untouched] == 7.0).all()
    # a layer that reads another layer's cache writes nothing
    kp2, vp2 = k_pool.to(DEV), v_pool.to(DEV)
    q2 = ops.qk_norm_rope_write(qkv.to(DEV), q_heads, kv_heads, head_dim, q_gain.to(DEV), k_gain.to(DEV), eps, cos,
                                sin, positions.to(DEV), row_entry.to(DEV), table.to(DEV), kp2, vp2, write_cache=False)
    assert torch.equal(q2, q_out) and torch.equal(kp2.cpu(), k_pool) and torch.equal(vp2.cpu(), v_pool)
    # no norm and no rotation: the heads come through as they are
    q3 = ops.qk_norm_rope_write(qkv.to(DEV), q_heads, kv_heads, head_dim, None, None, eps, None, None,
                                positions.to(DEV), row_entry.to(DEV), table.to(DEV), kp2, vp2)
    assert torch.equal(q3.cpu().view(n, q_heads, head_dim), q.to(dtype))
    # float32 input in planes (a product cut along K): the planes are added up in order, then the same work
    if dtype == torch.bfloat16:
        parts = torch.randn(3, n, width) * torch.tensor([1.0, 0.01, 1e-4]).view(3, 1, 1)
        total = (parts[0] + parts[1]) + parts[2]
        kp3, vp3 = k_pool.to(DEV), v_pool.to(DEV)
        q4 = ops.qk_norm_rope_write(parts.to(DEV), q_heads, kv_heads, head_dim, q_gain.to(DEV), k_gain.to(DEV), eps,
                                    cos, sin, positions.to(DEV), row_entry.to(DEV), table.to(DEV), kp3, vp3,
                                    out_dtype=dtype)
        tq = total[:, :q_heads * head_dim].view(n, q_heads, head_dim)
        tk = total[:, q_heads * head_dim:(q_heads + kv_heads) * head_dim].view(n, kv_heads, head_dim)
        tv = total[:, (q_heads + kv_heads) * head_dim:].view(n, kv_heads, head_dim)
        close(q4.view(n, q_heads, head_dim), plain.rope_half_split(plain.rms_norm(tq, q_gain, eps), positions, theta),
              atol, rtol, "q from planes")
        k4, v4 = unpack(kp3, vp3)
        for i, (e, p) in enumerate(rows_meta):
            page, off = int(table[e, p // page_tokens]), p % page_tokens
            close(k4[page, :, off], plain.rope_half_split(plain.rms_norm(tk, k_gain, eps), positions, theta)[i],
                  atol, rtol, f"k row {i} from planes")
            assert torch.equal(v4[page, :, off], tv[i].to(dtype))
        assert (k4[untouched] == 7.0).all() and (v4[untouched] == 7.0).all()


@pytest.mark.parametrize("shape", [(4, 2, 16, 16), (5, 5, 48, 16), (3, 1, 112, 32), (8, 2, 128, 64)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_qk_norm_rope_write_many_rows(dtype, shape):
    """Enough rows for the values to go through the kernel that writes whole runs: a portion whose rows do not
    line up with runs of eight tokens, one that does, and page edges inside both."""
    from leone_amd import ops
    q_heads, kv_heads, head_dim, page_tokens = shape
    torch.manual_seed(6)
    portions = [(0, 5, 70), (1, 16, 34), (2, 64, 48)]               # (entry, first position, rows); the third lines up
    rows_meta = [(e, start + i) for e, start, count in portions for i in range(count)]
    n = len(rows_meta)
    assert n >= 64 and sum(c for _, _, c in portions[:2]) % 8 == 0
    qkv = torch.randn(n, (q_heads + 2 * kv_heads) * head_dim).to(dtype)
    q_gain, k_gain = 1 + 0.1 * torch.randn(head_dim), 1 + 0.1 * torch.randn(head_dim)
    eps, theta = 1e-5, 1e4
    max_blocks = 128 // page_tokens
    n_pages = 3 * max_blocks + 1
    order = torch.randperm(n_pages - 1)[:3 * max_blocks].view(3, max_blocks).int() + 1     # page 0 stays unused
    k_pool = torch.full((n_pages, kv_heads, head_dim // 8, page_tokens, 8), 7.0).to(dtype)
    v_pool = torch.full((n_pages, kv_heads, page_tokens // 8, head_dim, 8), 7.0).to(dtype)
    cos, sin = ops.rope_table(theta, head_dim, 256, DEV)
    positions = torch.tensor([p for _, p in rows_meta], dtype=torch.int32)
    row_entry = torch.tensor([e for e, _ in rows_meta], dtype=torch.int32)
    kp, vp = k_pool.to(DEV), v_pool.to(DEV)
    q_out = ops.qk_norm_rope_write(qkv.to(DEV), q_heads, kv_heads, head_dim, q_gain.to(DEV), k_gain.to(DEV), eps,
                                   cos, sin, positions.to(DEV), row_entry.to(DEV), order.to(DEV), kp, vp)
    x = qkv.float()
    q = x[:, :q_heads * head_dim].view(n, q_heads, head_dim)
    k = x[:, q_heads * head_dim:(q_heads + kv_heads) * head_dim].view(n, kv_heads, head_dim)
    v = x[:, (q_heads + kv_heads) * head_dim:].view(n, kv_heads, head_dim)
    atol, rtol = (5e-6, 2e-5) if dtype == torch.float32 else (2e-2, 1e-2)
    close(q_out.view(n, q_heads, head_dim), plain.rope_half_split(plain.rms_norm(q, q_gain, eps), positions, theta),
          atol, rtol, "q")
    want_k = plain.rope_half_split(plain.rms_norm(k, k_gain, eps), positions, theta)
    k_plain = kp.cpu().transpose(2, 3).reshape(n_pages, kv_heads, page_tokens, head_dim)
    v_plain = vp.cpu().transpose(3, 4).reshape(n_pages, kv_heads, page_tokens, head_dim)
    touched = torch.zeros(n_pages, page_tokens, dtype=torch.bool)
    for i, (e, p) in enumerate(rows_meta):
        page, off = int(order[e, p // page_tokens]), p % page_tokens
        touched[page, off] = True
        close(k_plain[page, :, off], want_k[i], atol, rtol, f"k row {i}")
        assert torch.equal(v_plain[page, :, off], v[i].to(dtype)), (i, e, p)
    untouched = ~touched[:, None, :].expand(-1, kv_heads, -1)
    assert (k_plain[untouched] == 7.0).all() and (v_plain[untouched] == 7.0).all()


@pytest.mark.parametrize("pairing", ["half_split", "adjacent"])
@pytest.mark.parametrize("shape", [(4, 2, 32, 16, 16), (3, 1, 64, 32, 16), (5, 5, 48, 24, 16), (8, 2, 128, 64, 64),
                                   (2, 2, 128, 128, 64), (3, 3, 24, 8, 16)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_qk_norm_rope_write_with_the_rotation_shape_as_parameters(dtype, shape, pairing):
    """The position encoding owns the rotation's shape: ``rotary_dim`` of the head's elements (here half, a
    third or all of them) in half-split or adjacent pairs; the rest is normalised and left unrotated.  Against
    the plain implementation and, in float32, the scalar reference of the entry point."""
    from leone_amd import ops
    from tests import scalar
    q_heads, kv_heads, head_dim, rotary_dim, page_tokens = shape
    torch.manual_seed(8)
    rows_meta = [(0, 0), (0, 1), (1, 15), (1, 16), (2, 700)]
    n = len(rows_meta)
    qkv = torch.randn(n, (q_heads + 2 * kv_heads) * head_dim).to(dtype)
    q_gain, k_gain = 1 + 0.1 * torch.randn(head_dim), 1 + 0.1 * torch.randn(head_dim)
    eps, theta = 1e-5, 1e4
    max_blocks = 700 // page_tokens + 1
    table = torch.full((3, max_blocks), -1, dtype=torch.int32)
    table[0, 0], table[1, 0], table[1, 16 // page_tokens], table[2, 700 // page_tokens] = 4, 2, 2 if page_tokens > 16 else 5, 1
    n_pages = 6
    kp = torch.zeros((n_pages, kv_heads, head_dim // 8, page_tokens, 8), dtype=dtype, device=DEV)
    vp = torch.zeros((n_pages, kv_heads, page_tokens // 8, head_dim, 8), dtype=dtype, device=DEV)
    cos, sin = ops.rope_table(theta, rotary_dim, 1024, DEV)
    assert cos.shape == (1024, rotary_dim // 2)
    positions = torch.tensor([p for _, p in rows_meta], dtype=torch.int32)
    row_entry = torch.tensor([e for e, _ in rows_meta], dtype=torch.int32)
    q_out = ops.qk_norm_rope_write(qkv.to(DEV), q_heads, kv_heads, head_dim, q_gain.to(DEV), k_gain.to(DEV), eps,
                                   cos, sin, positions.to(DEV), row_entry.to(DEV), table.to(DEV), kp, vp, pairing=pairing)
    x = qkv.float()
    q = x[:, :q_heads * head_dim].view(n, q_heads, head_dim)
    k = x[:, q_heads * head_dim:(q_heads + kv_heads) * head_dim].view(n, kv_heads, head_dim)
    want_q = plain.rope_pairs(plain.rms_norm(q, q_gain, eps), positions, theta, rotary_dim, pairing)
    want_k = plain.rope_pairs(plain.rms_norm(k, k_gain, eps), positions, theta, rotary_dim, pairing)
    atol, rtol = (5e-6, 2e-5) if dtype == torch.float32 else (2e-2, 1e-2)
    close(q_out.view(n, q_heads, head_dim), want_q, atol, rtol, "q")
    k_plain = kp.cpu().transpose(2, 3).reshape(n_pages, kv_heads, page_tokens, head_dim)
    for i, (e, p) in enumerate(rows_meta):
        close(k_plain[int(table[e, p // page_tokens]), :, p % page_tokens], want_k[i], atol, rtol, f"k row {i}")
    if rotary_dim < head_dim or pairing == "adjacent":
        # the other shape would be far off: the test can tell them apart
        other = plain.rope_pairs(plain.rms_norm(q, q_gain, eps), positions, theta, head_dim, "half_split")
        assert (other - want_q).abs().max() > 0.1
    if dtype == torch.float32:
        k_ref = np.zeros(tuple(kp.shape), dtype=np.float32)
        v_ref = np.zeros(tuple(vp.shape), dtype=np.float32)
        q_ref = scalar.qk_norm_rope_write(qkv.numpy(), q_heads, kv_heads, head_dim, q_gain.numpy(), k_gain.numpy(), eps,
                                          cos.cpu().numpy(), sin.cpu().numpy(), positions.numpy(), row_entry.numpy(),
                                          table.numpy(), k_ref, v_ref, pairing=ops.PAIRINGS[pairing])
        assert np.abs(q_ref - q_out.cpu().numpy()).max() < 2e-5
        assert np.abs(k_ref - kp.cpu().numpy()).max() < 2e-5 and np.array_equal(v_ref, vp.cpu().numpy())


def test_kernels_refuse_rotations_they_are_not_built_for():
    """The decode kernel that takes the projection itself rotates whole heads in half-split pairs; given another
    shape it says so instead of rotating wrongly, and tables wider than the head are refused everywhere."""
    from leone_amd import ops
    from leone_amd.ops import KernelError
    q_heads, kv_heads, head_dim, page = 4, 1, 64, 16
    qkv = torch.randn(2, (q_heads + 2 * kv_heads) * head_dim, device=DEV).bfloat16()
    kp = torch.zeros((2, kv_heads, head_dim // 8, page, 8), dtype=torch.bfloat16, device=DEV)
    vp = torch.zeros((2, kv_heads, page // 8, head_dim, 8), dtype=torch.bfloat16, device=DEV)
    positions = torch.tensor([3, 5], dtype=torch.int32, device=DEV)
    rows = torch.tensor([0, 1], dtype=torch.int32, device=DEV)
    table = torch.tensor([[0], [1]], dtype=torch.int32, device=DEV)
    half_cos, half_sin = ops.rope_table(1e4, head_dim // 2, 32, DEV)
    full_cos, full_sin = ops.rope_table(1e4, head_dim, 32, DEV)
    wide_cos, wide_sin = ops.rope_table(1e4, 2 * head_dim, 32, DEV)
    assert ops.decode_projected_supported(head_dim, head_dim) and not ops.decode_projected_supported(head_dim, head_dim // 2)
    assert not ops.decode_projected_supported(head_dim, head_dim, "adjacent") and ops.decode_projected_supported(head_dim, 0)
    for cos, sin, pairing, word in ((half_cos, half_sin, "half_split", "whole heads"), (full_cos, full_sin, "adjacent", "whole heads"),
                                    (wide_cos, wide_sin, "half_split", "a head has"), (full_cos, full_sin, "spiral", "unknown pairing")):
        with pytest.raises(KernelError, match=word):
            ops.attention_decode_projected(qkv, q_heads, kv_heads, head_dim, None, None, 1e-6, cos, sin, kp, vp, positions,
                                           rows, table, 0.125, pairing=pairing)
    with pytest.raises(KernelError, match="a head has"):
        ops.qk_norm_rope_write(qkv, q_heads, kv_heads, head_dim, None, None, 1e-6, wide_cos, wide_sin, positions, rows, table, kp, vp)
    assert float(kp.abs().max()) == 0.0 and float(vp.abs().max()) == 0.0          # a refused call wrote nothing


@pytest.mark.parametrize("mnk", [(1, 777, 80), (5, 64, 64), (130, 192, 96), (67, 1000, 333), (300, 130, 1029)])
def test_gemm_f32(mnk):
    from leone_amd import ops
    m, n, k = mnk
    torch.manual_seed(6)
    a, b = torch.randn(m, k, device=DEV), torch.randn(n, k, device=DEV)
    out = ops.gemm_f32(a, b)
    want = a.double() @ b.double().T
    close(out, want, 1e-5 * math.sqrt(k), 1e-5, "gemm_f32")


def test_argmax_rules():
    """[1, 4, 4, NaN] -> 1; no finite value -> -1 (crates/leone/src/sampler/tests.rs:521-537)."""
    from leone_amd import ops
    nan, inf = float("nan"), float("inf")
    rows = torch.tensor([[1.0, 4.0, 4.0, nan], [nan, -inf, inf, nan], [inf, -5.0, nan, -7.0], [0.0, 0.0, 0.0, 0.0]],
                        device=DEV)
    assert ops.argmax(rows).tolist() == [1, -1, 1, 0]
    torch.manual_seed(7)
    big = torch.randn(5, 151936, device=DEV)
    big[2, 1000] = big[2, 150000] = 9.0
    assert ops.argmax(big).tolist() == [int(r.argmax()) if i != 2 else 1000 for i, r in enumerate(big)]


@pytest.mark.parametrize("splits", [1, 3, None])
@pytest.mark.parametrize("window", [0, 5, 37])
@pytest.mark.parametrize("shape", [(4, 2, 16, 16), (6, 1, 32, 64), (5, 5, 48, 16), (32, 8, 128, 64), (40, 8, 128, 16),
                                   (64, 2, 64, 32), (3, 3, 256, 16), (34, 2, 240, 16)])
def test_attention_decode(shape, window, splits):
    """The matrix-core kernel on the same cases as the row kernel, whatever the number of splits."""
    from leone_amd import ops
    q_heads, kv_heads, head_dim, page_tokens = shape
    dtype = torch.bfloat16
    assert ops.decode_attention_supported(dtype, head_dim, page_tokens, q_heads // kv_heads)
    lengths = [1, 17, 70, 130]
    table, k_pool, v_pool, keys, values = paged_setup(lengths, kv_heads, head_dim, page_tokens, dtype, seed=13)
    rows = [(0, 0)] + [(1, 16)] + [(2, p) for p in range(40, 70)] + [(3, p) for p in range(0, 130, 3)] + [(3, 129)]
    g = torch.Generator().manual_seed(14)
    q = torch.randn(len(rows), q_heads, head_dim, generator=g).to(dtype)
    positions = torch.tensor([p for _, p in rows], dtype=torch.int32)
    row_entry = torch.tensor([r for r, _ in rows], dtype=torch.int32)
    scale = 1.0 / math.sqrt(head_dim)
    args = (q.reshape(len(rows), -1).to(DEV), k_pool.to(DEV), v_pool.to(DEV), positions.to(DEV), row_entry.to(DEV),
            table.to(DEV), q_heads, scale, window)
    out = ops.attention_decode(*args, max_context=130, splits=splits)
    assert torch.isfinite(out.float()).all()
    want = torch.stack([plain.attend_one(q[i].float(), keys[r][:p + 1], values[r][:p + 1], window or None)
                        for i, (r, p) in enumerate(rows)])
    close(out.reshape(len(rows), q_heads, head_dim), want, 2e-2, 2e-2, "attention_decode")
    again = ops.attention_decode(*args, max_context=130, splits=splits)
    assert torch.equal(out, again)                                   # fixed order of additions


@pytest.mark.parametrize("kernel", ["rows", "decode"])
def test_attention_finds_the_one_key_that_matters(kernel):
    """Each query is a scaled copy of one key far back in its request, so that key takes all the weight
    and the output must be its value row: a key taken from the wrong page, slot or request shows at once,
    well above bfloat16 rounding."""
    from leone_amd import ops
    q_heads, kv_heads, head_dim, page_tokens = 8, 2, 64, 16
    dtype = torch.bfloat16
    lengths = [300, 517]
    table, k_pool, v_pool, keys, values = paged_setup(lengths, kv_heads, head_dim, page_tokens, dtype, seed=21)
    picks = [(0, 299, 0), (0, 299, 15), (0, 299, 16), (0, 255, 31), (0, 200, 199), (1, 516, 1), (1, 516, 255),
             (1, 516, 256), (1, 516, 511), (1, 516, 512), (1, 400, 47), (1, 64, 63), (1, 64, 64)]
    q = torch.zeros(len(picks), q_heads, head_dim)
    for i, (r, p, j) in enumerate(picks):
        for h in range(q_heads):
            k = keys[r][j, h // (q_heads // kv_heads)]
            q[i, h] = k * (60.0 * math.sqrt(head_dim) / float(k @ k))     # its own score is 60, others ~N(0, 60/8)
    q = q.to(dtype)
    positions = torch.tensor([p for _, p, _ in picks], dtype=torch.int32)
    row_entry = torch.tensor([r for r, _, _ in picks], dtype=torch.int32)
    args = (q.reshape(len(picks), -1).to(DEV), k_pool.to(DEV), v_pool.to(DEV), positions.to(DEV), row_entry.to(DEV),
            table.to(DEV), q_heads, 1.0 / math.sqrt(head_dim))
    out = (ops.attention_rows(*args) if kernel == "rows" else ops.attention_decode(*args, max_context=517))
    out = out.float().cpu().view(len(picks), q_heads, head_dim)
    for i, (r, p, j) in enumerate(picks):
        want = values[r][j].repeat_interleave(q_heads // kv_heads, dim=0)
        exact = plain.attend_one(q[i].float(), keys[r][:p + 1], values[r][:p + 1])
        assert (out[i] - exact).abs().max() < 3e-2, (i, r, p, j)
        assert (out[i] - want).abs().max() < 0.25, (i, r, p, j)       # nearly all the weight is on key j


@pytest.mark.parametrize("kernel", ["rows", "decode", "prefill"])
def test_attention_finds_one_key_among_seventy_thousand(kernel):
    """The same far into a long request: more than a thousand pages, key ranges in both kernels, targets at
    the edges of pages, of 4,096 and of 65,536 keys."""
    from leone_amd import ops
    q_heads, kv_heads, head_dim, page_tokens = 8, 2, 64, 64
    dtype = torch.bfloat16
    n = 70_000
    table, k_pool, v_pool, keys, values = paged_setup([n], kv_heads, head_dim, page_tokens, dtype, seed=61)
    edges = [0, 63, 64, 4095, 4096, 32767, 32768, 65535, 65536, 69839]
    count = 160 if kernel == "prefill" else 24
    first = n - count if kernel == "prefill" else n - 1
    g = torch.Generator().manual_seed(62)
    targets = [edges[i] if i < len(edges) else int(torch.randint(0, n - count, (1,), generator=g)) for i in range(count)]
    positions = [first + i if kernel == "prefill" else n - 1 for i in range(count)]
    targets[-1] = positions[-1]                                   # the last row looks at itself
    q = torch.zeros(count, q_heads, head_dim)
    for i, j in enumerate(targets):
        for h in range(q_heads):
            k = keys[0][j, h // (q_heads // kv_heads)]
            q[i, h] = k * (60.0 * math.sqrt(head_dim) / float(k @ k))
    q = q.to(dtype).reshape(count, -1).to(DEV)
    where = torch.tensor(positions, dtype=torch.int32, device=DEV)
    scale = 1.0 / math.sqrt(head_dim)
    if kernel == "prefill":
        out = torch.zeros((count, q_heads * head_dim), dtype=dtype, device=DEV)
        tiles = ops.prefill_tiles([(0, 0, count)])
        assert ops.choose_prefill_splits(tiles.shape[0] // ops.PREFILL_GROUP_TILES, q_heads, n) > 1
        ops.attention_prefill(q, out, k_pool.to(DEV), v_pool.to(DEV), where, tiles.to(DEV), table.to(DEV), q_heads, scale,
                              mean_keys=n)
    elif kernel == "decode":
        out = ops.attention_decode(q, k_pool.to(DEV), v_pool.to(DEV), where, torch.zeros(count, dtype=torch.int32, device=DEV),
                                   table.to(DEV), q_heads, scale, max_context=n)
    else:
        out = ops.attention_rows(q, k_pool.to(DEV), v_pool.to(DEV), where, torch.zeros(count, dtype=torch.int32, device=DEV),
                                 table.to(DEV), q_heads, scale)
    out = out.float().cpu().view(count, q_heads, head_dim)
    for i, j in enumerate(targets):
        want = values[0][j].repeat_interleave(q_heads // kv_heads, dim=0)
        assert (out[i] - want).abs().max() < 0.25, (i, positions[i], j)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mnk", [(1, 777, 80), (5, 64, 64), (8, 6144, 4096), (16, 1000, 96), (13, 130, 1032),
                                 (9, 48, 176), (16, 4096, 12288), (1, 151936, 256), (3, 20, 8)])
def test_gemm_fused_plain(mnk, out_dtype):
    """The weight-streaming product with nothing folded in.  Inputs rounded to bfloat16 as the kernel sees
    them, products summed in double (the reference's way for its matrix-core product,
    crates/leone-cuda/tests/gpu.rs:287-386)."""
    from leone_amd import ops
    m, n, k = mnk
    torch.manual_seed(8)
    x, w = torch.randn(m, k, device=DEV).bfloat16(), (torch.randn(n, k, device=DEV) * 0.05).bfloat16()
    out = ops.gemm_fused(x, w, out_dtype)
    want = x.double() @ w.double().T
    if out_dtype == torch.float32:
        close(out, want, 2e-6 * k, 1e-5, "gemm_fused")
    else:
        close(out, want, 2e-6 * k + 1e-3, 8e-3, "gemm_fused bf16")
    assert torch.equal(out, ops.gemm_fused(x, w, out_dtype))
    # a row alone gives the same bits as the row inside a batch (crates/leone-cuda/tests/gpu.rs:770)
    assert torch.equal(ops.gemm_fused(x[m - 1:m].contiguous(), w, out_dtype)[0], out[m - 1])


@pytest.mark.parametrize("splits", [1, 2, 5, 32])
@pytest.mark.parametrize("window", [0, 5, 37])
@pytest.mark.parametrize("shape", [(4, 2, 16, 16), (6, 1, 32, 64), (5, 5, 48, 16), (32, 8, 128, 64), (3, 3, 112, 32)])
def test_attention_prefill(shape, window, splits):
    """Portions that start at position 0 and in the middle of a request, longer and shorter than a
    128-row tile, over scattered pages; rows of the step that belong to no tile stay untouched.  The keys
    of a workgroup in one range or cut into several, down to ranges of one 64-key stage and empty ones."""
    from leone_amd import ops
    q_heads, kv_heads, head_dim, page_tokens = shape
    dtype = torch.bfloat16
    assert ops.prefill_attention_supported(dtype, head_dim, page_tokens)
    lengths = [300, 77, 200]
    table, k_pool, v_pool, keys, values = paged_setup(lengths, kv_heads, head_dim, page_tokens, dtype, seed=31)
    portions = [(0, 0, 300), (1, 60, 17), (2, 33, 130)]            # (request, first position, rows)
    rows, listed = [], []
    for entry, (r, start, count) in enumerate(portions):
        listed.append((entry, len(rows), count))
        rows += [(r, start + i) for i in range(count)]
    rows += [(1, 76)]                                               # a row outside every tile
    tiles = ops.prefill_tiles(listed)
    g = torch.Generator().manual_seed(32)
    q = torch.randn(len(rows), q_heads, head_dim, generator=g).to(dtype)
    positions = torch.tensor([p for _, p in rows], dtype=torch.int32)
    scale = 1.0 / math.sqrt(head_dim)
    out = torch.full((len(rows), q_heads * head_dim), 5.0, dtype=dtype, device=DEV)
    ops.attention_prefill(q.reshape(len(rows), -1).to(DEV), out, k_pool.to(DEV), v_pool.to(DEV), positions.to(DEV),
                          tiles.to(DEV), table.to(DEV), q_heads, scale, window, splits=splits)
    assert torch.isfinite(out.float()).all()
    assert (out[-1] == 5.0).all()
    want = torch.stack([plain.attend_one(q[i].float(), keys[r][:p + 1], values[r][:p + 1], window or None)
                        for i, (r, p) in enumerate(rows[:-1])])
    close(out[:-1].reshape(len(rows) - 1, q_heads, head_dim), want, 2e-2, 2e-2, "attention_prefill")


@pytest.mark.parametrize("portions", [[(0, 0, 200)], [(0, 0, 40), (1, 10, 20), (2, 0, 100), (3, 5, 16)],
                                      [(0, 0, 500)], [(0, 3, 900)], [(0, 0, 130), (1, 0, 385)]],
                         ids=["2groups", "4groups", "4groups-one", "8groups", "6groups"])
@pytest.mark.parametrize("shape", [(4, 2, 16, 16), (6, 1, 32, 64), (12, 4, 64, 16), (20, 4, 32, 32), (32, 8, 128, 64),
                                   (2, 1, 16, 16), (8, 8, 48, 16)])
def test_attention_prefill_every_head_of_every_group(shape, portions):
    """Head counts that are no multiple of eight with 2, 4, 6 and 8 tile groups in one launch: every
    (head, group) pair must be computed (a numbering of workgroups by dies once left some out).  The
    output starts as NaN, so a pair that nobody takes shows."""
    from leone_amd import ops
    q_heads, kv_heads, head_dim, page_tokens = shape
    dtype = torch.bfloat16
    lengths = {}
    for r, start, count in portions:
        lengths[r] = max(lengths.get(r, 0), start + count)
    table, k_pool, v_pool, keys, values = paged_setup([lengths[r] for r in sorted(lengths)], kv_heads, head_dim,
                                                      page_tokens, dtype, seed=71)
    rows, listed = [], []
    for entry, (r, start, count) in enumerate(portions):
        listed.append((entry, len(rows), count))
        rows += [(r, start + i) for i in range(count)]
    tiles = ops.prefill_tiles(listed)
    # an entry's block table is its request's
    entry_table = table[[r for r, _, _ in portions]].contiguous()
    g = torch.Generator().manual_seed(72)
    q = torch.randn(len(rows), q_heads, head_dim, generator=g).to(dtype)
    positions = torch.tensor([p for _, p in rows], dtype=torch.int32)
    out = torch.full((len(rows), q_heads * head_dim), float("nan"), dtype=dtype, device=DEV)
    ops.attention_prefill(q.reshape(len(rows), -1).to(DEV), out, k_pool.to(DEV), v_pool.to(DEV), positions.to(DEV),
                          tiles.to(DEV), entry_table.to(DEV), q_heads, 1.0 / math.sqrt(head_dim), splits=1)
    assert torch.isfinite(out.float()).all(), "some (head, group) pair was not computed"
    picked = list(range(0, len(rows), 7)) + [len(rows) - 1]
    want = torch.stack([plain.attend_one(q[i].float(), keys[rows[i][0]][:rows[i][1] + 1], values[rows[i][0]][:rows[i][1] + 1], None)
                        for i in picked])
    close(out[picked].reshape(len(picked), q_heads, head_dim), want, 2e-2, 2e-2, "attention_prefill")


@pytest.mark.parametrize("splits", [1, 3])
@pytest.mark.parametrize("dealt", [False, True])
def test_attention_prefill_finds_the_one_key_that_matters(dealt, splits):
    """``dealt``: the tiles of the portion stand in another order, first and last tiles together in a group;
    the kernel takes the tiles of a group as they come."""
    from leone_amd import ops
    q_heads, kv_heads, head_dim, page_tokens = 4, 2, 64, 16
    dtype = torch.bfloat16
    lengths = [400]
    table, k_pool, v_pool, keys, values = paged_setup(lengths, kv_heads, head_dim, page_tokens, dtype, seed=41)
    start, count = 100, 300
    rows = [(0, start + i) for i in range(count)]
    g = torch.Generator().manual_seed(42)
    targets = [int(torch.randint(0, p + 1, (1,), generator=g)) for _, p in rows]     # any key up to its own position
    for i in (0, 31, 32, 63, 64, 299):                                              # tile edges look at themselves
        targets[i] = rows[i][1]
    for i in (5, 64, 200):                                                            # and at the very first key
        targets[i] = 0
    q = torch.zeros(count, q_heads, head_dim)
    for i, j in enumerate(targets):
        for h in range(q_heads):
            k = keys[0][j, h // 2]
            q[i, h] = k * (60.0 * math.sqrt(head_dim) / float(k @ k))
    q = q.to(dtype)
    tiles = ops.prefill_tiles([(0, 0, count)])
    if dealt:
        own = [tuple(t) for t in tiles.tolist() if t[2] > 0]
        assert len(own) == 10
        order = [0, 9, 1, 8, 7, 2, 3, 6, 5, 4]
        tiles = torch.tensor([own[i] for i in order] + [(0, 0, 0)] * 2, dtype=torch.int32)
    out = torch.zeros((count, q_heads * head_dim), dtype=dtype, device=DEV)
    ops.attention_prefill(q.reshape(count, -1).to(DEV), out, k_pool.to(DEV), v_pool.to(DEV),
                          torch.tensor([p for _, p in rows], dtype=torch.int32, device=DEV),
                          tiles.to(DEV), table.to(DEV), q_heads, 1.0 / math.sqrt(head_dim), splits=splits)
    out = out.float().cpu().view(count, q_heads, head_dim)
    for i, j in enumerate(targets):
        want = values[0][j].repeat_interleave(2, dim=0)
        assert (out[i] - want).abs().max() < 0.25, (i, rows[i][1], j)


@pytest.mark.parametrize("gain_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mnk", [(1, 6144, 4096), (5, 777, 80), (16, 1000, 176), (8, 96, 1032), (3, 4096, 12288)])
def test_gemm_fused_norm_and_store(mnk, gain_dtype):
    """The norm folded into the product equals norm, then product: the row factor 1/rms commutes with the sum."""
    from leone_amd import ops
    m, n, k = mnk
    torch.manual_seed(9)
    stream = torch.randn(m + 3, k, device=DEV) * 2
    gain = (1 + 0.1 * torch.randn(k, device=DEV)).to(gain_dtype)
    w = (torch.randn(n, k, device=DEV) * 0.05).bfloat16()
    eps = 1e-5
    rows = torch.tensor([(3 * i + 1) % (m + 3) for i in range(m)], dtype=torch.int32, device=DEV)
    for picked in (None, rows):
        x = stream[:m] if picked is None else stream
        lazy = ops.NormedRows(x.contiguous(), gain, eps, torch.bfloat16, picked)
        out = ops.gemm_fused(lazy, w, torch.float32)
        src = x[:m] if picked is None else x[picked.long()]
        # the kernel's operand is bf16(x * gain); its rounding is the only difference from double
        operand = (src * gain.float()).bfloat16().double()
        inv = 1.0 / torch.sqrt((src.double() ** 2).mean(dim=1, keepdim=True) + eps)
        want = (operand @ w.double().T) * inv
        close(out, want, 2e-6 * k, 2e-5, "norm + product")
        assert torch.equal(out, ops.gemm_fused(lazy, w, torch.float32))
        # and it agrees with the unfused pair within bfloat16 rounding of the normalised rows
        unfused = ops.gemm_fused(lazy.materialize(), w, torch.float32)
        close(out, unfused.double(), 2e-2 * math.sqrt(k) * 0.05 * 3, 2e-2, "fused against unfused")


@pytest.mark.parametrize("mnk", [(1, 4096, 4096), (7, 80, 176), (16, 777, 64)])
def test_gemm_fused_residual(mnk):
    from leone_amd import ops
    m, n, k = mnk
    torch.manual_seed(10)
    x = torch.randn(m, k, device=DEV).bfloat16()
    w = (torch.randn(n, k, device=DEV) * 0.05).bfloat16()
    stream = torch.randn(m, n, device=DEV)
    before = stream.clone()
    assert ops.gemm_fused(x, w, residual=stream) is None
    want = before.double() + x.double() @ w.double().T
    close(stream, want, 2e-6 * k, 1e-5, "product added into the stream")
    # the same bits as product, then one float addition (crates/leone-cuda/tests/gpu.rs:1921)
    assert torch.equal(stream, before + ops.gemm_fused(x, w, torch.float32))


@pytest.mark.parametrize("mfk", [(1, 12288, 4096), (6, 88, 80), (16, 256, 96)])
def test_gemm_fused_gated(mfk):
    from leone_amd import ops
    m, f, k = mfk
    torch.manual_seed(11)
    stream = torch.randn(m, k, device=DEV)
    gain = 1 + 0.1 * torch.randn(k, device=DEV)
    wg, wu = (torch.randn(f, k, device=DEV) * 0.1).bfloat16(), (torch.randn(f, k, device=DEV) * 0.1).bfloat16()
    w = ops.interleave_gate_up(wg, wu).contiguous()
    lazy = ops.NormedRows(stream, gain, 1e-6, torch.bfloat16)
    out = ops.gemm_fused(lazy, w, gated=True)
    assert out.shape == (m, f) and out.dtype == torch.bfloat16
    operand = (stream * gain).bfloat16().double()
    inv = 1.0 / torch.sqrt((stream.double() ** 2).mean(dim=1, keepdim=True) + 1e-6)
    want = plain.swiglu((operand @ wg.double().T) * inv, (operand @ wu.double().T) * inv)
    close(out, want, 1e-2, 1e-2, "gated product")
    # through linear(): the same call falls back to product + swiglu kernel beyond ops.FUSED_ROWS rows
    many = torch.randn(40, k, device=DEV)
    lazy40 = ops.NormedRows(many, gain, 1e-6, torch.bfloat16)
    got = ops.linear(lazy40, w, gated=True)
    y = lazy40.materialize().double().cpu()
    close(got, plain.swiglu(y @ wg.double().cpu().T, y @ wu.double().cpu().T), 3e-2, 3e-2, "unfused gated")


ROWS_SHAPES = [(16, 6144, 4096), (17, 777, 264), (33, 130, 1032), (64, 4096, 4096), (100, 1000, 96), (128, 4096, 12288),
               (48, 24576, 4096), (11, 20, 8), (128, 333, 72), (96, 151936, 4096), (1, 4096, 4096)]


@pytest.mark.parametrize("mnk", ROWS_SHAPES)
def test_gemm_rows_plain(mnk):
    """The multi-row weight-streaming product (crates/leone/src/runtime.rs:7865-7906 is the reference's place
    for it) against double sums of the bfloat16 inputs (crates/leone-cuda/tests/gpu.rs:287-386), for every
    workgroup size and several cuts of K, and as the plan would run it."""
    from leone_amd import ops
    m, n, k = mnk
    torch.manual_seed(21)
    x, w = torch.randn(m, k, device=DEV).bfloat16(), (torch.randn(n, k, device=DEV) * 0.05).bfloat16()
    want = x.double() @ w.double().T
    big = n * k > 1 << 27
    from leone_amd.ops.library import library
    shared = 0
    for waves in ((6,) if big else ops.ROWS_WAVES):
        for ways in (1, 2):                       # waves that share a tile of the weight: built for more than 64 rows
            if not library().leone_gemm_rows_shape_built(m, waves, ways):
                continue
            shared += ways > 1
            for splits in ((1,) if big else (1, 2, 5)):
                out = ops.gemm_rows(x, w, torch.float32, splits=splits, waves=waves, ways=ways)
                if out.dim() == 3:
                    assert out.shape[1:] == (m, n)
                    out = out.double().sum(0)
                close(out, want, 2e-6 * k, 1e-5, f"gemm_rows waves {waves} ways {ways} splits {splits}")
    assert (shared > 0) == (m > 64)
    planned = ops.gemm_rows(x, w, torch.float32)
    assert torch.equal(planned, ops.gemm_rows(x, w, torch.float32))            # a launch repeats bit for bit
    close(planned.double().sum(0) if planned.dim() == 3 else planned, want, 2e-6 * k, 1e-5, "gemm_rows as planned")
    rounded = ops.gemm_rows(x, w, torch.bfloat16, may_split=False)
    assert rounded.shape == (m, n) and rounded.dtype == torch.bfloat16
    close(rounded, want, 2e-6 * k + 1e-3, 8e-3, "gemm_rows bf16")
    # a row gives the same bits whatever the other rows are (crates/leone-cuda/tests/gpu.rs:770)
    waves, splits = ops.rows_plan(m, n, k, False)
    whole = ops.gemm_rows(x, w, torch.float32, splits=1, waves=waves)
    other = x.clone()
    other[:m - 1] = torch.randn(m - 1, k, device=DEV).bfloat16()
    assert torch.equal(ops.gemm_rows(other, w, torch.float32, splits=1, waves=waves)[m - 1], whole[m - 1])


@pytest.mark.parametrize("nk", [(4096, 4096), (777, 192), (6144, 4096), (130, 1024), (40, 64), (24576, 4096), (4096, 12288)])
def test_products_read_the_tiled_copy_of_a_weight_to_the_same_bits(nk):
    """Both weight-streaming products, given a weight whose tiled copy is kept, read that copy (every load of
    a wave one piece of 1 KB, with the non-temporal hint) and give what they give from the rows: the same
    bits, in every output mode, for rows of the last tile and columns of the last chunk that do not exist.
    The copy goes when the weight goes."""
    from leone_amd import ops
    n, k = nk
    torch.manual_seed(29)
    w = (torch.randn(n, k, device=DEV) * 0.05).bfloat16()
    gain = (1 + 0.1 * torch.randn(k, device=DEV)).bfloat16()
    next_gain = (1 + 0.1 * torch.randn(n, device=DEV)).bfloat16()
    ops.drop_streamed_copies()

    def run_all():
        found = []
        for m in (1, 3, 8, 10, 16, 37, 64, 128):
            x = torch.randn(m, k, generator=torch.Generator(device=DEV).manual_seed(m), device=DEV).bfloat16()
            stream = torch.randn(m, k, generator=torch.Generator(device=DEV).manual_seed(100 + m), device=DEV)
            if m <= ops.FUSED_ROWS:
                found.append(ops.gemm_fused(x, w, torch.float32))
                found.append(ops.gemm_fused(x, w, torch.bfloat16))
                found.append(ops.gemm_fused(ops.NormedRows(stream, gain, 1e-6, torch.bfloat16), w, torch.float32))
                res = torch.ones(m, n, device=DEV)
                ops.gemm_fused(x, w, residual=res)
                found.append(res)
                if n % 64 == 0 and ops.prepared_fits(m, n):
                    res = torch.ones(m, n, device=DEV)
                    prepared = ops.gemm_fused(x, w, residual=res, next_norm=(next_gain, 1e-6, torch.bfloat16))
                    found += [res, prepared.operand, prepared.squares]
                if ops.prepared_fits(m, k):
                    found.append(ops.gemm_fused(ops.NormedRows(stream, gain, 1e-6, torch.bfloat16).prepare(), w, torch.float32))
                if n % 16 == 0:
                    found.append(ops.gemm_fused(x, w, gated=True))
            found.append(ops.gemm_rows(x, w, torch.float32, may_split=False))
            found.append(ops.gemm_rows(x, w, torch.float32, splits=3, waves=4))
            found.append(ops.gemm_rows(x, w, torch.bfloat16, may_split=False, waves=8))
            res = torch.ones(m, n, device=DEV)
            ops.gemm_rows(x, w, residual=res, splits=1)
            found.append(res)
            if n % 16 == 0:
                found.append(ops.gemm_rows(x, w, gated=True))
        return found

    from_rows = run_all()
    assert ops.streamed_copy(w) is None
    assert ops.keep_streamed_copy(w) == -(-n // 16) * 16 * k * 2
    tiles = ops.streamed_copy(w)
    assert tiles is not None and tiles.shape == (-(-n // 16), k // 64, 2, 4, 16, 8)
    from_tiles = run_all()
    assert len(from_rows) == len(from_tiles) > 40
    for index, (a, b) in enumerate(zip(from_rows, from_tiles)):
        assert torch.equal(a, b), f"result {index} differs"
    # the copy is the weight's: another tensor of the same values has none, and it goes with the weight
    assert ops.streamed_copy(w.clone()) is None
    del w, tiles
    assert not ops._streamed


@pytest.mark.parametrize("tiled", [False, True])
@pytest.mark.parametrize("m", [5, 40, 100])
def test_weight_streaming_products_do_not_read_weights_beyond_k_as_numbers(m, tiled):
    """K that is no multiple of a chunk: the kernels load the row's end again for the runs beyond K and must count
    those as zero themselves, not only through the zeros that stand for X there: with an infinite weight in a
    row's last columns the sum of that row of W is infinite, as the plain sum is, and not NaN (infinity times
    the zero beyond K)."""
    from leone_amd import ops
    n, k = 96, 320 if tiled else 328              # 256 + 64 (whole steps of the tiled copy), 256 + 72
    torch.manual_seed(31)
    x = torch.randn(m, k, device=DEV).bfloat16()
    x[:, k - 1] = x[:, k - 1].abs() + 0.5
    w = (torch.randn(n, k, device=DEV) * 0.05).bfloat16()
    w[3, k - 1] = float("inf")
    ops.drop_streamed_copies()
    if tiled:
        ops.keep_streamed_copy(w)
    finite = w.clone()
    finite[3, k - 1] = 0
    want = x.double() @ finite.double().T
    outs = {"rows": ops.gemm_rows(x, w, torch.float32, may_split=False)}
    if m <= ops.FUSED_ROWS:
        outs["fused"] = ops.gemm_fused(x, w, torch.float32)
    keep = torch.ones(n, dtype=torch.bool, device=DEV)
    keep[3] = False
    for name, out in outs.items():
        close(out[:, keep], want[:, keep], 2e-6 * k, 1e-5, name)
        assert (out[:, 3] == float("inf")).all(), (name, out[:, 3])
    ops.drop_streamed_copies()


def test_gemm_rows_plan_fills_the_compute_units():
    """The plan at the shapes it was measured on, and that it never names an empty range of K."""
    from leone_amd import ops
    assert ops.rows_plan(64, 6144, 4096, True) == (4, 2)
    assert ops.rows_plan(64, 51200, 5120, False) == (8, 1)        # 400 workgroups, two rounds; four waves would need four
    assert ops.rows_plan(24, 34816, 5120, False) == (6, 1)
    assert ops.rows_plan(64, 4096, 4096, True) == (4, 4)
    assert ops.rows_plan(64, 24576, 4096, False) == (6, 1)
    assert ops.rows_plan(64, 4096, 12288, True) == (4, 4)
    assert ops.rows_plan(128, 151936, 4096, False) == (8, 1)
    assert ops.rows_plan(128, 4096, 4096, True) == (4, 4)
    for m, n, k in [(16, 40, 8), (128, 100000, 72), (33, 5120, 25600), (90, 51200, 5120), (20, 7168, 5120)]:
        for may in (False, True):
            waves, splits = ops.rows_plan(m, n, k, may)
            chunks = -(-k // (256 if m <= 64 else 128))
            assert waves in ops.ROWS_WAVES and 1 <= splits <= (16 if may else 1)
            assert -(-chunks // splits) * (splits - 1) < chunks


@pytest.mark.parametrize("mnk", [(16, 4096, 4096), (37, 80, 176), (128, 777, 64), (64, 4096, 12288)])
def test_gemm_rows_residual(mnk):
    from leone_amd import ops
    m, n, k = mnk
    torch.manual_seed(22)
    x = torch.randn(m, k, device=DEV).bfloat16()
    w = (torch.randn(n, k, device=DEV) * 0.05).bfloat16()
    stream = torch.randn(m, n, device=DEV)
    before = stream.clone()
    assert ops.gemm_rows(x, w, residual=stream, splits=1, waves=4) is None
    want = before.double() + x.double() @ w.double().T
    close(stream, want, 2e-6 * k, 1e-5, "product added into the stream")
    assert torch.equal(stream, before + ops.gemm_rows(x, w, torch.float32, splits=1, waves=4))
    # as the engine runs it: what comes back (planes, if K was cut) is added by the next norm's kernel
    stream2 = before.clone()
    delta = ops.linear(x, w, residual=stream2)
    gain = torch.ones(n, device=DEV)
    ops.add_rmsnorm(stream2, delta, gain, 1e-6, torch.bfloat16)
    close(stream2, want, 2e-6 * k, 1e-5, "planes added by the norm")


@pytest.mark.parametrize("mfk", [(16, 12288, 4096), (17, 1024, 512), (36, 88, 80), (128, 256, 96), (64, 17408, 5120)])
def test_gemm_rows_gated(mfk):
    from leone_amd import ops
    m, f, k = mfk
    torch.manual_seed(23)
    x = torch.randn(m, k, device=DEV).bfloat16()
    wg, wu = (torch.randn(f, k, device=DEV) * 0.05).bfloat16(), (torch.randn(f, k, device=DEV) * 0.05).bfloat16()
    w = ops.interleave_gate_up(wg, wu).contiguous()
    for waves in ops.ROWS_WAVES:
        out = ops.gemm_rows(x, w, gated=True, waves=waves)
        assert out.shape == (m, f) and out.dtype == torch.bfloat16
        want = plain.swiglu(x.double() @ wg.double().T, x.double() @ wu.double().T)
        close(out, want, 1e-2, 1e-2, "gated product")
    if m > ops.FUSED_ROWS:                            # fewer rows go to the kernel for few rows
        assert torch.equal(ops.linear(x, w, gated=True), ops.gemm_rows(x, w, gated=True))


@pytest.mark.parametrize("gain_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mnk", [(1, 4096, 4096), (7, 128, 176), (10, 960, 64), (16, 4096, 12288), (4, 5120, 5120)])
def test_gemm_fused_prepares_the_next_norm(mnk, gain_dtype):
    """The product that adds into the stream leaves bf16(stream * gain) and partial sums of squares behind;
    the next product takes them in place of a norm kernel (the reference's fused norm + residual store,
    crates/leone/src/backend.rs:2371-2390).  Both halves against double, and against the kernels they replace."""
    from leone_amd import ops
    m, n, k = mnk
    torch.manual_seed(31)
    x = torch.randn(m, k, device=DEV).bfloat16()
    w = (torch.randn(n, k, device=DEV) * 0.05).bfloat16()
    gain = (1 + 0.1 * torch.randn(n, device=DEV)).to(gain_dtype)
    eps = 1e-5
    stream = torch.randn(m, n, device=DEV) * 2
    plain_stream = stream.clone()
    assert ops.gemm_fused(x, w, residual=plain_stream) is None
    prepared = ops.gemm_fused(x, w, residual=stream, next_norm=(gain, eps, torch.bfloat16))
    assert isinstance(prepared, ops.PreparedRows) and prepared.x is stream
    assert torch.equal(stream, plain_stream)                                    # the same sum, the same bits
    assert torch.equal(prepared.operand, (stream * gain.float()).bfloat16())
    assert prepared.squares.shape == (m, -(-n // 16))
    close(prepared.squares.double().sum(1), (stream.double() ** 2).sum(1), 1e-4, 1e-5, "sums of squares")
    # the consumer: scaled by 1/rms of the stream, like the folded norm and like norm, then product
    n2 = 96
    w2 = (torch.randn(n2, n, device=DEV) * 0.05).bfloat16()
    out = ops.gemm_fused(prepared, w2, torch.float32)
    inv = 1.0 / torch.sqrt((stream.double() ** 2).mean(dim=1, keepdim=True) + eps)
    want = (prepared.operand.double() @ w2.double().T) * inv
    close(out, want, 2e-6 * n, 2e-5, "prepared operand, then product")
    folded = ops.gemm_fused(ops.NormedRows(stream, gain, eps, torch.bfloat16), w2, torch.float32)
    close(out, folded.double(), 1e-5, 1e-5, "prepared against folded")
    assert torch.equal(out, ops.gemm_fused(prepared, w2, torch.float32))
    # anyone else normalises the stream in the usual way
    assert torch.equal(prepared.materialize(), ops.add_rmsnorm(stream, None, gain, eps, torch.bfloat16))
    # and linear() takes the prepared rows for a gated product as well (beyond FUSED_ROWS rows it normalises
    # the stream itself and rounds in another place)
    if m > ops.FUSED_ROWS:
        return
    wg, wu = (torch.randn(40, n, device=DEV) * 0.1).bfloat16(), (torch.randn(40, n, device=DEV) * 0.1).bfloat16()
    got = ops.linear(prepared, ops.interleave_gate_up(wg, wu).contiguous(), gated=True)
    operand = prepared.operand.double()
    close(got, plain.swiglu((operand @ wg.double().T) * inv, (operand @ wu.double().T) * inv), 1e-2, 1e-2, "gated")


@pytest.mark.parametrize("planes", [1, 3])
@pytest.mark.parametrize("window", [0, 37])
@pytest.mark.parametrize("shape", [(32, 8, 128, 64), (6, 1, 64, 16), (40, 2, 128, 32), (4, 4, 192, 16)])
def test_attention_decode_from_the_projection(shape, window, planes):
    """One launch for head norms, rotation, cache write and attention of single decoded tokens gives what the
    two kernels give one after the other: the same cache contents bit for bit, the same output to the rounding
    of the queries (a product and a sum may be contracted differently in the two kernels)."""
    from leone_amd import ops
    q_heads, kv_heads, dim, page = shape
    torch.manual_seed(41)
    lengths = [1, 5, page, page + 1, 3 * page + 7, 700]               # keys each row sees, its own included
    rows = len(lengths)
    blocks = -(-max(lengths) // page)
    n_pages = rows * blocks + 2
    order = torch.randperm(n_pages)[:rows * blocks].int().view(rows, blocks)
    k_pool = (torch.randn(n_pages, kv_heads, dim // 8, page, 8) * 0.5).bfloat16().to(DEV)
    v_pool = (torch.randn(n_pages, kv_heads, page // 8, dim, 8) * 0.5).bfloat16().to(DEV)
    table = order.to(DEV).contiguous()
    positions = torch.tensor([n - 1 for n in lengths], dtype=torch.int32, device=DEV)
    entry = torch.arange(rows, dtype=torch.int32, device=DEV)
    width = (q_heads + 2 * kv_heads) * dim
    if planes == 1:
        qkv = torch.randn(rows, width, device=DEV).bfloat16()
    else:
        qkv = torch.randn(planes, rows, width, device=DEV) * torch.tensor([1.0, 0.02, 3e-4], device=DEV).view(3, 1, 1)
    q_gain = (1 + 0.1 * torch.randn(dim, device=DEV)).bfloat16()
    k_gain = (1 + 0.1 * torch.randn(dim, device=DEV)).bfloat16()
    cos, sin = ops.rope_table(1e6, dim, 1024, DEV)
    scale = 1 / math.sqrt(dim)
    k1, v1, k2, v2 = k_pool.clone(), v_pool.clone(), k_pool.clone(), v_pool.clone()
    q = ops.qk_norm_rope_write(qkv, q_heads, kv_heads, dim, q_gain, k_gain, 1e-6, cos, sin, positions, entry, table,
                               k1, v1, out_dtype=torch.bfloat16)
    want = ops.attention_decode(q, k1, v1, positions, entry, table, q_heads, scale, window, max_context=700)
    got = ops.attention_decode_projected(qkv, q_heads, kv_heads, dim, q_gain, k_gain, 1e-6, cos, sin, k2, v2, positions,
                                         entry, table, scale, window, max_context=700)
    assert torch.equal(k1, k2) and torch.equal(v1, v2) and not torch.equal(k1, k_pool)
    close(got, want.double(), 2e-2, 2e-2, "attention from the projection")
    assert (got.double() - want.double()).abs().mean() < 2e-4
    # a run that reads another run's cache writes nothing; no norm, no rotation
    k3, v3 = k1.clone(), v1.clone()
    plain_q = ops.qk_norm_rope_write(qkv, q_heads, kv_heads, dim, None, None, 1.0, None, None, positions, entry, table,
                                     k3, v3, write_cache=False, out_dtype=torch.bfloat16)
    want3 = ops.attention_decode(plain_q, k3, v3, positions, entry, table, q_heads, scale, window, max_context=700)
    got3 = ops.attention_decode_projected(qkv, q_heads, kv_heads, dim, None, None, 1.0, None, None, k3, v3, positions,
                                          entry, table, scale, window, max_context=700, write_cache=False)
    assert torch.equal(k3, k1) and torch.equal(v3, v1)
    assert torch.equal(got3, want3)                                   # nothing to contract: the same bits


def test_library_products_with_a_measured_choice_of_algorithm():
    """The vendor library's product for many rows, once with the algorithm its heuristic names (through torch) and
    once with the one that was fastest when timed: both against a float64 product, for the three forms ``linear``
    asks for (bfloat16 out, float32 out, added into the float32 stream); a problem of another size stays with
    the heuristic."""
    from leone_amd import ops
    assert ops.library_product_available(), "hipBLASLt was not found in the process"
    generator = torch.Generator().manual_seed(31)
    n, k, rows = 384, 512, 200
    weights = [(torch.randn(n, k, generator=generator) * 0.05).bfloat16().cuda() for _ in range(3)]
    x = torch.randn(rows, k, generator=generator).bfloat16().cuda()
    stream = torch.randn(rows, n, generator=generator).cuda()
    exact = x.double() @ weights[1].double().t()
    try:
        for out_dtype, adds in ((torch.bfloat16, False), (torch.float32, False), (torch.float32, True)):
            record = ops.tune_library_product(rows, weights, out_dtype, adds, candidates=64)
            assert record["kept"] and record["timed"] >= 1, record
            assert 0 < record["tuned_us"] <= record["library_us"], record
            problem = (0, rows, n, k, ops.F32 if out_dtype == torch.float32 else ops.BF16, int(adds))
            assert problem in ops._tuned_products
            for m in (rows, rows + 8):                          # tuned, and left to the heuristic
                with ops.record_library_products() as seen:
                    if adds:
                        y = stream[:1].repeat(m, 1).contiguous()
                        base = y.double().clone()
                        assert ops.linear(x[:1].repeat(m, 1).contiguous() if m != rows else x, weights[1], residual=y) is None
                    else:
                        base = 0.0
                        y = ops.linear(x[:1].repeat(m, 1).contiguous() if m != rows else x, weights[1], out_dtype=out_dtype)
                assert list(seen.problems) == [(m, n, k, problem[4], problem[5])]
                want = base + (exact if m == rows else exact[:1].expand(m, n))
                err = (y.double() - want).abs().max().item()
                bound = 2e-2 if out_dtype == torch.bfloat16 else 2e-5      # half a bfloat16 step at |y| < 4; float sums of 512 terms
                assert err <= bound, (out_dtype, adds, m, err)
    finally:
        ops.forget_tuned_products()
    assert not ops._tuned_products
    with pytest.raises(ops.KernelError, match="not tuned"):
        y = torch.empty(rows, n, dtype=torch.float32, device="cuda")
        ops.call("leone_library_product", x.data_ptr(), weights[0].data_ptr(), y.data_ptr(), rows, n, k, ops.F32, 0, None)

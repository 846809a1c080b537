"""Kunudra on the GPU against the plain model (`plain_kunudra`, NumPy float64): every kernel of its
own alone, each mixer alone in a one-layer model, then whole models of several tiny configurations
under every kind of schedule, in the 32-bit engine and in bfloat16 (held against the plain model
with bfloat16 storage as a yardstick)."""

import copy
import io
import json

import numpy as np
import pytest
import torch

import plain_kunudra as pk
import replay_util as ru
import tiny_kunudra as tk

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def dev(values, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(values)).to(device=DEV, dtype=dtype)


def ints(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


def rounded(values, dtype):
    """What the engine reads when `values` are stored in `dtype`, as float64."""
    return values.astype(np.float64) if dtype == "float32" else tk.bf16_round(values).astype(np.float64)


def tolerance(dtype, scale=1.0):
    return (2e-6 if dtype == "float32" else 1.2e-2) * scale


_ORACLES: dict = {}


def oracle(name, cfg, weights, tokens) -> ru.Oracle:
    key = (name, tuple(tokens))
    if key not in _ORACLES:
        wide = {k: v.astype(np.float64) for k, v in weights.items()}
        _ORACLES[key] = ru.Oracle(pk.logits(cfg, wide, tokens), pk.logits(cfg, wide, tokens, store=pk.bf16_round))
        # how far float32 storage alone, with exact arithmetic between, moves the logits of this very input
        _ORACLES[key].moved_by_float32 = moved_by_float32(cfg, wide, tokens, _ORACLES[key].exact)
    return _ORACLES[key]


def f32_round(a):
    return np.asarray(a, dtype=np.float32).astype(np.float64)


def moved_by_float32(cfg, wide, tokens, exact) -> float:
    """How far float32 storage and float32 rotation angles alone, with exact arithmetic between, move the
    logits of this input."""
    pk.ANGLE_TYPE = np.float32
    try:
        return float(np.abs(pk.logits(cfg, wide, tokens, store=f32_round) - exact).max())
    finally:
        pk.ANGLE_TYPE = np.float64


def assert_close(got, want: ru.Oracle, dtype, what, bf16_max_factor=ru.BF16_MAX_FACTOR):
    """The engine against the plain model: bfloat16 against its yardstick; float32 within 1e-4, or, where
    float32 storage and angles alone move this input's logits further than half of that, within twice that far."""
    ru.assert_close(got, want, dtype, what, fp32_tol=max(ru.FP32_TOL, 2.0 * getattr(want, "moved_by_float32", 0.0)),
                    bf16_max_factor=bf16_max_factor)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    """Per configuration and engine dtype: (name of the pair, config, page size, weights, folder).  The
    bfloat16 engine gets weights whose experts are chosen steadily (see `tiny_kunudra.make_weights`)."""
    out = {}
    for number, (name, (cfg, block)) in enumerate(tk.CONFIGS.items()):
        for dtype in DTYPES:
            weights = tk.make_weights(cfg, seed=70 + number, steady_choice=dtype == "bfloat16")
            folder = tk.write_model_dir(tmp_path_factory.mktemp("kunudra") / f"{name}-{dtype}", cfg, weights)
            out[name, dtype] = (f"{name}-{dtype}", cfg, block, weights, folder)
    return out


def runner_for(folder, dtype, block, pages=64, seats=4, graphs=True):
    from mini_infer_amd.engine import ModelRunner

    return ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=pages, block_size=block, max_concurrent=seats,
                                       cuda_graph=graphs)


# ---------------------------------------------------------------------------------------------
# each kernel alone
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [10, 64, 2500])
def test_token_rows_plus_hashed_pair_rows_and_the_token_kept_between_steps(dtype, width):
    """Three requests in scattered slots over three steps: one begins in the first step, one has
    begun before (its last token is in its slot), one brings a single token; then portions that
    begin where the last step ended.  A slot's second owner starts from the last row again."""
    from mini_infer_amd import ops

    rng = np.random.default_rng(width)
    vocab, buckets, mp, mc = 57, 23, 31, 5
    table = rng.standard_normal((vocab, width)).astype(np.float32)
    pairs = rng.standard_normal((buckets + 1, width)).astype(np.float32)
    state = torch.zeros((6, 3), dtype=torch.int32, device=DEV)[:, :1]  # rows strided like the engine's
    sequences = {2: rng.integers(0, vocab, 9).tolist(), 4: rng.integers(0, vocab, 7).tolist(), 0: rng.integers(0, vocab, 3).tolist()}
    fed = {2: 0, 4: 0, 0: 0}

    def plain(tokens, n):
        row = buckets if n == 0 else (tokens[n - 1] * mp + tokens[n] * mc) % buckets
        return rounded(table, dtype)[tokens[n]] + rounded(pairs, dtype)[row]

    for step in ({2: 4, 4: 1}, {4: 3, 0: 1, 2: 1}, {0: 2, 2: 4, 4: 3}):
        ids, pos, req, cu, slots, want = [], [], [], [0], [], []
        for b, (slot, count) in enumerate(step.items()):
            for n in range(fed[slot], fed[slot] + count):
                ids.append(sequences[slot][n]), pos.append(n), req.append(b)
                want.append(plain(sequences[slot], n))
            fed[slot] += count
            cu.append(len(ids)), slots.append(slot)
        out, cast = ops.embed_pair_hash(dev(table, TORCH[dtype]), dev(pairs, TORCH[dtype]), ints(ids), ints(pos), ints(req), ints(cu),
                                        ints(slots), state, mul_prev=mp, mul_cur=mc, want_cast=True)
        np.testing.assert_allclose(out.cpu().numpy(), np.array(want), rtol=0, atol=2e-6)
        np.testing.assert_allclose(cast.float().cpu().numpy(), np.array(want), rtol=0, atol=tolerance(dtype, 4))
        for slot in step:
            assert int(state[slot, 0]) == sequences[slot][fed[slot] - 1]
    # a request that begins in a slot that was used before, and a padding row (slot -1: nobody's row)
    out, _ = ops.embed_pair_hash(dev(table, TORCH[dtype]), dev(pairs, TORCH[dtype]), ints([5, 6, 7]), ints([0, 1, 0]), ints([0, 0, 1]),
                                 ints([0, 2, 3]), ints([2, -1]), state, mul_prev=mp, mul_cur=mc)
    want = [plain([5, 6], 0), plain([5, 6], 1), plain([7], 0)]
    np.testing.assert_allclose(out.cpu().numpy(), np.array(want), rtol=0, atol=1e-6)
    assert int(state[2, 0]) == 6 and int(state[5, 0]) == 7


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [10, 64, 2500, 5000])
@pytest.mark.parametrize("scaled", [True, False])
def test_the_norm_behind_the_sum(dtype, width, scaled):
    from mini_infer_amd import ops

    rng = np.random.default_rng(width + scaled)
    rows, alpha, eps = 7, 1.7, 1e-5
    x = rng.standard_normal((rows, width)).astype(np.float32)
    y = rng.standard_normal((rows, width)).astype(np.float32) * 2
    scale = rng.uniform(0.5, 1.5, width).astype(np.float32)
    factor = rng.uniform(0.5, 1.5, width).astype(np.float32)
    stream = dev(x)
    cast = ops.scale_add_norm(stream, dev(y, TORCH[dtype]), dev(scale) if scaled else None, dev(factor), alpha, eps, TORCH[dtype])
    total = alpha * x.astype(np.float64) + (scale if scaled else 1.0) * rounded(y, dtype)
    want = total / np.sqrt((total ** 2).mean(axis=1, keepdims=True) + eps) * factor
    np.testing.assert_allclose(stream.cpu().numpy(), want, rtol=0, atol=3e-6)
    np.testing.assert_allclose(cast.float().cpu().numpy(), want, rtol=0, atol=tolerance(dtype, 4))
    # the norm alone on picked rows: the stream stays
    before = stream.clone()
    picked = ops.scale_add_norm(stream, None, None, dev(factor), 1.0, eps, TORCH[dtype], rows=ints([5, 0, 5]))
    assert torch.equal(stream, before)
    again = want[[5, 0, 5]]
    again = again / np.sqrt((again ** 2).mean(axis=1, keepdims=True) + eps) * factor
    np.testing.assert_allclose(picked.float().cpu().numpy(), again, rtol=0, atol=tolerance(dtype, 4))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width, extra", [(7, 3), (80, 144), (300, 0)])
def test_a_norm_over_the_first_columns_of_wider_rows(dtype, width, extra):
    from mini_infer_amd import ops

    rng = np.random.default_rng(width)
    x = rng.standard_normal((5, width + extra)).astype(np.float32) * 3
    w = rng.uniform(0.5, 1.5, width).astype(np.float32)
    got = ops.norm_rows(dev(x, TORCH[dtype]), dev(w), 1e-5, width=width).float().cpu().numpy()
    head = rounded(x, dtype)[:, :width]
    np.testing.assert_allclose(got, head / np.sqrt((head ** 2).mean(axis=1, keepdims=True) + 1e-5) * w, rtol=0, atol=tolerance(dtype, 4))


def paged(rows: np.ndarray, page_size: int, order: list[int], dtype) -> torch.Tensor:
    """[tokens, heads, dim] laid into pages [num_pages, heads, page_size, dim], page i of the
    request at page id order[i]."""
    tokens, heads, dim = rows.shape
    pages = np.zeros((max(order) + 1, heads, page_size, dim), dtype=np.float32)
    for t in range(tokens):
        pages[order[t // page_size], :, t % page_size] = rows[t]
    return dev(pages, TORCH[dtype])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, page, mixing", [(4, 2, 16, 24, 8, True), (3, 3, 10, 6, 4, False), (8, 4, 40, 24, 16, True),
                                                                       (2, 1, 6, 2, 8, True)])
def test_whole_projection_norms_mixed_values_and_the_cache_write(dtype, heads, kv_heads, dim, vdim, page, mixing):
    from mini_infer_amd import ops

    rng = np.random.default_rng(dim)
    tokens, eps, lam = 11, 1e-5, 0.37
    qw, kw, vw = heads * dim, kv_heads * dim, kv_heads * vdim
    spare = (8, 8) if dim == 40 else (5, 3)  # (rows that the vector loads take, and rows they do not)
    rows = rng.standard_normal((tokens, qw + kw + vw + spare[0])).astype(np.float32) * 2
    other = rng.standard_normal((tokens, vw + spare[1])).astype(np.float32)
    q_weight, k_weight = rng.uniform(0.5, 1.5, qw).astype(np.float32), rng.uniform(0.5, 1.5, kw).astype(np.float32)
    slots = rng.permutation(5 * page)[:tokens].astype(np.int32)
    slots[3] = -1  # a row that writes nowhere
    k_pages = torch.zeros((5, kv_heads, page, dim), dtype=TORCH[dtype], device=DEV)
    v_pages = torch.zeros((5, kv_heads, page, vdim), dtype=TORCH[dtype], device=DEV)
    qkv = dev(rows, TORCH[dtype])
    ops.qkv_norm_write(qkv, dev(q_weight), dev(k_weight), ints(slots), k_pages, v_pages, q_width=qw, kv_heads=kv_heads, head_dim=dim,
                       v_head_dim=vdim, eps=eps, other_values=dev(other, TORCH[dtype])[:, :vw] if mixing else None,
                       mix=dev(np.array([lam], dtype=np.float32)) if mixing else None)
    r, o = rounded(rows, dtype), rounded(other, dtype)
    q, k, v = r[:, :qw], r[:, qw:qw + kw], r[:, qw + kw:qw + kw + vw]
    want_q = q / np.sqrt((q ** 2).mean(axis=1, keepdims=True) + eps) * q_weight
    want_k = k / np.sqrt((k ** 2).mean(axis=1, keepdims=True) + eps) * k_weight
    want_v = (1 - lam) * v + lam * o[:, :vw] if mixing else v
    got = qkv.float().cpu().numpy()
    np.testing.assert_allclose(got[:, :qw], want_q, rtol=0, atol=tolerance(dtype, 4))
    np.testing.assert_array_equal(got[:, qw:], tk.bf16_round(rows)[:, qw:] if dtype == "bfloat16" else rows[:, qw:])  # k, v stay
    kp, vp = k_pages.float().cpu().numpy(), v_pages.float().cpu().numpy()
    for t, slot in enumerate(slots):
        if slot < 0:
            continue
        np.testing.assert_allclose(kp[slot // page, :, slot % page].reshape(-1), want_k[t], rtol=0, atol=tolerance(dtype, 4))
        np.testing.assert_allclose(vp[slot // page, :, slot % page].reshape(-1), want_v[t], rtol=0, atol=tolerance(dtype, 4))
    assert np.count_nonzero(kp) == (tokens - 1) * kw  # nothing else was written


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, page, window", [(4, 2, 16, 24, 8, 40), (3, 3, 10, 6, 4, 37), (8, 4, 40, 24, 16, 72),
                                                                       (2, 1, 130, 66, 16, 333)])
def test_capped_scores_distance_bias_window_and_a_sink_per_head(dtype, heads, kv_heads, dim, vdim, page, window):
    """One request of 333 keys in scattered pages, queries at its last 5 positions (a portion) and
    the last one alone (a decoded token).  Head 0's last query singles out the LAST key inside its
    window (without a window that reaches back to the start: key 3, hundreds of positions away) and head
    1's last query the first key OUTSIDE it (which must not show); the cap is small
    enough to flatten the largest scores, the slopes and sinks are those of no particular model."""
    from mini_infer_amd import ops

    rng = np.random.default_rng(dim)
    keys_n, queries_n, scale, cap = 333, 5, 1.0 / np.sqrt(dim), 8.0
    k = rng.standard_normal((keys_n, kv_heads, dim)).astype(np.float32)
    v = rng.standard_normal((keys_n, kv_heads, vdim)).astype(np.float32)
    q = rng.standard_normal((queries_n, heads, dim)).astype(np.float32)
    group = heads // kv_heads
    inside, outside = keys_n - window, keys_n - window - 1
    if outside < 0:  # every key is seen: a far one, 329 positions back, is made to stand out
        q[-1, 0] = 8.0 * k[3, 0] / np.linalg.norm(k[3, 0])
        k[3, 0] *= 3.0
    if outside >= 0:
        q[-1, 0] = 8.0 * k[inside, 0] / np.linalg.norm(k[inside, 0])
        k[inside, 0] *= 3.0
        if heads > 1 and 1 // group != 0:
            q[-1, 1] = 8.0 * k[outside, 1 // group] / np.linalg.norm(k[outside, 1 // group])
            k[outside, 1 // group] *= 3.0
    slopes = (0.05 * 2.0 ** (-6.0 * (np.arange(heads) + 1) / heads)).astype(np.float32)
    sinks = (rng.standard_normal(heads) * 2).astype(np.float32)
    order = list(rng.permutation(-(-keys_n // page) + 3))[: -(-keys_n // page)]
    positions = np.arange(keys_n - queries_n, keys_n)
    kq, vq, qq = rounded(k, dtype), rounded(v, dtype), rounded(q, dtype)
    want = np.zeros((queries_n, heads, vdim))
    for i, p in enumerate(positions):
        lo = max(0, p - window + 1)
        for a in range(heads):
            s = kq[lo: p + 1, a // group] @ qq[i, a] * scale
            s = cap * np.tanh(s / cap) - slopes[a] * (p - np.arange(lo, p + 1))
            e = np.exp(s)
            want[i, a] = e @ vq[lo: p + 1, a // group] / (np.exp(sinks[a]) + e.sum())
            if i == queries_n - 1 and a == 0:
                # the key at the window's edge (or the far key) is what the answer is made of
                assert e[0 if outside >= 0 else 3] / e.sum() > 0.5
    for rows in (slice(0, queries_n), slice(queries_n - 1, queries_n)):
        n = rows.stop - rows.start
        got = ops.paged_attention(
            dev(q[rows].reshape(n, -1), TORCH[dtype]), paged(k, page, order, dtype), paged(v, page, order, dtype),
            ints(order).view(1, -1), ints([0] * n), ints(positions[rows]), ints([0, n]), [0, n],
            q_heads=heads, kv_heads=kv_heads, head_dim=dim, scale=scale, window=window, max_seq_len=keys_n, v_head_dim=vdim,
            slopes=dev(slopes), sinks=dev(sinks), softcap=cap,
        ).float().cpu().numpy().reshape(n, heads, vdim)
        np.testing.assert_allclose(got, want[rows], rtol=0, atol=tolerance(dtype, 4))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim", [32, 64, 128])
@pytest.mark.parametrize("shaped", [False, True])
def test_a_sink_per_head_capped_scores_and_distance_bias_on_the_matrix_cores(dtype, dim, shaped):
    """The matrix-core kernel (bfloat16, values transposed inside a page) with a window and a sink of
    its own for every head, and (`shaped`) scores capped and biased by the distance, as a prompt's last
    portion and as a decoded token."""
    from mini_infer_amd import ops

    if dtype != "bfloat16":
        pytest.skip("the matrix-core kernel is bfloat16's")
    rng = np.random.default_rng(dim)
    heads, kv_heads, page, keys_n, queries_n, scale, window = 4, 2, 16, 300, 70, 0.3, 50
    cap = 3.0 if shaped else None  # (scores of std 0.3 * sqrt(dim): many lie beyond the cap)
    slopes = (0.3 * 2.0 ** (-6.0 * (np.arange(heads) + 1) / heads)).astype(np.float32) if shaped else None
    k = rng.standard_normal((keys_n, kv_heads, dim)).astype(np.float32)
    v = rng.standard_normal((keys_n, kv_heads, dim)).astype(np.float32)
    q = rng.standard_normal((queries_n, heads, dim)).astype(np.float32)
    sinks = (rng.standard_normal(heads) * 3).astype(np.float32)
    order = list(rng.permutation(-(-keys_n // page) + 3))[: -(-keys_n // page)]
    positions = np.arange(keys_n - queries_n, keys_n)
    kq, vq, qq = rounded(k, dtype), rounded(v, dtype), rounded(q, dtype)
    want = np.zeros((queries_n, heads, dim))
    for i, p in enumerate(positions):
        lo = max(0, p - window + 1)
        for a in range(heads):
            score = kq[lo: p + 1, a // 2] @ qq[i, a] * scale
            if shaped:
                score = cap * np.tanh(score / cap) - slopes[a] * (p - np.arange(lo, p + 1))
            e = np.exp(score)
            want[i, a] = e @ vq[lo: p + 1, a // 2] / (np.exp(sinks[a]) + e.sum())
    v_t = paged(v, page, order, dtype).transpose(2, 3).contiguous()
    for rows in (slice(0, queries_n), slice(queries_n - 1, queries_n)):
        n = rows.stop - rows.start
        got = ops.paged_attention(
            dev(q[rows].reshape(n, -1), TORCH[dtype]), paged(k, page, order, dtype), v_t, ints(order).view(1, -1), ints([0] * n),
            ints(positions[rows]), ints([0, n]), [0, n], q_heads=heads, kv_heads=kv_heads, head_dim=dim, scale=scale,
            window=window, max_seq_len=keys_n, v_transposed=True, sinks=dev(sinks), softcap=cap,
            slopes=dev(slopes) if shaped else None,
        ).float().cpu().numpy().reshape(n, heads, dim)
        np.testing.assert_allclose(got, want[rows], rtol=0, atol=tolerance(dtype, 4))


def plain_experts(x, gate_up, down, router, correction, gate_row, shared, top, route_scale):
    """Routed experts on stacked weights, the plain way (float64)."""
    experts, ff = gate_up.shape[0], gate_up.shape[1] // 2
    out, chosen, weights = np.zeros_like(x), [], []
    for t in range(x.shape[0]):
        z = router @ x[t]
        s = np.exp(z - z.max())
        s /= s.sum()
        picks = np.argsort(-(s + (0 if correction is None else correction)), kind="stable")[:top]
        chosen.append(picks), weights.append(s[picks] * route_scale)
        for e in picks:
            if e >= experts:
                out[t] += s[e] * route_scale * x[t]
            else:
                g, u = gate_up[e, :ff] @ x[t], gate_up[e, ff:] @ x[t]
                out[t] += s[e] * route_scale * (down[e] @ (g / (1 + np.exp(-g)) * u))
    gates = None
    if gate_row is not None:
        gates = 1 / (1 + np.exp(-(x @ gate_row)))
        out += gates[:, None] * shared
    return out, np.array(chosen), np.array(weights), gates


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows, width, ff, experts, identity, top, with_shared", [
    (1, 24, 10, 3, 0, 1, False), (9, 64, 48, 6, 2, 2, True), (40, 90, 26, 5, 3, 4, True), (70, 256, 128, 16, 1, 4, False),
    (5, 48, 16, 1, 1, 2, True), (3, 2048, 72, 4, 1, 2, False), (130, 136, 40, 3, 0, 2, True)])
def test_the_router_and_both_forms_of_the_experts(dtype, rows, width, ff, experts, identity, top, with_shared):
    """The router's choice and weights against NumPy, then the experts pair by pair (few rows) and
    sorted by expert (many rows) against the plain sum; identity experts, a shared expert with its
    gate, an expert nobody chose."""
    from mini_infer_amd import ops

    rng = np.random.default_rng(rows * 7 + width)
    outputs = experts + identity
    x = rng.standard_normal((rows, width)).astype(np.float32)
    router = (rng.standard_normal((outputs, width)) * 2.5 / np.sqrt(width)).astype(np.float32)
    correction = (rng.standard_normal(outputs) * 0.15).astype(np.float32)
    if experts > 2:
        correction[1] = -5.0  # an expert that nobody chooses
    gate_row = (rng.standard_normal(width) * 2 / np.sqrt(width)).astype(np.float32) if with_shared else None
    gate_up = (rng.standard_normal((experts, 2 * ff, width)) / np.sqrt(width)).astype(np.float32)
    down = (rng.standard_normal((experts, width, ff)) / np.sqrt(ff)).astype(np.float32)
    shared = rng.standard_normal((rows, width)).astype(np.float32) if with_shared else None
    xr = rounded(x, dtype)
    want, picks, weights, gates = plain_experts(xr, rounded(gate_up, dtype), rounded(down, dtype), router.astype(np.float64),
                                                correction.astype(np.float64), None if gate_row is None else gate_row.astype(np.float64),
                                                None if shared is None else rounded(shared, dtype), top, 1.3)
    xd = dev(x, TORCH[dtype])
    chosen, w, g = ops.route_top_k(xd, dev(router), dev(correction), None if gate_row is None else dev(gate_row), top=top, route_scale=1.3)
    np.testing.assert_array_equal(chosen.cpu().numpy(), picks)
    np.testing.assert_allclose(w.cpu().numpy(), weights, rtol=0, atol=2e-6)
    if with_shared:
        np.testing.assert_allclose(g.cpu().numpy(), gates, rtol=0, atol=2e-6)
    if experts > 2:
        assert not (picks == 1).any()
    sd = None if shared is None else dev(shared, TORCH[dtype])
    forms = [ops.experts_few_rows, ops.experts_grouped]
    if ops.experts_by_expert_take(xd, dev(gate_up, TORCH[dtype])):
        # (16 rows of an expert a pass, and the tiles of 64 rows x 64 features that prompts take)
        forms += [lambda *a: ops.experts_by_expert(*a, many_rows=False), lambda *a: ops.experts_by_expert(*a, many_rows=True)]
    assert len(forms) == 4 or width % 8 or ff % 8
    for form in forms:
        got = form(xd, dev(gate_up, TORCH[dtype]), dev(down, TORCH[dtype]), chosen, w, sd, g).float().cpu().numpy()
        np.testing.assert_allclose(got, want, rtol=0, atol=tolerance(dtype, 8) * max(1.0, np.abs(want).max()))


# ---------------------------------------------------------------------------------------------
# each mixer and each feed-forward alone in a one-layer model
# ---------------------------------------------------------------------------------------------

ALONE = {
    "attention": tk.attention(4, 2, 16, 24, 0.9, window=20, softcap=3.0, v_mix=True),
    "attention_plain": tk.attention(3, None, 10, 6, 1.1),
    "latent": tk.latent(3, 10, 6, 14, 22, 18, 0.8, 50.0, window=13),
    "latent_no_window": tk.latent(2, 4, 4, 6, 10, 12, 1.0, 1000.0),
    "experts": tk.attention(2, 2, 8, 8, 1.0, mlp=tk.moe(24, 5, 3, identity=2, scale=1.4, shared=20)),
    "dense": tk.attention(2, 1, 8, 8, 1.0, window=2, mlp=tk.dense(50)),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("part", sorted(ALONE))
def test_each_part_alone_whole_and_token_by_token(tmp_path, dtype, part):
    from mini_infer_amd.engine import StepEntry

    cfg = tk.config(90, 48, [ALONE[part]], eps=1e-5, alpha=1.3, pairs=(29, 7, 3))
    weights = tk.make_weights(cfg, seed=len(part), steady_choice=dtype == "bfloat16")
    folder = tk.write_model_dir(tmp_path / "m", cfg, weights)
    tokens = tk.random_tokens(cfg, 45, seed=9)
    want = oracle(f"{part}-{dtype}", cfg, weights, tokens)
    runner = runner_for(folder, dtype, 8, pages=12, seats=2)
    whole = runner.step([StepEntry("w", tokens, list(range(45)))]).cpu().numpy()
    # (one layer, 45 tokens: the yardstick's largest error is the largest of few draws, so it gets more room)
    assert_close(whole, want, dtype, f"{part} whole", bf16_max_factor=3.0)
    one_by_one = np.concatenate([runner.step([StepEntry("d", [t], [0])]).cpu().numpy() for t in tokens])
    assert_close(one_by_one, want, dtype, f"{part} token by token", bf16_max_factor=3.0)


# ---------------------------------------------------------------------------------------------
# whole models under every kind of schedule
# ---------------------------------------------------------------------------------------------

LENGTHS = {"A": (70, 41, 9, 33, 58, 1), "B": (45, 64, 17, 2, 39), "C": (130, 40, 77, 5), "D": (50, 21, 36, 3, 44)}


def requests_of(name, cfg):
    return {f"{name}{i}": tk.random_tokens(cfg, n, seed=100 * len(name) + 7 * i + n) for i, n in enumerate(LENGTHS[name])}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(tk.CONFIGS))
@pytest.mark.parametrize("family", ["whole", "decode", "portions", "mixed"])
def test_logits_do_not_depend_on_the_schedule(folders, name, dtype, family):
    """Whole prompts; a prompt and then its last tokens one by one (windows pass over decoded
    tokens); portions down to two tokens; up to four live requests of unequal length in one batch,
    in a pool so small that pages and state slots are used again.  Each request is held against
    itself alone."""
    name, cfg, block, weights, folder = folders[name, dtype]
    requests = requests_of(name[0], cfg)
    schedule = {
        "whole": lambda: ru.schedule_whole(requests),
        "decode": lambda: ru.schedule_prefill_then_decode(requests, tail=36),
        "portions": lambda: ru.schedule_portions(requests, seed=3),
        "mixed": lambda: ru.schedule_mixed(requests, seed=5, max_live=4, tail=12),
    }[family]()
    pages = ru.peak_pages(requests, schedule, block)
    runner = runner_for(folder, dtype, block, pages=pages, seats=4 if family == "mixed" else 1)
    got = ru.run_schedule(runner, requests, schedule)
    for rid, tokens in requests.items():
        assert_close(got[rid], oracle(name, cfg, weights, tokens), dtype, f"{name} {family} {rid}")
    runner.cache.check()
    assert runner.cache.states.num_free == runner.cache.states.max_requests
    assert runner.num_free_blocks() == pages


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_experts_sorted_by_expert_inside_whole_models(folders, dtype):
    """The form for many rows, forced on a tiny model: whole prompts side by side and portions."""
    from mini_infer_amd.engine import StepEntry
    from mini_infer_amd.parts.feed_forward import RoutedExperts

    name, cfg, block, weights, folder = folders["A", dtype]
    first, second = tk.random_tokens(cfg, 50, seed=21), tk.random_tokens(cfg, 23, seed=22)
    runner = runner_for(folder, dtype, block, pages=8, seats=2, graphs=False)
    forced = [b.feed_forward for b in runner.model.blocks if isinstance(b.feed_forward, RoutedExperts)]
    assert len(forced) == 2
    for part in forced:
        part.force_form = "grouped"
    both = runner.step([StepEntry("a", first[:30], list(range(30))), StepEntry("b", second, list(range(23)))]).cpu().numpy()
    rest = runner.step([StepEntry("a", first[30:], list(range(20)))]).cpu().numpy()
    assert_close(np.concatenate([both[:30], rest]), oracle(name, cfg, weights, first), dtype, "sorted by expert, in portions")
    assert_close(both[30:], oracle(name, cfg, weights, second), dtype, "sorted by expert, beside it")


def test_prompts_that_come_whole_write_latent_keys_and_values_out_per_head(folders, monkeypatch):
    """bfloat16, latent attention layers whose head sizes the matrix-core kernel takes, one with a
    window and both with a sink per head: a step in which every request begins takes the expanded
    form (two prompts side by side, neither filling its last page), any other step the folded one;
    both agree with the plain model."""
    from mini_infer_amd.engine import StepEntry
    from mini_infer_amd.parts.latent_attention import LatentAttention

    name, cfg, block, weights, folder = folders["C", "bfloat16"]
    first, second = tk.random_tokens(cfg, 90, seed=11), tk.random_tokens(cfg, 75, seed=12)
    calls = {"expanded": 0}
    original = LatentAttention._forward_expanded

    def counted(self, *args, **kwargs):
        calls["expanded"] += 1
        return original(self, *args, **kwargs)

    monkeypatch.setattr(LatentAttention, "_forward_expanded", counted)
    runner = runner_for(folder, "bfloat16", block, pages=24, seats=2)
    both = runner.step([StepEntry("a", first, list(range(90))), StepEntry("b", second, list(range(75)))]).cpu().numpy()
    assert calls["expanded"] == 2
    assert_close(both[:90], oracle(name, cfg, weights, first), "bfloat16", "expanded form")
    assert_close(both[90:], oracle(name, cfg, weights, second), "bfloat16", "beside it")
    runner.free_request("a"), runner.free_request("b")
    half = runner.step([StepEntry("c", first[:64], list(range(64)))]).cpu().numpy()
    rest = runner.step([StepEntry("c", first[64:], list(range(26)))]).cpu().numpy()
    assert calls["expanded"] == 4
    assert_close(np.concatenate([half, rest]), oracle(name, cfg, weights, first), "bfloat16", "expanded, then folded")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_slot_and_pages_used_again_start_clean(folders, dtype):
    """One seat, pages for one request: the second request gets the first one's slot (with the
    first one's last token in it) and pages."""
    from mini_infer_amd.engine import StepEntry

    name, cfg, block, weights, folder = folders["A", dtype]
    first, second = tk.random_tokens(cfg, 30, seed=1), tk.random_tokens(cfg, 26, seed=2)
    runner = runner_for(folder, dtype, block, pages=2, seats=1)
    runner.step([StepEntry("a", first, [])])
    slot = runner.cache.state_slot("a")
    runner.free_request("a")
    got = runner.step([StepEntry("b", second[:2], [0, 1])]).cpu().numpy()
    assert runner.cache.state_slot("b") == slot
    got = np.concatenate([got, runner.step([StepEntry("b", second[2:], list(range(24)))]).cpu().numpy()])
    assert_close(got, oracle(name, cfg, weights, second), dtype, "second owner of a slot")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_through_recorded_steps_with_windows_passing_over_decoded_tokens(folders, dtype):
    """Two requests decoded side by side for 150 steps after prompts of 210 and 7 tokens, across
    many page borders and several window lengths; the single-token steps are replayed graphs."""
    from mini_infer_amd.engine import StepEntry

    name, cfg, block, weights, folder = folders["A", dtype]
    requests = {"x": tk.random_tokens(cfg, 360, seed=31), "y": tk.random_tokens(cfg, 157, seed=32)}
    runner = runner_for(folder, dtype, block, pages=34, seats=2)
    got = {rid: [] for rid in requests}
    both = runner.step([StepEntry("x", requests["x"][:210], list(range(210))), StepEntry("y", requests["y"][:7], list(range(7)))]).cpu().numpy()
    got["x"].append(both[:210])
    got["y"].append(both[210:])
    for k in range(150):
        logits = runner.step([StepEntry("x", [requests["x"][210 + k]], [0]), StepEntry("y", [requests["y"][7 + k]], [0])]).cpu().numpy()
        got["x"].append(logits[:1])
        got["y"].append(logits[1:])
    assert runner.decode_graphs is not None and runner.decode_graphs.replays == 150
    for rid, tokens in requests.items():
        assert_close(np.concatenate(got[rid]), oracle(name, cfg, weights, tokens), dtype, f"long decoding {rid}")


def widened(cfg, layer, by):
    other = copy.deepcopy(cfg)
    other["layers"][layer]["mixer"]["mask"]["size"] += by
    return other


def test_every_window_ends_where_it_should_beside_page_borders(folders):
    """Pages of 4 and windows of 4, 5, 8 and 3: the engine agrees with the plain model of these
    windows, in a whole prompt, in portions of two and token by token, and is far from the plain
    models whose window in any one layer is a key longer or shorter."""
    from mini_infer_amd.engine import StepEntry

    _, cfg, block, weights, folder = folders["D", "float32"]
    tokens = tk.random_tokens(cfg, 40, seed=77)
    wide = {k: v.astype(np.float64) for k, v in weights.items()}
    want = pk.logits(cfg, wide, tokens)
    runner = runner_for(folder, "float32", block, pages=12, seats=1)
    runs = {
        "whole": [tokens],
        "pairs": [tokens[i:i + 2] for i in range(0, 40, 2)],
        "decoded": [tokens[:3]] + [[t] for t in tokens[3:]],
    }
    for how, portions in runs.items():
        got = np.concatenate([runner.step([StepEntry(how, part, list(range(len(part))))]).cpu().numpy() for part in portions])
        runner.free_request(how)
        assert np.abs(got - want).max() < ru.FP32_TOL, how
        for layer in range(len(cfg["layers"])):
            for by in (-1, 1):
                if cfg["layers"][layer]["mixer"]["mask"]["size"] + by < 1:
                    continue
                other = pk.logits(widened(cfg, layer, by), wide, tokens)
                assert np.abs(other - want).max() > 100 * ru.FP32_TOL  # the test can tell
                assert np.abs(got - other).max() > 100 * ru.FP32_TOL, f"{how}: window of layer {layer} off by {by}"


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_llm_and_the_scheduler(folders, name):
    """Five prompts for two seats, prompts cut into portions of 8 under a 20-token budget: every
    generated token is the plain model's greedy choice."""
    from mini_infer_amd.engine.llm import LLM

    _, cfg, block, weights, folder = folders[name, "float32"]
    wide = {k: v.astype(np.float64) for k, v in weights.items()}
    lengths, new_tokens = (5, 19, 33, 2, 11), 9
    prompts = [tk.random_tokens(cfg, n, seed=300 + n) for n in lengths]
    llm = LLM(folder, dtype="float32", num_blocks=12, block_size=block, max_concurrent=2, max_num_batched_tokens=20, chunk_size=8)
    results = llm.generate(prompts, max_tokens=new_tokens)
    for prompt, result in zip(prompts, results):
        sequence = list(prompt)
        for _ in range(new_tokens):
            sequence.append(pk.greedy(pk.logits(cfg, wide, sequence)[-1]))
        assert result.tokens == sequence[len(prompt):] and result.finish_reason == "length"
    assert llm.runner.cache.states.num_free == 2
    llm.runner.cache.check()


def test_the_command_line_writes_random_weights_and_generates_greedily_and_by_seeded_sampling(tmp_path, capsys):
    """`random-weights` from a config.json, then `generate`: greedy twice the same, sampled with one seed
    twice the same and (at this temperature) different from greedy."""
    from mini_infer_amd.__main__ import main

    cfg, block = tk.CONFIGS["A"]
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    assert main(["random-weights", "--config", str(tmp_path / "config.json"), "--seed", "3", "--out", str(tmp_path / "m"),
                 "--std", "0.3", "--norm-jitter", "0.1"]) == 0
    capsys.readouterr()

    def generate(*extra):
        assert main(["generate", "--model", str(tmp_path / "m"), "--prompt-ids", "5 9 100 3 77", "--prompt-ids", "1,2",
                     "--max-tokens", "12", "--num-blocks", "16", "--block-size", str(block), "--max-concurrent", "2",
                     "--ignore-eos", *extra]) == 0
        lines = [json.loads(line) for line in capsys.readouterr().out.strip().splitlines()]
        assert [line["prompt_tokens"] for line in lines] == [5, 2] and all(len(line["tokens"]) == 12 for line in lines)
        return [line["tokens"] for line in lines]

    greedy = generate()
    assert generate() == greedy
    sampled = generate("--temperature", "1.5", "--top-k", "40", "--top-p", "0.95", "--seed", "11")
    assert generate("--temperature", "1.5", "--top-k", "40", "--top-p", "0.95", "--seed", "11") == sampled
    assert sampled != greedy and all(0 <= t < cfg["vocab"] for tokens in sampled for t in tokens)


def test_the_replay_program_runs_a_trace_of_this_design(folders, tmp_path):
    from mini_infer_amd.engine import replay, trace

    name, cfg, block, weights, folder = folders["B", "float32"]
    requests = {f"t{i}": tk.random_tokens(cfg, n, seed=i) for i, n in enumerate((70, 41, 9, 33, 58))}
    schedule = trace.make_schedule("mixed", requests, seed=1, tail=10)
    lines = trace.to_trace_lines(requests, schedule)
    limit = trace.peak_pages(requests, schedule, 64) * 64
    args = replay.build_parser().parse_args(["--model", str(folder), "--dtype", "float32", "--out", str(tmp_path / "out"),
                                             "--max-tokens", str(limit)])
    said = io.StringIO()
    assert replay.run(args, lines=lines, out=said) == 0
    assert said.getvalue().split() == [w for n in range(len(lines)) for w in ("done", str(n))]
    fed = {rid: 0 for rid in requests}
    for number, line in enumerate(lines):
        step = json.loads(line)
        got = np.fromfile(tmp_path / "out" / f"{number}.f32", dtype="<f4").reshape(-1, cfg["vocab"])
        at = 0
        for entry in step["entries"]:
            n, rid = len(entry["tokens"]), entry["id"]
            whole = oracle(name, cfg, weights, requests[rid])
            want = whole[slice(fed[rid], fed[rid] + n)]
            want.moved_by_float32 = whole.moved_by_float32
            assert_close(got[at: at + n], want, "float32", f"trace step {number} {rid}")
            fed[rid] += n
            at += n

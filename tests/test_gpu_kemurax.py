"""Kemurax on the GPU against the plain model (`plain_kemurax`, NumPy float64): every kernel of
its own alone, each mixer alone in a one-layer model, then whole models of several tiny
configurations under every kind of schedule, in the 32-bit engine and in bfloat16 (held against
the plain model with bfloat16 storage as a yardstick)."""

import io
import json

import numpy as np
import pytest
import torch

import plain_kemurax as pk
import replay_util as ru
import tiny_kemurax as tk

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
    return np.asarray(values, dtype=np.float64) if dtype == "float32" else pk.bf16_round(values)


def tolerance(dtype, scale=1.0):
    return (2e-6 if dtype == "float32" else 1.2e-2) * scale


_ORACLES: dict = {}
# Yardsticks, as for the other designs: the plain model with every stored tensor rounded (to
# bfloat16, to float32) and all arithmetic exact shows how far storage alone moves the logits of
# this very input.  The 32-bit engine also sums in float32 and keeps its recurrent states in
# float32 over hundreds of tokens, and the logits of these tiny models reach 30 to 150, so its
# limit is the larger of the fixed one and eight times the float32 yardstick (measured, where the
# fixed one is passed: up to 5.4 times); a mechanism left out moves these logits by more than 1e-2.  In bfloat16 the worst
# logit of a short request may lie 2.5 times as far as the yardstick's worst (measured: up to
# 2.2); the limit on the 99th percentile is the common one.
F32_YARD_FACTOR = 8.0
BF16_MAX_FACTOR = 2.5


def float32_round(values):
    return np.asarray(values, dtype=np.float32).astype(np.float64)


class Want(ru.Oracle):
    def __init__(self, exact, rounded, yard=None, yard32: float = 0.0):
        super().__init__(exact, rounded, yard)
        self.yard32 = yard32

    def __getitem__(self, rows):
        return Want(self.exact[rows], self.rounded[rows], (self.yard_max, self.yard_p99), self.yard32)


def oracle(name, cfg, weights, tokens) -> Want:
    key = (name, tuple(tokens))
    if key not in _ORACLES:
        wide = {k: v.astype(np.float64) for k, v in weights.items()}
        exact = pk.logits(cfg, wide, tokens)
        in_float32 = pk.logits(cfg, wide, tokens, store=float32_round)
        _ORACLES[key] = Want(exact, pk.logits(cfg, wide, tokens, store=pk.bf16_round), yard32=float(np.abs(in_float32 - exact).max()))
    return _ORACLES[key]


def assert_close(got, want: Want, dtype: str, what: str = "") -> None:
    ru.assert_close(got, want, dtype, what, fp32_tol=max(ru.FP32_TOL, F32_YARD_FACTOR * want.yard32), bf16_max_factor=BF16_MAX_FACTOR)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, (cfg, block) in tk.CONFIGS.items():
        weights = tk.make_weights(cfg, seed=40 + len(out))
        out[name] = (cfg, block, weights, tk.write_model_dir(tmp_path_factory.mktemp("kemurax") / name, cfg, weights))
    return out


def runner_for(folder, dtype, block, pages=64, seats=4, graphs=True):
    from mini_infer_amd.engine import ModelRunner

    return ModelRunner.from_pretrained(folder, dtype=dtype, num_blocks=pages, block_size=block, max_concurrent=seats,
                                       cuda_graph=graphs)


# ---------------------------------------------------------------------------------------------
# each kernel alone
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width, copies", [(10, 1), (64, 3), (2500, 2), (130, 8)])
def test_the_normed_embedding_starts_every_copy_of_the_stream(dtype, width, copies):
    from mini_infer_amd import ops

    rng = np.random.default_rng(width)
    table = rng.standard_normal((37, width)).astype(np.float32)
    factor = rng.uniform(0.5, 1.5, width).astype(np.float32)
    ids = [5, 0, 36, 5, 17]
    got = ops.embed_norm_streams(dev(table, TORCH[dtype]), ints(ids), dev(factor), copies, 1e-5).cpu().numpy()
    rows = rounded(table, dtype)[ids]
    want = pk.rms_unit(rows, 1e-5) * factor
    assert got.shape == (5, copies, width)
    for c in range(copies):
        np.testing.assert_allclose(got[:, c], want, rtol=0, atol=2e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width, copies", [(10, 1), (64, 3), (2500, 2), (130, 8)])
@pytest.mark.parametrize("parts", ["a", "ab", "none"])
def test_the_streams_write_the_next_read_and_its_norm_are_one_launch(dtype, width, copies, parts):
    from mini_infer_amd import ops

    rng = np.random.default_rng(width + copies + len(parts))
    rows, eps = 7, 1e-5
    xs = rng.standard_normal((rows, copies, width)).astype(np.float32)
    a = rng.standard_normal((rows, width)).astype(np.float32)
    b = rng.standard_normal((rows, width)).astype(np.float32)
    mix = rng.standard_normal((copies, copies)).astype(np.float32)
    out_vec, read = rng.standard_normal(copies).astype(np.float32), rng.standard_normal(copies).astype(np.float32)
    factor = rng.uniform(0.5, 1.5, width).astype(np.float32)
    write, new = None, xs.astype(np.float64)
    if parts != "none":
        y = 0.7 * rounded(a, dtype) + (1.3 * rounded(b, dtype) if parts == "ab" else 0.0)
        # streams as the plain model keeps them: [copies, rows, width]
        new = pk.hyper_write(np.swapaxes(new, 0, 1), y, {"mix": mix.astype(np.float64), "out": out_vec.astype(np.float64)}, "")
        new = np.swapaxes(new, 0, 1)
        write = ops.StreamsWrite(dev(a, TORCH[dtype]), dev(mix), dev(out_vec), b=dev(b, TORCH[dtype]) if parts == "ab" else None,
                                 scale_a=0.7, scale_b=1.3)
    for reader in (read, None):  # (None: the plain sum of the copies, how the model ends)
        u = new.sum(1) if reader is None else np.einsum("s,tsw->tw", reader.astype(np.float64), new)
        normed = pk.rms_unit(u, eps) * factor
        stream = dev(xs)
        got = ops.streams_update_norm(write, stream, None if reader is None else dev(reader), dev(factor), eps, TORCH[dtype])
        np.testing.assert_allclose(stream.cpu().numpy(), new, rtol=0, atol=4e-6 * copies)
        np.testing.assert_allclose(got.float().cpu().numpy(), normed, rtol=0, atol=tolerance(dtype, 4))
        # at chosen rows only: the stream stays as it was
        stream = dev(xs)
        some = ops.streams_update_norm(write, stream, None if reader is None else dev(reader), dev(factor), eps, TORCH[dtype],
                                       rows=ints([5, 0]))
        np.testing.assert_array_equal(stream.cpu().numpy(), xs)
        np.testing.assert_allclose(some.float().cpu().numpy(), normed[[5, 0]], rtol=0, atol=tolerance(dtype, 4))
    if write is not None:  # the write alone
        stream = dev(xs)
        write.apply(stream)
        np.testing.assert_allclose(stream.cpu().numpy(), new, rtol=0, atol=4e-6 * copies)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("activation", ["silu", "gelu_tanh", "logistic"])
def test_the_gates_that_multiply_inner_rows(dtype, activation):
    from mini_infer_amd import ops

    rng = np.random.default_rng(len(activation))
    both = (rng.standard_normal((9, 2 * 70 + 3)) * 2.5).astype(np.float32)  # (column ranges of wider rows)
    a, b = rounded(both[:, :70], dtype), rounded(both[:, 70:140], dtype)
    want = {"silu": pk.silu, "gelu_tanh": pk.gelu_tanh, "logistic": pk.logistic}[activation](a) * b
    t = dev(both, TORCH[dtype])
    got = ops.gated_mul(t[:, :70], t[:, 70:140], activation)
    np.testing.assert_allclose(got.float().cpu().numpy(), want, rtol=0, atol=tolerance(dtype, 8))


@pytest.mark.parametrize("rows, inter, k", [(1, 24, 64), (8, 70, 256), (16, 320, 256), (17, 48, 96), (32, 130, 512), (33, 24, 64)])
def test_gated_product_with_the_tanh_gelu_in_its_last_step(rows, inter, k):
    """Few bfloat16 rows: one kernel, equal to the product followed by the gate's kernel up to the
    last bit of a bfloat16 value (33 rows: the two in turn, on both sides)."""
    from mini_infer_amd import ops

    rng = np.random.default_rng(rows * inter)
    x = dev(rng.standard_normal((rows, k)).astype(np.float32), torch.bfloat16)
    weight = dev((rng.standard_normal((2 * inter, k)) / np.sqrt(k) * 2.5).astype(np.float32), torch.bfloat16)
    fused = ops.linear_geglu(x, weight)
    both = ops.linear(x, weight)
    in_turn = ops.gated_mul(both[:, :inter], both[:, inter:], "gelu_tanh")
    np.testing.assert_allclose(fused.float().cpu().numpy(), in_turn.float().cpu().numpy(), rtol=2 ** -7, atol=1e-6)
    z = (x.double() @ weight.double().T).cpu().numpy()
    np.testing.assert_allclose(fused.float().cpu().numpy(), pk.gelu_tanh(z[:, :inter]) * z[:, inter:], rtol=2 ** -6, atol=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("channels, taps", [(10, 1), (70, 2), (256, 4), (33, 7)])
def test_the_short_convolution_with_a_bias_carries_each_requests_tail(dtype, channels, taps):
    """Four steps over four requests of unequal length, among them portions shorter than the
    tail, a request that brings nothing, steps of one launch and of two."""
    from mini_infer_amd import ops

    rng = np.random.default_rng(channels)
    weight = (rng.standard_normal((channels, taps)) * 0.6).astype(np.float32)
    bias = rng.standard_normal(channels).astype(np.float32)
    tails = torch.zeros((6, max(taps - 1, 0), channels), dtype=TORCH[dtype], device=DEV)
    plain = {slot: np.zeros((taps - 1, channels)) for slot in range(5)}
    for step, lengths in enumerate([(1, 9, 0, 2), (2, 1, 5, 1), (80, 1, 1, 3), (30, 2, 70, 1)]):
        slots = [3, 0, 4, 1]
        x = rng.standard_normal((sum(lengths), channels + 5)).astype(np.float32)
        cu = np.concatenate([[0], np.cumsum(lengths)])
        request_of = np.repeat(np.arange(4), lengths)
        got = ops.short_conv(dev(x, TORCH[dtype]), channels, dev(weight), tails, ints(cu), ints(slots), ints(request_of), bias=dev(bias))
        for r, slot in enumerate(slots):
            z = np.concatenate([plain[slot], rounded(x[cu[r]:cu[r + 1], :channels], dtype)])
            y = np.stack([np.einsum("jc,cj->c", z[t:t + taps], weight.astype(np.float64)) + bias for t in range(lengths[r])]) \
                if lengths[r] else np.zeros((0, channels))
            if taps > 1:
                plain[slot] = z[len(z) - (taps - 1):]
                np.testing.assert_array_equal(tails[slot].float().cpu().numpy(), plain[slot])
            np.testing.assert_allclose(got[cu[r]:cu[r + 1]].float().cpu().numpy(), pk.silu(y), rtol=0, atol=tolerance(dtype, 4),
                                       err_msg=f"step {step} request {r}")


def plain_scan(q, k, v, a, S, scale_v=None, skip=None):
    """S <- diag(a_t) S + k_t v_t^T; o_t = S^T q_t (+ skip v_t) for one head; S [dim, vdim] advanced in place."""
    out = np.empty((len(q), S.shape[1]))
    for t in range(len(q)):
        vt = v[t] if scale_v is None else v[t] * scale_v[t]
        S[:] = a[t][:, None] * S + np.outer(k[t], vt)
        out[t] = S.T @ q[t] + (0.0 if skip is None else skip * v[t])
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, dim, vdim", [(3, 12, 20), (2, 7, 9), (4, 64, 64), (1, 128, 130), (2, 200, 24), (2, 32, 64)])
def test_the_recurrence_with_a_decay_per_key_channel(dtype, heads, dim, vdim):
    """Three steps over three requests in scattered slots (a long portion, single tokens, a
    request that sits a step out and one that brings nothing): read-outs and the state left
    behind against the token loop."""
    from mini_infer_amd import ops

    rng = np.random.default_rng(dim)
    tau, q_scale = 4.0, dim ** -0.5
    bias = (rng.standard_normal(heads * dim) + 1.0).astype(np.float32)
    pad = ops.decay_state_shape(heads, dim, vdim)[2]
    state = torch.zeros((6, heads, vdim, pad), dtype=torch.float32, device=DEV)
    plain = {slot: np.zeros((heads, dim, vdim)) for slot in range(5)}
    for step, (slots, lengths) in enumerate([((4, 1, 2), (45, 1, 3)), ((1, 4), (1, 1)), ((2, 4, 1), (0, 19, 2))]):
        tokens = sum(lengths)
        width = 2 * heads * dim + heads * vdim + 3
        rows = rng.standard_normal((tokens, width)).astype(np.float32)
        logits = (rng.standard_normal((tokens, heads * dim)) * 2.0).astype(np.float32)
        cu = np.concatenate([[0], np.cumsum(lengths)])
        r = dev(rows, TORCH[dtype])
        got = ops.decay_scan(r, 0, r, heads * dim, r, 2 * heads * dim, dev(logits, TORCH[dtype]), 0, dev(bias), state, ints(cu),
                             ints(slots), heads=heads, groups=heads, dim=dim, vdim=vdim, per_head=False, inv_tau=1.0 / tau,
                             q_scale=q_scale).cpu().numpy()
        rr = rounded(rows, dtype)
        alpha = pk.logistic(rounded(logits, dtype) + bias) ** (1.0 / tau)
        for i, slot in enumerate(slots):
            span = slice(cu[i], cu[i + 1])
            for h in range(heads):
                want = plain_scan(rr[span, h * dim:(h + 1) * dim] * q_scale, rr[span, (heads + h) * dim:(heads + h + 1) * dim],
                                  rr[span, 2 * heads * dim + h * vdim: 2 * heads * dim + (h + 1) * vdim],
                                  alpha[span, h * dim:(h + 1) * dim], plain[slot][h])
                np.testing.assert_allclose(got[span, h * vdim:(h + 1) * vdim], want, rtol=0, atol=3e-5 * dim ** 0.5,
                                           err_msg=f"step {step} slot {slot} head {h}")
    kept = state.cpu().numpy()
    for slot in range(5):  # stored transposed and padded; slot 0 and 3 never touched
        np.testing.assert_allclose(kept[slot, :, :, :dim], np.swapaxes(plain[slot], 1, 2), rtol=0, atol=3e-5 * dim ** 0.5)
    assert np.abs(kept[0]).max() == 0 and np.abs(kept[3]).max() == 0 and np.abs(kept[4]).max() > 0.1


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, groups, state_size, vdim", [(4, 2, 10, 12), (3, 3, 9, 7), (6, 1, 32, 32), (8, 2, 64, 32), (2, 1, 256, 64),
                                                             (4, 4, 128, 64)])
def test_the_recurrence_with_a_decay_per_head_and_shared_rows_per_group(dtype, heads, groups, state_size, vdim):
    from mini_infer_amd import ops

    rng = np.random.default_rng(state_size + heads)
    step_bias = rng.standard_normal(heads).astype(np.float32)
    rate = rng.uniform(-2.5, 0.5, heads).astype(np.float32)
    skip = rng.standard_normal(heads).astype(np.float32)
    pad = ops.decay_state_shape(heads, state_size, vdim)[2]
    state = torch.zeros((5, heads, vdim, pad), dtype=torch.float32, device=DEV)
    plain = {slot: np.zeros((heads, state_size, vdim)) for slot in range(4)}
    inner, span_bc = heads * vdim, groups * state_size
    for step, (slots, lengths) in enumerate([((3, 0), (40, 2)), ((0, 3), (1, 1)), ((2, 3, 0), (5, 0, 17))]):
        tokens = sum(lengths)
        conv = rng.standard_normal((tokens, inner + 2 * span_bc)).astype(np.float32)  # [x | B | C]
        raw = (rng.standard_normal((tokens, heads + 2)) * 2.0).astype(np.float32)  # (raw step sizes from column 2 on)
        cu = np.concatenate([[0], np.cumsum(lengths)])
        c = dev(conv, TORCH[dtype])
        got = ops.decay_scan(c, inner + span_bc, c, inner, c, 0, dev(raw, TORCH[dtype]), 2, dev(step_bias), state, ints(cu), ints(slots),
                             heads=heads, groups=groups, dim=state_size, vdim=vdim, per_head=True, rate=dev(rate), skip=dev(skip),
                             ).cpu().numpy()
        cc = rounded(conv, dtype)
        dt = pk.softplus(rounded(raw, dtype)[:, 2:] + step_bias)
        for i, slot in enumerate(slots):
            rows = slice(cu[i], cu[i + 1])
            for h in range(heads):
                g = h // (heads // groups)
                decay = np.exp(-np.exp(float(rate[h])) * dt[rows, h])
                want = plain_scan(cc[rows, inner + span_bc + g * state_size: inner + span_bc + (g + 1) * state_size],
                                  cc[rows, inner + g * state_size: inner + (g + 1) * state_size], cc[rows, h * vdim:(h + 1) * vdim],
                                  np.repeat(decay[:, None], state_size, 1), plain[slot][h], scale_v=dt[rows, h], skip=float(skip[h]))
                np.testing.assert_allclose(got[rows, h * vdim:(h + 1) * vdim], want, rtol=0, atol=5e-5 * state_size ** 0.5,
                                           err_msg=f"step {step} slot {slot} head {h}")
    kept = state.cpu().numpy()
    for slot in range(4):
        np.testing.assert_allclose(kept[slot, :, :, :state_size], np.swapaxes(plain[slot], 1, 2), rtol=0, atol=5e-5 * state_size ** 0.5)
    assert np.abs(kept[1]).max() == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width, group, period, gate_first", [(60, 20, 20, False), (27, 9, 9, False), (48, 24, 48, True), (20, 4, 20, True),
                                                              (512, 512, 512, True), (1024, 128, 128, False)])
def test_norm_and_gate_behind_a_recurrences_read_outs(dtype, width, group, period, gate_first):
    """A weight shared by the groups (per head) or one over the whole row; the gate before the
    norm or after it."""
    from mini_infer_amd import ops

    rng = np.random.default_rng(width)
    o = (rng.standard_normal((6, width)) * 3.0).astype(np.float32)
    gate = rng.standard_normal((6, width + 7)).astype(np.float32)
    weight = rng.uniform(0.5, 1.5, period).astype(np.float32)
    g = pk.silu(rounded(gate[:, :width], dtype))
    w = np.tile(weight.astype(np.float64), width // period)
    y = o.astype(np.float64) * g if gate_first else o.astype(np.float64)
    y = pk.rms_unit(y.reshape(6, width // group, group), 1e-5).reshape(6, width) * w
    want = y if gate_first else y * g
    got = ops.readout_gate_norm(dev(o), dev(gate, TORCH[dtype]), dev(weight), group_width=group, gate_first=gate_first, eps=1e-5)
    np.testing.assert_allclose(got.float().cpu().numpy(), want, rtol=0, atol=tolerance(dtype, 6))
    other = y * g if gate_first else pk.rms_unit((o * g).reshape(6, width // group, group), 1e-5).reshape(6, width) * w
    assert np.abs(other - want).max() > 0.05  # (the order of gate and norm shows)


def paged(rows: np.ndarray, page_size: int, order: list[int], dtype, transposed=False) -> torch.Tensor:
    """[tokens, heads, dim] laid into pages [num_pages, heads, page_size, dim] (or [.., dim, page_size]),
    page i of the request at page id order[i]."""
    tokens, heads, dim = rows.shape
    pages = np.zeros((max(order) + 1, heads, page_size, dim), dtype=np.float32)
    for t in range(tokens):
        pages[order[t // page_size], :, t % page_size] = rows[t]
    if transposed:
        pages = np.ascontiguousarray(np.swapaxes(pages, 2, 3))
    return dev(pages, TORCH[dtype])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, rot, page", [(4, 2, 16, 8, 8), (3, 3, 10, 10, 4), (8, 1, 64, 64, 16), (2, 2, 128, 32, 16),
                                                             (5, 1, 6, 2, 8)])
def test_heads_normed_one_by_one_then_rotated_and_written_into_pages(dtype, heads, kv_heads, dim, rot, page):
    from mini_infer_amd import ops

    rng = np.random.default_rng(dim + rot)
    tokens, eps, vdim = 11, 1e-5, dim + 2
    width = (heads + kv_heads) * dim + kv_heads * vdim + 5
    rows = (rng.standard_normal((tokens, width)) * 2.0).astype(np.float32)
    qw, kw = rng.uniform(0.5, 1.5, dim).astype(np.float32), rng.uniform(0.5, 1.5, dim).astype(np.float32)
    positions = np.arange(40, 40 + tokens)
    freq = 50.0 ** (-2.0 * np.arange(rot // 2) / rot)
    angles = positions[:, None] * freq
    slots = rng.permutation(5 * page)[:tokens].astype(np.int64)
    slots[4] = -1  # (a padding row of a recorded step writes nowhere)
    k_pages = torch.zeros((5, kv_heads, page, dim), dtype=TORCH[dtype], device=DEV)
    v_pages = torch.zeros((5, kv_heads, page, vdim), dtype=TORCH[dtype], device=DEV)
    qkv = dev(rows, TORCH[dtype])
    ops.head_norm_rope_kv_write(qkv, dev(np.cos(angles)), dev(np.sin(angles)), ints(slots), k_pages, v_pages, dev(qw), dev(kw), eps,
                                q_heads=heads, kv_heads=kv_heads, head_dim=dim, rotary_dim=rot, v_head_dim=vdim)
    r = rounded(rows, dtype)
    got_q = qkv.float().cpu().numpy()[:, :heads * dim].reshape(tokens, heads, dim)
    got_k = k_pages.float().cpu().numpy().transpose(0, 2, 1, 3).reshape(5 * page, kv_heads, dim)
    got_v = v_pages.float().cpu().numpy().transpose(0, 2, 1, 3).reshape(5 * page, kv_heads, vdim)
    for t in range(tokens):
        for a in range(heads):
            want = pk.rotate(pk.rms_unit(r[t, a * dim:(a + 1) * dim], eps) * qw, int(positions[t]), freq)
            np.testing.assert_allclose(got_q[t, a], want, rtol=0, atol=tolerance(dtype, 4))
        if slots[t] < 0:
            continue
        for a in range(kv_heads):
            at = (heads + a) * dim
            want = pk.rotate(pk.rms_unit(r[t, at:at + dim], eps) * kw, int(positions[t]), freq)
            np.testing.assert_allclose(got_k[slots[t], a], want, rtol=0, atol=tolerance(dtype, 4))
            at = (heads + kv_heads) * dim + a * vdim
            np.testing.assert_array_equal(got_v[slots[t], a], r[t, at:at + vdim])
    assert np.count_nonzero(np.abs(got_k).sum((1, 2))) == tokens - 1


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim, page, chunk", [
    (4, 2, 16, 24, 8, 12), (3, 3, 10, 6, 4, 5), (8, 1, 64, 64, 16, 64), (4, 1, 64, 64, 16, 50), (2, 2, 128, 128, 16, 300),
    (4, 4, 32, 32, 32, 1), (2, 1, 64, 64, 16, 16), (8, 2, 64, 64, 16, 1024), (4, 2, 16, 24, 8, 400),
])
def test_attention_inside_chunks_edges_in_prompts_and_for_decoded_tokens(dtype, heads, kv_heads, dim, vdim, page, chunk):
    """One request of 333 keys in scattered pages.  Queries: a prompt's last portion of 40
    positions (it crosses chunk edges wherever chunks are shorter), and the last position alone
    as a decoded token.  For every query, head 0 is made to single out the first key of the
    query's chunk (just inside) and head 1 the key before it (just outside, with a score that
    would take all the weight if it were seen).  Chunks longer than the request: the first key of
    the sequence, hundreds of positions back, is the one that stands out."""
    from mini_infer_amd import ops

    rng = np.random.default_rng(dim + chunk)
    keys_n, queries_n, scale = 333, 40, 0.5
    k = rng.standard_normal((keys_n, kv_heads, dim)).astype(np.float32)
    v = rng.standard_normal((keys_n, kv_heads, vdim)).astype(np.float32)
    q = rng.standard_normal((queries_n, heads, dim)).astype(np.float32)
    positions = np.arange(keys_n - queries_n, keys_n)
    group = heads // kv_heads
    marks = sorted({(p // chunk) * chunk for p in positions})
    for start in marks:  # chunk starts get keys of their own direction (one per chunk), far longer than the rest
        k[start, 0] = 0.0
        k[start, 0, (start // chunk * 3) % dim] = 12.0
        if start > 0 and heads > 1:
            k[start - 1, 1 // group] = 0.0
            k[start - 1, 1 // group, (start // chunk * 3 + 1) % dim] = 12.0
    for i, p in enumerate(positions):
        start = (p // chunk) * chunk
        q[i, 0] = 0.0
        q[i, 0, (start // chunk * 3) % dim] = 3.0
        if heads > 1 and start > 0:
            q[i, 1] = rng.standard_normal(dim) * 0.3
            q[i, 1, (start // chunk * 3 + 1) % dim] = 3.0
    order = list(rng.permutation(-(-keys_n // page) + 3))[: -(-keys_n // page)]
    kq, vq, qq = rounded(k, dtype), rounded(v, dtype), rounded(q, dtype)
    want = np.zeros((queries_n, heads, vdim))
    on_first = []
    for i, p in enumerate(positions):
        lo = (p // chunk) * chunk
        for a in range(heads):
            s = kq[lo: p + 1, a // group] @ qq[i, a] * scale
            e = np.exp(s - s.max())
            want[i, a] = e @ vq[lo: p + 1, a // group] / e.sum()
            if a == 0:
                on_first.append(e[0] / e.sum())
            if a == 1 and lo > 0:  # what seeing the key before the chunk would make of it
                s2 = kq[lo - 1: p + 1, a // group] @ qq[i, a] * scale
                e2 = np.exp(s2 - s2.max())
                leaked = e2 @ vq[lo - 1: p + 1, a // group] / e2.sum()
                assert e2[0] / e2.sum() > 0.9 and np.abs(leaked - want[i, a]).max() > 0.05
    assert min(on_first) > 0.9 or chunk == 1  # the chunk's first key is what head 0's answer is made of

    def run(rows, transposed):
        n = rows.stop - rows.start
        return ops.paged_attention(
            dev(q[rows].reshape(n, -1), TORCH[dtype]), paged(k, page, order, dtype), paged(v, page, order, dtype, transposed),
            ints(order).view(1, -1), ints([0] * n), ints(positions[rows]), ints([0, n]), [0, n], q_heads=heads, kv_heads=kv_heads,
            head_dim=dim, scale=scale, window=None, max_seq_len=keys_n, v_head_dim=vdim, v_transposed=transposed, chunk=chunk,
        ).float().cpu().numpy().reshape(n, heads, vdim)

    for rows in (slice(0, queries_n), slice(queries_n - 1, queries_n), slice(queries_n - 7, queries_n - 5)):
        np.testing.assert_allclose(run(rows, False), want[rows], rtol=0, atol=tolerance(dtype, 4))
        if ops.mfma_attention_supported(TORCH[dtype], dim, page) and vdim == dim:
            np.testing.assert_allclose(run(rows, True), want[rows], rtol=0, atol=tolerance(dtype, 4))


# ---------------------------------------------------------------------------------------------
# each mixer alone: a model of one layer without a feed-forward
# ---------------------------------------------------------------------------------------------

NO_SSM = tk.state_space(1, 2, 2, 1, 1, 1)
ALONE = {
    "gla": (tk.gla(3, 12, 20, 4.0), None),
    "gla_odd_sizes_tau_one": (tk.gla(3, 7, 9, 1.0), 1),
    "gla_large_heads": (tk.gla(1, 132, 80, 16.0), 2),
    "pair": (tk.parallel(tk.attention(4, 2, 16, 24, 0.8, 12, (100.0, 8), (4.0, 1.0, 4.0, 64)), tk.state_space(4, 12, 10, 2, 3, 2), 0.7, 1.3), 3),
    "pair_attention_only": (tk.parallel(tk.attention(6, 1, 10, 4, 0.9, 7, (20.0, 10)), NO_SSM, 1.0, 0.0), None),
    "pair_state_space_only": (tk.parallel(tk.attention(2, 1, 2, 2, 1.0, 3, (20.0, 2)), tk.state_space(6, 5, 6, 3, 5, 2), 0.0, 1.0), 2),
    "pair_one_tap_one_group": (tk.parallel(tk.attention(2, 2, 8, 8, 1.0, 64, (20.0, 4)), tk.state_space(3, 7, 9, 1, 1, 1), 0.5, 0.5), 1),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mixer", sorted(ALONE))
def test_each_mixer_alone_whole_and_token_by_token(tmp_path, dtype, mixer):
    from mini_infer_amd.engine import StepEntry

    layer, streams = ALONE[mixer]
    cfg = tk.config(90, 48, [layer], eps=1e-5, streams=streams)
    weights = tk.make_weights(cfg, seed=len(mixer))
    folder = tk.write_model_dir(tmp_path / "m", cfg, weights)
    tokens = tk.random_tokens(cfg, 45, seed=9)
    want = oracle(mixer, cfg, weights, tokens)
    runner = runner_for(folder, dtype, 8, pages=12, seats=2)
    whole = runner.step([StepEntry("w", tokens, list(range(45)))]).cpu().numpy()
    assert_close(whole, want, dtype, f"{mixer} whole")
    one_by_one = np.concatenate([runner.step([StepEntry("d", [t], [0])]).cpu().numpy() for t in tokens])
    assert_close(one_by_one, want, dtype, f"{mixer} token by token")


# ---------------------------------------------------------------------------------------------
# whole models under every kind of schedule
# ---------------------------------------------------------------------------------------------

LENGTHS = {"A": (70, 41, 9, 33, 58, 1), "B": (45, 64, 17, 2, 39), "C": (130, 40, 77, 5), "D": (50, 21, 36, 3, 44),
           "E": (90, 35, 66, 3)}


def requests_of(name, cfg):
    return {f"{name}{i}": tk.random_tokens(cfg, n, seed=100 * len(name) + 7 * i + n) for i, n in enumerate(LENGTHS[name])}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(tk.CONFIGS))
@pytest.mark.parametrize("family", ["whole", "decode", "portions", "mixed"])
def test_logits_do_not_depend_on_the_schedule(folders, name, dtype, family):
    """Whole prompts; a prompt and then its last tokens one by one (across chunk edges); portions
    down to two tokens; up to four live requests of unequal length in one batch, in a pool so
    small that pages and state slots are used again.  Each request is held against itself alone."""
    cfg, block, weights, folder = folders[name]
    requests = requests_of(name, cfg)
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
def test_after_every_layer_the_sum_of_the_streams_is_the_plain_models(folders, dtype):
    """The copies of the stream after each layer, read through a hook on the blocks: their sum
    against the plain model's, layer by layer (the last block's write is still pending when it
    returns, so the hook makes it on a copy)."""
    from mini_infer_amd.engine import StepEntry

    cfg, block, weights, folder = folders["A"]
    tokens = tk.random_tokens(cfg, 29, seed=12)
    wide = {k: v.astype(np.float64) for k, v in weights.items()}
    want: list = []
    pk.logits(cfg, wide, tokens, layers_out=want)
    runner = runner_for(folder, dtype, block, pages=4, seats=1, graphs=False)
    seen = []
    for blk in runner.model.blocks:
        original = blk.forward

        def hooked(delta, residual, ctx, cache, writes_cache=True, _original=original):
            pending = _original(delta, residual, ctx, cache, writes_cache)
            copy = residual.clone()
            pending.apply(copy)
            seen.append(copy.sum(1).cpu().numpy())
            return pending

        blk.forward = hooked
    runner.step([StepEntry("r", tokens, [])])
    assert len(seen) == len(want) == 4
    for layer, (got, exact) in enumerate(zip(seen, want)):
        limit = 2e-5 if dtype == "float32" else 0.03 * np.abs(exact).max()
        assert np.abs(got - exact).max() < limit, f"after layer {layer}: {np.abs(got - exact).max():.3e}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_slot_and_pages_used_again_start_clean(folders, dtype):
    """One seat, pages for one request: the second request gets the first one's slot (matrix
    states and convolution tails of every layer) and pages."""
    from mini_infer_amd.engine import StepEntry

    cfg, block, weights, folder = folders["A"]
    first, second = tk.random_tokens(cfg, 30, seed=1), tk.random_tokens(cfg, 26, seed=2)
    runner = runner_for(folder, dtype, block, pages=2, seats=1)
    runner.step([StepEntry("a", first, [])])
    slot = runner.cache.state_slot("a")
    runner.free_request("a")
    got = runner.step([StepEntry("b", second[:2], [0, 1])]).cpu().numpy()
    assert runner.cache.state_slot("b") == slot
    got = np.concatenate([got, runner.step([StepEntry("b", second[2:], list(range(24)))]).cpu().numpy()])
    assert_close(got, oracle("A", cfg, weights, second), dtype, "second owner of a slot")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "E"])
def test_long_decoding_through_recorded_steps_across_many_pages_and_chunks(folders, dtype, name):
    """Two requests decoded side by side for 150 steps after prompts of 210 and 7 tokens; the
    single-token steps are replayed graphs.  (E: one chunk holds everything, so the last tokens
    attend to keys hundreds of positions back, beside a layer with chunks of 30.)"""
    from mini_infer_amd.engine import StepEntry

    cfg, block, weights, folder = folders[name]
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


@pytest.mark.parametrize("name", ["A", "D"])
def test_greedy_generation_through_llm_and_the_scheduler(folders, name):
    """Five prompts for two seats, prompts cut into portions of 8 under a 20-token budget: every
    generated token is the plain model's greedy choice."""
    from mini_infer_amd.engine.llm import LLM

    cfg, block, weights, folder = folders[name]
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

    cfg, block, weights, folder = folders["B"]
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
            want = oracle("B", cfg, weights, requests[rid])[slice(fed[rid], fed[rid] + n)]
            assert_close(got[at: at + n], want, "float32", f"trace step {number} {rid}")
            fed[rid] += n
            at += n

"""Kemurax without a GPU: configuration, the model as data (tensor names, running order, cache
needs), and the plain model against itself (a sequence fed whole and in portions) and against
what each mechanism is meant to do."""

import copy

import numpy as np
import pytest
import torch

import plain_kemurax as pk
import tiny_kemurax as tk
from mini_infer_amd.exceptions import ConfigError
from mini_infer_amd.models import architecture_for


def model_of(cfg, dtype=torch.bfloat16, shapes=None):
    arch = architecture_for(cfg)
    parsed = arch.parse_config(cfg)
    if shapes is not None:
        parsed = arch.with_checkpoint_shapes(parsed, shapes)
    return arch.make_model(parsed, dtype, "cpu")


@pytest.mark.parametrize("name", sorted(tk.CONFIGS))
def test_the_model_asks_for_exactly_the_checkpoints_tensors(name):
    cfg, _ = tk.CONFIGS[name]
    shapes = tk.tensor_shapes(cfg)
    specs = model_of(cfg, shapes=shapes).param_specs()
    assert {k: tuple(v.shape) for k, v in specs.items()} == shapes
    # what enters a recurrence, a norm or the streams stays 32-bit whatever the engine's dtype
    for leaf in ("A_log", "dt_bias", ".D", "mix.norm", "right.norm", "q.norm", "k.norm", "a2.b", "conv", "conv.b", "norm1", "norm2",
                 "hc1.in", "hc1.out", "hc1.mix", "hc2.mix", "embed.norm", "final.norm"):
        assert all(v.dtype == "float32" for k, v in specs.items() if k.endswith(leaf)), leaf


def test_the_width_of_the_decay_projection_comes_from_the_checkpoint():
    cfg, _ = tk.CONFIGS["D"]
    by_default = model_of(cfg).param_specs()
    assert by_default["l0.mix.a1"].shape == (16, 48) and by_default["l0.mix.a2"].shape == (16, 16)
    from_shapes = model_of(cfg, shapes=tk.tensor_shapes(cfg)).param_specs()
    assert from_shapes["l0.mix.a1"].shape == (5, 48) and from_shapes["l1.mix.a2"].shape == (60, 6)


def test_a_layer_without_a_feed_forward_may_still_come_with_its_second_norm_and_vectors():
    cfg, _ = tk.CONFIGS["A"]  # layers 2 and 3 have no feed-forward
    model = model_of(cfg, shapes=tk.tensor_shapes(cfg))
    assert {"l2.norm2", "l2.hc2.in", "l2.hc2.out", "l2.hc2.mix", "l3.norm2"} <= model.optional_names()
    assert not any(name.startswith(("l0.", "l1.")) for name in model.optional_names())
    assert not any(name.startswith("l2.hc2") or name == "l2.norm2" for name in model.param_specs())


def test_cache_needs_pages_for_the_attention_and_state_for_everything_recurrent():
    cfg, block = tk.CONFIGS["A"]
    needs = model_of(cfg, shapes=tk.tensor_shapes(cfg)).cache_needs(block)
    assert len(needs) == 4 and all(need is not None for need in needs)
    assert needs[0].pages is None and needs[0].state.shape == (3, 20, 16) and needs[0].state.dtype == torch.float32
    pair = needs[1]
    assert (pair.pages.num_kv_heads, pair.pages.head_dim, pair.pages.value_dim) == (2, 16, 24)
    assert set(pair.state) == {"right.recurrent", "right.tail"}
    assert pair.state["right.recurrent"].shape == (4, 12, 16) and pair.state["right.recurrent"].dtype == torch.float32
    assert pair.state["right.tail"].shape == (2, 4 * 12 + 2 * 2 * 10) and pair.state["right.tail"].dtype == torch.bfloat16
    one_tap = model_of(tk.CONFIGS["B"][0]).cache_needs(8)[0].state
    assert set(one_tap) == {"right.recurrent"}  # a convolution of one tap has nothing to carry
    assert all(need.pages is None for need in model_of(tk.CONFIGS["D"][0]).cache_needs(4))
    assert model_of(tk.CONFIGS["A"][0], torch.float32).cache_needs(16)[1].state["right.tail"].dtype == torch.float32


def test_the_model_is_made_of_registered_parts_that_other_designs_can_use():
    from mini_infer_amd.registry import BLOCKS, EMBEDDINGS, FEED_FORWARDS, MIXERS, NORMS

    for registry, kind in ((BLOCKS, "hyper_connections"), (NORMS, "streams_rms_norm"), (EMBEDDINGS, "normed_streams_embedding"),
                           (MIXERS, "gated_linear_attention"), (MIXERS, "state_space_duality"), (MIXERS, "side_by_side"),
                           (MIXERS, "gqa_attention"), (FEED_FORWARDS, "swiglu")):
        assert registry.lookup(kind) is not None
    spec = model_of(tk.CONFIGS["A"][0]).spec
    assert [layer.block["mixer"]["kind"] for layer in spec.layers] == ["gated_linear_attention", "side_by_side", "side_by_side",
                                                                      "gated_linear_attention"]
    left = spec.layers[1].block["mixer"]["left"]
    assert (left["chunk"], left["scale"], left["v_head_dim"], left["position"]["rotary_dim"]) == (12, 0.9, 24, 8)
    assert left["position"]["llama3"]["original_max_position_embeddings"] == 64
    assert "llama3" not in spec.layers[2].block["mixer"]["left"]["position"]
    assert spec.layers[0].block["copies"] == 3 and spec.layers[0].block["learned"]
    plain = model_of(tk.CONFIGS["C"][0]).spec.layers[0].block  # no `streams` key: one copy, no vectors
    assert plain["copies"] == 1 and not plain["learned"]
    assert not any(".hc" in name for name in model_of(tk.CONFIGS["C"][0]).param_specs())


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][1]["mixer"]["left"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=18), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"]["scaling"].update(high=0.5), "scaling"),
    (lambda c: c["layers"][1]["mixer"]["left"]["mask"].update(size=0), "mask.size"),
    (lambda c: c["layers"][1]["mixer"]["right"].update(groups=3), "groups"),
    (lambda c: c["layers"][1]["mixer"]["right"].update(norm_groups=5), "norm_groups"),
    (lambda c: c["layers"][1]["mixer"].pop("left_scale"), "left_scale"),
    (lambda c: c["layers"][0]["mixer"].update(tau=0), "tau"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "mlp"),
    (lambda c: c.update(streams=0), "streams"),
    (lambda c: c["norm"].update(eps=0), "eps"),
    (lambda c: c.pop("width"), "width"),
])
def test_configurations_the_design_does_not_have_are_refused(change, message):
    cfg = copy.deepcopy(tk.CONFIGS["A"][0])
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        architecture_for(cfg).parse_config(cfg)


def wide_weights(cfg, seed):
    return {k: v.astype(np.float64) for k, v in tk.make_weights(cfg, seed=seed).items()}


@pytest.mark.parametrize("name", sorted(tk.CONFIGS))
def test_the_plain_model_gives_the_same_logits_whole_and_in_portions(name):
    cfg, _ = tk.CONFIGS[name]
    weights = wide_weights(cfg, 3)
    tokens = tk.random_tokens(cfg, 31, seed=4)
    whole = pk.logits(cfg, weights, tokens)
    model = pk.Model(cfg, weights)
    parts = [model.feed(tokens[a:b]) for a, b in ((0, 1), (1, 3), (3, 4), (4, 15), (15, 29), (29, 31))]
    np.testing.assert_allclose(np.concatenate(parts), whole, rtol=0, atol=1e-9)
    assert np.abs(whole).max() > 0.5  # (not a model whose logits say nothing)


def test_scaled_frequencies_keep_short_waves_stretch_long_ones_and_blend_between():
    rot = {"base": 100.0, "dims": 8, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}}
    plain = np.array([100.0 ** (-2.0 * i / 8) for i in range(4)])
    got = pk.rotary_frequencies(rot)
    waves = 2 * np.pi / plain  # 6.3, 19.9, 62.8, 198.7 against the borders 16 and 64
    assert waves[0] < 16 < waves[1] < 64 < waves[3] and 16 < waves[2] < 64
    assert got[0] == plain[0] and got[3] == plain[3] / 4.0
    for i in (1, 2):
        s = (64 / waves[i] - 1.0) / 3.0
        assert got[i] == pytest.approx((1 - s) * plain[i] / 4.0 + s * plain[i]) and plain[i] / 4.0 < got[i] < plain[i]
    # the engine's table is made of the same numbers
    from mini_infer_amd.registry import POSITION_ENCODINGS

    desc = model_of(tk.CONFIGS["A"][0]).spec.layers[1].block["mixer"]["left"]["position"]
    position = POSITION_ENCODINGS.lookup(desc["kind"])(desc, torch.float32, "cpu", None)
    np.testing.assert_array_equal(position.inv_freq.numpy(), got.astype(np.float32))


def test_a_chunk_hides_everything_before_its_first_position():
    """The attention alone in the plain model: changing a token that lies before the chunk of the
    last position does not move that position's output; changing the chunk's first token does."""
    m = tk.attention(2, 1, 8, 8, 1.2, 6, (30.0, 8))
    rng = np.random.default_rng(0)
    w = {"q": rng.standard_normal((16, 20)), "k": rng.standard_normal((8, 20)), "v": rng.standard_normal((8, 20)),
         "g": rng.standard_normal((16, 20)), "o": rng.standard_normal((20, 16)), "q.norm": np.ones(8), "k.norm": np.ones(8)}
    h = rng.standard_normal((15, 20))  # the last position, 14, is in the chunk 12..17
    base, _ = pk.chunked_attention(h, "", m, w, 1e-6)
    before = h.copy()
    before[11] += 1.0
    moved, _ = pk.chunked_attention(before, "", m, w, 1e-6)
    assert np.abs(moved[14] - base[14]).max() == 0 and np.abs(moved[11] - base[11]).max() > 1e-3
    inside = h.copy()
    inside[12] += 1.0
    moved, _ = pk.chunked_attention(inside, "", m, w, 1e-6)
    assert np.abs(moved[14] - base[14]).max() > 1e-3
    # fed in two portions cut inside a chunk: the same rows
    head, past = pk.chunked_attention(h[:13], "", m, w, 1e-6)
    tail, _ = pk.chunked_attention(h[13:], "", m, w, 1e-6, first_position=13, past=past)
    np.testing.assert_allclose(np.concatenate([head, tail]), base, atol=1e-12)


def test_the_streams_are_rewritten_all_at_once_through_a_matrix_indexed_from_to():
    rng = np.random.default_rng(1)
    xs, y = rng.standard_normal((3, 2, 5)), rng.standard_normal((2, 5))
    w = {"in": np.array([0.5, -1.0, 2.0]), "out": np.array([1.0, 0.0, -1.0]), "mix": rng.standard_normal((3, 3))}
    np.testing.assert_allclose(pk.hyper_read(xs, w, ""), 0.5 * xs[0] - xs[1] + 2.0 * xs[2])
    new = pk.hyper_write(xs, y, w, "")
    for to in range(3):
        want = sum(w["mix"][frm, to] * xs[frm] for frm in range(3)) + w["out"][to] * y
        np.testing.assert_allclose(new[to], want, atol=1e-12)
    assert np.abs(new - (np.einsum("ts,sjw->tjw", w["mix"], xs) + w["out"][:, None, None] * y[None])).max() > 0.1


def test_every_mechanism_matters_to_the_logits_of_the_tiny_models():
    """The tiny weights let a mechanism that is left out, or a state that is lost, show: the plain
    model with one thing changed is far from the plain model."""
    cfg, _ = tk.CONFIGS["A"]
    weights = wide_weights(cfg, 40)
    tokens = tk.random_tokens(cfg, 40, seed=77)
    base = pk.logits(cfg, weights, tokens)

    def far(other) -> bool:
        return np.abs(other - base).max() > 1e-2

    def changed(**tensors):
        return pk.logits(cfg, {**weights, **tensors}, tokens)

    assert far(changed(**{"l1.hc1.mix": weights["l1.hc1.mix"].T}))  # the matrix read [to, from]
    assert far(changed(**{"l0.hc2.in": weights["l0.hc2.in"][::-1]}))
    assert far(changed(**{"l0.norm1": weights["l0.norm1"] - 1.0}))  # a weight taken as it is stored
    assert far(changed(**{"l1.mix.left.q.norm": weights["l1.mix.left.q.norm"] + 1.0}))  # a plain weight taken as one-plus
    assert far(changed(**{"l1.mix.right.D": np.zeros(4)})) and far(changed(**{"l1.mix.right.conv.b": np.zeros(88)}))
    assert far(changed(**{"l0.mix.a2.b": np.zeros(36)})) and far(changed(**{"l1.mix.right.dt_bias": np.zeros(4)}))
    for change in (lambda c: c["layers"][1]["mixer"]["left"]["mask"].update(size=13),
                   lambda c: c["layers"][1]["mixer"]["left"]["mask"].update(size=4096),
                   lambda c: c["layers"][1]["mixer"]["left"]["rot"].pop("scaling"),
                   lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=16),
                   lambda c: c["layers"][1]["mixer"].update(left_scale=1.3, right_scale=0.7),
                   lambda c: c["layers"][1]["mixer"]["right"].update(norm_groups=1),
                   lambda c: c["layers"][0]["mixer"].update(tau=1.0)):
        other = copy.deepcopy(cfg)
        change(other)
        assert far(pk.logits(other, weights, tokens))
    # state lost between two portions, one layer at a time
    for layer in range(4):
        model = pk.Model(cfg, weights)
        head = model.feed(tokens[:30])
        kept = model.state[layer]
        if cfg["layers"][layer]["type"] == "gla":
            model.state[layer] = np.zeros_like(kept)
            assert far(np.concatenate([head, model.feed(tokens[30:])])), f"matrix state of layer {layer}"
        else:
            (keys, values), (S, tail) = kept
            model.state[layer] = ((keys, values), (np.zeros_like(S), tail))
            assert far(np.concatenate([head, model.feed(tokens[30:])])), f"state-space state of layer {layer}"
            model = pk.Model(cfg, weights)
            head = model.feed(tokens[:30])
            (keys, values), (S, tail) = model.state[layer]
            model.state[layer] = ((keys, values), (S, np.zeros_like(tail)))
            assert far(np.concatenate([head, model.feed(tokens[30:])])), f"convolution tail of layer {layer}"

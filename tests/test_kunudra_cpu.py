"""Kunudra without a GPU: configuration, the model as data (tensor names, cache needs, which layer
gives the shared values), and the plain model against itself (every mechanism matters, windows end
where they should)."""

import copy

import numpy as np
import pytest
import torch

import plain_kunudra as pk
import tiny_kunudra as tk
from mini_infer_amd.exceptions import ConfigError
from mini_infer_amd.models import architecture_for


def model_of(cfg, dtype=torch.bfloat16):
    arch = architecture_for(cfg)
    return arch.make_model(arch.parse_config(cfg), dtype, "cpu")


@pytest.mark.parametrize("name", sorted(tk.CONFIGS))
def test_the_model_asks_for_exactly_the_checkpoints_tensors(name):
    cfg, _ = tk.CONFIGS[name]
    model = model_of(cfg)
    specs = model.param_specs()
    shapes = tk.tensor_shapes(cfg)
    # the layer that gives the shared values has a mixing weight in the checkpoint and does not read it
    unread = {k for k in shapes if k not in specs}
    assert unread <= model.optional_names() and all(k.endswith("mix.vmix") for k in unread)
    assert {k: tuple(v.shape) for k, v in specs.items()} == {k: v for k, v in shapes.items() if k not in unread}
    # what enters a norm, a softmax or the router stays 32-bit whatever the engine's dtype
    for leaf in ("norm1", "norm2", "ls1", "ls2", "mix.q.norm", "mix.k.norm", "mix.dq.norm", "mix.dkv.norm", "mix.sink", "mix.vmix",
                 "mlp.router", "mlp.correction", "mlp.shared.sg", "final.norm"):
        assert all(v.dtype == "float32" for k, v in specs.items() if k.endswith(leaf))


def test_the_first_layer_that_shares_values_gives_and_the_others_take():
    cfg, _ = tk.CONFIGS["A"]
    mixers = [block.mixer for block in model_of(cfg).blocks]
    assert [(m.mix_key is not None, m.mix_source) for m in (mixers[0], mixers[2], mixers[3])] == [(True, True), (True, False), (True, False)]
    alone = [block.mixer for block in model_of(tk.CONFIGS["B"][0]).blocks]
    assert alone[2].mix_source and alone[1].mix_key is None
    assert "l2.mix.vmix" not in model_of(tk.CONFIGS["B"][0]).param_specs()


def test_cache_needs_pages_by_window_and_one_number_of_state_for_the_pair_table():
    cfg, block = tk.CONFIGS["A"]
    needs = model_of(cfg).cache_needs(block)
    assert len(needs) == 5  # four layers, then the embedding's state
    pages = needs[0].pages
    assert (pages.num_kv_heads, pages.head_dim, pages.value_dim, pages.window) == (2, 16, 24, 20) and needs[0].state is None
    latent = needs[1].pages  # one row [latent | rotated part] per token, no value pages
    assert (latent.num_kv_heads, latent.head_dim, latent.value_dim, latent.window) == (1, 22 + 6, 0, 33)
    assert needs[4].pages is None and needs[4].state.shape == (1,) and needs[4].state.dtype == torch.int32
    plain = model_of(tk.CONFIGS["B"][0]).cache_needs(8)
    assert len(plain) == 4 and plain[0].pages.window is None and plain[2].pages.window == 1  # no pair table: no state


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=4), "rot_dim"),
    (lambda c: c["layers"][1]["mixer"].pop("q_rank"), "q_rank"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "mlp"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "top"),
    (lambda c: c["layers"][0]["mixer"].update(softcap=0), "softcap"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(size=0), "mask.size"),
    (lambda c: c["layers"][2]["mixer"].update(vdim=20), "mix values"),
    (lambda c: c["embedding"]["bigram"].update(buckets=0), "buckets"),
    (lambda c: c["norm"].update(eps=0), "eps"),
])
def test_configurations_the_design_does_not_have_are_refused(change, message):
    cfg = copy.deepcopy(tk.CONFIGS["A"][0])
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        architecture_for(cfg).parse_config(cfg)


def test_a_key_that_config_json_does_not_hold_switches_its_mechanism_off():
    cfg = copy.deepcopy(tk.CONFIGS["B"][0])
    parsed = architecture_for(cfg).parse_config(cfg)
    assert parsed.alpha == 1.0 and parsed.pair_table is None
    assert parsed.layers[1].kv_heads == parsed.layers[1].heads and parsed.layers[1].window is None and parsed.layers[2].softcap is None
    assert parsed.layers[1].moe.identity == 0 and parsed.layers[1].moe.shared_ff is None and parsed.layers[1].moe.scale == 1.0
    spec = model_of(cfg).spec
    assert spec.embedding["kind"] == "token_embedding" and spec.head["tied"]


def logits_of(cfg, weights, tokens):
    return pk.logits(cfg, {k: v.astype(np.float64) for k, v in weights.items()}, tokens)


def test_every_mechanism_of_the_tiny_weights_matters():
    """A constant or a tensor left out moves the plain model's logits by far more than any tolerance."""
    cfg, _ = tk.CONFIGS["A"]
    weights = tk.make_weights(cfg, seed=70)
    tokens = tk.random_tokens(cfg, 60, seed=4)
    base = logits_of(cfg, weights, tokens)

    def moved(other_cfg=None, **tensors):
        return np.abs(logits_of(other_cfg or cfg, {**weights, **tensors}, tokens) - base).max()

    def with_mixer(layer, **keys):
        other = copy.deepcopy(cfg)
        for key, value in keys.items():
            if value is None:
                other["layers"][layer]["mixer"].pop(key)
            else:
                other["layers"][layer]["mixer"][key] = value
        return other

    def with_router(layer, **keys):
        other = copy.deepcopy(cfg)
        other["layers"][layer]["mlp"]["router"].update(keys)
        return other

    zero = lambda name: {name: np.zeros_like(weights[name])}  # noqa: E731
    assert moved(**zero("bigram")) > 0.05
    assert moved({**cfg, "postln_alpha": 1.0}) > 0.05
    assert moved({**cfg, "embedding": {"bigram": {"buckets": 97, "mul_prev": 5, "mul_cur": 31}}}) > 0.05
    for name in ("l0.ls1", "l0.ls2", "l1.norm1", "l3.norm2", "final.norm", "l0.mix.q.norm", "l2.mix.k.norm", "l1.mix.dq.norm", "l1.mix.dkv.norm"):
        assert moved(**{name: np.ones_like(weights[name])}) > 0.05, name
    for name in ("l0.mix.sink", "l1.mix.sink", "l2.mix.vmix", "l3.mix.vmix", "l0.mlp.correction", "l0.mlp.shared.sg"):
        assert moved(**zero(name)) > 0.02, name
    assert moved(with_mixer(0, softcap=None)) > 0.02 and moved(with_mixer(3, softcap=None)) > 1e-3
    assert moved(with_mixer(0, v_mix=None)) > 0.02  # (layer 2 then gives, and mixes nothing in)
    for layer in range(4):
        size = cfg["layers"][layer]["mixer"]["mask"]["size"]
        assert moved(with_mixer(layer, mask={"size": size + 1})) > 1e-3 and moved(with_mixer(layer, mask={"size": size - 1})) > 1e-3
    assert moved(with_router(0, scale=1.0)) > 0.02 and moved(with_router(0, top=1)) > 0.02
    # the distance bias: a model whose heads change places inside a layer differs only by it, the sink and the weights' order
    swapped = {k: v.copy() for k, v in weights.items()}
    swapped["l2.mix.sink"] = weights["l2.mix.sink"][::-1].copy()
    assert moved(**{"l2.mix.sink": swapped["l2.mix.sink"]}) > 0.02


def test_identity_experts_return_their_input_and_the_weights_are_not_renormalized():
    rng = np.random.default_rng(0)
    width, ff = 12, 6
    mlp = tk.moe(ff, 2, 2, identity=1, scale=1.5)
    w = {"router": rng.standard_normal((3, width)), "correction": np.array([0.0, -9.0, 9.0])}
    for e in range(2):
        w.update({f"e{e}.gate": rng.standard_normal((ff, width)), f"e{e}.up": rng.standard_normal((ff, width)),
                  f"e{e}.down": rng.standard_normal((width, ff))})
    x = rng.standard_normal((4, width))
    got = pk.routed_feed_forward(x, w, mlp)
    for t in range(4):
        z = w["router"] @ x[t]
        s = np.exp(z) / np.exp(z).sum()
        # the correction decides the choice (the identity expert and expert 0) and is no part of the weights
        want = 1.5 * s[2] * x[t] + 1.5 * s[0] * pk.gated_feed_forward(x[t:t + 1], {k[3:]: v for k, v in w.items() if k.startswith("e0.")})[0]
        np.testing.assert_allclose(got[t], want, rtol=0, atol=1e-12)


def test_the_pair_table_row_of_a_first_token_is_the_last_row():
    weights = {"embed": np.eye(5), "bigram": np.arange(4 * 5, dtype=np.float64).reshape(4, 5)}
    x = pk.embed([2, 4, 1], weights, {"buckets": 3, "mul_prev": 7, "mul_cur": 2})
    np.testing.assert_array_equal(x[0], np.eye(5)[2] + weights["bigram"][3])
    np.testing.assert_array_equal(x[1], np.eye(5)[4] + weights["bigram"][(2 * 7 + 4 * 2) % 3])
    np.testing.assert_array_equal(x[2], np.eye(5)[1] + weights["bigram"][(4 * 7 + 1 * 2) % 3])


def test_a_sink_takes_weight_off_the_keys_and_a_window_counts_the_query_itself():
    p = pk.softmax_with_sink(np.array([0.0, 0.0]), 0.0)
    np.testing.assert_allclose(p, [1 / 3, 1 / 3])
    np.testing.assert_allclose(pk.softmax_with_sink(np.array([1.0, 2.0]), None).sum(), 1.0)
    assert list(pk.visible(10, {"size": 3})) == [8, 9, 10] and list(pk.visible(1, {"size": 3})) == [0, 1] and list(pk.visible(4, None)) == [0, 1, 2, 3, 4]

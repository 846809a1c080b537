"""Kunudra, the plain way: NumPy float64, one function per mechanism, loops over tokens.

The yardstick the engine's Kunudra is measured against.  It shares no code with the package:
it reads the raw config.json keys itself, keeps no cache (every call sees a whole sequence)
and evaluates every sum in 64-bit.

Notation: `x` is the stream [T, W] (here it is what the last norm left, so sublayers read it
as it is); `p`, `i`, `j` positions counted from 0.

`store` (default: nothing) is applied to every tensor an engine would keep in its compute dtype
(projections, activations, sublayer outputs, cached rows; never the stream or anything inside a
softmax, a norm or a router).  With `bf16_round` the model shows how far bfloat16 storage alone,
with exact arithmetic between, moves the logits: the yardstick of the bfloat16 tests.
"""

from __future__ import annotations

import math

import numpy as np


def keep(a):
    return a


def bf16_round(a: np.ndarray) -> np.ndarray:
    import torch

    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).bfloat16().double().numpy()


def rms_norm(x: np.ndarray, weight: np.ndarray | None, eps: float) -> np.ndarray:
    y = x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return y if weight is None else y * weight


def logistic(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * logistic(z)


# np.float32 here makes the angles the way a float32 engine makes them (frequency rounded to float32, then
# the product with the position rounded to float32): at position p that alone moves an angle by up to
# p * 6e-8, far more than rounding a stored value does, and a yardstick for float32 engines has to know it
ANGLE_TYPE = np.float64


def rotate_pairs(v: np.ndarray, position: int, base: float, dims: int) -> np.ndarray:
    """Rotate the first `dims` entries of `v`, entry 2i with entry 2i+1, by position * base^(-2i/dims)."""
    out = np.array(v, dtype=np.float64)
    for i in range(dims // 2):
        angle = float(ANGLE_TYPE(position) * ANGLE_TYPE(base ** (-2.0 * i / dims)))
        a, b = v[2 * i], v[2 * i + 1]
        out[2 * i] = a * math.cos(angle) - b * math.sin(angle)
        out[2 * i + 1] = b * math.cos(angle) + a * math.sin(angle)
    return out


def embed(tokens, weights: dict, bigram: dict | None) -> np.ndarray:
    """Token rows, plus the row of the pair table that the token and the one before it hash to
    (a sequence's first token: the table's last row)."""
    x = np.stack([weights["embed"][t] for t in tokens]).astype(np.float64)
    if bigram is not None:
        buckets = bigram["buckets"]
        for n, token in enumerate(tokens):
            row = buckets if n == 0 else (tokens[n - 1] * bigram["mul_prev"] + token * bigram["mul_cur"]) % buckets
            x[n] += weights["bigram"][row]
    return x


def softmax_with_sink(scores: np.ndarray, sink: float | None) -> np.ndarray:
    """Weights of the keys when the denominator holds exp(sink) too (no sink: the usual softmax)."""
    top = scores.max() if sink is None else max(scores.max(), sink)
    e = np.exp(scores - top)
    return e / (e.sum() + (0.0 if sink is None else math.exp(sink - top)))


def visible(i: int, mask: dict | None) -> range:
    """Positions that position i sees."""
    if mask is None:
        return range(0, i + 1)
    return range(max(0, i - mask["size"] + 1), i + 1)


def biased_attention(x: np.ndarray, w: dict, m: dict, eps: float, shared: dict, first_mixing: bool, store=keep) -> np.ndarray:
    """Grouped-query attention: q and k normed over their whole projection, capped scores, a
    distance bias per head, a window, a sink per head, values mixed with an earlier layer's."""
    T = x.shape[0]
    H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    q = store(rms_norm(store(x @ w["q"].T), w["q.norm"], eps))
    k = store(rms_norm(store(x @ w["k"].T), w["k.norm"], eps))
    v = store(x @ w["v"].T)
    if m.get("v_mix"):
        if first_mixing:
            shared["v_first"] = v
        else:
            lam = float(w["vmix"])
            v = store((1.0 - lam) * v + lam * shared["v_first"])
    out = np.zeros((T, H * dv))
    cap = m.get("softcap")
    for h in range(H):
        g = h // (H // G)
        slope = 2.0 ** (-8.0 * (h + 1) / H)
        for i in range(T):
            js = list(visible(i, m.get("mask")))
            s = np.array([q[i, h * d:(h + 1) * d] @ k[j, g * d:(g + 1) * d] for j in js]) * m["scale"]
            if cap is not None:
                s = cap * np.tanh(s / cap)
            s = s - slope * (i - np.array(js))
            p = softmax_with_sink(s, float(w["sink"][h]) if "sink" in w else None)
            out[i, h * dv:(h + 1) * dv] = sum(p[n] * v[j, g * dv:(g + 1) * dv] for n, j in enumerate(js))
    return store(store(out) @ w["o"].T)


def latent_attention(x: np.ndarray, w: dict, m: dict, eps: float, store=keep) -> np.ndarray:
    """Queries through a normed latent; keys and values of all heads as maps of one normed latent
    row per token, beside one rotated key part that the heads share; a window and a sink."""
    T = x.shape[0]
    H, d, r, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    cq = store(rms_norm(store(x @ w["dq"].T), w["dq.norm"], eps))
    q = store(cq @ w["uq"].T)
    down = store(x @ w["dkv"].T)
    c = store(rms_norm(down[:, :rank], w["dkv.norm"], eps))
    shared_key = store(np.stack([rotate_pairs(down[i, rank:], i, base, dims) for i in range(T)]))
    keys, values = c @ w["uk"].T, c @ w["uv"].T
    out = np.zeros((T, H * dv))
    for h in range(H):
        head = q[:, h * (d + r):(h + 1) * (d + r)]
        for i in range(T):
            q_rot = rotate_pairs(head[i, d:], i, base, dims)
            js = list(visible(i, m.get("mask")))
            s = np.array([head[i, :d] @ keys[j, h * d:(h + 1) * d] + q_rot @ shared_key[j] for j in js]) * m["scale"]
            p = softmax_with_sink(s, float(w["sink"][h]) if "sink" in w else None)
            out[i, h * dv:(h + 1) * dv] = sum(p[n] * values[j, h * dv:(h + 1) * dv] for n, j in enumerate(js))
    return store(store(out) @ w["o"].T)


def gated_feed_forward(h: np.ndarray, w: dict, store=keep) -> np.ndarray:
    return store(store(silu(store(h @ w["gate"].T)) * store(h @ w["up"].T)) @ w["down"].T)


# a list here collects, for every token of every routed layer, how far the last chosen expert's choice
# score lies above the best one left out (a test can then keep to inputs whose choices no rounding turns)
CHOICE_MARGINS: list | None = None


def routed_feed_forward(x: np.ndarray, w: dict, mlp: dict, store=keep) -> np.ndarray:
    """Each token's `top` experts by score plus correction, weighted by the score itself times a
    constant; the last router outputs stand for experts that return their input; a shared expert
    behind a gate of one number a token."""
    router = mlp["router"]
    experts, identity, top = router["experts"], router.get("identity", 0), router["top"]
    out = np.zeros_like(x)
    margins = CHOICE_MARGINS
    for t in range(x.shape[0]):
        z = w["router"].astype(np.float64) @ x[t]
        s = np.exp(z - z.max())
        s = s / s.sum()
        choice = s + (w["correction"] if "correction" in w else 0.0)
        ranked = np.argsort(-choice, kind="stable")
        if margins is not None and top < len(ranked):
            margins.append(float(choice[ranked[top - 1]] - choice[ranked[top]]))
        for e in ranked[:top]:
            weight = s[e] * router.get("scale", 1.0)
            if e >= experts:
                assert e < experts + identity
                out[t] += weight * x[t]
            else:
                sub = {name: w[f"e{e}.{name}"] for name in ("gate", "up", "down")}
                out[t] += weight * gated_feed_forward(x[t:t + 1], sub, store)[0]
    if mlp.get("shared") is not None:
        sub = {name: w[f"shared.{name}"] for name in ("gate", "up", "down")}
        gate = logistic(x @ w["shared.sg"].astype(np.float64).T)  # [T, 1]
        out += gate * gated_feed_forward(x, sub, store)
    return store(out)


def split_weights(weights: dict, prefix: str) -> dict:
    return {name[len(prefix):]: np.asarray(value, dtype=np.float64) for name, value in weights.items() if name.startswith(prefix)}


def forward(config: dict, weights: dict, tokens, store=keep, layers_out: list | None = None) -> np.ndarray:
    """The stream after the last layer, [T, W]; `layers_out` collects it after every layer."""
    eps, alpha = config["norm"]["eps"], config.get("postln_alpha", 1.0)
    x = embed(list(tokens), weights, (config.get("embedding") or {}).get("bigram"))
    shared: dict = {}
    seen_mixing = False
    for n, layer in enumerate(config["layers"]):
        w = split_weights(weights, f"l{n}.")
        mix = split_weights(weights, f"l{n}.mix.")
        h = store(x)
        if layer["type"] == "attention":
            first = bool(layer["mixer"].get("v_mix")) and not seen_mixing
            y = biased_attention(h, mix, layer["mixer"], eps, shared, first, store)
            seen_mixing = seen_mixing or bool(layer["mixer"].get("v_mix"))
        elif layer["type"] == "latent_attention":
            y = latent_attention(h, mix, layer["mixer"], eps, store)
        else:
            raise ValueError(layer["type"])
        x = rms_norm(alpha * x + w["ls1"] * y, 1.0 + w["norm1"], eps)
        if layer.get("mlp") is not None:
            mlp = split_weights(weights, f"l{n}.mlp.")
            h = store(x)
            y = gated_feed_forward(h, mlp, store) if layer["mlp"]["kind"] == "dense" else routed_feed_forward(h, mlp, layer["mlp"], store)
            x = rms_norm(alpha * x + w["ls2"] * y, 1.0 + w["norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    return x


def logits(config: dict, weights: dict, tokens, store=keep, layers_out: list | None = None) -> np.ndarray:
    x = forward(config, weights, tokens, store, layers_out)
    h = store(rms_norm(x, 1.0 + np.asarray(weights["final.norm"], dtype=np.float64), config["norm"]["eps"]))
    return h @ np.asarray(weights["embed"], dtype=np.float64).T


def greedy(row: np.ndarray) -> int:
    return int(np.argmax(row))

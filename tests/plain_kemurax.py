"""Kemurax, plain and slow: NumPy float64, one function per mechanism, token loops for
everything that runs along the sequence.  It shares no code with the engine.

`config` is the raw config.json dictionary, `weights` maps tensor names to float64 arrays.
`store` (optional) rounds what an engine keeps in a narrower type: it is applied to the
outputs of products and to activations, never to what the design computes in 32-bit (norms,
scores, the streams, recurrent state, decays and gates of a recurrence).  With `store=None`
the model is exact.
"""

from __future__ import annotations

import math

import numpy as np


def _same(x):
    return x


def bf16_round(a: np.ndarray) -> np.ndarray:
    """What is left of `a` when it is stored in bfloat16 (round to nearest even), as float64."""
    bits = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    bits = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) << 16
    return bits.astype(np.uint32).view(np.float32).astype(np.float64).reshape(np.shape(a))


def greedy(row: np.ndarray) -> int:
    return int(np.argmax(row))


def rms_unit(x: np.ndarray, eps: float) -> np.ndarray:
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def one_plus_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """RMS norm whose weight is stored around zero."""
    return rms_unit(x, eps) * (1.0 + w)


def logistic(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * logistic(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z**3)))


# -- rotation ---------------------------------------------------------------------------


def rotary_frequencies(rot: dict) -> np.ndarray:
    dims = int(rot["dims"])
    f = np.array([float(rot["base"]) ** (-2.0 * i / dims) for i in range(dims // 2)])
    scaling = rot.get("scaling")
    if scaling is None:
        return f
    factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = np.empty_like(f)
    for i, fi in enumerate(f):
        wavelength = 2.0 * math.pi / fi
        if wavelength < original / high:
            out[i] = fi
        elif wavelength > original / low:
            out[i] = fi / factor
        else:
            s = (original / wavelength - low) / (high - low)
            out[i] = (1.0 - s) * fi / factor + s * fi
    return out


def rotate(x: np.ndarray, position: int, freq: np.ndarray) -> np.ndarray:
    """One head row: dimension i is turned together with dimension i + dims/2; the rest passes."""
    half = len(freq)
    out = x.copy()
    for i in range(half):
        a = position * freq[i]
        u, v = x[i], x[i + half]
        out[i] = u * math.cos(a) - v * math.sin(a)
        out[i + half] = v * math.cos(a) + u * math.sin(a)
    return out


# -- mixers -----------------------------------------------------------------------------


def gla_mixer(h: np.ndarray, p: str, m: dict, w: dict, eps: float, store=_same, state=None):
    """Gated linear attention, token by token.  h [T, width] -> [T, width]; `state` [heads, dim, vdim]."""
    heads, dim, vdim, tau = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["tau"])
    T = h.shape[0]
    q = store(h @ w[p + "q"].T).reshape(T, heads, dim) * dim**-0.5
    k = store(h @ w[p + "k"].T).reshape(T, heads, dim)
    v = store(h @ w[p + "v"].T).reshape(T, heads, vdim)
    g = store(h @ w[p + "g"].T)
    z = store(store(h @ w[p + "a1"].T) @ w[p + "a2"].T) + w[p + "a2.b"]
    alpha = (logistic(z) ** (1.0 / tau)).reshape(T, heads, dim)
    S = np.zeros((heads, dim, vdim)) if state is None else state
    out = np.empty((T, heads, vdim))
    for t in range(T):
        for a in range(heads):
            S[a] = alpha[t, a][:, None] * S[a] + np.outer(k[t, a], v[t, a])
            out[t, a] = S[a].T @ q[t, a]
    out = rms_unit(out, eps) * w[p + "norm"]
    gated = store(out.reshape(T, heads * vdim) * silu(g))
    return store(gated @ w[p + "o"].T), S


def chunked_attention(h: np.ndarray, p: str, m: dict, w: dict, eps: float, store=_same, first_position: int = 0, past=None):
    """Grouped-query attention inside chunks of `mask.size` positions counted from the sequence's start.
    `past`: (keys, values) of the tokens before `h`, as lists of [kv_heads, ...] rows."""
    H, G, dim, vdim = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    size, scale = int(m["mask"]["size"]), float(m["scale"])
    freq = rotary_frequencies(m["rot"])
    T = h.shape[0]
    q = store(h @ w[p + "q"].T).reshape(T, H, dim)
    k = store(h @ w[p + "k"].T).reshape(T, G, dim)
    v = store(h @ w[p + "v"].T).reshape(T, G, vdim)
    q = rms_unit(q, eps) * w[p + "q.norm"]
    k = rms_unit(k, eps) * w[p + "k.norm"]
    keys, values = ([], []) if past is None else past
    out = np.empty((T, H, vdim))
    for t in range(T):
        pos = first_position + t
        keys.append(store(np.stack([rotate(k[t, a], pos, freq) for a in range(G)])))
        values.append(v[t])
        lo = (pos // size) * size
        for a in range(H):
            qa = store(rotate(q[t, a], pos, freq))
            kv = a // (H // G)
            scores = np.array([qa @ keys[j][kv] for j in range(lo, pos + 1)]) * scale
            weights = np.exp(scores - scores.max())
            weights /= weights.sum()
            out[t, a] = sum(weights[j - lo] * values[j][kv] for j in range(lo, pos + 1))
    gate = logistic(store(h @ w[p + "g"].T))
    gated = store(store(out.reshape(T, H * vdim)) * gate)
    return store(gated @ w[p + "o"].T), (keys, values)


def ssd_mixer(h: np.ndarray, p: str, m: dict, w: dict, eps: float, store=_same, state=None):
    """Mamba-2 in its recurrent form.  `state`: (S [heads, N, vdim], the last taps-1 conv inputs [taps-1, channels])."""
    heads, vdim, N, G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
    taps, norm_groups = int(m["conv"]), int(m["norm_groups"])
    inner = heads * vdim
    channels = inner + 2 * G * N
    T = h.shape[0]
    proj = store(h @ w[p + "in"].T)
    z, xbc, dt = proj[:, :inner], proj[:, inner:inner + channels], proj[:, inner + channels:]
    assert dt.shape[1] == heads
    if state is None:
        S, tail = np.zeros((heads, N, vdim)), np.zeros((taps - 1, channels))
    else:
        S, tail = state
    padded = np.concatenate([tail, xbc], axis=0)
    conv = np.empty((T, channels))
    for t in range(T):
        window = padded[t:t + taps]  # the last row is the current token's
        conv[t] = np.einsum("jc,cj->c", window, w[p + "conv"]) + w[p + "conv.b"]
    tail = padded[T:] if taps > 1 else tail
    conv = store(silu(conv))
    x = conv[:, :inner].reshape(T, heads, vdim)
    B = conv[:, inner:inner + G * N].reshape(T, G, N)
    C = conv[:, inner + G * N:].reshape(T, G, N)
    step = softplus(dt + w[p + "dt_bias"])
    rate = np.exp(w[p + "A_log"])
    y = np.empty((T, heads, vdim))
    for t in range(T):
        for a in range(heads):
            grp = a // (heads // G)
            S[a] = math.exp(-rate[a] * step[t, a]) * S[a] + step[t, a] * np.outer(B[t, grp], x[t, a])
            y[t, a] = S[a].T @ C[t, grp] + w[p + "D"][a] * x[t, a]
    y = y.reshape(T, inner) * silu(z)
    y = rms_unit(y.reshape(T, norm_groups, inner // norm_groups), eps).reshape(T, inner) * w[p + "norm"]
    return store(store(y) @ w[p + "o"].T), (S, tail)


def parallel_mixer(h, p, m, w, eps, store=_same, first_position=0, state=None):
    left_state, right_state = (None, None) if state is None else state
    left, left_state = chunked_attention(h, p + "left.", m["left"], w, eps, store, first_position, left_state)
    right, right_state = ssd_mixer(h, p + "right.", m["right"], w, eps, store, right_state)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right, (left_state, right_state)


def dense_feed_forward(h, p, w, store=_same):
    act = store(gelu_tanh(store(h @ w[p + "gate"].T)) * store(h @ w[p + "up"].T))
    return store(act @ w[p + "down"].T)


# -- the stack --------------------------------------------------------------------------


def hyper_read(streams: np.ndarray, w: dict, p: str) -> np.ndarray:
    """streams [S, T, width] -> the sublayer's input before its norm."""
    return np.einsum("s,stw->tw", w[p + "in"], streams)


def hyper_write(streams: np.ndarray, y: np.ndarray, w: dict, p: str) -> np.ndarray:
    """All streams at once from the old ones; the mix matrix is indexed [from, to]."""
    return np.einsum("st,sjw->tjw", w[p + "mix"], streams) + w[p + "out"][:, None, None] * y[None]


class Model:
    """Holds a request's caches and state, so tokens can be fed in portions."""

    def __init__(self, config: dict, weights: dict, store=None):
        self.c, self.w, self.store = config, weights, (store or _same)
        self.eps = float(config["norm"]["eps"])
        self.streams = config.get("streams")
        self.reset()

    def reset(self):
        self.position = 0
        self.state = [None] * len(self.c["layers"])

    def feed(self, tokens, layers_out: list | None = None) -> np.ndarray:
        """Logits [len(tokens), vocab] of the next portion of the sequence."""
        c, w, store, eps = self.c, self.w, self.store, self.eps
        x = one_plus_norm(w["embed"][np.asarray(tokens)], w["embed.norm"], eps)
        count = 1 if self.streams is None else int(self.streams)
        xs = np.stack([x] * count)
        for i, layer in enumerate(c["layers"]):
            p = f"l{i}."
            for q, kind in ((1, "mixer"), (2, "mlp")):
                if kind == "mlp" and layer.get("mlp") is None:
                    continue
                u = xs[0] if self.streams is None else hyper_read(xs, w, f"{p}hc{q}.")
                hn = store(one_plus_norm(u, w[f"{p}norm{q}"], eps))
                if kind == "mlp":
                    y = dense_feed_forward(hn, p + "mlp.", w, store)
                elif layer["type"] == "gla":
                    y, self.state[i] = gla_mixer(hn, p + "mix.", layer["mixer"], w, eps, store, self.state[i])
                else:
                    y, self.state[i] = parallel_mixer(hn, p + "mix.", layer["mixer"], w, eps, store, self.position, self.state[i])
                xs = xs + y[None] if self.streams is None else hyper_write(xs, y, w, f"{p}hc{q}.")
            if layers_out is not None:
                layers_out.append(xs.sum(axis=0))
        self.position += len(tokens)
        final = store(one_plus_norm(xs.sum(axis=0), w["final.norm"], eps))
        return final @ w["embed"].T


def logits(config: dict, weights: dict, tokens, store=None, layers_out=None) -> np.ndarray:
    return Model(config, weights, store).feed(tokens, layers_out)

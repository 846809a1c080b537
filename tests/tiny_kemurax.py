"""Tiny Kemurax configurations, weights and model folders for the tests.

The configurations differ in every size and constant and in the order of layers: streams in
three copies, two, one with learned vectors, and none (a plain residual add); chunks that are
no multiple of a page, smaller than a page, larger than any prompt, of one position; one
key/value head, several, as many as query heads; value heads wider and narrower than query
heads; rotation of a whole head and of a part, with and without frequency scaling whose three
ranges all occur; state-space groups of one head, several, all; a norm in one part and in
several; convolutions of one tap (no tail to carry) to five; layers without a feed-forward; a
model without attention (no pages at all) and one without gated linear attention.  Weights are
made with NumPy and rounded to bfloat16, so both engines and the plain model read the same
numbers.
"""

from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import torch
from safetensors.torch import save_file


def mlp(ff):
    return None if ff is None else {"kind": "dense", "ff": ff}


def gla(heads, dim, vdim, tau, ff=None):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}, "mlp": mlp(ff)}


def attention(heads, kv_heads, dim, vdim, scale, chunk, rot, scaling=None):
    """`rot` = (base, dims); `scaling` = (factor, low, high, original) or None."""
    r = {"base": rot[0], "dims": rot[1]}
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": chunk}, "rot": r}


def state_space(heads, vdim, state, groups, conv, norm_groups):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def parallel(left, right, left_scale, right_scale, ff=None):
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale},
            "mlp": mlp(ff)}


def config(vocab, width, layers, *, eps, streams=None):
    out = {"architecture": "Kemurax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if streams is not None:
        out["streams"] = streams
    return out


# three copies of the stream; a chunk of 12 under pages of 16 (edges in the middle of a page);
# part of a head rotated, scaled frequencies of all three ranges; two key/value heads, value heads
# wider than query heads; state-space heads in two groups, norm in two parts, three taps
TINY_A = config(160, 64, [
    gla(3, 12, 20, 4.0, ff=96),
    parallel(attention(4, 2, 16, 24, 0.9, 12, (100.0, 8), (4.0, 1.0, 4.0, 64)), state_space(4, 12, 10, 2, 3, 2), 0.7, 1.3, ff=80),
    parallel(attention(2, 1, 8, 8, 1.2, 12, (30.0, 8)), state_space(2, 16, 6, 1, 2, 1), 1.1, 0.6),
    gla(2, 16, 8, 9.0),
], eps=1e-5, streams=3)
TINY_A_BLOCK = 16
# sizes nothing divides; one copy of the stream with vectors of its own; a single tap; whole heads
# rotated; value heads narrower; as many key/value heads as query heads; every head a group of its
# own; a chunk of 5 under pages of 8, and a chunk of one position
TINY_B = config(131, 90, [
    parallel(attention(3, 3, 10, 6, 1.1, 5, (1000.0, 10)), state_space(3, 7, 9, 3, 1, 3), 0.5, 1.5, ff=70),
    gla(3, 7, 9, 2.5, ff=26),
    parallel(attention(2, 1, 6, 6, 0.7, 1, (50.0, 2)), state_space(6, 5, 6, 2, 5, 2), 1.0, 1.0),
    parallel(attention(5, 1, 6, 10, 1.3, 21, (7.0, 4), (8.0, 0.5, 2.0, 40)), state_space(1, 20, 12, 1, 4, 5), 0.9, 0.8, ff=50),
], eps=3e-6, streams=1)
TINY_B_BLOCK = 8
# sizes at which the fast bfloat16 paths run (weight-streaming products, whole vector loads, the
# matrix-core attention kernel); no `streams` key: one stream and a plain add
TINY_C = config(300, 256, [
    parallel(attention(8, 2, 64, 64, 0.3, 48, (500000.0, 32), (8.0, 1.0, 4.0, 128)), state_space(8, 32, 64, 2, 4, 1), 0.8, 0.9, ff=512),
    gla(4, 64, 64, 16.0, ff=384),
    parallel(attention(4, 4, 32, 32, 0.45, 64, (10000.0, 32)), state_space(4, 64, 128, 4, 4, 4), 1.0, 1.0),
    gla(2, 128, 128, 8.0, ff=256),
], eps=2e-6)
TINY_C_BLOCK = 16
# no attention anywhere: state slots only
TINY_D = config(97, 48, [gla(2, 8, 8, 3.0, ff=64), gla(3, 20, 12, 1.0), gla(1, 4, 30, 32.0, ff=32)], eps=1e-6, streams=2)
TINY_D_BLOCK = 4
# no gated linear attention; the largest heads; a chunk longer than every prompt of the tests (one
# chunk: plain causal attention) beside a short one; two copies of the stream
TINY_E = config(200, 128, [
    parallel(attention(2, 2, 128, 128, 0.12, 4096, (10000.0, 128), (2.0, 1.0, 8.0, 256)), state_space(2, 64, 256, 1, 2, 2), 0.6, 0.4, ff=192),
    parallel(attention(4, 1, 64, 32, 0.25, 30, (50.0, 2)), state_space(8, 8, 16, 4, 3, 1), 1.4, 0.7, ff=96),
], eps=1e-6, streams=2)
TINY_E_BLOCK = 16

CONFIGS = {"A": (TINY_A, TINY_A_BLOCK), "B": (TINY_B, TINY_B_BLOCK), "C": (TINY_C, TINY_C_BLOCK), "D": (TINY_D, TINY_D_BLOCK),
           "E": (TINY_E, TINY_E_BLOCK)}


def bf16_round(values: np.ndarray) -> np.ndarray:
    return torch.from_numpy(np.ascontiguousarray(values, dtype=np.float32)).bfloat16().float().numpy()


def decay_rank(m: dict) -> int:
    """How wide the tests' checkpoints make the narrow projection in front of the decay gates
    (config.json does not say; the engine reads it off the tensor's shape)."""
    return 3 + m["heads"]


def tensor_shapes(cfg: dict) -> dict[str, tuple[int, ...]]:
    w, v, s = cfg["width"], cfg["vocab"], cfg.get("streams")
    shapes: dict[str, tuple[int, ...]] = {"embed": (v, w), "embed.norm": (w,), "final.norm": (w,)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        shapes[p + "norm1"] = (w,)
        connections = ["hc1."]
        if layer["type"] == "gla":
            qk, vw = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            shapes.update({p + "mix.q": (qk, w), p + "mix.k": (qk, w), p + "mix.v": (vw, w), p + "mix.g": (vw, w),
                           p + "mix.o": (w, vw), p + "mix.norm": (m["vdim"],), p + "mix.a1": (decay_rank(m), w),
                           p + "mix.a2": (qk, decay_rank(m)), p + "mix.a2.b": (qk,)})
        else:
            a, r = m["left"], m["right"]
            q = p + "mix.left."
            shapes.update({q + "q": (a["heads"] * a["dim"], w), q + "k": (a["kv_heads"] * a["dim"], w),
                           q + "v": (a["kv_heads"] * a["vdim"], w), q + "q.norm": (a["dim"],), q + "k.norm": (a["dim"],),
                           q + "g": (a["heads"] * a["vdim"], w), q + "o": (w, a["heads"] * a["vdim"])})
            q = p + "mix.right."
            inner, span = r["heads"] * r["vdim"], r["groups"] * r["state"]
            shapes.update({q + "in": (2 * inner + 2 * span + r["heads"], w), q + "conv": (inner + 2 * span, r["conv"]),
                           q + "conv.b": (inner + 2 * span,), q + "dt_bias": (r["heads"],), q + "A_log": (r["heads"],),
                           q + "D": (r["heads"],), q + "norm": (inner,), q + "o": (w, inner)})
        if layer["mlp"] is not None:
            ff = layer["mlp"]["ff"]
            shapes.update({p + "norm2": (w,), p + "mlp.gate": (ff, w), p + "mlp.up": (ff, w), p + "mlp.down": (w, ff)})
            connections.append("hc2.")
        if s is not None:
            for c in connections:
                shapes.update({p + c + "in": (s,), p + c + "out": (s,), p + c + "mix": (s, s)})
    return shapes


def make_weights(cfg: dict, seed: int) -> dict[str, np.ndarray]:
    """Activations of order one everywhere.  Norm weights stored around zero are spread over
    -0.5 .. 0.5 and plain ones over 0.5 .. 1.5 (a weight left out, or a one added where none
    belongs, shows); biases of order one; decay gates, rates and step biases such that a head
    forgets over a few to a few dozen tokens; the streams' vectors and matrices far from the
    identity, so that a transposed matrix or a copy read for another shows."""
    rng = np.random.default_rng(seed)
    out: dict[str, np.ndarray] = {}
    for name, shape in sorted(tensor_shapes(cfg).items()):
        leaf = name.split(".", 1)[-1] if name.startswith("l") and name[1].isdigit() else name
        last = leaf.rsplit(".", 1)[-1]
        if leaf in ("norm1", "norm2", "final.norm", "embed.norm"):
            values = rng.uniform(-0.5, 0.5, size=shape)
        elif leaf in ("mix.norm", "mix.right.norm", "mix.left.q.norm", "mix.left.k.norm"):
            values = rng.uniform(0.5, 1.5, size=shape)
        elif leaf in ("mix.right.dt_bias", "mix.right.conv.b", "mix.right.D"):
            values = rng.standard_normal(shape)
        elif leaf == "mix.a2.b":
            values = rng.standard_normal(shape) + 1.0
        elif leaf == "mix.right.A_log":
            values = rng.uniform(-2.5, 0.5, size=shape)
        elif leaf == "mix.right.conv":
            values = rng.standard_normal(shape) * 0.6
        elif leaf.startswith("hc") and last == "mix":
            values = np.eye(shape[0]) * 0.8 + rng.uniform(-0.4, 0.4, size=shape)
        elif leaf.startswith("hc") and last == "in":
            values = rng.uniform(0.3, 0.9, size=shape) * rng.choice([1.0, 1.0, -1.0], size=shape)
        elif leaf.startswith("hc") and last == "out":
            values = rng.uniform(0.5, 1.2, size=shape)
        elif name == "embed":
            values = rng.standard_normal(shape)
        elif leaf == "mix.a2":
            values = rng.standard_normal(shape) / np.sqrt(shape[1]) * 2.0
        else:
            values = rng.standard_normal(shape) / np.sqrt(shape[1]) * (2.0 if last in ("q", "k") else 1.0)
        out[name] = bf16_round(np.asarray(values, dtype=np.float32)).reshape(shape)
    return out


def write_model_dir(path: Path, cfg: dict, weights: dict[str, np.ndarray], dtype=torch.bfloat16) -> Path:
    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    with (path / "config.json").open("w") as handle:
        json.dump(cfg, handle)
    tensors = {k: torch.from_numpy(np.ascontiguousarray(v, dtype=np.float32)).reshape(v.shape).to(dtype) for k, v in weights.items()}
    save_file(tensors, str(path / "model.safetensors"))
    return path


def random_tokens(cfg: dict, length: int, seed: int) -> list[int]:
    return np.random.default_rng(seed).integers(0, cfg["vocab"], size=length).tolist()

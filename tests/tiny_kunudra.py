"""Tiny Kunudra configurations, weights and model folders for the tests.

The configurations differ in every size and constant and in the order of layers: attention first
or latent attention first; windows of one position, smaller than a page, a page's multiple, longer
than any prompt, and none; scores capped hard, softly and not at all; one key/value head, several,
as many as query heads; value heads wider and narrower than key heads; values shared by three
layers, by one (which then only gives) and by none; a query latent narrower and wider than a head;
experts with and without identity experts, with and without a shared expert, one chosen, several,
all; dense feed-forwards and layers without any; with and without the pair table; sizes that no
vector width divides.  Weights are made with NumPy and rounded to bfloat16, so both engines and the
plain model read the same numbers.
"""

from __future__ import annotations

import json
from pathlib import Path

import numpy as np
import torch
from safetensors.torch import save_file


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, identity=None, scale=None, shared=None):
    router = {"experts": experts, "top": top}
    if identity is not None:
        router["identity"] = identity
    if scale is not None:
        router["scale"] = scale
    out = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def attention(heads, kv_heads, dim, vdim, scale, window=None, softcap=None, v_mix=False, mlp=None):
    mixer = {"heads": heads, "dim": dim, "vdim": vdim, "scale": scale}
    if kv_heads is not None:
        mixer["kv_heads"] = kv_heads
    if window is not None:
        mixer["mask"] = {"size": window}
    if softcap is not None:
        mixer["softcap"] = softcap
    if v_mix:
        mixer["v_mix"] = True
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base, window=None, mlp=None):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
             "rot": {"base": base, "dims": rot_dim}}
    if window is not None:
        mixer["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def config(vocab, width, layers, *, eps, alpha=None, pairs=None):
    out = {"architecture": "Kunudra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if alpha is not None:
        out["postln_alpha"] = alpha
    if pairs is not None:
        out["embedding"] = {"bigram": {"buckets": pairs[0], "mul_prev": pairs[1], "mul_cur": pairs[2]}}
    return out


# attention first; values shared by three layers; a hard cap (scores of several units against a cap of 2),
# a soft one and none; identity experts and a shared expert; a layer without feed-forward
TINY_A = config(150, 64, [
    attention(4, 2, 16, 24, 0.9, window=20, softcap=2.0, v_mix=True, mlp=moe(48, 6, 2, identity=2, scale=1.3, shared=40)),
    latent(3, 10, 6, 14, 22, 18, 0.8, 50.0, window=33, mlp=dense(80)),
    attention(4, 2, 8, 24, 1.2, window=7, v_mix=True),
    attention(8, 2, 12, 24, 0.7, window=50, softcap=30.0, v_mix=True, mlp=moe(32, 4, 1)),
], eps=1e-5, alpha=1.5, pairs=(97, 31, 5))
TINY_A_BLOCK = 16
# sizes nothing divides; latent attention first; no pair table, no alpha; a window of one position; all
# experts chosen; a single layer that shares values (it only gives); as many key/value heads as query heads
# (the key is left out of config.json) and a single one; page size 8
TINY_B = config(131, 90, [
    latent(5, 6, 2, 10, 18, 7, 1.3, 7.0, mlp=dense(70)),
    attention(3, None, 10, 6, 1.1, softcap=4.0, mlp=moe(26, 3, 3)),
    attention(6, 1, 6, 10, 0.9, window=1, v_mix=True),
    latent(2, 4, 4, 6, 10, 12, 1.0, 1000.0, window=9, mlp=moe(22, 5, 4, identity=3, scale=0.7, shared=30)),
], eps=3e-6)
TINY_B_BLOCK = 8
# sizes at which the fast bfloat16 paths run (weight-streaming products, whole vector loads, latent heads
# that the matrix cores take when a prompt comes whole: 32 + 32 and 64 + 64)
TINY_C = config(300, 256, [
    latent(4, 32, 32, 64, 96, 64, 0.25, 10000.0, window=48, mlp=moe(128, 8, 2, identity=1, scale=2.0, shared=128)),
    attention(8, 2, 64, 64, 0.2, window=40, softcap=20.0, v_mix=True, mlp=dense(384)),
    attention(8, 2, 32, 64, 0.3, window=100, v_mix=True, mlp=moe(64, 16, 4, scale=1.0)),
    latent(2, 64, 64, 32, 128, 32, 0.2, 500000.0),
], eps=2e-6, alpha=2.5, pairs=(257, 3, 1))
TINY_C_BLOCK = 16
# windows beside page borders: a page of 4 with windows of 4, 5, 8 and 3; one expert of one chosen
TINY_D = config(97, 48, [
    attention(2, 1, 8, 8, 1.0, window=4, softcap=50.0, mlp=moe(16, 1, 1, identity=1, scale=1.0)),
    latent(2, 8, 4, 8, 12, 8, 0.9, 100.0, window=5),
    attention(4, 4, 4, 6, 1.4, window=8, v_mix=True, mlp=dense(40)),
    attention(2, 2, 12, 12, 0.8, window=3, v_mix=True),
], eps=1e-6, alpha=0.75, pairs=(11, 2, 3))
TINY_D_BLOCK = 4

CONFIGS = {"A": (TINY_A, TINY_A_BLOCK), "B": (TINY_B, TINY_B_BLOCK), "C": (TINY_C, TINY_C_BLOCK), "D": (TINY_D, TINY_D_BLOCK)}


def bf16_round(values: np.ndarray) -> np.ndarray:
    return torch.from_numpy(np.ascontiguousarray(values, dtype=np.float32)).bfloat16().float().numpy()


def tensor_shapes(cfg: dict) -> dict[str, tuple[int, ...]]:
    w, v = cfg["width"], cfg["vocab"]
    shapes: dict[str, tuple[int, ...]] = {"embed": (v, w), "final.norm": (w,)}
    pairs = (cfg.get("embedding") or {}).get("bigram")
    if pairs:
        shapes["bigram"] = (pairs["buckets"] + 1, w)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        shapes.update({p + "norm1": (w,), p + "ls1": (w,), p + "mix.sink": (m["heads"],), p + "mix.o": (w, m["heads"] * m["vdim"])})
        if layer["type"] == "attention":
            kv = m.get("kv_heads", m["heads"])
            shapes.update({p + "mix.q": (m["heads"] * m["dim"], w), p + "mix.k": (kv * m["dim"], w), p + "mix.v": (kv * m["vdim"], w),
                           p + "mix.q.norm": (m["heads"] * m["dim"],), p + "mix.k.norm": (kv * m["dim"],)})
            if m.get("v_mix"):
                shapes[p + "mix.vmix"] = ()
        else:
            shapes.update({p + "mix.dq": (m["q_rank"], w), p + "mix.dq.norm": (m["q_rank"],),
                           p + "mix.uq": (m["heads"] * (m["dim"] + m["rot_dim"]), m["q_rank"]),
                           p + "mix.dkv": (m["kv_rank"] + m["rot_dim"], w), p + "mix.dkv.norm": (m["kv_rank"],),
                           p + "mix.uk": (m["heads"] * m["dim"], m["kv_rank"]), p + "mix.uv": (m["heads"] * m["vdim"], m["kv_rank"])})
        mlp = layer["mlp"]
        if mlp is None:
            continue
        shapes.update({p + "norm2": (w,), p + "ls2": (w,)})
        if mlp["kind"] == "dense":
            shapes.update({p + "mlp.gate": (mlp["ff"], w), p + "mlp.up": (mlp["ff"], w), p + "mlp.down": (w, mlp["ff"])})
        else:
            router, ff = mlp["router"], mlp["expert"]["ff"]
            outputs = router["experts"] + router.get("identity", 0)
            shapes.update({p + "mlp.router": (outputs, w), p + "mlp.correction": (outputs,)})
            for e in range(router["experts"]):
                shapes.update({p + f"mlp.e{e}.gate": (ff, w), p + f"mlp.e{e}.up": (ff, w), p + f"mlp.e{e}.down": (w, ff)})
            if mlp.get("shared"):
                sff = mlp["shared"]["ff"]
                shapes.update({p + "mlp.shared.gate": (sff, w), p + "mlp.shared.up": (sff, w), p + "mlp.shared.down": (w, sff),
                               p + "mlp.shared.sg": (1, w)})
    return shapes


def make_weights(cfg: dict, seed: int, steady_choice: bool = False) -> dict[str, np.ndarray]:
    """Activations of order one or a little below everywhere; norm weights (stored around zero) and layer scales spread
    widely (one left out shows), sinks of order one with both signs, mixing weights between 0.2 and
    0.8, routers with rows of order several (peaked scores, so the choice rarely hangs on the last
    digits) and corrections large enough to change choices.

    `steady_choice`: corrections further apart than any two scores can be, so every token chooses the
    same experts (each with the token's own weights).  The stream of a bfloat16 engine differs from the
    exact one by a percent or so after a few layers, which moves a token's scores by several hundredths,
    and among hundreds of tokens some choice always hangs on less than that; a chosen expert that differs
    is no rounding error.  Whole models in bfloat16 are therefore tested with steady choices, and the
    choice itself where the inputs are the same bits on both sides: the router's kernel alone, in both
    dtypes, and whole models in the 32-bit engine."""
    rng = np.random.default_rng(seed)
    out: dict[str, np.ndarray] = {}
    for name, shape in sorted(tensor_shapes(cfg).items()):
        leaf = name.split(".", 1)[-1] if name.startswith("l") and name[1].isdigit() else name
        if leaf in ("norm1", "norm2", "final.norm"):
            values = rng.uniform(-0.5, 0.5, size=shape)
        elif leaf in ("mix.dkv.norm", "mix.dq.norm", "mix.q.norm", "mix.k.norm", "ls1", "ls2"):
            values = rng.uniform(0.5, 1.5, size=shape)
        elif leaf == "mix.sink":
            values = rng.standard_normal(shape) * 1.5
        elif leaf == "mix.vmix":
            values = rng.uniform(0.2, 0.8, size=shape)
        elif leaf == "mlp.correction" and steady_choice:
            values = rng.permutation(shape[0]) * 1.25
        elif leaf == "mlp.correction":
            values = rng.standard_normal(shape) * 0.15
        elif leaf == "mlp.router":
            values = rng.standard_normal(shape) * 2.5 / np.sqrt(shape[1])
        elif leaf == "mlp.shared.sg":
            values = rng.standard_normal(shape) * 2.0 / np.sqrt(shape[1])
        elif name in ("embed", "bigram"):
            values = rng.standard_normal(shape) * 0.4  # (the table is the head too: logits of a few units)
        else:
            values = rng.standard_normal(shape) / np.sqrt(shape[1]) * (2.0 if leaf in ("mix.q", "mix.k", "mix.uq", "mix.uk") else 1.0)
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

"""Recurrent mixers: state of fixed size per request instead of pages of keys and values.

`GatedDeltaRule` (below) keeps a matrix per head that is written by the delta rule.  `MinGRU` is a gated recurrence whose gates read only the current token, so all gates of a
portion come from one stacked product and only the recurrence itself walks the tokens:

    z_t = sigmoid(W_z h_t + b_z)        u_t = W_x h_t + b_x
    c_t = u_t + 1/2  where u_t >= 0,  sigmoid(u_t)  where u_t < 0
    S_t = (1 - z_t) S_(t-1) + z_t c_t   (per column)
    y_t = W_o (S_t * silu(W_g h_t))

S starts at zero, is float32 whatever the compute dtype, and lives in the request's state
slot between steps (`cache.state`, one row per slot).
"""

from __future__ import annotations

import torch

from mini_infer_amd import ops
from mini_infer_amd.parts.base import (
    CacheNeeds,
    LayerCache,
    Mixer,
    ParamSpec,
    StateNeeds,
    StepContext,
    TensorGetter,
)
from mini_infer_amd.parts.linear import Linear
from mini_infer_amd.registry import register_mixer

DEFAULT_NAMES = {"z": "z", "x": "x", "g": "g", "o": "o", "z_bias": "z.b", "x_bias": "x.b"}


class MinGRU(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, width: int, dtype: torch.dtype, device, *, names: dict[str, str] | None = None,
                 suffix: str = "") -> None:
        super().__init__(dtype, device)
        if hidden_size <= 0 or width <= 0:
            raise ValueError(f"minGRU needs positive sizes, got hidden_size={hidden_size} width={width}")
        self.hidden_size = hidden_size
        self.width = width
        self.names = {**DEFAULT_NAMES, **(names or {})}
        n = self.names
        # one product yields [z | x | g] for every token of the step
        self.zxg = Linear(hidden_size, [width, width, width], [n["z"], n["x"], n["g"]], dtype, device, suffix=suffix)
        self.out = Linear(width, hidden_size, n["o"], dtype, device, suffix=suffix)
        self.bias_z: torch.Tensor | None = None
        self.bias_x: torch.Tensor | None = None

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        return {
            **self.zxg.param_specs(prefix),
            **self.out.param_specs(prefix),
            prefix + self.names["z_bias"]: ParamSpec((self.width,), dtype="float32"),
            prefix + self.names["x_bias"]: ParamSpec((self.width,), dtype="float32"),
        }

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.zxg.load_params(prefix, get)
        self.out.load_params(prefix, get)
        self.bias_z = get(prefix + self.names["z_bias"]).float().contiguous()
        self.bias_x = get(prefix + self.names["x_bias"]).float().contiguous()

    def cache_needs(self, page_size: int) -> CacheNeeds:
        return CacheNeeds(state=StateNeeds((self.width,), torch.float32))

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache, writes_cache: bool = True) -> torch.Tensor:
        if not writes_cache:
            raise NotImplementedError("a recurrent mixer owns its state; it cannot read another call's")
        assert self.bias_z is not None and self.bias_x is not None, "minGRU used before its weights were loaded"
        assert isinstance(cache.state, torch.Tensor), "minGRU needs its state rows from the cache manager"
        assert self.zxg.weight is not None
        if (
            ctx.host_cu_seqlens_q is not None
            and ctx.max_q_len == 1
            and x.shape[0] == ctx.state_slots.numel()
            and ops.linear_gru_takes(x, self.zxg.weight)
        ):
            # a step of single tokens, few rows: the stacked product and the step of the recurrence are one kernel
            gated = ops.linear_gru(x, self.zxg.weight, self.bias_z, self.bias_x, cache.state, ctx.state_slots)
            return self.out.forward(gated)
        projected = self.zxg.forward(x)
        # (the most rows a request brings: known only where the host knows the step's boundaries)
        max_rows = ctx.max_q_len if ctx.host_cu_seqlens_q is not None else None
        gated = ops.gated_scan(projected, self.bias_z, self.bias_x, cache.state, ctx.cu_seqlens_q, ctx.state_slots, max_rows)
        return self.out.forward(gated)


@register_mixer("min_gru")
def build_min_gru(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> MinGRU:
    return MinGRU(int(desc["hidden_size"]), int(desc["width"]), dtype, device, names=desc.get("names"),
                  suffix=str(desc.get("suffix", "")))


DELTA_NAMES = {
    "q": "q", "k": "k", "v": "v", "write": "b", "decay": "a", "gate": "g", "out": "o", "conv": ".conv",
    "rate": "A_log", "step_bias": "dt_bias", "norm": "norm",
}
DELTA_UNIT_NORM_EPS = 1e-6  # inside the root that makes q and k unit vectors (fixed by the kernel)


class GatedDeltaRule(Mixer):
    """A matrix state S (head_dim x v_head_dim, float32) per head, written by the gated delta rule:

        q, k, v = silu(short_conv(W_q h)), silu(short_conv(W_k h)), silu(short_conv(W_v h))
        q, k  <- unit vectors per head (q also times head_dim^-1/2)
        w_t = logistic(W_b h)                  d_t = exp(-exp(A) * softplus(W_a h + bias))   (per head)
        S <- d_t S;   u = w_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t
        y_t = W_o (rms_norm(o_t) * weight * silu(W_g h))

    with `num_kv_heads` heads of q and k shared by groups of the `num_heads` value heads.  A
    request's S and the last taps-1 inputs of the three convolutions live in its state slot."""

    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int, taps: int,
                 norm_eps: float, dtype: torch.dtype, device, *, names: dict[str, str] | None = None, suffix: str = "") -> None:
        super().__init__(dtype, device)
        for what, value in (("hidden_size", hidden_size), ("num_heads", num_heads), ("num_kv_heads", num_kv_heads),
                            ("head_dim", head_dim), ("v_head_dim", v_head_dim), ("taps", taps)):
            if value <= 0:
                raise ValueError(f"gated delta rule: {what} must be positive, got {value}")
        if num_heads % num_kv_heads != 0:
            raise ValueError(f"num_heads={num_heads} is not a multiple of num_kv_heads={num_kv_heads}")
        if head_dim > 256 or v_head_dim > 256 or taps > 16:
            raise ValueError(f"gated delta rule: the kernels take heads up to 256 x 256 and 16 taps, got {head_dim} x {v_head_dim}, {taps}")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.head_dim, self.v_head_dim, self.taps, self.norm_eps = head_dim, v_head_dim, taps, float(norm_eps)
        self.names = {**DELTA_NAMES, **(names or {})}
        self.suffix = suffix
        n = self.names
        qk, vw = num_kv_heads * head_dim, num_heads * v_head_dim
        self.channels = 2 * qk + vw  # what passes the convolution: q | k | v
        # one product yields [q | k | v | write | decay | gate] for every token of the step
        self.inputs = Linear(hidden_size, [qk, qk, vw, num_heads, num_heads, vw],
                             [n["q"], n["k"], n["v"], n["write"], n["decay"], n["gate"]], dtype, device, suffix=suffix)
        self.col_write, self.col_decay, self.col_gate = self.channels, self.channels + num_heads, self.channels + 2 * num_heads
        self.out = Linear(vw, hidden_size, n["out"], dtype, device, suffix=suffix)
        self.conv_weight: torch.Tensor | None = None  # float32 [channels, taps]
        self.rate: torch.Tensor | None = None
        self.step_bias: torch.Tensor | None = None
        self.norm_weight: torch.Tensor | None = None

    def _conv_names(self, prefix: str) -> list[tuple[str, int]]:
        n, qk = self.names, self.num_kv_heads * self.head_dim
        return [(prefix + n[part] + self.suffix + n["conv"], rows)
                for part, rows in (("q", qk), ("k", qk), ("v", self.num_heads * self.v_head_dim))]

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        n = self.names
        specs = {**self.inputs.param_specs(prefix), **self.out.param_specs(prefix)}
        for name, rows in self._conv_names(prefix):
            specs[name] = ParamSpec((rows, self.taps), dtype="float32")
        specs[prefix + n["rate"]] = ParamSpec((self.num_heads,), dtype="float32")
        specs[prefix + n["step_bias"]] = ParamSpec((self.num_heads,), dtype="float32")
        specs[prefix + n["norm"]] = ParamSpec((self.v_head_dim,), init="norm_weight", dtype="float32")
        return specs

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        n = self.names
        self.inputs.load_params(prefix, get)
        self.out.load_params(prefix, get)
        self.conv_weight = torch.cat([get(name).float() for name, _ in self._conv_names(prefix)], dim=0).contiguous()
        self.rate = get(prefix + n["rate"]).float().contiguous()
        self.step_bias = get(prefix + n["step_bias"]).float().contiguous()
        self.norm_weight = get(prefix + n["norm"]).float().contiguous()

    def cache_needs(self, page_size: int) -> CacheNeeds:
        state = {"recurrent": StateNeeds(ops.delta_state_shape(self.num_heads, self.head_dim, self.v_head_dim), torch.float32)}
        if self.taps > 1:
            state["tail"] = StateNeeds((self.taps - 1, self.channels), self.dtype)
        return CacheNeeds(state=state)

    def forward(self, x, ctx: StepContext, cache: LayerCache, writes_cache: bool = True) -> torch.Tensor:
        if not writes_cache:
            raise NotImplementedError("a recurrent mixer owns its state; it cannot read another call's")
        assert self.conv_weight is not None and self.rate is not None, "gated delta rule used before its weights were loaded"
        assert isinstance(cache.state, dict), "the gated delta rule needs its state rows from the cache manager"
        if hasattr(x, "finish"):
            x = x.finish()
        proj = self.inputs.forward(x)
        if self.taps > 1:
            tail = cache.state["tail"]
        else:  # (no taps before the current one: nothing to remember)
            tail = torch.empty((2, 0, self.channels), dtype=proj.dtype, device=proj.device)
        qkv = ops.short_conv(proj, self.channels, self.conv_weight, tail, ctx.cu_seqlens_q, ctx.state_slots, ctx.token_request)
        mixed = ops.gated_delta(
            qkv, proj, self.col_write, self.col_decay, self.col_gate, self.rate, self.step_bias, self.norm_weight,
            cache.state["recurrent"], ctx.cu_seqlens_q, ctx.state_slots, heads=self.num_heads, kv_heads=self.num_kv_heads,
            dim=self.head_dim, vdim=self.v_head_dim, eps=self.norm_eps,
        )
        return self.out.forward(mixed)


@register_mixer("gated_delta_rule")
def build_gated_delta_rule(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> GatedDeltaRule:
    return GatedDeltaRule(
        int(desc["hidden_size"]), int(desc["num_heads"]), int(desc["num_kv_heads"]), int(desc["head_dim"]),
        int(desc["v_head_dim"]), int(desc["taps"]), float(desc["norm_eps"]), dtype, device, names=desc.get("names"),
        suffix=str(desc.get("suffix", "")),
    )


GLA_NAMES = {"q": "q", "k": "k", "v": "v", "gate": "g", "out": "o", "decay_down": "a1", "decay_up": "a2",
             "decay_bias": "a2.b", "norm": "norm"}


class GatedLinearAttention(Mixer):
    """Linear attention whose matrix state S (head_dim x v_head_dim, float32) per head decays by a
    gate per key channel:

        q = W_q h * head_dim^-1/2,  k = W_k h,  v = W_v h
        a = logistic(W_a2 (W_a1 h) + bias) ^ (1 / tau)                      (per head and key channel)
        S <- diag(a_t) S + k_t v_t^T;    o_t = S^T q_t
        y_t = W_o (rms_norm(o_t) * weight * silu(W_g h))                    (norm per head over v_head_dim)

    A request's S lives in its state slot."""

    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, v_head_dim: int, decay_rank: int, tau: float,
                 norm_eps: float, dtype: torch.dtype, device, *, names: dict[str, str] | None = None, suffix: str = "") -> None:
        super().__init__(dtype, device)
        for what, value in (("hidden_size", hidden_size), ("num_heads", num_heads), ("head_dim", head_dim),
                            ("v_head_dim", v_head_dim), ("decay_rank", decay_rank)):
            if value <= 0:
                raise ValueError(f"gated linear attention: {what} must be positive, got {value}")
        if tau <= 0:
            raise ValueError(f"gated linear attention: tau must be positive, got {tau}")
        self.hidden_size, self.num_heads, self.head_dim, self.v_head_dim = hidden_size, num_heads, head_dim, v_head_dim
        self.decay_rank, self.tau, self.norm_eps = decay_rank, float(tau), float(norm_eps)
        self.names = {**GLA_NAMES, **(names or {})}
        self.suffix = suffix
        ops.decay_state_shape(num_heads, head_dim, v_head_dim)  # (refuses widths the kernel does not take)
        n, qk, vw = self.names, num_heads * head_dim, num_heads * v_head_dim
        # one product yields [q | k | v | gate | decay, narrow] for every token of the step
        self.inputs = Linear(hidden_size, [qk, qk, vw, vw, decay_rank],
                             [n["q"], n["k"], n["v"], n["gate"], n["decay_down"]], dtype, device, suffix=suffix)
        self.col_k, self.col_v, self.col_gate, self.col_decay = qk, 2 * qk, 2 * qk + vw, 2 * qk + 2 * vw
        self.decay_up = Linear(decay_rank, qk, n["decay_up"], dtype, device, suffix=suffix)
        self.out = Linear(vw, hidden_size, n["out"], dtype, device, suffix=suffix)
        self.decay_bias: torch.Tensor | None = None
        self.norm_weight: torch.Tensor | None = None

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        n = self.names
        return {
            **self.inputs.param_specs(prefix), **self.decay_up.param_specs(prefix), **self.out.param_specs(prefix),
            prefix + n["decay_bias"]: ParamSpec((self.num_heads * self.head_dim,), dtype="float32"),
            prefix + n["norm"]: ParamSpec((self.v_head_dim,), init="norm_weight", dtype="float32"),
        }

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        for part in (self.inputs, self.decay_up, self.out):
            part.load_params(prefix, get)
        self.decay_bias = get(prefix + self.names["decay_bias"]).float().contiguous()
        self.norm_weight = get(prefix + self.names["norm"]).float().contiguous()

    def cache_needs(self, page_size: int) -> CacheNeeds:
        return CacheNeeds(state=StateNeeds(ops.decay_state_shape(self.num_heads, self.head_dim, self.v_head_dim), torch.float32))

    def forward(self, x, ctx: StepContext, cache: LayerCache, writes_cache: bool = True) -> torch.Tensor:
        if not writes_cache:
            raise NotImplementedError("a recurrent mixer owns its state; it cannot read another call's")
        assert self.decay_bias is not None and self.norm_weight is not None, "gated linear attention used before its weights were loaded"
        assert isinstance(cache.state, torch.Tensor), "gated linear attention needs its state rows from the cache manager"
        if hasattr(x, "finish"):
            x = x.finish()
        proj = self.inputs.forward(x)
        logits = self.decay_up.forward(proj[:, self.col_decay:self.col_decay + self.decay_rank])
        readout = ops.decay_scan(
            proj, 0, proj, self.col_k, proj, self.col_v, logits, 0, self.decay_bias, cache.state, ctx.cu_seqlens_q,
            ctx.state_slots, heads=self.num_heads, groups=self.num_heads, dim=self.head_dim, vdim=self.v_head_dim,
            per_head=False, inv_tau=1.0 / self.tau, q_scale=self.head_dim ** -0.5,
        )
        mixed = ops.readout_gate_norm(readout, proj[:, self.col_gate:], self.norm_weight, group_width=self.v_head_dim,
                                      gate_first=False, eps=self.norm_eps)
        return self.out.forward(mixed)


@register_mixer("gated_linear_attention")
def build_gated_linear_attention(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> GatedLinearAttention:
    return GatedLinearAttention(
        int(desc["hidden_size"]), int(desc["num_heads"]), int(desc["head_dim"]), int(desc["v_head_dim"]),
        int(desc["decay_rank"]), float(desc["tau"]), float(desc["norm_eps"]), dtype, device, names=desc.get("names"),
        suffix=str(desc.get("suffix", "")),
    )


SSD_NAMES = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "step_bias": "dt_bias", "rate": "A_log", "skip": "D",
             "norm": "norm", "out": "o"}


class StateSpaceDuality(Mixer):
    """A selective state-space layer with one decay per head (the recurrent form of state-space
    duality).  One product yields [z | x | B | C | dt]; x, B and C pass a short causal convolution
    with a bias and silu; then per head, with B and C shared by the heads of a group,

        dt = softplus(dt + bias);   S <- exp(-exp(rate) dt) S + dt B_t x_t^T;   y_t = S^T C_t + skip * x_t

    (S is state x v_head_dim, float32).  y times silu(z) is RMS-normed in `norm_groups` equal
    parts, times a weight, and projected out.  A request's S and the last taps - 1 inputs of the
    convolution live in its state slot."""

    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, v_head_dim: int, state_size: int, groups: int, taps: int,
                 norm_groups: int, norm_eps: float, dtype: torch.dtype, device, *, names: dict[str, str] | None = None,
                 suffix: str = "") -> None:
        super().__init__(dtype, device)
        for what, value in (("hidden_size", hidden_size), ("num_heads", num_heads), ("v_head_dim", v_head_dim),
                            ("state_size", state_size), ("groups", groups), ("taps", taps), ("norm_groups", norm_groups)):
            if value <= 0:
                raise ValueError(f"state-space layer: {what} must be positive, got {value}")
        self.inner = num_heads * v_head_dim
        if num_heads % groups != 0 or self.inner % norm_groups != 0:
            raise ValueError(f"state-space layer: heads={num_heads} must be a multiple of groups={groups}, "
                             f"heads*v_head_dim={self.inner} of norm_groups={norm_groups}")
        if taps > 16:
            raise ValueError(f"state-space layer: the convolution kernel takes up to 16 taps, got {taps}")
        self.hidden_size, self.num_heads, self.v_head_dim, self.state_size = hidden_size, num_heads, v_head_dim, state_size
        self.groups, self.taps, self.norm_groups, self.norm_eps = groups, taps, norm_groups, float(norm_eps)
        self.names = {**SSD_NAMES, **(names or {})}
        ops.decay_state_shape(num_heads, state_size, v_head_dim)
        self.channels = self.inner + 2 * groups * state_size  # what passes the convolution: x | B | C
        n = self.names
        self.inputs = Linear(hidden_size, 2 * self.inner + 2 * groups * state_size + num_heads, n["in"], dtype, device, suffix=suffix)
        self.out = Linear(self.inner, hidden_size, n["out"], dtype, device, suffix=suffix)
        self.conv_weight: torch.Tensor | None = None
        self.conv_bias: torch.Tensor | None = None
        self.step_bias: torch.Tensor | None = None
        self.rate: torch.Tensor | None = None
        self.skip: torch.Tensor | None = None
        self.norm_weight: torch.Tensor | None = None

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        n = self.names
        return {
            **self.inputs.param_specs(prefix), **self.out.param_specs(prefix),
            prefix + n["conv"]: ParamSpec((self.channels, self.taps), dtype="float32"),
            prefix + n["conv_bias"]: ParamSpec((self.channels,), dtype="float32"),
            prefix + n["step_bias"]: ParamSpec((self.num_heads,), dtype="float32"),
            prefix + n["rate"]: ParamSpec((self.num_heads,), dtype="float32"),
            prefix + n["skip"]: ParamSpec((self.num_heads,), init="norm_weight", dtype="float32"),
            prefix + n["norm"]: ParamSpec((self.inner,), init="norm_weight", dtype="float32"),
        }

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        n = self.names
        self.inputs.load_params(prefix, get)
        self.out.load_params(prefix, get)
        self.conv_weight = get(prefix + n["conv"]).float().contiguous()
        self.conv_bias = get(prefix + n["conv_bias"]).float().contiguous()
        self.step_bias = get(prefix + n["step_bias"]).float().contiguous()
        self.rate = get(prefix + n["rate"]).float().contiguous()
        self.skip = get(prefix + n["skip"]).float().contiguous()
        self.norm_weight = get(prefix + n["norm"]).float().contiguous()

    def cache_needs(self, page_size: int) -> CacheNeeds:
        state = {"recurrent": StateNeeds(ops.decay_state_shape(self.num_heads, self.state_size, self.v_head_dim), torch.float32)}
        if self.taps > 1:
            state["tail"] = StateNeeds((self.taps - 1, self.channels), self.dtype)
        return CacheNeeds(state=state)

    def forward(self, x, ctx: StepContext, cache: LayerCache, writes_cache: bool = True) -> torch.Tensor:
        if not writes_cache:
            raise NotImplementedError("a recurrent mixer owns its state; it cannot read another call's")
        assert self.conv_weight is not None and self.rate is not None, "state-space layer used before its weights were loaded"
        assert isinstance(cache.state, dict), "the state-space layer needs its state rows from the cache manager"
        if hasattr(x, "finish"):
            x = x.finish()
        proj = self.inputs.forward(x)  # [z | x | B | C | dt]
        if self.taps > 1:
            tail = cache.state["tail"]
        else:
            tail = torch.empty((2, 0, self.channels), dtype=proj.dtype, device=proj.device)
        conv = ops.short_conv(proj[:, self.inner:], self.channels, self.conv_weight, tail, ctx.cu_seqlens_q, ctx.state_slots,
                              ctx.token_request, bias=self.conv_bias)  # [x | B | C]
        span = self.groups * self.state_size
        readout = ops.decay_scan(
            conv, self.inner + span, conv, self.inner, conv, 0, proj, self.inner + self.channels, self.step_bias,
            cache.state["recurrent"], ctx.cu_seqlens_q, ctx.state_slots, heads=self.num_heads, groups=self.groups,
            dim=self.state_size, vdim=self.v_head_dim, per_head=True, rate=self.rate, skip=self.skip,
        )
        mixed = ops.readout_gate_norm(readout, proj, self.norm_weight, group_width=self.inner // self.norm_groups,
                                      gate_first=True, eps=self.norm_eps)
        return self.out.forward(mixed)


@register_mixer("state_space_duality")
def build_state_space_duality(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> StateSpaceDuality:
    return StateSpaceDuality(
        int(desc["hidden_size"]), int(desc["num_heads"]), int(desc["v_head_dim"]), int(desc["state_size"]), int(desc["groups"]),
        int(desc["taps"]), int(desc["norm_groups"]), float(desc["norm_eps"]), dtype, device, names=desc.get("names"),
        suffix=str(desc.get("suffix", "")),
    )

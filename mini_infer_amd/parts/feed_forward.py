"""Dense gated feed-forward: `down(act(gate(x)) * up(x))`, no biases; act is silu unless a
layer's description says otherwise (the tanh form of gelu is the other one built).

Formula: models/blocks/swiglu.py:44-46 and activations.py:36-45 of the
reference.  Gate and up are two tensors in the checkpoint; they are stacked at
load so one product yields [gate | up], and the activation reads both halves
(the reference runs two products and one fused SiLU*mul kernel); for few rows
the product and the activation are one kernel.
"""

from __future__ import annotations

import torch

from mini_infer_amd import ops
from mini_infer_amd.parts.base import FeedForward, ParamSpec, StepContext, TensorGetter
from mini_infer_amd.parts.linear import Linear
from mini_infer_amd.registry import register_feed_forward


class SwiGLU(FeedForward):
    graph_safe = True
    takes_scaled_rows = True
    can_defer_output = True

    ACTIVATIONS = ("silu", "gelu_tanh")

    def __init__(self, hidden_size: int, intermediate_size: int, dtype: torch.dtype, device, *, activation: str = "silu",
                 names: tuple[str, str, str] = ("gate_proj", "up_proj", "down_proj"), suffix: str = ".weight") -> None:
        super().__init__(dtype, device)
        if activation not in self.ACTIVATIONS:
            raise NotImplementedError(f"gated feed-forward activation {activation!r}; built: {self.ACTIVATIONS}")
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.activation = activation
        self.gate_up = Linear(
            hidden_size, [intermediate_size, intermediate_size], [names[0], names[1]], dtype, device, suffix=suffix
        )
        self.down = Linear(intermediate_size, hidden_size, names[2], dtype, device, suffix=suffix)
        if activation != "silu":  # the kernels that fold a norm's factors or the down product in are silu's
            self.takes_scaled_rows = False

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        return {**self.gate_up.param_specs(prefix), **self.down.param_specs(prefix)}

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.gate_up.load_params(prefix, get)
        self.down.load_params(prefix, get)

    def wants_scaled_rows(self, rows: int) -> bool:
        """Where the gated product runs as the weight-streaming kernel that applies the rows' factors."""
        return (self.activation == "silu" and self.dtype == torch.bfloat16
                and ops.scaled_rows_product_takes(rows, self.gate_up.weight, self.hidden_size))

    def forward(self, x: "torch.Tensor | ops.ScaledRows", ctx: StepContext) -> torch.Tensor:
        assert self.gate_up.weight is not None, "SwiGLU used before its weights were loaded"
        assert self.down.weight is not None
        if self.activation == "silu":
            act = ops.linear_swiglu(x, self.gate_up.weight)
        else:
            if isinstance(x, ops.ScaledRows):
                x = x.finish()
            act = ops.linear_geglu(x, self.gate_up.weight)
        if (
            self.emit_pending_output
            and self.dtype == torch.bfloat16
            and ops.pending_product_pays(act.shape[0], self.hidden_size, self.intermediate_size, self.emit_partial_sums)
        ):
            # few rows: the down product is left to the norm that follows (one kernel makes it,
            # adds it to the residual and begins the norm)
            return ops.PendingProduct(act, self.down.weight)
        return self.down.forward(act, partial_ok=self.emit_partial_sums)


@register_feed_forward("swiglu")
def build_swiglu(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> SwiGLU:
    extra = {k: desc[k] for k in ("activation", "suffix") if k in desc}
    if "names" in desc:
        extra["names"] = tuple(desc["names"])
    return SwiGLU(int(desc["hidden_size"]), int(desc["intermediate_size"]), dtype, device, **extra)


class PolyNormFeedForward(FeedForward):
    """Dense, ungated: `down(act(up(x)))` with a polynomial activation of normed powers,

        act(z) = a N(z) + b N(z^2) + c N(z^3) + e,     N(v) = v / sqrt(mean(v^2) + eps)

    where the powers are elementwise and the mean runs over a token's feed-forward values.
    The four numbers are one float32 tensor."""

    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, eps: float, dtype: torch.dtype, device, *,
                 names: tuple[str, str, str] = ("up", "down", "act"), suffix: str = "") -> None:
        super().__init__(dtype, device)
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.eps = float(eps)
        self.act_name = names[2]
        self.up = Linear(hidden_size, intermediate_size, names[0], dtype, device, suffix=suffix)
        self.down = Linear(intermediate_size, hidden_size, names[1], dtype, device, suffix=suffix)
        self.coefficients: torch.Tensor | None = None

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        return {**self.up.param_specs(prefix), **self.down.param_specs(prefix),
                prefix + self.act_name: ParamSpec((4,), dtype="float32")}

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.up.load_params(prefix, get)
        self.down.load_params(prefix, get)
        self.coefficients = get(prefix + self.act_name).float().contiguous()

    def forward(self, x, ctx: StepContext) -> torch.Tensor:
        assert self.coefficients is not None, "feed-forward used before its weights were loaded"
        if isinstance(x, ops.ScaledRows):
            x = x.finish()
        return self.down.forward(ops.poly_norm(self.up.forward(x), self.coefficients, self.eps))


@register_feed_forward("dense_poly_norm")
def build_poly_norm_feed_forward(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> PolyNormFeedForward:
    extra = {k: desc[k] for k in ("names", "suffix") if k in desc}
    if "names" in extra:
        extra["names"] = tuple(extra["names"])
    return PolyNormFeedForward(int(desc["hidden_size"]), int(desc["intermediate_size"]), float(desc["eps"]), dtype, device, **extra)


class _SharedTable:
    """A table that several parts of one model read slices of: loaded once per load pass."""

    def __init__(self, name: str, shape: tuple[int, int]) -> None:
        self.name, self.shape = name, shape
        self.tensor: torch.Tensor | None = None
        self._loaded_with = None

    def load(self, get: TensorGetter) -> torch.Tensor:
        if self.tensor is None or self._loaded_with is not get:
            self.tensor, self._loaded_with = get(self.name).contiguous(), get
        return self.tensor


class TokenSideInput(FeedForward):
    """A per-layer input that depends on the token's identity: the layer's slice
    `table[token, first : first + dim]` of a table shared by all layers, gated by the stream,

        y = proj(gelu_tanh(gate(x)) * slice)

    `table_name` is the tensor's whole name (it belongs to the model, not to the layer); the
    parts of one model that name the same table share one copy through `shared`."""

    graph_safe = True

    def __init__(self, hidden_size: int, dim: int, first_col: int, table: _SharedTable, dtype: torch.dtype, device, *,
                 names: tuple[str, str] = ("gate", "proj"), suffix: str = "") -> None:
        super().__init__(dtype, device)
        if first_col < 0 or first_col + dim > table.shape[1]:
            raise ValueError(f"columns {first_col}..{first_col + dim} lie outside a table of {table.shape[1]} columns")
        self.hidden_size, self.dim, self.first_col, self.table = hidden_size, dim, first_col, table
        self.gate = Linear(hidden_size, dim, names[0], dtype, device, suffix=suffix)
        self.proj = Linear(dim, hidden_size, names[1], dtype, device, suffix=suffix)

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        return {**self.gate.param_specs(prefix), **self.proj.param_specs(prefix),
                self.table.name: ParamSpec(self.table.shape)}

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.gate.load_params(prefix, get)
        self.proj.load_params(prefix, get)
        self.table.load(get)

    def forward(self, x, ctx: StepContext) -> torch.Tensor:
        assert self.table.tensor is not None, "side input used before its table was loaded"
        if isinstance(x, ops.ScaledRows):
            x = x.finish()
        assert self.gate.weight is not None
        # (few rows: the gate product, its activation and the gather are one kernel)
        gated = ops.linear_gelu_table(x, self.gate.weight, self.table.tensor, ctx.token_ids, self.first_col)
        return self.proj.forward(gated)


@register_feed_forward("token_side_input")
def build_token_side_input(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> TokenSideInput:
    shared = {} if shared is None else shared
    name, shape = str(desc["table_name"]), (int(desc["vocab_size"]), int(desc["table_columns"]))
    key = ("shared_table", name)
    table = shared.get(key)
    if table is None:
        table = shared[key] = _SharedTable(name, shape)
    elif table.shape != shape:
        raise ValueError(f"table {name!r} is described as {shape} and as {table.shape}")
    extra = {k: desc[k] for k in ("names", "suffix") if k in desc}
    if "names" in extra:
        extra["names"] = tuple(extra["names"])
    return TokenSideInput(int(desc["hidden_size"]), int(desc["dim"]), int(desc["first_col"]), table, dtype, device, **extra)


GATE_SLOPE = 1.702  # of the logistic that gates: g * logistic(1.702 g) approximates gelu(g)


class ClampedGatedFeedForward(FeedForward):
    """Gated, with biases on all three products and both branches clamped before they meet:

        g = min(W_gate x + b_gate, limit)          u = clamp(W_up x + b_up, -limit, limit)
        y = W_down (g * logistic(slope * g) * (u + 1)) + b_down

    Gate and up are stacked at load so one product yields [gate | up]; their biases and the
    activation are one kernel.  The down product's bias is not added here: `forward` returns the
    product, and `output_bias` (float32) is for whoever adds the result to the stream to add with
    it (`ops.StreamUpdate.bias`)."""

    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, limit: float, dtype: torch.dtype, device, *,
                 slope: float = GATE_SLOPE, names: tuple[str, str, str] = ("gate", "up", "down"), suffix: str = "",
                 bias_suffix: str = ".b") -> None:
        super().__init__(dtype, device)
        if limit <= 0:
            raise ValueError(f"clamped gated feed-forward: the limit must be positive, got {limit}")
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.limit, self.slope = float(limit), float(slope)
        self.names, self.suffix, self.bias_suffix = tuple(names), suffix, bias_suffix
        self.gate_up = Linear(hidden_size, [intermediate_size, intermediate_size], [names[0], names[1]], dtype, device, suffix=suffix)
        self.down = Linear(intermediate_size, hidden_size, names[2], dtype, device, suffix=suffix)
        self.gate_up_bias: torch.Tensor | None = None
        self.output_bias: torch.Tensor | None = None

    def _bias_name(self, prefix: str, which: int) -> str:
        return prefix + self.names[which] + self.suffix + self.bias_suffix

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        return {
            **self.gate_up.param_specs(prefix), **self.down.param_specs(prefix),
            self._bias_name(prefix, 0): ParamSpec((self.intermediate_size,), dtype="float32"),
            self._bias_name(prefix, 1): ParamSpec((self.intermediate_size,), dtype="float32"),
            self._bias_name(prefix, 2): ParamSpec((self.hidden_size,), dtype="float32"),
        }

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.gate_up.load_params(prefix, get)
        self.down.load_params(prefix, get)
        self.gate_up_bias = torch.cat([get(self._bias_name(prefix, 0)).float(), get(self._bias_name(prefix, 1)).float()]).contiguous()
        self.output_bias = get(self._bias_name(prefix, 2)).float().contiguous()

    def forward(self, x, ctx: StepContext) -> torch.Tensor:
        assert self.gate_up_bias is not None, "feed-forward used before its weights were loaded"
        if isinstance(x, ops.ScaledRows):
            x = x.finish()
        assert self.gate_up.weight is not None
        # (few rows: the product, the biases, the clamps and the activation are one kernel)
        act = ops.linear_clamped_glu(x, self.gate_up.weight, self.gate_up_bias, self.limit, self.slope)
        return self.down.forward(act)


@register_feed_forward("clamped_glu")
def build_clamped_gated_feed_forward(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> ClampedGatedFeedForward:
    extra = {k: desc[k] for k in ("slope", "suffix", "bias_suffix") if k in desc}
    if "names" in desc:
        extra["names"] = tuple(desc["names"])
    return ClampedGatedFeedForward(int(desc["hidden_size"]), int(desc["intermediate_size"]), float(desc["limit"]), dtype, device, **extra)


class RoutedExperts(FeedForward):
    """A mixture of experts: `experts` small gated feed-forwards (`W_down (silu(W_gate x) * W_up x)`, no
    biases), of which every token goes through `top`.

        z = R x (float32)        s = softmax(z) over ALL router outputs        choice = s + correction
        y = sum over the `top` outputs e with the largest choice of  (s_e * route_scale) * expert_e(x)

    The weights are the scores themselves (without the correction, not renormalized).  The last
    `identity` router outputs stand for experts without tensors whose output is their input.  A
    shared expert of the same form may run for every token beside them, gated by one number a
    token, `logistic(w_sg . x)`.

    Few rows (and every step that is recorded to be replayed) run expert by expert without the host
    knowing anything: the (token, expert) pairs are listed by expert on the device, and every chosen
    expert's weights are streamed once for up to eight of its rows at a time (sizes that are not read
    16 bytes at a time work each pair on its own instead, the expert's weights read by index).  Many
    rows are sorted by expert and every chosen expert runs the engine's own products once over all
    its rows.  Router, correction and the shared expert's gate row stay float32."""

    graph_safe = True

    # rows * top pairs, times the bytes of an expert, from which on sorting by expert pays for the
    # launches of a loop over the experts (each pair reads its expert's weights once otherwise)
    GROUPED_BYTES_PER_EXPERT = 64 << 20

    def __init__(self, hidden_size: int, intermediate_size: int, experts: int, top: int, dtype: torch.dtype, device, *,
                 identity: int = 0, route_scale: float = 1.0, correction: bool = True, shared_size: int | None = None,
                 names: dict[str, str] | None = None) -> None:
        super().__init__(dtype, device)
        if experts <= 0 or identity < 0 or not 0 < top <= experts + identity:
            raise ValueError(f"routed experts: {top} of {experts} experts + {identity} identity experts")
        if experts + identity > ops.kernels.ROUTER_MAX_OUTPUTS:
            raise ValueError(f"routed experts: the router takes at most {ops.kernels.ROUTER_MAX_OUTPUTS} outputs")
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.experts, self.identity, self.top, self.route_scale = experts, identity, top, float(route_scale)
        self.has_correction, self.shared_size = bool(correction), shared_size
        self.names = {"router": "router", "correction": "correction", "expert": "e{}.", "gate": "gate", "up": "up",
                      "down": "down", "shared": "shared.", "shared_gate": "shared.sg", **(names or {})}
        self.shared = None if shared_size is None else SwiGLU(
            hidden_size, shared_size, dtype, device,
            names=tuple(self.names["shared"] + self.names[k] for k in ("gate", "up", "down")), suffix="")
        if self.shared is not None:
            self.shared.takes_scaled_rows = False
        self.router: torch.Tensor | None = None  # float32 [experts + identity, hidden]
        self.correction: torch.Tensor | None = None  # float32 [experts + identity]
        self.shared_gate_row: torch.Tensor | None = None  # float32 [hidden]
        self.gate_up: torch.Tensor | None = None  # [experts, 2 * ff, hidden]
        self.down: torch.Tensor | None = None  # [experts, hidden, ff]
        self.force_form: str | None = None  # "few", "by_expert" or "grouped": for tests and measurements

    def _expert_name(self, prefix: str, e: int, which: str) -> str:
        return prefix + self.names["expert"].format(e) + self.names[which]

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        outputs, ff, hidden = self.experts + self.identity, self.intermediate_size, self.hidden_size
        specs = {prefix + self.names["router"]: ParamSpec((outputs, hidden), dtype="float32")}
        if self.has_correction:
            specs[prefix + self.names["correction"]] = ParamSpec((outputs,), dtype="float32")
        for e in range(self.experts):
            specs[self._expert_name(prefix, e, "gate")] = ParamSpec((ff, hidden))
            specs[self._expert_name(prefix, e, "up")] = ParamSpec((ff, hidden))
            specs[self._expert_name(prefix, e, "down")] = ParamSpec((hidden, ff))
        if self.shared is not None:
            specs.update(self.shared.param_specs(prefix))
            specs[prefix + self.names["shared_gate"]] = ParamSpec((1, hidden), dtype="float32")
        return specs

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.router = get(prefix + self.names["router"]).float().contiguous()
        if self.has_correction:
            self.correction = get(prefix + self.names["correction"]).float().contiguous()
        ff, hidden = self.intermediate_size, self.hidden_size
        first = get(self._expert_name(prefix, 0, "gate"))
        self.gate_up = torch.empty((self.experts, 2 * ff, hidden), dtype=first.dtype, device=first.device)
        self.down = torch.empty((self.experts, hidden, ff), dtype=first.dtype, device=first.device)
        for e in range(self.experts):
            self.gate_up[e, :ff] = get(self._expert_name(prefix, e, "gate"))
            self.gate_up[e, ff:] = get(self._expert_name(prefix, e, "up"))
            self.down[e] = get(self._expert_name(prefix, e, "down"))
        if self.shared is not None:
            self.shared.load_params(prefix, get)
            self.shared_gate_row = get(prefix + self.names["shared_gate"]).float().reshape(-1).contiguous()

    def _grouped(self, rows: int, ctx: StepContext) -> bool:
        if self.force_form is not None:
            return self.force_form == "grouped"
        if ctx.host_cu_seqlens_q is None or torch.cuda.is_current_stream_capturing():
            return False  # (the sorted form reads the experts' row counts on the host)
        element = 2 if self.dtype == torch.bfloat16 else 4
        expert_bytes = 3 * self.intermediate_size * self.hidden_size * element
        return rows * self.top * expert_bytes > self.experts * self.GROUPED_BYTES_PER_EXPERT

    def forward(self, x, ctx: StepContext) -> torch.Tensor:
        assert self.router is not None and self.gate_up is not None and self.down is not None, \
            "feed-forward used before its weights were loaded"
        if hasattr(x, "finish"):
            x = x.finish()
        chosen, weights, gates = ops.route_top_k(x, self.router, self.correction, self.shared_gate_row, top=self.top,
                                                 route_scale=self.route_scale)
        shared = None
        if self.shared is not None:
            shared = self.shared.forward(x, ctx)
            shared = shared.finish() if hasattr(shared, "finish") else shared
        if self._grouped(x.shape[0], ctx):
            run = ops.experts_grouped
        elif self.force_form == "by_expert" or (self.force_form is None and ops.experts_by_expert_take(x, self.gate_up)):
            run = ops.experts_by_expert
        else:
            run = ops.experts_few_rows
        return run(x, self.gate_up, self.down, chosen, weights, shared, gates)


@register_feed_forward("routed_experts")
def build_routed_experts(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> RoutedExperts:
    extra = {k: desc[k] for k in ("identity", "route_scale", "correction", "shared_size", "names") if k in desc}
    return RoutedExperts(int(desc["hidden_size"]), int(desc["intermediate_size"]), int(desc["experts"]), int(desc["top"]),
                         dtype, device, **extra)

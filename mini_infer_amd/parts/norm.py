"""RMSNorm with the residual add folded in.

Formula: models/blocks/rmsnorm.py:81-93 of the reference; the add-then-norm
pairing is its `_add_and_norm` (:63-79) and kernel (rms_norm_kernel.py:109-144).
Here the residual stream is float32 in both compute dtypes, so the sum is
exact to float32 and the statistics see the unrounded sum.
"""

from __future__ import annotations

import torch

from mini_infer_amd import ops
from mini_infer_amd.parts.base import Norm, ParamSpec, TensorGetter
from mini_infer_amd.registry import register_norm


class RMSNorm(Norm):
    graph_safe = True
    takes_partial_sums = True
    takes_pending_products = True

    def __init__(self, hidden_size: int, eps: float, dtype: torch.dtype, device, name: str = "weight") -> None:
        super().__init__(dtype, device)
        self.hidden_size = hidden_size
        self.eps = float(eps)
        self.name = name  # the tensor is `prefix + name`
        self.weight: torch.Tensor | None = None
        self._weight_f32: torch.Tensor | None = None

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        return {prefix + self.name: ParamSpec((self.hidden_size,), init="norm_weight")}

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.weight = get(prefix + self.name).contiguous()
        self._weight_f32 = None

    def add_output(self, y, residual, scale=None, want_cast=False):
        """`residual += y / rms(y) * weight (* scale)`: the norm on a sublayer's output."""
        assert self.weight is not None, "RMSNorm used before its weight was loaded"
        if self._weight_f32 is None:
            self._weight_f32 = self.weight.float().contiguous()
        by_column = self._weight_f32 if scale is None else self._weight_f32 * scale
        return ops.norm_scale_add(y, residual, None, by_column, self.eps, want_cast)

    def forward(
        self,
        delta: "torch.Tensor | ops.PartialSums | ops.PendingProduct | None",
        residual: torch.Tensor,
        rows: torch.Tensor | None = None,
    ) -> "torch.Tensor | ops.ScaledRows":
        assert self.weight is not None, "RMSNorm used before its weight was loaded"
        if isinstance(delta, ops.StreamUpdate):
            # the sublayers' outputs of a layer that adds them together, scaled: the add and
            # the norm are one launch
            return ops.stream_update_norm(delta, residual, self.weight, self.eps, rows)
        if isinstance(delta, ops.PendingProduct):
            # few rows: the product, the add and the norm but for the rows' factors are one
            # kernel, if the part that follows has a kernel that applies the factors in this step
            consumer = self.scaled_rows_consumer
            if (
                self.emit_scaled_rows
                and rows is None
                and consumer is not None
                and consumer.wants_scaled_rows(residual.shape[0])
                and ops.linear_add_norm_takes(delta, residual, self.weight)
            ):
                return ops.linear_add_norm(delta, residual, self.weight, self.eps)
            delta = delta.finish()
        return ops.add_rmsnorm(delta, residual, self.weight, self.eps, rows)


@register_norm("rms_norm")
def build_rms_norm(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> RMSNorm:
    return RMSNorm(int(desc["hidden_size"]), float(desc["eps"]), dtype, device, name=str(desc.get("name", "weight")))


class ScalarGainRMSNorm(Norm):
    """RMS norm whose weight is ONE number for all columns: `x / sqrt(mean(x^2) + eps) * gain`.

    As a final norm (`forward`) it runs the row-wise norm kernel with the gain spread over the
    columns; on a sublayer's output (`add_output`) the one-number form is a kernel argument.
    The gain stays float32."""

    graph_safe = True

    def __init__(self, hidden_size: int, eps: float, dtype: torch.dtype, device, name: str = "weight") -> None:
        super().__init__(dtype, device)
        self.hidden_size = hidden_size
        self.eps = float(eps)
        self.name = name
        self.gain: torch.Tensor | None = None  # float32 [1]
        self._spread: torch.Tensor | None = None  # the gain as a weight row in the compute dtype

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        return {prefix + self.name: ParamSpec((), init="norm_weight", dtype="float32")}

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.gain = get(prefix + self.name).reshape(1).float().contiguous()
        self._spread = self.gain.to(self.dtype).expand(self.hidden_size).contiguous()

    def forward(self, delta, residual, rows=None):
        assert self._spread is not None, "norm used before its gain was loaded"
        if delta is not None and hasattr(delta, "finish"):
            delta = delta.finish()
        return ops.add_rmsnorm(delta, residual, self._spread, self.eps, rows)

    def add_output(self, y, residual, scale=None, want_cast=False):
        assert self.gain is not None, "norm used before its gain was loaded"
        return ops.norm_scale_add(y, residual, self.gain, scale, self.eps, want_cast)


@register_norm("scalar_rms_norm")
def build_scalar_rms_norm(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> ScalarGainRMSNorm:
    return ScalarGainRMSNorm(int(desc["hidden_size"]), float(desc["eps"]), dtype, device, name=str(desc.get("name", "weight")))


class StreamsRMSNorm(Norm):
    """RMS norm in front of a sublayer of a model whose residual stream is kept in several copies
    x_1 .. x_S (float32 [T, S, H]).  It reads `u = sum_s read[s] * x_s` (no `read`: the plain
    sum, which is how such a model ends) and returns `u / sqrt(mean(u^2) + eps) * (offset + w)`:
    `weight_offset=1.0` is a weight stored around zero.

    What the sublayer before it left to be written comes as `ops.StreamsWrite` (the copies are
    rewritten all at once from the old ones through a small matrix, plus the sublayer's output
    times a vector); write, read and norm are one launch.  `read` is set by the block that owns
    the vectors."""

    graph_safe = True

    def __init__(self, hidden_size: int, eps: float, copies: int, dtype: torch.dtype, device, name: str = "weight",
                 weight_offset: float = 0.0) -> None:
        super().__init__(dtype, device)
        if not 1 <= copies <= ops.MAX_STREAM_COPIES:
            raise ValueError(f"a stream is kept in 1..{ops.MAX_STREAM_COPIES} copies, got {copies}")
        self.hidden_size, self.eps, self.copies = hidden_size, float(eps), int(copies)
        self.name, self.weight_offset = name, float(weight_offset)
        self.factor: torch.Tensor | None = None  # float32 [H]: offset + weight
        self.read: torch.Tensor | None = None  # float32 [S], or None for the plain sum

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        init = "norm_weight" if self.weight_offset == 0.0 else "normal"
        return {prefix + self.name: ParamSpec((self.hidden_size,), init=init, dtype="float32")}

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.factor = (get(prefix + self.name).float() + self.weight_offset).contiguous()

    def forward(self, delta, residual: torch.Tensor, rows: torch.Tensor | None = None) -> torch.Tensor:
        assert self.factor is not None, "norm used before its weight was loaded"
        if residual.dim() != 3 or residual.shape[1] != self.copies:
            raise ValueError(f"this norm reads a stream of {self.copies} copies [T, {self.copies}, H], got {tuple(residual.shape)}")
        if delta is not None and not isinstance(delta, ops.StreamsWrite):
            if self.copies != 1:
                raise TypeError("a stream kept in several copies is written through `ops.StreamsWrite` only")
            # one copy: a plain residual add
            delta = delta.finish() if hasattr(delta, "finish") else delta
            one = torch.ones(1, dtype=torch.float32, device=residual.device)
            delta = ops.StreamsWrite(delta, one.reshape(1, 1), one)
        return ops.streams_update_norm(delta, residual, self.read, self.factor, self.eps, self.dtype, rows)


@register_norm("streams_rms_norm")
def build_streams_rms_norm(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> StreamsRMSNorm:
    return StreamsRMSNorm(int(desc["hidden_size"]), float(desc["eps"]), int(desc.get("copies", 1)), dtype, device,
                          name=str(desc.get("name", "weight")), weight_offset=float(desc.get("weight_offset", 0.0)))


class PostRMSNorm(Norm):
    """RMS norm that stands BEHIND the residual sum: `x <- (alpha x + scale y) / rms(alpha x + scale y) *
    (offset + w)`, the stream itself being what the norm left (`norm_sum`).  `weight_offset=1.0`
    is a weight stored around zero.  As a model's last norm (`forward`) it norms the wanted rows of
    the stream as they are.  Sum, statistics and the weight stay float32; the same launch leaves the
    new rows in the compute dtype for the products that read them next."""

    graph_safe = True

    def __init__(self, hidden_size: int, eps: float, dtype: torch.dtype, device, name: str = "weight",
                 weight_offset: float = 0.0) -> None:
        super().__init__(dtype, device)
        self.hidden_size, self.eps, self.name, self.weight_offset = hidden_size, float(eps), name, float(weight_offset)
        self.factor: torch.Tensor | None = None  # float32 [H]: offset + weight

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        init = "norm_weight" if self.weight_offset == 0.0 else "normal"
        return {prefix + self.name: ParamSpec((self.hidden_size,), init=init, dtype="float32")}

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.factor = (get(prefix + self.name).float() + self.weight_offset).contiguous()

    def norm_sum(self, y, residual, scale=None, alpha=1.0, want_cast=False):
        assert self.factor is not None, "norm used before its weight was loaded"
        y = y.finish() if hasattr(y, "finish") else y
        return ops.scale_add_norm(residual, y, scale, self.factor, alpha, self.eps, self.dtype, want_cast=want_cast)

    def forward(self, delta, residual: torch.Tensor, rows: torch.Tensor | None = None) -> torch.Tensor:
        assert self.factor is not None, "norm used before its weight was loaded"
        if delta is not None:  # a block of another arrangement left its output to be added
            residual.add_(delta.finish() if hasattr(delta, "finish") else delta)
        if rows is None:
            rows = torch.arange(residual.shape[0], dtype=torch.int32, device=residual.device)
        return ops.scale_add_norm(residual, None, None, self.factor, 1.0, self.eps, self.dtype, rows=rows)


@register_norm("post_rms_norm")
def build_post_rms_norm(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> PostRMSNorm:
    return PostRMSNorm(int(desc["hidden_size"]), float(desc["eps"]), dtype, device, name=str(desc.get("name", "weight")),
                       weight_offset=float(desc.get("weight_offset", 0.0)))

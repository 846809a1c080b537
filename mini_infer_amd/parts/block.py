"""Arrangement of a layer's parts around the residual stream.

`PreNormBlock` is the reference's `TransformerBlock` with `defer_add=True`
(models/blocks/transformer_block.py:95-120): norm, mixer, add+norm,
feed-forward; the block's own last add is left to the next norm
(`run_decoder_layers`, :142-153).
"""

from __future__ import annotations

import torch

from mini_infer_amd.parts.base import (
    Block,
    FeedForward,
    LayerCache,
    Mixer,
    Norm,
    ParamSpec,
    StepContext,
    TensorGetter,
)
from mini_infer_amd.registry import FEED_FORWARDS, MIXERS, NORMS, register_block


class PreNormBlock(Block):
    def __init__(
        self,
        mixer_norm: Norm,
        mixer: Mixer,
        ffn_norm: Norm,
        feed_forward: FeedForward,
        names: dict[str, str],
        dtype: torch.dtype,
        device,
    ) -> None:
        super().__init__(dtype, device)
        self.mixer_norm = mixer_norm
        self.mixer = mixer
        self.ffn_norm = ffn_norm
        self.feed_forward = feed_forward
        self.names = names  # part -> its prefix inside the layer, e.g. "self_attn."
        # Where all three say they can, the mixer leaves its last product to the norm that
        # follows, and that norm leaves the rows' factors to the feed-forward's first product:
        # for few rows one launch between two weight-streaming products is saved.
        if mixer.can_defer_output and ffn_norm.takes_pending_products and feed_forward.takes_scaled_rows:
            mixer.emit_pending_output = True
            ffn_norm.emit_scaled_rows = True
            ffn_norm.scaled_rows_consumer = feed_forward
        # The same between the block before this one and this block's mixer: its first norm may
        # be handed a product not made yet (if the model arranges that, `enable_pending_output`
        # of the block before), and leaves the rows' factors to the mixer's first product.
        if mixer_norm.takes_pending_products and mixer.takes_scaled_rows:
            mixer_norm.emit_scaled_rows = True
            mixer_norm.scaled_rows_consumer = mixer

    @property
    def graph_safe(self) -> bool:  # type: ignore[override]
        return all(part.graph_safe for _, part in self._children())

    @property
    def takes_partial_sums(self) -> bool:  # type: ignore[override]
        return self.mixer_norm.takes_partial_sums and self.ffn_norm.takes_partial_sums

    def enable_partial_sums(self) -> None:
        self.mixer.emit_partial_sums = True
        self.feed_forward.emit_partial_sums = True

    @property
    def takes_pending_products(self) -> bool:  # type: ignore[override]
        return self.mixer_norm.takes_pending_products

    def enable_pending_output(self) -> None:
        if self.feed_forward.can_defer_output:
            self.feed_forward.emit_pending_output = True

    def _children(self):
        return (
            (self.names["mixer_norm"], self.mixer_norm),
            (self.names["mixer"], self.mixer),
            (self.names["ffn_norm"], self.ffn_norm),
            (self.names["feed_forward"], self.feed_forward),
        )

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        specs: dict[str, ParamSpec] = {}
        for sub, part in self._children():
            specs.update(part.param_specs(prefix + sub))
        return specs

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        for sub, part in self._children():
            part.load_params(prefix + sub, get)

    def forward(
        self,
        delta: torch.Tensor | None,
        residual: torch.Tensor,
        ctx: StepContext,
        cache: LayerCache,
        writes_cache: bool = True,
    ) -> torch.Tensor:
        h = self.mixer_norm.forward(delta, residual)
        mixed = self.mixer.forward(h, ctx, cache, writes_cache)
        h = self.ffn_norm.forward(mixed, residual)
        return self.feed_forward.forward(h, ctx)


@register_block("pre_norm")
def build_pre_norm_block(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> PreNormBlock:
    """`desc` holds `norm`, `mixer` and `feed_forward` descriptions (each with a `kind`)
    and `names`, the prefix of each part inside the layer."""
    shared = {} if shared is None else shared
    norm_desc, mixer_desc, ffn_desc = desc["norm"], desc["mixer"], desc["feed_forward"]
    return PreNormBlock(
        NORMS.lookup(norm_desc["kind"])(norm_desc, dtype, device, shared),
        MIXERS.lookup(mixer_desc["kind"])(mixer_desc, dtype, device, shared),
        NORMS.lookup(norm_desc["kind"])(norm_desc, dtype, device, shared),
        FEED_FORWARDS.lookup(ffn_desc["kind"])(ffn_desc, dtype, device, shared),
        dict(desc["names"]),
        dtype,
        device,
    )


class ParallelBlock(Block):
    """One norm, and every sublayer reads its output; their results are added to the stream
    together, scaled by one number:

        h = norm(x);    x <- x + scale * (mixer(h) + feed_forward(h))       (a layer may have no feed-forward)

    The add is left to whatever norm comes next, as `ops.StreamUpdate` (with the bias of the
    feed-forward's last product, where it has one, riding along): a norm that knows such an
    update makes it in the launch that also begins the next layer."""

    def __init__(self, norm: Norm, mixer: Mixer, feed_forward: FeedForward | None, scale: float,
                 names: dict[str, str], dtype: torch.dtype, device) -> None:
        super().__init__(dtype, device)
        self.norm, self.mixer, self.feed_forward = norm, mixer, feed_forward
        self.scale, self.names = float(scale), names

    def _children(self):
        parts = [(self.names["norm"], self.norm), (self.names["mixer"], self.mixer)]
        if self.feed_forward is not None:
            parts.append((self.names["feed_forward"], self.feed_forward))
        return parts

    @property
    def graph_safe(self) -> bool:  # type: ignore[override]
        return all(part.graph_safe for _, part in self._children())

    @property
    def takes_pending_products(self) -> bool:  # type: ignore[override]
        return self.norm.takes_pending_products

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        specs: dict[str, ParamSpec] = {}
        for sub, part in self._children():
            specs.update(part.param_specs(prefix + sub))
        return specs

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        for sub, part in self._children():
            part.load_params(prefix + sub, get)

    def forward(self, delta, residual: torch.Tensor, ctx: StepContext, cache: LayerCache, writes_cache: bool = True):
        from mini_infer_amd import ops

        h = self.norm.forward(delta, residual)
        if hasattr(h, "finish"):
            h = h.finish()
        mixed = self.mixer.forward(h, ctx, cache, writes_cache)
        mixed = mixed.finish() if hasattr(mixed, "finish") else mixed
        fed = bias = None
        if self.feed_forward is not None:
            fed = self.feed_forward.forward(h, ctx)
            fed = fed.finish() if hasattr(fed, "finish") else fed
            bias = getattr(self.feed_forward, "output_bias", None)
        return ops.StreamUpdate(mixed, fed, bias, None, self.scale)


@register_block("parallel")
def build_parallel_block(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> ParallelBlock:
    """`desc`: `norm`, `mixer`, optional `feed_forward` (descriptions with a `kind`), `scale` (the
    number the sublayers' sum is multiplied with before it is added) and `names`."""
    shared = {} if shared is None else shared
    ffn = desc.get("feed_forward")
    return ParallelBlock(
        NORMS.lookup(desc["norm"]["kind"])(desc["norm"], dtype, device, shared),
        MIXERS.lookup(desc["mixer"]["kind"])(desc["mixer"], dtype, device, shared),
        FEED_FORWARDS.lookup(ffn["kind"])(ffn, dtype, device, shared) if ffn is not None else None,
        float(desc.get("scale", 1.0)), dict(desc["names"]), dtype, device,
    )


class OutputNormBlock(Block):
    """Sublayers that read the stream itself and are normed on the way OUT:

        x <- x + scale1 * norm1(mixer(x))
        x <- x + scale2 * norm2(feed_forward(x))        (a layer may have none)
        x <- x + side_norm(side(x, tokens))             (a layer may have none)

    `scale1`, `scale2` are per-column layer scales (float32).  Every add is done here, by the
    norm's kernel, so the block hands nothing pending to what follows.  In the bfloat16 engine
    the same kernel leaves the stream's copy in bfloat16 for the next sublayer's products."""

    takes_pending_products = False

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm | None, feed_forward: FeedForward | None,
                 side: FeedForward | None, side_norm: Norm | None, hidden_size: int, layer_scale: bool,
                 names: dict[str, str], dtype: torch.dtype, device) -> None:
        super().__init__(dtype, device)
        self.mixer_norm, self.mixer = mixer_norm, mixer
        self.ffn_norm, self.feed_forward = ffn_norm, feed_forward
        self.side, self.side_norm = side, side_norm
        self.hidden_size, self.layer_scale, self.names = hidden_size, layer_scale, names
        self.mixer_scale: torch.Tensor | None = None
        self.ffn_scale: torch.Tensor | None = None

    def _children(self):
        parts = [(self.names["mixer_norm"], self.mixer_norm), (self.names["mixer"], self.mixer)]
        if self.feed_forward is not None:
            parts += [(self.names["ffn_norm"], self.ffn_norm), (self.names["feed_forward"], self.feed_forward)]
        if self.side is not None:
            parts += [(self.names["side"], self.side), (self.names["side_norm"], self.side_norm)]
        return parts

    @property
    def graph_safe(self) -> bool:  # type: ignore[override]
        return all(part.graph_safe for _, part in self._children())

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        specs: dict[str, ParamSpec] = {}
        for sub, part in self._children():
            specs.update(part.param_specs(prefix + sub))
        if self.layer_scale:
            specs[prefix + self.names["mixer_scale"]] = ParamSpec((self.hidden_size,), init="norm_weight", dtype="float32")
            if self.feed_forward is not None:
                specs[prefix + self.names["ffn_scale"]] = ParamSpec((self.hidden_size,), init="norm_weight", dtype="float32")
        return specs

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        for sub, part in self._children():
            part.load_params(prefix + sub, get)
        if self.layer_scale:
            self.mixer_scale = get(prefix + self.names["mixer_scale"]).float().contiguous()
            if self.feed_forward is not None:
                self.ffn_scale = get(prefix + self.names["ffn_scale"]).float().contiguous()

    def forward(self, delta, residual: torch.Tensor, ctx: StepContext, cache: LayerCache, writes_cache: bool = True):
        from mini_infer_amd.parts.embedding import STREAM_CAST, stream_for_products

        if delta is not None:  # a block of another arrangement left its output to be added
            residual.add_(delta.finish() if hasattr(delta, "finish") else delta)
        narrow = self.dtype != torch.float32

        def added(cast):
            if cast is not None:
                ctx.shared[STREAM_CAST] = (residual, cast)

        mixed = self.mixer.forward(stream_for_products(residual, ctx, self.dtype), ctx, cache, writes_cache)
        added(self.mixer_norm.add_output(mixed, residual, self.mixer_scale, narrow))
        if self.feed_forward is not None:
            fed = self.feed_forward.forward(stream_for_products(residual, ctx, self.dtype), ctx)
            added(self.ffn_norm.add_output(fed, residual, self.ffn_scale, narrow))
        if self.side is not None:
            extra = self.side.forward(stream_for_products(residual, ctx, self.dtype), ctx)
            added(self.side_norm.add_output(extra, residual, None, narrow))
        return None


@register_block("output_norm")
def build_output_norm_block(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> OutputNormBlock:
    """`desc`: `norm` (for both sublayers), `mixer`, optional `feed_forward`, optional `side` with
    `side_norm`, `hidden_size`, `layer_scale` (whether the layer has per-column scales) and
    `names` (each part's name inside the layer)."""
    shared = {} if shared is None else shared

    def build(registry, part):
        return registry.lookup(part["kind"])(part, dtype, device, shared) if part is not None else None

    ffn, side = desc.get("feed_forward"), desc.get("side")
    return OutputNormBlock(
        build(NORMS, desc["norm"]), build(MIXERS, desc["mixer"]),
        build(NORMS, desc["norm"]) if ffn is not None else None, build(FEED_FORWARDS, ffn),
        build(FEED_FORWARDS, side), build(NORMS, desc.get("side_norm")) if side is not None else None,
        int(desc["hidden_size"]), bool(desc.get("layer_scale", False)), dict(desc["names"]), dtype, device,
    )


class HyperConnectionBlock(Block):
    """Pre-norm sublayers around a residual stream that is kept in S copies x_1 .. x_S
    (float32 [T, S, H]).  Sublayer q (the mixer, then the feed-forward if the layer has one) has
    a read vector, a write vector and a matrix of its own:

        u = sum_s in_q[s] x_s;    y = sublayer(norm_q(u));    x_t <- sum_s mix_q[s, t] x_s + out_q[t] y

    (every copy rewritten at once from the old ones).  Without learned vectors (`learned=False`)
    there is one copy, read as it is and written by a plain add: the usual pre-norm layer.

    The norms are `streams_rms_norm`s: each makes the write the sublayer before it left, its own
    read and its statistics in one launch, so the block's last write is handed on as
    `ops.StreamsWrite` to whatever norm comes next."""

    takes_pending_products = False

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm | None, feed_forward: FeedForward | None, copies: int,
                 learned: bool, names: dict[str, str], dtype: torch.dtype, device) -> None:
        super().__init__(dtype, device)
        self.mixer_norm, self.mixer, self.ffn_norm, self.feed_forward = mixer_norm, mixer, ffn_norm, feed_forward
        self.copies, self.learned, self.names = int(copies), bool(learned), names
        if not learned and copies != 1:
            raise ValueError("a stream in several copies needs its read and write vectors")
        self.vectors: dict[str, torch.Tensor] = {}

    def _children(self):
        parts = [(self.names["mixer_norm"], self.mixer_norm), (self.names["mixer"], self.mixer)]
        if self.feed_forward is not None:
            parts += [(self.names["ffn_norm"], self.ffn_norm), (self.names["feed_forward"], self.feed_forward)]
        return parts

    def _connections(self) -> list[str]:
        return [self.names["mixer_connection"]] + ([self.names["ffn_connection"]] if self.feed_forward is not None else [])

    @property
    def graph_safe(self) -> bool:  # type: ignore[override]
        return all(part.graph_safe for _, part in self._children())

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        specs: dict[str, ParamSpec] = {}
        for sub, part in self._children():
            specs.update(part.param_specs(prefix + sub))
        if self.learned:
            S = self.copies
            for sub in self._connections():
                specs[prefix + sub + "in"] = ParamSpec((S,), init="norm_weight", dtype="float32")
                specs[prefix + sub + "out"] = ParamSpec((S,), init="norm_weight", dtype="float32")
                specs[prefix + sub + "mix"] = ParamSpec((S, S), init="identity", dtype="float32")
        return specs

    def optional_names(self, prefix: str) -> set[str]:
        """A layer without a feed-forward has no use for the second sublayer's norm and vectors;
        a checkpoint that stores them all the same is read without them."""
        if self.feed_forward is not None:
            return set()
        sub = self.names["ffn_connection"]
        return {prefix + self.names["ffn_norm"]} | {prefix + sub + what for what in ("in", "out", "mix")}

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        for sub, part in self._children():
            part.load_params(prefix + sub, get)
        for sub in self._connections():
            for what in ("in", "out", "mix"):
                if self.learned:
                    self.vectors[sub + what] = get(prefix + sub + what).float().contiguous()
                else:
                    shape = (1, 1) if what == "mix" else (1,)
                    self.vectors[sub + what] = torch.ones(shape, dtype=torch.float32, device=self.device)
        self.mixer_norm.read = self.vectors[self.names["mixer_connection"] + "in"] if self.learned else None
        if self.ffn_norm is not None:
            self.ffn_norm.read = self.vectors[self.names["ffn_connection"] + "in"] if self.learned else None

    def _write(self, y, connection: str):
        from mini_infer_amd import ops

        mix, out = self.vectors[connection + "mix"], self.vectors[connection + "out"]
        if isinstance(y, ops.WeightedSum):
            return ops.StreamsWrite(y.a, mix, out, b=y.b, scale_a=y.scale_a, scale_b=y.scale_b)
        return ops.StreamsWrite(y.finish() if hasattr(y, "finish") else y, mix, out)

    def forward(self, delta, residual: torch.Tensor, ctx: StepContext, cache: LayerCache, writes_cache: bool = True):
        h = self.mixer_norm.forward(delta, residual)
        pending = self._write(self.mixer.forward(h, ctx, cache, writes_cache), self.names["mixer_connection"])
        if self.feed_forward is None:
            return pending
        h = self.ffn_norm.forward(pending, residual)
        return self._write(self.feed_forward.forward(h, ctx), self.names["ffn_connection"])


@register_block("hyper_connections")
def build_hyper_connection_block(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> HyperConnectionBlock:
    """`desc`: `norm` (for both sublayers), `mixer`, optional `feed_forward`, `copies`, `learned`
    (whether the layer has read and write vectors of its own) and `names`."""
    shared = {} if shared is None else shared
    ffn = desc.get("feed_forward")
    return HyperConnectionBlock(
        NORMS.lookup(desc["norm"]["kind"])(desc["norm"], dtype, device, shared),
        MIXERS.lookup(desc["mixer"]["kind"])(desc["mixer"], dtype, device, shared),
        NORMS.lookup(desc["norm"]["kind"])(desc["norm"], dtype, device, shared) if ffn is not None else None,
        FEED_FORWARDS.lookup(ffn["kind"])(ffn, dtype, device, shared) if ffn is not None else None,
        int(desc.get("copies", 1)), bool(desc.get("learned", True)), dict(desc["names"]), dtype, device,
    )


class PostNormBlock(Block):
    """Sublayers that read the stream itself, which is normed BEHIND every sum:

        x <- norm1(alpha * x + scale1 * mixer(x))
        x <- norm2(alpha * x + scale2 * feed_forward(x))        (a layer may have none)

    `scale1`, `scale2` are per-column layer scales (float32; a layer may have none), `alpha` one
    number of the model.  Every sum is made here, by the norm's kernel (`Norm.norm_sum`), which also
    leaves the stream's copy in the compute dtype for the next sublayer's products, so the block
    hands nothing pending to what follows."""

    takes_pending_products = False

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm | None, feed_forward: FeedForward | None,
                 hidden_size: int, alpha: float, layer_scale: bool, names: dict[str, str], dtype: torch.dtype, device) -> None:
        super().__init__(dtype, device)
        self.mixer_norm, self.mixer, self.ffn_norm, self.feed_forward = mixer_norm, mixer, ffn_norm, feed_forward
        self.hidden_size, self.alpha, self.layer_scale, self.names = hidden_size, float(alpha), bool(layer_scale), names
        self.mixer_scale: torch.Tensor | None = None
        self.ffn_scale: torch.Tensor | None = None

    def _children(self):
        parts = [(self.names["mixer_norm"], self.mixer_norm), (self.names["mixer"], self.mixer)]
        if self.feed_forward is not None:
            parts += [(self.names["ffn_norm"], self.ffn_norm), (self.names["feed_forward"], self.feed_forward)]
        return parts

    @property
    def graph_safe(self) -> bool:  # type: ignore[override]
        return all(part.graph_safe for _, part in self._children())

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        specs: dict[str, ParamSpec] = {}
        for sub, part in self._children():
            specs.update(part.param_specs(prefix + sub))
        if self.layer_scale:
            specs[prefix + self.names["mixer_scale"]] = ParamSpec((self.hidden_size,), init="norm_weight", dtype="float32")
            if self.feed_forward is not None:
                specs[prefix + self.names["ffn_scale"]] = ParamSpec((self.hidden_size,), init="norm_weight", dtype="float32")
        return specs

    def optional_names(self, prefix: str) -> set[str]:
        """A layer without a feed-forward has no use for the second norm and scale; a checkpoint
        that stores them all the same is read without them."""
        names = set(self.mixer.optional_names(prefix + self.names["mixer"])) if hasattr(self.mixer, "optional_names") else set()
        if self.feed_forward is None:
            names |= {prefix + self.names["ffn_norm"], prefix + self.names["ffn_scale"]}
        return names

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        for sub, part in self._children():
            part.load_params(prefix + sub, get)
        if self.layer_scale:
            self.mixer_scale = get(prefix + self.names["mixer_scale"]).float().contiguous()
            if self.feed_forward is not None:
                self.ffn_scale = get(prefix + self.names["ffn_scale"]).float().contiguous()

    def forward(self, delta, residual: torch.Tensor, ctx: StepContext, cache: LayerCache, writes_cache: bool = True):
        from mini_infer_amd.parts.embedding import STREAM_CAST, stream_for_products

        if delta is not None:  # a block of another arrangement left its output to be added
            residual.add_(delta.finish() if hasattr(delta, "finish") else delta)
        narrow = self.dtype != torch.float32

        def normed(cast):
            if cast is not None:
                ctx.shared[STREAM_CAST] = (residual, cast)

        mixed = self.mixer.forward(stream_for_products(residual, ctx, self.dtype), ctx, cache, writes_cache)
        normed(self.mixer_norm.norm_sum(mixed, residual, self.mixer_scale, self.alpha, narrow))
        if self.feed_forward is not None:
            fed = self.feed_forward.forward(stream_for_products(residual, ctx, self.dtype), ctx)
            normed(self.ffn_norm.norm_sum(fed, residual, self.ffn_scale, self.alpha, narrow))
        return None


@register_block("post_norm")
def build_post_norm_block(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> PostNormBlock:
    """`desc`: `norm` (for both sublayers), `mixer`, optional `feed_forward`, `hidden_size`, `alpha`,
    `layer_scale` (whether the layer has per-column scales) and `names` (each part's name inside the layer)."""
    shared = {} if shared is None else shared
    ffn = desc.get("feed_forward")
    return PostNormBlock(
        NORMS.lookup(desc["norm"]["kind"])(desc["norm"], dtype, device, shared),
        MIXERS.lookup(desc["mixer"]["kind"])(desc["mixer"], dtype, device, shared),
        NORMS.lookup(desc["norm"]["kind"])(desc["norm"], dtype, device, shared) if ffn is not None else None,
        FEED_FORWARDS.lookup(ffn["kind"])(ffn, dtype, device, shared) if ffn is not None else None,
        int(desc["hidden_size"]), float(desc.get("alpha", 1.0)), bool(desc.get("layer_scale", False)), dict(desc["names"]),
        dtype, device,
    )

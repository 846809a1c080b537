"""Grouped-query attention over the paged cache.

Order of operations as in the reference's `GroupedQueryAttention.forward`
(models/blocks/gqa.py:107-154): one merged q|k|v projection, rotary encoding of
q and k fused with the write of k and v into cache pages
(rope_write_kernel.py:75-152), causal attention over the pages with scale
1/sqrt(head_dim) (cache/packed_attention.py:126-127, :296-338), output
projection.  A window, if given, limits each query to the last `window` keys; a chunk to
the keys of its own stretch of `chunk` positions.  Queries and keys may be normed head by
head before the rotation, and the attended rows may be gated by a projection of the
layer's input before the output projection.
"""

from __future__ import annotations

import math

import torch

from mini_infer_amd import ops
from mini_infer_amd.parts.base import (
    CacheNeeds,
    LayerCache,
    Mixer,
    PagedKVNeeds,
    ParamSpec,
    PositionEncoding,
    StepContext,
    TensorGetter,
)
from mini_infer_amd.parts.linear import Linear
from mini_infer_amd.registry import POSITION_ENCODINGS, register_mixer


class GQAttention(Mixer):
    graph_safe = True
    can_defer_output = True
    takes_scaled_rows = True

    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        position: PositionEncoding | None,
        dtype: torch.dtype,
        device,
        *,
        window: int | None = None,
        scale: float | None = None,
        names: tuple[str, str, str, str] = ("q_proj", "k_proj", "v_proj", "o_proj"),
        suffix: str = ".weight",
        v_head_dim: int | None = None,
        sink_logit: float | None = None,
        chunk: int | None = None,
        head_norm: dict | None = None,
        gate: dict | None = None,
    ) -> None:
        """`v_head_dim`: value heads of another width than the query and key heads (`head_dim`).
        `sink_logit`: the softmax's denominator gets one more term exp(sink_logit), a sink that
        takes weight off the keys and carries no value (0.0: the denominator grows by exp(0) = 1).
        `chunk`: position i sees j <= i only if i // chunk == j // chunk (chunks are counted from
        position 0 of the sequence, wherever a prompt was cut).
        `head_norm` = {"eps": e, "names": (q_name, k_name)}: every query head and every key head is
        divided by its own root mean square over the head and multiplied by a weight of `head_dim`
        entries that the heads share, before the rotation.
        `gate` = {"name": n, "activation": "logistic"}: one more projection of the layer's input, as wide as
        the concatenated value heads; the attended rows are multiplied by its activation, element
        by element, before the output projection."""
        super().__init__(dtype, device)
        if num_heads % num_kv_heads != 0:
            raise ValueError(f"num_heads={num_heads} is not a multiple of num_kv_heads={num_kv_heads}")
        if window is not None and window <= 0:
            raise ValueError(f"window must be positive, got {window}")
        if chunk is not None and chunk <= 0:
            raise ValueError(f"chunk must be positive, got {chunk}")
        self.chunk = None if chunk is None else int(chunk)
        self.head_norm_eps = None if head_norm is None else float(head_norm["eps"])
        self.head_norm_names = None if head_norm is None else tuple(head_norm.get("names", ("q_norm", "k_norm")))
        self.gate_name = None if gate is None else str(gate["name"])
        self.gate_activation = None if gate is None else str(gate.get("activation", "logistic"))
        # the few-row kernels that fold projection, rotation and cache write (and the output
        # projection's hand-over) know neither head norms nor gates
        self._plain_heads = head_norm is None and gate is None
        self.q_norm_weight: torch.Tensor | None = None
        self.k_norm_weight: torch.Tensor | None = None
        if head_dim <= 0 or head_dim % ops.ATTENTION_HEAD_DIM_STEP != 0 or head_dim > ops.ATTENTION_MAX_HEAD_DIM:
            raise ValueError(
                f"head_dim={head_dim}: the attention kernels take even head sizes "
                f"up to {ops.ATTENTION_MAX_HEAD_DIM}"
            )
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.v_head_dim = head_dim if v_head_dim is None else int(v_head_dim)
        if self.v_head_dim <= 0 or self.v_head_dim % ops.ATTENTION_HEAD_DIM_STEP != 0:
            raise ValueError(f"v_head_dim={self.v_head_dim}: the attention kernels take even value head sizes")
        self.sink_logit = None if sink_logit is None else float(sink_logit)
        # what the matrix-core kernel and the fused few-row kernels take: values as wide as keys
        self._same_widths = self.v_head_dim == head_dim
        self.position = position
        self.window = window
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        # per-head slopes of a score bias linear in the distance, if the encoding has one
        self.slopes = position.score_slopes(num_heads) if position is not None else None
        if self.slopes is not None and (
            self.slopes.dtype != torch.float32 or tuple(self.slopes.shape) != (num_heads,)
        ):
            raise ValueError(f"score slopes must be float32 [{num_heads}], got {self.slopes.dtype} {tuple(self.slopes.shape)}")
        q_width, kv_width = num_heads * head_dim, num_kv_heads * head_dim
        self.qkv = self._input_projection(hidden_size, q_width, kv_width, names, suffix)
        self.out = Linear(num_heads * self.v_head_dim, hidden_size, names[3], dtype, device, suffix=suffix)

    def _input_projection(self, hidden_size: int, q_width: int, kv_width: int, names, suffix: str) -> Linear:
        """The stacked product that feeds the attention: q | k | v here."""
        v_width = self.num_kv_heads * self.v_head_dim
        widths, parts = [q_width, kv_width, v_width], list(names[:3])
        if self.gate_name is not None:  # q | k | v | gate
            widths.append(self.num_heads * self.v_head_dim)
            parts.append(self.gate_name)
        return Linear(hidden_size, widths, parts, self.dtype, self.device, suffix=suffix)

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        specs = {**self.qkv.param_specs(prefix), **self.out.param_specs(prefix)}
        if self.head_norm_names is not None:
            for name in self.head_norm_names:
                specs[prefix + name] = ParamSpec((self.head_dim,), init="norm_weight", dtype="float32")
        return specs

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.qkv.load_params(prefix, get)
        self.out.load_params(prefix, get)
        if self.head_norm_names is not None:
            self.q_norm_weight = get(prefix + self.head_norm_names[0]).float().contiguous()
            self.k_norm_weight = get(prefix + self.head_norm_names[1]).float().contiguous()

    def wants_scaled_rows(self, rows: int) -> bool:
        """Only where projection, rotation and cache write will run as the one kernel that
        applies the rows' factors: few bfloat16 rows, whole heads rotated in half pairing."""
        layout = self.position.rotary_layout() if self.position is not None else None
        return (
            self.dtype == torch.bfloat16
            and self._same_widths
            and self._plain_heads
            and layout == (self.head_dim, False)
            and self.head_dim % 32 == 0
            and ops.scaled_rows_product_takes(rows, self.qkv.weight, self.hidden_size)
        )

    def cache_needs(self, page_size: int) -> CacheNeeds:
        # values lie transposed inside a page where the matrix-core kernel will read them
        # (that kernel knows no score bias: such layers keep the plain layout and kernel)
        transposed = (
            self.slopes is None and self._same_widths
            and ops.mfma_attention_supported(self.dtype, self.head_dim, page_size)
        )
        v_head_dim = None if self.v_head_dim == self.head_dim else self.v_head_dim
        return CacheNeeds(
            pages=PagedKVNeeds(self.num_kv_heads, self.head_dim, self.window, v_head_dim=v_head_dim, v_transposed=transposed)
        )

    def forward(
        self, x: torch.Tensor, ctx: StepContext, cache: LayerCache, writes_cache: bool = True
    ) -> torch.Tensor:
        assert cache.group is not None and cache.k_pages is not None and cache.v_pages is not None
        q_width = self.num_heads * self.head_dim
        assert self.qkv.weight is not None
        rotary = self.position.rotary(ctx) if self.position is not None else None
        if isinstance(x, ops.ScaledRows) and not (
            rotary is not None
            and self._same_widths
            and self._plain_heads
            and ops.qkv_rope_write_takes(x, self.qkv.weight, self.head_dim, rotary.rotary_dim, rotary.interleaved)
        ):
            x = x.finish()  # rows but for their norm factors, and no kernel here that applies them
        if rotary is not None and self._same_widths and self._plain_heads and ops.qkv_rope_write_takes(
            x, self.qkv.weight, self.head_dim, rotary.rotary_dim, rotary.interleaved
        ):
            # few rows (decode): projection, rotation and cache write are one kernel
            kv_heads = self.num_kv_heads if writes_cache else 0
            queries = ops.qkv_rope_write(
                x, self.qkv.weight if writes_cache else self.qkv.weight[:q_width], rotary.cos, rotary.sin,
                ctx.slot_mapping[cache.group] if writes_cache else None, cache.k_pages, cache.v_pages,
                q_heads=self.num_heads, kv_heads=kv_heads, head_dim=self.head_dim,
                v_transposed=cache.v_transposed,
            )
            return self._project(self._attend(queries, ctx, cache))
        if writes_cache:
            qkv = self.qkv.forward(x)
            kv_heads, slots = self.num_kv_heads, ctx.slot_mapping[cache.group]
        else:
            # reads another call's keys and values: only q is projected
            qkv = ops.linear(x, self.qkv.weight[:q_width])
            kv_heads, slots = 0, None
        if rotary is not None:
            cos, sin, rotary_dim, interleaved = rotary.cos, rotary.sin, rotary.rotary_dim, rotary.interleaved
        else:
            cos = sin = torch.empty((ctx.num_tokens, 0), dtype=torch.float32, device=x.device)
            rotary_dim, interleaved = 0, False
        if self.head_norm_eps is not None:
            assert self.q_norm_weight is not None, "attention used before its weights were loaded"
            ops.head_norm_rope_kv_write(
                qkv, cos, sin, slots, cache.k_pages, cache.v_pages, self.q_norm_weight,
                self.k_norm_weight if writes_cache else None, self.head_norm_eps,
                q_heads=self.num_heads, kv_heads=kv_heads, head_dim=self.head_dim,
                rotary_dim=rotary_dim, interleaved=interleaved, v_transposed=cache.v_transposed,
                v_head_dim=self.v_head_dim,
            )
        else:
            ops.rope_kv_write(
                qkv, cos, sin, slots, cache.k_pages, cache.v_pages,
                q_heads=self.num_heads, kv_heads=kv_heads, head_dim=self.head_dim,
                rotary_dim=rotary_dim, interleaved=interleaved, v_transposed=cache.v_transposed,
                v_head_dim=self.v_head_dim,
            )
        attended = self._attend(qkv, ctx, cache)
        if self.gate_name is not None:
            if not writes_cache:
                raise NotImplementedError("a gated attention layer that reads another call's keys projects its own gate; not built")
            width = self.num_heads * self.v_head_dim
            first = (self.num_heads + self.num_kv_heads) * self.head_dim + self.num_kv_heads * self.v_head_dim
            attended = ops.gated_mul(qkv[:, first:first + width], attended, self.gate_activation)
        return self._project(attended)

    def _project(self, attended):
        """The output projection of what `_attend` returned; for few rows, where the block
        asked for it, not made here but handed on to the norm that follows."""
        assert self.out.weight is not None
        if self.emit_pending_output and self.dtype == torch.bfloat16:
            rows = attended.tokens if isinstance(attended, ops.AttentionPieces) else attended.shape[0]
            q_width = self.num_heads * self.v_head_dim
            if ops.pending_product_pays(rows, self.hidden_size, q_width, self.emit_partial_sums):
                return ops.PendingProduct(attended, self.out.weight)
        if isinstance(attended, ops.AttentionPieces):
            return ops.linear_from_attention(attended, self.out.weight)
        return self.out.forward(attended, partial_ok=self.emit_partial_sums)

    def _attend(self, queries: torch.Tensor, ctx: StepContext, cache: LayerCache):
        """Attention of the rotated queries (the first columns of `queries`) over the cache pages.
        At the smallest batches the key ranges may come back uncombined, for the output
        projection to combine on its way (one launch less a layer)."""
        few = (
            queries.dtype == torch.bfloat16 and self._same_widths and self.sink_logit is None
            and self._plain_heads and self.chunk is None
            and ops.attention_pieces_pay(ctx.num_tokens, self.num_heads, self.head_dim)
        )
        return ops.paged_attention(
            queries, cache.k_pages, cache.v_pages, ctx.block_tables[cache.group], ctx.token_request,
            ctx.positions, ctx.cu_seqlens_q, ctx.host_cu_seqlens_q, q_heads=self.num_heads,
            kv_heads=self.num_kv_heads, head_dim=self.head_dim, scale=self.scale, window=self.window,
            max_seq_len=ctx.max_seq_len, v_transposed=cache.v_transposed, combine=not few, slopes=self.slopes,
            v_head_dim=self.v_head_dim, sink_logit=self.sink_logit, chunk=self.chunk,
        )


class KeysAsValuesAttention(GQAttention):
    """Grouped-query attention without a value projection: the values are the keys as
    projected, before the keys' norm.  Queries and keys are RMS-normed over their WHOLE
    projection (all heads at once, one weight per column) before they are split into heads.
    Positions enter the scores only if a position encoding is given (none: the window and the
    causal order are all the layer knows of positions).

    The pages hold two streams as everywhere else: normed keys in the key pages, the un-normed
    key projection in the value pages, so the paged attention kernels run unchanged."""

    can_defer_output = False
    takes_scaled_rows = False

    def __init__(self, hidden_size, num_heads, num_kv_heads, head_dim, dtype, device, *, norm_eps: float,
                 window=None, scale=None, names=("q", "k", "", "o"), suffix="",
                 norm_names=("q.norm", "k.norm")) -> None:
        super().__init__(hidden_size, num_heads, num_kv_heads, head_dim, None, dtype, device, window=window,
                         scale=scale, names=names, suffix=suffix)
        self.norm_eps = float(norm_eps)
        self.norm_names = tuple(norm_names)
        self.q_norm: torch.Tensor | None = None
        self.k_norm: torch.Tensor | None = None

    def _input_projection(self, hidden_size, q_width, kv_width, names, suffix):
        return Linear(hidden_size, [q_width, kv_width], [names[0], names[1]], self.dtype, self.device, suffix=suffix)

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        q_width, kv_width = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim
        return {
            **super().param_specs(prefix),
            prefix + self.norm_names[0]: ParamSpec((q_width,), init="norm_weight", dtype="float32"),
            prefix + self.norm_names[1]: ParamSpec((kv_width,), init="norm_weight", dtype="float32"),
        }

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        super().load_params(prefix, get)
        self.q_norm = get(prefix + self.norm_names[0]).float().contiguous()
        self.k_norm = get(prefix + self.norm_names[1]).float().contiguous()

    def wants_scaled_rows(self, rows: int) -> bool:
        return False

    def forward(self, x, ctx: StepContext, cache: LayerCache, writes_cache: bool = True):
        assert cache.group is not None and cache.k_pages is not None and cache.v_pages is not None
        assert self.qkv.weight is not None and self.q_norm is not None, "attention used before its weights were loaded"
        if isinstance(x, ops.ScaledRows):
            x = x.finish()
        q_width = self.num_heads * self.head_dim
        if writes_cache:
            qk = self.qkv.forward(x)
            kv_heads, slots = self.num_kv_heads, ctx.slot_mapping[cache.group]
        else:
            qk = ops.linear(x, self.qkv.weight[:q_width])
            kv_heads, slots = 0, None
        ops.qk_norm_kv_write(
            qk, self.q_norm, self.k_norm if writes_cache else None, slots, cache.k_pages, cache.v_pages,
            q_width=q_width, kv_heads=kv_heads, head_dim=self.head_dim, eps=self.norm_eps,
            v_transposed=cache.v_transposed,
        )
        return self._project(self._attend(qk, ctx, cache))


class WholeNormAttention(GQAttention):
    """Grouped-query attention whose queries and keys are RMS-normed over their WHOLE projection
    (all heads at once, one plain weight per column) before they are split into heads, with
    values of their own and, each optional:

    * `softcap`: a scaled score s becomes `softcap * tanh(s / softcap)` before anything else is done to it;
    * `position`: any encoding; one that gives `score_slopes` takes `slope_h * distance` off the capped score;
    * `learned_sink`: the softmax's denominator holds `exp(sink_h)` too, `sink_h` a learned number
      per query head (tensor `sink_name`); it has no key and no value and is neither scaled nor capped;
    * `value_mix` = {"key": k, "source": bool, "name": n}: layers that name the same key share values.
      The source layer leaves its values of the step's tokens where the others find them; every
      other layer caches `(1 - m) v + m v_source` of the same token, `m` its own learned number
      (tensor `n`; the source's own is not read).

    What is cached is the normed key and the (mixed) value, so decoding reads them as they are."""

    can_defer_output = False
    takes_scaled_rows = False

    def __init__(self, hidden_size, num_heads, num_kv_heads, head_dim, position, dtype, device, *, norm_eps: float,
                 v_head_dim=None, window=None, scale=None, names=("q", "k", "v", "o"), suffix="",
                 norm_names=("q.norm", "k.norm"), softcap: float | None = None, learned_sink: bool = False,
                 sink_name: str = "sink", value_mix: dict | None = None) -> None:
        super().__init__(hidden_size, num_heads, num_kv_heads, head_dim, position, dtype, device, window=window,
                         scale=scale, names=names, suffix=suffix, v_head_dim=v_head_dim)
        if softcap is not None and not softcap > 0:
            raise ValueError(f"a cap on the scores must be positive, got {softcap}")
        if position is not None and position.rotary_layout() is not None:
            raise NotImplementedError("attention normed over the whole projection with a rotation on top; not built")
        self.norm_eps, self.norm_names = float(norm_eps), tuple(norm_names)
        self.softcap = None if softcap is None else float(softcap)
        self.learned_sink, self.sink_name = bool(learned_sink), sink_name
        self.mix_key = None if value_mix is None else ("value_mix", str(value_mix["key"]))
        self.mix_source = bool(value_mix["source"]) if value_mix is not None else False
        self.mix_name = None if value_mix is None else str(value_mix.get("name", "vmix"))
        self.q_norm: torch.Tensor | None = None
        self.k_norm: torch.Tensor | None = None
        self.sinks: torch.Tensor | None = None
        self.mix: torch.Tensor | None = None

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        q_width, kv_width = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim
        specs = {
            **super().param_specs(prefix),
            prefix + self.norm_names[0]: ParamSpec((q_width,), init="norm_weight", dtype="float32"),
            prefix + self.norm_names[1]: ParamSpec((kv_width,), init="norm_weight", dtype="float32"),
        }
        if self.learned_sink:
            specs[prefix + self.sink_name] = ParamSpec((self.num_heads,), dtype="float32")
        if self.mix_key is not None and not self.mix_source:
            specs[prefix + self.mix_name] = ParamSpec((), dtype="float32")
        return specs

    def optional_names(self, prefix: str) -> set[str]:
        return {prefix + self.mix_name} if self.mix_key is not None and self.mix_source else set()

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        super().load_params(prefix, get)
        self.q_norm = get(prefix + self.norm_names[0]).float().contiguous()
        self.k_norm = get(prefix + self.norm_names[1]).float().contiguous()
        if self.learned_sink:
            self.sinks = get(prefix + self.sink_name).float().contiguous()
        if self.mix_key is not None and not self.mix_source:
            self.mix = get(prefix + self.mix_name).float().reshape(1).contiguous()

    def wants_scaled_rows(self, rows: int) -> bool:
        return False

    def cache_needs(self, page_size: int) -> CacheNeeds:
        # values lie transposed inside a page where the matrix-core kernel will read them (it knows
        # the cap, the distance bias and the sinks; values of another width than the keys run the plain kernel)
        transposed = self._same_widths and ops.mfma_attention_supported(self.dtype, self.head_dim, page_size)
        v_head_dim = None if self.v_head_dim == self.head_dim else self.v_head_dim
        return CacheNeeds(pages=PagedKVNeeds(self.num_kv_heads, self.head_dim, self.window, v_head_dim=v_head_dim,
                                             v_transposed=transposed))

    def forward(self, x, ctx: StepContext, cache: LayerCache, writes_cache: bool = True):
        assert cache.group is not None and cache.k_pages is not None and cache.v_pages is not None
        assert self.qkv.weight is not None and self.q_norm is not None, "attention used before its weights were loaded"
        if isinstance(x, ops.ScaledRows):
            x = x.finish()
        q_width, k_width = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim
        v_width = self.num_kv_heads * self.v_head_dim
        other = None
        if writes_cache:
            qkv = self.qkv.forward(x)
            kv_heads, slots = self.num_kv_heads, ctx.slot_mapping[cache.group]
            if self.mix_key is not None:
                values = qkv[:, q_width + k_width: q_width + k_width + v_width]
                if self.mix_source:
                    ctx.shared[self.mix_key] = values  # (a view: the projection's rows stay as they are)
                else:
                    other = ctx.shared.get(self.mix_key)
                    if other is None:
                        raise RuntimeError("a layer that mixes values in ran before the layer whose values it mixes in")
        else:
            if self.mix_key is not None:
                raise NotImplementedError("a layer that shares values and reads another call's cache; not built")
            qkv = ops.linear(x, self.qkv.weight[:q_width])
            kv_heads, slots = 0, None
        ops.qkv_norm_write(
            qkv, self.q_norm, self.k_norm if writes_cache else None, slots, cache.k_pages, cache.v_pages,
            q_width=q_width, kv_heads=kv_heads, head_dim=self.head_dim, v_head_dim=self.v_head_dim, eps=self.norm_eps,
            v_transposed=cache.v_transposed, other_values=other, mix=self.mix,
        )
        attended = ops.paged_attention(
            qkv, cache.k_pages, cache.v_pages, ctx.block_tables[cache.group], ctx.token_request,
            ctx.positions, ctx.cu_seqlens_q, ctx.host_cu_seqlens_q, q_heads=self.num_heads,
            kv_heads=self.num_kv_heads, head_dim=self.head_dim, scale=self.scale, window=self.window,
            max_seq_len=ctx.max_seq_len, v_transposed=cache.v_transposed, slopes=self.slopes,
            v_head_dim=self.v_head_dim, sinks=self.sinks, softcap=self.softcap,
        )
        return self.out.forward(attended)


@register_mixer("whole_norm_attention")
def build_whole_norm_attention(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> WholeNormAttention:
    position = None
    pos_desc = desc.get("position")
    if pos_desc is not None:
        position = POSITION_ENCODINGS.lookup(pos_desc["kind"])(pos_desc, dtype, device, shared)
    extra = {k: desc[k] for k in ("suffix", "v_head_dim", "softcap", "learned_sink", "sink_name", "value_mix", "norm_names") if k in desc}
    if "names" in desc:
        extra["names"] = tuple(desc["names"])
    return WholeNormAttention(
        int(desc["hidden_size"]), int(desc["num_heads"]), int(desc["num_kv_heads"]), int(desc["head_dim"]), position, dtype,
        device, norm_eps=float(desc["norm_eps"]), window=desc.get("window"), scale=desc.get("scale"), **extra,
    )


@register_mixer("keys_as_values_attention")
def build_keys_as_values_attention(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> KeysAsValuesAttention:
    extra = {k: desc[k] for k in ("names", "suffix", "norm_names") if k in desc}
    if "names" in extra:
        extra["names"] = tuple(extra["names"])
    return KeysAsValuesAttention(
        int(desc["hidden_size"]), int(desc["num_heads"]), int(desc["num_kv_heads"]), int(desc["head_dim"]), dtype, device,
        norm_eps=float(desc["norm_eps"]), window=desc.get("window"), scale=desc.get("scale"), **extra,
    )


@register_mixer("gqa_attention")
def build_gqa_attention(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> GQAttention:
    position = None
    pos_desc = desc.get("position")
    if pos_desc is not None:
        key = ("position", repr(sorted(pos_desc.items(), key=lambda kv: kv[0])))
        if shared is not None and key in shared:
            position = shared[key]
        else:
            position = POSITION_ENCODINGS.lookup(pos_desc["kind"])(pos_desc, dtype, device, shared)
            if shared is not None:
                shared[key] = position
    extra = {k: desc[k] for k in ("suffix", "v_head_dim", "sink_logit", "chunk", "head_norm", "gate") if k in desc}
    if "names" in desc:
        extra["names"] = tuple(desc["names"])
    return GQAttention(
        int(desc["hidden_size"]),
        int(desc["num_heads"]),
        int(desc["num_kv_heads"]),
        int(desc["head_dim"]),
        position,
        dtype,
        device,
        window=desc.get("window"),
        scale=desc.get("scale"),
        **extra,
    )

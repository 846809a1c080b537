"""Token embedding and output head.

Embedding: a row lookup that starts the float32 residual stream
(models/llama/llama.py:159 of the reference).  Head: `logits = h @ W.T` on the
requested rows only (llama.py:169-171); with tied embeddings the head's matrix is
the embedding table and the checkpoint holds no `lm_head.weight` (llama.py:143-147).

Both are chosen by kind like every other part, so a model whose stream starts or
ends differently (a scaled embedding, learned positions added to it, capped logits)
registers a part of its own and names it in its `ModelSpec`.
"""

from __future__ import annotations

import torch

from mini_infer_amd import ops
from mini_infer_amd.parts.base import CacheNeeds, Embedding, Head, LayerCache, ParamSpec, StateNeeds, StepContext, TensorGetter
from mini_infer_amd.registry import register_embedding, register_head


class TokenEmbedding(Embedding):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, name: str, dtype: torch.dtype, device) -> None:
        super().__init__(dtype, device)
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.name = name
        self.weight: torch.Tensor | None = None

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        return {prefix + self.name: ParamSpec((self.vocab_size, self.hidden_size))}

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.weight = get(prefix + self.name).contiguous()

    def forward(self, ctx: StepContext, cache: LayerCache | None = None) -> torch.Tensor:
        assert self.weight is not None, "embedding used before its table was loaded"
        return ops.embed_gather(self.weight, ctx.token_ids)


class ScaledEmbedding(TokenEmbedding):
    """`table[token] * scale`."""

    def __init__(self, vocab_size: int, hidden_size: int, name: str, scale: float, dtype: torch.dtype, device) -> None:
        super().__init__(vocab_size, hidden_size, name, dtype, device)
        self.scale = float(scale)

    def forward(self, ctx: StepContext, cache: LayerCache | None = None) -> torch.Tensor:
        assert self.weight is not None, "embedding used before its table was loaded"
        return ops.embed_gather(self.weight, ctx.token_ids, self.scale)


SINUSOID_BASE = 10000.0
STREAM_CAST = "stream_cast"  # key in `StepContext.shared`: (the stream, its latest copy in the compute dtype)


def stream_for_products(residual: torch.Tensor, ctx: StepContext, dtype: torch.dtype) -> torch.Tensor:
    """The float32 stream as the products of a sublayer that reads it un-normed take it: itself
    in the 32-bit engine, else its copy in the compute dtype (left in `ctx.shared` by whichever
    kernel last wrote the stream, or made here)."""
    if dtype == torch.float32:
        return residual
    kept = ctx.shared.get(STREAM_CAST)
    if kept is not None and kept[0] is residual:
        return kept[1]
    cast = ops.cast_rows(residual)
    ctx.shared[STREAM_CAST] = (residual, cast)
    return cast


class ScaledSinusoidEmbedding(TokenEmbedding):
    """`table[token] * scale` plus a fixed wave of the position: column 2i gets
    sin(p * base^(-2i/H)), column 2i+1 the cosine of the same angle.  Frequencies are made in
    64-bit on the host; the kernel takes the angle in float32 (64-bit in the 32-bit engine)."""

    def __init__(self, vocab_size: int, hidden_size: int, name: str, scale: float, dtype: torch.dtype, device,
                 base: float = SINUSOID_BASE) -> None:
        super().__init__(vocab_size, hidden_size, name, dtype, device)
        self.scale = float(scale)
        pairs = torch.arange((hidden_size + 1) // 2, dtype=torch.float64)
        self.freq_host = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * pairs / hidden_size)
        self._freq: torch.Tensor | None = None

    def forward(self, ctx: StepContext, cache: LayerCache | None = None) -> torch.Tensor:
        assert self.weight is not None, "embedding used before its table was loaded"
        if self._freq is None:
            self._freq = self.freq_host.to(self.device).contiguous()
        residual, cast = ops.embed_sinusoid(
            self.weight, ctx.token_ids, ctx.positions, self._freq, self.scale, want_cast=self.dtype != torch.float32
        )
        if cast is not None:
            ctx.shared[STREAM_CAST] = (residual, cast)
        return residual


class OutputHead(Head):
    graph_safe = True

    def __init__(
        self,
        hidden_size: int,
        vocab_size: int,
        name: str,
        dtype: torch.dtype,
        device,
        *,
        tied_to: TokenEmbedding | None = None,
    ) -> None:
        super().__init__(dtype, device)
        self.hidden_size = hidden_size
        self.vocab_size = vocab_size
        self.name = name
        self.tied_to = tied_to
        self._weight: torch.Tensor | None = None

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        if self.tied_to is not None:
            return {}
        return {prefix + self.name: ParamSpec((self.vocab_size, self.hidden_size))}

    def optional_names(self, prefix: str) -> set[str]:
        """Names a checkpoint may hold without the model needing them."""
        return {prefix + self.name} if self.tied_to is not None else set()

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        if self.tied_to is None:
            self._weight = get(prefix + self.name).contiguous()

    @property
    def weight(self) -> torch.Tensor:
        w = self.tied_to.weight if self.tied_to is not None else self._weight
        assert w is not None, "output head used before its matrix was loaded"
        return w

    def forward(self, h: torch.Tensor, ctx: StepContext | None = None) -> torch.Tensor:
        """Logits [rows, vocab] in float32."""
        return ops.linear_f32_out(h, self.weight)


@register_embedding("token_embedding")
def build_token_embedding(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> TokenEmbedding:
    return TokenEmbedding(int(desc["vocab_size"]), int(desc["hidden_size"]), str(desc["name"]), dtype, device)


@register_embedding("scaled_embedding")
def build_scaled_embedding(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> ScaledEmbedding:
    return ScaledEmbedding(int(desc["vocab_size"]), int(desc["hidden_size"]), str(desc["name"]), float(desc["scale"]), dtype, device)


@register_embedding("scaled_sinusoid_embedding")
def build_scaled_sinusoid_embedding(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> ScaledSinusoidEmbedding:
    return ScaledSinusoidEmbedding(
        int(desc["vocab_size"]), int(desc["hidden_size"]), str(desc["name"]), float(desc["scale"]), dtype, device,
        base=float(desc.get("base", SINUSOID_BASE)),
    )


@register_head("linear_head")
def build_linear_head(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> OutputHead:
    """`desc["tied"]`: the head's matrix is the table of the model's embedding part (which the
    model leaves under `shared["embedding"]` before it builds the head)."""
    tied_to = None
    if desc.get("tied", False):
        tied_to = (shared or {}).get("embedding")
        if tied_to is None or not hasattr(tied_to, "weight"):
            raise ValueError("a tied output head needs the model's embedding part to hold a `weight` table")
    return OutputHead(
        int(desc["hidden_size"]), int(desc["vocab_size"]), str(desc["name"]), dtype, device, tied_to=tied_to
    )


class NormedStreamsEmbedding(TokenEmbedding):
    """`table[token]` divided by its root mean square and multiplied by `offset + w` (`w` of its
    own: `norm_name`), written `copies` times: the start of a residual stream that is kept in
    several copies, float32 [T, copies, H]."""

    def __init__(self, vocab_size: int, hidden_size: int, name: str, norm_name: str, eps: float, copies: int,
                 dtype: torch.dtype, device, weight_offset: float = 0.0) -> None:
        super().__init__(vocab_size, hidden_size, name, dtype, device)
        self.norm_name, self.eps, self.copies, self.weight_offset = norm_name, float(eps), int(copies), float(weight_offset)
        self.factor: torch.Tensor | None = None

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        init = "norm_weight" if self.weight_offset == 0.0 else "normal"
        return {**super().param_specs(prefix), prefix + self.norm_name: ParamSpec((self.hidden_size,), init=init, dtype="float32")}

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        super().load_params(prefix, get)
        self.factor = (get(prefix + self.norm_name).float() + self.weight_offset).contiguous()

    def forward(self, ctx: StepContext, cache: LayerCache | None = None) -> torch.Tensor:
        assert self.weight is not None and self.factor is not None, "embedding used before its tensors were loaded"
        return ops.embed_norm_streams(self.weight, ctx.token_ids, self.factor, self.copies, self.eps)


@register_embedding("normed_streams_embedding")
def build_normed_streams_embedding(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> NormedStreamsEmbedding:
    return NormedStreamsEmbedding(
        int(desc["vocab_size"]), int(desc["hidden_size"]), str(desc["name"]), str(desc["norm_name"]), float(desc["eps"]),
        int(desc.get("copies", 1)), dtype, device, weight_offset=float(desc.get("weight_offset", 0.0)),
    )


class PairHashEmbedding(TokenEmbedding):
    """`table[token]` plus a row of a second table chosen by the token AND the one before it:

        row = (previous * mul_prev + token * mul_cur) mod buckets        (the table has buckets + 1 rows)

    and the last row, number `buckets`, for a sequence's first token.  The token before a step's
    first one belongs to the request's state: one int32 per request, asked of the cache manager
    like a mixer's state (zeroed at admission, freed with the request, copied aside and put back
    around a failing step), read and left behind by the kernel that gathers the rows."""

    def __init__(self, vocab_size: int, hidden_size: int, name: str, pair_name: str, buckets: int, mul_prev: int,
                 mul_cur: int, dtype: torch.dtype, device) -> None:
        super().__init__(vocab_size, hidden_size, name, dtype, device)
        if buckets <= 0:
            raise ValueError(f"a pair table needs a positive number of buckets, got {buckets}")
        self.pair_name, self.buckets, self.mul_prev, self.mul_cur = pair_name, int(buckets), int(mul_prev), int(mul_cur)
        self.pairs: torch.Tensor | None = None

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        return {**super().param_specs(prefix), prefix + self.pair_name: ParamSpec((self.buckets + 1, self.hidden_size))}

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        super().load_params(prefix, get)
        self.pairs = get(prefix + self.pair_name).contiguous()

    def cache_needs(self, page_size: int) -> CacheNeeds:
        return CacheNeeds(state=StateNeeds((1,), torch.int32))

    def forward(self, ctx: StepContext, cache: LayerCache | None = None) -> torch.Tensor:
        assert self.weight is not None and self.pairs is not None, "embedding used before its tables were loaded"
        if cache is None or cache.state is None:
            raise ValueError("a pair-hash embedding needs its state rows (the token before each request's next one)")
        residual, cast = ops.embed_pair_hash(
            self.weight, self.pairs, ctx.token_ids, ctx.positions, ctx.token_request, ctx.cu_seqlens_q, ctx.state_slots,
            cache.state, mul_prev=self.mul_prev, mul_cur=self.mul_cur, want_cast=self.dtype != torch.float32,
        )
        if cast is not None:
            ctx.shared[STREAM_CAST] = (residual, cast)
        return residual


@register_embedding("pair_hash_embedding")
def build_pair_hash_embedding(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> PairHashEmbedding:
    return PairHashEmbedding(
        int(desc["vocab_size"]), int(desc["hidden_size"]), str(desc["name"]), str(desc["pair_name"]), int(desc["buckets"]),
        int(desc["mul_prev"]), int(desc["mul_cur"]), dtype, device,
    )

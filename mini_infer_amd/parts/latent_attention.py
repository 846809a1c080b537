"""Attention over one small latent row per token.

Every head's keys and values are linear maps of a latent `c` of `kv_rank` numbers per token;
beside it one rotated key part `r` of `rot_dim` numbers is shared by all heads:

    [x_c | x_r] = W_dkv h        c = rms_norm(x_c) * w_c        r = rotate(x_r, position)
    q_a = W_q h  laid out per head as [plain (head_dim) | to rotate (rot_dim)]
    score_a(i, j) = (q_a,plain(i) . W_uk,a c(j) + rotate(q_a,rot(i)) . r(j)) * scale
    out = W_o concat_a( sum_j softmax_j(score_a(i, .)) W_uv,a c(j) )

Only `[c | r]` is cached: one key head of `kv_rank + rot_dim` numbers a token, whatever the
number of heads.  Over the cache the key map is folded into the query, `q'_a = W_uk,a^T
q_a,plain`, so a head's score is `[q'_a | q_a,rot] . [c | r]`, and the value map is applied
after the attention, `W_uv,a (sum_j p_j c(j))`: the attention itself is the paged kernel with
a single key/value head whose value row is the front part of its key row.

A step in which every request begins (prompts that come whole, or first portions) has all its
keys at hand, and there the folded form is the dearer one: every head would score against
kv_rank + rot_dim numbers a key instead of head_dim + rot_dim.  Such a step writes keys and
values out per head into pages of its own and runs the matrix-core attention kernel over them
like any other layer (bfloat16, head sizes it takes); the cache gets the same `[c | r]` rows
either way.  The two forms differ by rounding only.
"""

from __future__ import annotations

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

DEFAULT_NAMES = {"q": "q", "down": "dkv", "down_norm": "dkv.norm", "up_k": "uk", "up_v": "uv", "out": "o",
                 "q_down": "dq", "q_down_norm": "dq.norm", "q_up": "uq", "sink": "sink"}


class LatentAttention(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, v_head_dim: int, kv_rank: int,
                 position: PositionEncoding, scale: float, norm_eps: float, dtype: torch.dtype, device, *,
                 names: dict[str, str] | None = None, suffix: str = "", q_rank: int | None = None, window: int | None = None,
                 learned_sink: bool = False) -> None:
        """`q_rank`: the queries go through a latent of their own, `q = W_uq rms_norm(W_dq h)` (tensors
        `q_down`, `q_down_norm`, `q_up` of `names`) instead of one product `W_q h`.  `window`: position i
        sees only the last `window` positions, itself included.  `learned_sink`: the softmax's
        denominator holds `exp(sink_h)` too, `sink_h` a learned number per head (tensor `sink`)."""
        super().__init__(dtype, device)
        if q_rank is not None and q_rank <= 0:
            raise ValueError(f"latent attention: q_rank must be positive, got {q_rank}")
        if window is not None and window <= 0:
            raise ValueError(f"latent attention: the window must be positive, got {window}")
        self.q_rank, self.window, self.learned_sink = q_rank, window, bool(learned_sink)
        for what, value in (("hidden_size", hidden_size), ("num_heads", num_heads), ("head_dim", head_dim),
                            ("v_head_dim", v_head_dim), ("kv_rank", kv_rank)):
            if value <= 0:
                raise ValueError(f"latent attention: {what} must be positive, got {value}")
        if rot_dim < 0 or rot_dim % 2 or kv_rank % 2:
            raise ValueError(f"latent attention: rot_dim={rot_dim} and kv_rank={kv_rank} must be even")
        layout = position.rotary_layout()
        if layout != (rot_dim, True):
            raise ValueError(f"latent attention rotates {rot_dim} entries in neighbouring pairs; the encoding gives {layout}")
        if kv_rank + rot_dim > ops.kernels.GENERAL_ATTENTION_MAX_KEY_DIM or kv_rank > ops.kernels.GENERAL_ATTENTION_MAX_VALUE_DIM:
            raise ValueError(
                f"latent attention: cached rows of {kv_rank} + {rot_dim} exceed what the attention kernel takes "
                f"({ops.kernels.GENERAL_ATTENTION_MAX_VALUE_DIM} for the latent, {ops.kernels.GENERAL_ATTENTION_MAX_KEY_DIM} in all)"
            )
        self.hidden_size, self.num_heads, self.head_dim, self.rot_dim = hidden_size, num_heads, head_dim, rot_dim
        self.v_head_dim, self.kv_rank = v_head_dim, kv_rank
        self.position, self.scale, self.norm_eps = position, float(scale), float(norm_eps)
        self.names = {**DEFAULT_NAMES, **(names or {})}
        n = self.names
        self.q_head_width = head_dim + rot_dim
        if q_rank is None:
            # one product yields [q of every head | x_c | x_r]
            self.q_down = Linear(hidden_size, [num_heads * self.q_head_width, kv_rank + rot_dim], [n["q"], n["down"]], dtype,
                                 device, suffix=suffix)
            self.q_up = None
        else:
            # one product yields [the queries' latent | x_c | x_r]; the queries are a second product
            self.q_down = Linear(hidden_size, [q_rank, kv_rank + rot_dim], [n["q_down"], n["down"]], dtype, device, suffix=suffix)
            self.q_up = Linear(q_rank, num_heads * self.q_head_width, n["q_up"], dtype, device, suffix=suffix)
        self.q_latent_norm: torch.Tensor | None = None
        self.sinks: torch.Tensor | None = None
        self.up_k = Linear(kv_rank, num_heads * head_dim, n["up_k"], dtype, device, suffix=suffix)
        self.up_v = Linear(kv_rank, num_heads * v_head_dim, n["up_v"], dtype, device, suffix=suffix)
        self.out = Linear(num_heads * v_head_dim, hidden_size, n["out"], dtype, device, suffix=suffix)
        self.latent_norm: torch.Tensor | None = None
        self.fold_k: torch.Tensor | None = None  # [heads, kv_rank, head_dim]: W_uk,a transposed
        self.map_v: torch.Tensor | None = None  # [heads, v_head_dim, kv_rank]
        self._out_padded: torch.Tensor | None = None  # W_o with zero columns where expanded value heads are padded

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        specs = {
            **self.q_down.param_specs(prefix), **self.up_k.param_specs(prefix), **self.up_v.param_specs(prefix),
            **self.out.param_specs(prefix),
            prefix + self.names["down_norm"]: ParamSpec((self.kv_rank,), init="norm_weight", dtype="float32"),
        }
        if self.q_up is not None:
            specs.update(self.q_up.param_specs(prefix))
            specs[prefix + self.names["q_down_norm"]] = ParamSpec((self.q_rank,), init="norm_weight", dtype="float32")
        if self.learned_sink:
            specs[prefix + self.names["sink"]] = ParamSpec((self.num_heads,), dtype="float32")
        return specs

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        self.q_down.load_params(prefix, get)
        self.up_k.load_params(prefix, get)
        self.up_v.load_params(prefix, get)
        self.out.load_params(prefix, get)
        self.latent_norm = get(prefix + self.names["down_norm"]).float().contiguous()
        if self.q_up is not None:
            self.q_up.load_params(prefix, get)
            self.q_latent_norm = get(prefix + self.names["q_down_norm"]).float().contiguous()
        if self.learned_sink:
            self.sinks = get(prefix + self.names["sink"]).float().contiguous()
        assert self.up_k.weight is not None and self.up_v.weight is not None
        self.fold_k = self.up_k.weight.view(self.num_heads, self.head_dim, self.kv_rank).transpose(1, 2).contiguous()
        self.map_v = self.up_v.weight.view(self.num_heads, self.v_head_dim, self.kv_rank)
        self._out_padded = None

    def cache_needs(self, page_size: int) -> CacheNeeds:
        # one key head, rows [c | r]; the values are the rows' front part: no value pages
        return CacheNeeds(pages=PagedKVNeeds(1, self.kv_rank + self.rot_dim, self.window, v_head_dim=0))

    EXPAND_MIN_TOKENS = 64  # steps of fewer tokens take the folded form whatever they hold

    def _expands(self, ctx: StepContext) -> bool:
        """Whether this step writes keys and values out per head: every request begins in it (known
        on the host), and the matrix-core attention kernel takes the sizes."""
        width = self.head_dim + self.rot_dim
        if self.dtype != torch.bfloat16 or ctx.host_cu_seqlens_q is None or ctx.host_seq_lens is None:
            return False
        if ctx.num_tokens < self.EXPAND_MIN_TOKENS or ctx.max_q_len < 2 or self.v_head_dim > width:
            return False  # (a step of single tokens that is being recorded says nothing true about lengths)
        if torch.cuda.is_current_stream_capturing():
            return False  # (this form makes its index on the host)
        if not ops.mfma_attention_supported(self.dtype, width, ctx.page_size):
            return False
        cu = ctx.host_cu_seqlens_q
        return all(ctx.host_seq_lens[b] == cu[b + 1] - cu[b] for b in range(len(ctx.host_seq_lens)))

    def _own_pages(self, ctx: StepContext) -> tuple[torch.Tensor, torch.Tensor, int]:
        """Write slots, block table and page count of pages that hold this step's tokens alone, each
        request from a page of its own on (made once a step, on the host, for all layers that expand)."""
        key = ("latent_attention_own_pages", ctx.page_size)
        if key not in ctx.shared:
            import numpy as np

            cu, page = np.asarray(ctx.host_cu_seqlens_q, dtype=np.int64), ctx.page_size
            lengths = cu[1:] - cu[:-1]
            pages = -(-lengths // page)
            first = np.concatenate([[0], np.cumsum(pages)])
            request_of = np.repeat(np.arange(len(lengths)), lengths)
            slots = first[request_of] * page + (np.arange(cu[-1]) - cu[request_of])
            table = np.zeros((len(lengths), max(1, int(pages.max()))), dtype=np.int32)
            for b, count in enumerate(pages):
                table[b, :count] = first[b] + np.arange(count)
            both = torch.from_numpy(np.concatenate([slots.astype(np.int32), table.reshape(-1)])).to(self.device)
            ctx.shared[key] = (both[: slots.size], both[slots.size:].view(table.shape), int(first[-1]))
        return ctx.shared[key]

    def _forward_expanded(self, proj: torch.Tensor, down, c_col: int, ctx: StepContext, cache: LayerCache,
                          writes_cache: bool) -> torch.Tensor:
        heads, rank, rot, dim, vdim = self.num_heads, self.kv_rank, self.rot_dim, self.head_dim, self.v_head_dim
        width, tokens = dim + rot, proj.shape[0]
        rotary = self.position.rotary(ctx)
        latent = torch.empty((tokens, rank), dtype=proj.dtype, device=proj.device)
        ops.latent_prepare(
            proj, rotary.cos, rotary.sin, self.latent_norm, ctx.slot_mapping[cache.group] if writes_cache else None,
            cache.k_pages, None, heads=heads, q_head_width=self.q_head_width, q_rot_at=dim, c_col=c_col,
            rank=rank, rot=rot, eps=self.norm_eps, latent_out=latent, down=down,
        )
        qkv = ops.latent_expand(proj, self.up_k.forward(latent), self.up_v.forward(latent), rotary.cos, rotary.sin, heads=heads,
                                dim=dim, rot=rot, vdim=vdim, r_col=c_col + rank, down=down)
        slots, table, pages = self._own_pages(ctx)
        # (zeroed: the kernel multiplies what lies past a request's last key by a weight of zero)
        k_own = torch.zeros((pages, heads, ctx.page_size, width), dtype=proj.dtype, device=proj.device)
        v_own = torch.zeros((pages, heads, width, ctx.page_size), dtype=proj.dtype, device=proj.device)
        nothing = torch.empty((tokens, 0), dtype=torch.float32, device=proj.device)
        ops.rope_kv_write(qkv, nothing, nothing, slots, k_own, v_own, q_heads=heads, kv_heads=heads, head_dim=width,
                          rotary_dim=0, v_transposed=True)
        mixed = ops.paged_attention(
            qkv, k_own, v_own, table, ctx.token_request, ctx.positions, ctx.cu_seqlens_q, ctx.host_cu_seqlens_q, q_heads=heads,
            kv_heads=heads, head_dim=width, scale=self.scale, window=self.window, max_seq_len=ctx.max_q_len, v_transposed=True,
            sinks=self.sinks,
        )
        if self._out_padded is None:  # W_o with zero columns under the padding of every value head
            assert self.out.weight is not None
            padded = torch.zeros((self.hidden_size, heads, width), dtype=self.out.weight.dtype, device=self.out.weight.device)
            padded[:, :, :vdim] = self.out.weight.view(self.hidden_size, heads, vdim)
            self._out_padded = padded.view(self.hidden_size, heads * width)
        return ops.linear(mixed, self._out_padded)

    def forward(self, x, ctx: StepContext, cache: LayerCache, writes_cache: bool = True):
        assert cache.group is not None and cache.k_pages is not None
        assert self.fold_k is not None and self.map_v is not None and self.latent_norm is not None, \
            "latent attention used before its weights were loaded"
        if hasattr(x, "finish"):
            x = x.finish()
        heads, rank, rot, width = self.num_heads, self.kv_rank, self.rot_dim, self.kv_rank + self.rot_dim
        proj = self.q_down.forward(x)
        down, c_col = None, heads * self.q_head_width
        if self.q_up is not None:
            # [the queries' latent | x_c | x_r]: the latent is normed, and the queries are a product of their own
            assert self.q_latent_norm is not None
            down, c_col = proj, self.q_rank
            proj = self.q_up.forward(ops.norm_rows(proj, self.q_latent_norm, self.norm_eps, width=self.q_rank))
        if self._expands(ctx):
            return self._forward_expanded(proj, down, c_col, ctx, cache, writes_cache)
        tokens = proj.shape[0]
        rotary = self.position.rotary(ctx)
        queries = torch.empty((tokens, heads * width), dtype=proj.dtype, device=proj.device)
        ops.latent_prepare(
            proj, rotary.cos, rotary.sin, self.latent_norm, ctx.slot_mapping[cache.group] if writes_cache else None,
            cache.k_pages, queries, heads=heads, q_head_width=self.q_head_width, q_rot_at=self.head_dim,
            c_col=c_col, rank=rank, rot=rot, eps=self.norm_eps, down=down,
        )
        # the key map folded into the queries: q'_a = W_uk,a^T q_a,plain
        plain = proj[:, : heads * self.q_head_width].unflatten(1, (heads, self.q_head_width))[:, :, : self.head_dim]
        ops.linear_per_head(plain, self.fold_k, queries.unflatten(1, (heads, width))[:, :, :rank])
        mixed = ops.paged_attention(
            queries, cache.k_pages, None, ctx.block_tables[cache.group], ctx.token_request, ctx.positions,
            ctx.cu_seqlens_q, ctx.host_cu_seqlens_q, q_heads=heads, kv_heads=1, head_dim=width, scale=self.scale,
            window=self.window, max_seq_len=ctx.max_seq_len, v_head_dim=rank, sinks=self.sinks,
        )
        # the value map after the attention: W_uv,a (sum_j p_j c_j)
        values = torch.empty((tokens, heads * self.v_head_dim), dtype=proj.dtype, device=proj.device)
        ops.linear_per_head(mixed.unflatten(1, (heads, rank)), self.map_v, values.unflatten(1, (heads, self.v_head_dim)))
        return self.out.forward(values)


@register_mixer("latent_attention")
def build_latent_attention(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> LatentAttention:
    pos_desc = desc["position"]
    key = ("position", repr(sorted(pos_desc.items(), key=lambda kv: kv[0])))
    position = shared.get(key) if shared is not None else None
    if position is None:
        position = POSITION_ENCODINGS.lookup(pos_desc["kind"])(pos_desc, dtype, device, shared)
        if shared is not None:
            shared[key] = position
    return LatentAttention(
        int(desc["hidden_size"]), int(desc["num_heads"]), int(desc["head_dim"]), int(desc["rot_dim"]),
        int(desc["v_head_dim"]), int(desc["kv_rank"]), position, float(desc["scale"]), float(desc["norm_eps"]), dtype, device,
        names=desc.get("names"), suffix=str(desc.get("suffix", "")), q_rank=desc.get("q_rank"), window=desc.get("window"),
        learned_sink=bool(desc.get("learned_sink", False)),
    )

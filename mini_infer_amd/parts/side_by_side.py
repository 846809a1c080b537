"""Two mixers side by side: both read the same input, and the layer's mixer output is a
weighted sum of theirs.

    y = left_scale * left(h) + right_scale * right(h)

Each child keeps what it keeps (pages, state of fixed size): the pair asks the cache manager
for the union and hands each child its own share.  The sum is left to whoever writes it into
the stream (`ops.WeightedSum`), so it costs no launch of its own.
"""

from __future__ import annotations

import dataclasses

import torch

from mini_infer_amd import ops
from mini_infer_amd.parts.base import CacheNeeds, LayerCache, Mixer, ParamSpec, StateNeeds, StepContext, TensorGetter
from mini_infer_amd.registry import MIXERS, register_mixer


class SideBySideMixer(Mixer):
    def __init__(self, left: Mixer, right: Mixer, left_scale: float, right_scale: float, dtype: torch.dtype, device, *,
                 names: tuple[str, str] = ("left.", "right.")) -> None:
        super().__init__(dtype, device)
        self.children = (left, right)
        self.scales = (float(left_scale), float(right_scale))
        self.names = tuple(names)

    @property
    def graph_safe(self) -> bool:  # type: ignore[override]
        return all(child.graph_safe for child in self.children)

    def param_specs(self, prefix: str) -> dict[str, ParamSpec]:
        specs: dict[str, ParamSpec] = {}
        for name, child in zip(self.names, self.children):
            specs.update(child.param_specs(prefix + name))
        return specs

    def load_params(self, prefix: str, get: TensorGetter) -> None:
        for name, child in zip(self.names, self.children):
            child.load_params(prefix + name, get)

    def cache_needs(self, page_size: int) -> CacheNeeds:
        """The children's needs together: pages from the one child that asks for them, every
        state tensor under its child's name."""
        pages, state = None, {}
        for name, child in zip(self.names, self.children):
            need = child.cache_needs(page_size)
            if need.pages is not None:
                if pages is not None:
                    raise ValueError("two mixers side by side that both keep pages share one call's cache; not built")
                pages = need.pages
            if isinstance(need.state, StateNeeds):
                state[name] = need.state
            elif need.state is not None:
                state.update({name + key: one for key, one in need.state.items()})
        return CacheNeeds(pages=pages, state=state or None)

    def _share(self, cache: LayerCache, name: str, child: Mixer, page_size: int) -> LayerCache:
        need = child.cache_needs(page_size).state
        mine = None
        if isinstance(need, StateNeeds):
            mine = cache.state[name]
        elif need is not None:
            mine = {key: cache.state[name + key] for key in need}
        return dataclasses.replace(cache, state=mine)

    def forward(self, x, ctx: StepContext, cache: LayerCache, writes_cache: bool = True):
        if hasattr(x, "finish"):
            x = x.finish()
        left, right = (
            child.forward(x, ctx, self._share(cache, name, child, ctx.page_size), writes_cache)
            for name, child in zip(self.names, self.children)
        )
        left = left.finish() if hasattr(left, "finish") else left
        right = right.finish() if hasattr(right, "finish") else right
        return ops.WeightedSum(left, right, self.scales[0], self.scales[1])


@register_mixer("side_by_side")
def build_side_by_side(desc: dict, dtype: torch.dtype, device, shared: dict | None = None) -> SideBySideMixer:
    """`desc`: `left`, `right` (mixer descriptions with a `kind`), `left_scale`, `right_scale`, optional `names`."""
    left = MIXERS.lookup(desc["left"]["kind"])(desc["left"], dtype, device, shared)
    right = MIXERS.lookup(desc["right"]["kind"])(desc["right"], dtype, device, shared)
    extra = {"names": tuple(desc["names"])} if "names" in desc else {}
    return SideBySideMixer(left, right, float(desc.get("left_scale", 1.0)), float(desc.get("right_scale", 1.0)), dtype, device, **extra)

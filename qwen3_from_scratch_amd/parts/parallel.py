"""Two mixers side by side."""

import torch

from .. import ops
from ..cache.storage import LayerCacheView
from ..config.registry import register_part
from .base import CacheNeed, PagedTensor, Part, build_part


@register_part("mixer", "parallel")
class ParallelMixers(Part):
    """left_scale * left(h) + right_scale * right(h): two mixers of any registered kinds that read
    the same input, with their tensors under `<prefix>.left` and `<prefix>.right`. The layer's
    cache plane holds what both keep: the paged tensors of either under the side's name
    ("left.keys"), and one float32 state vector in which each side's state has its own stretch;
    each side sees a view of the cache with its own names and its own stretch."""

    graph_safe = True

    def __init__(self, prefix, precision, device, left, right, left_scale=1.0, right_scale=1.0):
        super().__init__(prefix, precision, device)
        self.sides = (("left", build_part(left, self._name("left"), precision, device), float(left_scale)),
                      ("right", build_part(right, self._name("right"), precision, device), float(right_scale)))
        if not all(getattr(side, "graph_safe", False) for _, side, _ in self.sides):
            self.graph_safe = False
        self._stretches = {}
        self._need = self._joined_need()

    def attach_position(self, position):
        for _, side, _ in self.sides:
            if hasattr(side, "attach_position"):
                side.attach_position(position)

    def cache_need(self):
        return self._need

    def _joined_need(self):
        paged, windows, at = [], set(), 0
        for name, side, _ in self.sides:
            need = side.cache_need() if hasattr(side, "cache_need") else None
            if need is None:
                continue
            for t in need.paged:
                paged.append(PagedTensor(name + "." + t.name, t.shape, t.token_axis, t.dtype))
            if need.paged:
                windows.add(need.window)
            if need.has_state:
                if len(need.state_shape) != 1 or need.state_dtype != torch.float32:
                    raise ValueError("sides of a parallel mixer keep their state as one float32 vector")
                self._stretches[name] = (at, at + need.state_shape[0])
                at += need.state_shape[0]
        if len(windows) > 1:
            raise ValueError("the sides of a parallel mixer page behind different windows")
        return CacheNeed(paged=tuple(paged), window=windows.pop() if windows else 0, state_shape=(at,) if at else (),
                         state_dtype=torch.float32)

    def tensors(self):
        names = {}
        for _, side, _ in self.sides:
            names.update(side.tensors())
        return names

    def load(self, fetch):
        for _, side, _ in self.sides:
            side.load(fetch)

    def _view(self, name, cache):
        view = LayerCacheView(writes=cache.writes, block_table=cache.block_table)
        view.paged = {key[len(name) + 1:]: t for key, t in cache.paged.items() if key.startswith(name + ".")}
        if name in self._stretches:
            first, last = self._stretches[name]
            view.state = cache.state[:, first:last]
        return view

    def forward(self, x, batch, cache):
        (ln, left, ls), (rn, right, rs) = self.sides
        a = left.forward(x, batch, self._view(ln, cache))
        b = right.forward(x, batch, self._view(rn, cache))
        return ops.scaled_sum(a, ls, b, rs)

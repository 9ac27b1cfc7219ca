"""Two mixers on one input, their results scaled and summed:
y = left_scale left(x) + right_scale right(x).

Either side is any registered mixer that takes an `out_scale` (applied to its result before its last
product, so the sum costs no pass of its own: the second side's product adds onto the first's).  A cache entry
holds what both sides ask for: pages for the one that attends, a fixed-size state for the one that recurs
(at most one of each kind).
"""
from __future__ import annotations

from ..cache.paged import split_request
from .base import MIXERS, Mixer, make_part, register_mixer
from .spec import PartSpec


@register_mixer("side_by_side")
class SideBySide(Mixer):
    """params: left, right (PartSpecs of mixers), left_scale, right_scale, left_prefix, right_prefix (put
    before the sides' tensor names)."""

    takes_normed = True
    can_overwrite = True

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        p = spec.params
        self.sides = []
        for side in ("left", "right"):
            inner = p[side]
            scaled = PartSpec(inner.kind, dict(inner.params, out_scale=float(p.get(side + "_scale", 1.0))))
            part = make_part(MIXERS, scaled, rt, "mixer")
            if not getattr(part, "can_overwrite", False) or not hasattr(part, "out_scale"):
                raise ValueError(f"side_by_side: the mixer {inner.kind!r} takes no out_scale")
            self.sides.append((p.get(side + "_prefix", side + "."), part))
        kinds = [split_request(part.cache_request()) for _, part in self.sides]
        if sum(kv is not None for kv, _ in kinds) > 1 or sum(st is not None for _, st in kinds) > 1:
            raise ValueError("side_by_side: both sides ask the cache for the same kind of storage")

    def tensor_specs(self):
        return {prefix + name: ts for prefix, part in self.sides for name, ts in part.tensor_specs().items()}

    def load(self, get):
        for prefix, part in self.sides:
            part.load(lambda name, p=prefix: get(p + name))

    def cache_request(self):
        asked = []
        for _, part in self.sides:
            asked += [r for r in split_request(part.cache_request()) if r is not None]
        return tuple(asked) if len(asked) > 1 else (asked[0] if asked else None)

    def decode_copies(self, make: bool, min_row_length: int = 0) -> int:
        return sum(part.decode_copies(make, min_row_length) for _, part in self.sides)

    def prepare(self, max_len: int) -> None:
        for _, part in self.sides:
            part.prepare(max_len)

    def forward(self, x, h, ctx, entry: int, writes_cache: bool, accumulate: bool = True) -> None:
        for i, (_, part) in enumerate(self.sides):
            part.forward(x, h, ctx, entry, writes_cache, accumulate=accumulate or i > 0)

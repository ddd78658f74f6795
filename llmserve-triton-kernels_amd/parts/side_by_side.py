"""Two mixers side by side: both read the same input, and the result is scale_a * a(h) + scale_b * b(h).

Parameters (a `PartSpec` of kind "side_by_side"): `mixers`, a list of two {"spec": PartSpec of a mixer, "scale": its
factor, "prefix": what its tensor names start with inside this part}.  Each keeps what it keeps by itself: the pair's
`cache_spec` is the tuple of both (pages for one, a state for the other), and each is handed its own view.  The two
results arrive unrounded (the mixers are asked for 32-bit results) and are summed in 32-bit.
"""

from __future__ import annotations

import torch

from ..ops import library as ops
from .registry import MIXERS, Mixer, register_mixer
from .spec import PagedCacheSpec, StateCacheSpec


@register_mixer("side_by_side")
class SideBySide(Mixer):
    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        entries = list(spec["mixers"])
        if len(entries) != 2:
            raise ValueError("two mixers stand side by side")
        self.members = [MIXERS.build(e["spec"], ctx) for e in entries]
        self.scales = [float(e.get("scale", 1.0)) for e in entries]
        self.prefixes = [str(e["prefix"]) for e in entries]
        if self.prefixes[0] == self.prefixes[1]:
            raise ValueError("the two mixers need different prefixes for their tensors")
        kinds = [self._kind(m.cache_spec()) for m in self.members]
        if kinds[0] is not None and kinds[0] == kinds[1]:
            raise ValueError("the two mixers keep the same kind of thing; one may keep pages and the other a state")
        self._kinds = kinds

    @staticmethod
    def _kind(spec):
        if spec is None:
            return None
        if isinstance(spec, PagedCacheSpec):
            return "pages"
        if isinstance(spec, StateCacheSpec):
            return "state"
        raise ValueError("a mixer that stands beside another keeps pages, a state or nothing")

    @property
    def graph_safe(self):
        return all(m.graph_safe for m in self.members)

    def libraries(self, dtype_name):
        names = ("stream32",)
        for m in self.members:
            names += tuple(m.libraries(dtype_name))
        return names

    def cache_spec(self):
        specs = tuple(s for s in (m.cache_spec() for m in self.members) if s is not None)
        return specs if len(specs) > 1 else (specs[0] if specs else None)

    def param_infos(self):
        infos = {}
        for prefix, m in zip(self.prefixes, self.members):
            for name, info in m.param_infos().items():
                infos[prefix + name] = info
        return infos

    def load(self, tensors):
        for prefix, m in zip(self.prefixes, self.members):
            m.load({name: tensors[prefix + name] for name in m.param_infos()})

    def forward(self, x, batch, cache):
        from ..cache.storage import PagedLayerCache

        views = cache if isinstance(cache, tuple) else (cache,)
        results = []
        for m, kind in zip(self.members, self._kinds):
            own = None
            for v in views:
                if v is not None and (kind == "pages") == isinstance(v, PagedLayerCache) and kind is not None:
                    own = v
            y = m.forward(x, batch, own)
            results.append(y if y.dtype == torch.float32 else y.float())
        a, b = results
        return ops.weighted_sum(a, a, b, self.scales[0], self.scales[1])

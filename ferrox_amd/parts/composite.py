"""Mixers made of other mixers.

`side_by_side`: several mixers read the same input rows, and the layer's output is their weighted sum,
    y = sum_i scale_i * mixer_i(x).
Each member adds its output, times its constant, into the float32 stream in its last product; nothing is summed in
between.  With `member_norms` every member's output is first normed over the model width,
    y = sum_i scale_i * N_i(mixer_i(x)),
N_i an RMS norm of the member's own (its constant folded into the norm's float32 weight): the member then writes
float32 rows of its own, which one kernel norms and adds.  What the members keep (pages, state) is kept side by side under the member's name: a member sees a cache of
its own with its own names.  At most one cache group of pages per layer: members that keep pages must name the
same group.
"""
from __future__ import annotations

import torch

from .. import debug, ops
from .base import MIXERS, NORMS, LayerCache, Mixer, PartSpec


@MIXERS.register("side_by_side")
class SideBySide(Mixer):
    def __init__(self, members: dict, scales: dict | None = None, member_norms: dict | None = None):
        """`members`: name -> PartSpec of a mixer whose `forward` takes `out_scale` (its tensors lie under the
        spec's prefix); `scales`: name -> constant (1 where absent); `member_norms`: name -> PartSpec of an RMS norm
        with a weight over the model width, applied to that member's output before it is scaled and added (its
        tensor is named by the spec, under this mixer's own prefix)."""
        if not members:
            raise ValueError("a side-by-side mixer needs members")
        self.members = {name: MIXERS.build(spec) for name, spec in members.items()}
        self._prefixes = {name: spec.prefix for name, spec in members.items()}
        self.scales = {name: float((scales or {}).get(name, 1.0)) for name in members}
        unknown = set(member_norms or {}) - set(members)
        if unknown:
            raise ValueError(f"norms for {sorted(unknown)}, which are no members")
        # (a member's constant rides on its norm's weight, which is kept in float32)
        self.norms = {name: NORMS.build(PartSpec(spec.kind, dict(spec.args, gain=spec.args.get("gain", 1.0) * self.scales[name])))
                      for name, spec in (member_norms or {}).items()}
        self._norm_prefixes = {name: spec.prefix for name, spec in (member_norms or {}).items()}
        unknown = set(scales or {}) - set(members)
        if unknown:
            raise ValueError(f"scales for {sorted(unknown)}, which are no members")
        self.graph_safe = all(m.graph_safe for m in self.members.values())
        libs = []
        for m in self.members.values():
            libs += [lib for lib in m.kernel_libraries if lib not in libs]
        self.kernel_libraries = tuple(libs)
        groups = {m.cache_group() for m in self.members.values() if m.page_shapes(16)}
        if len(groups) > 1:
            raise ValueError(f"the members of a side-by-side mixer keep pages of different cache groups: {sorted(map(str, groups))}")
        self._group = next(iter(groups)) if groups else None
        windows = [m.window for m in self.members.values() if m.page_shapes(16)]
        self.window = windows[0] if windows else None

    def children(self):
        return [(self._prefixes[name], m) for name, m in self.members.items()] \
            + [(self._norm_prefixes[name], n) for name, n in self.norms.items()]

    def page_shapes(self, block_size: int) -> dict:
        return {f"{name}.{key}": shape for name, m in self.members.items() for key, shape in m.page_shapes(block_size).items()}

    def state_shapes(self) -> dict:
        return {f"{name}.{key}": shape for name, m in self.members.items() for key, shape in m.state_shapes().items()}

    def cache_group(self):
        return self._group if self._group is not None else super().cache_group()

    @staticmethod
    def _own(tensors: dict, name: str) -> dict:
        return {key[len(name) + 1:]: t for key, t in tensors.items() if key.startswith(name + ".")}

    def forward(self, x, ctx, cache, residual) -> None:
        for name, m in self.members.items():
            own = LayerCache(self._own(cache.pages, name), self._own(cache.state, name), cache.group, cache.block_size, cache.writes)
            norm = self.norms.get(name)
            if norm is None:
                m.forward(x, ctx, own, residual, out_scale=self.scales[name])
                continue
            rms = norm.rms_params()
            if rms is None:
                raise ValueError(f"member '{name}': its output's norm must be an RMS norm with a weight")
            rows = torch.empty_like(residual)
            if getattr(m, "takes_fresh", False):      # the member stores its rows; any other adds into zeroed ones
                m.forward(x, ctx, own, rows, fresh=True)
            else:
                ops.fill_u32(rows, 0)
                m.forward(x, ctx, own, rows)
            debug.region("member norm")
            ops.rmsnorm_add(residual, rows, rms[0], rms[1])

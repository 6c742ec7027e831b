"""Several mixers side by side: each reads the same input, and the result is the weighted sum
sum_i scales[i] * mixers[i](x), added up in floats.

At most one of them keeps pages of keys and values; what the others keep per request (and what
that one keeps beside its pages) lies one behind the other in the request's state slot.
"""
from __future__ import annotations

from dataclasses import replace
from typing import List

from ..runtime.device import F32, Tensor
from .base import PagedKV, Part, StateNeed, build_part, register_part

MOST = 4       # terms of the kernel that adds them up


class SideBySide(Part):
    graph_safe = True      # its own launch takes nothing from the host; its mixers say so for theirs

    def __init__(self, spec):
        self.spec = spec
        if not (1 <= len(spec.mixers) <= MOST) or len(spec.mixers) != len(spec.scales):
            raise ValueError(f"1 to {MOST} mixers side by side, each with a scale: got {len(spec.mixers)} and "
                             f"{len(spec.scales)}")
        self.mixers = [build_part("mixer", m) for m in spec.mixers]
        needs = [m.cache_need() for m in self.mixers]
        paged = [i for i, n in enumerate(needs) if isinstance(n, PagedKV)]
        if len(paged) > 1:
            raise ValueError("at most one of the mixers side by side keeps pages of keys")
        self.paged = paged[0] if paged else None
        # where each mixer's state begins, counted from the start of the whole
        self.offsets, at = [], 0
        for n in needs:
            self.offsets.append(at)
            nbytes = n.nbytes if isinstance(n, StateNeed) else getattr(n, "state_bytes", 0) if n is not None else 0
            at += (int(nbytes) + 15) // 16 * 16
        self.state_bytes = at
        self._needs = needs

    def children(self):
        return list(self.mixers)

    def cache_need(self):
        if self.paged is not None:
            return replace(self._needs[self.paged], state_bytes=self.state_bytes)
        return StateNeed(self.state_bytes) if self.state_bytes else None

    def flops_per_key(self) -> float:
        return self.mixers[self.paged].flops_per_key() if self.paged is not None else 0.0

    def wants_v_transposed(self, kernels, dtype: str, page_size: int) -> bool:
        m = self.mixers[self.paged] if self.paged is not None else None
        return bool(m is not None and hasattr(m, "wants_v_transposed") and m.wants_v_transposed(kernels, dtype, page_size))

    def forward(self, ctx, x: Tensor, cache) -> Tensor:
        T = x.shape[0]
        ys = []
        for m, off in zip(self.mixers, self.offsets):
            ys.append(m.forward(ctx, x, replace(cache, state_offset=cache.state_offset + off)))
        if any(y.layout == "parts" or y.dtype != ctx.dtype for y in ys):
            raise ValueError("mixers side by side hand back plain activations")
        W = ys[0].shape[1]
        ptrs = [y.ptr for y in ys] + [None] * (MOST - len(ys))
        sc = [float(v) for v in self.spec.scales] + [0.0] * (MOST - len(ys))
        out = ctx.alloc((1, T, W), F32)
        ctx.k.zk_weighted_sum(ptrs[0], sc[0], ptrs[1], sc[1], ptrs[2], sc[2], ptrs[3], sc[3], out.ptr, T, W, ctx.stream)
        if getattr(ctx, "plane_welcome", None) is self:
            # one float plane: the block's joining kernel reads it as it reads a product's partial sums
            return Tensor(out.ptr, (1, T, W), F32, out.owner, layout="parts")
        y = ctx.alloc((T, W))
        ctx.k.zk_planes_sum(out.ptr, 1, y.ptr, T, W, ctx.stream)
        return y


register_part("mixer", "side_by_side", SideBySide)

"""Differential attention over the paged cache: two softmax maps per head over the same values.

    q = [q1 | q2] per head, k = [k1 | k2] per key head, v per key head; no rotation
    q <- q (1 + coef ln(floor((p + 1) / every) + 1))                a temperature of the position p
    s_m = cap tanh((q_m . k_m) scale / cap),   a_m = softmax(s_m) v,   m = 1, 2
    lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff                  one number a layer
    o = a_1 - lambda a_2;   o <- o / sqrt(mean(o^2) + eps) (1 - diff);   out = W_o o

A key head of the cache holds both maps' keys side by side (2 D channels), so a token's keys are
stored once and one block table serves both maps.  Keys and values go to the cache as projected;
the temperature is applied to the float queries inside the attention kernel, so no rounding
lies between.  One path for whole prompts, portions and decoded tokens, reading the cache alone.
"""
from __future__ import annotations

import math
from typing import List

import numpy as np

from ..runtime.device import Tensor
from .base import ROLE_GAIN, PagedKV, Part, TensorReq, register_part
from .ops import linear


class DifferentialAttention(Part):
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        s = self.spec = spec
        if s.num_heads % s.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if not (1 <= s.head_dim <= 256 and 1 <= s.value_dim <= 256):
            raise ValueError(f"head_dim and value_dim must lie in 1..256, got {s.head_dim} and {s.value_dim}")
        if s.temp_every < 0 or (s.window is not None and s.window < 1):
            raise ValueError(f"temp_every must not be negative and a window positive, got {s.temp_every} and {s.window}")
        self.w_qkv = self.w_o = None
        self.lam = float(s.diff)

    def tensor_reqs(self) -> List[TensorReq]:
        s, n = self.spec, self.spec.names
        H, G, D, E, W = s.num_heads, s.num_kv_heads, s.head_dim, s.value_dim, s.hidden_size
        return [TensorReq(n["q"], (H * 2 * D, W)), TensorReq(n["k"], (G * 2 * D, W)), TensorReq(n["v"], (G * E, W)),
                TensorReq(n["o"], (W, H * E))] + [TensorReq(n[r], (D,), ROLE_GAIN) for r in ("lq1", "lk1", "lq2", "lk2")]

    def load(self, weights, rt, dtype):
        s, n = self.spec, self.spec.names
        strip = getattr(weights, "wants_strip", None)
        self.w_qkv = weights.matrix([n["q"], n["k"], n["v"]], strip=bool(strip and strip(s.hidden_size)))
        self.w_o = weights.matrix([n["o"]], strip=bool(strip and strip(s.num_heads * s.value_dim)))
        # lambda is a constant of the layer: made once, in double precision, from the four vectors
        vec = {r: rt.download(weights.vector(n[r])).astype(np.float64) for r in ("lq1", "lk1", "lq2", "lk2")}
        self.lam = (math.exp(float((vec["lq1"] * vec["lk1"]).sum())) - math.exp(float((vec["lq2"] * vec["lk2"]).sum()))
                    + float(s.diff))

    def cache_need(self):
        s = self.spec
        return PagedKV(s.num_kv_heads, 2 * s.head_dim, s.window, value_dim=s.value_dim)

    def flops_per_key(self) -> float:
        s = self.spec
        return 2.0 * s.num_heads * 2 * (s.head_dim + s.value_dim)        # two maps: q.k and p.v each

    def forward(self, ctx, x: Tensor, cache) -> Tensor:
        s, k = self.spec, ctx.k
        T = x.shape[0]
        H, G, D, E = s.num_heads, s.num_kv_heads, s.head_dim, s.value_dim
        width = (H + G) * 2 * D + G * E
        g = ctx.group(cache.group)
        qkv = linear(ctx, x, self.w_qkv, ctx.alloc((T, width)))
        k.zk_cache_store(qkv.ptr, width, H * 2 * D, (H + G) * 2 * D, g.slot_map, cache.k.ptr, cache.v.ptr, T, G, 2 * D, E,
                         g.page_size, 1 if cache.v_transposed else 0, ctx.stream)
        o = ctx.alloc((T, H * E))
        k.zk_diff_attention_plain(qkv.ptr, width, cache.k.ptr, cache.v.ptr, g.block_table, g.max_blocks, ctx.req_of_token,
                                  ctx.positions, o.ptr, T, H, G, D, E, g.page_size, float(s.scale),
                                  float(s.softcap) if s.softcap else 0.0, int(s.window) if s.window else 0,
                                  1 if cache.v_transposed else 0, float(self.lam), float(s.diff), float(s.eps),
                                  float(s.temp_coef), int(s.temp_every), ctx.stream)
        return linear(ctx, o, self.w_o, ctx.alloc((T, s.hidden_size)), last_of=self)


register_part("mixer", "differential_attention", DifferentialAttention)

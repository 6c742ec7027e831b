"""Differential attention over the paged cache: two softmax maps per head over the same values.

    q = [q1 | q2] per head, k = [k1 | k2] per key head, v per key head; no rotation
    q <- q (1 + coef ln(floor((p + 1) / every) + 1))                a temperature of the position p
    s_m = cap tanh((q_m . k_m) scale / cap),   a_m = softmax(s_m) v,   m = 1, 2
    lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff                  one number a layer
    o = a_1 - lambda a_2;   o <- o / sqrt(mean(o^2) + eps) (1 - diff);   out = W_o o

The cache keeps a key head per (key/value head, map) and one value head per key/value head
(``PagedKV.value_heads``): one block table serves both maps, and the values are stored once.  Keys
and values go to the cache as projected.  One path for whole prompts, portions and decoded tokens,
reading the cache alone.  Two kernels: the plain one (any sizes, 32-bit) does both maps, the
temperature on the float queries and the join in one launch; where keys and values have one of the
matrix-core attention's sizes (bfloat16), that kernel runs the 2 H maps as heads of their own whose
pairs share a value head, behind a launch that scales the queries and before one that joins the pairs.
"""
from __future__ import annotations

import math
from typing import List

import numpy as np

from ..runtime.device import BF16, Tensor
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
        self.decode_chunk = 64                     # keys a wave of the split decode attention takes

    def wants_v_transposed(self, kernels, dtype: str, page_size: int) -> bool:
        """Whether the matrix-core kernel serves this layer (it reads V as [page][head][channel][slot])."""
        s = self.spec
        return bool(dtype == BF16 and s.value_dim == s.head_dim and kernels.has("zk_attention_bf16_maps") and
                    kernels.zk_attention_bf16_supports(2 * s.num_heads, 2 * s.num_kv_heads, s.head_dim, page_size))

    def prepare(self, kernels, dtype, max_seqs, max_model_len, page_size, max_batch_tokens=0) -> int:
        """Workspace of the split attention of decoded tokens at the runner's limits, and the number
        of keys a wave of it takes (fixed by the limits, never by a step's batch)."""
        s = self.spec
        if not self.wants_v_transposed(kernels, dtype, page_size):
            return 0
        nh, nkv = 2 * s.num_heads, 2 * s.num_kv_heads
        chunks = -(-int(max_model_len) // 64)
        self.decode_chunk = 32 if int(max_seqs) * nkv * chunks <= 512 else 64
        longest = int(kernels.zk_attention_bf16_max_context(nh, nkv, s.head_dim, self.decode_chunk))
        if max_model_len > longest:
            raise ValueError(f"differential attention with {s.num_heads} heads, {s.num_kv_heads} KV heads of {s.head_dim}: the "
                             f"longest context its decode kernel takes is {longest} tokens, the runner asks for {max_model_len}")
        need = int(kernels.zk_attention_bf16_workspace(int(max_seqs), nh, s.head_dim, int(max_model_len)))
        if max_batch_tokens > 0 and kernels.has("zk_attention_bf16_portion_workspace"):
            extra = int(kernels.zk_attention_bf16_portion_workspace(int(max_batch_tokens), nh, nkv, s.head_dim))
            need = (need + 255) // 256 * 256 + min(extra, 192 << 20)
        return need

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
        return PagedKV(2 * s.num_kv_heads, s.head_dim, s.window, value_dim=s.value_dim, value_heads=s.num_kv_heads)

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
        fast = bool(cache.v_transposed and ctx.tuned)
        store = (g.slot_map, cache.k.ptr, cache.v.ptr, T, 2 * G, D, G, E, g.page_size, 1 if cache.v_transposed else 0)
        if fast and s.temp_every > 0:
            # the matrix-core kernel takes its queries as they lie: the temperature in the storing launch
            k.zk_cache_store_temperature(qkv.ptr, width, H * 2 * D, H * 2 * D, (H + G) * 2 * D, ctx.positions, *store,
                                         float(s.temp_coef), int(s.temp_every), ctx.stream)
        else:
            k.zk_cache_store(qkv.ptr, width, H * 2 * D, (H + G) * 2 * D, *store, ctx.stream)
        o = ctx.alloc((T, H * E))
        cap, win = float(s.softcap) if s.softcap else 0.0, int(s.window) if s.window else 0
        if fast:
            # the 2 H maps as heads of the matrix-core kernel; a pair of key heads shares a value head
            maps = ctx.alloc((T, 2 * H * E))
            k.zk_attention_bf16_maps(qkv.ptr, width, cache.k.ptr, cache.v.ptr, g.block_table, g.max_blocks, ctx.q_start,
                                     ctx.ctx_len, maps.ptr, ctx.R, ctx.n_multi, ctx.max_q_len, ctx.max_ctx, 2 * H, 2 * G, D,
                                     g.page_size, float(s.scale), cap, win, self.decode_chunk, ctx.workspace.ptr,
                                     ctx.workspace.nbytes, 0, 0, 1 if getattr(s, "wide_weights", False) else 0, 1, ctx.stream)
            k.zk_diff_join(maps.ptr, o.ptr, T, H, E, float(self.lam), float(s.diff), float(s.eps), ctx.stream)
            return linear(ctx, o, self.w_o, ctx.alloc((T, s.hidden_size)), last_of=self)
        k.zk_diff_attention_plain(qkv.ptr, width, cache.k.ptr, cache.v.ptr, g.block_table, g.max_blocks, ctx.req_of_token,
                                  ctx.positions, o.ptr, T, H, G, D, E, g.page_size, float(s.scale),
                                  float(s.softcap) if s.softcap else 0.0, int(s.window) if s.window else 0,
                                  1 if cache.v_transposed else 0, float(self.lam), float(s.diff), float(s.eps),
                                  float(s.temp_coef), int(s.temp_every), ctx.stream)
        return linear(ctx, o, self.w_o, ctx.alloc((T, s.hidden_size)), last_of=self)


register_part("mixer", "differential_attention", DifferentialAttention)

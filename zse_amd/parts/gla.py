"""Gated linear attention: a recurrent mixer with a matrix state per head whose rows decay each
at its own rate.

Per head, D query/key channels and E value channels; the state S [D, E] starts at zero and is
carried as floats in the request's state slot:

    q = W_q x D^(-1/2),   k = W_k x,   v = W_v x
    alpha = sigmoid(W_a2 (W_a1 x) + b)^(1/tau)                       (per key channel, float)
    S <- diag(alpha) S + k v^T;   o = S^T q
    out = W_o ( o / sqrt(mean(o^2) + eps) * gain * silu(W_g x) )     (the mean per head, gain [E] shared by heads)

q, k, v, the gate and the narrow W_a1 are one product; W_a2 reads the last of its columns and
leaves floats.  One kernel walks the tokens of every (request, head), so steps of single tokens
and portions of prompts run the same arithmetic in the same order.  Where few long portions
would leave most of the chip idle, the kernel walks segments of a portion side by side (twice:
what each adds from zero, then, from the starting states that follow, the read-outs): the same
sums grouped by segments.
"""
from __future__ import annotations

from typing import List

from ..runtime.device import F32, ITEMSIZE, Tensor
from .base import ROLE_GAIN, Part, StateNeed, TensorReq, register_part
from .ops import linear


class GatedLinearAttention(Part):
    graph_safe = True      # rows, requests and slots are read by the kernels from device memory
    SEGMENT = 64           # tokens of a segment of a long portion
    ENOUGH_BLOCKS = 1024   # a plain walk with this many blocks fills the chip without segments

    def __init__(self, spec):
        s = self.spec = spec
        if s.key_dim > 256 or s.value_dim > 1024:
            raise ValueError(f"up to 256 key and 1024 value channels a head, got {s.key_dim} and {s.value_dim}")
        if not s.tau > 0 or s.decay_rank < 0:
            raise ValueError(f"tau must be positive and the decays' rank not negative, got {s.tau} and {s.decay_rank}")
        self.rank = int(s.decay_rank)          # 0: the checkpoint's tensors say it, at load
        self.qk = s.num_heads * s.key_dim
        self.vv = s.num_heads * s.value_dim
        self.w_in = self.w_a2 = self.w_o = self.a_bias = self.gain = None

    def tensor_reqs(self) -> List[TensorReq]:
        s, n, W = self.spec, self.spec.names, self.spec.hidden_size
        rank = s.decay_rank or -1
        return [TensorReq(n["q"], (self.qk, W)), TensorReq(n["k"], (self.qk, W)), TensorReq(n["v"], (self.vv, W)),
                TensorReq(n["gate"], (self.vv, W)), TensorReq(n["a1"], (rank, W)),
                TensorReq(n["a2"], (self.qk, rank)), TensorReq(n["a2_bias"], (self.qk,), ROLE_GAIN),
                TensorReq(n["o"], (W, self.vv)), TensorReq(n["norm"], (s.value_dim,), ROLE_GAIN)]

    def load(self, weights, rt, dtype):
        s, n = self.spec, self.spec.names
        self.rank = weights.shape_of(n["a1"])[0]
        if weights.shape_of(n["a2"])[1] != self.rank:
            raise ValueError(f"{n['a2']} has {weights.shape_of(n['a2'])[1]} columns, {n['a1']} {self.rank} rows")
        strip = getattr(weights, "wants_strip", None)
        self.w_in = weights.matrix([n["q"], n["k"], n["v"], n["gate"], n["a1"]], strip=bool(strip and strip(s.hidden_size)))
        self.w_a2 = weights.matrix([n["a2"]])
        self.w_o = weights.matrix([n["o"]], strip=bool(strip and strip(self.vv)))
        self.a_bias, self.gain = weights.vector(n["a2_bias"]), weights.vector(n["norm"])

    def state_words(self) -> int:
        return self.qk * self.spec.value_dim

    def cache_need(self):
        return StateNeed(self.state_words() * 4)

    def flops_per_token(self) -> float:
        s, W = self.spec, self.spec.hidden_size
        own = 2.0 * (W * (2 * self.qk + 2 * self.vv + self.rank) + self.rank * self.qk + self.vv * W)
        return own + 4.0 * s.num_heads * s.key_dim * s.value_dim    # k v^T and S^T q

    def forward(self, ctx, x: Tensor, cache) -> Tensor:
        s, k = self.spec, ctx.k
        T = x.shape[0]
        H, D, E = s.num_heads, s.key_dim, s.value_dim
        item = ITEMSIZE[ctx.dtype]
        ld = 2 * self.qk + 2 * self.vv + self.rank
        rows = linear(ctx, x, self.w_in, ctx.alloc((T, ld)))
        low = Tensor(rows.ptr + (2 * self.qk + 2 * self.vv) * item, (T, self.rank), ctx.dtype, rows.owner)
        z = linear(ctx, low, self.w_a2, ctx.alloc((T, self.qk), F32), lda=ld)
        out = ctx.alloc((T, self.vv))
        # read-outs before their norm, for steps in which a head's value channels spread over several blocks
        raw = ctx.alloc((T, self.vv), F32) if (E > 64 or ctx.max_q_len > 16) else None
        seg_len, seg_state, seg_decay = 0, None, None
        if raw is not None and ctx.max_q_len >= 2 * self.SEGMENT and ctx.R * H * -(-E // 16) < self.ENOUGH_BLOCKS:
            seg_len = self.SEGMENT
            segs = ctx.R * -(-int(ctx.max_q_len) // seg_len)
            seg_state = ctx.alloc((segs, self.state_words()), F32).ptr
            seg_decay = ctx.alloc((segs, self.qk), F32).ptr
        k.zk_gla(rows.ptr, ld, self.qk, 2 * self.qk, rows.ptr + (2 * self.qk + self.vv) * item, ld, z.ptr, self.qk,
                 self.a_bias.ptr, float(s.tau), self.gain.ptr, ctx.state.ptr, ctx.state.shape[1], cache.state_offset // 4,
                 ctx.q_start, ctx.slot_of_req, ctx.positions, out.ptr, raw.ptr if raw is not None else None, T, ctx.R,
                 int(ctx.max_q_len), H, D, E, float(s.eps), seg_len, seg_state, seg_decay, ctx.stream)
        return linear(ctx, out, self.w_o, ctx.alloc((T, s.hidden_size)), last_of=self)


register_part("mixer", "gated_linear_attention", GatedLinearAttention)

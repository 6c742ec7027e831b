"""A selective scan (Mamba): a recurrence with N state values per channel whose decay and input
follow from the token.

    [u | z] = W_in x;   u <- silu(conv(u) + b)                (a short causal convolution per channel)
    [dt | B | C] = W_x u;   step = softplus(W_dt dt + b_dt)    (one per channel, float)
    S[c, n] <- exp(step_c A[c, n]) S[c, n] + step_c u_c B_n,   A = -exp(A_log)
    y_c = sum_n S[c, n] C_n + D_c u_c;   out = W_o (y silu(z))

S [inner, N] starts at zero and is carried as floats in the request's state slot; the
convolution's last ``taps - 1`` inputs lie behind it.  One kernel walks the tokens of every
(request, 64 channels), so steps of single tokens and portions of prompts run the same
arithmetic in the same order.
"""
from __future__ import annotations

from typing import List

from ..config.plan import ShortConvSpec
from ..runtime.device import F32, ITEMSIZE, Tensor
from .base import ROLE_GAIN, Part, StateNeed, TensorReq, build_part, register_part
from .ops import linear


class SelectiveScan(Part):
    graph_safe = True      # rows, requests and slots are read by the kernels from device memory
    SEGMENT = 64           # tokens of a segment of a long portion
    ENOUGH_BLOCKS = 1024   # a plain walk with this many blocks fills the chip without segments

    def __init__(self, spec):
        s = self.spec = spec
        if s.state > 128 or s.state < 1:
            raise ValueError(f"1 to 128 state values a channel, got {s.state}")
        if s.inner < 1 or s.dt_rank < 1:
            raise ValueError(f"inner and dt_rank must be positive, got {s.inner} and {s.dt_rank}")
        n = s.names
        self.conv = build_part("filter", ShortConvSpec(size=s.inner, taps=s.conv_taps, weight=n["conv"], residual=False,
                                                       activation="silu", bias=n["conv_bias"]))
        self.w_in = self.w_x = self.w_dt = self.w_o = None
        self.dt_bias = self.A_log = self.D = None

    def children(self):
        return [self.conv]

    def tensor_reqs(self) -> List[TensorReq]:
        s, n, W, I = self.spec, self.spec.names, self.spec.hidden_size, self.spec.inner
        return [TensorReq(n["in"], (2 * I, W)), TensorReq(n["x"], (s.dt_rank + 2 * s.state, I)),
                TensorReq(n["dt"], (I, s.dt_rank)), TensorReq(n["dt_bias"], (I,), ROLE_GAIN),
                TensorReq(n["A_log"], (I, s.state), ROLE_GAIN), TensorReq(n["D"], (I,), ROLE_GAIN),
                TensorReq(n["o"], (W, I))]

    def load(self, weights, rt, dtype):
        s, n = self.spec, self.spec.names
        strip = getattr(weights, "wants_strip", None)
        self.w_in = weights.matrix([n["in"]], strip=bool(strip and strip(s.hidden_size)))
        self.w_x = weights.matrix([n["x"]], strip=bool(strip and strip(s.inner)))
        self.w_dt = weights.matrix([n["dt"]])
        self.w_o = weights.matrix([n["o"]], strip=bool(strip and strip(s.inner)))
        self.dt_bias, self.A_log, self.D = weights.vector(n["dt_bias"]), weights.vector(n["A_log"]), weights.vector(n["D"])

    def state_words(self) -> int:
        return self.spec.inner * self.spec.state

    def cache_need(self):
        # S of every channel, then the convolution's rows
        return StateNeed(self.state_words() * 4 + self.conv.state_bytes())

    def flops_per_token(self) -> float:
        s = self.spec
        return super().flops_per_token() + 6.0 * s.inner * s.state      # the decay, the input and the read-out

    def forward(self, ctx, x: Tensor, cache) -> Tensor:
        s, k = self.spec, ctx.k
        T, I, N, R = x.shape[0], s.inner, s.state, s.dt_rank
        item = ITEMSIZE[ctx.dtype]
        uz = linear(ctx, x, self.w_in, ctx.alloc((T, 2 * I)))
        u = self.conv.forward(ctx, uz, cache.state_offset + self.state_words() * 4, ld=2 * I)
        ldp = R + 2 * N
        p = linear(ctx, u, self.w_x, ctx.alloc((T, ldp)))
        dt = linear(ctx, Tensor(p.ptr, (T, R), ctx.dtype, p.owner), self.w_dt, ctx.alloc((T, I), F32), lda=ldp)
        out = ctx.alloc((T, I))
        # few long portions: segments of a portion walked side by side (see the kernel's file)
        seg_len, seg_state, seg_steps = 0, None, None
        if ctx.max_q_len >= 2 * self.SEGMENT and ctx.R * -(-I // 64) < self.ENOUGH_BLOCKS:
            seg_len = self.SEGMENT
            segs = ctx.R * -(-int(ctx.max_q_len) // seg_len)
            seg_state = ctx.alloc((segs, self.state_words()), F32).ptr
            seg_steps = ctx.alloc((segs, I), F32).ptr
        k.zk_selective_scan(u.ptr, I, dt.ptr, I, self.dt_bias.ptr, p.ptr, ldp, R, R + N, self.A_log.ptr, self.D.ptr,
                            uz.ptr + I * item, 2 * I, ctx.state.ptr, ctx.state.shape[1], cache.state_offset // 4,
                            ctx.q_start, ctx.slot_of_req, out.ptr, T, ctx.R, I, N, int(ctx.max_q_len), seg_len,
                            seg_state, seg_steps, ctx.stream)
        return linear(ctx, out, self.w_o, ctx.alloc((T, s.hidden_size)), last_of=self)


register_part("mixer", "selective_scan", SelectiveScan)

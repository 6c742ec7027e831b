"""A short causal convolution over time on each channel, added to its input:
out_t = x_t + sum_j w[:, j] x_(t - taps + 1 + j), rows before a sequence's start being zero
(``residual`` False: the sum alone; ``activation`` "silu": silu of the result; ``bias``: a
number per channel that the sum starts from).
The ``taps - 1`` rows before a request's next token are its state (float, in its state slot,
which starts as zeros): a step reads them for its first tokens and renews them afterwards.
"""
from __future__ import annotations

from typing import List

from ..runtime.device import Tensor
from .base import ROLE_GAIN, Part, TensorReq, register_part


class ShortConv(Part):
    graph_safe = True      # rows, requests and slots are read by the kernels from device memory

    def __init__(self, spec):
        if spec.taps < 1:
            raise ValueError(f"a convolution has at least one tap, got {spec.taps}")
        if getattr(spec, "activation", None) not in (None, "silu"):
            raise ValueError(f"a convolution's activation is None or 'silu', got {spec.activation!r}")
        self.spec = spec
        self.weight = self.bias = None
        self.bias_name = getattr(spec, "bias", None)
        self.names = [spec.weight] if isinstance(spec.weight, str) else list(spec.weight)

    def tensor_reqs(self) -> List[TensorReq]:
        s = self.spec
        extra = [TensorReq(self.bias_name, (s.size,), ROLE_GAIN)] if self.bias_name else []
        if len(self.names) == 1:
            return [TensorReq(self.names[0], (s.size, s.taps), ROLE_GAIN)] + extra
        sizes = getattr(s, "channel_counts", None)
        if sizes is None or len(sizes) != len(self.names) or sum(sizes) != s.size:
            raise ValueError("a convolution over several tensors says how many channels each has (channel_counts)")
        return [TensorReq(n, (c, s.taps), ROLE_GAIN) for n, c in zip(self.names, sizes)] + extra

    def load(self, weights, rt, dtype):
        self.weight = weights.vectors(self.names)
        self.bias = weights.vector(self.bias_name) if self.bias_name else None

    def state_bytes(self) -> int:
        return (self.spec.taps - 1) * self.spec.size * 4

    def flops_per_token(self) -> float:
        return 2.0 * self.spec.size * self.spec.taps

    def forward(self, ctx, x: Tensor, state_offset: int, ld: int = 0) -> Tensor:
        """``x``: [T, size], or the first ``size`` channels of rows ``ld`` apart."""
        s, k = self.spec, ctx.k
        T = x.shape[0]
        ld = int(ld) or s.size
        out = ctx.alloc((T, s.size))
        state = ctx.state.ptr if ctx.state is not None else None
        words = ctx.state.shape[1] if ctx.state is not None else 0
        residual = 1 if getattr(s, "residual", True) else 0
        act = 1 if getattr(s, "activation", None) == "silu" else 0
        bias = self.bias.ptr if self.bias is not None else None
        if ctx.max_q_len == 1 and T == ctx.R:
            # every request brings one token: one launch computes and moves the state on
            k.zk_short_conv_token_bias(x.ptr, ld, self.weight.ptr, state, words, state_offset // 4, ctx.positions,
                                       ctx.req_of_token, ctx.q_start, ctx.slot_of_req, out.ptr, s.size, T, s.size, s.taps,
                                       residual, act, bias, ctx.stream)
            return out
        k.zk_short_conv_bias(x.ptr, ld, self.weight.ptr, state, words, state_offset // 4, ctx.positions, ctx.req_of_token,
                             ctx.q_start, ctx.slot_of_req, out.ptr, s.size, T, s.size, s.taps, residual, act, bias,
                             ctx.stream)
        k.zk_short_conv_state_ext(x.ptr, ld, state, words, state_offset // 4, ctx.q_start, ctx.slot_of_req, ctx.R, s.size,
                                  s.taps, ctx.stream)
        return out


register_part("filter", "short_conv", ShortConv)

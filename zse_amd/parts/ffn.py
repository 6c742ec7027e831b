"""Gated feed-forward: act(x Wg^T) * (x Wu^T), then Wd^T.

act is one of gelu_tanh, silu and relu (max(z, 0)).
gelu_tanh(z) = 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))) is the
reference's GeGLU kernel (orchestrator/kernels.py:1678-1697, wiring
model_runner.py:518-530); silu is its Llama activation (kernels.py:228-244).
Gate and up are two products there (model_runner.py:1270-1275), one here.
"""
from __future__ import annotations

from typing import List

from ..runtime.device import BF16, F32, I32, Tensor
from .base import Part, TensorReq, build_part, register_part
from .ops import linear, tuned_gemm

ACTIVATION_CODES = {"gelu_tanh": 0, "silu": 1, "relu": 2}
CLAMPED = "clamped_swiglu"     # g = min(gate, limit), u = clamp(up, +-limit): g sigmoid(1.702 g) (u + 1)


class GatedMLP(Part):
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        if spec.activation not in ACTIVATION_CODES and spec.activation != CLAMPED:
            raise ValueError(f"activation must be one of {sorted(ACTIVATION_CODES) + [CLAMPED]}, got {spec.activation!r}")
        if spec.activation == CLAMPED and not (getattr(spec, "limit", None) or 0) > 0:
            raise ValueError(f"{CLAMPED} needs a positive limit, got {getattr(spec, 'limit', None)!r}")
        self.spec = spec
        self.w_gu = self.w_down = None

    def tensor_reqs(self) -> List[TensorReq]:
        s = self.spec
        return [TensorReq(s.names["gate"], (s.intermediate_size, s.hidden_size)),
                TensorReq(s.names["up"], (s.intermediate_size, s.hidden_size)),
                TensorReq(s.names["down"], (s.hidden_size, s.intermediate_size))]

    def load(self, weights, rt, dtype):
        s = self.spec
        strip = getattr(weights, "wants_strip", None)
        gu = [s.names["gate"], s.names["up"]]
        self.w_gu = (weights.matrix(gu, strip=True) if strip and strip(s.hidden_size, s.intermediate_size)
                     else weights.matrix(gu))
        self.w_down = (weights.matrix([s.names["down"]], strip=True) if strip and strip(s.intermediate_size)
                       else weights.matrix([s.names["down"]]))

    def forward(self, ctx, x: Tensor, out: Tensor = None) -> Tensor:
        """``out``: where the result goes (activations or float32 [T, hidden]); the product that
        ends the layer then never hands partial sums back."""
        s = self.spec
        T, I = x.shape[0], s.intermediate_size
        last = None if out is not None else self
        if s.activation == CLAMPED and tuned_gemm(ctx, s.hidden_size):
            # the activation in the product's epilogue, on the float sums
            a = linear(ctx, x, self.w_gu, ctx.alloc((T, I)), epilogue=CLAMPED, cap=float(s.limit))
            return linear(ctx, a, self.w_down, out if out is not None else ctx.alloc((T, s.hidden_size)), last_of=last)
        if s.activation == CLAMPED:
            gu = linear(ctx, x, self.w_gu, ctx.alloc((T, 2 * I)))
            a = ctx.alloc((T, I))
            ctx.k.zk_clamped_glu(gu.ptr, a.ptr, T, I, float(s.limit), ctx.stream)
            return linear(ctx, a, self.w_down, out if out is not None else ctx.alloc((T, s.hidden_size)), last_of=last)
        if tuned_gemm(ctx, s.hidden_size):
            a = linear(ctx, x, self.w_gu, ctx.alloc((T, I)), epilogue=s.activation)
            return linear(ctx, a, self.w_down, out if out is not None else ctx.alloc((T, s.hidden_size)), last_of=last)
        gu = linear(ctx, x, self.w_gu, ctx.alloc((T, 2 * I)))
        a = ctx.alloc((T, I))
        ctx.k.zk_gated_act(gu.ptr, a.ptr, T, I, ACTIVATION_CODES[s.activation], ctx.stream)
        return linear(ctx, a, self.w_down, out if out is not None else ctx.alloc((T, s.hidden_size)), last_of=last)


UNARY_CODES = {"relu2": 0}     # max(z, 0)^2


class MLP(Part):
    """act(x Wu^T) Wd^T without a gate; the activation rides in the first product's epilogue where
    the matrix-core product serves the step."""
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        if spec.activation not in UNARY_CODES:
            raise ValueError(f"activation must be one of {sorted(UNARY_CODES)}, got {spec.activation!r}")
        self.spec = spec
        self.w_up = self.w_down = None

    def tensor_reqs(self) -> List[TensorReq]:
        s = self.spec
        return [TensorReq(s.names["up"], (s.intermediate_size, s.hidden_size)),
                TensorReq(s.names["down"], (s.hidden_size, s.intermediate_size))]

    def load(self, weights, rt, dtype):
        s = self.spec
        strip = getattr(weights, "wants_strip", None)
        self.w_up = weights.matrix([s.names["up"]], strip=bool(strip and strip(s.hidden_size)))
        self.w_down = weights.matrix([s.names["down"]], strip=bool(strip and strip(s.intermediate_size)))

    def forward(self, ctx, x: Tensor) -> Tensor:
        s = self.spec
        T, I = x.shape[0], s.intermediate_size
        if tuned_gemm(ctx, s.hidden_size) and x.ptr % 16 == 0:
            a = linear(ctx, x, self.w_up, ctx.alloc((T, I)), epilogue=s.activation)
        else:
            up = linear(ctx, x, self.w_up, ctx.alloc((T, I)))
            a = ctx.alloc((T, I))
            ctx.k.zk_unary_act(up.ptr, a.ptr, T * I, UNARY_CODES[s.activation], ctx.stream)
        return linear(ctx, a, self.w_down, ctx.alloc((T, s.hidden_size)), last_of=self)


class RoutedMLP(Part):
    """A mixture of small gated layers: scores from a float router product (sigmoids, or a softmax
    over all experts), the ``top_k`` largest chosen on the device (the lower index among equals),
    the chosen scores as weights on the experts' inputs or on their outputs, the experts' results
    added in the order they were chosen, a shared layer on top (optionally times the sigmoid of a
    number a token, whose row rides below the router's in one product).  Steps of few tokens read each chosen expert's rows once per (token, choice); steps of
    many tokens sort the pairs by expert on the device and run a grouped matrix-core product.
    Nothing comes back to the host, so steps are captured and written down like any other."""
    graph_safe = True
    GROUPED_FROM = 64          # (token, choice) pairs from which the grouped product is used (bfloat16)
    # experts of 2M weights a matrix and more: from 16 pairs on (two tokens an expert re-read its rows
    # row by row; measured at 8 requests, 2 of 8 experts: 1.26 -> 1.20 ms a step at 2048 x 2048,
    # 1.51 -> 1.14 ms at 4096 x 3584, but 0.72 -> 0.76 ms at 1024 x 1024)
    GROUPED_WIDE_FROM, WIDE = 16, 2 << 20

    def __init__(self, spec):
        s = self.spec = spec
        if s.activation not in (CLAMPED, "silu"):
            raise ValueError(f"routed experts are {CLAMPED} or silu layers, got {s.activation!r}")
        if not (1 <= s.top_k <= min(s.num_experts, 16)) or s.num_experts > 1024:
            raise ValueError(f"1 to 16 of up to 1024 experts a token, got {s.top_k} of {s.num_experts}")
        if s.activation == CLAMPED and not (s.limit or 0) > 0:
            raise ValueError(f"{CLAMPED} needs a positive limit, got {s.limit!r}")
        self.scoring = getattr(s, "scoring", "sigmoid")
        if self.scoring not in ("sigmoid", "softmax"):
            raise ValueError(f"scores are sigmoid or softmax, got {self.scoring!r}")
        self.shared = build_part("ffn", s.shared) if s.shared is not None else None
        self.shared_gate = getattr(s, "shared_gate", None)
        if self.shared_gate and self.shared is None:
            raise ValueError("a gate on the shared layer needs a shared layer")
        self.w_router = self.w_gu = self.w_down = None

    def children(self):
        return [self.shared] if self.shared is not None else []

    def _name(self, e: int, role: str) -> str:
        return self.spec.expert_names.format(e=e, role=role)

    def tensor_reqs(self) -> List[TensorReq]:
        s = self.spec
        out = [TensorReq(s.router, (s.num_experts, s.hidden_size))]
        if self.shared_gate:
            out.append(TensorReq(self.shared_gate, (1, s.hidden_size)))
        for e in range(s.num_experts):
            out += [TensorReq(self._name(e, "gate"), (s.intermediate_size, s.hidden_size)),
                    TensorReq(self._name(e, "up"), (s.intermediate_size, s.hidden_size)),
                    TensorReq(self._name(e, "down"), (s.hidden_size, s.intermediate_size))]
        return out

    def load(self, weights, rt, dtype):
        s = self.spec
        self.w_router = weights.matrix([s.router] + ([self.shared_gate] if self.shared_gate else []))
        # expert e: rows [e 2F, e 2F + F) its gate, the next F its up; down: rows [e W, (e + 1) W)
        self.w_gu = weights.matrix([self._name(e, r) for e in range(s.num_experts) for r in ("gate", "up")])
        self.w_down = weights.matrix([self._name(e, "down") for e in range(s.num_experts)])

    def flops_per_token(self) -> float:
        s = self.spec
        return 2.0 * s.num_experts * s.hidden_size + s.top_k * 6.0 * s.intermediate_size * s.hidden_size

    def forward(self, ctx, x: Tensor) -> Tensor:
        s, k = self.spec, ctx.k
        T, W, F, E, top = x.shape[0], s.hidden_size, s.intermediate_size, s.num_experts, s.top_k
        ld = E + (1 if self.shared_gate else 0)
        logits = linear(ctx, x, self.w_router, ctx.alloc((T, ld), F32))
        ids, wts = ctx.alloc((T, top), I32), ctx.alloc((T, top), F32)
        k.zk_moe_route_ext(logits.ptr, ld, ids.ptr, wts.ptr, T, E, top, 1 if self.scoring == "softmax" else 0, ctx.stream)
        act, on_out, limit = (1 if s.activation == "silu" else 0), (0 if s.scale_input else 1), float(s.limit or 0.0)
        P = 2 if self.shared is not None else 1
        planes = ctx.alloc((P, T, W), F32)
        y = ctx.alloc((T * top, F))
        enough = T * top >= (self.GROUPED_WIDE_FROM if W * F >= self.WIDE else self.GROUPED_FROM)
        grouped = (ctx.dtype == BF16 and ctx.tuned and enough and W % 8 == 0 and F % 8 == 0
                   and k.has("zk_moe_experts_grouped_ext"))
        if grouped:
            work = ctx.alloc((E + 1 + 2 * T * top,), I32)
            xg, rows = ctx.alloc((T * top, W)), ctx.alloc((T * top, W), F32)
            k.zk_moe_experts_grouped_ext(x.ptr, ids.ptr, wts.ptr, self.w_gu.ptr, self.w_down.ptr, work.ptr, xg.ptr, y.ptr,
                                         rows.ptr, planes.ptr, T, E, top, W, F, limit, act, on_out, ctx.stream)
        else:
            k.zk_moe_experts_ext(x.ptr, ids.ptr, wts.ptr, self.w_gu.ptr, self.w_down.ptr, y.ptr, planes.ptr, T, top, W, F,
                                 limit, act, on_out, ctx.stream)
        if self.shared is not None:
            second = planes.rows(1, 2).view(T, W)
            self.shared.forward(ctx, x, out=second)
            if self.shared_gate:
                k.zk_gate_rows(second.ptr, logits.ptr + E * 4, ld, T, W, ctx.stream)
        if getattr(ctx, "sums_welcome", None) is self:
            # the block's joining kernel adds the planes up itself
            return Tensor(planes.ptr, (P, T, W), F32, planes.owner, layout="parts")
        out = ctx.alloc((T, W))
        k.zk_planes_sum(planes.ptr, P, out.ptr, T, W, ctx.stream)
        return out


register_part("ffn", "gated_mlp", GatedMLP)
register_part("ffn", "mlp", MLP)
register_part("ffn", "routed_mlp", RoutedMLP)

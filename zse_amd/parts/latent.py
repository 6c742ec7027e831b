"""Softmax attention whose keys and values are made from one cached latent row per token.

    c_t = rms_norm(first C rows of W_down x_t) * gain;   r_t = rot_t(last R rows of W_down x_t)
    head h:  key_j = [W_uk,h c_j, r_j],  value_j = W_uv,h c_j,  query = [q_plain, rot_t(q_rot)]
    weights  p_j = exp(s_j) / (sum_i exp(s_i) + exp(sink_h)),   s_j = (query . key_j) * scale

Only [c_t, r_t] is cached: one key head of C + R channels a token, and no values.  Since
q_plain . (W_uk,h c) = (W_uk,h^T q_plain) . c and sum_j p_j W_uv,h c_j = W_uv,h sum_j p_j c_j, a query
head is carried over to [W_uk,h^T q_plain, q_rot], attends to the cached rows as keys and to their
first C channels as values, and its result goes through W_uv,h; the two small per-head products
run before and after the attention kernel.  One path for whole prompts, portions and decoded
tokens, reading the cache alone.

Options of the spec: queries through a latent of their own (c_q = rms_norm(W_q_down x) * gain,
q = W_q c_q), a window over the keys, and a gate of one number a head, sigmoid(W_gate x)_h, on the
heads' outputs (its rows ride behind the down-projection's in one product).
"""
from __future__ import annotations

from typing import List

from ..runtime.device import BF16, ITEMSIZE, Tensor
from .base import ROLE_GAIN, PagedKV, Part, TensorReq, build_part, register_part
from .ops import linear


class LatentAttention(Part):
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        s = self.spec = spec
        if s.rotary_dim % 2:
            raise ValueError(f"the rotated part must be even, got {s.rotary_dim}")
        if s.latent_dim + s.rotary_dim > 1024:
            raise ValueError(f"latent and rotated part together up to 1024 channels, got {s.latent_dim + s.rotary_dim}")
        self.position = build_part("position", s.position)
        if self.position.rotary_tables is None or getattr(s.position, "rotary_dim", None) != s.rotary_dim:
            raise ValueError("a latent attention's rotated part needs a rotary encoding over all of its channels")
        self.w_in = self.w_uk = self.w_uv = self.w_o = None
        self.gain = self.sinks = None
        self.q_rank = int(getattr(s, "query_latent_dim", None) or 0)
        self.gate_name = s.names.get("gate")
        if self.q_rank and not (s.names.get("q_down") and s.names.get("q_down_norm")):
            raise ValueError("queries through a latent need the tensors q_down and q_down_norm")
        self.w_q_down = self.w_q = self.q_gain = None

    def children(self):
        return [self.position]

    def tensor_reqs(self) -> List[TensorReq]:
        s, n = self.spec, self.spec.names
        H, D, R, E, C, W = s.num_heads, s.head_dim, s.rotary_dim, s.value_dim, s.latent_dim, s.hidden_size
        out = [TensorReq(n["q"], (H * (D + R), self.q_rank or W)), TensorReq(n["down"], (C + R, W)),
               TensorReq(n["down_norm"], (C,), ROLE_GAIN), TensorReq(n["up_k"], (H * D, C)),
               TensorReq(n["up_v"], (H * E, C)), TensorReq(n["o"], (W, H * E))]
        if n.get("sinks"):
            out.append(TensorReq(n["sinks"], (H,), ROLE_GAIN))
        if self.q_rank:
            out += [TensorReq(n["q_down"], (self.q_rank, W)), TensorReq(n["q_down_norm"], (self.q_rank,), ROLE_GAIN)]
        if self.gate_name:
            out.append(TensorReq(self.gate_name, (H, W)))
        return out

    def load(self, weights, rt, dtype):
        s, n = self.spec, self.spec.names
        strip = getattr(weights, "wants_strip", None)
        tail = [n["down"]] + ([self.gate_name] if self.gate_name else [])
        if self.q_rank:
            # the query's own latent is a product, a norm and a second product; the down-projection
            # (and the gate) is a product of its own
            self.w_q_down = weights.matrix([n["q_down"]], strip=bool(strip and strip(s.hidden_size)))
            self.w_q = weights.matrix([n["q"]], strip=bool(strip and strip(self.q_rank)))
            self.q_gain = weights.vector(n["q_down_norm"])
            self.w_in = weights.matrix(tail, strip=bool(strip and strip(s.hidden_size)))
        else:
            self.w_in = weights.matrix([n["q"]] + tail, strip=bool(strip and strip(s.hidden_size)))
        self.w_uk, self.w_uv = weights.matrix([n["up_k"]]), weights.matrix([n["up_v"]])      # row-major: read per head
        self.w_o = weights.matrix([n["o"]], strip=bool(strip and strip(s.num_heads * s.value_dim)))
        self.gain = weights.vector(n["down_norm"])
        self.sinks = weights.vector(n["sinks"]) if n.get("sinks") else None

    def cache_need(self):
        s = self.spec
        return PagedKV(1, s.latent_dim + s.rotary_dim, s.window, value_dim=s.latent_dim, values_in_keys=True)

    def flops_per_token(self) -> float:
        return super().flops_per_token()     # the per-head products are the matrices up_k and up_v, once a token

    SPLIT_ROWS, SPLITS = 32, 32              # tokens and ranges of keys that the workspace is sized for

    def _fast(self, kernels, dtype: str, page_size: int) -> bool:
        """Whether the matrix-core attention kernel serves this layer."""
        s = self.spec
        return bool(dtype == BF16 and kernels.has("zk_latent_attention_bf16_window") and
                    kernels.zk_latent_attention_bf16_supports(s.latent_dim + s.rotary_dim, s.latent_dim, page_size))

    def prepare(self, kernels, dtype, max_seqs, max_model_len, page_size, max_batch_tokens=0) -> int:
        """Workspace that lets steps of few rows behind long contexts cut their keys into ranges."""
        if not self._fast(kernels, dtype, page_size):
            return 0
        s = self.spec
        return int(kernels.zk_latent_attention_bf16_workspace(max(int(max_seqs), self.SPLIT_ROWS), s.num_heads,
                                                               s.latent_dim, self.SPLITS))

    def flops_per_key(self) -> float:
        s = self.spec
        return 2.0 * s.num_heads * (2 * s.latent_dim + s.rotary_dim)

    def forward(self, ctx, x: Tensor, cache) -> Tensor:
        s, k = self.spec, ctx.k
        T = x.shape[0]
        H, D, R, E, C = s.num_heads, s.head_dim, s.rotary_dim, s.value_dim, s.latent_dim
        g = ctx.group(cache.group)
        item = ITEMSIZE[ctx.dtype]
        n_gate = H if self.gate_name else 0
        if self.q_rank:
            cq = linear(ctx, x, self.w_q_down, ctx.alloc((T, self.q_rank)))
            cn = ctx.alloc((T, self.q_rank))
            k.zk_rmsnorm(cq.ptr, 0, None, self.q_gain.ptr, cn.ptr, float(s.eps), 0, T, self.q_rank, ctx.stream)
            qd = linear(ctx, cn, self.w_q, ctx.alloc((T, H * (D + R))))
            ld = H * (D + R)
            ldd = C + R + n_gate
            down = linear(ctx, x, self.w_in, ctx.alloc((T, ldd)))
            down_ptr = down.ptr
        else:
            ld = ldd = H * (D + R) + C + R + n_gate
            qd = linear(ctx, x, self.w_in, ctx.alloc((T, ld)))
            down_ptr = qd.ptr + H * (D + R) * item
        qa = ctx.alloc((T, H * (C + R)))
        tables = self.position.rotary_tables()
        mag = float(self.position.magnitude()) if hasattr(self.position, "magnitude") else 1.0
        inter = 1 if getattr(self.position, "interleaved", False) else 0
        k.zk_latent_prep_ext(qd.ptr, ld, down_ptr, ldd, ctx.positions, g.slot_map, self.gain.ptr, float(s.eps),
                             tables[0].ptr, mag, inter, qa.ptr, cache.k.ptr, T, H, D, R, C, g.page_size, ctx.stream)
        # the plain part of every query head, carried over to the latent's channels
        k.zk_heads_linear(qd.ptr, ld, D + R, self.w_uk.ptr, 1, qa.ptr, H * (C + R), C + R, T, H, D, C, ctx.stream)
        o = ctx.alloc((T, H * C))
        sinks = self.sinks.ptr if self.sinks is not None else None
        if ctx.tuned and self._fast(k, ctx.dtype, g.page_size):
            k.zk_latent_attention_bf16_window(qa.ptr, cache.k.ptr, g.block_table, g.max_blocks, ctx.q_start, ctx.ctx_len,
                                              ctx.positions, sinks, o.ptr, ctx.workspace.ptr, ctx.workspace.nbytes, T, ctx.R,
                                              max(int(ctx.max_q_len), 1), int(ctx.max_ctx), H, C + R, C, g.page_size,
                                              float(s.scale), int(s.window) if s.window else 0,
                                              1 if getattr(s, "wide_weights", False) else 0, ctx.stream)
        else:
            k.zk_attention_plain_sink(qa.ptr, H * (C + R), cache.k.ptr, cache.k.ptr, g.block_table, g.max_blocks,
                                      ctx.req_of_token, ctx.positions, o.ptr, T, H, 1, C + R, C, g.page_size,
                                      float(s.scale), 0.0, int(s.window) if s.window else 0, 0, None, 0, sinks, 1, ctx.stream)
        v = ctx.alloc((T, H * E))
        k.zk_heads_linear(o.ptr, H * C, C, self.w_uv.ptr, 0, v.ptr, H * E, E, T, H, C, E, ctx.stream)
        if self.gate_name:
            # a head's output times the sigmoid of its gate column, which lies behind the down-projection's
            k.zk_gate_heads_per(v.ptr, down_ptr + (C + R) * item, ldd, T, H * E, E, ctx.stream)
        return linear(ctx, v, self.w_o, ctx.alloc((T, s.hidden_size)), last_of=self)


register_part("mixer", "latent_attention", LatentAttention)

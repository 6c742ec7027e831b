"""Grouped-query softmax attention over the paged cache.

One forward for every kind of step: project q, k, v in one product, rotate q
and k and store k, v at each token's place in the cache, then let every token
attend to the cache alone, over the positions [max(0, pos - window + 1), pos]
(all earlier positions without a window).  The reference writes the cache
first as well (orchestrator/model_runner.py:1184-1194) but its prefill reads
contiguous K/V and never masks a window (orchestrator/kernels.py:883,
model_runner.py:489-490); its scale is fixed at 1/sqrt(head_dim)
(model_runner.py:80) where this part takes the scale and the soft cap as
parameters.  q, k, v stay separate products in the reference
(model_runner.py:1151-1165); here they are one.
"""
from __future__ import annotations

from typing import List

import numpy as np

from ..runtime.device import BF16, ITEMSIZE, Tensor
from .base import ROLE_GAIN, PagedKV, Part, TensorReq, build_part, register_part
from .ops import linear, tuned_gemm


class PagedAttention(Part):
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        s = self.spec = spec
        if s.num_heads % s.num_kv_heads:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if s.head_dim > 256 or s.head_dim < 1:
            raise ValueError(f"head_dim must lie in 1..256, got {s.head_dim}")
        self.position = build_part("position", s.position)
        self.shared_kv = "k" not in s.names        # reads another call's cache, writes none
        self.w_qkv = self.w_o = None
        # optional steps between the product and the attention (see AttentionSpec): any of them
        # sends the mixer down the general path, whose kernels take them all as parameters
        self.value_dim = int(getattr(s, "value_dim", None) or s.head_dim)
        self.q_norm_name, self.k_norm_name = getattr(s, "q_norm", None), getattr(s, "k_norm", None)
        self.head_scale_name = getattr(s, "head_scale", None)
        self.value_base = getattr(s, "value_rotation", None)
        self.bias_names = dict(getattr(s, "biases", None) or {})
        self.rot_scale = float(self.position.magnitude()) if hasattr(self.position, "magnitude") else 1.0
        self.rot_interleaved = bool(getattr(self.position, "interleaved", False))
        self.chunk = int(getattr(s, "chunk", None) or 0)
        self.unit_sink = bool(getattr(s, "unit_sink", False))
        self.unit_norm = bool(getattr(s, "qk_unit_norm", False))
        self.gate_name = getattr(s, "gate", None)
        self.wide_weights = bool(getattr(s, "wide_weights", False))
        # a norm over a token's whole query row and whole key row, and values that are the keys as
        # projected: one kernel of their own between the product and the attention
        self.q_row_norm_name, self.k_row_norm_name = getattr(s, "q_row_norm", None), getattr(s, "k_row_norm", None)
        self.values_are_keys = bool(getattr(s, "values_are_keys", False))
        self.by_rows = bool(self.q_row_norm_name or self.k_row_norm_name or self.values_are_keys)
        if self.chunk and s.window:
            raise ValueError("an attention has a window or a chunk, not both")
        if self.chunk < 0:
            raise ValueError(f"chunk must be positive, got {self.chunk}")
        self.general = bool(self.value_dim != s.head_dim or self.q_norm_name or self.k_norm_name or
                            self.head_scale_name or self.value_base or self.bias_names or
                            self.rot_scale != 1.0 or self.rot_interleaved or self.chunk or self.unit_sink or self.wide_weights or
                            self.unit_norm or self.gate_name or self.by_rows)
        if self.by_rows:
            if (self.q_norm_name or self.k_norm_name or self.head_scale_name or self.value_base or self.unit_norm
                    or self.rot_scale != 1.0 or self.rot_interleaved or self.shared_kv):
                raise ValueError("an attention with norms over whole rows, or whose values are its keys, takes biases, "
                                 "a rotation of pairs (i, i + dims/2), a window or chunk, a sink and a gate, nothing else")
            if self.values_are_keys and self.value_dim != s.head_dim:
                raise ValueError(f"values that are keys have the keys' size: value_dim {self.value_dim}, head_dim {s.head_dim}")
            if self.values_are_keys and ("v" in s.names or "v" in self.bias_names):
                raise ValueError("values that are keys have no projection and no bias of their own")
        self.in_bias = self.o_bias = None
        if self.value_dim > 256:
            raise ValueError(f"value_dim up to 256, got {self.value_dim}")
        if self.value_base and self.value_dim % 2:
            raise ValueError(f"rotated values need an even value_dim, got {self.value_dim}")
        self.q_gain = self.k_gain = self.head_scale = self.value_freq = None
        self.q_row_gain = self.k_row_gain = None
        self.decode_chunk = 64                     # keys a wave of the split decode attention takes

    def children(self):
        return [self.position]

    def tensor_reqs(self) -> List[TensorReq]:
        s = self.spec
        out = [TensorReq(s.names["q"], (s.num_heads * s.head_dim, s.hidden_size)),
               TensorReq(s.names["o"], (s.hidden_size, s.num_heads * self.value_dim))]
        if self.q_norm_name:
            out.append(TensorReq(self.q_norm_name, (s.head_dim,), ROLE_GAIN))
        if self.head_scale_name:
            out.append(TensorReq(self.head_scale_name, (s.num_heads,), ROLE_GAIN))
        if self.gate_name:
            out.append(TensorReq(self.gate_name, (s.num_heads * self.value_dim, s.hidden_size)))
        for role, rows in (("q", s.num_heads * s.head_dim), ("o", s.hidden_size)):
            if role in self.bias_names:
                out.append(TensorReq(self.bias_names[role], (rows,), ROLE_GAIN))
        if self.q_row_norm_name:
            out.append(TensorReq(self.q_row_norm_name, (s.num_heads * s.head_dim,), ROLE_GAIN))
        if self.shared_kv:
            return out
        for role, rows in (("k", s.num_kv_heads * s.head_dim), ("v", s.num_kv_heads * self.value_dim)):
            if role in self.bias_names:
                out.append(TensorReq(self.bias_names[role], (rows,), ROLE_GAIN))
        out.append(TensorReq(s.names["k"], (s.num_kv_heads * s.head_dim, s.hidden_size)))
        if not self.values_are_keys:
            out.append(TensorReq(s.names["v"], (s.num_kv_heads * self.value_dim, s.hidden_size)))
        if self.k_row_norm_name:
            out.append(TensorReq(self.k_row_norm_name, (s.num_kv_heads * s.head_dim,), ROLE_GAIN))
        if self.k_norm_name:
            out.append(TensorReq(self.k_norm_name, (s.head_dim,), ROLE_GAIN))
        return out

    def load(self, weights, rt, dtype):
        s = self.spec
        stored = ("q", "k") if self.values_are_keys else ("q", "k", "v")
        names = [s.names["q"]] if self.shared_kv else [s.names[r] for r in stored]
        if self.gate_name:
            names.append(self.gate_name)       # the gate's rows behind q, k, v: one product
        strip = getattr(weights, "wants_strip", None)
        self.w_qkv = weights.matrix(names, strip=True) if strip and strip(s.hidden_size) else weights.matrix(names)
        o_cols = s.num_heads * self.value_dim
        self.w_o = (weights.matrix([s.names["o"]], strip=True) if strip and strip(o_cols)
                    else weights.matrix([s.names["o"]]))
        if self.q_norm_name:
            self.q_gain = weights.vector(self.q_norm_name)
        if self.k_norm_name and not self.shared_kv:
            self.k_gain = weights.vector(self.k_norm_name)
        if self.head_scale_name:
            self.head_scale = weights.vector(self.head_scale_name)
        if self.q_row_norm_name:
            self.q_row_gain = weights.vector(self.q_row_norm_name)
        if self.k_row_norm_name:
            self.k_row_gain = weights.vector(self.k_row_norm_name)
        roles = ("q",) if self.shared_kv else stored
        if any(r in self.bias_names for r in roles):
            if not all(r in self.bias_names for r in roles):
                raise ValueError("biases on the projections: all of q, k, v or none")
            self.in_bias = weights.vectors([self.bias_names[r] for r in roles])
        if "o" in self.bias_names:
            self.o_bias = weights.vector(self.bias_names["o"])
        if self.value_base:
            m = np.arange(self.value_dim // 2, dtype=np.float64)
            self.value_freq = rt.upload(np.power(float(self.value_base), -2.0 * m / self.value_dim).astype(np.float32))

    def cache_need(self):
        s = self.spec
        return PagedKV(s.num_kv_heads, s.head_dim, s.window,
                       self.value_dim if self.value_dim != s.head_dim else None, chunk=self.chunk or None)

    def flops_per_key(self) -> float:
        return 2.0 * self.spec.num_heads * (self.spec.head_dim + self.value_dim)        # q.k and p.v

    PORTION_RANGES_BYTES = 192 << 20

    def wants_v_transposed(self, kernels, dtype: str, page_size: int) -> bool:
        """The matrix-core kernel reads V as [page][kv head][hd][bs]."""
        s = self.spec
        if (self.chunk or self.unit_sink or self.wide_weights) and not kernels.has("zk_attention_bf16_masked"):
            return False
        return bool(dtype == BF16 and self.value_dim == s.head_dim and kernels.has("zk_attention_bf16") and
                    kernels.zk_attention_bf16_supports(s.num_heads, s.num_kv_heads, s.head_dim, page_size))

    def prepare(self, kernels, dtype, max_seqs, max_model_len, page_size, max_batch_tokens=0) -> int:
        """Workspace of the split attention of decoded tokens at the runner's limits, and the
        number of keys a wave of it takes.  That number fixes where the sums over keys are cut:
        it follows from the limits alone, never from a step's batch, so a request's result does
        not depend on who shares its step."""
        s = self.spec
        if not self.wants_v_transposed(kernels, dtype, page_size):
            return 0
        chunks = -(-int(max_model_len) // 64)
        self.decode_chunk = 32 if int(max_seqs) * s.num_kv_heads * chunks <= 512 else 64
        longest = int(kernels.zk_attention_bf16_max_context(s.num_heads, s.num_kv_heads, s.head_dim,
                                                            self.decode_chunk))
        if max_model_len > longest:
            raise ValueError(f"attention with {s.num_heads} heads, {s.num_kv_heads} KV heads of "
                             f"{s.head_dim}: the longest context its decode kernel takes is {longest} "
                             f"tokens, the runner asks for {max_model_len}")
        need = int(kernels.zk_attention_bf16_workspace(int(max_seqs), s.num_heads, s.head_dim, int(max_model_len)))
        # room for a launch of few, long portions to cut its keys into ranges: as much as a step's
        # tokens can ask for, but no more than PORTION_RANGES_BYTES (a launch that would need more
        # has blocks enough without the ranges, or runs on the kernels that need no workspace)
        if max_batch_tokens > 0 and kernels.has("zk_attention_bf16_portion_workspace"):
            extra = int(kernels.zk_attention_bf16_portion_workspace(int(max_batch_tokens), s.num_heads, s.num_kv_heads,
                                                                    s.head_dim))
            need = (need + 255) // 256 * 256 + min(extra, self.PORTION_RANGES_BYTES)
        return need

    def between_product_and_rotation(self, ctx, qkv: Tensor) -> None:
        """A mixer that differs from this one only in what it does to queries and keys before
        they are rotated and stored (a norm over each head, say) overrides this and changes
        ``qkv`` in place: rows are tokens, a row holds the query heads, then the key heads, then
        the value heads (the last two absent in a mixer that reads another entry's cache), each
        ``head_dim`` wide.  Everything else of the mixer stays as it is; the product that
        rotates and stores its own results is then not used, since this step lies in between."""

    def _forward_general(self, ctx, x: Tensor, cache) -> Tensor:
        """The path of a mixer with head norms, a number per head, values of their own size or
        rotated values: product, one kernel for everything up to the cache, attention, and
        the turning back of the output where values are stored rotated."""
        s, k = self.spec, ctx.k
        T = x.shape[0]
        nh, nkv, hd, vd = s.num_heads, s.num_kv_heads, s.head_dim, self.value_dim
        n_store = 0 if self.shared_kv else nkv
        heads_width = (nh + n_store) * hd + (0 if self.values_are_keys else n_store * vd)
        width = heads_width + (nh * vd if self.gate_name else 0)
        g = ctx.group(cache.group)
        tables = self.position.rotary_tables()
        qkv = linear(ctx, x, self.w_qkv, ctx.alloc((T, width)))
        if tables is None:
            self.position.apply(ctx, qkv, nh, n_store, hd)
        ptr = lambda t: t.ptr if t is not None else None
        vfreq = ptr(self.value_freq)
        inter = 1 if getattr(s, "value_pairs_interleaved", False) else 0
        if self.by_rows:
            # bias, the norms over whole rows, rotation and the store of keys and values, one launch
            k.zk_row_prep(qkv.ptr, width, ctx.positions, g.slot_map, ptr(self.in_bias), ptr(self.q_row_gain),
                          ptr(self.k_row_gain), float(s.norm_eps), tables[0].ptr if tables is not None else None,
                          tables[1] if tables is not None else 0, cache.k.ptr, cache.v.ptr, T, nh, nkv, hd, vd,
                          g.page_size, 1 if cache.v_transposed else 0, 1 if self.values_are_keys else 0, ctx.stream)
        prep = None if self.by_rows else (qkv.ptr, ctx.positions, None if self.shared_kv else g.slot_map, ptr(self.q_gain),
                ptr(self.k_gain), ptr(self.head_scale), float(s.norm_eps),
                tables[0].ptr if tables is not None else None, tables[1] if tables is not None else 0, vfreq,
                inter, cache.k.ptr, cache.v.ptr, T, nh, n_store, hd, vd, g.page_size,
                1 if cache.v_transposed else 0, ptr(self.in_bias), self.rot_scale,
                1 if self.rot_interleaved else 0)
        if prep is None:
            pass
        elif self.unit_norm or width != heads_width:
            k.zk_head_prep_unit(*prep, width, 1 if self.unit_norm else 0, ctx.stream)
        else:
            k.zk_head_prep_ext(*prep, ctx.stream)
        o = ctx.alloc((T, nh * vd))
        cap = float(s.softcap) if s.softcap else 0.0
        win = int(s.window) if s.window else 0
        masked = bool(self.chunk or self.unit_sink or self.wide_weights)
        if masked and cache.v_transposed and ctx.tuned and vd == hd:
            k.zk_attention_bf16_masked(qkv.ptr, width, cache.k.ptr, cache.v.ptr, g.block_table, g.max_blocks,
                                       ctx.q_start, ctx.ctx_len, o.ptr, ctx.R, ctx.n_multi, ctx.max_q_len,
                                       ctx.max_ctx, nh, nkv, hd, g.page_size, s.scale, cap, win,
                                       self.decode_chunk, ctx.workspace.ptr, ctx.workspace.nbytes, self.chunk,
                                       1 if self.unit_sink else 0, 1 if self.wide_weights else 0, ctx.stream)
        elif masked:
            k.zk_attention_plain_masked(qkv.ptr, width, cache.k.ptr, cache.v.ptr, g.block_table, g.max_blocks,
                                        ctx.req_of_token, ctx.positions, o.ptr, T, nh, nkv, hd, vd, g.page_size, s.scale,
                                        cap, win, 1 if cache.v_transposed else 0, vfreq, inter, None, 0, self.chunk,
                                        1 if self.unit_sink else 0, ctx.stream)
        elif cache.v_transposed and ctx.tuned and vd == hd:
            k.zk_attention_bf16(qkv.ptr, width, cache.k.ptr, cache.v.ptr, g.block_table, g.max_blocks,
                                ctx.q_start, ctx.ctx_len, o.ptr, ctx.R, ctx.n_multi, ctx.max_q_len,
                                ctx.max_ctx, nh, nkv, hd, g.page_size, s.scale, cap, win,
                                self.decode_chunk, ctx.workspace.ptr, ctx.workspace.nbytes, ctx.stream)
            if vfreq is not None:
                k.zk_rotate_heads(o.ptr, ctx.positions, vfreq, T, nh, vd, inter, -1.0, ctx.stream)
        else:
            k.zk_attention_plain_ext(qkv.ptr, width, cache.k.ptr, cache.v.ptr, g.block_table, g.max_blocks,
                                     ctx.req_of_token, ctx.positions, o.ptr, T, nh, nkv, hd, vd, g.page_size, s.scale,
                                     cap, win, 1 if cache.v_transposed else 0, vfreq, inter, ctx.stream)
        if self.gate_name:
            # the heads times sigmoid(W_g x); the gate's columns lie behind the heads' in the product's rows
            k.zk_gate_heads(o.ptr, qkv.ptr + heads_width * ITEMSIZE[ctx.dtype], width, T, nh * vd, ctx.stream)
        y = linear(ctx, o, self.w_o, ctx.alloc((T, s.hidden_size)), last_of=self if self.o_bias is None else None)
        if self.o_bias is not None:
            if getattr(ctx, "bias_welcome", None) is self:
                ctx.result_bias = self.o_bias          # the block's joining kernel adds it
            else:
                k.zk_add_bias(y.ptr, self.o_bias.ptr, T, s.hidden_size, ctx.stream)
        return y

    def forward(self, ctx, x: Tensor, cache) -> Tensor:
        if self.general:
            return self._forward_general(ctx, x, cache)
        s, k = self.spec, ctx.k
        T = x.shape[0]
        nh, nkv, hd = s.num_heads, s.num_kv_heads, s.head_dim
        n_store = 0 if self.shared_kv else nkv
        width = (nh + 2 * n_store) * hd
        g = ctx.group(cache.group)
        tables = self.position.rotary_tables()
        hooked = type(self).between_product_and_rotation is not PagedAttention.between_product_and_rotation
        if (not hooked and tables is not None and tuned_gemm(ctx, s.hidden_size) and k.has("zk_qkv_rope_bf16")
                and k.zk_qkv_rope_bf16_supports(T, s.hidden_size, hd, tables[1])):
            # few decoded tokens: the product rotates and stores its own results
            qkv = ctx.alloc((T, width))
            k.zk_qkv_rope_bf16(x.ptr, s.hidden_size, self.w_qkv.ptr, qkv.ptr, width, T, s.hidden_size,
                               1 if self.w_qkv.layout == "strip" else 0, ctx.positions,
                               None if self.shared_kv else g.slot_map, tables[0].ptr, cache.k.ptr,
                               cache.v.ptr, nh, n_store, hd, g.page_size, 1 if cache.v_transposed else 0,
                               ctx.stream)
        else:
            # a product that splits K may leave the adding up of its partial sums to the kernel
            # that rotates and stores, unless something has to look at the rows in between
            direct = not hooked and tables is not None and k.has("zk_rope_cache_write_sums")
            qkv = ctx.alloc((T, width))
            got = linear(ctx, x, self.w_qkv, qkv, sums_ok=direct)
            if hooked:
                self.between_product_and_rotation(ctx, qkv)
            if tables is None:
                self.position.apply(ctx, qkv, nh, n_store, hd)
                inv_freq, rotary_dim = 0, 0
            else:
                inv_freq, rotary_dim = tables[0].ptr, tables[1]
            args = (ctx.positions, None if self.shared_kv else g.slot_map, inv_freq or None, rotary_dim, cache.k.ptr,
                    cache.v.ptr, T, nh, n_store, hd, g.page_size, 1 if cache.v_transposed else 0, ctx.stream)
            if got.layout == "parts":
                k.zk_rope_cache_write_sums(qkv.ptr, got.ptr, got.shape[0], *args)
            else:
                k.zk_rope_cache_write(qkv.ptr, *args)
        o = ctx.alloc((T, nh * hd))
        cap = float(s.softcap) if s.softcap else 0.0
        win = int(s.window) if s.window else 0
        if cache.v_transposed and ctx.tuned:
            # the matrix-core kernel; requests with more than one token come first in the batch
            k.zk_attention_bf16(qkv.ptr, width, cache.k.ptr, cache.v.ptr, g.block_table, g.max_blocks,
                                ctx.q_start, ctx.ctx_len, o.ptr, ctx.R, ctx.n_multi, ctx.max_q_len,
                                ctx.max_ctx, nh, nkv, hd, g.page_size, s.scale, cap, win,
                                self.decode_chunk, ctx.workspace.ptr, ctx.workspace.nbytes, ctx.stream)
        else:
            k.zk_attention_plain(qkv.ptr, width, cache.k.ptr, cache.v.ptr, g.block_table,
                                 g.max_blocks, ctx.req_of_token, ctx.positions, o.ptr, T, nh, nkv,
                                 hd, g.page_size, s.scale, cap, win, 1 if cache.v_transposed else 0,
                                 ctx.stream)
        return linear(ctx, o, self.w_o, ctx.alloc((T, s.hidden_size)), last_of=self)


register_part("mixer", "attention", PagedAttention)

"""One layer: how a mixer and a feed-forward join the float residual stream.

"sandwich" is Gemma 2's order of four norms,
    h += post_m(mixer(pre_m(h)));  h += post_f(ffn(pre_f(h)))
the order of the reference's Gemma-family block (orchestrator/model_runner.py:425-439,
450-537).  "prenorm" leaves the post norms out (its Llama block, :1123-1297).  The
residual sum stays float throughout (orchestrator/vram_allocator.py:70-72).
"""
from __future__ import annotations

from ..runtime.device import Tensor
from .base import Part, build_part, register_part
from .norm import LayerNorm, RMSNorm

ARRANGEMENTS = {"sandwich": ("pre_mixer", "post_mixer", "pre_ffn", "post_ffn"),
                "prenorm": ("pre_mixer", "pre_ffn")}


class Block(Part):
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        if spec.arrangement not in ARRANGEMENTS:
            raise ValueError(f"arrangement must be one of {sorted(ARRANGEMENTS)}, got {spec.arrangement!r}")
        self.spec = spec
        roles = ARRANGEMENTS[spec.arrangement]
        missing = [r for r in roles if r not in spec.norms]
        if missing:
            raise ValueError(f"a {spec.arrangement} block needs norms {missing}")
        self.norms = {r: build_part("norm", spec.norms[r]) for r in roles}
        self.mixer = build_part("mixer", spec.mixer)
        self.ffn = build_part("ffn", spec.ffn)

    def children(self):
        return list(self.norms.values()) + [self.mixer, self.ffn]

    def _join(self, ctx, sub: Tensor, post, h: Tensor, nxt, out: Tensor = None):
        """h += post(sub) (post None: h += sub); returns nxt(h) if nxt is given, written
        to ``out`` when the caller brings a buffer."""
        T, H = h.shape
        fused_post = post is None or isinstance(post, RMSNorm)
        fused_next = nxt is None or isinstance(nxt, RMSNorm)
        if not fused_post:
            sub, post = post.forward(ctx, sub), None
        if nxt is None or not fused_next:
            out = None
        elif out is None:
            out = ctx.alloc((T, H))
        ps = post.spec if post is not None else None
        ns = nxt.spec if (nxt is not None and fused_next) else None
        parts = sub.shape[0] if sub.layout == "parts" else 0     # partial sums of a product that split K
        ctx.k.zk_norm_add_norm(
            sub.ptr, parts, post.weight.ptr if post is not None else None, ps.eps if ps else 0.0,
            int(ps.unit_offset) if ps else 0, h.ptr,
            nxt.weight.ptr if ns else None, ns.eps if ns else 0.0, int(ns.unit_offset) if ns else 0,
            out.ptr if out is not None else None, T, H, ctx.stream)
        if nxt is not None and not fused_next:
            out = nxt.forward(ctx, h)
        return out

    @staticmethod
    def _joins_sums(post) -> bool:
        return post is None or isinstance(post, RMSNorm)

    def entry_norm(self):
        """The norm this block applies to the stream first; the block before may apply it
        for us in the kernel that ends its own work (see ``forward``)."""
        return self.norms["pre_mixer"]

    def forward(self, ctx, h: Tensor, cache, x_in: Tensor = None, next_norm=None, x_out: Tensor = None):
        """Update the stream ``h`` in place.  ``x_in``: this block's entry norm of ``h``,
        if the caller already has it.  ``next_norm``: the entry norm of whatever runs
        next; its output is returned (computed in the same kernel as the last
        residual sum), in ``x_out`` if given."""
        n = self.norms
        x = x_in if x_in is not None else n["pre_mixer"].forward(ctx, h)
        # the joining kernel adds up the partial sums of a part's last product itself
        ctx.sums_welcome = self.mixer if self._joins_sums(n.get("post_mixer")) else None
        a = self.mixer.forward(ctx, x, cache)
        x = self._join(ctx, a, n.get("post_mixer"), h, n["pre_ffn"])
        ctx.sums_welcome = self.ffn if self._joins_sums(n.get("post_ffn")) else None
        m = self.ffn.forward(ctx, x)
        ctx.sums_welcome = None
        if not isinstance(next_norm, RMSNorm):
            next_norm = None         # a norm the closing kernel does not know: the next block applies it
        return self._join(ctx, m, n.get("post_ffn"), h, next_norm, x_out)


class ParallelBlock(Part):
    """x = norm(h); h += mixer(x) + ffn(x): both sublayers read the same stream, and their results
    are summed before they join it (``ffn`` None: the mixer alone).  With a second norm
    ``pre_ffn`` the feed-forward reads that norm of the same h instead, and with
    ``residual_scale`` m the sum joins as h += m (mixer + ffn).  One kernel does the sum, the
    mixer's output bias if it has one, the residual sum and the norms of whatever runs next (RMS
    norms, or one layer norm with gain and bias over a single stream)."""
    graph_safe = True      # its launches take what changes from step to step from device memory alone

    def __init__(self, spec):
        self.spec = spec
        if "pre_mixer" not in spec.norms:
            raise ValueError("a parallel block needs the norm pre_mixer")
        self.norms = {"pre_mixer": build_part("norm", spec.norms["pre_mixer"])}
        self.mixer = build_part("mixer", spec.mixer)
        self.ffn = build_part("ffn", spec.ffn) if spec.ffn is not None else None
        if self.ffn is not None and "pre_ffn" in spec.norms:
            self.norms["pre_ffn"] = build_part("norm", spec.norms["pre_ffn"])
        self.mult = float(getattr(spec, "residual_scale", 1.0))

    def children(self):
        return list(self.norms.values()) + [self.mixer] + ([self.ffn] if self.ffn is not None else [])

    def entry_norm(self):
        """The norm of the stream that the block reads first, or both of them."""
        if "pre_ffn" in self.norms:
            return (self.norms["pre_mixer"], self.norms["pre_ffn"])
        return self.norms["pre_mixer"]

    @staticmethod
    def _fusable(norms) -> bool:
        """Whether the closing kernel can make these norms: RMS norms of one eps and one kind of gain."""
        return all(isinstance(n, RMSNorm) for n in norms) and \
            len({(float(n.spec.eps), bool(n.spec.unit_offset)) for n in norms}) == 1

    def _entry(self, ctx, h: Tensor, x_in):
        """The block's own norms of the stream, from the caller where it brings them."""
        mine = self.entry_norm()
        if not isinstance(mine, tuple):
            return (x_in if x_in is not None else mine.forward(ctx, h)), None
        if isinstance(x_in, tuple):
            return x_in
        if not self._fusable(mine):
            return mine[0].forward(ctx, h), mine[1].forward(ctx, h)
        T, H = h.shape
        x1, x2 = ctx.alloc((T, H)), ctx.alloc((T, H))
        sp = mine[0].spec
        ctx.k.zk_sum_norm_pair(h.ptr, None, 0, None, 0, None, 1.0, mine[0].weight.ptr, x1.ptr, mine[1].weight.ptr, x2.ptr,
                               float(sp.eps), int(sp.unit_offset), T, H, ctx.stream)
        return x1, x2

    def forward(self, ctx, h: Tensor, cache, x_in=None, next_norm=None, x_out=None):
        """``x_in``, ``next_norm`` and ``x_out`` are single or pairs, as ``entry_norm`` of this block
        and of the next one are."""
        T, H = h.shape
        x, x2 = self._entry(ctx, h, x_in)
        # the mixer's result has to outlive the feed-forward's products: no partial sums in the
        # products' shared workspace (a float plane in the step's own memory is welcome); its
        # output bias is added by the joining kernel
        ctx.sums_welcome, ctx.bias_welcome, ctx.result_bias, ctx.plane_welcome = None, self.mixer, None, self.mixer
        a = self.mixer.forward(ctx, x, cache)
        bias, ctx.bias_welcome, ctx.result_bias, ctx.plane_welcome = ctx.result_bias, None, None, None
        m = None
        if self.ffn is not None:
            ctx.sums_welcome = self.ffn
            m = self.ffn.forward(ctx, x2 if x2 is not None else x)
            ctx.sums_welcome = None
        nxt = next_norm if isinstance(next_norm, tuple) else ((next_norm,) if next_norm is not None else ())
        layer_norm = (len(nxt) == 1 and isinstance(nxt[0], LayerNorm) and nxt[0].spec.streams == 1 and self.mult == 1.0)
        if not nxt or not (self._fusable(nxt) or layer_norm) or len(nxt) > 2:
            nxt = ()             # norms the closing kernel does not know: the next block applies them
        outs = []
        for i in range(len(nxt)):
            buf = (x_out[i] if isinstance(x_out, (tuple, list)) else x_out if i == 0 else None) if x_out is not None else None
            outs.append(ctx.alloc((T, H)) if buf is None else Tensor(buf.ptr, (T, H), ctx.dtype, buf.owner))
        planes = lambda t: t.shape[0] if (t is not None and t.layout == "parts") else 0
        ptr = lambda t: t.ptr if t is not None else None
        if nxt and layer_norm:
            n0 = nxt[0]
            ctx.k.zk_sum_layer_norm(h.ptr, a.ptr, planes(a), ptr(m), planes(m), ptr(bias), n0.weight.ptr, ptr(n0.bias),
                                    float(n0.spec.eps), outs[0].ptr, T, H, ctx.stream)
        elif self.mult == 1.0 and len(nxt) <= 1:
            ns = nxt[0].spec if nxt else None
            ctx.k.zk_sum_norm(h.ptr, a.ptr, planes(a), ptr(m), planes(m), ptr(bias), nxt[0].weight.ptr if nxt else None,
                              float(ns.eps) if ns is not None else 0.0, int(ns.unit_offset) if ns is not None else 0,
                              outs[0].ptr if outs else None, T, H, ctx.stream)
        else:
            ns = nxt[0].spec if nxt else None
            w = [n.weight.ptr for n in nxt] + [None, None]
            o = [t.ptr for t in outs] + [None, None]
            ctx.k.zk_sum_norm_pair(h.ptr, a.ptr, planes(a), ptr(m), planes(m), ptr(bias), self.mult, w[0], o[0], w[1], o[1],
                                   float(ns.eps) if ns is not None else 0.0, int(ns.unit_offset) if ns is not None else 0,
                                   T, H, ctx.stream)
        if not outs:
            return None
        return tuple(outs) if isinstance(next_norm, tuple) else outs[0]


def _block(spec):
    return ParallelBlock(spec) if spec.arrangement == "parallel" else Block(spec)


register_part("block", "block", _block)

"""Rotalorn: a decoder-only model whose layers are listed one by one in its config.json.

The embedded row of a token is joined by a row of a table of token pairs (a hash of the previous
token and the token; a row of its own for a sequence's first token).  A layer is a parallel
layer: one layer norm with gain and bias, and a mixer and a feed-forward that both read it;
their sum joins the residual.  The mixer is
  - ``attention``: grouped-query attention with biases on q and k, an RMS norm over the whole query
    row and the whole key row, rotary positions (pairs (i, i + dims/2)) whose frequencies may be
    scaled by their wavelengths, a sliding window, and values that are the keys as projected;
  - ``latent_attention``: attention over one cached latent row a token, the queries through a
    latent of their own, one rotated key part shared by the heads, a sliding window, and a gate of
    one number a head on the outputs;
  - ``attention_2``: differential attention, two softmax maps a head over the same values, a query
    temperature of the position, capped scores, every earlier key visible.
The feed-forward is a dense gated layer (gelu, tanh form) or a mixture of silu-gated experts
with softmax scores that weigh the chosen experts' outputs, and a shared expert times the
sigmoid of a number a token.  The model's last norm is a layer norm; the logits come from the
embedding table.

config.json: ``vocab``, ``width``, ``norm.eps``, optional ``embedding.bigram`` (``buckets``,
``mul_prev``, ``mul_cur``), ``layers`` (a list of ``{type, mixer, mlp}``).  ``attention``: ``heads``,
``kv_heads``, ``dim``, ``vdim``, ``scale``, optional ``rot`` (``base``, ``dims``, optional ``scaling`` with
``factor``, ``low``, ``high``, ``original``), optional ``mask.size``.  ``latent_attention``: ``heads``,
``dim``, ``rot_dim``, ``vdim``, ``kv_rank``, ``q_rank``, ``scale``, ``rot.base``, optional ``mask.size``.
``attention_2``: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``diff``, optional ``softcap``,
``q_temp`` (``coef``, ``every``), ``mask.size``.  ``mlp``: null, ``{kind: "dense", ff}`` or ``{kind: "moe",
expert: {ff}, router: {experts, top}, shared: {ff} or null}``.  Tensor names: ``embed``, ``bigram``,
``final.norm``, ``final.norm.b`` and, for layer i, ``l<i>.norm1``, ``l<i>.norm1.b``, ``l<i>.mix.*``,
``l<i>.mlp.*``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from ..config.base import Architecture, Problems, need, register_architecture
from ..config.plan import (AttentionSpec, BlockSpec, DifferentialAttentionSpec, EmbeddingSpec, GatedMLPSpec, HeadSpec,
                           LatentAttentionSpec, LayerCall, LayerNormSpec, ModelPlan, NoPositionSpec, PairTableSpec,
                           RotarySpec, RoutedMLPSpec)

NAME = "Rotalorn"
MAX_POSITION = 1 << 16        # the config names no longest sequence; tables and pools follow the runner's own limits
# the softmax's weights are 32-bit numbers of the design: where a matrix-core kernel multiplies them with
# the values they go in as two bfloat16 halves (16 bits of mantissa), not rounded to one
WIDE_WEIGHTS = True
DENSE_ACTIVATION = "gelu_tanh"
EXPERT_ACTIVATION = "silu"
TYPES = ("attention", "latent_attention", "attention_2")


@dataclass(frozen=True)
class RotalornMLP:
    kind: str                          # "dense" | "moe"
    ff: int                            # of the dense layer, or of one expert
    experts: int = 0
    top: int = 0
    shared_ff: Optional[int] = None


@dataclass(frozen=True)
class RotalornLayer:
    type: str
    heads: int
    dim: int
    vdim: int
    mlp: Optional[RotalornMLP]
    scale: float = 1.0
    kv_heads: int = 0
    window: Optional[int] = None
    rot_base: Optional[float] = None
    rot_dims: int = 0
    rot_scaling: Optional[Tuple[float, float, float, float]] = None      # factor, low, high, original
    rot_dim: int = 0                   # latent attention: the rotated part of a head
    kv_rank: int = 0
    q_rank: int = 0
    diff: float = 0.0                  # differential attention
    softcap: Optional[float] = None
    temp_coef: float = 0.0
    temp_every: int = 0


@dataclass(frozen=True)
class RotalornConfig:
    vocab: int
    width: int
    eps: float
    bigram: Optional[Tuple[int, int, int]]     # buckets, mul_prev, mul_cur
    layers: Tuple[RotalornLayer, ...]
    raw: dict

    @staticmethod
    def _mlp(mlp: dict, q: Problems) -> Optional[RotalornMLP]:
        kind = need(mlp, "kind", str, q, required=True)
        if kind == "dense":
            ff = need(mlp, "ff", int, q, required=True)
            q.require(ff is None or ff > 0, f"mlp.ff must be positive, got {ff}")
            return RotalornMLP("dense", ff or 0) if not q.items else None
        if kind != "moe":
            q.add(f"mlp.kind must be 'dense' or 'moe', got {kind!r}")
            return None
        ex = need(mlp, "expert", dict, q, required=True) or {}
        ro = need(mlp, "router", dict, q, required=True) or {}
        sh = need(mlp, "shared", dict, q, default=None, allow_none=True)
        ff = need(ex, "ff", int, q, required=True)
        experts = need(ro, "experts", int, q, required=True)
        top = need(ro, "top", int, q, required=True)
        sff = need(sh, "ff", int, q, required=True) if sh is not None else None
        if q.items:
            return None
        q.require(ff > 0, f"mlp.expert.ff must be positive, got {ff}")
        q.require(1 <= top <= experts, f"mlp.router: top must lie in 1..experts, got {top} of {experts}")
        q.require(top <= 16 and experts <= 1024, f"mlp.router: up to 16 of up to 1024 experts, got {top} of {experts}")
        q.require(sh is None or sff > 0, f"mlp.shared.ff must be positive, got {sff}")
        return RotalornMLP("moe", ff, experts, top, sff)

    @staticmethod
    def _scaling(rot: Optional[dict], q: Problems):
        sc = need(rot, "scaling", dict, q, default=None, allow_none=True) if rot is not None else None
        if sc is None:
            return None
        vals = [need(sc, key, float, q, required=True) for key in ("factor", "low", "high", "original")]
        if None in vals:
            return None
        q.require(vals[0] > 0 and vals[3] > 0 and 0 < vals[1] < vals[2],
                  f"rot.scaling: factor and original positive and 0 < low < high, got {vals}")
        return tuple(vals)

    @staticmethod
    def _window(mx: dict, q: Problems) -> Optional[int]:
        mask = need(mx, "mask", dict, q, default=None, allow_none=True)
        if mask is None:
            return None
        size = need(mask, "size", int, q, required=True)
        q.require(size is None or size >= 1, f"mask.size must be at least 1, got {size}")
        return size

    @staticmethod
    def from_dict(raw: dict) -> "RotalornConfig":
        p = Problems("Rotalorn config.json")
        V = need(raw, "vocab", int, p, required=True)
        W = need(raw, "width", int, p, required=True)
        norm = need(raw, "norm", dict, p, required=True) or {}
        eps = need(norm, "eps", float, p, required=True)
        layers_raw = need(raw, "layers", list, p, required=True) or []
        emb = need(raw, "embedding", dict, p, default=None, allow_none=True) or {}
        bg = need(emb, "bigram", dict, p, default=None, allow_none=True)
        bigram = None
        if bg is not None:
            vals = [need(bg, key, int, p, required=True) for key in ("buckets", "mul_prev", "mul_cur")]
            if None not in vals:
                p.require(vals[0] >= 1, f"embedding.bigram.buckets must be at least 1, got {vals[0]}")
                bigram = tuple(vals)
        p.raise_if_any()
        p.require(V > 0 and W > 0, f"'vocab' and 'width' must be positive, got {V} and {W}")
        p.require(eps > 0, f"'norm.eps' must be positive, got {eps}")
        p.require(len(layers_raw) > 0, "'layers' is empty")
        layers = []
        for i, lr in enumerate(layers_raw):
            q = Problems(f"layer {i}")
            if not isinstance(lr, dict):
                p.add(f"layer {i} must be an object")
                continue
            typ = need(lr, "type", str, q, required=True)
            mx = need(lr, "mixer", dict, q, required=True) or {}
            mlp_raw = need(lr, "mlp", dict, q, default=None, allow_none=True)
            mlp = RotalornConfig._mlp(mlp_raw, q) if mlp_raw is not None else None
            heads = need(mx, "heads", int, q, required=True)
            dim = need(mx, "dim", int, q, required=True)
            vdim = need(mx, "vdim", int, q, required=True)
            scale = need(mx, "scale", float, q, required=True)
            window = RotalornConfig._window(mx, q)
            if q.items:
                p.add(f"layer {i}: " + "; ".join(q.items))
                continue
            q.require(heads > 0 and dim > 0 and vdim > 0, "heads, dim and vdim must be positive")
            if typ == "attention":
                kvh = need(mx, "kv_heads", int, q, default=heads)
                rot = need(mx, "rot", dict, q, default=None, allow_none=True)
                base = need(rot, "base", float, q, required=True) if rot is not None else None
                dims = need(rot, "dims", int, q, default=dim) if rot is not None else 0
                scaling = RotalornConfig._scaling(rot, q)
                if not q.items:
                    q.require(kvh > 0 and heads % kvh == 0, f"heads ({heads}) must be a multiple of kv_heads ({kvh})")
                    q.require(rot is None or (base > 0 and base != 1 and dims % 2 == 0 and 0 < dims <= dim),
                              f"rot.base must be positive and rot.dims even and in (0, dim], got {base} and {dims}")
                    q.require(vdim == dim, f"the values are the keys: vdim ({vdim}) must equal dim ({dim})")
                    q.require(dim <= 256, f"an attention layer takes dim up to 256, got {dim}")
                layers.append(RotalornLayer("attention", heads, dim, vdim, mlp, scale=scale, kv_heads=kvh or heads,
                                            window=window, rot_base=base, rot_dims=dims or 0, rot_scaling=scaling))
            elif typ == "latent_attention":
                rdim = need(mx, "rot_dim", int, q, required=True)
                rank = need(mx, "kv_rank", int, q, required=True)
                qrank = need(mx, "q_rank", int, q, required=True)
                rot = need(mx, "rot", dict, q, required=True) or {}
                base = need(rot, "base", float, q, required=True)
                dims = need(rot, "dims", int, q, default=rdim)
                scaling = RotalornConfig._scaling(rot, q)
                if not q.items:
                    q.require(rdim > 0 and rdim % 2 == 0 and rank > 0 and qrank > 0,
                              f"rot_dim must be even and positive, kv_rank and q_rank positive, got {rdim}, {rank}, {qrank}")
                    q.require(dims == rdim, f"rot.dims ({dims}) must equal rot_dim ({rdim})")
                    q.require(base > 0 and base != 1, f"rot.base must be positive, got {base}")
                    q.require(rank + rdim <= 1024, f"kv_rank + rot_dim up to 1024, got {rank + rdim}")
                layers.append(RotalornLayer("latent_attention", heads, dim, vdim, mlp, scale=scale, window=window,
                                            rot_base=base, rot_dim=rdim or 0, kv_rank=rank or 0, q_rank=qrank or 0,
                                            rot_scaling=scaling))
            elif typ == "attention_2":
                kvh = need(mx, "kv_heads", int, q, default=heads)
                diff = need(mx, "diff", float, q, required=True)
                cap = need(mx, "softcap", float, q, default=None, allow_none=True)
                qt = need(mx, "q_temp", dict, q, default=None, allow_none=True)
                coef = need(qt, "coef", float, q, required=True) if qt is not None else 0.0
                every = need(qt, "every", int, q, required=True) if qt is not None else 0
                if not q.items:
                    q.require(kvh > 0 and heads % kvh == 0, f"heads ({heads}) must be a multiple of kv_heads ({kvh})")
                    q.require(cap is None or cap > 0, f"softcap must be positive, got {cap}")
                    q.require(qt is None or every >= 1, f"q_temp.every must be at least 1, got {every}")
                    q.require(dim <= 256 and vdim <= 256, f"a differential attention takes dim and vdim up to 256, got {dim} and {vdim}")
                layers.append(RotalornLayer("attention_2", heads, dim, vdim, mlp, scale=scale, kv_heads=kvh or heads,
                                            window=window, diff=diff or 0.0, softcap=cap, temp_coef=coef or 0.0,
                                            temp_every=every or 0))
            else:
                q.add(f"unknown type {typ!r} {TYPES}")
            if q.items:
                p.add(f"layer {i}: " + "; ".join(q.items))
        p.raise_if_any()
        return RotalornConfig(V, W, eps, bigram, tuple(layers), dict(raw))

    def to_dict(self) -> dict:
        return dict(self.raw)


def rotalorn_plan(c: RotalornConfig) -> ModelPlan:
    layers = []
    for i, l in enumerate(c.layers):
        pre = f"l{i}."
        mix = pre + "mix."
        if l.type == "attention":
            rotary = (RotarySpec(head_dim=l.dim, rotary_dim=l.rot_dims, theta=l.rot_base, wavelength_scaling=l.rot_scaling)
                      if l.rot_base is not None else NoPositionSpec())
            mixer = AttentionSpec(
                hidden_size=c.width, num_heads=l.heads, num_kv_heads=l.kv_heads, head_dim=l.dim, scale=l.scale,
                softcap=None, window=l.window, position=rotary, names={r: mix + r for r in ("q", "k", "o")},
                biases={r: f"{mix}{r}.b" for r in ("q", "k")}, norm_eps=c.eps,
                q_row_norm=mix + "q.norm", k_row_norm=mix + "k.norm", values_are_keys=True, wide_weights=WIDE_WEIGHTS)
        elif l.type == "latent_attention":
            mixer = LatentAttentionSpec(
                hidden_size=c.width, num_heads=l.heads, head_dim=l.dim, rotary_dim=l.rot_dim, value_dim=l.vdim,
                latent_dim=l.kv_rank, scale=l.scale, eps=c.eps,
                position=RotarySpec(head_dim=l.rot_dim, rotary_dim=l.rot_dim, theta=l.rot_base,
                                    wavelength_scaling=l.rot_scaling),
                names={"q": mix + "uq", "q_down": mix + "dq", "q_down_norm": mix + "dq.norm", "down": mix + "dkv",
                       "down_norm": mix + "dkv.norm", "up_k": mix + "uk", "up_v": mix + "uv", "gate": mix + "g",
                       "o": mix + "o"},
                window=l.window, query_latent_dim=l.q_rank, wide_weights=WIDE_WEIGHTS)
        else:
            mixer = DifferentialAttentionSpec(
                hidden_size=c.width, num_heads=l.heads, num_kv_heads=l.kv_heads, head_dim=l.dim, value_dim=l.vdim,
                scale=l.scale, softcap=l.softcap, window=l.window, diff=l.diff, eps=c.eps, temp_coef=l.temp_coef,
                temp_every=l.temp_every,
                names={r: mix + r for r in ("q", "k", "v", "o", "lq1", "lk1", "lq2", "lk2")}, wide_weights=WIDE_WEIGHTS)
        ffn = None
        if l.mlp is not None and l.mlp.kind == "dense":
            ffn = GatedMLPSpec(hidden_size=c.width, intermediate_size=l.mlp.ff, activation=DENSE_ACTIVATION,
                               names={r: f"{pre}mlp.{r}" for r in ("gate", "up", "down")})
        elif l.mlp is not None:
            m, mlp = l.mlp, pre + "mlp."
            shared = None
            if m.shared_ff is not None:
                shared = GatedMLPSpec(hidden_size=c.width, intermediate_size=m.shared_ff, activation=EXPERT_ACTIVATION,
                                      names={r: f"{mlp}shared.{r}" for r in ("gate", "up", "down")})
            ffn = RoutedMLPSpec(hidden_size=c.width, intermediate_size=m.ff, num_experts=m.experts, top_k=m.top,
                                activation=EXPERT_ACTIVATION, limit=None, router=mlp + "router",
                                expert_names=mlp + "e{e}.{role}", shared=shared, scale_input=False, scoring="softmax",
                                shared_gate=(mlp + "shared.sg") if shared is not None else None)
        layers.append(BlockSpec(arrangement="parallel", mixer=mixer, ffn=ffn,
                                norms={"pre_mixer": LayerNormSpec(c.width, c.eps, pre + "norm1", pre + "norm1.b")}))
    pairs = PairTableSpec(c.bigram[0], c.bigram[1], c.bigram[2], "bigram") if c.bigram is not None else None
    return ModelPlan(
        architecture=NAME, hidden_size=c.width, vocab_size=c.vocab, max_position=MAX_POSITION,
        embedding=EmbeddingSpec(c.vocab, c.width, 1.0, "embed", pairs=pairs),
        layers=tuple(layers), order=tuple(LayerCall(i) for i in range(len(layers))),
        final_norm=LayerNormSpec(c.width, c.eps, "final.norm", "final.norm.b"),
        head=HeadSpec(c.vocab, c.width, None, "embed"),
        optional_prefixes=())


ROTALORN = register_architecture(Architecture(
    name=NAME, config_from_dict=RotalornConfig.from_dict, plan=rotalorn_plan, model_types=("rotalorn",)))

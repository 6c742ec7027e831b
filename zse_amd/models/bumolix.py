"""Bumolix: a decoder-only model whose layers are listed one by one in its config.json.

A layer is a parallel layer with two RMS norms (plain gain) of the same stream: the mixer reads
the first, the feed-forward the second, and h <- h + m (mixer + ffn) with m = ``residual_mult``.
The mixer is either two mixers side by side whose weighted results are added (``parallel``), or
a selective scan (``mamba1``).  Side by side stand a grouped-query attention (biases on q, k, v;
rotary positions on part of a head with all frequencies divided by a factor; q and k divided by
their root mean square after the rotation; keys of the query's own chunk of positions only; a
sink of score 0 in the softmax's denominator; heads gated by sigmoid(W_g x)) and a gated linear
attention (a matrix state per head with a decay per key channel).  The feed-forward is
W_down relu(W_up x)^2.  The logits come from the embedding table.

config.json: ``vocab``, ``width``, ``norm.eps``, ``residual_mult``, ``layers`` (a list of
``{type, mixer, mlp}``).  A ``parallel`` mixer: ``left`` (``heads``, ``kv_heads``, ``dim``, ``vdim``,
``scale``, optional ``mask.size``, optional ``rot`` with ``base``, ``dims`` and optional
``scaling.factor``), ``right`` (``heads``, ``dim``, ``vdim``, ``tau``), ``left_scale``, ``right_scale``.
A ``mamba1`` mixer: ``inner``, ``state``, ``dt_rank``, ``conv``.  ``mlp``: null or ``{kind: "dense",
ff}``.  Sizes that the config does not name (the rank of the decays' projection) are read off
the tensors' shapes by the loader's check.  Tensor names: ``embed``, ``final.norm`` and, for layer
i, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from ..config.base import Architecture, Problems, need, register_architecture
from ..config.plan import (AttentionSpec, BlockSpec, EmbeddingSpec, HeadSpec, LayerCall, LinearAttentionSpec, MLPSpec,
                           ModelPlan, NoPositionSpec, NormSpec, RotarySpec, SelectiveScanSpec, SideBySideSpec)

NAME = "Bumolix"
MAX_POSITION = 1 << 16        # the config names no longest sequence; tables and pools follow the runner's own limits
ACTIVATION = "relu2"


@dataclass(frozen=True)
class BumolixLeft:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: Optional[int]
    rot_base: Optional[float]
    rot_dims: int
    rot_factor: Optional[float]


@dataclass(frozen=True)
class BumolixRight:
    heads: int
    dim: int
    vdim: int
    tau: float
    rank: int                          # rows of the decays' first projection


@dataclass(frozen=True)
class BumolixScan:
    inner: int
    state: int
    dt_rank: int
    conv: int


@dataclass(frozen=True)
class BumolixLayer:
    type: str                          # "parallel" | "mamba1"
    ff: Optional[int]
    left: Optional[BumolixLeft] = None
    right: Optional[BumolixRight] = None
    left_scale: float = 1.0
    right_scale: float = 1.0
    scan: Optional[BumolixScan] = None


@dataclass(frozen=True)
class BumolixConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float
    layers: Tuple[BumolixLayer, ...]
    raw: dict

    @staticmethod
    def _left(mx: dict, q: Problems) -> Optional[BumolixLeft]:
        heads = need(mx, "heads", int, q, required=True)
        kvh = need(mx, "kv_heads", int, q, default=heads)
        dim = need(mx, "dim", int, q, required=True)
        vdim = need(mx, "vdim", int, q, default=dim)
        scale = need(mx, "scale", float, q, required=True)
        mask = need(mx, "mask", dict, q, default=None, allow_none=True)
        chunk = need(mask, "size", int, q, required=True) if mask is not None else None
        rot = need(mx, "rot", dict, q, default=None, allow_none=True)
        base = need(rot, "base", float, q, required=True) if rot is not None else None
        dims = need(rot, "dims", int, q, default=dim) if rot is not None else 0
        sc = need(rot, "scaling", dict, q, default=None, allow_none=True) if rot is not None else None
        factor = need(sc, "factor", float, q, required=True) if sc is not None else None
        if q.items:
            return None
        q.require(heads > 0 and dim > 0 and vdim > 0, "left: heads, dim and vdim must be positive")
        q.require(kvh > 0 and heads % max(kvh, 1) == 0, f"left: heads ({heads}) must be a multiple of kv_heads ({kvh})")
        q.require(dim <= 256 and vdim <= 256, f"left: dim and vdim up to 256, got {dim} and {vdim}")
        q.require(chunk is None or chunk > 0, f"left: mask.size must be positive, got {chunk}")
        q.require(rot is None or (base > 0 and base != 1 and dims % 2 == 0 and 0 < dims <= dim),
                  f"left: rot.base must be positive and rot.dims even and in (0, dim], got {base} and {dims}")
        q.require(factor is None or factor > 0, f"left: rot.scaling.factor must be positive, got {factor}")
        return BumolixLeft(heads, kvh, dim, vdim, scale, chunk, base, dims or 0, factor)

    @staticmethod
    def _right(mx: dict, q: Problems) -> Optional[BumolixRight]:
        heads = need(mx, "heads", int, q, required=True)
        dim = need(mx, "dim", int, q, required=True)
        vdim = need(mx, "vdim", int, q, default=dim)
        tau = need(mx, "tau", float, q, required=True)
        rank = need(mx, "rank", int, q, default=0)        # not a key of the format: the tensors' shapes say it
        if q.items:
            return None
        q.require(heads > 0 and dim > 0 and vdim > 0, "right: heads, dim and vdim must be positive")
        q.require(dim <= 256 and vdim <= 1024, f"right: dim up to 256 and vdim up to 1024, got {dim} and {vdim}")
        q.require(tau > 0, f"right: tau must be positive, got {tau}")
        return BumolixRight(heads, dim, vdim, tau, rank)

    @staticmethod
    def from_dict(raw: dict) -> "BumolixConfig":
        p = Problems("Bumolix config.json")
        V = need(raw, "vocab", int, p, required=True)
        W = need(raw, "width", int, p, required=True)
        norm = need(raw, "norm", dict, p, required=True) or {}
        eps = need(norm, "eps", float, p, required=True)
        mult = need(raw, "residual_mult", float, p, default=1.0)
        layers_raw = need(raw, "layers", list, p, required=True) or []
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
            mlp = need(lr, "mlp", dict, q, default=None, allow_none=True)
            ff = None
            if mlp is not None:
                kind = need(mlp, "kind", str, q, default="dense")
                q.require(kind == "dense", f"mlp.kind must be 'dense', got {kind!r}")
                ff = need(mlp, "ff", int, q, required=True)
                q.require(ff is None or ff > 0, f"mlp.ff must be positive, got {ff}")
            if typ == "parallel":
                left_raw = need(mx, "left", dict, q, required=True)
                right_raw = need(mx, "right", dict, q, required=True)
                ls = need(mx, "left_scale", float, q, default=1.0)
                rs = need(mx, "right_scale", float, q, default=1.0)
                left = BumolixConfig._left(left_raw, q) if left_raw is not None else None
                right = BumolixConfig._right(right_raw, q) if right_raw is not None else None
                layers.append(BumolixLayer("parallel", ff, left=left, right=right, left_scale=ls, right_scale=rs))
            elif typ == "mamba1":
                inner = need(mx, "inner", int, q, required=True)
                state = need(mx, "state", int, q, required=True)
                rank = need(mx, "dt_rank", int, q, required=True)
                taps = need(mx, "conv", int, q, required=True)
                if not q.items:
                    q.require(inner > 0 and rank > 0 and taps >= 1, f"inner, dt_rank and conv must be positive, got {inner}, {rank}, {taps}")
                    q.require(0 < state <= 128, f"state must lie in 1..128, got {state}")
                layers.append(BumolixLayer("mamba1", ff, scan=BumolixScan(inner or 1, state or 1, rank or 1, taps or 1)))
            else:
                q.add(f"unknown type {typ!r} (parallel, mamba1)")
            if q.items:
                p.add(f"layer {i}: " + "; ".join(q.items))
        p.raise_if_any()
        return BumolixConfig(V, W, eps, mult, tuple(layers), dict(raw))

    def to_dict(self) -> dict:
        return dict(self.raw)


def bumolix_plan(c: BumolixConfig) -> ModelPlan:
    layers = []
    for i, l in enumerate(c.layers):
        pre = f"l{i}."
        mix = pre + "mix."
        if l.type == "parallel":
            a, g = l.left, l.right
            lm, rm = mix + "left.", mix + "right."
            rotary = (RotarySpec(head_dim=a.dim, rotary_dim=a.rot_dims, theta=a.rot_base, linear_factor=a.rot_factor)
                      if a.rot_base is not None else NoPositionSpec())
            left = AttentionSpec(
                hidden_size=c.width, num_heads=a.heads, num_kv_heads=a.kv_heads, head_dim=a.dim, scale=a.scale,
                softcap=None, window=None, position=rotary, names={r: lm + r for r in ("q", "k", "v", "o")},
                value_dim=a.vdim, norm_eps=c.eps, biases={r: f"{lm}{r}.b" for r in ("q", "k", "v")}, chunk=a.chunk,
                unit_sink=True, qk_unit_norm=True, gate=lm + "g", wide_weights=True)
            right = LinearAttentionSpec(
                hidden_size=c.width, num_heads=g.heads, key_dim=g.dim, value_dim=g.vdim, decay_rank=g.rank, tau=g.tau,
                eps=c.eps, names={"q": rm + "q", "k": rm + "k", "v": rm + "v", "gate": rm + "g", "o": rm + "o",
                                  "norm": rm + "norm", "a1": rm + "a1", "a2": rm + "a2", "a2_bias": rm + "a2.b"})
            mixer = SideBySideSpec(mixers=(left, right), scales=(l.left_scale, l.right_scale))
        else:
            s = l.scan
            mixer = SelectiveScanSpec(
                hidden_size=c.width, inner=s.inner, state=s.state, dt_rank=s.dt_rank, conv_taps=s.conv,
                names={"in": mix + "in", "conv": mix + "conv", "conv_bias": mix + "conv.b", "x": mix + "x", "dt": mix + "dt",
                       "dt_bias": mix + "dt.b", "A_log": mix + "A_log", "D": mix + "D", "o": mix + "o"})
        ffn = None
        norms = {"pre_mixer": NormSpec(c.width, c.eps, False, pre + "norm1")}
        if l.ff is not None:
            ffn = MLPSpec(hidden_size=c.width, intermediate_size=l.ff, activation=ACTIVATION,
                          names={"up": pre + "mlp.up", "down": pre + "mlp.down"})
            norms["pre_ffn"] = NormSpec(c.width, c.eps, False, pre + "norm2")
        layers.append(BlockSpec(arrangement="parallel", mixer=mixer, ffn=ffn, norms=norms, residual_scale=c.residual_mult))
    return ModelPlan(
        architecture=NAME, hidden_size=c.width, vocab_size=c.vocab, max_position=MAX_POSITION,
        embedding=EmbeddingSpec(c.vocab, c.width, 1.0, "embed"),
        layers=tuple(layers), order=tuple(LayerCall(i) for i in range(len(layers))),
        final_norm=NormSpec(c.width, c.eps, False, "final.norm"),
        head=HeadSpec(c.vocab, c.width, None, "embed"),
        optional_prefixes=())


BUMOLIX = register_architecture(Architecture(
    name=NAME, config_from_dict=BumolixConfig.from_dict, plan=bumolix_plan, model_types=("bumolix",)))

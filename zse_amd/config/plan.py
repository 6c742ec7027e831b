"""The data an architecture hands to the engine: parts, layers, and their order.

A ``ModelPlan`` is plain data.  Every part is described by a small frozen
dataclass carrying a ``kind`` (the key of the part's class in
``zse_amd.parts.registry``), its sizes and constants, and the checkpoint
names of its tensors.  No part description names the model it belongs to.

The reference keeps one flat ``ModelConfig`` for every architecture and picks
a forward path by ``config.arch`` (format/config.py:33-95,
orchestrator/model_runner.py:127-130); here the choice is made layer by layer
from these records instead.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass(frozen=True)
class NormSpec:
    """Root-mean-square norm over the last axis: x * rsqrt(mean(x^2)+eps) * gain,
    gain = (1 + w) when ``unit_offset`` else w."""
    size: int
    eps: float
    unit_offset: bool
    weight: str                      # checkpoint tensor name
    kind: str = "rmsnorm"


@dataclass(frozen=True)
class LayerNormSpec:
    """Layer norm over the last axis: (x - mean) / sqrt(var + eps) * gain + bias, var the mean of
    the squared deviations.  ``streams`` > 1: the input holds that many residual streams per
    token and the norm reads their plain sum."""
    size: int
    eps: float
    weight: str
    bias: Optional[str]
    streams: int = 1
    kind: str = "layernorm"


@dataclass(frozen=True)
class ShortConvSpec:
    """x_t + sum_j w[:, j] x_(t - taps + 1 + j): a causal convolution over time on each channel,
    zeros before a sequence's start; the last ``taps - 1`` rows are a request's state."""
    size: int
    taps: int
    weight: Any                      # [size, taps]: a name, or several whose tensors are stacked along the channels
    kind: str = "short_conv"
    residual: bool = True            # False: the sum alone, without x_t added
    activation: Optional[str] = None  # "silu": applied to the result
    channel_counts: Optional[Tuple[int, ...]] = None   # with several weight names: the channels of each
    bias: Optional[str] = None       # [size]: where the sum over the taps starts


@dataclass(frozen=True)
class RotarySpec:
    """Rotate-half rotary encoding of the first ``rotary_dim`` channels of a head."""
    head_dim: int
    rotary_dim: int
    theta: float
    kind: str = "rotary"
    interleaved: bool = False        # pairs (2i, 2i + 1) instead of (i, i + rotary_dim / 2)
    # (factor, original, fast, slow): frequencies that turn fewer than ``slow`` times in ``original``
    # positions are divided by ``factor``, those that turn more than ``fast`` times stay, a linear
    # ramp over the pair numbers in between; sines and cosines are multiplied by 0.1 ln(factor) + 1
    scaling: Optional[Tuple[float, float, float, float]] = None
    linear_factor: Optional[float] = None   # every frequency is divided by it (positions stretched); magnitudes stay 1
    # (factor, low, high, original): each frequency f judged by its wavelength l = 2 pi / f: it stays where
    # l < original / high, is divided by ``factor`` where l > original / low, and in between becomes
    # (1 - s) f / factor + s f with s = (original / l - low) / (high - low); magnitudes stay 1
    wavelength_scaling: Optional[Tuple[float, float, float, float]] = None


@dataclass(frozen=True)
class NoPositionSpec:
    kind: str = "none"


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query softmax attention over a paged key/value cache."""
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float                     # multiplies q.k
    softcap: Optional[float]         # cap * tanh(s / cap) on scaled scores
    window: Optional[int]            # keys i-j < window visible; None = all
    position: Any                    # a position-encoding spec
    names: Dict[str, str]            # roles q, k, v, o -> checkpoint names
    kind: str = "attention"
    # what follows is optional; a model that uses none of it runs as before
    value_dim: Optional[int] = None          # size of a head's values (None: head_dim)
    q_norm: Optional[str] = None             # gain [head_dim] of an RMS norm over each query head, before rotation
    k_norm: Optional[str] = None             # the same for key heads
    norm_eps: float = 1e-6
    head_scale: Optional[str] = None         # [num_heads]: a number per query head that multiplies its scores
    value_rotation: Optional[float] = None   # base: values are cached turned by their position over all their
    #                                          channels (pair m by pos * base^(-2m/value_dim)), outputs turned back
    value_pairs_interleaved: bool = False    # pairs (2m, 2m + 1) instead of (m, m + value_dim / 2)
    biases: Optional[Dict[str, str]] = None  # roles q, k, v, o -> names of vectors added in the projections
    chunk: Optional[int] = None              # keys of the query's own chunk only: floor(i / chunk) == floor(j / chunk),
    #                                          chunks counted from position 0 of the sequence (not together with window)
    unit_sink: bool = False                  # a sink of score 0 without a value: weights exp(s_j) / (1 + sum exp(s))
    qk_unit_norm: bool = False               # q and k divided by their root mean square per head, no gain, AFTER rotation
    gate: Optional[str] = None               # [num_heads * value_dim, hidden]: heads times sigmoid(W_g x) before W_o
    wide_weights: bool = False               # the softmax's weights are not rounded to 8 bits of mantissa before they
    #                                          meet the values (the matrix-core kernel sends them in two halves)
    q_row_norm: Optional[str] = None         # gain [num_heads * head_dim] of an RMS norm over a token's whole query row
    #                                          (all heads at once, after the bias, before rotation; eps is norm_eps)
    k_row_norm: Optional[str] = None         # the same over the whole key row, gain [num_kv_heads * head_dim]
    values_are_keys: bool = False            # no value projection: a value is its key as projected (with its bias,
    #                                          before norm and rotation); ``names`` and ``biases`` hold no role v


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Softmax attention whose keys and values are made from one cached latent row per token:
    c = rms_norm(first ``latent_dim`` rows of W_down x) * gain; the last ``rotary_dim`` rows, rotated,
    are a key part that all heads share.  Head h's key is [W_uk,h c, rotated part], its value
    W_uv,h c; a query head has ``head_dim`` plain and ``rotary_dim`` rotated channels.
    ``sinks``: a learned number per head whose exponential joins the softmax's denominator."""
    hidden_size: int
    num_heads: int
    head_dim: int                    # unrotated query/key channels of a head
    rotary_dim: int                  # rotated ones (the shared key part's size)
    value_dim: int
    latent_dim: int
    scale: float
    eps: float                       # of the latent's norm
    position: Any                    # a rotary spec over rotary_dim channels
    names: Dict[str, str]            # roles q, down, down_norm, up_k, up_v, o, sinks (optional),
    #                                  q_down, q_down_norm, gate (optional, below)
    window: Optional[int] = None
    kind: str = "latent_attention"
    # queries through a latent of their own: c_q = rms_norm(W_q_down x) * gain (eps as above), q = W_q c_q;
    # ``names["q"]`` is then [heads * (head_dim + rotary_dim), query_latent_dim]
    query_latent_dim: Optional[int] = None
    # names["gate"]: [num_heads, hidden]; head h's output times sigmoid(W_gate x)_h, one number a head
    wide_weights: bool = False       # as AttentionSpec.wide_weights


@dataclass(frozen=True)
class DifferentialAttentionSpec:
    """Two softmax maps per head over the same values, combined as a difference.  A query head's
    row is [map 1 | map 2] of ``head_dim`` each, a key head's likewise; a value head has
    ``value_dim``.  No rotation.  Queries are multiplied by a temperature of their position,
    1 + temp_coef ln(floor((p + 1) / temp_every) + 1) (``temp_every`` 0: none); scores
    (q . k) scale, then cap tanh(s / cap); with lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff the
    head's result is o = a1 - lambda a2, divided by its root mean square (eps, no gain), times
    (1 - diff)."""
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int                    # of one map
    value_dim: int
    scale: float
    softcap: Optional[float]
    window: Optional[int]
    diff: float
    eps: float
    temp_coef: float
    temp_every: int
    names: Dict[str, str]            # roles q, k, v, o, lq1, lk1, lq2, lk2
    kind: str = "differential_attention"
    wide_weights: bool = False       # as AttentionSpec.wide_weights


@dataclass(frozen=True)
class DeltaRuleSpec:
    """A recurrent mixer with a matrix state per head, written by the gated delta rule:
    S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q, with q and k unit vectors (q times
    key_dim^(-1/2)), beta = sigmoid(W_b x), g = exp(-exp(A) softplus(W_a x + dt)); q, k, v pass a
    short causal convolution and silu first; the read-out is divided by its root mean square per
    head, times a gain [value_dim] and silu(W_g x)."""
    hidden_size: int
    num_heads: int                   # value heads
    num_kv_heads: int                # query/key heads; value head h reads head h // (num_heads / num_kv_heads)
    key_dim: int
    value_dim: int
    conv_taps: int
    eps: float
    names: Dict[str, str]            # roles q, k, v, q_conv, k_conv, v_conv, b, a, A_log, dt_bias, norm, gate, o
    kind: str = "delta_rule"


@dataclass(frozen=True)
class LinearAttentionSpec:
    """Gated linear attention: a matrix state per head that decays per key channel,
    S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, with q = W_q x key_dim^(-1/2) and
    alpha = sigmoid(W_a2 (W_a1 x) + b)^(1/tau) (a low-rank projection; decays and state float).
    The read-out is divided by its root mean square per head, times a gain [value_dim] shared by
    the heads and silu(W_g x), then W_o."""
    hidden_size: int
    num_heads: int
    key_dim: int
    value_dim: int
    decay_rank: int                  # rows of W_a1
    tau: float
    eps: float                       # of the read-out's unit RMS
    names: Dict[str, str]            # roles q, k, v, gate, o, norm, a1, a2, a2_bias
    kind: str = "gated_linear_attention"


@dataclass(frozen=True)
class SelectiveScanSpec:
    """A selective scan (Mamba): [u | z] = W_in x; u passes a short causal convolution with bias
    and silu; [dt | B | C] = W_x u; step = softplus(W_dt dt + b) per channel; A = -exp(A_log);
    S[c, n] <- exp(step_c A[c, n]) S[c, n] + step_c u_c B_n;  y_c = sum_n S[c, n] C_n + D_c u_c;
    out = W_o (y silu(z)).  S float [inner, state] per request, beside the convolution's rows."""
    hidden_size: int
    inner: int
    state: int
    dt_rank: int
    conv_taps: int
    names: Dict[str, str]            # roles in, conv, conv_bias, x, dt, dt_bias, A_log, D, o
    kind: str = "selective_scan"


@dataclass(frozen=True)
class SideBySideSpec:
    """Several mixers that read the same input; the result is sum_i scales[i] * mixers[i](x).
    At most one of them keeps pages of keys; their states lie one behind the other."""
    mixers: Tuple[Any, ...]
    scales: Tuple[float, ...]
    kind: str = "side_by_side"


@dataclass(frozen=True)
class MatrixMemorySpec:
    """A recurrent mixer with a matrix state per head (mLSTM): exponential input gate, sigmoid
    forget gate in the log domain, both capped as cap * tanh(x / cap), a running maximum that
    starts at 0; per-head unit RMS of the read-out, a gain, a sigmoid output gate."""
    hidden_size: int
    num_heads: int
    key_dim: int                     # per head, queries and keys
    value_dim: int                   # per head
    gate_cap: float
    eps: float                       # of the read-out's unit RMS
    names: Dict[str, str]            # roles q, k, v, gate, o, norm, i, i_bias, f, f_bias
    kind: str = "mlstm"


@dataclass(frozen=True)
class GatedMLPSpec:
    """act(x Wg^T) * (x Wu^T), then Wd^T."""
    hidden_size: int
    intermediate_size: int
    activation: str                  # "gelu_tanh" | "silu" | "relu" | "clamped_swiglu"
    names: Dict[str, str]            # roles gate, up, down
    kind: str = "gated_mlp"
    # clamped_swiglu: g = min(gate, limit), u = clamp(up, -limit, limit), g sigmoid(1.702 g) (u + 1)
    limit: Optional[float] = None


@dataclass(frozen=True)
class MLPSpec:
    """act(x Wu^T), then Wd^T, without a gate.  ``activation``: "relu2" = max(z, 0)^2."""
    hidden_size: int
    intermediate_size: int
    activation: str
    names: Dict[str, str]            # roles up, down
    kind: str = "mlp"


@dataclass(frozen=True)
class RoutedMLPSpec:
    """A mixture of ``num_experts`` gated layers of which a token uses ``top_k``: scores
    sigmoid(W_router x), the largest chosen, the chosen scores themselves as weights (not
    renormalised).  ``scale_input``: the weight multiplies the expert's input, expert(w x), not its
    output.  ``shared``: a gated layer that every token passes, added to the sum (or None)."""
    hidden_size: int
    intermediate_size: int           # of one expert
    num_experts: int
    top_k: int
    activation: str                  # as GatedMLPSpec's
    limit: Optional[float]
    router: str                      # [num_experts, hidden]
    expert_names: str                # a pattern with {e} and {role}: role is gate, up or down
    shared: Any = None               # a GatedMLPSpec or None
    scale_input: bool = True
    kind: str = "routed_mlp"
    scoring: str = "sigmoid"         # or "softmax": scores exp(z) / sum over all experts
    shared_gate: Optional[str] = None   # [1, hidden]: the shared layer's result times sigmoid(W x), a number a token


@dataclass(frozen=True)
class BlockSpec:
    """One layer: a mixer and a feed-forward joined to the residual stream.

    ``arrangement``:
      "sandwich": h += post_m(mixer(pre_m(h))); h += post_f(ffn(pre_f(h)))
      "prenorm" : h += mixer(pre_m(h));         h += ffn(pre_f(h))
      "parallel": x = pre_m(h);  h += mixer(x) + ffn(x)      (``ffn`` may be None); with a norm
                  ``pre_ffn`` among the norms the feed-forward reads pre_f(h) of the same h instead
    ``norms`` holds the roles pre_mixer, post_mixer, pre_ffn, post_ffn that the
    arrangement uses.  ``residual_scale`` (parallel): h += residual_scale * (mixer + ffn).
    """
    arrangement: str
    mixer: Any
    ffn: Any
    norms: Dict[str, Any]
    kind: str = "block"
    residual_scale: float = 1.0


@dataclass(frozen=True)
class StreamsBlockSpec:
    """One layer over ``streams`` residual streams (hyper-connections).  Sublayer q (1: the
    mixer, 2: the feed-forward, which may be absent) reads u = sum_s in_q[s] x_s, computes
    y = sublayer(norm_q(u)) and writes x_r <- sum_s mix_q[s, r] x_s + out_q[r] y, every stream from
    the old ones.  ``conv``: a short convolution over time between the first norm and the mixer.
    ``streams`` None: one stream and the plain residual sum x <- x + y (no weights)."""
    streams: Optional[int]
    mixer: Any
    ffn: Any                         # None: the layer has no second sublayer
    norms: Dict[str, Any]            # pre_mixer, pre_ffn
    conv: Any                        # ShortConvSpec or None
    names: Dict[str, str]            # in1, out1, mix1, in2, out2, mix2 (absent without streams)
    kind: str = "streams"


@dataclass(frozen=True)
class PairTableSpec:
    """A table of token pairs whose row (previous token * mul_prev + token * mul_cur) mod buckets is
    added to the embedded row; a sequence's first token takes row ``buckets`` (the table's last).
    The previous token is part of a request's state."""
    buckets: int
    mul_prev: int
    mul_cur: int
    weight: str                      # [buckets + 1, hidden]


@dataclass(frozen=True)
class EmbeddingSpec:
    vocab_size: int
    hidden_size: int
    scale: float                     # multiplies the gathered row
    weight: str
    kind: str = "embedding"
    copies: int = 1                  # the row is written this many times (one per residual stream)
    pairs: Optional[PairTableSpec] = None


@dataclass(frozen=True)
class HeadSpec:
    vocab_size: int
    hidden_size: int
    softcap: Optional[float]
    weight: str                      # may equal the embedding's name (tied)
    kind: str = "lm_head"


@dataclass(frozen=True)
class LayerCall:
    """One entry of the execution order.

    ``layer`` indexes ``ModelPlan.layers``.  ``cache_of`` names an earlier
    entry of the order whose cache this call reads instead of keeping its own
    (None: the call owns a cache, if its mixer needs one).
    """
    layer: int
    cache_of: Optional[int] = None
    add_embedding: bool = False      # the embedding's output is added to the stream right before this entry


@dataclass(frozen=True)
class ModelPlan:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_position: int
    embedding: EmbeddingSpec
    layers: Tuple[BlockSpec, ...]
    order: Tuple[LayerCall, ...]
    final_norm: Any
    head: HeadSpec
    ignored_tensors: Tuple[str, ...] = ()   # checkpoint names that may be present and are not used
    # what a checkpoint may or may not put in front of a tensor's name: "model.layers.0..." and
    # "layers.0..." are the same tensor (format/arch/gemma2.py:50-55 accepts both)
    optional_prefixes: Tuple[str, ...] = ("model.",)

    def describe(self) -> List[str]:
        out = []
        for i, call in enumerate(self.order):
            b = self.layers[call.layer]
            win = getattr(b.mixer, "window", None)
            out.append(f"call {i}: layer {call.layer} {getattr(b, 'arrangement', b.kind)} mixer={b.mixer.kind}"
                       f"(window={win}) ffn={getattr(b.ffn, 'kind', None)}"
                       + (f" cache_of={call.cache_of}" if call.cache_of is not None else ""))
        return out

"""A plain, slow Bumolix forward pass over whole sequences (NumPy, no cache, no state carried
between calls).

Test-only oracle: one function per mechanism, written from the design's equations, sharing
nothing with the engine's product path.  It reads config.json keys itself and looks weights up
by their checkpoint names.  Every function takes ``dt`` (``np.float32`` or ``np.float64``) and
carries out all arithmetic in that type.

Notation: T tokens, W the model width, H query heads, G key/value heads, D the query/key size
of a head, E its value size, I the inner channels of the selective scan, N its state size.
"""
from __future__ import annotations

import math

import numpy as np


# ---------------------------------------------------------------- small functions
def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def log_sigmoid(z):
    return -np.logaddexp(0.0, -z)


def unit_rms(x, eps, dt):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    x = x.astype(dt)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + dt(eps))


def rms_norm(x, w, eps, dt):
    """unit_rms(x) * w."""
    return unit_rms(x, eps, dt) * w.astype(dt)


def linear(x, w, name, dt, bias=False):
    y = x @ w[name].astype(dt).T
    return y + w[name + ".b"].astype(dt) if bias else y


# ---------------------------------------------------------------- rotation
def rotary_frequencies(dims, base, factor=1.0):
    """f_i = base^(-2i/dims) / factor, i < dims/2."""
    i = np.arange(dims // 2, dtype=np.float64)
    return np.power(float(base), -2.0 * i / dims) / float(factor)


def rotate_half(x, positions, freqs, dt):
    """Rotate the first 2n channels of the last axis, n = len(freqs); channel i pairs with i + n.
    x: [T, heads, size]."""
    x = x.astype(dt).copy()
    n = len(freqs)
    ang = positions.astype(np.float64)[:, None] * freqs[None, :]
    cs, sn = np.cos(ang).astype(dt)[:, None, :], np.sin(ang).astype(dt)[:, None, :]
    a, b = x[..., :n].copy(), x[..., n:2 * n].copy()
    x[..., :n] = a * cs - b * sn
    x[..., n:2 * n] = b * cs + a * sn
    return x


# ---------------------------------------------------------------- softmax attention in chunks, with a sink
def chunk_mask(positions, size):
    """[T, T] bool: token i sees j iff j <= i and both lie in the same chunk of ``size`` positions
    counted from position 0 (``size`` None: every earlier token)."""
    p = positions.astype(np.int64)
    seen = p[None, :] <= p[:, None]
    if size is not None:
        seen &= (p[None, :] // size) == (p[:, None] // size)
    return seen


def sink_softmax_attention(q, k, v, scale, seen, dt, sink=True):
    """q: [T, H, D], k: [T, G, D], v: [T, G, E] -> [T, H, E]; weights exp(s_j) / (1 + sum exp(s_j)):
    a sink of score 0 that has no value joins the denominator."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]), dt)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h, :] @ k[:, g, :].T) * dt(scale)
        s = np.where(seen, s, -np.inf)
        m = np.maximum(s.max(axis=1, keepdims=True), dt(0.0)) if sink else s.max(axis=1, keepdims=True)
        p = np.exp(s - m)
        den = p.sum(axis=1, keepdims=True) + (np.exp(-m) if sink else 0.0)
        out[:, h, :] = (p / den) @ v[:, g, :]
    return out


def left_mixer(x, positions, w, pre, m, eps, dt):
    """Grouped-query attention: biases on q, k, v; part of a head rotated (frequencies divided by
    a factor); q and k divided by their root mean square per head after the rotation; chunked
    mask; sink softmax; heads times sigmoid(W_g x); W_o."""
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = x.shape[0]
    q = linear(x, w, pre + "q", dt, True).reshape(T, H, D)
    k = linear(x, w, pre + "k", dt, True).reshape(T, G, D)
    v = linear(x, w, pre + "v", dt, True).reshape(T, G, E)
    rot = m.get("rot")
    if rot:
        f = rotary_frequencies(rot["dims"], rot["base"], (rot.get("scaling") or {}).get("factor", 1.0))
        q, k = rotate_half(q, positions, f, dt), rotate_half(k, positions, f, dt)
    q, k = unit_rms(q, eps, dt), unit_rms(k, eps, dt)
    size = (m.get("mask") or {}).get("size")
    o = sink_softmax_attention(q, k, v, m["scale"], chunk_mask(positions, size), dt)
    o = o.reshape(T, H * E) * sigmoid(linear(x, w, pre + "g", dt))
    return linear(o, w, pre + "o", dt)


# ---------------------------------------------------------------- gated linear attention
def decayed_outer_products(q, k, v, alpha, dt):
    """Per head S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, S_0 = 0.
    q, k, alpha: [T, H, D]; v: [T, H, E] -> [T, H, E]."""
    T, H, D = q.shape
    E = v.shape[2]
    S = np.zeros((H, D, E), dt)
    out = np.zeros((T, H, E), dt)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = np.einsum("hde,hd->he", S, q[t])
    return out


def right_mixer(x, w, pre, m, eps, dt):
    H, D, E = m["heads"], m["dim"], m["vdim"]
    T = x.shape[0]
    q = (linear(x, w, pre + "q", dt) * dt(D ** -0.5)).reshape(T, H, D)
    k = linear(x, w, pre + "k", dt).reshape(T, H, D)
    v = linear(x, w, pre + "v", dt).reshape(T, H, E)
    z = linear(linear(x, w, pre + "a1", dt), w, pre + "a2", dt, True).reshape(T, H, D)
    alpha = np.exp(log_sigmoid(z) / dt(m["tau"])).astype(dt)
    o = decayed_outer_products(q, k, v, alpha, dt)
    o = rms_norm(o, w[pre + "norm"], eps, dt).reshape(T, H * E)
    return linear(o * silu(linear(x, w, pre + "g", dt)), w, pre + "o", dt)


def parallel_mixer(x, positions, w, pre, m, eps, dt):
    left = left_mixer(x, positions, w, pre + "left.", m["left"], eps, dt)
    right = right_mixer(x, w, pre + "right.", m["right"], eps, dt)
    return dt(m["left_scale"]) * left + dt(m["right_scale"]) * right


# ---------------------------------------------------------------- selective scan
def causal_conv(x, taps_w, bias, dt):
    """y_t[c] = bias[c] + sum_j w[c, j] x_(t - taps + 1 + j)[c], zeros before the start."""
    T, C = x.shape
    taps = taps_w.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, C), dt), x.astype(dt)], axis=0)
    y = np.tile(bias.astype(dt)[None, :], (T, 1))
    for j in range(taps):
        y = y + padded[j:j + T] * taps_w[:, j].astype(dt)[None, :]
    return y


def selective_scan(x, dt_, A, B, C, D, dt):
    """S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n; y_c = sum_n S[c, n] C_n + D_c x_c."""
    T, I = x.shape
    S = np.zeros((I, A.shape[1]), dt)
    y = np.zeros((T, I), dt)
    for t in range(T):
        S = np.exp(dt_[t][:, None] * A) * S + (dt_[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + D * x[t]
    return y


def mamba_mixer(x, w, pre, m, dt):
    I, N, R = m["inner"], m["state"], m["dt_rank"]
    xz = linear(x, w, pre + "in", dt)
    u, z = xz[:, :I], xz[:, I:]
    u = silu(causal_conv(u, w[pre + "conv"], w[pre + "conv.b"], dt))
    p = linear(u, w, pre + "x", dt)
    step = softplus(linear(p[:, :R], w, pre + "dt", dt, True))
    A = -np.exp(w[pre + "A_log"].astype(dt))
    y = selective_scan(u, step, A, p[:, R:R + N], p[:, R + N:R + 2 * N], w[pre + "D"].astype(dt), dt)
    return linear(y * silu(z), w, pre + "o", dt)


# ---------------------------------------------------------------- feed-forward, layer, model
def dense_ffn(x, w, pre, dt):
    a = np.maximum(linear(x, w, pre + "up", dt), dt(0.0))
    return linear(a * a, w, pre + "down", dt)


def layer(h, positions, w, i, cfg, dt):
    l, eps, pre = cfg["layers"][i], cfg["norm"]["eps"], f"l{i}."
    x1 = rms_norm(h, w[pre + "norm1"], eps, dt)
    if l["type"] == "parallel":
        a = parallel_mixer(x1, positions, w, pre + "mix.", l["mixer"], eps, dt)
    elif l["type"] == "mamba1":
        a = mamba_mixer(x1, w, pre + "mix.", l["mixer"], dt)
    else:
        raise ValueError(l["type"])
    if l.get("mlp") is not None:
        a = a + dense_ffn(rms_norm(h, w[pre + "norm2"], eps, dt), w, pre + "mlp.", dt)
    return h + dt(cfg["residual_mult"]) * a


def forward(cfg, w, tokens, dt=np.float64, keep_layers=False):
    """Logits [T, vocab] of one sequence from position 0 (and the stream after every layer)."""
    tokens = np.asarray(tokens)
    positions = np.arange(len(tokens))
    h = w["embed"].astype(dt)[tokens]
    kept = []
    for i in range(len(cfg["layers"])):
        h = layer(h, positions, w, i, cfg, dt)
        kept.append(h.copy())
    logits = rms_norm(h, w["final.norm"], cfg["norm"]["eps"], dt) @ w["embed"].astype(dt).T
    return (logits, np.stack(kept)) if keep_layers else logits

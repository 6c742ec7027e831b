"""A plain, slow Rotalorn forward pass over whole sequences (NumPy, no cache, no state carried
between calls).

Test-only oracle: one function per mechanism, written from the design's equations, sharing
nothing with the engine's product path.  It reads config.json keys itself and looks weights up
by their checkpoint names.  Every function takes ``dt`` (``np.float32`` or ``np.float64``) and
carries out all arithmetic in that type.

Notation: T tokens, W the model width, H query heads, G key/value heads, D the query/key size
of a head, E its value size, C the size of the key/value latent, R the rotated part of a latent
head, Cq the size of the query latent.
"""
from __future__ import annotations

import math

import numpy as np


# ---------------------------------------------------------------- small functions
def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z * z * z)))


def unit_rms(x, eps, dt):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    x = x.astype(dt)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + dt(eps))


def rms_norm(x, w, eps, dt):
    return unit_rms(x, eps, dt) * w.astype(dt)


def layer_norm(x, w, b, eps, dt):
    """(x - mean) / sqrt(var + eps) * w + b, var the mean of the squared deviations."""
    x = x.astype(dt)
    d = x - x.mean(axis=-1, keepdims=True)
    return d / np.sqrt((d * d).mean(axis=-1, keepdims=True) + dt(eps)) * w.astype(dt) + b.astype(dt)


# ---------------------------------------------------------------- embedding
def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the pair table for every token: (prev * mul_prev + cur * mul_cur) mod buckets, and
    row ``buckets`` (the table's last) for the first token of a sequence."""
    rows = []
    for t, tok in enumerate(tokens):
        rows.append(buckets if t == 0 else (int(tokens[t - 1]) * mul_prev + int(tok) * mul_cur) % buckets)
    return np.array(rows, dtype=np.int64)


def embed(cfg, w, tokens, dt):
    x = w["embed"][np.asarray(tokens)].astype(dt)
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        x = x + w["bigram"][bigram_rows(tokens, bg["buckets"], bg["mul_prev"], bg["mul_cur"])].astype(dt)
    return x


# ---------------------------------------------------------------- rotations
def rotary_frequencies(dims, base, scaling=None):
    """f_i = base^(-2i/dims), i < dims/2.  With ``scaling`` (factor, low, high, original) a
    frequency is judged by its wavelength l = 2 pi / f: shorter than original/high it stays,
    longer than original/low it is divided by the factor, and in between it is
    (1 - s) f / factor + s f with s = (original / l - low) / (high - low)."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            l = 2.0 * math.pi / f
            if l < orig / high:
                pass
            elif l > orig / low:
                f = f / factor
            else:
                s = (orig / l - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return np.array(out, dtype=np.float64)


def rotate_half(x, positions, freqs, dt):
    """Rotate the first 2 n channels of the last axis, n = len(freqs): channel i with channel
    i + n by the angle position * f_i; x: [T, heads, size]."""
    x = x.astype(dt).copy()
    n = len(freqs)
    ang = np.asarray(positions, dtype=np.float64)[:, None] * freqs[None, :]
    cs, sn = np.cos(ang).astype(dt)[:, None, :], np.sin(ang).astype(dt)[:, None, :]
    a, b = x[..., :n].copy(), x[..., n:2 * n].copy()
    x[..., :n] = a * cs - b * sn
    x[..., n:2 * n] = b * cs + a * sn
    return x


# ---------------------------------------------------------------- attention over whole sequences
def visible(T, window):
    """mask[i, j]: j <= i, and i - j < window where there is one."""
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    m = j <= i
    if window:
        m &= (i - j) < window
    return m


def softmax_attention(q, k, v, scale, window, softcap, dt):
    """q [T, H, D], k [T, G, D], v [T, G, E] -> [T, H, E]; query head h reads key/value head
    h // (H / G).  Scores (q . k) scale, optionally cap tanh(s / cap), softmax over visible keys."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]), dtype=dt)
    mask = visible(T, window)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h].astype(dt) @ k[:, g].astype(dt).T) * dt(scale)
        if softcap:
            s = dt(softcap) * np.tanh(s / dt(softcap))
        s = np.where(mask, s, -np.inf)
        p = np.exp(s - s.max(axis=1, keepdims=True))
        p = p / p.sum(axis=1, keepdims=True)
        out[:, h] = p @ v[:, g].astype(dt)
    return out


# ---------------------------------------------------------------- the three mixers
def attention_mixer(mx, w, pre, x, eps, dt):
    """Grouped-query attention whose values are its keys as projected (no value projection):
    biases on q and k, an RMS norm over the whole q row and the whole k row (gain of that size),
    rotary positions on the first rot.dims channels of each head, a window."""
    T = x.shape[0]
    H, G, D = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"]
    q = x @ w[pre + "q"].astype(dt).T + w[pre + "q.b"].astype(dt)
    k = x @ w[pre + "k"].astype(dt).T + w[pre + "k.b"].astype(dt)
    v = k.reshape(T, G, D).copy()
    q = rms_norm(q, w[pre + "q.norm"], eps, dt).reshape(T, H, D)
    k = rms_norm(k, w[pre + "k.norm"], eps, dt).reshape(T, G, D)
    rot = mx.get("rot")
    if rot:
        f = rotary_frequencies(rot.get("dims", D), rot["base"], rot.get("scaling"))
        pos = np.arange(T)
        q, k = rotate_half(q, pos, f, dt), rotate_half(k, pos, f, dt)
    window = (mx.get("mask") or {}).get("size")
    o = softmax_attention(q, k, v, mx["scale"], window, None, dt)
    return o.reshape(T, -1) @ w[pre + "o"].astype(dt).T


def latent_mixer(mx, w, pre, x, eps, dt):
    """Attention over a latent: queries through c_q = rms_norm(W_dq x), q = W_uq c_q, laid out per
    head as [D plain, R rotated]; W_dkv x = [C rows -> rms-normed latent c | R rows -> one rotated
    key part shared by the heads]; head h's key is [W_uk,h c, rotated part], its value W_uv,h c;
    each head's output times sigmoid(W_g x)_h."""
    T = x.shape[0]
    H, D, R, E, C = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
    cq = rms_norm(x @ w[pre + "dq"].astype(dt).T, w[pre + "dq.norm"], eps, dt)
    q = (cq @ w[pre + "uq"].astype(dt).T).reshape(T, H, D + R)
    dkv = x @ w[pre + "dkv"].astype(dt).T
    c = rms_norm(dkv[:, :C], w[pre + "dkv.norm"], eps, dt)
    f = rotary_frequencies(R, mx["rot"]["base"], mx["rot"].get("scaling"))
    pos = np.arange(T)
    kr = rotate_half(dkv[:, None, C:], pos, f, dt)                       # [T, 1, R]
    qr = rotate_half(q[:, :, D:], pos, f, dt)
    kn = (c @ w[pre + "uk"].astype(dt).T).reshape(T, H, D)
    v = (c @ w[pre + "uv"].astype(dt).T).reshape(T, H, E)
    qq = np.concatenate([q[:, :, :D], qr], axis=2)
    kk = np.concatenate([kn, np.repeat(kr, H, axis=1)], axis=2)
    window = (mx.get("mask") or {}).get("size")
    o = softmax_attention(qq, kk, v, mx["scale"], window, None, dt)
    gate = sigmoid(x @ w[pre + "g"].astype(dt).T)                        # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(T, -1) @ w[pre + "o"].astype(dt).T


def query_temperature(positions, coef, every, dt):
    """1 + coef ln(floor((p + 1) / every) + 1)."""
    p = np.asarray(positions, dtype=np.int64)
    return (1.0 + coef * np.log((p + 1) // every + 1.0)).astype(dt)


def differential_lambda(w, pre, diff):
    f = lambda n: w[pre + n].astype(np.float64)
    return math.exp(float((f("lq1") * f("lk1")).sum())) - math.exp(float((f("lq2") * f("lk2")).sum())) + diff


def differential_mixer(mx, w, pre, x, eps, dt):
    """Two softmax maps per head over the same values: q rows per head [map 1 | map 2], k rows
    per key head likewise; no rotation, queries times a temperature of the position, capped
    scores, every earlier key visible; o = a1 - lambda a2, divided by its root mean square per
    head, times (1 - diff)."""
    T = x.shape[0]
    H, G, D, E = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx["vdim"]
    diff = mx["diff"]
    q = (x @ w[pre + "q"].astype(dt).T).reshape(T, H, 2, D)
    k = (x @ w[pre + "k"].astype(dt).T).reshape(T, G, 2, D)
    v = (x @ w[pre + "v"].astype(dt).T).reshape(T, G, E)
    qt = mx.get("q_temp")
    if qt:
        q = q * query_temperature(np.arange(T), qt["coef"], qt["every"], dt)[:, None, None, None]
    window = (mx.get("mask") or {}).get("size")
    a = [softmax_attention(q[:, :, m], k[:, :, m], v, mx["scale"], window, mx.get("softcap"), dt) for m in (0, 1)]
    lam = dt(differential_lambda(w, pre, diff))
    o = unit_rms(a[0] - lam * a[1], eps, dt) * dt(1.0 - diff)
    return o.reshape(T, -1) @ w[pre + "o"].astype(dt).T


MIXERS = {"attention": attention_mixer, "latent_attention": latent_mixer, "attention_2": differential_mixer}


# ---------------------------------------------------------------- feed-forward
def gated(x, w, pre, act, dt):
    return (act(x @ w[pre + "gate"].astype(dt).T) * (x @ w[pre + "up"].astype(dt).T)) @ w[pre + "down"].astype(dt).T


def route(x, w_router, top, dt):
    """softmax over all experts of the router's logits; the ``top`` largest (the lower index among
    equals), their scores as weights, not renormalised.  Returns ids [T, top], weights [T, top]
    and each token's margin between the logits of the last chosen and the first left-out expert."""
    z = x.astype(np.float32).astype(dt) @ w_router.astype(dt).T
    s = np.exp(z - z.max(axis=1, keepdims=True))
    s = s / s.sum(axis=1, keepdims=True)
    order = np.argsort(-s, axis=1, kind="stable")
    ids = order[:, :top]
    srt = np.take_along_axis(z, order, axis=1)              # the margin is taken between logits
    margin = srt[:, top - 1] - srt[:, top] if s.shape[1] > top else np.full(len(s), np.inf)
    return ids, np.take_along_axis(s, ids, axis=1), margin


def mixture(ml, w, pre, x, dt, margins=None):
    """sum over the chosen experts of score * expert(x), experts silu-gated; plus the shared
    expert times sigmoid(W_sg x) (one number a token)."""
    ids, wts, margin = route(x, w[pre + "router"], ml["router"]["top"], dt)
    if margins is not None:
        margins.append(margin)
    out = np.zeros_like(x, dtype=dt)
    for t in range(x.shape[0]):
        for e, s in zip(ids[t], wts[t]):
            out[t] += s * gated(x[t:t + 1], w, f"{pre}e{e}.", silu, dt)[0]
    if ml.get("shared"):
        out += gated(x, w, pre + "shared.", silu, dt) * sigmoid(x @ w[pre + "shared.sg"].astype(dt).T)
    return out


def feed_forward(ml, w, pre, x, dt, margins=None):
    if ml["kind"] == "dense":
        return gated(x, w, pre, gelu_tanh, dt)
    return mixture(ml, w, pre, x, dt, margins)


# ---------------------------------------------------------------- the model
def forward(cfg, w, tokens, dt=np.float64, layers_out=None, margins=None):
    """Logits [T, vocab] of one sequence.  ``layers_out``: a list that receives the stream after
    every layer; ``margins``: a list that receives each routed layer's per-token margins."""
    eps = cfg["norm"]["eps"]
    x = embed(cfg, w, tokens, dt)
    for i, l in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps, dt)
        y = MIXERS[l["type"]](l["mixer"], w, p + "mix.", h, eps, dt)
        if l.get("mlp"):
            y = y + feed_forward(l["mlp"], w, p + "mlp.", h, dt, margins)
        x = x + y
        if layers_out is not None:
            layers_out.append(x.copy())
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps, dt)
    return x @ w["embed"].astype(dt).T

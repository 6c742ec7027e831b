"""Small Bumolix models for tests: configurations, random weights written as model folders."""
import numpy as np

from dafotar_util import write_model  # noqa: F401  (a folder with config.json and model.safetensors)


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def left(heads=4, kv_heads=2, dim=16, vdim=24, chunk=12, rot_dims=8, base=500.0, factor=4.0, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else 0.5}
    if chunk is not None:
        m["mask"] = {"size": chunk}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
        if factor is not None:
            m["rot"]["scaling"] = {"factor": factor}
    return m


def right(heads=3, dim=8, vdim=12, tau=4.0, rank=6):
    """``rank`` is no key of the format (the tensors say it); a model of random weights made on
    the device, which has no tensors to read it from, takes it from here."""
    return {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "rank": rank}


def parallel_layer(l=None, r=None, left_scale=0.8, right_scale=1.3, mlp=None):
    return {"type": "parallel", "mixer": {"left": l or left(), "right": r or right(), "left_scale": left_scale,
                                          "right_scale": right_scale}, "mlp": mlp}


def scan_layer(inner=24, state=6, dt_rank=5, conv=3, mlp=None):
    return {"type": "mamba1", "mixer": {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}, "mlp": mlp}


def config(layers, vocab=96, width=32, eps=1e-5, mult=0.5):
    return {"architecture": "Bumolix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
            "layers": layers}


# Three configurations that differ in every size and option.  A: both kinds of layer, values
# wider and narrower than keys, part of a head rotated with divided frequencies, a chunk that is
# no multiple of a page, a layer without feed-forward, an odd rank of the decays.  B: the scan
# first, one key head per query head, a whole head rotated without a factor, sizes that the
# matrix-core kernels take, two taps, scales of one, a multiplier of one.  C: a width that is no
# multiple of eight, one head everywhere, one tap, no rotation at all on one layer and no mask
# on another, a state of one value a channel.
CFG_A = config([
    parallel_layer(left(4, 2, 16, 24, chunk=12, rot_dims=8, base=500.0, factor=4.0, scale=0.4), right(3, 8, 12, 4.0, 6),
                   0.8, 1.3, dense(40)),
    scan_layer(24, 6, 5, 3, dense(56)),
    parallel_layer(left(6, 2, 8, 8, chunk=7, rot_dims=8, base=100.0, factor=1.5, scale=0.7), right(2, 20, 10, 16.0, 3),
                   1.4, 0.6, None),
    scan_layer(40, 17, 3, 4, None),
], vocab=200, width=48, eps=1e-5, mult=0.4)
CFG_B = config([
    scan_layer(64, 16, 8, 2, dense(64)),
    parallel_layer(left(2, 2, 32, 32, chunk=32, rot_dims=32, base=2000.0, factor=None, scale=0.18), right(2, 32, 32, 1.0, 8),
                   1.0, 1.0, dense(48)),
    parallel_layer(left(4, 1, 64, 64, chunk=48, rot_dims=16, base=10000.0, factor=2.0, scale=0.125), right(1, 64, 64, 8.0, 16),
                   0.5, 2.0, dense(32)),
], vocab=131, width=64, eps=1e-6, mult=1.0)
CFG_C = config([
    parallel_layer(left(1, 1, 10, 6, chunk=5, rot_dims=0, scale=0.9), right(1, 12, 70, 2.0, 1), 1.1, 0.9, dense(20)),
    scan_layer(9, 1, 1, 1, dense(12)),
    parallel_layer(left(3, 3, 12, 20, chunk=None, rot_dims=4, base=10.0, factor=3.0, scale=0.3), right(5, 4, 4, 3.0, 2),
                   0.7, 0.7, None),
], vocab=64, width=36, eps=1e-6, mult=0.25)


def tensor_shapes(cfg):
    W = cfg["width"]
    out = {"embed": (cfg["vocab"], W), "final.norm": (W,)}
    for i, l in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", l["mixer"]
        out[p + "norm1"] = (W,)
        m = p + "mix."
        if l["type"] == "parallel":
            a, g = mx["left"], mx["right"]
            H, G, D, E = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            n = m + "left."
            out.update({n + "q": (H * D, W), n + "q.b": (H * D,), n + "k": (G * D, W), n + "k.b": (G * D,),
                        n + "v": (G * E, W), n + "v.b": (G * E,), n + "g": (H * E, W), n + "o": (W, H * E)})
            H, D, E, R = g["heads"], g["dim"], g["vdim"], g["rank"]
            n = m + "right."
            out.update({n + "q": (H * D, W), n + "k": (H * D, W), n + "v": (H * E, W), n + "g": (H * E, W),
                        n + "o": (W, H * E), n + "norm": (E,), n + "a1": (R, W), n + "a2": (H * D, R), n + "a2.b": (H * D,)})
        else:
            I, N, R, taps = mx["inner"], mx["state"], mx["dt_rank"], mx["conv"]
            out.update({m + "in": (2 * I, W), m + "conv": (I, taps), m + "conv.b": (I,), m + "x": (R + 2 * N, I),
                        m + "dt": (I, R), m + "dt.b": (I,), m + "A_log": (I, N), m + "D": (I,), m + "o": (W, I)})
        if l["mlp"]:
            ff = l["mlp"]["ff"]
            out[p + "norm2"] = (W,)
            out.update({p + "mlp.up": (ff, W), p + "mlp.down": (W, ff)})
    return out


def random_weights(cfg, seed, sharp=1.0):
    """float32 arrays, already rounded to bfloat16 values so that either storage type holds the
    same numbers.  ``sharp`` widens the left mixer's query and key projections: scores far
    apart, a softmax close to a choice of one key."""
    from zse_amd.weights.safetensors import bf16_bits_to_f32, f32_to_bf16_bits
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.split(".")[-1]
        if name == "embed":
            a = rng.normal(0, 0.7, shape)
        elif last in ("norm1", "norm2", "norm") :
            a = 1.0 + rng.normal(0, 0.2, shape)
        elif name.endswith("a2.b"):
            a = rng.normal(2.0, 1.0, shape)                   # decays mostly near one, some well below
        elif name.endswith("dt.b"):
            a = rng.normal(-1.0, 1.0, shape)
        elif last == "b" and len(shape) == 1:
            a = rng.normal(0, 0.3, shape)
        elif last == "conv":
            a = rng.normal(0, 0.6, shape)
        elif last == "A_log":
            a = rng.normal(-0.5, 0.8, shape)
        elif last == "D":
            a = rng.normal(0, 1.0, shape)
        elif name.endswith("left.q") or name.endswith("left.k"):
            a = rng.normal(0, sharp / np.sqrt(shape[-1]), shape)
        elif last == "up":
            a = rng.normal(0, 1.5 / np.sqrt(shape[-1]), shape)
        else:
            a = rng.normal(0, 1.0 / np.sqrt(shape[-1]), shape)
        out[name] = bf16_bits_to_f32(f32_to_bf16_bits(a.astype(np.float32)))
    return out

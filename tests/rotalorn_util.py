"""Small Rotalorn models for tests: configurations, random weights written as model folders."""
import numpy as np

from dafotar_util import write_model  # noqa: F401  (a folder with config.json and model.safetensors)


def dense(ff=48):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, top=2, ff=24, shared_ff=40):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    m["shared"] = {"ff": shared_ff} if shared_ff else None
    return m


def attention_layer(heads=4, kv_heads=2, dim=24, rot_dims=12, base=500.0, scaling=None, scale=None, window=20, mlp=None):
    rot = {"base": base, "dims": rot_dims}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale if scale is not None else dim ** -0.5,
          "rot": rot}
    if window:
        mx["mask"] = {"size": window}
    return {"type": "attention", "mixer": mx, "mlp": mlp}


def latent_layer(heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=20, q_rank=16, base=3000.0, scale=None, window=13, mlp=None):
    mx = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
          "scale": scale if scale is not None else (dim + rot_dim) ** -0.5, "rot": {"base": base, "dims": rot_dim}}
    if window:
        mx["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": mx, "mlp": mlp}


def diff_layer(heads=4, kv_heads=2, dim=12, vdim=24, diff=0.4, softcap=15.0, q_temp=(0.5, 16), scale=None, mlp=None):
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff,
          "scale": scale if scale is not None else dim ** -0.5}
    if softcap:
        mx["softcap"] = softcap
    if q_temp:
        mx["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return {"type": "attention_2", "mixer": mx, "mlp": mlp}


def config(layers, vocab=96, width=32, eps=1e-5, bigram=(61, 7, 3)):
    cfg = {"architecture": "Rotalorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if bigram is not None:
        cfg["embedding"] = {"bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), bigram))}
    return cfg


# Three configurations that differ in every size and option.  A: every kind of layer and both
# feed-forwards, part of a head rotated with scaled frequencies, windows that are no multiple of a
# page, two of five experts.  B: sizes that the matrix-core kernels take (heads of 64 and 32,
# width 64), as many key heads as query heads, a whole head rotated, one expert of three and no
# shared expert, a layer without feed-forward, a latent layer without window, no pair table,
# no temperature and no cap.  C: a width that is no multiple of eight, one head everywhere, every
# expert chosen, window 1 and window 2, a temperature that changes at every position, multipliers
# of 1, one bucket.
CFG_A = config([
    latent_layer(heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=20, q_rank=16, base=3000.0, window=13, mlp=dense(40)),
    diff_layer(heads=4, kv_heads=2, dim=12, vdim=24, diff=0.4, softcap=15.0, q_temp=(0.5, 16), mlp=moe(5, 2, 24, 40)),
    attention_layer(heads=4, kv_heads=2, dim=24, rot_dims=12, base=500.0, scaling=(6.0, 1.0, 3.0, 64), scale=0.3, window=21,
                    mlp=moe(4, 3, 16, 24)),
    diff_layer(heads=2, kv_heads=2, dim=8, vdim=8, diff=0.7, softcap=None, q_temp=(1.5, 5), mlp=dense(56)),
], vocab=200, width=48, eps=1e-5, bigram=(61, 7, 3))
CFG_B = config([
    attention_layer(heads=2, kv_heads=2, dim=64, rot_dims=64, base=2000.0, window=24, mlp=moe(3, 1, 40, None)),
    latent_layer(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=56, q_rank=24, base=100.0, scale=0.2, window=None, mlp=None),
    diff_layer(heads=2, kv_heads=1, dim=32, vdim=32, diff=0.2, softcap=None, q_temp=None, mlp=dense(128)),
    attention_layer(heads=4, kv_heads=1, dim=32, rot_dims=16, base=50.0, scaling=(4.0, 1.0, 2.0, 32), window=None, mlp=dense(64)),
], vocab=131, width=64, eps=1e-6, bigram=None)
CFG_C = config([
    diff_layer(heads=1, kv_heads=1, dim=10, vdim=6, diff=0.5, softcap=2.0, q_temp=(2.0, 1), mlp=moe(2, 2, 12, 12)),
    attention_layer(heads=1, kv_heads=1, dim=10, rot_dims=4, base=10.0, scaling=(2.0, 1.0, 4.0, 16), window=1, mlp=None),
    latent_layer(heads=1, dim=12, rot_dim=2, vdim=20, kv_rank=9, q_rank=5, base=50.0, window=2, mlp=moe(3, 2, 20, None)),
], vocab=64, width=36, eps=1e-6, bigram=(1, 1, 1))


def tensor_shapes(cfg):
    W = cfg["width"]
    out = {"embed": (cfg["vocab"], W), "final.norm": (W,), "final.norm.b": (W,)}
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        out["bigram"] = (bg["buckets"] + 1, W)
    for i, l in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", l["mixer"]
        H, D, E = mx["heads"], mx["dim"], mx["vdim"]
        out[p + "norm1"] = (W,)
        out[p + "norm1.b"] = (W,)
        m = p + "mix."
        if l["type"] == "attention":
            G = mx.get("kv_heads", H)
            out.update({m + "q": (H * D, W), m + "q.b": (H * D,), m + "k": (G * D, W), m + "k.b": (G * D,),
                        m + "q.norm": (H * D,), m + "k.norm": (G * D,), m + "o": (W, H * E)})
        elif l["type"] == "latent_attention":
            R, C, Cq = mx["rot_dim"], mx["kv_rank"], mx["q_rank"]
            out.update({m + "dq": (Cq, W), m + "dq.norm": (Cq,), m + "uq": (H * (D + R), Cq), m + "dkv": (C + R, W),
                        m + "dkv.norm": (C,), m + "uk": (H * D, C), m + "uv": (H * E, C), m + "g": (H, W),
                        m + "o": (W, H * E)})
        else:
            G = mx.get("kv_heads", H)
            out.update({m + "q": (H * 2 * D, W), m + "k": (G * 2 * D, W), m + "v": (G * E, W), m + "o": (W, H * E),
                        m + "lq1": (D,), m + "lk1": (D,), m + "lq2": (D,), m + "lk2": (D,)})
        ml = l["mlp"]
        f = p + "mlp."
        if ml and ml["kind"] == "dense":
            out.update({f + "gate": (ml["ff"], W), f + "up": (ml["ff"], W), f + "down": (W, ml["ff"])})
        elif ml:
            out[f + "router"] = (ml["router"]["experts"], W)
            for e in range(ml["router"]["experts"]):
                ff = ml["expert"]["ff"]
                out.update({f"{f}e{e}.gate": (ff, W), f"{f}e{e}.up": (ff, W), f"{f}e{e}.down": (W, ff)})
            if ml.get("shared"):
                ff = ml["shared"]["ff"]
                out.update({f + "shared.gate": (ff, W), f + "shared.up": (ff, W), f + "shared.down": (W, ff),
                            f + "shared.sg": (1, W)})
    return out


def random_weights(cfg, seed, sharp=1.0):
    """float32 arrays, already rounded to bfloat16 values so that either storage type holds the
    same numbers.  ``sharp`` widens the query projections: scores far apart, a softmax close to a
    choice of one key."""
    from zse_amd.weights.safetensors import bf16_bits_to_f32, f32_to_bf16_bits
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.split(".")[-1]
        if name == "embed":
            a = rng.normal(0, 0.7, shape)
        elif name == "bigram":
            a = rng.normal(0, 0.5, shape)
        elif last == "norm1" or name == "final.norm" or last == "norm":
            a = 1.0 + rng.normal(0, 0.2, shape)
        elif last == "b":
            a = rng.normal(0, 0.3, shape)
        elif last in ("lq1", "lk1", "lq2", "lk2"):
            a = rng.normal(0, 0.3, shape)
        elif last == "router":
            a = rng.normal(0, 3.0 / np.sqrt(shape[-1]), shape)
        elif name.endswith("mix.q") or name.endswith("mix.uq"):
            a = rng.normal(0, sharp / np.sqrt(shape[-1]), shape)
        elif last in ("gate", "up"):
            a = rng.normal(0, 1.5 / np.sqrt(shape[-1]), shape)
        else:
            a = rng.normal(0, 1.0 / np.sqrt(shape[-1]), shape)
        out[name] = bf16_bits_to_f32(f32_to_bf16_bits(a.astype(np.float32)))
    return out

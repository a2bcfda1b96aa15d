"""Small Pubunex models for tests: configurations, random weights written as model folders."""
import numpy as np

from dafotar_util import write_model  # noqa: F401  (a folder with config.json and model.safetensors)


def moe(experts=5, top=2, ff=24, limit=1.5, shared_ff=40, shared_limit=2.5):
    m = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
    m["shared"] = {"ff": shared_ff, "limit": shared_limit} if shared_ff else None
    return m


def delta_layer(heads=4, kv_heads=2, dim=16, vdim=24, conv=3, mlp=None):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": mlp}


def attention_layer(heads=4, kv_heads=2, dim=24, vdim=16, rot_dims=12, base=500.0, scaling=None, scale=None, mlp=None):
    rot = {"base": base, "dims": rot_dims}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                           "scale": scale if scale is not None else dim ** -0.5, "rot": rot}, "mlp": mlp}


def latent_layer(heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=20, base=3000.0, scale=None, mlp=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
                      "scale": scale if scale is not None else (dim + rot_dim) ** -0.5,
                      "rot": {"base": base, "dims": rot_dim}}, "mlp": mlp}


def config(layers, vocab=96, width=32, eps=1e-5, loop=None):
    cfg = {"architecture": "Pubunex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if loop is not None:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


# Three configurations that differ in every size and option.  A: every kind of layer, fewer
# query/key heads than value heads in the delta rule, values wider and narrower than keys,
# part of a head rotated with scaled frequencies, two of five experts, the first two layers
# twice.  B: no loop, a layer without feed-forward, one expert of three and no shared layer,
# as many key heads as query heads, a whole head rotated, sizes that the matrix-core attention
# takes, two taps.  C: a width that is no multiple of eight, every expert chosen, one tap,
# one head, the middle layer three times.
CFG_A = config([
    delta_layer(heads=4, kv_heads=2, dim=16, vdim=24, conv=3, mlp=moe(5, 2, 24, 1.5, 40, 2.5)),
    attention_layer(heads=4, kv_heads=2, dim=24, vdim=16, rot_dims=12, base=500.0, scaling=(8.0, 64, 16.0, 2.0), scale=0.3,
                    mlp=moe(4, 3, 16, 3.0, 24, 1.0)),
    latent_layer(heads=3, dim=8, rot_dim=4, vdim=12, kv_rank=20, base=3000.0, mlp=moe(6, 2, 32, 2.0, None)),
    delta_layer(heads=2, kv_heads=2, dim=24, vdim=8, conv=4, mlp=moe(5, 1, 24, 1.0, 16, 4.0)),
], vocab=200, width=48, eps=1e-5, loop=(0, 2, 2))
CFG_B = config([
    attention_layer(heads=2, kv_heads=2, dim=32, vdim=32, rot_dims=32, base=2000.0, mlp=moe(3, 1, 40, 2.5, None)),
    delta_layer(heads=3, kv_heads=3, dim=32, vdim=8, conv=2, mlp=None),
    latent_layer(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=24, base=100.0, scale=0.2, mlp=moe(8, 4, 16, 1.5, 56, 1.5)),
], vocab=131, width=40, eps=1e-6)
CFG_C = config([
    latent_layer(heads=1, dim=12, rot_dim=2, vdim=20, kv_rank=9, base=50.0, mlp=moe(2, 2, 12, 2.0, 12, 2.0)),
    delta_layer(heads=1, kv_heads=1, dim=12, vdim=70, conv=1, mlp=moe(3, 2, 20, 0.75, None)),
    attention_layer(heads=1, kv_heads=1, dim=10, vdim=6, rot_dims=4, base=10.0, scaling=(2.0, 16, 4.0, 1.0), mlp=None),
], vocab=64, width=36, eps=1e-6, loop=(1, 2, 3))


def tensor_shapes(cfg):
    W = cfg["width"]
    out = {"embed": (cfg["vocab"], W), "head": (cfg["vocab"], W), "final.norm": (W,)}
    for i, l in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", l["mixer"]
        H, D, E = mx["heads"], mx["dim"], mx["vdim"]
        out[p + "norm1"] = (W,)
        m = p + "mix."
        if l["type"] == "delta":
            G, taps = mx["kv_heads"], mx["conv"]
            out.update({m + "q": (G * D, W), m + "k": (G * D, W), m + "v": (H * E, W), m + "g": (H * E, W),
                        m + "q.conv": (G * D, taps), m + "k.conv": (G * D, taps), m + "v.conv": (H * E, taps),
                        m + "b": (H, W), m + "a": (H, W), m + "A_log": (H,), m + "dt_bias": (H,), m + "norm": (E,),
                        m + "o": (W, H * E)})
        elif l["type"] == "attention":
            G = mx["kv_heads"]
            out.update({m + "q": (H * D, W), m + "q.b": (H * D,), m + "k": (G * D, W), m + "k.b": (G * D,),
                        m + "v": (G * E, W), m + "v.b": (G * E,), m + "o": (W, H * E), m + "o.b": (W,)})
        else:
            R, C = mx["rot_dim"], mx["kv_rank"]
            out.update({m + "q": (H * (D + R), W), m + "dkv": (C + R, W), m + "dkv.norm": (C,), m + "uk": (H * D, C),
                        m + "uv": (H * E, C), m + "sink": (H,), m + "o": (W, H * E)})
        if l["mlp"]:
            ml, f = l["mlp"], p + "mlp."
            out[f + "router"] = (ml["router"]["experts"], W)
            for e in range(ml["router"]["experts"]):
                ff = ml["expert"]["ff"]
                out.update({f"{f}e{e}.gate": (ff, W), f"{f}e{e}.up": (ff, W), f"{f}e{e}.down": (W, ff)})
            if ml.get("shared"):
                ff = ml["shared"]["ff"]
                out.update({f + "shared.gate": (ff, W), f + "shared.up": (ff, W), f + "shared.down": (W, ff)})
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
        elif last == "norm1" or name == "final.norm":
            a = rng.normal(0, 0.2, shape)                     # the gain is 1 + w
        elif name.endswith("mix.norm") or name.endswith("dkv.norm"):
            a = 1.0 + rng.normal(0, 0.2, shape)
        elif last == "b" and len(shape) == 1:
            a = rng.normal(0, 0.3, shape)
        elif last == "conv":
            a = rng.normal(0, 0.6, shape)
        elif last in ("A_log", "dt_bias"):
            a = rng.normal(0, 0.7, shape)
        elif last == "sink":
            a = rng.normal(0.5, 1.5, shape)
        elif last == "router":
            a = rng.normal(0, 3.0 / np.sqrt(shape[-1]), shape)
        elif name.endswith("mix.q"):
            a = rng.normal(0, sharp / np.sqrt(shape[-1]), shape)
        elif last in ("gate", "up"):
            a = rng.normal(0, 2.0 / np.sqrt(shape[-1]), shape)     # wide enough for the clamps to bite
        else:
            a = rng.normal(0, 1.0 / np.sqrt(shape[-1]), shape)
        out[name] = bf16_bits_to_f32(f32_to_bf16_bits(a.astype(np.float32)))
    return out

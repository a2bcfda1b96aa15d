"""Small Dafotar models for tests: configurations, random weights written as model folders."""
import json
import os

import numpy as np


def attention_layer(heads=4, kv_heads=2, dim=16, vdim=16, window=12, rot_dims=None, base=1000.0, scale=None,
                    ff=None, kv_from=None):
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if window is not None:
        mx["mask"] = {"size": window}
    if base is not None:
        mx["rot"] = {"base": base, "dims": rot_dims if rot_dims is not None else dim}
    if kv_from is not None:
        mx["kv_from"] = kv_from
    return {"type": "attention", "mixer": mx, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def mlstm_layer(heads=2, dim=8, vdim=16, cap=10.0, ff=None):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, vocab=96, width=32, streams=3, taps=3, eps=1e-5):
    cfg = {"architecture": "Dafotar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if streams is not None:
        cfg["streams"] = streams
    if taps is not None:
        cfg["canon"] = {"taps": taps}
    return cfg


# Two configurations that differ in every size and option: A has every kind of layer, values
# wider and narrower than keys, part of a head rotated, a layer that reads another's keys
# through a wider window; B has no streams, no convolution, no mask, as many key heads as
# query heads, one residual, odd sizes.
CFG_A = config([
    mlstm_layer(heads=2, dim=8, vdim=16, cap=6.0, ff=48),
    attention_layer(heads=4, kv_heads=2, dim=24, vdim=16, window=20, rot_dims=12, base=500.0, scale=0.3),
    attention_layer(heads=4, kv_heads=2, dim=24, vdim=16, window=33, rot_dims=12, base=500.0, scale=0.25, ff=80, kv_from=1),
    mlstm_layer(heads=1, dim=16, vdim=8, cap=12.0),
    attention_layer(heads=2, kv_heads=1, dim=8, vdim=40, window=7, base=10000.0, ff=40),
], vocab=200, width=48, streams=3, taps=3, eps=1e-5)
CFG_B = config([
    attention_layer(heads=3, kv_heads=3, dim=20, vdim=12, window=None, base=2000.0, ff=56),
    mlstm_layer(heads=3, dim=12, vdim=20, cap=15.0, ff=56),
    attention_layer(heads=3, kv_heads=3, dim=20, vdim=12, window=None, base=None, ff=None),
], vocab=131, width=40, streams=None, taps=None, eps=1e-6)
CFG_C = config([
    attention_layer(heads=2, kv_heads=1, dim=16, vdim=16, window=1, base=100.0, ff=32),
    mlstm_layer(heads=2, dim=16, vdim=16, cap=3.0),
    attention_layer(heads=2, kv_heads=1, dim=16, vdim=16, window=9, base=100.0, kv_from=0),
], vocab=64, width=32, streams=1, taps=2, eps=1e-6)


def tensor_shapes(cfg):
    W, S = cfg["width"], cfg.get("streams")
    taps = (cfg.get("canon") or {}).get("taps")
    out = {"embed": (cfg["vocab"], W), "final.norm": (W,), "final.norm.b": (W,)}
    for i, l in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", l["mixer"]
        H, D, E = mx["heads"], mx["dim"], mx["vdim"]
        subs = (1, 2) if l["mlp"] else (1,)
        for q in subs:
            out[f"{p}norm{q}"] = (W,)
            out[f"{p}norm{q}.b"] = (W,)
            if S is not None:
                out[f"{p}hc{q}.in"], out[f"{p}hc{q}.out"], out[f"{p}hc{q}.mix"] = (S,), (S,), (S, S)
        if taps is not None:
            out[p + "canon1"] = (W, taps)
        if l["type"] == "attention":
            G = mx["kv_heads"]
            out[p + "mix.q"], out[p + "mix.o"] = (H * D, W), (W, H * E)
            out[p + "mix.q.norm"], out[p + "mix.temp"] = (D,), (H,)
            if "kv_from" not in mx:
                out[p + "mix.k"], out[p + "mix.v"], out[p + "mix.k.norm"] = (G * D, W), (G * E, W), (D,)
        else:
            out[p + "mix.q"], out[p + "mix.k"] = (H * D, W), (H * D, W)
            out[p + "mix.v"], out[p + "mix.g"] = (H * E, W), (H * E, W)
            out[p + "mix.o"], out[p + "mix.norm"] = (W, H * E), (H * E,)
            out[p + "mix.i"], out[p + "mix.f"] = (H, W), (H, W)
            out[p + "mix.i.b"], out[p + "mix.f.b"] = (H,), (H,)
        if l["mlp"]:
            ff = l["mlp"]["ff"]
            out[p + "mlp.gate"], out[p + "mlp.up"], out[p + "mlp.down"] = (ff, W), (ff, W), (W, ff)
    return out


def random_weights(cfg, seed, temp=1.0):
    """float32 arrays, already rounded to bfloat16 values so that either storage type holds
    the same numbers.  Gains near 1, biases small, stream weights near the plain residual."""
    from zse_amd.weights.safetensors import bf16_bits_to_f32, f32_to_bf16_bits
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.split(".")[-1]
        if name == "embed":
            a = rng.normal(0, 0.5, shape)
        elif last in ("norm1", "norm2") or name in ("final.norm",) or name.endswith("mix.norm") or \
                name.endswith("q.norm") or name.endswith("k.norm"):
            a = 1.0 + rng.normal(0, 0.2, shape)
        elif last == "b":
            a = rng.normal(0, 0.2, shape)
        elif last == "temp":
            a = temp * (1.0 + rng.normal(0, 0.2, shape))
        elif last == "canon1":
            a = rng.normal(0, 0.4, shape)
        elif last == "in":
            a = rng.normal(1.0 / shape[0], 0.2, shape)
        elif last == "out":
            a = rng.normal(1.0, 0.3, shape)
        elif last == "mix" and len(shape) == 2 and ".hc" in name:
            a = np.eye(shape[0]) + rng.normal(0, 0.2, shape)
        else:
            a = rng.normal(0, 1.0 / np.sqrt(shape[-1]), shape)
        out[name] = bf16_bits_to_f32(f32_to_bf16_bits(a.astype(np.float32)))
    return out


def write_model(folder, cfg, weights, dtype="bfloat16"):
    from zse_amd.weights import safetensors as st
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    if dtype == "bfloat16":
        packed = {n: ("BF16", st.f32_to_bf16_bits(a)) for n, a in weights.items()}
    else:
        packed = {n: ("F32", a.astype(np.float32)) for n, a in weights.items()}
    st.write_file(os.path.join(folder, "model.safetensors"), packed, metadata={"format": "pt"})
    return folder

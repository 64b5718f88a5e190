"""Small random Mepatar checkpoints for the tests: a config dict and a name -> tensor dict in the checkpoint's naming, optionally written to a folder
(config.json + model.safetensors) so the tests go through the registry and the loader like a user does."""

import json
import os

import torch


def retention(heads=3, dim=24, vdim=40, decay=None, rot_dims=None, base=10000.0):
    decay = decay or [1.0 - 2.0 ** (-3 - 1.5 * i) for i in range(heads)]
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay, "rot": {"dims": dim if rot_dims is None else rot_dims, "base": base}}}


def attention(heads=4, kv_heads=2, dim=24, vdim=40, size=20, keep_first=3, rot_dims=16, base=5000.0, scale=None):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": size, "keep_first": keep_first},
                                           "rot": {"dims": rot_dims, "base": base}, "scale": dim ** -0.5 if scale is None else scale}}


def delta(heads=4, kv_heads=2, dim=24, vdim=40, conv=4):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def dense(ff=88):
    return {"kind": "dense", "ff": ff}


def moe(experts=12, top=3, ff=40, limit=1.0):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def make_config(layers, width=72, vocab=131, eps=1e-5, groups=3, taps=3, embed_scale=1.7):
    """layers: list of (mixer entry, mlp entry or None)."""
    out = []
    for mixer, mlp in layers:
        e = dict(mixer)
        e["mlp"] = mlp
        out.append(e)
    return {"architecture": "Mepatar", "vocab": vocab, "width": width, "norm": {"eps": eps, "groups": groups}, "canon": {"taps": taps},
            "embedding": {"scale": embed_scale}, "layers": out}


def make_weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def lin(o, i, gain=1.0):
        return (torch.randn(o, i, generator=g) * gain / i ** 0.5).to(torch.bfloat16)

    def vec(n, mean=1.0, std=0.1):
        return (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)

    w = {"embed": torch.randn(cfg["vocab"], W, generator=g).to(torch.bfloat16), "head": lin(cfg["vocab"], W), "final.norm": vec(W)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        w[p + "norm1"] = vec(W)
        w[p + "canon1"] = (0.3 * torch.randn(W, cfg["canon"]["taps"], generator=g)).to(torch.bfloat16)
        x = p + "mix."
        if layer["type"] == "retention":
            H, dk, dv = m["heads"], m["dim"], m["vdim"]
            w[x + "q"], w[x + "k"], w[x + "v"], w[x + "g"] = lin(H * dk, W, 2.0), lin(H * dk, W, 2.0), lin(H * dv, W), lin(H * dv, W, 2.0)
            w[x + "o"] = lin(W, H * dv)
        elif layer["type"] == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for n, o in (("q", H * d), ("k", G * d), ("v", G * dv)):
                w[x + n], w[x + n + ".b"] = lin(o, W, 2.0), vec(o, 0.0, 0.3)
            w[x + "q.norm"], w[x + "k.norm"] = vec(d, 1.5, 0.3), vec(d, 1.5, 0.3)
            w[x + "temp"] = vec(H, 1.2, 0.4)
            w[x + "o"], w[x + "o.b"] = lin(W, H * dv), vec(W, 0.0, 0.2)
        else:
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for n, o in (("q", G * dk), ("k", G * dk), ("v", H * dv)):
                w[x + n], w[x + n + ".conv"] = lin(o, W, 2.0), (0.5 * torch.randn(o, m["conv"], generator=g)).to(torch.bfloat16)
            w[x + "b"], w[x + "a"], w[x + "g"] = lin(H, W, 2.0), lin(H, W, 2.0), lin(H * dv, W, 2.0)
            w[x + "A_log"], w[x + "dt_bias"] = vec(H, -1.0, 0.7), vec(H, 0.0, 0.5)
            w[x + "norm"], w[x + "o"] = vec(dv), lin(W, H * dv)
        mlp = layer.get("mlp")
        if mlp:
            w[p + "norm2"] = vec(W)
            e = p + "mlp."
            if mlp["kind"] == "dense":
                w[e + "gate"], w[e + "up"], w[e + "down"] = lin(mlp["ff"], W, 2.0), lin(mlp["ff"], W), lin(W, mlp["ff"])
            else:
                w[e + "router"] = lin(mlp["router"]["experts"], W, 3.0)
                ff = mlp["expert"]["ff"]
                for j in range(mlp["router"]["experts"]):
                    w[f"{e}e{j}.gate"], w[f"{e}e{j}.up"], w[f"{e}e{j}.down"] = lin(ff, W, 2.0), lin(ff, W, 2.0), lin(W, ff, 1.5)
    return w


def save(folder, cfg, weights):
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def default_layers():
    """Every mixer with every kind of feed-forward; grouped queries 2:1 and 1:1, a window shorter than the prompts, a partial rotation."""
    return [(retention(), moe()),
            (attention(), dense()),
            (delta(), moe(experts=6, top=1, ff=24, limit=0.7)),
            (retention(heads=2, dim=40, vdim=72, rot_dims=12, base=300.0), None),
            (attention(heads=3, kv_heads=3, dim=40, vdim=16, size=7, keep_first=0, rot_dims=40), moe(experts=9, top=2, ff=56, limit=2.5)),
            (delta(heads=2, kv_heads=2, dim=40, vdim=72, conv=2), dense(ff=50))]

"""Small random Gemepel checkpoints for the tests: a config dict and a name -> tensor dict in the checkpoint's naming, optionally written to a folder
(config.json + model.safetensors) so the tests go through the registry and the loader like a user does."""

import json
import os

import torch


def latent(heads=3, dim=24, rot_dim=16, vdim=40, q_rank=48, kv_rank=56, rot_dims=None, base=10000.0, kv_from=None, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "rot": {"dims": rot_dim if rot_dims is None else rot_dims, "base": base}, "scale": (dim + rot_dim) ** -0.5 if scale is None else scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def gla(heads=2, dim=24, vdim=48, tau=8.0):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}}


def moe(experts=12, top=3, groups=4, keep=2, ff=40, scale=2.5):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}, "scale": scale}}


def make_config(layers, width=72, vocab=131, eps=1e-5, alpha=2.0, embed_scale=0.7, bigram=(257, 13, 5)):
    """layers: list of (mixer entry, mlp entry or None)."""
    out = []
    for mixer, mlp in layers:
        e = dict(mixer)
        e["mlp"] = mlp
        out.append(e)
    cfg = {"architecture": "Gemepel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "postln_alpha": alpha,
           "embedding": {"scale": embed_scale}, "layers": out}
    if bigram:
        cfg["embedding"]["bigram"] = {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}
    return cfg


def make_weights(cfg, seed=0, decay_rank=8):
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def lin(o, i, gain=1.0):
        return (torch.randn(o, i, generator=g) * gain / i ** 0.5).to(torch.bfloat16)

    def vec(n, mean=1.0, std=0.1):
        return (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)

    w = {"embed": torch.randn(cfg["vocab"], W, generator=g).to(torch.bfloat16), "head": lin(cfg["vocab"], W), "final.norm": vec(W), "final.norm.b": vec(W, 0.0)}
    bg = cfg["embedding"].get("bigram")
    if bg:
        w["bigram"] = (0.5 * torch.randn(bg["buckets"] + 1, W, generator=g)).to(torch.bfloat16)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        w[p + "norm1"], w[p + "norm1.b"] = vec(W), vec(W, 0.0)
        if layer["type"] == "latent_attention":
            H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            w[p + "mix.dq"], w[p + "mix.dq.norm"] = lin(m["q_rank"], W), vec(m["q_rank"])
            w[p + "mix.uq"] = lin(H * (dn + dr), m["q_rank"], 2.0)
            if "kv_from" not in m:
                w[p + "mix.dkv"], w[p + "mix.dkv.norm"] = lin(m["kv_rank"] + dr, W, 2.0), vec(m["kv_rank"])
            w[p + "mix.uk"], w[p + "mix.uv"] = lin(H * dn, m["kv_rank"], 2.0), lin(H * dv, m["kv_rank"])
            w[p + "mix.o"] = lin(W, H * dv)
        else:
            H, dk, dv = m["heads"], m["dim"], m["vdim"]
            for n, o in (("q", H * dk), ("k", H * dk), ("v", H * dv), ("g", H * dv), ("a1", decay_rank)):
                w[p + "mix." + n] = lin(o, W)
            w[p + "mix.a2"], w[p + "mix.a2.b"] = lin(H * dk, decay_rank), vec(H * dk, 3.0, 1.0)
            w[p + "mix.norm"], w[p + "mix.o"] = vec(dv), lin(W, H * dv)
        mlp = layer.get("mlp")
        if mlp:
            r = mlp["router"]
            w[p + "norm2"], w[p + "norm2.b"] = vec(W), vec(W, 0.0)
            w[p + "mlp.router"] = lin(r["experts"], W, 3.0)
            w[p + "mlp.correction"] = vec(r["experts"], -0.3, 0.4)  # mostly negative: choice scores below zero occur
            for e in range(r["experts"]):
                w[f"{p}mlp.e{e}.up"], w[f"{p}mlp.e{e}.down"] = lin(mlp["expert"]["ff"], W, 1.5), lin(W, mlp["expert"]["ff"], 1.5)
    return w


def save(folder, cfg, weights):
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def default_layers():
    """latent, latent reading the first one's rows, gla, gla with other sizes, latent with a partial rotation and no feed-forward in one layer."""
    return [(latent(), moe()),
            (gla(), moe(experts=6, top=1, groups=1, keep=1, ff=24, scale=1.0)),
            (latent(heads=5, dim=16, vdim=24, q_rank=40, kv_from=0), moe(experts=8, top=4, groups=2, keep=2, ff=16)),
            (gla(heads=3, dim=40, vdim=72, tau=3.0), None),
            (latent(heads=2, dim=40, rot_dim=24, vdim=16, q_rank=32, kv_rank=72, rot_dims=12, base=500.0), moe(experts=9, top=2, groups=3, keep=1, ff=56))]

"""Plain PyTorch-CPU oracle of the Gemepel decoder (test infrastructure only, one function per mechanism).

Gemepel is a post-norm decoder: token embedding plus a hashed bigram embedding, a configurable sequence of layers whose token mixer is
either multi-head latent attention (low-rank query and key/value paths, one rotated key part shared by all heads, optionally reading
an earlier layer's cached latent) or gated linear attention (per-channel decays, a matrix state per head), each followed by a grouped
sigmoid-routed mixture of squared-ReLU experts, a final LayerNorm and an untied head.

Everything here works on one sequence at a time, in the dtype of the tensors handed in (fp32 or fp64), token by token where a recurrence
is involved, and shares no code with ``llm_quest_amd``.  ``weights`` maps the checkpoint's tensor names to tensors; ``cfg`` is the parsed
``config.json``.
"""

import math

import torch


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def layer_norm(x, w, b, eps):
    mu = x.mean(dim=-1, keepdim=True)
    var = ((x - mu) ** 2).mean(dim=-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def embed(tokens, weights, cfg, prev_token=None):
    """tokens: list of ints of ONE sequence (a continuation if ``prev_token`` is given) -> [len, width]."""
    e = cfg["embedding"]
    out = []
    for t in tokens:
        row = weights["embed"][t] * e["scale"]
        if "bigram" in e and e["bigram"]:
            bg = e["bigram"]
            idx = bg["buckets"] if prev_token is None else (prev_token * bg["mul_prev"] + t * bg["mul_cur"]) % bg["buckets"]
            row = row + weights["bigram"][idx]
        out.append(row)
        prev_token = t
    return torch.stack(out)


def rotate_pairs(x, positions, dims, base):
    """Interleaved rotary embedding on the first ``dims`` entries of the last axis: entries (2i, 2i+1) turn by p * base^(-2i/dims)."""
    out = x.clone()
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    ang = positions.to(x.dtype).unsqueeze(-1) * freq  # [T, half]
    while ang.dim() < x.dim():
        ang = ang.unsqueeze(1)
    c, s = torch.cos(ang), torch.sin(ang)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def latent_kv(h, positions, weights, pre, m, eps):
    """The cached part of a latent-attention layer: (normalised latent [T, kv_rank], rotated shared key part [T, rot_dim])."""
    r = m["kv_rank"]
    d = h @ weights[pre + "dkv"].T
    c = rms_unit(d[:, :r], eps) * weights[pre + "dkv.norm"]
    kr = rotate_pairs(d[:, r:], positions, m["rot"]["dims"], m["rot"]["base"])
    return c, kr


def latent_attention(h, positions, weights, pre, m, eps, c, kr):
    """h [T, width] attends causally over the keys (c, kr) [T, ...] of the same positions."""
    T = h.shape[0]
    H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    cq = rms_unit(h @ weights[pre + "dq"].T, eps) * weights[pre + "dq.norm"]
    q = (cq @ weights[pre + "uq"].T).view(T, H, dn + dr)
    qn = q[..., :dn]
    qr = rotate_pairs(q[..., dn:], positions, m["rot"]["dims"], m["rot"]["base"])
    kn = (c @ weights[pre + "uk"].T).view(T, H, dn)
    v = (c @ weights[pre + "uv"].T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for i in range(T):
        s = (torch.einsum("hd,jhd->hj", qn[i], kn[: i + 1]) + qr[i] @ kr[: i + 1].T) * m["scale"]
        p = torch.softmax(s, dim=-1)
        out[i] = torch.einsum("hj,jhd->hd", p, v[: i + 1])
    return out.reshape(T, H * dv) @ weights[pre + "o"].T


def gla(h, weights, pre, m, eps, state=None):
    """Gated linear attention, token by token.  state [heads, dim, vdim] or None; returns (output [T, width], final state)."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ weights[pre + "q"].T).view(T, H, dk) * dk ** -0.5
    k = (h @ weights[pre + "k"].T).view(T, H, dk)
    v = (h @ weights[pre + "v"].T).view(T, H, dv)
    z = (h @ weights[pre + "a1"].T) @ weights[pre + "a2"].T + weights[pre + "a2.b"]
    decay = torch.sigmoid(z).pow(1.0 / m["tau"]).view(T, H, dk)
    S = torch.zeros(H, dk, dv, dtype=h.dtype) if state is None else state.clone()
    o = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        S = decay[t].unsqueeze(-1) * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    o = rms_unit(o, eps) * weights[pre + "norm"]
    g = h @ weights[pre + "g"].T
    return (o.reshape(T, H * dv) * torch.nn.functional.silu(g)) @ weights[pre + "o"].T, S


def route(h, weights, pre, r):
    """Grouped sigmoid router -> (expert ids [T, top], weights [T, top]); the ids are in descending order of the choice score."""
    E, top = r["experts"], r["top"]
    s = torch.sigmoid(h @ weights[pre + "router"].T)
    choice = s + weights[pre + "correction"] if (pre + "correction") in weights else s.clone()
    g = r.get("groups")
    if g and g["count"] > 1:
        per = E // g["count"]
        grp = choice.view(-1, g["count"], per)
        gscore = torch.topk(grp, min(2, per), dim=-1)[0].sum(dim=-1)
        keep = torch.topk(gscore, g["keep"], dim=-1)[1]
        allowed = torch.zeros_like(gscore, dtype=torch.bool).scatter_(1, keep, True)
        choice = torch.where(allowed.unsqueeze(-1).expand(-1, -1, per).reshape(-1, E), choice, torch.full_like(choice, -math.inf))
    ids = torch.topk(choice, top, dim=-1)[1]
    w = torch.gather(s, 1, ids)
    w = w / (w.sum(dim=-1, keepdim=True) + 1e-20) * r["scale"]
    return ids, w


def moe(h, weights, pre, mlp):
    ids, w = route(h, weights, pre, mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            e = int(ids[t, j])
            a = torch.relu(weights[f"{pre}e{e}.up"] @ h[t]) ** 2
            out[t] += w[t, j] * (weights[f"{pre}e{e}.down"] @ a)
    return out


def forward(tokens, weights, cfg, dtype=torch.float32, return_layers=False):
    """Logits [T, vocab] of one whole sequence (positions 0 .. T-1); optionally the residual stream after every layer."""
    weights = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    x = embed(tokens, weights, cfg)
    pos = torch.arange(len(tokens))
    kv, layers = {}, []
    for i, layer in enumerate(cfg["layers"]):
        m, pre = layer["mixer"], f"l{i}.mix."
        if layer["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                kv[i] = latent_kv(x, pos, weights, pre, m, eps)
                src = i
            y = latent_attention(x, pos, weights, pre, m, eps, *kv[src])
        elif layer["type"] == "gla":
            y, _ = gla(x, weights, pre, m, eps)
        else:
            raise KeyError(layer["type"])
        x = layer_norm(alpha * x + y, weights[f"l{i}.norm1"], weights[f"l{i}.norm1.b"], eps)
        if layer.get("mlp"):
            y = moe(x, weights, f"l{i}.mlp.", layer["mlp"])
            x = layer_norm(alpha * x + y, weights[f"l{i}.norm2"], weights[f"l{i}.norm2.b"], eps)
        layers.append(x)
    x = layer_norm(x, weights["final.norm"], weights["final.norm.b"], eps)
    logits = x @ weights["head"].T
    return (logits, torch.stack(layers)) if return_layers else logits

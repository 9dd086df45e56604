"""Goluzen written out plainly: whole sequences, no cache, float64, one function per mechanism.

The model is a dictionary of tensors under their checkpoint names and the configuration as the nested dictionary
that `config.json` holds. Nothing here is shared with the engine: it is what the engine is compared with.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, eps):
    """The layers' norm: the stored weight lies around zero."""
    return unit_rms(x, eps) * (1.0 + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ------------------------------------------------------------------ rotations

def linear_frequencies(dims, base, factor):
    i = torch.arange(dims // 2, dtype=F64)
    return base ** (-2.0 * i / dims) / factor


def yarn_frequencies(dims, base, scaling):
    """-> (frequencies, the factor on cos and sin)."""
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    where = lambda turns: dims * math.log(scaling["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(where(scaling["fast"])), 0)
    hi = min(math.ceil(where(scaling["slow"])), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / scaling["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(scaling["factor"]) + 1.0


def rotate(x, positions, freqs, dims, interleaved, mult=1.0):
    """x [T, heads, n]: the first `dims` of n turn; pairs (i, i + dims/2) or (2i, 2i + 1)."""
    a = positions.to(F64)[:, None] * freqs[None, :]                  # [T, dims/2]
    c, s = (torch.cos(a) * mult)[:, None, :], (torch.sin(a) * mult)[:, None, :]
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        u, v = x[..., : dims // 2], x[..., dims // 2: dims]
        out[..., : dims // 2] = u * c - v * s
        out[..., dims // 2: dims] = v * c + u * s
    return out


# ------------------------------------------------------------------ mixers

def attention(h, w, pre, m, eps):
    """Grouped heads, biases, a rotation of the first dimensions, unit q and k, capped scores, a window that keeps the
    first tokens, a sink in the denominator."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = (h @ w[pre + "q"].T + w[pre + "q.b"]).view(T, H, D)
    k = (h @ w[pre + "k"].T + w[pre + "k.b"]).view(T, G, D)
    v = (h @ w[pre + "v"].T + w[pre + "v.b"]).view(T, G, Dv)
    rot = m.get("rot")
    if rot:
        f = linear_frequencies(rot["dims"], rot["base"], (rot.get("scaling") or {}).get("factor", 1.0))
        q, k = rotate(q, pos, f, rot["dims"], False), rotate(k, pos, f, rot["dims"], False)
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    i, j = pos[:, None], pos[None, :]
    seen = j <= i
    if m.get("mask"):
        seen = seen & ((i - j < m["mask"]["size"]) | (j < m["mask"].get("keep_first", 0)))
    out = torch.zeros(T, H, Dv, dtype=F64)
    for head in range(H):
        kv = head // (H // G)
        s = (q[:, head] @ k[:, kv].T) * m["scale"]
        if m.get("softcap"):
            s = m["softcap"] * torch.tanh(s / m["softcap"])
        s = s.masked_fill(~seen, -math.inf)
        sink = w[pre + "sink"][head]
        top = torch.maximum(s.max(-1, keepdim=True).values, sink)
        e = torch.exp(s - top)
        out[:, head] = (e / (e.sum(-1, keepdim=True) + torch.exp(sink - top))) @ v[:, kv]
    return out.reshape(T, H * Dv) @ w[pre + "o"].T


def latent_frequencies(m):
    sc = m["rot"].get("scaling")
    if sc:
        return yarn_frequencies(m["rot_dim"], m["rot"]["base"], sc)
    return linear_frequencies(m["rot_dim"], m["rot"]["base"], 1.0), 1.0


def latent_of(h, w, pre, m, eps):
    """What a latent-attention layer caches: the normed latent and the rotated key part that all heads share."""
    T = h.shape[0]
    R, r = m["kv_rank"], m["rot_dim"]
    rows = h @ w[pre + "dkv"].T
    c = unit_rms(rows[:, :R], eps) * w[pre + "dkv.norm"]
    f, mult = latent_frequencies(m)
    shared = rotate(rows[:, R:].view(T, 1, r), torch.arange(T), f, r, True, mult)[:, 0]
    return c, shared


def latent_attention(h, w, pre, m, eps, cached):
    """cached: (latent [T, rank], rotated key part [T, rot_dim]), this layer's own or another's."""
    T = h.shape[0]
    H, D, r, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    c, shared = cached
    q = (h @ w[pre + "q"].T).view(T, H, D + r)
    f, mult = latent_frequencies(m)
    q_rot = rotate(q[..., D:], torch.arange(T), f, r, True, mult)
    keys = (c @ w[pre + "uk"].T).view(T, H, D)
    values = (c @ w[pre + "uv"].T).view(T, H, Dv)
    pos = torch.arange(T)
    d = pos[:, None] - pos[None, :]
    seen = (d >= 0) & (d < m["mask"]["size"]) if m.get("mask") else d >= 0
    out = torch.zeros(T, H, Dv, dtype=F64)
    for head in range(H):
        s = (q[:, head, :D] @ keys[:, head].T + q_rot[:, head] @ shared.T) * m["scale"]
        out[:, head] = torch.softmax(s.masked_fill(~seen, -math.inf), -1) @ values[:, head]
    gate = torch.sigmoid(h @ w[pre + "g"].T)
    return (out.reshape(T, H * Dv) * gate) @ w[pre + "o"].T


def gated_linear_attention(h, w, pre, m, eps):
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w[pre + "k"].T).view(T, H, D)
    v = (h @ w[pre + "v"].T).view(T, H, Dv)
    z = (h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "a2.b"]
    alpha = (torch.sigmoid(z) ** (1.0 / m["tau"])).view(T, H, D)
    S = torch.zeros(H, D, Dv, dtype=F64)
    o = torch.zeros(T, H, Dv, dtype=F64)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hd,hdv->hv", q[t], S)
    o = unit_rms(o, eps) * w[pre + "norm"]
    g = h @ w[pre + "g"].T
    return (o.reshape(T, H * Dv) * (g * torch.sigmoid(g))) @ w[pre + "o"].T


# ------------------------------------------------------------------ feed-forwards

def dense(h, w, pre):
    return gelu_tanh(h @ w[pre + "up"].T) @ w[pre + "down"].T


def relu2_expert(h, up, down):
    return torch.relu(h @ up.T) ** 2 @ down.T


def choose_experts(z, correction, r):
    """z: router logits [T, E] -> (ids [T, top], weights [T, top])."""
    E, top = r["experts"], r["top"]
    s = torch.sigmoid(z)
    choice = s + correction
    groups, keep = (r["groups"]["count"], r["groups"]["keep"]) if r.get("groups") else (1, 1)
    per = E // groups
    score = choice.view(-1, groups, per).topk(min(2, per), -1).values.sum(-1)
    kept = torch.zeros_like(score, dtype=torch.bool)
    kept.scatter_(1, score.topk(keep, -1).indices, True)
    eligible = kept[:, :, None].expand(-1, -1, per).reshape(-1, E)
    ids = choice.masked_fill(~eligible, -math.inf).topk(top, -1).indices
    return ids, s.gather(1, ids) * r.get("scale", 1.0)


def mixture(h, w, pre, f):
    r = f["router"]
    ids, weights = choose_experts(h @ w[pre + "router"].T, w[pre + "correction"], r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(ids[t].tolist(), weights[t]):
            out[t] += a * relu2_expert(h[t], w[f"{pre}e{e}.up"], w[f"{pre}e{e}.down"])
    if f.get("shared") is not None:
        gate = torch.sigmoid(h @ w[pre + "shared.sg"].T)               # [T, 1]
        out = out + gate * relu2_expert(h, w[pre + "shared.up"], w[pre + "shared.down"])
    return out


# ------------------------------------------------------------------ the model

def forward(config, weights, tokens, keep_layers: bool = False):
    """tokens: a list of ids -> logits [T, vocab] (and the stream after every layer, [layers, T, width])."""
    w = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * (config.get("embedding") or {}).get("scale", 1.0)
    latents, after = {}, []
    for i, layer in enumerate(config["layers"]):
        m, pre = layer["mixer"], f"l{i}.mix."
        h = layer_norm(x, w[f"l{i}.norm1"], eps)
        if layer["type"] == "attention":
            a = attention(h, w, pre, m, eps)
        elif layer["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                latents[i] = latent_of(h, w, pre, m, eps)
            a = latent_attention(h, w, pre, m, eps, latents[i if src is None else src])
        elif layer["type"] == "gla":
            a = gated_linear_attention(h, w, pre, m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + a
        f = layer.get("mlp")
        if f is not None:
            h = layer_norm(x, w[f"l{i}.norm2"], eps)
            x = x + (dense(h, w, f"l{i}.mlp.") if f["kind"] == "dense" else mixture(h, w, f"l{i}.mlp.", f))
        after.append(x)
    logits = layer_norm(x, w["final.norm"], eps) @ w["head"].T
    return (logits, torch.stack(after)) if keep_layers else logits


def read_folder(folder: str):
    """(config.json as a dictionary, the checkpoint's tensors by name) of a model folder."""
    import json
    import os

    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json")) as f:
        config = json.load(f)
    return config, load_file(os.path.join(folder, "model.safetensors"))


def logits(config, weights, tokens):
    return forward(config, weights, tokens)

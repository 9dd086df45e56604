"""A plain, slow evaluation of the Tavevik design: whole sequences, float64, one function per mechanism,
token-by-token loops wherever the design is a recurrence or a mask. It shares nothing with the engine: it reads
a model folder's config.json and tensors by their stored names and knows no cache, page, slot or step.

Layer:      x <- x + N1(mixer(x));  x <- x + N2(ff(x)) when the layer has a feed-forward.
            N(y) = y / sqrt(mean(y^2) + eps) * w: the norm sits on the sublayer's output only.
Mixer:      two mixers read the same input; the result is left_scale * left + right_scale * right.
            Left: softmax attention with grouped key/value heads, per-head q/k norm, a rotation of the first
            dimensions of each head (pairs half the rotating width apart), and a trailing window. Type
            `parallel`: the first positions stay visible behind the window, scores pass cap * tanh(s / cap),
            the heads are gated element by element by sigmoid(W_g h). Type `parallel_2`: biases on q, k, v and o,
            and a per-head sink: one more term exp(sink) in the softmax's denominator.
            Right, type `parallel`: a recurrence over a matrix per head with one decay per key channel that the
            token chooses, inputs mixed with the previous token's, and a bonus for the current token.
            Right, type `parallel_2`: a delta-rule recurrence with one decay per key channel, short causal
            convolutions on q, k, v, unit-length q and k, a write strength per head.
Feed-forward: g = min(W_gate x, limit), u = clamp(W_up x, -limit, limit); W_down (g sigmoid(1.702 g) (u + 1)).
Head:       the final norm, then the embedding matrix.
"""
from __future__ import annotations

import json
import math
import os

import torch


def read_folder(folder: str, dtype=torch.float64):
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt", device="cpu") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            w[name] = t.to(dtype) if t.is_floating_point() else t
    return cfg, w


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(x):
    return x * torch.sigmoid(x)


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def rotate_halves(x, dims, base):
    """x [T, heads, dim]: dimensions (i, i + dims/2), i < dims/2, turn by position * base^(-2i/dims)."""
    out = x.clone()
    half = dims // 2
    for t in range(x.shape[0]):
        for i in range(half):
            a = t * base ** (-2.0 * i / dims)
            c, s = math.cos(a), math.sin(a)
            u, v = x[t, :, i], x[t, :, i + half]
            out[t, :, i] = u * c - v * s
            out[t, :, i + half] = v * c + u * s
    return out


def visible(i: int, j: int, size: int, keep_first: int) -> bool:
    return j <= i and (i - j < size or j < keep_first)


def attention(kind, m, w, pre, h, eps):
    T = h.shape[0]
    H, G, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    biased, gated = kind == "parallel_2", kind == "parallel"
    b = (lambda name: w[pre + name + ".b"]) if biased else (lambda name: 0.0)
    q = (h @ w[pre + "q"].T + b("q")).view(T, H, dim)
    k = (h @ w[pre + "k"].T + b("k")).view(T, G, dim)
    v = (h @ w[pre + "v"].T + b("v")).view(T, G, vdim)
    q = unit_rms(q, eps) * w[pre + "q.norm"]
    k = unit_rms(k, eps) * w[pre + "k.norm"]
    if m.get("rot"):
        q = rotate_halves(q, m["rot"]["dims"], m["rot"]["base"])
        k = rotate_halves(k, m["rot"]["dims"], m["rot"]["base"])
    size = m["mask"]["size"]
    keep = m["mask"].get("keep_first", 0) if gated else 0
    cap = m.get("softcap") if gated else None
    out = torch.zeros(T, H, vdim, dtype=h.dtype)
    for i in range(T):
        js = [j for j in range(i + 1) if visible(i, j, size, keep)]
        for head in range(H):
            g = head // (H // G)
            s = (k[js, g] @ q[i, head]) * m["scale"]
            if cap:
                s = cap * torch.tanh(s / cap)
            top = s.max()
            e = torch.exp(s - top)
            denom = e.sum()
            if biased:
                denom = denom + torch.exp(w[pre + "sink"][head] - top)
            out[i, head] = ((e / denom)[:, None] * v[js, g]).sum(0)
    out = out.reshape(T, H * vdim)
    if gated:
        out = out * torch.sigmoid(h @ w[pre + "g"].T)
    return out @ w[pre + "o"].T + (b("o") if biased else 0.0)


def shifted_mix(m, w, pre, h):
    """Right mixer of `parallel`: per-channel decays chosen by the token, a bonus for the token itself."""
    T = h.shape[0]
    H, dim = m["heads"], m["dim"]
    before = torch.cat((torch.zeros_like(h[:1]), h[:-1]), 0)
    mix = lambda s: h + (before - h) * w[pre + "mu." + s]
    r = (mix("r") @ w[pre + "r"].T).view(T, H, dim)
    k = (mix("k") @ w[pre + "k"].T).view(T, H, dim)
    v = (mix("v") @ w[pre + "v"].T).view(T, H, dim)
    gate = silu(mix("g") @ w[pre + "g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(mix("w") @ w[pre + "w1"].T) @ w[pre + "w2"].T + w[pre + "w0"])).view(T, H, dim)
    u = w[pre + "u"]
    o = torch.zeros(T, H, dim, dtype=h.dtype)
    S = torch.zeros(H, dim, dim, dtype=h.dtype)
    for t in range(T):
        for head in range(H):
            kv = torch.outer(k[t, head], v[t, head])
            o[t, head] = (S[head] + u[head][:, None] * kv).T @ r[t, head]
            S[head] = decay[t, head][:, None] * S[head] + kv
    return o, gate


def shifted_mix_output(m, w, pre, o, gate, eps):
    T = o.shape[0]
    return (unit_rms(o, eps).reshape(T, -1) * w[pre + "norm"] * gate) @ w[pre + "o"].T


def short_conv(x, taps_weight):
    """x [T, C], taps_weight [C, taps] (the last column is the current token's); zeros before the start."""
    T, taps = x.shape[0], taps_weight.shape[1]
    out = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                out[t] = out[t] + taps_weight[:, j] * x[src]
    return out


def unit_length(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def delta_rule(m, w, pre, h, eps):
    """Right mixer of `parallel_2`."""
    T = h.shape[0]
    H, G, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ w[pre + "q"].T, w[pre + "q.conv"])).view(T, G, dim)
    k = silu(short_conv(h @ w[pre + "k"].T, w[pre + "k.conv"])).view(T, G, dim)
    v = silu(short_conv(h @ w[pre + "v"].T, w[pre + "v.conv"])).view(T, H, vdim)
    q = unit_length(q) * dim ** -0.5
    k = unit_length(k)
    beta = torch.sigmoid(h @ w[pre + "b"].T)                                     # [T, H]
    step = softplus((h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "dt_bias"]).view(T, H, dim)
    decay = torch.exp(-torch.exp(w[pre + "A_log"])[None, :, None] * step)
    o = torch.zeros(T, H, vdim, dtype=h.dtype)
    S = torch.zeros(H, dim, vdim, dtype=h.dtype)
    for t in range(T):
        for head in range(H):
            g = head // (H // G)
            S[head] = decay[t, head][:, None] * S[head]
            u = beta[t, head] * (v[t, head] - S[head].T @ k[t, g])
            S[head] = S[head] + torch.outer(k[t, g], u)
            o[t, head] = S[head].T @ q[t, g]
    o = unit_rms(o, eps) * w[pre + "norm"]
    gate = torch.sigmoid((h @ w[pre + "g1"].T) @ w[pre + "g2"].T)
    return (o.reshape(T, H * vdim) * gate) @ w[pre + "o"].T


def mixer(kind, m, w, pre, h, eps):
    left = attention(kind, m["left"], w, pre + "left.", h, eps)
    if kind == "parallel":
        o, gate = shifted_mix(m["right"], w, pre + "right.", h)
        right = shifted_mix_output(m["right"], w, pre + "right.", o, gate, eps)
    elif kind == "parallel_2":
        right = delta_rule(m["right"], w, pre + "right.", h, eps)
    else:
        raise ValueError(kind)
    return m["left_scale"] * left + m["right_scale"] * right


def feed_forward(f, w, pre, h):
    limit = f["limit"]
    g = torch.clamp(h @ w[pre + "gate"].T, max=limit)
    u = torch.clamp(h @ w[pre + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ w[pre + "down"].T


def out_norm(y, weight, eps):
    return unit_rms(y, eps) * weight


def logits(cfg, w, ids, layers_out: list | None = None):
    """float64 logits [len(ids), vocab]; `layers_out` collects the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(ids, dtype=torch.long)]
    for i, layer in enumerate(cfg["layers"]):
        x = x + out_norm(mixer(layer["type"], layer["mixer"], w, f"l{i}.mix.", x, eps), w[f"l{i}.norm1"], eps)
        if layer.get("mlp") is not None:
            x = x + out_norm(feed_forward(layer["mlp"], w, f"l{i}.mlp.", x), w[f"l{i}.norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return out_norm(x, w["final.norm"], eps) @ w["embed"].T

"""A plain, slow evaluation of the Sigosun design: whole sequences, float64, one function per mechanism,
token-by-token loops wherever the design is a recurrence. It shares nothing with the engine: it reads a
model folder's config.json and tensors by their stored names and knows no cache, page, slot or step.

Layer:      x <- x + N1(mixer(x));  x <- x + N2(ff(x)) when the layer has a feed-forward.
            N(y) = y / sqrt(mean(y^2) + eps) * (1 + w): the norm sits on the sublayer's output only.
Mixers:     softmax attention under a block mask (query i sees key j <= i of its own block of positions),
            with per-head q/k norm, a rotation of the first dimensions of each head in adjacent pairs, a
            sigmoid gate per head, optionally on the keys and values another layer made;
            a selective state-space recurrence (short causal convolution, softplus step sizes, gated and
            group-normed output); a linear-attention recurrence with one fixed decay per head.
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


def rotate_pairs(x, dims, base):
    """x [T, heads, dim]: dimensions (2i, 2i+1), i < dims/2, turn by position * base^(-2i/dims)."""
    T = x.shape[0]
    out = x.clone()
    for t in range(T):
        for i in range(dims // 2):
            a = t * base ** (-2.0 * i / dims)
            c, s = math.cos(a), math.sin(a)
            u, v = x[t, :, 2 * i], x[t, :, 2 * i + 1]
            out[t, :, 2 * i] = u * c - v * s
            out[t, :, 2 * i + 1] = v * c + u * s
    return out


def attention_keys_values(m, w, pre, h, eps):
    T = h.shape[0]
    G, dim, vdim = m["kv_heads"], m["dim"], m["vdim"]
    k = (h @ w[pre + "k"].T).view(T, G, dim)
    v = (h @ w[pre + "v"].T).view(T, G, vdim)
    k = unit_rms(k, eps) * w[pre + "k.norm"]
    if m.get("rot"):
        k = rotate_pairs(k, m["rot"]["dims"], m["rot"]["base"])
    return k, v


def attention(m, w, pre, h, eps, kv):
    """kv: (keys [T, G, dim] after norm and rotation, values [T, G, vdim])."""
    T = h.shape[0]
    H, G, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).view(T, H, dim)
    q = unit_rms(q, eps) * w[pre + "q.norm"]
    if m.get("rot"):
        q = rotate_pairs(q, m["rot"]["dims"], m["rot"]["base"])
    k, v = kv
    gate = torch.sigmoid(h @ w[pre + "g"].T)                # [T, H]
    block = m["mask"]["size"] if m.get("mask") else None
    out = torch.zeros(T, H, vdim, dtype=h.dtype)
    for i in range(T):
        lo = (i // block) * block if block else 0
        for head in range(H):
            g = head // (H // G)
            s = (k[lo:i + 1, g] @ q[i, head]) * m["scale"]
            p = torch.softmax(s, 0)
            out[i, head] = (p[:, None] * v[lo:i + 1, g]).sum(0) * gate[i, head]
    return out.reshape(T, H * vdim) @ w[pre + "o"].T


def mamba2(m, w, pre, h, eps):
    T = h.shape[0]
    H, P, N, G, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner = H * P
    proj = h @ w[pre + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    cw, cb = w[pre + "conv"], w[pre + "conv.b"]
    conv = torch.zeros_like(xbc)
    for t in range(T):
        acc = cb.clone()
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                acc = acc + cw[:, j] * xbc[src]
        conv[t] = acc
    conv = silu(conv)
    x = conv[:, :inner].view(T, H, P)
    B = conv[:, inner:inner + G * N].view(T, G, N)
    C = conv[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + w[pre + "dt_bias"])                  # [T, H]
    rate = torch.exp(w[pre + "A_log"])
    y = torch.zeros(T, H, P, dtype=h.dtype)
    S = torch.zeros(H, N, P, dtype=h.dtype)
    for t in range(T):
        for head in range(H):
            g = head // (H // G)
            S[head] = torch.exp(-rate[head] * dt[t, head]) * S[head] + dt[t, head] * torch.outer(B[t, g], x[t, head])
            y[t, head] = S[head].T @ C[t, g] + w[pre + "D"][head] * x[t, head]
    y = y.reshape(T, inner) * silu(z)
    parts = m["norm_groups"]
    y = unit_rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * w[pre + "norm"]
    return y @ w[pre + "o"].T


def lightning(m, w, pre, h, eps):
    T = h.shape[0]
    H, dim, vdim = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[pre + "q"].T).view(T, H, dim)
    k = silu(h @ w[pre + "k"].T).view(T, H, dim)
    v = silu(h @ w[pre + "v"].T).view(T, H, vdim)
    o = torch.zeros(T, H, vdim, dtype=h.dtype)
    S = torch.zeros(H, dim, vdim, dtype=h.dtype)
    for t in range(T):
        for head in range(H):
            S[head] = m["decay"][head] * S[head] + torch.outer(k[t, head], v[t, head])
            o[t, head] = S[head].T @ q[t, head]
    o = unit_rms(o.reshape(T, H * vdim), eps) * w[pre + "norm"]
    return (o * torch.sigmoid(h @ w[pre + "g"].T)) @ w[pre + "o"].T


def feed_forward(w, pre, h):
    return torch.relu(h @ w[pre + "up"].T) ** 2 @ w[pre + "down"].T


def out_norm(y, weight, eps):
    return unit_rms(y, eps) * (1 + weight)


def logits(cfg, w, ids, layers_out: list | None = None):
    """float64 logits [len(ids), vocab]; `layers_out` collects the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(ids, dtype=torch.long)]
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        m, pre = layer["mixer"], f"l{i}.mix."
        if layer["type"] == "attention":
            if m.get("kv_from") is None:
                kept[i] = attention_keys_values(m, w, pre, x, eps)
            a = attention(m, w, pre, x, eps, kept[i if m.get("kv_from") is None else m["kv_from"]])
        elif layer["type"] == "mamba2":
            a = mamba2(m, w, pre, x, eps)
        elif layer["type"] == "lightning":
            a = lightning(m, w, pre, x, eps)
        else:
            raise ValueError(layer["type"])
        x = x + out_norm(a, w[f"l{i}.norm1"], eps)
        if layer.get("mlp") is not None:
            x = x + out_norm(feed_forward(w, f"l{i}.mlp.", x), w[f"l{i}.norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return out_norm(x, w["final.norm"], eps) @ w["head"].T

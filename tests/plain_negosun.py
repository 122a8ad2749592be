"""The Negosun design evaluated plainly, in float64, token by token: the oracle of the engine's tests. One function per
mechanism; nothing here is shared with the engine. It reads a model folder (config.json, model.safetensors) itself.

In this file's notation: x is the stream at one position, n(x, w) = w * x / sqrt(mean(x^2) + eps). A layer is
    x <- x + m * (s1 * A(n(x, w1)) + s2 * F(n(x, w2)))
with the attention A over this and all earlier positions and the feed-forward F; s1, s2 and w1, w2 are vectors.
"""
from __future__ import annotations

import json
import math
import os

import torch


def read_folder(folder: str):
    from safetensors import safe_open
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt", device="cpu") as f:
        for name in f.keys():
            w[name] = f.get_tensor(name).to(torch.float64)
    return cfg, w


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean() + eps)


def temperature(mixer: dict, p: int) -> float:
    """What the query at position p is multiplied by."""
    t = mixer.get("q_temp")
    if not t:
        return 1.0
    return 1.0 + t["coef"] * math.log((p + 1) // t["every"] + 1)


def project(w, name, u, eps, normed: bool):
    """W u + b, then (for q and k) the norm over the whole vector."""
    y = w[name] @ u + w[name + ".b"]
    return unit_rms(y, eps) * w[name + ".norm"] if normed else y


def attend(q, keys, values, heads, kv_heads, dim, vdim, scale):
    """One position: q [heads * dim] against the kept keys [n, kv_heads * dim] and values [n, kv_heads * vdim]."""
    per = heads // kv_heads
    K, V = torch.stack(keys), torch.stack(values)
    out = []
    for h in range(heads):
        g = h // per                                     # the key/value head of query head h
        scores = (K[:, g * dim:(g + 1) * dim] @ q[h * dim:(h + 1) * dim]) * scale
        out.append(torch.softmax(scores, 0) @ V[:, g * vdim:(g + 1) * vdim])
    return torch.cat(out)


def gated(w, name, u):
    a = w[name + ".gate"] @ u
    return w[name + ".down"] @ (a * torch.sigmoid(a) * (w[name + ".up"] @ u))


def choose(scores, top: int, groups: dict | None):
    """Indices of the chosen experts, best first."""
    n = scores.numel()
    allowed = [True] * n
    if groups and groups["count"] > 1:
        size = n // groups["count"]
        best = [max(scores[g * size:(g + 1) * size]).item() for g in range(groups["count"])]
        kept = sorted(range(groups["count"]), key=lambda g: (-best[g], g))[:groups["keep"]]
        allowed = [e // size in kept for e in range(n)]
    ranked = sorted((e for e in range(n) if allowed[e]), key=lambda e: (-scores[e].item(), e))
    return ranked[:top]


def experts(w, name, mlp: dict, u):
    r = mlp["router"]
    scores = torch.softmax(w[name + ".router"] @ u, 0)
    chosen = choose(scores, r["top"], r.get("groups"))
    total = sum(scores[e] for e in chosen) + 1e-20
    y = sum(scores[e] / total * gated(w, f"{name}.e{e}", u) for e in chosen)
    if mlp.get("shared"):
        y = y + gated(w, name + ".shared", u)
    return y


def logits(cfg: dict, w: dict, ids: list, streams: list | None = None) -> torch.Tensor:
    """float64 [len(ids), vocab]. `streams`: if a list, the stream after every layer is appended ([T, width] each)."""
    eps, m = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    xs = [w["embed"][t].clone() for t in ids]
    first_values = None                                  # per position: the values of the first layer that mixes
    for i, layer in enumerate(cfg["layers"]):
        mx = layer["mixer"]
        keys, values, new = [], [], []
        mixes = bool(mx.get("v_mix"))
        starts_mixing = mixes and first_values is None
        kept_values = []
        for p, x in enumerate(xs):
            u = unit_rms(x, eps) * w[f"l{i}.norm1"]
            q = project(w, f"l{i}.mix.q", u, eps, True) * temperature(mx, p)
            k = project(w, f"l{i}.mix.k", u, eps, True)
            v = project(w, f"l{i}.mix.v", u, eps, False)
            if starts_mixing:
                kept_values.append(v)
            elif mixes:
                lam = w[f"l{i}.mix.vmix"]
                v = (1 - lam) * v + lam * first_values[p]
            keys.append(k); values.append(v)
            a = w[f"l{i}.mix.o"] @ attend(q, keys, values, mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"], mx["scale"])
            total = w[f"l{i}.ls1"] * a
            if layer.get("mlp"):
                total = total + w[f"l{i}.ls2"] * experts(w, f"l{i}.mlp", layer["mlp"], unit_rms(x, eps) * w[f"l{i}.norm2"])
            new.append(x + m * total)
        if starts_mixing:
            first_values = kept_values
        xs = new
        if streams is not None:
            streams.append(torch.stack(xs))
    z = torch.stack([w["embed"] @ (unit_rms(x, eps) * w["final.norm"]) for x in xs])
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z

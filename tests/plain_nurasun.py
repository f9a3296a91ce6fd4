"""The Nurasun design, plainly: whole sequences, float64, no cache, one function per mechanism.

Slow on purpose (loops over tokens and heads where a loop says most clearly what is computed)
and independent of ``pyre_amd``: it reads ``config.json`` as a dictionary and the tensors by
their names. The tests compare the engine with it.

Notation: ``h`` the rows [T, width] that both sublayers of a layer read, ``i`` a query's
position, ``j`` a key's, both counted from 0 within the sequence.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch

F = torch.float64


def read_folder(folder) -> tuple[dict, dict]:
    """(config as a dictionary, tensors as float64 / int64) of a model folder."""
    from safetensors.torch import load_file

    folder = Path(folder)
    cfg = json.loads((folder / "config.json").read_text())
    raw = load_file(str(folder / "model.safetensors"))
    return cfg, {k: (v.to(F) if v.is_floating_point() else v.long()) for k, v in raw.items()}


# ----------------------------------------------------------------------------- small pieces


def squash_norm(x, w, name):
    """tanh(alpha x) * gain + shift, element by element: no statistic of the row enters."""
    return torch.tanh(w[name + ".alpha"] * x) * w[name] + w[name + ".b"]


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate(x, pos, dims, base):
    """The first ``dims`` elements of every head of x [T, heads, d] turned by position: element e pairs with
    e + dims/2, the pair's angle is pos * base^(-2e/dims); the other elements pass."""
    out = x.clone()
    half = dims // 2
    for e in range(half):
        ang = torch.tensor([p * base ** (-2.0 * e / dims) for p in pos], dtype=F)
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
        u, v = x[:, :, e], x[:, :, e + half]
        out[:, :, e] = u * c - v * s
        out[:, :, e + half] = v * c + u * s
    return out


def softmax_rows(scores, visible):
    """Row i: softmax over the keys j with visible(i, j); scores [T, T] -> weights [T, T]."""
    T = scores.shape[0]
    out = torch.zeros_like(scores)
    for i in range(T):
        js = [j for j in range(T) if visible(i, j)]
        out[i, js] = torch.softmax(scores[i, js], dim=0)
    return out


# ----------------------------------------------------------------------------- mixers


def same_chunk(size: int):
    return lambda i, j: j <= i and i // size == j // size


def causal(i, j):
    return j <= i


def chunked_attention(h, w, p, m):
    """Grouped heads, biased projections, the keys (before they are turned) double as values."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w[p + ".q"].T + w[p + ".q.b"]).view(T, H, d)
    k = (h @ w[p + ".k"].T + w[p + ".k.b"]).view(T, G, d)
    v = k
    pos = list(range(T))
    rot = m.get("rot")
    if rot:
        q, k = rotate(q, pos, rot["dims"], rot["base"]), rotate(k, pos, rot["dims"], rot["base"])
    size = (m.get("mask") or {}).get("size") or 0
    visible = same_chunk(size) if size else causal
    out = torch.zeros(T, H, v.shape[-1], dtype=F)
    for head in range(H):
        g = head // (H // G)
        a = softmax_rows((q[:, head] @ k[:, g].T) * m["scale"], visible)
        out[:, head] = a @ v[:, g]
    return out.reshape(T, -1) @ w[p + ".o"].T


def latent_of(h, w, p, eps):
    """The compressed row that every head's keys and values are made of."""
    return unit_rms(h @ w[p + ".dkv"].T, eps) * w[p + ".dkv.norm"]


def latent_attention(h, c, w, p, m):
    """No positions; ``c`` [T, rank] are the latents (this layer's own or another's)."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + ".q"].T).view(T, H, d)
    k = (c @ w[p + ".uk"].T).view(T, H, d)
    v = (c @ w[p + ".uv"].T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        a = softmax_rows((q[:, head] @ k[:, head].T) * m["scale"], causal)
        out[:, head] = a @ v[:, head]
    return out.reshape(T, -1) @ w[p + ".o"].T


# ----------------------------------------------------------------------------- feed-forwards


def gated_dense(h, w, p):
    return (gelu_tanh(h @ w[p + ".gate"].T) * (h @ w[p + ".up"].T)) @ w[p + ".down"].T


def squared_relu_expert(h, w, p):
    return (torch.relu(h @ w[p + ".up"].T) ** 2) @ w[p + ".down"].T


def route(h, w, p, top):
    """Per token the ``top`` experts of largest sigmoid score and their scores over the scores' sum."""
    s = torch.sigmoid(h @ w[p + ".router"].T)
    picks = []
    for t in range(h.shape[0]):
        order = sorted(range(s.shape[1]), key=lambda e: (-float(s[t, e]), e))[:top]
        total = sum(s[t, e] for e in order) + 1e-20
        picks.append([(e, s[t, e] / total) for e in order])
    return picks


def mixture(h, w, p, mlp):
    out = torch.zeros(h.shape[0], w[p + ".e0.down"].shape[0], dtype=F)
    for t, chosen in enumerate(route(h, w, p, mlp["router"]["top"])):
        for e, weight in chosen:
            out[t] += weight * squared_relu_expert(h[t:t + 1], w, f"{p}.e{e}")[0]
    if mlp.get("shared"):
        out = out + squared_relu_expert(h, w, p + ".shared")
    return out


def feed_forward(h, w, p, mlp):
    return gated_dense(h, w, p) if mlp["kind"] == "dense" else mixture(h, w, p, mlp)


# ----------------------------------------------------------------------------- the model


def forward(w, cfg, ids, return_hidden=False):
    """ids: one sequence -> logits [T, vocab] (float64); with ``return_hidden`` also the residual
    stream after every layer."""
    x = w["embed"][torch.as_tensor(ids, dtype=torch.long)].clone()
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    latents, hidden = {}, []
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}", layer["mixer"]
        h = squash_norm(x, w, p + ".norm1")
        if layer["type"] == "attention":
            y = chunked_attention(h, w, p + ".mix", m)
        elif layer["type"] == "latent_attention":
            src = m.get("kv_from")
            latents[i] = latents[src] if src is not None else latent_of(h, w, p + ".mix", eps)
            y = latent_attention(h, latents[i], w, p + ".mix", m)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp") is not None:
            y = y + feed_forward(h, w, p + ".mlp", layer["mlp"])
        x = x + mult * y
        hidden.append(x.clone())
    z = squash_norm(x, w, "final.norm") @ w["head"].T
    cap = cfg.get("logit_softcap") or 0.0
    if cap:
        z = cap * torch.tanh(z / cap)
    return (z, hidden) if return_hidden else z


def closest_call(w, cfg, ids):
    """Per position the smallest gap, over the layers with a mixture, between the scores of the last expert that is
    chosen and the first that is not (infinite where nothing is left out): where it is tiny, rounding decides which
    experts a token goes through, and its row is no measure of an engine in 16 bits."""
    x = w["embed"][torch.as_tensor(ids, dtype=torch.long)].clone()
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    latents, gap = {}, torch.full((len(ids),), float("inf"), dtype=F)
    for i, layer in enumerate(cfg["layers"]):
        p, m, mlp = f"l{i}", layer["mixer"], layer.get("mlp")
        h = squash_norm(x, w, p + ".norm1")
        if layer["type"] == "attention":
            y = chunked_attention(h, w, p + ".mix", m)
        else:
            src = m.get("kv_from")
            latents[i] = latents[src] if src is not None else latent_of(h, w, p + ".mix", eps)
            y = latent_attention(h, latents[i], w, p + ".mix", m)
        if mlp is not None:
            if mlp["kind"] == "moe" and mlp["router"]["top"] < mlp["router"]["experts"]:
                s = torch.sigmoid(h @ w[p + ".mlp.router"].T).sort(dim=-1, descending=True).values
                top = mlp["router"]["top"]
                gap = torch.minimum(gap, s[:, top - 1] - s[:, top])
            y = y + feed_forward(h, w, p + ".mlp", mlp)
        x = x + mult * y
    return gap

"""The Mafurax design, plainly: whole sequences, float64, no cache, one function per mechanism.

Slow on purpose (loops over tokens and heads where a loop says most clearly what is computed)
and independent of ``pyre_amd``: it reads ``config.json`` as a dictionary and the tensors by
their names. The tests compare the engine with it.

Notation: ``h`` the rows [T, width] that a sublayer reads, ``i`` a query's position, ``j`` a
key's, both counted from 0 within the sequence.
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


def layer_norm(x, gain, eps):
    """(x - mean) / sqrt(var + eps) * gain, var = mean of squared deviations; no bias."""
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * gain


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def distance_bucket(n: int, rows: int, far: float) -> int:
    """Row of the distance table for a key n tokens back: one row per distance below rows/2,
    then rows spaced evenly in log(distance) up to ``far``, the last row for everything beyond."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def sees(i: int, j: int, window: int, keep_first: int) -> bool:
    """Causal, the last ``window`` positions, and the sequence's first ``keep_first`` always
    (no window, written as 0: every earlier position)."""
    return j <= i and (not window or i - j < window or j < keep_first)


# ----------------------------------------------------------------------------- the softmax branch


def capped_biased_attention(h, w, p, c, eps):
    """Grouped-query softmax attention without rotation: unit-RMS queries and keys, scores
    scaled, squashed by cap * tanh(s / cap), a learned bias by distance added after that, a
    window that keeps the first tokens, one sigmoid gate per head on the output."""
    T = h.shape[0]
    H, G, d, dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = unit_rms((h @ w[f"{p}.q"].T).view(T, H, d), eps)
    k = unit_rms((h @ w[f"{p}.k"].T).view(T, G, d), eps)
    v = (h @ w[f"{p}.v"].T).view(T, G, dv)
    gate = torch.sigmoid(h @ w[f"{p}.g"].T)                      # [T, H]
    rel = w[f"{p}.rel"]                                          # [rows, H]
    rows = rel.shape[0]
    cap = c.get("softcap")
    mask = c.get("mask") or {}
    window, keep = mask.get("size") or 0, mask.get("keep_first") or 0
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    seen = torch.tensor([[sees(a, b, window, keep) for b in range(T)] for a in range(T)])
    row_of = torch.tensor([distance_bucket(n, rows, c["bias_max"]) for n in range(T)])
    bias_row = row_of[(i - j).clamp(min=0)]                      # [T, T]
    out = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * c["scale"]
        if cap:
            s = cap * torch.tanh(s / cap)
        s = (s + rel[bias_row, head]).masked_fill(~seen, -math.inf)
        out[:, head] = (torch.softmax(s, 1) @ v[:, g]) * gate[:, head, None]
    return out.reshape(T, H * dv) @ w[f"{p}.o"].T


# ----------------------------------------------------------------------------- the recurrent branch


def gated_linear_attention(h, w, p, c, eps):
    """Per head a matrix state S [dim, vdim]: S <- diag(alpha_t) S + k_t v_t^T, read by
    o_t = S^T q_t. alpha_t = sigmoid(z_t)^(1/tau) per key channel, z_t from a low-rank product
    with a bias. The outputs are unit-RMS normed with a gain over vdim, gated by silu."""
    T = h.shape[0]
    H, d, dv = c["heads"], c["dim"], c["vdim"]
    q = (h @ w[f"{p}.q"].T).view(T, H, d) * d ** -0.5
    k = (h @ w[f"{p}.k"].T).view(T, H, d)
    v = (h @ w[f"{p}.v"].T).view(T, H, dv)
    z = ((h @ w[f"{p}.a1"].T) @ w[f"{p}.a2"].T + w[f"{p}.a2.b"]).view(T, H, d)
    alpha = torch.sigmoid(z) ** (1.0 / c["tau"])
    S = torch.zeros(H, d, dv, dtype=F)
    o = torch.zeros(T, H, dv, dtype=F)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = unit_rms(o, eps) * w[f"{p}.norm"]
    gate = h @ w[f"{p}.g"].T
    return (o.reshape(T, H * dv) * (gate * torch.sigmoid(gate))) @ w[f"{p}.o"].T


def parallel_mixer(h, w, p, c, eps):
    return (c["left_scale"] * capped_biased_attention(h, w, f"{p}.left", c["left"], eps)
            + c["right_scale"] * gated_linear_attention(h, w, f"{p}.right", c["right"], eps))


MIXERS = {"parallel": parallel_mixer}


# ----------------------------------------------------------------------------- feed-forward


def clamped_glu(h, w, p, c):
    """gate clipped from above, up clipped on both sides; gate * sigmoid(1.702 gate) * (up + 1)."""
    lim = c["limit"]
    g = torch.clamp(h @ w[f"{p}.gate"].T, max=lim)
    u = torch.clamp(h @ w[f"{p}.up"].T, -lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[f"{p}.down"].T


FEED_FORWARDS = {"dense": clamped_glu}


# ----------------------------------------------------------------------------- the model


def forward(cfg: dict, w: dict, ids, layers_out: list | None = None):
    """Logits [T, vocab] (float64) of one whole sequence; ``layers_out`` collects the residual
    stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(ids).long()]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}"
        mixed = MIXERS[layer["type"]](layer_norm(x, w[f"{p}.norm1"], eps), w, f"{p}.mix", layer["mixer"], eps)
        x = x + layer_norm(mixed, w[f"{p}.norm1b"], eps) * w[f"{p}.ls1"]
        if layer.get("mlp") is not None:
            y = FEED_FORWARDS[layer["mlp"]["kind"]](layer_norm(x, w[f"{p}.norm2"], eps), w, f"{p}.mlp", layer["mlp"])
            x = x + layer_norm(y, w[f"{p}.norm2b"], eps) * w[f"{p}.ls2"]
        if layers_out is not None:
            layers_out.append(x.clone())
    return (layer_norm(x, w["final.norm"], eps) @ w["embed"].T) * cfg["logit_scale"]

"""A plain, slow forward pass of the Tosisun design: whole sequences, no cache, no paging, one function per
mechanism, float32 or float64 torch on the CPU.  It shares no code with the engine: it reads a model folder with
``json`` and the ``safetensors`` package and writes every sum as a loop or a dense matrix expression.

The design in short (x_t is the residual stream of token t, positions count from 0):

* x = table[token]; every layer: x <- x + LN1(mixer(x)); x <- x + LN2(ff(x)) (the sublayers read x itself, the layer
  norm with gain and bias sits on their output); logits = cap * tanh(head(LN_final(x)) / cap).
* mixer "attention": grouped-query softmax attention over all earlier positions.  q, k, v are projections with
  bias that then pass a short causal convolution over time (per channel), q and k an RMS norm over the whole
  projection (all heads at once), and a split-half rotation of the first dims of every head whose frequencies are
  stretched for long wavelengths; the softmax's denominator also holds exp(sink) of a learned number per head.
* ff "dense": down(relu(up x)^2).  ff "moe": experts down(g sigmoid(1.702 g) (u + 1)) with g = min(gate x, limit)
  and u = clamp(up x, -limit, limit), chosen by the largest router logits (with bias), weighted by the softmax over
  the chosen logits, plus a shared expert of the same form that every token uses.
* a layer may run with another layer's weights (``weights_of``).
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Sequence

import torch


# --------------------------------------------------------------------------
# mechanisms
# --------------------------------------------------------------------------
def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    """(x - mean) / sqrt(var + eps) * w + b over the last axis, var the mean of squared deviations."""
    mu = x.mean(dim=-1, keepdim=True)
    d = x - mu
    var = (d * d).mean(dim=-1, keepdim=True)
    return d / torch.sqrt(var + eps) * w + b


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def short_conv(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, K]: y_t = sum_j taps[:, j] * x_{t - (K-1) + j}, zeros before the start."""
    T, C = x.shape
    K = taps.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(K):
            s = t - (K - 1) + j
            if s >= 0:
                y[t] += taps[:, j] * x[s]
    return y


def stretched_frequencies(dims: int, base: float, scaling) -> List[float]:
    """f_i = base^(-2i/dims), i < dims/2; with ``scaling`` (factor, low, high, original) a frequency whose
    wavelength 2 pi / f is longer than original/low is divided by factor, one shorter than original/high stays,
    and between the two the divided and the plain frequency are mixed linearly in original/wavelength."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wl = 2.0 * math.pi / f
            if wl < orig / high:
                pass
            elif wl > orig / low:
                f = f / factor
            else:
                s = (orig / wl - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate_half(x: torch.Tensor, pos: torch.Tensor, freqs: Sequence[float]) -> torch.Tensor:
    """x [T, heads, d]: dims i and i + R/2 (R = 2 len(freqs)) of every head turn by pos * freqs[i]; the rest passes."""
    out = x.clone()
    half = len(freqs)
    for i, f in enumerate(freqs):
        a = (pos.to(torch.float64) * f).to(x.dtype).view(-1, 1)
        u, v = x[..., i], x[..., i + half]
        out[..., i] = u * torch.cos(a) - v * torch.sin(a)
        out[..., i + half] = v * torch.cos(a) + u * torch.sin(a)
    return out


def sink_attention(q, k, v, scale: float, sink: torch.Tensor, group: int) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, dv]; head h reads key/value head h // group; token t sees 0..t; the
    softmax's denominator also counts exp(sink[h])."""
    T, H, _ = q.shape
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for h in range(H):
        g = h // group
        for t in range(T):
            s = (k[:t + 1, g] @ q[t, h]) * scale
            m = torch.maximum(s.max(), sink[h])
            e = torch.exp(s - m)
            den = e.sum() + torch.exp(sink[h] - m)
            out[t, h] = (e / den) @ v[:t + 1, g]
    return out


def relu_squared_mlp(x, up, down):
    z = torch.clamp(x @ up.T, min=0.0)
    return (z * z) @ down.T


def clamped_expert(x, gate, up, down, limit: float):
    g = torch.clamp(x @ gate.T, max=limit)
    u = torch.clamp(x @ up.T, min=-limit, max=limit)
    y = g * torch.sigmoid(1.702 * g) * (u + 1.0)
    return y @ down.T


def route(z: torch.Tensor, top: int):
    """z [T, E]: the ``top`` largest logits of every token (the lowest index among equals) and the softmax over them."""
    T, E = z.shape
    idx = torch.zeros(T, top, dtype=torch.long)
    wt = torch.zeros(T, top, dtype=z.dtype)
    for t in range(T):
        order = sorted(range(E), key=lambda e: (-float(z[t, e]), e))[:top]
        chosen = z[t, order]
        e = torch.exp(chosen - chosen.max())
        idx[t] = torch.tensor(order)
        wt[t] = e / e.sum()
    return idx, wt


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------
def load_folder(folder: str, dtype=torch.float64):
    from safetensors import safe_open
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w: Dict[str, torch.Tensor] = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            w[name] = t.to(dtype) if t.is_floating_point() else t
    return cfg, w


def attention_mixer(cfg, m, w, p: str, x: torch.Tensor) -> torch.Tensor:
    T = x.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    eps = float(cfg["norm"]["eps"])
    q = x @ w[p + "q"].T + w[p + "q.b"]
    k = x @ w[p + "k"].T + w[p + "k.b"]
    v = x @ w[p + "v"].T + w[p + "v.b"]
    q, k, v = short_conv(q, w[p + "q.conv"]), short_conv(k, w[p + "k.conv"]), short_conv(v, w[p + "v.conv"])
    q = rms(q, eps) * w[p + "q.norm"]
    k = rms(k, eps) * w[p + "k.norm"]
    rot = m["rot"]
    freqs = stretched_frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
    pos = torch.arange(T)
    q = rotate_half(q.view(T, H, d), pos, freqs)
    k = rotate_half(k.view(T, G, d), pos, freqs)
    o = sink_attention(q, k, v.view(T, G, dv), float(m["scale"]), w[p + "sink"], H // G)
    return o.reshape(T, H * dv) @ w[p + "o"].T


def feed_forward(cfg, mlp, w, p: str, x: torch.Tensor, margins=None) -> torch.Tensor:
    if mlp["kind"] == "dense":
        return relu_squared_mlp(x, w[p + "up"], w[p + "down"])
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    limit = float(mlp["expert"]["limit"])
    z = x @ w[p + "router"].T + w[p + "router.b"]
    if margins is not None and top < E:
        # how far the last chosen logit lies above the first one left out: a choice within rounding is a close call
        zs = torch.sort(z, dim=1, descending=True).values
        margins.append(zs[:, top - 1] - zs[:, top])
    idx, wt = route(z, top)
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for c in range(top):
            e = int(idx[t, c])
            out[t] += wt[t, c] * clamped_expert(x[t:t + 1], w[f"{p}e{e}.gate"], w[f"{p}e{e}.up"], w[f"{p}e{e}.down"], limit)[0]
    sh = mlp.get("shared")
    if sh is not None:
        out = out + clamped_expert(x, w[p + "shared.gate"], w[p + "shared.up"], w[p + "shared.down"], float(sh["limit"]))
    return out


def forward(cfg, w, tokens: Sequence[int], return_layers: bool = False, margins=None):
    """Logits [T, vocab] of a whole sequence (and the residual stream after every layer).  ``margins``: a list that
    receives, for every layer with a router that leaves experts out, each token's margin of the choice [T]."""
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.tensor(list(tokens), dtype=torch.long)]
    after = []
    for i, layer in enumerate(cfg["layers"]):
        src = layer.get("weights_of")
        p = f"l{i if src is None else int(src)}."
        if layer["type"] != "attention":
            raise ValueError(f"layer {i}: unknown type {layer['type']!r}")
        a = attention_mixer(cfg, layer["mixer"], w, p + "mix.", x)
        x = x + layer_norm(a, w[p + "norm1"], w[p + "norm1.b"], eps)
        if layer.get("mlp") is not None:
            f = feed_forward(cfg, layer["mlp"], w, p + "mlp.", x, margins)
            x = x + layer_norm(f, w[p + "norm2"], w[p + "norm2.b"], eps)
        after.append(x.clone())
    y = layer_norm(x, w["final.norm"], w["final.norm.b"], eps) @ w["head"].T
    cap = cfg.get("logit_softcap")
    if cap:
        y = float(cap) * torch.tanh(y / float(cap))
    return (y, torch.stack(after)) if return_layers else y


def greedy_generate(cfg, w, prompt: Sequence[int], new_tokens: int) -> List[int]:
    ids = list(prompt)
    out = []
    for _ in range(new_tokens):
        nxt = int(torch.argmax(forward(cfg, w, ids)[-1]))
        out.append(nxt)
        ids.append(nxt)
    return out

"""A plain, slow forward pass of the Dedelorn design: whole sequences, no cache, no paging, one function
per mechanism, float32 or float64 torch on the CPU.  It shares no code with the engine: it reads a model
folder with ``json`` and the ``safetensors`` package, and loops token by token where the design recurs.

The design in short (x_t is the residual stream of token t, positions count from 0):

* x = rms(table[token]) * g_embed; every layer: n = rms(x) * g; x <- x + mixer(n) + ff(n); logits = head(rms(x) * g_final).
* mixer "delta": a gated delta rule per head over a matrix state S [dim, vdim];
* mixer "latent_attention": softmax attention inside a sliding window whose keys and values are made from one
  short latent per token plus one rotated key part that all heads share; a layer may read another layer's latents;
* ff "dense": down(gelu_tanh(gate n) * (up n)); ff "moe": experts down(gelu_erf(up n)) chosen by a softmax router
  with an additive correction that steers the choice and not the weights.
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
def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1.0 + torch.exp(-z))


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def rotate_pairs(x: torch.Tensor, pos: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [T, ..., d]: the first ``dims`` values of the last axis turn in neighbouring pairs (2i, 2i+1) by the angle
    pos * base^(-2i/dims); the rest passes."""
    out = x.clone()
    T = x.shape[0]
    for i in range(dims // 2):
        a = pos.to(x.dtype) * (float(base) ** (-2.0 * i / dims))
        a = a.view((T,) + (1,) * (x.dim() - 2))
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * torch.cos(a) - v * torch.sin(a)
        out[..., 2 * i + 1] = v * torch.cos(a) + u * torch.sin(a)
    return out


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


def delta_rule(q, k, v, beta, g):
    """q, k [T, dim] (unit length; q scaled), v [T, vdim], beta, g [T]: one head's recurrence, token by token."""
    T, dim = q.shape
    S = torch.zeros(dim, v.shape[1], dtype=q.dtype)
    out = torch.zeros_like(v)
    for t in range(T):
        S = g[t] * S
        u = beta[t] * (v[t] - S.t() @ k[t])
        S = S + torch.outer(k[t], u)
        out[t] = S.t() @ q[t]
    return out


def delta_mixer(n: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    T = n.shape[0]
    heads, kvh, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(n @ w[p + "q"].t(), w[p + "q.conv"])).view(T, kvh, dim)
    k = silu(short_conv(n @ w[p + "k"].t(), w[p + "k.conv"])).view(T, kvh, dim)
    v = silu(short_conv(n @ w[p + "v"].t(), w[p + "v.conv"])).view(T, heads, vdim)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(n @ w[p + "b"].t())                                    # [T, heads]
    g = torch.exp(-torch.exp(w[p + "A_log"]) * softplus(n @ w[p + "a"].t() + w[p + "dt_bias"]))
    gate = silu(n @ w[p + "g"].t()).view(T, heads, vdim)
    out = torch.zeros(T, heads, vdim, dtype=n.dtype)
    for h in range(heads):
        kh = h // (heads // kvh)
        o = delta_rule(q[:, kh], k[:, kh], v[:, h], beta[:, h], g[:, h])
        out[:, h] = rms(o, eps) * w[p + "norm"] * gate[:, h]
    return out.reshape(T, heads * vdim) @ w[p + "o"].t()


def latents(n: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float, pos: torch.Tensor):
    """What a latent-attention layer keeps per token: the normed latent c [T, kv_rank] and the rotated shared key
    part [T, rot_dim]."""
    r = m["kv_rank"]
    d = n @ w[p + "dkv"].t()
    c = rms(d[:, :r], eps) * w[p + "dkv.norm"]
    kr = rotate_pairs(d[:, r:], pos, m["rot"]["base"], m["rot"]["dims"])
    return c, kr


def latent_attention(n, w, p, m, c, kr, pos):
    T = n.shape[0]
    H, dim, rd, vdim = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    q = (n @ w[p + "q"].t()).view(T, H, dim + rd)
    q_plain = q[..., :dim]
    q_rot = rotate_pairs(q[..., dim:], pos, m["rot"]["base"], m["rot"]["dims"])
    k_plain = (c @ w[p + "uk"].t()).view(T, H, dim)
    val = (c @ w[p + "uv"].t()).view(T, H, vdim)
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = (j <= i)
    size = (m.get("mask") or {}).get("size")
    if size:
        seen &= (i - j) < size
    out = torch.zeros(T, H, vdim, dtype=n.dtype)
    for h in range(H):
        s = (q_plain[:, h] @ k_plain[:, h].t() + q_rot[:, h] @ kr.t()) * m["scale"]
        s = s.masked_fill(~seen, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ val[:, h]
    return out.reshape(T, H * vdim) @ w[p + "o"].t()


def dense_ff(n, w, p):
    return (gelu_tanh(n @ w[p + "gate"].t()) * (n @ w[p + "up"].t())) @ w[p + "down"].t()


def route(n, w, p, router):
    """For every token the chosen experts and their weights."""
    z = n @ w[p + "router"].t()
    s = torch.softmax(z, dim=-1)
    choice = s + w[p + "correction"]
    idx = torch.topk(choice, router["top"], dim=-1).indices
    return idx, torch.gather(s, 1, idx) * router["scale"]


def moe_ff(n, w, p, mlp):
    idx, wt = route(n, w, p, mlp["router"])
    out = torch.zeros_like(n)
    for t in range(n.shape[0]):
        for e, a in zip(idx[t].tolist(), wt[t]):
            out[t] += a * (gelu_erf(n[t] @ w[f"{p}e{e}.up"].t()) @ w[f"{p}e{e}.down"].t())
    return out


# --------------------------------------------------------------------------
# the whole model
# --------------------------------------------------------------------------
def forward(cfg: dict, w: Dict[str, torch.Tensor], ids: Sequence[int], layers_out: List[torch.Tensor] = None):
    """Logits [T, vocab] of one sequence from position 0; ``layers_out`` collects the stream after every layer."""
    eps = cfg["norm"]["eps"]
    T = len(ids)
    pos = torch.arange(T)
    x = rms(w["embed"][torch.tensor(list(ids), dtype=torch.long)], eps) * w["embed.norm"]
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        n = rms(x, eps) * w[p + "norm1"]
        m = layer["mixer"]
        if layer["type"] == "delta":
            a = delta_mixer(n, w, p + "mix.", m, eps)
        elif layer["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                kept[i] = latents(n, w, p + "mix.", m, eps, pos)
                src = i
            a = latent_attention(n, w, p + "mix.", m, *kept[src], pos)
        else:
            raise ValueError(layer["type"])
        mlp = layer.get("mlp")
        if mlp is None:
            f = 0.0
        elif mlp["kind"] == "dense":
            f = dense_ff(n, w, p + "mlp.")
        else:
            f = moe_ff(n, w, p + "mlp.", mlp)
        x = x + (a + f)
        if layers_out is not None:
            layers_out.append(x.clone())
    return (rms(x, eps) * w["final.norm"]) @ w["head"].t()


def load_folder(folder: str, dtype=torch.float32):
    from safetensors import safe_open
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as st:
        for name in st.keys():
            t = st.get_tensor(name)
            w[name] = t.to(dtype) if t.is_floating_point() else t
    return cfg, w


def greedy_generate(cfg, w, prompt: Sequence[int], n: int) -> List[int]:
    ids = list(prompt)
    out = []
    for _ in range(n):
        logits = forward(cfg, w, ids)[-1]
        best = int(torch.argmax(logits))            # the lowest index among equals
        out.append(best)
        ids.append(best)
    return out

"""A plain, slow implementation of the Nufavik decoder: whole sequences, no cache, one function per
mechanism, CPU only.  It shares no code with the engine: it reads config.json and model.safetensors by
itself and works on torch tensors in ``dtype`` (float64 by default).

Notation.  T tokens, width W.  A layer has one norm and two branches that both read it:
    n = w * x / sqrt(mean(x^2) + eps),    x <- x + (mixer(n) + ff(n)).
The mixer is grouped-query attention whose projected q, k and v each pass a short causal convolution
over time before q and k are rotated; a query sees the last ``size`` keys and the first ``keep_first``
keys of its sequence, and the softmax has a 1 added to its denominator.  The feed-forward is a
mixture of squared-relu experts of which some are the identity.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch


def read_folder(folder: str):
    from safetensors import safe_open
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name)
    return cfg, tensors


# ---- norm ---------------------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w


# ---- convolution over time --------------------------------------------------------------------------
def causal_conv(u: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """u [T, C], w [C, taps]:  y_t = sum_j w[:, j] u_(t - taps + 1 + j), nothing before the start."""
    T, taps = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] = y[t] + w[:, j] * u[s]
    return y


# ---- rotation -----------------------------------------------------------------------------------------
def rotate_half_split(v: torch.Tensor, pos: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """v [T, heads, D]: coordinate i < dims / 2 is paired with i + dims / 2 and the pair is turned by
    pos * base^(-2 i / dims); coordinates from dims on stay."""
    out = v.clone()
    half = dims // 2
    p = pos.to(v.dtype).reshape(-1, 1)
    for i in range(half):
        a = p * (base ** (-2.0 * i / dims))
        c, s = torch.cos(a), torch.sin(a)
        a0, a1 = v[..., i], v[..., i + half]
        out[..., i] = a0 * c - a1 * s
        out[..., i + half] = a1 * c + a0 * s
    return out


# ---- mask and softmax ---------------------------------------------------------------------------------
def sees(i: int, j: int, size: int, keep_first: int) -> bool:
    return j <= i and (i - j < size or j < keep_first)


def softmax_with_sink(s: torch.Tensor) -> torch.Tensor:
    """p_j = exp(s_j) / (1 + sum_k exp(s_k)): one more entry of score 0 that carries no value."""
    m = max(float(s.max()), 0.0)
    e = torch.exp(s - m)
    return e / (math.exp(-m) + e.sum())


# ---- the mixer ----------------------------------------------------------------------------------------
def attention(h: torch.Tensor, pos: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, m: dict) -> torch.Tensor:
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]

    def proj(name):
        y = h @ w[f"{pre}.{name}"].T + w[f"{pre}.{name}.b"]
        return causal_conv(y, w[f"{pre}.{name}.conv"])

    q = proj("q").reshape(T, H, D)
    k = proj("k").reshape(T, G, D)
    v = proj("v").reshape(T, G, Dv)
    base, dims = float(m["rot"]["base"]), int(m["rot"]["dims"])
    q = rotate_half_split(q, pos, base, dims)
    k = rotate_half_split(k, pos, base, dims)
    size, keep = int(m["mask"]["size"]), int(m["mask"]["keep_first"])
    scale = float(m["scale"])
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for i in range(T):
        js = [j for j in range(T) if sees(int(pos[i]), int(pos[j]), size, keep)]
        for hh in range(H):
            g = hh // (H // G)
            s = torch.stack([(q[i, hh] * k[j, g]).sum() * scale for j in js])
            p = softmax_with_sink(s)
            for pj, j in zip(p, js):
                out[i, hh] = out[i, hh] + pj * v[j, g]
    return out.reshape(T, H * Dv) @ w[f"{pre}.o"].T


# ---- the feed-forward ---------------------------------------------------------------------------------
def route(z: torch.Tensor, correction: torch.Tensor, top: int, scale: float):
    """z [E] router logits of one token -> (chosen experts, their weights)."""
    s = torch.softmax(z, dim=-1)
    choice = s + correction
    order = sorted(range(z.shape[0]), key=lambda e: (-float(choice[e]), e))[:top]
    chosen = torch.stack([s[e] for e in order])
    return order, chosen / (chosen.sum() + 1e-20) * scale


def expert(h: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    a = torch.relu(up @ h)
    return down @ (a * a)


def mixture(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, mlp: dict, router_dtype=None) -> torch.Tensor:
    r = mlp["router"]
    E, ident, top, scale = int(r["experts"]), int(r["identity"]), int(r["top"]), float(r["scale"])
    out = torch.zeros_like(h)
    wr, corr = w[f"{pre}.router"], w[f"{pre}.correction"]
    for t in range(h.shape[0]):
        z = wr @ h[t]
        ids, wts = route(z, corr, top, scale)
        for e, wt in zip(ids, wts):
            if e >= E:
                assert e < E + ident
                out[t] = out[t] + wt * h[t]
            else:
                out[t] = out[t] + wt * expert(h[t], w[f"{pre}.e{e}.up"], w[f"{pre}.e{e}.down"])
    return out


# ---- the model ----------------------------------------------------------------------------------------
def forward(cfg: dict, tensors: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64,
            layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from its start; layers_out, if a list, gets the stream after
    every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps = float(cfg["norm"]["eps"])
    ids = torch.tensor(tokens, dtype=torch.long)
    pos = torch.arange(len(tokens))
    x = w["embed"][ids] * float(cfg["embedding"]["scale"])
    for i, layer in enumerate(cfg["layers"]):
        if layer["type"] != "attention":
            raise ValueError(f"layer {i}: mixer {layer['type']!r}")
        n = rms_norm(x, w[f"l{i}.norm1"], eps)
        y = attention(n, pos, w, f"l{i}.mix", layer["mixer"])
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] != "moe":
                raise ValueError(f"layer {i}: feed-forward {layer['mlp']['kind']!r}")
            y = y + mixture(n, w, f"l{i}.mlp", layer["mlp"])
        x = x + y
        if layers_out is not None:
            layers_out.append(x.clone())
    x = rms_norm(x, w["final.norm"], eps)
    return x @ w["embed"].T

"""A plain, slow implementation of the Zarorax decoder: whole sequences, no cache, one
function per mechanism, CPU only.  It shares no code with the engine: it reads
config.json and model.safetensors by itself and works on lists and torch tensors in
``dtype`` (float64 by default).

Notation.  T tokens, width W.  rms(v) = sqrt(mean(v^2) + eps).  A layer keeps a
post-norm stream:  x <- n1(alpha x + mixer(x + conv(x))),  x <- n2(alpha x + ff(x)),
n(v) = g v / rms(v) with one number g.
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


# ---- norms -------------------------------------------------------------------------------
def unit_rms(v: torch.Tensor, eps: float) -> torch.Tensor:
    """v / sqrt(mean(v^2) + eps) over the last dimension."""
    return v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)


def scalar_norm(v: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    """The layer norms and the final norm: one gain for all coordinates."""
    return unit_rms(v, eps) * g.reshape(())


def vector_norm(v: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """The latents' norms: a gain per coordinate."""
    return unit_rms(v, eps) * weight


# ---- the convolution before a mixer ------------------------------------------------------------
def short_conv(h: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """h [T, W], w [W, taps]:  out_t = h_t + sum_j w[:, j] h_(t - taps + 1 + j), zeros before the start."""
    T, taps = h.shape[0], w.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] = out[t] + w[:, j] * h[s]
    return out


# ---- rotation ------------------------------------------------------------------------------------
def rotate_interleaved(v: torch.Tensor, pos: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """v [T, ..., D]: the first ``dims`` coordinates in neighbouring pairs (2i, 2i + 1), turned by
    pos * base^(-2i/dims); the rest unchanged."""
    out = v.clone()
    shape = [v.shape[0]] + [1] * (v.dim() - 2)
    p = pos.to(v.dtype).reshape(shape)
    for i in range(dims // 2):
        a = p * (base ** (-2.0 * i / dims))
        c, s = torch.cos(a), torch.sin(a)
        u, w = v[..., 2 * i], v[..., 2 * i + 1]
        out[..., 2 * i] = u * c - w * s
        out[..., 2 * i + 1] = w * c + u * s
    return out


# ---- the two mixers ------------------------------------------------------------------------------
def latent_attention(h: torch.Tensor, pos: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, m: dict,
                     eps: float, gated: bool) -> torch.Tensor:
    """Attention whose keys and values are expanded from one latent per token, with one rotated key
    part shared by the heads.  ``gated``: direct queries and a sigmoid gate on the heads' outputs;
    else queries through a normed latent of their own."""
    T = h.shape[0]
    H, dn, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    if gated:
        q = h @ w[f"{pre}.q"].t()
    else:
        cq = vector_norm(h @ w[f"{pre}.dq"].t(), w[f"{pre}.dq.norm"], eps)
        q = cq @ w[f"{pre}.uq"].t()
    q = q.view(T, H, dn + dr)
    q_plain, q_rot = q[..., :dn], q[..., dn:]
    kv = h @ w[f"{pre}.dkv"].t()
    c = vector_norm(kv[:, :r], w[f"{pre}.dkv.norm"], eps)
    k_rot = kv[:, r:]                                       # [T, dr], one for all heads
    base, dims = float(m["rot"]["base"]), int(m["rot"]["dims"])
    q_rot = rotate_interleaved(q_rot, pos, base, dims)
    k_rot = rotate_interleaved(k_rot, pos, base, dims)
    k_plain = (c @ w[f"{pre}.uk"].t()).view(T, H, dn)
    v = (c @ w[f"{pre}.uv"].t()).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for head in range(H):
        scores = (q_plain[:, head] @ k_plain[:, head].t() + q_rot[:, head] @ k_rot.t()) * m["scale"]
        mask = pos[:, None] >= pos[None, :]
        scores = scores.masked_fill(~mask, float("-inf"))
        out[:, head] = torch.softmax(scores, dim=-1) @ v[:, head]
    o = out.reshape(T, H * dv)
    if gated:
        o = o * torch.sigmoid(h @ w[f"{pre}.g"].t())
    return o @ w[f"{pre}.o"].t()


# ---- the feed-forwards ---------------------------------------------------------------------------
def poly_ffn(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, eps: float) -> torch.Tensor:
    z = h @ w[f"{pre}.up"].t()
    a, b, c, e = [w[f"{pre}.act"][i] for i in range(4)]
    act = a * unit_rms(z, eps) + b * unit_rms(z * z, eps) + c * unit_rms(z * z * z, eps) + e
    return act @ w[f"{pre}.down"].t()


def route(h: torch.Tensor, router: torch.Tensor, r: dict):
    """Per token: the chosen experts and their weights.  softmax over all experts; the groups of
    neighbours are ranked by their best expert, only the best ``keep`` groups stay; the ``top`` largest
    scores among those are chosen and weigh the experts as they are."""
    E, top = r["experts"], r["top"]
    count, keep = r["groups"]["count"], r["groups"]["keep"]
    s = torch.softmax((h.double() @ router.double().t()), dim=-1)
    chosen = []
    for t in range(h.shape[0]):
        per = E // count
        best = [max(s[t, g * per:(g + 1) * per]).item() for g in range(count)]
        kept = sorted(range(count), key=lambda g: -best[g])[:keep]
        allowed = [e for g in kept for e in range(g * per, (g + 1) * per)]
        ids = sorted(allowed, key=lambda e: -s[t, e].item())[:top]
        chosen.append([(e, s[t, e].item()) for e in ids])
    return chosen


def expert_ffn(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, limit: float) -> torch.Tensor:
    g = torch.clamp(h @ w[f"{pre}.gate"].t(), max=limit)
    u = torch.clamp(h @ w[f"{pre}.up"].t(), min=-limit, max=limit)
    y = g * torch.sigmoid(1.702 * g) * (u + 1)
    return y @ w[f"{pre}.down"].t()


def moe_ffn(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, mlp: dict) -> torch.Tensor:
    chosen = route(h, w[f"{pre}.router"], mlp["router"])
    out = torch.zeros_like(h)
    for t, picks in enumerate(chosen):
        for e, weight in picks:
            out[t] = out[t] + weight * expert_ffn(h[t:t + 1], w, f"{pre}.e{e}", mlp["expert"]["limit"])[0]
    return out


# ---- the model -------------------------------------------------------------------------------------
def forward(cfg: dict, tensors: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64,
            layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  ``layers_out``: a list that gets the stream after
    every layer run."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    pos = torch.arange(len(tokens))
    x = w["embed"][torch.tensor(tokens)]
    for i, layer in enumerate(cfg["layers"]):
        src = layer.get("weights_of", i)
        pre = f"l{src}"
        h = short_conv(x, w[f"{pre}.canon1"])
        y = latent_attention(h, pos, w, f"{pre}.mix", layer["mixer"], eps, gated=layer["type"] == "latent_attention_2")
        x = scalar_norm(alpha * x + y, w[f"{pre}.norm1"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            y = poly_ffn(x, w, f"{pre}.mlp", eps) if mlp["kind"] == "dense" else moe_ffn(x, w, f"{pre}.mlp", mlp)
            x = scalar_norm(alpha * x + y, w[f"{pre}.norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = scalar_norm(x, w["final.norm"], eps)
    return x @ w["head"].t()


def greedy_generate(cfg: dict, tensors: Dict[str, torch.Tensor], prompt: List[int], n: int) -> List[int]:
    toks, out = list(prompt), []
    for _ in range(n):
        nxt = int(forward(cfg, tensors, toks)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out

"""Tiny Nufavik configurations for tests, with random weights of a scale at which every mechanism moves the
logits (scores of order one, router scores that differ, corrections that change choices, biases and gains away
from zero and one), written as model folders.  Sizes differ from one another wherever the design allows."""
import json
import math
import os

import torch


def _layer(heads, kv, dim, vdim, conv, size, keep, dims, scale, base=10000.0, mlp=None):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv, "scale": scale,
                      "mask": {"size": size, "keep_first": keep}, "rot": {"base": base, "dims": dims}},
            "mlp": mlp}


def _moe(experts, identity, top, ff, scale):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top, "scale": scale}}


# A: value heads larger and smaller than key heads, two to five taps, a layer without a feed-forward, a layer that
# rotates whole heads and one that rotates nothing, windows shorter than a page and longer than two, kept first keys
# within a page, beyond one, and more than the window is long
NA = {"architecture": "Nufavik", "vocab": 211, "width": 96, "embedding": {"scale": 0.7}, "norm": {"eps": 1e-6},
      "layers": [
          _layer(4, 2, 16, 24, 3, 24, 3, 8, 0.3, 1000.0, _moe(6, 2, 2, 40, 1.25)),
          _layer(3, 3, 24, 8, 2, 7, 0, 24, 0.25, 50000.0, None),
          _layer(6, 1, 8, 40, 5, 37, 20, 0, 0.4, 100.0, _moe(3, 1, 3, 24, 0.8)),
          _layer(2, 1, 32, 16, 4, 9, 12, 2, 0.2, 10.0, _moe(5, 0, 1, 56, 2.0)),
      ]}
# B: sizes that fill whole tiles of the matrix-unit kernels (heads of 64 and 128, groups of 4 and 1)
NB = {"architecture": "Nufavik", "vocab": 300, "width": 128, "embedding": {"scale": 2.0}, "norm": {"eps": 1e-5},
      "layers": [
          _layer(8, 2, 64, 64, 4, 33, 5, 16, 0.11, 500000.0, _moe(8, 0, 1, 64, 1.0)),
          _layer(4, 4, 128, 96, 3, 100, 17, 64, 0.08, 10000.0, _moe(4, 3, 3, 128, 2.5)),
      ]}
# C: values that are 1 or equal: embedding scale 1, route scale 1, one head, keys and values of one size, one expert
# and one identity expert that are both always chosen, one tap, a window that no sequence of the tests outgrows
NC = {"architecture": "Nufavik", "vocab": 150, "width": 64, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-5},
      "layers": [
          _layer(1, 1, 16, 16, 1, 1000, 4, 16, 0.25, 2000.0, _moe(1, 1, 2, 32, 1.0)),
          _layer(16, 1, 16, 16, 3, 1, 1, 8, 0.25, 2000.0, _moe(70, 3, 5, 8, 1.0)),
      ]}
TINY = {"A": (NA, 31, 8), "B": (NB, 32, 16), "C": (NC, 33, 4)}      # config, seed, page size


def tensor_shapes(cfg):
    """name -> (shape, kind of values) of every tensor of a configuration, from the design's naming."""
    w = cfg["width"]
    out = {"embed": ((cfg["vocab"], w), "embed"), "final.norm": ((w,), "gains")}
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}"
        out[f"{p}.norm1"] = ((w,), "gains")
        for name, n in (("q", m["heads"] * m["dim"]), ("k", m["kv_heads"] * m["dim"]), ("v", m["kv_heads"] * m["vdim"])):
            out[f"{p}.mix.{name}"] = ((n, w), "matrix")
            out[f"{p}.mix.{name}.b"] = ((n,), "bias")
            out[f"{p}.mix.{name}.conv"] = ((n, m["conv"]), "conv")
        out[f"{p}.mix.o"] = ((w, m["heads"] * m["vdim"]), "matrix")
        mlp = layer["mlp"]
        if mlp is None:
            continue
        r, f = mlp["router"], mlp["expert"]["ff"]
        out[f"{p}.mlp.router"] = ((r["experts"] + r["identity"], w), "router")
        out[f"{p}.mlp.correction"] = ((r["experts"] + r["identity"],), "correction")
        for e in range(r["experts"]):
            out[f"{p}.mlp.e{e}.up"] = ((f, w), "matrix")
            out[f"{p}.mlp.e{e}.down"] = ((w, f), "matrix")
    return out


def random_tensors(cfg, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, (shape, kind) in tensor_shapes(cfg).items():
        n = lambda *s: torch.randn(*s, generator=g)
        if kind == "embed":
            t = n(*shape)
        elif kind == "matrix":
            t = n(*shape) * (1.6 / math.sqrt(shape[-1]))
        elif kind == "router":
            t = n(*shape) * (3.0 / math.sqrt(shape[-1]))
        elif kind == "correction":
            t = n(*shape) * 0.15
        elif kind == "bias":
            t = n(*shape) * 0.3
        elif kind == "conv":
            t = n(*shape) * 0.6
        elif kind == "gains":
            t = 1.0 + 0.3 * n(*shape)
        out[name] = t.to(dtype)
    return out


def write_folder(folder, cfg, tensors):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def make_folder(tmp, which, dtype=torch.bfloat16):
    cfg, seed, _ = TINY[which]
    return write_folder(os.path.join(str(tmp), f"nufavik_{which}"), cfg, random_tensors(cfg, seed, dtype))

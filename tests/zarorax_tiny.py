"""Tiny Zarorax configurations for tests, with random weights of a scale at which every mechanism
moves the logits (scores of order one, router scores that differ, gains away from one), written as model
folders.  Sizes differ from one another wherever the design allows."""
import json
import math
import os

import torch

# P: three tokens of convolution, queries through a latent, value size unlike the key sizes, fewer rotated
# numbers than the rotated part holds; a dense layer, a mixture with groups, a layer run again.
ZP = {
    "architecture": "Zarorax", "vocab": 211, "width": 96, "postln_alpha": 1.5, "norm": {"eps": 1e-6},
    "canon": {"taps": 3},
    "layers": [
        {"type": "latent_attention",
         "mixer": {"heads": 3, "dim": 16, "rot_dim": 8, "vdim": 24, "kv_rank": 40, "q_rank": 56, "scale": 0.21,
                   "rot": {"base": 1000.0, "dims": 6}},
         "mlp": {"kind": "dense", "ff": 160}},
        {"type": "latent_attention_2",
         "mixer": {"heads": 5, "dim": 8, "rot_dim": 12, "vdim": 20, "kv_rank": 24, "scale": 0.3,
                   "rot": {"base": 30000.0, "dims": 12}},
         "mlp": {"kind": "moe", "expert": {"ff": 40, "limit": 0.8},
                 "router": {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}}}},
        {"type": "latent_attention",
         "mixer": {"heads": 3, "dim": 16, "rot_dim": 8, "vdim": 24, "kv_rank": 40, "q_rank": 56, "scale": 0.21,
                   "rot": {"base": 1000.0, "dims": 6}},
         "mlp": {"kind": "dense", "ff": 160}, "weights_of": 0},
        {"type": "latent_attention_2",
         "mixer": {"heads": 2, "dim": 24, "rot_dim": 4, "vdim": 16, "kv_rank": 72, "scale": 0.15,
                   "rot": {"base": 500.0, "dims": 4}},
         "mlp": None},
    ],
}
# Q: two taps, one head, one group, one expert chosen; sizes that fill whole tiles of the kernels
ZQ = {
    "architecture": "Zarorax", "vocab": 300, "width": 128, "postln_alpha": 3.0, "norm": {"eps": 1e-5},
    "canon": {"taps": 2},
    "layers": [
        {"type": "latent_attention_2",
         "mixer": {"heads": 1, "dim": 64, "rot_dim": 64, "vdim": 64, "kv_rank": 64, "scale": 0.09,
                   "rot": {"base": 10000.0, "dims": 64}},
         "mlp": {"kind": "moe", "expert": {"ff": 64, "limit": 2.0},
                 "router": {"experts": 4, "top": 1, "groups": {"count": 1, "keep": 1}}}},
        {"type": "latent_attention",
         "mixer": {"heads": 4, "dim": 16, "rot_dim": 16, "vdim": 16, "kv_rank": 96, "q_rank": 64, "scale": 0.17,
                   "rot": {"base": 100000.0, "dims": 16}},
         "mlp": {"kind": "moe", "expert": {"ff": 160, "limit": 1.0},
                 "router": {"experts": 8, "top": 3, "groups": {"count": 4, "keep": 4}}}},
    ],
}
# R: five taps (a state of four inputs), sixteen heads on a latent of 64
ZR = {
    "architecture": "Zarorax", "vocab": 150, "width": 64, "postln_alpha": 1.0, "norm": {"eps": 1e-5},
    "canon": {"taps": 5},
    "layers": [
        {"type": "latent_attention",
         "mixer": {"heads": 16, "dim": 16, "rot_dim": 16, "vdim": 8, "kv_rank": 64, "q_rank": 32, "scale": 0.18,
                   "rot": {"base": 2000.0, "dims": 16}},
         "mlp": {"kind": "dense", "ff": 96}},
        {"type": "latent_attention",
         "mixer": {"heads": 16, "dim": 16, "rot_dim": 16, "vdim": 8, "kv_rank": 64, "q_rank": 32, "scale": 0.18,
                   "rot": {"base": 2000.0, "dims": 16}},
         "mlp": {"kind": "dense", "ff": 96}, "weights_of": 0},
    ],
}
TINY = {"P": (ZP, 11, 8), "Q": (ZQ, 12, 16), "R": (ZR, 13, 4)}      # config, seed, page size


def tensor_shapes(cfg):
    """name -> (shape, kind of values) of every tensor of a configuration, from the design's naming."""
    w, out = cfg["width"], {"embed": ((cfg["vocab"], cfg["width"]), "embed"), "final.norm": ((), "gain"),
                            "head": ((cfg["vocab"], cfg["width"]), "matrix")}
    for i, layer in enumerate(cfg["layers"]):
        if "weights_of" in layer:
            continue
        m, p = layer["mixer"], f"l{i}"
        h, dq, dv, r = m["heads"], m["dim"] + m["rot_dim"], m["vdim"], m["kv_rank"]
        out[f"{p}.norm1"] = ((), "gain")
        out[f"{p}.canon1"] = ((w, cfg["canon"]["taps"]), "conv")
        if layer["type"] == "latent_attention":
            out[f"{p}.mix.dq"] = ((m["q_rank"], w), "matrix")
            out[f"{p}.mix.dq.norm"] = ((m["q_rank"],), "gains")
            out[f"{p}.mix.uq"] = ((h * dq, m["q_rank"]), "matrix")
        else:
            out[f"{p}.mix.q"] = ((h * dq, w), "matrix")
            out[f"{p}.mix.g"] = ((h * dv, w), "matrix")
        out[f"{p}.mix.dkv"] = ((r + m["rot_dim"], w), "matrix")
        out[f"{p}.mix.dkv.norm"] = ((r,), "gains")
        out[f"{p}.mix.uk"] = ((h * m["dim"], r), "matrix")
        out[f"{p}.mix.uv"] = ((h * dv, r), "matrix")
        out[f"{p}.mix.o"] = ((w, h * dv), "matrix")
        mlp = layer["mlp"]
        if mlp is None:
            continue
        out[f"{p}.norm2"] = ((), "gain")
        if mlp["kind"] == "dense":
            out[f"{p}.mlp.up"] = ((mlp["ff"], w), "matrix")
            out[f"{p}.mlp.down"] = ((w, mlp["ff"]), "matrix")
            out[f"{p}.mlp.act"] = ((4,), "coef")
        else:
            f = mlp["expert"]["ff"]
            out[f"{p}.mlp.router"] = ((mlp["router"]["experts"], w), "router")
            for e in range(mlp["router"]["experts"]):
                out[f"{p}.mlp.e{e}.gate"] = ((f, w), "matrix")
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
        elif kind == "conv":
            t = n(*shape) * 0.4
        elif kind == "gain":
            t = (1.0 + 0.3 * n(1)).reshape(())
        elif kind == "gains":
            t = 1.0 + 0.3 * n(*shape)
        elif kind == "coef":
            t = torch.tensor([0.9, 0.5, -0.4, 0.1]) + 0.1 * n(4)
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
    return write_folder(os.path.join(str(tmp), f"zarorax_{which}"), cfg, random_tensors(cfg, seed, dtype))

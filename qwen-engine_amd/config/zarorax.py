"""Typed configuration of the Zarorax decoder, read from config.json.

A post-norm decoder: every layer is a short causal convolution in front of a latent-attention mixer
(queries through a latent of their own, or direct queries with a sigmoid gate on the heads' outputs),
then a dense feed-forward with a polynomial activation or a routed mixture of experts, each followed
by an RMS norm with one gain over ``alpha * x + branch``.  ``layers`` lists the layers in running
order; an entry with ``weights_of: j`` runs layer j's weights again with a cache and state of its own.

Keys: architecture, vocab, width, postln_alpha, norm.eps, canon.taps, layers[i].type
(latent_attention | latent_attention_2), layers[i].mixer {heads, dim, rot_dim, vdim, kv_rank, q_rank,
scale, rot {base, dims}}, layers[i].mlp (null | {kind: dense, ff} | {kind: moe, expert {ff, limit},
router {experts, top, groups {count, keep}}}), layers[i].weights_of.  No size has a default.
"""
from __future__ import annotations

import copy
from typing import Any, Dict, List, Optional, Tuple

from .qwen3 import ConfigError
from .spec import (GroupedMoESpec, LatentAttentionSpec, ModelSpec, PolyNormMLPSpec, PostNormLayerSpec,
                   RopePairsSpec, ScalarRMSNormSpec, ScheduleEntry, ShortConvSpec)

ARCHITECTURE = "Zarorax"
MIXER_TYPES = {"latent_attention": False, "latent_attention_2": True}    # type -> direct queries and output gate
MAX_POSITIONS = 1 << 20      # the design names no limit; positions stay exact in 32-bit floats far beyond this


def _get(d: Dict[str, Any], path: str, where: str):
    cur: Any = d
    for key in path.split("."):
        if not isinstance(cur, dict) or key not in cur:
            raise ConfigError(f"config.json lacks {where}{path}")
        cur = cur[key]
    return cur


class ZaroraxConfig:
    architecture = ARCHITECTURE

    def __init__(self, d: Dict[str, Any]):
        self.raw = copy.deepcopy(d)
        self.vocab = int(_get(d, "vocab", ""))
        self.width = int(_get(d, "width", ""))
        self.alpha = float(_get(d, "postln_alpha", ""))
        self.eps = float(_get(d, "norm.eps", ""))
        self.taps = int(_get(d, "canon.taps", "")) if "canon" in d and d["canon"] is not None else 0
        self.layers: List[Dict[str, Any]] = list(_get(d, "layers", ""))
        self.max_positions = int(d.get("max_positions", MAX_POSITIONS))
        self.validate()

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ZaroraxConfig":
        return cls(d)

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(self.raw)

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("vocab and width must be positive")
        if not self.eps > 0:
            raise ConfigError("norm.eps must be positive")
        if self.taps < 0:
            raise ConfigError("canon.taps must not be negative")
        if not self.layers:
            raise ConfigError("the model has no layers")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]."
            if layer.get("type") not in MIXER_TYPES:
                raise ConfigError(f"{where}type is {layer.get('type')!r}; known: {sorted(MIXER_TYPES)}")
            src = layer.get("weights_of")
            if src is not None:
                if not (isinstance(src, int) and 0 <= src < len(self.layers)) or src == i or \
                        self.layers[src].get("weights_of") is not None:
                    raise ConfigError(f"{where}weights_of names layer {src!r}, which has no weights of its own")
            self._mixer(layer, where)
            self._ffn(layer, where)

    # ---- one layer's parts ---------------------------------------------------------------------------------
    def _mixer(self, layer: Dict[str, Any], where: str) -> LatentAttentionSpec:
        m = _get(layer, "mixer", where)
        w = where + "mixer."
        direct = MIXER_TYPES[layer["type"]]
        rot_dim = int(_get(m, "rot_dim", w))
        dims = int(_get(m, "rot.dims", w))
        if dims % 2 or not 0 <= dims <= rot_dim:
            raise ConfigError(f"{w}rot.dims = {dims} must be even and at most rot_dim = {rot_dim}")
        spec = LatentAttentionSpec(
            num_heads=int(_get(m, "heads", w)), head_dim=int(_get(m, "dim", w)), rot_dim=rot_dim,
            v_head_dim=int(_get(m, "vdim", w)), kv_rank=int(_get(m, "kv_rank", w)),
            scale=float(_get(m, "scale", w)), norm_eps=self.eps,
            q_rank=None if direct else int(_get(m, "q_rank", w)), output_gate=direct,
            position=RopePairsSpec(theta=float(_get(m, "rot.base", w)), rotary_dim=dims))
        for k in ("num_heads", "v_head_dim", "kv_rank"):
            if getattr(spec, k) <= 0:
                raise ConfigError(f"{w}{k} must be positive")
        if spec.head_dim < 0 or spec.head_dim + spec.rot_dim <= 0:
            raise ConfigError(f"{w}dim and rot_dim leave no query")
        return spec

    def _ffn(self, layer: Dict[str, Any], where: str):
        mlp = layer.get("mlp")
        if mlp is None:
            return None
        w = where + "mlp."
        kind = _get(mlp, "kind", w)
        if kind == "dense":
            return PolyNormMLPSpec(intermediate_size=int(_get(mlp, "ff", w)), eps=self.eps)
        if kind == "moe":
            r = _get(mlp, "router", w)
            groups = r.get("groups") or {}
            spec = GroupedMoESpec(
                num_experts=int(_get(r, "experts", w + "router.")), top=int(_get(r, "top", w + "router.")),
                num_groups=int(groups.get("count", 1)), keep_groups=int(groups.get("keep", groups.get("count", 1))),
                intermediate_size=int(_get(mlp, "expert.ff", w)), limit=float(_get(mlp, "expert.limit", w)))
            if spec.num_experts % spec.num_groups or not 1 <= spec.keep_groups <= spec.num_groups or \
                    not 1 <= spec.top <= spec.keep_groups * (spec.num_experts // spec.num_groups):
                raise ConfigError(f"{w}router: top {spec.top} of {spec.keep_groups} of {spec.num_groups} groups "
                                  f"over {spec.num_experts} experts cannot be chosen")
            return spec
        raise ConfigError(f"{w}kind is {kind!r}; known: dense, moe")

    # ---- the model this configuration describes --------------------------------------------------------------
    def to_model_spec(self) -> ModelSpec:
        norm = ScalarRMSNormSpec(eps=self.eps)
        conv = ShortConvSpec(taps=self.taps) if self.taps > 0 else None
        own: Dict[int, int] = {}          # layer of config.json with weights of its own -> index into the spec's layers
        layers: List[PostNormLayerSpec] = []
        schedule: List[ScheduleEntry] = []
        for i, layer in enumerate(self.layers):
            src = layer.get("weights_of")
            if src is None:
                where = f"layers[{i}]."
                ffn = self._ffn(layer, where)
                own[i] = len(layers)
                layers.append(PostNormLayerSpec(
                    prefix=f"l{i}", mixer=self._mixer(layer, where), mixer_norm=norm, ffn=ffn,
                    ffn_norm=norm if ffn is not None else None, alpha=self.alpha, conv=conv))
        for i, layer in enumerate(self.layers):
            src = layer.get("weights_of")
            schedule.append(ScheduleEntry(layer=own[i if src is None else src]))
        spec = ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab, hidden_size=self.width,
            layers=tuple(layers), schedule=tuple(schedule), final_norm=norm,
            embed_name="embed", final_norm_name="final.norm", head_name="head", tie_head=False,
            max_positions=self.max_positions)
        spec.validate()
        return spec

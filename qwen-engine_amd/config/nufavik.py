"""Typed configuration of the Nufavik decoder, read from config.json.

A decoder of parallel blocks: one RMS norm a layer, whose output both the mixer and the feed-forward read,
and one residual sum of the two.  The mixer is grouped-query attention with biased projections, a short
causal convolution over time on every channel of q, k and v, a half-split rotation of the first numbers
of every q and k head, a sliding window that also keeps a request's first keys, and a softmax with a 1
added to its denominator.  The feed-forward is a routed mixture of squared-relu experts with a correction
added to the scores for the choice only, renormalised and scaled weights, and identity experts.  The
embedding is scaled; the head is the embedding table itself.

Keys: architecture, vocab, width, embedding.scale, norm.eps, layers[i].type (attention),
layers[i].mixer {heads, kv_heads, dim, vdim, conv, scale, rot {base, dims}, mask {size, keep_first}},
layers[i].mlp (null | {kind: moe, expert {ff}, router {experts, identity, top, scale}}).  No size has a default.
"""
from __future__ import annotations

import copy
from typing import Any, Dict, List

from .qwen3 import ConfigError
from .spec import (BareRMSNormSpec, BiasedMoESpec, ConvAttentionSpec, ModelSpec, ParallelLayerSpec,
                   RopeHalfAnglesSpec, ScheduleEntry, StreamScaleSpec)

ARCHITECTURE = "Nufavik"
MAX_POSITIONS = 1 << 20      # the design names no limit; positions stay exact in 32-bit floats far beyond this


def _get(d: Dict[str, Any], path: str, where: str):
    cur: Any = d
    for key in path.split("."):
        if not isinstance(cur, dict) or key not in cur:
            raise ConfigError(f"config.json lacks {where}{path}")
        cur = cur[key]
    return cur


class NufavikConfig:
    architecture = ARCHITECTURE

    def __init__(self, d: Dict[str, Any]):
        self.raw = copy.deepcopy(d)
        self.vocab = int(_get(d, "vocab", ""))
        self.width = int(_get(d, "width", ""))
        self.embedding_scale = float(_get(d, "embedding.scale", ""))
        self.eps = float(_get(d, "norm.eps", ""))
        self.layers: List[Dict[str, Any]] = list(_get(d, "layers", ""))
        self.max_positions = int(d.get("max_positions", MAX_POSITIONS))
        self.validate()

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "NufavikConfig":
        return cls(d)

    def to_dict(self) -> Dict[str, Any]:
        return copy.deepcopy(self.raw)

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("vocab and width must be positive")
        if not self.eps > 0:
            raise ConfigError("norm.eps must be positive")
        if not self.layers:
            raise ConfigError("the model has no layers")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]."
            if layer.get("type") != "attention":
                raise ConfigError(f"{where}type is {layer.get('type')!r}; known: attention")
            self._mixer(layer, where)
            self._ffn(layer, where)

    # ---- one layer's parts ---------------------------------------------------------------------------------
    def _mixer(self, layer: Dict[str, Any], where: str) -> ConvAttentionSpec:
        m = _get(layer, "mixer", where)
        w = where + "mixer."
        dim = int(_get(m, "dim", w))
        dims = int(_get(m, "rot.dims", w))
        if dims % 2 or not 0 <= dims <= dim:
            raise ConfigError(f"{w}rot.dims = {dims} must be even and at most dim = {dim}")
        size, keep = int(_get(m, "mask.size", w)), int(_get(m, "mask.keep_first", w))
        if size <= 0 or keep < 0:
            raise ConfigError(f"{w}mask: a window of {size} keys that keeps the first {keep}")
        spec = ConvAttentionSpec(
            num_heads=int(_get(m, "heads", w)), num_kv_heads=int(_get(m, "kv_heads", w)), head_dim=dim,
            v_head_dim=int(_get(m, "vdim", w)), scale=float(_get(m, "scale", w)), conv_taps=int(_get(m, "conv", w)),
            qkv_bias=True, window=size, keep_first=keep, sink=True,
            position=RopeHalfAnglesSpec(theta=float(_get(m, "rot.base", w)), rotary_dim=dims) if dims else None)
        if spec.num_heads <= 0 or spec.num_kv_heads <= 0 or spec.num_heads % spec.num_kv_heads:
            raise ConfigError(f"{w}{spec.num_heads} heads over {spec.num_kv_heads} key/value heads")
        if spec.head_dim <= 0 or spec.v_head_dim <= 0 or spec.conv_taps < 1:
            raise ConfigError(f"{w}dim, vdim and conv must be positive")
        return spec

    def _ffn(self, layer: Dict[str, Any], where: str):
        mlp = layer.get("mlp")
        if mlp is None:
            return None
        w = where + "mlp."
        kind = _get(mlp, "kind", w)
        if kind != "moe":
            raise ConfigError(f"{w}kind is {kind!r}; known: moe")
        r = _get(mlp, "router", w)
        spec = BiasedMoESpec(
            num_experts=int(_get(r, "experts", w + "router.")), num_identity=int(_get(r, "identity", w + "router.")),
            top=int(_get(r, "top", w + "router.")), intermediate_size=int(_get(mlp, "expert.ff", w)),
            route_scale=float(_get(r, "scale", w + "router.")))
        if spec.num_experts < 1 or spec.num_identity < 0 or spec.intermediate_size < 1 or \
                not 1 <= spec.top <= spec.num_experts + spec.num_identity:
            raise ConfigError(f"{w}router: top {spec.top} of {spec.num_experts} experts and {spec.num_identity} "
                              f"identity experts cannot be chosen")
        return spec

    # ---- the model this configuration describes --------------------------------------------------------------
    def to_model_spec(self) -> ModelSpec:
        norm = BareRMSNormSpec(eps=self.eps)
        layers = []
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]."
            layers.append(ParallelLayerSpec(prefix=f"l{i}", norm=norm, mixer=self._mixer(layer, where),
                                            ffn=self._ffn(layer, where)))
        spec = ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab, hidden_size=self.width,
            layers=tuple(layers), schedule=tuple(ScheduleEntry(layer=i) for i in range(len(layers))),
            final_norm=norm, embed_name="embed", final_norm_name="final.norm", head_name="embed", tie_head=True,
            max_positions=self.max_positions,
            stream_prologue=StreamScaleSpec(scale=self.embedding_scale) if self.embedding_scale != 1.0 else None)
        spec.validate()
        return spec

"""Typed configuration of Telapel, read from its config.json keys.

Telapel is a decoder whose sublayers read the residual stream itself and whose norm (RMS, plain weight) stands on a
sublayer's OUTPUT: x += N1(mixer(x)), then x += N2(ff(x)). ``layers`` lists the layers, each with its ``type``:
``rglru`` (a recurrent block around a gated linear recurrence per channel, see ``parts/rglru.py``: ``width``, ``blocks``,
``conv`` taps), ``latent_attention`` (softmax attention over a cached latent with a rotated key part that all heads
share, see ``parts/latent.py``: ``heads``, ``dim``, ``rot_dim``, ``vdim``, ``q_rank``, ``kv_rank``, ``scale``, ``rot.base`` /
``rot.dims``) or ``attention`` (grouped heads whose values are their keys, short convolutions and biases on q and k, a
per-head norm, a query factor that grows with the position ``q_temp.coef`` / ``q_temp.every``, capped scores ``softcap``,
a bias by distance, a sliding window ``mask.size`` and a softmax with one more term of 1 in its denominator, see
``parts/attention.py``). ``mlp`` is ``null`` or ``{"kind": "moe", "router": {"experts", "top", "groups": {"count", "keep"}},
"expert": {"ff", "limit"}, "shared": {"ff", "limit"}}``: a mixture of clamped gated units chosen among the best groups of
experts, with one unit that every token runs. An entry with ``weights_of: j`` brings no weights: the layer is run with those
that layer j loaded, while its pages or its slot are kept apart from layer j's. The head is the embedding table behind the
final norm. A checkpoint names its tensors ``l<i>.<part>`` without a ".weight" suffix.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional, Tuple

from .spec import ConfigError, LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from .vavelorn import _get, _groups, _int, _number, _or, _scale

LAYER_TYPES = ("rglru", "latent_attention", "attention")
DISTANCE_SLOPE_EXPONENT = 8.0       # a head's slope of the bias by distance is 2^(-8 (h + 1) / heads)
DECAY_RATE = 8.0                    # log a = -8 r softplus(lam) in the recurrence
GLU_ALPHA, GLU_SHIFT = 1.702, 1.0   # a unit is g sigmoid(1.702 g) (u + 1)
NO_POSITION_LIMIT = 1 << 30


@dataclass(frozen=True)
class RecurrentSizes:
    width: int
    blocks: int
    conv: int

    kind = "rglru"

    @classmethod
    def from_dict(cls, data, where) -> "RecurrentSizes":
        sizes = cls(width=_int(data, "width", where), blocks=_or(data, "blocks", where, 1), conv=_or(data, "conv", where, 1))
        if sizes.width % sizes.blocks:
            raise ConfigError(f"config.json: {where}: {sizes.width} channels are not {sizes.blocks} equal blocks")
        return sizes

    def to_dict(self) -> Dict[str, Any]:
        return {"blocks": self.blocks, "conv": self.conv, "width": self.width}


@dataclass(frozen=True)
class LatentSizes:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_dims: int
    rot_base: float

    kind = "latent_attention"

    @classmethod
    def from_dict(cls, data, where) -> "LatentSizes":
        rot = data.get("rot") if isinstance(data, Mapping) else None
        dim, rot_dim = _int(data, "dim", where), _or(data, "rot_dim", where, 0, least=0)
        sizes = cls(heads=_int(data, "heads", where), dim=dim, rot_dim=rot_dim, vdim=_or(data, "vdim", where, dim),
                    q_rank=_int(data, "q_rank", where), kv_rank=_int(data, "kv_rank", where), scale=_scale(data, where, dim + rot_dim),
                    rot_dims=_or(rot, "dims", where + ".rot", rot_dim, least=0) if rot is not None else 0,
                    rot_base=_number(rot, "base", where + ".rot", positive=True) if rot is not None else 1.0)
        if sizes.rot_dim % 2 or sizes.rot_dims % 2 or sizes.rot_dims > sizes.rot_dim:
            raise ConfigError(f"config.json: {where}: rot_dim {sizes.rot_dim} and rot.dims {sizes.rot_dims} must be even, rot.dims at most rot_dim")
        return sizes

    def to_dict(self) -> Dict[str, Any]:
        return {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "q_rank": self.q_rank,
                "rot": {"base": self.rot_base, "dims": self.rot_dims}, "rot_dim": self.rot_dim, "scale": self.scale, "vdim": self.vdim}


@dataclass(frozen=True)
class KeyValueAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    scale: float
    conv: int                           # taps of the convolutions on q and k (0: none)
    window: Optional[int]               # None: every earlier key
    softcap: float                      # 0: none
    temp_coef: float
    temp_every: Optional[int]           # None: no factor on the queries

    kind = "attention"

    @classmethod
    def from_dict(cls, data, where) -> "KeyValueAttentionSizes":
        mask, temp = data.get("mask"), data.get("q_temp")
        heads, dim = _int(data, "heads", where), _int(data, "dim", where)
        sizes = cls(heads=heads, kv_heads=_or(data, "kv_heads", where, heads), dim=dim, scale=_scale(data, where, dim),
                    conv=_or(data, "conv", where, 0),
                    window=_int(mask, "size", where + ".mask") if mask is not None else None,
                    softcap=_number(data, "softcap", where, positive=True) if data.get("softcap") is not None else 0.0,
                    temp_coef=_number(temp, "coef", where + ".q_temp") if temp is not None else 0.0,
                    temp_every=_int(temp, "every", where + ".q_temp") if temp is not None else None)
        _groups(sizes.heads, sizes.kv_heads, where)
        if _or(data, "vdim", where, dim) != dim:
            raise ConfigError(f"config.json: {where}.vdim: the values are the keys and have their size, {dim}")
        return sizes

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale, "vdim": self.dim}
        if self.conv:
            out["conv"] = self.conv
        if self.window is not None:
            out["mask"] = {"size": self.window}
        if self.temp_every is not None:
            out["q_temp"] = {"coef": self.temp_coef, "every": self.temp_every}
        if self.softcap:
            out["softcap"] = self.softcap
        return out


@dataclass(frozen=True)
class MixtureSizes:
    experts: int
    top: int
    groups: int
    keep: int
    ff: int
    limit: float
    shared_ff: Optional[int] = None
    shared_limit: Optional[float] = None

    @classmethod
    def from_dict(cls, data, where) -> "MixtureSizes":
        kind = _get(data, "kind", where)
        if kind != "moe":
            raise ConfigError(f"config.json: {where}.kind is {kind!r}; known: moe")
        router, expert, shared = _get(data, "router", where), _get(data, "expert", where), data.get("shared")
        groups = router.get("groups") if isinstance(router, Mapping) else None
        count = _int(groups, "count", where + ".router.groups") if groups is not None else 1
        sizes = cls(experts=_int(router, "experts", where + ".router"), top=_int(router, "top", where + ".router"), groups=count,
                    keep=_or(groups, "keep", where + ".router.groups", count) if groups is not None else 1,
                    ff=_int(expert, "ff", where + ".expert"), limit=_number(expert, "limit", where + ".expert", positive=True),
                    shared_ff=_int(shared, "ff", where + ".shared") if shared is not None else None,
                    shared_limit=_number(shared, "limit", where + ".shared", positive=True) if shared is not None else None)
        if sizes.experts % sizes.groups or sizes.keep > sizes.groups or sizes.top > sizes.keep * (sizes.experts // sizes.groups):
            raise ConfigError(f"config.json: {where}.router: {sizes.top} of {sizes.experts} experts from {sizes.keep} of {sizes.groups} equal groups")
        return sizes

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"expert": {"ff": self.ff, "limit": self.limit}, "kind": "moe",
                               "router": {"experts": self.experts, "groups": {"count": self.groups, "keep": self.keep}, "top": self.top}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return out


_MIXERS = {cls.kind: cls for cls in (RecurrentSizes, LatentSizes, KeyValueAttentionSizes)}


@dataclass(frozen=True)
class TelapelLayer:
    mixer: Any                          # one of the three sizes classes; its ``kind`` is the layer's type
    mlp: Optional[MixtureSizes]         # None: the layer has no feed-forward
    weights_of: Optional[int] = None    # the layer whose tensors this one runs (None: its own)


@dataclass(frozen=True)
class TelapelConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[TelapelLayer, ...]

    architecture = "Telapel"

    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "TelapelConfig":
        if not isinstance(data, Mapping):
            raise ConfigError("config.json must hold a JSON object")
        listed = _get(data, "layers", "the model")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: 'layers' must be a list of at least one layer")
        layers: List[TelapelLayer] = []
        for index, entry in enumerate(listed):
            where = f"layers[{index}]"
            kind = _get(entry, "type", where)
            if kind not in _MIXERS:
                raise ConfigError(f"config.json: {where}.type is {kind!r}; known: {', '.join(LAYER_TYPES)}")
            mlp = entry.get("mlp")
            layers.append(TelapelLayer(
                mixer=_MIXERS[kind].from_dict(_get(entry, "mixer", where), where + ".mixer"),
                mlp=MixtureSizes.from_dict(mlp, where + ".mlp") if mlp is not None else None,
                weights_of=_int(entry, "weights_of", where, least=0) if entry.get("weights_of") is not None else None))
        for index, layer in enumerate(layers):
            if layer.weights_of is None:
                continue
            where = f"layers[{index}].weights_of"
            if layer.weights_of >= len(layers) or layer.weights_of == index or layers[layer.weights_of].weights_of is not None:
                raise ConfigError(f"config.json: {where} = {layer.weights_of} must name another layer, one that loads weights itself")
            owner = layers[layer.weights_of]
            if (owner.mixer, owner.mlp) != (layer.mixer, layer.mlp):
                raise ConfigError(f"config.json: {where}: a layer that runs layer {layer.weights_of}'s weights has that layer's sizes")
        return cls(vocab=_int(data, "vocab", "the model"), width=_int(data, "width", "the model"),
                   norm_eps=_number(_get(data, "norm", "the model"), "eps", "norm", positive=True), layers=tuple(layers))

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for layer in self.layers:
            entry: Dict[str, Any] = {"mixer": layer.mixer.to_dict(), "mlp": None if layer.mlp is None else layer.mlp.to_dict(),
                                     "type": layer.mixer.kind}
            if layer.weights_of is not None:
                entry["weights_of"] = layer.weights_of
            layers.append(entry)
        return {"architecture": self.architecture, "layers": layers, "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as handle:
            json.dump(self.to_dict(), handle, indent=1)

    # sizes the engine's command line and scheduler ask any configuration for
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def max_position_embeddings(self) -> int:
        return NO_POSITION_LIMIT

    def _mixer_spec(self, sizes, prefix: str) -> PartSpec:
        D = self.width
        if sizes.kind == "rglru":
            return PartSpec("rglru", {"hidden_size": D, "width": sizes.width, "blocks": sizes.blocks, "taps": sizes.conv,
                                      "decay_rate": DECAY_RATE}, prefix=prefix)
        if sizes.kind == "latent_attention":
            position = PartSpec("rotary_interleaved", {"theta": sizes.rot_base, "rotary_dim": sizes.rot_dims, "head_dim": max(sizes.rot_dim, 2)})
            return PartSpec("latent_attention", {
                "hidden_size": D, "num_heads": sizes.heads, "head_dim": sizes.dim, "v_head_dim": sizes.vdim, "q_rank": sizes.q_rank,
                "kv_rank": sizes.kv_rank, "norm_eps": self.norm_eps, "softmax_scale": sizes.scale, "output_gate": False,
                "rot_dim": sizes.rot_dim, "position": position}, prefix=prefix)
        return PartSpec("gqa_attention", {
            "hidden_size": D, "num_heads": sizes.heads, "num_kv_heads": sizes.kv_heads, "head_dim": sizes.dim,
            "softmax_scale": sizes.scale, "window": sizes.window, "score_softcap": sizes.softcap or None,
            "qk_norm": True, "qk_norm_eps": self.norm_eps, "values": "keys", "qk_conv": sizes.conv, "qk_bias": True, "sink": "unit",
            "distance_slope_exponent": DISTANCE_SLOPE_EXPONENT,
            "query_temperature": None if sizes.temp_every is None else (sizes.temp_coef, sizes.temp_every),
            "position": PartSpec("none", {}),
            "names": {"q": "q", "k": "k", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "q_bias": "q.b", "k_bias": "k.b",
                      "q_conv": "q.conv", "k_conv": "k.conv"}, "weight_suffix": "",
        }, prefix=prefix)

    def _ffn_spec(self, mlp: MixtureSizes, prefix: str) -> PartSpec:
        return PartSpec("moe_glu", {
            "hidden_size": self.width, "num_experts": mlp.experts, "top": mlp.top, "intermediate_size": mlp.ff,
            "shared_intermediate_size": mlp.shared_ff, "router_bias": False, "router_scores": "softmax_all",
            "router_groups": (mlp.groups, mlp.keep), "unit": "clamped", "limit": mlp.limit, "alpha": GLU_ALPHA, "shift": GLU_SHIFT,
            "shared_limit": mlp.shared_limit}, prefix=prefix)

    def model_spec(self) -> ModelSpec:
        D = self.width

        def norm(tensor: str) -> PartSpec:
            return PartSpec("rmsnorm", {"eps": self.norm_eps, "size": D, "tensor": tensor})

        # A layer that runs another's weights adds no layer of its own: the schedule names the owner's layer
        # with a cache entry (pages or state) of the borrower's own.
        layers: List[LayerSpec] = []
        spec_of: Dict[int, int] = {}
        for index, layer in enumerate(self.layers):
            if layer.weights_of is not None:
                continue
            base = f"l{index}."
            spec_of[index] = len(layers)
            layers.append(LayerSpec(
                arrangement="output_norm_residual", mixer_norm=norm(base + "norm1"), mixer=self._mixer_spec(layer.mixer, base + "mix."),
                ffn_norm=None if layer.mlp is None else norm(base + "norm2"),
                ffn=None if layer.mlp is None else self._ffn_spec(layer.mlp, base + "mlp."), params={"residual_mult": 1.0}))
        schedule = [ScheduleEntry(layer=spec_of[index if layer.weights_of is None else layer.weights_of], cache=index)
                    for index, layer in enumerate(self.layers)]
        spec = ModelSpec(
            architecture=self.architecture, hidden_size=D, vocab_size=self.vocab, max_positions=NO_POSITION_LIMIT,
            layers=tuple(layers), schedule=tuple(schedule), final_norm=norm("final.norm"), embedding_name="embed", lm_head_name=None)
        spec.validate()
        return spec

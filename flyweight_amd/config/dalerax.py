"""Typed configuration of Dalerax, read from its config.json keys.

Dalerax is a decoder of parallel layers: with h = N(x) (an RMS norm whose weight is stored around zero), a
layer adds mixer(h) + ff(h) to the residual stream; there is one norm a layer and both sublayers read it. The
embedding rows are scaled (``embedding.scale``) and a learned vector per position is added (table ``pos`` of
``max_positions`` rows); the logits are scaled (``logit_scale``). ``layers`` lists the layers, each with its
``type``: ``wkv`` (a linear recurrence over a matrix state per head with a decay that the token forms, see
``parts/wkv.py``) or ``attention`` (grouped-query softmax attention with rotary positions on the first
``rot.dims`` channels of a head in the half-split layout, optionally stretched by wavelength (``rot.scaling``:
factor, low, high, original), a sliding window ``mask.size`` that also keeps the first ``mask.keep_first`` keys,
and a learned sink per head in the softmax's denominator; with ``kv_from: j`` the layer has no key and value
projections and reads the cache of layer j). ``mlp`` is ``null``, ``{"kind": "dense", "ff"}`` or ``{"kind":
"moe", "router": {"experts", "top"}, "expert": {"ff"}, "shared": {"ff"}}``. A checkpoint names its tensors
``l<i>.<part>`` without a ".weight" suffix. The one size that stands in no key, the inner width of the decay's
low-rank map, comes from the checkpoint's tensor shapes (``from_model_dir``) or from ``decay_rank``.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional, Tuple

from .spec import ConfigError, LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from .vavelorn import _get, _groups, _int, _number, _or, _scale

LAYER_TYPES = ("wkv", "attention")
FF_KINDS = ("dense", "moe")
DEFAULT_DECAY_RANK = 32


@dataclass(frozen=True)
class WkvSizes:
    heads: int
    dim: int
    decay_rank: Optional[int] = None        # None: not known yet (the checkpoint says)

    kind = "wkv"

    @classmethod
    def from_dict(cls, data, where) -> "WkvSizes":
        return cls(heads=_int(data, "heads", where), dim=_int(data, "dim", where),
                   decay_rank=_int(data, "decay_rank", where) if data.get("decay_rank") is not None else None)

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"dim": self.dim, "heads": self.heads}
        if self.decay_rank is not None:
            out["decay_rank"] = self.decay_rank
        return out


@dataclass(frozen=True)
class SinkAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]               # None: every earlier key
    keep_first: int
    rot_dims: int
    rot_base: float
    rot_scaling: Optional[Tuple[float, float, float, float]]    # factor, low, high, original
    kv_from: Optional[int]

    kind = "attention"

    @classmethod
    def from_dict(cls, data, where) -> "SinkAttentionSizes":
        rot, mask = data.get("rot"), data.get("mask")
        heads, dim = _int(data, "heads", where), _int(data, "dim", where)
        scaling = rot.get("scaling") if rot is not None else None
        sizes = cls(
            heads=heads, kv_heads=_or(data, "kv_heads", where, heads), dim=dim, vdim=_or(data, "vdim", where, dim),
            scale=_scale(data, where, dim),
            window=_int(mask, "size", where + ".mask") if mask is not None else None,
            keep_first=_or(mask, "keep_first", where + ".mask", 0, least=0) if mask is not None else 0,
            rot_dims=_int(rot, "dims", where + ".rot", least=0) if rot is not None else 0,
            rot_base=_number(rot, "base", where + ".rot", positive=True) if rot is not None else 1.0,
            rot_scaling=None if scaling is None else tuple(_number(scaling, key, where + ".rot.scaling", positive=key != "low")
                                                           for key in ("factor", "low", "high", "original")),
            kv_from=_int(data, "kv_from", where, least=0) if data.get("kv_from") is not None else None)
        _groups(sizes.heads, sizes.kv_heads, where)
        if sizes.rot_dims % 2 or sizes.rot_dims > sizes.dim:
            raise ConfigError(f"config.json: {where}.rot.dims {sizes.rot_dims} must be even and at most dim {sizes.dim}")
        if sizes.rot_scaling is not None and not sizes.rot_scaling[2] > sizes.rot_scaling[1]:
            raise ConfigError(f"config.json: {where}.rot.scaling needs high > low")
        return sizes

    def to_dict(self) -> Dict[str, Any]:
        rot: Dict[str, Any] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.rot_scaling is not None:
            rot["scaling"] = dict(zip(("factor", "low", "high", "original"), self.rot_scaling))
        out: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "rot": rot, "scale": self.scale,
                               "vdim": self.vdim}
        if self.window is not None:
            out["mask"] = {"keep_first": self.keep_first, "size": self.window}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass(frozen=True)
class FeedForwardSizes:
    kind: str                           # "dense" or "moe"
    ff: int                             # of the dense unit, or of one expert
    experts: int = 0
    top: int = 0
    shared_ff: Optional[int] = None

    @classmethod
    def from_dict(cls, data, where) -> "FeedForwardSizes":
        kind = _get(data, "kind", where)
        if kind not in FF_KINDS:
            raise ConfigError(f"config.json: {where}.kind is {kind!r}; known: {', '.join(FF_KINDS)}")
        if kind == "dense":
            return cls(kind=kind, ff=_int(data, "ff", where))
        router, shared = _get(data, "router", where), data.get("shared")
        sizes = cls(kind=kind, ff=_int(_get(data, "expert", where), "ff", where + ".expert"),
                    experts=_int(router, "experts", where + ".router"), top=_int(router, "top", where + ".router"),
                    shared_ff=_int(shared, "ff", where + ".shared") if shared is not None else None)
        if sizes.top > sizes.experts:
            raise ConfigError(f"config.json: {where}.router chooses {sizes.top} of {sizes.experts} experts")
        return sizes

    def to_dict(self) -> Dict[str, Any]:
        if self.kind == "dense":
            return {"ff": self.ff, "kind": "dense"}
        out: Dict[str, Any] = {"expert": {"ff": self.ff}, "kind": "moe", "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


_MIXERS = {cls.kind: cls for cls in (WkvSizes, SinkAttentionSizes)}


@dataclass(frozen=True)
class DaleraxLayer:
    mixer: Any                          # WkvSizes or SinkAttentionSizes; its ``kind`` is the layer's type
    mlp: Optional[FeedForwardSizes]     # None: the layer has no feed-forward


@dataclass(frozen=True)
class DaleraxConfig:
    vocab: int
    width: int
    max_positions: int
    norm_eps: float
    embedding_scale: float
    logit_scale: float
    layers: Tuple[DaleraxLayer, ...]

    architecture = "Dalerax"

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], decay_ranks: Optional[Mapping[int, int]] = None) -> "DaleraxConfig":
        """``decay_ranks``: layer -> inner width of its decay map, where the checkpoint has been looked at."""
        if not isinstance(data, Mapping):
            raise ConfigError("config.json must hold a JSON object")
        listed = _get(data, "layers", "the model")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: 'layers' must be a list of at least one layer")
        layers: List[DaleraxLayer] = []
        for index, entry in enumerate(listed):
            where = f"layers[{index}]"
            kind = _get(entry, "type", where)
            if kind not in _MIXERS:
                raise ConfigError(f"config.json: {where}.type is {kind!r}; known: {', '.join(LAYER_TYPES)}")
            mixer = _MIXERS[kind].from_dict(_get(entry, "mixer", where), where + ".mixer")
            if kind == "wkv" and decay_ranks is not None and index in decay_ranks:
                mixer = WkvSizes(mixer.heads, mixer.dim, int(decay_ranks[index]))
            mlp = entry.get("mlp")
            layers.append(DaleraxLayer(mixer=mixer, mlp=FeedForwardSizes.from_dict(mlp, where + ".mlp") if mlp is not None else None))
        for index, layer in enumerate(layers):
            source = getattr(layer.mixer, "kv_from", None)
            if source is None:
                continue
            where = f"layers[{index}].mixer.kv_from"
            if source >= index or layers[source].mixer.kind != "attention" or layers[source].mixer.kv_from is not None:
                raise ConfigError(f"config.json: {where} = {source} must name an earlier attention layer with keys and values of its own")
            theirs, mine = layers[source].mixer, layer.mixer
            if (theirs.kv_heads, theirs.dim, theirs.vdim) != (mine.kv_heads, mine.dim, mine.vdim):
                raise ConfigError(f"config.json: {where}: layer {source} keeps {theirs.kv_heads} kv heads of {theirs.dim} / {theirs.vdim} "
                                  f"channels, this layer reads {mine.kv_heads} of {mine.dim} / {mine.vdim}")
        embedding = data.get("embedding") or {}
        return cls(vocab=_int(data, "vocab", "the model"), width=_int(data, "width", "the model"),
                   max_positions=_int(data, "max_positions", "the model"),
                   norm_eps=_number(_get(data, "norm", "the model"), "eps", "norm", positive=True),
                   embedding_scale=_number(embedding, "scale", "embedding") if embedding.get("scale") is not None else 1.0,
                   logit_scale=_number(data, "logit_scale", "the model") if data.get("logit_scale") is not None else 1.0,
                   layers=tuple(layers))

    @classmethod
    def from_model_dir(cls, model_dir: str, data: Mapping[str, Any]) -> "DaleraxConfig":
        """The inner widths of the decay maps stand in no key: the shape of ``l<i>.mix.w1`` gives them."""
        from ..weights.safetensors_io import SafetensorsFile, checkpoint_files
        ranks: Dict[int, int] = {}
        listed = data.get("layers") if isinstance(data, Mapping) else None
        wanted = {f"l{index}.mix.w1": index for index, entry in enumerate(listed or [])
                  if isinstance(entry, Mapping) and entry.get("type") == "wkv"}
        if wanted:
            for path in checkpoint_files(model_dir):
                handle = SafetensorsFile(path)
                try:
                    for name, index in wanted.items():
                        if name in handle.entries and len(handle.entries[name].shape) == 2:
                            ranks[index] = int(handle.entries[name].shape[0])
                finally:
                    handle.close()
        return cls.from_dict(data, decay_ranks=ranks)

    def to_dict(self) -> Dict[str, Any]:
        layers = [{"mixer": layer.mixer.to_dict(), "mlp": None if layer.mlp is None else layer.mlp.to_dict(), "type": layer.mixer.kind}
                  for layer in self.layers]
        return {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale}, "layers": layers,
                "logit_scale": self.logit_scale, "max_positions": self.max_positions, "norm": {"eps": self.norm_eps},
                "vocab": self.vocab, "width": self.width}

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
        return self.max_positions

    def _mixer_spec(self, sizes, prefix: str) -> PartSpec:
        D = self.width
        if sizes.kind == "wkv":
            return PartSpec("wkv", {"hidden_size": D, "num_heads": sizes.heads, "head_dim": sizes.dim,
                                    "decay_rank": sizes.decay_rank or DEFAULT_DECAY_RANK, "norm_eps": self.norm_eps}, prefix=prefix)
        position = {"theta": sizes.rot_base, "rotary_dim": sizes.rot_dims, "head_dim": sizes.dim}
        if sizes.rot_scaling is not None:
            position["wavelength_scaling"] = tuple(sizes.rot_scaling)
        return PartSpec("gqa_attention", {
            "hidden_size": D, "num_heads": sizes.heads, "num_kv_heads": sizes.kv_heads, "head_dim": sizes.dim,
            "v_head_dim": sizes.vdim, "softmax_scale": sizes.scale, "window": sizes.window, "keep_first": sizes.keep_first,
            "sink": True, "shared_kv": sizes.kv_from is not None,
            "position": PartSpec("rotary_neox" if sizes.rot_dims else "none", position),
            "names": {"q": "q", "k": "k", "v": "v", "o": "o", "sink": "sink"}, "weight_suffix": "",
        }, prefix=prefix)

    def _ffn_spec(self, mlp: FeedForwardSizes, prefix: str) -> PartSpec:
        names = {"gate": "gate", "up": "up", "down": "down"}
        if mlp.kind == "dense":
            return PartSpec("swiglu", {"hidden_size": self.width, "intermediate_size": mlp.ff, "names": names, "weight_suffix": ""},
                            prefix=prefix)
        return PartSpec("moe_swiglu", {"hidden_size": self.width, "num_experts": mlp.experts, "top": mlp.top,
                                       "intermediate_size": mlp.ff, "shared_intermediate_size": mlp.shared_ff, "router_bias": True},
                        prefix=prefix)

    def model_spec(self) -> ModelSpec:
        D = self.width

        def norm(tensor: str) -> PartSpec:
            return PartSpec("rmsnorm", {"eps": self.norm_eps, "size": D, "tensor": tensor, "one_centered": True})

        layers: List[LayerSpec] = []
        schedule: List[ScheduleEntry] = []
        for index, layer in enumerate(self.layers):
            base = f"l{index}."
            layers.append(LayerSpec(
                arrangement="parallel_residual", mixer_norm=norm(base + "norm1"), mixer=self._mixer_spec(layer.mixer, base + "mix."),
                ffn_norm=None, ffn=None if layer.mlp is None else self._ffn_spec(layer.mlp, base + "mlp.")))
            source = getattr(layer.mixer, "kv_from", None)
            # a layer that reads another's keys and values names that layer's cache entry and does not write it
            schedule.append(ScheduleEntry(layer=index, cache=index if source is None else source, writes_cache=source is None))
        spec = ModelSpec(
            architecture=self.architecture, hidden_size=D, vocab_size=self.vocab, max_positions=self.max_positions,
            layers=tuple(layers), schedule=tuple(schedule), final_norm=norm("final.norm"), embedding_name="embed",
            lm_head_name="head", embedding_scale=self.embedding_scale, logit_scale=self.logit_scale, position_table_name="pos")
        spec.validate()
        return spec

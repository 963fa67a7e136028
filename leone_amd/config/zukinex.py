"""Zukinex configuration: a list of attention layers, each with a dense or a routed feed-forward, or none.

config.json keys: ``architecture`` ("Zukinex"), ``vocab``, ``width``, ``max_positions`` (rows of the learned position
table), ``norm.eps``, and ``layers``: a list of ``{"type": "attention", "mixer", "mlp"}``.

  ``mixer`` = {heads, kv_heads, dim, vdim, scale, rot: {dims, base}, mask: {size, keep_first}, kv_from}
              ``rot`` may be absent (no rotation); ``mask`` may be absent (every earlier key is seen);
              ``kv_from`` (absent or a layer's index): the layer has no keys and values of its own and reads that layer's.
  ``mlp``   = null, {kind: "dense", ff}, or
              {kind: "moe", expert: {ff}, router: {experts, top, identity, groups: {count, keep}}, shared: {ff} or absent}
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple, Union

from .base import ConfigError, FieldReader


def _sub(raw: Mapping[str, Any], key: str, where: str, optional: bool = False) -> Optional[FieldReader]:
    value = raw.get(key)
    if value is None and optional:
        return None
    if not isinstance(value, dict):
        raise ConfigError(f"{where}{key}", f"expected an object, found {value!r}")
    return FieldReader(value)


def _index(reader: FieldReader, key: str, where: str, default=None) -> Optional[int]:
    value = reader.optional(key)
    if value is None:
        return default
    if isinstance(value, bool) or not isinstance(value, int) or value < 0:
        raise ConfigError(f"{where}{key}", f"expected an integer that is not negative, found {value!r}")
    return value


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int                 # 0: no rotation
    rot_base: float
    window: Optional[int]         # None: every earlier key is seen
    keep_first: int               # with a window: keys at positions below this stay in sight
    kv_from: Optional[int]        # the layer whose keys and values this one reads; None: its own


@dataclass(frozen=True)
class DenseConfig:
    ff: int


@dataclass(frozen=True)
class MoeConfig:
    experts: int                  # experts with matrices
    identity: int                 # router outputs behind them that hand the input on
    top: int
    group_count: int
    group_keep: int
    expert_ff: int
    shared_ff: Optional[int]      # None: no shared expert


@dataclass(frozen=True)
class LayerConfig:
    mixer: AttentionConfig
    mlp: Union[DenseConfig, MoeConfig, None]


def _attention(raw: Mapping[str, Any], where: str, index: int) -> AttentionConfig:
    m = _sub(raw, "mixer", where)
    w = where + "mixer."
    try:
        heads, kv_heads = m.positive_int("heads"), m.positive_int("kv_heads")
        dim, vdim = m.positive_int("dim"), m.positive_int("vdim")
        scale = m.positive_float("scale")
    except ConfigError as error:
        raise ConfigError(w + error.field, str(error).split(": ", 2)[-1]) from None
    if heads % kv_heads:
        raise ConfigError(w + "kv_heads", f"{heads} query heads cannot be shared out over {kv_heads} key/value heads")
    rot_dims, rot_base = 0, 1.0
    rot = _sub(m.raw, "rot", w, optional=True)
    if rot is not None:
        try:
            rot_dims, rot_base = rot.positive_int("dims"), rot.positive_float("base")
        except ConfigError as error:
            raise ConfigError(w + "rot." + error.field, str(error).split(": ", 2)[-1]) from None
        if rot_dims % 2 or rot_dims > dim:
            raise ConfigError(w + "rot.dims", f"must be even and at most the head's {dim}, found {rot_dims}")
    window, keep_first = None, 0
    mask = _sub(m.raw, "mask", w, optional=True)
    if mask is not None:
        try:
            window = mask.positive_int("size")
        except ConfigError as error:
            raise ConfigError(w + "mask." + error.field, str(error).split(": ", 2)[-1]) from None
        keep_first = _index(mask, "keep_first", w + "mask.", 0)
    kv_from = _index(m, "kv_from", w)
    if kv_from is not None and kv_from >= index:
        raise ConfigError(w + "kv_from", f"layer {index} can only read the keys of an earlier layer, found {kv_from}")
    return AttentionConfig(heads, kv_heads, dim, vdim, scale, rot_dims, rot_base, window, keep_first, kv_from)


def _mlp(raw: Mapping[str, Any], where: str) -> Union[DenseConfig, MoeConfig, None]:
    if raw.get("mlp") is None:
        return None
    f = _sub(raw, "mlp", where)
    w = where + "mlp."
    kind = f.optional("kind")
    try:
        if kind == "dense":
            return DenseConfig(f.positive_int("ff"))
        if kind != "moe":
            raise ConfigError("kind", f"expected \"dense\" or \"moe\", found {kind!r}")
        expert, router = _sub(f.raw, "expert", w), _sub(f.raw, "router", w)
        expert_ff = expert.positive_int("ff")
        experts, top = router.positive_int("experts"), router.positive_int("top")
        identity = _index(router, "identity", w + "router.", 0)
        groups = _sub(router.raw, "groups", w + "router.", optional=True)
        count, keep = (groups.positive_int("count"), groups.positive_int("keep")) if groups is not None else (1, 1)
        shared = _sub(f.raw, "shared", w, optional=True)
        shared_ff = shared.positive_int("ff") if shared is not None else None
    except ConfigError as error:
        if error.field.startswith(where):
            raise
        raise ConfigError(w + error.field, str(error).split(": ", 2)[-1]) from None
    total = experts + identity
    if top > total:
        raise ConfigError(w + "router.top", f"{top} of {total} router outputs cannot be chosen")
    if total % count or keep > count:
        raise ConfigError(w + "router.groups", f"{total} router outputs in {count} equal groups of which {keep} stay open")
    if top > keep * (total // count):
        raise ConfigError(w + "router.groups", f"{keep} groups of {total // count} cannot give {top} choices")
    return MoeConfig(experts, identity, top, count, keep, expert_ff, shared_ff)


@dataclass(frozen=True)
class ZukinexConfig:
    vocab: int
    width: int
    max_positions: int
    eps: float
    layers: Tuple[LayerConfig, ...]
    architecture: str = "Zukinex"

    ARCHITECTURE = "Zukinex"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "ZukinexConfig":
        top = FieldReader(raw)
        vocab, width = top.positive_int("vocab"), top.positive_int("width")
        max_positions = top.positive_int("max_positions")
        eps = _sub(raw, "norm", "").positive_float("eps")
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("layers", f"expected a list of layers, found {listed!r}")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]."
            if not isinstance(entry, dict):
                raise ConfigError(f"layers[{i}]", f"expected an object, found {entry!r}")
            if entry.get("type") != "attention":
                raise ConfigError(where + "type", f"expected \"attention\", found {entry.get('type')!r}")
            layers.append(LayerConfig(_attention(entry, where, i), _mlp(entry, where)))
        for i, layer in enumerate(layers):
            source = layer.mixer.kv_from
            if source is None:
                continue
            other, mine = layers[source].mixer, layer.mixer
            if other.kv_from is not None:
                raise ConfigError(f"layers[{i}].mixer.kv_from", f"layer {source} has no keys of its own")
            if (other.kv_heads, other.dim, other.vdim, other.rot_dims, other.rot_base) != \
                    (mine.kv_heads, mine.dim, mine.vdim, mine.rot_dims, mine.rot_base):
                raise ConfigError(f"layers[{i}].mixer.kv_from", f"layer {source}'s key/value heads or rotation differ from this layer's")
        return cls(vocab, width, max_positions, eps, tuple(layers))

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for layer in self.layers:
            m = layer.mixer
            mixer: Dict[str, Any] = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale}
            if m.rot_dims:
                mixer["rot"] = {"dims": m.rot_dims, "base": m.rot_base}
            if m.window is not None:
                mixer["mask"] = {"size": m.window, "keep_first": m.keep_first}
            if m.kv_from is not None:
                mixer["kv_from"] = m.kv_from
            f = layer.mlp
            if f is None:
                mlp = None
            elif isinstance(f, DenseConfig):
                mlp = {"kind": "dense", "ff": f.ff}
            else:
                mlp = {"kind": "moe", "expert": {"ff": f.expert_ff},
                       "router": {"experts": f.experts, "top": f.top, "identity": f.identity,
                                  "groups": {"count": f.group_count, "keep": f.group_keep}}}
                if f.shared_ff is not None:
                    mlp["shared"] = {"ff": f.shared_ff}
            layers.append({"type": "attention", "mixer": mixer, "mlp": mlp})
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "max_positions": self.max_positions, "norm": {"eps": self.eps}, "layers": layers}

    # what the generic entry points ask a configuration for
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def max_position_embeddings(self) -> int:
        return self.max_positions

    eos_token_id = None

    def kv_retention(self, layer: int) -> Tuple[Optional[int], int]:
        """(window, keep_first) that the cache of ``layer`` must keep: the widest of its own mask and of the masks
        of the layers that read its keys and values (None: everything)."""
        masks = [self.layers[layer].mixer] + [l.mixer for l in self.layers if l.mixer.kv_from == layer]
        if any(m.window is None for m in masks):
            return None, 0
        return max(m.window for m in masks), max(m.keep_first for m in masks)

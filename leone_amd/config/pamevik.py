"""Pamevik configuration: a list of layers, each with one of three kinds of mixer and an optional feed-forward.

config.json keys: ``architecture`` ("Pamevik"), ``vocab``, ``width``, ``norm.eps``, ``canon.taps`` (taps of the
input convolutions), and ``layers``: a list of ``{"type", "mixer", "mlp"}``.  ``type`` names the mixer:

  ``mlstm``          ``mixer`` = {heads, dim, vdim, gate_cap}
  ``parallel``       ``mixer`` = {left: {heads, kv_heads, dim, vdim, scale, rot: {dims, base}},
                                  right: {heads, dim, vdim, decay: [one a head], rot: {dims, base}}}
  ``channel_delta``  ``mixer`` = {heads, kv_heads, dim, vdim, conv}

``mlp`` is null or {kind: "dense", ff}.  The ranks of the low-rank projections of ``channel_delta`` are not in
config.json; they are read from the tensors' shapes when the weights are bound (``low_rank``, filled by
``with_shapes``).  ``max_positions`` (optional) bounds the rotary tables and a request's length.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field, replace
from typing import Any, Dict, Mapping, Optional, Tuple

from .base import ConfigError, FieldReader

DEFAULT_MAX_POSITIONS = 32768


def _sub(raw: Mapping[str, Any], key: str, where: str) -> FieldReader:
    value = raw.get(key)
    if not isinstance(value, dict):
        raise ConfigError(f"{where}{key}", f"expected an object, found {value!r}")
    return FieldReader(value)


def _rotation(reader: FieldReader, where: str, dim: int) -> Tuple[int, float]:
    rot = _sub(reader.raw, "rot", where)
    dims, base = rot.positive_int("dims"), rot.positive_float("base")
    if dims % 2 or dims > dim:
        raise ConfigError(f"{where}rot.dims", f"must be even and at most the head's {dim}, found {dims}")
    return dims, base


@dataclass(frozen=True)
class MlstmConfig:
    heads: int
    dim: int
    vdim: int
    gate_cap: float


@dataclass(frozen=True)
class SoftmaxBranchConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int
    rot_base: float


@dataclass(frozen=True)
class RetentionBranchConfig:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot_dims: int
    rot_base: float


@dataclass(frozen=True)
class ParallelConfig:
    left: SoftmaxBranchConfig
    right: RetentionBranchConfig


@dataclass(frozen=True)
class ChannelDeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    a_rank: Optional[int] = None      # from the tensors' shapes
    g_rank: Optional[int] = None


@dataclass(frozen=True)
class PamevikLayer:
    type: str
    mixer: Any
    ff: Optional[int]                 # None: the layer has no feed-forward


def _mixer(kind: str, raw: Mapping[str, Any], where: str):
    r = FieldReader(raw)
    if kind == "mlstm":
        return MlstmConfig(r.positive_int("heads"), r.positive_int("dim"), r.positive_int("vdim"),
                           r.positive_float("gate_cap"))
    if kind == "channel_delta":
        heads, kv_heads = r.positive_int("heads"), r.positive_int("kv_heads")
        if heads % kv_heads:
            raise ConfigError(f"{where}kv_heads", f"{heads} heads cannot be grouped over {kv_heads} query/key heads")
        taps = r.positive_int("conv")
        if taps < 2:
            raise ConfigError(f"{where}conv", f"a convolution needs at least 2 taps, found {taps}")
        # the ranks are the tensors' affair; a folder written from a configuration notes them so that it reads back
        return ChannelDeltaConfig(heads, kv_heads, r.positive_int("dim"), r.positive_int("vdim"), taps,
                                  r.positive_int("a_rank", None), r.positive_int("g_rank", None))
    if kind == "parallel":
        left, right = _sub(raw, "left", where), _sub(raw, "right", where)
        heads, kv_heads, dim = left.positive_int("heads"), left.positive_int("kv_heads"), left.positive_int("dim")
        if heads % kv_heads:
            raise ConfigError(f"{where}left.kv_heads", f"{heads} query heads cannot be grouped over {kv_heads} key/value heads")
        if dim % 8:
            raise ConfigError(f"{where}left.dim", f"the key cache holds heads in runs of 8 elements: dim must be a "
                                                  f"multiple of 8, found {dim}")
        vdim = left.positive_int("vdim")
        if vdim % 2:
            raise ConfigError(f"{where}left.vdim", f"must be even, found {vdim}")
        soft = SoftmaxBranchConfig(heads, kv_heads, dim, vdim, left.positive_float("scale"),
                                   *_rotation(left, f"{where}left.", dim))
        r_heads, r_dim = right.positive_int("heads"), right.positive_int("dim")
        decay = right.raw.get("decay")
        if not isinstance(decay, list) or len(decay) != r_heads or not all(
                isinstance(d, (int, float)) and not isinstance(d, bool) and math.isfinite(d) and 0.0 <= d <= 1.0 for d in decay):
            raise ConfigError(f"{where}right.decay", f"expected {r_heads} numbers in [0, 1], found {decay!r}")
        ret = RetentionBranchConfig(r_heads, r_dim, right.positive_int("vdim"), tuple(float(d) for d in decay),
                                    *_rotation(right, f"{where}right.", r_dim))
        return ParallelConfig(soft, ret)
    raise ConfigError(f"{where[:-6]}type", f"unknown layer type {kind!r}; known: mlstm, parallel, channel_delta")


@dataclass(frozen=True)
class PamevikConfig:
    architecture: str
    vocab: int
    width: int
    eps: float
    taps: int
    layers: Tuple[PamevikLayer, ...]
    max_positions: int = DEFAULT_MAX_POSITIONS
    raw: Dict[str, Any] = field(default_factory=dict, compare=False, repr=False)

    ARCHITECTURE = "Pamevik"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "PamevikConfig":
        read = FieldReader(raw)
        eps = _sub(raw, "norm", "").positive_float("eps")
        taps = _sub(raw, "canon", "").positive_int("taps")
        if taps < 2:
            raise ConfigError("canon.taps", f"a convolution needs at least 2 taps, found {taps}")
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("layers", "expected a list of layers")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]."
            if not isinstance(entry, dict) or not isinstance(entry.get("type"), str) or not isinstance(entry.get("mixer"), dict):
                raise ConfigError(where[:-1], "expected {type, mixer, mlp}")
            mixer = _mixer(entry["type"], entry["mixer"], where + "mixer.")
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                m = _sub(entry, "mlp", where)
                kind = m.string("kind")
                if kind != "dense":
                    raise ConfigError(where + "mlp.kind", f"unknown feed-forward kind {kind!r}; known: dense")
                ff = m.positive_int("ff")
            layers.append(PamevikLayer(entry["type"], mixer, ff))
        return cls(architecture=cls.ARCHITECTURE, vocab=read.positive_int("vocab"), width=read.positive_int("width"),
                   eps=eps, taps=taps, layers=tuple(layers),
                   max_positions=read.positive_int("max_positions", DEFAULT_MAX_POSITIONS),
                   raw={k: v for k, v in raw.items() if k != "torch_dtype"})

    def with_shapes(self, shapes: Mapping[str, tuple]) -> "PamevikConfig":
        """The configuration with the sizes that only the tensors give: the ranks of the low-rank projections."""
        layers = []
        for i, layer in enumerate(self.layers):
            mixer = layer.mixer
            if isinstance(mixer, ChannelDeltaConfig):
                a1, g1 = shapes.get(f"l{i}.mix.a1"), shapes.get(f"l{i}.mix.g1")
                if a1 is not None and g1 is not None:
                    mixer = replace(mixer, a_rank=int(a1[0]), g_rank=int(g1[0]))
            layers.append(replace(layer, mixer=mixer))
        return replace(self, layers=tuple(layers))

    def with_ranks(self, a_rank: int, g_rank: int) -> "PamevikConfig":
        """The same for a model made from random weights: every ``channel_delta`` layer gets these ranks."""
        return replace(self, layers=tuple(
            replace(layer, mixer=replace(layer.mixer, a_rank=a_rank, g_rank=g_rank))
            if isinstance(layer.mixer, ChannelDeltaConfig) else layer for layer in self.layers))

    def to_dict(self) -> dict:
        """The config.json that reads back as this configuration."""
        def mixer(m):
            if isinstance(m, MlstmConfig):
                return {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "gate_cap": m.gate_cap}
            if isinstance(m, ChannelDeltaConfig):
                out = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "conv": m.conv}
                if m.a_rank is not None and m.g_rank is not None:
                    out.update(a_rank=m.a_rank, g_rank=m.g_rank)
                return out
            l, r = m.left, m.right
            return {"left": {"heads": l.heads, "kv_heads": l.kv_heads, "dim": l.dim, "vdim": l.vdim, "scale": l.scale,
                             "rot": {"dims": l.rot_dims, "base": l.rot_base}},
                    "right": {"heads": r.heads, "dim": r.dim, "vdim": r.vdim, "decay": list(r.decay),
                              "rot": {"dims": r.rot_dims, "base": r.rot_base}}}
        out = {"architecture": self.ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
               "canon": {"taps": self.taps},
               "layers": [{"type": layer.type, "mixer": mixer(layer.mixer),
                           "mlp": None if layer.ff is None else {"kind": "dense", "ff": layer.ff}} for layer in self.layers]}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        return out

    # what the generic entry points ask a configuration for
    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def max_position_embeddings(self) -> int:
        return self.max_positions

    eos_token_id = None

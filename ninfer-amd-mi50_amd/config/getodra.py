"""Typed configuration of Getodra, a decoder-only model whose layers are listed one by one.

config.json keys: `architecture` ("Getodra"), `vocab`, `width`, `max_positions` (rows of the
table of learned positions), `norm.eps`, `canon.taps` (taps of the short convolution in
front of every sublayer), and `layers`: a list of objects with `type` ('latent_attention'
or 'lightning'), `mixer` (the mixer's sizes and constants), `mlp` ({'kind': 'dense', 'ff': n}
or null) and optionally `weights_of`: the index of the layer whose tensors this layer runs
with (it has none of its own, and a cache and state of its own).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, KeyReader


@dataclass(frozen=True)
class RotaryScaling:
    factor: float
    original: float
    fast: float
    slow: float


@dataclass(frozen=True)
class LatentMixerConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot_dims: int          # how many of the rot_dim numbers turn
    rot_base: float
    rot_scaling: Optional[RotaryScaling]


@dataclass(frozen=True)
class LightningMixerConfig:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]


@dataclass(frozen=True)
class GetodraLayer:
    type: str                       # 'latent_attention' | 'lightning'
    mixer: Any                      # LatentMixerConfig | LightningMixerConfig
    ff: Optional[int]               # inner size of the dense feed-forward, None: no feed-forward
    weights_of: Optional[int]       # the layer whose tensors this one uses, None: its own


@dataclass(frozen=True)
class GetodraConfig:
    vocab: int
    width: int
    max_positions: int
    eps: float
    taps: int
    layers: Tuple[GetodraLayer, ...]
    architecture: str = "Getodra"

    def owner(self, layer: int) -> int:
        """The layer whose tensors layer `layer` runs with."""
        seen = set()
        while self.layers[layer].weights_of is not None:
            if layer in seen:
                raise ConfigError(f"config.json: 'weights_of' of layer {layer} goes in a circle")
            seen.add(layer)
            layer = self.layers[layer].weights_of
        return layer

    @staticmethod
    def from_dict(raw: Dict[str, Any]) -> "GetodraConfig":
        r = KeyReader(raw)
        vocab = r.need_int("vocab", 1)
        width = r.need_int("width", 1)
        max_positions = r.need_int("max_positions", 1)
        eps = _sub(r, "norm").need_float("eps")
        if not eps > 0:
            raise ConfigError(f"config.json: key 'norm.eps' must be > 0, got {eps}")
        taps = _sub(r, "canon").need_int("taps", 1)
        entries = r.opt_raw("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: key 'layers' must be a non-empty list")
        layers = tuple(_layer(e, i, len(entries)) for i, e in enumerate(entries))
        cfg = GetodraConfig(vocab, width, max_positions, eps, taps, layers)
        for i, layer in enumerate(layers):
            j = cfg.owner(i)
            if j != i and (layers[j].type != layer.type or layers[j].mixer != layer.mixer
                           or layers[j].ff != layer.ff):
                raise ConfigError(f"config.json: layers[{i}] uses the weights of layer {j} but "
                                  f"its entry differs from that layer's")
        return cfg


def _sub(r: KeyReader, key: str) -> KeyReader:
    v = r.opt_raw(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{r.where}: key '{key}' must be an object")
    return KeyReader(v, f"{r.where}: {key}")


def _layer(entry: Any, i: int, n: int) -> GetodraLayer:
    where = f"config.json: layers[{i}]"
    if not isinstance(entry, dict):
        raise ConfigError(f"{where} must be an object")
    r = KeyReader(entry, where)
    kind = r.opt_str("type", None)
    m = _sub(r, "mixer")
    if kind == "latent_attention":
        rot_dim = m.need_int("rot_dim", 0)
        rot_dims, base, scaling = 0, 10000.0, None
        if rot_dim:
            rot = _sub(m, "rot")
            rot_dims = rot.opt_int("dims", rot_dim, 0)
            base = rot.need_float("base")
            if rot_dims % 2 or rot_dims > rot_dim:
                raise ConfigError(f"{where}: 'rot.dims' must be even and at most 'rot_dim'")
            if rot.opt_raw("scaling") is not None:
                s = _sub(rot, "scaling")
                scaling = RotaryScaling(s.need_float("factor"), s.need_float("original"),
                                        s.need_float("fast"), s.need_float("slow"))
        mixer = LatentMixerConfig(m.need_int("heads", 1), m.need_int("dim", 1), rot_dim,
                                  m.need_int("vdim", 1), m.need_int("kv_rank", 1),
                                  m.need_float("scale"), rot_dims, base, scaling)
    elif kind == "lightning":
        heads = m.need_int("heads", 1)
        decay = m.opt_raw("decay")
        if not isinstance(decay, list) or len(decay) != heads or not all(
                isinstance(d, (int, float)) and not isinstance(d, bool) for d in decay):
            raise ConfigError(f"{where}: 'mixer.decay' must be a list of {heads} numbers")
        mixer = LightningMixerConfig(heads, m.need_int("dim", 1), m.need_int("vdim", 1),
                                     tuple(float(d) for d in decay))
    else:
        raise ConfigError(f"{where}: 'type' must be 'latent_attention' or 'lightning', got {kind!r}")
    ff = None
    mlp = r.opt_raw("mlp")
    if mlp is not None:
        f = _sub(r, "mlp")
        if f.opt_str("kind", "dense") != "dense":
            raise ConfigError(f"{where}: 'mlp.kind' must be 'dense'")
        ff = f.need_int("ff", 1)
    weights_of = r.opt_int("weights_of", None, 0)
    if weights_of is not None and (weights_of >= n or weights_of == i):
        raise ConfigError(f"{where}: 'weights_of' must name another layer")
    return GetodraLayer(kind, mixer, ff, weights_of)

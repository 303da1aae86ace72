"""Typed configuration of Sosepel, a decoder-only model of parallel sublayers.

config.json keys: `architecture` ("Sosepel"), `vocab`, `width`, `norm.eps`, `logit_softcap`,
`embedding` (`scale`, and optionally `bigram`: `buckets`, `mul_prev`, `mul_cur`), `layers`: a
list of objects with `type` ('attention'), `mixer` (the mixer's sizes and constants) and `mlp`
(null, {'kind': 'dense', 'ff'} or {'kind': 'moe', 'expert': {'ff'}, 'router': {'experts',
'top', 'groups': {'count', 'keep'}}, 'shared': {'ff'} or null}), and optionally `loop`
(`start`, `stop`, `times`): layers start .. stop - 1 run `times` times in a row.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple

from .base import ConfigError, KeyReader


@dataclass(frozen=True)
class PairTable:
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass(frozen=True)
class DiffMixerConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float          # 0: scores are not capped
    diff: float
    temp_coef: float        # 0: no query temperature
    temp_every: int


@dataclass(frozen=True)
class MlpConfig:
    kind: str               # 'dense' | 'moe'
    ff: int                 # inner size (of one routed expert for 'moe')
    experts: int = 0
    top: int = 0
    groups: int = 1
    groups_kept: int = 1
    shared_ff: int = 0      # 0: no shared expert


@dataclass(frozen=True)
class SosepelLayer:
    type: str
    mixer: DiffMixerConfig
    mlp: Optional[MlpConfig]


@dataclass(frozen=True)
class Loop:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class SosepelConfig:
    vocab: int
    width: int
    eps: float
    logit_softcap: float    # 0: none
    embedding_scale: float
    pairs: Optional[PairTable]
    layers: Tuple[SosepelLayer, ...]
    loop: Optional[Loop]
    architecture: str = "Sosepel"

    def runs(self) -> List[Tuple[int, bool]]:
        """(layer, whether a pass of the loop begins with this run) in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        lp = self.loop
        out = [(i, False) for i in range(lp.start)]
        for _ in range(lp.times):
            out += [(i, i == lp.start) for i in range(lp.start, lp.stop)]
        return out + [(i, False) for i in range(lp.stop, n)]

    @staticmethod
    def from_dict(raw: Dict[str, Any]) -> "SosepelConfig":
        r = KeyReader(raw)
        vocab = r.need_int("vocab", 1)
        width = r.need_int("width", 1)
        eps = _sub(r, "norm").need_float("eps")
        if not eps > 0:
            raise ConfigError(f"config.json: key 'norm.eps' must be > 0, got {eps}")
        cap = r.opt_float("logit_softcap", 0.0)
        if cap < 0:
            raise ConfigError("config.json: key 'logit_softcap' must not be negative")
        e = _sub(r, "embedding")
        pairs = None
        if e.opt_raw("bigram") is not None:
            b = _sub(e, "bigram")
            pairs = PairTable(b.need_int("buckets", 1), b.need_int("mul_prev", 0),
                              b.need_int("mul_cur", 0))
        entries = r.opt_raw("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: key 'layers' must be a non-empty list")
        layers = tuple(_layer(x, i) for i, x in enumerate(entries))
        loop = None
        if r.opt_raw("loop") is not None:
            lp = _sub(r, "loop")
            loop = Loop(lp.need_int("start", 0), lp.need_int("stop", 0), lp.need_int("times", 1))
            if not loop.start < loop.stop <= len(layers):
                raise ConfigError(f"config.json: 'loop' must hold 0 <= start < stop <= {len(layers)} "
                                  f"layers, got {loop.start} and {loop.stop}")
        return SosepelConfig(vocab, width, eps, cap, e.opt_float("scale", 1.0), pairs, layers, loop)


def _sub(r: KeyReader, key: str) -> KeyReader:
    v = r.opt_raw(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{r.where}: key '{key}' must be an object")
    return KeyReader(v, f"{r.where}: {key}")


def _layer(entry: Any, i: int) -> SosepelLayer:
    where = f"config.json: layers[{i}]"
    if not isinstance(entry, dict):
        raise ConfigError(f"{where} must be an object")
    r = KeyReader(entry, where)
    kind = r.opt_str("type", None)
    if kind != "attention":
        raise ConfigError(f"{where}: 'type' must be 'attention', got {kind!r}")
    m = _sub(r, "mixer")
    heads = m.need_int("heads", 1)
    kv_heads = m.opt_int("kv_heads", heads, 1)
    if heads % kv_heads:
        raise ConfigError(f"{where}: 'mixer.heads' must be a multiple of 'mixer.kv_heads'")
    coef, every = 0.0, 1
    if m.opt_raw("q_temp") is not None:
        t = _sub(m, "q_temp")
        coef, every = t.need_float("coef"), t.need_int("every", 1)
    diff = m.need_float("diff")
    cap = m.opt_float("softcap", 0.0)
    if cap < 0:
        raise ConfigError(f"{where}: 'mixer.softcap' must not be negative")
    mixer = DiffMixerConfig(heads, kv_heads, m.need_int("dim", 1), m.need_int("vdim", 1),
                            m.need_float("scale"), cap, diff, coef, every)
    mlp = None
    if r.opt_raw("mlp") is not None:
        f = _sub(r, "mlp")
        fk = f.opt_str("kind", "dense")
        if fk == "dense":
            mlp = MlpConfig("dense", f.need_int("ff", 1))
        elif fk == "moe":
            rt = _sub(f, "router")
            experts, top = rt.need_int("experts", 1), rt.need_int("top", 1)
            groups, kept = 1, 1
            if rt.opt_raw("groups") is not None:
                g = _sub(rt, "groups")
                groups = g.need_int("count", 1)
                kept = g.opt_int("keep", groups, 1)
            if top > experts or experts % groups or kept > groups \
                    or kept * (experts // groups) < top:
                raise ConfigError(f"{where}: 'mlp.router' does not fit: {experts} experts, top {top}, "
                                  f"{groups} groups of which {kept} are kept")
            shared = 0
            if f.opt_raw("shared") is not None:
                shared = _sub(f, "shared").need_int("ff", 1)
            mlp = MlpConfig("moe", _sub(f, "expert").need_int("ff", 1), experts, top, groups, kept,
                            shared)
        else:
            raise ConfigError(f"{where}: 'mlp.kind' must be 'dense' or 'moe', got {fk!r}")
    return SosepelLayer(kind, mixer, mlp)

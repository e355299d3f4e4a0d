"""Configuration of the Rupezen decoder, read from its config.json keys.

The file names the design under "architecture" and describes every layer by itself:

    vocab, width                      sizes of the embedding and of the residual stream
    norm.eps                          epsilon of every RMS norm
    residual_mult                     factor on every sublayer's output as it enters the stream (absent: 1)
    layers[i].type                    "attention": the layer's mixer (differential attention)
    layers[i].mixer                   heads, kv_heads, dim (of one score map), vdim, scale, diff (the
                                      lambda's constant), mask {size} (chunk length; absent: plain causal),
                                      rot {base, dims} (absent: no rotation)
    layers[i].mlp                     {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top",
                                      "groups": {"count", "keep"}}}, or null for a layer without feed-forward
    loop.start, loop.stop, loop.times layers start..stop-1 run `times` times in a row (absent: once); every
                                      pass begins with the projection of the stream beside the embedding's output
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, List, Optional

from .base import ConfigError, ModelConfig

MIXERS = ("attention",)


def _int(where: str, d: dict, key: str, least: int = 1) -> int:
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)) or float(v) != int(v) or int(v) < least:
        raise ConfigError(f"Rupezen: {where}.{key} must be an integer of at least {least}, got {v!r}")
    return int(v)


def _float(where: str, d: dict, key: str) -> float:
    v = d.get(key) if isinstance(d, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"Rupezen: {where}.{key} must be a number, got {v!r}")
    return float(v)


@dataclasses.dataclass(frozen=True)
class RupezenConfig(ModelConfig):
    vocab: int
    width: int
    layers: List[Dict[str, Any]]
    norm: Dict[str, Any]
    residual_mult: float = 1.0
    loop: Optional[Dict[str, Any]] = None

    def validate(self, raw):
        if self.vocab < 1 or self.width < 1:
            raise ConfigError(f"Rupezen: vocab {self.vocab} and width {self.width} must be positive")
        _float("norm", self.norm, "eps")
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("Rupezen: layers must be a list with at least one layer")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]"
            if not isinstance(layer, dict) or layer.get("type") not in MIXERS:
                raise ConfigError(f"Rupezen: {where}.type must be one of {MIXERS}, got "
                                  f"{layer.get('type') if isinstance(layer, dict) else layer!r}")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"Rupezen: {where}.mixer must be a dictionary")
            w = where + ".mixer"
            heads, kv = _int(w, m, "heads"), _int(w, m, "kv_heads")
            if heads % kv:
                raise ConfigError(f"Rupezen: {w}: {heads} heads are not a multiple of {kv} kv_heads")
            dim = _int(w, m, "dim")
            _int(w, m, "vdim")
            _float(w, m, "scale")
            _float(w, m, "diff")
            if m.get("mask") is not None:
                _int(w + ".mask", m["mask"], "size")
            if m.get("rot") is not None:
                dims = _int(w + ".rot", m["rot"], "dims", 2)
                if dims % 2 or dims > dim or _float(w + ".rot", m["rot"], "base") <= 0:
                    raise ConfigError(f"Rupezen: {w}.rot: dims {dims} must be even and at most dim {dim}, base positive")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "moe":
                    raise ConfigError(f"Rupezen: {where}.mlp.kind must be 'moe' (or mlp null), got {mlp!r}")
                _int(where + ".mlp.expert", mlp.get("expert"), "ff")
                r = mlp.get("router")
                experts, top = _int(where + ".mlp.router", r, "experts"), _int(where + ".mlp.router", r, "top")
                count, keep = 1, 1
                if r.get("groups") is not None:
                    count = _int(where + ".mlp.router.groups", r["groups"], "count")
                    keep = _int(where + ".mlp.router.groups", r["groups"], "keep")
                if experts % count or keep > count or top > keep * (experts // count):
                    raise ConfigError(f"Rupezen: {where}.mlp.router: {experts} experts in {count} groups, {keep} kept, "
                                      f"top {top} do not fit together")
        if self.loop is not None:
            start, stop = _int("loop", self.loop, "start", 0), _int("loop", self.loop, "stop", 0)
            _int("loop", self.loop, "times")
            if not start < stop <= len(self.layers):
                raise ConfigError(f"Rupezen: loop {start}..{stop} does not lie within the {len(self.layers)} layers")

    def run_order(self):
        """(layer, pass, whether the pass begins here) in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, 0, False) for i in range(n)]
        start, stop, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        order = [(i, 0, False) for i in range(start)]
        for p in range(times):
            order += [(i, p, i == start) for i in range(start, stop)]
        return order + [(i, 0, False) for i in range(stop, n)]

    def to_dict(self):
        out = {"architecture": self.architecture}
        for f in dataclasses.fields(self):
            if f.name != "architecture" and getattr(self, f.name) is not None:
                out[f.name] = getattr(self, f.name)
        return out

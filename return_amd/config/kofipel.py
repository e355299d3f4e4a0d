"""Configuration of the Kofipel decoder, read from its config.json keys.

The file names the design under "architecture" and describes every layer by itself:

    vocab, width                      sizes of the embedding and of the residual stream
    norm.eps                          epsilon of every RMS norm
    layers[i].type                    "attention" | "channel_delta": the layer's mixer
    layers[i].mixer                   the mixer's sizes and constants (see below)
    layers[i].mlp                     {"kind": "dense", "ff": n}, or null for a layer without feed-forward
    canon.taps                        taps of the causal convolution in front of every sublayer (absent: none)
    token_side.dim                    channels of the per-layer token input (absent: none)
    loop.start, loop.stop, loop.times layers start..stop-1 run `times` times in a row (absent: once)

attention mixer:      heads, kv_heads, dim, vdim, scale, softcap (absent or 0: none),
                      mask {size, keep_first} (absent: plain causal), rot {base, dims} (absent: no rotation)
channel_delta mixer:  heads, kv_heads, dim, vdim, conv (taps of the short convolution on q, k and v)
A mixer may name "rank", the width of its low-rank maps, which only the random-weights mode reads:
a stored model gives it by its tensors' shapes.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, List, Optional

from .base import ConfigError, ModelConfig

MIXERS = ("attention", "channel_delta")


def _int(where: str, d: dict, key: str, least: int = 1) -> int:
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)) or float(v) != int(v) or int(v) < least:
        raise ConfigError(f"Kofipel: {where}.{key} must be an integer of at least {least}, got {v!r}")
    return int(v)


def _float(where: str, d: dict, key: str) -> float:
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"Kofipel: {where}.{key} must be a number, got {v!r}")
    return float(v)


@dataclasses.dataclass(frozen=True)
class KofipelConfig(ModelConfig):
    vocab: int
    width: int
    layers: List[Dict[str, Any]]
    norm: Dict[str, Any]
    canon: Optional[Dict[str, Any]] = None
    token_side: Optional[Dict[str, Any]] = None
    loop: Optional[Dict[str, Any]] = None

    def validate(self, raw):
        if self.vocab < 1 or self.width < 1:
            raise ConfigError(f"Kofipel: vocab {self.vocab} and width {self.width} must be positive")
        if not isinstance(self.norm, dict):
            raise ConfigError("Kofipel: norm must be a dictionary with eps")
        _float("norm", self.norm, "eps")
        if not isinstance(self.layers, list) or not self.layers:
            raise ConfigError("Kofipel: layers must be a list with at least one layer")
        for i, layer in enumerate(self.layers):
            where = f"layers[{i}]"
            if not isinstance(layer, dict) or layer.get("type") not in MIXERS:
                raise ConfigError(f"Kofipel: {where}.type must be one of {MIXERS}, got "
                                  f"{layer.get('type') if isinstance(layer, dict) else layer!r}")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"Kofipel: {where}.mixer must be a dictionary")
            heads, kv = _int(where + ".mixer", m, "heads"), _int(where + ".mixer", m, "kv_heads")
            if heads % kv:
                raise ConfigError(f"Kofipel: {where}.mixer: {heads} heads are not a multiple of {kv} kv_heads")
            dim, vdim = _int(where + ".mixer", m, "dim"), _int(where + ".mixer", m, "vdim")
            if layer["type"] == "attention":
                _float(where + ".mixer", m, "scale")
                if vdim != dim:
                    raise ConfigError(f"Kofipel: {where}.mixer: the values are the keys, so vdim {vdim} must be dim {dim}")
                if m.get("softcap") is not None and _float(where + ".mixer", m, "softcap") < 0:
                    raise ConfigError(f"Kofipel: {where}.mixer.softcap must not be negative")
                if m.get("mask") is not None:
                    _int(where + ".mixer.mask", m["mask"], "size")
                    _int(where + ".mixer.mask", m["mask"], "keep_first", 0)
                if m.get("rot") is not None:
                    dims = _int(where + ".mixer.rot", m["rot"], "dims", 2)
                    if dims % 2 or dims > dim or _float(where + ".mixer.rot", m["rot"], "base") <= 0:
                        raise ConfigError(f"Kofipel: {where}.mixer.rot: dims {dims} must be even and at most dim {dim}, "
                                          "base positive")
            else:
                _int(where + ".mixer", m, "conv")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise ConfigError(f"Kofipel: {where}.mlp.kind must be 'dense' (or mlp null), got {mlp!r}")
                _int(where + ".mlp", mlp, "ff")
        if self.canon is not None:
            _int("canon", self.canon, "taps")
        if self.token_side is not None:
            _int("token_side", self.token_side, "dim")
        if self.loop is not None:
            start, stop = _int("loop", self.loop, "start", 0), _int("loop", self.loop, "stop", 0)
            _int("loop", self.loop, "times")
            if not start < stop <= len(self.layers):
                raise ConfigError(f"Kofipel: loop {start}..{stop} does not lie within the {len(self.layers)} layers")

    def run_order(self):
        """(layer, pass) in the order the layers run: layers loop.start..loop.stop-1 `times` times in a row."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, 0) for i in range(n)]
        start, stop, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        order = [(i, 0) for i in range(start)]
        for p in range(times):
            order += [(i, p) for i in range(start, stop)]
        return order + [(i, 0) for i in range(stop, n)]

    def to_dict(self):
        out = {"architecture": self.architecture}
        for f in dataclasses.fields(self):
            if f.name != "architecture" and getattr(self, f.name) is not None:
                out[f.name] = getattr(self, f.name)
        return out

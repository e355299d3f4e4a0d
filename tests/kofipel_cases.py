"""Small Kofipel configurations for the tests, each with random weights of its own. They differ from
one another in every size and option: layer order, head counts with and without grouping, key and
value sizes that differ, sizes that are no power of two, windows, kept keys, rotations over part of
a head or none, loops over some or all layers, layers without feed-forward, with and without the
convolutions and the token input."""
from __future__ import annotations

import copy


def _delta(heads, kv_heads, dim, vdim, conv, rank):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                               "conv": conv, "rank": rank}}


def _attn(heads, kv_heads, dim, scale, softcap=None, mask=None, rot=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if softcap is not None:
        m["softcap"] = softcap
    if mask is not None:
        m["mask"] = {"size": mask[0], "keep_first": mask[1]}
    if rot is not None:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
    return {"type": "attention", "mixer": m}


def _with_mlp(layer, ff):
    layer = copy.deepcopy(layer)
    layer["mlp"] = {"kind": "dense", "ff": ff} if ff else None
    return layer


# loop over the two middle layers, grouped heads, window that passes 64, kept keys, rotation over half a head
KOFI_A = {
    "architecture": "Kofipel", "vocab": 200, "width": 64, "norm": {"eps": 1e-5},
    "canon": {"taps": 3}, "token_side": {"dim": 8}, "loop": {"start": 1, "stop": 3, "times": 2},
    "layers": [
        _with_mlp(_delta(2, 1, 16, 32, 4, 8), 96),
        _with_mlp(_attn(4, 2, 16, 0.4, softcap=8.0, mask=(70, 3), rot=(10000.0, 8)), 96),
        _with_mlp(_delta(4, 4, 8, 16, 2, 4), 80),
        _with_mlp(_attn(2, 2, 32, 0.25, softcap=30.0, mask=(20, 17), rot=(500000.0, 32)), 96),
    ]}
KOFI_A_INIT = dict(seed=11, std=0.12, embedding_std=1.0, norm_jitter=0.1)

# nothing a power of two, no grouping, a layer without feed-forward, a window without kept keys, no loop
KOFI_B = {
    "architecture": "Kofipel", "vocab": 131, "width": 72, "norm": {"eps": 3e-6},
    "canon": {"taps": 2}, "token_side": {"dim": 5},
    "layers": [
        _with_mlp(_attn(3, 3, 24, 0.2, mask=(9, 0), rot=(1000.0, 24)), 100),
        _with_mlp(_delta(3, 3, 12, 20, 3, 6), None),
        _with_mlp(_attn(6, 1, 12, 0.5, softcap=4.0, mask=(33, 40), rot=(100.0, 4)), 52),
        _with_mlp(_delta(6, 2, 20, 12, 5, 3), 60),
    ]}
KOFI_B_INIT = dict(seed=12, std=0.1, embedding_std=0.7, norm_jitter=0.2)

# no convolutions, no token input, plain causal attention without rotation, every layer looped three times
KOFI_C = {
    "architecture": "Kofipel", "vocab": 96, "width": 48, "norm": {"eps": 1e-6},
    "loop": {"start": 0, "stop": 2, "times": 3},
    "layers": [
        _with_mlp(_attn(2, 1, 16, 0.3), 64),
        _with_mlp(_delta(1, 1, 64, 48, 1, 2), 64),
    ]}
KOFI_C_INIT = dict(seed=13, std=0.12, embedding_std=1.0, norm_jitter=0.05)

CASES = {"a": (KOFI_A, KOFI_A_INIT), "b": (KOFI_B, KOFI_B_INIT), "c": (KOFI_C, KOFI_C_INIT)}


def make_folder(tmp_path_factory, name, dtype="bfloat16"):
    from tests.conftest import make_folder as make
    raw, init = CASES[name]
    return make(tmp_path_factory, "kofipel_" + name, dict(raw, architectures=[raw["architecture"]]), init, dtype)

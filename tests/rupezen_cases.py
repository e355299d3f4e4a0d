"""Small Rupezen configurations for the tests, each with random weights of its own. They differ from one
another in every size and option: head counts with and without grouping, map and value sizes (value rows
narrower than, as wide as and wider than a key row of two maps), sizes that are no power of two, chunks
that are and are not multiples of a page, rotation over part of a map, all of it or none, loops over
some or all layers or none, layers without feed-forward, routers with and without groups, groups of one
expert, top 1, stream factors other than a power of two."""
from __future__ import annotations


def _layer(heads, kv_heads, dim, vdim, scale, diff, chunk=None, rot=None, moe=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff}
    if chunk is not None:
        m["mask"] = {"size": chunk}
    if rot is not None:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
    mlp = None
    if moe is not None:
        ff, experts, top, count, keep = moe
        mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
        if count is not None:
            mlp["router"]["groups"] = {"count": count, "keep": keep}
    return {"type": "attention", "mixer": m, "mlp": mlp}


# loop over the two middle layers; grouped heads; value rows wider and narrower than the two maps; chunks
# that are no multiple of a page and one that is
RUPE_A = {
    "architecture": "Rupezen", "vocab": 211, "width": 64, "norm": {"eps": 1e-5}, "residual_mult": 0.7,
    "loop": {"start": 1, "stop": 3, "times": 2},
    "layers": [
        _layer(4, 2, 8, 24, 0.4, 0.3, chunk=20, rot=(10000.0, 4), moe=(24, 8, 2, 4, 2)),
        _layer(2, 1, 16, 8, 0.3, 0.6, chunk=48, rot=(100.0, 16), moe=(40, 6, 3, 2, 1)),
        _layer(6, 3, 4, 12, 0.5, 0.2, chunk=7, rot=None, moe=None),
        _layer(2, 2, 12, 24, 0.25, 0.8, chunk=33, rot=(500000.0, 6), moe=(16, 5, 1, None, None)),
    ]}
RUPE_A_INIT = dict(seed=21, std=0.12, embedding_std=1.0, norm_jitter=0.1)

# no loop; nothing a power of two; one layer with plain causal attention; groups of one expert; a factor of 1
RUPE_B = {
    "architecture": "Rupezen", "vocab": 97, "width": 76, "norm": {"eps": 3e-6}, "residual_mult": 1.0,
    "layers": [
        _layer(3, 3, 10, 20, 0.3, 0.5, chunk=17, rot=(1000.0, 10), moe=(20, 6, 2, 6, 3)),
        _layer(6, 1, 6, 14, 0.4, 0.1, chunk=None, rot=(50.0, 2), moe=(28, 9, 4, 3, 2)),
        _layer(3, 1, 12, 36, 0.2, 0.4, chunk=64, rot=(10000.0, 12), moe=None),
    ]}
RUPE_B_INIT = dict(seed=22, std=0.1, embedding_std=0.7, norm_jitter=0.2)

# every layer looped three times, sizes the matrix-core kernels take (multiples of 16 and of 8), a chunk of one page
RUPE_C = {
    "architecture": "Rupezen", "vocab": 128, "width": 96, "norm": {"eps": 1e-6}, "residual_mult": 0.5,
    "loop": {"start": 0, "stop": 2, "times": 3},
    "layers": [
        _layer(4, 2, 16, 32, 0.25, 0.5, chunk=16, rot=(10000.0, 8), moe=(32, 8, 2, 2, 1)),
        _layer(2, 1, 32, 96, 0.18, 0.35, chunk=40, rot=(10000.0, 32), moe=(64, 4, 2, 1, 1)),
    ]}
RUPE_C_INIT = dict(seed=23, std=0.12, embedding_std=1.0, norm_jitter=0.05)

CASES = {"a": (RUPE_A, RUPE_A_INIT), "b": (RUPE_B, RUPE_B_INIT), "c": (RUPE_C, RUPE_C_INIT)}


def random_case(seed):
    """A configuration drawn from a seed: one to four layers, every size and option drawn on its own (sizes that the
    matrix-core kernels take and sizes they do not, value rows of any width beside the maps, chunks from 1 on, with
    and without rotation, mask, feed-forward, groups, loop)."""
    import random
    rng = random.Random(seed)
    n_layers = rng.choice([1, 2, 3, 4])
    layers = []
    for _ in range(n_layers):
        kv = rng.choice([1, 1, 2, 3])
        heads = kv * rng.choice([1, 2, 4, 5, 18] if kv == 1 else [1, 2, 4])
        if rng.random() < 0.5:
            dim, vdim = rng.choice([16, 32, 48, 64]), rng.choice([32, 64, 96, 128])
        else:
            dim, vdim = rng.choice([2, 4, 6, 10, 24, 40]), rng.choice([2, 5, 8, 20, 33, 48])
        chunk = rng.choice([None, 1, 2, 5, 16, 31, 32, 64, 100, 128])
        rot = (rng.choice([10.0, 10000.0, 1e6]), rng.choice(range(2, dim + 1, 2))) if rng.random() < 0.8 else None
        moe = None
        if rng.random() < 0.8:
            count, per = rng.choice([1, 2, 3, 4]), rng.choice([1, 2, 3, 5])
            keep = rng.randint(1, count)
            moe = (rng.choice([4, 8, 12, 24, 40]), count * per, rng.randint(1, min(keep * per, 6)), count, keep)
        layers.append(_layer(heads, kv, dim, vdim, rng.choice([dim ** -0.5, 0.3, 2.0 / dim]), rng.choice([0.1, 0.35, 0.5, 0.8]),
                             chunk=chunk, rot=rot, moe=moe))
    raw = {"architecture": "Rupezen", "vocab": rng.choice([50, 97, 256]), "width": rng.choice([16, 24, 40, 64, 96, 200]),
           "norm": {"eps": rng.choice([1e-6, 1e-5])}, "residual_mult": rng.choice([0.5, 1.0, 0.7, 1.5]), "layers": layers}
    if rng.random() < 0.7:
        start = rng.randrange(0, n_layers)
        raw["loop"] = {"start": start, "stop": rng.randint(start + 1, n_layers), "times": rng.choice([1, 2, 3])}
    return raw, dict(seed=seed, std=0.15, embedding_std=1.0, norm_jitter=0.1)


def make_folder(tmp_path_factory, name, dtype="bfloat16"):
    from tests.conftest import make_folder as make
    raw, init = random_case(name) if isinstance(name, int) else CASES[name]
    name = str(name)
    return make(tmp_path_factory, "rupezen_" + name, dict(raw, architectures=[raw["architecture"]]), init, dtype)

"""Rupezen as a ModelSpec: a decoder whose layers are described one by one in config.json.

Every layer is a pre-norm block whose sublayers enter the stream times residual_mult: a differential
attention (two score maps per head over the same values, chunked causal mask, interleaved rotation over
the first elements of each map) and a routed feed-forward (sigmoid router with a correction on the
choice, groups of experts) or none. A run of layers may repeat with the same weights; every pass keeps
a cache of its own and begins with  h <- W_in [h ; h0] + step[pass]  (h0: the embedding's output).
The head is the embedding table. Tensor names: "embed", "final.norm", "loop.in", "loop.step", and
"l<i>." + norm1, norm2, mix.{q,k,v,o,lq1,lk1,lq2,lk2}, mlp.router, mlp.correction, mlp.e<j>.{gate,up,down}.
"""
from __future__ import annotations

from ..config.base import register_architecture
from ..config.rupezen import RupezenConfig
from ..parts.moe import GroupedRoutedExperts
from ..parts.spec import BlockSpec, LayerCall, ModelSpec, PartSpec


def _attention(cfg, i, m, positions):
    p = f"l{i}.mix."
    mask, rot = m.get("mask"), m.get("rot")
    position = None
    if rot is not None:
        position = f"rotary_pairs_{int(m['dim'])}_{int(rot['dims'])}_{float(rot['base'])!r}"
        positions.setdefault(position, PartSpec("rotary", {
            "head_dim": int(m["dim"]), "rotary_dim": int(rot["dims"]), "theta": float(rot["base"]),
            "max_position": None, "exact_tables": True, "pairing": "interleaved"}))
    params = {"hidden_size": cfg.width, "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]),
              "head_dim": int(m["dim"]), "value_dim": int(m["vdim"]), "scale": float(m["scale"]),
              "lambda_init": float(m["diff"]), "eps": float(cfg.norm["eps"]), "position": position,
              "chunk": int(mask["size"]) if mask else None}
    tensors = {"q_proj": p + "q", "k_proj": p + "k", "v_proj": p + "v", "o_proj": p + "o",
               "lq1": p + "lq1", "lk1": p + "lk1", "lq2": p + "lq2", "lk2": p + "lk2"}
    return PartSpec("differential_attention", params, tensors)


def _experts(cfg, i, mlp):
    r = mlp["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    params = {"hidden_size": cfg.width, "expert_size": int(mlp["expert"]["ff"]), "experts": int(r["experts"]),
              "top": int(r["top"]), "groups": int(groups["count"]), "keep": int(groups["keep"]), "norm_eps": 1e-20}
    return PartSpec("grouped_routed_experts", params,
                    GroupedRoutedExperts.tensor_names(f"l{i}.mlp.", int(r["experts"])))


def build_spec(cfg: RupezenConfig) -> ModelSpec:
    W, eps = cfg.width, float(cfg.norm["eps"])
    norm = lambda name: PartSpec("rms_norm", {"size": W, "eps": eps, "offset": 0.0}, {"weight": name})
    positions, blocks = {}, []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        parts = {"mixer_norm": ("norm", norm(p + "norm1")),
                 "mixer": ("mixer", _attention(cfg, i, layer["mixer"], positions)),
                 "residual": ("norm", PartSpec("factor", {"factor": float(cfg.residual_mult)}))}
        if layer.get("mlp") is not None:
            parts["feed_forward_norm"] = ("norm", norm(p + "norm2"))
            parts["feed_forward"] = ("feed_forward", _experts(cfg, i, layer["mlp"]))
        blocks.append(BlockSpec(parts, "pre_norm_scaled"))
    # a layer without feed-forward has no use for a second norm: a file that stores one all the same loads
    ignorable = [f"l{i}.norm2" for i, layer in enumerate(cfg.layers) if layer.get("mlp") is None]
    schedule = [LayerCall(block=i, cache=n, writes_cache=True, pass_input=p if first else None)
                for n, (i, p, first) in enumerate(cfg.run_order())]
    pass_input = None
    if cfg.loop is not None:
        pass_input = PartSpec("concat_linear", {"hidden_size": W, "passes": int(cfg.loop["times"])},
                              {"weight": "loop.in", "step": "loop.step"})
    return ModelSpec(
        architecture=cfg.architecture, hidden_size=W, vocab_size=cfg.vocab, max_position=None,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": W}, {"weight": "embed"}),
        positions=positions, blocks=blocks, schedule=schedule, final_norm=norm("final.norm"),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": W, "tied": True}, {"weight": "embed"}),
        ignorable=ignorable, pass_input=pass_input)


register_architecture("Rupezen", RupezenConfig, build_spec)

"""Kofipel as a ModelSpec: a decoder whose layers are described one by one in config.json.

Every layer is a pre-norm block with a causal convolution in front of each sublayer, a mixer that
is either an attention (sliding window with kept first keys, a sink in the softmax, a soft cap on
the scores, a learned temperature per head, values that are the keys) or a gated delta rule with a
decay per key channel, a dense feed-forward with a squared ReLU (or none), and a token input at the
end. A run of layers may repeat several times with the same weights; every pass keeps a cache and
state of its own, and from the second pass on the embedding's output is added to the stream before
the pass begins. Tensor names: "embed", "head", "final.norm", "side.embed", and "l<i>." + norm1,
norm2, canon1, canon2, mix.*, mlp.up, mlp.down, side.gate, side.proj, side.norm.
"""
from __future__ import annotations

from ..config.base import register_architecture
from ..config.kofipel import KofipelConfig
from ..parts.spec import BlockSpec, LayerCall, ModelSpec, PartSpec


def _attention(cfg, i, m, positions):
    p = f"l{i}.mix."
    mask, rot = m.get("mask"), m.get("rot")
    position = None
    if rot is not None:
        position = f"rotary_{int(m['dim'])}_{int(rot['dims'])}_{float(rot['base'])!r}"
        positions.setdefault(position, PartSpec("rotary", {
            "head_dim": int(m["dim"]), "rotary_dim": int(rot["dims"]), "theta": float(rot["base"]),
            "max_position": None, "exact_tables": True}))
    params = {"hidden_size": cfg.width, "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]),
              "head_dim": int(m["dim"]), "scale": float(m["scale"]), "qk_norm_eps": None, "position": position,
              "window": int(mask["size"]) if mask else None, "keep_first": int(mask["keep_first"]) if mask else 0,
              "softcap": float(m.get("softcap") or 0.0), "sink": True, "head_temperature": True, "bias": True,
              "values": "keys"}
    tensors = {"q_proj": p + "q", "k_proj": p + "k", "o_proj": p + "o", "q_bias": p + "q.b", "k_bias": p + "k.b",
               "o_bias": p + "o.b", "temp": p + "temp"}
    return PartSpec("attention", params, tensors)


def _channel_delta(cfg, i, m):
    p = f"l{i}.mix."
    rank = m.get("rank")
    params = {"hidden_size": cfg.width, "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]),
              "head_dim": int(m["dim"]), "value_dim": int(m["vdim"]), "conv_taps": int(m["conv"]),
              "eps": float(cfg.norm["eps"]), "decay_rank": rank, "gate_rank": rank}
    tensors = {"q_proj": p + "q", "k_proj": p + "k", "v_proj": p + "v", "q_conv": p + "q.conv", "k_conv": p + "k.conv",
               "v_conv": p + "v.conv", "b_proj": p + "b", "A_log": p + "A_log", "dt_bias": p + "dt_bias",
               "o_norm": p + "norm", "a1_proj": p + "a1", "a2_proj": p + "a2", "g1_proj": p + "g1", "g2_proj": p + "g2",
               "o_proj": p + "o"}
    return PartSpec("channel_delta", params, tensors)


def build_spec(cfg: KofipelConfig) -> ModelSpec:
    W, eps = cfg.width, float(cfg.norm["eps"])
    norm = lambda name: PartSpec("rms_norm", {"size": W, "eps": eps, "offset": 0.0}, {"weight": name})
    taps = int(cfg.canon["taps"]) if cfg.canon else None
    side = int(cfg.token_side["dim"]) if cfg.token_side else None
    n_layers = len(cfg.layers)
    positions, blocks = {}, []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        m = layer["mixer"]
        mixer = _attention(cfg, i, m, positions) if layer["type"] == "attention" else _channel_delta(cfg, i, m)
        parts = {"mixer_norm": ("norm", norm(p + "norm1")), "mixer": ("mixer", mixer)}
        conv = lambda name: ("input_conv", PartSpec("residual_causal_conv", {"size": W, "taps": taps}, {"weight": name}))
        if taps:
            parts["mixer_conv"] = conv(p + "canon1")
        if layer.get("mlp") is not None:
            parts["feed_forward_norm"] = ("norm", norm(p + "norm2"))
            parts["feed_forward"] = ("feed_forward", PartSpec(
                "relu2", {"hidden_size": W, "intermediate_size": int(layer["mlp"]["ff"])},
                {"up_proj": p + "mlp.up", "down_proj": p + "mlp.down"}))
            if taps:
                parts["feed_forward_conv"] = conv(p + "canon2")
        if side:
            parts["token_input"] = ("token_input", PartSpec(
                "gated_token_side", {"hidden_size": W, "dim": side, "offset": i * side, "table_width": n_layers * side,
                                     "vocab_size": cfg.vocab, "eps": eps},
                {"table": "side.embed", "gate": p + "side.gate", "proj": p + "side.proj", "norm": p + "side.norm"}))
        blocks.append(BlockSpec(parts, "pre_norm_conv_side"))
    # a layer without feed-forward has no use for a second norm and convolution: a file that stores them all the same loads
    ignorable = [f"l{i}.{name}" for i, layer in enumerate(cfg.layers) if layer.get("mlp") is None
                 for name in ("norm2", "canon2")]
    # every run of a layer has cache layers of its own: the mixer's, then the convolutions' tails
    schedule, layer_no = [], 0
    start = int(cfg.loop["start"]) if cfg.loop else None
    for i, p in cfg.run_order():
        kept = 1 + (1 if taps else 0)
        schedule.append(LayerCall(block=i, cache=layer_no if kept == 1 else tuple(range(layer_no, layer_no + kept)),
                                  writes_cache=True, add_input=bool(p > 0 and i == start)))
        layer_no += kept
    return ModelSpec(
        architecture=cfg.architecture, hidden_size=W, vocab_size=cfg.vocab, max_position=None,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": W}, {"weight": "embed"}),
        positions=positions, blocks=blocks, schedule=schedule, final_norm=norm("final.norm"),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": W, "tied": False}, {"weight": "head"}),
        ignorable=ignorable)


register_architecture("Kofipel", KofipelConfig, build_spec)

"""The Kofipel decoder, plain and slow: whole sequences in 64-bit, no cache, no batches, one function
per mechanism, written from the design's equations. Nothing here is shared with return_amd; the engine
is compared against this.

Notation: x is the residual stream [T, W]; a weight named W_foo is stored [out, in] and applied as
x @ W_foo^T; positions count from 0.
"""
from __future__ import annotations

import json
import math
import os

import torch
from safetensors import safe_open

F = torch.float64


def read_folder(folder):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            w[name] = f.get_tensor(name).to(F)
    return cfg, w


# ---------------------------------------------------------------- small pieces
def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * weight, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def causal_filter(x, taps_w):
    """y_t = sum_j w[:, j] x_(t - taps + 1 + j) on each channel; x [T, C], w [C, taps]; zeros before t = 0."""
    T, C = x.shape
    taps = taps_w.shape[1]
    y = torch.zeros(T, C, dtype=F)
    for t in range(T):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                y[t] += taps_w[:, j] * x[src]
    return y


def rotate_half(x, positions, base, dims):
    """The first ``dims`` elements of every head, element i paired with i + dims/2:
    (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = position * base^(-2i/dims). x [T, heads, D]."""
    half = dims // 2
    out = x.clone()
    for i in range(half):
        a = positions.to(F) * base ** (-2.0 * i / dims)
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, v = x[:, :, i], x[:, :, i + half]
        out[:, :, i] = u * c - v * s
        out[:, :, i + half] = v * c + u * s
    return out


def visible(i, j, window, keep_first):
    """Whether the query at position i reads the key at position j."""
    if j > i:
        return False
    if window is None:
        return True
    return i - j < window or j < keep_first


# ---------------------------------------------------------------- mixers
def window_sink_attention(h, w, pre, m):
    """Attention whose values are its keys as projected (before rotation), with biases on q, k and the
    output, a temperature per head, a soft cap, a sliding window with kept first keys, and a softmax
    with one added to its denominator."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w[pre + "q"].T + w[pre + "q.b"]).view(T, H, D)
    k = (h @ w[pre + "k"].T + w[pre + "k.b"]).view(T, G, D)
    v = k.clone()
    pos = torch.arange(T)
    if m.get("rot"):
        q = rotate_half(q, pos, float(m["rot"]["base"]), int(m["rot"]["dims"]))
        k = rotate_half(k, pos, float(m["rot"]["base"]), int(m["rot"]["dims"]))
    mask = m.get("mask")
    window = mask["size"] if mask else None
    keep = mask["keep_first"] if mask else 0
    cap = m.get("softcap") or 0.0
    see = torch.tensor([[visible(i, j, window, keep) for j in range(T)] for i in range(T)])
    out = torch.zeros(T, H, D, dtype=F)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * m["scale"] * w[pre + "temp"][head]
        if cap:
            s = cap * torch.tanh(s / cap)
        e = torch.exp(s) * see                      # the keys a query does not read weigh nothing
        p = e / (1.0 + e.sum(-1, keepdim=True))     # one more key of score 0, which has no value
        out[:, head] = p @ v[:, g]
    return out.reshape(T, H * D) @ w[pre + "o"].T + w[pre + "o.b"]


def channel_delta(h, w, pre, m, eps):
    """Gated delta rule with a decay per head and key channel, a matrix S [D, V] per head."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    silu = lambda z: z * torch.sigmoid(z)
    q = silu(causal_filter(h @ w[pre + "q"].T, w[pre + "q.conv"])).view(T, G, D)
    k = silu(causal_filter(h @ w[pre + "k"].T, w[pre + "k.conv"])).view(T, G, D)
    v = silu(causal_filter(h @ w[pre + "v"].T, w[pre + "v.conv"])).view(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[pre + "b"].T)
    step = torch.nn.functional.softplus((h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "dt_bias"]).view(T, H, D)
    decay = torch.exp(-torch.exp(w[pre + "A_log"])[None, :, None] * step)
    gate = torch.sigmoid((h @ w[pre + "g1"].T) @ w[pre + "g2"].T).view(T, H, V)
    out = torch.zeros(T, H, V, dtype=F)
    for head in range(H):
        g = head // (H // G)
        S = torch.zeros(D, V, dtype=F)
        for t in range(T):
            S = decay[t, head][:, None] * S
            u = beta[t, head] * (v[t, head] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, head] = S.T @ q[t, g]
    out = out / torch.sqrt((out * out).mean(-1, keepdim=True) + eps) * w[pre + "norm"] * gate
    return out.reshape(T, H * V) @ w[pre + "o"].T


def dense_mlp(h, w, pre):
    return torch.relu(h @ w[pre + "up"].T) ** 2 @ w[pre + "down"].T


def token_side(x, tokens, w, i, dim, eps):
    """What layer i adds for the token itself: its columns of the side table, gated by the stream."""
    e = w["side.embed"][tokens][:, i * dim:(i + 1) * dim]
    g = gelu_tanh(x @ w[f"l{i}.side.gate"].T) * e
    y = g @ w[f"l{i}.side.proj"].T
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps) * w[f"l{i}.side.norm"]


# ---------------------------------------------------------------- the model
def run_order(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, 0) for i in range(n)]
    order = [(i, 0) for i in range(loop["start"])]
    for p in range(loop["times"]):
        order += [(i, p) for i in range(loop["start"], loop["stop"])]
    return order + [(i, 0) for i in range(loop["stop"], n)]


def hidden_states(cfg, w, tokens):
    """The residual stream after every layer run, and the final one."""
    eps = cfg["norm"]["eps"]
    tok = torch.tensor(list(tokens), dtype=torch.long)
    x0 = w["embed"][tok]
    x = x0.clone()
    taps = (cfg.get("canon") or {}).get("taps")
    side = (cfg.get("token_side") or {}).get("dim")
    loop = cfg.get("loop")
    states = []
    for i, p in run_order(cfg):
        if loop and p > 0 and i == loop["start"]:
            x = x + x0
        layer, pre = cfg["layers"][i], f"l{i}."
        h = rms_norm(x, w[pre + "norm1"], eps)
        if taps:
            h = h + causal_filter(h, w[pre + "canon1"])
        if layer["type"] == "attention":
            x = x + window_sink_attention(h, w, pre + "mix.", layer["mixer"])
        else:
            x = x + channel_delta(h, w, pre + "mix.", layer["mixer"], eps)
        if layer.get("mlp"):
            h = rms_norm(x, w[pre + "norm2"], eps)
            if taps:
                h = h + causal_filter(h, w[pre + "canon2"])
            x = x + dense_mlp(h, w, pre + "mlp.")
        if side:
            x = x + token_side(x, tok, w, i, side, eps)
        states.append(x.clone())
    return states


def logits(cfg, w, tokens):
    """fp32 logits [T, vocab] of a whole sequence."""
    with torch.no_grad():
        x = hidden_states(cfg, w, tokens)[-1]
        return (rms_norm(x, w["final.norm"], cfg["norm"]["eps"]) @ w["head"].T).float()


def greedy(cfg, w, prompt, n_new):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(logits(cfg, w, toks)[-1].argmax()))
    return toks[len(prompt):]

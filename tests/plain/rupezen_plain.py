"""The Rupezen decoder, plain and slow: whole sequences in 64-bit, no cache, no batches, one function
per mechanism, written from the design's equations. Nothing here is shared with return_amd; the engine
is compared against this.

Notation: x is the residual stream [T, W]; a weight W_foo is stored [out, in] and applied as
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
    """x / sqrt(mean(x^2) + eps) * weight, eps inside the root (weight None: no weight)."""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def rotate_pairs(x, positions, base, dims):
    """The first ``dims`` elements of the last axis, element 2i paired with 2i + 1:
    (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = position * base^(-2i/dims). x [T, ..., D]."""
    out = x.clone()
    shape = [-1] + [1] * (x.dim() - 2)
    for i in range(dims // 2):
        a = positions.to(F) * base ** (-2.0 * i / dims)
        c, s = torch.cos(a).view(shape), torch.sin(a).view(shape)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def sees(i, j, chunk):
    """Whether the query at position i reads the key at position j: j <= i, and with a chunked mask
    both in the same chunk, chunks counted from position 0."""
    if j > i:
        return False
    return chunk is None or i // chunk == j // chunk


# ---------------------------------------------------------------- mixer
def differential_lambda(w, pre, diff):
    """exp(lq1 . lk1) - exp(lq2 . lk2) + diff: one number for the layer."""
    return math.exp(float((w[pre + "lq1"] * w[pre + "lk1"]).sum())) - \
        math.exp(float((w[pre + "lq2"] * w[pre + "lk2"]).sum())) + diff


def softmax_map(q, k, v, scale, see):
    """One attention map: softmax over the visible keys of q k^T * scale, times v."""
    s = (q @ k.T) * scale
    s = s.masked_fill(~see, float("-inf"))
    return torch.softmax(s, dim=-1) @ v


def differential_attention(h, w, pre, m, eps):
    """Two softmax maps per head over the same values, subtracted with the layer's lambda, the result
    normed over the head's values (no weight) and scaled by 1 - diff."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    diff = float(m["diff"])
    q = (h @ w[pre + "q"].T).view(T, H, 2, D)
    k = (h @ w[pre + "k"].T).view(T, G, 2, D)
    v = (h @ w[pre + "v"].T).view(T, G, V)
    pos = torch.arange(T)
    if m.get("rot"):
        q = rotate_pairs(q, pos, float(m["rot"]["base"]), int(m["rot"]["dims"]))
        k = rotate_pairs(k, pos, float(m["rot"]["base"]), int(m["rot"]["dims"]))
    chunk = int(m["mask"]["size"]) if m.get("mask") else None
    see = torch.tensor([[sees(i, j, chunk) for j in range(T)] for i in range(T)])
    lam = differential_lambda(w, pre, diff)
    out = torch.zeros(T, H, V, dtype=F)
    for head in range(H):
        g = head // (H // G)
        a1 = softmax_map(q[:, head, 0], k[:, g, 0], v[:, g], m["scale"], see)
        a2 = softmax_map(q[:, head, 1], k[:, g, 1], v[:, g], m["scale"], see)
        out[:, head] = rms_norm(a1 - lam * a2, None, eps) * (1.0 - diff)
    return out.reshape(T, H * V) @ w[pre + "o"].T


# ---------------------------------------------------------------- feed-forward
def route(z, correction, top, group_count, group_keep):
    """Which experts each token uses and with what weights. z: router logits [T, E]. Returns
    (chosen [T, top] expert numbers, weights [T, top])."""
    T, E = z.shape
    s = torch.sigmoid(z)
    choice = s + correction
    per = E // group_count
    grouped = choice.view(T, group_count, per)
    group_score = grouped.topk(min(2, per), dim=-1).values.sum(-1)            # [T, groups]
    best = group_score.topk(group_keep, dim=-1).indices                       # [T, keep]
    allowed = torch.zeros(T, group_count, dtype=torch.bool)
    allowed.scatter_(1, best, True)
    allowed = allowed[:, :, None].expand(T, group_count, per).reshape(T, E)
    masked = choice.masked_fill(~allowed, float("-inf"))
    chosen = masked.topk(top, dim=-1).indices
    picked = s.gather(1, chosen)
    return chosen, picked / (picked.sum(-1, keepdim=True) + 1e-20)


def expert(h, w, pre):
    z = h @ w[pre + "gate"].T
    return ((z * torch.sigmoid(z)) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def routed_feed_forward(h, w, pre, mlp):
    r = mlp["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}                      # (no groups: one group of all)
    chosen, weights = route(h @ w[pre + "router"].T, w[pre + "correction"], int(r["top"]),
                            int(groups["count"]), int(groups["keep"]))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t].tolist(), weights[t]):
            out[t] += a * expert(h[t:t + 1], w, f"{pre}e{e}.")[0]
    return out


# ---------------------------------------------------------------- the model
def run_order(cfg):
    """(layer, pass, first of its pass) in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, 0, i == 0) for i in range(n)], 1
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, 0, False) for i in range(start)]
    for p in range(times):
        order += [(i, p, i == start) for i in range(start, stop)]
    return order + [(i, 0, False) for i in range(stop, n)], times


def layer(x, w, i, spec, cfg):
    eps, mult = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    pre = f"l{i}."
    x = x + mult * differential_attention(rms_norm(x, w[pre + "norm1"], eps), w, pre + "mix.", spec["mixer"], eps)
    if spec.get("mlp") is not None:
        x = x + mult * routed_feed_forward(rms_norm(x, w[pre + "norm2"], eps), w, pre + "mlp.", spec["mlp"])
    return x


def hidden_states(cfg, w, tokens):
    """The residual stream after every layer run, [runs, T, W], and the stream at the end."""
    x0 = w["embed"][torch.tensor(tokens)]
    x = x0.clone()
    loop = cfg.get("loop")
    after = []
    for i, p, first in run_order(cfg)[0]:
        if loop and first:
            x = torch.cat([x, x0], dim=-1) @ w["loop.in"].T + w["loop.step"][p]
        x = layer(x, w, i, cfg["layers"][i], cfg)
        after.append(x)
    return torch.stack(after), x


def logits(cfg, w, tokens):
    _, x = hidden_states(cfg, w, tokens)
    return rms_norm(x, w["final.norm"], float(cfg["norm"]["eps"])) @ w["embed"].T


def greedy_generate(cfg, w, prompt, n_new):
    toks, out = list(prompt), []
    for _ in range(n_new):
        nxt = int(logits(cfg, w, toks)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out
